// A launch thread for the convolution calls of a forward.
//
// A forward of a network makes ~60 convolution calls; each costs the calling thread ~5 us inside
// the library (argument checks, the plan, hipLaunchKernel) on top of the ~5 us its binding spends
// preparing it.  Between tsmi_launch_thread_open and _close the three packed convolution calls
// can be handed to ONE worker thread instead (tsmi_launch_thread_submit): the worker carries them
// out in the order they were handed over, while the caller prepares the next one.  Launches
// reach each stream in submission order; everything else the caller does on those streams itself
// (other library calls, the framework's own kernels, event records) is ordered against the
// submitted calls only by tsmi_launch_thread_flush, which returns once every submitted call has
// been carried out.  The caller keeps the buffers of a submitted call alive until
// *tsmi_launch_thread_completed() has reached the call's ticket.
//
// Status codes of submitted calls surface at the next flush (the first failure and its message).
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <thread>

#include "common.h"

namespace {

constexpr int kRing = 256;
constexpr int kWords = 21;

struct Job {
  int kind;    // 0: tsmi_conv_implicit_gemm_packed, 1: ..._segments_packed, 2: ..._grouped_packed
  int device;  // the device that was current when the call was handed over
  int64_t a[kWords];
};

Job g_ring[kRing];
std::atomic<int64_t> g_submitted{0};  // tickets handed out
std::atomic<int64_t> g_completed{0};  // calls carried out (the worker is the only writer)
std::atomic<int> g_open{0};           // regions open
std::atomic<int> g_error{0};          // first failing status since the last flush
char g_message[512] = "";
// (never destroyed: the worker outlives the static destructors of a process that exits)
std::mutex &g_submit_mutex = *new std::mutex;  // several host threads may hand calls over
std::mutex &g_park_mutex = *new std::mutex;
std::condition_variable &g_wake = *new std::condition_variable;
bool g_started = false;

void run_job(const Job &j, int *current_device) {
  if (j.device != *current_device) {
    if (hipSetDevice(j.device) != hipSuccess) {
      if (!g_error.load()) {
        snprintf(g_message, sizeof(g_message), "launch thread: cannot select device %d", j.device);
        g_error.store(TSMI_ERR_HIP);
      }
      return;
    }
    *current_device = j.device;
  }
  int status;
  switch (j.kind) {
    case 0: status = tsmi_conv_implicit_gemm_packed(j.a); break;
    case 1: status = tsmi_conv_implicit_gemm_segments_packed(j.a); break;
    default: status = tsmi_conv_implicit_gemm_grouped_packed(j.a); break;
  }
  if (status != TSMI_OK && !g_error.load()) {
    strncpy(g_message, tsmi_last_error(), sizeof(g_message) - 1);  // (the worker's own last error)
    g_message[sizeof(g_message) - 1] = 0;
    g_error.store(status);
  }
}

void worker() {
  int current_device = -1;
  int idle = 0;
  for (;;) {
    const int64_t done = g_completed.load(std::memory_order_relaxed);
    if (done == g_submitted.load(std::memory_order_acquire)) {
      // nothing to do: spin while a region is open (its calls arrive microseconds apart),
      // sleep otherwise
      // (and for ~2 ms after the last call: the next forward of a loop finds the worker awake)
      if (idle < (g_open.load(std::memory_order_relaxed) > 0 ? 2000000 : 50000)) {
        ++idle;
        __builtin_ia32_pause();
        continue;
      }
      std::unique_lock<std::mutex> lock(g_park_mutex);
      g_wake.wait_for(lock, std::chrono::milliseconds(50), [&] {
        return g_completed.load(std::memory_order_relaxed) != g_submitted.load(std::memory_order_acquire);
      });
      idle = 0;
      continue;
    }
    idle = 0;
    run_job(g_ring[done % kRing], &current_device);
    g_completed.store(done + 1, std::memory_order_release);
  }
}

}  // namespace

extern "C" int tsmi_launch_thread_open(void) {
  {
    std::lock_guard<std::mutex> lock(g_park_mutex);
    if (!g_started) {
      std::thread(worker).detach();  // lives until the process ends
      g_started = true;
    }
  }
  g_open.fetch_add(1);
  g_wake.notify_one();
  return TSMI_OK;
}

extern "C" int64_t tsmi_launch_thread_submit(int kind, const int64_t *args, int n_words) {
  if (kind < 0 || kind > 2 || !args || n_words < 1 || n_words > kWords || g_open.load() <= 0) return -1;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return -1;
  std::lock_guard<std::mutex> lock(g_submit_mutex);
  const int64_t ticket = g_submitted.load(std::memory_order_relaxed);
  while (ticket - g_completed.load(std::memory_order_acquire) >= kRing) __builtin_ia32_pause();
  Job &j = g_ring[ticket % kRing];
  j.kind = kind;
  j.device = device;
  memcpy(j.a, args, sizeof(int64_t) * n_words);
  for (int i = n_words; i < kWords; ++i) j.a[i] = 0;
  g_submitted.store(ticket + 1, std::memory_order_release);
  g_wake.notify_one();  // (the worker sleeps only after it has been idle for a while)
  return ticket + 1;
}

extern "C" const int64_t *tsmi_launch_thread_completed(void) {
  static_assert(sizeof(std::atomic<int64_t>) == sizeof(int64_t), "the counter is read as a plain int64");
  return reinterpret_cast<const int64_t *>(&g_completed);
}

extern "C" int tsmi_launch_thread_flush(void) {
  const int64_t target = g_submitted.load(std::memory_order_acquire);
  while (g_completed.load(std::memory_order_acquire) < target) __builtin_ia32_pause();
  const int status = g_error.exchange(0);
  if (status != TSMI_OK) return tsmi::fail(status, "%s", g_message);
  return TSMI_OK;
}

extern "C" int tsmi_launch_thread_close(void) {
  const int status = tsmi_launch_thread_flush();
  if (g_open.load() > 0) g_open.fetch_sub(1);
  return status;
}
