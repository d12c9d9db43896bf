// Open-addressing hash table over two caller-owned arrays (keys int64, vals int32).
//
// Slot layout: groups of 4 consecutive slots.  The group is chosen by a mixed
// hash of (key >> 2) and the slot inside the group by the low two key bits, so
// the packed coordinates z-1, z, z+1 of one column land in the same or the next
// 32-byte key segment and a 3-wide neighbourhood touches 9 cache lines instead
// of 27.  Collisions resolve by linear probing over the whole table.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tsmi {

constexpr int kCoordBits = 18;            // x, y, z each in [-2^17, 2^17): packed with a bias
constexpr int kCoordLimit = 1 << kCoordBits;
constexpr int kCoordBias = 1 << (kCoordBits - 1);
constexpr int kBatchLimit = 512;          // keeps key + 1 positive in int64

struct TableView {
  unsigned long long *keys;  // 0 = empty, otherwise key + 1
  int32_t *vals;             // row index + 1
  uint32_t cap;              // multiple of 8
  uint32_t groups;           // cap / 4
};

__device__ __forceinline__ bool coords_packable(int b, int x, int y, int z) {
  return (unsigned)(x + kCoordBias) < (unsigned)kCoordLimit &&
         (unsigned)(y + kCoordBias) < (unsigned)kCoordLimit &&
         (unsigned)(z + kCoordBias) < (unsigned)kCoordLimit && (unsigned)b < (unsigned)kBatchLimit;
}

__device__ __forceinline__ unsigned long long pack_coords(int b, int x, int y, int z) {
  // the bias keeps ascending key order = ascending (b, x, y, z) order for negative values too
  return ((unsigned long long)(unsigned)b << (3 * kCoordBits)) |
         ((unsigned long long)(unsigned)(x + kCoordBias) << (2 * kCoordBits)) |
         ((unsigned long long)(unsigned)(y + kCoordBias) << kCoordBits) |
         (unsigned long long)(unsigned)(z + kCoordBias);
}

__device__ __forceinline__ void unpack_coords(unsigned long long key, int *c) {
  const unsigned mask = kCoordLimit - 1;
  c[3] = (int)(key & mask) - kCoordBias;
  c[2] = (int)((key >> kCoordBits) & mask) - kCoordBias;
  c[1] = (int)((key >> (2 * kCoordBits)) & mask) - kCoordBias;
  c[0] = (int)(key >> (3 * kCoordBits));
}

__device__ __forceinline__ uint32_t home_slot(const TableView &t, unsigned long long key) {
  unsigned long long h = key >> 2;
  h ^= h >> 33;
  h *= 0xff51afd7ed558ccdULL;
  h ^= h >> 33;
  uint32_t g = (uint32_t)(((h >> 32) * (unsigned long long)t.groups) >> 32);
  return (g << 2) | (uint32_t)(key & 3);
}

// Returns the slot holding `key` (inserting it if absent) or 0xFFFFFFFF when the
// table is full.  *fresh tells whether this call created the entry.
// kLoadFirst: read the slot with a plain load before the compare-and-swap.  That pays when
// most calls find their key already there (de-duplicating candidates): device-scope atomics
// are an order of magnitude slower than loads here, and a slot never changes once it is
// non-empty, so only slots that read as empty (possibly stale) need the atomic.  Distinct
// keys going into a mostly empty table take the atomic at once and save the round trip.
template <bool kLoadFirst = true>
__device__ __forceinline__ uint32_t table_insert(const TableView &t, unsigned long long key,
                                                 bool *fresh) {
  const unsigned long long stored = key + 1;
  uint32_t slot = home_slot(t, key);
  for (uint32_t probe = 0; probe < t.cap; ++probe) {
    unsigned long long prev = kLoadFirst ? t.keys[slot] : 0ULL;
    if (prev == 0ULL) prev = atomicCAS(&t.keys[slot], 0ULL, stored);
    if (prev == 0ULL) {
      *fresh = true;
      return slot;
    }
    if (prev == stored) {
      *fresh = false;
      return slot;
    }
    slot = slot + 1 == t.cap ? 0 : slot + 1;
  }
  *fresh = false;
  return 0xFFFFFFFFu;
}

// Returns the slot holding `key` or 0xFFFFFFFF when absent.  A lane reads the four slots of a
// group (32 aligned bytes) at once and checks them in registers: at the reserved load factor
// of one half a miss walks three slots on average (a hit two), nearly always inside one group or
// into the next, so a look-up is one memory round trip instead of a chain of two or three.  (A
// wavefront probing one key with all its lanes would still read only these 32 bytes per step:
// keys are independent, so a lane per key and a group per load is the cooperative form that
// keeps every lane on work of its own.)
__device__ __forceinline__ uint32_t table_find(const TableView &t, unsigned long long key) {
  const unsigned long long stored = key + 1;
  uint32_t slot = home_slot(t, key);
  uint32_t base = slot & ~3u;  // the capacity is a multiple of 8: groups never straddle the end
  for (uint32_t probed = 0; probed < t.cap;) {
    const ulonglong2 lo = *(const ulonglong2 *)(t.keys + base);
    const ulonglong2 hi = *(const ulonglong2 *)(t.keys + base + 2);
    const unsigned long long k4[4] = {lo.x, lo.y, hi.x, hi.y};
    const uint32_t first = slot - base;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
      if (j < first) continue;
      if (k4[j] == stored) return base + j;
      if (k4[j] == 0ULL) return 0xFFFFFFFFu;
    }
    probed += 4 - first;
    base = base + 4 == t.cap ? 0 : base + 4;
    slot = base;
  }
  return 0xFFFFFFFFu;
}

}  // namespace tsmi
