// Python binding for the reference's own CPU sources (compiled where they lie
// under /root/reference; nothing is copied).  Test infrastructure only: used
// to validate oracle.c and, optionally, as the cpu_baseline of the benchmark.
#include <torch/extension.h>

#include "convolution/convolution_gather_scatter_cpu.h"
#include "devoxelize/devoxelize_cpu.h"
#include "hash/hash_cpu.h"
#include "others/count_cpu.h"
#include "voxelize/voxelize_cpu.h"

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("conv_forward_gather_scatter_cpu", &conv_forward_gather_scatter_cpu);
  m.def("conv_backward_gather_scatter_cpu", &conv_backward_gather_scatter_cpu);
  m.def("hash_cpu", &hash_cpu);
  m.def("kernel_hash_cpu", &kernel_hash_cpu);
  m.def("count_cpu", &count_cpu);
  m.def("voxelize_forward_cpu", &voxelize_forward_cpu);
  m.def("voxelize_backward_cpu", &voxelize_backward_cpu);
  m.def("devoxelize_forward_cpu", &devoxelize_forward_cpu);
}
