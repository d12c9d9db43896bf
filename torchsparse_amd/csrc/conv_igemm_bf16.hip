// bf16 instantiation of the implicit-GEMM convolution (fp32 accumulation,
// v_mfma_f32_16x16x32_bf16).
#include "conv_ops.h"

namespace tsmi {
struct TraitsBF16 {
  using elem_t = __bf16;
  using vec_t = __bf16 __attribute__((ext_vector_type(8)));
  using acc_t = float __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ vec_t zero() {
    const __bf16 z = (__bf16)0.0f;
    return vec_t{z, z, z, z, z, z, z, z};
  }
  static __device__ __forceinline__ acc_t mma(vec_t a, vec_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec_t load_ragged(const elem_t *src, int remaining) {
    vec_t v = zero();
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < remaining) v[j] = src[j];
    return v;
  }
  static __device__ __forceinline__ float to_float(elem_t v) { return (float)v; }
  static __device__ __forceinline__ elem_t from_float(float v) { return (elem_t)v; }
  static __device__ __forceinline__ void store4(elem_t *dst, const float *v) {
    typedef __bf16 b4 __attribute__((ext_vector_type(4)));
    *(b4 *)dst = b4{(elem_t)v[0], (elem_t)v[1], (elem_t)v[2], (elem_t)v[3]};
  }
};
}  // namespace tsmi

#define TSMI_TRAITS TraitsBF16
#define TSMI_SUFFIX bf16
// 16-bit types also get the densely packed kernel for layers of at most 8 input channels
#define TSMI_SMALL_CIN 1
#include "conv_igemm.inc"
#include "conv_small_cin.inc"
#include "conv_tile.inc"
#include "conv_igemm2.inc"
#include "conv_segments.inc"
#include "conv_plan.inc"
#include "conv_wgrad.inc"
#include "conv_wgrad_pairs.inc"
#include "conv_igemm_tail.inc"

namespace tsmi {
const ConvOps &conv_ops_bf16() { return bf16::kOps; }
}  // namespace tsmi
