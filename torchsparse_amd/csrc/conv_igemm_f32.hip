// fp32 instantiation of the implicit-GEMM convolution (v_mfma_f32_16x16x4_f32;
// a lane's 16-byte load feeds four consecutive MFMAs, one reduction index each).
#include "conv_ops.h"

namespace tsmi {
struct TraitsF32 {
  using elem_t = float;
  using vec_t = float __attribute__((ext_vector_type(4)));
  using acc_t = float __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ vec_t zero() { return vec_t{0.f, 0.f, 0.f, 0.f}; }
  static __device__ __forceinline__ acc_t mma(vec_t a, vec_t b, acc_t c) {
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], c, 0, 0, 0);
    return c;
  }
  static __device__ __forceinline__ vec_t load_ragged(const elem_t *src, int remaining) {
    vec_t v = zero();
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (j < remaining) v[j] = src[j];
    return v;
  }
  static __device__ __forceinline__ float to_float(elem_t v) { return v; }
  static __device__ __forceinline__ elem_t from_float(float v) { return v; }
  static __device__ __forceinline__ void store4(elem_t *dst, const float *v) {
    *(vec_t *)dst = vec_t{v[0], v[1], v[2], v[3]};
  }
};
}  // namespace tsmi

#define TSMI_TRAITS TraitsF32
#define TSMI_SUFFIX f32
#include "conv_igemm.inc"
#include "conv_tile.inc"
#include "conv_igemm2.inc"
#include "conv_plan.inc"
#include "conv_wgrad.inc"
#include "conv_wgrad_pairs.inc"
#include "conv_igemm_tail.inc"

namespace tsmi {
const ConvOps &conv_ops_f32() { return f32::kOps; }
}  // namespace tsmi
