// Shared by the kernels of libaphrodite_mi355x_mixers.so: dtype dispatch and block reductions.  wave = 64 lanes.
#pragma once
#include "../common.h"
#include "../../../include/aphrodite_mi355x_mixers.h"

namespace aphro {

// Activation / weight storage of this library: bf16 or fp32 (APHRO_BF16 / APHRO_F32).  fp32 is a true 32-bit path:
// no reduced-precision product anywhere.
#define MIX_DISPATCH_DTYPE(dtype, ...)                                             \
  do {                                                                             \
    if ((dtype) == APHRO_BF16) { typedef ::aphro::BFloat T; __VA_ARGS__; }          \
    else if ((dtype) == APHRO_F32) { typedef ::aphro::Float T; __VA_ARGS__; }       \
    else { ::aphro::set_error("dtype %d: this library serves bf16 (1) and fp32 (2)", (int)(dtype)); return APHRO_ERR_INVALID; } \
  } while (0)

// sum over a workgroup of up to 16 waves; every thread gets the total.  red: >= 16 floats of LDS.
__device__ __forceinline__ float wg_sum(float v, float* red) {
  v = wave_sum(v);
  const int nw = (blockDim.x + 63) >> 6;
  if (nw == 1) return v;
  __syncthreads();                     // a previous use of red may still be read
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.f;
  for (int w = 0; w < nw; ++w) t += red[w];
  return t;
}

// Sums over groups of 2^LOG adjacent lanes with DPP moves (no LDS round trip): quad permutes for 2 and 4, the half-row and
// row mirrors for 8 and 16 (after the quad steps every lane of a quad holds the quad's total, so the mirror partner brings
// in the other half); every lane of a group ends with the group's total.  Wider groups finish with ds_bpermute shuffles.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int LOG>
__device__ __forceinline__ float group_sum(float v) {
  if (LOG >= 1) v += dpp_f<0xB1>(v);       // quad_perm [1, 0, 3, 2]
  if (LOG >= 2) v += dpp_f<0x4E>(v);       // quad_perm [2, 3, 0, 1]
  if (LOG >= 3) v += dpp_f<0x141>(v);      // row_half_mirror
  if (LOG >= 4) v += dpp_f<0x140>(v);      // row_mirror
  if (LOG >= 5) v += __shfl_xor(v, 16, 64);
  if (LOG >= 6) v += __shfl_xor(v, 32, 64);
  return v;
}

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + __expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + __expf(-z)); }
__device__ __forceinline__ float gelu_tanh_f(float z) {
  const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.0f + tanhf(u));
}
// log(sigmoid(z)) without overflow on either side
__device__ __forceinline__ float log_sigmoid_f(float z) {
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

}  // namespace aphro
