// Memory-bound pieces around an fp32 residual stream: embedding gather, the fused "post-norm + residual add + next
// pre-norm" launch, gated activations, and the gated group RMS norm that follows a recurrent memory.
// One workgroup per token, fp32 math, wave64 reductions; any width (no divisibility assumed).
#include <stdarg.h>
#include <stdio.h>

#include "mixers_common.h"

namespace aphro {
static thread_local char g_mix_err[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_mix_err, sizeof(g_mix_err), fmt, ap);
  va_end(ap);
}
}  // namespace aphro
extern "C" const char* aphro_mixers_last_error(void) { return aphro::g_mix_err; }

namespace aphro {

template <typename T>
__global__ void embed_scale_kernel(float* __restrict__ residual, const typename T::storage* __restrict__ table,
                                   const int64_t* __restrict__ ids, int width, int64_t vocab, float scale) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  if (id < 0 || id >= vocab) id = 0;           // the host validates ids; never read outside the table
  const typename T::storage* row = table + id * (int64_t)width;
  float* o = residual + t * (int64_t)width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = T::to_f32(row[i]) * scale;
}

// mean and 1/sqrt(var + eps) of the row held in LDS (fp32), variance as the mean of squared deviations
__device__ __forceinline__ void row_stats(const float* row, int width, float eps, float* red, float& mean, float& rstd) {
  float s = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) s += row[i];
  mean = wg_sum(s, red) / (float)width;
  float v = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float d = row[i] - mean;
    v += d * d;
  }
  rstd = 1.0f / sqrtf(wg_sum(v, red) / (float)width + eps);
}

template <typename T>
__global__ void residual_layer_norm_kernel(float* __restrict__ residual, const typename T::storage* __restrict__ y,
                                           int64_t y_stride, const float* __restrict__ y_bias,
                                           const typename T::storage* __restrict__ post_w,
                                           const typename T::storage* __restrict__ post_b,
                                           const typename T::storage* __restrict__ add_vec,
                                           const typename T::storage* __restrict__ pre_w,
                                           const typename T::storage* __restrict__ pre_b,
                                           typename T::storage* __restrict__ out, int width, float eps) {
  extern __shared__ float row[];               // width floats
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  float* r = residual + t * (int64_t)width;
  if (y != nullptr) {
    const typename T::storage* yr = y + t * y_stride;
    for (int i = threadIdx.x; i < width; i += blockDim.x) row[i] = T::to_f32(yr[i]) + (y_bias ? y_bias[i] : 0.f);
    __syncthreads();
    float mean, rstd;
    row_stats(row, width, eps, red, mean, rstd);
    __syncthreads();
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      float x = r[i] + ((row[i] - mean) * rstd * T::to_f32(post_w[i]) + T::to_f32(post_b[i]));
      if (add_vec) x += T::to_f32(add_vec[i]);
      row[i] = x;
      r[i] = x;
    }
  } else {
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      float x = r[i];
      if (add_vec) {
        x += T::to_f32(add_vec[i]);
        r[i] = x;
      }
      row[i] = x;
    }
  }
  if (out == nullptr) return;
  __syncthreads();
  float mean, rstd;
  row_stats(row, width, eps, red, mean, rstd);
  typename T::storage* o = out + t * (int64_t)width;
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    o[i] = T::from_f32((row[i] - mean) * rstd * T::to_f32(pre_w[i]) + T::to_f32(pre_b[i]));
}

// ---- the same two kernels for rows that are a multiple of 8 elements and 16-byte aligned: every thread owns 8 consecutive
// elements in registers (no LDS row), all of a row's inputs are requested before the first reduction.
template <typename T>
__device__ __forceinline__ void load8(const typename T::storage* p, float* o) {
  if constexpr (sizeof(typename T::storage) == 2) {
    const u16x8 v = *reinterpret_cast<const u16x8*>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = T::to_f32(v[j]);
  } else {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[j] = a[j];
      o[4 + j] = b[j];
    }
  }
}
template <typename T>
__device__ __forceinline__ void store8(typename T::storage* p, const float* v) {
  if constexpr (sizeof(typename T::storage) == 2) {
    u16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = T::from_f32(v[j]);
    *reinterpret_cast<u16x8*>(p) = r;
  } else {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4*>(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
}

__device__ __forceinline__ void stats8(const float* x, bool act, int width, float eps, float* red, float& mean, float& rstd) {
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) s += act ? x[j] : 0.f;
  mean = wg_sum(s, red) / (float)width;
  float v = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float d = act ? x[j] - mean : 0.f;
    v += d * d;
  }
  rstd = 1.0f / sqrtf(wg_sum(v, red) / (float)width + eps);
}

template <typename T>
__global__ void residual_layer_norm_vec8_kernel(float* __restrict__ residual, const typename T::storage* __restrict__ y,
                                                int64_t y_stride, const float* __restrict__ y_bias,
                                                const typename T::storage* __restrict__ post_w,
                                                const typename T::storage* __restrict__ post_b,
                                                const typename T::storage* __restrict__ add_vec,
                                                const typename T::storage* __restrict__ pre_w,
                                                const typename T::storage* __restrict__ pre_b,
                                                typename T::storage* __restrict__ out, int width, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int i0 = threadIdx.x * 8;
  const bool act = i0 < width;
  const int ia = act ? i0 : 0;
  float* r = residual + t * (int64_t)width;
  float x[8], rv[8], w[8], b[8], av[8], qw[8], qb[8];
  load8<Float>(r + ia, rv);
  if (y) {
    load8<T>(y + t * y_stride + ia, x);
    load8<T>(post_w + ia, w);
    load8<T>(post_b + ia, b);
    if (y_bias) {
      float yb[8];
      load8<Float>(y_bias + ia, yb);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += yb[j];
    }
  }
  if (add_vec) load8<T>(add_vec + ia, av);
  if (out) {
    load8<T>(pre_w + ia, qw);
    load8<T>(pre_b + ia, qb);
  }
  if (y) {
    float mean, rstd;
    stats8(x, act, width, eps, red, mean, rstd);
#pragma unroll
    for (int j = 0; j < 8; ++j) rv[j] += (x[j] - mean) * rstd * w[j] + b[j];
  }
  if (add_vec) {
#pragma unroll
    for (int j = 0; j < 8; ++j) rv[j] += av[j];
  }
  if ((y || add_vec) && act) store8<Float>(r + i0, rv);
  if (out == nullptr) return;
  float mean, rstd;
  stats8(rv, act, width, eps, red, mean, rstd);
#pragma unroll
  for (int j = 0; j < 8; ++j) x[j] = (rv[j] - mean) * rstd * qw[j] + qb[j];
  if (act) store8<T>(out + t * (int64_t)width + i0, x);
}

template <typename T, int ACT>
__global__ void act_and_mul_vec8_kernel(typename T::storage* __restrict__ out, const typename T::storage* __restrict__ in,
                                        int64_t in_stride, int d) {
  const int64_t t = blockIdx.y;
  const int i0 = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i0 >= d) return;
  float g[8], u[8];
  load8<T>(in + t * in_stride + i0, g);
  load8<T>(in + t * in_stride + d + i0, u);
#pragma unroll
  for (int j = 0; j < 8; ++j) g[j] = (ACT == 0 ? silu_f(g[j]) : gelu_tanh_f(g[j])) * u[j];
  store8<T>(out + t * (int64_t)d + i0, g);
}

template <typename T, int ACT>
__global__ void act_and_mul_kernel(typename T::storage* __restrict__ out, const typename T::storage* __restrict__ in,
                                   int64_t in_stride, int d) {
  const int64_t t = blockIdx.x;
  const typename T::storage* a = in + t * in_stride;
  typename T::storage* o = out + t * (int64_t)d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float g = T::to_f32(a[i]), u = T::to_f32(a[d + i]);
    o[i] = T::from_f32((ACT == 0 ? silu_f(g) : gelu_tanh_f(g)) * u);
  }
}

template <typename T>
__global__ void gated_group_rms_norm_kernel(typename T::storage* __restrict__ out, int64_t out_stride,
                                            const float* __restrict__ x, const typename T::storage* __restrict__ weight,
                                            const typename T::storage* __restrict__ gate, int64_t gate_stride, int n,
                                            int group, float eps, float out_scale) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float* xr = x + t * (int64_t)n;
  const typename T::storage* gr = gate ? gate + t * gate_stride : nullptr;
  typename T::storage* o = out + t * out_stride;
  for (int g0 = 0; g0 < n; g0 += group) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < group; i += blockDim.x) ss += xr[g0 + i] * xr[g0 + i];
    const float inv = out_scale / sqrtf(wg_sum(ss, red) / (float)group + eps);
    for (int i = threadIdx.x; i < group; i += blockDim.x) {
      float val = xr[g0 + i] * inv;
      if (weight) val *= T::to_f32(weight[g0 + i]);
      if (gr) val *= sigmoid_f(T::to_f32(gr[g0 + i]));
      o[g0 + i] = T::from_f32(val);
    }
  }
}

static int block_for(int width) { return width >= 1024 ? 256 : (width > 256 ? 128 : 64); }

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_embed_scale_f32(float* residual, const void* table, const int64_t* ids, int64_t num_tokens, int width,
                                     int64_t vocab, float scale, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(residual && table && ids && num_tokens > 0 && width > 0 && vocab > 0, "embed_scale: bad arguments");
  MIX_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((embed_scale_kernel<T>), dim3((unsigned)num_tokens), dim3(block_for(width)),
                                               0, (hipStream_t)stream, residual, (const typename T::storage*)table, ids, width,
                                               vocab, scale));
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_residual_layer_norm(float* residual, const void* y, int64_t y_stride, const float* y_bias,
                                         const void* post_w, const void* post_b, const void* add_vec, const void* pre_w,
                                         const void* pre_b, void* out, int64_t num_tokens, int width, float eps, int dtype,
                                         void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(residual && num_tokens > 0 && width > 0 && width <= 16000, "residual_layer_norm: bad sizes (width %d)", width);
  APHRO_CHECK(!y || (post_w && post_b && y_stride >= width), "residual_layer_norm: y needs post_w, post_b and a row stride >= width");
  APHRO_CHECK(!out || (pre_w && pre_b), "residual_layer_norm: out needs pre_w and pre_b");
  APHRO_CHECK(y || add_vec || out, "residual_layer_norm: nothing to do");
  const auto al16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
  const bool vec = (width & 7) == 0 && width <= 8192 && (y_stride & 7) == 0 && al16(residual) && al16(y) && al16(y_bias) &&
                   al16(post_w) && al16(post_b) && al16(add_vec) && al16(pre_w) && al16(pre_b) && al16(out);
  if (vec) {
    const int threads = ((width / 8) + 63) / 64 * 64;
    MIX_DISPATCH_DTYPE(dtype, {
      typedef typename T::storage S;
      hipLaunchKernelGGL((residual_layer_norm_vec8_kernel<T>), dim3((unsigned)num_tokens), dim3(threads), 0, (hipStream_t)stream,
                         residual, (const S*)y, y_stride, y_bias, (const S*)post_w, (const S*)post_b, (const S*)add_vec,
                         (const S*)pre_w, (const S*)pre_b, (S*)out, width, eps);
    });
    APHRO_LAUNCH_CHECK();
    return APHRO_OK;
  }
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((residual_layer_norm_kernel<T>), dim3((unsigned)num_tokens), dim3(block_for(width)),
                       (size_t)width * sizeof(float), (hipStream_t)stream, residual, (const S*)y, y_stride, y_bias,
                       (const S*)post_w, (const S*)post_b, (const S*)add_vec, (const S*)pre_w, (const S*)pre_b, (S*)out,
                       width, eps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_act_and_mul(void* out, const void* in, int64_t in_stride, int64_t num_tokens, int d, int act, int dtype,
                                 void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && in && d > 0 && in_stride >= 2 * (int64_t)d && (act == 0 || act == 1), "act_and_mul: bad arguments");
  if ((d & 7) == 0 && (in_stride & 7) == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0 && num_tokens <= 65535) {
    const int per_row = d / 8, threads = per_row >= 256 ? 256 : (per_row + 63) / 64 * 64;
    const dim3 grid((unsigned)((per_row + threads - 1) / threads), (unsigned)num_tokens);
    MIX_DISPATCH_DTYPE(dtype, {
      typedef typename T::storage S;
      if (act == 0)
        hipLaunchKernelGGL((act_and_mul_vec8_kernel<T, 0>), grid, dim3(threads), 0, (hipStream_t)stream, (S*)out, (const S*)in, in_stride, d);
      else
        hipLaunchKernelGGL((act_and_mul_vec8_kernel<T, 1>), grid, dim3(threads), 0, (hipStream_t)stream, (S*)out, (const S*)in, in_stride, d);
    });
    APHRO_LAUNCH_CHECK();
    return APHRO_OK;
  }
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (act == 0)
      hipLaunchKernelGGL((act_and_mul_kernel<T, 0>), dim3((unsigned)num_tokens), dim3(block_for(d)), 0, (hipStream_t)stream,
                         (S*)out, (const S*)in, in_stride, d);
    else
      hipLaunchKernelGGL((act_and_mul_kernel<T, 1>), dim3((unsigned)num_tokens), dim3(block_for(d)), 0, (hipStream_t)stream,
                         (S*)out, (const S*)in, in_stride, d);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_gated_group_rms_norm(void* out, int64_t out_stride, const float* x, const void* weight, const void* gate,
                                          int64_t gate_stride, int64_t num_tokens, int n, int group, float eps,
                                          float out_scale, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && x && n > 0 && group > 0 && n % group == 0 && out_stride >= n && (!gate || gate_stride >= n),
              "gated_group_rms_norm: bad arguments (n %d group %d)", n, group);
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((gated_group_rms_norm_kernel<T>), dim3((unsigned)num_tokens), dim3(block_for(group)), 0,
                       (hipStream_t)stream, (S*)out, out_stride, x, (const S*)weight, (const S*)gate, gate_stride, n, group,
                       eps, out_scale);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
