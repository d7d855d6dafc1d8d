// Launches around an fp32 residual stream whose layers are joined by a learned average over depth:
//   * depth_residual_rms_norm: residual add, the depth-weighted average over the stack of layer results, and the RMS norm
//     (scalar gain, optional per-channel weight) that feeds the next sublayer -- one launch;
//   * poly_norm: a N(z) + b N(z^2) + c N(z^3) + e, N = division by the row's root mean square;
//   * differential_norm_gate: o = a_1 - lambda a_2 of two attention maps, unit RMS per head, sigmoid gate.
// fp32 math whatever the storage type.  Rows that are a multiple of 8 elements and 16-byte aligned are held in registers
// (8 elements per thread, every input requested before the first reduction); any other width goes through an LDS row.
#include "mixers_common.h"

namespace aphro {

template <typename T>
__device__ __forceinline__ void dn_load8(const typename T::storage* p, float* o) {
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
__device__ __forceinline__ void dn_store8(typename T::storage* p, const float* v) {
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

// generic form: one workgroup per row, the row in LDS
template <typename T>
__global__ void depth_residual_rms_norm_kernel(const float* __restrict__ x_in, float* __restrict__ x_out,
                                               const typename T::storage* __restrict__ y, int64_t y_stride,
                                               float* __restrict__ history, int64_t hist_stride, int n_hist,
                                               const float* __restrict__ depth_w, float gain,
                                               const typename T::storage* __restrict__ weight,
                                               typename T::storage* __restrict__ out, int width, float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float* xi = x_in + t * (int64_t)width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float r = xi[i];
    if (y) r += T::to_f32(y[t * y_stride + i]);
    if (depth_w) {
      float* hrow = history + t * (int64_t)width + i;
      hrow[(int64_t)n_hist * hist_stride] = r;
      float a = 0.f;
      for (int j = 0; j < n_hist; ++j) a += depth_w[j] * hrow[(int64_t)j * hist_stride];
      r = a + depth_w[n_hist] * r;
    }
    if (x_out) x_out[t * (int64_t)width + i] = r;
    row[i] = r;
    ss += r * r;
  }
  if (out == nullptr) return;
  const float rstd = gain / sqrtf(wg_sum(ss, red) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = row[i] * rstd;
    if (weight) v *= T::to_f32(weight[i]);
    out[t * (int64_t)width + i] = T::from_f32(v);
  }
}

// register form: thread = 8 consecutive elements of the row
template <typename T>
__global__ void depth_residual_rms_norm_vec8_kernel(const float* __restrict__ x_in, float* __restrict__ x_out,
                                                    const typename T::storage* __restrict__ y, int64_t y_stride,
                                                    float* __restrict__ history, int64_t hist_stride, int n_hist,
                                                    const float* __restrict__ depth_w, float gain,
                                                    const typename T::storage* __restrict__ weight,
                                                    typename T::storage* __restrict__ out, int width, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int i0 = threadIdx.x * 8;
  const bool act = i0 < width;
  const int ia = act ? i0 : 0;
  const int64_t at = t * (int64_t)width + ia;
  float r[8], yv[8], w[8];
  dn_load8<Float>(x_in + at, r);
  if (y) dn_load8<T>(y + t * y_stride + ia, yv);
  if (out && weight) dn_load8<T>(weight + ia, w);
  if (y) {
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] += yv[j];
  }
  if (depth_w) {
    if (act) dn_store8<Float>(history + (int64_t)n_hist * hist_stride + at, r);
    float a[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) a[j] = 0.f;
    int k = 0;
    for (; k + 2 <= n_hist; k += 2) {          // two stack entries in flight
      float h0[8], h1[8];
      dn_load8<Float>(history + (int64_t)k * hist_stride + at, h0);
      dn_load8<Float>(history + (int64_t)(k + 1) * hist_stride + at, h1);
      const float w0 = depth_w[k], w1 = depth_w[k + 1];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        a[j] += w0 * h0[j];
        a[j] += w1 * h1[j];
      }
    }
    if (k < n_hist) {
      float h0[8];
      dn_load8<Float>(history + (int64_t)k * hist_stride + at, h0);
      const float w0 = depth_w[k];
#pragma unroll
      for (int j = 0; j < 8; ++j) a[j] += w0 * h0[j];
    }
    const float wl = depth_w[n_hist];
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = a[j] + wl * r[j];
  }
  if (x_out && act) dn_store8<Float>(x_out + at, r);
  if (out == nullptr) return;
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) ss += act ? r[j] * r[j] : 0.f;
  const float rstd = gain / sqrtf(wg_sum(ss, red) / (float)width + eps);
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = r[j] * rstd * (weight ? w[j] : 1.0f);
  if (act) dn_store8<T>(out + at, r);
}

// three sums over a workgroup of up to 16 waves in one LDS round trip; red: >= 48 floats
__device__ __forceinline__ void wg_sum3(float& a, float& b, float& c, float* red) {
  a = wave_sum(a);
  b = wave_sum(b);
  c = wave_sum(c);
  const int nw = (blockDim.x + 63) >> 6;
  if (nw == 1) return;
  if ((threadIdx.x & 63) == 0) {
    red[3 * (threadIdx.x >> 6)] = a;
    red[3 * (threadIdx.x >> 6) + 1] = b;
    red[3 * (threadIdx.x >> 6) + 2] = c;
  }
  __syncthreads();
  a = b = c = 0.f;
  for (int w = 0; w < nw; ++w) {
    a += red[3 * w];
    b += red[3 * w + 1];
    c += red[3 * w + 2];
  }
}

template <typename T>
__global__ void poly_norm_kernel(typename T::storage* __restrict__ out, const typename T::storage* __restrict__ z,
                                 int64_t z_stride, int n, float a, float b, float c, float e, float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = T::to_f32(z[t * z_stride + i]);
    row[i] = v;
    const float v2 = v * v;
    s2 += v2;
    s4 += v2 * v2;
    s6 += v2 * v2 * v2;
  }
  const float inv = 1.0f / (float)n;
  const float r1 = a / sqrtf(wg_sum(s2, red) * inv + eps);
  const float r2 = b / sqrtf(wg_sum(s4, red) * inv + eps);
  const float r3 = c / sqrtf(wg_sum(s6, red) * inv + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = row[i], v2 = v * v;
    out[t * (int64_t)n + i] = T::from_f32(v * r1 + v2 * r2 + v2 * v * r3 + e);
  }
}

// register form: up to 16 elements per thread in two 8-element pieces, blockDim.x * 16 >= n
template <typename T>
__global__ void poly_norm_vec8_kernel(typename T::storage* __restrict__ out, const typename T::storage* __restrict__ z,
                                      int64_t z_stride, int n, float a, float b, float c, float e, float eps) {
  __shared__ float red[48];
  const int64_t t = blockIdx.x;
  float v[2][8];
  bool act[2];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int i0 = (threadIdx.x + h * blockDim.x) * 8;
    act[h] = i0 < n;
    dn_load8<T>(z + t * z_stride + (act[h] ? i0 : 0), v[h]);
  }
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v2 = act[h] ? v[h][j] * v[h][j] : 0.f;
      s2 += v2;
      s4 += v2 * v2;
      s6 += v2 * v2 * v2;
    }
  const float inv = 1.0f / (float)n;
  wg_sum3(s2, s4, s6, red);
  const float r1 = a / sqrtf(s2 * inv + eps);
  const float r2 = b / sqrtf(s4 * inv + eps);
  const float r3 = c / sqrtf(s6 * inv + eps);
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int i0 = (threadIdx.x + h * blockDim.x) * 8;
    float o[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float x = v[h][j], x2 = x * x;
      o[j] = x * r1 + x2 * r2 + x2 * x * r3 + e;
    }
    if (act[h]) dn_store8<T>(out + t * (int64_t)n + i0, o);
  }
}

// one wave per (row, head): a [T, heads * maps * vdim] fp32 (head by head, map after map), maps is 1 or 2
template <typename T>
__global__ void differential_norm_gate_kernel(typename T::storage* __restrict__ out, int64_t out_stride,
                                              const float* __restrict__ a, int64_t a_stride,
                                              const typename T::storage* __restrict__ gate, int64_t gate_stride, int heads,
                                              int maps, int vdim, float lambda, float out_scale, float eps) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  for (int h = threadIdx.x >> 6; h < heads; h += nw) {
    const float* a1 = a + t * a_stride + (int64_t)h * maps * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) {
      const float o = maps == 2 ? a1[c] - lambda * a1[vdim + c] : a1[c];
      ss += o * o;
    }
    const float inv = out_scale / sqrtf(wave_sum(ss) / (float)vdim + eps);
    for (int c = lane; c < vdim; c += 64) {
      float o = (maps == 2 ? a1[c] - lambda * a1[vdim + c] : a1[c]) * inv;
      if (gate) o *= sigmoid_f(T::to_f32(gate[t * gate_stride + h * vdim + c]));
      out[t * out_stride + h * vdim + c] = T::from_f32(o);
    }
  }
}

static int dn_block_for(int width) { return width >= 1024 ? 256 : (width > 256 ? 128 : 64); }

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_depth_residual_rms_norm(const float* x_in, float* x_out, const void* y, int64_t y_stride, float* history,
                                             int64_t hist_stride, int n_hist, const float* depth_w, float gain,
                                             const void* weight, void* out, int64_t num_tokens, int width, float eps,
                                             int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(x_in && num_tokens > 0 && width > 0 && width <= 16000, "depth_residual_rms_norm: bad sizes (width %d)", width);
  APHRO_CHECK(!y || y_stride >= width, "depth_residual_rms_norm: y's row stride is smaller than the row");
  APHRO_CHECK(!depth_w || (history && n_hist >= 0 && hist_stride >= num_tokens * (int64_t)width),
              "depth_residual_rms_norm: the depth average needs the stack of layer results");
  APHRO_CHECK(x_out || out, "depth_residual_rms_norm: nothing to write");
  const auto al16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
  const bool vec = (width & 7) == 0 && width <= 8192 && (y_stride & 7) == 0 && (hist_stride & 3) == 0 && al16(x_in) &&
                   al16(x_out) && al16(y) && al16(history) && al16(weight) && al16(out);
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (vec)
      hipLaunchKernelGGL((depth_residual_rms_norm_vec8_kernel<T>), dim3((unsigned)num_tokens), dim3(((width / 8) + 63) / 64 * 64),
                         0, (hipStream_t)stream, x_in, x_out, (const S*)y, y_stride, history, hist_stride, n_hist, depth_w, gain,
                         (const S*)weight, (S*)out, width, eps);
    else
      hipLaunchKernelGGL((depth_residual_rms_norm_kernel<T>), dim3((unsigned)num_tokens), dim3(dn_block_for(width)),
                         (size_t)width * sizeof(float), (hipStream_t)stream, x_in, x_out, (const S*)y, y_stride, history,
                         hist_stride, n_hist, depth_w, gain, (const S*)weight, (S*)out, width, eps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_poly_norm(void* out, const void* z, int64_t z_stride, int64_t num_tokens, int n, float a, float b, float c,
                               float e, float eps, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && z && n > 0 && n <= 16000 && z_stride >= n, "poly_norm: bad arguments (n %d)", n);
  const bool vec = (n & 7) == 0 && n <= 16 * 1024 && (z_stride & 7) == 0 && ((uintptr_t)z & 15) == 0 && ((uintptr_t)out & 15) == 0;
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (vec)
      hipLaunchKernelGGL((poly_norm_vec8_kernel<T>), dim3((unsigned)num_tokens), dim3(((n / 8 + 1) / 2 + 63) / 64 * 64), 0,
                         (hipStream_t)stream, (S*)out, (const S*)z, z_stride, n, a, b, c, e, eps);
    else
      hipLaunchKernelGGL((poly_norm_kernel<T>), dim3((unsigned)num_tokens), dim3(dn_block_for(n)), (size_t)n * sizeof(float),
                         (hipStream_t)stream, (S*)out, (const S*)z, z_stride, n, a, b, c, e, eps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_differential_norm_gate(void* out, int64_t out_stride, const float* a, int64_t a_stride, const void* gate,
                                            int64_t gate_stride, int64_t num_tokens, int heads, int maps, int vdim,
                                            float lambda, float out_scale, float eps, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && a && heads > 0 && vdim > 0 && (maps == 1 || maps == 2), "differential_norm_gate: bad arguments");
  APHRO_CHECK(out_stride >= (int64_t)heads * vdim && a_stride >= (int64_t)heads * maps * vdim &&
                  (!gate || gate_stride >= (int64_t)heads * vdim), "differential_norm_gate: row strides smaller than the rows");
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((differential_norm_gate_kernel<T>), dim3((unsigned)num_tokens), dim3(heads >= 4 ? 256 : 64 * heads), 0,
                       (hipStream_t)stream, (S*)out, out_stride, a, a_stride, (const S*)gate, gate_stride, heads, maps, vdim,
                       lambda, out_scale, eps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
