// Mixture of small feed-forward experts on unquantised weights (bf16 on the matrix cores, fp32 on the vector ALUs):
//   moe_route          softmax over the router's outputs, choice by score + correction, weight = the score itself
//   moe_align          the (token, choice) slots sorted by expert into blocks of 16 rows, one expert per block
//   moe_glu_gemm       per block: [gate | up] product of its expert with the clamped gated activation in the epilogue
//   moe_down_gemm      per block: the expert's down product, fp32 rows scattered back to their slots
//   moe_combine        per token: weighted sum over its choices (identity experts pass the input through), plus the
//                      sigmoid-gated shared expert
//   clamped_glu        the experts' activation alone (for the shared expert, whose products are plain dense ones)
// Nothing here depends on what else is in the batch: a slot's row is the same whichever block and row it lands in.
#include "mixers_common.h"

namespace aphro {

constexpr int MOE_BM = 16;

// g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha g) * (u + 1)
__device__ __forceinline__ float clamped_glu_f(float gate, float up, float limit, float alpha) {
  const float g = fminf(gate, limit);
  const float u = fminf(fmaxf(up, -limit), limit);
  return g * sigmoid_f(alpha * g) * (u + 1.0f);
}

// one wave per token; scores and choice values of the token in LDS
__global__ __launch_bounds__(256) void moe_route_kernel(int32_t* __restrict__ ids, float* __restrict__ weights,
                                                        const float* __restrict__ z, const float* __restrict__ correction,
                                                        int64_t num_tokens, int outputs, int top) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* s = lds + (size_t)wave * 2 * outputs;
  float* ch = s + outputs;
  const int64_t tt = (int64_t)blockIdx.x * 4 + wave;
  const bool live = tt < num_tokens;
  const int64_t t = live ? tt : num_tokens - 1;
  const float* zr = z + t * outputs;
  float mx = -INFINITY;
  for (int i = lane; i < outputs; i += 64) mx = fmaxf(mx, zr[i]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int i = lane; i < outputs; i += 64) {
    const float e = expf(zr[i] - mx);
    s[i] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
  for (int i = lane; i < outputs; i += 64) {
    const float p = s[i] * inv;
    s[i] = p;
    ch[i] = p + (correction ? correction[i] : 0.f);
  }
  __syncthreads();
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lane; i < outputs; i += 64) {
      const float v = ch[i];
      if (v > bv) {
        bv = v;
        bi = i;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi >= outputs) bi = 0;                // every value was NaN: still a valid index
    if (lane == 0) {
      if (live) {
        ids[t * top + k] = bi;
        weights[t * top + k] = s[bi];
      }
      ch[bi] = -INFINITY;
    }
    __syncthreads();
  }
}

// one workgroup sorts every slot of the step
__global__ __launch_bounds__(1024) void moe_align_kernel(int32_t* __restrict__ sorted_slots, int32_t* __restrict__ block_expert,
                                                         int32_t* __restrict__ num_blocks, const int32_t* __restrict__ ids,
                                                         int64_t num_slots, int experts) {
  extern __shared__ int32_t li[];
  int32_t* count = li;
  int32_t* start = li + experts;
  __shared__ int32_t total;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < num_slots; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0;
    for (int e = 0; e < experts; ++e) {
      start[e] = off;
      off += (count[e] + MOE_BM - 1) / MOE_BM * MOE_BM;
    }
    total = off;
    num_blocks[0] = off / MOE_BM;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += blockDim.x) {
    const int nb = (count[e] + MOE_BM - 1) / MOE_BM;
    for (int j = 0; j < nb; ++j) block_expert[start[e] / MOE_BM + j] = e;
    count[e] = 0;                              // becomes the expert's cursor
  }
  for (int i = threadIdx.x; i < total; i += blockDim.x) sorted_slots[i] = -1;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < num_slots; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < experts) sorted_slots[start[e] + atomicAdd(&count[e], 1)] = (int32_t)i;
  }
}

// bf16 on v_mfma_f32_16x16x32_bf16: the weight rows are the A operand (16 output columns), the block's 16 rows the B operand,
// so a lane ends with 4 consecutive output columns of one row.  One wave per 16 output columns, four waves per workgroup; both
// operands come straight from global memory in 16-byte pieces along K (the block's rows are re-read by the four waves out of
// the cache; the weights are read once per block).
template <bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_bf16_kernel(void* __restrict__ out, const uint16_t* __restrict__ a, int64_t a_stride,
                                                            const uint16_t* __restrict__ w, const int32_t* __restrict__ sorted_slots,
                                                            const int32_t* __restrict__ block_expert,
                                                            const int32_t* __restrict__ num_blocks, int top, int N, int K,
                                                            float limit, float alpha) {
  const int b = blockIdx.x;
  if (b >= num_blocks[0]) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  const int n0 = (blockIdx.y * 4 + wave) * 16;
  if (n0 >= N) return;
  const int e = block_expert[b];
  const int slot = sorted_slots[b * MOE_BM + c];
  const uint16_t* ar;
  bool a_live = true;
  if (GLU) {
    a_live = slot >= 0;
    ar = a + (int64_t)(a_live ? slot / top : 0) * a_stride + 8 * g;
  } else {
    ar = a + (int64_t)(b * MOE_BM + c) * a_stride + 8 * g;
  }
  const uint16_t* w0 = w + ((int64_t)e * (GLU ? 2 : 1) * N + n0 + c) * K + 8 * g;
  const uint16_t* w1 = w0 + (int64_t)N * K;                 // GLU: the up rows
  f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll 4
  for (int k0 = 0; k0 < K; k0 += 32) {
    u32x4 af = *reinterpret_cast<const u32x4*>(ar + k0);
    if (GLU && !a_live) af = zero;
    const u32x4 wf0 = *reinterpret_cast<const u32x4*>(w0 + k0);
    acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf0), __builtin_bit_cast(bf16x8, af), acc0, 0, 0, 0);
    if (GLU) {
      const u32x4 wf1 = *reinterpret_cast<const u32x4*>(w1 + k0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf1), __builtin_bit_cast(bf16x8, af), acc1, 0, 0, 0);
    }
  }
  if (GLU) {
    uint16_t* y = (uint16_t*)out + (int64_t)(b * MOE_BM + c) * N + n0 + 4 * g;
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = a_live ? clamped_glu_f(acc0[r], acc1[r], limit, alpha) : 0.f;
    *reinterpret_cast<u32x2*>(y) = u32x2{pack2_16<true>(v[0], v[1]), pack2_16<true>(v[2], v[3])};
  } else if (slot >= 0) {
    *reinterpret_cast<f32x4*>((float*)out + (int64_t)slot * N + n0 + 4 * g) = acc0;
  }
}

// any storage type and size: thread = one output element of the block, fp32 multiply-adds along K
template <typename T, bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_plain_kernel(void* __restrict__ out, const typename T::storage* __restrict__ a,
                                                             int64_t a_stride, const typename T::storage* __restrict__ w,
                                                             const int32_t* __restrict__ sorted_slots,
                                                             const int32_t* __restrict__ block_expert,
                                                             const int32_t* __restrict__ num_blocks, int top, int N, int K,
                                                             float limit, float alpha) {
  const int b = blockIdx.x;
  if (b >= num_blocks[0]) return;
  const int m = threadIdx.x & 15, n = blockIdx.y * 16 + (threadIdx.x >> 4);
  if (n >= N) return;
  const int e = block_expert[b];
  const int slot = sorted_slots[b * MOE_BM + m];
  if (slot < 0) {
    if (GLU) ((typename T::storage*)out)[(int64_t)(b * MOE_BM + m) * N + n] = T::from_f32(0.f);
    return;
  }
  const typename T::storage* ar = GLU ? a + (int64_t)(slot / top) * a_stride : a + (int64_t)(b * MOE_BM + m) * a_stride;
  const typename T::storage* w0 = w + ((int64_t)e * (GLU ? 2 : 1) * N + n) * K;
  const typename T::storage* w1 = w0 + (int64_t)N * K;
  float acc0 = 0.f, acc1 = 0.f;
  for (int k = 0; k < K; ++k) {
    const float x = T::to_f32(ar[k]);
    acc0 += x * T::to_f32(w0[k]);
    if (GLU) acc1 += x * T::to_f32(w1[k]);
  }
  if (GLU) ((typename T::storage*)out)[(int64_t)(b * MOE_BM + m) * N + n] = T::from_f32(clamped_glu_f(acc0, acc1, limit, alpha));
  else ((float*)out)[(int64_t)slot * N + n] = acc0;
}

template <typename T>
__global__ void moe_combine_kernel(typename T::storage* __restrict__ out, const float* __restrict__ expert_out,
                                   const int32_t* __restrict__ ids, const float* __restrict__ weights,
                                   const typename T::storage* __restrict__ h, int64_t h_stride,
                                   const typename T::storage* __restrict__ shared, int64_t shared_stride,
                                   const typename T::storage* __restrict__ shared_gate, int64_t shared_gate_stride, int width,
                                   int top, int experts) {
  const int64_t t = blockIdx.x;
  const float sg = (shared && shared_gate) ? sigmoid_f(T::to_f32(shared_gate[t * shared_gate_stride])) : 1.0f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = ids[t * top + k];
      const float wk = weights[t * top + k];
      acc += wk * (e < experts ? expert_out[(t * top + k) * (int64_t)width + i] : T::to_f32(h[t * h_stride + i]));
    }
    if (shared) acc += sg * T::to_f32(shared[t * shared_stride + i]);
    out[t * (int64_t)width + i] = T::from_f32(acc);
  }
}

template <typename T>
__global__ void clamped_glu_kernel(typename T::storage* __restrict__ out, const typename T::storage* __restrict__ in,
                                   int64_t in_stride, int d, float limit, float alpha) {
  const int64_t t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= d) return;
  out[t * (int64_t)d + i] = T::from_f32(clamped_glu_f(T::to_f32(in[t * in_stride + i]), T::to_f32(in[t * in_stride + d + i]), limit, alpha));
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_experts_route(int32_t* ids, float* weights, const float* router_out, const float* correction,
                               int64_t num_tokens, int outputs, int top, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(ids && weights && router_out && outputs > 0 && top > 0 && top <= outputs && outputs <= 2048,
              "moe_route: %d router outputs (<= 2048), top %d", outputs, top);
  hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)((num_tokens + 3) / 4)), dim3(256), (size_t)8 * outputs * sizeof(float),
                     (hipStream_t)stream, ids, weights, router_out, correction, num_tokens, outputs, top);
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int64_t aphro_experts_align_capacity(int64_t num_slots, int experts) {
  return (num_slots + (int64_t)experts * (MOE_BM - 1) + MOE_BM - 1) / MOE_BM * MOE_BM;
}

extern "C" int aphro_experts_align(int32_t* sorted_slots, int64_t capacity, int32_t* block_expert, int32_t* num_blocks,
                               const int32_t* ids, int64_t num_slots, int experts, void* stream) {
  APHRO_CHECK(sorted_slots && block_expert && num_blocks && ids && num_slots > 0 && experts > 0 && experts <= 4096,
              "moe_align: bad arguments (%d experts)", experts);
  APHRO_CHECK(capacity >= aphro_experts_align_capacity(num_slots, experts) && capacity < 0x7fffffff, "moe_align: capacity too small");
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (size_t)2 * experts * sizeof(int32_t), (hipStream_t)stream,
                     sorted_slots, block_expert, num_blocks, ids, num_slots, experts);
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

static int moe_gemm(bool glu, void* out, const void* a, int64_t a_stride, const void* w, const int32_t* sorted_slots,
                    const int32_t* block_expert, const int32_t* num_blocks, int64_t capacity, int top, int N, int K, float limit,
                    float alpha, int dtype, void* stream) {
  APHRO_CHECK(out && a && w && sorted_slots && block_expert && num_blocks && capacity > 0 && capacity % MOE_BM == 0 && top > 0 &&
                  N > 0 && K > 0 && a_stride >= K, "moe gemm: bad arguments");
  const unsigned blocks = (unsigned)(capacity / MOE_BM);
  const bool mfma = dtype == APHRO_BF16 && N % 16 == 0 && K % 32 == 0 && a_stride % 8 == 0 && ((uintptr_t)a & 15) == 0 &&
                    ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 15) == 0;
  if (mfma) {
    const dim3 grid(blocks, (unsigned)((N + 63) / 64));
    if (glu)
      hipLaunchKernelGGL((moe_gemm_bf16_kernel<true>), grid, dim3(256), 0, (hipStream_t)stream, out, (const uint16_t*)a, a_stride,
                         (const uint16_t*)w, sorted_slots, block_expert, num_blocks, top, N, K, limit, alpha);
    else
      hipLaunchKernelGGL((moe_gemm_bf16_kernel<false>), grid, dim3(256), 0, (hipStream_t)stream, out, (const uint16_t*)a, a_stride,
                         (const uint16_t*)w, sorted_slots, block_expert, num_blocks, top, N, K, limit, alpha);
  } else {
    const dim3 grid(blocks, (unsigned)((N + 15) / 16));
    MIX_DISPATCH_DTYPE(dtype, {
      typedef typename T::storage S;
      if (glu)
        hipLaunchKernelGGL((moe_gemm_plain_kernel<T, true>), grid, dim3(256), 0, (hipStream_t)stream, out, (const S*)a, a_stride,
                           (const S*)w, sorted_slots, block_expert, num_blocks, top, N, K, limit, alpha);
      else
        hipLaunchKernelGGL((moe_gemm_plain_kernel<T, false>), grid, dim3(256), 0, (hipStream_t)stream, out, (const S*)a, a_stride,
                           (const S*)w, sorted_slots, block_expert, num_blocks, top, N, K, limit, alpha);
    });
  }
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_experts_glu_gemm(void* y, const void* h, int64_t h_stride, const void* w_gate_up, const int32_t* sorted_slots,
                                  const int32_t* block_expert, const int32_t* num_blocks, int64_t capacity, int top, int ff,
                                  int width, float limit, float alpha, int dtype, void* stream) {
  return moe_gemm(true, y, h, h_stride, w_gate_up, sorted_slots, block_expert, num_blocks, capacity, top, ff, width, limit, alpha,
                  dtype, stream);
}

extern "C" int aphro_experts_down_gemm(float* expert_out, const void* y, const void* w_down, const int32_t* sorted_slots,
                                   const int32_t* block_expert, const int32_t* num_blocks, int64_t capacity, int top, int width,
                                   int ff, int dtype, void* stream) {
  return moe_gemm(false, expert_out, y, ff, w_down, sorted_slots, block_expert, num_blocks, capacity, top, width, ff, 0.f, 0.f,
                  dtype, stream);
}

extern "C" int aphro_experts_combine(void* out, const float* expert_out, const int32_t* ids, const float* weights, const void* h,
                                 int64_t h_stride, const void* shared, int64_t shared_stride, const void* shared_gate,
                                 int64_t shared_gate_stride, int64_t num_tokens, int width, int top, int experts, int dtype,
                                 void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && expert_out && ids && weights && h && width > 0 && top > 0 && experts >= 0 && h_stride >= width &&
                  (!shared || shared_stride >= width), "moe_combine: bad arguments");
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((moe_combine_kernel<T>), dim3((unsigned)num_tokens), dim3(width >= 1024 ? 256 : 128), 0, (hipStream_t)stream,
                       (S*)out, expert_out, ids, weights, (const S*)h, h_stride, (const S*)shared, shared_stride,
                       (const S*)shared_gate, shared_gate_stride, width, top, experts);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_clamped_glu(void* out, const void* in, int64_t in_stride, int64_t num_tokens, int d, float limit, float alpha,
                                 int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && in && d > 0 && in_stride >= 2 * (int64_t)d && num_tokens <= 0x7fffffff && (d + 255) / 256 <= 65535,
              "clamped_glu: bad arguments");
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((clamped_glu_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((d + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (S*)out, (const S*)in, in_stride, d, limit, alpha);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
