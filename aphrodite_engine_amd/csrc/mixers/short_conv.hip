// Short causal convolution over time on every channel of a projection's output, for a batch of segments:
//   y_t[c] = sum_j w[c, j] * u_(t - taps + 1 + j)[c],   zeros before the sequence's start.
// The taps - 1 inputs that precede a segment come from the request's state slot, which afterwards holds the last taps - 1
// inputs of the sequence.  A segment that starts a sequence never reads its slot, and no input older than the sequence's
// start is read from it either, so a slot taken over from another request needs no clearing.
//
// The channels are [q | k | v]: the q part goes to a dense output, the k and v parts straight into the token-major paged
// cache at the rows' slots (what attention reads is the convolved key and value).  Products and sums are fp32, one rounding
// to the storage type.
#include "mixers_common.h"

namespace aphro {

constexpr int SC_MAX_TAPS = 16;

template <typename T>
__global__ void short_conv_kernel(typename T::storage* __restrict__ q_out, int64_t q_out_stride,
                                  typename T::storage* __restrict__ k_cache, typename T::storage* __restrict__ v_cache,
                                  const int64_t* __restrict__ cache_slots, int64_t num_cache_slots,
                                  const typename T::storage* __restrict__ u, int64_t u_stride,
                                  const typename T::storage* __restrict__ w, const typename T::storage* __restrict__ state,
                                  const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start,
                                  const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ seq_of_token, int cq, int ck,
                                  int cv, int taps) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int C = cq + ck + cv;
  if (c >= C) return;
  const int s = seq_of_token[t];
  const int r = (int)t - q_start[s], ctx = ctx_len[s];
  const typename T::storage* st = state ? state + ((int64_t)state_slots[s] * (taps - 1)) * C + c : nullptr;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int i = r - taps + 1 + j;            // row of the segment, negative: before it
    float x = 0.f;
    if (i >= 0) x = T::to_f32(u[(t - r + i) * u_stride + c]);
    else if (ctx + i >= 0) x = T::to_f32(st[(int64_t)(taps - 1 + i) * C]);
    acc += T::to_f32(w[(int64_t)c * taps + j]) * x;
  }
  const typename T::storage y = T::from_f32(acc);
  if (c < cq) {
    q_out[t * q_out_stride + c] = y;
  } else {
    const int64_t slot = cache_slots[t];
    if (slot < 0 || slot >= num_cache_slots) return;
    if (c < cq + ck) k_cache[slot * ck + (c - cq)] = y;
    else v_cache[slot * cv + (c - cq - ck)] = y;
  }
}

// After the convolution: the slot takes the last taps - 1 inputs of the sequence (from the segment, or -- for a segment
// shorter than that -- from what the slot held, moved up).  One thread owns a channel of a segment and reads all it needs
// before it writes.
template <typename T>
__global__ void short_conv_state_kernel(typename T::storage* __restrict__ state, const typename T::storage* __restrict__ u,
                                        int64_t u_stride, const int32_t* __restrict__ state_slots,
                                        const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                        const int32_t* __restrict__ ctx_len, int C, int taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int n = q_len[s], ctx = ctx_len[s], keep = taps - 1;
  typename T::storage* st = state + ((int64_t)state_slots[s] * keep) * C + c;
  typename T::storage val[SC_MAX_TAPS];
  for (int m = 0; m < keep; ++m) {
    const int p = ctx + n - keep + m;          // position in the sequence
    typename T::storage x = T::from_f32(0.f);
    if (p >= ctx) x = u[((int64_t)q_start[s] + (p - ctx)) * u_stride + c];
    else if (p >= 0) x = st[(int64_t)(p - ctx + keep) * C];
    val[m] = x;
  }
  for (int m = 0; m < keep; ++m) st[(int64_t)m * C] = val[m];
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_short_conv(void* q_out, int64_t q_out_stride, void* k_cache, void* v_cache, const int64_t* cache_slots,
                                int64_t num_cache_slots, const void* u, int64_t u_stride, const void* w, void* state,
                                const int32_t* state_slots, const int32_t* q_start, const int32_t* q_len,
                                const int32_t* ctx_len, const int32_t* seq_of_token, int64_t num_tokens, int num_seqs, int cq,
                                int ck, int cv, int taps, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  const int C = cq + ck + cv;
  APHRO_CHECK(u && w && q_start && q_len && ctx_len && seq_of_token && num_seqs > 0 && cq >= 0 && ck >= 0 && cv >= 0 && C > 0,
              "short_conv: bad arguments");
  APHRO_CHECK(taps >= 1 && taps <= SC_MAX_TAPS, "short_conv: %d taps (1 .. %d)", taps, SC_MAX_TAPS);
  APHRO_CHECK(taps == 1 || (state && state_slots), "short_conv: more than one tap needs the state slots");
  APHRO_CHECK(u_stride >= C && (cq == 0 || (q_out && q_out_stride >= cq)), "short_conv: row strides smaller than the rows");
  APHRO_CHECK(ck + cv == 0 || (k_cache && v_cache && cache_slots && num_cache_slots > 0 && ck > 0 && cv > 0),
              "short_conv: key / value channels need the cache and the rows' slots");
  APHRO_CHECK(num_tokens <= 0x7fffffff && (C + 255) / 256 <= 65535, "short_conv: too large");
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((short_conv_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((C + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (S*)q_out, q_out_stride, (S*)k_cache, (S*)v_cache, cache_slots, num_cache_slots,
                       (const S*)u, u_stride, (const S*)w, (const S*)state, state_slots, q_start, ctx_len, seq_of_token, cq, ck,
                       cv, taps);
    if (taps > 1)
      hipLaunchKernelGGL((short_conv_state_kernel<T>), dim3((unsigned)num_seqs, (unsigned)((C + 255) / 256)), dim3(256), 0,
                         (hipStream_t)stream, (S*)state, (const S*)u, u_stride, state_slots, q_start, q_len, ctx_len, C, taps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
