// Softmax attention over a token-major paged cache with a tabulated distance bias, a position-dependent query
// temperature and a per-head sigmoid output gate -- one kernel for prompt portions and single decoded tokens (a batch
// is a list of segments; every query row attends to keys 0 .. its own position, all read from the cache).
//
// Work split: one workgroup of four waves per (query row, head).  The waves take the 64-key tiles round-robin; inside a
// tile lane = key for the scores (fp32 dot product, online softmax with wave-wide max / sum), then lane = output column
// for P V (the probability of key jj is broadcast with v_readlane).  The four partial (max, sum, accumulator) triples
// are merged through LDS.  Scores, softmax and the accumulators are fp32 whatever the storage type.
#include "mixers_common.h"

namespace aphro {

template <typename T>
__global__ void paged_kv_write_kernel(typename T::storage* __restrict__ k_cache, typename T::storage* __restrict__ v_cache,
                                      const typename T::storage* __restrict__ k, int64_t k_stride,
                                      const typename T::storage* __restrict__ v, int64_t v_stride,
                                      const int64_t* __restrict__ slots, int kd, int vd, int64_t num_slots) {
  const int64_t t = blockIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0 || slot >= num_slots) return;
  const typename T::storage* kr = k + t * k_stride;
  const typename T::storage* vr = v + t * v_stride;
  for (int i = threadIdx.x; i < kd; i += blockDim.x) k_cache[slot * kd + i] = kr[i];
  for (int i = threadIdx.x; i < vd; i += blockDim.x) v_cache[slot * vd + i] = vr[i];
}

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ qsh, const typename T::storage* __restrict__ kr, int dim) {
  float d0 = 0.f, d1 = 0.f;
  if constexpr (sizeof(typename T::storage) == 2) {
    if ((dim & 7) == 0) {
      for (int i = 0; i < dim; i += 8) {
        const u16x8 kk = *reinterpret_cast<const u16x8*>(kr + i);
        const f32x4 qa = *reinterpret_cast<const f32x4*>(qsh + i), qb = *reinterpret_cast<const f32x4*>(qsh + i + 4);
        d0 += qa[0] * T::to_f32(kk[0]) + qa[1] * T::to_f32(kk[1]) + qa[2] * T::to_f32(kk[2]) + qa[3] * T::to_f32(kk[3]);
        d1 += qb[0] * T::to_f32(kk[4]) + qb[1] * T::to_f32(kk[5]) + qb[2] * T::to_f32(kk[6]) + qb[3] * T::to_f32(kk[7]);
      }
      return d0 + d1;
    }
  } else {
    if ((dim & 3) == 0) {
      for (int i = 0; i < dim; i += 4) {
        const f32x4 kk = *reinterpret_cast<const f32x4*>(kr + i);
        const f32x4 qa = *reinterpret_cast<const f32x4*>(qsh + i);
        d0 += qa[0] * kk[0] + qa[1] * kk[1];
        d1 += qa[2] * kk[2] + qa[3] * kk[3];
      }
      return d0 + d1;
    }
  }
  for (int i = 0; i < dim; ++i) d0 += qsh[i] * T::to_f32(kr[i]);
  return d0;
}

constexpr int DBA_WAVES = 4;
constexpr int DBA_MAX_DIM = 512;
constexpr int DBA_MAX_VDIM = 256;

template <typename T, int EPL>
__global__ __launch_bounds__(256) void distance_bias_attention_kernel(
    typename T::storage* __restrict__ out, int64_t out_stride, const typename T::storage* __restrict__ q, int64_t q_stride,
    const typename T::storage* __restrict__ gate, int64_t gate_stride, const typename T::storage* __restrict__ k_cache,
    const typename T::storage* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    int64_t num_blocks, int block_size, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ seq_of_token, int heads, int kv_heads, int dim, int vdim, float scale,
    const float* __restrict__ bias_lut, int lut_len, float temp_coef, int temp_every, float out_scale) {
  __shared__ __attribute__((aligned(16))) float qsh[DBA_MAX_DIM];
  __shared__ float merge[DBA_WAVES][2 + EPL * 64];
  const int t = blockIdx.x, h = blockIdx.y;
  const int s = seq_of_token[t];
  const int pos = ctx_len[s] + (t - q_start[s]);
  const int nkeys = pos + 1;
  const int g = h / (heads / kv_heads);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float qs = scale;
  if (temp_coef != 0.f) qs *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every + 1));
  for (int i = threadIdx.x; i < dim; i += blockDim.x) qsh[i] = T::to_f32(q[(int64_t)t * q_stride + h * dim + i]);
  __syncthreads();
  const int32_t* bt = block_tables + (int64_t)s * max_blocks;
  const float* lut = bias_lut ? bias_lut + (int64_t)h * lut_len : nullptr;
  const int64_t krow = (int64_t)kv_heads * dim, vrow = (int64_t)kv_heads * vdim;
  float m = -INFINITY, l = 0.f, acc[EPL];
#pragma unroll
  for (int c = 0; c < EPL; ++c) acc[c] = 0.f;
  const int ntiles = (nkeys + 63) >> 6;
  for (int tile = wave; tile < ntiles; tile += DBA_WAVES) {
    const int j = tile * 64 + lane;
    float sc = -INFINITY;
    if (j < nkeys) {
      const int blk = bt[j / block_size];
      if (blk >= 0 && blk < num_blocks) {
        const typename T::storage* kr = k_cache + ((int64_t)blk * block_size + j % block_size) * krow + g * dim;
        sc = dot_row<T>(qsh, kr, dim) * qs;
        if (lut) {
          const int dist = pos - j;
          sc += lut[dist < lut_len ? dist : lut_len - 1];
        }
      }
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);     // a wave's first tile
    const float p = (sc == -INFINITY) ? 0.f : expf(sc - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int c = 0; c < EPL; ++c) acc[c] *= alpha;
    const int cnt = min(64, nkeys - tile * 64);
#pragma unroll 4
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p), jj));
      const int j2 = tile * 64 + jj;
      int blk = bt[j2 / block_size];
      if (blk < 0 || blk >= num_blocks) blk = 0;           // its probability is 0 (masked above)
      const typename T::storage* vr = v_cache + ((int64_t)blk * block_size + j2 % block_size) * vrow + g * vdim;
#pragma unroll
      for (int c = 0; c < EPL; ++c) {
        const int col = lane + 64 * c;
        if (col < vdim) acc[c] += pj * T::to_f32(vr[col]);
      }
    }
  }
  if (lane == 0) {
    merge[wave][0] = m;
    merge[wave][1] = l;
  }
#pragma unroll
  for (int c = 0; c < EPL; ++c) merge[wave][2 + lane + 64 * c] = acc[c];
  __syncthreads();
  if (wave != 0) return;
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < DBA_WAVES; ++w) M = fmaxf(M, merge[w][0]);
  float L = 0.f, f[DBA_WAVES];
#pragma unroll
  for (int w = 0; w < DBA_WAVES; ++w) {
    f[w] = (merge[w][0] == -INFINITY) ? 0.f : expf(merge[w][0] - M);
    L += merge[w][1] * f[w];
  }
  float sig = out_scale;
  if (gate) sig *= sigmoid_f(T::to_f32(gate[(int64_t)t * gate_stride + h]));
  const float inv = sig / L;
#pragma unroll
  for (int c = 0; c < EPL; ++c) {
    const int col = lane + 64 * c;
    if (col < vdim) {
      float o = 0.f;
#pragma unroll
      for (int w = 0; w < DBA_WAVES; ++w) o += merge[w][2 + col] * f[w];
      out[(int64_t)t * out_stride + h * vdim + col] = T::from_f32(o * inv);
    }
  }
}

// biased_attention_fast.hip
struct DBAParams {
  uint16_t* out;
  const uint16_t* q;
  const uint16_t* gate;
  const uint16_t* k_cache;
  const uint16_t* v_cache;
  const int32_t* block_tables;
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* ctx_len;
  const int32_t* seq_of_token;
  const float* bias_lut;
  int64_t out_stride, q_stride, gate_stride, num_blocks;
  int max_blocks, block_size, heads, kv_heads, dim, vdim, lut_len, temp_every, min_len;
  float scale, temp_coef, out_scale;
  float* ws;
  int bs_shift;
  int max_tiles;
};
bool dba_prefill_supported(int dim, int vdim);
bool dba_decode_supported(int heads, int kv_heads, int dim, int vdim);
void dba_prefill_launch(const DBAParams& p, int max_q_len, int num_seqs, hipStream_t st);
void dba_decode_launch(const DBAParams& p, int64_t num_tokens, int nsplit, hipStream_t st);
int dba_decode_splits(int64_t num_tokens, int kv_heads, int max_kv_len, int64_t ws_floats, int heads, int vdim);
constexpr int DBA_MFMA_MIN_LEN = 8;     // segments at least this long go to the matrix-core kernel

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_paged_kv_write(void* k_cache, void* v_cache, const void* k, int64_t k_stride, const void* v,
                                    int64_t v_stride, const int64_t* slots, int64_t num_tokens, int kv_heads, int dim,
                                    int vdim, int64_t num_slots, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(k_cache && v_cache && k && v && slots && kv_heads > 0 && dim > 0 && vdim > 0 && num_slots > 0,
              "paged_kv_write: bad arguments");
  const int kd = kv_heads * dim, vd = kv_heads * vdim;
  APHRO_CHECK(k_stride >= kd && v_stride >= vd, "paged_kv_write: row strides smaller than the rows");
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((paged_kv_write_kernel<T>), dim3((unsigned)num_tokens), dim3(128), 0, (hipStream_t)stream,
                       (S*)k_cache, (S*)v_cache, (const S*)k, k_stride, (const S*)v, v_stride, slots, kd, vd, num_slots);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_distance_bias_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* gate,
                                             int64_t gate_stride, const void* k_cache, const void* v_cache,
                                             const int32_t* block_tables, int max_blocks, int64_t num_blocks, int block_size,
                                             const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                                             const int32_t* seq_of_token, int64_t num_tokens, int num_seqs, int min_q_len,
                                             int max_q_len, int heads, int kv_heads, int dim, int vdim, float scale,
                                             const float* bias_lut, int lut_len, float temp_coef, int temp_every,
                                             float out_scale, int max_kv_len, float* workspace, int64_t workspace_floats,
                                             int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && q && k_cache && v_cache && block_tables && q_start && ctx_len && seq_of_token,
              "distance_bias_attention: null argument");
  APHRO_CHECK(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && heads <= 65535, "distance_bias_attention: heads %d / kv heads %d",
              heads, kv_heads);
  APHRO_CHECK(dim > 0 && dim <= DBA_MAX_DIM && vdim > 0 && vdim <= DBA_MAX_VDIM,
              "distance_bias_attention: dim %d (<= %d) / vdim %d (<= %d)", dim, DBA_MAX_DIM, vdim, DBA_MAX_VDIM);
  APHRO_CHECK(block_size > 0 && max_blocks > 0 && num_blocks > 0 && num_seqs > 0, "distance_bias_attention: bad cache geometry");
  APHRO_CHECK(q_stride >= (int64_t)heads * dim && out_stride >= (int64_t)heads * vdim && (!gate || gate_stride >= heads),
              "distance_bias_attention: row strides smaller than the rows");
  APHRO_CHECK(!bias_lut || lut_len > 0, "distance_bias_attention: empty bias table");
  APHRO_CHECK(temp_coef == 0.f || temp_every > 0, "distance_bias_attention: temp_every must be positive");
  // bf16 with 16-byte-aligned rows: the matrix-core kernel for the long segments, the shared-key kernel for the rest
  if (dtype == APHRO_BF16 && q_len && max_q_len >= min_q_len && min_q_len > 0 && ((uintptr_t)q & 15) == 0 && (q_stride & 7) == 0) {
    DBAParams p;
    p.out = (uint16_t*)out; p.q = (const uint16_t*)q; p.gate = (const uint16_t*)gate;
    p.k_cache = (const uint16_t*)k_cache; p.v_cache = (const uint16_t*)v_cache;
    p.block_tables = block_tables; p.q_start = q_start; p.q_len = q_len; p.ctx_len = ctx_len; p.seq_of_token = seq_of_token;
    p.bias_lut = bias_lut; p.out_stride = out_stride; p.q_stride = q_stride; p.gate_stride = gate_stride; p.num_blocks = num_blocks;
    p.max_blocks = max_blocks; p.block_size = block_size; p.heads = heads; p.kv_heads = kv_heads; p.dim = dim; p.vdim = vdim;
    p.lut_len = lut_len; p.temp_every = temp_every; p.scale = scale; p.temp_coef = temp_coef; p.out_scale = out_scale;
    p.ws = workspace;
    p.max_tiles = 0;
    p.bs_shift = -1;
    for (int sft = 0; sft < 20; ++sft)
      if ((1 << sft) == block_size) p.bs_shift = sft;
    const int nsplit = workspace ? dba_decode_splits(num_tokens, kv_heads, max_kv_len, workspace_floats, heads, vdim) : 1;
    const bool pf = dba_prefill_supported(dim, vdim) && max_q_len >= DBA_MFMA_MIN_LEN;
    const bool dc = dba_decode_supported(heads, kv_heads, dim, vdim);
    const bool all_long = min_q_len >= DBA_MFMA_MIN_LEN;
    if (pf && (all_long || dc)) {
      p.min_len = DBA_MFMA_MIN_LEN;
      dba_prefill_launch(p, max_q_len, num_seqs, (hipStream_t)stream);
      if (!all_long) dba_decode_launch(p, num_tokens, nsplit, (hipStream_t)stream);
      APHRO_LAUNCH_CHECK();
      return APHRO_OK;
    }
    if (dc) {
      p.min_len = 0x7fffffff;
      dba_decode_launch(p, num_tokens, nsplit, (hipStream_t)stream);
      APHRO_LAUNCH_CHECK();
      return APHRO_OK;
    }
  }
  const dim3 grid((unsigned)num_tokens, (unsigned)heads);
  const int epl = (vdim + 63) / 64;
#define DBA_LAUNCH(EPL)                                                                                                   \
  hipLaunchKernelGGL((distance_bias_attention_kernel<T, EPL>), grid, dim3(256), 0, (hipStream_t)stream, (S*)out, out_stride, \
                     (const S*)q, q_stride, (const S*)gate, gate_stride, (const S*)k_cache, (const S*)v_cache, block_tables,  \
                     max_blocks, num_blocks, block_size, q_start, ctx_len, seq_of_token, heads, kv_heads, dim, vdim, scale,  \
                     bias_lut, lut_len, temp_coef, temp_every, out_scale)
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    switch (epl) {
      case 1: DBA_LAUNCH(1); break;
      case 2: DBA_LAUNCH(2); break;
      case 3: DBA_LAUNCH(3); break;
      default: DBA_LAUNCH(4); break;
    }
  });
#undef DBA_LAUNCH
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
