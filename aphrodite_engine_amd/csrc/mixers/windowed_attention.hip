// Softmax attention over a token-major paged cache under a sliding window that also keeps the sequence's first tokens:
// row i sees key j if j <= i and (i - j < window or j < keep_first); no rotation and no bias: positions enter only through
// the mask.  A head may carry several MAPS -- attentions of their own, each with its own queries and keys, over the SAME
// values (the two maps of differential attention): q is [T, heads * maps * dim] and the key cache holds kv_heads * maps key
// rows per token, head by head, map after map; the value cache holds kv_heads rows.  The result is every map's normalised
// output in fp32, [T, heads * maps * vdim]: what combines the maps (differential_norm_gate) reads full precision.
//
// One kernel for prompt portions and single decoded tokens: a batch is a list of segments, every query row reads the keys it
// sees from the cache (which already holds the segment's own).  Only the visible keys are walked: they are numbered
// 0 .. n_vis - 1, the kept first tokens and then the window.
//
// windowed_attention_kernel is the fp32-math kernel of any size and storage type: a workgroup of four waves per (row, head,
// map); the waves take 64-key tiles round-robin, lane = key for the scores, lane = column for P V; (max, sum, accumulator)
// merged through LDS.
#include "mixers_common.h"

namespace aphro {

constexpr int WA_WAVES = 4;
constexpr int WA_MAX_DIM = 512;
constexpr int WA_MAX_VDIM = 256;

// the visible keys of a row at position pos: [0, ns) and [lo, pos]
struct Visible {
  int ns, lo, n;
  __device__ __forceinline__ Visible(int pos, int window, int keep_first) {
    lo = window > 0 ? max(0, pos - window + 1) : 0;
    ns = min(keep_first, lo);
    n = ns + pos - lo + 1;
  }
  __device__ __forceinline__ int key(int r) const { return r < ns ? r : lo + (r - ns); }
};

template <typename T>
__device__ __forceinline__ float wa_dot(const float* __restrict__ qsh, const typename T::storage* __restrict__ kr, int dim) {
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

template <typename T, int EPL>
__global__ __launch_bounds__(256) void windowed_attention_kernel(
    float* __restrict__ out, int64_t out_stride, const typename T::storage* __restrict__ q, int64_t q_stride,
    const typename T::storage* __restrict__ k_cache, const typename T::storage* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int max_blocks, int64_t num_blocks, int block_size,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ seq_of_token, int heads,
    int kv_heads, int maps, int dim, int vdim, float scale, int window, int keep_first) {
  __shared__ __attribute__((aligned(16))) float qsh[WA_MAX_DIM];
  __shared__ float merge[WA_WAVES][2 + EPL * 64];
  const int t = blockIdx.x, hm = blockIdx.y;            // hm = head * maps + map
  const int h = hm / maps, mp = hm % maps;
  const int s = seq_of_token[t];
  const int pos = ctx_len[s] + (t - q_start[s]);
  const Visible vis(pos, window, keep_first);
  const int g = h / (heads / kv_heads);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) qsh[i] = T::to_f32(q[(int64_t)t * q_stride + (int64_t)hm * dim + i]);
  __syncthreads();
  const int32_t* bt = block_tables + (int64_t)s * max_blocks;
  const int64_t krow = (int64_t)kv_heads * maps * dim, vrow = (int64_t)kv_heads * vdim;
  const int koff = (g * maps + mp) * dim, voff = g * vdim;
  float m = -INFINITY, l = 0.f, acc[EPL];
#pragma unroll
  for (int c = 0; c < EPL; ++c) acc[c] = 0.f;
  const int ntiles = (vis.n + 63) >> 6;
  for (int tile = wave; tile < ntiles; tile += WA_WAVES) {
    const int r = tile * 64 + lane;
    float sc = -INFINITY;
    if (r < vis.n) {
      const int j = vis.key(r);
      const int blk = bt[j / block_size];
      if (blk >= 0 && blk < num_blocks)
        sc = wa_dot<T>(qsh, k_cache + ((int64_t)blk * block_size + j % block_size) * krow + koff, dim) * scale;
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    const float p = (sc == -INFINITY) ? 0.f : expf(sc - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int c = 0; c < EPL; ++c) acc[c] *= alpha;
    const int cnt = min(64, vis.n - tile * 64);
#pragma unroll 4
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p), jj));
      const int j2 = vis.key(tile * 64 + jj);
      int blk = bt[j2 / block_size];
      if (blk < 0 || blk >= num_blocks) blk = 0;           // its probability is 0
      const typename T::storage* vr = v_cache + ((int64_t)blk * block_size + j2 % block_size) * vrow + voff;
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
  for (int w = 0; w < WA_WAVES; ++w) M = fmaxf(M, merge[w][0]);
  float L = 0.f, f[WA_WAVES];
#pragma unroll
  for (int w = 0; w < WA_WAVES; ++w) {
    f[w] = (merge[w][0] == -INFINITY) ? 0.f : expf(merge[w][0] - M);
    L += merge[w][1] * f[w];
  }
  const float inv = 1.0f / L;
#pragma unroll
  for (int c = 0; c < EPL; ++c) {
    const int col = lane + 64 * c;
    if (col < vdim) {
      float o = 0.f;
#pragma unroll
      for (int w = 0; w < WA_WAVES; ++w) o += merge[w][2 + col] * f[w];
      out[(int64_t)t * out_stride + (int64_t)hm * vdim + col] = o * inv;
    }
  }
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_windowed_attention(float* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                                        const void* v_cache, const int32_t* block_tables, int max_blocks, int64_t num_blocks,
                                        int block_size, const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                                        const int32_t* seq_of_token, int64_t num_tokens, int num_seqs, int min_q_len,
                                        int max_q_len, int heads, int kv_heads, int maps, int dim, int vdim, float scale,
                                        int window, int keep_first, int max_kv_len, float* workspace, int64_t workspace_floats,
                                        int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && q && k_cache && v_cache && block_tables && q_start && q_len && ctx_len && seq_of_token,
              "windowed_attention: null argument");
  APHRO_CHECK(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && maps >= 1 && (int64_t)heads * maps <= 65535,
              "windowed_attention: heads %d / kv heads %d / maps %d", heads, kv_heads, maps);
  APHRO_CHECK(dim > 0 && dim <= WA_MAX_DIM && vdim > 0 && vdim <= WA_MAX_VDIM, "windowed_attention: dim %d (<= %d) / vdim %d (<= %d)",
              dim, WA_MAX_DIM, vdim, WA_MAX_VDIM);
  APHRO_CHECK(block_size > 0 && max_blocks > 0 && num_blocks > 0 && num_seqs > 0, "windowed_attention: bad cache geometry");
  APHRO_CHECK(q_stride >= (int64_t)heads * maps * dim && out_stride >= (int64_t)heads * maps * vdim,
              "windowed_attention: row strides smaller than the rows");
  APHRO_CHECK(keep_first >= 0, "windowed_attention: keep_first %d", keep_first);
  const dim3 grid((unsigned)num_tokens, (unsigned)(heads * maps));
  const int epl = (vdim + 63) / 64;
#define WA_LAUNCH(EPL)                                                                                                      \
  hipLaunchKernelGGL((windowed_attention_kernel<T, EPL>), grid, dim3(256), 0, (hipStream_t)stream, out, out_stride, (const S*)q, \
                     q_stride, (const S*)k_cache, (const S*)v_cache, block_tables, max_blocks, num_blocks, block_size, q_start,   \
                     ctx_len, seq_of_token, heads, kv_heads, maps, dim, vdim, scale, window, keep_first)
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    switch (epl) {
      case 1: WA_LAUNCH(1); break;
      case 2: WA_LAUNCH(2); break;
      case 3: WA_LAUNCH(3); break;
      default: WA_LAUNCH(4); break;
    }
  });
#undef WA_LAUNCH
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
