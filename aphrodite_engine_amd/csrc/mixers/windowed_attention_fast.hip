// bf16 fast paths of differential attention under a sliding window that keeps the first tokens (same semantics as
// windowed_attention.hip followed by differential_norm_gate, in one launch: the two maps of a head are computed side by side,
// joined as a_1 - lambda a_2, brought to unit RMS over the head's values, scaled and gated, and leave as bf16):
//
//  * wa_prefill_kernel<DK, DV>: segments of >= WA_MFMA_MIN_LEN rows.  A workgroup of four waves owns 64 consecutive query rows
//    of one (segment, head) and BOTH maps: per key tile of 64 it stages the two maps' key rows and the one shared value tile in
//    LDS (K chunk-swizzled, V transposed, the next tile's cache rows in flight in registers meanwhile), S^T = K Q^T on
//    v_mfma_f32_16x16x32_bf16 for each map, so that the probabilities come out as the B operand of O^T = V^T P^T and the V
//    fragments read from LDS feed both maps.  Only key tiles that some row of the workgroup can see are visited: the tiles of the
//    kept first tokens, then from the tile of the lowest window start on; a wave skips tiles none of its 16 rows sees, and the
//    mask is applied only on tiles that are not wholly visible to the wave.
//  * wa_decode_mfma_kernel<DK, DV>: the other rows (single decoded tokens, short portions), one workgroup per (row, kv head):
//    the columns of a score tile are the kv head's query heads, the keys are the row's visible ones -- numbered kept tokens
//    first, then the window -- staged through LDS like a prompt tile; long key ranges are split over workgroups and merged
//    (wa_merge_kernel).  Measured before it: the same rows on the vector ALUs (a key row over 16 lanes, DPP-folded dot products)
//    took 2 to 2.4 times as long at 1028 visible keys -- instruction-bound, whatever the split.
#include "mixers_common.h"

namespace aphro {

struct WAParams {
  uint16_t* out;              // bf16 [T, heads * vdim]
  const uint16_t* q;          // bf16 [T, heads * 2 * dim]
  const uint16_t* gate;       // bf16 [T, heads * vdim] raw, or null
  const uint16_t* k_cache;    // [blocks, block, kv_heads * 2, dim]
  const uint16_t* v_cache;    // [blocks, block, kv_heads, vdim]
  const int32_t* block_tables;
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* ctx_len;
  const int32_t* seq_of_token;
  int64_t out_stride, q_stride, gate_stride, num_blocks;
  int max_blocks, block_size, heads, kv_heads, dim, vdim, window, keep_first, min_len, bs_shift, max_tiles;
  float scale, lambda, out_scale, eps;
  float* ws;                  // decoded rows, key range split over workgroups: partials [T, heads, 2 maps, nsplit, 2 + vdim]
  int nsplit;
};

__device__ __forceinline__ int wa_slot(const WAParams& p, const int32_t* bt, int key) {
  int blk, off;
  if (p.bs_shift >= 0) {
    blk = bt[key >> p.bs_shift];
    off = key & (p.block_size - 1);
  } else {
    blk = bt[key / p.block_size];
    off = key % p.block_size;
  }
  if (blk < 0 || blk >= p.num_blocks) blk = 0;             // never read outside the pool
  return blk * p.block_size + off;
}

constexpr int WA_BM = 64, WA_BN = 64, WA_VT = WA_BN + 4;

template <int DK, int DV>
struct WAStage {
  static constexpr int NCHK = DK / 8, NCHV = DV / 8;
  static constexpr int KI = (WA_BN * NCHK + 255) / 256, VI = (WA_BN / 2 * NCHV + 255) / 256;
  u16x8 k[2][KI], v0[VI], v1[VI];
};

// Rows t0 .. t0 + 63 of a key numbering in which number r stands for key r below ns and for key lo + (r - ns) from there on
// (a prompt tile passes ns = INT_MAX: the numbering is the keys themselves); nk: numbers in all.
template <int DK, int DV>
__device__ __forceinline__ void wa_load(WAStage<DK, DV>& st, const WAParams& p, const int32_t* bt, int kvh, int t0, int nk,
                                        int ns = 0x7fffffff, int lo = 0) {
  constexpr int NCHK = DK / 8, NCHV = DV / 8;
  const int64_t krow = (int64_t)p.kv_heads * 2 * DK, vrow = (int64_t)p.kv_heads * DV;
#pragma unroll
  for (int it = 0; it < WAStage<DK, DV>::KI; ++it) {
    const int i = threadIdx.x + 256 * it;
    if (i < WA_BN * NCHK) {
      const int tok = i / NCHK, ch = i % NCHK;
      const int r = min(t0 + tok, nk - 1);
      const uint16_t* kr = p.k_cache + (int64_t)wa_slot(p, bt, r < ns ? r : lo + (r - ns)) * krow + (int64_t)kvh * 2 * DK + 8 * ch;
      st.k[0][it] = *reinterpret_cast<const u16x8*>(kr);
      st.k[1][it] = *reinterpret_cast<const u16x8*>(kr + DK);
    }
  }
#pragma unroll
  for (int it = 0; it < WAStage<DK, DV>::VI; ++it) {
    const int i = threadIdx.x + 256 * it;
    if (i < WA_BN / 2 * NCHV) {
      const int tp = i / NCHV, ch = i % NCHV;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int r = min(t0 + 2 * tp + half, nk - 1);
        const int key = r < ns ? r : lo + (r - ns);
        u16x8 vv = *reinterpret_cast<const u16x8*>(p.v_cache + (int64_t)wa_slot(p, bt, key) * vrow + kvh * DV + 8 * ch);
        if (t0 + 2 * tp + half >= nk) vv = u16x8{0, 0, 0, 0, 0, 0, 0, 0};    // beyond the sequence: no NaN into P V
        if (half == 0) st.v0[it] = vv;
        else st.v1[it] = vv;
      }
    }
  }
}

template <int DK, int DV>
__device__ __forceinline__ void wa_store(const WAStage<DK, DV>& st, uint16_t* k_lds, uint16_t* vt_lds) {
  constexpr int NCHK = DK / 8, NCHV = DV / 8;
  constexpr int SWZ = (NCHK & -NCHK) - 1;
#pragma unroll
  for (int it = 0; it < WAStage<DK, DV>::KI; ++it) {
    const int i = threadIdx.x + 256 * it;
    if (i < WA_BN * NCHK) {
      const int tok = i / NCHK, ch = i % NCHK;
      *reinterpret_cast<u16x8*>(&k_lds[tok * DK + 8 * (ch ^ (tok & SWZ))]) = st.k[0][it];
      *reinterpret_cast<u16x8*>(&k_lds[WA_BN * DK + tok * DK + 8 * (ch ^ (tok & SWZ))]) = st.k[1][it];
    }
  }
#pragma unroll
  for (int it = 0; it < WAStage<DK, DV>::VI; ++it) {
    const int i = threadIdx.x + 256 * it;
    if (i < WA_BN / 2 * NCHV) {
      const int tp = i / NCHV, ch = i % NCHV;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        *reinterpret_cast<uint32_t*>(&vt_lds[(8 * ch + j) * WA_VT + 2 * tp]) = (uint32_t)st.v0[it][j] | ((uint32_t)st.v1[it][j] << 16);
    }
  }
}

template <int DK, int DV>
__global__ __launch_bounds__(256) void wa_prefill_kernel(WAParams p) {
  constexpr int NCHK = DK / 8, NKS = DK / 32, NDT = DV / 16, NH = WA_BN / 16, NPK = WA_BN / 32;
  constexpr int SWZ = (NCHK & -NCHK) - 1;
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[2 * WA_BN * DK];
  __shared__ __attribute__((aligned(16))) uint16_t vt_lds[DV * WA_VT];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
  const int seq = blockIdx.y;
  const int len = p.q_len[seq];
  if (len < p.min_len) return;
  const int ntiles = (len + WA_BM - 1) / WA_BM;
  // Workgroups go to the 8 XCDs round-robin by their linear index and each XCD has its own L2: the (tile, head) pairs are
  // numbered so that the query heads of one kv head -- the workgroups that read the same keys and values -- share an XCD.
  int head, rank;
  {
    constexpr int NX = 8;
    const int G = p.kv_heads, QU = p.heads / p.kv_heads, x = blockIdx.x % NX, j = blockIdx.x / NX;
    if (G % NX == 0) {
      const int ux = (G / NX) * QU, ul = j % ux;
      rank = j / ux;
      head = ((ul / QU) * NX + x) * QU + ul % QU;
    } else if (NX % G == 0) {
      const int share = NX / G, pair = j * share + x / G;
      rank = pair / QU;
      head = (x % G) * QU + pair % QU;
    } else {
      rank = blockIdx.x / p.heads;
      head = blockIdx.x % p.heads;
    }
  }
  const int tile = ntiles - 1 - rank;
  if (tile < 0 || rank >= p.max_tiles) return;
  const int ctx = p.ctx_len[seq], s0 = p.q_start[seq];
  const int kvh = head / (p.heads / p.kv_heads);
  const int q0 = tile * WA_BM;
  const int qrow = q0 + 16 * wave + c;
  const bool qvalid = qrow < len;
  const int qpos = ctx + qrow;
  const int window = p.window > 0 ? p.window : 0x3fffffff, keep = p.keep_first;
  constexpr float LOG2E = 1.4426950408889634f;
  const float qs = p.scale * LOG2E;                        // scores in units of ln 2: the exponentials are exp2
  u32x4 qf[2][NKS];
  {
    const uint16_t* qp = p.q + (int64_t)(s0 + min(qrow, len - 1)) * p.q_stride + (int64_t)head * 2 * DK;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) qf[t][ks] = *reinterpret_cast<const u32x4*>(qp + t * DK + 32 * ks + 8 * g);
  }
  f32x4 o[2][NDT];
  float m_run[2], l_run[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    m_run[t] = -INFINITY;
    l_run[t] = 0.f;
#pragma unroll
    for (int i = 0; i < NDT; ++i) o[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int32_t* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const int nk = ctx + min(len, q0 + WA_BM);               // keys the tile's last row sees
  const int lo_wg = max(0, ctx + q0 - window + 1);         // the lowest window start among the workgroup's rows
  const int win_tile = lo_wg / WA_BN * WA_BN;
  const int pw0 = ctx + q0 + 16 * wave, pw1 = pw0 + 15;    // positions of the wave's rows

  WAStage<DK, DV> st;
  int t0 = keep > 0 ? 0 : win_tile;
  wa_load<DK, DV>(st, p, bt, kvh, t0, nk);
  while (t0 < nk) {
    int t_next = t0 + WA_BN;
    if (t_next >= keep && t_next < win_tile) t_next = win_tile;        // past the kept tokens: on to the window
    __syncthreads();                                        // the previous tile is consumed
    wa_store<DK, DV>(st, k_lds, vt_lds);
    __syncthreads();
    if (t_next < nk) wa_load<DK, DV>(st, p, bt, kvh, t_next, nk);      // in flight during this tile's products
    const int tc = t0;
    t0 = t_next;
    if (tc > pw1) continue;                                 // every key of the tile is ahead of the wave's rows
    if (tc >= keep && tc + WA_BN - 1 < pw0 - window + 1) continue;     // ... or behind every row's window, none of them kept
    f32x4 s[2][NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      const int tok = 16 * h + c;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        s[t][h] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const int ch = (4 * ks + g) ^ (tok & SWZ);
          const u32x4 kf = *reinterpret_cast<const u32x4*>(&k_lds[t * WA_BN * DK + tok * DK + 8 * ch]);
          s[t][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[t][ks]),
                                                            s[t][h], 0, 0, 0);
        }
      }
    }
    // wholly visible to the wave: behind its first row and inside its last row's window
    const bool masked = !(tc + WA_BN - 1 <= pw0 && pw1 - tc < window);
    u32x4 pf[2][NPK];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      float pv[NH][4];
      float mx = -INFINITY;
#pragma unroll
      for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float xv = s[t][h][r] * qs;
          if (masked) {
            const int j = tc + 16 * h + 4 * g + r;
            xv = (j <= qpos && (qpos - j < window || j < keep)) ? xv : -INFINITY;
          }
          pv[h][r] = xv;
          mx = fmaxf(mx, xv);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run[t], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;          // a row that has seen no key yet
      const float alpha = __builtin_amdgcn_exp2f(m_run[t] - m_safe);
      m_run[t] = m_new;
      float lsum = 0.f;
#pragma unroll
      for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float e = __builtin_amdgcn_exp2f(pv[h][r] - m_safe);  // a masked score is -inf: exactly 0
          pv[h][r] = e;
          lsum += e;
        }
      l_run[t] = l_run[t] * alpha + lsum;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) o[t][dt] *= alpha;
#pragma unroll
      for (int pk = 0; pk < NPK; ++pk)
        pf[t][pk] = u32x4{pack2_16<true>(pv[2 * pk][0], pv[2 * pk][1]), pack2_16<true>(pv[2 * pk][2], pv[2 * pk][3]),
                          pack2_16<true>(pv[2 * pk + 1][0], pv[2 * pk + 1][1]), pack2_16<true>(pv[2 * pk + 1][2], pv[2 * pk + 1][3])};
    }
#pragma unroll
    for (int pk = 0; pk < NPK; ++pk) {
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        const uint16_t* vr = &vt_lds[(16 * dt + c) * WA_VT + 32 * pk + 4 * g];
        const u32x2 lo = *reinterpret_cast<const u32x2*>(vr);
        const u32x2 hi = *reinterpret_cast<const u32x2*>(vr + 16);
        const u32x4 vf = {lo[0], lo[1], hi[0], hi[1]};
#pragma unroll
        for (int t = 0; t < 2; ++t)
          o[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf), __builtin_bit_cast(bf16x8, pf[t][pk]),
                                                             o[t][dt], 0, 0, 0);
      }
    }
  }
  // join the maps: the row's DV values sit in the four lanes c, c + 16, c + 32, c + 48
  float inv[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    float l = l_run[t];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    inv[t] = l > 0.f ? 1.f / l : 0.f;
  }
  const float f1 = p.lambda * inv[1];
  float ss = 0.f;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float d = o[0][dt][r] * inv[0] - f1 * o[1][dt][r];
      o[0][dt][r] = d;
      ss += d * d;
    }
  ss += __shfl_xor(ss, 16, 64);
  ss += __shfl_xor(ss, 32, 64);
  if (!qvalid) return;
  const float rstd = p.out_scale / sqrtf(ss / (float)DV + p.eps);
  uint16_t* op = p.out + (int64_t)(s0 + qrow) * p.out_stride + head * DV + 4 * g;
  const uint16_t* gp = p.gate ? p.gate + (int64_t)(s0 + qrow) * p.gate_stride + head * DV + 4 * g : nullptr;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = o[0][dt][r] * rstd;
    if (gp) {
      const u16x4 gg = *reinterpret_cast<const u16x4*>(gp + 16 * dt);
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] *= sigmoid_f(BFloat::to_f32(gg[r]));
    }
    *reinterpret_cast<u32x2*>(op + 16 * dt) = u32x2{pack2_16<true>(v[0], v[1]), pack2_16<true>(v[2], v[3])};
  }
}

// Decoded rows on the matrix cores: a workgroup owns one row and one kv head; the 16 columns of a score tile are the kv head's
// query heads (up to 16), so the two maps' keys and the shared values of a 64-key tile -- staged in LDS exactly as for a prompt
// portion, over the row's visible keys numbered kept tokens first -- serve all of them.  The four waves divide a tile's work
// by map and by half: wave 2 m + h takes map m and keys 32 h .. 32 h + 31, keeps its own running maximum, sum and output, and
// the halves, then the maps, meet in LDS at the end (or, when the key range is split over workgroups, in wa_merge_kernel).
template <int DK, int DV>
__global__ __launch_bounds__(256) void wa_decode_mfma_kernel(WAParams p) {
  constexpr int NCHK = DK / 8, NKS = DK / 32, NDT = DV / 16;
  constexpr int SWZ = (NCHK & -NCHK) - 1;
  constexpr int KBYTES = 2 * WA_BN * DK * 2, VBYTES = DV * WA_VT * 2, MROW = DV + 2;
  static_assert(KBYTES + VBYTES >= 2 * 16 * MROW * 4, "the merge buffer reuses the tiles' memory");
  __shared__ __attribute__((aligned(16))) unsigned char smem[KBYTES + VBYTES];
  uint16_t* k_lds = reinterpret_cast<uint16_t*>(smem);
  uint16_t* vt_lds = reinterpret_cast<uint16_t*>(smem + KBYTES);
  float* mrg = reinterpret_cast<float*>(smem);             // [2 maps][16 heads][2 + DV], after the last tile
  const int t = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  const int seq = p.seq_of_token[t];
  if (p.q_len[seq] >= p.min_len) return;                   // the prompt kernel's share
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
  const int mp = wave >> 1, pk = wave & 1;
  const int QH = p.heads / p.kv_heads;
  const int pos = p.ctx_len[seq] + (t - p.q_start[seq]);
  const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int ns = min(p.keep_first, lo);
  const int nvis = ns + pos - lo + 1;                      // visible keys: [0, ns) and [lo, pos]
  constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;
  const float qs = p.scale * LOG2E;
  const int head = kvh * QH + min(c, QH - 1);              // columns beyond the kv head's query heads repeat the last one
  u32x4 qf[NKS];
  {
    const uint16_t* qp = p.q + (int64_t)t * p.q_stride + ((int64_t)head * 2 + mp) * DK;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qf[ks] = *reinterpret_cast<const u32x4*>(qp + 32 * ks + 8 * g);
  }
  f32x4 o[NDT];
#pragma unroll
  for (int i = 0; i < NDT; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const int32_t* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const int ntiles = (nvis + WA_BN - 1) / WA_BN;
  const int tps = (ntiles + p.nsplit - 1) / p.nsplit;
  const int r_end = min(ntiles, (split + 1) * tps) * WA_BN;
  int r0 = split * tps * WA_BN;
  WAStage<DK, DV> st;
  if (r0 < r_end) wa_load<DK, DV>(st, p, bt, kvh, r0, nvis, ns, lo);
  for (; r0 < r_end; r0 += WA_BN) {
    __syncthreads();                                        // the previous tile is consumed
    wa_store<DK, DV>(st, k_lds, vt_lds);
    __syncthreads();
    if (r0 + WA_BN < r_end) wa_load<DK, DV>(st, p, bt, kvh, r0 + WA_BN, nvis, ns, lo);
    f32x4 s[2];
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      const int tok = 16 * (2 * pk + h2) + c;
      s[h2] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int ch = (4 * ks + g) ^ (tok & SWZ);
        const u32x4 kf = *reinterpret_cast<const u32x4*>(&k_lds[mp * WA_BN * DK + tok * DK + 8 * ch]);
        s[h2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[ks]), s[h2], 0, 0, 0);
      }
    }
    float pv[2][4];
    float mx = -INFINITY;
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int idx = r0 + 16 * (2 * pk + h2) + 4 * g + r;
        const float xv = idx < nvis ? s[h2][r] * qs : -INFINITY;
        pv[h2][r] = xv;
        mx = fmaxf(mx, xv);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
    m_run = m_new;
    float lsum = 0.f;
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float e = __builtin_amdgcn_exp2f(pv[h2][r] - m_safe);
        pv[h2][r] = e;
        lsum += e;
      }
    l_run = l_run * alpha + lsum;
    const u32x4 pf = {pack2_16<true>(pv[0][0], pv[0][1]), pack2_16<true>(pv[0][2], pv[0][3]), pack2_16<true>(pv[1][0], pv[1][1]),
                      pack2_16<true>(pv[1][2], pv[1][3])};
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      o[dt] *= alpha;
      const uint16_t* vr = &vt_lds[(16 * dt + c) * WA_VT + 32 * pk + 4 * g];
      const u32x2 vlo = *reinterpret_cast<const u32x2*>(vr);
      const u32x2 vhi = *reinterpret_cast<const u32x2*>(vr + 16);
      const u32x4 vf = {vlo[0], vlo[1], vhi[0], vhi[1]};
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf), __builtin_bit_cast(bf16x8, pf), o[dt], 0, 0, 0);
    }
  }
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  __syncthreads();                                          // the tiles' memory becomes the merge buffer
  float* mine = mrg + (mp * 16 + c) * MROW;
  if (pk == 1) {                                            // the second half of the keys hands over to the first
    if (g == 0) {
      mine[0] = m_run;
      mine[1] = l_run;
    }
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) mine[2 + 16 * dt + 4 * g + r] = o[dt][r];
  }
  __syncthreads();
  if (pk == 0) {
    const float m2 = mine[0], l2 = mine[1];
    const float M = fmaxf(m_run, m2);
    const float Ms = M == -INFINITY ? 0.f : M;
    const float f1 = __builtin_amdgcn_exp2f(m_run - Ms), f2 = __builtin_amdgcn_exp2f(m2 - Ms);
    l_run = l_run * f1 + l2 * f2;
    m_run = M;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[dt][r] = o[dt][r] * f1 + mine[2 + 16 * dt + 4 * g + r] * f2;
  }
  if (p.nsplit > 1) {                                       // this split's share of (head, map); wa_merge_kernel finishes the row
    if (pk == 0 && c < QH) {
      float* w = p.ws + ((((int64_t)t * p.heads + head) * 2 + mp) * p.nsplit + split) * (2 + DV);
      if (g == 0) {
        w[0] = m_run * LN2;                                 // wa_merge_kernel weighs with natural exponentials
        w[1] = l_run;
      }
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f32x4*>(w + 2 + 16 * dt + 4 * g) = o[dt];
    }
    return;
  }
  __syncthreads();                                          // map 1's first half has read what it was handed
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
  if (wave == 2) {
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) mine[2 + 16 * dt + 4 * g + r] = o[dt][r] * inv;
  }
  __syncthreads();
  if (wave != 0) return;
  const float* a2 = mrg + (16 + c) * MROW + 2;
  float ss = 0.f;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float d = o[dt][r] * inv - p.lambda * a2[16 * dt + 4 * g + r];
      o[dt][r] = d;
      ss += d * d;
    }
  ss += __shfl_xor(ss, 16, 64);
  ss += __shfl_xor(ss, 32, 64);
  if (c >= QH) return;
  const float rstd = p.out_scale / sqrtf(ss / (float)DV + p.eps);
  uint16_t* op = p.out + (int64_t)t * p.out_stride + head * DV + 4 * g;
  const uint16_t* gp = p.gate ? p.gate + (int64_t)t * p.gate_stride + head * DV + 4 * g : nullptr;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = o[dt][r] * rstd;
    if (gp) {
      const u16x4 gg = *reinterpret_cast<const u16x4*>(gp + 16 * dt);
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] *= sigmoid_f(BFloat::to_f32(gg[r]));
    }
    *reinterpret_cast<u32x2*>(op + 16 * dt) = u32x2{pack2_16<true>(v[0], v[1]), pack2_16<true>(v[2], v[3])};
  }
}

// one wave per (row, head): merges the key splits (at most 8) of both maps, joins, norms and gates.  vdim <= 256.  Every load
// of a map is requested before the first is used.
__global__ __launch_bounds__(64) void wa_merge_kernel(WAParams p) {
  constexpr int MAXS = 8;
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  if (p.q_len[p.seq_of_token[t]] >= p.min_len) return;
  const int stride = 2 + p.vdim;
  float a[2][4];
#pragma unroll
  for (int mp = 0; mp < 2; ++mp) {
    const float* w = p.ws + (((int64_t)t * p.heads + head) * 2 + mp) * p.nsplit * stride;
    float mz[MAXS], lz[MAXS], oz[MAXS][4];
#pragma unroll
    for (int z = 0; z < MAXS; ++z) {
      const bool on = z < p.nsplit;
      mz[z] = on ? w[z * stride] : -INFINITY;
      lz[z] = on ? w[z * stride + 1] : 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) oz[z][i] = (on && lane + 64 * i < p.vdim) ? w[z * stride + 2 + lane + 64 * i] : 0.f;
    }
    float M = -INFINITY;
#pragma unroll
    for (int z = 0; z < MAXS; ++z) M = fmaxf(M, mz[z]);
    float L = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int z = 0; z < MAXS; ++z) {
      const float f = mz[z] == -INFINITY ? 0.f : __expf(mz[z] - M);
      L += lz[z] * f;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] += oz[z][i] * f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) a[mp][i] = o[i] / L;
  }
  float d[4], ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    d[i] = a[0][i] - p.lambda * a[1][i];
    ss += d[i] * d[i];
  }
  const float rstd = p.out_scale / sqrtf(wave_sum(ss) / (float)p.vdim + p.eps);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int col = lane + 64 * i;
    if (col >= p.vdim) continue;
    float v = d[i] * rstd;
    if (p.gate) v *= sigmoid_f(BFloat::to_f32(p.gate[(int64_t)t * p.gate_stride + head * p.vdim + col]));
    p.out[(int64_t)t * p.out_stride + head * p.vdim + col] = BFloat::from_f32(v);
  }
}

template <int DK>
static void wa_launch_prefill_dv(const WAParams& p, dim3 grid, hipStream_t st) {
  switch (p.vdim) {
    case 32: hipLaunchKernelGGL((wa_prefill_kernel<DK, 32>), grid, dim3(256), 0, st, p); break;
    case 64: hipLaunchKernelGGL((wa_prefill_kernel<DK, 64>), grid, dim3(256), 0, st, p); break;
    case 96: hipLaunchKernelGGL((wa_prefill_kernel<DK, 96>), grid, dim3(256), 0, st, p); break;
    case 128: hipLaunchKernelGGL((wa_prefill_kernel<DK, 128>), grid, dim3(256), 0, st, p); break;
  }
}

static bool wa_prefill_supported(int dim, int vdim) {
  auto ok = [](int d) { return d == 32 || d == 64 || d == 96 || d == 128; };
  return ok(dim) && ok(vdim);
}

static void wa_prefill_launch(const WAParams& p0, int max_q_len, int num_seqs, hipStream_t st) {
  WAParams p = p0;
  p.max_tiles = (max_q_len + WA_BM - 1) / WA_BM;
  const int per_seq = (p.max_tiles * p.heads + 7) / 8 * 8;   // a multiple of the XCD count: the numbering repeats per segment
  const dim3 grid((unsigned)per_seq, (unsigned)num_seqs);
  switch (p.dim) {
    case 32: wa_launch_prefill_dv<32>(p, grid, st); break;
    case 64: wa_launch_prefill_dv<64>(p, grid, st); break;
    case 96: wa_launch_prefill_dv<96>(p, grid, st); break;
    case 128: wa_launch_prefill_dv<128>(p, grid, st); break;
  }
}

template <int DK>
static void wa_launch_decode_mfma_dv(const WAParams& p, dim3 grid, hipStream_t st) {
  switch (p.vdim) {
    case 32: hipLaunchKernelGGL((wa_decode_mfma_kernel<DK, 32>), grid, dim3(256), 0, st, p); break;
    case 64: hipLaunchKernelGGL((wa_decode_mfma_kernel<DK, 64>), grid, dim3(256), 0, st, p); break;
    case 96: hipLaunchKernelGGL((wa_decode_mfma_kernel<DK, 96>), grid, dim3(256), 0, st, p); break;
    case 128: hipLaunchKernelGGL((wa_decode_mfma_kernel<DK, 128>), grid, dim3(256), 0, st, p); break;
  }
}

// decoded rows on the matrix cores: kv heads of up to 16 query heads, the prompt kernel's sizes
static bool wa_decode_mfma_supported(int heads, int kv_heads, int dim, int vdim) {
  return wa_prefill_supported(dim, vdim) && heads / kv_heads <= 16 && vdim % 4 == 0;
}

static void wa_decode_mfma_launch(const WAParams& p, int64_t num_tokens, hipStream_t st) {
  const dim3 grid((unsigned)num_tokens, (unsigned)p.kv_heads, (unsigned)p.nsplit);
  switch (p.dim) {
    case 32: wa_launch_decode_mfma_dv<32>(p, grid, st); break;
    case 64: wa_launch_decode_mfma_dv<64>(p, grid, st); break;
    case 96: wa_launch_decode_mfma_dv<96>(p, grid, st); break;
    case 128: wa_launch_decode_mfma_dv<128>(p, grid, st); break;
  }
  if (p.nsplit > 1) hipLaunchKernelGGL(wa_merge_kernel, dim3((unsigned)num_tokens, (unsigned)p.heads), dim3(64), 0, st, p);
}

// key splits of the matrix-core decode kernel: a thousand workgroups, at least two tiles each
static int wa_decode_mfma_splits(int64_t num_tokens, int heads, int kv_heads, int vdim, int max_visible, int64_t ws_floats) {
  const int tiles = (max_visible + WA_BN - 1) / WA_BN;
  const int64_t wgs = num_tokens * kv_heads;
  int64_t n = (1024 + wgs - 1) / wgs;
  if (n > tiles / 2) n = tiles / 2;
  if (n > 8) n = 8;
  while (n > 1 && num_tokens * heads * 2 * n * (2 + vdim) > ws_floats) --n;
  return n < 1 ? 1 : (int)n;
}

constexpr int WA_MFMA_MIN_LEN = 8;

}  // namespace aphro

using namespace aphro;

/* 1 if aphro_differential_window_attention serves these sizes (bf16 only), else 0 */
extern "C" int aphro_differential_window_attention_supported(int heads, int kv_heads, int dim, int vdim, int dtype) {
  if (dtype != APHRO_BF16 || heads <= 0 || kv_heads <= 0 || heads % kv_heads) return 0;
  return wa_decode_mfma_supported(heads, kv_heads, dim, vdim) ? 1 : 0;
}

extern "C" int aphro_differential_window_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* gate,
                                                   int64_t gate_stride, const void* k_cache, const void* v_cache,
                                                   const int32_t* block_tables, int max_blocks, int64_t num_blocks, int block_size,
                                                   const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                                                   const int32_t* seq_of_token, int64_t num_tokens, int num_seqs, int min_q_len,
                                                   int max_q_len, int heads, int kv_heads, int dim, int vdim, float scale, int window,
                                                   int keep_first, float lambda, float out_scale, float eps, int max_kv_len,
                                                   float* workspace, int64_t workspace_floats, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && q && k_cache && v_cache && block_tables && q_start && q_len && ctx_len && seq_of_token,
              "differential_window_attention: null argument");
  APHRO_CHECK(aphro_differential_window_attention_supported(heads, kv_heads, dim, vdim, dtype),
              "differential_window_attention: bf16 with dim, vdim in {32, 64, 96, 128} only (heads %d / %d, dim %d, vdim %d, dtype %d)",
              heads, kv_heads, dim, vdim, dtype);
  APHRO_CHECK(block_size > 0 && max_blocks > 0 && num_blocks > 0 && num_seqs > 0 && keep_first >= 0 && 0 < min_q_len &&
                  min_q_len <= max_q_len, "differential_window_attention: bad geometry");
  APHRO_CHECK(q_stride >= (int64_t)heads * 2 * dim && out_stride >= (int64_t)heads * vdim && (!gate || gate_stride >= (int64_t)heads * vdim),
              "differential_window_attention: row strides smaller than the rows");
  APHRO_CHECK(((uintptr_t)q & 15) == 0 && (q_stride & 7) == 0 && ((uintptr_t)out & 7) == 0 && (out_stride & 3) == 0 &&
                  ((uintptr_t)gate & 7) == 0 && (gate_stride & 3) == 0 && ((uintptr_t)k_cache & 15) == 0 && ((uintptr_t)v_cache & 15) == 0,
              "differential_window_attention: rows must be 16-byte aligned (q, caches) and 8-byte aligned (out, gate)");
  WAParams p;
  p.out = (uint16_t*)out; p.q = (const uint16_t*)q; p.gate = (const uint16_t*)gate;
  p.k_cache = (const uint16_t*)k_cache; p.v_cache = (const uint16_t*)v_cache;
  p.block_tables = block_tables; p.q_start = q_start; p.q_len = q_len; p.ctx_len = ctx_len; p.seq_of_token = seq_of_token;
  p.out_stride = out_stride; p.q_stride = q_stride; p.gate_stride = gate_stride; p.num_blocks = num_blocks;
  p.max_blocks = max_blocks; p.block_size = block_size; p.heads = heads; p.kv_heads = kv_heads; p.dim = dim; p.vdim = vdim;
  p.window = window; p.keep_first = keep_first; p.scale = scale; p.lambda = lambda; p.out_scale = out_scale; p.eps = eps;
  p.max_tiles = 0;
  p.bs_shift = -1;
  for (int sft = 0; sft < 20; ++sft)
    if ((1 << sft) == block_size) p.bs_shift = sft;
  p.min_len = WA_MFMA_MIN_LEN;
  p.ws = workspace;
  p.nsplit = 1;
  if (workspace && max_kv_len > 0) {
    const int vis = window > 0 && window + keep_first < max_kv_len ? window + keep_first : max_kv_len;
    p.nsplit = wa_decode_mfma_splits(num_tokens, heads, kv_heads, vdim, vis, workspace_floats);
  }
  if (max_q_len >= WA_MFMA_MIN_LEN) wa_prefill_launch(p, max_q_len, num_seqs, (hipStream_t)stream);
  if (min_q_len < WA_MFMA_MIN_LEN) wa_decode_mfma_launch(p, num_tokens, (hipStream_t)stream);
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
