// bf16 fast paths of the distance-biased attention (same semantics as biased_attention.hip, which stays the fp32 path and
// the path of sizes these do not tile):
//
//  * dba_prefill_kernel<DK, DV>: segments of >= DBA_MFMA_MIN_LEN rows.  A workgroup of four waves owns 64 consecutive
//    query rows of one (segment, head), 16 rows per wave, and walks the visible keys 64 at a time: the K rows and V rows of
//    the tile come from the paged cache with 16-byte loads into LDS (K chunk-swizzled, V transposed), together with the 127
//    bias values the tile can need (the table is indexed by distance, and a 64 x 64 tile spans 127 distances); the next
//    tile's cache rows are fetched into registers while the current tile's products run.
//    S^T = K Q^T on v_mfma_f32_16x16x32_bf16, so that the probabilities come out in the B-operand layout of O^T = V^T P^T
//    (keys of the two 16-key halves interleaved per lane group, V fragments read in the same order); temperature, bias,
//    mask and the online softmax are fp32 on the accumulator registers.
//  * dba_decode_kernel<QH, CHL>: the other rows (single decoded tokens, short portions), one workgroup per (row, kv head)
//    serving all QH query heads of that kv head from one pass over the keys.  A key row is read by 2^CHL lanes x 16 bytes,
//    64 / 2^CHL keys per load instruction (fully coalesced); the partial dot products fold over the lanes of a key with
//    DPP shuffles; scores and probabilities stay in that layout (4 keys x QH per lane and step), which is also the layout
//    the V pass wants, so nothing is redistributed; K and V of a step are fetched together.  Four waves take the steps
//    round-robin and merge their (max, sum, acc) in LDS; long key ranges are also split over workgroups (grid z), whose
//    partial results dba_merge_kernel combines.
#include "mixers_common.h"

namespace aphro {

struct DBAParams {          // (declared alike in biased_attention.hip, which fills it)
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
  float* ws;          // decode split partials [T, heads, nsplit, 2 + vdim]
  int bs_shift;       // log2(block_size), or -1 when it is no power of two
  int max_tiles;      // prompt kernel: 64-row tiles of the longest segment
};

// row of key `key` in the token-major cache ([block, offset] -> block * block_size + offset), following the block table
__device__ __forceinline__ int dba_slot(const DBAParams& p, const int32_t* bt, int key) {
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

__device__ __forceinline__ float dba_temp(const DBAParams& p, int pos) {
  return p.temp_coef != 0.f ? 1.0f + p.temp_coef * logf((float)((pos + 1) / p.temp_every + 1)) : 1.0f;
}

constexpr int PF_BM = 64, PF_BN = 64, PF_VT = PF_BN + 4;

// One thread's share of a key tile on its way from the cache to LDS: K chunks (one key, 16 bytes) and V chunk pairs (two
// neighbouring keys, so that the transposed LDS stores are whole dwords).
template <int DK, int DV>
struct PFStage {
  static constexpr int NCHK = DK / 8, NCHV = DV / 8;
  static constexpr int KI = (PF_BN * NCHK + 255) / 256, VI = (PF_BN / 2 * NCHV + 255) / 256;
  u16x8 k[KI], v0[VI], v1[VI];
};

template <int DK, int DV>
__device__ __forceinline__ void pf_load(PFStage<DK, DV>& st, const DBAParams& p, const int32_t* bt, int kvh, int t0, int nk) {
  constexpr int NCHK = DK / 8, NCHV = DV / 8;
  const int64_t krow = (int64_t)p.kv_heads * DK, vrow = (int64_t)p.kv_heads * DV;
#pragma unroll
  for (int it = 0; it < PFStage<DK, DV>::KI; ++it) {
    const int i = threadIdx.x + 256 * it;
    if (i < PF_BN * NCHK) {
      const int tok = i / NCHK, ch = i % NCHK;
      const int key = min(t0 + tok, nk - 1);
      st.k[it] = *reinterpret_cast<const u16x8*>(p.k_cache + (int64_t)dba_slot(p, bt, key) * krow + kvh * DK + 8 * ch);
    }
  }
#pragma unroll
  for (int it = 0; it < PFStage<DK, DV>::VI; ++it) {
    const int i = threadIdx.x + 256 * it;
    if (i < PF_BN / 2 * NCHV) {
      const int tp = i / NCHV, ch = i % NCHV;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int key = min(t0 + 2 * tp + half, nk - 1);
        u16x8 vv = *reinterpret_cast<const u16x8*>(p.v_cache + (int64_t)dba_slot(p, bt, key) * vrow + kvh * DV + 8 * ch);
        if (t0 + 2 * tp + half >= nk) vv = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (half == 0) st.v0[it] = vv;
        else st.v1[it] = vv;
      }
    }
  }
}

template <int DK, int DV>
__device__ __forceinline__ void pf_store(const PFStage<DK, DV>& st, uint16_t* k_lds, uint16_t* vt_lds) {
  constexpr int NCHK = DK / 8, NCHV = DV / 8;
  constexpr int SWZ = (NCHK & -NCHK) - 1;
#pragma unroll
  for (int it = 0; it < PFStage<DK, DV>::KI; ++it) {
    const int i = threadIdx.x + 256 * it;
    if (i < PF_BN * NCHK) {
      const int tok = i / NCHK, ch = i % NCHK;
      *reinterpret_cast<u16x8*>(&k_lds[tok * DK + 8 * (ch ^ (tok & SWZ))]) = st.k[it];
    }
  }
#pragma unroll
  for (int it = 0; it < PFStage<DK, DV>::VI; ++it) {
    const int i = threadIdx.x + 256 * it;
    if (i < PF_BN / 2 * NCHV) {
      const int tp = i / NCHV, ch = i % NCHV;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        *reinterpret_cast<uint32_t*>(&vt_lds[(8 * ch + j) * PF_VT + 2 * tp]) = (uint32_t)st.v0[it][j] | ((uint32_t)st.v1[it][j] << 16);
    }
  }
}

// QT query heads of one kv head share a workgroup: the K and V fragments read from LDS feed QT products each, and the
// tile's trip from the cache to LDS is paid once for them.
template <int DK, int DV, int QT>
__global__ __launch_bounds__(256) void dba_prefill_kernel(DBAParams p) {
  constexpr int NCHK = DK / 8, NKS = DK / 32, NDT = DV / 16, NH = PF_BN / 16, NPK = PF_BN / 32;
  constexpr int SWZ = (NCHK & -NCHK) - 1;
  constexpr int NWIN = PF_BM + PF_BN - 1;
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[PF_BN * DK];
  __shared__ __attribute__((aligned(16))) uint16_t vt_lds[DV * PF_VT];
  __shared__ float bias_win[QT][NWIN + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
  const int seq = blockIdx.y;
  const int len = p.q_len[seq];
  if (len < p.min_len) return;
  const int ntiles = (len + PF_BM - 1) / PF_BM;
  // Workgroups go to the 8 XCDs round-robin by their linear index, and each XCD has its own L2: the (tile, head unit) pairs
  // are numbered so that every query head of one kv head -- the workgroups that read the same keys and values -- lands on
  // the same XCD (or the same few, when there are fewer kv heads than XCDs).  Within an XCD: longest key ranges first.
  int unit, rank;                                           // head unit: QT consecutive query heads
  {
    constexpr int NX = 8;
    const int G = p.kv_heads, QU = p.heads / p.kv_heads / QT, x = blockIdx.x % NX, j = blockIdx.x / NX;
    if (G % NX == 0) {
      const int ux = (G / NX) * QU, ul = j % ux;            // units served by this XCD, this workgroup's among them
      rank = j / ux;
      unit = ((ul / QU) * NX + x) * QU + ul % QU;
    } else if (NX % G == 0) {
      const int share = NX / G, pair = j * share + x / G;   // XCDs per kv head; (tile, unit) pair of that kv head
      rank = pair / QU;
      unit = (x % G) * QU + pair % QU;
    } else {
      rank = blockIdx.x / (p.heads / QT);
      unit = blockIdx.x % (p.heads / QT);
    }
  }
  const int tile = ntiles - 1 - rank;
  if (tile < 0 || rank >= p.max_tiles) return;
  const int head0 = unit * QT;
  const int ctx = p.ctx_len[seq], s0 = p.q_start[seq];
  const int kvh = head0 / (p.heads / p.kv_heads);
  const int q0 = tile * PF_BM;
  const int qrow = q0 + 16 * wave + c;
  const bool qvalid = qrow < len;
  const int qpos = ctx + qrow;
  constexpr float LOG2E = 1.4426950408889634f;
  const float qs = p.scale * dba_temp(p, qpos) * LOG2E;     // scores in units of ln 2: the exponentials are exp2
  u32x4 qf[QT][NKS];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const uint16_t* qp = p.q + (int64_t)(s0 + min(qrow, len - 1)) * p.q_stride + (head0 + t) * DK;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qf[t][ks] = *reinterpret_cast<const u32x4*>(qp + 32 * ks + 8 * g);
  }
  f32x4 o[QT][NDT];
  float m_run[QT], l_run[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m_run[t] = -1e30f;
    l_run[t] = 0.f;
#pragma unroll
    for (int i = 0; i < NDT; ++i) o[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int32_t* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const int nk = ctx + min(len, q0 + PF_BM);               // keys the tile's last row sees

  PFStage<DK, DV> st;
  pf_load<DK, DV>(st, p, bt, kvh, 0, nk);
  for (int t0 = 0; t0 < nk; t0 += PF_BN) {
    __syncthreads();                                        // the previous tile is consumed
    pf_store<DK, DV>(st, k_lds, vt_lds);
    const int dmin = ctx + q0 - t0 - (PF_BN - 1);           // distance of (first row, last key of the tile)
    if (threadIdx.x < QT * 128) {
      const int t = threadIdx.x >> 7, x = threadIdx.x & 127;
      if (x < NWIN) {
        float b = 0.f;
        if (p.bias_lut) {
          const int dist = dmin + x;
          b = p.bias_lut[(int64_t)(head0 + t) * p.lut_len + (dist < 0 ? 0 : (dist < p.lut_len ? dist : p.lut_len - 1))] * LOG2E;
        }
        bias_win[t][x] = b;
      }
    }
    __syncthreads();
    if (t0 + PF_BN < nk) pf_load<DK, DV>(st, p, bt, kvh, t0 + PF_BN, nk);      // in flight during this tile's products
    if (t0 > ctx + q0 + 16 * wave + 15) continue;           // every key of the tile is ahead of the wave's rows
    f32x4 s[QT][NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) {
#pragma unroll
      for (int t = 0; t < QT; ++t) s[t][h] = f32x4{0.f, 0.f, 0.f, 0.f};
      const int tok = 16 * h + c;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int ch = (4 * ks + g) ^ (tok & SWZ);
        const u32x4 kf = *reinterpret_cast<const u32x4*>(&k_lds[tok * DK + 8 * ch]);
#pragma unroll
        for (int t = 0; t < QT; ++t)
          s[t][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[t][ks]),
                                                            s[t][h], 0, 0, 0);
      }
    }
    const bool diag = t0 + PF_BN - 1 > ctx + q0 + 16 * wave; // some key of the tile is ahead of some row of the wave
    u32x4 pf[QT][NPK];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float pv[NH][4];
      float mx = -1e30f;
      const float* bw = &bias_win[t][qpos - t0 - dmin - 4 * g];    // bias of (this row, key t0 + 4 g); keys count downwards
#pragma unroll
      for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float xv = s[t][h][r] * qs + bw[-(16 * h + r)];
          if (diag) xv = t0 + 16 * h + 4 * g + r <= qpos ? xv : -1e30f;
          pv[h][r] = xv;
          mx = fmaxf(mx, xv);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run[t], mx);              // finite for every row that is kept: key 0 is visible
      const float alpha = __builtin_amdgcn_exp2f(m_run[t] - m_new);
      m_run[t] = m_new;
      float lsum = 0.f;
#pragma unroll
      for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float e = __builtin_amdgcn_exp2f(pv[h][r] - m_new);    // a masked score is 1e30 below: exactly 0
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
        const uint16_t* vr = &vt_lds[(16 * dt + c) * PF_VT + 32 * pk + 4 * g];
        const u32x2 lo = *reinterpret_cast<const u32x2*>(vr);
        const u32x2 hi = *reinterpret_cast<const u32x2*>(vr + 16);
        const u32x4 vf = {lo[0], lo[1], hi[0], hi[1]};
#pragma unroll
        for (int t = 0; t < QT; ++t)
          o[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf), __builtin_bit_cast(bf16x8, pf[t][pk]),
                                                             o[t][dt], 0, 0, 0);
      }
    }
  }
  if (!qvalid) return;                                      // (after the last shuffle-free point: the sums below are per lane group)
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    float l = l_run[t];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    float f = (l > 0.f ? 1.f / l : 0.f) * p.out_scale;
    if (p.gate) f *= sigmoid_f(BFloat::to_f32(p.gate[(int64_t)(s0 + qrow) * p.gate_stride + head0 + t]));
    uint16_t* op = p.out + (int64_t)(s0 + qrow) * p.out_stride + (head0 + t) * DV;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) op[16 * dt + 4 * g + r] = BFloat::from_f32(o[t][dt][r] * f);
    }
  }
}

template <int QH, int CHL>
__global__ __launch_bounds__(256) void dba_decode_kernel(DBAParams p) {
  constexpr int CH = 1 << CHL;       // lanes per key row (16 bytes each)
  constexpr int KP = 64 / CH;        // keys per load instruction
  constexpr int NI = 4;              // load instructions per step of the online softmax (few: registers buy occupancy)
  constexpr int KT = NI * KP;        // keys per step
  __shared__ float merge[4][QH][2 + 8 * CH];
  const int t = blockIdx.x, kvh = blockIdx.y;
  const int seq = p.seq_of_token[t];
  if (p.q_len[seq] >= p.min_len) return;                   // the prompt kernel's share
  const int pos = p.ctx_len[seq] + (t - p.q_start[seq]);
  const int nkeys = pos + 1;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ck = lane & (CH - 1), kg = lane >> CHL;
  const bool kin = 8 * ck < p.dim, vin = 8 * ck < p.vdim;
  const float qs = p.scale * dba_temp(p, pos);
  float qv[QH][8];
#pragma unroll
  for (int qh = 0; qh < QH; ++qh) {
    u16x8 raw = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (kin) raw = *reinterpret_cast<const u16x8*>(p.q + (int64_t)t * p.q_stride + (kvh * QH + qh) * p.dim + 8 * ck);
#pragma unroll
    for (int j = 0; j < 8; ++j) qv[qh][j] = BFloat::to_f32(raw[j]);
  }
  const int32_t* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const int64_t krow = (int64_t)p.kv_heads * p.dim, vrow = (int64_t)p.kv_heads * p.vdim;
  float m[QH], l[QH], acc[QH][8];
#pragma unroll
  for (int qh = 0; qh < QH; ++qh) {
    m[qh] = -INFINITY;
    l[qh] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[qh][j] = 0.f;
  }
  const int ntiles = (nkeys + KT - 1) / KT;
  const int nsplit = gridDim.z, tps = (ntiles + nsplit - 1) / nsplit;
  const int tile_end = min(ntiles, ((int)blockIdx.z + 1) * tps);
  for (int tile = (int)blockIdx.z * tps + wave; tile < tile_end; tile += 4) {
    float sc[NI][QH];
    u16x8 vv[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int key = tile * KT + i * KP + kg;
      const bool valid = key < nkeys;
      const int64_t slot = dba_slot(p, bt, valid ? key : 0);
      u16x8 kk = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
      vv[i] = kk;
      if (valid && kin) kk = *reinterpret_cast<const u16x8*>(p.k_cache + slot * krow + kvh * p.dim + 8 * ck);
      if (valid && vin) vv[i] = *reinterpret_cast<const u16x8*>(p.v_cache + slot * vrow + kvh * p.vdim + 8 * ck);
      float kf[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) kf[j] = BFloat::to_f32(kk[j]);
      const int dist = pos - key;
#pragma unroll
      for (int qh = 0; qh < QH; ++qh) {
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) d += qv[qh][j] * kf[j];
        d = group_sum<CHL>(d);
        float b = 0.f;
        if (p.bias_lut && valid) b = p.bias_lut[(int64_t)(kvh * QH + qh) * p.lut_len + (dist < p.lut_len ? dist : p.lut_len - 1)];
        sc[i][qh] = valid ? d * qs + b : -INFINITY;
      }
    }
#pragma unroll
    for (int qh = 0; qh < QH; ++qh) {
      float mx = sc[0][qh];
#pragma unroll
      for (int i = 1; i < NI; ++i) mx = fmaxf(mx, sc[i][qh]);
#pragma unroll
      for (int o = CH; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      const float m_new = fmaxf(m[qh], mx);                // finite: the tile's first key exists
      const float alpha = (m[qh] == -INFINITY) ? 0.f : __expf(m[qh] - m_new);
      m[qh] = m_new;
      float ls = 0.f;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const float e = (sc[i][qh] == -INFINITY) ? 0.f : __expf(sc[i][qh] - m_new);
        sc[i][qh] = e;
        ls += e;
      }
      l[qh] = l[qh] * alpha + ls;                          // this key group's share; groups are summed at the end
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[qh][j] *= alpha;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float vf = BFloat::to_f32(vv[i][j]);
#pragma unroll
        for (int qh = 0; qh < QH; ++qh) acc[qh][j] += sc[i][qh] * vf;
      }
    }
  }
  // fold the key groups of the wave, then the four waves
#pragma unroll
  for (int qh = 0; qh < QH; ++qh) {
#pragma unroll
    for (int o = CH; o < 64; o <<= 1) {
      l[qh] += __shfl_xor(l[qh], o, 64);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[qh][j] += __shfl_xor(acc[qh][j], o, 64);
    }
    if (lane == 0) {
      merge[wave][qh][0] = m[qh];
      merge[wave][qh][1] = l[qh];
    }
    if (kg == 0) {
#pragma unroll
      for (int j = 0; j < 8; ++j) merge[wave][qh][2 + 8 * ck + j] = acc[qh][j];
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < QH * p.vdim; idx += 256) {
    const int qh = idx / p.vdim, col = idx % p.vdim;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) M = fmaxf(M, merge[w][qh][0]);
    float L = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = (merge[w][qh][0] == -INFINITY) ? 0.f : __expf(merge[w][qh][0] - M);
      L += merge[w][qh][1] * f;
      o += merge[w][qh][2 + col] * f;
    }
    const int head = kvh * QH + qh;
    if (nsplit > 1) {                                       // this split's share; dba_merge_kernel finishes the row
      float* w = p.ws + (((int64_t)t * p.heads + head) * nsplit + blockIdx.z) * (2 + p.vdim);
      if (col == 0) {
        w[0] = M;
        w[1] = L;
      }
      w[2 + col] = o;
      continue;
    }
    float sig = p.out_scale;
    if (p.gate) sig *= sigmoid_f(BFloat::to_f32(p.gate[(int64_t)t * p.gate_stride + head]));
    p.out[(int64_t)t * p.out_stride + head * p.vdim + col] = BFloat::from_f32(o * sig / L);
  }
}

__global__ void dba_merge_kernel(DBAParams p, int nsplit) {
  const int t = blockIdx.x, head = blockIdx.y;
  if (p.q_len[p.seq_of_token[t]] >= p.min_len) return;
  const float* w = p.ws + ((int64_t)t * p.heads + head) * nsplit * (2 + p.vdim);
  float M = -INFINITY;
  for (int z = 0; z < nsplit; ++z) M = fmaxf(M, w[z * (2 + p.vdim)]);
  float L = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float mz = w[z * (2 + p.vdim)];
    if (mz != -INFINITY) L += w[z * (2 + p.vdim) + 1] * __expf(mz - M);
  }
  float sig = p.out_scale;
  if (p.gate) sig *= sigmoid_f(BFloat::to_f32(p.gate[(int64_t)t * p.gate_stride + head]));
  for (int col = threadIdx.x; col < p.vdim; col += blockDim.x) {
    float o = 0.f;
    for (int z = 0; z < nsplit; ++z) {
      const float mz = w[z * (2 + p.vdim)];
      if (mz != -INFINITY) o += w[z * (2 + p.vdim) + 2 + col] * __expf(mz - M);
    }
    p.out[(int64_t)t * p.out_stride + head * p.vdim + col] = BFloat::from_f32(o * sig / L);
  }
}

template <int DK, int QT>
static void launch_prefill_dv(const DBAParams& p, dim3 grid, hipStream_t st) {
  switch (p.vdim) {
    case 32: hipLaunchKernelGGL((dba_prefill_kernel<DK, 32, QT>), grid, dim3(256), 0, st, p); break;
    case 64: hipLaunchKernelGGL((dba_prefill_kernel<DK, 64, QT>), grid, dim3(256), 0, st, p); break;
    case 96: hipLaunchKernelGGL((dba_prefill_kernel<DK, 96, QT>), grid, dim3(256), 0, st, p); break;
    case 128: hipLaunchKernelGGL((dba_prefill_kernel<DK, 128, QT>), grid, dim3(256), 0, st, p); break;
  }
}

bool dba_prefill_supported(int dim, int vdim) {
  auto ok = [](int d) { return d == 32 || d == 64 || d == 96 || d == 128; };
  return ok(dim) && ok(vdim);
}

template <int QT>
static void launch_prefill_dk(const DBAParams& p, dim3 grid, hipStream_t st) {
  switch (p.dim) {
    case 32: launch_prefill_dv<32, QT>(p, grid, st); break;
    case 64: launch_prefill_dv<64, QT>(p, grid, st); break;
    case 96: launch_prefill_dv<96, QT>(p, grid, st); break;
    case 128: launch_prefill_dv<128, QT>(p, grid, st); break;
  }
}

void dba_prefill_launch(const DBAParams& p0, int max_q_len, int num_seqs, hipStream_t st) {
  DBAParams p = p0;
  p.max_tiles = (max_q_len + PF_BM - 1) / PF_BM;
  const int qt = (p.heads / p.kv_heads) % 2 == 0 ? 2 : 1;   // two query heads of a kv head per workgroup where they pair up
  const int per_seq = (p.max_tiles * (p.heads / qt) + 7) / 8 * 8;      // a multiple of the XCD count: the numbering repeats per segment
  const dim3 grid((unsigned)per_seq, (unsigned)num_seqs);
  if (qt == 2) launch_prefill_dk<2>(p, grid, st);
  else launch_prefill_dk<1>(p, grid, st);
}

// lanes per key row: the smallest power of two that covers both row lengths in 16-byte pieces
static int decode_chl(int dim, int vdim) {
  const int pieces = (max(dim, vdim) + 7) / 8;
  int chl = 2;
  while ((1 << chl) < pieces) ++chl;
  return chl;
}

bool dba_decode_supported(int heads, int kv_heads, int dim, int vdim) {
  const int qh = heads / kv_heads, chl = decode_chl(dim, vdim);
  if ((dim & 7) || (vdim & 7) || chl > 5) return false;
  if (qh != 1 && qh != 2 && qh != 4 && qh != 8) return false;
  return qh * (1 << chl) <= 64;
}

void dba_decode_launch(const DBAParams& p, int64_t num_tokens, int nsplit, hipStream_t st) {
  const dim3 grid((unsigned)num_tokens, (unsigned)p.kv_heads, (unsigned)nsplit);
  const int qh = p.heads / p.kv_heads, chl = decode_chl(p.dim, p.vdim);
#define DEC(QH, CHL) hipLaunchKernelGGL((dba_decode_kernel<QH, CHL>), grid, dim3(256), 0, st, p)
#define DEC_BY_CHL(QH)                          \
  switch (chl) {                                \
    case 2: DEC(QH, 2); break;                  \
    case 3: DEC(QH, 3); break;                  \
    case 4: if (QH <= 4) DEC((QH <= 4 ? QH : 1), 4); break; \
    case 5: if (QH <= 2) DEC((QH <= 2 ? QH : 1), 5); break; \
  }
  switch (qh) {
    case 1: DEC_BY_CHL(1); break;
    case 2: DEC_BY_CHL(2); break;
    case 4: DEC_BY_CHL(4); break;
    case 8: DEC_BY_CHL(8); break;
  }
#undef DEC_BY_CHL
#undef DEC
  if (nsplit > 1)
    hipLaunchKernelGGL(dba_merge_kernel, dim3((unsigned)num_tokens, (unsigned)p.heads), dim3(64), 0, st, p, nsplit);
}

// Key splits of the decode kernel: enough workgroups to fill the chip, at least four 64-key tiles (one per wave) each.
int dba_decode_splits(int64_t num_tokens, int kv_heads, int max_kv_len, int64_t ws_floats, int heads, int vdim) {
  const int tiles = (max_kv_len + 63) / 64;
  int64_t n = (1024 + num_tokens * kv_heads - 1) / (num_tokens * kv_heads);
  if (n > tiles / 4) n = tiles / 4;
  if (n > 8) n = 8;
  while (n > 1 && num_tokens * heads * n * (2 + vdim) > ws_floats) --n;
  return n < 1 ? 1 : (int)n;
}

}  // namespace aphro
