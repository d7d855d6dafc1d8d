// bf16 fast paths of the distance-biased attention (same semantics as biased_attention.hip, which stays the fp32 path and
// the path of sizes these do not tile):
//
//  * dba_prefill_kernel<DK, DV>: segments of >= DBA_MFMA_MIN_LEN rows.  A workgroup of four waves owns 64 consecutive
//    query rows of one (segment, head), 16 rows per wave, and walks the visible keys 32 at a time: the K rows and V rows of
//    the tile come from the paged cache with 16-byte loads into LDS (K chunk-swizzled, V transposed), together with the 95
//    bias values the tile can need (the table is indexed by distance, and a 64 x 32 tile spans 95 distances).
//    S^T = K Q^T on v_mfma_f32_16x16x32_bf16, so that the probabilities come out in the B-operand layout of O^T = V^T P^T
//    (keys of the two 16-key halves interleaved per lane group, V fragments read in the same order); temperature, bias,
//    mask and the online softmax are fp32 on the accumulator registers.
//  * dba_decode_kernel<QH, CHL>: the other rows (single decoded tokens, short portions), one workgroup per (row, kv head)
//    serving all QH query heads of that kv head from one pass over the keys.  A key row is read by 2^CHL lanes x 16 bytes,
//    64 / 2^CHL keys per load instruction (fully coalesced); the partial dot products fold over the lanes of a key with
//    DPP shuffles; scores and probabilities stay in that layout (16 keys x QH per lane), which is also the layout the V
//    pass wants, so nothing is redistributed.  Four waves split the 64-key tiles; partial (max, sum, acc) merge in LDS.
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
};

__device__ __forceinline__ float dba_temp(const DBAParams& p, int pos) {
  return p.temp_coef != 0.f ? 1.0f + p.temp_coef * logf((float)((pos + 1) / p.temp_every + 1)) : 1.0f;
}

constexpr int PF_BM = 64, PF_BN = 32, PF_VT = 36;

template <int DK, int DV>
__global__ __launch_bounds__(256) void dba_prefill_kernel(DBAParams p) {
  constexpr int NCHK = DK / 8, NCHV = DV / 8, NKS = DK / 32, NDT = DV / 16;
  constexpr int SWZ = (NCHK & -NCHK) - 1;
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[PF_BN * DK];
  __shared__ __attribute__((aligned(16))) uint16_t vt_lds[DV * PF_VT];
  __shared__ float bias_win[96];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int len = p.q_len[seq];
  if (len < p.min_len) return;
  const int ntiles = (len + PF_BM - 1) / PF_BM;
  const int tile = ntiles - 1 - (int)blockIdx.x;           // the longest key ranges first
  if (tile < 0) return;
  const int ctx = p.ctx_len[seq], s0 = p.q_start[seq];
  const int kvh = head / (p.heads / p.kv_heads);
  const int q0 = tile * PF_BM;
  const int qrow = q0 + 16 * wave + c;
  const bool qvalid = qrow < len;
  const int qpos = ctx + qrow;
  const float qs = p.scale * dba_temp(p, qpos);
  u32x4 qf[NKS];
  {
    const uint16_t* qp = p.q + (int64_t)(s0 + min(qrow, len - 1)) * p.q_stride + head * DK;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qf[ks] = *reinterpret_cast<const u32x4*>(qp + 32 * ks + 8 * g);
  }
  f32x4 o[NDT];
#pragma unroll
  for (int i = 0; i < NDT; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -1e30f, l_run = 0.f;
  const int32_t* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  const float* lut = p.bias_lut ? p.bias_lut + (int64_t)head * p.lut_len : nullptr;
  const int nk = ctx + min(len, q0 + PF_BM);               // keys the tile's last row sees
  const int64_t krow = (int64_t)p.kv_heads * DK, vrow = (int64_t)p.kv_heads * DV;

  for (int t0 = 0; t0 < nk; t0 += PF_BN) {
    __syncthreads();
    for (int i = threadIdx.x; i < PF_BN * NCHK; i += 256) {
      const int tok = i / NCHK, ch = i % NCHK;
      const int key = min(t0 + tok, nk - 1);
      int blk = bt[key / p.block_size];
      if (blk < 0 || blk >= p.num_blocks) blk = 0;
      const u16x8 kk = *reinterpret_cast<const u16x8*>(p.k_cache + ((int64_t)blk * p.block_size + key % p.block_size) * krow +
                                                       kvh * DK + 8 * ch);
      *reinterpret_cast<u16x8*>(&k_lds[tok * DK + 8 * (ch ^ (tok & SWZ))]) = kk;
    }
    for (int i = threadIdx.x; i < PF_BN * NCHV; i += 256) {
      const int tok = i / NCHV, ch = i % NCHV;
      const int key = min(t0 + tok, nk - 1);
      int blk = bt[key / p.block_size];
      if (blk < 0 || blk >= p.num_blocks) blk = 0;
      u16x8 vv = *reinterpret_cast<const u16x8*>(p.v_cache + ((int64_t)blk * p.block_size + key % p.block_size) * vrow +
                                                 kvh * DV + 8 * ch);
      if (t0 + tok >= nk) vv = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) vt_lds[(8 * ch + j) * PF_VT + tok] = vv[j];
    }
    const int dmin = ctx + q0 - t0 - (PF_BN - 1);           // distance of (first row, last key of the tile)
    if (threadIdx.x < 95) {
      float b = 0.f;
      if (lut) {
        const int dist = dmin + (int)threadIdx.x;
        b = lut[dist < 0 ? 0 : (dist < p.lut_len ? dist : p.lut_len - 1)];
      }
      bias_win[threadIdx.x] = b;
    }
    __syncthreads();
    if (t0 > ctx + q0 + 16 * wave + 15) continue;           // every key of the tile is ahead of the wave's rows
    f32x4 s[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      s[h] = f32x4{0.f, 0.f, 0.f, 0.f};
      const int tok = 16 * h + c;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int ch = (4 * ks + g) ^ (tok & SWZ);
        const u32x4 kf = *reinterpret_cast<const u32x4*>(&k_lds[tok * DK + 8 * ch]);
        s[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[ks]), s[h], 0, 0, 0);
      }
    }
    float pv[2][4];
    float mx = -1e30f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = t0 + 16 * h + 4 * g + r;
        float xv = s[h][r] * qs + bias_win[qpos - key - dmin];
        xv = key <= qpos ? xv : -1e30f;
        pv[h][r] = xv;
        mx = fmaxf(mx, xv);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __expf(m_run - m_new);
    m_run = m_new;
    float lsum = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float e = pv[h][r] > -1e29f ? __expf(pv[h][r] - m_new) : 0.f;
        pv[h][r] = e;
        lsum += e;
      }
    l_run = l_run * alpha + lsum;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[dt] *= alpha;
    const u32x4 pf = {pack2_16<true>(pv[0][0], pv[0][1]), pack2_16<true>(pv[0][2], pv[0][3]), pack2_16<true>(pv[1][0], pv[1][1]),
                      pack2_16<true>(pv[1][2], pv[1][3])};
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const uint16_t* vr = &vt_lds[(16 * dt + c) * PF_VT + 4 * g];
      const u32x2 lo = *reinterpret_cast<const u32x2*>(vr);
      const u32x2 hi = *reinterpret_cast<const u32x2*>(vr + 16);
      const u32x4 vf = {lo[0], lo[1], hi[0], hi[1]};
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf), __builtin_bit_cast(bf16x8, pf), o[dt], 0, 0, 0);
    }
  }
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if (!qvalid) return;
  float f = (l_run > 0.f ? 1.f / l_run : 0.f) * p.out_scale;
  if (p.gate) f *= sigmoid_f(BFloat::to_f32(p.gate[(int64_t)(s0 + qrow) * p.gate_stride + head]));
  uint16_t* op = p.out + (int64_t)(s0 + qrow) * p.out_stride + head * DV;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) op[16 * dt + 4 * g + r] = BFloat::from_f32(o[dt][r] * f);
  }
}

template <int QH, int CHL>
__global__ __launch_bounds__(256) void dba_decode_kernel(DBAParams p) {
  constexpr int CH = 1 << CHL;       // lanes per key row (16 bytes each)
  constexpr int KP = 64 / CH;        // keys per load instruction
  constexpr int NI = CH;             // load instructions per 64-key tile
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
  const int ntiles = (nkeys + 63) >> 6;
  for (int tile = wave; tile < ntiles; tile += 4) {
    float sc[NI][QH];
    int64_t voff[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int key = tile * 64 + i * KP + kg;
      const bool valid = key < nkeys;
      int blk = valid ? bt[key / p.block_size] : 0;
      if (blk < 0 || blk >= p.num_blocks) blk = 0;
      const int64_t slot = (int64_t)blk * p.block_size + (valid ? key % p.block_size : 0);
      voff[i] = slot * vrow + kvh * p.vdim + 8 * ck;
      u16x8 kk = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (valid && kin) kk = *reinterpret_cast<const u16x8*>(p.k_cache + slot * krow + kvh * p.dim + 8 * ck);
      float kf[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) kf[j] = BFloat::to_f32(kk[j]);
      const int dist = pos - key;
#pragma unroll
      for (int qh = 0; qh < QH; ++qh) {
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) d += qv[qh][j] * kf[j];
#pragma unroll
        for (int o = 1; o < CH; o <<= 1) d += __shfl_xor(d, o, 64);
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
      const float m_new = fmaxf(m[qh], mx);                // finite: key tile*64 exists
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
      const int key = tile * 64 + i * KP + kg;
      u16x8 vv = u16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (key < nkeys && vin) vv = *reinterpret_cast<const u16x8*>(p.v_cache + voff[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float vf = BFloat::to_f32(vv[j]);
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
    float sig = p.out_scale;
    if (p.gate) sig *= sigmoid_f(BFloat::to_f32(p.gate[(int64_t)t * p.gate_stride + head]));
    p.out[(int64_t)t * p.out_stride + head * p.vdim + col] = BFloat::from_f32(o * sig / L);
  }
}

template <int DK>
static bool launch_prefill_dv(const DBAParams& p, dim3 grid, hipStream_t st) {
  switch (p.vdim) {
    case 32: hipLaunchKernelGGL((dba_prefill_kernel<DK, 32>), grid, dim3(256), 0, st, p); return true;
    case 64: hipLaunchKernelGGL((dba_prefill_kernel<DK, 64>), grid, dim3(256), 0, st, p); return true;
    case 96: hipLaunchKernelGGL((dba_prefill_kernel<DK, 96>), grid, dim3(256), 0, st, p); return true;
    case 128: hipLaunchKernelGGL((dba_prefill_kernel<DK, 128>), grid, dim3(256), 0, st, p); return true;
  }
  return false;
}

bool dba_prefill_supported(int dim, int vdim) {
  auto ok = [](int d) { return d == 32 || d == 64 || d == 96 || d == 128; };
  return ok(dim) && ok(vdim);
}

void dba_prefill_launch(const DBAParams& p, int max_q_len, int num_seqs, hipStream_t st) {
  const dim3 grid((unsigned)((max_q_len + PF_BM - 1) / PF_BM), (unsigned)p.heads, (unsigned)num_seqs);
  switch (p.dim) {
    case 32: launch_prefill_dv<32>(p, grid, st); break;
    case 64: launch_prefill_dv<64>(p, grid, st); break;
    case 96: launch_prefill_dv<96>(p, grid, st); break;
    case 128: launch_prefill_dv<128>(p, grid, st); break;
  }
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

void dba_decode_launch(const DBAParams& p, int64_t num_tokens, hipStream_t st) {
  const dim3 grid((unsigned)num_tokens, (unsigned)p.kv_heads);
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
}

}  // namespace aphro
