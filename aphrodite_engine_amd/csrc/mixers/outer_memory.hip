// Gated outer-product memories: per (request slot, head) a matrix state S [dim, vdim] with
//     S <- a_t S + b_t k_t v_t^T,     o_t = S^T q_t   [ / normaliser ]
// scanned token by token over each segment of the batch -- prompt portions and single decoded tokens alike -- from the
// state an earlier step left in the slot (or from zero for a sequence's first tokens), and written back in place.
//   mode 0, decay linear attention: q, k, v through silu, a_t = a fixed per-head decay, b_t = 1.
//   mode 1, mLSTM: exponential input gate and sigmoid forget gate in log space under a running maximum m (which starts at
//   ZERO), a normaliser vector n that follows the same recurrence with k alone, and the guarded division of the output.
// State, gates, decays and the accumulation are fp32 whatever the activations' storage.
//
// Work split: a workgroup of 256 threads owns 64 (or, for prompt portions, 16) value columns of one (segment, head): thread
// = (column c, slice sl) with the key dimension cut into 4 (or 16) slices of DPT rows held in registers; q / k / v of 16 tokens at a time are staged in LDS with
// their activations applied (the next 16 tokens' raw values are already in flight in registers), the per-token partial dot products are folded over the slices with DPP moves.  The
// mLSTM gate recurrence of a 16-token stage runs in wave 0 (lane = token for the transcendental parts, a 16-step max-plus
// loop for m) before the stage is released to all waves.
#include "mixers_common.h"

namespace aphro {

constexpr int OMS_CH = 16;

template <typename T, int MODE, int DPT, int SLOG>
__global__ __launch_bounds__(256) void outer_memory_scan_kernel(
    float* __restrict__ out, const typename T::storage* __restrict__ q, int64_t q_stride,
    const typename T::storage* __restrict__ k, int64_t k_stride, const typename T::storage* __restrict__ v, int64_t v_stride,
    const typename T::storage* __restrict__ gate_i, const typename T::storage* __restrict__ gate_f, int64_t gate_stride,
    float* __restrict__ state_s, float* __restrict__ state_n, float* __restrict__ state_m,
    const int32_t* __restrict__ slot_of_seq, int num_slots, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ ctx_len, int heads, int dim, int vdim,
    const float* __restrict__ decay, float q_scale, float gate_cap) {
  constexpr int NS = 1 << SLOG;        // slices of the key dimension = lanes that share a column
  constexpr int TW = 256 >> SLOG;      // value columns per workgroup
  constexpr int DP = NS * DPT;
  __shared__ __attribute__((aligned(16))) float qs[OMS_CH][DP];
  __shared__ __attribute__((aligned(16))) float ks[OMS_CH][DP];
  __shared__ float vs[OMS_CH][TW];
  __shared__ float a_s[OMS_CH], b_s[OMS_CH], em_s[OMS_CH];
  const int s = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * TW;
  const int ncopy = (vdim + 15) >> 4, copy0 = c0 >> 4;          // n and m are kept once per 16 value columns
  const int tid = threadIdx.x, c = tid >> SLOG, sl = tid & (NS - 1), col = c0 + c;
  const int n = q_len[s];
  const int slot = slot_of_seq[s];
  if (n <= 0 || slot < 0 || slot >= num_slots) return;
  const int64_t t0 = q_start[s];
  const bool fresh = ctx_len[s] == 0;
  float S[DPT], nv[DPT];
  float m = 0.f;                                            // wave 0 only (uniform)
  float* sbase = state_s + ((int64_t)slot * heads + h) * dim * (int64_t)vdim;
  float* nbase = MODE == 1 ? state_n + (((int64_t)slot * heads + h) * ncopy + copy0) * dim : nullptr;
  float* mptr = MODE == 1 ? state_m + ((int64_t)slot * heads + h) * ncopy + copy0 : nullptr;
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int r = sl * DPT + i;
    S[i] = (!fresh && r < dim && col < vdim) ? sbase[(int64_t)r * vdim + col] : 0.f;
    nv[i] = (MODE == 1 && !fresh && r < dim) ? nbase[r] : 0.f;
  }
  if (MODE == 1 && !fresh) m = *mptr;
  const float dec = MODE == 0 ? decay[h] : 0.f;

  // raw q / k / v (and gates) of the next stage travel in registers while the current stage is scanned
  constexpr int NQ = (OMS_CH * DP + 255) / 256, NV = (OMS_CH * TW + 255) / 256;
  float rq[NQ], rk[NQ], rv[NV], rgi = 0.f, rgf = 0.f;
  auto fetch = [&](int base) {
    const int cnt = min(OMS_CH, n - base);
#pragma unroll
    for (int it = 0; it < NQ; ++it) {
      const int idx = tid + 256 * it, tt = idx / DP, r = idx % DP;
      rq[it] = rk[it] = 0.f;
      if (tt < cnt && r < dim) {
        rq[it] = T::to_f32(q[(t0 + base + tt) * q_stride + h * dim + r]);
        rk[it] = T::to_f32(k[(t0 + base + tt) * k_stride + h * dim + r]);
      }
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = tid + 256 * it, tt = idx / TW, cc = idx % TW;
      rv[it] = (tt < cnt && c0 + cc < vdim) ? T::to_f32(v[(t0 + base + tt) * v_stride + h * vdim + c0 + cc]) : 0.f;
    }
    if (MODE == 1 && tid < cnt) {
      rgi = T::to_f32(gate_i[(t0 + base + tid) * gate_stride + h]);
      rgf = T::to_f32(gate_f[(t0 + base + tid) * gate_stride + h]);
    }
  };
  fetch(0);
  for (int base = 0; base < n; base += OMS_CH) {
    const int cnt = min(OMS_CH, n - base);
    __syncthreads();                                        // the previous stage is consumed
#pragma unroll
    for (int it = 0; it < NQ; ++it) {
      const int idx = tid + 256 * it, tt = idx / DP, r = idx % DP;
      if (tt < OMS_CH) {
        qs[tt][r] = MODE == 0 ? silu_f(rq[it]) : rq[it] * q_scale;
        ks[tt][r] = MODE == 0 ? silu_f(rk[it]) : rk[it];
      }
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = tid + 256 * it;
      if (idx < OMS_CH * TW) vs[idx / TW][idx % TW] = MODE == 0 ? silu_f(rv[it]) : rv[it];
    }
    if (MODE == 1 && tid < 64) {
      float gi = 0.f, gf = 0.f;
      if (tid < cnt) {
        gi = gate_cap * tanhf(rgi / gate_cap);
        gf = log_sigmoid_f(gate_cap * tanhf(rgf / gate_cap));
      }
      float m_prev_mine = 0.f, m_mine = 0.f;
      for (int tt = 0; tt < cnt; ++tt) {
        const float f = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, gf), tt));
        const float ig = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, gi), tt));
        const float m_new = fmaxf(f + m, ig);
        if (tid == tt) {
          m_prev_mine = m;
          m_mine = m_new;
        }
        m = m_new;
      }
      if (tid < cnt) {
        a_s[tid] = expf(gf + m_prev_mine - m_mine);
        b_s[tid] = expf(gi - m_mine);
        em_s[tid] = expf(-m_mine);
      }
    }
    __syncthreads();
    if (base + OMS_CH < n) fetch(base + OMS_CH);
#pragma unroll 4
    for (int tt = 0; tt < cnt; ++tt) {
      const float a = MODE == 1 ? a_s[tt] : dec;
      const float b = MODE == 1 ? b_s[tt] : 1.0f;
      const float vv = vs[tt][c] * b;
      float part[4] = {0.f, 0.f, 0.f, 0.f}, npart[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i4 = 0; i4 < DPT; i4 += 4) {
        const f32x4 kk = *reinterpret_cast<const f32x4*>(&ks[tt][sl * DPT + i4]);
        const f32x4 qq = *reinterpret_cast<const f32x4*>(&qs[tt][sl * DPT + i4]);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          S[i4 + u] = a * S[i4 + u] + kk[u] * vv;
          part[u] += S[i4 + u] * qq[u];
          if (MODE == 1) {
            nv[i4 + u] = a * nv[i4 + u] + b * kk[u];
            npart[u] += nv[i4 + u] * qq[u];
          }
        }
      }
      float po = (part[0] + part[1]) + (part[2] + part[3]);
      po = group_sum<SLOG>(po);
      if (MODE == 1) {
        float pn = (npart[0] + npart[1]) + (npart[2] + npart[3]);
        pn = group_sum<SLOG>(pn);
        po = po / (fmaxf(fabsf(pn), em_s[tt]) + 1e-6f);
      }
      if (sl == 0 && col < vdim) out[(t0 + base + tt) * ((int64_t)heads * vdim) + h * vdim + col] = po;
    }
  }
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int r = sl * DPT + i;
    if (r < dim && col < vdim) sbase[(int64_t)r * vdim + col] = S[i];
    if (MODE == 1 && c == 0 && r < dim)
      for (int cp = 0; cp < TW / 16 && copy0 + cp < ncopy; ++cp) nbase[(int64_t)cp * dim + r] = nv[i];
  }
  if (MODE == 1 && tid == 0)
    for (int cp = 0; cp < TW / 16 && copy0 + cp < ncopy; ++cp) mptr[cp] = m;
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_outer_memory_scan(float* out, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                                       const void* v, int64_t v_stride, const void* gate_i, const void* gate_f,
                                       int64_t gate_stride, float* state_s, float* state_n, float* state_m,
                                       const int32_t* slot_of_seq, int num_slots, const int32_t* q_start, const int32_t* q_len,
                                       const int32_t* ctx_len, int num_seqs, int64_t num_tokens, int heads, int dim, int vdim,
                                       int mode, const float* decay, float q_scale, float gate_cap, int max_q_len, int dtype,
                                       void* stream) {
  if (num_tokens == 0 || num_seqs == 0) return APHRO_OK;
  APHRO_CHECK(out && q && k && v && state_s && slot_of_seq && q_start && q_len && ctx_len, "outer_memory_scan: null argument");
  APHRO_CHECK(mode == 0 || mode == 1, "outer_memory_scan: mode %d", mode);
  APHRO_CHECK(mode == 0 ? decay != nullptr : (gate_i && gate_f && state_n && state_m && gate_cap > 0.f && gate_stride >= heads),
              "outer_memory_scan: mode %d lacks its gate arguments", mode);
  APHRO_CHECK(heads > 0 && heads <= 65535 && dim > 0 && dim <= 256 && vdim > 0 && vdim <= 64 * 65535 && num_slots > 0 && num_seqs > 0,
              "outer_memory_scan: heads %d dim %d (<= 256) vdim %d", heads, dim, vdim);
  APHRO_CHECK(q_stride >= (int64_t)heads * dim && k_stride >= (int64_t)heads * dim && v_stride >= (int64_t)heads * vdim,
              "outer_memory_scan: row strides smaller than the rows");
  // Prompt portions: 16 lanes per value column (16 columns per workgroup), so that a long sequential scan spreads over four
  // times as many waves with a quarter of the work per token and lane.  Single tokens: 4 lanes per column (64 columns per
  // workgroup), whose state loads and stores come in 64-byte pieces.
  const bool wide = max_q_len >= 32;
  const int tw = wide ? 16 : 64;
  const dim3 grid((unsigned)num_seqs, (unsigned)heads, (unsigned)((vdim + tw - 1) / tw));
#define OMS_LAUNCH(MODE, DPT, SLOG)                                                                                         \
  hipLaunchKernelGGL((outer_memory_scan_kernel<T, MODE, DPT, SLOG>), grid, dim3(256), 0, (hipStream_t)stream, out, (const S*)q, \
                     q_stride, (const S*)k, k_stride, (const S*)v, v_stride, (const S*)gate_i, (const S*)gate_f, gate_stride, \
                     state_s, state_n, state_m, slot_of_seq, num_slots, q_start, q_len, ctx_len, heads, dim, vdim, decay,     \
                     q_scale, gate_cap)
#define OMS_BY_DIM(MODE)                               \
  do {                                                 \
    if (wide) {                                        \
      if (dim <= 64) OMS_LAUNCH(MODE, 4, 4);           \
      else if (dim <= 128) OMS_LAUNCH(MODE, 8, 4);     \
      else OMS_LAUNCH(MODE, 16, 4);                    \
    } else if (dim <= 32) OMS_LAUNCH(MODE, 8, 2);      \
    else if (dim <= 48) OMS_LAUNCH(MODE, 12, 2);       \
    else if (dim <= 64) OMS_LAUNCH(MODE, 16, 2);       \
    else if (dim <= 96) OMS_LAUNCH(MODE, 24, 2);       \
    else if (dim <= 128) OMS_LAUNCH(MODE, 32, 2);      \
    else OMS_LAUNCH(MODE, 64, 2);                      \
  } while (0)
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (mode == 0) OMS_BY_DIM(0);
    else OMS_BY_DIM(1);
  });
#undef OMS_BY_DIM
#undef OMS_LAUNCH
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
