// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// mLSTM: a recurrent mixer with a matrix memory per head (models/kafilorn.py).  Per head, with q, k [D],
// v [Dv] from the projections and the log gates i_t (input) and f_t (forget), all state in fp32:
//
//   m_t = max(f_t + m_(t-1), i_t)                      running maximum (starts at 0)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k v^T        [D, Dv], starts at 0
//   n_t = (the same two factors) n_(t-1) + ... k                         [D]
//   o_t = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)
//
// `mlstm_gates`: the two gate pre-activations per head from the layer input in fp32 (weights [2H, W] fp32,
// one wave per output), soft-capped by cap * tanh(. / cap) when cap > 0; the forget gate then through
// log-sigmoid.  `mlstm_scan`: the recurrence over the rows that each sequence brings to this step, from the
// state in the sequence's slot and back into it; a row at position 0 starts from the zero state, so a slot
// needs no clearing between requests.  The scalar chain (running maximum, the two factors of every row) runs
// once per (sequence, head) in a launch of its own; then one workgroup per (sequence, head, 16 value columns):
// a column is held by 16 lanes, each with D / 16 rows of S in registers; rows are staged 16 .. 64 at a time in LDS.
// The same launch serves a decode step (one row per sequence) and a prompt portion of any length; the
// arithmetic per token does not depend on how the rows were cut into steps.
#include "rows_f32.h"

namespace {
using namespace rows;

constexpr int VB = 16;   // value columns per workgroup
constexpr int DP = 16;   // lanes per column

template <typename AT>
__global__ __launch_bounds__(NT) void mlstm_gates_kernel(float* __restrict__ gates, const AT* __restrict__ h,
                                                         const float* __restrict__ w, const float* __restrict__ b,
                                                         int width, int H, float cap) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const AT* hr = h + (size_t)t * width;
  for (int j = wave; j < 2 * H; j += NW) {
    const float* wj = w + (size_t)j * width;
    float s = 0.f;
    for (int i = lane; i < width; i += 64) s += ldf(hr + i) * wj[i];
    s = wave_sum(s) + b[j];
    if (cap > 0.f) s = cap * tanhf(s / cap);
    if (j >= H) s = fminf(s, 0.f) - log1pf(expf(-fabsf(s)));   // log sigmoid
    if (lane == 0) gates[(size_t)t * 2 * H + j] = s;
  }
}

// bf16 on the matrix cores: 16 tokens per workgroup as the M rows, the 2H gate outputs as N (blocks of 16), the
// width split over the four waves and summed through LDS; the products of bf16 inputs are exact and accumulate
// in fp32, so this computes what the kernel above computes with fp32 copies of the same weights.
template <int NBLK>
__global__ __launch_bounds__(NT) void mlstm_gates_mfma_kernel(float* __restrict__ gates, const bf16_t* __restrict__ h,
                                                              const bf16_t* __restrict__ w, const float* __restrict__ b,
                                                              int T, int width, int H, float cap) {
  __shared__ float red[NW][16][NBLK * 16 + 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int t0 = blockIdx.x * 16, N = 2 * H;
  const bf16_t* hr = h + (size_t)min(t0 + col, T - 1) * width + 8 * grp;
  const bf16_t* wr[NBLK];
  f32x4 acc[NBLK];
#pragma unroll
  for (int nb = 0; nb < NBLK; ++nb) {
    wr[nb] = w + (size_t)min(nb * 16 + col, N - 1) * width + 8 * grp;
    acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int kper = width / NW, kbeg = wave * kper;
#pragma unroll 4
  for (int k0 = kbeg; k0 < kbeg + kper; k0 += 32) {
    const bf16x8 a = as_bf16x8(*reinterpret_cast<const uint4*>(hr + k0));
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb)
      acc[nb] = mfma16x16x32(a, as_bf16x8(*reinterpret_cast<const uint4*>(wr[nb] + k0)), acc[nb]);
  }
#pragma unroll
  for (int nb = 0; nb < NBLK; ++nb)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][4 * grp + r][nb * 16 + col] = acc[nb][r];
  __syncthreads();
  for (int idx = tid; idx < 16 * N; idx += NT) {
    const int r = idx / N, j = idx % N;
    if (t0 + r >= T) continue;
    float s = b[j];
#pragma unroll
    for (int wv = 0; wv < NW; ++wv) s += red[wv][r][j];
    if (cap > 0.f) s = cap * tanhf(s / cap);
    if (j >= H) s = fminf(s, 0.f) - log1pf(expf(-fabsf(s)));
    gates[(size_t)(t0 + r) * N + j] = s;
  }
}

struct ScanArgs {
  const int* q_starts;     // [num_seqs + 1] or null (row t is sequence t)
  const int* seq_slots;    // [num_seqs] state slot, < 0: skip
  const int* positions;    // [T]
  int ps, q_off, k_off, v_off;   // proj row stride and column offsets
  int H, D, Dv;
  float qscale;
  int vec;                 // q / k rows can be read in aligned 16-byte pieces
};

// The scalar part of the recurrence, once per (sequence, head) instead of in every workgroup of the state
// update: from the running maximum in the sequence's slot (0 for a fresh sequence) the factors of every row,
//   dec[t, h] = (exp(f + m_prev - m_new), exp(i - m_new), exp(-m_new)),
// and the new maximum back into the slot.  One thread per head; rows are read eight at a time.
__global__ __launch_bounds__(64) void mlstm_decay_kernel(float* __restrict__ dec, const float* __restrict__ gates,
                                                         float* __restrict__ st_m, ScanArgs a) {
  const int seq = blockIdx.x, h = blockIdx.y * 64 + threadIdx.x;
  const int slot = a.seq_slots[seq];
  if (slot < 0 || h >= a.H) return;
  const int r0 = a.q_starts ? a.q_starts[seq] : seq, r1 = a.q_starts ? a.q_starts[seq + 1] : seq + 1;
  if (r1 <= r0) return;
  const int H = a.H;
  float m = a.positions[r0] == 0 ? 0.f : st_m[(size_t)slot * H + h];
  for (int t0 = r0; t0 < r1; t0 += 8) {
    float ig[8], fg[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = min(t0 + u, r1 - 1);
      ig[u] = gates[(size_t)t * 2 * H + h];
      fg[u] = gates[(size_t)t * 2 * H + H + h];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (t0 + u < r1) {
        const float mn = fmaxf(fg[u] + m, ig[u]);
        float* d = dec + ((size_t)(t0 + u) * H + h) * 3;
        d[0] = expf(fg[u] + m - mn);
        d[1] = expf(ig[u] - mn);
        d[2] = expf(-mn);
        m = mn;
      }
    }
  }
  st_m[(size_t)slot * H + h] = m;
}

// state layout: S [slots, H, Dv, D] (a column's D entries are contiguous), n [slots, H, D], m [slots, H]
template <typename AT, int RPT>
__global__ __launch_bounds__(NT) void mlstm_scan_kernel(float* __restrict__ out, const AT* __restrict__ proj,
                                                        const float* __restrict__ dec, float* __restrict__ st_S,
                                                        float* __restrict__ st_n, ScanArgs a, int TB) {
  extern __shared__ float lds[];
  constexpr int Dp = DP * RPT;          // D padded
  float* qs = lds;                      // [TB][Dp]
  float* ks = qs + TB * Dp;             // [TB][Dp]
  float* vs = ks + TB * Dp;             // [TB][VB]
  float* df = vs + TB * VB;             // [TB][3] the row's factors (forget, input, exp(-maximum))
  const int seq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * VB;
  const int slot = a.seq_slots[seq];
  if (slot < 0) return;
  const int r0 = a.q_starts ? a.q_starts[seq] : seq, r1 = a.q_starts ? a.q_starts[seq + 1] : seq + 1;
  if (r1 <= r0) return;
  const int H = a.H, D = a.D, Dv = a.Dv;
  const int col = threadIdx.x / DP, dp = threadIdx.x % DP;
  const int v = v0 + col;
  const bool vok = v < Dv;
  float S[RPT], n[RPT];
  float* Sp = st_S + (((size_t)slot * H + h) * Dv + (vok ? v : 0)) * D;
  float* np = st_n + ((size_t)slot * H + h) * D;
  const bool fresh = a.positions[r0] == 0;
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int d = dp + DP * r;
    const bool ok = !fresh && d < D;
    S[r] = ok && vok ? Sp[d] : 0.f;
    n[r] = ok ? np[d] : 0.f;
  }
  if (a.vec)
    for (int idx = threadIdx.x; idx < 2 * TB * Dp; idx += NT) qs[idx] = 0.f;   // q and k tiles, pad entries included
  for (int t0 = r0; t0 < r1; t0 += TB) {
    const int nt = min(TB, r1 - t0);
    __syncthreads();
    if (a.vec) {
      // 16-byte pieces of the q and k rows, all requested before any is unpacked (the pad entries d >= D stay 0)
      constexpr int CE = 16 / (int)sizeof(AT), MAXIT = 8;
      const int cpr = D / CE, total = nt * cpr;
      uint4 rq[MAXIT], rk[MAXIT];
#pragma unroll
      for (int it = 0; it < MAXIT; ++it) {
        const int idx = threadIdx.x + it * NT;
        if (idx < total) {
          const AT* row = proj + (size_t)(t0 + idx / cpr) * a.ps + h * D + (idx % cpr) * CE;
          rq[it] = *reinterpret_cast<const uint4*>(row + a.q_off);
          rk[it] = *reinterpret_cast<const uint4*>(row + a.k_off);
        }
      }
#pragma unroll
      for (int it = 0; it < MAXIT; ++it) {
        const int idx = threadIdx.x + it * NT;
        if (idx < total) {
          float* qd = qs + (idx / cpr) * Dp + (idx % cpr) * CE;
          float* kd = ks + (idx / cpr) * Dp + (idx % cpr) * CE;
          const uint32_t wq[4] = {rq[it].x, rq[it].y, rq[it].z, rq[it].w}, wk[4] = {rk[it].x, rk[it].y, rk[it].z, rk[it].w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if constexpr (sizeof(AT) == 2) {
              qd[2 * i] = lo_f(wq[i]) * a.qscale;
              qd[2 * i + 1] = hi_f(wq[i]) * a.qscale;
              kd[2 * i] = lo_f(wk[i]);
              kd[2 * i + 1] = hi_f(wk[i]);
            } else {
              qd[i] = __uint_as_float(wq[i]) * a.qscale;
              kd[i] = __uint_as_float(wk[i]);
            }
          }
        }
      }
    } else {
      for (int idx = threadIdx.x; idx < nt * Dp; idx += NT) {
        const int tt = idx / Dp, d = idx % Dp;
        const AT* row = proj + (size_t)(t0 + tt) * a.ps;
        qs[idx] = d < D ? ldf(row + a.q_off + h * D + d) * a.qscale : 0.f;
        ks[idx] = d < D ? ldf(row + a.k_off + h * D + d) : 0.f;
      }
    }
    for (int idx = threadIdx.x; idx < nt * VB; idx += NT) {
      const int tt = idx / VB, c = idx % VB;
      vs[idx] = v0 + c < Dv ? ldf(proj + (size_t)(t0 + tt) * a.ps + a.v_off + h * Dv + v0 + c) : 0.f;
    }
    for (int idx = threadIdx.x; idx < nt * 3; idx += NT) df[idx] = dec[((size_t)(t0 + idx / 3) * H + h) * 3 + idx % 3];
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float fa = df[tt * 3], ia = df[tt * 3 + 1];
      const float vv = vs[tt * VB + col] * ia;
      float pq = 0.f, pn = 0.f;
#pragma unroll
      for (int r = 0; r < RPT; ++r) {
        const float kd = ks[tt * Dp + dp + DP * r], qd = qs[tt * Dp + dp + DP * r];
        S[r] = fa * S[r] + kd * vv;
        n[r] = fa * n[r] + ia * kd;
        pq += S[r] * qd;
        pn += n[r] * qd;
      }
      pq = row16_sum(pq);
      pn = row16_sum(pn);
      if (dp == 0 && vok) out[((size_t)(t0 + tt) * H + h) * Dv + v] = pq / (fmaxf(fabsf(pn), df[tt * 3 + 2]) + 1e-6f);
    }
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    const int d = dp + DP * r;
    if (d < D) {
      if (vok) Sp[d] = S[r];
      if (blockIdx.z == 0 && col == 0) np[d] = n[r];
    }
  }
}

template <typename AT, int RPT>
int launch_scan(float* out, const AT* proj, const float* dec, float* S, float* n, const ScanArgs& a, int num_seqs,
                hipStream_t st) {
  // rows staged per tile: as many as 32 KB of q and k allow, 16 .. 64
  int TB = 4096 / (DP * RPT);
  TB = TB < 16 ? 16 : (TB > 64 ? 64 : TB);
  const size_t lds = (size_t)(2 * TB * DP * RPT + TB * VB + 3 * TB) * sizeof(float);
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mlstm_scan_kernel<AT, RPT>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  dim3 grid(num_seqs, a.H, (a.Dv + VB - 1) / VB);
  mlstm_scan_kernel<AT, RPT><<<grid, NT, lds, st>>>(out, proj, dec, S, n, a, TB);
  KA_CHECK_LAUNCH();
}

template <typename AT>
int dispatch_scan(float* out, const AT* proj, const float* dec, float* S, float* n, const ScanArgs& a, int num_seqs,
                  hipStream_t st) {
  const int need = (a.D + DP - 1) / DP;
  if (need <= 1) return launch_scan<AT, 1>(out, proj, dec, S, n, a, num_seqs, st);
  if (need <= 2) return launch_scan<AT, 2>(out, proj, dec, S, n, a, num_seqs, st);
  if (need <= 4) return launch_scan<AT, 4>(out, proj, dec, S, n, a, num_seqs, st);
  if (need <= 8) return launch_scan<AT, 8>(out, proj, dec, S, n, a, num_seqs, st);
  if (need <= 16) return launch_scan<AT, 16>(out, proj, dec, S, n, a, num_seqs, st);
  if (need <= 32) return launch_scan<AT, 32>(out, proj, dec, S, n, a, num_seqs, st);
  return (int)hipErrorInvalidValue;
}

}  // namespace

extern "C" int ka_mlstm_gates(float* gates, const void* h, const float* w, const float* b, int T, int width, int H,
                              float cap, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (f32) mlstm_gates_kernel<float><<<T, NT, 0, st>>>(gates, (const float*)h, w, b, width, H, cap);
  else mlstm_gates_kernel<bf16_t><<<T, NT, 0, st>>>(gates, (const bf16_t*)h, w, b, width, H, cap);
  KA_CHECK_LAUNCH();
}

// dec: scratch [T, H, 3] fp32 (the rows' factors, written by the first launch and read by the second)
extern "C" int ka_mlstm_scan(float* out, const void* proj, int ps, int q_off, int k_off, int v_off, const float* gates,
                             float* dec, float* st_S, float* st_n, float* st_m, const int* seq_slots, const int* q_starts,
                             int num_seqs, const int* positions, int H, int D, int Dv, float qscale, int f32,
                             hipStream_t st) {
  if (num_seqs <= 0) return 0;
  if (H <= 0 || D <= 0 || Dv <= 0 || H > 65535) return (int)hipErrorInvalidValue;
  const int ce = f32 ? 4 : 8;
  const int need = (D + DP - 1) / DP;
  const int rpt = need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : need <= 8 ? 8 : need <= 16 ? 16 : 32;
  int tb = 4096 / (DP * rpt);
  tb = tb < 16 ? 16 : (tb > 64 ? 64 : tb);
  const int vec = D % ce == 0 && ps % ce == 0 && q_off % ce == 0 && k_off % ce == 0 &&
                  ((uintptr_t)proj & 15) == 0 && tb * (D / ce) <= 8 * NT;
  ScanArgs a{q_starts, seq_slots, positions, ps, q_off, k_off, v_off, H, D, Dv, qscale, vec};
  mlstm_decay_kernel<<<dim3(num_seqs, (H + 63) / 64), 64, 0, st>>>(dec, gates, st_m, a);
  if (f32) return dispatch_scan<float>(out, (const float*)proj, dec, st_S, st_n, a, num_seqs, st);
  return dispatch_scan<bf16_t>(out, (const bf16_t*)proj, dec, st_S, st_n, a, num_seqs, st);
}

// bf16 activations with a bf16 copy of the gate weights [2H, width]; width a multiple of 128, 2H <= 128
extern "C" int ka_mlstm_gates_mfma(float* gates, const void* h, const void* w, const float* b, int T, int width, int H,
                                   float cap, hipStream_t st) {
  if (T <= 0) return 0;
  if (width % 128 || H <= 0 || 2 * H > 128) return (int)hipErrorInvalidValue;
  const int grid = (T + 15) / 16, nblk = (2 * H + 15) / 16;
#define KA_G(NBLK) mlstm_gates_mfma_kernel<NBLK><<<grid, NT, 0, st>>>(gates, (const bf16_t*)h, (const bf16_t*)w, b, T, width, H, cap)
  if (nblk <= 1) KA_G(1);
  else if (nblk <= 2) KA_G(2);
  else if (nblk <= 4) KA_G(4);
  else KA_G(8);
#undef KA_G
  KA_CHECK_LAUNCH();
}
