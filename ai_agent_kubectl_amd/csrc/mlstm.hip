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
// needs no clearing between requests.  The scalar chain (running maximum, the rows' factors) runs once per
// (sequence, head) in a launch of its own; the state update follows (below).
// The same launch serves a decode step (one row per sequence) and a prompt portion of any length; the
// arithmetic per token does not depend on how the rows were cut into steps.
#include "rows_f32.h"

namespace {
using namespace rows;


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
#pragma unroll 8
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

// The scalar chain, once per (sequence, head) in a launch of its own: a wave takes 64 rows at a time, every lane
// loads its row's gates, the chain m_t = max(f_t + m_(t-1), i_t) runs over the 64 rows on lane-broadcast values
// (two operations a row, the same expression and order as a row-by-row decode, so the factors do not depend on how
// a prompt was cut), and every lane then forms its own row's
//   dec[t, h] = (exp(f + m_prev - m), exp(i - m), exp(-m))
// in parallel; the maximum goes from / to the sequence's slot (0 for a fresh sequence).
__global__ __launch_bounds__(64) void mlstm_decay_kernel(float* __restrict__ dec, const float* __restrict__ gates,
                                                         float* __restrict__ st_m, ScanArgs a) {
  const int seq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int slot = a.seq_slots[seq];
  if (slot < 0) return;
  const int r0 = a.q_starts ? a.q_starts[seq] : seq, r1 = a.q_starts ? a.q_starts[seq + 1] : seq + 1;
  if (r1 <= r0) return;
  const int H = a.H;
  float m = a.positions[r0] == 0 ? 0.f : st_m[(size_t)slot * H + h];   // the maximum before the block (the same in every lane)
  for (int t0 = r0; t0 < r1; t0 += 64) {
    const int t = t0 + lane;
    const bool ok = t < r1;
    const float ig = ok ? gates[(size_t)t * 2 * H + h] : -INFINITY;   // a row past the end leaves the maximum as it is
    const float fg = ok ? gates[(size_t)t * 2 * H + H + h] : 0.f;
    float mp = 0.f, mt = 0.f;
    const int nrow = min(64, r1 - t0);
    for (int j = 0; j < nrow; ++j) {
      const float fj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, fg), j));
      const float ij = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ig), j));
      const float prev = m;
      m = fmaxf(fj + m, ij);
      if (lane == j) {
        mp = prev;
        mt = m;
      }
    }
    if (ok) {
      float* d = dec + ((size_t)t * H + h) * 3;
      d[0] = expf(fg + mp - mt);
      d[1] = expf(ig - mt);
      d[2] = expf(-mt);
    }
  }
  if (lane == 0) st_m[(size_t)slot * H + h] = m;
}

// rows t0 .. t0 + nt of head h: q (scaled) and k as fp32 into LDS tiles [nt][Dp] (pad entries d >= D are not written)
template <typename AT>
KA_DEV void stage_qk(float* qs, float* ks, int Dp, const AT* __restrict__ proj, const ScanArgs& a, int h, int t0, int nt) {
  const int D = a.D;
  if (a.vec) {   // 16-byte pieces, all requested before any is unpacked
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
    for (int idx = threadIdx.x; idx < nt * D; idx += NT) {
      const int tt = idx / D, d = idx % D;
      const AT* row = proj + (size_t)(t0 + tt) * a.ps + h * D + d;
      qs[tt * Dp + d] = ldf(row + a.q_off) * a.qscale;
      ks[tt * Dp + d] = ldf(row + a.k_off);
    }
  }
}

// The state update and read-out.  S [slots, H, Dv, D] (a column's D entries contiguous), n [slots, H, D].
// The normaliser n obeys the same update as a column of S whose value is 1, and n . q is that column's
// read-out: the columns of a head are numbered c = 0 .. Dv with c = 0 the normaliser and c >= 1 the value column
// c - 1.  A column is held by DPL adjacent lanes, each with RPT consecutive entries in registers (the q and k
// rows come from LDS as broadcast 16-byte pieces); a workgroup takes (sequence, head, 256 / DPL columns).  The
// numerators go to `out`, the denominators max(|n . q|, exp(-m)) + 1e-6 to `den` [T, H]; the division is the
// first step of the head norm that follows.
template <typename AT, int RPT, int DPL>
__global__ __launch_bounds__(NT) void mlstm_scan_kernel(float* __restrict__ out, float* __restrict__ den,
                                                        const AT* __restrict__ proj, const float* __restrict__ dec,
                                                        float* __restrict__ st_S, float* __restrict__ st_n, ScanArgs a,
                                                        int TB) {
  extern __shared__ float lds[];
  constexpr int Dp = DPL * RPT, CW = NT / DPL;   // D padded; columns per workgroup
  float* qs = lds;                      // [TB][Dp]
  float* ks = qs + TB * Dp;             // [TB][Dp]
  float* vs = ks + TB * Dp;             // [TB][CW]
  float* df = vs + TB * CW;             // [TB][3] the row's factors (forget, input, exp(-maximum))
  const int seq = blockIdx.x, h = blockIdx.y;
  const int slot = a.seq_slots[seq];
  if (slot < 0) return;
  const int r0 = a.q_starts ? a.q_starts[seq] : seq, r1 = a.q_starts ? a.q_starts[seq + 1] : seq + 1;
  if (r1 <= r0) return;
  const int H = a.H, D = a.D, Dv = a.Dv;
  const int col = threadIdx.x / DPL, dp = threadIdx.x % DPL;
  const int c = blockIdx.z * CW + col;            // 0: the normaliser, else value column c - 1
  const bool cok = c <= Dv;
  float* Sp = c == 0 ? st_n + ((size_t)slot * H + h) * D : st_S + (((size_t)slot * H + h) * Dv + (cok ? c - 1 : 0)) * D;
  const bool fresh = a.positions[r0] == 0;
  float S[RPT];
  const bool whole = cok && (dp + 1) * RPT <= D && (D & 3) == 0;   // this lane's entries in aligned 16-byte pieces
#pragma unroll
  for (int u = 0; u < RPT / 4; ++u) {
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
    if (!fresh) {
      if (whole) {
        x = *reinterpret_cast<const f32x4*>(Sp + dp * RPT + 4 * u);
      } else if (cok) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (dp * RPT + 4 * u + i < D) x[i] = Sp[dp * RPT + 4 * u + i];
      }
    }
    S[4 * u] = x[0];
    S[4 * u + 1] = x[1];
    S[4 * u + 2] = x[2];
    S[4 * u + 3] = x[3];
  }
  if (Dp != D)
    for (int idx = threadIdx.x; idx < 2 * TB * Dp; idx += NT) qs[idx] = 0.f;   // q and k tiles, pad entries included
  const int c0 = blockIdx.z * CW;
  for (int t0 = r0; t0 < r1; t0 += TB) {
    const int nt = min(TB, r1 - t0);
    __syncthreads();
    stage_qk(qs, ks, Dp, proj, a, h, t0, nt);
    for (int idx = threadIdx.x; idx < nt * CW; idx += NT) {
      const int tt = idx / CW, cc = c0 + idx % CW;
      vs[idx] = cc == 0 ? 1.f : (cc <= Dv ? ldf(proj + (size_t)(t0 + tt) * a.ps + a.v_off + h * Dv + cc - 1) : 0.f);
    }
    for (int idx = threadIdx.x; idx < nt * 3; idx += NT) df[idx] = dec[((size_t)(t0 + idx / 3) * H + h) * 3 + idx % 3];
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float fa = df[tt * 3];
      const float vv = vs[tt * CW + col] * df[tt * 3 + 1];
      const f32x4* k4 = reinterpret_cast<const f32x4*>(ks + tt * Dp + dp * RPT);
      const f32x4* q4 = reinterpret_cast<const f32x4*>(qs + tt * Dp + dp * RPT);
      float p0 = 0.f, p1 = 0.f;
#pragma unroll
      for (int u = 0; u < RPT / 4; ++u) {
        const f32x4 kc = k4[u], qc = q4[u];
        S[4 * u] = fa * S[4 * u] + kc[0] * vv;
        S[4 * u + 1] = fa * S[4 * u + 1] + kc[1] * vv;
        S[4 * u + 2] = fa * S[4 * u + 2] + kc[2] * vv;
        S[4 * u + 3] = fa * S[4 * u + 3] + kc[3] * vv;
        p0 += S[4 * u] * qc[0] + S[4 * u + 2] * qc[2];
        p1 += S[4 * u + 1] * qc[1] + S[4 * u + 3] * qc[3];
      }
      float pq = p0 + p1;
      if constexpr (DPL == 4) {
        pq += dpp_f<0xB1>(pq);
        pq += dpp_f<0x4E>(pq);
      } else {
        pq = row16_sum(pq);
      }
      if (dp == 0 && cok) {
        if (c == 0) den[(size_t)(t0 + tt) * H + h] = fmaxf(fabsf(pq), df[tt * 3 + 2]) + 1e-6f;
        else out[((size_t)(t0 + tt) * H + h) * Dv + c - 1] = pq;
      }
    }
  }
  if (whole) {
#pragma unroll
    for (int u = 0; u < RPT / 4; ++u)
      *reinterpret_cast<f32x4*>(Sp + dp * RPT + 4 * u) = f32x4{S[4 * u], S[4 * u + 1], S[4 * u + 2], S[4 * u + 3]};
  } else if (cok) {
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
      const int d = dp * RPT + r;
      if (d < D) Sp[d] = S[r];
    }
  }
}

template <typename AT, int RPT, int DPL>
int launch_scan(float* out, float* den, const AT* proj, const float* dec, float* S, float* n, ScanArgs a, int num_seqs,
                hipStream_t st) {
  constexpr int Dp = RPT * DPL, CW = NT / DPL;
  int TB = 4096 / Dp;   // rows staged per tile: as many as 32 KB of q and k allow, 16 .. 64
  TB = TB < 16 ? 16 : (TB > 64 ? 64 : TB);
  const int ce = 16 / (int)sizeof(AT);
  a.vec = a.D % ce == 0 && a.ps % ce == 0 && a.q_off % ce == 0 && a.k_off % ce == 0 && ((uintptr_t)proj & 15) == 0 &&
          TB * (a.D / ce) <= 8 * NT;
  const size_t lds = (size_t)(2 * TB * Dp + TB * CW + 3 * TB) * sizeof(float);
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mlstm_scan_kernel<AT, RPT, DPL>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  dim3 grid(num_seqs, a.H, (a.Dv + 1 + CW - 1) / CW);
  mlstm_scan_kernel<AT, RPT, DPL><<<grid, NT, lds, st>>>(out, den, proj, dec, S, n, a, TB);
  KA_CHECK_LAUNCH();
}

template <typename AT>
int dispatch_scan(float* out, float* den, const AT* proj, const float* gates, float* dec, float* S, float* n, float* m,
                  const ScanArgs& a, int num_seqs, hipStream_t st) {
  mlstm_decay_kernel<<<dim3(num_seqs, a.H), 64, 0, st>>>(dec, gates, m, a);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  const int D = a.D;
  if (D <= 16) return launch_scan<AT, 4, 4>(out, den, proj, dec, S, n, a, num_seqs, st);
  if (D <= 32) return launch_scan<AT, 8, 4>(out, den, proj, dec, S, n, a, num_seqs, st);
  if (D <= 64) return launch_scan<AT, 16, 4>(out, den, proj, dec, S, n, a, num_seqs, st);
  if (D <= 128) return launch_scan<AT, 32, 4>(out, den, proj, dec, S, n, a, num_seqs, st);
  if (D <= 256) return launch_scan<AT, 64, 4>(out, den, proj, dec, S, n, a, num_seqs, st);
  return launch_scan<AT, 32, 16>(out, den, proj, dec, S, n, a, num_seqs, st);
}

}  // namespace

extern "C" int ka_mlstm_gates(float* gates, const void* h, const float* w, const float* b, int T, int width, int H,
                              float cap, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (f32) mlstm_gates_kernel<float><<<T, NT, 0, st>>>(gates, (const float*)h, w, b, width, H, cap);
  else mlstm_gates_kernel<bf16_t><<<T, NT, 0, st>>>(gates, (const bf16_t*)h, w, b, width, H, cap);
  KA_CHECK_LAUNCH();
}

// out [T, H * Dv]: the numerators; den [T, H]: the denominators; dec: scratch [T, H, 3] fp32 (the rows' factors,
// written by the first launch and read by the second)
extern "C" int ka_mlstm_scan(float* out, float* den, const void* proj, int ps, int q_off, int k_off, int v_off,
                             const float* gates, float* dec, float* st_S, float* st_n, float* st_m, const int* seq_slots,
                             const int* q_starts, int num_seqs, const int* positions, int H, int D, int Dv, float qscale,
                             int f32, hipStream_t st) {
  if (num_seqs <= 0) return 0;
  if (H <= 0 || D <= 0 || D > 512 || Dv <= 0 || H > 65535) return (int)hipErrorInvalidValue;
  ScanArgs a{q_starts, seq_slots, positions, ps, q_off, k_off, v_off, H, D, Dv, qscale, 0};
  if (f32) return dispatch_scan<float>(out, den, (const float*)proj, gates, dec, st_S, st_n, st_m, a, num_seqs, st);
  return dispatch_scan<bf16_t>(out, den, (const bf16_t*)proj, gates, dec, st_S, st_n, st_m, a, num_seqs, st);
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
