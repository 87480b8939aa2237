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
// needs no clearing between requests.  One workgroup per (sequence, head, 16 value columns); a column is
// held by 16 lanes, each with D / 16 rows of S in registers; rows are staged 16 tokens at a time in LDS.
// The same launch serves a decode step (one row per sequence) and a prompt portion of any length; the
// arithmetic per token does not depend on how the rows were cut into steps.
#include "rows_f32.h"

namespace {
using namespace rows;

constexpr int VB = 16;   // value columns per workgroup
constexpr int DP = 16;   // lanes per column
constexpr int TB = 16;   // tokens staged per tile

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

struct ScanArgs {
  const int* q_starts;     // [num_seqs + 1] or null (row t is sequence t)
  const int* seq_slots;    // [num_seqs] state slot, < 0: skip
  const int* positions;    // [T]
  int ps, q_off, k_off, v_off;   // proj row stride and column offsets
  int H, D, Dv;
  float qscale;
};

// state layout: S [slots, H, Dv, D] (a column's D entries are contiguous), n [slots, H, D], m [slots, H]
template <typename AT, int RPT>
__global__ __launch_bounds__(NT) void mlstm_scan_kernel(float* __restrict__ out, const AT* __restrict__ proj,
                                                        const float* __restrict__ gates, float* __restrict__ st_S,
                                                        float* __restrict__ st_n, float* __restrict__ st_m, ScanArgs a) {
  extern __shared__ float lds[];
  constexpr int Dp = DP * RPT;          // D padded
  float* qs = lds;                      // [TB][Dp]
  float* ks = qs + TB * Dp;             // [TB][Dp]
  float* vs = ks + TB * Dp;             // [TB][VB]
  float* gi = vs + TB * VB;             // [TB]
  float* gf = gi + TB;                  // [TB]
  const int seq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * VB;
  const int slot = a.seq_slots[seq];
  if (slot < 0) return;
  const int r0 = a.q_starts ? a.q_starts[seq] : seq, r1 = a.q_starts ? a.q_starts[seq + 1] : seq + 1;
  if (r1 <= r0) return;
  const int H = a.H, D = a.D, Dv = a.Dv;
  const int col = threadIdx.x / DP, dp = threadIdx.x % DP;
  const int v = v0 + col;
  const bool vok = v < Dv;
  float S[RPT], n[RPT], m = 0.f;
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
  if (!fresh) m = st_m[(size_t)slot * H + h];
  for (int t0 = r0; t0 < r1; t0 += TB) {
    const int nt = min(TB, r1 - t0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < nt * Dp; idx += NT) {
      const int tt = idx / Dp, d = idx % Dp;
      const AT* row = proj + (size_t)(t0 + tt) * a.ps;
      qs[idx] = d < D ? ldf(row + a.q_off + h * D + d) * a.qscale : 0.f;
      ks[idx] = d < D ? ldf(row + a.k_off + h * D + d) : 0.f;
    }
    for (int idx = threadIdx.x; idx < nt * VB; idx += NT) {
      const int tt = idx / VB, c = idx % VB;
      vs[idx] = v0 + c < Dv ? ldf(proj + (size_t)(t0 + tt) * a.ps + a.v_off + h * Dv + v0 + c) : 0.f;
    }
    if (threadIdx.x < nt) {
      gi[threadIdx.x] = gates[(size_t)(t0 + threadIdx.x) * 2 * H + h];
      gf[threadIdx.x] = gates[(size_t)(t0 + threadIdx.x) * 2 * H + H + h];
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float fg = gf[tt], ig = gi[tt];
      const float mn = fmaxf(fg + m, ig);
      const float fa = expf(fg + m - mn), ia = expf(ig - mn);
      m = mn;
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
      if (dp == 0 && vok) out[((size_t)(t0 + tt) * H + h) * Dv + v] = pq / (fmaxf(fabsf(pn), expf(-m)) + 1e-6f);
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
  if (blockIdx.z == 0 && threadIdx.x == 0) st_m[(size_t)slot * H + h] = m;
}

template <typename AT, int RPT>
int launch_scan(float* out, const AT* proj, const float* gates, float* S, float* n, float* m, const ScanArgs& a,
                int num_seqs, hipStream_t st) {
  const size_t lds = (size_t)(2 * TB * DP * RPT + TB * VB + 2 * TB) * sizeof(float);
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mlstm_scan_kernel<AT, RPT>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  dim3 grid(num_seqs, a.H, (a.Dv + VB - 1) / VB);
  mlstm_scan_kernel<AT, RPT><<<grid, NT, lds, st>>>(out, proj, gates, S, n, m, a);
  KA_CHECK_LAUNCH();
}

template <typename AT>
int dispatch_scan(float* out, const AT* proj, const float* gates, float* S, float* n, float* m, const ScanArgs& a,
                  int num_seqs, hipStream_t st) {
  const int need = (a.D + DP - 1) / DP;
  if (need <= 1) return launch_scan<AT, 1>(out, proj, gates, S, n, m, a, num_seqs, st);
  if (need <= 2) return launch_scan<AT, 2>(out, proj, gates, S, n, m, a, num_seqs, st);
  if (need <= 4) return launch_scan<AT, 4>(out, proj, gates, S, n, m, a, num_seqs, st);
  if (need <= 8) return launch_scan<AT, 8>(out, proj, gates, S, n, m, a, num_seqs, st);
  if (need <= 16) return launch_scan<AT, 16>(out, proj, gates, S, n, m, a, num_seqs, st);
  if (need <= 32) return launch_scan<AT, 32>(out, proj, gates, S, n, m, a, num_seqs, st);
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

extern "C" int ka_mlstm_scan(float* out, const void* proj, int ps, int q_off, int k_off, int v_off, const float* gates,
                             float* st_S, float* st_n, float* st_m, const int* seq_slots, const int* q_starts,
                             int num_seqs, const int* positions, int H, int D, int Dv, float qscale, int f32,
                             hipStream_t st) {
  if (num_seqs <= 0) return 0;
  if (H <= 0 || D <= 0 || Dv <= 0 || H > 65535) return (int)hipErrorInvalidValue;
  ScanArgs a{q_starts, seq_slots, positions, ps, q_off, k_off, v_off, H, D, Dv, qscale};
  if (f32) return dispatch_scan<float>(out, (const float*)proj, gates, st_S, st_n, st_m, a, num_seqs, st);
  return dispatch_scan<bf16_t>(out, (const bf16_t*)proj, gates, st_S, st_n, st_m, a, num_seqs, st);
}
