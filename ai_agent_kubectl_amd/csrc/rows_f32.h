// Helpers shared by the row kernels of the fp32-residual models (streams_f32.hip, mlstm.hip,
// attention_latent.hip, moe_route.hip): typed loads / stores (AT = bf16_t or float, arithmetic always in
// fp32) and a block-wide sum for workgroups of NT = 256 threads.
#pragma once
#include "common.h"

namespace rows {

constexpr int NT = 256;
constexpr int NW = NT / 64;

template <typename T>
KA_DEV float ldf(const T* p) {
  if constexpr (sizeof(T) == 4) return *p;
  else return bf2f(*p);
}
template <typename T>
KA_DEV void stf(T* p, float v) {
  if constexpr (sizeof(T) == 4) *p = v;
  else *p = f2bf(v);
}

// sum of one value per thread over the block; every thread gets the total.  red: [NW] floats of LDS.
KA_DEV float block_sum(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v = wave_sum(v);
  __syncthreads();   // red may still be read from the previous call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) s += red[w];
  return s;
}

// the sequence whose rows hold token t: q_starts[seq] <= t < q_starts[seq + 1] (q_starts null: token t is sequence t)
KA_DEV int seq_of(const int* q_starts, int num_seqs, int t) {
  if (q_starts == nullptr) return t;
  int lo = 0, hi = num_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_starts[mid] <= t) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

}  // namespace rows
