// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Attention over a paged cache with the score and weight options that the Llama kernels
// (attention.hip) do not have, each a launch parameter:
//   * per-head RMS norm of q and k with a shared weight, rotary positions on the first `rot` entries
//     of each head (pairs (i, i + rot/2), angle = position * inv_freq[i]), appended to the cache
//     together with the values (`headnorm_rope_append`); values may be the un-normed, un-rotated keys;
//   * a chunked causal mask: query position p sees keys floor(p / chunk) * chunk .. p (chunk 0: all
//     keys 0 .. p); positions count from the start of the sequence, so the mask does not depend on
//     where a prompt was cut into steps;
//   * score soft-capping: s <- cap * tanh(s / cap) (cap 0: none);
//   * a sink: one more term exp(0) in the softmax denominator that carries no value (sink 0: none);
//   * head mixing: the normalised weights of the H heads are mixed by a matrix [H, H] before they
//     are applied to the values: w'_h(j) = sum_g mix[h, g] w_g(j) (mix null: none).
//
// Scores, weights and all accumulation are fp32; AT (bf16_t or float) is the type of q, the cache
// and the output.  Cache layout: k_cache [NB, G, BS, D], v_cache [NB, G, BS, Dv], token-major pages;
// slot = page * BS + offset (-1: a padding row, nothing is written or attended).
//
// `chunk_attention`: one workgroup per query token with all its heads (head mixing needs every
// head's weight for a key in one place).  Pass 1 finds each head's maximum and denominator over the
// visible keys, pass 2 recomputes the scores tile by tile, normalises, mixes the heads and
// accumulates weights x values.  A decode step is the same launch with one token per sequence.
#include "attention_chunk.h"

namespace {

constexpr int NT = 256;
constexpr int NW = NT / 64;
constexpr int KT = 64;        // keys per tile
constexpr int MAX_HEADS = 64;
static_assert(KT == 64, "pass 1 reads one key of the tile per lane");
constexpr int MAX_ACC = 32;   // output values per thread: H * Dv <= NT * MAX_ACC
constexpr int MAX_DL = 8;     // head entries per lane: D <= 64 * MAX_DL

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

// One workgroup per token; each wave takes the heads w, w + NW, ... of the fused [q | k] projection row.
template <typename AT>
__global__ __launch_bounds__(NT) void headnorm_rope_append_kernel(
    AT* __restrict__ q_out, const AT* __restrict__ qk, const float* __restrict__ q_w, const float* __restrict__ k_w,
    const float* __restrict__ inv_freq, const int* __restrict__ positions, const int* __restrict__ slots,
    AT* __restrict__ k_cache, AT* __restrict__ v_cache, int H, int G, int D, int rot, float eps, int BS) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = rot >> 1;
  const float pos = (float)positions[t];
  const int slot = slots[t];
  const AT* row = qk + (size_t)t * (H + G) * D;
  for (int hh = wave; hh < H + G; hh += NW) {
    const bool is_k = hh >= H;
    if (is_k && slot < 0) continue;
    const AT* x = row + (size_t)hh * D;
    const float* w = is_k ? k_w : q_w;
    float v[MAX_DL];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < MAX_DL; ++u) {
      const int i = lane + 64 * u;
      v[u] = i < D ? ldf(x + i) : 0.f;
      ss += v[u] * v[u];
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)D + eps);
    AT* dst;
    AT* vdst = nullptr;
    if (is_k) {
      const int g = hh - H;
      const size_t at = ((size_t)(slot / BS) * G + g) * BS + (slot % BS);
      dst = k_cache + at * D;
      vdst = v_cache + at * D;
    } else {
      dst = q_out + ((size_t)t * H + hh) * D;
    }
#pragma unroll
    for (int u = 0; u < MAX_DL; ++u) {
      const int i = lane + 64 * u;
      if (i < D) {
        float o = v[u] * inv * w[i];
        if (i < rot) {
          // the partner of the pair is normed by this lane too (one more cached load, no exchange)
          const int j = i < half ? i : i - half;
          const int pi = i < half ? i + half : i - half;
          const float po = ldf(x + pi) * inv * w[pi];
          float sn, cs;
          sincosf(pos * inv_freq[j], &sn, &cs);
          o = i < half ? o * cs - po * sn : o * cs + po * sn;
        }
        stf(dst + i, o);
        if (vdst) vdst[i] = x[i];   // the value is the key as projected
      }
    }
  }
}


template <typename AT>
__global__ __launch_bounds__(NT) void chunk_attention_kernel(AT* __restrict__ out, const AT* __restrict__ q,
                                                             const AT* __restrict__ k_cache,
                                                             const AT* __restrict__ v_cache, AttnArgs a) {
  extern __shared__ float lds[];
  const int H = a.H, G = a.G, D = a.D, Dv = a.Dv, BS = a.BS;
  float* qs = lds;                  // [H * D]
  float* sc = qs + H * D;           // [H * KT] normalised weights of a tile
  float* pm = sc + H * KT;          // [H * KT] mixed weights
  float* mx = pm + H * KT;          // [H] maximum (with the sink's 0)
  float* rd = mx + H;               // [H] 1 / denominator
  __shared__ int page[KT];          // page of each key of the tile
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int HV = H * Dv;
  AT* orow = out + (size_t)t * HV;
  if (a.slots[t] < 0) {
    for (int i = threadIdx.x; i < HV; i += NT) stf(orow + i, 0.f);
    return;
  }
  const int p = a.positions[t];
  int seq = t;
  if (a.q_starts != nullptr) {   // the sequence whose rows hold token t: q_starts[seq] <= t < q_starts[seq + 1]
    int lo = 0, hi = a.num_seqs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (a.q_starts[mid] <= t) lo = mid;
      else hi = mid - 1;
    }
    seq = lo;
  }
  const int* bt = a.block_tables + (size_t)seq * a.max_blocks;
  const int start = a.chunk > 0 ? (p / a.chunk) * a.chunk : 0;
  const int n = p - start + 1;
  const int rep = H / G;
  for (int i = threadIdx.x; i < H * D; i += NT) qs[i] = ldf(q + (size_t)t * H * D + i);
  for (int g = threadIdx.x; g < H; g += NT) {
    mx[g] = a.sink ? 0.f : -INFINITY;
    rd[g] = 0.f;
  }
  __syncthreads();

  // score of (head g, key j of the tile at k0), soft-capped
  auto score = [&](int g, int j) -> float {
    const int pos = start + j;
    const AT* kr = k_cache + (((size_t)page[j - (j / KT) * KT] * G + g / rep) * BS + pos % BS) * D;
    const float* qg = qs + g * D;
    float s = 0.f;
    if constexpr (sizeof(AT) == 2) {
      if ((D & 7) == 0) {   // 16-byte loads: 8 bf16 keys entries against 8 fp32 query entries from LDS
        for (int i = 0; i < D; i += 8) {
          const uint4 kv = *reinterpret_cast<const uint4*>(kr + i);
          const f32x4 qa = *reinterpret_cast<const f32x4*>(qg + i), qb = *reinterpret_cast<const f32x4*>(qg + i + 4);
          s += qa[0] * lo_f(kv.x) + qa[1] * hi_f(kv.x) + qa[2] * lo_f(kv.y) + qa[3] * hi_f(kv.y) +
               qb[0] * lo_f(kv.z) + qb[1] * hi_f(kv.z) + qb[2] * lo_f(kv.w) + qb[3] * hi_f(kv.w);
        }
      } else {
        for (int i = 0; i < D; ++i) s += qg[i] * ldf(kr + i);
      }
    } else {
      if ((D & 3) == 0) {
        for (int i = 0; i < D; i += 4) {
          const f32x4 kv = *reinterpret_cast<const f32x4*>(kr + i);
          const f32x4 qa = *reinterpret_cast<const f32x4*>(qg + i);
          s += qa[0] * kv[0] + qa[1] * kv[1] + qa[2] * kv[2] + qa[3] * kv[3];
        }
      } else {
        for (int i = 0; i < D; ++i) s += qg[i] * ldf(kr + i);
      }
    }
    s *= a.scale;
    return a.cap > 0.f ? a.cap * tanhf(s / a.cap) : s;
  };

  // ---- pass 1: per head, the maximum and the sum of exp(score - maximum) ----
  // (running values live in registers of the head's wave: head g belongs to wave g % NW)
  float run_m[MAX_HEADS / NW], run_l[MAX_HEADS / NW];
#pragma unroll
  for (int u = 0; u < MAX_HEADS / NW; ++u) {
    run_m[u] = a.sink ? 0.f : -INFINITY;
    run_l[u] = a.sink ? 1.f : 0.f;
  }
  for (int k0 = 0; k0 < n; k0 += KT) {
    const int nk = min(KT, n - k0);
    __syncthreads();
    if (threadIdx.x < nk) page[threadIdx.x] = bt[(start + k0 + threadIdx.x) / BS];
    __syncthreads();
    for (int it = threadIdx.x; it < H * KT; it += NT) {
      const int g = it / KT, j = it % KT;
      sc[it] = j < nk ? score(g, k0 + j) : -INFINITY;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < MAX_HEADS / NW; ++u) {
      const int g = wave + u * NW;
      if (g < H) {
        const float s = sc[g * KT + lane];
        const float m = fmaxf(run_m[u], wave_max(s));
        const float e = wave_sum(s == -INFINITY ? 0.f : expf(s - m));
        run_l[u] = run_l[u] * (run_m[u] == -INFINITY ? 0.f : expf(run_m[u] - m)) + e;
        run_m[u] = m;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < MAX_HEADS / NW; ++u) {
    const int g = wave + u * NW;
    if (g < H && lane == 0) {
      mx[g] = run_m[u];
      rd[g] = 1.0f / run_l[u];
    }
  }

  // ---- pass 2: weights, head mixing, weights x values ----
  float acc[MAX_ACC];
#pragma unroll
  for (int u = 0; u < MAX_ACC; ++u) acc[u] = 0.f;
  for (int k0 = 0; k0 < n; k0 += KT) {
    const int nk = min(KT, n - k0);
    __syncthreads();
    if (threadIdx.x < nk) page[threadIdx.x] = bt[(start + k0 + threadIdx.x) / BS];
    __syncthreads();
    for (int it = threadIdx.x; it < H * KT; it += NT) {
      const int g = it / KT, j = it % KT;
      sc[it] = j < nk ? expf(score(g, k0 + j) - mx[g]) * rd[g] : 0.f;
    }
    __syncthreads();
    const float* wt = sc;
    if (a.mix != nullptr) {
      for (int it = threadIdx.x; it < H * KT; it += NT) {
        const int h = it / KT, j = it % KT;
        float s = 0.f;
        for (int g = 0; g < H; ++g) s += a.mix[h * H + g] * sc[g * KT + j];
        pm[it] = s;
      }
      __syncthreads();
      wt = pm;
    }
#pragma unroll
    for (int u = 0; u < MAX_ACC; ++u) {
      const int i = threadIdx.x + u * NT;
      if (i < HV) {
        const int h = i / Dv, d = i % Dv;
        const float* wh = wt + h * KT;
        float s = acc[u];
        for (int j = 0; j < nk; ++j) {
          const int pos = start + k0 + j;
          s += wh[j] * ldf(v_cache + (((size_t)page[j] * G + h / rep) * BS + pos % BS) * Dv + d);
        }
        acc[u] = s;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < MAX_ACC; ++u) {
    const int i = threadIdx.x + u * NT;
    if (i < HV) stf(orow + i, acc[u]);
  }
}

}  // namespace

extern "C" int ka_headnorm_rope_append(void* q_out, const void* qk, const float* q_w, const float* k_w,
                                       const float* inv_freq, const int* positions, const int* slots, void* k_cache,
                                       void* v_cache, int T, int H, int G, int D, int rot, float eps, int BS, int f32,
                                       hipStream_t st) {
  if (T <= 0) return 0;
  if (D <= 0 || D > 64 * MAX_DL || rot < 0 || rot > D || (rot & 1) || BS <= 0 || H <= 0 || G <= 0)
    return (int)hipErrorInvalidValue;
  if (f32)
    headnorm_rope_append_kernel<float><<<T, NT, 0, st>>>((float*)q_out, (const float*)qk, q_w, k_w, inv_freq, positions,
                                                         slots, (float*)k_cache, (float*)v_cache, H, G, D, rot, eps, BS);
  else
    headnorm_rope_append_kernel<bf16_t><<<T, NT, 0, st>>>((bf16_t*)q_out, (const bf16_t*)qk, q_w, k_w, inv_freq,
                                                          positions, slots, (bf16_t*)k_cache, (bf16_t*)v_cache, H, G, D,
                                                          rot, eps, BS);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_chunk_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                  const int* block_tables, const int* q_starts, int num_seqs, const int* positions,
                                  const int* slots, const float* mix, int T, int H, int G, int D, int Dv, int chunk, int BS,
                                  int max_blocks, int sink, float scale, float cap, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || H > MAX_HEADS || H * Dv > NT * MAX_ACC || D <= 0 || Dv <= 0 || BS <= 0 || chunk < 0)
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(H * D + 2 * H * KT + 2 * H) * sizeof(float);
  if (lds > 150 * 1024) return (int)hipErrorInvalidValue;
  AttnArgs a{block_tables, q_starts, num_seqs, positions, slots, mix, H, G, D, Dv, chunk, BS, max_blocks, sink, scale, cap};
  if (lds > 48 * 1024) {   // wide models: more dynamic LDS than the default limit
    const void* fn = f32 ? reinterpret_cast<const void*>(chunk_attention_kernel<float>)
                         : reinterpret_cast<const void*>(chunk_attention_kernel<bf16_t>);
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  if (f32)
    chunk_attention_kernel<float><<<T, NT, lds, st>>>((float*)out, (const float*)q, (const float*)k_cache,
                                                      (const float*)v_cache, a);
  else
    chunk_attention_kernel<bf16_t><<<T, NT, lds, st>>>((bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache,
                                                       (const bf16_t*)v_cache, a);
  KA_CHECK_LAUNCH();
}
