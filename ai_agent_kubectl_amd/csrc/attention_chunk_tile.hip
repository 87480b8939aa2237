// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Chunk-masked attention for prompt portions (bf16 activations and cache): one workgroup of 16 waves
// per (sequence, 16 consecutive query rows) with ALL heads, because the head mixing needs every
// head's weight of a (row, key) pair in one place before any value is touched.
//
//   scores     S_g = Q_g K_c(g)^T on MFMA 16x16x32 (bf16 in, fp32 out): wave w owns the heads w, w + 16, ...;
//              its Q fragments stay in registers, the K fragments are 16-byte loads straight from the
//              token-major pages (lane = key, 8 consecutive head entries), no LDS staging;
//   pass 1     per head and row, the running maximum and denominator over the row's visible keys
//              (soft cap, chunk mask, sink), kept in LDS as (maximum, 1 / denominator);
//   pass 2     per tile of 16 keys: the normalised fp32 weights of all heads go to LDS, are mixed over
//              the heads (mix[h, g] read as wave-uniform scalars), and each thread adds weight x value
//              for 16 rows x 4 consecutive value entries of one head in fp32 registers.
// Weights, mixing and the weights x values sums are fp32 on the vector ALUs (the weights are never
// rounded to bf16); only Q K^T runs on the matrix cores, where bf16 inputs lose nothing.
//
// Shapes it takes (the launcher returns hipErrorInvalidValue otherwise and the caller uses the
// per-token kernel): D a multiple of 32 up to 256, H <= 64, H * Dv <= 4096, Dv a multiple of 4.
#include "attention_chunk.h"

namespace {

constexpr int NT = 1024;
constexpr int NWV = NT / 64;
constexpr int QT = 16;   // query rows per workgroup
constexpr int KT = 16;   // keys per tile

template <int NF, int HPW>
__global__ __launch_bounds__(NT) void chunk_attention_tile_kernel(bf16_t* __restrict__ out,
                                                                  const bf16_t* __restrict__ q,
                                                                  const bf16_t* __restrict__ k_cache,
                                                                  const bf16_t* __restrict__ v_cache, AttnArgs a) {
  extern __shared__ float lds[];
  const int H = a.H, G = a.G, Dv = a.Dv, BS = a.BS;
  constexpr int D = NF * 32;
  float* P = lds;                    // [H][QT][KT] normalised weights of the current key tile
  float* PM = P + H * QT * KT;       // [H][QT][KT] mixed weights
  float* ST = PM + H * QT * KT;      // [H][QT][2]  (maximum, 1 / denominator)
  __shared__ int s_pos[QT];
  const int seq = blockIdx.y;
  const int q0 = a.q_starts[seq], q1 = a.q_starts[seq + 1];
  const int row0 = q0 + QT * blockIdx.x;
  if (row0 >= q1) return;
  const int nr = min(QT, q1 - row0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  if (tid < QT) s_pos[tid] = tid < nr ? a.positions[row0 + tid] : -1;
  __syncthreads();
  const int p_last = s_pos[nr - 1];
  const int cs0 = a.chunk > 0 ? (s_pos[0] / a.chunk) * a.chunk : 0;
  const int j_begin = cs0 & ~(KT - 1);
  const int* bt = a.block_tables + (size_t)seq * a.max_blocks;
  const int rep = H / G;
  // the four S rows of this lane: row = 4 * grp + r; visible keys lo[r] .. hi[r] (hi < lo: no row)
  int lo[4], hi[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int p = s_pos[4 * grp + r];
    hi[r] = p;
    lo[r] = p < 0 ? 0 : (a.chunk > 0 ? (p / a.chunk) * a.chunk : 0);
  }
  // Q fragments (A operand): row = col, head entries 32 ks + 8 grp .. + 8
  uint4 qf[HPW][NF];
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    const int g = wave + NWV * u;
    if (g < H) {
      const bf16_t* qp = q + ((size_t)(row0 + min(col, nr - 1)) * H + g) * D + 8 * grp;
#pragma unroll
      for (int ks = 0; ks < NF; ++ks) qf[u][ks] = *reinterpret_cast<const uint4*>(qp + 32 * ks);
    }
  }

  // soft-capped, masked scores of head g (slot u) against the key tile at jt: x[r] for row 4 grp + r, key jt + col
  auto scores = [&](int u, int g, int jt, float (&x)[4]) {
    const int j = min(jt + col, p_last);      // keys past the tile's last row: a valid address, masked below
    const bf16_t* kp = k_cache + (((size_t)bt[j / BS] * G + g / rep) * BS + j % BS) * D + 8 * grp;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < NF; ++ks)
      acc = mfma16x16x32(as_bf16x8(qf[u][ks]), as_bf16x8(*reinterpret_cast<const uint4*>(kp + 32 * ks)), acc);
    const int jj = jt + col;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float s = acc[r] * a.scale;
      if (a.cap > 0.f) s = a.cap * tanhf(s / a.cap);
      x[r] = (jj <= hi[r] && jj >= lo[r]) ? s : -INFINITY;
    }
  };

  // ---- pass 1 ----
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    const int g = wave + NWV * u;
    if (g < H) {
      float m[4], l[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        m[r] = a.sink ? 0.f : -INFINITY;
        l[r] = a.sink ? 1.f : 0.f;
      }
      for (int jt = j_begin; jt <= p_last; jt += KT) {
        float x[4];
        scores(u, g, jt, x);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float mn = fmaxf(m[r], row16_max(x[r]));
          const float e = row16_sum(x[r] == -INFINITY ? 0.f : expf(x[r] - mn));
          l[r] = l[r] * (m[r] == -INFINITY ? 0.f : expf(m[r] - mn)) + e;
          m[r] = mn;
        }
      }
      if (col == 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          ST[(g * QT + 4 * grp + r) * 2] = m[r];
          ST[(g * QT + 4 * grp + r) * 2 + 1] = l[r] > 0.f ? 1.0f / l[r] : 0.f;
        }
      }
    }
  }
  __syncthreads();

  // ---- pass 2 ----
  // weights x values: this thread's head and its four consecutive value entries
  const int nquads = (H * Dv) >> 2;
  const bool has_quad = tid < nquads;
  const int hq = has_quad ? (4 * tid) / Dv : 0, d0 = has_quad ? (4 * tid) % Dv : 0;
  float acc[QT][4];
#pragma unroll
  for (int r = 0; r < QT; ++r) acc[r][0] = acc[r][1] = acc[r][2] = acc[r][3] = 0.f;
  // mixing: this thread's (row, key) of the tile and its heads h0, h0 + 4, ...
  const int rj = tid & (QT * KT - 1);
  const int h0 = __builtin_amdgcn_readfirstlane(tid >> 8);
  constexpr int HK = 16;   // heads per thread in the mixing: H <= 4 * HK

  for (int jt = j_begin; jt <= p_last; jt += KT) {
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      const int g = wave + NWV * u;
      if (g < H) {
        float x[4];
        scores(u, g, jt, x);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = 4 * grp + r;
          const float w = x[r] == -INFINITY ? 0.f : expf(x[r] - ST[(g * QT + row) * 2]) * ST[(g * QT + row) * 2 + 1];
          P[(g * QT + row) * KT + col] = w;
        }
      }
    }
    __syncthreads();
    const float* W = P;
    if (a.mix != nullptr) {
      float s[HK];
#pragma unroll
      for (int k = 0; k < HK; ++k) s[k] = 0.f;
      for (int g = 0; g < H; ++g) {
        const float pv = P[g * QT * KT + rj];
#pragma unroll
        for (int k = 0; k < HK; ++k) {
          const int h = h0 + 4 * k;
          if (h < H) s[k] += a.mix[h * H + g] * pv;
        }
      }
#pragma unroll
      for (int k = 0; k < HK; ++k) {
        const int h = h0 + 4 * k;
        if (h < H) PM[h * QT * KT + rj] = s[k];
      }
      __syncthreads();
      W = PM;
    }
    if (has_quad) {
      const float* wh = W + hq * QT * KT;
#pragma unroll
      for (int j4 = 0; j4 < KT; j4 += 4) {
        float v[4][4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int j = min(jt + j4 + jj, p_last);   // past the last row: weight 0, any valid value
          const uint2 raw = *reinterpret_cast<const uint2*>(
              v_cache + (((size_t)bt[j / BS] * G + hq / rep) * BS + j % BS) * Dv + d0);
          v[jj][0] = lo_f(raw.x);
          v[jj][1] = hi_f(raw.x);
          v[jj][2] = lo_f(raw.y);
          v[jj][3] = hi_f(raw.y);
        }
#pragma unroll
        for (int r = 0; r < QT; ++r) {
          const f32x4 w4 = *reinterpret_cast<const f32x4*>(wh + r * KT + j4);
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[r][e] += w4[jj] * v[jj][e];
          }
        }
      }
    }
    if (a.mix == nullptr) __syncthreads();   // P is rewritten by the next tile
  }
  if (has_quad) {
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      if (r < nr) {
        uint2 o;
        o.x = pack2(acc[r][0], acc[r][1]);
        o.y = pack2(acc[r][2], acc[r][3]);
        *reinterpret_cast<uint2*>(out + (size_t)(row0 + r) * H * Dv + hq * Dv + d0) = o;
      }
    }
  }
}

template <int NF, int HPW>
int launch(bf16_t* out, const bf16_t* q, const bf16_t* k, const bf16_t* v, const AttnArgs& a, int tiles, size_t lds,
           hipStream_t st) {
  auto kern = chunk_attention_tile_kernel<NF, HPW>;
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  kern<<<dim3(tiles, a.num_seqs), NT, lds, st>>>(out, q, k, v, a);
  return (int)hipGetLastError();
}

template <int NF>
int launch_nf(bf16_t* out, const bf16_t* q, const bf16_t* k, const bf16_t* v, const AttnArgs& a, int tiles, size_t lds,
              hipStream_t st) {
  const int hpw = (a.H + NWV - 1) / NWV;
  if (hpw <= 1) return launch<NF, 1>(out, q, k, v, a, tiles, lds, st);
  if (hpw <= 2) return launch<NF, 2>(out, q, k, v, a, tiles, lds, st);
  return launch<NF, 4>(out, q, k, v, a, tiles, lds, st);
}

}  // namespace

// 1 when ka_chunk_attention_tile takes the shape (see the head of this file)
extern "C" int ka_chunk_attention_tile_ok(int H, int G, int D, int Dv, int BS) {
  const int nf = D / 32;
  const int hpw = H <= NWV ? 1 : (H <= 2 * NWV ? 2 : 4);
  const size_t lds = (size_t)(2 * H * QT * KT + 2 * H * QT) * sizeof(float);
  return H > 0 && G > 0 && H % G == 0 && H <= 64 && D % 32 == 0 && (nf <= 4 || nf == 6 || nf == 8) && hpw * nf <= 8 &&
         Dv % 4 == 0 &&
         H * Dv <= 4 * NT && BS > 0 && lds <= 150 * 1024;
}

// max_q: the longest run of rows of one sequence in this step (the grid's x extent is ceil(max_q / 16))
extern "C" int ka_chunk_attention_tile(void* out, const void* q, const void* k_cache, const void* v_cache,
                                       const int* block_tables, const int* q_starts, int num_seqs, const int* positions,
                                       const int* slots, const float* mix, int max_q, int H, int G, int D, int Dv,
                                       int chunk, int BS, int max_blocks, int sink, float scale, float cap,
                                       hipStream_t st) {
  if (num_seqs <= 0 || max_q <= 0) return 0;
  if (!ka_chunk_attention_tile_ok(H, G, D, Dv, BS) || q_starts == nullptr || chunk < 0) return (int)hipErrorInvalidValue;
  AttnArgs a{block_tables, q_starts, num_seqs, positions, slots, mix, H, G, D, Dv, chunk, BS, max_blocks, sink, scale, cap};
  const size_t lds = (size_t)(2 * H * QT * KT + 2 * H * QT) * sizeof(float);
  const int tiles = (max_q + QT - 1) / QT;
  bf16_t* o = (bf16_t*)out;
  const bf16_t *qq = (const bf16_t*)q, *kk = (const bf16_t*)k_cache, *vv = (const bf16_t*)v_cache;
  switch (D / 32) {
    case 1: return launch_nf<1>(o, qq, kk, vv, a, tiles, lds, st);
    case 2: return launch_nf<2>(o, qq, kk, vv, a, tiles, lds, st);
    case 3: return launch_nf<3>(o, qq, kk, vv, a, tiles, lds, st);
    case 4: return launch_nf<4>(o, qq, kk, vv, a, tiles, lds, st);
    case 6: return launch_nf<6>(o, qq, kk, vv, a, tiles, lds, st);
    case 8: return launch_nf<8>(o, qq, kk, vv, a, tiles, lds, st);
  }
  return (int)hipErrorInvalidValue;
}
