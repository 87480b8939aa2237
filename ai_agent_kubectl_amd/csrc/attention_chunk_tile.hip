// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Chunk-masked attention for prompt portions (bf16 activations and cache): one workgroup of 8 waves
// per (sequence, 16 consecutive query rows) with ALL heads, because the head mixing needs every
// head's weight of a (row, key) pair in one place before any value is touched.
//
//   scores     S_g = Q_g K_c(g)^T on MFMA 16x16x32 (bf16 in, fp32 out): wave w owns the heads w, w + 8, ...;
//              its Q fragments stay in registers, the K fragments are 16-byte loads straight from the
//              token-major pages (lane = key, 8 consecutive head entries), no LDS staging;
//   pass 1     per head and row, the running maximum and denominator over the row's visible keys
//              (soft cap, chunk mask, sink), kept in LDS as (maximum, 1 / denominator);
//   pass 2     per tile of 16 keys: the normalised fp32 weights of all heads go to LDS and are mixed over
//              the heads on the fp32 matrix instruction (mfma 16x16x4 f32); weights x values runs on
//              mfma 16x16x16 bf16 with each fp32 weight split exactly into three bf16 terms
//              (hi + mid + lo = the fp32 value), so no weight is rounded and the sums stay fp32.
// A decode step (q_starts null) runs the same kernel with one row per workgroup: scores on MFMA with
// one useful row, mixing and weights x values for that row on the vector ALUs.
//
// Shapes it takes (the launcher returns hipErrorInvalidValue otherwise and the caller uses the
// per-token kernel): D a multiple of 32 up to 256, Dv == D, H <= 64, heads per wave x D <= 512.
#include "attention_chunk.h"

namespace {

constexpr int NT = 1024;   // 16 waves, 4 per SIMD
constexpr int NWV = NT / 64;
constexpr int QT = 16;   // query rows per workgroup
constexpr int KT = 16;   // keys per tile
constexpr int VST = 20;        // keys per value entry in the staged value tile (16 + padding, 8-byte aligned rows)
constexpr int MAXPG = 4096;   // staged block-table entries (the launcher checks max_blocks against it)

typedef short s16x4 __attribute__((ext_vector_type(4)));

// exp and tanh through the hardware exponential (v_exp_f32, about 1 ulp): this kernel serves the bf16
// engine; the fp32 engine's attention (attention_chunk.hip) keeps the library functions
KA_DEV float fast_tanh(float y) {
  y = fminf(fmaxf(y, -15.f), 15.f);
  const float e = __expf(2.f * y);
  return (e - 1.f) * __frcp_rn(e + 1.f);
}

// p = hi + mid + lo exactly, each term a bf16: an fp32 weight as three bf16 MFMA operands
KA_DEV void split3(const f32x4& p, s16x4& hi, s16x4& mid, s16x4& lo) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bf16_t h = f2bf(p[i]);
    const float r1 = p[i] - bf2f(h);
    const bf16_t m = f2bf(r1);
    const float r2 = r1 - bf2f(m);
    hi[i] = (short)h;
    mid[i] = (short)m;
    lo[i] = (short)f2bf(r2);
  }
}

template <int NF, int HPW, int ROWS>
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
  float* TM = ST + 2 * H * QT;       // [H][H]      the mixing matrix
  int* PG = reinterpret_cast<int*>(TM + H * H);   // [max_blocks] pages of the keys this workgroup visits
  // [G][Dv][VST] the key tile's values, entry-major (16 keys of one value entry side by side): the B
  // operand of weights x values is then one 8-byte LDS read; filled from 16-byte global loads
  bf16_t* VS = reinterpret_cast<bf16_t*>(PG + a.max_blocks);
  __shared__ int s_pos[QT];
  // grid (sequences, tiles): the sequence index runs fastest and the tiles run from the last (most keys)
  // to the first, so the longest workgroups of every sequence start first and the short ones fill in
  const int seq = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  int row0, nr;
  if constexpr (ROWS == 1) {   // a decode step: token `seq` is the one row of sequence `seq`
    row0 = seq;
    nr = 1;
    if (a.slots[row0] < 0) {   // a padding row of the batch bucket
      for (int i = tid; i < H * Dv; i += NT) out[(size_t)row0 * H * Dv + i] = 0;
      return;
    }
  } else {
    const int q0 = a.q_starts[seq], q1 = a.q_starts[seq + 1];
    row0 = q0 + QT * (gridDim.y - 1 - blockIdx.y);
    if (row0 >= q1) return;
    nr = min(QT, q1 - row0);
  }
  if (tid < QT) s_pos[tid] = tid < nr ? a.positions[row0 + tid] : -1;
  if (a.mix != nullptr)
    for (int i = tid; i < H * H; i += NT) TM[i] = a.mix[i];
  __syncthreads();
  const int p_last = s_pos[nr - 1];
  const int cs0 = a.chunk > 0 ? (s_pos[0] / a.chunk) * a.chunk : 0;
  const int j_begin = cs0 & ~(KT - 1);
  const int rep = H / G;
  // the pages of keys j_begin .. p_last, staged once: every later page lookup is an LDS read instead of
  // a global load in front of the key / value loads that depend on it
  const int bs_sh = __builtin_ctz(BS);   // the page size is a power of two (the launcher checks)
  const int pg0 = j_begin >> bs_sh;
  {
    const int* btg = a.block_tables + (size_t)seq * a.max_blocks;
    const int npg = (p_last >> bs_sh) - pg0 + 1;
    for (int i = tid; i < npg; i += NT) PG[i] = btg[pg0 + i];   // npg <= max_blocks, which sized PG
  }
  __syncthreads();
  const int* bt = PG - pg0;   // bt[j / BS] as before
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

  const float inv_cap = a.cap > 0.f ? 1.0f / a.cap : 0.f;
  // soft-capped, masked scores of head g (slot u) against the key tile at jt: x[r] for row 4 grp + r, key jt + col
  // kbase_of(jt): this lane's key row of the tile (head 0) in the cache; keys past the tile's last row
  // take a valid address and are masked in `scores`
  auto kbase_of = [&](int jt) -> size_t {
    const int j = min(jt + col, p_last);
    return ((size_t)bt[j >> bs_sh] * G * BS + (j & (BS - 1))) * D + 8 * grp;
  };
  auto scores = [&](int u, int g, int jt, size_t kb, float (&x)[4]) {
    const bf16_t* kp = k_cache + kb + (size_t)(g / rep) * BS * D;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < NF; ++ks)
      acc = mfma16x16x32(as_bf16x8(qf[u][ks]), as_bf16x8(*reinterpret_cast<const uint4*>(kp + 32 * ks)), acc);
    const int jj = jt + col;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float s = acc[r] * a.scale;
      if (a.cap > 0.f) s = a.cap * fast_tanh(s * inv_cap);
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
        scores(u, g, jt, kbase_of(jt), x);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float mn = fmaxf(m[r], row16_max(x[r]));
          const float e = row16_sum(x[r] == -INFINITY ? 0.f : __expf(x[r] - mn));
          l[r] = l[r] * (m[r] == -INFINITY ? 0.f : __expf(m[r] - mn)) + e;
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
  constexpr int NDB = 2 * NF;   // 16-wide blocks of a head's values (Dv == D)
  // ROWS == 16: out[16 rows x 16 values] blocks of this wave's heads on the fp32 matrix cores
  f32x4 pacc[ROWS == QT ? HPW : 1][ROWS == QT ? NDB : 1];
  // ROWS == 1 (a decode row): this thread's head and four consecutive value entries on the vector ALUs
  // (H * Dv <= 4096 for every shape the launcher takes: at most MAXQ quads per thread)
  constexpr int MAXQ = 1;
  const int nquads = (H * Dv) >> 2;
  float acc1[MAXQ][4];
#pragma unroll
  for (int qi = 0; qi < MAXQ; ++qi) acc1[qi][0] = acc1[qi][1] = acc1[qi][2] = acc1[qi][3] = 0.f;
  if constexpr (ROWS == QT) {
#pragma unroll
    for (int u = 0; u < HPW; ++u)
#pragma unroll
      for (int db = 0; db < NDB; ++db) pacc[u][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int HB = (H + 15) >> 4;

  for (int jt = j_begin; jt <= p_last; jt += KT) {
    const size_t kb = kbase_of(jt);
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      const int g = wave + NWV * u;
      if (g < H) {
        float x[4];
        scores(u, g, jt, kb, x);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = 4 * grp + r;
          const float w = x[r] == -INFINITY ? 0.f : __expf(x[r] - ST[(g * QT + row) * 2]) * ST[(g * QT + row) * 2 + 1];
          P[(g * QT + row) * KT + col] = w;
        }
      }
    }
    __syncthreads();
    if constexpr (ROWS == QT) {
      // stage the tile's values (every workgroup-mate is past the previous tile's reads of VS here)
      const int c8 = Dv >> 3;
      for (int it = tid; it < G * KT * c8; it += NT) {
        const int d8 = it % c8, key = (it / c8) % KT, c = it / (c8 * KT);
        const int j = min(jt + key, p_last);
        const uint4 raw = *reinterpret_cast<const uint4*>(
            v_cache + (((size_t)bt[j >> bs_sh] * G + c) * BS + (j & (BS - 1))) * Dv + 8 * d8);
        bf16_t* dst = VS + ((size_t)(c * Dv + 8 * d8)) * VST + key;
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          dst[(2 * i) * VST] = (bf16_t)(w[i] & 0xffffu);
          dst[(2 * i + 1) * VST] = (bf16_t)(w[i] >> 16);
        }
      }
    }
    const float* W = P;
    if (a.mix != nullptr) {
      if constexpr (ROWS == QT) {
        // PM[h][rj] = sum_g mix[h][g] P[g][rj] as 16 x 16 blocks (16 heads x 16 of the tile's 256 (row, key)
        // pairs) on mfma 16x16x4 f32: A = mix[h block][g .. g + 4], B = P[g .. g + 4][rj block]
        for (int blk = wave; blk < HB * QT; blk += NWV) {
          const int hb = blk / QT, rjb = blk % QT;
          const int h = hb * 16 + col;
          f32x4 c = {0.f, 0.f, 0.f, 0.f};
          for (int g0 = 0; g0 < H; g0 += 4) {
            const int g = g0 + grp;
            const float av = (h < H && g < H) ? TM[h * H + g] : 0.f;
            const float bv = g < H ? P[g * QT * KT + rjb * 16 + col] : 0.f;
            c = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, c, 0, 0, 0);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int ho = hb * 16 + 4 * grp + r;
            if (ho < H) PM[ho * QT * KT + rjb * 16 + col] = c[r];
          }
        }
      } else {
        for (int it = tid; it < H * KT; it += NT) {   // row 0 only
          const int h = it / KT, j = it % KT;
          float sm = 0.f;
          for (int g = 0; g < H; ++g) sm += TM[h * H + g] * P[g * QT * KT + j];
          PM[h * QT * KT + j] = sm;
        }
      }
      __syncthreads();
      W = PM;
    } else if (ROWS == QT) {
      __syncthreads();   // the staged values are read below
    }
    if constexpr (ROWS == QT) {
      // out[row][d] += sum_key W[h][row][key] V[key][d] on mfma 16x16x16 bf16, three times: the fp32
      // weight is split exactly into three bf16 terms (split3), the values are bf16 already.
      // A = W[h][row = col][4 grp .. + 4], B = V[key 4 grp .. + 4][16 db + col]
#pragma unroll
      for (int u = 0; u < HPW; ++u) {
        const int h = wave + NWV * u;
        if (h < H) {
          s16x4 ahi, amid, alo;
          split3(*reinterpret_cast<const f32x4*>(W + (h * QT + col) * KT + 4 * grp), ahi, amid, alo);
          const bf16_t* vs = VS + ((size_t)((h / rep) * Dv + col)) * VST + 4 * grp;
#pragma unroll
          for (int db = 0; db < NDB; ++db) {
            const s16x4 b = *reinterpret_cast<const s16x4*>(vs + 16 * db * VST);
            pacc[u][db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ahi, b, pacc[u][db], 0, 0, 0);
            pacc[u][db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(amid, b, pacc[u][db], 0, 0, 0);
            pacc[u][db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(alo, b, pacc[u][db], 0, 0, 0);
          }
        }
      }
    } else {
#pragma unroll
      for (int qi = 0; qi < MAXQ; ++qi) {
        const int quad = tid + qi * NT;
        if (quad < nquads) {
          const int hq = (4 * quad) / Dv, d0 = (4 * quad) % Dv;
          const float* wh = W + hq * QT * KT;   // row 0
#pragma unroll
          for (int j4 = 0; j4 < KT; j4 += 4) {
            const f32x4 w4 = *reinterpret_cast<const f32x4*>(wh + j4);
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
              const int j = min(jt + j4 + jj, p_last);
              const uint2 raw = *reinterpret_cast<const uint2*>(
                  v_cache + (((size_t)bt[j >> bs_sh] * G + hq / rep) * BS + (j & (BS - 1))) * Dv + d0);
              acc1[qi][0] += w4[jj] * lo_f(raw.x);
              acc1[qi][1] += w4[jj] * hi_f(raw.x);
              acc1[qi][2] += w4[jj] * lo_f(raw.y);
              acc1[qi][3] += w4[jj] * hi_f(raw.y);
            }
          }
        }
      }
    }
    if (a.mix == nullptr) __syncthreads();   // P is rewritten by the next tile
  }
  if constexpr (ROWS == QT) {
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      const int h = wave + NWV * u;
      if (h < H) {
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int row = 4 * grp + r;
            if (row < nr) out[(size_t)(row0 + row) * H * Dv + h * Dv + 16 * db + col] = f2bf(pacc[u][db][r]);
          }
        }
      }
    }
  } else {
#pragma unroll
    for (int qi = 0; qi < MAXQ; ++qi) {
      const int quad = tid + qi * NT;
      if (quad < nquads) {
        uint2 o;
        o.x = pack2(acc1[qi][0], acc1[qi][1]);
        o.y = pack2(acc1[qi][2], acc1[qi][3]);
        *reinterpret_cast<uint2*>(out + (size_t)row0 * H * Dv + 4 * quad) = o;
      }
    }
  }
}

template <int NF, int HPW>
int launch(bf16_t* out, const bf16_t* q, const bf16_t* k, const bf16_t* v, const AttnArgs& a, int tiles, size_t lds,
           hipStream_t st) {
  auto kern = a.q_starts == nullptr ? chunk_attention_tile_kernel<NF, HPW, 1> : chunk_attention_tile_kernel<NF, HPW, QT>;
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  kern<<<dim3(a.num_seqs, tiles), NT, lds, st>>>(out, q, k, v, a);
  return (int)hipGetLastError();
}

template <int NF>
int launch_nf(bf16_t* out, const bf16_t* q, const bf16_t* k, const bf16_t* v, const AttnArgs& a, int tiles, size_t lds,
              hipStream_t st) {
  const int hpw = (a.H + NWV - 1) / NWV;
  if (hpw <= 1) return launch<NF, 1>(out, q, k, v, a, tiles, lds, st);
  if (hpw <= 2) return launch<NF, 2>(out, q, k, v, a, tiles, lds, st);
  if constexpr (NF <= 2) return launch<NF, 4>(out, q, k, v, a, tiles, lds, st);
  return (int)hipErrorInvalidValue;
}

}  // namespace

// 1 when ka_chunk_attention_tile takes the shape (see the head of this file)
extern "C" int ka_chunk_attention_tile_ok(int H, int G, int D, int Dv, int BS) {
  const int nf = D / 32;
  const int hpw = H <= NWV ? 1 : (H <= 2 * NWV ? 2 : 4);
  const size_t lds = (size_t)(2 * H * QT * KT + 2 * H * QT + H * H) * sizeof(float) + (size_t)G * Dv * VST * 2;   // + the staged pages
  return H > 0 && G > 0 && H % G == 0 && H <= 64 && D % 32 == 0 && (nf <= 4 || nf == 6 || nf == 8) && hpw * nf <= 8 &&
         Dv == D && (BS & (BS - 1)) == 0 && BS > 0 && lds <= 140 * 1024;
}

// max_q: the longest run of rows of one sequence in this step (the grid's y extent is ceil(max_q / 16)).
// q_starts null: a decode step, token t is the single row of block-table row t (one workgroup per token).
extern "C" int ka_chunk_attention_tile(void* out, const void* q, const void* k_cache, const void* v_cache,
                                       const int* block_tables, const int* q_starts, int num_seqs, const int* positions,
                                       const int* slots, const float* mix, int max_q, int H, int G, int D, int Dv,
                                       int chunk, int BS, int max_blocks, int sink, float scale, float cap,
                                       hipStream_t st) {
  if (num_seqs <= 0 || max_q <= 0) return 0;
  if (!ka_chunk_attention_tile_ok(H, G, D, Dv, BS) || chunk < 0) return (int)hipErrorInvalidValue;
  AttnArgs a{block_tables, q_starts, num_seqs, positions, slots, mix, H, G, D, Dv, chunk, BS, max_blocks, sink, scale, cap};
  if (max_blocks > MAXPG) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(2 * H * QT * KT + 2 * H * QT + H * H + max_blocks) * sizeof(float) + (size_t)G * Dv * VST * 2;
  const int tiles = q_starts == nullptr ? 1 : (max_q + QT - 1) / QT;
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
