// Launch arguments shared by the chunk-masked attention kernels (attention_chunk.hip: one workgroup per
// token, any dtype and shape; attention_chunk_tile.hip: one workgroup per 16 query rows, bf16, MFMA scores).
#pragma once
#include "common.h"

struct AttnArgs {
  const int* block_tables;   // [S, max_blocks]
  const int* q_starts;       // [S + 1] first token of each sequence's rows (varlen step); null: token t is row t
  int num_seqs;
  const int* positions;      // [T]
  const int* slots;          // [T]  < 0: padding row
  const float* mix;          // [H, H] or null
  int H, G, D, Dv, chunk, BS, max_blocks, sink;
  float scale, cap;
};
