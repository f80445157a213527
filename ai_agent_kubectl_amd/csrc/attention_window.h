// Launch arguments shared by the sliding-window attention kernels (attention_window.hip: vector kernel;
// attention_window_tile.hip: matrix-core kernel).
// Cache layout: k_cache [NB, G, BS, D] (a key's entries contiguous), v_cache [NB, G, Dv, BS] (a page's BS values
// of one entry contiguous: the key index is the reduction index of weights x values, so a matrix-core operand is one
// 8-byte load and a vector lane reads a page's values of its entry in 16-byte pieces).
#pragma once
#include "rows_f32.h"

struct SlideArgs {
  const int* block_tables;   // [num_seqs, max_blocks]
  const int* q_starts;       // [num_seqs + 1] or null (token t is block-table row t)
  const int* positions;      // [T]
  const int* slots;          // [T]
  int num_seqs, H, G, D, Dv, window, keep_first, BS, max_blocks;
  int gs, g_off;             // gate row stride and column offset
  float scale;
  const float* dist;         // [3, H] or null.  Set: no softmax; a visible key's weight is
                             // sigmoid(score - dist[0][h] * log(1 + dist[1][h] * (p - j)) + dist[2][h]), not normalised
};

// the unnormalised weight of the key at distance `d` behind the query (SlideArgs::dist of head h in r1, r2, pb)
KA_DEV float dist_sigmoid(float score, float r1, float r2, float pb, int d) {
  return 1.0f / (1.0f + expf(-(score - r1 * log1pf(r2 * (float)d) + pb)));
}

// the matrix-core kernel (bf16): 1 if it takes the shape
extern "C" int ka_sliding_attention_tile_ok(int H, int G, int D, int Dv, int BS);
int sliding_attention_tile(bf16_t* out, const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const bf16_t* gate,
                           const SlideArgs& a, int max_q, int rows_, hipStream_t st);
