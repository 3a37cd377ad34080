// How many queries a tile of each attention kernel's work list holds: the one place where these
// sizes are written.  The kernels include it; who makes the lists asks eng_attn_tile_sizes().
#pragma once

// The optional terms of a score and of the output that the attention kernels' `_terms` entry
// points take (a null pointer or 0 where a term is absent).  A score is made in this order:
//   s = (q . k) * scale            (head_scale[h] instead of scale where given)
//   s = softcap * tanh(s / softcap)                       (softcap > 0)
//   s -= slopes[h] * (query position - key position)
//   s += dist_bias[h * n_dist + min(distance, n_dist - 1)]      (a table of float, a row a head)
// keep_first: with a window, the first so many keys stay visible.  gate (rows of stride ldg, the
// queries' element type): the output is multiplied by its sigmoid.
struct AttnTerms {
  const float* head_scale;
  const float* slopes;
  const void* gate;
  int ldg, keep_first;
  float softcap;
  const float* dist_bias;
  int n_dist;
};

#define ATTN_TILE_QUERIES 16           // attn_tile (attention.hip): queries a block
#define ATTN_PREFILL_TILE_QUERIES 128  // attn_prefill (attention_prefill.hip): queries a block

// How the decode kernel (attention_decode.hip) is launched for n_rows single rows of n_heads
// heads whose longest walk is `keys` keys (a window's and its kept first keys' at most): in how
// many parts a row's keys go at most, the waves a block, the keys a wave takes at a time.
// Eight waves a block (four where the rows' blocks alone are more than the CUs, or the keys no
// more than four waves' tiles); tiles of 32 keys, of 64 where the blocks are more than three a CU
// and the walk is 640 keys or more; splits only where a wave would walk 96 keys or more, as many
// as leave it a tile, and no more than give every block a compute unit at once.
#define ATTN_DECODE_ROW_WAVES 8
#define ATTN_DECODE_SPLIT_KEYS_A_WAVE 96
static inline void attn_decode_row_work(int n_compute_units, int n_rows, int n_heads, int head_dim, long keys,
                                        int* n_splits, int* n_waves, int* key_tile) {
  const long c = keys;
  const long tiles = c + 31 < 32 ? 1 : (c + 31) / 32;
  const long blocks = n_rows * n_heads < 1 ? 1 : (long)n_rows * n_heads;
  int nw = blocks > n_compute_units ? 4 : ATTN_DECODE_ROW_WAVES;
  const int fewest = head_dim > 128 ? 4 : 2;  // (the block's threads write a column of the head each)
  while (nw > fewest && nw / 2 >= tiles) nw /= 2;
  const long keys_a_wave = c / nw;
  long ns = 1;
  if (keys_a_wave >= ATTN_DECODE_SPLIT_KEYS_A_WAVE) {
    ns = keys_a_wave / 32;
    if (n_compute_units / blocks < ns) ns = n_compute_units / blocks;
    if (ns > 64) ns = 64;
    if (ns < 1) ns = 1;
  }
  *n_splits = (int)ns, *n_waves = nw, *key_tile = 32;
  if (blocks > 3 * n_compute_units && c >= 640) {
    // many rows and a long walk: tiles of 64 keys, and as many waves a block as make eight a CU
    const long want = (8L * n_compute_units + blocks - 1) / blocks;
    nw = fewest;
    while (nw < 8 && nw < want) nw *= 2;
    *n_waves = nw, *key_tile = 64;
  }
}
