// The prompt-portion attention kernel for tiles of 128 rows (attention_wide_bf16.hip), called from the launch code
// in attention_bf16.hip.
#pragma once
#include "common.h"

constexpr int ATTN_WIDE_ROWS = 128;  // rows of a tile

// True for the head sizes (128 and 64) and page sizes the kernel takes (pages of a power of two, at least 16 positions).
bool attn_wide_takes(int d, int page_tokens);
// Arguments as apc_attention_prefill_bf16; tiles of up to ATTN_WIDE_ROWS rows.  n_splits > 1: the keys of every tile
// are cut into that many ranges, a block each, and a second kernel adds the ranges; `parts` then has room for
// n_splits * part_rows * H * (d + 2) floats, part_rows being at least the largest row index of a tile + 1.
int launch_attn_prefill_wide(const bf16_t* q, int ldq, int q_off, bf16_t* out, int ldo, int H, int Hk,
                             const bf16_t* cache, int page_tokens, const int* block_table, int max_blocks,
                             const int* positions, const int* row_seg, const int* tile_row0, const int* tile_rows,
                             int n_tiles, int window, float scale, int n_splits, int part_rows, float* parts,
                             int d, hipStream_t stream);
