// The host side of the engine in C++: what lies between a step's description and its kernel launches (exec.cpp),
// the cache manager's books (cache.cpp), the step packer (pack.cpp) and the scheduler (sched.cpp).  Python keeps the
// entry points (Engine, ModelRunner) and the registries of parts; a model whose parts all describe themselves to the
// executor runs its steps from one call, over a work space the caller sizes once.
// The reference keeps this bookkeeping in compiled code behind a flat kernel interface too (CONTEXT.md:52-53) and
// sizes its step buffers once (crates/allpaca-core/src/model.rs:10930-10939).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#define APC_HOST_EXPORT extern "C" __attribute__((visibility("default")))

// error codes beside the kernels' own (-1 bad argument, -2 unsupported)
#define APC_HOST_ERR_ARENA (-10)      // the work space is too small for this step (ask apc_host_step_bytes)
#define APC_HOST_ERR_STATE (-11)      // calls out of order (a range of the plan without a begun step)

enum { APC_DT_F32 = 0, APC_DT_BF16 = 1, APC_DT_I32 = 2 };

extern "C" {

// A weight matrix [N, K] as the kernels take it: tiled for the MFMA kernels (packed = 1, bfloat16, `chunks` tiles of
// 32 columns a band) or row-major with leading dimension ld.
struct ApcMatrix {
  const void* data;
  int packed, dtype, N, K, chunks, ld;
};

// One block in the pre-norm arrangement: x += attention(norm1(x)); x += swiglu(norm2(x)).
struct ApcLayer {
  const float* norm1_w;
  const float* norm2_w;
  float norm1_eps, norm2_eps;
  ApcMatrix w_qkv, w_o;
  int H, Hk, d, window;       // window 0: none
  float scale;                // 0: 1 / sqrt(d)
  int rot;                    // rotated width (0: no rotation), pairs (i, i + rot / 2)
  const float* cos_sin;       // [positions][2][rot / 2]
  ApcMatrix w_gate, w_up;     // packed: the two tiled matrices; else w_gate is [2F, D] (gate rows, then up rows)
  ApcMatrix w_down;
  int F;
};

// A plan entry: which layer runs, against which pages.
struct ApcPlanEntry {
  int layer;
  void* kv;                   // [pages + 1][2][Hk][page_tokens][d] of this entry's (or the lender's) layer
  int kv_dtype, group, page_tokens, writes;
};

// The batch on the device (int32 arrays; allpaca_amd/engine/batch.py says what each holds).
struct ApcStep {
  int T, S, R, n_decode, n_tiles;
  const int* tokens;
  const int* positions;
  const int* row_seg;
  const int* seg_row0;
  const int* seg_rows;
  const int* seg_pos0;
  const int* state_slots;
  const int* logit_rows;
  const int* decode_rows;
  const int* tile_row0;
  const int* tile_rows;
  int n_groups;
  const int* table[8];        // per paged group: [S][table_width]
  int table_width[8];
  int max_decode_context;     // largest position + 1 among the single-row segments
  int all_rows_decode;        // every row is a single-row segment (decode_rows is then not read)
  int max_prompt_keys;        // largest position + rows among the longer segments (how attention cuts their keys)
};

// Rules that tests and measurements move; the defaults are the kernels' wrappers' own.
struct ApcTunables {
  int whole_min_pairs, last_block_merges, wide_tiles, key_splits_max, key_range_min, force_plain;
};

}  // extern "C"
