// The plan executor: a model described once (layers, plan entries, embedding, final norm, head) and a step's
// launches issued from one call, every intermediate in a work space that the caller brings (no allocation in a
// step).  The sequence of operations is the one the Python parts run (allpaca_amd/parts: attention.py, mlp.py,
// block.py, models/decoder.py); a model with a part that does not describe itself here is walked in Python instead.
//
// Work space: a bump allocator over the caller's buffer, reset at the start of a step.  `apc_host_step_bytes` runs
// the same code without launching and returns the peak, so the caller can size the buffer before the first step of a
// shape (and once for the largest step it will ever run).
#include "host.h"
#include "kernels.h"
#include "rules.h"

#include <chrono>
#include <cmath>
#include <string>
#include <vector>

namespace {

using namespace apc_rules;

struct Buf {  // rows of activations
  void* p = nullptr;
  int dtype = APC_DT_BF16, rows = 0, cols = 0, ld = 0;
};

struct Emit {  // what a product into the residual left for the RMS norm (weight g) that reads the residual next
  const float* g = nullptr;
  float eps = 0.f;
  Buf raw;
  float* ss = nullptr;
  int ss_rows = 0, ss_cols = 0;
  bool filled = false;
  // where raw and ss are taken from: a slot that outlives the layer (what a layer leaves for the next one), or the
  // layer's own scratch (null)
  char* slot = nullptr;
  size_t slot_at = 0;
};

struct Timed {
  const char* name;
  hipEvent_t e0, e1;
};

struct Program {
  int D = 0, V = 0, run_dtype = APC_DT_BF16;
  ApcMatrix embedding{}, head{};
  const float* final_norm_w = nullptr;
  float final_norm_eps = 0.f;
  std::vector<ApcLayer> layers;
  std::vector<ApcPlanEntry> plan;
  ApcTunables tun{256, 1, 1, 8, 2048, 0};
  int* pair_counters = nullptr;
  int pair_capacity = 0;
  // ---- the step in work
  bool begun = false;
  bool dry = false;
  char* arena = nullptr;
  size_t cap = 0, at = 0, peak = 0;
  bool overflow = false;
  hipStream_t stream = nullptr;
  ApcStep step{};
  Buf x;          // the float32 residual stream [T, D]
  Emit left;      // for the first norm of the next plan entry
  // Behind x: two slots that take turns in holding what a layer leaves for the next one's first norm; behind them the
  // scratch of the layer in work, which starts anew with every layer.
  char* slot[2] = {nullptr, nullptr};
  size_t slot_cap = 0, scratch_mark = 0;
  // ---- per-launch timers (a pass of its own beside the measured one)
  bool timing = false;
  std::vector<Timed> timed;
  std::string report;

  void* take(size_t bytes) {
    at = (at + 255) & ~(size_t)255;
    void* p = arena + at;
    at += bytes;
    if (at > peak) peak = at;
    if (!dry && at > cap) overflow = true;
    return p;
  }
  Buf rows(int n, int cols, int dtype) {
    Buf b;
    b.dtype = dtype;
    b.rows = n;
    b.cols = cols;
    b.ld = cols;
    b.p = take((size_t)n * cols * (dtype == APC_DT_BF16 ? 2 : 4));
    return b;
  }
  float* floats(size_t n) { return (float*)take(n * sizeof(float)); }
  void* emit_take(Emit& e, size_t bytes) {
    if (!e.slot) return take(bytes);
    e.slot_at = (e.slot_at + 255) & ~(size_t)255;
    void* p = e.slot + e.slot_at;
    e.slot_at += bytes;
    if (e.slot_at > slot_cap) overflow = true;   // (the slots are sized for the largest of what the kernels leave)
    return p;
  }
  Buf emit_rows(Emit& e, int n, int cols) {
    Buf b;
    b.dtype = APC_DT_BF16;
    b.rows = n;
    b.cols = cols;
    b.ld = cols;
    b.p = emit_take(e, (size_t)n * cols * 2);
    return b;
  }
};

// A launch: skipped in a sizing run; with timers on, bracketed by events.
#define LAUNCH(P_, NAME_, CALL_)                                           \
  do {                                                                     \
    if ((P_).overflow) return APC_HOST_ERR_ARENA;                          \
    if (!(P_).dry) {                                                       \
      Timed t_{NAME_, nullptr, nullptr};                                   \
      if ((P_).timing) {                                                   \
        hipEventCreate(&t_.e0);                                            \
        hipEventCreate(&t_.e1);                                            \
        hipEventRecord(t_.e0, (P_).stream);                                \
      }                                                                    \
      const int rc_ = (CALL_);                                             \
      if ((P_).timing) {                                                   \
        hipEventRecord(t_.e1, (P_).stream);                                \
        (P_).timed.push_back(t_);                                          \
      }                                                                    \
      if (rc_) return rc_;                                                 \
    }                                                                      \
  } while (0)

bool act_ok(const Buf& a) {
  return a.dtype == APC_DT_BF16 && a.cols % 8 == 0 && a.ld % 8 == 0 && ((uintptr_t)a.p & 15u) == 0;
}
int elem_size(int dtype) { return dtype == APC_DT_BF16 ? 2 : 4; }

// ------------------------------------------------------------------------------------------------ products
// out = a . w^T (mode 0 bfloat16 / 1 float32 by out's type), or out += a . w^T (float32)
int gemm_bf16(Program& P, const Buf& a, const ApcMatrix& w, const Buf& out, bool accumulate) {
  const int M = a.rows, K = a.cols, N = w.N;
  if (w.K != K || out.rows != M || out.cols != N || !act_ok(a)) return -1;
  if (accumulate && out.dtype != APC_DT_F32) return -1;
  const int mode = accumulate ? 2 : (out.dtype == APC_DT_BF16 ? 0 : 1);
  if (M > SKINNY_MAX_ROWS) {
    const int ks = M <= MANY_ROWS_SPLIT_MAX ? tiled_k_split(M, N, K) : apc_gemm_direct_k_split(M, N, K);
    if (ks > 1) {
      float* ws = P.floats((size_t)ks * M * N);
      LAUNCH(P, "gemm_splitk_bf16",
             apc_gemm_splitk_bf16(a.p, a.ld, w.data, nullptr, out.p, out.ld, M, N, K, mode, ks, ws, P.stream));
      return 0;
    }
    LAUNCH(P, "gemm_bf16", apc_gemm_bf16(a.p, a.ld, w.data, out.p, out.ld, M, N, K, mode, P.stream));
    return 0;
  }
  LAUNCH(P, "skinny_gemm_bf16", apc_skinny_gemm_bf16(a.p, a.ld, w.data, out.p, out.ld, M, N, K, mode, P.stream));
  return 0;
}

int gemm_plain(Program& P, const Buf& a, const ApcMatrix& w, const Buf& out, bool accumulate) {
  const int M = a.rows, K = a.cols, N = w.N;
  if (w.K != K || out.rows != M || out.cols != N || (accumulate && out.dtype != APC_DT_F32)) return -1;
  for (long r0 = 0; r0 < M; r0 += 1L << 21) {  // grid.y limit of the kernel: 65535 tiles of 64 rows
    const int n = (int)std::min((long)(1L << 21), (long)M - r0);
    LAUNCH(P, "gemm_plain",
           apc_gemm_plain((const char*)a.p + (size_t)r0 * a.ld * elem_size(a.dtype), a.dtype, a.ld, w.data, w.dtype, w.ld,
                          (char*)out.p + (size_t)r0 * out.ld * elem_size(out.dtype), out.dtype, out.ld, n, N, K,
                          accumulate ? 1 : 0, P.stream));
  }
  return 0;
}

// residual += a . w^T leaving the row for the norm with weight g; returns 1 if done (emit filled), 0 if no kernel
// takes these sizes (nothing done), < 0 on error
int gemm_emit_bf16(Program& P, const Buf& a, const ApcMatrix& w, const Buf& residual, Emit& emit) {
  const int M = a.rows, K = a.cols, N = w.N;
  if (!act_ok(a) || residual.dtype != APC_DT_F32 || !emit.g) return 0;
  if (w.K != K || residual.rows != M || residual.cols != N) return -1;
  if (M > MANY_ROWS_SPLIT_MAX) {
    const int parts = apc_gemm_direct_emit_parts(a.p, a.ld, residual.p, residual.ld, M, N, K);
    if (!parts) return 0;
    emit.raw = P.emit_rows(emit, M, N);
    emit.ss = (float*)P.emit_take(emit, sizeof(float) * (size_t)M * parts);
    emit.ss_rows = M;
    emit.ss_cols = parts;
    const int ks = apc_gemm_direct_k_split(M, N, K);
    float* ws = ks > 1 ? P.floats((size_t)ks * M * N) : nullptr;
    LAUNCH(P, "gemm_direct_emit_bf16",
           apc_gemm_direct_emit_bf16(a.p, a.ld, w.data, (float*)residual.p, residual.ld, M, N, K, emit.g, emit.raw.p, N,
                                     emit.ss, parts, ws, P.stream));
    emit.filled = true;
    return 1;
  }
  if (M > SKINNY_MAX_ROWS) {
    const int ks = tiled_k_split(M, N, K);
    if (ks == 1) return 0;
    emit.raw = P.emit_rows(emit, M, N);
    emit.ss_rows = M;
    emit.ss_cols = (int)cdiv(N, 256);
    emit.ss = (float*)P.emit_take(emit, sizeof(float) * (size_t)M * emit.ss_cols);
    float* ws = P.floats((size_t)ks * M * N);
    LAUNCH(P, "gemm_splitk_emit_bf16",
           apc_gemm_splitk_emit_bf16(a.p, a.ld, w.data, residual.p, residual.ld, M, N, K, ks, ws, emit.g, emit.raw.p, N,
                                     emit.ss, P.stream));
    emit.filled = true;
    return 1;
  }
  emit.raw = P.emit_rows(emit, M, N);
  emit.ss_rows = 16;
  emit.ss_cols = (int)cdiv(cdiv(N, 16), 4) * 4;
  emit.ss = (float*)P.emit_take(emit, sizeof(float) * (size_t)16 * emit.ss_cols);
  LAUNCH(P, "skinny_gemm_emit_bf16",
         apc_skinny_gemm_emit_bf16(a.p, a.ld, w.data, residual.p, residual.ld, M, N, K, emit.g, emit.raw.p, N, emit.ss,
                                   P.stream));
  emit.filled = true;
  return 1;
}

int linear(Program& P, const Buf& a, const ApcMatrix& w, const Buf& out, bool accumulate, Emit* emit) {
  if (w.packed) {
    if (emit && accumulate) {
      const int rc = gemm_emit_bf16(P, a, w, out, *emit);
      if (rc) return rc < 0 ? rc : 0;
    }
    return gemm_bf16(P, a, w, out, accumulate);
  }
  return gemm_plain(P, a, w, out, accumulate);
}

bool pre_ok_skinny(const Emit& e, int K) {
  return e.raw.rows <= SKINNY_MAX_ROWS && act_ok(e.raw) && e.ss_rows == 16 && e.ss_cols == (int)cdiv(cdiv(K, 16), 4) * 4;
}

// the storing products on a row that a product into the residual left, more than 16 rows; 1 done, 0 not taken
int pre_tiled(Program& P, const Emit& e, const ApcMatrix& w, const ApcMatrix* wu, const Buf& out, int n_cols, int mode) {
  const int M = e.raw.rows, K = e.raw.cols;
  if (!(M > SKINNY_MAX_ROWS && act_ok(e.raw) && e.ss_rows == M && e.ss_cols >= 1 && e.ss_cols <= 256)) return 0;
  const int n_mats = wu ? 2 : 1;
  const int ks = tiled_k_split(M, n_cols * n_mats, K);
  if (ks == 1) {
    LAUNCH(P, "gemm_pre_bf16",
           apc_gemm_pre_bf16(e.raw.p, e.raw.ld, e.ss, e.ss_cols, e.eps, w.data, wu ? wu->data : nullptr, out.p, out.ld, M,
                             n_cols, K, mode, P.stream));
    return 1;
  }
  float* ws = P.floats((size_t)n_mats * ks * M * n_cols);
  LAUNCH(P, "gemm_splitk_pre_bf16",
         apc_gemm_splitk_pre_bf16(e.raw.p, e.raw.ld, e.ss, e.ss_cols, e.eps, w.data, wu ? wu->data : nullptr, out.p,
                                  out.ld, M, n_cols, K, mode, ks, ws, P.stream));
  return 1;
}

int linear_pre(Program& P, const Emit& e, const ApcMatrix& w, const Buf& out) {  // 1 done, 0 not taken
  if (!w.packed || P.tun.force_plain) return 0;
  const int M = e.raw.rows, K = e.raw.cols;
  if (w.K != K || out.rows != M || out.cols != w.N) return -1;
  const int mode = out.dtype == APC_DT_BF16 ? 0 : 1;
  if (M > SKINNY_MAX_ROWS) return pre_tiled(P, e, w, nullptr, out, w.N, mode);
  if (!pre_ok_skinny(e, K)) return 0;
  LAUNCH(P, "skinny_gemm_pre_bf16",
         apc_skinny_gemm_pre_bf16(e.raw.p, e.raw.ld, e.ss, (int)cdiv(K, 16), e.eps, w.data, out.p, out.ld, M, w.N, K, mode,
                                  P.stream));
  return 1;
}

int swiglu_pre(Program& P, const Emit& e, const ApcLayer& L, const Buf& out) {  // 1 done, 0 not taken
  if (!L.w_gate.packed || P.tun.force_plain || out.dtype != APC_DT_BF16) return 0;
  const int M = e.raw.rows, K = e.raw.cols, F = out.cols;
  if (L.w_gate.N != F || L.w_gate.K != K || out.rows != M) return -1;
  if (M > SKINNY_MAX_ROWS) return pre_tiled(P, e, L.w_gate, &L.w_up, out, F, 3);
  if (!pre_ok_skinny(e, K)) return 0;
  LAUNCH(P, "skinny_swiglu_pre_bf16",
         apc_skinny_swiglu_pre_bf16(e.raw.p, e.raw.ld, e.ss, (int)cdiv(K, 16), e.eps, L.w_gate.data, L.w_up.data, out.p,
                                    out.ld, M, F, K, P.stream));
  return 1;
}

int swiglu(Program& P, const Buf& h, const ApcLayer& L, const Buf& out) {
  const int M = h.rows, K = h.cols, F = out.cols;
  if (L.w_gate.packed) {
    if (!act_ok(h) || out.dtype != APC_DT_BF16 || L.w_gate.K != K || L.w_gate.N != F) return -1;
    const int ks = M > SKINNY_MAX_ROWS ? tiled_k_split(M, 2 * F, K) : 1;
    if (ks > 1) {
      float* ws = P.floats((size_t)2 * ks * M * F);
      LAUNCH(P, "gemm_splitk_bf16 (swiglu)",
             apc_gemm_splitk_bf16(h.p, h.ld, L.w_gate.data, L.w_up.data, out.p, out.ld, M, F, K, 3, ks, ws, P.stream));
      return 0;
    }
    if (M <= SKINNY_MAX_ROWS)
      LAUNCH(P, "skinny_swiglu_bf16",
             apc_skinny_swiglu_bf16(h.p, h.ld, L.w_gate.data, L.w_up.data, out.p, out.ld, M, F, K, P.stream));
    else
      LAUNCH(P, "gemm_swiglu_bf16",
             apc_gemm_swiglu_bf16(h.p, h.ld, L.w_gate.data, L.w_up.data, out.p, out.ld, M, F, K, P.stream));
    return 0;
  }
  Buf gu = P.rows(M, 2 * F, h.dtype == APC_DT_F32 ? APC_DT_F32 : out.dtype);
  int rc = gemm_plain(P, h, L.w_gate, gu, false);
  if (rc) return rc;
  for (long r0 = 0; r0 < M; r0 += 32768) {
    const int n = (int)std::min(32768L, (long)M - r0);
    LAUNCH(P, "silu_mul",
           apc_silu_mul((const char*)gu.p + (size_t)r0 * gu.ld * elem_size(gu.dtype), gu.dtype, gu.ld,
                        (char*)out.p + (size_t)r0 * out.ld * elem_size(out.dtype), out.dtype, out.ld, n, F, P.stream));
  }
  return 0;
}

// ------------------------------------------------------------------------------------------------ a norm's input
// The normalised input of a part, not computed yet (parts/base.py: NormedInput).
struct Normed {
  const float* g;
  float eps;
  const Emit* pre;   // what the product before the norm left for it, or null
  Buf h;             // the normalised rows once computed
  bool have = false;
};

int normed_tensor(Program& P, Normed& n) {
  if (n.have) return 0;
  n.h = P.rows(P.x.rows, P.x.cols, P.run_dtype);
  LAUNCH(P, "rmsnorm_rows",
         apc_rmsnorm_rows(P.x.p, APC_DT_F32, P.x.ld, nullptr, n.g, n.eps, n.h.p, n.h.dtype, n.h.ld, P.x.rows, P.x.cols,
                          P.stream));
  n.have = true;
  return 0;
}

int normed_linear(Program& P, Normed& n, const ApcMatrix& w, const Buf& out) {
  if (n.pre && !n.have) {
    const int rc = linear_pre(P, *n.pre, w, out);
    if (rc) return rc < 0 ? rc : 0;
  }
  const int rc = normed_tensor(P, n);
  if (rc) return rc;
  return linear(P, n.h, w, out, false, nullptr);
}

// ------------------------------------------------------------------------------------------------ attention
// q, k, v in one product that rotates whole heads and fills the pages; 1 done, 0 not taken
int qkv_rope(Program& P, const Buf& a, const Emit* pre, const ApcLayer& L, const Buf& qkv, const ApcPlanEntry& E) {
  if (!L.w_qkv.packed || P.tun.force_plain) return 0;
  const int M = a.rows, K = a.cols, H = L.H, Hk = L.Hk, d = L.d, N = (H + 2 * Hk) * d;
  const bool few = M <= SKINNY_MAX_ROWS;
  if (!(act_ok(a) && qkv.dtype == APC_DT_BF16 && E.kv_dtype == APC_DT_BF16)) return 0;
  if (few && !(d % 32 == 0 && qkv.ld % 4 == 0 && ((uintptr_t)qkv.p & 7u) == 0)) return 0;
  const int ks = few ? 1 : tiled_k_split(M, N, K);
  if (!few && (ks == 1 || 256 % d || d % 2)) return 0;
  if (pre) {
    if (few && !pre_ok_skinny(*pre, K)) return 0;
    if (!few && !(pre->ss_rows == M && pre->ss_cols >= 1 && pre->ss_cols <= 256)) return 0;
  }
  if (L.w_qkv.K != K || L.w_qkv.N != N || qkv.rows != M || qkv.cols < H * d) return -1;
  const ApcStep& s = P.step;
  const int* table = s.table[E.group];
  const int width = s.table_width[E.group];
  if (few) {
    LAUNCH(P, "skinny_qkv_rope_bf16",
           apc_skinny_qkv_rope_bf16(a.p, a.ld, pre ? pre->ss : nullptr, pre ? (int)cdiv(K, 16) : 0, pre ? pre->eps : 0.f,
                                    L.w_qkv.data, qkv.p, qkv.ld, M, K, H, Hk, d, L.cos_sin, s.positions,
                                    s.row_seg, table, width, E.kv, E.page_tokens, P.stream));
    return 1;
  }
  float* ws = P.floats((size_t)ks * M * N);
  LAUNCH(P, "gemm_splitk_qkv_rope_bf16",
         apc_gemm_splitk_qkv_rope_bf16(a.p, a.ld, pre ? pre->ss : nullptr, pre ? pre->ss_cols : 0, pre ? pre->eps : 0.f,
                                       L.w_qkv.data, qkv.p, qkv.ld, M, K, H, Hk, d, L.cos_sin, s.positions,
                                       s.row_seg, table, width, E.kv, E.page_tokens, ks, ws, P.stream));
  return 1;
}

int rope_kv_write(Program& P, const Buf& qkv, const ApcLayer& L, const ApcPlanEntry& E, bool write) {
  const int H = L.H, Hk = L.Hk, d = L.d, q_off = 0, k_off = H * d, v_off = (H + Hk) * d;
  const ApcStep& s = P.step;
  const int* table = s.table[E.group];
  const int width = s.table_width[E.group];
  void* cache = write ? E.kv : nullptr;
  if (!P.tun.force_plain && qkv.dtype == APC_DT_BF16 && (!write || E.kv_dtype == APC_DT_BF16) && d % 8 == 0 &&
      L.rot % 16 == 0 && qkv.ld % 8 == 0 && k_off % 8 == 0 && v_off % 8 == 0 && ((uintptr_t)qkv.p & 15u) == 0) {
    LAUNCH(P, "rope_kv_write_bf16",
           apc_rope_kv_write_bf16(qkv.p, qkv.ld, q_off, k_off, v_off, qkv.rows, H, Hk, d, L.rot, L.rot ? L.cos_sin : nullptr,
                                  s.positions, s.row_seg, table, width, cache, E.page_tokens, P.stream));
    return 0;
  }
  LAUNCH(P, "rope_kv_write",
         apc_rope_kv_write(qkv.p, qkv.dtype, qkv.ld, q_off, k_off, v_off, qkv.rows, H, Hk, d, L.rot,
                           L.rot ? L.cos_sin : nullptr, s.positions, s.row_seg, table, width, cache,
                           write ? E.kv_dtype : 0, E.page_tokens, P.stream));
  return 0;
}

// attention of the whole step on the MFMA kernels; 1 done, 0 sizes they do not take
int attention_bf16(Program& P, const Buf& q, const Buf& out, const ApcLayer& L, const ApcPlanEntry& E) {
  const ApcStep& s = P.step;
  const int H = L.H, Hk = L.Hk, d = L.d, page = E.page_tokens, T = q.rows, window = L.window;
  if (L.scale != 0.f && !(L.scale > 0.f)) return 0;
  if (d % 16 || d > 256 || page % 8 || q.ld % 8 || ((uintptr_t)q.p & 15u) || ((uintptr_t)E.kv & 15u)) return 0;
  const float sc = L.scale != 0.f ? L.scale : 1.0f / std::sqrt((float)d);
  const int* table = s.table[E.group];
  const int width = s.table_width[E.group];
  if (s.n_tiles) {
    const bool wide = P.tun.wide_tiles && apc_attention_prefill_wide_takes(d, page, s.n_tiles, T - s.n_decode);
    const int splits = wide
                           ? key_splits(s.n_tiles, H, s.max_prompt_keys, window, P.tun.key_splits_max,
                                        std::max(1, P.tun.key_range_min))
                           : 1;
    float* parts = splits > 1 ? P.floats((size_t)splits * T * H * (d + 2)) : nullptr;
    LAUNCH(P, "attention_prefill_bf16",
           apc_attention_prefill_bf16(q.p, q.ld, 0, out.p, out.ld, H, Hk, d, E.kv, page, table, width,
                                      s.positions, s.row_seg, s.tile_row0, s.tile_rows,
                                      s.n_tiles, P.tun.wide_tiles ? T - s.n_decode : 0, window, sc, splits, T, parts,
                                      P.stream));
  }
  if (s.n_decode) {
    const int n = s.n_decode;
    const int span = window ? std::min(s.max_decode_context, window) : s.max_decode_context;
    const int* rows = s.all_rows_decode ? nullptr : s.decode_rows;
    const long pairs = (long)n * Hk * cdiv(H / Hk, 16);
    const int n_parts = decode_parts(pairs, span);
    // (rows so short that one block's waves take a pair's ranges need no partial results either)
    if ((pairs >= P.tun.whole_min_pairs || n_parts <= WHOLE_WAVES) && apc_attention_decode_whole_fits(H, Hk, d)) {
      // no length of the ranges: every row's own keys, one range a wave of its block
      LAUNCH(P, "attention_decode_bf16 (whole)",
             apc_attention_decode_bf16(q.p, q.ld, 0, out.p, out.ld, n, H, Hk, d, E.kv, page, table, width,
                                       s.positions, s.row_seg, rows, window, sc, 0, 0, nullptr, nullptr,
                                       P.stream));
      return 1;
    }
    const int kw = 0;  // every row's own keys in n_parts ranges
    if (P.tun.last_block_merges && pairs <= P.pair_capacity && apc_attention_decode_last_fits(H, Hk, d, n_parts)) {
      const int nz = (int)cdiv(n_parts, WHOLE_WAVES);
      float* ws = P.floats((size_t)n * H * nz * (d + 2));
      LAUNCH(P, "attention_decode_bf16 (last block merges)",
             apc_attention_decode_bf16(q.p, q.ld, 0, out.p, out.ld, n, H, Hk, d, E.kv, page, table, width,
                                       s.positions, s.row_seg, rows, window, sc, kw, n_parts, ws,
                                       P.pair_counters, P.stream));
      return 1;
    }
    float* ws = P.floats((size_t)n * H * n_parts * (d + 2));
    LAUNCH(P, "attention_decode_bf16",
           apc_attention_decode_bf16(q.p, q.ld, 0, out.p, out.ld, n, H, Hk, d, E.kv, page, table, width,
                                     s.positions, s.row_seg, rows, window, sc, kw, n_parts, ws, nullptr,
                                     P.stream));
  }
  return 1;
}

int attention(Program& P, const Buf& qkv, const Buf& out, const ApcLayer& L, const ApcPlanEntry& E) {
  if (!P.tun.force_plain && qkv.dtype == APC_DT_BF16 && E.kv_dtype == APC_DT_BF16 && out.dtype == APC_DT_BF16) {
    const int rc = attention_bf16(P, qkv, out, L, E);
    if (rc) return rc < 0 ? rc : 0;
  }
  const ApcStep& s = P.step;
  if (L.d > 256) return -2;
  const float sc = L.scale != 0.f ? L.scale : 1.0f / std::sqrt((float)L.d);
  LAUNCH(P, "paged_attention_plain",
         apc_paged_attention_plain(qkv.p, qkv.dtype, qkv.ld, 0, out.p, out.dtype, out.ld, qkv.rows, L.H, L.Hk, L.d, E.kv,
                                   E.kv_dtype, E.page_tokens, s.table[E.group], s.table_width[E.group],
                                   s.positions, s.row_seg, L.window, sc, P.stream));
  return 0;
}

// ------------------------------------------------------------------------------------------------ a layer
// x += attention(norm1(x)); x += swiglu(norm2(x)).  `pre`: what the entry before left for norm1 (or unfilled);
// `next_g`: the weight of the norm that reads x after this entry (null: none); what is left for it goes to `out`.
int run_layer(Program& P, const ApcLayer& L, const ApcPlanEntry& E, const Emit& pre, const float* next_g, float next_eps,
              Emit& out) {
  const int T = P.x.rows;
  // ---- mixer
  Normed h1{L.norm1_w, L.norm1_eps, (pre.filled && pre.g == L.norm1_w) ? &pre : nullptr, Buf{}, false};
  Emit mid;
  mid.g = L.norm2_w;
  mid.eps = L.norm2_eps;
  Buf qkv = P.rows(T, (L.H + 2 * L.Hk) * L.d, P.run_dtype);
  bool fused = false;
  if (E.writes && L.rot == L.d && L.rot > 0) {
    int rc;
    if (h1.pre) {
      rc = qkv_rope(P, h1.pre->raw, h1.pre, L, qkv, E);
    } else {
      rc = normed_tensor(P, h1);
      if (rc) return rc;
      rc = qkv_rope(P, h1.h, nullptr, L, qkv, E);
    }
    if (rc < 0) return rc;
    fused = rc == 1;
  }
  if (!fused) {
    int rc = normed_linear(P, h1, L.w_qkv, qkv);
    if (rc) return rc;
    if (E.writes || L.rot) {
      rc = rope_kv_write(P, qkv, L, E, E.writes != 0);
      if (rc) return rc;
    }
  }
  Buf att = P.rows(T, L.H * L.d, P.run_dtype);
  int rc = attention(P, qkv, att, L, E);
  if (rc) return rc;
  rc = linear(P, att, L.w_o, P.x, true, &mid);
  if (rc) return rc;
  // ---- feed-forward
  Normed h2{L.norm2_w, L.norm2_eps, mid.filled ? &mid : nullptr, Buf{}, false};
  char* const out_slot = out.slot;
  out = Emit{};
  out.slot = out_slot;
  out.g = next_g;
  out.eps = next_eps;
  Buf act = P.rows(T, L.F, P.run_dtype);
  bool done = false;
  if (h2.pre) {
    rc = swiglu_pre(P, *h2.pre, L, act);
    if (rc < 0) return rc;
    done = rc == 1;
  }
  if (!done) {
    rc = normed_tensor(P, h2);
    if (rc) return rc;
    rc = swiglu(P, h2.h, L, act);
    if (rc) return rc;
  }
  return linear(P, act, L.w_down, P.x, true, next_g ? &out : nullptr);
}

int begin_step(Program& P, const ApcStep* step, void* arena, size_t bytes, hipStream_t stream, bool dry) {
  P.step = *step;
  P.dry = dry;
  // a sizing run walks the same addresses from a made-up base, so that what depends on alignment decides alike
  P.arena = dry ? (char*)(uintptr_t)(1u << 20) : (char*)arena;
  P.cap = bytes;
  P.at = 0;
  P.peak = 0;
  P.overflow = false;
  P.stream = stream;
  P.left = Emit{};
  P.begun = true;
  if (!dry && (((uintptr_t)arena & 255u) != 0)) return -1;
  if (step->n_groups < 0 || step->n_groups > 8 || step->T <= 0) return -1;
  P.x = P.rows(step->T, P.D, APC_DT_F32);
  {
    const size_t rows = (size_t)std::max(step->T, 16);
    P.slot_cap = (((size_t)step->T * P.D * 2 + 255) & ~(size_t)255) +
                 rows * (size_t)std::max(256L, cdiv(P.D, 16) + 4) * sizeof(float);
    P.slot[0] = (char*)P.take(P.slot_cap);
    P.slot[1] = (char*)P.take(P.slot_cap);
    P.scratch_mark = P.at;
  }
  if (P.embedding.packed)
    LAUNCH(P, "embed_rows_tiled",
           apc_embed_rows_tiled(P.embedding.data, P.embedding.chunks, step->tokens, P.x.p, APC_DT_F32, step->T, P.D,
                                P.x.ld, stream));
  else
    LAUNCH(P, "embed_rows",
           apc_embed_rows(P.embedding.data, P.embedding.dtype, step->tokens, P.x.p, APC_DT_F32, step->T, P.D, P.x.ld,
                          stream));
  return 0;
}

int run_range(Program& P, int lo, int hi) {
  if (!P.begun) return APC_HOST_ERR_STATE;
  const int n = (int)P.plan.size();
  if (lo < 0 || hi > n || lo > hi) return -1;
  for (int i = lo; i < hi; ++i) {
    const ApcPlanEntry& E = P.plan[i];
    const ApcLayer& L = P.layers[E.layer];
    const ApcLayer* nxt = i + 1 < n ? &P.layers[P.plan[i + 1].layer] : nullptr;
    Emit out;
    out.slot = P.slot[i & 1];
    const Emit pre = P.left;
    P.at = P.scratch_mark;
    const int rc = run_layer(P, L, E, pre, nxt ? nxt->norm1_w : nullptr, nxt ? nxt->norm1_eps : 0.f, out);
    if (rc) return rc;
    P.left = out.filled ? out : Emit{};
  }
  return 0;
}

int finish_step(Program& P, float* logits) {
  if (!P.begun) return APC_HOST_ERR_STATE;
  const ApcStep& s = P.step;
  P.begun = false;
  if (s.R <= 0) return P.overflow ? APC_HOST_ERR_ARENA : 0;
  P.at = P.scratch_mark;
  Buf h = P.rows(s.R, P.D, P.run_dtype);
  LAUNCH(P, "rmsnorm_rows (wanted rows)",
         apc_rmsnorm_rows(P.x.p, APC_DT_F32, P.x.ld, s.logit_rows, P.final_norm_w, P.final_norm_eps, h.p, h.dtype,
                          h.ld, s.R, P.D, P.stream));
  Buf out;
  out.p = logits;
  out.dtype = APC_DT_F32;
  out.rows = s.R;
  out.cols = P.V;
  out.ld = P.V;
  const int rc = linear(P, h, P.head, out, false, nullptr);
  if (rc) return rc;
  return P.overflow ? APC_HOST_ERR_ARENA : 0;
}

}  // namespace

// ==================================================================================================== interface
APC_HOST_EXPORT void* apc_host_program_new(int hidden, int vocab, int run_dtype, const ApcMatrix* embedding,
                                           const float* final_norm_w, float final_norm_eps, const ApcMatrix* head) {
  if (hidden <= 0 || vocab <= 0 || !embedding || !head || !final_norm_w) return nullptr;
  Program* p = new Program();
  p->D = hidden;
  p->V = vocab;
  p->run_dtype = run_dtype;
  p->embedding = *embedding;
  p->head = *head;
  p->final_norm_w = final_norm_w;
  p->final_norm_eps = final_norm_eps;
  return p;
}

APC_HOST_EXPORT void apc_host_program_free(void* prog) { delete (Program*)prog; }

APC_HOST_EXPORT int apc_host_program_add_layer(void* prog, const ApcLayer* layer) {
  Program& P = *(Program*)prog;
  if (!layer || layer->H <= 0 || layer->Hk <= 0 || layer->H % layer->Hk || layer->d <= 0 || layer->F <= 0) return -1;
  if (layer->rot && !layer->cos_sin) return -1;
  P.layers.push_back(*layer);
  return (int)P.layers.size() - 1;
}

APC_HOST_EXPORT int apc_host_program_add_entry(void* prog, const ApcPlanEntry* entry) {
  Program& P = *(Program*)prog;
  if (!entry || entry->layer < 0 || entry->layer >= (int)P.layers.size() || !entry->kv || entry->group < 0 ||
      entry->group >= 8 || entry->page_tokens <= 0)
    return -1;
  P.plan.push_back(*entry);
  return (int)P.plan.size() - 1;
}

APC_HOST_EXPORT void apc_host_program_tunables(void* prog, const ApcTunables* t, int* pair_counters, int pair_capacity) {
  Program& P = *(Program*)prog;
  if (t) P.tun = *t;
  P.pair_counters = pair_counters;
  P.pair_capacity = pair_counters ? pair_capacity : 0;
}

// Bytes of work space that the step needs (entries lo .. hi-1 of the plan and, with `with_logits`, the head).
APC_HOST_EXPORT long long apc_host_step_bytes(void* prog, const ApcStep* step) {
  Program& P = *(Program*)prog;
  int rc = begin_step(P, step, nullptr, 0, nullptr, true);
  if (!rc) rc = run_range(P, 0, (int)P.plan.size());
  if (!rc) rc = finish_step(P, nullptr);
  P.begun = false;
  if (rc) return rc;
  return (long long)((P.peak + 255) & ~(size_t)255);
}

// A step in up to three calls (a caller that records it into more than one graph makes them separately):
// begin (embedding), ranges of plan entries in order, finish (final norm and head on the wanted rows into `logits`,
// float32 [R, vocab]).  The work space must stay as it is until the step's kernels have run.
APC_HOST_EXPORT int apc_host_step_begin(void* prog, const ApcStep* step, void* arena, size_t arena_bytes,
                                        hipStream_t stream) {
  return begin_step(*(Program*)prog, step, arena, arena_bytes, stream, false);
}
APC_HOST_EXPORT int apc_host_step_range(void* prog, int lo, int hi) { return run_range(*(Program*)prog, lo, hi); }
APC_HOST_EXPORT int apc_host_step_finish(void* prog, float* logits) { return finish_step(*(Program*)prog, logits); }

// The whole step in one call.
APC_HOST_EXPORT int apc_host_step(void* prog, const ApcStep* step, void* arena, size_t arena_bytes, float* logits,
                                  hipStream_t stream) {
  Program& P = *(Program*)prog;
  int rc = begin_step(P, step, arena, arena_bytes, stream, false);
  if (!rc) rc = run_range(P, 0, (int)P.plan.size());
  if (!rc) rc = finish_step(P, logits);
  P.begun = false;
  return rc;
}

// Where the residual stream of the step in work (or of the last one) lies in the work space, in bytes.
APC_HOST_EXPORT long long apc_host_residual_offset(void* prog) {
  Program& P = *(Program*)prog;
  return (long long)((char*)P.x.p - P.arena);
}

// Per-launch timers: on, every launch is bracketed by events; the report is one line a launch, "name<TAB>microseconds",
// in launch order, and waits for the GPU.
APC_HOST_EXPORT void apc_host_timing(void* prog, int on) {
  Program& P = *(Program*)prog;
  P.timing = on != 0;
  for (auto& t : P.timed) {
    hipEventDestroy(t.e0);
    hipEventDestroy(t.e1);
  }
  P.timed.clear();
}
APC_HOST_EXPORT const char* apc_host_timing_report(void* prog) {
  Program& P = *(Program*)prog;
  P.report.clear();
  for (auto& t : P.timed) {
    hipEventSynchronize(t.e1);
    float ms = 0.f;
    hipEventElapsedTime(&ms, t.e0, t.e1);
    P.report += t.name;
    P.report += '\t';
    P.report += std::to_string(ms * 1000.0f);
    P.report += '\n';
  }
  return P.report.c_str();
}

// ---- the rules, for tests that hold them against the Python wrappers' own
APC_HOST_EXPORT int apc_host_rule_tiled_k_split(int M, int N, int K) { return apc_rules::tiled_k_split(M, N, K); }
APC_HOST_EXPORT int apc_host_rule_decode_parts(long long pairs, int span) {
  return apc_rules::decode_parts((long)pairs, span);
}
APC_HOST_EXPORT int apc_host_rule_key_splits(int n_tiles, int n_heads, int keys, int window, int splits_max,
                                             int range_min) {
  return apc_rules::key_splits(n_tiles, n_heads, keys, window, splits_max, std::max(1, range_min));
}
