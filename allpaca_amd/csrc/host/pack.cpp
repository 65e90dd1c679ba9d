// The step packer: a step's entries (request, its next tokens, the wanted places among them) checked against the
// cache manager's books, their pages taken (for all or for none), and the batch's description written as the
// kernels read it: one int32 buffer, laid out as allpaca_amd/engine/batch.py::StepLayout says (tokens, positions,
// row_seg, seg_row0, seg_rows, seg_pos0, state_slots, logit_rows, decode_rows, tile_row0, tile_rows, then one block
// table [segments][width] per paged group).  The caller copies the buffer to the device.
// The reference describes a batch as tokens plus {start_pos, n_rows, page_ids} per sequence
// (crates/allpaca-core/src/model.rs:36-42, 10865-10885).
#include "cache.h"

#include <algorithm>
#include <unordered_set>

using namespace apc_host;

extern "C" {

// What is wrong with a step (apc_step_prepare): the first finding, in the order the entries are given.
enum {
  APC_STEP_OK = 0,
  APC_STEP_TWICE = 1,          // entry `entry` names a request that an earlier entry names
  APC_STEP_NOT_ADMITTED = 2,
  APC_STEP_NO_TOKENS = 3,
  APC_STEP_TOKEN_RANGE = 4,    // `value`: the token
  APC_STEP_WANT_RANGE = 5,     // `value`: the wanted place
  APC_STEP_POSITION = 6,       // `value`: the position beyond the run's limit
  APC_STEP_OUT_OF_PAGES = 7,   // `entry`: the paged group, `value`: pages needed, `extra`: pages free
};
struct ApcStepFinding {
  int what, entry, value, extra;
};

// Where the arrays lie in the packed buffer (offsets in ints) and what the host keeps of the step.
struct ApcPacked {
  int T, S, R, n_decode, n_tiles, total;
  int off[11];                 // the arrays in the order above
  int n_groups;
  int table_off[APC_MAX_GROUPS], table_width[APC_MAX_GROUPS];
  int max_decode_context, max_prompt_keys, max_context, max_rows;
};

}  // extern "C"

// Checks the entries and takes the pages their tokens need, for all requests or for none.
APC_HOST_EXPORT int apc_step_prepare(void* cache, int vocab, int max_positions, int n, const long long* ids,
                                     const int* n_tokens, const int* tokens, const int* n_want, const int* wants,
                                     ApcStepFinding* finding) {
  Cache& C = *(Cache*)cache;
  ApcStepFinding f{APC_STEP_OK, 0, 0, 0};
  std::unordered_set<long long> seen;
  int need_all[APC_MAX_GROUPS] = {0};
  int tok_at = 0, want_at = 0;
  for (int e = 0; e < n && !f.what; ++e) {
    f.entry = e;
    const int nt = n_tokens[e];
    const Seq* s = C.find(ids[e]);
    if (!seen.insert(ids[e]).second) f.what = APC_STEP_TWICE;
    else if (!s) f.what = APC_STEP_NOT_ADMITTED;
    else if (nt <= 0) f.what = APC_STEP_NO_TOKENS;
    for (int i = 0; i < nt && !f.what; ++i)
      if (tokens[tok_at + i] < 0 || tokens[tok_at + i] >= vocab) {
        f.what = APC_STEP_TOKEN_RANGE;
        f.value = tokens[tok_at + i];
      }
    for (int i = 0; i < n_want[e] && !f.what; ++i)
      if (wants[want_at + i] < 0 || wants[want_at + i] >= nt) {
        f.what = APC_STEP_WANT_RANGE;
        f.value = wants[want_at + i];
      }
    if (!f.what && s->length + nt > max_positions) {
      f.what = APC_STEP_POSITION;
      f.value = s->length + nt - 1;
    }
    if (!f.what) {
      int need[APC_MAX_GROUPS];
      C.pages_needed(*s, nt, need);
      for (size_t g = 0; g < C.pools.size(); ++g) need_all[g] += need[g];
    }
    tok_at += std::max(nt, 0);
    want_at += n_want[e];
  }
  for (size_t g = 0; g < C.pools.size() && !f.what; ++g)
    if (need_all[g] > C.pools[g].free_count()) {
      f.what = APC_STEP_OUT_OF_PAGES;
      f.entry = (int)g;
      f.value = need_all[g];
      f.extra = C.pools[g].free_count();
    }
  if (finding) *finding = f;
  if (f.what) return f.what;
  for (int e = 0; e < n; ++e) {
    const int rc = C.reserve(ids[e], n_tokens[e]);
    if (rc) return rc;
  }
  return 0;
}

APC_HOST_EXPORT int apc_step_commit(void* cache, int n, const long long* ids, const int* n_tokens) {
  Cache& C = *(Cache*)cache;
  for (int e = 0; e < n; ++e) {
    const int rc = C.commit(ids[e], n_tokens[e]);
    if (rc) return rc;
  }
  return 0;
}

// Ints the packed buffer of these entries takes (block tables as wide as the longest of the step, at least
// `min_blocks`); fills `p` but for what depends on the tokens.
static int layout(Cache& C, int n, const long long* ids, const int* n_tokens, const int* n_want, int tile_rows,
                  int min_blocks, ApcPacked& p) {
  p = ApcPacked{};
  p.S = n;
  p.n_groups = (int)C.pools.size();
  for (int g = 0; g < p.n_groups; ++g) p.table_width[g] = std::max(1, min_blocks);
  for (int e = 0; e < n; ++e) {
    const Seq* s = C.find(ids[e]);
    if (!s) return APC_CACHE_UNKNOWN;
    const int nt = n_tokens[e];
    p.T += nt;
    p.R += n_want[e];
    if (nt == 1) {
      ++p.n_decode;
      p.max_decode_context = std::max(p.max_decode_context, s->length + 1);
    } else {
      p.n_tiles += (nt + tile_rows - 1) / tile_rows;
      p.max_prompt_keys = std::max(p.max_prompt_keys, s->length + nt);
    }
    p.max_context = std::max(p.max_context, s->length + nt);
    p.max_rows = std::max(p.max_rows, nt);
    for (int g = 0; g < p.n_groups; ++g) p.table_width[g] = std::max(p.table_width[g], (int)s->tables[g].size());
  }
  const int sizes[11] = {p.T, p.T, p.T, p.S, p.S, p.S, p.S, p.R, p.n_decode, p.n_tiles, p.n_tiles};
  int at = 0;
  for (int i = 0; i < 11; ++i) {
    p.off[i] = at;
    at += sizes[i];
  }
  for (int g = 0; g < p.n_groups; ++g) {
    p.table_off[g] = at;
    at += p.S * p.table_width[g];
  }
  p.total = at;
  return 0;
}

APC_HOST_EXPORT int apc_pack_layout(void* cache, int n, const long long* ids, const int* n_tokens, const int* n_want,
                                    int tile_rows, int min_blocks, ApcPacked* packed) {
  if (tile_rows <= 0 || !packed) return -1;
  return layout(*(Cache*)cache, n, ids, n_tokens, n_want, tile_rows, min_blocks, *packed);
}

// Writes the step's description into `out` (`cap` ints; the pages of the step's tokens are taken already).
// `pad_pages[g]`: the spare page of group g, which stands for pages that a window has passed and fills the tables'
// unused ends.
APC_HOST_EXPORT int apc_pack_step(void* cache, int n, const long long* ids, const int* n_tokens, const int* tokens,
                                  const int* n_want, const int* wants, int tile_rows, int min_blocks,
                                  const int* pad_pages, int* out, int cap, ApcPacked* packed) {
  Cache& C = *(Cache*)cache;
  if (tile_rows <= 0 || !packed || !out) return -1;
  ApcPacked& p = *packed;
  const int rc = layout(C, n, ids, n_tokens, n_want, tile_rows, min_blocks, p);
  if (rc) return rc;
  if (p.total > cap) return APC_HOST_ERR_ARENA;
  int* tok = out + p.off[0];
  int* pos = out + p.off[1];
  int* row_seg = out + p.off[2];
  int* seg_row0 = out + p.off[3];
  int* seg_rows = out + p.off[4];
  int* seg_pos0 = out + p.off[5];
  int* slots = out + p.off[6];
  int* logit_rows = out + p.off[7];
  int* decode_rows = out + p.off[8];
  int* tile_row0 = out + p.off[9];
  int* tile_rows_out = out + p.off[10];
  int row = 0, want_at = 0, r = 0, nd = 0, ntile = 0;
  for (int e = 0; e < n; ++e) {
    const Seq& s = *C.find(ids[e]);
    const int nt = n_tokens[e];
    seg_row0[e] = row;
    seg_rows[e] = nt;
    seg_pos0[e] = s.length;
    slots[e] = s.slot;
    for (int i = 0; i < nt; ++i) {
      tok[row + i] = tokens[row + i];
      pos[row + i] = s.length + i;
      row_seg[row + i] = e;
    }
    for (int i = 0; i < n_want[e]; ++i) logit_rows[r++] = row + wants[want_at + i];
    want_at += n_want[e];
    if (nt == 1) {
      decode_rows[nd++] = row;
    } else {
      for (int a = 0; a < nt; a += tile_rows) {
        tile_row0[ntile] = row + a;
        tile_rows_out[ntile++] = std::min(tile_rows, nt - a);
      }
    }
    for (int g = 0; g < p.n_groups; ++g) {
      int* bt = out + p.table_off[g] + (size_t)e * p.table_width[g];
      const auto& t = s.tables[g];
      const int pad = pad_pages[g];
      for (int i = 0; i < p.table_width[g]; ++i) bt[i] = (i < (int)t.size() && t[i] >= 0) ? t[i] : pad;
    }
    row += nt;
  }
  return 0;
}
