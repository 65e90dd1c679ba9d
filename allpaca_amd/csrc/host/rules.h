// The rules by which a step's operations choose their kernels: how many slices of K, how many keys a wave, how many
// ranges of keys a tile.  The same rules as the Python wrappers of the kernels (allpaca_amd/kernels/tuned.py), where
// each is explained with what was measured; tests/test_dispatch_rules.py holds the two against each other.
#pragma once
#include <algorithm>
#include <cmath>

namespace apc_rules {

constexpr int SKINNY_MAX_ROWS = 16;
constexpr int SPLITK_MAX_ROWS = 128;
constexpr int MANY_ROWS_SPLIT_MAX = 1024;
constexpr int WHOLE_WAVES = 4;
constexpr int CHIP_UNITS = 256;     // compute units the rules below were measured on

inline long cdiv(long a, long b) { return (a + b - 1) / b; }

inline int k_split(int M, int N, int K) {  // 17..128 rows: about 240 blocks in all
  const long blocks = cdiv(N, 128) * cdiv(M, 128);
  const int s = (int)std::max(1L, std::min(12L, (long)std::nearbyint(240.0 / (double)blocks)));  // half to even
  return std::max(1, std::min(s, K / 256));
}

inline int k_split_many_rows(int M, int N, int K) {  // 129..1024 rows
  const long blocks = cdiv(N, 128) * cdiv(M, 128);
  int s;
  if (blocks <= 56) s = 5;
  else if (blocks <= 68) s = 4;
  else if (blocks <= 88) s = 3;
  else if (blocks <= 208 && !(blocks >= 150 && N > K)) s = 2;
  else s = 1;
  return std::max(1, std::min(s, K / 256));
}

inline int tiled_k_split(int M, int N, int K) {
  if (M <= SPLITK_MAX_ROWS) return k_split(M, N, K);
  return M <= MANY_ROWS_SPLIT_MAX ? k_split_many_rows(M, N, K) : 1;
}

// ranges that the decode kernel cuts every row's keys into (the kernel sizes them from the row's own length)
inline int decode_parts(long pairs, int span) {
  const long per_pair = std::max(1L, (long)CHIP_UNITS / std::max(1L, pairs));
  return (int)std::max(1L, std::min((long)WHOLE_WAVES * per_pair, cdiv(span, 64)));
}

// ranges of keys that the 128-row attention kernel cuts every tile of a step into; `keys`: of the longest prompt
inline int key_splits(int n_tiles, int n_heads, int keys, int window, int splits_max, int range_min) {
  const long blocks = (long)n_tiles * n_heads;
  if (!splits_max || blocks <= 0 || keys <= 0) return 1;
  if (window) keys = std::min(keys, window + 128);
  const long few = std::min((long)keys / std::max(1, range_min / 2), (long)(CHIP_UNITS / 2) / blocks);
  const long s = std::min({(long)splits_max, (long)CHIP_UNITS / blocks, std::max((long)keys / range_min, few)});
  return (int)std::max(1L, s);
}

}  // namespace apc_rules
