// Token choice on the GPU: first-maximum argmax, and temperature / top-k / top-p
// sampling with a uniform number given per row.  Two ways to the same tokens: one block
// per row of logits (thresholds by bisection; needs no working memory), and, for rows as
// long as a real vocabulary, many blocks a row with thresholds by radix descent (second
// half of this file).
//
// Semantics follow crates/allpaca-core/src/sampling.rs:24-67, 215-331:
//   all logits non-finite -> token 0;  temperature <= 1e-5 -> argmax (first maximum);
//   else v = logit / max(T, 1e-5) for finite logits;  top-k keeps the k largest in
//   the order (v descending, id ascending);  top-p (0 <= p < 1) keeps the shortest
//   prefix of that order whose probability (over what top-k left) reaches p;
//   softmax over the survivors;  the draw walks r -= p_i until r <= 0, in sorted
//   order if top-k or top-p cut or sorted the list, else in id order.
// The random number is an input, so a token depends on (seed, request, position)
// only, never on the batch.
#include "common.h"
#include "no_alloc.h"
#include <math.h>
#include <mutex>

constexpr int SNT = 256;
constexpr int SMALL_MAX = 1024;  // survivors of top-k handled in LDS in the reference's own sequential order

__device__ __forceinline__ uint32_t key_of(float v) {  // monotone map; 0 is reserved for "not a candidate"
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float value_of(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
__device__ __forceinline__ bool finite_f(float v) { return fabsf(v) <= 3.402823466e+38f; }  // false for NaN, inf

struct Cut {  // the set { key > tau  or  (key == tau and id <= id_cut) }
  uint32_t tau;
  int id_cut;
};
__device__ __forceinline__ bool in_cut(const Cut& c, uint32_t key, int id) {
  return key > c.tau || (key == c.tau && id <= c.id_cut);
}

template <typename T>
__device__ __forceinline__ T block_sum_t(T v, T* smem) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  __syncthreads();
  if (threadIdx.x % WAVE == 0) smem[threadIdx.x / WAVE] = v;
  __syncthreads();
  T t = smem[0];
#pragma unroll
  for (int i = 1; i < SNT / WAVE; ++i) t += smem[i];
  return t;
}

struct RowView {
  const float* logits;
  int V;
  float inv_t;  // scaled value = logit / t, computed as a division to match the reference
  float t;
  __device__ __forceinline__ uint32_t key(int i) const {
    const float x = logits[i];
    return finite_f(x) ? key_of(x / t) : 0u;
  }
};

// number of elements of `set` with key >= trial
__device__ uint32_t count_ge(const RowView& rv, const Cut& set, uint32_t trial, uint32_t* smem) {
  uint32_t c = 0;
  for (int i = threadIdx.x; i < rv.V; i += SNT) {
    const uint32_t k = rv.key(i);
    c += (k != 0u && k >= trial && in_cut(set, k, i)) ? 1u : 0u;
  }
  return block_sum_t<uint32_t>(c, smem);
}
// number of elements of `set` with key == tau and id < id_trial
__device__ uint32_t count_eq_below(const RowView& rv, const Cut& set, uint32_t tau, int id_trial, uint32_t* smem) {
  uint32_t c = 0;
  for (int i = threadIdx.x; i < rv.V && i < id_trial; i += SNT) {
    const uint32_t k = rv.key(i);
    c += (k == tau && in_cut(set, k, i)) ? 1u : 0u;
  }
  return block_sum_t<uint32_t>(c, smem);
}
// mass = sum exp(v - vmax) over elements of `set` with key >= trial
__device__ float mass_ge(const RowView& rv, const Cut& set, uint32_t trial, float vmax, float* smem) {
  float s = 0.f;
  for (int i = threadIdx.x; i < rv.V; i += SNT) {
    const uint32_t k = rv.key(i);
    if (k != 0u && k >= trial && in_cut(set, k, i)) s += expf(value_of(k) - vmax);
  }
  return block_sum_t<float>(s, smem);
}

// the `need`-th (1-based) smallest id among elements of `set` with key == tau
__device__ int nth_tie(const RowView& rv, const Cut& set, uint32_t tau, uint32_t need, uint32_t* smem) {
  int id = 0;
  int top = 1;
  while (top < rv.V) top <<= 1;
  for (int bit = top; bit > 0; bit >>= 1) {
    const int trial = id | bit;
    if (count_eq_below(rv, set, tau, trial, smem) < need) id = trial;
  }
  return id;
}

// the k largest elements of `set` (|set| >= k >= 1) in (key desc, id asc) order
__device__ Cut select_by_count(const RowView& rv, const Cut& set, uint32_t k, uint32_t* smem) {
  uint32_t tau = 0;
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t trial = tau | (1u << bit);
    if (count_ge(rv, set, trial, smem) >= k) tau = trial;
  }
  const uint32_t c_ge = count_ge(rv, set, tau, smem);
  const uint32_t c_gt = (tau == 0xffffffffu) ? 0u : count_ge(rv, set, tau + 1u, smem);
  Cut out;
  out.tau = tau;
  if (c_ge <= k) { out.id_cut = set.tau == tau ? set.id_cut : 0x7fffffff; return out; }
  out.id_cut = nth_tie(rv, set, tau, k - c_gt, smem);
  return out;
}

// the shortest prefix of `set` in sorted order whose mass reaches `target`; *reached = false if none does
__device__ Cut select_by_mass(const RowView& rv, const Cut& set, float target, float vmax, bool* reached, float* fsm,
                              uint32_t* usm) {
  const uint32_t lowest = set.tau == 0u ? 1u : set.tau;
  if (!(mass_ge(rv, set, lowest, vmax, fsm) >= target)) { *reached = false; return set; }
  *reached = true;
  uint32_t tau = 0;
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t trial = tau | (1u << bit);
    const float ms = mass_ge(rv, set, trial, vmax, fsm);
    if (ms >= target && ms > 0.f) tau = trial;  // ms > 0 keeps tau on an element when target <= 0
  }
  if (tau < lowest) tau = lowest;
  const float m_gt = (tau == 0xffffffffu) ? 0.f : mass_ge(rv, set, tau + 1u, vmax, fsm);
  const uint32_t c_eq = count_ge(rv, set, tau, usm) - ((tau == 0xffffffffu) ? 0u : count_ge(rv, set, tau + 1u, usm));
  const float p_tau = expf(value_of(tau) - vmax);
  uint32_t need = 1;
  if (p_tau > 0.f) {
    const float n = ceilf((target - m_gt) / p_tau);
    need = n < 1.f ? 1u : (n > (float)c_eq ? c_eq : (uint32_t)n);
  }
  if (need < 1u) need = 1u;
  Cut out;
  out.tau = tau;
  out.id_cut = nth_tie(rv, set, tau, need, usm);
  return out;
}

__global__ __launch_bounds__(SNT) void argmax_rows_kernel(const float* __restrict__ logits, int ldl, int V,
                                                          int* __restrict__ out) {
  __shared__ float bv[SNT / WAVE];
  __shared__ int bi[SNT / WAVE];
  const float* row = logits + (size_t)blockIdx.x * ldl;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = threadIdx.x; i < V; i += SNT) {
    const float v = row[i];
    if (v > best) { best = v; best_i = i; }  // strict: the first maximum of this thread's ascending ids
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, WAVE);
    const int oi = __shfl_xor(best_i, o, WAVE);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  if (threadIdx.x % WAVE == 0) { bv[threadIdx.x / WAVE] = best; bi[threadIdx.x / WAVE] = best_i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SNT / WAVE; ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < best_i)) { best = bv[w]; best_i = bi[w]; }
    out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;  // nothing above -inf: token 0 (sampling.rs:215-225)
  }
}

// Wide rows are cut into pieces so that more than one block works on a row: a first pass leaves the first
// maximum of every piece (value, id), a second pass takes the first maximum of those.
__global__ __launch_bounds__(SNT) void argmax_pieces_kernel(const float* __restrict__ logits, int ldl, int V, int piece,
                                                            float* __restrict__ pv, int* __restrict__ pi) {
  __shared__ float bv[SNT / WAVE];
  __shared__ int bi[SNT / WAVE];
  const float* row = logits + (size_t)blockIdx.x * ldl;
  const int lo = blockIdx.y * piece, hi = min(V, lo + piece);
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += SNT) {
    const float v = row[i];
    if (v > best) { best = v; best_i = i; }
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, WAVE);
    const int oi = __shfl_xor(best_i, o, WAVE);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  if (threadIdx.x % WAVE == 0) { bv[threadIdx.x / WAVE] = best; bi[threadIdx.x / WAVE] = best_i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SNT / WAVE; ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < best_i)) { best = bv[w]; best_i = bi[w]; }
    pv[(size_t)blockIdx.x * gridDim.y + blockIdx.y] = best;
    pi[(size_t)blockIdx.x * gridDim.y + blockIdx.y] = best_i;
  }
}

__global__ __launch_bounds__(WAVE) void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                                            int pieces, int* __restrict__ out) {
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int p = threadIdx.x; p < pieces; p += WAVE) {
    const float v = pv[(size_t)blockIdx.x * pieces + p];
    const int i = pi[(size_t)blockIdx.x * pieces + p];
    if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, WAVE);
    const int oi = __shfl_xor(best_i, o, WAVE);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  if (threadIdx.x == 0) out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
}

// `scratch`: room for 2 * n_rows * 64 four-byte values, or null for the one-pass kernel
APC_EXPORT int apc_argmax_rows(const float* logits, int ldl, int n_rows, int V, int* out, void* scratch,
                               hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V <= 0 || ldl < V) return APC_ERR_BAD_ARG;
  if (!scratch || V < 8192 || n_rows > 65535) {
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(n_rows), dim3(SNT), 0, stream, logits, ldl, V, out);
    APC_LAUNCH_CHECK();
    return 0;
  }
  const int pieces = 64;
  const int piece = ceil_div(V, pieces);
  float* pv = (float*)scratch;
  int* pi = (int*)scratch + (size_t)n_rows * pieces;
  hipLaunchKernelGGL(argmax_pieces_kernel, dim3(n_rows, pieces), dim3(SNT), 0, stream, logits, ldl, V, piece, pv, pi);
  APC_LAUNCH_CHECK();
  hipLaunchKernelGGL(argmax_final_kernel, dim3(n_rows), dim3(WAVE), 0, stream, pv, pi, pieces, out);
  APC_LAUNCH_CHECK();
  return 0;
}

// ---- the variant that allocates nothing (declared in no_alloc.h) ----
// Room for the pieces of APC_ARGMAX_NO_ALLOC_MAX_ROWS rows: values [rows][64], then indices [rows][64].  Each GPU holds
// its own copy of the array at its own address; in host code the array's name is not that address, so the address is
// asked for once per device (hipGetSymbolAddress, with that device current) and only the answer is handed to kernels.
constexpr int NO_ALLOC_PIECES = 64;
static __device__ __align__(256) unsigned char argmax_scratch[(size_t)APC_ARGMAX_NO_ALLOC_MAX_ROWS * NO_ALLOC_PIECES * 8];
constexpr int NO_ALLOC_MAX_DEVICES = 64;
static void* argmax_scratch_ptr[NO_ALLOC_MAX_DEVICES];  // per device, null until its first call
static std::mutex argmax_scratch_lock;

APC_EXPORT int apc_argmax_rows_no_alloc(const float* logits, int ldl, int n_rows, int V, int* out,
                                        hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V <= 0 || ldl < V || !logits || !out) return APC_ERR_BAD_ARG;
  if (n_rows > APC_ARGMAX_NO_ALLOC_MAX_ROWS) return APC_ERR_TOO_LARGE;
  if (V < 8192) {  // one block a row: no pieces, nothing beyond input and output
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(n_rows), dim3(SNT), 0, stream, logits, ldl, V, out);
    APC_LAUNCH_CHECK();
    return 0;
  }
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= NO_ALLOC_MAX_DEVICES) return APC_ERR_UNSUPPORTED;
  void* ptr;
  {
    std::lock_guard<std::mutex> hold(argmax_scratch_lock);
    if (!argmax_scratch_ptr[dev]) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_scratch));
      if (e != hipSuccess) return (int)e;
      if (!p) return (int)hipErrorInvalidSymbol;
      argmax_scratch_ptr[dev] = p;
    }
    ptr = argmax_scratch_ptr[dev];
  }
  const int piece = ceil_div(V, NO_ALLOC_PIECES);
  float* pv = (float*)ptr;
  int* pi = (int*)ptr + (size_t)n_rows * NO_ALLOC_PIECES;
  hipLaunchKernelGGL(argmax_pieces_kernel, dim3(n_rows, NO_ALLOC_PIECES), dim3(SNT), 0, stream, logits, ldl, V, piece,
                     pv, pi);
  APC_LAUNCH_CHECK();
  hipLaunchKernelGGL(argmax_final_kernel, dim3(n_rows), dim3(WAVE), 0, stream, pv, pi, NO_ALLOC_PIECES, out);
  APC_LAUNCH_CHECK();
  return 0;
}

// What a block's threads share while they choose one row's token
struct SampleShared {
  float fsm[SNT / WAVE];
  uint32_t usm[SNT / WAVE];
  float bv[SNT / WAVE];
  int bi[SNT / WAVE];
  uint32_t s_key[SMALL_MAX], s_key2[SMALL_MAX];
  int s_id[SMALL_MAX], s_id2[SMALL_MAX];
  uint32_t s_count;
  int s_answer;
};

// The few survivors of a cut (cnt of them, in sh.s_key / sh.s_id in any order): sorted by (value descending, id
// ascending), then one thread does the reference's sequential arithmetic.
__device__ __forceinline__ void sample_few(SampleShared& sh, int cnt, bool use_top_p, float tp, float r, int* out_row) {
  uint32_t* s_key = sh.s_key; uint32_t* s_key2 = sh.s_key2;
  int* s_id = sh.s_id; int* s_id2 = sh.s_id2;
  for (int e = threadIdx.x; e < cnt; e += SNT) {
    const uint32_t k = s_key[e];
    const int id = s_id[e];
    int rank = 0;
    for (int j = 0; j < cnt; ++j) rank += (s_key[j] > k || (s_key[j] == k && s_id[j] < id)) ? 1 : 0;
    s_key2[rank] = k;
    s_id2[rank] = id;
  }
  __syncthreads();
  // the exponentials by all threads (the unsorted keys are done with: their place holds them), the sums by one
  float* e = reinterpret_cast<float*>(s_key);
  const float vmax = value_of(s_key2[0]);
  for (int i = threadIdx.x; i < cnt; i += SNT) e[i] = expf(value_of(s_key2[i]) - vmax);
  __syncthreads();
  if (threadIdx.x == 0) {
    int m = cnt;
    if (use_top_p) {
      float sum = 0.f;
      for (int i = 0; i < m; ++i) sum += e[i];
      if (sum == 0.f || !finite_f(sum)) {
        int keep = (int)ceilf(tp * (float)m);
        m = keep < 1 ? 1 : (keep > m ? m : keep);
      } else {
        float acc = 0.f;
        for (int i = 0; i < m; ++i) {
          acc += e[i] / sum;
          if (acc >= tp) { m = i + 1; break; }
        }
      }
    }
    float sum = 0.f;
    for (int i = 0; i < m; ++i) sum += e[i];
    float rr = r;
    int pick = s_id2[m - 1];
    for (int i = 0; i < m; ++i) {
      const float p = sum == 0.f ? 1.0f / (float)m : e[i] / sum;
      rr -= p;
      if (rr <= 0.f) { pick = s_id2[i]; break; }
    }
    *out_row = pick;
  }
}

// One row by one block, every step a pass of the block over the whole row (thresholds by bisection): the way for
// callers without working memory, and for rows that the kernels below hand back.
__device__ __forceinline__ void sample_row_one_block(SampleShared& sh, const float* __restrict__ lg, int V, float T,
                                                     int tk, float tp, float r, int* out_row) {
  float* fsm = sh.fsm; uint32_t* usm = sh.usm; float* bv = sh.bv; int* bi = sh.bi;
  uint32_t* s_key = sh.s_key; int* s_id = sh.s_id;
  uint32_t& s_count = sh.s_count; int& s_answer = sh.s_answer;

  // pass 1: argmax of the raw logits (first maximum) and the number of finite ones
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  uint32_t nfin = 0;
  for (int i = threadIdx.x; i < V; i += SNT) {
    const float v = lg[i];
    if (v > best) { best = v; best_i = i; }
    nfin += finite_f(v) ? 1u : 0u;
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, WAVE);
    const int oi = __shfl_xor(best_i, o, WAVE);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  if (threadIdx.x % WAVE == 0) { bv[threadIdx.x / WAVE] = best; bi[threadIdx.x / WAVE] = best_i; }
  __syncthreads();
  for (int w = 0; w < SNT / WAVE; ++w)
    if (bv[w] > best || (bv[w] == best && bi[w] < best_i)) { best = bv[w]; best_i = bi[w]; }
  const int arg = best_i == 0x7fffffff ? 0 : best_i;
  nfin = block_sum_t<uint32_t>(nfin, usm);

  if (nfin == 0u) { if (threadIdx.x == 0) *out_row = 0; return; }
  if (T <= 1e-5f) { if (threadIdx.x == 0) *out_row = arg; return; }

  RowView rv;
  rv.logits = lg;
  rv.V = V;
  rv.t = fmaxf(T, 1e-5f);
  rv.inv_t = 1.0f / rv.t;

  Cut set;  // all finite logits
  set.tau = 0u;
  set.id_cut = -1;
  uint32_t n = nfin;
  bool sorted = false;
  if (tk > 0 && n > (uint32_t)tk) {
    set = select_by_count(rv, set, (uint32_t)tk, usm);
    n = (uint32_t)tk;
    sorted = true;
  }
  const bool use_top_p = tp >= 0.0f && tp < 1.0f && n > 1u;

  if (n <= (uint32_t)SMALL_MAX && (sorted || use_top_p)) {
    // few survivors: gather, sort, then one thread does the reference's sequential arithmetic
    if (threadIdx.x == 0) s_count = 0u;
    __syncthreads();
    for (int i = threadIdx.x; i < V; i += SNT) {
      const uint32_t k = rv.key(i);
      if (k != 0u && in_cut(set, k, i)) {
        const uint32_t at = atomicAdd(&s_count, 1u);
        if (at < (uint32_t)SMALL_MAX) { s_key[at] = k; s_id[at] = i; }
      }
    }
    __syncthreads();
    const int cnt = (int)min(s_count, (uint32_t)SMALL_MAX);
    sample_few(sh, cnt, use_top_p, tp, r, out_row);
    return;
  }

  // many survivors: thresholds found by bisection on the key, sums by block reductions
  const float vmax = best / rv.t;  // the largest finite scaled logit (best is finite here unless +inf is present)
  float vmax_f = vmax;
  if (!finite_f(best)) {           // +inf among the logits: take the largest finite one instead
    float fm = -INFINITY;
    for (int i = threadIdx.x; i < V; i += SNT) { const float v = lg[i]; if (finite_f(v)) fm = fmaxf(fm, v); }
    fm = block_max<SNT>(fm, fsm);
    vmax_f = fm / rv.t;
  }
  if (use_top_p) {
    const uint32_t lowest = set.tau == 0u ? 1u : set.tau;
    const float total = mass_ge(rv, set, lowest, vmax_f, fsm);
    if (total == 0.f || !finite_f(total)) {
      const int keep = (int)ceilf(tp * (float)n);
      const uint32_t kk = (uint32_t)(keep < 1 ? 1 : (keep > (int)n ? (int)n : keep));
      set = select_by_count(rv, set, kk, usm);
    } else {
      bool reached;
      const Cut c = select_by_mass(rv, set, tp * total, vmax_f, &reached, fsm, usm);
      if (reached) set = c;
    }
    sorted = true;
  }
  const uint32_t lowest = set.tau == 0u ? 1u : set.tau;
  const float total = mass_ge(rv, set, lowest, vmax_f, fsm);
  const float target = r * total;
  if (sorted) {
    bool reached;
    const Cut c = select_by_mass(rv, set, target, vmax_f, &reached, fsm, usm);
    if (reached) { if (threadIdx.x == 0) *out_row = c.id_cut; return; }
    // rounding left r above the whole mass: the last candidate in sorted order
    uint32_t kmin = 0xffffffffu;
    for (int i = threadIdx.x; i < V; i += SNT) {
      const uint32_t k = rv.key(i);
      if (k != 0u && in_cut(set, k, i)) kmin = min(kmin, k);
    }
    // min over the block through the float-free path: reuse count_ge by bisection is overkill; do an LDS min
    __syncthreads();
    if (threadIdx.x == 0) s_count = 0xffffffffu;
    __syncthreads();
    atomicMin(&s_count, kmin);
    __syncthreads();
    kmin = s_count;
    int imax = -1;
    for (int i = threadIdx.x; i < V; i += SNT) {
      const uint32_t k = rv.key(i);
      if (k == kmin && in_cut(set, k, i)) imax = max(imax, i);
    }
    __syncthreads();
    if (threadIdx.x == 0) s_answer = -1;
    __syncthreads();
    atomicMax(&s_answer, imax);
    __syncthreads();
    if (threadIdx.x == 0) *out_row = s_answer < 0 ? 0 : s_answer;
    return;
  }
  // id order: the first id whose running mass reaches the target
  if (threadIdx.x == 0) s_answer = -1;
  __syncthreads();
  float running = 0.f;
  int last_in = -1;
  for (int base = 0; base < V; base += SNT) {
    const int i = base + threadIdx.x;
    float e = 0.f;
    bool in = false;
    if (i < V) {
      const uint32_t k = rv.key(i);
      in = k != 0u && in_cut(set, k, i);
      if (in) { e = expf(value_of(k) - vmax_f); last_in = i; }
    }
    // inclusive scan over the block in id order
    float s = e;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
      const float up = __shfl_up(s, o, WAVE);
      if ((threadIdx.x % WAVE) >= o) s += up;
    }
    __syncthreads();
    if (threadIdx.x % WAVE == WAVE - 1) fsm[threadIdx.x / WAVE] = s;
    __syncthreads();
    float before = running;
    for (int w = 0; w < threadIdx.x / WAVE; ++w) before += fsm[w];
    float chunk = 0.f;
    for (int w = 0; w < SNT / WAVE; ++w) chunk += fsm[w];
    const float cum = before + s;
    if (in && cum >= target) atomicMin((unsigned int*)&s_answer, (unsigned int)i);  // -1 is the largest unsigned
    running += chunk;
    __syncthreads();
    if (s_answer >= 0) break;
  }
  if (s_answer < 0) {  // r above the whole mass by rounding: the last candidate
    __syncthreads();
    if (threadIdx.x == 0) s_count = 0u;
    __syncthreads();
    if (last_in >= 0) atomicMax(&s_count, (uint32_t)last_in);
    __syncthreads();
    if (threadIdx.x == 0) *out_row = (int)s_count;
    return;
  }
  if (threadIdx.x == 0) *out_row = s_answer;
}

__global__ __launch_bounds__(SNT) void sample_rows_kernel(const float* __restrict__ logits, int ldl, int V,
                                                          const float* __restrict__ temperature,
                                                          const int* __restrict__ top_k,
                                                          const float* __restrict__ top_p,
                                                          const float* __restrict__ uniform, int* __restrict__ out) {
  __shared__ SampleShared sh;
  const int row = blockIdx.x;
  sample_row_one_block(sh, logits + (size_t)row * ldl, V, temperature[row], top_k[row], top_p[row], uniform[row],
                       out + row);
}

// ---- The same rules with many blocks a row ----
// A row of a real vocabulary is half a megabyte, and one block's passes over it (about a hundred of them for top-p)
// took 4-17 ms.  Here every step is one launch over (pieces of a row) x (rows), and the thresholds come from radix
// descents instead of bisection.  The candidates stand in one order, by (value descending, id ascending), written as
// one 64-bit sort key (the value's key, then the id counted down); the candidate at which a running weight first
// reaches a target is found digit by digit, 13 bits at a time, from a histogram of the weights per digit value: four
// launches a threshold for vocabularies up to a million, and equal values need no special case.  The weights are
// integers (1 for top-k; for probabilities exp(v - vmax) in units of 2^-40, at least 1), so that sums do not depend
// on the order in which blocks and threads add them: a row's token is the same whatever the batch and the grid.
// Launches, each of which a row sits out if it has no use for it:  the maximum;  top-k: 4;  top-p: 4;  the draw: 4
// (a list that no cut has sorted is walked in id order: the sort key is then the id alone);  the end, which writes the
// tokens.  What one launch finds the next one reads: every block of a row first works out, from the histogram of
// the launch before, where the row stands (the same arithmetic in each of them), then adds its piece of the row to
// the next histogram.  A histogram has two levels (8,192 values and their sums in groups of 32), so that a block
// reads 256 + 32 numbers of it, not all.
// Few survivors (up to SMALL_MAX after top-k) are gathered and go through the reference's sequential arithmetic as
// above.
namespace {

typedef unsigned long long u64;
constexpr int PNT = 1024;                // threads of a block that works on a piece of a row
constexpr int DIGIT_BITS = 13;
constexpr int FINE = 1 << DIGIT_BITS;    // digit values
constexpr int GROUP = 8;                 // digit values a group
constexpr int COARSE = FINE / GROUP;     // groups
static_assert(COARSE == PNT, "a thread adds one group");
constexpr int MAX_PIECES = 32;
constexpr int N_SELECTS = 3;             // top-k, top-p, the draw
constexpr int MAX_DIGITS = 5;            // 64 bits of sort key
constexpr int ROTA = 3;                  // histograms in use in turn: written, read, cleared
constexpr float MASS_ONE = 0x1p40f;      // weight of the row's largest value

enum { ST_TOPK = 0, ST_TOPP = 1, ST_DRAW = 2 };
enum { PH_ACTIVE = 1, PH_FEW = 2, PH_DONE = 3, PH_ONE_BLOCK = 4 };
enum { SEEN_TOPK = 1, SEEN_TOPP = 2 };

// digit d is bits [digit_lo, digit_hi) of the sort key
__host__ __device__ constexpr int digit_hi(int d) { return 64 - DIGIT_BITS * d; }
__host__ __device__ constexpr int digit_lo(int d) { return digit_hi(d) > DIGIT_BITS ? digit_hi(d) - DIGIT_BITS : 0; }

struct RowState {
  int phase, result;
  float t, vmax;           // temperature in use, the largest finite scaled value
  uint32_t n;              // candidates left
  int sorted;              // a cut has put the list in sorted order
  uint32_t set_tau;        // the candidates: key > set_tau, or key == set_tau and id <= set_id
  int set_id;
  int descending;          // the launch before left a histogram of this row
  int by_id;               // ... ordered by id (the draw from an unsorted list)
  int seen;                // cuts this row has passed
  int pad;
  u64 prefix;              // digits found so far
  u64 above;               // weight in front of the prefix
  u64 target;              // the threshold stands at the first candidate with this much weight up to and including it
  u64 total;
};

// Sizes of a call: what the kernels need to know of the row and of its sort key
struct SampleShape {
  int ldl, V, R, chunk, pieces;
  int vec;                 // rows start at multiples of 16 bytes: four values a load
  int id_bits;             // bits of an id
  int key_digits;          // digits of a sort key by (value, id)
  int id_digits;           // ... by id alone
};

struct SampleSpace {
  u64* fine;               // [ROTA][row][FINE]
  u64* coarse;             // [ROTA][row][COARSE]
  uint32_t* few_count;     // [row]
  float* piece_best;       // [row][MAX_PIECES] ...
  int* piece_arg;
  uint32_t* piece_finite;
  float* piece_finite_max;
  RowState* state;         // [launch + 1][row]
  uint32_t* few_key;       // [row][SMALL_MAX]
  int* few_id;
  size_t bytes;
};

constexpr size_t round16(size_t n) { return (n + 15) / 16 * 16; }

SampleSpace carve(void* base, int R) {
  SampleSpace s;
  size_t at = 0;
  auto take = [&](size_t bytes) { char* q = (char*)((uintptr_t)base + at); at += round16(bytes); return q; };
  const size_t r = (size_t)R;
  s.fine = (u64*)take(ROTA * r * FINE * sizeof(u64));
  s.coarse = (u64*)take(ROTA * r * COARSE * sizeof(u64));
  s.few_count = (uint32_t*)take(r * 4);
  s.piece_best = (float*)take(r * MAX_PIECES * 4);
  s.piece_arg = (int*)take(r * MAX_PIECES * 4);
  s.piece_finite = (uint32_t*)take(r * MAX_PIECES * 4);
  s.piece_finite_max = (float*)take(r * MAX_PIECES * 4);
  s.state = (RowState*)take((N_SELECTS * MAX_DIGITS + 1) * r * sizeof(RowState));
  s.few_key = (uint32_t*)take(r * SMALL_MAX * 4);
  s.few_id = (int*)take(r * SMALL_MAX * 4);
  s.bytes = at;
  return s;
}

// pieces of a row: enough blocks for the chip when the rows are few, at least 4 values a thread
void cut_row(int R, int V, int* pieces, int* chunk) {
  int want = ceil_div(512, R);
  want = want > MAX_PIECES ? MAX_PIECES : want;
  const int most = ceil_div(V, 4 * PNT);
  *pieces = want < most ? want : most;
  *chunk = ceil_div(ceil_div(V, *pieces), 4) * 4;
  *pieces = ceil_div(V, *chunk);
}

// f(i, logits[i]) for the values i0 <= i < i1 of a row, a thread's values in ascending order
template <typename F>
__device__ __forceinline__ void for_piece(const float* __restrict__ lg, int vec, int i0, int i1, F&& f) {
  if (vec) {  // i0 is a multiple of 4
    for (int i = i0 + 4 * (int)threadIdx.x; i < i1; i += 4 * PNT) {
      if (i + 3 < i1) {
        const float4 x = *reinterpret_cast<const float4*>(lg + i);
        f(i, x.x);
        f(i + 1, x.y);
        f(i + 2, x.z);
        f(i + 3, x.w);
      } else {
        for (int j = i; j < i1; ++j) f(j, lg[j]);
      }
    }
  } else {
    for (int i = i0 + (int)threadIdx.x; i < i1; i += PNT) f(i, lg[i]);
  }
}

// inclusive sums over the block's NT threads in thread order, and the sum of all
template <int NT>
__device__ __forceinline__ u64 block_scan(u64 v, u64* total, u64* smem) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    const u64 up = __shfl_up(v, o, WAVE);
    if (lane >= o) v += up;
  }
  __syncthreads();
  if (lane == WAVE - 1) smem[wave] = v;
  __syncthreads();
  u64 before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < NT / WAVE; ++w) {
    const u64 x = smem[w];
    all += x;
    if (w < wave) before += x;
  }
  *total = all;
  return v + before;
}

// The sort key: larger = earlier.  The id part counts down and stands in the top bits of its half, so that the
// digits that matter come first; by id alone it stands in the upper half.
__device__ __forceinline__ u64 sort_key(uint32_t key, int i, int id_bits, int by_id) {
  const uint32_t ik = (((1u << id_bits) - 1u) - (uint32_t)i) << (32 - id_bits);
  return by_id ? ((u64)ik << 32) : (((u64)key << 32) | ik);
}
__device__ __forceinline__ int id_of_sort_key(u64 c, int id_bits, int by_id) {
  const uint32_t ik = by_id ? (uint32_t)(c >> 32) : (uint32_t)c;
  return (int)(((1u << id_bits) - 1u) - (ik >> (32 - id_bits)));
}
__device__ __forceinline__ u64 mass_of(uint32_t key, float vmax) {
  const u64 q = (u64)(expf(value_of(key) - vmax) * MASS_ONE);
  return q < 1 ? 1 : q;
}

struct SettleShared {
  u64 scan[PNT / WAVE];
  int bin;
  u64 above;
};

// Where the row stands after launch (stage, digit), whose histogram is (fine, coarse): all NT threads of the block,
// the same result in each.
template <int NT>
__device__ __forceinline__ void settle(RowState& S, const SampleShape& sz, int stage, int digit,
                                       const u64* __restrict__ fine, const u64* __restrict__ coarse, float frac,
                                       SettleShared& sh) {
  if (S.phase != PH_ACTIVE || !S.descending) return;
  constexpr int PER = COARSE / NT;  // groups a thread, threads in descending order of the digit's value
  const int top = COARSE - 1 - threadIdx.x * PER;
  u64 groups[PER], local = 0;
#pragma unroll
  for (int g = 0; g < PER; ++g) {
    groups[g] = coarse[top - g];
    local += groups[g];
  }
  if (threadIdx.x == 0) sh.bin = -1;
  u64 all;
  const u64 incl = block_scan<NT>(local, &all, sh.scan);
  if (digit == 0 && stage != ST_TOPK) {  // every candidate is in this histogram: the threshold as a weight
    S.total = all;
    const double want = ceil((double)frac * (double)all);
    const u64 target = want <= 1.0 ? 1 : (want >= (double)all ? all : (u64)want);
    S.target = target > all ? all : target;
  }
  u64 before = S.above + incl - local;
  if (before < S.target && S.target <= before + local) {
#pragma unroll
    for (int g = 0; g < PER; ++g) {
      if (before < S.target && S.target <= before + groups[g]) {
        u64 mine[GROUP];
#pragma unroll
        for (int k = 0; k < GROUP; ++k) mine[k] = fine[(top - g) * GROUP + GROUP - 1 - k];
        u64 at = before;
#pragma unroll
        for (int k = 0; k < GROUP; ++k) {
          if (at < S.target && S.target <= at + mine[k]) {
            sh.bin = (top - g) * GROUP + GROUP - 1 - k;
            sh.above = at;
          }
          at += mine[k];
        }
      }
      before += groups[g];
    }
  }
  __syncthreads();
  const int bin = sh.bin;
  const u64 above = sh.above;
  __syncthreads();
  if (bin < 0) {  // the weight asked for is not there (it always is): the one-block way decides
    S.phase = PH_ONE_BLOCK;
    return;
  }
  S.prefix |= (u64)bin << digit_lo(digit);
  S.above = above;
  if (digit < (S.by_id ? sz.id_digits : sz.key_digits) - 1) return;
  // the sort key is whole: it names one candidate
  S.descending = 0;
  const int id = id_of_sort_key(S.prefix, sz.id_bits, S.by_id);
  if (stage == ST_DRAW) {
    S.phase = PH_DONE;
    S.result = id;
    return;
  }
  S.set_tau = (uint32_t)(S.prefix >> 32);
  S.set_id = id;
  S.sorted = 1;
  if (stage == ST_TOPK) S.n = (uint32_t)S.target;
}

__global__ __launch_bounds__(PNT) void sample_max_kernel(const float* __restrict__ logits, SampleShape sz,
                                                         SampleSpace sp) {
  __shared__ float bv[PNT / WAVE], fv[PNT / WAVE];
  __shared__ int bi[PNT / WAVE];
  __shared__ uint32_t nv[PNT / WAVE];
  const int row = blockIdx.y, piece = blockIdx.x;
  // what the first of the later launches adds to (each of them clears the histogram of the one after it)
  for (int j = piece * PNT + threadIdx.x; j < FINE; j += sz.pieces * PNT) sp.fine[(size_t)row * FINE + j] = 0;
  if (piece == 0) {
    sp.coarse[(size_t)row * COARSE + threadIdx.x] = 0;
    if (threadIdx.x == 0) sp.few_count[row] = 0u;
  }
  const float* lg = logits + (size_t)row * sz.ldl;
  const int i0 = piece * sz.chunk, i1 = min(sz.V, i0 + sz.chunk);
  float best = -INFINITY, fmax = -INFINITY;
  int best_i = 0x7fffffff;
  uint32_t nfin = 0;
  for_piece(lg, sz.vec, i0, i1, [&](int i, float v) {
    if (v > best) { best = v; best_i = i; }
    if (finite_f(v)) { ++nfin; fmax = fmaxf(fmax, v); }
  });
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, WAVE);
    const int oi = __shfl_xor(best_i, o, WAVE);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    fmax = fmaxf(fmax, __shfl_xor(fmax, o, WAVE));
    nfin += __shfl_xor(nfin, o, WAVE);
  }
  if (threadIdx.x % WAVE == 0) {
    bv[threadIdx.x / WAVE] = best;
    bi[threadIdx.x / WAVE] = best_i;
    fv[threadIdx.x / WAVE] = fmax;
    nv[threadIdx.x / WAVE] = nfin;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < PNT / WAVE; ++w) {
      if (bv[w] > best || (bv[w] == best && bi[w] < best_i)) { best = bv[w]; best_i = bi[w]; }
      fmax = fmaxf(fmax, fv[w]);
      nfin += nv[w];
    }
    const size_t at = (size_t)row * MAX_PIECES + piece;
    sp.piece_best[at] = best;
    sp.piece_arg[at] = best_i;
    sp.piece_finite[at] = nfin;
    sp.piece_finite_max[at] = fmax;
  }
}

struct PassShared {
  u64 hist[FINE];
  SettleShared settle;
};

// Launch `q` of the descents: digit `digit` of `stage`; the one before was (prev_stage, prev_digit), none if q == 0.
__global__ __launch_bounds__(PNT) void sample_pass_kernel(const float* __restrict__ logits, SampleShape sz,
                                                          const float* __restrict__ temperature,
                                                          const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                          const float* __restrict__ uniform, SampleSpace sp, int q,
                                                          int stage, int digit, int prev_stage, int prev_digit) {
  extern __shared__ __attribute__((aligned(16))) unsigned char pass_smem[];
  PassShared& sh = *reinterpret_cast<PassShared*>(pass_smem);
  const int row = blockIdx.y, piece = blockIdx.x, R = sz.R;
  const float* lg = logits + (size_t)row * sz.ldl;
  const float tp = top_p[row];
  const int tk = top_k[row];
  {  // the histogram of the launch after this one
    const size_t next = ((size_t)((q + 1) % ROTA) * R + row);
    for (int j = piece * PNT + threadIdx.x; j < FINE; j += sz.pieces * PNT) sp.fine[next * FINE + j] = 0;
    if (piece == 0) sp.coarse[next * COARSE + threadIdx.x] = 0;
  }
  RowState S;
  if (q == 0) {
    float best = -INFINITY, fmax = -INFINITY;
    int best_i = 0x7fffffff;
    uint32_t nfin = 0;
    for (int p = 0; p < sz.pieces; ++p) {
      const size_t at = (size_t)row * MAX_PIECES + p;
      const float v = sp.piece_best[at];
      const int vi = sp.piece_arg[at];
      if (v > best || (v == best && vi < best_i)) { best = v; best_i = vi; }
      nfin += sp.piece_finite[at];
      fmax = fmaxf(fmax, sp.piece_finite_max[at]);
    }
    const float T = temperature[row];
    S = RowState{};
    S.phase = PH_ACTIVE;
    S.t = fmaxf(T, 1e-5f);
    S.vmax = (finite_f(best) ? best : fmax) / S.t;
    S.n = nfin;
    S.set_tau = 0u;
    S.set_id = -1;
    if (nfin == 0u) { S.phase = PH_DONE; S.result = 0; }
    else if (T <= 1e-5f) { S.phase = PH_DONE; S.result = best_i == 0x7fffffff ? 0 : best_i; }
  } else {
    S = sp.state[(size_t)q * R + row];
    const size_t prev = (size_t)((q - 1) % ROTA) * R + row;
    settle<PNT>(S, sz, prev_stage, prev_digit, sp.fine + prev * FINE, sp.coarse + prev * COARSE,
                prev_stage == ST_TOPP ? tp : uniform[row], sh.settle);
  }
  bool gather = false;
  if (S.phase == PH_ACTIVE && S.descending && digit == 0) S.phase = PH_ONE_BLOCK;  // (the launches of a descent ran out)
  if (S.phase == PH_ACTIVE && !S.descending && digit == 0) {
    auto begin = [&](int by_id, u64 target) {
      S.descending = 1;
      S.by_id = by_id;
      S.prefix = 0;
      S.above = 0;
      S.target = target;
    };
    const bool wants_k = tk > 0 && S.n > (uint32_t)tk && !(S.seen & SEEN_TOPK);
    if (stage == ST_TOPK) {
      if (wants_k) begin(0, (u64)tk);
      S.seen |= SEEN_TOPK;
    } else if (wants_k) {
      S.phase = PH_ONE_BLOCK;          // the caller left out the launches of a cut that this row asks for
    } else {
      const bool use_top_p = tp >= 0.0f && tp < 1.0f && S.n > 1u;
      if (S.n <= (uint32_t)SMALL_MAX && (S.sorted || use_top_p)) {
        S.phase = PH_FEW;
        gather = true;
      } else if (stage == ST_TOPP) {
        if (use_top_p) begin(0, 0);    // the target follows from the sum of this launch's histogram
        S.seen |= SEEN_TOPP;
      } else if (use_top_p && !(S.seen & SEEN_TOPP)) {
        S.phase = PH_ONE_BLOCK;
      } else {
        begin(S.sorted ? 0 : 1, 0);
      }
    }
  }
  if (piece == 0 && threadIdx.x == 0) sp.state[(size_t)(q + 1) * R + row] = S;
  const int i0 = piece * sz.chunk, i1 = min(sz.V, i0 + sz.chunk);
  if (gather) {
    for_piece(lg, sz.vec, i0, i1, [&](int i, float x) {
      if (!finite_f(x)) return;
      const uint32_t k = key_of(x / S.t);
      if (!(k > S.set_tau || (k == S.set_tau && i <= S.set_id))) return;
      const uint32_t at = atomicAdd(&sp.few_count[row], 1u);
      if (at < (uint32_t)SMALL_MAX) {
        sp.few_key[(size_t)row * SMALL_MAX + at] = k;
        sp.few_id[(size_t)row * SMALL_MAX + at] = i;
      }
    });
    return;
  }
  if (S.phase != PH_ACTIVE || !S.descending) return;
#pragma unroll
  for (int k = 0; k < GROUP; ++k) sh.hist[k * PNT + threadIdx.x] = 0;
  __syncthreads();
  const int lo = digit_lo(digit), hi = digit_hi(digit);
  const uint32_t mask = (1u << (hi - lo)) - 1u;
  for_piece(lg, sz.vec, i0, i1, [&](int i, float x) {
    if (!finite_f(x)) return;
    const uint32_t k = key_of(x / S.t);
    if (!(k > S.set_tau || (k == S.set_tau && i <= S.set_id))) return;
    const u64 c = sort_key(k, i, sz.id_bits, S.by_id);
    if (digit > 0 && (c >> hi) != (S.prefix >> hi)) return;
    atomicAdd(&sh.hist[(uint32_t)(c >> lo) & mask], stage == ST_TOPK ? (u64)1 : mass_of(k, S.vmax));
  });
  __syncthreads();
  // thread t adds group t; it starts t values into the group, so that the threads of a wave read different banks
  const size_t cur = (size_t)(q % ROTA) * R + row;
  u64* fine = sp.fine + cur * FINE + threadIdx.x * GROUP;
  u64 sum = 0;
#pragma unroll
  for (int k = 0; k < GROUP; ++k) {
    const int j = (k + threadIdx.x) % GROUP;
    const u64 h = sh.hist[threadIdx.x * GROUP + j];
    if (h) {
      atomicAdd(&fine[j], h);
      sum += h;
    }
  }
  if (sum) atomicAdd(&sp.coarse[cur * COARSE + threadIdx.x], sum);
}

union EndShared {
  SettleShared settle;
  SampleShared one;
};

// The last launch: (last_stage, last_digit) was the one before
__global__ __launch_bounds__(SNT) void sample_end_kernel(const float* __restrict__ logits, SampleShape sz,
                                                         const float* __restrict__ temperature,
                                                         const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                         const float* __restrict__ uniform, SampleSpace sp, int q,
                                                         int last_stage, int last_digit, int* __restrict__ out) {
  __shared__ EndShared sh;
  const int row = blockIdx.x, R = sz.R;
  const float tp = top_p[row], r = uniform[row];
  RowState S = sp.state[(size_t)q * R + row];
  const size_t prev = (size_t)((q - 1) % ROTA) * R + row;
  settle<SNT>(S, sz, last_stage, last_digit, sp.fine + prev * FINE, sp.coarse + prev * COARSE,
              last_stage == ST_TOPP ? tp : r, sh.settle);
  if (S.phase == PH_DONE) {
    if (threadIdx.x == 0) out[row] = S.result;
    return;
  }
  __syncthreads();
  if (S.phase == PH_FEW) {
    const int cnt = (int)min(sp.few_count[row], (uint32_t)SMALL_MAX);
    for (int e = threadIdx.x; e < cnt; e += SNT) {
      sh.one.s_key[e] = sp.few_key[(size_t)row * SMALL_MAX + e];
      sh.one.s_id[e] = sp.few_id[(size_t)row * SMALL_MAX + e];
    }
    __syncthreads();
    const bool use_top_p = tp >= 0.0f && tp < 1.0f && S.n > 1u;
    sample_few(sh.one, cnt, use_top_p, tp, r, out + row);
    return;
  }
  // a row whose cut or draw the launches did not cover (the caller's word on its rows was wrong), or is not through
  sample_row_one_block(sh.one, logits + (size_t)row * sz.ldl, sz.V, temperature[row], top_k[row], tp, r, out + row);
}

std::mutex pass_attr_lock;
bool pass_attr_set[64];

}  // namespace

// KiB of working memory that apc_sample_rows wants for n_rows rows (it takes the one-block way without)
APC_EXPORT int apc_sample_rows_scratch_kib(int n_rows) {
  if (n_rows <= 0 || n_rows > 65535) return 0;
  return (int)((carve(nullptr, n_rows).bytes + 1023) / 1024);
}

// `cuts`: bit 0 set if some row may have top-k > 0, bit 1 if some row may have 0 <= top-p < 1, bit 2 if every row that
// samples has 0 < top-k <= 1,024 (its survivors are then few, and the launches of top-p and of the draw fall away).
// A caller that does not know its rows passes 3.  A row for which the caller's word is wrong still gets its token,
// the slow way.
APC_EXPORT int apc_sample_rows(const float* logits, int ldl, int n_rows, int V, const float* temperature,
                               const int* top_k, const float* top_p, const float* uniform, int* out, void* scratch,
                               size_t scratch_bytes, int cuts, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V <= 0 || ldl < V) return APC_ERR_BAD_ARG;
  int dev = -1;
  if (scratch) {
    const hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
  }
  // (a row's weights add up in 64 bits: 2^40 a candidate at most, so 2^22 candidates stay far inside)
  if (!scratch || n_rows > 65535 || dev < 0 || dev >= 64 || V > (1 << 22)) {
    hipLaunchKernelGGL(sample_rows_kernel, dim3(n_rows), dim3(SNT), 0, stream, logits, ldl, V, temperature, top_k,
                       top_p, uniform, out);
    APC_LAUNCH_CHECK();
    return 0;
  }
  if (((uintptr_t)scratch & 15u) || scratch_bytes < carve(nullptr, n_rows).bytes) return APC_ERR_BAD_ARG;
  {
    std::lock_guard<std::mutex> hold(pass_attr_lock);
    if (!pass_attr_set[dev]) {
      const hipError_t e = hipFuncSetAttribute((const void*)sample_pass_kernel,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(PassShared));
      if (e != hipSuccess) return (int)e;
      pass_attr_set[dev] = true;
    }
  }
  const SampleSpace sp = carve(scratch, n_rows);
  SampleShape sz;
  sz.ldl = ldl;
  sz.V = V;
  sz.R = n_rows;
  cut_row(n_rows, V, &sz.pieces, &sz.chunk);
  sz.vec = ((uintptr_t)logits % 16 == 0 && ldl % 4 == 0) ? 1 : 0;
  sz.id_bits = 1;
  while (sz.id_bits < 31 && (1u << sz.id_bits) < (unsigned)V) ++sz.id_bits;
  sz.key_digits = ceil_div(32 + sz.id_bits, DIGIT_BITS);
  sz.id_digits = ceil_div(sz.id_bits, DIGIT_BITS);
  const dim3 grid(sz.pieces, n_rows);
  hipLaunchKernelGGL(sample_max_kernel, grid, dim3(PNT), 0, stream, logits, sz, sp);
  APC_LAUNCH_CHECK();
  const bool few = (cuts & 5) == 5;
  int q = 0, prev_stage = -1, prev_digit = -1;
  for (int stage = 0; stage < N_SELECTS; ++stage) {
    int digits = sz.key_digits;
    if (stage == ST_TOPK && !(cuts & 1)) continue;
    if (stage == ST_TOPP && (!(cuts & 2) || few)) continue;
    if (stage == ST_DRAW) digits = few ? 1 : ((cuts & 3) ? sz.key_digits : sz.id_digits);
    for (int digit = 0; digit < digits; ++digit) {
      hipLaunchKernelGGL(sample_pass_kernel, grid, dim3(PNT), sizeof(PassShared), stream, logits, sz, temperature,
                         top_k, top_p, uniform, sp, q, stage, digit, prev_stage, prev_digit);
      APC_LAUNCH_CHECK();
      ++q;
      prev_stage = stage;
      prev_digit = digit;
    }
  }
  hipLaunchKernelGGL(sample_end_kernel, dim3(n_rows), dim3(SNT), 0, stream, logits, sz, temperature, top_k, top_p,
                     uniform, sp, q, prev_stage, prev_digit, out);
  APC_LAUNCH_CHECK();
  return 0;
}
