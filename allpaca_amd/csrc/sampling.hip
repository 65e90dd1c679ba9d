// Token choice on the GPU: first-maximum argmax, and temperature / top-k / top-p
// sampling with a uniform number given per row.  One block per row of logits.
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

__global__ __launch_bounds__(SNT) void sample_rows_kernel(const float* __restrict__ logits, int ldl, int V,
                                                          const float* __restrict__ temperature,
                                                          const int* __restrict__ top_k,
                                                          const float* __restrict__ top_p,
                                                          const float* __restrict__ uniform, int* __restrict__ out) {
  __shared__ float fsm[SNT / WAVE];
  __shared__ uint32_t usm[SNT / WAVE];
  __shared__ float bv[SNT / WAVE];
  __shared__ int bi[SNT / WAVE];
  __shared__ uint32_t s_key[SMALL_MAX], s_key2[SMALL_MAX];
  __shared__ int s_id[SMALL_MAX], s_id2[SMALL_MAX];
  __shared__ uint32_t s_count;
  __shared__ int s_answer;

  const int row = blockIdx.x;
  const float* lg = logits + (size_t)row * ldl;
  const float T = temperature[row];
  const float r = uniform[row];
  const float tp = top_p[row];
  const int tk = top_k[row];

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

  if (nfin == 0u) { if (threadIdx.x == 0) out[row] = 0; return; }
  if (T <= 1e-5f) { if (threadIdx.x == 0) out[row] = arg; return; }

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
    for (int e = threadIdx.x; e < cnt; e += SNT) {
      const uint32_t k = s_key[e];
      const int id = s_id[e];
      int rank = 0;
      for (int j = 0; j < cnt; ++j) rank += (s_key[j] > k || (s_key[j] == k && s_id[j] < id)) ? 1 : 0;
      s_key2[rank] = k;
      s_id2[rank] = id;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int m = cnt;
      const float vmax = value_of(s_key2[0]);
      if (use_top_p) {
        float sum = 0.f;
        for (int i = 0; i < m; ++i) sum += expf(value_of(s_key2[i]) - vmax);
        if (sum == 0.f || !finite_f(sum)) {
          int keep = (int)ceilf(tp * (float)m);
          m = keep < 1 ? 1 : (keep > m ? m : keep);
        } else {
          float acc = 0.f;
          for (int i = 0; i < m; ++i) {
            acc += expf(value_of(s_key2[i]) - vmax) / sum;
            if (acc >= tp) { m = i + 1; break; }
          }
        }
      }
      float sum = 0.f;
      for (int i = 0; i < m; ++i) sum += expf(value_of(s_key2[i]) - vmax);
      float rr = r;
      int pick = s_id2[m - 1];
      for (int i = 0; i < m; ++i) {
        const float p = sum == 0.f ? 1.0f / (float)m : expf(value_of(s_key2[i]) - vmax) / sum;
        rr -= p;
        if (rr <= 0.f) { pick = s_id2[i]; break; }
      }
      out[row] = pick;
    }
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
    if (reached) { if (threadIdx.x == 0) out[row] = c.id_cut; return; }
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
    if (threadIdx.x == 0) out[row] = s_answer < 0 ? 0 : s_answer;
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
    if (threadIdx.x == 0) out[row] = (int)s_count;
    return;
  }
  if (threadIdx.x == 0) out[row] = s_answer;
}

APC_EXPORT int apc_sample_rows(const float* logits, int ldl, int n_rows, int V, const float* temperature,
                               const int* top_k, const float* top_p, const float* uniform, int* out,
                               hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V <= 0 || ldl < V) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL(sample_rows_kernel, dim3(n_rows), dim3(SNT), 0, stream, logits, ldl, V, temperature, top_k, top_p,
                     uniform, out);
  APC_LAUNCH_CHECK();
  return 0;
}
