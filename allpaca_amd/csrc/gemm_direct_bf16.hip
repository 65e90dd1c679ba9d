// Matrix product for many rows whose weight operand never touches LDS:  C[M,N] = A[M,K] . W[N,K]^T.
//
// The tiled layout of W (16 outputs x 32 columns = 1 KiB in the lane order of a v_mfma_f32_16x16x32_bf16 operand)
// is what a wave's load of 16 bytes a lane returns, so a wave takes its weight fragments straight from global memory
// into a ring of registers, three steps of 32 columns ahead of their use.  The four waves of a block stand side by
// side along N: each owns NF bands of 16 outputs and all 128 rows of the block, so no weight byte is loaded twice and
// none crosses LDS.  The activations are shared by the four waves: they go from global memory into LDS with direct
// loads (no registers in between), already in fragment order (a 16 x 32 fragment = one load instruction = 1 KiB
// that a later ds_read_b128 returns lane by lane, free of bank conflicts), in four stages of 64 columns.
// Per 64 columns a block moves 16 KiB of A and 8 NF KiB of W through the load path and reads 64 KiB from LDS, where
// the 128 x 128 tile of gemm_bf16.hip moves 32 KiB and 96 KiB for half as many MFMAs (NF = 8).  At the shapes of a
// 2,048-row step it waits for its loads: every block streams (128 + 64 NF) K 2 bytes through the L2, which the
// counters show busy three quarters of the time or more; 60 % fewer requests to the L2 (four waves made to load
// the same bands, timing only) bought 13 %, and the vendor library's products take about the same time.
//
// The accumulators (8 row groups x NF bands x 4 registers) live in the accumulation registers; the MFMA is written as
// an instruction with that register class, because left to itself the compiler moved accumulators between the two
// files inside the loop for some epilogues.  Waits on the direct loads are counted by hand (they return in order:
// at the barrier in front of a stage, all but the NVM youngest loads are complete); the loop issues the same loads
// in every stage, beyond the end of K they fetch the last stage again, so that the count holds to the end.
// MFMA operands are swapped against gemm_bf16.hip (weights as the first operand): a lane then holds four
// consecutive outputs of one row and stores them as one 8 or 16 byte piece.
// Sums are added in the same order as in gemm_bf16.hip (K ascending, 32 at a time): results are equal bit for bit.
// K must be a multiple of 128, N of 4.
// Reference counterpart: gemm_nt_bf16_tiled_kernel, hip/src/kernels.cpp:634 (no matrix cores there).
#include "gemm_direct.h"
#include "mfma.h"

namespace {

// D_..._PRE: A is a row that a product into the residual left for the RMS norm, and the sums are scaled by the row's
// 1 / sqrt(mean of x^2 + eps).  D_ACC_EMIT: add into the residual and leave that row for the norm that reads it next.
enum { D_STORE_BF16 = 0, D_STORE_F32 = 1, D_ACC_F32 = 2, D_SWIGLU = 3, D_SWIGLU_PRE = 4, D_ACC_EMIT = 5,
       D_STORE_BF16_PRE = 6 };
__host__ __device__ constexpr bool is_swiglu(int mode) { return mode == D_SWIGLU || mode == D_SWIGLU_PRE; }
__host__ __device__ constexpr bool is_pre(int mode) { return mode == D_SWIGLU_PRE || mode == D_STORE_BF16_PRE; }

// What goes with a norm folded into the product.  PRE: ss [M][parts] sums of x^2 of the rows (read), eps.
// EMIT: g the norm's weight [N]; raw [M][ldr] takes bfloat16(x g); ss [M][parts] takes the sums of x^2 of the block's
// columns at part0 + the block's column tile.
struct DirectPre {
  float* ss;
  int parts;
  float eps;
  const float* g;
  bf16_t* raw;
  int ldr;
  int part0;
};

constexpr int R = 4;           // ring slots of W fragments: loads run R - 1 steps of 32 columns ahead
constexpr int S = 4;           // LDS stages of A, 64 columns each
constexpr int LEAD = R - 1;
constexpr int PA = 3;          // fragments of A read from LDS ahead of the MFMAs that use them

__device__ __forceinline__ void load_to_lds(BufferRsrc rsrc, void* lds, int lane_bytes, int scalar_bytes) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds, 16, lane_bytes,
                                           scalar_bytes, 0, 0);
}

// c += a . b with c in accumulation registers
__device__ __forceinline__ void mfma16_acc(floatx4& c, const Frag& a, const Frag& b) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 av = __builtin_bit_cast(u32x4, a), bv = __builtin_bit_cast(u32x4, b);
  asm("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(av), "v"(bv));
}

template <int N>
__device__ __forceinline__ void wait_loads_but() {  // until at most N vector memory loads of this wave are in flight
  // vmcnt: bits [3:0] and [15:14]; expcnt [6:4] = 7 and lgkmcnt [11:8] = 15 wait for nothing
  __builtin_amdgcn_s_waitcnt(((N & 15) | ((N >> 4) << 14)) | 0x0f70);
}

// Row group a (0..BMG-1) of a step issues the load of band f of the step LEAD ahead when a == f * BMG / NF
// (BMG row groups of 16 rows a block: one load in some of the groups, or several a group when NF > BMG).
template <int BMG, int NF>
__host__ __device__ constexpr bool band_loaded_at(int f, int a) { return f * BMG / NF == a; }
// W loads that a stage issues behind its last direct load of A (which goes out in group BMG / 2 - 1)
template <int BMG, int NF>
__host__ __device__ constexpr int loads_behind_a() {
  int n = 0;
  for (int g = BMG / 2; g < 2 * BMG; ++g)
    for (int f = 0; f < NF; ++f)
      if (band_loaded_at<BMG, NF>(f, g % BMG)) ++n;
  return n;
}

// The tile of block `bid` of a product with BMG * 16 rows a block.
template <int BMG, int NF, int MODE>
__device__ __forceinline__ void direct_tile(int bid, const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W,
                                            const bf16_t* __restrict__ W2, int chunks, void* __restrict__ C, int ldc,
                                            int M, int N, int K, DirectPre pre = DirectPre{}) {
  static_assert(R % 2 == 0, "ring slots are static over two stages");
  constexpr int NP = BMG / 2;  // direct loads of A a wave and stage (BMG * 2 fragments over 4 waves)
  constexpr int G = 2 * BMG;   // groups of NF MFMAs a stage: (chunk of 32 columns, row group)
  static_assert(NP % 2 == 0 && G % (PA + 1) == 0, "a wave loads whole row groups; fragment registers are static");
  constexpr int U = R / 2;     // stages per pass of the loop
  // loads a wave issues between its last direct load of a stage and the barrier in front of that stage's use
  constexpr int NVM = loads_behind_a<BMG, NF>() + (S - 2) * (NP + 2 * NF);
  static_assert(NVM < 64, "the counter has 6 bits");
  __shared__ __attribute__((aligned(1024))) unsigned char As[S][BMG * 2][1024];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  constexpr int NOUT = is_swiglu(MODE) ? NF / 2 : NF;  // bands of outputs a wave writes
  constexpr int NB = 4 * NOUT * 16;                     // outputs of a block
  int mt, nt;
  {
    // Consecutive block ids go to the 8 XCDs in turn (an L2 each).  The tiles are put in one order: groups of up to 16
    // row tiles, inside a group column tile by column tile, row tile fastest; XCD x takes the x-th eighth of that
    // order, so the blocks that run on an XCD at one time share a few panels of W, and every XCD gets the same number
    // of tiles whatever the number of column tiles (20 column tiles of 12 rows each dealt out by whole columns gave
    // four XCDs 36 tiles for their 32 compute units and the others 24: two rounds for 240 tiles).
    const int MT = ceil_div(M, BMG * 16), NT = ceil_div(N, NB);
    constexpr int GM = 16;
    const int per_xcd = ceil_div(MT * NT, 8);
    const int slot = bid / 8;
    const int t = (bid % 8) * per_xcd + slot;
    if (slot >= per_xcd || t >= MT * NT) return;
    const int group = t / (GM * NT), first_m = group * GM, gsz = min(MT - first_m, GM), r = t - group * GM * NT;
    nt = r / gsz;
    mt = first_m + r % gsz;
  }
  const int m0 = mt * BMG * 16;
  const int bands = (N + 15) / 16;
  const int band0 = nt * (4 * NOUT) + wave * NOUT;  // first band of this wave
  const int base_band = min(band0, bands - 1);
  const BufferRsrc abuf = make_rsrc(A + (size_t)m0 * lda);
  const BufferRsrc wbuf = make_rsrc(W + (size_t)base_band * chunks * 512);
  const BufferRsrc ubuf = make_rsrc((is_swiglu(MODE) ? W2 : W) + (size_t)base_band * chunks * 512);
  int woff[NF];  // SwiGLU: NOUT gate bands, then the same bands of up
#pragma unroll
  for (int f = 0; f < NF; ++f) woff[f] = (min(band0 + f % NOUT, bands - 1) - base_band) * chunks * 1024 + lane * 16;
  int aoff[NP / 2];  // this wave's row groups wave * NP / 2 + j: lane -> (row lane % 16, 8 columns lane / 16)
#pragma unroll
  for (int j = 0; j < NP / 2; ++j)
    aoff[j] = (min(m0 + (wave * (NP / 2) + j) * 16 + lane % 16, M - 1) - m0) * lda * 2 + (lane / 16) * 16;

  floatx4 acc[BMG][NF];
#pragma unroll
  for (int a = 0; a < BMG; ++a)
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[a][f] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int ktiles = K / 64;
  auto a_piece = [&](int kt, int p) {  // piece p (0..NP-1) of this wave's share of stage kt
    const int j = p / 2, c = p % 2;
    load_to_lds(abuf, &As[kt % S][(wave * (NP / 2) + j) * 2 + c][0], aoff[j], min(kt, ktiles - 1) * 128 + c * 64);
  };
  Frag ring[R][NF];
  auto w_piece = [&](int slot, int q, int f) {  // band f of step q (32 columns)
    ring[slot][f] = load_frag_buffer((is_swiglu(MODE) && f >= NOUT) ? ubuf : wbuf, woff[f],
                                     min(q, 2 * ktiles - 1) * 1024);
  };
  // stages 0..S-2 of A and steps 0..LEAD-1 of W
#pragma unroll
  for (int s = 0; s < S - 1; ++s)
#pragma unroll
    for (int p = 0; p < NP; ++p) a_piece(s, p);
#pragma unroll
  for (int d = 0; d < LEAD; ++d)
#pragma unroll
    for (int f = 0; f < NF; ++f) w_piece(d, d, f);
  wait_loads_but<0>();
  // the compiler may have moved the W loads behind that wait; a use makes it wait for them here, so that the loop
  // starts with nothing in flight and the counts below hold from the first stage on
#pragma unroll
  for (int d = 0; d < LEAD; ++d)
#pragma unroll
    for (int f = 0; f < NF; ++f)
      asm volatile("" : "+v"(ring[d][f].w[0]), "+v"(ring[d][f].w[1]), "+v"(ring[d][f].w[2]), "+v"(ring[d][f].w[3]));

  for (int t = 0; t < ktiles; t += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int stage = t + u;
      __builtin_amdgcn_sched_barrier(0);
      wait_loads_but<NVM>();             // this wave's pieces of the stage are in LDS ...
      __builtin_amdgcn_s_barrier();      // ... and so are the other waves'; all have left the stage before
      __builtin_amdgcn_sched_barrier(0);
      const unsigned char* abase = &As[stage % S][0][lane * 16];
      Frag fa[PA + 1];  // group g reads fragment (row group g % BMG, chunk g / BMG)
#pragma unroll
      for (int g = 0; g < PA; ++g) fa[g] = *reinterpret_cast<const Frag*>(abase + g * 2048);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const int c = g / BMG, a = g % BMG;
        const int slot = (2 * u + c) % R;          // ring slot of step 2 * stage + c
        const int into = (2 * u + c + LEAD) % R;   // slot of the step LEAD ahead: the step before this one has left it
        if (g + PA < G)
          fa[(g + PA) % (PA + 1)] =
              *reinterpret_cast<const Frag*>(abase + ((g + PA) % BMG) * 2048 + ((g + PA) / BMG) * 1024);
        if (g < NP) a_piece(stage + S - 1, g);     // into the stage that every wave left at the barrier above
#pragma unroll
        for (int f = 0; f < NF; ++f)
          if (band_loaded_at<BMG, NF>(f, a)) w_piece(into, 2 * stage + c + LEAD, f);
#pragma unroll
        for (int f = 0; f < NF; ++f) mfma16_acc(acc[a][f], ring[slot][f], fa[g % (PA + 1)]);
        __builtin_amdgcn_sched_barrier(0);         // keeps a group's memory instructions with its MFMAs
      }
    }
    // The last MFMAs must have left the matrix cores before their results are read.  The compiler does not know these
    // instructions, so it neither waits by itself nor keeps its reads of the accumulators behind a wait that stands
    // after the loop (it has read them right behind the last MFMA); inside the loop it reads none.
    if (t + U >= ktiles) asm volatile("s_nop 15\n\ts_nop 15");
  }
  wait_loads_but<0>();

  // D[i][j]: i = output (lane / 16) * 4 + r within the band, j = row lane % 16 within the row group
  const int mi = lane % 16, nq = lane / 16;
  float row_scale[BMG];
  if constexpr (is_pre(MODE)) {
    // 1 / sqrt(mean of x^2 + eps) of the block's rows, a thread a row, through the LDS that the stages have left
    float* scales = reinterpret_cast<float*>(&As[0][0][0]);
    __syncthreads();
    if (tid < BMG * 16) {
      const float* row = pre.ss + (size_t)min(m0 + tid, M - 1) * pre.parts;
      float sum = 0.f;
      for (int p0 = 0; p0 < pre.parts; p0 += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = p0 + j < pre.parts ? row[p0 + j] : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) sum += v[j];
      }
      scales[tid] = 1.0f / sqrtf(sum / (float)K + pre.eps);
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < BMG; ++a) row_scale[a] = scales[a * 16 + mi];
  }
  float emit_sq[BMG];
#pragma unroll
  for (int a = 0; a < BMG; ++a) {
    const int m = m0 + a * 16 + mi;
    if constexpr (MODE == D_ACC_EMIT) {
      floatx4 cv[NOUT];
      float sq = 0.f;
#pragma unroll
      for (int f = 0; f < NOUT; ++f) {
        const int n = (band0 + f) * 16 + nq * 4;
        cv[f] = (m < M && n < N) ? *reinterpret_cast<const floatx4*>((const float*)C + (size_t)m * ldc + n)
                                 : floatx4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int f = 0; f < NOUT; ++f) {
        const int n = (band0 + f) * 16 + nq * 4;
        if (m < M && n < N) {
          const floatx4 x = cv[f] + acc[a][f];
          const floatx4 gv = *reinterpret_cast<const floatx4*>(pre.g + n);
          *reinterpret_cast<floatx4*>((float*)C + (size_t)m * ldc + n) = x;
          uint2 o;
          o.x = pack_bf16x2(x[0] * gv[0], x[1] * gv[1]);
          o.y = pack_bf16x2(x[2] * gv[2], x[3] * gv[3]);
          *reinterpret_cast<uint2*>(pre.raw + (size_t)m * pre.ldr + n) = o;
          sq += x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
        }
      }
      // the row's sum over the wave's columns: the four lanes that hold pieces of row mi
      sq += __shfl_xor(sq, 16, WAVE);
      sq += __shfl_xor(sq, 32, WAVE);
      emit_sq[a] = sq;
    } else if constexpr (MODE == D_ACC_F32) {
      floatx4 cv[NOUT];  // all loads of the residual first: a store between two loads would make the second wait
#pragma unroll
      for (int f = 0; f < NOUT; ++f) {
        const int n = (band0 + f) * 16 + nq * 4;
        cv[f] = (m < M && n < N) ? *reinterpret_cast<const floatx4*>((const float*)C + (size_t)m * ldc + n)
                                 : floatx4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int f = 0; f < NOUT; ++f) {
        const int n = (band0 + f) * 16 + nq * 4;
        if (m < M && n < N) *reinterpret_cast<floatx4*>((float*)C + (size_t)m * ldc + n) = cv[f] + acc[a][f];
      }
    } else {
      if (m >= M) continue;
#pragma unroll
      for (int f = 0; f < NOUT; ++f) {
        const int n = (band0 + f) * 16 + nq * 4;
        if (n >= N) continue;  // N is a multiple of 4: a piece is inside or outside as a whole
        if constexpr (MODE == D_STORE_F32) {
          *reinterpret_cast<floatx4*>((float*)C + (size_t)m * ldc + n) = acc[a][f];
        } else {
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r)
            v[r] = MODE == D_STORE_BF16       ? acc[a][f][r]
                   : MODE == D_STORE_BF16_PRE ? acc[a][f][r] * row_scale[a]
                   : MODE == D_SWIGLU         ? silu_f(acc[a][f][r]) * acc[a][NOUT + f][r]
                                              : silu_f(acc[a][f][r] * row_scale[a]) * (acc[a][NOUT + f][r] * row_scale[a]);
          uint2 o;
          o.x = pack_bf16x2(v[0], v[1]);
          o.y = pack_bf16x2(v[2], v[3]);
          *reinterpret_cast<uint2*>((bf16_t*)C + (size_t)m * ldc + n) = o;
        }
      }
    }
  }
  if constexpr (MODE == D_ACC_EMIT) {
    // the rows' sums of squares over the block's columns: the four waves' sums added in wave order through the LDS
    // that the stages have left
    float* sums = reinterpret_cast<float*>(&As[0][0][0]);  // [wave][BMG * 16]
    __syncthreads();
    if (nq == 0) {
#pragma unroll
      for (int a = 0; a < BMG; ++a) sums[wave * (BMG * 16) + a * 16 + mi] = emit_sq[a];
    }
    __syncthreads();
    if (tid < BMG * 16 && m0 + tid < M) {
      float sum = sums[tid];
#pragma unroll
      for (int w = 1; w < 4; ++w) sum += sums[w * (BMG * 16) + tid];
      pre.ss[(size_t)(m0 + tid) * pre.parts + pre.part0 + nt] = sum;
    }
  }
}

// What follows a product with K in slices when the row goes on to an RMS norm: the slices are added in order, then
// added into the residual, and the row for the norm is left (as D_ACC_EMIT does).  A block has 1,024 columns of a row,
// a thread four of them; ss is [M][ceil(N / 1024)].
__global__ __launch_bounds__(256) void gemm_direct_finish_emit_kernel(const float* __restrict__ partials, int k_split, int M,
                                                                      int N, float* __restrict__ C, int ldc,
                                                                      const float* __restrict__ g, bf16_t* __restrict__ raw,
                                                                      int ldr, float* __restrict__ ss) {
  __shared__ float red[4];
  const int m = blockIdx.y, n = (blockIdx.x * 256 + threadIdx.x) * 4;
  float sq = 0.f;
  if (n < N) {
    const size_t plane = (size_t)M * N;
    const float* src = partials + (size_t)m * N + n;
    floatx4 x = *reinterpret_cast<const floatx4*>(src);
    for (int s = 1; s < k_split; ++s) x += *reinterpret_cast<const floatx4*>(src + s * plane);
    floatx4* dst = reinterpret_cast<floatx4*>(C + (size_t)m * ldc + n);
    x += *dst;
    *dst = x;
    const floatx4 gv = *reinterpret_cast<const floatx4*>(g + n);
    uint2 o;
    o.x = pack_bf16x2(x[0] * gv[0], x[1] * gv[1]);
    o.y = pack_bf16x2(x[2] * gv[2], x[3] * gv[3]);
    *reinterpret_cast<uint2*>(raw + (size_t)m * ldr + n) = o;
    sq = x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
  }
  const float total = block_sum<256>(sq, red);
  if (threadIdx.x == 0) ss[(size_t)m * gridDim.x + blockIdx.x] = total;
}

template <int NF, int MODE>
__global__ __launch_bounds__(256, 1) void gemm_direct_kernel(const bf16_t* __restrict__ A, int lda,
                                                             const bf16_t* __restrict__ W,
                                                             const bf16_t* __restrict__ W2, int chunks,
                                                             void* __restrict__ C, int ldc, int M, int N, int K,
                                                             DirectPre pre) {
  direct_tile<8, NF, MODE>(blockIdx.x, A, lda, W, W2, chunks, C, ldc, M, N, K, pre);
}

// K in `gridDim.y` slices of k_slice columns: slice s leaves its float32 sums in partials[s][M][N] (the tiled product's
// finishing kernel adds the slices in order and runs the epilogue).
template <int NF>
__global__ __launch_bounds__(256, 1) void gemm_direct_slices_kernel(const bf16_t* __restrict__ A, int lda,
                                                                    const bf16_t* __restrict__ W, int chunks,
                                                                    float* __restrict__ partials, int M, int N,
                                                                    int k_slice) {
  const int s = blockIdx.y;
  direct_tile<8, NF, D_STORE_F32>(blockIdx.x, A + (size_t)s * k_slice, lda, W + (size_t)s * (k_slice / 32) * 512, nullptr,
                                  chunks, partials + (size_t)s * M * N, N, M, N, k_slice);
}

// Which NF takes a shape: a launch runs ceil(blocks / 256) rounds of one block a compute unit, and a round of blocks
// with NF bands a wave takes about 27 + 10.8 NF time units (measured at 2,048 rows with weights from HBM: 58, 74, 86, 92
// and 112 us a round of 4,096 columns of K for NF = 3, 4, 5, 6, 8); 3 and 5 bands give the 3,072 and 5,120 columns of
// a 3B model one full round.
// (Tried and taken out: one launch in which the columns of a nearly empty last round go to tiles of 64 rows.  With
// 2,048 rows x 14,336 SwiGLU outputs, 3.5 rounds of 128-row tiles, it took 589 us against 453 us: a 64-row tile moves
// 72 KiB through the load path per 64 columns of K for half the MFMAs.)
constexpr double round_cost(int nf) { return 27.0 + 10.8 * nf; }
int pick_bands(int M, int N, bool swiglu, int k_split = 1, double* cost_out = nullptr) {
  const int mt = ceil_div(M, 128);
  int best = 0;
  double best_cost = 0.0;
  for (int nf : {3, 4, 5, 6, 8}) {
    if (swiglu && nf % 2) continue;  // half of a wave's bands are gate, half up
    const int nb = 4 * (swiglu ? nf / 2 : nf) * 16;
    const long blocks = (long)mt * ceil_div(N, nb) * k_split;
    const double cost = (double)((blocks + 255) / 256) * round_cost(nf);
    if (!best || cost <= best_cost) best = nf, best_cost = cost;
  }
  if (cost_out) *cost_out = best_cost;
  return best;
}

template <int NF, int MODE>
int launch(const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M, int N, int K,
           hipStream_t stream, DirectPre pre) {
  constexpr int NB = 4 * (is_swiglu(MODE) ? NF / 2 : NF) * 16;
  const long blocks = 8L * ceil_div((long)ceil_div(N, NB) * ceil_div(M, 128), 8L);
  if (blocks > 0x7fffffffL) return APC_ERR_BAD_ARG;
  hipLaunchKernelGGL((gemm_direct_kernel<NF, MODE>), dim3((unsigned)blocks), dim3(256), 0, stream, A, lda, W, W2,
                     ceil_div(K, 32), C, ldc, M, N, K, pre);
  APC_LAUNCH_CHECK();
  return 0;
}

template <int MODE>
int launch_mode(int nf, const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M, int N,
                int K, hipStream_t stream, DirectPre pre) {
  if constexpr (!is_swiglu(MODE)) {
    if (nf == 3) return launch<3, MODE>(A, lda, W, W2, C, ldc, M, N, K, stream, pre);
    if (nf == 5) return launch<5, MODE>(A, lda, W, W2, C, ldc, M, N, K, stream, pre);
  }
  if (nf == 4) return launch<4, MODE>(A, lda, W, W2, C, ldc, M, N, K, stream, pre);
  if (nf == 6) return launch<6, MODE>(A, lda, W, W2, C, ldc, M, N, K, stream, pre);
  return launch<8, MODE>(A, lda, W, W2, C, ldc, M, N, K, stream, pre);
}

}  // namespace

// A product with few output columns fills one round of blocks only with narrow tiles (4 bands a wave for the 4,096
// columns of an 8B model at 2,048 rows), which move the most bytes through L2 per MFMA.  K in two slices gives the
// wide tiles (8 bands) a full round: down of an 8B model (K = 14,336) 276 -> 207 us plus the kernel that adds the
// slices.  Time units as in pick_bands, per 4,096 columns of K; the adding kernel about 22 units per 2,048 x 4,096
// outputs and slice pair, and a launch 3.
int gemm_direct_k_split(int M, int N, int K) {
  if (M < GEMM_DIRECT_MIN_ROWS || K % 256 || N % 4 || K < 4096) return 1;
  double whole = 0.0, halves = 0.0;
  pick_bands(M, N, false, 1, &whole);
  pick_bands(M, N, false, 2, &halves);
  const double k_units = K / 4096.0;
  const double add = 22.0 * ((double)M * N / (2048.0 * 4096.0)) + 3.0;
  return halves * k_units / 2 + add < 0.92 * whole * k_units ? 2 : 1;
}

int launch_gemm_direct_slices(const bf16_t* A, int lda, const bf16_t* W, float* partials, int M, int N, int K,
                              int k_split, hipStream_t stream) {
  if (k_split < 1 || k_split > 65535 || K % k_split) return APC_ERR_UNSUPPORTED;
  const int k_slice = K / k_split;
  if (!gemm_direct_takes(D_STORE_F32, A, lda, partials, N, M, N, k_slice)) return APC_ERR_UNSUPPORTED;
  const int nf = pick_bands(M, N, false, k_split);
  const int nb = 4 * nf * 16;
  const long blocks = 8L * ceil_div((long)ceil_div(N, nb) * ceil_div(M, 128), 8L);
  if (blocks > 0x7fffffffL) return APC_ERR_BAD_ARG;
  const dim3 grid((unsigned)blocks, (unsigned)k_split);
#define SLICES(NF_)                                                                                              \
  hipLaunchKernelGGL((gemm_direct_slices_kernel<NF_>), grid, dim3(256), 0, stream, A, lda, W, ceil_div(K, 32), partials, \
                     M, N, k_slice)
  if (nf == 3) SLICES(3);
  else if (nf == 4) SLICES(4);
  else if (nf == 5) SLICES(5);
  else if (nf == 6) SLICES(6);
  else SLICES(8);
#undef SLICES
  APC_LAUNCH_CHECK();
  return 0;
}

namespace {
bool direct_takes(int mode, int min_rows, const void* A, int lda, const void* C, int ldc, int M, int N, int K) {
  if (mode < 0 || mode > D_STORE_BF16_PRE || M < min_rows || K < 128 || K % 128 || N % 4 || ldc % 4) return false;
  if (((uintptr_t)A & 15u) || ((uintptr_t)C & 15u) || lda % 8) return false;
  // the lanes' byte offsets into the block's rows of A and the wave's bands of W are 32-bit
  if ((long)128 * lda * 2 >= 0x7fffffffL || (long)8 * ceil_div(K, 32) * 1024 >= 0x7fffffffL) return false;
  return true;
}

int launch_columns(int nf, int mode, const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M,
                   int N, int K, hipStream_t stream, DirectPre pre) {
  switch (mode) {
    case D_STORE_BF16: return launch_mode<D_STORE_BF16>(nf, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
    case D_STORE_F32: return launch_mode<D_STORE_F32>(nf, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
    case D_ACC_F32: return launch_mode<D_ACC_F32>(nf, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
    case D_SWIGLU: return launch_mode<D_SWIGLU>(nf, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
    case D_SWIGLU_PRE: return launch_mode<D_SWIGLU_PRE>(nf, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
    case D_ACC_EMIT: return launch_mode<D_ACC_EMIT>(nf, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
    default: return launch_mode<D_STORE_BF16_PRE>(nf, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
  }
}

// How a product's columns go out: one launch of tiles with nf1 bands a wave, or, where the last round of blocks would
// be far from full (2,048 rows x 14,336 SwiGLU outputs: 3.5 rounds of tiles with 8 bands a wave), the first cols1
// columns, which make whole rounds, on nf1 and the rest on whatever tile fills a round best (there: 4 bands, a round
// of 0.72 of the time).  3 time units for the second launch.
struct ColumnPlan {
  int nf1, cols1, nf2;  // cols1 == 0: one launch
};
ColumnPlan plan_columns(int M, int N, bool swiglu) {
  double whole = 0.0;
  const int nf = pick_bands(M, N, swiglu, 1, &whole);
  const int mt = ceil_div(M, 128);
  ColumnPlan plan{nf, 0, 0};
  double best = whole;
  if (mt <= 256) {
    for (int f : {3, 4, 5, 6, 8}) {
      if (swiglu && f % 2) continue;
      const int nb = 4 * (swiglu ? f / 2 : f) * 16, nt = ceil_div(N, nb);
      const int big_cols = (int)((long)mt * nt / 256 * 256 / mt);
      if (big_cols <= 0 || big_cols >= nt) continue;
      double rest = 0.0;
      const int rf = pick_bands(M, N - big_cols * nb, swiglu, 1, &rest);
      const double cost = (double)ceil_div((long)big_cols * mt, 256L) * round_cost(f) + rest + 3.0;
      if (cost < 0.97 * best) best = cost, plan = ColumnPlan{f, big_cols * nb, rf};
    }
  }
  return plan;
}
int tile_columns(int nf, bool swiglu) { return 4 * (swiglu ? nf / 2 : nf) * 16; }
// column tiles of the plan's launches together (the parts of the sums of squares that D_ACC_EMIT leaves)
int column_tiles(const ColumnPlan& plan, int N, bool swiglu) {
  if (!plan.cols1) return ceil_div(N, tile_columns(plan.nf1, swiglu));
  return plan.cols1 / tile_columns(plan.nf1, swiglu) + ceil_div(N - plan.cols1, tile_columns(plan.nf2, swiglu));
}

int launch_direct(int mode, const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M, int N,
                  int K, hipStream_t stream, DirectPre pre) {
  const bool swiglu = is_swiglu(mode);
  const ColumnPlan plan = plan_columns(M, N, swiglu);
  if (!plan.cols1) return launch_columns(plan.nf1, mode, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
  const int e = launch_columns(plan.nf1, mode, A, lda, W, W2, C, ldc, M, plan.cols1, K, stream, pre);
  if (e) return e;
  const size_t w_skip = (size_t)(plan.cols1 / 16) * ceil_div(K, 32) * 512;  // whole bands of the tiled layout
  const size_t elem = (mode == D_STORE_BF16 || mode == D_STORE_BF16_PRE || swiglu) ? 2 : 4;
  if (mode == D_ACC_EMIT) {
    pre.g += plan.cols1;
    pre.raw += plan.cols1;
    pre.part0 += plan.cols1 / tile_columns(plan.nf1, swiglu);
  }
  return launch_columns(plan.nf2, mode, A, lda, W + w_skip, swiglu ? W2 + w_skip : W2, (char*)C + (size_t)plan.cols1 * elem,
                        ldc, M, N - plan.cols1, K, stream, pre);
}
}  // namespace

bool gemm_direct_takes(int mode, const void* A, int lda, const void* C, int ldc, int M, int N, int K) {
  return mode <= D_SWIGLU && direct_takes(mode, GEMM_DIRECT_MIN_ROWS, A, lda, C, ldc, M, N, K);
}

int launch_gemm_direct(int mode, const bf16_t* A, int lda, const bf16_t* W, const bf16_t* W2, void* C, int ldc, int M,
                       int N, int K, hipStream_t stream) {
  if (!gemm_direct_takes(mode, A, lda, C, ldc, M, N, K) || (mode == D_SWIGLU) != (W2 != nullptr)) return APC_ERR_UNSUPPORTED;
  return launch_direct(mode, A, lda, W, W2, C, ldc, M, N, K, stream, DirectPre{});
}

bool gemm_direct_pre_takes(int mode, const void* A, int lda, const void* C, int ldc, int M, int N, int K, int ss_parts) {
  if (ss_parts <= 0 || (mode != D_STORE_BF16 && mode != D_SWIGLU)) return false;
  // SwiGLU's many outputs fill a round of 128-row tiles from 384 rows on; other products only where the direct kernel
  // takes them without a folded norm too
  const int min_rows = mode == D_SWIGLU ? GEMM_DIRECT_PRE_MIN_ROWS : GEMM_DIRECT_MIN_ROWS;
  return direct_takes(mode, min_rows, A, lda, C, ldc, M, N, K);
}

int launch_gemm_direct_pre(int mode, const bf16_t* A, int lda, const float* ss, int ss_parts, float eps, const bf16_t* W,
                           const bf16_t* W2, void* C, int ldc, int M, int N, int K, hipStream_t stream) {
  if (!ss || !gemm_direct_pre_takes(mode, A, lda, C, ldc, M, N, K, ss_parts) || (mode == D_SWIGLU) != (W2 != nullptr))
    return APC_ERR_UNSUPPORTED;
  DirectPre pre{};
  pre.ss = const_cast<float*>(ss);
  pre.parts = ss_parts;
  pre.eps = eps;
  return launch_direct(mode == D_SWIGLU ? D_SWIGLU_PRE : D_STORE_BF16_PRE, A, lda, W, W2, C, ldc, M, N, K, stream, pre);
}

int gemm_direct_emit_parts(const void* A, int lda, const void* C, int ldc, int M, int N, int K) {
  if (!direct_takes(D_ACC_EMIT, GEMM_DIRECT_MIN_ROWS, A, lda, C, ldc, M, N, K) || M > 65535) return 0;
  if (gemm_direct_k_split(M, N, K) > 1) return ceil_div(N, 1024);
  return column_tiles(plan_columns(M, N, false), N, false);
}

int launch_gemm_direct_emit(const bf16_t* A, int lda, const bf16_t* W, float* C, int ldc, int M, int N, int K,
                            const float* g, bf16_t* raw, int ldr, float* ss, int ss_parts, float* workspace,
                            hipStream_t stream) {
  const int parts = gemm_direct_emit_parts(A, lda, C, ldc, M, N, K);
  if (!parts || parts != ss_parts || !g || !raw || !ss || ldr < N || ldr % 4 || ((uintptr_t)raw & 7u) ||
      ((uintptr_t)g & 15u))
    return APC_ERR_UNSUPPORTED;
  const int k_split = gemm_direct_k_split(M, N, K);
  if (k_split > 1) {
    if (!workspace) return APC_ERR_BAD_ARG;
    const int e = launch_gemm_direct_slices(A, lda, W, workspace, M, N, K, k_split, stream);
    if (e) return e;
    hipLaunchKernelGGL(gemm_direct_finish_emit_kernel, dim3(parts, M), dim3(256), 0, stream, workspace, k_split, M, N, C,
                       ldc, g, raw, ldr, ss);
    APC_LAUNCH_CHECK();
    return 0;
  }
  DirectPre pre{};
  pre.ss = ss;
  pre.parts = parts;
  pre.g = g;
  pre.raw = raw;
  pre.ldr = ldr;
  pre.part0 = 0;
  return launch_direct(D_ACC_EMIT, A, lda, W, nullptr, C, ldc, M, N, K, stream, pre);
}
