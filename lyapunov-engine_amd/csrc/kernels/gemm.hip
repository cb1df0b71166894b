// C[M,N] = A[M,K] . W[N,K]^T on the matrix cores, for bfloat16 and for true
// 32-bit floats (the 32x32x2 float instruction, no reduced-precision mode).
// Both operands are row-major with the inner dimension contiguous, which is
// how a projection's weight [out_features, in_features] is stored.
//
// The reference has no kernel of its own here: its projections are nn.Linear
// calls (python/lyapunov_engine/models/llama.py:45-48, 112-117, 177).
//
// Two kernels: a tiled one for any M, N, K (rows that are not 16-byte aligned
// take a scalar load path), and one for M <= 64 that streams the weights once.
// In both the order of the additions for an output element is fixed by the
// sizes of the product alone (no atomics), so a token's result does not depend
// on which other tokens are in the batch beyond the choice of kernel, which
// follows M.
#include <algorithm>
#include <type_traits>

#include "common.h"

namespace lyp {

enum GemmMode : int {
  kStoreAct = 0,    // C has the operands' type
  kStoreF32 = 1,    // C is float
  kAccumF32 = 2,    // C is float and is added to (the residual stream)
};

template <typename T>
struct VecOf;
template <>
struct VecOf<float> {
  static constexpr int kVec = 4;
};
template <>
struct VecOf<bf16_t> {
  static constexpr int kVec = 8;
};

constexpr int kBK = 32;

template <typename T, int BM, int BN, int WGM, int WGN, int MODE>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const T* __restrict__ A,
                                                      const T* __restrict__ W, void* __restrict__ Cv,
                                                      int M, int N, int K, int lda, int ldw, int ldc,
                                                      int vec_ok) {
  static_assert(WGM * WGN == 4, "four waves per workgroup");
  constexpr int VEC = VecOf<T>::kVec;
  constexpr int KF = Mma32<T>::kElems;
  constexpr int PAD = VEC;
  constexpr int LDS_LD = kBK + PAD;
  constexpr int IM = BM / (WGM * 32);
  constexpr int JN = BN / (WGN * 32);
  static_assert(IM >= 1 && JN >= 1, "tile too small for the wave grid");
  using Frag = typename Mma32<T>::Frag;

  __shared__ __attribute__((aligned(16))) T As[BM * LDS_LD];
  __shared__ __attribute__((aligned(16))) T Ws[BN * LDS_LD];

  const int tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  const int wm = wave / WGN, wn = wave % WGN;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

  f32x16 acc[IM][JN];
#pragma unroll
  for (int i = 0; i < IM; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  constexpr int VPR = kBK / VEC;  // vectors per tile row
  typedef T VecT __attribute__((ext_vector_type(VEC)));

  auto load_tile = [&](const T* __restrict__ src, int ld, int row0, int nrows_total, int k0, T* dst,
                       int tile_rows) {
    for (int v = tid; v < tile_rows * VPR; v += 256) {
      const int r = v / VPR, cv = v % VPR;
      const int gr = row0 + r, gk = k0 + cv * VEC;
      VecT val;
      if (gr < nrows_total && vec_ok && gk + VEC <= K) {
        val = *reinterpret_cast<const VecT*>(src + static_cast<size_t>(gr) * ld + gk);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const bool in = gr < nrows_total && gk + e < K;
          val[e] = in ? src[static_cast<size_t>(gr) * ld + gk + e] : from_f32<T>(0.f);
        }
      }
      *reinterpret_cast<VecT*>(dst + r * LDS_LD + cv * VEC) = val;
    }
  };

  for (int k0 = 0; k0 < K; k0 += kBK) {
    __syncthreads();
    load_tile(A, lda, m0, M, k0, As, BM);
    load_tile(W, ldw, n0, N, k0, Ws, BN);
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kBK; kk += 2 * KF) {
      Frag a[IM], b[JN];
      const int kofs = kk + (lane / 32) * KF;
#pragma unroll
      for (int i = 0; i < IM; ++i)
        a[i] = *reinterpret_cast<const Frag*>(As + ((wm * IM + i) * 32 + lane % 32) * LDS_LD + kofs);
#pragma unroll
      for (int j = 0; j < JN; ++j)
        b[j] = *reinterpret_cast<const Frag*>(Ws + ((wn * JN + j) * 32 + lane % 32) * LDS_LD + kofs);
#pragma unroll
      for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j) acc[i][j] = Mma32<T>::mma(a[i], b[j], acc[i][j]);
    }
  }

#pragma unroll
  for (int i = 0; i < IM; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j) {
      const int n = n0 + (wn * JN + j) * 32 + lane % 32;
      if (n >= N) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + (wm * IM + i) * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
        if (m >= M) continue;
        const size_t idx = static_cast<size_t>(m) * ldc + n;
        if constexpr (MODE == kStoreAct) {
          static_cast<T*>(Cv)[idx] = from_f32<T>(acc[i][j][v]);
        } else if constexpr (MODE == kStoreF32) {
          static_cast<float*>(Cv)[idx] = acc[i][j][v];
        } else {
          static_cast<float*>(Cv)[idx] += acc[i][j][v];
        }
      }
    }
}

// ------------------------------------------------------- many rows, bfloat16
// The same product for prompt steps in bfloat16 with K a multiple of 64 and 16-byte aligned rows:
// tiles of TM tokens x TN features x 64 values of K, eight waves as 2 x 4, each with (TM / 2) x (TN / 4)
// of the output in registers as 16x16 tiles of the 16x16x32 instruction (W's rows are the row operand, so
// a lane ends with four neighbouring features of one token).  Two LDS buffers: while a step's tiles
// are multiplied, the next step's are on their way from memory into the other buffer; one barrier a step.
// Workgroups go to the chip's eight dies in turn by their number; a die keeps to its own tiles of
// features (number % 8) and walks all tiles of tokens for each, so a tile of W is read from memory by
// one die only and the activations, which are small, by all.
template <int TM, int TN>
struct WideGemm {
  static constexpr int kTK = 64;                       // values of K a step; a row of a tile is 128 bytes, eight pieces of 16
  static constexpr int kStage = (TM + TN) * kTK;       // elements of one buffer: the tokens' tile, then the features'
  static constexpr int kIM = TM / 2 / 16, kJN = TN / 4 / 16;   // 16x16 tiles of a wave
  static constexpr int kLoadsA = TM / 8 / 8, kLoadsW = TN / 8 / 8;  // load instructions per wave and step: 8 rows each
};

// One step's tiles go from memory to LDS without passing registers: a wave's load instruction brings
// 1 KB, eight rows of 128 bytes, lane l the piece at row l / 8, place l % 8.  Rows are not padded;
// instead place p of row r holds piece p ^ ((r / 2) % 8) of the row's eight, so that the 16 rows a
// fragment read touches lie in 16 different groups of four banks.
template <int TM, int TN>
__device__ __forceinline__ void wide_ask(const bf16_t* const* ga, const bf16_t* const* gw, int k0, bf16_t* stage, int wave) {
  using G = WideGemm<TM, TN>;
  using LdsPtr = __attribute__((address_space(3))) void*;
#pragma unroll
  for (int i = 0; i < G::kLoadsA; ++i)
    __builtin_amdgcn_global_load_lds(ga[i] + k0, (LdsPtr)(stage + (wave * G::kLoadsA + i) * 8 * G::kTK), 16, 0, 0);
#pragma unroll
  for (int i = 0; i < G::kLoadsW; ++i)
    __builtin_amdgcn_global_load_lds(gw[i] + k0, (LdsPtr)(stage + TM * G::kTK + (wave * G::kLoadsW + i) * 8 * G::kTK), 16, 0, 0);
}

// this wave's loads have arrived (the count of outstanding vector memory loads is zero; the other counters are left alone)
__device__ __forceinline__ void wide_arrived() { __builtin_amdgcn_s_waitcnt(0x0F70); }

template <int TM, int TN, int MODE>
__global__ __launch_bounds__(512) void gemm_bf16_wide_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                             void* __restrict__ Cv, int M, int N, int K, int lda, int ldw,
                                                             int ldc, int m_tiles, int n_tiles) {
  using G = WideGemm<TM, TN>;
  constexpr int IM = G::kIM, JN = G::kJN, TK = G::kTK;
  // two buffers
  __shared__ __attribute__((aligned(1024))) bf16_t stage0[G::kStage];
  __shared__ __attribute__((aligned(1024))) bf16_t stage1[G::kStage];

  // which tile: die = number % 8 owns the feature tiles die, die + 8, ...
  const int id = blockIdx.x;
  const int die = id % 8, local = id / 8;
  if (local >= ((n_tiles - die + 7) / 8) * m_tiles) return;   // the launch is rounded up to whole rounds of eight
  const int nt = die + 8 * (local / m_tiles), mt = local % m_tiles;
  const int m0 = mt * TM, n0 = nt * TN;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / 4, wn = wave % 4;
  const int r = lane % 16, j = lane / 16;

  // this lane's piece of each of the wave's load instructions
  const bf16_t* ga[G::kLoadsA];
  const bf16_t* gw[G::kLoadsW];
  {
    const int row8 = lane / 8, place = lane % 8;
#pragma unroll
    for (int i = 0; i < G::kLoadsA; ++i) {
      const int row = (wave * G::kLoadsA + i) * 8 + row8;
      ga[i] = A + static_cast<size_t>(min(m0 + row, M - 1)) * lda + (place ^ ((row / 2) % 8)) * 8;
    }
#pragma unroll
    for (int i = 0; i < G::kLoadsW; ++i) {
      const int row = (wave * G::kLoadsW + i) * 8 + row8;
      gw[i] = W + static_cast<size_t>(min(n0 + row, N - 1)) * ldw + (place ^ ((row / 2) % 8)) * 8;
    }
  }

  f32x4 acc[IM][JN];
#pragma unroll
  for (int i = 0; i < IM; ++i)
#pragma unroll
    for (int jn = 0; jn < JN; ++jn) acc[i][jn] = f32x4{0.f, 0.f, 0.f, 0.f};

  // fragment of values 32 kk + 8 j .. of row r of a 16-row tile: piece 4 kk + j, at place (4 kk + j) ^ (r / 2)
  const int a_frag = (wm * (TM / 2) + r) * TK + (j ^ (r / 2)) * 8;              // + i * 16 * TK, ^ 32 for kk = 1
  const int w_frag = TM * TK + (wn * (TN / 4) + r) * TK + (j ^ (r / 2)) * 8;    // + jn * 16 * TK

  auto ask = [&](int k0, bf16_t* stage) { wide_ask<TM, TN>(ga, gw, k0, stage, wave); };
  // A half step: every fragment first, then the products (the scheduler is told so: left alone it
  // asks for two fragments at a time and waits for them before every eight products).
  auto step = [&](const bf16_t* stage) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      // (the second half of the step's 64 values: four pieces on, which in a swizzled row is the place with bit 2 flipped)
      const bf16_t* wrow = stage + (kk == 0 ? w_frag : w_frag ^ 32);
      const bf16_t* arow = stage + (kk == 0 ? a_frag : a_frag ^ 32);
      bf16x8 wf[JN], xf[IM];
#pragma unroll
      for (int jn = 0; jn < JN; ++jn) wf[jn] = *reinterpret_cast<const bf16x8*>(wrow + jn * 16 * TK);
#pragma unroll
      for (int i = 0; i < IM; ++i) xf[i] = *reinterpret_cast<const bf16x8*>(arow + i * 16 * TK);
#pragma unroll
      for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int jn = 0; jn < JN; ++jn) acc[i][jn] = Mma16Wide<bf16_t>::mma(wf[jn], xf[i], acc[i][jn]);
      __builtin_amdgcn_sched_group_barrier(0x100, IM + JN, 0);   // LDS reads
      __builtin_amdgcn_sched_group_barrier(0x008, IM * JN, 0);   // matrix instructions
    }
  };
  // (Letting the workgroups that share a tile of W start at different places of K, so that one of them asks
  // memory for a slice and the others find it in the die's cache, was measured: 5 % slower.  They walk K in
  // step, and the cache merges their requests.)
  const int steps = K / TK;
  ask(0, stage0);
  wide_arrived();
  __syncthreads();
  bf16_t* cur = stage0;
  bf16_t* nxt = stage1;
#pragma unroll 1
  for (int s = 0; s < steps; ++s) {
    if (s + 1 < steps) ask((s + 1) * TK, nxt);
    __builtin_amdgcn_sched_barrier(0);   // the loads go out before the products, not where the scheduler finds room for them
    step(cur);
    wide_arrived();
    __syncthreads();
    bf16_t* t = cur;
    cur = nxt;
    nxt = t;
  }

  // acc[i][jn][v]: token m0 + wm TM/2 + 16 i + r, feature n0 + wn TN/4 + 16 jn + 4 j + v
#pragma unroll
  for (int i = 0; i < IM; ++i) {
    const int m = m0 + wm * (TM / 2) + 16 * i + r;
    if (m >= M) continue;
#pragma unroll
    for (int jn = 0; jn < JN; ++jn) {
      const int n = n0 + wn * (TN / 4) + 16 * jn + 4 * j;
      if (n >= N) continue;
      const size_t idx = static_cast<size_t>(m) * ldc + n;
      const bool whole = n + 3 < N && ldc % 4 == 0;
      if constexpr (MODE == kStoreAct) {
        bf16_t* dst = static_cast<bf16_t*>(Cv) + idx;
        if (whole) {
          bf16x4 o;
#pragma unroll
          for (int v = 0; v < 4; ++v) o[v] = from_f32<bf16_t>(acc[i][jn][v]);
          *reinterpret_cast<bf16x4*>(dst) = o;
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (n + v < N) dst[v] = from_f32<bf16_t>(acc[i][jn][v]);
        }
      } else {
        float* dst = static_cast<float*>(Cv) + idx;
        if (whole) {
          f32x4 o = acc[i][jn];
          if constexpr (MODE == kAccumF32) o += *reinterpret_cast<const f32x4*>(dst);
          *reinterpret_cast<f32x4*>(dst) = o;
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (n + v < N) dst[v] = MODE == kAccumF32 ? dst[v] + acc[i][jn][v] : acc[i][jn][v];
        }
      }
    }
  }
}

// ---------------------------------------------------------------- few rows
// M <= 64 (decode steps): the weight matrix is read once from memory and the
// time is what that read takes, so the shape is chosen for memory parallelism.
// A workgroup owns 16 rows of W (16 output features) and, when the matrix has
// few rows, one of several slices of the inner dimension (grid.y); its waves
// split the slice between them and add their parts through LDS, in a fixed
// order.  A wave keeps the 16 x (16 MB) output tile in registers: W rows are the
// row operand, tokens the columns.  Per 64 values of the inner dimension a lane
// reads one contiguous run of 16 values of its row; activations come through
// the cache, they are small.  Needs K % 64 == 0 and 16-byte aligned rows.
//
// Epilogues: store in the operands' type; store float; SiLU-gate (rows 0-7 of
// the tile are gate features, rows 8-15 the matching up features: the output
// has half as many columns); float partial sums per slice, [slice][M][N],
// which the consumer adds up (the RMSNorm kernels do); or the whole tail of a
// fused q/k/v projection: rotate query and key heads by position and put keys
// and values into their pages.
enum SkinnyEpilogue : int {
  kEpiAct = 0, kEpiF32 = 1, kEpiSwiglu = 2, kEpiParts = 3, kEpiRope = 4,
  kEpiResidual = 5,  // C is the float residual stream: C += A . W^T
};

// The residual epilogue's by-products for the RMS norm that follows: with
// h' = h + A . W^T it also stores xs = h' * next_weight (rounded to the
// operands' type, not yet divided by the row's rms) and, per workgroup, the
// sum of h'^2 over the workgroup's features.
struct ResidualTail {
  const void* next_w;  // [N] the following norm's weights; null: no by-products
  int next_w_f32;
  void* xs;            // [M][ldx]
  int ldx;
  float* ssq_part;     // [workgroups][16]: rows past M get zeros
};

// For a product whose activations are such an xs: the sums are scaled by the
// row's 1 / sqrt(mean(h'^2) + eps), from the n_parts partial sums of squares
// (added up in a fixed order), before the epilogue proper.  `width` is the
// number of features of h'.
struct NormHead {
  const float* ssq_part;  // [n_parts][16]
  int n_parts, width;
  float eps;
};

// What the rotating epilogue needs.  W's rows are heads of `hd` features: nh
// query heads, then (has_kv) nkv key heads and nkv value heads.  In the first
// `rot` features of a query or key head, feature i < rot / 2 is rotated with
// feature i + rot / 2 (rope_kv_kernel has the formula); a workgroup of such a
// region therefore does not take 16 neighbouring rows of W but features
// 8 t .. 8 t + 7 and their partners, so that both halves of a pair meet in it.
struct RopeTail {
  const int32_t* positions;  // [M]
  const float* cos_sin;      // [max_pos][rot]: cosines, then sines; unused when rot == 0
  const int32_t* slots;      // [M] page * bs + offset of the token's key and value, -1: not stored
  void* kpool;               // [page][nkv][bs][hd]
  void* vpool;               // [page][nkv][hd][bs]
  int nh, nkv, hd, rot, bs, has_kv;
};

// The feature (row of W, column of the output) that row r of the 16-row tile at n0 stands for.
__device__ __forceinline__ int rope_feature(const RopeTail& t, int n0, int r) {
  const int head = n0 / t.hd, blk = (n0 % t.hd) / 16;
  const bool rotated = head < t.nh + (t.has_kv ? t.nkv : 0) && blk < t.rot / 16;
  const int f = rotated ? (r < 8 ? 8 * blk + r : t.rot / 2 + 8 * blk + (r - 8)) : 16 * blk + r;
  return head * t.hd + f;
}

// PAIRED (8 rows of W, or two tiles of 8; at most 8 tokens): the tile's upper half repeats the 8 rows of W and the
// tile's upper 8 columns the tokens, both 64 values of K further on, so that one matrix instruction
// does two chunks of K (on the tile's diagonal blocks; the other two are not used) and no load
// asks for a value twice.  With TB = 2 (9 to 16 tokens, 8 rows of W) a wave keeps two such tiles over
// one set of weights: tokens 0-7 and 8-15.
// RT > 1 (steps of 17 to 64 tokens): a workgroup owns RT tiles of 16 rows of W, and a wave keeps all of them
// over one set of activations: what a compute unit asks the cache for per row of W falls accordingly.
template <typename T, int MB, int EPI, bool NORMED = false, int ROWS = 16, bool PAIRED = false, int TB = 1, int RT = 1>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(const T* __restrict__ A, const T* __restrict__ W,
                                                           void* __restrict__ Cv, int M, int N, int K, int lda,
                                                           int ldw, int ldc, RopeTail tail, NormHead head,
                                                           ResidualTail res) {
  using MM = Mma16Wide<T>;
  using Frag = typename MM::Frag;
  constexpr int NF = 16 / MM::kElems;  // fragments per lane per 64 values of K
  static_assert(ROWS == 16 || ROWS == 8, "a workgroup owns 16 rows of W, or 8 (the tile's lower half repeats them)");
  // With 16 rows of W a paired wave keeps two tiles, rows 0-7 and 8-15, over the same tokens: MB counts them.
  static_assert(!PAIRED || (EPI == kEpiResidual && ((ROWS == 8 && MB == 1) || (ROWS == 16 && MB == 2))),
                "two chunks per tile: 8 rows (or twice 8), 8 tokens");
  static_assert(TB == 1 || (TB == 2 && PAIRED && MB == 1), "blocks of 8 tokens: for the paired tile of 8 rows");
  static_assert(RT == 1 || (!PAIRED && !NORMED && ROWS == 16 && EPI != kEpiResidual), "several row tiles: the plain tile only");
  constexpr int NT = MB * TB * RT;           // tiles (accumulators) a wave keeps: tile rt * MB + b is row tile rt, token block b
  constexpr int NB = PAIRED ? TB : MB;       // blocks of tokens whose activations it loads
  constexpr int CHUNK = PAIRED ? 128 : 64;  // values of K per step of a wave
  extern __shared__ float red[];       // [waves][NT][64][4], then [waves][16] floats for the epilogues' row values

  const int lane = threadIdx.x % kWave;
  // the same in every lane, and said so: the loop over this wave's share of K then has scalar bounds and
  // can be unrolled, which is what keeps several chunks' loads in flight
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int nwaves = blockDim.x / kWave;
  const int n0 = blockIdx.x * ROWS * RT;
  const int r = lane % 16, j = lane / 16;
  int wrow = min(n0 + r % (PAIRED ? 8 : ROWS), N - 1);  // rows past the end read the last row and are not stored
  if constexpr (EPI == kEpiRope) wrow = rope_feature(tail, n0, r);  // N is a multiple of 16 here

  const int chunks = K / CHUNK;
  const int per_slice = (chunks + gridDim.y - 1) / gridDim.y;
  const int s_begin = min(chunks, static_cast<int>(blockIdx.y) * per_slice), s_end = min(chunks, s_begin + per_slice);
  const int per_wave = (s_end - s_begin + nwaves - 1) / nwaves;
  const int c_begin = min(s_end, s_begin + wave * per_wave), c_end = min(s_end, c_begin + per_wave);

  f32x4 acc[NT];
#pragma unroll
  for (int b = 0; b < NT; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Small loads that the epilogue needs are started here, ahead of the stream of weights.
  float* row_val = red + static_cast<size_t>(nwaves) * NT * 256;  // [waves][16]
  if constexpr (NORMED) {
    // Every token's sum of squares, from the producer's partial sums [parts][16]: thread t adds up
    // four tokens (t % 4) over every (threads / 4)-th part, the lanes of a wave meet by shuffles, the
    // waves in the epilogue (row_val[wave][token]).  The order is fixed by the launch.
    static_assert(MB == 1, "sums of squares come for at most 16 rows");
    const f32x4* src = reinterpret_cast<const f32x4*>(head.ssq_part);
    const int n4 = head.n_parts * 4;  // 16-byte pieces: piece i holds tokens 4 (i % 4) .. + 3 of part i / 4
    f32x4 sq = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int base = threadIdx.x; base < n4; base += 4 * blockDim.x) {
      f32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int idx = base + u * blockDim.x;
        v[u] = idx < n4 ? src[idx] : f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) sq += v[u];
    }
#pragma unroll
    for (int off = 4; off < kWave; off *= 2)
#pragma unroll
      for (int i = 0; i < 4; ++i) sq[i] += __shfl_xor(sq[i], off, kWave);
    if (lane < 4) *reinterpret_cast<f32x4*>(row_val + wave * 16 + 4 * lane) = sq;
  }
  float h_first = 0.f, nw_first = 0.f;  // kEpiResidual: what the thread's first element adds to and is weighted by
  if constexpr (EPI == kEpiResidual) {
    const int e = threadIdx.x, l = (e % 256) / 4, in_tile = 4 * (l / 16) + e % 4;
    const int row = PAIRED ? 8 * (e / 256 / TB) + in_tile : in_tile;
    const int m = (PAIRED ? 8 * (e / 256 % TB) : (e / 256) * 16) + l % 16, n = n0 + row;
    if (e < NT * 256 && in_tile < (PAIRED ? 8 : ROWS) && (!PAIRED || l % 16 < 8) && m < M && n < N) {
      h_first = static_cast<const float*>(Cv)[static_cast<size_t>(m) * ldc + n];
      if (res.next_w)
        nw_first = res.next_w_f32 ? static_cast<const float*>(res.next_w)[n]
                                  : to_f32(static_cast<const bf16_t*>(res.next_w)[n]);
    }
  }

  // kEpiRope: the position and the cache slot of the token that the thread's first element belongs
  // to are asked for now, and the cosine and sine after the products, while the waves' sums meet in LDS;
  // the epilogue would otherwise walk from one to the next, a trip to memory each.
  int pos_first = 0, slot_first = -1;
  float cos_first = 1.f, sin_first = 0.f;
  [[maybe_unused]] auto rope_first = [&](int e, int& m, int& fi, bool& rotated) {
    const int l = (e % 256) / 4, row = 4 * (l / 16) + e % 4;
    const int tile_n0 = n0 + 16 * (RT == 1 ? 0 : e / 256 / MB);
    const int head_ix = tile_n0 / tail.hd, blk = (tile_n0 % tail.hd) / 16;
    m = (RT == 1 ? e / 256 : (e / 256) % MB) * 16 + l % 16;
    rotated = head_ix < tail.nh + (tail.has_kv ? tail.nkv : 0) && blk < tail.rot / 16 && row < 8;
    fi = 8 * blk + row;
    return e < NT * 256 && m < M && tile_n0 < N;
  };
  if constexpr (EPI == kEpiRope) {
    int m, fi;
    bool rotated;
    if (rope_first(threadIdx.x, m, fi, rotated)) {
      pos_first = tail.positions[m];
      if (tail.has_kv) slot_first = tail.slots[m];
    }
  }

  // of 64 values of K, fragment f of lane group j holds values 4 E f + E j .. + E - 1 (E = MM::kElems): the
  // four lane groups of one load instruction read 4 E neighbouring values of a row, whole 64-byte pieces
  const int second = PAIRED ? (r / 8) * 64 : 0;  // the tile's upper half: the chunk's second 64 values
  const T* wp = W + static_cast<size_t>(wrow) * ldw + j * MM::kElems + second;
  const T* wpt[RT];        // the further row tiles' rows (a tile past the end of W reads its last row and is not stored)
  wpt[0] = wp;
#pragma unroll
  for (int rt = 1; rt < RT; ++rt) {
    int row = min(n0 + 16 * rt + r, N - 1);
    if constexpr (EPI == kEpiRope) row = n0 + 16 * rt < N ? rope_feature(tail, n0 + 16 * rt, r) : N - 1;
    wpt[rt] = W + static_cast<size_t>(row) * ldw + j * MM::kElems;
  }
  const T* wp_upper = wp;  // PAIRED with 16 rows: the same lanes' rows 8-15
  if constexpr (PAIRED && MB == 2) wp_upper = W + static_cast<size_t>(min(n0 + 8 + r % 8, N - 1)) * ldw + j * MM::kElems + second;
  const T* ap[NB];  // rows past the end read the last row and are not stored
#pragma unroll
  for (int b = 0; b < NB; ++b)
    ap[b] = A + static_cast<size_t>(min(PAIRED ? 8 * b + r % 8 : b * 16 + r, M - 1)) * lda + j * MM::kElems + second;

  // U chunks of 64 values of K at once: all of their loads are asked for before the first product
  // needs one.  (The matrix instruction counts as a convergent operation, and the compiler does not
  // unroll a loop of unknown length around one by itself: hence the two loops written out.)
  auto chunks_at = [&](auto count, int c) {
    constexpr int U = decltype(count)::value;
    Frag wf[U][NF];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int f = 0; f < NF; ++f)
        wf[u][f] = *reinterpret_cast<const Frag*>(wp + (c + u) * CHUNK + f * 4 * MM::kElems);
    if constexpr (PAIRED && MB == 2) {  // two tiles of weights over one set of activations
      Frag wu[U][NF], xf[U][NF];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          wu[u][f] = *reinterpret_cast<const Frag*>(wp_upper + (c + u) * CHUNK + f * 4 * MM::kElems);
          xf[u][f] = *reinterpret_cast<const Frag*>(ap[0] + (c + u) * CHUNK + f * 4 * MM::kElems);
        }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          acc[0] = MM::mma(wf[u][f], xf[u][f], acc[0]);
          acc[1] = MM::mma(wu[u][f], xf[u][f], acc[1]);
        }
      return;
    }
    Frag wx[RT > 1 ? RT - 1 : 1][U][NF];
    if constexpr (RT > 1) {
#pragma unroll
      for (int rt = 1; rt < RT; ++rt)
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int f = 0; f < NF; ++f)
            wx[rt - 1][u][f] = *reinterpret_cast<const Frag*>(wpt[rt] + (c + u) * CHUNK + f * 4 * MM::kElems);
    }
    // the activations come from the cache: four chunks of them at a time are enough
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
      for (int u0 = 0; u0 < U; u0 += 4) {
        constexpr int V = U < 4 ? U : 4;
        Frag xf[V][NF];
#pragma unroll
        for (int u = 0; u < V; ++u)
#pragma unroll
          for (int f = 0; f < NF; ++f)
            xf[u][f] = *reinterpret_cast<const Frag*>(ap[b] + (c + u0 + u) * CHUNK + f * 4 * MM::kElems);
#pragma unroll
        for (int u = 0; u < V; ++u)
#pragma unroll
          for (int f = 0; f < NF; ++f) {
            acc[b] = MM::mma(wf[u0 + u][f], xf[u][f], acc[b]);
            if constexpr (RT > 1) {
#pragma unroll
              for (int rt = 1; rt < RT; ++rt) acc[rt * MB + b] = MM::mma(wx[rt - 1][u0 + u][f], xf[u][f], acc[rt * MB + b]);
            }
          }
      }
    }
  };
  int c = c_begin;
  // (a wave whose share is two or three chunks asks for two of them at once rather than one after the
  // other: the second chunk's loads would otherwise wait for the first chunk's products, a trip to memory more)
  if constexpr (RT == 1) {
    for (; c + 4 <= c_end; c += 4) chunks_at(std::integral_constant<int, 4>{}, c);
  }
  for (; c + 2 <= c_end; c += 2) chunks_at(std::integral_constant<int, 2>{}, c);  // (several row tiles: two at a time at most)
  for (; c < c_end; ++c) chunks_at(std::integral_constant<int, 1>{}, c);

  if constexpr (EPI == kEpiRope) {
    int m, fi;
    bool rotated;
    if (rope_first(threadIdx.x, m, fi, rotated) && rotated) {
      const float* cs = tail.cos_sin + static_cast<size_t>(pos_first) * tail.rot;
      cos_first = cs[fi];
      sin_first = cs[tail.rot / 2 + fi];
    }
  }
  // acc[rt * MB + b][i]: output feature n0 + 16 rt + 4 j + i, token 16 b + r
  float* mine = red + (static_cast<size_t>(wave) * NT * 64 + lane) * 4;
#pragma unroll
  for (int b = 0; b < NT; ++b) *reinterpret_cast<f32x4*>(mine + b * 256) = acc[b];
  __syncthreads();
  // The sum over the waves, in order; NORMED: times the row's 1 / rms.
  auto total = [&](int e) {
    float sum = 0.f;
    for (int w = 0; w < nwaves; ++w) sum += red[static_cast<size_t>(w) * NT * 256 + e];
    if constexpr (PAIRED) {  // row + 8, token + 8: the chunks' second halves
      float upper = 0.f;
      for (int w = 0; w < nwaves; ++w) upper += red[static_cast<size_t>(w) * NT * 256 + e + 160];
      sum += upper;
    }
    if constexpr (NORMED) {
      float sq = 0.f;
      for (int w = 0; w < nwaves; ++w) sq += row_val[w * 16 + ((e % 256) / 4) % 16];
      sum *= 1.0f / sqrtf(sq / static_cast<float>(head.width) + head.eps);
    }
    return sum;
  };
  float* sq_el = row_val + nwaves * 16;  // kEpiResidual with by-products: [NT][256] squares of the new h, by element
  const int n0_wg = n0;
  for (int e = threadIdx.x; e < NT * 256; e += blockDim.x) {
    const int b = RT == 1 ? e / 256 : (e / 256) % MB, l = (e % 256) / 4, i = e % 4;
    const int n0 = RT == 1 ? n0_wg : n0_wg + 16 * (e / 256 / MB);   // this tile's first row of W
    if (RT > 1 && n0 >= N) continue;
    const int in_tile = 4 * (l / 16) + i;
    // PAIRED: tile b holds rows 8 (b / TB) .. + 7 of W for tokens 8 (b % TB) .. + 7 (its lower left block; the
    // upper right one is added by total()); else rows 0-15 for tokens 16 b .. + 15
    const int row = PAIRED ? 8 * (b / TB) + in_tile : in_tile;
    const int m = (PAIRED ? 8 * (b % TB) : b * 16) + l % 16, n = n0 + row;
    if (in_tile >= (PAIRED ? 8 : ROWS) || (PAIRED && l % 16 >= 8) || m >= M || n >= N) continue;
    if constexpr (EPI == kEpiRope) {
      const int head = n0 / tail.hd, blk = (n0 % tail.hd) / 16;
      const bool is_q = head < tail.nh, is_k = !is_q && head < tail.nh + tail.nkv;
      const bool rotated = (is_q || is_k) && blk < tail.rot / 16;
      if (rotated && row >= 8) continue;  // done by the thread of the partner
      // as two kernels would do it: the product rounded to the activations' type, then rotated
      T y0 = from_f32<T>(total(e)), y1 = y0;
      int f0 = 16 * blk + row, f1 = f0;
      const bool first = e == static_cast<int>(threadIdx.x);
      if (rotated) {
        const int half = tail.rot / 2, fi = 8 * blk + row;
        float c = cos_first, sn = sin_first;
        if (!first) {
          const float* cs = tail.cos_sin + static_cast<size_t>(tail.positions[m]) * tail.rot;
          c = cs[fi], sn = cs[half + fi];
        }
        const float x0 = to_f32(y0), x1 = to_f32(from_f32<T>(total(e + 128)));  // the same token, row + 8
        float r0, r1;
        rotate_pair(x0, x1, c, sn, r0, r1);
        y0 = from_f32<T>(r0);
        y1 = from_f32<T>(r1);
        f0 = fi;
        f1 = fi + half;
      }
      if (is_q) {
        T* orow = static_cast<T*>(Cv) + static_cast<size_t>(m) * ldc + head * tail.hd;
        orow[f0] = y0;
        if (rotated) orow[f1] = y1;
        continue;
      }
      const int slot = first ? slot_first : tail.slots[m];
      if (slot < 0) continue;
      const size_t page = slot / tail.bs, off = slot % tail.bs;
      if (is_k) {
        T* krow = static_cast<T*>(tail.kpool) + ((page * tail.nkv + (head - tail.nh)) * tail.bs + off) * tail.hd;
        krow[f0] = y0;
        if (rotated) krow[f1] = y1;
      } else {
        T* vhead = static_cast<T*>(tail.vpool) + (page * tail.nkv + (head - tail.nh - tail.nkv)) * tail.hd * tail.bs;
        vhead[static_cast<size_t>(f0) * tail.bs + off] = y0;
      }
    } else if constexpr (EPI == kEpiSwiglu) {
      if (row >= 8) continue;
      const float gate = total(e), up = total(e + 128);  // the same token, row + 8
      static_cast<T*>(Cv)[static_cast<size_t>(m) * ldc + (n0 / 2 + row)] =
          from_f32<T>((gate / (1.0f + expf(-gate))) * up);
    } else if constexpr (EPI == kEpiResidual) {
      float* hp = static_cast<float*>(Cv) + static_cast<size_t>(m) * ldc + n;
      const bool first = e == static_cast<int>(threadIdx.x);
      const float v = (first ? h_first : *hp) + total(e);
      *hp = v;
      if (res.next_w) {
        const float nw = first ? nw_first
                               : (res.next_w_f32 ? static_cast<const float*>(res.next_w)[n]
                                                 : to_f32(static_cast<const bf16_t*>(res.next_w)[n]));
        static_cast<T*>(res.xs)[static_cast<size_t>(m) * res.ldx + n] = from_f32<T>(v * nw);
        sq_el[e] = v * v;
      }
    } else if constexpr (EPI == kEpiParts) {
      static_cast<float*>(Cv)[(static_cast<size_t>(blockIdx.y) * M + m) * ldc + n] = total(e);
    } else if constexpr (EPI == kEpiF32) {
      static_cast<float*>(Cv)[static_cast<size_t>(m) * ldc + n] = total(e);
    } else {
      static_cast<T*>(Cv)[static_cast<size_t>(m) * ldc + n] = from_f32<T>(total(e));
    }
  }
  if constexpr (EPI == kEpiResidual) {
    if (res.next_w) {
      // A token's squares over this workgroup's features, added up in a fixed order (features past
      // the end of the matrix left no square behind).
      __syncthreads();
      for (int t = threadIdx.x; t < 16; t += blockDim.x) {  // rows that do not exist leave a zero
        const int m = t;
        float sq = 0.f;
        for (int row = 0; row < ROWS && n0 + row < N && m < M; ++row) {
          const int in_tile = PAIRED ? row % 8 : row;
          sq += sq_el[(PAIRED ? 256 * ((row / 8) * TB + t / 8) + 4 * (t % 8 + 16 * (in_tile / 4))
                              : 4 * (t % 16 + 16 * (in_tile / 4))) + in_tile % 4];
        }
        res.ssq_part[static_cast<size_t>(blockIdx.x) * 16 + m] = sq;
      }
    }
  }
}


// ------------------------------------------------------------ the output head
// Float logits of few rows (a decode step's) against a matrix of very many rows: C[M, N] = A . W^T
// with N in the hundred thousands.  The work is one long read of W, and such a read is fastest
// with few, long-lived waves (two workgroups of four waves per compute unit reached 6.1 TB/s in a
// plain read of this size, one wave per 16 rows of W as gemm_skinny_kernel would have it 4.6-4.8):
// a wave here takes 16 rows of W at a time, all of K, and then the next 16 that are its turn.
// With `cand` every workgroup also leaves, per token, the largest logit among the rows it computed
// and the first place it stands at: cand[token][workgroup].  The sampler then needs no pass over
// the row to find the maximum.
template <typename T, int MB>
__global__ __launch_bounds__(256) void lm_head_kernel(const T* __restrict__ A, const T* __restrict__ W,
                                                      float* __restrict__ C, int M, int N, int K, int lda, int ldw,
                                                      int ldc, ArgMax* __restrict__ cand) {
  using MM = Mma16Wide<T>;
  using Frag = typename MM::Frag;
  constexpr int NF = 16 / MM::kElems;
  constexpr int kWaves = 4;
  __shared__ ArgMax s_best[kWaves][MB][16];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int r = lane % 16, j = lane / 16;
  const int row_blocks = (N + 15) / 16, chunks = K / 64;
  const T* ap[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) ap[b] = A + static_cast<size_t>(min(b * 16 + r, M - 1)) * lda + j * MM::kElems;
  ArgMax best[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) best[b] = ArgMax{LYP_NEG_INF, 0x7fffffff};

  for (int blk = blockIdx.x * kWaves + wave; blk < row_blocks; blk += gridDim.x * kWaves) {
    const int n0 = blk * 16;
    const T* wp = W + static_cast<size_t>(min(n0 + r, N - 1)) * ldw + j * MM::kElems;
    f32x4 acc[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    auto chunks_at = [&](auto count, int c) {
      constexpr int U = decltype(count)::value;
      Frag wf[U][NF];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int f = 0; f < NF; ++f) wf[u][f] = *reinterpret_cast<const Frag*>(wp + (c + u) * 64 + f * 4 * MM::kElems);
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        Frag xf[U][NF];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int f = 0; f < NF; ++f) xf[u][f] = *reinterpret_cast<const Frag*>(ap[b] + (c + u) * 64 + f * 4 * MM::kElems);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int f = 0; f < NF; ++f) acc[b] = MM::mma(wf[u][f], xf[u][f], acc[b]);
      }
    };
    int c = 0;
    for (; c + 4 <= chunks; c += 4) chunks_at(std::integral_constant<int, 4>{}, c);
    for (; c < chunks; ++c) chunks_at(std::integral_constant<int, 1>{}, c);

    // acc[b][i]: row n0 + 4 j + i of W (a logit's index), token 16 b + r
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const int m = 16 * b + r, n = n0 + 4 * j;
      ArgMax mine{LYP_NEG_INF, 0x7fffffff};
      if (m < M) {
        float* crow = C + static_cast<size_t>(m) * ldc + n;
        if (n + 3 < N && ldc % 4 == 0) {
          *reinterpret_cast<f32x4*>(crow) = acc[b];
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) crow[i] = acc[b][i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) mine = better(mine, ArgMax{acc[b][i], n + i});
      }
      if (cand) {
#pragma unroll
        for (int off = 16; off < kWave; off *= 2) mine = better(mine, ArgMax{__shfl_xor(mine.v, off, kWave), __shfl_xor(mine.i, off, kWave)});
        best[b] = better(best[b], mine);
      }
    }
  }
  if (cand) {
    if (j == 0)
#pragma unroll
      for (int b = 0; b < MB; ++b) s_best[wave][b][r] = best[b];
    __syncthreads();
    for (int t = threadIdx.x; t < MB * 16; t += blockDim.x) {
      if (t >= M) continue;
      ArgMax a = s_best[0][t / 16][t % 16];
      for (int w = 1; w < kWaves; ++w) a = better(a, s_best[w][t / 16][t % 16]);
      cand[static_cast<size_t>(t) * gridDim.x + blockIdx.x] = a;
    }
  }
}

// The same for at most 16 tokens of bfloat16, as one steady stream.  The tokens' activations are put
// into LDS once (16 rows of K values, a row's start shifted by 16 bytes against the one before so
// that the 16 rows a fragment read touches lie in different banks); after that a wave asks global
// memory for nothing but weights, RING chunks of 64 values ahead, across the end of its 16 rows of W
// into the next 16 that are its turn.  Loads come back in the order they were asked for, so an
// activation fetched from global memory between the weights would wait for every weight asked
// before it; from LDS it does not.  One workgroup per compute unit is enough to keep the memory busy
// (8 tokens on 128256 x 2048: 256 workgroups 106.5 us, 512 107.0, 1024 111.5, against 115.7 of
// lm_head_kernel; 16 tokens 114 against 131, one token 100 against 105).
// MB blocks of 16 tokens (what LDS holds of them: 32 tokens of 2,048 values): a fragment of weights is then used MB times.
template <int RING, int MB>
__global__ __launch_bounds__(256) void lm_head_stream_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                             float* __restrict__ C, int M, int N, int K, int lda, int ldw,
                                                             int ldc, ArgMax* __restrict__ cand) {
  using MM = Mma16Wide<bf16_t>;
  constexpr int kWaves = 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char x_lds[];   // [16 MB][2 K + 16] bytes
  __shared__ ArgMax s_best[kWaves][MB][16];
  const int row_bytes = 2 * K + 16;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int r = lane % 16, j = lane / 16;
  const int chunks = K / 64;
  const int tiles = (N + 15) / 16;
  const int stride = gridDim.x * kWaves;
  int tile = static_cast<int>(blockIdx.x) * kWaves + wave;
  // the first weights are asked for before the activations are staged; a wave without a tile reads the last one's
  const bf16_t* wp = W + static_cast<size_t>(min(min(tile, tiles - 1) * 16 + r, N - 1)) * ldw + j * 8;
  bf16x8 wf[RING][2];
#pragma unroll
  for (int u = 0; u < RING; ++u)
#pragma unroll
    for (int f = 0; f < 2; ++f) wf[u][f] = *reinterpret_cast<const bf16x8*>(wp + min(u, chunks - 1) * 64 + f * 32);
  for (int p = tid; p < 16 * MB * (K / 8); p += 256) {
    const int row = p / (K / 8), c16 = p % (K / 8);
    *reinterpret_cast<bf16x8*>(x_lds + row * row_bytes + c16 * 16) =
        *reinterpret_cast<const bf16x8*>(A + static_cast<size_t>(min(row, M - 1)) * lda + c16 * 8);
  }
  __syncthreads();
  const unsigned char* xl = x_lds + r * row_bytes + j * 16;
  ArgMax best[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) best[b] = ArgMax{LYP_NEG_INF, 0x7fffffff};
  for (; tile < tiles; tile += stride) {
    const bf16_t* wn = W + static_cast<size_t>(min(min(tile + stride, tiles - 1) * 16 + r, N - 1)) * ldw + j * 8;
    f32x4 acc[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int c = 0; c < chunks; c += RING) {
#pragma unroll
      for (int u = 0; u < RING; ++u) {
        if (c + u < chunks) {
#pragma unroll
          for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int b = 0; b < MB; ++b) {
              const bf16x8 xf = *reinterpret_cast<const bf16x8*>(xl + b * 16 * row_bytes + (c + u) * 128 + f * 64);
              acc[b] = MM::mma(wf[u][f], xf, acc[b]);
            }
        }
        // slot u next holds chunk c + u + RING of this tile, or the next tile's chunk past this one's end
        const int nc = c + u + RING;
        const int past = nc - ((chunks + RING - 1) / RING) * RING;   // >= 0: the next tile's chunk `past`
        const bf16_t* src = past < 0 ? wp + min(nc, chunks - 1) * 64 : wn + min(past, chunks - 1) * 64;
#pragma unroll
        for (int f = 0; f < 2; ++f) wf[u][f] = *reinterpret_cast<const bf16x8*>(src + f * 32);
      }
    }
    // acc[b][i]: row 16 tile + 4 j + i of W (a logit's index), token 16 b + r
    const int n = tile * 16 + 4 * j;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const int m = 16 * b + r;
      ArgMax mine{LYP_NEG_INF, 0x7fffffff};
      if (m < M) {
        float* crow = C + static_cast<size_t>(m) * ldc + n;
        if (n + 3 < N && ldc % 4 == 0) {
          *reinterpret_cast<f32x4*>(crow) = acc[b];
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) crow[i] = acc[b][i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) mine = better(mine, ArgMax{acc[b][i], n + i});
      }
      if (cand) {
#pragma unroll
        for (int off = 16; off < kWave; off *= 2) mine = better(mine, ArgMax{__shfl_xor(mine.v, off, kWave), __shfl_xor(mine.i, off, kWave)});
        best[b] = better(best[b], mine);
      }
    }
    wp = wn;
  }
  if (cand) {
    if (j == 0)
#pragma unroll
      for (int b = 0; b < MB; ++b) s_best[wave][b][r] = best[b];
    __syncthreads();
    if (tid < M) {
      ArgMax a = s_best[0][tid / 16][tid % 16];
      for (int w = 1; w < kWaves; ++w) a = better(a, s_best[w][tid / 16][tid % 16]);
      cand[static_cast<size_t>(tid) * gridDim.x + blockIdx.x] = a;
    }
  }
}

static bool skinny_ok(int M, int K, int lda, int ldw, const void* A, const void* W, int dtype) {
  const int vec = dtype == kF32 ? 4 : 8;
  return M >= 1 && M <= 64 && K % 64 == 0 && lda % vec == 0 && ldw % vec == 0 &&
         reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0;
}

// Slices of the inner dimension for a product whose result may come as partial
// sums: a matrix with few rows does not give every compute unit a workgroup.
static int skinny_slices(int N, int K) {
  const int row_blocks = (N + 15) / 16;
  int slices = 1;
  while (slices < 8 && row_blocks * slices < 512 && K / (slices * 2) >= 512) slices *= 2;
  return slices;
}

// Waves per workgroup: enough of them over the whole launch to keep every
// compute unit loading, within what LDS holds for the final sum (a kilobyte per
// wave and tile a wave keeps).
constexpr int kMostSumKilobytes = 96;

static int skinny_waves(int N, int K, int tiles, int slices, int rows = 16, int chunk = 64) {
  const int row_blocks = (N + rows - 1) / rows;
  const int chunks = K / chunk / slices;
  // up to 16 rows of tokens as it was measured for them: 32 kilobytes at most
  const int most = tiles <= 2 ? 32 : kMostSumKilobytes;
  int waves = 1;
  while (waves < 16 && waves * 2 * tiles <= most && row_blocks * slices * waves < 4096 && waves * 2 <= chunks) waves *= 2;
  return waves;
}

// Row tiles per workgroup for a step of more than 16 tokens (0: the rule below).  A workgroup
// reads the step's activations over its whole share of K whatever rows of W it owns, so with two
// tiles of 16 rows it asks the cache for half as much per row of W; fewer, larger workgroups in
// exchange.  `g_row_tiles` (lyp_skinny_row_tiles_override) is there for measurements.
static int g_row_tiles = 0;

static int skinny_row_tiles(int M, int N, int slices) {
  if (M <= 16) return 1;
  if (g_row_tiles > 0) return g_row_tiles;
  return (N / 32) * slices >= 128 ? 2 : 1;
}

template <typename T, int EPI, bool NORMED = false, int ROWS = 16, bool PAIRED = false, int RT = 1>
static void launch_skinny(const T* A, const T* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                          int slices, hipStream_t stream, const RopeTail& tail = RopeTail{},
                          const NormHead& head = NormHead{}, const ResidualTail& res = ResidualTail{}) {
  // tiles a wave keeps: paired, 8 rows of W each for 8 tokens each; else 16 rows of W for 16 tokens each
  const int MB = PAIRED ? (ROWS / 8) * ((M + 7) / 8) : (M + 15) / 16;
  const int waves = skinny_waves(N, K, MB * RT, slices, ROWS * RT, PAIRED ? 128 : 64);
  const dim3 grid((N + ROWS * RT - 1) / (ROWS * RT), slices), block(waves * kWave);
  const size_t lds = (static_cast<size_t>(waves) * MB * RT * 256 + waves * 16 + (EPI == kEpiResidual ? MB * 256 : 0)) *
                     sizeof(float);
#define LYP_SKINNY_TB(MBV, TBV)                                                                                        \
  do {                                                                                                                 \
    auto kernel = gemm_skinny_kernel<T, MBV, EPI, NORMED, ROWS, PAIRED, TBV, RT>;                                      \
    if (lds > 48 * 1024) {   /* more than a kernel gets without asking: said once per kernel */                       \
      static bool asked = false;                                                                                       \
      if (!asked) {                                                                                                    \
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                  (kMostSumKilobytes + 8) * 1024);                                                     \
        asked = true;                                                                                                  \
      }                                                                                                                \
    }                                                                                                                  \
    kernel<<<grid, block, lds, stream>>>(A, W, C, M, N, K, lda, ldw, ldc, tail, head, res);                            \
  } while (0)
#define LYP_SKINNY(MBV) LYP_SKINNY_TB(MBV, 1)
  if constexpr (PAIRED && ROWS == 16) {
    LYP_SKINNY(2);  // at most 8 rows: the caller has checked
  } else if constexpr (PAIRED) {
    if (M <= 8) LYP_SKINNY(1);
    else LYP_SKINNY_TB(1, 2);  // at most 16 rows: the caller has checked
  } else if constexpr (NORMED) {
    LYP_SKINNY(1);  // at most 16 rows: the callers have checked
  } else if constexpr (RT > 1) {
    if (MB == 2) LYP_SKINNY(2);  // more than 16 rows: the caller has checked
    else if (MB == 3) LYP_SKINNY(3);
    else LYP_SKINNY(4);
  } else {
    if (MB == 1) LYP_SKINNY(1);
    else if (MB == 2) LYP_SKINNY(2);
    else if (MB == 3) LYP_SKINNY(3);
    else LYP_SKINNY(4);
  }
#undef LYP_SKINNY
#undef LYP_SKINNY_TB
}

// The plain tile with one or two row tiles per workgroup, as skinny_row_tiles says.
template <typename T, int EPI>
static void launch_skinny_rows(const T* A, const T* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                               int slices, hipStream_t stream, const RopeTail& tail = RopeTail{}) {
  if (skinny_row_tiles(M, N, slices) >= 2)
    launch_skinny<T, EPI, false, 16, false, 2>(A, W, C, M, N, K, lda, ldw, ldc, slices, stream, tail);
  else
    launch_skinny<T, EPI>(A, W, C, M, N, K, lda, ldw, ldc, slices, stream, tail);
}

static int g_wide_gemm = 1;   // many bfloat16 rows: 1 the wide kernel, tile by rule; for tests and measurements 0 the general kernel, 2 / 3 tiles of 128 / 256 features
template <int TM, int TN, int MODE>
static void launch_wide(const bf16_t* A, const bf16_t* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                        hipStream_t stream) {
  const int m_tiles = (M + TM - 1) / TM, n_tiles = (N + TN - 1) / TN;
  const int grid = 8 * ((n_tiles + 7) / 8) * m_tiles;   // every die's share rounded up to that of the first
  gemm_bf16_wide_kernel<TM, TN, MODE><<<grid, 512, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc, m_tiles, n_tiles);
}

template <typename T, int MODE>
static void launch_gemm(const T* A, const T* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                        int vec_ok, hipStream_t stream) {
  if constexpr (std::is_same_v<T, bf16_t>) {
    if (M > 128 && vec_ok && K % 64 == 0 && g_wide_gemm) {
      // tiles of 256 features while there is one for every compute unit, of 128 otherwise
      const long long tiles = static_cast<long long>((M + 255) / 256) * ((N + 255) / 256);
      if (g_wide_gemm == 2 || (g_wide_gemm == 1 && tiles < compute_units()))
        launch_wide<256, 128, MODE>(A, W, C, M, N, K, lda, ldw, ldc, stream);
      else
        launch_wide<256, 256, MODE>(A, W, C, M, N, K, lda, ldw, ldc, stream);
      return;
    }
  }
  if (M <= 32) {
    dim3 grid((N + 127) / 128, (M + 31) / 32);
    gemm_nt_kernel<T, 32, 128, 1, 4, MODE><<<grid, 256, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc, vec_ok);
  } else if (M <= 64) {
    dim3 grid((N + 127) / 128, (M + 63) / 64);
    gemm_nt_kernel<T, 64, 128, 2, 2, MODE><<<grid, 256, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc, vec_ok);
  } else {
    dim3 grid((N + 127) / 128, (M + 127) / 128);
    gemm_nt_kernel<T, 128, 128, 2, 2, MODE><<<grid, 256, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc, vec_ok);
  }
}

}  // namespace lyp

using namespace lyp;

extern "C" int lyp_gemm_wide(int which) {
  LYP_REQUIRE(which >= 0 && which <= 3, "wide product: 0 to 3, not %d", which);
  g_wide_gemm = which;
  return 0;
}

extern "C" int lyp_gemm_nt(const void* A, const void* W, void* C, int dtype, int mode, int M, int N, int K,
                           int lda, int ldw, int ldc, hipStream_t stream) {
  LYP_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  LYP_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: leading dimensions %d %d %d too small", lda, ldw, ldc);
  LYP_REQUIRE(mode >= 0 && mode <= 2, "gemm: unknown output mode %d", mode);
  LYP_REQUIRE((M + 127) / 128 <= 65535, "gemm: M=%d too large for one launch", M);
  if (M == 0) return 0;
  const int vec = dtype == kF32 ? 4 : 8;
  const size_t esz = dtype == kF32 ? 4 : 2;
  const int vec_ok = (lda % vec == 0) && (ldw % vec == 0) &&
                     (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(W) % 16 == 0);
  (void)esz;
#define LYP_GEMM(T, MODE)                                                                             \
  launch_gemm<T, MODE>(static_cast<const T*>(A), static_cast<const T*>(W), C, M, N, K, lda, ldw, ldc, \
                       vec_ok, stream)
  if (mode != kAccumF32 && skinny_ok(M, K, lda, ldw, A, W, dtype)) {
    if (dtype == kF32)
      launch_skinny_rows<float, kEpiF32>(static_cast<const float*>(A), static_cast<const float*>(W), C, M, N, K, lda, ldw, ldc, 1, stream);
    else if (dtype == kBF16 && mode == kStoreF32)
      launch_skinny_rows<bf16_t, kEpiF32>(static_cast<const bf16_t*>(A), static_cast<const bf16_t*>(W), C, M, N, K, lda, ldw, ldc, 1, stream);
    else if (dtype == kBF16)
      launch_skinny_rows<bf16_t, kEpiAct>(static_cast<const bf16_t*>(A), static_cast<const bf16_t*>(W), C, M, N, K, lda, ldw, ldc, 1, stream);
    else
      LYP_REQUIRE(false, "gemm: unknown dtype %d", dtype);
    LYP_LAUNCH_CHECK("gemm_skinny");
    return 0;
  }
  if (dtype == kF32) {
    if (mode == kStoreAct || mode == kStoreF32) LYP_GEMM(float, kStoreF32);
    else LYP_GEMM(float, kAccumF32);
  } else if (dtype == kBF16) {
    if (mode == kStoreAct) LYP_GEMM(bf16_t, kStoreAct);
    else if (mode == kStoreF32) LYP_GEMM(bf16_t, kStoreF32);
    else LYP_GEMM(bf16_t, kAccumF32);
  } else {
    LYP_REQUIRE(false, "gemm: unknown dtype %d", dtype);
  }
#undef LYP_GEMM
  LYP_LAUNCH_CHECK("gemm_nt");
  return 0;
}

constexpr size_t kHeadStageBytes = 144 * 1024;   // of the 160 KB of LDS; the rest is the kernel's own
constexpr int kHeadRing = 8;   // chunks a wave of lm_head_stream_kernel asks for ahead (16: 2-3 us slower)

// Float logits C[M, N] = A . W^T for up to 64 rows (see lm_head_kernel), with `blocks` workgroups
// (0: two per compute unit of this machine's 256, as a plain read of such a matrix likes it).
// cand (optional): [M][blocks] pairs of (float, int32) that receive every workgroup's largest logit
// per row and its index.  Returns the number of workgroups used (the stride of cand), 0 when the
// kernel does not take the operands (then use lyp_gemm_nt), negative on error.
extern "C" int lyp_lm_head(const void* A, const void* W, float* C, int dtype, int M, int N, int K, int lda, int ldw,
                           int ldc, void* cand, int blocks, hipStream_t stream) {
  LYP_REQUIRE(N > 0 && K > 0 && ldc >= N && blocks >= 0 && blocks <= 4096, "lm_head: N=%d K=%d stride %d blocks %d", N, K,
              ldc, blocks);
  if (!skinny_ok(M, K, lda, ldw, A, W, dtype)) return 0;
  if (blocks == 0) blocks = 512;
  blocks = std::min(blocks, (N + 63) / 64);  // no workgroup without a wave's worth of rows
  ArgMax* cd = static_cast<ArgMax*>(cand);
  // bfloat16 tokens whose activations fit LDS (16 of up to 4,600 values, 32 of up to 2,296): the steady stream, one
  // workgroup per compute unit
  const int token_blocks = (M + 15) / 16;
  const size_t staged = static_cast<size_t>(16) * token_blocks * (2 * K + 16);
  if (dtype == kBF16 && token_blocks <= 2 && staged <= kHeadStageBytes) {
    blocks = std::min(blocks, compute_units());
    auto kernel = token_blocks == 1 ? lm_head_stream_kernel<kHeadRing, 1> : lm_head_stream_kernel<kHeadRing, 2>;
    static bool asked[2] = {false, false};
    if (!asked[token_blocks - 1]) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(kHeadStageBytes));
      asked[token_blocks - 1] = true;
    }
    kernel<<<blocks, 256, staged, stream>>>(static_cast<const bf16_t*>(A), static_cast<const bf16_t*>(W), C, M, N, K, lda,
                                            ldw, ldc, cd);
    LYP_LAUNCH_CHECK("lm_head_stream");
    return blocks;
  }
  if (M > 16) return 0;   // beyond that the general products are ahead of lm_head_kernel
#define LYP_HEAD(T, MB) \
  lm_head_kernel<T, MB><<<blocks, 256, 0, stream>>>(static_cast<const T*>(A), static_cast<const T*>(W), C, M, N, K, lda, ldw, ldc, cd)
#define LYP_HEAD_T(T)                  \
  do {                                 \
    if (M <= 16) LYP_HEAD(T, 1);       \
    else if (M <= 32) LYP_HEAD(T, 2);  \
    else if (M <= 48) LYP_HEAD(T, 3);  \
    else LYP_HEAD(T, 4);               \
  } while (0)
  if (dtype == kF32) LYP_HEAD_T(float);
  else if (dtype == kBF16) LYP_HEAD_T(bf16_t);
  else LYP_REQUIRE(false, "lm_head: unknown dtype %d", dtype);
#undef LYP_HEAD_T
#undef LYP_HEAD
  LYP_LAUNCH_CHECK("lm_head");
  return blocks;
}

// Row tiles per workgroup of the few-rows kernel in steps of more than 16 tokens (0: the built-in rule); for measurements.
extern "C" int lyp_skinny_row_tiles_override(int row_tiles) {
  LYP_REQUIRE(row_tiles >= 0 && row_tiles <= 2, "row tiles per workgroup: 0 (the rule), 1 or 2, not %d", row_tiles);
  g_row_tiles = row_tiles;
  return 0;
}

// Workgroups the few-rows kernel would launch for this product (with_slices: as partial sums over
// slices of K, where lyp_gemm_parts_hint cuts it), 0 if the kernel does not take the shape.  The kernel
// is one burst of loads per workgroup, so it is at its best while the launch is a single round of
// workgroups on the machine: what the caller holds this number against.
extern "C" int lyp_skinny_workgroups(int M, int N, int K, int with_slices) {
  if (M < 1 || M > 64 || K % 64 != 0) return 0;
  const int slices = with_slices ? skinny_slices(N, K) : 1;
  const int rows = 16 * skinny_row_tiles(M, N, slices);
  return ((N + rows - 1) / rows) * slices;
}


// Slices of K that lyp_gemm_nt_parts would cut this matrix into (1: none).
extern "C" int lyp_skinny_slices(int N, int K) { return K % 64 == 0 ? skinny_slices(N, K) : 1; }

// How many partial sums lyp_gemm_nt_parts would produce for this product; 0 if
// it does not apply (then use lyp_gemm_nt).
extern "C" int lyp_gemm_parts_hint(const void* A, const void* W, int dtype, int M, int N, int K, int lda, int ldw) {
  if (!skinny_ok(M, K, lda, ldw, A, W, dtype)) return 0;
  const int slices = skinny_slices(N, K);
  return slices > 1 ? slices : 0;
}

// parts[slice][M][N] (float) = partial sums of A . W^T over slices of the inner
// dimension; their sum, in order, is the product.  `slices` must be what
// lyp_gemm_parts_hint said.
extern "C" int lyp_gemm_nt_parts(const void* A, const void* W, float* parts, int dtype, int slices, int M, int N,
                                 int K, int lda, int ldw, hipStream_t stream) {
  LYP_REQUIRE(skinny_ok(M, K, lda, ldw, A, W, dtype) && slices == skinny_slices(N, K) && slices > 1,
              "gemm_parts: M=%d N=%d K=%d slices=%d is not a case for partial sums", M, N, K, slices);
  if (dtype == kF32)
    launch_skinny_rows<float, kEpiParts>(static_cast<const float*>(A), static_cast<const float*>(W), parts, M, N, K, lda, ldw, N, slices, stream);
  else if (dtype == kBF16)
    launch_skinny_rows<bf16_t, kEpiParts>(static_cast<const bf16_t*>(A), static_cast<const bf16_t*>(W), parts, M, N, K, lda, ldw, N, slices, stream);
  else
    LYP_REQUIRE(false, "gemm_parts: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("gemm_parts");
  return 0;
}

// out[M, N/2] = silu(gate) * up where W's rows come in tiles of 16: eight gate
// features, then the eight up features that go with them.  Returns 1 (and does
// nothing) when the few-rows kernel does not apply: then run lyp_gemm_nt and
// lyp_swiglu with the same interleave.
extern "C" int lyp_gemm_swiglu(const void* A, const void* W, void* out, int dtype, int M, int N, int K, int lda,
                               int ldw, int ldo, hipStream_t stream) {
  LYP_REQUIRE(N % 16 == 0 && ldo >= N / 2, "gemm_swiglu: %d rows of weights, output stride %d", N, ldo);
  if (!skinny_ok(M, K, lda, ldw, A, W, dtype)) return 1;
  if (dtype == kF32)
    launch_skinny_rows<float, kEpiSwiglu>(static_cast<const float*>(A), static_cast<const float*>(W), out, M, N, K, lda, ldw, ldo, 1, stream);
  else if (dtype == kBF16)
    launch_skinny_rows<bf16_t, kEpiSwiglu>(static_cast<const bf16_t*>(A), static_cast<const bf16_t*>(W), out, M, N, K, lda, ldw, ldo, 1, stream);
  else
    LYP_REQUIRE(false, "gemm_swiglu: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("gemm_swiglu");
  return 0;
}

// The fused q/k/v projection of a step with few rows, finished in one kernel:
// out[M, nh * hd] receives the query heads, rotated; the key heads, rotated,
// and the value heads go to the pages that `slots` names (see RopeTail; what
// lyp_gemm_nt followed by lyp_rope_kv_write does, to the last bit).  W has
// (nh + 2 nkv) * hd rows, or nh * hd without has_kv.  Returns 1 (and does
// nothing) when the few-rows kernel does not apply or the rotated part of a
// head is no multiple of 16.
extern "C" int lyp_gemm_rope_kv(const void* A, const void* W, void* out, int dtype, int M, int K, int lda, int ldw,
                                int ldo, const int32_t* positions, const float* cos_sin, const int32_t* slots,
                                void* kpool, void* vpool, int nh, int nkv, int hd, int rot, int bs, int has_kv,
                                hipStream_t stream) {
  LYP_REQUIRE(nh > 0 && nkv >= 0 && hd > 0 && hd % 16 == 0, "gemm_rope_kv: %d heads, %d key/value heads of %d", nh,
              nkv, hd);
  LYP_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "gemm_rope_kv: rotary size %d of head size %d", rot, hd);
  LYP_REQUIRE(positions && (rot == 0 || cos_sin), "gemm_rope_kv: positions and the rotation table are needed");
  LYP_REQUIRE(!has_kv || (slots && kpool && vpool && bs > 0 && nkv > 0), "gemm_rope_kv: no pages to store to");
  const int N = (has_kv ? nh + 2 * nkv : nh) * hd;
  LYP_REQUIRE(ldo >= nh * hd, "gemm_rope_kv: output stride %d", ldo);
  if (rot % 16 != 0 || !skinny_ok(M, K, lda, ldw, A, W, dtype)) return 1;
  const RopeTail tail{positions, cos_sin, slots, kpool, vpool, nh, nkv, hd, rot, bs, has_kv};
  if (dtype == kF32)
    launch_skinny_rows<float, kEpiRope>(static_cast<const float*>(A), static_cast<const float*>(W), out, M, N, K, lda, ldw, ldo, 1, stream, tail);
  else if (dtype == kBF16)
    launch_skinny_rows<bf16_t, kEpiRope>(static_cast<const bf16_t*>(A), static_cast<const bf16_t*>(W), out, M, N, K, lda, ldw, ldo, 1, stream, tail);
  else
    LYP_REQUIRE(false, "gemm_rope_kv: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("gemm_rope_kv");
  return 0;
}

// h[M, N] += A . W^T on the float residual stream, for a step with few rows.
// With next_w (the weights of the RMS norm that follows) it also
// stores xs[M, N] = h * next_w in the operands' type and, per workgroup, every
// row's sum of squares over the workgroup's features: ssq_part[parts][16], with
// `parts` = lyp_gemm_residual_parts(M, N, K) workgroups.  A product normed that way
// (lyp_gemm_swiglu_normed, lyp_gemm_rope_kv_normed) takes xs and ssq_part in
// place of the normed activations.  Returns 1 (and does nothing) when the
// few-rows kernel does not apply.
// Weight rows per workgroup: 8, so that a matrix of 2,048 rows gives every compute unit a
// workgroup; 16 (as two paired tiles, the activations loaded once for both) from 3,072 rows on,
// where that was measured ahead.
static int residual_rows(int M, int N, int K) { return M <= 8 && K % 128 == 0 && N >= 3072 ? 16 : 8; }

extern "C" int lyp_gemm_residual_parts(int M, int N, int K) {
  const int rows = residual_rows(M, N, K);
  return (N + rows - 1) / rows;
}

extern "C" int lyp_gemm_residual(const void* A, const void* W, float* h, int dtype, int M, int N, int K, int lda,
                                 int ldw, int ldh, const void* next_w, int next_w_dtype, void* xs, int ldx,
                                 float* ssq_part, hipStream_t stream) {
  LYP_REQUIRE(N > 0 && K > 0 && ldh >= N, "gemm_residual: N=%d K=%d stride %d", N, K, ldh);
  LYP_REQUIRE(!next_w || (xs && ssq_part && ldx >= N && M <= 16), "gemm_residual: by-products for %d rows", M);
  if (!skinny_ok(M, K, lda, ldw, A, W, dtype)) return 1;
  const ResidualTail res{next_w, next_w_dtype == kF32, xs, ldx, ssq_part};
  const bool paired = M <= 16 && K % 128 == 0;  // two chunks of K per matrix instruction
  const bool wide = residual_rows(M, N, K) == 16;
#define LYP_RESIDUAL(T, ROWS, PAIRED)                                                                           \
  launch_skinny<T, kEpiResidual, false, ROWS, PAIRED>(static_cast<const T*>(A), static_cast<const T*>(W), h, M, N, \
                                                      K, lda, ldw, ldh, 1, stream, RopeTail{}, NormHead{}, res)
  if (dtype == kF32) {
    if (wide) LYP_RESIDUAL(float, 16, true);
    else if (paired) LYP_RESIDUAL(float, 8, true);
    else LYP_RESIDUAL(float, 8, false);
  } else if (dtype == kBF16) {
    if (wide) LYP_RESIDUAL(bf16_t, 16, true);
    else if (paired) LYP_RESIDUAL(bf16_t, 8, true);
    else LYP_RESIDUAL(bf16_t, 8, false);
  } else
    LYP_REQUIRE(false, "gemm_residual: unknown dtype %d", dtype);
#undef LYP_RESIDUAL
  LYP_LAUNCH_CHECK("gemm_residual");
  return 0;
}

// lyp_gemm_swiglu on activations xs that still lack their rows' 1 / rms (see
// lyp_gemm_residual): silu(g) * u of (xs / rms) . W^T, `width` being the number
// of features the sums of squares run over.
extern "C" int lyp_gemm_swiglu_normed(const void* xs, int ldx, const float* ssq_part, int n_parts, int width,
                                      float eps, const void* W, void* out, int dtype, int M, int N, int K, int ldw,
                                      int ldo, hipStream_t stream) {
  LYP_REQUIRE(N % 16 == 0 && ldo >= N / 2, "gemm_swiglu: %d rows of weights, output stride %d", N, ldo);
  LYP_REQUIRE(ssq_part && n_parts > 0 && width > 0, "gemm_swiglu: no sums of squares");
  if (M > 16 || !skinny_ok(M, K, ldx, ldw, xs, W, dtype)) return 1;
  const NormHead head{ssq_part, n_parts, width, eps};
  if (dtype == kF32)
    launch_skinny<float, kEpiSwiglu, true>(static_cast<const float*>(xs), static_cast<const float*>(W), out, M, N, K, ldx, ldw, ldo, 1, stream, RopeTail{}, head);
  else if (dtype == kBF16)
    launch_skinny<bf16_t, kEpiSwiglu, true>(static_cast<const bf16_t*>(xs), static_cast<const bf16_t*>(W), out, M, N, K, ldx, ldw, ldo, 1, stream, RopeTail{}, head);
  else
    LYP_REQUIRE(false, "gemm_swiglu: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("gemm_swiglu_normed");
  return 0;
}

// lyp_gemm_rope_kv on such activations.
extern "C" int lyp_gemm_rope_kv_normed(const void* xs, int ldx, const float* ssq_part, int n_parts, int width,
                                       float eps, const void* W, void* out, int dtype, int M, int K, int ldw,
                                       int ldo, const int32_t* positions, const float* cos_sin,
                                       const int32_t* slots, void* kpool, void* vpool, int nh, int nkv, int hd,
                                       int rot, int bs, int has_kv, hipStream_t stream) {
  LYP_REQUIRE(nh > 0 && nkv >= 0 && hd > 0 && hd % 16 == 0, "gemm_rope_kv: %d heads, %d key/value heads of %d", nh,
              nkv, hd);
  LYP_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "gemm_rope_kv: rotary size %d of head size %d", rot, hd);
  LYP_REQUIRE(positions && (rot == 0 || cos_sin), "gemm_rope_kv: positions and the rotation table are needed");
  LYP_REQUIRE(!has_kv || (slots && kpool && vpool && bs > 0 && nkv > 0), "gemm_rope_kv: no pages to store to");
  LYP_REQUIRE(ssq_part && n_parts > 0 && width > 0, "gemm_rope_kv: no sums of squares");
  const int N = (has_kv ? nh + 2 * nkv : nh) * hd;
  LYP_REQUIRE(ldo >= nh * hd, "gemm_rope_kv: output stride %d", ldo);
  if (M > 16 || rot % 16 != 0 || !skinny_ok(M, K, ldx, ldw, xs, W, dtype)) return 1;
  const RopeTail tail{positions, cos_sin, slots, kpool, vpool, nh, nkv, hd, rot, bs, has_kv};
  const NormHead head{ssq_part, n_parts, width, eps};
  if (dtype == kF32)
    launch_skinny<float, kEpiRope, true>(static_cast<const float*>(xs), static_cast<const float*>(W), out, M, N, K, ldx, ldw, ldo, 1, stream, tail, head);
  else if (dtype == kBF16)
    launch_skinny<bf16_t, kEpiRope, true>(static_cast<const bf16_t*>(xs), static_cast<const bf16_t*>(W), out, M, N, K, ldx, ldw, ldo, 1, stream, tail, head);
  else
    LYP_REQUIRE(false, "gemm_rope_kv: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("gemm_rope_kv_normed");
  return 0;
}
