// Attention over the paged cache, on the matrix cores, compiled for one head
// size (LYP_HEAD_DIM, a multiple of 16) and both element types.
//
// The kernels share the fragment loaders and the online softmax:
//   * attn_prefill: a workgroup takes a run of new tokens of one request and up
//     to four query heads of one key/value head; the keys and values they may
//     see pass through LDS, shared by its waves (a wave: one head, 16 or 32
//     tokens).  attn_prefill_wide is the same work for bfloat16 on the
//     16x16x32 instruction, with eight waves and loads two tiles ahead.
//   * attn_decode:  a wave takes one request's single new token, all query
//     heads of one key/value head (as the 16 columns of the tile), and a
//     multiple of 64 keys of the context; a workgroup merges its waves,
//     attn_combine the workgroups.
// Both read keys and values from pages through the request's block table, and
// both run after the step's new keys and values have been written, so a
// prompt portion needs no second source of keys.
//
// What is computed follows the reference: scale 1/sqrt(hd), grouped heads
// (query head h reads key/value head h / g), causal mask, online softmax with
// a running maximum and sum, 0 when nothing is visible
// (csrc/kernels/flash_attn_v2.cu:30-31, 87, 114-166, 197;
//  csrc/kernels/paged_attention.cu:25-30, 69-105;
//  csrc/kernels/flash_decoding.cu:12-147).  Unlike the reference the mask uses
// absolute positions, so a portion that starts in the middle of a prompt sees
// the keys before it, and the page size is a run-time value.
//
// Page layouts (one page of one key/value head):
//   keys   [bs][hd]   a key's head is contiguous
//   values [hd][bs]   the keys of a page are contiguous per dimension, which is
//                     the operand layout of the P.V product
//
// Every 16-key block starts at a multiple of 16 in absolute positions and the
// decode partitions at multiples of 64 (waves) and of 64 times the waves of a
// workgroup, so the order of the additions for a
// token depends on its position and its window alone, never on how the tokens
// were cut into steps or on what else is in the batch.
#include "common.h"

#ifndef LYP_HEAD_DIM
#error "compile with -DLYP_HEAD_DIM=<multiple of 16>"
#endif
#ifndef LYP_PREFILL_QB   // 16-token blocks per wave when a workgroup takes four heads
#if LYP_HEAD_DIM <= 64
#define LYP_PREFILL_QB 2
#else
#define LYP_PREFILL_QB 1
#endif
#endif

namespace lyp {

constexpr int HD = LYP_HEAD_DIM;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16, at most 256");
constexpr int kSteps = HD / 16;     // matrix steps over the head dimension; also 16-row blocks of it
constexpr int kSlice = HD / 4;      // contiguous run of the head dimension one lane group loads
constexpr int kPartKeys = 64;       // a wave's share of a decode partition is a multiple of this
constexpr float kLog2e = 1.4426950408889634f;

template <typename T>
using Frag = typename Mma16<T>::Frag;

template <typename T>
__device__ __forceinline__ Frag<T> zero_frag() {
  Frag<T> f;
#pragma unroll
  for (int i = 0; i < 4; ++i) f[i] = from_f32<T>(0.f);
  return f;
}

struct PagedKV {
  const void* kpool;
  const void* vpool;
  const int32_t* table;  // this request's row of the block table
  int nkv, bs, kvh;
  int max_blocks;        // width of the row: an index below it may always be read
};

// The table entry for a key, read whether or not the key is inside the
// request: the index is clamped to the row, the result is used only for keys
// that exist.  Lets the read start before the request's length is known.
__device__ __forceinline__ int page_of(const PagedKV& kv, int key) {
  return kv.table[min(key / kv.bs, kv.max_blocks - 1)];
}

// Keys kb0 .. kb0+15 as the row operand of S^T = K . Q^T.  Lane (r, j) holds
// key kb0 + r, dimensions j * kSlice + 4 * step + {0..3}.
template <typename T>
__device__ __forceinline__ void load_k_page(Frag<T> (&kf)[kSteps], const PagedKV& kv, int kb0, int lo, int hi,
                                            int lane, int page) {
  const int key = kb0 + lane % 16;
  if (key >= lo && key < hi) {
    if (page >= 0) {
      const T* row = static_cast<const T*>(kv.kpool) +
                     ((static_cast<size_t>(page) * kv.nkv + kv.kvh) * kv.bs + key % kv.bs) * HD +
                     (lane / 16) * kSlice;
#pragma unroll
      for (int s = 0; s < kSteps; ++s) kf[s] = *reinterpret_cast<const Frag<T>*>(row + 4 * s);
      return;
    }
  }
#pragma unroll
  for (int s = 0; s < kSteps; ++s) kf[s] = zero_frag<T>();
}

template <typename T>
__device__ __forceinline__ void load_k(Frag<T> (&kf)[kSteps], const PagedKV& kv, int kb0, int lo, int hi,
                                       int lane) {
  load_k_page<T>(kf, kv, kb0, lo, hi, lane, page_of(kv, kb0 + lane % 16));
}

// Values of the same 16 keys as the row operand of O^T = V^T . P^T.  Lane
// (r, j) holds, per 16-row block db of the head dimension, dimension
// db * 16 + r and keys kb0 + 4 j + {0..3}.  Anything outside [lo, hi) reads as
// zero: a page that was never written may hold any bit pattern.
// `page0` is the table entry of the lane's first key (used when a page holds a
// multiple of four keys, so that the lane's four keys share it).
template <typename T>
__device__ __forceinline__ void load_v_page(Frag<T> (&vf)[kSteps], const PagedKV& kv, int kb0, int lo, int hi,
                                            int lane, int page0) {
  const int key0 = kb0 + 4 * (lane / 16);
  const int r = lane % 16;
  const T* vpool = static_cast<const T*>(kv.vpool);
#pragma unroll
  for (int db = 0; db < kSteps; ++db) vf[db] = zero_frag<T>();
  if (kv.bs % 4 == 0) {
    if (key0 < hi && key0 + 3 >= lo) {
      const int page = page0;
      if (page >= 0) {
        const T* base = vpool + (static_cast<size_t>(page) * kv.nkv + kv.kvh) * HD * kv.bs + key0 % kv.bs;
#pragma unroll
        for (int db = 0; db < kSteps; ++db) {
          Frag<T> f = *reinterpret_cast<const Frag<T>*>(base + static_cast<size_t>(db * 16 + r) * kv.bs);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (key0 + i < lo || key0 + i >= hi) f[i] = from_f32<T>(0.f);
          vf[db] = f;
        }
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = key0 + i;
      if (key < lo || key >= hi) continue;
      const int page = kv.table[key / kv.bs];
      if (page < 0) continue;
      const T* base = vpool + (static_cast<size_t>(page) * kv.nkv + kv.kvh) * HD * kv.bs + key % kv.bs;
#pragma unroll
      for (int db = 0; db < kSteps; ++db) vf[db][i] = base[static_cast<size_t>(db * 16 + r) * kv.bs];
    }
  }
}

template <typename T>
__device__ __forceinline__ void load_v(Frag<T> (&vf)[kSteps], const PagedKV& kv, int kb0, int lo, int hi,
                                       int lane) {
  load_v_page<T>(vf, kv, kb0, lo, hi, lane, page_of(kv, kb0 + 4 * (lane / 16)));
}

// A query row as the column operand, in the same order of dimensions as load_k.
template <typename T>
__device__ __forceinline__ void load_q(Frag<T> (&qf)[kSteps], const T* row, bool valid, int lane) {
  if (valid) {
    const T* p = row + (lane / 16) * kSlice;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) qf[s] = *reinterpret_cast<const Frag<T>*>(p + 4 * s);
  } else {
#pragma unroll
    for (int s = 0; s < kSteps; ++s) qf[s] = zero_frag<T>();
  }
}

// Running softmax of one 16-column block (lane l owns column l % 16).
struct Softmax {
  float m;     // running maximum, in the base-2 domain; the same in the four lane groups
  float lsum;  // this lane group's part of the running sum
};

// 2^x by the hardware instruction alone: arguments here are at most 0 and
// results below the normal range may be flushed.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// The maximum over the four lanes l, l ^ 16, l ^ 32, l ^ 48, in every one of them, with the two
// row-swap instructions of this chip (no trip through LDS).  v_permlane16_swap exchanges the odd
// 16-lane rows of its first operand with the even rows of its second, v_permlane32_swap the upper
// half of the first with the lower half of the second; fed with two copies of a value, the two
// results hold it and its neighbour's.
__device__ __forceinline__ float lane_groups_max(float m) {
  float a = m, b = m;
  asm volatile(
      "s_nop 1\n\t"
      "v_permlane16_swap_b32 %0, %1\n\t"
      "s_nop 1\n\t"
      "v_max_f32 %0, %0, %1\n\t"
      "v_mov_b32 %1, %0\n\t"
      "s_nop 1\n\t"
      "v_permlane32_swap_b32 %0, %1\n\t"
      "s_nop 1\n\t"
      "v_max_f32 %0, %0, %1"
      : "+v"(a), "+v"(b));
  return a;
}

// Take the scores of NB consecutive 16-key blocks (s[u]: rows = keys
// kb0 + 16 u + 4 (l / 16) + i, column = l % 16), update the running state,
// rescale the output accumulator and return the probabilities as the column
// operands of the P.V products: one maximum, one rescaling and one pass of
// exponentials for all of them, which is most of the arithmetic outside the
// matrix cores.  `pos` is the column's absolute position; a key is visible when
// key <= pos, key < hi and (window == 0 or key > pos - window).  With MASKED
// false every key is visible to every column and the tests are skipped.
template <typename T, bool MASKED, int NB>
__device__ __forceinline__ void softmax_group(const f32x4 (&s)[NB], Frag<T> (&pf)[NB], float scale_log2, int kb0,
                                              int pos, int window, int hi, Softmax& st, f32x4 (&o)[kSteps],
                                              int lane) {
  float sv[NB][4];
  float mx = LYP_NEG_INF;
#pragma unroll
  for (int u = 0; u < NB; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (MASKED) {
        const int key = kb0 + 16 * u + 4 * (lane / 16) + i;
        const bool vis = key <= pos && key < hi && (window == 0 || key > pos - window);
        sv[u][i] = vis ? s[u][i] * scale_log2 : LYP_NEG_INF;
      } else {
        sv[u][i] = s[u][i] * scale_log2;
      }
      mx = fmaxf(mx, sv[u][i]);
    }
  mx = lane_groups_max(mx);
  const float m_new = fmaxf(st.m, mx);
  const float m_safe = m_new == LYP_NEG_INF ? 0.f : m_new;
  const float alpha = fast_exp2(st.m - m_safe);
  float psum = 0.f;
#pragma unroll
  for (int u = 0; u < NB; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p = fast_exp2(sv[u][i] - m_safe);
      psum += p;
      pf[u][i] = from_f32<T>(p);
    }
  st.lsum = st.lsum * alpha + psum;
  st.m = m_new;
#pragma unroll
  for (int db = 0; db < kSteps; ++db)
#pragma unroll
    for (int i = 0; i < 4; ++i) o[db][i] *= alpha;
}

__device__ __forceinline__ float lane_groups_sum(float v) {
  v += __shfl_xor(v, 16, kWave);
  v += __shfl_xor(v, 32, kWave);
  return v;
}

// --------------------------------------------------------------------- prefill
// grid (tiles * sub-tiles, nkv * head_groups); 256 threads (four waves).  A
// workgroup takes QW consecutive new tokens of one request and GH query heads of
// one key/value head; wave w takes head w % GH and token sub-block w / GH (QB
// blocks of 16 tokens).  The keys and values the tokens may see are brought
// into LDS tile by tile (the next tile travels while the current one is used)
// and shared by the four waves, so that a key is read from memory once for all
// the heads of its group.
template <typename T>
struct PrefillTile {
  static constexpr int kKeys = HD * sizeof(T) <= 128 ? 64 : (HD * sizeof(T) <= 256 ? 32 : 16);
  static constexpr int kVec = 16 / sizeof(T);          // elements per 16-byte access
  static constexpr int kKLd = HD + 4;                  // padded row of the key tile [keys][hd]
  static constexpr int kVLd = kKeys + 4;               // padded row of the value tile [hd][keys]
  static constexpr int kElems = kKeys * kKLd + HD * kVLd;
  static constexpr int kBufs = 2 * kElems * sizeof(T) <= 60 * 1024 ? 2 : 1;
  static constexpr int kKVecs = kKeys * HD / kVec;     // 16-byte pieces of a key tile
  static constexpr int kPerThread = (kKVecs + 255) / 256;
};

template <typename T, int GH, int QB>
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride, const void* kpool,
    const void* vpool, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_q0, int n_tiles, int nh, int nkv,
    int bs, int window, float scale_log2) {
  using PT = PrefillTile<T>;
  constexpr int KT = PT::kKeys, NB = KT / 16, VEC = PT::kVec;
  constexpr int QW = (4 / GH) * QB * 16;  // new tokens per workgroup
  constexpr int kSubs = 64 / QW;          // workgroups per 64-token tile of the host's list
  static_assert(QW <= 64 && 64 % QW == 0, "a workgroup takes a whole fraction of a 64-token tile");
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  __shared__ __attribute__((aligned(16))) T lds[PT::kBufs * PT::kElems];

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int g = nh / nkv;
  const int head_groups = (g + GH - 1) / GH;
  const int kvh = blockIdx.y / head_groups;
  const int hsub = (blockIdx.y % head_groups) * GH;

  // The host lists tiles in rising order of position; the longest are started first.
  const int tile = n_tiles - 1 - static_cast<int>(blockIdx.x) / kSubs;
  const int seq = tile_seq[tile];
  const int tok0 = q_start[seq];
  const int q_len = q_start[seq + 1] - tok0;
  const int ctx = ctx_len[seq];
  const int q0_wg = tile_q0[tile] + (static_cast<int>(blockIdx.x) % kSubs) * QW;
  if (q0_wg >= q_len) return;  // the whole workgroup
  const int pos_first = ctx - q_len + q0_wg;
  const int pos_last_wg = pos_first + min(QW, q_len - q0_wg) - 1;
  const int lo_wg = window > 0 ? max(0, pos_first - window + 1) : 0;
  const int hi_wg = pos_last_wg + 1;

  // this wave's head and tokens
  const int hw = hsub + wave % GH;
  const int q0_w = q0_wg + (wave / GH) * QB * 16;
  const bool wave_active = hw < g && q0_w < q_len;
  const int col = lane % 16;
  const int head = kvh * g + (hw < g ? hw : 0);

  Frag<T> qf[QB][kSteps];
  f32x4 o[QB][kSteps];
  Softmax st[QB];
  int pos0[QB];
  bool col_valid[QB];
#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const int qi = q0_w + 16 * b + col;
    col_valid[b] = wave_active && qi < q_len;
    pos0[b] = ctx - q_len + q0_w + 16 * b;
    load_q<T>(qf[b], q + (static_cast<size_t>(tok0) + qi) * q_stride + static_cast<size_t>(head) * HD, col_valid[b],
              lane);
    st[b] = Softmax{LYP_NEG_INF, 0.f};
#pragma unroll
    for (int db = 0; db < kSteps; ++db) o[b][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int pos_last_w = min(pos_last_wg, pos0[0] + QB * 16 - 1);

  // ---- bringing a tile in: global -> registers -> LDS
  const int32_t* table = block_tables + static_cast<size_t>(seq) * max_blocks;
  const T* kp = static_cast<const T*>(kpool);
  const T* vp = static_cast<const T*>(vpool);
  const bool v_vectors = bs % VEC == 0;
  VecT kreg[PT::kPerThread], vreg[PT::kPerThread];
  auto zero_vec = [] {
    VecT z;
#pragma unroll
    for (int e = 0; e < VEC; ++e) z[e] = from_f32<T>(0.f);
    return z;
  };
  // Where this thread's pieces of a tile lie (the same for every tile).
  constexpr int kPer16 = 16 / VEC;
  int k_row[PT::kPerThread], k_d0[PT::kPerThread], v_blk[PT::kPerThread], v_d[PT::kPerThread], v_c[PT::kPerThread];
#pragma unroll
  for (int n = 0; n < PT::kPerThread; ++n) {
    const int v = tid + n * 256;
    k_row[n] = v / (HD / VEC);
    k_d0[n] = (v % (HD / VEC)) * VEC;
    v_blk[n] = v / (HD * kPer16);
    v_d[n] = (v % (HD * kPer16)) / kPer16;
    v_c[n] = (v % kPer16) * VEC;
  }
  const bool aligned = bs % 16 == 0;
  // Table entries of a tile's 16-key blocks: the same for the whole workgroup,
  // and read a tile ahead of the data so that the two reads do not queue up.
  auto tile_pages = [&](int kt0, int (&pg)[NB]) {
#pragma unroll
    for (int u = 0; u < NB; ++u) pg[u] = table[min((kt0 + 16 * u) / bs, max_blocks - 1)];
  };
  auto fetch = [&](int kt0, const int (&pg)[NB]) {
    if (aligned && kt0 >= lo_wg && kt0 + KT <= hi_wg) {
      // the whole tile exists and is wanted: no tests, one table entry per 16 keys
#pragma unroll
      for (int n = 0; n < PT::kPerThread; ++n) {
        if (tid + n * 256 >= PT::kKVecs) continue;
        int page_k = pg[0], page_v = pg[0];
#pragma unroll
        for (int u = 1; u < NB; ++u) {
          if (k_row[n] / 16 == u) page_k = pg[u];
          if (v_blk[n] == u) page_v = pg[u];
        }
        const int off_k = (kt0 + (k_row[n] / 16) * 16) % bs + k_row[n] % 16;
        kreg[n] = *reinterpret_cast<const VecT*>(
            kp + ((static_cast<size_t>(page_k) * nkv + kvh) * bs + off_k) * HD + k_d0[n]);
        const int off_v = (kt0 + 16 * v_blk[n]) % bs + v_c[n];
        vreg[n] = *reinterpret_cast<const VecT*>(
            vp + ((static_cast<size_t>(page_v) * nkv + kvh) * HD + v_d[n]) * bs + off_v);
      }
      return;
    }
#pragma unroll
    for (int n = 0; n < PT::kPerThread; ++n) {
      kreg[n] = zero_vec();
      vreg[n] = zero_vec();
      if (tid + n * 256 >= PT::kKVecs) continue;
      {  // keys: 16 bytes of key kt0 + k_row
        const int key = kt0 + k_row[n];
        if (key >= lo_wg && key < hi_wg) {
          const int page = table[key / bs];
          if (page >= 0)
            kreg[n] = *reinterpret_cast<const VecT*>(
                kp + ((static_cast<size_t>(page) * nkv + kvh) * bs + key % bs) * HD + k_d0[n]);
        }
      }
      {  // values: 16-key blocks one after the other, inside a block dimension by dimension
        const int d = v_d[n], key0 = kt0 + 16 * v_blk[n] + v_c[n];
        if (key0 < hi_wg && key0 + VEC > lo_wg) {
          if (v_vectors) {
            const int page = table[key0 / bs];
            if (page >= 0) {
              VecT x = *reinterpret_cast<const VecT*>(
                  vp + ((static_cast<size_t>(page) * nkv + kvh) * HD + d) * bs + key0 % bs);
#pragma unroll
              for (int e = 0; e < VEC; ++e)
                if (key0 + e < lo_wg || key0 + e >= hi_wg) x[e] = from_f32<T>(0.f);
              vreg[n] = x;
            }
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
              const int key = key0 + e;
              if (key < lo_wg || key >= hi_wg) continue;
              const int page = table[key / bs];
              if (page >= 0) vreg[n][e] = vp[((static_cast<size_t>(page) * nkv + kvh) * HD + d) * bs + key % bs];
            }
          }
        }
      }
    }
  };
  auto stash = [&](int buf) {
    T* ks = lds + buf * PT::kElems;
    T* vs = ks + KT * PT::kKLd;
#pragma unroll
    for (int n = 0; n < PT::kPerThread; ++n) {
      if (tid + n * 256 >= PT::kKVecs) continue;
      const int kr = k_row[n], d0 = k_d0[n];
      // rows are padded by 4 elements, so a 16-byte store may straddle an 8-byte boundary: two halves
      typedef T HalfT __attribute__((ext_vector_type(VEC / 2)));
      HalfT lo_h, hi_h;
#pragma unroll
      for (int e = 0; e < VEC / 2; ++e) {
        lo_h[e] = kreg[n][e];
        hi_h[e] = kreg[n][e + VEC / 2];
      }
      *reinterpret_cast<HalfT*>(ks + kr * PT::kKLd + d0) = lo_h;
      *reinterpret_cast<HalfT*>(ks + kr * PT::kKLd + d0 + VEC / 2) = hi_h;
      const int d = v_d[n], c0 = 16 * v_blk[n] + v_c[n];
#pragma unroll
      for (int e = 0; e < VEC / 2; ++e) {
        lo_h[e] = vreg[n][e];
        hi_h[e] = vreg[n][e + VEC / 2];
      }
      *reinterpret_cast<HalfT*>(vs + d * PT::kVLd + c0) = lo_h;
      *reinterpret_cast<HalfT*>(vs + d * PT::kVLd + c0 + VEC / 2) = hi_h;
    }
  };

  // ---- one tile's worth of work for this wave
  auto compute = [&](int buf, int kt0) {
    const T* ks = lds + buf * PT::kElems;
    const T* vs = ks + KT * PT::kKLd;
    f32x4 sc[QB][NB];
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      Frag<T> kf[kSteps];
      const T* krow = ks + (16 * u + lane % 16) * PT::kKLd + (lane / 16) * kSlice;
#pragma unroll
      for (int k = 0; k < kSteps; ++k) kf[k] = *reinterpret_cast<const Frag<T>*>(krow + 4 * k);
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        sc[b][u] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < kSteps; ++k) sc[b][u] = Mma16<T>::mma(kf[k], qf[b][k], sc[b][u]);
      }
    }
    Frag<T> pf[QB][NB];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      // every token of the block sees the whole tile: no masks
      const bool full = kt0 + KT - 1 <= pos0[b] && kt0 >= lo_wg && pos0[b] + 15 <= pos_last_wg &&
                        (window == 0 || kt0 > pos0[b] + 15 - window);
      if (full)
        softmax_group<T, false, NB>(sc[b], pf[b], scale_log2, kt0, pos0[b] + col, window, hi_wg, st[b], o[b], lane);
      else
        softmax_group<T, true, NB>(sc[b], pf[b], scale_log2, kt0, col_valid[b] ? pos0[b] + col : -1, window, hi_wg,
                                   st[b], o[b], lane);
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      Frag<T> vf[kSteps];
      const T* vrow = vs + (lane % 16) * PT::kVLd + 16 * u + 4 * (lane / 16);
#pragma unroll
      for (int db = 0; db < kSteps; ++db) vf[db] = *reinterpret_cast<const Frag<T>*>(vrow + db * 16 * PT::kVLd);
#pragma unroll
      for (int b = 0; b < QB; ++b)
#pragma unroll
        for (int db = 0; db < kSteps; ++db) o[b][db] = Mma16<T>::mma(vf[db], pf[b][u], o[b][db]);
    }
  };

  const int kt_first = (lo_wg / KT) * KT;
  int pages[NB];
  tile_pages(kt_first, pages);
  fetch(kt_first, pages);
  tile_pages(kt_first + KT, pages);
  stash(0);
  __syncthreads();
  int buf = 0;
  for (int kt0 = kt_first; kt0 < hi_wg; kt0 += KT) {
    const bool more = kt0 + KT < hi_wg;
    if (more) {
      fetch(kt0 + KT, pages);
      tile_pages(kt0 + 2 * KT, pages);  // for the fetch of the next round
    }
    if (wave_active && kt0 <= pos_last_w) compute(buf, kt0);
    if (PT::kBufs == 1) __syncthreads();  // everyone is done with the only buffer before it is overwritten
    const int next = PT::kBufs == 2 ? buf ^ 1 : 0;
    if (more) stash(next);
    __syncthreads();
    buf = next;
  }

#pragma unroll
  for (int b = 0; b < QB; ++b) {
    const float l = lane_groups_sum(st[b].lsum);
    if (!col_valid[b]) continue;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    const size_t token = static_cast<size_t>(tok0) + q0_w + 16 * b + col;
    T* orow = out + token * out_stride + static_cast<size_t>(head) * HD + 4 * (lane / 16);
#pragma unroll
    for (int db = 0; db < kSteps; ++db) {
      Frag<T> f;
#pragma unroll
      for (int i = 0; i < 4; ++i) f[i] = from_f32<T>(o[b][db][i] * inv);
      *reinterpret_cast<Frag<T>*>(orow + db * 16) = f;
    }
  }
}

#if LYP_HEAD_DIM % 32 == 0
// ------------------------------------------------- prefill, bfloat16, wide steps
// The same work with the 16x16x32 matrix instruction (head sizes that are
// multiples of 32), more waves per workgroup and loads that run further ahead:
// NW waves, wave w takes head w % GH and the 16 tokens of sub-block w / GH, so
// a workgroup covers (NW / GH) * 16 tokens (a unit).  The page size must be a
// multiple of 16, so that a 16-key block never straddles two pages.
//   * A lane holds eight consecutive values of the inner dimension.  For P.V the
//     inner dimension is the key: the score tiles leave lane group j with keys
//     4 j + {0..3} of two neighbouring 16-key blocks, so the value tile is
//     stored in LDS with its columns in that order (key 32 w + 16 h + 4 j + i at
//     column 32 w + 8 j + 4 h + i) and a lane reads its eight values in one piece.
//   * Tiles travel memory -> registers -> LDS two tiles ahead of their use: two
//     sets of registers, two LDS buffers.  Every round of the loop asks for
//     exactly the same loads (past the end of the keys the addresses are clamped
//     and the data is dropped), which lets the waits for them be counted exactly.
//   * When `paired`, a workgroup takes two units one after the other, number b
//     from the heavy end of the host's list and number b from the light end, so
//     that with a causal mask every workgroup has the same amount of work.
//   * The exponent is formed as fma(score, scale, -maximum); the accumulators are rescaled only
//     when a maximum grew; the sum of the probabilities is one more row of the P.V product.
struct WideTile {
  static constexpr int kKeys = HD <= 64 ? 64 : 32;
  static constexpr int kKLd = HD + 8;     // rows stay 16-byte aligned and skewed by four banks
  static constexpr int kVLd = kKeys + 8;
  static constexpr int kElems = kKeys * kKLd + HD * kVLd;
  static constexpr int kBufs = 2 * kElems * 2 <= 64 * 1024 ? 2 : 1;
  static constexpr int kVecs = kKeys * HD / 8;  // 16-byte pieces of a key tile (and of a value tile)
};

// The scores of one tile (s[u]: rows = keys kb0 + 16 u + 4 (l / 16) + i, column l % 16): update
// the running maximum `m_run` (base-2 domain), rescale the accumulators when some column's
// maximum grew (o: the output; lacc: the sum of the probabilities, which the matrix unit adds up
// with a row of ones), and return the probabilities as the column operand of the P.V product.
template <bool MASKED, int NB>
__device__ __forceinline__ void softmax_wide(const f32x4 (&s)[NB], bf16x8 (&pw)[NB / 2], float scale_log2, int kb0,
                                             int pos, int window, int hi, float& m_run, f32x4& lacc,
                                             f32x4 (&o)[kSteps], int lane) {
  bool vis[NB][4];
  float mx = LYP_NEG_INF;
#pragma unroll
  for (int u = 0; u < NB; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (MASKED) {
        const int key = kb0 + 16 * u + 4 * (lane / 16) + i;
        vis[u][i] = key <= pos && key < hi && (window == 0 || key > pos - window);
        mx = fmaxf(mx, vis[u][i] ? s[u][i] : LYP_NEG_INF);
      } else {
        vis[u][i] = true;
        mx = fmaxf(mx, s[u][i]);
      }
    }
  mx = lane_groups_max(mx);
  const float m_new = fmaxf(m_run, mx * scale_log2);  // the scale is positive
  if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
    const float alpha = fast_exp2(m_run - (m_new == LYP_NEG_INF ? 0.f : m_new));  // 0 while nothing was seen
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < 4; ++i) lacc[i] *= alpha;
#pragma unroll
    for (int db = 0; db < kSteps; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[db][i] *= alpha;
  }
  const float m_safe = m_run == LYP_NEG_INF ? 0.f : m_run;
#pragma unroll
  for (int u = 0; u < NB; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float p = fast_exp2(__builtin_fmaf(s[u][i], scale_log2, -m_safe));
      if constexpr (MASKED) p = vis[u][i] ? p : 0.f;
      pw[u / 2][4 * (u % 2) + i] = from_f32<bf16_t>(p);
    }
}

// One thread's share of a tile on its way from memory to LDS.
template <int PER>
struct TileRegs {
  bf16x8 k[PER], v[PER];
  bool lost[PER];  // the table had no page for the piece's block
};

// n_parts > 1 (grid z): a unit's key tiles are dealt to n_parts workgroups in runs; each leaves its
// running result (not normalised) in part_o [tile][token of the tile][head][part][hd] and part_ml
// [...][part][2] = (maximum in the base-2 domain, sum), and attn_merge_parts_kernel puts them together:
// for few new tokens over many keys, which would otherwise be one long walk on few compute units.
// KS = 2: two sets of NW waves share a unit; set 0 takes the unit's key tiles 0, 2, 4, ..., set 1 the
// tiles 1, 3, 5, ..., each through LDS buffers of its own, and the two running results are merged
// at the end.  Half as many tiles in a row for one unit: for launches with few units, whose time
// is that of the unit with most keys.
template <int GH, int NW, int KS>
__global__ __launch_bounds__(NW* KS* kWave, HD <= 64 ? 4 : 1) void attn_prefill_wide_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride, const void* kpool,
    const void* vpool, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_q0, int n_tiles, int nh, int nkv,
    int bs, int window, float scale_log2, int paired, float* __restrict__ part_o, float* __restrict__ part_ml,
    int n_parts) {
  using T = bf16_t;
  using WT = WideTile;
  using MMA = Mma16Wide<bf16_t>;
  constexpr int KT = WT::kKeys, NB = KT / 16, NWIDE = KT / 32, DSTEPS = HD / 32;
  constexpr int THREADS = NW * kWave;  // of one set
  constexpr int PER = (WT::kVecs + THREADS - 1) / THREADS;
  constexpr int KSTEP = KS * KT;       // from one tile of a set to its next
  constexpr int QW = (NW / GH) * 16;  // new tokens per unit
  constexpr int kSubs = 64 / QW;      // units per 64-token tile of the host's list
  static_assert(NW % GH == 0 && QW <= 64 && 64 % QW == 0, "a unit is a whole fraction of a 64-token tile");
  constexpr int kMergeFloats = 4 * kSteps + 2;  // what a lane of set 1 hands to its partner in set 0
  static_assert(KS == 1 || (KS == 2 && NW * kMergeFloats * kWave * 4 <= KS * WT::kBufs * WT::kElems * 2),
                "one or two sets; the hand-over goes through the tile buffers");
  __shared__ __attribute__((aligned(16))) T lds_all[KS * WT::kBufs * WT::kElems];

  const int lane = threadIdx.x % kWave;
  const int set = KS == 1 ? 0 : __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / THREADS);
  const int tid = threadIdx.x % THREADS;  // within the set
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  T* lds = lds_all + set * (WT::kBufs * WT::kElems);
  const int col = lane % 16, grp = lane / 16;
  const int g = nh / nkv;
  const int head_groups = (g + GH - 1) / GH;
  // grid (key/value heads x head groups, units): workgroups go to the chip's eight dies in turn by
  // their number in the launch, x fastest, so with eight key/value heads a die only ever sees the
  // keys and values of one of them and its second-level cache keeps them between tiles.
  const int kvh = blockIdx.x / head_groups;
  const int hsub = (blockIdx.x % head_groups) * GH;
  const int hw = hsub + wave % GH;
  const int head = kvh * g + (hw < g ? hw : 0);
  const T* kp = static_cast<const T*>(kpool);
  const T* vp = static_cast<const T*>(vpool);
  const size_t page_stride = static_cast<size_t>(nkv) * bs * HD;  // of both pools, in elements
  const size_t head_base = static_cast<size_t>(kvh) * bs * HD;
  const int step_blk = KSTEP / bs, step_off = KSTEP % bs;

  // Where this thread's pieces of a tile lie (the same for every tile).  Piece n is 16 bytes of
  // the keys and 16 bytes of the values of one 16-key block of the tile, so of one page.
  // A thread beyond the tile's pieces asks for some piece all the same (every thread issues the
  // same loads) and only leaves out the store to LDS.
  int p_blk[PER], p_key[PER], p_vkey[PER], k_off[PER], v_off[PER], k_lds[PER], v_lds[PER];
  bool p_live[PER];
#pragma unroll
  for (int n = 0; n < PER; ++n) {
    p_live[n] = tid + n * THREADS < WT::kVecs;
    const int v = (tid + n * THREADS) % WT::kVecs;
    const int k_row = v / (HD / 8), k_d0 = (v % (HD / 8)) * 8;
    const int v_d = (v % (HD * 2)) / 2, v_c = (v % 2) * 8;
    p_blk[n] = v / (HD * 2);                // the 16-key block, the same for both halves
    p_key[n] = k_row;                       // the key of the tile that the key piece belongs to
    p_vkey[n] = 16 * p_blk[n] + v_c;        // the first of the eight keys of the value piece
    k_off[n] = (k_row % 16) * HD + k_d0;    // from the block's first key, in the key pool
    v_off[n] = v_d * bs + v_c;              // the same in the value pool
    k_lds[n] = k_row * WT::kKLd + k_d0;
    // keys 16 blk + c .. + 7 (c = 0 or 8) are lane groups c / 4 and c / 4 + 1 of half blk % 2
    v_lds[n] = v_d * WT::kVLd + 32 * (p_blk[n] / 2) + 8 * (v_c / 4) + 4 * (p_blk[n] % 2);
  }
  auto zero_vec = [] {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = from_f32<T>(0.f);
    return z;
  };

  const int n_units = n_tiles * kSubs;
  for (int round = 0; round < (paired ? 2 : 1); ++round) {
    // the host lists tiles in rising order of position
    int unit = n_units - 1 - static_cast<int>(blockIdx.y);
    if (round == 1) {
      if (2 * static_cast<int>(blockIdx.y) >= n_units - 1) break;  // the middle unit has no partner
      unit = blockIdx.y;
    }
    const int tile = unit / kSubs;
    const int seq = tile_seq[tile];
    const int tok0 = q_start[seq];
    const int q_len = q_start[seq + 1] - tok0;
    const int ctx = ctx_len[seq];
    const int q0_wg = tile_q0[tile] + (unit % kSubs) * QW;
    if (q0_wg >= q_len) continue;  // the whole workgroup
    const int pos_first = ctx - q_len + q0_wg;
    const int pos_last_wg = pos_first + min(QW, q_len - q0_wg) - 1;
    const int lo_wg = window > 0 ? max(0, pos_first - window + 1) : 0;
    const int hi_wg = pos_last_wg + 1;

    // this wave's tokens
    const int q0_w = q0_wg + (wave / GH) * 16;
    const bool wave_active = hw < g && q0_w < q_len;
    const bool col_valid = wave_active && q0_w + col < q_len;
    const int pos0 = ctx - q_len + q0_w;
    const int pos_last_w = min(pos_last_wg, pos0 + 15);
    bf16x8 qf[DSTEPS];
    {
      const T* row = q + (static_cast<size_t>(tok0) + q0_w + col) * q_stride + static_cast<size_t>(head) * HD + 8 * grp;
#pragma unroll
      for (int s = 0; s < DSTEPS; ++s) qf[s] = col_valid ? *reinterpret_cast<const bf16x8*>(row + 32 * s) : zero_vec();
    }
    f32x4 o[kSteps];
#pragma unroll
    for (int db = 0; db < kSteps; ++db) o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = LYP_NEG_INF;
    f32x4 lacc = f32x4{0.f, 0.f, 0.f, 0.f};  // every row: the running sum of this column's probabilities
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = from_f32<T>(1.f);

    // ---- bringing tiles in.  A thread follows the block of each of its pieces from tile to
    // tile (index into the table and place in the page, without a division); the table entry is
    // read one tile ahead of the data, the data two tiles ahead of its use.  Past the last block
    // that holds a key of interest the table may hold anything, so the index is clamped there.
    const int32_t* table = block_tables + static_cast<size_t>(seq) * max_blocks;
    const int blk_last = (hi_wg - 1) / bs;
    int kt_base = (lo_wg / KT) * KT;            // the first tile of the unit, then of this workgroup's run
    int kt_end = hi_wg;                         // where the run ends
    if (n_parts > 1) {
      const int run = ((hi_wg - kt_base + KT - 1) / KT + n_parts - 1) / n_parts * KT;
      kt_base += static_cast<int>(blockIdx.z) * run;
      kt_end = min(hi_wg, kt_base + run);
    }
    const int kt_first = kt_base + set * KT;    // this set's first tile
    int w_blk[PER], w_off[PER];      // the walk: the block of the tile whose table entry is read next
    int page[PER], page_off[PER];    // for the tile whose data is asked for next
#pragma unroll
    for (int n = 0; n < PER; ++n) {
      const int x = kt_first + 16 * p_blk[n];
      w_blk[n] = x / bs;
      w_off[n] = x - w_blk[n] * bs;
    }
    auto read_table = [&](int (&pg)[PER], int (&po)[PER]) {  // for the tile of the walk, which moves on
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        pg[n] = table[min(w_blk[n], blk_last)];
        po[n] = w_off[n];
        w_blk[n] += step_blk;
        w_off[n] += step_off;
        if (w_off[n] >= bs) {
          w_off[n] -= bs;
          w_blk[n] += 1;
        }
      }
    };
    auto ask = [&](TileRegs<PER>& r, const int (&pg)[PER], const int (&po)[PER]) {
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        r.lost[n] = pg[n] < 0;
        const size_t base = static_cast<size_t>(max(pg[n], 0)) * page_stride + head_base;
        r.k[n] = *reinterpret_cast<const bf16x8*>(kp + base + (po[n] * HD + k_off[n]));
        r.v[n] = *reinterpret_cast<const bf16x8*>(vp + base + (po[n] + v_off[n]));
      }
    };
    // Keys outside [lo_wg, hi_wg) are stored as zeros: a page that was never written, or that
    // belongs to someone else by now, may hold any bit pattern.
    auto stash = [&](const TileRegs<PER>& r, int buf, int kt0) {
      T* ks = lds + buf * WT::kElems;
      T* vs = ks + KT * WT::kKLd;
      const bool inside = kt0 >= lo_wg && kt0 + KT <= hi_wg;
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        bf16x8 kx = r.k[n], vx = r.v[n];
        if (!inside || r.lost[n]) {
          const int key = kt0 + p_key[n];
          if (key < lo_wg || key >= hi_wg || r.lost[n]) kx = zero_vec();
          const int key0 = kt0 + p_vkey[n];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (key0 + e < lo_wg || key0 + e >= hi_wg || r.lost[n]) vx[e] = from_f32<T>(0.f);
        }
        if (!p_live[n]) continue;
        *reinterpret_cast<bf16x8*>(ks + k_lds[n]) = kx;
        bf16x4 lo_h, hi_h;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo_h[e] = vx[e];
          hi_h[e] = vx[e + 4];
        }
        *reinterpret_cast<bf16x4*>(vs + v_lds[n]) = lo_h;
        *reinterpret_cast<bf16x4*>(vs + v_lds[n] + 8) = hi_h;
      }
    };

    // ---- one tile's worth of work for this wave
    auto compute = [&](int buf, int kt0) {
      const T* ks = lds + buf * WT::kElems;
      const T* vs = ks + KT * WT::kKLd;
      f32x4 sc[NB];
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        const T* krow = ks + (16 * u + col) * WT::kKLd + 8 * grp;
        sc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < DSTEPS; ++s)
          sc[u] = MMA::mma(*reinterpret_cast<const bf16x8*>(krow + 32 * s), qf[s], sc[u]);
      }
      bf16x8 pw[NWIDE];
      const bool full = kt0 + KT - 1 <= pos0 && kt0 >= lo_wg && pos0 + 15 <= pos_last_wg &&
                        (window == 0 || kt0 > pos0 + 15 - window);
      if (full)
        softmax_wide<false, NB>(sc, pw, scale_log2, kt0, pos0 + col, window, hi_wg, m_run, lacc, o, lane);
      else
        softmax_wide<true, NB>(sc, pw, scale_log2, kt0, col_valid ? pos0 + col : -1, window, hi_wg, m_run, lacc, o,
                               lane);
#pragma unroll
      for (int w = 0; w < NWIDE; ++w) {
        lacc = MMA::mma(ones, pw[w], lacc);
        const T* vrow = vs + col * WT::kVLd + 32 * w + 8 * grp;
#pragma unroll
        for (int db = 0; db < kSteps; ++db)
          o[db] = MMA::mma(*reinterpret_cast<const bf16x8*>(vrow + db * 16 * WT::kVLd), pw[w], o[db]);
      }
    };

    // One round of the loop, in tiles of this set: tile kt0 is in LDS buffer `buf`, the next in
    // `ready`; the loads of the one after that are started into `filling`, whose last content is
    // in LDS already.  A set whose tile lies past the unit's keys still passes the barriers.
    auto step = [&](int kt0, int buf, TileRegs<PER>& filling, const TileRegs<PER>& ready) {
      int page_n[PER], page_off_n[PER];
      read_table(page_n, page_off_n);      // for the third tile after kt0
      ask(filling, page, page_off);        // the second after kt0
#pragma unroll
      for (int n = 0; n < PER; ++n) {
        page[n] = page_n[n];
        page_off[n] = page_off_n[n];
      }
      if (wave_active && kt0 <= pos_last_w && kt0 < kt_end) compute(buf, kt0);
      if (WT::kBufs == 1) __syncthreads();  // everyone is done with the only buffer before it is overwritten
      if (kt0 + KSTEP < kt_end) stash(ready, WT::kBufs == 2 ? buf ^ 1 : 0, kt0 + KSTEP);
      __syncthreads();
    };

    TileRegs<PER> ra, rb;
    read_table(page, page_off);
    ask(ra, page, page_off);     // the first tile
    read_table(page, page_off);
    ask(rb, page, page_off);     // the second
    read_table(page, page_off);  // for the third
    stash(ra, 0, kt_first);
    __syncthreads();
    // the bounds are those of set 0, so that every wave passes the same barriers
    for (int kb = kt_base; kb < kt_end; kb += 2 * KSTEP) {
      step(kb + set * KT, 0, ra, rb);
      if (kb + KSTEP >= kt_end) break;
      step(kb + KSTEP + set * KT, WT::kBufs == 2 ? 1 : 0, rb, ra);
    }

    if constexpr (KS == 2) {
      // Set 1 hands its maximum, sum and output to the same wave and lane of set 0.
      float* hand = reinterpret_cast<float*>(lds_all) + wave * (kMergeFloats * kWave) + lane;
      if (set == 1) {
        hand[0] = m_run;
        hand[kWave] = lacc[0];
#pragma unroll
        for (int db = 0; db < kSteps; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) hand[(2 + 4 * db + i) * kWave] = o[db][i];
      }
      __syncthreads();
      if (set == 0) {
        const float m_other = hand[0];
        const float m_new = fmaxf(m_run, m_other);
        const float m_safe = m_new == LYP_NEG_INF ? 0.f : m_new;
        const float a0 = fast_exp2(m_run - m_safe), a1 = fast_exp2(m_other - m_safe);  // 0 for a set that saw nothing
        lacc[0] = lacc[0] * a0 + hand[kWave] * a1;
#pragma unroll
        for (int db = 0; db < kSteps; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[db][i] = o[db][i] * a0 + hand[(2 + 4 * db + i) * kWave] * a1;
        m_run = m_new;  // what the sum and the output are relative to now
      }
      __syncthreads();  // the buffers are free for the next unit
    }

    if (n_parts > 1) {
      if (col_valid && set == 0) {
        const int in_tile = q0_w - tile_q0[tile] + col;
        const size_t pidx = ((static_cast<size_t>(tile) * 64 + in_tile) * nh + head) * n_parts + blockIdx.z;
        float* po = part_o + pidx * HD + 4 * grp;
#pragma unroll
        for (int db = 0; db < kSteps; ++db) *reinterpret_cast<f32x4*>(po + db * 16) = o[db];
        if (grp == 0) {
          part_ml[pidx * 2] = m_run;
          part_ml[pidx * 2 + 1] = lacc[0];
        }
      }
    } else if (col_valid && set == 0) {
      const float inv = lacc[0] > 0.f ? 1.0f / lacc[0] : 0.f;
      T* orow = out + (static_cast<size_t>(tok0) + q0_w + col) * out_stride + static_cast<size_t>(head) * HD + 4 * grp;
#pragma unroll
      for (int db = 0; db < kSteps; ++db) {
        bf16x4 f;
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = from_f32<T>(o[db][i] * inv);
        *reinterpret_cast<bf16x4*>(orow + db * 16) = f;
      }
    }
  }
}

// grid (nh, 64, tiles); one wave: the parts of one new token and head, put together.
template <typename T>
__global__ __launch_bounds__(64) void attn_merge_parts_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, int n_parts,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_q0,
    T* __restrict__ out, int out_stride, int nh) {
  const int head = blockIdx.x, in_tile = blockIdx.y, tile = blockIdx.z, lane = threadIdx.x;
  const int seq = tile_seq[tile];
  const int tok0 = q_start[seq], q_len = q_start[seq + 1] - tok0;
  const int q = tile_q0[tile] + in_tile;
  if (q >= q_len) return;
  const size_t base = ((static_cast<size_t>(tile) * 64 + in_tile) * nh + head) * n_parts;
  const float2* ml = reinterpret_cast<const float2*>(part_ml) + base;
  float m = LYP_NEG_INF;
  for (int p = 0; p < n_parts; ++p) m = fmaxf(m, ml[p].x);
  const float m_safe = m == LYP_NEG_INF ? 0.f : m;
  float l = 0.f;
  for (int p = 0; p < n_parts; ++p) l += fast_exp2(ml[p].x - m_safe) * ml[p].y;
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  T* orow = out + (static_cast<size_t>(tok0) + q) * out_stride + static_cast<size_t>(head) * HD;
  for (int d = lane; d < HD; d += kWave) {
    float acc = 0.f;
    for (int p = 0; p < n_parts; ++p) acc += fast_exp2(ml[p].x - m_safe) * part_o[(base + p) * HD + d];
    orow[d] = from_f32<T>(acc * inv);
  }
}
#endif

// ---------------------------------------------------------------------- decode
// grid (partitions, nkv * column_groups, requests); kDecodeWaves waves.  A
// workgroup takes one partition of kDecodeWaves * keys_per_wave keys and merges
// its waves' results through LDS, in a fixed order.  Column c of the tile is
// query head kvh * g + 16 * column_group + c of the request's one new token.
// How many keys a wave takes is the launch's choice (lyp_attn_decode_plan): few
// when there is little work, so that it spreads over the chip; many when there
// is a lot, so that the fixed cost of a workgroup is paid less often.
// Partials: part_o [request][head][part][hd] (not normalised), part_ml
// [request][head][part][2] = (maximum in the base-2 domain, sum).  A launch with one partition
// per request writes no partials: its workgroups normalise and write the output themselves
// (batch 64 at 2,300 keys: one kernel of 4.7 us less in each layer).
constexpr int kDecodeWaves = HD <= 128 ? 4 : 2;
constexpr int kDecodeDepth = HD <= 64 ? 4 : (HD <= 128 ? 2 : 1);  // 16-key blocks in flight per wave

// The keys one wave takes of a request of `ctx` keys when a partition may hold up to
// kDecodeWaves * keys_per_wave of them: the request gets as many partitions as that needs, and its
// keys are shared out evenly between them, in whole blocks of 16 per wave.  (With partitions of
// the full size a request just over one partition's length would fill one and barely touch the
// next, and the launch lasts as long as its fullest workgroup: batch 32 at 2,300 keys, partitions
// of 2,048: 35.9 us a layer against 27.)  Both kernels below use it, so they agree on which
// partition holds what.
__device__ __forceinline__ int decode_keys_per_wave(int ctx, int keys_per_wave) {
  const int block_keys = kDecodeWaves * keys_per_wave;
  const int parts = max(1, (ctx + block_keys - 1) / block_keys);
  const int per_part = (ctx + parts - 1) / parts;
  return max(16, (per_part + kDecodeWaves * 16 - 1) / (kDecodeWaves * 16) * 16);
}

// Floats of LDS a decode workgroup needs: every wave's output for the columns that hold a head
// (at most min(16, g) of the 16), and its maxima and sums.
constexpr int decode_lds_floats(int g) { return kDecodeWaves * ((g < 16 ? g : 16) * HD + 32); }

// WHOLE: the launch has one partition per request, which therefore holds all its keys; the
// workgroup normalises and writes the attention's output itself, and no combine pass follows.
template <typename T, bool WHOLE>
__global__ __launch_bounds__(kDecodeWaves* kWave) void attn_decode_kernel(
    const T* __restrict__ q, int q_stride, const void* kpool, const void* vpool,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ dec_seqs,
    float* __restrict__ part_o, float* __restrict__ part_ml, int max_parts, int most_keys_per_wave, int nh, int nkv,
    int bs, int window, float scale_log2, T* __restrict__ out, int out_stride) {
  extern __shared__ float s_decode[];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // the same in every lane: keeps what follows scalar
  const int g = nh / nkv;
  const int cols_most = min(16, g);
  float* s_o = s_decode;                          // [kDecodeWaves][cols_most][HD]
  float* s_m = s_decode + kDecodeWaves * cols_most * HD;  // [kDecodeWaves][16]
  float* s_l = s_m + kDecodeWaves * 16;                   // [kDecodeWaves][16]
  const int col_groups = (g + 15) / 16;
  const int kvh = blockIdx.y / col_groups;
  const int h0 = (blockIdx.y % col_groups) * 16;
  const int slot = blockIdx.z;
  const int seq = dec_seqs ? dec_seqs[slot] : slot;
  const int part = blockIdx.x;
  // The table entries of this wave's first blocks are asked for together with the request's length,
  // for partitions of the full size (the index is clamped to the row; an entry past the request's
  // keys is not used): one trip to memory less before the first keys can be asked for.  A request
  // whose partitions come out smaller (see decode_keys_per_wave) asks again, below.
  const int32_t* table = block_tables + static_cast<size_t>(seq) * max_blocks;
  const int k_begin_full = (part * kDecodeWaves + wave) * most_keys_per_wave;
  int pg_first[kDecodeDepth];
#pragma unroll
  for (int u = 0; u < kDecodeDepth; ++u) pg_first[u] = table[min((k_begin_full + 16 * u) / bs, max_blocks - 1)];
  const int ctx = ctx_len[seq];
  const int keys_per_wave = decode_keys_per_wave(ctx, most_keys_per_wave);
  const int block_keys = kDecodeWaves * keys_per_wave;
  const int k_begin = part * block_keys + wave * keys_per_wave;
  const int pos = ctx - 1;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  // (A request without keys still gets its row of zeros written when no combine pass follows.)
  if (!WHOLE && (part * block_keys >= ctx || (part + 1) * block_keys <= lo)) return;  // the whole workgroup

  const int col = lane % 16;
  const bool col_valid = h0 + col < g;
  const int head = kvh * g + h0 + (col_valid ? col : 0);
  const size_t token = q_start[seq];

  Frag<T> qf[kSteps];
  load_q<T>(qf, q + token * q_stride + static_cast<size_t>(head) * HD, col_valid, lane);
  f32x4 o[kSteps];
#pragma unroll
  for (int db = 0; db < kSteps; ++db) o[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  Softmax st{LYP_NEG_INF, 0.f};

  PagedKV kv{kpool, vpool, table, nkv, bs, kvh, max_blocks};
  const bool aligned = bs % 16 == 0;
  const int k_first = max(k_begin, (lo / 16) * 16);
  const int k_end = min(ctx, k_begin + keys_per_wave);

  Frag<T> kf[kDecodeDepth][kSteps], vf[kDecodeDepth][kSteps];
  auto is_full = [&](int kb0) { return aligned && kb0 >= lo && kb0 + 16 <= ctx; };
  // kDecodeDepth blocks of 16 keys are taken together: their scores first (after which the key
  // buffers are refilled for the next group), one maximum, one rescaling and one pass of
  // exponentials for all of them, then the products with the values (and the value buffers are
  // refilled).  Keys from k_end on are another wave's, or do not exist: masked.
  constexpr int GK = 16 * kDecodeDepth;
  int pg[kDecodeDepth];  // the pages of the group whose blocks are being asked for (blocks that lie in one page)
  auto load_k_of = [&](int u, int kb0) {
    if (is_full(kb0) && kb0 + 16 <= k_end) {
      const T* krow = static_cast<const T*>(kv.kpool) +
                      ((static_cast<size_t>(pg[u]) * nkv + kvh) * bs + kb0 % bs) * HD + (lane % 16) * HD +
                      (lane / 16) * kSlice;
#pragma unroll
      for (int s = 0; s < kSteps; ++s) kf[u][s] = *reinterpret_cast<const Frag<T>*>(krow + 4 * s);
    } else {
      load_k<T>(kf[u], kv, kb0, lo, k_end, lane);
    }
  };
  auto load_v_of = [&](int u, int kb0) {
    if (is_full(kb0) && kb0 + 16 <= k_end) {
      const T* vrow = static_cast<const T*>(kv.vpool) +
                      (static_cast<size_t>(pg[u]) * nkv + kvh) * HD * bs + kb0 % bs + (lane % 16) * bs +
                      4 * (lane / 16);
#pragma unroll
      for (int db = 0; db < kSteps; ++db)
        vf[u][db] = *reinterpret_cast<const Frag<T>*>(vrow + static_cast<size_t>(db) * 16 * bs);
    } else {
      load_v<T>(vf[u], kv, kb0, lo, k_end, lane);
    }
  };
  auto pages_of = [&](int kb0) {
#pragma unroll
    for (int u = 0; u < kDecodeDepth; ++u) pg[u] = table[min((kb0 + 16 * u) / bs, max_blocks - 1)];
  };
  if (k_first == k_begin_full) {
#pragma unroll
    for (int u = 0; u < kDecodeDepth; ++u) pg[u] = pg_first[u];
  } else {
    pages_of(k_first);
  }
#pragma unroll
  for (int u = 0; u < kDecodeDepth; ++u) {
    load_k_of(u, k_first + 16 * u);
    load_v_of(u, k_first + 16 * u);
  }
  for (int kb0 = k_first; kb0 < k_end; kb0 += GK) {
    const bool more = kb0 + GK < k_end;
    f32x4 s[kDecodeDepth];
#pragma unroll
    for (int u = 0; u < kDecodeDepth; ++u) {
      s[u] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k = 0; k < kSteps; ++k) s[u] = Mma16<T>::mma(kf[u][k], qf[k], s[u]);
    }
    if (more) {
      pages_of(kb0 + GK);  // the values of the next group, asked for below, lie in the same pages
#pragma unroll
      for (int u = 0; u < kDecodeDepth; ++u) load_k_of(u, kb0 + GK + 16 * u);
    }
    Frag<T> pf[kDecodeDepth];
    if (aligned && kb0 >= lo && kb0 + GK <= k_end)
      softmax_group<T, false, kDecodeDepth>(s, pf, scale_log2, kb0, pos, window, k_end, st, o, lane);
    else
      softmax_group<T, true, kDecodeDepth>(s, pf, scale_log2, kb0, col_valid ? pos : -1, window, k_end, st, o, lane);
#pragma unroll
    for (int u = 0; u < kDecodeDepth; ++u)
#pragma unroll
      for (int db = 0; db < kSteps; ++db) o[db] = Mma16<T>::mma(vf[u][db], pf[u], o[db]);
    if (more) {
#pragma unroll
      for (int u = 0; u < kDecodeDepth; ++u) load_v_of(u, kb0 + GK + 16 * u);
    }
  }

  const float l = lane_groups_sum(st.lsum);
  if (col < cols_most) {
#pragma unroll
    for (int db = 0; db < kSteps; ++db)
      *reinterpret_cast<f32x4*>(&s_o[(wave * cols_most + col) * HD + db * 16 + 4 * (lane / 16)]) = o[db];
  }
  if (lane < 16) {
    s_m[wave * 16 + col] = col_valid ? st.m : LYP_NEG_INF;
    s_l[wave * 16 + col] = l;
  }
  __syncthreads();

  const int ncols = min(16, g - h0);
  for (int e = threadIdx.x; e < ncols * HD; e += kDecodeWaves * kWave) {
    const int c = e / HD, d = e % HD;
    float m = s_m[c];
#pragma unroll
    for (int w = 1; w < kDecodeWaves; ++w) m = fmaxf(m, s_m[w * 16 + c]);
    float acc = 0.f, lsum = 0.f;
    if (m != LYP_NEG_INF) {
#pragma unroll
      for (int w = 0; w < kDecodeWaves; ++w) {
        if (s_m[w * 16 + c] == LYP_NEG_INF) continue;
        const float wgt = fast_exp2(s_m[w * 16 + c] - m);
        acc += wgt * s_o[(w * cols_most + c) * HD + d];
        lsum += wgt * s_l[w * 16 + c];
      }
    }
    if constexpr (WHOLE) {
      out[token * out_stride + static_cast<size_t>(kvh * g + h0 + c) * HD + d] =
          from_f32<T>(lsum > 0.f ? acc / lsum : 0.f);
    } else {
      const size_t pidx = (static_cast<size_t>(slot) * nh + kvh * g + h0 + c) * max_parts + part;
      part_o[pidx * HD + d] = acc;
      if (d == 0) {
        part_ml[pidx * 2] = m;
        part_ml[pidx * 2 + 1] = lsum;
      }
    }
  }
}

// grid (nh, requests); one wave.  Lanes first share out the partitions to find
// the overall maximum and sum, then the dimensions of the head.
template <typename T>
__global__ __launch_bounds__(64) void attn_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, int max_parts,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ dec_seqs, T* __restrict__ out, int out_stride, int nh, int window,
    int most_block_keys) {
  const int head = blockIdx.x, slot = blockIdx.y, lane = threadIdx.x;
  const int seq = dec_seqs ? dec_seqs[slot] : slot;
  const size_t base = (static_cast<size_t>(slot) * nh + head) * max_parts;
  const float2* ml = reinterpret_cast<const float2*>(part_ml) + base;
  // The kernel is a chain of trips to memory and little else, so everything that can be asked for
  // at once is: the request's length and place, and the first kFirst partitions' maxima, sums and
  // outputs whether or not the request has that many (a partition it lacks holds whatever the
  // workspace held; it is dropped once the length is known).  More partitions than that are
  // walked afterwards.
  constexpr int kFirst = 8;
  const int ctx = ctx_len[seq];
  const int tok = q_start[seq];
  constexpr int kPerLane = HD / kWave > 0 ? HD / kWave : 1;   // head dimensions a lane owns (d = lane + 64 k)
  float2 ml_first[kFirst];
  float o_first[kPerLane][kFirst];
#pragma unroll
  for (int p = 0; p < kFirst; ++p) {
    const int pc = min(p, max_parts - 1);
    ml_first[p] = ml[pc];
#pragma unroll
    for (int k = 0; k < kPerLane; ++k) {
      const int d = lane + kWave * k;
      o_first[k][p] = d < HD ? part_o[(base + pc) * HD + d] : 0.f;
    }
  }
  const int block_keys = kDecodeWaves * decode_keys_per_wave(ctx, most_block_keys / kDecodeWaves);
  const int lo = window > 0 ? max(0, ctx - window) : 0;
  const int p_lo = lo / block_keys;
  const int p_hi = (ctx + block_keys - 1) / block_keys;

  float m = LYP_NEG_INF;
#pragma unroll
  for (int p = 0; p < kFirst; ++p)
    if (p >= p_lo && p < p_hi) m = fmaxf(m, ml_first[p].x);
  for (int p = max(p_lo, kFirst) + lane; p < p_hi; p += kWave) m = fmaxf(m, ml[p].x);
  m = wave_max(m);
  const float m_safe = m == LYP_NEG_INF ? 0.f : m;
  // every lane adds up the same terms in the same order: partitions 0 .. kFirst - 1, then the rest by lanes
  float l = 0.f;
  float w_first[kFirst];
#pragma unroll
  for (int p = 0; p < kFirst; ++p) {
    w_first[p] = (p >= p_lo && p < p_hi) ? fast_exp2(ml_first[p].x - m_safe) : 0.f;
    l += (p >= p_lo && p < p_hi) ? w_first[p] * ml_first[p].y : 0.f;
  }
  float l_rest = 0.f;
  for (int p = max(p_lo, kFirst) + lane; p < p_hi; p += kWave) l_rest += fast_exp2(ml[p].x - m_safe) * ml[p].y;
  l += wave_sum(l_rest);
  const float inv = l > 0.f ? 1.0f / l : 0.f;

  T* orow = out + static_cast<size_t>(tok) * out_stride + static_cast<size_t>(head) * HD;
#pragma unroll
  for (int k = 0; k < kPerLane; ++k) {
    const int d = lane + kWave * k;
    if (d >= HD) continue;
    float acc = 0.f;
#pragma unroll
    for (int p = 0; p < kFirst; ++p) acc += (p >= p_lo && p < p_hi) ? w_first[p] * o_first[k][p] : 0.f;
#pragma unroll 4
    for (int p = max(p_lo, kFirst); p < p_hi; ++p) acc += fast_exp2(ml[p].x - m_safe) * part_o[(base + p) * HD + d];
    orow[d] = from_f32<T>(acc * inv);
  }
  if constexpr (HD < kWave || HD % kWave != 0) {   // head sizes that are no multiple of 64: the dimensions past the lanes' share
    for (int d = lane + kWave * kPerLane; d < HD; d += kWave) {
      float acc = 0.f;
      for (int p = p_lo; p < p_hi; ++p) acc += fast_exp2(ml[p].x - m_safe) * part_o[(base + p) * HD + d];
      orow[d] = from_f32<T>(acc * inv);
    }
  }
}

constexpr int kPrefillPartsMost = 16;

static int check_common(const char* name, int nh, int nkv, int bs, int max_blocks, int q_stride,
                        int out_stride, int window) {
  LYP_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "%s: %d query heads over %d key/value heads", name, nh, nkv);
  LYP_REQUIRE(bs > 0 && max_blocks > 0, "%s: page size %d, table width %d", name, bs, max_blocks);
  LYP_REQUIRE(q_stride >= nh * HD && q_stride % 4 == 0, "%s: query row stride %d", name, q_stride);
  LYP_REQUIRE(out_stride >= nh * HD && out_stride % 4 == 0, "%s: output row stride %d", name, out_stride);
  LYP_REQUIRE(window >= 0, "%s: window %d", name, window);
  return 0;
}

}  // namespace lyp

using namespace lyp;

extern "C" {

int lyp_attn_head_dim() { return HD; }
// Keys per workgroup for a decode launch over n_seqs requests whose longest
// context is max_ctx.  Both are rounded up to powers of two first, so that a
// captured launch (sized for a bucket) and a direct one choose alike.
int lyp_attn_decode_plan(int n_seqs, int max_ctx, int nh, int nkv) {
  auto pow2 = [](int v, int least) {
    int p = least;
    while (p < v) p *= 2;
    return p;
  };
  const int B = pow2(n_seqs, 1), C = pow2(max_ctx, 256);
  const int g = nh / (nkv > 0 ? nkv : 1);
  const long long base = static_cast<long long>(B) * nkv * ((g + 15) / 16);
  // Partitions grow while the launch keeps this many workgroups: one or two requests do best with one
  // workgroup per compute unit (on 256 units, batch 1 at 32,768 keys: 21.2 us a layer with 256
  // workgroups of 1,024 keys, 23.7 with 512 of 512), more requests with two; with heads of more than
  // 64 values (a key is twice the bytes) one per compute unit at every batch (heads of 128, batch 8
  // at 8,192 keys: 53.2 us with partitions of 2,048 keys, 56.7 with 1,024).
  const int enough = compute_units() * ((base < 32 || HD > 64) ? 1 : 2);
  int kpw = kPartKeys;
  while (kpw < 1024) {
    const int next_block = kDecodeWaves * kpw * 2;
    if (base * ((C + next_block - 1) / next_block) < enough) break;
    kpw *= 2;
  }
  // Two partitions per request are not worth the combine pass they need: one workgroup takes the
  // request (batch 32 at 2,300 keys: 31.4 us a layer against 36.4; at 1,000 keys 19.5 against 21.7).
  if (kDecodeWaves * kpw * 2 == C && C <= kDecodeWaves * 1024) kpw *= 2;
  return kDecodeWaves * kpw;
}

// Into how many runs lyp_attn_prefill had better cut every unit's keys (1: not at all), for
// n_tiles tiles of 64 new tokens of which one sees max_keys keys.  More than one needs a workspace:
// n_tiles * 64 * nh * parts * hd floats for part_o, n_tiles * 64 * nh * parts * 2 for part_ml.
int lyp_attn_prefill_plan(int n_tiles, int max_keys, int nh, int nkv, int dtype, int bs) {
#if LYP_HEAD_DIM % 32 == 0 && !defined(LYP_PREFILL_NARROW)
  if (dtype != kBF16 || bs <= 0 || bs % 16 != 0 || nkv <= 0 || n_tiles <= 0) return 1;
  const int g = nh / nkv;
  const int gh = g >= 4 ? 4 : (g >= 2 ? 2 : 1);
  const int unit_tokens = ((gh == 1 ? 4 : 8) / gh) * 16;
  const long long wgs = static_cast<long long>(n_tiles) * (64 / unit_tokens) * nkv * ((g + gh - 1) / gh);
  const int tiles = (max_keys + WideTile::kKeys - 1) / WideTile::kKeys;
  int parts = 1;
  // as measured: up to a workgroup per compute unit, and runs of 8 tiles at least
  while (parts < kPrefillPartsMost && wgs * parts < compute_units() && tiles / (2 * parts) >= 8) parts *= 2;
  return parts;
#else
  (void)n_tiles, (void)max_keys, (void)nh, (void)nkv, (void)dtype, (void)bs;
  return 1;
#endif
}

int lyp_attn_prefill(const void* q, int q_stride, void* out, int out_stride, const void* kpool,
                     const void* vpool, int dtype, const int32_t* block_tables, int max_blocks,
                     const int32_t* q_start, const int32_t* ctx_len, const int32_t* tile_seq,
                     const int32_t* tile_q0, int n_tiles, int nh, int nkv, int bs, int window, float scale,
                     int pair, float* part_o, float* part_ml, int n_parts, hipStream_t stream) {
  if (check_common("attn_prefill", nh, nkv, bs, max_blocks, q_stride, out_stride, window)) return -1;
  LYP_REQUIRE(n_tiles >= 0, "attn_prefill: %d tiles", n_tiles);
  LYP_REQUIRE(n_parts >= 1 && n_parts <= kPrefillPartsMost && (n_parts == 1 || (part_o && part_ml)),
              "attn_prefill: %d parts of the keys (at most %d, with a workspace)", n_parts, kPrefillPartsMost);
  if (n_tiles == 0) return 0;
  const int g = nh / nkv;
  // Heads per workgroup: as many of the group as four waves hold; the waves
  // that are left over take further tokens.
  const int gh = g >= 4 ? 4 : (g >= 2 ? 2 : 1);
  const int head_groups = (g + gh - 1) / gh;
  LYP_REQUIRE(nkv * head_groups <= 65535 && n_tiles <= 16383, "attn_prefill: too many heads or tiles for one launch");
  const float scale_log2 = scale * kLog2e;
#define LYP_PREFILL(T, GH, QB)                                                                              \
  do {                                                                                                      \
    constexpr int kQW = (4 / GH) * QB * 16;                                                                 \
    dim3 grid(n_tiles*(64 / kQW), nkv * head_groups);                                                      \
    attn_prefill_kernel<T, GH, QB><<<grid, 256, 0, stream>>>(                                               \
        static_cast<const T*>(q), q_stride, static_cast<T*>(out), out_stride, kpool, vpool, block_tables,   \
        max_blocks, q_start, ctx_len, tile_seq, tile_q0, n_tiles, nh, nkv, bs, window, scale_log2);         \
  } while (0)
#define LYP_PREFILL_T(T)                    \
  do {                                      \
    if (gh == 4) LYP_PREFILL(T, 4, kQB4);   \
    else if (gh == 2) LYP_PREFILL(T, 2, 1); \
    else LYP_PREFILL(T, 1, 1);              \
  } while (0)
  constexpr int kQB4 = LYP_PREFILL_QB;
#if LYP_HEAD_DIM % 32 == 0 && !defined(LYP_PREFILL_NARROW)
  if (dtype == kBF16 && q_stride % 8 == 0 && bs % 16 == 0) {
    // Bit 0 of `pair` is the caller's word on whether the tiles differ much in the keys they see
    // (0: no); bit 1 forbids the two sets of waves per unit (for tests and measurements).
    // Units (workgroups before pairing) beyond one per compute unit share compute units anyway;
    // pairing then evens out the causal mask's triangle of work.
#define LYP_PREFILL_WIDE_KS(GH, NW, KS)                                                                       \
  attn_prefill_wide_kernel<GH, NW, KS><<<grid, NW * KS * kWave, 0, stream>>>(                                 \
      static_cast<const bf16_t*>(q), q_stride, static_cast<bf16_t*>(out), out_stride, kpool, vpool,           \
      block_tables, max_blocks, q_start, ctx_len, tile_seq, tile_q0, n_tiles, nh, nkv, bs, window,            \
      scale_log2, paired, part_o, part_ml, n_parts)
    // Two sets of waves per unit while the launch has at most `kSplitBelow` workgroups per
    // compute unit: its time is then that of the unit with most keys, not of the sum.
#define LYP_PREFILL_WIDE(GH, NW)                                                                              \
  do {                                                                                                        \
    constexpr int kQW = (NW / GH) * 16;                                                                       \
    const int units = n_tiles * (64 / kQW);                                                                   \
    const long long wgs = static_cast<long long>(units) * nkv * head_groups * n_parts;                        \
    const int paired = (pair & 1) != 0 && n_parts == 1 && wgs > compute_units();                              \
    dim3 grid(nkv * head_groups, paired ? (units + 1) / 2 : units, n_parts);                                  \
    if (HD <= 64 && split_ok && wgs <= static_cast<long long>(kSplitBelow) * compute_units()) {               \
      if constexpr (HD <= 64) LYP_PREFILL_WIDE_KS(GH, NW, 2);                                                 \
    } else {                                                                                                  \
      LYP_PREFILL_WIDE_KS(GH, NW, 1);                                                                         \
    }                                                                                                         \
  } while (0)
    constexpr int kSplitBelow = 2;
    const bool split_ok = (pair & 2) == 0;
    if (gh == 4) LYP_PREFILL_WIDE(4, 8);
    else if (gh == 2) LYP_PREFILL_WIDE(2, 8);
    else LYP_PREFILL_WIDE(1, 4);
#undef LYP_PREFILL_WIDE
#undef LYP_PREFILL_WIDE_KS
    if (n_parts > 1)
      attn_merge_parts_kernel<bf16_t><<<dim3(nh, 64, n_tiles), 64, 0, stream>>>(
          part_o, part_ml, n_parts, q_start, tile_seq, tile_q0, static_cast<bf16_t*>(out), out_stride, nh);
    LYP_LAUNCH_CHECK("attn_prefill");
    return 0;
  }
#endif
  if (dtype == kF32) LYP_PREFILL_T(float);
  else if (dtype == kBF16) LYP_PREFILL_T(bf16_t);
  else LYP_REQUIRE(false, "attn_prefill: unknown dtype %d", dtype);
#undef LYP_PREFILL_T
#undef LYP_PREFILL
  LYP_LAUNCH_CHECK("attn_prefill");
  return 0;
}

// part_keys: keys per workgroup, from lyp_attn_decode_plan.  part_o needs
// n_seqs * nh * max_parts * hd floats, part_ml n_seqs * nh * max_parts * 2.
// Precondition, which only the caller can check (the contexts are on the device): every request's
// context is at most max_parts * part_keys.  The grid has max_parts workgroups per request and
// head group; keys of a longer request beyond those partitions would be left out without a sign
// (with max_parts == 1 the one workgroup writes the output itself from part_keys keys at most).
int lyp_attn_decode(const void* q, int q_stride, void* out, int out_stride, const void* kpool,
                    const void* vpool, int dtype, const int32_t* block_tables, int max_blocks,
                    const int32_t* q_start, const int32_t* ctx_len, const int32_t* dec_seqs, int n_seqs,
                    float* part_o, float* part_ml, int max_parts, int part_keys, int nh, int nkv, int bs,
                    int window, float scale, hipStream_t stream) {
  if (check_common("attn_decode", nh, nkv, bs, max_blocks, q_stride, out_stride, window)) return -1;
  LYP_REQUIRE(n_seqs >= 0 && max_parts > 0, "attn_decode: %d requests, %d partitions", n_seqs, max_parts);
  if (n_seqs == 0) return 0;
  const int g = nh / nkv;
  const int col_groups = (g + 15) / 16;
  LYP_REQUIRE(n_seqs <= 65535 && nkv * col_groups <= 65535, "attn_decode: launch too large");
  // One partition per request: the workgroup writes the output itself and no combine pass follows.
  const bool whole = max_parts == 1;
  LYP_REQUIRE(part_keys > 0 && part_keys % (kDecodeWaves * kPartKeys) == 0,
              "attn_decode: %d keys per workgroup is no multiple of %d", part_keys, kDecodeWaves * kPartKeys);
  LYP_REQUIRE(whole || (part_o && part_ml), "attn_decode: no workspace");
  const int keys_per_wave = part_keys / kDecodeWaves;
  const size_t lds = decode_lds_floats(g) * sizeof(float);
  dim3 grid(max_parts, nkv * col_groups, n_seqs);
  dim3 cgrid(nh, n_seqs);
  const float scale_log2 = scale * kLog2e;
#define LYP_DECODE(T, WHOLE)                                                                             \
  attn_decode_kernel<T, WHOLE><<<grid, kDecodeWaves * kWave, lds, stream>>>(                            \
      static_cast<const T*>(q), q_stride, kpool, vpool, block_tables, max_blocks, q_start, ctx_len,      \
      dec_seqs, part_o, part_ml, max_parts, keys_per_wave, nh, nkv, bs, window, scale_log2,              \
      static_cast<T*>(out), out_stride)
#define LYP_DECODE_T(T)                                                                                  \
  do {                                                                                                   \
    if (whole) {                                                                                         \
      LYP_DECODE(T, true);                                                                               \
    } else {                                                                                             \
      LYP_DECODE(T, false);                                                                              \
      attn_combine_kernel<T><<<cgrid, 64, 0, stream>>>(part_o, part_ml, max_parts, q_start, ctx_len,     \
                                                       dec_seqs, static_cast<T*>(out), out_stride, nh,   \
                                                       window, part_keys);                               \
    }                                                                                                    \
  } while (0)
  if (dtype == kF32) {
    LYP_DECODE_T(float);
  } else if (dtype == kBF16) {
    LYP_DECODE_T(bf16_t);
  } else {
    LYP_REQUIRE(false, "attn_decode: unknown dtype %d", dtype);
  }
#undef LYP_DECODE_T
#undef LYP_DECODE
  LYP_LAUNCH_CHECK("attn_decode");
  return 0;
}

}  // extern "C"
