// Row-wise kernels of a decoder step: embedding gather, RMSNorm fused with the
// residual add, rotary position encoding fused with the paged K/V write, the
// SwiGLU gate and a dtype cast.  All arithmetic is 32-bit; only loads and
// stores see the storage type.
//
// What they compute follows the reference:
//   embedding         python/lyapunov_engine/models/llama.py:205
//   RMSNorm           csrc/kernels/fused_rmsnorm_swiglu.cu:15-113 (optional
//                     residual add :42-48, x * inv_rms * gamma :96-101)
//   rotary + K/V page csrc/kernels/fused_rope_paged.cu:7-86 (pairs (i, i+hd/2),
//                     V copied unrotated, key slot ((page*nkv+head)*bs+off)*hd;
//                     values are stored here as [hd][bs] per page and head,
//                     the layout the attention kernels read)
//   SwiGLU            csrc/kernels/fused_rmsnorm_swiglu.cu:152-179
#include "common.h"

namespace lyp {

// ------------------------------------------------------------------ embedding
template <typename TW>
__global__ void embedding_kernel(const int32_t* __restrict__ ids, const TW* __restrict__ table,
                                 float* __restrict__ out, int H) {
  const int t = blockIdx.x;
  const TW* row = table + static_cast<size_t>(ids[t]) * H;
  float* o = out + static_cast<size_t>(t) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32(row[i]);
}

// -------------------------------------------------------------------- RMSNorm
// h is the 32-bit residual stream.  With `delta`, h + delta is normed, and
// written back to h unless `rows` selects a subset (the last norm before the
// output head, where h is not used again).
// `delta` may come as n_parts partial sums, part_stride elements apart, that
// are added up here in order (what the few-rows product leaves behind).
template <typename TW, typename TD, typename T>
__global__ void rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, int n_parts,
                               size_t part_stride, const TW* __restrict__ w, T* __restrict__ out,
                               const int32_t* __restrict__ rows, int H, float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* hrow = h + src * H;
  const TD* drow = delta ? delta + src * H : nullptr;
  const bool write_back = drow != nullptr && rows == nullptr;
  auto delta_at = [&](int i) {
    float d = 0.f;
    for (int p = 0; p < n_parts; ++p) d += to_f32(drow[p * part_stride + i]);
    return d;
  };

  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = hrow[i];
    if (drow) {
      v += delta_at(i);
      if (write_back) hrow[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps);

  T* orow = out + static_cast<size_t>(r) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = hrow[i];
    if (drow && !write_back) v += delta_at(i);
    orow[i] = from_f32<T>((v * inv) * to_f32(w[i]));
  }
}

// The same for rows whose length is a multiple of 4 and fits in registers: one
// read of the row, 16-byte accesses.
template <typename TW, typename TD, typename T, int MAXV>
__global__ void rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta, int n_parts,
                                   size_t part_stride, const TW* __restrict__ w, T* __restrict__ out,
                                   const int32_t* __restrict__ rows, int H, float eps) {
  typedef T Vec4T __attribute__((ext_vector_type(4)));
  typedef TD Vec4D __attribute__((ext_vector_type(4)));
  typedef TW Vec4W __attribute__((ext_vector_type(4)));
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  f32x4* hrow = reinterpret_cast<f32x4*>(h + src * H);
  const Vec4D* drow = delta ? reinterpret_cast<const Vec4D*>(delta + src * H) : nullptr;
  const bool write_back = drow != nullptr && rows == nullptr;
  const int nvec = H / 4;
  const size_t part_vecs = part_stride / 4;

  f32x4 vals[MAXV];
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int idx = threadIdx.x + v * blockDim.x;
    if (idx < nvec) {
      f32x4 x = hrow[idx];
      if (drow) {
        for (int p = 0; p < n_parts; ++p) {
          const Vec4D d = drow[p * part_vecs + idx];
#pragma unroll
          for (int i = 0; i < 4; ++i) x[i] += to_f32(d[i]);
        }
        if (write_back) hrow[idx] = x;
      }
      vals[v] = x;
      ss += x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps);
  Vec4T* orow = reinterpret_cast<Vec4T*>(out + static_cast<size_t>(r) * H);
  const Vec4W* wrow = reinterpret_cast<const Vec4W*>(w);
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int idx = threadIdx.x + v * blockDim.x;
    if (idx < nvec) {
      const Vec4W wv = wrow[idx];
      Vec4T o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = from_f32<T>((vals[v][i] * inv) * to_f32(wv[i]));
      orow[idx] = o;
    }
  }
}

// RMSNorm of rows of activations in their own type (no residual stream); for
// parts that norm something other than the hidden state.
template <typename TW, typename T>
__global__ void rmsnorm_act_kernel(const T* __restrict__ x, const TW* __restrict__ w,
                                   T* __restrict__ out, int H, float eps) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const T* xrow = x + r * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = to_f32(xrow[i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps);
  T* orow = out + r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    orow[i] = from_f32<T>((to_f32(xrow[i]) * inv) * to_f32(w[i]));
}

// ------------------------------------------------- rotary encoding + K/V write
// qkv row of a token: nh query heads, nkv key heads, nkv value heads, hd each.
// The first `rot` dimensions of every query and key head are rotated in place
// (pair (i, i + rot/2)) by the angle of the token's absolute position; then the
// key and value heads are copied into the token's slot of the paged cache.
template <typename T>
__global__ void rope_kv_kernel(T* __restrict__ qkv, const int32_t* __restrict__ positions,
                               const float* __restrict__ cos_sin,
                               const int32_t* __restrict__ slots, T* __restrict__ kpool,
                               T* __restrict__ vpool, int nh, int nkv, int hd, int rot, int bs,
                               int has_kv) {
  const int t = blockIdx.x;
  const int n_rot_heads = has_kv ? nh + nkv : nh;
  const int width = has_kv ? (nh + 2 * nkv) * hd : nh * hd;
  T* row = qkv + static_cast<size_t>(t) * width;

  if (rot > 0) {
    const int half = rot / 2;
    const float* cs = cos_sin + static_cast<size_t>(positions[t]) * rot;
    for (int it = threadIdx.x; it < n_rot_heads * half; it += blockDim.x) {
      const int head = it / half, i = it % half;
      const float c = cs[i], s = cs[half + i];
      T* x = row + head * hd;
      float y1, y2;
      rotate_pair(to_f32(x[i]), to_f32(x[i + half]), c, s, y1, y2);
      x[i] = from_f32<T>(y1);
      x[i + half] = from_f32<T>(y2);
    }
  }
  if (!has_kv) return;
  const int slot = slots[t];
  if (slot < 0) return;  // uniform over the block: no barrier is skipped by part of it
  __syncthreads();
  const size_t page = slot / bs, off = slot % bs;
  const T* k = row + nh * hd;
  const T* v = row + (nh + nkv) * hd;
  for (int it = threadIdx.x; it < nkv * hd; it += blockDim.x) {
    const int kvh = it / hd, d = it % hd;
    kpool[((page * nkv + kvh) * bs + off) * hd + d] = k[it];
    vpool[((page * nkv + kvh) * hd + d) * bs + off] = v[it];
  }
}

// The same with 16-byte accesses and 16 tokens per workgroup: a thread rotates
// a run of VEC pairs, copies VEC values of a key at a time, and stores one
// dimension of the values of all 16 tokens at once when their slots are 16
// neighbouring places of one page (the usual case in a prompt: the value pages
// are [hd][bs], so a single token's values are 2-byte stores 2 bs bytes apart).
// Needs hd % VEC == 0, (rot / 2) % VEC == 0 and 16-byte aligned rows (the
// launcher checks).  The arithmetic, element by element, is that of
// rope_kv_kernel.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_tile_kernel(T* __restrict__ qkv, const int32_t* __restrict__ positions,
                                                           const float* __restrict__ cos_sin,
                                                           const int32_t* __restrict__ slots, T* __restrict__ kpool,
                                                           T* __restrict__ vpool, int n_tokens, int nh, int nkv, int hd,
                                                           int rot, int bs, int has_kv) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int TOK = 16;
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  __shared__ int s_slot[TOK];
  __shared__ int s_run;  // 1: the slots are TOK neighbouring places of one page, the first at a multiple of VEC
  const int t0 = blockIdx.x * TOK;
  const int n = min(TOK, n_tokens - t0);
  const int width = has_kv ? (nh + 2 * nkv) * hd : nh * hd;
  T* rows = qkv + static_cast<size_t>(t0) * width;

  // The heads are dealt out over the workgroups of a tile of tokens (blockIdx.y): query head h
  // goes to workgroup h % Y, key/value head k to workgroup k % Y, which rotates that key head and
  // stores its keys and values.
  const int Y = gridDim.y, y = blockIdx.y;
  const int my_q = (nh - y + Y - 1) / Y, my_kv = has_kv ? (nkv - y + Y - 1) / Y : 0;
  if (rot > 0) {
    const int half = rot / 2, runs = half / VEC, per_token = (my_q + my_kv) * runs;
    for (int it = threadIdx.x; it < n * per_token; it += blockDim.x) {
      const int j = it / per_token, rest = it % per_token;
      const int mine = rest / runs, i0 = (rest % runs) * VEC;
      const int head = mine < my_q ? y + mine * Y : nh + y + (mine - my_q) * Y;
      const float* cs = cos_sin + static_cast<size_t>(positions[t0 + j]) * rot;
      T* x = rows + static_cast<size_t>(j) * width + head * hd + i0;
      VecT a = *reinterpret_cast<const VecT*>(x), b = *reinterpret_cast<const VecT*>(x + half);
      VecT ra, rb;
#pragma unroll
      for (int q = 0; q < VEC / 4; ++q) {
        const f32x4 c = *reinterpret_cast<const f32x4*>(cs + i0 + 4 * q);
        const f32x4 sn = *reinterpret_cast<const f32x4*>(cs + half + i0 + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float y1, y2;
          rotate_pair(to_f32(a[4 * q + e]), to_f32(b[4 * q + e]), c[e], sn[e], y1, y2);
          ra[4 * q + e] = from_f32<T>(y1);
          rb[4 * q + e] = from_f32<T>(y2);
        }
      }
      *reinterpret_cast<VecT*>(x) = ra;
      *reinterpret_cast<VecT*>(x + half) = rb;
    }
  }
  if (!has_kv) return;
  if (threadIdx.x < TOK) s_slot[threadIdx.x] = threadIdx.x < n ? slots[t0 + threadIdx.x] : -1;
  __syncthreads();  // the rotated keys are in place, the slots are known
  if (threadIdx.x == 0) {
    const int first = s_slot[0];
    bool run = n == TOK && first >= 0 && first % bs % VEC == 0 && first % bs + TOK <= bs;
    for (int j = 1; j < TOK && run; ++j) run = s_slot[j] == first + j;
    s_run = run;
  }
  const int kv_runs = my_kv * hd / VEC;
  for (int it = threadIdx.x; it < n * kv_runs; it += blockDim.x) {
    const int j = it / kv_runs, rest = it % kv_runs;
    const int slot = s_slot[j];
    if (slot < 0) continue;
    const size_t page = slot / bs, off = slot % bs;
    const int kvh = y + (rest * VEC / hd) * Y, d = rest * VEC % hd;
    *reinterpret_cast<VecT*>(kpool + ((page * nkv + kvh) * bs + off) * hd + d) =
        *reinterpret_cast<const VecT*>(rows + static_cast<size_t>(j) * width + (nh + kvh) * hd + d);
  }
  __syncthreads();  // s_run
  const T* v0 = rows + (nh + nkv) * hd;
  if (s_run) {
    const size_t page = s_slot[0] / bs, off = s_slot[0] % bs;
    for (int it = threadIdx.x; it < my_kv * hd; it += blockDim.x) {
      const int kvh = y + (it / hd) * Y, d = it % hd;
      T* dst = vpool + ((page * nkv + kvh) * hd + d) * bs + off;
#pragma unroll
      for (int q = 0; q < TOK / VEC; ++q) {
        VecT x;
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[e] = v0[static_cast<size_t>(q * VEC + e) * width + kvh * hd + d];
        *reinterpret_cast<VecT*>(dst + q * VEC) = x;
      }
    }
  } else {
    for (int it = threadIdx.x; it < n * my_kv * hd; it += blockDim.x) {
      const int j = it / (my_kv * hd), rest = it % (my_kv * hd);
      const int slot = s_slot[j];
      if (slot < 0) continue;
      const size_t page = slot / bs, off = slot % bs;
      const int kvh = y + (rest / hd) * Y, d = rest % hd;
      vpool[((page * nkv + kvh) * hd + d) * bs + off] = v0[static_cast<size_t>(j) * width + kvh * hd + d];
    }
  }
}

// --------------------------------------------------------------------- SwiGLU
// interleave == 0: a row of gu is all gates, then all ups.  interleave == 8:
// tiles of 16 columns, eight gates then the eight ups that go with them.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total, int interleave) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / I, i = idx % I;
  const size_t gi = interleave ? (i / 8) * 16 + i % 8 : i;
  const size_t ui = interleave ? gi + 8 : I + i;
  const float g = to_f32(gu[t * 2 * I + gi]);
  const float u = to_f32(gu[t * 2 * I + ui]);
  out[idx] = from_f32<T>((g / (1.0f + expf(-g))) * u);
}

// The same, eight outputs per thread with 16-byte accesses; needs I % 8 == 0
// and 16-byte aligned rows.  In the tiled layout a thread's eight gates and
// eight ups are 32 consecutive bytes (bfloat16) of the input.
template <typename T>
__global__ void swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total8,
                                  int interleave) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;  // one run of eight outputs
  if (idx >= total8) return;
  const size_t per_row = I / 8;
  const size_t t = idx / per_row, c = idx % per_row;
  const T* row = gu + t * 2 * I;
  const T* gp = interleave ? row + c * 16 : row + c * 8;
  const T* up = interleave ? gp + 8 : row + I + c * 8;
  T* op = out + t * I + c * 8;
#pragma unroll
  for (int h = 0; h < 8 / VEC; ++h) {
    const VecT g = *reinterpret_cast<const VecT*>(gp + h * VEC);
    const VecT u = *reinterpret_cast<const VecT*>(up + h * VEC);
    VecT o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float gf = to_f32(g[e]);
      const float ex = sizeof(T) == 4 ? expf(-gf) : __expf(-gf);
      o[e] = from_f32<T>((gf / (1.0f + ex)) * to_f32(u[e]));
    }
    *reinterpret_cast<VecT*>(op + h * VEC) = o;
  }
}

// ----------------------------------------------------------------------- cast
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx < n) out[idx] = from_f32<TO>(to_f32(in[idx]));
}

// out[i] = parts[0][i] + parts[1][i] + ... in that order, in 32-bit: the float partial sums of a
// product whose inner dimension was cut into slices, for a consumer that is not a norm.
template <typename TO>
__global__ void sum_parts_kernel(const float* __restrict__ parts, int n_parts, size_t n, TO* __restrict__ out) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  float acc = parts[idx];
  for (int s = 1; s < n_parts; ++s) acc += parts[static_cast<size_t>(s) * n + idx];
  out[idx] = from_f32<TO>(acc);
}

// Threads per row of the two-pass norm kernels (rows whose length or alignment keeps them from
// the one-pass kernel).  Measured on gfx950 with 2,048 rows (kernel_bench rmsnorm): up to 1,024
// values one or two waves are as good as any size; at 2,050 values 256 threads take 11.4 us where
// 128 take 15.0, 320 16.1 and 512 13.9; from 4,100 values on every size from 64 to 1,024 gives
// the same time.  `g_norm_threads` (set by lyp_norm_threads_override, 0: this rule) is there
// for that measurement.
static int g_norm_threads = 0;
static int norm_threads(int H) {
  if (g_norm_threads > 0) return g_norm_threads;
  if (H <= 1024) return H <= 512 ? 64 : 128;
  return H < 4096 ? 256 : 512;
}

// Reads `n` 16-byte words once and keeps one word per workgroup: what memory gives a kernel that
// does nothing but stream (the yardstick the weight-streaming products are held against).
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ src, size_t n,
                                                          uint32_t* __restrict__ sink) {
  uint32_t acc = 0;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  // four loads in flight per thread
  for (; i + 3 * stride < n; i += 4 * stride) {
    const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < n; i += stride) {
    const uint4 a = src[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) acc ^= __shfl_xor(acc, off, kWave);
  if (threadIdx.x % kWave == 0) sink[blockIdx.x * (256 / kWave) + threadIdx.x / kWave] = acc;
}

// The same bytes read the way the weight-streaming products read a matrix [rows][row_bytes]: a wave
// takes 16 rows at a time, an instruction 64 bytes of each of them, 8 steps of 128 bytes per row in
// flight; then the next 16 rows that are its turn.  row_bytes a multiple of 2048.
// FULL: 8 rows a wave and 128 bytes (a whole cache line) of each per load instead.
template <bool FULL>
__global__ __launch_bounds__(256) void stream_rows_kernel(const uint4* __restrict__ src, int rows, int row_bytes,
                                                         uint32_t* __restrict__ sink) {
  constexpr int R = FULL ? 8 : 16;       // rows a wave walks at a time
  constexpr int G = kWave / R;           // 16-byte pieces of a row per load instruction
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int r = lane % R, j = lane / R;
  const int tiles = rows / R, row_words = row_bytes / 16;
  uint32_t acc = 0;
  for (int tile = blockIdx.x * 4 + wave; tile < tiles; tile += gridDim.x * 4) {
    const uint4* p = src + static_cast<size_t>(tile * R + r) * row_words + j;
    for (int c = 0; c < row_words; c += 16 * G) {   // 16 loads in flight: 16 G pieces of every row
      uint4 v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = p[c + u * G];
#pragma unroll
      for (int u = 0; u < 16; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) acc ^= __shfl_xor(acc, off, kWave);
  if (lane == 0) sink[blockIdx.x * 4 + wave] = acc;
}

// A step's table of small integers from pinned host memory (which the device reads through the
// same address) to its place on the device, in one launch; `n_patch` words from `patch_at` on come
// from `patch` on the device instead (token ids that only the device knows yet).
__global__ __launch_bounds__(256) void table_load_kernel(const int32_t* __restrict__ src, int32_t* __restrict__ dst,
                                                         int n, const int32_t* __restrict__ patch, int patch_at,
                                                         int n_patch) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int k = i - patch_at;
  dst[i] = (patch != nullptr && k >= 0 && k < n_patch) ? patch[k] : src[i];
}

}  // namespace lyp

using namespace lyp;

extern "C" {

// Threads per row for the two-pass norm kernels instead of the built-in rule (0: the rule again).
// A multiple of 64 up to 1024; for measurements.
int lyp_norm_threads_override(int threads) {
  LYP_REQUIRE(threads >= 0 && threads <= 1024 && threads % 64 == 0, "norm threads: %d", threads);
  g_norm_threads = threads;
  return 0;
}

// Streams `bytes` (a multiple of 16) of device memory through `blocks` workgroups of 256 threads;
// sink: blocks * 4 words.
int lyp_stream_read(const void* src, long long bytes, int blocks, uint32_t* sink, hipStream_t stream) {
  LYP_REQUIRE(src && sink && bytes > 0 && bytes % 16 == 0 && blocks > 0 && blocks <= 65535 &&
              reinterpret_cast<uintptr_t>(src) % 16 == 0, "stream_read: %lld bytes in %d workgroups", bytes, blocks);
  stream_read_kernel<<<blocks, 256, 0, stream>>>(static_cast<const uint4*>(src), static_cast<size_t>(bytes / 16), sink);
  LYP_LAUNCH_CHECK("stream_read");
  return 0;
}

// The same through stream_rows_kernel, as a matrix of rows of row_bytes (a multiple of 2048; bytes a multiple of 16 rows).
int lyp_stream_rows(const void* src, long long bytes, int row_bytes, int whole_lines, int blocks, uint32_t* sink,
                    hipStream_t stream) {
  LYP_REQUIRE(src && sink && bytes > 0 && row_bytes > 0 && row_bytes % 2048 == 0 && bytes % (16LL * row_bytes) == 0 &&
              blocks > 0 && blocks <= 65535 && bytes / row_bytes < (1LL << 31),
              "stream_rows: %lld bytes in rows of %d, %d workgroups", bytes, row_bytes, blocks);
  if (whole_lines)
    stream_rows_kernel<true><<<blocks, 256, 0, stream>>>(static_cast<const uint4*>(src), static_cast<int>(bytes / row_bytes), row_bytes, sink);
  else
    stream_rows_kernel<false><<<blocks, 256, 0, stream>>>(static_cast<const uint4*>(src), static_cast<int>(bytes / row_bytes), row_bytes, sink);
  LYP_LAUNCH_CHECK("stream_rows");
  return 0;
}

// dst[0..n) on the device = src[0..n) in pinned host memory, except dst[patch_at .. patch_at + n_patch)
// = patch[0..n_patch) (on the device; may be null).
int lyp_table_load(const int32_t* src, int32_t* dst, int n, const int32_t* patch, int patch_at, int n_patch,
                   hipStream_t stream) {
  LYP_REQUIRE(n >= 0 && src && dst, "table_load: %d words", n);
  LYP_REQUIRE(!patch || (patch_at >= 0 && n_patch >= 0 && patch_at + n_patch <= n), "table_load: patch %d + %d of %d",
              patch_at, n_patch, n);
  if (n == 0) return 0;
  void* mapped = nullptr;  // the device's address of the host memory (the same one, where memory is mapped so)
  LYP_REQUIRE(hipHostGetDevicePointer(&mapped, const_cast<int32_t*>(src), 0) == hipSuccess && mapped,
              "table_load: the source is no pinned host memory that the device can read");
  table_load_kernel<<<(n + 255) / 256, 256, 0, stream>>>(static_cast<const int32_t*>(mapped), dst, n, patch, patch_at,
                                                         n_patch);
  LYP_LAUNCH_CHECK("table_load");
  return 0;
}

int lyp_embedding(const int32_t* ids, const void* table, int table_dtype, float* out, int T, int H,
                  hipStream_t stream) {
  LYP_REQUIRE(T >= 0 && H > 0, "embedding: bad sizes T=%d H=%d", T, H);
  if (T == 0) return 0;
  const int threads = H >= 1024 ? 256 : 128;
  if (table_dtype == kF32)
    embedding_kernel<float><<<T, threads, 0, stream>>>(ids, static_cast<const float*>(table), out, H);
  else if (table_dtype == kBF16)
    embedding_kernel<bf16_t><<<T, threads, 0, stream>>>(ids, static_cast<const bf16_t*>(table), out, H);
  else
    LYP_REQUIRE(false, "embedding: unknown table dtype %d", table_dtype);
  LYP_LAUNCH_CHECK("embedding");
  return 0;
}

// h [*, H] float; out of act_dtype; w of w_dtype; rows optional [n_rows].
// delta (optional) is either one tensor of act_dtype (delta_parts == 0) or
// delta_parts float tensors, part_stride elements apart, whose sum is meant.
int lyp_rmsnorm(float* h, const void* delta, int delta_parts, long long part_stride, const void* w, int w_dtype,
                void* out, int act_dtype, const int32_t* rows, int n_rows, int H, float eps, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && H > 0, "rmsnorm: bad sizes rows=%d H=%d", n_rows, H);
  LYP_REQUIRE(delta_parts >= 0 && (delta_parts == 0 || delta != nullptr), "rmsnorm: partial sums without data");
  if (n_rows == 0) return 0;
  int threads = norm_threads(H);
  const bool parts = delta_parts > 0;
  const int n_parts = parts ? delta_parts : 1;
  const size_t stride = parts ? static_cast<size_t>(part_stride) : 0;
  // rows of up to 16384 values in steps of 4, and 16-byte aligned operands, take the one-pass kernel
  const bool vec = H % 4 == 0 && H <= 16384 && reinterpret_cast<uintptr_t>(h) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(delta) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out) % 16 == 0 && stride % 4 == 0;
  if (vec) threads = H <= 1024 ? 64 * ((H / 4 + 255) / 256) : (H <= 4096 ? 256 : (H <= 8192 ? 512 : 1024));
#define LYP_NORM(TW, TD, T)                                                                           \
  do {                                                                                                \
    if (vec)                                                                                          \
      rmsnorm_vec_kernel<TW, TD, T, 4><<<n_rows, threads, 0, stream>>>(                               \
          h, static_cast<const TD*>(delta), n_parts, stride, static_cast<const TW*>(w),               \
          static_cast<T*>(out), rows, H, eps);                                                        \
    else                                                                                              \
      rmsnorm_kernel<TW, TD, T><<<n_rows, threads, 0, stream>>>(                                      \
          h, static_cast<const TD*>(delta), n_parts, stride, static_cast<const TW*>(w),               \
          static_cast<T*>(out), rows, H, eps);                                                        \
  } while (0)
#define LYP_NORM_D(TW, T)               \
  do {                                  \
    if (parts) LYP_NORM(TW, float, T);  \
    else LYP_NORM(TW, T, T);            \
  } while (0)
  if (w_dtype == kF32 && act_dtype == kF32) LYP_NORM_D(float, float);
  else if (w_dtype == kF32 && act_dtype == kBF16) LYP_NORM_D(float, bf16_t);
  else if (w_dtype == kBF16 && act_dtype == kF32) LYP_NORM_D(bf16_t, float);
  else if (w_dtype == kBF16 && act_dtype == kBF16) LYP_NORM_D(bf16_t, bf16_t);
  else LYP_REQUIRE(false, "rmsnorm: unknown dtypes w=%d act=%d", w_dtype, act_dtype);
#undef LYP_NORM_D
#undef LYP_NORM
  LYP_LAUNCH_CHECK("rmsnorm");
  return 0;
}

int lyp_rmsnorm_act(const void* x, const void* w, int w_dtype, void* out, int act_dtype, int n_rows,
                    int H, float eps, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && H > 0, "rmsnorm_act: bad sizes rows=%d H=%d", n_rows, H);
  if (n_rows == 0) return 0;
  const int threads = norm_threads(H);
#define LYP_NORM(TW, T)                                                                      \
  rmsnorm_act_kernel<TW, T><<<n_rows, threads, 0, stream>>>(                                 \
      static_cast<const T*>(x), static_cast<const TW*>(w), static_cast<T*>(out), H, eps)
  if (w_dtype == kF32 && act_dtype == kF32) LYP_NORM(float, float);
  else if (w_dtype == kF32 && act_dtype == kBF16) LYP_NORM(float, bf16_t);
  else if (w_dtype == kBF16 && act_dtype == kF32) LYP_NORM(bf16_t, float);
  else if (w_dtype == kBF16 && act_dtype == kBF16) LYP_NORM(bf16_t, bf16_t);
  else LYP_REQUIRE(false, "rmsnorm_act: unknown dtypes w=%d act=%d", w_dtype, act_dtype);
#undef LYP_NORM
  LYP_LAUNCH_CHECK("rmsnorm_act");
  return 0;
}

// qkv [T, (nh + 2 nkv) hd] (or [T, nh hd] when has_kv == 0), rotated in place.
// cos_sin [max_pos, rot]: rot/2 cosines then rot/2 sines per position; rot == 0
// means no rotation.  slots [T]: page * bs + offset, or -1 for "do not store".
int lyp_rope_kv_write(void* qkv, int dtype, const int32_t* positions, const float* cos_sin,
                      const int32_t* slots, void* kpool, void* vpool, int T, int nh, int nkv, int hd,
                      int rot, int bs, int has_kv, hipStream_t stream) {
  LYP_REQUIRE(T >= 0 && nh > 0 && nkv >= 0 && hd > 0 && bs > 0, "rope_kv_write: bad sizes");
  LYP_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "rope_kv_write: rotary width %d of head %d", rot, hd);
  LYP_REQUIRE(rot == 0 || cos_sin != nullptr, "rope_kv_write: rotation without a table");
  LYP_REQUIRE(!has_kv || (slots && kpool && vpool), "rope_kv_write: cache write without a cache");
  if (T == 0) return 0;
  const int threads = 256;
  const int vec = dtype == kF32 ? 4 : 8;
  const int width = (has_kv ? nh + 2 * nkv : nh) * hd;
  // With 16 or more tokens: the kernel that takes 16 of them per workgroup, if everything is
  // aligned for 16-byte accesses (bs % vec: the value pages' rows then are, too).
  const bool aligned = T >= 16 && hd % vec == 0 && (rot / 2) % vec == 0 && width % vec == 0 && bs % vec == 0 &&
                       reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && reinterpret_cast<uintptr_t>(cos_sin) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(kpool) % 16 == 0 && reinterpret_cast<uintptr_t>(vpool) % 16 == 0;
  // the heads of a tile of tokens go to 8 workgroups, to more while the launch would leave compute units without one
  int per_tile = 8;
  while (((T + 15) / 16) * per_tile < compute_units() && per_tile < nh) per_tile *= 2;
  const dim3 tiles((T + 15) / 16, per_tile);
  if (aligned && dtype == kF32) {
    rope_kv_tile_kernel<float><<<tiles, threads, 0, stream>>>(static_cast<float*>(qkv), positions, cos_sin, slots,
                                                              static_cast<float*>(kpool), static_cast<float*>(vpool),
                                                              T, nh, nkv, hd, rot, bs, has_kv);
  } else if (aligned && dtype == kBF16) {
    rope_kv_tile_kernel<bf16_t><<<tiles, threads, 0, stream>>>(static_cast<bf16_t*>(qkv), positions, cos_sin, slots,
                                                               static_cast<bf16_t*>(kpool),
                                                               static_cast<bf16_t*>(vpool), T, nh, nkv, hd, rot, bs,
                                                               has_kv);
  } else if (dtype == kF32)
    rope_kv_kernel<float><<<T, threads, 0, stream>>>(static_cast<float*>(qkv), positions, cos_sin, slots,
                                                     static_cast<float*>(kpool), static_cast<float*>(vpool),
                                                     nh, nkv, hd, rot, bs, has_kv);
  else if (dtype == kBF16)
    rope_kv_kernel<bf16_t><<<T, threads, 0, stream>>>(static_cast<bf16_t*>(qkv), positions, cos_sin, slots,
                                                      static_cast<bf16_t*>(kpool),
                                                      static_cast<bf16_t*>(vpool), nh, nkv, hd, rot, bs,
                                                      has_kv);
  else
    LYP_REQUIRE(false, "rope_kv_write: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

int lyp_swiglu(const void* gate_up, void* out, int dtype, int T, int I, int interleave, hipStream_t stream) {
  LYP_REQUIRE(T >= 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
  LYP_REQUIRE(interleave == 0 || (interleave == 8 && I % 8 == 0), "swiglu: interleave %d with I=%d", interleave, I);
  const size_t total = static_cast<size_t>(T) * I;
  if (total == 0) return 0;
  const int threads = 256;
  const bool vec = I % 8 == 0 && reinterpret_cast<uintptr_t>(gate_up) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const size_t work = vec ? total / 8 : total;
  LYP_REQUIRE((work + threads - 1) / threads <= 2147483647u, "swiglu: too many elements for one launch");
  const unsigned blocks = static_cast<unsigned>((work + threads - 1) / threads);
#define LYP_SWIGLU(T)                                                                                         \
  do {                                                                                                        \
    if (vec)                                                                                                  \
      swiglu_vec_kernel<T><<<blocks, threads, 0, stream>>>(static_cast<const T*>(gate_up), static_cast<T*>(out), \
                                                           I, work, interleave);                              \
    else                                                                                                      \
      swiglu_kernel<T><<<blocks, threads, 0, stream>>>(static_cast<const T*>(gate_up), static_cast<T*>(out), I, \
                                                       total, interleave);                                    \
  } while (0)
  if (dtype == kF32) LYP_SWIGLU(float);
  else if (dtype == kBF16) LYP_SWIGLU(bf16_t);
  else LYP_REQUIRE(false, "swiglu: unknown dtype %d", dtype);
#undef LYP_SWIGLU
  LYP_LAUNCH_CHECK("swiglu");
  return 0;
}

int lyp_cast(const void* in, int in_dtype, void* out, int out_dtype, long long n, hipStream_t stream) {
  LYP_REQUIRE(n >= 0, "cast: negative count");
  if (n == 0) return 0;
  const int threads = 256;
  const unsigned blocks = static_cast<unsigned>((n + threads - 1) / threads);
  if (in_dtype == kBF16 && out_dtype == kF32)
    cast_kernel<bf16_t, float><<<blocks, threads, 0, stream>>>(static_cast<const bf16_t*>(in),
                                                               static_cast<float*>(out), n);
  else if (in_dtype == kF32 && out_dtype == kBF16)
    cast_kernel<float, bf16_t><<<blocks, threads, 0, stream>>>(static_cast<const float*>(in),
                                                               static_cast<bf16_t*>(out), n);
  else
    LYP_REQUIRE(false, "cast: unsupported pair %d -> %d", in_dtype, out_dtype);
  LYP_LAUNCH_CHECK("cast");
  return 0;
}

// out [n] (float or the activation type) = the sum over parts [n_parts][n] (float), slice by slice.
int lyp_sum_parts(const float* parts, int n_parts, long long n, void* out, int out_dtype, hipStream_t stream) {
  LYP_REQUIRE(n >= 0 && n_parts >= 1, "sum_parts: %d parts of %lld values", n_parts, n);
  if (n == 0) return 0;
  const int threads = 256;
  const unsigned blocks = static_cast<unsigned>((n + threads - 1) / threads);
  if (out_dtype == kF32)
    sum_parts_kernel<float><<<blocks, threads, 0, stream>>>(parts, n_parts, static_cast<size_t>(n), static_cast<float*>(out));
  else if (out_dtype == kBF16)
    sum_parts_kernel<bf16_t><<<blocks, threads, 0, stream>>>(parts, n_parts, static_cast<size_t>(n), static_cast<bf16_t*>(out));
  else
    LYP_REQUIRE(false, "sum_parts: unknown output type %d", out_dtype);
  LYP_LAUNCH_CHECK("sum_parts");
  return 0;
}

}  // extern "C"
