// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wave64 reductions and thin wrappers over the MFMA builtins.
//
// Counterpart of the reference's csrc/include/utils/cuda_utils.cuh:13-149
// (WARP_SIZE 32, shuffle reductions, to_float/from_float); written for 64-wide
// wavefronts and matrix cores instead.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>

namespace lyp {

constexpr int kWave = 64;
#define LYP_NEG_INF (-__builtin_huge_valf())

using bf16_t = __bf16;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// ---------------------------------------------------------------- conversions
__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return static_cast<float>(x); }

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) {
  return static_cast<bf16_t>(x);  // round to nearest even
}

// One rotation of a pair of features by an angle with cosine c and sine s:
// (x1 c - x2 s, x2 c + x1 s).  The roundings are written out (one product
// rounded, then a fused multiply-add) so that every kernel that rotates gives
// the same bits, whatever the compiler would contract by itself.
__device__ __forceinline__ void rotate_pair(float x1, float x2, float c, float s, float& y1, float& y2) {
  y1 = __builtin_fmaf(x1, c, -(x2 * s));
  y2 = __builtin_fmaf(x2, c, x1 * s);
}

// ----------------------------------------------------------------- reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a whole workgroup; every thread gets the result.  `scratch` holds
// one float per wave.  The order of the additions is fixed by the launch shape
// alone, so a row's result does not depend on what else is in the batch.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();  // scratch may still be read from an earlier call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < nwaves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// ----------------------------------------------------------------------- MFMA
// One step of a 16x16 output tile over 16 values of the inner dimension.
// Fragment layout (both element types): lane l holds, for row (A) or column (B)
// l % 16, the four inner-dimension values 4 * (l / 16) + {0,1,2,3}.  The
// accumulator holds column l % 16, rows 4 * (l / 16) + {0,1,2,3}.
//
// float uses the true 32-bit matrix instruction (16x16x4, four issues); there
// is no reduced-precision mode involved.
template <typename T>
struct Mma16;

template <>
struct Mma16<float> {
  using Frag = f32x4;
  static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) {
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], c, 0, 0, 0);
    return c;
  }
};

template <>
struct Mma16<bf16_t> {
  using Frag = bf16x4;
  static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a),
                                                     __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
};

// A 16x16 output tile fed with 16-byte fragments: bfloat16 takes eight values
// per lane and one 16x16x32 instruction, float four values and four 16x16x4
// instructions.  Lane l holds row/column l % 16 and kElems consecutive
// inner-dimension values of group l / 16; the accumulator is laid out as in
// Mma16.
template <typename T>
struct Mma16Wide;

template <>
struct Mma16Wide<float> {
  static constexpr int kElems = 4;
  using Frag = f32x4;
  static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) { return Mma16<float>::mma(a, b, c); }
};

template <>
struct Mma16Wide<bf16_t> {
  static constexpr int kElems = 8;
  using Frag = bf16x8;
  static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

// A 32x32 output tile.  Lane l holds row/column l % 32 and kElems consecutive
// inner-dimension values of group l / 32; one call covers 2 * kElems values.
// Accumulator register v of lane l is row 8 * (v / 4) + 4 * (l / 32) + v % 4,
// column l % 32.
template <typename T>
struct Mma32;

template <>
struct Mma32<float> {
  static constexpr int kElems = 4;
  using Frag = f32x4;
  static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b[3], c, 0, 0, 0);
    return c;
  }
};

template <>
struct Mma32<bf16_t> {
  static constexpr int kElems = 8;
  using Frag = bf16x8;
  static __device__ __forceinline__ f32x16 mma(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// ------------------------------------------------------------------- maxima
// A value and where it stands; of two equal values the one that stands first wins.
struct ArgMax {
  float v;
  int i;
};
__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

// ------------------------------------------------------------- host-side glue
// Every exported function returns 0 or a negative code and leaves a message
// for lyp_last_error().
void set_error(const char* fmt, ...);

#define LYP_REQUIRE(cond, ...)   \
  do {                           \
    if (!(cond)) {               \
      lyp::set_error(__VA_ARGS__); \
      return -1;                 \
    }                            \
  } while (0)

#define LYP_LAUNCH_CHECK(name)                                                   \
  do {                                                                           \
    hipError_t e_ = hipGetLastError();                                           \
    if (e_ != hipSuccess) {                                                      \
      lyp::set_error("%s: launch failed: %s", name, hipGetErrorString(e_));      \
      return -2;                                                                 \
    }                                                                            \
  } while (0)

enum DType : int { kF32 = 0, kBF16 = 1 };

// Compute units of the current device (asked once per process).
inline int compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      n = v;
    else
      n = 256;
  }
  return n;
}


}  // namespace lyp
