// Next-token choice on the device, one workgroup per row of logits.
//
// Follows the reference's sampler (python/lyapunov_engine/engine/sampling.py:
// 15-72): greedy when the temperature is below 1e-4 (:34-38), else logits / T
// (:41), top-k keeps everything not below the k-th largest value (:44-51),
// top-p drops a token when the probability mass of the tokens before it, in
// descending order, already exceeds p, and never the first (:54-66), then one
// draw from the softmax of what is left (:68-69).  The reference sorts; here
// both cut-offs are found by bisection on the bit pattern of the values, which
// needs no sort and gives the same set (tokens that tie with the last kept one
// are all kept).  The draw is the inverse of the cumulative distribution in
// token order at a uniform number the caller supplies, so a request's tokens
// depend on its own seed and not on what else is in the batch.
#include "common.h"

namespace lyp {

constexpr int kSampleThreads = 1024;

__device__ __forceinline__ uint32_t order_key(float z) {
  const uint32_t b = __float_as_uint(z);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

struct ArgMax {
  float v;
  int i;
};
__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ __forceinline__ ArgMax block_argmax(ArgMax a, ArgMax* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    ArgMax o{__shfl_xor(a.v, off, kWave), __shfl_xor(a.i, off, kWave)};
    a = better(a, o);
  }
  __syncthreads();
  if (lane == 0) scratch[wave] = a;
  __syncthreads();
  ArgMax r = scratch[0];
  for (int w = 1; w < kSampleThreads / kWave; ++w) r = better(r, scratch[w]);
  return r;
}

__device__ __forceinline__ int block_count(int c, int* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) c += __shfl_xor(c, off, kWave);
  __syncthreads();
  if (lane == 0) scratch[wave] = c;
  __syncthreads();
  int total = 0;
  for (int w = 0; w < kSampleThreads / kWave; ++w) total += scratch[w];
  return total;
}

// First pass over the logits with the whole chip: the row is cut into
// kArgmaxChunks pieces, one workgroup each, and every piece leaves its largest
// value and the first index that has it.
constexpr int kArgmaxChunks = 32;

__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ logits, int ld, int V,
                                                            ArgMax* __restrict__ cand) {
  __shared__ ArgMax s_arg[4];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int per = (V + kArgmaxChunks - 1) / kArgmaxChunks;
  const int begin = min(V, chunk * per), end = min(V, begin + per);
  const float* x = logits + static_cast<size_t>(row) * ld;
  ArgMax am{LYP_NEG_INF, 0x7fffffff};
  for (int i = begin + threadIdx.x; i < end; i += 256) am = better(am, ArgMax{x[i], i});
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    ArgMax o{__shfl_xor(am.v, off, kWave), __shfl_xor(am.i, off, kWave)};
    am = better(am, o);
  }
  if (threadIdx.x % kWave == 0) s_arg[threadIdx.x / kWave] = am;
  __syncthreads();
  if (threadIdx.x == 0) {
    ArgMax r = s_arg[0];
    for (int w = 1; w < 4; ++w) r = better(r, s_arg[w]);
    cand[row * kArgmaxChunks + chunk] = r;
  }
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
    const int32_t* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ uniform,
    const ArgMax* __restrict__ cand, int32_t* __restrict__ out, int32_t* __restrict__ mirror) {
  __shared__ ArgMax s_arg[kSampleThreads / kWave];
  __shared__ int s_cnt[kSampleThreads / kWave];
  __shared__ float s_f[kSampleThreads / kWave];
  __shared__ float s_chunk[kSampleThreads];
  __shared__ int s_pick;
  __shared__ float s_prefix;

  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + static_cast<size_t>(row) * ld;

  ArgMax am{LYP_NEG_INF, 0x7fffffff};
  if (cand) {  // the pieces' winners instead of the whole row
    if (tid < kArgmaxChunks) am = cand[row * kArgmaxChunks + tid];
  } else {
    for (int i = tid; i < V; i += kSampleThreads) am = better(am, ArgMax{x[i], i});
  }
  am = block_argmax(am, s_arg);
  const float T = temperature[row];
  if (T < 1e-4f) {
    if (tid == 0) {
      out[row] = am.i;
      if (mirror) mirror[row] = am.i;
    }
    return;
  }
  const float zmax = am.v / T;

  // Smallest order key that survives the cut-offs; 0 keeps everything.
  uint32_t keep = 0;
  const int k = top_k[row];
  if (k > 0 && k < V) {
    uint32_t K = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = K | (1u << bit);
      int c = 0;
      for (int i = tid; i < V; i += kSampleThreads) c += order_key(x[i] / T) >= cand;
      if (block_count(c, s_cnt) >= k) K = cand;
    }
    keep = K;  // the key of the k-th largest value
  }
  const float p = top_p[row];
  if (p < 1.0f) {
    float z = 0.f;
    for (int i = tid; i < V; i += kSampleThreads) {
      const float zi = x[i] / T;
      if (order_key(zi) >= keep) z += expf(zi - zmax);
    }
    const float budget = p * block_sum(z, s_f);
    // Largest key whose strictly-greater mass still exceeds the budget; the
    // next key is the smallest that is kept.
    uint32_t K = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = K | (1u << bit);
      float mass = 0.f;
      for (int i = tid; i < V; i += kSampleThreads) {
        const float zi = x[i] / T;
        const uint32_t key = order_key(zi);
        if (key > cand && key >= keep) mass += expf(zi - zmax);
      }
      if (block_sum(mass, s_f) > budget) K = cand;
    }
    if (K + 1 > keep) keep = K + 1;
  }

  // Inverse CDF in token order: each thread owns one contiguous run of tokens.
  const int chunk = (V + kSampleThreads - 1) / kSampleThreads;
  const int begin = min(V, tid * chunk), end = min(V, begin + chunk);
  float mine = 0.f;
  for (int i = begin; i < end; ++i) {
    const float zi = x[i] / T;
    if (order_key(zi) >= keep) mine += expf(zi - zmax);
  }
  s_chunk[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int t = 0; t < kSampleThreads; ++t) total += s_chunk[t];
    const float target = uniform[row] * total;
    float prefix = 0.f;
    int pick = -1, last_nonempty = 0;
    for (int t = 0; t < kSampleThreads; ++t) {
      if (s_chunk[t] > 0.f) last_nonempty = t;
      if (pick < 0 && prefix + s_chunk[t] > target && s_chunk[t] > 0.f) {
        pick = t;
        s_prefix = prefix;
      }
      if (pick < 0) prefix += s_chunk[t];
    }
    if (pick < 0) {  // rounding pushed the target to the total: take the last token that has mass
      pick = last_nonempty;
      s_prefix = LYP_NEG_INF;
    }
    s_pick = pick;
    s_chunk[0] = target;
  }
  __syncthreads();
  if (tid == s_pick) {
    const float target = s_chunk[0];
    float run = s_prefix;
    int token = -1, last_kept = begin;
    for (int i = begin; i < end; ++i) {
      const float zi = x[i] / T;
      if (order_key(zi) < keep) continue;
      const float e = expf(zi - zmax);
      if (e <= 0.f) continue;
      last_kept = i;
      run += e;
      if (run > target) {
        token = i;
        break;
      }
    }
    const int pick = token >= 0 ? token : last_kept;
    out[row] = pick;
    if (mirror) mirror[row] = pick;
  }
}

}  // namespace lyp

using namespace lyp;

// Bytes of workspace lyp_sample wants for this many rows.
extern "C" long long lyp_sample_workspace(int rows) {
  return static_cast<long long>(rows) * kArgmaxChunks * sizeof(ArgMax);
}

// logits [rows, ld] float; temperature, top_k, top_p, uniform: one per row.
// workspace: lyp_sample_workspace(rows) bytes, or null (then one workgroup per
// row scans its whole row for the maximum).  mirror (optional): a second place
// the tokens are written to, for instance pinned host memory that the host reads
// once the kernel is done.
extern "C" int lyp_sample(const float* logits, int ld, int rows, int V, const float* temperature,
                          const int32_t* top_k, const float* top_p, const float* uniform, void* workspace,
                          int32_t* out, int32_t* mirror, hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && V > 0 && ld >= V, "sample: bad sizes rows=%d V=%d ld=%d", rows, V, ld);
  if (rows == 0) return 0;
  LYP_REQUIRE(rows <= 65535, "sample: %d rows in one launch", rows);
  if (mirror) {
    void* mapped = nullptr;
    LYP_REQUIRE(hipHostGetDevicePointer(&mapped, mirror, 0) == hipSuccess && mapped,
                "sample: the mirror is no pinned host memory that the device can write");
    mirror = static_cast<int32_t*>(mapped);
  }
  ArgMax* cand = static_cast<ArgMax*>(workspace);
  if (cand) argmax_chunks_kernel<<<dim3(kArgmaxChunks, rows), 256, 0, stream>>>(logits, ld, V, cand);
  sample_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, ld, V, temperature, top_k, top_p, uniform, cand, out,
                                                      mirror);
  LYP_LAUNCH_CHECK("sample");
  return 0;
}
