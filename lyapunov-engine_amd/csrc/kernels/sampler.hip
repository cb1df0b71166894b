// Next-token choice on the device, one workgroup per row of logits.
//
// Follows the reference's sampler (python/lyapunov_engine/engine/sampling.py:
// 15-72): greedy when the temperature is below 1e-4 (:34-38), else logits / T
// (:41), top-k keeps everything not below the k-th largest value (:44-51),
// top-p drops a token when the probability mass of the tokens before it, in
// descending order, already exceeds p, and never the first (:54-66), then one
// draw from the softmax of what is left (:68-69).  The reference sorts; here
// both cut-offs are found on the bit pattern of the values (through buckets of
// the distance from the largest value, then by digits within one bucket; by
// bisection over the row where that does not apply), which needs no sort and
// gives the same set (tokens that tie with the last kept one are all kept).
// Values are logits times 1 / T and the exponentials the fast ones, so a
// probability differs from the reference's in its last bits.  The draw is the inverse of the cumulative distribution in
// token order at a uniform number the caller supplies, so a request's tokens
// depend on its own seed and not on what else is in the batch.
#include "common.h"
#include "sampler_api.h"

#include <mutex>

namespace lyp {

constexpr int kSampleThreads = 1024;

__device__ __forceinline__ uint32_t order_key(float z) {
  const uint32_t b = __float_as_uint(z);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
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

// ---- the cut-offs without 32 passes over the row
//
// A token's distance from the row's largest value, in steps of 1/128, is its bucket (the last
// bucket takes everything from 32 on).  One pass over the row counts the tokens and adds up their
// mass per bucket; the bucket in which a cut-off falls follows from the running totals; a second
// pass collects that bucket's keys (a few hundred as a rule) and the cut-off is found among them,
// exactly, by digits.  Masses are added as integers (2^40 for the largest token), so a sum does not
// depend on the order in which the threads arrive.  When a bucket holds more keys than the list
// does, or the cut-off falls into the last bucket, the bisection over the whole row does the work.
using u64 = unsigned long long;
constexpr int kBuckets = 4096;
constexpr float kBucketsPerUnit = 128.f;
constexpr int kListCap = 8192;
constexpr int kMaxSegs = 8192;
constexpr float kFix = 1099511627776.f;  // 2^40
static_assert(kBuckets == 4 * kSampleThreads, "a thread looks after four buckets");

__device__ __forceinline__ int bucket_of(float zi, float zmax) {
  const float d = (zmax - zi) * kBucketsPerUnit;  // >= 0: zmax is the row's largest
  return d < static_cast<float>(kBuckets - 1) ? static_cast<int>(d) : kBuckets - 1;  // -inf and NaN: the last
}
__device__ __forceinline__ u64 mass_of(float zi, float zmax) { return static_cast<u64>(__expf(zi - zmax) * kFix); }
__device__ __forceinline__ float value_of_key(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}
__device__ __forceinline__ u64 shfl_up_u64(u64 v, int delta) {
  const uint32_t lo = __shfl_up(static_cast<uint32_t>(v), delta, kWave);
  const uint32_t hi = __shfl_up(static_cast<uint32_t>(v >> 32), delta, kWave);
  return (static_cast<u64>(hi) << 32) | lo;
}
__device__ __forceinline__ u64 shfl_u64(u64 v, int src) {
  const uint32_t lo = __shfl(static_cast<uint32_t>(v), src, kWave);
  const uint32_t hi = __shfl(static_cast<uint32_t>(v >> 32), src, kWave);
  return (static_cast<u64>(hi) << 32) | lo;
}
// Within a wave: the sum over the lanes before this one, and (every lane) the sum over all.
__device__ __forceinline__ u64 wave_excl_scan(u64 v, u64& total) {
  const int lane = threadIdx.x % kWave;
  u64 incl = v;
#pragma unroll
  for (int off = 1; off < kWave; off *= 2) {
    const u64 t = shfl_up_u64(incl, off);
    if (lane >= off) incl += t;
  }
  total = shfl_u64(incl, kWave - 1);
  return incl - v;
}
// Over the workgroup, in thread order.  scratch: one u64 per wave.
__device__ __forceinline__ u64 block_excl_scan(u64 v, u64* scratch, u64& total) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  u64 wave_total;
  const u64 excl = wave_excl_scan(v, wave_total);
  __syncthreads();
  if (lane == 0) scratch[wave] = wave_total;
  __syncthreads();
  u64 before = 0, all = 0;
  for (int w = 0; w < kSampleThreads / kWave; ++w) {
    if (w < wave) before += scratch[w];
    all += scratch[w];
  }
  total = all;
  return before + excl;
}

struct Found {
  int bucket;   // -1: the running total never got there
  u64 before;   // the total of the buckets before it
};
// The first bucket, from the row's largest value on, at which the running total reaches `need`
// (strict: exceeds it).
template <typename H>
__device__ Found find_bucket(const H* hist, u64 need, bool strict, u64* scratch, Found* out) {
  const int tid = threadIdx.x;
  u64 loc[4], mine = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    loc[j] = hist[4 * tid + j];
    mine += loc[j];
  }
  if (tid == 0) out->bucket = -1;
  u64 total;
  u64 run = block_excl_scan(mine, scratch, total);  // its barriers order the line above and the ones below
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const u64 next = run + loc[j];
    if (strict ? (run <= need && next > need) : (run < need && next >= need)) {
      out->bucket = 4 * tid + j;
      out->before = run;
    }
    run = next;
  }
  __syncthreads();
  const Found f = *out;
  __syncthreads();
  return f;
}

// The keys of bucket b into the list; returns how many there are (more than kListCap: too many).
__device__ int collect_bucket(const float* x, int V, float inv_t, float zmax, int b, uint32_t* list, int* counter) {
  if (threadIdx.x == 0) *counter = 0;
  __syncthreads();
  constexpr int U = 8;  // loads in flight per thread
  for (int i0 = threadIdx.x; i0 < V; i0 += U * kSampleThreads) {
    float v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = i0 + u * kSampleThreads < V ? x[i0 + u * kSampleThreads] : 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float zi = v[u] * inv_t;
      if (i0 + u * kSampleThreads < V && bucket_of(zi, zmax) == b) {
        const int at = atomicAdd(counter, 1);
        if (at < kListCap) list[at] = order_key(zi);
      }
    }
  }
  __syncthreads();
  const int n = *counter;
  __syncthreads();
  return n;
}

// The largest key K for which before + (weight of the list's keys >= K, those below `floor_key` left out)
// reaches `need` (strict: exceeds it).  The weight of a key is 1, or its mass.  The caller knows that the
// whole list gets there and that `before` alone does not.  By digits of at most 8 bits, from the
// highest bit in which the list's keys differ.
template <bool BY_MASS>
__device__ uint32_t select_in_list(const uint32_t* list, int n, uint32_t floor_key, float zmax, u64 before, u64 need,
                                   bool strict, u64* hist256, uint32_t* range, Found* out) {
  const int tid = threadIdx.x, lane = tid % kWave;
  if (tid == 0) {
    range[0] = 0xffffffffu;
    range[1] = 0;
  }
  __syncthreads();
  for (int i = tid; i < n; i += kSampleThreads) {
    atomicMin(&range[0], list[i]);
    atomicMax(&range[1], list[i]);
  }
  __syncthreads();
  const uint32_t kmin = range[0], kmax = range[1];
  __syncthreads();
  if (kmin == kmax) return kmax;
  int bits_left = 32 - __clz(kmin ^ kmax);  // the bits above are the same in every key
  uint32_t prefix = bits_left == 32 ? 0u : (kmax >> bits_left) << bits_left;
  while (bits_left > 0) {
    const int nb = bits_left < 8 ? bits_left : 8, shift = bits_left - nb;
    if (tid < 256) hist256[tid] = 0;
    __syncthreads();
    for (int i0 = 0; i0 < n; i0 += kSampleThreads) {
      const int i = i0 + tid;
      uint32_t key = 0;
      bool live = false;
      if (i < n) {
        key = list[i];
        live = key >= floor_key && (bits_left == 32 || (key >> bits_left) == (prefix >> bits_left));
      }
      const int digit = (key >> shift) & ((1u << nb) - 1u);
      const u64 w = !live ? 0 : (BY_MASS ? mass_of(value_of_key(key), zmax) : 1);
      // when the wave's live keys all have the same digit (the keys of a bucket are close), one add does it
      const unsigned long long live_mask = __builtin_amdgcn_ballot_w64(live);
      if (live_mask == 0) continue;
      const int first = __ffsll(static_cast<long long>(live_mask)) - 1;
      const int d0 = __shfl(digit, first, kWave);
      if (__builtin_amdgcn_ballot_w64(live && digit != d0) == 0) {
        u64 dummy, all;
        dummy = wave_excl_scan(w, all);
        (void)dummy;
        if (lane == first) atomicAdd(&hist256[d0], all);
      } else if (live) {
        atomicAdd(&hist256[digit], w);
      }
    }
    __syncthreads();
    if (tid < kWave) {  // the first wave: lane l looks after digits 255 - 4 l .. 252 - 4 l, from the top down
      u64 loc[4], mine = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        loc[j] = hist256[255 - 4 * lane - j];
        mine += loc[j];
      }
      u64 all;
      u64 run = before + wave_excl_scan(mine, all);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u64 next = run + loc[j];
        if (strict ? (run <= need && next > need) : (run < need && next >= need)) {
          out->bucket = 255 - 4 * lane - j;
          out->before = run;
        }
        run = next;
      }
    }
    __syncthreads();
    prefix |= static_cast<uint32_t>(out->bucket) << shift;
    before = out->before;
    bits_left = shift;
    __syncthreads();
  }
  return prefix;
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
    const int32_t* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ uniform,
    const ArgMax* __restrict__ cand, int n_cand, int32_t* __restrict__ out, int32_t* __restrict__ mirror) {
  __shared__ ArgMax s_arg[kSampleThreads / kWave];
  __shared__ int s_cnt[kSampleThreads / kWave];
  __shared__ float s_f[kSampleThreads / kWave];
  __shared__ u64 s_scan[kSampleThreads / kWave];
  __shared__ uint32_t s_hist_cnt[kBuckets];
  __shared__ u64 s_hist_mass[kBuckets];  // later: the segments' sums of the draw (floats)
  __shared__ uint32_t s_list[kListCap];
  __shared__ u64 s_hist256[256];
  __shared__ uint32_t s_range[2];
  __shared__ Found s_found;
  __shared__ int s_counter;
  __shared__ int s_pick, s_last;
  __shared__ float s_prefix, s_target;

  const int row = blockIdx.x, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const float* x = logits + static_cast<size_t>(row) * ld;

  ArgMax am{LYP_NEG_INF, 0x7fffffff};
  if (cand) {  // the pieces' winners instead of the whole row
    for (int i = tid; i < n_cand; i += kSampleThreads) am = better(am, cand[static_cast<size_t>(row) * n_cand + i]);
  } else {
    for (int i = tid; i < V; i += kSampleThreads) am = better(am, ArgMax{x[i], i});
  }
  am = block_argmax(am, s_arg);
  // A row without a single logit that compares (all NaN, or all -inf) has no largest one: token 0
  // stands for it, so that what is written is a token in any case (the next step looks it up).
  if (am.i < 0 || am.i >= V) am = ArgMax{LYP_NEG_INF, 0};
  const float T = temperature[row];
  if (T < 1e-4f) {
    if (tid == 0) {
      out[row] = am.i;
      if (mirror) mirror[row] = am.i;
    }
    return;
  }
  // a token's value is its logit times 1 / T, here and in every pass below
  const float inv_t = 1.0f / T;
  const float zmax = am.v * inv_t;

  // Smallest order key that survives the cut-offs; 0 keeps everything.
  uint32_t keep = 0;
  const int k = top_k[row];
  const float p = top_p[row];
  const bool cut_k = k > 0 && k < V, cut_p = p < 1.0f;
  bool whole_row = false;  // the cut-offs by bisection over the whole row
  if (cut_k || cut_p) {
    for (int b = tid; b < kBuckets; b += kSampleThreads) {
      s_hist_cnt[b] = 0;
      s_hist_mass[b] = 0;
    }
    __syncthreads();
    constexpr int U = 8;  // loads in flight per thread
    for (int i0 = tid; i0 < V; i0 += U * kSampleThreads) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = i0 + u * kSampleThreads < V ? x[i0 + u * kSampleThreads] : 0.f;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (i0 + u * kSampleThreads >= V) continue;
        const float zi = v[u] * inv_t;
        const int b = bucket_of(zi, zmax);
        if (cut_k) atomicAdd(&s_hist_cnt[b], 1u);
        if (cut_p) atomicAdd(&s_hist_mass[b], mass_of(zi, zmax));
      }
    }
    __syncthreads();
    int bucket_k = -1, n_list = 0;
    if (cut_k) {
      const Found f = find_bucket(s_hist_cnt, static_cast<u64>(k), false, s_scan, &s_found);
      bucket_k = f.bucket;
      if (f.bucket < 0 || f.bucket == kBuckets - 1) {
        whole_row = true;
      } else {
        n_list = collect_bucket(x, V, inv_t, zmax, f.bucket, s_list, &s_counter);
        if (n_list > kListCap) whole_row = true;
        else
          keep = select_in_list<false>(s_list, n_list, 0u, zmax, f.before, static_cast<u64>(k), false, s_hist256,
                                       s_range, &s_found);
      }
    }
    if (cut_p && !whole_row) {
      if (cut_k) {
        // what top-k dropped leaves the masses: the buckets after its bucket, and of that bucket
        // the keys below the cut-off
        u64 kept = 0;
        for (int i = tid; i < n_list; i += kSampleThreads)
          if (s_list[i] >= keep) kept += mass_of(value_of_key(s_list[i]), zmax);
        u64 kept_all;
        (void)block_excl_scan(kept, s_scan, kept_all);
        for (int b = tid; b < kBuckets; b += kSampleThreads)
          if (b > bucket_k) s_hist_mass[b] = 0;
        if (tid == 0) s_hist_mass[bucket_k] = kept_all;
        __syncthreads();
      }
      u64 mine = 0, total;
#pragma unroll
      for (int j = 0; j < 4; ++j) mine += s_hist_mass[4 * tid + j];
      (void)block_excl_scan(mine, s_scan, total);
      const u64 budget = static_cast<u64>(static_cast<double>(p) * static_cast<double>(total));
      const Found f = find_bucket(s_hist_mass, budget, true, s_scan, &s_found);
      if (f.bucket == kBuckets - 1) {
        whole_row = true;
      } else if (f.bucket >= 0) {
        if (f.bucket != bucket_k) n_list = collect_bucket(x, V, inv_t, zmax, f.bucket, s_list, &s_counter);
        if (n_list > kListCap) {
          whole_row = true;
        } else {
          const uint32_t keep_p = select_in_list<true>(s_list, n_list, keep, zmax, f.before, budget, true, s_hist256,
                                                       s_range, &s_found);
          if (keep_p > keep) keep = keep_p;
        }
      }
    }
  }
  if (whole_row) {
    keep = 0;
    if (cut_k) {
      uint32_t K = 0;
      for (int bit = 31; bit >= 0; --bit) {
        const uint32_t cand = K | (1u << bit);
        int c = 0;
        for (int i = tid; i < V; i += kSampleThreads) c += order_key(x[i] * inv_t) >= cand;
        if (block_count(c, s_cnt) >= k) K = cand;
      }
      keep = K;  // the key of the k-th largest value
    }
    if (cut_p) {
      float z = 0.f;
      for (int i = tid; i < V; i += kSampleThreads) {
        const float zi = x[i] * inv_t;
        if (order_key(zi) >= keep) z += __expf(zi - zmax);
      }
      const float budget = p * block_sum(z, s_f);
      // Largest key whose strictly-greater mass still exceeds the budget; the
      // next key is the smallest that is kept.
      uint32_t K = 0;
      for (int bit = 31; bit >= 0; --bit) {
        const uint32_t cand = K | (1u << bit);
        float mass = 0.f;
        for (int i = tid; i < V; i += kSampleThreads) {
          const float zi = x[i] * inv_t;
          const uint32_t key = order_key(zi);
          if (key > cand && key >= keep) mass += __expf(zi - zmax);
        }
        if (block_sum(mass, s_f) > budget) K = cand;
      }
      if (K + 1 > keep) keep = K + 1;
    }
  }

  // The draw: the inverse of the cumulative distribution in token order.  The row in segments of
  // `seg` tokens (64, more for a vocabulary beyond 64 * kMaxSegs): every wave adds up segments, the
  // segment that holds the target follows from the running totals, and one wave finds the token in it.
  float* s_seg = reinterpret_cast<float*>(s_hist_mass);
  constexpr int kSegBlocks = 8;  // a segment is at least 8 x 64 tokens: one sum across the lanes per 512 tokens
  const int seg = kWave * max(kSegBlocks, (V + kWave * kMaxSegs - 1) / (kWave * kMaxSegs));
  const int nseg = (V + seg - 1) / seg;
  auto weight_of = [&](float v) {
    const float zi = v * inv_t;
    return order_key(zi) >= keep ? __expf(zi - zmax) : 0.f;
  };
  auto weight = [&](int i) { return i < V ? weight_of(x[i]) : 0.f; };
  __syncthreads();
  constexpr int kWaves = kSampleThreads / kWave;
  if (seg == kSegBlocks * kWave) {
    for (int sg = wave; sg < nseg; sg += kWaves) {
      float v[kSegBlocks];  // the segment's loads all in flight
#pragma unroll
      for (int u = 0; u < kSegBlocks; ++u) {
        const int i = sg * seg + u * kWave + lane;
        v[u] = i < V ? x[i] : LYP_NEG_INF;
      }
      float acc = 0.f;
#pragma unroll
      for (int u = 0; u < kSegBlocks; ++u) acc += (sg * seg + u * kWave + lane) < V ? weight_of(v[u]) : 0.f;
      acc = wave_sum(acc);
      if (lane == 0) s_seg[sg] = acc;
    }
  } else {
    for (int sg = wave; sg < nseg; sg += kWaves) {
      float acc = 0.f;
      for (int j = 0; j < seg; j += kWave) acc += weight(sg * seg + j + lane);
      acc = wave_sum(acc);
      if (lane == 0) s_seg[sg] = acc;
    }
  }
  if (tid == 0) {
    s_pick = -1;
    s_last = 0;
  }
  __syncthreads();
  const int per = (nseg + kSampleThreads - 1) / kSampleThreads;
  const int sg_begin = min(nseg, tid * per), sg_end = min(nseg, sg_begin + per);
  float mine = 0.f;
  for (int sg = sg_begin; sg < sg_end; ++sg) mine += s_seg[sg];
  // running totals over the threads, in thread order: within a wave by shuffles, the waves one after the other
  float incl = mine;
#pragma unroll
  for (int off = 1; off < kWave; off *= 2) {
    const float t = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += t;
  }
  if (lane == kWave - 1) s_f[wave] = incl;
  __syncthreads();
  float before = 0.f, total = 0.f;
  for (int w = 0; w < kSampleThreads / kWave; ++w) {
    if (w < wave) before += s_f[w];
    total += s_f[w];
  }
  const float target = uniform[row] * total;
  float run = before + (incl - mine);
  for (int sg = sg_begin; sg < sg_end; ++sg) {
    const float sv = s_seg[sg], next = run + sv;
    if (sv > 0.f) {
      atomicMax(&s_last, sg);
      if (run <= target && next > target) {
        s_pick = sg;
        s_prefix = run;
      }
    }
    run = next;
  }
  __syncthreads();
  if (wave == 0) {
    // rounding may have pushed the target to the total: then the last token that has mass is taken
    const bool found = s_pick >= 0;
    const int sg = found ? s_pick : s_last;
    float run_w = found ? s_prefix : LYP_NEG_INF;
    int token = -1, last_kept = -1;
    for (int j = 0; j < seg && token < 0; j += kWave) {
      const int i = sg * seg + j + lane;
      const float e = weight(i);
      float in = e;
#pragma unroll
      for (int off = 1; off < kWave; off *= 2) {
        const float t = __shfl_up(in, off, kWave);
        if (lane >= off) in += t;
      }
      const unsigned long long has = __builtin_amdgcn_ballot_w64(e > 0.f);
      const unsigned long long hit = __builtin_amdgcn_ballot_w64(e > 0.f && run_w + in > target);
      if (has) last_kept = sg * seg + j + (63 - __clzll(static_cast<long long>(has)));
      if (hit) token = sg * seg + j + (__ffsll(static_cast<long long>(hit)) - 1);
      run_w += __shfl(in, kWave - 1, kWave);
    }
    if (lane == 0) {
      const int pick = token >= 0 ? token : (last_kept >= 0 ? last_kept : am.i);
      out[row] = pick;
      if (mirror) mirror[row] = pick;
    }
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
  sample_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, ld, V, temperature, top_k, top_p, uniform, cand,
                                                      kArgmaxChunks, out, mirror);
  LYP_LAUNCH_CHECK("sample");
  return 0;
}

// The same for logits whose maxima are known in pieces already: cand [rows][n_cand] (value, index)
// pairs, each the largest logit of one piece of its row and the first place it stands at, the
// pieces together covering the row (what lyp_lm_head leaves behind).  One kernel instead of two.
extern "C" int lyp_sample_cand(const float* logits, int ld, int rows, int V, const float* temperature,
                               const int32_t* top_k, const float* top_p, const float* uniform, const void* cand,
                               int n_cand, int32_t* out, int32_t* mirror, hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && V > 0 && ld >= V, "sample: bad sizes rows=%d V=%d ld=%d", rows, V, ld);
  LYP_REQUIRE(cand && n_cand > 0, "sample: %d candidates per row", n_cand);
  if (rows == 0) return 0;
  LYP_REQUIRE(rows <= 65535, "sample: %d rows in one launch", rows);
  if (mirror) {
    void* mapped = nullptr;
    LYP_REQUIRE(hipHostGetDevicePointer(&mapped, mirror, 0) == hipSuccess && mapped,
                "sample: the mirror is no pinned host memory that the device can write");
    mirror = static_cast<int32_t*>(mapped);
  }
  sample_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, ld, V, temperature, top_k, top_p, uniform,
                                                      static_cast<const ArgMax*>(cand), n_cand, out, mirror);
  LYP_LAUNCH_CHECK("sample");
  return 0;
}

// ------------------------------------------------ the same, allocating nothing
namespace lyp {
constexpr int kStaticSampleRows = 1024;
constexpr int kMaxDevices = 64;

// The per-piece maxima of lyp_sample_static.  In host code this name is only a
// handle for hipGetSymbolAddress; the address each GPU holds its copy at is
// looked up once per device and kept in g_scratch_ptr.
static __device__ __align__(256) unsigned char scratch[kStaticSampleRows * kArgmaxChunks * sizeof(ArgMax)];

static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

// The current device's copy of `scratch`, or null with the error text set.
static void* static_scratch() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    set_error("sample_static: no current device (or one beyond %d)", kMaxDevices);
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      set_error("sample_static: the scratch array's address on device %d: %s", device, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[device] = ptr;
  }
  return g_scratch_ptr[device];
}
}  // namespace lyp

extern "C" int lyp_sample_static_max_rows(void) { return kStaticSampleRows; }

extern "C" int lyp_sample_static(const float* logits, int ld, int rows, int V, const float* temperature,
                                 const int32_t* top_k, const float* top_p, const float* uniform, int32_t* out,
                                 int32_t* mirror, hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && V > 0 && ld >= V, "sample_static: bad sizes rows=%d V=%d ld=%d", rows, V, ld);
  LYP_REQUIRE(rows <= kStaticSampleRows, "sample_static: %d rows, the built-in scratch array holds %d", rows,
              kStaticSampleRows);
  if (rows == 0) return 0;
  void* ptr = static_scratch();
  if (!ptr) return -1;
  return lyp_sample(logits, ld, rows, V, temperature, top_k, top_p, uniform, ptr, out, mirror, stream);
}
