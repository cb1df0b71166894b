// C interface of the sampler library code (sampler.hip).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

extern "C" {

// Bytes of workspace lyp_sample wants for this many rows.
long long lyp_sample_workspace(int rows);

// One token per row of logits [rows, ld] (float); temperature, top_k, top_p,
// uniform: one per row.  workspace: lyp_sample_workspace(rows) bytes of device
// memory (the per-piece maxima of every row), or null.
int lyp_sample(const float* logits, int ld, int rows, int V, const float* temperature, const int32_t* top_k,
               const float* top_p, const float* uniform, void* workspace, int32_t* out, int32_t* mirror,
               hipStream_t stream);

// lyp_sample for logits whose row maxima are known in pieces: cand [rows][n_cand] pairs of (float
// value, int32 index), the largest logit of each piece and the first place it stands at.
int lyp_sample_cand(const float* logits, int ld, int rows, int V, const float* temperature, const int32_t* top_k,
                    const float* top_p, const float* uniform, const void* cand, int n_cand, int32_t* out,
                    int32_t* mirror, hipStream_t stream);

// lyp_sample for callers that cannot allocate device memory: code under graph
// capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
// counterpart in the reference (whose sampler, engine/sampling.py:15-72, runs
// torch operators that allocate as they go).  The per-piece maxima live in an
// array that is part of the library's code object (256 KiB on every GPU the
// library runs on, held until the process ends) instead of a workspace the
// caller brings; nothing is allocated or freed, on the first call or later.
//   * at most lyp_sample_static_max_rows() rows; more are refused with an error;
//   * every call on a GPU uses that GPU's one array, which keeps the last call's
//     contents.  Nothing in it has to start at zero: the first kernel writes
//     every value the second one reads.  Calls that overlap on one GPU (two
//     streams, two threads) race on it and must be ordered by the caller;
//   * the device that owns `stream` has to be the current one.
int lyp_sample_static(const float* logits, int ld, int rows, int V, const float* temperature, const int32_t* top_k,
                      const float* top_p, const float* uniform, int32_t* out, int32_t* mirror, hipStream_t stream);
int lyp_sample_static_max_rows(void);

}  // extern "C"
