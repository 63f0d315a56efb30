// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  `br_attn_decode_bf16` needs scratch memory from its caller when a sequence's
// pages are cut into several runs (the runs' partial sums, `part_o` and `part_ml`); this
// variant keeps that scratch in a file-scope device array of BR_NO_ALLOC_SCRATCH_FLOATS
// floats (4 MB, held by every GPU the library runs on until the process ends) and takes the
// same arguments otherwise.  It calls no hipMalloc, hipFree or allocating library routine.
//
// Limits: nsplit == 1, or  roundup64(B * nq * nsplit * hd) + B * nq * nsplit * 2
// <= BR_NO_ALLOC_SCRATCH_FLOATS; beyond that it returns BR_TOO_LARGE and prints why.
// Nothing in the scratch has to start at zero: every run writes its partial sums before
// the combining kernel reads them, so the contents a call leaves behind do no harm.
// Every call on one GPU uses that GPU's one array: calls that overlap on a GPU (two
// streams, two threads) race on it and must be ordered by the caller.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

#define BR_NO_ALLOC_SCRATCH_FLOATS (1u << 20)

extern "C" int br_attn_decode_bf16_no_alloc(const void* q, size_t q_stride, void* out, const int* slots,
                                            const int* ctx_lens, const int* block_table, int table_stride,
                                            void* cache, int B, int nq, int nkv, int hd, int page, int window,
                                            float scale, int nsplit, int variant, int fuse, const float* cs,
                                            const float* sn, int write_cache, hipStream_t s);
