// An entry point for callers that cannot allocate device memory: code that runs under HIP graph
// capture, tight serving loops that must not touch the allocator, harnesses that forbid it.  It has
// no counterpart in the reference (whose engine allocates its scratch tensors per call).
//
// da_attn_decode_split_static is da_attn_decode_split (attn_decode.hip: decode attention with every
// (sequence, head) pair's keys shared out over n_splits workgroups) without the workspace argument:
// the partial results go through a buffer that is part of the library's own device image,
// DA_DECODE_STATIC_SCRATCH_BYTES long, of which every GPU the library runs on holds its own copy
// until the process ends.  The caller passes inputs and outputs only.  No hipMalloc, hipFree or
// other allocating call is made.
//
//  * Sizes: S * Hq * n_splits * (D + 2) * 4 bytes must fit the buffer; more is refused with a
//    message (da_last_error), nothing is launched.
//  * The buffer keeps the last call's contents.  Nothing in it needs to start at zero: every
//    workgroup of the first kernel writes all D + 2 floats of its share (an empty share writes a
//    zero sum and a maximum of -inf) before the merge kernel, which follows on the same stream,
//    reads them.
//  * Every call on a GPU uses that GPU's one buffer: calls that overlap in time on one GPU (two
//    streams, two host threads) race on it.  Calls on one stream follow each other and are safe.
#pragma once

#define DA_DECODE_STATIC_SCRATCH_BYTES (8 << 20)

// One stream at a time per GPU: two calls whose kernels may overlap on one GPU (two streams, two host
// threads, two engines of one process) race on that GPU's one buffer, and nothing detects it.
extern "C" int da_attn_decode_split_static(const void* q, int q_ld, const void* cache, const int* block_table,
                                           int max_blocks, const int* seq_lens, int S, int Hq, int Hkv, int D,
                                           int page, float scale, int window, void* out, int out_ld, int n_splits,
                                           void* stream);
