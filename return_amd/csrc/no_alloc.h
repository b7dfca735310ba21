// The one entry point of the library that allocates nothing.
//
// It has no counterpart in the reference. It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// Every other entry point takes the memory for partial results from its caller.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// Floats of partial results the library holds per GPU for ra_attention_decode_static_bf16
// (16 MiB; each GPU the library runs on keeps it until the process ends).
#define RA_DECODE_STATIC_FLOATS (4 * 1024 * 1024)

#define RA_ERR_SCRATCH 3      // the call needs more partial results than RA_DECODE_STATIC_FLOATS
#define RA_ERR_SETUP 4        // the address of the library's own buffer could not be found

// ra_attention_decode_bf16 without its part_acc / part_ml arguments: the partial sums of the
// splits, n_dec * Hq * max_splits * (D + 2) floats, lie in a buffer that the library itself holds
// on the device that is current at the call (the stream must belong to it). Beyond
// RA_DECODE_STATIC_FLOATS the call is refused with RA_ERR_SCRATCH and nothing is launched.
// No hipMalloc, hipFree or other allocating routine is called. Nothing in the buffer has to start
// at zero: every split whose values the merge uses has been written by the same call. (The merge
// kernel asks for a fixed number of splits' sums before it knows how many of them hold keys; what
// an earlier call, or nobody, left in the places of the others is loaded, within the buffer, and
// discarded by the test `s < ns` before any arithmetic. That test must stay ahead of the sums.)
// All calls on one
// GPU share that GPU's buffer, so two calls that overlap in time on one GPU (different streams,
// threads or processes' graphs on the same library instance) race; calls on one stream do not.
// With merge != 0 the splits are merged inside the workgroups and the buffer is not touched.
int ra_attention_decode_static_bf16(const void* q, void* out, const void* k_pool, const void* v_pool,
                                    const int* page_table, const int* cu_pages, const int* kv_start,
                                    const int* cu_q, const int* q_start, const int* seg_ids, int n_dec,
                                    int Hq, int Hkv, int D, int P, float scale, int window,
                                    int split_tokens, int max_splits, int merge, void* stream);

#ifdef __cplusplus
}
#endif
