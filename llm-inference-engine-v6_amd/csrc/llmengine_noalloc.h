// Entry points of libllmengine_hip.so for callers that cannot allocate device memory: code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. They have no counterpart
// in the reference engine (shivaskumar01/llm-inference-engine-v6, whose attention runs on the CPU and
// needs no device workspace); they exist for those callers only. The library's other entry points
// are declared by the Python package that loads it (llmengine/ops) and take their workspaces as
// arguments.
#pragma once

#include <hip/hip_runtime.h>

// Size of the fixed device array that the entry points below keep their partial results in:
// 2 Mi floats = 8 MiB. Every GPU the library runs on holds one such array until the process ends.
#define LLME_NOALLOC_SCRATCH_FLOATS (2u << 20)

#ifdef __cplusplus
extern "C" {
#endif

// Looks up the fixed array's address on the current device (once per device). Optional: the entry
// point below does it at its first call on a device; a caller that will run under graph capture
// calls this once per device at set-up instead. 0 on success, otherwise a HIP error code.
int llme_noalloc_init(void);

// Floats of the fixed array that a call of llme_attention_decode_noalloc with these sizes uses.
long llme_attention_decode_noalloc_scratch_floats(int n_seq, int n_q, int hd, int nsplit);

// Attention of a decode step over bfloat16 cache pages, the keys of every request cut into nsplit
// splits of split_len keys that are joined by a second kernel: what llme_attention_bf16 does for
// requests that bring one token, with the splits' partial results in the library's fixed array
// instead of a workspace. Calls no hipMalloc, hipFree or other allocating routine.
//
//   q, out        bfloat16 [n_seq, n_q * hd], one row per request (q_start[s + 1] - q_start[s] must
//                 be 1; a request with another number of rows is left alone)
//   k_cache       bfloat16 [pages, n_kv, page, hd];  v_cache bfloat16 [pages, n_kv, hd, page]
//   q_start       int32 [n_seq + 1];  ctx_len int32 [n_seq]: keys cached before the request's token,
//                 which is its own last key (it must be in the pages already)
//   block_table   int32 [n_seq, max_blocks]
//   split_len     keys per split, a multiple of 32, with nsplit * split_len >= the longest request's
//                 ctx_len + 1;  nsplit 1 .. 64
//
// Limits: hd a multiple of 16 up to 128, page a multiple of 16, n_q a multiple of n_kv, and
// n_seq * n_q * nsplit * (hd + 2) <= LLME_NOALLOC_SCRATCH_FLOATS when nsplit > 1. Returns 0, a HIP
// error code, 10001 for arguments it refuses or 10002 for sizes beyond these limits.
//
// All calls on one GPU share that GPU's array, which keeps the last call's contents (every part a
// call reads it has written before, so nothing needs clearing): calls that overlap on one GPU,
// on different streams or from different threads, race. Calls on one stream are ordered.
int llme_attention_decode_noalloc(const void* q, const void* k_cache, const void* v_cache, void* out,
                                  const int* q_start, const int* ctx_len, const int* block_table,
                                  int max_blocks, int n_seq, int n_q, int n_kv, int hd, int page, float scale,
                                  int window, int split_len, int nsplit, hipStream_t stream);

#ifdef __cplusplus
}
#endif
