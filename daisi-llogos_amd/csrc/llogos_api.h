// Entry points of the kernel library that are meant for callers outside the package's own
// Python face (which declares what it calls through ctypes).  C linkage; every function
// returns 0, a negative code (-1 bad argument, -2 shape not supported, -3 larger than a fixed
// capacity) or a positive hipError_t, and launches on the current device.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Decode attention that allocates nothing.  It has no counterpart in the reference; it is
// for callers that cannot allocate device memory: code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc.  Same arguments, kernels and results as
// llogos_attn_decode_bf16 (one query token per sequence over the paged bfloat16 cache, head
// sizes 64 and 128, up to 16 query heads per key/value head) without the workspace: the
// partial results of the blocks along the context go to a device array of fixed size that the
// library holds on every GPU it runs on, until the process ends
// (llogos_attn_decode_static_capacity() floats, 16 MiB).  The caller passes inputs and the
// output [batch, n_heads * head_dim] (bfloat16); neither this call nor anything it calls
// allocates or frees memory.
//   -3  the step needs more scratch than the array holds
//       (llogos_attn_decode_workspace(batch, n_heads, n_kv_heads, head_dim, table_width) floats);
//       nothing is launched.
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams,
// two threads) race, so order them.  Nothing in the array needs clearing between calls.
// The first call on a device looks the array's address up (hipGetSymbolAddress), with that
// device current; llogos_attn_decode_static_init() does the same ahead of time, for a caller
// that wants no first-call work inside a captured or timed region.
int llogos_attn_decode_static_bf16(void* out, const void* q, int q_stride, const void* k_pool,
                                   const void* v_pool, const int* table, int table_stride, int table_width,
                                   const int* tok_pos, int batch, int n_heads, int n_kv_heads, int head_dim,
                                   float scale, int window, int sinks, hipStream_t stream);
int llogos_attn_decode_static_init(void);
long long llogos_attn_decode_static_capacity(void);

// floats of workspace that the decode attention needs for a step (0 when one block a sequence
// and kv head covers the whole page table)
long long llogos_attn_decode_workspace(int batch, int n_heads, int n_kv_heads, int head_dim, int table_width);

#ifdef __cplusplus
}
#endif
