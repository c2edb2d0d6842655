// An entry point of libtorchless_hip.so that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops,
// and harnesses that forbid hipMalloc.  The caller passes inputs and outputs;
// the scratch that the kernels need (the partial results of the splits of the
// keys) lies in a file-scope array of device memory of fixed size that every
// GPU the library runs on holds until the process ends.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

// Size in bytes of the scratch array (one per GPU).
#define TL_STATIC_SCRATCH_BYTES (8u << 20)

size_t tl_static_scratch_bytes(void);

// Looks up the array's device address for the current device (hipGetDevice,
// hipGetSymbolAddress; the latter may load the code object on that device) and
// keeps it.  Returns 0, or non-zero with a message in tl_last_error().  Call it
// once per device at set-up, OUTSIDE any stream capture: the lookup is no
// stream operation and must not happen while a stream of the device is
// capturing.  tl_attn_decode_bf16_static does the same lookup at its first call
// on a device if this was not called, so that first call then has to be made
// outside capture too (a warm-up step before the capture is enough).
int tl_static_scratch_ready(void);

// tl_attn_decode_bf16 without its `part` argument: bfloat16 attention of one
// new token per sequence over its pages (the token's own key is already
// committed), the keys cut into `n_splits` parts whose partial results
// (max, sum, O[d] per sequence, head and split, float) meet in the static
// scratch array and are merged by a second kernel.
//
//   q      [B, nq, d]                       bfloat16
//   pages  [n_pages, 2, nkv, 64, d]         bfloat16 (keys [64][d], values [d][64])
//   table  [B, table_stride]                page ids of each sequence, in ring order
//   row_pos[B]                              position of the new token
//   out    [B, nq, d]                       bfloat16
//
// Returns 0, or non-zero with a message in tl_last_error().  It refuses a call
// whose partial results, B * nq * n_splits * (d + 2) floats, exceed
// TL_STATIC_SCRATCH_BYTES.  It calls no hipMalloc, hipFree or allocating
// library routine; the array's device address is looked up once per device
// (tl_static_scratch_ready, or the first call with that device current, which
// therefore must not be made under stream capture).  Later calls may be
// captured into a HIP graph: they only launch kernels on `stream`.
//
// Every call on a GPU shares that GPU's array, which keeps the contents of the
// last call.  Nothing in it has to start at zero: each call's first kernel
// writes every partial that its second kernel reads.  Calls that overlap on
// one GPU (two streams, two threads) race on the array; run them one after
// the other.
int tl_attn_decode_bf16_static(const void* q, const void* pages, const int* table, int table_stride,
                               int ring_pages, const int* row_pos, int B, int nq, int nkv, int d,
                               int window, float scale, int n_splits, void* out, hipStream_t stream);

#ifdef __cplusplus
}
#endif
