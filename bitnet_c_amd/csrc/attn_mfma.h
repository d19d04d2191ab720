// Entry points of attn_mfma.hip that other native code may call.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Floats of the library's own scratch array (see bn_attn_mfma_decode_static): 16 MiB on every GPU
// that loads this library, held until the process ends.
#define BN_ATTN_STATIC_SCRATCH_FLOATS (4u * 1024u * 1024u)

// Returned when a call needs more scratch than BN_ATTN_STATIC_SCRATCH_FLOATS; nothing was launched.
#define BN_ERR_SCRATCH (-3)

// The decode form of bn_attn_mfma (one new token per sequence over the paged bf16 cache, the keys
// split over n_splits workgroups and merged in split order) for callers that cannot allocate: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The reference has
// no counterpart; its back-ends allocate their work buffers themselves.
//
// k_pages and vt_pages are blocked pages (common.h: [pages, Hkv, 64 * hs] each, keys and values of a page in the order in
// which the kernel loads them), as everywhere in attn_mfma.hip.  block_table [n_seqs, bt_stride >= 1]: every entry names a
// page of the pool, also those behind a sequence's last page (a workgroup asks for its first block of keys before it
// knows the sequence's length, and drops it if the sequence ends before it).
// Same arguments and the same result, bit for bit, as bn_attn_mfma with tiles == null, except that
// the split partials (n_seqs * H * n_splits * (hs + 2) floats) live in a file-scope device array
// of BN_ATTN_STATIC_SCRATCH_FLOATS floats instead of buffers the caller brings.  It calls no
// hipMalloc, hipFree or allocating library routine.  A call that needs more scratch returns
// BN_ERR_SCRATCH and launches nothing.  Every call on a GPU shares that GPU's array: calls that
// overlap on one GPU (two streams, two threads) race on it, so keep them on one stream.  Nothing in
// the array has to start at zero (every partial that the merge reads is written first by the same
// call), and the array keeps the last call's contents.  The first call on a GPU looks the array's
// address up (hipGetSymbolAddress, under a lock), which is no stream operation: a caller that records
// graphs makes one call outside any capture first; every later call only launches kernels.
int bn_attn_mfma_decode_static(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                               const void* vt_pages, const int* block_table, int bt_stride, const int* seq_lens,
                               int n_seqs, int H, int Hkv, int hs, int GT, int window, float scale, int n_splits,
                               int chunk, const float* inv_freq, int rotate, int write_kv, const int* by_length,
                               hipStream_t s);

#ifdef __cplusplus
}
#endif
