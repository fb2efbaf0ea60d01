// Entry points that allocate nothing.
//
// They have no counterpart in the reference.  They are for callers that cannot allocate device
// memory around a call: code that runs under HIP graph capture, tight serving loops, and
// harnesses that forbid hipMalloc.  Such a caller brings the inputs and outputs; what the kernels
// need beyond those (the partial results of a sequence's keys shared among workgroups) lives in
// a device array that the library itself holds, one copy on every GPU the library runs on, until
// the process ends.
#pragma once
#include <hip/hip_runtime.h>

// The array's size: 2 Mi floats = 8 MiB on each GPU.
#define AGAVE_NOALLOC_SCRATCH_FLOATS (2u << 20)

extern "C" {

// Looks up the array's address on the current device and raises the kernels' LDS allowance.
// Call it once per device, with that device current, before a graph capture that contains the
// entry point below (outside a capture the entry point does it by itself at its first call on a
// device).  Returns 0, or a negative code with a message in agave_last_error().
int agave_attn_noalloc_init(void);

// Decode attention over the paged cache, as agave_attn_decode_mfma, with the partial results of
// a split plan kept in the library's own array instead of buffers the caller allocates.
//   needs  N * nh * splits * (hd + 2) <= AGAVE_NOALLOC_SCRATCH_FLOATS  when splits > 1;
//   larger steps are refused with a message (use agave_attn_decode_mfma with buffers of your own).
// It calls no hipMalloc, hipFree or other allocating routine.  Every call on a GPU shares that
// GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls on one
// stream do not.  Nothing in the array has to start at zero: every slot a call reads, it has
// written first.
int agave_attn_decode_mfma_noalloc(const void* q, long ldq, void* out, long ldo, const void* k_pages,
                                   const void* v_pages, const int* table, int width, const int* base, int n_pages,
                                   const int* tok_seq, const int* tok_pos, int N, int nh, int nkv, int hd, float scale,
                                   int window, int splits, int pages_per_split, int seq_is_token,
                                   int table_from_reach, hipStream_t stream);
}
