// An entry point that allocates nothing.
//
// It has no counterpart in the reference. It is for callers that cannot allocate device memory: code that
// runs while a HIP graph is being recorded, tight serving loops, and harnesses that forbid hipMalloc.
//
// nhv_decode_attention_bf16_no_alloc is nhv_decode_attention_bf16 (attention of single tokens over the paged
// cache, keys split over waves, then merged) without the two scratch arguments: the splits' partial results
// live in an array that is part of the library's own device image. The caller passes inputs and the output
// only. Neither this entry point nor anything it calls allocates or frees memory.
//
// Limits and rules:
//  * T * Hq * n_splits * (head size + 2) floats must fit into NHV_NO_ALLOC_SCRATCH_BYTES (4 MiB); a larger
//    call is refused with an error (return value 1, nhv_last_error() names the sizes). At head size 128 that
//    is T * Hq * n_splits <= 8065, e.g. 8 tokens of 32 heads over 31 splits.
//  * Every GPU that the library runs on holds the array (4 MiB) from the first call until the process ends.
//  * All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads)
//    race. The array keeps the last call's contents; nothing in it has to start at zero, since a call reads
//    only the entries that it has written itself.
//  * Arguments are those of nhv_decode_attention_bf16, in its order, without part_o and part_ml. As there,
//    n_splits * split_len must cover every position of the batch: a token whose position lies beyond loses the
//    keys of the splits that were not launched (nothing is read past the array).
//  * The first call on a device asks the runtime for the array's address on that device (a symbol lookup, under
//    a lock). That one call must not happen while a stream of the device is being captured into a graph: call
//    nhv_decode_attention_no_alloc_init() (which allocates nothing either) or make one ordinary call on every
//    device first; later calls only launch kernels and may be recorded.
#pragma once
#include <stddef.h>

#define NHV_NO_ALLOC_SCRATCH_BYTES ((size_t)4 << 20)

extern "C" int nhv_decode_attention_bf16_no_alloc(const void* q, const void* k_cache, const void* v_cache, void* out,
                                                  const void* token_req, const void* positions,
                                                  const void* block_tables, int max_blocks, int T, int Hq, int Hkv,
                                                  int page_size, float scale, int window, int split_len, int n_splits,
                                                  void* stream);

// asks for the array's address on the current device and keeps it (0, or 1 with nhv_last_error() set); a
// call on a device whose address is known already does nothing
extern "C" int nhv_decode_attention_no_alloc_init();

// bytes of the scratch array (NHV_NO_ALLOC_SCRATCH_BYTES), for callers that size their calls by it
extern "C" size_t nhv_decode_attention_no_alloc_limit();
