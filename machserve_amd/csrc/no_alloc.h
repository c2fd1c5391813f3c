// Decode attention for callers that cannot allocate device memory.
//
// This entry point has no counterpart in the reference.  It is for callers that cannot call hipMalloc:
// code under HIP graph capture, tight serving loops, harnesses that forbid allocation.  It is
// ms_decode_attention_nd<N> (attention of a step in which request s has the single row s, over the paged
// cache) with the workspace of the key splits in a static device array of the library instead of two
// buffers that the caller brings: S * H * nsplit * (hd + 2) floats, at most
// ms_decode_attention_noalloc_max_floats_nd<N>() = 1,048,576 (4 MiB); a larger step is refused with a
// message (ms_last_error).  It calls no hipMalloc, hipFree or allocating library routine.  Every GPU the
// library runs on holds its own array until the process ends; all calls on one GPU share it, so calls
// that overlap on one GPU race: the caller orders them (one stream, or events between streams).
// ms_decode_attention_noalloc_max_floats_nd<N>() also does the entry point's set-up for the current device (it
// looks up the array's device address, which the entry point would otherwise do at its first call there): call
// it once per device before a stream capture, and the entry point makes nothing but kernel launches.
//
// One library per head-size tile: <N> is the tile in units of 16 (1, 2, 3, 4, 6, 8, 12, 16); a head size
// runs in the next larger tile.  Operands as in ms_decode_attention_nd<N>: q [S, H * hd], key pool
// [pages, KV, ps, hd], value pool [pages, KV, hd, ps], out [S, H * hd] in the library's element type;
// block_table int32 [S, table_stride] (-1: no page); seq_pos0 int32 [S]: the row's position; window 0 = all
// keys; nsplit blocks share a request's keys (1 to 64).  Returns 0, or non-zero with ms_last_error() set.
#pragma once
#include <hip/hip_runtime.h>

#define MS_DECLARE_DECODE_ATTENTION_NOALLOC(N)                                                                            \
    extern "C" int ms_decode_attention_noalloc_nd##N(const void* q, const void* kpool, const void* vpool, void* out,      \
                                                     const int* block_table, int table_stride, const int* seq_pos0, int S, \
                                                     int H, int KV, int hd, int ps, int window, int nsplit, float scale,   \
                                                     hipStream_t stream);                                                  \
    extern "C" long ms_decode_attention_noalloc_max_floats_nd##N();

MS_DECLARE_DECODE_ATTENTION_NOALLOC(1)
MS_DECLARE_DECODE_ATTENTION_NOALLOC(2)
MS_DECLARE_DECODE_ATTENTION_NOALLOC(3)
MS_DECLARE_DECODE_ATTENTION_NOALLOC(4)
MS_DECLARE_DECODE_ATTENTION_NOALLOC(6)
MS_DECLARE_DECODE_ATTENTION_NOALLOC(8)
MS_DECLARE_DECODE_ATTENTION_NOALLOC(12)
MS_DECLARE_DECODE_ATTENTION_NOALLOC(16)
