/* kvx_debug.h -- measurement and test hooks of libkvx.so.

   NOT part of the drop-in boundary: nothing here replaces an interface of the reference, no
   engine needs it, and it may change without notice.  The library's own tests and bench.py use
   it to tell which kernels a call ran on and what the memory system delivers for a page list. */
#ifndef KVX_DEBUG_H
#define KVX_DEBUG_H

#include "kvx.h"

#ifdef __cplusplus
extern "C" {
#endif

/* How many attend calls of this process went to the format-generic kernels and how many to the
   matrix-core (MFMA) kernels, so tests can tell which path they measured. */
void kvx_debug_attend_paths(uint64_t *generic_calls, uint64_t *matrix_core_calls);

/* How many consecutive 8-row tiles of a kv_attend_prefill call at head dimension 64 or 128 share
   a workgroup and a staged page (1 = every tile on its own; 0 = invalid arguments), so tests can
   tell which kernel a chunk ran on. */
uint32_t kvx_debug_prefill_tiles_together(const kvx_layout *layout, uint32_t query_heads,
                                          uint32_t committed_tokens, uint32_t rows, uint32_t splits);

/* Streams the pages of `page_table` (n_pages device entries of an int4, head dimension 256
   storage) with exactly the loads of the int4 decode kernel, two waves per SIMD, and nothing
   behind them; workgroup x reads entries x * pages_per_wave onward, one wave per KV head,
   heads_per_workgroup (1, 2 or 4, a divisor of the KV heads) of them in a workgroup.  `sink`:
   one device word that is never written in practice.  KVX_EINVAL for other formats. */
int kvx_calibrate_stream(const kvx_storage *storage, uint32_t layer, const uint64_t *page_table,
                         uint32_t n_pages, uint32_t pages_per_wave, uint32_t heads_per_workgroup,
                         uint32_t *sink, void *stream);

/* Forms that are not the decode kernel's shape, to tell what of its rate is the memory system's
   and what is its own.  All read the same bytes per page and KV head as the decode kernel (a 4 KiB
   key slab, a 4 KiB value slab, 128 B of each scale row; int4, head dimension 256).
     KVX_STREAM_COALESCED: the page list read with 16-byte loads only, every instruction a whole
       contiguous KiB, `depth` (1, 2 or 4) pages requested ahead per wave, one wave per (run of
       pages_per_wave pages, KV head); at most waves_per_simd (1, 2, 4 or 8) waves on a SIMD.
     KVX_STREAM_LINEAR: the page list is ignored; n_pages x KV heads x 8448 bytes are read from
       the start of the extent that holds page `layer` x extent_pages (one extent per launch, so
       that launches over `layer` = 0, 1, ... do not find each other's lines in a cache), each
       wave taking 4 KiB pieces in a row, pages_per_wave x 2 of them. */
#define KVX_STREAM_COALESCED 1u
#define KVX_STREAM_LINEAR 2u
int kvx_calibrate_stream_form(const kvx_storage *storage, uint32_t layer, const uint64_t *page_table,
                              uint32_t n_pages, uint32_t pages_per_wave, uint32_t form, uint32_t depth,
                              uint32_t waves_per_simd, uint32_t *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KVX_DEBUG_H */
