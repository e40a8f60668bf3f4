/*
 * emm_kv_hooks.h — entry points that exist only in libemm_kv_hooks.so, the build of
 * emm_kv.hip with -DEMM_BENCH_HOOKS used by bench.py and the GPU tests. The product
 * library libemm_kv.so (include/emm_kv.h) exports none of them and carries no
 * run-time switch. The hooks library also exports the whole product ABI, so a
 * benchmark can route its calls through it and select launch variants.
 */
#ifndef EMM_KV_HOOKS_H
#define EMM_KV_HOOKS_H

#include <stdint.h>

#include "emm_kv.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Launch variants of the hooks library's own kernels: 0 = the product's defaults.
 * bits 8-11: 1 = non-temporal stores in the 16-byte block moves (default: sc0 sc1);
 * bits 12-15: shape of the 16-byte copy append (token rows per wave, waves per workgroup):
 *   0 = default ((4, 1) for a per-layer launch, (1, 1) for a whole-step launch), 1 = (1, 4), 2 = (2, 4),
 *   3 = (4, 1), 4 = (1, 1), 5 = (2, 1); for the fp8 append the same bits read: bit 12 = waves that convert a whole
 *   row, bit 13 = waves that convert 512 elements (0 = by launch size);
 * bits 16-19: log2 of the blocks per plane visit of pack / unpack (15 = plain order);
 * bits 20-21: token tile of the paged-layout append (1 = 16 tokens, 2 = 4 tokens; 0 = by token count);
 * bits 22-23: row elements per workgroup of a one-layer paged-layout append (1 = 256, 2 = 128; 0 = by launch size);
 * bit 24: fp8 append with the IEEE division instead of the reciprocal form;
 * bits 25 / 26 / 27: tile-to-XCD mapping of the block moves forced to plain / whole chunks per XCD / pairs of tiles
 *   per XCD (default: chosen per launch by kind, table length, tiles per chunk and plane size);
 * bit 28: the paged-layout append always through the general kernel (256-thread workgroups, block barrier) instead of
 *   the kernel of one-wave workgroups that the usual shapes take;
 * bits 29-30: column width of the one-wave paged-layout append (1 = 128 row elements, 2 = 32, 3 = 256; 0 = by launch
 *   size); with it bits 20-21: 1 = K and V of a column in one wave, 2 = in two waves (0 = by launch size).
 * Process-wide, not thread-safe. Returns the previous value. */
int emm_hook_set_move_variant(int variant);

/* Memory-system yardsticks with the grid of pack / unpack (one 4 KiB tile per workgroup):
 * sequential kinds touch `linear` [num_layers * num_kv, n, chunk]; pool kinds touch the
 * n blocks block_idx[] of every plane of the pool. Reads write nothing (sink may be null). */
#define EMM_PROBE_SEQ_READ 0
#define EMM_PROBE_SEQ_WRITE 1
#define EMM_PROBE_GATHER_READ 2
#define EMM_PROBE_SCATTER_WRITE 3
/* what the block-id fetch costs: the gathered read and a whole pack (gathered read + sequential write to
 * `linear`) with block ids computed from the block's position instead of fetched, and the pack with fetched
 * ids through the same probe kernel */
#define EMM_PROBE_GATHER_READ_COMPUTED_IDS 4
#define EMM_PROBE_PACK_COMPUTED_IDS 5
#define EMM_PROBE_PACK 6
/* the pack with computed ids and computed plane bases (pool in one allocation): no scalar load before the data */
#define EMM_PROBE_PACK_NOTHING_FETCHED 7
int emm_hook_probe(int kind, void *const *layer_ptrs, int num_layers, int num_kv, int64_t num_blocks,
                   int64_t chunk_bytes, const int64_t *block_idx, int64_t n, void *linear, uint32_t *sink,
                   emm_stream_t stream);

/* The pack (device table, whole call in one launch) through another kernel shape, so that the product's choice — one
 * 16-byte load and one 16-byte store per lane, a 4 KiB tile per 256-thread workgroup — can be re-measured against:
 * two tiles per workgroup with both loads in flight before the first store; four tiles (a whole 16 KiB chunk) per
 * workgroup; loads straight into LDS (global_load_lds_dwordx4) with 4 KiB per one-wave workgroup, 4 x 4 KiB per
 * four-wave workgroup, 8 KiB per one-wave workgroup; loader waves and storer waves split inside a workgroup
 * (double-buffered LDS, one barrier per 8 KiB step). Same result as emm_kv_pack. n <= 65535; chunk_bytes a
 * multiple of the variant's piece (8 KiB: U2, LDS_8K, SPLIT; 4 KiB: LDS_1W; 16 KiB: CHUNK, LDS_4W). */
#define EMM_PACK_VARIANT_U2 1
#define EMM_PACK_VARIANT_CHUNK 2
#define EMM_PACK_VARIANT_LDS_1W 3
#define EMM_PACK_VARIANT_LDS_4W 4
#define EMM_PACK_VARIANT_LDS_8K 5
#define EMM_PACK_VARIANT_SPLIT 6
int emm_hook_pack_variant(int variant, const void *const *layer_ptrs, int num_layers, int num_kv, int64_t num_blocks,
                          int64_t chunk_bytes, const int64_t *block_idx, int64_t n, void *packed, emm_stream_t stream);

/* Launch a kernel that does nothing (one wave): a chain of these in a HIP graph measures the cost of a
 * dependent launch by itself, the floor under every per-layer launch. */
int emm_hook_empty_launch(emm_stream_t stream);

/* Exhaustive check of the fp8 append's reciprocal-form quotient: for x = +-1.m * 2^x_exp over all
 * 2^10 ten-bit m and scale = 1.f * 2^s_exp for f in [s_begin, s_end) (23-bit significand fields),
 * compare with the IEEE division. counters (DEVICE, 5 x uint64, zeroed by the caller):
 * [0] differing fp32 quotients (where the division gives a normal number), [1] differing e4m3fn
 * bytes in torch mode, [2] in saturating mode, [3] pairs checked, [4] one differing pair
 * (x bits << 32 | scale bits). */
int emm_hook_fp8_quotient_sweep(int x_exp, int s_exp, uint32_t s_begin, uint32_t s_end, uint64_t *counters,
                                emm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* EMM_KV_HOOKS_H */
