/*
 * emm_kv.h — C ABI of libemm_kv.so: the KV-cache data-movement path of ElasticMM
 * (pack / unpack / reshape_and_cache / copy_blocks / vision-row concat) as
 * hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions (all entry points):
 *   - returns 0 on success, a negative EMM_E* code on failure; the text of the
 *     last failure on the calling thread is available from emm_last_error();
 *   - every launch is asynchronous on `stream` (a hipStream_t passed as void*;
 *     NULL = the null stream). The library never synchronises;
 *   - the library takes no ownership: every device pointer must stay alive
 *     until the stream has run past the call;
 *   - `layer_ptrs` is a HOST array of `num_layers` DEVICE base pointers, one
 *     per layer tensor of the block pool (the reference pool is a Python list
 *     of separately allocated per-layer tensors, elasticmm/engine/v0/worker.py:388-394;
 *     a monolithic [L,2,NB,...] pool, elasticmm/engine/v0/nccl_transfer.py:215,
 *     is passed as base + l*layer_stride). The table is copied into the kernel
 *     argument block at launch, so the host array may be freed on return and
 *     nothing is allocated on the device. num_layers <= EMM_MAX_LAYERS per
 *     call (split larger models over several calls);
 *   - a layer tensor is [num_kv, num_blocks, chunk] contiguous, where
 *     chunk = block_size * num_kv_heads * head_dim elements is the contiguous
 *     unit of one block (layout [2, num_blocks, block_size, num_heads, head_size],
 *     elasticmm/engine/v0/worker.py:594);
 *   - block indices, slot mappings and block mappings are int64 DEVICE arrays.
 *     A negative block index marks padding and is skipped (the reference's
 *     fixed-size request convention, elasticmm/engine/v0/worker.py:924-925); an
 *     index >= num_blocks is never dereferenced (skipped), the Python layer
 *     raises IndexError for it before launch when indices arrive as a list;
 *   - no allocation, no global mutable state; re-entrant from any host thread
 *     (the only per-thread state is the text behind emm_last_error()).
 */
#ifndef EMM_KV_H
#define EMM_KV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EMM_KV_ABI_VERSION 3
#define EMM_MAX_LAYERS 96   /* layer pointers carried in one kernel argument block */
#define EMM_MAX_SEGMENTS 128 /* ragged segments carried by one emm_concat_rows launch */
#define EMM_MAX_INLINE_IDS 512 /* block ids carried by one launch of emm_kv_*_host_ids (longer tables: several launches) */

/* error codes */
#define EMM_OK 0
#define EMM_EINVAL (-1)  /* bad argument (null pointer, size, alignment, count) */
#define EMM_ELAUNCH (-2) /* hipLaunchKernel / hipGetLastError reported an error */

/* element types of the 16-bit side of the fp8 kernels */
#define EMM_DTYPE_BF16 0
#define EMM_DTYPE_F16 1
/* or-ed into the src_dtype of the fp8 appends: clamp the quotient to +-448 before the
 * cast (see emm_reshape_and_cache_fp8) */
#define EMM_FP8_SATURATE 0x100

typedef void *emm_stream_t; /* hipStream_t */

/* Text of the last error raised on the calling thread ("" if none). */
const char *emm_last_error(void);
/* EMM_KV_ABI_VERSION the library was built with. */
int emm_abi_version(void);

/*
 * pack — gather n scattered blocks of every layer (K and V) into one
 * contiguous transfer buffer `packed` of layout [num_layers, num_kv, n, chunk].
 * Replaces V0Worker.extract_kv_blocks (elasticmm/engine/v0/worker.py:578-610:
 * per-layer `layer_kv[:, idx]` followed by torch.stack), the per-layer gather
 * of p2p_send_kv / p2p_serve_kv (worker.py:676-682, :931-934; call with
 * num_layers = 1 or slice `packed` per layer) and the 6-D-pool gather of
 * V0NCCLTransferManager.transfer_kv_cache_blocks (nccl_transfer.py:241-247).
 * With num_kv = 1 it is the vision-block gather of nccl_transfer.py:329-332.
 */
int emm_kv_pack(const void *const *layer_ptrs, int num_layers, int num_kv,
                int64_t num_blocks, int64_t chunk_bytes,
                const int64_t *block_idx, int64_t n, void *packed,
                emm_stream_t stream);

/*
 * unpack — scatter `packed` [num_layers, num_kv, n, chunk] into the pool under
 * block table `block_idx` (unique entries). Replaces V0Worker.write_kv_blocks
 * (worker.py:612-633), the scatter half of p2p_recv_kv /
 * p2p_coordinated_transfer_kv / p2p_pull_kv (worker.py:715-722, :804-820,
 * :900-904) and the per-block loop of nccl_transfer.py:287-289 (:363-364 with
 * num_kv = 1).
 */
int emm_kv_unpack(void *const *layer_ptrs, int num_layers, int num_kv,
                  int64_t num_blocks, int64_t chunk_bytes,
                  const int64_t *block_idx, int64_t n, const void *packed,
                  emm_stream_t stream);

/*
 * pack / unpack with the block table given as a HOST array of n ids — the form in
 * which the reference holds a request's table (a Python
 * List[int] from V0BlockManager, elasticmm/engine/v0/block_manager.py:264-266,
 * passed to extract_kv_blocks / write_kv_blocks, worker.py:578, :612). The ids are
 * copied into the kernel argument block at launch: no device-side table, no
 * host-to-device copy, nothing to keep alive after the call returns, and the kernels
 * fetch an id with a scalar load from the argument block that the whole launch
 * shares (EMM_MAX_INLINE_IDS ids per launch; a longer table takes one launch per
 * EMM_MAX_INLINE_IDS ids). Same results as emm_kv_pack / emm_kv_unpack (negative and
 * too-large ids are skipped). A launch recorded into a HIP graph keeps the ids it was
 * recorded with.
 */
int emm_kv_pack_host_ids(const void *const *layer_ptrs, int num_layers, int num_kv,
                         int64_t num_blocks, int64_t chunk_bytes,
                         const int64_t *host_block_idx, int64_t n, void *packed,
                         emm_stream_t stream);
int emm_kv_unpack_host_ids(void *const *layer_ptrs, int num_layers, int num_kv,
                           int64_t num_blocks, int64_t chunk_bytes,
                           const int64_t *host_block_idx, int64_t n,
                           const void *packed, emm_stream_t stream);

/*
 * copy_blocks — for every layer and every pair p: pool[:, dst_p] = pool[:, src_p].
 * `block_mapping` is int64 [num_pairs, 2] row-major (src, dst), the argument
 * shape of vLLM's copy_blocks(kv_caches, block_mapping) that the reference
 * reaches through CacheEngine (worker.py:380); the in-reference analogue is
 * the src->dst block lists of migrate_instance (elasticmm/engine/v0/backend.py:674-708).
 * Destinations must be pairwise distinct and disjoint from the sources.
 */
int emm_copy_blocks(void *const *layer_ptrs, int num_layers, int num_kv,
                    int64_t num_blocks, int64_t chunk_bytes,
                    const int64_t *block_mapping, int64_t num_pairs,
                    emm_stream_t stream);

/*
 * migrate — pack and unpack fused for two pools on one device:
 * dst_pool[l][:, dst_idx[j]] = src_pool[l][:, src_idx[j]] without the staging
 * buffer. Same-device form of V0KVTransferManager.transfer_kv_cache
 * (elasticmm/engine/v0/kv_transfer.py:224-262). Both pools share num_kv and
 * chunk_bytes; block counts may differ.
 */
int emm_kv_migrate(const void *const *src_layer_ptrs, int64_t src_num_blocks,
                   void *const *dst_layer_ptrs, int64_t dst_num_blocks,
                   int num_layers, int num_kv, int64_t chunk_bytes,
                   const int64_t *src_idx, const int64_t *dst_idx, int64_t n,
                   emm_stream_t stream);

/*
 * dequant-unpack — scatter an fp8-e4m3fn transfer buffer
 * [num_layers, 2, n, chunk_elems] (bytes) into a 16-bit pool, converting
 * out = round_to_nearest_even_16bit(float(q) * scale), scale = k_scales[l] for
 * kv = 0 and v_scales[l] for kv = 1 (DEVICE float arrays of num_layers). NaN
 * bytes (0x7F / 0xFF) become the canonical quiet NaN (bf16 0x7FC0, f16 0x7E00).
 * No counterpart in the reference (its transfer rejects fp8,
 * worker.py:956-966); defined by the fp8 KV configuration of this build.
 */
int emm_kv_unpack_dequant_fp8(void *const *layer_ptrs, int num_layers,
                              int64_t num_blocks, int64_t chunk_elems,
                              const int64_t *block_idx, int64_t n,
                              const void *packed_fp8, const float *k_scales,
                              const float *v_scales, int out_dtype,
                              emm_stream_t stream);

/*
 * reshape_and_cache (flash layout) — append: for token t with
 * s = slot_mapping[t] >= 0: key_cache[s] = key[t], value_cache[s] = value[t],
 * rows of row_bytes = num_heads * head_size * elem_bytes; s < 0 (padding) and
 * s >= num_slots are skipped. The cache is addressed as [num_slots, row] with
 * num_slots = num_blocks * block_size (blocks contiguous). key/value rows are
 * `key_stride_bytes` / `value_stride_bytes` apart. Replaces vLLM's
 * reshape_and_cache_flash as reached from model_runner.execute_model
 * (elasticmm/engine/v0/worker_steps.py:281, :438) on the pool bound at
 * worker.py:408-412.
 */
int emm_reshape_and_cache(const void *key, const void *value, void *key_cache,
                          void *value_cache, const int64_t *slot_mapping,
                          int64_t num_tokens, int64_t row_bytes,
                          int64_t key_stride_bytes, int64_t value_stride_bytes,
                          int64_t num_slots, emm_stream_t stream);

/*
 * Same append for all layers of one step in a single launch: key_ptrs[l] /
 * value_ptrs[l] are that layer's [num_tokens, row] inputs, the cache pointers
 * that layer's K and V planes. HOST arrays of num_layers DEVICE pointers.
 * All layers share slot_mapping (one table per step, worker_steps.py:219-234).
 */
int emm_reshape_and_cache_layers(const void *const *key_ptrs,
                                 const void *const *value_ptrs,
                                 void *const *key_cache_ptrs,
                                 void *const *value_cache_ptrs, int num_layers,
                                 const int64_t *slot_mapping,
                                 int64_t num_tokens, int64_t row_bytes,
                                 int64_t key_stride_bytes,
                                 int64_t value_stride_bytes, int64_t num_slots,
                                 emm_stream_t stream);

/*
 * fp8 append — as emm_reshape_and_cache with a 16-bit source (src_dtype) and an
 * fp8-e4m3fn cache: q = e4m3fn_rne(float(x) / scale) with a correctly rounded
 * fp32 division, round-to-nearest-even, ties at 464 -> 448 and at 2^-10 -> 0.
 * Overflow follows src_dtype:
 *   EMM_DTYPE_BF16 / EMM_DTYPE_F16: |x/scale| >= 465, inf and NaN -> sign|0x7F (no
 *     saturation) — the rule of torch's (x.float() / scale).to(torch.float8_e4m3fn);
 *   the same or-ed with EMM_FP8_SATURATE: the quotient is clamped to [-448, 448]
 *     first, so overflow and +-inf give sign|0x7E and only NaN gives sign|0x7F —
 *     torch.clamp(x.float() / scale, -448, 448).to(torch.float8_e4m3fn), the
 *     convention of vLLM's fp8 KV cache (the cache_dtype the reference leaves open
 *     at elasticmm/engine/v0/worker.py:194). Never the default.
 * scale must be finite and non-zero. k_scale / v_scale are DEVICE pointers to one
 * float each (per-layer per-tensor scale). Strides in elements.
 */
int emm_reshape_and_cache_fp8(const void *key, const void *value,
                              void *key_cache, void *value_cache,
                              const int64_t *slot_mapping, int64_t num_tokens,
                              int64_t row_elems, int64_t key_stride_elems,
                              int64_t value_stride_elems, int64_t num_slots,
                              const float *k_scale, const float *v_scale,
                              int src_dtype, emm_stream_t stream);

/* fp8 append for all layers in one launch; k_scales / v_scales are DEVICE
 * float arrays of num_layers. */
int emm_reshape_and_cache_fp8_layers(const void *const *key_ptrs,
                                     const void *const *value_ptrs,
                                     void *const *key_cache_ptrs,
                                     void *const *value_cache_ptrs,
                                     int num_layers,
                                     const int64_t *slot_mapping,
                                     int64_t num_tokens, int64_t row_elems,
                                     int64_t key_stride_elems,
                                     int64_t value_stride_elems,
                                     int64_t num_slots, const float *k_scales,
                                     const float *v_scales, int src_dtype,
                                     emm_stream_t stream);

/*
 * reshape_and_cache (flash layout, free cache strides) — the same append for a
 * cache whose blocks, slots and heads are block_stride / page_stride /
 * head_stride bytes apart, e.g. the head-major pool
 * [num_blocks, num_heads, block_size, head_size] that vLLM passes to
 * reshape_and_cache_flash as a permuted view: head h of token t goes to
 * cache + b * block_stride + o * page_stride + h * head_stride with
 * b, o = divmod(slot_mapping[t], block_size); head rows (head_bytes) stay
 * contiguous. One launch for num_layers layers (HOST pointer tables as in
 * emm_reshape_and_cache_layers; all layers share the geometry). Same-width
 * copy only (emm_reshape_and_cache_strided_fp8 quantises). Same call sites as emm_reshape_and_cache
 * (elasticmm/engine/v0/worker_steps.py:281, :438).
 */
int emm_reshape_and_cache_strided(const void *const *key_ptrs,
                                  const void *const *value_ptrs,
                                  void *const *key_cache_ptrs,
                                  void *const *value_cache_ptrs, int num_layers,
                                  const int64_t *slot_mapping,
                                  int64_t num_tokens, int num_heads,
                                  int64_t head_bytes, int block_size,
                                  int64_t num_blocks, int64_t key_stride_bytes,
                                  int64_t value_stride_bytes,
                                  int64_t block_stride_bytes,
                                  int64_t page_stride_bytes,
                                  int64_t head_stride_bytes,
                                  emm_stream_t stream);

/*
 * reshape_and_cache (flash layout, free cache strides, fp8-e4m3fn cache) — the
 * quantising append of emm_reshape_and_cache_fp8 for the strided caches of
 * emm_reshape_and_cache_strided: a 1-byte cache whose blocks, slots and heads are
 * block_stride / page_stride / head_stride bytes apart (an fp8 pool in the
 * head-major layout [num_blocks, num_heads, block_size, head_size] passed as a
 * permuted view). Element d of head h of token t goes to
 * cache + b * block_stride + o * page_stride + h * head_stride + d as
 * e4m3fn(float(x) / scale), same rounding and overflow modes as
 * emm_reshape_and_cache_fp8 (src_dtype: EMM_DTYPE_BF16 / EMM_DTYPE_F16, optionally
 * | EMM_FP8_SATURATE). key / value strides in source elements; k_scales / v_scales
 * are DEVICE float arrays of num_layers. One launch for num_layers layers (HOST
 * pointer tables; all layers share the geometry). The cache dtype the reference
 * leaves open at elasticmm/engine/v0/worker.py:194, reached from
 * elasticmm/engine/v0/worker_steps.py:281, :438.
 */
int emm_reshape_and_cache_strided_fp8(const void *const *key_ptrs,
                                      const void *const *value_ptrs,
                                      void *const *key_cache_ptrs,
                                      void *const *value_cache_ptrs,
                                      int num_layers,
                                      const int64_t *slot_mapping,
                                      int64_t num_tokens, int num_heads,
                                      int64_t head_elems, int block_size,
                                      int64_t num_blocks,
                                      int64_t key_stride_elems,
                                      int64_t value_stride_elems,
                                      int64_t block_stride_bytes,
                                      int64_t page_stride_bytes,
                                      int64_t head_stride_bytes,
                                      const float *k_scales,
                                      const float *v_scales, int src_dtype,
                                      emm_stream_t stream);

/*
 * reshape_and_cache (paged-attention layout) — append into the transposed pool
 * of vLLM's PagedAttention backends:
 *   key_cache   [num_blocks, num_heads, head_size / x, block_size, x]
 *   value_cache [num_blocks, num_heads, head_size, block_size]
 * with x = 16 / cache_elem_bytes (8 for a 16-bit cache, 16 for fp8). For token t
 * with s = slot_mapping[t], b = s / block_size, o = s % block_size:
 *   key_cache[b, h, d / x, o, d % x] = key[t, h, d]
 *   value_cache[b, h, d, o]          = value[t, h, d]
 * s < 0 and s >= num_blocks * block_size are skipped. cache_elem_bytes = 2 copies
 * bits (any 16-bit type); cache_elem_bytes = 1 quantises to e4m3fn with the rule of
 * emm_reshape_and_cache_fp8 (k_scale / v_scale: DEVICE pointers to one float each,
 * ignored for a 16-bit cache). Strides in elements. This is vLLM's
 * reshape_and_cache(key, value, key_cache, value_cache, slot_mapping,
 * kv_cache_dtype, k_scale, v_scale), the append that
 * elasticmm/engine/v0/worker_steps.py:281, :438 reaches when vLLM selects a
 * PagedAttention backend (its default on ROCm) instead of flash-attn; the pool
 * bound at worker.py:408-412 is then [2, num_blocks, block_size * H * D] per layer,
 * which pack / unpack / copy_blocks move unchanged (one block is still one chunk).
 * Limits: num_tokens and num_heads * head_size below 2^31, token strides below 2^32
 * elements (EMM_EINVAL otherwise).
 */
int emm_reshape_and_cache_paged(const void *key, const void *value,
                                void *key_cache, void *value_cache,
                                const int64_t *slot_mapping, int64_t num_tokens,
                                int num_heads, int head_size, int block_size,
                                int64_t num_blocks, int64_t key_stride_elems,
                                int64_t value_stride_elems, int src_dtype,
                                int cache_elem_bytes, const float *k_scale,
                                const float *v_scale, emm_stream_t stream);

/* Paged-layout append for all layers of one step in a single launch (pointer
 * tables as in emm_reshape_and_cache_layers; k_scales / v_scales: DEVICE float
 * arrays of num_layers, fp8 caches only). */
int emm_reshape_and_cache_paged_layers(const void *const *key_ptrs,
                                       const void *const *value_ptrs,
                                       void *const *key_cache_ptrs,
                                       void *const *value_cache_ptrs,
                                       int num_layers,
                                       const int64_t *slot_mapping,
                                       int64_t num_tokens, int num_heads,
                                       int head_size, int block_size,
                                       int64_t num_blocks,
                                       int64_t key_stride_elems,
                                       int64_t value_stride_elems,
                                       int src_dtype, int cache_elem_bytes,
                                       const float *k_scales,
                                       const float *v_scales,
                                       emm_stream_t stream);

/*
 * concat_rows — copy n ragged segments back to back into `dst`: segment i is
 * nbytes[i] bytes at srcs[i]. HOST arrays (n <= EMM_MAX_SEGMENTS per call;
 * `dst_offset_bytes` lets the caller continue a longer list). Replaces
 * torch.cat(vision_embeds, dim=0) of elasticmm/engine/v0/worker_steps.py:264-267
 * on the tensors held by V0Worker.ve_cache (worker.py:1007-1036).
 */
int emm_concat_rows(const void *const *srcs, const int64_t *nbytes, int n,
                    void *dst, int64_t dst_offset_bytes, emm_stream_t stream);

/*
 * Plain device-to-device copy with the same tile engine as pack/unpack: the
 * yardstick the block-move kernels are compared with (no indirection).
 */
int emm_stream_copy(const void *src, void *dst, int64_t nbytes,
                    emm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* EMM_KV_H */
