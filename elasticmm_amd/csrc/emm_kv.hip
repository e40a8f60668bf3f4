// libemm_kv — KV-cache data-movement kernels for gfx950 (MI355X) behind the C ABI
// declared in include/emm_kv.h.
//
// Everything here is HBM-bandwidth work. The shape every kernel follows was found
// by measurement on MI355X: a 256-thread workgroup moves one 4 KiB tile, each lane
// issues ONE 16-byte non-temporal load and ONE 16-byte store, every wave
// instruction covers 1 KiB of contiguous memory, and stores are system-scope
// write-through (sc0 sc1). Unrolled or persistent variants are slower on this part
// (the memory counter of gfx9 retires loads and stores in order, so a lane that
// loads after it has stored waits for a write acknowledgement). Block-table and
// slot-mapping entries are wave-uniform: they are fetched once per wave and all
// address arithmetic that depends on them stays in scalar registers; loads that do
// not depend on them are issued before they are waited for.
//
// Pool layout (per layer): [num_kv, num_blocks, chunk] contiguous, where
// chunk = block_size * num_kv_heads * head_dim elements.
// Transfer-buffer layout: [num_layers, num_kv, n, chunk] contiguous.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <string.h>
#include <type_traits>

#include "emm_kv.h"

// The kernels and their host-side launch code, one file per family (all in this translation unit):
#include "emm_common.inc"
#include "emm_block_move.inc"
#include "emm_fp8.inc"
#include "emm_append.inc"
#include "emm_append_paged.inc"
#include "emm_concat.inc"

// ============================================================================
// C ABI
// ============================================================================
extern "C" {

const char *emm_last_error(void) { return g_last_error; }
int emm_abi_version(void) { return EMM_KV_ABI_VERSION; }

int emm_kv_pack(const void *const *layer_ptrs, int num_layers, int num_kv,
                int64_t num_blocks, int64_t chunk_bytes, const int64_t *block_idx,
                int64_t n, void *packed, emm_stream_t stream) {
  int rc = check_pool_args("emm_kv_pack", layer_ptrs, num_layers, num_kv, num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!block_idx || !packed) return fail(EMM_EINVAL, "emm_kv_pack: null block_idx / packed");
  return move_planes<kPack>(layer_ptrs, num_blocks, nullptr, 0, num_layers, num_kv, chunk_bytes,
                            block_idx, nullptr, false, n, packed, as_stream(stream), "emm_kv_pack");
}

int emm_kv_unpack(void *const *layer_ptrs, int num_layers, int num_kv,
                  int64_t num_blocks, int64_t chunk_bytes, const int64_t *block_idx,
                  int64_t n, const void *packed, emm_stream_t stream) {
  int rc = check_pool_args("emm_kv_unpack", (const void *const *)layer_ptrs, num_layers, num_kv,
                           num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!block_idx || !packed) return fail(EMM_EINVAL, "emm_kv_unpack: null block_idx / packed");
  return move_planes<kUnpack>(nullptr, 0, layer_ptrs, num_blocks, num_layers, num_kv, chunk_bytes,
                              nullptr, block_idx, false, n, packed, as_stream(stream), "emm_kv_unpack");
}

int emm_kv_pack_host_ids(const void *const *layer_ptrs, int num_layers, int num_kv,
                         int64_t num_blocks, int64_t chunk_bytes, const int64_t *host_block_idx,
                         int64_t n, void *packed, emm_stream_t stream) {
  const char *what = "emm_kv_pack_host_ids";
  int rc = check_pool_args(what, layer_ptrs, num_layers, num_kv, num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!host_block_idx || !packed) return fail(EMM_EINVAL, "%s: null host_block_idx / packed", what);
  return move_planes<kPack>(layer_ptrs, num_blocks, nullptr, 0, num_layers, num_kv, chunk_bytes,
                            nullptr, nullptr, false, n, packed, as_stream(stream), what, host_block_idx);
}

int emm_kv_unpack_host_ids(void *const *layer_ptrs, int num_layers, int num_kv,
                           int64_t num_blocks, int64_t chunk_bytes, const int64_t *host_block_idx,
                           int64_t n, const void *packed, emm_stream_t stream) {
  const char *what = "emm_kv_unpack_host_ids";
  int rc = check_pool_args(what, (const void *const *)layer_ptrs, num_layers, num_kv, num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!host_block_idx || !packed) return fail(EMM_EINVAL, "%s: null host_block_idx / packed", what);
  return move_planes<kUnpack>(nullptr, 0, layer_ptrs, num_blocks, num_layers, num_kv, chunk_bytes,
                              nullptr, nullptr, false, n, packed, as_stream(stream), what, host_block_idx);
}

int emm_copy_blocks(void *const *layer_ptrs, int num_layers, int num_kv,
                    int64_t num_blocks, int64_t chunk_bytes,
                    const int64_t *block_mapping, int64_t num_pairs, emm_stream_t stream) {
  int rc = check_pool_args("emm_copy_blocks", (const void *const *)layer_ptrs, num_layers, num_kv,
                           num_blocks, chunk_bytes, num_pairs);
  if (rc != EMM_OK) return rc;
  if (num_pairs == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!block_mapping) return fail(EMM_EINVAL, "emm_copy_blocks: null block_mapping");
  return move_planes<kPoolToPool>((const void *const *)layer_ptrs, num_blocks, layer_ptrs, num_blocks,
                                  num_layers, num_kv, chunk_bytes, block_mapping, nullptr, true,
                                  num_pairs, nullptr, as_stream(stream), "emm_copy_blocks");
}

int emm_kv_migrate(const void *const *src_layer_ptrs, int64_t src_num_blocks,
                   void *const *dst_layer_ptrs, int64_t dst_num_blocks, int num_layers,
                   int num_kv, int64_t chunk_bytes, const int64_t *src_idx,
                   const int64_t *dst_idx, int64_t n, emm_stream_t stream) {
  int rc = check_pool_args("emm_kv_migrate", src_layer_ptrs, num_layers, num_kv, src_num_blocks,
                           chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  rc = check_pool_args("emm_kv_migrate", (const void *const *)dst_layer_ptrs, num_layers, num_kv,
                       dst_num_blocks, chunk_bytes, n);
  if (rc != EMM_OK) return rc;
  if (n == 0 || num_layers == 0 || num_kv == 0 || chunk_bytes == 0) return EMM_OK;
  if (!src_idx || !dst_idx) return fail(EMM_EINVAL, "emm_kv_migrate: null index array");
  return move_planes<kPoolToPool>(src_layer_ptrs, src_num_blocks, dst_layer_ptrs, dst_num_blocks,
                                  num_layers, num_kv, chunk_bytes, src_idx, dst_idx, false, n, nullptr,
                                  as_stream(stream), "emm_kv_migrate");
}

int emm_stream_copy(const void *src, void *dst, int64_t nbytes, emm_stream_t stream) {
  if (nbytes < 0) return fail(EMM_EINVAL, "emm_stream_copy: negative size");
  if (nbytes == 0) return EMM_OK;
  if (!src || !dst) return fail(EMM_EINVAL, "emm_stream_copy: null pointer");
  int vec = common_align(common_align(16, src), dst);
  while (vec > 1 && nbytes % vec) vec >>= 1;
  if (vec == 8) vec = 4;
  const int64_t tile = (int64_t)(vec == 16 ? 1 : 4) * kThreads * vec;
  const int64_t tiles = (nbytes + tile - 1) / tile;
  if (tiles > 0x7fffffffLL) return fail(EMM_EINVAL, "emm_stream_copy: %lld bytes need too many tiles", (long long)nbytes);
  const dim3 grid((uint32_t)tiles);
  hipStream_t s = as_stream(stream);
  const char *a = (const char *)src;
  char *b = (char *)dst;
  switch (vec) {
  case 16: emm_stream_copy_kernel<u32x4, 1, 1><<<grid, kThreads, 0, s>>>(a, b, nbytes); break;
  case 4: emm_stream_copy_kernel<uint32_t, 4, 0><<<grid, kThreads, 0, s>>>(a, b, nbytes); break;
  case 2: emm_stream_copy_kernel<uint16_t, 4, 0><<<grid, kThreads, 0, s>>>(a, b, nbytes); break;
  default: emm_stream_copy_kernel<uint8_t, 4, 0><<<grid, kThreads, 0, s>>>(a, b, nbytes); break;
  }
  return check_launch("emm_stream_copy");
}

int emm_kv_unpack_dequant_fp8(void *const *layer_ptrs, int num_layers, int64_t num_blocks,
                              int64_t chunk_elems, const int64_t *block_idx, int64_t n,
                              const void *packed_fp8, const float *k_scales,
                              const float *v_scales, int out_dtype, emm_stream_t stream) {
  const char *what = "emm_kv_unpack_dequant_fp8";
  int rc = check_pool_args(what, (const void *const *)layer_ptrs, num_layers, 2, num_blocks,
                           chunk_elems, n);
  if (rc != EMM_OK) return rc;
  if (out_dtype != EMM_DTYPE_BF16 && out_dtype != EMM_DTYPE_F16)
    return fail(EMM_EINVAL, "%s: unknown out_dtype %d", what, out_dtype);
  if (n == 0 || num_layers == 0 || chunk_elems == 0) return EMM_OK;
  if (!block_idx || !packed_fp8 || !k_scales || !v_scales)
    return fail(EMM_EINVAL, "%s: null pointer argument", what);
  if (chunk_elems % 16 != 0 || !aligned(packed_fp8, 16))
    return fail(EMM_EINVAL, "%s: chunk_elems (%lld) and packed_fp8 must be multiples of 16",
                what, (long long)chunk_elems);
  if (chunk_elems > 0x3fffffffLL || num_blocks > 0x7fffffffLL)
    return fail(EMM_EINVAL, "%s: chunk_elems / num_blocks too large", what);
  LayerTable t;
  for (int l = 0; l < num_layers; ++l) {
    if (!aligned(layer_ptrs[l], 16))
      return fail(EMM_EINVAL, "%s: layer_ptrs[%d] not 16-byte aligned", what, l);
    t.base[l] = (char *)layer_ptrs[l];
  }
  const int64_t tile = (int64_t)kThreads * 16;
  const int64_t tpc = (chunk_elems + tile - 1) / tile;
  hipStream_t s = as_stream(stream);
  for (int64_t j0 = 0; j0 < n; j0 += kMaxGridY) {
    const int64_t ny = (n - j0 < kMaxGridY) ? (n - j0) : kMaxGridY;
    const char *packed = (const char *)packed_fp8 + j0 * chunk_elems;
    const int64_t *idx = block_idx + j0;
    const int64_t stride = n * chunk_elems;
    const bool grouped = ny >= 1024 && ((2 * num_layers) << 8) <= kMaxGridY; // groups of 256 blocks, as in unpack
    const uint32_t remap = xcd_mapping(kMapDequant, ny, tpc, num_blocks, 2 * chunk_elems);
    const dim3 grid = grouped ? dim3((uint32_t)tpc, (uint32_t)((2 * num_layers) << 8), (uint32_t)((ny + 255) >> 8))
                              : dim3((uint32_t)tpc, (uint32_t)ny, (uint32_t)(2 * num_layers));
#define EMM_DQ_LAUNCH(DT, G) \
  emm_unpack_dequant_fp8_kernel<DT, G><<<grid, kThreads, 0, s>>>(packed, idx, k_scales, v_scales, stride, \
      (uint32_t)chunk_elems, (uint32_t)num_blocks, (uint32_t)ny, 8u | remap, t)
    if (out_dtype == EMM_DTYPE_BF16) { if (grouped) EMM_DQ_LAUNCH(EMM_DTYPE_BF16, true); else EMM_DQ_LAUNCH(EMM_DTYPE_BF16, false); }
    else { if (grouped) EMM_DQ_LAUNCH(EMM_DTYPE_F16, true); else EMM_DQ_LAUNCH(EMM_DTYPE_F16, false); }
#undef EMM_DQ_LAUNCH
    const int rc2 = check_launch(what);
    if (rc2 != EMM_OK) return rc2;
  }
  return EMM_OK;
}

int emm_reshape_and_cache(const void *key, const void *value, void *key_cache,
                          void *value_cache, const int64_t *slot_mapping,
                          int64_t num_tokens, int64_t row_bytes, int64_t key_stride_bytes,
                          int64_t value_stride_bytes, int64_t num_slots, emm_stream_t stream) {
  return append_copy(&key, &value, &key_cache, &value_cache, 1, slot_mapping, num_tokens,
                     row_bytes, key_stride_bytes, value_stride_bytes, num_slots, false,
                     as_stream(stream), "emm_reshape_and_cache");
}

int emm_reshape_and_cache_layers(const void *const *key_ptrs, const void *const *value_ptrs,
                                 void *const *key_cache_ptrs, void *const *value_cache_ptrs,
                                 int num_layers, const int64_t *slot_mapping,
                                 int64_t num_tokens, int64_t row_bytes,
                                 int64_t key_stride_bytes, int64_t value_stride_bytes,
                                 int64_t num_slots, emm_stream_t stream) {
  return append_copy(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers,
                     slot_mapping, num_tokens, row_bytes, key_stride_bytes, value_stride_bytes,
                     num_slots, true, as_stream(stream), "emm_reshape_and_cache_layers");
}

int emm_reshape_and_cache_fp8(const void *key, const void *value, void *key_cache,
                              void *value_cache, const int64_t *slot_mapping,
                              int64_t num_tokens, int64_t row_elems, int64_t key_stride_elems,
                              int64_t value_stride_elems, int64_t num_slots,
                              const float *k_scale, const float *v_scale, int src_dtype,
                              emm_stream_t stream) {
  return append_fp8(&key, &value, &key_cache, &value_cache, 1, slot_mapping, num_tokens,
                    row_elems, key_stride_elems, value_stride_elems, num_slots, k_scale, v_scale,
                    src_dtype, false, as_stream(stream), "emm_reshape_and_cache_fp8");
}

int emm_reshape_and_cache_fp8_layers(const void *const *key_ptrs, const void *const *value_ptrs,
                                     void *const *key_cache_ptrs, void *const *value_cache_ptrs,
                                     int num_layers, const int64_t *slot_mapping,
                                     int64_t num_tokens, int64_t row_elems,
                                     int64_t key_stride_elems, int64_t value_stride_elems,
                                     int64_t num_slots, const float *k_scales,
                                     const float *v_scales, int src_dtype, emm_stream_t stream) {
  return append_fp8(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers,
                    slot_mapping, num_tokens, row_elems, key_stride_elems, value_stride_elems,
                    num_slots, k_scales, v_scales, src_dtype, true, as_stream(stream),
                    "emm_reshape_and_cache_fp8_layers");
}

int emm_reshape_and_cache_strided(const void *const *key_ptrs, const void *const *value_ptrs,
                                  void *const *key_cache_ptrs, void *const *value_cache_ptrs,
                                  int num_layers, const int64_t *slot_mapping, int64_t num_tokens,
                                  int num_heads, int64_t head_bytes, int block_size, int64_t num_blocks,
                                  int64_t key_stride_bytes, int64_t value_stride_bytes,
                                  int64_t block_stride_bytes, int64_t page_stride_bytes,
                                  int64_t head_stride_bytes, emm_stream_t stream) {
  return append_strided(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers, slot_mapping,
                        num_tokens, num_heads, head_bytes, block_size, num_blocks, key_stride_bytes,
                        value_stride_bytes, block_stride_bytes, page_stride_bytes, head_stride_bytes,
                        as_stream(stream), "emm_reshape_and_cache_strided");
}

int emm_reshape_and_cache_strided_fp8(const void *const *key_ptrs, const void *const *value_ptrs,
                                      void *const *key_cache_ptrs, void *const *value_cache_ptrs, int num_layers,
                                      const int64_t *slot_mapping, int64_t num_tokens, int num_heads,
                                      int64_t head_elems, int block_size, int64_t num_blocks,
                                      int64_t key_stride_elems, int64_t value_stride_elems,
                                      int64_t block_stride_bytes, int64_t page_stride_bytes,
                                      int64_t head_stride_bytes, const float *k_scales, const float *v_scales,
                                      int src_dtype, emm_stream_t stream) {
  return append_strided_fp8(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers, slot_mapping,
                            num_tokens, num_heads, head_elems, block_size, num_blocks, key_stride_elems,
                            value_stride_elems, block_stride_bytes, page_stride_bytes, head_stride_bytes, k_scales,
                            v_scales, src_dtype, as_stream(stream), "emm_reshape_and_cache_strided_fp8");
}

int emm_reshape_and_cache_paged(const void *key, const void *value, void *key_cache, void *value_cache,
                                const int64_t *slot_mapping, int64_t num_tokens, int num_heads,
                                int head_size, int block_size, int64_t num_blocks,
                                int64_t key_stride_elems, int64_t value_stride_elems, int src_dtype,
                                int cache_elem_bytes, const float *k_scale, const float *v_scale,
                                emm_stream_t stream) {
  return append_paged(&key, &value, &key_cache, &value_cache, 1, slot_mapping, num_tokens, num_heads,
                      head_size, block_size, num_blocks, key_stride_elems, value_stride_elems, src_dtype,
                      cache_elem_bytes, k_scale, v_scale, as_stream(stream), "emm_reshape_and_cache_paged");
}

int emm_reshape_and_cache_paged_layers(const void *const *key_ptrs, const void *const *value_ptrs,
                                       void *const *key_cache_ptrs, void *const *value_cache_ptrs,
                                       int num_layers, const int64_t *slot_mapping, int64_t num_tokens,
                                       int num_heads, int head_size, int block_size, int64_t num_blocks,
                                       int64_t key_stride_elems, int64_t value_stride_elems,
                                       int src_dtype, int cache_elem_bytes, const float *k_scales,
                                       const float *v_scales, emm_stream_t stream) {
  return append_paged(key_ptrs, value_ptrs, key_cache_ptrs, value_cache_ptrs, num_layers, slot_mapping,
                      num_tokens, num_heads, head_size, block_size, num_blocks, key_stride_elems,
                      value_stride_elems, src_dtype, cache_elem_bytes, k_scales, v_scales, as_stream(stream),
                      "emm_reshape_and_cache_paged_layers");
}

int emm_concat_rows(const void *const *srcs, const int64_t *nbytes, int n, void *dst,
                    int64_t dst_offset_bytes, emm_stream_t stream) {
  const char *what = "emm_concat_rows";
  if (n < 0 || n > EMM_MAX_SEGMENTS)
    return fail(EMM_EINVAL, "%s: n=%d outside [0, %d]", what, n, EMM_MAX_SEGMENTS);
  if (n == 0) return EMM_OK;
  if (!srcs || !nbytes || !dst || dst_offset_bytes < 0)
    return fail(EMM_EINVAL, "%s: null pointer / negative offset", what);
  ConcatParams p;
  memset(&p, 0, sizeof(p));
  int al = common_align(16, (const char *)dst + dst_offset_bytes);
  int64_t off = dst_offset_bytes;
  int m = 0;
  for (int i = 0; i < n; ++i) {
    if (nbytes[i] < 0) return fail(EMM_EINVAL, "%s: nbytes[%d] negative", what, i);
    if (nbytes[i] == 0) continue;
    if (!srcs[i]) return fail(EMM_EINVAL, "%s: srcs[%d] is null", what, i);
    p.src[m] = (const char *)srcs[i];
    p.dst_off[m] = off;
    p.nbytes[m] = nbytes[i];
    al = common_align(al, srcs[i]);
    while (al > 1 && (off % al || nbytes[i] % al)) al >>= 1;
    off += nbytes[i];
    ++m;
  }
  if (m == 0) return EMM_OK;
  if (al == 8) al = 4;
  // 16-byte lanes: one vector per lane (4 KiB tiles); narrower lanes: four
  const int unroll = al == 16 ? 1 : 4;
  const int64_t tile = (int64_t)unroll * kThreads * al;
  uint64_t tiles = 0;
  for (int i = 0; i < EMM_MAX_SEGMENTS; ++i) p.tile_start[i] = 0xffffffffu;
  for (int i = 0; i < m; ++i) {
    p.tile_start[i] = (uint32_t)tiles;
    tiles += (uint64_t)((p.nbytes[i] + tile - 1) / tile);
    if (tiles > 0x7fffffffULL) return fail(EMM_EINVAL, "%s: grid too large", what);
  }
  for (int g = 0; g < kSegGroups; ++g) p.group_start[g] = p.tile_start[g * kSegGroup];
  p.dst = (char *)dst;
  dim3 grid((uint32_t)tiles);
  hipStream_t s = as_stream(stream);
  switch (al) {
  case 16: emm_concat_rows_kernel<u32x4, 1><<<grid, kThreads, 0, s>>>(p); break;
  case 4: emm_concat_rows_kernel<uint32_t, 4><<<grid, kThreads, 0, s>>>(p); break;
  case 2: emm_concat_rows_kernel<uint16_t, 4><<<grid, kThreads, 0, s>>>(p); break;
  default: emm_concat_rows_kernel<uint8_t, 4><<<grid, kThreads, 0, s>>>(p); break;
  }
  return check_launch(what);
}

} // extern "C"

// ============================================================================
// Benchmark / test hooks (libemm_kv_hooks.so only)
// ============================================================================
#ifdef EMM_BENCH_HOOKS
#include "emm_kv_hooks.h"
#include "emm_kv_hooks.inc"
#endif // EMM_BENCH_HOOKS
