/*
 * A C program (no Python, no torch) that drives libemm_kv.so through include/emm_kv.h and checks
 * every data-moving entry point (pack, unpack, their host-table forms, copy_blocks, migrate, the appends in the
 * flash, strided and paged layouts, 16-bit and fp8, per layer and for all layers, the dequantising unpack,
 * concat_rows, the plain copy) against the loops of oracle/kv_oracle.c on seeded data. Built and run by tests/test_c_abi_program.py.
 *
 *   gcc -std=c11 -O2 -D__HIP_PLATFORM_AMD__ -Iinclude -I/opt/rocm/include -o tests/c_abi/c_abi_check \
 *       tests/c_abi/c_abi_check.c oracle/kv_oracle.c -Lelasticmm_amd -lemm_kv -L/opt/rocm/lib -lamdhip64 -lm \
 *       -Wl,-rpath,'$ORIGIN/../../elasticmm_amd' -Wl,-rpath,/opt/rocm/lib
 */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "emm_kv.h"

/* oracle (oracle/kv_oracle.c) */
void orc_kv_pack(const void *const *layers, int num_layers, int num_kv, int64_t num_blocks, int64_t chunk_bytes,
                 const int64_t *idx, int64_t n, void *packed);
void orc_kv_unpack(void *const *layers, int num_layers, int num_kv, int64_t num_blocks, int64_t chunk_bytes,
                   const int64_t *idx, int64_t n, const void *packed);
void orc_copy_blocks(void *const *layers, int num_layers, int num_kv, int64_t num_blocks, int64_t chunk_bytes,
                     const int64_t *mapping, int64_t num_pairs);
void orc_reshape_and_cache(const void *key, const void *value, void *key_cache, void *value_cache,
                           const int64_t *slot_mapping, int64_t num_tokens, int64_t row_bytes,
                           int64_t key_stride_bytes, int64_t value_stride_bytes, int64_t num_slots);
void orc_concat_rows(const void *const *srcs, const int64_t *nbytes, int n, void *dst);
void orc_reshape_and_cache_fp8(const uint16_t *key, const uint16_t *value, uint8_t *key_cache, uint8_t *value_cache,
                               const int64_t *slot_mapping, int64_t num_tokens, int64_t row_elems, int64_t key_stride,
                               int64_t value_stride, int64_t num_slots, float k_scale, float v_scale, int src_dtype);
void orc_reshape_and_cache_paged(const uint16_t *key, const uint16_t *value, void *key_cache, void *value_cache,
                                 const int64_t *slot_mapping, int64_t num_tokens, int num_heads, int head_size,
                                 int block_size, int64_t num_blocks, int64_t key_stride, int64_t value_stride,
                                 int src_dtype, int cache_elem_bytes, float k_scale, float v_scale);
void orc_kv_unpack_dequant_fp8(void *const *layers, int num_layers, int64_t num_blocks, int64_t chunk_elems,
                               const int64_t *idx, int64_t n, const uint8_t *packed, const float *k_scales,
                               const float *v_scales, int out_dtype);

#define HIP(x)                                                                                  \
  do {                                                                                          \
    hipError_t e_ = (x);                                                                        \
    if (e_ != hipSuccess) {                                                                     \
      fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);            \
      return 2;                                                                                 \
    }                                                                                           \
  } while (0)
#define EMM(x)                                                                                  \
  do {                                                                                          \
    int rc_ = (x);                                                                              \
    if (rc_ != 0) {                                                                             \
      fprintf(stderr, "emm error %d (%s) at line %d\n", rc_, emm_last_error(), __LINE__);       \
      return 3;                                                                                 \
    }                                                                                           \
  } while (0)

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint64_t rnd(void) {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return rng_state;
}
static void fill(void *p, size_t nbytes) {
  uint8_t *b = (uint8_t *)p;
  for (size_t i = 0; i < nbytes; ++i) b[i] = (uint8_t)(rnd() >> 32);
}
static void permutation(int64_t *out, int64_t n_total, int64_t n) {
  int64_t *all = (int64_t *)malloc(sizeof(int64_t) * n_total);
  for (int64_t i = 0; i < n_total; ++i) all[i] = i;
  for (int64_t i = 0; i < n; ++i) {
    int64_t j = i + (int64_t)(rnd() % (uint64_t)(n_total - i));
    int64_t t = all[i];
    all[i] = all[j];
    all[j] = t;
    out[i] = all[i];
  }
  free(all);
}
static int same(const void *a, const void *b, size_t n, const char *what) {
  if (memcmp(a, b, n) == 0) {
    printf("ok   %s (%zu bytes)\n", what, n);
    return 0;
  }
  const uint8_t *x = (const uint8_t *)a, *y = (const uint8_t *)b;
  size_t i = 0;
  while (x[i] == y[i]) ++i;
  printf("FAIL %s: first difference at byte %zu (got %u, want %u)\n", what, i, x[i], y[i]);
  return 1;
}

/* device copy of a host buffer; the program ends on a HIP error */
static void *to_device(const void *h, size_t nbytes) {
  void *d = NULL;
  if (hipMalloc(&d, nbytes) != hipSuccess || hipMemcpy(d, h, nbytes, hipMemcpyHostToDevice) != hipSuccess) {
    fprintf(stderr, "HIP error while staging %zu bytes\n", nbytes);
    exit(2);
  }
  return d;
}
/* compares a device buffer with what the oracle left in a host buffer */
static int same_on_device(const void *d, const void *h_want, size_t nbytes, const char *what) {
  void *h = malloc(nbytes);
  if (hipDeviceSynchronize() != hipSuccess || hipMemcpy(h, d, nbytes, hipMemcpyDeviceToHost) != hipSuccess) {
    fprintf(stderr, "HIP error while reading back %s\n", what);
    exit(2);
  }
  const int bad = same(h, h_want, nbytes, what);
  free(h);
  return bad;
}
/* 16-bit patterns that are finite and moderate as bf16 and as f16 (exponent field kept mid-range) */
static void fill_halves(uint16_t *p, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    const uint16_t r = (uint16_t)(rnd() >> 40);
    p[i] = (uint16_t)((r & 0x83ffu) | 0x3800u | (r & 0x0400u));
  }
}

int main(void) {
  enum { L = 3, KV = 2, NB = 37, N = 9, T = 21, PAIRS = 4 };
  const int64_t chunk = 16 * 2 * 64 * 2; /* block_size 16, 2 heads, head 64, 16-bit elements */
  const size_t layer_bytes = (size_t)KV * NB * chunk;
  int bad = 0;
  if (emm_abi_version() != EMM_KV_ABI_VERSION) {
    printf("FAIL abi version\n");
    return 1;
  }

  /* host copies (oracle side) and device pools */
  void *h_src[L], *h_dst[L], *d_src[L], *d_dst[L];
  for (int l = 0; l < L; ++l) {
    h_src[l] = malloc(layer_bytes);
    h_dst[l] = malloc(layer_bytes);
    fill(h_src[l], layer_bytes);
    memset(h_dst[l], 0xA5, layer_bytes);
    HIP(hipMalloc(&d_src[l], layer_bytes));
    HIP(hipMalloc(&d_dst[l], layer_bytes));
    HIP(hipMemcpy(d_src[l], h_src[l], layer_bytes, hipMemcpyHostToDevice));
    HIP(hipMemcpy(d_dst[l], h_dst[l], layer_bytes, hipMemcpyHostToDevice));
  }
  int64_t h_si[N], h_di[N], *d_si, *d_di;
  permutation(h_si, NB, N);
  permutation(h_di, NB, N);
  HIP(hipMalloc((void **)&d_si, sizeof(h_si)));
  HIP(hipMalloc((void **)&d_di, sizeof(h_di)));
  HIP(hipMemcpy(d_si, h_si, sizeof(h_si), hipMemcpyHostToDevice));
  HIP(hipMemcpy(d_di, h_di, sizeof(h_di), hipMemcpyHostToDevice));
  hipStream_t stream;
  HIP(hipStreamCreate(&stream));

  /* pack */
  const size_t packed_bytes = (size_t)L * KV * N * chunk;
  void *d_packed, *h_packed = malloc(packed_bytes), *h_want = malloc(packed_bytes);
  HIP(hipMalloc(&d_packed, packed_bytes));
  EMM(emm_kv_pack((const void *const *)d_src, L, KV, NB, chunk, d_si, N, d_packed, stream));
  HIP(hipStreamSynchronize(stream));
  HIP(hipMemcpy(h_packed, d_packed, packed_bytes, hipMemcpyDeviceToHost));
  orc_kv_pack((const void *const *)h_src, L, KV, NB, chunk, h_si, N, h_want);
  bad += same(h_packed, h_want, packed_bytes, "emm_kv_pack");

  /* the same pack with the block table on the host (ids travel in the kernel argument block) */
  HIP(hipMemset(d_packed, 0, packed_bytes));
  EMM(emm_kv_pack_host_ids((const void *const *)d_src, L, KV, NB, chunk, h_si, N, d_packed, stream));
  HIP(hipStreamSynchronize(stream));
  HIP(hipMemcpy(h_packed, d_packed, packed_bytes, hipMemcpyDeviceToHost));
  bad += same(h_packed, h_want, packed_bytes, "emm_kv_pack_host_ids");

  /* unpack under another table, then copy_blocks inside the destination pool */
  EMM(emm_kv_unpack(d_dst, L, KV, NB, chunk, d_di, N, d_packed, stream));
  orc_kv_unpack(h_dst, L, KV, NB, chunk, h_di, N, h_want);
  int64_t h_map[PAIRS * 2], *d_map, used[NB], free_ids[NB];
  memset(used, 0, sizeof(used));
  for (int i = 0; i < N; ++i) used[h_di[i]] = 1;
  int nf = 0;
  for (int b = 0; b < NB; ++b)
    if (!used[b]) free_ids[nf++] = b;
  for (int p = 0; p < PAIRS; ++p) {
    h_map[2 * p] = h_di[p];
    h_map[2 * p + 1] = free_ids[p];
  }
  HIP(hipMalloc((void **)&d_map, sizeof(h_map)));
  HIP(hipMemcpy(d_map, h_map, sizeof(h_map), hipMemcpyHostToDevice));
  EMM(emm_copy_blocks(d_dst, L, KV, NB, chunk, d_map, PAIRS, stream));
  orc_copy_blocks(h_dst, L, KV, NB, chunk, h_map, PAIRS);
  HIP(hipStreamSynchronize(stream));
  void *h_back = malloc(layer_bytes);
  for (int l = 0; l < L; ++l) {
    HIP(hipMemcpy(h_back, d_dst[l], layer_bytes, hipMemcpyDeviceToHost));
    char what[64];
    snprintf(what, sizeof(what), "emm_kv_unpack + emm_copy_blocks, layer %d", l);
    bad += same(h_back, h_dst[l], layer_bytes, what);
  }

  /* reshape_and_cache with two padded tokens, into layer 0 of the destination pool */
  const int64_t row = 2 * 64 * 2, num_slots = (int64_t)NB * 16;
  void *h_key = malloc(T * row), *h_val = malloc(T * row), *d_key, *d_val;
  fill(h_key, T * row);
  fill(h_val, T * row);
  int64_t h_slots[T], *d_slots;
  permutation(h_slots, num_slots, T);
  h_slots[3] = -1;
  h_slots[17] = -1;
  HIP(hipMalloc(&d_key, T * row));
  HIP(hipMalloc(&d_val, T * row));
  HIP(hipMalloc((void **)&d_slots, sizeof(h_slots)));
  HIP(hipMemcpy(d_key, h_key, T * row, hipMemcpyHostToDevice));
  HIP(hipMemcpy(d_val, h_val, T * row, hipMemcpyHostToDevice));
  HIP(hipMemcpy(d_slots, h_slots, sizeof(h_slots), hipMemcpyHostToDevice));
  char *d_kc = (char *)d_dst[0], *d_vc = d_kc + (size_t)NB * chunk;
  char *h_kc = (char *)h_dst[0], *h_vc = h_kc + (size_t)NB * chunk;
  EMM(emm_reshape_and_cache(d_key, d_val, d_kc, d_vc, d_slots, T, row, row, row, num_slots, stream));
  HIP(hipStreamSynchronize(stream));
  orc_reshape_and_cache(h_key, h_val, h_kc, h_vc, h_slots, T, row, row, row, num_slots);
  HIP(hipMemcpy(h_back, d_dst[0], layer_bytes, hipMemcpyDeviceToHost));
  bad += same(h_back, h_dst[0], layer_bytes, "emm_reshape_and_cache");

  /* concat_rows of three ragged segments taken from the source pool */
  const void *d_segs[3] = {d_src[0], (char *)d_src[1] + 4096, d_src[2]};
  const void *h_segs[3] = {h_src[0], (char *)h_src[1] + 4096, h_src[2]};
  const int64_t seg_bytes[3] = {7168 * 3, 7168, 7168 * 5};
  const size_t cat_bytes = 7168 * 9;
  void *d_cat, *h_cat = malloc(cat_bytes), *h_cat_want = malloc(cat_bytes);
  HIP(hipMalloc(&d_cat, cat_bytes));
  EMM(emm_concat_rows(d_segs, seg_bytes, 3, d_cat, 0, stream));
  HIP(hipStreamSynchronize(stream));
  HIP(hipMemcpy(h_cat, d_cat, cat_bytes, hipMemcpyDeviceToHost));
  orc_concat_rows(h_segs, seg_bytes, 3, h_cat_want);
  bad += same(h_cat, h_cat_want, cat_bytes, "emm_concat_rows");

  /* unpack with the table on the host, then the fused pool-to-pool move: both against pack + unpack of the oracle */
  int64_t h_di2[N];
  permutation(h_di2, NB, N);
  EMM(emm_kv_unpack_host_ids(d_dst, L, KV, NB, chunk, h_di2, N, d_packed, stream));
  orc_kv_unpack(h_dst, L, KV, NB, chunk, h_di2, N, h_want);
  for (int l = 0; l < L; ++l) bad += same_on_device(d_dst[l], h_dst[l], layer_bytes, "emm_kv_unpack_host_ids");
  int64_t h_si3[N], h_di3[N];
  permutation(h_si3, NB, N);
  permutation(h_di3, NB, N);
  int64_t *d_si3 = (int64_t *)to_device(h_si3, sizeof(h_si3)), *d_di3 = (int64_t *)to_device(h_di3, sizeof(h_di3));
  EMM(emm_kv_migrate((const void *const *)d_src, NB, d_dst, NB, L, KV, chunk, d_si3, d_di3, N, stream));
  orc_kv_pack((const void *const *)h_src, L, KV, NB, chunk, h_si3, N, h_want);
  orc_kv_unpack(h_dst, L, KV, NB, chunk, h_di3, N, h_want);
  for (int l = 0; l < L; ++l) bad += same_on_device(d_dst[l], h_dst[l], layer_bytes, "emm_kv_migrate");

  /* the append for all layers in one launch, token rows 8 bytes further apart than they are long */
  enum { BS = 16, H = 2, D = 64 };
  const int64_t row_elems = H * D, stride_elems = row_elems + 4;
  uint16_t *h_keys[L], *h_vals[L];
  void *d_keys[L], *d_vals[L], *d_kcs[L], *d_vcs[L];
  for (int l = 0; l < L; ++l) {
    h_keys[l] = (uint16_t *)malloc(T * stride_elems * 2);
    h_vals[l] = (uint16_t *)malloc(T * stride_elems * 2);
    fill_halves(h_keys[l], T * stride_elems);
    fill_halves(h_vals[l], T * stride_elems);
    d_keys[l] = to_device(h_keys[l], T * stride_elems * 2);
    d_vals[l] = to_device(h_vals[l], T * stride_elems * 2);
    d_kcs[l] = d_dst[l];
    d_vcs[l] = (char *)d_dst[l] + (size_t)NB * chunk;
    orc_reshape_and_cache(h_keys[l], h_vals[l], h_dst[l], (char *)h_dst[l] + (size_t)NB * chunk, h_slots, T, row,
                          stride_elems * 2, stride_elems * 2, num_slots);
  }
  EMM(emm_reshape_and_cache_layers((const void *const *)d_keys, (const void *const *)d_vals, d_kcs, d_vcs, L, d_slots, T,
                                   row, stride_elems * 2, stride_elems * 2, num_slots, stream));
  for (int l = 0; l < L; ++l) bad += same_on_device(d_dst[l], h_dst[l], layer_bytes, "emm_reshape_and_cache_layers");

  /* the same tokens into a head-major cache [NB, H, BS, D] through the strided entry point */
  {
    const int64_t head_bytes = D * 2;
    for (int l = 0; l < L; ++l)
      for (int kv = 0; kv < 2; ++kv) {
        char *plane = (char *)h_dst[l] + (size_t)kv * NB * chunk;
        const uint16_t *x = kv ? h_vals[l] : h_keys[l];
        for (int t = 0; t < T; ++t) {
          if (h_slots[t] < 0) continue;
          const int64_t b = h_slots[t] / BS, o = h_slots[t] % BS;
          for (int h = 0; h < H; ++h)
            memcpy(plane + b * chunk + h * BS * head_bytes + o * head_bytes, x + t * stride_elems + h * D, head_bytes);
        }
      }
    EMM(emm_reshape_and_cache_strided((const void *const *)d_keys, (const void *const *)d_vals, d_kcs, d_vcs, L, d_slots,
                                      T, H, head_bytes, BS, NB, stride_elems * 2, stride_elems * 2, chunk, head_bytes,
                                      BS * head_bytes, stream));
    for (int l = 0; l < L; ++l) bad += same_on_device(d_dst[l], h_dst[l], layer_bytes, "emm_reshape_and_cache_strided");
  }

  /* fp8 caches: the quantising append per layer and for all layers, then pack + dequantising unpack */
  {
    const int64_t chunk_elems = BS * row_elems;
    const size_t plane8 = (size_t)NB * chunk_elems, layer8 = 2 * plane8;
    const float h_ks[L] = {0.05f, 0.011f, 0.3f}, h_vs[L] = {0.02f, 0.09f, 0.0071f};
    float *d_ks = (float *)to_device(h_ks, sizeof(h_ks)), *d_vs = (float *)to_device(h_vs, sizeof(h_vs));
    uint8_t *h_p8[L];
    void *d_p8[L], *d_kc8[L], *d_vc8[L];
    for (int l = 0; l < L; ++l) {
      h_p8[l] = (uint8_t *)malloc(layer8);
      fill(h_p8[l], layer8);
      for (size_t i = 0; i < layer8; ++i)
        if ((h_p8[l][i] & 0x7f) == 0x7f) h_p8[l][i] ^= 1; /* no NaN bytes: their 16-bit form is not part of the contract */
      d_p8[l] = to_device(h_p8[l], layer8);
      d_kc8[l] = d_p8[l];
      d_vc8[l] = (char *)d_p8[l] + plane8;
    }
    EMM(emm_reshape_and_cache_fp8(d_keys[0], d_vals[0], d_kc8[0], d_vc8[0], d_slots, T, row_elems, stride_elems,
                                  stride_elems, num_slots, d_ks, d_vs, EMM_DTYPE_BF16, stream));
    orc_reshape_and_cache_fp8(h_keys[0], h_vals[0], h_p8[0], h_p8[0] + plane8, h_slots, T, row_elems, stride_elems,
                              stride_elems, num_slots, h_ks[0], h_vs[0], EMM_DTYPE_BF16);
    bad += same_on_device(d_p8[0], h_p8[0], layer8, "emm_reshape_and_cache_fp8 (bf16 source)");
    int64_t h_slots2[T];
    permutation(h_slots2, num_slots, T);
    h_slots2[0] = -1;
    int64_t *d_slots2 = (int64_t *)to_device(h_slots2, sizeof(h_slots2));
    EMM(emm_reshape_and_cache_fp8_layers((const void *const *)d_keys, (const void *const *)d_vals, d_kc8, d_vc8, L, d_slots2,
                                         T, row_elems, stride_elems, stride_elems, num_slots, d_ks, d_vs, EMM_DTYPE_F16,
                                         stream));
    for (int l = 0; l < L; ++l) {
      orc_reshape_and_cache_fp8(h_keys[l], h_vals[l], h_p8[l], h_p8[l] + plane8, h_slots2, T, row_elems, stride_elems,
                                stride_elems, num_slots, h_ks[l], h_vs[l], EMM_DTYPE_F16);
      bad += same_on_device(d_p8[l], h_p8[l], layer8, "emm_reshape_and_cache_fp8_layers (f16 source)");
    }
    /* the quantising append into a head-major fp8 cache [NB, H, BS, D] through the strided entry point: the contiguous
     * append of the oracle on a copy of the pool, permuted, is the expected content */
    {
      int64_t h_slots3[T];
      permutation(h_slots3, num_slots, T);
      h_slots3[1] = -1;
      int64_t *d_slots3 = (int64_t *)to_device(h_slots3, sizeof(h_slots3));
      uint8_t *h_flat = (uint8_t *)malloc(layer8), *h_hm = (uint8_t *)malloc(layer8);
      void *d_hm[L], *d_hk[L], *d_hv[L];
      for (int l = 0; l < L; ++l) {
        for (int kv = 0; kv < 2; ++kv)
          for (int64_t b = 0; b < NB; ++b)
            for (int o = 0; o < BS; ++o)
              for (int h = 0; h < H; ++h)
                memcpy(h_hm + kv * plane8 + b * chunk_elems + ((size_t)h * BS + o) * D,
                       h_p8[l] + kv * plane8 + b * chunk_elems + ((size_t)o * H + h) * D, D);
        d_hm[l] = to_device(h_hm, layer8);
        d_hk[l] = d_hm[l];
        d_hv[l] = (char *)d_hm[l] + plane8;
      }
      EMM(emm_reshape_and_cache_strided_fp8((const void *const *)d_keys, (const void *const *)d_vals, d_hk, d_hv, L, d_slots3,
                                            T, H, D, BS, NB, stride_elems, stride_elems, chunk_elems, D, (int64_t)BS * D,
                                            d_ks, d_vs, EMM_DTYPE_BF16, stream));
      for (int l = 0; l < L; ++l) {
        memcpy(h_flat, h_p8[l], layer8);
        orc_reshape_and_cache_fp8(h_keys[l], h_vals[l], h_flat, h_flat + plane8, h_slots3, T, row_elems, stride_elems,
                                  stride_elems, num_slots, h_ks[l], h_vs[l], EMM_DTYPE_BF16);
        for (int kv = 0; kv < 2; ++kv)
          for (int64_t b = 0; b < NB; ++b)
            for (int o = 0; o < BS; ++o)
              for (int h = 0; h < H; ++h)
                memcpy(h_hm + kv * plane8 + b * chunk_elems + ((size_t)h * BS + o) * D,
                       h_flat + kv * plane8 + b * chunk_elems + ((size_t)o * H + h) * D, D);
        bad += same_on_device(d_hm[l], h_hm, layer8, "emm_reshape_and_cache_strided_fp8");
      }
    }
    /* fp8 bytes travel through pack unchanged (chunk = chunk_elems bytes); the receiving pool is bf16 */
    const size_t packed8 = (size_t)L * 2 * N * chunk_elems;
    uint8_t *h_packed8 = (uint8_t *)malloc(packed8);
    void *d_packed8;
    HIP(hipMalloc(&d_packed8, packed8));
    EMM(emm_kv_pack((const void *const *)d_p8, L, 2, NB, chunk_elems, d_si, N, d_packed8, stream));
    orc_kv_pack((const void *const *)h_p8, L, 2, NB, chunk_elems, h_si, N, h_packed8);
    bad += same_on_device(d_packed8, h_packed8, packed8, "emm_kv_pack of an fp8 pool");
    EMM(emm_kv_unpack_dequant_fp8(d_dst, L, NB, chunk_elems, d_di, N, d_packed8, d_ks, d_vs, EMM_DTYPE_BF16, stream));
    orc_kv_unpack_dequant_fp8(h_dst, L, NB, chunk_elems, h_di, N, h_packed8, h_ks, h_vs, EMM_DTYPE_BF16);
    for (int l = 0; l < L; ++l) bad += same_on_device(d_dst[l], h_dst[l], layer_bytes, "emm_kv_unpack_dequant_fp8");

    /* paged-attention layout: one prompt filling blocks in order plus scattered tokens; 16-bit and fp8 caches */
    enum { TP = 50 };
    int64_t h_ps[TP], blocks[NB];
    permutation(blocks, NB, NB);
    for (int t = 0; t < 37; ++t) h_ps[t] = blocks[t / BS] * BS + t % BS; /* two whole blocks and 5 tokens of a third */
    for (int t = 37; t < TP; ++t) h_ps[t] = blocks[3 + (t - 37)] * BS + (int64_t)(rnd() % BS);
    h_ps[40] = -1;
    int64_t *d_ps = (int64_t *)to_device(h_ps, sizeof(h_ps));
    uint16_t *h_pk[L], *h_pv[L];
    void *d_pk[L], *d_pv[L];
    for (int l = 0; l < L; ++l) {
      h_pk[l] = (uint16_t *)malloc(TP * row_elems * 2);
      h_pv[l] = (uint16_t *)malloc(TP * row_elems * 2);
      fill_halves(h_pk[l], TP * row_elems);
      fill_halves(h_pv[l], TP * row_elems);
      d_pk[l] = to_device(h_pk[l], TP * row_elems * 2);
      d_pv[l] = to_device(h_pv[l], TP * row_elems * 2);
    }
    EMM(emm_reshape_and_cache_paged(d_pk[0], d_pv[0], d_kcs[0], d_vcs[0], d_ps, TP, H, D, BS, NB, row_elems, row_elems,
                                    EMM_DTYPE_BF16, 2, NULL, NULL, stream));
    orc_reshape_and_cache_paged(h_pk[0], h_pv[0], h_dst[0], (char *)h_dst[0] + (size_t)NB * chunk, h_ps, TP, H, D, BS, NB,
                                row_elems, row_elems, EMM_DTYPE_BF16, 2, 1.0f, 1.0f);
    bad += same_on_device(d_dst[0], h_dst[0], layer_bytes, "emm_reshape_and_cache_paged (16-bit cache)");
    EMM(emm_reshape_and_cache_paged_layers((const void *const *)d_pk, (const void *const *)d_pv, d_kcs, d_vcs, L, d_ps, TP,
                                           H, D, BS, NB, row_elems, row_elems, EMM_DTYPE_F16, 2, NULL, NULL, stream));
    EMM(emm_reshape_and_cache_paged_layers((const void *const *)d_pk, (const void *const *)d_pv, d_kc8, d_vc8, L, d_ps, TP,
                                           H, D, BS, NB, row_elems, row_elems, EMM_DTYPE_BF16, 1, d_ks, d_vs, stream));
    for (int l = 0; l < L; ++l) {
      orc_reshape_and_cache_paged(h_pk[l], h_pv[l], h_dst[l], (char *)h_dst[l] + (size_t)NB * chunk, h_ps, TP, H, D, BS,
                                  NB, row_elems, row_elems, EMM_DTYPE_F16, 2, 1.0f, 1.0f);
      bad += same_on_device(d_dst[l], h_dst[l], layer_bytes, "emm_reshape_and_cache_paged_layers (16-bit cache)");
      orc_reshape_and_cache_paged(h_pk[l], h_pv[l], h_p8[l], h_p8[l] + plane8, h_ps, TP, H, D, BS, NB, row_elems,
                                  row_elems, EMM_DTYPE_BF16, 1, h_ks[l], h_vs[l]);
      bad += same_on_device(d_p8[l], h_p8[l], layer8, "emm_reshape_and_cache_paged_layers (fp8 cache)");
    }
  }

  /* the plain copy */
  EMM(emm_stream_copy(d_src[1], d_dst[2], (int64_t)layer_bytes - 3, stream));
  memcpy(h_dst[2], h_src[1], layer_bytes - 3);
  bad += same_on_device(d_dst[2], h_dst[2], layer_bytes, "emm_stream_copy");

  /* an argument error is reported, not raised */
  if (emm_kv_pack((const void *const *)d_src, EMM_MAX_LAYERS + 1, KV, NB, chunk, d_si, N, d_packed, stream) != EMM_EINVAL ||
      strstr(emm_last_error(), "num_layers") == NULL) {
    printf("FAIL argument error path\n");
    ++bad;
  } else {
    printf("ok   argument error: %s\n", emm_last_error());
  }
  printf(bad ? "C ABI CHECK FAILED (%d)\n" : "C ABI CHECK PASSED\n", bad);
  return bad ? 1 : 0;
}
