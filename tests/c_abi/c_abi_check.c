/*
 * A C program (no Python, no torch) that drives libemm_kv.so through include/emm_kv.h and checks
 * pack, unpack, copy_blocks, reshape_and_cache and concat_rows against the loops of
 * oracle/kv_oracle.c on seeded data. Built and run by tests/test_c_abi_program.py.
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
