/*
 * kv_oracle.c — TEST INFRASTRUCTURE, not product code.
 *
 * Plain-C, single-threaded CPU restatement of the KV-cache data-movement path
 * of ElasticMM, used only as the checker in tests/, in __graft_entry__.smoke()
 * and as an optional CPU-baseline leg of bench.py. Nothing under
 * elasticmm_amd/ may link, load or call it.
 *
 * The reference expresses the path as torch tensor indexing; each function
 * below restates one of those expressions as explicit loops over
 * (layer, K|V, block) with a memcpy of one chunk, where
 *   pool layer   = [num_kv][num_blocks][chunk_bytes]   (worker.py:594)
 *   packed       = [num_layers][num_kv][n][chunk_bytes] (worker.py:587, :608)
 *
 * Pinning of each function (what independent fact checks it) is listed in
 * tests/test_oracle.py; the header of oracle/kv_oracle.py summarises it.
 *
 * Build: gcc -O2 -fPIC -shared -o oracle/libkv_oracle.so oracle/kv_oracle.c
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- pack: V0Worker.extract_kv_blocks, elasticmm/engine/v0/worker.py:597-608
 * (out[l] = layer_kv[:, idx]; stack over l). Negative / out-of-range ids are
 * skipped (their output chunk is left as it was), mirroring the -1 padding
 * convention of worker.py:924-925. */
void orc_kv_pack(const void *const *layers, int num_layers, int num_kv,
                 int64_t num_blocks, int64_t chunk_bytes, const int64_t *idx,
                 int64_t n, void *packed) {
  char *out = (char *)packed;
  for (int l = 0; l < num_layers; ++l)
    for (int kv = 0; kv < num_kv; ++kv)
      for (int64_t j = 0; j < n; ++j) {
        const int64_t b = idx[j];
        if (b < 0 || b >= num_blocks) continue;
        const char *src = (const char *)layers[l] + ((int64_t)kv * num_blocks + b) * chunk_bytes;
        char *dst = out + ((((int64_t)l * num_kv + kv) * n) + j) * chunk_bytes;
        memcpy(dst, src, (size_t)chunk_bytes);
      }
}

/* ---- unpack: V0Worker.write_kv_blocks, worker.py:628-633
 * (layer_kv[:, idx] = kv_data[l]). */
void orc_kv_unpack(void *const *layers, int num_layers, int num_kv,
                   int64_t num_blocks, int64_t chunk_bytes, const int64_t *idx,
                   int64_t n, const void *packed) {
  const char *in = (const char *)packed;
  for (int l = 0; l < num_layers; ++l)
    for (int kv = 0; kv < num_kv; ++kv)
      for (int64_t j = 0; j < n; ++j) {
        const int64_t b = idx[j];
        if (b < 0 || b >= num_blocks) continue;
        char *dst = (char *)layers[l] + ((int64_t)kv * num_blocks + b) * chunk_bytes;
        const char *src = in + ((((int64_t)l * num_kv + kv) * n) + j) * chunk_bytes;
        memcpy(dst, src, (size_t)chunk_bytes);
      }
}

/* ---- copy_blocks: vLLM copy_blocks(kv_caches, block_mapping[P,2]) reached via
 * CacheEngine (worker.py:380); analogue backend.py:674-708. Disjoint src/dst. */
void orc_copy_blocks(void *const *layers, int num_layers, int num_kv,
                     int64_t num_blocks, int64_t chunk_bytes,
                     const int64_t *mapping, int64_t num_pairs) {
  for (int l = 0; l < num_layers; ++l)
    for (int kv = 0; kv < num_kv; ++kv)
      for (int64_t p = 0; p < num_pairs; ++p) {
        const int64_t s = mapping[2 * p], d = mapping[2 * p + 1];
        if (s < 0 || s >= num_blocks || d < 0 || d >= num_blocks) continue;
        char *base = (char *)layers[l] + (int64_t)kv * num_blocks * chunk_bytes;
        memmove(base + d * chunk_bytes, base + s * chunk_bytes, (size_t)chunk_bytes);
      }
}

/* ---- reshape_and_cache_flash (vLLM; call sites worker_steps.py:281, :438):
 * cache.view(num_slots, row)[slot[t]] = x[t] for slot[t] >= 0. */
void orc_reshape_and_cache(const void *key, const void *value, void *key_cache,
                           void *value_cache, const int64_t *slot_mapping,
                           int64_t num_tokens, int64_t row_bytes,
                           int64_t key_stride_bytes, int64_t value_stride_bytes,
                           int64_t num_slots) {
  for (int64_t t = 0; t < num_tokens; ++t) {
    const int64_t s = slot_mapping[t];
    if (s < 0 || s >= num_slots) continue;
    memcpy((char *)key_cache + s * row_bytes, (const char *)key + t * key_stride_bytes, (size_t)row_bytes);
    memcpy((char *)value_cache + s * row_bytes, (const char *)value + t * value_stride_bytes, (size_t)row_bytes);
  }
}

/* ---- scalar conversions --------------------------------------------------
 * fp32 -> e4m3fn: round to nearest, ties to even, no saturation; what rounds
 * beyond 448 (the first such input is the tie 464 -> 448, anything above
 * rounds to 480 which has no encoding), +-inf and NaN all give sign|0x7F.
 * Derived from the format definition (OCP FP8 E4M3: bias 7, 3 mantissa bits,
 * subnormal step 2^-9, S.1111.111 = NaN), NOT from any library's source: the
 * value is scaled onto the integer grid of its binade and rounded with
 * nearbyint() under the default round-to-nearest-even mode. */
uint8_t orc_f32_to_e4m3fn(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  const float a = fabsf(f);
  if (!(a == a) || a == INFINITY) return sign | 0x7f;
  if (a == 0.0f) return sign;
  int e;
  (void)frexpf(a, &e); /* a = m * 2^e, m in [0.5, 1) -> binade exponent e-1 */
  int ex = e - 1;
  if (ex < -6) ex = -6; /* subnormals share the grid of the lowest binade */
  /* grid step of this binade is 2^(ex-3); q = a / step is exact (power of 2) */
  const double q = nearbyint(ldexp((double)a, 3 - ex));
  /* q in [0, 16]; q == 16 means it rounded up into the next binade */
  int64_t qi = (int64_t)q;
  if (qi == 16) { qi = 8; ex += 1; }
  if (ex > 8) return sign | 0x7f;
  uint8_t code;
  if (qi < 8) code = (uint8_t)qi; /* subnormal (only possible with ex == -6) */
  else code = (uint8_t)(((ex + 7) << 3) | (qi - 8));
  if (code == 0x7f) return sign | 0x7f; /* 480 is not representable */
  return sign | code;
}

float orc_e4m3fn_to_f32(uint8_t b) {
  const int s = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 15 && m == 7) v = NAN;
  else if (e == 0) v = ldexpf((float)m, -9);
  else v = ldexpf((float)(8 + m), e - 10);
  return s ? -v : v;
}

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static float f16_to_f32(uint16_t h) {
  const int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  float v;
  if (e == 31) v = m ? NAN : INFINITY;
  else if (e == 0) v = ldexpf((float)m, -24);
  else v = ldexpf((float)(1024 + m), e - 25);
  return s ? -v : v;
}

/* fp32 -> bf16, RNE, NaN -> 0x7FC0 */
uint16_t orc_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  const uint32_t lsb = (u >> 16) & 1u;
  return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}

/* fp32 -> f16 (bias 15, 10 mantissa bits, subnormal step 2^-24), RNE on the
 * binade's integer grid, overflow -> inf, NaN -> 0x7E00 */
uint16_t orc_f32_to_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const float a = fabsf(f);
  if (a != a) return 0x7e00;
  if (a == INFINITY) return sign | 0x7c00;
  if (a == 0.0f) return sign;
  int e;
  (void)frexpf(a, &e);
  int ex = e - 1;
  if (ex < -14) ex = -14;
  int64_t q = (int64_t)nearbyint(ldexp((double)a, 10 - ex));
  if (q == 2048) { q = 1024; ex += 1; }
  if (ex > 15) return sign | 0x7c00;
  if (q < 1024) return sign | (uint16_t)q;
  return sign | (uint16_t)(((ex + 15) << 10) | (q - 1024));
}

/* src_dtype: 0 = bf16, 1 = f16 */
static float half_to_f32(uint16_t h, int dtype) { return dtype == 0 ? bf16_to_f32(h) : f16_to_f32(h); }

/* quantise n 16-bit values: q = e4m3fn(float(x) / scale) */
void orc_quant_fp8(const uint16_t *x, int64_t n, float scale, int src_dtype, uint8_t *q) {
  for (int64_t i = 0; i < n; ++i) {
    volatile float d = half_to_f32(x[i], src_dtype) / scale; /* one fp32 division */
    q[i] = orc_f32_to_e4m3fn(d);
  }
}

/* saturating variant: the quotient is clamped to [-448, 448] before the cast (NaN stays NaN), so
 * overflow and +-inf give sign|0x7E and only NaN gives sign|0x7F:
 * torch.clamp(x.float() / scale, -448, 448).to(torch.float8_e4m3fn), the convention of vLLM's fp8
 * KV cache (the cache dtype the reference leaves open at elasticmm/engine/v0/worker.py:194). */
void orc_quant_fp8_sat(const uint16_t *x, int64_t n, float scale, int src_dtype, uint8_t *q) {
  for (int64_t i = 0; i < n; ++i) {
    volatile float d = half_to_f32(x[i], src_dtype) / scale; /* one fp32 division */
    float c = d;
    if (c > 448.0f) c = 448.0f;   /* comparisons with NaN are false: NaN passes through */
    if (c < -448.0f) c = -448.0f;
    q[i] = orc_f32_to_e4m3fn(c);
  }
}

/* dequantise n fp8 bytes: out = 16bit_rne(float(q) * scale) */
void orc_dequant_fp8(const uint8_t *q, int64_t n, float scale, int out_dtype, uint16_t *out) {
  for (int64_t i = 0; i < n; ++i) {
    volatile float p = orc_e4m3fn_to_f32(q[i]) * scale;
    out[i] = out_dtype == 0 ? orc_f32_to_bf16(p) : orc_f32_to_f16(p);
  }
}

/* ---- fp8 append: reshape_and_cache with quantisation on write. Strides and
 * row size in elements; one scale for K and one for V (per layer). */
void orc_reshape_and_cache_fp8(const uint16_t *key, const uint16_t *value,
                               uint8_t *key_cache, uint8_t *value_cache,
                               const int64_t *slot_mapping, int64_t num_tokens,
                               int64_t row_elems, int64_t key_stride,
                               int64_t value_stride, int64_t num_slots,
                               float k_scale, float v_scale, int src_dtype) {
  for (int64_t t = 0; t < num_tokens; ++t) {
    const int64_t s = slot_mapping[t];
    if (s < 0 || s >= num_slots) continue;
    orc_quant_fp8(key + t * key_stride, row_elems, k_scale, src_dtype, key_cache + s * row_elems);
    orc_quant_fp8(value + t * value_stride, row_elems, v_scale, src_dtype, value_cache + s * row_elems);
  }
}

/* ---- reshape_and_cache, paged-attention layout (vLLM; same call sites when a
 * PagedAttention backend is selected): key_cache [NB, H, D/x, bs, x],
 * value_cache [NB, H, D, bs], x = 16 / cache element bytes. Written from the
 * layout definition with explicit index arithmetic; cache_elem_bytes 2 copies
 * bits, 1 quantises to e4m3fn. */
void orc_reshape_and_cache_paged(const uint16_t *key, const uint16_t *value,
                                 void *key_cache, void *value_cache,
                                 const int64_t *slot_mapping, int64_t num_tokens,
                                 int num_heads, int head_size, int block_size,
                                 int64_t num_blocks, int64_t key_stride,
                                 int64_t value_stride, int src_dtype,
                                 int cache_elem_bytes, float k_scale, float v_scale) {
  const int x = 16 / cache_elem_bytes;
  for (int64_t t = 0; t < num_tokens; ++t) {
    const int64_t s = slot_mapping[t];
    if (s < 0 || s >= num_blocks * block_size) continue;
    const int64_t b = s / block_size, o = s % block_size;
    for (int h = 0; h < num_heads; ++h)
      for (int d = 0; d < head_size; ++d) {
        const uint16_t kx = key[t * key_stride + (int64_t)h * head_size + d];
        const uint16_t vx = value[t * value_stride + (int64_t)h * head_size + d];
        const int64_t ki = ((((b * num_heads + h) * (head_size / x) + d / x) * block_size + o) * x) + d % x;
        const int64_t vi = ((b * num_heads + h) * head_size + d) * block_size + o;
        if (cache_elem_bytes == 2) {
          ((uint16_t *)key_cache)[ki] = kx;
          ((uint16_t *)value_cache)[vi] = vx;
        } else {
          ((uint8_t *)key_cache)[ki] = orc_f32_to_e4m3fn(half_to_f32(kx, src_dtype) / k_scale);
          ((uint8_t *)value_cache)[vi] = orc_f32_to_e4m3fn(half_to_f32(vx, src_dtype) / v_scale);
        }
      }
  }
}

/* ---- dequant-unpack: packed fp8 [L,2,n,chunk] -> 16-bit pool under idx */
void orc_kv_unpack_dequant_fp8(void *const *layers, int num_layers,
                               int64_t num_blocks, int64_t chunk_elems,
                               const int64_t *idx, int64_t n,
                               const uint8_t *packed, const float *k_scales,
                               const float *v_scales, int out_dtype) {
  for (int l = 0; l < num_layers; ++l)
    for (int kv = 0; kv < 2; ++kv)
      for (int64_t j = 0; j < n; ++j) {
        const int64_t b = idx[j];
        if (b < 0 || b >= num_blocks) continue;
        uint16_t *dst = (uint16_t *)layers[l] + ((int64_t)kv * num_blocks + b) * chunk_elems;
        const uint8_t *src = packed + ((((int64_t)l * 2 + kv) * n) + j) * chunk_elems;
        orc_dequant_fp8(src, chunk_elems, kv == 0 ? k_scales[l] : v_scales[l], out_dtype, dst);
      }
}

/* ---- concat_rows: torch.cat(vision_embeds, dim=0), worker_steps.py:264-267 */
void orc_concat_rows(const void *const *srcs, const int64_t *nbytes, int n, void *dst) {
  char *o = (char *)dst;
  for (int i = 0; i < n; ++i) {
    memcpy(o, srcs[i], (size_t)nbytes[i]);
    o += nbytes[i];
  }
}
