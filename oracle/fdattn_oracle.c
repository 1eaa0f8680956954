/*
 * fdattn_oracle.c - CPU restatement of the paged-KV attention path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the fastdeploy_amd package,
 * libfdattn.so) may link, import or call this file; it is the checker the
 * tests, the smoke run and the benchmark's CPU-baseline leg compare the HIP
 * kernels against.
 *
 * Parity status: the reference tree holds no implementation, test or golden
 * vector of this path (no RoPE, KV quantisation, paged attention, block
 * selection or append attention anywhere under it), so against the reference
 * every function here is PARITY UNPINNED.  What the tests do pin it against:
 *   - fdo_f32_to_bf16 / fdo_f32_to_e4m3 / fdo_e4m3_to_f32: torch's CPU casts,
 *     exhaustively over all 65,536 bf16 patterns (and all 256 fp8 codes);
 *   - fdo_write_cache_kv: closed forms (pos 0 = identity, pair norms kept,
 *     complex multiplication in fp64), |x - q*s| <= s/2, max-abs -> +-127;
 *     its epilogue (bias, RMS norm of Q and K heads): torch's bf16 add and an
 *     fp64 RMS norm, unit weights -> unit mean square, scale invariance;
 *     its dynamic formats (one scale per stored row): the stored scale is the
 *     row's numpy max-abs / 127 (/ 448), the row's largest element maps to
 *     +-127 (+-448), and the bytes equal those of the static writer run with
 *     that row's scale in every channel;
 *   - decode / prefill over the dynamic formats: equal to the same functions
 *     over a static cache when every row of a head carries the same scale, and
 *     to fp64 SDPA on the dequantised cache otherwise;
 *   - fdo_decode_attention: torch CPU scaled_dot_product_attention in fp64 on
 *     the dequantised gathered cache, block-table permutation invariance,
 *     kv_len 1 = V row, constant K = mean of V; its softmax against the
 *     known-answer vectors of tests/function/test_softmax.cc:28-33;
 *   - fdo_splitkv_combine: split-count invariance against the unsplit result;
 *   - fdo_sqattn_block_scores: brute force in numpy fp64 (per-channel and
 *     dynamic formats);
 *   - fdo_topk_select: torch.topk / stable argsort, the tie rule of
 *     fastdeploy/vision/utils/utils.h:41-60 and the sort vectors of
 *     tests/function/test_sort.cc:26-106;
 *   - fdo_append_attention_prefill: dense causal SDPA in fp64, chunking
 *     invariance, one-token chunk = decode.
 *
 * Conventions the reference does supply and this file follows:
 *   softmax = subtract the row max, exponentiate, normalise
 *             (fastdeploy/function/softmax.cc:58-86; its clip at -64 is a
 *             property of that op, not of attention, and is not applied);
 *   saturation = clip to the representable range (fastdeploy/function/clip.cc:20-30);
 *   top-k ties go to the lowest index (fastdeploy/vision/utils/utils.h:41-60);
 *   comparison tolerance is "abs OR rel" (tests/gtest_utils.h:47-61).
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (see oracle/Makefile).
 * -ffp-contract=off matters: the cache bytes are defined by separately rounded
 * fp32 multiplies, adds and one division.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FDO_CACHE_INT8 1
#define FDO_CACHE_FP8 2
/* the same byte formats with one scale per (token, KV head), computed by the writer from the row it
 * stores: scale caches fp32 [num_blocks, kv_heads, block_size] in place of the [kv_heads, head_dim] ones */
#define FDO_CACHE_INT8_DYNAMIC 3
#define FDO_CACHE_FP8_DYNAMIC 4

static inline int is_dynamic(int cache_type) { return cache_type == FDO_CACHE_INT8_DYNAMIC || cache_type == FDO_CACHE_FP8_DYNAMIC; }
static inline int byte_format(int cache_type) {
  return cache_type == FDO_CACHE_INT8_DYNAMIC ? FDO_CACHE_INT8 : (cache_type == FDO_CACHE_FP8_DYNAMIC ? FDO_CACHE_FP8 : cache_type);
}

/* ---------------------------------------------------------------- scalars */

float fdo_bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even; NaN -> quiet NaN with the sign kept */
uint16_t fdo_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* fp8 e4m3fn: 1-4-3, bias 7, no infinities, 0x7f/0xff = NaN, max 448. */
float fdo_e4m3_to_f32(uint8_t c) {
  int e = (c >> 3) & 0xf, m = c & 7;
  float v;
  if (e == 0xf && m == 7) return NAN;
  if (e == 0)
    v = ldexpf((float)m, -9);
  else
    v = ldexpf((float)(8 + m), e - 10);
  return (c & 0x80) ? -v : v;
}

/* clamp to +-448, then round to nearest even onto the e4m3fn grid */
uint8_t fdo_f32_to_e4m3(float x) {
  uint8_t s = signbit(x) ? 0x80 : 0;
  float a = fabsf(x);
  if (isnan(x)) return (uint8_t)(s | 0x7f);
  if (a >= 448.0f) return (uint8_t)(s | 0x7e);
  if (a < 0.015625f) { /* below 2^-6: subnormal grid of 2^-9 */
    int q = (int)rintf(a * 512.0f);
    return (uint8_t)(s | q); /* q == 8 is the first normal code */
  }
  int e;
  (void)frexpf(a, &e); /* a = f * 2^e, f in [0.5, 1) -> a in [2^(e-1), 2^e) */
  e -= 1;
  int m = (int)rintf(ldexpf(a, 3 - e)); /* in [8, 16] */
  if (m == 16) {
    m = 8;
    e += 1;
  }
  return (uint8_t)(s | ((e + 7) << 3) | (m - 8));
}

/* int8: x / scale with one IEEE division, ties-to-even, clamp to [-127, 127] */
int8_t fdo_quant_int8(float x, float scale) {
  float r = rintf(x / scale);
  if (r > 127.0f) r = 127.0f;
  if (r < -127.0f) r = -127.0f;
  if (isnan(r)) r = 0.0f;
  return (int8_t)r;
}

uint8_t fdo_quant_fp8(float x, float scale) { return fdo_f32_to_e4m3(x / scale); }

static inline float dequant(uint8_t byte, int cache_type) {
  return byte_format(cache_type) == FDO_CACHE_INT8 ? (float)(int8_t)byte : fdo_e4m3_to_f32(byte);
}

/*
 * The scale of one stored row of the dynamic formats: (largest magnitude of the row) / 127 for int8,
 * / 448 for fp8, one IEEE division; a row of zeros gets the scale 1.  NaNs do not take part in the maximum.
 */
float fdo_row_scale(const float* x, int d, int cache_type) {
  float m = 0.f;
  for (int c = 0; c < d; ++c) m = fmaxf(m, fabsf(x[c]));
  if (!(m > 0.f)) return 1.0f;
  return m / (byte_format(cache_type) == FDO_CACHE_INT8 ? 127.0f : 448.0f);
}

/* ------------------------------------------------------------ cache writer */

/*
 * y1 = x1*cos - x2*sin ; y2 = x2*cos + x1*sin, every product and sum rounded
 * to fp32 on its own.  Pair (j, j + d/2) for the NeoX style, (2j, 2j+1) for
 * the interleaved one.
 */
static void rope_row(const float* x, float* y, int d, const float* cs, const float* sn, int style) {
  int half = d / 2;
  for (int j = 0; j < half; ++j) {
    int i1 = style ? j : 2 * j;
    int i2 = style ? j + half : 2 * j + 1;
    float x1 = x[i1], x2 = x[i2];
    if (cs) {
      float c = cs[j], s = sn[j];
      float a = x1 * c, b = x2 * s, e = x2 * c, f = x1 * s;
      y[i1] = a - b;
      y[i2] = e + f;
    } else {
      y[i1] = x1;
      y[i2] = x2;
    }
  }
}

/*
 * The QKV projection's epilogue on one head: x = bf16(x + bias) when a bias is given, then the
 * RMS norm x / sqrt(mean(x^2) + eps) * w when a weight is given.  The sum of squares has a fixed
 * order: the rotation pairs j = 0 .. d/2-1 are taken in groups of 8; a group's sum is (squares of
 * its 8 first members, added one after the other from 0) + (the same over its 8 second members);
 * the d/16 group sums are combined by a butterfly, t[u] <- t[u] + t[u ^ o] for o = 1, 2, 4, ...
 * (d/16 must be a power of two).  mean = sum / d, then one add, one square root, one division,
 * and two products per channel, each rounded to fp32.
 */
static void epilogue_row(const uint16_t* x, const uint16_t* bias, const float* w, float eps, int d, int style,
                         float* out) {
  for (int c = 0; c < d; ++c) {
    float v = fdo_bf16_to_f32(x[c]);
    if (bias) v = fdo_bf16_to_f32(fdo_f32_to_bf16(v + fdo_bf16_to_f32(bias[c])));
    out[c] = v;
  }
  if (!w) return;
  int half = d / 2, groups = d / 16;
  float t[64], t2[64];
  for (int u = 0; u < groups; ++u) {
    float s1 = 0.f, s2 = 0.f;
    for (int i = 0; i < 8; ++i) {
      int j = 8 * u + i;
      float a = out[style ? j : 2 * j], b = out[style ? j + half : 2 * j + 1];
      float aa = a * a, bb = b * b;
      s1 = s1 + aa;
      s2 = s2 + bb;
    }
    t[u] = s1 + s2;
  }
  for (int o = 1; o < groups; o <<= 1) {
    for (int u = 0; u < groups; ++u) t2[u] = t[u] + t[u ^ o];
    memcpy(t, t2, sizeof(float) * groups);
  }
  float ms = t[0] / (float)d;
  float r = 1.0f / sqrtf(ms + eps);
  for (int c = 0; c < d; ++c) {
    float v = out[c] * r;
    out[c] = v * w[c];
  }
}

int fdo_write_cache_kv_ex(const uint16_t* qkv, uint16_t* q_out, uint16_t* k_out, uint16_t* v_out,
                          uint8_t* key_cache, uint8_t* value_cache, const float* k_scale,
                          const float* v_scale, const float* rope_cos, const float* rope_sin,
                          const int32_t* block_tables, const int32_t* seq_lens_decoder,
                          const int32_t* cu_seqlens_q, int num_tokens, int batch, int hq, int hkv,
                          int d, int block_size, int max_blocks_per_seq, int num_blocks, int max_pos,
                          int rope_style, int cache_type, const uint16_t* qkv_bias, const float* q_norm_w,
                          const float* k_norm_w, float eps) {
  int row = (hq + 2 * hkv) * d;
  if ((q_norm_w || k_norm_w) && (d % 16 != 0 || d / 16 > 64 || ((d / 16) & (d / 16 - 1)) != 0)) return -2;
  float* x = (float*)malloc(sizeof(float) * d * 3);
  float* y = x + d;
  float* vx = x + 2 * d;
  int b = 0;
  for (int i = 0; i < num_tokens; ++i) {
    while (b < batch && i >= cu_seqlens_q[b + 1]) ++b;
    if (b >= batch) break;
    int pos = seq_lens_decoder[b] + (i - cu_seqlens_q[b]);
    if (pos < 0 || (rope_cos && pos >= max_pos)) {
      free(x);
      return -2;
    }
    const float* cs = rope_cos ? rope_cos + (size_t)pos * (d / 2) : NULL;
    const float* sn = rope_cos ? rope_sin + (size_t)pos * (d / 2) : NULL;
    const uint16_t* r = qkv + (size_t)i * row;
    for (int h = 0; h < hq; ++h) {
      epilogue_row(r + h * d, qkv_bias ? qkv_bias + h * d : NULL, q_norm_w, eps, d, rope_style, x);
      rope_row(x, y, d, cs, sn, rope_style);
      for (int c = 0; c < d; ++c) q_out[((size_t)i * hq + h) * d + c] = fdo_f32_to_bf16(y[c]);
    }
    int lb = pos / block_size, slot = pos % block_size;
    int pb = lb < max_blocks_per_seq ? block_tables[(size_t)b * max_blocks_per_seq + lb] : -1;
    if (pb >= num_blocks) {
      free(x);
      return -2;
    }
    for (int h = 0; h < hkv; ++h) {
      const uint16_t* kr = r + (size_t)(hq + h) * d;
      const uint16_t* vr = r + (size_t)(hq + hkv + h) * d;
      epilogue_row(kr, qkv_bias ? qkv_bias + (size_t)(hq + h) * d : NULL, k_norm_w, eps, d, rope_style, x);
      rope_row(x, y, d, cs, sn, rope_style);
      epilogue_row(vr, qkv_bias ? qkv_bias + (size_t)(hq + hkv + h) * d : NULL, NULL, 0.f, d, rope_style, vx);
      size_t base = (((size_t)pb * hkv + h) * block_size + slot) * d;
      int dyn = is_dynamic(cache_type);
      float dk = 1.f, dv = 1.f;
      if (dyn && pb >= 0) {
        /* the scale caches are outputs here: the writer stores the scale beside the row */
        dk = fdo_row_scale(y, d, cache_type);
        dv = fdo_row_scale(vx, d, cache_type);
        ((float*)k_scale)[((size_t)pb * hkv + h) * block_size + slot] = dk;
        ((float*)v_scale)[((size_t)pb * hkv + h) * block_size + slot] = dv;
      }
      for (int c = 0; c < d; ++c) {
        float sk = dyn ? dk : k_scale[h * d + c], sv = dyn ? dv : v_scale[h * d + c];
        float v = vx[c];
        if (k_out) k_out[((size_t)i * hkv + h) * d + c] = fdo_f32_to_bf16(y[c]);
        if (v_out) v_out[((size_t)i * hkv + h) * d + c] = fdo_f32_to_bf16(v); /* exact: v is a bf16 value */
        if (pb < 0) continue;
        if (byte_format(cache_type) == FDO_CACHE_INT8) {
          key_cache[base + c] = (uint8_t)fdo_quant_int8(y[c], sk);
          value_cache[base + c] = (uint8_t)fdo_quant_int8(v, sv);
        } else {
          key_cache[base + c] = fdo_quant_fp8(y[c], sk);
          value_cache[base + c] = fdo_quant_fp8(v, sv);
        }
      }
    }
  }
  free(x);
  return 0;
}

int fdo_write_cache_kv(const uint16_t* qkv, uint16_t* q_out, uint16_t* k_out, uint16_t* v_out,
                       uint8_t* key_cache, uint8_t* value_cache, const float* k_scale,
                       const float* v_scale, const float* rope_cos, const float* rope_sin,
                       const int32_t* block_tables, const int32_t* seq_lens_decoder,
                       const int32_t* cu_seqlens_q, int num_tokens, int batch, int hq, int hkv,
                       int d, int block_size, int max_blocks_per_seq, int num_blocks, int max_pos,
                       int rope_style, int cache_type) {
  return fdo_write_cache_kv_ex(qkv, q_out, k_out, v_out, key_cache, value_cache, k_scale, v_scale, rope_cos,
                               rope_sin, block_tables, seq_lens_decoder, cu_seqlens_q, num_tokens, batch, hq,
                               hkv, d, block_size, max_blocks_per_seq, num_blocks, max_pos, rope_style,
                               cache_type, NULL, NULL, NULL, 0.f);
}

/* ------------------------------------------------------- decode attention */

/*
 * One query row against the tokens of the logical blocks blk[0..nblk) (or all
 * blocks 0..ceil(kv_len/bs) when blk is NULL).  fp32 throughout, two passes:
 * logits and their max, then exp / sum / weighted V.
 */
static void attend_row(const float* qs /* q*k_scale, [d] */, const uint8_t* key_cache,
                       const uint8_t* value_cache, const float* v_scale /* [d] */,
                       const float* k_tok /* dynamic formats: [num_blocks,hkv,bs], else NULL */,
                       const float* v_tok, const int32_t* table, const int32_t* blk, int nblk, int kv_len, int h,
                       int hkv, int d, int bs, int cache_type, float sm_scale, float* logits,
                       float* acc, uint16_t* out) {
  cache_type = byte_format(cache_type);
  int n = 0;
  float mx = -INFINITY;
  for (int bi = 0; bi < nblk; ++bi) {
    int lb = blk ? blk[bi] : bi;
    int t0 = lb * bs, t1 = t0 + bs < kv_len ? t0 + bs : kv_len;
    const uint8_t* kp = key_cache + ((size_t)table[lb] * hkv + h) * bs * d;
    for (int t = t0; t < t1; ++t) {
      const uint8_t* kr = kp + (size_t)(t - t0) * d;
      float s = 0.f;
      if (cache_type == FDO_CACHE_INT8)
        for (int c = 0; c < d; ++c) s += qs[c] * (float)(int8_t)kr[c];
      else
        for (int c = 0; c < d; ++c) s += qs[c] * fdo_e4m3_to_f32(kr[c]);
      if (k_tok) s *= k_tok[((size_t)table[lb] * hkv + h) * bs + (t - t0)];
      s *= sm_scale;
      logits[n++] = s;
      if (s > mx) mx = s;
    }
  }
  for (int c = 0; c < d; ++c) acc[c] = 0.f;
  float l = 0.f;
  n = 0;
  for (int bi = 0; bi < nblk; ++bi) {
    int lb = blk ? blk[bi] : bi;
    int t0 = lb * bs, t1 = t0 + bs < kv_len ? t0 + bs : kv_len;
    const uint8_t* vp = value_cache + ((size_t)table[lb] * hkv + h) * bs * d;
    for (int t = t0; t < t1; ++t) {
      float p = expf(logits[n++] - mx);
      l += p;
      if (v_tok) p *= v_tok[((size_t)table[lb] * hkv + h) * bs + (t - t0)];
      const uint8_t* vr = vp + (size_t)(t - t0) * d;
      if (cache_type == FDO_CACHE_INT8)
        for (int c = 0; c < d; ++c) acc[c] += p * (float)(int8_t)vr[c];
      else
        for (int c = 0; c < d; ++c) acc[c] += p * fdo_e4m3_to_f32(vr[c]);
    }
  }
  for (int c = 0; c < d; ++c) out[c] = fdo_f32_to_bf16(n ? acc[c] * (v_tok ? 1.0f : v_scale[c]) / l : 0.f);
}

/*
 * kept_blocks == NULL: dense over [0, kv_lens[b]).  Otherwise only the logical
 * blocks kept_blocks[b,h,0..kept_counts[b,h]).
 */
int fdo_decode_attention(const uint16_t* q, const uint8_t* key_cache, const uint8_t* value_cache,
                         const float* k_scale, const float* v_scale, const int32_t* block_tables,
                         const int32_t* kv_lens, const int32_t* kept_blocks,
                         const int32_t* kept_counts, int max_kept, uint16_t* out, int batch,
                         int hq, int hkv, int d, int bs, int max_blocks_per_seq, int cache_type,
                         float sm_scale) {
  int g = hq / hkv;
#pragma omp parallel
  {
    float* logits = (float*)malloc(sizeof(float) * (size_t)max_blocks_per_seq * bs);
    float* acc = (float*)malloc(sizeof(float) * d);
    float* qs = (float*)malloc(sizeof(float) * d);
#pragma omp for schedule(dynamic, 1) collapse(2)
    for (int b = 0; b < batch; ++b)
      for (int qh = 0; qh < hq; ++qh) {
        int h = qh / g;
        int kv_len = kv_lens[b];
        const uint16_t* qr = q + ((size_t)b * hq + qh) * d;
        int dyn = is_dynamic(cache_type);
        for (int c = 0; c < d; ++c) qs[c] = fdo_bf16_to_f32(qr[c]) * (dyn ? 1.0f : k_scale[h * d + c]);
        const int32_t* blk = NULL;
        int nblk = (kv_len + bs - 1) / bs;
        if (kept_blocks) {
          blk = kept_blocks + ((size_t)b * hkv + h) * max_kept;
          nblk = kept_counts[b * hkv + h];
        }
        attend_row(qs, key_cache, value_cache, dyn ? NULL : v_scale + h * d, dyn ? k_scale : NULL,
                   dyn ? v_scale : NULL, block_tables + (size_t)b * max_blocks_per_seq, blk, nblk, kv_len, h, hkv, d,
                   bs, cache_type, sm_scale, logits, acc, out + ((size_t)b * hq + qh) * d);
      }
    free(logits);
    free(acc);
    free(qs);
  }
  return 0;
}

/* -------------------------------------------------------- split-KV combine */

int fdo_splitkv_combine(const float* part_o, const float* part_m, const float* part_l,
                        const int32_t* num_splits, uint16_t* out, int rows, int max_splits,
                        int d) {
  for (int r = 0; r < rows; ++r) {
    int ns = num_splits ? num_splits[r] : max_splits;
    float m = -INFINITY;
    for (int s = 0; s < ns; ++s)
      if (part_m[(size_t)r * max_splits + s] > m) m = part_m[(size_t)r * max_splits + s];
    float l = 0.f;
    for (int s = 0; s < ns; ++s) {
      float ms = part_m[(size_t)r * max_splits + s];
      if (ms > -INFINITY) l += part_l[(size_t)r * max_splits + s] * expf(ms - m);
    }
    for (int c = 0; c < d; ++c) {
      float o = 0.f;
      for (int s = 0; s < ns; ++s) {
        float ms = part_m[(size_t)r * max_splits + s];
        if (ms > -INFINITY) o += part_o[((size_t)r * max_splits + s) * d + c] * expf(ms - m);
      }
      out[(size_t)r * d + c] = fdo_f32_to_bf16(l > 0.f ? o / l : 0.f);
    }
  }
  return 0;
}

/* --------------------------------------------------------- SQAttn selector */

/*
 * score[b,h,j] = max_{t in block j, t < kv_len} max_{g in group h}
 *                sum_c (double)(float)(q[b,g,c] * k_scale[h,c]) * (double)K8[t,c]
 * summed over c = 0..d-1 in that order in fp64.  The fp32 product q*scale is a
 * single rounding; K8 (an int8 integer or an e4m3 value) is exact in fp64, and
 * so is every product (24 + 8 significant bits).  Blocks past the sequence get
 * -inf.  Dynamic formats (k_scale = the scale cache [num_blocks, hkv, bs]): q enters
 * unscaled and the token's sum is multiplied by its row's scale at the end, one more
 * fp64 rounding:  (double)k_scale[row of t] * sum_c (double)q[b,g,c] * (double)K8[t,c].
 */
int fdo_sqattn_block_scores(const uint16_t* q, const uint8_t* key_cache, const float* k_scale,
                            const int32_t* block_tables, const int32_t* kv_lens, double* scores,
                            int batch, int hq, int hkv, int d, int bs, int max_blocks_per_seq,
                            int cache_type) {
  int g = hq / hkv;
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
  for (int b = 0; b < batch; ++b)
    for (int h = 0; h < hkv; ++h) {
      double* qs = (double*)malloc(sizeof(double) * g * d);
      for (int gi = 0; gi < g; ++gi)
        for (int c = 0; c < d; ++c) {
          float f = fdo_bf16_to_f32(q[((size_t)b * hq + h * g + gi) * d + c]);
          if (!is_dynamic(cache_type)) f = f * k_scale[h * d + c];
          qs[gi * d + c] = (double)f;
        }
      int kv_len = kv_lens[b];
      for (int j = 0; j < max_blocks_per_seq; ++j) {
        double best = -INFINITY;
        int t0 = j * bs, t1 = t0 + bs < kv_len ? t0 + bs : kv_len;
        if (t0 < kv_len) {
          size_t tile = (size_t)block_tables[(size_t)b * max_blocks_per_seq + j] * hkv + h;
          const uint8_t* kp = key_cache + tile * bs * d;
          for (int t = t0; t < t1; ++t)
            for (int gi = 0; gi < g; ++gi) {
              double s = 0.0;
              for (int c = 0; c < d; ++c)
                s += qs[gi * d + c] * (double)dequant(kp[(size_t)(t - t0) * d + c], cache_type);
              if (is_dynamic(cache_type)) s = s * (double)k_scale[tile * bs + (t - t0)];
              if (s > best) best = s;
            }
        }
        scores[((size_t)b * hkv + h) * max_blocks_per_seq + j] = best;
      }
      free(qs);
    }
  return 0;
}

/*
 * k passes of arg-max with strict '>' scanning ascending index, so that equal
 * scores resolve to the lowest index (fastdeploy/vision/utils/utils.h:41-60),
 * then the kept indices are emitted in ascending order.
 */
int fdo_topk_select(const double* scores, const int32_t* kv_lens, int32_t* kept_blocks,
                    int32_t* kept_counts, int batch, int hkv, int bs, int max_blocks_per_seq,
                    int top_k) {
  char* taken = (char*)malloc(max_blocks_per_seq);
  for (int b = 0; b < batch; ++b)
    for (int h = 0; h < hkv; ++h) {
      const double* s = scores + ((size_t)b * hkv + h) * max_blocks_per_seq;
      int nblk = (kv_lens[b] + bs - 1) / bs;
      if (nblk > max_blocks_per_seq) nblk = max_blocks_per_seq;
      int k = top_k < nblk ? top_k : nblk;
      memset(taken, 0, max_blocks_per_seq);
      for (int i = 0; i < k; ++i) {
        int best = -1;
        for (int j = 0; j < nblk; ++j) {
          if (taken[j]) continue;
          if (best < 0 || s[j] > s[best]) best = j;
        }
        taken[best] = 1;
      }
      int32_t* o = kept_blocks + ((size_t)b * hkv + h) * top_k;
      int n = 0;
      for (int j = 0; j < nblk; ++j)
        if (taken[j]) o[n++] = j;
      for (int j = n; j < top_k; ++j) o[j] = -1;
      kept_counts[b * hkv + h] = k;
    }
  free(taken);
  return 0;
}

/* ------------------------------------------------ chunked-prefill attention */

/*
 * New token i of sequence b (chunk offset ci) attends to the p_b cached tokens
 * (dequantised pages) and to chunk tokens 0..ci (bf16 k_new / v_new).
 * token_ids (optional) restricts the computed rows to the listed global token
 * indices; the other rows of out are left untouched.
 */
int fdo_append_attention_prefill(const uint16_t* q, const uint16_t* k_new, const uint16_t* v_new,
                                 const uint8_t* key_cache, const uint8_t* value_cache,
                                 const float* k_scale, const float* v_scale,
                                 const int32_t* block_tables, const int32_t* seq_lens_decoder,
                                 const int32_t* cu_seqlens_q, uint16_t* out,
                                 const int32_t* token_ids, int n_ids, int num_tokens, int batch,
                                 int hq, int hkv, int d, int bs, int max_blocks_per_seq,
                                 int cache_type, float sm_scale) {
  int g = hq / hkv;
  int nrows = token_ids ? n_ids : num_tokens;
  int max_len = 0;
  for (int b = 0; b < batch; ++b) {
    int len = seq_lens_decoder[b] + cu_seqlens_q[b + 1] - cu_seqlens_q[b];
    if (len > max_len) max_len = len;
  }
#pragma omp parallel
  {
    float* logits = (float*)malloc(sizeof(float) * (size_t)(max_len + 1));
    float* acc = (float*)malloc(sizeof(float) * d);
    float* qf = (float*)malloc(sizeof(float) * d);
#pragma omp for schedule(dynamic, 1) collapse(2)
    for (int r = 0; r < nrows; ++r)
      for (int qh = 0; qh < hq; ++qh) {
        int i = token_ids ? token_ids[r] : r;
        int b = 0;
        while (b < batch - 1 && i >= cu_seqlens_q[b + 1]) ++b;
        int ci = i - cu_seqlens_q[b], p = seq_lens_decoder[b], h = qh / g;
        const int32_t* table = block_tables + (size_t)b * max_blocks_per_seq;
        const uint16_t* qr = q + ((size_t)i * hq + qh) * d;
        for (int c = 0; c < d; ++c) qf[c] = fdo_bf16_to_f32(qr[c]);
        float mx = -INFINITY;
        for (int t = 0; t < p; ++t) {
          const uint8_t* kr =
              key_cache + (((size_t)table[t / bs] * hkv + h) * bs + t % bs) * d;
          float s = 0.f;
          if (is_dynamic(cache_type)) {
            for (int c = 0; c < d; ++c) s += qf[c] * dequant(kr[c], cache_type);
            s *= k_scale[((size_t)table[t / bs] * hkv + h) * bs + t % bs];
          } else {
            for (int c = 0; c < d; ++c) s += qf[c] * (dequant(kr[c], cache_type) * k_scale[h * d + c]);
          }
          s *= sm_scale;
          logits[t] = s;
          if (s > mx) mx = s;
        }
        for (int j = 0; j <= ci; ++j) {
          const uint16_t* kr = k_new + ((size_t)(cu_seqlens_q[b] + j) * hkv + h) * d;
          float s = 0.f;
          for (int c = 0; c < d; ++c) s += qf[c] * fdo_bf16_to_f32(kr[c]);
          s *= sm_scale;
          logits[p + j] = s;
          if (s > mx) mx = s;
        }
        for (int c = 0; c < d; ++c) acc[c] = 0.f;
        float l = 0.f;
        for (int t = 0; t < p; ++t) {
          const uint8_t* vr =
              value_cache + (((size_t)table[t / bs] * hkv + h) * bs + t % bs) * d;
          float pr = expf(logits[t] - mx);
          l += pr;
          if (is_dynamic(cache_type)) {
            float pv = pr * v_scale[((size_t)table[t / bs] * hkv + h) * bs + t % bs];
            for (int c = 0; c < d; ++c) acc[c] += pv * dequant(vr[c], cache_type);
          } else {
            for (int c = 0; c < d; ++c) acc[c] += pr * (dequant(vr[c], cache_type) * v_scale[h * d + c]);
          }
        }
        for (int j = 0; j <= ci; ++j) {
          const uint16_t* vr = v_new + ((size_t)(cu_seqlens_q[b] + j) * hkv + h) * d;
          float pr = expf(logits[p + j] - mx);
          l += pr;
          for (int c = 0; c < d; ++c) acc[c] += pr * fdo_bf16_to_f32(vr[c]);
        }
        uint16_t* o = out + ((size_t)i * hq + qh) * d;
        for (int c = 0; c < d; ++c) o[c] = fdo_f32_to_bf16(acc[c] / l);
      }
    free(logits);
    free(acc);
    free(qf);
  }
  return 0;
}

/* softmax of one row, the primitive the attention functions above inline */
void fdo_softmax_row(const float* x, float* y, int n) {
  float mx = -INFINITY, l = 0.f;
  for (int i = 0; i < n; ++i)
    if (x[i] > mx) mx = x[i];
  for (int i = 0; i < n; ++i) {
    y[i] = expf(x[i] - mx);
    l += y[i];
  }
  for (int i = 0; i < n; ++i) y[i] /= l;
}
