/*
 * CPU oracle for the quantized linear-layer path: TEST INFRASTRUCTURE ONLY
 * (see oracle.h for what pins each function). Build: make -C oracle.
 * Compiled with -ffp-contract=off so every float step rounds on its own.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static uint32_t bits_of(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static float float_of(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint16_t load_u16(const uint8_t* p) {
  uint16_t v;
  memcpy(&v, p, 2);
  return v;
}

static void store_u16(uint8_t* p, uint16_t v) { memcpy(p, &v, 2); }

int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------ conversions */

/* decode.cc:341-353 */
float orc_f16_to_f32(uint16_t bits) {
  const float sign = (bits & 0x8000u) ? -1.0f : 1.0f;
  const unsigned exponent = (bits >> 10) & 31u;
  const unsigned mantissa = bits & 1023u;
  if (exponent == 31) return mantissa ? NAN : sign * INFINITY;
  if (exponent == 0) return sign * ldexpf((float)mantissa, -24);
  return sign * ldexpf((float)(1024u + mantissa), (int)exponent - 25);
}

/* decode.cc:355-382 */
uint16_t orc_f32_to_f16(float value) {
  const uint32_t x = bits_of(value);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t magnitude = x & 0x7FFFFFFFu;
  if (magnitude >= 0x7F800000u) return (uint16_t)(sign | (magnitude > 0x7F800000u ? 0x7E00u : 0x7C00u));
  if (magnitude >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);
  if (magnitude < 0x38800000u) {
    const uint32_t exponent = magnitude >> 23;
    const uint32_t shift = 126u - exponent;
    if (exponent == 0 || shift > 24) return sign;
    const uint32_t significand = (magnitude & 0x7FFFFFu) | 0x800000u;
    uint32_t q = significand >> shift;
    const uint32_t rest = significand & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1u);
    if (rest > half || (rest == half && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
  }
  const uint32_t rounded = magnitude + 0xFFFu + ((magnitude >> 13) & 1u);
  return (uint16_t)(sign | ((rounded - 0x38000000u) >> 13));
}

/* decode.cc:384-392 */
float orc_bf16_to_f32(uint16_t bits) { return float_of((uint32_t)bits << 16); }
uint16_t orc_f32_to_bf16(float value) {
  const uint32_t x = bits_of(value);
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
  return (uint16_t)((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}

/* decode.cc:394-405 */
float orc_e4m3_to_f32(uint8_t bits) {
  const float sign = (bits & 0x80u) ? -1.0f : 1.0f;
  const unsigned exponent = (bits >> 3) & 15u;
  const unsigned mantissa = bits & 7u;
  if (exponent == 15 && mantissa == 7) return NAN;
  if (exponent == 0) return sign * ldexpf((float)mantissa, -9);
  return sign * ldexpf((float)(8u + mantissa), (int)exponent - 10);
}

/* decode.cc:417-422 */
float orc_e8m0_to_f32(uint8_t bits) {
  if (bits == 0xFF) return NAN;
  return ldexpf(1.0f, (int)bits - 127);
}

/* OCP E4M3 from float: nearest, ties to even, saturating to +-448; NaN -> 0x7F. */
uint8_t orc_f32_to_e4m3(float value) {
  const uint8_t sign = (bits_of(value) >> 31) ? 0x80u : 0u;
  if (isnan(value)) return (uint8_t)(sign | 0x7Fu);
  const float a = fabsf(value);
  if (a > 448.0f) return (uint8_t)(sign | 0x7Eu);
  if (a < 0.015625f) { /* below 2^-6: units of 2^-9 */
    const int q = (int)nearbyintf(a * 512.0f);
    return (uint8_t)(sign | (uint8_t)q); /* q == 8 is the least normal's encoding */
  }
  int e;
  (void)frexpf(a, &e); /* a = m * 2^e, m in [0.5, 1) */
  int exponent = e - 1;
  int q = (int)nearbyintf(ldexpf(a, 3 - exponent)); /* in [8, 16] */
  if (q == 16) {
    q = 8;
    ++exponent;
  }
  return (uint8_t)(sign | ((unsigned)(exponent + 7) << 3) | (unsigned)(q - 8));
}

/* ------------------------------------------------------------------ Q8_1 */

/* The 32 lanes' xor-butterfly sum, offsets 16, 8, 4, 2, 1 (a warp reduction's order). */
static float butterfly32(const float* x) {
  float a[32];
  memcpy(a, x, sizeof(a));
  for (int h = 16; h >= 1; h /= 2)
    for (int i = 0; i < h; ++i) a[i] = a[i] + a[i + h];
  return a[0];
}

void orc_q8_1_quantize_row(const float* x, int64_t k, int64_t padded_k, uint8_t* out, int flavor) {
  for (int64_t b = 0; b < padded_k / 32; ++b) {
    uint8_t* blk = out + b * 36;
    float v[32];
    for (int j = 0; j < 32; ++j) {
      const int64_t i = b * 32 + j;
      v[j] = i < k ? x[i] : 0.0f;
    }
    float amax = 0.0f;
    for (int j = 0; j < 32; ++j) {
      const float a = fabsf(v[j]);
      amax = amax > a ? amax : a;
    }
    const float d = amax / 127.0f;
    int8_t q[32];
    uint16_t s16;
    if (flavor == ORC_Q8_GGML_CPU) {
      /* kv_quant.cuh:35-42 (d, id, codes); s = d * sum(q) as ggml's quantize_row_q8_1_ref. */
      const float id = d != 0.0f ? 1.0f / d : 0.0f;
      int sum = 0;
      for (int j = 0; j < 32; ++j) {
        q[j] = (int8_t)roundf(v[j] * id);
        sum += q[j];
      }
      s16 = orc_f32_to_f16((float)sum * d);
    } else {
      /* llmp_moe.cu:521-536 without fast math: q = roundf(x / d), 0 for a zero block. */
      for (int j = 0; j < 32; ++j) q[j] = amax == 0.0f ? 0 : (int8_t)roundf(v[j] / d);
      s16 = orc_f32_to_f16(butterfly32(v));
    }
    const uint16_t d16 = orc_f32_to_f16(d);
    memcpy(blk, &d16, 2);
    memcpy(blk + 2, &s16, 2);
    memcpy(blk + 4, q, 32);
  }
}

void orc_q8_1_decode_row(const uint8_t* blocks, int64_t k, float* y) {
  for (int64_t b = 0; b < k / 32; ++b) {
    const uint8_t* x = blocks + b * 36;
    const float d = orc_f16_to_f32(load_u16(x));
    for (int j = 0; j < 32; ++j) y[b * 32 + j] = d * (float)(int8_t)x[4 + j];
  }
}

/* ------------------------------------------------ KV cache block quantizers */

/* src/kernels/ggml/kv_quant.cuh:27-43 (quantize_row_q8_0_ref step by step). */
static void kv_q8_0_block(const float* x, uint8_t* out) {
  float amax = 0.0f;
  for (int j = 0; j < 32; ++j) {
    const float v = fabsf(x[j]);
    amax = amax > v ? amax : v;
  }
  const float d = amax / 127.0f;
  const float id = d != 0.0f ? 1.0f / d : 0.0f;
  store_u16(out, orc_f32_to_f16(d));
  for (int j = 0; j < 32; ++j) out[2 + j] = (uint8_t)(int8_t)roundf(x[j] * id);
}

/* kv_quant.cuh:45-69 (quantize_row_q4_0_ref step by step). */
static void kv_q4_0_block(const float* x, uint8_t* out) {
  float amax = 0.0f, vmax = 0.0f;
  for (int j = 0; j < 32; ++j) {
    const float v = x[j];
    if (amax < fabsf(v)) {
      amax = fabsf(v);
      vmax = v;
    }
  }
  const float d = vmax / -8.0f;
  const float id = d != 0.0f ? 1.0f / d : 0.0f;
  store_u16(out, orc_f32_to_f16(d));
  for (int j = 0; j < 16; ++j) {
    const float x0 = x[j] * id;
    const float x1 = x[16 + j] * id;
    int xi0 = (int)(int8_t)(x0 + 8.5f);
    int xi1 = (int)(int8_t)(x1 + 8.5f);
    if (xi0 > 15) xi0 = 15;
    if (xi1 > 15) xi1 = 15;
    out[2 + j] = (uint8_t)(xi0 | (xi1 << 4));
  }
}

void orc_kv_quantize_row(int type, const float* x, int64_t k, uint8_t* out) {
  for (int64_t b = 0; b < k / 32; ++b) {
    if (type == ORC_TYPE_Q8_0) {
      kv_q8_0_block(x + b * 32, out + b * 34);
    } else {
      kv_q4_0_block(x + b * 32, out + b * 18);
    }
  }
}

/* --------------------------------------------------------- weight blocks */

/* src/format/encoding.cc:110-116; the legacy blocks as tests/unit/dsv4_fast_test.cc:141-157 reads
 * them: {f16 d; [f16 m;] [u32 high bits;] u8 nibbles[16]}. */
int orc_block_bytes(int type) {
  switch (type) {
    case ORC_TYPE_Q4_0: return 18;
    case ORC_TYPE_Q4_1: return 20;
    case ORC_TYPE_Q5_0: return 22;
    case ORC_TYPE_Q5_1: return 24;
    case ORC_TYPE_Q8_0: return 34;
    case ORC_TYPE_Q4_K: return 144;
    case ORC_TYPE_Q6_K: return 210; /* encoding.cc:117: {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d} */
    case ORC_TYPE_Q5_K: return 176; /* encoding.cc:116: {f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]} */
    case ORC_TYPE_MXFP4: return 17; /* encoding.cc:130-138 */
    case ORC_TYPE_IQ4_NL: return 18; /* {f16 d; u8 nibbles[16]}: Q4_0's bytes */
    default: return 0;
  }
}
int orc_block_elements(int type) { return type == ORC_TYPE_Q4_K || type == ORC_TYPE_Q5_K || type == ORC_TYPE_Q6_K ? 256 : orc_block_bytes(type) != 0 ? 32 : 0; }

static int legacy_affine(int type) { return type == ORC_TYPE_Q4_1 || type == ORC_TYPE_Q5_1; }
static int legacy_five(int type) { return type == ORC_TYPE_Q5_0 || type == ORC_TYPE_Q5_1; }
static int legacy(int type) {
  return type == ORC_TYPE_Q4_0 || type == ORC_TYPE_Q4_1 || type == ORC_TYPE_Q5_0 || type == ORC_TYPE_Q5_1;
}
/* Code i of a legacy block: dsv4_fast_test.cc:149-158. */
static int legacy_code(int type, const uint8_t* w, int i) {
  const int prefix = legacy_affine(type) ? 4 : 2;
  uint32_t high = 0;
  if (legacy_five(type)) memcpy(&high, w + prefix, 4);
  const uint8_t* codes = w + prefix + (legacy_five(type) ? 4 : 0);
  const int low = i < 16 ? codes[i] & 15 : codes[i - 16] >> 4;
  return low + (legacy_five(type) ? (int)((high >> i) & 1u) * 16 : 0);
}

/* Q6_K (src/kernels/ggml/vecq.cu:76-77 of the reference reads it through ggml's vec_dot_q6_K_q8_1, which is not
 * vendored: ggml-quants.c of llama.cpp d812350, dequantize_row_q6_K, restated): value v = 128 h + 32 t + l of a block is
 * nibble t / 2 of ql[64 h + 32 (t % 2) + l] plus 16 times bits 2t, 2t + 1 of qh[32 h + l], minus 32; it is scaled by
 * scales[v / 16] (int8) and d. Parity unpinned: the reference holds no vector for this type. */
static int q6_k_value(const uint8_t* w, int v) {
  const int h = v / 128, t = (v % 128) / 32, l = v % 32;
  const int low = w[64 * h + 32 * (t % 2) + l];
  const int nibble = t / 2 ? low >> 4 : low & 15;
  return (nibble | (((w[128 + 32 * h + l] >> (2 * t)) & 3) << 4)) - 32;
}

/* IQ4_NL (src/kernels/ggml/vecq.cu:375-396 of the reference reads it through ggml's
 * kvalues_iq4nl, which is not vendored: ggml-common.h of llama.cpp d812350, restated): code i of a
 * block is the low (i < 16) or high nibble of byte 2 + i % 16, its value the codebook's entry, the
 * block's values d times those. Parity unpinned: the reference holds no vector for this type. */
static const int8_t iq4_nl_values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
static int iq4_nl_value(const uint8_t* w, int i) { return iq4_nl_values[i < 16 ? w[2 + i] & 15 : w[2 + i - 16] >> 4]; }

/* decode.cc:424-428: the E2M1 value of a four-bit code. */
float orc_e2m1_to_f32(uint8_t code) {
  static const float values[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
  const float v = values[code & 7u];
  return (code & 8u) ? -v : v;
}
/* Code i of a block_mxfp4 {e8m0 e; u8 qs[16]}: byte j holds values j (low nibble) and j + 16
 * (decode.cc:239-248). */
static int mxfp4_code(const uint8_t* w, int i) { return i < 16 ? w[1 + i] & 15 : w[1 + i - 16] >> 4; }
/* Twice the E2M1 value, an integer (the table vecq.cu:424 looks codes up in). */
static int mxfp4_twice(int code) { return (int)(2.0f * orc_e2m1_to_f32((uint8_t)code)); }

/* dsv4_fast_test.cc:180-183 */
void orc_q4_k_scale_min(const uint8_t* scales, int g, int* scale, int* minimum) {
  *scale = g < 4 ? scales[g] & 63 : (scales[g + 4] & 15) | ((scales[g - 4] >> 6) << 4);
  *minimum = g < 4 ? scales[g + 4] & 63 : (scales[g + 4] >> 4) | ((scales[g] >> 6) << 4);
}

static int q4_k_code(const uint8_t* codes, int g, int i) {
  return (codes[(g / 2) * 32 + i] >> ((g % 2) * 4)) & 15; /* dsv4_fast_test.cc:187 */
}
/* Q5_K (src/kernels/ggml/vecq.cu:74-75 of the reference reads it through ggml's vec_dot_q5_K_q8_1, which is
 * not vendored: ggml-quants.c of llama.cpp d812350, dequantize_row_q5_K, restated): Q4_K's header and
 * nibbles, plus bit g of byte i of qh as the fifth bit of value i of sub-block g. Parity unpinned: the
 * reference holds no vector for this type. The codes of a block of either type: */
static int k_code(int type, const uint8_t* w, int g, int i) {
  if (type == ORC_TYPE_Q5_K) return q4_k_code(w + 48, g, i) + 16 * ((w[16 + i] >> g) & 1);
  return q4_k_code(w + 16, g, i);
}

void orc_decode_row(int type, const uint8_t* row, int64_t k, float* y) {
  if (type == ORC_TYPE_MXFP4) { /* decode.cc:239-248 */
    for (int64_t j = 0; j < k; ++j) {
      const uint8_t* x = row + j / 32 * 17;
      y[j] = orc_e2m1_to_f32((uint8_t)mxfp4_code(x, (int)(j % 32))) * orc_e8m0_to_f32(x[0]);
    }
    return;
  }
  if (type == ORC_TYPE_Q6_K) {
    for (int64_t j = 0; j < k; ++j) {
      const uint8_t* x = row + j / 256 * 210;
      const int v = (int)(j % 256);
      y[j] = orc_f16_to_f32(load_u16(x + 208)) * (float)(int8_t)x[192 + v / 16] * (float)q6_k_value(x, v);
    }
    return;
  }
  if (type == ORC_TYPE_IQ4_NL) {
    for (int64_t j = 0; j < k; ++j) {
      const uint8_t* x = row + j / 32 * 18;
      y[j] = orc_f16_to_f32(load_u16(x)) * (float)iq4_nl_value(x, (int)(j % 32));
    }
    return;
  }
  if (legacy(type)) {
    /* ggml's dequantization of these bytes: d * (code - 8 or 16), or d * code + m. */
    const int bs = orc_block_bytes(type);
    for (int64_t b = 0; b < k / 32; ++b) {
      const uint8_t* x = row + b * bs;
      const float d = orc_f16_to_f32(load_u16(x));
      const float m = legacy_affine(type) ? orc_f16_to_f32(load_u16(x + 2)) : 0.0f;
      const int offset = legacy_affine(type) ? 0 : legacy_five(type) ? 16 : 8;
      for (int j = 0; j < 32; ++j) y[b * 32 + j] = d * (float)(legacy_code(type, x, j) - offset) + m;
    }
    return;
  }
  if (type == ORC_TYPE_Q8_0) {
    for (int64_t b = 0; b < k / 32; ++b) {
      const uint8_t* x = row + b * 34;
      const float d = orc_f16_to_f32(load_u16(x));
      for (int j = 0; j < 32; ++j) y[b * 32 + j] = d * (float)(int8_t)x[2 + j];
    }
    return;
  }
  /* Q4_K, Q5_K: y = d * sc * code - dmin * m (ggml's dequantize_row_q4_K, _q5_K of these bytes). */
  for (int64_t b = 0; b < k / 256; ++b) {
    const uint8_t* x = row + b * orc_block_bytes(type);
    const float d = orc_f16_to_f32(load_u16(x));
    const float dmin = orc_f16_to_f32(load_u16(x + 2));
    for (int g = 0; g < 8; ++g) {
      int sc, m;
      orc_q4_k_scale_min(x + 4, g, &sc, &m);
      const float d1 = d * (float)sc;
      const float m1 = dmin * (float)m;
      for (int i = 0; i < 32; ++i) y[b * 256 + g * 32 + i] = d1 * (float)k_code(type, x, g, i) - m1;
    }
  }
}

void orc_block_sums(int type, const uint8_t* w, const uint8_t* q8, int32_t* sums) {
  if (type == ORC_TYPE_MXFP4) { /* vecq.cu:421-435: the doubled values times the codes */
    int32_t s = 0;
    for (int i = 0; i < 32; ++i) s += mxfp4_twice(mxfp4_code(w, i)) * (int32_t)(int8_t)q8[4 + i];
    sums[0] = s;
    return;
  }
  if (type == ORC_TYPE_Q6_K) { /* the sixteen sub-blocks' sums of value times code */
    for (int j = 0; j < 16; ++j) {
      int32_t s = 0;
      for (int i = 0; i < 16; ++i) s += q6_k_value(w, 16 * j + i) * (int32_t)(int8_t)q8[(j / 2) * 36 + 4 + (j % 2) * 16 + i];
      sums[j] = s;
    }
    return;
  }
  if (type == ORC_TYPE_IQ4_NL) { /* vecq.cu:379-392: the codebook's values times the codes */
    int32_t s = 0;
    for (int i = 0; i < 32; ++i) s += iq4_nl_value(w, i) * (int32_t)(int8_t)q8[4 + i];
    sums[0] = s;
    return;
  }
  if (legacy(type)) { /* dsv4_fast_test.cc:154-158 */
    int32_t s = 0;
    for (int i = 0; i < 32; ++i) s += legacy_code(type, w, i) * (int32_t)(int8_t)q8[4 + i];
    sums[0] = s;
    return;
  }
  if (type == ORC_TYPE_Q8_0) {
    int32_t s = 0;
    for (int i = 0; i < 32; ++i) s += (int32_t)(int8_t)w[2 + i] * (int32_t)(int8_t)q8[4 + i];
    sums[0] = s;
    return;
  }
  for (int g = 0; g < 8; ++g) {
    const uint8_t* a = q8 + g * 36;
    int32_t product = 0, sum = 0;
    for (int i = 0; i < 32; ++i) {
      const int value = (int8_t)a[4 + i];
      product += k_code(type, w, g, i) * value;
      sum += value;
    }
    sums[g] = product;
    sums[8 + g] = sum;
  }
}

double orc_block_product(int type, const uint8_t* w, const uint8_t* q8) {
  int32_t sums[16];
  orc_block_sums(type, w, q8, sums);
  if (type == ORC_TYPE_MXFP4) { /* vecq.cu:426,437: half the block's scale, times d8, times the sum */
    return (double)orc_e8m0_to_f32(w[0]) * 0.5 * (double)orc_f16_to_f32(load_u16(q8)) * (double)sums[0];
  }
  if (type == ORC_TYPE_Q6_K) { /* d * sum over the eight activation blocks of d8 * (sc * sum, both sub-blocks) */
    double total = 0;
    for (int b = 0; b < 8; ++b) {
      const double d8 = orc_f16_to_f32(load_u16(q8 + b * 36));
      total += d8 * ((double)(int8_t)w[192 + 2 * b] * sums[2 * b] + (double)(int8_t)w[192 + 2 * b + 1] * sums[2 * b + 1]);
    }
    return (double)orc_f16_to_f32(load_u16(w + 208)) * total;
  }
  if (type == ORC_TYPE_IQ4_NL) { /* vecq.cu:394-395: dw * d8, times the sum */
    return (double)orc_f16_to_f32(load_u16(w)) * (double)orc_f16_to_f32(load_u16(q8)) * (double)sums[0];
  }
  if (legacy(type)) { /* dsv4_fast_test.cc:145-164: the Q8_1 block's s is the rounded sum of its inputs */
    const float dw = orc_f16_to_f32(load_u16(w));
    const float da = orc_f16_to_f32(load_u16(q8));
    const float sa = orc_f16_to_f32(load_u16(q8 + 2));
    if (legacy_affine(type)) {
      const float scale = orc_f16_to_f32(orc_f32_to_f16(dw * da));
      const float minimum = orc_f16_to_f32(orc_f32_to_f16(orc_f16_to_f32(load_u16(w + 2)) * sa));
      return (double)sums[0] * scale + minimum;
    }
    return (double)dw * ((double)sums[0] * da - (legacy_five(type) ? 16.0 : 8.0) * sa);
  }
  if (type == ORC_TYPE_Q8_0) {
    /* vecq.cu:415-416: d8_0 * d8_1 * sumi */
    return (double)orc_f16_to_f32(load_u16(w)) * (double)orc_f16_to_f32(load_u16(q8)) * (double)sums[0];
  }
  /* dsv4_fast_test.cc:179-193 */
  const double d = orc_f16_to_f32(load_u16(w));
  const double dmin = orc_f16_to_f32(load_u16(w + 2));
  double total = 0;
  for (int g = 0; g < 8; ++g) {
    int sc, m;
    orc_q4_k_scale_min(w + 4, g, &sc, &m);
    const double d8 = orc_f16_to_f32(load_u16(q8 + g * 36));
    total += d8 * (d * sc * sums[g] - dmin * m * sums[8 + g]);
  }
  return total;
}

/* -------------------------------------------------------- decode products */

/* decode.cc:407-411 */
float orc_ue4m3_to_f32(uint8_t bits) { return bits < 0x7Fu ? orc_e4m3_to_f32(bits) : NAN; }

/* The E2M1 code j of a row of adjacent nibbles (decode.cc:86-91: value 2i in byte i's low nibble). */
static float fp4_at(const uint8_t* codes, uint64_t j) {
  const uint8_t b = codes[j / 2];
  return orc_e2m1_to_f32((uint8_t)((j % 2) ? b >> 4 : b & 15));
}

float orc_decode_value(int decoder, const orc_decode_operand* w, uint64_t row, uint64_t j) {
  const uint8_t* data = w->data + row * w->row_bytes;
  const uint64_t k = w->k;
  switch (decoder) {
    case ORC_DECODER_BF16_DENSE: /* decode.cc:52 */
      return orc_bf16_to_f32(load_u16(data + 2 * j));
    case ORC_DECODER_F16_DENSE:
      return orc_f16_to_f32(load_u16(data + 2 * j));
    case ORC_DECODER_Q8_0_BLOCKS: { /* d * q, ggml's dequantization of these bytes */
      const uint8_t* block = data + j / 32 * 34;
      return orc_f16_to_f32(load_u16(block)) * (float)(int8_t)block[2 + j % 32];
    }
    case ORC_DECODER_NVFP4_SPLIT: /* decode.cc:296-317 */
      return fp4_at(data, j) * orc_ue4m3_to_f32(w->scales[row * (k / 16) + j / 16]);
    case ORC_DECODER_NVFP4_ATOMS:
      return fp4_at(data, j) * orc_ue4m3_to_f32(w->scales[orc_scale_atom_offset(row, j / 16, k / 16)]);
    case ORC_DECODER_NVFP4_INTERLEAVED: /* decode.cc:300-304: a row's codes, then its scales */
      return fp4_at(data, j) * orc_ue4m3_to_f32(data[k / 2 + j / 16]);
    case ORC_DECODER_NVFP4_GGML_BLOCKS: { /* decode.cc:260-272 */
      const uint8_t* x = data + j / 64 * 36;
      const uint64_t sub = (j % 64) / 16, t = j % 16;
      const uint8_t b = x[4 + sub * 8 + t % 8];
      return orc_e2m1_to_f32((uint8_t)(t >= 8 ? b >> 4 : b & 15)) * orc_ue4m3_to_f32(x[sub]);
    }
    case ORC_DECODER_MXFP8_SPLIT:
      return orc_e4m3_to_f32(data[j]) * orc_e8m0_to_f32(w->scales[row * (k / 32) + j / 32]);
    case ORC_DECODER_MXFP8_ATOMS:
      return orc_e4m3_to_f32(data[j]) * orc_e8m0_to_f32(w->scales[orc_scale_atom_offset(row, j / 32, k / 32)]);
    case ORC_DECODER_MXFP4_SPLIT:
      return fp4_at(data, j) * orc_e8m0_to_f32(w->scales[row * (k / 32) + j / 32]);
    case ORC_DECODER_MXFP4_ATOMS:
      return fp4_at(data, j) * orc_e8m0_to_f32(w->scales[orc_scale_atom_offset(row, j / 32, k / 32)]);
    case ORC_DECODER_AFFINE_SPLIT: { /* decode.cc:173-220: s * q + b rounded once, or s * (q - z) */
      const uint64_t g = j / w->group, groups = k / w->group;
      const int element = w->scale_type & 0x7F; /* 1 F16, 2 BF16, 3 F32 (operand.h:96) */
      const uint8_t* srow = w->scales + row * w->scale_row_bytes;
      float sc, b = 0.0f;
      uint32_t q = 0, z = 0;
      for (uint32_t i = 0; i < w->bits; ++i) {
        const uint64_t bit = j * w->bits + i;
        q |= (uint32_t)((data[bit / 8] >> (bit % 8)) & 1u) << i;
      }
      if (element == 3) memcpy(&sc, srow + 4 * g, 4);
      else sc = element == 2 ? orc_bf16_to_f32(load_u16(srow + 2 * g)) : orc_f16_to_f32(load_u16(srow + 2 * g));
      if (w->scale_type & 0x80) {
        const uint8_t* zeros = w->biases + row * ((groups * w->bits + 7) / 8);
        for (uint32_t i = 0; i < w->bits; ++i) {
          const uint64_t bit = g * w->bits + i;
          z |= (uint32_t)((zeros[bit / 8] >> (bit % 8)) & 1u) << i;
        }
        return sc * (float)((int32_t)q - (int32_t)z);
      }
      if (w->biases != NULL) {
        const uint8_t* brow = w->biases + row * w->scale_row_bytes;
        if (element == 3) memcpy(&b, brow + 4 * g, 4);
        else b = element == 2 ? orc_bf16_to_f32(load_u16(brow + 2 * g)) : orc_f16_to_f32(load_u16(brow + 2 * g));
      }
      return fmaf(sc, (float)q, b);
    }
    default:
      return NAN;
  }
}

int orc_decode_vector(int decoder, const orc_decode_operand* w, uint64_t first, uint64_t outputs, const float* x,
                      uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride, int threads) {
  if (decoder < 0 || decoder > ORC_DECODER_AFFINE_SPLIT) return 1;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t j = 0; j < (int64_t)outputs; ++j) {
    const uint64_t row = first + (uint64_t)j;
    const double scale = w->tensor_scale != NULL ? (double)w->tensor_scale[row / w->rows_per_scale] : 1.0;
    for (uint64_t t = 0; t < rows; ++t) {
      double sum = 0;
      for (uint64_t c = 0; c < w->k; ++c) sum += (double)orc_decode_value(decoder, w, row, c) * (double)x[t * x_stride + c];
      y[t * y_stride + (uint64_t)j] = (float)(sum * scale);
    }
  }
  return 0;
}

/* exec.cc:248-262 with ir::GluKind's numbering (src/ir/op.h:455): SwiGLU 0, GeGLU (erf) 1, GeGLU (tanh) 2, SwiGLU
 * with a clamp 3. */
static double decode_glu(int kind, double g, double u, double limit) {
  switch (kind) {
    case 1: return 0.5 * g * (1.0 + erf(g / sqrt(2.0))) * u;
    case 2: return 0.5 * g * (1.0 + tanh(sqrt(2.0 / M_PI) * g * (1.0 + 0.044715 * g * g))) * u;
    case 3: {
      const double gc = g < limit ? g : limit;
      const double uc = u < -limit ? -limit : (u > limit ? limit : u);
      return gc / (1.0 + exp(-gc)) * uc;
    }
    default: return g / (1.0 + exp(-g)) * u;
  }
}

int orc_decode_vector_glu(int decoder, const orc_decode_operand* gate, uint64_t gate_first, int up_decoder,
                          const orc_decode_operand* up, uint64_t up_first, uint64_t outputs, int glu, float limit,
                          const float* x, uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride, int threads) {
  if (decoder < 0 || decoder > ORC_DECODER_AFFINE_SPLIT || up_decoder < 0 || up_decoder > ORC_DECODER_AFFINE_SPLIT || glu < 0 ||
      glu > 3 || gate->k != up->k)
    return 1;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t j = 0; j < (int64_t)outputs; ++j) {
    const uint64_t grow = gate_first + (uint64_t)j, urow = up_first + (uint64_t)j;
    const double gs = gate->tensor_scale != NULL ? (double)gate->tensor_scale[grow / gate->rows_per_scale] : 1.0;
    const double us = up->tensor_scale != NULL ? (double)up->tensor_scale[urow / up->rows_per_scale] : 1.0;
    for (uint64_t t = 0; t < rows; ++t) {
      double g = 0, u = 0;
      for (uint64_t c = 0; c < gate->k; ++c) {
        const double xv = (double)x[t * x_stride + c];
        g += (double)orc_decode_value(decoder, gate, grow, c) * xv;
        u += (double)orc_decode_value(up_decoder, up, urow, c) * xv;
      }
      y[t * y_stride + (uint64_t)j] = (float)decode_glu(glu, g * gs, u * us, (double)limit);
    }
  }
  return 0;
}

/* products.h:27-33: the matrix path rounds weights and inputs to the decoder's matrix element (F16 for F16 and
 * Q8_0 weights, BF16 otherwise) and sums in F32; here the sums are double. */
int orc_decode_matrix(int decoder, const orc_decode_operand* w, uint64_t first, uint64_t outputs, const float* x,
                      uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride, int threads) {
  if (decoder < 0 || decoder > ORC_DECODER_AFFINE_SPLIT) return 1;
  const int half = decoder == ORC_DECODER_F16_DENSE || decoder == ORC_DECODER_Q8_0_BLOCKS;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t j = 0; j < (int64_t)outputs; ++j) {
    const uint64_t row = first + (uint64_t)j;
    const double scale = w->tensor_scale != NULL ? (double)w->tensor_scale[row / w->rows_per_scale] : 1.0;
    for (uint64_t t = 0; t < rows; ++t) {
      double sum = 0;
      for (uint64_t c = 0; c < w->k; ++c) {
        const float wv = orc_decode_value(decoder, w, row, c), xv = x[t * x_stride + c];
        const float wr = half ? orc_f16_to_f32(orc_f32_to_f16(wv)) : orc_bf16_to_f32(orc_f32_to_bf16(wv));
        const float xr = half ? orc_f16_to_f32(orc_f32_to_f16(xv)) : orc_bf16_to_f32(orc_f32_to_bf16(xv));
        sum += (double)wr * (double)xr;
      }
      y[t * y_stride + (uint64_t)j] = (float)(sum * scale);
    }
  }
  return 0;
}

/* products.h:141-170 */
int orc_decode_grouped(int decoder, const orc_decode_operand* experts, uint64_t experts_count, uint32_t k, uint32_t n,
                       uint64_t first, uint64_t outputs, const int32_t* offsets, const int32_t* pair_rows,
                       const int32_t* pair_out, uint64_t pairs, const float* x, uint64_t x_rows, uint64_t x_stride, float* y,
                       uint64_t y_rows, uint64_t y_stride) {
  if (decoder < 0 || decoder > ORC_DECODER_AFFINE_SPLIT) return 1;
  for (uint64_t e = 0; e < experts_count; ++e) {
    const orc_decode_operand* w = &experts[e];
    if (w->k != k || w->rows != n) continue;
    int64_t begin = offsets[e], end = offsets[e + 1];
    if (begin < 0) begin = 0;
    if (end > (int64_t)pairs) end = (int64_t)pairs;
    for (int64_t p = begin; p < end; ++p) {
      const int64_t from = pair_rows[p], to = pair_out != NULL ? pair_out[p] : p;
      if (from < 0 || from >= (int64_t)x_rows || to < 0 || to >= (int64_t)y_rows) continue;
      for (uint64_t j = 0; j < outputs; ++j) {
        const uint64_t row = first + j;
        const double scale = w->tensor_scale != NULL ? (double)w->tensor_scale[row / w->rows_per_scale] : 1.0;
        double sum = 0;
        for (uint64_t c = 0; c < k; ++c) sum += (double)orc_decode_value(decoder, w, row, c) * (double)x[(uint64_t)from * x_stride + c];
        y[(uint64_t)to * y_stride + j] = (float)(sum * scale);
      }
    }
  }
  return 0;
}

/* -------------------------------------------------------------------- GLU */

static double sigmoid_d(double x) { return 1.0 / (1.0 + exp(-x)); }
static double silu_d(double x) { return x * sigmoid_d(x); }
static double gelu_tanh_d(double x) {
  const double c = sqrt(2.0 / M_PI);
  return 0.5 * x * (1.0 + tanh(c * x * (1.0 + 0.044715 * x * x)));
}

/* exec.cc:248-262 */
double orc_glu(int kind, double gate, double up, double limit) {
  switch (kind) {
    case ORC_GLU_SWIGLU:
      return silu_d(gate) * up;
    case ORC_GLU_GEGLU:
      return gelu_tanh_d(gate) * up;
    case ORC_GLU_SWIGLU_CLAMP: {
      const double g = gate < limit ? gate : limit;
      const double u = up < -limit ? -limit : (up > limit ? limit : up);
      return silu_d(g) * u;
    }
    default:
      return up;
  }
}

/* ------------------------------------------------------------------- vecq */

static double row_product(int type, const uint8_t* wrow, const uint8_t* y, int k) {
  const int qk = orc_block_elements(type);
  const int bs = orc_block_bytes(type);
  double s = 0;
  for (int b = 0; b < k / qk; ++b) s += orc_block_product(type, wrow + (int64_t)b * bs, y + (int64_t)b * (qk / 32) * 36);
  return s;
}

int orc_vecq(int type, const orc_vecq_desc* d, int experts, int threads) {
  const int bs = orc_block_bytes(type);
  const int routed = d->ids != NULL;
  const int pairs = routed ? d->tokens * d->used : d->tokens * d->used;
  for (int p = 0; routed && p < pairs; ++p) {
    const int id = d->ids[(p / d->used) * d->ids_stride + (p % d->used)];
    if (experts > 0 && (id < 0 || id >= experts)) return 1;
  }
  (void)threads;
  for (int p = 0; p < pairs; ++p) {
    const int t = p / d->used;
    const int u = p % d->used;
    const int expert = routed ? d->ids[t * d->ids_stride + u] : u;
    const uint8_t* y = (const uint8_t*)d->y + ((int64_t)t * d->y_token + (int64_t)u * d->y_slot) * 36;
    float* dst = d->dst + (int64_t)t * d->dst_token + (int64_t)u * d->dst_slot;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int r = 0; r < d->nrows; ++r) {
      const int64_t at = ((int64_t)expert * d->stride_expert + (int64_t)r * d->stride_row) * bs;
      const double up = row_product(type, (const uint8_t*)d->w + at, y, d->ncols_x);
      double v = up;
      if (d->g != NULL) {
        const double gate = row_product(type, (const uint8_t*)d->g + at, y, d->ncols_x);
        v = orc_glu(d->glu, gate, up, d->limit);
      }
      dst[r] = (float)v;
    }
  }
  return 0;
}

void orc_vecq_block_sums(int type, const void* w, const void* y, int k, int nrows, int stride_row,
                         int32_t* out) {
  const int qk = orc_block_elements(type);
  const int bs = orc_block_bytes(type);
  const int per = type == ORC_TYPE_Q4_K || type == ORC_TYPE_Q5_K || type == ORC_TYPE_Q6_K ? 16 : 1;
  const int blocks = k / qk;
  for (int r = 0; r < nrows; ++r)
    for (int b = 0; b < blocks; ++b)
      orc_block_sums(type, (const uint8_t*)w + ((int64_t)r * stride_row + b) * bs,
                     (const uint8_t*)y + (int64_t)b * (qk / 32) * 36, out + ((int64_t)r * blocks + b) * per);
}

/* ------------------------------------------------------------------ MXFP8 */

/* mxfp8_quant.cuh:22-29 */
uint32_t orc_mxfp8_scale_code(float amax) {
  const uint32_t bits = bits_of(amax * (1.0f / 448.0f));
  uint32_t e = (bits >> 23) & 0xFFu;
  if (bits & 0x7FFFFFu) ++e;
  return e > 253u ? 253u : e;
}
/* mxfp8_quant.cuh:33-35 */
float orc_mxfp8_inverse_scale(uint32_t e) { return float_of((254u - e) << 23); }

/* layout.h:108-113 */
uint64_t orc_scale_atom_offset(uint64_t row, uint64_t block, uint64_t blocks) {
  return ((((row / 128) * (blocks / 4)) + (block / 4)) * 512) + ((row % 32) * 16) + (((row % 128) / 32) * 4) +
         (block % 4);
}

/* llmp_ops.cu:610-648 */
void orc_mxfp8_quantize(const float* x, int64_t x_stride, int64_t k, int64_t rows, uint8_t* codes,
                        uint8_t* scales) {
  const int64_t blocks = k / 32;
  const int64_t padded = (rows + 127) / 128 * 128;
  for (int64_t r = 0; r < padded; ++r) {
    for (int64_t b = 0; b < blocks; ++b) {
      const uint64_t at = orc_scale_atom_offset((uint64_t)r, (uint64_t)b, (uint64_t)blocks);
      if (r >= rows) {
        scales[at] = 0;
        continue;
      }
      const float* v = x + r * x_stride + b * 32;
      float amax = 0.0f;
      for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(v[j]));
      const uint32_t e = orc_mxfp8_scale_code(amax);
      const float inverse = orc_mxfp8_inverse_scale(e);
      for (int j = 0; j < 32; ++j) codes[r * k + b * 32 + j] = orc_f32_to_e4m3(v[j] * inverse);
      scales[at] = (uint8_t)e;
    }
  }
}

/* llmp_ops.cu:652-663 */
void orc_mxfp8_swizzle(const uint8_t* in, int64_t n, int64_t blocks, uint8_t* out) {
  const int64_t padded = (n + 127) / 128 * 128;
  for (int64_t r = 0; r < padded; ++r)
    for (int64_t b = 0; b < blocks; ++b)
      out[orc_scale_atom_offset((uint64_t)r, (uint64_t)b, (uint64_t)blocks)] = r < n ? in[r * blocks + b] : 0;
}

double orc_mxfp8_dot(const uint8_t* a_codes, const uint8_t* a_scales, int64_t row_a,
                     const uint8_t* b_codes, const uint8_t* b_scales, int64_t row_b, int64_t k) {
  const int64_t blocks = k / 32;
  double total = 0;
  for (int64_t b = 0; b < blocks; ++b) {
    const double sa = orc_e8m0_to_f32(a_scales[orc_scale_atom_offset((uint64_t)row_a, (uint64_t)b, (uint64_t)blocks)]);
    const double sb = orc_e8m0_to_f32(b_scales[orc_scale_atom_offset((uint64_t)row_b, (uint64_t)b, (uint64_t)blocks)]);
    double s = 0;
    for (int j = 0; j < 32; ++j)
      s += (double)orc_e4m3_to_f32(a_codes[row_a * k + b * 32 + j]) * (double)orc_e4m3_to_f32(b_codes[row_b * k + b * 32 + j]);
    total += s * sa * sb;
  }
  return total;
}

void orc_mxfp8_gemm(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                    const uint8_t* b_scales, int64_t m, int64_t n, int64_t k, float* d, int threads) {
  /* Dequantize both operands once (exact in float: an E4M3 value times a power of two,
   * subnormal results aside), then float-accumulated dot products. */
  const int64_t blocks = k / 32;
  float table[256];
  for (int i = 0; i < 256; ++i) table[i] = orc_e4m3_to_f32((uint8_t)i);
  float* a = (float*)malloc(sizeof(float) * (size_t)(m * k));
  float* b = (float*)malloc(sizeof(float) * (size_t)(n * k));
  for (int64_t r = 0; r < m; ++r)
    for (int64_t c = 0; c < k; ++c)
      a[r * k + c] = table[a_codes[r * k + c]] *
                     orc_e8m0_to_f32(a_scales[orc_scale_atom_offset((uint64_t)r, (uint64_t)(c / 32), (uint64_t)blocks)]);
  for (int64_t r = 0; r < n; ++r)
    for (int64_t c = 0; c < k; ++c)
      b[r * k + c] = table[b_codes[r * k + c]] *
                     orc_e8m0_to_f32(b_scales[orc_scale_atom_offset((uint64_t)r, (uint64_t)(c / 32), (uint64_t)blocks)]);
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t i = 0; i < m; ++i) {
    for (int64_t j = 0; j < n; ++j) {
      const float* ar = a + i * k;
      const float* br = b + j * k;
      float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      for (int64_t c = 0; c < k; c += 8)
        for (int l = 0; l < 8; ++l) acc[l] += ar[c + l] * br[c + l];
      d[i * n + j] = ((acc[0] + acc[4]) + (acc[2] + acc[6])) + ((acc[1] + acc[5]) + (acc[3] + acc[7]));
    }
  }
  free(a);
  free(b);
}

void orc_mxfp8_gemv(const uint8_t* codes, const uint8_t* scales, int64_t n, int64_t k,
                    const float* x, int64_t tokens, float* y) {
  const int64_t blocks = k / 32;
  for (int64_t t = 0; t < tokens; ++t)
    for (int64_t r = 0; r < n; ++r) {
      double total = 0;
      for (int64_t b = 0; b < blocks; ++b) {
        double s = 0;
        for (int j = 0; j < 32; ++j) s += (double)orc_e4m3_to_f32(codes[r * k + b * 32 + j]) * (double)x[t * k + b * 32 + j];
        total += s * (double)orc_e8m0_to_f32(scales[r * blocks + b]);
      }
      y[t * n + r] = (float)total;
    }
}

/* -------------------------------------------------------------------- MoE */

/* exec.cc:279-315,1728-1818 (kSoftmaxTopK, no bias) */
void orc_route(const float* logits, int64_t experts, int64_t used, int64_t tokens, int normalize,
               float scale, int32_t* ids, float* weights) {
  double* p = (double*)malloc(sizeof(double) * (size_t)experts);
  int64_t* idx = (int64_t*)malloc(sizeof(int64_t) * (size_t)experts);
  for (int64_t t = 0; t < tokens; ++t) {
    const float* l = logits + t * experts;
    double max = -INFINITY;
    for (int64_t i = 0; i < experts; ++i) max = max < (double)l[i] ? (double)l[i] : max; /* std::max */
    if (!isfinite(max)) {
      for (int64_t i = 0; i < experts; ++i) p[i] = 0.0;
    } else {
      double sum = 0.0;
      for (int64_t i = 0; i < experts; ++i) {
        p[i] = exp((double)l[i] - max);
        sum += p[i];
      }
      for (int64_t i = 0; i < experts; ++i) p[i] = sum > 0.0 ? p[i] / sum : 0.0;
    }
    /* Order(): stable, descending, NaN last (insertion sort keeps equal keys in index order). */
    for (int64_t i = 0; i < experts; ++i) idx[i] = i;
    for (int64_t i = 1; i < experts; ++i) {
      const int64_t v = idx[i];
      int64_t j = i;
      while (j > 0) {
        const double x = p[v], y = p[idx[j - 1]];
        const int before = (isnan(x) || isnan(y)) ? (!isnan(x) && isnan(y)) : (x > y);
        if (!before) break;
        idx[j] = idx[j - 1];
        --j;
      }
      idx[j] = v;
    }
    double sum = 0.0;
    for (int64_t i = 0; i < used; ++i) sum += p[idx[i]];
    for (int64_t i = 0; i < used; ++i) {
      double w = p[idx[i]];
      if (normalize) w /= (sum > 0x1p-14 ? sum : 0x1p-14);
      ids[t * used + i] = (int32_t)idx[i];
      weights[t * used + i] = (float)(w * (double)scale);
    }
  }
  free(p);
  free(idx);
}

/* exec.cc:1003-1025 */
int orc_expert_sort(const int32_t* ids, int64_t pairs, int64_t experts, int32_t* order,
                    int32_t* offsets) {
  for (int64_t i = 0; i < pairs; ++i)
    if (ids[i] < 0 || ids[i] >= experts) return 1;
  int64_t n = 0;
  for (int64_t e = 0; e < experts; ++e) {
    offsets[e] = (int32_t)n;
    for (int64_t i = 0; i < pairs; ++i)
      if (ids[i] == e) order[n++] = (int32_t)i;
  }
  offsets[experts] = (int32_t)n;
  return 0;
}

/* exec.cc:1837-1853 in the float arithmetic of llmp_fused.cu:219-235 */
void orc_expert_reduce(const float* x, const float* w, int64_t width, int64_t used, int64_t tokens,
                       float* out) {
  for (int64_t t = 0; t < tokens; ++t)
    for (int64_t i = 0; i < width; ++i) {
      float acc = 0.0f;
      for (int64_t u = 0; u < used; ++u) {
        const float e = x[(t * used + u) * width + i] * w[t * used + u];
        acc = u == 0 ? e : acc + e;
      }
      out[t * width + i] = acc;
    }
}

/* ------------------------------------------------------------------- EXL3 */

static uint32_t lop3(uint32_t x) { return (x & 0x8FFF8FFFu) ^ 0x3B603B60u; } /* decode_exl3.cc:28 */
static uint16_t half_sum(uint32_t x) {                                       /* decode_exl3.cc:33-37 */
  const float sum = orc_f16_to_f32((uint16_t)(x & 0xFFFFu)) + orc_f16_to_f32((uint16_t)(x >> 16));
  return orc_f32_to_f16(sum);
}

/* decode_exl3.cc:41-66 */
uint16_t orc_exl3_codebook(int codebook, uint16_t state) {
  uint32_t x = state;
  switch (codebook) {
    case ORC_CB_3INST:
      x = x * 89226354u + 64248484u;
      return half_sum(lop3(x));
    case ORC_CB_MCG:
      x *= 0xCBAC1FEDu;
      return half_sum(lop3(x));
    case ORC_CB_MUL1: {
      x *= 0x83DCD12Du;
      const uint32_t sum = (x & 0xFFu) + ((x >> 8) & 0xFFu) + ((x >> 16) & 0xFFu) + (x >> 24) + 0x6400u;
      const float h = orc_f16_to_f32((uint16_t)(sum & 0xFFFFu));
      return orc_f32_to_f16(fmaf(h, orc_f16_to_f32(0x1EEEu), orc_f16_to_f32(0xC931u)));
    }
    default:
      return 0x7E00u;
  }
}

static uint32_t tile_word(const uint8_t* tile, uint32_t w) {
  uint32_t v;
  memcpy(&v, tile + 4 * (size_t)w, 4);
  return v;
}

/* decode_exl3.cc:82-96 */
uint16_t orc_exl3_state(const uint8_t* tile, uint32_t bits, uint32_t t) {
  const uint32_t words = bits * 256 / 32;
  const uint32_t b0 = t * bits + bits - 16 + 256 * bits;
  const uint32_t b1 = b0 + 16;
  const uint32_t i0 = b0 / 32;
  const uint32_t i1 = (b1 - 1) / 32;
  const uint32_t s0 = (i1 + 1) * 32 - b1;
  const uint64_t merged = ((uint64_t)tile_word(tile, i0 % words) << 32) | tile_word(tile, i1 % words);
  return (uint16_t)((merged >> s0) & 0xFFFFu);
}

/* decode_exl3.cc:98-127 */
void orc_exl3_placement(uint8_t* at) {
  for (int lane = 0; lane < 32; ++lane) {
    if (lane & 4) continue;
    for (int reg = 0; reg < 4; ++reg)
      for (int high = 0; high < 2; ++high) {
        const int row = (lane % 4) * 2 + (reg % 2) * 8 + high;
        const int pair = lane / 8 + (reg / 2) * 4;
        const int position = 8 * lane + 2 * reg + high;
        at[position] = (uint8_t)(row * 16 + 2 * pair);
        at[position + 32] = (uint8_t)(row * 16 + 2 * pair + 1);
      }
  }
}

static const uint16_t* codebook_table(int codebook) {
  static uint16_t tables[3][65536];
  static int ready[3];
#pragma omp critical(orc_codebook)
  if (!ready[codebook]) {
    for (uint32_t s = 0; s < 65536; ++s) tables[codebook][s] = orc_exl3_codebook(codebook, (uint16_t)s);
    ready[codebook] = 1;
  }
  return tables[codebook];
}

/* decode_exl3.cc:157-171: one tile's 256 values, F16 bits, row-major. */
static void tile_values(const uint8_t* tile, int bits, const uint16_t* table, const uint8_t* place, uint16_t* out) {
  for (uint32_t t = 0; t < 256; ++t) out[place[t]] = table[orc_exl3_state(tile, (uint32_t)bits, t)];
}

/* decode_exl3.cc:202-215 */
void orc_exl3_rotated(const uint8_t* trellis, int64_t k, int64_t n, int bits, int codebook,
                      int64_t first, int64_t count, uint16_t* out) {
  uint8_t place[256];
  orc_exl3_placement(place);
  const uint16_t* table = codebook_table(codebook);
  const int64_t tile_bytes = 32 * (int64_t)bits;
  uint16_t tile[256];
  for (int64_t kt = 0; kt < k / 16; ++kt)
    for (int64_t nt = first / 16; nt < (first + count) / 16; ++nt) {
      tile_values(trellis + (kt * (n / 16) + nt) * tile_bytes, bits, table, place, tile);
      for (int r = 0; r < 16; ++r) memcpy(&out[(kt * 16 + r) * count + nt * 16 - first], &tile[r * 16], 32);
    }
}

/* decode_exl3.cc:173-188 */
static void hadamard128(double* v) {
  for (int h = 1; h < 128; h *= 2)
    for (int i = 0; i < 128; i += 2 * h)
      for (int j = i; j < i + h; ++j) {
        const double a = v[j], b = v[j + h];
        v[j] = a + b;
        v[j + h] = a - b;
      }
}

/* decode_exl3.cc:217-265 */
void orc_exl3_rows(const uint8_t* trellis, const uint16_t* suh, const uint16_t* svh, int64_t k,
                   int64_t n, int bits, int codebook, int64_t first, int64_t count, float* out) {
  const int64_t end = first + count;
  uint16_t* rot = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(k * 128));
  double* block = (double*)malloc(sizeof(double) * (size_t)(k * 128));
  double* column = (double*)malloc(sizeof(double) * (size_t)k);
  for (int64_t b = first / 128; b * 128 < end; ++b) {
    orc_exl3_rotated(trellis, k, n, bits, codebook, b * 128, 128, rot);
    for (int64_t i = 0; i < k * 128; ++i) block[i] = orc_f16_to_f32(rot[i]);
    for (int64_t row = 0; row < k; ++row) hadamard128(&block[row * 128]);
    const int64_t lo = first > b * 128 ? first : b * 128;
    const int64_t hi = end < (b + 1) * 128 ? end : (b + 1) * 128;
    for (int64_t c = lo; c < hi; ++c) {
      const int64_t j = c - b * 128;
      for (int64_t row = 0; row < k; ++row) column[row] = block[row * 128 + j];
      for (int64_t kb = 0; kb < k; kb += 128) hadamard128(&column[kb]);
      const double sv = orc_f16_to_f32(svh[c]);
      float* y = out + (c - first) * k;
      for (int64_t row = 0; row < k; ++row) y[row] = (float)(column[row] * (double)orc_f16_to_f32(suh[row]) * sv / 128.0);
    }
  }
  free(rot);
  free(block);
  free(column);
}

void orc_exl3_input(const uint16_t* suh, int64_t k, const uint16_t* x, int64_t m, uint16_t* xh) {
  const double r = 0.088388347648; /* validate.h:64 */
  double* row = (double*)malloc(sizeof(double) * (size_t)k);
  for (int64_t i = 0; i < m; ++i) {
    for (int64_t c = 0; c < k; ++c) row[c] = (double)orc_f16_to_f32(x[i * k + c]) * (double)orc_f16_to_f32(suh[c]);
    for (int64_t kb = 0; kb < k; kb += 128) hadamard128(&row[kb]);
    for (int64_t c = 0; c < k; ++c) xh[i * k + c] = orc_f32_to_f16((float)(row[c] * r));
  }
  free(row);
}

void orc_exl3_product(const uint8_t* trellis, const uint16_t* svh, int64_t k, int64_t n, int bits,
                      int codebook, const uint16_t* xh, int64_t m, float* y, int threads) {
  const double r = 0.088388347648;
  (void)codebook_table(codebook);
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t b = 0; b < n / 128; ++b) {
    uint16_t* rot = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(k * 128));
    float* rotf = (float*)malloc(sizeof(float) * (size_t)(k * 128));
    orc_exl3_rotated(trellis, k, n, bits, codebook, b * 128, 128, rot);
    for (int64_t i = 0; i < k * 128; ++i) rotf[i] = orc_f16_to_f32(rot[i]);
    for (int64_t i = 0; i < m; ++i) {
      double acc[128];
      for (int j = 0; j < 128; ++j) acc[j] = 0;
      for (int64_t c = 0; c < k; ++c) {
        const double xv = orc_f16_to_f32(xh[i * k + c]);
        const float* wr = rotf + c * 128;
        for (int j = 0; j < 128; ++j) acc[j] += xv * (double)wr[j];
      }
      hadamard128(acc);
      for (int j = 0; j < 128; ++j) y[i * n + b * 128 + j] = (float)(acc[j] * r * (double)orc_f16_to_f32(svh[b * 128 + j]));
    }
    free(rot);
    free(rotf);
  }
}

void orc_exl3_linear(const uint8_t* trellis, const uint16_t* suh, const uint16_t* svh, int64_t k,
                     int64_t n, int bits, int codebook, const uint16_t* x, int64_t m, float* y,
                     int threads) {
  uint16_t* xh = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(m * k));
  orc_exl3_input(suh, k, x, m, xh);
  orc_exl3_product(trellis, svh, k, n, bits, codebook, xh, m, y, threads);
  free(xh);
}

/* ------------------------------------------------------------------ attention over a quantized KV cache
 * The reference executor's attention (src/kernels/reference/exec.cc:1027-1085, SoftmaxRow :279-299) over K and V
 * rows stored as Q8_0 or Q4_0 blocks, decoded exactly (orc_decode_row), everything else in double: what the
 * reference's own test holds its quantized vector attention to (tests/unit/kv_quant_gpu_test.cc:826-950, NMSE
 * 5e-4). q F32 [heads][rows][d] (a head's rows together, as ggml's [D, rows, heads]); k, v uint8, the row of
 * (cell, kv head) at cell * cell_stride + head * head_stride bytes; mask F16 bits [mask_rows][cells] or NULL;
 * sinks F32 [heads] or NULL; out F32 [rows][heads][d] (ggml's [D, heads, rows]). No ALiBi (slope 1).
 * q8_1_q != 0: each query row is first quantized to Q8_1 and decoded again, which is what the device multiplies K
 * with (kv_quant.h:16-19 of the reference: "quantizing Q to Q8_1 in shared memory for the K product"): the
 * comparison that leaves accumulation order alone. */
void orc_attention_quant(int type, const float* q, const uint8_t* k, const uint8_t* v, int64_t cell_stride,
                         int64_t head_stride, const uint16_t* mask, const float* sinks, int64_t d, int64_t heads,
                         int64_t kv_heads, int64_t rows, int64_t cells, float scale, float softcap, int q8_1_q,
                         float* out, int threads) {
  const int64_t group = heads / kv_heads;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(dynamic)
  for (int64_t h = 0; h < heads; ++h) {
    const int64_t kh = h / group;
    float* kd = (float*)malloc((size_t)(cells * d) * sizeof(float));
    float* vd = (float*)malloc((size_t)(cells * d) * sizeof(float));
    double* s = (double*)malloc((size_t)cells * sizeof(double));
    float* qrow = (float*)malloc((size_t)d * sizeof(float));
    uint8_t* q8 = (uint8_t*)malloc((size_t)((d + 511) / 512 * 512 / 32 * 36));
    for (int64_t c = 0; c < cells; ++c) {
      orc_decode_row(type, k + c * cell_stride + kh * head_stride, d, kd + c * d);
      orc_decode_row(type, v + c * cell_stride + kh * head_stride, d, vd + c * d);
    }
    for (int64_t iq = 0; iq < rows; ++iq) {
      const float* qsrc = q + (h * rows + iq) * d;
      if (q8_1_q) {
        orc_q8_1_quantize_row(qsrc, d, (d + 511) / 512 * 512, q8, 0);
        orc_q8_1_decode_row(q8, d, qrow);
      } else {
        memcpy(qrow, qsrc, (size_t)d * sizeof(float));
      }
      double max = -INFINITY;
      for (int64_t c = 0; c < cells; ++c) {
        double dot = 0.0;
        for (int64_t j = 0; j < d; ++j) dot += (double)qrow[j] * (double)kd[c * d + j];
        double score = dot * (double)scale;
        if (softcap > 0.0f) score = (double)softcap * tanh(score / (double)softcap);
        if (mask != NULL) score += (double)orc_f16_to_f32(mask[iq * cells + c]);
        s[c] = score;
        if (score > max) max = score;
      }
      if (sinks != NULL && (double)sinks[h] > max) max = (double)sinks[h];
      float* o = out + (iq * heads + h) * d;
      if (!isfinite(max)) { /* a row with nothing finite (and no sink) is zero */
        for (int64_t j = 0; j < d; ++j) o[j] = 0.0f;
        continue;
      }
      double sum = sinks != NULL ? exp((double)sinks[h] - max) : 0.0;
      for (int64_t c = 0; c < cells; ++c) {
        s[c] = exp(s[c] - max);
        sum += s[c];
      }
      for (int64_t j = 0; j < d; ++j) {
        double acc = 0.0;
        for (int64_t c = 0; c < cells; ++c) {
          const double p = sum > 0.0 ? s[c] / sum : 0.0;
          if (p != 0.0) acc += p * (double)vd[c * d + j];
        }
        o[j] = (float)acc;
      }
    }
    free(kd);
    free(vd);
    free(s);
    free(qrow);
    free(q8);
  }
}
