/*
 * orangu_oracle.c -- CPU restatement of orangu-server's quantized vec_dot / matmul path.
 * TEST INFRASTRUCTURE ONLY: see orangu_oracle.h for what may load this and how it is pinned.
 *
 * Build: gcc -O3 -ffp-contract=off -fopenmp -fPIC -shared (oracle/Makefile).  Never -ffast-math:
 * the reference is Rust, which neither contracts a*b+c nor reassociates.
 */
#include "orangu_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#if defined(__x86_64__)
#include <immintrin.h>
#endif
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ formats */

/* quant.rs:511-528.  Shift exponent/mantissa into f32 position, rebias, fix up the two special
 * exponents.  A NaN keeps its payload. */
float ogo_f16_bits_to_f32(uint16_t bits) {
  const uint32_t SHIFTED_EXP = 0x7c00u << 13;
  uint32_t out = ((uint32_t)bits & 0x7fffu) << 13;
  uint32_t exp = SHIFTED_EXP & out;
  out += (127u - 15u) << 23;
  if (exp == SHIFTED_EXP) {
    out += (128u - 16u) << 23;
  } else if (exp == 0) {
    out += 1u << 23;
    float a, b;
    uint32_t magic = 113u << 23;
    memcpy(&a, &out, 4);
    memcpy(&b, &magic, 4);
    a = a - b;
    memcpy(&out, &a, 4);
  }
  out |= ((uint32_t)bits & 0x8000u) << 16;
  float f;
  memcpy(&f, &out, 4);
  return f;
}

/* quant.rs:530-533 */
static inline float read_f16(const uint8_t *bytes, size_t offset) {
  return ogo_f16_bits_to_f32((uint16_t)(bytes[offset] | ((uint16_t)bytes[offset + 1] << 8)));
}

/* quant.rs:653-662 */
void ogo_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
  if (j < 4) {
    *sc = q[j] & 63;
    *m = q[j + 4] & 63;
  } else {
    *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
    *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
  }
}

/* quant.rs:132-169, the three quantized types on the path plus the two float ones */
int ogo_block_layout(uint32_t ggml_type, size_t *block_bytes, size_t *block_elems) {
  size_t bb, be;
  switch (ggml_type) {
    case OGO_TYPE_F32: bb = 4; be = 1; break;
    case OGO_TYPE_F16: bb = 2; be = 1; break;
    case OGO_TYPE_Q4_0: bb = 2 + 16; be = 32; break;
    case OGO_TYPE_Q5_0: bb = 2 + 4 + 16; be = 32; break;
    case OGO_TYPE_Q5_1: bb = 2 + 2 + 4 + 16; be = 32; break;
    case OGO_TYPE_Q8_0: bb = 2 + 32; be = 32; break;
    case OGO_TYPE_Q2_K: bb = 16 + 64 + 2 + 2; be = 256; break;
    case OGO_TYPE_IQ4_XS: bb = 2 + 2 + 4 + 128; be = 256; break;
    case OGO_TYPE_IQ4_NL: bb = 2 + 16; be = 32; break;
    case OGO_TYPE_Q3_K: bb = 32 + 64 + 12 + 2; be = 256; break;
    case OGO_TYPE_Q4_K: bb = 2 + 2 + 12 + 128; be = 256; break;
    case OGO_TYPE_Q5_K: bb = 2 + 2 + 12 + 32 + 128; be = 256; break;
    case OGO_TYPE_Q6_K: bb = 128 + 64 + 16 + 2; be = 256; break;
    default: return -1;
  }
  if (block_bytes) *block_bytes = bb;
  if (block_elems) *block_elems = be;
  return 0;
}

/* quant.rs:344-357 */
int64_t ogo_tensor_byte_size(uint32_t ggml_type, uint64_t element_count) {
  size_t bb, be;
  if (ogo_block_layout(ggml_type, &bb, &be) != 0) return -1;
  if (element_count % be != 0) return -2;
  return (int64_t)(element_count / be * bb);
}

/* quant.rs:639-649 */
static void dequantize_q8_0(const uint8_t *bytes, size_t n, float *out) {
  for (size_t b = 0; b < n / 32; b++) {
    const uint8_t *block = bytes + b * 34;
    float d = read_f16(block, 0);
    for (int i = 0; i < 32; i++) out[b * 32 + i] = (float)(int8_t)block[2 + i] * d;
  }
}

/* quant.rs:666-697 */
static void dequantize_q4_k(const uint8_t *bytes, size_t n, float *out) {
  for (size_t s = 0; s < n / 256; s++) {
    const uint8_t *block = bytes + s * 144;
    float d = read_f16(block, 0);
    float dmin = read_f16(block, 2);
    const uint8_t *scales = block + 4;
    const uint8_t *qs = block + 16;
    float *o = out + s * 256;
    int is = 0;
    for (int q_offset = 0; q_offset < 256; q_offset += 64) {
      uint8_t sc1, m1, sc2, m2;
      ogo_get_scale_min_k4(is, scales, &sc1, &m1);
      float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
      ogo_get_scale_min_k4(is + 1, scales, &sc2, &m2);
      float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
      const uint8_t *q = qs + q_offset / 2;
      for (int l = 0; l < 32; l++) *o++ = d1 * (float)(q[l] & 0x0F) - mm1;
      for (int l = 0; l < 32; l++) *o++ = d2 * (float)(q[l] >> 4) - mm2;
      is += 2;
    }
  }
}

/* quant.rs:703-742: Q4_K plus a fifth bit; bit j of qh[l] belongs to element l of sub-block j */
static void dequantize_q5_k(const uint8_t *bytes, size_t n, float *out) {
  for (size_t s = 0; s < n / 256; s++) {
    const uint8_t *block = bytes + s * 176;
    float d = read_f16(block, 0);
    float dmin = read_f16(block, 2);
    const uint8_t *scales = block + 4;
    const uint8_t *qh = block + 16;
    const uint8_t *qs = block + 48;
    float *o = out + s * 256;
    int is = 0;
    uint8_t u1 = 1, u2 = 2;
    for (int q_offset = 0; q_offset < 256; q_offset += 64) {
      uint8_t sc1, m1, sc2, m2;
      ogo_get_scale_min_k4(is, scales, &sc1, &m1);
      float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
      ogo_get_scale_min_k4(is + 1, scales, &sc2, &m2);
      float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
      const uint8_t *ql = qs + q_offset / 2;
      for (int l = 0; l < 32; l++) *o++ = d1 * (float)((int)(ql[l] & 0x0F) + ((qh[l] & u1) ? 16 : 0)) - mm1;
      for (int l = 0; l < 32; l++) *o++ = d2 * (float)((int)(ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - mm2;
      is += 2;
      u1 = (uint8_t)(u1 << 2);
      u2 = (uint8_t)(u2 << 2);
    }
  }
}

/* iq_grids.rs:5941-5943 */
static const int8_t KVALUES_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10,
                                          1,    13,   25,  38,  53,  69,  89,  113};

/* unpack_block_q5_bits / unpack_block_q4_0 / _q5_0 / _iq4_nl (vecdot.rs:913-1039): elements 0..16
 * from the low nibbles, 16..32 from the high nibbles; Q5_0 adds bit j (resp. j + 16) of qh as a
 * fifth bit; Q4_0 and Q5_0 subtract their zero point (8, 16), IQ4_NL looks its nibble up. */
float ogo_unpack_flat_block(uint32_t ggml_type, const uint8_t *block, int8_t *w) {
  float dw = read_f16(block, 0);
  if (ggml_type == OGO_TYPE_Q8_0) {
    memcpy(w, block + 2, 32);
  } else if (ggml_type == OGO_TYPE_IQ4_NL) {
    const uint8_t *qs = block + 2;
    for (int j = 0; j < 16; j++) {
      w[j] = KVALUES_IQ4NL[qs[j] & 0x0F];
      w[j + 16] = KVALUES_IQ4NL[qs[j] >> 4];
    }
  } else {
    uint32_t qh = 0;
    const uint8_t *qs = block + 2;
    int bias = 8;
    if (ggml_type == OGO_TYPE_Q5_0) {
      qh = (uint32_t)block[2] | ((uint32_t)block[3] << 8) | ((uint32_t)block[4] << 16) | ((uint32_t)block[5] << 24);
      qs = block + 6;
      bias = 16;
    }
    for (int j = 0; j < 16; j++) {
      uint32_t hi_lo = ((qh >> j) << 4) & 0x10;
      uint32_t hi_hi = (qh >> (j + 12)) & 0x10;
      w[j] = (int8_t)((int32_t)((uint32_t)(qs[j] & 0x0F) | hi_lo) - bias);
      w[16 + j] = (int8_t)((int32_t)((uint32_t)(qs[j] >> 4) | hi_hi) - bias);
    }
  }
  return dw;
}

/* quant.rs:537-554 (Q4_0), 560-580 (Q5_0), 1320-1337 (IQ4_NL).  Q4_0 and Q5_0 multiply
 * (float)q * d, IQ4_NL d * (float)level: the products commute, the values are the same. */
static void dequantize_flat32(uint32_t ggml_type, const uint8_t *bytes, size_t n, float *out) {
  size_t bb, be;
  ogo_block_layout(ggml_type, &bb, &be);
  int8_t w[32];
  for (size_t b = 0; b < n / 32; b++) {
    float d = ogo_unpack_flat_block(ggml_type, bytes + b * bb, w);
    for (int j = 0; j < 32; j++) out[b * 32 + (size_t)j] = (float)w[j] * d;
  }
}

/* unpack_block_q5_1 (vecdot.rs:1032-1034, :1001-1017 with bias 0): block = d | m | qh | qs[16] */
static inline void unpack_block_q5_1(const uint8_t *block, int8_t *w) {
  uint32_t qh = (uint32_t)block[4] | ((uint32_t)block[5] << 8) | ((uint32_t)block[6] << 16) | ((uint32_t)block[7] << 24);
  const uint8_t *qs = block + 8;
  for (int j = 0; j < 16; j++) {
    uint32_t hi_lo = ((qh >> j) << 4) & 0x10;
    uint32_t hi_hi = (qh >> (j + 12)) & 0x10;
    w[j] = (int8_t)((uint32_t)(qs[j] & 0x0F) | hi_lo);
    w[16 + j] = (int8_t)((uint32_t)(qs[j] >> 4) | hi_hi);
  }
}

/* quant.rs:615-636 */
static void dequantize_q5_1(const uint8_t *bytes, size_t n, float *out) {
  int8_t w[32];
  for (size_t b = 0; b < n / 32; b++) {
    const uint8_t *block = bytes + b * 24;
    float d = read_f16(block, 0), m = read_f16(block, 2);
    unpack_block_q5_1(block, w);
    for (int j = 0; j < 32; j++) out[b * 32 + (size_t)j] = (float)w[j] * d + m;
  }
}

/* unpack_block_iq4_nl (vecdot.rs:937-942) */
static inline void unpack_block_iq4_nl(const uint8_t *qs, int8_t *w) {
  for (int j = 0; j < 16; j++) {
    w[j] = KVALUES_IQ4NL[qs[j] & 0x0F];
    w[j + 16] = KVALUES_IQ4NL[qs[j] >> 4];
  }
}

/* The six-bit scale of sub-block ib, biased by 32 (vecdot.rs:3257-3259): block = d | scales_h:u16 | scales_l[4] | qs[128] */
static inline int32_t iq4_xs_scale(const uint8_t *block, int ib) {
  uint32_t scales_h = (uint32_t)block[2] | ((uint32_t)block[3] << 8);
  uint32_t low = (block[4 + ib / 2] >> (4 * (ib % 2))) & 0x0F;
  uint32_t high = (scales_h >> (2 * ib)) & 3;
  return (int32_t)(low | (high << 4)) - 32;
}

/* quant.rs:1350-1375 */
static void dequantize_iq4_xs(const uint8_t *bytes, size_t n, float *out) {
  for (size_t s = 0; s < n / 256; s++) {
    const uint8_t *block = bytes + s * 136;
    float d = read_f16(block, 0);
    for (int ib = 0; ib < 8; ib++) {
      float dl = d * (float)iq4_xs_scale(block, ib);
      const uint8_t *qs = block + 8 + 16 * ib;
      for (int j = 0; j < 16; j++) {
        out[s * 256 + 32 * (size_t)ib + (size_t)j] = dl * (float)KVALUES_IQ4NL[qs[j] & 0xF];
        out[s * 256 + 32 * (size_t)ib + (size_t)j + 16] = dl * (float)KVALUES_IQ4NL[qs[j] >> 4];
      }
    }
  }
}

/* quant.rs:798-827 */
static void dequantize_q2_k(const uint8_t *bytes, size_t n, float *out) {
  for (size_t s = 0; s < n / 256; s++) {
    const uint8_t *block = bytes + s * 84;
    const uint8_t *scales = block, *qs = block + 16;
    float d = read_f16(block, 80), dmin = read_f16(block, 82);
    int is = 0;
    size_t o = s * 256;
    for (int q_off = 0; q_off < 64; q_off += 32) {
      const uint8_t *q = qs + q_off;
      for (int shift = 0; shift < 8; shift += 2) {
        for (int half = 0; half < 2; half++) {
          uint8_t sc = scales[is++];
          float dl = d * (float)(sc & 0xF), ml = dmin * (float)(sc >> 4);
          for (int l = 0; l < 16; l++) out[o++] = dl * (float)((q[half * 16 + l] >> shift) & 3) - ml;
        }
      }
    }
  }
}

/* quant.rs:883-897 */
void ogo_unpack_q3_k_scales(const uint8_t *packed, int32_t *scales) {
  for (int i = 0; i < 16; i++) {
    uint8_t low = i < 8 ? (uint8_t)(packed[i] & 0xF) : (uint8_t)(packed[i - 8] >> 4);
    /* scale i's two high bits sit at bit 2 * (i / 4) of byte 8 + i % 4 */
    uint8_t high = (uint8_t)((packed[8 + (i % 4)] >> (2 * (i / 4))) & 3);
    scales[i] = (int32_t)(low | (high << 4));
  }
}

/* quant.rs:841-871: hmask[32] | qs[64] | scales[12] | d; the third bit is stored inverted (clear
 * means subtract 4), the mask bit advances once per 32 elements */
static void dequantize_q3_k(const uint8_t *bytes, size_t n, float *out) {
  for (size_t s = 0; s < n / 256; s++) {
    const uint8_t *block = bytes + s * 110;
    const uint8_t *hmask = block, *qs = block + 32;
    int32_t scales[16];
    ogo_unpack_q3_k_scales(block + 96, scales);
    float d_all = read_f16(block, 108);
    float *o = out + s * 256;
    int is = 0;
    uint8_t m = 1;
    for (size_t q_off = 0; q_off < 64; q_off += 32) {
      for (int shift = 0; shift < 8; shift += 2) {
        for (int half = 0; half < 2; half++) {
          float dl = d_all * (float)(scales[is] - 32);
          is += 1;
          for (int l = 0; l < 16; l++) {
            int idx = half * 16 + l;
            int hi = (hmask[idx] & m) ? 0 : 4;
            *o++ = dl * (float)((int)((qs[q_off + (size_t)idx] >> shift) & 3) - hi);
          }
        }
        m = (uint8_t)(m << 1);
      }
    }
  }
}

/* quant.rs:746-787 */
static void dequantize_q6_k(const uint8_t *bytes, size_t n, float *out) {
  for (size_t s = 0; s < n / 256; s++) {
    const uint8_t *block = bytes + s * 210;
    const uint8_t *ql = block, *qh = block + 128, *sc = block + 192;
    float d = read_f16(block, 208);
    float *values = out + s * 256;
    size_t ql_off = 0, qh_off = 0, sc_off = 0;
    for (size_t y_off = 0; y_off < 256; y_off += 128) {
      for (size_t l = 0; l < 32; l++) {
        size_t is = l / 16;
        int32_t q1 = (int32_t)((ql[ql_off + l] & 0xF) | ((qh[qh_off + l] & 3) << 4)) - 32;
        int32_t q2 =
            (int32_t)((ql[ql_off + l + 32] & 0xF) | (((qh[qh_off + l] >> 2) & 3) << 4)) - 32;
        int32_t q3 = (int32_t)((ql[ql_off + l] >> 4) | (((qh[qh_off + l] >> 4) & 3) << 4)) - 32;
        int32_t q4 =
            (int32_t)((ql[ql_off + l + 32] >> 4) | (((qh[qh_off + l] >> 6) & 3) << 4)) - 32;
        values[y_off + l] = d * (float)(int8_t)sc[sc_off + is] * (float)q1;
        values[y_off + l + 32] = d * (float)(int8_t)sc[sc_off + is + 2] * (float)q2;
        values[y_off + l + 64] = d * (float)(int8_t)sc[sc_off + is + 4] * (float)q3;
        values[y_off + l + 96] = d * (float)(int8_t)sc[sc_off + is + 6] * (float)q4;
      }
      ql_off += 64;
      qh_off += 32;
      sc_off += 8;
    }
  }
}

int ogo_dequantize(uint32_t ggml_type, const uint8_t *bytes, size_t element_count, float *out) {
  size_t bb, be;
  if (ogo_block_layout(ggml_type, &bb, &be) != 0) return -1;
  if (element_count % be != 0) return -2;
  switch (ggml_type) {
    case OGO_TYPE_Q8_0: dequantize_q8_0(bytes, element_count, out); return 0;
    case OGO_TYPE_Q4_0:
    case OGO_TYPE_Q5_0:
    case OGO_TYPE_IQ4_NL: dequantize_flat32(ggml_type, bytes, element_count, out); return 0;
    case OGO_TYPE_Q5_1: dequantize_q5_1(bytes, element_count, out); return 0;
    case OGO_TYPE_Q2_K: dequantize_q2_k(bytes, element_count, out); return 0;
    case OGO_TYPE_IQ4_XS: dequantize_iq4_xs(bytes, element_count, out); return 0;
    case OGO_TYPE_Q3_K: dequantize_q3_k(bytes, element_count, out); return 0;
    case OGO_TYPE_Q4_K: dequantize_q4_k(bytes, element_count, out); return 0;
    case OGO_TYPE_Q5_K: dequantize_q5_k(bytes, element_count, out); return 0;
    case OGO_TYPE_Q6_K: dequantize_q6_k(bytes, element_count, out); return 0;
    default: return -1;
  }
}

/* ------------------------------------------------------------------ fixtures */

/* quant.rs:1427-1437 */
void ogo_fixture_bytes(size_t len, uint8_t *out) {
  uint64_t state = 0x2545F4914F6CDD1Dull;
  for (size_t i = 0; i < len; i++) {
    state ^= state << 13;
    state ^= state >> 7;
    state ^= state << 17;
    out[i] = (uint8_t)(state >> 33);
  }
}

/* quant.rs:1442-1446 */
uint64_t ogo_bit_checksum(const float *values, size_t n) {
  uint64_t acc = 0xcbf29ce484222325ull;
  for (size_t i = 0; i < n; i++) {
    uint32_t bits;
    memcpy(&bits, &values[i], 4);
    acc = (acc ^ (uint64_t)bits) * 0x00000100000001b3ull;
  }
  return acc;
}

/* vecdot.rs:3415-3423 */
void ogo_pseudo_bytes(size_t n, uint32_t seed, uint8_t *out) {
  uint32_t s = seed | 1u;
  for (size_t i = 0; i < n; i++) {
    s = s * 1664525u + 1013904223u;
    out[i] = (uint8_t)(s >> 16);
  }
}

/* ------------------------------------------------------------------ quantizers */

/* `(v * inv).round().clamp(-127.0, 127.0) as i8`: roundf is ties-away; clamp propagates NaN and
 * the saturating cast then maps NaN to 0 (vecdot.rs:117, 3042). */
static inline int8_t quantize_one(float v, float inv) {
  float r = roundf(v * inv);
  if (r != r) return 0;
  if (r < -127.0f) r = -127.0f;
  if (r > 127.0f) r = 127.0f;
  return (int8_t)r;
}

/* amax fold of vecdot.rs:103 / 3037: `fold(0f32, |m, v| m.max(v.abs()))`, f32::max ignores NaN */
static inline float abs_max(const float *x, size_t n) {
  float m = 0.0f;
  for (size_t i = 0; i < n; i++) m = fmaxf(m, fabsf(x[i]));
  return m;
}

/* vecdot.rs:95-126 quantize_act_scalar */
void ogo_quantize_act(const float *x, size_t n, int8_t *q, float *d, int32_t *sums) {
  for (size_t b = 0; b < n / 32; b++) {
    const float *chunk = x + b * 32;
    float amax = abs_max(chunk, 32);
    float scale = amax / 127.0f;
    float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
    for (int half = 0; half < 2; half++) {
      int32_t sum = 0;
      for (int i = 0; i < 16; i++) {
        int8_t qi = quantize_one(chunk[half * 16 + i], inv);
        q[b * 32 + (size_t)half * 16 + (size_t)i] = qi;
        sum += qi;
      }
      if (sums) sums[b * 2 + (size_t)half] = sum;
    }
    d[b] = scale;
  }
}

/* vecdot.rs:3030-3053 quantize_act_k_row */
void ogo_quantize_act_k_row(const float *x, size_t n, int8_t *q, float *d, int32_t *sums) {
  for (size_t s = 0; s < n / 256; s++) {
    const float *chunk = x + s * 256;
    float amax = abs_max(chunk, 256);
    float scale = amax / 127.0f;
    float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
    for (int g = 0; g < 16; g++) {
      int32_t sum = 0;
      for (int i = 0; i < 16; i++) {
        int8_t qi = quantize_one(chunk[g * 16 + i], inv);
        q[s * 256 + (size_t)g * 16 + (size_t)i] = qi;
        sum += qi;
      }
      if (sums) sums[s * 16 + (size_t)g] = sum;
    }
    d[s] = scale;
  }
}

/* vecdot.rs:1858-1910 ActQ8K::quantize.  Arrays must arrive zero-filled (padding tokens stay 0). */
void ogo_act_q8k_quantize(const float *x, size_t in_dim, size_t n_tokens, int8_t *q, float *d,
                          int16_t *bsum) {
  size_t n_block = in_dim / 32, n_super = in_dim / 256;
  size_t n_tile = (n_tokens + 3) / 4;
  for (size_t tl = 0; tl < n_tile; tl++) {
    for (size_t k = 0; k < 4; k++) {
      size_t t = tl * 4 + k;
      if (t >= n_tokens) break;
      const float *row = x + t * in_dim;
      for (size_t s = 0; s < n_super; s++) {
        const float *chunk = row + s * 256;
        float amax = abs_max(chunk, 256);
        float scale = amax / 127.0f;
        float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
        d[(tl * n_super + s) * 4 + k] = scale;
        for (size_t j = 0; j < 8; j++) {
          size_t b = s * 8 + j;
          const float *src = chunk + j * 32;
          int8_t *dst = q + ((tl * n_block + b) * 4 + k) * 32;
          int32_t sum = 0;
          for (int i = 0; i < 32; i++) {
            int8_t qi = quantize_one(src[i], inv);
            dst[i] = qi;
            sum += qi;
          }
          bsum[((tl * n_super + s) * 4 + k) * 8 + j] = (int16_t)sum;
        }
      }
    }
  }
}

/* vecdot.rs:2483-2525 ActQ8Flat::quantize (quantize_block::<false>, :219-240) */
void ogo_act_q8flat_quantize(const float *x, size_t in_dim, size_t n_tokens, int8_t *q, float *d) {
  size_t n_block = in_dim / 32;
  size_t n_tile = (n_tokens + 3) / 4;
  for (size_t tl = 0; tl < n_tile; tl++) {
    for (size_t k = 0; k < 4; k++) {
      size_t t = tl * 4 + k;
      if (t >= n_tokens) break;
      const float *row = x + t * in_dim;
      for (size_t b = 0; b < n_block; b++) {
        const float *chunk = row + b * 32;
        int8_t *dst = q + ((tl * n_block + b) * 4 + k) * 32;
        float amax = abs_max(chunk, 32);
        float scale = amax / 127.0f;
        float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
        for (int i = 0; i < 32; i++) dst[i] = quantize_one(chunk[i], inv);
        d[(tl * n_block + b) * 4 + k] = scale;
      }
    }
  }
}

/* ------------------------------------------------------------------ unpacked rows */

/* vecdot.rs:1074-1075 Q6K_RUNS */
static const struct {
  size_t ql_add;
  int hshift;
  int high;
} Q6K_RUNS[4] = {{0, 0, 0}, {32, 2, 0}, {0, 4, 1}, {32, 6, 1}};

/* vecdot.rs:1919-1936 KRow */
typedef struct {
  int8_t *q;     /* in_dim */
  int16_t *sc;   /* per 32 (Q4_K) or per 16 (Q6_K) */
  int16_t *mins; /* per 32, Q4_K only */
  float *d;      /* per super-block */
  float *dmin;   /* per super-block, Q4_K only */
} ogo_krow;

/* vecdot.rs:1836-1856 ActQ8K */
typedef struct {
  size_t n_tokens, n_block, n_super, n_tile;
  int8_t *q;
  float *d;
  int16_t *bsum;
} ogo_actq8k;

/* vecdot.rs:2469-2481 ActQ8Flat */
typedef struct {
  size_t n_tokens, n_block, n_tile;
  int8_t *q;
  float *d;
} ogo_actq8flat;

static int krow_alloc(ogo_krow *r, size_t in_dim) {
  r->q = (int8_t *)malloc(in_dim);
  r->sc = (int16_t *)malloc(sizeof(int16_t) * (in_dim / 16));
  r->mins = (int16_t *)malloc(sizeof(int16_t) * (in_dim / 32));
  r->d = (float *)malloc(sizeof(float) * (in_dim / 256));
  r->dmin = (float *)malloc(sizeof(float) * (in_dim / 256));
  return (r->q && r->sc && r->mins && r->d && r->dmin) ? 0 : -1;
}
static void krow_free(ogo_krow *r) {
  free(r->q);
  free(r->sc);
  free(r->mins);
  free(r->d);
  free(r->dmin);
}

/* vecdot.rs:2036-2058 unpack_k_q4_k */
static void unpack_k_q4_k(const uint8_t *row, size_t in_dim, ogo_krow *out) {
  size_t sb = 0;
  for (size_t s = 0; s < in_dim / 256; s++) {
    const uint8_t *block = row + s * 144;
    out->d[s] = read_f16(block, 0);
    out->dmin[s] = read_f16(block, 2);
    const uint8_t *scales = block + 4;
    const uint8_t *qs = block + 16;
    for (int g = 0; g < 4; g++) {
      const uint8_t *bytes = qs + g * 32;
      for (int half = 0; half < 2; half++) {
        int shift = half ? 4 : 0;
        uint8_t sc, m;
        ogo_get_scale_min_k4(g * 2 + half, scales, &sc, &m);
        int8_t *w = out->q + (sb + (size_t)half) * 32;
        for (int j = 0; j < 32; j++) w[j] = (int8_t)((bytes[j] >> shift) & 0x0F);
        out->sc[sb + (size_t)half] = (int16_t)sc;
        out->mins[sb + (size_t)half] = (int16_t)m;
      }
      sb += 2;
    }
  }
}

/* vecdot.rs:2064-2088 unpack_k_q5_k: unpack_k_q4_k with the high-bit plane applied */
static void unpack_k_q5_k(const uint8_t *row, size_t in_dim, ogo_krow *out) {
  size_t sb = 0;
  for (size_t s = 0; s < in_dim / 256; s++) {
    const uint8_t *block = row + s * 176;
    out->d[s] = read_f16(block, 0);
    out->dmin[s] = read_f16(block, 2);
    const uint8_t *scales = block + 4;
    const uint8_t *qh = block + 16;
    const uint8_t *qs = block + 48;
    for (int g = 0; g < 4; g++) {
      const uint8_t *bytes = qs + g * 32;
      for (int half = 0; half < 2; half++) {
        int shift = half ? 4 : 0;
        uint8_t sc, m;
        ogo_get_scale_min_k4(g * 2 + half, scales, &sc, &m);
        uint8_t hi_mask = (uint8_t)(1u << (g * 2 + half));
        int8_t *w = out->q + (sb + (size_t)half) * 32;
        for (int j = 0; j < 32; j++)
          w[j] = (int8_t)(((bytes[j] >> shift) & 0x0F) + ((qh[j] & hi_mask) ? 16 : 0));
        out->sc[sb + (size_t)half] = (int16_t)sc;
        out->mins[sb + (size_t)half] = (int16_t)m;
      }
      sb += 2;
    }
  }
}

/* vecdot.rs:1098-1107 Q2K_RUNS: (qs byte offset, low-bit shift) of the eight 32-element runs */
static const struct { size_t off; int shift; } Q2K_RUNS[8] = {
    {0, 0}, {0, 2}, {0, 4}, {0, 6}, {32, 0}, {32, 2}, {32, 4}, {32, 6}};

/* vecdot.rs:1117-1121 unpack_q2k_run */
static inline void unpack_q2k_run(const uint8_t *qs, int shift, int8_t *w) {
  for (int j = 0; j < 32; j++) w[j] = (int8_t)((qs[j] >> shift) & 3);
}

/* vecdot.rs:2333-2350 unpack_k_iq4_xs */
static void unpack_k_iq4_xs(const uint8_t *row, size_t in_dim, ogo_krow *out) {
  for (size_t s = 0; s < in_dim / 256; s++) {
    const uint8_t *block = row + s * 136;
    out->d[s] = read_f16(block, 0);
    for (int ib = 0; ib < 8; ib++) {
      out->sc[s * 8 + (size_t)ib] = (int16_t)iq4_xs_scale(block, ib);
      unpack_block_iq4_nl(block + 8 + ib * 16, out->q + (s * 8 + (size_t)ib) * 32);
    }
  }
}

/* vecdot.rs:1131-1136 unpack_q3k_run */
static inline void unpack_q3k_run(const uint8_t *qs, const uint8_t *hmask, int shift, uint8_t bit,
                                  int8_t *w) {
  for (int j = 0; j < 32; j++) {
    int8_t lo = (int8_t)((qs[j] >> shift) & 3);
    w[j] = (int8_t)(lo - ((hmask[j] & bit) ? 0 : 4));
  }
}

/* vecdot.rs:2100-2117 unpack_k_q3_k: a KKind::Q6K row (per-16 integer scales sc - 32) */
static void unpack_k_q3_k(const uint8_t *row, size_t in_dim, ogo_krow *out) {
  for (size_t s = 0; s < in_dim / 256; s++) {
    const uint8_t *block = row + s * 110;
    const uint8_t *hmask = block, *qs = block + 32;
    int32_t sc[16];
    ogo_unpack_q3_k_scales(block + 96, sc);
    out->d[s] = read_f16(block, 108);
    size_t base = s * 256;
    for (int p = 0; p < 8; p++) {
      size_t e0 = base + (size_t)p * 32;
      unpack_q3k_run(qs + Q2K_RUNS[p].off, hmask, Q2K_RUNS[p].shift, (uint8_t)(1u << p), out->q + e0);
      size_t gi = e0 / 16;
      out->sc[gi] = (int16_t)(sc[2 * p] - 32);
      out->sc[gi + 1] = (int16_t)(sc[2 * p + 1] - 32);
    }
  }
}

/* vecdot.rs:2119-2143 unpack_k_q6_k */
static void unpack_k_q6_k(const uint8_t *row, size_t in_dim, ogo_krow *out) {
  for (size_t s = 0; s < in_dim / 256; s++) {
    const uint8_t *block = row + s * 210;
    const uint8_t *ql = block, *qh = block + 128, *sc = block + 192;
    out->d[s] = read_f16(block, 208);
    size_t base = s * 256;
    for (size_t h = 0; h < 2; h++) {
      const uint8_t *qh_run = qh + h * 32;
      for (size_t run = 0; run < 4; run++) {
        size_t e0 = base + h * 128 + run * 32;
        const uint8_t *ql_run = ql + h * 64 + Q6K_RUNS[run].ql_add;
        int8_t *w = out->q + e0;
        for (int l = 0; l < 32; l++) {
          uint8_t nib = Q6K_RUNS[run].high ? (uint8_t)(ql_run[l] >> 4) : (uint8_t)(ql_run[l] & 0x0F);
          w[l] = (int8_t)((int8_t)(nib | (uint8_t)(((qh_run[l] >> Q6K_RUNS[run].hshift) & 3) << 4)) -
                          32);
        }
        size_t gi = e0 / 16;
        out->sc[gi] = (int16_t)(int8_t)sc[gi % 16];
        out->sc[gi + 1] = (int16_t)(int8_t)sc[(gi + 1) % 16];
      }
    }
  }
}

/* vecdot.rs:2402-2406 store_tile */
static inline void store_tile(size_t tl, const float *acc, float *out, size_t n_tokens) {
  size_t base = tl * 4;
  for (size_t k = 0; k < 4 && base + k < n_tokens; k++) out[base + k] = acc[k];
}

/* ------------------------------------------------------------------ ISA copies */

#define OGO_FN(name) name##_scalar
#define OGO_TARGET
#include "oracle_kernels.inc"
#undef OGO_FN
#undef OGO_TARGET

#if defined(__x86_64__)
#define OGO_HAVE_AVX2_BUILD 1
#define OGO_FN(name) name##_avx2
#define OGO_TARGET __attribute__((target("avx2")))
#define OGO_USE_AVX2 1
#include "oracle_kernels.inc"
#undef OGO_FN
#undef OGO_TARGET
#undef OGO_USE_AVX2
#endif

static int g_force_scalar = 0;

static int use_avx2(void) {
#ifdef OGO_HAVE_AVX2_BUILD
  static int cached = -1;
  if (cached < 0) {
    __builtin_cpu_init();
    cached = __builtin_cpu_supports("avx2") ? 1 : 0;
  }
  return cached && !g_force_scalar;
#else
  return 0;
#endif
}

/* Test hook: force the scalar integer dots so the two ISA copies can be compared. */
void ogo_force_scalar(int on) { g_force_scalar = on; }

const char *ogo_isa_name(void) { return use_avx2() ? "avx2" : "scalar"; }

#ifdef OGO_HAVE_AVX2_BUILD
#define DISPATCH(name, ...) (use_avx2() ? name##_avx2(__VA_ARGS__) : name##_scalar(__VA_ARGS__))
#else
#define DISPATCH(name, ...) name##_scalar(__VA_ARGS__)
#endif

int32_t ogo_dot16_scalar(const int8_t *w, const int8_t *x) { return dot16_scalar(w, x); }
int32_t ogo_dot16(const int8_t *w, const int8_t *x) { return DISPATCH(dot16, w, x); }
int32_t ogo_dot32(const int8_t *w, const int8_t *x) { return DISPATCH(dot32, w, x); }

float ogo_dot_q8_0(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d) {
  return DISPATCH(dot_q8_0, row, in_dim, q, d, NULL);
}
float ogo_dot_flat32(uint32_t ggml_type, const uint8_t *row, size_t in_dim, const int8_t *q,
                     const float *d, int32_t *isum_out) {
  return DISPATCH(dot_flat32, ggml_type, row, in_dim, q, d, isum_out);
}
void ogo_block_sums_q8_0(const uint8_t *row, size_t in_dim, const int8_t *q, int32_t *isum_out) {
  float *d = (float *)calloc(in_dim / 32, sizeof(float));
  (void)DISPATCH(dot_q8_0, row, in_dim, q, d, isum_out);
  free(d);
}
float ogo_dot_q4_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                   const int32_t *sums) {
  return DISPATCH(dot_q4_k, row, in_dim, q, d, sums);
}
float ogo_dot_q6_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d) {
  return DISPATCH(dot_q6_k, row, in_dim, q, d);
}
float ogo_dot_k_row_q4_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                         const int32_t *sums, int32_t *isum_out, int32_t *imin_out) {
  return DISPATCH(dot_k_row_q4_k, row, in_dim, q, d, sums, isum_out, imin_out);
}
float ogo_dot_k_row_q5_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                         const int32_t *sums, int32_t *isum_out, int32_t *imin_out) {
  return DISPATCH(dot_k_row_q5_k, row, in_dim, q, d, sums, isum_out, imin_out);
}
float ogo_dot_k_row_q6_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                         int32_t *isum_out) {
  return DISPATCH(dot_k_row_q6_k, row, in_dim, q, d, isum_out);
}
float ogo_dot_q5_1(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d, const int32_t *sums,
                   int32_t *isum_out) {
  return DISPATCH(dot_q5_1, row, in_dim, q, d, sums, isum_out);
}
float ogo_dot_k_row_iq4_xs(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d, int32_t *isum_out) {
  return DISPATCH(dot_k_row_iq4_xs, row, in_dim, q, d, isum_out);
}
float ogo_dot_k_row_q2_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d, const int32_t *sums,
                         int32_t *isum_out, int32_t *imin_out) {
  return DISPATCH(dot_k_row_q2_k, row, in_dim, q, d, sums, isum_out, imin_out);
}
float ogo_dot_unpacked_q2_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d, const int32_t *sums) {
  return DISPATCH(dot_unpacked_q2_k, row, in_dim, q, d, sums);
}
float ogo_dot_k_row_q3_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                         int32_t *isum_out) {
  return DISPATCH(dot_k_row_q3_k, row, in_dim, q, d, isum_out);
}

/* ------------------------------------------------------------------ predicates */

/* vecdot.rs:274-283 */
int ogo_supports(uint32_t t, size_t in_dim) {
  if (t == OGO_TYPE_Q8_0 || t == OGO_TYPE_Q5_0 || t == OGO_TYPE_Q4_0 || t == OGO_TYPE_Q5_1 || t == OGO_TYPE_IQ4_NL)
    return in_dim % 32 == 0;
  if (t == OGO_TYPE_Q2_K || t == OGO_TYPE_Q3_K || t == OGO_TYPE_Q4_K || t == OGO_TYPE_Q5_K || t == OGO_TYPE_Q6_K ||
      t == OGO_TYPE_IQ4_XS)
    return in_dim % 256 == 0;
  return 0;
}
/* vecdot.rs:1821-1826 */
int ogo_supports_k(uint32_t t, size_t in_dim) {
  return (t == OGO_TYPE_Q3_K || t == OGO_TYPE_Q4_K || t == OGO_TYPE_Q5_K || t == OGO_TYPE_Q6_K || t == OGO_TYPE_IQ4_XS) &&
         in_dim % 256 == 0;
}
/* vecdot.rs:3083-3093 */
int ogo_supports_k_row(uint32_t t, size_t in_dim) {
  return (t == OGO_TYPE_Q2_K || t == OGO_TYPE_Q3_K || t == OGO_TYPE_Q4_K || t == OGO_TYPE_Q5_K || t == OGO_TYPE_Q6_K ||
          t == OGO_TYPE_IQ4_XS) &&
         in_dim % 256 == 0;
}
/* vecdot.rs:2456-2461 */
int ogo_supports_flat(uint32_t t, size_t in_dim) {
  return (t == OGO_TYPE_Q8_0 || t == OGO_TYPE_Q5_0 || t == OGO_TYPE_Q4_0 || t == OGO_TYPE_IQ4_NL) && in_dim % 32 == 0;
}

/* ------------------------------------------------------------------ CpuBackend */

int ogo_host_threads(void) {
#ifdef _OPENMP
  return omp_get_num_procs();
#else
  return 1;
#endif
}

static int pick_threads(int n_threads) {
  int all = ogo_host_threads();
  if (n_threads <= 0 || n_threads > all) return all;
  return n_threads;
}

/* backend/cpu.rs:385-396 finish_into: [out_dim][n_tokens] -> [n_tokens][out_dim] */
static void finish_into(float *y, const float *yt, size_t n_tokens, size_t out_dim) {
  if (n_tokens == 1) {
    memcpy(y, yt, out_dim * sizeof(float));
    return;
  }
  for (size_t o = 0; o < out_dim; o++)
    for (size_t t = 0; t < n_tokens; t++) y[t * out_dim + o] = yt[o * n_tokens + t];
}

/* vecdot.rs:2151-2172 dot_k_pair dispatch by kind */
static void dot_k_pair(uint32_t ggml_type, const ogo_krow *w0, const ogo_krow *w1,
                       const ogo_actq8k *a, float *out0, float *out1) {
  if (ggml_type == OGO_TYPE_Q4_K || ggml_type == OGO_TYPE_Q5_K) {   /* both fill a KKind::Q4K row */
    DISPATCH(gemm_k_q4_k, w0, w1, a, out0, out1);
  } else if (ggml_type == OGO_TYPE_IQ4_XS) {
    DISPATCH(gemm_k_iq4_xs, w0, w1, a, out0, out1);
  } else {
    DISPATCH(gemm_k_q6_k, w0, w1, a, out0, out1);
  }
}

static void unpack_k_row(uint32_t ggml_type, const uint8_t *row, size_t in_dim, ogo_krow *out) {
  if (ggml_type == OGO_TYPE_Q4_K) {
    unpack_k_q4_k(row, in_dim, out);
  } else if (ggml_type == OGO_TYPE_Q5_K) {
    unpack_k_q5_k(row, in_dim, out);
  } else if (ggml_type == OGO_TYPE_Q3_K) {
    unpack_k_q3_k(row, in_dim, out);
  } else if (ggml_type == OGO_TYPE_IQ4_XS) {
    unpack_k_iq4_xs(row, in_dim, out);
  } else {
    unpack_k_q6_k(row, in_dim, out);
  }
}

/* backend/cpu.rs:173-203 matmul_k_gemm_into; yt is [out_dim][n_tokens] */
static int k_gemm_t(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                    size_t out_dim, const float *x, size_t n_tokens, float *yt, int threads) {
  ogo_actq8k a;
  a.n_tokens = n_tokens;
  a.n_block = in_dim / 32;
  a.n_super = in_dim / 256;
  a.n_tile = (n_tokens + 3) / 4;
  a.q = (int8_t *)calloc(a.n_tile * a.n_block * 4 * 32, 1);
  a.d = (float *)calloc(a.n_tile * a.n_super * 4, sizeof(float));
  a.bsum = (int16_t *)calloc(a.n_tile * a.n_super * 4 * 8, sizeof(int16_t));
  if (!a.q || !a.d || !a.bsum) return -3;
  ogo_act_q8k_quantize(x, in_dim, n_tokens, a.q, a.d, a.bsum);
  size_t n_pair = (out_dim + 1) / 2;
  int failed = 0;
#pragma omp parallel num_threads(threads)
  {
    ogo_krow s0, s1;
    float *scratch = (float *)malloc(sizeof(float) * n_tokens);
    int ok = krow_alloc(&s0, in_dim) == 0 && krow_alloc(&s1, in_dim) == 0 && scratch;
    if (!ok) {
#pragma omp atomic write
      failed = 1;
    }
#pragma omp for schedule(dynamic, 8)
    for (size_t pair = 0; pair < n_pair; pair++) {
      if (!ok) continue;
      size_t o0 = pair * 2;
      unpack_k_row(ggml_type, raw + o0 * row_bytes, in_dim, &s0);
      if (o0 + 1 < out_dim) {
        unpack_k_row(ggml_type, raw + (o0 + 1) * row_bytes, in_dim, &s1);
        dot_k_pair(ggml_type, &s0, &s1, &a, yt + o0 * n_tokens, yt + (o0 + 1) * n_tokens);
      } else {
        /* vecdot.rs:2207-2211 dot_k_multi: the row against itself, duplicate discarded */
        dot_k_pair(ggml_type, &s0, &s0, &a, yt + o0 * n_tokens, scratch);
      }
    }
    krow_free(&s0);
    krow_free(&s1);
    free(scratch);
  }
  free(a.q);
  free(a.d);
  free(a.bsum);
  return failed ? -3 : 0;
}

int ogo_k_gemm_t(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                 size_t out_dim, const float *x, size_t n_tokens, float *yt) {
  if (!ogo_supports_k(ggml_type, in_dim)) return -1;
  return k_gemm_t(ggml_type, raw, row_bytes, in_dim, out_dim, x, n_tokens, yt, 1);
}

/* backend/cpu.rs:209-245 matmul_flat_gemm_into: unpack_q8_0 / _q5_0 / _q4_0 / _iq4_nl
 * (vecdot.rs:1246-1296, 1351-1362) then dot_flat_pair */
static int flat_gemm_t(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim, size_t out_dim,
                       const float *x, size_t n_tokens, float *yt, int threads) {
  ogo_actq8flat a;
  a.n_tokens = n_tokens;
  a.n_block = in_dim / 32;
  a.n_tile = (n_tokens + 3) / 4;
  a.q = (int8_t *)calloc(a.n_tile * a.n_block * 4 * 32, 1);
  a.d = (float *)calloc(a.n_tile * a.n_block * 4, sizeof(float));
  if (!a.q || !a.d) return -3;
  ogo_act_q8flat_quantize(x, in_dim, n_tokens, a.q, a.d);
  size_t n_pair = (out_dim + 1) / 2;
  size_t nb = in_dim / 32;
  size_t bb, be;
  ogo_block_layout(ggml_type, &bb, &be);
#pragma omp parallel num_threads(threads)
  {
    int8_t *q0 = (int8_t *)malloc(in_dim), *q1 = (int8_t *)malloc(in_dim);
    float *s0 = (float *)malloc(sizeof(float) * nb), *s1 = (float *)malloc(sizeof(float) * nb);
    float *scratch = (float *)malloc(sizeof(float) * n_tokens);
#pragma omp for schedule(dynamic, 8)
    for (size_t pair = 0; pair < n_pair; pair++) {
      size_t o0 = pair * 2;
      const uint8_t *r0 = raw + o0 * row_bytes;
      for (size_t b = 0; b < nb; b++) s0[b] = ogo_unpack_flat_block(ggml_type, r0 + b * bb, q0 + b * 32);
      if (o0 + 1 < out_dim) {
        const uint8_t *r1 = raw + (o0 + 1) * row_bytes;
        for (size_t b = 0; b < nb; b++) s1[b] = ogo_unpack_flat_block(ggml_type, r1 + b * bb, q1 + b * 32);
        DISPATCH(dot_flat_pair, q0, s0, q1, s1, &a, yt + o0 * n_tokens, yt + (o0 + 1) * n_tokens);
      } else {
        DISPATCH(dot_flat_pair, q0, s0, q0, s0, &a, yt + o0 * n_tokens, scratch);
      }
    }
    free(q0);
    free(q1);
    free(s0);
    free(s1);
    free(scratch);
  }
  free(a.q);
  free(a.d);
  return 0;
}

/* One GEMV per (row, token) with the kernel cpu.rs picks at n_tokens == 1; yt is
 * [out_dim][n_tokens].  Shared by matmul at T == 1 (cpu.rs:100-137) and matmul_decode at any T
 * (cpu.rs:265-317). */
/* generic: the rows-unpacked-once path of matmul at n_tokens > 1 for a type with neither a K GEMM nor a
 * flat one (cpu.rs:113-163): per-32 activations for every type.  Per token it is dot_unpacked_impl's
 * arithmetic, which for Q5_1 equals dot_q5_1's bit for bit (scale * isum - (-m) * bsum) and for Q2_K
 * does not equal dot_k_row_q2_k's. */
static int gemv_t(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                  size_t out_dim, const float *x, size_t n_tokens, float *yt, int threads,
                  int32_t *isum_out, int32_t *imin_out, int generic) {
  int k_row = !generic && ogo_supports_k_row(ggml_type, in_dim);
  size_t n_d = k_row ? in_dim / 256 : in_dim / 32;
  int8_t *q = (int8_t *)malloc(n_tokens * in_dim);
  float *d = (float *)malloc(sizeof(float) * n_tokens * n_d);
  int32_t *sums = (int32_t *)malloc(sizeof(int32_t) * n_tokens * (in_dim / 16));
  if (!q || !d || !sums) return -3;
  for (size_t t = 0; t < n_tokens; t++) {
    if (k_row)
      ogo_quantize_act_k_row(x + t * in_dim, in_dim, q + t * in_dim, d + t * n_d,
                             sums + t * (in_dim / 16));
    else
      ogo_quantize_act(x + t * in_dim, in_dim, q + t * in_dim, d + t * n_d,
                       sums + t * (in_dim / 16));
  }
  long long n_out = (long long)out_dim;
#pragma omp parallel for schedule(dynamic, 16) num_threads(threads)
  for (long long oo = 0; oo < n_out; oo++) {
    size_t o = (size_t)oo;
    const uint8_t *row = raw + o * row_bytes;
    for (size_t t = 0; t < n_tokens; t++) {
      const int8_t *qt = q + t * in_dim;
      const float *dt = d + t * n_d;
      const int32_t *st = sums + t * (in_dim / 16);
      int32_t *io = isum_out ? isum_out + (t * out_dim + o) * n_d : NULL;
      int32_t *mo = imin_out ? imin_out + (t * out_dim + o) * n_d : NULL;
      float v;
      if (ggml_type == OGO_TYPE_Q4_K)
        v = DISPATCH(dot_k_row_q4_k, row, in_dim, qt, dt, st, io, mo);
      else if (ggml_type == OGO_TYPE_Q5_K)
        v = DISPATCH(dot_k_row_q5_k, row, in_dim, qt, dt, st, io, mo);
      else if (ggml_type == OGO_TYPE_Q6_K)
        v = DISPATCH(dot_k_row_q6_k, row, in_dim, qt, dt, io);
      else if (ggml_type == OGO_TYPE_Q3_K)
        v = DISPATCH(dot_k_row_q3_k, row, in_dim, qt, dt, io);
      else if (ggml_type == OGO_TYPE_IQ4_XS)
        v = DISPATCH(dot_k_row_iq4_xs, row, in_dim, qt, dt, io);
      else if (ggml_type == OGO_TYPE_Q2_K)
        v = generic ? DISPATCH(dot_unpacked_q2_k, row, in_dim, qt, dt, st)
                    : DISPATCH(dot_k_row_q2_k, row, in_dim, qt, dt, st, io, mo);
      else if (ggml_type == OGO_TYPE_Q5_1)
        v = DISPATCH(dot_q5_1, row, in_dim, qt, dt, st, io);
      else if (ggml_type == OGO_TYPE_Q8_0)
        v = DISPATCH(dot_q8_0, row, in_dim, qt, dt, io);
      else
        v = DISPATCH(dot_flat32, ggml_type, row, in_dim, qt, dt, io);
      yt[o * n_tokens + t] = v;
    }
  }
  free(q);
  free(d);
  free(sums);
  return 0;
}

/* The single-token GEMV of gemv_t over an activation that is already quantized (q, d and the per-16
 * sums as quantize_act / quantize_act_k_row leave them): the same dot_row / dot_k_row calls, so a
 * test can continue from a device's int8 activations.  y is [out_dim]. */
int ogo_gemv_act(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim, size_t out_dim,
                 const int8_t *q, const float *d, const int32_t *sums, float *y, int n_threads) {
  if (!ogo_supports(ggml_type, in_dim)) return -1;
  int threads = pick_threads(n_threads);
  long long n_out = (long long)out_dim;
#pragma omp parallel for schedule(dynamic, 16) num_threads(threads)
  for (long long oo = 0; oo < n_out; oo++) {
    const uint8_t *row = raw + (size_t)oo * row_bytes;
    float v;
    if (ggml_type == OGO_TYPE_Q4_K)
      v = DISPATCH(dot_k_row_q4_k, row, in_dim, q, d, sums, NULL, NULL);
    else if (ggml_type == OGO_TYPE_Q5_K)
      v = DISPATCH(dot_k_row_q5_k, row, in_dim, q, d, sums, NULL, NULL);
    else if (ggml_type == OGO_TYPE_Q6_K)
      v = DISPATCH(dot_k_row_q6_k, row, in_dim, q, d, NULL);
    else if (ggml_type == OGO_TYPE_Q3_K)
      v = DISPATCH(dot_k_row_q3_k, row, in_dim, q, d, NULL);
    else if (ggml_type == OGO_TYPE_IQ4_XS)
      v = DISPATCH(dot_k_row_iq4_xs, row, in_dim, q, d, NULL);
    else if (ggml_type == OGO_TYPE_Q2_K)
      v = DISPATCH(dot_k_row_q2_k, row, in_dim, q, d, sums, NULL, NULL);
    else if (ggml_type == OGO_TYPE_Q5_1)
      v = DISPATCH(dot_q5_1, row, in_dim, q, d, sums, NULL);
    else if (ggml_type == OGO_TYPE_Q8_0)
      v = DISPATCH(dot_q8_0, row, in_dim, q, d, NULL);
    else
      v = DISPATCH(dot_flat32, ggml_type, row, in_dim, q, d, NULL);
    y[oo] = v;
  }
  return 0;
}

/* backend/cpu.rs:55-167 matmul_fused_into + :445-458 */
int ogo_matmul(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
               size_t out_dim, const float *x, size_t n_tokens, float *y, int n_threads) {
  if (!ogo_supports(ggml_type, in_dim)) return -1;
  if (n_tokens == 0 || out_dim == 0) return 0;
  int threads = pick_threads(n_threads);
  float *yt = (float *)malloc(sizeof(float) * out_dim * n_tokens);
  if (!yt) return -3;
  int rc;
  if (n_tokens > 1 && ogo_supports_k(ggml_type, in_dim))
    rc = k_gemm_t(ggml_type, raw, row_bytes, in_dim, out_dim, x, n_tokens, yt, threads);
  else if (n_tokens > 1 && ogo_supports_flat(ggml_type, in_dim))
    rc = flat_gemm_t(ggml_type, raw, row_bytes, in_dim, out_dim, x, n_tokens, yt, threads);
  else
    rc = gemv_t(ggml_type, raw, row_bytes, in_dim, out_dim, x, n_tokens, yt, threads, NULL, NULL, n_tokens > 1);
  if (rc == 0) finish_into(y, yt, n_tokens, out_dim);
  free(yt);
  return rc;
}

/* backend/cpu.rs:265-317 matmul_fused_decode_into + :466-480 */
int ogo_matmul_decode(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                      size_t out_dim, const float *x, size_t n_tokens, float *y, int n_threads) {
  if (!ogo_supports(ggml_type, in_dim)) return -1;
  if (n_tokens == 0 || out_dim == 0) return 0;
  int threads = pick_threads(n_threads);
  float *yt = (float *)malloc(sizeof(float) * out_dim * n_tokens);
  if (!yt) return -3;
  int rc = gemv_t(ggml_type, raw, row_bytes, in_dim, out_dim, x, n_tokens, yt, threads, NULL, NULL, 0);
  if (rc == 0) finish_into(y, yt, n_tokens, out_dim);
  free(yt);
  return rc;
}

/* The integer stage on its own.  Both K-quant quantizers (per-256) produce the same int8 and
 * sums, so GEMV and GEMM share these values (vecdot.rs:1858-1910 vs 3030-3053). */
int ogo_block_sums(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                   size_t out_dim, const float *x, size_t n_tokens, int32_t *isum, int32_t *imin) {
  if (!ogo_supports(ggml_type, in_dim)) return -1;
  float *yt = (float *)malloc(sizeof(float) * out_dim * n_tokens);
  if (!yt) return -3;
  int rc = gemv_t(ggml_type, raw, row_bytes, in_dim, out_dim, x, n_tokens, yt, pick_threads(0), isum,
                  (ggml_type == OGO_TYPE_Q4_K || ggml_type == OGO_TYPE_Q5_K || ggml_type == OGO_TYPE_Q2_K) ? imin : NULL, 0);
  free(yt);
  return rc;
}

/* backend/cpu.rs:409-432 matmul_dequant: dequantize(row) . x with unquantized activations.  The
 * reference's tensor::dot uses FMA lanes on x86, so its bits are ISA-dependent; this sums in f32
 * left to right, which is what the reference's own tests do (vecdot.rs:3487-3492).  A float
 * yardstick for budget checks, never a bit-exact target. */
int ogo_matmul_dequant(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                       size_t out_dim, const float *x, size_t n_tokens, float *y, int n_threads) {
  size_t bb, be;
  if (ogo_block_layout(ggml_type, &bb, &be) != 0 || in_dim % be != 0) return -1;
  int threads = pick_threads(n_threads);
  long long n_out = (long long)out_dim;
#pragma omp parallel num_threads(threads)
  {
    float *w = (float *)malloc(sizeof(float) * in_dim);
#pragma omp for schedule(dynamic, 16)
    for (long long oo = 0; oo < n_out; oo++) {
      size_t o = (size_t)oo;
      ogo_dequantize(ggml_type, raw + o * row_bytes, in_dim, w);
      for (size_t t = 0; t < n_tokens; t++) {
        const float *xs = x + t * in_dim;
        float acc = 0.0f;
        for (size_t i = 0; i < in_dim; i++) acc += w[i] * xs[i];
        y[t * out_dim + o] = acc;
      }
    }
    free(w);
  }
  return 0;
}
