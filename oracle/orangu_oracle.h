/*
 * orangu_oracle.h -- CPU restatement of orangu-server's quantized vec_dot / matmul path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It exists to check the HIP kernels and to
 * be timed as the CPU baseline.  Only tests, the smoke check and the benchmark's cpu_baseline
 * leg may load it; the shipped library never calls into it and has no CPU fallback.
 *
 * Every function follows the *scalar* definition in the reference, operation for operation:
 * IEEE-754 binary32, each operation rounded on its own (build with -ffp-contract=off, never
 * -ffast-math), roundf (ties away from zero), fmaxf (ignores a NaN operand), saturating
 * float->int8 with NaN -> 0.  Integer dots may run on AVX2: integer sums are exact, so the
 * ISA cannot change a bit (the reference does the same, vecdot.rs:751-781).
 *
 * Reference files (paths relative to src/bin/orangu-server/engine/ of orangu 1.2.0):
 *   quant.rs      block formats, f16 decode, dequantize
 *   vecdot.rs     activation quantizers, fused GEMV and GEMM kernels
 *   backend/cpu.rs  kernel choice per (type, n_tokens, entry point)
 *
 * Pinning (what each part is checked against, without running the reference):
 *   dequantize / f16 / get_scale_min_k4   golden bit checksums quant.rs:1389-1463 (q8_0, q4_0, q5_0,
 *   / unpack_q3_k_scales / block unpacks  iq4_nl, q3_k, q4_k, q5_k, q6_k) and the hand-built blocks
 *                                         quant.rs:1768-1921, vecdot.rs:3866-3968, 4141-4165,
 *                                         4226-4237                              -> PINNED
 *   quantizers                            ties-away, zero block, adversarial blocks
 *                                         vecdot.rs:4259-4410 (expected bytes derived by hand
 *                                         from the stated rules)                 -> PINNED
 *   integer dots                          known-answer cases vecdot.rs:577-594, brute force
 *                                                                                -> PINNED
 *   fused GEMV / GEMM values              closed-form budgets against dequantize . x
 *                                         (vecdot.rs:3436-3526, 4011-4040, 4479-4506), exact
 *                                         invariants (batch independence, decode == alone,
 *                                         flat GEMM == GEMV)                     -> PINNED to
 *                                         the budget; the exact f32 bits of these outputs have
 *                                         no golden vector in the reference: "parity unpinned"
 *                                         at bit level, pinned by construction (same operation
 *                                         order) and by the budgets above.
 */
#ifndef ORANGU_ORACLE_H
#define ORANGU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids, quant.rs:50-61 */
#define OGO_TYPE_F32 0u
#define OGO_TYPE_F16 1u
#define OGO_TYPE_Q4_0 2u
#define OGO_TYPE_Q5_0 6u
#define OGO_TYPE_Q5_1 7u
#define OGO_TYPE_Q8_0 8u
#define OGO_TYPE_Q2_K 10u
#define OGO_TYPE_Q3_K 11u
#define OGO_TYPE_Q4_K 12u
#define OGO_TYPE_Q5_K 13u
#define OGO_TYPE_Q6_K 14u
#define OGO_TYPE_IQ4_NL 20u
#define OGO_TYPE_IQ4_XS 23u

#define OGO_ACT_BLOCK 32   /* vecdot.rs ACT_BLOCK */
#define OGO_GROUP 16       /* vecdot.rs:63 */
#define OGO_SUPER_BLOCK 256
#define OGO_SUBS 8
#define OGO_TOKEN_TILE 4

/* ---- formats (quant.rs) ---- */
float ogo_f16_bits_to_f32(uint16_t bits);                                  /* quant.rs:511-528 */
void ogo_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m); /* quant.rs:653-662 */
int ogo_block_layout(uint32_t ggml_type, size_t *block_bytes, size_t *block_elems); /* quant.rs:132-169 */
int64_t ogo_tensor_byte_size(uint32_t ggml_type, uint64_t element_count);  /* quant.rs:344-357 */
int ogo_dequantize(uint32_t ggml_type, const uint8_t *bytes, size_t element_count, float *out);
                                                       /* quant.rs:639-649, 666-697, 746-787 */

/* ---- the reference's deterministic test fixtures ---- */
void ogo_fixture_bytes(size_t len, uint8_t *out);                          /* quant.rs:1427-1437 */
uint64_t ogo_bit_checksum(const float *values, size_t n);                  /* quant.rs:1442-1446 */
void ogo_pseudo_bytes(size_t n, uint32_t seed, uint8_t *out);              /* vecdot.rs:3415-3423 */

/* ---- activation quantizers (vecdot.rs) ---- */
/* per-32 scale; q[n], d[n/32], sums[n/16]                      vecdot.rs:95-126 */
void ogo_quantize_act(const float *x, size_t n, int8_t *q, float *d, int32_t *sums);
/* per-256 scale; q[n], d[n/256], sums[n/16]                    vecdot.rs:3030-3053 */
void ogo_quantize_act_k_row(const float *x, size_t n, int8_t *q, float *d, int32_t *sums);
/* ActQ8K: q[tile][n/32][4][32], d[tile][n/256][4], bsum[tile][n/256][4][8]; caller zero-fills.
 * vecdot.rs:1858-1910 */
void ogo_act_q8k_quantize(const float *x, size_t in_dim, size_t n_tokens, int8_t *q, float *d,
                          int16_t *bsum);
/* ActQ8Flat: q[tile][n/32][4][32], d[tile][n/32][4]; caller zero-fills.  vecdot.rs:2483-2525 */
void ogo_act_q8flat_quantize(const float *x, size_t in_dim, size_t n_tokens, int8_t *q, float *d);

/* ---- integer dots (exact) ---- */
int32_t ogo_dot16_scalar(const int8_t *w, const int8_t *x);                /* vecdot.rs:801-807 */
int32_t ogo_dot16(const int8_t *w, const int8_t *x); /* best ISA on this host, same value */
int32_t ogo_dot32(const int8_t *w, const int8_t *x);
const char *ogo_isa_name(void);

/* ---- GEMV: one row, one token ---- */
float ogo_dot_q8_0(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d); /* :2829-2838 */
float ogo_dot_q4_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                   const int32_t *sums);                                  /* per-32 form :2904-2930 */
float ogo_dot_q6_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d); /* :3379-3406 */
/* per-256 forms; isum_out/imin_out (may be NULL) receive the per-super-block integer sums */
float ogo_dot_k_row_q4_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                         const int32_t *sums, int32_t *isum_out, int32_t *imin_out); /* :3152-3178 */
float ogo_dot_k_row_q5_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                         const int32_t *sums, int32_t *isum_out, int32_t *imin_out); /* :3181-3213 */
float ogo_dot_k_row_q6_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                         int32_t *isum_out);                                          /* :3215-3241 */
/* vecdot.rs:2886-2899 dot_q5_1 (per-32 activations; sums are the per-16 sums of quantize_act) */
float ogo_dot_q5_1(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d, const int32_t *sums,
                   int32_t *isum_out);
/* vecdot.rs:3245-3266 dot_k_row_iq4_xs, :3296-3318 dot_k_row_q2_k (per-256 activations) */
float ogo_dot_k_row_iq4_xs(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d, int32_t *isum_out);
float ogo_dot_k_row_q2_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d, const int32_t *sums,
                         int32_t *isum_out, int32_t *imin_out);
/* vecdot.rs:1144-1164 unpack_q2_k + :407-428 dot_unpacked_impl: Q2_K against per-32 activations, a term per
 * group of 16 (the prefill path of a type that supports_k leaves out) */
float ogo_dot_unpacked_q2_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d, const int32_t *sums);
float ogo_dot_k_row_q3_k(const uint8_t *row, size_t in_dim, const int8_t *q, const float *d,
                         int32_t *isum_out);                                          /* :3273-3292 */
/* quant.rs:883-897: the 16 six-bit scales of a Q3_K block, still biased by 32 */
void ogo_unpack_q3_k_scales(const uint8_t *packed, int32_t *scales);
/* the other symmetric per-32 types (Q5_0, Q4_0, IQ4_NL): dot_q5_0 / dot_q4_0 / dot_iq4_nl,
 * vecdot.rs:2842-2883; isum_out (may be NULL) receives the per-32 integer sums */
float ogo_dot_flat32(uint32_t ggml_type, const uint8_t *row, size_t in_dim, const int8_t *q,
                     const float *d, int32_t *isum_out);
/* one block of such a type as 32 int8 weights (unpack_block_*, vecdot.rs:913-1039); returns dw */
float ogo_unpack_flat_block(uint32_t ggml_type, const uint8_t *block, int8_t *w);
/* per-32 integer sums of a Q8_0 row (isum_out[in_dim/32]) */
void ogo_block_sums_q8_0(const uint8_t *row, size_t in_dim, const int8_t *q, int32_t *isum_out);

/* ---- routing predicates ---- */
int ogo_supports(uint32_t ggml_type, size_t in_dim);        /* vecdot.rs:274-283 (3 types kept) */
int ogo_supports_k(uint32_t ggml_type, size_t in_dim);      /* vecdot.rs:1821-1826 */
int ogo_supports_k_row(uint32_t ggml_type, size_t in_dim);  /* vecdot.rs:3083-3093 */
int ogo_supports_flat(uint32_t ggml_type, size_t in_dim);   /* vecdot.rs:2456-2461 */

/* ---- CpuBackend (backend/cpu.rs) ----
 * x is [n_tokens][in_dim], y is [n_tokens][out_dim], both row-major host memory.
 * n_threads <= 0 means every host core (rayon's default pool, main.rs:2785-2788).
 * Returns 0, or -1 for a type / in_dim without a fused kernel. */
int ogo_matmul(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
               size_t out_dim, const float *x, size_t n_tokens, float *y, int n_threads);
                                                                    /* cpu.rs:55-245, 445-458 */
int ogo_gemv_act(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim, size_t out_dim,
                 const int8_t *q, const float *d, const int32_t *sums, float *y, int n_threads);
int ogo_matmul_decode(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                      size_t out_dim, const float *x, size_t n_tokens, float *y, int n_threads);
                                                                    /* cpu.rs:265-317 */
int ogo_matmul_dequant(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                       size_t out_dim, const float *x, size_t n_tokens, float *y, int n_threads);
                                                                    /* cpu.rs:409-432 */
/* The K-quant GEMM exactly as the reference's k_gemm test helper runs it, transposed result
 * yt[out_dim][n_tokens] (vecdot.rs:4450-4477). */
int ogo_k_gemm_t(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                 size_t out_dim, const float *x, size_t n_tokens, float *yt);
/* Per (token, row, super-block) integer sums of the matmul above, for bit-exact checks of the
 * integer stage: isum/imin are [n_tokens][out_dim][in_dim/256] (Q4_K, Q6_K; imin Q4_K only)
 * or isum [n_tokens][out_dim][in_dim/32] (Q8_0).  imin may be NULL. */
int ogo_block_sums(uint32_t ggml_type, const uint8_t *raw, size_t row_bytes, size_t in_dim,
                   size_t out_dim, const float *x, size_t n_tokens, int32_t *isum, int32_t *imin);

int ogo_host_threads(void);

#ifdef __cplusplus
}
#endif
#endif
