/*
 * orangu_mi355x.h -- C ABI of the MI355X (gfx950) quantized matmul backend for orangu-server.
 *
 * This is the boundary a Rust `impl Backend` binds through FFI.  It replaces, for the eleven GGUF types of the
 * reference's fused path (vecdot.rs:274-283: Q8_0, Q5_0, Q5_1, Q4_0, IQ4_NL, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K and
 * IQ4_XS), what `engine::backend::Backend` asks of a device
 * (src/bin/orangu-server/engine/backend/mod.rs:309-496) and reproduces the arithmetic of
 * `CpuBackend` (engine/backend/cpu.rs:55-317) over `engine::vecdot`:
 *   - activation int8 quantization, per-block integer sums: bit-exact with the CPU path;
 *   - f32 outputs: the per-block terms are combined in the CPU path's order, so they are
 *     bit-identical as well (the contract asked for is 1e-3 relative / 1e-5 absolute).
 *
 * Conventions
 *   - Every function returns OGM_OK (0) or a negative ogm_status.  Nothing aborts, throws or
 *     exits across this boundary (the existing vendor backends panic on a HIP error,
 *     engine/backend/rocm.rs:333-347; the shim decides what to do with a status).
 *   - `x` is [n_tokens][in_dim] f32 row-major, `y` is [n_tokens][out_dim] f32 row-major
 *     (backend/mod.rs:310-313).
 *   - Host-pointer entry points copy in and out and return when `y` is complete.  `_dev` entry
 *     points take device pointers, enqueue on `stream` (a hipStream_t, NULL = the context's own
 *     stream) and return without synchronizing.
 *   - A context is thread-safe: calls on one context serialize on an internal mutex, as
 *     RocmBackend does (engine/backend/rocm.rs:30-41).
 *   - There is no CPU fallback.  Without a usable gfx950 device ogm_init fails.
 */
#ifndef ORANGU_MI355X_H
#define ORANGU_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ogm_ctx ogm_ctx;       /* one device + stream + weight cache */
typedef struct ogm_weight ogm_weight; /* one uploaded, repacked QuantMatrix */

typedef enum ogm_status {
  OGM_OK = 0,
  OGM_ERR_INVALID = -1,     /* bad argument (null pointer, zero dimension, size mismatch) */
  OGM_ERR_UNSUPPORTED = -2, /* ggml type / in_dim without a kernel (vecdot.rs:274-283) */
  OGM_ERR_NO_DEVICE = -3,   /* no HIP device, or not a gfx950 */
  OGM_ERR_HIP = -4,         /* a HIP call failed; see ogm_last_error */
  OGM_ERR_OOM = -5          /* host or device allocation failed */
} ogm_status;

/* ggml type ids (engine/quant.rs:50-61) */
#define OGM_TYPE_Q4_0 2u
#define OGM_TYPE_Q5_0 6u
#define OGM_TYPE_Q5_1 7u
#define OGM_TYPE_Q8_0 8u
#define OGM_TYPE_Q2_K 10u
#define OGM_TYPE_Q3_K 11u
#define OGM_TYPE_Q4_K 12u
#define OGM_TYPE_Q5_K 13u
#define OGM_TYPE_Q6_K 14u
#define OGM_TYPE_IQ4_NL 20u
#define OGM_TYPE_IQ4_XS 23u

/* Activation quantization modes */
#define OGM_ACT_PER_32 0  /* vecdot::quantize_act,       vecdot.rs:79-126   (Q8_0 weights)   */
#define OGM_ACT_PER_256 1 /* vecdot::quantize_act_k_row, vecdot.rs:3030-3053 (K-quants)      */

/* ---- lifetime -------------------------------------------------------------------------- */

/* RocmBackend::try_init (engine/backend/rocm.rs:168-305): never aborts; a missing device is a
 * status.  `device` is the HIP ordinal. */
int ogm_init(int device, ogm_ctx **out);
/* Frees every weight and buffer of the context.  Drop of the backend. */
void ogm_destroy(ogm_ctx *ctx);
/* Text of the last failure on this context (or of the last failed ogm_init when ctx is NULL).
 * Valid until the next call on the same thread. */
const char *ogm_last_error(ogm_ctx *ctx);
/* RocmBackend::device_name (engine/backend/rocm.rs:307-316). */
int ogm_device_name(ogm_ctx *ctx, char *buf, size_t buf_len);

/* ---- capabilities ---------------------------------------------------------------------- */

/* Backend::supports_type (backend/mod.rs:493): 1 for Q8_0, Q5_0, Q4_0, IQ4_NL, Q3_K, Q4_K, Q5_K,
 * Q6_K, else 0. */
int ogm_supports_type(uint32_t ggml_type);
/* vecdot::supports (vecdot.rs:274-283) for those types: Q8_0 needs in_dim % 32 == 0, the
 * K-quants in_dim % 256 == 0. */
int ogm_supports(uint32_t ggml_type, uint32_t in_dim);
/* quant::block_layout (quant.rs:132-169).  Returns OGM_ERR_UNSUPPORTED for other types. */
int ogm_block_layout(uint32_t ggml_type, uint32_t *block_bytes, uint32_t *block_elems);

/* ---- weights: the uploader --------------------------------------------------------------- */

/* Bytes of the repacked ("tile-planar") form of a matrix: the raw GGUF blocks regrouped in tiles
 * of 64 blocks (R rows x C blocks, C = 4, 2 or 1) so that every 16-byte piece of a block lies in
 * a plane that 64 lanes read as one contiguous kilobyte; no bit of any block is altered and only
 * the rows that pad the last row block to R are zero. */
size_t ogm_repacked_size(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim);
/* Host-side repack and its exact inverse.  `raw` is QuantMatrix::raw_bytes()
 * (engine/loader.rs:608-610): out_dim rows of row_bytes. */
int ogm_repack_host(uint32_t ggml_type, const void *raw, size_t row_bytes, uint32_t in_dim,
                    uint32_t out_dim, void *repacked);
int ogm_unrepack_host(uint32_t ggml_type, const void *repacked, size_t row_bytes, uint32_t in_dim,
                      uint32_t out_dim, void *raw);

/* Uploads one QuantMatrix (engine/loader.rs:561-680): repacks `raw` and copies it to the device.
 * Idempotent per (key_addr, key_len) = QuantMatrix::cache_key() (loader.rs:674-679): a second
 * call with a known key returns the first handle and touches no memory, the way the vendor
 * backends cache weights by key and never evict (engine/backend/rocm.rs:329-350).  key_len == 0
 * disables caching. */
int ogm_weight_upload(ogm_ctx *ctx, uint32_t ggml_type, const void *raw, size_t row_bytes,
                      uint32_t in_dim, uint32_t out_dim, uint64_t key_addr, uint64_t key_len,
                      ogm_weight **out);
/* Copies the matrix back from the device and undoes the repack: `raw_out` receives exactly the
 * bytes that were uploaded. */
int ogm_weight_download(ogm_ctx *ctx, const ogm_weight *w, void *raw_out, size_t raw_len);
/* Frees one weight (and its cache entry).  The reference never evicts; tests and long-running
 * hosts may. */
int ogm_weight_free(ogm_ctx *ctx, ogm_weight *w);
int ogm_weight_info(const ogm_weight *w, uint32_t *ggml_type, uint32_t *in_dim, uint32_t *out_dim,
                    size_t *device_bytes);

/* ---- matmul: Backend ----------------------------------------------------------------------- */

/* Backend::matmul / matmul_into (backend/mod.rs:313, 342) with CpuBackend's kernel choice
 * (backend/cpu.rs:55-167): n_tokens == 1 -> the decode GEMV; n_tokens > 1 -> the prefill GEMM
 * (K-quants: per-256 activations, min pass then dot pass; Q8_0: per-32 activations). */
int ogm_matmul(ogm_ctx *ctx, const ogm_weight *w, const float *x, uint32_t n_tokens, float *y);
/* Backend::matmul_decode / matmul_decode_into (backend/mod.rs:386, 349; backend/cpu.rs:265-317):
 * the n_tokens == 1 kernel once per (row, token), so row t equals decoding token t alone. */
int ogm_matmul_decode(ogm_ctx *ctx, const ogm_weight *w, const float *x, uint32_t n_tokens,
                      float *y);

/* MatmulOp (backend/mod.rs:121-125). */
typedef struct ogm_op {
  const ogm_weight *w;
  const float *x;    /* [n_tokens][w.in_dim] */
  uint32_t n_tokens;
  float *y;          /* [n_tokens][w.out_dim] */
} ogm_op;
/* Backend::matmul_batch / matmul_batch_decode (backend/mod.rs:362, 405): independent ops, all
 * launched before one synchronization.  Ops longer than `max_tokens_per_phase`
 * (ORANGU_MAX_TOKENS_PER_SUBMISSION, default 256; backend/mod.rs:131-172) run in token stripes;
 * 0 selects the default.  Striping never changes a value (vecdot.rs:4522-4549). */
int ogm_matmul_batch(ogm_ctx *ctx, const ogm_op *ops, size_t n_ops, int decode,
                     uint32_t max_tokens_per_phase);

/* Device-pointer forms: x and y already live in HBM.  Enqueues the activation quantize and the
 * matmul kernels on `stream` and returns. */
int ogm_matmul_dev(ogm_ctx *ctx, const ogm_weight *w, const float *x_dev, uint32_t n_tokens,
                   float *y_dev, int decode, void *stream);

/* ogm_matmul_dev for callers that cannot allocate.  It has no counterpart in the reference; it is for
 * code that must not call hipMalloc -- a HIP graph under capture, a tight serving loop, a harness that
 * forbids allocation.  Same arguments and values as ogm_matmul_dev (bit for bit), but the quantized
 * activations go to a static device array the library holds on every GPU it runs on (400 KiB, kept
 * until the process ends) instead of the context's grown-on-demand scratch, and no hipMalloc, hipFree
 * or other allocating routine is called.  Limits: n_tokens <= 8 and n_tokens * in_dim <= 262144;
 * beyond them the call returns OGM_ERR_INVALID and enqueues nothing.  Every call on one GPU -- from
 * any context or thread -- shares that GPU's array: calls that overlap on one GPU (two streams, two
 * contexts) race on it; calls on one stream do not.  The array keeps the last call's contents; each
 * call overwrites all it reads. */
int ogm_matmul_dev_static(ogm_ctx *ctx, const ogm_weight *w, const float *x_dev, uint32_t n_tokens,
                          float *y_dev, int decode, void *stream);

/* The same path in two steps, so that ops reading one input (a layer's q/k/v, or gate/up:
 * engine/arch/mod.rs:1082-1096) quantize it once.  ogm_act_quantize_dev quantizes x_dev
 * ([n_tokens][in_dim]) into the context's activation buffer with the mode `ggml_type` needs
 * (backend/cpu.rs:100-116); ogm_matmul_act_dev then multiplies any weight of the same in_dim and
 * activation mode by it.  Values equal ogm_matmul_dev's: the quantizer is a pure function of x.
 * ogm_act_quantize_dev quantizes for a following call with decode = 0 (Backend::matmul),
 * ogm_act_quantize_decode_dev for one with decode = 1 (Backend::matmul_decode).  The two differ for one case
 * only: Q2_K at n_tokens > 1, which matmul runs over per-32 activations (backend/cpu.rs:113-163) and
 * matmul_decode over per-256 ones (cpu.rs:265-317); a matmul step over the other mode's activations returns
 * OGM_ERR_INVALID and says which quantizer it needs. */
int ogm_act_quantize_dev(ogm_ctx *ctx, uint32_t ggml_type, const float *x_dev, uint32_t in_dim,
                         uint32_t n_tokens, void *stream);
int ogm_act_quantize_decode_dev(ogm_ctx *ctx, uint32_t ggml_type, const float *x_dev, uint32_t in_dim,
                                uint32_t n_tokens, void *stream);
int ogm_matmul_act_dev(ogm_ctx *ctx, const ogm_weight *w, uint32_t n_tokens, float *y_dev,
                       int decode, void *stream);

/* Several weights of one type and in_dim over the same device-resident input, as the forward pass
 * issues them (q/k/v and gate/up: engine/arch/mod.rs:1082-1096, through Backend::matmul_batch,
 * backend/mod.rs:362-366): the input is quantized once and, at one token, a single kernel launch
 * covers all the weights.  ys_dev[i] is [n_tokens][ws[i].out_dim].  Values equal ogm_matmul_dev
 * per weight. */
int ogm_matmul_multi_dev(ogm_ctx *ctx, const ogm_weight *const *ws, size_t n_ws, const float *x_dev,
                         uint32_t n_tokens, float *const *ys_dev, int decode, void *stream);
/* The same over activations already quantized by ogm_act_quantize_dev (the grouped form of
 * ogm_matmul_act_dev). */
int ogm_matmul_multi_act_dev(ogm_ctx *ctx, const ogm_weight *const *ws, size_t n_ws,
                             uint32_t n_tokens, float *const *ys_dev, int decode, void *stream);

/* ---- the integer stage, exposed for parity checks ------------------------------------------- */

/* The fused activation quantizer on its own.  mode OGM_ACT_PER_32: d has n/32 entries
 * (vecdot.rs:95-126); OGM_ACT_PER_256: n/256 (vecdot.rs:3030-3053).  q has n, sums n/16
 * (per-16 sums of q, i32).  Host pointers; n % 32 (resp. 256) must be 0. */
int ogm_quantize_act(ogm_ctx *ctx, int mode, const float *x, size_t n, int8_t *q, float *d,
                     int32_t *sums);
/* The same quantizer over a batch, as the multi-token matmuls launch it: x is [n_tokens][in_dim]
 * (host), the results token-major -- q [T][in_dim], d [T][in_dim/group], sums i32 [T][in_dim/16], bsum
 * i16 [T][in_dim/32] (ActQ8K's per-32 sums, vecdot.rs:1849-1852) and, per 256 only, bs16 [T][in_dim/16]:
 * per super-block eight f16 values floor(bsum_j / 64) followed by eight f16 values bsum_j mod 64, the
 * K-quant GEMMs' first-pass operand.  The values are those of ActQ8K::quantize / ActQ8Flat::quantize
 * (vecdot.rs:1858-1910, 2483-2525); only their 4-token interleave is not materialised.  sums, bsum
 * and bs16 may be null. */
int ogm_quantize_act_tokens(ogm_ctx *ctx, int mode, const float *x, uint32_t in_dim, uint32_t n_tokens,
                            int8_t *q, float *d, int32_t *sums, int16_t *bsum, uint16_t *bs16);
/* Per (token, row, block) integer sums the matmul kernels form before any float is touched:
 * Q4_K and Q5_K: isum = sum_j sc_j * dot32_j and imin = sum_j m_j * bsum_j per super-block
 * (vecdot.rs:3152-3213); Q6_K and Q3_K: isum per super-block (vecdot.rs:3215-3241, 3273-3292),
 * imin untouched;
 * Q8_0, Q5_0, Q4_0, IQ4_NL: isum per 32-block (vecdot.rs:2829-2883).  Arrays are [n_tokens][out_dim][blocks per
 * row]; imin may be NULL.  Runs the same kernels as ogm_matmul_decode with a dump switch. */
int ogm_dump_block_sums(ogm_ctx *ctx, const ogm_weight *w, const float *x, uint32_t n_tokens,
                        int32_t *isum, int32_t *imin);

/* f16 -> f32 as the kernels convert block scales, for all `n` inputs (host pointers).  Lets a
 * test compare the device conversion with quant::f16_bits_to_f32 (quant.rs:511-528). */
int ogm_f16_to_f32(ogm_ctx *ctx, const uint16_t *bits, size_t n, float *out);

/* ---- Llama-family decode step (the callers either side of the matmuls) ------------------------ */

/* One token through every layer without returning to the host: what LlamaModel::run_layers +
 * forward do at n_tokens == 1 (engine/arch/llama.rs:594-932, 1007-1032) -- RMSNorm
 * (tensor.rs:732-757), q/k/v, NORM-paired RoPE (tensor.rs:1115-1177; freq_scale 1, no YaRN, no
 * frequency factors), KV-cache append, causal grouped-query attention (attention.rs:426-549), wo,
 * residual, RMSNorm, SwiGLU FFN (arch/mod.rs:1071-1106), residual; then the output norm and the
 * vocabulary projection.  The matmuls are ogm_matmul's single-token path, bit for bit; the
 * element-wise kernels use tree reductions and the KV cache is f16 (the reference's host cache is
 * f32, kv_cache.rs:75-78), so logits agree with the CPU forward pass to tolerance, not to the bit. */
typedef struct ogm_llama ogm_llama;
typedef struct ogm_llama_config {
  uint32_t n_layer, n_embd, n_head, n_head_kv, head_dim, n_ff, n_vocab;
  uint32_t rope_dim;    /* rotated dimensions per head, <= head_dim */
  uint32_t max_ctx;     /* KV-cache capacity in positions */
  float rms_eps, rope_freq_base;
  /* RoPE pairing (rope_layout_for, llama.rs:115-120): 0 = NORM, pairs (2i, 2i+1), for "llama" and
   * "mistral" files; 1 = NEOX, pairs (i, i + rope_dim/2), for qwen2 / qwen3 and the rest. */
  uint32_t rope_neox;
  /* rope_freqs.weight (llama.rs:186-201): host f32 [rope_dim/2] divisors of the pair frequencies,
   * copied; null when the file has none. */
  const float *rope_freq_factors;
} ogm_llama_config;
typedef struct ogm_llama_layer {
  const ogm_weight *wq, *wk, *wv, *wo, *w_gate, *w_up, *w_down;
  const float *attn_norm, *ffn_norm;   /* host f32 [n_embd], copied */
  /* optional, host f32, copied, null when the file has no such tensor (llama.rs:174-178):
   * projection biases [n_head*head_dim], [n_head_kv*head_dim] x 2 (added first, llama.rs:757-765)
   * and per-head RMSNorm weights [head_dim] of q and k (applied before RoPE, llama.rs:770-787). */
  const float *q_bias, *k_bias, *v_bias, *q_norm, *k_norm;
} ogm_llama_layer;

/* Builds the device-side model over weights already uploaded with ogm_weight_upload (they must
 * outlive it).  `layers` has cfg->n_layer entries; output_norm is host f32 [n_embd].
 * OGM_ERR_UNSUPPORTED for shapes the forward-pass kernels are not built for: head_dim other than 64 or 128; a
 * number of query heads per K/V head that is neither 1..8 nor, up to 64, divisible into equal parts of at most
 * eight (16, 12, 10, 24 ... are taken; 9, 11, 13 ... are not); n_embd above 16384 or not a multiple of 32. */
int ogm_llama_create(ogm_ctx *ctx, const ogm_llama_config *cfg, const ogm_llama_layer *layers,
                     const float *output_norm, const ogm_weight *output, ogm_llama **out);
void ogm_llama_destroy(ogm_ctx *ctx, ogm_llama *m);

/* Writes cache rows pos0 .. pos0+n_pos of one layer from host f32 [n_pos][n_head_kv*head_dim]
 * (K already rotated), as a CPU prefill hands its cache over (LayerCache::push, kv_cache.rs:756-768). */
int ogm_llama_kv_write(ogm_ctx *ctx, ogm_llama *m, uint32_t layer, uint32_t pos0, uint32_t n_pos,
                       const float *k, const float *v);

/* The reverse: cache rows pos0 .. pos0+n_pos of one layer as the f16 bit patterns the device holds
 * ([n_pos][n_head_kv*head_dim] each, K rotated), e.g. to park a sequence on the host as the
 * reference's slot store does with LayerCache rows (kv_cache.rs:756-768).  Waits for the stream. */
int ogm_llama_kv_read(ogm_ctx *ctx, ogm_llama *m, uint32_t layer, uint32_t pos0, uint32_t n_pos,
                      uint16_t *k_bits, uint16_t *v_bits);

/* Decodes the token at position `pos` whose embedding row is x ([n_embd] f32; the caller looks it
 * up as run_layers does, llama.rs:609-614).  Appends its K/V at `pos`, attends to 0..pos.
 * logits ([n_vocab]) and argmax may each be null.  Host pointers; synchronizes. */
int ogm_llama_decode(ogm_ctx *ctx, ogm_llama *m, const float *x, uint32_t pos, float *logits,
                     uint32_t *argmax);
/* The same with device pointers, enqueued on `stream` (null = the context's) without waiting. */
int ogm_llama_decode_dev(ogm_ctx *ctx, ogm_llama *m, const float *x_dev, uint32_t pos, float *logits_dev,
                         uint32_t *argmax_dev, void *stream);
/* Prefill: n_tokens embedding rows x ([n_tokens][n_embd], host f32) at positions pos0 .. pos0+n_tokens
 * through run_layers at n_tokens > 1 (llama.rs:594-932): the matmuls in the GEMM kernels' float order
 * (Backend::matmul, cpu.rs:445-458), K/V rows appended to the cache, causal attention; then the last
 * row alone through the output norm and projection (forward, llama.rs:1007-1032).  last_logits
 * ([n_vocab]) and argmax may each be null.  Runs in passes of up to 2048 tokens (tuning key prefill_chunk_tokens); synchronizes. */
int ogm_llama_prefill(ogm_ctx *ctx, ogm_llama *m, const float *x, uint32_t pos0, uint32_t n_tokens,
                      float *last_logits, uint32_t *argmax);
/* The same from token ids (host), their embedding rows read on the device from an uploaded
 * [n_embd -> n_vocab] matrix (llama.rs:609-614). */
int ogm_llama_prefill_tokens(ogm_ctx *ctx, ogm_llama *m, const ogm_weight *tok_embd, const uint32_t *tokens,
                             uint32_t pos0, uint32_t n_tokens, float *last_logits, uint32_t *argmax);

/* Model::forward_all_logits (the trait's contract, engine/arch/mod.rs:2110-2132; speculative_next's verify step
 * calls it, engine/generate.rs:1641): like ogm_llama_prefill -- n_tokens positions appended at pos0, from embedding
 * rows x [n_tokens][n_embd] or, with x null, from token ids into tok_embd -- but returns the next-token logits of
 * EVERY position, logits [n_tokens][n_vocab] (may be null), and each position's greedy token, argmax [n_tokens]
 * (may be null; sampling.rs:336-343's order): every row through the output norm and ONE matmul of all rows with
 * the output matrix, the composition engine/arch/gemma.rs:2179-2186 uses (llama.rs itself leaves the trait's
 * default, an error).  A rejected draft is rolled back by calling again at the position after the accepted
 * prefix: cache rows from there on are overwritten (KvCache::truncate).  At most 64 positions a call. */
int ogm_llama_forward_all_logits(ogm_ctx *ctx, ogm_llama *m, const float *x, const ogm_weight *tok_embd,
                                 const uint32_t *tokens, uint32_t pos0, uint32_t n_tokens, float *logits,
                                 uint32_t *argmax);

/* forward_hidden_states (llama.rs:1034-1045): the n_tokens tokens at positions 0 .. through run_layers
 * from an empty cache, then every row through the output norm: out is [n_tokens][n_embd] (host f32),
 * what an embeddings request pools over.  The tokens come as embedding rows x ([n_tokens][n_embd], host)
 * or, with x null, as ids into tok_embd (an uploaded [n_embd -> n_vocab] matrix).  The reference makes a
 * cache of its own for the call; here the model's cache rows 0 .. n_tokens-1 are overwritten, so a decode in
 * progress on this model does not survive the call.  Synchronizes. */
int ogm_llama_hidden_states(ogm_ctx *ctx, ogm_llama *m, const float *x, const ogm_weight *tok_embd,
                            const uint32_t *tokens, uint32_t n_tokens, float *out);

/* Rows row0 .. row0+n_rows of an uploaded matrix as f32 ([n_rows][in_dim], host memory), from the
 * device copy: dequantize_q8_0 / _q4_k / _q6_k (engine/quant.rs:639-649, 666-697, 746-787), bit for
 * bit.  This is the embedding lookup of run_layers (llama.rs:609-614). */
int ogm_dequant_rows(ogm_ctx *ctx, const ogm_weight *w, uint32_t row0, uint32_t n_rows, float *out);

/* Greedy generation without leaving the device: starting from `first_token` at position pos0,
 * n_tokens times { embedding row of the current token from tok_embd (an uploaded [n_embd ->
 * n_vocab] matrix); decode step; argmax (sampling.rs:336-343) becomes the next token }.
 * tokens_out receives the n_tokens generated ids, last_logits (nullable) the final step's logits.
 * One synchronization at the end. */
int ogm_llama_generate(ogm_ctx *ctx, ogm_llama *m, const ogm_weight *tok_embd, uint32_t first_token,
                       uint32_t pos0, uint32_t n_tokens, uint32_t *tokens_out, float *last_logits);

/* The decode step's greedy pick on its own, for parity checks: index of the maximum of n logits (host
 * pointers) as sampling::argmax takes it (engine/sampling.rs:336-343) -- Iterator::max_by over
 * f32::total_cmp, so -0 < +0, a positive NaN beats every number, and of equal maxima the last wins. */
int ogm_argmax(ogm_ctx *ctx, const float *logits, uint32_t n, uint32_t *out);

/* The last decode's final hidden state, before the output norm ([n_embd] host f32; what
 * run_layers returns), for parity checks. */
int ogm_llama_debug_hidden(ogm_ctx *ctx, ogm_llama *m, float *x_out);

/* Debug capture for parity checks.  With capture on, every decode step also keeps the quantized
 * activations each group of matmuls read (the int8 values and their scales, as the producing kernel
 * left them): site 4*layer + 0 the q/k/v input, + 1 the wo input, + 2 the gate/up input, + 3 the down
 * input, site 4*n_layer the vocabulary projection's input.  A test compares them with
 * vecdot::quantize_act / quantize_act_k_row (vecdot.rs:79-126, 3030-3053) of the CPU forward pass and
 * lets the CPU continue from the device's values where an f32 last-bit difference tipped a rounding.
 * ogm_llama_debug_act copies one site of the last step: q has room for max(n_embd, n_ff,
 * n_head*head_dim) values, d for a 32nd of that; *n receives the element count, *group 32 or 256. */
int ogm_llama_debug_capture(ogm_ctx *ctx, ogm_llama *m, int enable);
int ogm_llama_debug_act(ogm_ctx *ctx, ogm_llama *m, uint32_t site, int8_t *q, float *d, uint32_t *n,
                        uint32_t *group);

/* Measurement only, no counterpart in the reference: the wall-clock stamps (100 MHz) the decode step's attention
 * kernel leaves in a variant of the library built with -DOGM_ATTN_STAMPS=1 -- eight per workgroup of the last
 * launch, in the grid's order: start, q rotated, scores, V sum, partial results acknowledged, ticket drawn, and for
 * the workgroup that merges: chunks merged, row quantized.  Reads n_words of them and clears them.
 * OGM_ERR_UNSUPPORTED from the shipped library, which keeps none. */
int ogm_debug_attn_stamps(ogm_ctx *ctx, uint64_t *out, size_t n_words);

/* ---- GGUF reader -> uploader -------------------------------------------------------------------- */

/* Reads a GGUF file's header, metadata and tensor table (GgufFile::open_at / read, src/gguf.rs:149-280,
 * value types :386-415) and views its 2-D tensors as matrices (LoadedModel::matrix,
 * engine/loader.rs:1552-1580), so that a .gguf file loads without the Rust host.  `offset` is where
 * the GGUF segment starts inside the file (0 for a plain .gguf).  The file is mapped read-only
 * and stays mapped until ogm_gguf_close; weights uploaded from it do not refer to the mapping.
 * On failure `err` (when given) receives a message.  GGUF v2+ only (gguf.rs:38). */
typedef struct ogm_gguf ogm_gguf;
int ogm_gguf_open(const char *path, uint64_t offset, ogm_gguf **out, char *err, size_t err_len);
/* The same over bytes the caller holds (they must outlive the handle). */
int ogm_gguf_parse(const void *bytes, size_t len, ogm_gguf **out, char *err, size_t err_len);
void ogm_gguf_close(ogm_gguf *g);
const char *ogm_gguf_last_error(const ogm_gguf *g);
/* alignment = general.alignment when present and positive, else 32; data_offset = end of the
 * tensor table rounded up to it, relative to the segment (gguf.rs:258-266). */
int ogm_gguf_info(const ogm_gguf *g, uint32_t *version, uint64_t *alignment, uint64_t *data_offset,
                  uint64_t *n_tensors, uint64_t *n_metadata);
/* Metadata by key.  _u64 follows GgufValue::as_u64 (gguf.rs:70-83: unsigned, non-negative signed,
 * bool); _f64 also takes the float types; _array reports element type and count. */
int ogm_gguf_meta_u64(const ogm_gguf *g, const char *key, uint64_t *out);
int ogm_gguf_meta_f64(const ogm_gguf *g, const char *key, double *out);
int ogm_gguf_meta_string(const ogm_gguf *g, const char *key, const char **out, size_t *len);
int ogm_gguf_meta_array(const ogm_gguf *g, const char *key, uint32_t *elem_type, uint64_t *count);
/* Tensor table: index by name (-1 when absent), entry by index (dims has room for 8), and the
 * tensor's bytes (size from the block layout, engine/quant.rs:344-357; bounds-checked). */
int64_t ogm_gguf_find_tensor(const ogm_gguf *g, const char *name);
int ogm_gguf_tensor(const ogm_gguf *g, uint64_t index, const char **name, uint32_t *n_dims, uint64_t dims[8],
                    uint32_t *ggml_type, uint64_t *offset);
int ogm_gguf_tensor_data(ogm_gguf *g, uint64_t index, const void **data, uint64_t *len);
/* A 2-D tensor as a matrix: dims[0] = in_dim, dims[1] = out_dim, row_bytes * out_dim must equal the
 * tensor's size (loader.rs:1565-1579). */
int ogm_gguf_matrix(ogm_gguf *g, const char *name, uint32_t *ggml_type, uint32_t *in_dim, uint32_t *out_dim,
                    size_t *row_bytes, const void **raw);
/* ogm_gguf_matrix + ogm_weight_upload, keyed by the mapped bytes' address and length. */
int ogm_gguf_upload_matrix(ogm_ctx *ctx, ogm_gguf *g, const char *name, ogm_weight **out);

/* A Llama-style file (general.architecture llama, mistral, qwen2, qwen3 or qwen3vl: loader.rs:190) as a
 * device-resident decoder: the hyperparameters as read_model_config derives them (loader.rs:1652-1714:
 * head_count_kv defaults to head_count, key_length to embedding_length / head_count,
 * rope.dimension_count to the head width, freq_base to 10000, the epsilon to 1e-5, vocab_size to the
 * token list's length), the tensors LlamaModel::load_with_backend takes (llama.rs:123-220: output.weight
 * falls back to token_embd.weight, the bias / per-head-norm / rope_freqs tensors are optional), the
 * pairing rope_layout_for gives the architecture.  Every matrix goes through ogm_gguf_upload_matrix
 * (the context keeps them); *tok_embd (nullable) receives the embedding matrix for
 * ogm_llama_generate / ogm_dequant_rows, *cfg_out (nullable) the configuration used.  Errors are
 * reported through ogm_gguf_last_error.  Hyperparameters that do not fit 32 bits (or whose
 * head_count * key_length does not) are rejected before any upload.  Matrices uploaded before a later
 * failure stay in the context's weight cache, keyed by their mapped bytes, until ogm_destroy: a retry
 * over the same mapping finds them there. */
int ogm_llama_load_gguf(ogm_ctx *ctx, ogm_gguf *g, uint32_t max_ctx, ogm_llama **model,
                        const ogm_weight **tok_embd, ogm_llama_config *cfg_out);

/* ---- tuning / introspection ------------------------------------------------------------------ */

/* Kernel choices the host makes per shape, exposed so that a benchmark can sweep them and a test can reach
 * every kernel on small shapes.  Unknown keys and values out of range return OGM_ERR_INVALID.  Only
 * "gemm_one_pass", "attn_prefill_variant" and "attn_decode_chunks" can change a result bit; every other
 * setting selects among kernels that produce the same bits.
 *   "gemv_wg_waves"            waves per workgroup of the GEMV kernel, 1..16; 0 = by the row's tile count
 *   "gemm_min_tokens"          ogm_matmul takes a matrix-core GEMM from this many tokens on; 0 = default (6 for
 *                              Q4_K, Q5_K and Q6_K; 9 for Q8_0, Q5_0, Q4_0 and IQ4_NL where their small-batch
 *                              kernel would run, or as soon as the GEMV kernel would need two passes over
 *                              the weights; 17 otherwise); below it the multi-token GEMV kernel runs in the
 *                              GEMM's float order
 *   "gemm_small_max_tokens"    GEMMs of at most this many tokens take the small-batch kernel of their type, whose
 *                              waves work on different super-blocks (blocks, for the per-32 types: by default
 *                              while the launch has at most 1792 workgroups of 32 rows x 32 tokens) of the same rows; 0 = default (K-quants: 64, more
 *                              for matrices of few rows: 128 up to 8192 rows, 256 up to 4096 -- and up to 6144
 *                              for Q4_K / Q5_K rows of more than 8192 inputs --, 384 up to 2048, 512 there for
 *                              Q4_K / Q5_K; Q6_K launches that "gemm_interleave" sends to its kernel by their size
 *                              go there first), 1 = never
 *   "gemm_act_chunks"          whether a K-quant batch's int8 activations are also written in the operand order
 *                              of the matrix-core kernels (1 KiB chunks of 32 tokens x 32 inputs; the small-batch
 *                              kernels then load a chunk in one piece instead of gathering 32 rows, the plane
 *                              and medium-batch kernels need no relayout launch): 0 = default, from 25 tokens
 *                              (the forward pass's own producers from 17), 1 = never, 2 = from 9.  Same bits
 *   "gemm_sb_waves"            waves of a small-batch workgroup: 8 or 16; 0 = by the size of the launch (sixteen
 *                              where it has at most 256 workgroups and the rows the blocks for two rounds of them)
 *   "gemm_medium"              the Q4_K / Q5_K kernel for one nearly full tile of 128 tokens, or two (32 rows x
 *                              128 tokens a workgroup, its waves on different super-blocks): 0 = by the size of
 *                              the launch, 1 = never, 2 = whenever the shape allows
 *   "gemm_tile_rows"           feeding-wave GEMMs: 64 = always their 64-row tiles; 0 = by the size of the launch
 *   "gemm_few_tokens_min_rows" 2 to 16 tokens over a Q6_K matrix (matmul and matmul_decode alike) take the
 *                              kernel that streams the weights once when the matrix has at least this many
 *                              rows; 0 = default (30000 rows and three tokens), 1 = whenever the shape allows,
 *                              -1 = never
 *   "gemm_plane_cache_mb"      device memory, in MiB, that the K-quant and IQ4_XS matrices' prefill planes may take
 *                              in all (default 32768): on a matrix's first GEMM that would read them its scale-folded
 *                              int8 planes (2 bytes per weight, 1 for Q3_K) are built once and kept; a matrix
 *                              that does not fit, and every matrix at 0, is unpacked on every call (IQ4_XS, whose
 *                              GEMM kernels beyond its small batches read planes, then stays on the GEMV kernel);
 *                              ogm_weight_download is unaffected
 *   "gemm_plane_kernel"        when the kernel that multiplies the planes (all waves multiply, operands loaded
 *                              straight into LDS) runs: 0 = default, when the launch has more than 256 tiles of
 *                              128 rows x 128 tokens (the feeding-wave kernels unpack otherwise); 2 = whatever
 *                              the grid, from 32 tokens
 *   "gemm_interleave"          the plane kernel with 64-row tiles that adds a super-block up between the next
 *                              one's matrix instructions (Q4_K, Q5_K, Q6_K): 0 = default, on launches of at most
 *                              512 tiles of 64 rows x 128 tokens: Q6_K from 128 such tiles with the last token
 *                              tile more than three quarters full or with three token tiles, or from 160 with
 *                              more than 96 tokens; Q4_K / Q5_K from three token tiles (two over rows of more
 *                              than 8192 inputs) and 160 tiles, with rows longer than 5120 inputs at most 256 (the
 *                              8B shapes' q/k/v, wo and down projections at 257 to 1024 tokens; their planes are
 *                              built then); 1 = never; 2 = wherever the plane kernel runs.  Same bits
 *   "gemm_one_pass"            0 = default.  1: Q4_K and Q5_K on that kernel skip the reference GEMM's separate
 *                              first pass over the mins (vecdot.rs:2229-2240) and add
 *                              ad * (d * isum - dmin * imin) per super-block, the single-token expression of
 *                              vecdot.rs:3152-3178.  The integer sums are the same; the f32 result is within
 *                              rounding of the reference GEMM's, not its bits: an output whose terms cancel to
 *                              near zero can differ from the reference's by more than 1e-3 of itself
 *   "gemv_mma"                 2 to 16 tokens over Q4_K / Q5_K / Q6_K rows on the kernel
 *                              that gives a workgroup one row block and multiplies on the matrix cores: 1 =
 *                              default, where it measured faster (Q6_K from four tokens, Q4_K / Q5_K from five, all
 *                              up to eight; rows of up to 4096 inputs, longer ones only in launches of few rows);
 *                              2 = wherever it can (two to sixteen); 0 = never.  Same bits as the other kernels
 *   "attn_decode_chunks"       chunks of 128 cached positions that a workgroup of the decode step's attention
 *                              takes one after the other, 1..64; 0 = default: one up to about 4000 positions of
 *                              eight K/V heads (fewer than 256 workgroups), then as many as keep the launch near
 *                              264 workgroups (2 at 8192 positions, 8 at 32768); the per-token kernel of a
 *                              small prefill batch likewise, near 528 workgroups.  Agrees with one chunk a
 *                              workgroup to f32 rounding
 *   "attn_prefill_variant"     attention of a prefill batch: 1 = the decode step's kernel per token and chunk of
 *                              the cache; 2 = the matrix-core kernel; 0 = default: the first for batches of up to
 *                              48 tokens (speculative-decode verify batches), the second above; they agree to
 *                              f32 rounding
 *   "prefill_chunk_tokens"     tokens per pass of ogm_llama_prefill over the layers, default 2048; a model keeps
 *                              the value of its first prefill, whose row buffers are allocated for it
 *   "host_zero_copy"           1 = default: a host-pointer call (ogm_matmul, ogm_matmul_decode,
 *                              ogm_matmul_batch) whose x and y together are at most 512 KiB runs its kernels
 *                              directly on the pinned staging buffers, with no copy-engine transfer; 0 = always
 *                              stage through device memory, as larger calls do.  The staging buffers are
 *                              allocated as coherent (fine-grained) host memory by name; where the runtime
 *                              refuses that, the context behaves as with 0 and "host_flag_wait" 0
 *   "host_flag_wait"           1 = default: such a call waits for its results by polling a word in that pinned
 *                              memory which a one-thread kernel behind the call's kernels stores, instead of
 *                              waiting on the stream; after 5 ms without the word, and on every 256th call,
 *                              the stream is synchronized after all; 0 = always hipStreamSynchronize; 2 = for
 *                              tests of the bounded wait: the word never matches and every call runs into the
 *                              5 ms */
int ogm_set_tuning(ogm_ctx *ctx, const char *key, int value);
/* For benchmarks driven from an interpreter: runs host-pointer calls from compiled code and writes each
 * repetition's wall time in microseconds to us_out[reps].  `ops` holds n_variants sets of n_ops ops;
 * repetition r walks set r % n_variants, in groups of group_sizes[] ops: a group of one is an ogm_matmul,
 * a longer one an ogm_matmul_batch.  No counterpart in the reference. */
int ogm_time_host_calls(ogm_ctx *ctx, const ogm_op *ops, size_t n_ops, size_t n_variants,
                        const uint32_t *group_sizes, size_t n_groups, uint32_t reps, double *us_out);
/* For benchmarks: one launch that only reads the device bytes of 1..4 uploaded weights (each of 9 KiB or
 * more) with the GEMV's non-temporal 16-byte loads and stores nothing -- the rate the memory system gives
 * that footprint with no arithmetic behind the loads.  No counterpart in the reference. */
int ogm_weights_read_probe(ogm_ctx *ctx, const ogm_weight *const *ws, size_t n_ws, void *stream);
/* For benchmarks: one launch of `workgroups` (1..1048576) workgroups of 256 threads that does nothing -- what
 * a kernel boundary costs behind a launch of that width.  No counterpart in the reference. */
int ogm_empty_launch(ogm_ctx *ctx, uint32_t workgroups, void *stream);
/* For benchmarks driven from an interpreter: enqueues `reps` launches back to back from compiled code, so that
 * the caller's own overhead per call leaves no gap between short kernels.  `ws` holds n_variants sets of n_ws
 * weights; launch r takes set (first + r) % n_variants.  kind 0: ogm_matmul_multi_act_dev over the set into
 * ys_dev[n_ws]; kind 1: ogm_weights_read_probe over the set; kind 2: ogm_empty_launch of n_tokens workgroups (ws
 * unused).  No counterpart in the reference. */
int ogm_enqueue_repeated(ogm_ctx *ctx, int kind, const ogm_weight *const *ws, size_t n_ws, size_t n_variants,
                         uint32_t n_tokens, float *const *ys_dev, int decode, uint32_t first, uint32_t reps,
                         void *stream);
/* Bytes of device and pinned host scratch this context has allocated so far (activation buffers, staging;
 * weights and prefill planes not counted).  It grows on demand and never shrinks before ogm_destroy; a call
 * that leaves it unchanged has allocated no scratch.  No counterpart in the reference. */
size_t ogm_scratch_bytes(ogm_ctx *ctx);
/* Name of the kernel the last matmul on this context launched (for profiles). */
const char *ogm_last_kernel(ogm_ctx *ctx);

#ifdef __cplusplus
}
#endif
#endif
