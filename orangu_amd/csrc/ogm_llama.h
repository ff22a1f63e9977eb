// Launchers of the decode-step kernels around the quantized matmuls (ogm_llama.hip): what a
// Llama-family layer does between two matmuls at one token (engine/arch/llama.rs:594-932 of
// orangu-server), with the activation quantizer of the next matmul fused into each producer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ogm_kernels.h"

#define OGM_ATTN_CHUNK 128u       // cache positions per workgroup of the attention kernel ...
// The tickets of the K/V heads are 128 bytes apart: the workgroups of a launch draw theirs within a microsecond
// of each other, and tickets that share a line queue up behind one another at the memory's atomic unit (136 of
// them in one line: the last came back 2.9 us after its store; a line each: see the decode step's timeline).
#define OGM_ATTN_TICKET_STRIDE 32u
// A decode step over a long context gives a workgroup several chunks in a row, as many as keep the launch near
// OGM_ATTN_SUB_TARGET workgroups (one to a compute unit and a few), at most OGM_ATTN_SUB_MAX.
#define OGM_ATTN_SUB_TARGET 264u
#define OGM_ATTN_SUB_TARGET_ROWS 528u   // for a batch of tokens (two workgroups to a compute unit)
#define OGM_ATTN_SUB_MAX 64u
#define OGM_ATTN_CHUNK_MIN 64u    // ... or half as many while the launch stays within one round of workgroups;
                                  // the partial-result buffers are sized for this one

// x += delta (when delta is given; x is updated in place), then
// normed = x * (1 / sqrt(mean(x^2) + eps)) * weight        (tensor.rs:732-757)
// quantized for the next matmul in `mode` (0: per 32, 1: per 256) into `act`; `normed` (f32) is
// also stored when not null.  n <= 16384, n % 32 == 0.  With n_rows > 1: that many rows of x, delta,
// normed and act, one workgroup each.
hipError_t ogm_launch_norm_quant(int mode, float *x, const float *delta, const float *weight, uint32_t n,
                                 float eps, float *normed, OgmActDev act, hipStream_t stream, uint32_t n_rows = 1,
                                 const float *x_src = nullptr);   // x_src: the rows are read from there and stored to x

// cos / sin of pos * freq[p] for the rope_dim / 2 rotated pairs, as float2 (cos, sin): once per
// token, every layer rotates by the same angles (tensor.rs:1147-1160, freq_scale 1, no YaRN;
// `freq` already holds base^(-2p / rope_dim) divided by the pair's frequency factor).
// Row t of `cs` (rope_dim / 2 pairs each) is the table of the token at position pos + t.
hipError_t ogm_launch_rope_table(const float *freq, uint32_t pos, uint32_t n_tokens, uint32_t rope_dim, void *cs,
                                 hipStream_t stream);

// What a layer applies to its projections before they meet (engine/arch/llama.rs:757-810): the
// projection biases (Qwen2), then the per-head RMSNorm of q and k (Qwen3), then RoPE in the
// architecture's pairing.  Null pointers mean "the file has no such tensor".
struct OgmAttnPre {
  const float *q_bias, *k_bias, *v_bias;   // [n_head * head_dim], [kv_dim], [kv_dim]
  const float *q_norm, *k_norm;            // [head_dim] each
  float eps;                               // of the per-head norms
  uint32_t neox;                           // 0: pairs (2i, 2i+1); 1: pairs (i, i + rope_dim / 2)
};

// One token's attention, from the q / k / v the projections left (f32) to the quantized input of
// the output projection:
//   * bias, per-head norm and RoPE (tensor.rs:1233-1240, 691-706, 1115-1177) of q and k with the
//     table `cs`, k and v rounded to f16 into the cache rows of position `pos`;
//   * causal attention over cache positions 0..pos (engine/attention.rs:426-549): scores =
//     (q . k) * scale, softmax over positions, out = sum w * v; grouped-query heads share their
//     K/V head (a count ogm_attn_head_parts accepts: up to eight in one workgroup, more in equal parts of at
//     most eight).  Split over chunks of `chunk` positions (64 or 128; 0 = by the size of the launch), of which a
//     workgroup takes `chunks_per_wg` in a row (0 = by the size of the launch: one, more on long contexts), and
//     merged;
//   * the merged output quantized for the next matmul in `mode`, and stored as f32 when attn_out
//     is not null.
// part_o: [n_head][max_splits][head_dim] f32, part_ml: [n_head][max_splits][2] f32 scratch, with
// max_splits >= the number of workgroups per head, at most pos / chunk + 1; counters: 2 * n_head_kv * parts * OGM_ATTN_TICKET_STRIDE words (one ticket per
// cache line), zero before the first launch (the kernel leaves them zero).
// ogm_attn_head_parts: the workgroups a K/V head's query heads are dealt to (1 for up to eight heads, else the
// fewest equal parts of at most eight), or 0 for a count the kernels do not take (none, more than 64, or one that
// does not divide: 9, 11, 13, ...).
uint32_t ogm_attn_head_parts(uint32_t heads_per_kv);
hipError_t ogm_launch_attn_decode(const float *q, const float *k_new, const float *v_new, const void *cs,
                                  uint32_t rope_dim, const OgmAttnPre &pre, void *k_cache_layer,
                                  void *v_cache_layer, uint32_t pos, uint32_t max_splits, uint32_t n_head,
                                  uint32_t n_head_kv, uint32_t head_dim, float scale, float *part_o,
                                  float *part_ml, uint32_t *counters, int mode, float *attn_out, OgmActDev act,
                                  hipStream_t stream, uint32_t chunk = 0, uint32_t chunks_per_wg = 0);

// h = silu(gate) * up with silu(g) = g / (1 + exp(-g))     (tensor.rs:825-827, arch/mod.rs:1071-1106)
// quantized for the down projection in `mode`; h (f32) is also stored when not null.  With
// n_rows > 1: that many rows of n values each.
hipError_t ogm_launch_swiglu_quant(int mode, const float *gate, const float *up, uint32_t n, float *h,
                                   OgmActDev act, hipStream_t stream, uint32_t n_rows = 1);

// Index of the largest logit; of several equal ones the last (sampling.rs:336-343).  `scratch`
// holds 2 * 256 words.
hipError_t ogm_launch_argmax(const float *logits, uint32_t n, uint32_t *scratch, uint32_t *out,
                             hipStream_t stream);

// f32 -> f16 (round to nearest even) for cache rows handed over by the host.
hipError_t ogm_launch_f32_to_f16(const float *src, void *dst, size_t n, hipStream_t stream);

// Rows row .. row + n_rows (or row_dev[0 .. n_rows) when not null) of a tile-planar quantized matrix
// as f32 [n_rows][in_dim]: the embedding lookup (llama.rs:609-614 over quant.rs:639-649, 666-697,
// 746-787), bit-identical.
hipError_t ogm_launch_dequant_row(const uint8_t *wt, uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim,
                                  uint32_t row, const uint32_t *row_dev, uint32_t n_rows, float *out,
                                  hipStream_t stream);

// ---- the same layer over a batch of tokens (prefill, llama.rs:594-932 at n_tokens > 1) ----------
// The norm and the SwiGLU are the decode step's kernels over n_rows rows (they quantize their own
// output for the GEMMs that follow); the rest works on plain f32 rows.

// q [n_tokens][n_head*head_dim] in place, k and v [n_tokens][n_head_kv*head_dim] into the cache
// rows pos0 .. pos0 + n_tokens as f16: bias, per-head norm, RoPE (row t of `cs`) as in
// ogm_launch_attn_decode.
hipError_t ogm_launch_qkv_pre(float *q, const float *k, const float *v, const void *cs, uint32_t rope_dim,
                              const OgmAttnPre &pre, uint32_t n_head, uint32_t n_head_kv, uint32_t head_dim,
                              void *k_cache_layer, void *v_cache_layer, uint32_t pos0, uint32_t n_tokens,
                              hipStream_t stream);

// Causal attention of n_tokens query rows (already rotated) at positions pos0 .. over cache rows
// 0 .. pos0 + t for token t; attn_out [n_tokens][n_head*head_dim].
// part_o: [n_tokens][n_head][max_splits][head_dim], part_ml: [n_tokens][n_head][max_splits][2].
// quant_mode >= 0 (0: per 32, 1: per 256): the merge also quantizes every token's row into row t of `act` for the
// next matmul, and attn_out may be null.  chunks_per_wg: as for ogm_launch_attn_decode (0 = by the size of the launch).
hipError_t ogm_launch_attn_prefill(const float *q, void *k_cache_layer, void *v_cache_layer, uint32_t pos0,
                                   uint32_t n_tokens, uint32_t max_splits, uint32_t n_head, uint32_t n_head_kv,
                                   uint32_t head_dim, float scale, float *part_o, float *part_ml, float *attn_out,
                                   hipStream_t stream, int quant_mode = -1, OgmActDev act = OgmActDev{},
                                   uint32_t chunks_per_wg = 0);

// The same on the matrix cores, one launch and no partial results: query tiles of 32 tokens, cache
// tiles of 64 positions, running softmax.  head_dim 64 or 128, at most 8 query heads per K/V head.
hipError_t ogm_launch_attn_prefill_mfma(const float *q, void *k_cache_layer, void *v_cache_layer, uint32_t pos0,
                                        uint32_t n_tokens, uint32_t n_head, uint32_t n_head_kv, uint32_t head_dim,
                                        float scale, float *attn_out, hipStream_t stream);

// Timeline builds only (-DOGM_ATTN_STAMPS=1): the wall-clock stamps (100 MHz) of the last attention launch, eight per
// workgroup; hipErrorNotSupported from the shipped library.
hipError_t ogm_attn_stamps_read(unsigned long long *host_out, size_t n_words);
