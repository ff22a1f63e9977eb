// Launchers of the gfx950 kernels, called by the C ABI in ogm_api.cpp.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// Quantized activations of up to n_tokens tokens, token-major, on the device:
//   q    int8 [T][in_dim]
//   d    f32  [T][in_dim/32] (per-32 mode) or [T][in_dim/256] (per-256 mode)
//   sums i32  [T][in_dim/16]   per-16 sums of q   (ActQ8 / ActQ8KRow .sums, vecdot.rs:66-75, 3020-3026)
//   bsum i16  [T][in_dim/32]   per-32 sums of q   (ActQ8K .bsum, vecdot.rs:1849-1852)
struct OgmActDev {
  int8_t *q;
  float *d;
  int32_t *sums;
  int16_t *bsum;
  // per-256 mode only: the sums per 32 once more as f16 pairs (bsum >> 6, bsum & 63), sixteen halves
  // per super-block (eight high parts, then eight low parts): the K-quant GEMMs' first-pass operand
  uint16_t *bs16;
  // per-256 mode, batches of rows only: when not null, the int8 activations are also written here in the operand
  // chunks of the GEMMs whose waves all multiply (ogm_gemm_xh_bytes() bytes; the chunks' tokens past the last stay
  // as they were: they are multiplied, never stored)
  int8_t *xt = nullptr;
};

// mode 0: one scale per 32 (vecdot.rs:95-126); mode 1: one per 256 (vecdot.rs:3030-3053).
// xt (per-256 mode only): when not null, the int8 activations are also written there in the operand chunks of
// the GEMM whose waves all multiply (ogm_gemm_xh_bytes() bytes), which then needs no relayout pass of its own.
hipError_t ogm_launch_quantize(int mode, const float *x, uint32_t in_dim, uint32_t n_tokens,
                               OgmActDev act, hipStream_t stream, int8_t *xt = nullptr);

#define OGM_GEMV_MAX_MATS 4

struct OgmGemvArgs {
  uint32_t ggml_type;
  const uint8_t *wt;  // tile-planar weights
  uint32_t in_dim, out_dim;
  OgmActDev act;      // matching the type's activation mode
  uint32_t n_tokens;  // tokens in this launch (<= ogm_gemv_max_tokens)
  float *y;           // [n_tokens][out_dim], row stride out_dim
  int gemm_order;     // 0: GEMV float order (cpu.rs T==1 / matmul_decode), 1: GEMM order (T>1)
  uint32_t wg_waves;     // waves per workgroup, 0 = by shape
  int32_t *dump_isum;    // optional [n_tokens][out_dim][blocks/row]
  int32_t *dump_imin;    // optional, Q4_K only
  // Further matrices of the same type and in_dim that read the same activations (q/k/v,
  // gate/up): one launch covers all of them.  Not combined with the dumps.
  uint32_t n_extra;
  const uint8_t *extra_wt[OGM_GEMV_MAX_MATS - 1];
  uint32_t extra_out_dim[OGM_GEMV_MAX_MATS - 1];
  float *extra_y[OGM_GEMV_MAX_MATS - 1];
};

// Largest token count one launch can take for this shape (LDS budget), at least 1.
uint32_t ogm_gemv_max_tokens(uint32_t ggml_type, uint32_t in_dim, int gemm_order);
hipError_t ogm_launch_gemv(const OgmGemvArgs &a, hipStream_t stream, const char **kernel_name);
// Prefill GEMM on MFMA (ogm_gemm.hip).  Same operands as the GEMV plus a scratch buffer `xh` of
// ogm_gemm_xh_bytes() for the int8 activations in operand chunks.  Follows the CPU path's GEMM float order.
#define OGM_GEMM_MAX_MATS 3   // matrices one GEMM launch can take (q, k, v)
struct OgmGemmArgs {
  uint32_t ggml_type;
  const uint8_t *wt;
  uint32_t in_dim, out_dim;
  OgmActDev act;       // per-256 quantized activations of all n_tokens
  uint32_t n_tokens;
  float *y;            // [n_tokens][out_dim]
  void *xh;            // scratch
  bool xt_ready = false;   // the quantizer has already written the operand chunks to xh
  uint32_t tile_rows = 0;          // feeding-wave kernels: 64 forces their 64-row tiles (0 = by the size of the launch)
  uint32_t small_max_tokens = 0;   // most tokens for the small-batch kernel (0 = default 64, 1 = never)
  uint32_t sb_waves = 0;           // waves of a small-batch workgroup: 8 or 16 (0 = by the size of the launch)
  uint32_t medium = 0;             // Q4_K / Q5_K medium-batch kernel: 0 by the size of the launch, 1 never, 2 whenever it can
  // K-quants: further matrices of the same type and in_dim over the same activations, in the same launch
  uint32_t n_extra = 0;
  const uint8_t *extra_wt[OGM_GEMM_MAX_MATS - 1] = {};
  uint32_t extra_out_dim[OGM_GEMM_MAX_MATS - 1] = {};
  float *extra_y[OGM_GEMM_MAX_MATS - 1] = {};
  // K-quants: the matrices' scale-folded int8 planes (ogm_gemm_build_planes), or null.  When every
  // matrix of the launch has them, the kernel whose waves all multiply reads them (operands by load-to-LDS).
  const uint8_t *planes = nullptr;
  const uint8_t *extra_planes[OGM_GEMM_MAX_MATS - 1] = {};
  // when that kernel runs: 0 when the grid fills the device twice (else the feeding waves unpack), 2 whatever
  // the grid
  uint32_t plane_kernel = 0;
  uint32_t interleave = 0;   // the plane kernel with 64-row tiles that adds a super-block up between the next one's matrix instructions: 0 by the size of the launch, 1 never, 2 whenever it can
  uint32_t one_pass = 0;   // Q4_K / Q5_K on the all-waves-multiply kernel: fold the min pass into the super-block step (f32 to rounding, not to the bit)
};
// Whether this launch would run a tiled int8 plane kernel, i.e. whether planes would be read.
bool ogm_gemm_uses_planes(const OgmGemmArgs &a);
// Whether this K-quant or IQ4_XS launch would run the small-batch kernel of its type (which needs no planes).
bool ogm_gemm_takes_small_batch(const OgmGemmArgs &a);
// Bytes of a K-quant matrix's planes (0: the type has none), and the kernel that builds them from
// the tile-planar bytes (2 bytes per weight, 1 for Q3_K; rows padded to a multiple of 64).
size_t ogm_gemm_plane_bytes(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim);
hipError_t ogm_gemm_build_planes(uint32_t ggml_type, const uint8_t *wt, uint32_t in_dim, uint32_t out_dim,
                                 uint8_t *planes, hipStream_t stream);
bool ogm_gemm_supported(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t n_tokens);
// Whether a GEMM of a per-32 type (Q8_0, Q5_0, Q4_0, IQ4_NL; Q5_1, which has no other) of this shape would take their
// small-batch kernel by the size of the launch: what makes a GEMM pay below seventeen tokens.
bool ogm_gemm_flat_small_batch(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t n_tokens);
size_t ogm_gemm_xh_bytes(uint32_t in_dim, uint32_t n_tokens);
hipError_t ogm_launch_gemm(const OgmGemmArgs &a, hipStream_t stream, const char **kernel_name);

// 2 to 16 tokens over a Q6_K matrix of many rows (ogm_gemm_ft.hip): every wave streams 32 rows once and
// multiplies them with all tokens on the matrix cores.  Reads a.wt, a.act.q, a.act.d; writes a.y.
// gemm_order as OgmGemvArgs.  min_rows: fewest rows from which it is taken (0: the default rule, 30000
// rows and three tokens).
bool ogm_gemm_ft_eligible(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t n_tokens,
                          uint32_t min_rows);
hipError_t ogm_launch_gemm_ft(const OgmGemmArgs &a, int gemm_order, hipStream_t stream, const char **kernel_name);
// Two to sixteen tokens over Q4_K / Q5_K / Q6_K (ogm_gemm_ft.hip): one workgroup per group of 16 rows, waves on
// different super-blocks, products on the matrix cores, either float order.
bool ogm_gemv_mma_eligible(uint32_t ggml_type, uint32_t in_dim, uint32_t n_tokens, int gemm_order);
hipError_t ogm_launch_gemv_mma(const OgmGemvArgs &a, hipStream_t stream, const char **kernel_name);

hipError_t ogm_launch_f16_to_f32(const uint16_t *bits, size_t n, float *out, hipStream_t stream);

// One launch that only reads the given buffers (each at least 9 KiB, 16-byte aligned) with the GEMV's
// non-temporal loads; `sink` is one device word that is never written.
#define OGM_PROBE_MAX_BUFS 4u
hipError_t ogm_launch_read_probe(const uint8_t *const *bufs, const size_t *bytes, uint32_t n, uint32_t *sink,
                                 hipStream_t stream);
// Stores `value` to the pinned host word `flag` once everything before it on the stream has finished.
hipError_t ogm_launch_empty(uint32_t workgroups, uint32_t *sink, hipStream_t stream);
hipError_t ogm_launch_host_flag(uint32_t *flag, uint32_t value, hipStream_t stream);

// The library's static scratch (ogm_static.hip): a file-scope device array every GPU holds its own
// copy of, for the entry point that must not allocate.  It takes the quantized activations of up to
// OGM_STATIC_MAX_TOKENS tokens totalling OGM_STATIC_MAX_ELEMS elements (400 KiB in all).
#define OGM_STATIC_MAX_TOKENS 8u
#define OGM_STATIC_MAX_ELEMS 262144u
// Address of the array on the device that is current, from hipGetSymbolAddress; call once per device.
hipError_t ogm_static_scratch_address(uint8_t **ptr);
// The array cut into the five activation buffers, for OGM_STATIC_MAX_ELEMS elements.
OgmActDev ogm_static_act_view(uint8_t *scratch);
