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
};

// mode 0: one scale per 32 (vecdot.rs:95-126); mode 1: one per 256 (vecdot.rs:3030-3053).
hipError_t ogm_launch_quantize(int mode, const float *x, uint32_t in_dim, uint32_t n_tokens,
                               OgmActDev act, hipStream_t stream);

#define OGM_GEMV_MAX_MATS 4

// What the last workgroup of a single-token GEMV launch to finish does with the launch's outputs,
// in place of a kernel of its own (per-256 activations only):
//   OGM_TAIL_NORM   x += y; act = quantize(rmsnorm(x) * weight)       one matrix, out_dim = n
//   OGM_TAIL_SWIGLU act = quantize(silu(y0) * y1)                     two matrices, out_dims = n
// `ticket` is OGM_TAIL_TICKETS zeroed uint32 on the device that the launch leaves zero again.  `act` may be
// the buffer the launch read its own activations from: every workgroup has finished by then.
#define OGM_TAIL_TICKETS 65u
#define OGM_TAIL_NONE 0u
#define OGM_TAIL_NORM 1u
#define OGM_TAIL_SWIGLU 2u
struct OgmGemvTail {
  uint32_t kind = OGM_TAIL_NONE;
  uint32_t n = 0;
  uint32_t *ticket = nullptr;
  float *x = nullptr;             // NORM: the residual stream, updated in place
  const float *weight = nullptr;  // NORM: the norm's weights
  float eps = 0.0f;
  OgmActDev act = {};
};

// What extra workgroups at the front of a single-token GEMV launch (per-256 activations) compute before
// its other workgroups read their activations, in place of a kernel of its own ahead of the launch:
//   OGM_HEAD_NORM   x += delta; act = quantize(rmsnorm(x) * weight)    one producer workgroup, n = in_dim
//   OGM_HEAD_SWIGLU act = quantize(silu(gate) * up)                    ceil(in_dim / 256 / waves) of them
// The launch's `act` is what the producers write and the others read.  The producers are the launch's
// first workgroups, which the hardware starts first; they store device-coherently, and the last of
// them to finish raises flag[0] to `epoch`.  Every other workgroup requests its first tile of
// weights, then polls the flag (at most spin_limit times; it then sets the gave-up word and goes on
// with whatever the activations hold, so every wave ends) and reads the activations.
// flag: OGM_HEAD_FLAG_WORDS uint32 on the device, zero before the first launch: OGM_HEAD_FLAG_COPIES
// copies of the flag, 128 bytes apart (a waiting workgroup polls copy `its index % copies`: polls of
// one address are served one after the other), which only ever grow; then the producers' own counter,
// zero between launches, and the word a workgroup that gave up sets.  epoch: the flag's value before
// the launch plus one (launches over one flag must be stream-ordered).
#define OGM_HEAD_FLAG_COPIES 64u
#define OGM_HEAD_FLAG_WORDS (OGM_HEAD_FLAG_COPIES * 32u + 2u)
#define OGM_HEAD_NONE 0u
#define OGM_HEAD_NORM 1u
#define OGM_HEAD_SWIGLU 2u
struct OgmGemvHead {
  uint32_t kind = OGM_HEAD_NONE;
  uint32_t *flag = nullptr;
  uint32_t epoch = 0;
  uint32_t spin_limit = 0;        // 0: the default (about a tenth of a second)
  float *x = nullptr;             // NORM: the residual stream, updated in place
  const float *delta = nullptr;   // NORM: what is added to x first (may be null)
  const float *weight = nullptr;  // NORM: the norm's weights
  float eps = 0.0f;
  const float *gate = nullptr;    // SWIGLU
  const float *up = nullptr;
  uint32_t delay = 0;             // what the other workgroups sleep before their first weight loads, in units of 64 clocks
  uint32_t n_prod = 0;            // filled in by the launcher
};

struct OgmGemvArgs {
  uint32_t ggml_type;
  const uint8_t *wt;  // tile-planar weights
  uint32_t in_dim, out_dim;
  OgmActDev act;      // matching the type's activation mode
  uint32_t n_tokens;  // tokens in this launch (<= ogm_gemv_max_tokens)
  float *y;           // [n_tokens][out_dim], row stride out_dim
  int gemm_order;     // 0: GEMV float order (cpu.rs T==1 / matmul_decode), 1: GEMM order (T>1)
  uint32_t wg_waves;     // waves per workgroup, 0 = by shape
  uint32_t rb_per_wg;    // row blocks per workgroup, 0 = by shape
  int32_t *dump_isum;    // optional [n_tokens][out_dim][blocks/row]
  int32_t *dump_imin;    // optional, Q4_K only
  // Further matrices of the same type and in_dim that read the same activations (q/k/v,
  // gate/up): one launch covers all of them.  Not combined with the dumps.
  uint32_t n_extra;
  const uint8_t *extra_wt[OGM_GEMV_MAX_MATS - 1];
  uint32_t extra_out_dim[OGM_GEMV_MAX_MATS - 1];
  float *extra_y[OGM_GEMV_MAX_MATS - 1];
  // When set (one token, GEMV order, no dumps): f32 activations [in_dim]; every workgroup
  // quantizes them itself on its way in and `act` is not read.
  const float *x_f32;
  OgmGemvTail tail;   // one token, GEMV order, no dumps, no x_f32
  OgmGemvHead head;   // one token, GEMV order, no dumps, no x_f32, no tail; per-256 activations
};

// Largest token count one launch can take for this shape (LDS budget), at least 1.
uint32_t ogm_gemv_max_tokens(uint32_t ggml_type, uint32_t in_dim, int gemm_order);
hipError_t ogm_launch_gemv(const OgmGemvArgs &a, hipStream_t stream, const char **kernel_name);
// Longest row an OGM_TAIL_NORM tail of a single-token launch over this matrix can take (0: none).
uint32_t ogm_gemv_norm_tail_max(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t wg_waves);
// Waves per workgroup of a single-token launch with a head over this matrix (0: the type takes none).
// An OGM_HEAD_NORM head needs in_dim <= 1024 * that.
uint32_t ogm_gemv_head_waves(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t wg_waves);

// Prefill GEMM on MFMA (ogm_gemm.hip).  Same operands as the GEMV plus a scratch buffer `xh` of
// ogm_gemm_xh_bytes() for the activations as f16.  Follows the CPU path's GEMM float order.
#define OGM_GEMM_MAX_MATS 3   // matrices one GEMM launch can take (q, k, v)
struct OgmGemmArgs {
  uint32_t ggml_type;
  const uint8_t *wt;
  uint32_t in_dim, out_dim;
  OgmActDev act;       // per-256 quantized activations of all n_tokens
  uint32_t n_tokens;
  float *y;            // [n_tokens][out_dim]
  void *xh;            // scratch
  uint32_t wide_min_wgs = 0;   // Q4_K: least 128x128 workgroups from which the wide tiling runs (0 = default)
  uint32_t q4k_variant = 0;    // K-quants: 0 / 1 the int8 plane kernels, 2 the f16 kernels, 3 int8 multiply-adds
  uint32_t small_max_tokens = 0;   // most tokens for the small-batch kernel (0 = default 64, 1 = never)
  uint32_t sb_waves = 0;           // waves of a small-batch workgroup: 8 or 16 (0 = by the size of the launch)
  // K-quants: further matrices of the same type and in_dim over the same activations, in the same launch
  uint32_t n_extra = 0;
  const uint8_t *extra_wt[OGM_GEMM_MAX_MATS - 1] = {};
  uint32_t extra_out_dim[OGM_GEMM_MAX_MATS - 1] = {};
  float *extra_y[OGM_GEMM_MAX_MATS - 1] = {};
  // K-quants: the matrices' scale-folded int8 planes (ogm_gemm_build_planes), or null.  When every
  // matrix of the launch has them, the tiled int8 kernels read them instead of unpacking the
  // weights again on every call.
  const uint8_t *planes = nullptr;
  const uint8_t *extra_planes[OGM_GEMM_MAX_MATS - 1] = {};
  // which kernel reads planes: 0 the one whose waves all multiply (operands by load-to-LDS) when the
  // grid fills the device twice, else none (the feeding waves unpack); 1 the feeding-wave kernels; 2
  // the former whatever the grid
  uint32_t plane_kernel = 0;
  uint32_t one_pass = 0;   // Q4_K / Q5_K on the all-waves-multiply kernel: fold the min pass into the super-block step (f32 to rounding, not to the bit)
};
// Whether this launch would run a tiled int8 plane kernel, i.e. whether planes would be read.
bool ogm_gemm_uses_planes(const OgmGemmArgs &a);
// Bytes of a K-quant matrix's planes (0: the type has none), and the kernel that builds them from
// the tile-planar bytes (2 bytes per weight, 1 for Q3_K; rows padded to a multiple of 64).
size_t ogm_gemm_plane_bytes(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim);
hipError_t ogm_gemm_build_planes(uint32_t ggml_type, const uint8_t *wt, uint32_t in_dim, uint32_t out_dim,
                                 uint8_t *planes, hipStream_t stream);
bool ogm_gemm_supported(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t n_tokens);
size_t ogm_gemm_xh_bytes(uint32_t in_dim, uint32_t n_tokens);
hipError_t ogm_launch_gemm(const OgmGemmArgs &a, hipStream_t stream, const char **kernel_name);

// 2 to 16 tokens over a Q6_K matrix of many rows (ogm_gemm_ft.hip): every wave streams 32 rows once and
// multiplies them with all tokens on the matrix cores.  Reads a.wt, a.act.q, a.act.d; writes a.y.
// gemm_order as OgmGemvArgs.  min_rows: fewest rows from which it is taken (0: the default rule, 30000
// rows and three tokens).
bool ogm_gemm_ft_eligible(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t n_tokens,
                          uint32_t min_rows);
hipError_t ogm_launch_gemm_ft(const OgmGemmArgs &a, int gemm_order, hipStream_t stream, const char **kernel_name);

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
