// Few tokens over a large Q6_K matrix: the weights stream from HBM once, every wave keeps 32 rows
// to itself over the whole of k, and the products run on the matrix cores.
//
// The decode GEMV takes a batch token by token: every token unpacks the block's 6-bit values again
// or, unpacked once, runs its own 64 dot instructions per block, and beyond four tokens that vector
// work outlasts the stream (4096 -> 128256: 65 us at one token, 88 at four, 160 at eight).  Here a
// group of 16 weights of 32 rows is unpacked once into the column operand of one
// v_mfma_i32_32x32x16_i8 whose row operand holds the same 16 activations of up to 16 tokens: K = 16
// is exactly the run one Q6_K scale covers, so the instruction leaves dot16(q - 32, x) of every
// (token, row) and `isum += sc_g * dot16` (vecdot.rs:2352-2398, 3215-3241) is one 24-bit integer
// multiply-add per token in the lane that owns the row.  A lane holds row (lane & 31) and the
// tokens 4 * (lane >> 5) + {0..3} (+ 8 for the second set of four), so the f32 step of a
// super-block, in the reference's order, stays in the lane as well: no reduction across lanes, no
// LDS traffic but the activations.
//
// Layout of a launch: workgroup = 4 waves = 128 rows; lane (row r, half h) loads bytes 8h..8h+7 of
// every 16-byte piece of its row's block (the 8 weights of each group it supplies to the matrix
// instruction; both halves together read a tile's 16 rows x 16 bytes as one 256-byte run), two
// super-blocks in flight per wave.  The int8 activations sit in LDS as [k / 8][token][8 bytes].
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ogm_kernels.h"
#include "ogm_layout.h"

typedef int ft_int16v __attribute__((ext_vector_type(16)));
typedef uint32_t ft_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t ft_u32x4 __attribute__((ext_vector_type(4)));

#define FT_WAVES 4u
#define FT_ROWS (32u * FT_WAVES)
#define FT_TILE_BYTES (64u * 210u)

struct GemmFtParams {
  const uint8_t *wt;   // tile-planar Q6_K, four blocks per tile row
  const int8_t *xq;    // [n_tokens][in_dim]
  const float *ad;     // [n_tokens][nsb]
  float *y;            // [n_tokens][out_dim]
  uint32_t in_dim, out_dim, n_tokens, nsb, nct, nrb;
};

__device__ __forceinline__ float ft_f16_bits_to_f32(uint32_t bits16) {
  union { unsigned short u; _Float16 h; } v;
  v.u = (unsigned short)bits16;
  return (float)v.h;
}

// One super-block of one row, the half of every group this lane multiplies.
struct FtRegs {
  ft_u32x2 ql[8];
  ft_u32x2 qh[4];
  ft_u32x4 sc;
  uint32_t d16;
};

// `unit`: the lane's unit in its tile, column 0; s: the super-block.
__device__ __forceinline__ void ft_load(FtRegs &r, const uint8_t *rb_base, uint32_t r16, uint32_t lh, uint32_t s) {
  const uint8_t *tile = rb_base + (size_t)(s >> 2) * FT_TILE_BYTES;
  const uint32_t lt = (s & 3u) * 16u + r16;
  const uint8_t *b = tile + lt * 16u;
#pragma unroll
  for (int i = 0; i < 8; i++) r.ql[i] = __builtin_nontemporal_load((const ft_u32x2 *)(b + i * 1024 + lh * 8u));
#pragma unroll
  for (int i = 0; i < 4; i++) r.qh[i] = __builtin_nontemporal_load((const ft_u32x2 *)(b + (8 + i) * 1024 + lh * 8u));
  r.sc = __builtin_nontemporal_load((const ft_u32x4 *)(b + 12 * 1024));
  r.d16 = __builtin_nontemporal_load((const uint16_t *)(tile + 13 * 1024 + lt * 2u));
}

// Four 6-bit values of run rr (0..3) of a half block as int8 (q - 32): the nibble, two bits of qh on
// top; then, all four bytes at once, v + 0x60 (no carry: v <= 63) with the top bit flipped is v - 32.
template <int RR>
__device__ __forceinline__ uint32_t ft_unpack4(uint32_t ql, uint32_t qh) {
  const uint32_t n = (RR < 2 ? ql : (ql >> 4)) & 0x0F0F0F0Fu;
  const uint32_t t = RR == 0 ? (qh << 4) : RR == 1 ? (qh << 2) : RR == 2 ? qh : (qh >> 2);
  const uint32_t v = (t & 0x30303030u) | n;
  return (v + 0x60606060u) ^ 0x80808080u;
}

template <int G>
__device__ __forceinline__ long ft_group_operand(const FtRegs &r) {
  constexpr int H = G >> 3, RR = (G >> 1) & 3, K = G & 1;
  const ft_u32x2 ql = r.ql[4 * H + 2 * (RR & 1) + K], qh = r.qh[2 * H + K];
  union { ft_u32x2 v; long l; } o;
  o.v.x = ft_unpack4<RR>(ql.x, qh.x);
  o.v.y = ft_unpack4<RR>(ql.y, qh.y);
  return o.l;
}

template <int G>
__device__ __forceinline__ int ft_scale(const FtRegs &r) {
  const uint32_t w = G < 4 ? r.sc.x : G < 8 ? r.sc.y : G < 12 ? r.sc.z : r.sc.w;
  return (int)(int8_t)(w >> (8 * (G & 3)));
}

// NREG: results a lane keeps per matrix instruction: 4 (up to 8 tokens) or 8 (up to 16).
// GEMM_ORDER: acc += ad * (d * isum) (gemm_k_q6_k, vecdot.rs:2389-2390); else the decode dot's
// total += ad * d * isum (vecdot.rs:3238).
template <int NREG, bool GEMM_ORDER>
__global__ __launch_bounds__(64 * FT_WAVES) void ogm_gemm_ft_q6k_kernel(GemmFtParams p) {
  constexpr uint32_t TP = 2 * NREG;   // token slots
  extern __shared__ __align__(16) uint8_t lds[];
  ft_u32x2 *l_x = (ft_u32x2 *)lds;                         // [in_dim / 8][TP]
  float *l_ad = (float *)(lds + (size_t)p.in_dim * TP);   // [nsb][TP]
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const uint32_t T = p.n_tokens, nsb = p.nsb;

  // ---- the activations: 16-byte pieces of the token-major rows, requested first ...
  const uint32_t ppt = p.in_dim / 16u, n_piece = T * ppt;
  constexpr int XPEEL = 8;
  ft_u32x4 xs[XPEEL];
#pragma unroll
  for (int i = 0; i < XPEEL; i++) {
    const uint32_t idx = min(tid + i * 64u * FT_WAVES, n_piece - 1u);
    xs[i] = *(const ft_u32x4 *)(p.xq + (size_t)idx * 16u);
  }
  // ---- ... then this wave's first super-block of weights
  const uint32_t row0 = (blockIdx.x * FT_WAVES + wave) * 32u;
  const uint32_t rb = min(row0 / 16u + (l32 >> 4), p.nrb - 1u);   // rows beyond the matrix: any block
  const uint8_t *rb_base = p.wt + (size_t)rb * p.nct * FT_TILE_BYTES;
  const uint32_t r16 = l32 & 15u;
  FtRegs A, B;
  ft_load(A, rb_base, r16, lh, 0);
  __builtin_amdgcn_sched_barrier(0);

  auto park = [&](uint32_t idx, const ft_u32x4 &v) {
    if (idx < n_piece) {
      const uint32_t t = idx / ppt, c = idx - t * ppt;
      ft_u32x2 a, b;
      a.x = v.x; a.y = v.y; b.x = v.z; b.y = v.w;
      l_x[(2u * c) * TP + t] = a;
      l_x[(2u * c + 1u) * TP + t] = b;
    }
  };
#pragma unroll
  for (int i = 0; i < XPEEL; i++) park(tid + i * 64u * FT_WAVES, xs[i]);
  for (uint32_t idx = tid + XPEEL * 64u * FT_WAVES; idx < n_piece; idx += 64u * FT_WAVES)
    park(idx, *(const ft_u32x4 *)(p.xq + (size_t)idx * 16u));
  for (uint32_t i = tid; i < nsb * TP; i += 64u * FT_WAVES) {
    const uint32_t s = i / TP, t = i - s * TP;
    l_ad[i] = t < T ? p.ad[(size_t)t * nsb + s] : 0.0f;
  }
  __syncthreads();

  float acc[NREG];
#pragma unroll
  for (int j = 0; j < NREG; j++) acc[j] = 0.0f;
  // this lane's activations of super-block s, group g: l_x[(32 s + 2 g + lh) * TP + token slot]
  const ft_u32x2 *xl = l_x + lh * TP + (l32 & (TP - 1u));
  const ft_int16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  auto process = [&](const FtRegs &r, uint32_t s) {
    const ft_u32x2 *xg = xl + (size_t)s * 32u * TP;
    int isum[NREG];
    // One matrix instruction under way while the one before it is scaled and added; the fence keeps
    // the compiler from starting all sixteen at once (sixteen result registers each).
    ft_int16v D0, D1;
#define FT_MFMA(G, D)                                                                             \
    {                                                                                             \
      union { ft_u32x2 v; long l; } xa;                                                           \
      xa.v = xg[2 * (G) * TP];                                                                    \
      D = __builtin_amdgcn_mfma_i32_32x32x16_i8(xa.l, ft_group_operand<(G)>(r), zero, 0, 0, 0);   \
    }
#define FT_ADD(G, D)                                                                              \
    {                                                                                             \
      const int sc = ft_scale<(G)>(r);                                                            \
      _Pragma("unroll") for (int j = 0; j < NREG; j++)                                            \
        isum[j] = (G) == 0 ? __mul24(sc, D[j]) : __mul24(sc, D[j]) + isum[j];                     \
      __builtin_amdgcn_sched_barrier(0);                                                          \
    }
    FT_MFMA(0, D0)
    FT_MFMA(1, D1) FT_ADD(0, D0) FT_MFMA(2, D0) FT_ADD(1, D1)
    FT_MFMA(3, D1) FT_ADD(2, D0) FT_MFMA(4, D0) FT_ADD(3, D1)
    FT_MFMA(5, D1) FT_ADD(4, D0) FT_MFMA(6, D0) FT_ADD(5, D1)
    FT_MFMA(7, D1) FT_ADD(6, D0) FT_MFMA(8, D0) FT_ADD(7, D1)
    FT_MFMA(9, D1) FT_ADD(8, D0) FT_MFMA(10, D0) FT_ADD(9, D1)
    FT_MFMA(11, D1) FT_ADD(10, D0) FT_MFMA(12, D0) FT_ADD(11, D1)
    FT_MFMA(13, D1) FT_ADD(12, D0) FT_MFMA(14, D0) FT_ADD(13, D1)
    FT_MFMA(15, D1) FT_ADD(14, D0) FT_ADD(15, D1)
#undef FT_MFMA
#undef FT_ADD
    const float d = ft_f16_bits_to_f32(r.d16);
#pragma unroll
    for (int j = 0; j < NREG; j++) {
      const float ad = l_ad[s * TP + 8u * (j >> 2) + 4u * lh + (j & 3)];
      if (GEMM_ORDER) acc[j] += ad * (d * (float)isum[j]);
      else acc[j] += ad * d * (float)isum[j];
    }
  };

  uint32_t s = 0;
  for (; s + 2 < nsb; s += 2) {
    ft_load(B, rb_base, r16, lh, s + 1);
    process(A, s);
    ft_load(A, rb_base, r16, lh, s + 2);
    process(B, s + 1);
  }
  ft_load(B, rb_base, r16, lh, s + 1);
  process(A, s);
  process(B, s + 1);

  // (pins the sums before the branch: the compiler would otherwise sink the last super-blocks'
  // vector work into it and keep all their matrix results alive until then)
#pragma unroll
  for (int j = 0; j < NREG; j++) asm volatile("" : "+v"(acc[j]));
  const uint32_t row = row0 + l32;
  if (row < p.out_dim) {
#pragma unroll
    for (int j = 0; j < NREG; j++) {
      const uint32_t t = 8u * (j >> 2) + 4u * lh + (j & 3);
      if (t < T) p.y[(size_t)t * p.out_dim + row] = acc[j];
    }
  }
}

// Shapes the kernel takes: Q6_K rows of a multiple of four super-blocks (tiles of 16 rows); 2 to 16
// tokens whose int8 rows fit LDS; and at least min_rows rows, since a wave streams its 32 rows alone,
// two super-blocks in flight, and the launch needs a few waves per SIMD.  min_rows 0, the default
// rule: from 30000 rows (a 32000-row vocabulary: 25 us at 4 tokens against 29 us token by token, 26
// against 34 at 8; at 14336 rows the other kernels win, 18 against 22) and from three tokens (at two
// the GEMV kernel is level or ahead).
bool ogm_gemm_ft_eligible(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t n_tokens,
                          uint32_t min_rows) {
  if (ggml_type != OGM_Q6_K || in_dim == 0 || in_dim % 1024u != 0 || n_tokens < 2u || n_tokens > 16u) return false;
  const uint32_t tp = n_tokens <= 8u ? 8u : 16u;
  if ((size_t)in_dim * tp + (size_t)(in_dim / 256u) * tp * 4u > 160u * 1024u) return false;
  if ((uint64_t)n_tokens * in_dim >= (1ull << 31)) return false;
  return min_rows ? out_dim >= min_rows : (out_dim >= 30000u && n_tokens >= 3u);
}

hipError_t ogm_launch_gemm_ft(const OgmGemmArgs &a, int gemm_order, hipStream_t stream, const char **kernel_name) {
  if (!ogm_gemm_ft_eligible(a.ggml_type, a.in_dim, a.out_dim, a.n_tokens, 1u)) return hipErrorInvalidValue;
  GemmFtParams p;
  p.wt = a.wt;
  p.xq = a.act.q;
  p.ad = a.act.d;
  p.y = a.y;
  p.in_dim = a.in_dim;
  p.out_dim = a.out_dim;
  p.n_tokens = a.n_tokens;
  p.nsb = a.in_dim / 256u;
  const OgmTiling tl = ogm_tiling_for(p.nsb, a.out_dim);
  p.nct = tl.nct;
  p.nrb = tl.nrb;
  const uint32_t tp = a.n_tokens <= 8u ? 8u : 16u;
  const uint32_t lds_bytes = a.in_dim * tp + p.nsb * tp * 4u;
  const void *fn = tp == 8u ? (gemm_order ? (const void *)ogm_gemm_ft_q6k_kernel<4, true> : (const void *)ogm_gemm_ft_q6k_kernel<4, false>)
                            : (gemm_order ? (const void *)ogm_gemm_ft_q6k_kernel<8, true> : (const void *)ogm_gemm_ft_q6k_kernel<8, false>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return e;
  void *kargs[] = {(void *)&p};
  e = hipLaunchKernel(fn, dim3((a.out_dim + FT_ROWS - 1u) / FT_ROWS), dim3(64 * FT_WAVES), kargs, lds_bytes, stream);
  if (e != hipSuccess) return e;
  if (kernel_name) *kernel_name = tp == 8u ? "ogm_gemm_ft_q6k_kernel" : "ogm_gemm_ft_q6k_t16_kernel";
  return hipGetLastError();
}
