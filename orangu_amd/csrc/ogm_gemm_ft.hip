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

// ------------------------------------------------------------------------------------------
// Few tokens over a K-quant matrix of any height (the projections of a speculative-decode verify batch: 2 to 16
// tokens over 1024 .. 30000 rows): the decode GEMV's distribution -- one workgroup per row block of 16 rows, its
// waves on different column tiles, every block's f32 term left in LDS and added per (token, row) in the row's
// order afterwards -- with the products on the matrix cores.  One instruction has 32 x 32 outputs; the batch has
// at most 16 tokens and the row block 16 rows, so one instruction multiplies TWO runs of k at once: its column
// operand holds the 16 rows' weights of run a (columns 0..15) and of run b (columns 16..31), its row operand the
// tokens' activations of run a (rows 0..TS-1) and of run b (rows TS..2TS-1); the outputs (token, run a) x (row,
// run a) and (token, run b) x (row, run b) are the two runs' dot products and the mixed quadrants are ignored.
// A run is what one scale covers: 16 weights of Q6_K (v_mfma_i32_32x32x16_i8, run b eight scales after run a:
// the other half of the super-block), a sub-block of 32 of Q4_K / Q5_K (v_mfma_i32_32x32x32_i8, run b four
// sub-blocks on).  Lane (column n, half h) thus owns row n % 16 and the runs of half n / 16 of the super-block:
// it adds sc_run * dot as 24-bit integer multiply-adds for its four (or eight) tokens, the two halves' sums meet
// with one lane exchange, and the lane of the lower half turns them into the super-block's f32 term
// (vecdot.rs:2229-2303, 2352-2398 in GEMM order; vecdot.rs:3152-3178, 3215-3241 in the decode dot's).
// Q4_K / Q5_K: the mins' sum_j m_j * bsum_j of a super-block is one f16 matrix instruction over the quantizer's
// sums per 32, split into two exact parts (OgmActDev::bs16).
//
// The int8 activations of all tokens sit in LDS as [k / 16][TS] 16-byte entries (Q6_K: [k / 8][TS] 8-byte ones),
// token slots TS = 8 or 16; a wave keeps two super-blocks of weights in flight.

typedef uint32_t fk_u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 fk_half8 __attribute__((ext_vector_type(8)));
typedef float fk_float16v __attribute__((ext_vector_type(16)));
typedef int fk_int4v __attribute__((ext_vector_type(4)));

#ifndef FK_ABL
#define FK_ABL 0   // timing experiments only: 1 no arithmetic, 2 no activation staging
#endif
struct GemmFkParams {
  const uint8_t *wt[OGM_GEMV_MAX_MATS];
  float *y[OGM_GEMV_MAX_MATS];
  uint32_t out_dim[OGM_GEMV_MAX_MATS];
  uint32_t wg_end[OGM_GEMV_MAX_MATS];   // workgroups (row blocks) of matrices 0..m, running total
  const int8_t *xq;                     // [n_tokens][in_dim]
  const float *ad;                      // [n_tokens][nsb]
  const uint16_t *bs16;                 // [n_tokens][nsb][16] f16 bits (Q4_K / Q5_K)
  uint32_t in_dim, n_tokens, nsb, nct;
  uint32_t c_shift, r_shift;            // log2 of the tiling's blocks per tile row (4, 2 or 1) and rows per tile (16, 32, 64)
  uint32_t rb_per_wg;                   // groups of 16 rows a workgroup takes (1 or 2)
};

#define FK_Q4K 0
#define FK_Q5K 1
#define FK_Q6K 2

template <int KIND>
struct FkRegs {   // Q4_K / Q5_K: one super-block of one row, the pieces of this lane's half
  fk_u32x4 hd;     // d, dmin, scales and mins
  fk_u32x4 w[2];   // 16 bytes of qs of each of the half's two sub-block pairs
  fk_u32x4 qh;     // Q5_K: 16 bytes of the fifth bits
  fk_u32x4 bs;     // this lane's token: eight f16 of the quantizer's sums per 32
};
template <>
struct FkRegs<FK_Q6K> {
  ft_u32x2 ql[4];
  ft_u32x2 qh[2];
  ft_u32x2 sc;
  uint32_t d16;
};

template <int KIND>
__device__ __forceinline__ constexpr uint32_t fk_tile_bytes() {
  return KIND == FK_Q4K ? 64u * 144u : KIND == FK_Q5K ? 64u * 176u : 64u * 210u;
}

// rb_base: the row block's first tile; s: the super-block; rt: the lane's row in the tile; hn: its half of the
// super-block; lh: its half of every run; cr: the tiling's shifts, c_shift | r_shift << 8.
template <int KIND>
__device__ __forceinline__ void fk_load(FkRegs<KIND> &r, const uint8_t *rb_base, uint32_t s, uint32_t rt, uint32_t hn,
                                        uint32_t lh, const uint16_t *bs_tok, uint32_t cr) {
  const uint32_t c_shift = cr & 0xFFu, r_shift = cr >> 8;
  const uint8_t *tile = rb_base + (size_t)(s >> c_shift) * fk_tile_bytes<KIND>();
  const uint32_t lt = ((s & ((1u << c_shift) - 1u)) << r_shift) + rt;
  const uint8_t *b = tile + lt * 16u;
  if constexpr (KIND == FK_Q6K) {
#pragma unroll
    for (int i = 0; i < 4; i++)
      r.ql[i] = __builtin_nontemporal_load((const ft_u32x2 *)(b + (4u * hn + i) * 1024u + lh * 8u));
#pragma unroll
    for (int i = 0; i < 2; i++)
      r.qh[i] = __builtin_nontemporal_load((const ft_u32x2 *)(b + (8u + 2u * hn + i) * 1024u + lh * 8u));
    r.sc = __builtin_nontemporal_load((const ft_u32x2 *)(b + 12u * 1024u + 8u * hn));
    r.d16 = __builtin_nontemporal_load((const uint16_t *)(tile + 13u * 1024u + lt * 2u));
  } else {
    constexpr uint32_t QS0 = KIND == FK_Q5K ? 3u : 1u;
    r.hd = __builtin_nontemporal_load((const fk_u32x4 *)b);
#pragma unroll
    for (int i = 0; i < 2; i++)
      r.w[i] = __builtin_nontemporal_load((const fk_u32x4 *)(b + (QS0 + 2u * (2u * hn + i) + lh) * 1024u));
    if constexpr (KIND == FK_Q5K) r.qh = __builtin_nontemporal_load((const fk_u32x4 *)(b + (1u + lh) * 1024u));
    r.bs = *(const fk_u32x4 *)(bs_tok + (size_t)s * 16u + 8u * lh);
  }
}

// One of two results of a matrix instruction, by the lane's half.  (Written as `hn ? D[b] : D[a]` the compiler
// indexes the result vector by a lane-dependent number: a chain of sixteen selects per value.)
__device__ __forceinline__ int fk_pick(int lo, int hi, uint32_t hn) {
  asm volatile("" : "+v"(lo), "+v"(hi));
  return hn ? hi : lo;
}

__device__ __forceinline__ float fk_pickf(float lo, float hi, uint32_t hn) {
  asm volatile("" : "+v"(lo), "+v"(hi));
  return hn ? hi : lo;
}

// acc (+|-)= p[0], p[stride], ... in ascending order, one accumulator; eight LDS reads in flight.
template <bool NEGATE>
__device__ __forceinline__ float fk_ordered_sum(float acc, const float *p, uint32_t n, uint32_t stride) {
  uint32_t s = 0;
  for (; s + 8 <= n; s += 8) {
    float a[8];
#pragma unroll
    for (int j = 0; j < 8; j++) a[j] = p[(s + j) * stride];
#pragma unroll
    for (int j = 0; j < 8; j++) acc = NEGATE ? acc - a[j] : acc + a[j];
  }
  for (; s < n; s++) acc = NEGATE ? acc - p[s * stride] : acc + p[s * stride];
  return acc;
}

// TS: token slots (8: up to 8 tokens, four results a lane; 16: up to 16, eight results a lane).
// GEMM_ORDER: the GEMM kernels' f32 sequence (mins first, acc += ad * (d * isum)); else the decode dot's.
// (sixteen token slots fit LDS up to some 8000 inputs, i.e. at most eight column tiles and waves)
template <int KIND, int TS, bool GEMM_ORDER>
__global__ __launch_bounds__(TS == 8 ? 1024 : 512) void ogm_gemm_fk_kernel(GemmFkParams p) {
  constexpr int NREG = TS / 2;
  constexpr bool K4 = KIND != FK_Q6K;
  constexpr bool TWO = K4 && GEMM_ORDER;   // two term arrays: the mins', then the products'
  extern __shared__ __align__(16) uint8_t lds[];
  // RB row blocks a workgroup (1 or 2): its waves split into RB teams that share the staged activations
  const uint32_t RB = p.rb_per_wg;
  const uint32_t tid = threadIdx.x, nthr = blockDim.x, lane = tid & 63u;
  const uint32_t n_wave = (nthr >> 6) / RB, team = (tid >> 6) / n_wave, wave = (tid >> 6) - team * n_wave;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const uint32_t r16 = l32 & 15u, hn = l32 >> 4;
  const uint32_t ts = l32 & (uint32_t)(TS - 1), hm = (l32 / (uint32_t)TS) & 1u;   // as a row operand: token slot, half
  const uint32_t T = p.n_tokens, nsb = p.nsb;
  uint8_t *l_x = lds;                                                   // in_dim * TS bytes
  float *l_ad = (float *)(lds + (size_t)p.in_dim * TS);                 // [nsb][TS]
  const uint32_t team_floats = (TWO ? 2u : 1u) * nsb * TS * 16u;
  float *l_tdot = l_ad + nsb * TS + team * team_floats;                 // [nsb][TS][16] per team
  float *l_tmin = l_tdot + (TWO ? nsb * TS * 16u : 0u);                 // [nsb][TS][16] when TWO

  // ---- which matrix of the launch, which of its row blocks (a team past the last row block repeats it and stores nothing)
  const bool idle = blockIdx.x * RB + team >= p.wg_end[OGM_GEMV_MAX_MATS - 1];
  const uint32_t bid = idle ? p.wg_end[OGM_GEMV_MAX_MATS - 1] - 1u : blockIdx.x * RB + team;
  uint32_t m = 0;
  if (bid >= p.wg_end[0]) m = 1;
  if (bid >= p.wg_end[1]) m = 2;
  if (bid >= p.wg_end[2]) m = 3;
  // g16: the group of 16 rows within its matrix; a row block of the tiling holds 1, 2 or 4 such groups
  const uint32_t g16 = bid - (m == 0 ? 0u : m == 1 ? p.wg_end[0] : m == 2 ? p.wg_end[1] : p.wg_end[2]);
  const uint8_t *wt = m == 0 ? p.wt[0] : m == 1 ? p.wt[1] : m == 2 ? p.wt[2] : p.wt[3];
  float *y = m == 0 ? p.y[0] : m == 1 ? p.y[1] : m == 2 ? p.y[2] : p.y[3];
  const uint32_t out_dim = m == 0 ? p.out_dim[0] : m == 1 ? p.out_dim[1] : m == 2 ? p.out_dim[2] : p.out_dim[3];
  const uint32_t sub_shift = p.r_shift - 4u;
  const uint8_t *rb_base = wt + (size_t)(g16 >> sub_shift) * p.nct * fk_tile_bytes<KIND>();
  const uint32_t rt = 16u * (g16 & ((1u << sub_shift) - 1u)) + r16;   // the lane's row in its tile
  const uint32_t cr = p.c_shift | (p.r_shift << 8);

  // ---- the activations: 16-byte pieces of the token-major rows, requested first ...
  const uint32_t ppt = p.in_dim / 16u, n_piece = T * ppt;
  constexpr int XPEEL = 8;
  fk_u32x4 xs[XPEEL];
#pragma unroll
  for (int i = 0; i < XPEEL; i++) {
    const uint32_t idx = min(tid + i * nthr, n_piece - 1u);
    xs[i] = *(const fk_u32x4 *)(p.xq + (size_t)idx * 16u);
  }
  // ---- ... then this wave's first super-block of weights
  // the wave's super-blocks: wave, wave + n_wave, ... (n_wave <= nsb: every wave has one)
  auto sb_of = [&](uint32_t k) -> uint32_t { return wave + n_wave * k; };
  const uint32_t n_my = (nsb - wave + n_wave - 1u) / n_wave;
  const uint16_t *bs_tok = K4 ? p.bs16 + (size_t)min(ts, T - 1u) * nsb * 16u : nullptr;
  FkRegs<KIND> A, B;
  fk_load<KIND>(A, rb_base, sb_of(0), rt, hn, lh, bs_tok, cr);
  __builtin_amdgcn_sched_barrier(0);

  auto park = [&](uint32_t idx, const fk_u32x4 &v) {
    if (idx < n_piece) {
      const uint32_t t = idx / ppt, c = idx - t * ppt;
      if constexpr (K4) {
        ((fk_u32x4 *)l_x)[c * TS + t] = v;
      } else {
        ft_u32x2 a, b;
        a.x = v.x; a.y = v.y; b.x = v.z; b.y = v.w;
        ((ft_u32x2 *)l_x)[(2u * c) * TS + t] = a;
        ((ft_u32x2 *)l_x)[(2u * c + 1u) * TS + t] = b;
      }
    }
  };
#if !(FK_ABL & 2)
#pragma unroll
  for (int i = 0; i < XPEEL; i++) park(tid + i * nthr, xs[i]);
  for (uint32_t idx = tid + XPEEL * nthr; idx < n_piece; idx += nthr) park(idx, *(const fk_u32x4 *)(p.xq + (size_t)idx * 16u));
#endif
  for (uint32_t i = tid; i < nsb * TS; i += nthr) {
    const uint32_t s = i / TS, t = i - s * TS;
    l_ad[i] = t < T ? p.ad[(size_t)t * nsb + s] : 0.0f;
  }
  __syncthreads();

  const ft_int16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  auto process = [&](const FkRegs<KIND> &r, uint32_t s) {
#if FK_ABL & 1
    {
      uint32_t acc_ = 0;
      if constexpr (K4) acc_ = r.hd.x ^ r.w[0].x ^ r.w[1].y ^ r.bs.x; else acc_ = r.ql[0].x ^ r.ql[3].y ^ r.qh[1].x ^ r.sc.x ^ r.d16;
      l_tdot[(s * TS + (lane & 7u)) * 16u + r16] = (float)acc_;
      if constexpr (TWO) l_tmin[(s * TS + (lane & 7u)) * 16u + r16] = 0.0f;
      return;
    }
#endif
    int isum[NREG];
    [[maybe_unused]] float im[NREG];
    float d, dmin = 0.0f;
    if constexpr (K4) {
      uint32_t sca, scb, mna, mnb;
      sca = r.hd.y & 0x3F3F3F3Fu;                                        // get_scale_min_k4, quant.rs:653-662
      scb = (r.hd.w & 0x0F0F0F0Fu) | ((r.hd.y >> 2) & 0x30303030u);
      mna = r.hd.z & 0x3F3F3F3Fu;
      mnb = ((r.hd.w >> 4) & 0x0F0F0F0Fu) | ((r.hd.z >> 2) & 0x30303030u);
      {
        // sum_j m_j * bsum_j: k 0..7 pair the mins with bsum_j >> 6 (weight 64), k 8..15 with bsum_j & 63
        const float side = lh ? 1.0f : 64.0f;
        fk_half8 mo;
#pragma unroll
        for (int j = 0; j < 4; j++) {
          mo[j] = (_Float16)(side * (float)((mna >> (8 * j)) & 0xFFu));
          mo[4 + j] = (_Float16)(side * (float)((mnb >> (8 * j)) & 0xFFu));
        }
        union { fk_u32x4 u; fk_half8 h; } bo;
        bo.u = r.bs;
        fk_float16v zf;
#pragma unroll
        for (int j = 0; j < 16; j++) zf[j] = 0.0f;
        const fk_float16v Dm = __builtin_amdgcn_mfma_f32_32x32x16_f16(bo.h, mo, zf, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < NREG; j++) im[j] = Dm[j];
      }
      const uint32_t scw = hn ? scb : sca;
      uint32_t q5[4] = {0, 0, 0, 0};
      if constexpr (KIND == FK_Q5K) {
#pragma unroll
        for (int k = 0; k < 4; k++) q5[k] = hn ? (r.qh[k] >> 4) : r.qh[k];
      }
      const fk_u32x4 *xg = (const fk_u32x4 *)l_x + ((16u * s + 8u * hm + lh) * TS + ts);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        fk_int4v wv;
#pragma unroll
        for (int k = 0; k < 4; k++) {
          uint32_t v = ((i & 1) ? (r.w[i >> 1][k] >> 4) : r.w[i >> 1][k]) & 0x0F0F0F0Fu;
          if constexpr (KIND == FK_Q5K) v |= ((q5[k] >> i) & 0x01010101u) << 4;
          wv[k] = (int)v;
        }
        union { fk_u32x4 u; fk_int4v v; } xa;
        xa.u = xg[2 * i * TS];
        const ft_int16v D = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa.v, wv, zero, 0, 0, 0);
        const int sc = (int)((scw >> (8 * i)) & 0xFFu);
#pragma unroll
        for (int j = 0; j < NREG; j++) isum[j] = i == 0 ? __mul24(sc, fk_pick(D[j], D[NREG + j], hn)) : __mul24(sc, fk_pick(D[j], D[NREG + j], hn)) + isum[j];
      }
      d = ft_f16_bits_to_f32(r.hd.x & 0xFFFFu);
      dmin = ft_f16_bits_to_f32(r.hd.x >> 16);
    } else {
      const ft_u32x2 *xg = (const ft_u32x2 *)l_x + ((32u * s + 16u * hm + lh) * TS + ts);
#define FK_G6(GI)                                                                                 \
      {                                                                                           \
        constexpr int RR = (GI) >> 1, K = (GI) & 1;                                               \
        union { ft_u32x2 v; long l; } wo, xa;                                                     \
        wo.v.x = ft_unpack4<RR>(r.ql[2 * (RR & 1) + K].x, r.qh[K].x);                             \
        wo.v.y = ft_unpack4<RR>(r.ql[2 * (RR & 1) + K].y, r.qh[K].y);                             \
        xa.v = xg[2 * (GI) * TS];                                                                 \
        const ft_int16v D = __builtin_amdgcn_mfma_i32_32x32x16_i8(xa.l, wo.l, zero, 0, 0, 0);     \
        const int sc = (int)(int8_t)(((GI) < 4 ? r.sc.x : r.sc.y) >> (8 * ((GI) & 3)));           \
        _Pragma("unroll") for (int j = 0; j < NREG; j++) {                                        \
          const int v = fk_pick(D[j], D[NREG + j], hn);                                           \
          isum[j] = (GI) == 0 ? __mul24(sc, v) : __mul24(sc, v) + isum[j];                        \
        }                                                                                         \
      }
      FK_G6(0) FK_G6(1) FK_G6(2) FK_G6(3) FK_G6(4) FK_G6(5) FK_G6(6) FK_G6(7)
#undef FK_G6
      d = ft_f16_bits_to_f32(r.d16);
    }
    // the other half's runs: the lanes 16 columns on
#pragma unroll
    for (int j = 0; j < NREG; j++) isum[j] += __shfl_xor(isum[j], 16, 64);
    // the lower half's lane turns results 0, 1 (of every four) into terms, the upper half's lane 2, 3; slots of
    // tokens beyond the batch exist and are never read
#pragma unroll
    for (int jj = 0; jj < NREG / 2; jj++) {
      const int j0 = 4 * (jj >> 1) + (jj & 1);                     // 0, 1, (4, 5)
      const int is = fk_pick(isum[j0], isum[j0 + 2], hn);
      const uint32_t t = 8u * (uint32_t)(jj >> 1) + 4u * lh + (uint32_t)(jj & 1) + 2u * hn;
      const float ad = l_ad[s * TS + t];
      const uint32_t slot = (s * TS + t) * 16u + r16;
      if constexpr (K4) {
        const float imv = fk_pickf(im[j0], im[j0 + 2], hn);
        if (GEMM_ORDER) {
          l_tmin[slot] = ad * dmin * imv;
          l_tdot[slot] = ad * (d * (float)is);
        } else {
          l_tdot[slot] = ad * (d * (float)is - dmin * imv);
        }
      } else {
        l_tdot[slot] = GEMM_ORDER ? ad * (d * (float)is) : ad * d * (float)is;
      }
    }
  };

  for (uint32_t k = 0; k < n_my; k += 2) {   // wave-uniform branches
    const bool has_b = k + 1 < n_my;
    if (has_b) fk_load<KIND>(B, rb_base, sb_of(k + 1), rt, hn, lh, bs_tok, cr);
    process(A, sb_of(k));
    if (has_b) {
      if (k + 2 < n_my) fk_load<KIND>(A, rb_base, sb_of(k + 2), rt, hn, lh, bs_tok, cr);
      process(B, sb_of(k + 1));
    }
  }
  __syncthreads();

  // ---- one lane per (token, row) of the team's row block: the row's terms in ascending order, one accumulator
  for (uint32_t i = tid - team * (n_wave * 64u); i < 16u * T; i += n_wave * 64u) {
    const uint32_t t = i >> 4, r = i & 15u;
    const uint32_t row = g16 * 16u + r;
    if (row < out_dim && !idle) {
      float acc = 0.0f;
      if constexpr (TWO) acc = fk_ordered_sum<true>(acc, l_tmin + t * 16u + r, nsb, TS * 16u);
      acc = fk_ordered_sum<false>(acc, l_tdot + t * 16u + r, nsb, TS * 16u);
      y[(size_t)t * out_dim + row] = acc;
    }
  }
}

static size_t fk_lds_bytes(uint32_t ggml_type, uint32_t in_dim, uint32_t ts, int gemm_order, uint32_t rb_per_wg = 1) {
  const size_t nsb = in_dim / 256u;
  const size_t arrays = (ggml_type != OGM_Q6_K && gemm_order) ? 2 : 1;
  return (size_t)in_dim * ts + nsb * ts * 4u + rb_per_wg * arrays * nsb * ts * 16u * 4u;
}

// Shapes the kernel takes: Q4_K, Q5_K and Q6_K, 2 to 16 tokens, activations and term tables within a workgroup's
// LDS (any row length: a workgroup takes 16 rows of a tile of 16, 32 or 64).
bool ogm_gemv_mma_eligible(uint32_t ggml_type, uint32_t in_dim, uint32_t n_tokens, int gemm_order) {
  if (ggml_type != OGM_Q4_K && ggml_type != OGM_Q5_K && ggml_type != OGM_Q6_K) return false;
  if (in_dim == 0 || in_dim % 256u != 0 || n_tokens < 2u || n_tokens > 16u) return false;
  if ((uint64_t)n_tokens * in_dim >= (1ull << 31)) return false;
  return fk_lds_bytes(ggml_type, in_dim, n_tokens <= 8u ? 8u : 16u, gemm_order) <= 160u * 1024u;
}

hipError_t ogm_launch_gemv_mma(const OgmGemvArgs &a, hipStream_t stream, const char **kernel_name) {
  if (!ogm_gemv_mma_eligible(a.ggml_type, a.in_dim, a.n_tokens, a.gemm_order) || a.n_extra > OGM_GEMV_MAX_MATS - 1 ||
      a.dump_isum || a.dump_imin)
    return hipErrorInvalidValue;
  GemmFkParams p;
  p.xq = a.act.q;
  p.ad = a.act.d;
  p.bs16 = a.act.bs16;
  p.in_dim = a.in_dim;
  p.n_tokens = a.n_tokens;
  p.nsb = a.in_dim / 256u;
  const OgmTiling tl = ogm_tiling_for(p.nsb, a.out_dim);
  p.nct = tl.nct;
  p.c_shift = tl.C == 4u ? 2u : tl.C == 2u ? 1u : 0u;
  p.r_shift = tl.R == 16u ? 4u : tl.R == 32u ? 5u : 6u;
  uint32_t n_wg = 0;
  for (uint32_t m = 0; m < OGM_GEMV_MAX_MATS; m++) {
    if (m <= a.n_extra) {
      p.wt[m] = m ? a.extra_wt[m - 1] : a.wt;
      p.y[m] = m ? a.extra_y[m - 1] : a.y;
      p.out_dim[m] = m ? a.extra_out_dim[m - 1] : a.out_dim;
      n_wg += (p.out_dim[m] + 15u) / 16u;
    } else {
      p.wt[m] = nullptr;
      p.y[m] = nullptr;
      p.out_dim[m] = 0;
    }
    p.wg_end[m] = n_wg;
  }
  if (n_wg == 0) return hipSuccess;
  if (a.ggml_type != OGM_Q6_K && p.bs16 == nullptr) return hipErrorInvalidValue;
  // waves: the largest divisor of the column tiles up to 16 (4096 inputs: 4 waves, one tile each; 14336: 14)
  const uint32_t ts = a.n_tokens <= 8u ? 8u : 16u;
  // Waves per workgroup: a wave takes every waves-th super-block of the row block.  Few workgroups (1024 rows:
  // 64) want many waves, each with a short chain of super-blocks; many workgroups (28672 rows: 1792) fill the
  // device with four waves each and keep several workgroups per compute unit.  Aim at sixteen waves per unit.
  // Many row blocks (the gate and up projections together: 1792): two per workgroup, whose eight waves share one
  // copy of the activations in LDS -- four row blocks resident on a compute unit instead of three, half the
  // staging traffic (28672 rows at 8 tokens: 23.7 -> 21.1 us).
  const uint32_t rbw = (n_wg >= 1024u && fk_lds_bytes(a.ggml_type, a.in_dim, ts, a.gemm_order, 2) <= 80u * 1024u) ? 2u : 1u;
  p.rb_per_wg = rbw;
  uint32_t want = a.wg_waves ? a.wg_waves : 4096u / n_wg;
  const uint32_t cap = ts == 8u ? 16u : 8u;
  want = want < 4u ? 4u : want > cap ? cap : want;
  if (want > p.nsb) want = p.nsb;
  const uint32_t chain = (p.nsb + want - 1u) / want;            // super-blocks of the busiest wave
  const uint32_t waves = (p.nsb + chain - 1u) / chain;          // the fewest waves with that chain
  const size_t lds_bytes = fk_lds_bytes(a.ggml_type, a.in_dim, ts, a.gemm_order, rbw);
  const void *fn = nullptr;
  const char *name = "";
#define FK_PICK(KIND_, NAME_)                                                                                 \
  do {                                                                                                        \
    fn = ts == 8u ? (a.gemm_order ? (const void *)ogm_gemm_fk_kernel<KIND_, 8, true>                          \
                                  : (const void *)ogm_gemm_fk_kernel<KIND_, 8, false>)                        \
                  : (a.gemm_order ? (const void *)ogm_gemm_fk_kernel<KIND_, 16, true>                         \
                                  : (const void *)ogm_gemm_fk_kernel<KIND_, 16, false>);                      \
    name = NAME_;                                                                                             \
  } while (0)
  if (a.ggml_type == OGM_Q4_K) FK_PICK(FK_Q4K, "ogm_gemm_fk_kernel<Q4_K>");
  else if (a.ggml_type == OGM_Q5_K) FK_PICK(FK_Q5K, "ogm_gemm_fk_kernel<Q5_K>");
  else FK_PICK(FK_Q6K, "ogm_gemm_fk_kernel<Q6_K>");
#undef FK_PICK
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return e;
  void *kargs[] = {(void *)&p};
  e = hipLaunchKernel(fn, dim3((n_wg + rbw - 1u) / rbw), dim3(64u * waves * rbw), kargs, lds_bytes, stream);
  if (e != hipSuccess) return e;
  if (kernel_name) *kernel_name = name;
  return hipGetLastError();
}
