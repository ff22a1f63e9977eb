// gfx950 prefill GEMM for Q4_K weights on MFMA, bit-compatible with the CPU path's K-quant GEMM
// (gemm_k_q4_k + accumulate_sym32, engine/vecdot.rs:2213-2303 of orangu-server).
//
// The integer stage stays exact on the matrix cores by keeping every operand an *integer-valued
// f16*.  A weight enters centred and pre-scaled, sc_j * (q - 8) with |.| <= 504; an activation as
// its int8 value.  Products are exact in f32 and a whole super-block (256 k) sums to at most
// 63 * 8 * 127 * 256 = 16 386 048 < 2^24, so the MFMA's f32 accumulator holds
//   c = sum_j sc_j * dot32(q_j - 8, x_j)
// exactly.  The centring is undone by one more MFMA per super-block over the per-32 activation
// sums, corr = 8 * sum_j sc_j * bsum_j (bsum split as 64*bh + bl so that every operand is exact in
// f16; |corr| < 2^24), and `c + corr` is one f32 add of two exact integers: it rounds the exact
// isum once, to nearest even -- the value of the reference's `isum as f32`.  The min term
// sum_j m_j * bsum_j comes from the same kind of MFMA.  The f32 epilogue then follows the
// reference's order: first `acc -= (ad*dmin) * imin` over all super-blocks, then
// `acc += ad * (d * isum)` over all super-blocks.
//
// Tiling: a workgroup owns 128 rows x 128 tokens and has sixteen waves, four per SIMD.  Eight
// "multiplying" waves own 64 rows x 32 tokens each = two v_mfma_f32_32x32x16_f16 tiles; eight
// "feeding" waves do the global loads, the dequantization (v_perm byte spread, magic-number
// int->f16, packed f16 add and multiply: half a 16-byte piece of qs per thread and stage) and the
// LDS stores, so that on every SIMD the matrix pipe and the vector pipe are busy at the same time.
// The k loop advances 64 at a time (a quarter super-block: one piece pair of qs, i.e. sub-blocks
// 2g and 2g+1); LDS is double buffered, global loads run two stages ahead through three rotating
// register sets, and there is one barrier per stage.
#include <hip/hip_runtime.h>

#include "ogm_kernels.h"
#include "ogm_layout.h"
#include "ogm_nib32_dev.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));

#define GM_BN 128   // rows per workgroup
#define GM_BT 128   // tokens per workgroup
#define GM_KS 64    // k per stage
#define GM_STAGE_HALFS (128 * GM_KS)   // f16 per staged tile (A or B) of one stage

struct GemmParams {
  const uint8_t *wt;      // tile-planar Q4_K
  const _Float16 *xh;     // [T][in_dim] int8 activations as f16
  const int8_t *xq;       // [T][in_dim] the int8 activations themselves (wide kernel)
  const _Float16 *bs16;   // [T][nsb][16]: floor(bsum_j / 64) for j = 0..7, then bsum_j mod 64
  const float *ad;        // [T][nsb] activation scales (per 256)
  float *y;               // [T][out_dim]
  uint32_t in_dim, out_dim, n_tokens, nsb;
  uint32_t c_shift, r_shift, nct;  // weight tiles of R = 1 << r_shift rows x C = 1 << c_shift blocks
  // further matrices over the same activations (q, k, v), their row tiles following in grid.y
  uint32_t n_extra;
  const uint8_t *extra_wt[OGM_GEMM_MAX_MATS - 1];
  float *extra_y[OGM_GEMM_MAX_MATS - 1];
  uint32_t extra_out_dim[OGM_GEMM_MAX_MATS - 1];
};

// The matrix a workgroup's row tile belongs to: rewrites p for it and returns the tile's index
// within that matrix.
__device__ __forceinline__ uint32_t gm_pick_matrix(GemmParams &p, uint32_t row_tile) {
#pragma unroll
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
    const uint32_t tiles = (p.out_dim + 127u) / 128u;
    if (m < p.n_extra && row_tile >= tiles) {
      row_tile -= tiles;
      p.wt = p.extra_wt[m];
      p.y = p.extra_y[m];
      p.out_dim = p.extra_out_dim[m];
    } else {
      break;
    }
  }
  return row_tile;
}

__device__ __forceinline__ float gm_f16_bits_to_f32(uint32_t bits16) {
  union { unsigned short u; _Float16 h; } v;
  v.u = (unsigned short)bits16;
  return (float)v.h;
}

// int8 activations -> f16 and per-32 sums -> (bh, bl) f16 pairs, once per matmul.
__global__ void ogm_gemm_prep_kernel(const int8_t *__restrict__ q, const int16_t *__restrict__ bsum,
                                     _Float16 *__restrict__ xh, _Float16 *__restrict__ bs16, size_t n8,
                                     size_t n_sb) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (xh && i < n8) {
    const int2 v = ((const int2 *)q)[i];
    half8 o;
    o[0] = (_Float16)(float)(int8_t)(v.x);
    o[1] = (_Float16)(float)(int8_t)(v.x >> 8);
    o[2] = (_Float16)(float)(int8_t)(v.x >> 16);
    o[3] = (_Float16)(float)(int8_t)(v.x >> 24);
    o[4] = (_Float16)(float)(int8_t)(v.y);
    o[5] = (_Float16)(float)(int8_t)(v.y >> 8);
    o[6] = (_Float16)(float)(int8_t)(v.y >> 16);
    o[7] = (_Float16)(float)(int8_t)(v.y >> 24);
    ((half8 *)xh)[i] = o;
  }
  if (i < n_sb) {
    const uint4 b = ((const uint4 *)bsum)[i];  // eight i16
    const uint32_t w[4] = {b.x, b.y, b.z, b.w};
    half8 bh, bl;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int b0 = (int)(int16_t)(w[j] & 0xFFFFu), b1 = ((int)w[j]) >> 16;
      bh[2 * j] = (_Float16)(float)(b0 >> 6);  // floor(b / 64)
      bl[2 * j] = (_Float16)(float)(b0 & 63);
      bh[2 * j + 1] = (_Float16)(float)(b1 >> 6);
      bl[2 * j + 1] = (_Float16)(float)(b1 & 63);
    }
    ((half8 *)bs16)[2 * i] = bh;
    ((half8 *)bs16)[2 * i + 1] = bl;
  }
}

// Bytes b0..b3 of `w`: low nibbles (q - 8) * sl and high nibbles (q - 8) * sh as packed f16.
// 0x6400 | n is the f16 1024 + n and 0x5400 | (n << 4) the f16 64 + n: subtracting 1032 or 72
// leaves n - 8 exactly and the product with a scale <= 63 is an integer below 2^11, exact too.
__device__ __forceinline__ void dequant8(uint32_t w, half2v sl2, half2v sh2, uint32_t &lo01,
                                         uint32_t &lo23, uint32_t &hi01, uint32_t &hi23) {
  const uint32_t p01 = __builtin_amdgcn_perm(0u, w, 0x0c010c00u);  // (b0, 0, b1, 0)
  const uint32_t p23 = __builtin_amdgcn_perm(0u, w, 0x0c030c02u);  // (b2, 0, b3, 0)
  union { uint32_t u; half2v h; } a, b, c, d;
  const half2v k1032 = {(_Float16)-1032.0f, (_Float16)-1032.0f};
  const half2v k72 = {(_Float16)-72.0f, (_Float16)-72.0f};
  a.u = (p01 & 0x000F000Fu) | 0x64006400u;
  b.u = (p23 & 0x000F000Fu) | 0x64006400u;
  c.u = (p01 & 0x00F000F0u) | 0x54005400u;
  d.u = (p23 & 0x00F000F0u) | 0x54005400u;
  a.h = (a.h + k1032) * sl2;
  b.h = (b.h + k1032) * sl2;
  c.h = (c.h + k72) * sh2;
  d.h = (d.h + k72) * sh2;
  lo01 = a.u;
  lo23 = b.u;
  hi01 = c.u;
  hi23 = d.u;
}

// get_scale_min_k4 (quant.rs:653-662) for all eight sub-blocks: sc 0..3 | sc 4..7, one per byte.
__device__ __forceinline__ void q4k_scales(const uint4 &hd, uint32_t &sca, uint32_t &scb) {
  sca = hd.y & 0x3F3F3F3Fu;
  scb = (hd.w & 0x0F0F0F0Fu) | ((hd.y >> 2) & 0x30303030u);
}
__device__ __forceinline__ void q4k_mins(const uint4 &hd, uint32_t &mna, uint32_t &mnb) {
  mna = hd.z & 0x3F3F3F3Fu;
  mnb = ((hd.w >> 4) & 0x0F0F0F0Fu) | ((hd.z >> 2) & 0x30303030u);
}

// The K = 16 operand of the side MFMAs for one row: k 0..7 pair with bh_j, k 8..15 with bl_j, so
// a lane of the upper half (lh = 0) carries hi_scale * v_j and of the lower half v_j * lo_scale.
__device__ __forceinline__ half8 side_operand(uint32_t va, uint32_t vb, float scale) {
  half8 o;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    o[j] = (_Float16)(scale * (float)((va >> (8 * j)) & 0xFFu));
    o[4 + j] = (_Float16)(scale * (float)((vb >> (8 * j)) & 0xFFu));
  }
  return o;
}

// LDS rows of the staged tiles are 128 bytes (64 f16) without padding; the 16-byte chunk c of row
// r sits at chunk c ^ (r & 7) ^ ((r >> 3) & 1).  Eight consecutive rows then cover all eight chunk
// positions (no conflict if a 128-bit access is served eight lanes at a time over 32 banks), and
// in sixteen consecutive rows two rows with the same chunk position differ in row parity, i.e.
// in the 128-byte half of a 256-byte bank line (no conflict with sixteen lanes over 64 banks).
__device__ __forceinline__ uint32_t gm_swz(uint32_t row, uint32_t chunk) {
  return row * 64u + ((chunk ^ (row & 7u) ^ ((row >> 3) & 1u)) << 3);  // in f16 units
}

__global__ __launch_bounds__(1024) void ogm_gemm_q4k_kernel(GemmParams p) {
  extern __shared__ __align__(16) uint8_t lds[];
  _Float16 *A_l = (_Float16 *)lds;                  // [2][128][64]
  _Float16 *B_l = A_l + 2 * GM_STAGE_HALFS;         // [2][128][64]
  _Float16 *a2_l = B_l + 2 * GM_STAGE_HALFS;        // [128 rows][16]: 512*sc_j | 8*sc_j
  _Float16 *b2_l = a2_l + 128 * 16;                 // [128 tokens][16]: bh_j | bl_j
  float *d_l = (float *)(b2_l + 128 * 16);          // [128]
  float *dmin_t = d_l + 128;                        // pass 1 only: [nsb][128]

  // Sixteen waves, four per SIMD: waves 0..7 multiply (MFMA and the f32 steps), waves 8..15 feed
  // them (global loads, dequantization, LDS stores), so that on every SIMD the matrix pipe and the
  // vector pipe work at the same time.  Both halves run the same number of barriers.
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const bool producer = wave >= 8u;
  const uint32_t rt = tid & 511u;                   // thread index within its half
  const uint32_t wr = wave & 1u, wt_ = (wave & 7u) >> 1;   // multiplying wave: row half (64 rows), token quarter (32)
  const uint32_t t0 = blockIdx.x * GM_BT, r0 = gm_pick_matrix(p, blockIdx.y) * GM_BN;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;

  // Address of block `s` of row `row` in the tile-planar layout (piece 0: d, dmin, scales).
  // Rows past the matrix are clamped onto its last row; their results are never stored.
  // Byte offsets stay below 4 GiB (checked by the launcher), so they are 32-bit: a row part
  // that a thread computes once and a super-block part that is the same for every thread.
  auto row_off = [&](uint32_t row) -> uint32_t {
    row = min(row, p.out_dim - 1u);
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    return rb * p.nct * 9216u + r * 16u;
  };
  auto sb_off = [&](uint32_t s) -> uint32_t {
    const uint32_t ct = s >> p.c_shift, cl = s & ((1u << p.c_shift) - 1u);
    return ct * 9216u + (cl << p.r_shift) * 16u;
  };
  // token of this lane's column, clamped like the rows
  const uint32_t tk = min(t0 + 32u * wt_ + l32, p.n_tokens - 1u);

  float16v y0, y1;  // rows 64 wr + 0..31 and + 32..63, tokens 32 wt_ + 0..31
#pragma unroll
  for (int r = 0; r < 16; r++) y0[r] = y1[r] = 0.0f;
  float16v zero;
#pragma unroll
  for (int r = 0; r < 16; r++) zero[r] = 0.0f;

  // ---------------- pass 1: acc -= (ad * dmin) * sum_j m_j * bsum_j, all super-blocks first
  for (uint32_t i = tid; i < p.nsb * 128u; i += 1024u) {
    const uint32_t s = i >> 7, lr = i & 127u;
    const uint32_t h = *(const uint32_t *)(p.wt + (row_off(r0 + lr) + sb_off(s)));
    dmin_t[i] = gm_f16_bits_to_f32(h >> 16);
  }
  __syncthreads();
  const uint32_t ro0 = row_off(r0 + 64u * wr + l32), ro1 = row_off(r0 + 64u * wr + 32u + l32);
  const uint32_t tko = tk * p.nsb;  // this token's first (token, super-block) index
  if (!producer) {
    const float side_scale = lh ? 1.0f : 64.0f;
    // four super-blocks at a time, so that four sets of loads share one trip to memory
#pragma unroll 1
    for (uint32_t sg = 0; sg < p.nsb; sg += 4u) {
      uint4 hd0[4], hd1[4];
      half8 b2[4];
      float adv[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const uint32_t su = min(sg + u, p.nsb - 1u);
        hd0[u] = *(const uint4 *)(p.wt + (ro0 + sb_off(su)));
        hd1[u] = *(const uint4 *)(p.wt + (ro1 + sb_off(su)));
        b2[u] = *(const half8 *)(p.bs16 + ((tko + su) * 16u + 8u * lh));
        adv[u] = p.ad[tko + su];
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        if (sg + u < p.nsb) {
          uint32_t mna, mnb;
          q4k_mins(hd0[u], mna, mnb);
          const half8 a10 = side_operand(mna, mnb, side_scale);
          q4k_mins(hd1[u], mna, mnb);
          const half8 a11 = side_operand(mna, mnb, side_scale);
          const float16v im0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a10, b2[u], zero, 0, 0, 0);
          const float16v im1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a11, b2[u], zero, 0, 0, 0);
          const float *dm = dmin_t + (sg + u) * 128u + 64u * wr + 4u * lh;
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++) {
            const float4 m0 = *(const float4 *)(dm + 8 * q4), m1 = *(const float4 *)(dm + 32 + 8 * q4);
            y0[4 * q4 + 0] -= adv[u] * m0.x * im0[4 * q4 + 0];
            y0[4 * q4 + 1] -= adv[u] * m0.y * im0[4 * q4 + 1];
            y0[4 * q4 + 2] -= adv[u] * m0.z * im0[4 * q4 + 2];
            y0[4 * q4 + 3] -= adv[u] * m0.w * im0[4 * q4 + 3];
            y1[4 * q4 + 0] -= adv[u] * m1.x * im1[4 * q4 + 0];
            y1[4 * q4 + 1] -= adv[u] * m1.y * im1[4 * q4 + 1];
            y1[4 * q4 + 2] -= adv[u] * m1.z * im1[4 * q4 + 2];
            y1[4 * q4 + 3] -= adv[u] * m1.w * im1[4 * q4 + 3];
          }
        }
      }
    }
  }

  // ---------------- pass 2: acc += ad * (d * sum_j sc_j * dot32_j)
  // Staging roles.  Weights: half a 16-byte piece of qs per thread (8 bytes = 8 low-nibble and 8
  // high-nibble weights).  Activations: two 16-byte chunks per thread.  Once per super-block
  // also the row's scales (side operand and d) and one chunk of bh | bl.
  const uint32_t pid = rt >> 1, half = rt & 1u;
  const uint32_t lr_a = (pid >> 5) * 16u + (pid & 15u), hh = (pid >> 4) & 1u;
  const uint32_t btok = rt >> 3, bpart = rt & 7u;   // chunk i: token btok + 64 i, part bpart
  const uint32_t bt0 = min(t0 + btok, p.n_tokens - 1u), bt1 = min(t0 + btok + 64u, p.n_tokens - 1u);
  const uint32_t roa = row_off(r0 + lr_a) + hh * 1024u + 8u * half;   // this thread's half piece
  const uint32_t bo0 = bt0 * p.in_dim + bpart * 8u, bo1 = bt1 * p.in_dim + bpart * 8u;  // in f16
  // (the upper half of the workgroup repeats the lower half's bh | bl chunk: no branch needed)
  const uint32_t b2o = min(t0 + ((rt & 255u) >> 1), p.n_tokens - 1u) * p.nsb * 16u + 8u * (rt & 1u);
  // Loads run two stages ahead of the MFMAs through three rotating register sets (a stage is
  // shorter than a trip to memory); the header and bh | bl loads of a super-block have one
  // set, which is consumed before the next super-block's are issued.
  uint2 qv_0, qv_1, qv_2;
  uint4 bx0_0, bx0_1, bx0_2, bx1_0, bx1_1, bx1_2;
  uint4 hdx = make_uint4(0, 0, 0, 0), b2x = make_uint4(0, 0, 0, 0);
  uint32_t sca = 0, scb = 0;
  float dnext = 0.0f;

#define GM_LOAD_STAGE(S, G, K)                                                                    \
  do {                                                                                            \
    const uint32_t so_ = sb_off(S);                                                               \
    if ((G) == 0) hdx = *(const uint4 *)(p.wt + (roa - hh * 1024u - 8u * half + so_));            \
    if ((G) == 1) b2x = *(const uint4 *)(p.bs16 + (b2o + (S) * 16u));                              \
    qv_##K = *(const uint2 *)(p.wt + (roa + so_ + (1u + 2u * (G)) * 1024u));                      \
    const uint32_t ko_ = (S) * 256u + (G) * 64u;                                                  \
    bx0_##K = *(const uint4 *)(p.xh + (bo0 + ko_));                                               \
    bx1_##K = *(const uint4 *)(p.xh + (bo1 + ko_));                                               \
  } while (0)

#define GM_STORE_STAGE(G, BUF, K)                                                                 \
  do {                                                                                            \
    if ((G) == 0) {                                                                               \
      q4k_scales(hdx, sca, scb);                                                                  \
      dnext = gm_f16_bits_to_f32(hdx.x & 0xFFFFu);                                                \
    }                                                                                             \
    const uint32_t scw_ = (G) < 2 ? sca : scb;                                                    \
    const uint32_t sh_ = ((G) & 1u) * 16u;                                                        \
    const _Float16 slo_ = (_Float16)(float)((scw_ >> sh_) & 0xFFu);                               \
    const _Float16 shi_ = (_Float16)(float)((scw_ >> (sh_ + 8u)) & 0xFFu);                        \
    const half2v sl2_ = {slo_, slo_}, sh2_ = {shi_, shi_};                                        \
    uint4 lo_, hi_; /* 8 low-nibble weights, 8 high-nibble weights, as f16 */                     \
    dequant8(qv_##K.x, sl2_, sh2_, lo_.x, lo_.y, hi_.x, hi_.y);                                   \
    dequant8(qv_##K.y, sl2_, sh2_, lo_.z, lo_.w, hi_.z, hi_.w);                                   \
    /* piece 1+2g+hh holds qs[32g+16hh ..]: low nibbles are k 16hh.. of the stage, high 32+16hh.. */ \
    _Float16 *ab_ = A_l + (BUF) * GM_STAGE_HALFS;                                                 \
    *(uint4 *)(ab_ + gm_swz(lr_a, 2u * hh + half)) = lo_;                                         \
    *(uint4 *)(ab_ + gm_swz(lr_a, 4u + 2u * hh + half)) = hi_;                                    \
    _Float16 *bb_ = B_l + (BUF) * GM_STAGE_HALFS;                                                 \
    *(uint4 *)(bb_ + gm_swz(btok, bpart)) = bx0_##K;                                              \
    *(uint4 *)(bb_ + gm_swz(btok + 64u, bpart)) = bx1_##K;                                        \
    if ((G) == 1) {                                                                               \
      /* Side tables of this super-block.  Their readers (after stage 3) of the last super-block \
         are two barriers behind, their next readers two barriers ahead. */                      \
      /* the four threads of a row write the same values */                                      \
      *(half8 *)(a2_l + lr_a * 16u + 8u * half) = side_operand(sca, scb, half ? 8.0f : 512.0f);   \
      d_l[lr_a] = dnext;                                                                          \
      *(uint4 *)(b2_l + ((rt & 255u) >> 1) * 16u + 8u * (rt & 1u)) = b2x;                         \
    }                                                                                             \
  } while (0)

  // One stage of a feeding wave: issue the loads of the stage two ahead, dequantize and park
  // the next stage in the LDS buffer the multiplying waves are not reading.
#define GM_PRODUCE(G, KL, KS)                                                                     \
  do {                                                                                            \
    /* past the end the last super-block is loaded again and parked in the idle buffer */        \
    GM_LOAD_STAGE(min((G) < 2 ? s : s + 1u, p.nsb - 1u), (uint32_t)(((G) + 2) & 3), KL);          \
    GM_STORE_STAGE((uint32_t)(((G) + 1) & 3), ((G) & 1u) ^ 1u, KS);                               \
    __syncthreads();                                                                              \
  } while (0)

  // One stage of a multiplying wave: this stage's MFMAs from LDS, then, after the super-block's
  // last stage, its f32 step.
#define GM_CONSUME(G)                                                                             \
  do {                                                                                            \
    const uint32_t buf = (G) & 1u;                                                                \
    if ((G) == 0) adv = p.ad[tko + s]; /* needed three stages from now */                         \
    const _Float16 *ab = A_l + buf * GM_STAGE_HALFS, *bb = B_l + buf * GM_STAGE_HALFS;            \
    half8 a0 = *(const half8 *)(ab + gm_swz(ra, lh));                                             \
    half8 a1 = *(const half8 *)(ab + gm_swz(ra + 32u, lh));                                       \
    half8 b0 = *(const half8 *)(bb + gm_swz(rbk, lh));                                            \
    _Pragma("unroll") for (int kk = 0; kk < 4; kk++) {                                            \
      half8 na0 = a0, na1 = a1, nb0 = b0;                                                         \
      if (kk < 3) {                                                                               \
        na0 = *(const half8 *)(ab + gm_swz(ra, 2u * (kk + 1) + lh));                              \
        na1 = *(const half8 *)(ab + gm_swz(ra + 32u, 2u * (kk + 1) + lh));                        \
        nb0 = *(const half8 *)(bb + gm_swz(rbk, 2u * (kk + 1) + lh));                             \
      }                                                                                           \
      /* the super-block's first step starts a fresh accumulator */                              \
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b0, ((G) == 0 && kk == 0) ? zero : c0, 0, 0, 0); \
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b0, ((G) == 0 && kk == 0) ? zero : c1, 0, 0, 0); \
      a0 = na0; a1 = na1; b0 = nb0;                                                               \
    }                                                                                             \
    if ((G) == 3) GM_SB_EPILOGUE();                                                               \
    __syncthreads();                                                                              \
  } while (0)

  // isum = c + corr (one rounding of the exact integer), then the reference's f32 steps
#define GM_SB_EPILOGUE()                                                                          \
  do {                                                                                            \
    const half8 b2 = *(const half8 *)(b2_l + rbk * 16u + 8u * lh);                                \
    const half8 a20 = *(const half8 *)(a2_l + ra * 16u + 8u * lh);                                \
    const half8 a21 = *(const half8 *)(a2_l + (ra + 32u) * 16u + 8u * lh);                        \
    const float16v corr0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a20, b2, zero, 0, 0, 0);        \
    const float16v corr1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a21, b2, zero, 0, 0, 0);        \
    const float *dp = d_l + 64u * wr + 4u * lh;                                                   \
    _Pragma("unroll") for (int q4 = 0; q4 < 4; q4++) {                                            \
      const float4 d0 = *(const float4 *)(dp + 8 * q4), d1 = *(const float4 *)(dp + 32 + 8 * q4); \
      y0[4 * q4 + 0] += adv * (d0.x * (c0[4 * q4 + 0] + corr0[4 * q4 + 0]));                      \
      y0[4 * q4 + 1] += adv * (d0.y * (c0[4 * q4 + 1] + corr0[4 * q4 + 1]));                      \
      y0[4 * q4 + 2] += adv * (d0.z * (c0[4 * q4 + 2] + corr0[4 * q4 + 2]));                      \
      y0[4 * q4 + 3] += adv * (d0.w * (c0[4 * q4 + 3] + corr0[4 * q4 + 3]));                      \
      y1[4 * q4 + 0] += adv * (d1.x * (c1[4 * q4 + 0] + corr1[4 * q4 + 0]));                      \
      y1[4 * q4 + 1] += adv * (d1.y * (c1[4 * q4 + 1] + corr1[4 * q4 + 1]));                      \
      y1[4 * q4 + 2] += adv * (d1.z * (c1[4 * q4 + 2] + corr1[4 * q4 + 2]));                      \
      y1[4 * q4 + 3] += adv * (d1.w * (c1[4 * q4 + 3] + corr1[4 * q4 + 3]));                      \
    }                                                                                             \
  } while (0)

  if (producer) {   // while the multiplying waves run pass 1
    GM_LOAD_STAGE(0u, 0u, 0);
    GM_LOAD_STAGE(0u, 1u, 1);
    GM_STORE_STAGE(0u, 0u, 0);
  }
  __syncthreads();

  const uint32_t ra = 64u * wr + l32, rbk = 32u * wt_ + l32;
  if (producer) {
    // the set of stage n = 4 s + g is n mod 3, so three super-blocks make one period
#define GM_PRODUCE_SB(K0, K1, K2)                                                                 \
  do {                                                                                            \
    GM_PRODUCE(0, K2, K1);   /* loads stage 4s+2, parks stage 4s+1 */                             \
    GM_PRODUCE(1, K0, K2);                                                                        \
    GM_PRODUCE(2, K1, K0);                                                                        \
    GM_PRODUCE(3, K2, K1);                                                                        \
    s++;                                                                                          \
  } while (0)
    uint32_t s = 0;
    while (s < p.nsb) {
      GM_PRODUCE_SB(0, 1, 2);
      if (s >= p.nsb) break;
      GM_PRODUCE_SB(1, 2, 0);
      if (s >= p.nsb) break;
      GM_PRODUCE_SB(2, 0, 1);
    }
#undef GM_PRODUCE_SB
    return;
  }
#pragma unroll 1
  for (uint32_t s = 0; s < p.nsb; s++) {
    float16v c0, c1;
    float adv;
    GM_CONSUME(0);
    GM_CONSUME(1);
    GM_CONSUME(2);
    GM_CONSUME(3);
  }
#undef GM_LOAD_STAGE
#undef GM_STORE_STAGE
#undef GM_PRODUCE
#undef GM_CONSUME
#undef GM_SB_EPILOGUE

  // ---------------- store: a lane holds one token column and its rows in runs of four
  const uint32_t t = t0 + 32u * wt_ + l32;
  if (t < p.n_tokens) {
    const bool vec = (p.out_dim & 3u) == 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const float16v &yy = i ? y1 : y0;
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const uint32_t row = r0 + 64u * wr + 32u * i + 8u * q4 + 4u * lh;
        float *dst = p.y + (size_t)t * p.out_dim + row;
        if (vec && row + 3u < p.out_dim) {
          *(float4 *)dst = make_float4(yy[4 * q4], yy[4 * q4 + 1], yy[4 * q4 + 2], yy[4 * q4 + 3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++)
            if (row + e < p.out_dim) dst[e] = yy[4 * q4 + e];
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Q4_K on the int8 matrix cores: 128 rows x 128 tokens per workgroup, four multiplying and four
// feeding waves.
//
// The f16 kernels above fold the sub-block scale into the weight operand (sc_j * (q - 8) as f16)
// so that the matrix cores produce isum directly; the price is two-byte operands and, for the
// other K-quants, two chains.  Here the operands stay int8 - the nibbles as they are, and the
// activations as the quantizer left them - and one v_mfma_i32_32x32x32_i8 produces the 32 x 32
// exact dot products of ONE sub-block (dot32 of vecdot.rs:471-502); the scale is applied to that
// partial sum with integer multiply-adds, isum += sc_j * dot32_j exactly as accumulate_sym32
// (vecdot.rs:2271-2303) does, in 32-bit integers with no 2^24 bound to respect.  The tokens are
// the matrix instruction's row operand and the weight rows its column operand: a lane then
// owns one weight row (its column) and 16 tokens (its registers), so the scale of a
// multiply-add is one register for all sixteen.  Half the LDS bytes per product, twice the
// matrix rate, sixteen integer multiply-adds per matrix instruction.
//
// LDS rows hold the 64 bytes of a stage (two sub-blocks) in 80 bytes; a lane's operand is the 16
// bytes at 32 * sub-block + 16 * (lane / 32) of its row - both operands use the same bytes of k,
// which is all the dot product asks.

typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int16v __attribute__((ext_vector_type(16)));

#define GI_ROW 80u                   // bytes of an LDS row (64 int8 + padding)
#define GI_WTILE (128u * GI_ROW)     // the weight tile of a stage

// Twelve waves: eight multiply (wave w: rows 64 (w / 4) .. + 63, tokens 32 (w % 4) .. + 31 of the
// workgroup's 128 x 128) and four feed them.  Two multiplying waves per SIMD, so that one's matrix
// instructions run under the other's multiply-adds; the two kinds of waves run loops of their
// own (same number of barriers), so that what one keeps in registers is not kept alive in the other.
// Q5_K (KKind::Q4K rows as well, vecdot.rs:2064-2088) differs in the staging alone: the weight is
// the nibble with bit j of qh[l] on top, 0..31, and its unit has 11 pieces (header, qh, qs).
template <bool Q5>
__device__ __forceinline__ void gemm_i8_body(GemmParams p) {
  constexpr uint32_t TILE_BYTES = Q5 ? 11264u : 9216u;   // 64 units of 176 / 144 bytes
  constexpr uint32_t QS_PIECE0 = Q5 ? 3u : 1u;           // first piece of qs
  __shared__ __align__(16) uint8_t w_l[2][GI_WTILE];   // weights 0..15 (Q5_K: 0..31), [row][64 of 80]
  __shared__ __align__(16) uint8_t x_l[2][GI_WTILE];   // activations, [token][64 of 80]
  __shared__ __align__(8) uint2 sc_l[2][128];          // per super-block: the rows' eight scales, one byte each
  __shared__ __align__(16) float d_l[2][128];          // the rows' d
  __shared__ __align__(16) float ad_l[2][128];         // the tokens' activation scale
  __shared__ __align__(16) float p1_dmin[8][128];      // pass 1, eight super-blocks at a time
  __shared__ __align__(16) float p1_ad[8][128];

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const bool producer = wave >= 8u;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const uint32_t tq = wave & 3u, rh = (wave >> 2) & 1u;
  const uint32_t t0 = blockIdx.x * 128u, r0 = gm_pick_matrix(p, blockIdx.y) * 128u;
  const uint32_t tw = 32u * tq;   // the wave's first token within the workgroup

  auto row_off = [&](uint32_t row) -> uint32_t {
    row = min(row, p.out_dim - 1u);
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    return rb * p.nct * TILE_BYTES + r * 16u;
  };
  auto sb_off = [&](uint32_t s) -> uint32_t {
    const uint32_t ct = s >> p.c_shift, cl = s & ((1u << p.c_shift) - 1u);
    return ct * TILE_BYTES + (cl << p.r_shift) * 16u;
  };

  // y0 / y1: tokens t0 + tw + (8 (r / 4) + 4 lh + r % 4), rows r0 + 64 rh + l32 and + 32
  float16v y0, y1;
#pragma unroll
  for (int r = 0; r < 16; r++) y0[r] = y1[r] = 0.0f;

  // ---------------- pass 1: acc -= (ad * dmin) * sum_j m_j * bsum_j, all super-blocks first
  // (vecdot.rs:2226-2240), on the f16 matrix cores as in the kernels above, tokens as rows
  {
    float16v zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.0f;
    const uint32_t ro0 = row_off(r0 + 64u * rh + l32), ro1 = row_off(r0 + 64u * rh + 32u + l32);
    const uint32_t tk = min(t0 + tw + l32, p.n_tokens - 1u) * p.nsb;
    const float side_scale = lh ? 1.0f : 64.0f;
    for (uint32_t sg = 0; sg < p.nsb; sg += 8u) {
      // the tables of this round: dmin of (super-block, row) and ad of (super-block, token)
      for (uint32_t i = tid; i < 8u * 128u; i += 768u) {
        const uint32_t u = i >> 7, k = i & 127u, su = min(sg + u, p.nsb - 1u);
        const uint32_t h = *(const uint32_t *)(p.wt + (row_off(r0 + k) + sb_off(su)));
        p1_dmin[u][k] = gm_f16_bits_to_f32(h >> 16);
        p1_ad[u][k] = p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + su];
      }
      __syncthreads();
      if (!producer) {
#pragma unroll 2
        for (uint32_t u = 0; u < 8u; u++) {
          if (sg + u >= p.nsb) break;
          const uint32_t su = sg + u;
          const uint4 hd0 = *(const uint4 *)(p.wt + (ro0 + sb_off(su)));
          const uint4 hd1 = *(const uint4 *)(p.wt + (ro1 + sb_off(su)));
          const half8 b2 = *(const half8 *)(p.bs16 + ((tk + su) * 16u + 8u * lh));
          uint32_t mna, mnb;
          q4k_mins(hd0, mna, mnb);
          const half8 a10 = side_operand(mna, mnb, side_scale);
          q4k_mins(hd1, mna, mnb);
          const half8 a11 = side_operand(mna, mnb, side_scale);
          const float dm0 = p1_dmin[u][64u * rh + l32], dm1 = p1_dmin[u][64u * rh + 32u + l32];
          const float16v im0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b2, a10, zero, 0, 0, 0);
          const float16v im1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b2, a11, zero, 0, 0, 0);
          const float *adp = &p1_ad[u][tw + 4u * lh];
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++) {
            const float4 a4 = *(const float4 *)(adp + 8 * q4);
            y0[4 * q4 + 0] -= a4.x * dm0 * im0[4 * q4 + 0];
            y0[4 * q4 + 1] -= a4.y * dm0 * im0[4 * q4 + 1];
            y0[4 * q4 + 2] -= a4.z * dm0 * im0[4 * q4 + 2];
            y0[4 * q4 + 3] -= a4.w * dm0 * im0[4 * q4 + 3];
            y1[4 * q4 + 0] -= a4.x * dm1 * im1[4 * q4 + 0];
            y1[4 * q4 + 1] -= a4.y * dm1 * im1[4 * q4 + 1];
            y1[4 * q4 + 2] -= a4.z * dm1 * im1[4 * q4 + 2];
            y1[4 * q4 + 3] -= a4.w * dm1 * im1[4 * q4 + 3];
          }
        }
      }
      __syncthreads();
    }
  }

  // ---------------- pass 2: acc += ad * (d * sum_j sc_j * dot32_j)
  if (producer) {
    // Feeding thread pt stages half a stage row of weights (one 16-byte piece of qs: 16 low
    // nibbles for sub-block 2g, 16 high nibbles for 2g + 1) and half a stage row of activations
    // (32 bytes); once per super-block 128 of them the rows' scales and d, the other 128 the
    // tokens' ad.
    const uint32_t pt = tid - 512u;
    const uint32_t prow = pt >> 1, phalf = pt & 1u;
    const uint32_t wro = row_off(r0 + prow) + (QS_PIECE0 + phalf) * 1024u;          // + sb_off + 2048 g
    const uint32_t qho = row_off(r0 + prow) + (1u + phalf) * 1024u;                 // Q5_K: the thread's 16 bytes of qh
    const uint32_t xro = min(t0 + prow, p.n_tokens - 1u) * p.in_dim + 32u * phalf;  // + 256 s + 64 g
    const uint32_t hro = row_off(r0 + (pt & 127u));
    const uint32_t aro = min(t0 + (pt & 127u), p.n_tokens - 1u) * p.nsb;
    // the ring of stages in flight, slot = stage % 4 = g (named registers: an array handed to a
    // function by reference ends up in scratch memory)
    uint4 wq0, wq1, wq2, wq3, xa0_, xa1_, xa2_, xa3_, xb0_, xb1_, xb2_, xb3_;
    uint4 hdr = make_uint4(0, 0, 0, 0);
    uint4 qhn = make_uint4(0, 0, 0, 0), qhc = make_uint4(0, 0, 0, 0);   // Q5_K: qh of the next / the stored super-block
    float adn = 0.0f;
#define GI_LOAD(S, G, K)                                                                          \
  do {                                                                                            \
    const uint32_t s_ = min((uint32_t)(S), p.nsb - 1u); /* past the end: loaded again, never used */ \
    wq##K = *(const uint4 *)(p.wt + (wro + sb_off(s_) + 2048u * (G)));                            \
    const uint4 *xp_ = (const uint4 *)(p.xq + (xro + 256u * s_ + 64u * (G)));                     \
    xa##K##_ = xp_[0];                                                                            \
    xb##K##_ = xp_[1];                                                                            \
    if ((G) == 0u) {                                                                              \
      if (pt < 128u) hdr = *(const uint4 *)(p.wt + (hro + sb_off(s_)));                           \
      else adn = p.ad[aro + s_];                                                                  \
      if constexpr (Q5) qhn = *(const uint4 *)(p.wt + (qho + sb_off(s_)));                        \
    }                                                                                             \
  } while (0)
  // The nibbles are unsigned weights 0..15 (the minimum is a term of its own): int8 as they are;
  // Q5_K puts bit 2g (2g + 1) of the qh byte on top of the low (high) nibble
#define GI_STORE(S, G, BUF, K)                                                                    \
  do {                                                                                            \
    if constexpr (Q5) { if ((G) == 0u) qhc = qhn; }                                               \
    uint8_t *wr_ = &w_l[BUF][prow * GI_ROW + 16u * phalf];                                        \
    uint4 lo_ = make_uint4(wq##K.x & 0x0F0F0F0Fu, wq##K.y & 0x0F0F0F0Fu, wq##K.z & 0x0F0F0F0Fu,   \
                           wq##K.w & 0x0F0F0F0Fu);                                                \
    uint4 hi_ = make_uint4((wq##K.x >> 4) & 0x0F0F0F0Fu, (wq##K.y >> 4) & 0x0F0F0F0Fu,            \
                           (wq##K.z >> 4) & 0x0F0F0F0Fu, (wq##K.w >> 4) & 0x0F0F0F0Fu);           \
    if constexpr (Q5) {                                                                           \
      lo_.x |= ((qhc.x >> (2u * (G))) & 0x01010101u) << 4;                                        \
      lo_.y |= ((qhc.y >> (2u * (G))) & 0x01010101u) << 4;                                        \
      lo_.z |= ((qhc.z >> (2u * (G))) & 0x01010101u) << 4;                                        \
      lo_.w |= ((qhc.w >> (2u * (G))) & 0x01010101u) << 4;                                        \
      hi_.x |= ((qhc.x >> (2u * (G) + 1u)) & 0x01010101u) << 4;                                   \
      hi_.y |= ((qhc.y >> (2u * (G) + 1u)) & 0x01010101u) << 4;                                   \
      hi_.z |= ((qhc.z >> (2u * (G) + 1u)) & 0x01010101u) << 4;                                   \
      hi_.w |= ((qhc.w >> (2u * (G) + 1u)) & 0x01010101u) << 4;                                   \
    }                                                                                             \
    *(uint4 *)wr_ = lo_;                                                                          \
    *(uint4 *)(wr_ + 32u) = hi_;                                                                  \
    uint8_t *xr_ = &x_l[BUF][prow * GI_ROW + 32u * phalf];                                        \
    *(uint4 *)xr_ = xa##K##_;                                                                     \
    *(uint4 *)(xr_ + 16u) = xb##K##_;                                                             \
    if ((G) == 0u) {                                                                              \
      if (pt < 128u) {                                                                            \
        uint32_t sca_, scb_;                                                                      \
        q4k_scales(hdr, sca_, scb_);                                                              \
        sc_l[(S) & 1u][pt] = make_uint2(sca_, scb_);                                              \
        d_l[(S) & 1u][pt] = gm_f16_bits_to_f32(hdr.x & 0xFFFFu);                                  \
      } else {                                                                                    \
        ad_l[(S) & 1u][pt - 128u] = adn;                                                          \
      }                                                                                           \
    }                                                                                             \
  } while (0)
    GI_LOAD(0u, 0u, 0);
    GI_LOAD(0u, 1u, 1);
    GI_LOAD(0u, 2u, 2);
    GI_STORE(0u, 0u, 0u, 0);
    GI_LOAD(0u, 3u, 3);
    __syncthreads();
    // During stage n = 4 s + g (in LDS buffer g % 2): stage n + 1 goes to the other buffer (it
    // arrived long ago), stage n + 4 is requested into the slot stage n left
    for (uint32_t s = 0; s < p.nsb; s++) {
      GI_STORE(s, 1u, 1u, 1);
      GI_LOAD(s + 1u, 0u, 0);
      __syncthreads();
      GI_STORE(s, 2u, 0u, 2);
      GI_LOAD(s + 1u, 1u, 1);
      __syncthreads();
      GI_STORE(s, 3u, 1u, 3);
      GI_LOAD(s + 1u, 2u, 2);
      __syncthreads();
      if (s + 1u < p.nsb) GI_STORE(s + 1u, 0u, 0u, 0);
      GI_LOAD(s + 1u, 3u, 3);
      __syncthreads();
    }
#undef GI_LOAD
#undef GI_STORE
  } else {
    __syncthreads();
    int16v i0, i1;   // isum of the running super-block
    const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const uint32_t xrow = (tw + l32) * GI_ROW + 16u * lh;
    const uint32_t wrow0 = (64u * rh + l32) * GI_ROW + 16u * lh, wrow1 = wrow0 + 32u * GI_ROW;
    for (uint32_t s = 0; s < p.nsb; s++) {
      const uint2 scw0 = sc_l[s & 1u][64u * rh + l32], scw1 = sc_l[s & 1u][64u * rh + 32u + l32];
#pragma unroll
      for (uint32_t g = 0; g < 4u; g++) {
        const uint32_t buf = g & 1u;
        // both sub-blocks' matrix instructions first, then their multiply-adds: four results in
        // flight keep the matrix pipe busy under the vector work
        const uint32_t ja = 2u * g, jb = 2u * g + 1u;
        const int sc0a = (int)(((ja < 4u ? scw0.x : scw0.y) >> (8u * (ja & 3u))) & 0xFFu);
        const int sc1a = (int)(((ja < 4u ? scw1.x : scw1.y) >> (8u * (ja & 3u))) & 0xFFu);
        const int sc0b = (int)(((jb < 4u ? scw0.x : scw0.y) >> (8u * (jb & 3u))) & 0xFFu);
        const int sc1b = (int)(((jb < 4u ? scw1.x : scw1.y) >> (8u * (jb & 3u))) & 0xFFu);
        const int4v xa_a = *(const int4v *)&x_l[buf][xrow];
        const int4v wb0a = *(const int4v *)&w_l[buf][wrow0];
        const int4v wb1a = *(const int4v *)&w_l[buf][wrow1];
        const int4v xa_b = *(const int4v *)&x_l[buf][xrow + 32u];
        const int4v wb0b = *(const int4v *)&w_l[buf][wrow0 + 32u];
        const int4v wb1b = *(const int4v *)&w_l[buf][wrow1 + 32u];
        const int16v p0a = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_a, wb0a, zi, 0, 0, 0);
        const int16v p1a = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_a, wb1a, zi, 0, 0, 0);
        const int16v p0b = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_b, wb0b, zi, 0, 0, 0);
        const int16v p1b = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_b, wb1b, zi, 0, 0, 0);
        if (g == 0u) {   // the super-block starts fresh sums
#pragma unroll
          for (int r = 0; r < 16; r++) i0[r] = __mul24(p0a[r], sc0a);
#pragma unroll
          for (int r = 0; r < 16; r++) i1[r] = __mul24(p1a[r], sc1a);
        } else {
#pragma unroll
          for (int r = 0; r < 16; r++) i0[r] = __mul24(p0a[r], sc0a) + i0[r];
#pragma unroll
          for (int r = 0; r < 16; r++) i1[r] = __mul24(p1a[r], sc1a) + i1[r];
        }
#pragma unroll
        for (int r = 0; r < 16; r++) i0[r] = __mul24(p0b[r], sc0b) + i0[r];
#pragma unroll
        for (int r = 0; r < 16; r++) i1[r] = __mul24(p1b[r], sc1b) + i1[r];
        if (g == 3u) {
          const float d0 = d_l[s & 1u][64u * rh + l32], d1 = d_l[s & 1u][64u * rh + 32u + l32];
          const float *adp = &ad_l[s & 1u][tw + 4u * lh];
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++) {
            const float4 a4 = *(const float4 *)(adp + 8 * q4);
            y0[4 * q4 + 0] += a4.x * (d0 * (float)i0[4 * q4 + 0]);
            y0[4 * q4 + 1] += a4.y * (d0 * (float)i0[4 * q4 + 1]);
            y0[4 * q4 + 2] += a4.z * (d0 * (float)i0[4 * q4 + 2]);
            y0[4 * q4 + 3] += a4.w * (d0 * (float)i0[4 * q4 + 3]);
            y1[4 * q4 + 0] += a4.x * (d1 * (float)i1[4 * q4 + 0]);
            y1[4 * q4 + 1] += a4.y * (d1 * (float)i1[4 * q4 + 1]);
            y1[4 * q4 + 2] += a4.z * (d1 * (float)i1[4 * q4 + 2]);
            y1[4 * q4 + 3] += a4.w * (d1 * (float)i1[4 * q4 + 3]);
          }
        }
        __syncthreads();
      }
    }
    const uint32_t row0 = r0 + 64u * rh + l32;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const uint32_t t = t0 + tw + 8u * (r >> 2) + 4u * lh + (r & 3);
      if (t < p.n_tokens) {
        if (row0 < p.out_dim) p.y[(size_t)t * p.out_dim + row0] = y0[r];
        if (row0 + 32u < p.out_dim) p.y[(size_t)t * p.out_dim + row0 + 32u] = y1[r];
      }
    }
  }
}

__global__ __launch_bounds__(768) void ogm_gemm_q4k_i8_kernel(GemmParams p) { gemm_i8_body<false>(p); }
__global__ __launch_bounds__(768) void ogm_gemm_q5k_i8_kernel(GemmParams p) { gemm_i8_body<true>(p); }

// ------------------------------------------------------------------------------------------
// Q6_K on the int8 matrix cores (gemm_k_q6_k, vecdot.rs:2352-2398): scales per 16 weights would
// mean one multiply-add per output for every 16 products, so here the feeding waves fold the
// scale into the weight, w' = sc_g * (q - 32) in [-4064, 4096], and split it into two int8
// planes, w' = 256 h + l with l in [-128, 127] and h in [-16, 16].  The multiplying waves then run
// two plain chains of v_mfma_i32_32x32x32_i8 over the whole super-block, accumulating in the
// instruction itself, and isum = 256 H + L in 32-bit integers: exact, one `as f32` per super-block.  Same tile, waves and orientation as gemm_i8_body.

typedef short short2v __attribute__((ext_vector_type(2)));

struct GemmI8pParams {
  const uint8_t *wt;      // tile-planar weights
  const int8_t *xq;       // [T][in_dim] int8 activations
  const float *ad;        // [T][nsb]
  const _Float16 *bs16;   // Q4_K / Q5_K: the quantizer's sums per 32 as (bsum / 64, bsum % 64) in f16
  float *y;               // [T][out_dim]
  uint32_t in_dim, out_dim, n_tokens, nsb;
  uint32_t c_shift, r_shift, nct;
  uint32_t n_extra;
  const uint8_t *extra_wt[OGM_GEMM_MAX_MATS - 1];
  float *extra_y[OGM_GEMM_MAX_MATS - 1];
  uint32_t extra_out_dim[OGM_GEMM_MAX_MATS - 1];
  // PRE kernels: the planes built once per matrix by ogm_gemm_build_planes_kernel
  const uint8_t *planes;
  const uint8_t *extra_planes[OGM_GEMM_MAX_MATS - 1];
};

// The planes of a matrix, built once and kept beside its tile-planar bytes (2 bytes per weight; 1
// for Q3_K): what the feeding waves of the kernels below otherwise recompute on every call.  Row
// blocks of 64 rows; for row block rb, super-block s, stage g (64 weights), group t (16 weights):
// 64 rows x 16 bytes of plane h, then (two-plane types) 64 rows x 16 bytes of plane l -- one
// feeding wave's share of a stage is one contiguous run of 1 or 2 KiB.
__host__ __device__ inline size_t gp_plane_offset(uint32_t rb, uint32_t nsb, uint32_t s, uint32_t g, uint32_t t16,
                                                  uint32_t npl) {
  return ((((size_t)rb * nsb + s) * 4u + g) * 4u + t16) * (npl * 1024u);
}

// ROWS = 128: eight multiplying waves (32 rows x 64 tokens each) and eight feeding ones; ROWS = 64:
// four and four, and half the LDS: twice as many workgroups, which fills the chip when a launch has
// few row tiles.  As many feeding as multiplying waves, because a stage's unpacking, behind the
// latency of its loads, takes a feeding wave about as long as eight matrix instructions and their
// operand reads take a multiplying one (with half as many feeding waves the multiplying ones sat
// idle for more than half of every stage).
#define GP_Q6K 0
#define GP_Q3K 1
#define GP_Q4K 2
#define GP_Q5K 3
// Ablation switches for timing experiments (scratch builds define them; the library never does):
// each removes one ingredient of the kernel below, results become wrong, and the time that goes
// away is what that ingredient costs.
#ifndef GP_ABL_NOMFMA
#define GP_ABL_NOMFMA 0
#endif
#ifndef GP_ABL_NOLDSREAD
#define GP_ABL_NOLDSREAD 0
#endif
#ifndef GP_ABL_NOFEED
#define GP_ABL_NOFEED 0
#endif
#ifndef GP_ABL_NOBARRIER
#define GP_ABL_NOBARRIER 0
#endif
#ifndef GP_ABL_NOPASS1
#define GP_ABL_NOPASS1 0
#endif
#ifndef GP_ABL_NOEPI
#define GP_ABL_NOEPI 0
#endif
#define GP_SYNC() do { if (!GP_ABL_NOBARRIER) __syncthreads(); } while (0)

template <uint32_t ROWS, int KIND, bool PRE = false>
__device__ __forceinline__ void gemm_q6k_i8_body(GemmI8pParams p) {
  constexpr bool Q3 = KIND == GP_Q3K, Q45 = KIND == GP_Q4K || KIND == GP_Q5K, Q5 = KIND == GP_Q5K;
  constexpr uint32_t NC = ROWS / 16u;                // multiplying waves
  constexpr uint32_t WT = ROWS * GI_ROW;             // bytes of a plane's stage
  // Q6_K: 64 units of 210 bytes are 13 pieces of 1 KiB, then 64 two-byte tails; Q3_K: 7 pieces;
  // Q4_K: 9 (header, qs); Q5_K: 11 (header, qh, qs)
  constexpr uint32_t TILE_BYTES = Q3 ? 7168u : KIND == GP_Q4K ? 9216u : Q5 ? 11264u : 13440u;
  constexpr uint32_t QS_PIECE0 = Q5 ? 3u : 1u;       // Q4_K / Q5_K: first piece of qs
  constexpr uint32_t NPL = Q3 ? 1u : 2u;             // operand planes
  // three stages of 64 weights in LDS: one being multiplied, the next being read into registers
  // behind it, the third being written by the feeding waves
  extern __shared__ __align__(16) uint8_t lds[];
  uint8_t *wh_l = lds;                                      // [3][ROWS][64 of 80]: plane h
  uint8_t *wl_l = lds + 3u * WT;                            // plane l (Q6_K)
  uint8_t *x_l = lds + 3u * NPL * WT;                       // [3][128 tokens][64 of 80]: activations
  float *d_l = (float *)(lds + 3u * NPL * WT + 3u * GI_WTILE);   // [2][ROWS] the rows' d
  float *ad_l = d_l + 2u * ROWS;                            // [2][128] the tokens' activation scale

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const bool producer = wave >= NC;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  // a multiplying wave: 32 rows (block rq) x 64 tokens (half th): one weight operand per plane feeds
  // two matrix instructions, which keeps the LDS reads at four per 32 k
  const uint32_t rq = wave % (ROWS / 32u), th = (wave / (ROWS / 32u)) & 1u;
  uint32_t row_tile = blockIdx.y;
#pragma unroll
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {   // the matrix this row tile belongs to
    const uint32_t tiles = (p.out_dim + ROWS - 1u) / ROWS;
    if (m < p.n_extra && row_tile >= tiles) {
      row_tile -= tiles;
      p.wt = p.extra_wt[m];
      p.y = p.extra_y[m];
      p.out_dim = p.extra_out_dim[m];
      p.planes = p.extra_planes[m];
    } else {
      break;
    }
  }
  const uint32_t t0 = blockIdx.x * 128u, r0 = row_tile * ROWS;
  const uint32_t tw = 64u * th;   // the wave's first token within the workgroup

  auto sb_tile = [&](uint32_t s) -> uint32_t { return (s >> p.c_shift) * TILE_BYTES; };
  auto sb_lane = [&](uint32_t s) -> uint32_t { return (s & ((1u << p.c_shift) - 1u)) << p.r_shift; };

  // y0 / y1 of a multiplying wave: row r0 + 32 rq + l32, tokens t0 + tw + (8 (r / 4) + 4 lh + r % 4) and + 32
  float16v y0, y1;
#pragma unroll
  for (int r = 0; r < 16; r++) y0[r] = y1[r] = 0.0f;

  if constexpr (Q45 && !GP_ABL_NOPASS1) {
    // ---------------- pass 1 of gemm_k_q4_k: acc -= (ad * dmin) * sum_j m_j * bsum_j, all super-blocks
    // first (vecdot.rs:2226-2240), on the f16 matrix cores with tokens as rows: 64 m_j against
    // bsum_j / 64 and m_j against bsum_j % 64 in one K = 16 instruction per 32 x 32 outputs.  The
    // tokens' ad of every super-block go to LDS once; a row's dmin and mins come with its header.
    float *ad_all = ad_l + 256;   // [nsb][128]
    for (uint32_t i = tid; i < 128u * p.nsb; i += blockDim.x) {
      const uint32_t k = i / p.nsb, su = i - k * p.nsb;   // consecutive threads: consecutive super-blocks of a token
      ad_all[su * 128u + k] = p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + su];
    }
    __syncthreads();
    if (!producer) {
      float16v zero;
#pragma unroll
      for (int r = 0; r < 16; r++) zero[r] = 0.0f;
      uint32_t ro0;
      {
        const uint32_t row = min(r0 + 32u * rq + l32, p.out_dim - 1u);
        ro0 = (row >> p.r_shift) * p.nct * TILE_BYTES + (row & ((1u << p.r_shift) - 1u)) * 16u;
      }
      const uint32_t tk0 = min(t0 + tw + l32, p.n_tokens - 1u) * p.nsb;
      const uint32_t tk1 = min(t0 + tw + 32u + l32, p.n_tokens - 1u) * p.nsb;
      const float side_scale = lh ? 1.0f : 64.0f;
      for (uint32_t su = 0; su < p.nsb; su++) {
        const uint4 hd0 = *(const uint4 *)(p.wt + (ro0 + sb_tile(su) + sb_lane(su) * 16u));
        const half8 b20 = *(const half8 *)(p.bs16 + ((tk0 + su) * 16u + 8u * lh));
        const half8 b21 = *(const half8 *)(p.bs16 + ((tk1 + su) * 16u + 8u * lh));
        uint32_t mna, mnb;
        q4k_mins(hd0, mna, mnb);
        const half8 a1 = side_operand(mna, mnb, side_scale);
        const float dm = gm_f16_bits_to_f32(hd0.x >> 16);
        const float16v im0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b20, a1, zero, 0, 0, 0);
        const float16v im1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b21, a1, zero, 0, 0, 0);
        const float *adp = &ad_all[su * 128u + tw + 4u * lh];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const float4 a4 = *(const float4 *)(adp + 8 * q4), b4 = *(const float4 *)(adp + 32 + 8 * q4);
          const float a4v[4] = {a4.x, a4.y, a4.z, a4.w}, b4v[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
          for (int e = 0; e < 4; e++) {
            y0[4 * q4 + e] -= a4v[e] * dm * im0[4 * q4 + e];
            y1[4 * q4 + e] -= b4v[e] * dm * im1[4 * q4 + e];
          }
        }
      }
    }
  }

  // ---------------- the products: acc += ad * (d * isum) per super-block
  if (producer) {
    // Feeding thread pt stages one group of 16 weights per stage: one ql piece, one qh piece, one
    // scale.  A wave has one group index and 64 consecutive rows: its loads are 1 KiB runs and its
    // LDS rows are 80 bytes apart, which spreads over all banks.  And 16 bytes of a token's
    // activations (32 with half as many feeding threads).  Once per super-block the rows' d and the
    // tokens' ad.
    const uint32_t pt = tid - 64u * NC;
    const uint32_t t16 = __builtin_amdgcn_readfirstlane(pt / ROWS), prw = pt % ROWS;
    uint32_t uo, dto;   // the row's 16-byte pieces and its two-byte tail (d)
    {
      const uint32_t row = min(r0 + prw, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
      const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
      uo = rb * p.nct * TILE_BYTES + r * 16u;
      dto = rb * p.nct * TILE_BYTES + 13u * 1024u + r * 2u;
    }
    // PRE: this thread's 16 bytes of each plane, per (super-block, stage): row block of 64 rows
    // (clamped to the matrix's last one; such rows are never stored), its row within it
    [[maybe_unused]] const uint32_t prb = min((r0 + prw) >> 6, (p.out_dim - 1u) >> 6);
    [[maybe_unused]] const uint8_t *pl_base = PRE ? p.planes + (prw & 63u) * 16u : nullptr;
    constexpr uint32_t XB = ROWS == 128u ? 16u : 32u;   // bytes of a token's stage per feeding thread
    const uint32_t xrow_ = pt / (64u / XB), xpart = pt % (64u / XB);
    const uint32_t xro = min(t0 + xrow_, p.n_tokens - 1u) * p.in_dim + XB * xpart;   // + 256 s + 64 g
    const bool has_d = pt < ROWS, has_ad = pt >= ROWS && pt < ROWS + 128u;
    const uint32_t ad_tok = pt - ROWS;
    const uint32_t aro = min(t0 + (ad_tok & 127u), p.n_tokens - 1u) * p.nsb;
    // the ring of stages in flight, slot = stage % 4 = g, in named registers
    uint4 qla0, qla1, qla2, qla3, qha0, qha1, qha2, qha3;
    uint4 xa0_, xa1_, xa2_, xa3_;
    uint4 xb0_, xb1_, xb2_, xb3_;   // ROWS = 64: the thread's other 16 bytes
    uint4 scxa = make_uint4(0, 0, 0, 0);      // the 16 scales of the row, next super-block
    uint32_t sca[4] = {0, 0, 0, 0};           // ... of the super-block being stored
    uint4 hmxn = make_uint4(0, 0, 0, 0);      // Q3_K: the group's 16 bytes of hmask, next super-block
    uint32_t hmw[4] = {0, 0, 0, 0};           // ... of the super-block being stored
    uint32_t d16 = 0;
    float adn = 0.0f;
#define GP_LOAD(S, G, K)                                                                          \
  do {                                                                                            \
    if (GP_ABL_NOFEED) break;                                                                     \
    const uint32_t s_ = min((uint32_t)(S), p.nsb - 1u); /* past the end: loaded again, never used */ \
    const uint32_t so_ = sb_tile(s_) + sb_lane(s_) * 16u, h_ = (G) >> 1;                          \
    if constexpr (PRE) {                                                                          \
      const uint8_t *pp_ = pl_base + gp_plane_offset(prb, p.nsb, s_, (G), t16, NPL);              \
      qla##K = *(const uint4 *)pp_;                                                               \
      if constexpr (!Q3) qha##K = *(const uint4 *)(pp_ + 1024u);                                  \
    } else if constexpr (Q3) {                                                                    \
      /* pieces: hmask 0..1, qs 2..5, then scales[12] | d | two bytes of padding */               \
      qla##K = *(const uint4 *)(p.wt + (uo + so_ + (2u + 2u * h_ + (t16 & 1u)) * 1024u));         \
    } else if constexpr (Q45) {                                                                   \
      /* 32 bytes of qs per pair of sub-blocks: low nibbles 2 G, high nibbles 2 G + 1 */          \
      qla##K = *(const uint4 *)(p.wt + (uo + so_ + (QS_PIECE0 + 2u * (G) + (t16 & 1u)) * 1024u)); \
    } else {                                                                                      \
      qla##K = *(const uint4 *)(p.wt + (uo + so_ + (4u * h_ + t16) * 1024u));                     \
      qha##K = *(const uint4 *)(p.wt + (uo + so_ + (8u + 2u * h_ + (t16 & 1u)) * 1024u));         \
    }                                                                                             \
    const uint4 *xp_ = (const uint4 *)(p.xq + (xro + 256u * s_ + 64u * (G)));                     \
    xa##K##_ = xp_[0];                                                                            \
    if constexpr (ROWS == 64u) xb##K##_ = xp_[1];                                                 \
    if ((G) == 0u) {                                                                              \
      if constexpr (Q3) {                                                                         \
        if (!PRE || has_d) scxa = *(const uint4 *)(p.wt + (uo + so_ + 6u * 1024u));               \
        if constexpr (!PRE) hmxn = *(const uint4 *)(p.wt + (uo + so_ + (t16 & 1u) * 1024u));      \
      } else if constexpr (Q45) {                                                                 \
        if (!PRE || has_d) scxa = *(const uint4 *)(p.wt + (uo + so_));   /* d | dmin, then the 12 scale bytes */ \
        if constexpr (Q5 && !PRE) hmxn = *(const uint4 *)(p.wt + (uo + so_ + (1u + (t16 & 1u)) * 1024u)); \
      } else {                                                                                    \
        if constexpr (!PRE) scxa = *(const uint4 *)(p.wt + (uo + so_ + 12u * 1024u));             \
        if (has_d) d16 = *(const uint16_t *)(p.wt + (dto + sb_tile(s_) + sb_lane(s_) * 2u));      \
      }                                                                                           \
      if (has_ad) adn = p.ad[aro + s_];                                                           \
    }                                                                                             \
  } while (0)
  // sixteen 6-bit weights of one group -> the two int8 planes of sc * (q - 32), into the group's
  // 16 bytes of the row in each plane's tile.  u = sc * q + (128 - 32 sc) is a 16-bit lane whose
  // high byte is h and whose low byte, top bit flipped and read as int8, is l = (u & 255) - 128.
#define GP_GROUP(QL, QH, SCW, G, BUF, ROWOFF, T16)                                                  \
  do {                                                                                            \
    const int sc_ = (int)(int8_t)(((SCW)[(G)] >> (8u * (T16))) & 0xFFu);                          \
    const short2v sc2_ = {(short)sc_, (short)sc_};                                                \
    const short2v c2_ = {(short)(128 - 32 * sc_), (short)(128 - 32 * sc_)};                       \
    const uint32_t rr_ = 2u * ((G) & 1u) + ((T16) >> 1);      /* run of 32 inside the half block */ \
    const uint32_t qlw_[4] = {QL.x, QL.y, QL.z, QL.w}, qhw_[4] = {QH.x, QH.y, QH.z, QH.w};        \
    uint32_t ph_[4], pl_[4];                                                                      \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      const uint32_t nib_ = (((G) & 1u) ? (qlw_[w_] >> 4) : qlw_[w_]) & 0x0F0F0F0Fu;              \
      const uint32_t v_ = nib_ | ((((qhw_[w_] >> (2u * rr_)) << 4)) & 0x30303030u);               \
      union { uint32_t u; short2v s; } e_, f_;                                                    \
      e_.u = __builtin_amdgcn_perm(0u, v_, 0x0c010c00u);   /* (b0, b1) as 16-bit lanes */         \
      f_.u = __builtin_amdgcn_perm(0u, v_, 0x0c030c02u);   /* (b2, b3) */                         \
      e_.s = e_.s * sc2_ + c2_;                                                                   \
      f_.s = f_.s * sc2_ + c2_;                                                                   \
      ph_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x07050301u);                /* high bytes */   \
      pl_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x06040200u) ^ 0x80808080u;  /* low bytes */    \
    }                                                                                             \
    *(uint4 *)&wh_l[(BUF) + (ROWOFF) * GI_ROW + 16u * (T16)] = make_uint4(ph_[0], ph_[1], ph_[2], ph_[3]); \
    *(uint4 *)&wl_l[(BUF) + (ROWOFF) * GI_ROW + 16u * (T16)] = make_uint4(pl_[0], pl_[1], pl_[2], pl_[3]); \
  } while (0)
  // Q3_K (gemm_k_q6_k over unpacked rows, vecdot.rs:2100-2117): sixteen 3-bit weights, q - 4 in
  // [-4, 3], times the group's scale sc - 32 in [-32, 31] (quant.rs:883-897: low four bits in a
  // nibble of byte i % 8, two high bits at bit 2 (i / 4) of byte 8 + i % 4, i = 4 G + t16).  The
  // product reaches +128, its negative fits int8: one plane of sc * (4 - q), and isum = -H.
#define GP_GROUP3(QL, G, BUF, ROWOFF, T16)                                                        \
  do {                                                                                            \
    const uint32_t lw_ = ((G) & 1u) ? sca[1] : sca[0];                                            \
    const uint32_t low_ = ((lw_ >> (8u * (T16))) >> ((G) >= 2u ? 4u : 0u)) & 0xFu;                \
    const uint32_t high_ = ((sca[2] >> (8u * (T16))) >> (2u * (G))) & 3u;                         \
    const int sc_ = (int)(low_ | (high_ << 4)) - 32;                                              \
    const short2v msc2_ = {(short)(-sc_), (short)(-sc_)};                                         \
    const short2v c2_ = {(short)(4 * sc_), (short)(4 * sc_)};                                     \
    const uint32_t rr_ = 2u * ((G) & 1u) + ((T16) >> 1);      /* run of 32 inside the half block */ \
    const uint32_t qlw_[4] = {QL.x, QL.y, QL.z, QL.w};                                            \
    uint32_t ph_[4];                                                                              \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      /* run p = 2 G + t16 / 2 of 32: two bits at 2 (p % 4), third bit = bit p of hmask */        \
      const uint32_t v_ = ((qlw_[w_] >> (2u * rr_)) & 0x03030303u) |                              \
                          (((hmw[w_] >> (2u * (G) + ((T16) >> 1))) & 0x01010101u) << 2);          \
      union { uint32_t u; short2v s; } e_, f_;                                                    \
      e_.u = __builtin_amdgcn_perm(0u, v_, 0x0c010c00u);   /* (b0, b1) as 16-bit lanes */         \
      f_.u = __builtin_amdgcn_perm(0u, v_, 0x0c030c02u);   /* (b2, b3) */                         \
      e_.s = e_.s * msc2_ + c2_;                                                                  \
      f_.s = f_.s * msc2_ + c2_;                                                                  \
      ph_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x06040200u);   /* the lanes' low bytes */      \
    }                                                                                             \
    *(uint4 *)&wh_l[(BUF) + (ROWOFF) * GI_ROW + 16u * (T16)] = make_uint4(ph_[0], ph_[1], ph_[2], ph_[3]); \
  } while (0)
  // Q4_K / Q5_K (KKind::Q4K rows, vecdot.rs:2064-2088): sixteen weights 0..15 (Q5_K: 0..31 with
  // bit j of qh on top) of sub-block j = 2 G + T16 / 2, times its scale 0..63 (get_scale_min_k4,
  // quant.rs:653-662): u = sc * q + 128 <= 2081, planes as for Q6_K.
#define GP_GROUP45(QL, G, BUF, ROWOFF, T16)                                                       \
  do {                                                                                            \
    uint32_t sc4a_, sc4b_;   /* the scales of sub-blocks 0..3 and 4..7, a byte each */            \
    {                                                                                             \
      const uint4 hd_ = make_uint4(sca[0], sca[1], sca[2], sca[3]);                               \
      q4k_scales(hd_, sc4a_, sc4b_);                                                              \
    }                                                                                             \
    const uint32_t hi_ = (T16) >> 1, j_ = 2u * (G) + hi_;                                         \
    const uint32_t scw_ = (G) < 2u ? sc4a_ : sc4b_;                                               \
    const int sc_ = (int)((scw_ >> (8u * (j_ & 3u))) & 0xFFu);                                    \
    const short2v sc2_ = {(short)sc_, (short)sc_};                                                \
    const short2v c2_ = {128, 128};                                                               \
    const uint32_t qlw_[4] = {QL.x, QL.y, QL.z, QL.w};                                            \
    uint32_t ph_[4], pl_[4];                                                                      \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      uint32_t v_ = (hi_ ? (qlw_[w_] >> 4) : qlw_[w_]) & 0x0F0F0F0Fu;                             \
      if constexpr (Q5) v_ |= ((hmw[w_] >> j_) & 0x01010101u) << 4;                               \
      union { uint32_t u; short2v s; } e_, f_;                                                    \
      e_.u = __builtin_amdgcn_perm(0u, v_, 0x0c010c00u);   /* (b0, b1) as 16-bit lanes */         \
      f_.u = __builtin_amdgcn_perm(0u, v_, 0x0c030c02u);   /* (b2, b3) */                         \
      e_.s = e_.s * sc2_ + c2_;                                                                   \
      f_.s = f_.s * sc2_ + c2_;                                                                   \
      ph_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x07050301u);                /* high bytes */   \
      pl_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x06040200u) ^ 0x80808080u;  /* low bytes */    \
    }                                                                                             \
    *(uint4 *)&wh_l[(BUF) + (ROWOFF) * GI_ROW + 16u * (T16)] = make_uint4(ph_[0], ph_[1], ph_[2], ph_[3]); \
    *(uint4 *)&wl_l[(BUF) + (ROWOFF) * GI_ROW + 16u * (T16)] = make_uint4(pl_[0], pl_[1], pl_[2], pl_[3]); \
  } while (0)
#define GP_STORE(S, G, K)                                                                         \
  do {                                                                                            \
    if (GP_ABL_NOFEED) break;                                                                     \
    if ((G) == 0u) {                                                                              \
      sca[0] = scxa.x; sca[1] = scxa.y; sca[2] = scxa.z; sca[3] = scxa.w;                         \
      if constexpr (Q3) {                                                                         \
        hmw[0] = hmxn.x; hmw[1] = hmxn.y; hmw[2] = hmxn.z; hmw[3] = hmxn.w;                       \
        if (has_d) d_l[ROWS * ((S) & 1u) + pt] = gm_f16_bits_to_f32(scxa.w & 0xFFFFu);            \
      } else if constexpr (Q45) {                                                                 \
        if constexpr (Q5) { hmw[0] = hmxn.x; hmw[1] = hmxn.y; hmw[2] = hmxn.z; hmw[3] = hmxn.w; } \
        if (has_d) d_l[ROWS * ((S) & 1u) + pt] = gm_f16_bits_to_f32(scxa.x & 0xFFFFu);            \
      } else {                                                                                    \
        if (has_d) d_l[ROWS * ((S) & 1u) + pt] = gm_f16_bits_to_f32(d16);                         \
      }                                                                                           \
      if (has_ad) ad_l[128u * ((S) & 1u) + ad_tok] = adn;                                         \
    }                                                                                             \
    if constexpr (PRE) {                                                                          \
      *(uint4 *)&wh_l[pw + prw * GI_ROW + 16u * t16] = qla##K;                                    \
      if constexpr (!Q3) *(uint4 *)&wl_l[pw + prw * GI_ROW + 16u * t16] = qha##K;                 \
    } else if constexpr (Q3) GP_GROUP3(qla##K, G, pw, prw, t16);                                  \
    else if constexpr (Q45) GP_GROUP45(qla##K, G, pw, prw, t16);                                  \
    else GP_GROUP(qla##K, qha##K, sca, G, pw, prw, t16);                                          \
    uint8_t *xr_ = &x_l[px + xrow_ * GI_ROW + XB * xpart];                                        \
    *(uint4 *)xr_ = xa##K##_;                                                                     \
    if constexpr (ROWS == 64u) *(uint4 *)(xr_ + 16u) = xb##K##_;                                  \
    /* stages go round the three buffers */                                                       \
    pw = pw == 2u * WT ? 0u : pw + WT;                                                            \
    px = px == 2u * GI_WTILE ? 0u : px + GI_WTILE;                                                \
  } while (0)
    uint32_t pw = 0, px = 0;   // byte offsets of the stage being stored: weight planes, activations
    GP_LOAD(0u, 0u, 0);
    GP_LOAD(0u, 1u, 1);
    GP_LOAD(0u, 2u, 2);
    GP_STORE(0u, 0u, 0);
    GP_LOAD(0u, 3u, 3);
    GP_STORE(0u, 1u, 1);
    GP_LOAD(1u, 0u, 0);
    GP_SYNC();
    // each period stores the stage two ahead of the one being multiplied and loads the one five ahead
    for (uint32_t s = 0; s < p.nsb; s++) {
      GP_STORE(s, 2u, 2);
      GP_LOAD(s + 1u, 1u, 1);
      GP_SYNC();
      GP_STORE(s, 3u, 3);
      GP_LOAD(s + 1u, 2u, 2);
      GP_SYNC();
      if (s + 1u < p.nsb) GP_STORE(s + 1u, 0u, 0);
      GP_LOAD(s + 1u, 3u, 3);
      GP_SYNC();
      if (s + 1u < p.nsb) GP_STORE(s + 1u, 1u, 1);
      GP_LOAD(s + 2u, 0u, 0);
      GP_SYNC();
    }
#undef GP_LOAD
#undef GP_GROUP
#undef GP_GROUP3
#undef GP_GROUP45
#undef GP_STORE
  } else {
    GP_SYNC();
#if GP_ABL_NOMFMA
#define GP_MFMA(A, B, C, X, Y, Z) ((C) + (A).x + (B).x)   /* keeps the operands alive */
#else
#define GP_MFMA(A, B, C, X, Y, Z) __builtin_amdgcn_mfma_i32_32x32x32_i8(A, B, C, X, Y, Z)
#endif
    int16v h0, h1, l0, l1;   // the two planes' sums of the running super-block
    const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const uint32_t xrow0 = (tw + l32) * GI_ROW + 16u * lh, xrow1 = xrow0 + 32u * GI_ROW;
    const uint32_t wrow = (32u * rq + l32) * GI_ROW + 16u * lh;
    // operands of the stage's first 32 weights (a) and last 32 (b); a of the next stage is read
    // while b multiplies, b while a does
    int4v x0a = {0, 0, 0, 0}, x1a = x0a, wha = x0a, wla = x0a, x0b = x0a, x1b = x0a, whb = x0a, wlb = x0a;
    uint32_t cw = 0, cx = 0;   // byte offsets of the stage's buffers: weight planes, activations
#define GP_READ(SUF, OFFW, OFFX)                              \
  do {                                                        \
    if (GP_ABL_NOLDSREAD) break;                              \
    x0##SUF = *(const int4v *)&x_l[(OFFX) + xrow0];           \
    x1##SUF = *(const int4v *)&x_l[(OFFX) + xrow1];           \
    wh##SUF = *(const int4v *)&wh_l[(OFFW) + wrow];           \
    if constexpr (!Q3) wl##SUF = *(const int4v *)&wl_l[(OFFW) + wrow]; \
  } while (0)
    GP_READ(a, 0u, 0u);
    for (uint32_t s = 0; s < p.nsb; s++) {
#pragma unroll
      for (uint32_t g = 0; g < 4u; g++) {
        const uint32_t nw = cw == 2u * WT ? 0u : cw + WT, nx = cx == 2u * GI_WTILE ? 0u : cx + GI_WTILE;
        GP_READ(b, cw + 32u, cx + 32u);
        if (g == 0u) {   // the super-block starts fresh sums
          h0 = GP_MFMA(x0a, wha, zi, 0, 0, 0);
          h1 = GP_MFMA(x1a, wha, zi, 0, 0, 0);
          if constexpr (!Q3) {
            l0 = GP_MFMA(x0a, wla, zi, 0, 0, 0);
            l1 = GP_MFMA(x1a, wla, zi, 0, 0, 0);
          }
        } else {
          h0 = GP_MFMA(x0a, wha, h0, 0, 0, 0);
          h1 = GP_MFMA(x1a, wha, h1, 0, 0, 0);
          if constexpr (!Q3) {
            l0 = GP_MFMA(x0a, wla, l0, 0, 0, 0);
            l1 = GP_MFMA(x1a, wla, l1, 0, 0, 0);
          }
        }
        GP_READ(a, nw, nx);   // complete since the last barrier; past the last stage: read, never used
        h0 = GP_MFMA(x0b, whb, h0, 0, 0, 0);
        h1 = GP_MFMA(x1b, whb, h1, 0, 0, 0);
        if constexpr (!Q3) {
          l0 = GP_MFMA(x0b, wlb, l0, 0, 0, 0);
          l1 = GP_MFMA(x1b, wlb, l1, 0, 0, 0);
        }
        cw = nw;
        cx = nx;
        if (g == 3u && !GP_ABL_NOEPI) {
          const float d0 = d_l[ROWS * (s & 1u) + 32u * rq + l32];
          const float *adp = &ad_l[128u * (s & 1u) + tw + 4u * lh];
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++) {
            const float4 a4 = *(const float4 *)(adp + 8 * q4), b4 = *(const float4 *)(adp + 32 + 8 * q4);
            const float a4v[4] = {a4.x, a4.y, a4.z, a4.w}, b4v[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const int is0 = Q3 ? -h0[4 * q4 + e] : h0[4 * q4 + e] * 256 + l0[4 * q4 + e];
              const int is1 = Q3 ? -h1[4 * q4 + e] : h1[4 * q4 + e] * 256 + l1[4 * q4 + e];
              y0[4 * q4 + e] += a4v[e] * (d0 * (float)is0);
              y1[4 * q4 + e] += b4v[e] * (d0 * (float)is1);
            }
          }
        }
        GP_SYNC();
      }
    }
#undef GP_READ
#undef GP_MFMA
    const uint32_t row0 = r0 + 32u * rq + l32;
    if (row0 < p.out_dim) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const uint32_t t = t0 + tw + 8u * (r >> 2) + 4u * lh + (r & 3);
        if (t < p.n_tokens) p.y[(size_t)t * p.out_dim + row0] = y0[r];
        if (t + 32u < p.n_tokens) p.y[(size_t)(t + 32u) * p.out_dim + row0] = y1[r];
      }
    }
  }
}

__global__ __launch_bounds__(1024) void ogm_gemm_q6k_i8_kernel(GemmI8pParams p) { gemm_q6k_i8_body<128u, GP_Q6K>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q6k_i8_r64_kernel(GemmI8pParams p) { gemm_q6k_i8_body<64u, GP_Q6K>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_q3k_i8_kernel(GemmI8pParams p) { gemm_q6k_i8_body<128u, GP_Q3K>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q3k_i8_r64_kernel(GemmI8pParams p) { gemm_q6k_i8_body<64u, GP_Q3K>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_q4k_i8p_kernel(GemmI8pParams p) { gemm_q6k_i8_body<128u, GP_Q4K>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q4k_i8p_r64_kernel(GemmI8pParams p) { gemm_q6k_i8_body<64u, GP_Q4K>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_q5k_i8p_kernel(GemmI8pParams p) { gemm_q6k_i8_body<128u, GP_Q5K>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q5k_i8p_r64_kernel(GemmI8pParams p) { gemm_q6k_i8_body<64u, GP_Q5K>(p); }
// the same kernels over planes built beforehand: the feeding waves only copy
__global__ __launch_bounds__(1024) void ogm_gemm_q6k_i8_pre_kernel(GemmI8pParams p) { gemm_q6k_i8_body<128u, GP_Q6K, true>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q6k_i8_pre_r64_kernel(GemmI8pParams p) { gemm_q6k_i8_body<64u, GP_Q6K, true>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_q3k_i8_pre_kernel(GemmI8pParams p) { gemm_q6k_i8_body<128u, GP_Q3K, true>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q3k_i8_pre_r64_kernel(GemmI8pParams p) { gemm_q6k_i8_body<64u, GP_Q3K, true>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_q4k_i8p_pre_kernel(GemmI8pParams p) { gemm_q6k_i8_body<128u, GP_Q4K, true>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q4k_i8p_pre_r64_kernel(GemmI8pParams p) { gemm_q6k_i8_body<64u, GP_Q4K, true>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_q5k_i8p_pre_kernel(GemmI8pParams p) { gemm_q6k_i8_body<128u, GP_Q5K, true>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q5k_i8p_pre_r64_kernel(GemmI8pParams p) { gemm_q6k_i8_body<64u, GP_Q5K, true>(p); }

// Builds a matrix's planes from its tile-planar bytes: thread (t = tid / 64, r = tid % 64) of
// workgroup (4 s + g, rb) turns the sixteen weights 256 s + 64 g + 16 t .. of row 64 rb + r into their
// 16 bytes of each plane -- the arithmetic of the feeding waves above, done once.
//   Q6_K: u = sc_g (q - 32) + 128, sc the int8 scale of the group of 16       (vecdot.rs:2119-2143)
//   Q3_K: one plane, (sc - 32)(4 - q) with the six-bit scale of the group      (vecdot.rs:2100-2117)
//   Q4_K / Q5_K: u = sc_j q + 128, sc the six-bit scale of the sub-block of 32 (vecdot.rs:2036-2088)
// h = u >> 8, l = (u & 255) - 128 as int8: sc * q' = 256 h + l.
struct GemmPlaneBuildParams {
  const uint8_t *wt;
  uint8_t *planes;
  uint32_t out_dim, nsb, c_shift, r_shift, nct;
};

template <int KIND>
__global__ __launch_bounds__(256) void ogm_gemm_build_planes_kernel(GemmPlaneBuildParams p) {
  constexpr bool Q3 = KIND == GP_Q3K, Q45 = KIND == GP_Q4K || KIND == GP_Q5K, Q5 = KIND == GP_Q5K;
  constexpr uint32_t TILE_BYTES = Q3 ? 7168u : KIND == GP_Q4K ? 9216u : Q5 ? 11264u : 13440u;
  constexpr uint32_t QS_PIECE0 = Q5 ? 3u : 1u;
  constexpr uint32_t NPL = Q3 ? 1u : 2u;
  const uint32_t t16 = threadIdx.x >> 6, r = threadIdx.x & 63u;
  const uint32_t s = blockIdx.x >> 2, g = blockIdx.x & 3u, rb = blockIdx.y;
  const uint32_t row = min(64u * rb + r, p.out_dim - 1u);   // rows past the matrix repeat its last one
  const uint32_t uo = (row >> p.r_shift) * p.nct * TILE_BYTES + (row & ((1u << p.r_shift) - 1u)) * 16u;
  const uint32_t so = (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 16u;
  const uint8_t *u0 = p.wt + uo + so;
  const uint32_t h_ = g >> 1;
  uint4 ql, qh = make_uint4(0, 0, 0, 0);
  int sc;
  short addc;   // the constant added to sc * q
  uint32_t shift_q = 0, mask_q, hi_shift = 0, hi_mask = 0, hi_lsh = 0;   // q = (ql >> shift_q) & mask_q | ((qh >> hi_shift) & hi_mask) << hi_lsh
  if constexpr (Q3) {
    // run of 32: rr = 2 (g & 1) + t16 / 2 inside the half block; two bits at 2 rr, third bit = bit 2 g + t16 / 2 of hmask
    ql = *(const uint4 *)(u0 + (2u + 2u * h_ + (t16 & 1u)) * 1024u);
    qh = *(const uint4 *)(u0 + (t16 & 1u) * 1024u);
    const uint4 scx = *(const uint4 *)(u0 + 6u * 1024u);
    const uint32_t lw = (g & 1u) ? scx.y : scx.x;
    const uint32_t low = ((lw >> (8u * t16)) >> (g >= 2u ? 4u : 0u)) & 0xFu;
    const uint32_t high = ((scx.z >> (8u * t16)) >> (2u * g)) & 3u;
    const int scv = (int)(low | (high << 4)) - 32;
    sc = -scv;
    addc = (short)(4 * scv);
    shift_q = 2u * (2u * (g & 1u) + (t16 >> 1));
    mask_q = 0x03030303u;
    hi_shift = 2u * g + (t16 >> 1);
    hi_mask = 0x01010101u;
    hi_lsh = 2;
  } else if constexpr (Q45) {
    ql = *(const uint4 *)(u0 + (QS_PIECE0 + 2u * g + (t16 & 1u)) * 1024u);
    if constexpr (Q5) qh = *(const uint4 *)(u0 + (1u + (t16 & 1u)) * 1024u);
    const uint4 hd = *(const uint4 *)u0;
    uint32_t sc4a, sc4b;
    q4k_scales(hd, sc4a, sc4b);
    const uint32_t hi = t16 >> 1, j = 2u * g + hi;
    sc = (int)(((g < 2u ? sc4a : sc4b) >> (8u * (j & 3u))) & 0xFFu);
    addc = 128;
    shift_q = hi ? 4u : 0u;
    mask_q = 0x0F0F0F0Fu;
    hi_shift = j;
    hi_mask = Q5 ? 0x01010101u : 0u;
    hi_lsh = 4;
  } else {
    ql = *(const uint4 *)(u0 + (4u * h_ + t16) * 1024u);
    qh = *(const uint4 *)(u0 + (8u + 2u * h_ + (t16 & 1u)) * 1024u);
    const uint4 scx = *(const uint4 *)(u0 + 12u * 1024u);
    const uint32_t scw[4] = {scx.x, scx.y, scx.z, scx.w};
    sc = (int)(int8_t)((scw[g] >> (8u * t16)) & 0xFFu);
    addc = (short)(128 - 32 * sc);
    shift_q = (g & 1u) ? 4u : 0u;
    mask_q = 0x0F0F0F0Fu;
    hi_shift = 2u * (2u * (g & 1u) + (t16 >> 1));
    hi_mask = 0x03030303u;
    hi_lsh = 4;
  }
  const short2v sc2 = {(short)sc, (short)sc}, c2 = {addc, addc};
  const uint32_t qlw[4] = {ql.x, ql.y, ql.z, ql.w}, qhw[4] = {qh.x, qh.y, qh.z, qh.w};
  uint32_t ph[4], pl[4];
#pragma unroll
  for (int w = 0; w < 4; w++) {
    const uint32_t v = ((qlw[w] >> shift_q) & mask_q) | (((qhw[w] >> hi_shift) & hi_mask) << hi_lsh);
    union { uint32_t u; short2v s; } e, f;
    e.u = __builtin_amdgcn_perm(0u, v, 0x0c010c00u);   // (b0, b1) as 16-bit lanes
    f.u = __builtin_amdgcn_perm(0u, v, 0x0c030c02u);   // (b2, b3)
    e.s = e.s * sc2 + c2;
    f.s = f.s * sc2 + c2;
    if constexpr (Q3) {
      ph[w] = __builtin_amdgcn_perm(f.u, e.u, 0x06040200u);   // the lanes' low bytes
    } else {
      ph[w] = __builtin_amdgcn_perm(f.u, e.u, 0x07050301u);                 // high bytes
      pl[w] = __builtin_amdgcn_perm(f.u, e.u, 0x06040200u) ^ 0x80808080u;   // low bytes, top bit flipped
    }
  }
  uint8_t *dst = p.planes + gp_plane_offset(rb, p.nsb, s, g, t16, NPL) + r * 16u;
  *(uint4 *)dst = make_uint4(ph[0], ph[1], ph[2], ph[3]);
  if constexpr (!Q3) *(uint4 *)(dst + 1024u) = make_uint4(pl[0], pl[1], pl[2], pl[3]);
}

// ------------------------------------------------------------------------------------------
// The K-quant GEMM over prebuilt planes with every wave multiplying (no feeding waves): operands
// go from global memory straight into LDS (global_load_lds_dwordx4: no registers, no vector
// work), in the order the matrix instruction wants them, so a wave's operand read is 64 lanes x 16
// consecutive bytes.  Same arithmetic and f32 order as gemm_q6k_i8_body; bit-identical results.
//
//   workgroup  256 threads = 4 waves; 128 rows x 128 tokens; wave w: rows 32 w .. + 31, all tokens.
//              Two workgroups share a compute unit (two waves per SIMD, 74 KiB of LDS each): while
//              one adds a super-block's sums up in f32 the other multiplies.
//   step       32 weights of k: per wave the planes of its 32 rows (1 KiB each, fetched by the wave
//              itself), per workgroup four token blocks of activations (1 KiB each, one per wave)
//   ring       six steps in LDS: one multiplied, the next being read into registers behind it,
//              four in flight.  At the top of step k a wave waits until its loads of step k + 1
//              have landed (all but the newest three steps' loads), meets the others at a barrier,
//              and fetches step k + 5 into the slot step k - 1 left.
//   per super-block: the tokens' activation scales and the rows' d, fetched the same way one
//              super-block ahead (4 bytes a lane), then acc += ad * (d * isum) as the CPU path adds it
//
// The compiler cannot tell which LDS reads a load-to-LDS in flight may alias and would wait for all
// of them before every LDS read; the operand and table reads of the main loop are therefore written
// as ds_read instructions with their own waits (LDS reads return in order: "at most N outstanding"
// means all but the newest N have landed).  No scalar loads may be issued inside the loop (they
// share the counter and return out of order), which the launch parameters being read up front ensures.
//
// Registers: 8 accumulators of the planes (4 token blocks x h, l), 4 of y, 6 operands: 216 of a wave's 256.
struct GemmDmaParams {
  const uint8_t *wt;       // tile-planar weights (headers: d, dmin, mins)
  const uint8_t *planes;   // ogm_gemm_build_planes_kernel's output
  const int8_t *xt;        // ogm_gemm_xtile_kernel's output: [T / 32][in_dim / 32] operand chunks of 1 KiB
  const float *ad;         // [T][nsb]
  const _Float16 *bs16;    // Q4_K / Q5_K first pass
  float *y;
  uint32_t in_dim, out_dim, n_tokens, nsb;
  uint32_t c_shift, r_shift, nct;
  uint32_t n_extra;
  const uint8_t *extra_wt[OGM_GEMM_MAX_MATS - 1];
  const uint8_t *extra_planes[OGM_GEMM_MAX_MATS - 1];
  float *extra_y[OGM_GEMM_MAX_MATS - 1];
  uint32_t extra_out_dim[OGM_GEMM_MAX_MATS - 1];
};

#define GD_NW 4u                       // waves of a workgroup
#define GD_ROWS (32u * GD_NW)
#define GD_TOK 128u
// timing experiments only (results are wrong with any of these set)
#ifndef GD_ABL_SAMEROW
#define GD_ABL_SAMEROW 0   // every workgroup reads row block 0's planes
#endif
#ifndef GD_ABL_NOSWZ
#define GD_ABL_NOSWZ 0     // workgroups keep the grid's order
#endif
#ifndef GD_ABL_NOPASS1
#define GD_ABL_NOPASS1 0
#endif
#ifndef GD_ABL_NOEPI
#define GD_ABL_NOEPI 0
#endif
#ifndef GD_ABL_NOMFMA
#define GD_ABL_NOMFMA 0
#endif
#ifndef GD_ABL_NODMA
#define GD_ABL_NODMA 0
#endif
#ifndef GD_ABL_NOBAR
#define GD_ABL_NOBAR 0
#endif
#ifndef GD_ABL_NOLDS
#define GD_ABL_NOLDS 0
#endif
#ifndef GD_RING
#define GD_RING 6u
#endif
#define GD_AHEAD (GD_RING - 1u)        // steps fetched ahead of the one multiplied
#define GD_XOFF (GD_NW * 2048u)        // activations of a step, after the weights' 2 KiB per wave
#define GD_SLOT (GD_XOFF + 4096u)      // bytes of a step in LDS (one-plane types leave half the weights' part unused)
#define GD_TAB (GD_RING * GD_SLOT)     // two slots of per-super-block tables: 128 ad, then the rows' header words
#define GD_TAB_SLOT (512u + 4u * GD_ROWS)
#define GD_LDS_BYTES (GD_TAB + 2u * GD_TAB_SLOT)
// one-pass variant: 128 ad, the rows' 16-byte headers, the tokens' sums per 32 as f16 pairs (32 bytes a token)
#define GD_RING_ONEPASS 5u
#define GD_TAB_SLOT_ONEPASS (512u + 16u * GD_ROWS + 32u * GD_TOK)
#define GD_LDS_BYTES_ONEPASS (GD_RING_ONEPASS * GD_SLOT + 2u * GD_TAB_SLOT_ONEPASS)

__device__ __forceinline__ void gd_dma16(const uint8_t *src, uint8_t *lds_chunk) {
  // 16 bytes per lane from src (per lane) to lds_chunk + 16 * lane (lds_chunk is wave-uniform)
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                   (__attribute__((address_space(3))) void *)lds_chunk, 16, 0, 0);
}
__device__ __forceinline__ void gd_dma4(const uint8_t *src, uint8_t *lds_chunk) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                   (__attribute__((address_space(3))) void *)lds_chunk, 4, 0, 0);
}
// LDS reads the compiler does not see, and the waits that go with them.  A wait names the
// registers it makes valid, so that their uses stay behind it.
#define GD_READ16(DST, ADDR, OFF) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(DST) : "v"(ADDR), "n"(OFF))
#define GD_READ4(DST, ADDR, OFF) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(DST) : "v"(ADDR), "n"(OFF))
#define GD_WAIT1(N, A) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(A) : "n"(N))
#define GD_WAIT2(N, A, B) asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(A), "+v"(B) : "n"(N))
// all loads of this wave but the newest N have landed; then the workgroup's barrier (no fence: the
// data other waves wait for came by load-to-LDS, which the wait covers)
#if GD_ABL_NOBAR
#define GD_SYNC(N) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory")
#else
#define GD_SYNC(N) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory")
#endif

// The activations in the matrix instruction's operand order: chunk (token block of 32, step of 32 k)
// is 1 KiB, lane (l32, lh)'s 16 bytes -- the activations 32 step + 16 lh .. of token 32 block + l32 --
// at 16 (32 lh + l32).  A chunk is then one contiguous load; fetched row by row it would be 32 pieces
// of 32 distinct cache lines.  Tokens past the last repeat it (never stored).
__global__ __launch_bounds__(256) void ogm_gemm_xtile_kernel(const int8_t *__restrict__ xq, int8_t *__restrict__ xt,
                                                             uint32_t in_dim, uint32_t n_tokens) {
  // workgroup = 32 tokens x 128 activations = four chunks: read as eight 16-byte pieces a token (whole
  // 128-byte lines), turned through LDS (rows padded by a piece against bank conflicts), written as 4 KiB
  // in a row
  __shared__ uint4 tile[32][9];
  const uint32_t tid = threadIdx.x, tb = blockIdx.y, k0 = blockIdx.x * 128u;
  {
    const uint32_t tok = min(tb * 32u + (tid >> 3), n_tokens - 1u), piece = tid & 7u;
    tile[tid >> 3][piece] = *(const uint4 *)(xq + (size_t)tok * in_dim + k0 + 16u * piece);
  }
  __syncthreads();
  const uint32_t step = tid >> 6, slot = tid & 63u;   // the chunk of the four, the lane of its operand
  const uint4 v = tile[slot & 31u][2u * step + (slot >> 5)];
  *(uint4 *)(xt + ((size_t)tb * (in_dim / 32u) + k0 / 32u + step) * 1024u + slot * 16u) = v;
}

#if GD_ABL_NOMFMA
#define GD_MFMA(A, B, C, X, Y, Z) ((C) + (A).x + (B).x)
#else
#define GD_MFMA(A, B, C, X, Y, Z) __builtin_amdgcn_mfma_i32_32x32x32_i8(A, B, C, X, Y, Z)
#endif
#if GD_ABL_NOLDS
#define GD_RD if (0)
#else
#define GD_RD
#endif
// ONEPASS (Q4_K, Q5_K): no first pass; a super-block's step is acc += ad * (d * isum - dmin * imin), the
// single-token expression (vecdot.rs:3152-3178), with imin from the same K = 16 f16 instruction.  The integer
// sums are the same; the f32 result differs from the two-pass order by rounding only.  The rows' whole headers
// and the tokens' sums per 32 then travel with the tables, and the ring is one step shorter to make room.
template <int KIND, bool ONEPASS = false>
__global__ __launch_bounds__(64 * GD_NW, 2) void ogm_gemm_dma_kernel(GemmDmaParams p) {
  constexpr bool Q3 = KIND == GP_Q3K, Q45 = KIND == GP_Q4K || KIND == GP_Q5K, Q5 = KIND == GP_Q5K, Q6 = KIND == GP_Q6K;
  static_assert(!ONEPASS || Q45, "only the types with mins have a first pass to fold");
  constexpr uint32_t RING = ONEPASS ? GD_RING_ONEPASS : GD_RING, AHEAD = RING - 1u;
  constexpr uint32_t TAB = RING * GD_SLOT, TAB_SLOT = ONEPASS ? GD_TAB_SLOT_ONEPASS : GD_TAB_SLOT;
  constexpr uint32_t TILE_BYTES = Q3 ? 7168u : KIND == GP_Q4K ? 9216u : Q5 ? 11264u : 13440u;
  constexpr uint32_t NPL = Q3 ? 1u : 2u;
  constexpr int PER = (int)NPL + 1;   // loads a wave issues per step
  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  // Workgroups are dealt to the eight XCDs in turn, each with an L2 of its own: the token tiles of
  // one row tile go to one XCD back to back, so the row tile's planes leave memory once.
  uint32_t tok_tile = blockIdx.x, row_tile = blockIdx.y;
  {
    const uint32_t nt = gridDim.x, lin = blockIdx.y * nt + blockIdx.x;
    if (!GD_ABL_NOSWZ && lin < (gridDim.y & ~7u) * nt) {
      const uint32_t j = lin >> 3;
      tok_tile = j % nt;
      row_tile = (j / nt) * 8u + (lin & 7u);
    }
  }
#pragma unroll
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {   // the matrix this row tile belongs to
    const uint32_t tiles = (p.out_dim + GD_ROWS - 1u) / GD_ROWS;
    if (m < p.n_extra && row_tile >= tiles) {
      row_tile -= tiles;
      p.wt = p.extra_wt[m];
      p.planes = p.extra_planes[m];
      p.y = p.extra_y[m];
      p.out_dim = p.extra_out_dim[m];
    } else {
      break;
    }
  }
  const uint32_t t0 = tok_tile * GD_TOK, r0 = row_tile * GD_ROWS;
  auto sb_off = [&](uint32_t s) -> uint32_t {
    return (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 16u;
  };

  float16v y[4];
#pragma unroll
  for (int tb = 0; tb < 4; tb++)
#pragma unroll
    for (int r = 0; r < 16; r++) y[tb][r] = 0.0f;

  if constexpr (Q45 && !ONEPASS && !GD_ABL_NOPASS1) {
    // ---------------- pass 1 of gemm_k_q4_k: acc -= (ad * dmin) * sum_j m_j * bsum_j over all
    // super-blocks first (vecdot.rs:2226-2240), as gemm_q6k_i8_body does it: 64 m_j against bsum_j / 64
    // and m_j against bsum_j % 64 in one K = 16 f16 instruction per 32 x 32 outputs.  The tokens' ad of
    // every super-block sit in LDS (where the ring will be) for this pass.
    // this lane's weight row (clamped: rows past the matrix are computed and never stored)
    const uint32_t row = min(r0 + 32u * wave + l32, p.out_dim - 1u);
    const uint32_t uo = (row >> p.r_shift) * p.nct * TILE_BYTES + (row & ((1u << p.r_shift) - 1u)) * 16u;
    float *ad_all = (float *)lds;   // [nsb][128]
    for (uint32_t i = tid; i < GD_TOK * p.nsb; i += 64u * GD_NW) {
      const uint32_t k = i / p.nsb, su = i - k * p.nsb;
      ad_all[su * GD_TOK + k] = p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + su];
    }
    __syncthreads();
    float16v zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.0f;
    uint32_t tk[4];
#pragma unroll
    for (int tb = 0; tb < 4; tb++) tk[tb] = min(t0 + 32u * tb + l32, p.n_tokens - 1u) * p.nsb;
    const float side_scale = lh ? 1.0f : 64.0f;
    // the header and the four tokens' sums of the next super-block are loaded while this one is added up
    uint4 hd_n = *(const uint4 *)(p.wt + uo);
    half8 b2_n[4];
#pragma unroll
    for (int tb = 0; tb < 4; tb++) b2_n[tb] = *(const half8 *)(p.bs16 + (tk[tb] * 16u + 8u * lh));
    for (uint32_t su = 0; su < p.nsb; su++) {
      const uint4 hd0 = hd_n;
      half8 b2[4];
#pragma unroll
      for (int tb = 0; tb < 4; tb++) b2[tb] = b2_n[tb];
      {
        const uint32_t sn = min(su + 1u, p.nsb - 1u);   // past the end: loaded again, never used
        hd_n = *(const uint4 *)(p.wt + (uo + sb_off(sn)));
#pragma unroll
        for (int tb = 0; tb < 4; tb++) b2_n[tb] = *(const half8 *)(p.bs16 + ((tk[tb] + sn) * 16u + 8u * lh));
      }
      uint32_t mna, mnb;
      q4k_mins(hd0, mna, mnb);
      const half8 a1 = side_operand(mna, mnb, side_scale);
      const float dm = gm_f16_bits_to_f32(hd0.x >> 16);
#pragma unroll
      for (int tb = 0; tb < 4; tb++) {
        const float16v im = __builtin_amdgcn_mfma_f32_32x32x16_f16(b2[tb], a1, zero, 0, 0, 0);
        const float *adp = &ad_all[su * GD_TOK + 32u * tb + 4u * lh];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const float4 a4 = *(const float4 *)(adp + 8 * q4);
          const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
          for (int e = 0; e < 4; e++) y[tb][4 * q4 + e] -= a4v[e] * dm * im[4 * q4 + e];
        }
      }
    }
    __syncthreads();   // the table's LDS becomes the ring
  }

  // ---------------- the products
  // What this wave fetches per step: the plane chunks of its 32 rows (lane (l32, lh): the 16 weights
  // 16 lh .. of row l32, the matrix instruction's operand), and token block `wave` of the activations
  // (one chunk of ogm_gemm_xtile_kernel's layout).
  const uint32_t prb = GD_ABL_SAMEROW ? 0u : min((r0 + 32u * wave) >> 6, (p.out_dim - 1u) >> 6);
  uint32_t w_src = (prb * p.nsb * 16u + lh) * (NPL * 1024u) + (32u * (wave & 1u) + l32) * 16u;   // + step * NPL * 2048
  // (token blocks past the last one read it again; their outputs are never stored)
  uint32_t x_src = min((t0 >> 5) + wave, (p.n_tokens - 1u) >> 5) * (p.in_dim / 32u) * 1024u + lane * 16u;   // + step * 1024
  const uint32_t w_dst = wave * 2048u, x_dst = GD_XOFF + wave * 1024u;
  // tables: waves 0, 1 fetch 64 tokens' ad each, waves 2, 3 the header word of 64 rows each
  uint32_t tab_src;   // byte offset from p.ad (waves 0, 1) or p.wt (waves 2..5) for super-block 0
  if (wave < 2u) {
    tab_src = min(t0 + 64u * wave + lane, p.n_tokens - 1u) * p.nsb * 4u;
  } else {
    const uint32_t tab_row = min(r0 + 64u * ((wave - 2u) & 3u) + lane, p.out_dim - 1u);
    const uint32_t tab_rb = tab_row >> p.r_shift, tab_r = tab_row & ((1u << p.r_shift) - 1u);
    if constexpr (Q6)        // d is the block's two-byte tail behind the 13 pieces: the aligned word that holds it
      tab_src = tab_rb * p.nct * TILE_BYTES + 13u * 1024u + ((tab_r * 2u) & ~3u);
    else if constexpr (Q3)   // scales[12] | d | padding
      tab_src = tab_rb * p.nct * TILE_BYTES + tab_r * 16u + 6u * 1024u + 12u;
    else                     // d | dmin
      tab_src = tab_rb * p.nct * TILE_BYTES + tab_r * 16u;
  }
  // one-pass: token block `wave`'s sums per 32 (lane (l32, lh): the eight f16 of half lh of token l32)
  const uint32_t bs_src = (min(t0 + 32u * wave + l32, p.n_tokens - 1u) * p.nsb * 16u + 8u * lh) * 2u;   // + 32 s
  auto fetch_tables = [&](uint32_t s) {   // for super-block s, into table slot s & 1
    uint8_t *slot = lds + TAB + (s & 1u) * TAB_SLOT;
    if (wave < 2u) {
      gd_dma4((const uint8_t *)p.ad + (tab_src + 4u * s), slot + 256u * wave);
    } else {
      const uint32_t so = Q6 ? (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 2u : sb_off(s);
      if constexpr (ONEPASS) gd_dma16(p.wt + (tab_src + so), slot + 512u + 1024u * (wave - 2u));
      else gd_dma4(p.wt + (tab_src + so), slot + 512u + 256u * (wave - 2u));
    }
    if constexpr (ONEPASS)
      gd_dma16((const uint8_t *)p.bs16 + (bs_src + 32u * s), slot + 512u + 16u * GD_ROWS + 1024u * wave);
  };
  uint32_t slot_fetch = 0;   // byte offset of the ring slot of the next step to fetch
  auto fetch_step = [&]() {   // the next step (they are fetched in ascending order) into its ring slot
    uint8_t *slot = lds + slot_fetch;
    slot_fetch = slot_fetch == (RING - 1u) * GD_SLOT ? 0u : slot_fetch + GD_SLOT;
#if !GD_ABL_NOWDMA
    gd_dma16(p.planes + w_src, slot + w_dst);
    if constexpr (!Q3) gd_dma16(p.planes + (w_src + 1024u), slot + w_dst + 1024u);
#endif
#if !GD_ABL_NOXDMA
    gd_dma16((const uint8_t *)p.xt + x_src, slot + x_dst);
#endif
    w_src += NPL * 2048u;
    x_src += 1024u;
  };

  fetch_tables(0u);
#pragma unroll
  for (uint32_t k = 0; k < AHEAD; k++) fetch_step();
  GD_SYNC((AHEAD - 1) * PER);   // step 0 and the first tables have landed

  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
  const uint32_t w_rd = lds0 + w_dst + lane * 16u, x_rd = lds0 + GD_XOFF + lane * 16u;
  const uint32_t tab_rd = lds0 + TAB + 16u * lh;                    // + 128 tb + 32 q4: four tokens' ad
  // the row's header word (one-pass: its 16-byte header)
  const uint32_t hw_rd = lds0 + TAB + 512u + (ONEPASS ? 16u : 4u) * (32u * wave + l32);
  const uint32_t bs_rd = lds0 + TAB + 512u + 16u * GD_ROWS + 16u * lane;   // one-pass: + 1024 tb
  int16v h[4], l[4];
  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  int4v wh, wl = {0, 0, 0, 0}, x0, x1, x2, x3;
  // LDS reads outstanding at the top of a step, oldest first: wh, x0, x1, x2, x3, wl (one-plane types: no wl)
  GD_READ16(wh, w_rd, 0);
  GD_READ16(x0, x_rd, 0);
  GD_READ16(x1, x_rd, 1024);
  GD_READ16(x2, x_rd, 2048);
  GD_READ16(x3, x_rd, 3072);
  if constexpr (!Q3) GD_READ16(wl, w_rd, 1024);
  uint32_t slot_next = GD_SLOT;   // byte offset of step k + 1's ring slot
  for (uint32_t s = 0; s < p.nsb; s++) {
#pragma unroll
    for (uint32_t kk = 0; kk < 8u; kk++) {
      // step k = 8 s + kk: step k + 1 landed (all but the loads of the steps after it, at most four), for every wave
      const bool more = s + 1u < p.nsb;   // in the last super-block the steps in flight run out
      // (steps after k + 1 in flight: GD_AHEAD - 2, fewer at the end)
      if (kk + AHEAD <= 8u || more) GD_SYNC((AHEAD - 2) * PER);
      else GD_SYNC(kk >= 6u ? 0 : (int)(6u - kk) * PER);
      if (kk == 0u && more) fetch_tables(s + 1u);
      if ((kk + AHEAD < 8u || more) && !GD_ABL_NODMA) fetch_step();   // step k + AHEAD
      const uint32_t w_nx = w_rd + slot_next, x_nx = x_rd + slot_next;
      slot_next = slot_next == (RING - 1u) * GD_SLOT ? 0u : slot_next + GD_SLOT;
      if constexpr (!Q3) {
        constexpr int A0 = 4;   // outstanding after wh and x0: x1, x2, x3, wl
        GD_WAIT2(A0, wh, x0);
        h[0] = GD_MFMA(x0, wh, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : h[0], 0, 0, 0);
        GD_WAIT1(3, x1);
        h[1] = GD_MFMA(x1, wh, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : h[1], 0, 0, 0);
        GD_WAIT1(2, x2);
        h[2] = GD_MFMA(x2, wh, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : h[2], 0, 0, 0);
        GD_WAIT1(1, x3);
        h[3] = GD_MFMA(x3, wh, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : h[3], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:0" : "=v"(wh) : "0"(wh), "v"(w_nx));
        GD_WAIT1(1, wl);
        l[0] = GD_MFMA(x0, wl, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : l[0], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:0" : "=v"(x0) : "0"(x0), "v"(x_nx));
        l[1] = GD_MFMA(x1, wl, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : l[1], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:1024" : "=v"(x1) : "0"(x1), "v"(x_nx));
        l[2] = GD_MFMA(x2, wl, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : l[2], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:2048" : "=v"(x2) : "0"(x2), "v"(x_nx));
        l[3] = GD_MFMA(x3, wl, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : l[3], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:3072" : "=v"(x3) : "0"(x3), "v"(x_nx));
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:1024" : "=v"(wl) : "0"(wl), "v"(w_nx));
      } else {
        // one plane: the next step's weights go to a second register set (this one is in use to the
        // end); outstanding at the top, oldest first: wh, x0, x1, x2, x3
        int4v wn;
        GD_READ16(wn, w_nx, 0);
        GD_WAIT2(4, wh, x0);
        h[0] = GD_MFMA(x0, wh, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : h[0], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:0" : "=v"(x0) : "0"(x0), "v"(x_nx));
        GD_WAIT1(4, x1);
        h[1] = GD_MFMA(x1, wh, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : h[1], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:1024" : "=v"(x1) : "0"(x1), "v"(x_nx));
        GD_WAIT1(4, x2);
        h[2] = GD_MFMA(x2, wh, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : h[2], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:2048" : "=v"(x2) : "0"(x2), "v"(x_nx));
        GD_WAIT1(4, x3);
        h[3] = GD_MFMA(x3, wh, (kk == 0u && (!GD_ABL_NOEPI || s == 0u)) ? zi : h[3], 0, 0, 0);
        GD_RD asm volatile("ds_read_b128 %0, %2 offset:3072" : "=v"(x3) : "0"(x3), "v"(x_nx));
        // the next step wants wn first in line: it was issued before these four
        GD_WAIT1(4, wn);
        wh = wn;
      }
      if (kk == 7u && (!GD_ABL_NOEPI || s + 1u == p.nsb)) {
        // acc += ad * (d * isum) for the super-block (vecdot.rs:2242-2300 in the order of its sums)
        const uint32_t tsl = (s & 1u) * TAB_SLOT;
        uint32_t hw;
        half8 a1 = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr (ONEPASS) {
          int4v hd;
          GD_READ16(hd, hw_rd + tsl, 0);
          GD_WAIT1(0, hd);
          hw = (uint32_t)hd.x;
          uint32_t mna, mnb;
          q4k_mins(make_uint4((uint32_t)hd.x, (uint32_t)hd.y, (uint32_t)hd.z, (uint32_t)hd.w), mna, mnb);
          a1 = side_operand(mna, mnb, lh ? 1.0f : 64.0f);
        } else {
          GD_READ4(hw, hw_rd + tsl, 0);
          GD_WAIT1(0, hw);
        }
        // Q6_K's word holds the d of a pair of rows
        const float d0 = gm_f16_bits_to_f32(Q6 && (l32 & 1u) ? (hw >> 16) : (hw & 0xFFFFu));
        const float ndm = -gm_f16_bits_to_f32(hw >> 16);   // one-pass: -dmin
        const uint32_t ta = tab_rd + tsl;
#pragma unroll
        for (int tb = 0; tb < 4; tb++) {
          typedef float float4v __attribute__((ext_vector_type(4)));
          float4v a40, a41, a42, a43;
          if constexpr (ONEPASS) {
            // d * isum of the block's 16 outputs first (the integer sums die here), then imin into the registers
            // they leave, then one multiply-add each for the mins and for the token's scale
            half8 b2;
            GD_READ16(b2, bs_rd + tsl, 1024 * tb);
            float t[16];
#pragma unroll
            for (int r = 0; r < 16; r++) t[r] = d0 * (float)(h[tb][r] * 256 + l[tb][r]);
            GD_WAIT1(0, b2);
            const float16v zf = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const float16v im = __builtin_amdgcn_mfma_f32_32x32x16_f16(b2, a1, zf, 0, 0, 0);
            GD_READ16(a40, ta, 128 * tb);
            GD_READ16(a41, ta, 128 * tb + 32);
            GD_READ16(a42, ta, 128 * tb + 64);
            GD_READ16(a43, ta, 128 * tb + 96);
            GD_WAIT2(0, a40, a41);
            GD_WAIT2(0, a42, a43);
            const float4v a4[4] = {a40, a41, a42, a43};
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
              const float a4v[4] = {a4[q4].x, a4[q4].y, a4[q4].z, a4[q4].w};
#pragma unroll
              for (int e = 0; e < 4; e++)
                y[tb][4 * q4 + e] = __builtin_fmaf(a4v[e], __builtin_fmaf(ndm, im[4 * q4 + e], t[4 * q4 + e]), y[tb][4 * q4 + e]);
            }
            continue;
          }
          GD_READ16(a40, ta, 128 * tb);
          GD_READ16(a41, ta, 128 * tb + 32);
          GD_READ16(a42, ta, 128 * tb + 64);
          GD_READ16(a43, ta, 128 * tb + 96);
          GD_WAIT2(0, a40, a41);
          GD_WAIT2(0, a42, a43);
          const float4v a4[4] = {a40, a41, a42, a43};
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++) {
            const float a4v[4] = {a4[q4].x, a4[q4].y, a4[q4].z, a4[q4].w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const int is = Q3 ? -h[tb][4 * q4 + e] : h[tb][4 * q4 + e] * 256 + l[tb][4 * q4 + e];
              y[tb][4 * q4 + e] += a4v[e] * (d0 * (float)is);
            }
          }
        }
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wh), "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3), "+v"(wl));   // the reads past the last step
  const uint32_t row0 = r0 + 32u * wave + l32;
  if (row0 < p.out_dim) {
#pragma unroll
    for (int tb = 0; tb < 4; tb++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const uint32_t t = t0 + 32u * tb + 8u * (r >> 2) + 4u * lh + (r & 3);
        if (t < p.n_tokens) p.y[(size_t)t * p.out_dim + row0] = y[tb][r];
      }
  }
}

// ------------------------------------------------------------------------------------------
// Small batches (up to a few dozen tokens): the tiled kernels above cost the same for 9 tokens as
// for 128, because a workgroup walks its rows' super-blocks one after the other.  Here a workgroup
// owns 32 rows x 32 tokens and its eight waves take different super-blocks of those rows at the same
// time, each unpacking the weights straight into the matrix instruction's operand registers (a
// lane's operand is 16 consecutive weights of one row) and reading the int8 activations from
// memory as they are.  A super-block's contribution ad * (d * isum) does not depend on the others;
// only the additions are ordered, so the waves leave their terms in LDS and after every round of
// eight super-blocks the terms are added in ascending order, as gemm_k_q6_k does
// (vecdot.rs:2352-2398).  The chain of a workgroup is nsb / 8 rounds long instead of 4 nsb stages.

struct GemmSbParams {
  const uint8_t *wt;      // tile-planar weights
  const int8_t *xq;       // [T][in_dim] int8 activations
  const float *ad;        // [T][nsb]
  const _Float16 *bs16;   // Q4_K / Q5_K: the quantizer's sums per 32 as (bsum / 64, bsum % 64) in f16
  float *y;               // [T][out_dim]
  uint32_t in_dim, out_dim, n_tokens, nsb;
  uint32_t c_shift, r_shift, nct;
  uint32_t n_extra;
  const uint8_t *extra_wt[OGM_GEMM_MAX_MATS - 1];
  float *extra_y[OGM_GEMM_MAX_MATS - 1];
  uint32_t extra_out_dim[OGM_GEMM_MAX_MATS - 1];
};

// NW waves (8 or 16): sixteen halve the chain once more and suit launches of few workgroups.
template <uint32_t NW>
__device__ __forceinline__ void gemm_sb_q6k_body(GemmSbParams p) {
  constexpr uint32_t NT = 64u * NW, NACC = 1024u / NT;
  constexpr uint32_t TILE_BYTES = 13440u;
  extern __shared__ __align__(16) uint8_t sb_lds[];
  float *terms = (float *)sb_lds;            // [NW waves][32 tokens][32 rows]
  float *ad_l = terms + NW * 32u * 32u;      // [nsb][32 tokens]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  uint32_t row_tile = blockIdx.y;
#pragma unroll
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {   // the matrix this row tile belongs to
    const uint32_t tiles = (p.out_dim + 31u) / 32u;
    if (m < p.n_extra && row_tile >= tiles) {
      row_tile -= tiles;
      p.wt = p.extra_wt[m];
      p.y = p.extra_y[m];
      p.out_dim = p.extra_out_dim[m];
    } else {
      break;
    }
  }
  const uint32_t t0 = blockIdx.x * 32u, r0 = row_tile * 32u;
  uint32_t uo, to;   // this lane's row: its 16-byte pieces (the upper lane half: the next piece) and its tail
  {
    const uint32_t row = min(r0 + l32, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    uo = rb * p.nct * TILE_BYTES + r * 16u + lh * 1024u;
    to = rb * p.nct * TILE_BYTES + 13u * 1024u + r * 2u;
  }
  auto sb_off = [&](uint32_t s) -> uint32_t {
    return (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 16u;
  };
  auto sb_tail = [&](uint32_t s) -> uint32_t {
    return (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 2u;
  };
  const uint32_t xro = min(t0 + l32, p.n_tokens - 1u) * p.in_dim + 16u * lh;   // + 256 s + 32 sub
  const uint32_t sc_shift = 8u * lh;

  // the tokens' ad of every super-block: ad_l[s][token]
  for (uint32_t i = tid; i < 32u * p.nsb; i += NT) {
    const uint32_t k = i / p.nsb, s = i - k * p.nsb;
    ad_l[s * 32u + k] = p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + s];
  }

  uint4 wA0, wB0, wQ0, wA1, wB1, wQ1, scw;
  uint32_t d16;
#define SB_LOADW(S)                                                                               \
  do {                                                                                            \
    const uint32_t s_ = min((uint32_t)(S), p.nsb - 1u); /* past the end: loaded, never used */    \
    const uint32_t so_ = uo + sb_off(s_);                                                         \
    wA0 = *(const uint4 *)(p.wt + so_);                                                           \
    wB0 = *(const uint4 *)(p.wt + (so_ + 2u * 1024u));                                            \
    wA1 = *(const uint4 *)(p.wt + (so_ + 4u * 1024u));                                            \
    wB1 = *(const uint4 *)(p.wt + (so_ + 6u * 1024u));                                            \
    wQ0 = *(const uint4 *)(p.wt + (so_ + 8u * 1024u));                                            \
    wQ1 = *(const uint4 *)(p.wt + (so_ + 10u * 1024u));                                           \
    scw = *(const uint4 *)(p.wt + (so_ - lh * 1024u + 12u * 1024u));                              \
    d16 = *(const uint16_t *)(p.wt + (to + sb_tail(s_)));                                         \
  } while (0)
  // 16 weights of run 2 (G % 2) + SUB of a half block -> the two operand planes: u = sc * q +
  // (128 - 32 sc) as a 16-bit lane, high byte h, low byte with its top bit flipped l
#define SB_UNPACK(DH, DL, QL, QH, SCW, G, SUB)                                                    \
  do {                                                                                            \
    const int sc_ = __builtin_amdgcn_sbfe((int)(SCW), sc_shift + 16u * (SUB), 8u);                \
    const short2v sc2_ = {(short)sc_, (short)sc_};                                                \
    const short2v c2_ = {(short)(128 - 32 * sc_), (short)(128 - 32 * sc_)};                       \
    constexpr uint32_t rr_ = 2u * ((G) & 1u) + (SUB);                                             \
    const uint32_t qlw_[4] = {QL.x, QL.y, QL.z, QL.w}, qhw_[4] = {QH.x, QH.y, QH.z, QH.w};        \
    uint32_t ph_[4], pl_[4];                                                                      \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      const uint32_t nib_ = (((G) & 1u) ? (qlw_[w_] >> 4) : qlw_[w_]) & 0x0F0F0F0Fu;              \
      const uint32_t hi_ = rr_ < 2u ? (qhw_[w_] << (4u - 2u * rr_)) : (qhw_[w_] >> (2u * rr_ - 4u)); \
      const uint32_t v_ = (hi_ & 0x30303030u) | nib_;                                             \
      union { uint32_t u; short2v s; } e_, f_;                                                    \
      e_.u = __builtin_amdgcn_perm(0u, v_, 0x0c010c00u);   /* (b0, b1) as 16-bit lanes */         \
      f_.u = __builtin_amdgcn_perm(0u, v_, 0x0c030c02u);   /* (b2, b3) */                         \
      e_.s = e_.s * sc2_ + c2_;                                                                   \
      f_.s = f_.s * sc2_ + c2_;                                                                   \
      ph_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x07050301u);                                   \
      pl_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x06040200u) ^ 0x80808080u;                     \
    }                                                                                             \
    DH = (int4v){(int)ph_[0], (int)ph_[1], (int)ph_[2], (int)ph_[3]};                             \
    DL = (int4v){(int)pl_[0], (int)pl_[1], (int)pl_[2], (int)pl_[3]};                             \
  } while (0)
#define SB_STEP(QL, QH, SCW, G, SUB, FIRST)                                                       \
  do {                                                                                            \
    int4v bh_, bl_;                                                                               \
    SB_UNPACK(bh_, bl_, QL, QH, SCW, G, SUB);                                                     \
    const int4v xa_ = *(const int4v *)(p.xq + (xs_ + 64u * (G) + 32u * (SUB)));                   \
    H = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_, bh_, (FIRST) ? zi : H, 0, 0, 0);               \
    L = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_, bl_, (FIRST) ? zi : L, 0, 0, 0);               \
  } while (0)

  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float acc[NACC];   // outputs (token, row) = (tid / 32 + a NT / 32, tid % 32)
#pragma unroll
  for (uint32_t a = 0; a < NACC; a++) acc[a] = 0.0f;
  SB_LOADW(wave);
  __syncthreads();   // ad_l
  for (uint32_t s0 = 0; s0 < p.nsb; s0 += NW) {
    const uint32_t s = s0 + wave;
    if (s < p.nsb) {   // wave-uniform
      const uint32_t xs_ = xro + 256u * s;
      int16v H, L;
      SB_STEP(wA0, wQ0, scw.x, 0, 0, true);
      SB_STEP(wB0, wQ0, scw.x, 0, 1, false);
      SB_STEP(wA0, wQ0, scw.y, 1, 0, false);
      SB_STEP(wB0, wQ0, scw.y, 1, 1, false);
      SB_STEP(wA1, wQ1, scw.z, 2, 0, false);
      SB_STEP(wB1, wQ1, scw.z, 2, 1, false);
      SB_STEP(wA1, wQ1, scw.w, 3, 0, false);
      SB_STEP(wB1, wQ1, scw.w, 3, 1, false);
      const float d = gm_f16_bits_to_f32(d16);
      const float *adp = &ad_l[s * 32u + 4u * lh];
      float *tp = terms + (wave * 32u + 4u * lh) * 32u + l32;   // [wave][token][row]
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const float4 a4 = *(const float4 *)(adp + 8 * q4);
        const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int is_ = H[4 * q4 + e] * 256 + L[4 * q4 + e];
          tp[(8 * q4 + e) * 32] = a4v[e] * (d * (float)is_);
        }
      }
    }
    SB_LOADW(s + NW);   // the next round's weights, in flight over the barrier and the additions
    __syncthreads();
    {
      const uint32_t n_here = min(NW, p.nsb - s0);
      for (uint32_t w = 0; w < n_here; w++) {   // ascending super-blocks, one accumulator per output
#pragma unroll
        for (uint32_t a = 0; a < NACC; a++) acc[a] += terms[w * 1024u + a * NT + tid];
      }
    }
    __syncthreads();
  }
#undef SB_LOADW
#undef SB_UNPACK
#undef SB_STEP
  {
    const uint32_t row = r0 + (tid & 31u);
#pragma unroll
    for (uint32_t a = 0; a < NACC; a++) {
      const uint32_t tok = t0 + (tid >> 5) + a * (NT / 32u);
      if (row < p.out_dim && tok < p.n_tokens) p.y[(size_t)tok * p.out_dim + row] = acc[a];
    }
  }
}

__global__ __launch_bounds__(512) void ogm_gemm_sb_q6k_kernel(GemmSbParams p) { gemm_sb_q6k_body<8u>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_sb_q6k_w16_kernel(GemmSbParams p) { gemm_sb_q6k_body<16u>(p); }

// The same for Q4_K and Q5_K (gemm_k_q4_k, vecdot.rs:2213-2303): first a sweep over the super-blocks
// for the terms (ad * dmin) * imin, which the reference subtracts before anything else (rounds of
// sixteen super-blocks, two per wave: header and the quantizer's sums per 32 only, one f16 matrix
// instruction each), then the sweep of the products as above.  A lane's 16 weights of sub-block j
// are the low (j even) or high nibbles of one 16-byte piece of qs, Q5_K's fifth bit is bit j of
// its piece of qh.
template <bool Q5, uint32_t NW>
__device__ __forceinline__ void gemm_sb_q45k_body(GemmSbParams p) {
  constexpr uint32_t NT = 64u * NW, NACC = 1024u / NT;
  constexpr uint32_t TILE_BYTES = Q5 ? 11264u : 9216u;
  constexpr uint32_t QS_PIECE0 = Q5 ? 3u : 1u;
  extern __shared__ __align__(16) uint8_t sb_lds[];
  float *terms = (float *)sb_lds;             // [16 super-blocks][32 tokens][32 rows] (second sweep: NW)
  float *ad_l = terms + 16u * 32u * 32u;      // [nsb][32 tokens]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  uint32_t row_tile = blockIdx.y;
#pragma unroll
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {   // the matrix this row tile belongs to
    const uint32_t tiles = (p.out_dim + 31u) / 32u;
    if (m < p.n_extra && row_tile >= tiles) {
      row_tile -= tiles;
      p.wt = p.extra_wt[m];
      p.y = p.extra_y[m];
      p.out_dim = p.extra_out_dim[m];
    } else {
      break;
    }
  }
  const uint32_t t0 = blockIdx.x * 32u, r0 = row_tile * 32u;
  uint32_t uo;   // this lane's row: its header piece
  {
    const uint32_t row = min(r0 + l32, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    uo = rb * p.nct * TILE_BYTES + r * 16u;
  }
  auto sb_off = [&](uint32_t s) -> uint32_t {
    return (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 16u;
  };
  const uint32_t tok = min(t0 + l32, p.n_tokens - 1u);
  const uint32_t xro = tok * p.in_dim + 16u * lh;   // + 256 s + 32 j
  const uint32_t tk = tok * p.nsb;

  for (uint32_t i = tid; i < 32u * p.nsb; i += NT) {
    const uint32_t k = i / p.nsb, s = i - k * p.nsb;
    ad_l[s * 32u + k] = p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + s];
  }
  __syncthreads();

  float acc[NACC];   // outputs (token, row) = (tid / 32 + a NT / 32, tid % 32)
#pragma unroll
  for (uint32_t a = 0; a < NACC; a++) acc[a] = 0.0f;
  // ---- first sweep: acc -= (ad * dmin) * sum_j m_j * bsum_j
  {
    float16v zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.0f;
    const float side_scale = lh ? 1.0f : 64.0f;
    for (uint32_t s0 = 0; s0 < p.nsb; s0 += 16u) {
#pragma unroll
      for (uint32_t u = 0; u < 16u / NW; u++) {
        const uint32_t sl = wave + NW * u, s = s0 + sl;
        if (s < p.nsb) {   // wave-uniform
          const uint4 hd = *(const uint4 *)(p.wt + (uo + sb_off(s)));
          const half8 b2 = *(const half8 *)(p.bs16 + ((tk + s) * 16u + 8u * lh));
          uint32_t mna, mnb;
          q4k_mins(hd, mna, mnb);
          const half8 a1 = side_operand(mna, mnb, side_scale);
          const float dm = gm_f16_bits_to_f32(hd.x >> 16);
          const float16v im = __builtin_amdgcn_mfma_f32_32x32x16_f16(b2, a1, zero, 0, 0, 0);
          const float *adp = &ad_l[s * 32u + 4u * lh];
          float *tp = terms + (sl * 32u + 4u * lh) * 32u + l32;   // [super-block][token][row]
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++) {
            const float4 a4 = *(const float4 *)(adp + 8 * q4);
            const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
            for (int e = 0; e < 4; e++) tp[(8 * q4 + e) * 32] = a4v[e] * dm * im[4 * q4 + e];
          }
        }
      }
      __syncthreads();
      const uint32_t n_here = min(16u, p.nsb - s0);
      for (uint32_t w = 0; w < n_here; w++) {
#pragma unroll
        for (uint32_t a = 0; a < NACC; a++) acc[a] -= terms[w * 1024u + a * NT + tid];
      }
      __syncthreads();
    }
  }
  // ---- second sweep: acc += ad * (d * sum_j sc_j * dot32_j)
  uint4 hdr, w0, w1, w2, w3, qh5 = make_uint4(0, 0, 0, 0);
#define SB_LOADW(S)                                                                               \
  do {                                                                                            \
    const uint32_t s_ = min((uint32_t)(S), p.nsb - 1u); /* past the end: loaded, never used */    \
    const uint32_t so_ = uo + sb_off(s_);                                                         \
    hdr = *(const uint4 *)(p.wt + so_);                                                           \
    w0 = *(const uint4 *)(p.wt + (so_ + (QS_PIECE0 + 0u + lh) * 1024u));                          \
    w1 = *(const uint4 *)(p.wt + (so_ + (QS_PIECE0 + 2u + lh) * 1024u));                          \
    w2 = *(const uint4 *)(p.wt + (so_ + (QS_PIECE0 + 4u + lh) * 1024u));                          \
    w3 = *(const uint4 *)(p.wt + (so_ + (QS_PIECE0 + 6u + lh) * 1024u));                          \
    if constexpr (Q5) qh5 = *(const uint4 *)(p.wt + (so_ + (1u + lh) * 1024u));                   \
  } while (0)
  // One matrix instruction per sub-block on the bare quants (K = 32 is exactly a sub-block; a lane's
  // operand is its row's 16 nibbles, with Q5_K's fifth bit on top), then isum += sc_j * dot_j as
  // 24-bit integer multiply-adds (|dot_j| <= 31 * 127 * 32 < 2^17, sc_j < 64): the same integer.
#define SB_MMA(D, QS, J)                                                                          \
  do {                                                                                            \
    const uint32_t qsw_[4] = {QS.x, QS.y, QS.z, QS.w}, q5w_[4] = {qh5.x, qh5.y, qh5.z, qh5.w};    \
    uint32_t v_[4];                                                                               \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      v_[w_] = (((J) & 1) ? (qsw_[w_] >> 4) : qsw_[w_]) & 0x0F0F0F0Fu;                            \
      if constexpr (Q5) v_[w_] |= ((q5w_[w_] >> (J)) & 0x01010101u) << 4;                         \
    }                                                                                             \
    const int4v b_ = {(int)v_[0], (int)v_[1], (int)v_[2], (int)v_[3]};                            \
    const int4v xa_ = *(const int4v *)(p.xq + (xs_ + 32u * (J)));                                 \
    D = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_, b_, zi, 0, 0, 0);                              \
  } while (0)
#define SB_ACC(D, J, FIRST)                                                                       \
  do {                                                                                            \
    const int sc_ = (int)((((J) < 4 ? sca_ : scb_) >> (8u * ((J) & 3u))) & 0xFFu);                \
    _Pragma("unroll") for (int r_ = 0; r_ < 16; r_++)                                             \
      I[r_] = (FIRST) ? __mul24(sc_, D[r_]) : __mul24(sc_, D[r_]) + I[r_];                        \
  } while (0)
  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  SB_LOADW(wave);
  for (uint32_t s0 = 0; s0 < p.nsb; s0 += NW) {
    const uint32_t s = s0 + wave;
    if (s < p.nsb) {   // wave-uniform
      const uint32_t xs_ = xro + 256u * s;
      uint32_t sca_, scb_;
      q4k_scales(hdr, sca_, scb_);
      int16v I, Da, Db;   // the products of a sub-block are under way while the one before is added
      SB_MMA(Da, w0, 0);
      SB_MMA(Db, w0, 1);
      SB_ACC(Da, 0, true);
      SB_MMA(Da, w1, 2);
      SB_ACC(Db, 1, false);
      SB_MMA(Db, w1, 3);
      SB_ACC(Da, 2, false);
      SB_MMA(Da, w2, 4);
      SB_ACC(Db, 3, false);
      SB_MMA(Db, w2, 5);
      SB_ACC(Da, 4, false);
      SB_MMA(Da, w3, 6);
      SB_ACC(Db, 5, false);
      SB_MMA(Db, w3, 7);
      SB_ACC(Da, 6, false);
      SB_ACC(Db, 7, false);
      const float d = gm_f16_bits_to_f32(hdr.x & 0xFFFFu);
      const float *adp = &ad_l[s * 32u + 4u * lh];
      float *tp = terms + (wave * 32u + 4u * lh) * 32u + l32;   // [wave][token][row]
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const float4 a4 = *(const float4 *)(adp + 8 * q4);
        const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int is_ = I[4 * q4 + e];
          tp[(8 * q4 + e) * 32] = a4v[e] * (d * (float)is_);
        }
      }
    }
    SB_LOADW(s + NW);   // the next round's weights, in flight over the barrier and the additions
    __syncthreads();
    {
      const uint32_t n_here = min(NW, p.nsb - s0);
      for (uint32_t w = 0; w < n_here; w++) {   // ascending super-blocks, one accumulator per output
#pragma unroll
        for (uint32_t a = 0; a < NACC; a++) acc[a] += terms[w * 1024u + a * NT + tid];
      }
    }
    __syncthreads();
  }
#undef SB_LOADW
#undef SB_MMA
#undef SB_ACC
  {
    const uint32_t row = r0 + (tid & 31u);
#pragma unroll
    for (uint32_t a = 0; a < NACC; a++) {
      const uint32_t tok_o = t0 + (tid >> 5) + a * (NT / 32u);
      if (row < p.out_dim && tok_o < p.n_tokens) p.y[(size_t)tok_o * p.out_dim + row] = acc[a];
    }
  }
}

template <bool Q5>
__global__ __launch_bounds__(512) void ogm_gemm_sb_q45k_kernel(GemmSbParams p) { gemm_sb_q45k_body<Q5, 8u>(p); }
template <bool Q5>
__global__ __launch_bounds__(1024) void ogm_gemm_sb_q45k_w16_kernel(GemmSbParams p) { gemm_sb_q45k_body<Q5, 16u>(p); }

// ------------------------------------------------------------------------------------------
// Q4_K, wide tile: 128 rows x 256 tokens per workgroup, twelve waves.
//
// The 128 x 128 kernel above is bound by LDS bandwidth: a multiplying wave reads (64 + 32) k-rows
// from LDS per pair of MFMAs.  Here a multiplying wave owns 64 rows x 64 tokens (four 32 x 32
// tiles, so the same reads feed twice the MFMAs), the activations stay int8 in LDS (half the
// bytes; the multiplying wave turns them into f16 with the 0x6400 | (x + 128) = 1024 + (x + 128)
// trick, exact), and a workgroup has eight multiplying and four feeding waves, three per SIMD,
// which leaves 168 registers per lane.  The four integer-sum and four f32 accumulator tiles take
// 128 of them, so the loop is written to keep little else alive (a fence after every MFMA step
// keeps later steps' LDS reads from being hoisted; without it accumulators spill).
//
// k order inside a stage: MFMA step kk of the lane half lh covers k = 32 (kk >> 1) + 16 lh +
// 8 (kk & 1) + 0..7, so that a lane's activations for two steps are 16 contiguous bytes.
//
// Pass 1 (the min terms of all super-blocks, first, as the reference orders them) takes its
// operands from LDS tables that all twelve waves fill for eight super-blocks at a time: one trip
// to memory per group instead of one per four super-blocks.  The tables alias the stage buffers.

#define GW_BT 256u           // tokens per workgroup
#define GW_PG 8u             // super-blocks per pass-1 group
// Staged tiles are padded by one 16-byte chunk per row (weights: 64 f16 + 8, activations: 64 bytes
// + 16).  Sixteen consecutive rows then start 36 (or 20) banks apart, which puts their 16-byte
// accesses on sixteen disjoint groups of four banks, and a chunk's position is a compile-time
// offset from the row's address: no swizzle arithmetic in the loop.
#define GW_A_ROW 72u                     // f16 per staged weight row
#define GW_B_ROW 80u                     // bytes per staged activation row
#define GW_A_STAGE (128u * GW_A_ROW)     // f16 per staged weight tile (18 KB)
#define GW_B_STAGE (256u * GW_B_ROW)     // bytes per staged activation tile (20 KB)
// main loop: A [2] 36 KB | B [2] 40 KB | a2 4 KB | b2 8 KB | d 512 B
// pass 1:    a1_t [8][128][16] f16 32 KB | b2_t [8][256][16] f16 64 KB | dm_t [8][128] f32 4 KB | ad_t [8][256] f32 8 KB
#define GW_B_OFF (2u * GW_A_STAGE * 2u)              // bytes
#define GW_SIDE_OFF (GW_B_OFF + 2u * GW_B_STAGE)     // bytes
static const uint32_t GW_LDS_BYTES = 32768u + 65536u + 4096u + 8192u;

// Eight int8 activations (two dwords) -> eight f16, exact: with u = x + 128 (the sign bit flipped),
// 0x6400 | u is the f16 1024 + u, and 1024 + u - 1152 = x.
__device__ __forceinline__ half8 gw_i8_to_f16(uint32_t w0, uint32_t w1) {
  union { uint32_t u[4]; half8 h; half2v p[4]; } r;
  const uint32_t u0 = w0 ^ 0x80808080u, u1 = w1 ^ 0x80808080u;
  r.u[0] = __builtin_amdgcn_perm(0x64646464u, u0, 0x04010400u);  // (b0, 0x64, b1, 0x64)
  r.u[1] = __builtin_amdgcn_perm(0x64646464u, u0, 0x04030402u);
  r.u[2] = __builtin_amdgcn_perm(0x64646464u, u1, 0x04010400u);
  r.u[3] = __builtin_amdgcn_perm(0x64646464u, u1, 0x04030402u);
  const half2v k = {(_Float16)-1152.0f, (_Float16)-1152.0f};
#pragma unroll
  for (int i = 0; i < 4; i++) r.p[i] = r.p[i] + k;
  return r.h;
}

__global__ __launch_bounds__(768) void ogm_gemm_q4k_wide_kernel(GemmParams p) {
  extern __shared__ __align__(16) uint8_t lds[];
  _Float16 *A_l = (_Float16 *)lds;                       // [2][128][72]
  uint8_t *B_l = lds + GW_B_OFF;                         // [2][256][80]
  _Float16 *a2_l = (_Float16 *)(lds + GW_SIDE_OFF);      // [128 rows][16]: 512*sc_j | 8*sc_j
  _Float16 *b2_l = a2_l + 128 * 16;                      // [256 tokens][16]: bh_j | bl_j
  float *d_l = (float *)(b2_l + 256 * 16);               // [128]
  _Float16 *a1_t = (_Float16 *)lds;                      // pass 1: 64*m_j | m_j per (super-block, row)
  _Float16 *b2_t = (_Float16 *)(lds + 32768);            //         bh_j | bl_j per (super-block, token)
  float *dm_t = (float *)(lds + 32768 + 65536);          //         dmin per (super-block, row)
  float *ad_t = dm_t + GW_PG * 128;                      //         activation scale per (super-block, token)

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const bool producer = wave >= 8u;
  const uint32_t wr = wave & 1u, wt_ = (wave & 7u) >> 1;   // multiplying wave: row half, token quarter (64)
  const uint32_t t0 = blockIdx.x * GW_BT, r0 = gm_pick_matrix(p, blockIdx.y) * GM_BN;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;

  auto row_off = [&](uint32_t row) -> uint32_t {
    row = min(row, p.out_dim - 1u);
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    return rb * p.nct * 9216u + r * 16u;
  };
  auto sb_off = [&](uint32_t s) -> uint32_t {
    const uint32_t ct = s >> p.c_shift, cl = s & ((1u << p.c_shift) - 1u);
    return ct * 9216u + (cl << p.r_shift) * 16u;
  };

  // multiplying wave: rows ra (+32), local tokens tl (+32)
  const uint32_t ra = 64u * wr + l32, tl = 64u * wt_ + l32;
  float16v y00, y01, y10, y11;   // y<row tile><token tile>
#pragma unroll
  for (int r = 0; r < 16; r++) y00[r] = y01[r] = y10[r] = y11[r] = 0.0f;
  const float16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // ---------------- pass 1: acc -= (ad * dmin) * sum_j m_j * bsum_j, all super-blocks first
#pragma unroll 1
  for (uint32_t g0 = 0; g0 < p.nsb; g0 += GW_PG) {
    const uint32_t ng = min(GW_PG, p.nsb - g0);
    for (uint32_t i = tid; i < ng * 256u; i += 768u) {          // (super-block, row, half of the operand)
      const uint32_t sb = i >> 8, row = (i >> 1) & 127u, hf = i & 1u;
      const uint4 hd = *(const uint4 *)(p.wt + (row_off(r0 + row) + sb_off(g0 + sb)));
      uint32_t mna, mnb;
      q4k_mins(hd, mna, mnb);
      *(half8 *)(a1_t + (sb * 128u + row) * 16u + 8u * hf) = side_operand(mna, mnb, hf ? 1.0f : 64.0f);
      if (hf == 0) dm_t[sb * 128u + row] = gm_f16_bits_to_f32(hd.x >> 16);
    }
    for (uint32_t i = tid; i < ng * 512u; i += 768u) {          // (super-block, token, half)
      const uint32_t sb = i >> 9, tok = (i >> 1) & 255u, hf = i & 1u;
      const uint32_t t = min(t0 + tok, p.n_tokens - 1u);
      *(uint4 *)(b2_t + (sb * 256u + tok) * 16u + 8u * hf) =
          *(const uint4 *)(p.bs16 + ((t * p.nsb + g0 + sb) * 16u + 8u * hf));
    }
    for (uint32_t i = tid; i < ng * 256u; i += 768u) {
      const uint32_t sb = i >> 8, tok = i & 255u;
      ad_t[sb * 256u + tok] = p.ad[min(t0 + tok, p.n_tokens - 1u) * p.nsb + g0 + sb];
    }
    __syncthreads();
    if (!producer) {
#pragma unroll 1
      for (uint32_t sb = 0; sb < ng; sb++) {
        const half8 a10 = *(const half8 *)(a1_t + (sb * 128u + ra) * 16u + 8u * lh);
        const half8 a11 = *(const half8 *)(a1_t + (sb * 128u + ra + 32u) * 16u + 8u * lh);
        const half8 b20 = *(const half8 *)(b2_t + (sb * 256u + tl) * 16u + 8u * lh);
        const half8 b21 = *(const half8 *)(b2_t + (sb * 256u + tl + 32u) * 16u + 8u * lh);
        const float adv0 = ad_t[sb * 256u + tl], adv1 = ad_t[sb * 256u + tl + 32u];
        const float *dm = dm_t + sb * 128u + 64u * wr + 4u * lh;
#define GW_MIN_TILE(Y, A1, B2, ADV, DMO)                                                   \
  do {                                                                                     \
    const float16v im = __builtin_amdgcn_mfma_f32_32x32x16_f16(A1, B2, zero, 0, 0, 0);     \
    _Pragma("unroll") for (int q4 = 0; q4 < 4; q4++) {                                     \
      const float4 m = *(const float4 *)(dm + (DMO) + 8 * q4);                             \
      Y[4 * q4 + 0] -= ADV * m.x * im[4 * q4 + 0];                                         \
      Y[4 * q4 + 1] -= ADV * m.y * im[4 * q4 + 1];                                         \
      Y[4 * q4 + 2] -= ADV * m.z * im[4 * q4 + 2];                                         \
      Y[4 * q4 + 3] -= ADV * m.w * im[4 * q4 + 3];                                         \
    }                                                                                      \
  } while (0)
        GW_MIN_TILE(y00, a10, b20, adv0, 0);
        GW_MIN_TILE(y01, a10, b21, adv1, 0);
        GW_MIN_TILE(y10, a11, b20, adv0, 32);
        GW_MIN_TILE(y11, a11, b21, adv1, 32);
#undef GW_MIN_TILE
      }
    }
    __syncthreads();   // the tables are rewritten (next group) or become the stage buffers
  }

  // ---------------- pass 2: acc += ad * (d * sum_j sc_j * dot32_j)
  // Feeding roles (256 threads).  Weights: one 16-byte piece of qs per thread and stage (16 low-
  // nibble and 16 high-nibble weights of one row).  Activations: four 16-byte chunks per thread.
  // Once per super-block also the row's header (scales, d) and two chunks of bh | bl.
  const uint32_t rt = tid & 255u;
  const uint32_t arow = rt & 127u, ah = rt >> 7;
  const uint32_t hdo = row_off(r0 + arow), roa = hdo + (1u + ah) * 1024u;
  const uint32_t btok = rt >> 2, bch = rt & 3u;
  const uint32_t bo0 = min(t0 + btok, p.n_tokens - 1u) * p.in_dim + 16u * bch;
  const uint32_t bo1 = min(t0 + btok + 64u, p.n_tokens - 1u) * p.in_dim + 16u * bch;
  const uint32_t bo2 = min(t0 + btok + 128u, p.n_tokens - 1u) * p.in_dim + 16u * bch;
  const uint32_t bo3 = min(t0 + btok + 192u, p.n_tokens - 1u) * p.in_dim + 16u * bch;
  const uint32_t bso = btok * GW_B_ROW + 16u * bch;       // byte offset in a staged activation tile
  const uint32_t aso = arow * GW_A_ROW + 16u * ah;        // f16 offset of chunk 2 ah in a staged weight tile
  const uint32_t tok2 = rt >> 1, hf2 = rt & 1u;
  const uint32_t b2o0 = min(t0 + tok2, p.n_tokens - 1u) * p.nsb * 16u + 8u * hf2;
  const uint32_t b2o1 = min(t0 + tok2 + 128u, p.n_tokens - 1u) * p.nsb * 16u + 8u * hf2;
  // Loads run three stages ahead of the MFMAs (two ahead of their LDS store: a stage is shorter
  // than a trip to memory) through three rotating register sets; stage m uses set m mod 3.
  uint4 qv_0, qv_1, qv_2;
  uint4 bxa_0, bxb_0, bxc_0, bxd_0, bxa_1, bxb_1, bxc_1, bxd_1, bxa_2, bxb_2, bxc_2, bxd_2;
  uint4 hdx = make_uint4(0, 0, 0, 0), b2x0 = make_uint4(0, 0, 0, 0), b2x1 = make_uint4(0, 0, 0, 0);
  uint32_t sca = 0, scb = 0;
  float dnext = 0.0f;

#define GW_LOAD_STAGE(S, G, K)                                                                    \
  do {                                                                                            \
    const uint32_t so_ = sb_off(S);                                                               \
    if ((G) == 0) hdx = *(const uint4 *)(p.wt + (hdo + so_));                                     \
    if ((G) == 1) {                                                                               \
      b2x0 = *(const uint4 *)(p.bs16 + (b2o0 + (S) * 16u));                                        \
      b2x1 = *(const uint4 *)(p.bs16 + (b2o1 + (S) * 16u));                                        \
    }                                                                                             \
    qv_##K = *(const uint4 *)(p.wt + (roa + so_ + 2u * (G) * 1024u));                             \
    const uint32_t ko_ = (S) * 256u + (G) * 64u;                                                  \
    bxa_##K = *(const uint4 *)(p.xq + (bo0 + ko_));                                               \
    bxb_##K = *(const uint4 *)(p.xq + (bo1 + ko_));                                               \
    bxc_##K = *(const uint4 *)(p.xq + (bo2 + ko_));                                               \
    bxd_##K = *(const uint4 *)(p.xq + (bo3 + ko_));                                               \
  } while (0)

#define GW_STORE_STAGE(G, BUF, K)                                                                 \
  do {                                                                                            \
    if ((G) == 0) {                                                                               \
      q4k_scales(hdx, sca, scb);                                                                  \
      dnext = gm_f16_bits_to_f32(hdx.x & 0xFFFFu);                                                \
    }                                                                                             \
    const uint32_t scw_ = (G) < 2 ? sca : scb;                                                    \
    const uint32_t sh_ = ((G) & 1u) * 16u;                                                        \
    const _Float16 slo_ = (_Float16)(float)((scw_ >> sh_) & 0xFFu);                               \
    const _Float16 shi_ = (_Float16)(float)((scw_ >> (sh_ + 8u)) & 0xFFu);                        \
    const half2v sl2_ = {slo_, slo_}, sh2_ = {shi_, shi_};                                        \
    uint4 la_, lb_, ha_, hb_; /* low nibbles of bytes 0..7 and 8..15, then the high nibbles */    \
    dequant8(qv_##K.x, sl2_, sh2_, la_.x, la_.y, ha_.x, ha_.y);                                   \
    dequant8(qv_##K.y, sl2_, sh2_, la_.z, la_.w, ha_.z, ha_.w);                                   \
    dequant8(qv_##K.z, sl2_, sh2_, lb_.x, lb_.y, hb_.x, hb_.y);                                   \
    dequant8(qv_##K.w, sl2_, sh2_, lb_.z, lb_.w, hb_.z, hb_.w);                                   \
    /* piece 1+2g+ah holds qs[32g+16ah ..]: low nibbles are k 16ah.. of the stage, high 32+16ah.. */ \
    _Float16 *ab_ = A_l + (BUF) * GW_A_STAGE;                                                     \
    *(uint4 *)(ab_ + aso) = la_;              /* chunk 2 ah */                                    \
    *(uint4 *)(ab_ + aso + 8u) = lb_;                                                             \
    *(uint4 *)(ab_ + aso + 32u) = ha_;        /* chunk 4 + 2 ah */                                \
    *(uint4 *)(ab_ + aso + 40u) = hb_;                                                            \
    uint8_t *bb_ = B_l + (BUF) * GW_B_STAGE;                                                      \
    /* stored as x + 128: the multiplying waves' conversion starts from unsigned bytes */         \
    *(uint4 *)(bb_ + bso) = bxa_##K;                                                  \
    *(uint4 *)(bb_ + bso + 64u * GW_B_ROW) = bxb_##K;                                 \
    *(uint4 *)(bb_ + bso + 128u * GW_B_ROW) = bxc_##K;                                \
    *(uint4 *)(bb_ + bso + 192u * GW_B_ROW) = bxd_##K;                                \
    if ((G) == 1) {                                                                               \
      /* side tables of this super-block: their last readers are two barriers behind, their      \
         next readers two barriers ahead; the two threads of a row write the same d */           \
      *(half8 *)(a2_l + arow * 16u + 8u * ah) = side_operand(sca, scb, ah ? 8.0f : 512.0f);       \
      d_l[arow] = dnext;                                                                          \
      *(uint4 *)(b2_l + tok2 * 16u + 8u * hf2) = b2x0;                                            \
      *(uint4 *)(b2_l + (tok2 + 128u) * 16u + 8u * hf2) = b2x1;                                   \
    }                                                                                             \
  } while (0)

#define GW_PRODUCE(G, KL, KS)                                                                     \
  do {                                                                                            \
    /* past the end the last super-block is loaded again and parked in the idle buffer */        \
    GW_LOAD_STAGE(min((G) < 1 ? s : s + 1u, p.nsb - 1u), (uint32_t)(((G) + 3) & 3), KL);          \
    GW_STORE_STAGE((uint32_t)(((G) + 1) & 3), ((G) & 1u) ^ 1u, KS);                               \
    __syncthreads();                                                                              \
  } while (0)

  if (producer) {
    // the feeding wave of a SIMD has little to do per stage but everybody waits for it at the
    // barrier: let it go first
    GW_LOAD_STAGE(0u, 0u, 0);
    GW_LOAD_STAGE(0u, 1u, 1);
    GW_LOAD_STAGE(0u, 2u, 2);
    GW_STORE_STAGE(0u, 0u, 0);
  }
  __syncthreads();

  if (producer) {
#define GW_PRODUCE_SB(K0, K1, K2)                                                                 \
  do {                                                                                            \
    GW_PRODUCE(0, K0, K1);   /* loads stage 4s+3, parks stage 4s+1 */                             \
    GW_PRODUCE(1, K1, K2);                                                                        \
    GW_PRODUCE(2, K2, K0);                                                                        \
    GW_PRODUCE(3, K0, K1);                                                                        \
    s++;                                                                                          \
  } while (0)
    uint32_t s = 0;
    while (s < p.nsb) {
      GW_PRODUCE_SB(0, 1, 2);
      if (s >= p.nsb) break;
      GW_PRODUCE_SB(1, 2, 0);
      if (s >= p.nsb) break;
      GW_PRODUCE_SB(2, 0, 1);
    }
#undef GW_PRODUCE_SB
    return;
  }
#undef GW_LOAD_STAGE
#undef GW_STORE_STAGE
#undef GW_PRODUCE

  // ---- multiplying waves
  const uint32_t tk0 = min(t0 + tl, p.n_tokens - 1u), tk1 = min(t0 + tl + 32u, p.n_tokens - 1u);
  const uint32_t aro = ra * GW_A_ROW + 16u * lh;   // f16 offset of chunk 2 lh of row ra
  const uint32_t bro = tl * GW_B_ROW + 16u * lh;   // byte offset of chunk lh of token tl
  float16v c00, c01, c10, c11;
  float adv0 = 0.0f, adv1 = 0.0f;

#define GW_CONSUME(G)                                                                             \
  do {                                                                                            \
    const uint32_t buf = (G) & 1u;                                                                \
    if ((G) == 0) {                                                                               \
      adv0 = p.ad[tk0 * p.nsb + s];                                                               \
      adv1 = p.ad[tk1 * p.nsb + s];                                                               \
    }                                                                                             \
    const _Float16 *ab = A_l + buf * GW_A_STAGE;                                                  \
    const uint8_t *bb = B_l + buf * GW_B_STAGE;                                                   \
    _Pragma("unroll") for (int m = 0; m < 2; m++) {                                               \
      const uint4 bq0 = *(const uint4 *)(bb + bro + 32u * m);                                     \
      const uint4 bq1 = *(const uint4 *)(bb + bro + 32u * GW_B_ROW + 32u * m);                    \
      _Pragma("unroll") for (int e = 0; e < 2; e++) {                                             \
        /* chunk 4 m + 2 lh + e of rows ra and ra + 32 */                                         \
        const half8 a0 = *(const half8 *)(ab + aro + 32u * m + 8u * e);                           \
        const half8 a1 = *(const half8 *)(ab + aro + 32u * GW_A_ROW + 32u * m + 8u * e);          \
        /* the super-block's first step starts fresh accumulators */                             \
        const bool first = (G) == 0 && m == 0 && e == 0;                                          \
        const half8 b0 = e ? gw_i8_to_f16(bq0.z, bq0.w) : gw_i8_to_f16(bq0.x, bq0.y);             \
        c00 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b0, first ? zero : c00, 0, 0, 0);        \
        c10 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b0, first ? zero : c10, 0, 0, 0);        \
        const half8 b1 = e ? gw_i8_to_f16(bq1.z, bq1.w) : gw_i8_to_f16(bq1.x, bq1.y);             \
        c01 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b1, first ? zero : c01, 0, 0, 0);        \
        c11 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b1, first ? zero : c11, 0, 0, 0);        \
        asm volatile("" ::: "memory");  /* later steps' LDS reads stay behind */                  \
      }                                                                                           \
    }                                                                                             \
    if ((G) == 3) {                                                                               \
      const half8 b20 = *(const half8 *)(b2_l + tl * 16u + 8u * lh);                              \
      const half8 b21 = *(const half8 *)(b2_l + (tl + 32u) * 16u + 8u * lh);                      \
      const half8 a20 = *(const half8 *)(a2_l + ra * 16u + 8u * lh);                              \
      const half8 a21 = *(const half8 *)(a2_l + (ra + 32u) * 16u + 8u * lh);                      \
      const float *dp = d_l + 64u * wr + 4u * lh;                                                 \
      GW_SB_TILE(y00, c00, a20, b20, adv0, 0);                                                    \
      GW_SB_TILE(y01, c01, a20, b21, adv1, 0);                                                    \
      GW_SB_TILE(y10, c10, a21, b20, adv0, 32);                                                   \
      GW_SB_TILE(y11, c11, a21, b21, adv1, 32);                                                   \
    }                                                                                             \
    __syncthreads();                                                                              \
  } while (0)

  // isum = c + corr (one rounding of the exact integer), then the reference's f32 steps
#define GW_SB_TILE(Y, C, A2, B2, ADV, DO)                                                         \
  do {                                                                                            \
    const float16v corr = __builtin_amdgcn_mfma_f32_32x32x16_f16(A2, B2, zero, 0, 0, 0);          \
    _Pragma("unroll") for (int q4 = 0; q4 < 4; q4++) {                                            \
      const float4 d = *(const float4 *)(dp + (DO) + 8 * q4);                                     \
      Y[4 * q4 + 0] += ADV * (d.x * (C[4 * q4 + 0] + corr[4 * q4 + 0]));                          \
      Y[4 * q4 + 1] += ADV * (d.y * (C[4 * q4 + 1] + corr[4 * q4 + 1]));                          \
      Y[4 * q4 + 2] += ADV * (d.z * (C[4 * q4 + 2] + corr[4 * q4 + 2]));                          \
      Y[4 * q4 + 3] += ADV * (d.w * (C[4 * q4 + 3] + corr[4 * q4 + 3]));                          \
    }                                                                                             \
  } while (0)

#pragma unroll 1
  for (uint32_t s = 0; s < p.nsb; s++) {
    GW_CONSUME(0);
    GW_CONSUME(1);
    GW_CONSUME(2);
    GW_CONSUME(3);
  }
#undef GW_CONSUME
#undef GW_SB_TILE

  // ---------------- store: a lane holds one token column per token tile and its rows in runs of four
  const bool vec = (p.out_dim & 3u) == 0;
#define GW_STORE_TILE(Y, TI, RI)                                                                  \
  do {                                                                                            \
    const uint32_t t = t0 + tl + 32u * (TI);                                                      \
    if (t < p.n_tokens) {                                                                         \
      _Pragma("unroll") for (int q4 = 0; q4 < 4; q4++) {                                          \
        const uint32_t row = r0 + 64u * wr + 32u * (RI) + 8u * q4 + 4u * lh;                      \
        float *dst = p.y + (size_t)t * p.out_dim + row;                                           \
        if (vec && row + 3u < p.out_dim) {                                                        \
          *(float4 *)dst = make_float4(Y[4 * q4], Y[4 * q4 + 1], Y[4 * q4 + 2], Y[4 * q4 + 3]);   \
        } else {                                                                                  \
          _Pragma("unroll") for (int e = 0; e < 4; e++)                                           \
            if (row + e < p.out_dim) dst[e] = Y[4 * q4 + e];                                      \
        }                                                                                         \
      }                                                                                           \
    }                                                                                             \
  } while (0)
  GW_STORE_TILE(y00, 0, 0);
  GW_STORE_TILE(y01, 1, 0);
  GW_STORE_TILE(y10, 0, 1);
  GW_STORE_TILE(y11, 1, 1);
#undef GW_STORE_TILE
}

// ------------------------------------------------------------------------------------------
// The symmetric per-32 types (Q8_0, Q5_0, Q4_0, IQ4_NL): the flat-activation GEMM
// (dot_flat_pair, engine/vecdot.rs:2598-2629): acc += (ad * dw) * dot32 per 32-block.
//
// A block's integer dot is exact on the matrix cores: weights and activations are int8 values as
// f16, a 32-long sum is at most 32 * 127 * 127 < 2^24.  Each block (two K = 16 MFMA steps) starts a
// fresh accumulator and ends with the reference's f32 step, so the f32 work per MFMA is eight times
// Q4_K's: this kernel is bound by the vector pipe, not by the matrix cores.
//
// Workgroup = 128 rows x 128 tokens, twelve waves: eight multiplying (64 rows x 32 tokens each),
// four feeding.  A stage is 64 k = two blocks.  LDS rows are padded by one chunk (see the wide
// Q4_K kernel); activations stay int8 in LDS.  Loads run three stages ahead of the MFMAs.

struct GemmFlatParams {
  const uint8_t *wt;      // tile-planar weights
  const int8_t *xq;       // [T][in_dim] int8 activations
  const float *ad;        // [T][in_dim / 32] activation scales
  float *y;               // [T][out_dim]
  uint32_t in_dim, out_dim, n_tokens, nblk;   // nblk = in_dim / 32 (even)
  uint32_t c_shift, r_shift, nct;             // tiles of R = 1 << r_shift rows x C = 1 << c_shift blocks
};

#define GF_A_ROW 72u                       // f16 per staged weight row (64 + one chunk of padding)
#define GF_B_ROW 80u                       // bytes per staged activation row
#define GF_A_STAGE (128u * GF_A_ROW)       // f16
#define GF_B_STAGE (128u * GF_B_ROW)       // bytes

// KIND 0: Q4_0, 1: Q5_0, 2: IQ4_NL, 3: Q8_0
template <int KIND>
__global__ __launch_bounds__(768) void ogm_gemm_flat_kernel(GemmFlatParams p) {
  constexpr uint32_t PIECES = KIND == 3 ? 2u : 1u;
  constexpr uint32_t TAIL = KIND == 1 ? 6u : 2u;
  constexpr uint32_t TILE = 64u * (16u * PIECES + TAIL);
  __shared__ __align__(16) _Float16 A_l[2 * GF_A_STAGE];   // [2][128][72]
  __shared__ __align__(16) uint8_t B_l[2 * GF_B_STAGE];    // [2][128][80]
  __shared__ __align__(16) float dw_l[2 * 2 * 128];        // [2][block of the stage][128 rows]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const bool producer = wave >= 8u;
  const uint32_t wr = wave & 1u, wt_ = (wave & 7u) >> 1;   // multiplying wave: row half, token quarter
  const uint32_t t0 = blockIdx.x * 128u, r0 = blockIdx.y * 128u;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const uint32_t n_st = p.nblk >> 1;

  if (producer) {
    // ---- feeding waves: one block of one row per thread and stage, two activation chunks
    const uint32_t rt = tid & 255u;
    const uint32_t arow = rt & 127u, abl = rt >> 7;
    const uint32_t row = min(r0 + arow, p.out_dim - 1u);
    const uint32_t rb = row >> p.r_shift, rr = row & ((1u << p.r_shift) - 1u);
    const uint32_t tile_row = rb * p.nct * TILE;
    // unit (row, block b): tile (b >> c_shift), lane ((b & (C - 1)) << r_shift) + rr
    auto unit_off = [&](uint32_t b, uint32_t *tail) -> uint32_t {
      const uint32_t to = tile_row + (b >> p.c_shift) * TILE;
      const uint32_t ln = ((b & ((1u << p.c_shift) - 1u)) << p.r_shift) + rr;
      *tail = to + PIECES * 1024u + ln * TAIL;
      return to + ln * 16u;
    };
    const uint32_t btok0 = rt >> 2, bch = rt & 3u;   // chunk i: token btok0 + 64 i, 16-byte chunk bch
    const uint32_t bo0 = min(t0 + btok0, p.n_tokens - 1u) * p.in_dim + 16u * bch;
    const uint32_t bo1 = min(t0 + btok0 + 64u, p.n_tokens - 1u) * p.in_dim + 16u * bch;
    const uint32_t bso = btok0 * GF_B_ROW + 16u * bch;
    const uint32_t aso = arow * GF_A_ROW + 32u * abl;   // f16 offset of the block's first chunk

    uint4 qa_0, qa_1, qa_2, qb_0, qb_1, qb_2;          // weight pieces (qb only for Q8_0)
    uint32_t tl_0, tl_1, tl_2, th_0, th_1, th_2;       // tail: d16 (and qh for Q5_0)
    uint4 bx_0, bx_1, bx_2, by_0, by_1, by_2;          // activation chunks

#define GF_LOAD(ST, K)                                                                             \
  do {                                                                                             \
    const uint32_t st_ = min((uint32_t)(ST), n_st - 1u);                                           \
    uint32_t tail_;                                                                                \
    const uint32_t uo_ = unit_off(2u * st_ + abl, &tail_);                                         \
    qa_##K = *(const uint4 *)(p.wt + uo_);                                                         \
    if (KIND == 3) qb_##K = *(const uint4 *)(p.wt + uo_ + 1024u);                                  \
    const uint16_t *tp_ = (const uint16_t *)(p.wt + tail_);                                        \
    tl_##K = tp_[0];                                                                               \
    th_##K = KIND == 1 ? ((uint32_t)tp_[1] | ((uint32_t)tp_[2] << 16)) : 0u;                       \
    bx_##K = *(const uint4 *)(p.xq + (bo0 + st_ * 64u));                                           \
    by_##K = *(const uint4 *)(p.xq + (bo1 + st_ * 64u));                                           \
  } while (0)

#define GF_STORE(BUF, K)                                                                           \
  do {                                                                                             \
    uint32_t w_[8]; /* the block's 32 int8 weights, k order */                                     \
    if (KIND == 3) {                                                                               \
      w_[0] = qa_##K.x; w_[1] = qa_##K.y; w_[2] = qa_##K.z; w_[3] = qa_##K.w;                      \
      w_[4] = qb_##K.x; w_[5] = qb_##K.y; w_[6] = qb_##K.z; w_[7] = qb_##K.w;                      \
    } else {                                                                                       \
      const uint32_t q_[4] = {qa_##K.x, qa_##K.y, qa_##K.z, qa_##K.w};                             \
      _Pragma("unroll") for (int k_ = 0; k_ < 4; k_++) {                                           \
        w_[k_] = ogm_nib32_weights<KIND>(q_[k_] & 0x0F0F0F0Fu, (th_##K >> (4 * k_)) & 0xFu);       \
        w_[4 + k_] = ogm_nib32_weights<KIND>((q_[k_] >> 4) & 0x0F0F0F0Fu,                          \
                                             (th_##K >> (16 + 4 * k_)) & 0xFu);                    \
      }                                                                                            \
    }                                                                                              \
    _Float16 *ab_ = A_l + (BUF) * GF_A_STAGE + aso;                                                \
    _Pragma("unroll") for (int c_ = 0; c_ < 4; c_++)                                               \
      *(half8 *)(ab_ + 8 * c_) = gw_i8_to_f16(w_[2 * c_], w_[2 * c_ + 1]);                         \
    dw_l[(BUF) * 256u + abl * 128u + arow] = gm_f16_bits_to_f32(tl_##K);                           \
    uint8_t *bb_ = B_l + (BUF) * GF_B_STAGE + bso;                                                 \
    *(uint4 *)(bb_) = bx_##K;                                                                      \
    *(uint4 *)(bb_ + 64u * GF_B_ROW) = by_##K;                                                     \
  } while (0)

    // stage m uses register set m mod 3; at the barrier of stage st the loads of st + 3 are
    // requested and stage st + 1 is parked in the buffer the multiplying waves are not reading
#define GF_PRODUCE(KL, KS)                                                                         \
  do {                                                                                             \
    GF_LOAD(st + 3u, KL);                                                                          \
    GF_STORE((st + 1u) & 1u, KS);                                                                  \
    __syncthreads();                                                                               \
  } while (0)

    GF_LOAD(0u, 0);
    GF_LOAD(1u, 1);
    GF_LOAD(2u, 2);
    GF_STORE(0u, 0);
    __syncthreads();
    uint32_t st = 0;
    while (true) {
      GF_PRODUCE(0, 1);
      if (++st == n_st) break;
      GF_PRODUCE(1, 2);
      if (++st == n_st) break;
      GF_PRODUCE(2, 0);
      if (++st == n_st) break;
    }
#undef GF_LOAD
#undef GF_STORE
#undef GF_PRODUCE
    return;
  }

  // ---- multiplying waves: rows ra (+32), tokens tl
  const uint32_t ra = 64u * wr + l32, tl = 32u * wt_ + l32;
  const uint32_t tk = min(t0 + tl, p.n_tokens - 1u);
  const uint32_t aro = ra * GF_A_ROW + 16u * lh;    // f16 offset of chunk 2 lh of row ra
  const uint32_t bro = tl * GF_B_ROW + 16u * lh;    // byte offset of the lane half's 16 bytes
  const float *adp = p.ad + (size_t)tk * p.nblk;
  float16v y0, y1;
#pragma unroll
  for (int r = 0; r < 16; r++) y0[r] = y1[r] = 0.0f;
  const float16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float2 adv = *(const float2 *)adp;   // the two blocks of stage 0
  __syncthreads();
#pragma unroll 1
  for (uint32_t st = 0; st < n_st; st++) {
    const uint32_t buf = st & 1u;
    const float2 adn = *(const float2 *)(adp + 2u * min(st + 1u, n_st - 1u));
    const _Float16 *ab = A_l + buf * GF_A_STAGE + aro;
    const uint8_t *bb = B_l + buf * GF_B_STAGE + bro;
    const float *dwp = dw_l + buf * 256u + 64u * wr + 4u * lh;
#pragma unroll
    for (int bl = 0; bl < 2; bl++) {
      // the lane's 16 activations of this block: MFMA step kk takes bytes 8 kk .. 8 kk + 7
      const uint4 bq = *(const uint4 *)(bb + 32u * bl);
      float16v c0, c1;
#pragma unroll
      for (int kk = 0; kk < 2; kk++) {
        const half8 a0 = *(const half8 *)(ab + 32u * bl + 8u * kk);
        const half8 a1 = *(const half8 *)(ab + 32u * GF_A_ROW + 32u * bl + 8u * kk);
        const half8 b = kk ? gw_i8_to_f16(bq.z, bq.w) : gw_i8_to_f16(bq.x, bq.y);
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b, kk ? c0 : zero, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b, kk ? c1 : zero, 0, 0, 0);
      }
      // acc += d * s * dot32 (vecdot.rs:2622): (ad * dw) * (f32)isum
      const float ad = bl ? adv.y : adv.x;
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const float4 d0 = *(const float4 *)(dwp + 128 * bl + 8 * q4);
        const float4 d1 = *(const float4 *)(dwp + 128 * bl + 32 + 8 * q4);
        y0[4 * q4 + 0] += ad * d0.x * c0[4 * q4 + 0];
        y0[4 * q4 + 1] += ad * d0.y * c0[4 * q4 + 1];
        y0[4 * q4 + 2] += ad * d0.z * c0[4 * q4 + 2];
        y0[4 * q4 + 3] += ad * d0.w * c0[4 * q4 + 3];
        y1[4 * q4 + 0] += ad * d1.x * c1[4 * q4 + 0];
        y1[4 * q4 + 1] += ad * d1.y * c1[4 * q4 + 1];
        y1[4 * q4 + 2] += ad * d1.z * c1[4 * q4 + 2];
        y1[4 * q4 + 3] += ad * d1.w * c1[4 * q4 + 3];
      }
    }
    adv = adn;
    __syncthreads();
  }

  // ---------------- store: a lane holds one token column and its rows in runs of four
  const uint32_t t = t0 + tl;
  if (t < p.n_tokens) {
    const bool vec = (p.out_dim & 3u) == 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const float16v &yy = i ? y1 : y0;
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const uint32_t row = r0 + 64u * wr + 32u * i + 8u * q4 + 4u * lh;
        float *dst = p.y + (size_t)t * p.out_dim + row;
        if (vec && row + 3u < p.out_dim) {
          *(float4 *)dst = make_float4(yy[4 * q4], yy[4 * q4 + 1], yy[4 * q4 + 2], yy[4 * q4 + 3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++)
            if (row + e < p.out_dim) dst[e] = yy[4 * q4 + e];
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Q6_K (gemm_k_q6_k, engine/vecdot.rs:2352-2398): acc += ad * (d * sum_g sc_g * dot16(q_g - 32, x_g))
// over the 16 groups of a super-block, sc_g a signed byte.
//
// sc_g * (q - 32) reaches 4096 and is not exact in f16, so the scale is split in base 16,
// sc = 16 a + b with a = sc >> 4 in [-8, 7] and b = sc & 15: the operands a*(q-32) (|.| <= 256)
// and b*(q-32) (|.| <= 480) are exact, their 256-long chains stay below 2^24
// (256*127*256 = 8.3e6, 480*127*256 = 1.56e7), and isum = 16 * c_hi + c_lo is an exact scaling
// by a power of two followed by one f32 add of exact integers: the rounding of `isum as f32`.
//
// Same tiling as the Q4_K kernel: eight waves, 128 rows x 128 tokens, k in stages of 64.  A thread
// stages one group of 16 weights (one ql piece, one qh piece, one scale) into both operand tiles.
// Block layout (quant.rs:744-787): element 128h + 32r + 16k + j of a super-block has its low four
// bits in ql[64h + 32(r&1) + 16k + j] (low nibble for r < 2, high for r >= 2), bits 4..5 in
// qh[32h + 16k + j] >> 2r, and scale sc[8h + 2r + k].

//
// The same two chains carry the other K-quants whose scaled weights leave f16's exact range:
//   Q3_K (a KKind::Q6K row, vecdot.rs:2100-2117): 16 groups with scales sc - 32 in [-32, 31] and
//     weights in [-4, 3]; element 32p + l has its low two bits in qs[32(p/4) + l] >> 2(p%4) and its
//     third bit, stored inverted, in bit p of hmask[l] (quant.rs:841-871).
//   Q5_K (a KKind::Q4K row, vecdot.rs:2064-2088): 8 sub-blocks of 32 with scales in [0, 63] and
//     unsigned weights in [0, 31] (nibble of qs[32(j/2) + l], fifth bit = bit j of qh[l]); chains
//     3*31*127*256 = 3.0e6 and 15*31*127*256 = 1.5e7.  Its -dmin*m correction runs first, over
//     every super-block, as in gemm_k_q4_k (vecdot.rs:2213-2255).

#define GK_Q6K 0
#define GK_Q3K 1
#define GK_Q5K 2

struct Gemm6Params {
  const uint8_t *wt;      // tile-planar weights
  const _Float16 *xh;     // [T][in_dim] int8 activations as f16
  const float *ad;        // [T][nsb] activation scales (per 256)
  const _Float16 *bs16;   // [T][nsb][16]: floor(bsum_j / 64) for j = 0..7, then bsum_j mod 64 (Q5_K's mins)
  float *y;               // [T][out_dim]
  uint32_t in_dim, out_dim, n_tokens, nsb;
  uint32_t c_shift, r_shift, nct;
  // further matrices over the same activations, their row tiles following in grid.y
  uint32_t n_extra;
  const uint8_t *extra_wt[OGM_GEMM_MAX_MATS - 1];
  float *extra_y[OGM_GEMM_MAX_MATS - 1];
  uint32_t extra_out_dim[OGM_GEMM_MAX_MATS - 1];
};

#define G6_LDS_BYTES_STATIC (6u * GM_STAGE_HALFS * 2u + 2u * 128u * 4u)   // three tiles, two buffers each, and d

template <int KIND>
__device__ __forceinline__ void gemm_k2_body(Gemm6Params p) {
  // bytes of a tile of 64 units: Q6_K 13 pieces of 1 KiB and 64 two-byte tails; Q3_K 7 pieces;
  // Q5_K 11 pieces
  constexpr uint32_t G6_TILE_BYTES = KIND == GK_Q6K ? 13440u : KIND == GK_Q3K ? 7168u : 11264u;
  extern __shared__ __align__(16) uint8_t lds[];
  _Float16 *Ah_l = (_Float16 *)lds;                 // [2][128][64]  a * (q - 32)
  _Float16 *Al_l = Ah_l + 2 * GM_STAGE_HALFS;       // [2][128][64]  b * (q - 32)
  _Float16 *B_l = Al_l + 2 * GM_STAGE_HALFS;        // [2][128][64]
  float *d_l = (float *)(B_l + 2 * GM_STAGE_HALFS); // [2][128]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t wr = wave & 1u, wt_ = wave >> 1;   // wave's row half (64 rows) and token quarter (32)
  uint32_t row_tile = blockIdx.y;
#pragma unroll
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {   // the matrix this row tile belongs to
    const uint32_t tiles = (p.out_dim + 127u) / 128u;
    if (m < p.n_extra && row_tile >= tiles) {
      row_tile -= tiles;
      p.wt = p.extra_wt[m];
      p.y = p.extra_y[m];
      p.out_dim = p.extra_out_dim[m];
    } else {
      break;
    }
  }
  const uint32_t t0 = blockIdx.x * GM_BT, r0 = row_tile * GM_BN;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;

  // staging role: row lr_a, group t16 (16 weights) of the stage
  const uint32_t lr_a = (tid >> 6) * 16u + (tid & 15u), t16 = (tid >> 4) & 3u;
  uint32_t unit_off, tail_off;   // the row's unit inside a tile: pieces at unit_off + 1024 p, d at tail_off
  {
    const uint32_t row = min(r0 + lr_a, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    unit_off = rb * p.nct * G6_TILE_BYTES + r * 16u;
    tail_off = rb * p.nct * G6_TILE_BYTES + 13u * 1024u + r * 2u;
  }
  auto sb_tile = [&](uint32_t s) -> uint32_t { return (s >> p.c_shift) * G6_TILE_BYTES; };
  auto sb_lane = [&](uint32_t s) -> uint32_t { return (s & ((1u << p.c_shift) - 1u)) << p.r_shift; };
  const uint32_t btok = tid >> 3, bpart = tid & 7u;   // activation chunk i: token btok + 64 i, part bpart
  const uint32_t bo0 = min(t0 + btok, p.n_tokens - 1u) * p.in_dim + bpart * 8u;
  const uint32_t bo1 = min(t0 + btok + 64u, p.n_tokens - 1u) * p.in_dim + bpart * 8u;
  const uint32_t tko = min(t0 + 32u * wt_ + l32, p.n_tokens - 1u) * p.nsb;

  float16v y0, y1;
  const float16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int r = 0; r < 16; r++) y0[r] = y1[r] = 0.0f;

  if constexpr (KIND == GK_Q5K) {
    // pass 1 (vecdot.rs:2226-2240): acc -= (ad * dmin) * imin for every super-block first, imin =
    // sum_j m_j * bsum_j on the matrix cores exactly as the Q4_K kernel forms it (the two formats
    // share their 16-byte header): operand k 0..7 = 64 m_j against floor(bsum_j / 64), k 8..15 =
    // m_j against bsum_j mod 64, all exact in f16, the sum below 2^24.
    float *dmin_t = (float *)(lds + G6_LDS_BYTES_STATIC);   // [nsb][128]
    auto unit_of = [&](uint32_t row) -> uint32_t {
      row = min(row, p.out_dim - 1u);
      return (row >> p.r_shift) * p.nct * G6_TILE_BYTES + (row & ((1u << p.r_shift) - 1u)) * 16u;
    };
    for (uint32_t i = tid; i < p.nsb * 128u; i += 512u) {
      const uint32_t s = i >> 7, lr = i & 127u;
      const uint32_t h = *(const uint32_t *)(p.wt + (unit_of(r0 + lr) + sb_tile(s) + sb_lane(s) * 16u));
      dmin_t[i] = gm_f16_bits_to_f32(h >> 16);
    }
    __syncthreads();
    const uint32_t ro0 = unit_of(r0 + 64u * wr + l32), ro1 = unit_of(r0 + 64u * wr + 32u + l32);
    const float side_scale = lh ? 1.0f : 64.0f;
    // four super-blocks at a time, so that four sets of loads share one trip to memory
#pragma unroll 1
    for (uint32_t sg = 0; sg < p.nsb; sg += 4u) {
      uint4 hd0[4], hd1[4];
      half8 b2[4];
      float adv1[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const uint32_t su = min(sg + u, p.nsb - 1u);
        const uint32_t so = sb_tile(su) + sb_lane(su) * 16u;
        hd0[u] = *(const uint4 *)(p.wt + (ro0 + so));
        hd1[u] = *(const uint4 *)(p.wt + (ro1 + so));
        b2[u] = *(const half8 *)(p.bs16 + ((tko + su) * 16u + 8u * lh));
        adv1[u] = p.ad[tko + su];
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        if (sg + u < p.nsb) {
          uint32_t mna, mnb;
          q4k_mins(hd0[u], mna, mnb);
          const half8 a10 = side_operand(mna, mnb, side_scale);
          q4k_mins(hd1[u], mna, mnb);
          const half8 a11 = side_operand(mna, mnb, side_scale);
          const float16v im0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a10, b2[u], zero, 0, 0, 0);
          const float16v im1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a11, b2[u], zero, 0, 0, 0);
          const float *dm = dmin_t + (sg + u) * 128u + 64u * wr + 4u * lh;
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++) {
            const float4 m0 = *(const float4 *)(dm + 8 * q4), m1 = *(const float4 *)(dm + 32 + 8 * q4);
            y0[4 * q4 + 0] -= adv1[u] * m0.x * im0[4 * q4 + 0];
            y0[4 * q4 + 1] -= adv1[u] * m0.y * im0[4 * q4 + 1];
            y0[4 * q4 + 2] -= adv1[u] * m0.z * im0[4 * q4 + 2];
            y0[4 * q4 + 3] -= adv1[u] * m0.w * im0[4 * q4 + 3];
            y1[4 * q4 + 0] -= adv1[u] * m1.x * im1[4 * q4 + 0];
            y1[4 * q4 + 1] -= adv1[u] * m1.y * im1[4 * q4 + 1];
            y1[4 * q4 + 2] -= adv1[u] * m1.z * im1[4 * q4 + 2];
            y1[4 * q4 + 3] -= adv1[u] * m1.w * im1[4 * q4 + 3];
          }
        }
      }
    }
    __syncthreads();   // dmin_t is not reused, but the stage buffers below are written next
  }

  // loads run two stages ahead through three rotating register sets
  uint4 ql_0, ql_1, ql_2, qh_0, qh_1, qh_2, bx0_0, bx0_1, bx0_2, bx1_0, bx1_1, bx1_2;
  uint4 hmx = make_uint4(0, 0, 0, 0);   // Q3_K / Q5_K: the thread's piece of the high-bit plane
  uint32_t hmw[4] = {0, 0, 0, 0};
  uint4 scx = make_uint4(0, 0, 0, 0);   // the super-block's 16 scales
  uint32_t d16 = 0;
  uint32_t scw[4] = {0, 0, 0, 0};
  float dnext = 0.0f;

#define G6_LOAD_STAGE(S, G, K)                                                                    \
  do {                                                                                            \
    const uint32_t uo_ = unit_off + sb_tile(S) + sb_lane(S) * 16u;                                \
    const uint32_t h_ = (G) >> 1;                                                                 \
    if constexpr (KIND == GK_Q6K) {                                                               \
      if ((G) == 0) {                                                                             \
        scx = *(const uint4 *)(p.wt + (uo_ + 12u * 1024u));                                       \
        d16 = *(const uint16_t *)(p.wt + (tail_off + sb_tile(S) + sb_lane(S) * 2u));              \
      }                                                                                           \
      ql_##K = *(const uint4 *)(p.wt + (uo_ + (4u * h_ + t16) * 1024u));                          \
      qh_##K = *(const uint4 *)(p.wt + (uo_ + (8u + 2u * h_ + (t16 & 1u)) * 1024u));              \
    } else if constexpr (KIND == GK_Q3K) {                                                        \
      /* pieces: hmask 0..1, qs 2..5, then scales[12] | d | two bytes of padding */               \
      if ((G) == 0) {                                                                             \
        scx = *(const uint4 *)(p.wt + (uo_ + 6u * 1024u));                                        \
        hmx = *(const uint4 *)(p.wt + (uo_ + (t16 & 1u) * 1024u));                                \
      }                                                                                           \
      ql_##K = *(const uint4 *)(p.wt + (uo_ + (2u + 2u * h_ + (t16 & 1u)) * 1024u));              \
      qh_##K = ql_##K;                                                                            \
    } else {                                                                                      \
      /* pieces: d | dmin | scales[12], qh 1..2, qs 3..10 */                                      \
      if ((G) == 0) {                                                                             \
        scx = *(const uint4 *)(p.wt + uo_);                                                       \
        hmx = *(const uint4 *)(p.wt + (uo_ + (1u + (t16 & 1u)) * 1024u));                         \
      }                                                                                           \
      ql_##K = *(const uint4 *)(p.wt + (uo_ + (3u + 2u * (G) + (t16 & 1u)) * 1024u));             \
      qh_##K = ql_##K;                                                                            \
    }                                                                                             \
    const uint32_t ko_ = (S) * 256u + (G) * 64u;                                                  \
    bx0_##K = *(const uint4 *)(p.xh + (bo0 + ko_));                                               \
    bx1_##K = *(const uint4 *)(p.xh + (bo1 + ko_));                                               \
  } while (0)

  // Four bytes of small unsigned values v -> (v - zero point) * a and (v - zero point) * b as f16
  // (zero point 32 for Q6_K, 4 for Q3_K, 0 for Q5_K)
#define G6_DEQ(V, HI01, HI23, LO01, LO23)                                                         \
  do {                                                                                            \
    union { uint32_t u; half2v h; } e_, f_;                                                       \
    e_.u = __builtin_amdgcn_perm(0u, (V), 0x0c010c00u) | 0x64006400u; /* 1024 + v */              \
    f_.u = __builtin_amdgcn_perm(0u, (V), 0x0c030c02u) | 0x64006400u;                             \
    e_.h = e_.h + koff_;                                                                          \
    f_.h = f_.h + koff_;                                                                          \
    union { uint32_t u; half2v h; } o_;                                                           \
    o_.h = e_.h * a2_; HI01 = o_.u;                                                               \
    o_.h = f_.h * a2_; HI23 = o_.u;                                                               \
    o_.h = e_.h * b2_; LO01 = o_.u;                                                               \
    o_.h = f_.h * b2_; LO23 = o_.u;                                                               \
  } while (0)

#define G6_STORE_STAGE(S, G, BUF, K)                                                              \
  do {                                                                                            \
    if ((G) == 0) {                                                                               \
      scw[0] = scx.x; scw[1] = scx.y; scw[2] = scx.z; scw[3] = scx.w;                             \
      hmw[0] = hmx.x; hmw[1] = hmx.y; hmw[2] = hmx.z; hmw[3] = hmx.w;                             \
      if constexpr (KIND == GK_Q6K) dnext = gm_f16_bits_to_f32(d16);                              \
      else if constexpr (KIND == GK_Q3K) dnext = gm_f16_bits_to_f32(scx.w & 0xFFFFu);             \
      else dnext = gm_f16_bits_to_f32(scx.x & 0xFFFFu);                                           \
    }                                                                                             \
    /* scale of group 4G + t16, split as 16 a + b */                                              \
    int sc_;                                                                                      \
    uint32_t zp_;      /* zero point of the stored values, as f16 bits of -(1024 + zero point) */ \
    if constexpr (KIND == GK_Q6K) {                                                               \
      const uint32_t sw_ = (G) == 0 ? scw[0] : (G) == 1 ? scw[1] : (G) == 2 ? scw[2] : scw[3];    \
      sc_ = (int)(int8_t)((sw_ >> (8u * t16)) & 0xFFu);                                           \
      zp_ = 1056u;                                                                                \
    } else if constexpr (KIND == GK_Q3K) {                                                        \
      /* quant.rs:883-897: scale i = 4G + t16 has its low four bits in a nibble of byte i % 8 and \
         its two high bits at bit 2 (i / 4) of byte 8 + i % 4; all biased by 32 */                \
      const uint32_t lw_ = ((G) & 1u) ? scw[1] : scw[0];      /* bytes 4(G&1) .. 4(G&1) + 3 */     \
      const uint32_t low_ = ((lw_ >> (8u * t16)) >> ((G) >= 2 ? 4u : 0u)) & 0xFu;                 \
      const uint32_t high_ = ((scw[2] >> (8u * t16)) >> (2u * (G))) & 3u;                         \
      sc_ = (int)(low_ | (high_ << 4)) - 32;                                                      \
      zp_ = 1028u;                                                                                \
    } else {                                                                                      \
      /* get_scale_min_k4 (quant.rs:653-662) of sub-block j = 2G + t16/2 over scales bytes        \
         q[0..12) = scw[1..3]: sc = q[j] & 63 for j < 4, else (q[j+4] & 15) | ((q[j-4] >> 6) << 4) */ \
      const uint32_t j_ = 2u * (G) + (t16 >> 1);                                                  \
      const uint32_t qa_ = (scw[1] >> (8u * (j_ & 3u))) & 0xFFu;  /* q[j] or q[j-4] */            \
      const uint32_t qb_ = (scw[3] >> (8u * (j_ & 3u))) & 0xFFu;  /* q[j+4] for j >= 4 */         \
      sc_ = (G) < 2 ? (int)(qa_ & 63u) : (int)((qb_ & 15u) | ((qa_ >> 6) << 4));                  \
      zp_ = 1024u;                                                                                \
    }                                                                                             \
    const _Float16 af_ = (_Float16)(float)(sc_ >> 4), bf_ = (_Float16)(float)(sc_ & 15);          \
    const half2v a2_ = {af_, af_}, b2_ = {bf_, bf_};                                              \
    const _Float16 kz_ = (_Float16)(-(float)zp_);                                                 \
    const half2v koff_ = {kz_, kz_};                                                              \
    const uint32_t m4_ = 0x0F0F0F0Fu, m2_ = 0x30303030u;                                          \
    const uint32_t rr_ = 2u * ((G) & 1u) + (t16 >> 1);        /* run of 32 inside the half block */ \
    const uint32_t qlw_[4] = {ql_##K.x, ql_##K.y, ql_##K.z, ql_##K.w};                            \
    const uint32_t qhw_[4] = {qh_##K.x, qh_##K.y, qh_##K.z, qh_##K.w};                            \
    uint32_t hi_[8], lo_[8];                                                                      \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      uint32_t v_;                                                                                \
      if constexpr (KIND == GK_Q6K) {                                                             \
        const uint32_t nib_ = (((G) & 1u) ? (qlw_[w_] >> 4) : qlw_[w_]) & m4_;                    \
        v_ = nib_ | ((((qhw_[w_] >> (2u * rr_)) << 4)) & m2_);                                    \
      } else if constexpr (KIND == GK_Q3K) {                                                      \
        /* run p = 2G + t16/2 of 32: two bits at 2 (p % 4) = 2 rr, third bit = bit p of hmask */  \
        v_ = ((qlw_[w_] >> (2u * rr_)) & 0x03030303u) |                                           \
             (((hmw[w_] >> (2u * (G) + (t16 >> 1))) & 0x01010101u) << 2);                         \
      } else {                                                                                    \
        const uint32_t nib_ = ((t16 >> 1) ? (qlw_[w_] >> 4) : qlw_[w_]) & m4_;                    \
        v_ = nib_ | (((hmw[w_] >> (2u * (G) + (t16 >> 1))) & 0x01010101u) << 4);                  \
      }                                                                                           \
      G6_DEQ(v_, hi_[2 * w_], hi_[2 * w_ + 1], lo_[2 * w_], lo_[2 * w_ + 1]);                     \
    }                                                                                             \
    _Float16 *ah_ = Ah_l + (BUF) * GM_STAGE_HALFS, *al_ = Al_l + (BUF) * GM_STAGE_HALFS;          \
    *(uint4 *)(ah_ + gm_swz(lr_a, 2u * t16)) = make_uint4(hi_[0], hi_[1], hi_[2], hi_[3]);        \
    *(uint4 *)(ah_ + gm_swz(lr_a, 2u * t16 + 1u)) = make_uint4(hi_[4], hi_[5], hi_[6], hi_[7]);   \
    *(uint4 *)(al_ + gm_swz(lr_a, 2u * t16)) = make_uint4(lo_[0], lo_[1], lo_[2], lo_[3]);        \
    *(uint4 *)(al_ + gm_swz(lr_a, 2u * t16 + 1u)) = make_uint4(lo_[4], lo_[5], lo_[6], lo_[7]);   \
    _Float16 *bb_ = B_l + (BUF) * GM_STAGE_HALFS;                                                 \
    *(uint4 *)(bb_ + gm_swz(btok, bpart)) = bx0_##K;                                              \
    *(uint4 *)(bb_ + gm_swz(btok + 64u, bpart)) = bx1_##K;                                        \
    if ((G) == 0) d_l[((S) & 1u) * 128u + lr_a] = dnext; /* the four threads of a row agree */    \
  } while (0)

  // One stage: loads of the stage two ahead, this stage's MFMAs with the next stage's
  // dequantization in their shadow, then, after the super-block's last stage, its f32 step.
#define G6_STAGE(G, KL, KS)                                                                       \
  do {                                                                                            \
    const uint32_t buf = (G) & 1u;                                                                \
    if ((G) == 0) adv = p.ad[tko + s];                                                            \
    /* past the end the last super-block is loaded again and parked in the idle buffer */        \
    G6_LOAD_STAGE(min((G) < 2 ? s : s + 1u, p.nsb - 1u), (uint32_t)(((G) + 2) & 3), KL);          \
    __builtin_amdgcn_sched_barrier(0);                                                            \
    const _Float16 *ah = Ah_l + buf * GM_STAGE_HALFS, *al = Al_l + buf * GM_STAGE_HALFS;          \
    const _Float16 *bb = B_l + buf * GM_STAGE_HALFS;                                              \
    _Pragma("unroll") for (int kk = 0; kk < 4; kk++) {                                            \
      const half8 ah0 = *(const half8 *)(ah + gm_swz(ra, 2u * kk + lh));                          \
      const half8 ah1 = *(const half8 *)(ah + gm_swz(ra + 32u, 2u * kk + lh));                    \
      const half8 al0 = *(const half8 *)(al + gm_swz(ra, 2u * kk + lh));                          \
      const half8 al1 = *(const half8 *)(al + gm_swz(ra + 32u, 2u * kk + lh));                    \
      const half8 b0 = *(const half8 *)(bb + gm_swz(rbk, 2u * kk + lh));                          \
      const bool first_ = (G) == 0 && kk == 0;   /* the super-block starts fresh accumulators */  \
      ch0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah0, b0, first_ ? zero : ch0, 0, 0, 0);        \
      ch1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah1, b0, first_ ? zero : ch1, 0, 0, 0);        \
      cl0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al0, b0, first_ ? zero : cl0, 0, 0, 0);        \
      cl1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al1, b0, first_ ? zero : cl1, 0, 0, 0);        \
    }                                                                                             \
    G6_STORE_STAGE(((G) + 1) < 4 ? s : min(s + 1u, p.nsb - 1u), (uint32_t)(((G) + 1) & 3), buf ^ 1u, KS); \
    __builtin_amdgcn_sched_barrier(0);                                                            \
    if ((G) == 3) {                                                                               \
      /* isum = 16 c_hi + c_lo (one rounding), then the reference's f32 steps */                  \
      const float *dp = d_l + (s & 1u) * 128u + 64u * wr + 4u * lh;                               \
      _Pragma("unroll") for (int q4 = 0; q4 < 4; q4++) {                                          \
        const float4 d0 = *(const float4 *)(dp + 8 * q4), d1 = *(const float4 *)(dp + 32 + 8 * q4); \
        const float d0v[4] = {d0.x, d0.y, d0.z, d0.w}, d1v[4] = {d1.x, d1.y, d1.z, d1.w};         \
        _Pragma("unroll") for (int e = 0; e < 4; e++) {                                           \
          y0[4 * q4 + e] += adv * (d0v[e] * (ch0[4 * q4 + e] * 16.0f + cl0[4 * q4 + e]));         \
          y1[4 * q4 + e] += adv * (d1v[e] * (ch1[4 * q4 + e] * 16.0f + cl1[4 * q4 + e]));         \
        }                                                                                         \
      }                                                                                           \
    }                                                                                             \
    __syncthreads();                                                                              \
  } while (0)

  G6_LOAD_STAGE(0u, 0u, 0);
  G6_LOAD_STAGE(0u, 1u, 1);
  G6_STORE_STAGE(0u, 0u, 0u, 0);
  __syncthreads();

  const uint32_t ra = 64u * wr + l32, rbk = 32u * wt_ + l32;
  // Stages rotate through three register sets while a super-block has four stages, so the set
  // of a stage is (4 s + g) mod 3: three super-blocks make one period of the loop body.
  uint32_t s = 0;
  float16v ch0, ch1, cl0, cl1;
  float adv = 0.0f;
#define G6_SB(K0, K1, K2)            /* sets of stages g = 0, 1, 2; g = 3 uses K0 again */          \
  do {                                                                                            \
    G6_STAGE(0, K2, K1);   /* loads stage 4s+2 into the set two ahead, parks stage 4s+1 */        \
    G6_STAGE(1, K0, K2);                                                                          \
    G6_STAGE(2, K1, K0);                                                                          \
    G6_STAGE(3, K2, K1);                                                                          \
    s++;                                                                                          \
  } while (0)
  while (s < p.nsb) {
    G6_SB(0, 1, 2);                 // stages 4s..4s+3 in sets 0 1 2 0
    if (s >= p.nsb) break;
    G6_SB(1, 2, 0);                 // 1 2 0 1
    if (s >= p.nsb) break;
    G6_SB(2, 0, 1);                 // 2 0 1 2
  }
#undef G6_SB
#undef G6_STAGE
#undef G6_STORE_STAGE
#undef G6_LOAD_STAGE
#undef G6_DEQ

  const uint32_t t = t0 + 32u * wt_ + l32;
  if (t < p.n_tokens) {
    const bool vec = (p.out_dim & 3u) == 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const float16v &yy = i ? y1 : y0;
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const uint32_t row = r0 + 64u * wr + 32u * i + 8u * q4 + 4u * lh;
        float *dst = p.y + (size_t)t * p.out_dim + row;
        if (vec && row + 3u < p.out_dim) {
          *(float4 *)dst = make_float4(yy[4 * q4], yy[4 * q4 + 1], yy[4 * q4 + 2], yy[4 * q4 + 3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++)
            if (row + e < p.out_dim) dst[e] = yy[4 * q4 + e];
        }
      }
    }
  }
}

__global__ __launch_bounds__(512) void ogm_gemm_q6k_kernel(Gemm6Params p) { gemm_k2_body<GK_Q6K>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q3k_kernel(Gemm6Params p) { gemm_k2_body<GK_Q3K>(p); }
__global__ __launch_bounds__(512) void ogm_gemm_q5k_kernel(Gemm6Params p) { gemm_k2_body<GK_Q5K>(p); }

static const uint32_t G6_LDS_BYTES = G6_LDS_BYTES_STATIC;

static const uint32_t GM_LDS_BYTES = 4 * GM_STAGE_HALFS * 2 + 2 * 128 * 16 * 2 + 128 * 4;
static const uint32_t GM_LDS_MAX = 160 * 1024;   // LDS of a CU

size_t ogm_gemm_xh_bytes(uint32_t in_dim, uint32_t n_tokens) {
  // f16 activations, then the (bh, bl) pairs: 16 f16 per (token, super-block)
  return (size_t)in_dim * n_tokens * 2 + (size_t)(in_dim / 256) * n_tokens * 32;
}

static bool is_flat32(uint32_t t) { return t == OGM_Q8_0 || t == OGM_Q5_0 || t == OGM_Q4_0 || t == OGM_IQ4_NL; }

bool ogm_gemm_supported(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t n_tokens) {
  // the kernels address weights and activations with 32-bit byte offsets
  const uint64_t lim = 0xFFFFFFFFull;
  if (is_flat32(ggml_type)) {
    // two blocks per stage
    if (in_dim == 0 || in_dim % 64u != 0) return false;
    OgmLayout l;
    ogm_layout_for(ggml_type, &l);
    return (uint64_t)ogm_tiling_for(in_dim / 32u, out_dim).nrb * 64u * (in_dim / 32u) * l.block_bytes <= lim &&
           (uint64_t)in_dim * n_tokens <= lim;
  }
  if ((ggml_type != OGM_Q4_K && ggml_type != OGM_Q6_K && ggml_type != OGM_Q3_K && ggml_type != OGM_Q5_K) ||
      in_dim == 0 || in_dim % 256u != 0)
    return false;
  // Q4_K's pass 1 keeps one f32 per (row, super-block) of the workgroup in LDS
  if (ggml_type == OGM_Q4_K && GM_LDS_BYTES + (size_t)(in_dim / 256u) * 512u > GM_LDS_MAX) return false;
  if (ggml_type == OGM_Q5_K && G6_LDS_BYTES + (size_t)(in_dim / 256u) * 512u > GM_LDS_MAX) return false;
  const uint64_t block = ggml_type == OGM_Q4_K ? 144u : ggml_type == OGM_Q6_K ? 210u : ggml_type == OGM_Q3_K ? 112u : 176u;
  return (uint64_t)ogm_tiling_for(in_dim / 256u, out_dim).nrb * 64u * (in_dim / 256u) * block <= lim &&
         (uint64_t)in_dim * n_tokens * 2u <= lim;
}

size_t ogm_gemm_plane_bytes(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim) {
  if ((ggml_type != OGM_Q4_K && ggml_type != OGM_Q6_K && ggml_type != OGM_Q3_K && ggml_type != OGM_Q5_K) ||
      in_dim == 0 || in_dim % 256u != 0 || out_dim == 0)
    return 0;
  const uint32_t npl = ggml_type == OGM_Q3_K ? 1u : 2u;
  return gp_plane_offset((out_dim + 63u) / 64u, in_dim / 256u, 0, 0, 0, npl);
}

hipError_t ogm_gemm_build_planes(uint32_t ggml_type, const uint8_t *wt, uint32_t in_dim, uint32_t out_dim,
                                 uint8_t *planes, hipStream_t stream) {
  if (ogm_gemm_plane_bytes(ggml_type, in_dim, out_dim) == 0 || !wt || !planes) return hipErrorInvalidValue;
  GemmPlaneBuildParams p;
  p.wt = wt;
  p.planes = planes;
  p.out_dim = out_dim;
  p.nsb = in_dim / 256u;
  const OgmTiling tl = ogm_tiling_for(p.nsb, out_dim);
  p.c_shift = tl.C == 4 ? 2 : (tl.C == 2 ? 1 : 0);
  p.r_shift = 6 - p.c_shift;
  p.nct = tl.nct;
  const dim3 grid(4u * p.nsb, (out_dim + 63u) / 64u);
  if (grid.y > 65535u) return hipErrorInvalidValue;
  switch (ggml_type) {
    case OGM_Q6_K: hipLaunchKernelGGL(ogm_gemm_build_planes_kernel<GP_Q6K>, grid, dim3(256), 0, stream, p); break;
    case OGM_Q3_K: hipLaunchKernelGGL(ogm_gemm_build_planes_kernel<GP_Q3K>, grid, dim3(256), 0, stream, p); break;
    case OGM_Q4_K: hipLaunchKernelGGL(ogm_gemm_build_planes_kernel<GP_Q4K>, grid, dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL(ogm_gemm_build_planes_kernel<GP_Q5K>, grid, dim3(256), 0, stream, p); break;
  }
  return hipGetLastError();
}

// Which family of kernels a K-quant launch takes: 0 the f16 kernels, 1 the int8 multiply-add kernel,
// 2 the small-batch kernel, 3 a tiled int8 plane kernel.
static int gemm_k_path(const OgmGemmArgs &a) {
  const uint32_t nsb = a.in_dim / 256;
  const bool q45 = a.ggml_type == OGM_Q4_K || a.ggml_type == OGM_Q5_K;
  // (the plane kernel keeps a table of nsb * 512 bytes in LDS next to its 94 KB of stages)
  const bool i8 = q45 && (a.q4k_variant == 3u || nsb * 512u + 98304u > GM_LDS_MAX);
  if (i8) return 1;
  if (a.q4k_variant == 2u) return 0;
  uint32_t tiles64_all = (a.out_dim + 63u) / 64u;
  for (uint32_t m = 0; m < a.n_extra; m++) tiles64_all += (a.extra_out_dim[m] + 63u) / 64u;
  // (measured, Q4_K from 4096 inputs, small-batch against tiled, us: 4096 rows at 192 / 256 / 384 tokens 36 against 45,
  // 39 against 46, 57 against 49; 6144 rows at 128 / 192: 37 against 47, 47 against 47; 14336 rows at 64 / 96: 38 against 44,
  // 51 against 46)
  const uint32_t small_max =
      a.small_max_tokens ? a.small_max_tokens : (tiles64_all <= 64u ? 256u : tiles64_all <= 128u ? 128u : 64u);
  if (a.ggml_type != OGM_Q3_K && a.small_max_tokens != 1u && a.n_tokens <= small_max &&
      (q45 ? 16u : 8u) * 4096u + 128u * nsb <= GM_LDS_MAX)
    return 2;
  return 3;
}

// Whether a tiled plane launch (gemm_k_path 3) goes to the kernel whose waves all multiply, given
// planes.  It wants more 128 x 128 workgroups than there are compute units (two share one, and one
// alone is slower than the feeding-wave kernels: Q4_K 4096 -> 14336 at 256 tokens 69 us against 57, at
// 384 tokens 87 against 104), the activations in operand chunks, for which the f16 scratch has room
// from 32 tokens, and everything within 32-bit byte offsets.  (plane_kernel 2: whatever the grid.)
static bool gemm_dma_eligible(const OgmGemmArgs &a) {
  const uint32_t nsb = a.in_dim / 256;
  const bool q45 = a.ggml_type == OGM_Q4_K || a.ggml_type == OGM_Q5_K;
  const uint32_t t_pad = (a.n_tokens + 31u) & ~31u;
  if (a.plane_kernel == 1u || (q45 && nsb * 512u > GD_TAB) || a.n_tokens < 32u || !a.xh ||
      (uint64_t)t_pad * a.in_dim >= (1ull << 32))
    return false;
  uint32_t tiles = 0;
  for (uint32_t m = 0; m <= a.n_extra; m++) {
    const uint32_t od = m ? a.extra_out_dim[m - 1] : a.out_dim;
    if ((uint64_t)((od + 63u) / 64u) * 64u * a.in_dim * 2u >= (1ull << 32)) return false;
    tiles += (od + GD_ROWS - 1u) / GD_ROWS;
  }
  return a.plane_kernel == 2u || ((a.n_tokens + GD_TOK - 1u) / GD_TOK) * tiles > 256u;
}

bool ogm_gemm_uses_planes(const OgmGemmArgs &a) {
  if (a.n_tokens == 0 || a.out_dim == 0 || is_flat32(a.ggml_type)) return false;
  if (!ogm_gemm_supported(a.ggml_type, a.in_dim, a.out_dim, a.n_tokens)) return false;
  // the feeding-wave kernels read planes only when asked to (they are no faster for it: Q4_K 4096 -> 14336 at 256
  // tokens 66 against 66 us; Q6_K 14336 -> 4096 at 512 tokens 96 against 98)
  return gemm_k_path(a) == 3 && (a.plane_kernel == 1u || gemm_dma_eligible(a));
}

hipError_t ogm_launch_gemm(const OgmGemmArgs &a, hipStream_t stream, const char **kernel_name) {
  if (a.n_tokens == 0 || a.out_dim == 0) return hipSuccess;
  if (!ogm_gemm_supported(a.ggml_type, a.in_dim, a.out_dim, a.n_tokens)) return hipErrorInvalidValue;
  if (a.n_extra > OGM_GEMM_MAX_MATS - 1 || (is_flat32(a.ggml_type) && a.n_extra != 0)) return hipErrorInvalidValue;
  if (is_flat32(a.ggml_type)) {
    GemmFlatParams p;
    p.wt = a.wt;
    p.xq = a.act.q;
    p.ad = a.act.d;
    p.y = a.y;
    p.in_dim = a.in_dim;
    p.out_dim = a.out_dim;
    p.n_tokens = a.n_tokens;
    p.nblk = a.in_dim / 32;
    const OgmTiling tl = ogm_tiling_for(p.nblk, a.out_dim);
    p.c_shift = tl.C == 4 ? 2 : 1;   // in_dim % 64 == 0: at least two blocks per tile row
    p.r_shift = 6 - p.c_shift;
    p.nct = tl.nct;
    const dim3 grid((a.n_tokens + 127u) / 128u, (a.out_dim + 127u) / 128u);
    switch (a.ggml_type) {
      case OGM_Q4_0: hipLaunchKernelGGL(ogm_gemm_flat_kernel<0>, grid, dim3(768), 0, stream, p); break;
      case OGM_Q5_0: hipLaunchKernelGGL(ogm_gemm_flat_kernel<1>, grid, dim3(768), 0, stream, p); break;
      case OGM_IQ4_NL: hipLaunchKernelGGL(ogm_gemm_flat_kernel<2>, grid, dim3(768), 0, stream, p); break;
      default: hipLaunchKernelGGL(ogm_gemm_flat_kernel<3>, grid, dim3(768), 0, stream, p); break;
    }
    if (kernel_name) *kernel_name = "ogm_gemm_flat_kernel";
    return hipGetLastError();
  }
  const uint32_t nsb = a.in_dim / 256;
  const size_t n8 = (size_t)a.in_dim * a.n_tokens / 8, n_sb = (size_t)nsb * a.n_tokens;
  _Float16 *xh = (_Float16 *)a.xh;
  _Float16 *bs16 = xh + (size_t)a.in_dim * a.n_tokens;
  // Q4_K beyond two token tiles of 128 runs the wide kernel, which reads the int8 activations as
  // they are and needs only the (bh, bl) pairs prepared
  // Q4_K beyond two token tiles of 128 runs the wide kernel (which reads the int8 activations as
  // they are and needs only the (bh, bl) pairs prepared) once the 128 x 128 tiling would need more
  // than one round of workgroups over the 256 compute units: within one round the smaller tile's
  // shorter chain per workgroup wins (4096 -> 4096 at 512 tokens: 76 us against 103 us), beyond it
  // the wide tile's halved weight traffic does (4096 -> 14336: 119 us against 166 us)
  uint32_t row_tiles = (a.out_dim + GM_BN - 1) / GM_BN;
  for (uint32_t m = 0; m < a.n_extra; m++) row_tiles += (a.extra_out_dim[m] + GM_BN - 1) / GM_BN;
  const uint32_t wgs128 = ((a.n_tokens + GM_BT - 1) / GM_BT) * row_tiles;
  // K-quants run on the int8 kernels unless the f16 kernels are asked for (q4k_variant 2): the ones
  // with scale-folded weight planes, or for Q4_K and Q5_K the one that scales partial sums by
  // integer multiply-adds (q4k_variant 3).  Of the f16 Q4_K kernels the wide one takes over as
  // described above.
  const bool q45 = a.ggml_type == OGM_Q4_K || a.ggml_type == OGM_Q5_K;
  const int path = gemm_k_path(a);
  const bool i8 = path == 1;
  const bool i8p = path >= 2;
  const bool wide = a.ggml_type == OGM_Q4_K && a.q4k_variant == 2u && a.n_tokens > 256u &&
                    wgs128 > (a.wide_min_wgs ? a.wide_min_wgs : 256u);
  const bool raw_x = wide || i8 || i8p;   // these read the int8 activations as they are: only (bh, bl) to prepare
  // The first-pass operand (the quantizer's sums per 32 as f16 pairs) comes from the quantizer itself
  // when it wrote one; the f16 kernels also want the activations as f16.  The plane kernels of Q6_K
  // and Q3_K need neither.
  const bool have_bs16 = raw_x && a.act.bs16 != nullptr;
  if (have_bs16) bs16 = (_Float16 *)a.act.bs16;
  if ((!i8p || q45) && !have_bs16)
    hipLaunchKernelGGL(ogm_gemm_prep_kernel, dim3((unsigned)(((raw_x ? n_sb : n8) + 255) / 256)), dim3(256), 0,
                       stream, a.act.q, a.act.bsum, raw_x ? (_Float16 *)nullptr : xh, bs16, n8, n_sb);
  const OgmTiling tl = ogm_tiling_for(nsb, a.out_dim);
  const uint32_t c_shift = tl.C == 4 ? 2 : (tl.C == 2 ? 1 : 0);
  // token tiles vary fastest: workgroups that run together share weight rows, and with a
  // power-of-two number of token tiles each XCD's L2 sees few distinct activation tiles
  const dim3 grid((a.n_tokens + GM_BT - 1) / GM_BT, row_tiles);
  hipError_t e;
  if (i8) {
    GemmParams p;
    p.wt = a.wt;
    p.xh = nullptr;
    p.bs16 = bs16;
    p.ad = a.act.d;
    p.y = a.y;
    p.in_dim = a.in_dim;
    p.out_dim = a.out_dim;
    p.n_tokens = a.n_tokens;
    p.nsb = nsb;
    p.c_shift = c_shift;
    p.r_shift = 6 - c_shift;
    p.nct = tl.nct;
    p.xq = a.act.q;
    p.n_extra = a.n_extra;
    for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
      p.extra_wt[m] = m < a.n_extra ? a.extra_wt[m] : nullptr;
      p.extra_y[m] = m < a.n_extra ? a.extra_y[m] : nullptr;
      p.extra_out_dim[m] = m < a.n_extra ? a.extra_out_dim[m] : 0u;
    }
    if (a.ggml_type == OGM_Q4_K) {
      hipLaunchKernelGGL(ogm_gemm_q4k_i8_kernel, grid, dim3(768), 0, stream, p);
      if (kernel_name) *kernel_name = "ogm_gemm_q4k_i8_kernel";
    } else {
      hipLaunchKernelGGL(ogm_gemm_q5k_i8_kernel, grid, dim3(768), 0, stream, p);
      if (kernel_name) *kernel_name = "ogm_gemm_q5k_i8_kernel";
    }
    return hipGetLastError();
  }
  // Small batches: the kernel whose waves take different super-blocks.  By default up to 64 tokens
  // (Q4_K 4096 -> 14336: 18 / 35 / 50 us at 32 / 64 / 96 tokens against 42-45 us tiled), and up to 128
  // when the tiled kernel's grid would leave half the CUs idle (4096 -> 4096: 12 / 15 / 21 us at 32 /
  // 64 / 128 tokens against 38-41; 14336 -> 4096: 36 / 39 / 57 against 123-130).
  if (path == 2) {
    GemmSbParams p;
    p.wt = a.wt;
    p.xq = a.act.q;
    p.ad = a.act.d;
    p.bs16 = bs16;
    p.y = a.y;
    p.in_dim = a.in_dim;
    p.out_dim = a.out_dim;
    p.n_tokens = a.n_tokens;
    p.nsb = nsb;
    p.c_shift = c_shift;
    p.r_shift = 6 - c_shift;
    p.nct = tl.nct;
    p.n_extra = a.n_extra;
    uint32_t tiles = (a.out_dim + 31u) / 32u;
    for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
      p.extra_wt[m] = m < a.n_extra ? a.extra_wt[m] : nullptr;
      p.extra_y[m] = m < a.n_extra ? a.extra_y[m] : nullptr;
      p.extra_out_dim[m] = m < a.n_extra ? a.extra_out_dim[m] : 0u;
      if (m < a.n_extra) tiles += (a.extra_out_dim[m] + 31u) / 32u;
    }
    // sixteen waves when the launch leaves compute units idle and the rows are long enough
    const uint32_t n_wg = ((a.n_tokens + 31u) / 32u) * tiles;
    const bool w16 = (a.sb_waves ? a.sb_waves == 16u : (n_wg <= 256u && nsb >= 16u)) &&
                     16u * 4096u + 128u * nsb <= GM_LDS_MAX;
    const uint32_t lds_bytes = ((q45 || w16) ? 16u : 8u) * 4096u + 128u * nsb;
    const void *fn = a.ggml_type == OGM_Q6_K   ? (w16 ? (const void *)ogm_gemm_sb_q6k_w16_kernel : (const void *)ogm_gemm_sb_q6k_kernel)
                     : a.ggml_type == OGM_Q4_K ? (w16 ? (const void *)ogm_gemm_sb_q45k_w16_kernel<false> : (const void *)ogm_gemm_sb_q45k_kernel<false>)
                                               : (w16 ? (const void *)ogm_gemm_sb_q45k_w16_kernel<true> : (const void *)ogm_gemm_sb_q45k_kernel<true>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
    void *kargs[] = {(void *)&p};
    e = hipLaunchKernel(fn, dim3((a.n_tokens + 31u) / 32u, tiles), dim3(w16 ? 1024 : 512), kargs, lds_bytes, stream);
    if (e != hipSuccess) return e;
    if (kernel_name)
      *kernel_name = a.ggml_type == OGM_Q6_K   ? (w16 ? "ogm_gemm_sb_q6k_w16_kernel" : "ogm_gemm_sb_q6k_kernel")
                     : a.ggml_type == OGM_Q4_K ? (w16 ? "ogm_gemm_sb_q4k_w16_kernel" : "ogm_gemm_sb_q4k_kernel")
                                               : (w16 ? "ogm_gemm_sb_q5k_w16_kernel" : "ogm_gemm_sb_q5k_kernel");
    return hipGetLastError();
  }
  if (i8p) {
    GemmI8pParams p;
    p.wt = a.wt;
    p.xq = a.act.q;
    p.ad = a.act.d;
    p.bs16 = bs16;
    p.y = a.y;
    p.in_dim = a.in_dim;
    p.out_dim = a.out_dim;
    p.n_tokens = a.n_tokens;
    p.nsb = nsb;
    p.c_shift = c_shift;
    p.r_shift = 6 - c_shift;
    p.nct = tl.nct;
    p.n_extra = a.n_extra;
    bool pre = a.planes != nullptr;
    p.planes = a.planes;
    for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
      p.extra_wt[m] = m < a.n_extra ? a.extra_wt[m] : nullptr;
      p.extra_y[m] = m < a.n_extra ? a.extra_y[m] : nullptr;
      p.extra_out_dim[m] = m < a.n_extra ? a.extra_out_dim[m] : 0u;
      p.extra_planes[m] = m < a.n_extra ? a.extra_planes[m] : nullptr;
      if (m < a.n_extra && !a.extra_planes[m]) pre = false;   // every matrix of the launch, or none
    }
    const uint32_t t_pad = (a.n_tokens + 31u) & ~31u;
    const bool dma = pre && gemm_dma_eligible(a);
    if (a.plane_kernel != 1u) pre = false;   // planes given, but not for the feeding-wave kernels
    if (dma) {
      hipLaunchKernelGGL(ogm_gemm_xtile_kernel, dim3(a.in_dim / 128u, t_pad / 32u), dim3(256), 0, stream, a.act.q,
                         (int8_t *)a.xh, a.in_dim, a.n_tokens);
      GemmDmaParams d;
      d.wt = a.wt;
      d.planes = a.planes;
      d.xt = (const int8_t *)a.xh;
      d.ad = a.act.d;
      d.bs16 = bs16;
      d.y = a.y;
      d.in_dim = a.in_dim;
      d.out_dim = a.out_dim;
      d.n_tokens = a.n_tokens;
      d.nsb = nsb;
      d.c_shift = c_shift;
      d.r_shift = 6 - c_shift;
      d.nct = tl.nct;
      d.n_extra = a.n_extra;
      uint32_t tiles256 = (a.out_dim + GD_ROWS - 1u) / GD_ROWS;
      for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
        d.extra_wt[m] = p.extra_wt[m];
        d.extra_planes[m] = p.extra_planes[m];
        d.extra_y[m] = p.extra_y[m];
        d.extra_out_dim[m] = p.extra_out_dim[m];
        if (m < a.n_extra) tiles256 += (a.extra_out_dim[m] + GD_ROWS - 1u) / GD_ROWS;
      }
      const bool one_pass = q45 && a.one_pass != 0u;
      const void *fn = a.ggml_type == OGM_Q6_K   ? (const void *)ogm_gemm_dma_kernel<GP_Q6K>
                       : a.ggml_type == OGM_Q3_K ? (const void *)ogm_gemm_dma_kernel<GP_Q3K>
                       : a.ggml_type == OGM_Q4_K ? (one_pass ? (const void *)ogm_gemm_dma_kernel<GP_Q4K, true>
                                                             : (const void *)ogm_gemm_dma_kernel<GP_Q4K>)
                                                 : (one_pass ? (const void *)ogm_gemm_dma_kernel<GP_Q5K, true>
                                                             : (const void *)ogm_gemm_dma_kernel<GP_Q5K>);
      const uint32_t dma_lds = one_pass ? GD_LDS_BYTES_ONEPASS : GD_LDS_BYTES;
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)dma_lds);
      if (e != hipSuccess) return e;
      void *kargs[] = {(void *)&d};
      e = hipLaunchKernel(fn, dim3((a.n_tokens + GD_TOK - 1u) / GD_TOK, tiles256), dim3(64u * GD_NW), kargs, dma_lds, stream);
      if (e != hipSuccess) return e;
      if (kernel_name)
        *kernel_name = a.ggml_type == OGM_Q6_K   ? "ogm_gemm_q6k_dma_kernel"
                       : a.ggml_type == OGM_Q3_K ? "ogm_gemm_q3k_dma_kernel"
                       : a.ggml_type == OGM_Q4_K ? (one_pass ? "ogm_gemm_q4k_dma_onepass_kernel" : "ogm_gemm_q4k_dma_kernel")
                                                 : (one_pass ? "ogm_gemm_q5k_dma_onepass_kernel" : "ogm_gemm_q5k_dma_kernel");
      return hipGetLastError();
    }
    // 64-row tiles when asked for (q4k_variant 1), or when they still come one to a CU: then twice
    // as many CUs work (14336 -> 4096 x 512 tokens: 150 us against 180 us).  Two of them sharing a CU
    // are slower than one 128-row tile (4096 -> 14336 x 512: 165 us against 118 us).
    uint32_t tiles64 = (a.out_dim + 63u) / 64u;
    for (uint32_t m = 0; m < a.n_extra; m++) tiles64 += (a.extra_out_dim[m] + 63u) / 64u;
    const bool r64 = a.q4k_variant == 1u || ((a.n_tokens + 127u) / 128u) * tiles64 <= 256u;
    const uint32_t rows = r64 ? 64u : 128u;
    const uint32_t tiles = r64 ? tiles64 : row_tiles;
    const dim3 pgrid((a.n_tokens + 127u) / 128u, tiles);
    const bool q3 = a.ggml_type == OGM_Q3_K;
    // Q4_K / Q5_K: + the tokens' ad of every super-block for the first pass
    const uint32_t lds_bytes = (q3 ? 3u : 6u) * rows * GI_ROW + 3u * GI_WTILE + (2u * rows + 256u) * 4u +
                               (q45 ? nsb * 512u : 0u);
    struct Pick { uint32_t type; bool r64, pre; const void *fn; const char *name; };
    const Pick picks[] = {
        {OGM_Q6_K, false, false, (const void *)ogm_gemm_q6k_i8_kernel, "ogm_gemm_q6k_i8_kernel"},
        {OGM_Q6_K, true, false, (const void *)ogm_gemm_q6k_i8_r64_kernel, "ogm_gemm_q6k_i8_r64_kernel"},
        {OGM_Q3_K, false, false, (const void *)ogm_gemm_q3k_i8_kernel, "ogm_gemm_q3k_i8_kernel"},
        {OGM_Q3_K, true, false, (const void *)ogm_gemm_q3k_i8_r64_kernel, "ogm_gemm_q3k_i8_r64_kernel"},
        {OGM_Q4_K, false, false, (const void *)ogm_gemm_q4k_i8p_kernel, "ogm_gemm_q4k_i8p_kernel"},
        {OGM_Q4_K, true, false, (const void *)ogm_gemm_q4k_i8p_r64_kernel, "ogm_gemm_q4k_i8p_r64_kernel"},
        {OGM_Q5_K, false, false, (const void *)ogm_gemm_q5k_i8p_kernel, "ogm_gemm_q5k_i8p_kernel"},
        {OGM_Q5_K, true, false, (const void *)ogm_gemm_q5k_i8p_r64_kernel, "ogm_gemm_q5k_i8p_r64_kernel"},
        {OGM_Q6_K, false, true, (const void *)ogm_gemm_q6k_i8_pre_kernel, "ogm_gemm_q6k_i8_pre_kernel"},
        {OGM_Q6_K, true, true, (const void *)ogm_gemm_q6k_i8_pre_r64_kernel, "ogm_gemm_q6k_i8_pre_r64_kernel"},
        {OGM_Q3_K, false, true, (const void *)ogm_gemm_q3k_i8_pre_kernel, "ogm_gemm_q3k_i8_pre_kernel"},
        {OGM_Q3_K, true, true, (const void *)ogm_gemm_q3k_i8_pre_r64_kernel, "ogm_gemm_q3k_i8_pre_r64_kernel"},
        {OGM_Q4_K, false, true, (const void *)ogm_gemm_q4k_i8p_pre_kernel, "ogm_gemm_q4k_i8p_pre_kernel"},
        {OGM_Q4_K, true, true, (const void *)ogm_gemm_q4k_i8p_pre_r64_kernel, "ogm_gemm_q4k_i8p_pre_r64_kernel"},
        {OGM_Q5_K, false, true, (const void *)ogm_gemm_q5k_i8p_pre_kernel, "ogm_gemm_q5k_i8p_pre_kernel"},
        {OGM_Q5_K, true, true, (const void *)ogm_gemm_q5k_i8p_pre_r64_kernel, "ogm_gemm_q5k_i8p_pre_r64_kernel"},
    };
    const Pick *pick = nullptr;
    for (const Pick &c : picks)
      if (c.type == a.ggml_type && c.r64 == r64 && c.pre == pre) pick = &c;
    if (!pick) return hipErrorInvalidValue;
    hipError_t e = hipFuncSetAttribute(pick->fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
    void *kargs[] = {(void *)&p};
    e = hipLaunchKernel(pick->fn, pgrid, dim3(r64 ? 512 : 1024), kargs, lds_bytes, stream);
    if (e != hipSuccess) return e;
    const char *name = pick->name;
    if (kernel_name) *kernel_name = name;
    return hipGetLastError();
  }
  if (a.ggml_type != OGM_Q4_K) {
    Gemm6Params p;
    p.wt = a.wt;
    p.xh = xh;
    p.ad = a.act.d;
    p.bs16 = bs16;
    p.n_extra = a.n_extra;
    for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
      p.extra_wt[m] = m < a.n_extra ? a.extra_wt[m] : nullptr;
      p.extra_y[m] = m < a.n_extra ? a.extra_y[m] : nullptr;
      p.extra_out_dim[m] = m < a.n_extra ? a.extra_out_dim[m] : 0u;
    }
    p.y = a.y;
    p.in_dim = a.in_dim;
    p.out_dim = a.out_dim;
    p.n_tokens = a.n_tokens;
    p.nsb = nsb;
    p.c_shift = c_shift;
    p.r_shift = 6 - c_shift;
    p.nct = tl.nct;
    // more dynamic LDS than the 64 KB a kernel gets without asking
    const void *fn = a.ggml_type == OGM_Q6_K   ? (const void *)ogm_gemm_q6k_kernel
                     : a.ggml_type == OGM_Q3_K ? (const void *)ogm_gemm_q3k_kernel
                                               : (const void *)ogm_gemm_q5k_kernel;
    const uint32_t lds5 = G6_LDS_BYTES + nsb * 512u;   // Q5_K: + the table of dmin of its first pass
    e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)(a.ggml_type == OGM_Q5_K ? GM_LDS_MAX : G6_LDS_BYTES));
    if (e != hipSuccess) return e;
    if (a.ggml_type == OGM_Q6_K) {
      hipLaunchKernelGGL(ogm_gemm_q6k_kernel, grid, dim3(512), G6_LDS_BYTES, stream, p);
      if (kernel_name) *kernel_name = "ogm_gemm_q6k_kernel";
    } else if (a.ggml_type == OGM_Q3_K) {
      hipLaunchKernelGGL(ogm_gemm_q3k_kernel, grid, dim3(512), G6_LDS_BYTES, stream, p);
      if (kernel_name) *kernel_name = "ogm_gemm_q3k_kernel";
    } else {
      hipLaunchKernelGGL(ogm_gemm_q5k_kernel, grid, dim3(512), lds5, stream, p);
      if (kernel_name) *kernel_name = "ogm_gemm_q5k_kernel";
    }
    return hipGetLastError();
  }
  GemmParams p;
  p.wt = a.wt;
  p.xh = xh;
  p.bs16 = bs16;
  p.ad = a.act.d;
  p.y = a.y;
  p.in_dim = a.in_dim;
  p.out_dim = a.out_dim;
  p.n_tokens = a.n_tokens;
  p.nsb = nsb;
  p.c_shift = c_shift;
  p.r_shift = 6 - c_shift;
  p.nct = tl.nct;
  p.xq = a.act.q;
  p.n_extra = a.n_extra;
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
    p.extra_wt[m] = m < a.n_extra ? a.extra_wt[m] : nullptr;
    p.extra_y[m] = m < a.n_extra ? a.extra_y[m] : nullptr;
    p.extra_out_dim[m] = m < a.n_extra ? a.extra_out_dim[m] : 0u;
  }
  if (wide) {
    const dim3 wgrid((a.n_tokens + GW_BT - 1) / GW_BT, row_tiles);
    e = hipFuncSetAttribute((const void *)ogm_gemm_q4k_wide_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)GW_LDS_BYTES);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(ogm_gemm_q4k_wide_kernel, wgrid, dim3(768), GW_LDS_BYTES, stream, p);
    if (kernel_name) *kernel_name = "ogm_gemm_q4k_wide_kernel";
    return hipGetLastError();
  }
  const uint32_t lds4 = GM_LDS_BYTES + nsb * 512u;   // + pass 1's table of dmin
  e = hipFuncSetAttribute((const void *)ogm_gemm_q4k_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)GM_LDS_MAX);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ogm_gemm_q4k_kernel, grid, dim3(1024), lds4, stream, p);
  if (kernel_name) *kernel_name = "ogm_gemm_q4k_kernel";
  return hipGetLastError();
}
