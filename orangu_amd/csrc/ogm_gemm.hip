// gfx950 prefill GEMMs for the K-quants and the per-32 types on the matrix cores, bit-compatible with the CPU
// path's GEMMs (gemm_k_q4_k + accumulate_sym32, gemm_k_q6_k, dot_flat_pair: engine/vecdot.rs:2213-2303,
// 2352-2398, 2598-2629 of orangu-server).
//
// The integer stage stays exact on the int8 matrix cores: a K-quant weight enters with its integer
// sub-block scale folded in and split by bytes, u = sc * q + 128 = 256 h + (l + 128), two int8 planes, so that
// isum = 256 H + L after two plain chains of v_mfma_i32_32x32x32_i8 over a super-block; the f32 stage then
// follows the reference's order per super-block (for Q4_K / Q5_K: first acc -= (ad * dmin) * imin over all
// super-blocks, imin from one K = 16 f16 instruction over exact operands, then acc += ad * (d * isum)).
//
// Kernels, by the size of the launch (ogm_launch_gemm at the end of the file):
//   * gemm_sb_*: small batches, 32 rows x 32 tokens per workgroup, its waves on different super-blocks;
//   * gemm_q6k_i8_body: 128 (64) rows x 128 tokens, feeding waves unpack per call, as many multiply;
//   * ogm_gemm_dma_kernel: the same tile over planes built once per matrix, all waves multiply;
//   * ogm_gemm_flat_kernel: the per-32 types (f16 operands, one block per accumulator).
#include <hip/hip_runtime.h>
#include <type_traits>

#include "ogm_kernels.h"
#include "ogm_layout.h"
#include "ogm_nib32_dev.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));

#define GM_BN 128   // rows per workgroup of the tiled kernels
#define GM_BT 128   // tokens per workgroup

__device__ __forceinline__ float gm_f16_bits_to_f32(uint32_t bits16) {
  union { unsigned short u; _Float16 h; } v;
  v.u = (unsigned short)bits16;
  return (float)v.h;
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

typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int16v __attribute__((ext_vector_type(16)));

#define GI_ROW 80u                   // bytes of an LDS row (64 int8 + padding)
#define GI_WTILE (128u * GI_ROW)     // the weight tile of a stage


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
#define GP_IQ4XS 4   // plane kernels only: the sums of Q6_K's GEMM (a scale per sub-block, no mins), tiles of Q4_K's size, d where Q4_K has it
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

template <uint32_t ROWS, int KIND>
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
    if constexpr (Q3) {                                                                           \
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
        scxa = *(const uint4 *)(p.wt + (uo + so_ + 6u * 1024u));                                  \
        hmxn = *(const uint4 *)(p.wt + (uo + so_ + (t16 & 1u) * 1024u));                          \
      } else if constexpr (Q45) {                                                                 \
        scxa = *(const uint4 *)(p.wt + (uo + so_));   /* d | dmin, then the 12 scale bytes */     \
        if constexpr (Q5) hmxn = *(const uint4 *)(p.wt + (uo + so_ + (1u + (t16 & 1u)) * 1024u)); \
      } else {                                                                                    \
        scxa = *(const uint4 *)(p.wt + (uo + so_ + 12u * 1024u));                                 \
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
    if constexpr (Q3) GP_GROUP3(qla##K, G, pw, prw, t16);                                         \
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

// Builds a matrix's planes from its tile-planar bytes: thread (t = tid / 64, r = tid % 64) of
// workgroup (4 s + g, rb) turns the sixteen weights 256 s + 64 g + 16 t .. of row 64 rb + r into their
// 16 bytes of each plane -- the arithmetic of the feeding waves above, done once.
//   Q6_K: u = sc_g (q - 32) + 128, sc the int8 scale of the group of 16       (vecdot.rs:2119-2143)
//   Q3_K: one plane, (sc - 32)(4 - q) with the six-bit scale of the group      (vecdot.rs:2100-2117)
//   Q4_K / Q5_K: u = sc_j q + 128, sc the six-bit scale of the sub-block of 32 (vecdot.rs:2036-2088)
//   IQ4_XS: u = (ls_j - 32) level + 128, the sub-block's six-bit scale and IQ4_NL's levels  (vecdot.rs:2333-2350)
// h = u >> 8, l = (u & 255) - 128 as int8: sc * q' = 256 h + l.
struct GemmPlaneBuildParams {
  const uint8_t *wt;
  uint8_t *planes;
  uint32_t out_dim, nsb, c_shift, r_shift, nct;
};

template <int KIND>
__global__ __launch_bounds__(256) void ogm_gemm_build_planes_kernel(GemmPlaneBuildParams p) {
  constexpr bool Q3 = KIND == GP_Q3K, Q45 = KIND == GP_Q4K || KIND == GP_Q5K, Q5 = KIND == GP_Q5K, XS = KIND == GP_IQ4XS;
  constexpr uint32_t TILE_BYTES = Q3 ? 7168u : (KIND == GP_Q4K || XS) ? 9216u : Q5 ? 11264u : 13440u;
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
  } else if constexpr (XS) {
    // sub-block ib = 2 g + t16 / 2 of the super-block, its elements 16 (t16 & 1) ..: the low or the high nibbles of
    // block bytes 8 + 16 ib .. (the upper half of piece ib, the lower half of piece ib + 1), through IQ4_NL's sixteen
    // levels; the six-bit scale ls - 32 from scales_l / scales_h (vecdot.rs:2333-2350).  The signed level goes in as
    // the byte level + 128: u = ls (level + 128) + (128 - 128 ls)
    const uint32_t ib = 2u * g + (t16 >> 1);
    const uint4 pa = *(const uint4 *)(u0 + ib * 1024u), pb = *(const uint4 *)(u0 + (ib + 1u) * 1024u);
    const uint4 hd = *(const uint4 *)u0;
    const uint32_t sh = hd.x >> 16, sl = hd.y, nsh = 4u * (t16 & 1u);
    ql = make_uint4(ogm_nib32_weights<2>((pa.z >> nsh) & 0x0F0F0F0Fu, 0u) ^ 0x80808080u,
                    ogm_nib32_weights<2>((pa.w >> nsh) & 0x0F0F0F0Fu, 0u) ^ 0x80808080u,
                    ogm_nib32_weights<2>((pb.x >> nsh) & 0x0F0F0F0Fu, 0u) ^ 0x80808080u,
                    ogm_nib32_weights<2>((pb.y >> nsh) & 0x0F0F0F0Fu, 0u) ^ 0x80808080u);
    sc = (int)(((sl >> (4u * ib)) & 0xFu) | (((sh >> (2u * ib)) & 3u) << 4)) - 32;
    addc = (short)(128 - 128 * sc);
    mask_q = 0xFFFFFFFFu;
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
  constexpr bool XS = KIND == GP_IQ4XS;   // (no first pass, as Q6_K; its d is the first half of the header word, as Q4_K's)
  static_assert(!ONEPASS || Q45, "only the types with mins have a first pass to fold");
  constexpr uint32_t RING = ONEPASS ? GD_RING_ONEPASS : GD_RING, AHEAD = RING - 1u;
  constexpr uint32_t TAB = RING * GD_SLOT, TAB_SLOT = ONEPASS ? GD_TAB_SLOT_ONEPASS : GD_TAB_SLOT;
  constexpr uint32_t TILE_BYTES = Q3 ? 7168u : (KIND == GP_Q4K || XS) ? 9216u : Q5 ? 11264u : 13440u;
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
// The same multiplication on 64-row tiles, for launches too small to fill the 128-row kernel's places (its grid
// wants 384 tiles of 128 x 128; a 4096 x 4096 matrix at 512 tokens has 128), with the f32 step of a super-block
// issued *between* the matrix instructions of the next one.  A SIMD runs a matrix instruction for 32 clocks; the
// wave that issued it can issue about five vector instructions behind it for nothing (measured: eight matrix
// instructions 128 ns, with five dependent v_fma behind each 131 ns, with eight 166 ns), while vector work that
// waits for the end of a run of matrix instructions is paid in full: a workgroup that has a compute unit to itself
// has no second wave on its SIMDs to hide it behind.  The step acc += ad * (d * isum) is five vector instructions
// per output: one output per matrix instruction.  For that the planes' sums live in two register sets, one filled
// while the other is added up, which a wave tile of 32 rows x 64 tokens leaves room for (2 sets x 64 + 32 of y).
// On grids that fill the 128-row kernel this one is slower (4096 -> 14336 at 512 / 2048 tokens: 115 / 375 us
// against 98 / 322): a step of four matrix instructions a wave carries the same waits, barrier and loads as one
// of eight.
//
//   workgroup  256 threads = 4 waves; 64 rows x 128 tokens; wave w: rows 32 (w & 1) .. + 31, tokens
//              64 (w >> 1) .. + 63.  Two workgroups share a compute unit (67 KiB of LDS each).
//   step       32 weights of k: the row block's two planes (4 KiB, one piece of 1 KiB per wave) and
//              four token blocks of activations (1 KiB each, one per wave), by load-to-LDS, issued behind
//              the step's first matrix instruction
//   ring       eight steps in LDS = the steps of a super-block (step kk of any super-block sits in slot kk:
//              every LDS address of the loop is a constant), six in flight; one wait + barrier per step
//   tables     per super-block the tokens' activation scales and the rows' header words, three slots:
//              the one being added up, the one being multiplied, the one arriving
//   LDS reads  of a step, in issue order: [header word], four tokens' ad, h plane, two token blocks,
//              l plane -- issued one step ahead, between the matrix instructions, waited for by count
//   first pass (Q4_K, Q5_K) two super-blocks in turn: the matrix instructions of the next are issued before the
//              vector work of this one
// Same arithmetic and f32 order as ogm_gemm_dma_kernel; bit-identical results.
#define GX_NW 4u
#define GX_ROWS 64u
#define GX_TOK 128u
#define GX_RING 8u
#define GX_AHEAD (GX_RING - 1u)
#define GX_SLOT 8192u                 // a step's planes (4 KiB) and activations (4 KiB)
#define GX_TAB (GX_RING * GX_SLOT)
#define GX_TAB_SLOT 1024u             // 128 ad | 64 header words | 256 bytes that absorb wave 3's load
#define GX_LDS_BYTES (GX_TAB + 3u * GX_TAB_SLOT)
// timing experiments only (results are wrong with any of these set)
#ifndef GX_ABL_NOEPI
#define GX_ABL_NOEPI 0   // the f32 step left out of the loop
#endif
#ifndef GX_ABL_NOPASS1
#define GX_ABL_NOPASS1 0
#endif
#ifndef GX_ABL_NOMFMA
#define GX_ABL_NOMFMA 0
#endif
#ifndef GX_ABL_NODMA
#define GX_ABL_NODMA 0
#endif
#if GX_ABL_NOMFMA
#define GX_MFMA(A, B, C) (C)
#else
#define GX_MFMA(A, B, C) __builtin_amdgcn_mfma_i32_32x32x32_i8(A, B, C, 0, 0, 0)
#endif
#define GX_SYNC(N) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory")
#define GX_PIN() __builtin_amdgcn_sched_barrier(0)
#define GX_WAITN(N) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory")

template <int KIND>
__global__ __launch_bounds__(64 * GX_NW, 2) void ogm_gemm_dmx_kernel(GemmDmaParams p) {
  constexpr uint32_t NW = GX_NW, ROWS = GX_ROWS, SLOT = GX_SLOT, TAB = GX_TAB, TAB_SLOT = GX_TAB_SLOT;
  constexpr bool Q45 = KIND == GP_Q4K || KIND == GP_Q5K, Q5 = KIND == GP_Q5K, Q6 = KIND == GP_Q6K, XS = KIND == GP_IQ4XS;
  static_assert(Q45 || Q6 || XS, "two-plane types only");
  constexpr uint32_t TILE_BYTES = (KIND == GP_Q4K || XS) ? 9216u : Q5 ? 11264u : 13440u;
  constexpr uint32_t AHEAD = GX_AHEAD, PER = 2u;   // loads a wave issues per step
  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const uint32_t rs = wave & 1u, th = wave >> 1;   // row slice of 32, token half
  // token tiles of one row tile go to one XCD back to back (see ogm_gemm_dma_kernel)
  uint32_t tok_tile = blockIdx.x, row_tile = blockIdx.y;
  {
    const uint32_t nt = gridDim.x, lin = blockIdx.y * nt + blockIdx.x;
    if (lin < (gridDim.y & ~7u) * nt) {
      const uint32_t j = lin >> 3;
      tok_tile = j % nt;
      row_tile = (j / nt) * 8u + (lin & 7u);
    }
  }
#pragma unroll
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {   // the matrix this row tile belongs to
    const uint32_t tiles = (p.out_dim + ROWS - 1u) / ROWS;
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
  const uint32_t t0 = tok_tile * GX_TOK, r0 = row_tile * ROWS;
  auto sb_off = [&](uint32_t s) -> uint32_t {
    return (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 16u;
  };

  float16v y[2];
#pragma unroll
  for (int tb = 0; tb < 2; tb++)
#pragma unroll
    for (int r = 0; r < 16; r++) y[tb][r] = 0.0f;

  if constexpr (Q45 && !GX_ABL_NOPASS1) {
    // pass 1 of gemm_k_q4_k: acc -= (ad * dmin) * sum_j m_j * bsum_j over all super-blocks first
    // (vecdot.rs:2226-2240), as in ogm_gemm_dma_kernel, for this wave's two token blocks
    const uint32_t row = min(r0 + 32u * rs + l32, p.out_dim - 1u);
    const uint32_t uo = (row >> p.r_shift) * p.nct * TILE_BYTES + (row & ((1u << p.r_shift) - 1u)) * 16u;
    float *ad_all = (float *)lds;   // [nsb][128]
    {
      // element i of the tile's [128 tokens][nsb] block goes to [su][token]; eight loads in flight a thread, and the
      // (token, su) of i + 256 from those of i without dividing again
      const uint32_t total = GX_TOK * p.nsb, dq = (64u * NW) / p.nsb, dr = (64u * NW) % p.nsb;
      uint32_t k = tid / p.nsb, su = tid - k * p.nsb;
      for (uint32_t i0 = tid; i0 < total; i0 += 8u * 64u * NW) {
        float v[8];
        uint32_t dst[8];
#pragma unroll
        for (uint32_t j = 0; j < 8u; j++) {
          const bool in = i0 + j * 64u * NW < total;
          dst[j] = in ? su * GX_TOK + k : 0xFFFFFFFFu;
          v[j] = in ? p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + su] : 0.0f;
          k += dq;
          su += dr;
          if (su >= p.nsb) {
            su -= p.nsb;
            k++;
          }
        }
#pragma unroll
        for (uint32_t j = 0; j < 8u; j++)
          if (dst[j] != 0xFFFFFFFFu) ad_all[dst[j]] = v[j];
      }
    }
    __syncthreads();
    float16v zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.0f;
    uint32_t tk[2];
#pragma unroll
    for (int tb = 0; tb < 2; tb++) tk[tb] = min(t0 + 64u * th + 32u * tb + l32, p.n_tokens - 1u) * p.nsb;
    const float side_scale = lh ? 1.0f : 64.0f;
    // Two super-blocks in turn (sets X and Y): the matrix instructions of the next one are issued before the vector
    // work of this one, and each set's header and token sums are loaded two super-blocks ahead.
    uint4 hdX, hdY;
    half8 b2X[2], b2Y[2];
    float16v imX[2], imY[2];
    float dmX = 0.0f, dmY = 0.0f;
    auto load = [&](uint32_t su, uint4 &hd, half8(&b2)[2]) {
      const uint32_t sn = min(su, p.nsb - 1u);   // past the end: loaded again, never used
      hd = *(const uint4 *)(p.wt + (uo + sb_off(sn)));
#pragma unroll
      for (int tb = 0; tb < 2; tb++) b2[tb] = *(const half8 *)(p.bs16 + ((tk[tb] + sn) * 16u + 8u * lh));
    };
    auto stage = [&](const uint4 &hd, const half8(&b2)[2], float16v(&im)[2], float &dm) {
      uint32_t mna, mnb;
      q4k_mins(hd, mna, mnb);
      const half8 a1 = side_operand(mna, mnb, side_scale);
      dm = gm_f16_bits_to_f32(hd.x >> 16);
#pragma unroll
      for (int tb = 0; tb < 2; tb++) im[tb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b2[tb], a1, zero, 0, 0, 0);
    };
    auto consume = [&](uint32_t su, const float16v(&im)[2], float dm) {
#pragma unroll
      for (int tb = 0; tb < 2; tb++) {
        const float *adp = &ad_all[su * GX_TOK + 64u * th + 32u * tb + 4u * lh];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const float4 a4 = *(const float4 *)(adp + 8 * q4);
          const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
          for (int e = 0; e < 4; e++) y[tb][4 * q4 + e] -= a4v[e] * dm * im[tb][4 * q4 + e];
        }
      }
    };
    load(0u, hdX, b2X);
    load(1u, hdY, b2Y);
    stage(hdX, b2X, imX, dmX);
    load(2u, hdX, b2X);
    for (uint32_t su = 0; su < p.nsb; su += 2u) {
      const bool two = su + 1u < p.nsb;
      if (two) {
        stage(hdY, b2Y, imY, dmY);
        load(su + 3u, hdY, b2Y);
      }
      GX_PIN();
      consume(su, imX, dmX);
      GX_PIN();
      if (two) {
        if (su + 2u < p.nsb) {
          stage(hdX, b2X, imX, dmX);
          load(su + 4u, hdX, b2X);
        }
        GX_PIN();
        consume(su + 1u, imY, dmY);
        GX_PIN();
      }
    }
    __syncthreads();   // the table's LDS becomes the ring
  }

  // ---------------- the products
  // per step wave w fetches piece w of the row block's planes ((half of k, plane) = (w >> 1, w & 1): 64 rows x 16
  // bytes) and token block w of the activations.  The ring has as many slots as a super-block has steps: step kk of
  // any super-block sits in slot kk, so every LDS address of the loop is a constant.
  static_assert(GX_RING == 8u, "the ring's slots are the steps of a super-block");
  uint32_t w_src = row_tile * p.nsb * 8u * 4096u + wave * 1024u + lane * 16u;   // + 4096 per step
  uint32_t x_src = min((t0 >> 5) + wave, (p.n_tokens - 1u) >> 5) * (p.in_dim / 32u) * 1024u + lane * 16u;   // + 1024 per step
  const uint32_t w_dst = wave * 1024u, x_dst = 4096u + wave * 1024u;
  // tables: waves 0, 1 fetch 64 tokens' ad each, wave 2 the header words of the 64 rows (wave 3 the same again,
  // into spare bytes: every wave has the same number of loads in flight)
  uint32_t tab_src;
  if (wave < 2u) {
    tab_src = min(t0 + 64u * wave + lane, p.n_tokens - 1u) * p.nsb * 4u;
  } else {
    const uint32_t tab_row = min(r0 + lane, p.out_dim - 1u);
    const uint32_t tab_rb = tab_row >> p.r_shift, tab_r = tab_row & ((1u << p.r_shift) - 1u);
    if constexpr (Q6) tab_src = tab_rb * p.nct * TILE_BYTES + 13u * 1024u + ((tab_r * 2u) & ~3u);
    else tab_src = tab_rb * p.nct * TILE_BYTES + tab_r * 16u;
  }
  uint32_t tsl_prev = 0u, tsl_cur = 0u, tsl_next = TAB_SLOT;   // table slots of super-blocks s - 1, s, s + 1
  auto fetch_tables = [&](uint32_t s, uint32_t tsl) {
    uint8_t *slot = lds + TAB + tsl;
    if (wave < 2u) {
      gd_dma4((const uint8_t *)p.ad + (tab_src + 4u * s), slot + 256u * wave);
    } else {
      const uint32_t so = Q6 ? (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 2u : sb_off(s);
      gd_dma4(p.wt + (tab_src + so), slot + 512u + 256u * (wave - 2u));
    }
  };
  auto fetch_step = [&](uint32_t slot_off) {   // the next step (they are fetched in ascending order) into ring slot slot_off / SLOT
    uint8_t *slot = lds + slot_off;
    gd_dma16(p.planes + w_src, slot + w_dst);
    gd_dma16((const uint8_t *)p.xt + x_src, slot + x_dst);
    w_src += 4096u;
    x_src += 1024u;
  };

  fetch_tables(0u, 0u);
#pragma unroll
  for (uint32_t k = 0; k < AHEAD; k++) fetch_step(k * SLOT);
#define GX_SYNC_STEPS(N) GX_SYNC((N) * (int)PER)   // all but the newest N steps' loads of this wave have landed, then the barrier
  GX_SYNC_STEPS(AHEAD - 1);   // step 0 and the first tables have landed

  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
  const uint32_t w_rd = lds0 + lh * 2048u + (32u * rs + l32) * 16u;      // h plane; l plane + 1024
  const uint32_t x_rd = lds0 + 4096u + 2048u * th + lane * 16u;          // token block 0 of the wave; block 1 + 1024
  const uint32_t ad_rd = lds0 + TAB + 4u * (64u * th + 4u * lh);      // + 128 tb + 32 q4: four tokens' ad
  const uint32_t hw_rd = lds0 + TAB + 512u + 4u * (32u * rs + l32);   // the row's header word
  typedef float float4v __attribute__((ext_vector_type(4)));
  int16v hA[2], lA[2], hB[2], lB[2];
  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  int4v wh, wl, x0, x1;
  float4v a4[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
  uint32_t hw = 0;
  float d0 = 0.0f;
  GD_READ16(wh, w_rd, 0);
  GD_READ16(x0, x_rd, 0);
  GD_READ16(x1, x_rd, 1024);
  GD_READ16(wl, w_rd, 1024);

  // One super-block: its 8 steps accumulate into (hc, lc) while, with EPI, the sums of the one before in
  // (hp, lp) are added to y, one output behind every matrix instruction.
  auto super_block = [&](auto set_c, auto epi_c, uint32_t s) {
    constexpr bool SET = decltype(set_c)::value, EPI = decltype(epi_c)::value && !GX_ABL_NOEPI;
    const bool more = s + 1u < p.nsb;   // in the last super-block the steps in flight run out
    int16v(&hc)[2] = SET ? hB : hA;
    int16v(&lc)[2] = SET ? lB : lA;
    int16v(&hp)[2] = SET ? hA : hB;
    int16v(&lp)[2] = SET ? lA : lB;
    auto step = [&](auto kk_c) {
      constexpr uint32_t kk = decltype(kk_c)::value;
      // step k = 8 s + kk: step k + 1 has landed for every wave (all but the loads of the steps after it)
      if (kk + AHEAD <= 8u || more) GX_SYNC_STEPS(AHEAD - 2);
      else GX_SYNC_STEPS(kk >= 6u ? 0 : (int)(6u - kk));
      constexpr uint32_t NX = ((kk + 1u) & 7u) * SLOT;   // step k + 1's ring slot
      constexpr int tq = (int)(kk >> 2), q4 = (int)(kk & 3u);   // the four outputs added up in this step: y[tq][4 q4 ..]
      constexpr int cur = (int)(kk & 1u), nxt = cur ^ 1;
      // the next step's four ad: of the same super-block, or (from step 7) of this one, whose sums are complete then
      const uint32_t ad_nx = ad_rd + (kk == 7u ? tsl_cur : tsl_prev) + 128u * (((kk + 1u) & 7u) >> 2) + 32u * ((kk + 1u) & 3u);
      auto add_up = [&](auto e_c) {
        constexpr int e = decltype(e_c)::value;
        if constexpr (EPI) {
          const int is = hp[tq][4 * q4 + e] * 256 + lp[tq][4 * q4 + e];
          y[tq][4 * q4 + e] += a4[cur][e] * (d0 * (float)is);
        }
      };
      GX_PIN();
      // outstanding, oldest first: [hw at step 0], a4[cur], wh, x0, x1, wl  (without EPI and before step 7: no a4)
      GX_WAITN(2);
      asm volatile("" : "+v"(wh), "+v"(x0), "+v"(a4[cur]), "+v"(hw));
      if (EPI && kk == 0u) d0 = gm_f16_bits_to_f32(Q6 && (l32 & 1u) ? (hw >> 16) : (hw & 0xFFFFu));
      hc[0] = GX_MFMA(x0, wh, kk == 0u ? zi : hc[0]);
      GX_PIN();
      // the loads of step k + AHEAD (into the slot step k - 1 left) go out behind a matrix instruction
      if (kk == 0u && more) fetch_tables(s + 1u, tsl_next);
      if ((kk + AHEAD < 8u || more) && !GX_ABL_NODMA) fetch_step(((kk + AHEAD) & 7u) * SLOT);
      GX_PIN();
      add_up(std::integral_constant<int, 0>{});
      GX_PIN();
      GX_WAITN(1);
      asm volatile("" : "+v"(x1));
      hc[1] = GX_MFMA(x1, wh, kk == 0u ? zi : hc[1]);
      GX_PIN();
      if (kk == 7u) asm volatile("ds_read_b32 %0, %1" : "=v"(hw) : "v"(hw_rd + tsl_cur));
      if (EPI || kk == 7u) asm volatile("ds_read_b128 %0, %1" : "=v"(a4[nxt]) : "v"(ad_nx));
      asm volatile("ds_read_b128 %0, %2 offset:%3" : "=v"(wh) : "0"(wh), "v"(w_rd), "n"(NX));
      GX_PIN();
      add_up(std::integral_constant<int, 1>{});
      GX_PIN();
      // outstanding: wl, [hw], [a4 next], wh
      if (kk == 7u) GX_WAITN(3);
      else if (EPI) GX_WAITN(2);
      else GX_WAITN(1);
      asm volatile("" : "+v"(wl));
      lc[0] = GX_MFMA(x0, wl, kk == 0u ? zi : lc[0]);
      GX_PIN();
      asm volatile("ds_read_b128 %0, %2 offset:%3" : "=v"(x0) : "0"(x0), "v"(x_rd), "n"(NX));
      GX_PIN();
      add_up(std::integral_constant<int, 2>{});
      GX_PIN();
      lc[1] = GX_MFMA(x1, wl, kk == 0u ? zi : lc[1]);
      GX_PIN();
      asm volatile("ds_read_b128 %0, %2 offset:%3" : "=v"(x1) : "0"(x1), "v"(x_rd), "n"(NX + 1024u));
      asm volatile("ds_read_b128 %0, %2 offset:%3" : "=v"(wl) : "0"(wl), "v"(w_rd), "n"(NX + 1024u));
      GX_PIN();
      add_up(std::integral_constant<int, 3>{});
      GX_PIN();
    };
    step(std::integral_constant<uint32_t, 0u>{});
    step(std::integral_constant<uint32_t, 1u>{});
    step(std::integral_constant<uint32_t, 2u>{});
    step(std::integral_constant<uint32_t, 3u>{});
    step(std::integral_constant<uint32_t, 4u>{});
    step(std::integral_constant<uint32_t, 5u>{});
    step(std::integral_constant<uint32_t, 6u>{});
    step(std::integral_constant<uint32_t, 7u>{});
    const uint32_t t = tsl_prev;   // the slots turn: s - 1's is free for s + 2
    tsl_prev = tsl_cur;
    tsl_cur = tsl_next;
    tsl_next = (s == 0u) ? 2u * TAB_SLOT : t;
  };
  using std::false_type;
  using std::true_type;
  super_block(false_type{}, false_type{}, 0u);
  for (uint32_t s = 1; s < p.nsb; s += 2u) {
    super_block(true_type{}, true_type{}, s);
    if (s + 1u < p.nsb) super_block(false_type{}, true_type{}, s + 1u);
  }
  // the last super-block's sums (its header word and first four ad were asked for in its last step)
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wh), "+v"(x0), "+v"(x1), "+v"(wl), "+v"(a4[0]), "+v"(hw));
  {
    d0 = gm_f16_bits_to_f32(Q6 && (l32 & 1u) ? (hw >> 16) : (hw & 0xFFFFu));
    const uint32_t ta = ad_rd + tsl_prev;   // (the slots have turned once more)
    const bool odd = (p.nsb & 1u) == 0u;    // the last super-block filled set B
#pragma unroll
    for (int tb = 0; tb < 2; tb++) {
      float4v b40, b41, b42, b43;
      GD_READ16(b40, ta, 128 * tb);
      GD_READ16(b41, ta, 128 * tb + 32);
      GD_READ16(b42, ta, 128 * tb + 64);
      GD_READ16(b43, ta, 128 * tb + 96);
      GD_WAIT2(0, b40, b41);
      GD_WAIT2(0, b42, b43);
      const float4v b4[4] = {b40, b41, b42, b43};
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const float b4v[4] = {b4[q4].x, b4[q4].y, b4[q4].z, b4[q4].w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int is = odd ? hB[tb][4 * q4 + e] * 256 + lB[tb][4 * q4 + e] : hA[tb][4 * q4 + e] * 256 + lA[tb][4 * q4 + e];
          y[tb][4 * q4 + e] += b4v[e] * (d0 * (float)is);
        }
      }
    }
  }
  const uint32_t row0 = r0 + 32u * rs + l32;
  if (row0 < p.out_dim) {
#pragma unroll
    for (int tb = 0; tb < 2; tb++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const uint32_t t = t0 + 64u * th + 32u * tb + 8u * (r >> 2) + 4u * lh + (r & 3);
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
  uint32_t x_chunks;      // xq holds the activations in operand chunks (ogm_xt_row) instead of rows
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
  // a lane's 16 activations of a run of 32: from its token's row, or (x_chunks) from the 1 KiB operand chunk of
  // the tile's 32 tokens and the run's 32 k, where they lie in the instruction's own order
  const uint32_t xmul = p.x_chunks ? 32u : 1u;
  const uint32_t xro = p.x_chunks ? blockIdx.x * p.in_dim * 32u + 16u * lane
                                  : min(t0 + l32, p.n_tokens - 1u) * p.in_dim + 16u * lh;   // + (256 s + 32 sub) xmul
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
    const int4v xa_ = *(const int4v *)(p.xq + (xs_ + (64u * (G) + 32u * (SUB)) * xmul));          \
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
      const uint32_t xs_ = xro + 256u * s * xmul;
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

// The same for Q3_K, whose GEMM is Q6_K's loop (vecdot.rs:2014-2021) over weights (sc - 32)(q - 4) of seven bits:
// one operand plane, w' = (sc - 32)(4 - q) as an int8, and isum = -sum.  A unit's seven pieces: hmask (2), qs (4),
// scales[12] | d | padding (vecdot.rs:2100-2117).
template <uint32_t NW>
__device__ __forceinline__ void gemm_sb_q3k_body(GemmSbParams p) {
  constexpr uint32_t NT = 64u * NW, NACC = 1024u / NT;
  constexpr uint32_t TILE_BYTES = 7168u;
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
  uint32_t uo;   // this lane's row: piece 0 of its unit in super-block 0's tile
  {
    const uint32_t row = min(r0 + l32, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    uo = rb * p.nct * TILE_BYTES + r * 16u;
  }
  auto sb_off = [&](uint32_t s) -> uint32_t {
    return (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 16u;
  };
  // a lane's 16 activations of a run of 32: from its token's row, or (x_chunks) from the 1 KiB operand chunk of
  // the tile's 32 tokens and the run's 32 k, where they lie in the instruction's own order
  const uint32_t xmul = p.x_chunks ? 32u : 1u;
  const uint32_t xro = p.x_chunks ? blockIdx.x * p.in_dim * 32u + 16u * lane
                                  : min(t0 + l32, p.n_tokens - 1u) * p.in_dim + 16u * lh;   // + (256 s + 32 step) xmul

  for (uint32_t i = tid; i < 32u * p.nsb; i += NT) {
    const uint32_t k = i / p.nsb, s = i - k * p.nsb;
    ad_l[s * 32u + k] = p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + s];
  }

  // the lane's sixteen weights of step 2 g + sub are elements 64 g + 32 sub + 16 lh ..: run t16 = 2 sub + lh of group g.
  // Their two low bits sit in qs piece 2 (g / 2) + lh at bit 2 (2 (g & 1) + sub), the third in hmask piece lh at bit
  // 2 g + sub; the group's six-bit scale: four low bits in scales[4 (g & 1) + t16] (the high nibble for g >= 2), two
  // high bits in scales[8 + t16] at bit 2 g.
  uint4 wH, wQ0, wQ1, scx;
#define SB3_LOADW(S)                                                                              \
  do {                                                                                            \
    const uint32_t s_ = min((uint32_t)(S), p.nsb - 1u); /* past the end: loaded, never used */    \
    const uint32_t so_ = uo + sb_off(s_);                                                         \
    wH = *(const uint4 *)(p.wt + (so_ + lh * 1024u));                                             \
    wQ0 = *(const uint4 *)(p.wt + (so_ + (2u + lh) * 1024u));                                     \
    wQ1 = *(const uint4 *)(p.wt + (so_ + (4u + lh) * 1024u));                                     \
    scx = *(const uint4 *)(p.wt + (so_ + 6u * 1024u));                                            \
  } while (0)
#define SB3_STEP(G, SUB, FIRST)                                                                   \
  do {                                                                                            \
    const uint32_t t16_ = 2u * (SUB) + lh;                                                        \
    const uint32_t lw_ = ((G) & 1u) ? scx.y : scx.x;                                              \
    const uint32_t low_ = ((lw_ >> (8u * t16_)) >> ((G) >= 2u ? 4u : 0u)) & 0xFu;                 \
    const uint32_t high_ = ((scx.z >> (8u * t16_)) >> (2u * (G))) & 3u;                           \
    const int scv_ = (int)(low_ | (high_ << 4)) - 32;                                             \
    const short2v sc2_ = {(short)-scv_, (short)-scv_};                                            \
    const short2v c2_ = {(short)(4 * scv_), (short)(4 * scv_)};                                   \
    const uint4 &Q_ = (G) >= 2u ? wQ1 : wQ0;                                                      \
    const uint32_t qlw_[4] = {Q_.x, Q_.y, Q_.z, Q_.w}, qhw_[4] = {wH.x, wH.y, wH.z, wH.w};        \
    uint32_t pw_[4];                                                                              \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      const uint32_t v_ = ((qlw_[w_] >> (2u * (2u * ((G) & 1u) + (SUB)))) & 0x03030303u) |        \
                          (((qhw_[w_] >> (2u * (G) + (SUB))) & 0x01010101u) << 2);                \
      union { uint32_t u; short2v s; } e_, f_;                                                    \
      e_.u = __builtin_amdgcn_perm(0u, v_, 0x0c010c00u);   /* (b0, b1) as 16-bit lanes */         \
      f_.u = __builtin_amdgcn_perm(0u, v_, 0x0c030c02u);   /* (b2, b3) */                         \
      e_.s = e_.s * sc2_ + c2_;                                                                   \
      f_.s = f_.s * sc2_ + c2_;                                                                   \
      pw_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x06040200u);   /* the lanes' low bytes */      \
    }                                                                                             \
    const int4v bw_ = {(int)pw_[0], (int)pw_[1], (int)pw_[2], (int)pw_[3]};                       \
    const int4v xa_ = *(const int4v *)(p.xq + (xs_ + (64u * (G) + 32u * (SUB)) * xmul));          \
    H = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_, bw_, (FIRST) ? zi : H, 0, 0, 0);               \
  } while (0)

  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float acc[NACC];   // outputs (token, row) = (tid / 32 + a NT / 32, tid % 32)
#pragma unroll
  for (uint32_t a = 0; a < NACC; a++) acc[a] = 0.0f;
  SB3_LOADW(wave);
  __syncthreads();   // ad_l
  for (uint32_t s0 = 0; s0 < p.nsb; s0 += NW) {
    const uint32_t s = s0 + wave;
    if (s < p.nsb) {   // wave-uniform
      const uint32_t xs_ = xro + 256u * s * xmul;
      int16v H;
      SB3_STEP(0u, 0u, true);
      SB3_STEP(0u, 1u, false);
      SB3_STEP(1u, 0u, false);
      SB3_STEP(1u, 1u, false);
      SB3_STEP(2u, 0u, false);
      SB3_STEP(2u, 1u, false);
      SB3_STEP(3u, 0u, false);
      SB3_STEP(3u, 1u, false);
      const float d = gm_f16_bits_to_f32(scx.w & 0xFFFFu);
      const float *adp = &ad_l[s * 32u + 4u * lh];
      float *tp = terms + (wave * 32u + 4u * lh) * 32u + l32;   // [wave][token][row]
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const float4 a4 = *(const float4 *)(adp + 8 * q4);
        const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
        for (int e = 0; e < 4; e++) tp[(8 * q4 + e) * 32] = a4v[e] * (d * (float)(-H[4 * q4 + e]));
      }
    }
    SB3_LOADW(s + NW);   // the next round's weights, in flight over the barrier and the additions
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
#undef SB3_LOADW
#undef SB3_STEP
  {
    const uint32_t row = r0 + (tid & 31u);
#pragma unroll
    for (uint32_t a = 0; a < NACC; a++) {
      const uint32_t tok = t0 + (tid >> 5) + a * (NT / 32u);
      if (row < p.out_dim && tok < p.n_tokens) p.y[(size_t)tok * p.out_dim + row] = acc[a];
    }
  }
}

__global__ __launch_bounds__(512) void ogm_gemm_sb_q3k_kernel(GemmSbParams p) { gemm_sb_q3k_body<8u>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_sb_q3k_w16_kernel(GemmSbParams p) { gemm_sb_q3k_body<16u>(p); }

// The same for IQ4_XS (gemm_k_iq4_xs, vecdot.rs:2305-2322: Q6_K's loop with a scale per sub-block of 32).  A unit's
// 136 bytes are nine pieces (the last half used): d | scales_h | scales_l, then the eight sub-blocks' sixteen bytes of
// nibbles from byte 8 on, so sub-block ib is the upper half of piece ib and the lower half of piece ib + 1; both
// lane halves read the same bytes, the lower one their low nibbles (elements 0..15), the upper one the high ones.
// Operand planes as the plane builder makes them: u = ls (level + 128) + (128 - 128 ls).
template <uint32_t NW>
__device__ __forceinline__ void gemm_sb_iq4xs_body(GemmSbParams p) {
  constexpr uint32_t NT = 64u * NW, NACC = 1024u / NT;
  constexpr uint32_t TILE_BYTES = 9216u;
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
  uint32_t uo;
  {
    const uint32_t row = min(r0 + l32, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    uo = rb * p.nct * TILE_BYTES + r * 16u;
  }
  auto sb_off = [&](uint32_t s) -> uint32_t {
    return (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 16u;
  };
  // a lane's 16 activations of a run of 32: from its token's row, or (x_chunks) from the 1 KiB operand chunk of
  // the tile's 32 tokens and the run's 32 k, where they lie in the instruction's own order
  const uint32_t xmul = p.x_chunks ? 32u : 1u;
  const uint32_t xro = p.x_chunks ? blockIdx.x * p.in_dim * 32u + 16u * lane
                                  : min(t0 + l32, p.n_tokens - 1u) * p.in_dim + 16u * lh;   // + (256 s + 32 ib) xmul
  const uint32_t nsh = 4u * lh;

  for (uint32_t i = tid; i < 32u * p.nsb; i += NT) {
    const uint32_t k = i / p.nsb, s = i - k * p.nsb;
    ad_l[s * 32u + k] = p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + s];
  }

  uint4 pc[9];
#define SBX_LOADW(S)                                                                              \
  do {                                                                                            \
    const uint32_t s_ = min((uint32_t)(S), p.nsb - 1u); /* past the end: loaded, never used */    \
    const uint32_t so_ = uo + sb_off(s_);                                                         \
    _Pragma("unroll") for (int i_ = 0; i_ < 9; i_++) pc[i_] = *(const uint4 *)(p.wt + (so_ + i_ * 1024u)); \
  } while (0)
#define SBX_STEP(IB, FIRST)                                                                       \
  do {                                                                                            \
    const int ls_ = (int)(((sl_ >> (4u * (IB))) & 0xFu) | (((sh_ >> (2u * (IB))) & 3u) << 4)) - 32; \
    const short2v sc2_ = {(short)ls_, (short)ls_};                                                \
    const short2v c2_ = {(short)(128 - 128 * ls_), (short)(128 - 128 * ls_)};                     \
    const uint32_t qw_[4] = {pc[IB].z, pc[IB].w, pc[(IB) + 1].x, pc[(IB) + 1].y};                 \
    uint32_t ph_[4], pl_[4];                                                                      \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      const uint32_t v_ = ogm_nib32_weights<2>((qw_[w_] >> nsh) & 0x0F0F0F0Fu, 0u) ^ 0x80808080u; \
      union { uint32_t u; short2v s; } e_, f_;                                                    \
      e_.u = __builtin_amdgcn_perm(0u, v_, 0x0c010c00u);   /* (b0, b1) as 16-bit lanes */         \
      f_.u = __builtin_amdgcn_perm(0u, v_, 0x0c030c02u);   /* (b2, b3) */                         \
      e_.s = e_.s * sc2_ + c2_;                                                                   \
      f_.s = f_.s * sc2_ + c2_;                                                                   \
      ph_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x07050301u);                                   \
      pl_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x06040200u) ^ 0x80808080u;                     \
    }                                                                                             \
    const int4v bh_ = {(int)ph_[0], (int)ph_[1], (int)ph_[2], (int)ph_[3]};                       \
    const int4v bl_ = {(int)pl_[0], (int)pl_[1], (int)pl_[2], (int)pl_[3]};                       \
    const int4v xa_ = *(const int4v *)(p.xq + (xs_ + 32u * (IB) * xmul));                         \
    H = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_, bh_, (FIRST) ? zi : H, 0, 0, 0);               \
    L = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_, bl_, (FIRST) ? zi : L, 0, 0, 0);               \
  } while (0)

  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float acc[NACC];   // outputs (token, row) = (tid / 32 + a NT / 32, tid % 32)
#pragma unroll
  for (uint32_t a = 0; a < NACC; a++) acc[a] = 0.0f;
  SBX_LOADW(wave);
  __syncthreads();   // ad_l
  for (uint32_t s0 = 0; s0 < p.nsb; s0 += NW) {
    const uint32_t s = s0 + wave;
    if (s < p.nsb) {   // wave-uniform
      const uint32_t xs_ = xro + 256u * s * xmul;
      const uint32_t sh_ = pc[0].x >> 16, sl_ = pc[0].y;
      int16v H, L;
      SBX_STEP(0, true);
      SBX_STEP(1, false);
      SBX_STEP(2, false);
      SBX_STEP(3, false);
      SBX_STEP(4, false);
      SBX_STEP(5, false);
      SBX_STEP(6, false);
      SBX_STEP(7, false);
      const float d = gm_f16_bits_to_f32(pc[0].x & 0xFFFFu);
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
    SBX_LOADW(s + NW);   // the next round's weights, in flight over the barrier and the additions
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
#undef SBX_LOADW
#undef SBX_STEP
  {
    const uint32_t row = r0 + (tid & 31u);
#pragma unroll
    for (uint32_t a = 0; a < NACC; a++) {
      const uint32_t tok = t0 + (tid >> 5) + a * (NT / 32u);
      if (row < p.out_dim && tok < p.n_tokens) p.y[(size_t)tok * p.out_dim + row] = acc[a];
    }
  }
}

__global__ __launch_bounds__(512) void ogm_gemm_sb_iq4xs_kernel(GemmSbParams p) { gemm_sb_iq4xs_body<8u>(p); }
__global__ __launch_bounds__(1024) void ogm_gemm_sb_iq4xs_w16_kernel(GemmSbParams p) { gemm_sb_iq4xs_body<16u>(p); }

// Q2_K at several tokens: the reference's rows-unpacked-once path over per-32 activations (unpack_q2_k +
// dot_unpacked, vecdot.rs:1144-1164, 420-425, 1722-1728) leaves sixteen f32 terms a super-block, one per group of 16,
//   act.d[g / 2] * ((d * sc_g) * isum_g - (dmin * mn_g) * sums[g]),
// added in group order.  A workgroup owns 32 rows x 32 tokens; a round is one super-block, wave w its groups 2 w and
// 2 w + 1 (the run of 32 two-bit values w): a group is one v_mfma_i32_32x32x16_i8, the activations' sums per 16 a
// second one against ones, and the sixteen terms of the round are added in ascending order, one accumulator per
// output.  A unit's 84 bytes: scales[16], qs[64] in four pieces, d | dmin behind the tile's pieces.
typedef long sbq2_i64;

__global__ __launch_bounds__(512) void ogm_gemm_sb_q2k_kernel(GemmSbParams p) {
  constexpr uint32_t NW = 8u, NT = 64u * NW, NACC = 1024u / NT;
  constexpr uint32_t TILE_BYTES = 64u * 84u;
  extern __shared__ __align__(16) uint8_t sb_lds[];
  float *terms = (float *)sb_lds;            // [16 groups][32 tokens][32 rows]
  float *ad_l = terms + 16u * 1024u;         // [in_dim / 32][32 tokens]
  const uint32_t nblk = p.in_dim / 32u;

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
  uint32_t tile_row, rr;
  {
    const uint32_t row = min(r0 + l32, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
    const uint32_t rb = row >> p.r_shift;
    rr = row & ((1u << p.r_shift) - 1u);
    tile_row = rb * p.nct * TILE_BYTES;
  }
  const uint32_t xro = min(t0 + l32, p.n_tokens - 1u) * p.in_dim + 8u * lh;   // + 256 s + 16 g

  for (uint32_t i = tid; i < 32u * nblk; i += NT) {
    const uint32_t k = i / nblk, b = i - k * nblk;
    ad_l[b * 32u + k] = p.ad[min(t0 + k, p.n_tokens - 1u) * nblk + b];
  }

  // the wave's part of a unit: the scales, the two pieces of its run's 32 bytes (bytes 16 h .. of qs[32 (w / 4) ..]),
  // d | dmin
  uint4 wsc, wq0, wq1;
  uint32_t dd;
  const uint32_t qpiece = 1u + 2u * (wave >> 2), qshift = 2u * (wave & 3u);
#define SBQ2_LOADW(S)                                                                             \
  do {                                                                                            \
    const uint32_t s_ = min((uint32_t)(S), p.nsb - 1u); /* past the end: loaded, never used */    \
    const uint32_t to_ = tile_row + (s_ >> p.c_shift) * TILE_BYTES;                               \
    const uint32_t ln_ = ((s_ & ((1u << p.c_shift) - 1u)) << p.r_shift) + rr;                     \
    wsc = *(const uint4 *)(p.wt + (to_ + ln_ * 16u));                                             \
    wq0 = *(const uint4 *)(p.wt + (to_ + ln_ * 16u + qpiece * 1024u));                            \
    wq1 = *(const uint4 *)(p.wt + (to_ + ln_ * 16u + (qpiece + 1u) * 1024u));                     \
    dd = *(const uint32_t *)(p.wt + (to_ + 5u * 1024u + ln_ * 4u));                               \
  } while (0)

  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const sbq2_i64 ones = 0x0101010101010101L;
  float acc[NACC];   // outputs (token, row) = (tid / 32 + a NT / 32, tid % 32)
#pragma unroll
  for (uint32_t a = 0; a < NACC; a++) acc[a] = 0.0f;
  SBQ2_LOADW(0u);
  __syncthreads();   // ad_l
  for (uint32_t s = 0; s < p.nsb; s++) {
    const float d = gm_f16_bits_to_f32(dd & 0xFFFFu), dmin = gm_f16_bits_to_f32(dd >> 16);
    const uint32_t scw = wave < 2u ? wsc.x : wave < 4u ? wsc.y : wave < 6u ? wsc.z : wsc.w;   // scales[2 w], [2 w + 1] in it
#pragma unroll
    for (uint32_t h = 0; h < 2u; h++) {
      const uint32_t g = 2u * wave + h;
      const uint4 &Q = h ? wq1 : wq0;
      union { uint32_t w[2]; sbq2_i64 v; } bw, xa;
      bw.w[0] = ((lh ? Q.z : Q.x) >> qshift) & 0x03030303u;   // the lane's eight weights: k 8 lh .. of its row's group
      bw.w[1] = ((lh ? Q.w : Q.y) >> qshift) & 0x03030303u;
      const uint2 xv = *(const uint2 *)(p.xq + (xro + 256u * s + 16u * g));
      xa.w[0] = xv.x;
      xa.w[1] = xv.y;
      const int16v C = __builtin_amdgcn_mfma_i32_32x32x16_i8(xa.v, bw.v, zi, 0, 0, 0);
      const int16v S = __builtin_amdgcn_mfma_i32_32x32x16_i8(xa.v, ones, zi, 0, 0, 0);   // the tokens' sums of the group
      const uint32_t scb = (scw >> (8u * (2u * (wave & 1u) + h))) & 0xFFu;
      const float scale = d * (float)(scb & 0xFu), mn = dmin * (float)(scb >> 4);
      const float *adp = &ad_l[(8u * s + wave) * 32u + 4u * lh];
      float *tp = terms + (g * 32u + 4u * lh) * 32u + l32;   // [group][token][row]
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        const float4 a4 = *(const float4 *)(adp + 8 * q4);
        const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
        for (int e = 0; e < 4; e++)
          tp[(8 * q4 + e) * 32] = a4v[e] * (scale * (float)C[4 * q4 + e] - mn * (float)S[4 * q4 + e]);
      }
    }
    SBQ2_LOADW(s + 1u);   // the next round's weights, in flight over the barrier and the additions
    __syncthreads();
#pragma unroll
    for (uint32_t g = 0; g < 16u; g++) {   // ascending groups, one accumulator per output
#pragma unroll
      for (uint32_t a = 0; a < NACC; a++) acc[a] += terms[g * 1024u + a * NT + tid];
    }
    __syncthreads();
  }
#undef SBQ2_LOADW
  {
    const uint32_t row = r0 + (tid & 31u);
#pragma unroll
    for (uint32_t a = 0; a < NACC; a++) {
      const uint32_t tok = t0 + (tid >> 5) + a * (NT / 32u);
      if (row < p.out_dim && tok < p.n_tokens) p.y[(size_t)tok * p.out_dim + row] = acc[a];
    }
  }
}

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
  float *terms = (float *)sb_lds;             // [NW super-blocks][32 tokens][32 rows]
  float *ad_l = terms + NW * 32u * 32u;       // [nsb][32 tokens]

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
  // a lane's 16 activations of a sub-block: from its token's row, or (x_chunks) from the 1 KiB operand chunk of
  // the tile's 32 tokens and the sub-block's 32 k, where they lie in the instruction's own order
  const uint32_t xmul = p.x_chunks ? 32u : 1u;
  const uint32_t xro = p.x_chunks ? blockIdx.x * p.in_dim * 32u + 16u * lane : tok * p.in_dim + 16u * lh;   // + (256 s + 32 j) xmul
  const uint32_t tk = tok * p.nsb;

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
  SB_LOADW(wave);   // the second sweep's first weights: under way during the first sweep
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
    for (uint32_t s0 = 0; s0 < p.nsb; s0 += NW) {
      {
        const uint32_t sl = wave, s = s0 + sl;
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
      const uint32_t n_here = min(NW, p.nsb - s0);
      for (uint32_t w = 0; w < n_here; w++) {
#pragma unroll
        for (uint32_t a = 0; a < NACC; a++) acc[a] -= terms[w * 1024u + a * NT + tid];
      }
      __syncthreads();
    }
  }
  // ---- second sweep: acc += ad * (d * sum_j sc_j * dot32_j)
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
    const int4v xa_ = *(const int4v *)(p.xq + (xs_ + 32u * (J) * xmul));                          \
    D = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa_, b_, zi, 0, 0, 0);                              \
  } while (0)
#define SB_ACC(D, J, FIRST)                                                                       \
  do {                                                                                            \
    const int sc_ = (int)((((J) < 4 ? sca_ : scb_) >> (8u * ((J) & 3u))) & 0xFFu);                \
    _Pragma("unroll") for (int r_ = 0; r_ < 16; r_++)                                             \
      I[r_] = (FIRST) ? __mul24(sc_, D[r_]) : __mul24(sc_, D[r_]) + I[r_];                        \
  } while (0)
  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  for (uint32_t s0 = 0; s0 < p.nsb; s0 += NW) {
    const uint32_t s = s0 + wave;
    if (s < p.nsb) {   // wave-uniform
      const uint32_t xs_ = xro + 256u * s * xmul;
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
// Medium batches of Q4_K / Q5_K (some 65 to 256 tokens over a matrix whose 128 x 128 tiles would leave compute
// units idle): the small-batch scheme on 32 rows x 128 tokens.  A workgroup has four waves, wave w takes the
// super-blocks s = w (mod 4); it unpacks a sub-block's 16 weights per lane once into the two scale-folded int8
// planes (u = sc_j q + 128 = 256 h + (l + 128)) and multiplies them with the four token blocks' activations,
// which it reads as whole operand chunks (the quantizer's second layout) straight from memory: two plain chains of
// v_mfma_i32_32x32x32_i8 per token block over the super-block, isum = 256 H + L.  The terms ad * (d * isum) -- and,
// in a sweep of their own before, (ad * dmin) * imin -- go to LDS and are added in ascending super-block order after
// every round of four, one accumulator per output: gemm_k_q4_k's sequence (vecdot.rs:2213-2303).

struct GemmSbwParams {
  const uint8_t *wt;      // tile-planar weights
  const int8_t *xt;       // the int8 activations in operand chunks: [T / 32][in_dim / 32] x 1 KiB
  const float *ad;        // [T][nsb]
  const _Float16 *bs16;   // the quantizer's sums per 32 as (bsum / 64, bsum % 64) in f16
  float *y;               // [T][out_dim]
  uint32_t in_dim, out_dim, n_tokens, nsb;
  uint32_t c_shift, r_shift, nct;
  uint32_t n_extra;
  const uint8_t *extra_wt[OGM_GEMM_MAX_MATS - 1];
  float *extra_y[OGM_GEMM_MAX_MATS - 1];
  uint32_t extra_out_dim[OGM_GEMM_MAX_MATS - 1];
};

#ifndef SBW_ABL
#define SBW_ABL 0   // timing experiments only: 1 no activation loads after a super-block's first, 2 no first sweep, 4 no ordered adds
#endif
#define SBW_NW 4u
#define SBW_TOK 128u
#define SBW_TERMS_BYTES (SBW_NW * SBW_TOK * 32u * 4u)   // 64 KB

template <bool Q5>
__global__ __launch_bounds__(64 * SBW_NW, 2) void ogm_gemm_sbw_q45k_kernel(GemmSbwParams p) {
  constexpr uint32_t TILE_BYTES = Q5 ? 11264u : 9216u;
  constexpr uint32_t QS_PIECE0 = Q5 ? 3u : 1u;
  constexpr uint32_t NT = 64u * SBW_NW, NACC = SBW_TOK * 32u / NT;   // 16 outputs a thread
  extern __shared__ __align__(16) uint8_t sbw_lds[];
  float *terms = (float *)sbw_lds;                 // [4 waves][128 tokens][32 rows]
  float *ad_l = terms + SBW_NW * SBW_TOK * 32u;    // [nsb][128 tokens]

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
  const uint32_t t0 = blockIdx.x * SBW_TOK, r0 = row_tile * 32u;
  uint32_t uo;   // this lane's row: its header piece
  {
    const uint32_t row = min(r0 + l32, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
    const uint32_t rb = row >> p.r_shift, r = row & ((1u << p.r_shift) - 1u);
    uo = rb * p.nct * TILE_BYTES + r * 16u;
  }
  auto sb_off = [&](uint32_t s) -> uint32_t {
    return (s >> p.c_shift) * TILE_BYTES + ((s & ((1u << p.c_shift) - 1u)) << p.r_shift) * 16u;
  };

  for (uint32_t i = tid; i < SBW_TOK * p.nsb; i += NT) {
    const uint32_t k = i / p.nsb, s = i - k * p.nsb;
    ad_l[s * SBW_TOK + k] = p.ad[min(t0 + k, p.n_tokens - 1u) * p.nsb + s];
  }
  __syncthreads();

  float acc[NACC];   // outputs (token, row) = (tid / 32 + 8 a, tid % 32)
#pragma unroll
  for (uint32_t a = 0; a < NACC; a++) acc[a] = 0.0f;
  // the first round's weights of the second sweep are in flight over the first
  uint4 hdr, w0, w1, w2, w3, qh5 = make_uint4(0, 0, 0, 0);
#define SBW_LOADW(S)                                                                              \
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
  SBW_LOADW(wave);

  // ---- first sweep: acc -= (ad * dmin) * sum_j m_j * bsum_j, every super-block, in order
  if (!(SBW_ABL & 2)) {
    float16v zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.0f;
    const float side_scale = lh ? 1.0f : 64.0f;
    uint32_t tk[4];
#pragma unroll
    for (int tb = 0; tb < 4; tb++) tk[tb] = min(t0 + 32u * tb + l32, p.n_tokens - 1u) * p.nsb;
    // (a round's header and sums are requested a round ahead: past the end they are loaded again, never used)
    uint4 hd_n = *(const uint4 *)(p.wt + (uo + sb_off(min(wave, p.nsb - 1u))));
    half8 b2_n[4];
#pragma unroll
    for (int tb = 0; tb < 4; tb++) b2_n[tb] = *(const half8 *)(p.bs16 + ((tk[tb] + min(wave, p.nsb - 1u)) * 16u + 8u * lh));
    for (uint32_t s0 = 0; s0 < p.nsb; s0 += SBW_NW) {
      const uint32_t s = s0 + wave;
      const uint4 hd = hd_n;
      half8 b2[4];
#pragma unroll
      for (int tb = 0; tb < 4; tb++) b2[tb] = b2_n[tb];
      {
        const uint32_t sn = min(s + SBW_NW, p.nsb - 1u);
        hd_n = *(const uint4 *)(p.wt + (uo + sb_off(sn)));
#pragma unroll
        for (int tb = 0; tb < 4; tb++) b2_n[tb] = *(const half8 *)(p.bs16 + ((tk[tb] + sn) * 16u + 8u * lh));
      }
      if (s < p.nsb) {   // wave-uniform
        uint32_t mna, mnb;
        q4k_mins(hd, mna, mnb);
        const half8 a1 = side_operand(mna, mnb, side_scale);
        const float dm = gm_f16_bits_to_f32(hd.x >> 16);
#pragma unroll
        for (int tb = 0; tb < 4; tb++) {
          const float16v im = __builtin_amdgcn_mfma_f32_32x32x16_f16(b2[tb], a1, zero, 0, 0, 0);
          const float *adp = &ad_l[s * SBW_TOK + 32u * tb + 4u * lh];
          float *tp = terms + (wave * SBW_TOK + 32u * tb + 4u * lh) * 32u + l32;   // [wave][token][row]
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
      const uint32_t n_here = min(SBW_NW, p.nsb - s0);
      for (uint32_t w = 0; w < n_here; w++) {
#pragma unroll
        for (uint32_t a = 0; a < NACC; a++) acc[a] -= terms[w * (SBW_TOK * 32u) + a * NT + tid];
      }
      __syncthreads();
    }
  }

  // ---- second sweep: acc += ad * (d * sum_j sc_j * dot32_j)
  // (token blocks past the last one read it again; their outputs are never stored)
  uint32_t xo[4];
#pragma unroll
  for (int tb = 0; tb < 4; tb++)
    xo[tb] = min((t0 >> 5) + (uint32_t)tb, (p.n_tokens - 1u) >> 5) * (p.in_dim / 32u) * 1024u + lane * 16u;   // + (8 s + j) * 1024
#define SBW_LOADX(DST, XS, J)                                                                     \
  do {                                                                                            \
    if ((SBW_ABL & 1) && (J) > 1) break;                                                          \
    _Pragma("unroll") for (int tb_ = 0; tb_ < 4; tb_++)                                           \
      DST[tb_] = *(const int4v *)(p.xt + (xo[tb_] + (XS) + 1024u * (J)));                         \
  } while (0)
  // sub-block J: its 16 weights per lane -> the two planes, then the four token blocks
#define SBW_STEP(QS, J, XA, FIRST)                                                                \
  do {                                                                                            \
    const int sc_ = (int)((((J) < 4 ? sca_ : scb_) >> (8u * ((J) & 3u))) & 0xFFu);                \
    const short2v sc2_ = {(short)sc_, (short)sc_};                                                \
    const short2v c2_ = {(short)128, (short)128};                                                 \
    const uint32_t qsw_[4] = {QS.x, QS.y, QS.z, QS.w}, q5w_[4] = {qh5.x, qh5.y, qh5.z, qh5.w};    \
    uint32_t ph_[4], pl_[4];                                                                      \
    _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                            \
      uint32_t v_ = (((J) & 1) ? (qsw_[w_] >> 4) : qsw_[w_]) & 0x0F0F0F0Fu;                       \
      if constexpr (Q5) v_ |= ((q5w_[w_] >> (J)) & 0x01010101u) << 4;                             \
      union { uint32_t u; short2v s; } e_, f_;                                                    \
      e_.u = __builtin_amdgcn_perm(0u, v_, 0x0c010c00u);   /* (b0, b1) as 16-bit lanes */         \
      f_.u = __builtin_amdgcn_perm(0u, v_, 0x0c030c02u);   /* (b2, b3) */                         \
      e_.s = e_.s * sc2_ + c2_;                                                                   \
      f_.s = f_.s * sc2_ + c2_;                                                                   \
      ph_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x07050301u);                                   \
      pl_[w_] = __builtin_amdgcn_perm(f_.u, e_.u, 0x06040200u) ^ 0x80808080u;                     \
    }                                                                                             \
    const int4v bh_ = {(int)ph_[0], (int)ph_[1], (int)ph_[2], (int)ph_[3]};                       \
    const int4v bl_ = {(int)pl_[0], (int)pl_[1], (int)pl_[2], (int)pl_[3]};                       \
    _Pragma("unroll") for (int tb_ = 0; tb_ < 4; tb_++) {                                         \
      H[tb_] = __builtin_amdgcn_mfma_i32_32x32x32_i8(XA[tb_], bh_, (FIRST) ? zi : H[tb_], 0, 0, 0); \
      L[tb_] = __builtin_amdgcn_mfma_i32_32x32x32_i8(XA[tb_], bl_, (FIRST) ? zi : L[tb_], 0, 0, 0); \
    }                                                                                             \
  } while (0)
  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  for (uint32_t s0 = 0; s0 < p.nsb; s0 += SBW_NW) {
    const uint32_t s = s0 + wave;
    if (s < p.nsb) {   // wave-uniform
      const uint32_t xs_ = 8192u * s;   // eight chunks a super-block
      uint32_t sca_, scb_;
      q4k_scales(hdr, sca_, scb_);
      int16v H[4], L[4];
      int4v xa[4], xb[4];
      SBW_LOADX(xa, xs_, 0);
      SBW_LOADX(xb, xs_, 1);
      SBW_STEP(w0, 0, xa, true);
      SBW_LOADX(xa, xs_, 2);
      SBW_STEP(w0, 1, xb, false);
      SBW_LOADX(xb, xs_, 3);
      SBW_STEP(w1, 2, xa, false);
      SBW_LOADX(xa, xs_, 4);
      SBW_STEP(w1, 3, xb, false);
      SBW_LOADX(xb, xs_, 5);
      SBW_STEP(w2, 4, xa, false);
      SBW_LOADX(xa, xs_, 6);
      SBW_STEP(w2, 5, xb, false);
      SBW_LOADX(xb, xs_, 7);
      SBW_STEP(w3, 6, xa, false);
      SBW_STEP(w3, 7, xb, false);
      const float d = gm_f16_bits_to_f32(hdr.x & 0xFFFFu);
#pragma unroll
      for (int tb = 0; tb < 4; tb++) {
        const float *adp = &ad_l[s * SBW_TOK + 32u * tb + 4u * lh];
        float *tp = terms + (wave * SBW_TOK + 32u * tb + 4u * lh) * 32u + l32;   // [wave][token][row]
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const float4 a4 = *(const float4 *)(adp + 8 * q4);
          const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const int is_ = H[tb][4 * q4 + e] * 256 + L[tb][4 * q4 + e];
            tp[(8 * q4 + e) * 32] = a4v[e] * (d * (float)is_);
          }
        }
      }
    }
    SBW_LOADW(s + SBW_NW);   // the next round's weights, in flight over the barrier and the additions
    __syncthreads();
    if (!(SBW_ABL & 4) || s0 == 0) {
      const uint32_t n_here = min(SBW_NW, p.nsb - s0);
      for (uint32_t w = 0; w < n_here; w++) {   // ascending super-blocks, one accumulator per output
#pragma unroll
        for (uint32_t a = 0; a < NACC; a++) acc[a] += terms[w * (SBW_TOK * 32u) + a * NT + tid];
      }
    }
    __syncthreads();
  }
#undef SBW_LOADW
#undef SBW_LOADX
#undef SBW_STEP
  {
    const uint32_t row = r0 + (tid & 31u);
#pragma unroll
    for (uint32_t a = 0; a < NACC; a++) {
      const uint32_t tok_o = t0 + (tid >> 5) + a * (NT / 32u);
      if (row < p.out_dim && tok_o < p.n_tokens) p.y[(size_t)tok_o * p.out_dim + row] = acc[a];
    }
  }
}

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
// Small batches of the per-32 types: the workgroup above walks a row's blocks one stage after the other, 70 us for
// 4096 inputs however few the tokens.  Here, as in the K-quants' small-batch kernel, a workgroup owns 32 rows x 32
// tokens and its eight waves take different blocks at the same time -- a block is one v_mfma_i32_32x32x32_i8, the
// int8 weights unpacked straight into the operand registers, the activations read from memory as they are -- and
// leave the blocks' terms (ad * dw) * dot32 (vecdot.rs:2622) in LDS; after every round of sixteen blocks the terms
// are added in ascending order, one accumulator per output, as dot_flat_pair does (vecdot.rs:2598-2629).
#define SBF_NB 2u   // blocks a wave takes per round

// KIND 0: Q4_0, 1: Q5_0, 2: IQ4_NL, 3: Q8_0, 4: Q5_1 -- whose blocks also have a minimum: the term of a block is
// ad * (dw * dot32 + m * block_sum) (dot_q5_1, vecdot.rs:2886-2899, which its several-token path equals bit for
// bit), the block's sum of activations per token from a second matrix instruction against ones.
template <int KIND, uint32_t NW>
__device__ __forceinline__ void gemm_sb_flat_body(GemmSbParams p) {
  constexpr uint32_t NT = 64u * NW, NACC = 1024u / NT;
  constexpr uint32_t PIECES = KIND == 3 ? 2u : 1u;
  constexpr uint32_t TAIL = KIND == 1 ? 6u : KIND == 4 ? 8u : 2u;
  constexpr int NIB = KIND == 4 ? 3 : KIND;   // ogm_nib32_weights' kind
  constexpr uint32_t TILE = 64u * (16u * PIECES + TAIL);
  extern __shared__ __align__(16) uint8_t sb_lds[];
  // The tokens' ad of one round at a time, in two buffers: every thread fetches one value (block, token) a round
  // ahead and stores it behind the round's additions, so no pass over all of a row's blocks comes first and the
  // LDS does not grow with the rows.
  constexpr uint32_t RB = NW * SBF_NB;             // blocks of a round (NT = 32 RB threads)
  constexpr uint32_t ADS = 36u;                    // floats between the blocks of a round's ad: 16-byte rows, spread over the banks
  float *terms = (float *)sb_lds;                  // [RB blocks of the round][32 tokens][32 rows]
  float *ad_l = terms + RB * 1024u;                // [2][RB blocks][ADS]
  const uint32_t nblk = p.nsb;                     // (blocks of 32 here)

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const uint32_t t0 = blockIdx.x * 32u, r0 = blockIdx.y * 32u;
  uint32_t tile_row, rr;
  {
    const uint32_t row = min(r0 + l32, p.out_dim - 1u);   // rows past the matrix: clamped, never stored
    const uint32_t rb = row >> p.r_shift;
    rr = row & ((1u << p.r_shift) - 1u);
    tile_row = rb * p.nct * TILE;
  }
  const uint32_t xro = min(t0 + l32, p.n_tokens - 1u) * p.in_dim + 16u * lh;   // + 32 b

  const uint32_t ad_k = tid / RB, ad_b = tid % RB;   // this thread's token and block of a round
  const uint32_t ad_src = min(t0 + ad_k, p.n_tokens - 1u) * nblk;
  ad_l[ad_b * ADS + ad_k] = p.ad[ad_src + min(ad_b, nblk - 1u)];

  uint4 wq[SBF_NB];
  uint32_t tl[SBF_NB], th[SBF_NB];
#define SBF_LOADW(B0)                                                                                   \
  do {                                                                                                  \
    _Pragma("unroll") for (uint32_t j_ = 0; j_ < SBF_NB; j_++) {                                        \
      const uint32_t b_ = min((uint32_t)(B0) + j_, nblk - 1u); /* past the end: loaded, never used */   \
      const uint32_t to_ = tile_row + (b_ >> p.c_shift) * TILE;                                         \
      const uint32_t ln_ = ((b_ & ((1u << p.c_shift) - 1u)) << p.r_shift) + rr;                         \
      wq[j_] = *(const uint4 *)(p.wt + (to_ + ln_ * 16u + (KIND == 3 ? lh * 1024u : 0u)));              \
      const uint16_t *tp_ = (const uint16_t *)(p.wt + (to_ + PIECES * 1024u + ln_ * TAIL));             \
      tl[j_] = KIND == 4 ? ((uint32_t)tp_[0] | ((uint32_t)tp_[1] << 16)) : (uint32_t)tp_[0]; /* d (| m) */ \
      th[j_] = KIND == 1 ? ((uint32_t)tp_[1] | ((uint32_t)tp_[2] << 16))                                \
               : KIND == 4 ? ((uint32_t)tp_[2] | ((uint32_t)tp_[3] << 16)) : 0u;                        \
    }                                                                                                   \
  } while (0)

  const int16v zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float acc[NACC];   // outputs (token, row) = (tid / 32 + a NT / 32, tid % 32)
#pragma unroll
  for (uint32_t a = 0; a < NACC; a++) acc[a] = 0.0f;
  SBF_LOADW(wave * SBF_NB);
  __syncthreads();   // ad_l
  uint32_t ad_buf = 0;   // the buffer of this round
  for (uint32_t s0 = 0; s0 < nblk; s0 += RB) {
    const uint32_t b0 = s0 + wave * SBF_NB;
    const float ad_next = p.ad[ad_src + min(s0 + RB + ad_b, nblk - 1u)];   // (past the end: never used)
#pragma unroll
    for (uint32_t j = 0; j < SBF_NB; j++) {
      const uint32_t b = b0 + j;
      if (b < nblk) {   // wave-uniform
        int4v bw;   // the lane's sixteen weights: k 16 lh .. 16 lh + 15 of its row's block
        if (KIND == 3) {
          bw = (int4v){(int)wq[j].x, (int)wq[j].y, (int)wq[j].z, (int)wq[j].w};
        } else {
          // byte i of the sixteen: weight i in its low nibble, weight 16 + i in its high one; Q5_0's fifth bits: bit i
          const uint32_t q_[4] = {wq[j].x, wq[j].y, wq[j].z, wq[j].w};
          uint32_t w_[4];
#pragma unroll
          for (int k_ = 0; k_ < 4; k_++)
            w_[k_] = ogm_nib32_weights<NIB>((lh ? q_[k_] >> 4 : q_[k_]) & 0x0F0F0F0Fu, (th[j] >> (16u * lh + 4u * k_)) & 0xFu);
          bw = (int4v){(int)w_[0], (int)w_[1], (int)w_[2], (int)w_[3]};
        }
        const int4v xa = *(const int4v *)(p.xq + (xro + 32u * b));
        const int16v C = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa, bw, zi, 0, 0, 0);
        int16v S = zi;   // Q5_1: the tokens' sums of this block's activations, in every column
        if constexpr (KIND == 4) {
          const int4v ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
          S = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa, ones, zi, 0, 0, 0);
        }
        const float d = gm_f16_bits_to_f32(tl[j] & 0xFFFFu), mn = KIND == 4 ? gm_f16_bits_to_f32(tl[j] >> 16) : 0.0f;
        const float *adp = &ad_l[ad_buf * (RB * ADS) + (b - s0) * ADS + 4u * lh];
        float *tp = terms + ((wave * SBF_NB + j) * 32u + 4u * lh) * 32u + l32;   // [block of the round][token][row]
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          const float4 a4 = *(const float4 *)(adp + 8 * q4);
          const float a4v[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if constexpr (KIND == 4)
              tp[(8 * q4 + e) * 32] = a4v[e] * (d * (float)C[4 * q4 + e] + mn * (float)S[4 * q4 + e]);
            else
              tp[(8 * q4 + e) * 32] = (a4v[e] * d) * (float)C[4 * q4 + e];
          }
        }
      }
    }
    SBF_LOADW(b0 + RB);   // the next round's weights, in flight over the barrier and the additions
    __syncthreads();
    {
      const uint32_t n_here = min(RB, nblk - s0);
      for (uint32_t w = 0; w < n_here; w++) {   // ascending blocks, one accumulator per output
#pragma unroll
        for (uint32_t a = 0; a < NACC; a++) acc[a] += terms[w * 1024u + a * NT + tid];
      }
    }
    ad_buf ^= 1u;   // the next round's ad into the buffer the round before this one read
    ad_l[ad_buf * (RB * ADS) + ad_b * ADS + ad_k] = ad_next;
    __syncthreads();
  }
#undef SBF_LOADW
  {
    const uint32_t row = r0 + (tid & 31u);
#pragma unroll
    for (uint32_t a = 0; a < NACC; a++) {
      const uint32_t tok = t0 + (tid >> 5) + a * (NT / 32u);
      if (row < p.out_dim && tok < p.n_tokens) p.y[(size_t)tok * p.out_dim + row] = acc[a];
    }
  }
}

template <int KIND>
__global__ __launch_bounds__(512) void ogm_gemm_sb_flat_kernel(GemmSbParams p) { gemm_sb_flat_body<KIND, 8u>(p); }
// Sixteen waves: half as many rounds, for launches that leave compute units idle.
template <int KIND>
__global__ __launch_bounds__(1024) void ogm_gemm_sb_flat_w16_kernel(GemmSbParams p) { gemm_sb_flat_body<KIND, 16u>(p); }

static const uint32_t GM_LDS_MAX = 160 * 1024;   // LDS of a CU

size_t ogm_gemm_xh_bytes(uint32_t in_dim, uint32_t n_tokens) {
  // the int8 activations in operand chunks (token count rounded up to 32), for the all-waves-multiply kernel
  return (size_t)in_dim * ((n_tokens + 31u) & ~31u);
}

// LDS of the per-32 types' small-batch kernel with NW waves: a round's terms and two rounds' ad.
static uint32_t gemm_flat_small_lds(uint32_t nw) { return nw * SBF_NB * 4096u + 2u * nw * SBF_NB * 36u * 4u; }

// Whether a launch of the per-32 types takes their small-batch kernel: while its workgroups of 32 rows x 32 tokens
// are few enough, about seven rounds of the device's compute units (two workgroups share one).  Measured on MI355X,
// Q8_0, whole calls, us, small-batch against tiled: 4096 -> 4096 at 32 / 128 / 384 / 512 tokens 14.5 / 24.5 / 62 / 91
// against 72 / 76 / 82 / 84; 4096 -> 14336 at 32 / 128 / 192: 26 / 73 / 125 against 77 / 82 / 89; 14336 -> 4096 at 32 /
// 128 / 256: 42 / 73 / 134 against 239 / 243 / 252; 8192 -> 2048 at 128 / 384: 28 / 67.  (Q4_0, Q5_0, IQ4_NL within a
// few per cent.)
static bool gemm_flat_small(uint32_t n_tokens, uint32_t out_dim) {
  const uint32_t wgs = ((n_tokens + 31u) / 32u) * ((out_dim + 31u) / 32u);
  return wgs <= 1792u;
}

bool ogm_gemm_flat_small_batch(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim, uint32_t n_tokens) {
  if (in_dim % 64u != 0) return false;
  return ggml_type == OGM_Q5_1 || gemm_flat_small(n_tokens, out_dim);   // (Q5_1 has no other GEMM kernel)
}

// The per-32 types with a GEMM kernel: the four symmetric ones (small-batch and tiled), and Q5_1 (small-batch only).
static bool is_flat32(uint32_t t) {
  return t == OGM_Q8_0 || t == OGM_Q5_0 || t == OGM_Q4_0 || t == OGM_IQ4_NL || t == OGM_Q5_1;
}

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
  // (IQ4_XS: a small-batch kernel, and beyond the small batches only the kernels over prebuilt planes, where its
  // planes can be had: see ogm_gemm_takes_small_batch)
  // Q2_K (over per-32 activations): one kernel, whose table of the tokens' scales must fit beside its terms; it pays
  // from about nine tokens (4096 -> 4096 at 4 / 9 / 16 / 512 tokens 35 / 36 / 36 / 186 us against the GEMV kernel's
  // 20 / 29 / 56 / 1467; 14336 -> 4096 at 4 / 9 / 512: 111 / 109 / 912 against 83 / 184 / 10014)
  if (ggml_type == OGM_Q2_K)
    return n_tokens >= 9u && in_dim != 0 && in_dim % 256u == 0 && 16u * 4096u + 128u * (in_dim / 32u) <= GM_LDS_MAX &&
           (uint64_t)ogm_tiling_for(in_dim / 256u, out_dim).nrb * 64u * (in_dim / 256u) * 84u <= lim &&
           (uint64_t)in_dim * n_tokens <= lim;
  if ((ggml_type != OGM_Q4_K && ggml_type != OGM_Q6_K && ggml_type != OGM_Q3_K && ggml_type != OGM_Q5_K &&
       ggml_type != OGM_IQ4_XS) ||
      in_dim == 0 || in_dim % 256u != 0)
    return false;
  // Q4_K and Q5_K: the first pass of the tiled kernels keeps the tokens' scales of every super-block in LDS
  // (512 bytes a super-block beside 96 KB of stages); longer rows stay on the GEMV kernel, in chunks of tokens
  if ((ggml_type == OGM_Q4_K || ggml_type == OGM_Q5_K) && (size_t)(in_dim / 256u) * 512u + 98304u > GM_LDS_MAX) return false;
  const uint64_t block = (ggml_type == OGM_Q4_K || ggml_type == OGM_IQ4_XS) ? 144u : ggml_type == OGM_Q6_K ? 210u
                         : ggml_type == OGM_Q3_K ? 112u : 176u;   // bytes a block takes in the tile-planar copy
  return (uint64_t)ogm_tiling_for(in_dim / 256u, out_dim).nrb * 64u * (in_dim / 256u) * block <= lim &&
         (uint64_t)in_dim * n_tokens * 2u <= lim;
}

size_t ogm_gemm_plane_bytes(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim) {
  if ((ggml_type != OGM_Q4_K && ggml_type != OGM_Q6_K && ggml_type != OGM_Q3_K && ggml_type != OGM_Q5_K &&
       ggml_type != OGM_IQ4_XS) ||
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
    case OGM_IQ4_XS: hipLaunchKernelGGL(ogm_gemm_build_planes_kernel<GP_IQ4XS>, grid, dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL(ogm_gemm_build_planes_kernel<GP_Q5K>, grid, dim3(256), 0, stream, p); break;
  }
  return hipGetLastError();
}

// Whether a launch over planes takes the kernel with 64-row tiles that adds a super-block up between the next one's
// matrix instructions (ogm_gemm_dmx_kernel) instead of the one with 128-row tiles (ogm_gemm_dma_kernel).
// interleave: 0 by the size of the launch, 1 never, 2 whenever the type allows.  Measured on MI355X, whole calls at
// 512 tokens, us, 64-row interleaved / 128-row / feeding waves: Q6_K 14336 -> 4096 103 / 153 / 126, Q4_K 4096 ->
// 4096 42 / 64 / 49, 4096 -> 6144 54 / 67 / 64, 14336 -> 4096 130 / 204 / 150; but 4096 -> 14336 115 / 98 / -.
// Its workgroups (64 rows x 128 tokens) must fit the device in one round, two to a compute unit: beyond 512 of
// them the 128-row kernel is ahead (Q4_K 4096 -> 14336 at 384 tokens, 672 workgroups: 91 against 87; 5120 -> 13824
// at 288: 104 against 99; 8192 -> 10240 at 512: 174 against 165).
//   Q6_K has no first pass to pay for and no medium-batch kernel beside it, so it takes this kernel from 128
// workgroups on, and from 96 with at least 192 tokens, before the small-batch kernel is asked (against the small-batch
// and feeding-wave kernels: 14336 -> 4096 at 256 tokens 87 against 101, 4096 -> 4096 at 256 28 against 38, 8192 ->
// 2048 at 384 50 against 61, 13824 -> 5120 at 160 79 against 93, 28672 -> 8192 at 128 171 against 199; level with
// them at 160 tokens of the 4096-row matrices; behind with fewer workgroups: 8192 -> 2048 at 256 tokens, 64 of them,
// 47 against 38).  A lone token tile wants to be nearly full.
//   Q4_K / Q5_K want three token tiles and 160 workgroups (at 256 tokens it only draws with the medium-batch kernel,
// which needs no planes: 4096 -> 6144 37 against 37), and with longer rows than 5120 inputs no more workgroups than
// compute units (8192 -> 8192 at 384 / 512 tokens, 384 / 512 workgroups, 114 / 127 against 101 / 113 for the
// feeding-wave kernel, 8192 -> 10240 at 384 120 against 108; but 14336 -> 4096 at 384 / 512 tokens, 192 / 256
// workgroups, 121 / 127 against 135 / 143).
// for_small_batch: asked by gemm_small_batch, whether the launch is one this kernel takes ahead of the small batches.
static bool gemm_interleaved(const OgmGemmArgs &a, bool for_small_batch = false) {
  const uint32_t nsb = a.in_dim / 256;
  const bool q45 = a.ggml_type == OGM_Q4_K || a.ggml_type == OGM_Q5_K, xs = a.ggml_type == OGM_IQ4_XS;
  if (a.interleave == 1u || a.ggml_type == OGM_Q3_K || (q45 && a.one_pass != 0u) || nsb * 512u > GX_TAB ||
      a.n_tokens < (xs ? 17u : 32u))
    return false;
  if (a.interleave == 2u) return true;
  uint32_t tiles64 = 0;
  for (uint32_t m = 0; m <= a.n_extra; m++) tiles64 += ((m ? a.extra_out_dim[m - 1] : a.out_dim) + 63u) / 64u;
  const uint32_t tok_tiles = (a.n_tokens + 127u) / 128u;
  const uint32_t n_wg = tok_tiles * tiles64;
  if (n_wg > 512u) return false;
  // (beyond its small batches IQ4_XS has the two plane kernels only: 4096 -> 4096 at 32 tokens 28 us against 46 on the
  // 128-row tiles, 14336 -> 4096 77 against 141, 4096 -> 14336 33 against 50)
  if (xs && !for_small_batch) return true;
  if (!q45) {
    const uint32_t last = a.n_tokens - (tok_tiles - 1u) * 128u;   // tokens of the last token tile
    return (n_wg >= 160u && (tok_tiles >= 2u || a.n_tokens > 96u)) || (n_wg >= 128u && last > 96u) ||
           (n_wg >= 128u && tok_tiles >= 3u);
  }
  return (tok_tiles >= 3u || (tok_tiles == 2u && nsb > 32u)) && n_wg >= 160u && (nsb <= 20u || n_wg <= 256u);
}

// Whether a tiled launch goes to a kernel whose waves all multiply, given planes.  The one with 128 x 128
// workgroups wants more of them than there are compute units (two share one, and one alone is slower than the
// feeding-wave kernels: Q4_K 4096 -> 14336 at 256 tokens 69 us against 57, at 384 tokens 87 against 104), the
// activations in operand chunks, and everything within 32-bit byte offsets.  (plane_kernel 2: whatever the
// grid.)
static bool gemm_dma_eligible(const OgmGemmArgs &a) {
  const uint32_t nsb = a.in_dim / 256;
  const bool q45 = a.ggml_type == OGM_Q4_K || a.ggml_type == OGM_Q5_K;
  const uint32_t t_pad = (a.n_tokens + 31u) & ~31u;
  if ((q45 && nsb * 512u > GD_TAB) || a.n_tokens < (a.ggml_type == OGM_IQ4_XS ? 17u : 32u) || !a.xh ||
      (uint64_t)t_pad * a.in_dim >= (1ull << 32))
    return false;
  uint32_t tiles = 0;
  for (uint32_t m = 0; m <= a.n_extra; m++) {
    const uint32_t od = m ? a.extra_out_dim[m - 1] : a.out_dim;
    if ((uint64_t)((od + 63u) / 64u) * 64u * a.in_dim * 2u >= (1ull << 32)) return false;
    tiles += (od + GD_ROWS - 1u) / GD_ROWS;
  }
  // (IQ4_XS has no other GEMM kernel)
  if (a.plane_kernel == 2u || a.ggml_type == OGM_IQ4_XS || ((a.n_tokens + GD_TOK - 1u) / GD_TOK) * tiles > 256u) return true;
  return gemm_interleaved(a);
}

// Whether a K-quant launch takes the small-batch kernel (workgroups of 32 rows x 32 tokens whose waves take
// different super-blocks) rather than a tiled one.
// planes_possible: whether the launch has (or, asked before they are built, may get) every matrix's planes.
static bool gemm_small_batch(const OgmGemmArgs &a, bool planes_possible) {
  const uint32_t nsb = a.in_dim / 256;
  const bool q45 = a.ggml_type == OGM_Q4_K || a.ggml_type == OGM_Q5_K;
  // Q6_K and IQ4_XS launches the interleaved plane kernel wants by their size go there (see gemm_interleaved)
  if ((a.ggml_type == OGM_Q6_K || a.ggml_type == OGM_IQ4_XS) && a.small_max_tokens == 0u && a.interleave == 0u &&
      planes_possible && gemm_dma_eligible(a) && gemm_interleaved(a, true))
    return false;
  uint32_t tiles64_all = (a.out_dim + 63u) / 64u;
  for (uint32_t m = 0; m < a.n_extra; m++) tiles64_all += (a.extra_out_dim[m] + 63u) / 64u;
  // Measured on MI355X with the activations in operand chunks, whole calls, us, small-batch against the best other
  // kernel.  Q4_K: 4096 -> 4096 (64 tiles of 64 rows) at 128 / 192 / 256 / 384 tokens 20 / 30 / 32 / 41 against 33 / 33 /
  // 34 / 40; 4096 -> 6144 (96 tiles) at 128 / 192 / 256: 29 / 38 / 43 against 33 / 37 / 38; 8192 -> 8192 (128 tiles) at
  // 128 / 192: 54 / 76 against 57 / 70; 4096 -> 14336 (224 tiles) at 64 / 96 / 128: 31 / 42 / 48 against 37 / 38 / 39;
  // 2048 -> 2048 (32 tiles) at 256 / 512: 14 / 23 against 20 / 22.  Rows of more than 8192 inputs, where the plane
  // kernels' first pass weighs most and no medium-batch kernel runs: 14336 -> 4096 (64 tiles) at 192 / 256 / 384: 81 /
  // 90 / 117 against 95 / 95 / 121; 14336 -> 5120 (80 tiles) at 192 / 256 / 384: 87 / 118 / 149 against 116 / 122 / 123;
  // 14336 -> 8192 (128 tiles) at 128 / 192 / 256: 89 / 127 / 168 against 94 / 126 / 131.  Q6_K: 8192 -> 2048 (32 tiles)
  // at 256 / 384 / 512: 32 / 48 / 50 against 47 / 50 / 51; 4096 -> 2048 at 384 / 512: 25 / 31 against 29 / 29; the
  // launches of more tiles leave earlier for the 64-row plane kernel (gemm_interleaved).
  const bool long_rows = q45 && nsb > 32u;   // no medium-batch kernel there, and a first pass in the plane kernels
  const uint32_t small_max = a.small_max_tokens ? a.small_max_tokens
                             : (tiles64_all <= 32u   ? (q45 ? 512u : 384u)
                                : tiles64_all <= 64u ? 256u
                                : tiles64_all <= 96u ? (long_rows ? 256u : 128u)
                                : tiles64_all <= 128u ? 128u
                                                      : 64u);
  return a.small_max_tokens != 1u && a.n_tokens <= small_max &&
         8u * 4096u + 128u * nsb <= GM_LDS_MAX;
}

// Whether a Q4_K / Q5_K launch beyond the small batches takes the medium-batch kernel (32 rows x 128 tokens per
// workgroup, its waves on different super-blocks) instead of a tiled one.  medium: 0 by the size of the launch,
// 1 never, 2 whenever the shape allows.
static bool gemm_medium_batch(const OgmGemmArgs &a) {
  const uint32_t nsb = a.in_dim / 256;
  const bool q45 = a.ggml_type == OGM_Q4_K || a.ggml_type == OGM_Q5_K;
  const uint32_t t_pad = (a.n_tokens + 31u) & ~31u;
  if (!q45 || a.medium == 1u || !a.xh || SBW_TERMS_BYTES + SBW_TOK * 4u * nsb > GM_LDS_MAX ||
      (uint64_t)t_pad * a.in_dim >= (1ull << 32))
    return false;
  if (a.medium == 2u) return true;
  // Measured on MI355X against the kernels it displaces, whole calls, us: 4096 -> 14336 at 128 tokens 39 against 50
  // (feeding waves) and 48 (small batch), at 192 / 256 tokens 78 / 77 against 65 / 65; 4096 -> 6144 at 192 / 256 tokens
  // 38 / 39 against 43 / 46 (feeding waves) and 38 / 43 (small batch); 8192 -> 8192 at 192 / 256: 70 / 71 against 76 / 97
  // (small batch).  (The small-batch kernel comes first and keeps what gemm_small_batch gives it.)  It wants a lone token tile of 128 nearly full (below, the small batches), and at two
  // of them, full or not, matrices of at most 8192 rows (4096 -> 6144 at 144 / 192 tokens 38 / 37 against 43 / 43 for
  // the feeding waves, 8192 -> 8192 68 / 69 against 80 / 82; beyond 8192 rows the 128-row tiles of the feeding-wave
  // kernels outnumber the compute units' halves).  Its
  // workgroups of 32 rows must fit the device in one round, two to a compute unit: gate and up together (28672 rows,
  // 896 workgroups) take 63 us against 56 for the feeding-wave kernel (128-token prefill of the 8B shapes 7.0
  // against 6.65 ms), so at one token tile the launch may have at most 16384 rows.
  uint32_t tiles64_all = (a.out_dim + 63u) / 64u;
  for (uint32_t m = 0; m < a.n_extra; m++) tiles64_all += (a.extra_out_dim[m] + 63u) / 64u;
  const uint32_t tok_tiles = (a.n_tokens + SBW_TOK - 1u) / SBW_TOK;
  const bool full_enough = tok_tiles * SBW_TOK - a.n_tokens <= 32u;
  // (rows of more than 8192 inputs: 16384 -> 16384 at 128 tokens 205 us against 154 for the feeding waves)
  return nsb <= 32u && ((tok_tiles == 1u && full_enough && tiles64_all <= 256u) || (tok_tiles == 2u && tiles64_all <= 128u));
}

bool ogm_gemm_takes_small_batch(const OgmGemmArgs &a) {
  if (a.n_tokens == 0 || a.out_dim == 0 || is_flat32(a.ggml_type)) return false;
  if (!ogm_gemm_supported(a.ggml_type, a.in_dim, a.out_dim, a.n_tokens)) return false;
  return a.ggml_type == OGM_Q2_K || gemm_small_batch(a, true);
}

bool ogm_gemm_uses_planes(const OgmGemmArgs &a) {
  if (a.n_tokens == 0 || a.out_dim == 0 || is_flat32(a.ggml_type) || a.ggml_type == OGM_Q2_K) return false;
  if (!ogm_gemm_supported(a.ggml_type, a.in_dim, a.out_dim, a.n_tokens)) return false;
  // (the feeding-wave kernels unpack on every call: reading planes made them no faster -- Q4_K 4096 -> 14336 at 256
  // tokens 66 against 66 us, Q6_K 14336 -> 4096 at 512 tokens 96 against 98)
  return !gemm_small_batch(a, true) && gemm_dma_eligible(a);
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
    // small batches: the kernel whose waves take different blocks (small_max_tokens as for the K-quants: 0 by the
    // size of the launch, 1 never, otherwise up to that many tokens)
    const uint32_t sbf_lds = gemm_flat_small_lds(8u);
    const bool q51 = a.ggml_type == OGM_Q5_1;   // (this kernel only, whatever the batch)
    const bool sbf = q51 || (a.small_max_tokens ? a.n_tokens <= a.small_max_tokens : gemm_flat_small(a.n_tokens, a.out_dim));
    if ((q51 || a.small_max_tokens != 1u) && sbf && sbf_lds <= GM_LDS_MAX) {
      GemmSbParams q{};
      q.wt = a.wt;
      q.xq = a.act.q;
      q.ad = a.act.d;
      q.y = a.y;
      q.in_dim = a.in_dim;
      q.out_dim = a.out_dim;
      q.n_tokens = a.n_tokens;
      q.nsb = p.nblk;
      q.c_shift = p.c_shift;
      q.r_shift = p.r_shift;
      q.nct = p.nct;
      // sixteen waves when the launch leaves compute units idle and the rows have the blocks for two rounds of them
      const uint32_t n_wg = ((a.n_tokens + 31u) / 32u) * ((a.out_dim + 31u) / 32u);
      const uint32_t lds16 = gemm_flat_small_lds(16u);
      const bool w16 = (a.sb_waves ? a.sb_waves == 16u : (n_wg <= 256u && p.nblk >= 64u)) && lds16 <= GM_LDS_MAX;
      const uint32_t lds_here = w16 ? lds16 : sbf_lds;
      const void *fn = a.ggml_type == OGM_Q4_0   ? (w16 ? (const void *)ogm_gemm_sb_flat_w16_kernel<0> : (const void *)ogm_gemm_sb_flat_kernel<0>)
                       : a.ggml_type == OGM_Q5_0 ? (w16 ? (const void *)ogm_gemm_sb_flat_w16_kernel<1> : (const void *)ogm_gemm_sb_flat_kernel<1>)
                       : a.ggml_type == OGM_IQ4_NL ? (w16 ? (const void *)ogm_gemm_sb_flat_w16_kernel<2> : (const void *)ogm_gemm_sb_flat_kernel<2>)
                       : q51                       ? (w16 ? (const void *)ogm_gemm_sb_flat_w16_kernel<4> : (const void *)ogm_gemm_sb_flat_kernel<4>)
                                                   : (w16 ? (const void *)ogm_gemm_sb_flat_w16_kernel<3> : (const void *)ogm_gemm_sb_flat_kernel<3>);
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_here);
      if (e != hipSuccess) return e;
      void *kargs[] = {(void *)&q};
      e = hipLaunchKernel(fn, dim3((a.n_tokens + 31u) / 32u, (a.out_dim + 31u) / 32u), dim3(w16 ? 1024 : 512), kargs, lds_here, stream);
      if (e != hipSuccess) return e;
      if (kernel_name) *kernel_name = w16 ? "ogm_gemm_sb_flat_w16_kernel" : "ogm_gemm_sb_flat_kernel";
      return hipGetLastError();
    }
    if (q51) return hipErrorInvalidValue;
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
  const bool q45 = a.ggml_type == OGM_Q4_K || a.ggml_type == OGM_Q5_K;
  if (a.ggml_type == OGM_Q2_K) {   // its one GEMM kernel, whatever the batch
    GemmSbParams q{};
    q.wt = a.wt;
    q.xq = a.act.q;
    q.ad = a.act.d;   // per 32
    q.y = a.y;
    q.in_dim = a.in_dim;
    q.out_dim = a.out_dim;
    q.n_tokens = a.n_tokens;
    q.nsb = nsb;
    const OgmTiling tl2 = ogm_tiling_for(nsb, a.out_dim);
    const uint32_t cs2 = tl2.C == 4 ? 2 : (tl2.C == 2 ? 1 : 0);
    q.c_shift = cs2;
    q.r_shift = 6 - cs2;
    q.nct = tl2.nct;
    q.n_extra = a.n_extra;
    uint32_t tiles = (a.out_dim + 31u) / 32u;
    for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
      q.extra_wt[m] = m < a.n_extra ? a.extra_wt[m] : nullptr;
      q.extra_y[m] = m < a.n_extra ? a.extra_y[m] : nullptr;
      q.extra_out_dim[m] = m < a.n_extra ? a.extra_out_dim[m] : 0u;
      if (m < a.n_extra) tiles += (a.extra_out_dim[m] + 31u) / 32u;
    }
    const uint32_t lds_bytes = 16u * 4096u + 128u * (a.in_dim / 32u);
    const void *fn = (const void *)ogm_gemm_sb_q2k_kernel;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
    void *kargs[] = {(void *)&q};
    e = hipLaunchKernel(fn, dim3((a.n_tokens + 31u) / 32u, tiles), dim3(512), kargs, lds_bytes, stream);
    if (e != hipSuccess) return e;
    if (kernel_name) *kernel_name = "ogm_gemm_sb_q2k_kernel";
    return hipGetLastError();
  }
  // Q4_K / Q5_K: the first pass's operand, the quantizer's sums per 32 as f16 pairs, comes from the quantizer
  const _Float16 *bs16 = (const _Float16 *)a.act.bs16;
  if (q45 && !bs16) return hipErrorInvalidValue;
  uint32_t row_tiles = (a.out_dim + GM_BN - 1) / GM_BN;
  for (uint32_t m = 0; m < a.n_extra; m++) row_tiles += (a.extra_out_dim[m] + GM_BN - 1) / GM_BN;
  const OgmTiling tl = ogm_tiling_for(nsb, a.out_dim);
  const uint32_t c_shift = tl.C == 4 ? 2 : (tl.C == 2 ? 1 : 0);
  // Small batches: the kernel whose waves take different super-blocks, up to 64 tokens and longer over matrices of
  // few rows (gemm_small_batch).
  bool have_planes = a.planes != nullptr;
  for (uint32_t m = 0; m < a.n_extra; m++) have_planes = have_planes && a.extra_planes[m] != nullptr;   // every matrix of the launch, or none
  if (gemm_small_batch(a, have_planes)) {
    GemmSbParams p;
    p.wt = a.wt;
    p.x_chunks = (a.xt_ready && a.xh) ? 1u : 0u;   // the operand chunks where a producer wrote them
    p.xq = p.x_chunks ? (const int8_t *)a.xh : a.act.q;
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
    const uint32_t lds_bytes = (w16 ? 16u : 8u) * 4096u + 128u * nsb;
    const void *fn = a.ggml_type == OGM_Q6_K   ? (w16 ? (const void *)ogm_gemm_sb_q6k_w16_kernel : (const void *)ogm_gemm_sb_q6k_kernel)
                     : a.ggml_type == OGM_Q3_K ? (w16 ? (const void *)ogm_gemm_sb_q3k_w16_kernel : (const void *)ogm_gemm_sb_q3k_kernel)
                     : a.ggml_type == OGM_IQ4_XS ? (w16 ? (const void *)ogm_gemm_sb_iq4xs_w16_kernel : (const void *)ogm_gemm_sb_iq4xs_kernel)
                     : a.ggml_type == OGM_Q4_K ? (w16 ? (const void *)ogm_gemm_sb_q45k_w16_kernel<false> : (const void *)ogm_gemm_sb_q45k_kernel<false>)
                                               : (w16 ? (const void *)ogm_gemm_sb_q45k_w16_kernel<true> : (const void *)ogm_gemm_sb_q45k_kernel<true>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
    void *kargs[] = {(void *)&p};
    e = hipLaunchKernel(fn, dim3((a.n_tokens + 31u) / 32u, tiles), dim3(w16 ? 1024 : 512), kargs, lds_bytes, stream);
    if (e != hipSuccess) return e;
    if (kernel_name)
      *kernel_name = a.ggml_type == OGM_Q6_K   ? (w16 ? "ogm_gemm_sb_q6k_w16_kernel" : "ogm_gemm_sb_q6k_kernel")
                     : a.ggml_type == OGM_Q3_K ? (w16 ? "ogm_gemm_sb_q3k_w16_kernel" : "ogm_gemm_sb_q3k_kernel")
                     : a.ggml_type == OGM_IQ4_XS ? (w16 ? "ogm_gemm_sb_iq4xs_w16_kernel" : "ogm_gemm_sb_iq4xs_kernel")
                     : a.ggml_type == OGM_Q4_K ? (w16 ? "ogm_gemm_sb_q4k_w16_kernel" : "ogm_gemm_sb_q4k_kernel")
                                               : (w16 ? "ogm_gemm_sb_q5k_w16_kernel" : "ogm_gemm_sb_q5k_kernel");
    return hipGetLastError();
  }
  const bool dma = have_planes && gemm_dma_eligible(a);
  if ((!dma || a.medium == 2u) && gemm_medium_batch(a)) {   // (asked for by name, it comes before the planes)
    const uint32_t t_pad = (a.n_tokens + 31u) & ~31u;
    if (!a.xt_ready)
      hipLaunchKernelGGL(ogm_gemm_xtile_kernel, dim3(a.in_dim / 128u, t_pad / 32u), dim3(256), 0, stream, a.act.q,
                         (int8_t *)a.xh, a.in_dim, a.n_tokens);
    GemmSbwParams p;
    p.wt = a.wt;
    p.xt = (const int8_t *)a.xh;
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
    const uint32_t lds_bytes = SBW_TERMS_BYTES + SBW_TOK * 4u * nsb;
    const void *fn = a.ggml_type == OGM_Q4_K ? (const void *)ogm_gemm_sbw_q45k_kernel<false>
                                             : (const void *)ogm_gemm_sbw_q45k_kernel<true>;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
    void *kargs[] = {(void *)&p};
    e = hipLaunchKernel(fn, dim3((a.n_tokens + SBW_TOK - 1u) / SBW_TOK, tiles), dim3(64u * SBW_NW), kargs, lds_bytes, stream);
    if (e != hipSuccess) return e;
    if (kernel_name) *kernel_name = a.ggml_type == OGM_Q4_K ? "ogm_gemm_sbw_q4k_kernel" : "ogm_gemm_sbw_q5k_kernel";
    return hipGetLastError();
  }
  if (dma) {
    const uint32_t t_pad = (a.n_tokens + 31u) & ~31u;
    if (!a.xt_ready)
      hipLaunchKernelGGL(ogm_gemm_xtile_kernel, dim3(a.in_dim / 128u, t_pad / 32u), dim3(256), 0, stream, a.act.q,
                         (int8_t *)a.xh, a.in_dim, a.n_tokens);
    // the kernel that adds a super-block up between the next one's matrix instructions (64-row tiles)
    const bool interleaved = gemm_interleaved(a);
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
    uint32_t tiles = (a.out_dim + GD_ROWS - 1u) / GD_ROWS;
    for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
      d.extra_wt[m] = m < a.n_extra ? a.extra_wt[m] : nullptr;
      d.extra_planes[m] = m < a.n_extra ? a.extra_planes[m] : nullptr;
      d.extra_y[m] = m < a.n_extra ? a.extra_y[m] : nullptr;
      d.extra_out_dim[m] = m < a.n_extra ? a.extra_out_dim[m] : 0u;
      if (m < a.n_extra) tiles += (a.extra_out_dim[m] + GD_ROWS - 1u) / GD_ROWS;
    }
    if (interleaved) {
      uint32_t tiles_x = (a.out_dim + GX_ROWS - 1u) / GX_ROWS;
      for (uint32_t m = 0; m < a.n_extra; m++) tiles_x += (a.extra_out_dim[m] + GX_ROWS - 1u) / GX_ROWS;
      const void *fx = a.ggml_type == OGM_Q6_K     ? (const void *)ogm_gemm_dmx_kernel<GP_Q6K>
                       : a.ggml_type == OGM_IQ4_XS ? (const void *)ogm_gemm_dmx_kernel<GP_IQ4XS>
                       : a.ggml_type == OGM_Q4_K   ? (const void *)ogm_gemm_dmx_kernel<GP_Q4K>
                                                   : (const void *)ogm_gemm_dmx_kernel<GP_Q5K>;
      hipError_t ex = hipFuncSetAttribute(fx, hipFuncAttributeMaxDynamicSharedMemorySize, (int)GX_LDS_BYTES);
      if (ex != hipSuccess) return ex;
      void *xargs[] = {(void *)&d};
      ex = hipLaunchKernel(fx, dim3((a.n_tokens + GX_TOK - 1u) / GX_TOK, tiles_x), dim3(64u * GX_NW), xargs, GX_LDS_BYTES, stream);
      if (ex != hipSuccess) return ex;
      if (kernel_name)
        *kernel_name = a.ggml_type == OGM_Q6_K     ? "ogm_gemm_q6k_dmx_kernel"
                       : a.ggml_type == OGM_IQ4_XS ? "ogm_gemm_iq4xs_dmx_kernel"
                       : a.ggml_type == OGM_Q4_K   ? "ogm_gemm_q4k_dmx_kernel"
                                                   : "ogm_gemm_q5k_dmx_kernel";
      return hipGetLastError();
    }
    const bool one_pass = q45 && a.one_pass != 0u;
    const void *fn = a.ggml_type == OGM_Q6_K   ? (const void *)ogm_gemm_dma_kernel<GP_Q6K>
                     : a.ggml_type == OGM_IQ4_XS ? (const void *)ogm_gemm_dma_kernel<GP_IQ4XS>
                     : a.ggml_type == OGM_Q3_K ? (const void *)ogm_gemm_dma_kernel<GP_Q3K>
                     : a.ggml_type == OGM_Q4_K ? (one_pass ? (const void *)ogm_gemm_dma_kernel<GP_Q4K, true>
                                                           : (const void *)ogm_gemm_dma_kernel<GP_Q4K>)
                                               : (one_pass ? (const void *)ogm_gemm_dma_kernel<GP_Q5K, true>
                                                           : (const void *)ogm_gemm_dma_kernel<GP_Q5K>);
    const uint32_t dma_lds = one_pass ? GD_LDS_BYTES_ONEPASS : GD_LDS_BYTES;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)dma_lds);
    if (e != hipSuccess) return e;
    void *kargs[] = {(void *)&d};
    e = hipLaunchKernel(fn, dim3((a.n_tokens + GD_TOK - 1u) / GD_TOK, tiles), dim3(64u * GD_NW), kargs, dma_lds, stream);
    if (e != hipSuccess) return e;
    if (kernel_name)
      *kernel_name = a.ggml_type == OGM_Q6_K   ? "ogm_gemm_q6k_dma_kernel"
                     : a.ggml_type == OGM_IQ4_XS ? "ogm_gemm_iq4xs_dma_kernel"
                     : a.ggml_type == OGM_Q3_K ? "ogm_gemm_q3k_dma_kernel"
                     : a.ggml_type == OGM_Q4_K ? (one_pass ? "ogm_gemm_q4k_dma_onepass_kernel" : "ogm_gemm_q4k_dma_kernel")
                                               : (one_pass ? "ogm_gemm_q5k_dma_onepass_kernel" : "ogm_gemm_q5k_dma_kernel");
    return hipGetLastError();
  }
  // The feeding-wave kernels: eight (or four) waves unpack the tile-planar bytes into the two planes per call
  // while as many multiply.
  if (a.ggml_type == OGM_IQ4_XS) return hipErrorInvalidValue;   // (its GEMMs need its planes: ogm_gemm_uses_planes)
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
  for (uint32_t m = 0; m < OGM_GEMM_MAX_MATS - 1; m++) {
    p.extra_wt[m] = m < a.n_extra ? a.extra_wt[m] : nullptr;
    p.extra_y[m] = m < a.n_extra ? a.extra_y[m] : nullptr;
    p.extra_out_dim[m] = m < a.n_extra ? a.extra_out_dim[m] : 0u;
  }
  // 64-row tiles when asked for (tile_rows 64), or when they still come one to a CU: then twice
  // as many CUs work (14336 -> 4096 x 512 tokens: 150 us against 180 us).  Two of them sharing a CU
  // are slower than one 128-row tile (4096 -> 14336 x 512: 165 us against 118 us).
  uint32_t tiles64 = (a.out_dim + 63u) / 64u;
  for (uint32_t m = 0; m < a.n_extra; m++) tiles64 += (a.extra_out_dim[m] + 63u) / 64u;
  const bool r64 = a.tile_rows == 64u || ((a.n_tokens + 127u) / 128u) * tiles64 <= 256u;
  const uint32_t rows = r64 ? 64u : 128u;
  const dim3 pgrid((a.n_tokens + 127u) / 128u, r64 ? tiles64 : row_tiles);
  const bool q3 = a.ggml_type == OGM_Q3_K;
  // Q4_K / Q5_K: + the tokens' ad of every super-block for the first pass
  const uint32_t lds_bytes = (q3 ? 3u : 6u) * rows * GI_ROW + 3u * GI_WTILE + (2u * rows + 256u) * 4u +
                             (q45 ? nsb * 512u : 0u);
  struct Pick { uint32_t type; bool r64; const void *fn; const char *name; };
  const Pick picks[] = {
      {OGM_Q6_K, false, (const void *)ogm_gemm_q6k_i8_kernel, "ogm_gemm_q6k_i8_kernel"},
      {OGM_Q6_K, true, (const void *)ogm_gemm_q6k_i8_r64_kernel, "ogm_gemm_q6k_i8_r64_kernel"},
      {OGM_Q3_K, false, (const void *)ogm_gemm_q3k_i8_kernel, "ogm_gemm_q3k_i8_kernel"},
      {OGM_Q3_K, true, (const void *)ogm_gemm_q3k_i8_r64_kernel, "ogm_gemm_q3k_i8_r64_kernel"},
      {OGM_Q4_K, false, (const void *)ogm_gemm_q4k_i8p_kernel, "ogm_gemm_q4k_i8p_kernel"},
      {OGM_Q4_K, true, (const void *)ogm_gemm_q4k_i8p_r64_kernel, "ogm_gemm_q4k_i8p_r64_kernel"},
      {OGM_Q5_K, false, (const void *)ogm_gemm_q5k_i8p_kernel, "ogm_gemm_q5k_i8p_kernel"},
      {OGM_Q5_K, true, (const void *)ogm_gemm_q5k_i8p_r64_kernel, "ogm_gemm_q5k_i8p_r64_kernel"},
  };
  const Pick *pick = nullptr;
  for (const Pick &c : picks)
    if (c.type == a.ggml_type && c.r64 == r64) pick = &c;
  if (!pick) return hipErrorInvalidValue;
  hipError_t e = hipFuncSetAttribute(pick->fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return e;
  void *kargs[] = {(void *)&p};
  e = hipLaunchKernel(pick->fn, pgrid, dim3(r64 ? 512 : 1024), kargs, lds_bytes, stream);
  if (e != hipSuccess) return e;
  if (kernel_name) *kernel_name = pick->name;
  return hipGetLastError();
}
