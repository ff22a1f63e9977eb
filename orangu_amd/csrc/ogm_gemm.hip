// gfx950 prefill GEMM for Q4_K weights on MFMA, bit-compatible with the CPU path's K-quant GEMM
// (gemm_k_q4_k + accumulate_sym32, engine/vecdot.rs:2213-2303 of orangu-server).
//
// The integer stage stays exact on the matrix cores by keeping every operand an *integer-valued
// f16*: a weight enters as sc_j * q (0..945, exact in f16: 11-bit significand), an activation as
// its int8 value.  Products are exact in f32 and a chain of 128 of them stays below 2^24, so a
// half super-block accumulates exactly in the MFMA's f32 accumulator; the two halves are added
// with one f32 add, which rounds the exact integer sum once -- the same value as the
// reference's `isum as f32`.  The min term sum_j m_j * bsum_j goes through one more MFMA per
// super-block with bsum split as 64*bh + bl (both exact in f16).  The f32 epilogue then follows
// the reference's order: first `acc -= (ad*dmin) * imin` over all super-blocks, then
// `acc += ad * (d * isum)` over all super-blocks.
//
// Tiling: a workgroup of four waves owns 64 rows (four row blocks of the tile-planar layout)
// x 128 tokens; a wave owns 32 rows x 64 tokens = two 32x32 MFMA tiles.  Per half super-block
// (128 k) the workgroup dequantizes its 64 x 128 weight tile to f16 in LDS (each thread one
// 16-byte piece: v_perm nibble split, magic-number int->f16, one packed f16 fma per two
// weights) and copies the 128 x 128 f16 activation tile, then runs 8 x v_mfma_f32_32x32x16_f16
// per MFMA tile.
#include <hip/hip_runtime.h>

#include "ogm_kernels.h"
#include "ogm_layout.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));

#define GM_BN 64    // rows per workgroup
#define GM_BT 128   // tokens per workgroup
#define GM_KH 128   // k per staging step: half a super-block
#define GM_LD (GM_KH + 8)   // f16 per LDS row: 16 bytes of padding keep 16-byte row reads conflict-free
#define GM_LD2 24           // f16 per LDS row of the min-term operands (16 + padding)

struct GemmParams {
  const uint8_t *wt;      // tile-planar Q4_K, C = 4 (16 rows x 4 blocks per tile)
  const _Float16 *xh;     // [T][in_dim] int8 activations as f16
  const float *ad;        // [T][nsb] activation scales (per 256)
  const int16_t *bsum;    // [T][in_dim/32] per-32 sums of q
  float *y;               // [T][out_dim]
  uint32_t in_dim, out_dim, n_tokens, nsb, nct, nrb;
};

__device__ __forceinline__ float gm_f16_bits_to_f32(uint32_t bits16) {
  union { unsigned short u; _Float16 h; } v;
  v.u = (unsigned short)bits16;
  return (float)v.h;
}

// int8 activations -> f16, once per matmul.
__global__ void ogm_q8_to_f16_kernel(const int8_t *__restrict__ q, _Float16 *__restrict__ xh, size_t n8) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n8) return;
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

// Four bytes b0..b3 of `w`, one nibble each (shift 0: low, 4: high), scaled by sc:
// out = { sc*n(b0), sc*n(b1) }, { sc*n(b2), sc*n(b3) } as packed f16.
__device__ __forceinline__ void dequant4(uint32_t w, int shift, half2v sc2, half2v nc2, uint32_t &o01,
                                         uint32_t &o23) {
  const uint32_t p01 = __builtin_amdgcn_perm(0u, w, 0x0c010c00u) >> shift;  // (b0, 0, b1, 0)
  const uint32_t p23 = __builtin_amdgcn_perm(0u, w, 0x0c030c02u) >> shift;  // (b2, 0, b3, 0)
  // 0x6400 | n is the f16 1024 + n; (1024 + n) * sc - 1024 * sc = n * sc exactly (one rounding
  // of an exactly representable result)
  union { uint32_t u; half2v h; } a, b;
  a.u = (p01 & 0x000F000Fu) | 0x64006400u;
  b.u = (p23 & 0x000F000Fu) | 0x64006400u;
  a.h = __builtin_elementwise_fma(a.h, sc2, nc2);
  b.h = __builtin_elementwise_fma(b.h, sc2, nc2);
  o01 = a.u;
  o23 = b.u;
}

__global__ __launch_bounds__(256) void ogm_gemm_q4k_kernel(GemmParams p) {
  extern __shared__ __align__(16) uint8_t lds[];
  _Float16 *A_l = (_Float16 *)lds;                    // [64][GM_LD]   (pass 1: [64][GM_LD2])
  _Float16 *B_l = A_l + GM_BN * GM_LD;                // [128][GM_LD]  (pass 1: [128][GM_LD2])
  float *d_l = (float *)(B_l + GM_BT * GM_LD);        // [64]
  float *dmin_l = d_l + GM_BN;                        // [64]
  float *ad_l = dmin_l + GM_BN;                       // [128]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t wr = wave & 1u, wt_ = wave >> 1;     // wave's row half and token half
  const uint32_t r0 = blockIdx.x * GM_BN, t0 = blockIdx.y * GM_BT;
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  const uint32_t rb0 = r0 / 16u;

  float16v y0 = {}, y1 = {};  // this wave's 32 rows x (2 x 32) tokens

  // ---------------- pass 1: acc -= (ad * dmin) * sum_j m_j * bsum_j, all super-blocks first
  for (uint32_t s = 0; s < p.nsb; s++) {
    if (tid < GM_BN) {
      const uint32_t lr = tid;
      // (row blocks past the matrix are clamped: their rows are never stored)
      const size_t tile = (size_t)min(rb0 + lr / 16u, p.nrb - 1u) * p.nct + s / 4u;
      const uint4 h = *(const uint4 *)(p.wt + tile * 9216u + ((s & 3u) * 16u + (lr & 15u)) * 16u);
      const uint32_t mna = h.z & 0x3F3F3F3Fu;                                      // m 0..3
      const uint32_t mnb = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);  // m 4..7
      half8 hi, lo;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float ma = (float)((mna >> (8 * j)) & 0xFFu), mb = (float)((mnb >> (8 * j)) & 0xFFu);
        lo[j] = (_Float16)ma;
        lo[4 + j] = (_Float16)mb;
        hi[j] = (_Float16)(64.0f * ma);
        hi[4 + j] = (_Float16)(64.0f * mb);
      }
      *(half8 *)(A_l + lr * GM_LD2) = hi;       // k 0..7 : 64 * m_j  (pairs with bh_j)
      *(half8 *)(A_l + lr * GM_LD2 + 8) = lo;   // k 8..15: m_j       (pairs with bl_j)
      dmin_l[lr] = gm_f16_bits_to_f32(h.x >> 16);
    } else if (tid < GM_BN + GM_BT) {
      const uint32_t tt = tid - GM_BN, tk = t0 + tt;
      half8 bh = {}, bl = {};
      float adv = 0.0f;
      if (tk < p.n_tokens) {
        const uint4 b = *(const uint4 *)(p.bsum + ((size_t)tk * p.nsb + s) * 8u);
        const uint32_t w[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const int b0 = (int)(int16_t)(w[j] & 0xFFFFu), b1 = ((int)w[j]) >> 16;
          bh[2 * j] = (_Float16)(float)(b0 >> 6);      // floor(b / 64)
          bl[2 * j] = (_Float16)(float)(b0 & 63);
          bh[2 * j + 1] = (_Float16)(float)(b1 >> 6);
          bl[2 * j + 1] = (_Float16)(float)(b1 & 63);
        }
        adv = p.ad[(size_t)tk * p.nsb + s];
      }
      *(half8 *)(B_l + tt * GM_LD2) = bh;
      *(half8 *)(B_l + tt * GM_LD2 + 8) = bl;
      ad_l[tt] = adv;
    }
    __syncthreads();
    {
      const half8 a = *(const half8 *)(A_l + (32u * wr + l32) * GM_LD2 + 8u * lh);
      const half8 b0 = *(const half8 *)(B_l + (64u * wt_ + l32) * GM_LD2 + 8u * lh);
      const half8 b1 = *(const half8 *)(B_l + (64u * wt_ + 32u + l32) * GM_LD2 + 8u * lh);
      float16v z = {};
      const float16v i0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b0, z, 0, 0, 0);
      const float16v i1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b1, z, 0, 0, 0);
      const float ad0 = ad_l[64u * wt_ + l32], ad1 = ad_l[64u * wt_ + 32u + l32];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const uint32_t row_l = 32u * wr + 8u * (r / 4) + 4u * lh + (r % 4);
        const float dm = dmin_l[row_l];
        y0[r] -= ad0 * dm * i0[r];
        y1[r] -= ad1 * dm * i1[r];
      }
    }
    __syncthreads();
  }

  // ---------------- pass 2: acc += ad * (d * sum_j sc_j * dot32_j)
  for (uint32_t s = 0; s < p.nsb; s++) {
    float16v c0 = {}, c1 = {};   // first half of the super-block
    float16v e0 = {}, e1 = {};   // second half
#pragma unroll
    for (int h = 0; h < 2; h++) {
      // ---- stage the weight tile: thread -> (row block rbl, piece pi of this half, row r)
      {
        const uint32_t rbl = tid >> 6, j = tid & 63u, pi = j >> 4, r = j & 15u;
        const uint32_t lr = rbl * 16u + r;
        const size_t tile = (size_t)min(rb0 + rbl, p.nrb - 1u) * p.nct + s / 4u;
        const uint8_t *ub = p.wt + tile * 9216u + ((s & 3u) * 16u + r) * 16u;
        const uint4 hd = *(const uint4 *)ub;
        const uint4 qv = *(const uint4 *)(ub + (1u + 4u * h + pi) * 1024u);
        // get_scale_min_k4 (quant.rs:653-662): scales of sub-blocks 2g (low nibbles), 2g+1 (high)
        const uint32_t sca = hd.y & 0x3F3F3F3Fu;
        const uint32_t scb = (hd.w & 0x0F0F0F0Fu) | ((hd.y >> 2) & 0x30303030u);
        const uint32_t g = 2u * h + (pi >> 1);
        const uint32_t scw = g < 2 ? sca : scb;
        const uint32_t sh = (g & 1u) * 16u;
        const float slo = (float)((scw >> sh) & 0xFFu), shi = (float)((scw >> (sh + 8u)) & 0xFFu);
        half2v sl2, nl2, sh2, nh2;
        sl2[0] = sl2[1] = (_Float16)slo;
        nl2[0] = nl2[1] = (_Float16)(-1024.0f * slo);
        sh2[0] = sh2[1] = (_Float16)shi;
        nh2[0] = nh2[1] = (_Float16)(-1024.0f * shi);
        uint4 lo_a, lo_b, hi_a, hi_b;  // 16 low-nibble weights, 16 high-nibble weights, as f16
        dequant4(qv.x, 0, sl2, nl2, lo_a.x, lo_a.y);
        dequant4(qv.y, 0, sl2, nl2, lo_a.z, lo_a.w);
        dequant4(qv.z, 0, sl2, nl2, lo_b.x, lo_b.y);
        dequant4(qv.w, 0, sl2, nl2, lo_b.z, lo_b.w);
        dequant4(qv.x, 4, sh2, nh2, hi_a.x, hi_a.y);
        dequant4(qv.y, 4, sh2, nh2, hi_a.z, hi_a.w);
        dequant4(qv.z, 4, sh2, nh2, hi_b.x, hi_b.y);
        dequant4(qv.w, 4, sh2, nh2, hi_b.z, hi_b.w);
        // piece 1+2g+hh holds qs[32g+16hh ..]: low nibbles are elements 64g+16hh.., high +32
        _Float16 *dst = A_l + lr * GM_LD + 64u * (pi >> 1) + 16u * (pi & 1u);
        *(uint4 *)(dst) = lo_a;
        *(uint4 *)(dst + 8) = lo_b;
        *(uint4 *)(dst + 32) = hi_a;
        *(uint4 *)(dst + 40) = hi_b;
        if (h == 0 && pi == 0) d_l[lr] = gm_f16_bits_to_f32(hd.x & 0xFFFFu);
      }
      // ---- stage the activation tile: thread -> (token tt, 64 k)
      {
        const uint32_t tt = tid >> 1, kh = tid & 1u, tk = t0 + tt;
        uint4 v[8];
        if (tk < p.n_tokens) {
          const uint4 *src = (const uint4 *)(p.xh + (size_t)tk * p.in_dim + (size_t)s * 256u + 128u * h + 64u * kh);
#pragma unroll
          for (int i = 0; i < 8; i++) v[i] = src[i];
        } else {
#pragma unroll
          for (int i = 0; i < 8; i++) v[i] = make_uint4(0, 0, 0, 0);
        }
        uint4 *dst = (uint4 *)(B_l + tt * GM_LD + 64u * kh);
#pragma unroll
        for (int i = 0; i < 8; i++) dst[i] = v[i];
        if (h == 0 && tid < GM_BT) {
          const uint32_t tk2 = t0 + tid;
          ad_l[tid] = tk2 < p.n_tokens ? p.ad[(size_t)tk2 * p.nsb + s] : 0.0f;
        }
      }
      __syncthreads();
      // ---- 8 k-steps of 16
      const _Float16 *ap = A_l + (32u * wr + l32) * GM_LD + 8u * lh;
      const _Float16 *bp0 = B_l + (64u * wt_ + l32) * GM_LD + 8u * lh;
      const _Float16 *bp1 = bp0 + 32u * GM_LD;
#pragma unroll
      for (int kk = 0; kk < 8; kk++) {
        const half8 a = *(const half8 *)(ap + 16 * kk);
        const half8 b0 = *(const half8 *)(bp0 + 16 * kk);
        const half8 b1 = *(const half8 *)(bp1 + 16 * kk);
        if (h == 0) {
          c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b0, c0, 0, 0, 0);
          c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b1, c1, 0, 0, 0);
        } else {
          e0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b0, e0, 0, 0, 0);
          e1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b1, e1, 0, 0, 0);
        }
      }
      if (h == 1) {
        const float ad0 = ad_l[64u * wt_ + l32], ad1 = ad_l[64u * wt_ + 32u + l32];
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const uint32_t row_l = 32u * wr + 8u * (r / 4) + 4u * lh + (r % 4);
          const float d = d_l[row_l];
          y0[r] += ad0 * (d * (c0[r] + e0[r]));
          y1[r] += ad1 * (d * (c1[r] + e1[r]));
        }
      }
      __syncthreads();
    }
  }

  // ---------------- store: lane holds token column l32 (+32), rows in runs of four
#pragma unroll
  for (int jt = 0; jt < 2; jt++) {
    const uint32_t tk = t0 + 64u * wt_ + 32u * jt + l32;
    if (tk >= p.n_tokens) continue;
    const float16v &yy = jt ? y1 : y0;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const uint32_t row = r0 + 32u * wr + 8u * (r / 4) + 4u * lh + (r % 4);
      if (row < p.out_dim) p.y[(size_t)tk * p.out_dim + row] = yy[r];
    }
  }
}

size_t ogm_gemm_xh_bytes(uint32_t in_dim, uint32_t n_tokens) { return (size_t)in_dim * n_tokens * 2; }

bool ogm_gemm_supported(uint32_t ggml_type, uint32_t in_dim) {
  return ggml_type == OGM_Q4_K && in_dim % 1024u == 0;  // tiles of 16 rows x 4 super-blocks
}

hipError_t ogm_launch_gemm(const OgmGemmArgs &a, hipStream_t stream, const char **kernel_name) {
  if (a.n_tokens == 0 || a.out_dim == 0) return hipSuccess;
  if (!ogm_gemm_supported(a.ggml_type, a.in_dim)) return hipErrorInvalidValue;
  const size_t n8 = (size_t)a.in_dim * a.n_tokens / 8;
  hipLaunchKernelGGL(ogm_q8_to_f16_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, stream,
                     a.act.q, (_Float16 *)a.xh, n8);
  GemmParams p;
  p.wt = a.wt;
  p.xh = (const _Float16 *)a.xh;
  p.ad = a.act.d;
  p.bsum = a.act.bsum;
  p.y = a.y;
  p.in_dim = a.in_dim;
  p.out_dim = a.out_dim;
  p.n_tokens = a.n_tokens;
  p.nsb = a.in_dim / 256;
  p.nct = p.nsb / 4;
  p.nrb = (a.out_dim + 15) / 16;
  const size_t lds = (size_t)(GM_BN + GM_BT) * GM_LD * 2 + (GM_BN * 2 + GM_BT) * 4;
  const dim3 grid((a.out_dim + GM_BN - 1) / GM_BN, (a.n_tokens + GM_BT - 1) / GM_BT);
  hipLaunchKernelGGL(ogm_gemm_q4k_kernel, grid, dim3(256), lds, stream, p);
  if (kernel_name) *kernel_name = "ogm_gemm_q4k_kernel";
  return hipGetLastError();
}
