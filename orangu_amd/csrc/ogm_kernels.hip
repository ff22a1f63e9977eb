// gfx950 kernels of the quantized matmul path: the fused activation quantizer and the
// decode GEMV for Q8_0 / Q4_K / Q6_K weights in the tile-planar layout (ogm_layout.h).
//
// Arithmetic contract (engine/vecdot.rs of orangu-server):
//   * the quantizer reproduces quantize_act / quantize_act_k_row bit for bit;
//   * every per-block integer sum (isum, imin) is formed exactly, in i32;
//   * the f32 stage evaluates the reference's expression per block and then adds the block
//     terms in ascending block order with one accumulator, so the f32 result has the
//     reference's bits as well.  Build with -ffp-contract=off: an FMA would change them.
//
// Work mapping: one lane owns one block ("unit").  A workgroup owns one row block of the
// tile-planar layout (R rows); each of its waves takes one tile (R rows x C blocks) at a time and
// lane l reads piece p of its unit at tile*tile_bytes + p*1024 + l*16, so each load instruction
// of a wave covers one contiguous kilobyte.  The int8 activations sit in LDS.  Each lane leaves
// its block's f32 term in LDS; one lane per (row, token) then adds the row's terms in order.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "ogm_kernels.h"
#include "ogm_layout.h"
#include "ogm_nib32_dev.h"
#include "ogm_quant_dev.h"


// ------------------------------------------------------------------------------------------
// small helpers

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits16) {
  // Block scales are IEEE binary16 (quant.rs:511-528); the hardware conversion is exact for every
  // finite value, subnormal and infinity.
  return __half2float(__ushort_as_half((unsigned short)bits16));
}

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int acc) {
  // v_dot4_i32_i8: four signed int8 products added to acc, exact (dot16/dot32 of vecdot.rs:471-707)
  return __builtin_amdgcn_sdot4((int)a, (int)b, acc, false);
}

// Weights are read exactly once per launch: non-temporal loads keep them from displacing the
// activations (which every workgroup re-reads) in the caches, and measure ~6 % faster on a
// 66 MB launch.  OGM_WEIGHT_NT=0 builds plain loads, for comparison.
#ifndef OGM_WEIGHT_NT
#define OGM_WEIGHT_NT 1
#endif
typedef uint32_t ogm_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ldw16(const uint8_t *p) {
#if OGM_WEIGHT_NT
  const ogm_u32x4 v = __builtin_nontemporal_load((const ogm_u32x4 *)p);
  return make_uint4(v.x, v.y, v.z, v.w);
#else
  return *(const uint4 *)p;
#endif
}
__device__ __forceinline__ uint32_t ldw2(const uint8_t *p) {
#if OGM_WEIGHT_NT
  return __builtin_nontemporal_load((const uint16_t *)p);
#else
  return *(const uint16_t *)p;
#endif
}

__device__ __forceinline__ uint32_t ldw4(const uint8_t *p) {
#if OGM_WEIGHT_NT
  return __builtin_nontemporal_load((const uint32_t *)p);
#else
  return *(const uint32_t *)p;
#endif
}
// component c (a constant after unrolling) of a four-word piece
__device__ __forceinline__ uint32_t u4c(const uint4 &v, int c) { return c == 0 ? v.x : c == 1 ? v.y : c == 2 ? v.z : v.w; }

__device__ __forceinline__ int byte_of(uint32_t w, int i) { return (int)((w >> (8 * i)) & 0xFFu); }
__device__ __forceinline__ int sbyte_of(uint32_t w, int i) { return (int)(int8_t)((w >> (8 * i)) & 0xFFu); }
__device__ __forceinline__ int lo16(uint32_t w) { return (int)(int16_t)(w & 0xFFFFu); }
__device__ __forceinline__ int hi16(uint32_t w) { return ((int)w) >> 16; }

// ------------------------------------------------------------------------------------------
// activation quantizer
//
// One wave per 256 activations of one token; lane l holds elements 4l..4l+3.
//   amax  = fold(0, max(m, |v|)) ignoring NaN          (vecdot.rs:103, 3037)
//   scale = amax / 127 ; inv = scale > 0 ? 1/scale : 0   (vecdot.rs:106-107)
//   q     = clamp(round_half_away(v * inv), -127, 127), NaN -> 0   (vecdot.rs:117)
// GROUP = 32: scale per 32 (quantize_act); GROUP = 256: per 256 (quantize_act_k_row).

template <int GROUP>
__global__ __launch_bounds__(64) void ogm_quantize_kernel(const float *__restrict__ x,
                                                          uint32_t in_dim, OgmActDev act) {
  const uint32_t lane = threadIdx.x;
  const uint32_t t = blockIdx.y;
  const uint32_t e0 = blockIdx.x * 256u + lane * 4u;
  const bool active = e0 < in_dim;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (active) v = *(const float4 *)(x + (size_t)t * in_dim + e0);
  ogm_quantize_store<GROUP>(v, e0, active, lane, act.q + (size_t)t * in_dim,
                            act.d + (size_t)t * (in_dim / GROUP), act.sums + (size_t)t * (in_dim / 16),
                            act.bsum + (size_t)t * (in_dim / 32),
                            act.bs16 ? act.bs16 + (size_t)t * (in_dim / 16) : nullptr);
}

// The per-256 quantizer of a prefill batch that also lays the int8 activations out in the operand order of the
// GEMM whose waves all multiply (ogm_gemm.hip): chunk (token block of 32, step of 32 k) is 1 KiB, lane (l32, lh)'s
// 16 bytes -- the activations 32 step + 16 lh .. of token 32 block + l32 -- at 16 (32 lh + l32).  A workgroup takes
// 32 tokens x 256 activations, each of its eight waves four of the tokens; the eight chunks it fills are 8 KiB in
// a row, written as whole lines out of LDS.  Tokens past the last repeat it in the chunks (never multiplied into
// a stored output); their token-major outputs are not written.
__global__ __launch_bounds__(512) void ogm_quantize_xt_kernel(const float *__restrict__ x, uint32_t in_dim,
                                                              uint32_t n_tokens, OgmActDev act, int8_t *__restrict__ xt) {
  __shared__ uint4 tile[32][17];   // [token][16-byte piece], rows padded by a piece against bank conflicts
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t run = blockIdx.x, tb = blockIdx.y;
  const uint32_t e0 = run * 256u + lane * 4u;
  float4 v[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t t = min(tb * 32u + wave + 8u * i, n_tokens - 1u);
    v[i] = *(const float4 *)(x + (size_t)t * in_dim + e0);
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t tl = wave + 8u * i, t = tb * 32u + tl;
    const bool active = t < n_tokens;
    const uint32_t tc = min(t, n_tokens - 1u);
    const uint32_t packed = ogm_quantize_store<256>(v[i], e0, active, lane, act.q + (size_t)tc * in_dim,
                                                    act.d + (size_t)tc * (in_dim / 256), act.sums + (size_t)tc * (in_dim / 16),
                                                    act.bsum + (size_t)tc * (in_dim / 32),
                                                    act.bs16 ? act.bs16 + (size_t)tc * (in_dim / 16) : nullptr);
    ((uint32_t *)&tile[tl][lane >> 2])[lane & 3u] = packed;
  }
  __syncthreads();
  const uint32_t step = tid >> 6, slot = tid & 63u;   // the chunk of the eight, the lane of its operand
  const uint4 o = tile[slot & 31u][2u * step + (slot >> 5)];
  *(uint4 *)(xt + ((size_t)tb * (in_dim / 32u) + run * 8u + step) * 1024u + slot * 16u) = o;
}

hipError_t ogm_launch_quantize(int mode, const float *x, uint32_t in_dim, uint32_t n_tokens,
                               OgmActDev act, hipStream_t stream, int8_t *xt) {
  if (n_tokens == 0) return hipSuccess;
  if (xt != nullptr) {
    if (mode != 1 || in_dim % 256u != 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(ogm_quantize_xt_kernel, dim3(in_dim / 256u, (n_tokens + 31u) / 32u), dim3(512), 0, stream, x,
                       in_dim, n_tokens, act, xt);
    return hipGetLastError();
  }
  dim3 grid((in_dim + 255) / 256, n_tokens);
  if (mode == 0)
    hipLaunchKernelGGL(ogm_quantize_kernel<32>, grid, dim3(64), 0, stream, x, in_dim, act);
  else
    hipLaunchKernelGGL(ogm_quantize_kernel<256>, grid, dim3(64), 0, stream, x, in_dim, act);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// formats: how one lane loads its block and forms the block's integer sums

// LDS views of one token's activations, as the formats read them.
struct ActLds {
  const uint4 *xq;   // 16-byte chunks of q; chunk c of block `col` at [c * upr + col]
  const float *d;    // activation scale per scale group
  const uint4 *aux;  // per-block integer side sums (AUX16 chunks per block, [k * upr + col])
  uint32_t upr;      // blocks per row
};

// Q4_K: d:f16 | dmin:f16 | scales:u8[12] | qs:u8[128]            (quant.rs:664-697)
struct FmtQ4K {
  static constexpr int TERMS = 1;   // f32 terms a block leaves for the ordered sum
  static constexpr uint32_t TYPE = OGM_Q4_K;
  static constexpr int PIECES = 9, TILE_BYTES = 64 * 144, ELEMS = 256;
  static constexpr int XPIECES = 16;   // 16-byte activation chunks per block
  static constexpr int AUX16 = 1;      // bsum: 8 x i16 per block
  static constexpr int ACT_GROUP = 256;
  static constexpr bool HAS_MIN = true;
  static constexpr int MAX_THREADS = 512;   // launch bound: leaves 256 VGPRs to a lane
  static constexpr int MAX_THREADS_SINGLE = 1024;
  static constexpr bool HAS_UNPACK = false;
  struct Regs {
    uint4 p[PIECES];
  };
  __device__ static __forceinline__ void load(Regs &r, const uint8_t *wt, size_t tile, uint32_t lane) {
    const uint8_t *base = wt + tile * TILE_BYTES + lane * 16u;
#pragma unroll
    for (int i = 0; i < PIECES; i++) r.p[i] = ldw16(base + i * 1024);
  }
  // isum = sum_j sc_j * dot32(nibbles_j, x_j), imin = sum_j m_j * bsum_j     (vecdot.rs:3152-3178)
  template <int UPR>
  __device__ static __forceinline__ void sums(const Regs &r, const ActLds &a, uint32_t col,
                                              int &isum, int &imin) {
    // get_scale_min_k4 (quant.rs:653-662) for all eight sub-blocks at once, four bytes a word
    const uint32_t w0 = r.p[0].y, w1 = r.p[0].z, w2 = r.p[0].w;
    const uint32_t sca = w0 & 0x3F3F3F3Fu;                                   // sc 0..3
    const uint32_t mna = w1 & 0x3F3F3F3Fu;                                   // m  0..3
    const uint32_t scb = (w2 & 0x0F0F0F0Fu) | ((w0 >> 2) & 0x30303030u);     // sc 4..7
    const uint32_t mnb = ((w2 >> 4) & 0x0F0F0F0Fu) | ((w1 >> 2) & 0x30303030u);  // m 4..7
    const uint32_t m4 = 0x0F0F0F0Fu;
    const uint4 *xp = a.xq + col;
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;  // compile-time: LDS offsets become immediates
    // The four activation chunks of group g+1 are requested before group g is consumed.
    uint4 xa0 = xp[0], xa1 = xp[st], xb0 = xp[2 * st], xb1 = xp[3 * st];
    const uint4 b = a.aux[col];  // bsum_0..7 as i16
    isum = 0;
#pragma unroll
    for (int g = 0; g < 4; g++) {
      // qs[32g .. 32g+32): low nibbles are sub-block 2g (elements 64g..), high nibbles sub-block
      // 2g+1 (elements 64g+32..); piece 1+2g holds bytes 0..15 of the run, piece 2+2g bytes 16..31
      uint4 na0 = xa0, na1 = xa1, nb0 = xb0, nb1 = xb1;
      if (g < 3) {
        const uint4 *q = xp + 4 * (g + 1) * st;
        na0 = q[0];
        na1 = q[st];
        nb0 = q[2 * st];
        nb1 = q[3 * st];
      }
      const uint4 wa = r.p[1 + 2 * g], wb = r.p[2 + 2 * g];
      int dlo = 0, dhi = 0;
      dlo = dot4(wa.x & m4, xa0.x, dlo);
      dlo = dot4(wa.y & m4, xa0.y, dlo);
      dlo = dot4(wa.z & m4, xa0.z, dlo);
      dlo = dot4(wa.w & m4, xa0.w, dlo);
      dlo = dot4(wb.x & m4, xa1.x, dlo);
      dlo = dot4(wb.y & m4, xa1.y, dlo);
      dlo = dot4(wb.z & m4, xa1.z, dlo);
      dlo = dot4(wb.w & m4, xa1.w, dlo);
      dhi = dot4((wa.x >> 4) & m4, xb0.x, dhi);
      dhi = dot4((wa.y >> 4) & m4, xb0.y, dhi);
      dhi = dot4((wa.z >> 4) & m4, xb0.z, dhi);
      dhi = dot4((wa.w >> 4) & m4, xb0.w, dhi);
      dhi = dot4((wb.x >> 4) & m4, xb1.x, dhi);
      dhi = dot4((wb.y >> 4) & m4, xb1.y, dhi);
      dhi = dot4((wb.z >> 4) & m4, xb1.z, dhi);
      dhi = dot4((wb.w >> 4) & m4, xb1.w, dhi);
      const int j = 2 * g;
      const int sc_lo = j < 4 ? byte_of(sca, j) : byte_of(scb, j - 4);
      const int sc_hi = j + 1 < 4 ? byte_of(sca, j + 1) : byte_of(scb, j - 3);
      isum += sc_lo * dlo + sc_hi * dhi;
      xa0 = na0;
      xa1 = na1;
      xb0 = nb0;
      xb1 = nb1;
    }
    imin = byte_of(mna, 0) * lo16(b.x) + byte_of(mna, 1) * hi16(b.x) +
           byte_of(mna, 2) * lo16(b.y) + byte_of(mna, 3) * hi16(b.y) +
           byte_of(mnb, 0) * lo16(b.z) + byte_of(mnb, 1) * hi16(b.z) +
           byte_of(mnb, 2) * lo16(b.w) + byte_of(mnb, 3) * hi16(b.w);
  }
  // GEMV: total += act.d[s] * (d*isum - dmin*imin)                           (vecdot.rs:3175)
  __device__ static __forceinline__ float term_gemv(const Regs &r, float ad, int isum, int imin) {
    const float d = f16_bits_to_f32(r.p[0].x & 0xFFFFu), dmin = f16_bits_to_f32(r.p[0].x >> 16);
    return ad * (d * (float)isum - dmin * (float)imin);
  }
  // GEMM: acc -= (ad*dmin)*imin [all blocks first]; acc += ad*(d*isum)       (vecdot.rs:2229-2303)
  __device__ static __forceinline__ void term_gemm(const Regs &r, float ad, int isum, int imin,
                                                   float &tmin, float &tdot) {
    const float d = f16_bits_to_f32(r.p[0].x & 0xFFFFu), dmin = f16_bits_to_f32(r.p[0].x >> 16);
    tmin = ad * dmin * (float)imin;
    tdot = ad * (d * (float)isum);
  }
};

// Q3_K: hmask:u8[32] | qs:u8[64] | scales:u8[12] | d:f16                    (quant.rs:826-871)
// Eight runs of 32 elements; run p takes qs[32 (p / 4) + j] >> 2 (p % 4) and bit p of hmask[j],
// stored inverted: clear means subtract 4.  Sixteen six-bit scales, biased by 32, one per 16.
// Repacked as seven pieces, the last one holding scales and d (and two bytes of padding).
struct FmtQ3K {
  static constexpr int TERMS = 1;   // f32 terms a block leaves for the ordered sum
  static constexpr uint32_t TYPE = OGM_Q3_K;
  static constexpr int PIECES = 7, TILE_BYTES = 64 * 112, ELEMS = 256;
  static constexpr int XPIECES = 16;
  static constexpr int AUX16 = 2;  // per-16 sums of q: 16 x i16 per block
  static constexpr int ACT_GROUP = 256;
  static constexpr bool HAS_MIN = false;
  static constexpr int MAX_THREADS = 1024;
  static constexpr int MAX_THREADS_SINGLE = 1024;
  static constexpr bool HAS_UNPACK = false;
  struct Regs {
    uint4 p[PIECES];
  };
  __device__ static __forceinline__ void load(Regs &r, const uint8_t *wt, size_t tile, uint32_t lane) {
    const uint8_t *base = wt + tile * TILE_BYTES + lane * 16u;
#pragma unroll
    for (int i = 0; i < PIECES; i++) r.p[i] = ldw16(base + i * 1024);
  }
  // unpack_q3_k_scales (quant.rs:883-897) for scale i, minus the bias
  __device__ static __forceinline__ int scale(const uint4 &t, int i) {
    const uint32_t w[3] = {t.x, t.y, t.z};
    const int lowb = i < 8 ? i : i - 8;               // byte holding the low four bits
    const uint32_t lb = (w[lowb >> 2] >> (8 * (lowb & 3))) & 0xFFu;
    const uint32_t low = i < 8 ? (lb & 0xFu) : (lb >> 4);
    const uint32_t hb = (w[2] >> (8 * (i & 3))) & 0xFFu;   // byte 8 + i % 4
    const uint32_t high = (hb >> (2 * (i >> 2))) & 3u;
    return (int)(low | (high << 4)) - 32;
  }
  // isum = sum over 16 groups of (sc_g - 32) * dot16(q_g, x_g), q = two bits | inverted third bit
  // minus 4 (vecdot.rs:3273-3292); dot16(v - 4, x) = dot16(v, x) - 4 * sum16(x), exact.
  template <int UPR>
  __device__ static __forceinline__ void sums(const Regs &r, const ActLds &a, uint32_t col,
                                              int &isum, int &imin) {
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;
    const uint4 s_lo = a.aux[col], s_hi = a.aux[st + col];  // sum16 of groups 0..7, 8..15
    const uint32_t sw[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
    isum = 0;
    imin = 0;
#pragma unroll
    for (int p = 0; p < 8; p++) {
#pragma unroll
      for (int k = 0; k < 2; k++) {
        const int g = 2 * p + k;                       // group of 16: elements 32p + 16k ..
        const uint4 qs = r.p[2 + 2 * (p >> 2) + k];    // qs[32 (p / 4) + 16 k ..]
        const uint4 hm = r.p[k];                       // hmask[16 k ..]
        const uint4 x = a.xq[g * st + col];
        const int sh = 2 * (p & 3);
        const uint32_t m2 = 0x03030303u, m1 = 0x01010101u;
        int dot = 0;
        dot = dot4(((qs.x >> sh) & m2) | (((hm.x >> p) & m1) << 2), x.x, dot);
        dot = dot4(((qs.y >> sh) & m2) | (((hm.y >> p) & m1) << 2), x.y, dot);
        dot = dot4(((qs.z >> sh) & m2) | (((hm.z >> p) & m1) << 2), x.z, dot);
        dot = dot4(((qs.w >> sh) & m2) | (((hm.w >> p) & m1) << 2), x.w, dot);
        const int s16 = (g & 1) ? hi16(sw[g >> 1]) : lo16(sw[g >> 1]);
        isum += scale(r.p[6], g) * (dot - 4 * s16);
      }
    }
  }
  // GEMV: total += act.d[s] * d * isum                                       (vecdot.rs:3289)
  __device__ static __forceinline__ float term_gemv(const Regs &r, float ad, int isum, int) {
    return ad * f16_bits_to_f32(r.p[6].w & 0xFFFFu) * (float)isum;
  }
  // GEMM: the K-quant GEMM of Q6_K over a row unpacked by unpack_k_q3_k: acc += ad * (d * isum)
  // (vecdot.rs:2018-2021, 2389-2390)
  __device__ static __forceinline__ void term_gemm(const Regs &r, float ad, int isum, int,
                                                   float &tmin, float &tdot) {
    tmin = 0.0f;
    tdot = ad * (f16_bits_to_f32(r.p[6].w & 0xFFFFu) * (float)isum);
  }
};

// Q5_K: d:f16 | dmin:f16 | scales:u8[12] | qh:u8[32] | qs:u8[128]          (quant.rs:699-742)
// Q4_K with a fifth bit: bit j of qh[l] belongs to element l of sub-block j.
struct FmtQ5K {
  static constexpr int TERMS = 1;   // f32 terms a block leaves for the ordered sum
  static constexpr uint32_t TYPE = OGM_Q5_K;
  static constexpr int PIECES = 11, TILE_BYTES = 64 * 176, ELEMS = 256;
  static constexpr int XPIECES = 16;
  static constexpr int AUX16 = 1;      // bsum: 8 x i16 per block
  static constexpr int ACT_GROUP = 256;
  static constexpr bool HAS_MIN = true;
  static constexpr int MAX_THREADS = 512;
  static constexpr int MAX_THREADS_SINGLE = 512;
  static constexpr bool HAS_UNPACK = false;
  struct Regs {
    uint4 p[PIECES];
  };
  __device__ static __forceinline__ void load(Regs &r, const uint8_t *wt, size_t tile, uint32_t lane) {
    const uint8_t *base = wt + tile * TILE_BYTES + lane * 16u;
#pragma unroll
    for (int i = 0; i < PIECES; i++) r.p[i] = ldw16(base + i * 1024);
  }
  // Four weights of sub-block `bit`: nibbles n (already masked) plus 16 where the qh bytes have
  // bit `bit` set.
  __device__ static __forceinline__ uint32_t with_high(uint32_t n, uint32_t qh, int bit) {
    return n | (((qh >> bit) & 0x01010101u) << 4);
  }
  // isum = sum_j sc_j * dot32(q5_j, x_j), imin = sum_j m_j * bsum_j          (vecdot.rs:3181-3213)
  template <int UPR>
  __device__ static __forceinline__ void sums(const Regs &r, const ActLds &a, uint32_t col,
                                              int &isum, int &imin) {
    const uint32_t w0 = r.p[0].y, w1 = r.p[0].z, w2 = r.p[0].w;
    const uint32_t sca = w0 & 0x3F3F3F3Fu;                                   // sc 0..3
    const uint32_t mna = w1 & 0x3F3F3F3Fu;                                   // m  0..3
    const uint32_t scb = (w2 & 0x0F0F0F0Fu) | ((w0 >> 2) & 0x30303030u);     // sc 4..7
    const uint32_t mnb = ((w2 >> 4) & 0x0F0F0F0Fu) | ((w1 >> 2) & 0x30303030u);  // m 4..7
    const uint32_t m4 = 0x0F0F0F0Fu;
    const uint4 ha = r.p[1], hb = r.p[2];   // qh[0..16), qh[16..32)
    const uint4 *xp = a.xq + col;
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;
    uint4 xa0 = xp[0], xa1 = xp[st], xb0 = xp[2 * st], xb1 = xp[3 * st];
    const uint4 b = a.aux[col];  // bsum_0..7 as i16
    isum = 0;
#pragma unroll
    for (int g = 0; g < 4; g++) {
      // qs[32g .. 32g+32): low nibbles are sub-block 2g, high nibbles sub-block 2g+1; piece
      // 3+2g holds bytes 0..15 of the run (qh bytes 0..15), piece 4+2g bytes 16..31
      uint4 na0 = xa0, na1 = xa1, nb0 = xb0, nb1 = xb1;
      if (g < 3) {
        const uint4 *q = xp + 4 * (g + 1) * st;
        na0 = q[0];
        na1 = q[st];
        nb0 = q[2 * st];
        nb1 = q[3 * st];
      }
      const uint4 wa = r.p[3 + 2 * g], wb = r.p[4 + 2 * g];
      const int lo = 2 * g, hi = 2 * g + 1;
      int dlo = 0, dhi = 0;
      dlo = dot4(with_high(wa.x & m4, ha.x, lo), xa0.x, dlo);
      dlo = dot4(with_high(wa.y & m4, ha.y, lo), xa0.y, dlo);
      dlo = dot4(with_high(wa.z & m4, ha.z, lo), xa0.z, dlo);
      dlo = dot4(with_high(wa.w & m4, ha.w, lo), xa0.w, dlo);
      dlo = dot4(with_high(wb.x & m4, hb.x, lo), xa1.x, dlo);
      dlo = dot4(with_high(wb.y & m4, hb.y, lo), xa1.y, dlo);
      dlo = dot4(with_high(wb.z & m4, hb.z, lo), xa1.z, dlo);
      dlo = dot4(with_high(wb.w & m4, hb.w, lo), xa1.w, dlo);
      dhi = dot4(with_high((wa.x >> 4) & m4, ha.x, hi), xb0.x, dhi);
      dhi = dot4(with_high((wa.y >> 4) & m4, ha.y, hi), xb0.y, dhi);
      dhi = dot4(with_high((wa.z >> 4) & m4, ha.z, hi), xb0.z, dhi);
      dhi = dot4(with_high((wa.w >> 4) & m4, ha.w, hi), xb0.w, dhi);
      dhi = dot4(with_high((wb.x >> 4) & m4, hb.x, hi), xb1.x, dhi);
      dhi = dot4(with_high((wb.y >> 4) & m4, hb.y, hi), xb1.y, dhi);
      dhi = dot4(with_high((wb.z >> 4) & m4, hb.z, hi), xb1.z, dhi);
      dhi = dot4(with_high((wb.w >> 4) & m4, hb.w, hi), xb1.w, dhi);
      const int sc_lo = lo < 4 ? byte_of(sca, lo) : byte_of(scb, lo - 4);
      const int sc_hi = hi < 4 ? byte_of(sca, hi) : byte_of(scb, hi - 4);
      isum += sc_lo * dlo + sc_hi * dhi;
      xa0 = na0;
      xa1 = na1;
      xb0 = nb0;
      xb1 = nb1;
    }
    imin = byte_of(mna, 0) * lo16(b.x) + byte_of(mna, 1) * hi16(b.x) +
           byte_of(mna, 2) * lo16(b.y) + byte_of(mna, 3) * hi16(b.y) +
           byte_of(mnb, 0) * lo16(b.z) + byte_of(mnb, 1) * hi16(b.z) +
           byte_of(mnb, 2) * lo16(b.w) + byte_of(mnb, 3) * hi16(b.w);
  }
  // GEMV: total += act.d[s] * (d*isum - dmin*imin)                           (vecdot.rs:3210)
  __device__ static __forceinline__ float term_gemv(const Regs &r, float ad, int isum, int imin) {
    const float d = f16_bits_to_f32(r.p[0].x & 0xFFFFu), dmin = f16_bits_to_f32(r.p[0].x >> 16);
    return ad * (d * (float)isum - dmin * (float)imin);
  }
  // GEMM: the K-quant GEMM of Q4_K over a row unpacked with the fifth bit    (vecdot.rs:2010-2013, 2229-2303)
  __device__ static __forceinline__ void term_gemm(const Regs &r, float ad, int isum, int imin,
                                                   float &tmin, float &tdot) {
    const float d = f16_bits_to_f32(r.p[0].x & 0xFFFFu), dmin = f16_bits_to_f32(r.p[0].x >> 16);
    tmin = ad * dmin * (float)imin;
    tdot = ad * (d * (float)isum);
  }
};

// Q6_K: ql:u8[128] | qh:u8[64] | scales:i8[16] | d:f16                      (quant.rs:744-787)
struct FmtQ6K {
  static constexpr int TERMS = 1;   // f32 terms a block leaves for the ordered sum
  static constexpr uint32_t TYPE = OGM_Q6_K;
  static constexpr int PIECES = 13, TILE_BYTES = 64 * 210, ELEMS = 256;
  static constexpr int XPIECES = 16;
  static constexpr int AUX16 = 2;  // per-16 sums of q: 16 x i16 per block
  static constexpr int ACT_GROUP = 256;
  static constexpr bool HAS_MIN = false;
  static constexpr int MAX_THREADS = 512;  // 13 pieces a lane: needs more than 128 registers
  static constexpr int MAX_THREADS_SINGLE = 512;
  struct Regs {
    uint4 p[PIECES];
    uint32_t d16;
  };
  __device__ static __forceinline__ void load(Regs &r, const uint8_t *wt, size_t tile, uint32_t lane) {
    const uint8_t *tb = wt + tile * TILE_BYTES;
    const uint8_t *base = tb + lane * 16u;
#pragma unroll
    for (int i = 0; i < PIECES; i++) r.p[i] = ldw16(base + i * 1024);
    r.d16 = ldw2(tb + PIECES * 1024 + lane * 2u);
  }
  __device__ static __forceinline__ int run_dot(uint4 ql, uint4 qh, uint4 x, int r) {
    // 6-bit value = nibble | (two bits of qh) << 4, still carrying the +32 bias (0..63)
    const uint32_t m4 = 0x0F0F0F0Fu, m2 = 0x30303030u;
    uint32_t v0, v1, v2, v3;
    if (r < 2) {
      v0 = ql.x & m4; v1 = ql.y & m4; v2 = ql.z & m4; v3 = ql.w & m4;
    } else {
      v0 = (ql.x >> 4) & m4; v1 = (ql.y >> 4) & m4; v2 = (ql.z >> 4) & m4; v3 = (ql.w >> 4) & m4;
    }
    // ((qh >> 2r) & 3) << 4
    if (r == 0) { v0 |= (qh.x << 4) & m2; v1 |= (qh.y << 4) & m2; v2 |= (qh.z << 4) & m2; v3 |= (qh.w << 4) & m2; }
    if (r == 1) { v0 |= (qh.x << 2) & m2; v1 |= (qh.y << 2) & m2; v2 |= (qh.z << 2) & m2; v3 |= (qh.w << 2) & m2; }
    if (r == 2) { v0 |= qh.x & m2; v1 |= qh.y & m2; v2 |= qh.z & m2; v3 |= qh.w & m2; }
    if (r == 3) { v0 |= (qh.x >> 2) & m2; v1 |= (qh.y >> 2) & m2; v2 |= (qh.z >> 2) & m2; v3 |= (qh.w >> 2) & m2; }
    int acc = 0;
    acc = dot4(v0, x.x, acc);
    acc = dot4(v1, x.y, acc);
    acc = dot4(v2, x.z, acc);
    acc = dot4(v3, x.w, acc);
    return acc;
  }
  // isum = sum over 16 groups of sc_g * dot16(q_g - 32, x_g)                (vecdot.rs:3215-3241)
  // with dot16(q - 32, x) = dot16(q, x) - 32 * sum16(x), exact in integers.
  template <int UPR>
  __device__ static __forceinline__ void sums(const Regs &r, const ActLds &a, uint32_t col,
                                              int &isum, int &imin) {
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;
    const uint4 s_lo = a.aux[col], s_hi = a.aux[st + col];  // sum16 of groups 0..7, 8..15
    const uint32_t sw[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
    const uint32_t scw[4] = {r.p[12].x, r.p[12].y, r.p[12].z, r.p[12].w};
    isum = 0;
    imin = 0;
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
        const int R = 4 * h + rr;  // run of 32 elements: 128h + 32rr ..
#pragma unroll
        for (int k = 0; k < 2; k++) {
          const int g = 2 * R + k;  // group of 16
          const uint4 ql = r.p[4 * h + 2 * (rr & 1) + k];
          const uint4 qh = r.p[8 + 2 * h + k];
          const uint4 x = a.xq[g * st + col];
          const int dot = run_dot(ql, qh, x, rr);
          const int s16 = (g & 1) ? hi16(sw[g >> 1]) : lo16(sw[g >> 1]);
          isum += sbyte_of(scw[g >> 2], g & 3) * (dot - 32 * s16);
        }
      }
    }
  }
  // For several tokens per launch: the block's 6-bit values (still carrying the +32) unpacked
  // once, four per word, group g of 16 at v[4g .. 4g+3]; every token then only runs the dots.
  static constexpr bool HAS_UNPACK = true;
  struct Unpacked {
    uint32_t v[64];
  };
  __device__ static __forceinline__ void unpack(const Regs &r, Unpacked &u) {
    const uint32_t m4 = 0x0F0F0F0Fu, m2 = 0x30303030u;
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
      for (int rr = 0; rr < 4; rr++) {
#pragma unroll
        for (int k = 0; k < 2; k++) {
          const int g = 2 * (4 * h + rr) + k;
          const uint4 ql = r.p[4 * h + 2 * (rr & 1) + k];
          const uint4 qh = r.p[8 + 2 * h + k];
          const uint32_t qlw[4] = {ql.x, ql.y, ql.z, ql.w}, qhw[4] = {qh.x, qh.y, qh.z, qh.w};
#pragma unroll
          for (int w = 0; w < 4; w++) {
            const uint32_t nib = (rr < 2 ? qlw[w] : (qlw[w] >> 4)) & m4;
            // ((qh >> 2 rr) & 3) << 4
            const uint32_t hi = rr == 0 ? (qhw[w] << 4) : rr == 1 ? (qhw[w] << 2) : rr == 2 ? qhw[w] : (qhw[w] >> 2);
            u.v[4 * g + w] = nib | (hi & m2);
          }
        }
      }
    }
  }
  template <int UPR>
  __device__ static __forceinline__ void sums_unpacked(const Unpacked &u, const Regs &r, const ActLds &a,
                                                       uint32_t col, int &isum, int &imin) {
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;
    const uint4 s_lo = a.aux[col], s_hi = a.aux[st + col];  // sum16 of groups 0..7, 8..15
    const uint32_t sw[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
    const uint32_t scw[4] = {r.p[12].x, r.p[12].y, r.p[12].z, r.p[12].w};
    isum = 0;
    imin = 0;
#pragma unroll
    for (int g = 0; g < 16; g++) {
      const uint4 x = a.xq[g * st + col];
      int dot = 0;
      dot = dot4(u.v[4 * g + 0], x.x, dot);
      dot = dot4(u.v[4 * g + 1], x.y, dot);
      dot = dot4(u.v[4 * g + 2], x.z, dot);
      dot = dot4(u.v[4 * g + 3], x.w, dot);
      const int s16 = (g & 1) ? hi16(sw[g >> 1]) : lo16(sw[g >> 1]);
      isum += sbyte_of(scw[g >> 2], g & 3) * (dot - 32 * s16);
    }
  }
  // GEMV: total += act.d[s] * d * isum                                       (vecdot.rs:3238)
  __device__ static __forceinline__ float term_gemv(const Regs &r, float ad, int isum, int) {
    return ad * f16_bits_to_f32(r.d16) * (float)isum;
  }
  // GEMM: acc += ad * (d * isum)                                              (vecdot.rs:2389-2390)
  __device__ static __forceinline__ void term_gemm(const Regs &r, float ad, int isum, int,
                                                   float &tmin, float &tdot) {
    tmin = 0.0f;
    tdot = ad * (f16_bits_to_f32(r.d16) * (float)isum);
  }
};

// Q8_0: d:f16 | qs:i8[32]                                                     (quant.rs:638-649)
struct FmtQ80 {
  static constexpr int TERMS = 1;   // f32 terms a block leaves for the ordered sum
  static constexpr uint32_t TYPE = OGM_Q8_0;
  static constexpr int PIECES = 2, TILE_BYTES = 64 * 34, ELEMS = 32;
  static constexpr int XPIECES = 2;
  static constexpr int AUX16 = 0;
  static constexpr int ACT_GROUP = 32;
  static constexpr bool HAS_MIN = false;
  static constexpr int MAX_THREADS = 1024;
  static constexpr int MAX_THREADS_SINGLE = 1024;
  static constexpr bool HAS_UNPACK = false;
  struct Regs {
    uint4 p[PIECES];
    uint32_t d16;
  };
  __device__ static __forceinline__ void load(Regs &r, const uint8_t *wt, size_t tile, uint32_t lane) {
    const uint8_t *tb = wt + tile * TILE_BYTES;
    const uint8_t *base = tb + lane * 16u;
    r.p[0] = ldw16(base);
    r.p[1] = ldw16(base + 1024);
    r.d16 = ldw2(tb + PIECES * 1024 + lane * 2u);
  }
  template <int UPR>
  __device__ static __forceinline__ void sums(const Regs &r, const ActLds &a, uint32_t col,
                                              int &isum, int &imin) {
    const uint4 x0 = a.xq[col], x1 = a.xq[(UPR ? (uint32_t)UPR : a.upr) + col];
    int acc = 0;
    acc = dot4(r.p[0].x, x0.x, acc);
    acc = dot4(r.p[0].y, x0.y, acc);
    acc = dot4(r.p[0].z, x0.z, acc);
    acc = dot4(r.p[0].w, x0.w, acc);
    acc = dot4(r.p[1].x, x1.x, acc);
    acc = dot4(r.p[1].y, x1.y, acc);
    acc = dot4(r.p[1].z, x1.z, acc);
    acc = dot4(r.p[1].w, x1.w, acc);
    isum = acc;
    imin = 0;
  }
  // GEMV: total += dw * act.d[b] * isum (vecdot.rs:2835); the flat GEMM's ad*dw*isum
  // (vecdot.rs:2623) is the same product, so one form serves both orders.
  __device__ static __forceinline__ float term_gemv(const Regs &r, float ad, int isum, int) {
    return f16_bits_to_f32(r.d16) * ad * (float)isum;
  }
  __device__ static __forceinline__ void term_gemm(const Regs &r, float ad, int isum, int,
                                                   float &tmin, float &tdot) {
    tmin = 0.0f;
    tdot = ad * f16_bits_to_f32(r.d16) * (float)isum;
  }
};

// The other symmetric per-32 types (vecdot.rs:2842-2883): one 16-byte piece of nibbles per block,
// elements 0..16 from the low nibbles, 16..32 from the high nibbles, total += dw * act.d[b] * isum
// like Q8_0.  KIND 0: Q4_0 (nibble - 8); 1: Q5_0 (nibble | fifth bit from qh, - 16); 2: IQ4_NL
// (nibble indexes the sixteen levels of iq_grids.rs:5941-5943).
template <int KIND>
struct FmtNib32 {
  static constexpr int TERMS = 1;
  static constexpr uint32_t TYPE = KIND == 0 ? OGM_Q4_0 : (KIND == 1 ? OGM_Q5_0 : (KIND == 2 ? OGM_IQ4_NL : OGM_Q5_1));
  static constexpr int TAIL = KIND == 1 ? 6 : (KIND == 3 ? 8 : 2);
  static constexpr int PIECES = 1, TILE_BYTES = 64 * (16 + TAIL), ELEMS = 32;
  static constexpr int XPIECES = 2;
  static constexpr int AUX16 = 0;
  static constexpr int ACT_GROUP = 32;
  static constexpr bool HAS_MIN = false;
  static constexpr int MAX_THREADS = 1024;
  static constexpr int MAX_THREADS_SINGLE = 1024;
  static constexpr bool HAS_UNPACK = false;
  struct Regs {
    uint4 p[PIECES];
    uint32_t d16, qh;   // Q5_1: d16 = d | m << 16
  };
  __device__ static __forceinline__ void load(Regs &r, const uint8_t *wt, size_t tile, uint32_t lane) {
    const uint8_t *tb = wt + tile * TILE_BYTES;
    r.p[0] = ldw16(tb + lane * 16u);
    const uint8_t *t = tb + 1024 + lane * TAIL;   // d, then qh (two-byte aligned); Q5_1: d, m, qh (eight-byte aligned)
    if constexpr (KIND == 3) {
      r.d16 = ldw4(t);
      r.qh = ldw4(t + 4);
    } else {
      r.d16 = ldw2(t);
      r.qh = KIND == 1 ? (ldw2(t + 2) | (ldw2(t + 4) << 16)) : 0u;
    }
  }
  __device__ static __forceinline__ uint32_t weights(uint32_t n, uint32_t h4) {
    return ogm_nib32_weights<KIND>(n, h4);
  }
  template <int UPR>
  __device__ static __forceinline__ void sums(const Regs &r, const ActLds &a, uint32_t col,
                                              int &isum, int &imin) {
    const uint4 x0 = a.xq[col], x1 = a.xq[(UPR ? (uint32_t)UPR : a.upr) + col];
    const uint32_t m4 = 0x0F0F0F0Fu;
    const uint32_t qw[4] = {r.p[0].x, r.p[0].y, r.p[0].z, r.p[0].w};
    const uint32_t xl[4] = {x0.x, x0.y, x0.z, x0.w}, xh[4] = {x1.x, x1.y, x1.z, x1.w};
    int acc = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
      // bytes 4k .. 4k+3 of qs: elements 4k.. (bits 4k.. of qh) and 16+4k.. (bits 16+4k..)
      acc = dot4(weights(qw[k] & m4, (r.qh >> (4 * k)) & 0xFu), xl[k], acc);
      acc = dot4(weights((qw[k] >> 4) & m4, (r.qh >> (16 + 4 * k)) & 0xFu), xh[k], acc);
    }
    isum = acc;
    imin = 0;
    if constexpr (KIND == 3) {   // Q5_1: the block's activation sum (block_sum, vecdot.rs:2701-2703), from the int8 themselves
      int bs = 0;
#pragma unroll
      for (int k = 0; k < 4; k++) {
        bs = dot4(0x01010101u, xl[k], bs);
        bs = dot4(0x01010101u, xh[k], bs);
      }
      imin = bs;
    }
  }
  // Q5_1 (vecdot.rs:2886-2899): total += act.d[b] * (dw * isum + m * block_sum); the rows-unpacked-once
  // form of several tokens (scale * isum - (-m) * block_sum, vecdot.rs:1302-1314, 1698) has the same bits
  __device__ static __forceinline__ float term_gemv(const Regs &r, float ad, int isum, int bs) {
    if constexpr (KIND == 3)
      return ad * (f16_bits_to_f32(r.d16 & 0xFFFFu) * (float)isum + f16_bits_to_f32(r.d16 >> 16) * (float)bs);
    else
      return f16_bits_to_f32(r.d16) * ad * (float)isum;
  }
  // flat GEMM: acc += d * s * dot32 (vecdot.rs:2622-2623)
  __device__ static __forceinline__ void term_gemm(const Regs &r, float ad, int isum, int bs,
                                                   float &tmin, float &tdot) {
    tmin = 0.0f;
    if constexpr (KIND == 3) tdot = term_gemv(r, ad, isum, bs);
    else tdot = ad * f16_bits_to_f32(r.d16) * (float)isum;
  }
};
typedef FmtNib32<0> FmtQ40;
typedef FmtNib32<1> FmtQ50;
typedef FmtNib32<2> FmtIQ4NL;
typedef FmtNib32<3> FmtQ51;

// IQ4_XS: d:f16 | scales_h:u16 | scales_l:u8[4] | qs:u8[128]                 (quant.rs:1350-1375)
// Eight sub-blocks of 32: sixteen bytes of nibbles each (elements 0..16 low, 16..32 high, through
// IQ4_NL's sixteen levels), a six-bit scale biased by 32.  The block's 136 bytes are cut at
// multiples of 16 from its start, so sub-block ib's bytes are the upper half of piece ib and the
// lower half of piece ib + 1.
struct FmtIQ4XS {
  static constexpr int TERMS = 1;
  static constexpr uint32_t TYPE = OGM_IQ4_XS;
  static constexpr int PIECES = 9, TILE_BYTES = 64 * 144, ELEMS = 256;
  static constexpr int XPIECES = 16;
  static constexpr int AUX16 = 0;
  static constexpr int ACT_GROUP = 256;
  static constexpr bool HAS_MIN = false;
  static constexpr int MAX_THREADS = 512;
  static constexpr int MAX_THREADS_SINGLE = 1024;
  static constexpr bool HAS_UNPACK = false;
  struct Regs {
    uint4 p[PIECES];
  };
  __device__ static __forceinline__ void load(Regs &r, const uint8_t *wt, size_t tile, uint32_t lane) {
    const uint8_t *base = wt + tile * TILE_BYTES + lane * 16u;
#pragma unroll
    for (int i = 0; i < PIECES; i++) r.p[i] = ldw16(base + i * 1024);
  }
  // isum = sum_ib ls_ib * dot32(levels_ib, x_ib)                             (vecdot.rs:3245-3266)
  template <int UPR>
  __device__ static __forceinline__ void sums(const Regs &r, const ActLds &a, uint32_t col, int &isum, int &imin) {
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;
    const uint4 *xp = a.xq + col;
    const uint32_t sh = r.p[0].x >> 16, sl = r.p[0].y, m4 = 0x0F0F0F0Fu;
    isum = 0;
    imin = 0;
#pragma unroll
    for (int ib = 0; ib < 8; ib++) {
      const uint4 xl = xp[(2 * ib) * st], xh = xp[(2 * ib + 1) * st];
      int dot = 0;
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const int w = 2 + 4 * ib + k;   // word of the block: bytes 8 + 16 ib + 4 k ..
        const uint32_t qw = u4c(r.p[w >> 2], w & 3);
        dot = dot4(ogm_nib32_weights<2>(qw & m4, 0u), u4c(xl, k), dot);
        dot = dot4(ogm_nib32_weights<2>((qw >> 4) & m4, 0u), u4c(xh, k), dot);
      }
      const int ls = (int)(((sl >> (4 * ib)) & 0xFu) | (((sh >> (2 * ib)) & 3u) << 4)) - 32;
      isum += ls * dot;
    }
  }
  // GEMV: total += act.d[s] * d * isum                                        (vecdot.rs:3263)
  __device__ static __forceinline__ float term_gemv(const Regs &r, float ad, int isum, int) {
    return ad * f16_bits_to_f32(r.p[0].x & 0xFFFFu) * (float)isum;
  }
  // GEMM: acc += ad * (d * isum)                                             (vecdot.rs:2296-2300)
  __device__ static __forceinline__ void term_gemm(const Regs &r, float ad, int isum, int, float &tmin, float &tdot) {
    tmin = 0.0f;
    tdot = ad * (f16_bits_to_f32(r.p[0].x & 0xFFFFu) * (float)isum);
  }
};

// Q2_K: scales:u8[16] | qs:u8[64] | d:f16 | dmin:f16                         (quant.rs:798-827)
// Eight runs of 32 two-bit values: run p takes qs[32 (p / 4) + j] >> 2 (p % 4); group g of 16 has a
// four-bit scale (low nibble of scales[g]) and a four-bit min (high nibble).
// GENERIC false: one token against per-256 activations (dot_k_row_q2_k, vecdot.rs:3296-3318).
// GENERIC true: several tokens through matmul, the rows-unpacked-once path over per-32 activations
// (unpack_q2_k + dot_unpacked, vecdot.rs:1144-1164, 420-425, 1722-1728): sixteen f32 terms a block,
// act.d[g / 2] * ((d * sc_g) * isum_g - (dmin * mn_g) * sums[g]), added in group order.
template <bool GENERIC>
struct FmtQ2KT {
  static constexpr int TERMS = GENERIC ? 16 : 1;
  static constexpr uint32_t TYPE = OGM_Q2_K;
  static constexpr int PIECES = 5, TILE_BYTES = 64 * 84, ELEMS = 256;
  static constexpr int XPIECES = 16;
  static constexpr int AUX16 = 2;   // per-16 sums of q: 16 x i16 per block
  static constexpr int ACT_GROUP = GENERIC ? 32 : 256;
  static constexpr bool HAS_MIN = !GENERIC;
  static constexpr int MAX_THREADS = 512;
  static constexpr int MAX_THREADS_SINGLE = 1024;
  static constexpr bool HAS_UNPACK = false;
  struct Regs {
    uint4 p[PIECES];
    uint32_t dd;   // d | dmin << 16
  };
  __device__ static __forceinline__ void load(Regs &r, const uint8_t *wt, size_t tile, uint32_t lane) {
    const uint8_t *tb = wt + tile * TILE_BYTES;
    const uint8_t *base = tb + lane * 16u;
#pragma unroll
    for (int i = 0; i < PIECES; i++) r.p[i] = ldw16(base + i * 1024);
    r.dd = ldw4(tb + PIECES * 1024 + lane * 4u);
  }
  // the integer dot of group g (sixteen weights) and its activation sum
  template <int UPR>
  __device__ static __forceinline__ void group(const Regs &r, const ActLds &a, uint32_t col, const uint32_t *sw, int g,
                                               int &dot, int &s16, int &sc) {
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;
    const int p = g >> 1, shift = 2 * (p & 3);
    const uint4 q = r.p[1 + 2 * (p >> 2) + (g & 1)];   // bytes 16 (g & 1) .. of the run's 32
    const uint4 x = a.xq[g * st + col];
    dot = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) dot = dot4((u4c(q, k) >> shift) & 0x03030303u, u4c(x, k), dot);
    s16 = (g & 1) ? hi16(sw[g >> 1]) : lo16(sw[g >> 1]);
    sc = byte_of(u4c(r.p[0], g >> 2), g & 3);
  }
  template <int UPR>
  __device__ static __forceinline__ void sums(const Regs &r, const ActLds &a, uint32_t col, int &isum, int &imin) {
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;
    const uint4 s_lo = a.aux[col], s_hi = a.aux[st + col];  // sum16 of groups 0..7, 8..15
    const uint32_t sw[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
    isum = 0;
    imin = 0;
#pragma unroll
    for (int g = 0; g < 16; g++) {
      int dot, s16, sc;
      group<UPR>(r, a, col, sw, g, dot, s16, sc);
      isum += (sc & 0xF) * dot;
      imin += (sc >> 4) * s16;
    }
  }
  template <int UPR>
  __device__ static __forceinline__ void terms(const Regs &r, const ActLds &a, uint32_t col, float *out) {
    const uint32_t st = UPR ? (uint32_t)UPR : a.upr;
    const uint4 s_lo = a.aux[col], s_hi = a.aux[st + col];
    const uint32_t sw[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
    const float d = f16_bits_to_f32(r.dd & 0xFFFFu), dmin = f16_bits_to_f32(r.dd >> 16);
#pragma unroll
    for (int g = 0; g < 16; g++) {
      int dot, s16, sc;
      group<UPR>(r, a, col, sw, g, dot, s16, sc);
      const float scale = d * (float)(sc & 0xF), mn = dmin * (float)(sc >> 4);
      out[g] = a.d[col * 8u + (g >> 1)] * (scale * (float)dot - mn * (float)s16);
    }
  }
  // GEMV: total += act.d[s] * (d * isum - dmin * imin)                        (vecdot.rs:3315)
  __device__ static __forceinline__ float term_gemv(const Regs &r, float ad, int isum, int imin) {
    const float d = f16_bits_to_f32(r.dd & 0xFFFFu), dmin = f16_bits_to_f32(r.dd >> 16);
    return ad * (d * (float)isum - dmin * (float)imin);
  }
  // (the per-256 form has no several-token order of its own: matmul takes the GENERIC form)
  __device__ static __forceinline__ void term_gemm(const Regs &r, float ad, int isum, int imin, float &tmin, float &tdot) {
    tmin = 0.0f;
    tdot = term_gemv(r, ad, isum, imin);
  }
};
typedef FmtQ2KT<false> FmtQ2K;
typedef FmtQ2KT<true> FmtQ2KGen;

// ------------------------------------------------------------------------------------------
// GEMV kernel
//
// One workgroup per row block (R rows of the tile-planar layout), one tile (R rows x C blocks)
// per wave at a time; lane c*R + r of the wave owns block c of row r of its tile.  Every lane
// forms its block's f32 term and leaves it in the workgroup's LDS table [block][row]; after one
// barrier a lane per (row, token) adds the row's terms in ascending block order with one
// accumulator, which is the reference's summation order.
//
// Vector-memory data returns in issue order, so the few activation loads are issued first and a
// barrier (waiting for no data) keeps every one of them ahead of the workgroup's weight loads;
// the code then waits with vmcnt for the activations only and the weights stay in flight across
// the LDS hand-off.  All these loads use clamped indices instead of branches so that the
// compiler can count them.

struct GemvParams {
  // Up to OGM_GEMV_MAX_MATS matrices of one type and in_dim read the same activations; the
  // grid is the concatenation of their row blocks.
  const uint8_t *wt[OGM_GEMV_MAX_MATS];
  float *y[OGM_GEMV_MAX_MATS];
  uint32_t out_dim[OGM_GEMV_MAX_MATS];
  uint32_t wg_end[OGM_GEMV_MAX_MATS];  // workgroups of matrices 0..m, running total
  OgmActDev act;
  int32_t *dump_isum, *dump_imin;
  uint32_t in_dim, upr;            // upr = blocks per row
  uint32_t n_tokens;
  uint32_t C, nct;                // tile shape: C blocks x R rows, nct = ceil(upr / C) column tiles
  uint32_t lane_acc;              // formats of several terms a block, tiles one block wide, one wave: see gemv_lane_acc
};

template <class F, bool GEMM_ORDER>
__host__ __device__ constexpr int n_term_arrays() {
  return (GEMM_ORDER && F::HAS_MIN && F::TYPE != OGM_Q2_K) ? 2 : 1;   // Q4_K, Q5_K: the min pass first
}

static const size_t OGM_LDS_BUDGET = 80 * 1024;   // what a launch aims for (two workgroups to a compute unit): batches are cut to fit
static const size_t OGM_LDS_UNASKED = 64 * 1024;  // what a kernel gets without asking (hipFuncAttributeMaxDynamicSharedMemorySize)
static const size_t OGM_LDS_MAX = 160 * 1024;     // what a workgroup can have when even one token of one row block needs more

// Dynamic LDS bytes of one workgroup.
template <class F, bool GEMM_ORDER>
static size_t gemv_lds_bytes(uint32_t in_dim, uint32_t n_tokens) {
  const size_t upr = in_dim / F::ELEMS;
  const size_t n_scale = in_dim / F::ACT_GROUP;
  const OgmTiling tl = ogm_tiling_for((uint32_t)upr, 1);
  size_t b = (size_t)n_tokens * in_dim;                     // xq
  b += (size_t)n_tokens * upr * F::AUX16 * 16;              // aux
  b += (size_t)n_tokens * n_scale * 4;                      // act.d
  b = (b + 15) & ~(size_t)15;
  b += (size_t)n_term_arrays<F, GEMM_ORDER>() * n_tokens * upr * tl.R * 4 * F::TERMS;  // terms
  return b;
}

// A format that leaves several terms a block (Q2_K over per-32 activations: sixteen) keeps upr * R * TERMS floats
// per token for the ordered sum; where a row has an odd number of blocks the tiles are one block wide and 64 rows
// high, and a long row (Llama-2-7B's 11008 inputs: 43 blocks, 176 KB) no longer fits a workgroup's LDS.  In such
// tiles a lane owns its row's block of every column tile, so a workgroup of ONE wave that walks the column tiles in
// order can add the terms up as they come, in the row's order, and needs one float per token and lane.
template <class F, bool GEMM_ORDER>
static bool gemv_lane_acc(uint32_t in_dim) {
  if (F::TERMS <= 1 || n_term_arrays<F, GEMM_ORDER>() != 1) return false;
  const OgmTiling tl = ogm_tiling_for(in_dim / F::ELEMS, 1);
  return tl.C == 1 && gemv_lds_bytes<F, GEMM_ORDER>(in_dim, 1) > OGM_LDS_BUDGET;
}
template <class F>
static size_t gemv_lds_bytes_lane_acc(uint32_t in_dim, uint32_t n_tokens) {
  const size_t upr = in_dim / F::ELEMS, n_scale = in_dim / F::ACT_GROUP;
  size_t b = (size_t)n_tokens * in_dim + (size_t)n_tokens * upr * F::AUX16 * 16 + (size_t)n_tokens * n_scale * 4;
  b = (b + 15) & ~(size_t)15;
  return b + (size_t)n_tokens * 64 * 4;
}

#define OGM_STAGE_PEEL 4

// acc (+|-)= p[0], p[stride], ... in ascending order, one accumulator.  Eight LDS reads are in
// flight and the next eight are requested before these are added: the adds are a serial chain
// either way, the reads' latency need not be.
template <bool NEGATE>
__device__ __forceinline__ float ordered_sum(float acc, const float *p, uint32_t n, uint32_t stride) {
  uint32_t s = 0;
  if (n >= 8) {
    float a[8];
#pragma unroll
    for (int j = 0; j < 8; j++) a[j] = p[j * stride];
    for (s = 8; s + 8 <= n; s += 8) {
      float b[8];
#pragma unroll
      for (int j = 0; j < 8; j++) b[j] = p[(s + j) * stride];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        if (NEGATE) acc -= a[j];
        else acc += a[j];
      }
#pragma unroll
      for (int j = 0; j < 8; j++) a[j] = b[j];
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
      if (NEGATE) acc -= a[j];
      else acc += a[j];
    }
  }
  for (; s < n; s++) {
    if (NEGATE) acc -= p[s * stride];
    else acc += p[s * stride];
  }
  return acc;
}

struct NoUnpack {};
template <class F, bool WANT, bool HAS = F::HAS_UNPACK>
struct UnpackedOf { typedef NoUnpack type; };
template <class F>
struct UnpackedOf<F, true, true> { typedef typename F::Unpacked type; };

// UPR: blocks per row when known at compile time (the hot shapes), 0 = read it from the params.
// UNPACK: several tokens and a format whose block is expensive to unpack: unpack once per tile.
template <class F, int UPR, bool SINGLE, bool GEMM_ORDER, bool DUMP, bool UNPACK = false>
__global__ __launch_bounds__((SINGLE && !DUMP) ? F::MAX_THREADS_SINGLE : F::MAX_THREADS) void ogm_gemv_kernel(GemvParams p) {
  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t tid = threadIdx.x, nthr = blockDim.x;
  const uint32_t lane = tid & 63u, wave = tid >> 6, n_wave = nthr >> 6;
  const uint32_t T = SINGLE ? 1u : p.n_tokens;
  const uint32_t upr = UPR ? (uint32_t)UPR : p.upr;
  const uint32_t C = UPR ? ((UPR % 4 == 0) ? 4u : ((UPR % 2 == 0) ? 2u : 1u)) : p.C;   // (the UPR variants: 16, 56, 128)
  const uint32_t R = 64u / C, nct = UPR ? upr / C : p.nct;
  const uint32_t xch = upr * F::XPIECES;           // 16-byte chunks of q per token
  const uint32_t n_scale = upr * (F::ELEMS / F::ACT_GROUP);
  const uint32_t term_stride = upr * R * F::TERMS;  // floats per token in the term table
  constexpr int NT = n_term_arrays<F, GEMM_ORDER>();

  uint4 *l_xq = (uint4 *)lds;                                   // [T][xch]
  uint4 *l_aux = l_xq + (size_t)T * xch;                        // [T][AUX16][upr]
  float *l_d = (float *)(l_aux + (size_t)T * upr * F::AUX16);   // [T][n_scale]
  const size_t head = ((size_t)T * (xch * 16 + upr * F::AUX16 * 16 + n_scale * 4) + 15) & ~(size_t)15;
  float *l_term = (float *)(lds + head);                        // [NT][T][upr][R]

  // ---- which matrix of the launch this workgroup belongs to, and which of its row blocks
  const uint32_t bid = blockIdx.x;
  uint32_t m = 0;
  if (bid >= p.wg_end[0]) m = 1;
  if (bid >= p.wg_end[1]) m = 2;
  if (bid >= p.wg_end[2]) m = 3;
  const uint32_t rb0 = bid - (m == 0 ? 0u : m == 1 ? p.wg_end[0] : m == 2 ? p.wg_end[1] : p.wg_end[2]);
  const uint8_t *wt = m == 0 ? p.wt[0] : m == 1 ? p.wt[1] : m == 2 ? p.wt[2] : p.wt[3];
  float *y = m == 0 ? p.y[0] : m == 1 ? p.y[1] : m == 2 ? p.y[2] : p.y[3];
  const uint32_t out_dim = m == 0 ? p.out_dim[0] : m == 1 ? p.out_dim[1] : m == 2 ? p.out_dim[2] : p.out_dim[3];
  // The row block's tiles are consecutive in memory: item i is tile rb0 * nct + i, column tile i.
  const uint32_t n_items = nct;
  const size_t tile0 = (size_t)rb0 * nct;

  // ---- issue the activation loads (few, L2-resident) ...
  const uint32_t n_xq = T * xch, n_aux = T * upr * F::AUX16, n_d = T * n_scale;
  const uint4 *gq = (const uint4 *)p.act.q;
  uint4 st0, st1, st2, st3, st_aux = make_uint4(0, 0, 0, 0);
  float st_d = 0.0f;
  auto ld_bsum = [&](uint32_t i) -> uint4 {   // Q4_K: bsum, 8 x i16 per block
    return ((const uint4 *)p.act.bsum)[i];
  };
  auto ld_sums16 = [&](uint32_t i) -> uint4 {   // Q6_K: per-16 sums narrowed to i16, groups 0..7 / 8..15 of a block
    const int4 *src = (const int4 *)(p.act.sums + (size_t)(i >> 1) * 16 + (i & 1u) * 8);
    const int4 a = src[0], b = src[1];
    uint4 o;
    o.x = ((uint32_t)a.x & 0xFFFFu) | ((uint32_t)a.y << 16);
    o.y = ((uint32_t)a.z & 0xFFFFu) | ((uint32_t)a.w << 16);
    o.z = ((uint32_t)b.x & 0xFFFFu) | ((uint32_t)b.y << 16);
    o.w = ((uint32_t)b.z & 0xFFFFu) | ((uint32_t)b.w << 16);
    return o;
  };
  st0 = gq[min(tid, n_xq - 1)];
  st1 = gq[min(tid + nthr, n_xq - 1)];
  st2 = gq[min(tid + 2 * nthr, n_xq - 1)];
  st3 = gq[min(tid + 3 * nthr, n_xq - 1)];
  if (F::AUX16 == 1) st_aux = ld_bsum(min(tid, n_aux - 1));
  else if (F::AUX16 == 2) st_aux = ld_sums16(min(tid, n_aux - 1));
  st_d = p.act.d[min(tid, n_d - 1)];

  // Keeps every staging load of the workgroup ahead of every weight load in the CU's
  // memory pipeline (no data is waited for here).
  __syncthreads();

  // ---- ... then this wave's first tile of weights (the long pole) ...
  const uint32_t r_local = lane & (R - 1), c_local = lane / R;
  uint32_t it = wave;  // every wave has at least one item: n_wave <= nct
  typename F::Regs cur;
  F::load(cur, wt, tile0 + it, lane);
  // Nothing below may be scheduled above the weight loads: work on the activations would
  // otherwise wait for them first and hold the weight loads back by a memory round trip.
  __builtin_amdgcn_sched_barrier(0);

  // ---- ... and park the activations in LDS while the weights are in flight.
  // q is permuted so that chunk c of block `col` lands at [c*upr + col].
  {
    auto park = [&](uint32_t i, const uint4 &v) {
      if (i < n_xq) {
        const uint32_t t = i / xch, ch = i - t * xch;
        const uint32_t col = ch / F::XPIECES, c = ch - col * F::XPIECES;
        l_xq[(size_t)t * xch + c * upr + col] = v;
      }
    };
    park(tid, st0);
    park(tid + nthr, st1);
    park(tid + 2 * nthr, st2);
    park(tid + 3 * nthr, st3);
    if (F::AUX16 == 1) {
      if (tid < n_aux) l_aux[tid] = st_aux;
    } else if (F::AUX16 == 2) {
      if (tid < n_aux) {
        const uint32_t blk = tid >> 1, k = tid & 1u;
        const uint32_t t = blk / upr, col = blk - t * upr;
        l_aux[(size_t)t * upr * 2 + k * upr + col] = st_aux;
      }
    }
    if (tid < n_d) l_d[tid] = st_d;
    // Whatever the peeled loads did not cover (many tokens, or very long rows).
    for (uint32_t i = tid + OGM_STAGE_PEEL * nthr; i < n_xq; i += nthr) {
      const uint32_t t = i / xch, ch = i - t * xch;
      const uint32_t col = ch / F::XPIECES, c = ch - col * F::XPIECES;
      l_xq[(size_t)t * xch + c * upr + col] = gq[i];
    }
    if (F::AUX16 == 1) {
      for (uint32_t i = tid + nthr; i < n_aux; i += nthr) l_aux[i] = ld_bsum(i);
    } else if (F::AUX16 == 2) {
      for (uint32_t i = tid + nthr; i < n_aux; i += nthr) {
        const uint32_t blk = i >> 1, k = i & 1u;
        const uint32_t t = blk / upr, col = blk - t * upr;
        l_aux[(size_t)t * upr * 2 + k * upr + col] = ld_sums16(i);
      }
    }
    for (uint32_t i = tid + nthr; i < n_d; i += nthr) l_d[i] = p.act.d[i];
  }
  __syncthreads();

  if constexpr (F::TERMS > 1) {
    if (p.lane_acc)   // one wave: its lanes' running sums, one per token
      for (uint32_t t = 0; t < T; t++) l_term[t * 64u + lane] = 0.0f;
  }
  // ---- tiles of this wave
  for (; it < n_items; it += n_wave) {
    // block index within the row; a lane of a padded column tile past the row's last block works on that block
    // again (its own unit is zeros) and leaves nothing behind
    const uint32_t col_own = it * C + c_local;
    const bool live = col_own < upr;
    const uint32_t col = live ? col_own : upr - 1u;
    // many tokens: unpack the block once where that is the expensive part (Q6_K; measured at
    // 4096 -> 128256: 159 us against 182 us at 8 tokens, but 112 us against 97 us at 4)
    [[maybe_unused]] typename UnpackedOf<F, UNPACK>::type unp;
    if constexpr (UNPACK) F::unpack(cur, unp);
    for (uint32_t t = 0; t < T; t++) {
      ActLds a;
      a.xq = l_xq + (size_t)t * xch;
      a.aux = l_aux + (size_t)t * upr * F::AUX16;
      a.d = l_d + (size_t)t * n_scale;
      a.upr = upr;
      int isum, imin;
      if constexpr (UNPACK) F::template sums_unpacked<UPR>(unp, cur, a, col, isum, imin);
      else F::template sums<UPR>(cur, a, col, isum, imin);
      if constexpr (F::TERMS > 1) {
        // a block leaves several terms, in the order the row adds them
        float tt[F::TERMS];
        F::template terms<UPR>(cur, a, col, tt);
        if (!live) continue;
        if (p.lane_acc) {   // this lane's row, the column tiles in order: the row's own sequence of additions
          float acc = l_term[t * 64u + lane];
#pragma unroll
          for (int g = 0; g < F::TERMS; g++) acc += tt[g];
          l_term[t * 64u + lane] = acc;
          continue;
        }
        float *dst = l_term + (size_t)t * term_stride + (size_t)col * F::TERMS * R + r_local;
#pragma unroll
        for (int g = 0; g < F::TERMS; g++) dst[g * R] = tt[g];
        continue;
      }
      if (!live) continue;
      const float ad = a.d[col];  // one activation scale per block (per-32 and per-256 alike)
      const size_t slot = (size_t)t * term_stride + col * R + r_local;
      if (GEMM_ORDER) {
        float tmin, tdot;
        F::term_gemm(cur, ad, isum, imin, tmin, tdot);
        l_term[slot] = tdot;
        if (NT == 2) l_term[(size_t)T * term_stride + slot] = tmin;
      } else {
        l_term[slot] = F::term_gemv(cur, ad, isum, imin);
      }
      if (DUMP) {
        const uint32_t row = rb0 * R + r_local;
        if (row < out_dim) {
          const size_t o = ((size_t)t * out_dim + row) * upr + col;
          if (p.dump_isum) p.dump_isum[o] = isum;
          if (F::HAS_MIN && p.dump_imin) p.dump_imin[o] = imin;
        }
      }
    }
    if (it + n_wave < n_items) F::load(cur, wt, tile0 + it + n_wave, lane);
  }
  __syncthreads();

  if constexpr (F::TERMS > 1) {
    if (p.lane_acc) {
      const uint32_t orow = rb0 * R + lane;
      if (orow < out_dim)
        for (uint32_t t = 0; t < T; t++) y[(size_t)t * out_dim + orow] = l_term[t * 64u + lane];
      return;
    }
  }
  // One lane per (token, row): the row's block terms in ascending order, one accumulator.
  for (uint32_t i = tid; i < R * T; i += nthr) {
    const uint32_t t = i / R, r = i - t * R;
    const uint32_t orow = rb0 * R + r;
    if (orow < out_dim) {
      const float *terms = l_term + (size_t)t * term_stride + r;
      float acc = 0.0f;
      if (NT == 2) acc = ordered_sum<true>(acc, terms + (size_t)T * term_stride, upr, R);
      acc = ordered_sum<false>(acc, terms, upr * F::TERMS, R);
      y[(size_t)t * out_dim + orow] = acc;
    }
  }
}

// ------------------------------------------------------------------------------------------
// host side of the launch


template <class F, bool GEMM_ORDER>
static uint32_t max_tokens_t(uint32_t in_dim) {
  uint32_t t = 8;
  if (gemv_lane_acc<F, GEMM_ORDER>(in_dim)) {
    while (t > 1 && gemv_lds_bytes_lane_acc<F>(in_dim, t) > OGM_LDS_BUDGET) t--;
    return t;
  }
  while (t > 1 && gemv_lds_bytes<F, GEMM_ORDER>(in_dim, t) > OGM_LDS_BUDGET) t--;
  return t;
}

uint32_t ogm_gemv_max_tokens(uint32_t ggml_type, uint32_t in_dim, int gemm_order) {
  switch (ggml_type) {
    case OGM_Q4_K:
      return gemm_order ? max_tokens_t<FmtQ4K, true>(in_dim) : max_tokens_t<FmtQ4K, false>(in_dim);
    case OGM_Q5_K:
      return gemm_order ? max_tokens_t<FmtQ5K, true>(in_dim) : max_tokens_t<FmtQ5K, false>(in_dim);
    case OGM_Q3_K:
      return gemm_order ? max_tokens_t<FmtQ3K, true>(in_dim) : max_tokens_t<FmtQ3K, false>(in_dim);
    case OGM_Q6_K:
      return gemm_order ? max_tokens_t<FmtQ6K, true>(in_dim) : max_tokens_t<FmtQ6K, false>(in_dim);
    case OGM_Q8_0:
      return gemm_order ? max_tokens_t<FmtQ80, true>(in_dim) : max_tokens_t<FmtQ80, false>(in_dim);
    case OGM_Q4_0:
      return gemm_order ? max_tokens_t<FmtQ40, true>(in_dim) : max_tokens_t<FmtQ40, false>(in_dim);
    case OGM_Q5_0:
      return gemm_order ? max_tokens_t<FmtQ50, true>(in_dim) : max_tokens_t<FmtQ50, false>(in_dim);
    case OGM_IQ4_NL:
      return gemm_order ? max_tokens_t<FmtIQ4NL, true>(in_dim) : max_tokens_t<FmtIQ4NL, false>(in_dim);
    case OGM_Q5_1:
      return gemm_order ? max_tokens_t<FmtQ51, true>(in_dim) : max_tokens_t<FmtQ51, false>(in_dim);
    case OGM_IQ4_XS:
      return gemm_order ? max_tokens_t<FmtIQ4XS, true>(in_dim) : max_tokens_t<FmtIQ4XS, false>(in_dim);
    case OGM_Q2_K:
      return gemm_order ? max_tokens_t<FmtQ2KGen, true>(in_dim) : max_tokens_t<FmtQ2K, false>(in_dim);
    default:
      return 0;
  }
}

// Waves per workgroup: a wave takes every waves-th tile of the row block.  Up to 8 (16 for the small tiles of the
// per-32 formats): the count that divides the tile count where one exists in the upper half of that range
// (measured on MI355X: 4 waves x 1 tile at 4096 -> 14336, 7 waves x 2 tiles at 14336 -> 4096 beat 14 x 1), else the
// fewest waves that give the shortest chain of tiles per wave -- a row of 43 blocks (11008 inputs) has no divisor
// but 1, and one wave walking 43 tiles took 52 us where eight take a fraction of that.
static uint32_t pick_waves(uint32_t nct, uint32_t wg_waves, int max_threads, uint32_t auto_cap = 8) {
  uint32_t waves = wg_waves;
  if (waves == 0) {
    const uint32_t cap = auto_cap < nct ? auto_cap : nct;
    waves = 0;
    for (uint32_t w = cap; w >= 1u && 2u * w > cap; w--)
      if (nct % w == 0) {
        waves = w;
        break;
      }
    if (waves == 0) {
      const uint32_t chain = (nct + cap - 1u) / cap;
      waves = (nct + chain - 1u) / chain;
    }
  }
  if (waves > nct) waves = nct;
  if (waves > (uint32_t)max_threads / 64) waves = max_threads / 64;
  if (waves == 0) waves = 1;
  return waves;
}

template <class F>
static void launch_single(const GemvParams &p, dim3 g, dim3 b, size_t lds, hipStream_t stream) {
  // single-token decode: the hot shapes get their row length as a compile-time constant
  if (F::ELEMS == 256 && p.upr == 16)
    hipLaunchKernelGGL((ogm_gemv_kernel<F, 16, true, false, false>), g, b, lds, stream, p);
  else if (F::ELEMS == 256 && p.upr == 56)
    hipLaunchKernelGGL((ogm_gemv_kernel<F, 56, true, false, false>), g, b, lds, stream, p);
  else if (F::ELEMS == 32 && p.upr == 128)
    hipLaunchKernelGGL((ogm_gemv_kernel<F, 128, true, false, false>), g, b, lds, stream, p);
  else {
    // (a long row of an odd number of blocks -- 64-row tiles one block wide -- stages more than a launch gets unasked)
    if (lds > OGM_LDS_UNASKED &&
        hipFuncSetAttribute((const void *)ogm_gemv_kernel<F, 0, true, false, false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return;   // the launch below then fails and reports it
    hipLaunchKernelGGL((ogm_gemv_kernel<F, 0, true, false, false>), g, b, lds, stream, p);
  }
}

template <class F, bool GEMM_ORDER>
static hipError_t launch_t(const OgmGemvArgs &a, hipStream_t stream) {
  const bool dump = a.dump_isum || a.dump_imin;
  if (a.n_extra > OGM_GEMV_MAX_MATS - 1 || (dump && a.n_extra)) return hipErrorInvalidValue;
  GemvParams p;
  p.act = a.act;
  p.dump_isum = a.dump_isum;
  p.dump_imin = a.dump_imin;
  p.in_dim = a.in_dim;
  p.upr = a.in_dim / F::ELEMS;
  p.n_tokens = a.n_tokens;
  const OgmTiling tl = ogm_tiling_for(p.upr, a.out_dim);
  p.C = tl.C;
  p.nct = tl.nct;
  // One row block per workgroup: the measured optimum on MI355X at every shape tried (4096 -> 14336 x2: 2, 4 and 8
  // row blocks a workgroup cost 7 %, 25 % and 60 % more time): many small workgroups keep more loads in flight
  // than the shared activation staging saves.
  uint32_t n_wg = 0;
  for (uint32_t m = 0; m < OGM_GEMV_MAX_MATS; m++) {
    if (m <= a.n_extra) {
      p.wt[m] = m ? a.extra_wt[m - 1] : a.wt;
      p.y[m] = m ? a.extra_y[m - 1] : a.y;
      p.out_dim[m] = m ? a.extra_out_dim[m - 1] : a.out_dim;
      n_wg += (p.out_dim[m] + tl.R - 1) / tl.R;
    } else {
      p.wt[m] = nullptr;
      p.y[m] = nullptr;
      p.out_dim[m] = 0;
    }
    p.wg_end[m] = n_wg;
  }
  if (n_wg == 0) return hipSuccess;
  // (rows of many blocks in a format that leaves sixteen terms a block -- Q2_K over per-32 activations at
  // 14336 inputs: 74 KB for one token -- go beyond the budget; they get what they need, up to the hardware's limit)
  const bool lane_acc = gemv_lane_acc<F, GEMM_ORDER>(a.in_dim) && !dump;
  p.lane_acc = lane_acc ? 1u : 0u;
  const size_t lds = lane_acc ? gemv_lds_bytes_lane_acc<F>(a.in_dim, a.n_tokens) : gemv_lds_bytes<F, GEMM_ORDER>(a.in_dim, a.n_tokens);
  if (lds > OGM_LDS_MAX) return hipErrorInvalidValue;
  auto launch = [&](void (*kernel)(GemvParams), dim3 g_, dim3 b_) -> hipError_t {
    if (lds > OGM_LDS_UNASKED) {
      const hipError_t e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, g_, b_, lds, stream, p);
    return hipGetLastError();
  };
  // the plain single-token kernels of most formats need well under 128 registers and are built for up
  // to sixteen waves
  const bool plain_single = a.n_tokens == 1 && !GEMM_ORDER && !dump;
  // the per-32 formats' tiles are small (2 KB of Q8_0): sixteen of them per workgroup measure 7 %
  // faster than eight at 4096 x 4096
  const uint32_t waves = lane_acc ? 1u
                                  : pick_waves(tl.nct, a.wg_waves, plain_single ? F::MAX_THREADS_SINGLE : F::MAX_THREADS,
                                               (plain_single && F::ELEMS == 32) ? 16u : 8u);
  const dim3 g(n_wg), b(waves * 64);
  if (dump) return launch(ogm_gemv_kernel<F, 0, false, GEMM_ORDER, true>, g, b);
  if (a.n_tokens == 1 && !GEMM_ORDER) {
    launch_single<F>(p, g, b, lds, stream);
    return hipGetLastError();
  }
  if (F::HAS_UNPACK && a.n_tokens >= 6) return launch(ogm_gemv_kernel<F, 0, false, GEMM_ORDER, false, F::HAS_UNPACK>, g, b);
  return launch(ogm_gemv_kernel<F, 0, false, GEMM_ORDER, false>, g, b);
}

hipError_t ogm_launch_gemv(const OgmGemvArgs &a, hipStream_t stream, const char **kernel_name) {
  if (a.n_tokens == 0) return hipSuccess;
  switch (a.ggml_type) {
    case OGM_Q4_K:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ4K,gemm>" : "ogm_gemv_kernel<FmtQ4K,gemv>";
      return a.gemm_order ? launch_t<FmtQ4K, true>(a, stream) : launch_t<FmtQ4K, false>(a, stream);
    case OGM_Q5_K:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ5K,gemm>" : "ogm_gemv_kernel<FmtQ5K,gemv>";
      return a.gemm_order ? launch_t<FmtQ5K, true>(a, stream) : launch_t<FmtQ5K, false>(a, stream);
    case OGM_Q3_K:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ3K,gemm>" : "ogm_gemv_kernel<FmtQ3K,gemv>";
      return a.gemm_order ? launch_t<FmtQ3K, true>(a, stream) : launch_t<FmtQ3K, false>(a, stream);
    case OGM_Q6_K:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ6K,gemm>" : "ogm_gemv_kernel<FmtQ6K,gemv>";
      return a.gemm_order ? launch_t<FmtQ6K, true>(a, stream) : launch_t<FmtQ6K, false>(a, stream);
    case OGM_Q8_0:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ80,gemm>" : "ogm_gemv_kernel<FmtQ80,gemv>";
      return a.gemm_order ? launch_t<FmtQ80, true>(a, stream) : launch_t<FmtQ80, false>(a, stream);
    case OGM_Q4_0:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ40,gemm>" : "ogm_gemv_kernel<FmtQ40,gemv>";
      return a.gemm_order ? launch_t<FmtQ40, true>(a, stream) : launch_t<FmtQ40, false>(a, stream);
    case OGM_Q5_0:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ50,gemm>" : "ogm_gemv_kernel<FmtQ50,gemv>";
      return a.gemm_order ? launch_t<FmtQ50, true>(a, stream) : launch_t<FmtQ50, false>(a, stream);
    case OGM_IQ4_NL:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtIQ4NL,gemm>" : "ogm_gemv_kernel<FmtIQ4NL,gemv>";
      return a.gemm_order ? launch_t<FmtIQ4NL, true>(a, stream) : launch_t<FmtIQ4NL, false>(a, stream);
    case OGM_Q5_1:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ51,gemm>" : "ogm_gemv_kernel<FmtQ51,gemv>";
      return a.gemm_order ? launch_t<FmtQ51, true>(a, stream) : launch_t<FmtQ51, false>(a, stream);
    case OGM_IQ4_XS:
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtIQ4XS,gemm>" : "ogm_gemv_kernel<FmtIQ4XS,gemv>";
      return a.gemm_order ? launch_t<FmtIQ4XS, true>(a, stream) : launch_t<FmtIQ4XS, false>(a, stream);
    case OGM_Q2_K:
      // matmul of several tokens: the rows-unpacked-once arithmetic over per-32 activations; everything
      // else (one token, matmul_decode): per-256 activations
      if (kernel_name) *kernel_name = a.gemm_order ? "ogm_gemv_kernel<FmtQ2KGen,gemm>" : "ogm_gemv_kernel<FmtQ2K,gemv>";
      if (a.gemm_order) return (a.dump_isum || a.dump_imin) ? hipErrorInvalidValue : launch_t<FmtQ2KGen, true>(a, stream);
      return launch_t<FmtQ2K, false>(a, stream);
    default:
      return hipErrorInvalidValue;
  }
}

// ------------------------------------------------------------------------------------------
// f16 -> f32 as the kernels do it, exposed for a parity check

__global__ void ogm_f16_kernel(const uint16_t *bits, size_t n, float *out) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = f16_bits_to_f32(bits[i]);
}

// A launch that only reads: every wave pulls 9 KiB (nine non-temporal 16-byte loads a lane, the
// shape of a Q4_K tile) and folds them into a word nobody stores.  What the memory system delivers
// for a given footprint with no arithmetic, LDS or ordered sum behind the loads: the yardstick the
// benchmark prices the GEMV against.
struct ReadProbeParams {
  const uint8_t *buf[OGM_PROBE_MAX_BUFS];
  uint64_t chunks[OGM_PROBE_MAX_BUFS];   // 9 KiB chunks of each buffer (the last may overlap the one before)
  uint64_t bytes[OGM_PROBE_MAX_BUFS];
  uint32_t n;
  uint32_t *sink;
};
__global__ __launch_bounds__(512) void ogm_read_probe_kernel(ReadProbeParams p) {
  const uint32_t lane = threadIdx.x & 63u;
  uint64_t c = (uint64_t)blockIdx.x * 8u + (threadIdx.x >> 6);
  uint32_t b = 0;
  while (b < p.n && c >= p.chunks[b]) c -= p.chunks[b++];
  if (b == p.n) return;
  // the last chunk of a buffer that is not a multiple of 9 KiB long starts early enough to end with it
  const uint64_t off = min(c * 9216u, p.bytes[b] - 9216u);
  const uint8_t *src = p.buf[b] + off + lane * 16u;
  uint4 r[9];
#pragma unroll
  for (int i = 0; i < 9; i++) r[i] = ldw16(src + i * 1024);
  uint32_t acc = 0;
#pragma unroll
  for (int i = 0; i < 9; i++) acc ^= r[i].x ^ r[i].y ^ r[i].z ^ r[i].w;
  if (acc == 0x9E3779B9u) p.sink[blockIdx.x & 63u] = acc;   // practically never: keeps the loads alive
}

hipError_t ogm_launch_read_probe(const uint8_t *const *bufs, const size_t *bytes, uint32_t n, uint32_t *sink,
                                 hipStream_t stream) {
  if (n == 0 || n > OGM_PROBE_MAX_BUFS) return hipErrorInvalidValue;
  ReadProbeParams p = {};
  uint64_t total = 0;
  for (uint32_t i = 0; i < n; i++) {
    if (bytes[i] < 9216u || ((uintptr_t)bufs[i] & 15u)) return hipErrorInvalidValue;
    p.buf[i] = bufs[i];
    p.bytes[i] = bytes[i];
    p.chunks[i] = (bytes[i] + 9215u) / 9216u;
    total += p.chunks[i];
  }
  p.n = n;
  p.sink = sink;
  const uint64_t wgs = (total + 7u) / 8u;
  if (wgs > 0x7FFFFFFFull) return hipErrorInvalidValue;
  hipLaunchKernelGGL(ogm_read_probe_kernel, dim3((unsigned)wgs), dim3(512), 0, stream, p);
  return hipGetLastError();
}

// A launch of `workgroups` workgroups of 256 threads that does nothing (one pointer and one word of
// arguments, like a real kernel): what a kernel boundary costs behind a launch of a given width.
__global__ __launch_bounds__(256) void ogm_empty_kernel(uint32_t *sink, uint32_t never) {
  if (never == 0x9E3779B9u && threadIdx.x == 0) sink[blockIdx.x & 63u] = never;
}

hipError_t ogm_launch_empty(uint32_t workgroups, uint32_t *sink, hipStream_t stream) {
  if (workgroups == 0 || workgroups > 0x7FFFFFFFu || !sink) return hipErrorInvalidValue;
  hipLaunchKernelGGL(ogm_empty_kernel, dim3(workgroups), dim3(256), 0, stream, sink, 0u);
  return hipGetLastError();
}

hipError_t ogm_launch_f16_to_f32(const uint16_t *bits, size_t n, float *out, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(ogm_f16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, bits,
                     n, out);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// A word in pinned host memory that tells a polling host thread that everything enqueued on the stream
// before this launch has finished: a kernel starts only after its predecessors on the stream have completed
// and their stores have been acknowledged, and the store below goes out at system scope behind a fence.
__global__ __launch_bounds__(64) void ogm_host_flag_kernel(uint32_t *flag, uint32_t value) {
  if (threadIdx.x == 0) {
    __threadfence_system();
    __hip_atomic_store(flag, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

hipError_t ogm_launch_host_flag(uint32_t *flag, uint32_t value, hipStream_t stream) {
  if (!flag) return hipErrorInvalidValue;
  hipLaunchKernelGGL(ogm_host_flag_kernel, dim3(1), dim3(64), 0, stream, flag, value);
  return hipGetLastError();
}
