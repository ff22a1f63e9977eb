// Device-side core of the activation quantizer, shared by every kernel that quantizes
// (the standalone quantizer, the GEMV's optional prologue and the decode step's fused
// norm / attention-combine / SwiGLU kernels), so that all of them produce the same bits.
//
//   amax  = fold(0, max(m, |v|)) ignoring NaN            (vecdot.rs:103, 3037)
//   scale = amax / 127 ; inv = scale > 0 ? 1/scale : 0   (vecdot.rs:106-107)
//   q     = clamp(round_half_away(v * inv), -127, 127), NaN -> 0   (vecdot.rs:117)
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ogm_kernels.h"

__device__ __forceinline__ float ogm_nan_blind_max(float m, float a) { return a > m ? a : m; }

// One step of a butterfly all-reduce over the wave: joins groups of M lanes pairwise with a commutative
// `op`.  For a value that is already equal within each group of M lanes (the state of a butterfly after its
// steps 1 .. M / 2) any lane of the partner group serves, which lets the steps stay in the vector pipe --
// quad permutes, the row mirrors, and gfx950's swaps of 16- and 32-lane halves -- instead of going through
// LDS addressing (ds_bpermute) sixty-odd clocks at a time.  Same pairs as `v op shfl_xor(v, M)`: same bits.
template <int M, class Op>
__device__ __forceinline__ float ogm_butterfly_step(float v, Op op) {
  typedef unsigned ogm_u2 __attribute__((ext_vector_type(2)));
  if constexpr (M == 1) {
    return op(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true)));   // quad_perm 1,0,3,2
  } else if constexpr (M == 2) {
    return op(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true)));   // quad_perm 2,3,0,1
  } else if constexpr (M == 4) {
    return op(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true)));  // row_half_mirror
  } else if constexpr (M == 8) {
    return op(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true)));  // row_mirror
  } else if constexpr (M == 16) {
    const ogm_u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return op(__uint_as_float(r.x), __uint_as_float(r.y));   // every lane: its pair of rows' two values
  } else {
    static_assert(M == 32, "a wave has 64 lanes");
    const ogm_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return op(__uint_as_float(r.x), __uint_as_float(r.y));
  }
}
template <int M>
__device__ __forceinline__ int ogm_butterfly_add_i32(int v) {
  static_assert(M == 1 || M == 2 || M == 4, "the quantizer's sums stop at eight lanes");
  constexpr int CTRL = M == 1 ? 0xB1 : M == 2 ? 0x4E : 0x141;
  return v + __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
// The value lane ^ M holds, for M = 1 or 2 (any values: a quad permute is a true exchange).
template <int M>
__device__ __forceinline__ float ogm_quad_xor(float v) {
  static_assert(M == 1 || M == 2, "within a quad");
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), M == 1 ? 0xB1 : 0x4E, 0xF, 0xF, true));
}
// The value lane ^ M holds, for M = 16 or 32 (any values: the half swaps exchange lanes at equal positions);
// upper = whether this lane has bit M set.
template <int M>
__device__ __forceinline__ float ogm_half_xor(float v, bool upper) {
  typedef unsigned ogm_u2 __attribute__((ext_vector_type(2)));
  static_assert(M == 16 || M == 32, "rows of 16 or halves of 32");
  ogm_u2 r;
  if constexpr (M == 16) r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  else r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(upper ? r.x : r.y);
}
// op over the four quads of a row of 16 lanes, lane by lane of the quads (values may differ within a quad):
// two rotations of the row.  Quad 0 ends with (q0 op q1) op (q2 op q3), the butterfly's order.
template <class Op>
__device__ __forceinline__ float ogm_row_quads_allreduce(float v, Op op) {
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x12C, 0xF, 0xF, true)));   // row_ror:12 = from lane + 4
  return op(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true)));   // row_ror:8
}
struct OgmOpMax { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct OgmOpAdd { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };
struct OgmOpNanBlindMax { __device__ __forceinline__ float operator()(float a, float b) const { return ogm_nan_blind_max(a, b); } };
// v summed over the wave, in the butterfly's order: ((lane + lane^1) + ...) level by level
__device__ __forceinline__ float ogm_wave_sum(float v) {
  v = ogm_butterfly_step<1>(v, OgmOpAdd());
  v = ogm_butterfly_step<2>(v, OgmOpAdd());
  v = ogm_butterfly_step<4>(v, OgmOpAdd());
  v = ogm_butterfly_step<8>(v, OgmOpAdd());
  v = ogm_butterfly_step<16>(v, OgmOpAdd());
  return ogm_butterfly_step<32>(v, OgmOpAdd());
}

__device__ __forceinline__ int ogm_quantize_one(float v, float inv) {
  float r = roundf(v * inv);
  if (r != r) r = 0.0f;
  r = fminf(fmaxf(r, -127.0f), 127.0f);
  return (int)r;
}

// Quantizes the four values a lane holds (elements 4*lane .. 4*lane+3 of a run of 256 spread
// over the wave).  GROUP = 32: one scale per 8 lanes; GROUP = 256: one per wave.  Every lane of
// the wave must call it.  Returns the four int8 packed little-endian; s16 / s32 are the sums of
// the 16 / 32 quantized values this lane's group of 4 / 8 lanes holds.
template <int GROUP>
__device__ __forceinline__ uint32_t ogm_quantize4(const float4 &v, float &scale, int &s16, int &s32) {
  float amax = 0.0f;
  amax = ogm_nan_blind_max(amax, fabsf(v.x));
  amax = ogm_nan_blind_max(amax, fabsf(v.y));
  amax = ogm_nan_blind_max(amax, fabsf(v.z));
  amax = ogm_nan_blind_max(amax, fabsf(v.w));
  // (no lane's amax is NaN -- the fold starts at 0 and skips them -- so the max commutes)
  amax = ogm_butterfly_step<1>(amax, OgmOpNanBlindMax());
  amax = ogm_butterfly_step<2>(amax, OgmOpNanBlindMax());
  amax = ogm_butterfly_step<4>(amax, OgmOpNanBlindMax());
  if constexpr (GROUP == 256) {
    amax = ogm_butterfly_step<8>(amax, OgmOpNanBlindMax());
    amax = ogm_butterfly_step<16>(amax, OgmOpNanBlindMax());
    amax = ogm_butterfly_step<32>(amax, OgmOpNanBlindMax());
  } else {
    static_assert(GROUP == 32, "groups of 32 or 256");
  }
  scale = amax / 127.0f;
  const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
  const int q0 = ogm_quantize_one(v.x, inv), q1 = ogm_quantize_one(v.y, inv);
  const int q2 = ogm_quantize_one(v.z, inv), q3 = ogm_quantize_one(v.w, inv);
  int s = q0 + q1 + q2 + q3;
  s = ogm_butterfly_add_i32<1>(s);
  s = ogm_butterfly_add_i32<2>(s);
  s16 = s;
  s32 = ogm_butterfly_add_i32<4>(s);
  return (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
         ((uint32_t)(q3 & 0xFF) << 24);
}

// A store that workgroups of the same kernel on other compute dies may read (with a device-coherent
// load) once this wave's stores are acknowledged: it goes through to the level all dies share.
template <bool COHERENT, class T>
__device__ __forceinline__ void ogm_st(T *p, T v) {
  if constexpr (COHERENT) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}

// Quantizes and stores one lane's share of a 256-run whose first element is e0 (= 256*run +
// 4*lane) of token-major activations with row length in_dim; t_off* are the token's offsets.  Returns the
// lane's four quantized values, packed.
// COHERENT_OUT: the stores are for other workgroups of the same kernel (ogm_st).
template <int GROUP, bool COHERENT_OUT = false>
__device__ __forceinline__ uint32_t ogm_quantize_store(const float4 &v, uint32_t e0, bool active, uint32_t lane,
                                                       int8_t *q, float *d, int32_t *sums, int16_t *bsum,
                                                       uint16_t *bs16, int8_t *xt_row = nullptr) {
  float scale;
  int s16, s32;
  const uint32_t packed = ogm_quantize4<GROUP>(v, scale, s16, s32);
  if (active) {
    ogm_st<COHERENT_OUT>((uint32_t *)(q + e0), packed);
    if ((lane & 3u) == 0) ogm_st<COHERENT_OUT>(sums + e0 / 16, (int32_t)s16);
    if ((lane & 7u) == 0) {
      ogm_st<COHERENT_OUT>(bsum + e0 / 32, (int16_t)s32);
      if (GROUP == 256 && bs16 != nullptr) {
        // |s32| <= 32 * 127: floor(s32 / 64) and s32 mod 64 are exact in f16
        uint16_t *b = bs16 + (e0 / 256u) * 16u + ((e0 / 32u) & 7u);
        ogm_st<COHERENT_OUT>(b, __half_as_ushort(__float2half_rn((float)(s32 >> 6))));
        ogm_st<COHERENT_OUT>(b + 8, __half_as_ushort(__float2half_rn((float)(s32 & 63))));
      }
    }
    if ((lane & (GROUP / 4 - 1)) == 0) ogm_st<COHERENT_OUT>(d + e0 / GROUP, scale);
    // the token's place in the operand chunks (ogm_xt_row): chunk e0 / 32, half (e0 / 16) & 1 of its k, byte e0 & 15
    if (xt_row != nullptr) *(uint32_t *)(xt_row + (e0 >> 5) * 1024u + ((e0 >> 4) & 1u) * 512u + (e0 & 15u)) = packed;
  }
  return packed;   // the lane's four int8 values, also for callers that lay them out a second way
}

// Where token t's activations start in the operand chunks of a batch n wide: chunk (t / 32, k / 32) is 1 KiB, the
// 16 activations 16 h .. of its token l at 16 (32 h + l).
__device__ __forceinline__ int8_t *ogm_xt_row(int8_t *xt, uint32_t t, uint32_t n) {
  return xt ? xt + (size_t)(t >> 5) * (n / 32u) * 1024u + (t & 31u) * 16u : nullptr;
}

// The row a workgroup of a row-per-workgroup producer takes when it also writes the operand chunks.  Eight
// consecutive tokens share every 128-byte line of a chunk, and workgroups are dealt to the eight XCDs (each with an
// L2 of its own) in turn: rows in the grid's order would put the eight writers of a line on eight L2s, none of which
// ever holds the whole line.  Within a group of 64 workgroups, workgroup 8 i + x (on XCD x) takes row 8 x + i, so a
// line's writers share an L2 and run within a few workgroups of each other.  (The last, partial group keeps the
// grid's order.)
__device__ __forceinline__ uint32_t ogm_xt_row_of_workgroup(uint32_t b, uint32_t n) {
  if ((b | 63u) >= n) return b;
  return (b & ~63u) | ((b & 7u) << 3) | ((b >> 3) & 7u);
}

// Four floats that another workgroup of the same kernel may have stored device-coherently.
template <bool COHERENT>
__device__ __forceinline__ float4 ogm_ld4(const float *p) {
  if constexpr (COHERENT) {
    const uint64_t a = __hip_atomic_load((const uint64_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t b = __hip_atomic_load((const uint64_t *)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float4(__uint_as_float((uint32_t)a), __uint_as_float((uint32_t)(a >> 32)),
                       __uint_as_float((uint32_t)b), __uint_as_float((uint32_t)(b >> 32)));
  } else {
    return *(const float4 *)p;
  }
}

// Residual add, RMSNorm and quantization of one row by one workgroup of n_wave waves (n <= 1024 *
// n_wave): wave w owns the 256-runs w, w + n_wave, ... (at most four), lane l their elements
// 4l..4l+3, kept in registers between the two passes.  red: 64 floats of LDS.  COHERENT_DELTA:
// delta was written by other workgroups of the calling kernel.  COHERENT_OUT: the quantized row is
// for other workgroups of the calling kernel.  x_src (optional): the row is read from there instead of
// from x, and stored to x.
template <int GROUP, bool COHERENT_DELTA, bool COHERENT_OUT = false>
__device__ __forceinline__ void ogm_norm_quant_row(float *__restrict__ x, const float *__restrict__ delta,
                                                   const float *__restrict__ weight, uint32_t n, float eps,
                                                   float *__restrict__ normed, const OgmActDev &act,
                                                   float *red, uint32_t tid, uint32_t n_wave,
                                                   const float *__restrict__ x_src = nullptr) {
  const uint32_t lane = tid & 63u, wave = tid >> 6;
  float4 v[4], wv[4];
  float ss[4];
  // every load first (x, the residual delta and the norm weights share one trip to memory)
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const uint32_t e0 = (wave + k * n_wave) * 256u + 4u * lane;
    v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    wv[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
    if (e0 < n) {
      v[k] = *(const float4 *)((x_src ? x_src : x) + e0);
      wv[k] = *(const float4 *)(weight + e0);
      if (delta) d = ogm_ld4<COHERENT_DELTA>(delta + e0);
    }
    if (e0 < n && delta) { v[k].x += d.x; v[k].y += d.y; v[k].z += d.z; v[k].w += d.w; }
    if (e0 < n && (delta || x_src)) *(float4 *)(x + e0) = v[k];
    ss[k] = v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
  }
  // one sum per 256-run, then the runs in ascending order: the same value whatever the
  // number of waves
#pragma unroll
  for (int k = 0; k < 4; k++) {
    if ((wave + k * n_wave) * 256u < n) {   // wave-uniform: the run exists
      ss[k] = ogm_wave_sum(ss[k]);
      if (lane == 0) red[wave + k * n_wave] = ss[k];
    }
  }
  __syncthreads();
  float total = 0.0f;
  for (uint32_t r = 0; r * 256u < n; r++) total += red[r];
  const float mean_sq = total / (float)n;
  const float scale = 1.0f / sqrtf(mean_sq + eps);
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const uint32_t e0 = (wave + k * n_wave) * 256u + 4u * lane;
    const bool active = e0 < n;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) {
      o.x = v[k].x * scale * wv[k].x; o.y = v[k].y * scale * wv[k].y;
      o.z = v[k].z * scale * wv[k].z; o.w = v[k].w * scale * wv[k].w;
      if (normed) *(float4 *)(normed + e0) = o;
    }
    if ((wave + k * n_wave) * 256u < n)  // wave-uniform: the run exists
      ogm_quantize_store<GROUP, COHERENT_OUT>(o, e0, active, lane, act.q, act.d, act.sums, act.bsum, act.bs16, act.xt);
  }
}

// SwiGLU and quantization of one 256-run by one wave: h = silu(gate) * up.  COHERENT: gate and up were
// written by other workgroups of the calling kernel; COHERENT_OUT: the quantized run is for them.
template <int GROUP, bool COHERENT, bool COHERENT_OUT = false>
__device__ __forceinline__ void ogm_swiglu_quant_run(const float *__restrict__ gate, const float *__restrict__ up,
                                                     uint32_t n, float *__restrict__ h, const OgmActDev &act,
                                                     uint32_t run, uint32_t lane) {
  const uint32_t e0 = run * 256u + 4u * lane;
  const bool active = e0 < n;
  float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
  if (active) {
    const float4 g = ogm_ld4<COHERENT>(gate + e0), u = ogm_ld4<COHERENT>(up + e0);
    o.x = g.x / (1.0f + expf(-g.x)) * u.x;
    o.y = g.y / (1.0f + expf(-g.y)) * u.y;
    o.z = g.z / (1.0f + expf(-g.z)) * u.z;
    o.w = g.w / (1.0f + expf(-g.w)) * u.w;
    if (h) *(float4 *)(h + e0) = o;
  }
  ogm_quantize_store<GROUP, COHERENT_OUT>(o, e0, active, lane, act.q, act.d, act.sums, act.bsum, act.bs16, act.xt);
}
