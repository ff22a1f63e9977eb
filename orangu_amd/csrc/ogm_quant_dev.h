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

__device__ __forceinline__ float ogm_nan_blind_max(float m, float a) { return a > m ? a : m; }

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
#pragma unroll
  for (int m = 1; m < GROUP / 4; m <<= 1) amax = ogm_nan_blind_max(amax, __shfl_xor(amax, m, 64));
  scale = amax / 127.0f;
  const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
  const int q0 = ogm_quantize_one(v.x, inv), q1 = ogm_quantize_one(v.y, inv);
  const int q2 = ogm_quantize_one(v.z, inv), q3 = ogm_quantize_one(v.w, inv);
  int s = q0 + q1 + q2 + q3;
  s += __shfl_xor(s, 1, 64);
  s += __shfl_xor(s, 2, 64);
  s16 = s;
  s32 = s + __shfl_xor(s, 4, 64);
  return (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
         ((uint32_t)(q3 & 0xFF) << 24);
}

// Quantizes and stores one lane's share of a 256-run whose first element is e0 (= 256*run +
// 4*lane) of token-major activations with row length in_dim; t_off* are the token's offsets.
template <int GROUP>
__device__ __forceinline__ void ogm_quantize_store(const float4 &v, uint32_t e0, bool active, uint32_t lane,
                                                   int8_t *q, float *d, int32_t *sums, int16_t *bsum,
                                                   uint16_t *bs16) {
  float scale;
  int s16, s32;
  const uint32_t packed = ogm_quantize4<GROUP>(v, scale, s16, s32);
  if (active) {
    *(uint32_t *)(q + e0) = packed;
    if ((lane & 3u) == 0) sums[e0 / 16] = s16;
    if ((lane & 7u) == 0) {
      bsum[e0 / 32] = (int16_t)s32;
      if (GROUP == 256 && bs16 != nullptr) {
        // |s32| <= 32 * 127: floor(s32 / 64) and s32 mod 64 are exact in f16
        uint16_t *b = bs16 + (e0 / 256u) * 16u + ((e0 / 32u) & 7u);
        b[0] = __half_as_ushort(__float2half_rn((float)(s32 >> 6)));
        b[8] = __half_as_ushort(__float2half_rn((float)(s32 & 63)));
      }
    }
    if ((lane & (GROUP / 4 - 1)) == 0) d[e0 / GROUP] = scale;
  }
}
