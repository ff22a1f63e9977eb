// gfx950 kernels of the Llama decode step around the quantized matmuls: RMSNorm (with the
// residual add before it), NORM-paired RoPE with the KV-cache write, grouped-query attention
// over an f16 cache, SwiGLU and the greedy argmax (engine/arch/llama.rs:594-932,
// engine/tensor.rs:732-757, 825-827, 1115-1177, engine/attention.rs:426-549 of orangu-server).
//
// Every producer of a matmul input also quantizes it (ogm_quant_dev.h), bit for bit as the
// standalone quantizer would, so a decode step launches no quantizer kernels.  All of these
// kernels are bound by launch latency or by HBM reads of the cache; none has arithmetic worth
// the matrix cores.  Reductions are trees, so f32 results agree with the reference's sequential
// loops to rounding, not to the bit.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "ogm_llama.h"
#include "ogm_quant_dev.h"

// ------------------------------------------------------------------------------------------
// residual add + RMSNorm + quantize

// One workgroup; wave w owns the 256-runs w, w + n_wave, ... (at most four), lane l their
// elements 4l..4l+3, kept in registers between the two passes.
template <int GROUP>
__global__ __launch_bounds__(1024) void ogm_norm_quant_kernel(float *__restrict__ x,
                                                              const float *__restrict__ delta,
                                                              const float *__restrict__ weight, uint32_t n,
                                                              float eps, float *__restrict__ normed,
                                                              OgmActDev act) {
  __shared__ float red[16];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, n_wave = blockDim.x >> 6;
  float4 v[4];
  float ss = 0.0f;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const uint32_t e0 = (wave + k * n_wave) * 256u + 4u * lane;
    v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (e0 < n) {
      v[k] = *(const float4 *)(x + e0);
      if (delta) {
        const float4 d = *(const float4 *)(delta + e0);
        v[k].x += d.x; v[k].y += d.y; v[k].z += d.z; v[k].w += d.w;
        *(float4 *)(x + e0) = v[k];
      }
      ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
    }
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) ss += __shfl_xor(ss, m, 64);
  if (lane == 0) red[wave] = ss;
  __syncthreads();
  float total = 0.0f;
  for (uint32_t w = 0; w < n_wave; w++) total += red[w];
  const float mean_sq = total / (float)n;
  const float scale = 1.0f / sqrtf(mean_sq + eps);
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const uint32_t e0 = (wave + k * n_wave) * 256u + 4u * lane;
    const bool active = e0 < n;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) {
      const float4 w = *(const float4 *)(weight + e0);
      o.x = v[k].x * scale * w.x; o.y = v[k].y * scale * w.y;
      o.z = v[k].z * scale * w.z; o.w = v[k].w * scale * w.w;
      if (normed) *(float4 *)(normed + e0) = o;
    }
    if ((wave + k * n_wave) * 256u < n)  // wave-uniform: the run exists
      ogm_quantize_store<GROUP>(o, e0, active, lane, act.q, act.d, act.sums, act.bsum);
  }
}

hipError_t ogm_launch_norm_quant(int mode, float *x, const float *delta, const float *weight, uint32_t n,
                                 float eps, float *normed, OgmActDev act, hipStream_t stream) {
  if (n == 0 || n % 32u != 0 || n > 16384u) return hipErrorInvalidValue;
  const uint32_t runs = (n + 255u) / 256u;
  const uint32_t waves = runs < 16u ? runs : 16u;
  if (mode == 0)
    hipLaunchKernelGGL(ogm_norm_quant_kernel<32>, dim3(1), dim3(waves * 64), 0, stream, x, delta, weight,
                       n, eps, normed, act);
  else
    hipLaunchKernelGGL(ogm_norm_quant_kernel<256>, dim3(1), dim3(waves * 64), 0, stream, x, delta, weight,
                       n, eps, normed, act);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// RoPE + KV-cache write

__global__ __launch_bounds__(256) void ogm_rope_kv_kernel(float *__restrict__ q, const float *__restrict__ k,
                                                          const float *__restrict__ v,
                                                          const float *__restrict__ freq, uint32_t pos,
                                                          uint32_t n_head, uint32_t n_head_kv, uint32_t head_dim,
                                                          uint32_t rope_dim, __half *__restrict__ kc,
                                                          __half *__restrict__ vc) {
  const uint32_t half_dim = head_dim / 2, rope_half = rope_dim / 2;
  const uint32_t kv_dim = n_head_kv * head_dim;
  const uint32_t nq = n_head * half_dim, nk = n_head_kv * half_dim;
  __half *krow = kc + (size_t)pos * kv_dim, *vrow = vc + (size_t)pos * kv_dim;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < nq + nk; i += gridDim.x * blockDim.x) {
    const bool is_q = i < nq;
    const uint32_t j = is_q ? i : i - nq;
    const uint32_t h = j / half_dim, p = j - h * half_dim;   // pair p of head h: elements 2p, 2p+1
    const float *src = (is_q ? q : k) + h * head_dim + 2u * p;
    float a = src[0], b = src[1];
    if (p < rope_half) {
      const float theta = (float)pos * freq[p];
      float sn, cs;
      sincosf(theta, &sn, &cs);
      const float ra = a * cs - b * sn, rb = a * sn + b * cs;
      a = ra;
      b = rb;
    }
    if (is_q) {
      float *dst = q + h * head_dim + 2u * p;
      dst[0] = a;
      dst[1] = b;
    } else {
      krow[h * head_dim + 2u * p] = __float2half_rn(a);
      krow[h * head_dim + 2u * p + 1u] = __float2half_rn(b);
      vrow[h * head_dim + 2u * p] = __float2half_rn(v[h * head_dim + 2u * p]);
      vrow[h * head_dim + 2u * p + 1u] = __float2half_rn(v[h * head_dim + 2u * p + 1u]);
    }
  }
}

hipError_t ogm_launch_rope_kv(float *q, const float *k, const float *v, const float *freq, uint32_t pos,
                              uint32_t n_head, uint32_t n_head_kv, uint32_t head_dim, uint32_t rope_dim,
                              void *k_cache_layer, void *v_cache_layer, hipStream_t stream) {
  if (head_dim % 2u != 0 || rope_dim > head_dim || rope_dim % 2u != 0) return hipErrorInvalidValue;
  const uint32_t n = (n_head + n_head_kv) * head_dim / 2;
  hipLaunchKernelGGL(ogm_rope_kv_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, q, k, v, freq, pos,
                     n_head, n_head_kv, head_dim, rope_dim, (__half *)k_cache_layer, (__half *)v_cache_layer);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// attention: partial softmax per chunk of positions, then combine (+ quantize)

#define ATT_MAXG 8   // query heads per K/V head

// Workgroup (kvh, split): the query heads of K/V head kvh against positions
// split * 128 .. + 128.  Phase 1: thread t scores position t for every query head (its K row
// from HBM, q uniform).  Phase 2: thread t owns output dimension t and walks the positions.
template <int HD>
__global__ __launch_bounds__(128) void ogm_attn_partial_kernel(const float *__restrict__ q,
                                                               const __half *__restrict__ kc,
                                                               const __half *__restrict__ vc, uint32_t pos,
                                                               uint32_t max_splits, uint32_t n_head,
                                                               uint32_t n_head_kv, float scale,
                                                               float *__restrict__ part_o,
                                                               float *__restrict__ part_ml) {
  __shared__ float sc[ATT_MAXG][OGM_ATTN_CHUNK];
  __shared__ float red[ATT_MAXG][2];
  const uint32_t kvh = blockIdx.x, split = blockIdx.y;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t G = n_head / n_head_kv;
  const uint32_t kv_dim = n_head_kv * HD;
  const uint32_t n_pos = pos + 1u;
  const uint32_t p0 = split * OGM_ATTN_CHUNK;
  if (p0 >= n_pos) return;
  const uint32_t n_here = min(OGM_ATTN_CHUNK, n_pos - p0);
  const bool valid = tid < n_here;

  // ---- phase 1: scores
  float acc[ATT_MAXG];
#pragma unroll
  for (int g = 0; g < ATT_MAXG; g++) acc[g] = 0.0f;
  if (valid) {
    const __half *krow = kc + (size_t)(p0 + tid) * kv_dim + kvh * HD;
    const float *qb = q + (size_t)kvh * G * HD;
#pragma unroll 2
    for (int d = 0; d < HD; d += 8) {
      const uint4 raw = *(const uint4 *)(krow + d);
      const __half2 *h2 = (const __half2 *)&raw;
      float kf[8];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float2 f = __half22float2(h2[j]);
        kf[2 * j] = f.x;
        kf[2 * j + 1] = f.y;
      }
#pragma unroll
      for (int g = 0; g < ATT_MAXG; g++) {
        if ((uint32_t)g < G) {
#pragma unroll
          for (int j = 0; j < 8; j++) acc[g] += qb[g * HD + d + j] * kf[j];
        }
      }
    }
  }
  // block max and sum per query head
#pragma unroll
  for (int g = 0; g < ATT_MAXG; g++) {
    if ((uint32_t)g >= G) break;
    const float s = valid ? acc[g] * scale : -INFINITY;
    float m = s;
#pragma unroll
    for (int k = 1; k < 64; k <<= 1) m = fmaxf(m, __shfl_xor(m, k, 64));
    if (lane == 0) red[g][wave] = m;
    __syncthreads();
    m = fmaxf(red[g][0], red[g][1]);
    __syncthreads();
    const float e = valid ? expf(s - m) : 0.0f;
    sc[g][tid] = e;
    float l = e;
#pragma unroll
    for (int k = 1; k < 64; k <<= 1) l += __shfl_xor(l, k, 64);
    if (lane == 0) red[g][wave] = l;
    __syncthreads();
    if (tid == 0) {
      const uint32_t h = kvh * G + g;
      part_ml[((size_t)h * max_splits + split) * 2] = m;
      part_ml[((size_t)h * max_splits + split) * 2 + 1] = red[g][0] + red[g][1];
    }
    __syncthreads();
  }

  // ---- phase 2: weighted sum of V rows, one output dimension per thread
  if (tid < HD) {
    float o[ATT_MAXG];
#pragma unroll
    for (int g = 0; g < ATT_MAXG; g++) o[g] = 0.0f;
    const __half *vcol = vc + (size_t)p0 * kv_dim + kvh * HD + tid;
    for (uint32_t p = 0; p < n_here; p++) {
      const float vv = __half2float(vcol[(size_t)p * kv_dim]);
#pragma unroll
      for (int g = 0; g < ATT_MAXG; g++)
        if ((uint32_t)g < G) o[g] += sc[g][p] * vv;
    }
#pragma unroll
    for (int g = 0; g < ATT_MAXG; g++)
      if ((uint32_t)g < G)
        part_o[((size_t)(kvh * G + g) * max_splits + split) * HD + tid] = o[g];
  }
}

// One workgroup; wave w owns the 256-runs w, w + n_wave, ... of the output (n_head * HD values),
// lane l their elements 4l..4l+3 (one head, four dimensions): merges the chunks' partial
// softmaxes, stores and quantizes.
template <int GROUP>
__global__ __launch_bounds__(1024) void ogm_attn_combine_quant_kernel(const float *__restrict__ part_o,
                                                                      const float *__restrict__ part_ml,
                                                                      uint32_t n_splits, uint32_t max_splits,
                                                                      uint32_t n, uint32_t head_dim,
                                                                      float *__restrict__ attn_out,
                                                                      OgmActDev act) {
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, n_wave = blockDim.x >> 6;
  for (uint32_t run = wave; run * 256u < n; run += n_wave) {
    const uint32_t e0 = run * 256u + 4u * lane;
    const bool active = e0 < n;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) {
      const uint32_t h = e0 / head_dim, d = e0 - h * head_dim;
      const float *ml = part_ml + (size_t)h * max_splits * 2;
      float M = -INFINITY;
      for (uint32_t s = 0; s < n_splits; s++) M = fmaxf(M, ml[2 * s]);
      float den = 0.0f;
      for (uint32_t s = 0; s < n_splits; s++) {
        const float f = expf(ml[2 * s] - M);
        const float4 po = *(const float4 *)(part_o + ((size_t)h * max_splits + s) * head_dim + d);
        o.x += f * po.x; o.y += f * po.y; o.z += f * po.z; o.w += f * po.w;
        den += f * ml[2 * s + 1];
      }
      o.x /= den; o.y /= den; o.z /= den; o.w /= den;
      if (attn_out) *(float4 *)(attn_out + e0) = o;
    }
    ogm_quantize_store<GROUP>(o, e0, active, lane, act.q, act.d, act.sums, act.bsum);
  }
}

hipError_t ogm_launch_attn_decode(const float *q, const void *k_cache_layer, const void *v_cache_layer,
                                  uint32_t pos, uint32_t max_splits, uint32_t n_head, uint32_t n_head_kv,
                                  uint32_t head_dim, float scale, float *part_o, float *part_ml, int mode,
                                  float *attn_out, OgmActDev act, hipStream_t stream) {
  if (n_head_kv == 0 || n_head % n_head_kv != 0 || n_head / n_head_kv > ATT_MAXG) return hipErrorInvalidValue;
  const uint32_t n_splits = pos / OGM_ATTN_CHUNK + 1u;
  if (n_splits > max_splits) return hipErrorInvalidValue;
  const uint32_t n = n_head * head_dim;
  if (n % 32u != 0) return hipErrorInvalidValue;
  const dim3 grid(n_head_kv, n_splits);
  if (head_dim == 128)
    hipLaunchKernelGGL(ogm_attn_partial_kernel<128>, grid, dim3(128), 0, stream, q, (const __half *)k_cache_layer,
                       (const __half *)v_cache_layer, pos, max_splits, n_head, n_head_kv, scale, part_o, part_ml);
  else if (head_dim == 64)
    hipLaunchKernelGGL(ogm_attn_partial_kernel<64>, grid, dim3(128), 0, stream, q, (const __half *)k_cache_layer,
                       (const __half *)v_cache_layer, pos, max_splits, n_head, n_head_kv, scale, part_o, part_ml);
  else
    return hipErrorInvalidValue;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const uint32_t runs = (n + 255u) / 256u;
  const uint32_t waves = runs < 16u ? runs : 16u;
  if (mode == 0)
    hipLaunchKernelGGL(ogm_attn_combine_quant_kernel<32>, dim3(1), dim3(waves * 64), 0, stream, part_o, part_ml,
                       n_splits, max_splits, n, head_dim, attn_out, act);
  else
    hipLaunchKernelGGL(ogm_attn_combine_quant_kernel<256>, dim3(1), dim3(waves * 64), 0, stream, part_o, part_ml,
                       n_splits, max_splits, n, head_dim, attn_out, act);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// SwiGLU + quantize

template <int GROUP>
__global__ __launch_bounds__(64) void ogm_swiglu_quant_kernel(const float *__restrict__ gate,
                                                              const float *__restrict__ up, uint32_t n,
                                                              float *__restrict__ h, OgmActDev act) {
  const uint32_t lane = threadIdx.x;
  const uint32_t e0 = blockIdx.x * 256u + 4u * lane;
  const bool active = e0 < n;
  float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
  if (active) {
    const float4 g = *(const float4 *)(gate + e0), u = *(const float4 *)(up + e0);
    o.x = g.x / (1.0f + expf(-g.x)) * u.x;
    o.y = g.y / (1.0f + expf(-g.y)) * u.y;
    o.z = g.z / (1.0f + expf(-g.z)) * u.z;
    o.w = g.w / (1.0f + expf(-g.w)) * u.w;
    if (h) *(float4 *)(h + e0) = o;
  }
  ogm_quantize_store<GROUP>(o, e0, active, lane, act.q, act.d, act.sums, act.bsum);
}

hipError_t ogm_launch_swiglu_quant(int mode, const float *gate, const float *up, uint32_t n, float *h,
                                   OgmActDev act, hipStream_t stream) {
  if (n == 0 || n % 32u != 0) return hipErrorInvalidValue;
  const dim3 grid((n + 255u) / 256u);
  if (mode == 0)
    hipLaunchKernelGGL(ogm_swiglu_quant_kernel<32>, grid, dim3(64), 0, stream, gate, up, n, h, act);
  else
    hipLaunchKernelGGL(ogm_swiglu_quant_kernel<256>, grid, dim3(64), 0, stream, gate, up, n, h, act);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// argmax (last of equal maxima, as Iterator::max_by returns it)

__device__ __forceinline__ bool argmax_better(float v, uint32_t i, float bv, uint32_t bi) {
  return v > bv || (v == bv && i > bi);
}

__global__ __launch_bounds__(256) void ogm_argmax_kernel(const float *__restrict__ x, uint32_t n,
                                                         uint32_t *__restrict__ scratch, uint32_t *__restrict__ out,
                                                         int final_stage) {
  __shared__ float sv[256];
  __shared__ uint32_t si[256];
  const uint32_t tid = threadIdx.x;
  float bv = -INFINITY;
  uint32_t bi = 0;
  if (!final_stage) {
    for (uint32_t i = blockIdx.x * 256u + tid; i < n; i += gridDim.x * 256u)
      if (argmax_better(x[i], i, bv, bi)) { bv = x[i]; bi = i; }
  } else {
    // scratch: 256 values then 256 indices, one per first-stage workgroup
    if (tid < n) { bv = __uint_as_float(scratch[tid]); bi = scratch[256 + tid]; }
  }
  sv[tid] = bv;
  si[tid] = bi;
  __syncthreads();
  for (uint32_t s = 128; s > 0; s >>= 1) {
    if (tid < s && argmax_better(sv[tid + s], si[tid + s], sv[tid], si[tid])) {
      sv[tid] = sv[tid + s];
      si[tid] = si[tid + s];
    }
    __syncthreads();
  }
  if (tid == 0) {
    if (!final_stage) {
      scratch[blockIdx.x] = __float_as_uint(sv[0]);
      scratch[256 + blockIdx.x] = si[0];
    } else {
      *out = si[0];
    }
  }
}

hipError_t ogm_launch_argmax(const float *logits, uint32_t n, uint32_t *scratch, uint32_t *out,
                             hipStream_t stream) {
  if (n == 0) return hipErrorInvalidValue;
  uint32_t wgs = (n + 255u) / 256u;
  if (wgs > 256u) wgs = 256u;
  hipLaunchKernelGGL(ogm_argmax_kernel, dim3(wgs), dim3(256), 0, stream, logits, n, scratch, out, 0);
  hipLaunchKernelGGL(ogm_argmax_kernel, dim3(1), dim3(256), 0, stream, logits, wgs, scratch, out, 1);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------

__global__ void ogm_f32_to_f16_kernel(const float *__restrict__ src, __half *__restrict__ dst, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = __float2half_rn(src[i]);
}

hipError_t ogm_launch_f32_to_f16(const float *src, void *dst, size_t n, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(ogm_f32_to_f16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, src,
                     (__half *)dst, n);
  return hipGetLastError();
}
