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
  float4 v[4], wv[4];
  float ss = 0.0f;
  // every load first (x, the residual delta and the norm weights share one trip to memory)
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const uint32_t e0 = (wave + k * n_wave) * 256u + 4u * lane;
    v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    wv[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
    if (e0 < n) {
      v[k] = *(const float4 *)(x + e0);
      wv[k] = *(const float4 *)(weight + e0);
      if (delta) d = *(const float4 *)(delta + e0);
    }
    if (e0 < n && delta) {
      v[k].x += d.x; v[k].y += d.y; v[k].z += d.z; v[k].w += d.w;
      *(float4 *)(x + e0) = v[k];
    }
    ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
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
      o.x = v[k].x * scale * wv[k].x; o.y = v[k].y * scale * wv[k].y;
      o.z = v[k].z * scale * wv[k].z; o.w = v[k].w * scale * wv[k].w;
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


// Workgroup (kvh, split): the G query heads of K/V head kvh against positions
// split * 128 .. + 128.  Every load of the workgroup is requested first (its K rows and its V
// rows in one trip to memory).  Phase 1: thread t scores position t for every query head; q is
// uniform (scalar loads).  Phase 2: sixteen threads share a V row (eight dimensions each), eight
// rows per step, and LDS adds the eight partial sums.
template <int HD, int G>
__global__ __launch_bounds__(128) void ogm_attn_partial_kernel(const float *__restrict__ q,
                                                               const __half *__restrict__ kc,
                                                               const __half *__restrict__ vc, uint32_t pos,
                                                               uint32_t max_splits, uint32_t n_head_kv,
                                                               float scale, float *__restrict__ part_o,
                                                               float *__restrict__ part_ml) {
  constexpr int TPR = HD / 8;            // threads per V row
  constexpr int ROWS = 128 / TPR;        // V rows in flight per step
  constexpr int STEPS = OGM_ATTN_CHUNK / ROWS;
  __shared__ float sc[G][OGM_ATTN_CHUNK];
  __shared__ float red[2][G][2];
  __shared__ float osum[ROWS][G][HD];
  const uint32_t kvh = blockIdx.x, split = blockIdx.y;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t kv_dim = n_head_kv * HD;
  const uint32_t n_pos = pos + 1u;
  const uint32_t p0 = split * OGM_ATTN_CHUNK;
  if (p0 >= n_pos) return;
  const uint32_t n_here = min(OGM_ATTN_CHUNK, n_pos - p0);
  const bool valid = tid < n_here;

  const uint32_t rr = tid / TPR, dc = tid - rr * TPR;   // phase 2: row slot and 8-dimension chunk
  // rows past the chunk's end read the last valid row; their scores are discarded (weight 0)
  const __half *krow = kc + (size_t)(p0 + min(tid, n_here - 1u)) * kv_dim + kvh * HD;
  uint4 kr[HD / 8];
#pragma unroll
  for (int c = 0; c < HD / 8; c++) kr[c] = *(const uint4 *)(krow + 8 * c);
  const __half *vbase = vc + (size_t)p0 * kv_dim + kvh * HD + 8u * dc;
  uint4 vr[STEPS];
#pragma unroll
  for (int st = 0; st < STEPS; st++)
    vr[st] = *(const uint4 *)(vbase + (size_t)min((uint32_t)(st * ROWS) + rr, n_here - 1u) * kv_dim);

  // ---- phase 1: scores
  float acc[G];
#pragma unroll
  for (int g = 0; g < G; g++) acc[g] = 0.0f;
  {
    const float *qb = q + (size_t)kvh * G * HD;
#pragma unroll
    for (int c = 0; c < HD / 8; c++) {
      const __half2 *h2 = (const __half2 *)&kr[c];
      float kf[8];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float2 f = __half22float2(h2[j]);
        kf[2 * j] = f.x;
        kf[2 * j + 1] = f.y;
      }
#pragma unroll
      for (int g = 0; g < G; g++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[g] = fmaf(qb[g * HD + 8 * c + j], kf[j], acc[g]);
    }
  }
  // workgroup maximum and sum per query head: two barriers for all heads
  float sv[G], mv[G];
#pragma unroll
  for (int g = 0; g < G; g++) {
    sv[g] = valid ? acc[g] * scale : -INFINITY;
    float m = sv[g];
#pragma unroll
    for (int k = 1; k < 64; k <<= 1) m = fmaxf(m, __shfl_xor(m, k, 64));
    if (lane == 0) red[0][g][wave] = m;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; g++) {
    mv[g] = fmaxf(red[0][g][0], red[0][g][1]);
    const float e = valid ? expf(sv[g] - mv[g]) : 0.0f;
    sc[g][tid] = e;
    float l = e;
#pragma unroll
    for (int k = 1; k < 64; k <<= 1) l += __shfl_xor(l, k, 64);
    if (lane == 0) red[1][g][wave] = l;
  }
  __syncthreads();
  if (tid < G) {
    const uint32_t h = kvh * G + tid;
    part_ml[((size_t)h * max_splits + split) * 2] = fmaxf(red[0][tid][0], red[0][tid][1]);
    part_ml[((size_t)h * max_splits + split) * 2 + 1] = red[1][tid][0] + red[1][tid][1];
  }

  // ---- phase 2: weighted sum of V rows
  {
    float o[G][8];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
      for (int j = 0; j < 8; j++) o[g][j] = 0.0f;
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
      const uint32_t p = st * ROWS + rr;   // past the chunk's end the weight sc is 0
      const __half2 *h2 = (const __half2 *)&vr[st];
      float vf[8];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float2 f = __half22float2(h2[j]);
        vf[2 * j] = f.x;
        vf[2 * j + 1] = f.y;
      }
#pragma unroll
      for (int g = 0; g < G; g++) {
        const float w = sc[g][p];
#pragma unroll
        for (int j = 0; j < 8; j++) o[g][j] = fmaf(w, vf[j], o[g][j]);
      }
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
      *(float4 *)&osum[rr][g][8 * dc] = make_float4(o[g][0], o[g][1], o[g][2], o[g][3]);
      *(float4 *)&osum[rr][g][8 * dc + 4] = make_float4(o[g][4], o[g][5], o[g][6], o[g][7]);
    }
    __syncthreads();
    for (uint32_t i = tid; i < G * HD; i += 128u) {
      const uint32_t g = i / HD, d = i - g * HD;
      float t = 0.0f;
#pragma unroll
      for (int r = 0; r < ROWS; r++) t += osum[r][g][d];
      part_o[((size_t)(kvh * G + g) * max_splits + split) * HD + d] = t;
    }
  }
}

// One wave per 256-run of the output (n_head * HD values), lane l its elements 4l..4l+3 (one
// head, four dimensions): merges the chunks' partial softmaxes, stores and quantizes.
template <int GROUP>
__global__ __launch_bounds__(64) void ogm_attn_combine_quant_kernel(const float *__restrict__ part_o,
                                                                    const float *__restrict__ part_ml,
                                                                    uint32_t n_splits, uint32_t max_splits,
                                                                    uint32_t n, uint32_t head_dim,
                                                                    float *__restrict__ attn_out,
                                                                    OgmActDev act) {
  const uint32_t lane = threadIdx.x;
  const uint32_t e0 = blockIdx.x * 256u + 4u * lane;
  const bool active = e0 < n;
  float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
  if (active) {
    const uint32_t h = e0 / head_dim, d = e0 - h * head_dim;
    const float2 *ml = (const float2 *)(part_ml + (size_t)h * max_splits * 2);
    const float *po = part_o + (size_t)h * max_splits * head_dim + d;
    // eight chunks at a time: their loads are independent of the running maximum
    float M = -INFINITY, den = 0.0f;
    for (uint32_t s0 = 0; s0 < n_splits; s0 += 8u) {
      float2 mls[8];
      float4 pos_[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const uint32_t s = min(s0 + u, n_splits - 1u);
        mls[u] = ml[s];
        pos_[u] = *(const float4 *)(po + (size_t)s * head_dim);
      }
      float Mn = M;
#pragma unroll
      for (int u = 0; u < 8; u++)
        if (s0 + u < n_splits) Mn = fmaxf(Mn, mls[u].x);
      const float resc = expf(M - Mn);   // exp(-inf) = 0 on the first group
      o.x *= resc; o.y *= resc; o.z *= resc; o.w *= resc;
      den *= resc;
#pragma unroll
      for (int u = 0; u < 8; u++) {
        if (s0 + u < n_splits) {
          const float f = expf(mls[u].x - Mn);
          o.x += f * pos_[u].x; o.y += f * pos_[u].y; o.z += f * pos_[u].z; o.w += f * pos_[u].w;
          den += f * mls[u].y;
        }
      }
      M = Mn;
    }
    o.x /= den; o.y /= den; o.z /= den; o.w /= den;
    if (attn_out) *(float4 *)(attn_out + e0) = o;
  }
  ogm_quantize_store<GROUP>(o, e0, active, lane, act.q, act.d, act.sums, act.bsum);
}

hipError_t ogm_launch_attn_decode(const float *q, const void *k_cache_layer, const void *v_cache_layer,
                                  uint32_t pos, uint32_t max_splits, uint32_t n_head, uint32_t n_head_kv,
                                  uint32_t head_dim, float scale, float *part_o, float *part_ml, int mode,
                                  float *attn_out, OgmActDev act, hipStream_t stream) {
  if (n_head_kv == 0 || n_head % n_head_kv != 0) return hipErrorInvalidValue;
  const uint32_t n_splits = pos / OGM_ATTN_CHUNK + 1u;
  if (n_splits > max_splits) return hipErrorInvalidValue;
  const uint32_t n = n_head * head_dim;
  if (n % 32u != 0) return hipErrorInvalidValue;
  const dim3 grid(n_head_kv, n_splits);
  const uint32_t G = n_head / n_head_kv;
#define OGM_ATTN_LAUNCH(HD_, G_)                                                                    \
  hipLaunchKernelGGL((ogm_attn_partial_kernel<HD_, G_>), grid, dim3(128), 0, stream, q,              \
                     (const __half *)k_cache_layer, (const __half *)v_cache_layer, pos, max_splits,   \
                     n_head_kv, scale, part_o, part_ml)
  if (head_dim == 128 && G == 1) OGM_ATTN_LAUNCH(128, 1);
  else if (head_dim == 128 && G == 2) OGM_ATTN_LAUNCH(128, 2);
  else if (head_dim == 128 && G == 4) OGM_ATTN_LAUNCH(128, 4);
  else if (head_dim == 128 && G == 8) OGM_ATTN_LAUNCH(128, 8);
  else if (head_dim == 64 && G == 1) OGM_ATTN_LAUNCH(64, 1);
  else if (head_dim == 64 && G == 2) OGM_ATTN_LAUNCH(64, 2);
  else if (head_dim == 64 && G == 4) OGM_ATTN_LAUNCH(64, 4);
  else if (head_dim == 64 && G == 8) OGM_ATTN_LAUNCH(64, 8);
  else return hipErrorInvalidValue;
#undef OGM_ATTN_LAUNCH
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const dim3 cgrid((n + 255u) / 256u);
  if (mode == 0)
    hipLaunchKernelGGL(ogm_attn_combine_quant_kernel<32>, cgrid, dim3(64), 0, stream, part_o, part_ml,
                       n_splits, max_splits, n, head_dim, attn_out, act);
  else
    hipLaunchKernelGGL(ogm_attn_combine_quant_kernel<256>, cgrid, dim3(64), 0, stream, part_o, part_ml,
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

// ------------------------------------------------------------------------------------------
// one row of a quantized matrix as f32: the embedding lookup (LlamaModel::run_layers,
// llama.rs:609-614, over dequantize_q8_0 / _q4_k / _q6_k, quant.rs:639-649, 666-697, 746-787),
// reading the tile-planar device copy.  One thread per element; the f32 expressions are the
// reference's, so the values are bit-identical (built without FMA contraction).

#include "ogm_layout.h"

__device__ __forceinline__ float dq_f16(const uint8_t *p) {
  return __half2float(__ushort_as_half((unsigned short)(p[0] | (p[1] << 8))));
}

__global__ __launch_bounds__(256) void ogm_dequant_row_kernel(const uint8_t *__restrict__ wt, uint32_t ggml_type,
                                                              uint32_t in_dim, uint32_t out_dim, uint32_t row,
                                                              const uint32_t *__restrict__ row_dev,
                                                              float *__restrict__ out) {
  const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= in_dim) return;
  if (row_dev) row = *row_dev;
  if (row >= out_dim) row = out_dim - 1u;   // a token id beyond the table reads its last row
  OgmLayout l;
  ogm_layout_for(ggml_type, &l);
  const OgmTiling t = ogm_tiling_for(in_dim / l.block_elems, out_dim);
  const uint32_t s = e / l.block_elems, j = e - s * l.block_elems;
  size_t tile;
  uint32_t lane;
  ogm_unit_place(t, row, s, &tile, &lane);
  const uint8_t *tb = wt + tile * l.tile_bytes;
  // byte `o` of the block's piece area (the raw block minus its tail)
  auto piece_byte = [&](uint32_t o) -> uint32_t { return tb[(o >> 4) * 1024u + lane * 16u + (o & 15u)]; };
  float v;
  if (ggml_type == OGM_Q8_0) {
    const float d = dq_f16(tb + l.pieces * 1024u + lane * 2u);
    v = (float)(int8_t)piece_byte(j) * d;
  } else if (ggml_type == OGM_Q4_K) {
    const uint8_t *hd = tb + lane * 16u;   // piece 0: d, dmin, scales
    const float d = dq_f16(hd), dmin = dq_f16(hd + 2);
    const uint32_t g4 = j >> 6, hi = (j >> 5) & 1u, li = j & 31u;
    const uint32_t is = 2u * g4 + hi;      // sub-block
    // get_scale_min_k4 (quant.rs:653-662)
    const uint8_t *q = hd + 4;
    uint32_t sc, m;
    if (is < 4) {
      sc = q[is] & 63u;
      m = q[is + 4] & 63u;
    } else {
      sc = (q[is + 4] & 0xFu) | ((q[is - 4] >> 6) << 4);
      m = (q[is + 4] >> 4) | ((q[is] >> 6) << 4);
    }
    const uint32_t byte = piece_byte(16u + 32u * g4 + li);
    const uint32_t nib = hi ? (byte >> 4) : (byte & 0xFu);
    const float d1 = d * (float)sc, mm = dmin * (float)m;
    v = d1 * (float)nib - mm;
  } else {  // Q6_K
    const float d = dq_f16(tb + l.pieces * 1024u + lane * 2u);
    const uint32_t h = j >> 7, jj = j & 127u, qd = jj >> 5, li = jj & 31u;
    const uint32_t qlb = piece_byte(64u * h + li + ((qd & 1u) ? 32u : 0u));
    const uint32_t qhb = piece_byte(128u + 32u * h + li);
    const int sc = (int)(int8_t)piece_byte(192u + 8u * h + (li >> 4) + 2u * qd);
    const int qv = (int)(((qd < 2 ? qlb : (qlb >> 4)) & 0xFu) | (((qhb >> (2u * qd)) & 3u) << 4)) - 32;
    v = d * (float)sc * (float)qv;
  }
  out[e] = v;
}

hipError_t ogm_launch_dequant_row(const uint8_t *wt, uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim,
                                  uint32_t row, const uint32_t *row_dev, float *out, hipStream_t stream) {
  OgmLayout l;
  if (!ogm_layout_for(ggml_type, &l) || in_dim == 0 || in_dim % l.block_elems != 0 || out_dim == 0)
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(ogm_dequant_row_kernel, dim3((in_dim + 255u) / 256u), dim3(256), 0, stream, wt, ggml_type,
                     in_dim, out_dim, row, row_dev, out);
  return hipGetLastError();
}
