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

// One workgroup per row (ogm_norm_quant_row).
template <int GROUP>
__global__ __launch_bounds__(1024) void ogm_norm_quant_kernel(float *__restrict__ x,
                                                              const float *__restrict__ delta,
                                                              const float *__restrict__ weight, uint32_t n,
                                                              float eps, float *__restrict__ normed,
                                                              OgmActDev act, const float *__restrict__ x_src) {
  __shared__ float red[64];
  const uint32_t tid = threadIdx.x, n_wave = blockDim.x >> 6;
  {   // one workgroup per row of a batch
    const uint32_t r = act.xt ? ogm_xt_row_of_workgroup(blockIdx.x, gridDim.x) : blockIdx.x;
    const size_t row = (size_t)r * n;
    x += row;
    if (x_src) x_src += row;
    if (delta) delta += row;
    if (normed) normed += row;
    act.q += row;
    act.d += (size_t)r * (n / GROUP);
    act.sums += (size_t)r * (n / 16u);
    act.bsum += (size_t)r * (n / 32u);
    if (act.bs16) act.bs16 += (size_t)r * (n / 16u);
    act.xt = ogm_xt_row(act.xt, r, n);
  }
  ogm_norm_quant_row<GROUP, false>(x, delta, weight, n, eps, normed, act, red, tid, n_wave, x_src);
}

hipError_t ogm_launch_norm_quant(int mode, float *x, const float *delta, const float *weight, uint32_t n,
                                 float eps, float *normed, OgmActDev act, hipStream_t stream, uint32_t n_rows,
                                 const float *x_src) {
  if (n == 0 || n % 32u != 0 || n > 16384u || n_rows == 0) return hipErrorInvalidValue;
  const uint32_t runs = (n + 255u) / 256u;
  // few rows: a wave per run, the shortest chain; from 1024 rows (2048 rows: 2 % of a prefill): four runs per wave
  // (the row's bits do not depend on it)
  const uint32_t waves = n_rows >= 1024u ? (runs + 3u) / 4u : (runs < 16u ? runs : 16u);
  if (mode == 0)
    hipLaunchKernelGGL(ogm_norm_quant_kernel<32>, dim3(n_rows), dim3(waves * 64), 0, stream, x, delta, weight,
                       n, eps, normed, act, x_src);
  else
    hipLaunchKernelGGL(ogm_norm_quant_kernel<256>, dim3(n_rows), dim3(waves * 64), 0, stream, x, delta, weight,
                       n, eps, normed, act, x_src);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// RoPE table: cos and sin of pos * freq[p] for every rotated pair, once per token (all layers
// rotate by the same angles)

__global__ __launch_bounds__(64) void ogm_rope_table_kernel(const float *__restrict__ freq, uint32_t pos,
                                                            uint32_t rope_half, float2 *__restrict__ cs) {
  const uint32_t p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= rope_half) return;
  const float theta = (float)(pos + blockIdx.y) * freq[p];   // row blockIdx.y: the token at pos + blockIdx.y
  // The f32 angle's sine and cosine in double precision, rounded once: the correctly rounded f32 values but for
  // rare double roundings, which is what the C library's sinf / cosf (the reference's f32::sin_cos) return as
  // well.  The single-precision device routine differs from them in the last bit often enough to move a rotated
  // K component across an f16 rounding boundary in a visible share of a cache row.
  double sn, c;
  sincos((double)theta, &sn, &c);
  cs[(size_t)blockIdx.y * rope_half + p] = make_float2((float)c, (float)sn);
}

hipError_t ogm_launch_rope_table(const float *freq, uint32_t pos, uint32_t n_tokens, uint32_t rope_dim, void *cs,
                                 hipStream_t stream) {
  if (rope_dim % 2u != 0 || n_tokens == 0 || n_tokens > 65535u) return hipErrorInvalidValue;
  if (rope_dim == 0) return hipSuccess;
  hipLaunchKernelGGL(ogm_rope_table_kernel, dim3((rope_dim / 2u + 63u) / 64u, n_tokens), dim3(64), 0, stream, freq,
                     pos, rope_dim / 2u, (float2 *)cs);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// attention of one token: RoPE of q and of the new k, the cache write, a partial softmax per
// chunk of positions, and (in the workgroup that finishes last) the merge of the chunks with the
// quantizer of the next matmul

// K/V rows are cached as f16 (the reference's host cache is f32, kv_cache.rs:75-78): a component
// beyond the f16 range saturates at +-65504 instead of becoming an infinity, which would turn a
// zero weight into NaN in the weighted V sum and swamp every score it touches in K.  NaN stays NaN.
__device__ __forceinline__ __half ogm_f16_sat(float v) {
  return __float2half_rn(v != v ? v : fminf(fmaxf(v, -65504.0f), 65504.0f));
}

__device__ __forceinline__ float2 rope_pair(float2 ab, float2 cs) {
  return make_float2(ab.x * cs.x - ab.y * cs.y, ab.x * cs.y + ab.y * cs.x);
}

// Device-coherent accesses for results one workgroup hands to another inside a kernel: they go
// through to the level all compute dies share, so no cache write-back or invalidate is needed.
template <bool COHERENT>
__device__ __forceinline__ float2 ld_pair(const float *p) {
  if constexpr (COHERENT) {
    const uint64_t u = __hip_atomic_load((const uint64_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(__uint_as_float((uint32_t)u), __uint_as_float((uint32_t)(u >> 32)));
  } else {
    return *(const float2 *)p;
  }
}
template <bool COHERENT>
__device__ __forceinline__ void st_one(float *p, float v) {
  if constexpr (COHERENT) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}

// Wall-clock stamps for timeline builds of the attention kernel: a variant of the library built with
// -DOGM_ATTN_STAMPS=1 keeps eight stamps per workgroup of the last launch, and ogm_attn_stamps_read hands them out
// (the shipped library has neither stamps nor buffer, and the reader reports that).
#ifdef OGM_ATTN_STAMPS
__device__ unsigned long long ogm_attn_stamps[4096 * 8];
#define OGM_STAMP(i)                                                                              \
  do {                                                                                            \
    if (threadIdx.x == 0)                                                                         \
      ogm_attn_stamps[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 8 + (i)] = wall_clock64(); \
  } while (0)
#else
#define OGM_STAMP(i) do { } while (0)
#endif

// A partial softmax over some chunks of four neighbouring output elements: running maximum,
// denominator and weighted sums relative to that maximum.
struct AttnPart {
  float m, den;
  float4 o;
};

// Merges chunks s_first, s_first + s_step, ... (< n_splits) of the four output elements d .. d + 3
// of query head h.
template <bool COHERENT>
__device__ __forceinline__ AttnPart attn_merge_chunks(const float *part_o, const float *part_ml, uint32_t h,
                                                      uint32_t d, uint32_t s_first, uint32_t s_step,
                                                      uint32_t n_splits, uint32_t max_splits, uint32_t head_dim) {
  const float *ml = part_ml + (size_t)h * max_splits * 2;
  const float *po = part_o + (size_t)h * max_splits * head_dim + d;
  AttnPart r;
  r.o = make_float4(0.f, 0.f, 0.f, 0.f);
  r.m = -INFINITY;
  r.den = 0.0f;
  // eight chunks at a time: their loads are independent of the running maximum
  for (uint32_t s0 = s_first; s0 < n_splits; s0 += 8u * s_step) {
    float2 mls[8];
    float4 pos_[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const uint32_t s = min(s0 + u * s_step, n_splits - 1u);
      mls[u] = ld_pair<COHERENT>(ml + 2u * s);
      const float2 lo = ld_pair<COHERENT>(po + (size_t)s * head_dim), hi = ld_pair<COHERENT>(po + (size_t)s * head_dim + 2);
      pos_[u] = make_float4(lo.x, lo.y, hi.x, hi.y);
    }
    float Mn = r.m;
#pragma unroll
    for (int u = 0; u < 8; u++)
      if (s0 + u * s_step < n_splits) Mn = fmaxf(Mn, mls[u].x);
    const float resc = expf(r.m - Mn);   // exp(-inf) = 0 on the first group
    r.o.x *= resc; r.o.y *= resc; r.o.z *= resc; r.o.w *= resc;
    r.den *= resc;
#pragma unroll
    for (int u = 0; u < 8; u++) {
      if (s0 + u * s_step < n_splits) {
        const float f = expf(mls[u].x - Mn);
        r.o.x += f * pos_[u].x; r.o.y += f * pos_[u].y; r.o.z += f * pos_[u].z; r.o.w += f * pos_[u].w;
        r.den += f * mls[u].y;
      }
    }
    r.m = Mn;
  }
  return r;
}

// Workgroup (kvh, split), 512 threads: the G query heads of K/V head kvh against positions
// split * 128 .. + 128.
//   * Every cache load of the workgroup is requested first: four threads share a K row (each
//     every fourth 16-byte piece), HD / 8 threads a V row.
//   * q of the G heads is rotated into LDS (pairs 2i, 2i+1; tensor.rs:1115-1177).  The workgroup
//     of the last chunk also rotates the token's k, rounds k and v to f16, writes both cache rows
//     and uses the LDS copy for the row of the current position.
//   * Phase 1: scores; the partial dot products of a row are exchanged so that each of its four
//     lanes ends with the whole score of G / 4 heads.  Phase 2: weighted V sum, exchanged the
//     same way across the rows a wave holds, then summed over the eight waves in LDS.
//   * GROUP != 0 (G * HD is a multiple of the quantizer's group): the workgroup that takes the
//     last ticket of its K/V head merges the chunks and quantizes the G * HD outputs; no other
//     workgroup waits for anything.
//
// PREFILL: the same over a batch of query tokens (blockIdx.y; token t sits at position pos + t and
// attends to positions 0 .. pos + t).  q arrives with bias, norm and RoPE applied and every K/V
// row is in the cache already (ogm_qkv_pre_kernel), workgroups past a token's last chunk leave at
// once, and nothing is quantized: the next matmul is a GEMM that quantizes its own input.
template <int HD, int G, int GROUP, bool PREFILL = false, int CHUNK = (int)OGM_ATTN_CHUNK, bool MULTI = false>
__global__ __launch_bounds__(4 * CHUNK, (MULTI && G <= 4) ? 4 : 1) void ogm_attn_kernel(const float *__restrict__ q, const float *__restrict__ k_new,
                                                       const float *__restrict__ v_new,
                                                       const float2 *__restrict__ cs, uint32_t rope_half,
                                                       OgmAttnPre pre, uint32_t gq,
                                                       __half *__restrict__ kc, __half *__restrict__ vc,
                                                       uint32_t pos, uint32_t max_splits, uint32_t n_head_kv,
                                                       float scale, float *part_o, float *part_ml,
                                                       uint32_t *counters, float *__restrict__ attn_out,
                                                       OgmActDev act, uint32_t n_sub) {
  static_assert(!MULTI || CHUNK == 128, "several chunks a workgroup: chunks of 128");
  constexpr int NT = 4 * CHUNK, NW = NT / 64;   // four threads per cache position
  constexpr int KU = HD / 32;             // 16-byte pieces of a K row per thread
  constexpr int TPR = HD / 8;             // threads per V row
  constexpr int ROWS = NT / TPR;          // V rows in flight per step
  constexpr int STEPS = CHUNK / ROWS;
  constexpr int NV = G * 8;               // phase-2 partial sums per lane
  constexpr int NF = G >= 4 ? G / 4 : 1;  // scores a lane ends phase 1 with
  __shared__ __align__(16) float qs[G][HD];
  __shared__ __align__(16) __half kcur[HD];
  __shared__ __align__(16) __half vcur[HD];
  __shared__ float sc[G][CHUNK];
  __shared__ float red[2][G][NW];
  __shared__ __align__(16) float osum[NW][G][HD];
  __shared__ uint32_t s_last;
  __shared__ float mrg[GROUP != 0 ? 6 : 1][GROUP != 0 ? NT : 1];   // the final merge's slices
  static_assert(!PREFILL || GROUP == 0, "a prefill batch merges in its own launch");
  OGM_STAMP(0);
  // blockIdx.x: a K/V head and gq of the query heads (G head slots) that share it -- all of them, or one of
  // gridDim.x / n_head_kv equal parts of them when the model has more than eight per K/V head (the parts' workgroups
  // read the same cache rows; in the last chunk each writes the new rows, the same bytes)
  // (a batch: the tokens on y and the chunks on z, so that the workgroups that read the same cache rows, one per
  // token, start one after the other -- on the same XCD when the launch has eight workgroups on x -- and all but
  // the first find the rows in its L2)
  const uint32_t hg = blockIdx.x, split = PREFILL ? blockIdx.z : blockIdx.y, kvh = hg / (gridDim.x / n_head_kv);
  if constexpr (PREFILL) {
    const uint32_t tok = blockIdx.y;
    pos += tok;
    if (split * (MULTI ? n_sub : 1u) > pos / (uint32_t)CHUNK) return;   // the whole workgroup: this token has no such chunk
    const size_t n_head = (size_t)gridDim.x * gq;
    q += tok * n_head * HD;
    part_o += tok * n_head * max_splits * HD;
    part_ml += tok * n_head * max_splits * 2;
  }
  // MULTI (a decode step over a long context): the workgroup takes n_sub chunks in a row, see below.
  const uint32_t n_chunks = pos / (uint32_t)CHUNK + 1u;
  const uint32_t n_splits = PREFILL ? (MULTI ? (n_chunks + n_sub - 1u) / n_sub : n_chunks) : gridDim.y;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t kv_dim = n_head_kv * HD;
  const uint32_t n_pos = pos + 1u;
  const uint32_t c_first = MULTI ? split * n_sub : split;                       // the workgroup's first chunk ...
  const uint32_t c_end = MULTI ? min(c_first + n_sub, n_chunks) : split + 1u;   // ... and the one after its last
  const uint32_t p0 = c_first * (uint32_t)CHUNK;
  const uint32_t n_here = min((uint32_t)CHUNK, n_pos - p0);
  const bool is_last = !PREFILL && c_end == n_chunks;   // holds the current position, not yet cached
  const uint32_t cur = pos - p0;                 // meaningful in the last chunk only (MULTI: see there)

  const uint32_t rr = tid / TPR, dc = tid - rr * TPR;     // phase 2: row slot and 8-dimension chunk
  // phase 1: cache row and piece phase.  MULTI: a wave scores the sixteen rows whose V rows it sums in phase 2
  // (64 / TPR of every ROWS), so that the weights stay within the wave
  constexpr uint32_t R2 = 64u / (uint32_t)TPR;
  const uint32_t c = tid & 3u;
  const uint32_t r = MULTI ? (uint32_t)ROWS * ((lane >> 2) / R2) + R2 * wave + ((lane >> 2) % R2) : tid >> 2;
  // rows past the chunk's end read the last row; their scores are discarded (weight 0)
  const __half *krow = kc + (size_t)(p0 + min(r, n_here - 1u)) * kv_dim + kvh * HD;
  uint4 kr[KU];
#pragma unroll
  for (int j = 0; j < KU; j++) kr[j] = *(const uint4 *)(krow + 8 * (c + 4 * j));
  const __half *vbase = vc + (size_t)p0 * kv_dim + kvh * HD + 8u * dc;
  uint4 vr[STEPS];
#pragma unroll
  for (int st = 0; st < STEPS; st++)
    vr[st] = *(const uint4 *)(vbase + (size_t)min((uint32_t)(st * ROWS) + rr, n_here - 1u) * kv_dim);

  // ---- bias, per-head norm and RoPE: one wave per query head; in the workgroup of the last chunk
  // two more take the new k and v rows, which also go to the cache.  G counts the head slots of the
  // kernel, gq <= G the query heads the model has per K/V head: the other slots hold zeros and
  // store nothing.
  if constexpr (PREFILL) {
    for (uint32_t i = tid; i < (uint32_t)(G * HD / 4); i += NT) {
      const uint32_t g = i / (HD / 4), d4 = i - g * (HD / 4);
      float4 v4 = make_float4(0.f, 0.f, 0.f, 0.f);
      if (g < gq) v4 = *(const float4 *)(q + ((size_t)hg * gq + g) * HD + 4u * d4);
      *(float4 *)&qs[g][4u * d4] = v4;
    }
  } else {
    constexpr int PPL = (HD / 2 + 63) / 64;   // pairs per lane
    const uint32_t n_units = (uint32_t)G + (is_last ? 2u : 0u);
    for (uint32_t u = wave; u < n_units; u += NW) {
      const bool is_q = u < (uint32_t)G, is_v = u == (uint32_t)G + 1u;
      const bool live = !is_q || u < gq;
      const size_t row = (is_q ? (size_t)hg * gq + u : (size_t)kvh) * HD;
      const float *src = (is_q ? q : is_v ? v_new : k_new) + row;
      const float *bias = is_q ? pre.q_bias : is_v ? pre.v_bias : pre.k_bias;
      const float *nw = is_q ? pre.q_norm : is_v ? nullptr : pre.k_norm;
      float a[PPL], b[PPL];
      uint32_t ia[PPL], ib[PPL];
      float ss = 0.0f;
#pragma unroll
      for (int j = 0; j < PPL; j++) {
        const uint32_t p = lane + 64u * j;
        const bool have = p < (uint32_t)(HD / 2) && live;
        const bool split_pair = pre.neox != 0u && !is_v && p < rope_half;
        ia[j] = split_pair ? p : 2u * p;
        ib[j] = split_pair ? p + rope_half : 2u * p + 1u;
        a[j] = have ? src[ia[j]] : 0.0f;
        b[j] = have ? src[ib[j]] : 0.0f;
        if (bias != nullptr && have) {
          a[j] += bias[row + ia[j]];
          b[j] += bias[row + ib[j]];
        }
        ss += a[j] * a[j] + b[j] * b[j];
      }
      if (nw != nullptr) {
        ss = ogm_wave_sum(ss);
        const float sc_n = 1.0f / sqrtf(ss / (float)HD + pre.eps);
#pragma unroll
        for (int j = 0; j < PPL; j++) {
          const uint32_t p = lane + 64u * j;
          if (p < (uint32_t)(HD / 2)) {
            a[j] = a[j] * sc_n * nw[ia[j]];
            b[j] = b[j] * sc_n * nw[ib[j]];
          }
        }
      }
#pragma unroll
      for (int j = 0; j < PPL; j++) {
        const uint32_t p = lane + 64u * j;
        if (p >= (uint32_t)(HD / 2)) continue;
        float2 ab = make_float2(a[j], b[j]);
        if (!is_v && p < rope_half) ab = rope_pair(ab, cs[p]);
        if (is_q) {
          qs[u][ia[j]] = ab.x;
          qs[u][ib[j]] = ab.y;
        } else {
          const __half ha = ogm_f16_sat(ab.x), hb = ogm_f16_sat(ab.y);
          __half *lds = is_v ? vcur : kcur;
          __half *cache = (is_v ? vc : kc) + (size_t)pos * kv_dim + kvh * HD;
          lds[ia[j]] = ha;
          lds[ib[j]] = hb;
          cache[ia[j]] = ha;
          cache[ib[j]] = hb;
        }
      }
    }
  }
  // The cache loads requested above must stay up there: without this the row substitutions
  // below let the compiler move each load down to its use, one trip to memory after the other.
#pragma unroll
  for (int j = 0; j < KU; j++) asm volatile("" : "+v"(kr[j].x), "+v"(kr[j].y), "+v"(kr[j].z), "+v"(kr[j].w));
#pragma unroll
  for (int st = 0; st < STEPS; st++) asm volatile("" : "+v"(vr[st].x), "+v"(vr[st].y), "+v"(vr[st].z), "+v"(vr[st].w));
  __syncthreads();

  OGM_STAMP(1);
  if constexpr (MULTI) {
    // Several chunks in a row with no workgroup barrier between them: a wave keeps a running maximum per head of
    // its own sixteen rows of every chunk, its lanes their shares of the softmax sum and of the weighted V sum, and
    // the eight waves meet once, after the last chunk.  The next chunk's rows travel while this one is worked on,
    // into the registers this chunk's rows leave: K once the scores' products are formed, V once the weighted
    // sums are.  (They are requested whether or not the workgroup has a next chunk -- past its last one, the
    // cache's last chunk: under a condition the compiler keeps twice the registers.)
    float o[NV], l_lane[NF], m_run[NF];
#pragma unroll
    for (int i = 0; i < NV; i++) o[i] = 0.0f;
#pragma unroll
    for (int i = 0; i < NF; i++) {
      l_lane[i] = 0.0f;
      m_run[i] = -INFINITY;
    }
    uint32_t g0 = 0;        // first head this lane holds
    bool owner = true;      // of several lanes holding the same head, the one that stores
    for (uint32_t chunk_i = c_first; chunk_i < c_end; chunk_i++) {
      const uint32_t p0c = chunk_i * (uint32_t)CHUNK;
      const uint32_t n_here_c = min((uint32_t)CHUNK, n_pos - p0c);
      const bool last_chunk = is_last && chunk_i + 1u == n_chunks;
      const uint32_t cur_c = pos - p0c;
      const uint32_t next = min(chunk_i + 1u, n_chunks - 1u);
      if (chunk_i != c_first) {
#pragma unroll
        for (int j = 0; j < KU; j++) asm volatile("" : "+v"(kr[j].x), "+v"(kr[j].y), "+v"(kr[j].z), "+v"(kr[j].w));
      }
      if (last_chunk && r == cur_c) {
#pragma unroll
        for (int j = 0; j < KU; j++) kr[j] = *(const uint4 *)&kcur[8 * (c + 4 * j)];
      }
      float acc[G];
#pragma unroll
      for (int g = 0; g < G; g++) acc[g] = 0.0f;
#pragma unroll
      for (int j = 0; j < KU; j++) {
        const __half2 *h2 = (const __half2 *)&kr[j];
        float kf[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float2 f = __half22float2(h2[e]);
          kf[2 * e] = f.x;
          kf[2 * e + 1] = f.y;
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
          const float4 qa = *(const float4 *)&qs[g][8 * (c + 4 * j)];
          const float4 qb = *(const float4 *)&qs[g][8 * (c + 4 * j) + 4];
          acc[g] = fmaf(qa.x, kf[0], acc[g]); acc[g] = fmaf(qa.y, kf[1], acc[g]);
          acc[g] = fmaf(qa.z, kf[2], acc[g]); acc[g] = fmaf(qa.w, kf[3], acc[g]);
          acc[g] = fmaf(qb.x, kf[4], acc[g]); acc[g] = fmaf(qb.y, kf[5], acc[g]);
          acc[g] = fmaf(qb.z, kf[6], acc[g]); acc[g] = fmaf(qb.w, kf[7], acc[g]);
        }
      }
      {
        const uint32_t nh_ = min((uint32_t)CHUNK, n_pos - next * (uint32_t)CHUNK);
        const __half *krow_ = kc + (size_t)(next * (uint32_t)CHUNK + min(r, nh_ - 1u)) * kv_dim + kvh * HD;
#pragma unroll
        for (int j = 0; j < KU; j++) kr[j] = *(const uint4 *)(krow_ + 8 * (c + 4 * j));
      }
      // sum over the row's four lanes, as in the one-chunk path below
      g0 = 0;
      owner = true;
      {
        int n = G;
#pragma unroll
        for (int b = 1; b < 4; b <<= 1) {
          const bool up = (lane & b) != 0;
          if (n >= 2) {
            n >>= 1;
#pragma unroll
            for (int i = 0; i < n; i++) {
              float lo = acc[i], hi = acc[n + i];
              asm volatile("" : "+v"(lo), "+v"(hi));   // keeps the selects on values, not on array slots
              acc[i] = (up ? hi : lo) + (b == 1 ? ogm_quad_xor<1>(up ? lo : hi) : ogm_quad_xor<2>(up ? lo : hi));
            }
            g0 += up ? n : 0;
          } else {
            acc[0] += b == 1 ? ogm_quad_xor<1>(acc[0]) : ogm_quad_xor<2>(acc[0]);
            owner = owner && !up;
          }
        }
      }
      const bool valid = r < n_here_c;
#pragma unroll
      for (int i = 0; i < NF; i++) {
        const float sv = valid ? acc[i] * scale : -INFINITY;
        // over the wave's sixteen rows of four lanes, lane by lane of the row
        float m = ogm_row_quads_allreduce(sv, OgmOpMax());
        m = ogm_butterfly_step<16>(m, OgmOpMax());
        m = ogm_butterfly_step<32>(m, OgmOpMax());
        const float m_new = fmaxf(m_run[i], m);
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;   // (a wave may have seen no row yet: everything stays zero)
        const float a = expf(m_run[i] - m_use);
        const float e = valid ? expf(sv - m_use) : 0.0f;
        l_lane[i] = l_lane[i] * a + e;
        m_run[i] = m_new;
        if (owner) sc[g0 + i][r] = e;
        if (lane < 4u && owner) red[1][g0 + i][wave] = a;
      }
      __builtin_amdgcn_wave_barrier();   // the wave's LDS accesses run in order: its weights and factors are there
      {
        float al[G];
#pragma unroll
        for (int g = 0; g < G; g++) al[g] = red[1][g][wave];
#pragma unroll
        for (int i = 0; i < NV; i++) o[i] *= al[i >> 3];
      }
      if (chunk_i != c_first) {
#pragma unroll
        for (int st = 0; st < STEPS; st++) asm volatile("" : "+v"(vr[st].x), "+v"(vr[st].y), "+v"(vr[st].z), "+v"(vr[st].w));
      }
#pragma unroll
      for (int st = 0; st < STEPS; st++) {
        const uint32_t p = st * ROWS + rr;   // past the chunk's end the weight sc is 0
        if (last_chunk && p >= cur_c) vr[st] = *(const uint4 *)&vcur[8u * dc];   // the cache row is not written yet
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
          for (int j = 0; j < 8; j++) o[g * 8 + j] = fmaf(w, vf[j], o[g * 8 + j]);
        }
      }
      {
        const uint32_t nh_ = min((uint32_t)CHUNK, n_pos - next * (uint32_t)CHUNK);
        const __half *vbase_ = vc + (size_t)next * (uint32_t)CHUNK * kv_dim + kvh * HD + 8u * dc;
#pragma unroll
        for (int st = 0; st < STEPS; st++)
          vr[st] = *(const uint4 *)(vbase_ + (size_t)min((uint32_t)(st * ROWS) + rr, nh_ - 1u) * kv_dim);
      }
      __builtin_amdgcn_wave_barrier();   // before the next chunk's weights replace these
    }
    OGM_STAMP(2);
    // ---- the waves meet: each one's maximum and sum per head, and its weighted V sums
#pragma unroll
    for (int i = 0; i < NF; i++) {
      float l = ogm_row_quads_allreduce(l_lane[i], OgmOpAdd());
      l = ogm_butterfly_step<16>(l, OgmOpAdd());
      l = ogm_butterfly_step<32>(l, OgmOpAdd());
      if (lane < 4u && owner) {
        red[0][g0 + i][wave] = m_run[i];
        red[1][g0 + i][wave] = l;
      }
    }
    {
      uint32_t sel = 0;
      int n = NV;
#pragma unroll
      for (int b = TPR; b < 64; b <<= 1) {
        const bool up = (lane & b) != 0;
        n >>= 1;
#pragma unroll
        for (int i = 0; i < n; i++) {
          float lo = o[i], hi = o[n + i];
          asm volatile("" : "+v"(lo), "+v"(hi));   // keeps the selects on values, not on array slots
          const float send = up ? lo : hi;
          o[i] = (up ? hi : lo) + (b == 16 ? ogm_half_xor<16>(send, up) : b == 32 ? ogm_half_xor<32>(send, up)
                                                                                   : __shfl_xor(send, b, 64));
        }
        sel += up ? n : 0;
      }
      float *dst = &osum[wave][0][0] + (sel >> 3) * HD + (sel & 7u) + 8u * dc;
#pragma unroll
      for (int i = 0; i < n; i++) dst[(i >> 3) * HD + (i & 7)] = o[i];
    }
    __syncthreads();
    for (uint32_t i = tid; i < (uint32_t)(G * HD); i += NT) {
      const uint32_t g = i / HD, d = i - g * HD;
      float M = red[0][g][0];
#pragma unroll
      for (int w = 1; w < NW; w++) M = fmaxf(M, red[0][g][w]);
      float t = 0.0f, l = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; w++) {
        const float f = expf(red[0][g][w] - M);   // a wave that saw no row: exp(-inf) = 0
        t += osum[w][g][d] * f;
        l += red[1][g][w] * f;
      }
      if (g < gq) {
        const uint32_t h = hg * gq + g;
        st_one<GROUP != 0>(&part_o[((size_t)h * max_splits + split) * HD + d], t);
        if (d == 0u) {
          st_one<GROUP != 0>(&part_ml[((size_t)h * max_splits + split) * 2], M);
          st_one<GROUP != 0>(&part_ml[((size_t)h * max_splits + split) * 2 + 1], l);
        }
      }
    }
  } else {
  // ---- phase 1: scores
  if (is_last && r == cur) {
#pragma unroll
    for (int j = 0; j < KU; j++) kr[j] = *(const uint4 *)&kcur[8 * (c + 4 * j)];
  }
  float acc[G];
#pragma unroll
  for (int g = 0; g < G; g++) acc[g] = 0.0f;
#pragma unroll
  for (int j = 0; j < KU; j++) {
    const __half2 *h2 = (const __half2 *)&kr[j];
    float kf[8];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float2 f = __half22float2(h2[e]);
      kf[2 * e] = f.x;
      kf[2 * e + 1] = f.y;
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
      const float4 qa = *(const float4 *)&qs[g][8 * (c + 4 * j)];
      const float4 qb = *(const float4 *)&qs[g][8 * (c + 4 * j) + 4];
      acc[g] = fmaf(qa.x, kf[0], acc[g]); acc[g] = fmaf(qa.y, kf[1], acc[g]);
      acc[g] = fmaf(qa.z, kf[2], acc[g]); acc[g] = fmaf(qa.w, kf[3], acc[g]);
      acc[g] = fmaf(qb.x, kf[4], acc[g]); acc[g] = fmaf(qb.y, kf[5], acc[g]);
      acc[g] = fmaf(qb.z, kf[6], acc[g]); acc[g] = fmaf(qb.w, kf[7], acc[g]);
    }
  }
  // sum over the row's four lanes: while a lane holds two or more heads it keeps one half and
  // hands the other to its partner; afterwards plain butterflies
  uint32_t g0 = 0;        // first head this lane holds
  bool owner = true;      // of several lanes holding the same head, the one that stores
  {
    int n = G;
#pragma unroll
    for (int b = 1; b < 4; b <<= 1) {
      const bool up = (lane & b) != 0;
      if (n >= 2) {
        n >>= 1;
#pragma unroll
        for (int i = 0; i < n; i++) {
          float lo = acc[i], hi = acc[n + i];
          asm volatile("" : "+v"(lo), "+v"(hi));   // keeps the selects on values, not on array slots
          acc[i] = (up ? hi : lo) + (b == 1 ? ogm_quad_xor<1>(up ? lo : hi) : ogm_quad_xor<2>(up ? lo : hi));
        }
        g0 += up ? n : 0;
      } else {
        acc[0] += b == 1 ? ogm_quad_xor<1>(acc[0]) : ogm_quad_xor<2>(acc[0]);
        owner = owner && !up;
      }
    }
  }
  const bool valid = r < n_here;
  float sv[NF], mv[NF];
#pragma unroll
  for (int i = 0; i < NF; i++) {
    sv[i] = valid ? acc[i] * scale : -INFINITY;
    // over the wave's sixteen rows of four lanes, lane by lane of the row
    float m = ogm_row_quads_allreduce(sv[i], OgmOpMax());
    m = ogm_butterfly_step<16>(m, OgmOpMax());
    m = ogm_butterfly_step<32>(m, OgmOpMax());
    if (lane < 4u && owner) red[0][g0 + i][wave] = m;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < NF; i++) {
    float m = red[0][g0 + i][0];
#pragma unroll
    for (int w = 1; w < NW; w++) m = fmaxf(m, red[0][g0 + i][w]);
    mv[i] = m;
    const float e = valid ? expf(sv[i] - m) : 0.0f;
    if (owner) sc[g0 + i][r] = e;
    float l = ogm_row_quads_allreduce(e, OgmOpAdd());
    l = ogm_butterfly_step<16>(l, OgmOpAdd());
    l = ogm_butterfly_step<32>(l, OgmOpAdd());
    if (lane < 4u && owner) red[1][g0 + i][wave] = l;
  }
  __syncthreads();
  if (tid < gq) {
    float m = red[0][tid][0], l = red[1][tid][0];
#pragma unroll
    for (int w = 1; w < NW; w++) {
      m = fmaxf(m, red[0][tid][w]);
      l += red[1][tid][w];
    }
    const uint32_t h = hg * gq + tid;
    st_one<GROUP != 0>(&part_ml[((size_t)h * max_splits + split) * 2], m);
    st_one<GROUP != 0>(&part_ml[((size_t)h * max_splits + split) * 2 + 1], l);
  }

  OGM_STAMP(2);
  // ---- phase 2: weighted sum of V rows
  {
    float o[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) o[i] = 0.0f;
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
      const uint32_t p = st * ROWS + rr;   // past the chunk's end the weight sc is 0
      if (is_last && p >= cur) vr[st] = *(const uint4 *)&vcur[8u * dc];   // the cache row is not written yet
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
        for (int j = 0; j < 8; j++) o[g * 8 + j] = fmaf(w, vf[j], o[g * 8 + j]);
      }
    }
    // sum over the rows a wave holds (lanes that differ in the bits above the chunk index): each
    // exchange halves what a lane keeps
    uint32_t sel = 0;
    int n = NV;
#pragma unroll
    for (int b = TPR; b < 64; b <<= 1) {
      const bool up = (lane & b) != 0;
      n >>= 1;
#pragma unroll
      for (int i = 0; i < n; i++) {
        float lo = o[i], hi = o[n + i];
        asm volatile("" : "+v"(lo), "+v"(hi));   // keeps the selects on values, not on array slots
        const float send = up ? lo : hi;
        o[i] = (up ? hi : lo) + (b == 16 ? ogm_half_xor<16>(send, up) : b == 32 ? ogm_half_xor<32>(send, up)
                                                                                 : __shfl_xor(send, b, 64));
      }
      sel += up ? n : 0;
    }
    // o[0 .. n) are the wave's sums of flattened (head, dimension-in-chunk) indices sel .. sel + n
    // (sel is a multiple of n: the head and the dimension of index sel + i split into a lane part
    // and a compile-time part)
    float *dst = &osum[wave][0][0] + (sel >> 3) * HD + (sel & 7u) + 8u * dc;
#pragma unroll
    for (int i = 0; i < n; i++) dst[(i >> 3) * HD + (i & 7)] = o[i];
    __syncthreads();
    for (uint32_t i = tid; i < (uint32_t)(G * HD); i += NT) {
      const uint32_t g = i / HD, d = i - g * HD;
      float t = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; w++) t += osum[w][g][d];
      if (g < gq) st_one<GROUP != 0>(&part_o[((size_t)(hg * gq + g) * max_splits + split) * HD + d], t);
    }
  }
  }   // one chunk

  OGM_STAMP(3);
  // ---- the last workgroup of this K/V head merges the chunks and quantizes
  if constexpr (GROUP != 0) {
    // The partial results were stored device-coherently; once this wave's stores are acknowledged
    // (vmcnt 0) and the workgroup has met, one ticket tells whether every chunk of the head is in.
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    OGM_STAMP(4);
    if (tid == 0) {
      const uint32_t ticket =
          __hip_atomic_fetch_add(&counters[OGM_ATTN_TICKET_STRIDE * hg], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = ticket == n_splits - 1u;
      if (ticket == n_splits - 1u)
        __hip_atomic_store(&counters[OGM_ATTN_TICKET_STRIDE * hg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
    }
    __syncthreads();
    OGM_STAMP(5);
    if (!s_last) return;
    // every thread merges a slice of the chunks of one group of four outputs (one trip to memory
    // up to 8 * NSL chunks), then the slices meet in LDS
    constexpr int NG = G * HD / 4;    // groups of four outputs
    constexpr int NSL = NT / NG;      // slices of chunks
    static_assert(NG * NSL == NT, "the merge assumes whole slices");
    {
      const uint32_t eg = tid % NG, slice = tid / NG;
      const uint32_t el = 4u * eg;
      const AttnPart pt = attn_merge_chunks<true>(part_o, part_ml, hg * G + el / HD, el % HD, slice, NSL, n_splits,
                                                  max_splits, HD);
      mrg[0][tid] = pt.m; mrg[1][tid] = pt.den;
      mrg[2][tid] = pt.o.x; mrg[3][tid] = pt.o.y; mrg[4][tid] = pt.o.z; mrg[5][tid] = pt.o.w;
    }
    __syncthreads();
    OGM_STAMP(6);
    constexpr int RUNS = (NG + 63) / 64;
    for (int run = wave; run < RUNS; run += NW) {
      const uint32_t eg = run * 64u + lane;
      const bool active = eg < (uint32_t)NG;
      const uint32_t e0 = hg * (uint32_t)(G * HD) + 4u * eg;
      float4 ov = make_float4(0.f, 0.f, 0.f, 0.f);
      if (active) {
        float M = mrg[0][eg];   // slice 0 always holds chunk 0
#pragma unroll
        for (int k = 1; k < NSL; k++) M = fmaxf(M, mrg[0][k * NG + eg]);
        float den = 0.0f;
#pragma unroll
        for (int k = 0; k < NSL; k++) {
          const float f = expf(mrg[0][k * NG + eg] - M);   // a slice without chunks has m = -inf: f = 0
          den += f * mrg[1][k * NG + eg];
          ov.x += f * mrg[2][k * NG + eg]; ov.y += f * mrg[3][k * NG + eg];
          ov.z += f * mrg[4][k * NG + eg]; ov.w += f * mrg[5][k * NG + eg];
        }
        ov.x /= den; ov.y /= den; ov.z /= den; ov.w /= den;
        if (attn_out) *(float4 *)(attn_out + e0) = ov;
      }
      ogm_quantize_store<GROUP>(ov, e0, active, lane, act.q, act.d, act.sums, act.bsum, act.bs16);
    }
    OGM_STAMP(7);
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
    const AttnPart pt = attn_merge_chunks<false>(part_o, part_ml, e0 / head_dim, e0 % head_dim, 0u, 1u, n_splits,
                                                 max_splits, head_dim);
    o = make_float4(pt.o.x / pt.den, pt.o.y / pt.den, pt.o.z / pt.den, pt.o.w / pt.den);
    if (attn_out) *(float4 *)(attn_out + e0) = o;
  }
  ogm_quantize_store<GROUP>(o, e0, active, lane, act.q, act.d, act.sums, act.bsum, act.bs16);
}

uint32_t ogm_attn_head_parts(uint32_t heads_per_kv) {
  if (heads_per_kv == 0u || heads_per_kv > 64u) return 0u;
  const uint32_t parts = (heads_per_kv + 7u) / 8u;
  return heads_per_kv % parts == 0u ? parts : 0u;
}

hipError_t ogm_launch_attn_decode(const float *q, const float *k_new, const float *v_new, const void *cs,
                                  uint32_t rope_dim, const OgmAttnPre &pre, void *k_cache_layer,
                                  void *v_cache_layer, uint32_t pos, uint32_t max_splits, uint32_t n_head,
                                  uint32_t n_head_kv, uint32_t head_dim, float scale, float *part_o,
                                  float *part_ml, uint32_t *counters, int mode, float *attn_out, OgmActDev act,
                                  hipStream_t stream, uint32_t chunk, uint32_t chunks_per_wg) {
  if (n_head_kv == 0 || n_head % n_head_kv != 0) return hipErrorInvalidValue;
  if (rope_dim > head_dim || rope_dim % 2u != 0) return hipErrorInvalidValue;
  // Cache positions per workgroup: 128; 64 only for short contexts.  The kernel is a chain of
  // latencies (cache loads 2.1 us, scores 1.5, V sum 1.5, hand-over of the partial results 0.9,
  // merge 2.8, quantizer 1.0 at 2048 positions) of which only the two middle ones shrink with the
  // chunk, while the merge grows with the number of chunks: measured on MI355X with eight K/V heads,
  // 64 against 128 positions per workgroup take 8.4 against 8.9 us at 512 cached positions but 13.6
  // against 10.7 at 2048 and 20.5 against 14.1 at 4096.
  if (chunk == 0) chunk = (chunks_per_wg <= 1u && (pos / 64u + 1u) * n_head_kv <= 96u) ? 64u : 128u;
  if (chunk != 64u && chunk != 128u) return hipErrorInvalidValue;
  const uint32_t n_chunks = pos / chunk + 1u;
  const uint32_t n = n_head * head_dim;
  if (n % 32u != 0) return hipErrorInvalidValue;
  // more than eight query heads per K/V head: in equal parts of at most eight, a workgroup each
  const uint32_t parts = ogm_attn_head_parts(n_head / n_head_kv);
  if (parts == 0u) return hipErrorInvalidValue;
  const uint32_t gq = n_head / n_head_kv / parts;
  // Chunks a workgroup takes in a row (chunks of 128 only): one while the launch has fewer workgroups than the
  // device has compute units, then as many as keep it near OGM_ATTN_SUB_TARGET workgroups, at most
  // OGM_ATTN_SUB_MAX.  A workgroup pays for the rotation of q, the hand-over of its partial results and its
  // ticket once, its waves work through their chunks without meeting, and the merge at the end has that many
  // fewer partial results to read.  Measured on MI355X, 8B shapes (eight K/V heads), ms per token at 1 / 2 / 4 / 8 /
  // 16 chunks a workgroup: 2048 positions 1.80 / 1.86 / 1.97 / 2.18 / 2.60; 4096: 1.95 / 1.90 / 2.00 / 2.21 / 2.63;
  // 8192: 2.08 / 1.99 / 2.01 / 2.20 / 2.63; 16384: 2.38 / 2.34 / 2.19 / 2.27 / 2.65; 32768: 3.02 / 2.87 / 2.66 /
  // 2.60 / 2.84.
  uint32_t n_sub = chunks_per_wg;
  if (n_sub == 0u) {
    const uint32_t wgs = n_chunks * n_head_kv * parts;
    n_sub = (wgs + OGM_ATTN_SUB_TARGET - 1u) / OGM_ATTN_SUB_TARGET;
    if (wgs >= 256u && n_sub < 2u) n_sub = 2u;
    if (n_sub > OGM_ATTN_SUB_MAX) n_sub = OGM_ATTN_SUB_MAX;
  }
  if (n_sub == 0u || chunk != 128u) n_sub = 1u;   // (chunks of 64 are for contexts of a few hundred positions)
  if (n_sub > n_chunks) n_sub = n_chunks;
  const uint32_t n_splits = (n_chunks + n_sub - 1u) / n_sub;
  if (n_splits > max_splits) return hipErrorInvalidValue;
  const dim3 grid(n_head_kv * parts, n_splits);
  const uint32_t G = gq <= 2u ? gq : (gq <= 4u ? 4u : 8u);   // head slots of the kernel
  const uint32_t group = mode == 0 ? 32u : 256u;
  // the merge rides in the attention kernel when every head slot is a head and a K/V head's
  // outputs are whole quantizer groups
  const uint32_t fused = (G == gq && (G * head_dim) % group == 0) ? group : 0u;
#define OGM_ATTN_LAUNCH_C(HD_, G_, GR_, CH_, MULTI_)                                                    \
  hipLaunchKernelGGL((ogm_attn_kernel<HD_, G_, GR_, false, CH_, MULTI_>), grid, dim3(4 * CH_), 0, stream, q, k_new, \
                     v_new, (const float2 *)cs, rope_dim / 2u, pre, gq, (__half *)k_cache_layer,        \
                     (__half *)v_cache_layer, pos, max_splits, n_head_kv, scale, part_o, part_ml, \
                     counters, attn_out, act, n_sub)
#define OGM_ATTN_LAUNCH(HD_, G_, GR_)                    \
  do {                                                   \
    if (chunk == 64u) OGM_ATTN_LAUNCH_C(HD_, G_, GR_, 64, false); \
    else if (n_sub == 1u) OGM_ATTN_LAUNCH_C(HD_, G_, GR_, 128, false); \
    else OGM_ATTN_LAUNCH_C(HD_, G_, GR_, 128, true);     \
  } while (0)
#define OGM_ATTN_GROUPS(HD_, G_)                                \
  do {                                                          \
    if (fused == 32u) OGM_ATTN_LAUNCH(HD_, G_, 32);             \
    else if (fused == 256u) OGM_ATTN_LAUNCH(HD_, G_, 256);      \
    else OGM_ATTN_LAUNCH(HD_, G_, 0);                           \
  } while (0)
  if (head_dim == 128 && G == 1) OGM_ATTN_GROUPS(128, 1);
  else if (head_dim == 128 && G == 2) OGM_ATTN_GROUPS(128, 2);
  else if (head_dim == 128 && G == 4) OGM_ATTN_GROUPS(128, 4);
  else if (head_dim == 128 && G == 8) OGM_ATTN_GROUPS(128, 8);
  else if (head_dim == 64 && G == 1) OGM_ATTN_GROUPS(64, 1);
  else if (head_dim == 64 && G == 2) OGM_ATTN_GROUPS(64, 2);
  else if (head_dim == 64 && G == 4) OGM_ATTN_GROUPS(64, 4);
  else if (head_dim == 64 && G == 8) OGM_ATTN_GROUPS(64, 8);
  else return hipErrorInvalidValue;
#undef OGM_ATTN_GROUPS
#undef OGM_ATTN_LAUNCH
#undef OGM_ATTN_LAUNCH_C
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || fused != 0u) return e;
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
  // blockIdx.y: the row of a batch.  (With a multiple of eight runs a row, the eight rows that share a line of the
  // operand chunks are written from one XCD without further ado: workgroup (run, row) runs on XCD run % 8.)
  const uint32_t r = blockIdx.y, run = blockIdx.x;
  {
    const size_t row = (size_t)r * n;
    gate += row;
    up += row;
    if (h) h += row;
    act.q += row;
    act.d += (size_t)r * (n / GROUP);
    act.sums += (size_t)r * (n / 16u);
    act.bsum += (size_t)r * (n / 32u);
    if (act.bs16) act.bs16 += (size_t)r * (n / 16u);
    act.xt = ogm_xt_row(act.xt, r, n);
  }
  ogm_swiglu_quant_run<GROUP, false>(gate, up, n, h, act, run, lane);
}

hipError_t ogm_launch_swiglu_quant(int mode, const float *gate, const float *up, uint32_t n, float *h,
                                   OgmActDev act, hipStream_t stream, uint32_t n_rows) {
  if (n == 0 || n % 32u != 0 || n_rows == 0 || n_rows > 65535u) return hipErrorInvalidValue;
  const dim3 grid((n + 255u) / 256u, n_rows);
  if (mode == 0)
    hipLaunchKernelGGL(ogm_swiglu_quant_kernel<32>, grid, dim3(64), 0, stream, gate, up, n, h, act);
  else
    hipLaunchKernelGGL(ogm_swiglu_quant_kernel<256>, grid, dim3(64), 0, stream, gate, up, n, h, act);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// argmax as sampling.rs:336-343 takes it: Iterator::max_by over f32::total_cmp, which returns the
// last of several equal maxima.  total_cmp orders -NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN; the
// key below is the usual monotone map of that order onto signed integers.

__device__ __forceinline__ int32_t argmax_key(float v) {
  const int32_t k = __float_as_int(v);
  return k ^ ((k >> 31) & 0x7FFFFFFF);
}
__device__ __forceinline__ bool argmax_better(int32_t k, uint32_t i, int32_t bk, uint32_t bi) {
  return k > bk || (k == bk && i > bi);
}

__global__ __launch_bounds__(256) void ogm_argmax_kernel(const float *__restrict__ x, uint32_t n,
                                                         uint32_t *__restrict__ scratch, uint32_t *__restrict__ out,
                                                         int final_stage) {
  __shared__ int32_t sv[256];
  __shared__ uint32_t si[256];
  const uint32_t tid = threadIdx.x;
  int32_t bk = INT32_MIN;   // the key of the smallest value there is
  uint32_t bi = 0;
  if (!final_stage) {
    for (uint32_t i = blockIdx.x * 256u + tid; i < n; i += gridDim.x * 256u) {
      const int32_t k = argmax_key(x[i]);
      if (argmax_better(k, i, bk, bi)) { bk = k; bi = i; }
    }
  } else {
    // scratch: 256 keys then 256 indices, one per first-stage workgroup
    if (tid < n) { bk = (int32_t)scratch[tid]; bi = scratch[256 + tid]; }
  }
  sv[tid] = bk;
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
      scratch[blockIdx.x] = (uint32_t)sv[0];
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
  if (i < n) dst[i] = ogm_f16_sat(src[i]);
}

hipError_t ogm_launch_f32_to_f16(const float *src, void *dst, size_t n, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(ogm_f32_to_f16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, src,
                     (__half *)dst, n);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// one row of a quantized matrix as f32: the embedding lookup (LlamaModel::run_layers,
// llama.rs:609-614, over dequantize_q8_0 / _q4_0 / _q5_0 / _q5_1 / _iq4_nl / _iq4_xs / _q2_k / _q3_k / _q4_k /
// _q5_k / _q6_k, quant.rs:537-636, 639-649, 666-827, 841-871, 1320-1375),
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
  // blockIdx.y: the n-th row asked for (row + n, or row_dev[n]) into the n-th output row
  row = row_dev ? row_dev[blockIdx.y] : row + blockIdx.y;
  out += (size_t)blockIdx.y * in_dim;
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
  } else if (ggml_type == OGM_Q4_0 || ggml_type == OGM_Q5_0 || ggml_type == OGM_IQ4_NL) {
    // one piece of nibbles (elements 0..16 low, 16..32 high); the tail holds d, and qh for Q5_0
    const uint8_t *tail = tb + 1024u + lane * l.tail_bytes;
    const float d = dq_f16(tail);
    const uint32_t byte = piece_byte(j & 15u);
    const uint32_t nib = j < 16 ? (byte & 0xFu) : (byte >> 4);
    if (ggml_type == OGM_IQ4_NL) {
      const int8_t levels[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
      v = d * (float)levels[nib];
    } else if (ggml_type == OGM_Q4_0) {
      v = (float)((int)nib - 8) * d;
    } else {
      const uint32_t qh = tail[2] | (tail[3] << 8) | (tail[4] << 16) | ((uint32_t)tail[5] << 24);
      v = (float)((int)(nib | (((qh >> j) & 1u) << 4)) - 16) * d;
    }
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
  } else if (ggml_type == OGM_Q5_K) {
    const uint8_t *hd = tb + lane * 16u;   // piece 0: d, dmin, scales; then qh[32], then qs
    const float d = dq_f16(hd), dmin = dq_f16(hd + 2);
    const uint32_t g4 = j >> 6, hi = (j >> 5) & 1u, li = j & 31u;
    const uint32_t is = 2u * g4 + hi;
    const uint8_t *q = hd + 4;
    uint32_t sc, m;
    if (is < 4) {
      sc = q[is] & 63u;
      m = q[is + 4] & 63u;
    } else {
      sc = (q[is + 4] & 0xFu) | ((q[is - 4] >> 6) << 4);
      m = (q[is + 4] >> 4) | ((q[is] >> 6) << 4);
    }
    const uint32_t byte = piece_byte(48u + 32u * g4 + li);
    const uint32_t high = (piece_byte(16u + li) >> is) & 1u;
    const int qv = (int)(hi ? (byte >> 4) : (byte & 0xFu)) + (high ? 16 : 0);
    const float d1 = d * (float)sc, mm = dmin * (float)m;
    v = d1 * (float)qv - mm;
  } else if (ggml_type == OGM_Q3_K) {
    // hmask[32] | qs[64] | scales[12] | d, all inside the pieces (quant.rs:841-871)
    const uint32_t p = j >> 5, jj = j & 31u, g = j >> 4;
    const uint32_t lo = (piece_byte(32u + 32u * (p >> 2) + jj) >> (2u * (p & 3u))) & 3u;
    const int qv = (int)lo - (((piece_byte(jj) >> p) & 1u) ? 0 : 4);
    const uint32_t lb = piece_byte(96u + (g & 7u));
    const uint32_t low = g < 8 ? (lb & 0xFu) : (lb >> 4);
    const uint32_t high = (piece_byte(104u + (g & 3u)) >> (2u * (g >> 2))) & 3u;
    const int sc = (int)(low | (high << 4)) - 32;
    const float d = __half2float(__ushort_as_half((unsigned short)(piece_byte(108u) | (piece_byte(109u) << 8))));
    const float dl = d * (float)sc;
    v = dl * (float)qv;
  } else if (ggml_type == OGM_Q5_1) {
    // one piece of nibbles; the tail holds d, m and qh (quant.rs:615-636): value = q * d + m
    const uint8_t *tail = tb + 1024u + lane * 8u;
    const float d = dq_f16(tail), mm = dq_f16(tail + 2);
    const uint32_t qh = tail[4] | (tail[5] << 8) | (tail[6] << 16) | ((uint32_t)tail[7] << 24);
    const uint32_t byte = piece_byte(j & 15u);
    const uint32_t nib = j < 16 ? (byte & 0xFu) : (byte >> 4);
    v = (float)(nib | (((qh >> j) & 1u) << 4)) * d + mm;
  } else if (ggml_type == OGM_IQ4_XS) {
    // d | scales_h | scales_l[4] | qs[128], all inside the pieces (quant.rs:1350-1375)
    const int8_t levels[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
    const uint32_t ib = j >> 5, jj = j & 31u;
    const float d = __half2float(__ushort_as_half((unsigned short)(piece_byte(0u) | (piece_byte(1u) << 8))));
    const uint32_t sh = piece_byte(2u) | (piece_byte(3u) << 8);
    const uint32_t low = (piece_byte(4u + (ib >> 1)) >> (4u * (ib & 1u))) & 0xFu;
    const int ls = (int)(low | (((sh >> (2u * ib)) & 3u) << 4)) - 32;
    const uint32_t byte = piece_byte(8u + 16u * ib + (jj & 15u));
    const float dl = d * (float)ls;
    v = dl * (float)levels[jj < 16 ? (byte & 0xFu) : (byte >> 4)];
  } else if (ggml_type == OGM_Q2_K) {
    // scales[16] | qs[64] in the pieces, d and dmin in the tail (quant.rs:798-827)
    const uint8_t *tail = tb + l.pieces * 1024u + lane * 4u;
    const float d = dq_f16(tail), dmin = dq_f16(tail + 2);
    const uint32_t p = j >> 5, jj = j & 31u, g = j >> 4;
    const uint32_t sc = piece_byte(g);
    const uint32_t qv = (piece_byte(16u + 32u * (p >> 2) + jj) >> (2u * (p & 3u))) & 3u;
    const float dl = d * (float)(sc & 0xFu), ml = dmin * (float)(sc >> 4);
    v = dl * (float)qv - ml;
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
                                  uint32_t row, const uint32_t *row_dev, uint32_t n_rows, float *out,
                                  hipStream_t stream) {
  OgmLayout l;
  if (!ogm_layout_for(ggml_type, &l) || in_dim == 0 || in_dim % l.block_elems != 0 || out_dim == 0)
    return hipErrorInvalidValue;
  if (n_rows == 0 || n_rows > 65535u) return hipErrorInvalidValue;
  hipLaunchKernelGGL(ogm_dequant_row_kernel, dim3((in_dim + 255u) / 256u, n_rows), dim3(256), 0, stream, wt,
                     ggml_type, in_dim, out_dim, row, row_dev, out);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// prefill: the same layer over a batch of tokens.  The matmuls are GEMMs that quantize their
// own input, so these kernels leave plain f32 rows.

// One wave per (token, head of q | k | v): bias, per-head norm and RoPE as the decode kernel's
// first phase; q is rewritten in place, k and v go to their cache rows as f16.
template <int HD>
__global__ __launch_bounds__(256) void ogm_qkv_pre_kernel(float *__restrict__ q, const float *__restrict__ k,
                                                          const float *__restrict__ v,
                                                          const float2 *__restrict__ cs, uint32_t rope_half,
                                                          OgmAttnPre pre, uint32_t n_head, uint32_t n_head_kv,
                                                          __half *__restrict__ kc, __half *__restrict__ vc,
                                                          uint32_t pos0) {
  constexpr int PPL = (HD / 2 + 63) / 64;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t u = blockIdx.x * 4u + (threadIdx.x >> 6), tok = blockIdx.y;
  if (u >= n_head + 2u * n_head_kv) return;
  const bool is_q = u < n_head, is_v = u >= n_head + n_head_kv;
  const uint32_t head = is_q ? u : (is_v ? u - n_head - n_head_kv : u - n_head);
  const size_t kv_dim = (size_t)n_head_kv * HD;
  const size_t row = (size_t)head * HD;   // within a token's vector and within the bias
  float *qrow = q + (size_t)tok * n_head * HD + row;
  const float *src = is_q ? qrow : (is_v ? v : k) + (size_t)tok * kv_dim + row;
  const float *bias = is_q ? pre.q_bias : is_v ? pre.v_bias : pre.k_bias;
  const float *nw = is_q ? pre.q_norm : is_v ? nullptr : pre.k_norm;
  cs += (size_t)tok * rope_half;
  float a[PPL], b[PPL];
  uint32_t ia[PPL], ib[PPL];
  float ss = 0.0f;
#pragma unroll
  for (int j = 0; j < PPL; j++) {
    const uint32_t p = lane + 64u * j;
    const bool have = p < (uint32_t)(HD / 2);
    const bool split_pair = pre.neox != 0u && !is_v && p < rope_half;
    ia[j] = split_pair ? p : 2u * p;
    ib[j] = split_pair ? p + rope_half : 2u * p + 1u;
    a[j] = have ? src[ia[j]] : 0.0f;
    b[j] = have ? src[ib[j]] : 0.0f;
    if (bias != nullptr && have) {
      a[j] += bias[row + ia[j]];
      b[j] += bias[row + ib[j]];
    }
    ss += a[j] * a[j] + b[j] * b[j];
  }
  if (nw != nullptr) {
    ss = ogm_wave_sum(ss);
    const float sc_n = 1.0f / sqrtf(ss / (float)HD + pre.eps);
#pragma unroll
    for (int j = 0; j < PPL; j++) {
      const uint32_t p = lane + 64u * j;
      if (p < (uint32_t)(HD / 2)) {
        a[j] = a[j] * sc_n * nw[ia[j]];
        b[j] = b[j] * sc_n * nw[ib[j]];
      }
    }
  }
#pragma unroll
  for (int j = 0; j < PPL; j++) {
    const uint32_t p = lane + 64u * j;
    if (p >= (uint32_t)(HD / 2)) continue;
    float2 ab = make_float2(a[j], b[j]);
    if (!is_v && p < rope_half) ab = rope_pair(ab, cs[p]);
    if (is_q) {
      qrow[ia[j]] = ab.x;
      qrow[ib[j]] = ab.y;
    } else {
      __half *cache = (is_v ? vc : kc) + (size_t)(pos0 + tok) * kv_dim + row;
      cache[ia[j]] = ogm_f16_sat(ab.x);
      cache[ib[j]] = ogm_f16_sat(ab.y);
    }
  }
}

hipError_t ogm_launch_qkv_pre(float *q, const float *k, const float *v, const void *cs, uint32_t rope_dim,
                              const OgmAttnPre &pre, uint32_t n_head, uint32_t n_head_kv, uint32_t head_dim,
                              void *k_cache_layer, void *v_cache_layer, uint32_t pos0, uint32_t n_tokens,
                              hipStream_t stream) {
  if (rope_dim > head_dim || rope_dim % 2u != 0 || n_tokens == 0 || n_tokens > 65535u) return hipErrorInvalidValue;
  const dim3 grid((n_head + 2u * n_head_kv + 3u) / 4u, n_tokens);
  if (head_dim == 128)
    hipLaunchKernelGGL(ogm_qkv_pre_kernel<128>, grid, dim3(256), 0, stream, q, k, v, (const float2 *)cs,
                       rope_dim / 2u, pre, n_head, n_head_kv, (__half *)k_cache_layer, (__half *)v_cache_layer, pos0);
  else if (head_dim == 64)
    hipLaunchKernelGGL(ogm_qkv_pre_kernel<64>, grid, dim3(256), 0, stream, q, k, v, (const float2 *)cs,
                       rope_dim / 2u, pre, n_head, n_head_kv, (__half *)k_cache_layer, (__half *)v_cache_layer, pos0);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

// The chunks of every (token, head) merged: one wave per 256 outputs of a token.  GROUP != 0: the wave also
// quantizes its run for the next matmul (per 32 or per 256) into the token's row of `act`; n is then a multiple of
// GROUP and every lane of the run takes part.
template <int GROUP>
__global__ __launch_bounds__(64) void ogm_attn_combine_rows_kernel(const float *__restrict__ part_o,
                                                                   const float *__restrict__ part_ml, uint32_t pos0,
                                                                   uint32_t max_splits, uint32_t n, uint32_t head_dim,
                                                                   float *__restrict__ attn_out, OgmActDev act,
                                                                   uint32_t n_sub) {
  const uint32_t lane = threadIdx.x, tok = blockIdx.y;
  const uint32_t e0 = blockIdx.x * 256u + 4u * lane;
  const bool active = e0 < n;
  if (GROUP == 0 && !active) return;
  const uint32_t n_head = n / head_dim;
  const uint32_t n_splits = ((pos0 + tok) / OGM_ATTN_CHUNK + n_sub) / n_sub;   // workgroups of n_sub chunks each
  float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
  if (active) {
    const AttnPart pt = attn_merge_chunks<false>(part_o + (size_t)tok * n_head * max_splits * head_dim,
                                                 part_ml + (size_t)tok * n_head * max_splits * 2, e0 / head_dim,
                                                 e0 % head_dim, 0u, 1u, n_splits, max_splits, head_dim);
    o = make_float4(pt.o.x / pt.den, pt.o.y / pt.den, pt.o.z / pt.den, pt.o.w / pt.den);
    if (attn_out) *(float4 *)(attn_out + (size_t)tok * n + e0) = o;
  }
  if constexpr (GROUP != 0) {
    act.q += (size_t)tok * n;
    act.d += (size_t)tok * (n / GROUP);
    act.sums += (size_t)tok * (n / 16u);
    act.bsum += (size_t)tok * (n / 32u);
    if (act.bs16) act.bs16 += (size_t)tok * (n / 16u);
    ogm_quantize_store<GROUP>(o, e0, active, lane, act.q, act.d, act.sums, act.bsum, act.bs16);
  }
}

hipError_t ogm_launch_attn_prefill(const float *q, void *k_cache_layer, void *v_cache_layer, uint32_t pos0,
                                   uint32_t n_tokens, uint32_t max_splits, uint32_t n_head, uint32_t n_head_kv,
                                   uint32_t head_dim, float scale, float *part_o, float *part_ml, float *attn_out,
                                   hipStream_t stream, int quant_mode, OgmActDev act, uint32_t chunks_per_wg) {
  if (n_head_kv == 0 || n_head % n_head_kv != 0 || n_tokens == 0 || n_tokens > 65535u) return hipErrorInvalidValue;
  if (quant_mode >= 0 && (n_head * head_dim) % (quant_mode == 0 ? 32u : 256u) != 0) return hipErrorInvalidValue;
  if (quant_mode < 0 && attn_out == nullptr) return hipErrorInvalidValue;
  const uint32_t n_splits = (pos0 + n_tokens - 1u) / OGM_ATTN_CHUNK + 1u;   // of the last token
  if (n_splits > max_splits) return hipErrorInvalidValue;
  const uint32_t n = n_head * head_dim;
  if (n % 4u != 0) return hipErrorInvalidValue;
  const uint32_t parts = ogm_attn_head_parts(n_head / n_head_kv);
  if (parts == 0u) return hipErrorInvalidValue;
  const uint32_t gq = n_head / n_head_kv / parts;
  const uint32_t G = gq <= 2u ? gq : (gq <= 4u ? 4u : 8u);
  // Chunks a workgroup takes in a row, as in the decode step (ogm_launch_attn_decode), here to keep the launch near
  // OGM_ATTN_SUB_TARGET_ROWS workgroups: the time of such a batch over a long context is its workgroups' own, not the
  // memory's (the tokens' workgroups of a chunk find its rows in L2).
  uint32_t n_sub = chunks_per_wg;
  if (n_sub == 0u) {
    const uint64_t wgs = (uint64_t)n_splits * n_head_kv * parts * n_tokens;
    n_sub = (uint32_t)((wgs + OGM_ATTN_SUB_TARGET_ROWS - 1u) / OGM_ATTN_SUB_TARGET_ROWS);
    if (n_sub > OGM_ATTN_SUB_MAX) n_sub = OGM_ATTN_SUB_MAX;
  }
  if (n_sub > n_splits) n_sub = n_splits;
  const uint32_t n_wg_z = (n_splits + n_sub - 1u) / n_sub;
  if (n_wg_z > 65535u) return hipErrorInvalidValue;
  const dim3 grid(n_head_kv * parts, n_tokens, n_wg_z);
  const OgmAttnPre none{nullptr, nullptr, nullptr, nullptr, nullptr, 0.0f, 0u};
  const OgmActDev no_act{};
#define OGM_ATTN_PREFILL_M(HD_, G_, MULTI_)                                                                 \
  hipLaunchKernelGGL((ogm_attn_kernel<HD_, G_, 0, true, 128, MULTI_>), grid, dim3(512), 0, stream, q,       \
                     (const float *)nullptr, (const float *)nullptr, (const float2 *)nullptr, 0u, none, gq, \
                     (__half *)k_cache_layer, (__half *)v_cache_layer, pos0, max_splits, n_head_kv, scale,  \
                     part_o, part_ml, (uint32_t *)nullptr, (float *)nullptr, no_act, n_sub)
#define OGM_ATTN_PREFILL(HD_, G_)                  \
  do {                                             \
    if (n_sub == 1u) OGM_ATTN_PREFILL_M(HD_, G_, false); \
    else OGM_ATTN_PREFILL_M(HD_, G_, true);        \
  } while (0)
  if (head_dim == 128 && G == 1) OGM_ATTN_PREFILL(128, 1);
  else if (head_dim == 128 && G == 2) OGM_ATTN_PREFILL(128, 2);
  else if (head_dim == 128 && G == 4) OGM_ATTN_PREFILL(128, 4);
  else if (head_dim == 128 && G == 8) OGM_ATTN_PREFILL(128, 8);
  else if (head_dim == 64 && G == 1) OGM_ATTN_PREFILL(64, 1);
  else if (head_dim == 64 && G == 2) OGM_ATTN_PREFILL(64, 2);
  else if (head_dim == 64 && G == 4) OGM_ATTN_PREFILL(64, 4);
  else if (head_dim == 64 && G == 8) OGM_ATTN_PREFILL(64, 8);
  else return hipErrorInvalidValue;
#undef OGM_ATTN_PREFILL
#undef OGM_ATTN_PREFILL_M
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const dim3 cgrid((n + 255u) / 256u, n_tokens);
  if (quant_mode < 0)
    hipLaunchKernelGGL(ogm_attn_combine_rows_kernel<0>, cgrid, dim3(64), 0, stream, part_o, part_ml, pos0, max_splits, n,
                       head_dim, attn_out, no_act, n_sub);
  else if (quant_mode == 0)
    hipLaunchKernelGGL(ogm_attn_combine_rows_kernel<32>, cgrid, dim3(64), 0, stream, part_o, part_ml, pos0, max_splits, n,
                       head_dim, attn_out, act, n_sub);
  else
    hipLaunchKernelGGL(ogm_attn_combine_rows_kernel<256>, cgrid, dim3(64), 0, stream, part_o, part_ml, pos0, max_splits,
                       n, head_dim, attn_out, act, n_sub);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// Prefill attention on the matrix cores.  Workgroup (query tile of 32 tokens, K/V head, group of
// four query heads), eight waves: wave w takes query head 4 z + w % 4 of the K/V head and walks
// every second cache tile of 64 positions (the even ones for waves 0-3, the odd ones for waves 4-7)
// up to the tile's last query (causal), with a running maximum and sum per query (the softmax of
// llama.rs's attention, tensor.rs softmax_rows, regrouped); at the end the two halves' partial
// softmaxes meet in LDS.  A launch takes as long as its longest workgroup -- the last query tile,
// whose walk is the whole context (one workgroup alone on a compute unit: 3.0 us per cache tile) --
// so the walk is what the second set of waves halves.
//
//   scores^T = K . Q^T    A = K rows from LDS (16 bytes of a row are 8 consecutive dimensions),
//                         B = Q^T from registers; the result has one query per lane and 16
//                         positions per 32 x 32 block in its registers, so maximum and sum of a
//                         query are in-lane reductions plus one exchange between the lane halves
//   out^T += V^T . P^T    A = V^T from LDS, B = P^T: exactly the registers the scores came in
//
// V is transposed on its way into LDS (8 x 8 blocks in registers, byte permutes); its columns are
// stored in the order in which a lane half holds the positions (within each 16: 0-3, 8-11, 4-7,
// 12-15), so that an operand is 16 contiguous bytes.  K, V are f16 in the cache and exact in the
// products; q and the probabilities are f32 and go in as two f16 terms each (value = hi + lo),
// which keeps 22 bits of them: the results differ from f32 arithmetic by f32 rounding only.

typedef _Float16 ah8 __attribute__((ext_vector_type(8)));
typedef float af16 __attribute__((ext_vector_type(16)));

#define AM_KT 64u                      // positions per tile
#define AM_VROW (AM_KT * 2u + 16u)     // bytes of a row of V^T in LDS

__device__ __forceinline__ void am_split(float v, _Float16 &hi, _Float16 &lo) {
  hi = (_Float16)v;
  lo = (_Float16)(v - (float)hi);
}

template <int HD>
__global__ __launch_bounds__(512, 2) void ogm_attn_prefill_mfma_kernel(const float *__restrict__ q,
                                                                    const __half *__restrict__ kc,
                                                                    const __half *__restrict__ vc, uint32_t pos0,
                                                                    uint32_t n_tokens, uint32_t n_head_kv, uint32_t gq,
                                                                    float scale, float *__restrict__ attn_out) {
  constexpr uint32_t KROW = HD * 2u + 16u;   // bytes of a K row in LDS
  constexpr int NS = HD / 16;                // k steps of a score block
  constexpr int NDB = HD / 32;               // 32-dimension blocks of the output
  constexpr uint32_t PPR = HD / 8;           // 16-byte pieces per cache row
  constexpr int NK = (int)(AM_KT * PPR / 128u);   // pieces a K-copying thread moves per tile (8 or 4)
  constexpr uint32_t K_BYTES = AM_KT * KROW, V_BYTES = HD * AM_VROW;
  extern __shared__ __align__(16) uint8_t am_lds[];   // per half: a K tile, then a V^T tile
  const uint32_t half = threadIdx.x >> 8;             // which of the two tiles of an iteration
  uint8_t *const k_l = am_lds + half * (K_BYTES + V_BYTES);
  uint8_t *const vt_l = k_l + K_BYTES;

  const uint32_t tid = threadIdx.x & 255u, lane = tid & 63u, wave = tid >> 6;   // within the half
  const uint32_t l32 = lane & 31u, lh = lane >> 5;
  // Long tiles first, across the whole launch: workgroups start in the grid's order (x fastest), and a long tile
  // that starts late is what the launch then waits for (2048 tokens, 8 K/V heads, with the tiles on x: 165 us)
  const uint32_t qt = gridDim.y - 1u - blockIdx.y;
  const uint32_t kvh = blockIdx.x % n_head_kv, g = 4u * (blockIdx.x / n_head_kv) + wave;
  const bool live = g < gq;
  const uint32_t n_head = n_head_kv * gq, kv_dim = n_head_kv * HD;
  const uint32_t tok = min(32u * qt + l32, n_tokens - 1u);   // this lane's query (clamped: computed, not stored)
  const uint32_t q_abs = pos0 + tok;
  const uint32_t last_pos = pos0 + min(32u * qt + 31u, n_tokens - 1u);
  const uint32_t n_tiles = last_pos / AM_KT + 1u;
  const uint32_t max_row = pos0 + n_tokens - 1u;   // last cache row that holds data

  // q of this lane's query, head g: for k step s the dimensions 16 s + 8 lh + 0..7, as hi + lo.  A
  // row whose largest |q| is 2^14 or more is first scaled down by a power of two (the f16 terms
  // would overflow at 65504) and its scores scaled back up with `scale`: exact both ways.
  ah8 qh[NS], ql[NS];
  float scale_q = scale;
  {
    const float *qp = q + ((size_t)tok * n_head + (size_t)kvh * gq + (live ? g : 0u)) * HD + 8u * lh;
    float4 qa[NS], qb[NS];
    float amax = 0.0f;
#pragma unroll
    for (int s = 0; s < NS; s++) {
      qa[s] = *(const float4 *)(qp + 16 * s);
      qb[s] = *(const float4 *)(qp + 16 * s + 4);
      amax = fmaxf(amax, fmaxf(fmaxf(fabsf(qa[s].x), fabsf(qa[s].y)), fmaxf(fabsf(qa[s].z), fabsf(qa[s].w))));
      amax = fmaxf(amax, fmaxf(fmaxf(fabsf(qb[s].x), fabsf(qb[s].y)), fmaxf(fabsf(qb[s].z), fabsf(qb[s].w))));
    }
    amax = ogm_butterfly_step<32>(amax, OgmOpMax());   // the row's other dimensions are in the other lane half
    float down = 1.0f;
    if (amax >= 16384.0f && amax < INFINITY) {
      const int k = (int)((__float_as_uint(amax) >> 23) & 0xFFu) - 127 - 13;   // amax * 2^-k in [2^13, 2^14)
      down = __uint_as_float((uint32_t)(127 - k) << 23);
      scale_q = scale * __uint_as_float((uint32_t)(127 + k) << 23);
    }
#pragma unroll
    for (int s = 0; s < NS; s++) {
      const float v[8] = {qa[s].x, qa[s].y, qa[s].z, qa[s].w, qb[s].x, qb[s].y, qb[s].z, qb[s].w};
#pragma unroll
      for (int e = 0; e < 8; e++) {
        _Float16 hi, lo;
        am_split(v[e] * down, hi, lo);
        qh[s][e] = hi;
        ql[s][e] = lo;
      }
    }
  }

  // staging roles: threads 0..127 transpose V (one 8 x 8 block each: position group pg, dimension
  // block db), threads 128..255 copy K (NK pieces each)
  const bool v_thread = tid < 128u;
  const uint32_t vdb = tid % PPR, vpg = tid / PPR;           // pg = 4 pb + 2 j + lh', 8 of them
  const bool v_active = v_thread && vpg < 8u;
  const uint32_t vp0 = 32u * (vpg >> 2) + 16u * ((vpg >> 1) & 1u) + 4u * (vpg & 1u);   // positions vp0 + 0..3, vp0 + 8 + 0..3
  const uint32_t kt_ = tid - 128u;
  uint4 pf[8];
#define AM_LOAD(TILE)                                                                             \
  do {                                                                                            \
    const uint32_t base_ = (TILE) * AM_KT;                                                        \
    if (v_thread) {                                                                               \
      if (v_active) {                                                                             \
        _Pragma("unroll") for (int e = 0; e < 8; e++) {                                           \
          const uint32_t row_ = min(base_ + vp0 + 8u * (e >> 2) + (e & 3), max_row);              \
          pf[e] = *(const uint4 *)(vc + (size_t)row_ * kv_dim + kvh * HD + 8u * vdb);             \
        }                                                                                         \
      }                                                                                           \
    } else {                                                                                      \
      _Pragma("unroll") for (int u = 0; u < NK; u++) {                                            \
        const uint32_t i_ = kt_ + 128u * u;                                                       \
        const uint32_t row_ = min(base_ + i_ / PPR, max_row);                                     \
        pf[u] = *(const uint4 *)(kc + (size_t)row_ * kv_dim + kvh * HD + 8u * (i_ % PPR));        \
      }                                                                                           \
    }                                                                                             \
  } while (0)
#define AM_STORE()                                                                                \
  do {                                                                                            \
    if (v_thread) {                                                                               \
      if (v_active) {                                                                             \
        const uint32_t r_[8][4] = {{pf[0].x, pf[0].y, pf[0].z, pf[0].w}, {pf[1].x, pf[1].y, pf[1].z, pf[1].w}, \
                                   {pf[2].x, pf[2].y, pf[2].z, pf[2].w}, {pf[3].x, pf[3].y, pf[3].z, pf[3].w}, \
                                   {pf[4].x, pf[4].y, pf[4].z, pf[4].w}, {pf[5].x, pf[5].y, pf[5].z, pf[5].w}, \
                                   {pf[6].x, pf[6].y, pf[6].z, pf[6].w}, {pf[7].x, pf[7].y, pf[7].z, pf[7].w}}; \
        _Pragma("unroll") for (int w_ = 0; w_ < 4; w_++) {                                        \
          /* dimensions 2 w_ (low halves) and 2 w_ + 1 (high halves) of the eight positions */    \
          uint4 lo_, hi_;                                                                         \
          lo_.x = __builtin_amdgcn_perm(r_[1][w_], r_[0][w_], 0x05040100u);                       \
          lo_.y = __builtin_amdgcn_perm(r_[3][w_], r_[2][w_], 0x05040100u);                       \
          lo_.z = __builtin_amdgcn_perm(r_[5][w_], r_[4][w_], 0x05040100u);                       \
          lo_.w = __builtin_amdgcn_perm(r_[7][w_], r_[6][w_], 0x05040100u);                       \
          hi_.x = __builtin_amdgcn_perm(r_[1][w_], r_[0][w_], 0x07060302u);                       \
          hi_.y = __builtin_amdgcn_perm(r_[3][w_], r_[2][w_], 0x07060302u);                       \
          hi_.z = __builtin_amdgcn_perm(r_[5][w_], r_[4][w_], 0x07060302u);                       \
          hi_.w = __builtin_amdgcn_perm(r_[7][w_], r_[6][w_], 0x07060302u);                       \
          *(uint4 *)&vt_l[(8u * vdb + 2u * w_) * AM_VROW + 16u * vpg] = lo_;                      \
          *(uint4 *)&vt_l[(8u * vdb + 2u * w_ + 1u) * AM_VROW + 16u * vpg] = hi_;                 \
        }                                                                                         \
      }                                                                                           \
    } else {                                                                                      \
      _Pragma("unroll") for (int u = 0; u < NK; u++) {                                            \
        const uint32_t i_ = kt_ + 128u * u;                                                       \
        *(uint4 *)&k_l[(i_ / PPR) * KROW + 16u * (i_ % PPR)] = pf[u];                             \
      }                                                                                           \
    }                                                                                             \
  } while (0)

  af16 o[NDB];
#pragma unroll
  for (int d = 0; d < NDB; d++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[d][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;   // l_run: this lane half's share of the sum

  // iteration i: tile 2 i + half (a tile past the walk is loaded from clamped rows and not used)
  const uint32_t n_iter = (n_tiles + 1u) / 2u;
  const uint32_t q_min = pos0 + min(32u * qt, n_tokens - 1u);   // the tile's first query
  AM_LOAD(half);
  for (uint32_t i2 = 0; i2 < n_iter; i2++) {
    const uint32_t it = 2u * i2 + half;
    AM_STORE();
    __syncthreads();
    if (i2 + 1u < n_iter) AM_LOAD(it + 2u);
    if (live && it < n_tiles) {
      af16 s0, s1;
#pragma unroll
      for (int r = 0; r < 16; r++) s0[r] = s1[r] = 0.0f;
#pragma unroll
      for (int s = 0; s < NS; s++) {
        const ah8 a0 = *(const ah8 *)&k_l[l32 * KROW + 32u * s + 16u * lh];
        const ah8 a1 = *(const ah8 *)&k_l[(l32 + 32u) * KROW + 32u * s + 16u * lh];
        s0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, qh[s], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, qh[s], s1, 0, 0, 0);
        s0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, ql[s], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, ql[s], s1, 0, 0, 0);
      }
      // register r of block pb: position it * 64 + 32 pb + 8 (r / 4) + 4 lh + r % 4
      const uint32_t pbase = it * AM_KT + 4u * lh;
      float mt = -INFINITY;
      if (it * AM_KT + (AM_KT - 1u) <= q_min) {   // every query of the tile sees the whole cache tile
#pragma unroll
        for (int r = 0; r < 16; r++) {
          s0[r] *= scale_q;
          s1[r] *= scale_q;
          mt = fmaxf(mt, fmaxf(s0[r], s1[r]));
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const uint32_t p_ = pbase + 8u * (r >> 2) + (r & 3);
          s0[r] = p_ <= q_abs ? s0[r] * scale_q : -INFINITY;
          s1[r] = p_ + 32u <= q_abs ? s1[r] * scale_q : -INFINITY;
          mt = fmaxf(mt, fmaxf(s0[r], s1[r]));
        }
      }
      mt = ogm_butterfly_step<32>(mt, OgmOpMax());
      // (a query may see nothing of the odd half's first tile: then everything stays at zero)
      const float m_max = fmaxf(m_run, mt);
      const float m_new = m_max == -INFINITY ? 0.0f : m_max;
      const float alpha = __expf(m_run - m_new);
      m_run = m_max;
      float lsum = 0.0f;
      ah8 ph[4], pl[4];   // k step 2 pb + j: registers 8 j .. 8 j + 7 of block pb
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float p0_ = __expf(s0[r] - m_new), p1_ = __expf(s1[r] - m_new);
        lsum += p0_ + p1_;
        _Float16 hi, lo;
        am_split(p0_, hi, lo);
        ph[r >> 3][r & 7] = hi;
        pl[r >> 3][r & 7] = lo;
        am_split(p1_, hi, lo);
        ph[2 + (r >> 3)][r & 7] = hi;
        pl[2 + (r >> 3)][r & 7] = lo;
      }
      l_run = l_run * alpha + lsum;
#pragma unroll
      for (int d = 0; d < NDB; d++) {
#pragma unroll
        for (int r = 0; r < 16; r++) o[d][r] *= alpha;
#pragma unroll
        for (int js = 0; js < 4; js++) {
          const ah8 a = *(const ah8 *)&vt_l[(32u * d + l32) * AM_VROW + 32u * js + 16u * lh];
          o[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, ph[js], o[d], 0, 0, 0);
          o[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pl[js], o[d], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }
#undef AM_LOAD
#undef AM_STORE
  // the odd half's partial softmax goes through LDS (the tiles' space: the loop ended on a barrier) to the
  // even half's wave of the same head, lane to lane: [register][wave][lane]
  {
    float *mrg = (float *)am_lds;
    constexpr uint32_t NR = NDB * 16u + 2u;
    const uint32_t slot = wave * 64u + lane;
    if (half == 1u) {
#pragma unroll
      for (int d = 0; d < NDB; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) mrg[(16u * d + r) * 256u + slot] = o[d][r];
      mrg[(NR - 2u) * 256u + slot] = m_run;
      mrg[(NR - 1u) * 256u + slot] = l_run;
    }
    __syncthreads();
    if (half == 1u) return;
    const float m1 = mrg[(NR - 2u) * 256u + slot], l1 = mrg[(NR - 1u) * 256u + slot];
    const float m = fmaxf(m_run, m1);   // finite: the even half saw position 0
    const float a0 = __expf(m_run - m), a1 = __expf(m1 - m);
    l_run = l_run * a0 + l1 * a1;
#pragma unroll
    for (int d = 0; d < NDB; d++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[d][r] = o[d][r] * a0 + mrg[(16u * d + r) * 256u + slot] * a1;
  }
  if (live && 32u * qt + l32 < n_tokens) {
    const float l = ogm_butterfly_step<32>(l_run, OgmOpAdd());
    float *op = attn_out + ((size_t)tok * n_head + (size_t)kvh * gq + g) * HD + 4u * lh;
#pragma unroll
    for (int d = 0; d < NDB; d++)
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++)   // registers 4 r4 .. + 3: dimensions 32 d + 8 r4 + 4 lh + 0..3
        *(float4 *)(op + 32 * d + 8 * r4) = make_float4(o[d][4 * r4] / l, o[d][4 * r4 + 1] / l, o[d][4 * r4 + 2] / l,
                                                        o[d][4 * r4 + 3] / l);
  }
}

hipError_t ogm_launch_attn_prefill_mfma(const float *q, void *k_cache_layer, void *v_cache_layer, uint32_t pos0,
                                        uint32_t n_tokens, uint32_t n_head, uint32_t n_head_kv, uint32_t head_dim,
                                        float scale, float *attn_out, hipStream_t stream) {
  if (n_head_kv == 0 || n_head % n_head_kv != 0 || n_tokens == 0) return hipErrorInvalidValue;
  const uint32_t gq = n_head / n_head_kv;
  if (n_head_kv > 65535u || ogm_attn_head_parts(gq) == 0u) return hipErrorInvalidValue;
  if ((n_tokens + 31u) / 32u > 65535u) return hipErrorInvalidValue;
  const dim3 grid(n_head_kv * ((gq + 3u) / 4u), (n_tokens + 31u) / 32u);
  if (head_dim != 128 && head_dim != 64) return hipErrorInvalidValue;
  // two (K, V^T) tiles, rows padded by 16 bytes; at head_dim 128 more than a kernel gets without asking
  const uint32_t lds_bytes = 2u * (AM_KT * (head_dim * 2u + 16u) + head_dim * AM_VROW);
  const void *fn = head_dim == 128 ? (const void *)ogm_attn_prefill_mfma_kernel<128> : (const void *)ogm_attn_prefill_mfma_kernel<64>;
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return e;
  if (head_dim == 128)
    hipLaunchKernelGGL(ogm_attn_prefill_mfma_kernel<128>, grid, dim3(512), lds_bytes, stream, q, (const __half *)k_cache_layer,
                       (const __half *)v_cache_layer, pos0, n_tokens, n_head_kv, gq, scale, attn_out);
  else
    hipLaunchKernelGGL(ogm_attn_prefill_mfma_kernel<64>, grid, dim3(512), lds_bytes, stream, q, (const __half *)k_cache_layer,
                       (const __half *)v_cache_layer, pos0, n_tokens, n_head_kv, gq, scale, attn_out);
  return hipGetLastError();
}

// The stamps of the last attention launch, eight per workgroup in the grid's order (x fastest), then cleared.
hipError_t ogm_attn_stamps_read(unsigned long long *host_out, size_t n_words) {
#ifdef OGM_ATTN_STAMPS
  if (n_words > 4096u * 8u) return hipErrorInvalidValue;
  hipError_t e = hipMemcpyFromSymbol(host_out, HIP_SYMBOL(ogm_attn_stamps), n_words * 8u);
  if (e != hipSuccess) return e;
  void *dev = nullptr;
  e = hipGetSymbolAddress(&dev, HIP_SYMBOL(ogm_attn_stamps));
  if (e != hipSuccess) return e;
  return hipMemset(dev, 0, sizeof(unsigned long long) * 4096u * 8u);
#else
  (void)host_out;
  (void)n_words;
  return hipErrorNotSupported;
#endif
}
