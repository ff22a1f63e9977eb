// C ABI of the MI355X quantized matmul backend (include/orangu_mi355x.h): context, weight
// uploader and the Backend::matmul family (engine/backend/mod.rs:309-496 of orangu-server),
// over the kernels in ogm_kernels.hip.  No CPU fallback: every compute entry point runs the
// HIP kernels or returns an error status.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <map>
#include <chrono>
#include <mutex>
#include <new>
#include <string>
#include <utility>
#include <vector>

#include "../../include/orangu_mi355x.h"
#include "ogm_kernels.h"
#include "ogm_layout.h"

// ------------------------------------------------------------------------------------------

struct ogm_weight {
  uint32_t ggml_type, in_dim, out_dim;
  size_t row_bytes, device_bytes;
  uint8_t *dev;  // tile-planar
  uint64_t key_addr, key_len;
  // K-quants: the scale-folded int8 planes the tiled prefill GEMMs multiply (ogm_gemm_build_planes),
  // built on the matrix's first such GEMM and kept while the context's budget allows; null before
  // that.  A second, prefill-only layout: the tile-planar bytes stay what ogm_weight_download returns.
  uint8_t *planes = nullptr;
  size_t plane_bytes = 0;
  bool planes_refused = false;   // over budget or out of memory once: not tried again
};

struct DevBuf {
  void *p = nullptr;
  size_t cap = 0;
};

struct ogm_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  std::mutex mu;
  std::mutex err_mu;   // guards err alone: argument checks fail before mu is taken
  std::string err;
  std::string name;
  std::map<std::pair<uint64_t, uint64_t>, ogm_weight *> cache;
  std::vector<ogm_weight *> weights;
  // scratch, grown on demand and reused (the vendor backends allocate per call,
  // engine/backend/rocm.rs:352-376; a pool is what the Vulkan op_cache does instead)
  DevBuf x, y, q, d, sums, bsum, bs16, isum, imin, xh, probe_sink;
  DevBuf hx, hy;  // pinned host staging
  DevBuf hflag;   // pinned word a trailing kernel sets for host_wait
  uint32_t flag_epoch = 0, flag_unsynced = 0;
  int tune_wg_waves = 0;
  // matmul at n_tokens >= this takes the MFMA GEMM; 0 = by type: 9 for Q4_K, Q5_K and Q6_K, whose
  // small-batch kernel beats the GEMV kernel's chunks of 8 tokens from there on (Q4_K 4096 -> 4096 at 9
  // tokens: 12 against 16 us), 17 for the others, whose tiled kernels cost about the same from 9 to 128
  // tokens while the chunked GEMV grows with the count (they cross between 12 and 32 tokens).
  int tune_gemm_min_tokens = 0;
  int tune_gemm_medium = 0;      // Q4_K / Q5_K medium-batch kernel: 0 by the size of the launch, 1 never, 2 whenever the shape allows
  int tune_gemm_tile_rows = 0;   // feeding-wave GEMMs: 64 forces their 64-row tiles, 0 = by the size of the launch
  int tune_gemm_small_max = 0;   // most tokens for the small-batch GEMM kernel: 0 = default, 1 = never
  int tune_gemm_ft_min_rows = 0;  // few-token Q6_K kernel: fewest rows it takes (0 = default, 1 = any shape it can, -1 = never)
  int tune_gemm_sb_waves = 0;          // small-batch GEMM: 8 or 16 waves per workgroup, 0 = by the launch
  int tune_host_flag_wait = 1;         // zero-copy host calls wait on a word a trailing kernel stores to pinned memory instead of on the stream
  int tune_host_zero_copy = 1;         // host-pointer calls of up to OGM_ZERO_COPY_MAX bytes: kernels read x / write y in pinned host memory
  bool host_coherent = true;           // the pinned staging buffers are fine-grained (asked for by name); false once the runtime has refused
  int tune_gemv_mma = 1;               // few tokens over Q4_K / Q5_K / Q6_K on the row-block matrix-core kernel: 0 never, 1 where it measured faster, 2 wherever it can
  int tune_gemm_plane_kernel = 0;      // the all-waves-multiply kernel over planes: 0 on large grids, 2 whatever the grid
  int tune_gemm_act_chunks = 0;       // a K-quant batch's int8 activations also in the matrix-core kernels' operand chunks: 0 from 25 tokens (producers of the forward pass: 17), 1 never, 2 from 9
  int tune_gemm_interleave = 0;        // the 64-row plane kernel with the f32 step between the matrix instructions: 0 by the launch's size, 1 never, 2 whenever it can
  int tune_gemm_one_pass = 0;          // 1: Q4_K / Q5_K on that kernel fold the min pass into the super-block step (f32 to rounding, not to the bit)
  int tune_prefill_chunk = 2048;       // tokens per prefill pass over the layers (fixed per model at its first prefill)
  int tune_attn_decode_chunks = 0;     // chunks of the cache a workgroup of the decode step's attention takes in a row; 0: by the context
  int tune_attn_prefill_variant = 0;   // 0: by batch size; 1: the decode kernel per token and chunk; 2: the matrix-core kernel
  // Device memory the prefill planes of all weights may take, in MiB; 0 (the default) = build none.
  // A model's planes are 3.3 times its Q4_K bytes.
  int tune_plane_cache_mb = 32768;   // MiB the K-quant matrices' prefill planes may take in all
  size_t plane_bytes_used = 0;
  const char *last_kernel = "";
  uint8_t *static_scratch = nullptr;   // this device's copy of the library's static scratch array (ogm_static.hip)
  // what the activation buffer currently holds (ogm_act_quantize_dev)
  int act_mode = -1;
  uint32_t act_in_dim = 0, act_tokens = 0;
  bool act_xt = false;   // ... and xh holds the same activations in the tiled GEMM's operand chunks
};

static thread_local std::string g_init_err;

// Callable with or without ctx->mu held: the message has a lock of its own.
static int fail(ogm_ctx *ctx, int status, const std::string &msg) {
  if (ctx) {
    std::lock_guard<std::mutex> lock(ctx->err_mu);
    ctx->err = msg;
  } else {
    g_init_err = msg;
  }
  return status;
}

#define HIPCHK(ctx, call)                                                              \
  do {                                                                                 \
    hipError_t e_ = (call);                                                            \
    if (e_ != hipSuccess)                                                              \
      return fail(ctx, e_ == hipErrorOutOfMemory ? OGM_ERR_OOM : OGM_ERR_HIP,          \
                  std::string(#call) + ": " + hipGetErrorString(e_));                  \
  } while (0)

static int ensure_dev(ogm_ctx *ctx, DevBuf &b, size_t bytes) {
  if (bytes <= b.cap) return OGM_OK;
  // Kernels still in flight may read the old buffer.
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  if (b.p) HIPCHK(ctx, hipFree(b.p));
  b.p = nullptr;
  b.cap = 0;
  size_t cap = (bytes + 255) & ~(size_t)255;
  HIPCHK(ctx, hipMalloc(&b.p, cap));
  b.cap = cap;
  return OGM_OK;
}

// Pinned host memory the kernels of a zero-copy call read x from and store y and the completion word to.  The
// host reads y after seeing the word, with no runtime call between: that is only sound for fine-grained
// (coherent) host memory, where a kernel's stores are visible to the host as they are acknowledged.  So
// coherence is asked for by name; where the runtime refuses it, the memory is plain pinned memory and the
// context stops running kernels on it in place (host_coherent false: device copies and a stream
// synchronization per call instead).
static hipError_t host_alloc_coherent(ogm_ctx *ctx, void **p, size_t bytes) {
  if (ctx->host_coherent) {
    if (hipHostMalloc(p, bytes, hipHostMallocCoherent) == hipSuccess) return hipSuccess;
    (void)hipGetLastError();
    ctx->host_coherent = false;
  }
  return hipHostMalloc(p, bytes, hipHostMallocDefault);
}

static int ensure_host(ogm_ctx *ctx, DevBuf &b, size_t bytes) {
  if (bytes <= b.cap) return OGM_OK;
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  if (b.p) HIPCHK(ctx, hipHostFree(b.p));
  b.p = nullptr;
  b.cap = 0;
  size_t cap = (bytes + 4095) & ~(size_t)4095;
  HIPCHK(ctx, host_alloc_coherent(ctx, &b.p, cap));
  b.cap = cap;
  return OGM_OK;
}

static uint32_t block_elems_of(uint32_t ggml_type) {
  OgmLayout l;
  return ogm_layout_for(ggml_type, &l) ? l.block_elems : 256u;
}

static int act_mode_for(uint32_t ggml_type, uint32_t n_tokens = 1, int decode = 1) {
  // backend/cpu.rs:100-116: the K-quants take quantize_act_k_row (per 256), the per-32 types quantize_act.
  // Q2_K has a per-256 dot for one token (supports_k_row) but no K GEMM (supports_k): matmul of several
  // tokens unpacks its rows once and runs them against quantize_act's per-32 activations (cpu.rs:113-163).
  if (ggml_type == OGM_Q2_K && !decode && n_tokens > 1) return OGM_ACT_PER_32;
  return block_elems_of(ggml_type) == 32 ? OGM_ACT_PER_32 : OGM_ACT_PER_256;
}

static int ensure_act(ogm_ctx *ctx, uint32_t in_dim, uint32_t n_tokens) {
  int rc;
  size_t n = (size_t)in_dim * n_tokens;
  if ((rc = ensure_dev(ctx, ctx->q, n)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->d, n / 32 * 4)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->sums, n / 16 * 4)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->bsum, n / 32 * 2)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->bs16, n / 16 * 2)) != OGM_OK) return rc;
  return OGM_OK;
}

// The activations of token `token0` on in a token-major buffer set whose first token is `base`.
static OgmActDev act_offset(const OgmActDev &base, uint32_t in_dim, int mode, uint32_t token0) {
  OgmActDev a;
  a.q = base.q + (size_t)token0 * in_dim;
  a.d = base.d + (size_t)token0 * (in_dim / (mode == OGM_ACT_PER_32 ? 32 : 256));
  a.sums = base.sums + (size_t)token0 * (in_dim / 16);
  a.bsum = base.bsum + (size_t)token0 * (in_dim / 32);
  a.bs16 = (mode == OGM_ACT_PER_32 || !base.bs16) ? nullptr : base.bs16 + (size_t)token0 * (in_dim / 16);
  return a;
}

static OgmActDev act_view(ogm_ctx *ctx, uint32_t in_dim, int mode, uint32_t token0) {
  const OgmActDev base{(int8_t *)ctx->q.p, (float *)ctx->d.p, (int32_t *)ctx->sums.p, (int16_t *)ctx->bsum.p,
                       (uint16_t *)ctx->bs16.p};
  return act_offset(base, in_dim, mode, token0);
}

// ------------------------------------------------------------------------------------------
// lifetime

extern "C" int ogm_init(int device, ogm_ctx **out) {
  if (!out) return fail(nullptr, OGM_ERR_INVALID, "ogm_init: out is null");
  *out = nullptr;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0)
    return fail(nullptr, OGM_ERR_NO_DEVICE,
                std::string("no HIP device: ") + (e != hipSuccess ? hipGetErrorString(e) : "count 0"));
  if (device < 0 || device >= n)
    return fail(nullptr, OGM_ERR_NO_DEVICE, "device ordinal out of range");
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess)
    return fail(nullptr, OGM_ERR_HIP, std::string("hipGetDeviceProperties: ") + hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(nullptr, OGM_ERR_NO_DEVICE,
                std::string("device is ") + prop.gcnArchName + ", these kernels are built for gfx950 only");
  ogm_ctx *ctx = new (std::nothrow) ogm_ctx();
  if (!ctx) return fail(nullptr, OGM_ERR_OOM, "out of host memory");
  ctx->device = device;
  // Some driver stacks leave the marketing name empty: fall back to the architecture's name.
  const std::string board = prop.name[0] ? prop.name : "AMD Instinct (gfx950)";
  ctx->name = board + " (" + prop.gcnArchName + ")";
  e = hipSetDevice(device);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    std::string msg = std::string("stream creation: ") + hipGetErrorString(e);
    delete ctx;
    return fail(nullptr, OGM_ERR_HIP, msg);
  }
  // the device is current: resolve this device's address of the static scratch once, here
  e = ogm_static_scratch_address(&ctx->static_scratch);
  if (e != hipSuccess) {
    std::string msg = std::string("static scratch address: ") + hipGetErrorString(e);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return fail(nullptr, OGM_ERR_HIP, msg);
  }
  *out = ctx;
  return OGM_OK;
}

extern "C" void ogm_destroy(ogm_ctx *ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
  for (ogm_weight *w : ctx->weights) {
    if (w->dev) (void)hipFree(w->dev);
    if (w->planes) (void)hipFree(w->planes);
    delete w;
  }
  DevBuf *dev[] = {&ctx->x,    &ctx->y,    &ctx->q,    &ctx->d,  &ctx->sums,
                   &ctx->bsum, &ctx->bs16, &ctx->isum, &ctx->imin, &ctx->xh, &ctx->probe_sink};
  for (DevBuf *b : dev)
    if (b->p) (void)hipFree(b->p);
  if (ctx->hx.p) (void)hipHostFree(ctx->hx.p);
  if (ctx->hy.p) (void)hipHostFree(ctx->hy.p);
  if (ctx->hflag.p) (void)hipHostFree(ctx->hflag.p);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

extern "C" const char *ogm_last_error(ogm_ctx *ctx) {
  static thread_local std::string copy;
  if (ctx) {
    std::lock_guard<std::mutex> lock(ctx->err_mu);
    copy = ctx->err;
  } else {
    copy = g_init_err;
  }
  return copy.c_str();
}

extern "C" int ogm_device_name(ogm_ctx *ctx, char *buf, size_t buf_len) {
  if (!ctx || !buf || buf_len == 0) return OGM_ERR_INVALID;
  snprintf(buf, buf_len, "%s", ctx->name.c_str());
  return OGM_OK;
}

extern "C" int ogm_set_tuning(ogm_ctx *ctx, const char *key, int value) {
  if (!ctx || !key) return OGM_ERR_INVALID;
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (strcmp(key, "gemv_wg_waves") == 0) {
    if (value < 0 || value > 16) return fail(ctx, OGM_ERR_INVALID, "gemv_wg_waves must be 0..16");
    ctx->tune_wg_waves = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_min_tokens") == 0) {
    if (value < 0) return fail(ctx, OGM_ERR_INVALID, "gemm_min_tokens must be >= 0");
    ctx->tune_gemm_min_tokens = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_small_max_tokens") == 0) {
    if (value < 0 || value > 1024) return fail(ctx, OGM_ERR_INVALID, "gemm_small_max_tokens must be 0..1024");
    ctx->tune_gemm_small_max = value;
    return OGM_OK;
  }
  if (strcmp(key, "host_flag_wait") == 0) {
    if (value < 0 || value > 2) return fail(ctx, OGM_ERR_INVALID, "host_flag_wait must be 0, 1 or 2");
    ctx->tune_host_flag_wait = value;
    return OGM_OK;
  }
  if (strcmp(key, "host_zero_copy") == 0) {
    if (value != 0 && value != 1) return fail(ctx, OGM_ERR_INVALID, "host_zero_copy must be 0 or 1");
    ctx->tune_host_zero_copy = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_medium") == 0) {
    if (value < 0 || value > 2) return fail(ctx, OGM_ERR_INVALID, "gemm_medium must be 0, 1 or 2");
    ctx->tune_gemm_medium = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_tile_rows") == 0) {
    if (value != 0 && value != 64) return fail(ctx, OGM_ERR_INVALID, "gemm_tile_rows must be 0 or 64");
    ctx->tune_gemm_tile_rows = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_plane_kernel") == 0) {
    if (value != 0 && value != 2) return fail(ctx, OGM_ERR_INVALID, "gemm_plane_kernel must be 0 or 2");
    ctx->tune_gemm_plane_kernel = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_interleave") == 0) {
    if (value < 0 || value > 2) return fail(ctx, OGM_ERR_INVALID, "gemm_interleave must be 0, 1 or 2");
    ctx->tune_gemm_interleave = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_act_chunks") == 0) {
    if (value < 0 || value > 2) return fail(ctx, OGM_ERR_INVALID, "gemm_act_chunks must be 0, 1 or 2");
    ctx->tune_gemm_act_chunks = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_one_pass") == 0) {
    if (value != 0 && value != 1) return fail(ctx, OGM_ERR_INVALID, "gemm_one_pass must be 0 or 1");
    ctx->tune_gemm_one_pass = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_few_tokens_min_rows") == 0) {
    if (value < -1) return fail(ctx, OGM_ERR_INVALID, "gemm_few_tokens_min_rows must be >= -1");
    ctx->tune_gemm_ft_min_rows = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_sb_waves") == 0) {
    if (value != 0 && value != 8 && value != 16) return fail(ctx, OGM_ERR_INVALID, "gemm_sb_waves must be 0, 8 or 16");
    ctx->tune_gemm_sb_waves = value;
    return OGM_OK;
  }
  if (strcmp(key, "prefill_chunk_tokens") == 0) {
    if (value < 1 || value > 16384) return fail(ctx, OGM_ERR_INVALID, "prefill_chunk_tokens must be 1..16384");
    ctx->tune_prefill_chunk = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemv_mma") == 0) {
    if (value < 0 || value > 2) return fail(ctx, OGM_ERR_INVALID, "gemv_mma must be 0, 1 or 2");
    ctx->tune_gemv_mma = value;
    return OGM_OK;
  }
  if (strcmp(key, "attn_decode_chunks") == 0) {
    if (value < 0 || value > 64) return fail(ctx, OGM_ERR_INVALID, "attn_decode_chunks must be 0 to 64");
    ctx->tune_attn_decode_chunks = value;
    return OGM_OK;
  }
  if (strcmp(key, "attn_prefill_variant") == 0) {
    if (value < 0 || value > 2) return fail(ctx, OGM_ERR_INVALID, "attn_prefill_variant must be 0, 1 or 2");
    ctx->tune_attn_prefill_variant = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemm_plane_cache_mb") == 0) {
    if (value < 0) return fail(ctx, OGM_ERR_INVALID, "gemm_plane_cache_mb must be >= 0");
    ctx->tune_plane_cache_mb = value;
    return OGM_OK;
  }
  return fail(ctx, OGM_ERR_INVALID, std::string("unknown tuning key ") + key);
}

// Bytes of device and pinned host scratch the context has grown so far (weights and planes not counted).
extern "C" size_t ogm_scratch_bytes(ogm_ctx *ctx) {
  if (!ctx) return 0;
  std::lock_guard<std::mutex> lock(ctx->mu);
  const DevBuf *all[] = {&ctx->x,    &ctx->y,    &ctx->q,  &ctx->d,          &ctx->sums, &ctx->bsum, &ctx->bs16,
                         &ctx->isum, &ctx->imin, &ctx->xh, &ctx->probe_sink, &ctx->hx,   &ctx->hy,   &ctx->hflag};
  size_t n = 0;
  for (const DevBuf *b : all) n += b->cap;
  return n;
}

extern "C" const char *ogm_last_kernel(ogm_ctx *ctx) {
  if (!ctx) return "";
  std::lock_guard<std::mutex> lock(ctx->mu);   // launches write it under the same lock
  return ctx->last_kernel;
}

// ------------------------------------------------------------------------------------------
// weights

extern "C" int ogm_weight_upload(ogm_ctx *ctx, uint32_t ggml_type, const void *raw,
                                 size_t row_bytes, uint32_t in_dim, uint32_t out_dim,
                                 uint64_t key_addr, uint64_t key_len, ogm_weight **out) {
  if (!ctx || !out) return OGM_ERR_INVALID;
  std::lock_guard<std::mutex> lock(ctx->mu);
  *out = nullptr;
  if (key_len != 0) {
    auto it = ctx->cache.find({key_addr, key_len});
    if (it != ctx->cache.end()) {
      ogm_weight *w = it->second;
      if (w->ggml_type != ggml_type || w->in_dim != in_dim || w->out_dim != out_dim)
        return fail(ctx, OGM_ERR_INVALID, "cache key reused with a different shape or type");
      *out = w;
      return OGM_OK;
    }
  }
  if (!raw) return fail(ctx, OGM_ERR_INVALID, "raw is null");
  if (!ogm_supports_type(ggml_type)) return fail(ctx, OGM_ERR_UNSUPPORTED, "ggml type without a kernel");
  if (in_dim == 0 || out_dim == 0) return fail(ctx, OGM_ERR_INVALID, "zero dimension");
  if (!ogm_supports(ggml_type, in_dim))
    return fail(ctx, OGM_ERR_UNSUPPORTED, "in_dim is not a whole number of blocks");
  size_t bytes = ogm_repacked_size(ggml_type, in_dim, out_dim);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  void *staging = nullptr;
  HIPCHK(ctx, hipHostMalloc(&staging, bytes, hipHostMallocDefault));
  int rc = ogm_repack_host(ggml_type, raw, row_bytes, in_dim, out_dim, staging);
  if (rc != OGM_OK) {
    (void)hipHostFree(staging);
    return fail(ctx, rc, "row_bytes does not match in_dim for this type");
  }
  ogm_weight *w = new (std::nothrow) ogm_weight();
  if (!w) {
    (void)hipHostFree(staging);
    return fail(ctx, OGM_ERR_OOM, "out of host memory");
  }
  w->ggml_type = ggml_type;
  w->in_dim = in_dim;
  w->out_dim = out_dim;
  w->row_bytes = row_bytes;
  w->device_bytes = bytes;
  w->key_addr = key_addr;
  w->key_len = key_len;
  w->dev = nullptr;
  hipError_t e = hipMalloc((void **)&w->dev, bytes);
  if (e == hipSuccess) e = hipMemcpyAsync(w->dev, staging, bytes, hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  (void)hipHostFree(staging);
  if (e != hipSuccess) {
    if (w->dev) (void)hipFree(w->dev);
    delete w;
    return fail(ctx, e == hipErrorOutOfMemory ? OGM_ERR_OOM : OGM_ERR_HIP,
                std::string("weight upload: ") + hipGetErrorString(e));
  }
  ctx->weights.push_back(w);
  if (key_len != 0) ctx->cache[{key_addr, key_len}] = w;
  *out = w;
  return OGM_OK;
}

extern "C" int ogm_weight_download(ogm_ctx *ctx, const ogm_weight *w, void *raw_out, size_t raw_len) {
  if (!ctx || !w || !raw_out) return OGM_ERR_INVALID;
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (raw_len != w->row_bytes * w->out_dim) return fail(ctx, OGM_ERR_INVALID, "raw_len mismatch");
  HIPCHK(ctx, hipSetDevice(ctx->device));
  std::vector<uint8_t> tmp(w->device_bytes);
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  HIPCHK(ctx, hipMemcpy(tmp.data(), w->dev, w->device_bytes, hipMemcpyDeviceToHost));
  return ogm_unrepack_host(w->ggml_type, tmp.data(), w->row_bytes, w->in_dim, w->out_dim, raw_out);
}

extern "C" int ogm_weight_free(ogm_ctx *ctx, ogm_weight *w) {
  if (!ctx || !w) return OGM_ERR_INVALID;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  for (size_t i = 0; i < ctx->weights.size(); i++) {
    if (ctx->weights[i] == w) {
      ctx->weights.erase(ctx->weights.begin() + (long)i);
      if (w->key_len != 0) ctx->cache.erase({w->key_addr, w->key_len});
      if (w->dev) HIPCHK(ctx, hipFree(w->dev));
      if (w->planes) {
        HIPCHK(ctx, hipFree(w->planes));
        ctx->plane_bytes_used -= w->plane_bytes;
      }
      delete w;
      return OGM_OK;
    }
  }
  return fail(ctx, OGM_ERR_INVALID, "weight does not belong to this context");
}

extern "C" int ogm_weight_info(const ogm_weight *w, uint32_t *ggml_type, uint32_t *in_dim,
                               uint32_t *out_dim, size_t *device_bytes) {
  if (!w) return OGM_ERR_INVALID;
  if (ggml_type) *ggml_type = w->ggml_type;
  if (in_dim) *in_dim = w->in_dim;
  if (out_dim) *out_dim = w->out_dim;
  if (device_bytes) *device_bytes = w->device_bytes;
  return OGM_OK;
}

// ------------------------------------------------------------------------------------------
// matmul

// Whether the int8 activations of a batch over K-quant matrices of this type and width are also laid out in the
// operand chunks of the matrix-core GEMMs (ogm_xt_row): the plane and medium-batch kernels read nothing else, and the
// small-batch kernels load a chunk of 32 tokens x 32 k in one piece instead of gathering 32 rows.  from: the batch
// size from which the caller's producer writes them by default.
static bool act_chunks_wanted(const ogm_ctx *ctx, uint32_t ggml_type, uint32_t in_dim, uint32_t n_tokens, int decode,
                              uint32_t from) {
  if (decode || ctx->tune_gemm_act_chunks == 1 || ogm_gemm_plane_bytes(ggml_type, in_dim, 64u) == 0 ||
      act_mode_for(ggml_type, n_tokens, decode) != OGM_ACT_PER_256 ||
      (uint64_t)((n_tokens + 31u) & ~31u) * in_dim >= (1ull << 32))
    return false;
  return n_tokens >= (ctx->tune_gemm_act_chunks == 2 ? 9u : from);
}

// Enqueues the activation quantizer.  Caller holds the lock.
// with_xt: the int8 activations also go to ctx->xh in the operand chunks of the GEMM whose waves all multiply.
static int enqueue_quantize(ogm_ctx *ctx, int mode, const float *x_dev, uint32_t in_dim,
                            uint32_t n_tokens, hipStream_t stream, bool with_xt = false) {
  int rc = ensure_act(ctx, in_dim, n_tokens);
  if (rc != OGM_OK) return rc;
  if (with_xt && (rc = ensure_dev(ctx, ctx->xh, ogm_gemm_xh_bytes(in_dim, n_tokens))) != OGM_OK) return rc;
  HIPCHK(ctx, ogm_launch_quantize(mode, x_dev, in_dim, n_tokens, act_view(ctx, in_dim, mode, 0), stream,
                                  with_xt ? (int8_t *)ctx->xh.p : nullptr));
  ctx->act_mode = mode;
  ctx->act_in_dim = in_dim;
  ctx->act_tokens = n_tokens;
  ctx->act_xt = with_xt;
  return OGM_OK;
}

// One matrix and where its output goes; a group shares type, in_dim and the activations.
struct Target {
  const ogm_weight *w;
  float *y;
};

static int enqueue_gemv(ogm_ctx *ctx, const Target *tg, size_t n_tg, uint32_t n_tokens, int decode,
                        hipStream_t stream, int32_t *dump_isum, int32_t *dump_imin,
                        const OgmActDev *act_base = nullptr);

// Enqueues quantize + kernels for tokens of x_dev into the targets' outputs.  Caller holds the
// lock and has checked that the targets share type and in_dim.
static int enqueue_matmul(ogm_ctx *ctx, const Target *tg, size_t n_tg, const float *x_dev,
                          uint32_t n_tokens, int decode, hipStream_t stream, int32_t *dump_isum,
                          int32_t *dump_imin) {
  if (n_tokens == 0 || n_tg == 0) return OGM_OK;
  const ogm_weight *w = tg[0].w;
  // A batch that may go to a matrix-core GEMM of the K-quants has its activations laid out in that kernel's
  // operand chunks by the quantizer itself (from 25 tokens: below, the small-batch kernel's loads gather few enough
  // distinct rows that the plain quantizer's shorter launch decides: 4096 -> 4096 at 24 tokens 11.5 us from rows,
  // 12.2 from chunks; at 32 tokens 14.3 against 12.5); which kernel runs is decided per launch.
  const bool with_xt = !dump_isum && !dump_imin && act_chunks_wanted(ctx, w->ggml_type, w->in_dim, n_tokens, decode, 25u);
  int rc = enqueue_quantize(ctx, act_mode_for(w->ggml_type, n_tokens, decode), x_dev, w->in_dim, n_tokens, stream, with_xt);
  if (rc != OGM_OK) return rc;
  return enqueue_gemv(ctx, tg, n_tg, n_tokens, decode, stream, dump_isum, dump_imin);
}

static int enqueue_matmul(ogm_ctx *ctx, const ogm_weight *w, const float *x_dev, uint32_t n_tokens,
                          float *y_dev, int decode, hipStream_t stream, int32_t *dump_isum,
                          int32_t *dump_imin) {
  const Target t{w, y_dev};
  return enqueue_matmul(ctx, &t, 1, x_dev, n_tokens, decode, stream, dump_isum, dump_imin);
}

// Builds the prefill planes of a K-quant matrix on first use, within the context's budget.  Returns
// whether the matrix has planes afterwards; a refusal (budget, memory) is remembered and is no
// error: the kernels then unpack the tile-planar bytes as before.  Caller holds the lock.
static bool ensure_planes(ogm_ctx *ctx, const ogm_weight *cw, hipStream_t stream) {
  ogm_weight *w = const_cast<ogm_weight *>(cw);   // the planes are a cache beside the weight's bytes
  if (w->planes) return true;
  if (w->planes_refused) return false;
  const size_t bytes = ogm_gemm_plane_bytes(w->ggml_type, w->in_dim, w->out_dim);
  const size_t budget = (size_t)ctx->tune_plane_cache_mb << 20;
  if (bytes == 0 || ctx->plane_bytes_used + bytes > budget) {
    w->planes_refused = bytes == 0;   // a budget may be raised later
    return false;
  }
  uint8_t *p = nullptr;
  if (hipMalloc((void **)&p, bytes) != hipSuccess) {
    (void)hipGetLastError();
    w->planes_refused = true;
    return false;
  }
  if (ogm_gemm_build_planes(w->ggml_type, w->dev, w->in_dim, w->out_dim, p, stream) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipFree(p);
    w->planes_refused = true;
    return false;
  }
  w->planes = p;
  w->plane_bytes = bytes;
  ctx->plane_bytes_used += bytes;
  return true;
}

static bool all_gemm_supported(const Target *tg, size_t n_tg, uint32_t n_tokens) {
  for (size_t i = 0; i < n_tg; i++)
    if (!ogm_gemm_supported(tg[i].w->ggml_type, tg[i].w->in_dim, tg[i].w->out_dim, n_tokens)) return false;
  return true;
}

// Enqueues the matmul kernels over the context's quantized activations.  Caller holds the lock.
// act_base: the quantized activations to read instead of the context's scratch; such a call stays
// on the GEMV kernels whatever the token count (the tiled GEMMs stage through context buffers).
static int enqueue_gemv(ogm_ctx *ctx, const Target *tg, size_t n_tg, uint32_t n_tokens, int decode,
                        hipStream_t stream, int32_t *dump_isum, int32_t *dump_imin, const OgmActDev *act_base) {
  const ogm_weight *w0 = tg[0].w;
  const int mode = act_mode_for(w0->ggml_type, n_tokens, decode);
  // backend/cpu.rs:55-167: matmul at n_tokens > 1 takes the GEMM kernels (their float order);
  // n_tokens == 1 and every matmul_decode take the GEMV's.
  const int gemm_order = (!decode && n_tokens > 1) ? 1 : 0;
  const uint32_t t0 = w0->ggml_type;
  // (the per-32 types: from nine tokens, more than a pass of the GEMV kernel holds, where their small-batch GEMM
  // would run -- Q8_0 2048 -> 2048 at 12 tokens 11 us against the GEMV kernel's 14, at 8 tokens 11 against 9 -- and
  // from seventeen otherwise)
  bool flat_small = block_elems_of(t0) == 32 && ctx->tune_gemm_small_max != 1;
  for (size_t i = 0; flat_small && i < n_tg; i++)
    flat_small = ogm_gemm_flat_small_batch(tg[i].w->ggml_type, tg[i].w->in_dim, tg[i].w->out_dim, n_tokens);
  const uint32_t gemm_from = ctx->tune_gemm_min_tokens ? (uint32_t)ctx->tune_gemm_min_tokens
                             : (t0 == OGM_Q4_K || t0 == OGM_Q5_K || t0 == OGM_Q6_K) ? 6u : (flat_small ? 9u : 17u);
  // A few tokens over a Q6_K matrix of many rows (the vocabulary projection of a decode batch): one
  // streaming pass on the matrix cores, in either float order.
  if (n_tokens > 1 && !dump_isum && !dump_imin && !act_base && ctx->tune_gemm_ft_min_rows >= 0) {
    bool all = true;
    for (size_t i = 0; i < n_tg; i++)
      all = all && ogm_gemm_ft_eligible(tg[i].w->ggml_type, tg[i].w->in_dim, tg[i].w->out_dim, n_tokens,
                                        (uint32_t)ctx->tune_gemm_ft_min_rows);
    if (all) {
      for (size_t i = 0; i < n_tg; i++) {
        OgmGemmArgs g;
        g.ggml_type = tg[i].w->ggml_type;
        g.wt = tg[i].w->dev;
        g.in_dim = tg[i].w->in_dim;
        g.out_dim = tg[i].w->out_dim;
        g.act = act_view(ctx, w0->in_dim, mode, 0);
        g.n_tokens = n_tokens;
        g.y = tg[i].y;
        g.xh = nullptr;
        HIPCHK(ctx, ogm_launch_gemm_ft(g, gemm_order, stream, &ctx->last_kernel));
      }
      return OGM_OK;
    }
  }
  // Two to sixteen tokens over a K-quant matrix (a speculative-decode verify batch, a decode batch): the GEMV's
  // distribution with the products on the matrix cores, in either float order.  Its workgroups stage all their
  // tokens' activations of the whole row in LDS, so what it wins depends on the row length and on how many
  // workgroups the launch has.  Measured on MI355X against what runs otherwise (the GEMV kernel up to five tokens,
  // the small-batch GEMM from six), whole calls, rows = all matrices of the launch:
  //   Q4_K, 5 / 8 tokens, us   4096 -> 4096  8.6 / 8.8 against 9.4 / 10.4;  4096 -> 28672  23.8 / 23.4 against 23.3 / 29.6;
  //     4096 -> 57344  42 / 40 against 46 / 49;  5120 -> 8192  11.7 / 12.2 against 13.9 / 15.9;  5120 -> 16384  20.7 / 23.9
  //     against 26.8 / 20.8;  8192 -> 4096  10.7 / 11.1 against 12.2 / 16.1;  8192 -> 8192  18.4 / 19.3 against 17.2 /
  //     18.4;  8192 -> 28672  72 / 78 against 49 / 53 (64 KB of activations a workgroup: one or two to a compute unit)
  //   Q6_K, 2 / 4 / 8 tokens   14336 -> 4096  18.5 / 18.2 / 21.2 against 15.9 / 20.3 / 23.8;  14336 -> 8192  34 / 36 / 42
  //     against 26 / 36 / 30;  8192 -> 4096  12.9 / 13.1 / 13.6 against 11.2 / 13.2 / 14.7;  8192 -> 8192  23 / 23.5 / 27
  //     against 18.6 / 22.5 / 19.4
  // Nine to sixteen tokens need sixteen token slots, whose activations and terms leave one workgroup of four
  // waves to a compute unit (gate and up at 16 tokens: 56 us against 18 for the small-batch GEMM): by default the
  // kernel stops at eight.
  uint64_t rows_all = 0;
  for (size_t i = 0; i < n_tg; i++) rows_all += tg[i].w->out_dim;
  bool mma_pays;
  if (t0 == OGM_Q6_K)
    mma_pays = (n_tokens >= 4 && n_tokens < gemm_from && rows_all <= 8192) || (n_tokens >= gemm_from && rows_all <= 4096);
  else
    mma_pays = n_tokens >= 5 && (w0->in_dim <= 4096 || (w0->in_dim <= 5120 && (n_tokens == 5 || rows_all <= 8192)) ||
                                 (w0->in_dim <= 8192 && rows_all <= 4096));
  const uint32_t mma_from = ctx->tune_gemv_mma == 2 ? 2u : (mma_pays ? 2u : 17u);
  const uint32_t mma_to = ctx->tune_gemv_mma == 2 ? 16u : 8u;
  if (ctx->tune_gemv_mma != 0 && n_tokens >= mma_from && n_tokens <= mma_to && !dump_isum && !dump_imin && !act_base &&
      ogm_gemv_mma_eligible(w0->ggml_type, w0->in_dim, n_tokens, gemm_order)) {
    for (size_t g0 = 0; g0 < n_tg; g0 += OGM_GEMV_MAX_MATS) {
      const size_t ng = n_tg - g0 < OGM_GEMV_MAX_MATS ? n_tg - g0 : OGM_GEMV_MAX_MATS;
      OgmGemvArgs a;
      a.ggml_type = w0->ggml_type;
      a.wt = tg[g0].w->dev;
      a.in_dim = w0->in_dim;
      a.out_dim = tg[g0].w->out_dim;
      a.act = act_view(ctx, w0->in_dim, mode, 0);
      a.n_tokens = n_tokens;
      a.y = tg[g0].y;
      a.gemm_order = gemm_order;
      a.wg_waves = (uint32_t)ctx->tune_wg_waves;
      a.dump_isum = nullptr;
      a.dump_imin = nullptr;
      a.n_extra = (uint32_t)ng - 1;
      for (size_t i = 1; i < ng; i++) {
        a.extra_wt[i - 1] = tg[g0 + i].w->dev;
        a.extra_out_dim[i - 1] = tg[g0 + i].w->out_dim;
        a.extra_y[i - 1] = tg[g0 + i].y;
      }
      HIPCHK(ctx, ogm_launch_gemv_mma(a, stream, &ctx->last_kernel));
    }
    return OGM_OK;
  }
  // (also below that count when the GEMV kernel's LDS holds fewer tokens of such long rows than the batch has and
  // it would read the weights once per part: Q6_K 53248 -> 16384 at 4 tokens 450 us against 180, Q4_K 16384 -> 16384
  // 65 against 52; Q8_0 4096 -> 4096 at 8 / 16 tokens 21 / 31 against 17 / 18, 14336 -> 4096 at 4 / 16 tokens 85 / 330
  // against 53 / 55 -- the per-32 types where their small-batch GEMM would run)
  const uint32_t gemv_chunk = ogm_gemv_max_tokens(w0->ggml_type, w0->in_dim, gemm_order);
  // (the per-32 types likewise, where their small-batch kernel would run: Q8_0 14336 -> 4096 at 2 tokens, two parts,
  // 43 us against 40.5; 11008 -> 4096 at 3 / 4 tokens 37 / 39 against 32)
  const uint32_t gemv_parts = gemv_chunk ? (n_tokens + gemv_chunk - 1u) / gemv_chunk : 0u;
  const bool gemv_rereads = gemv_parts > 1u && ctx->tune_gemm_min_tokens == 0 &&
                            (block_elems_of(w0->ggml_type) == 256 ||
                             flat_small);
  if (gemm_order && !dump_isum && !dump_imin && !act_base && (n_tokens >= gemm_from || gemv_rereads) &&
      all_gemm_supported(tg, n_tg, n_tokens)) {
    // enough tokens to fill MFMA tiles: the tiled GEMM (same values, weights read once per 128 tokens)
    int rc = ensure_dev(ctx, ctx->xh, ogm_gemm_xh_bytes(w0->in_dim, n_tokens));
    if (rc != OGM_OK) return rc;
    // K-quant matrices over the same input (q, k, v; gate, up) share a launch, up to OGM_GEMM_MAX_MATS
    const size_t per_launch = block_elems_of(w0->ggml_type) == 256 ? OGM_GEMM_MAX_MATS : 1;
    auto fill = [&](OgmGemmArgs &g, size_t i, size_t ng) {
      g.ggml_type = w0->ggml_type;
      g.wt = tg[i].w->dev;
      g.in_dim = w0->in_dim;
      g.out_dim = tg[i].w->out_dim;
      g.act = act_view(ctx, w0->in_dim, mode, 0);
      g.n_tokens = n_tokens;
      g.y = tg[i].y;
      g.xh = ctx->xh.p;
      g.xt_ready = ctx->act_xt && ctx->act_in_dim == w0->in_dim && ctx->act_tokens == n_tokens;
      g.tile_rows = (uint32_t)ctx->tune_gemm_tile_rows;
      g.medium = (uint32_t)ctx->tune_gemm_medium;
      g.small_max_tokens = (uint32_t)ctx->tune_gemm_small_max;
      g.sb_waves = (uint32_t)ctx->tune_gemm_sb_waves;
      g.plane_kernel = (uint32_t)ctx->tune_gemm_plane_kernel;
      g.one_pass = (uint32_t)ctx->tune_gemm_one_pass;
      g.interleave = (uint32_t)ctx->tune_gemm_interleave;
      g.n_extra = (uint32_t)ng - 1;
      for (size_t j = 1; j < ng; j++) {
        g.extra_wt[j - 1] = tg[i + j].w->dev;
        g.extra_out_dim[j - 1] = tg[i + j].w->out_dim;
        g.extra_y[j - 1] = tg[i + j].y;
      }
    };
    // Beyond its small batches IQ4_XS has GEMM kernels over its planes only: without them (no room, or shapes beyond
    // the plane kernels' 32-bit offsets) the batch stays on the GEMV kernel
    bool planes_or_nothing = true;
    for (size_t i = 0; w0->ggml_type == OGM_IQ4_XS && planes_or_nothing && i < n_tg; i += per_launch) {
      const size_t ng = n_tg - i < per_launch ? n_tg - i : per_launch;
      OgmGemmArgs g;
      fill(g, i, ng);
      if (ogm_gemm_takes_small_batch(g)) continue;
      planes_or_nothing = ogm_gemm_uses_planes(g);
      for (size_t j = 0; planes_or_nothing && j < ng; j++) planes_or_nothing = ensure_planes(ctx, tg[i + j].w, stream);
    }
    for (size_t i = 0; planes_or_nothing && i < n_tg; i += per_launch) {
      const size_t ng = n_tg - i < per_launch ? n_tg - i : per_launch;
      OgmGemmArgs g;
      fill(g, i, ng);
      if (ogm_gemm_uses_planes(g)) {
        // a tiled int8 kernel: over the matrices' planes when all of them have (or now get) theirs
        bool all = true;
        for (size_t j = 0; j < ng; j++) all = ensure_planes(ctx, tg[i + j].w, stream) && all;
        if (all) {
          g.planes = tg[i].w->planes;
          for (size_t j = 1; j < ng; j++) g.extra_planes[j - 1] = tg[i + j].w->planes;
        }
      }
      HIPCHK(ctx, ogm_launch_gemm(g, stream, &ctx->last_kernel));
    }
    if (planes_or_nothing) return OGM_OK;
  }
  const uint32_t wg_waves = (uint32_t)ctx->tune_wg_waves;
  const uint32_t chunk = gemv_chunk;
  if (chunk == 0) return fail(ctx, OGM_ERR_UNSUPPORTED, "no kernel for this type");
  const uint32_t blocks_per_row = w0->in_dim / block_elems_of(w0->ggml_type);
  for (size_t g0 = 0; g0 < n_tg; g0 += OGM_GEMV_MAX_MATS) {
    const size_t ng = n_tg - g0 < OGM_GEMV_MAX_MATS ? n_tg - g0 : OGM_GEMV_MAX_MATS;
    for (uint32_t t0 = 0; t0 < n_tokens; t0 += chunk) {
      OgmGemvArgs a;
      a.ggml_type = w0->ggml_type;
      a.wt = tg[g0].w->dev;
      a.in_dim = w0->in_dim;
      a.out_dim = tg[g0].w->out_dim;
      a.act = act_base ? act_offset(*act_base, w0->in_dim, mode, t0) : act_view(ctx, w0->in_dim, mode, t0);
      a.n_tokens = n_tokens - t0 < chunk ? n_tokens - t0 : chunk;
      a.y = tg[g0].y + (size_t)t0 * a.out_dim;
      a.gemm_order = gemm_order;
      a.wg_waves = wg_waves;
      a.dump_isum = dump_isum ? dump_isum + (size_t)t0 * a.out_dim * blocks_per_row : nullptr;
      a.dump_imin = dump_imin ? dump_imin + (size_t)t0 * a.out_dim * blocks_per_row : nullptr;
      a.n_extra = (uint32_t)ng - 1;
      for (size_t i = 1; i < ng; i++) {
        a.extra_wt[i - 1] = tg[g0 + i].w->dev;
        a.extra_out_dim[i - 1] = tg[g0 + i].w->out_dim;
        a.extra_y[i - 1] = tg[g0 + i].y + (size_t)t0 * tg[g0 + i].w->out_dim;
      }
      HIPCHK(ctx, ogm_launch_gemv(a, stream, &ctx->last_kernel));
    }
  }
  return OGM_OK;
}

static int check_matmul_args(ogm_ctx *ctx, const ogm_weight *w, const void *x, const void *y,
                             uint32_t n_tokens) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!w) return fail(ctx, OGM_ERR_INVALID, "weight is null");
  if (n_tokens != 0 && (!x || !y)) return fail(ctx, OGM_ERR_INVALID, "x or y is null");
  return OGM_OK;
}

// Host-pointer calls whose x and y together stay under this size skip the copy engine: the pinned
// staging buffers are device-visible, and the quantizer and the matmul kernels use them in place.
#define OGM_ZERO_COPY_MAX (512u << 10)
static bool zero_copy(const ogm_ctx *ctx, size_t bytes) {
  return ctx->tune_host_zero_copy != 0 && ctx->host_coherent && bytes <= OGM_ZERO_COPY_MAX;
}

// Waits for what a host-pointer call has enqueued on the context's stream.  A zero-copy call's results land
// in pinned memory by the kernels' own stores, so the host need not go through the runtime's completion
// signal (measured: 6 us from the last kernel's end to hipStreamSynchronize's return): a one-thread kernel
// behind the call's kernels stores the call's number to a pinned word and the host polls that word
// (4096 -> 14336: 19 us a call against 23).  Bounded: if the word has not come after a few milliseconds --
// or a kernel has faulted -- the stream is synchronized after all and reports.  Every 256th call synchronizes
// anyway, so the runtime can retire its records of the launches.
static int host_wait(ogm_ctx *ctx, bool zero_copied) {
  if (!zero_copied || !ctx->host_coherent || ctx->tune_host_flag_wait == 0 || ++ctx->flag_unsynced >= 256u) {
    ctx->flag_unsynced = 0;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return OGM_OK;
  }
  if (!ctx->hflag.p) {
    HIPCHK(ctx, host_alloc_coherent(ctx, &ctx->hflag.p, 4096));
    ctx->hflag.cap = 4096;
    *(volatile uint32_t *)ctx->hflag.p = 0;
    if (!ctx->host_coherent) {   // refused just now: this call's y sits in plain pinned memory, so wait on the stream
      ctx->flag_unsynced = 0;
      HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
      return OGM_OK;
    }
  }
  const uint32_t epoch = ++ctx->flag_epoch;
  uint32_t *flag = (uint32_t *)ctx->hflag.p;
  // (2: the kernel stores another number, so the wait below runs into its bound -- for tests of that path)
  HIPCHK(ctx, ogm_launch_host_flag(flag, ctx->tune_host_flag_wait == 2 ? epoch ^ 0x80000000u : epoch, ctx->stream));
  const auto t0 = std::chrono::steady_clock::now();
  for (uint32_t spins = 0; __atomic_load_n(flag, __ATOMIC_ACQUIRE) != epoch; spins++) {
    __builtin_ia32_pause();
    if ((spins & 1023u) == 1023u && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(5)) {
      ctx->flag_unsynced = 0;
      HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
      return OGM_OK;
    }
  }
  return OGM_OK;
}

static int host_matmul(ogm_ctx *ctx, const ogm_weight *w, const float *x, uint32_t n_tokens,
                       float *y, int decode) {
  int rc = check_matmul_args(ctx, w, x, y, n_tokens);
  if (rc != OGM_OK) return rc;
  if (n_tokens == 0) return OGM_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  const size_t xb = (size_t)n_tokens * w->in_dim * 4, yb = (size_t)n_tokens * w->out_dim * 4;
  if ((rc = ensure_host(ctx, ctx->hx, xb)) != OGM_OK) return rc;
  if ((rc = ensure_host(ctx, ctx->hy, yb)) != OGM_OK) return rc;
  memcpy(ctx->hx.p, x, xb);
  const bool zc = zero_copy(ctx, xb + yb);
  if (zc) {
    // a decode-sized call: the kernels read x from, and write y to, the pinned staging buffers over
    // the bus themselves; two copy-engine transfers and their latencies fall away
    rc = enqueue_matmul(ctx, w, (const float *)ctx->hx.p, n_tokens, (float *)ctx->hy.p, decode, ctx->stream,
                        nullptr, nullptr);
    if (rc != OGM_OK) return rc;
  } else {
    if ((rc = ensure_dev(ctx, ctx->x, xb)) != OGM_OK) return rc;
    if ((rc = ensure_dev(ctx, ctx->y, yb)) != OGM_OK) return rc;
    HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, ctx->hx.p, xb, hipMemcpyHostToDevice, ctx->stream));
    rc = enqueue_matmul(ctx, w, (const float *)ctx->x.p, n_tokens, (float *)ctx->y.p, decode,
                        ctx->stream, nullptr, nullptr);
    if (rc != OGM_OK) return rc;
    HIPCHK(ctx, hipMemcpyAsync(ctx->hy.p, ctx->y.p, yb, hipMemcpyDeviceToHost, ctx->stream));
  }
  if ((rc = host_wait(ctx, zc)) != OGM_OK) return rc;   // (polling hipStreamQuery measured slower than hipStreamSynchronize)
  memcpy(y, ctx->hy.p, yb);
  return OGM_OK;
}

extern "C" int ogm_matmul(ogm_ctx *ctx, const ogm_weight *w, const float *x, uint32_t n_tokens,
                          float *y) {
  return host_matmul(ctx, w, x, n_tokens, y, 0);
}

extern "C" int ogm_matmul_decode(ogm_ctx *ctx, const ogm_weight *w, const float *x,
                                 uint32_t n_tokens, float *y) {
  return host_matmul(ctx, w, x, n_tokens, y, 1);
}

extern "C" int ogm_matmul_dev(ogm_ctx *ctx, const ogm_weight *w, const float *x_dev,
                              uint32_t n_tokens, float *y_dev, int decode, void *stream) {
  int rc = check_matmul_args(ctx, w, x_dev, y_dev, n_tokens);
  if (rc != OGM_OK) return rc;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  return enqueue_matmul(ctx, w, x_dev, n_tokens, y_dev, decode, s, nullptr, nullptr);
}

// ogm_matmul_dev for callers that cannot allocate: the quantized activations go to the library's
// static device array instead of the context's grown-on-demand scratch, and only the GEMV kernels
// run.  No hipMalloc, hipFree or allocating routine is reached from here.
extern "C" int ogm_matmul_dev_static(ogm_ctx *ctx, const ogm_weight *w, const float *x_dev, uint32_t n_tokens,
                                     float *y_dev, int decode, void *stream) {
  int rc = check_matmul_args(ctx, w, x_dev, y_dev, n_tokens);
  if (rc != OGM_OK) return rc;
  if (n_tokens == 0) return OGM_OK;
  if (n_tokens > OGM_STATIC_MAX_TOKENS || (uint64_t)n_tokens * w->in_dim > OGM_STATIC_MAX_ELEMS)
    return fail(ctx, OGM_ERR_INVALID,
                "ogm_matmul_dev_static: at most " + std::to_string(OGM_STATIC_MAX_TOKENS) + " tokens and " +
                    std::to_string(OGM_STATIC_MAX_ELEMS) + " activations (n_tokens * in_dim) fit the static scratch; got " +
                    std::to_string(n_tokens) + " x " + std::to_string(w->in_dim));
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  const int mode = act_mode_for(w->ggml_type, n_tokens, decode);
  const OgmActDev act = ogm_static_act_view(ctx->static_scratch);
  // The quantizer writes every value the kernels below read for these tokens: nothing in the
  // array has to start at zero, and what an earlier call left beyond them is never read.
  HIPCHK(ctx, ogm_launch_quantize(mode, x_dev, w->in_dim, n_tokens, act, s));
  const Target t{w, y_dev};
  return enqueue_gemv(ctx, &t, 1, n_tokens, decode, s, nullptr, nullptr, &act);
}

// For benchmarks driven from an interpreter: runs host-pointer calls `reps` times from compiled code and
// records each repetition's wall time.  A repetition walks one variant's ops (variant = rep % n_variants,
// so that weights rotate), split into groups: a group of one op is an ogm_matmul, a longer one an
// ogm_matmul_batch.
extern "C" int ogm_time_host_calls(ogm_ctx *ctx, const ogm_op *ops, size_t n_ops, size_t n_variants,
                                   const uint32_t *group_sizes, size_t n_groups, uint32_t reps, double *us_out) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!ops || !group_sizes || !us_out || n_ops == 0 || n_variants == 0 || n_groups == 0)
    return fail(ctx, OGM_ERR_INVALID, "ogm_time_host_calls: null or empty argument");
  size_t sum = 0;
  for (size_t g = 0; g < n_groups; g++) sum += group_sizes[g];
  if (sum != n_ops) return fail(ctx, OGM_ERR_INVALID, "ogm_time_host_calls: group sizes do not add up to n_ops");
  for (uint32_t r = 0; r < reps; r++) {
    const ogm_op *v = ops + (r % n_variants) * n_ops;
    const auto t0 = std::chrono::steady_clock::now();
    size_t at = 0;
    for (size_t g = 0; g < n_groups; g++) {
      const int rc = group_sizes[g] == 1 ? ogm_matmul(ctx, v[at].w, v[at].x, v[at].n_tokens, v[at].y)
                                         : ogm_matmul_batch(ctx, v + at, group_sizes[g], 0, 0);
      if (rc != OGM_OK) return rc;
      at += group_sizes[g];
    }
    us_out[r] = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
  }
  return OGM_OK;
}

// The device bytes of up to four weights streamed through one read-only launch (for benchmarks: the
// rate the memory system gives this footprint with nothing behind the loads).
extern "C" int ogm_weights_read_probe(ogm_ctx *ctx, const ogm_weight *const *ws, size_t n_ws, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (n_ws == 0) return OGM_OK;
  if (!ws || n_ws > OGM_PROBE_MAX_BUFS) return fail(ctx, OGM_ERR_INVALID, "ogm_weights_read_probe takes 1..4 weights");
  const uint8_t *bufs[OGM_PROBE_MAX_BUFS];
  size_t bytes[OGM_PROBE_MAX_BUFS];
  for (size_t i = 0; i < n_ws; i++) {
    if (!ws[i] || ws[i]->device_bytes < 9216) return fail(ctx, OGM_ERR_INVALID, "a weight is null or under 9 KiB");
    bufs[i] = ws[i]->dev;
    bytes[i] = ws[i]->device_bytes;
  }
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  int rc = ensure_dev(ctx, ctx->probe_sink, 256);
  if (rc != OGM_OK) return rc;
  HIPCHK(ctx, ogm_launch_read_probe(bufs, bytes, (uint32_t)n_ws, (uint32_t *)ctx->probe_sink.p, s));
  ctx->last_kernel = "ogm_read_probe_kernel";
  return OGM_OK;
}

// A launch that does nothing, `workgroups` workgroups wide (for benchmarks: the cost of a kernel boundary).
extern "C" int ogm_empty_launch(ogm_ctx *ctx, uint32_t workgroups, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (workgroups == 0 || workgroups > (1u << 20)) return fail(ctx, OGM_ERR_INVALID, "ogm_empty_launch takes 1..1048576 workgroups");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  int rc = ensure_dev(ctx, ctx->probe_sink, 256);
  if (rc != OGM_OK) return rc;
  HIPCHK(ctx, ogm_launch_empty(workgroups, (uint32_t *)ctx->probe_sink.p, s));
  ctx->last_kernel = "ogm_empty_kernel";
  return OGM_OK;
}

static int act_quantize_dev(ogm_ctx *ctx, uint32_t ggml_type, const float *x_dev, uint32_t in_dim, uint32_t n_tokens,
                            int decode, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!ogm_supports(ggml_type, in_dim)) return fail(ctx, OGM_ERR_UNSUPPORTED, "type / in_dim without a kernel");
  if (n_tokens == 0) return OGM_OK;
  if (!x_dev) return fail(ctx, OGM_ERR_INVALID, "x is null");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  return enqueue_quantize(ctx, act_mode_for(ggml_type, n_tokens, decode), x_dev, in_dim, n_tokens, s,
                          act_chunks_wanted(ctx, ggml_type, in_dim, n_tokens, decode, 25u));
}

// The activation mode of Backend::matmul (for Q2_K at several tokens: per 32, cpu.rs:113-163) ...
extern "C" int ogm_act_quantize_dev(ogm_ctx *ctx, uint32_t ggml_type, const float *x_dev,
                                    uint32_t in_dim, uint32_t n_tokens, void *stream) {
  return act_quantize_dev(ctx, ggml_type, x_dev, in_dim, n_tokens, 0, stream);
}

// ... and of Backend::matmul_decode (per 256 for Q2_K too: its k_row dot, cpu.rs:265-317).  The two differ for
// Q2_K at several tokens only.
extern "C" int ogm_act_quantize_decode_dev(ogm_ctx *ctx, uint32_t ggml_type, const float *x_dev,
                                           uint32_t in_dim, uint32_t n_tokens, void *stream) {
  return act_quantize_dev(ctx, ggml_type, x_dev, in_dim, n_tokens, 1, stream);
}

// Why the activation buffer does not fit a two-step call, in the caller's terms.
static std::string act_mismatch(const ogm_ctx *ctx, const ogm_weight *w, uint32_t n_tokens, int decode) {
  const int want = act_mode_for(w->ggml_type, n_tokens, decode);
  if (ctx->act_mode >= 0 && ctx->act_mode != want && ctx->act_in_dim == w->in_dim && ctx->act_tokens >= n_tokens)
    return std::string("the activations were quantized per ") + (ctx->act_mode == OGM_ACT_PER_32 ? "32" : "256") +
           " and this call needs per " + (want == OGM_ACT_PER_32 ? "32" : "256") +
           (w->ggml_type == OGM_Q2_K ? " (Q2_K at several tokens: ogm_act_quantize_dev serves decode = 0, "
                                       "ogm_act_quantize_decode_dev serves decode = 1)"
                                     : " (quantize with this weight's type)");
  return "the quantized activations do not fit this weight (call ogm_act_quantize_dev, or for decode = 1 "
         "ogm_act_quantize_decode_dev, with its type, in_dim and token count first)";
}

extern "C" int ogm_matmul_act_dev(ogm_ctx *ctx, const ogm_weight *w, uint32_t n_tokens,
                                  float *y_dev, int decode, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!w) return fail(ctx, OGM_ERR_INVALID, "weight is null");
  if (n_tokens == 0) return OGM_OK;
  if (!y_dev) return fail(ctx, OGM_ERR_INVALID, "y is null");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (ctx->act_mode != act_mode_for(w->ggml_type, n_tokens, decode) || ctx->act_in_dim != w->in_dim ||
      ctx->act_tokens < n_tokens)
    return fail(ctx, OGM_ERR_INVALID, act_mismatch(ctx, w, n_tokens, decode));
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  const Target t{w, y_dev};
  return enqueue_gemv(ctx, &t, 1, n_tokens, decode, s, nullptr, nullptr);
}

// Checks a group of weights and collects its targets.
static int group_targets(ogm_ctx *ctx, const ogm_weight *const *ws, size_t n_ws, const void *x,
                         uint32_t n_tokens, float *const *ys_dev, std::vector<Target> &tg) {
  if (!ws || !ys_dev) return fail(ctx, OGM_ERR_INVALID, "ws or ys is null");
  tg.resize(n_ws);
  for (size_t i = 0; i < n_ws; i++) {
    int rc = check_matmul_args(ctx, ws[i], x, ys_dev[i], n_tokens);
    if (rc != OGM_OK) return rc;
    if (ws[i]->ggml_type != ws[0]->ggml_type || ws[i]->in_dim != ws[0]->in_dim)
      return fail(ctx, OGM_ERR_INVALID, "weights of one call must share type and in_dim");
    tg[i] = Target{ws[i], ys_dev[i]};
  }
  return OGM_OK;
}

extern "C" int ogm_matmul_multi_dev(ogm_ctx *ctx, const ogm_weight *const *ws, size_t n_ws,
                                    const float *x_dev, uint32_t n_tokens, float *const *ys_dev,
                                    int decode, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (n_ws == 0) return OGM_OK;
  std::vector<Target> tg;
  int rc = group_targets(ctx, ws, n_ws, x_dev, n_tokens, ys_dev, tg);
  if (rc != OGM_OK) return rc;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  return enqueue_matmul(ctx, tg.data(), n_ws, x_dev, n_tokens, decode, s, nullptr, nullptr);
}

extern "C" int ogm_matmul_multi_act_dev(ogm_ctx *ctx, const ogm_weight *const *ws, size_t n_ws,
                                        uint32_t n_tokens, float *const *ys_dev, int decode,
                                        void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (n_ws == 0 || n_tokens == 0) return OGM_OK;
  std::vector<Target> tg;
  int rc = group_targets(ctx, ws, n_ws, ys_dev /* stands in for x: only null-checked */, n_tokens, ys_dev, tg);
  if (rc != OGM_OK) return rc;
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (ctx->act_mode != act_mode_for(ws[0]->ggml_type, n_tokens, decode) || ctx->act_in_dim != ws[0]->in_dim ||
      ctx->act_tokens < n_tokens)
    return fail(ctx, OGM_ERR_INVALID, act_mismatch(ctx, ws[0], n_tokens, decode));
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  return enqueue_gemv(ctx, tg.data(), n_ws, n_tokens, decode, s, nullptr, nullptr);
}

// `reps` launches enqueued back to back from compiled code (for benchmarks driven from an interpreter, whose
// own call overhead would otherwise leave the device idle between short kernels, under a profiler above all).
extern "C" int ogm_enqueue_repeated(ogm_ctx *ctx, int kind, const ogm_weight *const *ws, size_t n_ws, size_t n_variants,
                                    uint32_t n_tokens, float *const *ys_dev, int decode, uint32_t first,
                                    uint32_t reps, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (kind < 0 || kind > 2) return fail(ctx, OGM_ERR_INVALID, "ogm_enqueue_repeated: kind is 0, 1 or 2");
  if (kind != 2 && (!ws || n_ws == 0 || n_variants == 0)) return fail(ctx, OGM_ERR_INVALID, "ogm_enqueue_repeated: no weights");
  for (uint32_t r = 0; r < reps; r++) {
    const ogm_weight *const *set = kind == 2 ? nullptr : ws + ((size_t)first + r) % n_variants * n_ws;
    int rc = kind == 0   ? ogm_matmul_multi_act_dev(ctx, set, n_ws, n_tokens, ys_dev, decode, stream)
             : kind == 1 ? ogm_weights_read_probe(ctx, set, n_ws, stream)
                         : ogm_empty_launch(ctx, n_tokens, stream);
    if (rc != OGM_OK) return rc;
  }
  return OGM_OK;
}

// Backend::matmul_batch (backend/mod.rs:362-366) with guarded_matmul_op's token stripes
// (backend/mod.rs:154-172): every stripe of every op is enqueued, then one synchronization.
extern "C" int ogm_matmul_batch(ogm_ctx *ctx, const ogm_op *ops, size_t n_ops, int decode,
                                uint32_t max_tokens_per_phase) {
  if (!ctx) return OGM_ERR_INVALID;
  if (n_ops == 0) return OGM_OK;
  if (!ops) return fail(ctx, OGM_ERR_INVALID, "ops is null");
  const uint32_t cap = max_tokens_per_phase ? max_tokens_per_phase : 256;
  for (size_t i = 0; i < n_ops; i++) {
    int rc = check_matmul_args(ctx, ops[i].w, ops[i].x, ops[i].y, ops[i].n_tokens);
    if (rc != OGM_OK) return rc;
  }
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  // Every op gets its own slice of the transfer buffers; the activation scratch is shared,
  // which is safe because one stream runs each quantize after the kernels that read the last.
  // Ops that read the very same host slice (q/k/v, gate/up) share one device copy of it.
  // src[i] is the first op whose device copy of x op i shares (itself when it brings its own).  An
  // op without tokens brings and shares nothing, so it never stands in for a later op's input.
  std::vector<size_t> xoff(n_ops), yoff(n_ops), src(n_ops);
  size_t xb = 0, yb = 0;
  for (size_t i = 0; i < n_ops; i++) {
    size_t j = i;
    if (ops[i].n_tokens != 0) {
      j = 0;
      while (j < i && !(ops[j].n_tokens != 0 && ops[j].x == ops[i].x && ops[j].n_tokens == ops[i].n_tokens &&
                        ops[j].w->in_dim == ops[i].w->in_dim))
        j++;
    }
    src[i] = j;
    if (j < i) {
      xoff[i] = xoff[j];
    } else {
      xoff[i] = xb;
      xb += (size_t)ops[i].n_tokens * ops[i].w->in_dim * 4;
    }
    yoff[i] = yb;
    yb += (size_t)ops[i].n_tokens * ops[i].w->out_dim * 4;
  }
  if (xb == 0) return OGM_OK;
  int rc;
  if ((rc = ensure_host(ctx, ctx->hx, xb)) != OGM_OK) return rc;
  if ((rc = ensure_host(ctx, ctx->hy, yb)) != OGM_OK) return rc;
  const bool zc = zero_copy(ctx, xb + yb);   // see host_matmul (after the staging buffers exist: it asks whether they are coherent)
  if (!zc) {
    if ((rc = ensure_dev(ctx, ctx->x, xb)) != OGM_OK) return rc;
    if ((rc = ensure_dev(ctx, ctx->y, yb)) != OGM_OK) return rc;
  }
  uint8_t *const x_base = (uint8_t *)(zc ? ctx->hx.p : ctx->x.p), *const y_base = (uint8_t *)(zc ? ctx->hy.p : ctx->y.p);
  // Size the activation scratch for the largest stripe before anything is enqueued, so it is
  // never reallocated under kernels in flight.
  for (size_t i = 0; i < n_ops; i++) {
    uint32_t t = ops[i].n_tokens < cap ? ops[i].n_tokens : cap;
    if ((rc = ensure_act(ctx, ops[i].w->in_dim, t)) != OGM_OK) return rc;
  }
  for (size_t i = 0; i < n_ops; i++) {
    const ogm_op &op = ops[i];
    const size_t bytes = (size_t)op.n_tokens * op.w->in_dim * 4;
    if (bytes && src[i] == i) memcpy((uint8_t *)ctx->hx.p + xoff[i], op.x, bytes);
  }
  if (!zc) HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, ctx->hx.p, xb, hipMemcpyHostToDevice, ctx->stream));
  std::vector<Target> tg;
  for (size_t i = 0; i < n_ops;) {
    // a run of neighbouring ops over one input and one weight type: one group
    size_t e = i + 1;
    while (e < n_ops && ops[i].n_tokens != 0 && src[e] == src[i] && ops[e].n_tokens == ops[i].n_tokens &&
           ops[e].w->ggml_type == ops[i].w->ggml_type && ops[e].w->in_dim == ops[i].w->in_dim)
      e++;
    const ogm_op &op = ops[i];
    const float *xd = (const float *)(x_base + xoff[i]);
    for (uint32_t t0 = 0; t0 < op.n_tokens; t0 += cap) {
      const uint32_t nt = op.n_tokens - t0 < cap ? op.n_tokens - t0 : cap;
      tg.clear();
      for (size_t k = i; k < e; k++)
        tg.push_back(Target{ops[k].w, (float *)(y_base + yoff[k]) + (size_t)t0 * ops[k].w->out_dim});
      rc = enqueue_matmul(ctx, tg.data(), tg.size(), xd + (size_t)t0 * op.w->in_dim, nt, decode,
                          ctx->stream, nullptr, nullptr);
      if (rc != OGM_OK) return rc;
    }
    i = e;
  }
  if (!zc) HIPCHK(ctx, hipMemcpyAsync(ctx->hy.p, ctx->y.p, yb, hipMemcpyDeviceToHost, ctx->stream));
  if ((rc = host_wait(ctx, zc)) != OGM_OK) return rc;
  size_t yo = 0;
  for (size_t i = 0; i < n_ops; i++) {
    const size_t bytes = (size_t)ops[i].n_tokens * ops[i].w->out_dim * 4;
    if (bytes) memcpy(ops[i].y, (uint8_t *)ctx->hy.p + yo, bytes);
    yo += bytes;
  }
  return OGM_OK;
}

// ------------------------------------------------------------------------------------------
// integer stage, exposed

extern "C" int ogm_quantize_act(ogm_ctx *ctx, int mode, const float *x, size_t n, int8_t *q,
                                float *d, int32_t *sums) {
  if (!ctx) return OGM_ERR_INVALID;
  if (mode != OGM_ACT_PER_32 && mode != OGM_ACT_PER_256) return fail(ctx, OGM_ERR_INVALID, "bad mode");
  const size_t group = mode == OGM_ACT_PER_32 ? 32 : 256;
  if (n == 0) return OGM_OK;
  if (!x || !q || !d) return fail(ctx, OGM_ERR_INVALID, "null pointer");
  if (n % group != 0 || n > 0xFFFFFF00u) return fail(ctx, OGM_ERR_INVALID, "n is not a whole number of groups");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  int rc;
  if ((rc = ensure_dev(ctx, ctx->x, n * 4)) != OGM_OK) return rc;
  if ((rc = ensure_act(ctx, (uint32_t)n, 1)) != OGM_OK) return rc;
  HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, x, n * 4, hipMemcpyHostToDevice, ctx->stream));
  HIPCHK(ctx, ogm_launch_quantize(mode, (const float *)ctx->x.p, (uint32_t)n, 1,
                                  act_view(ctx, (uint32_t)n, mode, 0), ctx->stream));
  HIPCHK(ctx, hipMemcpyAsync(q, ctx->q.p, n, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipMemcpyAsync(d, ctx->d.p, n / group * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (sums) HIPCHK(ctx, hipMemcpyAsync(sums, ctx->sums.p, n / 16 * 4, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return OGM_OK;
}

// The quantizer as the multi-token matmuls launch it (one grid row per token), with everything it
// writes copied back.
extern "C" int ogm_quantize_act_tokens(ogm_ctx *ctx, int mode, const float *x, uint32_t in_dim, uint32_t n_tokens,
                                       int8_t *q, float *d, int32_t *sums, int16_t *bsum, uint16_t *bs16) {
  if (!ctx) return OGM_ERR_INVALID;
  if (mode != OGM_ACT_PER_32 && mode != OGM_ACT_PER_256) return fail(ctx, OGM_ERR_INVALID, "bad mode");
  const uint32_t group = mode == OGM_ACT_PER_32 ? 32u : 256u;
  if (n_tokens == 0) return OGM_OK;
  if (!x || !q || !d) return fail(ctx, OGM_ERR_INVALID, "null pointer");
  if (in_dim == 0 || in_dim % group != 0 || (uint64_t)in_dim * n_tokens > 0x7FFFFFFFu || n_tokens > 65535u)
    return fail(ctx, OGM_ERR_INVALID, "in_dim is not a whole number of groups, or the batch is too large");
  if (bs16 && mode != OGM_ACT_PER_256) return fail(ctx, OGM_ERR_INVALID, "the f16 sub-block sums exist per 256 only");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  const size_t n = (size_t)in_dim * n_tokens;
  int rc;
  if ((rc = ensure_dev(ctx, ctx->x, n * 4)) != OGM_OK) return rc;
  if ((rc = ensure_act(ctx, in_dim, n_tokens)) != OGM_OK) return rc;
  HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, x, n * 4, hipMemcpyHostToDevice, ctx->stream));
  HIPCHK(ctx, ogm_launch_quantize(mode, (const float *)ctx->x.p, in_dim, n_tokens, act_view(ctx, in_dim, mode, 0),
                                  ctx->stream));
  ctx->act_mode = -1;   // the scratch no longer holds what ogm_act_quantize_dev left
  HIPCHK(ctx, hipMemcpyAsync(q, ctx->q.p, n, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipMemcpyAsync(d, ctx->d.p, n / group * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (sums) HIPCHK(ctx, hipMemcpyAsync(sums, ctx->sums.p, n / 16 * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (bsum) HIPCHK(ctx, hipMemcpyAsync(bsum, ctx->bsum.p, n / 32 * 2, hipMemcpyDeviceToHost, ctx->stream));
  if (bs16) HIPCHK(ctx, hipMemcpyAsync(bs16, ctx->bs16.p, n / 16 * 2, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return OGM_OK;
}

extern "C" int ogm_dump_block_sums(ogm_ctx *ctx, const ogm_weight *w, const float *x,
                                   uint32_t n_tokens, int32_t *isum, int32_t *imin) {
  int rc = check_matmul_args(ctx, w, x, isum, n_tokens);
  if (rc != OGM_OK) return rc;
  if (n_tokens == 0) return OGM_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  const size_t blocks = (size_t)w->in_dim / block_elems_of(w->ggml_type);
  const size_t nb = (size_t)n_tokens * w->out_dim * blocks * 4;
  const size_t xb = (size_t)n_tokens * w->in_dim * 4, yb = (size_t)n_tokens * w->out_dim * 4;
  const bool want_min = imin && (w->ggml_type == OGM_Q4_K || w->ggml_type == OGM_Q5_K || w->ggml_type == OGM_Q2_K);
  if ((rc = ensure_dev(ctx, ctx->x, xb)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->y, yb)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->isum, nb)) != OGM_OK) return rc;
  if (want_min && (rc = ensure_dev(ctx, ctx->imin, nb)) != OGM_OK) return rc;
  HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, x, xb, hipMemcpyHostToDevice, ctx->stream));
  rc = enqueue_matmul(ctx, w, (const float *)ctx->x.p, n_tokens, (float *)ctx->y.p, 1, ctx->stream,
                      (int32_t *)ctx->isum.p, want_min ? (int32_t *)ctx->imin.p : nullptr);
  if (rc != OGM_OK) return rc;
  HIPCHK(ctx, hipMemcpyAsync(isum, ctx->isum.p, nb, hipMemcpyDeviceToHost, ctx->stream));
  if (want_min) HIPCHK(ctx, hipMemcpyAsync(imin, ctx->imin.p, nb, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return OGM_OK;
}

extern "C" int ogm_f16_to_f32(ogm_ctx *ctx, const uint16_t *bits, size_t n, float *out) {
  if (!ctx) return OGM_ERR_INVALID;
  if (n == 0) return OGM_OK;
  if (!bits || !out) return fail(ctx, OGM_ERR_INVALID, "null pointer");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  int rc;
  if ((rc = ensure_dev(ctx, ctx->x, n * 2)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->y, n * 4)) != OGM_OK) return rc;
  HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, bits, n * 2, hipMemcpyHostToDevice, ctx->stream));
  HIPCHK(ctx, ogm_launch_f16_to_f32((const uint16_t *)ctx->x.p, n, (float *)ctx->y.p, ctx->stream));
  HIPCHK(ctx, hipMemcpyAsync(out, ctx->y.p, n * 4, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return OGM_OK;
}

// ------------------------------------------------------------------------------------------
// Llama-family decode step

#include <math.h>

#include "ogm_llama.h"

struct ogm_llama {
  ogm_llama_config cfg;
  std::vector<ogm_llama_layer> layers;  // weight handles; the optional vectors as device pointers
  const ogm_weight *output = nullptr;
  // device memory
  float *norms = nullptr;     // [n_layer][2][n_embd] then output_norm [n_embd]
  float *pre = nullptr;       // [n_layer][q_bias qd | k_bias kvd | v_bias kvd | q_norm hd | k_norm hd]
  float *freq = nullptr;      // [rope_dim / 2], frequency factors applied
  float *rope_cs = nullptr;   // [rope_dim / 2] (cos, sin) of the token being decoded
  float *rope_all = nullptr;  // the same for every position of the cache, filled at creation (null: too large, computed per token)
  uint32_t *attn_counters = nullptr;  // [2 n_head_kv parts][OGM_ATTN_TICKET_STRIDE] the attention kernel's tickets, a line each; zero between launches
  void *k_cache = nullptr;    // f16 [n_layer][max_ctx][kv_dim]
  void *v_cache = nullptr;
  float *x = nullptr;         // hidden state [n_embd]
  float *q = nullptr, *k = nullptr, *v = nullptr;  // projections
  float *proj = nullptr;      // wo / down output [n_embd]
  float *gate = nullptr, *up = nullptr;            // [n_ff]
  float *part_o = nullptr, *part_ml = nullptr;     // attention partials
  float *logits = nullptr;    // [n_vocab]
  uint32_t *amax_scratch = nullptr, *amax_out = nullptr;
  // ogm_llama_forward_all_logits: every position's logits and greedy token, allocated at its first call
  float *logits_all = nullptr;      // [OGM_ALL_LOGITS_MAX_TOKENS][n_vocab]
  uint32_t *amax_all = nullptr;     // [OGM_ALL_LOGITS_MAX_TOKENS]
  float *stage = nullptr;     // host->device staging for ogm_llama_kv_write
  size_t stage_cap = 0;
  // prefill rows, allocated at the first prefill for the pass size of that moment (prefill_chunk_tokens)
  struct Prefill {
    float *x = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr;
    float *proj = nullptr, *gate = nullptr, *up = nullptr, *cs = nullptr;
    float *part_o = nullptr, *part_ml = nullptr;   // attn_prefill_variant 1 only, allocated when it first runs
    uint32_t *tokens = nullptr;
    uint32_t attn_tokens = 0;   // query rows one attention launch takes (bounded by part_o)
    uint32_t chunk = 0;         // tokens per pass over the layers: what the rows above were allocated for
    bool ready = false;
  } pf;
  uint32_t max_splits = 0;
  // debug capture (ogm_llama_debug_capture): the quantized activations every matmul group of the
  // last decode step read, site after site, cap_width bytes of q and cap_width / 32 scales each
  bool cap_on = false;
  int8_t *cap_q = nullptr;   // allocated when capture is first switched on, freed with the model
  float *cap_d = nullptr;
  uint32_t cap_width = 0;
  std::vector<uint32_t> cap_n, cap_group;   // per site: elements and quantizer group of the last step
  std::vector<void *> allocs;
};

static int llama_alloc(ogm_ctx *ctx, ogm_llama *m, void **p, size_t bytes) {
  HIPCHK(ctx, hipMalloc(p, bytes ? bytes : 1));
  m->allocs.push_back(*p);
  return OGM_OK;
}

static void llama_free(ogm_llama *m) {
  for (void *p : m->allocs) (void)hipFree(p);
  if (m->stage) (void)hipFree(m->stage);
  delete m;
}

static bool llama_weight_ok(const ogm_weight *w, uint32_t in_dim, uint32_t out_dim) {
  return w && w->in_dim == in_dim && w->out_dim == out_dim;
}

extern "C" int ogm_llama_create(ogm_ctx *ctx, const ogm_llama_config *cfg, const ogm_llama_layer *layers,
                                const float *output_norm, const ogm_weight *output, ogm_llama **out) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!cfg || !layers || !output_norm || !output || !out) return fail(ctx, OGM_ERR_INVALID, "null argument");
  const ogm_llama_config c = *cfg;
  if (c.n_layer == 0 || c.n_embd == 0 || c.n_head == 0 || c.n_head_kv == 0 || c.n_ff == 0 || c.max_ctx == 0)
    return fail(ctx, OGM_ERR_INVALID, "empty model dimension");
  const uint32_t gq = c.n_head % c.n_head_kv == 0 ? c.n_head / c.n_head_kv : 0;
  if (gq < 1 || ogm_attn_head_parts(gq) == 0)
    return fail(ctx, OGM_ERR_UNSUPPORTED, "query heads per K/V head must be 1 to 8, or up to 64 in equal parts of at most 8");
  if (c.rope_neox > 1) return fail(ctx, OGM_ERR_INVALID, "rope_neox is 0 (NORM pairs) or 1 (NEOX pairs)");
  if (c.rope_freq_factors)
    for (uint32_t i = 0; i < c.rope_dim / 2; i++)
      if (!(c.rope_freq_factors[i] != 0.0f)) return fail(ctx, OGM_ERR_INVALID, "rope frequency factor of zero");
  if (c.head_dim != 64 && c.head_dim != 128) return fail(ctx, OGM_ERR_UNSUPPORTED, "head_dim must be 64 or 128");
  if (c.rope_dim > c.head_dim || c.rope_dim % 2 != 0) return fail(ctx, OGM_ERR_INVALID, "bad rope_dim");
  if (c.n_embd > 16384 || c.n_embd % 32 != 0 || c.n_ff % 32 != 0)
    return fail(ctx, OGM_ERR_UNSUPPORTED, "n_embd must be a multiple of 32 up to 16384, n_ff a multiple of 32");
  const uint32_t qd = c.n_head * c.head_dim, kvd = c.n_head_kv * c.head_dim;
  for (uint32_t l = 0; l < c.n_layer; l++) {
    const ogm_llama_layer &L = layers[l];
    if (!llama_weight_ok(L.wq, c.n_embd, qd) || !llama_weight_ok(L.wk, c.n_embd, kvd) ||
        !llama_weight_ok(L.wv, c.n_embd, kvd) || !llama_weight_ok(L.wo, qd, c.n_embd) ||
        !llama_weight_ok(L.w_gate, c.n_embd, c.n_ff) || !llama_weight_ok(L.w_up, c.n_embd, c.n_ff) ||
        !llama_weight_ok(L.w_down, c.n_ff, c.n_embd) || !L.attn_norm || !L.ffn_norm)
      return fail(ctx, OGM_ERR_INVALID, "layer " + std::to_string(l) + ": missing weight or wrong shape");
  }
  if (!llama_weight_ok(output, c.n_embd, c.n_vocab)) return fail(ctx, OGM_ERR_INVALID, "output weight shape");

  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  ogm_llama *m = new (std::nothrow) ogm_llama();
  if (!m) return fail(ctx, OGM_ERR_OOM, "out of host memory");
  m->cfg = c;
  m->cfg.rope_freq_factors = nullptr;   // folded into the frequency table below; the caller's array is not kept
  m->layers.assign(layers, layers + c.n_layer);
  m->output = output;
  m->max_splits = (c.max_ctx + OGM_ATTN_CHUNK_MIN - 1) / OGM_ATTN_CHUNK_MIN;
  const size_t cache_bytes = (size_t)c.n_layer * c.max_ctx * kvd * 2;
  int rc = OGM_OK;
  auto A = [&](void **p, size_t b) { if (rc == OGM_OK) rc = llama_alloc(ctx, m, p, b); };
  A((void **)&m->norms, ((size_t)c.n_layer * 2 + 1) * c.n_embd * 4);
  const size_t pre_stride = (size_t)qd + 2 * (size_t)kvd + 2 * (size_t)c.head_dim;
  A((void **)&m->pre, (size_t)c.n_layer * pre_stride * 4);
  A((void **)&m->freq, (size_t)(c.rope_dim / 2 + 1) * 4);
  A((void **)&m->rope_cs, (size_t)(c.rope_dim / 2 + 1) * 8);
  // every position's rotation table once, where it stays small (64 pairs x 8 bytes x the context: 4 MiB at 8192
  // positions); a decode step then launches no table kernel
  const size_t rope_all_bytes = (size_t)c.max_ctx * (c.rope_dim / 2) * 8;
  if (c.rope_dim != 0 && rope_all_bytes <= ((size_t)64 << 20)) A((void **)&m->rope_all, rope_all_bytes);
  A((void **)&m->attn_counters, (size_t)2 * c.n_head_kv * ogm_attn_head_parts(gq) * OGM_ATTN_TICKET_STRIDE * 4);
  A(&m->k_cache, cache_bytes);
  A(&m->v_cache, cache_bytes);
  A((void **)&m->x, (size_t)c.n_embd * 4);
  A((void **)&m->q, (size_t)qd * 4);
  A((void **)&m->k, (size_t)kvd * 4);
  A((void **)&m->v, (size_t)kvd * 4);
  A((void **)&m->proj, (size_t)c.n_embd * 4);
  A((void **)&m->gate, (size_t)c.n_ff * 4);
  A((void **)&m->up, (size_t)c.n_ff * 4);
  A((void **)&m->part_o, (size_t)c.n_head * m->max_splits * c.head_dim * 4);
  A((void **)&m->part_ml, (size_t)c.n_head * m->max_splits * 2 * 4);
  A((void **)&m->logits, (size_t)c.n_vocab * 4);
  A((void **)&m->amax_scratch, 512 * 4);
  A((void **)&m->amax_out, 4);
  if (rc != OGM_OK) { llama_free(m); return rc; }
  // activation scratch for the widest matmul input
  uint32_t widest = c.n_embd > c.n_ff ? c.n_embd : c.n_ff;
  if (qd > widest) widest = qd;
  if ((rc = ensure_act(ctx, widest, 1)) != OGM_OK) { llama_free(m); return rc; }

  std::vector<float> host(((size_t)c.n_layer * 2 + 1) * c.n_embd);
  for (uint32_t l = 0; l < c.n_layer; l++) {
    memcpy(&host[((size_t)l * 2) * c.n_embd], layers[l].attn_norm, (size_t)c.n_embd * 4);
    memcpy(&host[((size_t)l * 2 + 1) * c.n_embd], layers[l].ffn_norm, (size_t)c.n_embd * 4);
  }
  memcpy(&host[(size_t)c.n_layer * 2 * c.n_embd], output_norm, (size_t)c.n_embd * 4);
  // freq_i = base^(-2i / rope_dim) [/ factor_i], in f32 as tensor.rs:1147-1150 computes it
  std::vector<float> freq(c.rope_dim / 2 + 1, 0.0f);
  for (uint32_t i = 0; i < c.rope_dim / 2; i++) {
    freq[i] = powf(c.rope_freq_base, -2.0f * (float)i / (float)c.rope_dim);
    if (c.rope_freq_factors) freq[i] /= c.rope_freq_factors[i];
  }
  // the optional per-layer vectors, side by side; the layer keeps a device pointer or null
  std::vector<float> pre_host((size_t)c.n_layer * pre_stride, 0.0f);
  for (uint32_t l = 0; l < c.n_layer; l++) {
    ogm_llama_layer &D = m->layers[l];
    float *hb = &pre_host[(size_t)l * pre_stride], *db = m->pre + (size_t)l * pre_stride;
    const float **slot[5] = {&D.q_bias, &D.k_bias, &D.v_bias, &D.q_norm, &D.k_norm};
    const size_t len[5] = {qd, kvd, kvd, c.head_dim, c.head_dim};
    size_t off = 0;
    for (int i = 0; i < 5; i++) {
      if (*slot[i]) {
        memcpy(hb + off, *slot[i], len[i] * 4);
        *slot[i] = db + off;
      }
      off += len[i];
    }
    D.attn_norm = D.ffn_norm = nullptr;   // copied into m->norms
  }
  hipError_t e = hipMemcpy(m->norms, host.data(), host.size() * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(m->pre, pre_host.data(), pre_host.size() * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(m->freq, freq.data(), freq.size() * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemset(m->attn_counters, 0, (size_t)2 * c.n_head_kv * ogm_attn_head_parts(gq) * OGM_ATTN_TICKET_STRIDE * 4);
  if (e == hipSuccess) e = hipMemset(m->k_cache, 0, cache_bytes);
  if (e == hipSuccess) e = hipMemset(m->v_cache, 0, cache_bytes);
  if (m->rope_all && e == hipSuccess) {
    // (cos, sin) of pos * freq_i for every cache position, by the host's sinf / cosf -- the functions the
    // reference's f32::sin_cos is (tensor.rs:1160) -- so a rotated row is the reference's to the bit given the
    // same q or k.  (A cache too long for the table has each token's row computed on the device instead.)
    const size_t half = c.rope_dim / 2;
    std::vector<float> table((size_t)c.max_ctx * half * 2);
    for (uint32_t p = 0; p < c.max_ctx; p++)
      for (size_t i = 0; i < half; i++) {
        const float theta = (float)p * freq[i];
        table[((size_t)p * half + i) * 2] = cosf(theta);
        table[((size_t)p * half + i) * 2 + 1] = sinf(theta);
      }
    e = hipMemcpy(m->rope_all, table.data(), table.size() * 4, hipMemcpyHostToDevice);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) {
    llama_free(m);
    return fail(ctx, OGM_ERR_HIP, std::string("ogm_llama_create: ") + hipGetErrorString(e));
  }
  *out = m;
  return OGM_OK;
}

extern "C" void ogm_llama_destroy(ogm_ctx *ctx, ogm_llama *m) {
  if (!ctx || !m) return;
  std::lock_guard<std::mutex> lock(ctx->mu);
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  llama_free(m);
}

extern "C" int ogm_llama_kv_write(ogm_ctx *ctx, ogm_llama *m, uint32_t layer, uint32_t pos0, uint32_t n_pos,
                                  const float *k, const float *v) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !k || !v) return fail(ctx, OGM_ERR_INVALID, "null argument");
  const ogm_llama_config &c = m->cfg;
  if (layer >= c.n_layer || (uint64_t)pos0 + n_pos > c.max_ctx)
    return fail(ctx, OGM_ERR_INVALID, "layer or position range outside the cache");
  if (n_pos == 0) return OGM_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  const size_t kvd = (size_t)c.n_head_kv * c.head_dim, n = (size_t)n_pos * kvd;
  if (m->stage_cap < n * 4) {
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    if (m->stage) HIPCHK(ctx, hipFree(m->stage));
    m->stage = nullptr;
    m->stage_cap = 0;
    HIPCHK(ctx, hipMalloc((void **)&m->stage, n * 4));
    m->stage_cap = n * 4;
  }
  const size_t row0 = ((size_t)layer * c.max_ctx + pos0) * kvd;
  const float *src[2] = {k, v};
  void *dst[2] = {(uint8_t *)m->k_cache + row0 * 2, (uint8_t *)m->v_cache + row0 * 2};
  for (int i = 0; i < 2; i++) {
    HIPCHK(ctx, hipMemcpyAsync(m->stage, src[i], n * 4, hipMemcpyHostToDevice, ctx->stream));
    HIPCHK(ctx, ogm_launch_f32_to_f16(m->stage, dst[i], n, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));  // the host buffer and the staging area are reused
  }
  return OGM_OK;
}

extern "C" int ogm_llama_kv_read(ogm_ctx *ctx, ogm_llama *m, uint32_t layer, uint32_t pos0, uint32_t n_pos,
                                 uint16_t *k_bits, uint16_t *v_bits) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !k_bits || !v_bits) return fail(ctx, OGM_ERR_INVALID, "null argument");
  const ogm_llama_config &c = m->cfg;
  if (layer >= c.n_layer || (uint64_t)pos0 + n_pos > c.max_ctx)
    return fail(ctx, OGM_ERR_INVALID, "layer or position range outside the cache");
  if (n_pos == 0) return OGM_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  const size_t kvd = (size_t)c.n_head_kv * c.head_dim, bytes = (size_t)n_pos * kvd * 2;
  const size_t row0 = ((size_t)layer * c.max_ctx + pos0) * kvd;
  HIPCHK(ctx, hipMemcpy(k_bits, (const uint8_t *)m->k_cache + row0 * 2, bytes, hipMemcpyDeviceToHost));
  HIPCHK(ctx, hipMemcpy(v_bits, (const uint8_t *)m->v_cache + row0 * 2, bytes, hipMemcpyDeviceToHost));
  return OGM_OK;
}

// Debug capture: keeps what the activation scratch holds right now (n elements quantized per
// `mode`) as the input of matmul site `site`.  A no-op unless capture is on.
static int llama_capture(ogm_ctx *ctx, ogm_llama *m, uint32_t site, uint32_t n, int mode, hipStream_t s) {
  if (!m->cap_on) return OGM_OK;
  const uint32_t group = mode == OGM_ACT_PER_32 ? 32u : 256u;
  const OgmActDev a = act_view(ctx, n, mode, 0);
  HIPCHK(ctx, hipMemcpyAsync(m->cap_q + (size_t)site * m->cap_width, a.q, n, hipMemcpyDeviceToDevice, s));
  HIPCHK(ctx, hipMemcpyAsync(m->cap_d + (size_t)site * (m->cap_width / 32u), a.d, (size_t)(n / group) * 4,
                             hipMemcpyDeviceToDevice, s));
  m->cap_n[site] = n;
  m->cap_group[site] = group;
  return OGM_OK;
}

// One matmul group of the step over the activations the previous kernel quantized.
static int llama_matmul(ogm_ctx *ctx, const ogm_weight *const *ws, float *const *ys, size_t n, hipStream_t s) {
  // weights of one type go out as one launch; a mixed group (Q4_K q/k with a Q6_K v) as several
  size_t i = 0;
  while (i < n) {
    Target tg[OGM_GEMV_MAX_MATS];
    size_t e = i;
    while (e < n && e - i < OGM_GEMV_MAX_MATS && ws[e]->ggml_type == ws[i]->ggml_type) {
      tg[e - i] = Target{ws[e], ys[e]};
      e++;
    }
    int rc = enqueue_gemv(ctx, tg, e - i, 1, 0, s, nullptr, nullptr);
    if (rc != OGM_OK) return rc;
    i = e;
  }
  return OGM_OK;
}

// LlamaModel::run_layers + forward at one token (arch/llama.rs:594-932, 1007-1032), eight launches a layer:
// norm (+ quantize), q/k/v, attention (+ quantize), wo, norm (+ quantize), gate/up, SwiGLU (+ quantize), down.
static int llama_decode_enqueue(ogm_ctx *ctx, ogm_llama *m, const float *x_dev, uint32_t pos, float *logits_dev,
                                uint32_t *argmax_dev, hipStream_t s) {
  const ogm_llama_config &c = m->cfg;
  if (pos >= c.max_ctx) return fail(ctx, OGM_ERR_INVALID, "position beyond the KV cache");
  const uint32_t qd = c.n_head * c.head_dim, kvd = c.n_head_kv * c.head_dim;
  const float scale = 1.0f / sqrtf((float)c.head_dim);
  // (the table of this position: from the one made at creation, or computed now)
  const float *rope_cs = m->rope_all ? m->rope_all + (size_t)pos * (c.rope_dim / 2) * 2 : m->rope_cs;
  if (!m->rope_all) HIPCHK(ctx, ogm_launch_rope_table(m->freq, pos, 1, c.rope_dim, m->rope_cs, s));
  const float *delta = nullptr;  // what the next norm adds to x first: the last block's output
  // The caller's row becomes the residual stream: the first norm reads it where it lies and stores it to m->x.
  const float *x_first = x_dev != m->x ? x_dev : nullptr;
  const int mode_out = act_mode_for(m->output->ggml_type);
  const float *out_norm = m->norms + (size_t)c.n_layer * 2 * c.n_embd;
  int rc;
  for (uint32_t l = 0; l < c.n_layer; l++) {
    const ogm_llama_layer &L = m->layers[l];
    const float *attn_norm = m->norms + (size_t)l * 2 * c.n_embd, *ffn_norm = attn_norm + c.n_embd;
    void *kc = (uint8_t *)m->k_cache + (size_t)l * c.max_ctx * kvd * 2;
    void *vc = (uint8_t *)m->v_cache + (size_t)l * c.max_ctx * kvd * 2;
    // q/k/v read one input; all supported types of a model share an activation mode only if they
    // are all K-quants or all Q8_0, which create() cannot assume: quantize per consumer mode
    const int mode_qkv = act_mode_for(L.wq->ggml_type);
    if (act_mode_for(L.wk->ggml_type) != mode_qkv || act_mode_for(L.wv->ggml_type) != mode_qkv)
      return fail(ctx, OGM_ERR_UNSUPPORTED, "wq, wk and wv must share an activation mode");
    const ogm_weight *w3[3] = {L.wq, L.wk, L.wv};
    float *y3[3] = {m->q, m->k, m->v};
    HIPCHK(ctx, ogm_launch_norm_quant(mode_qkv, m->x, delta, attn_norm, c.n_embd, c.rms_eps, nullptr,
                                      act_view(ctx, c.n_embd, mode_qkv, 0), s, 1, l == 0 ? x_first : nullptr));
    if ((rc = llama_capture(ctx, m, 4 * l, c.n_embd, mode_qkv, s)) != OGM_OK) return rc;
    if ((rc = llama_matmul(ctx, w3, y3, 3, s)) != OGM_OK) return rc;
    const int mode_o = act_mode_for(L.wo->ggml_type);
    const OgmAttnPre pre{L.q_bias, L.k_bias, L.v_bias, L.q_norm, L.k_norm, c.rms_eps, c.rope_neox};
    HIPCHK(ctx, ogm_launch_attn_decode(m->q, m->k, m->v, rope_cs, c.rope_dim, pre, kc, vc, pos, m->max_splits,
                                       c.n_head, c.n_head_kv, c.head_dim, scale, m->part_o, m->part_ml,
                                       m->attn_counters, mode_o, nullptr, act_view(ctx, qd, mode_o, 0), s, 0u,
                                       (uint32_t)ctx->tune_attn_decode_chunks));
    const int mode_ff = act_mode_for(L.w_gate->ggml_type);
    if (act_mode_for(L.w_up->ggml_type) != mode_ff)
      return fail(ctx, OGM_ERR_UNSUPPORTED, "w_gate and w_up must share an activation mode");
    const ogm_weight *w1[1] = {L.wo};
    float *y1[1] = {m->proj};
    if ((rc = llama_capture(ctx, m, 4 * l + 1, qd, mode_o, s)) != OGM_OK) return rc;
    if ((rc = llama_matmul(ctx, w1, y1, 1, s)) != OGM_OK) return rc;
    HIPCHK(ctx, ogm_launch_norm_quant(mode_ff, m->x, m->proj, ffn_norm, c.n_embd, c.rms_eps, nullptr,
                                      act_view(ctx, c.n_embd, mode_ff, 0), s));
    const ogm_weight *w2[2] = {L.w_gate, L.w_up};
    float *y2[2] = {m->gate, m->up};
    const int mode_d = act_mode_for(L.w_down->ggml_type);
    if ((rc = llama_capture(ctx, m, 4 * l + 2, c.n_embd, mode_ff, s)) != OGM_OK) return rc;
    if ((rc = llama_matmul(ctx, w2, y2, 2, s)) != OGM_OK) return rc;
    HIPCHK(ctx, ogm_launch_swiglu_quant(mode_d, m->gate, m->up, c.n_ff, nullptr, act_view(ctx, c.n_ff, mode_d, 0), s));
    const ogm_weight *wd[1] = {L.w_down};
    if ((rc = llama_capture(ctx, m, 4 * l + 3, c.n_ff, mode_d, s)) != OGM_OK) return rc;
    if ((rc = llama_matmul(ctx, wd, y1, 1, s)) != OGM_OK) return rc;
    delta = m->proj;
  }
  HIPCHK(ctx, ogm_launch_norm_quant(mode_out, m->x, delta, out_norm, c.n_embd, c.rms_eps, nullptr,
                                    act_view(ctx, c.n_embd, mode_out, 0), s));
  float *lg = logits_dev ? logits_dev : m->logits;
  const ogm_weight *wo_[1] = {m->output};
  float *yo[1] = {lg};
  if ((rc = llama_capture(ctx, m, 4 * c.n_layer, c.n_embd, mode_out, s)) != OGM_OK) return rc;
  if ((rc = llama_matmul(ctx, wo_, yo, 1, s)) != OGM_OK) return rc;
  if (argmax_dev) HIPCHK(ctx, ogm_launch_argmax(lg, c.n_vocab, m->amax_scratch, argmax_dev, s));
  // the activation scratch no longer holds what ogm_act_quantize_dev left there
  ctx->act_mode = -1;
  return OGM_OK;
}

extern "C" int ogm_llama_decode_dev(ogm_ctx *ctx, ogm_llama *m, const float *x_dev, uint32_t pos,
                                    float *logits_dev, uint32_t *argmax_dev, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !x_dev) return fail(ctx, OGM_ERR_INVALID, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  return llama_decode_enqueue(ctx, m, x_dev, pos, logits_dev, argmax_dev, stream ? (hipStream_t)stream : ctx->stream);
}

extern "C" int ogm_llama_decode(ogm_ctx *ctx, ogm_llama *m, const float *x, uint32_t pos, float *logits,
                                uint32_t *argmax) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !x) return fail(ctx, OGM_ERR_INVALID, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  const ogm_llama_config &c = m->cfg;
  // the embedding row goes straight into the residual stream
  HIPCHK(ctx, hipMemcpyAsync(m->x, x, (size_t)c.n_embd * 4, hipMemcpyHostToDevice, ctx->stream));
  int rc = llama_decode_enqueue(ctx, m, m->x, pos, nullptr, m->amax_out, ctx->stream);
  if (rc != OGM_OK) return rc;
  if (logits) HIPCHK(ctx, hipMemcpyAsync(logits, m->logits, (size_t)c.n_vocab * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (argmax) HIPCHK(ctx, hipMemcpyAsync(argmax, m->amax_out, 4, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return OGM_OK;
}

extern "C" int ogm_llama_debug_hidden(ogm_ctx *ctx, ogm_llama *m, float *x_out) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !x_out) return fail(ctx, OGM_ERR_INVALID, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  // the output norm added the last block's output to x in place before normalising
  HIPCHK(ctx, hipMemcpy(x_out, m->x, (size_t)m->cfg.n_embd * 4, hipMemcpyDeviceToHost));
  return OGM_OK;
}

extern "C" int ogm_debug_attn_stamps(ogm_ctx *ctx, uint64_t *out, size_t n_words) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!out) return fail(ctx, OGM_ERR_INVALID, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  const hipError_t e = ogm_attn_stamps_read((unsigned long long *)out, n_words);
  if (e == hipErrorNotSupported)
    return fail(ctx, OGM_ERR_UNSUPPORTED, "this build of the library keeps no attention stamps (build a variant with -DOGM_ATTN_STAMPS=1)");
  HIPCHK(ctx, e);
  return OGM_OK;
}

extern "C" int ogm_llama_debug_capture(ogm_ctx *ctx, ogm_llama *m, int enable) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m) return fail(ctx, OGM_ERR_INVALID, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  if (!enable || m->cap_q) {   // the buffers stay with the model until it is destroyed
    m->cap_on = enable != 0;
    return OGM_OK;
  }
  const ogm_llama_config &c = m->cfg;
  const uint32_t qd = c.n_head * c.head_dim;
  uint32_t widest = c.n_embd > c.n_ff ? c.n_embd : c.n_ff;
  if (qd > widest) widest = qd;
  const size_t sites = (size_t)4 * c.n_layer + 1;
  m->cap_width = (widest + 31u) & ~31u;
  int rc = llama_alloc(ctx, m, (void **)&m->cap_q, sites * m->cap_width);
  if (rc == OGM_OK) rc = llama_alloc(ctx, m, (void **)&m->cap_d, sites * (m->cap_width / 32u) * 4);
  if (rc != OGM_OK) {
    m->cap_q = nullptr;
    m->cap_d = nullptr;
    return rc;
  }
  m->cap_n.assign(sites, 0u);
  m->cap_group.assign(sites, 0u);
  m->cap_on = true;
  return OGM_OK;
}

extern "C" int ogm_llama_debug_act(ogm_ctx *ctx, ogm_llama *m, uint32_t site, int8_t *q, float *d, uint32_t *n,
                                   uint32_t *group) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !q || !d || !n || !group) return fail(ctx, OGM_ERR_INVALID, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (!m->cap_q) return fail(ctx, OGM_ERR_INVALID, "capture was never on (ogm_llama_debug_capture)");
  if (site >= m->cap_n.size() || m->cap_n[site] == 0) return fail(ctx, OGM_ERR_INVALID, "no such site in the last decode step");
  HIPCHK(ctx, hipSetDevice(ctx->device));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  *n = m->cap_n[site];
  *group = m->cap_group[site];
  HIPCHK(ctx, hipMemcpy(q, m->cap_q + (size_t)site * m->cap_width, *n, hipMemcpyDeviceToHost));
  HIPCHK(ctx, hipMemcpy(d, m->cap_d + (size_t)site * (m->cap_width / 32u), (size_t)(*n / *group) * 4, hipMemcpyDeviceToHost));
  return OGM_OK;
}

extern "C" int ogm_argmax(ogm_ctx *ctx, const float *logits, uint32_t n, uint32_t *out) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!logits || !out || n == 0) return fail(ctx, OGM_ERR_INVALID, "null pointer or no logits");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  int rc;
  if ((rc = ensure_dev(ctx, ctx->x, (size_t)n * 4)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->isum, 513 * 4)) != OGM_OK) return rc;   // 512 scratch words + the result
  uint32_t *scratch = (uint32_t *)ctx->isum.p;
  HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, logits, (size_t)n * 4, hipMemcpyHostToDevice, ctx->stream));
  HIPCHK(ctx, ogm_launch_argmax((const float *)ctx->x.p, n, scratch, scratch + 512, ctx->stream));
  HIPCHK(ctx, hipMemcpyAsync(out, scratch + 512, 4, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return OGM_OK;
}

extern "C" int ogm_dequant_rows(ogm_ctx *ctx, const ogm_weight *w, uint32_t row0, uint32_t n_rows, float *out) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!w || !out) return fail(ctx, OGM_ERR_INVALID, "null argument");
  if ((uint64_t)row0 + n_rows > w->out_dim) return fail(ctx, OGM_ERR_INVALID, "rows outside the matrix");
  if (n_rows == 0) return OGM_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  const size_t bytes = (size_t)n_rows * w->in_dim * 4;
  int rc = ensure_dev(ctx, ctx->y, bytes);
  if (rc != OGM_OK) return rc;
  for (uint32_t r = 0; r < n_rows; r += 32768u) {
    const uint32_t nr = n_rows - r < 32768u ? n_rows - r : 32768u;
    HIPCHK(ctx, ogm_launch_dequant_row(w->dev, w->ggml_type, w->in_dim, w->out_dim, row0 + r, nullptr, nr,
                                       (float *)ctx->y.p + (size_t)r * w->in_dim, ctx->stream));
  }
  HIPCHK(ctx, hipMemcpyAsync(out, ctx->y.p, bytes, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return OGM_OK;
}

extern "C" int ogm_llama_generate(ogm_ctx *ctx, ogm_llama *m, const ogm_weight *tok_embd, uint32_t first_token,
                                  uint32_t pos0, uint32_t n_tokens, uint32_t *tokens_out, float *last_logits) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !tok_embd || !tokens_out) return fail(ctx, OGM_ERR_INVALID, "null argument");
  const ogm_llama_config &c = m->cfg;
  if (tok_embd->in_dim != c.n_embd) return fail(ctx, OGM_ERR_INVALID, "embedding table row length != n_embd");
  if (first_token >= tok_embd->out_dim) return fail(ctx, OGM_ERR_INVALID, "token id is out of vocab range");
  if ((uint64_t)pos0 + n_tokens > c.max_ctx) return fail(ctx, OGM_ERR_INVALID, "positions beyond the KV cache");
  if (n_tokens == 0) return OGM_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  // token ids live on the device: slot 0 is the prompt's last token, slot i + 1 the i-th generated
  int rc = ensure_dev(ctx, ctx->isum, ((size_t)n_tokens + 1) * 4);
  if (rc != OGM_OK) return rc;
  uint32_t *toks = (uint32_t *)ctx->isum.p;
  HIPCHK(ctx, hipMemcpyAsync(toks, &first_token, 4, hipMemcpyHostToDevice, ctx->stream));
  for (uint32_t i = 0; i < n_tokens; i++) {
    // the embedding row goes straight into the residual stream
    HIPCHK(ctx, ogm_launch_dequant_row(tok_embd->dev, tok_embd->ggml_type, tok_embd->in_dim, tok_embd->out_dim, 0,
                                       toks + i, 1, m->x, ctx->stream));
    rc = llama_decode_enqueue(ctx, m, m->x, pos0 + i, nullptr, toks + i + 1, ctx->stream);
    if (rc != OGM_OK) return rc;
  }
  HIPCHK(ctx, hipMemcpyAsync(tokens_out, toks + 1, (size_t)n_tokens * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (last_logits)
    HIPCHK(ctx, hipMemcpyAsync(last_logits, m->logits, (size_t)c.n_vocab * 4, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return OGM_OK;
}

// ---- prefill: run_layers at n_tokens > 1 (llama.rs:594-932) ------------------------------------

static const size_t OGM_PREFILL_PART_BYTES = 256u << 20;   // attention partials per launch
static const uint32_t OGM_ATTN_PER_TOKEN_MAX = 48;         // batches up to this take the per-token attention kernel

static int llama_prefill_buffers(ogm_ctx *ctx, ogm_llama *m) {
  if (m->pf.ready) return OGM_OK;
  const ogm_llama_config &c = m->cfg;
  m->pf.chunk = (uint32_t)ctx->tune_prefill_chunk;
  const size_t T = m->pf.chunk, qd = (size_t)c.n_head * c.head_dim, kvd = (size_t)c.n_head_kv * c.head_dim;
  int rc = OGM_OK;
  auto A = [&](float **p, size_t n) { if (rc == OGM_OK) rc = llama_alloc(ctx, m, (void **)p, n * 4); };
  A(&m->pf.x, T * c.n_embd);
  A(&m->pf.q, T * qd);
  A(&m->pf.k, T * kvd);
  A(&m->pf.v, T * kvd);
  A(&m->pf.attn, T * qd);
  A(&m->pf.proj, T * c.n_embd);
  A(&m->pf.gate, T * c.n_ff);
  A(&m->pf.up, T * c.n_ff);
  A(&m->pf.cs, T * (c.rope_dim / 2 + 1) * 2);
  A((float **)&m->pf.tokens, T);
  if (rc != OGM_OK) return rc;
  m->pf.ready = true;
  return OGM_OK;
}

// The per-token attention kernel's partial results (attn_prefill_variant 1): query rows per launch
// as many as keep them within OGM_PREFILL_PART_BYTES.
static int llama_prefill_partials(ogm_ctx *ctx, ogm_llama *m) {
  if (m->pf.part_o) return OGM_OK;
  const ogm_llama_config &c = m->cfg;
  const size_t per_token = (size_t)c.n_head * m->max_splits * c.head_dim * 4;
  size_t at = OGM_PREFILL_PART_BYTES / per_token;
  if (at < 1) at = 1;
  if (at > m->pf.chunk) at = m->pf.chunk;
  if (ctx->tune_attn_prefill_variant == 0 && at > 64) at = 64;   // only small batches come here
  int rc = llama_alloc(ctx, m, (void **)&m->pf.part_o, at * per_token);
  if (rc == OGM_OK) rc = llama_alloc(ctx, m, (void **)&m->pf.part_ml, at * (size_t)c.n_head * m->max_splits * 2 * 4);
  if (rc != OGM_OK) return rc;
  m->pf.attn_tokens = (uint32_t)at;
  return OGM_OK;
}

// Matmuls over the same T input rows; weights of one type share the quantized activations.
static int llama_matmul_rows(ogm_ctx *ctx, const ogm_weight *const *ws, float *const *ys, size_t n, const float *x,
                             uint32_t T, hipStream_t s) {
  size_t i = 0;
  while (i < n) {
    Target tg[OGM_GEMV_MAX_MATS];
    size_t e = i;
    while (e < n && e - i < OGM_GEMV_MAX_MATS && ws[e]->ggml_type == ws[i]->ggml_type) {
      tg[e - i] = Target{ws[e], ys[e]};
      e++;
    }
    int rc = enqueue_matmul(ctx, tg, e - i, x, T, 0, s, nullptr, nullptr);
    if (rc != OGM_OK) return rc;
    i = e;
  }
  return OGM_OK;
}

// Matmuls of a batch over activations a producer kernel has already quantized into the context's
// scratch (mode `mode`, `in_dim` wide, T rows): the weights are grouped by type as in
// llama_matmul_rows; all of them must take that mode.
static int llama_matmul_quantized_rows(ogm_ctx *ctx, const ogm_weight *const *ws, float *const *ys, size_t n,
                                       int mode, uint32_t in_dim, uint32_t T, hipStream_t s, bool xt_written = false) {
  ctx->act_mode = mode;
  ctx->act_in_dim = in_dim;
  ctx->act_tokens = T;
  ctx->act_xt = xt_written;   // whether the producer also filled the tiled GEMMs' operand chunks (llama_producer_xt)
  size_t i = 0;
  while (i < n) {
    Target tg[OGM_GEMV_MAX_MATS];
    size_t e = i;
    while (e < n && e - i < OGM_GEMV_MAX_MATS && ws[e]->ggml_type == ws[i]->ggml_type) {
      tg[e - i] = Target{ws[e], ys[e]};
      e++;
    }
    int rc = enqueue_gemv(ctx, tg, e - i, T, 0, s, nullptr, nullptr);
    if (rc != OGM_OK) return rc;
    i = e;
  }
  return OGM_OK;
}

// Where a producer kernel of a batch (norm, SwiGLU) should also lay its int8 rows out in the operand chunks of the
// matrix-core GEMMs, or null.  Saves the tiled GEMM's own relayout launch (5 us a matmul at 512 tokens of the 8B
// shapes) and the small-batch kernel its gather of up to 32 rows a load; from 17 tokens, since a producer writes
// them at no launch of its own.
static int llama_producer_xt(ogm_ctx *ctx, const ogm_weight *w, int mode, uint32_t in_dim, uint32_t T, int8_t **xt) {
  *xt = nullptr;
  if (mode != OGM_ACT_PER_256 || !act_chunks_wanted(ctx, w->ggml_type, in_dim, T, 0, 17u)) return OGM_OK;
  const int rc = ensure_dev(ctx, ctx->xh, ogm_gemm_xh_bytes(in_dim, T));
  if (rc == OGM_OK) *xt = (int8_t *)ctx->xh.p;
  return rc;
}

// x += delta, RMSNorm, and the matmuls over the normed rows: the norm kernel quantizes its own
// output (the decode step's kernel, one workgroup per row) and the f32 rows are never stored.
static int llama_norm_matmul_rows(ogm_ctx *ctx, ogm_llama *m, const ogm_weight *const *ws, float *const *ys, size_t n,
                                  const float *delta, const float *norm_w, uint32_t T, hipStream_t s) {
  const ogm_llama_config &c = m->cfg;
  int rc = ensure_act(ctx, c.n_embd, T);
  if (rc != OGM_OK) return rc;
  // Matrices that take different activation formats (Q2_K at several tokens wants per-32 ones beside
  // K-quants' per-256) are served one format after the other; the residual is added once.
  bool first = true;
  for (int mode : {OGM_ACT_PER_256, OGM_ACT_PER_32}) {
    const ogm_weight *wm[OGM_GEMV_MAX_MATS];
    float *ym[OGM_GEMV_MAX_MATS];
    size_t k = 0;
    for (size_t i = 0; i < n && k < OGM_GEMV_MAX_MATS; i++)
      if (act_mode_for(ws[i]->ggml_type, T, 0) == mode) {
        wm[k] = ws[i];
        ym[k++] = ys[i];
      }
    if (k == 0) continue;
    OgmActDev act = act_view(ctx, c.n_embd, mode, 0);
    if ((rc = llama_producer_xt(ctx, wm[0], mode, c.n_embd, T, &act.xt)) != OGM_OK) return rc;
    HIPCHK(ctx, ogm_launch_norm_quant(mode, m->pf.x, first ? delta : nullptr, norm_w, c.n_embd, c.rms_eps, nullptr, act, s, T));
    first = false;
    if ((rc = llama_matmul_quantized_rows(ctx, wm, ym, k, mode, c.n_embd, T, s, act.xt != nullptr)) != OGM_OK) return rc;
  }
  return OGM_OK;
}

// One chunk of T <= m->pf.chunk tokens whose embedding rows sit in m->pf.x.  With `last`,
// the final row's hidden state ends in m->x and its logits in m->logits.
static int llama_prefill_chunk(ogm_ctx *ctx, ogm_llama *m, uint32_t pos0, uint32_t T, bool last, hipStream_t s,
                               float *normed_rows = nullptr, bool all_logits = false) {
  const ogm_llama_config &c = m->cfg;
  ogm_llama::Prefill &P = m->pf;
  const uint32_t qd = c.n_head * c.head_dim, kvd = c.n_head_kv * c.head_dim;
  const float scale = 1.0f / sqrtf((float)c.head_dim);
  HIPCHK(ctx, ogm_launch_rope_table(m->freq, pos0, T, c.rope_dim, P.cs, s));
  // The matrix-core attention kernel gives a workgroup 32 query tokens of four heads and the whole cache to walk: a
  // verify batch of a few tokens on a long cache leaves it sixteen workgroups (8B shapes, 4 tokens at 2048
  // positions: 79 us a layer).  The decode kernel over (K/V head, chunk of 128 positions, token) spreads the same
  // work over the device and measures faster up to 64 tokens at 512, 2048 and 8192 cached positions.
  const bool per_token = ctx->tune_attn_prefill_variant == 1 || (ctx->tune_attn_prefill_variant == 0 && T <= OGM_ATTN_PER_TOKEN_MAX);
  if (per_token) {
    const int rc = llama_prefill_partials(ctx, m);
    if (rc != OGM_OK) return rc;
  }
  const float *delta = nullptr;
  for (uint32_t l = 0; l < c.n_layer; l++) {
    const ogm_llama_layer &L = m->layers[l];
    const float *attn_norm = m->norms + (size_t)l * 2 * c.n_embd, *ffn_norm = attn_norm + c.n_embd;
    void *kc = (uint8_t *)m->k_cache + (size_t)l * c.max_ctx * kvd * 2;
    void *vc = (uint8_t *)m->v_cache + (size_t)l * c.max_ctx * kvd * 2;
    const ogm_weight *w3[3] = {L.wq, L.wk, L.wv};
    float *y3[3] = {P.q, P.k, P.v};
    int rc = llama_norm_matmul_rows(ctx, m, w3, y3, 3, delta, attn_norm, T, s);
    if (rc != OGM_OK) return rc;
    const OgmAttnPre pre{L.q_bias, L.k_bias, L.v_bias, L.q_norm, L.k_norm, c.rms_eps, c.rope_neox};
    HIPCHK(ctx, ogm_launch_qkv_pre(P.q, P.k, P.v, P.cs, c.rope_dim, pre, c.n_head, c.n_head_kv, c.head_dim, kc, vc,
                                   pos0, T, s));
    if (!per_token) {
      HIPCHK(ctx, ogm_launch_attn_prefill_mfma(P.q, kc, vc, pos0, T, c.n_head, c.n_head_kv, c.head_dim, scale, P.attn, s));
    }
    // A small batch's merge quantizes its rows for wo itself (the tiled GEMMs of larger batches want the
    // quantizer's second layout and keep their own quantizer launch).
    const int mode_o = act_mode_for(L.wo->ggml_type, T, 0);
    const bool fused_q = per_token && T < 32u && qd % (mode_o == OGM_ACT_PER_32 ? 32u : 256u) == 0;
    if (fused_q && (rc = ensure_act(ctx, qd, T)) != OGM_OK) return rc;
    for (uint32_t t0 = 0; per_token && t0 < T; t0 += P.attn_tokens) {
      const uint32_t nt = T - t0 < P.attn_tokens ? T - t0 : P.attn_tokens;
      HIPCHK(ctx, ogm_launch_attn_prefill(P.q + (size_t)t0 * qd, kc, vc, pos0 + t0, nt, m->max_splits, c.n_head,
                                          c.n_head_kv, c.head_dim, scale, P.part_o, P.part_ml,
                                          fused_q ? nullptr : P.attn + (size_t)t0 * qd, s, fused_q ? mode_o : -1,
                                          fused_q ? act_view(ctx, qd, mode_o, t0) : OgmActDev{},
                                          (uint32_t)ctx->tune_attn_decode_chunks));
    }
    const ogm_weight *w1[1] = {L.wo};
    float *y1[1] = {P.proj};
    if (fused_q) {
      if ((rc = llama_matmul_quantized_rows(ctx, w1, y1, 1, mode_o, qd, T, s)) != OGM_OK) return rc;
    } else if ((rc = llama_matmul_rows(ctx, w1, y1, 1, P.attn, T, s)) != OGM_OK) {
      return rc;
    }
    const ogm_weight *w2[2] = {L.w_gate, L.w_up};
    float *y2[2] = {P.gate, P.up};
    if ((rc = llama_norm_matmul_rows(ctx, m, w2, y2, 2, P.proj, ffn_norm, T, s)) != OGM_OK) return rc;
    // SwiGLU quantizes its own output for the down projection: h is never stored as f32
    const ogm_weight *wd[1] = {L.w_down};
    const int mode_d = act_mode_for(L.w_down->ggml_type, T, 0);
    if ((rc = ensure_act(ctx, c.n_ff, T)) != OGM_OK) return rc;
    OgmActDev act_d = act_view(ctx, c.n_ff, mode_d, 0);
    if ((rc = llama_producer_xt(ctx, L.w_down, mode_d, c.n_ff, T, &act_d.xt)) != OGM_OK) return rc;
    HIPCHK(ctx, ogm_launch_swiglu_quant(mode_d, P.gate, P.up, c.n_ff, nullptr, act_d, s, T));
    if ((rc = llama_matmul_quantized_rows(ctx, wd, y1, 1, mode_d, c.n_ff, T, s, act_d.xt != nullptr)) != OGM_OK) return rc;
    delta = P.proj;
  }
  ctx->act_mode = -1;   // the activation scratch was the matmuls'
  if (all_logits) {
    // forward_all_logits (the trait's contract, arch/mod.rs:2110-2132; composed as gemma.rs:2179-2186 does): every row
    // through the output norm, one matmul of all rows with the output matrix, and each row's greedy token
    int rc = ensure_act(ctx, c.n_embd, T);
    if (rc != OGM_OK) return rc;
    const int mode_out = act_mode_for(m->output->ggml_type, T, 0);
    HIPCHK(ctx, ogm_launch_norm_quant(mode_out, P.x, delta, m->norms + (size_t)c.n_layer * 2 * c.n_embd, c.n_embd,
                                      c.rms_eps, nullptr, act_view(ctx, c.n_embd, mode_out, 0), s, T));
    const ogm_weight *wo_[1] = {m->output};
    float *yo[1] = {m->logits_all};
    if ((rc = llama_matmul_quantized_rows(ctx, wo_, yo, 1, mode_out, c.n_embd, T, s)) != OGM_OK) return rc;
    for (uint32_t t = 0; t < T; t++)
      HIPCHK(ctx, ogm_launch_argmax(m->logits_all + (size_t)t * c.n_vocab, c.n_vocab, m->amax_scratch, m->amax_all + t, s));
    ctx->act_mode = -1;
    return OGM_OK;
  }
  if (normed_rows) {
    // forward_hidden_states (llama.rs:1034-1045): every row through the output norm, no projection
    int rc = ensure_act(ctx, c.n_embd, T);
    if (rc != OGM_OK) return rc;
    const int mode_out = act_mode_for(m->output->ggml_type, T, 0);
    HIPCHK(ctx, ogm_launch_norm_quant(mode_out, P.x, delta, m->norms + (size_t)c.n_layer * 2 * c.n_embd, c.n_embd,
                                      c.rms_eps, normed_rows, act_view(ctx, c.n_embd, mode_out, 0), s, T));
    return OGM_OK;
  }
  if (!last) return OGM_OK;
  // forward (llama.rs:1007-1032): the last row alone goes through the output norm and projection
  float *x_last = P.x + (size_t)(T - 1) * c.n_embd;
  const float *d_last = delta ? delta + (size_t)(T - 1) * c.n_embd : nullptr;
  const int mode_out = act_mode_for(m->output->ggml_type);
  int rc = ensure_act(ctx, c.n_embd, 1);
  if (rc != OGM_OK) return rc;
  HIPCHK(ctx, ogm_launch_norm_quant(mode_out, x_last, d_last, m->norms + (size_t)c.n_layer * 2 * c.n_embd, c.n_embd,
                                    c.rms_eps, nullptr, act_view(ctx, c.n_embd, mode_out, 0), s));
  HIPCHK(ctx, hipMemcpyAsync(m->x, x_last, (size_t)c.n_embd * 4, hipMemcpyDeviceToDevice, s));
  const ogm_weight *wo_[1] = {m->output};
  float *yo[1] = {m->logits};
  if ((rc = llama_matmul(ctx, wo_, yo, 1, s)) != OGM_OK) return rc;
  HIPCHK(ctx, ogm_launch_argmax(m->logits, c.n_vocab, m->amax_scratch, m->amax_out, s));
  ctx->act_mode = -1;
  return OGM_OK;
}

static int llama_prefill(ogm_ctx *ctx, ogm_llama *m, const float *x_host, const ogm_weight *tok_embd,
                         const uint32_t *tokens, uint32_t pos0, uint32_t n_tokens, float *last_logits,
                         uint32_t *argmax, float *hidden_rows = nullptr) {
  const ogm_llama_config &c = m->cfg;
  if (n_tokens == 0) return fail(ctx, OGM_ERR_INVALID, "no tokens");
  if ((uint64_t)pos0 + n_tokens > c.max_ctx) return fail(ctx, OGM_ERR_INVALID, "positions beyond the KV cache");
  if (tok_embd) {
    if (tok_embd->in_dim != c.n_embd) return fail(ctx, OGM_ERR_INVALID, "embedding matrix shape");
    for (uint32_t i = 0; i < n_tokens; i++)
      if (tokens[i] >= tok_embd->out_dim) return fail(ctx, OGM_ERR_INVALID, "token id outside the vocabulary");
  }
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  int rc = llama_prefill_buffers(ctx, m);
  if (rc != OGM_OK) return rc;
  hipStream_t s = ctx->stream;
  for (uint32_t t0 = 0; t0 < n_tokens; t0 += m->pf.chunk) {
    const uint32_t T = n_tokens - t0 < m->pf.chunk ? n_tokens - t0 : m->pf.chunk;
    if (tok_embd) {
      // the embedding rows (llama.rs:609-614), dequantized on the device
      HIPCHK(ctx, hipMemcpyAsync(m->pf.tokens, tokens + t0, (size_t)T * 4, hipMemcpyHostToDevice, s));
      HIPCHK(ctx, ogm_launch_dequant_row(tok_embd->dev, tok_embd->ggml_type, tok_embd->in_dim, tok_embd->out_dim, 0,
                                         m->pf.tokens, T, m->pf.x, s));
    } else {
      HIPCHK(ctx, hipMemcpyAsync(m->pf.x, x_host + (size_t)t0 * c.n_embd, (size_t)T * c.n_embd * 4,
                                 hipMemcpyHostToDevice, s));
    }
    // (the normed rows of a chunk land in the gate buffer, which the layers are done with: n_ff >= n_embd)
    rc = llama_prefill_chunk(ctx, m, pos0 + t0, T, t0 + T == n_tokens, s, hidden_rows ? m->pf.gate : nullptr);
    if (rc != OGM_OK) return rc;
    if (hidden_rows)
      HIPCHK(ctx, hipMemcpyAsync(hidden_rows + (size_t)t0 * c.n_embd, m->pf.gate, (size_t)T * c.n_embd * 4,
                                 hipMemcpyDeviceToHost, s));
    // the staging copies above read caller memory and m->pf.tokens is reused: finish the chunk first
    HIPCHK(ctx, hipStreamSynchronize(s));
  }
  if (hidden_rows) return OGM_OK;
  if (last_logits) HIPCHK(ctx, hipMemcpy(last_logits, m->logits, (size_t)c.n_vocab * 4, hipMemcpyDeviceToHost));
  if (argmax) HIPCHK(ctx, hipMemcpy(argmax, m->amax_out, 4, hipMemcpyDeviceToHost));
  return OGM_OK;
}

extern "C" int ogm_llama_prefill(ogm_ctx *ctx, ogm_llama *m, const float *x, uint32_t pos0, uint32_t n_tokens,
                                 float *last_logits, uint32_t *argmax) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !x) return fail(ctx, OGM_ERR_INVALID, "null argument");
  return llama_prefill(ctx, m, x, nullptr, nullptr, pos0, n_tokens, last_logits, argmax);
}

static const uint32_t OGM_ALL_LOGITS_MAX_TOKENS = 64;

extern "C" int ogm_llama_forward_all_logits(ogm_ctx *ctx, ogm_llama *m, const float *x, const ogm_weight *tok_embd,
                                            const uint32_t *tokens, uint32_t pos0, uint32_t n_tokens, float *logits,
                                            uint32_t *argmax) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || (x == nullptr) == (tok_embd == nullptr) || (tok_embd && !tokens))
    return fail(ctx, OGM_ERR_INVALID, "ogm_llama_forward_all_logits takes embedding rows or a matrix with token ids");
  const ogm_llama_config &c = m->cfg;
  if (n_tokens == 0) return fail(ctx, OGM_ERR_INVALID, "no tokens");
  if (n_tokens > OGM_ALL_LOGITS_MAX_TOKENS)
    return fail(ctx, OGM_ERR_UNSUPPORTED, "ogm_llama_forward_all_logits takes at most 64 positions a call");
  if ((uint64_t)pos0 + n_tokens > c.max_ctx) return fail(ctx, OGM_ERR_INVALID, "positions beyond the KV cache");
  if (tok_embd) {
    if (tok_embd->in_dim != c.n_embd) return fail(ctx, OGM_ERR_INVALID, "embedding matrix shape");
    for (uint32_t i = 0; i < n_tokens; i++)
      if (tokens[i] >= tok_embd->out_dim) return fail(ctx, OGM_ERR_INVALID, "token id outside the vocabulary");
  }
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  int rc = llama_prefill_buffers(ctx, m);
  if (rc != OGM_OK) return rc;
  if (n_tokens > m->pf.chunk) return fail(ctx, OGM_ERR_UNSUPPORTED, "more positions than one pass over the layers takes");
  if (!m->logits_all) {
    rc = llama_alloc(ctx, m, (void **)&m->logits_all, (size_t)OGM_ALL_LOGITS_MAX_TOKENS * c.n_vocab * 4);
    if (rc == OGM_OK) rc = llama_alloc(ctx, m, (void **)&m->amax_all, (size_t)OGM_ALL_LOGITS_MAX_TOKENS * 4);
    if (rc != OGM_OK) return rc;
  }
  hipStream_t s = ctx->stream;
  if (tok_embd) {
    HIPCHK(ctx, hipMemcpyAsync(m->pf.tokens, tokens, (size_t)n_tokens * 4, hipMemcpyHostToDevice, s));
    HIPCHK(ctx, ogm_launch_dequant_row(tok_embd->dev, tok_embd->ggml_type, tok_embd->in_dim, tok_embd->out_dim, 0,
                                       m->pf.tokens, n_tokens, m->pf.x, s));
  } else {
    HIPCHK(ctx, hipMemcpyAsync(m->pf.x, x, (size_t)n_tokens * c.n_embd * 4, hipMemcpyHostToDevice, s));
  }
  rc = llama_prefill_chunk(ctx, m, pos0, n_tokens, false, s, nullptr, true);
  if (rc != OGM_OK) return rc;
  if (argmax) HIPCHK(ctx, hipMemcpyAsync(argmax, m->amax_all, (size_t)n_tokens * 4, hipMemcpyDeviceToHost, s));
  if (logits)
    HIPCHK(ctx, hipMemcpyAsync(logits, m->logits_all, (size_t)n_tokens * c.n_vocab * 4, hipMemcpyDeviceToHost, s));
  HIPCHK(ctx, hipStreamSynchronize(s));
  return OGM_OK;
}

extern "C" int ogm_llama_hidden_states(ogm_ctx *ctx, ogm_llama *m, const float *x, const ogm_weight *tok_embd,
                                       const uint32_t *tokens, uint32_t n_tokens, float *out) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !out || (x == nullptr) == (tok_embd == nullptr) || (tok_embd && !tokens))
    return fail(ctx, OGM_ERR_INVALID, "ogm_llama_hidden_states takes embedding rows or a matrix with token ids");
  if (m->cfg.n_ff < m->cfg.n_embd) return fail(ctx, OGM_ERR_UNSUPPORTED, "n_ff below n_embd");
  return llama_prefill(ctx, m, x, tok_embd, tokens, 0, n_tokens, nullptr, nullptr, out);
}

extern "C" int ogm_llama_prefill_tokens(ogm_ctx *ctx, ogm_llama *m, const ogm_weight *tok_embd,
                                        const uint32_t *tokens, uint32_t pos0, uint32_t n_tokens,
                                        float *last_logits, uint32_t *argmax) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!m || !tok_embd || !tokens) return fail(ctx, OGM_ERR_INVALID, "null argument");
  return llama_prefill(ctx, m, nullptr, tok_embd, tokens, pos0, n_tokens, last_logits, argmax);
}
