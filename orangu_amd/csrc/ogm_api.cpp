// C ABI of the MI355X quantized matmul backend (include/orangu_mi355x.h): context, weight
// uploader and the Backend::matmul family (engine/backend/mod.rs:309-496 of orangu-server),
// over the kernels in ogm_kernels.hip.  No CPU fallback: every compute entry point runs the
// HIP kernels or returns an error status.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <map>
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
};

struct DevBuf {
  void *p = nullptr;
  size_t cap = 0;
};

struct ogm_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  std::mutex mu;
  std::string err;
  std::string name;
  std::map<std::pair<uint64_t, uint64_t>, ogm_weight *> cache;
  std::vector<ogm_weight *> weights;
  // scratch, grown on demand and reused (the vendor backends allocate per call,
  // engine/backend/rocm.rs:352-376; a pool is what the Vulkan op_cache does instead)
  DevBuf x, y, q, d, sums, bsum, isum, imin, xh;
  DevBuf hx, hy;  // pinned host staging
  int tune_wg_waves = 0;
  int tune_gemm_min_tokens = 9;  // matmul at n_tokens >= this takes the MFMA GEMM
  int tune_rb_per_wg = 0;        // row blocks per GEMV workgroup, 0 = by shape
  int tune_fuse_quant = 0;       // quantize inside the single-token GEMV: 0 no, 1 yes
  const char *last_kernel = "";
  // what the activation buffer currently holds (ogm_act_quantize_dev)
  int act_mode = -1;
  uint32_t act_in_dim = 0, act_tokens = 0;
};

static thread_local std::string g_init_err;

static int fail(ogm_ctx *ctx, int status, const std::string &msg) {
  if (ctx)
    ctx->err = msg;
  else
    g_init_err = msg;
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

static int ensure_host(ogm_ctx *ctx, DevBuf &b, size_t bytes) {
  if (bytes <= b.cap) return OGM_OK;
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  if (b.p) HIPCHK(ctx, hipHostFree(b.p));
  b.p = nullptr;
  b.cap = 0;
  size_t cap = (bytes + 4095) & ~(size_t)4095;
  HIPCHK(ctx, hipHostMalloc(&b.p, cap, hipHostMallocDefault));
  b.cap = cap;
  return OGM_OK;
}

static int act_mode_for(uint32_t ggml_type) {
  // backend/cpu.rs:100-116: K-quants take the per-256 quantizer, Q8_0 the per-32 one
  return ggml_type == OGM_Q8_0 ? OGM_ACT_PER_32 : OGM_ACT_PER_256;
}

static int ensure_act(ogm_ctx *ctx, uint32_t in_dim, uint32_t n_tokens) {
  int rc;
  size_t n = (size_t)in_dim * n_tokens;
  if ((rc = ensure_dev(ctx, ctx->q, n)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->d, n / 32 * 4)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->sums, n / 16 * 4)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->bsum, n / 32 * 2)) != OGM_OK) return rc;
  return OGM_OK;
}

static OgmActDev act_view(ogm_ctx *ctx, uint32_t in_dim, int mode, uint32_t token0) {
  OgmActDev a;
  a.q = (int8_t *)ctx->q.p + (size_t)token0 * in_dim;
  a.d = (float *)ctx->d.p + (size_t)token0 * (in_dim / (mode == OGM_ACT_PER_32 ? 32 : 256));
  a.sums = (int32_t *)ctx->sums.p + (size_t)token0 * (in_dim / 16);
  a.bsum = (int16_t *)ctx->bsum.p + (size_t)token0 * (in_dim / 32);
  return a;
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
  ctx->name = std::string(prop.name) + " (" + prop.gcnArchName + ")";
  e = hipSetDevice(device);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    std::string msg = std::string("stream creation: ") + hipGetErrorString(e);
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
    delete w;
  }
  DevBuf *dev[] = {&ctx->x, &ctx->y, &ctx->q, &ctx->d, &ctx->sums, &ctx->bsum, &ctx->isum, &ctx->imin, &ctx->xh};
  for (DevBuf *b : dev)
    if (b->p) (void)hipFree(b->p);
  if (ctx->hx.p) (void)hipHostFree(ctx->hx.p);
  if (ctx->hy.p) (void)hipHostFree(ctx->hy.p);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

extern "C" const char *ogm_last_error(ogm_ctx *ctx) {
  static thread_local std::string copy;
  if (ctx) {
    std::lock_guard<std::mutex> lock(ctx->mu);
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
    ctx->tune_gemm_min_tokens = value ? value : 9;
    return OGM_OK;
  }
  if (strcmp(key, "gemv_rb_per_wg") == 0) {
    if (value < 0 || value > 64) return fail(ctx, OGM_ERR_INVALID, "gemv_rb_per_wg must be 0..64");
    ctx->tune_rb_per_wg = value;
    return OGM_OK;
  }
  if (strcmp(key, "gemv_fuse_quant") == 0) {
    if (value < -1 || value > 1) return fail(ctx, OGM_ERR_INVALID, "gemv_fuse_quant must be -1, 0 or 1");
    ctx->tune_fuse_quant = value < 0 ? 0 : value;  // -1 = the default
    return OGM_OK;
  }
  return fail(ctx, OGM_ERR_INVALID, std::string("unknown tuning key ") + key);
}

extern "C" const char *ogm_last_kernel(ogm_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }

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

// Enqueues the activation quantizer.  Caller holds the lock.
static int enqueue_quantize(ogm_ctx *ctx, int mode, const float *x_dev, uint32_t in_dim,
                            uint32_t n_tokens, hipStream_t stream) {
  int rc = ensure_act(ctx, in_dim, n_tokens);
  if (rc != OGM_OK) return rc;
  HIPCHK(ctx, ogm_launch_quantize(mode, x_dev, in_dim, n_tokens, act_view(ctx, in_dim, mode, 0), stream));
  ctx->act_mode = mode;
  ctx->act_in_dim = in_dim;
  ctx->act_tokens = n_tokens;
  return OGM_OK;
}

// One matrix and where its output goes; a group shares type, in_dim and the activations.
struct Target {
  const ogm_weight *w;
  float *y;
};

static int enqueue_gemv(ogm_ctx *ctx, const Target *tg, size_t n_tg, uint32_t n_tokens, int decode,
                        hipStream_t stream, int32_t *dump_isum, int32_t *dump_imin,
                        const float *x_f32);

// Whether a single-token launch quantizes inside the GEMV (every workgroup repeats the
// quantizer on its way in) instead of running the quantizer kernel first.  Off unless asked
// for: on MI355X the repeated work costs more than the launch it saves (Llama-8B FFN block:
// 28.3 us per pass against 25.9 us).
static bool fuse_quantize(ogm_ctx *ctx, const Target *, size_t) { return ctx->tune_fuse_quant > 0; }

// Enqueues quantize + kernels for tokens of x_dev into the targets' outputs.  Caller holds the
// lock and has checked that the targets share type and in_dim.
static int enqueue_matmul(ogm_ctx *ctx, const Target *tg, size_t n_tg, const float *x_dev,
                          uint32_t n_tokens, int decode, hipStream_t stream, int32_t *dump_isum,
                          int32_t *dump_imin) {
  if (n_tokens == 0 || n_tg == 0) return OGM_OK;
  const ogm_weight *w = tg[0].w;
  if (n_tokens == 1 && !dump_isum && !dump_imin && fuse_quantize(ctx, tg, n_tg))
    return enqueue_gemv(ctx, tg, n_tg, 1, decode, stream, nullptr, nullptr, x_dev);
  int rc = enqueue_quantize(ctx, act_mode_for(w->ggml_type), x_dev, w->in_dim, n_tokens, stream);
  if (rc != OGM_OK) return rc;
  return enqueue_gemv(ctx, tg, n_tg, n_tokens, decode, stream, dump_isum, dump_imin, nullptr);
}

static int enqueue_matmul(ogm_ctx *ctx, const ogm_weight *w, const float *x_dev, uint32_t n_tokens,
                          float *y_dev, int decode, hipStream_t stream, int32_t *dump_isum,
                          int32_t *dump_imin) {
  const Target t{w, y_dev};
  return enqueue_matmul(ctx, &t, 1, x_dev, n_tokens, decode, stream, dump_isum, dump_imin);
}

static bool all_gemm_supported(const Target *tg, size_t n_tg, uint32_t n_tokens) {
  for (size_t i = 0; i < n_tg; i++)
    if (!ogm_gemm_supported(tg[i].w->ggml_type, tg[i].w->in_dim, tg[i].w->out_dim, n_tokens)) return false;
  return true;
}

// Enqueues the matmul kernels over the context's quantized activations (or, with x_f32, over
// one token of f32 activations that the kernel quantizes itself).  Caller holds the lock.
static int enqueue_gemv(ogm_ctx *ctx, const Target *tg, size_t n_tg, uint32_t n_tokens, int decode,
                        hipStream_t stream, int32_t *dump_isum, int32_t *dump_imin,
                        const float *x_f32) {
  const ogm_weight *w0 = tg[0].w;
  const int mode = act_mode_for(w0->ggml_type);
  // backend/cpu.rs:55-167: matmul at n_tokens > 1 takes the GEMM kernels (their float order);
  // n_tokens == 1 and every matmul_decode take the GEMV's.
  const int gemm_order = (!decode && n_tokens > 1) ? 1 : 0;
  if (gemm_order && !dump_isum && !dump_imin && n_tokens >= (uint32_t)ctx->tune_gemm_min_tokens &&
      all_gemm_supported(tg, n_tg, n_tokens)) {
    // enough tokens to fill MFMA tiles: the tiled GEMM (same values, weights read once per 128 tokens)
    int rc = ensure_dev(ctx, ctx->xh, ogm_gemm_xh_bytes(w0->in_dim, n_tokens));
    if (rc != OGM_OK) return rc;
    for (size_t i = 0; i < n_tg; i++) {
      OgmGemmArgs g;
      g.ggml_type = w0->ggml_type;
      g.wt = tg[i].w->dev;
      g.in_dim = w0->in_dim;
      g.out_dim = tg[i].w->out_dim;
      g.act = act_view(ctx, w0->in_dim, mode, 0);
      g.n_tokens = n_tokens;
      g.y = tg[i].y;
      g.xh = ctx->xh.p;
      HIPCHK(ctx, ogm_launch_gemm(g, stream, &ctx->last_kernel));
    }
    return OGM_OK;
  }
  const uint32_t wg_waves = (uint32_t)ctx->tune_wg_waves;
  const uint32_t chunk = ogm_gemv_max_tokens(w0->ggml_type, w0->in_dim, gemm_order);
  if (chunk == 0) return fail(ctx, OGM_ERR_UNSUPPORTED, "no kernel for this type");
  const uint32_t blocks_per_row = w0->in_dim / (w0->ggml_type == OGM_Q8_0 ? 32 : 256);
  for (size_t g0 = 0; g0 < n_tg; g0 += OGM_GEMV_MAX_MATS) {
    const size_t ng = n_tg - g0 < OGM_GEMV_MAX_MATS ? n_tg - g0 : OGM_GEMV_MAX_MATS;
    for (uint32_t t0 = 0; t0 < n_tokens; t0 += chunk) {
      OgmGemvArgs a;
      a.ggml_type = w0->ggml_type;
      a.wt = tg[g0].w->dev;
      a.in_dim = w0->in_dim;
      a.out_dim = tg[g0].w->out_dim;
      a.act = act_view(ctx, w0->in_dim, mode, t0);
      a.n_tokens = n_tokens - t0 < chunk ? n_tokens - t0 : chunk;
      a.y = tg[g0].y + (size_t)t0 * a.out_dim;
      a.gemm_order = gemm_order;
      a.wg_waves = wg_waves;
      a.rb_per_wg = (uint32_t)ctx->tune_rb_per_wg;
      a.dump_isum = dump_isum ? dump_isum + (size_t)t0 * a.out_dim * blocks_per_row : nullptr;
      a.dump_imin = dump_imin ? dump_imin + (size_t)t0 * a.out_dim * blocks_per_row : nullptr;
      a.n_extra = (uint32_t)ng - 1;
      for (size_t i = 1; i < ng; i++) {
        a.extra_wt[i - 1] = tg[g0 + i].w->dev;
        a.extra_out_dim[i - 1] = tg[g0 + i].w->out_dim;
        a.extra_y[i - 1] = tg[g0 + i].y + (size_t)t0 * tg[g0 + i].w->out_dim;
      }
      a.x_f32 = x_f32;
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

static int host_matmul(ogm_ctx *ctx, const ogm_weight *w, const float *x, uint32_t n_tokens,
                       float *y, int decode) {
  int rc = check_matmul_args(ctx, w, x, y, n_tokens);
  if (rc != OGM_OK) return rc;
  if (n_tokens == 0) return OGM_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  const size_t xb = (size_t)n_tokens * w->in_dim * 4, yb = (size_t)n_tokens * w->out_dim * 4;
  if ((rc = ensure_dev(ctx, ctx->x, xb)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->y, yb)) != OGM_OK) return rc;
  if ((rc = ensure_host(ctx, ctx->hx, xb)) != OGM_OK) return rc;
  if ((rc = ensure_host(ctx, ctx->hy, yb)) != OGM_OK) return rc;
  memcpy(ctx->hx.p, x, xb);
  HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, ctx->hx.p, xb, hipMemcpyHostToDevice, ctx->stream));
  rc = enqueue_matmul(ctx, w, (const float *)ctx->x.p, n_tokens, (float *)ctx->y.p, decode,
                      ctx->stream, nullptr, nullptr);
  if (rc != OGM_OK) return rc;
  HIPCHK(ctx, hipMemcpyAsync(ctx->hy.p, ctx->y.p, yb, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
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

extern "C" int ogm_act_quantize_dev(ogm_ctx *ctx, uint32_t ggml_type, const float *x_dev,
                                    uint32_t in_dim, uint32_t n_tokens, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!ogm_supports(ggml_type, in_dim)) return fail(ctx, OGM_ERR_UNSUPPORTED, "type / in_dim without a kernel");
  if (n_tokens == 0) return OGM_OK;
  if (!x_dev) return fail(ctx, OGM_ERR_INVALID, "x is null");
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  return enqueue_quantize(ctx, act_mode_for(ggml_type), x_dev, in_dim, n_tokens, s);
}

extern "C" int ogm_matmul_act_dev(ogm_ctx *ctx, const ogm_weight *w, uint32_t n_tokens,
                                  float *y_dev, int decode, void *stream) {
  if (!ctx) return OGM_ERR_INVALID;
  if (!w) return fail(ctx, OGM_ERR_INVALID, "weight is null");
  if (n_tokens == 0) return OGM_OK;
  if (!y_dev) return fail(ctx, OGM_ERR_INVALID, "y is null");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (ctx->act_mode != act_mode_for(w->ggml_type) || ctx->act_in_dim != w->in_dim ||
      ctx->act_tokens < n_tokens)
    return fail(ctx, OGM_ERR_INVALID, "the quantized activations do not fit this weight "
                "(call ogm_act_quantize_dev with its type, in_dim and token count first)");
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  const Target t{w, y_dev};
  return enqueue_gemv(ctx, &t, 1, n_tokens, decode, s, nullptr, nullptr, nullptr);
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
  if (ctx->act_mode != act_mode_for(ws[0]->ggml_type) || ctx->act_in_dim != ws[0]->in_dim ||
      ctx->act_tokens < n_tokens)
    return fail(ctx, OGM_ERR_INVALID, "the quantized activations do not fit these weights "
                "(call ogm_act_quantize_dev with their type, in_dim and token count first)");
  HIPCHK(ctx, hipSetDevice(ctx->device));
  hipStream_t s = stream ? (hipStream_t)stream : ctx->stream;
  return enqueue_gemv(ctx, tg.data(), n_ws, n_tokens, decode, s, nullptr, nullptr, nullptr);
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
  std::vector<size_t> xoff(n_ops), yoff(n_ops);
  size_t xb = 0, yb = 0;
  for (size_t i = 0; i < n_ops; i++) {
    size_t j = 0;
    while (j < i && !(ops[j].x == ops[i].x && ops[j].n_tokens == ops[i].n_tokens &&
                      ops[j].w->in_dim == ops[i].w->in_dim))
      j++;
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
  if ((rc = ensure_dev(ctx, ctx->x, xb)) != OGM_OK) return rc;
  if ((rc = ensure_dev(ctx, ctx->y, yb)) != OGM_OK) return rc;
  if ((rc = ensure_host(ctx, ctx->hx, xb)) != OGM_OK) return rc;
  if ((rc = ensure_host(ctx, ctx->hy, yb)) != OGM_OK) return rc;
  // Size the activation scratch for the largest stripe before anything is enqueued, so it is
  // never reallocated under kernels in flight.
  for (size_t i = 0; i < n_ops; i++) {
    uint32_t t = ops[i].n_tokens < cap ? ops[i].n_tokens : cap;
    if ((rc = ensure_act(ctx, ops[i].w->in_dim, t)) != OGM_OK) return rc;
  }
  for (size_t i = 0; i < n_ops; i++) {
    const ogm_op &op = ops[i];
    const size_t bytes = (size_t)op.n_tokens * op.w->in_dim * 4;
    bool first = true;
    for (size_t j = 0; j < i; j++) first = first && xoff[j] != xoff[i];
    if (bytes && first) memcpy((uint8_t *)ctx->hx.p + xoff[i], op.x, bytes);
  }
  HIPCHK(ctx, hipMemcpyAsync(ctx->x.p, ctx->hx.p, xb, hipMemcpyHostToDevice, ctx->stream));
  std::vector<Target> tg;
  for (size_t i = 0; i < n_ops;) {
    // a run of neighbouring ops over one input and one weight type: one group
    size_t e = i + 1;
    while (e < n_ops && xoff[e] == xoff[i] && ops[e].n_tokens == ops[i].n_tokens &&
           ops[e].w->ggml_type == ops[i].w->ggml_type && ops[e].w->in_dim == ops[i].w->in_dim)
      e++;
    const ogm_op &op = ops[i];
    const float *xd = (const float *)((uint8_t *)ctx->x.p + xoff[i]);
    for (uint32_t t0 = 0; t0 < op.n_tokens; t0 += cap) {
      const uint32_t nt = op.n_tokens - t0 < cap ? op.n_tokens - t0 : cap;
      tg.clear();
      for (size_t k = i; k < e; k++)
        tg.push_back(Target{ops[k].w, (float *)((uint8_t *)ctx->y.p + yoff[k]) + (size_t)t0 * ops[k].w->out_dim});
      rc = enqueue_matmul(ctx, tg.data(), tg.size(), xd + (size_t)t0 * op.w->in_dim, nt, decode,
                          ctx->stream, nullptr, nullptr);
      if (rc != OGM_OK) return rc;
    }
    i = e;
  }
  HIPCHK(ctx, hipMemcpyAsync(ctx->hy.p, ctx->y.p, yb, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
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

extern "C" int ogm_dump_block_sums(ogm_ctx *ctx, const ogm_weight *w, const float *x,
                                   uint32_t n_tokens, int32_t *isum, int32_t *imin) {
  int rc = check_matmul_args(ctx, w, x, isum, n_tokens);
  if (rc != OGM_OK) return rc;
  if (n_tokens == 0) return OGM_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  HIPCHK(ctx, hipSetDevice(ctx->device));
  const size_t blocks = (size_t)w->in_dim / (w->ggml_type == OGM_Q8_0 ? 32 : 256);
  const size_t nb = (size_t)n_tokens * w->out_dim * blocks * 4;
  const size_t xb = (size_t)n_tokens * w->in_dim * 4, yb = (size_t)n_tokens * w->out_dim * 4;
  const bool want_min = imin && w->ggml_type == OGM_Q4_K;
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
