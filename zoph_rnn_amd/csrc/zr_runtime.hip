// Context, error reporting and device memory helpers of the C-ABI.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "zr_internal.h"

// Scratch memory of the allocation-free entry point (zr_softmax_forward_static): every GPU the library runs on holds
// its own copy of this array until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; the device address differs per GPU and is looked up once per device, with that device
// current (static_scratch_address), and only that address is ever passed to kernels.
static __device__ __align__(256) unsigned char scratch[ZR_STATIC_SCRATCH_BYTES];
static void* g_static_scratch[64];
static std::mutex g_static_scratch_mu;

// Device address of `scratch` on the current device (which must be `device`).
static int static_scratch_address(int device, void** out) {
  std::lock_guard<std::mutex> lock(g_static_scratch_mu);
  if (device < 0 || device >= 64) return zr_set_error(ZR_EINVAL, "device %d has no static scratch slot", device);
  if (!g_static_scratch[device]) {
    void* ptr = nullptr;
    ZR_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return zr_set_error(ZR_EHIP, "hipGetSymbolAddress returned a null address for the static scratch array");
    g_static_scratch[device] = ptr;
  }
  *out = g_static_scratch[device];
  return ZR_OK;
}

static thread_local char g_err[512] = "";

// live contexts per device in this process (zr_live_contexts)
static std::atomic<int> g_live[64];

int zr_live_contexts(int device) { return (device >= 0 && device < 64) ? g_live[device].load() : 2; }

int zr_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int zr_bind_device(zr_ctx* ctx) {
  ZR_CHECK_ARG(ctx != nullptr, "null context");
  ZR_HIP(hipSetDevice(ctx->device));
  return ZR_OK;
}

int zr_ctx_scratch(zr_ctx* ctx, int slot, size_t bytes, void** out) {
  if (ctx->fixed_scratch) {
    if (bytes > ctx->fixed_bytes[slot])
      return zr_set_error(ZR_EINVAL, "this call needs %zu bytes of scratch memory (%s) but the allocation-free entry "
                          "point has %zu: use the allocating entry point for this size", bytes,
                          slot == 0 ? "re-laid-out activations" : "partial column statistics", ctx->fixed_bytes[slot]);
    *out = ctx->d_fixed[slot];
    return ZR_OK;
  }
  void** buf = slot == 0 ? &ctx->d_scratch : &ctx->d_scratch2;
  size_t* cap = slot == 0 ? &ctx->scratch_bytes : &ctx->scratch2_bytes;
  if (*cap < bytes) {
    // the old buffer may still be in use by queued kernels: drain the stream before releasing it
    ZR_HIP(hipStreamSynchronize(ctx->stream));
    if (*buf) ZR_HIP(hipFree(*buf));
    *buf = nullptr;
    *cap = 0;
    size_t want = bytes + bytes / 4;
    if (hipMalloc(buf, want) != hipSuccess) {
      (void)hipGetLastError();
      return zr_set_error(ZR_ENOMEM, "scratch allocation of %zu bytes failed", want);
    }
    *cap = want;
  }
  *out = *buf;
  return ZR_OK;
}

extern "C" {

const char* zr_last_error(void) { return g_err; }

const char* zr_version(void) { return "gfx950 hip zoph_rnn_amd 0.1"; }

int zr_ctx_create(int device, zr_ctx** out) {
  ZR_CHECK_ARG(out != nullptr, "zr_ctx_create: out is null");
  *out = nullptr;
  int ndev = 0;
  ZR_HIP(hipGetDeviceCount(&ndev));
  ZR_CHECK_ARG(device >= 0 && device < ndev, "zr_ctx_create: device %d not in [0,%d)", device, ndev);
  ZR_HIP(hipSetDevice(device));
  zr_ctx* c = new zr_ctx();
  memset(c, 0, sizeof(*c));
  c->device = device;
  hipError_t e = hipStreamCreate(&c->own_stream);  // default priority
  if (e != hipSuccess) {
    delete c;
    return zr_set_error(ZR_EHIP, "hipStreamCreate failed: %s", hipGetErrorString(e));
  }
  c->stream = c->own_stream;
  e = hipMalloc((void**)&c->d_flags, (4 + ZR_MAX_COUNTERS) * sizeof(int));
  if (e != hipSuccess) {
    (void)hipStreamDestroy(c->own_stream);
    delete c;
    return zr_set_error(ZR_ENOMEM, "flag allocation failed: %s", hipGetErrorString(e));
  }
  (void)hipMemset(c->d_flags, 0, (4 + ZR_MAX_COUNTERS) * sizeof(int));
  c->d_counters = c->d_flags + 4;
  {
    const int rc = static_scratch_address(device, &c->d_static_scratch);
    if (rc) {
      (void)hipFree(c->d_flags);
      (void)hipStreamDestroy(c->own_stream);
      delete c;
      return rc;
    }
  }
  c->lstm_fused = 1;
  // ZR_LSTM_SWEEP in the environment presets ZR_OPT_LSTM_SWEEP for every context of the process (0, 1 or 2): lets a
  // whole program, e.g. a test run, be put on one path or the other without touching its code
  if (const char* e = getenv("ZR_LSTM_SWEEP")) {
    const int v = atoi(e);
    if (v >= 0 && v <= 2) c->lstm_sweep = v;
  }
  // the same for ZR_OPT_LSTM_SWEEP_SPIN and ZR_OPT_LSTM_STEP_WAIT_EXTRA (tests of a whole program's give-up handling)
  if (const char* e = getenv("ZR_LSTM_SWEEP_SPIN")) {
    const int v = atoi(e);
    if (v >= 0) c->sweep_spin = v;
  }
  if (const char* e = getenv("ZR_LSTM_STEP_WAIT_EXTRA")) {
    const int v = atoi(e);
    if (v >= 0 && v <= 1024) c->step_wait_extra = v;
  }
  // ZR_LSTM_STACK_HELPERS=0 keeps the decoder step on its two-workgroups-per-tile schedules (timing comparisons)
  c->stack_helpers = 1;
  if (const char* e = getenv("ZR_LSTM_STACK_HELPERS")) c->stack_helpers = atoi(e) != 0 ? 1 : 0;
  if (device < 64) g_live[device].fetch_add(1);
  *out = c;
  return ZR_OK;
}

int zr_ctx_destroy(zr_ctx* ctx) {
  if (!ctx) return ZR_OK;
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  if (ctx->d_scratch) (void)hipFree(ctx->d_scratch);
  if (ctx->d_scratch2) (void)hipFree(ctx->d_scratch2);
  if (ctx->d_flags) (void)hipFree(ctx->d_flags);
  for (int i = 0; i < ZR_MAX_PACKED_D; ++i)
    if (ctx->packed_d[i].d_pack) (void)hipFree(ctx->packed_d[i].d_pack);
  if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
  if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
  (void)hipStreamDestroy(ctx->own_stream);
  if (ctx->device >= 0 && ctx->device < 64) g_live[ctx->device].fetch_sub(1);
  delete ctx;
  return ZR_OK;
}

int zr_ctx_sync(zr_ctx* ctx) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  ZR_LAUNCH_CHECK("queued work");
  int flags[4] = {0, 0, 0, 0};
  ZR_HIP(hipMemcpy(flags, ctx->d_flags, sizeof(flags), hipMemcpyDeviceToHost));
  if (flags[2] != 0) {
    ZR_HIP(hipMemset(ctx->d_flags, 0, sizeof(flags)));
    return zr_set_error(ZR_EHIP, "a whole-sweep LSTM launch gave up waiting for another workgroup: the outputs of "
                        "zr_lstm_stack_forward since the last zr_ctx_sync are incomplete (ZR_OPT_LSTM_SWEEP = 1 "
                        "selects one launch per diagonal)");
  }
  if (flags[0] != 0 || flags[1] != 0) {
    ZR_HIP(hipMemset(ctx->d_flags, 0, sizeof(flags)));
    return zr_set_error(ZR_EDATA, "%d token id(s) outside [0, vocab) and %d source position(s) outside the "
                        "attention table were clamped", flags[0], flags[1]);
  }
  return ZR_OK;
}

int zr_ctx_query(zr_ctx* ctx, int what, int* h_value) {
  ZR_CHECK_ARG(ctx != nullptr, "null context");
  ZR_CHECK_ARG(h_value != nullptr, "zr_ctx_query: h_value is null");
  switch (what) {
    case ZR_QUERY_LSTM_STACK_PATH:
      *h_value = ctx->last_stack_path;
      return ZR_OK;
    case ZR_QUERY_SCRATCH_KIB:
      *h_value = (int)((ctx->scratch_bytes + ctx->scratch2_bytes + 1023) / 1024);
      return ZR_OK;
    case ZR_QUERY_ATTN_PATH:
      *h_value = ctx->last_attn_path;
      return ZR_OK;
    case ZR_QUERY_LSTM_SWEEP_ABANDONED: {
      int rc = zr_bind_device(ctx);
      if (rc) return rc;
      ZR_HIP(hipStreamSynchronize(ctx->stream));
      int flag = 0;
      ZR_HIP(hipMemcpy(&flag, ctx->d_flags + 2, sizeof(int), hipMemcpyDeviceToHost));
      // Everything queued behind the abandoned launch ran on its NaN outputs: the word ids picked from them and the
      // window positions derived from them are out of range, so the data flags are up as well.  They say nothing about
      // the caller's data; all four go down together, and the caller's re-run starts from a clean slate.
      if (flag != 0) ZR_HIP(hipMemset(ctx->d_flags, 0, 4 * sizeof(int)));
      *h_value = flag != 0 ? 1 : 0;
      return ZR_OK;
    }
    default:
      return zr_set_error(ZR_EINVAL, "zr_ctx_query: unknown item %d", what);
  }
}

int zr_ctx_set_stream(zr_ctx* ctx, void* hip_stream) {
  ZR_CHECK_ARG(ctx != nullptr, "null context");
  ctx->stream = hip_stream ? (hipStream_t)hip_stream : ctx->own_stream;
  return ZR_OK;
}

int zr_ctx_set_option(zr_ctx* ctx, int option, int value) {
  ZR_CHECK_ARG(ctx != nullptr, "null context");
  switch (option) {
    case ZR_OPT_LSTM_FUSED_EPILOGUE:
      ctx->lstm_fused = value ? 1 : 0;
      return ZR_OK;
    case ZR_OPT_LSTM_TN:
      ZR_CHECK_ARG(value == 0 || value == 1 || value == 2 || value == 4, "ZR_OPT_LSTM_TN must be 0, 1, 2 or 4");
      ctx->lstm_tn = value;
      return ZR_OK;
    case ZR_OPT_LSTM_KSPLIT:
      ZR_CHECK_ARG(value == 0 || value == 4 || value == 8, "ZR_OPT_LSTM_KSPLIT must be 0, 4 or 8");
      ctx->lstm_ksplit = value;
      return ZR_OK;
    case ZR_OPT_LSTM_KERNEL:
      ZR_CHECK_ARG(value >= 0 && value <= 3, "ZR_OPT_LSTM_KERNEL must be 0, 1, 2 or 3");
      ctx->lstm_kernel = value;
      return ZR_OK;
    case ZR_OPT_LSTM_KPARTS:
      ZR_CHECK_ARG(value >= 0 && value <= 16, "ZR_OPT_LSTM_KPARTS must be in [0, 16]");
      ctx->lstm_kparts = value;
      return ZR_OK;
    case ZR_OPT_LSTM_SWEEP:
      ZR_CHECK_ARG(value >= 0 && value <= 2, "ZR_OPT_LSTM_SWEEP must be 0, 1 or 2");
      ctx->lstm_sweep = value;
      return ZR_OK;
    case ZR_OPT_LSTM_SWEEP_SPIN:
      ZR_CHECK_ARG(value >= 0, "ZR_OPT_LSTM_SWEEP_SPIN must not be negative");
      ctx->sweep_spin = value;
      return ZR_OK;
    case ZR_OPT_LSTM_STEP_WAIT_EXTRA:
      ZR_CHECK_ARG(value >= 0 && value <= 1024, "ZR_OPT_LSTM_STEP_WAIT_EXTRA must be in [0, 1024]");
      ctx->step_wait_extra = value;
      return ZR_OK;
    case ZR_OPT_ATTN_SINGLE_LAUNCH:
      ZR_CHECK_ARG(value == 0 || value == 1, "ZR_OPT_ATTN_SINGLE_LAUNCH must be 0 or 1");
      ctx->attn_single = value;
      return ZR_OK;
    case ZR_OPT_BF16_ACTIVATION_TERMS:
      ZR_CHECK_ARG(value == 1 || value == 2, "ZR_OPT_BF16_ACTIVATION_TERMS must be 1 or 2");
      ctx->bf16_terms = value;
      return ZR_OK;
    case ZR_OPT_GEMM_CFG:
      ZR_CHECK_ARG(value >= 0 && value <= 14, "ZR_OPT_GEMM_CFG out of range");
      ctx->gemm_cfg = value;
      return ZR_OK;
    default:
      return zr_set_error(ZR_EINVAL, "unknown option %d", option);
  }
}

int zr_malloc(zr_ctx* ctx, size_t bytes, void** d_out) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(d_out != nullptr, "zr_malloc: out is null");
  *d_out = nullptr;
  if (bytes == 0) bytes = 4;
  if (hipMalloc(d_out, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return zr_set_error(ZR_ENOMEM, "hipMalloc of %zu bytes failed", bytes);
  }
  return ZR_OK;
}

int zr_free(zr_ctx* ctx, void* d_ptr) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  if (!d_ptr) return ZR_OK;
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  ZR_HIP(hipFree(d_ptr));
  return ZR_OK;
}

int zr_h2d(zr_ctx* ctx, void* d_dst, const void* h_src, size_t bytes) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(bytes == 0 || (d_dst && h_src), "zr_h2d: null pointer");
  if (bytes == 0) return ZR_OK;
  // pageable host memory: the runtime stages the copy, and it is ordered after earlier work on the stream
  ZR_HIP(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->stream));
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  return ZR_OK;
}

int zr_d2h(zr_ctx* ctx, void* h_dst, const void* d_src, size_t bytes) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(bytes == 0 || (h_dst && d_src), "zr_d2h: null pointer");
  if (bytes == 0) return ZR_OK;
  ZR_HIP(hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  return ZR_OK;
}

int zr_d2d(zr_ctx* ctx, void* d_dst, const void* d_src, size_t bytes) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(bytes == 0 || (d_dst && d_src), "zr_d2d: null pointer");
  if (bytes == 0) return ZR_OK;
  ZR_HIP(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return ZR_OK;
}

}  // extern "C"

// Stream timer: two HIP events on the context's stream (the reference wraps phases in host wall-clock Timer
// objects after a device synchronise, src/memory_util.h:87-124).
extern "C" int zr_timer_start(zr_ctx* ctx) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  if (!ctx->ev_start) {
    ZR_HIP(hipEventCreate(&ctx->ev_start));
    ZR_HIP(hipEventCreate(&ctx->ev_stop));
  }
  ZR_HIP(hipEventRecord(ctx->ev_start, ctx->stream));
  return ZR_OK;
}

extern "C" int zr_timer_stop(zr_ctx* ctx, float* h_ms) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(ctx->ev_start != nullptr && h_ms != nullptr, "zr_timer_stop: no running timer or null output");
  ZR_HIP(hipEventRecord(ctx->ev_stop, ctx->stream));
  ZR_HIP(hipEventSynchronize(ctx->ev_stop));
  ZR_HIP(hipEventElapsedTime(h_ms, ctx->ev_start, ctx->ev_stop));
  return ZR_OK;
}
