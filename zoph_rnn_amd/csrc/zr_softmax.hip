// Output softmax: logits on MFMA (bias and per-32-row (max, sum exp) partials fused into the GEMM epilogue),
// then one read + one write of the V x mb matrix to normalise.
#include <math.h>

#include "zr_internal.h"
#include "zr_softmax_fold.h"

namespace {

// Folds the per-32-row partials of one column ([N][nblocks][2] floats: contiguous per column, nblocks
// (max, sum exp(x - max)) pairs) into the column's (max, sum).  One workgroup per column (zr_softmax_fold.h).
__global__ void __launch_bounds__(256)
softmax_colstats_kernel(const float* __restrict__ partials, int nblocks, float* __restrict__ colstats) {
  __shared__ float s_m[4], s_s[4];
  const int n = blockIdx.x;
  float mx, sum;
  zr_softmax_fold_column(partials + (size_t)n * nblocks * 2, nblocks, s_m, s_s, mx, sum, nullptr);
  if (threadIdx.x == 0) {
    colstats[2 * n] = mx;
    colstats[2 * n + 1] = sum;
  }
}

// out = exp(x - max) / sum   (MODE 0)   or   (x - max) - log(sum)   (MODE 1).  16-byte accesses when VEC.  One access
// per thread: four per thread, loaded before the first is used, measured slower (11.1 against 9.4 us at 50000 x 128).
template <int MODE, bool VEC>
__global__ void __launch_bounds__(256)
softmax_normalize_kernel(const float* in, float* out, int V, const float* __restrict__ colstats) {
  const int n = blockIdx.y;
  const float mx = colstats[2 * n];
  const float sum = colstats[2 * n + 1];
  const float lsum = logf(sum);
  const float* x = in + (size_t)n * V;
  float* y = out + (size_t)n * V;
  if (VEC) {
    const int i4 = blockIdx.x * 256 + threadIdx.x;
    if (i4 * 4 < V) {
      zr_f32x4 v = ((const zr_f32x4*)x)[i4];
      zr_f32x4 r;
      if (MODE == 0) {
        // expf(x - max) / sum, as the reference divides (custom_kernels.h:574-576)
        r.x = expf(v.x - mx) / sum;
        r.y = expf(v.y - mx) / sum;
        r.z = expf(v.z - mx) / sum;
        r.w = expf(v.w - mx) / sum;
      } else {
        r.x = (v.x - mx) - lsum;
        r.y = (v.y - mx) - lsum;
        r.z = (v.z - mx) - lsum;
        r.w = (v.w - mx) - lsum;
      }
      ((zr_f32x4*)y)[i4] = r;
    }
  } else {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < V) y[i] = (MODE == 0) ? expf(x[i] - mx) / sum : (x[i] - mx) - lsum;
  }
}

// Double-precision column statistics straight from the logits (outputdist_perplexity_kernel accumulates in
// double, reference: src/custom_kernels.h:583-660).  One workgroup per column, two passes over the column.
__global__ void __launch_bounds__(256)
softmax_colstats_f64_kernel(const float* __restrict__ logits, int V, double* __restrict__ colstats) {
  __shared__ double s[256];
  const int n = blockIdx.x;
  const int tid = threadIdx.x;
  const float* x = logits + (size_t)n * V;
  double mx = -1.7976931348623157e308;
  for (int i = tid; i < V; i += 256) mx = fmax(mx, (double)x[i]);
  s[tid] = mx;
  __syncthreads();
  for (int st = 128; st > 0; st >>= 1) {
    if (tid < st) s[tid] = fmax(s[tid], s[tid + st]);
    __syncthreads();
  }
  mx = s[0];
  __syncthreads();
  double sum = 0.0;
  for (int i = tid; i < V; i += 256) sum += exp((double)x[i] - mx);
  s[tid] = sum;
  __syncthreads();
  for (int st = 128; st > 0; st >>= 1) {
    if (tid < st) s[tid] += s[tid + st];
    __syncthreads();
  }
  if (tid == 0) {
    colstats[2 * n] = mx;
    colstats[2 * n + 1] = log(s[0]);
  }
}

__global__ void __launch_bounds__(256)
softmax_logprob_f64_kernel(const float* __restrict__ logits, double* __restrict__ out, int V,
                           const double* __restrict__ colstats) {
  const int n = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < V) out[(size_t)n * V + i] = ((double)logits[(size_t)n * V + i] - colstats[2 * n]) - colstats[2 * n + 1];
}

// loss = sum over unmasked columns of log p[target[b], b]; single workgroup, fixed summation order.
__global__ void __launch_bounds__(256)
softmax_loss_kernel(const float* __restrict__ logits, int V, int mb, const double* __restrict__ colstats,
                    const int* __restrict__ target, const int* __restrict__ mask01, double* __restrict__ loss,
                    int* __restrict__ flags) {
  __shared__ double s[256];
  const int tid = threadIdx.x;
  double acc = 0.0;
  for (int b = tid; b < mb; b += 256) {
    if (mask01[b] == 1) {
      int t = target[b];
      if (t < 0 || t >= V) {
        atomicAdd(&flags[0], 1);
        t = t < 0 ? 0 : V - 1;
      }
      acc += ((double)logits[(size_t)b * V + t] - colstats[2 * b]) - colstats[2 * b + 1];
    }
  }
  s[tid] = acc;
  __syncthreads();
  for (int st = 128; st > 0; st >>= 1) {
    if (tid < st) s[tid] += s[tid + st];
    __syncthreads();
  }
  if (tid == 0) loss[0] = s[0];
}

// d_h_packed: optional k-interleaved copy of d_h ([H/4][mb][4]); used when the product runs on the registered fp32 copy
// of D and H % 8 == 0 (the product then skips its own re-layout of d_h).
// d_partials_ext: where the [mb][nblocks][2] pairs go instead of context scratch (ZR_SOFTMAX_LOGITS_BLOCKS: the caller's
// buffer; no column statistics follow them there).
int logits_with_partials(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb,
                         float* d_logits, float** partials_out, int* nblocks_out, const float* d_h_packed = nullptr,
                         const unsigned short* d_h_hi = nullptr, const unsigned short* d_h_lo = nullptr,
                         float* d_partials_ext = nullptr) {
  const int nblocks = zr_softmax_partial_blocks(V);
  void* scratch = d_partials_ext;
  int rc = ZR_OK;
  if (!scratch) {
    // partials [mb][nblocks][2] followed by column stats (2 doubles per column, also used as 2 floats)
    const size_t pbytes = sizeof(float) * 2 * (size_t)nblocks * mb;
    rc = zr_ctx_scratch(ctx, 1, pbytes + sizeof(double) * 2 * (size_t)mb + 64, &scratch);
    if (rc) return rc;
  }
  ZrGemmDesc d = {};
  d.M = V;
  d.N = mb;
  d.nseg = 1;
  d.K[0] = H;
  d.A[0] = d_D;
  d.lda[0] = V;
  for (int i = 0; i < ZR_MAX_PACKED_D; ++i) {
    const zr_ctx::PackedD& e = ctx->packed_d[i];
    if (e.key == d_D && e.V == V && e.H == H) {  // registered with zr_softmax_prepare: use the MFMA-layout copy
      // ... unless the batch is thousands of columns wide (all time steps of a training minibatch at once): there
      // the LDS-staged kernel on the plain matrix is faster than the register-streaming one on the fp32 copy
      if (!e.bf16 && mb > 1024) break;
      d.A[0] = (const float*)e.d_pack;
      d.lda[0] = e.ldp;
      d.a_pack = e.bf16 ? 2 : 1;
      break;
    }
  }
  d.B[0] = d_h;
  d.ldb[0] = H;
  if (d_h_packed && d.a_pack == 1 && H % 8 == 0 && (((uintptr_t)d_h_packed & 15u) == 0)) {
    d.B[0] = d_h_packed;
    d.b_packed = 1;
  }
  if (d_h_hi && d.a_pack == 2) {  // the producer of h has left its bf16 terms (the GEMM takes them when they suffice)
    d.Bhi[0] = d_h_hi;
    d.Blo[0] = d_h_lo;
  }
  d.C = d_logits;
  d.ldc = V;
  d.batch = 1;
  d.bias = d_b_d;
  d.epilogue = ZR_EPI_SOFTMAX_PARTIAL;
  d.stream_a = (size_t)V * H * (d.a_pack == 2 ? 2 : 4) >= ((size_t)64 << 20) ? 1 : 0;
  d.partials = (float*)scratch;
  rc = zr_gemm_launch(ctx, d);
  if (rc) return rc;
  *partials_out = (float*)scratch;
  *nblocks_out = nblocks;
  return ZR_OK;
}

inline void* stats_ptr(float* partials, int nblocks, int mb) {
  size_t off = sizeof(float) * 2 * (size_t)nblocks * mb;
  off = (off + 63) & ~(size_t)63;
  return (char*)partials + off;
}

int check_softmax_args(const char* who, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb) {
  ZR_CHECK_ARG(V > 0 && H > 0 && mb > 0, "%s: V = %d, H = %d, mb = %d", who, V, H, mb);
  ZR_CHECK_ARG(mb <= 65535, "%s: mb = %d exceeds 65535", who, mb);
  ZR_CHECK_ARG(d_D && d_b_d && d_h, "%s: null pointer", who);
  return ZR_OK;
}

}  // namespace

extern "C" {

static int softmax_prepare(zr_ctx* ctx, const char* who, const float* d_D, int V, int H, bool bf16) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(d_D != nullptr && V > 0 && H > 0, "%s: d_D null or V = %d, H = %d", who, V, H);
  ZR_CHECK_ARG(!bf16 || H % 16 == 0, "%s: H = %d is not a multiple of 16", who, H);
  const int ldp = (V + 31) / 32 * 32, kp = bf16 ? H : (H + 7) / 8 * 8;
  ZR_CHECK_ARG(8LL * ldp + 8LL * V < (1LL << 31), "%s: V = %d too large", who, V);
  const size_t bytes = (bf16 ? sizeof(unsigned short) : sizeof(float)) * (size_t)kp * ldp;
  int slot = -1;
  for (int i = 0; i < ZR_MAX_PACKED_D; ++i)
    if (ctx->packed_d[i].key == d_D) slot = i;
  if (slot >= 0 && (ctx->packed_d[slot].V != V || ctx->packed_d[slot].H != H ||
                    ctx->packed_d[slot].bf16 != (bf16 ? 1 : 0))) {
    rc = zr_softmax_release(ctx, d_D);
    if (rc) return rc;
    slot = -1;
  }
  if (slot < 0) {
    for (int i = 0; i < ZR_MAX_PACKED_D && slot < 0; ++i)
      if (!ctx->packed_d[i].key) slot = i;
    ZR_CHECK_ARG(slot >= 0, "%s: all %d slots are in use (zr_softmax_release one)", who, ZR_MAX_PACKED_D);
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
      (void)hipGetLastError();
      return zr_set_error(ZR_ENOMEM, "%s: allocation of %zu bytes failed", who, bytes);
    }
    ctx->packed_d[slot].d_pack = p;
    ctx->packed_d[slot].V = V;
    ctx->packed_d[slot].H = H;
    ctx->packed_d[slot].ldp = ldp;
    ctx->packed_d[slot].bf16 = bf16 ? 1 : 0;
  }
  rc = bf16 ? zr_pack8_bf16_launch(ctx, d_D, V, H, V, ldp, kp, (unsigned short*)ctx->packed_d[slot].d_pack)
            : zr_pack4_launch(ctx, d_D, V, H, V, ldp, kp, (float*)ctx->packed_d[slot].d_pack);
  if (rc) {
    (void)hipFree(ctx->packed_d[slot].d_pack);
    ctx->packed_d[slot] = zr_ctx::PackedD{};
    return rc;
  }
  ctx->packed_d[slot].key = d_D;
  return ZR_OK;
}

int zr_softmax_prepare(zr_ctx* ctx, const float* d_D, int V, int H) {
  return softmax_prepare(ctx, "zr_softmax_prepare", d_D, V, H, false);
}

int zr_softmax_prepare_bf16(zr_ctx* ctx, const float* d_D, int V, int H) {
  return softmax_prepare(ctx, "zr_softmax_prepare_bf16", d_D, V, H, true);
}

int zr_softmax_release(zr_ctx* ctx, const float* d_D) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  for (int i = 0; i < ZR_MAX_PACKED_D; ++i) {
    if (ctx->packed_d[i].key == d_D && d_D) {
      ZR_HIP(hipStreamSynchronize(ctx->stream));
      (void)hipFree(ctx->packed_d[i].d_pack);
      ctx->packed_d[i] = zr_ctx::PackedD{};
    }
  }
  return ZR_OK;
}

int zr_softmax_forward(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb,
                       int mode, float* d_out, float* d_logits_scratch) {
  return zr_softmax_forward_packed(ctx, d_D, d_b_d, V, H, d_h, nullptr, mb, mode, d_out, d_logits_scratch);
}

int zr_softmax_block_count(int V) { return V > 0 ? zr_softmax_partial_blocks(V) : 0; }

long long zr_softmax_blocks_offset(int V, int cols) {
  return (V > 0 && cols > 0) ? (long long)zr_softmax_blocks_offset_floats(V, cols) : 0;
}

}  // extern "C"

int zr_softmax_colstats_launch(zr_ctx* ctx, const float* d_partials, int nblocks, int cols, float* d_colstats) {
  softmax_colstats_kernel<<<cols, 256, 0, ctx->stream>>>(d_partials, nblocks, d_colstats);
  ZR_LAUNCH_CHECK("softmax_colstats_kernel");
  return ZR_OK;
}

int zr_softmax_forward_packed(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h,
                              const float* d_h_packed, int mb, int mode, float* d_out, float* d_logits_scratch,
                              const unsigned short* d_h_hi, const unsigned short* d_h_lo) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  rc = check_softmax_args("zr_softmax_forward", d_D, d_b_d, V, H, d_h, mb);
  if (rc) return rc;
  ZR_CHECK_ARG(d_out != nullptr, "zr_softmax_forward: d_out is null");
  ZR_CHECK_ARG(mode == ZR_SOFTMAX_PROB || mode == ZR_SOFTMAX_LOGPROB || mode == ZR_SOFTMAX_LOGITS ||
                   mode == ZR_SOFTMAX_LOGITS_BLOCKS,
               "zr_softmax_forward: mode = %d", mode);
  const bool with_blocks = mode == ZR_SOFTMAX_LOGITS_BLOCKS;
  const bool logits_only = mode == ZR_SOFTMAX_LOGITS || with_blocks;
  ZR_CHECK_ARG(!logits_only || d_logits_scratch == nullptr,
               "zr_softmax_forward: ZR_SOFTMAX_LOGITS(_BLOCKS) writes the logits to d_out and takes no d_logits_scratch");
  float* logits = (d_logits_scratch && !logits_only) ? d_logits_scratch : d_out;
  float* partials = nullptr;
  int nblocks = 0;
  // ZR_SOFTMAX_LOGITS_BLOCKS: the product's per-block pairs go straight into the caller's buffer behind the logits and
  // that is all -- no launch folds them; the consumer (zr_beam_expand_blocks) does that itself
  rc = logits_with_partials(ctx, d_D, d_b_d, V, H, d_h, mb, logits, &partials, &nblocks, d_h_packed, d_h_hi, d_h_lo,
                            with_blocks ? d_out + zr_softmax_blocks_offset_floats(V, mb) : nullptr);
  if (rc) return rc;
  if (with_blocks) return ZR_OK;
  // ZR_SOFTMAX_LOGITS: the column statistics go behind the logits in the caller's buffer and no normalised matrix is
  // written -- a consumer that needs only a few entries per column (the beam search) normalises those itself
  float* colstats = logits_only ? d_out + (size_t)V * mb : (float*)stats_ptr(partials, nblocks, mb);
  softmax_colstats_kernel<<<mb, 256, 0, ctx->stream>>>(partials, nblocks, colstats);
  ZR_LAUNCH_CHECK("softmax_colstats_kernel");
  if (logits_only) return ZR_OK;
  const bool vec = (V % 4 == 0) && (((uintptr_t)logits & 15u) == 0) && (((uintptr_t)d_out & 15u) == 0);
  if (vec) {
    dim3 grid((V / 4 + 255) / 256, mb);
    if (mode == ZR_SOFTMAX_PROB)
      softmax_normalize_kernel<0, true><<<grid, 256, 0, ctx->stream>>>(logits, d_out, V, colstats);
    else
      softmax_normalize_kernel<1, true><<<grid, 256, 0, ctx->stream>>>(logits, d_out, V, colstats);
  } else {
    dim3 grid((V + 255) / 256, mb);
    if (mode == ZR_SOFTMAX_PROB)
      softmax_normalize_kernel<0, false><<<grid, 256, 0, ctx->stream>>>(logits, d_out, V, colstats);
    else
      softmax_normalize_kernel<1, false><<<grid, 256, 0, ctx->stream>>>(logits, d_out, V, colstats);
  }
  ZR_LAUNCH_CHECK("softmax_normalize_kernel");
  return ZR_OK;
}

extern "C" {

// zr_softmax_forward on the device's statically allocated scratch array: same kernels, no allocation.  The array is
// split into the two buffers the product needs (re-laid-out activations, then partial column statistics + column
// statistics); both are fully written before they are read, so nothing has to be cleared between calls.
int zr_softmax_forward_static(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb,
                              int mode, float* d_out, float* d_logits_scratch) {
  ZR_CHECK_ARG(ctx != nullptr && ctx->d_static_scratch != nullptr, "zr_softmax_forward_static: null context");
  ctx->fixed_scratch = 1;
  ctx->d_fixed[0] = ctx->d_static_scratch;
  ctx->fixed_bytes[0] = ZR_STATIC_SCRATCH_SLOT0_BYTES;
  ctx->d_fixed[1] = (char*)ctx->d_static_scratch + ZR_STATIC_SCRATCH_SLOT0_BYTES;
  ctx->fixed_bytes[1] = ZR_STATIC_SCRATCH_BYTES - ZR_STATIC_SCRATCH_SLOT0_BYTES;
  const int rc = zr_softmax_forward(ctx, d_D, d_b_d, V, H, d_h, mb, mode, d_out, d_logits_scratch);
  ctx->fixed_scratch = 0;
  return rc;
}

int zr_softmax_logprob_f64(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb,
                           double* d_logp, float* d_logits_scratch) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  rc = check_softmax_args("zr_softmax_logprob_f64", d_D, d_b_d, V, H, d_h, mb);
  if (rc) return rc;
  ZR_CHECK_ARG(d_logp && d_logits_scratch, "zr_softmax_logprob_f64: null output or scratch");
  float* partials = nullptr;
  int nblocks = 0;
  rc = logits_with_partials(ctx, d_D, d_b_d, V, H, d_h, mb, d_logits_scratch, &partials, &nblocks);
  if (rc) return rc;
  double* colstats = (double*)stats_ptr(partials, nblocks, mb);
  softmax_colstats_f64_kernel<<<mb, 256, 0, ctx->stream>>>(d_logits_scratch, V, colstats);
  ZR_LAUNCH_CHECK("softmax_colstats_f64_kernel");
  dim3 grid((V + 255) / 256, mb);
  softmax_logprob_f64_kernel<<<grid, 256, 0, ctx->stream>>>(d_logits_scratch, d_logp, V, colstats);
  ZR_LAUNCH_CHECK("softmax_logprob_f64_kernel");
  return ZR_OK;
}

int zr_softmax_loss(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb,
                    const int* d_target, const int* d_mask01, float* d_logits_scratch, double* h_loss) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  rc = check_softmax_args("zr_softmax_loss", d_D, d_b_d, V, H, d_h, mb);
  if (rc) return rc;
  ZR_CHECK_ARG(d_target && d_mask01 && d_logits_scratch && h_loss, "zr_softmax_loss: null pointer");
  float* partials = nullptr;
  int nblocks = 0;
  rc = logits_with_partials(ctx, d_D, d_b_d, V, H, d_h, mb, d_logits_scratch, &partials, &nblocks);
  if (rc) return rc;
  double* colstats = (double*)stats_ptr(partials, nblocks, mb);
  softmax_colstats_f64_kernel<<<mb, 256, 0, ctx->stream>>>(d_logits_scratch, V, colstats);
  ZR_LAUNCH_CHECK("softmax_colstats_f64_kernel");
  // the loss cell lives in the partials area, which is dead once the column stats exist
  double* d_loss = (double*)partials;
  softmax_loss_kernel<<<1, 256, 0, ctx->stream>>>(d_logits_scratch, V, mb, colstats, d_target, d_mask01, d_loss,
                                                  ctx->d_flags);
  ZR_LAUNCH_CHECK("softmax_loss_kernel");
  ZR_HIP(hipMemcpyAsync(h_loss, d_loss, sizeof(double), hipMemcpyDeviceToHost, ctx->stream));
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  return ZR_OK;
}

}  // extern "C"
