// HBM-bound element-wise pieces of the path: index preparation, the embedding-column gather, the decoder
// state shuffles and the stand-alone fused LSTM gate kernel.  All of them are one read and one write of
// their operands with 16-byte accesses along the contiguous (hidden) dimension.
#include "zr_internal.h"
#include "zr_math.h"

namespace {

__global__ void fill_zero_kernel(uint32_t* p, size_t n_words) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n_words; i += stride) p[i] = 0u;
}

// vocab_to_01 + vocab_to_nonM1 (reference: src/custom_kernels.h:10-32) in one pass.
// `nonneg` may alias `ids` (in-place -1 -> 0, as the reference's input layer does): each element is read and
// then written by the same thread, so neither pointer is declared restrict.
__global__ void vocab_prep_kernel(const int* ids, int n, int V, int* nonneg, int* __restrict__ mask01,
                                  int* __restrict__ flags) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int stride = gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    int id = ids[i];
    const int m = (id == -1) ? 0 : 1;
    if (id == -1) id = 0;
    if (V > 0 && (id < 0 || id >= V)) {
      atomicAdd(&flags[0], 1);
      id = id < 0 ? 0 : V - 1;
    }
    if (nonneg) nonneg[i] = id;
    if (mask01) mask01[i] = m;
  }
}

// vocab_softmax (reference: src/custom_kernels.h:38-50)
__global__ void vocab_softmax_kernel(int* __restrict__ ids, int n, int V, int* __restrict__ mask01,
                                     float* __restrict__ mask01f, int* __restrict__ flags) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int stride = gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    int id = ids[i];
    const int m = (id == -1) ? 0 : 1;
    if (id == -1) id = 0;
    if (V > 0 && (id < 0 || id >= V)) {
      atomicAdd(&flags[0], 1);
      id = id < 0 ? 0 : V - 1;
    }
    ids[i] = id;
    if (mask01) mask01[i] = m;
    if (mask01f) mask01f[i] = (float)m;
  }
}

// One 64-lane wave copies 256 consecutive floats of one column with 16-byte accesses (VEC) or 64 floats
// with 4-byte accesses.  src column index comes from ids (gather), a permutation, or is fixed (broadcast).
template <bool VEC>
__global__ void __launch_bounds__(64)
column_copy_kernel(const float* __restrict__ src, int H, int V, const int* __restrict__ col_ids, int fixed_col,
                   float* __restrict__ dst, int* __restrict__ flags) {
  const int col = blockIdx.y;
  int sc = col_ids ? col_ids[col] : fixed_col;
  if (V > 0 && (sc < 0 || sc >= V)) {
    if (threadIdx.x == 0 && blockIdx.x == 0) atomicAdd(&flags[0], 1);
    sc = sc < 0 ? 0 : V - 1;
  }
  const float* s = src + (size_t)sc * H;
  float* d = dst + (size_t)col * H;
  if (VEC) {
    const int i4 = blockIdx.x * 64 + threadIdx.x;  // index of the float4 inside the column
    if (i4 * 4 < H) ((zr_f32x4*)d)[i4] = ((const zr_f32x4*)s)[i4];
  } else {
    const int i = blockIdx.x * 64 + threadIdx.x;
    if (i < H) d[i] = s[i];
  }
}

// Many columns: a 64-lane wave copies one whole column, four 16-byte loads in flight per lane before the first store
// (a quarter of the workgroups of column_copy_kernel and four times the bytes in flight per wave).
__global__ void __launch_bounds__(256)
column_copy_wide_kernel(const float* __restrict__ src, int H, int V, const int* __restrict__ col_ids, int fixed_col,
                        int n_cols, float* __restrict__ dst, int* __restrict__ flags) {
  const int col = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (col >= n_cols) return;
  const int lane = threadIdx.x & 63;
  int sc = col_ids ? col_ids[col] : fixed_col;
  if (V > 0 && (sc < 0 || sc >= V)) {
    if (lane == 0) atomicAdd(&flags[0], 1);
    sc = sc < 0 ? 0 : V - 1;
  }
  const zr_f32x4* s = (const zr_f32x4*)(src + (size_t)sc * H);
  zr_f32x4* d = (zr_f32x4*)(dst + (size_t)col * H);
  const int n4 = H >> 2;
  for (int base = 0; base < n4; base += 256) {
    zr_f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i4 = base + u * 64 + lane;
      v[u] = s[i4 < n4 ? i4 : n4 - 1];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i4 = base + u * 64 + lane;
      if (i4 < n4) d[i4] = v[u];
    }
  }
}

// The same copy for up to kMaxMulti arrays at once (blockIdx.z picks the array): the per-layer state reorders of a
// decode step are each far too small to fill the chip, so they share one launch.
constexpr int kMaxMulti = 32;
struct MultiCopy {
  const float* src[kMaxMulti];
  float* dst[kMaxMulti];
};
template <bool VEC>
__global__ void __launch_bounds__(64)
multi_column_copy_kernel(MultiCopy a, int H, const int* __restrict__ col_ids, int n_src_cols, int* __restrict__ flags) {
  const int col = blockIdx.y;
  int sc = col_ids[col];
  if (sc < 0 || sc >= n_src_cols) {
    if (threadIdx.x == 0 && blockIdx.x == 0 && blockIdx.z == 0) atomicAdd(&flags[0], 1);
    sc = sc < 0 ? 0 : n_src_cols - 1;
  }
  const float* s = a.src[blockIdx.z] + (size_t)sc * H;
  float* d = a.dst[blockIdx.z] + (size_t)col * H;
  if (VEC) {
    const int i4 = blockIdx.x * 64 + threadIdx.x;
    if (i4 * 4 < H) ((zr_f32x4*)d)[i4] = ((const zr_f32x4*)s)[i4];
  } else {
    const int i = blockIdx.x * 64 + threadIdx.x;
    if (i < H) d[i] = s[i];
  }
}

// Fused gate kernel: the reference's forward_sigmoid_kernel x3, forward_tanh_kernel, forward_c_t_kernel,
// clip_mat_kernel, forward_h_t_kernel and zero_c_t_and_h_t (src/custom_kernels.h:58-192, 2222-2231) in one
// pass: 4 pre-activation reads + c_prev read, c and h written once.
template <bool VEC>
__global__ void __launch_bounds__(64)
lstm_gates_kernel(const float* __restrict__ preact, const float* __restrict__ b_i, const float* __restrict__ b_f,
                  const float* __restrict__ b_c, const float* __restrict__ b_o, const float* __restrict__ cprev,
                  const int* __restrict__ mask01, float clip, int H, int mb, float* __restrict__ h_out,
                  float* __restrict__ c_out, float* g_i, float* g_f, float* g_c, float* g_o) {
  const int n = blockIdx.y;
  const size_t plane = (size_t)H * mb;
  const float m = (float)mask01[n];
  constexpr int W = VEC ? 4 : 1;
  const int j0 = (blockIdx.x * 64 + threadIdx.x) * W;
  if (j0 >= H) return;
  const size_t ix = (size_t)n * H + j0;
  float zi[W], zf[W], zc[W], zo[W], cp[W], bi[W], bf[W], bc[W], bo[W];
  if (VEC) {
    *(zr_f32x4*)zi = *(const zr_f32x4*)(preact + ix);
    *(zr_f32x4*)zf = *(const zr_f32x4*)(preact + plane + ix);
    *(zr_f32x4*)zc = *(const zr_f32x4*)(preact + 2 * plane + ix);
    *(zr_f32x4*)zo = *(const zr_f32x4*)(preact + 3 * plane + ix);
    *(zr_f32x4*)cp = *(const zr_f32x4*)(cprev + ix);
    *(zr_f32x4*)bi = *(const zr_f32x4*)(b_i + j0);
    *(zr_f32x4*)bf = *(const zr_f32x4*)(b_f + j0);
    *(zr_f32x4*)bc = *(const zr_f32x4*)(b_c + j0);
    *(zr_f32x4*)bo = *(const zr_f32x4*)(b_o + j0);
  } else {
    zi[0] = preact[ix];
    zf[0] = preact[plane + ix];
    zc[0] = preact[2 * plane + ix];
    zo[0] = preact[3 * plane + ix];
    cp[0] = cprev[ix];
    bi[0] = b_i[j0];
    bf[0] = b_f[j0];
    bc[0] = b_c[j0];
    bo[0] = b_o[j0];
  }
  float hv[W], cv[W], gi[W], gf[W], gc[W], go[W];
#pragma unroll
  for (int q = 0; q < W; ++q)
    zr_lstm_cell(zi[q] + bi[q], zf[q] + bf[q], zc[q] + bc[q], zo[q] + bo[q], cp[q], m, clip, gi[q], gf[q], gc[q],
                 go[q], cv[q], hv[q]);
  if (VEC) {
    *(zr_f32x4*)(h_out + ix) = *(zr_f32x4*)hv;
    *(zr_f32x4*)(c_out + ix) = *(zr_f32x4*)cv;
    if (g_i) {
      *(zr_f32x4*)(g_i + ix) = *(zr_f32x4*)gi;
      *(zr_f32x4*)(g_f + ix) = *(zr_f32x4*)gf;
      *(zr_f32x4*)(g_c + ix) = *(zr_f32x4*)gc;
      *(zr_f32x4*)(g_o + ix) = *(zr_f32x4*)go;
    }
  } else {
    h_out[ix] = hv[0];
    c_out[ix] = cv[0];
    if (g_i) {
      g_i[ix] = gi[0];
      g_f[ix] = gf[0];
      g_c[ix] = gc[0];
      g_o[ix] = go[0];
    }
  }
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// add_two_mats_kernel (src/custom_kernels.h:1818-1822)
__global__ void __launch_bounds__(256) add_inplace_kernel(float* __restrict__ dst, const float* __restrict__ src,
                                                          long long n) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    dst[i] = dst[i] + src[i];
}

// clip_mat_kernel (src/custom_kernels.h:2220-2231)
__global__ void __launch_bounds__(256) clip_inplace_kernel(float* __restrict__ x, long long n, float threshold) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const float v = x[i];
    x[i] = v > threshold ? threshold : (v < -threshold ? -threshold : v);  // a NaN stays a NaN, as in the reference
  }
}

}  // namespace

extern "C" {

int zr_clip_inplace(zr_ctx* ctx, float* d_x, long long n, float threshold) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n >= 0 && (n == 0 || d_x) && threshold >= 0.0f, "zr_clip_inplace: null pointer, n = %lld or threshold = %g",
               n, (double)threshold);
  if (n == 0) return ZR_OK;
  const int blocks = (int)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
  clip_inplace_kernel<<<blocks, 256, 0, ctx->stream>>>(d_x, n, threshold);
  ZR_LAUNCH_CHECK("clip_inplace_kernel");
  return ZR_OK;
}

int zr_add_inplace(zr_ctx* ctx, float* d_dst, const float* d_src, long long n) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n >= 0 && (n == 0 || (d_dst && d_src)), "zr_add_inplace: null pointer or n = %lld", n);
  if (n == 0) return ZR_OK;
  const int blocks = (int)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
  add_inplace_kernel<<<blocks, 256, 0, ctx->stream>>>(d_dst, d_src, n);
  ZR_LAUNCH_CHECK("add_inplace_kernel");
  return ZR_OK;
}

int zr_memset_zero(zr_ctx* ctx, void* d_dst, size_t bytes) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(bytes == 0 || d_dst, "zr_memset_zero: null pointer");
  ZR_CHECK_ARG((bytes & 3u) == 0 && ((uintptr_t)d_dst & 3u) == 0, "zr_memset_zero: size/pointer must be 4-byte aligned");
  if (bytes == 0) return ZR_OK;
  const size_t words = bytes / 4;
  const int blocks = (int)((words + 255) / 256 < 2048 ? (words + 255) / 256 : 2048);
  fill_zero_kernel<<<blocks, 256, 0, ctx->stream>>>((uint32_t*)d_dst, words);
  ZR_LAUNCH_CHECK("fill_zero_kernel");
  return ZR_OK;
}

int zr_vocab_prep(zr_ctx* ctx, const int* d_ids, int n, int vocab_size, int* d_ids_nonneg, int* d_mask01) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n >= 0, "zr_vocab_prep: n = %d", n);
  ZR_CHECK_ARG(n == 0 || d_ids, "zr_vocab_prep: d_ids is null");
  if (n == 0) return ZR_OK;
  const int blocks = (n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024;
  vocab_prep_kernel<<<blocks, 256, 0, ctx->stream>>>(d_ids, n, vocab_size, d_ids_nonneg, d_mask01, ctx->d_flags);
  ZR_LAUNCH_CHECK("vocab_prep_kernel");
  return ZR_OK;
}

int zr_vocab_prep_softmax(zr_ctx* ctx, int* d_ids_inout, int n, int vocab_size, int* d_mask01, float* d_mask01_float) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n >= 0, "zr_vocab_prep_softmax: n = %d", n);
  ZR_CHECK_ARG(n == 0 || d_ids_inout, "zr_vocab_prep_softmax: d_ids is null");
  if (n == 0) return ZR_OK;
  const int blocks = (n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024;
  vocab_softmax_kernel<<<blocks, 256, 0, ctx->stream>>>(d_ids_inout, n, vocab_size, d_mask01, d_mask01_float,
                                                        ctx->d_flags);
  ZR_LAUNCH_CHECK("vocab_softmax_kernel");
  return ZR_OK;
}

static int column_copy(zr_ctx* ctx, const char* who, const float* src, int H, int V, const int* ids, int fixed_col,
                       int n, float* dst) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(H > 0 && n >= 0, "%s: H = %d, n = %d", who, H, n);
  ZR_CHECK_ARG(n == 0 || (src && dst), "%s: null pointer", who);
  ZR_CHECK_ARG(n <= 65535, "%s: at most 65535 columns per call (got %d)", who, n);
  if (n == 0) return ZR_OK;
  const bool vec = (H % 4 == 0) && aligned16(src) && aligned16(dst);
  if (vec && n >= 1024) {
    column_copy_wide_kernel<<<(n + 3) / 4, 256, 0, ctx->stream>>>(src, H, V, ids, fixed_col, n, dst, ctx->d_flags);
  } else if (vec) {
    dim3 grid((H / 4 + 63) / 64, n);
    column_copy_kernel<true><<<grid, 64, 0, ctx->stream>>>(src, H, V, ids, fixed_col, dst, ctx->d_flags);
  } else {
    dim3 grid((H + 63) / 64, n);
    column_copy_kernel<false><<<grid, 64, 0, ctx->stream>>>(src, H, V, ids, fixed_col, dst, ctx->d_flags);
  }
  ZR_LAUNCH_CHECK("column_copy_kernel");
  return ZR_OK;
}

int zr_embed_gather(zr_ctx* ctx, const float* d_W, int H, int V, const int* d_ids, int mb, float* d_x) {
  ZR_CHECK_ARG(V > 0, "zr_embed_gather: V = %d", V);
  ZR_CHECK_ARG(mb == 0 || d_ids, "zr_embed_gather: d_ids is null");
  return column_copy(ctx, "zr_embed_gather", d_W, H, V, d_ids, 0, mb, d_x);
}

int zr_gather_columns(zr_ctx* ctx, const float* d_src, int H, const int* d_perm, int n, float* d_dst) {
  ZR_CHECK_ARG(n == 0 || d_perm, "zr_gather_columns: d_perm is null");
  ZR_CHECK_ARG(d_src != d_dst || n == 0, "zr_gather_columns: d_dst must not alias d_src");
  return column_copy(ctx, "zr_gather_columns", d_src, H, 0, d_perm, 0, n, d_dst);
}

int zr_gather_columns_multi(zr_ctx* ctx, int n_arrays, const float* const d_src[], int H, const int* d_perm,
                            int n_src_cols, int n, float* const d_dst[]) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n_arrays >= 0 && n_arrays <= kMaxMulti, "zr_gather_columns_multi: %d arrays (at most %d)", n_arrays,
               kMaxMulti);
  ZR_CHECK_ARG(H > 0 && n >= 0 && n <= 65535 && n_src_cols > 0, "zr_gather_columns_multi: H = %d, n = %d, %d source columns",
               H, n, n_src_cols);
  if (n_arrays == 0 || n == 0) return ZR_OK;
  ZR_CHECK_ARG(d_src && d_dst && d_perm, "zr_gather_columns_multi: null pointer");
  MultiCopy a;
  bool vec = H % 4 == 0;
  for (int i = 0; i < kMaxMulti; ++i) {
    a.src[i] = i < n_arrays ? d_src[i] : nullptr;
    a.dst[i] = i < n_arrays ? d_dst[i] : nullptr;
    if (i < n_arrays) {
      ZR_CHECK_ARG(d_src[i] && d_dst[i], "zr_gather_columns_multi: array %d is null", i);
      ZR_CHECK_ARG(d_src[i] != d_dst[i], "zr_gather_columns_multi: array %d: d_dst must not alias d_src", i);
      vec = vec && aligned16(d_src[i]) && aligned16(d_dst[i]);
    }
  }
  if (vec) {
    dim3 grid((H / 4 + 63) / 64, n, n_arrays);
    multi_column_copy_kernel<true><<<grid, 64, 0, ctx->stream>>>(a, H, d_perm, n_src_cols, ctx->d_flags);
  } else {
    dim3 grid((H + 63) / 64, n, n_arrays);
    multi_column_copy_kernel<false><<<grid, 64, 0, ctx->stream>>>(a, H, d_perm, n_src_cols, ctx->d_flags);
  }
  ZR_LAUNCH_CHECK("multi_column_copy_kernel");
  return ZR_OK;
}

int zr_broadcast_column(zr_ctx* ctx, const float* d_src_col, int H, int n, float* d_dst) {
  return column_copy(ctx, "zr_broadcast_column", d_src_col, H, 0, nullptr, 0, n, d_dst);
}

int zr_lstm_gates(zr_ctx* ctx, const float* d_preact, const float* const d_b[4], const float* d_cprev,
                  const int* d_mask01, float clip_threshold, int H, int mb, float* d_h, float* d_c,
                  float* const d_gates[4]) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(H > 0 && mb > 0, "zr_lstm_gates: H = %d, mb = %d", H, mb);
  ZR_CHECK_ARG(mb <= 65535, "zr_lstm_gates: mb = %d exceeds 65535", mb);
  ZR_CHECK_ARG(d_preact && d_b && d_cprev && d_mask01 && d_h && d_c, "zr_lstm_gates: null pointer");
  for (int g = 0; g < 4; ++g) {
    ZR_CHECK_ARG(d_b[g] != nullptr, "zr_lstm_gates: d_b[%d] is null", g);
    ZR_CHECK_ARG(!d_gates || d_gates[g], "zr_lstm_gates: d_gates[%d] is null", g);
  }
  float* gi = d_gates ? d_gates[0] : nullptr;
  float* gf = d_gates ? d_gates[1] : nullptr;
  float* gc = d_gates ? d_gates[2] : nullptr;
  float* go = d_gates ? d_gates[3] : nullptr;
  bool vec = (H % 4 == 0) && aligned16(d_preact) && aligned16(d_cprev) && aligned16(d_h) && aligned16(d_c);
  for (int g = 0; g < 4; ++g) vec = vec && aligned16(d_b[g]) && (!d_gates || aligned16(d_gates[g]));
  if (vec) {
    dim3 grid((H / 4 + 63) / 64, mb);
    lstm_gates_kernel<true><<<grid, 64, 0, ctx->stream>>>(d_preact, d_b[0], d_b[1], d_b[2], d_b[3], d_cprev,
                                                          d_mask01, clip_threshold, H, mb, d_h, d_c, gi, gf, gc, go);
  } else {
    dim3 grid((H + 63) / 64, mb);
    lstm_gates_kernel<false><<<grid, 64, 0, ctx->stream>>>(d_preact, d_b[0], d_b[1], d_b[2], d_b[3], d_cprev,
                                                           d_mask01, clip_threshold, H, mb, d_h, d_c, gi, gf, gc, go);
  }
  ZR_LAUNCH_CHECK("lstm_gates_kernel");
  return ZR_OK;
}

}  // extern "C"
