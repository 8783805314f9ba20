// Training backward for the stacked LSTM, the output layer and the attention layer; dropout.
//
// Gradients are those of the log-likelihood, as in the reference (its loss layer's error is D^T (onehot - p),
// src/softmax.hpp:700-712; update_weights adds learning_rate * gradient, :232-300).
//
// What is different from the reference's schedule (src/LSTM.hpp:542-1270, src/LSTM_HH.hpp:336-900):
//  * the element-wise error kernels of a node (d_ERRt_ct_kernel, d_ERRnTOt_ot_kernel, d_ERRnTOt_ft_it_kernel x2,
//    d_ERRnTOt_tanhcpt_kernel, zero_columns_kernel x2, three cublas geam additions; src/custom_kernels.h:199-262)
//    are one kernel that reads the saved gates once and writes the four pre-activation errors once;
//  * the eight W^T * error products of a node are one batched product against the gate matrices stacked as
//    4H x H (error to h_{t-1} and error to the layer below share the right-hand side);
//  * the weight gradients are not accumulated step by step (8 rank-mb updates of H x H matrices per node, each a
//    full read-modify-write of the matrix): every node's pre-activation errors are kept (4H x T*mb per layer, a
//    few hundred MB) and each gradient is ONE product with K = T * mb after the sweep.
#include <math.h>

#include "zr_internal.h"

struct zr_lstm_train {
  int H;
  // [2][H x 4H] column-major: the TRANSPOSE of Wh stacked over the gates, then of M: element (k, g*H + j) = W_g[j][k].
  // The error products sum_g W_g^T err_g are then plain products with contiguous weight rows.
  float* d_stack;
  // the same two matrices in the matrix cores' k-interleaved layout ([kp/4][ldp][4], ldp = H rounded up to 32,
  // kp = 4H rounded up to 8), kp*ldp floats each: the operand of the whole-grid backward sweep
  float* d_stack_pack;
  int ldp, kp;
};

namespace {

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

__global__ void __launch_bounds__(256) stack_gates_kernel(const float* __restrict__ g0, const float* __restrict__ g1,
                                                          const float* __restrict__ g2, const float* __restrict__ g3,
                                                          int H, float* __restrict__ dst) {
  // dst: H x 4H column-major, dst[k + (g*H + j)*H] = W_g[j + k*H]; 32 x 32 tiles through LDS
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int g = blockIdx.z;
  const float* src = g == 0 ? g0 : (g == 1 ? g1 : (g == 2 ? g2 : g3));
  const int j0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
  for (int i = ty; i < 32; i += 8) {
    const int j = j0 + tx, k = k0 + i;
    tile[i][tx] = (j < H && k < H) ? src[j + (long long)k * H] : 0.0f;
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    const int k = k0 + tx, j = j0 + i;
    if (j < H && k < H) dst[k + ((long long)g * H + j) * H] = tile[tx][i];
  }
}

__global__ void __launch_bounds__(256) unstack_gates_kernel(const float* __restrict__ src, int H, float* __restrict__ g0,
                                                            float* __restrict__ g1, float* __restrict__ g2,
                                                            float* __restrict__ g3) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= 4LL * H * H) return;
  const int r = (int)(i % (4 * H));
  const int k = (int)(i / (4 * H));
  const int g = r / H, j = r - g * H;
  float* dst = g == 0 ? g0 : (g == 1 ? g1 : (g == 2 ? g2 : g3));
  dst[j + (long long)k * H] = src[i];
}

// One node: total error at h_t (from above + from t+1), cell error, the four pre-activation errors, error to c_{t-1}.
//   g_i, g_f, g_c, g_o: the node's saved gate activations (H x mb each); dg: the node's 4H x mb block of the layer's error matrix
//   (element (g*H + j, b) at dg[b*4H + g*H + j]); ec: in = error arriving at c_t from t+1 (or null at the last step),
//   out = error for c_{t-1} (may alias).
__global__ void __launch_bounds__(256) lstm_node_backward_kernel(
    const float* __restrict__ g_i, const float* __restrict__ g_f, const float* __restrict__ g_c,
    const float* __restrict__ g_o, const float* __restrict__ c, const float* __restrict__ cprev,
    const int* __restrict__ mask01, const float* __restrict__ err_above, const float* __restrict__ err_next,
    const float* ec_in, float* ec_out, int H, int mb, float* __restrict__ dg) {
  const int b = blockIdx.y;
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= H) return;
  const size_t ix = (size_t)b * H + j;
  const float m = (float)mask01[b];
  float eh = 0.0f;
  if (err_above) eh += err_above[ix];
  if (err_next) eh += err_next[ix];
  eh *= m;
  const float gi = g_i[ix], gf = g_f[ix], gc = g_c[ix], go = g_o[ix];
  const float th = tanhf(c[ix]);
  const float errt_ct = eh * go * (1.0f - th * th);
  const float ec = ((ec_in ? ec_in[ix] : 0.0f) + errt_ct) * m;
  float* d = dg + (size_t)b * 4 * H + j;
  d[0] = ec * gc * gi * (1.0f - gi);
  d[H] = ec * cprev[ix] * gf * (1.0f - gf);
  d[2 * (size_t)H] = ec * gi * (1.0f - gc * gc);
  d[3 * (size_t)H] = eh * th * go * (1.0f - go);
  ec_out[ix] = ec * gf;
}

// The same for up to 8 independent nodes in one launch (blockIdx.z picks the node).
struct NodeBackwardGroup {
  const float* gates[8];      // node's four gate planes, H*mb apart
  const float* c[8];
  const float* cprev[8];
  const int* mask01[8];
  const float* err_above[8];  // may be null
  const float* err_next[8];   // may be null
  float* ec[8];               // cell error, updated in place
  float* dg[8];
  float* dgp[8];              // non-null: second copy of dg, k-interleaved [4H/4][mb][4] (the grouped product's right side)
  int clamp_above[8];         // err_above is an error product of the layer above (clamped like err_next), not the loss layer's
};
// err_clip > 0: the error products a node receives are clamped to +-err_clip on arrival (clip_mat_kernel on
// d_ERRnTOt_htM1 and d_ERRnTOt_h_Below, src/LSTM.hpp:792, src/LSTM_HH.hpp:665,756; a NaN stays a NaN)
__device__ __forceinline__ float clamp_error(float v, float err_clip) {
  return v > err_clip ? err_clip : (v < -err_clip ? -err_clip : v);
}
__global__ void __launch_bounds__(256) lstm_node_backward_group_kernel(NodeBackwardGroup G, int H, int mb, float err_clip) {
  const int u = blockIdx.z;
  const int b = blockIdx.y;
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= H) return;
  const size_t n = (size_t)H * mb;
  const size_t ix = (size_t)b * H + j;
  const float m = (float)G.mask01[u][b];
  float eh = 0.0f;
  if (G.err_above[u]) {
    const float e = G.err_above[u][ix];
    eh += (err_clip > 0.0f && G.clamp_above[u]) ? clamp_error(e, err_clip) : e;
  }
  if (G.err_next[u]) {
    const float e = G.err_next[u][ix];
    eh += err_clip > 0.0f ? clamp_error(e, err_clip) : e;
  }
  eh *= m;
  const float* gt = G.gates[u];
  const float gi = gt[ix], gf = gt[n + ix], gc = gt[2 * n + ix], go = gt[3 * n + ix];
  const float th = tanhf(G.c[u][ix]);
  const float errt_ct = eh * go * (1.0f - th * th);
  const float ec = (G.ec[u][ix] + errt_ct) * m;
  float* d = G.dg[u] + (size_t)b * 4 * H + j;
  const float di = ec * gc * gi * (1.0f - gi), df = ec * G.cprev[u][ix] * gf * (1.0f - gf);
  const float dc = ec * gi * (1.0f - gc * gc), dob = eh * th * go * (1.0f - go);
  d[0] = di;
  d[H] = df;
  d[2 * (size_t)H] = dc;
  d[3 * (size_t)H] = dob;
  if (G.dgp[u]) {
    // row k = g*H + j of the 4H x mb matrix, column b
    float* p = G.dgp[u];
    const size_t k0 = (size_t)j, k1 = (size_t)H + j, k2 = 2 * (size_t)H + j, k3 = 3 * (size_t)H + j;
    p[((k0 >> 2) * mb + b) * 4 + (k0 & 3)] = di;
    p[((k1 >> 2) * mb + b) * 4 + (k1 & 3)] = df;
    p[((k2 >> 2) * mb + b) * 4 + (k2 & 3)] = dc;
    p[((k3 >> 2) * mb + b) * 4 + (k3 & 3)] = dob;
  }
  G.ec[u][ix] = ec * gf;
}

// Sum over the unmasked columns of log((double) p[target, column]): train_perplexity_kernel
// (src/custom_kernels.h:478-488), one workgroup, fixed summation order.
__global__ void __launch_bounds__(256) train_logprob_kernel(const float* __restrict__ prob, int V, int n,
                                                            const int* __restrict__ target,
                                                            const int* __restrict__ mask01, double* __restrict__ out) {
  __shared__ double part[256];
  double s = 0.0;
  for (int i = threadIdx.x; i < n; i += 256)
    if (mask01[i] == 1) s += log((double)prob[(size_t)i * V + target[i]]);
  part[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) part[threadIdx.x] += part[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = part[0];
}

// dst (cols x rows, column-major with leading dimension ldd, starting at row offset row0) = src^T, src rows x cols
// column-major (ld = rows): dst[row0 + c + r*ldd] = src[r + c*rows].  32 x 32 tiles through LDS.
__global__ void __launch_bounds__(256) transpose_kernel(const float* __restrict__ src, int rows, int cols,
                                                        float* __restrict__ dst, long long ldd, int row0) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const int r0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
  for (int i = ty; i < 32; i += 8) {
    const int r = r0 + tx, cc = c0 + i;
    tile[i][tx] = (r < rows && cc < cols) ? src[r + (long long)cc * rows] : 0.0f;
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    const int cc = c0 + tx, r = r0 + i;
    if (r < rows && cc < cols) dst[row0 + cc + (long long)r * ldd] = tile[tx][i];
  }
}

// The same with 64 x 64 tiles and 16-byte accesses on both sides, for rows, cols, ldd and row0 multiples of 4 and
// 16-byte aligned bases (a thread reads four consecutive rows of a source column and writes four consecutive
// columns, which are consecutive in dst, of a source row).
__global__ void __launch_bounds__(256) transpose_wide_kernel(const float* __restrict__ src, int rows, int cols,
                                                             float* __restrict__ dst, long long ldd, int row0) {
  __shared__ float tile[64][65];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;  // 16 x 16
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + 4 * tx, cl = ty + 16 * i, cc = c0 + cl;
    zr_f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    if (r < rows && cc < cols) v = *(const zr_f32x4*)(src + r + (long long)cc * rows);
#pragma unroll
    for (int k = 0; k < 4; ++k) tile[cl][4 * tx + k] = v[k];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int rl = ty + 16 * i, r = r0 + rl, cc = c0 + 4 * tx;
    if (r < rows && cc < cols) {
      zr_f32x4 v;
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = tile[4 * tx + k][rl];
      *(zr_f32x4*)(dst + row0 + cc + (long long)r * ldd) = v;
    }
  }
}

// Row sums of a (rows x n, column-major) in two stages with a fixed summation order: stage 1 sums column chunk
// blockIdx.y for 64 rows per wave into partial[chunk][rows]; stage 2 adds the chunks.
__global__ void __launch_bounds__(64) row_sum_partial_kernel(const float* __restrict__ a, int rows, long long n,
                                                             long long chunk, float* __restrict__ partial) {
  const int r = blockIdx.x * 64 + threadIdx.x;
  if (r >= rows) return;
  const long long k0 = (long long)blockIdx.y * chunk;
  const long long k1 = k0 + chunk < n ? k0 + chunk : n;
  float s = 0.0f;
  for (long long k = k0; k < k1; ++k) s += a[r + k * rows];
  partial[(size_t)blockIdx.y * rows + r] = s;
}
// The same sums in the same order, four consecutive rows per thread with 16-byte loads (rows % 4 == 0, a 16-byte
// aligned): 256 rows per wave.
__global__ void __launch_bounds__(64) row_sum_partial_wide_kernel(const float* __restrict__ a, int rows, long long n,
                                                                  long long chunk, float* __restrict__ partial) {
  const int r = (blockIdx.x * 64 + threadIdx.x) * 4;
  if (r >= rows) return;
  const long long k0 = (long long)blockIdx.y * chunk;
  const long long k1 = k0 + chunk < n ? k0 + chunk : n;
  zr_f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
  for (long long k = k0; k < k1; ++k) s += *(const zr_f32x4*)(a + r + k * rows);
  *(zr_f32x4*)(partial + (size_t)blockIdx.y * rows + r) = s;
}
__global__ void __launch_bounds__(64) row_sum_final_kernel(const float* __restrict__ partial, int rows, int chunks,
                                                           float* __restrict__ out, int accumulate) {
  const int r = blockIdx.x * 64 + threadIdx.x;
  if (r >= rows) return;
  float s = 0.0f;
  for (int c = 0; c < chunks; ++c) s += partial[(size_t)c * rows + r];
  out[r] = accumulate ? out[r] + s : s;
}

// Embedding gradient: column id[k] of dW += err column k for every unmasked position.  Float atomics: the order of
// the additions into one column is not fixed (the reference's sparse W gradient kernels use atomicAdd as well).
__global__ void __launch_bounds__(256) embed_grad_kernel(const float* __restrict__ err, const int* __restrict__ ids,
                                                         const int* __restrict__ mask01, int H, int V,
                                                         float* __restrict__ dW) {
  const int k = blockIdx.y;
  if (mask01[k] != 1) return;
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= H) return;
  int id = ids[k];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  atomicAdd(&dW[(size_t)id * H + j], err[(size_t)k * H + j]);
}

// p (V x n probabilities) -> e = onehot(target) - p on unmasked columns, 0 on masked ones, in place.
// VEC: four consecutive rows per thread with 16-byte accesses (V % 4 == 0, p 16-byte aligned).
template <bool VEC>
__global__ void __launch_bounds__(256) softmax_error_kernel(float* __restrict__ p, int V, const int* __restrict__ target,
                                                            const int* __restrict__ mask01) {
  const int col = blockIdx.y;
  const bool on = mask01[col] == 1;
  const int tg = target[col];
  if (VEC) {
    const int v = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (v >= V) return;
    zr_f32x4* q = (zr_f32x4*)(p + (size_t)col * V + v);
    const zr_f32x4 x = *q;
    zr_f32x4 e;
#pragma unroll
    for (int c = 0; c < 4; ++c) e[c] = on ? (v + c == tg ? 1.0f : 0.0f) - x[c] : 0.0f;
    *q = e;
  } else {
    const int v = blockIdx.x * 256 + threadIdx.x;
    if (v >= V) return;
    const size_t ix = (size_t)col * V + v;
    p[ix] = on ? (v == tg ? 1.0f : 0.0f) - p[ix] : 0.0f;
  }
}

// sum of squares, two deterministic stages.  1024 threads per block and 16-byte loads (when g is 16-byte aligned)
// keep enough bytes in flight to stream a large gradient at memory speed from only gridDim.x = 256 blocks, the
// number of partial sums the second stage adds up in a fixed order.
__global__ void __launch_bounds__(1024) sumsq_partial_kernel(const float* __restrict__ g, long long n, int vec,
                                                             double* __restrict__ partial) {
  __shared__ double s[1024];
  double acc = 0.0;
  const long long tid = (long long)blockIdx.x * 1024 + threadIdx.x, nthr = (long long)gridDim.x * 1024;
  long long done = 0;
  if (vec) {
    const long long n4 = n >> 2;
    const zr_f32x4* g4 = (const zr_f32x4*)g;
    for (long long i = tid; i < n4; i += nthr) {
      const zr_f32x4 v = g4[i];
#pragma unroll
      for (int c = 0; c < 4; ++c) acc += (double)v[c] * (double)v[c];
    }
    done = n4 << 2;
  }
  for (long long i = done + tid; i < n; i += nthr) {
    const double v = g[i];
    acc += v * v;
  }
  s[threadIdx.x] = acc;
  __syncthreads();
  for (int st = 512; st > 0; st >>= 1) {
    if ((int)threadIdx.x < st) s[threadIdx.x] += s[threadIdx.x + st];
    __syncthreads();
  }
  if (threadIdx.x == 0) partial[blockIdx.x] = s[0];
}

// second stage of the whole-model norm (norm_clip_GPU_v2_p1, src/custom_kernels.h:1083-1099): the partial sums added in a
// fixed order, times scale^2, into (or, with reset, over) the caller's accumulator
__global__ void sumsq_accumulate_kernel(const double* __restrict__ partial, int n_partial, float scale,
                                        double* __restrict__ sumsq, int reset) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  double ss = 0.0;
  for (int i = 0; i < n_partial; ++i) ss += partial[i];
  ss *= (double)scale * (double)scale;
  *sumsq = reset ? ss : *sumsq + ss;
}

// W += lr * clip(scale * g).  mode ZR_CLIP_MATRIX_NORM: the gradient is shrunk by threshold / ||scale * g|| when that norm
// (from `partial`) exceeds threshold; ZR_CLIP_WHOLE_NORM: the same with the norm sqrt(*sumsq) the caller accumulated
// over every gradient of the model; ZR_CLIP_ELEMENT: every element of scale * g is clamped to +-threshold.
__global__ void __launch_bounds__(256) sgd_apply_kernel(float* __restrict__ W, const float* __restrict__ g, long long n,
                                                        float scale, int mode, float threshold, float lr,
                                                        const double* __restrict__ partial, int n_partial,
                                                        const double* __restrict__ sumsq) {
  __shared__ float coef_s;
  if (threadIdx.x == 0) {
    float coef = 1.0f;
    if (mode == ZR_CLIP_MATRIX_NORM) {
      double ss = 0.0;
      for (int i = 0; i < n_partial; ++i) ss += partial[i];
      const float norm = (float)sqrt(ss) * fabsf(scale);
      if (norm > threshold) coef = threshold / norm;
    } else if (mode == ZR_CLIP_WHOLE_NORM) {
      const float norm = (float)sqrt(*sumsq);
      if (norm > threshold) coef = threshold / norm;
    }
    coef_s = coef;
  }
  __syncthreads();
  const long long first = (long long)blockIdx.x * 256 + threadIdx.x, stride = (long long)gridDim.x * 256;
  if (mode == ZR_CLIP_ELEMENT) {
    for (long long i = first; i < n; i += stride) {
      const float x = scale * g[i];
      W[i] += lr * (x > threshold ? threshold : (x < -threshold ? -threshold : x));  // a NaN stays a NaN (clip_mat_kernel)
    }
    return;
  }
  const float f = lr * coef_s * scale;
  for (long long i = first; i < n; i += stride) W[i] += f * g[i];
}


// ---- attention backward (attention_node::back_prop, src/attention_node.hpp:398-669) --------------------------------

__device__ __forceinline__ float bwd_wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
// Sum over the 256 threads of a workgroup, in every thread.  `red` holds 4 floats.
__device__ __forceinline__ float bwd_block_sum(float v, float* red) {
  v = bwd_wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// zero_h_t + tanh_grad_kernel (src/custom_kernels.h:2212, :1835): e = err * mask * (1 - h~^2)
__global__ void __launch_bounds__(256) attn_bwd_e_kernel(const float* __restrict__ err, const float* __restrict__ htild,
                                                         const int* __restrict__ mask01, int H, long long n,
                                                         float* __restrict__ e) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const float t = htild[i];
    e[i] = err[i] * (float)mask01[i / H] * (1.0f - t * t);
  }
}

// error_alignments_kernel_large + error_hs_ct_kernel_large (:1968, :2179), one workgroup per (window slot, column):
// err_as[j + W*b] = <err_ct[:, b], h_s>, and the error of that source state += err_ct[:, b] * a.  Distinct slots of a
// column are distinct source positions, so no two workgroups touch the same error column.
__global__ void __launch_bounds__(256) attn_bwd_align_kernel(const float* __restrict__ err_ct,
                                                             const float* const* __restrict__ table,
                                                             float* const* __restrict__ err_table,
                                                             const int* __restrict__ batch_info,
                                                             const int* __restrict__ indices,
                                                             const float* __restrict__ align, int H, int mb, int W,
                                                             int longest, float* __restrict__ err_as) {
  __shared__ float red[4];
  const int j = blockIdx.x, b = blockIdx.y;
  const int s = indices[b + (size_t)mb * j];
  if (s == -1) {
    if (threadIdx.x == 0) err_as[j + (size_t)W * b] = 0.0f;
    return;
  }
  int t = batch_info[b] - 1 - s + batch_info[mb + b];
  t = t < 0 ? 0 : (t >= longest ? longest - 1 : t);
  const float* hs = table[t] + (size_t)b * H;
  float* ehs = err_table[t] + (size_t)b * H;
  const float* ec = err_ct + (size_t)b * H;
  const float a = align[b + (size_t)mb * j];
  float sum = 0.0f;
  for (int i = threadIdx.x; i < H; i += 256) {
    const float v = ec[i];
    sum += v * hs[i];
    ehs[i] += v * a;
  }
  sum = bwd_block_sum(sum, red);
  if (threadIdx.x == 0) err_as[j + (size_t)W * b] = sum;
}

// Per column: sigma_1 again (sigmoid_kernel, double), error_pt_kernel (:2006), the factors of att_vp_error and
// grad_W_p_kernel (:2040, :2051) that depend on the column only, and get_ht_scalings_Wa_grad_kernel (:2094) with the
// Gaussian factors alignment_reduction_kernel caches (1 on empty slots).
//   col[0][b] = err_pt * sig * (1 - sig) * S_b     (times tanh_1: the v_p gradient's summand)
//   col[1][b] = err_pt * S_b,  col[2][b] = sig     (grad_W_p_kernel multiplies in the reference's order)
__global__ void __launch_bounds__(64) attn_bwd_column_kernel(const float* __restrict__ tanh1,
                                                             const float* __restrict__ v_p,
                                                             const int* __restrict__ batch_info,
                                                             const int* __restrict__ indices,
                                                             const float* __restrict__ align,
                                                             const float* __restrict__ p_t,
                                                             const float* __restrict__ err_as, int H, int mb, int W,
                                                             float sigma_sq, float* __restrict__ col,
                                                             float* __restrict__ scal) {
  const int b = blockIdx.x, lane = threadIdx.x;
  float s = 0.0f;
  for (int k = lane; k < H; k += 64) s += v_p[k] * tanh1[(size_t)b * H + k];
  s = bwd_wave_sum(s);
  const float sig = (float)(1.0 / (1.0 + exp(-1.0 * (double)s)));
  const float p = p_t[b];
  float ept = 0.0f, tot = 0.0f;  // tot = sum_k err_as[k] * a_k
  for (int j = lane; j < W; j += 64) {
    const float ea = err_as[j + (size_t)W * b] * align[b + (size_t)mb * j];
    tot += ea;
    ept += ea * (((float)indices[b + (size_t)mb * j] - p) / sigma_sq);
  }
  ept = bwd_wave_sum(ept);
  tot = bwd_wave_sum(tot);
  const float len = (float)batch_info[b];
  if (lane == 0) {
    col[b] = ept * sig * (1.0f - sig) * len;
    col[mb + b] = ept * len;
    col[2 * mb + b] = sig;
  }
  // scaling_j = err_as_j a_j (1 - a_j / g_j) - sum_{k != j} err_as_k a_k a_j / g_j  =  err_as_j a_j - (a_j / g_j) tot:
  // the reference's sum with the j-th term folded in, O(W) per slot instead of O(W^2)
  for (int j = lane; j < W; j += 64) {
    const int sidx = indices[b + (size_t)mb * j];
    float g = 1.0f;
    if (sidx != -1) {
      const float d = p - (float)sidx;
      g = expf((-1.0f * d * d) / (2.0f * sigma_sq));
    }
    const float aj = align[b + (size_t)mb * j];
    scal[j + (size_t)W * b] = err_as[j + (size_t)W * b] * aj - (aj / g) * tot;
  }
}

// att_vp_error and grad_W_p_kernel (:2040, :2051) in one pass over tanh_1
__global__ void __launch_bounds__(256) attn_bwd_vp_wp_kernel(const float* __restrict__ tanh1,
                                                             const float* __restrict__ v_p,
                                                             const float* __restrict__ col, int H, int mb, long long n,
                                                             float* __restrict__ tv, float* __restrict__ tw) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const int b = (int)(i / H), k = (int)(i % H);
    const float t = tanh1[i], sig = col[2 * mb + b];
    tv[i] = col[b] * t;
    tw[i] = col[mb + b] * v_p[k] * sig * (1.0f - sig) * (1.0f - t * t);
  }
}

// The loop of src/attention_node.hpp:580-601 for one column per workgroup: h_s_sum[:, b] = sum_j scaling_j h_s_j
// (scale_ht_kernel + add_two_mats_kernel) and the error of h_s_j += scaling_j * (W_a^T h)[:, b] (copy_errors_source).
__global__ void __launch_bounds__(256) attn_bwd_hs_kernel(const float* __restrict__ q,
                                                          const float* const* __restrict__ table,
                                                          float* const* __restrict__ err_table,
                                                          const int* __restrict__ batch_info,
                                                          const int* __restrict__ indices,
                                                          const float* __restrict__ scal, int H, int mb, int W,
                                                          int longest, float* __restrict__ hs_sum) {
  const int b = blockIdx.x;
  const int len = batch_info[b], off = batch_info[mb + b];
  for (int i0 = 0; i0 < H; i0 += 256) {
    const int i = i0 + threadIdx.x;
    const bool ok = i < H;
    const float qv = ok ? q[(size_t)b * H + i] : 0.0f;
    float acc = 0.0f;
    for (int j = 0; j < W; ++j) {
      const int s = indices[b + (size_t)mb * j];
      if (s == -1) continue;
      int t = len - 1 - s + off;
      t = t < 0 ? 0 : (t >= longest ? longest - 1 : t);
      const float sc = scal[j + (size_t)W * b];
      if (ok) {
        acc += table[t][(size_t)b * H + i] * sc;
        err_table[t][(size_t)b * H + i] += qv * sc;
      }
    }
    if (ok) hs_sum[(size_t)b * H + i] = acc;
  }
}

// dropout_kernel (src/custom_kernels.h:1556-1560)
__global__ void __launch_bounds__(256) dropout_kernel(const float* __restrict__ uniform, float rate, float* __restrict__ x,
                                                      long long n) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    x[i] = (float)(uniform[i] < rate) * (1.0f / rate) * x[i];
}

// Uniform numbers in (0, 1] from a counter-based generator (the reference fills its masks with curandGenerateUniform,
// whose stream cannot be reproduced; what matters is that the numbers are uniform, independent of each other and a
// pure function of (seed, call counter, index)): 32 bits of a 64-bit mix of the three, as (bits + 1) * 2^-32 rounded
// to float -- curand's convention, which never returns 0.
__global__ void __launch_bounds__(256) uniform_fill_kernel(unsigned long long seed, unsigned long long call,
                                                           float* __restrict__ out, long long n) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    unsigned long long z = seed + 0x9E3779B97F4A7C15ULL * (call * 0x100000001B3ULL + (unsigned long long)i + 1ULL);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    z = z ^ (z >> 31);
    const unsigned bits = (unsigned)(z >> 32);
    float u = ((float)bits + 1.0f) * 2.3283064365386963e-10f;
    out[i] = u > 1.0f ? 1.0f : u;
  }
}

int row_sum_launch(zr_ctx* ctx, const float* a, int rows, long long n, float* out, int accumulate = 0) {
  const long long chunk = 64;
  const int chunks = (int)((n + chunk - 1) / chunk);
  void* scratch = nullptr;
  int rc = zr_ctx_scratch(ctx, 0, sizeof(float) * (size_t)chunks * rows, &scratch);
  if (rc) return rc;
  if (rows % 4 == 0 && aligned16(a) && aligned16(scratch)) {
    dim3 grid((rows / 4 + 63) / 64, chunks);
    row_sum_partial_wide_kernel<<<grid, 64, 0, ctx->stream>>>(a, rows, n, chunk, (float*)scratch);
  } else {
    dim3 grid((rows + 63) / 64, chunks);
    row_sum_partial_kernel<<<grid, 64, 0, ctx->stream>>>(a, rows, n, chunk, (float*)scratch);
  }
  ZR_LAUNCH_CHECK("row_sum_partial_kernel");
  row_sum_final_kernel<<<(rows + 63) / 64, 64, 0, ctx->stream>>>((const float*)scratch, rows, chunks, out,
                                                                           accumulate);
  ZR_LAUNCH_CHECK("row_sum_final_kernel");
  return ZR_OK;
}

int transpose_launch(zr_ctx* ctx, const float* src, int rows, int cols, float* dst, long long ldd, int row0) {
  if (rows % 4 == 0 && cols % 4 == 0 && ldd % 4 == 0 && row0 % 4 == 0 && aligned16(src) && aligned16(dst)) {
    dim3 grid((rows + 63) / 64, (cols + 63) / 64);
    transpose_wide_kernel<<<grid, 256, 0, ctx->stream>>>(src, rows, cols, dst, ldd, row0);
  } else {
    dim3 grid((rows + 31) / 32, (cols + 31) / 32);
    transpose_kernel<<<grid, 256, 0, ctx->stream>>>(src, rows, cols, dst, ldd, row0);
  }
  ZR_LAUNCH_CHECK("transpose_kernel");
  return ZR_OK;
}

}  // namespace

extern "C" {

int zr_lstm_train_create(zr_ctx* ctx, const float* const d_M[4], const float* const d_Wh[4], int H,
                         zr_lstm_train** out) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(out != nullptr, "zr_lstm_train_create: out is null");
  *out = nullptr;
  ZR_CHECK_ARG(H > 0 && d_M && d_Wh, "zr_lstm_train_create: H = %d or null pointer array", H);
  for (int g = 0; g < 4; ++g) ZR_CHECK_ARG(d_M[g] && d_Wh[g], "zr_lstm_train_create: null matrix for gate %d", g);
  zr_lstm_train* w = new zr_lstm_train();
  w->H = H;
  w->d_stack = nullptr;
  w->d_stack_pack = nullptr;
  w->ldp = (H + 31) / 32 * 32;
  w->kp = (4 * H + 7) / 8 * 8;
  const size_t per = 4 * (size_t)H * H;
  if (hipMalloc((void**)&w->d_stack, sizeof(float) * 2 * per) != hipSuccess ||
      hipMalloc((void**)&w->d_stack_pack, sizeof(float) * 2 * (size_t)w->kp * w->ldp) != hipSuccess) {
    (void)hipGetLastError();
    if (w->d_stack) (void)hipFree(w->d_stack);
    delete w;
    return zr_set_error(ZR_ENOMEM, "zr_lstm_train_create: allocation failed (H = %d)", H);
  }
  *out = w;
  return zr_lstm_train_refresh(ctx, w, d_M, d_Wh);
}

int zr_lstm_train_refresh(zr_ctx* ctx, zr_lstm_train* w, const float* const d_M[4], const float* const d_Wh[4]) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(w && d_M && d_Wh, "zr_lstm_train_refresh: null pointer");
  const int H = w->H;
  const size_t per = 4 * (size_t)H * H;
  dim3 grid((H + 31) / 32, (H + 31) / 32, 4);
  stack_gates_kernel<<<grid, 256, 0, ctx->stream>>>(d_Wh[0], d_Wh[1], d_Wh[2], d_Wh[3], H, w->d_stack);
  ZR_LAUNCH_CHECK("stack_gates_kernel");
  stack_gates_kernel<<<grid, 256, 0, ctx->stream>>>(d_M[0], d_M[1], d_M[2], d_M[3], H, w->d_stack + per);
  ZR_LAUNCH_CHECK("stack_gates_kernel");
  for (int z = 0; z < 2; ++z) {
    rc = zr_pack4_launch(ctx, w->d_stack + z * per, H, 4 * H, H, w->ldp, w->kp,
                         w->d_stack_pack + (size_t)z * w->kp * w->ldp);
    if (rc) return rc;
  }
  return ZR_OK;
}

int zr_lstm_train_destroy(zr_ctx* ctx, zr_lstm_train* w) {
  if (!w) return ZR_OK;
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  if (w->d_stack) (void)hipFree(w->d_stack);
  if (w->d_stack_pack) (void)hipFree(w->d_stack_pack);
  delete w;
  return ZR_OK;
}

int zr_unstack_gates(zr_ctx* ctx, const float* d_stack, int H, float* const d_out[4]) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(d_stack && d_out && H > 0, "zr_unstack_gates: null pointer or H = %d", H);
  for (int g = 0; g < 4; ++g) ZR_CHECK_ARG(d_out[g] != nullptr, "zr_unstack_gates: d_out[%d] is null", g);
  const size_t per = 4 * (size_t)H * H;
  unstack_gates_kernel<<<(unsigned)((per + 255) / 256), 256, 0, ctx->stream>>>(d_stack, H, d_out[0], d_out[1], d_out[2],
                                                                               d_out[3]);
  ZR_LAUNCH_CHECK("unstack_gates_kernel");
  return ZR_OK;
}

int zr_lstm_stack_backward(zr_ctx* ctx, int nl, const zr_lstm_train* const layers[], int T, int mb,
                           const int* d_mask01, const float* const d_c0[], const float* const d_c_all[],
                           const float* const d_gates_all[], const float* d_err_top, const float* const d_err_hT[],
                           const float* const d_err_cT[], float* const d_dgates_all[], float* d_err_below0,
                           float* const d_err_h0[], float* const d_err_c0[]) {
  return zr_lstm_stack_backward_clamped(ctx, nl, layers, T, mb, d_mask01, d_c0, d_c_all, d_gates_all, d_err_top, d_err_hT,
                                        d_err_cT, d_dgates_all, d_err_below0, d_err_h0, d_err_c0, 0.0f);
}

int zr_lstm_stack_backward_clamped(zr_ctx* ctx, int nl, const zr_lstm_train* const layers[], int T, int mb,
                                   const int* d_mask01, const float* const d_c0[], const float* const d_c_all[],
                                   const float* const d_gates_all[], const float* d_err_top,
                                   const float* const d_err_hT[], const float* const d_err_cT[],
                                   float* const d_dgates_all[], float* d_err_below0, float* const d_err_h0[],
                                   float* const d_err_c0[], float err_clip) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(nl > 0 && nl <= 16 && T > 0 && mb > 0, "zr_lstm_stack_backward: L = %d, T = %d, mb = %d", nl, T, mb);
  ZR_CHECK_ARG(mb <= 65535, "zr_lstm_stack_backward: mb = %d exceeds 65535", mb);
  ZR_CHECK_ARG(layers && d_mask01 && d_c0 && d_c_all && d_gates_all && d_err_top && d_dgates_all && d_err_h0 &&
                   d_err_c0,
               "zr_lstm_stack_backward: null pointer");
  const int H = layers[0] ? layers[0]->H : 0;
  for (int l = 0; l < nl; ++l) {
    ZR_CHECK_ARG(layers[l] && layers[l]->H == H, "zr_lstm_stack_backward: layer %d missing or of different size", l);
    ZR_CHECK_ARG(d_c0[l] && d_c_all[l] && d_gates_all[l] && d_dgates_all[l] && d_err_h0[l] && d_err_c0[l],
                 "zr_lstm_stack_backward: null buffer for layer %d", l);
  }
  const size_t n = (size_t)H * mb;
  // The grid is walked by anti-diagonals d = l + t, highest first: node (l, t) needs the errors of (l+1, t) and
  // (l, t+1), both on diagonal d+1, so the nodes of a diagonal are independent and share two launches (the gate
  // derivatives of all of them, then all their error products as one grouped GEMM).
  // work: two sets (diagonal parity) of per-layer [2][H x mb] = (error to h_{t-1}, error to the layer below): a
  // node reads what diagonal d+1 wrote into the other set while its neighbours on diagonal d write this one.  The
  // cell error lives in d_err_c0[l] (updated in place step by step; one node per layer and diagonal touches it).
  const bool packed_ok = (H % 4 == 0) && layers[0]->d_stack_pack != nullptr;
  const bool bpack = packed_ok && (H % 2 == 0);  // K = 4H must be a multiple of 8
  void* scratch = nullptr;
  rc = zr_ctx_scratch(ctx, 1, sizeof(float) * (4 * n * nl + (bpack ? 8 * 4 * n : 0)), &scratch);
  if (rc) return rc;
  float* work = (float*)scratch;
  float* dgp_buf = work + 4 * n * nl;  // k-interleaved copies of the gate errors of the diagonal in flight
  auto wk = [&](int d, int l) { return work + ((size_t)(d & 1) * nl + l) * 2 * n; };
  for (int l = 0; l < nl; ++l) {
    // node (l, T-1) is on diagonal l + T - 1 and reads its "next step" error from the set of diagonal l + T
    float* first = wk(l + T, l);
    if (d_err_hT && d_err_hT[l])
      ZR_HIP(hipMemcpyAsync(first, d_err_hT[l], sizeof(float) * n, hipMemcpyDeviceToDevice, ctx->stream));
    else {
      rc = zr_memset_zero(ctx, first, sizeof(float) * n);
      if (rc) return rc;
    }
    if (d_err_cT && d_err_cT[l])
      ZR_HIP(hipMemcpyAsync(d_err_c0[l], d_err_cT[l], sizeof(float) * n, hipMemcpyDeviceToDevice, ctx->stream));
    else {
      rc = zr_memset_zero(ctx, d_err_c0[l], sizeof(float) * n);
      if (rc) return rc;
    }
  }
  for (int d = nl + T - 2; d >= 0; --d) {
    for (int lhi = nl - 1; lhi >= 0; lhi -= 8) {  // at most 8 nodes per launch
      NodeBackwardGroup G = {};
      ZrGemmDesc g = {};
      int nu = 0;
      for (int l = lhi; l >= 0 && l > lhi - 8; --l) {
        const int t = d - l;
        if (t < 0 || t >= T) continue;
        float* w_l = wk(d, l);
        G.gates[nu] = d_gates_all[l] + (size_t)t * 4 * n;
        G.c[nu] = d_c_all[l] + (size_t)t * n;
        G.cprev[nu] = (t == 0) ? d_c0[l] : d_c_all[l] + (size_t)(t - 1) * n;
        G.mask01[nu] = d_mask01 + (size_t)t * mb;
        G.err_above[nu] = (l == nl - 1) ? d_err_top + (size_t)t * n : wk(d + 1, l + 1) + n;
        G.clamp_above[nu] = (l == nl - 1) ? 0 : 1;
        G.err_next[nu] = wk(d + 1, l);
        G.ec[nu] = d_err_c0[l];
        G.dg[nu] = d_dgates_all[l] + (size_t)t * 4 * n;
        G.dgp[nu] = bpack ? dgp_buf + (size_t)nu * 4 * n : nullptr;
        g.gA[nu] = packed_ok ? layers[l]->d_stack_pack : layers[l]->d_stack;
        g.gB[nu] = bpack ? G.dgp[nu] : G.dg[nu];
        g.gC[nu] = w_l;
        ++nu;
      }
      if (nu == 0) continue;
      dim3 egrid((H + 255) / 256, mb, nu);
      lstm_node_backward_group_kernel<<<egrid, 256, 0, ctx->stream>>>(G, H, mb, err_clip);
      ZR_LAUNCH_CHECK("lstm_node_backward_group_kernel");
      // (error to h_{t-1}, error to below) = (Wh_stack^T, M_stack^T) * dg for every node: batch of 2 inside a group
      g.groups = nu;
      g.M = H;
      g.N = mb;
      g.nseg = 1;
      g.K[0] = 4 * H;
      g.ldb[0] = 4 * H;
      g.ldc = H;
      g.batch = 2;
      g.strideC = (long long)n;
      g.epilogue = ZR_EPI_STORE;
      if (packed_ok) {
        g.a_pack = 1;
        g.b_packed = bpack ? 1 : 0;
        g.lda[0] = layers[0]->ldp;
        g.strideA = (long long)layers[0]->kp * layers[0]->ldp;
      } else {
        g.lda[0] = H;
        g.strideA = 4LL * H * H;
      }
      rc = zr_gemm_launch(ctx, g);
      if (rc) return rc;
    }
    const int t0 = d;  // layer 0's node on this diagonal
    if (d_err_below0 && t0 < T)
      ZR_HIP(hipMemcpyAsync(d_err_below0 + (size_t)t0 * n, wk(d, 0) + n, sizeof(float) * n, hipMemcpyDeviceToDevice,
                            ctx->stream));
  }
  // node (l, 0) is on diagonal l
  for (int l = 0; l < nl; ++l) {
    ZR_HIP(hipMemcpyAsync(d_err_h0[l], wk(l, l), sizeof(float) * n, hipMemcpyDeviceToDevice, ctx->stream));
    if (err_clip > 0.0f) {  // node (l, 0)'s error to its initial state is an error to h_{t-1} like any other
      rc = zr_clip_inplace(ctx, d_err_h0[l], (long long)n, err_clip);
      if (rc) return rc;
    }
  }
  return ZR_OK;
}

static int weight_gradients(zr_ctx* ctx, int H, int T, int mb, const float* d_dgates, const float* d_in_all,
                            const float* d_h0, const float* d_h_all, float* d_dM_stack, float* d_dWh_stack,
                            float* d_db, int accumulate) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(H > 0 && T > 0 && mb > 0, "zr_lstm_weight_gradients: H = %d, T = %d, mb = %d", H, T, mb);
  ZR_CHECK_ARG(d_dgates && d_in_all && d_h0 && (d_h_all || T == 1) && d_dM_stack && d_dWh_stack && d_db,
               "zr_lstm_weight_gradients: null pointer");
  const long long K = (long long)T * mb;
  ZR_CHECK_ARG(K < (1LL << 31) / 4, "zr_lstm_weight_gradients: T * mb = %lld too large", K);
  void* scratch = nullptr;
  rc = zr_ctx_scratch(ctx, 0, sizeof(float) * (size_t)K * H, &scratch);  // the transposed right-hand side, K x H
  if (rc) return rc;
  float* xt = (float*)scratch;
  ZrGemmDesc g = {};
  g.M = 4 * H;
  g.N = H;
  g.nseg = 1;
  g.K[0] = (int)K;
  g.A[0] = d_dgates;
  g.lda[0] = 4 * H;
  g.B[0] = xt;
  g.ldb[0] = (int)K;
  g.ldc = 4 * H;
  g.batch = 1;
  g.epilogue = ZR_EPI_STORE;
  g.accumulate = accumulate;
  // dM = dgates * in^T
  rc = transpose_launch(ctx, d_in_all, H, (int)K, xt, K, 0);
  if (rc) return rc;
  g.C = d_dM_stack;
  rc = zr_gemm_launch(ctx, g);
  if (rc) return rc;
  // dWh = dgates * [h0, h_1 .. h_{T-1}]^T
  rc = transpose_launch(ctx, d_h0, H, mb, xt, K, 0);
  if (rc) return rc;
  if (T > 1) {
    rc = transpose_launch(ctx, d_h_all, H, (int)(K - mb), xt, K, mb);
    if (rc) return rc;
  }
  g.C = d_dWh_stack;
  rc = zr_gemm_launch(ctx, g);
  if (rc) return rc;
  return row_sum_launch(ctx, d_dgates, 4 * H, K, d_db, accumulate);
}

int zr_lstm_weight_gradients(zr_ctx* ctx, int H, int T, int mb, const float* d_dgates, const float* d_in_all,
                             const float* d_h0, const float* d_h_all, float* d_dM_stack, float* d_dWh_stack,
                             float* d_db) {
  return weight_gradients(ctx, H, T, mb, d_dgates, d_in_all, d_h0, d_h_all, d_dM_stack, d_dWh_stack, d_db, 0);
}

int zr_lstm_node_gradients(zr_ctx* ctx, int H, int mb, const float* d_dgates, const float* d_in, const float* d_h_prev,
                           float* d_dM_stack, float* d_dWh_stack, float* d_db) {
  return weight_gradients(ctx, H, 1, mb, d_dgates, d_in, d_h_prev, nullptr, d_dM_stack, d_dWh_stack, d_db, 1);
}

int zr_lstm_node_backward(zr_ctx* ctx, const zr_lstm_train* layer, int mb, const float* const d_gates[4],
                          const float* d_c, const float* d_c_prev, const int* d_mask01, const float* d_err_above,
                          const float* d_err_h_next, const float* d_err_c_next, float* d_dgates, float* d_err_h_prev,
                          float* d_err_c_prev, float* d_err_below) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(layer && mb > 0 && mb <= 65535, "zr_lstm_node_backward: null layer or mb = %d", mb);
  ZR_CHECK_ARG(d_gates && d_gates[0] && d_gates[1] && d_gates[2] && d_gates[3] && d_c && d_c_prev && d_mask01 &&
                   d_dgates && d_err_h_prev && d_err_c_prev,
               "zr_lstm_node_backward: null pointer");
  const int H = layer->H;
  const size_t n = (size_t)H * mb;
  dim3 egrid((H + 255) / 256, mb);
  lstm_node_backward_kernel<<<egrid, 256, 0, ctx->stream>>>(d_gates[0], d_gates[1], d_gates[2], d_gates[3], d_c,
                                                            d_c_prev, d_mask01, d_err_above, d_err_h_next,
                                                            d_err_c_next, d_err_c_prev, H, mb, d_dgates);
  ZR_LAUNCH_CHECK("lstm_node_backward_kernel");
  // the two error products share their right-hand side: one batched launch when the outputs are adjacent
  // (d_err_below == d_err_h_prev + H*mb), else through a scratch pair and two copies
  float* out = d_err_h_prev;
  const bool adjacent = d_err_below == d_err_h_prev + n;
  if (!adjacent) {
    void* scratch = nullptr;
    rc = zr_ctx_scratch(ctx, 1, sizeof(float) * 2 * n, &scratch);
    if (rc) return rc;
    out = (float*)scratch;
  }
  ZrGemmDesc g = {};
  g.M = H;
  g.N = mb;
  g.nseg = 1;
  g.K[0] = 4 * H;
  g.A[0] = layer->d_stack;
  g.lda[0] = H;
  g.B[0] = d_dgates;
  g.ldb[0] = 4 * H;
  g.C = out;
  g.ldc = H;
  g.batch = d_err_below ? 2 : 1;
  g.strideA = 4LL * H * H;
  g.strideC = (long long)n;
  g.epilogue = ZR_EPI_STORE;
  rc = zr_gemm_launch(ctx, g);
  if (rc) return rc;
  if (!adjacent) {
    ZR_HIP(hipMemcpyAsync(d_err_h_prev, out, sizeof(float) * n, hipMemcpyDeviceToDevice, ctx->stream));
    if (d_err_below)
      ZR_HIP(hipMemcpyAsync(d_err_below, out + n, sizeof(float) * n, hipMemcpyDeviceToDevice, ctx->stream));
  }
  return ZR_OK;
}

int zr_attn_set_error_tables(zr_ctx* ctx, zr_attn* a, float* const* h_err_tables, int n) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(a && h_err_tables, "zr_attn_set_error_tables: null pointer");
  ZR_CHECK_ARG(n == a->longest_sent, "zr_attn_set_error_tables: %d tables, the layer has %d source positions", n,
               a->longest_sent);
  for (int t = 0; t < n; ++t) ZR_CHECK_ARG(h_err_tables[t] != nullptr, "zr_attn_set_error_tables: entry %d is null", t);
  if (!a->d_err_table) {
    if (hipMalloc((void**)&a->d_err_table, sizeof(float*) * n) != hipSuccess) {
      (void)hipGetLastError();
      a->d_err_table = nullptr;
      return zr_set_error(ZR_ENOMEM, "zr_attn_set_error_tables: allocation failed");
    }
  }
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  ZR_HIP(hipMemcpy((void*)a->d_err_table, h_err_tables, sizeof(float*) * n, hipMemcpyHostToDevice));
  return ZR_OK;
}

int zr_attn_backward(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const float* d_h_t, const int* d_mask01,
                     const float* d_h_tild, const float* d_alignments, const int* d_indices, const float* d_p_t,
                     const float* d_c_t, const float* d_err_htild, float* d_err_h_t, const zr_attn_grads* grads) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(a != nullptr, "zr_attn_backward: attention object is null");
  ZR_CHECK_ARG(a->d_err_table != nullptr, "zr_attn_backward: call zr_attn_set_error_tables first");
  ZR_CHECK_ARG(d_batch_info && d_h_t && d_mask01 && d_h_tild && d_alignments && d_indices && d_p_t && d_c_t &&
                   d_err_htild && d_err_h_t && grads,
               "zr_attn_backward: null pointer");
  ZR_CHECK_ARG(grads->d_W_a && grads->d_W_p && grads->d_v_p && grads->d_out_bias && grads->d_W_c1 && grads->d_W_c2,
               "zr_attn_backward: null gradient array");
  ZR_CHECK_ARG(a->D >= 1, "zr_attn_backward: D = %d (the Gaussian's width D/2 must be positive)", a->D);
  const int H = a->H, mb = a->mb, W = 2 * a->D + 1;
  const size_t n = (size_t)H * mb;
  const float sigma_sq = (float)((a->D * a->D) / 4.0);  // src/attention_node.hpp:50
  void* scratch = nullptr;
  rc = zr_ctx_scratch(ctx, 1, sizeof(float) * (6 * n + 2 * (size_t)W * mb + 3 * (size_t)mb), &scratch);
  if (rc) return rc;
  float* e = (float*)scratch;
  float* err_ct = e + n;
  float* tv = e + 2 * n;
  float* tw = e + 3 * n;
  float* hs_sum = e + 4 * n;
  float* tr = e + 5 * n;  // a transposed right-hand side, mb x H
  float* err_as = e + 6 * n;
  float* scal = err_as + (size_t)W * mb;
  float* col = scal + (size_t)W * mb;
  const int eg = (int)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);

  // C (H x H) += A (H x mb) * B^T for B H x mb (cuBLAS gemm N, T with beta = 1 in the reference)
  auto outer_acc = [&](const float* A, const float* B, float* C) -> int {
    int r = transpose_launch(ctx, B, H, mb, tr, mb, 0);
    if (r) return r;
    ZrGemmDesc g = {};
    g.M = H;
    g.N = H;
    g.nseg = 1;
    g.K[0] = mb;
    g.A[0] = A;
    g.lda[0] = H;
    g.B[0] = tr;
    g.ldb[0] = mb;
    g.C = C;
    g.ldc = H;
    g.batch = 1;
    g.epilogue = ZR_EPI_STORE;
    g.accumulate = 1;
    return zr_gemm_launch(ctx, g);
  };
  // C (H x mb) (+)= op(A) (H x H) * B (H x mb)
  auto product = [&](const float* A, int trans, const float* B, float* C, int accumulate, int epilogue) -> int {
    ZrGemmDesc g = {};
    g.M = H;
    g.N = mb;
    g.nseg = 1;
    g.K[0] = H;
    g.A[0] = A;
    g.lda[0] = H;
    g.trans_a = trans;
    g.B[0] = B;
    g.ldb[0] = H;
    g.C = C;
    g.ldc = H;
    g.batch = 1;
    g.epilogue = epilogue;
    g.accumulate = accumulate;
    return zr_gemm_launch(ctx, g);
  };

  attn_bwd_e_kernel<<<eg, 256, 0, ctx->stream>>>(d_err_htild, d_h_tild, d_mask01, H, (long long)n, e);
  ZR_LAUNCH_CHECK("attn_bwd_e_kernel");
  if ((rc = outer_acc(e, d_c_t, grads->d_W_c1))) return rc;                     // :437
  if ((rc = outer_acc(e, d_h_t, grads->d_W_c2))) return rc;                     // :443
  if ((rc = row_sum_launch(ctx, e, H, mb, grads->d_out_bias, 1))) return rc;    // :456
  if ((rc = product(a->W_c1, 1, e, err_ct, 0, ZR_EPI_STORE))) return rc;        // :464
  if ((rc = product(a->W_c2, 1, e, d_err_h_t, 0, ZR_EPI_STORE))) return rc;     // :476
  attn_bwd_align_kernel<<<dim3(W, mb), 256, 0, ctx->stream>>>(err_ct, a->d_table, a->d_err_table, d_batch_info, d_indices,
                                                              d_alignments, H, mb, W, a->longest_sent, err_as);
  ZR_LAUNCH_CHECK("attn_bwd_align_kernel");
  if ((rc = product(a->W_p, 0, d_h_t, a->d_tanh1, 0, ZR_EPI_TANH))) return rc;  // tanh_1 of the forward pass again
  attn_bwd_column_kernel<<<mb, 64, 0, ctx->stream>>>(a->d_tanh1, a->v_p, d_batch_info, d_indices, d_alignments, d_p_t,
                                                     err_as, H, mb, W, sigma_sq, col, scal);
  ZR_LAUNCH_CHECK("attn_bwd_column_kernel");
  attn_bwd_vp_wp_kernel<<<eg, 256, 0, ctx->stream>>>(a->d_tanh1, a->v_p, col, H, mb, (long long)n, tv, tw);
  ZR_LAUNCH_CHECK("attn_bwd_vp_wp_kernel");
  if ((rc = row_sum_launch(ctx, tv, H, mb, grads->d_v_p, 1))) return rc;        // :536
  if ((rc = outer_acc(tw, d_h_t, grads->d_W_p))) return rc;                     // :545
  if ((rc = product(a->W_p, 1, tw, d_err_h_t, 1, ZR_EPI_STORE))) return rc;     // :551
  if ((rc = product(a->W_a, 1, d_h_t, a->d_q, 0, ZR_EPI_STORE))) return rc;     // W_a^T h of the forward pass again
  attn_bwd_hs_kernel<<<mb, 256, 0, ctx->stream>>>(a->d_q, a->d_table, a->d_err_table, d_batch_info, d_indices, scal, H, mb,
                                                  W, a->longest_sent, hs_sum);
  ZR_LAUNCH_CHECK("attn_bwd_hs_kernel");
  if ((rc = outer_acc(d_h_t, hs_sum, grads->d_W_a))) return rc;                 // :632
  return product(a->W_a, 0, hs_sum, d_err_h_t, 1, ZR_EPI_STORE);                // :636
}

int zr_dropout_apply(zr_ctx* ctx, const float* d_uniform, float keep_rate, float* d_x, long long n) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(d_uniform && d_x && n >= 0, "zr_dropout_apply: null pointer or n = %lld", n);
  ZR_CHECK_ARG(keep_rate > 0.0f && keep_rate <= 1.0f, "zr_dropout_apply: keep rate %g not in (0, 1]", (double)keep_rate);
  if (n == 0) return ZR_OK;
  const int grid = (int)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
  dropout_kernel<<<grid, 256, 0, ctx->stream>>>(d_uniform, keep_rate, d_x, n);
  ZR_LAUNCH_CHECK("dropout_kernel");
  return ZR_OK;
}

int zr_uniform_fill(zr_ctx* ctx, unsigned long long seed, unsigned long long call, float* d_out, long long n) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(d_out && n >= 0, "zr_uniform_fill: null pointer or n = %lld", n);
  if (n == 0) return ZR_OK;
  const int grid = (int)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
  uniform_fill_kernel<<<grid, 256, 0, ctx->stream>>>(seed, call, d_out, n);
  ZR_LAUNCH_CHECK("uniform_fill_kernel");
  return ZR_OK;
}

int zr_lstm_feed_backward(zr_ctx* ctx, const float* const d_Q[4], int H, int mb, const float* d_dgates,
                          const float* d_htild, float* d_err_htild, float* d_dQ_stack) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(H > 0 && mb > 0, "zr_lstm_feed_backward: H = %d, mb = %d", H, mb);
  ZR_CHECK_ARG(d_Q && d_dgates && d_htild && d_err_htild && d_dQ_stack, "zr_lstm_feed_backward: null pointer");
  for (int g = 0; g < 4; ++g) ZR_CHECK_ARG(d_Q[g] != nullptr, "zr_lstm_feed_backward: Q matrix %d is null", g);
  // error of h~ = sum_g Q_g^T d_g (src/LSTM.hpp:804-857: four products and add_four_matrices_kernel)
  for (int half = 0; half < 2; ++half) {
    ZrGemmDesc g = {};
    g.M = H;
    g.N = mb;
    g.nseg = 2;
    for (int s = 0; s < 2; ++s) {
      const int gate = 2 * half + s;
      g.K[s] = H;
      g.A[s] = d_Q[gate];
      g.lda[s] = H;
      g.B[s] = d_dgates + (size_t)gate * H;
      g.ldb[s] = 4 * H;
    }
    g.trans_a = 1;
    g.C = d_err_htild;
    g.ldc = H;
    g.batch = 1;
    g.epilogue = ZR_EPI_STORE;
    g.accumulate = half;
    rc = zr_gemm_launch(ctx, g);
    if (rc) return rc;
  }
  // Q gradients, stacked over the gates like the M and W_h gradients: dQ (4H x H) += dgates (4H x mb) * h~^T
  // (src/LSTM.hpp:1014-1050)
  void* scratch = nullptr;
  rc = zr_ctx_scratch(ctx, 1, sizeof(float) * (size_t)H * mb, &scratch);
  if (rc) return rc;
  float* tr = (float*)scratch;
  rc = transpose_launch(ctx, d_htild, H, mb, tr, mb, 0);
  if (rc) return rc;
  ZrGemmDesc w = {};
  w.M = 4 * H;
  w.N = H;
  w.nseg = 1;
  w.K[0] = mb;
  w.A[0] = d_dgates;
  w.lda[0] = 4 * H;
  w.B[0] = tr;
  w.ldb[0] = mb;
  w.C = d_dQ_stack;
  w.ldc = 4 * H;
  w.batch = 1;
  w.epilogue = ZR_EPI_STORE;
  w.accumulate = 1;
  return zr_gemm_launch(ctx, w);
}

int zr_embed_gradient(zr_ctx* ctx, int H, int V, const float* d_err, const int* d_ids_nonneg, const int* d_mask01,
                      int n, float* d_dW) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(H > 0 && V > 0 && n >= 0 && n <= 65535 * 64, "zr_embed_gradient: H = %d, V = %d, n = %d", H, V, n);
  if (n == 0) return ZR_OK;
  ZR_CHECK_ARG(d_err && d_ids_nonneg && d_mask01 && d_dW, "zr_embed_gradient: null pointer");
  for (int base = 0; base < n; base += 65535) {
    const int cnt = n - base < 65535 ? n - base : 65535;
    dim3 grid((H + 255) / 256, cnt);
    embed_grad_kernel<<<grid, 256, 0, ctx->stream>>>(d_err + (size_t)base * H, d_ids_nonneg + base, d_mask01 + base, H, V,
                                                     d_dW);
    ZR_LAUNCH_CHECK("embed_grad_kernel");
  }
  return ZR_OK;
}

static int softmax_backward(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int n,
                            const int* d_target, const int* d_mask01, float* d_prob_scratch, float* d_err_h,
                            float* d_dD, float* d_db, int accumulate, double* h_loss = nullptr) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(V > 0 && H > 0 && n > 0 && n <= 65535, "zr_softmax_backward: V = %d, H = %d, n = %d", V, H, n);
  ZR_CHECK_ARG(d_D && d_b_d && d_h && d_target && d_mask01 && d_prob_scratch && d_err_h && d_dD && d_db,
               "zr_softmax_backward: null pointer");
  rc = zr_softmax_forward(ctx, d_D, d_b_d, V, H, d_h, n, ZR_SOFTMAX_PROB, d_prob_scratch, nullptr);
  if (rc) return rc;
  // err_h = D^T e, computed as (e^T D)^T: with e^T as the left operand the product is tall (n rows) with contiguous
  // rows, the shape the large-matrix kernels are built for; the two transposes move 2 x V*n + 2 x n*H floats.
  void *s0 = nullptr, *s1 = nullptr;
  rc = zr_ctx_scratch(ctx, 1, sizeof(float) * (size_t)V * n, &s1);
  if (rc) return rc;
  rc = zr_ctx_scratch(ctx, 0, sizeof(float) * (size_t)n * H + sizeof(double), &s0);
  if (rc) return rc;
  if (h_loss) {
    // before the probabilities are turned into errors.  The cell is the head of scratch 0; the copy out is queued
    // ahead of the kernels that reuse that buffer, and waited for at the end of this call.
    train_logprob_kernel<<<1, 256, 0, ctx->stream>>>(d_prob_scratch, V, n, d_target, d_mask01, (double*)s0);
    ZR_LAUNCH_CHECK("train_logprob_kernel");
    ZR_HIP(hipMemcpyAsync(h_loss, s0, sizeof(double), hipMemcpyDeviceToHost, ctx->stream));
  }
  if (V % 4 == 0 && aligned16(d_prob_scratch)) {
    dim3 egrid((V / 4 + 255) / 256, n);
    softmax_error_kernel<true><<<egrid, 256, 0, ctx->stream>>>(d_prob_scratch, V, d_target, d_mask01);
  } else {
    dim3 egrid((V + 255) / 256, n);
    softmax_error_kernel<false><<<egrid, 256, 0, ctx->stream>>>(d_prob_scratch, V, d_target, d_mask01);
  }
  ZR_LAUNCH_CHECK("softmax_error_kernel");
  float* et = (float*)s1;   // n x V
  float* ct = (float*)s0;   // n x H
  ZrGemmDesc g = {};
  g.nseg = 1;
  g.K[0] = V;
  g.batch = 1;
  g.epilogue = ZR_EPI_STORE;
  if (n >= 1024) {
    rc = transpose_launch(ctx, d_prob_scratch, V, n, et, n, 0);
    if (rc) return rc;
    g.M = n;
    g.N = H;
    g.A[0] = et;
    g.lda[0] = n;
    g.B[0] = d_D;
    g.ldb[0] = V;
    g.C = ct;
    g.ldc = n;
    rc = zr_gemm_launch(ctx, g);
    if (rc) return rc;
    rc = transpose_launch(ctx, ct, n, H, d_err_h, H, 0);
    if (rc) return rc;
  } else {  // few columns (one time step): D^T e directly
    g.M = H;
    g.N = n;
    g.trans_a = 1;
    g.A[0] = d_D;
    g.lda[0] = V;
    g.B[0] = d_prob_scratch;
    g.ldb[0] = V;
    g.C = d_err_h;
    g.ldc = H;
    rc = zr_gemm_launch(ctx, g);
    if (rc) return rc;
  }
  // dD = e h^T : right-hand side h^T as an n x H column-major matrix
  float* ht = (float*)s0;  // the product above has been queued: the buffer is free again in stream order
  rc = transpose_launch(ctx, d_h, H, n, ht, n, 0);
  if (rc) return rc;
  ZrGemmDesc w = {};
  w.M = V;
  w.N = H;
  w.nseg = 1;
  w.K[0] = n;
  w.A[0] = d_prob_scratch;
  w.lda[0] = V;
  w.B[0] = ht;
  w.ldb[0] = n;
  w.C = d_dD;
  w.ldc = V;
  w.batch = 1;
  w.epilogue = ZR_EPI_STORE;
  w.accumulate = accumulate;
  rc = zr_gemm_launch(ctx, w);
  if (rc) return rc;
  rc = row_sum_launch(ctx, d_prob_scratch, V, n, d_db, accumulate);
  if (rc) return rc;
  if (h_loss) ZR_HIP(hipStreamSynchronize(ctx->stream));
  return ZR_OK;
}

int zr_softmax_backward(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int n,
                        const int* d_target, const int* d_mask01, float* d_prob_scratch, float* d_err_h, float* d_dD,
                        float* d_db) {
  return softmax_backward(ctx, d_D, d_b_d, V, H, d_h, n, d_target, d_mask01, d_prob_scratch, d_err_h, d_dD, d_db, 0);
}

int zr_softmax_backward_loss(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int n,
                             const int* d_target, const int* d_mask01, float* d_prob_scratch, float* d_err_h,
                             float* d_dD, float* d_db, double* h_loss) {
  ZR_CHECK_ARG(h_loss != nullptr, "zr_softmax_backward_loss: h_loss is null");
  return softmax_backward(ctx, d_D, d_b_d, V, H, d_h, n, d_target, d_mask01, d_prob_scratch, d_err_h, d_dD, d_db, 0,
                          h_loss);
}

int zr_softmax_backward_accumulate(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h,
                                   int n, const int* d_target, const int* d_mask01, float* d_prob_scratch,
                                   float* d_err_h, float* d_dD, float* d_db) {
  return softmax_backward(ctx, d_D, d_b_d, V, H, d_h, n, d_target, d_mask01, d_prob_scratch, d_err_h, d_dD, d_db, 1);
}

int zr_grad_sumsq_accumulate(zr_ctx* ctx, const float* d_grad, long long n, float scale, double* d_sumsq, int reset) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n >= 0 && d_sumsq && (n == 0 || d_grad), "zr_grad_sumsq_accumulate: null pointer or n = %lld", n);
  const int n_partial = n > 0 ? 256 : 0;
  void* scratch = nullptr;
  rc = zr_ctx_scratch(ctx, 1, sizeof(double) * 256, &scratch);
  if (rc) return rc;
  if (n > 0) {
    sumsq_partial_kernel<<<n_partial, 1024, 0, ctx->stream>>>(d_grad, n, aligned16(d_grad) ? 1 : 0, (double*)scratch);
    ZR_LAUNCH_CHECK("sumsq_partial_kernel");
  }
  sumsq_accumulate_kernel<<<1, 64, 0, ctx->stream>>>((const double*)scratch, n_partial, scale, d_sumsq, reset ? 1 : 0);
  ZR_LAUNCH_CHECK("sumsq_accumulate_kernel");
  return ZR_OK;
}

int zr_sgd_update_clipped(zr_ctx* ctx, float* d_W, const float* d_grad, long long n, float scale, int clip_mode,
                          float threshold, const double* d_sumsq, float learning_rate) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n >= 0 && (n == 0 || (d_W && d_grad)), "zr_sgd_update_clipped: null pointer or n = %lld", n);
  ZR_CHECK_ARG(clip_mode >= ZR_CLIP_NONE && clip_mode <= ZR_CLIP_ELEMENT, "zr_sgd_update_clipped: clip_mode = %d",
               clip_mode);
  ZR_CHECK_ARG(clip_mode == ZR_CLIP_NONE || threshold > 0.0f, "zr_sgd_update_clipped: threshold = %g", (double)threshold);
  ZR_CHECK_ARG(clip_mode != ZR_CLIP_WHOLE_NORM || d_sumsq, "zr_sgd_update_clipped: whole-model clipping without d_sumsq");
  if (n == 0) return ZR_OK;
  const int n_partial = 256;
  void* scratch = nullptr;
  rc = zr_ctx_scratch(ctx, 1, sizeof(double) * n_partial, &scratch);
  if (rc) return rc;
  if (clip_mode == ZR_CLIP_MATRIX_NORM) {
    sumsq_partial_kernel<<<n_partial, 1024, 0, ctx->stream>>>(d_grad, n, aligned16(d_grad) ? 1 : 0, (double*)scratch);
    ZR_LAUNCH_CHECK("sumsq_partial_kernel");
  }
  const long long blocks = (n + 255) / 256;
  sgd_apply_kernel<<<(unsigned)(blocks < 2048 ? blocks : 2048), 256, 0, ctx->stream>>>(
      d_W, d_grad, n, scale, clip_mode, threshold, learning_rate, (const double*)scratch, n_partial, d_sumsq);
  ZR_LAUNCH_CHECK("sgd_apply_kernel");
  return ZR_OK;
}

int zr_sgd_update(zr_ctx* ctx, float* d_W, const float* d_grad, long long n, float scale, float norm_clip,
                  float learning_rate) {
  return zr_sgd_update_clipped(ctx, d_W, d_grad, n, scale, norm_clip > 0.0f ? ZR_CLIP_MATRIX_NORM : ZR_CLIP_NONE,
                               norm_clip, nullptr, learning_rate);
}

}  // extern "C"
