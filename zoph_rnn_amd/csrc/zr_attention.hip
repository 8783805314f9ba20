// Luong local-p attention with the "general" score and feed-input output, forward only
// (reference: attention_node::forward_prop, src/attention_node.hpp:73-394).
//
// The reference materialises the (2D+1) x H x mb window of source states (load_in_hs_kernel) and reads it
// twice.  Here the score and context kernels read the source states in place through the pointer table, so
// the only traffic is the valid source columns themselves, once for the scores and once for the context.
#include <math.h>

#include "zr_internal.h"

struct zr_attn {
  int H, mb, D, longest_sent;
  bool tables_aligned;  // every source table is 16-byte aligned
  const float *W_a, *W_p, *v_p, *out_bias, *W_c1, *W_c2;  // borrowed device pointers
  const float** d_table;                                   // device copy of the pointer table
  float *d_tanh1, *d_q, *d_align, *d_pt, *d_ctx;
  int* d_idx;
  // zr_attn_use_bf16_weights: owned bf16 k-interleaved snapshots of W_p, W_a^T, W_c1, W_c2 ([H/8][ldp][8] each)
  unsigned short* d_bf16;
  int ldp;
};

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// p_t and the window.  sigmoid_kernel (double), alignment_pos_kernel, lower_upper_kernel and
// create_indicies_kernel of the reference (src/custom_kernels.h:1583-1673) for one column per wave.
__global__ void __launch_bounds__(64)
attn_window_kernel(const float* __restrict__ tanh1, const float* __restrict__ v_p, const int* __restrict__ batch_info,
                   const int* __restrict__ mask01, int H, int mb, int D, float* __restrict__ p_t,
                   int* __restrict__ indices) {
  const int b = blockIdx.x;
  const int lane = threadIdx.x;
  float s = 0.0f;
  for (int k = lane; k < H; k += 64) s += v_p[k] * tanh1[(size_t)b * H + k];
  s = wave_sum(s);
  const float sig = (float)(1.0 / (1.0 + exp(-1.0 * (double)s)));
  const int len = batch_info[b];
  const float p = (float)len * sig;
  const int ip = (int)p;
  const int lo = (0 > ip - D) ? 0 : (ip - D);
  const int hi = ((len - 1) < ip + D) ? (len - 1) : (ip + D);
  if (lane == 0) p_t[b] = p;
  const bool live = mask01[b] == 1;
  for (int j = lane; j < 2 * D + 1; j += 64) indices[b + (size_t)mb * j] = (live && lo + j <= hi) ? lo + j : -1;
}

// score[b + mb*j] = h_s . q[:,b] for the source state the slot points at (elem_reduce_kernel_large over the
// gathered column, src/custom_kernels.h:1892-1925; 0 for an empty slot).  One wave per (b, j).
template <bool VEC>
__global__ void __launch_bounds__(256)
attn_score_kernel(const float* const* __restrict__ table, int longest_sent, const float* __restrict__ q,
                  const int* __restrict__ indices, const int* __restrict__ batch_info, int H, int mb, int W,
                  float* __restrict__ align, int* __restrict__ flags) {
  const int lane = threadIdx.x & 63;
  const long long slot = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (slot >= (long long)mb * W) return;
  const int b = (int)(slot % mb);
  const int s_idx = indices[slot];
  float acc = 0.0f;
  if (s_idx != -1) {
    int t = batch_info[b] - 1 - s_idx + batch_info[mb + b];
    if (t < 0 || t >= longest_sent) {
      if (lane == 0) atomicAdd(&flags[1], 1);
      t = t < 0 ? 0 : longest_sent - 1;
    }
    const float* hs = table[t] + (size_t)b * H;
    const float* qc = q + (size_t)b * H;
    if (VEC) {
      for (int k4 = lane; k4 * 4 < H; k4 += 64) {
        const zr_f32x4 a = ((const zr_f32x4*)hs)[k4];
        const zr_f32x4 c = ((const zr_f32x4*)qc)[k4];
        acc += a.x * c.x + a.y * c.y + a.z * c.z + a.w * c.w;
      }
    } else {
      for (int k = lane; k < H; k += 64) acc += hs[k] * qc[k];
    }
    acc = wave_sum(acc);
  }
  if (lane == 0) align[slot] = acc;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// alignment_reduction_kernel (src/custom_kernels.h:1752-1794): the reference runs one thread per column; here
// one wave per column with the window slots spread over the lanes.  The max starts at 0 as in the reference.
__global__ void __launch_bounds__(64)
attn_align_kernel(float* __restrict__ align, const int* __restrict__ indices, const float* __restrict__ p_t, int mb,
                  int W, float sigma_sq) {
  const int b = blockIdx.x;
  const int lane = threadIdx.x;
  float max_val = 0.0f;
  for (int j = lane; j < W; j += 64)
    if (indices[b + (size_t)mb * j] != -1) max_val = fmaxf(max_val, align[b + (size_t)mb * j]);
  max_val = wave_max(max_val);
  float sum = 0.0f;
  for (int j = lane; j < W; j += 64)
    if (indices[b + (size_t)mb * j] != -1) sum += expf(align[b + (size_t)mb * j] - max_val);
  sum = wave_sum(sum);
  const float p = p_t[b];
  for (int j = lane; j < W; j += 64) {
    const size_t ix = b + (size_t)mb * j;
    const int s_idx = indices[ix];
    float a = 0.0f;
    if (s_idx != -1) {
      a = expf(align[ix] - max_val);
      const float d = p - (float)s_idx;
      const float g = expf((-1.0f * d * d) / (2.0f * sigma_sq));
      if (sum != 0.0f) a = (a / sum) * g;
    }
    align[ix] = a;
  }
}

// create_c_t_kernel (src/custom_kernels.h:1804-1813): c[:,b] = sum_j a[b + mb*j] * h_s(slot j).
template <bool VEC>
__global__ void __launch_bounds__(64)
attn_context_kernel(const float* const* __restrict__ table, int longest_sent, const float* __restrict__ align,
                    const int* __restrict__ indices, const int* __restrict__ batch_info, int H, int mb, int W,
                    float* __restrict__ ctx_out) {
  // The wave first compacts the valid slots of its column into LDS (source pointer + weight), so that the
  // accumulation loop has no data-dependent branches and several 16-byte loads are in flight per lane.
  constexpr int kMaxSlots = 512;
  __shared__ const float* s_src[kMaxSlots];
  __shared__ float s_a[kMaxSlots];
  const int b = blockIdx.y;
  const int lane = threadIdx.x;
  const int len = batch_info[b], off = batch_info[mb + b];
  int nvalid = 0;
  for (int j0 = 0; j0 < W; j0 += 64) {
    const int j = j0 + lane;
    int s_idx = -1;
    if (j < W) s_idx = indices[b + (size_t)mb * j];
    const bool valid = s_idx != -1;
    const unsigned long long m = __ballot(valid);
    if (valid) {
      int t = len - 1 - s_idx + off;
      t = t < 0 ? 0 : (t >= longest_sent ? longest_sent - 1 : t);
      const int pos = nvalid + __popcll(m & ((1ull << lane) - 1ull));
      if (pos < kMaxSlots) {
        s_src[pos] = table[t] + (size_t)b * H;
        s_a[pos] = align[b + (size_t)mb * j];
      }
    }
    nvalid += __popcll(m);
  }
  if (nvalid > kMaxSlots) nvalid = kMaxSlots;  // host guarantees W <= kMaxSlots
  __syncthreads();
  constexpr int WD = VEC ? 4 : 1;
  const int i0 = (blockIdx.x * 64 + lane) * WD;
  if (i0 >= H) return;
  float acc[WD];
#pragma unroll
  for (int q = 0; q < WD; ++q) acc[q] = 0.0f;
#pragma unroll 4
  for (int j = 0; j < nvalid; ++j) {
    const float a = s_a[j];
    const float* hs = s_src[j] + i0;
    if (VEC) {
      const zr_f32x4 v = *(const zr_f32x4*)hs;
      acc[0] += a * v.x;
      acc[1] += a * v.y;
      acc[2] += a * v.z;
      acc[3] += a * v.w;
    } else {
      acc[0] += a * hs[0];
    }
  }
  float* o = ctx_out + (size_t)b * H + i0;
  if (VEC)
    *(zr_f32x4*)o = *(zr_f32x4*)acc;
  else
    o[0] = acc[0];
}

}  // namespace

extern "C" {

int zr_attn_create(zr_ctx* ctx, int H, int mb, int D, const float* d_W_a, const float* d_W_p, const float* d_v_p,
                   const float* d_out_bias, const float* d_W_c1, const float* d_W_c2,
                   const float* const* h_hs_table, int longest_sent, zr_attn** out) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(out != nullptr, "zr_attn_create: out is null");
  *out = nullptr;
  ZR_CHECK_ARG(H > 0 && mb > 0 && D >= 0 && longest_sent > 0, "zr_attn_create: H = %d, mb = %d, D = %d, longest_sent = %d",
               H, mb, D, longest_sent);
  ZR_CHECK_ARG(mb <= 65535, "zr_attn_create: mb = %d exceeds 65535", mb);
  ZR_CHECK_ARG(2 * D + 1 <= 512, "zr_attn_create: attention width D = %d exceeds 255", D);
  ZR_CHECK_ARG(d_W_a && d_W_p && d_v_p && d_out_bias && d_W_c1 && d_W_c2 && h_hs_table, "zr_attn_create: null pointer");
  bool tables_aligned = true;
  for (int t = 0; t < longest_sent; ++t) {
    ZR_CHECK_ARG(h_hs_table[t] != nullptr, "zr_attn_create: hs table entry %d is null", t);
    tables_aligned = tables_aligned && (((uintptr_t)h_hs_table[t] & 15u) == 0);
  }
  zr_attn* a = new zr_attn();
  a->tables_aligned = tables_aligned;
  a->H = H;
  a->mb = mb;
  a->D = D;
  a->longest_sent = longest_sent;
  a->W_a = d_W_a;
  a->W_p = d_W_p;
  a->v_p = d_v_p;
  a->out_bias = d_out_bias;
  a->W_c1 = d_W_c1;
  a->W_c2 = d_W_c2;
  a->d_bf16 = nullptr;
  a->ldp = 0;
  const size_t n = (size_t)H * mb, W = 2 * (size_t)D + 1;
  // one allocation: table | tanh1 | q | ctx | align | p_t | idx
  const size_t tbytes = (sizeof(float*) * longest_sent + 255) & ~(size_t)255;
  const size_t fbytes = sizeof(float) * (3 * n + W * mb + mb);
  const size_t fpad = (fbytes + 255) & ~(size_t)255;
  char* base = nullptr;
  if (hipMalloc((void**)&base, tbytes + fpad + sizeof(int) * W * mb) != hipSuccess) {
    (void)hipGetLastError();
    delete a;
    return zr_set_error(ZR_ENOMEM, "zr_attn_create: allocation failed");
  }
  a->d_table = (const float**)base;
  float* f = (float*)(base + tbytes);
  a->d_tanh1 = f;
  a->d_q = f + n;
  a->d_ctx = f + 2 * n;
  a->d_align = f + 3 * n;
  a->d_pt = f + 3 * n + W * mb;
  a->d_idx = (int*)(base + tbytes + fpad);
  hipError_t e = hipMemcpy((void*)a->d_table, h_hs_table, sizeof(float*) * longest_sent, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(base);
    delete a;
    return zr_set_error(ZR_EHIP, "zr_attn_create: table upload failed: %s", hipGetErrorString(e));
  }
  *out = a;
  return ZR_OK;
}

int zr_attn_use_bf16_weights(zr_ctx* ctx, zr_attn* a) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(a != nullptr, "zr_attn_use_bf16_weights: attention object is null");
  const int H = a->H;
  ZR_CHECK_ARG(H % 16 == 0, "zr_attn_use_bf16_weights: H = %d is not a multiple of 16", H);
  const int ldp = (H + 31) / 32 * 32;
  const size_t per = (size_t)H * ldp;
  if (!a->d_bf16) {
    if (hipMalloc((void**)&a->d_bf16, sizeof(unsigned short) * 4 * per) != hipSuccess) {
      (void)hipGetLastError();
      a->d_bf16 = nullptr;
      return zr_set_error(ZR_ENOMEM, "zr_attn_use_bf16_weights: allocation failed");
    }
  }
  a->ldp = ldp;
  const float* src[4] = {a->W_p, a->W_a, a->W_c1, a->W_c2};
  for (int i = 0; i < 4; ++i) {
    rc = zr_pack8_bf16_launch(ctx, src[i], H, H, H, ldp, H, a->d_bf16 + i * per, i == 1 ? 1 : 0);  // W_a transposed
    if (rc) return rc;
  }
  return ZR_OK;
}

int zr_attn_destroy(zr_ctx* ctx, zr_attn* a) {
  if (!a) return ZR_OK;
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  if (a->d_bf16) (void)hipFree(a->d_bf16);
  (void)hipFree((void*)a->d_table);
  delete a;
  return ZR_OK;
}

int zr_attn_step(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const float* d_h_t, const int* d_mask01,
                 float* d_htild, float* d_alignments, int* d_indices, float* d_p_t, float* d_c_ctx) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(a != nullptr, "zr_attn_step: attention object is null");
  ZR_CHECK_ARG(d_batch_info && d_h_t && d_mask01 && d_htild, "zr_attn_step: null pointer");
  const int H = a->H, mb = a->mb, D = a->D, W = 2 * D + 1;
  float* align = d_alignments ? d_alignments : a->d_align;
  int* idx = d_indices ? d_indices : a->d_idx;
  float* pt = d_p_t ? d_p_t : a->d_pt;
  float* cctx = d_c_ctx ? d_c_ctx : a->d_ctx;

  // tanh(W_p h)  (reference: attention_node.hpp:132-141)
  ZrGemmDesc g = {};
  g.M = H;
  g.N = mb;
  g.nseg = 1;
  g.K[0] = H;
  const size_t per = (size_t)H * a->ldp;
  g.A[0] = a->W_p;
  g.lda[0] = H;
  if (a->d_bf16) {
    g.A[0] = (const float*)a->d_bf16;
    g.lda[0] = a->ldp;
    g.a_pack = 2;
  }
  g.B[0] = d_h_t;
  g.ldb[0] = H;
  g.C = a->d_tanh1;
  g.ldc = H;
  g.batch = 1;
  g.epilogue = ZR_EPI_TANH;
  rc = zr_gemm_launch(ctx, g);
  if (rc) return rc;
  attn_window_kernel<<<mb, 64, 0, ctx->stream>>>(a->d_tanh1, a->v_p, d_batch_info, d_mask01, H, mb, D, pt, idx);
  ZR_LAUNCH_CHECK("attn_window_kernel");
  // q = W_a^T h  (:195)
  g.A[0] = a->W_a;
  g.trans_a = 1;
  if (a->d_bf16) {
    g.A[0] = (const float*)(a->d_bf16 + per);  // already transposed
    g.trans_a = 0;
  }
  g.C = a->d_q;
  g.epilogue = ZR_EPI_STORE;
  rc = zr_gemm_launch(ctx, g);
  if (rc) return rc;
  // 16-byte loads need H % 4 == 0 and 16-byte aligned table / output bases (column offsets are multiples of H)
  const bool vec = (H % 4 == 0) && a->tables_aligned && (((uintptr_t)cctx & 15u) == 0);
  const long long slots = (long long)mb * W;
  const unsigned sgrid = (unsigned)((slots + 3) / 4);
  if (vec)
    attn_score_kernel<true><<<sgrid, 256, 0, ctx->stream>>>(a->d_table, a->longest_sent, a->d_q, idx, d_batch_info, H,
                                                            mb, W, align, ctx->d_flags);
  else
    attn_score_kernel<false><<<sgrid, 256, 0, ctx->stream>>>(a->d_table, a->longest_sent, a->d_q, idx, d_batch_info,
                                                             H, mb, W, align, ctx->d_flags);
  ZR_LAUNCH_CHECK("attn_score_kernel");
  const float sigma_sq = (float)((D * D) / 4.0);  // attention_node.hpp:50
  attn_align_kernel<<<mb, 64, 0, ctx->stream>>>(align, idx, pt, mb, W, sigma_sq);
  ZR_LAUNCH_CHECK("attn_align_kernel");
  if (vec) {
    dim3 cg((H / 4 + 63) / 64, mb);
    attn_context_kernel<true><<<cg, 64, 0, ctx->stream>>>(a->d_table, a->longest_sent, align, idx, d_batch_info, H,
                                                          mb, W, cctx);
  } else {
    dim3 cg((H + 63) / 64, mb);
    attn_context_kernel<false><<<cg, 64, 0, ctx->stream>>>(a->d_table, a->longest_sent, align, idx, d_batch_info, H,
                                                           mb, W, cctx);
  }
  ZR_LAUNCH_CHECK("attn_context_kernel");
  // h~ = tanh(W_c1 c + W_c2 h + b) * mask  (:354-379) as one two-segment GEMM with a fused epilogue
  ZrGemmDesc o = {};
  o.M = H;
  o.N = mb;
  o.nseg = 2;
  o.K[0] = H;
  o.A[0] = a->W_c1;
  o.lda[0] = H;
  o.B[0] = cctx;
  o.ldb[0] = H;
  o.K[1] = H;
  o.A[1] = a->W_c2;
  o.lda[1] = H;
  if (a->d_bf16) {
    o.A[0] = (const float*)(a->d_bf16 + 2 * per);
    o.A[1] = (const float*)(a->d_bf16 + 3 * per);
    o.lda[0] = o.lda[1] = a->ldp;
    o.a_pack = 2;
  }
  o.B[1] = d_h_t;
  o.ldb[1] = H;
  o.C = d_htild;
  o.ldc = H;
  o.batch = 1;
  o.bias = a->out_bias;
  o.mask = d_mask01;
  o.epilogue = ZR_EPI_TANH_BIAS_MASK;
  return zr_gemm_launch(ctx, o);
}

}  // extern "C"
