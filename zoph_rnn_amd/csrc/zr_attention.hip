// Luong local-p attention with the "general" score and feed-input output, forward only
// (reference: attention_node::forward_prop, src/attention_node.hpp:73-394).
//
// The reference materialises the (2D+1) x H x mb window of source states (load_in_hs_kernel) and reads it
// twice.  Here the score and context kernels read the source states in place through the pointer table, so
// the only traffic is the valid source columns themselves, once for the scores and once for the context.
#include <math.h>

#include "zr_internal.h"
#include "zr_mfma_core.h"


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

// The four consecutive rows 4*k4 .. 4*k4+3 of column b as bf16 terms, into arrays laid out [H/8][mb][8] (what the bf16
// products read: zr_split_pack_multi_kernel's layout and its hi / lo split).  lo may be null (single-term mode).
__device__ __forceinline__ void store_bf16_terms(const zr_f32x4& v, int k4, int b, int mb, unsigned short* hi,
                                                 unsigned short* lo) {
  typedef unsigned zr_u32x2 __attribute__((ext_vector_type(2)));
  unsigned h0, l0, h1, l1;
  zr_split_bf16_pair(v.x, v.y, h0, l0);
  zr_split_bf16_pair(v.z, v.w, h1, l1);
  const size_t o = ((size_t)(k4 >> 1) * mb + b) * 8 + (size_t)(k4 & 1) * 4;
  *(zr_u32x2*)(hi + o) = zr_u32x2{h0, h1};
  if (lo) *(zr_u32x2*)(lo + o) = zr_u32x2{l0, l1};
}

__device__ __forceinline__ float block_sum_256(float v, float* s_red, int tid) {
  v = wave_sum(v);
  __syncthreads();  // the previous use of s_red is over
  if ((tid & 63) == 0) s_red[tid >> 6] = v;
  __syncthreads();
  return s_red[0] + s_red[1] + s_red[2] + s_red[3];
}

// Everything of the attention step between the two projections and the output product, for one batch column per
// workgroup: p_t and the window (attn_window_kernel; `pre` holds W_p h BEFORE the tanh), the scores h_s . q of the
// valid window slots (attn_score_kernel), the reference's max-starts-at-0 softmax times the Gaussian
// (attn_align_kernel) and the context vector (attn_context_kernel).  The valid source columns come from memory once,
// for the scores; the context pass a few microseconds later finds them in the L2 the workgroup's CU sits behind.
// Requires H % 4 == 0 and 16-byte aligned source tables, pre, q and ctx_out; W <= 512.
__global__ void __launch_bounds__(256)
attn_fused_kernel(const float* const* __restrict__ table, int longest_sent, const float* __restrict__ pre,
                  const float* __restrict__ q, const float* __restrict__ v_p, const int* __restrict__ batch_info,
                  const int* __restrict__ mask01, int H, int mb, int D, float sigma_sq, float* __restrict__ p_t,
                  int* __restrict__ indices, float* __restrict__ align, float* __restrict__ ctx_out,
                  float* __restrict__ ctx_pack, unsigned short* __restrict__ ctx_hi,
                  unsigned short* __restrict__ ctx_lo, int* __restrict__ flags) {
  constexpr int kMaxSlots = 512;
  __shared__ float s_red[4];
  __shared__ float s_val[kMaxSlots];         // scores, then alignment weights, of the valid slots
  __shared__ const float* s_src[kMaxSlots];  // source column of each valid slot
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int W = 2 * D + 1;
  const int H4 = H >> 2;
  // p_t = S * sigmoid(v_p . tanh(W_p h)), sigmoid in double as the reference's sigmoid_kernel
  float part = 0.0f;
  for (int k4 = tid; k4 < H4; k4 += 256) {
    const zr_f32x4 t = ((const zr_f32x4*)(pre + (size_t)b * H))[k4];
    const zr_f32x4 v = ((const zr_f32x4*)v_p)[k4];
    part += v.x * tanhf(t.x) + v.y * tanhf(t.y) + v.z * tanhf(t.z) + v.w * tanhf(t.w);
  }
  const float sdot = block_sum_256(part, s_red, tid);
  const float sig = (float)(1.0 / (1.0 + exp(-1.0 * (double)sdot)));
  const int len = batch_info[b], off = batch_info[mb + b];
  const float p = (float)len * sig;
  const int ip = (int)p;
  const int lo = (0 > ip - D) ? 0 : (ip - D);
  const int hi = ((len - 1) < ip + D) ? (len - 1) : (ip + D);
  const bool live = mask01[b] == 1;
  int nvalid = live ? hi - lo + 1 : 0;
  nvalid = nvalid < 0 ? 0 : (nvalid > W ? W : nvalid);
  if (tid == 0) p_t[b] = p;
  for (int j = tid; j < W; j += 256) {
    indices[b + (size_t)mb * j] = j < nvalid ? lo + j : -1;
    if (j < nvalid) {
      int t = len - 1 - (lo + j) + off;
      if (t < 0 || t >= longest_sent) {
        atomicAdd(&flags[1], 1);
        t = t < 0 ? 0 : longest_sent - 1;
      }
      s_src[j] = table[t] + (size_t)b * H;
    }
  }
  __syncthreads();
  // scores: the slots go round the four waves, eight at a time per wave and four 16-byte pieces of each per lane, so
  // that 36 loads of a lane are in flight together (a column's source states are 4 * H * nvalid bytes that only this
  // workgroup asks for: what it keeps in flight is what it gets per memory latency)
  {
    constexpr int SG = 8;
    const zr_f32x4* qc = (const zr_f32x4*)(q + (size_t)b * H);
    const zr_f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j = wave * SG; j < nvalid; j += 4 * SG) {
      const zr_f32x4* hsrc[SG];
#pragma unroll
      for (int u = 0; u < SG; ++u) hsrc[u] = (const zr_f32x4*)s_src[j + u < nvalid ? j + u : j];
      float a[SG];
#pragma unroll
      for (int u = 0; u < SG; ++u) a[u] = 0.0f;
      for (int k0 = 0; k0 < H4; k0 += 256) {
        zr_f32x4 c[4], x[SG][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int k4 = k0 + 64 * i + lane;
          const bool ok = k4 < H4;
          c[i] = ok ? qc[k4] : zero4;
#pragma unroll
          for (int u = 0; u < SG; ++u) x[u][i] = ok ? hsrc[u][k4] : zero4;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (k0 + 64 * i + lane < H4) {
#pragma unroll
            for (int u = 0; u < SG; ++u)
              a[u] += x[u][i].x * c[i].x + x[u][i].y * c[i].y + x[u][i].z * c[i].z + x[u][i].w * c[i].w;
          }
      }
#pragma unroll
      for (int u = 0; u < SG; ++u) a[u] = wave_sum(a[u]);
      if (lane == 0) {
#pragma unroll
        for (int u = 0; u < SG; ++u)
          if (j + u < nvalid) s_val[j + u] = a[u];
      }
    }
  }
  __syncthreads();
  // alignment weights (alignment_reduction_kernel, src/custom_kernels.h:1752-1794): the maximum starts at 0
  if (wave == 0) {
    float max_val = 0.0f;
    for (int j = lane; j < nvalid; j += 64) max_val = fmaxf(max_val, s_val[j]);
    max_val = wave_max(max_val);
    float sum = 0.0f;
    for (int j = lane; j < nvalid; j += 64) sum += expf(s_val[j] - max_val);
    sum = wave_sum(sum);
    for (int j = lane; j < W; j += 64) {
      float a = 0.0f;
      if (j < nvalid) {
        a = expf(s_val[j] - max_val);
        const float d = p - (float)(lo + j);
        const float g = expf((-1.0f * d * d) / (2.0f * sigma_sq));
        if (sum != 0.0f) a = (a / sum) * g;
        s_val[j] = a;
      }
      align[b + (size_t)mb * j] = a;
    }
  }
  __syncthreads();
  // context: c[:, b] = sum_j a_j h_s(slot j): four rows per thread at two places of the column, eight slots of each
  // in flight (sixteen loads per lane)
  for (int k0 = 0; k0 < H4; k0 += 512) {
    const int ka = k0 + tid, kb = k0 + 256 + tid;
    const bool oka = ka < H4, okb = kb < H4;
    const zr_f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    zr_f32x4 acc_a = zero4, acc_b = zero4;
    int j = 0;
    for (; j + 8 <= nvalid; j += 8) {
      zr_f32x4 xa[8], xb[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const zr_f32x4* src = (const zr_f32x4*)s_src[j + u];
        xa[u] = oka ? src[ka] : zero4;
        xb[u] = okb ? src[kb] : zero4;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        acc_a += s_val[j + u] * xa[u];
        acc_b += s_val[j + u] * xb[u];
      }
    }
    for (; j < nvalid; ++j) {
      const zr_f32x4* src = (const zr_f32x4*)s_src[j];
      if (oka) acc_a += s_val[j] * src[ka];
      if (okb) acc_b += s_val[j] * src[kb];
    }
    if (oka) {
      ((zr_f32x4*)(ctx_out + (size_t)b * H))[ka] = acc_a;
      if (ctx_pack) ((zr_f32x4*)ctx_pack)[(size_t)ka * mb + b] = acc_a;
      if (ctx_hi) store_bf16_terms(acc_a, ka, b, mb, ctx_hi, ctx_lo);
    }
    if (okb) {
      ((zr_f32x4*)(ctx_out + (size_t)b * H))[kb] = acc_b;
      if (ctx_pack) ((zr_f32x4*)ctx_pack)[(size_t)kb * mb + b] = acc_b;
      if (ctx_hi) store_bf16_terms(acc_b, kb, b, mb, ctx_hi, ctx_lo);
    }
  }
}

// get_viterbi_alignment_kernel (src/custom_kernels.h:1623-1635): per column, the source position of the window slot with
// the largest alignment weight.  The reference scans the slots in order with a running maximum that starts at -1 and
// is replaced only by a strictly larger weight, so the first of equal maxima wins, and a column whose weights are all
// zero reports the index of its first slot (-1 when the column is masked).  One wave per column: every lane scans its
// slots in order, then the lanes' (weight, slot) pairs are merged, larger weight first and lower slot on a tie.
__global__ void __launch_bounds__(64)
attn_viterbi_kernel(const float* __restrict__ align, const int* __restrict__ indices, int mb, int W,
                    int* __restrict__ out) {
  const int b = blockIdx.x;
  const int lane = threadIdx.x;
  float best = -1.0f;
  int slot = 0x7fffffff;
  for (int j = lane; j < W; j += 64) {
    const float a = align[b + (size_t)mb * j];
    if (best < a) {
      best = a;
      slot = j;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ob = __shfl_xor(best, off, 64);
    const int os = __shfl_xor(slot, off, 64);
    if (ob > best || (ob == best && os < slot)) {
      best = ob;
      slot = os;
    }
  }
  if (lane == 0) out[b] = slot == 0x7fffffff ? -1 : indices[b + (size_t)mb * slot];
}

// The alignment vote of an ensemble (ensemble_factory::ensembles_models, src/ensemble_factory.hpp:797-834): every model
// spreads its window's alignment weights over a row of longest_sent source positions (zero elsewhere,
// src/attention_node.hpp:236-268), the rows are added in model order, and the column's alignment is the first position
// whose sum is strictly larger than every earlier one, starting from 0 (so -1 when no sum is positive).  One workgroup
// per column; the row lives in LDS, each model's window is added behind a barrier (a window's positions are distinct,
// so no two lanes meet on one element and the sum keeps the reference's order of additions).
constexpr int kMaxEnsembleAlign = 16;
struct EnsembleAlignArgs {
  const float* align[kMaxEnsembleAlign];
  const int* idx[kMaxEnsembleAlign];
};
__global__ void __launch_bounds__(256)
attn_viterbi_ensemble_kernel(EnsembleAlignArgs a, int n_models, int mb, int W, int longest, int* __restrict__ out) {
  extern __shared__ float s_score[];
  __shared__ float s_best[256];
  __shared__ int s_pos[256];
  const int b = blockIdx.x, tid = threadIdx.x;
  for (int j = tid; j < longest; j += 256) s_score[j] = 0.0f;
  __syncthreads();
  for (int k = 0; k < n_models; ++k) {
    for (int j = tid; j < W; j += 256) {
      const int ix = a.idx[k][b + (size_t)mb * j];
      if (ix >= 0 && ix < longest) s_score[ix] += a.align[k][b + (size_t)mb * j];
    }
    __syncthreads();
  }
  float best = 0.0f;
  int pos = -1;
  for (int j = tid; j < longest; j += 256) {
    const float v = s_score[j];
    if (v > best) {
      best = v;
      pos = j;
    }
  }
  s_best[tid] = best;
  s_pos[tid] = pos;
  __syncthreads();
  for (int st = 128; st > 0; st >>= 1) {
    if (tid < st) {
      const float ob = s_best[tid + st];
      const int op = s_pos[tid + st];
      if (ob > s_best[tid] || (ob == s_best[tid] && op < s_pos[tid])) {
        s_best[tid] = ob;
        s_pos[tid] = op;
      }
    }
    __syncthreads();
  }
  if (tid == 0) out[b] = s_pos[0];
}

// Sum over the 64 lanes of each of N values held one per register: lanes end up with the totals in all lanes.
template <int N>
__device__ __forceinline__ void wave_sum_many(float (&v)[N]) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += __shfl_xor(v[i], off, 64);
}

// attn_fused_kernel for H <= 1024 and at most MAXS window slots: every thread owns four consecutive rows and keeps
// them, for every valid slot, in registers -- all loads of a column's source states are in flight together, the
// scores are formed from the registers, and so is the context, so the source states are read exactly once and nothing
// is read twice.  Also writes the context k-interleaved ([H/4][mb][4]) for the output product when ctx_pack is given.
// (With global attention -- D at least the sentence length -- the window does not depend on p_t, and requesting the
// source states before p_t is computed was tried: the registers they occupy while the tanh, the reduction and the
// double-precision sigmoid run push those computations into scratch; 47.9 us against 44.3 for the config-3 attention
// step, and twice the time at H = 2000.)
template <int MAXS, int NT = 256>
__global__ void __launch_bounds__(NT)
attn_fused_reg_kernel(const float* const* __restrict__ table, int longest_sent, const float* __restrict__ pre,
                      const float* __restrict__ q, const float* __restrict__ v_p, const int* __restrict__ batch_info,
                      const int* __restrict__ mask01, int H, int mb, int D, float sigma_sq, float* __restrict__ p_t,
                      int* __restrict__ indices, float* __restrict__ align, float* __restrict__ ctx_out,
                      float* __restrict__ ctx_pack, unsigned short* __restrict__ ctx_hi,
                      unsigned short* __restrict__ ctx_lo, int* __restrict__ flags) {
  constexpr int NW = NT / 64;
  __shared__ float s_red[NW];
  __shared__ float s_part[NW][MAXS];
  __shared__ float s_val[MAXS];
  __shared__ const float* s_src[MAXS];
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int W = 2 * D + 1;
  const int H4 = H >> 2;
  const bool mine = tid < H4;
  const int k4 = mine ? tid : 0;
  float part = 0.0f;
  if (mine) {
    const zr_f32x4 t = ((const zr_f32x4*)(pre + (size_t)b * H))[k4];
    const zr_f32x4 v = ((const zr_f32x4*)v_p)[k4];
    part = v.x * tanhf(t.x) + v.y * tanhf(t.y) + v.z * tanhf(t.z) + v.w * tanhf(t.w);
  }
  const zr_f32x4 qv = ((const zr_f32x4*)(q + (size_t)b * H))[k4];
  float sdot = wave_sum(part);
  if (lane == 0) s_red[wave] = sdot;
  __syncthreads();
  sdot = s_red[0];
#pragma unroll
  for (int w = 1; w < NW; ++w) sdot += s_red[w];
  const float sig = (float)(1.0 / (1.0 + exp(-1.0 * (double)sdot)));
  const int len = batch_info[b], off = batch_info[mb + b];
  const float p = (float)len * sig;
  const int ip = (int)p;
  const int lo = (0 > ip - D) ? 0 : (ip - D);
  const int hi = ((len - 1) < ip + D) ? (len - 1) : (ip + D);
  const bool live = mask01[b] == 1;
  int nvalid = live ? hi - lo + 1 : 0;
  nvalid = nvalid < 0 ? 0 : (nvalid > W ? W : nvalid);
  nvalid = nvalid > MAXS ? MAXS : nvalid;  // the host picks MAXS >= min(W, longest_sent)
  if (tid == 0) p_t[b] = p;
  for (int j = tid; j < W; j += NT) indices[b + (size_t)mb * j] = j < nvalid ? lo + j : -1;
  if (tid < nvalid) {
    int t = len - 1 - (lo + tid) + off;
    if (t < 0 || t >= longest_sent) {
      atomicAdd(&flags[1], 1);
      t = t < 0 ? 0 : longest_sent - 1;
    }
    s_src[tid] = table[t] + (size_t)b * H;
  }
  __syncthreads();
  zr_f32x4 x[MAXS];
#pragma unroll
  for (int j = 0; j < MAXS; ++j) {
    x[j] = zr_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (j < nvalid && mine) x[j] = ((const zr_f32x4*)s_src[j])[k4];
  }
  // partial scores of this thread's four rows, summed over the wave in batches of 16 slots, then over the four waves
#pragma unroll
  for (int j0 = 0; j0 < MAXS; j0 += 16) {
    if (j0 < nvalid) {  // uniform over the workgroup
      float d[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        constexpr int kLast = MAXS - 1;
        const zr_f32x4& xv = x[j0 + i < MAXS ? j0 + i : kLast];  // (MAXS need not be a multiple of 16)
        d[i] = xv.x * qv.x + xv.y * qv.y + xv.z * qv.z + xv.w * qv.w;
      }
      wave_sum_many<16>(d);
      float dl = d[0];  // lane i keeps slot j0 + i
#pragma unroll
      for (int i = 1; i < 16; ++i) dl = lane == i ? d[i] : dl;
      if (lane < 16 && j0 + lane < MAXS) s_part[wave][j0 + lane] = dl;
    }
  }
  __syncthreads();
  if (wave == 0) {
    // alignment_reduction_kernel (src/custom_kernels.h:1752-1794): the maximum starts at 0
    float sc = 0.0f;
    const bool v = lane < nvalid;
    if (MAXS <= 64) {
      if (v) {
        sc = (s_part[0][lane] + s_part[1][lane]) + (s_part[2][lane] + s_part[3][lane]);
        if (NW == 8) sc += (s_part[4][lane] + s_part[5][lane]) + (s_part[6][lane] + s_part[7][lane]);
      }
      const float max_val = wave_max(v ? fmaxf(sc, 0.0f) : 0.0f);
      const float e = v ? expf(sc - max_val) : 0.0f;
      const float sum = wave_sum(e);
      float a = 0.0f;
      if (v) {
        const float dd = p - (float)(lo + lane);
        const float g = expf((-1.0f * dd * dd) / (2.0f * sigma_sq));
        a = sum != 0.0f ? (e / sum) * g : e;
        s_val[lane] = a;
      }
      for (int j = lane; j < W; j += 64) align[b + (size_t)mb * j] = j == lane ? a : 0.0f;
    }
  }
  __syncthreads();
  if (mine) {
    zr_f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < MAXS; ++j)
      if (j < nvalid) acc += s_val[j] * x[j];
    ((zr_f32x4*)(ctx_out + (size_t)b * H))[k4] = acc;
    if (ctx_pack) ((zr_f32x4*)ctx_pack)[(size_t)k4 * mb + b] = acc;
    if (ctx_hi) store_bf16_terms(acc, k4, b, mb, ctx_hi, ctx_lo);
  }
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
  a->d_pack32 = nullptr;
  a->d_pq = nullptr;
  a->d_err_table = nullptr;
  a->ldp32 = a->kp32 = 0;
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
    // the four matrices, then room for h_t as two bf16 terms (split once per step for its three products)
    if (hipMalloc((void**)&a->d_bf16, sizeof(unsigned short) * (4 * per + 6 * (size_t)H * a->mb)) != hipSuccess) {
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

int zr_attn_viterbi(zr_ctx* ctx, const zr_attn* a, const float* d_alignments, const int* d_indices, int* d_viterbi) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(a != nullptr && d_viterbi != nullptr, "zr_attn_viterbi: null attention object or output");
  const float* al = d_alignments ? d_alignments : a->d_align;
  const int* ix = d_indices ? d_indices : a->d_idx;
  attn_viterbi_kernel<<<a->mb, 64, 0, ctx->stream>>>(al, ix, a->mb, 2 * a->D + 1, d_viterbi);
  ZR_LAUNCH_CHECK("attn_viterbi_kernel");
  return ZR_OK;
}

int zr_attn_viterbi_ensemble(zr_ctx* ctx, int n_models, const float* const d_alignments[], const int* const d_indices[],
                             int slots, int cols, int longest_sent, int* d_viterbi) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n_models >= 1 && n_models <= kMaxEnsembleAlign && slots > 0 && cols > 0 && cols <= 65535 &&
                   longest_sent > 0 && longest_sent <= 8192 && d_alignments && d_indices && d_viterbi,
               "zr_attn_viterbi_ensemble: %d models (at most %d), %d slots, %d columns, longest_sent = %d (at most 8192), "
               "or a null pointer", n_models, kMaxEnsembleAlign, slots, cols, longest_sent);
  EnsembleAlignArgs a{};
  for (int k = 0; k < n_models; ++k) {
    ZR_CHECK_ARG(d_alignments[k] && d_indices[k], "zr_attn_viterbi_ensemble: model %d has a null array", k);
    a.align[k] = d_alignments[k];
    a.idx[k] = d_indices[k];
  }
  attn_viterbi_ensemble_kernel<<<cols, 256, (size_t)longest_sent * sizeof(float), ctx->stream>>>(a, n_models, cols, slots,
                                                                                                longest_sent, d_viterbi);
  ZR_LAUNCH_CHECK("attn_viterbi_ensemble_kernel");
  return ZR_OK;
}

int zr_attn_prepare(zr_ctx* ctx, zr_attn* a) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(a != nullptr, "zr_attn_prepare: attention object is null");
  const int H = a->H;
  const int ldp = (H + 31) / 32 * 32, kp = (H + 7) / 8 * 8;
  const size_t per = (size_t)kp * ldp;
  if (!a->d_pack32) {
    if (hipMalloc((void**)&a->d_pack32, sizeof(float) * (4 * per + 3 * (size_t)H * a->mb + 3 * (size_t)ldp * a->mb + 32)) !=
        hipSuccess) {
      (void)hipGetLastError();
      a->d_pack32 = nullptr;
      return zr_set_error(ZR_ENOMEM, "zr_attn_prepare: allocation failed");
    }
  }
  a->ldp32 = ldp;
  a->kp32 = kp;
  // the context's copy first, h_t's right behind it: together they are the k-interleaved [c; h_t] (2H x mb) that the
  // output product multiplies with [W_c1 | W_c2], whose snapshots are neighbours as well
  a->d_cpack = a->d_pack32 + 4 * per;
  a->d_hpack = a->d_cpack + (size_t)H * a->mb;
  a->d_htpack = a->d_hpack + (size_t)H * a->mb;
  // (every column of these two starts a 128-byte line, so that a line has one producing tile and one consuming column)
  a->d_pq = a->d_pack32 + (4 * per + 3 * (size_t)H * a->mb + 31) / 32 * 32;
  rc = zr_pack4_launch(ctx, a->W_p, H, H, H, ldp, kp, a->d_pack32);
  if (rc) return rc;
  rc = zr_pack4_trans_launch(ctx, a->W_a, H, H, H, ldp, kp, a->d_pack32 + per);  // W_a^T
  if (rc) return rc;
  rc = zr_pack4_launch(ctx, a->W_c1, H, H, H, ldp, kp, a->d_pack32 + 2 * per);
  if (rc) return rc;
  return zr_pack4_launch(ctx, a->W_c2, H, H, H, ldp, kp, a->d_pack32 + 3 * per);
}

int zr_attn_destroy(zr_ctx* ctx, zr_attn* a) {
  if (!a) return ZR_OK;
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  if (a->d_bf16) (void)hipFree(a->d_bf16);
  if (a->d_pack32) (void)hipFree(a->d_pack32);
  if (a->d_err_table) (void)hipFree((void*)a->d_err_table);
  (void)hipFree((void*)a->d_table);
  delete a;
  return ZR_OK;
}

static int attn_step_impl(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const float* d_h_t, const int* d_mask01,
                          float* d_htild, float* d_alignments, int* d_indices, float* d_p_t, float* d_c_ctx,
                          bool h_packed, float* d_htild_pack);

int zr_attn_step(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const float* d_h_t, const int* d_mask01,
                 float* d_htild, float* d_alignments, int* d_indices, float* d_p_t, float* d_c_ctx) {
  return attn_step_impl(ctx, a, d_batch_info, d_h_t, d_mask01, d_htild, d_alignments, d_indices, d_p_t, d_c_ctx, false,
                        nullptr);
}

// True when zr_attn_step on these operands runs on the k-interleaved fp32 snapshots (the single launch or the three
// launches): prepared matrices and everything it reads with 16-byte accesses aligned.  The one predicate for both the
// step itself and zr_decoder_step's choice of hand-over layout.
static bool attn_on_snapshots(const zr_attn* a, const float* d_h_t, const float* d_c_ctx) {
  const float* cctx = d_c_ctx ? d_c_ctx : a->d_ctx;
  return a->d_pack32 && !a->d_bf16 && (a->H % 4 == 0) && a->tables_aligned &&
         ((((uintptr_t)cctx | (uintptr_t)d_h_t | (uintptr_t)a->v_p) & 15u) == 0);
}
// ... and reads h_t from a->d_hpack (and can write h~ k-interleaved)
static bool attn_reads_packed_h(const zr_attn* a, const float* d_h_t, const float* d_c_ctx) {
  return attn_on_snapshots(a, d_h_t, d_c_ctx) && a->H % 8 == 0;
}

int zr_decoder_step(zr_ctx* ctx, int nl, const zr_lstm_weights* const layers[], const float* d_embed, int V_in,
                    const int* d_ids_nonneg, const float* const d_hprev[], const float* const d_cprev[],
                    const float* d_htild_prev, const int* d_mask01, float clip_threshold, int mb, float* const d_h[],
                    float* const d_c[], zr_attn* attn, const int* d_batch_info, float* d_htild, float* d_alignments,
                    int* d_indices, float* d_p_t, float* d_c_ctx, const float* d_D, const float* d_b_d, int V_out,
                    int mode, float* d_out) {
  ZR_CHECK_ARG(nl > 0 && d_h && d_D && d_b_d && d_out, "zr_decoder_step: null pointer or L = %d", nl);
  ZR_CHECK_ARG(!attn || (attn->mb == mb && d_batch_info && d_htild), "zr_decoder_step: attention layer of another width, or "
               "null batch info / h~");
  const float* top = d_h[nl - 1];
  const bool packed = attn && top && attn_reads_packed_h(attn, top, d_c_ctx);
  // bf16 weights on both sides: the top LSTM layer leaves h_t as bf16 terms in the attention layer's buffer
  const bool split16 = attn && top && attn->d_bf16 && layers && layers[0] && layers[0]->bf16 &&
                       layers[0]->H == attn->H && (((uintptr_t)top & 15u) == 0);
  // (an fp32 attention layer behind bf16 LSTM layers, or the other way round, re-lays h_t out itself)
  const bool pack32 = packed && layers && layers[0] && !layers[0]->bf16;
  float* hand_over = pack32 ? attn->d_hpack
                            : (split16 ? (float*)(attn->d_bf16 + 4 * (size_t)attn->H * attn->ldp) : nullptr);
  int wrote = 0;
  int rc = zr_lstm_decoder_step_packed(ctx, nl, layers, d_embed, V_in, d_ids_nonneg, d_hprev, d_cprev, d_htild_prev,
                                       d_mask01, clip_threshold, mb, d_h, d_c, hand_over, &wrote);
  if (rc) return rc;
  if (!attn)
    return zr_softmax_forward_packed(ctx, d_D, d_b_d, V_out, layers[0]->H, top, nullptr, mb, mode, d_out, nullptr);
  rc = attn_step_impl(ctx, attn, d_batch_info, top, d_mask01, d_htild, d_alignments, d_indices, d_p_t, d_c_ctx,
                      (pack32 || split16) && wrote, packed ? attn->d_htpack : nullptr);
  if (rc) return rc;
  // (the k-interleaved h~ only if the attention step says it wrote it)
  return zr_softmax_forward_packed(ctx, d_D, d_b_d, V_out, attn->H, d_htild,
                                   attn->wrote_htild_pack ? attn->d_htpack : nullptr, mb, mode, d_out, nullptr,
                                   attn->htild_hi, attn->htild_lo);
}

// Everything between the projections and the output product in one launch (d_tanh1 holds W_p h BEFORE the tanh, d_q
// holds W_a^T h): the register-resident kernel up to H = 1024 and 64 window slots, the two-pass one beyond.
static int launch_attn_middle(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const int* d_mask01, float* pt, int* idx,
                              float* align, float* cctx, float* cpack, unsigned short* chi = nullptr,
                              unsigned short* clo = nullptr) {
  const int H = a->H, mb = a->mb, D = a->D, W = 2 * D + 1;
  const float sigma_sq = (float)((D * D) / 4.0);  // attention_node.hpp:50
  const int max_slots = W < a->longest_sent ? W : a->longest_sent;
  if (H <= 1024 && max_slots <= 16)
    attn_fused_reg_kernel<16><<<mb, 256, 0, ctx->stream>>>(a->d_table, a->longest_sent, a->d_tanh1, a->d_q, a->v_p,
                                                           d_batch_info, d_mask01, H, mb, D, sigma_sq, pt, idx, align,
                                                           cctx, cpack, chi, clo, ctx->d_flags);
  else if (H <= 1024 && max_slots <= 32)
    attn_fused_reg_kernel<32><<<mb, 256, 0, ctx->stream>>>(a->d_table, a->longest_sent, a->d_tanh1, a->d_q, a->v_p,
                                                           d_batch_info, d_mask01, H, mb, D, sigma_sq, pt, idx, align,
                                                           cctx, cpack, chi, clo, ctx->d_flags);
  else if (H <= 1024 && max_slots <= 64)
    attn_fused_reg_kernel<64><<<mb, 256, 0, ctx->stream>>>(a->d_table, a->longest_sent, a->d_tanh1, a->d_q, a->v_p,
                                                           d_batch_info, d_mask01, H, mb, D, sigma_sq, pt, idx, align,
                                                           cctx, cpack, chi, clo, ctx->d_flags);
  else if (H <= 2048 && max_slots <= 52)
    // eight waves: every thread still holds one 16-byte piece of each slot (2 x 256 registers per lane pair of a SIMD)
    attn_fused_reg_kernel<52, 512><<<mb, 512, 0, ctx->stream>>>(a->d_table, a->longest_sent, a->d_tanh1, a->d_q, a->v_p,
                                                                d_batch_info, d_mask01, H, mb, D, sigma_sq, pt, idx, align,
                                                                cctx, cpack, chi, clo, ctx->d_flags);
  else
    attn_fused_kernel<<<mb, 256, 0, ctx->stream>>>(a->d_table, a->longest_sent, a->d_tanh1, a->d_q, a->v_p, d_batch_info,
                                                   d_mask01, H, mb, D, sigma_sq, pt, idx, align, cctx, cpack, chi, clo,
                                                   ctx->d_flags);
  ZR_LAUNCH_CHECK("attn_fused_kernel");
  return ZR_OK;
}

static int attn_step_impl(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const float* d_h_t, const int* d_mask01,
                          float* d_htild, float* d_alignments, int* d_indices, float* d_p_t, float* d_c_ctx,
                          bool h_packed, float* d_htild_pack) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(a != nullptr, "zr_attn_step: attention object is null");
  ZR_CHECK_ARG(d_batch_info && d_h_t && d_mask01 && d_htild, "zr_attn_step: null pointer");
  a->htild_hi = a->htild_lo = nullptr;
  const int H = a->H, mb = a->mb, D = a->D, W = 2 * D + 1;
  float* align = d_alignments ? d_alignments : a->d_align;
  int* idx = d_indices ? d_indices : a->d_idx;
  float* pt = d_p_t ? d_p_t : a->d_pt;
  float* cctx = d_c_ctx ? d_c_ctx : a->d_ctx;

  a->wrote_htild_pack = false;
  const bool fast = attn_on_snapshots(a, d_h_t, d_c_ctx);
  if (fast) {
    a->wrote_htild_pack = d_htild_pack != nullptr && H % 8 == 0;
    // Three launches.  (1) W_p h (before the tanh) and q = W_a^T h as one batch of two products on the k-interleaved
    // snapshots; d_tanh1 and d_q are neighbours in the object's allocation (stride H*mb).
    const size_t per = (size_t)a->kp32 * a->ldp32;
    ZrGemmDesc g = {};
    g.M = H;
    g.N = mb;
    g.nseg = 1;
    g.K[0] = H;
    g.A[0] = a->d_pack32;
    g.lda[0] = a->ldp32;
    g.a_pack = 1;
    // with H % 8 == 0 the products read k-interleaved activations (contiguous 16-byte loads instead of 16 bytes from
    // each of 32 lines per half-wave): h_t is re-laid-out once for both products, the context is written that way
    const bool bp = H % 8 == 0;
    if (bp && !h_packed) {
      rc = zr_pack4_x_launch(ctx, d_h_t, H, mb, H, a->d_hpack);
      if (rc) return rc;
    }
    if (bp && ctx->attn_single != 1) {
      int took = 0;
      rc = zr_attn_step_single_launch(ctx, a, d_batch_info, d_mask01, d_htild, d_htild_pack, align, idx, pt, cctx, &took);
      if (rc) return rc;
      if (took) {
        ctx->last_attn_path = ZR_ATTN_PATH_SINGLE_LAUNCH;
        return ZR_OK;
      }
    }
    ctx->last_attn_path = ZR_ATTN_PATH_THREE_LAUNCHES;
    g.B[0] = bp ? a->d_hpack : d_h_t;
    g.b_packed = bp ? 1 : 0;
    g.ldb[0] = H;
    g.C = a->d_tanh1;
    g.ldc = H;
    g.batch = 2;
    g.strideA = (long long)per;
    g.strideC = (long long)H * mb;
    g.epilogue = ZR_EPI_STORE;
    rc = zr_gemm_launch(ctx, g);
    if (rc) return rc;
    // (2) p_t, window, scores, alignment weights and context, one workgroup per column
    rc = launch_attn_middle(ctx, a, d_batch_info, d_mask01, pt, idx, align, cctx, bp ? a->d_cpack : nullptr);
    if (rc) return rc;
    // (3) h~ = tanh(W_c1 c + W_c2 h + b) * mask
    ZrGemmDesc o = {};
    o.M = H;
    o.N = mb;
    o.a_pack = 1;
    o.A[0] = a->d_pack32 + 2 * per;
    o.lda[0] = o.lda[1] = a->ldp32;
    if (bp) {
      // one K loop of 2H over [W_c1 | W_c2] and [c; h_t] (H % 8 == 0: no padding between the halves of either operand),
      // so the second half's operands are already on their way while the first half is multiplied
      o.nseg = 1;
      o.K[0] = 2 * H;
      o.B[0] = a->d_cpack;
      o.b_packed = 1;
      o.ldb[0] = 2 * H;
    } else {
      o.nseg = 2;
      o.K[0] = o.K[1] = H;
      o.A[1] = a->d_pack32 + 3 * per;
      o.B[0] = cctx;
      o.B[1] = d_h_t;
      o.ldb[0] = o.ldb[1] = H;
    }
    o.C = d_htild;
    o.Cpack = bp ? d_htild_pack : nullptr;
    o.ldc = H;
    o.batch = 1;
    o.bias = a->out_bias;
    o.mask = d_mask01;
    o.epilogue = ZR_EPI_TANH_BIAS_MASK;
    return zr_gemm_launch(ctx, o);
  }

  ctx->last_attn_path = ZR_ATTN_PATH_SEPARATE;
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
  // bf16 weights: h_t enters three products (W_p, W_a^T, W_c2); it is split into its bf16 terms once, here
  const unsigned short* h_hi = nullptr;
  const unsigned short* h_lo = nullptr;
  if (a->d_bf16 && (((uintptr_t)d_h_t & 15u) == 0)) {
    unsigned short* hs = a->d_bf16 + 4 * per;
    const bool two_terms = ctx->bf16_terms != 1;
    if (!h_packed) {  // (h_packed: the producer of h_t has left the terms there already)
      rc = zr_split_pack_x_launch(ctx, d_h_t, H, mb, H, hs, two_terms ? hs + (size_t)H * mb : nullptr);
      if (rc) return rc;
    }
    h_hi = hs;
    h_lo = two_terms ? hs + (size_t)H * mb : nullptr;
    g.Bhi[0] = h_hi;
    g.Blo[0] = h_lo;
  }
  g.C = a->d_tanh1;
  g.ldc = H;
  g.batch = 1;
  // With 16-byte loads available the window, scores, alignment weights and context are one launch (which applies the
  // tanh itself) instead of four: bf16 weights, or matrices not registered with zr_attn_prepare.
  const bool vec = (H % 4 == 0) && a->tables_aligned && ((((uintptr_t)cctx | (uintptr_t)a->v_p) & 15u) == 0);
  g.epilogue = vec ? ZR_EPI_STORE : ZR_EPI_TANH;
  // bf16 snapshots with the fused middle: W_p h and q = W_a^T h as one batch of two products (the snapshots of W_p and
  // of W_a^T are neighbours, and so are d_tanh1 and d_q), each of which alone would leave half the chip idle
  const bool both = vec && a->d_bf16 && mb > 32 && H < 8192 && a->d_q == a->d_tanh1 + (size_t)H * mb && per % 8 == 0;
  if (both) {
    g.batch = 2;
    g.strideA = (long long)per;
    g.strideC = (long long)H * mb;
  }
  rc = zr_gemm_launch(ctx, g);
  if (rc) return rc;
  // with bf16 matrices the fused middle also leaves the context as bf16 terms for the output product
  unsigned short* c_hi = nullptr;
  unsigned short* c_lo = nullptr;
  if (vec && h_hi && H % 8 == 0) {
    c_hi = a->d_bf16 + 4 * per + 2 * (size_t)H * mb;
    c_lo = h_lo ? c_hi + (size_t)H * mb : nullptr;
  }
  if (both) {
    rc = launch_attn_middle(ctx, a, d_batch_info, d_mask01, pt, idx, align, cctx, nullptr, c_hi, c_lo);
    if (rc) return rc;
  } else {
    if (!vec) {
      attn_window_kernel<<<mb, 64, 0, ctx->stream>>>(a->d_tanh1, a->v_p, d_batch_info, d_mask01, H, mb, D, pt, idx);
      ZR_LAUNCH_CHECK("attn_window_kernel");
    }
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
    if (vec) {
      rc = launch_attn_middle(ctx, a, d_batch_info, d_mask01, pt, idx, align, cctx, nullptr, c_hi, c_lo);
      if (rc) return rc;
    } else {
      const long long slots = (long long)mb * W;
      const unsigned sgrid = (unsigned)((slots + 3) / 4);
      attn_score_kernel<false><<<sgrid, 256, 0, ctx->stream>>>(a->d_table, a->longest_sent, a->d_q, idx, d_batch_info, H,
                                                               mb, W, align, ctx->d_flags);
      ZR_LAUNCH_CHECK("attn_score_kernel");
      const float sigma_sq = (float)((D * D) / 4.0);  // attention_node.hpp:50
      attn_align_kernel<<<mb, 64, 0, ctx->stream>>>(align, idx, pt, mb, W, sigma_sq);
      ZR_LAUNCH_CHECK("attn_align_kernel");
      dim3 cg((H + 63) / 64, mb);
      attn_context_kernel<false><<<cg, 64, 0, ctx->stream>>>(a->d_table, a->longest_sent, align, idx, d_batch_info, H, mb,
                                                             W, cctx);
      ZR_LAUNCH_CHECK("attn_context_kernel");
    }
  }
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
  o.Bhi[0] = c_hi;
  o.Blo[0] = c_lo;
  o.Bhi[1] = h_hi;
  o.Blo[1] = h_lo;
  o.C = d_htild;
  o.ldc = H;
  o.batch = 1;
  o.bias = a->out_bias;
  o.mask = d_mask01;
  o.epilogue = ZR_EPI_TANH_BIAS_MASK;
  if (c_hi) {  // bf16 matrices: h~ also as bf16 terms, for a bf16 output layer behind this step
    o.Chi = a->d_bf16 + 4 * per + 4 * (size_t)H * mb;
    o.Clo = c_lo ? o.Chi + (size_t)H * mb : nullptr;
    a->htild_hi = o.Chi;
    a->htild_lo = o.Clo;
  }
  return zr_gemm_launch(ctx, o);
}

}  // extern "C"
