// Beam search bookkeeping on the device (reference: decoder<dType>, src/decoder.h:162-1502, non-FSA path).
//
// The reference copies the V x beam probability matrix to the host every step and scans it there with two
// std::priority_queues.  Here the scan is a per-column top-(beam+1) selection that reads the probabilities
// once from HBM, and the cross-column merge, hypothesis bookkeeping and back-pointers stay on the device, so
// a decode step moves no V-sized data over PCIe.  n_sent independent sentences are decoded side by side;
// columns [s*beam, (s+1)*beam) belong to sentence s and never interact with another sentence's columns.
//
// Ordering rules (equal to the reference's for tie-free inputs):
//   per column: the beam+1 most probable words (src/decoder.h:1199-1212); equal probabilities rank by lower
//               word id first
//   per sentence: candidates ranked by logf(p) + score of their column (:1214-1219), equal values by
//               (column, rank within column); <START> = 0 is skipped, <EOF> = 1 finishes a hypothesis without
//               taking a beam slot (:1255-1297); step 0 looks at column 0 only (:1182-1184)
// With exactly tied values the reference's order is whatever libstdc++'s heap produces; that order is not
// reproduced.
#include <math.h>

#include "zr_internal.h"

struct zr_beam {
  int beam, vocab, n_sent, max_len, hyp_cap;
  float penalty;
  int current_index;        // host copy; the reference's decoder::current_index
  // device state, per sentence
  float* d_scores;          // [n_sent][beam]
  float* d_scores_tmp;
  int* d_words;             // [n_sent][beam] current_indices (-1 = dead slot)
  int* d_sent;              // [n_sent][beam][max_len] top_sentences
  int* d_sent_tmp;
  int* d_hyp_words;         // [n_sent][hyp_cap][max_len]
  int* d_hyp_len;           // [n_sent][hyp_cap]
  float* d_hyp_score;       // [n_sent][hyp_cap]
  int* d_hyp_count;         // [n_sent]
  // per step scratch
  float* d_cand_p;          // [n_sent*beam][beam+1]
  int* d_cand_w;            // [n_sent*beam][beam+1]
  float* d_part_p;          // [n_sent*beam][kChunks][beam+1] per-chunk candidates
  int* d_part_w;
  void* d_block;            // the single allocation behind all of the above
};

namespace {

constexpr int KMAX = 32;  // beam + 1 <= KMAX

// Per-column top-K in two stages.
// Stage 1 (beam_topk_kernel): grid (kChunks, columns).  A workgroup scans its quarter of the column with 16-byte
// loads; each thread keeps the K best of its share in registers (sorted, descending; bubble insertion with
// static indexing, guarded by the thread's current K-th best so the common case is one compare), then K rounds
// of workgroup arg-max over the thread heads emit the chunk's K best in descending order.
// Stage 2 (beam_topk_merge_kernel): one wave per column merges the kChunks sorted lists.
// Order everywhere: larger probability first, equal probabilities by lower word id.
constexpr int kChunks = 4;

__device__ __forceinline__ bool better(float pa, int wa, float pb, int wb) { return pa > pb || (pa == pb && wa < wb); }

__global__ void __launch_bounds__(256)
beam_topk_kernel(const float* __restrict__ prob, int V, int K, float* __restrict__ part_p, int* __restrict__ part_w) {
  __shared__ float s_p[4];
  __shared__ int s_w[4];
  const int chunk = blockIdx.x;
  const int col = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const float* p = prob + (size_t)col * V;
  // chunk boundaries are multiples of 4 elements so that 16-byte loads stay aligned when V % 4 == 0
  const int per = (((V + kChunks - 1) / kChunks) + 3) & ~3;
  const int v_begin = chunk * per;
  const int v_end = (v_begin + per < V) ? v_begin + per : V;
  float lp[KMAX];
  int lw[KMAX];
#pragma unroll
  for (int i = 0; i < KMAX; ++i) {
    lp[i] = -INFINITY;
    lw[i] = 0x7fffffff;
  }
  float kth = -INFINITY;  // this thread's current K-th best
  auto insert = [&](float x, int xw) {
    // strict comparison: an equal, earlier (lower id) entry stays in front
#pragma unroll
    for (int i = 0; i < KMAX; ++i) {
      if (i < K) {
        const bool sw = x > lp[i];
        const float tp = lp[i];
        const int tw = lw[i];
        lp[i] = sw ? x : tp;
        lw[i] = sw ? xw : tw;
        x = sw ? tp : x;
        xw = sw ? tw : xw;
      }
    }
#pragma unroll
    for (int i = 0; i < KMAX; ++i)
      if (i == K - 1) kth = lp[i];
  };
  const bool vec = ((V & 3) == 0) && ((((uintptr_t)prob) & 15u) == 0);
  if (vec) {
    for (int v = v_begin + 4 * tid; v < v_end; v += 4 * 256) {
      const zr_f32x4 q = *(const zr_f32x4*)(p + v);
      if (q.x > kth) insert(q.x, v);
      if (q.y > kth) insert(q.y, v + 1);
      if (q.z > kth) insert(q.z, v + 2);
      if (q.w > kth) insert(q.w, v + 3);
    }
  } else {
    for (int v = v_begin + tid; v < v_end; v += 256) {
      const float x = p[v];
      if (x > kth) insert(x, v);
    }
  }
  int head = 0;  // index of this thread's best unconsumed entry
  for (int r = 0; r < K; ++r) {
    float hp = -INFINITY;
    int hw = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < KMAX; ++i)
      if (i == head) {
        hp = lp[i];
        hw = lw[i];
      }
    float bp = hp;
    int bw = hw;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float op = __shfl_xor(bp, off, 64);
      const int ow = __shfl_xor(bw, off, 64);
      if (better(op, ow, bp, bw)) {
        bp = op;
        bw = ow;
      }
    }
    if (lane == 0) {
      s_p[wave] = bp;
      s_w[wave] = bw;
    }
    __syncthreads();
    float gp = s_p[0];
    int gw = s_w[0];
#pragma unroll
    for (int w = 1; w < 4; ++w)
      if (better(s_p[w], s_w[w], gp, gw)) {
        gp = s_p[w];
        gw = s_w[w];
      }
    if (hw == gw && gw != 0x7fffffff) head++;  // word ids are unique: exactly one owner
    if (tid == 0) {
      part_p[((size_t)col * kChunks + chunk) * K + r] = gp;
      part_w[((size_t)col * kChunks + chunk) * K + r] = gw;
    }
    __syncthreads();
  }
}

__global__ void __launch_bounds__(64)
beam_topk_merge_kernel(const float* __restrict__ part_p, const int* __restrict__ part_w, int K,
                       float* __restrict__ cand_p, int* __restrict__ cand_w) {
  const int col = blockIdx.x;
  const int lane = threadIdx.x;
  const int n = kChunks * K;  // <= 128: two entries per lane
  float p0 = -INFINITY, p1 = -INFINITY;
  int w0 = 0x7fffffff, w1 = 0x7fffffff;
  if (lane < n) {
    p0 = part_p[(size_t)col * n + lane];
    w0 = part_w[(size_t)col * n + lane];
  }
  if (lane + 64 < n) {
    p1 = part_p[(size_t)col * n + lane + 64];
    w1 = part_w[(size_t)col * n + lane + 64];
  }
  for (int r = 0; r < K; ++r) {
    float bp = p0;
    int bw = w0;
    if (better(p1, w1, bp, bw)) {
      bp = p1;
      bw = w1;
    }
    const float mine_p = bp;
    const int mine_w = bw;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float op = __shfl_xor(bp, off, 64);
      const int ow = __shfl_xor(bw, off, 64);
      if (better(op, ow, bp, bw)) {
        bp = op;
        bw = ow;
      }
    }
    if (mine_w == bw && bw != 0x7fffffff) {  // the owner retires the winner
      if (w0 == bw) {
        p0 = -INFINITY;
        w0 = 0x7fffffff;
      } else {
        p1 = -INFINITY;
        w1 = 0x7fffffff;
      }
    }
    (void)mine_p;
    if (lane == 0) {
      cand_p[(size_t)col * K + r] = bp;
      cand_w[(size_t)col * K + r] = bw;
    }
  }
}

// Cross-column merge and bookkeeping for one sentence per workgroup (expand_hypothesis_without_fsa,
// src/decoder.h:1214-1315).
__global__ void __launch_bounds__(256)
beam_merge_kernel(int beam, int K, int max_len, int hyp_cap, float penalty, int index, int current_index,
                  const float* __restrict__ cand_p, const int* __restrict__ cand_w, float* scores, float* scores_tmp,
                  int* words, int* sent, int* sent_tmp, int* hyp_words, int* hyp_len, float* hyp_score,
                  int* hyp_count, int* out_words, int* out_backptr) {
  constexpr int MAXC = KMAX * KMAX;
  __shared__ float c_val[MAXC];
  __shared__ int c_col[MAXC];
  __shared__ int c_word[MAXC];
  __shared__ int c_order[MAXC];
  __shared__ int s_ncand;
  __shared__ int s_parent[KMAX];   // parent column of each new beam slot (-1: empty-heap filler)
  __shared__ int s_word[KMAX];
  __shared__ float s_score[KMAX];
  __shared__ int s_fin_parent[MAXC];
  __shared__ float s_fin_score[MAXC];
  __shared__ int s_nfin;
  const int s = blockIdx.x;
  const int tid = threadIdx.x;
  float* sc = scores + (size_t)s * beam;
  int* wd = words + (size_t)s * beam;
  int* st = sent + (size_t)s * beam * max_len;
  int* stt = sent_tmp + (size_t)s * beam * max_len;

  if (tid == 0) {
    // live columns: all of them, or column 0 only at the first step; stop at the first dead slot (:1188-1191)
    int cols = (index == 0) ? 1 : beam;
    int n = 0;
    for (int i = 0; i < cols; ++i) {
      if (wd[i] == -1) break;
      // the reference pops its per-column heap in ascending probability and pushes into the global heap
      for (int r = K - 1; r >= 0; --r) {
        const size_t ci = ((size_t)s * beam + i) * K + r;
        c_val[n] = logf(cand_p[ci]) + sc[i];
        c_col[n] = i;
        c_word[n] = cand_w[ci];
        ++n;
      }
    }
    s_ncand = n;
  }
  __syncthreads();
  const int n = s_ncand;
  // rank = number of candidates that come before this one: larger value first, then (column, better rank)
  for (int a = tid; a < n; a += 256) {
    const float va = c_val[a];
    const int ka = c_col[a] * K + (K - 1 - (a % K));  // (column, rank within column) key
    int rank = 0;
    for (int b = 0; b < n; ++b) {
      const float vb = c_val[b];
      const int kb = c_col[b] * K + (K - 1 - (b % K));
      if (vb > va || (vb == va && kb < ka)) ++rank;
    }
    c_order[rank] = a;
  }
  __syncthreads();
  if (tid == 0) {
    int slot = 0, nfin = 0, pos = 0;
    while (slot < beam) {
      if (pos >= n) {  // global heap empty: filler slots (src/decoder.h:1231-1249)
        s_parent[slot] = -1;
        s_word[slot] = -1;
        s_score[slot] = 0.0f;
        ++slot;
        continue;
      }
      const int a = c_order[pos++];
      const int w = c_word[a];
      if (w == 0) continue;  // <START> never selected
      if (w == 1) {          // <EOF>: finished hypothesis, no beam slot consumed
        s_fin_parent[nfin] = c_col[a];
        s_fin_score[nfin] = c_val[a] + penalty;
        ++nfin;
      } else {
        s_parent[slot] = c_col[a];
        s_word[slot] = w;
        s_score[slot] = c_val[a] + penalty;
        ++slot;
      }
    }
    s_nfin = nfin;
  }
  __syncthreads();
  // finished hypotheses: parent's words [0, current_index+1) then <EOF>
  const int nfin = s_nfin;
  const int base = hyp_count[s];
  for (int f = 0; f < nfin; ++f) {
    const int h = base + f;
    if (h >= hyp_cap) break;
    int* hw = hyp_words + ((size_t)s * hyp_cap + h) * max_len;
    const int* src = st + (size_t)s_fin_parent[f] * max_len;
    for (int c = tid; c < current_index + 2 && c < max_len; c += 256) hw[c] = (c == current_index + 1) ? 1 : src[c];
    if (tid == 0) {
      hyp_len[(size_t)s * hyp_cap + h] = current_index + 2;
      hyp_score[(size_t)s * hyp_cap + h] = s_fin_score[f];
    }
  }
  // new beam rows
  for (int i = 0; i < beam; ++i) {
    const int parent = s_parent[i];
    const int* src = st + (size_t)(parent < 0 ? 0 : parent) * max_len;
    int* dst = stt + (size_t)i * max_len;
    for (int c = tid; c < max_len; c += 256) {
      int v = src[c];
      if (c == current_index + 1) v = (parent < 0) ? 0 : s_word[i];
      dst[c] = v;
    }
  }
  __syncthreads();
  if (tid < beam) {
    const int parent = s_parent[tid];
    scores_tmp[(size_t)s * beam + tid] = s_score[tid];
    out_words[(size_t)s * beam + tid] = s_word[tid];
    out_backptr[(size_t)s * beam + tid] = s * beam + (parent < 0 ? 0 : parent);
  }
  __syncthreads();
  if (tid < beam) {
    sc[tid] = scores_tmp[(size_t)s * beam + tid];
    wd[tid] = s_word[tid];
  }
  if (tid == 0) {
    const int total = base + nfin;
    hyp_count[s] = total;  // may exceed hyp_cap: the host reports the overflow
  }
  for (int c = tid; c < beam * max_len; c += 256) st[c] = stt[c];
}

// finish_current_hypotheses, non-FSA branch (src/decoder.h:672-688)
__global__ void __launch_bounds__(256)
beam_finish_kernel(int beam, int V, int max_len, int hyp_cap, float penalty, int current_index,
                   const float* __restrict__ prob, float* scores, const int* words, int* sent, int* hyp_words,
                   int* hyp_len, float* hyp_score, int* hyp_count) {
  const int s = blockIdx.x;
  const int tid = threadIdx.x;
  int base = hyp_count[s];
  __syncthreads();
  int added = 0;
  for (int i = 0; i < beam; ++i) {
    if (words[(size_t)s * beam + i] == -1) continue;
    int* row = sent + ((size_t)s * beam + i) * max_len;
    const float sc = scores[(size_t)s * beam + i] + logf(prob[((size_t)s * beam + i) * V + 1]) + penalty;
    const int h = base + added;
    if (h < hyp_cap) {
      int* hw = hyp_words + ((size_t)s * hyp_cap + h) * max_len;
      for (int c = tid; c < current_index + 2 && c < max_len; c += 256) hw[c] = (c == current_index + 1) ? 1 : row[c];
      if (tid == 0) {
        hyp_len[(size_t)s * hyp_cap + h] = current_index + 2;
        hyp_score[(size_t)s * hyp_cap + h] = sc;
      }
    }
    __syncthreads();
    if (tid == 0) {
      if (current_index + 1 < max_len) row[current_index + 1] = 1;
      scores[(size_t)s * beam + i] = sc;
    }
    ++added;
  }
  __syncthreads();
  if (tid == 0) hyp_count[s] = base + added;
}

__global__ void beam_init_kernel(int n_sent, int beam, int max_len, float* scores, int* words, int* sent, int* hyp_count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_sent * beam) {
    scores[i] = 0.0f;
    words[i] = 0;  // <START>
  }
  if (i < n_sent) hyp_count[i] = 0;
  for (int c = i; c < n_sent * beam * max_len; c += gridDim.x * blockDim.x) sent[c] = 0;
}

}  // namespace

extern "C" {

int zr_beam_create(zr_ctx* ctx, int beam, int vocab, int n_sent, int max_len, float penalty, zr_beam** out) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(out != nullptr, "zr_beam_create: out is null");
  *out = nullptr;
  ZR_CHECK_ARG(beam >= 1 && beam + 1 <= KMAX, "zr_beam_create: beam = %d not in [1, %d]", beam, KMAX - 1);
  ZR_CHECK_ARG(n_sent * beam <= 65535, "zr_beam_create: more than 65535 columns");
  ZR_CHECK_ARG(vocab > beam + 1 && n_sent >= 1 && max_len >= 3, "zr_beam_create: vocab = %d, n_sent = %d, max_len = %d",
               vocab, n_sent, max_len);
  // the reference caps the beam at floor(sqrt(V)) (src/ensemble_factory.hpp:19-21)
  ZR_CHECK_ARG((long long)beam * beam <= vocab, "zr_beam_create: beam %d exceeds sqrt(vocab %d)", beam, vocab);
  zr_beam* b = new zr_beam();
  b->beam = beam;
  b->vocab = vocab;
  b->n_sent = n_sent;
  b->max_len = max_len;
  b->penalty = penalty;
  b->current_index = 0;
  b->hyp_cap = 2 * beam * max_len;
  const size_t nb = (size_t)n_sent * beam, K = beam + 1;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    const size_t o = off;
    off += (bytes + 255) & ~(size_t)255;
    return o;
  };
  const size_t o_scores = take(nb * 4), o_scores_tmp = take(nb * 4), o_words = take(nb * 4);
  const size_t o_sent = take(nb * max_len * 4), o_sent_tmp = take(nb * max_len * 4);
  const size_t o_hw = take((size_t)n_sent * b->hyp_cap * max_len * 4), o_hl = take((size_t)n_sent * b->hyp_cap * 4);
  const size_t o_hs = take((size_t)n_sent * b->hyp_cap * 4), o_hc = take((size_t)n_sent * 4);
  const size_t o_cp = take(nb * K * 4), o_cw = take(nb * K * 4);
  const size_t o_pp = take(nb * 4 * K * 4), o_pw = take(nb * 4 * K * 4);  // kChunks = 4 lists per column
  char* base = nullptr;
  if (hipMalloc((void**)&base, off) != hipSuccess) {
    (void)hipGetLastError();
    delete b;
    return zr_set_error(ZR_ENOMEM, "zr_beam_create: allocation of %zu bytes failed", off);
  }
  b->d_block = base;
  b->d_scores = (float*)(base + o_scores);
  b->d_scores_tmp = (float*)(base + o_scores_tmp);
  b->d_words = (int*)(base + o_words);
  b->d_sent = (int*)(base + o_sent);
  b->d_sent_tmp = (int*)(base + o_sent_tmp);
  b->d_hyp_words = (int*)(base + o_hw);
  b->d_hyp_len = (int*)(base + o_hl);
  b->d_hyp_score = (float*)(base + o_hs);
  b->d_hyp_count = (int*)(base + o_hc);
  b->d_cand_p = (float*)(base + o_cp);
  b->d_cand_w = (int*)(base + o_cw);
  b->d_part_p = (float*)(base + o_pp);
  b->d_part_w = (int*)(base + o_pw);
  *out = b;
  return zr_beam_init(ctx, b);
}

int zr_beam_destroy(zr_ctx* ctx, zr_beam* b) {
  if (!b) return ZR_OK;
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  (void)hipFree(b->d_block);
  delete b;
  return ZR_OK;
}

int zr_beam_init(zr_ctx* ctx, zr_beam* b) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b != nullptr, "zr_beam_init: beam object is null");
  b->current_index = 0;
  beam_init_kernel<<<256, 256, 0, ctx->stream>>>(b->n_sent, b->beam, b->max_len, b->d_scores, b->d_words, b->d_sent,
                                                b->d_hyp_count);
  ZR_LAUNCH_CHECK("beam_init_kernel");
  return ZR_OK;
}

int zr_beam_expand(zr_ctx* ctx, zr_beam* b, const float* d_prob, int index, int* d_words, int* d_backptr) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b && d_prob && d_words && d_backptr, "zr_beam_expand: null pointer");
  ZR_CHECK_ARG(index >= 0, "zr_beam_expand: index = %d", index);
  ZR_CHECK_ARG(b->current_index + 2 < b->max_len, "zr_beam_expand: hypotheses reached max_len = %d", b->max_len);
  const int K = b->beam + 1;
  dim3 tgrid(kChunks, b->n_sent * b->beam);
  beam_topk_kernel<<<tgrid, 256, 0, ctx->stream>>>(d_prob, b->vocab, K, b->d_part_p, b->d_part_w);
  ZR_LAUNCH_CHECK("beam_topk_kernel");
  beam_topk_merge_kernel<<<b->n_sent * b->beam, 64, 0, ctx->stream>>>(b->d_part_p, b->d_part_w, K, b->d_cand_p,
                                                                      b->d_cand_w);
  ZR_LAUNCH_CHECK("beam_topk_merge_kernel");
  beam_merge_kernel<<<b->n_sent, 256, 0, ctx->stream>>>(b->beam, K, b->max_len, b->hyp_cap, b->penalty, index,
                                                        b->current_index, b->d_cand_p, b->d_cand_w, b->d_scores,
                                                        b->d_scores_tmp, b->d_words, b->d_sent, b->d_sent_tmp,
                                                        b->d_hyp_words, b->d_hyp_len, b->d_hyp_score, b->d_hyp_count,
                                                        d_words, d_backptr);
  ZR_LAUNCH_CHECK("beam_merge_kernel");
  b->current_index += 1;
  return ZR_OK;
}

int zr_beam_finish(zr_ctx* ctx, zr_beam* b, const float* d_prob) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b && d_prob, "zr_beam_finish: null pointer");
  beam_finish_kernel<<<b->n_sent, 256, 0, ctx->stream>>>(b->beam, b->vocab, b->max_len, b->hyp_cap, b->penalty,
                                                         b->current_index, d_prob, b->d_scores, b->d_words, b->d_sent,
                                                         b->d_hyp_words, b->d_hyp_len, b->d_hyp_score, b->d_hyp_count);
  ZR_LAUNCH_CHECK("beam_finish_kernel");
  b->current_index += 1;
  return ZR_OK;
}

int zr_beam_hypotheses(zr_ctx* ctx, zr_beam* b, int sentence, int cap, int* h_words, int* h_len, float* h_score) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b && sentence >= 0 && sentence < b->n_sent && cap >= 0, "zr_beam_hypotheses: bad argument");
  int count = 0;
  ZR_HIP(hipMemcpyAsync(&count, b->d_hyp_count + sentence, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  if (count > b->hyp_cap)
    return zr_set_error(ZR_EDATA, "zr_beam_hypotheses: %d finished hypotheses exceed the capacity %d", count, b->hyp_cap);
  const int n = count < cap ? count : cap;
  if (n > 0) {
    ZR_CHECK_ARG(h_words && h_len && h_score, "zr_beam_hypotheses: null output");
    ZR_HIP(hipMemcpyAsync(h_words, b->d_hyp_words + (size_t)sentence * b->hyp_cap * b->max_len,
                          sizeof(int) * (size_t)n * b->max_len, hipMemcpyDeviceToHost, ctx->stream));
    ZR_HIP(hipMemcpyAsync(h_len, b->d_hyp_len + (size_t)sentence * b->hyp_cap, sizeof(int) * n, hipMemcpyDeviceToHost,
                          ctx->stream));
    ZR_HIP(hipMemcpyAsync(h_score, b->d_hyp_score + (size_t)sentence * b->hyp_cap, sizeof(float) * n,
                          hipMemcpyDeviceToHost, ctx->stream));
    ZR_HIP(hipStreamSynchronize(ctx->stream));
  }
  return count;
}

int zr_beam_state(zr_ctx* ctx, zr_beam* b, int sentence, float* h_scores, int* h_words) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b && sentence >= 0 && sentence < b->n_sent && h_scores && h_words, "zr_beam_state: bad argument");
  ZR_HIP(hipMemcpyAsync(h_scores, b->d_scores + (size_t)sentence * b->beam, sizeof(float) * b->beam,
                        hipMemcpyDeviceToHost, ctx->stream));
  ZR_HIP(hipMemcpyAsync(h_words, b->d_words + (size_t)sentence * b->beam, sizeof(int) * b->beam, hipMemcpyDeviceToHost,
                        ctx->stream));
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  return ZR_OK;
}

}  // extern "C"
