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
#include "zr_softmax_fold.h"

struct zr_beam {
  int beam, vocab, n_sent, max_len, hyp_cap;
  float penalty;
  int current_index;        // host copy; the reference's decoder::current_index
  // device state, per sentence
  float* d_scores;          // [n_sent][beam]
  int* d_words;             // [n_sent][beam] current_indices (-1 = dead slot)
  int* d_sent;              // [n_sent][beam][max_len] top_sentences
  int* d_sent_tmp;
  int* d_hyp_words;         // [n_sent][hyp_cap][max_len]
  int* d_hyp_len;           // [n_sent][hyp_cap]
  float* d_hyp_score;       // [n_sent][hyp_cap]
  int* d_hyp_count;         // [n_sent]
  // Viterbi alignments carried with the words (decoder::top_sentences_viterbi, src/decoder.h:230-231), in use once
  // zr_beam_set_viterbi has switched them on
  int* d_vit;               // [n_sent][beam][max_len]
  int* d_vit_tmp;
  int* d_hyp_vit;           // [n_sent][hyp_cap][max_len]
  int track_viterbi;        // 0: the three arrays above are not touched
  const int* d_viterbi_in;  // alignment of every column for the next expand / finish call (null: -1)
  int* d_words_nn_out;      // zr_beam_set_input_ids: every expand call also writes max(word, 0) per slot here (null: no)
  // per step scratch
  float* d_cand_p;          // [n_sent*beam][beam+1]
  int* d_cand_w;            // [n_sent*beam][beam+1]
  float* d_part_p;          // [n_sent*beam][chunks][beam+1] per-chunk candidates of the first top-K stage
  int* d_part_w;
  float* d_colstats;        // [n_sent*beam][2] column statistics the selection on blocks leaves for zr_beam_finish_blocks
  void* d_block;            // the single allocation behind all of the above
};

namespace {

constexpr int KMAX = 32;  // beam + 1 <= KMAX

// Per-column top-K in two stages, both built on one total order: key = (probability as an order-preserving 32-bit
// pattern) << 32 | (0x7fffffff - word id).  Larger key = larger probability, equal probabilities by lower word id;
// keys of distinct words are distinct, so there are no ties to break anywhere.  Key 0 marks "no element" (a NaN
// probability is treated the same way and is never selected).
//
// Stage 1 (beam_topk_kernel): grid (chunks, columns).  A workgroup takes up to kTopkChunk consecutive words of a
// column into registers with 16-byte loads (one pass over HBM, no value-dependent work per element).  The K-th
// largest of a set of per-thread maxima, tau, is a lower bound of the chunk's K-th largest key, so the chunk's K best
// are among the elements with key >= tau; those are appended to a list in LDS.  tau is first taken per wave on the
// probabilities alone (a cross-lane sort of the 64 thread maxima) and the largest of the four used; should the list
// overflow, tau is recomputed over all 256 maxima as full keys: then at most K-1 threads have a maximum above tau, each
// holds 4*E4 elements, and one thread's maximum equals tau, so the list cannot exceed (K-1)*4*E4 + 1 entries whatever
// the data.  Each listed element then counts the
// listed keys above its own: that count is its rank, and ranks below K are written out in place.
// Stage 2 (beam_topk_merge_kernel): one workgroup per column ranks the chunks' K-lists the same way.
// Words per workgroup = 1024 * E4 (E4 16-byte loads per thread).  8192-word chunks measured best at 192 columns of
// 50 000 words (12.9 us against 14.2 with 16384 and 18.6 with 4096: every workgroup of the launch is resident at once
// and they load, then select, in step, so what counts is the length of one workgroup's chain of phases);
// vocabularies beyond kMaxChunks small chunks take the large ones.
constexpr int kTopkE4Small = 8, kTopkE4Large = 16;
constexpr int kMaxChunks = 64;                     // K-lists per column the merge stage holds
constexpr int topk_chunk(int e4) { return 256 * 4 * e4; }
constexpr int topk_cap(int e4) { return (KMAX - 1) * 4 * e4 + 64; }  // candidate list capacity
inline int topk_e4_for(int vocab) { return vocab > kMaxChunks * topk_chunk(kTopkE4Small) ? kTopkE4Large : kTopkE4Small; }

__device__ __forceinline__ unsigned long long topk_key(float p, int w) {
  unsigned u = __float_as_uint(p);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  if (p != p) return 0ull;
  return ((unsigned long long)u << 32) | (unsigned)(0x7fffffff - w);
}
__device__ __forceinline__ void topk_unkey(unsigned long long key, float& p, int& w) {
  if (key == 0ull) {
    p = -INFINITY;
    w = 0x7fffffff;
    return;
  }
  unsigned u = (unsigned)(key >> 32);
  u = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
  p = __uint_as_float(u);
  w = 0x7fffffff - (int)(unsigned)(key & 0xffffffffu);
}

// colstats (or null: the values are probabilities): the values are logits, and (max, sum of exp(x - max)) of the column
// turns a logit into the probability the full normalisation would write, exp(x - max) / sum (src/custom_kernels.h:
// 574-576).  The bound tau is then taken on the logits (the map is monotonic), but the candidates are keyed and ranked
// by that PROBABILITY: two logits a few ulp apart can round to one probability, and the reference, which only ever sees
// the probabilities, ranks such a pair by its tie rule, not by the logits.  So that every word whose probability could
// equal a listed one is listed too, the bound is lowered by a few ulp of the operands of x - max first.
template <int kTopkE4>
__global__ void __launch_bounds__(256)
beam_topk_kernel(const float* __restrict__ prob, int V, int K, int n_chunks, float* __restrict__ part_p,
                 int* __restrict__ part_w, const float* __restrict__ colstats) {
  constexpr int kTopkChunk = topk_chunk(kTopkE4), kTopkCap = topk_cap(kTopkE4);
  __shared__ unsigned long long s_max[256];
  __shared__ unsigned long long s_cand[kTopkCap];
  __shared__ unsigned long long s_tau_wave[4];
  __shared__ unsigned long long s_tau;
  __shared__ int s_count;
  const int chunk = blockIdx.x;
  const int col = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const float* p = prob + (size_t)col * V;
  const bool as_logits = colstats != nullptr;
  const float c_max = as_logits ? colstats[2 * col] : 0.0f, c_sum = as_logits ? colstats[2 * col + 1] : 1.0f;
  const int v_begin = chunk * kTopkChunk;
  const int v_end = (v_begin + kTopkChunk < V) ? v_begin + kTopkChunk : V;
  if (tid == 0) s_count = 0;
  // element e = 4*i + c of this thread is word v_begin + 4*(tid + 256*i) + c; words past the end read as -inf,
  // and -inf (like NaN) is never selected
  float x[4 * kTopkE4];
  const bool vec = ((V & 3) == 0) && ((((uintptr_t)prob) & 15u) == 0);
#pragma unroll
  for (int i = 0; i < kTopkE4; ++i) {
    const int v = v_begin + 4 * (tid + 256 * i);
    if (vec) {
      const bool ok = v + 3 < v_end;
      const zr_f32x4 q = *(const zr_f32x4*)(p + (ok ? v : 0));
      x[4 * i] = ok ? q.x : -INFINITY;
      x[4 * i + 1] = ok ? q.y : -INFINITY;
      x[4 * i + 2] = ok ? q.z : -INFINITY;
      x[4 * i + 3] = ok ? q.w : -INFINITY;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float q = p[v + c < v_end ? v + c : 0];
        x[4 * i + c] = v + c < v_end ? q : -INFINITY;
      }
    }
  }
  // The kernel is bound by vector instructions, not by memory: everything per element is kept to a compare or less.
  // This thread's largest probability (NaN never wins a maximum), as an order-preserving 32-bit pattern; 0 = none.
  float bm = -INFINITY;
#pragma unroll
  for (int i = 0; i < kTopkE4; ++i) bm = fmaxf(bm, fmaxf(fmaxf(x[4 * i], x[4 * i + 1]), fmaxf(x[4 * i + 2], x[4 * i + 3])));
  const unsigned mu = bm > -INFINITY ? (unsigned)(topk_key(bm, 0) >> 32) : 0u;
  // First bound, on the probabilities alone: the K-th largest thread maximum inside each wave (a bitonic sort of the
  // 64 lanes' values, 21 exchange steps), then the largest of the four waves' bounds.  The K-th largest of any set of
  // group maxima is a lower bound of the chunk's K-th largest element, so everything at or above it is listed -- with
  // equal probabilities around the bound that is a few more elements than the exact rule needs, and if the list
  // overflows the exact bound below takes over.
  {
    unsigned v = mu;
#pragma unroll
    for (int k = 2; k <= 64; k <<= 1)
#pragma unroll
      for (int j = k >> 1; j > 0; j >>= 1) {
        const unsigned o = (unsigned)__shfl_xor((int)v, j, 64);
        const bool keep_max = ((lane & j) == 0) == ((lane & k) == 0);
        v = keep_max ? (v > o ? v : o) : (v < o ? v : o);
      }
    if (lane == K - 1) s_tau_wave[wave] = (unsigned long long)v << 32;  // lowest key of that probability
  }
  __syncthreads();
  unsigned long long tau = s_tau_wave[0];
#pragma unroll
  for (int w = 1; w < 4; ++w) tau = s_tau_wave[w] > tau ? s_tau_wave[w] : tau;
  auto collect = [&](unsigned long long t, bool widen) {
    float tp;
    int tw;
    topk_unkey(t, tp, tw);
    if (as_logits && widen) {
      tp -= 1e-6f + 5e-7f * (fabsf(tp) + fabsf(c_max));  // (see above; an infinite bound stays what it is)
      tw = 0x7fffffff;
    }
    if (bm >= tp && mu != 0u) {
#pragma unroll
      for (int i = 0; i < kTopkE4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const float q = x[4 * i + c];
          if (q >= tp) {  // rare: the full test and the append sit behind one comparison per element
            const int v = v_begin + 4 * (tid + 256 * i) + c;
            if (q > -INFINITY && (q > tp || v <= tw)) {
              const int pos = atomicAdd(&s_count, 1);
              if (pos < kTopkCap) s_cand[pos] = topk_key(as_logits ? expf(q - c_max) / c_sum : q, v);
            }
          }
        }
    }
  };
  collect(tau, true);
  __syncthreads();
  if (s_count > kTopkCap) {
    // The wave-level bound let too many elements through (several waves holding threads whose whole share is large, or
    // many equal probabilities at the bound).  The K-th largest of all 256 thread maxima as full keys (probability,
    // then lower word id) bounds the list by (K-1) * 4*kTopkE4 + 1 entries whatever the data.
    int bv = 0x7fffffff;
#pragma unroll
    for (int i = kTopkE4 - 1; i >= 0; --i)
#pragma unroll
      for (int c = 3; c >= 0; --c)
        if (x[4 * i + c] == bm) bv = v_begin + 4 * (tid + 256 * i) + c;  // descending scan: the lowest id stays
    const unsigned long long mine = mu != 0u ? topk_key(bm, bv) : 0ull;
    s_max[tid] = mine;
    __syncthreads();
    int rank = 0;
    for (int j = 0; j < 256; ++j) {
      const unsigned long long o = s_max[j];
      rank += (o > mine || (o == mine && j < tid)) ? 1 : 0;
    }
    if (rank == K - 1) s_tau = mine;
    __syncthreads();
    if (tid == 0) s_count = 0;
    __syncthreads();
    collect(s_tau, false);  // (so many equal values that the list overflowed: the exact bound, on the values as they are)
    __syncthreads();
  }
  const int n = s_count < kTopkCap ? s_count : kTopkCap;
  float* out_p = part_p + ((size_t)col * n_chunks + chunk) * K;
  int* out_w = part_w + ((size_t)col * n_chunks + chunk) * K;
  for (int a = tid; a < n; a += 256) {
    const unsigned long long ka = s_cand[a];
    int rank = 0;
#pragma unroll 8
    for (int b = 0; b < n; ++b) rank += s_cand[b] > ka ? 1 : 0;
    if (rank < K) topk_unkey(ka, out_p[rank], out_w[rank]);
  }
  if (tid < K && tid >= n) {  // fewer than K words in the chunk
    out_p[tid] = -INFINITY;
    out_w[tid] = 0x7fffffff;
  }
}

__global__ void __launch_bounds__(256)
beam_topk_merge_kernel(const float* __restrict__ part_p, const int* __restrict__ part_w, int K, int n_chunks,
                       float* __restrict__ cand_p, int* __restrict__ cand_w) {
  __shared__ unsigned long long s_key[kMaxChunks * KMAX];
  const int col = blockIdx.x;
  const int tid = threadIdx.x;
  const int n = n_chunks * K;
  for (int a = tid; a < n; a += 256)
    s_key[a] = topk_key(part_p[(size_t)col * n + a], part_w[(size_t)col * n + a]);  // (-inf, 0x7fffffff) -> lowest
  __syncthreads();
  for (int a = tid; a < n; a += 256) {
    const unsigned long long ka = s_key[a];
    int rank = 0;
#pragma unroll 8
    for (int b = 0; b < n; ++b) {
      const unsigned long long kb = s_key[b];
      rank += (kb > ka || (kb == ka && b < a)) ? 1 : 0;  // fillers share one key: order them by position
    }
    if (rank < K) {
      cand_p[(size_t)col * K + rank] = part_p[(size_t)col * n + a];
      cand_w[(size_t)col * K + rank] = part_w[(size_t)col * n + a];
    }
  }
}

// Per-column top-K straight from the output product's per-block pairs (ZR_SOFTMAX_LOGITS_BLOCKS): one workgroup per
// column does what softmax_colstats_kernel, beam_topk_kernel and beam_topk_merge_kernel do in three launches, and reads
// of the column's V logits only the 32-row blocks that can hold one of its K largest entries.
//   1. The column's pairs ([nblocks][2], 12.5 KB at 50 000 words) are folded into (max, sum) exactly as
//      softmax_colstats_kernel folds them (zr_softmax_fold.h: the same bits, hence the same probabilities).
//   2. A thread's largest block maximum is the maximum of a group of the column's logits, so the K-th largest of the
//      threads' values (taken per wave, the largest of the four waves' results) is a lower bound of the K-th largest
//      logit; it is lowered by a few ulp as in beam_topk_kernel, so that every word whose PROBABILITY could equal a
//      listed one is listed.
//   3. The blocks whose maximum reaches the bound are listed (a second pass over the pairs, which are in cache), their
//      logits are read, 32 at a time per half-wave, and those at or above the bound go on the candidate list keyed by
//      probability and word id; the list is ranked by counting and the first K written out.
// Either list overflowing (hundreds of blocks within a few ulp of the K-th largest logit: constant columns) sends the
// workgroup down an exact path that needs no bound: K passes over the whole column, each taking the largest key below
// the previous one.  Keys, tie rule and fillers are those of the two-stage selection: the K-lists are the same bit for
// bit.
constexpr int kSelBlockCap = 512;   // candidate blocks per column
constexpr int kSelCandCap = 1024;   // candidate words per column

__global__ void __launch_bounds__(256)
beam_select_blocks_kernel(const float* __restrict__ logits, const float* __restrict__ blocks, int V, int K, int nblocks,
                          float* __restrict__ cand_p, int* __restrict__ cand_w, float* __restrict__ colstats_out) {
  __shared__ float s_m[4], s_s[4];
  __shared__ float s_stats[2];
  __shared__ unsigned s_tau_wave[4];
  __shared__ int s_blk[kSelBlockCap];
  __shared__ unsigned long long s_cand[kSelCandCap];
  __shared__ unsigned long long s_best[4];
  __shared__ int s_nblk, s_count;
  const int col = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const float* x = logits + (size_t)col * V;
  const float* pairs = blocks + (size_t)col * nblocks * 2;
  if (tid == 0) s_nblk = 0, s_count = 0;
  float mx, sum, bm;
  zr_softmax_fold_column(pairs, nblocks, s_m, s_s, mx, sum, &bm);
  if (tid == 0) {
    s_stats[0] = mx;
    s_stats[1] = sum;
    colstats_out[2 * col] = mx;
    colstats_out[2 * col + 1] = sum;
  }
  // the bound: K-th largest thread value inside each wave (bitonic sort of the 64 lanes), largest of the four waves
  {
    unsigned v = bm > -INFINITY ? (unsigned)(topk_key(bm, 0) >> 32) : 0u;
#pragma unroll
    for (int k = 2; k <= 64; k <<= 1)
#pragma unroll
      for (int j = k >> 1; j > 0; j >>= 1) {
        const unsigned o = (unsigned)__shfl_xor((int)v, j, 64);
        const bool keep_max = ((lane & j) == 0) == ((lane & k) == 0);
        v = keep_max ? (v > o ? v : o) : (v < o ? v : o);
      }
    if (lane == K - 1) s_tau_wave[wave] = v;
  }
  __syncthreads();
  const float c_max = s_stats[0], c_sum = s_stats[1];
  unsigned tu = s_tau_wave[0];
#pragma unroll
  for (int w = 1; w < 4; ++w) tu = s_tau_wave[w] > tu ? s_tau_wave[w] : tu;
  float tp;
  {
    int tw;
    topk_unkey((unsigned long long)tu << 32, tp, tw);  // (no thread value at all: -inf, which lists every block)
    tp -= 1e-6f + 5e-7f * (fabsf(tp) + fabsf(c_max));
  }
  // candidate blocks (the maxima again, eight loads in flight per thread)
  for (int b0 = 0; b0 < nblocks; b0 += 2048) {
    float pm[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int b = b0 + tid + 256 * u;
      pm[u] = b < nblocks ? pairs[2 * b] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (pm[u] >= tp && pm[u] > -INFINITY) {
        const int pos = atomicAdd(&s_nblk, 1);
        if (pos < kSelBlockCap) s_blk[pos] = b0 + tid + 256 * u;
      }
    }
  }
  __syncthreads();
  const int nblk = s_nblk;
  bool exact = nblk > kSelBlockCap;
  if (!exact) {
    // candidate words: a half-wave per block
    const int hw = tid >> 5, l32 = tid & 31;
    for (int i = hw; i < nblk; i += 8) {
      const int v = s_blk[i] * 32 + l32;
      const float q = v < V ? x[v] : -INFINITY;
      if (q >= tp && q > -INFINITY) {
        const int pos = atomicAdd(&s_count, 1);
        if (pos < kSelCandCap) s_cand[pos] = topk_key(expf(q - c_max) / c_sum, v);
      }
    }
    __syncthreads();
    exact = s_count > kSelCandCap;
  }
  float* out_p = cand_p + (size_t)col * K;
  int* out_w = cand_w + (size_t)col * K;
  if (exact) {
    // K passes over the column: the largest key below the previous pass's
    unsigned long long prev = ~0ull;
    for (int r = 0; r < K; ++r) {
      unsigned long long best = 0ull;
      for (int v = tid; v < V; v += 256) {
        const float q = x[v];
        const unsigned long long key = q > -INFINITY ? topk_key(expf(q - c_max) / c_sum, v) : 0ull;
        best = (key < prev && key > best) ? key : best;
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(best, off, 64);
        best = o > best ? o : best;
      }
      __syncthreads();  // (s_best of the previous pass has been read)
      if (lane == 0) s_best[wave] = best;
      __syncthreads();
      best = s_best[0];
#pragma unroll
      for (int w = 1; w < 4; ++w) best = s_best[w] > best ? s_best[w] : best;
      if (tid == 0) topk_unkey(best, out_p[r], out_w[r]);  // key 0 (nothing left): the filler (-inf, 0x7fffffff)
      prev = best != 0ull ? best : 0ull;
    }
    return;
  }
  const int n = s_count;
  for (int a = tid; a < n; a += 256) {
    const unsigned long long ka = s_cand[a];
    int rank = 0;
#pragma unroll 8
    for (int b = 0; b < n; ++b) rank += s_cand[b] > ka ? 1 : 0;
    if (rank < K) topk_unkey(ka, out_p[rank], out_w[rank]);
  }
  if (tid < K && tid >= n) {  // fewer than K words in the column
    out_p[tid] = -INFINITY;
    out_w[tid] = 0x7fffffff;
  }
}

// Cross-column merge and bookkeeping for one sentence per workgroup (expand_hypothesis_without_fsa,
// src/decoder.h:1214-1315).
__global__ void __launch_bounds__(256)
beam_merge_kernel(int beam, int K, int max_len, int hyp_cap, float penalty, int index, int current_index,
                  const float* __restrict__ cand_p, const int* __restrict__ cand_w, float* scores,
                  int* words, int* sent, int* sent_tmp, int* hyp_words, int* hyp_len, float* hyp_score,
                  int* hyp_count, int* out_words, int* out_words_nn, int* out_backptr, const int* __restrict__ vit,
                  int* vit_tmp,
                  int* hyp_vit, const int* __restrict__ viterbi_in) {
  constexpr int MAXC = KMAX * KMAX;
  __shared__ float c_val[MAXC];
  __shared__ int c_col[MAXC];
  __shared__ int c_word[MAXC];
  __shared__ int c_order[MAXC];
  // one sortable key per candidate: value (order-preserving bit pattern) above, then (column, rank within column)
  // inverted, so that a larger key comes first and equal values go by (column, better rank)
  __shared__ unsigned long long c_key[MAXC];
  __shared__ int s_ncand;
  __shared__ int s_parent[KMAX];   // parent column of each new beam slot (-1: empty-heap filler)
  __shared__ int s_word[KMAX];
  __shared__ float s_score[KMAX];
  __shared__ int s_fin_parent[MAXC];
  __shared__ float s_fin_score[MAXC];
  __shared__ int s_nfin;
  __shared__ int s_base;  // finished hypotheses of the sentence before this step
  const int s = blockIdx.x;
  const int tid = threadIdx.x;
  float* sc = scores + (size_t)s * beam;
  int* wd = words + (size_t)s * beam;
  int* st = sent + (size_t)s * beam * max_len;
  int* stt = sent_tmp + (size_t)s * beam * max_len;

  // live columns: all of them, or column 0 only at the first step; stop at the first dead slot (:1188-1191)
  if (tid < 64) {  // beam < 64: one ballot over the slots finds the first dead one
    const int all = (index == 0) ? 1 : beam;
    const unsigned long long dead = __ballot(tid < all && wd[tid] == -1);
    if (tid == 0) s_ncand = (dead ? __builtin_ctzll(dead) : all) * K;
  }
  __syncthreads();
  const int live = s_ncand / K;
  // candidate a = i*K + q of live column i: the reference pops its per-column heap in ascending probability and
  // pushes into the global heap, so q counts ranks from the worst (rank K-1) to the best (rank 0)
  for (int a = tid; a < live * K; a += 256) {
    const int i = a / K, r = K - 1 - a % K;
    const size_t ci = ((size_t)s * beam + i) * K + r;
    c_val[a] = logf(cand_p[ci]) + sc[i];
    c_col[a] = i;
    c_word[a] = cand_w[ci];
    unsigned u = __float_as_uint(c_val[a]);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    c_key[a] = ((unsigned long long)u << 32) | (unsigned)(0x7fffffff - (i * K + r));
  }
  __syncthreads();
  const int n = s_ncand;
  // rank = number of candidates that come before this one
  for (int a = tid; a < n; a += 256) {
    const unsigned long long ka = c_key[a];
    int rank = 0;
#pragma unroll 8
    for (int b = 0; b < n; ++b) rank += c_key[b] > ka ? 1 : 0;
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
    // read here, by the thread that updates it at the end, and handed on through shared memory: a wave that came late
    // to a load of its own could otherwise see the updated count
    s_base = hyp_count[s];
  }
  __syncthreads();
  // finished hypotheses: parent's words [0, current_index+1) then <EOF>
  const int nfin = s_nfin;
  const int base = s_base;
  for (int f = 0; f < nfin; ++f) {
    const int h = base + f;
    if (h >= hyp_cap) break;
    int* hw = hyp_words + ((size_t)s * hyp_cap + h) * max_len;
    const int* src = st + (size_t)s_fin_parent[f] * max_len;
    for (int c = tid; c < current_index + 2 && c < max_len; c += 256) hw[c] = (c == current_index + 1) ? 1 : src[c];
    if (vit) {  // the parent's alignments, then the alignment of this step's column (src/decoder.h:1266-1267)
      int* hv = hyp_vit + ((size_t)s * hyp_cap + h) * max_len;
      const int* vsrc = vit + ((size_t)s * beam + s_fin_parent[f]) * max_len;
      const int mine = viterbi_in ? viterbi_in[(size_t)s * beam + s_fin_parent[f]] : -1;
      for (int c = tid; c < current_index + 2 && c < max_len; c += 256) hv[c] = (c == current_index + 1) ? mine : vsrc[c];
    }
    if (tid == 0) {
      hyp_len[(size_t)s * hyp_cap + h] = current_index + 2;
      hyp_score[(size_t)s * hyp_cap + h] = s_fin_score[f];
    }
  }
  // new beam rows into the other sentence buffer (the host swaps the two after the launch): slot i continues its
  // parent's words [0, current_index] with its own word.  One flat loop over (slot, position), so that the loads of
  // all rows are in flight together; positions past current_index + 1 are never read.
  const int lim = current_index + 2 < max_len ? current_index + 2 : max_len;
  for (int e = tid; e < beam * lim; e += 256) {
    const int i = e / lim, c = e % lim;
    const int parent = s_parent[i];
    int v = st[(size_t)(parent < 0 ? 0 : parent) * max_len + c];
    if (c == current_index + 1) v = (parent < 0) ? 0 : s_word[i];
    stt[(size_t)i * max_len + c] = v;
  }
  if (vit) {
    // src/decoder.h:1281-1282; an empty-heap filler slot takes row 0 as it is (:1237)
    const int* vt = vit + (size_t)s * beam * max_len;
    int* vtt = vit_tmp + (size_t)s * beam * max_len;
    for (int e = tid; e < beam * lim; e += 256) {
      const int i = e / lim, c = e % lim;
      const int parent = s_parent[i];
      int v = vt[(size_t)(parent < 0 ? 0 : parent) * max_len + c];
      if (c == current_index + 1 && parent >= 0) v = viterbi_in ? viterbi_in[(size_t)s * beam + parent] : -1;
      vtt[(size_t)i * max_len + c] = v;
    }
  }
  if (tid < beam) {
    const int parent = s_parent[tid];
    out_words[(size_t)s * beam + tid] = s_word[tid];
    if (out_words_nn) out_words_nn[(size_t)s * beam + tid] = s_word[tid] < 0 ? 0 : s_word[tid];
    out_backptr[(size_t)s * beam + tid] = s * beam + (parent < 0 ? 0 : parent);
    sc[tid] = s_score[tid];  // s_score was filled from the old scores before the last barrier
    wd[tid] = s_word[tid];
  }
  if (tid == 0) hyp_count[s] = base + nfin;  // may exceed hyp_cap: the host reports the overflow
}

// finish_current_hypotheses, non-FSA branch (src/decoder.h:672-688)
__global__ void __launch_bounds__(256)
beam_finish_kernel(int beam, int V, int max_len, int hyp_cap, float penalty, int current_index,
                   const float* __restrict__ prob, const float* __restrict__ colstats, float* scores, const int* words,
                   int* sent, int* hyp_words, int* hyp_len, float* hyp_score, int* hyp_count,
                   const int* __restrict__ vit, int* hyp_vit, const int* __restrict__ viterbi_in) {
  const int s = blockIdx.x;
  const int tid = threadIdx.x;
  int base = hyp_count[s];
  __syncthreads();
  int added = 0;
  for (int i = 0; i < beam; ++i) {
    if (words[(size_t)s * beam + i] == -1) continue;
    int* row = sent + ((size_t)s * beam + i) * max_len;
    float p_eof = prob[((size_t)s * beam + i) * V + 1];
    if (colstats) p_eof = expf(p_eof - colstats[2 * (s * beam + i)]) / colstats[2 * (s * beam + i) + 1];  // logits
    const float sc = scores[(size_t)s * beam + i] + logf(p_eof) + penalty;
    const int h = base + added;
    if (h < hyp_cap) {
      int* hw = hyp_words + ((size_t)s * hyp_cap + h) * max_len;
      for (int c = tid; c < current_index + 2 && c < max_len; c += 256) hw[c] = (c == current_index + 1) ? 1 : row[c];
      if (vit) {  // src/decoder.h:683-684
        int* hv = hyp_vit + ((size_t)s * hyp_cap + h) * max_len;
        const int* vrow = vit + ((size_t)s * beam + i) * max_len;
        const int mine = viterbi_in ? viterbi_in[(size_t)s * beam + i] : -1;
        for (int c = tid; c < current_index + 2 && c < max_len; c += 256) hv[c] = (c == current_index + 1) ? mine : vrow[c];
      }
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

// ensemble_factory::ensembles_models (src/ensemble_factory.hpp:767-793): the models' output distributions are averaged
// element by element (summed in double, divided by the number of models) and every column is divided by its sum again.
// Two launches over (chunk of 4096 rows, column) workgroups, so that a few hundred columns still fill the chip: the
// first writes the averages and one partial sum (double) per workgroup; the second adds a column's partials in chunk
// order (every workgroup of the column gets the same total) and divides its chunk.  VEC: 16-byte accesses when the
// columns are 16-byte aligned.
constexpr int kMaxEnsemble = 16;
constexpr int kEnsembleChunk = 4096;
struct EnsembleArgs {
  const float* p[kMaxEnsemble];
};
template <bool VEC>
__global__ void __launch_bounds__(256)
ensemble_mean_kernel(EnsembleArgs a, int n_models, int V, float* out, double* partials) {
  __shared__ double s_sum[256];
  const int chunk = blockIdx.x, col = blockIdx.y, tid = threadIdx.x;
  const size_t base = (size_t)col * V;
  const int v0 = chunk * kEnsembleChunk, v1 = min(V, v0 + kEnsembleChunk);
  const double inv = (double)n_models;
  double sum = 0.0;
  if (VEC) {
    for (int v = v0 + 4 * tid; v < v1; v += 1024) {  // V % 4 == 0: a group of four never straddles v1
      double t[4] = {0.0, 0.0, 0.0, 0.0};
      for (int k = 0; k < n_models; ++k) {
        const float4 x = *(const float4*)(a.p[k] + base + v);
        t[0] += (double)x.x;
        t[1] += (double)x.y;
        t[2] += (double)x.z;
        t[3] += (double)x.w;
      }
      float4 r;
      r.x = (float)(t[0] / inv);
      r.y = (float)(t[1] / inv);
      r.z = (float)(t[2] / inv);
      r.w = (float)(t[3] / inv);
      *(float4*)(out + base + v) = r;
      sum += ((double)r.x + (double)r.y) + ((double)r.z + (double)r.w);
    }
  } else {
    for (int v = v0 + tid; v < v1; v += 256) {
      double t = 0.0;
      for (int k = 0; k < n_models; ++k) t += (double)a.p[k][base + v];
      const float avg = (float)(t / inv);
      out[base + v] = avg;
      sum += (double)avg;
    }
  }
  s_sum[tid] = sum;
  __syncthreads();
  for (int st = 128; st > 0; st >>= 1) {
    if (tid < st) s_sum[tid] += s_sum[tid + st];
    __syncthreads();
  }
  if (tid == 0) partials[(size_t)col * gridDim.x + chunk] = s_sum[0];
}

template <bool VEC>
__global__ void __launch_bounds__(256) ensemble_normalize_kernel(int V, float* out, const double* partials) {
  const int chunk = blockIdx.x, col = blockIdx.y, tid = threadIdx.x;
  double total = 0.0;
  for (int c = 0; c < (int)gridDim.x; ++c) total += partials[(size_t)col * gridDim.x + c];
  const float norm = (float)total;
  const size_t base = (size_t)col * V;
  const int v0 = chunk * kEnsembleChunk, v1 = min(V, v0 + kEnsembleChunk);
  if (VEC) {
    for (int v = v0 + 4 * tid; v < v1; v += 1024) {
      float4 x = *(float4*)(out + base + v);
      x.x = x.x / norm;
      x.y = x.y / norm;
      x.z = x.z / norm;
      x.w = x.w / norm;
      *(float4*)(out + base + v) = x;
    }
  } else {
    for (int v = v0 + tid; v < v1; v += 256) out[base + v] = out[base + v] / norm;
  }
}

__global__ void beam_init_kernel(int n_sent, int beam, int max_len, float* scores, int* words, int* sent, int* hyp_count,
                                 int* vit) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_sent * beam) {
    scores[i] = 0.0f;
    words[i] = 0;  // <START>
  }
  if (i < n_sent) hyp_count[i] = 0;
  for (int c = i; c < n_sent * beam * max_len; c += gridDim.x * blockDim.x) sent[c] = 0;
  if (vit)
    for (int c = i; c < n_sent * beam * max_len; c += gridDim.x * blockDim.x) vit[c] = -20;  // src/decoder.h:1335
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
  ZR_CHECK_ARG(vocab <= kMaxChunks * topk_chunk(kTopkE4Large), "zr_beam_create: vocab = %d exceeds %d", vocab,
               kMaxChunks * topk_chunk(kTopkE4Large));
  const int kTopkChunk = topk_chunk(topk_e4_for(vocab));
  ZR_CHECK_ARG(vocab > beam + 1 && n_sent >= 1 && max_len >= 3, "zr_beam_create: vocab = %d, n_sent = %d, max_len = %d",
               vocab, n_sent, max_len);
  // (the reference's driver caps the beam at floor(sqrt(V)) before it builds its decoder, src/ensemble_factory.hpp:19-21;
  // that is the caller's rule, as there: beam_decoder in host/zoph_model.h applies it)
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
  const size_t o_scores = take(nb * 4), o_words = take(nb * 4);
  const size_t o_sent = take(nb * max_len * 4), o_sent_tmp = take(nb * max_len * 4);
  const size_t o_hw = take((size_t)n_sent * b->hyp_cap * max_len * 4), o_hl = take((size_t)n_sent * b->hyp_cap * 4);
  const size_t o_hs = take((size_t)n_sent * b->hyp_cap * 4), o_hc = take((size_t)n_sent * 4);
  const size_t o_vit = take(nb * max_len * 4), o_vit_tmp = take(nb * max_len * 4);
  const size_t o_hv = take((size_t)n_sent * b->hyp_cap * max_len * 4);
  const size_t o_cp = take(nb * K * 4), o_cw = take(nb * K * 4);
  const size_t n_chunks = ((size_t)vocab + kTopkChunk - 1) / kTopkChunk;  // K-lists per column from the first stage
  const size_t o_pp = take(nb * n_chunks * K * 4), o_pw = take(nb * n_chunks * K * 4);
  const size_t o_cs = take(nb * 2 * 4);
  char* base = nullptr;
  if (hipMalloc((void**)&base, off) != hipSuccess) {
    (void)hipGetLastError();
    delete b;
    return zr_set_error(ZR_ENOMEM, "zr_beam_create: allocation of %zu bytes failed", off);
  }
  b->d_block = base;
  b->d_scores = (float*)(base + o_scores);
  b->d_words = (int*)(base + o_words);
  b->d_sent = (int*)(base + o_sent);
  b->d_sent_tmp = (int*)(base + o_sent_tmp);
  b->d_hyp_words = (int*)(base + o_hw);
  b->d_hyp_len = (int*)(base + o_hl);
  b->d_hyp_score = (float*)(base + o_hs);
  b->d_hyp_count = (int*)(base + o_hc);
  b->d_vit = (int*)(base + o_vit);
  b->d_vit_tmp = (int*)(base + o_vit_tmp);
  b->d_hyp_vit = (int*)(base + o_hv);
  b->track_viterbi = 0;
  b->d_viterbi_in = nullptr;
  b->d_cand_p = (float*)(base + o_cp);
  b->d_cand_w = (int*)(base + o_cw);
  b->d_part_p = (float*)(base + o_pp);
  b->d_part_w = (int*)(base + o_pw);
  b->d_colstats = (float*)(base + o_cs);
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
                                                b->d_hyp_count, b->track_viterbi ? b->d_vit : nullptr);
  ZR_LAUNCH_CHECK("beam_init_kernel");
  return ZR_OK;
}

// d_colstats null: d_values are probabilities; otherwise logits with their column statistics
// d_blocks: the values are logits with their per-block pairs behind them (one fused selection launch)
static int beam_expand_impl(zr_ctx* ctx, const char* who, zr_beam* b, const float* d_values, const float* d_colstats,
                            int index, int* d_words, int* d_backptr, const float* d_blocks = nullptr) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b && d_values && d_words && d_backptr, "%s: null pointer", who);
  ZR_CHECK_ARG(index >= 0, "%s: index = %d", who, index);
  ZR_CHECK_ARG(b->current_index + 2 < b->max_len, "%s: hypotheses reached max_len = %d", who, b->max_len);
  const int K = b->beam + 1;
  if (d_blocks) {
    beam_select_blocks_kernel<<<b->n_sent * b->beam, 256, 0, ctx->stream>>>(d_values, d_blocks, b->vocab, K,
                                                                            zr_softmax_partial_blocks(b->vocab),
                                                                            b->d_cand_p, b->d_cand_w, b->d_colstats);
    ZR_LAUNCH_CHECK("beam_select_blocks_kernel");
  } else {
    const int e4 = topk_e4_for(b->vocab);
    const int n_chunks = (b->vocab + topk_chunk(e4) - 1) / topk_chunk(e4);
    dim3 tgrid(n_chunks, b->n_sent * b->beam);
    if (e4 == kTopkE4Small)
      beam_topk_kernel<kTopkE4Small><<<tgrid, 256, 0, ctx->stream>>>(d_values, b->vocab, K, n_chunks, b->d_part_p,
                                                                     b->d_part_w, d_colstats);
    else
      beam_topk_kernel<kTopkE4Large><<<tgrid, 256, 0, ctx->stream>>>(d_values, b->vocab, K, n_chunks, b->d_part_p,
                                                                     b->d_part_w, d_colstats);
    ZR_LAUNCH_CHECK("beam_topk_kernel");
    beam_topk_merge_kernel<<<b->n_sent * b->beam, 256, 0, ctx->stream>>>(b->d_part_p, b->d_part_w, K, n_chunks,
                                                                         b->d_cand_p, b->d_cand_w);
    ZR_LAUNCH_CHECK("beam_topk_merge_kernel");
  }
  beam_merge_kernel<<<b->n_sent, 256, 0, ctx->stream>>>(b->beam, K, b->max_len, b->hyp_cap, b->penalty, index,
                                                        b->current_index, b->d_cand_p, b->d_cand_w, b->d_scores,
                                                        b->d_words, b->d_sent, b->d_sent_tmp,
                                                        b->d_hyp_words, b->d_hyp_len, b->d_hyp_score, b->d_hyp_count,
                                                        d_words, b->d_words_nn_out, d_backptr,
                                                        b->track_viterbi ? b->d_vit : nullptr,
                                                        b->d_vit_tmp, b->d_hyp_vit, b->d_viterbi_in);
  ZR_LAUNCH_CHECK("beam_merge_kernel");
  int* t = b->d_sent;  // the kernel wrote the new rows into d_sent_tmp
  b->d_sent = b->d_sent_tmp;
  b->d_sent_tmp = t;
  if (b->track_viterbi) {
    t = b->d_vit;
    b->d_vit = b->d_vit_tmp;
    b->d_vit_tmp = t;
  }
  b->current_index += 1;
  return ZR_OK;
}

static int beam_finish_impl(zr_ctx* ctx, const char* who, zr_beam* b, const float* d_values, const float* d_colstats) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b && d_values, "%s: null pointer", who);
  beam_finish_kernel<<<b->n_sent, 256, 0, ctx->stream>>>(b->beam, b->vocab, b->max_len, b->hyp_cap, b->penalty,
                                                         b->current_index, d_values, d_colstats, b->d_scores, b->d_words,
                                                         b->d_sent, b->d_hyp_words, b->d_hyp_len, b->d_hyp_score,
                                                         b->d_hyp_count, b->track_viterbi ? b->d_vit : nullptr,
                                                         b->d_hyp_vit, b->d_viterbi_in);
  ZR_LAUNCH_CHECK("beam_finish_kernel");
  b->current_index += 1;
  return ZR_OK;
}

int zr_beam_expand(zr_ctx* ctx, zr_beam* b, const float* d_prob, int index, int* d_words, int* d_backptr) {
  return beam_expand_impl(ctx, "zr_beam_expand", b, d_prob, nullptr, index, d_words, d_backptr);
}

int zr_beam_expand_logits(zr_ctx* ctx, zr_beam* b, const float* d_logits, const float* d_colstats, int index,
                          int* d_words, int* d_backptr) {
  ZR_CHECK_ARG(d_colstats != nullptr, "zr_beam_expand_logits: d_colstats is null");
  return beam_expand_impl(ctx, "zr_beam_expand_logits", b, d_logits, d_colstats, index, d_words, d_backptr);
}

int zr_beam_finish(zr_ctx* ctx, zr_beam* b, const float* d_prob) {
  return beam_finish_impl(ctx, "zr_beam_finish", b, d_prob, nullptr);
}

int zr_beam_finish_logits(zr_ctx* ctx, zr_beam* b, const float* d_logits, const float* d_colstats) {
  ZR_CHECK_ARG(d_colstats != nullptr, "zr_beam_finish_logits: d_colstats is null");
  return beam_finish_impl(ctx, "zr_beam_finish_logits", b, d_logits, d_colstats);
}

int zr_beam_expand_blocks(zr_ctx* ctx, zr_beam* b, const float* d_logits, const float* d_blocks, int index,
                          int* d_words, int* d_backptr) {
  ZR_CHECK_ARG(d_blocks != nullptr, "zr_beam_expand_blocks: d_blocks is null");
  return beam_expand_impl(ctx, "zr_beam_expand_blocks", b, d_logits, nullptr, index, d_words, d_backptr, d_blocks);
}

int zr_beam_finish_blocks(zr_ctx* ctx, zr_beam* b, const float* d_logits, const float* d_blocks) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b && d_logits && d_blocks, "zr_beam_finish_blocks: null pointer");
  rc = zr_softmax_colstats_launch(ctx, d_blocks, zr_softmax_partial_blocks(b->vocab), b->n_sent * b->beam, b->d_colstats);
  if (rc) return rc;
  return beam_finish_impl(ctx, "zr_beam_finish_blocks", b, d_logits, b->d_colstats);
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

int zr_ensemble_average(zr_ctx* ctx, int n_models, const float* const d_probs[], int V, int cols, float* d_out) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(n_models >= 1 && n_models <= kMaxEnsemble && V > 0 && cols > 0 && cols <= 65535 && d_probs && d_out,
               "zr_ensemble_average: %d models (at most %d), V = %d, cols = %d, or a null pointer", n_models, kMaxEnsemble,
               V, cols);
  EnsembleArgs a = {};
  for (int k = 0; k < n_models; ++k) {
    ZR_CHECK_ARG(d_probs[k] != nullptr, "zr_ensemble_average: distribution %d is null", k);
    a.p[k] = d_probs[k];
  }
  const int chunks = (V + kEnsembleChunk - 1) / kEnsembleChunk;
  void* ws = nullptr;
  rc = zr_ctx_scratch(ctx, 0, (size_t)chunks * cols * sizeof(double), &ws);
  if (rc) return rc;
  bool vec = V % 4 == 0 && ((uintptr_t)d_out & 15) == 0;
  for (int k = 0; k < n_models; ++k) vec = vec && ((uintptr_t)d_probs[k] & 15) == 0;
  const dim3 grid(chunks, cols);
  if (vec) {
    ensemble_mean_kernel<true><<<grid, 256, 0, ctx->stream>>>(a, n_models, V, d_out, (double*)ws);
    ZR_LAUNCH_CHECK("ensemble_mean_kernel");
    ensemble_normalize_kernel<true><<<grid, 256, 0, ctx->stream>>>(V, d_out, (const double*)ws);
  } else {
    ensemble_mean_kernel<false><<<grid, 256, 0, ctx->stream>>>(a, n_models, V, d_out, (double*)ws);
    ZR_LAUNCH_CHECK("ensemble_mean_kernel");
    ensemble_normalize_kernel<false><<<grid, 256, 0, ctx->stream>>>(V, d_out, (const double*)ws);
  }
  ZR_LAUNCH_CHECK("ensemble_normalize_kernel");
  return ZR_OK;
}

int zr_beam_set_input_ids(zr_ctx* ctx, zr_beam* b, int* d_words_nonneg) {
  (void)ctx;
  ZR_CHECK_ARG(b != nullptr, "zr_beam_set_input_ids: beam object is null");
  b->d_words_nn_out = d_words_nonneg;
  return ZR_OK;
}

int zr_beam_set_viterbi(zr_ctx* ctx, zr_beam* b, int enable, const int* d_viterbi) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b != nullptr, "zr_beam_set_viterbi: beam object is null");
  ZR_CHECK_ARG(enable || !d_viterbi, "zr_beam_set_viterbi: alignments given with tracking switched off");
  if (enable && !b->track_viterbi) {
    ZR_CHECK_ARG(b->current_index == 0, "zr_beam_set_viterbi: tracking can only be switched on before the first step");
    b->track_viterbi = 1;
    rc = zr_beam_init(ctx, b);  // fills the alignment rows with -20
    if (rc) return rc;
  }
  if (!enable) b->track_viterbi = 0;
  b->d_viterbi_in = d_viterbi;
  return ZR_OK;
}

int zr_beam_hypotheses_viterbi(zr_ctx* ctx, zr_beam* b, int sentence, int cap, int* h_viterbi) {
  int rc = zr_bind_device(ctx);
  if (rc) return rc;
  ZR_CHECK_ARG(b && sentence >= 0 && sentence < b->n_sent && cap >= 0, "zr_beam_hypotheses_viterbi: bad argument");
  ZR_CHECK_ARG(b->track_viterbi, "zr_beam_hypotheses_viterbi: alignments are not being tracked (zr_beam_set_viterbi)");
  int count = 0;
  ZR_HIP(hipMemcpyAsync(&count, b->d_hyp_count + sentence, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
  ZR_HIP(hipStreamSynchronize(ctx->stream));
  if (count > b->hyp_cap)
    return zr_set_error(ZR_EDATA, "zr_beam_hypotheses_viterbi: %d finished hypotheses exceed the capacity %d", count,
                        b->hyp_cap);
  const int n = count < cap ? count : cap;
  if (n > 0) {
    ZR_CHECK_ARG(h_viterbi != nullptr, "zr_beam_hypotheses_viterbi: null output");
    ZR_HIP(hipMemcpyAsync(h_viterbi, b->d_hyp_vit + (size_t)sentence * b->hyp_cap * b->max_len,
                          sizeof(int) * (size_t)n * b->max_len, hipMemcpyDeviceToHost, ctx->stream));
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
