// CPU restatement of the Zoph_RNN stacked-LSTM forward path.
//
// THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP path is compared
// with (tests, the smoke check, and the bench's cpu_baseline leg); nothing that
// ships may call it.  It restates, on host arrays, the arithmetic of the
// reference's forward kernels and cuBLAS call sites, citing the reference
// file:line each function follows.  All matrices are column-major
// (IDX2C, src/BZ_CUDA_UTIL.h:26); activations are H x minibatch.
//
// What pins each function (see tests/test_oracle_*.py): closed forms and
// brute-force restatements in numpy float64, invariants (column sums, shift
// invariance, linearity), and special cases that reduce to a textbook
// routine.  Checked by value against an independent float64 statement:
// the contractions, the LSTM cell (torch.nn.LSTMCell; feed-input term), the
// stacked sweep with non-zero initial states and the cell clip, every output
// of the attention step (p_t, alignments, context, h~; fails for W_a in place
// of W_a^T and for a missing tanh), the soft-max (scipy logsumexp), the beam
// step with a non-zero length penalty for survivors, <EOF> hypotheses and the
// forced finish, and the strict length-ratio filter of the k-best output.  The reference holds no golden vectors for this path and its
// contractions run inside cuBLAS (summation order unknown), so no function
// here is pinned by a reference-held vector: parity with the *reference* is
// therefore "pinned by mathematics only" for every function in this file.
//
// Build: see oracle/Makefile (g++ -O2 -fopenmp -shared -fPIC).

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <queue>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

#define IDX2C(i, j, ld) ((size_t)(j) * (size_t)(ld) + (size_t)(i))

namespace {

// ---------------------------------------------------------------------------
// Contractions.  The reference calls cublasSgemm (src/BZ_CUDA_UTIL.h:691-696)
// with alpha=1, beta=0.  acc64=1 accumulates in double and rounds once (the
// "exact" value any fp32 summation order must be close to); acc64=0
// accumulates in float (the timed CPU baseline).
// ---------------------------------------------------------------------------
template <typename Acc>
void gemm_nn_t(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc) {
  const int MB = 256, NB = 4;
  const int nmb = (M + MB - 1) / MB;
#pragma omp parallel for schedule(static)
  for (int mb = 0; mb < nmb; ++mb) {
    const int m0 = mb * MB;
    const int mlen = std::min(MB, M - m0);
    Acc acc[NB][MB];
    for (int n0 = 0; n0 < N; n0 += NB) {
      const int nlen = std::min(NB, N - n0);
      for (int q = 0; q < nlen; ++q)
        for (int i = 0; i < mlen; ++i) acc[q][i] = 0;
      for (int k = 0; k < K; ++k) {
        const float* a = A + IDX2C(m0, k, lda);
        for (int q = 0; q < nlen; ++q) {
          const Acc b = (Acc)B[IDX2C(k, n0 + q, ldb)];
          Acc* ac = acc[q];
          for (int i = 0; i < mlen; ++i) ac[i] += (Acc)a[i] * b;
        }
      }
      for (int q = 0; q < nlen; ++q)
        for (int i = 0; i < mlen; ++i) C[IDX2C(m0 + i, n0 + q, ldc)] = (float)acc[q][i];
    }
  }
}

// C(MxN) = A^T * B with A stored K x M (lda >= K): CUBLAS_OP_T on the first operand
// (src/attention_node.hpp:195).
template <typename Acc>
void gemm_tn_t(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int n = 0; n < N; ++n)
    for (int m = 0; m < M; ++m) {
      const float* a = A + IDX2C(0, m, lda);
      const float* b = B + IDX2C(0, n, ldb);
      Acc s = 0;
      for (int k = 0; k < K; ++k) s += (Acc)a[k] * (Acc)b[k];
      C[IDX2C(m, n, ldc)] = (float)s;
    }
}

void gemm_nn(int acc64, int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc) {
  if (acc64)
    gemm_nn_t<double>(M, N, K, A, lda, B, ldb, C, ldc);
  else
    gemm_nn_t<float>(M, N, K, A, lda, B, ldb, C, ldc);
}
void gemm_tn(int acc64, int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc) {
  if (acc64)
    gemm_tn_t<double>(M, N, K, A, lda, B, ldb, C, ldc);
  else
    gemm_tn_t<float>(M, N, K, A, lda, B, ldb, C, ldc);
}

// forward_sigmoid_kernel (float overload), src/custom_kernels.h:58-65.
inline float sigmoid_f32(float v) { return 1.0f / (1.0f + expf(-1.0f * v)); }
// forward_sigmoid_kernel_feed, src/custom_kernels.h:92-99: the literals are double, so the
// expression is evaluated in double and rounded to float on the store.
inline float sigmoid_via_f64(float v) { return (float)(1.0 / (1.0 + exp(-1.0 * (double)v))); }

}  // namespace

extern "C" {

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}

// vocab_to_01 + vocab_to_nonM1, src/custom_kernels.h:10-32, launched from
// Input_To_Hidden_Layer::prep_GPU_vocab_indices (src/Input_To_Hidden_Layer.hpp:1199-1202).
void orc_vocab_prep(const int* ids, int n, int* ids_nonneg, int* mask01) {
  for (int i = 0; i < n; ++i) {
    mask01[i] = (ids[i] == -1) ? 0 : 1;
    ids_nonneg[i] = (ids[i] == -1) ? 0 : ids[i];
  }
}

// vocab_softmax, src/custom_kernels.h:38-50 (in place on the ids, int and float masks).
void orc_vocab_softmax(int* ids, int n, int* mask01, float* mask01f) {
  for (int i = 0; i < n; ++i) {
    if (ids[i] == -1) {
      ids[i] = 0;
      mask01[i] = 0;
      mask01f[i] = 0.f;
    } else {
      mask01[i] = 1;
      mask01f[i] = 1.f;
    }
  }
}

// sparse_lookup_kernel, src/custom_kernels.h:342-348: x[:,b] = W[:,ids[b]].
void orc_embed_gather(const float* W, int H, int V, const int* ids, int mb, float* x) {
  (void)V;
  for (int b = 0; b < mb; ++b) memcpy(x + IDX2C(0, b, H), W + IDX2C(0, ids[b], H), sizeof(float) * (size_t)H);
}

void orc_gemm_nn(int acc64, int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc) {
  gemm_nn(acc64, M, N, K, A, lda, B, ldb, C, ldc);
}
void orc_gemm_tn(int acc64, int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc) {
  gemm_tn(acc64, M, N, K, A, lda, B, ldb, C, ldc);
}

// One LSTM node forward step.  LSTM_IH_Node::forward_prop_GPU (src/LSTM.hpp:76-421) and
// LSTM_HH_Node::forward_prop_GPU (src/LSTM_HH.hpp:103-333).  Gate order i,f,c,o.
//   M[g], Wh[g], Q[g]: H x H; b[g]: H; x, hprev, cprev, htild: H x mb; mask01: mb.
//   Q == NULL or htild == NULL: the non-feed kernels (float sigmoid); else the *_feed kernels
//   (third addend, sigmoid evaluated in double; src/LSTM.hpp:175-182).
//   Outputs (each H x mb): gate_i, gate_f, gate_c (tanh), gate_o, c, h.  Any gate pointer may be NULL.
void orc_lstm_step(int acc64, int H, int mb, const float* const* M, const float* const* Wh, const float* const* Q,
                   const float* const* b, const float* x, const float* hprev, const float* cprev,
                   const float* htild, const int* mask01, int clip_cell, float clip_threshold, float* gate_i,
                   float* gate_f, float* gate_c, float* gate_o, float* c, float* h) {
  const bool feed = (Q != nullptr && htild != nullptr);
  const size_t n = (size_t)H * mb;
  std::vector<float> t1(n), t2(n), t3(feed ? n : 0);
  std::vector<float> gates[4];
  for (int g = 0; g < 4; ++g) {
    gates[g].resize(n);
    // temp{1,3,5,7} = M_g x ; temp{2,4,6,8} = W_hg h_prev ; temp{9..12} = Q_g htild
    gemm_nn(acc64, H, mb, H, M[g], H, x, H, t1.data(), H);
    gemm_nn(acc64, H, mb, H, Wh[g], H, hprev, H, t2.data(), H);
    if (feed) gemm_nn(acc64, H, mb, H, Q[g], H, htild, H, t3.data(), H);
    for (int col = 0; col < mb; ++col)
      for (int i = 0; i < H; ++i) {
        const size_t ix = IDX2C(i, col, H);
        float v;
        if (feed)
          v = t1[ix] + t2[ix] + t3[ix] + b[g][i];  // custom_kernels.h:96,132
        else
          v = t1[ix] + t2[ix] + b[g][i];  // custom_kernels.h:62,110
        if (g == 2)
          gates[g][ix] = tanhf(v);  // forward_tanh_kernel(_feed), custom_kernels.h:106-135
        else
          gates[g][ix] = feed ? sigmoid_via_f64(v) : sigmoid_f32(v);
      }
  }
  for (int col = 0; col < mb; ++col)
    for (int i = 0; i < H; ++i) {
      const size_t ix = IDX2C(i, col, H);
      // forward_c_t_kernel, custom_kernels.h:141-147
      float cv = gates[1][ix] * cprev[ix] + gates[0][ix] * gates[2][ix];
      if (clip_cell) {  // clip_mat_kernel, custom_kernels.h:2222-2231 (BZ_CUDA::clip_cell, src/LSTM.hpp:369-371)
        if (cv > 0)
          cv = (cv > clip_threshold) ? clip_threshold : cv;
        else
          cv = (cv < -clip_threshold) ? -clip_threshold : cv;
      }
      // forward_h_t_kernel, custom_kernels.h:162-168
      float hv = gates[3][ix] * tanhf(cv);
      // zero_c_t_and_h_t, custom_kernels.h:184-192
      hv = hv * mask01[col];
      cv = cv * mask01[col];
      c[ix] = cv;
      h[ix] = hv;
    }
  float* outs[4] = {gate_i, gate_f, gate_c, gate_o};
  for (int g = 0; g < 4; ++g)
    if (outs[g]) memcpy(outs[g], gates[g].data(), n * sizeof(float));
}

// Logits: D h + b_d.  cublasSgemm + matrix_bias_kernel (src/softmax.hpp:539-547, custom_kernels.h:787-794).
void orc_softmax_logits(int acc64, const float* D, const float* b_d, int V, int H, const float* h, int mb,
                        float* logits) {
  gemm_nn(acc64, V, mb, H, D, V, h, H, logits, V);
  for (int col = 0; col < mb; ++col)
    for (int v = 0; v < V; ++v) logits[IDX2C(v, col, V)] = logits[IDX2C(v, col, V)] + b_d[v];
}

// outputdist_overflow_prevention_kernel, src/custom_kernels.h:503-577: per column, max, expf(x-max),
// sum, divide.  emulate_tree=1 reproduces the kernel's summation order (256 strided partial sums, then a
// binary tree, SOFTMAX_THREADS=256); emulate_tree=0 sums in double (the order-free value).
void orc_softmax_dist(const float* logits, int V, int mb, int emulate_tree, float* prob) {
  const int T = 256;
#pragma omp parallel for schedule(static)
  for (int col = 0; col < mb; ++col) {
    const float* in = logits + IDX2C(0, col, V);
    float* out = prob + IDX2C(0, col, V);
    float mx = -FLT_MAX;
    for (int v = 0; v < V; ++v)
      if (mx < in[v]) mx = in[v];
    if (emulate_tree) {
      float buf[T];
      for (int t = 0; t < T; ++t) buf[t] = 0.f;
      for (int v = 0; v < V; ++v) {
        const float z = expf(in[v] - mx);
        buf[v % T] += z;
        out[v] = z;
      }
      for (int stride = T / 2; stride > 0; stride >>= 1)
        for (int t = 0; t < stride; ++t) buf[t] += buf[t + stride];
      const float sum = buf[0];
      for (int v = 0; v < V; ++v) out[v] = out[v] / sum;
    } else {
      double sum = 0;
      for (int v = 0; v < V; ++v) {
        const float z = expf(in[v] - mx);
        out[v] = z;
        sum += (double)z;
      }
      const float sumf = (float)sum;
      for (int v = 0; v < V; ++v) out[v] = out[v] / sumf;
    }
  }
}

// outputdist_perplexity_kernel, src/custom_kernels.h:583-660: double log-probabilities,
// log(exp(x-max)) - log(sum) per column.
void orc_softmax_logprob_f64(const float* logits, int V, int mb, double* logp) {
#pragma omp parallel for schedule(static)
  for (int col = 0; col < mb; ++col) {
    const float* in = logits + IDX2C(0, col, V);
    double* out = logp + IDX2C(0, col, V);
    double mx = -DBL_MAX;
    for (int v = 0; v < V; ++v)
      if (mx < (double)in[v]) mx = (double)in[v];
    double sum = 0;
    for (int v = 0; v < V; ++v) {
      const double z = exp((double)in[v] - mx);
      sum += z;
      out[v] = z;
    }
    const double ls = log(sum);
    for (int v = 0; v < V; ++v) out[v] = log(out[v]) - ls;
  }
}

// softmax_layer::compute_loss_GPU, src/softmax.hpp:867-900: sum over unmasked columns of
// logp[target[b], b].
double orc_softmax_loss(const double* logp, int V, int mb, const int* target, const int* mask01) {
  double loss = 0;
  for (int b = 0; b < mb; ++b)
    if (mask01[b] == 1) loss += logp[IDX2C(target[b], b, V)];
  return loss;
}

// attention_node::forward_prop, src/attention_node.hpp:73-394 (single-source branch), with the kernels it
// launches: tanh_kernel (custom_kernels.h:1567), sigmoid_kernel (:1583, double), alignment_pos_kernel (:1598),
// lower_upper_kernel (:1608), create_indicies_kernel (:1650), load_in_hs_kernel (:1694),
// elem_reduce_kernel_large (:1892), alignment_reduction_kernel (:1752), create_c_t_kernel (:1804),
// tanh_att_forward_kernel (:1844), zero_h_t (:2212).
//   hs_table: the longest_sent source-side top-layer states, table t at hs_table + t*H*mb
//             (the reference keeps a pointer table d_total_hs_mat, src/attention_layer.hpp:106-160).
//   batch_info: [0,mb) true source lengths S_b, [mb,2mb) left-pad offsets (src/fileHelper.h:499-500).
//   outputs: h_tild H x mb; alignments and indices (2D+1) x mb laid out [b + mb*j]; p_t mb; c_ctx H x mb.
void orc_attention_forward(int acc64, int H, int mb, int D, const float* W_a, const float* W_p, const float* v_p,
                           const float* out_bias, const float* W_c1, const float* W_c2, const float* hs_table,
                           const int* batch_info, const float* h_t, const int* mask01, float* h_tild,
                           float* alignments, int* indices, float* p_t, float* c_ctx) {
  const int W = 2 * D + 1;
  const size_t n = (size_t)H * mb;
  std::vector<float> tanh1(n), sigma1(mb), q(n), f1(n), f2(n);
  std::vector<int> lower_upper(2 * (size_t)mb);
  const float sigma_sq = (float)((D * D) / 4.0);  // attention_node.hpp:50

  gemm_nn(acc64, H, mb, H, W_p, H, h_t, H, tanh1.data(), H);        // :132
  for (size_t i = 0; i < n; ++i) tanh1[i] = tanhf(tanh1[i]);        // :141
  gemm_nn(acc64, 1, mb, H, v_p, 1, tanh1.data(), H, sigma1.data(), 1);  // :147
  for (int b = 0; b < mb; ++b) {
    sigma1[b] = (float)(1.0 / (1.0 + exp(-1.0 * (double)sigma1[b])));  // sigmoid_kernel, double literals
    p_t[b] = batch_info[b] * sigma1[b];                                // alignment_pos_kernel
    const int ip = (int)p_t[b];
    lower_upper[IDX2C(0, b, 2)] = (0 > ip - D) ? 0 : (ip - D);
    lower_upper[IDX2C(1, b, 2)] = ((batch_info[b] - 1) < ip + D) ? (batch_info[b] - 1) : (ip + D);
  }
  for (int b = 0; b < mb; ++b) {  // create_indicies_kernel
    int cur = lower_upper[IDX2C(0, b, 2)];
    const int mx = lower_upper[IDX2C(1, b, 2)];
    for (int j = 0; j < W; ++j) {
      if (mask01[b] == 1) {
        indices[IDX2C(b, j, mb)] = (cur > mx) ? -1 : cur;
        cur++;
      } else {
        indices[IDX2C(b, j, mb)] = -1;
      }
    }
  }
  gemm_tn(acc64, H, mb, H, W_a, H, h_t, H, q.data(), H);  // :195, W_a^T h
  // load_in_hs_kernel + elem_reduce_kernel_large: score over the gathered (or zero) source column.
  auto hs_col = [&](int b, int j) -> const float* {
    const int s = indices[IDX2C(b, j, mb)];
    if (s == -1) return nullptr;
    const int t = batch_info[b] - 1 - s + batch_info[mb + b];
    return hs_table + (size_t)t * n + IDX2C(0, b, H);
  };
#pragma omp parallel for schedule(static)
  for (int b = 0; b < mb; ++b)
    for (int j = 0; j < W; ++j) {
      const float* hs = hs_col(b, j);
      if (acc64) {
        double s = 0;
        if (hs)
          for (int k = 0; k < H; ++k) s += (double)hs[k] * (double)q[IDX2C(k, b, H)];
        alignments[IDX2C(b, j, mb)] = (float)s;
      } else {
        float s = 0;
        if (hs)
          for (int k = 0; k < H; ++k) s += hs[k] * q[IDX2C(k, b, H)];
        alignments[IDX2C(b, j, mb)] = s;
      }
    }
  // alignment_reduction_kernel: note max_val starts at 0, not -inf.
  for (int b = 0; b < mb; ++b) {
    float sum = 0, max_val = 0;
    for (int j = 0; j < W; ++j)
      if (indices[IDX2C(b, j, mb)] != -1)
        if (alignments[IDX2C(b, j, mb)] > max_val) max_val = alignments[IDX2C(b, j, mb)];
    for (int j = 0; j < W; ++j) {
      if (indices[IDX2C(b, j, mb)] != -1) {
        alignments[IDX2C(b, j, mb)] = expf(alignments[IDX2C(b, j, mb)] - max_val);
        sum += alignments[IDX2C(b, j, mb)];
      } else {
        alignments[IDX2C(b, j, mb)] = 0;
      }
    }
    for (int j = 0; j < W; ++j) {
      if (indices[IDX2C(b, j, mb)] != -1) {
        const float d = p_t[b] - indices[IDX2C(b, j, mb)];
        const float temp = expf((-1 * powf(d, 2.0f)) / (2 * sigma_sq));
        if (sum != 0) alignments[IDX2C(b, j, mb)] = (alignments[IDX2C(b, j, mb)] / sum) * temp;
      } else {
        alignments[IDX2C(b, j, mb)] = 0;
      }
    }
  }
  // create_c_t_kernel: c[:,b] = sum_j a[b + mb*j] * hs[:, b + mb*j]
#pragma omp parallel for schedule(static)
  for (int b = 0; b < mb; ++b) {
    for (int i = 0; i < H; ++i) c_ctx[IDX2C(i, b, H)] = 0;
    for (int j = 0; j < W; ++j) {
      const float* hs = hs_col(b, j);
      if (!hs) continue;  // the gathered column is zero
      const float a = alignments[IDX2C(b, j, mb)];
      for (int i = 0; i < H; ++i) c_ctx[IDX2C(i, b, H)] += a * hs[i];
    }
  }
  gemm_nn(acc64, H, mb, H, W_c1, H, c_ctx, H, f1.data(), H);  // :354
  gemm_nn(acc64, H, mb, H, W_c2, H, h_t, H, f2.data(), H);    // :360
  for (int b = 0; b < mb; ++b)
    for (int i = 0; i < H; ++i) {
      const size_t ix = IDX2C(i, b, H);
      float v = tanhf(f1[ix] + f2[ix] + out_bias[i]);  // tanh_att_forward_kernel
      v *= mask01[b];                                   // zero_h_t
      h_tild[ix] = v;
    }
}

// get_viterbi_alignment_kernel, src/custom_kernels.h:1623-1635: for every column the window index of the largest
// alignment weight; the running maximum starts at -1 and only a strictly larger weight replaces it.
void orc_attention_viterbi(const float* alignments, const int* indices, int D, int mb, int* out) {
  for (int b = 0; b < mb; ++b) {
    float max_val = -1;
    int max_index = -1;
    for (int i = 0; i < 2 * D + 1; ++i) {
      if (max_val < alignments[IDX2C(b, i, mb)]) {
        max_val = alignments[IDX2C(b, i, mb)];
        max_index = indices[IDX2C(b, i, mb)];
      }
    }
    out[b] = max_index;
  }
}

// attention_node::back_prop, src/attention_node.hpp:398-669 (single-source branch), with the kernels it launches:
// zero_h_t (custom_kernels.h:2212), tanh_grad_kernel (:1835), error_alignments_kernel_large (:1968),
// error_hs_ct_kernel_large (:2179), error_pt_kernel (:2006), att_vp_error (:2040), grad_W_p_kernel (:2051),
// get_ht_scalings_Wa_grad_kernel (:2094), scale_ht_kernel (:2114), copy_errors_source (:2142), and its cuBLAS calls.
// The values the reference caches in the forward pass (tanh_1, sigma_1, W_a^T h, the gathered source columns and the
// Gaussian factors d_cached_exp) are recomputed here from h_t, p_t and the indices with the forward pass's formulas.
//   h_t:        the h_t the forward pass read (after the attention layer's dropout, where that is on)
//   err_htild:  error with respect to h~ (the caller has already added the feed-input error of the next step, :416)
//   outputs:    err_h_t (H x mb, overwritten; before the dropout of :647); err_hs_table (same layout as hs_table, +=);
//               dW_a, dW_p, dW_c1, dW_c2 (H x H), dv_p, dbias (H), all += as in the reference (beta = 1)
void orc_attention_backward(int H, int mb, int D, const float* W_a, const float* W_p, const float* v_p,
                            const float* W_c1, const float* W_c2, const float* hs_table, const int* batch_info,
                            const float* h_t, const int* mask01, const float* h_tild, const float* alignments,
                            const int* indices, const float* p_t, const float* c_ctx, const float* err_htild,
                            float* err_h_t, float* err_hs_table, float* dW_a, float* dW_p, float* dv_p, float* dbias,
                            float* dW_c1, float* dW_c2) {
  const int W = 2 * D + 1;
  const size_t n = (size_t)H * mb;
  const float sigma_sq = (float)((D * D) / 4.0);
  std::vector<float> e(n), err_ct(n), err_ht(n), tanh1(n), sigma1(mb), q(n), temp1(n), hs_sum(n, 0.0f), tmp(n);
  std::vector<float> err_as((size_t)W * mb), err_pt(mb), scal((size_t)W * mb), gauss((size_t)W * mb);
  auto hs_index = [&](int b, int j) -> long long {
    const int s = indices[IDX2C(b, j, mb)];
    if (s == -1) return -1;
    const int t = batch_info[b] - 1 - s + batch_info[mb + b];
    return (long long)((size_t)t * n + IDX2C(0, b, H));
  };
  // C (H x H) += A (H x mb) * B^T (B is H x mb): cublas gemm N,T with beta = 1, accumulated in double per element
  auto outer_acc = [&](const float* A, const float* B, float* C) {
#pragma omp parallel for schedule(static)
    for (int j = 0; j < H; ++j)
      for (int i = 0; i < H; ++i) {
        double sum = 0;
        for (int b = 0; b < mb; ++b) sum += (double)A[IDX2C(i, b, H)] * (double)B[IDX2C(j, b, H)];
        C[IDX2C(i, j, H)] += (float)sum;
      }
  };
  for (int b = 0; b < mb; ++b)
    for (int i = 0; i < H; ++i) {
      const size_t ix = IDX2C(i, b, H);
      const float v = err_htild[ix] * mask01[b];            // zero_h_t
      e[ix] = v * (1 - h_tild[ix] * h_tild[ix]);            // tanh_grad_kernel on d_final_temp_2
    }
  outer_acc(e.data(), c_ctx, dW_c1);                         // :437
  outer_acc(e.data(), h_t, dW_c2);                           // :443
  for (int i = 0; i < H; ++i) {                              // :456, gemv with the ones vector
    double sum = 0;
    for (int b = 0; b < mb; ++b) sum += e[IDX2C(i, b, H)];
    dbias[i] += (float)sum;
  }
  gemm_tn(1, H, mb, H, W_c1, H, e.data(), H, err_ct.data(), H);  // :464
  gemm_tn(1, H, mb, H, W_c2, H, e.data(), H, err_ht.data(), H);  // :476
  // error_alignments_kernel_large and error_hs_ct_kernel_large
  for (int b = 0; b < mb; ++b)
    for (int j = 0; j < W; ++j) {
      const long long at = hs_index(b, j);
      double sum = 0;
      if (at >= 0) {
        const float a = alignments[IDX2C(b, j, mb)];
        for (int i = 0; i < H; ++i) {
          sum += (double)err_ct[IDX2C(i, b, H)] * (double)hs_table[at + i];
          err_hs_table[at + i] += err_ct[IDX2C(i, b, H)] * a;
        }
      }
      err_as[IDX2C(j, b, W)] = (float)sum;
    }
  // error_pt_kernel
  for (int b = 0; b < mb; ++b) {
    double sum = 0;
    for (int j = 0; j < W; ++j)
      sum += (double)(err_as[IDX2C(j, b, W)] * alignments[IDX2C(b, j, mb)] *
                      ((indices[IDX2C(b, j, mb)] - p_t[b]) / sigma_sq));
    err_pt[b] = (float)sum;
  }
  // forward values again: tanh_1, sigma_1 (attention_node.hpp:132-150)
  gemm_nn(1, H, mb, H, W_p, H, h_t, H, tanh1.data(), H);
  for (size_t i = 0; i < n; ++i) tanh1[i] = tanhf(tanh1[i]);
  gemm_nn(1, 1, mb, H, v_p, 1, tanh1.data(), H, sigma1.data(), 1);
  for (int b = 0; b < mb; ++b) sigma1[b] = (float)(1.0 / (1.0 + exp(-1.0 * (double)sigma1[b])));
  // att_vp_error, then the gemv into v_p_grad (:536)
  for (int b = 0; b < mb; ++b)
    for (int i = 0; i < H; ++i)
      temp1[IDX2C(i, b, H)] = err_pt[b] * sigma1[b] * (1 - sigma1[b]) * batch_info[b] * tanh1[IDX2C(i, b, H)];
  for (int i = 0; i < H; ++i) {
    double sum = 0;
    for (int b = 0; b < mb; ++b) sum += temp1[IDX2C(i, b, H)];
    dv_p[i] += (float)sum;
  }
  // grad_W_p_kernel, the outer product into W_p_grad (:545) and W_p^T temp into the error of h_t (:551, beta = 1)
  for (int b = 0; b < mb; ++b)
    for (int i = 0; i < H; ++i) {
      const size_t ix = IDX2C(i, b, H);
      temp1[ix] = err_pt[b] * batch_info[b] * v_p[i] * sigma1[b] * (1 - sigma1[b]) * (1 - tanh1[ix] * tanh1[ix]);
    }
  outer_acc(temp1.data(), h_t, dW_p);
  gemm_tn(1, H, mb, H, W_p, H, temp1.data(), H, tmp.data(), H);
  for (size_t i = 0; i < n; ++i) err_ht[i] += tmp[i];
  // get_ht_scalings_Wa_grad_kernel; d_cached_exp as alignment_reduction_kernel leaves it (1 on empty slots)
  for (int b = 0; b < mb; ++b)
    for (int j = 0; j < W; ++j) {
      const int s = indices[IDX2C(b, j, mb)];
      float g = 1;
      if (s != -1) {
        const float d = p_t[b] - s;
        g = expf((-1 * powf(d, 2.0f)) / (2 * sigma_sq));
      }
      gauss[IDX2C(j, b, W)] = g;
    }
  for (int b = 0; b < mb; ++b)
    for (int j = 0; j < W; ++j) {
      const float aj = alignments[IDX2C(b, j, mb)], gj = gauss[IDX2C(j, b, W)];
      float v = err_as[IDX2C(j, b, W)] * aj * (1 - aj / gj);
      for (int k = 0; k < W; ++k)
        if (k != j) v += -1 * err_as[IDX2C(k, b, W)] * alignments[IDX2C(b, k, mb)] * aj / gj;
      scal[IDX2C(j, b, W)] = v;
    }
  // the loop of :580-601: h_s_sum += scaling * h_s; error of h_s += scaling * (W_a^T h)
  gemm_tn(1, H, mb, H, W_a, H, h_t, H, q.data(), H);
  for (int b = 0; b < mb; ++b)
    for (int j = 0; j < W; ++j) {
      const long long at = hs_index(b, j);
      if (at < 0) continue;  // the gathered column is zero and copy_errors_source skips the slot
      const float sc = scal[IDX2C(j, b, W)];
      for (int i = 0; i < H; ++i) {
        hs_sum[IDX2C(i, b, H)] += hs_table[at + i] * sc;
        err_hs_table[at + i] += q[IDX2C(i, b, H)] * sc;
      }
    }
  outer_acc(h_t, hs_sum.data(), dW_a);                              // :632
  gemm_nn(1, H, mb, H, W_a, H, hs_sum.data(), H, tmp.data(), H);    // :636, beta = 1
  for (size_t i = 0; i < n; ++i) err_h_t[i] = err_ht[i] + tmp[i];
}

// dropout_kernel, src/custom_kernels.h:1556-1560: `rate` is the probability of KEEPING a value, `uniform` the
// numbers curandGenerateUniform left in the mask array.
void orc_dropout(const float* uniform, float rate, float* x, size_t n) {
  for (size_t i = 0; i < n; ++i) x[i] = (uniform[i] < rate) * (1 / rate) * x[i];
}

// The feed-input part of LSTM_IH_Node::back_prop_GPU and compute_gradients_GPU (src/LSTM.hpp:804-866, under
// `feed_input && index != 0`, and the Q gradient products :1014-1050): error of h~_{t-1} = sum_g Q_g^T d_g, and
// Q_g_grad += d_g h~^T.
//   dgates: the four pre-activation errors stacked as [4H] x mb (i, f, c~, o); Q, dQ: four H x H matrices each
void orc_lstm_feed_backward(int H, int mb, const float* const* Q, const float* dgates, const float* htild,
                            float* err_htild, float* const* dQ) {
  const size_t n = (size_t)H * mb;
  std::vector<float> dg(n), tmp(n);
  for (size_t i = 0; i < n; ++i) err_htild[i] = 0;
  for (int g = 0; g < 4; ++g) {
    for (int b = 0; b < mb; ++b)
      for (int i = 0; i < H; ++i) dg[IDX2C(i, b, H)] = dgates[IDX2C(g * H + i, b, 4 * H)];
    gemm_tn(1, H, mb, H, Q[g], H, dg.data(), H, tmp.data(), H);
    for (size_t i = 0; i < n; ++i) err_htild[i] += tmp[i];
#pragma omp parallel for schedule(static)
    for (int j = 0; j < H; ++j)
      for (int i = 0; i < H; ++i) {
        double sum = 0;
        for (int b = 0; b < mb; ++b) sum += (double)dg[IDX2C(i, b, H)] * (double)htild[IDX2C(j, b, H)];
        dQ[g][IDX2C(i, j, H)] += (float)sum;
      }
  }
}

// Column gather used by the decoder state shuffles: dst[:,i] = src[:,perm[i]]
// (Input_To_Hidden_Layer::swap_states_decoding, src/Input_To_Hidden_Layer.hpp:1231-1242).
void orc_gather_columns(const float* src, int H, const int* perm, int n, float* dst) {
  for (int i = 0; i < n; ++i) memcpy(dst + IDX2C(0, i, H), src + IDX2C(0, perm[i], H), sizeof(float) * (size_t)H);
}

// transfer_decoding_states_GPU (src/Input_To_Hidden_Layer.hpp:1252-1266): broadcast one column to n columns.
void orc_broadcast_column(const float* src_col, int H, int n, float* dst) {
  for (int i = 0; i < n; ++i) memcpy(dst + IDX2C(0, i, H), src_col, sizeof(float) * (size_t)H);
}

}  // extern "C"

// ---------------------------------------------------------------------------
// Beam search.  decoder<dType> (src/decoder.h:162-1502), non-FSA path:
// init_decoder (:1317-1355), expand_hypothesis_without_fsa (:1158-1315),
// finish_current_hypotheses (:672-688), output_k_best_hypotheses (:1386-1413).
// The two heaps are std::priority_queue with the reference's comparators
// (pq_compare_functor / pq_global_compare_functor, :146-154) and the same
// push order, so tie behaviour follows libstdc++ exactly as in the reference.
// ---------------------------------------------------------------------------
namespace {

struct DecObj {
  float val;
  int vocab_index;
  int viterbi_alignment;  // src/decoder.h:62: the column's alignment rides along with every candidate
};
struct DecGlobalObj {
  float val;
  int beam_index;
  int vocab_index;
  int viterbi_alignment;  // src/decoder.h:35
};
struct PqCmp {
  bool operator()(const DecObj& a, const DecObj& b) const { return a.val < b.val; }
};
struct PqGlobalCmp {
  bool operator()(const DecGlobalObj& a, const DecGlobalObj& b) const { return a.val < b.val; }
};
struct Hypothesis {
  std::vector<int> words;
  std::vector<int> viterbi;  // src/decoder.h:126: one source position per word (entry 0 keeps the initial -20)
  float score;
};

struct OrcDecoder {
  int beam, vocab, start_symbol, end_symbol, max_len;
  float penalty, min_ratio;
  int current_index;
  std::vector<int> current_indices, new_indicies_changes;
  std::vector<int> top_sentences, top_sentences_temp;  // beam x max_len, row-major here
  std::vector<int> top_viterbi, top_viterbi_temp;      // top_sentences_viterbi (src/decoder.h:230-231), same shape
  std::vector<float> scores, scores_temp;
  std::vector<Hypothesis> hypotheses;
  std::priority_queue<DecObj, std::vector<DecObj>, PqCmp> pq;
  std::priority_queue<DecGlobalObj, std::vector<DecGlobalObj>, PqGlobalCmp> pq_global;
};

}  // namespace

extern "C" {

void* orc_decoder_create(int beam, int vocab, int start_symbol, int end_symbol, int max_len, float min_ratio,
                         float penalty) {
  OrcDecoder* d = new OrcDecoder();
  d->beam = beam;
  d->vocab = vocab;
  d->start_symbol = start_symbol;
  d->end_symbol = end_symbol;
  d->max_len = max_len;
  d->min_ratio = min_ratio;
  d->penalty = penalty;
  d->current_indices.resize(beam);
  d->new_indicies_changes.assign(beam, 0);
  d->top_sentences.resize((size_t)beam * max_len);
  d->top_sentences_temp.resize((size_t)beam * max_len);
  d->top_viterbi.resize((size_t)beam * max_len);
  d->top_viterbi_temp.resize((size_t)beam * max_len);
  d->scores.resize(beam);
  d->scores_temp.resize(beam);
  d->current_index = 0;
  return d;
}

void orc_decoder_destroy(void* p) { delete (OrcDecoder*)p; }

// init_decoder, src/decoder.h:1317-1355
void orc_decoder_init(void* p) {
  OrcDecoder* d = (OrcDecoder*)p;
  d->current_index = 0;
  std::fill(d->scores.begin(), d->scores.end(), 0.f);
  d->hypotheses.clear();
  for (int i = 0; i < d->beam; ++i) d->current_indices[i] = d->start_symbol;
  std::fill(d->top_sentences.begin(), d->top_sentences.end(), d->start_symbol);
  std::fill(d->top_viterbi.begin(), d->top_viterbi.end(), -20);  // src/decoder.h:1335
}

// expand_hypothesis_without_fsa, src/decoder.h:1158-1315.  outputdist: vocab x beam probabilities,
// column-major (column = beam entry).  viterbi: the attention layer's Viterbi alignment of every column
// (BZ_CUDA::viterbi_alignments), or NULL: the reference then fills in -1 for every column (:1174-1179).
void orc_decoder_expand_viterbi(void* p, const float* outputdist, int index, const int* viterbi) {
  OrcDecoder* d = (OrcDecoder*)p;
  const int beam = d->beam, V = d->vocab, L = d->max_len;
  int cols = beam;
  if (index == 0) cols = 1;
  while (!d->pq_global.empty()) d->pq_global.pop();
  for (int i = 0; i < cols; ++i) {
    while (!d->pq.empty()) d->pq.pop();
    if (d->current_indices[i] == -1) break;
    const int vit = viterbi ? viterbi[i] : -1;
    for (int j = 0; j < V; ++j) {
      const float pr = outputdist[IDX2C(j, i, V)];
      if ((int)d->pq.size() < beam + 1) {
        d->pq.push(DecObj{-pr, j, vit});
      } else if (-pr < d->pq.top().val) {
        d->pq.pop();
        d->pq.push(DecObj{-pr, j, vit});
      }
    }
    while (!d->pq.empty()) {
      DecObj t = d->pq.top();
      d->pq.pop();
      d->pq_global.push(DecGlobalObj{std::log(-t.val) + d->scores[i], i, t.vocab_index, t.viterbi_alignment});
    }
  }
  int i = 0;
  while (i < beam) {
    if (d->pq_global.empty()) {
      for (int c = 0; c < L; ++c) d->top_sentences_temp[(size_t)i * L + c] = d->top_sentences[c];
      d->top_sentences_temp[(size_t)i * L + d->current_index + 1] = d->start_symbol;
      for (int c = 0; c < L; ++c) d->top_viterbi_temp[(size_t)i * L + c] = d->top_viterbi[c];  // :1237, row 0 as it is
      d->current_indices[i] = -1;
      d->new_indicies_changes[i] = 0;
      d->scores_temp[i] = 0;
      i++;
      continue;
    }
    DecGlobalObj t = d->pq_global.top();
    d->pq_global.pop();
    if (t.vocab_index != d->start_symbol) {
      if (t.vocab_index == d->end_symbol) {
        Hypothesis hy;
        hy.words.assign(d->top_sentences.begin() + (size_t)t.beam_index * L,
                        d->top_sentences.begin() + (size_t)t.beam_index * L + d->current_index + 2);
        hy.words[d->current_index + 1] = d->end_symbol;
        hy.viterbi.assign(d->top_viterbi.begin() + (size_t)t.beam_index * L,
                          d->top_viterbi.begin() + (size_t)t.beam_index * L + d->current_index + 2);  // :1266-1267
        hy.viterbi[d->current_index + 1] = t.viterbi_alignment;
        hy.score = t.val + d->penalty;
        d->hypotheses.push_back(hy);
      } else {
        for (int c = 0; c < L; ++c)
          d->top_sentences_temp[(size_t)i * L + c] = d->top_sentences[(size_t)t.beam_index * L + c];
        d->top_sentences_temp[(size_t)i * L + d->current_index + 1] = t.vocab_index;
        for (int c = 0; c < L; ++c)
          d->top_viterbi_temp[(size_t)i * L + c] = d->top_viterbi[(size_t)t.beam_index * L + c];  // :1281-1282
        d->top_viterbi_temp[(size_t)i * L + d->current_index + 1] = t.viterbi_alignment;
        d->current_indices[i] = t.vocab_index;
        d->new_indicies_changes[i] = t.beam_index;
        d->scores_temp[i] = t.val + d->penalty;
        i++;
      }
    }
  }
  d->top_sentences = d->top_sentences_temp;
  d->top_viterbi = d->top_viterbi_temp;  // :1301
  d->scores = d->scores_temp;
  d->current_index += 1;
}
void orc_decoder_expand(void* p, const float* outputdist, int index) {
  orc_decoder_expand_viterbi(p, outputdist, index, nullptr);
}

// finish_current_hypotheses (non-FSA branch), src/decoder.h:672-688.
void orc_decoder_finish_viterbi(void* p, const float* outputdist, const int* viterbi) {
  OrcDecoder* d = (OrcDecoder*)p;
  const int L = d->max_len, V = d->vocab;
  for (int i = 0; i < d->beam; ++i) {
    if (d->current_indices[i] == -1) continue;
    d->top_sentences[(size_t)i * L + d->current_index + 1] = d->end_symbol;
    d->scores[i] += std::log(outputdist[IDX2C(1, i, V)]) + d->penalty;
    Hypothesis hy;
    hy.words.assign(d->top_sentences.begin() + (size_t)i * L,
                    d->top_sentences.begin() + (size_t)i * L + d->current_index + 2);
    hy.viterbi.assign(d->top_viterbi.begin() + (size_t)i * L,
                      d->top_viterbi.begin() + (size_t)i * L + d->current_index + 2);  // :683-684
    hy.viterbi[d->current_index + 1] = viterbi ? viterbi[i] : -1;
    hy.score = d->scores[i];
    d->hypotheses.push_back(hy);
  }
  d->current_index += 1;
}
void orc_decoder_finish(void* p, const float* outputdist) { orc_decoder_finish_viterbi(p, outputdist, nullptr); }

// a finished hypothesis's alignments, one per word
int orc_decoder_hypothesis_viterbi(void* p, int i, int* out, int cap) {
  const Hypothesis& hy = ((OrcDecoder*)p)->hypotheses[i];
  const int n = (int)hy.viterbi.size();
  for (int k = 0; k < n && k < cap; ++k) out[k] = hy.viterbi[k];
  return n;
}
void orc_decoder_top_viterbi(void* p, int* out) {
  OrcDecoder* d = (OrcDecoder*)p;
  memcpy(out, d->top_viterbi.data(), sizeof(int) * d->top_viterbi.size());
}

void orc_decoder_state(void* p, int* current_indices, int* new_indicies_changes, float* scores, int* top_sentences) {
  OrcDecoder* d = (OrcDecoder*)p;
  for (int i = 0; i < d->beam; ++i) {
    if (current_indices) current_indices[i] = d->current_indices[i];
    if (new_indicies_changes) new_indicies_changes[i] = d->new_indicies_changes[i];
    if (scores) scores[i] = d->scores[i];
  }
  if (top_sentences) memcpy(top_sentences, d->top_sentences.data(), sizeof(int) * d->top_sentences.size());
}

int orc_decoder_current_index(void* p) { return ((OrcDecoder*)p)->current_index; }
int orc_decoder_num_hypotheses(void* p) { return (int)((OrcDecoder*)p)->hypotheses.size(); }
int orc_decoder_hypothesis(void* p, int i, int* words, int cap, float* score) {
  OrcDecoder* d = (OrcDecoder*)p;
  const Hypothesis& hy = d->hypotheses[i];
  const int n = (int)hy.words.size();
  for (int k = 0; k < n && k < cap; ++k) words[k] = hy.words[k];
  *score = hy.score;
  return n;
}

// output_k_best_hypotheses selection, src/decoder.h:1386-1413: indices (into the hypothesis list) of the
// best num_hypotheses finished hypotheses with length/source_length > min_decoding_ratio, best first.
int orc_decoder_k_best(void* p, int source_length, int num_hypotheses, int* out_idx) {
  OrcDecoder* d = (OrcDecoder*)p;
  struct KB {
    float score;
    float index;
  };
  struct KBCmp {
    bool operator()(const KB& a, const KB& b) const { return a.score < b.score; }
  };
  std::priority_queue<KB, std::vector<KB>, KBCmp> best, best_temp;
  for (size_t i = 0; i < d->hypotheses.size(); ++i) {
    const float len_ratio = ((float)d->hypotheses[i].words.size()) / source_length;
    if (len_ratio > d->min_ratio) {
      if ((int)best.size() < num_hypotheses) {
        best.push(KB{-d->hypotheses[i].score, (float)i});
      } else if (-1 * best.top().score < d->hypotheses[i].score) {
        best.pop();
        best.push(KB{-d->hypotheses[i].score, (float)i});
      }
    }
  }
  while (!best.empty()) {
    best_temp.push(KB{-1 * best.top().score, best.top().index});
    best.pop();
  }
  int n = 0;
  while (!best_temp.empty()) {
    out_idx[n++] = (int)best_temp.top().index;
    best_temp.pop();
  }
  return n;
}

// ---------------------------------------------------------------------------
// Composite forward schedules (neuralMT_model::getError, src/model.hpp:1463-1802;
// forward_prop_source, :2367-2452).  Used for end-to-end parity and as the timed CPU baseline.
// ---------------------------------------------------------------------------

// Stacked encoder / LM stack: for t in [0,T): layer 0 (embedding gather + IH node), then layers 1..L-1 (HH
// nodes fed by the layer below at the same t).  Initial h,c per layer given (zeros for the LM / encoder,
// src/model.hpp:1546-1551,1672-1683).
//   weights[l][0..3]=M_g, [4..7]=Wh_g, [8..11]=b_g (gate order i,f,c,o); embed: H x V.
//   ids_nonneg / mask01: time-major [b + t*mb] (src/fileHelper.h:488).
//   h_all, c_all: L x T x (H*mb) (layer-major), every node's h_t and c_t.
void orc_lstm_stack_forward(int acc64, int L, int H, int mb, int T, int V, const float* embed,
                            const float* const* weights, const int* ids_nonneg, const int* mask01,
                            const float* h0, const float* c0, int clip_cell, float clip_threshold, float* h_all,
                            float* c_all) {
  const size_t n = (size_t)H * mb;
  std::vector<float> x(n);
  for (int t = 0; t < T; ++t) {
    for (int l = 0; l < L; ++l) {
      const float* const* w = weights + (size_t)l * 12;
      const float* in;
      if (l == 0) {
        orc_embed_gather(embed, H, V, ids_nonneg + (size_t)t * mb, mb, x.data());
        in = x.data();
      } else {
        in = h_all + ((size_t)(l - 1) * T + t) * n;
      }
      const float* hp = (t == 0) ? h0 + (size_t)l * n : h_all + ((size_t)l * T + t - 1) * n;
      const float* cp = (t == 0) ? c0 + (size_t)l * n : c_all + ((size_t)l * T + t - 1) * n;
      orc_lstm_step(acc64, H, mb, w, w + 4, nullptr, w + 8, in, hp, cp, nullptr, mask01 + (size_t)t * mb,
                    clip_cell, clip_threshold, nullptr, nullptr, nullptr, nullptr,
                    c_all + ((size_t)l * T + t) * n, h_all + ((size_t)l * T + t) * n);
    }
  }
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------------------
// Backward pass (training).  Gradients are those of the LOG-LIKELIHOOD (the reference ascends: its softmax error
// is D^T (onehot - p), src/softmax.hpp:700-712, and update_weights adds learning_rate * gradient, :232-300).
// ---------------------------------------------------------------------------------------------------------
namespace {

// C(MxN) = A * B^T with A stored M x K and B stored N x K (cublasSgemm OP_N, OP_T: the weight-gradient products,
// e.g. src/LSTM.hpp:1026-1100).  Always double accumulation.
void gemm_nt64(int M, int N, int K, const float* A, int lda, const float* B, int ldb, double* C, int ldc, bool add) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int n = 0; n < N; ++n)
    for (int m = 0; m < M; ++m) {
      double s = 0;
      for (int k = 0; k < K; ++k) s += (double)A[IDX2C(m, k, lda)] * (double)B[IDX2C(n, k, ldb)];
      if (add)
        C[IDX2C(m, n, ldc)] += s;
      else
        C[IDX2C(m, n, ldc)] = s;
    }
}

}  // namespace

extern "C" {

// One node's element-wise backward.  d_ERRt_ct_kernel, d_ERRnTOt_ot_kernel, d_ERRnTOt_ft_it_kernel,
// d_ERRnTOt_tanhcpt_kernel and zero_columns_kernel (src/custom_kernels.h:199-262), in the order of
// LSTM_IH_Node::back_prop_GPU (src/LSTM.hpp:542-700).
//   err_h: d_ERRnTOtp1_ht + d_ERRt_ht, the total error arriving at h_t; err_c_next: d_ERRnTOtp1_ct.
//   gates i, f, c~ (tanh), o and c_t, c_{t-1} as saved by the forward step.
//   Outputs: dgate[4] = error at the four PRE-activations (the reference's d_ERRnTOt_it, _ft, _tanhcpt, _ot), gate
//   order i,f,c,o; err_cprev = error passed to c_{t-1} (d_ERRnTOt_ct * f_t).
void orc_lstm_step_backward(int H, int mb, const float* gi, const float* gf, const float* gc, const float* go,
                            const float* c, const float* cprev, const int* mask01, const float* err_h,
                            const float* err_c_next, float* dgate_i, float* dgate_f, float* dgate_c, float* dgate_o,
                            float* err_cprev) {
  for (int col = 0; col < mb; ++col)
    for (int i = 0; i < H; ++i) {
      const size_t ix = IDX2C(i, col, H);
      const float m = (float)mask01[col];
      const float eh = err_h[ix] * m;  // zero_columns_kernel on d_ERRnTOt_ht
      const float th = tanhf(c[ix]);
      const float errt_ct = eh * go[ix] * (1.0f - th * th);                      // d_ERRt_ct_kernel
      const float ec = ((err_c_next ? err_c_next[ix] : 0.0f) + errt_ct) * m;     // d_ERRnTOt_ct, zero_columns_kernel
      dgate_o[ix] = eh * th * go[ix] * (1.0f - go[ix]);                           // d_ERRnTOt_ot_kernel
      dgate_f[ix] = ec * cprev[ix] * gf[ix] * (1.0f - gf[ix]);                    // d_ERRnTOt_ft_it_kernel
      dgate_i[ix] = ec * gc[ix] * gi[ix] * (1.0f - gi[ix]);                       // d_ERRnTOt_ft_it_kernel
      dgate_c[ix] = ec * gi[ix] * (1.0f - gc[ix] * gc[ix]);                       // d_ERRnTOt_tanhcpt_kernel
      err_cprev[ix] = ec * gf[ix];                                                // elementwise_mult (:750-760)
    }
}

// Forward sweep with saved gates, then back-propagation through time of the stacked LSTM (no attention, no dropout):
// the loops of neuralMT_model::compute_gradients (src/model.hpp:1823-2000) over LSTM_IH_Node / LSTM_HH_Node
// back_prop_GPU and compute_gradients_GPU (src/LSTM.hpp:542-1270, src/LSTM_HH.hpp:336-900).
//   weights as in orc_lstm_stack_forward.  err_top: T x (H*mb), error arriving at the top layer's h_t from the
//   loss layer (d_ERRt_ht).  err_hT / err_cT: L x (H*mb) errors arriving at the last time step from beyond (NULL = 0).
//   Outputs (double accumulation, rounded once): grads[l][0..3] = dM_g, [4..7] = dWh_g (H x H), [8..11] = db_g (H);
//   d_embed: H x V dense (zero where no token hit); err_h0 / err_c0: L x (H*mb) errors at the initial states.
//   cell_clip > 0: BZ_CUDA::clip_cell with that cell_clip_threshold in the forward sweep (src/LSTM.hpp:369-371; the
//   backward pass uses the clamped c_t and passes errors through the clamp unchanged), and err_clip as
//   BZ_CUDA::error_clip_threshold: the error a node sends to h_{t-1} (src/LSTM.hpp:792, src/LSTM_HH.hpp:756) and the
//   error a layer above the first sends to the layer below (src/LSTM_HH.hpp:665) are clamped to +-err_clip, each on
//   its own, before they are added to anything.  (The reference's third clamp, of d_ERRnTOt_ct at src/LSTM.hpp:888 /
//   src/LSTM_HH.hpp:774, is queued behind that array's last use in the node and changes no output: not restated.)
void orc_lstm_stack_backward_clip(int L, int H, int mb, int T, int V, const float* embed, const float* const* weights,
                                  const int* ids_nonneg, const int* mask01, const float* h0, const float* c0,
                                  const float* err_top, const float* err_hT, const float* err_cT, float cell_clip,
                                  float err_clip, float* const* grads, float* d_embed, float* err_h0, float* err_c0);
void orc_lstm_stack_backward(int L, int H, int mb, int T, int V, const float* embed, const float* const* weights,
                             const int* ids_nonneg, const int* mask01, const float* h0, const float* c0,
                             const float* err_top, const float* err_hT, const float* err_cT, float* const* grads,
                             float* d_embed, float* err_h0, float* err_c0) {
  orc_lstm_stack_backward_clip(L, H, mb, T, V, embed, weights, ids_nonneg, mask01, h0, c0, err_top, err_hT, err_cT, 0.0f,
                               0.0f, grads, d_embed, err_h0, err_c0);
}
void orc_lstm_stack_backward_clip(int L, int H, int mb, int T, int V, const float* embed, const float* const* weights,
                                  const int* ids_nonneg, const int* mask01, const float* h0, const float* c0,
                                  const float* err_top, const float* err_hT, const float* err_cT, float cell_clip,
                                  float err_clip, float* const* grads, float* d_embed, float* err_h0, float* err_c0) {
  auto clamp_errors = [&](float* e, size_t count) {  // clip_mat_kernel, src/custom_kernels.h:2220-2231
    if (!(cell_clip > 0.0f)) return;
    for (size_t i = 0; i < count; ++i) e[i] = e[i] > err_clip ? err_clip : (e[i] < -err_clip ? -err_clip : e[i]);
  };
  const size_t n = (size_t)H * mb;
  const size_t LT = (size_t)L * T;
  std::vector<float> h_all(LT * n), c_all(LT * n), g_all(LT * 4 * n), x_all((size_t)T * n);
  // forward, keeping the gates
  for (int t = 0; t < T; ++t)
    for (int l = 0; l < L; ++l) {
      const float* const* w = weights + (size_t)l * 12;
      const float* in;
      if (l == 0) {
        orc_embed_gather(embed, H, V, ids_nonneg + (size_t)t * mb, mb, x_all.data() + (size_t)t * n);
        in = x_all.data() + (size_t)t * n;
      } else {
        in = h_all.data() + ((size_t)(l - 1) * T + t) * n;
      }
      const float* hp = (t == 0) ? h0 + (size_t)l * n : h_all.data() + ((size_t)l * T + t - 1) * n;
      const float* cp = (t == 0) ? c0 + (size_t)l * n : c_all.data() + ((size_t)l * T + t - 1) * n;
      float* g = g_all.data() + ((size_t)l * T + t) * 4 * n;
      orc_lstm_step(1, H, mb, w, w + 4, nullptr, w + 8, in, hp, cp, nullptr, mask01 + (size_t)t * mb,
                    cell_clip > 0.0f ? 1 : 0, cell_clip, g, g + n, g + 2 * n, g + 3 * n,
                    c_all.data() + ((size_t)l * T + t) * n, h_all.data() + ((size_t)l * T + t) * n);
    }
  // backward
  std::vector<double> acc((size_t)L * 8 * H * H, 0.0), accb((size_t)L * 4 * H, 0.0), acce((size_t)H * V, 0.0);
  std::vector<float> eh_next((size_t)L * n, 0.0f), ec_next((size_t)L * n, 0.0f);  // from t+1, per layer
  if (err_hT) memcpy(eh_next.data(), err_hT, sizeof(float) * L * n);
  if (err_cT) memcpy(ec_next.data(), err_cT, sizeof(float) * L * n);
  std::vector<float> below(n), eh(n), dg(4 * n), ecp(n), tmp(n);
  for (int t = T - 1; t >= 0; --t) {
    std::fill(below.begin(), below.end(), 0.0f);
    for (int l = L - 1; l >= 0; --l) {
      const float* const* w = weights + (size_t)l * 12;
      const float* g = g_all.data() + ((size_t)l * T + t) * 4 * n;
      const float* cp = (t == 0) ? c0 + (size_t)l * n : c_all.data() + ((size_t)l * T + t - 1) * n;
      const float* hp = (t == 0) ? h0 + (size_t)l * n : h_all.data() + ((size_t)l * T + t - 1) * n;
      const float* in = (l == 0) ? x_all.data() + (size_t)t * n : h_all.data() + ((size_t)(l - 1) * T + t) * n;
      // total error at h_t: from t+1 plus from above (the loss layer for the top layer)
      const float* from_above = (l == L - 1) ? err_top + (size_t)t * n : below.data();
      for (size_t i = 0; i < n; ++i) eh[i] = eh_next[(size_t)l * n + i] + from_above[i];
      orc_lstm_step_backward(H, mb, g, g + n, g + 2 * n, g + 3 * n, c_all.data() + ((size_t)l * T + t) * n, cp,
                             mask01 + (size_t)t * mb, eh.data(), ec_next.data() + (size_t)l * n, dg.data(),
                             dg.data() + n, dg.data() + 2 * n, dg.data() + 3 * n, ecp.data());
      memcpy(ec_next.data() + (size_t)l * n, ecp.data(), sizeof(float) * n);
      // errors to h_{t-1} and to the layer below: sum over the gates of W^T dgate
      std::fill(eh_next.begin() + (size_t)l * n, eh_next.begin() + (size_t)(l + 1) * n, 0.0f);
      std::fill(below.begin(), below.end(), 0.0f);
      for (int q = 0; q < 4; ++q) {
        gemm_tn(1, H, mb, H, w[4 + q], H, dg.data() + (size_t)q * n, H, tmp.data(), H);
        for (size_t i = 0; i < n; ++i) eh_next[(size_t)l * n + i] += tmp[i];
        gemm_tn(1, H, mb, H, w[q], H, dg.data() + (size_t)q * n, H, tmp.data(), H);
        for (size_t i = 0; i < n; ++i) below[i] += tmp[i];
        // weight gradients: dM_g += dgate x^T, dWh_g += dgate h_{t-1}^T, db_g += row sums
        gemm_nt64(H, H, mb, dg.data() + (size_t)q * n, H, in, H, acc.data() + ((size_t)l * 8 + q) * H * H, H, true);
        gemm_nt64(H, H, mb, dg.data() + (size_t)q * n, H, hp, H, acc.data() + ((size_t)l * 8 + 4 + q) * H * H, H, true);
        for (int col = 0; col < mb; ++col)
          for (int i = 0; i < H; ++i) accb[((size_t)l * 4 + q) * H + i] += dg[(size_t)q * n + IDX2C(i, col, H)];
      }
      clamp_errors(eh_next.data() + (size_t)l * n, n);
      if (l > 0) clamp_errors(below.data(), n);
      if (l == 0) {  // sparse embedding gradient (W_gradient kernels, src/custom_kernels.h:1297-1390), dense here
        for (int col = 0; col < mb; ++col) {
          if (mask01[(size_t)t * mb + col] != 1) continue;
          const int id = ids_nonneg[(size_t)t * mb + col];
          for (int i = 0; i < H; ++i) acce[IDX2C(i, id, H)] += below[IDX2C(i, col, H)];
        }
      }
    }
  }
  for (int l = 0; l < L; ++l) {
    for (int q = 0; q < 8; ++q)
      for (size_t i = 0; i < (size_t)H * H; ++i) grads[(size_t)l * 12 + q][i] = (float)acc[((size_t)l * 8 + q) * H * H + i];
    for (int q = 0; q < 4; ++q)
      for (int i = 0; i < H; ++i) grads[(size_t)l * 12 + 8 + q][i] = (float)accb[((size_t)l * 4 + q) * H + i];
  }
  for (size_t i = 0; i < (size_t)H * V; ++i) d_embed[i] = (float)acce[i];
  memcpy(err_h0, eh_next.data(), sizeof(float) * L * n);
  memcpy(err_c0, ec_next.data(), sizeof(float) * L * n);
}

// Loss-layer backward for one step: softmax_layer::get_h_t_gradient_GPU, compute_D_gradient_GPU and
// compute_b_d_gradient_GPU (src/softmax.hpp:700-860).  With p = softmax(D h + b) per column and e = onehot(target) - p
// on unmasked columns (0 on masked ones):  err_h = D^T e (H x mb),  dD += e h^T (V x H),  db += row sums of e.
// dD / db accumulate (double) across calls when `add` is set.
void orc_softmax_backward(const float* D, const float* b_d, int V, int H, const float* h, int mb, const int* target,
                          const int* mask01, int add, float* err_h, double* dD, double* db) {
  std::vector<float> logits((size_t)V * mb), e((size_t)V * mb);
  std::vector<double> logp((size_t)V * mb);
  orc_softmax_logits(1, D, b_d, V, H, h, mb, logits.data());
  orc_softmax_logprob_f64(logits.data(), V, mb, logp.data());
  for (int col = 0; col < mb; ++col)
    for (int v = 0; v < V; ++v) {
      const size_t ix = IDX2C(v, col, V);
      double val = -exp(logp[ix]);
      if (v == target[col]) val += 1.0;
      e[ix] = mask01[col] == 1 ? (float)val : 0.0f;
    }
  gemm_tn(1, H, mb, V, D, V, e.data(), V, err_h, H);
  gemm_nt64(V, H, mb, e.data(), V, h, H, dD, V, add != 0);
  for (int v = 0; v < V; ++v) {
    double s = 0;
    for (int col = 0; col < mb; ++col) s += e[IDX2C(v, col, V)];
    db[v] = add ? db[v] + s : s;
  }
}

}  // extern "C"
