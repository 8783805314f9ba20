// Internal declarations shared by the HIP translation units of libzoph_rnn_hip.so.
#ifndef ZR_INTERNAL_H
#define ZR_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/zoph_rnn.h"

#define ZR_MAX_COUNTERS 4096
#define ZR_MAX_PACKED_D 8

struct zr_ctx {
  int device;
  hipStream_t own_stream;
  hipStream_t stream;  // the stream in use (own_stream or a caller-provided one)
  int* d_flags;        // [0]: count of token ids seen outside [0, V); [1]: attention table index clamps;
                       // [2]: a workgroup of the whole-sweep LSTM kernel abandoned a wait
  hipEvent_t ev_start, ev_stop;  // zr_timer_start / zr_timer_stop
  // options
  int lstm_fused;
  int lstm_tn;
  int lstm_ksplit;
  int lstm_kernel;   // 0 auto, 1 register-streaming kernel, 2 LDS / split-K kernel
  int lstm_kparts;   // K parts per segment for the split-K kernel (0 auto)
  int* d_counters;   // ZR_MAX_COUNTERS arrival counters, zero between launches
  int lstm_sweep;    // whole-sweep LSTM kernel: 0 auto, 1 never, 2 whenever the launch fits on the device
  int sweep_spin;    // polls before a waiting workgroup of that kernel gives up (0: default)
  int step_wait_extra;  // arrivals the decoder step's layer waits expect beyond the real ones (tests of giving up)
  int stack_helpers;    // 1 (default): the decoder step may run 32-column tiles with helper workgroups (zr_lstm.hip)
  int cu_count;      // compute units of the device (filled with sweep_capacity)
  int sweep_capacity[3];  // resident workgroups of lstm_sweep_kernel<TN> (0: not asked yet, -1: unknown)
  int stack_step_capacity;  // the same for lstm_decoder_stack_kernel (the lesser of its two tile widths)
  int attn_step_capacity[3];  // the same for attn_step_kernel<8 / 16 / 32>
  int attn_single;      // ZR_OPT_ATTN_SINGLE_LAUNCH
  int last_attn_path;   // ZR_ATTN_PATH_* of the last attention step (0: none yet)
  int gemm_cfg;
  int bf16_terms;       // bf16-weight products: 2 (default, 0 = 2) = activations as two bf16 terms, 1 = rounded to bf16 once
  int last_stack_path;  // ZR_LSTM_STACK_PATH_* of the last zr_lstm_stack_forward(_train) call (0: none yet)
  // scratch owned by the context (grown on demand, never shrunk)
  void* d_scratch;
  size_t scratch_bytes;
  void* d_scratch2;
  size_t scratch2_bytes;
  // the device's statically allocated scratch array (zr_runtime.hip), resolved when the context is created
  void* d_static_scratch;
  // while set, zr_ctx_scratch hands out these fixed buffers (slot 0 / slot 1) and never allocates
  int fixed_scratch;
  void* d_fixed[2];
  size_t fixed_bytes[2];
  // output-layer matrices registered with zr_softmax_prepare: the caller's D pointer -> its k-interleaved copy
  struct PackedD {
    const float* key;  // the caller's d_D (null: slot free)
    int V, H;
    int ldp;           // V rounded up to 32
    int bf16;          // 0: d_pack is fp32 [ceil8(H)/4][ldp][4]; 1: bf16 [H/8][ldp][8]
    void* d_pack;
  } packed_d[ZR_MAX_PACKED_D];
};

// error plumbing -------------------------------------------------------------------------------------------
int zr_set_error(int code, const char* fmt, ...);

#define ZR_CHECK_ARG(cond, ...)                  \
  do {                                           \
    if (!(cond)) return zr_set_error(ZR_EINVAL, __VA_ARGS__); \
  } while (0)

#define ZR_HIP(call)                                                                        \
  do {                                                                                      \
    hipError_t zr_e_ = (call);                                                              \
    if (zr_e_ != hipSuccess)                                                                \
      return zr_set_error(ZR_EHIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(zr_e_), \
                          __FILE__, __LINE__);                                              \
  } while (0)

#define ZR_LAUNCH_CHECK(name)                                                                  \
  do {                                                                                         \
    hipError_t zr_e_ = hipGetLastError();                                                      \
    if (zr_e_ != hipSuccess)                                                                   \
      return zr_set_error(ZR_EHIP, "launch of %s failed: %s", name, hipGetErrorString(zr_e_)); \
  } while (0)

int zr_bind_device(zr_ctx* ctx);
// Number of contexts of this process that are alive on `device`.
int zr_live_contexts(int device);
// Returns a context-owned scratch buffer of at least `bytes` (slot 0 or 1).
int zr_ctx_scratch(zr_ctx* ctx, int slot, size_t bytes, void** out);
// Size of the statically allocated device scratch array every GPU holds for the allocation-free entry point, and
// how that entry point divides it between the two scratch slots.
#define ZR_STATIC_SCRATCH_BYTES (32u << 20)
#define ZR_STATIC_SCRATCH_SLOT0_BYTES (8u << 20)

// MFMA vector types ------------------------------------------------------------------------------------------
typedef float zr_f32x16 __attribute__((ext_vector_type(16)));
typedef float zr_f32x4 __attribute__((ext_vector_type(4)));

// Generic multi-segment GEMM: C = sum_s op(A_s) * B_s, then an epilogue.  Up to 3 segments.
enum ZrEpilogue {
  ZR_EPI_STORE = 0,           // C = acc (+ bias[m] if bias)
  ZR_EPI_TANH = 1,            // C = tanhf(acc)
  ZR_EPI_TANH_BIAS_MASK = 2,  // C = tanhf(acc + bias[m]) * mask[n]
  ZR_EPI_SOFTMAX_PARTIAL = 3  // C = acc + bias[m]; per (n, 32-row block) partial (max, sum exp) -> partials
};

struct ZrGemmDesc {
  int M, N;
  int nseg;
  int K[3];
  const float* A[3];
  int lda[3];
  int trans_a;  // applies to every segment
  // 1: A is k-interleaved fp32: element (m, k) at ((k/4)*lda + m)*4 + k%4, lda = M rounded up to 32, K padded to
  //    a multiple of 8, pads zero (ZR_A_PACK4 in zr_mfma_core.h).
  // 2: A is k-interleaved bf16 (2-byte elements behind the float pointer): element (m, k) at
  //    ((k/8)*lda + m)*8 + k%8, K a multiple of 16 (ZR_A_PACK8_BF16).
  // Single batch, no transpose.
  int a_pack;
  const float* B[3];
  int ldb[3];
  float* C;
  int ldc;
  // batch (blockIdx.z): A/C/bias advance by these strides (elements; bf16 elements for a bf16 A); B is shared
  int batch;
  long long strideA, strideC, strideBias;
  const float* bias;  // per row m (may be NULL)
  const int* mask;    // per column n (ZR_EPI_TANH_BIAS_MASK)
  int epilogue;
  float* partials;  // ZR_EPI_SOFTMAX_PARTIAL: [N][ceil(M/32)][2] floats (contiguous per column)
  float* Cpack;     // ZR_EPI_TANH_BIAS_MASK, single batch: the result is also stored k-interleaved, element (m, n) at
                    // ((m/4)*N + n)*4 + m%4 -- the layout a following product with b_packed reads (null: not wanted)
  // ZR_EPI_TANH_BIAS_MASK, single batch, M % 8 == 0: the result also as bf16 terms (hi, and lo = the residue, or null),
  // each laid out [M/8][N][8] -- what a following product on bf16 weights reads as Bhi / Blo (null: not wanted)
  unsigned short* Chi;
  unsigned short* Clo;
  int accumulate;   // ZR_EPI_STORE only: C += product (+ bias) instead of C = ...
  // A is read once per step and is a large part of the memory-side cache: fetch it with the non-temporal hint so that
  // it does not push out what the rest of the step reads again (honoured by the kernel of the output layer's product)
  int stream_a;
  // groups > 0: that many independent problems of the same shape in one launch (at most 8; one segment, plain store
  // epilogue, no bias): problem g multiplies gA[g] (instead of A[0]) with gB[g] (instead of B[0]) into gC[g]
  // (instead of C); lda/ldb/ldc, the batch count and its strides apply inside every problem.
  // a_pack == 2: segment s's activations already split and k-interleaved by 8 (zr_split_pack_x_launch's layout): the
  // bf16 "hi" array, and the "lo" array in two-term mode (null entries: the launch splits B[s] itself)
  const unsigned short* Bhi[3];
  const unsigned short* Blo[3];
  int b_packed;  // with a_pack == 1: B (and every gB) is already k-interleaved, element (k, n) at ((k/4)*N + n)*4 + k%4
                 // (K a multiple of 8, 16-byte aligned); ldb is ignored
  int groups;
  const float* gA[8];
  const float* gB[8];
  float* gC[8];
};

int zr_gemm_launch(zr_ctx* ctx, const ZrGemmDesc& d);
// Packs one M x K column-major matrix (leading dimension ld) into the k-interleaved layout [kp/4][ldp][4] with
// zero padding (ldp >= M a multiple of 32, kp >= K a multiple of 8).  dst holds kp*ldp floats.
int zr_pack4_launch(zr_ctx* ctx, const float* src, int M, int K, long long ld, int ldp, int kp, float* dst);
// Activations X (K x N fp32, column n at src + n*ld, K % 4 == 0, 16-byte aligned) into the k-interleaved layout
// [K/4][N][4] (element (k, n) at ((k/4)*N + n)*4 + k%4).
int zr_pack4_x_launch(zr_ctx* ctx, const float* src, int K, int N, int ld, float* dst);
// The same from the transpose: element (row, k) of the packed matrix is src[k + row*ld].
int zr_pack4_trans_launch(zr_ctx* ctx, const float* src, int M, int K, long long ld, int ldp, int kp, float* dst);
// Same for the bf16 layout [kp/8][ldp][8] (round to nearest even); kp a multiple of 16.  dst holds kp*ldp elements.
// Activations X (K x N fp32, column-major with leading dimension ld, K % 8 == 0) split into bf16 hi + lo arrays
// (K*N elements each), both k-interleaved by 8.
// n_src (at most 12) K x N matrices split in one launch: matrix i to hi + i*stride (and lo + i*stride; lo null: single
// term).  d_ids non-null: matrix 0 is gathered, column n read from srcs[0] + clamp(d_ids[n], 0, V-1)*ld.
int zr_split_pack_multi_launch(zr_ctx* ctx, int n_src, const float* const* srcs, const int* d_ids, int V, int K, int N,
                               int ld, unsigned short* hi, unsigned short* lo, long long stride);
int zr_split_pack_x_launch(zr_ctx* ctx, const float* src, int K, int N, int ld, unsigned short* hi,
                           unsigned short* lo);
// trans != 0: the source holds the transpose (element (row, k) at src[k + row*ld]).
int zr_pack8_bf16_launch(zr_ctx* ctx, const float* src, int M, int K, long long ld, int ldp, int kp,
                         unsigned short* dst, int trans = 0);
// number of 32-row partial blocks the SOFTMAX_PARTIAL epilogue writes for M rows
static inline int zr_softmax_partial_blocks(int M) { return (M + 31) / 32; }
// ZR_SOFTMAX_LOGITS_BLOCKS: where the block pairs start in d_out (floats; a multiple of 4 behind the V x cols logits)
static inline size_t zr_softmax_blocks_offset_floats(int V, int cols) { return ((size_t)V * cols + 3) & ~(size_t)3; }
// softmax_colstats_kernel on [cols][nblocks][2] pairs -> colstats[cols][2] (zr_softmax.hip)
int zr_softmax_colstats_launch(zr_ctx* ctx, const float* d_partials, int nblocks, int cols, float* d_colstats);

struct zr_lstm_weights {
  int H;
  int nseg;        // 2 (M, Wh) or 3 (+Q)
  int bf16;        // 0: fp32 matrices, k-interleaved by 4; 1: bf16 matrices, k-interleaved by 8
  int ldw;         // H rounded up to 32: rows per packed k-block (rows >= H hold zeros)
  int kp;          // packed K extent: H rounded up to 8 (fp32) or 16 (bf16); k >= H hold zeros
  // [nseg][4] matrices.  fp32: each [kp/4][ldw][4], element (row, k) at ((k/4)*ldw + row)*4 + k%4.
  // bf16: each [kp/8][ldw][8], element (row, k) at ((k/8)*ldw + row)*8 + k%8 (2-byte elements).
  // A 32-row tile of one k-block is 512 contiguous, 128-byte aligned bytes, read with one 16-byte load per lane.
  void* d_W;
  float* d_bias;   // [4][H]
};

// Pieces of zr_decoder_step (zr_attention.hip): the three public calls with the hand-overs between them kept in the
// k-interleaved layout.  d_hp_top (zr_lstm_decoder_step): where the top layer's h is also written as [H/4][mb][4];
// *wrote_hp_top tells whether it was (only the single-launch path does).  With bf16 weights d_hp_top instead receives
// the top layer's h as bf16 terms, k-interleaved by 8: H*mb hi terms, then (two-term mode) H*mb lo terms.  h_packed (zr_attn_step): a->d_hpack already
// holds that copy of d_h_t; d_htild_pack: h~ is also written k-interleaved there.  d_h_packed (zr_softmax_forward):
// a k-interleaved copy of d_h, used when the registered matrix allows it.
int zr_lstm_decoder_step_packed(zr_ctx* ctx, int nl, const zr_lstm_weights* const layers[], const float* d_embed, int V,
                                const int* d_ids_nonneg, const float* const d_hprev[], const float* const d_cprev[],
                                const float* d_htild, const int* d_mask01, float clip_threshold, int mb,
                                float* const d_h[], float* const d_c[], float* d_hp_top, int* wrote_hp_top);
int zr_softmax_forward_packed(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h,
                              const float* d_h_packed, int mb, int mode, float* d_out, float* d_logits_scratch,
                              const unsigned short* d_h_hi = nullptr, const unsigned short* d_h_lo = nullptr);

// The attention step in one launch (zr_attn_step.hip).  a->d_hpack must hold h_t k-interleaved.  *took = 0: the
// conditions do not hold and nothing was launched (the caller goes on with one launch per stage).
struct zr_attn;
int zr_attn_step_single_launch(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const int* d_mask01, float* d_htild,
                               float* d_htild_pack, float* align, int* idx, float* pt, float* cctx, int* took);

// The attention layer's handle (zr_attention.hip; the backward pass lives in zr_backward.hip).
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
  // zr_attn_prepare: owned fp32 k-interleaved snapshots ([kp/4][ldp32][4] each) of W_p, W_a^T, W_c1, W_c2 in that
  // order, and the raw (pre-tanh) W_p h product next to q
  float* d_pack32;
  int ldp32, kp32;
  float *d_hpack, *d_cpack;  // k-interleaved copies ([H/4][mb][4]) of h_t and of the context (inside d_pack32's block)
  float* d_htpack;           // the same of h~, written by the output product for zr_decoder_step (same block)
  bool wrote_htild_pack;     // the last attention step wrote d_htpack
  float* d_pq;               // single-launch step: W_p h_t, W_a^T h_t and the context in padded columns (3 x ldp32 x mb,
                             // same block, 128-byte aligned)
  // bf16 matrices: h~ of the last step as bf16 terms ([H/8][mb][8], inside d_bf16's block), written by the output
  // product for a bf16 output layer behind it in zr_decoder_step; null when the last step did not write them
  const unsigned short* htild_hi;
  const unsigned short* htild_lo;
  float** d_err_table;       // zr_attn_set_error_tables: device copy of the source-state error pointers (null: none)
};

#endif
