/*
 * zoph_rnn.h -- C-ABI of the MI355X (gfx950) implementation of Zoph_RNN's stacked-LSTM forward path.
 *
 * The reference (isi-nlp/Zoph_RNN) has no FFI: the path lives behind C++ template members compiled into one
 * translation unit.  Each entry point below states which reference member / kernel / cuBLAS call site it
 * replaces (paths relative to the reference root).  The C++ classes under zoph_rnn_amd/host/ keep the
 * reference's class and member names and forward to these functions.
 *
 * Conventions
 *   - every function returns 0 on success and a negative ZR_E* code on failure; zr_last_error() returns a
 *     message for the calling thread.  Nothing here aborts the process (the reference exits on any CUDA
 *     error, src/BZ_CUDA_UTIL.h:193-270).
 *   - all matrices are column-major fp32 (IDX2C, src/BZ_CUDA_UTIL.h:26): activations are H x minibatch, the
 *     embedding is H x V, the softmax matrix D is V x H.
 *   - pointers named d_* are device pointers on the context's GPU, h_* are host pointers.
 *   - a context owns one in-order HIP stream; calls on one context are asynchronous with respect to the host
 *     and ordered with respect to each other.  A context is not re-entrant.
 *   - gate order everywhere is i, f, c, o (the reference's temp1..8 / i_t, f_t, c_prime_t_tanh, o_t order).
 */
#ifndef ZOPH_RNN_H
#define ZOPH_RNN_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ZR_OK 0
#define ZR_EINVAL (-1)   /* bad argument (null pointer, non-positive size, unsupported shape) */
#define ZR_EHIP (-2)     /* a HIP runtime call failed */
#define ZR_ENOMEM (-3)   /* device allocation failed */
#define ZR_EDATA (-4)    /* device-side data check failed (token id outside [0, V), ...) */

typedef struct zr_ctx zr_ctx;
typedef struct zr_lstm_weights zr_lstm_weights;
typedef struct zr_beam zr_beam;

/* ---- runtime ------------------------------------------------------------------------------------------ */

/* Replaces layer_gpu_info::init / softmax_layer_gpu_info::init (src/gpu_info_struct.h:67-172: per-layer
 * cudaSetDevice, 9+ streams, ~50 events, cublasCreate).  One in-order stream replaces the stream/event DAG. */
int zr_ctx_create(int device, zr_ctx** out);
int zr_ctx_destroy(zr_ctx* ctx);
/* devSynchAll (src/BZ_CUDA_UTIL.h:977-987) followed by CUDA_GET_LAST_ERROR (:262-270): waits for the stream and
 * reports launch errors and the device-side data flag (ZR_EDATA) instead of exiting. */
int zr_ctx_sync(zr_ctx* ctx);
/* Use a caller-owned hipStream_t (passed as void*) instead of the context's own; NULL restores the own stream. */
int zr_ctx_set_stream(zr_ctx* ctx, void* hip_stream);
/* Device-side timing of everything queued on the context's stream between the two calls (HIP events).  The
 * reference brackets phases with host wall-clock Timer objects after devSynchAll (src/memory_util.h:87-124,
 * src/model.hpp:2576-2686).  zr_timer_stop waits for the stream and returns milliseconds. */
int zr_timer_start(zr_ctx* ctx);
int zr_timer_stop(zr_ctx* ctx, float* h_ms);
/* Tuning / mode switches: see ZR_OPT_* below. */
int zr_ctx_set_option(zr_ctx* ctx, int option, int value);
/* State of the context that a caller may want to look at (no counterpart in the reference):
 *   ZR_QUERY_LSTM_STACK_PATH: which schedule the last zr_lstm_stack_forward(_train) or zr_lstm_decoder_step call on
 *     this context took -- 0 none yet, ZR_LSTM_STACK_PATH_SWEEP (one launch for the whole sweep),
 *     ZR_LSTM_STACK_PATH_DIAGONALS (one launch per diagonal), ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH or
 *     ZR_LSTM_STACK_PATH_STEP_PER_LAYER (zr_lstm_decoder_step).  Does not wait.
 *   ZR_QUERY_LSTM_SWEEP_ABANDONED: waits for the stream; 1 if a single-launch sweep or decoder step since the last look
 *     gave up a wait (its outputs were then overwritten with NaN; run it again with ZR_OPT_LSTM_SWEEP = 1), else 0.  Clears
 *     the flag -- and with it the data flags that launches queued behind the abandoned one raised on its NaN outputs --
 *     so a following zr_ctx_sync no longer reports it.  A decoder step called with d_c[l] == d_cprev[l] (cell state
 *     updated in place) has overwritten its own input by then: running it again needs the caller's copy of c_{t-1}.
 *   ZR_QUERY_SCRATCH_KIB: device memory the context has allocated for scratch buffers so far, in KiB (0 for a context
 *     that has only served calls that allocate nothing).  Does not wait.
 *   ZR_QUERY_ATTN_PATH: which schedule the last zr_attn_step (or the attention part of zr_decoder_step) on this
 *     context took -- 0 none yet, ZR_ATTN_PATH_SINGLE_LAUNCH, ZR_ATTN_PATH_THREE_LAUNCHES or ZR_ATTN_PATH_SEPARATE.
 *     Does not wait. */
int zr_ctx_query(zr_ctx* ctx, int what, int* h_value);
#define ZR_QUERY_LSTM_STACK_PATH 1
#define ZR_QUERY_LSTM_SWEEP_ABANDONED 2
#define ZR_QUERY_ATTN_PATH 3
#define ZR_QUERY_SCRATCH_KIB 4
#define ZR_ATTN_PATH_SINGLE_LAUNCH 1  /* projections, window / scores / context and output product in one launch */
#define ZR_ATTN_PATH_THREE_LAUNCHES 2 /* the same three stages as one launch each */
#define ZR_ATTN_PATH_SEPARATE 3       /* unprepared or bf16 matrices: products and the middle as separate launches */
#define ZR_LSTM_STACK_PATH_SWEEP 1
#define ZR_LSTM_STACK_PATH_DIAGONALS 2
#define ZR_LSTM_STACK_PATH_STEP_SINGLE_LAUNCH 3 /* zr_lstm_decoder_step: all layers in one launch */
#define ZR_LSTM_STACK_PATH_STEP_PER_LAYER 4     /* zr_lstm_decoder_step: one launch per layer */
const char* zr_last_error(void);
/* Library self-description: "gfx950 hip <build tag>". */
const char* zr_version(void);

#define ZR_OPT_LSTM_FUSED_EPILOGUE 1 /* 1 (default): gate maths in the GEMM epilogue; 0: GEMM then zr_lstm_gates */
#define ZR_OPT_LSTM_TN 2             /* columns per workgroup / 32 for the fused LSTM kernel: 1, 2 or 4 (0 = auto) */
#define ZR_OPT_GEMM_CFG 3            /* generic GEMM tile selection, for tuning runs (0 = auto).  Plain weights: 1..8 =
                                        wave tiles 64x128, 32x128, 32x64, 32x32, 32x32 K/4, 32x32 K/8, 64x64, 32x64 K/4;
                                        9 = LDS-shared rows, 10 = LDS-shared rows with 128-row tiles.  Prepared
                                        (k-interleaved) weights: 11 = one tile per workgroup instead of row ranges,
                                        12..14 = tiles 128x64, 64x64, 64x128 at one workgroup per CU */
#define ZR_OPT_LSTM_KSPLIT 4         /* waves per workgroup splitting K in the fused LSTM kernel: 4 or 8 (0 = auto) */
#define ZR_OPT_LSTM_KERNEL 5         /* 0 auto; 1: weights streamed to registers, K split inside the workgroup;
                                        2: weights through LDS, K split across workgroups;
                                        3: weights streamed to registers, K split inside and across workgroups */
#define ZR_OPT_LSTM_KPARTS 6         /* kernels 2 and 3: K parts per weight segment (0 = auto) */
#define ZR_OPT_LSTM_SWEEP 7          /* zr_lstm_stack_forward as ONE launch whose workgroups hand h to each other
                                        through device memory: 0 auto (when they fill most of the device, are all
                                        resident at once, the context is the process's only one on its device and
                                        runs on its own stream),
                                        1 never (one launch per diagonal), 2 whenever they fit.  The environment
                                        variable ZR_LSTM_SWEEP presets this option for every context created */
#define ZR_OPT_LSTM_SWEEP_SPIN 8     /* polls a workgroup of that launch spends on one wait before it gives up
                                        (0 = default, about a second); giving up is reported by zr_ctx_sync */

#define ZR_OPT_BF16_ACTIVATION_TERMS 9 /* products against bf16 weights (zr_lstm_pack_weights_bf16, zr_softmax_prepare_bf16,
                                        zr_attn_use_bf16_weights): 2 (default) = every fp32 activation enters as two
                                        bf16 terms (hi + lo: fp32-level accuracy, two matrix instructions per 16 k);
                                        1 = activations rounded to bf16 once (relative error 2^-9 per activation, half
                                        the matrix instructions and half the activation operand traffic) */
#define ZR_OPT_LSTM_STEP_WAIT_EXTRA 10 /* for tests of the give-up path of zr_lstm_decoder_step's single launch: the
                                        waits of a layer for the layer below expect this many arrivals more than there
                                        will be, so each of them runs to ZR_OPT_LSTM_SWEEP_SPIN polls and gives up
                                        whatever the timing (0 = off, the default) */
#define ZR_OPT_ATTN_SINGLE_LAUNCH 11 /* the attention step as ONE launch whose workgroups hand over through device
                                        memory (prepared fp32 matrices, H a multiple of 8 up to 1024, at most 64 window
                                        slots, all workgroups resident at once, own stream, only context on the
                                        device): 0 auto (taken whenever it applies; ZR_OPT_LSTM_SWEEP = 1 also
                                        switches it off), 1 never (three launches).  Its waits are bounded like the
                                        single-launch LSTM schedules' and reported the same way */

/* full_matrix_setup / cudaMalloc / cudaMemcpy / cudaMemset call sites (src/BZ_CUDA_UTIL.h:358-399 and the
 * layer constructors, e.g. src/LSTM.hpp:23-42). */
int zr_malloc(zr_ctx* ctx, size_t bytes, void** d_out);
int zr_free(zr_ctx* ctx, void* d_ptr);
int zr_h2d(zr_ctx* ctx, void* d_dst, const void* h_src, size_t bytes);
int zr_d2h(zr_ctx* ctx, void* h_dst, const void* d_src, size_t bytes); /* synchronous with the stream */
int zr_d2d(zr_ctx* ctx, void* d_dst, const void* d_src, size_t bytes);
int zr_memset_zero(zr_ctx* ctx, void* d_dst, size_t bytes);
/* d_dst[i] += d_src[i] (add_two_mats_kernel, src/custom_kernels.h:1818-1822; e.g. the feed-input error added to an
 * attention node's error, src/attention_node.hpp:416). */
int zr_add_inplace(zr_ctx* ctx, float* d_dst, const float* d_src, long long n);
/* d_x[i] clamped to [-threshold, threshold] (clip_mat_kernel, src/custom_kernels.h:2220-2231: with BZ_CUDA::clip_cell the
 * reference clamps the error a node sends to h_{t-1}, to the layer below and to the previous h~ to
 * +-BZ_CUDA::error_clip_threshold, src/LSTM.hpp:792,861 and src/LSTM_HH.hpp:665,756).  A NaN stays a NaN. */
int zr_clip_inplace(zr_ctx* ctx, float* d_x, long long n, float threshold);

/* ---- A1: index preparation ---------------------------------------------------------------------------- */

/* vocab_to_01 + vocab_to_nonM1 (src/custom_kernels.h:10-32) as launched by
 * Input_To_Hidden_Layer::prep_GPU_vocab_indices (src/Input_To_Hidden_Layer.hpp:1199-1202) and
 * Hidden_To_Hidden_Layer::prep_GPU_vocab_indices (src/Hidden_To_Hidden_Layer.hpp:763).
 * d_ids_nonneg or d_mask01 may be NULL.  vocab_size > 0 enables the [0,V) range check (flag read by zr_ctx_sync). */
int zr_vocab_prep(zr_ctx* ctx, const int* d_ids, int n, int vocab_size, int* d_ids_nonneg, int* d_mask01);
/* vocab_softmax (src/custom_kernels.h:38-50) from softmax_layer::prep_GPU_vocab_indices
 * (src/softmax.hpp:926-947): in place -1 -> 0 plus int and float masks. */
int zr_vocab_prep_softmax(zr_ctx* ctx, int* d_ids_inout, int n, int vocab_size, int* d_mask01, float* d_mask01_float);

/* ---- A2: embedding-column gather ---------------------------------------------------------------------- */

/* sparse_lookup_kernel (src/custom_kernels.h:342-348) from LSTM_IH_Node::forward_prop_GPU (src/LSTM.hpp:95):
 * d_x[:,b] = d_W[:, d_ids[b]], bit-exact.  Ids outside [0,V) are clamped and raise the data flag. */
int zr_embed_gather(zr_ctx* ctx, const float* d_W, int H, int V, const int* d_ids, int mb, float* d_x);

/* ---- A3-A5: LSTM node forward -------------------------------------------------------------------------- */

/* Packs one layer's parameters for zr_lstm_step.  Replaces the separate d_M_{i,f,c,o}, d_W_h{i,f,c,o},
 * d_Q_{i,f,c,o}, d_b_{i,f,c,o} members read by the 8/12 cublasSgemm calls of one node
 * (src/LSTM.hpp:140-339, src/LSTM_HH.hpp:148-271; members at src/Input_To_Hidden_Layer.h, src/Hidden_To_Hidden_Layer.h).
 * d_M/d_Wh/d_Q/d_b: arrays of 4 device pointers in gate order i,f,c,o; d_Q may be NULL (no feed-input). */
int zr_lstm_pack_weights(zr_ctx* ctx, const float* const d_M[4], const float* const d_Wh[4],
                         const float* const d_Q[4], const float* const d_b[4], int H, zr_lstm_weights** out);
/* Reduced-precision variant (no counterpart in the reference, whose only overloads are float and double,
 * src/BZ_CUDA_UTIL.h:691-703): the eight / twelve matrices are stored as bf16 (round to nearest even; exact when the
 * caller's values are already bf16-representable), biases stay fp32.  zr_lstm_step and zr_lstm_stack_forward take
 * the result like any other packed layer: products run on the bf16 matrix cores with each fp32 activation split into
 * two bf16 terms, accumulation and the cell state are fp32.  Against the fp32 path on the same (rounded) weights
 * the results agree within 1e-4 relative.  Requires H % 16 == 0 and 16-byte aligned activations. */
int zr_lstm_pack_weights_bf16(zr_ctx* ctx, const float* const d_M[4], const float* const d_Wh[4],
                              const float* const d_Q[4], const float* const d_b[4], int H, zr_lstm_weights** out);
int zr_lstm_weights_destroy(zr_ctx* ctx, zr_lstm_weights* w);

/* One node forward step: LSTM_IH_Node::forward_prop_GPU after the gather (src/LSTM.hpp:133-399) and
 * LSTM_HH_Node::forward_prop_GPU (src/LSTM_HH.hpp:103-333): the 8 (12 with feed-input) GEMMs, the four
 * activation kernels (custom_kernels.h:58-135), forward_c_t_kernel (:141), clip_mat_kernel (:2222),
 * forward_h_t_kernel (:162) and zero_c_t_and_h_t (:184) in one launch.
 *   d_in:    x (IH node) or h_t of the layer below (HH node), H x mb
 *   d_htild: NULL, or the previous attention output (feed-input; the reference skips it at index 0,
 *            src/LSTM.hpp:154) -- requires weights packed with Q
 *   clip_threshold <= 0 disables cell clipping (BZ_CUDA::clip_cell, src/BZ_CUDA_UTIL.h:107-108)
 *   d_gates: NULL or 4 device pointers (i, f, c~, o; each H x mb) for callers that keep them (the reference's
 *            node members d_i_t, d_f_t, d_c_prime_t_tanh, d_o_t)
 *   d_h / d_c may alias d_hprev / d_cprev only if d_in != d_hprev (every output element is written once, after
 *   all reads of the same element; other columns of h_prev are read by other workgroups, so in-place h is NOT
 *   allowed; in-place c is). */
int zr_lstm_step(zr_ctx* ctx, const zr_lstm_weights* w, const float* d_in, const float* d_hprev,
                 const float* d_cprev, const float* d_htild, const int* d_mask01, float clip_threshold, int mb,
                 float* d_h, float* d_c, float* const d_gates[4]);

/* The same node with the embedding lookup folded in: LSTM_IH_Node::forward_prop_GPU as a whole, sparse_lookup_kernel
 * included (src/LSTM.hpp:95 and :133-399).  Column b of the node's input is d_embed[:, d_ids_nonneg[b]] (d_embed is
 * H x V), read straight from the embedding by the product's own loads; no H x mb copy of the looked-up columns is
 * made.  Ids outside [0, V) are clamped and raise the data flag, as in zr_embed_gather. */
int zr_lstm_step_embed(zr_ctx* ctx, const zr_lstm_weights* w, const float* d_embed, int V, const int* d_ids_nonneg,
                       const float* d_hprev, const float* d_cprev, const float* d_htild, const int* d_mask01,
                       float clip_threshold, int mb, float* d_h, float* d_c, float* const d_gates[4]);

/* One decoder time step through all L layers: the LSTM part of neuralMT_model::forward_prop_target
 * (src/model.hpp:2573-2640) -- layer 0 is zr_lstm_step_embed on the current words (with d_htild, the previous step's
 * attention output, through Q when feed-input is on: src/LSTM.hpp:154-164), layer l > 0 is zr_lstm_step on this
 * step's h of layer l-1 (src/LSTM_HH.hpp:148-317).  The layers of one step form a chain, but the W_h and Q products
 * only read the previous step: when two workgroups per state tile fit on the device at once the whole step is ONE
 * launch, in which half of the workgroups stream those products for all layers while the other half walk up the
 * chain (same conditions, option and give-up reporting as the single-launch sweep: ZR_OPT_LSTM_SWEEP,
 * ZR_QUERY_LSTM_SWEEP_ABANDONED); otherwise one launch per layer.  Both give the same h and c to rounding.
 *   d_hprev / d_cprev / d_h / d_c: arrays of L device pointers (H x mb each).  No d_h[l] may alias another d_h, any
 *   d_hprev[m] or d_htild; d_c[l] may alias d_cprev[l]. */
int zr_lstm_decoder_step(zr_ctx* ctx, int L, const zr_lstm_weights* const layers[], const float* d_embed, int V,
                         const int* d_ids_nonneg, const float* const d_hprev[], const float* const d_cprev[],
                         const float* d_htild, const int* d_mask01, float clip_threshold, int mb,
                         float* const d_h[], float* const d_c[]);

/* The stand-alone fused gate kernel (the four activation kernels + c_t + clip + h_t + mask of the list above)
 * on pre-activations that are already in memory: d_preact is 4 planes (i,f,c,o) of H x mb holding
 * M x + W_h h (+ Q h~) without bias. */
int zr_lstm_gates(zr_ctx* ctx, const float* d_preact, const float* const d_b[4], const float* d_cprev,
                  const int* d_mask01, float clip_threshold, int H, int mb, float* d_h, float* d_c,
                  float* const d_gates[4]);

/* Whole stacked forward sweep (the time x layer loop of neuralMT_model::getError, src/model.hpp:1546-1621, and
 * forward_prop_source, :2367-2452): layer 0 gathers its input from d_embed by token id, layer l>0 reads layer
 * l-1's h_t.  Nodes that do not depend on each other run side by side: either the whole sweep is ONE launch whose
 * workgroups keep their tile of one layer for all T steps and hand h_t to each other through device memory (taken
 * when they fill most of the GPU and are all resident at once; see ZR_OPT_LSTM_SWEEP), or one launch per diagonal
 * l + t = d.  The single launch keeps its hand-over buffer and arrival counters in the context's scratch memory.
 *   d_ids_nonneg, d_mask01: time-major [b + t*mb] (src/fileHelper.h:488), outputs of zr_vocab_prep
 *   d_h0/d_c0: arrays of L device pointers (initial state per layer, H x mb) -- zeros for encoder / LM
 *   d_h_all/d_c_all: arrays of L device pointers, each T*H*mb floats: node t's h_t at offset t*H*mb */
int zr_lstm_stack_forward(zr_ctx* ctx, int L, const zr_lstm_weights* const layers[], const float* d_embed, int V,
                          const int* d_ids_nonneg, const int* d_mask01, int T, int mb,
                          const float* const d_h0[], const float* const d_c0[], float clip_threshold,
                          float* const d_h_all[], float* const d_c_all[]);

/* ---- dense contraction --------------------------------------------------------------------------------- */

/* cublas_gemm_wrapper / cublasSgemm (src/BZ_CUDA_UTIL.h:691-696) with alpha = 1, beta = 0:
 * C(M x N) = op(A) * B, trans_a = 0: A is M x K (lda >= M); trans_a = 1: A is K x M (lda >= K).  B is K x N. */
int zr_gemm(zr_ctx* ctx, int trans_a, int M, int N, int K, const float* d_A, int lda, const float* d_B, int ldb,
            float* d_C, int ldc);

/* ---- A8/A9: output softmax ------------------------------------------------------------------------------ */

/* Optional preparation of an output layer for repeated use (no counterpart in the reference, which hands the raw
 * V x H matrix d_D of softmax_layer, src/softmax.h:60, to cublasSgemm on every call): copies D into the layout the
 * matrix cores read fastest (four consecutive k per row side by side, 32-row tiles 128-byte aligned; V*H*4 more
 * bytes of device memory).  Afterwards every softmax entry point below that is given the same d_D, V and H uses the
 * copy.  The copy is a snapshot: call again after changing D (it re-packs in place), and call zr_softmax_release
 * before freeing d_D.  At most 8 matrices per context.  Results are the same with or without it. */
int zr_softmax_prepare(zr_ctx* ctx, const float* d_D, int V, int H);
/* Same, with the copy stored as bf16 (round to nearest even; half the bytes to stream): the reduced-precision
 * variant of the output layer, see zr_lstm_pack_weights_bf16 for the arithmetic.  Requires H % 16 == 0. */
int zr_softmax_prepare_bf16(zr_ctx* ctx, const float* d_D, int V, int H);
int zr_softmax_release(zr_ctx* ctx, const float* d_D);

#define ZR_SOFTMAX_PROB 0    /* probabilities: softmax_layer::get_distribution_GPU (src/softmax.hpp:514-632) */
#define ZR_SOFTMAX_LOGPROB 1 /* natural-log probabilities, fp32 */
/* The logits D h + b_d and, behind them, the column statistics of the reference's overflow-safe soft-max
 * (src/custom_kernels.h:503-577): d_out holds V*mb + 2*mb floats, the V x mb logits followed by (max, sum of
 * exp(x - max)) per column.  No normalised matrix is written: zr_beam_expand_logits / zr_beam_finish_logits form
 * exp(x - max) / sum for the few entries a decode step needs, so the V x mb matrix is written once and read once per
 * step instead of written twice and read twice.  d_logits_scratch must be NULL in this mode. */
#define ZR_SOFTMAX_LOGITS 2
/* As ZR_SOFTMAX_LOGITS, but instead of two statistics per column d_out receives what the product's epilogue already
 * has: one (max, sum of exp(x - max)) pair per block of 32 vocabulary rows and column, [mb][zr_softmax_block_count(V)][2]
 * floats starting zr_softmax_blocks_offset(V, mb) floats into d_out (d_out holds that offset + 2 * blocks * mb floats).
 * Nothing folds them: zr_beam_expand_blocks / zr_beam_finish_blocks do, and use the block maxima to find the few blocks
 * of a column that can hold one of its beam + 1 largest entries, so a decode step reads the V x mb logits it has just
 * written only there.  No counterpart in the reference (its decoder copies the whole normalised matrix to the host,
 * src/decoder_model_wrapper.hpp:418).  d_logits_scratch must be NULL in this mode. */
#define ZR_SOFTMAX_LOGITS_BLOCKS 3
int zr_softmax_block_count(int V);
long long zr_softmax_blocks_offset(int V, int cols);

/* D h + b_d on MFMA (cublasSgemm + matrix_bias_kernel, src/softmax.hpp:539-547) followed by the per-column
 * max / exp / sum / normalise of outputdist_overflow_prevention_kernel (src/custom_kernels.h:503-577).
 * d_out: V x mb (more in the two logits modes, see above).  d_logits_scratch: V x mb scratch for the logits, or
 * NULL to use d_out in place. */
int zr_softmax_forward(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb,
                       int mode, float* d_out, float* d_logits_scratch);
/* zr_softmax_forward for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments, same kernels and
 * bit-identical results, but the product's scratch memory (the activations re-laid-out for the matrix cores and the
 * per-32-row partial column statistics) lives in a 32 MiB array that is part of the library's device image on every
 * GPU it runs on, so the call itself allocates and frees nothing.  Limits (ZR_EINVAL beyond them, message in
 * zr_last_error): H*mb*4 <= 8 MiB and ceil(V/32)*mb*8 + 16*mb + 64 <= 24 MiB -- e.g. V = 80000 with 256 columns
 * of H = 2000 fits, 6400 columns of V = 50000 do not.  Every call on one GPU shares that GPU's array: calls that overlap
 * on one GPU (two contexts, two streams) race; calls on one context are ordered by its stream and safe.  Like every
 * entry point, it must not be called on one context from two host threads at once (a context is single-threaded: for
 * the duration of this call its scratch requests are redirected to the static array). */
int zr_softmax_forward_static(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h,
                              int mb, int mode, float* d_out, float* d_logits_scratch);
/* softmax_layer::get_perplexity_GPU (src/softmax.hpp:636-692) with outputdist_perplexity_kernel
 * (src/custom_kernels.h:583-660): double log-probabilities, V x mb. */
int zr_softmax_logprob_f64(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb,
                           double* d_logp, float* d_logits_scratch);
/* softmax_layer::compute_loss_GPU (src/softmax.hpp:867-900): sum over unmasked columns of
 * log p[target[b], b] (double), without materialising the V x mb log-probabilities.  Synchronous: *h_loss is
 * valid on return.  d_logits_scratch: V x mb floats. */
int zr_softmax_loss(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int mb,
                    const int* d_target, const int* d_mask01, float* d_logits_scratch, double* h_loss);

/* ---- A10: attention -------------------------------------------------------------------------------------- */

/* attention_layer constructor (src/attention_layer.hpp:3-173): keeps the six parameter pointers (borrowed, not
 * copied: d_W_a, d_W_p H x H; d_v_p H (stored 1 x H); d_out_bias H; d_W_c_p1, d_W_c_p2 H x H), uploads the
 * source-state pointer table (d_total_hs_mat, :106-160) and allocates the node temporaries.
 *   h_hs_table: host array of longest_sent device pointers; entry t = top-layer source h at source node t,
 *               H x mb.  The tables are read at zr_attn_step time and must stay valid. */
typedef struct zr_attn zr_attn;
int zr_attn_create(zr_ctx* ctx, int H, int mb, int D, const float* d_W_a, const float* d_W_p, const float* d_v_p,
                   const float* d_out_bias, const float* d_W_c1, const float* d_W_c2,
                   const float* const* h_hs_table, int longest_sent, zr_attn** out);
/* Reduced-precision variant (no counterpart in the reference): snapshots W_a, W_p, W_c_p1 and W_c_p2 as bf16 in the
 * matrix cores' layout; later zr_attn_step calls multiply with the snapshots (bf16 matrix cores, fp32 activations
 * split in two bf16 terms, fp32 accumulation).  v_p, the bias and everything element-wise stay fp32.  Call again
 * after changing the matrices.  Requires H % 16 == 0. */
int zr_attn_use_bf16_weights(zr_ctx* ctx, zr_attn* a);
/* Optional preparation for repeated use (no counterpart in the reference, which hands d_W_p, d_W_a, d_W_c_p1 and
 * d_W_c_p2 to cublasSgemm as they are, src/attention_node.hpp:132,195,354,360): snapshots the four matrices in the
 * layout the matrix cores read fastest (W_a transposed; 4*H*H*4 more bytes).  Later zr_attn_step calls then run as
 * one launch whose workgroups hand the projections and the contexts over through device memory (fp32, H % 8 == 0,
 * 32 <= H <= 1024, at most 64 window slots, the context's own stream: ZR_OPT_ATTN_SINGLE_LAUNCH), otherwise as three --
 * both projections of h_t as one batch, one kernel for p_t, window, scores, alignment weights and context that reads
 * each valid source state from memory once, and the output product -- instead of eight.  Results agree with the
 * unprepared path to rounding (different summation order).  Call again after changing the matrices. */
int zr_attn_prepare(zr_ctx* ctx, zr_attn* a);
int zr_attn_destroy(zr_ctx* ctx, zr_attn* a);
/* attention_node::forward_prop (src/attention_node.hpp:73-394), single-source branch: p_t, window, scores
 * h_s . (W_a^T h), the reference's softmax (max initialised to 0) times the Gaussian prior, context and
 * h~ = tanh(W_c1 c + W_c2 h + b) * mask.
 *   d_batch_info: [0,mb) source lengths, [mb,2mb) left-pad offsets (src/fileHelper.h:499-500; uploaded by
 *                 attention_layer::prep_minibatch_info, src/attention_layer.hpp:580-583)
 *   outputs: d_htild H x mb (the node's d_final_temp_2); optional (NULL = internal): d_alignments and
 *   d_indices ((2D+1) x mb, element [b + mb*j]), d_p_t (mb), d_c_ctx (H x mb). */
int zr_attn_step(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const float* d_h_t, const int* d_mask01,
                 float* d_htild, float* d_alignments, int* d_indices, float* d_p_t, float* d_c_ctx);

/* get_viterbi_alignment_kernel (src/custom_kernels.h:1623-1635, launched by attention_node::forward_prop when
 * BZ_CUDA::unk_replacement is set, src/attention_node.hpp:225-234): d_viterbi[b] = source position of the window slot
 * with the largest alignment weight of column b (first of equal maxima; -1 for a masked column), from the alignments
 * and window indices of the last zr_attn_step.  d_alignments / d_indices: what was passed to zr_attn_step, or NULL for
 * the object's internal arrays. */
int zr_attn_viterbi(zr_ctx* ctx, const zr_attn* a, const float* d_alignments, const int* d_indices, int* d_viterbi);

/* The alignment vote of an ensemble under unk replacement (ensemble_factory::ensembles_models,
 * src/ensemble_factory.hpp:797-834, on the per-model rows filled at src/attention_node.hpp:236-268): every model's
 * window weights (d_alignments[k], d_indices[k]: slots x cols as zr_attn_step leaves them, element (b, j) at b + cols*j;
 * index -1 = no source position) are spread over longest_sent (<= 8192) source positions, summed over the n_models
 * (<= 16) models in order, and d_viterbi[b] = the first position with the largest sum, -1 when no sum is positive. */
int zr_attn_viterbi_ensemble(zr_ctx* ctx, int n_models, const float* const d_alignments[], const int* const d_indices[],
                             int slots, int cols, int longest_sent, int* d_viterbi);

/* ---- A12: decoder state shuffles ------------------------------------------------------------------------- */

/* swap_states_decoding (src/Input_To_Hidden_Layer.hpp:1231-1242, src/Hidden_To_Hidden_Layer.hpp:780-791):
 * d_dst[:,i] = d_src[:, d_perm[i]] for i < n; d_dst must not alias d_src. */
int zr_gather_columns(zr_ctx* ctx, const float* d_src, int H, const int* d_perm, int n, float* d_dst);
/* The same reorder for n_arrays (<= 32) matrices of H rows in one launch: neuralMT_model::swap_decoding_states
 * (src/model.hpp:2704-2726) calls swap_states_decoding once per layer for h and c and reorders h~; each of those is
 * a sub-microsecond copy, so they share a kernel.  d_perm[i] must lie in [0, n_src_cols) (checked on the device,
 * reported by zr_ctx_sync). */
int zr_gather_columns_multi(zr_ctx* ctx, int n_arrays, const float* const d_src[], int H, const int* d_perm,
                            int n_src_cols, int n, float* const d_dst[]);
/* transfer_decoding_states_GPU (src/Input_To_Hidden_Layer.hpp:1252-1266): one column to n columns. */
int zr_broadcast_column(zr_ctx* ctx, const float* d_src_col, int H, int n, float* d_dst);

/* ---- A13: beam search ------------------------------------------------------------------------------------ */

/* decoder<dType> (src/decoder.h:162-1502), non-FSA path, for n_sent independent sentences decoded together
 * (the reference decodes one sentence per pass; columns [s*beam, (s+1)*beam) belong to sentence s).
 * start symbol 0, end symbol 1 (src/decoder.h:1325-1330). */
int zr_beam_create(zr_ctx* ctx, int beam, int vocab, int n_sent, int max_len, float penalty, zr_beam** out);
int zr_beam_destroy(zr_ctx* ctx, zr_beam* b);
/* init_decoder (src/decoder.h:1317-1355) */
int zr_beam_init(zr_ctx* ctx, zr_beam* b);
/* expand_hypothesis_without_fsa (src/decoder.h:1158-1315) on device: d_prob is V x (n_sent*beam)
 * probabilities.  Afterwards d_words (next input ids, -1 = dead slot) and d_backptr (new_indicies_changes)
 * are valid, n_sent*beam ints each. */
int zr_beam_expand(zr_ctx* ctx, zr_beam* b, const float* d_prob, int index, int* d_words, int* d_backptr);
/* finish_current_hypotheses (src/decoder.h:672-688). */
int zr_beam_finish(zr_ctx* ctx, zr_beam* b, const float* d_prob);
/* zr_beam_expand / zr_beam_finish on the output of ZR_SOFTMAX_LOGITS: d_logits V x (n_sent*beam), d_colstats 2 floats
 * per column (max, sum of exp(x - max)) -- d_out and d_out + V*cols of that call.  The per-column selection runs on the
 * logits (the soft-max is monotonic within a column) and only the beam+1 selected entries of a column are normalised,
 * with the same expression as the full matrix, and the candidates are ranked by those probabilities (words whose
 * probabilities round to one float follow the tie rule, whatever their logits), so candidates, scores, words and
 * back-pointers are those of zr_beam_expand on the probabilities. */
int zr_beam_expand_logits(zr_ctx* ctx, zr_beam* b, const float* d_logits, const float* d_colstats, int index,
                          int* d_words, int* d_backptr);
int zr_beam_finish_logits(zr_ctx* ctx, zr_beam* b, const float* d_logits, const float* d_colstats);
/* The same on the output of ZR_SOFTMAX_LOGITS_BLOCKS: d_logits V x (n_sent*beam), d_blocks the per-block pairs behind
 * them (d_out and d_out + zr_softmax_blocks_offset(V, cols) of that call).  One launch per step folds a column's pairs
 * into its statistics (in the order zr_softmax_forward does: the same bits), bounds the beam + 1 largest entries from
 * below by the block maxima, reads only the blocks that reach the bound and ranks what it finds there; results are
 * those of zr_beam_expand_logits bit for bit. */
int zr_beam_expand_blocks(zr_ctx* ctx, zr_beam* b, const float* d_logits, const float* d_blocks, int index,
                          int* d_words, int* d_backptr);
int zr_beam_finish_blocks(zr_ctx* ctx, zr_beam* b, const float* d_logits, const float* d_blocks);
/* Copies the finished hypotheses of sentence s to the host: returns their number (or a negative error);
 * h_words is n x max_len (row-major, -1 padded), h_len and h_score have n entries; at most cap are copied. */
int zr_beam_hypotheses(zr_ctx* ctx, zr_beam* b, int sentence, int cap, int* h_words, int* h_len, float* h_score);
/* ensemble_factory::ensembles_models (src/ensemble_factory.hpp:767-793): d_out = the element-wise mean of n_models
 * (<= 16) output distributions (V x cols each, summed in double), every column then divided by its sum.  d_out may be
 * one of the inputs.  The result feeds zr_beam_expand / zr_beam_finish.  The reference accumulates the column sums in
 * float, row after row, and takes a single model's distribution as it is (no renormalisation); here the sums are in
 * double for any number of models, which moves a column's log-probabilities by a common ~1e-5 at most. */
int zr_ensemble_average(zr_ctx* ctx, int n_models, const float* const d_probs[], int V, int cols, float* d_out);
/* Viterbi alignments through the beam, for unk replacement (decoder::top_sentences_viterbi and
 * eigen_mat_wrapper::viterbi_alignments, src/decoder.h:126,230-231; initialised to -20, :1335).  With enable != 0 every
 * later zr_beam_expand* / zr_beam_finish* call attaches to each candidate the alignment of the column it comes from,
 * read from d_viterbi (n_sent*beam ints in device memory, e.g. zr_attn_viterbi's output, read when that call runs;
 * NULL: -1 for every column, as the reference does when it is handed none, :1174-1179), a surviving hypothesis keeps
 * its parent's alignments plus its own at position current_index+1 (:1281-1282), and a finished one likewise
 * (:1266-1267, :683-684).  Switch it on before the first step of a sentence (the call then also runs zr_beam_init).
 * zr_beam_hypotheses_viterbi copies the alignments of the finished hypotheses of sentence s, n x max_len like
 * zr_beam_hypotheses' h_words and in the same order; returns their number. */
int zr_beam_set_viterbi(zr_ctx* ctx, zr_beam* b, int enable, const int* d_viterbi);
/* The words a step selects are the next step's input ids, after the -1 of a dead slot has become 0 (vocab_to_nonM1,
 * src/custom_kernels.h:23-34, which the reference runs on the decoder's current_indices in
 * Input_To_Hidden_Layer::prep_GPU_vocab_indices).  With d_words_nonneg set (n_sent*beam ints in device memory; NULL
 * switches it off) every later zr_beam_expand* call writes them there as well, in the launch that writes d_words, so
 * the caller needs no zr_vocab_prep launch between the steps. */
int zr_beam_set_input_ids(zr_ctx* ctx, zr_beam* b, int* d_words_nonneg);
int zr_beam_hypotheses_viterbi(zr_ctx* ctx, zr_beam* b, int sentence, int cap, int* h_viterbi);
/* Current beam state of sentence s (top_sentences_scores, current_indices). */
int zr_beam_state(zr_ctx* ctx, zr_beam* b, int sentence, float* h_scores, int* h_words);

/* ---- F4: training backward (stacked LSTM and output layer; no attention, no dropout) ------------------------ */

/* zr_lstm_stack_forward that also keeps every node's gate activations for the backward pass (the reference's nodes
 * keep d_i_t, d_f_t, d_c_prime_t_tanh, d_o_t; src/LSTM.h:30-60).  d_gates_all: L pointers, each T*4*H*mb floats;
 * gate g (order i, f, c~, o) of node t at offset (t*4 + g)*H*mb.  An entry may be NULL (that layer's gates are not
 * kept). */
int zr_lstm_stack_forward_train(zr_ctx* ctx, int L, const zr_lstm_weights* const layers[], const float* d_embed, int V,
                                const int* d_ids_nonneg, const int* d_mask01, int T, int mb,
                                const float* const d_h0[], const float* const d_c0[], float clip_threshold,
                                float* const d_h_all[], float* const d_c_all[], float* const d_gates_all[]);

/* Backward-side copy of one layer's matrices: M_g and W_hg stacked over the four gates and transposed (H x 4H,
 * element (k, g*H + j) = W_g[j][k]), the operands of the error products d_ERRnTOt_htM1 = sum_g W_hg^T err_g and d_ERRnTOt_h_Below =
 * sum_g M_g^T err_g (src/LSTM_HH.hpp:470-560).  Call zr_lstm_train_refresh after the weights change. */
typedef struct zr_lstm_train zr_lstm_train;
int zr_lstm_train_create(zr_ctx* ctx, const float* const d_M[4], const float* const d_Wh[4], int H, zr_lstm_train** out);
int zr_lstm_train_refresh(zr_ctx* ctx, zr_lstm_train* w, const float* const d_M[4], const float* const d_Wh[4]);
int zr_lstm_train_destroy(zr_ctx* ctx, zr_lstm_train* w);
/* 4H x H stacked matrix -> four H x H matrices (gate order i, f, c, o), e.g. the reference's d_M_i_grad ... */
int zr_unstack_gates(zr_ctx* ctx, const float* d_stack, int H, float* const d_out[4]);

/* Back-propagation through time over the whole (layer, time) grid: LSTM_IH_Node / LSTM_HH_Node::back_prop_GPU
 * (src/LSTM.hpp:542-900, src/LSTM_HH.hpp:336-640) in the order of neuralMT_model::compute_gradients
 * (src/model.hpp:1823-2000), errors only (weight gradients: zr_lstm_weight_gradients).
 *   d_c0, d_c_all, d_gates_all: as given to / written by zr_lstm_stack_forward_train.
 *   d_err_top: T*H*mb, the loss layer's error at the top layer's h_t (d_ERRt_ht).
 *   d_err_hT / d_err_cT: L pointers (or NULL, or NULL entries): errors arriving at the last step from beyond.
 *   Outputs: d_dgates_all[l]: 4H x (T*mb) column-major, the errors at the four pre-activations of every node
 *   (element (g*H + j, t*mb + b)); d_err_below0: T*H*mb, the error at layer 0's input (NULL: not wanted);
 *   d_err_h0 / d_err_c0: L pointers, errors at the initial states. */
int zr_lstm_stack_backward(zr_ctx* ctx, int L, const zr_lstm_train* const layers[], int T, int mb,
                           const int* d_mask01, const float* const d_c0[], const float* const d_c_all[],
                           const float* const d_gates_all[], const float* d_err_top, const float* const d_err_hT[],
                           const float* const d_err_cT[], float* const d_dgates_all[], float* d_err_below0,
                           float* const d_err_h0[], float* const d_err_c0[]);
/* The same with the error clamps of BZ_CUDA::clip_cell (src/LSTM.hpp:792-794, src/LSTM_HH.hpp:665-667,755-757): the error
 * a node sends to h_{t-1}, and the error a layer above the first sends to the layer below, are clamped to +-err_clip,
 * each on its own, before they are added to anything; d_err_h0 is clamped likewise (and d_err_hT on arrival: it is
 * the same kind of error, from a node beyond the last step), d_err_below0 (the embedding's error) is not.
 * err_clip <= 0: no clamp (zr_lstm_stack_backward). */
int zr_lstm_stack_backward_clamped(zr_ctx* ctx, int L, const zr_lstm_train* const layers[], int T, int mb,
                           const int* d_mask01, const float* const d_c0[], const float* const d_c_all[],
                           const float* const d_gates_all[], const float* d_err_top, const float* const d_err_hT[],
                           const float* const d_err_cT[], float* const d_dgates_all[], float* d_err_below0,
                           float* const d_err_h0[], float* const d_err_c0[], float err_clip);

/* One layer's weight gradients from the kept errors: compute_gradients_GPU (src/LSTM.hpp:1000-1270) summed over
 * all nodes in one product each.  d_in_all: the layer's inputs, H x (T*mb) (the layer below's h, or the gathered
 * embedding columns); d_h0, d_h_all: the layer's own initial state and outputs.
 * d_dM_stack, d_dWh_stack: 4H x H stacked gradients (zr_unstack_gates splits them); d_db: 4H. */
int zr_lstm_weight_gradients(zr_ctx* ctx, int H, int T, int mb, const float* d_dgates, const float* d_in_all,
                             const float* d_h0, const float* d_h_all, float* d_dM_stack, float* d_dWh_stack,
                             float* d_db);

/* One node of the same computation, for callers that drive the (layer, time) grid themselves as the reference's
 * layer classes do: the error part of LSTM_IH_Node::back_prop_GPU / LSTM_HH_Node::back_prop_GPU
 * (src/LSTM.hpp:542-960, src/LSTM_HH.hpp:452-700).
 *   d_gates: the node's saved i, f, c~, o (H x mb each); d_c, d_c_prev: c_t, c_{t-1}.
 *   d_err_above: error at h_t from the layer above or the loss layer (d_d_ERRt_ht; NULL = none);
 *   d_err_h_next / d_err_c_next: errors arriving from step t+1 (d_d_ERRnTOtp1_ht / _ct; NULL = none).
 *   Outputs: d_dgates 4H x mb (rows g*H + j; the reference's d_d_ERRnTOt_it, _ft, _tanhcpt, _ot stacked),
 *   d_err_h_prev, d_err_c_prev (d_d_ERRnTOt_htM1 / _ctM1; d_err_c_prev may alias d_err_c_next),
 *   d_err_below (d_d_ERRnTOt_h_Below; NULL = not wanted; fastest when it is d_err_h_prev + H*mb). */
int zr_lstm_node_backward(zr_ctx* ctx, const zr_lstm_train* layer, int mb, const float* const d_gates[4],
                          const float* d_c, const float* d_c_prev, const int* d_mask01, const float* d_err_above,
                          const float* d_err_h_next, const float* d_err_c_next, float* d_dgates, float* d_err_h_prev,
                          float* d_err_c_prev, float* d_err_below);
/* compute_gradients_GPU of one node (src/LSTM.hpp:963-1270, src/LSTM_HH.hpp:700-900): the rank-mb updates
 * dM += dgates in^T, dWh += dgates h_{t-1}^T, db += row sums, ACCUMULATED into the stacked 4H x H / 4H gradients
 * (zero them at the start of a minibatch).  d_in: the node's input (embedding columns or the h_t below), H x mb. */
int zr_lstm_node_gradients(zr_ctx* ctx, int H, int mb, const float* d_dgates, const float* d_in, const float* d_h_prev,
                           float* d_dM_stack, float* d_dWh_stack, float* d_db);

/* The feed-input part of a bottom-layer node's backward (LSTM_IH_Node::back_prop_GPU under `feed_input && index != 0`,
 * src/LSTM.hpp:804-866, and the Q gradient products of compute_gradients_GPU, :1014-1050):
 *   d_err_htild (d_ERRnTOt_h_tild, H x mb, overwritten) = sum_g Q_g^T dgates_g -- the error the previous step's
 *     attention node adds to its own (src/attention_node.hpp:416);
 *   d_dQ_stack (4H x H, stacked over the gates like zr_lstm_node_gradients' outputs, ACCUMULATED) += dgates h~^T.
 *   d_dgates: the node's stacked pre-activation errors (output of zr_lstm_node_backward); d_htild: the node's d_h_tild. */
int zr_lstm_feed_backward(zr_ctx* ctx, const float* const d_Q[4], int H, int mb, const float* d_dgates,
                          const float* d_htild, float* d_err_htild, float* d_dQ_stack);

/* attention_node::back_prop (src/attention_node.hpp:398-669, single-source branch) with its kernels (zero_h_t,
 * tanh_grad_kernel, error_alignments_kernel_large, error_hs_ct_kernel_large, error_pt_kernel, att_vp_error,
 * grad_W_p_kernel, get_ht_scalings_Wa_grad_kernel, scale_ht_kernel, copy_errors_source: src/custom_kernels.h:1835,
 * 1968-2196, 2212).  What the reference caches in the forward pass (tanh_1, sigma_1, W_a^T h, the Gaussian factors)
 * is computed again from d_h_t, d_p_t and d_indices.
 *   d_h_t: the h_t the forward step read (d_h_t_att: after the layer's dropout where that is on);
 *   d_h_tild, d_alignments, d_indices, d_p_t, d_c_t: outputs of that zr_attn_step call;
 *   d_err_htild: error of h~ (d_d_ERRt_ht_tild; the caller has added the feed-input error, :416);
 *   d_err_h_t (H x mb, overwritten): error of h_t (d_ERRnTOt_ht_p1, before the dropout of :647); may be d_err_htild;
 *   grads: the layer's six gradient arrays, ACCUMULATED into (beta = 1 in the reference);
 *   the errors of the source states are ADDED into the arrays registered with zr_attn_set_error_tables, entry t for
 *   the source position stored in hs table t (d_total_hs_error, src/attention_layer.hpp:106-160). */
typedef struct zr_attn_grads {
  float *d_W_a, *d_W_p, *d_v_p, *d_out_bias, *d_W_c1, *d_W_c2;
} zr_attn_grads;
int zr_attn_set_error_tables(zr_ctx* ctx, zr_attn* a, float* const* h_err_tables, int n);
int zr_attn_backward(zr_ctx* ctx, zr_attn* a, const int* d_batch_info, const float* d_h_t, const int* d_mask01,
                     const float* d_h_tild, const float* d_alignments, const int* d_indices, const float* d_p_t,
                     const float* d_c_t, const float* d_err_htild, float* d_err_h_t, const zr_attn_grads* grads);

/* One decoder time step from the current words to the output distribution: neuralMT_model::forward_prop_target
 * (src/model.hpp:2573-2688) as one call -- zr_lstm_decoder_step, then zr_attn_step on the top layer's h_t (attn may be
 * NULL: no attention), then zr_softmax_forward on h~ (or on the top h_t).  Same kernels and the same results as the three
 * calls; what the call adds is that the activations handed from one stage to the next stay in the matrix cores'
 * k-interleaved layout (the LSTM launch writes the top layer's h that way for the attention products, the attention
 * output product writes h~ that way for the output layer), so the two re-layout launches between the stages go away.
 *   V_in: rows of d_embed's vocabulary; V_out, d_D, d_b_d, mode, d_out: as in zr_softmax_forward;
 *   d_alignments, d_indices, d_p_t, d_c_ctx: as in zr_attn_step (NULL: not wanted). */
int zr_decoder_step(zr_ctx* ctx, int L, const zr_lstm_weights* const layers[], const float* d_embed, int V_in,
                    const int* d_ids_nonneg, const float* const d_hprev[], const float* const d_cprev[],
                    const float* d_htild_prev, const int* d_mask01, float clip_threshold, int mb, float* const d_h[],
                    float* const d_c[], zr_attn* attn, const int* d_batch_info, float* d_htild, float* d_alignments,
                    int* d_indices, float* d_p_t, float* d_c_ctx, const float* d_D, const float* d_b_d, int V_out,
                    int mode, float* d_out);

/* dropout_kernel (src/custom_kernels.h:1556-1560; forward call sites src/LSTM.hpp:118, src/LSTM_HH.hpp:124,
 * src/attention_node.hpp:105, src/softmax.hpp:477, backward :647, src/LSTM_HH.hpp:674, src/softmax.hpp:746):
 * x = (uniform < keep_rate) * (1 / keep_rate) * x, in place; keep_rate is the probability of KEEPING a value. */
int zr_dropout_apply(zr_ctx* ctx, const float* d_uniform, float keep_rate, float* d_x, long long n);
/* Fills d_out with n uniform numbers in (0, 1], a pure function of (seed, call, index): the stand-in for
 * curandGenerateUniform (src/BZ_CUDA_UTIL.h:793-795), whose stream cannot be reproduced. */
int zr_uniform_fill(zr_ctx* ctx, unsigned long long seed, unsigned long long call, float* d_out, long long n);

/* Embedding gradient (the sparse W gradient kernels, src/custom_kernels.h:1297-1390): d_dW[:, id[k]] += d_err[:, k]
 * for the n unmasked positions; d_dW is H x V and is accumulated into (zero it first).  Uses float atomics, like
 * the reference: the summation order within a column is not fixed. */
int zr_embed_gradient(zr_ctx* ctx, int H, int V, const float* d_err, const int* d_ids_nonneg, const int* d_mask01,
                      int n, float* d_dW);

/* Loss-layer backward for n columns at once (all time steps of a minibatch, n = T*mb <= 65535):
 * get_h_t_gradient_GPU, compute_D_gradient_GPU, compute_b_d_gradient_GPU (src/softmax.hpp:700-860).
 *   d_h: H x n; d_target (-1 already mapped to 0) and d_mask01: n ints (zr_vocab_prep_softmax).
 *   d_prob_scratch: V x n.  Outputs: d_err_h H x n (= D^T (onehot - p), 0 on masked columns), d_dD V x H,
 *   d_db V (overwritten, not accumulated: pass every column of the minibatch in one call). */
int zr_softmax_backward(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int n,
                        const int* d_target, const int* d_mask01, float* d_prob_scratch, float* d_err_h, float* d_dD,
                        float* d_db);
/* The same plus the minibatch's log-likelihood, sum over unmasked columns of log((double) p[target]) as the
 * reference's train_perplexity_kernel forms it from the float probabilities (src/custom_kernels.h:478-488,
 * src/softmax.hpp:616-619): no second logits product for the loss.  Waits for the stream (h_loss is host memory). */
int zr_softmax_backward_loss(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h, int n,
                             const int* d_target, const int* d_mask01, float* d_prob_scratch, float* d_err_h,
                             float* d_dD, float* d_db, double* h_loss);
/* The same with d_dD and d_db ADDED to: one call per time step (softmax_layer::back_prop1 / back_prop2,
 * src/softmax.hpp:600-700), gradients zeroed at the start of the minibatch. */
int zr_softmax_backward_accumulate(zr_ctx* ctx, const float* d_D, const float* d_b_d, int V, int H, const float* d_h,
                                   int n, const int* d_target, const int* d_mask01, float* d_prob_scratch,
                                   float* d_err_h, float* d_dD, float* d_db);

/* update_weights (src/softmax.hpp:232-300, src/Hidden_To_Hidden_Layer.hpp update_weights_GPU): the gradient is
 * scaled (the reference divides by the minibatch size), clipped to norm_clip in L2 norm if norm_clip > 0
 * (norm_clip_GPU_v2), and ADDED: W += learning_rate * clip(scale * grad). */
int zr_sgd_update(zr_ctx* ctx, float* d_W, const float* d_grad, long long n, float scale, float norm_clip,
                  float learning_rate);

/* The reference's three ways of clipping a gradient before the update (src/main.cu:495-511): per matrix
 * (--matrix-clip-gradients, norm_clip_GPU_v2, src/custom_kernels.h:1064-1078), over the whole model
 * (--whole-clip-gradients, norm_clip_GPU_v2_p1 / _p2, :1083-1135) and per element (--ind-clip-gradients,
 * clip_mat_kernel, :2220-2231). */
#define ZR_CLIP_NONE 0
#define ZR_CLIP_MATRIX_NORM 1
#define ZR_CLIP_WHOLE_NORM 2
#define ZR_CLIP_ELEMENT 3
/* calculate_global_norm (src/Hidden_To_Hidden_Layer.hpp:241-335, src/model.hpp:1850-1892): adds the squared L2 norm of
 * scale * grad to the double at d_sumsq (device memory; reset != 0 overwrites it instead, n == 0 with reset clears
 * it).  The sum stays on the device: no copy to the host, no wait. */
int zr_grad_sumsq_accumulate(zr_ctx* ctx, const float* d_grad, long long n, float scale, double* d_sumsq, int reset);
/* W += learning_rate * clip(scale * grad) with clip chosen by clip_mode: ZR_CLIP_NONE; ZR_CLIP_MATRIX_NORM (what
 * zr_sgd_update does with norm_clip = threshold); ZR_CLIP_WHOLE_NORM: shrunk by threshold / sqrt(*d_sumsq) when the
 * norm accumulated over every gradient of the model exceeds threshold (update_global_params,
 * src/Hidden_To_Hidden_Layer.hpp:353-382); ZR_CLIP_ELEMENT: every element of scale * grad clamped to +-threshold
 * (src/Hidden_To_Hidden_Layer.hpp:503-517).  d_sumsq is read in ZR_CLIP_WHOLE_NORM only. */
int zr_sgd_update_clipped(zr_ctx* ctx, float* d_W, const float* d_grad, long long n, float scale, int clip_mode,
                          float threshold, const double* d_sumsq, float learning_rate);

#ifdef __cplusplus
}
#endif
#endif /* ZOPH_RNN_H */
