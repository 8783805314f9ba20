// Host-side C++ classes that keep the names, public data members and forward-path member functions of the
// reference's layer objects and forward every device operation to the C-ABI in include/zoph_rnn.h.
//
//   reference class (file)                                   here
//   LSTM_IH_Node            (src/LSTM.h:19-106)              LSTM_IH_Node<float>
//   LSTM_HH_Node            (src/LSTM_HH.h:19-102)           LSTM_HH_Node<float>
//   Input_To_Hidden_Layer   (src/Input_To_Hidden_Layer.h:11) Input_To_Hidden_Layer<float>
//   Hidden_To_Hidden_Layer  (src/Hidden_To_Hidden_Layer.h:12) Hidden_To_Hidden_Layer<float>
//   softmax_layer           (src/softmax.h:14, base_loss.h)  softmax_layer<float> : base_loss_layer<float>
//   attention_layer / node  (src/attention_layer.h:14, src/attention_node.h:11)
//
// Differences that follow from running on one GPU behind a C-ABI:
//   - cublasHandle_t / cudaStream_t / cudaEvent_t members are replaced by one zr_ctx per layer_gpu_info; all
//     layers of a model share one context (one in-order stream), so the reference's event wiring is not needed;
//   - h_t is handed to the layer above by pointer (the reference's copy_h_t == false branch,
//     src/LSTM.hpp:492-515) instead of a device-to-device copy;
//   - only dType = float exists (typedef float precision, src/global_params.h:3);
//   - back-propagation members exist for the LSTM layers, the softmax and the attention layer (backprop_prep_GPU,
//     back_prop_GPU, compute_gradients_GPU, clear_gradients, update_weights; back_prop1 / back_prop2; back_prop),
//     feed-input and dropout included; multi-source attention
//     and feed-input have none.  Gradients of the four gate matrices are kept stacked (4H x H, gate order i, f, c, o)
//     in d_M_grad_stack / d_W_h_grad_stack / d_b_grad_stack; the reference's d_M_i_grad ... members are filled from
//     them by update_weights().  Training buffers are allocated by clear_gradients(true), not by the init calls;
//   - weights are initialised with std::mt19937 instead of boost::mt19937: the value stream differs, the
//     distribution (uniform in [BZ_CUDA::lower, BZ_CUDA::upper], forget bias 1) is the same.
// Like the reference, a failed device call prints the error and exits (src/BZ_CUDA_UTIL.h:193-201).
#ifndef ZOPH_LAYERS_H
#define ZOPH_LAYERS_H

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iomanip>
#include <limits>
#include <random>
#include <sstream>
#include <string>
#include <utility>
#include <vector>

#include "../../include/zoph_rnn.h"

typedef float precision;  // src/global_params.h:3

#define ZOPH_CALL(expr)                                                                    \
  do {                                                                                     \
    int zoph_rc_ = (expr);                                                                 \
    if (zoph_rc_ != ZR_OK) {                                                               \
      std::fprintf(stderr, "Error: %s failed (%d): %s\n", #expr, zoph_rc_, zr_last_error()); \
      std::exit(EXIT_FAILURE);                                                             \
    }                                                                                      \
  } while (0)

// Mutable globals of the reference that the forward path reads (src/BZ_CUDA_UTIL.h:59-159).
namespace BZ_CUDA {
inline bool clip_cell = false;
inline precision cell_clip_threshold = 50;
// With clip_cell set the reference also clamps the back-propagated errors to +-error_clip_threshold
// (src/BZ_CUDA_UTIL.h:109; src/LSTM.hpp:792,861; src/LSTM_HH.hpp:665,756): the node classes' back_prop_GPU members do
// the same.  (Its third clamp, of d_ERRnTOt_ct at src/LSTM.hpp:888 / src/LSTM_HH.hpp:774, is queued behind that
// array's last use in the node and changes no output; it has no counterpart here.)
inline precision error_clip_threshold = 1000;
inline void clip_error(zr_ctx* ctx, float* d_err, long long n) {
  if (clip_cell) ZOPH_CALL(zr_clip_inplace(ctx, d_err, n, error_clip_threshold));
}
// The three ways of clipping gradients (src/BZ_CUDA_UTIL.h:101-118), exclusive as src/main.cu:495-511 sets them: per
// matrix (neither flag: the layers' clip_gradients / norm_clip), over the whole model (global_clip_flag, threshold =
// the layers' norm_clip) and per element (individual_grad_clip, threshold = ind_norm_clip_thres).
inline bool global_clip_flag = false;
inline precision global_norm = 0;  // host copy of the last whole-model norm, fetched by read_global_norm only
inline bool individual_grad_clip = false;
inline precision ind_norm_clip_thres = 0.1f;
// The whole-model sum of squares lives in device memory, one double per context: the updates read it there, so the
// step needs no copy to the host and no wait (the reference copies every matrix's norm back, custom_kernels.h:1088).
inline std::vector<std::pair<zr_ctx*, double*>> global_sumsq_slots;
inline double* global_sumsq(zr_ctx* ctx) {
  for (auto& s : global_sumsq_slots)
    if (s.first == ctx) return s.second;
  double* p = nullptr;
  ZOPH_CALL(zr_malloc(ctx, sizeof(double), (void**)&p));
  ZOPH_CALL(zr_memset_zero(ctx, p, sizeof(double)));
  global_sumsq_slots.emplace_back(ctx, p);
  return p;
}
inline void reset_global_norm(zr_ctx* ctx) {  // BZ_CUDA::global_norm = 0 (src/model.hpp:1852)
  ZOPH_CALL(zr_grad_sumsq_accumulate(ctx, nullptr, 0, 1.0f, global_sumsq(ctx), 1));
}
inline void add_to_global_norm(zr_ctx* ctx, const float* grad, long long n, float scale) {  // norm_clip_GPU_v2_p1
  ZOPH_CALL(zr_grad_sumsq_accumulate(ctx, grad, n, scale, global_sumsq(ctx), 0));
}
inline precision read_global_norm(zr_ctx* ctx) {  // waits for the stream (src/model.hpp:1892 takes the root on the host)
  double ss = 0;
  ZOPH_CALL(zr_d2h(ctx, &ss, global_sumsq(ctx), sizeof(double)));
  global_norm = (precision)std::sqrt(ss);
  return global_norm;
}
// One gradient's share of update_weights / update_global_params under the mode in force.  matrix_clip: the per-matrix
// threshold, 0 for none; whole_threshold: the layer's norm_clip.
inline void apply_update(zr_ctx* ctx, float* W, const float* grad, long long n, float scale, float matrix_clip,
                         float whole_threshold, float learning_rate) {
  if (individual_grad_clip)
    ZOPH_CALL(zr_sgd_update_clipped(ctx, W, grad, n, scale, ZR_CLIP_ELEMENT, ind_norm_clip_thres, nullptr, learning_rate));
  else if (global_clip_flag)
    ZOPH_CALL(zr_sgd_update_clipped(ctx, W, grad, n, scale, ZR_CLIP_WHOLE_NORM, whole_threshold, global_sumsq(ctx),
                                    learning_rate));
  else
    ZOPH_CALL(zr_sgd_update(ctx, W, grad, n, scale, matrix_clip, learning_rate));
}
inline precision lower = -0.08f;
inline precision upper = 0.08f;
inline bool force_decode = false;
inline bool unk_replacement = false;          // src/BZ_CUDA_UTIL.h:78: attention nodes also report Viterbi alignments
inline std::vector<int> viterbi_alignments;   // src/BZ_CUDA_UTIL.h:82: per beam column, filled by attention_node::forward_prop
inline std::mt19937 gen(1234);
// No counterpart in the reference: when set before the layers are initialised / loaded, every matrix the matrix cores
// stream (LSTM M / W_h / Q, attention W_a / W_p / W_c, softmax D) is snapshotted as bf16; the fp32 members stay as
// the caller's copy.  Requires LSTM_size % 16 == 0.
inline bool bf16_weights = false;
// Dropout masks.  The reference fills them with curandGenerateUniform from per-layer generators; here a mask is
// zr_uniform_fill(seed, call): seed = dropout_seed + dropout_minibatch (the owner of the layers counts the minibatches
// it has trained on), call = dropout_call(stream, node index) with one stream number per layer.
inline unsigned long long dropout_seed = 1234;
inline unsigned long long dropout_minibatch = 0;
inline unsigned long long dropout_call(int stream, int index) { return ((unsigned long long)stream << 24) | (unsigned)index; }
enum { DROPOUT_STREAM_SOURCE_INPUT = 1, DROPOUT_STREAM_TARGET_INPUT = 2, DROPOUT_STREAM_SOURCE_HIDDEN = 16,
       DROPOUT_STREAM_TARGET_HIDDEN = 48, DROPOUT_STREAM_ATTENTION = 96, DROPOUT_STREAM_SOFTMAX = 97 };
}  // namespace BZ_CUDA

struct attention_params {  // src/global_params.h:8-22 (fields used by the forward path)
  bool attention_model = false;
  int D = 10;
  bool feed_input = false;
};

struct global_params {  // src/global_params.h:61-299 (fields the layers use)
  attention_params attent_params;
  bool clip_gradient = true;
  precision norm_clip = 5.0f;
  precision learning_rate = 0.5f;
  int LSTM_size = 100;
  int minibatch_size = 8;
  int longest_sent = 100;
  int target_vocab_size = 0;
  int source_vocab_size = 0;
  bool dropout = false;            // src/global_params.h:86-87
  precision dropout_rate = 1.0f;   // probability of KEEPING a value
};

// The reference passes a cublasHandle_t& into the attention layer's constructors (src/attention_layer.h:118-119,143-144);
// the handle of this library is the context, which owns the stream the layer's work is queued on.
typedef zr_ctx* cublasHandle_t;

template <typename dType>
struct neuralMT_model {  // only what the layers consult (src/model.h:37-217)
  bool train = false;
  bool decode = false;
  bool grad_check_flag = false;  // src/model.h: dropout masks are kept instead of drawn afresh
  attention_params attent_params;
  // What attention_layer's constructor reads from the model (src/attention_layer.hpp:106-160): the source side's
  // top-layer node states, entry t = d_h_t of node t of the last source layer (model->source_hidden_layers.back().nodes[t]
  // or model->input_layer_source.nodes[t] in the reference).  The owner of the layers fills it before constructing the
  // attention layer.
  std::vector<const dType*> source_top_h_t;
  // src/model.h:107: the decoder's copies of the source states, one LSTM_size x beam matrix per source position
  std::vector<dType*> top_source_states;
};

// One context per GPU (layer_gpu_info::init, src/gpu_info_struct.h:67-172).
struct layer_gpu_info {
  int device_number = 0;
  zr_ctx* ctx = nullptr;
  void init(int device) {
    device_number = device;
    ZOPH_CALL(zr_ctx_create(device, &ctx));
  }
  void share(const layer_gpu_info& other) { *this = other; }
};
typedef layer_gpu_info softmax_layer_gpu_info;
typedef layer_gpu_info attention_layer_gpu_info;

inline void devSynchAll(zr_ctx* ctx) { ZOPH_CALL(zr_ctx_sync(ctx)); }  // src/BZ_CUDA_UTIL.h:977-987

// full_matrix_setup (src/BZ_CUDA_UTIL.h:358-364): device matrix filled U(lower, upper); the host copy is not kept.
template <typename dType>
void full_matrix_setup(zr_ctx* ctx, dType** h_ptr, dType** d_ptr, int rows, int cols) {
  std::vector<dType> tmp((size_t)rows * cols);
  std::uniform_real_distribution<double> dist(BZ_CUDA::lower, BZ_CUDA::upper);
  for (auto& v : tmp) v = (dType)dist(BZ_CUDA::gen);
  ZOPH_CALL(zr_malloc(ctx, tmp.size() * sizeof(dType), (void**)d_ptr));
  ZOPH_CALL(zr_h2d(ctx, *d_ptr, tmp.data(), tmp.size() * sizeof(dType)));
  if (h_ptr) *h_ptr = nullptr;
}
template <typename dType>
void full_matrix_setup_0(zr_ctx* ctx, dType** d_ptr, int rows, int cols) {  // :381-399, zero filled
  ZOPH_CALL(zr_malloc(ctx, (size_t)rows * cols * sizeof(dType), (void**)d_ptr));
  ZOPH_CALL(zr_memset_zero(ctx, *d_ptr, (size_t)rows * cols * sizeof(dType)));
}
template <typename dType>
void device_fill(zr_ctx* ctx, dType* d_ptr, size_t n, dType value) {
  std::vector<dType> tmp(n, value);
  ZOPH_CALL(zr_h2d(ctx, d_ptr, tmp.data(), n * sizeof(dType)));
}

// read_matrix_GPU / write_matrix_GPU (src/Eigen_Util.h:84-163): one matrix row per text line, a blank line after
// the matrix, column-major on the device.
template <typename dType>
void read_matrix_GPU(zr_ctx* ctx, dType* d_mat, int rows, int cols, std::ifstream& input) {
  std::vector<dType> tmp((size_t)rows * cols);
  std::string line, tok;
  for (int i = 0; i < rows; i++) {
    std::getline(input, line);
    std::istringstream iss(line, std::istringstream::in);
    for (int j = 0; j < cols; j++) {
      iss >> tok;
      tmp[(size_t)j * rows + i] = (dType)std::stod(tok);
    }
  }
  std::getline(input, line);
  ZOPH_CALL(zr_h2d(ctx, d_mat, tmp.data(), tmp.size() * sizeof(dType)));
}
template <typename dType>
void write_matrix_GPU(zr_ctx* ctx, dType* d_mat, int rows, int cols, std::ofstream& output) {
  std::vector<dType> tmp((size_t)rows * cols);
  ZOPH_CALL(zr_d2h(ctx, tmp.data(), d_mat, tmp.size() * sizeof(dType)));
  for (int i = 0; i < rows; i++) {
    for (int j = 0; j < cols; j++) {
      output << tmp[(size_t)j * rows + i];
      if (j != cols - 1) output << " ";
    }
    output << "\n";
  }
  output << "\n";
}

template <typename dType> class Input_To_Hidden_Layer;
template <typename dType> class Hidden_To_Hidden_Layer;
template <typename dType> class attention_layer;
template <typename dType> class base_loss_layer;

// src/transfer_layer.h:18-41
template <typename dType>
struct upper_transfer_layer {
  bool upper_softmax = true;
  bool copy_h_t = false;
  bool source_side = true;
  base_loss_layer<dType>* softmax = nullptr;
  Hidden_To_Hidden_Layer<dType>* hidden_layer = nullptr;
  void init_upper_transfer_layer(bool upper_softmax, bool copy_h_t, bool source_side, base_loss_layer<dType>* softmax,
                                 Hidden_To_Hidden_Layer<dType>* hidden_layer) {
    this->upper_softmax = upper_softmax;
    this->copy_h_t = copy_h_t;
    this->source_side = source_side;
    this->softmax = softmax;
    this->hidden_layer = hidden_layer;
  }
};

// src/transfer_layer.h:38-55
template <typename dType>
struct lower_transfer_layer {
  bool lower_input = true;     // the layer below is the input layer (else a hidden layer)
  bool copy_d_Err_ht = false;  // one GPU: the error is handed down by pointer
  Input_To_Hidden_Layer<dType>* input_layer = nullptr;
  Hidden_To_Hidden_Layer<dType>* hidden_layer = nullptr;
  void init_lower_transfer_layer(bool lower_input, bool copy_d_Err_ht, Input_To_Hidden_Layer<dType>* input_layer,
                                 Hidden_To_Hidden_Layer<dType>* hidden_layer) {
    this->lower_input = lower_input;
    this->copy_d_Err_ht = copy_d_Err_ht;
    this->input_layer = input_layer;
    this->hidden_layer = hidden_layer;
  }
  inline void send_error(int index, dType* d_err);  // node `index` of the layer below takes d_err as its d_d_ERRt_ht
};

// ------------------------------------------------------------------------------------------------ attention
template <typename dType>
class attention_node {  // src/attention_node.h:11-86
 public:
  int LSTM_size, minibatch_size, device_number, D, index;
  bool feed_input;
  attention_layer<dType>* attent_layer;
  dType* d_h_t = nullptr;          // input: top-layer target hidden state
  dType* d_final_temp_2 = nullptr; // output h~
  dType* d_alignments = nullptr;
  dType* d_p_t = nullptr;
  dType* d_c_t = nullptr;
  int* d_indicies = nullptr;
  int** d_indicies_mask = nullptr;  // points at the owning LSTM node's 0/1 mask pointer
  dType* d_lower_htild = nullptr;   // feed-input destination: next step's bottom node d_h_tild
  // training
  bool dropout = false;
  dType dropout_rate = 1;
  dType* d_dropout_mask = nullptr;
  dType* d_h_t_att = nullptr;              // the h_t the step read: d_h_t, or its dropped-out copy
  dType* d_h_t_att_buf = nullptr;          // storage of that copy (dropout only)
  dType* d_d_ERRt_ht_tild = nullptr;       // error of h~ in, error of h_t out: the owning LSTM node's d_d_ERRt_ht
  dType* d_ERRtTOn_htild_below = nullptr;  // error of h~ arriving from the next step's bottom node (feed-input)

  attention_node(int LSTM_size, int minibatch_size, int device_number, int D, bool feed_input,
                 attention_layer<dType>* attent_layer, int index);
  void feed_input_init(dType* d_ptr_htild);  // src/attention_node.hpp:56-60
  void forward_prop();                        // src/attention_node.hpp:73-394
  void back_prop();                           // src/attention_node.hpp:398-669
};

template <typename dType>
class attention_layer {  // src/attention_layer.h:14-143
 public:
  attention_layer_gpu_info layer_info;
  int LSTM_size, minibatch_size, device_number, D, longest_sent;
  bool feed_input;
  dType *d_W_a = nullptr, *d_W_p = nullptr, *d_v_p = nullptr, *d_output_bias = nullptr, *d_W_c_p1 = nullptr,
        *d_W_c_p2 = nullptr;
  int* d_batch_info = nullptr;
  std::vector<const dType*> h_total_hs_mat;  // host copy of d_total_hs_mat (src/attention_layer.hpp:106-160)
  zr_attn* attn = nullptr;
  int* d_viterbi_alignments = nullptr;  // minibatch_size ints, allocated when BZ_CUDA::unk_replacement is set
  int* d_ones_minibatch_int = nullptr;  // init_att_decoder: the decode path runs every column with mask 1
  neuralMT_model<dType>* model = nullptr;
  std::vector<attention_node<dType>> nodes;
  // training (src/attention_layer.h:60-100; allocated by the first clear_gradients())
  dType *d_W_a_grad = nullptr, *d_W_p_grad = nullptr, *d_v_p_grad = nullptr, *d_output_bias_grad = nullptr,
        *d_W_c_p1_grad = nullptr, *d_W_c_p2_grad = nullptr;
  std::vector<dType*> h_total_hs_error;  // d_total_hs_error: entry t receives the error of source state t
  bool transfer_done = false;            // src/attention_layer.h: false until the last step's node has run backward
  bool clip_gradients = true, dropout = false;
  dType norm_clip = 5, learning_rate = 0.5f, dropout_rate = 1;

  attention_layer() {}

  // The reference's own parameter list (src/attention_layer.h:118-119, body src/attention_layer.hpp:3-173).  `handle`
  // is the context (cublasHandle_t above); the source states come from model->source_top_h_t.  The second source side
  // of a multi-source model is not built and is refused.
  attention_layer(int LSTM_size, int minibatch_size, int device_number, int D, int longest_sent, cublasHandle_t& handle,
                  neuralMT_model<dType>* model, bool feed_input, bool clip_gradients, dType norm_clip,
                  bool dropout, dType dropout_rate, global_params& params, bool bi_side) {
    if (bi_side || !model || (int)model->source_top_h_t.size() < longest_sent) {
      std::fprintf(stderr, "Error: attention_layer: multi-source attention is not built, and the model must list its "
                   "%d source top-layer states in source_top_h_t\n", longest_sent);
      std::exit(EXIT_FAILURE);
    }
    layer_gpu_info gpu;
    gpu.device_number = device_number;
    gpu.ctx = handle;
    this->model = model;
    this->clip_gradients = clip_gradients;
    this->norm_clip = norm_clip;
    this->learning_rate = params.learning_rate;
    this->dropout = dropout;
    this->dropout_rate = dropout_rate;
    setup(LSTM_size, minibatch_size, device_number, D, longest_sent, gpu, model->source_top_h_t, feed_input, longest_sent);
  }

  // src/attention_layer.hpp:3-173.  total_hs: the source top-layer node states, entry t = node t's d_h_t.
  attention_layer(int LSTM_size, int minibatch_size, int device_number, int D, int longest_sent,
                  const layer_gpu_info& gpu, const std::vector<const dType*>& total_hs, bool feed_input) {
    setup(LSTM_size, minibatch_size, device_number, D, longest_sent, gpu, total_hs, feed_input, longest_sent);
  }

  // The decode-time layer (src/attention_layer.h:143-144, body src/attention_layer.hpp:176-259): minibatch = beam, ONE
  // node whose mask is all ones, source states read from top_source_states (the decoder's LSTM_size x beam copies,
  // src/model.hpp:565-583).  feed_input is always false here as in the reference: the decode driver moves h~ itself.
  // multi_attention_v2 is not built.
  void init_att_decoder(int LSTM_size, int beam_size, int device_number, int D, int longest_sent, cublasHandle_t& handle,
                        neuralMT_model<dType>* model, bool feed_input, std::vector<dType*>& top_source_states,
                        bool multi_attention_v2, std::vector<dType*>& /*top_source_states_v2*/) {
    if (multi_attention_v2 || (int)top_source_states.size() < longest_sent) {
      std::fprintf(stderr, "Error: init_att_decoder: multi_attention_v2 is not built, and top_source_states must hold "
                   "%d matrices\n", longest_sent);
      std::exit(EXIT_FAILURE);
    }
    layer_gpu_info gpu;
    gpu.device_number = device_number;
    gpu.ctx = handle;
    this->model = model;
    std::vector<const dType*> total_hs(top_source_states.begin(), top_source_states.begin() + longest_sent);
    setup(LSTM_size, beam_size, device_number, D, longest_sent, gpu, total_hs, feed_input, 1);
    std::vector<int> ones((size_t)beam_size, 1);
    ZOPH_CALL(zr_malloc(gpu.ctx, ones.size() * sizeof(int), (void**)&d_ones_minibatch_int));
    ZOPH_CALL(zr_h2d(gpu.ctx, d_ones_minibatch_int, ones.data(), ones.size() * sizeof(int)));
    nodes[0].d_indicies_mask = &d_ones_minibatch_int;
  }

  void setup(int LSTM_size, int minibatch_size, int device_number, int D, int longest_sent, const layer_gpu_info& gpu,
             const std::vector<const dType*>& total_hs, bool feed_input, int n_nodes) {
    this->LSTM_size = LSTM_size;
    this->minibatch_size = minibatch_size;
    this->device_number = device_number;
    this->D = D;
    this->longest_sent = longest_sent;
    this->feed_input = feed_input;
    layer_info.share(gpu);
    zr_ctx* ctx = layer_info.ctx;
    dType* h = nullptr;
    full_matrix_setup(ctx, &h, &d_W_a, LSTM_size, LSTM_size);
    full_matrix_setup(ctx, &h, &d_W_p, LSTM_size, LSTM_size);
    full_matrix_setup(ctx, &h, &d_v_p, 1, LSTM_size);
    full_matrix_setup(ctx, &h, &d_output_bias, LSTM_size, 1);
    full_matrix_setup(ctx, &h, &d_W_c_p1, LSTM_size, LSTM_size);
    full_matrix_setup(ctx, &h, &d_W_c_p2, LSTM_size, LSTM_size);
    ZOPH_CALL(zr_malloc(ctx, 2 * (size_t)minibatch_size * sizeof(int), (void**)&d_batch_info));
    h_total_hs_mat = total_hs;
    ZOPH_CALL(zr_attn_create(ctx, LSTM_size, minibatch_size, D, d_W_a, d_W_p, d_v_p, d_output_bias, d_W_c_p1, d_W_c_p2,
                             h_total_hs_mat.data(), (int)h_total_hs_mat.size(), &attn));
    if (BZ_CUDA::bf16_weights)
      ZOPH_CALL(zr_attn_use_bf16_weights(ctx, attn));
    else
      ZOPH_CALL(zr_attn_prepare(ctx, attn));
    if (BZ_CUDA::unk_replacement) {  // src/attention_layer.hpp:252-255
      ZOPH_CALL(zr_malloc(ctx, (size_t)minibatch_size * sizeof(int), (void**)&d_viterbi_alignments));
      BZ_CUDA::viterbi_alignments.assign((size_t)minibatch_size, -1);
    }
    for (int i = 0; i < n_nodes; i++)
      nodes.push_back(attention_node<dType>(LSTM_size, minibatch_size, device_number, D, feed_input, this, i));
  }
  // ---- training.  clear_gradients (src/attention_layer.hpp:262-300) zeroes the six gradients (allocating them and the
  // source-state error arrays the first time) and the errors of the source states; the owner of the encoder's top
  // layer hands error array t to that layer's node t as its error from above (the reference points d_total_hs_error at
  // those nodes' d_d_ERRt_ht, src/attention_layer.hpp:106-160).
  void clear_gradients() {
    zr_ctx* ctx = layer_info.ctx;
    const size_t hh = (size_t)LSTM_size * LSTM_size, n = (size_t)LSTM_size * minibatch_size;
    if (!d_W_a_grad) {
      dType** mats[] = {&d_W_a_grad, &d_W_p_grad, &d_W_c_p1_grad, &d_W_c_p2_grad};
      for (dType** m : mats) ZOPH_CALL(zr_malloc(ctx, hh * sizeof(dType), (void**)m));
      ZOPH_CALL(zr_malloc(ctx, (size_t)LSTM_size * sizeof(dType), (void**)&d_v_p_grad));
      ZOPH_CALL(zr_malloc(ctx, (size_t)LSTM_size * sizeof(dType), (void**)&d_output_bias_grad));
      h_total_hs_error.resize(h_total_hs_mat.size());
      for (auto& e : h_total_hs_error) ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&e));
      ZOPH_CALL(zr_attn_set_error_tables(ctx, attn, h_total_hs_error.data(), (int)h_total_hs_error.size()));
    }
    dType* mats[] = {d_W_a_grad, d_W_p_grad, d_W_c_p1_grad, d_W_c_p2_grad};
    for (dType* m : mats) ZOPH_CALL(zr_memset_zero(ctx, m, hh * sizeof(dType)));
    ZOPH_CALL(zr_memset_zero(ctx, d_v_p_grad, (size_t)LSTM_size * sizeof(dType)));
    ZOPH_CALL(zr_memset_zero(ctx, d_output_bias_grad, (size_t)LSTM_size * sizeof(dType)));
    for (dType* e : h_total_hs_error) ZOPH_CALL(zr_memset_zero(ctx, e, n * sizeof(dType)));
    transfer_done = false;
  }
  // norm_p1 (src/attention_layer.hpp): this layer's share of the whole-model gradient norm
  void calculate_global_norm() {
    zr_ctx* ctx = layer_info.ctx;
    const float scale = 1.0f / (float)minibatch_size;
    const long long hh = (long long)LSTM_size * LSTM_size;
    for (const dType* g : {d_W_a_grad, d_W_p_grad, d_W_c_p1_grad, d_W_c_p2_grad}) BZ_CUDA::add_to_global_norm(ctx, g, hh, scale);
    for (const dType* g : {d_v_p_grad, d_output_bias_grad}) BZ_CUDA::add_to_global_norm(ctx, g, LSTM_size, scale);
  }
  void update_global_params() { update_weights(); }  // norm_p2 + update_params
  // scale_gradients, the clipping mode in force (norm_clip_GPU_v2 per matrix unless BZ_CUDA says otherwise),
  // update_params (src/attention_layer.hpp:303-420); then the snapshots the forward kernels read are rebuilt
  void update_weights() {
    zr_ctx* ctx = layer_info.ctx;
    const float scale = 1.0f / (float)minibatch_size, clip = clip_gradients ? (float)norm_clip : 0.0f;
    const long long hh = (long long)LSTM_size * LSTM_size;
    BZ_CUDA::apply_update(ctx, d_W_a, d_W_a_grad, hh, scale, clip, (float)norm_clip, learning_rate);
    BZ_CUDA::apply_update(ctx, d_W_p, d_W_p_grad, hh, scale, clip, (float)norm_clip, learning_rate);
    BZ_CUDA::apply_update(ctx, d_v_p, d_v_p_grad, LSTM_size, scale, clip, (float)norm_clip, learning_rate);
    BZ_CUDA::apply_update(ctx, d_output_bias, d_output_bias_grad, LSTM_size, scale, clip, (float)norm_clip, learning_rate);
    BZ_CUDA::apply_update(ctx, d_W_c_p1, d_W_c_p1_grad, hh, scale, clip, (float)norm_clip, learning_rate);
    BZ_CUDA::apply_update(ctx, d_W_c_p2, d_W_c_p2_grad, hh, scale, clip, (float)norm_clip, learning_rate);
    if (BZ_CUDA::bf16_weights)
      ZOPH_CALL(zr_attn_use_bf16_weights(ctx, attn));
    else
      ZOPH_CALL(zr_attn_prepare(ctx, attn));
  }
  // src/attention_layer.hpp:580-583
  void prep_minibatch_info(int* h_batch_info) {
    ZOPH_CALL(zr_h2d(layer_info.ctx, d_batch_info, h_batch_info, 2 * (size_t)minibatch_size * sizeof(int)));
  }
  // weight order of the model file: W_a, W_p, v_p (LSTM_size x 1), output_bias, W_c_p1, W_c_p2
  // (src/attention_layer.hpp:467-473)
  void dump_weights(std::ofstream& output) {
    zr_ctx* ctx = layer_info.ctx;
    write_matrix_GPU(ctx, d_W_a, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_W_p, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_v_p, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_output_bias, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_W_c_p1, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_W_c_p2, LSTM_size, LSTM_size, output);
  }
  void load_weights(std::ifstream& input) {
    zr_ctx* ctx = layer_info.ctx;
    read_matrix_GPU(ctx, d_W_a, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_W_p, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_v_p, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_output_bias, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_W_c_p1, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_W_c_p2, LSTM_size, LSTM_size, input);
    if (attn) {  // the snapshots follow the matrices
      if (BZ_CUDA::bf16_weights)
        ZOPH_CALL(zr_attn_use_bf16_weights(ctx, attn));
      else
        ZOPH_CALL(zr_attn_prepare(ctx, attn));
    }
  }
};

template <typename dType>
attention_node<dType>::attention_node(int LSTM_size, int minibatch_size, int device_number, int D, bool feed_input,
                                      attention_layer<dType>* attent_layer, int index) {
  this->LSTM_size = LSTM_size;
  this->minibatch_size = minibatch_size;
  this->device_number = device_number;
  this->D = D;
  this->feed_input = feed_input;
  this->attent_layer = attent_layer;
  this->index = index;
  this->dropout = attent_layer->dropout;
  this->dropout_rate = attent_layer->dropout_rate;
  zr_ctx* ctx = attent_layer->layer_info.ctx;
  const size_t n = (size_t)LSTM_size * minibatch_size, w = (size_t)(2 * D + 1) * minibatch_size;
  ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&d_final_temp_2));
  ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&d_c_t));
  ZOPH_CALL(zr_malloc(ctx, w * sizeof(dType), (void**)&d_alignments));
  ZOPH_CALL(zr_malloc(ctx, w * sizeof(int), (void**)&d_indicies));
  ZOPH_CALL(zr_malloc(ctx, (size_t)minibatch_size * sizeof(dType), (void**)&d_p_t));
}

template <typename dType>
void attention_node<dType>::feed_input_init(dType* d_ptr_htild) {
  d_lower_htild = d_ptr_htild;
  full_matrix_setup_0(attent_layer->layer_info.ctx, &d_ERRtTOn_htild_below, LSTM_size, minibatch_size);
}

template <typename dType>
void attention_node<dType>::forward_prop() {
  zr_ctx* ctx = attent_layer->layer_info.ctx;
  const size_t n = (size_t)LSTM_size * minibatch_size;
  d_h_t_att = d_h_t;
  if (dropout && attent_layer->model && attent_layer->model->train) {  // src/attention_node.hpp:98-106
    if (!d_dropout_mask) {
      ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&d_dropout_mask));
      ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&d_h_t_att_buf));
    }
    if (!attent_layer->model->grad_check_flag)
      ZOPH_CALL(zr_uniform_fill(ctx, BZ_CUDA::dropout_seed + BZ_CUDA::dropout_minibatch,
                                BZ_CUDA::dropout_call(BZ_CUDA::DROPOUT_STREAM_ATTENTION, index), d_dropout_mask,
                                (long long)n));
    ZOPH_CALL(zr_d2d(ctx, d_h_t_att_buf, d_h_t, n * sizeof(dType)));
    ZOPH_CALL(zr_dropout_apply(ctx, d_dropout_mask, dropout_rate, d_h_t_att_buf, (long long)n));
    d_h_t_att = d_h_t_att_buf;
  }
  ZOPH_CALL(zr_attn_step(ctx, attent_layer->attn, attent_layer->d_batch_info, d_h_t_att, *d_indicies_mask,
                         d_final_temp_2, d_alignments, d_indicies, d_p_t, d_c_t));
  if (BZ_CUDA::unk_replacement && attent_layer->d_viterbi_alignments) {  // src/attention_node.hpp:225-234
    ZOPH_CALL(zr_attn_viterbi(ctx, attent_layer->attn, d_alignments, d_indicies, attent_layer->d_viterbi_alignments));
    BZ_CUDA::viterbi_alignments.resize((size_t)minibatch_size);
    ZOPH_CALL(zr_d2h(ctx, BZ_CUDA::viterbi_alignments.data(), attent_layer->d_viterbi_alignments,
                     (size_t)minibatch_size * sizeof(int)));
  }
  // feed-input: h~ goes to the next time step's bottom node (src/attention_node.hpp:384-386)
  if (feed_input && index != (attent_layer->longest_sent - 1) && d_lower_htild)
    ZOPH_CALL(zr_d2d(ctx, d_lower_htild, d_final_temp_2, (size_t)LSTM_size * minibatch_size * sizeof(dType)));
}

// src/attention_node.hpp:398-669.  d_d_ERRt_ht_tild holds the error of h~ on entry (the loss layer's) and the error of
// h_t on return, as in the reference (:654).
template <typename dType>
void attention_node<dType>::back_prop() {
  zr_ctx* ctx = attent_layer->layer_info.ctx;
  const long long n = (long long)LSTM_size * minibatch_size;
  if (!attent_layer->d_W_a_grad) attent_layer->clear_gradients();
  // the error the next step's bottom node sent through its Q matrices; the last step has none (:407-422)
  if (feed_input && attent_layer->transfer_done && d_ERRtTOn_htild_below)
    ZOPH_CALL(zr_add_inplace(ctx, d_d_ERRt_ht_tild, d_ERRtTOn_htild_below, n));
  attent_layer->transfer_done = true;
  zr_attn_grads g = {attent_layer->d_W_a_grad, attent_layer->d_W_p_grad, attent_layer->d_v_p_grad,
                     attent_layer->d_output_bias_grad, attent_layer->d_W_c_p1_grad, attent_layer->d_W_c_p2_grad};
  ZOPH_CALL(zr_attn_backward(ctx, attent_layer->attn, attent_layer->d_batch_info, d_h_t_att ? d_h_t_att : d_h_t,
                             *d_indicies_mask, d_final_temp_2, d_alignments, d_indicies, d_p_t, d_c_t, d_d_ERRt_ht_tild,
                             d_d_ERRt_ht_tild, &g));
  if (dropout && d_dropout_mask && d_h_t_att == d_h_t_att_buf)  // :646-648
    ZOPH_CALL(zr_dropout_apply(ctx, d_dropout_mask, dropout_rate, d_d_ERRt_ht_tild, n));
}

// ------------------------------------------------------------------------------------------------ loss layer
template <typename dType>
class base_loss_layer {  // src/base_loss.h:13-64 (forward-path subset)
 public:
  virtual ~base_loss_layer() {}
  virtual softmax_layer_gpu_info gpu_init(int device_number) = 0;
  virtual void init_loss_layer(struct neuralMT_model<precision>* model, global_params& params) = 0;
  virtual void forward_prop(int index) = 0;
  virtual void back_prop1(int index) = 0;
  virtual void back_prop2(int index) = 0;
  virtual void clear_gradients() = 0;
  virtual void update_weights() = 0;
  virtual void update_learning_rate(dType learning_rate) = 0;
  virtual void init_lower_transfer_layer(bool lower_input, bool copy_d_Err_ht, Input_To_Hidden_Layer<dType>* input_layer,
                                         Hidden_To_Hidden_Layer<dType>* hidden_layer) = 0;
  virtual void backprop_prep_GPU(dType* d_h_t, int step) = 0;
  virtual void backprop_prep_GPU_mgpu(int step) = 0;
  virtual void prep_GPU_vocab_indices(int* h_output_vocab_indicies_target, int current_target_length) = 0;
  virtual double compute_loss_GPU(int index) = 0;
  virtual dType* get_ht_ptr(int index) = 0;
  virtual void set_ht_ptr(int index, dType* d_h_t) = 0;
  virtual void load_weights(std::ifstream& input) = 0;
  virtual void dump_weights(std::ofstream& output) = 0;
  virtual void get_distribution_GPU_decoder_wrapper() = 0;
  virtual dType* get_dist_ptr() = 0;
};

template <typename dType>
struct softmax_node {  // src/softmax_node.h:7-27
  dType* d_outputdist = nullptr;
  dType* d_h_t = nullptr;
  dType* d_d_ERRt_ht = nullptr;  // error at h_t of this step (allocated on first use by back_prop1)
  dType *d_dropout_mask = nullptr, *d_h_t_drop = nullptr;  // dropout: the mask and the dropped-out copy of d_h_t
  int index = 0;
};

template <typename dType>
class softmax_layer : public base_loss_layer<dType> {  // src/softmax.h:14-225
 public:
  softmax_layer_gpu_info s_layer_info;
  int output_vocab_size = 0, LSTM_size = 0, minibatch_size = 0, longest_sent = 0;
  dType *d_D = nullptr, *d_b_d = nullptr;
  dType* d_outputdist = nullptr;       // V x minibatch probabilities (decoder path)
  double* d_outputdist_perp = nullptr; // V x minibatch double log-probabilities (allocated on first use)
  dType* d_logits = nullptr;           // scratch
  dType* d_h_t = nullptr;
  int *d_output_vocab_indices = nullptr, *d_output_vocab_indices_01 = nullptr;
  dType* d_output_vocab_indices_01_float = nullptr;
  int *d_output_vocab_indices_single = nullptr, *d_output_vocab_indices_01_single = nullptr;
  std::vector<softmax_node<dType>> nodes;
  dType *d_D_grad = nullptr, *d_b_d_grad = nullptr;  // allocated by the first clear_gradients()
  bool clip_gradients = true;
  dType norm_clip = 5, learning_rate = 0.5f;
  lower_transfer_layer<dType> lower_layer;
  // dropout on the layer's input, models without attention only (src/softmax.hpp:474-478, :745-747)
  bool dropout = false;
  dType dropout_rate = 1;
  neuralMT_model<precision>* model = nullptr;
  // the h_t of node `index` as the loss layer reads it in training: dropped out once per node and minibatch
  dType* training_input(int index) {
    dType* h = nodes[index].d_h_t ? nodes[index].d_h_t : d_h_t;
    if (!(dropout && model && model->train && !model->attent_params.attention_model)) return h;
    zr_ctx* ctx = s_layer_info.ctx;
    const size_t n = (size_t)LSTM_size * minibatch_size;
    auto& nd = nodes[index];
    if (!nd.d_dropout_mask) {
      ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&nd.d_dropout_mask));
      ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&nd.d_h_t_drop));
    }
    if (!model->grad_check_flag)
      ZOPH_CALL(zr_uniform_fill(ctx, BZ_CUDA::dropout_seed + BZ_CUDA::dropout_minibatch,
                                BZ_CUDA::dropout_call(BZ_CUDA::DROPOUT_STREAM_SOFTMAX, index), nd.d_dropout_mask,
                                (long long)n));
    ZOPH_CALL(zr_d2d(ctx, nd.d_h_t_drop, h, n * sizeof(dType)));
    ZOPH_CALL(zr_dropout_apply(ctx, nd.d_dropout_mask, dropout_rate, nd.d_h_t_drop, (long long)n));
    return nd.d_h_t_drop;
  }

  softmax_layer_gpu_info gpu_init(int device_number) override {
    if (!s_layer_info.ctx) s_layer_info.init(device_number);
    return s_layer_info;
  }
  void share_gpu(const layer_gpu_info& gpu) { s_layer_info.share(gpu); }

  // src/softmax.hpp:3-100: sizes come from params; D and b_d are U(lower, upper)
  void init_loss_layer(struct neuralMT_model<precision>* model, global_params& params) override {
    this->model = model;
    dropout = params.dropout;
    dropout_rate = params.dropout_rate;
    output_vocab_size = params.target_vocab_size;
    LSTM_size = params.LSTM_size;
    minibatch_size = params.minibatch_size;
    longest_sent = params.longest_sent;
    clip_gradients = params.clip_gradient;
    norm_clip = params.norm_clip;
    learning_rate = params.learning_rate;
    zr_ctx* ctx = s_layer_info.ctx;
    dType* h = nullptr;
    full_matrix_setup(ctx, &h, &d_D, output_vocab_size, LSTM_size);
    full_matrix_setup(ctx, &h, &d_b_d, output_vocab_size, 1);
    const size_t vm = (size_t)output_vocab_size * minibatch_size;
    ZOPH_CALL(zr_malloc(ctx, vm * sizeof(dType), (void**)&d_outputdist));
    ZOPH_CALL(zr_malloc(ctx, vm * sizeof(dType), (void**)&d_logits));
    const size_t nt = (size_t)minibatch_size * longest_sent;
    ZOPH_CALL(zr_malloc(ctx, nt * sizeof(int), (void**)&d_output_vocab_indices));
    ZOPH_CALL(zr_malloc(ctx, nt * sizeof(int), (void**)&d_output_vocab_indices_01));
    ZOPH_CALL(zr_malloc(ctx, nt * sizeof(dType), (void**)&d_output_vocab_indices_01_float));
    nodes.resize(longest_sent);
    for (int i = 0; i < longest_sent; i++) nodes[i].index = i;
    prepare_weights();
  }
  // src/softmax.hpp:926-947
  void prep_GPU_vocab_indices(int* h_output_vocab_indicies_target, int current_target_length) override {
    zr_ctx* ctx = s_layer_info.ctx;
    const int n = minibatch_size * current_target_length;
    ZOPH_CALL(zr_h2d(ctx, d_output_vocab_indices, h_output_vocab_indicies_target, (size_t)n * sizeof(int)));
    ZOPH_CALL(zr_vocab_prep_softmax(ctx, d_output_vocab_indices, n, output_vocab_size, d_output_vocab_indices_01,
                                    d_output_vocab_indices_01_float));
  }
  // src/softmax.hpp:907-923
  void backprop_prep_GPU(dType* d_h_t, int step) override {
    this->d_h_t = d_h_t;
    backprop_prep_GPU_mgpu(step);
  }
  void backprop_prep_GPU_mgpu(int step) override {
    d_output_vocab_indices_single = d_output_vocab_indices + step;
    d_output_vocab_indices_01_single = d_output_vocab_indices_01 + step;
  }
  // src/softmax.hpp:459-485: probabilities of node `index` (training-style forward; the node keeps its d_h_t)
  void forward_prop(int index) override {
    zr_ctx* ctx = s_layer_info.ctx;
    if (!nodes[index].d_outputdist)
      ZOPH_CALL(zr_malloc(ctx, (size_t)output_vocab_size * minibatch_size * sizeof(dType),
                          (void**)&nodes[index].d_outputdist));
    ZOPH_CALL(zr_softmax_forward(ctx, d_D, d_b_d, output_vocab_size, LSTM_size, nodes[index].d_h_t, minibatch_size,
                                 ZR_SOFTMAX_PROB, nodes[index].d_outputdist, nullptr));
  }
  // src/softmax.hpp:867-900 (get_perplexity_GPU + the host-side sum)
  double compute_loss_GPU(int index) override {
    zr_ctx* ctx = s_layer_info.ctx;
    dType* h = nodes[index].d_h_t ? nodes[index].d_h_t : d_h_t;
    double loss = 0;
    ZOPH_CALL(zr_softmax_loss(ctx, d_D, d_b_d, output_vocab_size, LSTM_size, h, minibatch_size,
                              d_output_vocab_indices_single, d_output_vocab_indices_01_single, d_logits, &loss));
    return loss;
  }
  // src/softmax.hpp:636-692: the full double log-probability matrix of d_h_t into d_outputdist_perp
  void get_perplexity_GPU(dType* d_h_t_in, int /*index*/) {
    zr_ctx* ctx = s_layer_info.ctx;
    if (!d_outputdist_perp)
      ZOPH_CALL(zr_malloc(ctx, (size_t)output_vocab_size * minibatch_size * sizeof(double), (void**)&d_outputdist_perp));
    ZOPH_CALL(zr_softmax_logprob_f64(ctx, d_D, d_b_d, output_vocab_size, LSTM_size, d_h_t_in, minibatch_size,
                                     d_outputdist_perp, d_logits));
  }
  // ---- training (src/softmax.hpp:232-300, 600-860)
  void init_lower_transfer_layer(bool lower_input, bool copy_d_Err_ht, Input_To_Hidden_Layer<dType>* input_layer,
                                 Hidden_To_Hidden_Layer<dType>* hidden_layer) override {
    lower_layer.init_lower_transfer_layer(lower_input, copy_d_Err_ht, input_layer, hidden_layer);
  }
  void clear_gradients() override {
    zr_ctx* ctx = s_layer_info.ctx;
    const size_t vh = (size_t)output_vocab_size * LSTM_size;
    if (!d_D_grad) {
      ZOPH_CALL(zr_malloc(ctx, vh * sizeof(dType), (void**)&d_D_grad));
      ZOPH_CALL(zr_malloc(ctx, (size_t)output_vocab_size * sizeof(dType), (void**)&d_b_d_grad));
    }
    ZOPH_CALL(zr_memset_zero(ctx, d_D_grad, vh * sizeof(dType)));
    ZOPH_CALL(zr_memset_zero(ctx, d_b_d_grad, (size_t)output_vocab_size * sizeof(dType)));
  }
  // back_prop1: the error at h_t of step `index` (get_h_t_gradient_GPU), handed to the layer below.  The D and b_d
  // gradient terms of the step (compute_D_gradient_GPU, compute_b_d_gradient_GPU -- back_prop2 in the reference) come
  // out of the same library call, so they are accumulated here and back_prop2 has nothing left to do.  The step's
  // distribution is recomputed from nodes[index].d_h_t; backprop_prep_GPU(_, index * minibatch_size) must precede.
  void back_prop1(int index) override {
    zr_ctx* ctx = s_layer_info.ctx;
    if (!d_D_grad) clear_gradients();
    if (!nodes[index].d_d_ERRt_ht) full_matrix_setup_0(ctx, &nodes[index].d_d_ERRt_ht, LSTM_size, minibatch_size);
    dType* h = training_input(index);
    ZOPH_CALL(zr_softmax_backward_accumulate(ctx, d_D, d_b_d, output_vocab_size, LSTM_size, h, minibatch_size,
                                             d_output_vocab_indices_single, d_output_vocab_indices_01_single,
                                             d_logits, nodes[index].d_d_ERRt_ht, d_D_grad, d_b_d_grad));
    if (h == nodes[index].d_h_t_drop && h)  // src/softmax.hpp:745-747
      ZOPH_CALL(zr_dropout_apply(ctx, nodes[index].d_dropout_mask, dropout_rate, nodes[index].d_d_ERRt_ht,
                                 (long long)LSTM_size * minibatch_size));
    lower_layer.send_error(index, nodes[index].d_d_ERRt_ht);
  }
  void back_prop2(int /*index*/) override {}
  void calculate_global_norm() {  // src/softmax.hpp calculate_global_norm
    zr_ctx* ctx = s_layer_info.ctx;
    const float scale = 1.0f / (float)minibatch_size;
    BZ_CUDA::add_to_global_norm(ctx, d_D_grad, (long long)output_vocab_size * LSTM_size, scale);
    BZ_CUDA::add_to_global_norm(ctx, d_b_d_grad, output_vocab_size, scale);
  }
  void update_global_params() { update_weights(); }
  // scale by 1 / minibatch_size, clip (each gradient to norm_clip in L2 norm unless BZ_CUDA selects another mode), add
  // (gradient ascent on log-likelihood)
  void update_weights() override {
    zr_ctx* ctx = s_layer_info.ctx;
    const float scale = 1.0f / (float)minibatch_size, clip = clip_gradients ? norm_clip : 0.0f;
    BZ_CUDA::apply_update(ctx, d_D, d_D_grad, (long long)output_vocab_size * LSTM_size, scale, clip, (float)norm_clip, learning_rate);
    BZ_CUDA::apply_update(ctx, d_b_d, d_b_d_grad, output_vocab_size, scale, clip, (float)norm_clip, learning_rate);
    prepare_weights();
  }
  void update_learning_rate(dType lr) override { learning_rate = lr; }
  dType* get_ht_ptr(int index) override { return nodes[index].d_h_t; }
  void set_ht_ptr(int index, dType* d_h_t) override { nodes[index].d_h_t = d_h_t; }
  // src/softmax.hpp:1028-1030
  void get_distribution_GPU_decoder_wrapper() override {
    ZOPH_CALL(zr_softmax_forward(s_layer_info.ctx, d_D, d_b_d, output_vocab_size, LSTM_size, d_h_t, minibatch_size,
                                 ZR_SOFTMAX_PROB, d_outputdist, nullptr));
  }
  dType* get_dist_ptr() override { return d_outputdist; }
  // src/softmax.hpp:310-323
  void dump_weights(std::ofstream& output) override {
    write_matrix_GPU(s_layer_info.ctx, d_D, output_vocab_size, LSTM_size, output);
    write_matrix_GPU(s_layer_info.ctx, d_b_d, output_vocab_size, 1, output);
  }
  void load_weights(std::ifstream& input) override {
    read_matrix_GPU(s_layer_info.ctx, d_D, output_vocab_size, LSTM_size, input);
    read_matrix_GPU(s_layer_info.ctx, d_b_d, output_vocab_size, 1, input);
    prepare_weights();
  }
  // No counterpart in the reference: snapshots d_D into the layout the matrix cores read fastest.  Called after
  // init_loss_layer and load_weights; call again by hand after writing to d_D.
  void prepare_weights() {
    if (BZ_CUDA::bf16_weights)
      ZOPH_CALL(zr_softmax_prepare_bf16(s_layer_info.ctx, d_D, output_vocab_size, LSTM_size));
    else
      ZOPH_CALL(zr_softmax_prepare(s_layer_info.ctx, d_D, output_vocab_size, LSTM_size));
  }
};

// ------------------------------------------------------------------------------------------------ LSTM nodes
// Training-side members both LSTM layer classes carry (the reference declares them in each class:
// src/Hidden_To_Hidden_Layer.h:143-233, src/Input_To_Hidden_Layer.h).  Nothing here is allocated until
// clear_gradients(true) runs.
template <typename dType>
struct lstm_layer_training {
  zr_lstm_train* train_weights = nullptr;  // transposed, gate-stacked snapshot of M and W_h for the error products
  dType *d_M_grad_stack = nullptr, *d_W_h_grad_stack = nullptr, *d_b_grad_stack = nullptr;  // 4H x H, 4H x H, 4H
  dType *d_W_hi_grad = nullptr, *d_W_hf_grad = nullptr, *d_W_hc_grad = nullptr, *d_W_ho_grad = nullptr;
  dType *d_M_i_grad = nullptr, *d_M_f_grad = nullptr, *d_M_o_grad = nullptr, *d_M_c_grad = nullptr;
  dType *d_b_i_grad = nullptr, *d_b_f_grad = nullptr, *d_b_c_grad = nullptr, *d_b_o_grad = nullptr;
  // errors of the node being processed; d_d_ERRnTOt_h_Below sits directly behind d_d_ERRnTOt_htM1
  dType *d_d_ERRnTOt_htM1 = nullptr, *d_d_ERRnTOt_h_Below = nullptr, *d_d_ERRnTOt_ctM1 = nullptr;
  dType* d_d_ERRnTOt_gates = nullptr;  // 4H x minibatch: the reference's d_d_ERRnTOt_it, _ft, _tanhcpt, _ot stacked
  // feed-input (bottom target layer only; allocated by alloc_feed_training)
  dType* d_Q_grad_stack = nullptr;     // 4H x H
  dType *d_Q_i_grad = nullptr, *d_Q_f_grad = nullptr, *d_Q_c_grad = nullptr, *d_Q_o_grad = nullptr;
  dType* d_ERRnTOt_h_tild = nullptr;   // error of h~_{t-1} of the node being processed (first step: unused)
  dType *d_init_d_ERRnTOtp1_ht = nullptr, *d_init_d_ERRnTOtp1_ct = nullptr;  // zeros for the last time step
  dType learning_rate = 0.5f, norm_clip = 5;
  bool clip_gradients = true;
  lower_transfer_layer<dType> lower_layer;

  void alloc_training(zr_ctx* ctx, int H, int mb) {
    const size_t hh = (size_t)H * H, n = (size_t)H * mb;
    full_matrix_setup_0(ctx, &d_M_grad_stack, 4 * H, H);
    full_matrix_setup_0(ctx, &d_W_h_grad_stack, 4 * H, H);
    full_matrix_setup_0(ctx, &d_b_grad_stack, 4 * H, 1);
    dType** mats[] = {&d_W_hi_grad, &d_W_hf_grad, &d_W_hc_grad, &d_W_ho_grad, &d_M_i_grad, &d_M_f_grad, &d_M_c_grad, &d_M_o_grad};
    for (dType** m : mats) ZOPH_CALL(zr_malloc(ctx, hh * sizeof(dType), (void**)m));
    d_b_i_grad = d_b_grad_stack;
    d_b_f_grad = d_b_grad_stack + H;
    d_b_c_grad = d_b_grad_stack + 2 * (size_t)H;
    d_b_o_grad = d_b_grad_stack + 3 * (size_t)H;
    full_matrix_setup_0(ctx, &d_d_ERRnTOt_htM1, H, 2 * mb);
    d_d_ERRnTOt_h_Below = d_d_ERRnTOt_htM1 + n;
    full_matrix_setup_0(ctx, &d_d_ERRnTOt_ctM1, H, mb);
    full_matrix_setup_0(ctx, &d_d_ERRnTOt_gates, 4 * H, mb);
    full_matrix_setup_0(ctx, &d_init_d_ERRnTOtp1_ht, H, mb);
    full_matrix_setup_0(ctx, &d_init_d_ERRnTOtp1_ct, H, mb);
  }
  void alloc_feed_training(zr_ctx* ctx, int H, int mb) {
    full_matrix_setup_0(ctx, &d_Q_grad_stack, 4 * H, H);
    dType** mats[] = {&d_Q_i_grad, &d_Q_f_grad, &d_Q_c_grad, &d_Q_o_grad};
    for (dType** m : mats) ZOPH_CALL(zr_malloc(ctx, (size_t)H * H * sizeof(dType), (void**)m));
    full_matrix_setup_0(ctx, &d_ERRnTOt_h_tild, H, mb);
  }
  // the Q matrices' share of update_weights (src/Input_To_Hidden_Layer.hpp:690-790)
  void apply_feed_gradients(zr_ctx* ctx, int H, int mb, dType* const Q[4]) {
    const float scale = 1.0f / (float)mb, clip = clip_gradients ? (float)norm_clip : 0.0f;
    dType* gQ[4] = {d_Q_i_grad, d_Q_f_grad, d_Q_c_grad, d_Q_o_grad};
    ZOPH_CALL(zr_unstack_gates(ctx, d_Q_grad_stack, H, gQ));
    for (int g = 0; g < 4; g++) BZ_CUDA::apply_update(ctx, Q[g], gQ[g], (long long)H * H, scale, clip, (float)norm_clip, learning_rate);
  }
  // calculate_global_norm (src/Hidden_To_Hidden_Layer.hpp:241-335): the gate matrices' gradients are summed as the
  // stacks they are kept in
  void add_gradient_norms(zr_ctx* ctx, int H, int mb) {
    const float scale = 1.0f / (float)mb;
    const long long hh4 = 4LL * H * H;
    if (d_Q_grad_stack) BZ_CUDA::add_to_global_norm(ctx, d_Q_grad_stack, hh4, scale);
    BZ_CUDA::add_to_global_norm(ctx, d_M_grad_stack, hh4, scale);
    BZ_CUDA::add_to_global_norm(ctx, d_W_h_grad_stack, hh4, scale);
    BZ_CUDA::add_to_global_norm(ctx, d_b_grad_stack, 4LL * H, scale);
  }
  void zero_gradients(zr_ctx* ctx, int H) {
    if (d_Q_grad_stack) ZOPH_CALL(zr_memset_zero(ctx, d_Q_grad_stack, 4 * (size_t)H * H * sizeof(dType)));
    ZOPH_CALL(zr_memset_zero(ctx, d_M_grad_stack, 4 * (size_t)H * H * sizeof(dType)));
    ZOPH_CALL(zr_memset_zero(ctx, d_W_h_grad_stack, 4 * (size_t)H * H * sizeof(dType)));
    ZOPH_CALL(zr_memset_zero(ctx, d_b_grad_stack, 4 * (size_t)H * sizeof(dType)));
  }
  // scale_gradients + norm_clip_GPU_v2 per matrix + update_params (src/Hidden_To_Hidden_Layer.hpp:497-560): every
  // matrix and bias vector is scaled by 1 / minibatch_size, clipped on its own, and added
  void apply_gradients(zr_ctx* ctx, int H, int mb, dType* const M[4], dType* const Wh[4], dType* const b[4]) {
    const float scale = 1.0f / (float)mb, clip = clip_gradients ? (float)norm_clip : 0.0f;
    const long long hh = (long long)H * H;
    dType* gM[4] = {d_M_i_grad, d_M_f_grad, d_M_c_grad, d_M_o_grad};
    dType* gWh[4] = {d_W_hi_grad, d_W_hf_grad, d_W_hc_grad, d_W_ho_grad};
    dType* gb[4] = {d_b_i_grad, d_b_f_grad, d_b_c_grad, d_b_o_grad};
    ZOPH_CALL(zr_unstack_gates(ctx, d_M_grad_stack, H, gM));
    ZOPH_CALL(zr_unstack_gates(ctx, d_W_h_grad_stack, H, gWh));
    for (int g = 0; g < 4; g++) {
      BZ_CUDA::apply_update(ctx, M[g], gM[g], hh, scale, clip, (float)norm_clip, learning_rate);
      BZ_CUDA::apply_update(ctx, Wh[g], gWh[g], hh, scale, clip, (float)norm_clip, learning_rate);
      BZ_CUDA::apply_update(ctx, b[g], gb[g], H, scale, clip, (float)norm_clip, learning_rate);
    }
  }
};

template <typename dType>
class LSTM_HH_Node {  // src/LSTM_HH.h:19-102
 public:
  int minibatch_size, LSTM_size, index;
  bool attention_model = false;
  bool dropout;
  dType dropout_rate;
  Hidden_To_Hidden_Layer<dType>* model;
  dType *d_o_t = nullptr, *d_c_t = nullptr, *d_f_t = nullptr, *d_c_prime_t_tanh = nullptr, *d_i_t = nullptr,
        *d_h_t = nullptr;
  int* d_input_vocab_indices_01 = nullptr;
  dType *d_c_t_prev = nullptr, *d_h_t_prev = nullptr;
  dType* d_h_t_below = nullptr;
  dType* d_zeros = nullptr;
  // dropout (src/LSTM_HH.hpp:111-126): the node's input is a dropped-out copy of the state below.  The reference
  // always copies the state below into the node; here it is read in place unless dropout is on.
  dType *d_dropout_mask = nullptr, *d_h_t_below_drop = nullptr;
  dType* d_input = nullptr;  // what the step read: d_h_t_below or d_h_t_below_drop
  // errors arriving from step t+1 and from above (NULL: none); set by backprop_prep_GPU / the layer above
  dType *d_d_ERRnTOtp1_ht = nullptr, *d_d_ERRnTOtp1_ct = nullptr, *d_d_ERRt_ht = nullptr;

  LSTM_HH_Node(int LSTM_size, int minibatch_size, Hidden_To_Hidden_Layer<dType>* m, int index, dType* d_zeros,
               bool dropout, dType dropout_rate);
  void backprop_prep_GPU(dType* d_d_ERRnTOtp1_ht, dType* d_d_ERRnTOtp1_ct) {  // src/LSTM_HH.hpp:430-434
    this->d_d_ERRnTOtp1_ht = d_d_ERRnTOtp1_ht;
    this->d_d_ERRnTOtp1_ct = d_d_ERRnTOtp1_ct;
  }
  void back_prop_GPU(int index);     // src/LSTM_HH.hpp:452-700
  void compute_gradients_GPU();      // src/LSTM_HH.hpp:700-900
  void update_vectors_forward_GPU(int* d_input_vocab_indices_01, dType* d_h_t_prev, dType* d_c_t_prev) {
    this->d_h_t_prev = d_h_t_prev;
    this->d_c_t_prev = d_c_t_prev;
    this->d_input_vocab_indices_01 = d_input_vocab_indices_01;
  }
  void update_vectors_forward_decoder(int* d_input_vocab_indices_01) {
    this->d_input_vocab_indices_01 = d_input_vocab_indices_01;
  }
  void forward_prop() { forward_prop_GPU(); }
  void forward_prop_GPU();
  void send_h_t_above();
};

template <typename dType>
class LSTM_IH_Node {  // src/LSTM.h:19-106
 public:
  int minibatch_size, LSTM_size, index;
  bool dropout;
  dType dropout_rate;
  bool attention_model = false;
  bool feed_input = false;
  Input_To_Hidden_Layer<dType>* model;
  dType *d_o_t = nullptr, *d_c_t = nullptr, *d_f_t = nullptr, *d_c_prime_t_tanh = nullptr, *d_i_t = nullptr,
        *d_h_t = nullptr, *d_sparse_lookup = nullptr;
  int *d_input_vocab_indices = nullptr, *d_input_vocab_indices_01 = nullptr;
  dType *d_c_t_prev = nullptr, *d_h_t_prev = nullptr;
  dType* d_zeros = nullptr;
  dType* d_h_tild = nullptr;
  dType* d_dropout_mask = nullptr;            // src/LSTM.hpp:39-41, :112-119
  dType* d_ERRnTOt_h_tild_cpy = nullptr;      // where the error of h~_{t-1} goes: attention node t-1's d_ERRtTOn_htild_below
  dType *d_d_ERRnTOtp1_ht = nullptr, *d_d_ERRnTOtp1_ct = nullptr, *d_d_ERRt_ht = nullptr;

  LSTM_IH_Node(int LSTM_size, int minibatch_size, int vocab_size, Input_To_Hidden_Layer<dType>* m, int index,
               dType* d_zeros, bool dropout, dType dropout_rate);
  void backprop_prep_GPU(dType* d_d_ERRnTOtp1_ht, dType* d_d_ERRnTOtp1_ct) {  // src/LSTM.hpp:523-530
    this->d_d_ERRnTOtp1_ht = d_d_ERRnTOtp1_ht;
    this->d_d_ERRnTOtp1_ct = d_d_ERRnTOtp1_ct;
  }
  void back_prop_GPU(int index);     // src/LSTM.hpp:542-960
  void compute_gradients_GPU();      // src/LSTM.hpp:963-1270
  void update_vectors_forward_GPU(int* d_input_vocab_indices, int* d_input_vocab_indices_01, dType* d_h_t_prev,
                                  dType* d_c_t_prev) {
    this->d_h_t_prev = d_h_t_prev;
    this->d_c_t_prev = d_c_t_prev;
    this->d_input_vocab_indices = d_input_vocab_indices;
    this->d_input_vocab_indices_01 = d_input_vocab_indices_01;
  }
  void update_vectors_forward_decoder(int* d_input_vocab_indices, int* d_input_vocab_indices_01) {
    this->d_input_vocab_indices = d_input_vocab_indices;
    this->d_input_vocab_indices_01 = d_input_vocab_indices_01;
  }
  void forward_prop() { forward_prop_GPU(); }
  void forward_prop_GPU();
  void attention_extra();  // src/LSTM.hpp:533-539
  void send_h_t_above();
};

// Device copy of a host index vector for swap_states_decoding: the reference hands over an Eigen vector
// (const Eigen::MatrixBase<Derived>&, src/Input_To_Hidden_Layer.h:345); anything indexable with (i) or [i] that holds
// minibatch_size entries is accepted here.
namespace zoph_detail {
template <typename V>
auto index_at(const V& v, int i, int) -> decltype((int)v(i)) { return (int)v(i); }
template <typename V>
auto index_at(const V& v, int i, long) -> decltype((int)v[i]) { return (int)v[i]; }
template <typename V>
inline int* upload_indices(zr_ctx* ctx, const V& indicies, int n, int** d_cache) {
  std::vector<int> h((size_t)n);
  for (int i = 0; i < n; i++) h[(size_t)i] = index_at(indicies, i, 0);
  if (!*d_cache) ZOPH_CALL(zr_malloc(ctx, (size_t)n * sizeof(int), (void**)d_cache));
  ZOPH_CALL(zr_h2d(ctx, *d_cache, h.data(), (size_t)n * sizeof(int)));
  return *d_cache;
}
}  // namespace zoph_detail

// ------------------------------------------------------------------------------------------------ layers
template <typename dType>
class Hidden_To_Hidden_Layer : public lstm_layer_training<dType> {  // src/Hidden_To_Hidden_Layer.h:12-313
 public:
  layer_gpu_info hh_layer_info;
  std::vector<LSTM_HH_Node<dType>> nodes;
  dType *d_W_hi = nullptr, *d_W_hf = nullptr, *d_W_hc = nullptr, *d_W_ho = nullptr;
  dType *d_b_i = nullptr, *d_b_f = nullptr, *d_b_c = nullptr, *d_b_o = nullptr;
  dType *d_M_i = nullptr, *d_M_f = nullptr, *d_M_o = nullptr, *d_M_c = nullptr;
  dType *d_init_hidden_vector = nullptr, *d_init_cell_vector = nullptr, *d_zeros = nullptr;
  int *d_input_vocab_indices_01_full = nullptr, *d_input_vocab_indices_full = nullptr;
  int LSTM_size = 0, minibatch_size = 0, longest_sent = 0, layer_number = -1;
  neuralMT_model<precision>* model = nullptr;
  upper_transfer_layer<dType> upper_layer;
  attention_layer<dType>* attent_layer = nullptr;
  zr_lstm_weights* packed = nullptr;  // repacked lazily after init / load_weights

  // src/Hidden_To_Hidden_Layer.hpp:125-155 (and :4-112 for the device side)
  void init_Hidden_To_Hidden_Layer(int LSTM_size, int minibatch_size, int longest_sent, bool /*debug_temp*/,
                                   dType learning_rate, bool clip_gradients, dType norm_clip,
                                   struct neuralMT_model<precision>* model, int /*seed*/, bool dropout,
                                   dType dropout_rate, bool /*bi_dir*/, int layer_number) {
    this->learning_rate = learning_rate;
    this->clip_gradients = clip_gradients;
    this->norm_clip = norm_clip;
    this->LSTM_size = LSTM_size;
    this->minibatch_size = minibatch_size;
    this->longest_sent = longest_sent;
    this->model = model;
    this->layer_number = layer_number;
    zr_ctx* ctx = hh_layer_info.ctx;
    dType* h = nullptr;
    dType** mats[] = {&d_W_hi, &d_W_hf, &d_W_hc, &d_W_ho, &d_M_i, &d_M_f, &d_M_o, &d_M_c};
    for (dType** m : mats) full_matrix_setup(ctx, &h, m, LSTM_size, LSTM_size);
    dType** vecs[] = {&d_b_i, &d_b_f, &d_b_c, &d_b_o};
    for (dType** v : vecs) full_matrix_setup(ctx, &h, v, LSTM_size, 1);
    device_fill(ctx, d_b_f, LSTM_size, (dType)1);  // forget bias 1 (:31-34)
    full_matrix_setup_0(ctx, &d_init_hidden_vector, LSTM_size, minibatch_size);
    full_matrix_setup_0(ctx, &d_init_cell_vector, LSTM_size, minibatch_size);
    full_matrix_setup_0(ctx, &d_zeros, LSTM_size, minibatch_size);
    const size_t nt = (size_t)minibatch_size * longest_sent;
    ZOPH_CALL(zr_malloc(ctx, nt * sizeof(int), (void**)&d_input_vocab_indices_full));
    ZOPH_CALL(zr_malloc(ctx, nt * sizeof(int), (void**)&d_input_vocab_indices_01_full));
    for (int i = 0; i < longest_sent; i++)
      nodes.push_back(LSTM_HH_Node<dType>(LSTM_size, minibatch_size, this, i, d_zeros, dropout, dropout_rate));
  }
  void repack() {
    zr_ctx* ctx = hh_layer_info.ctx;
    if (packed) ZOPH_CALL(zr_lstm_weights_destroy(ctx, packed));
    const dType* M[4] = {d_M_i, d_M_f, d_M_c, d_M_o};
    const dType* Wh[4] = {d_W_hi, d_W_hf, d_W_hc, d_W_ho};
    const dType* b[4] = {d_b_i, d_b_f, d_b_c, d_b_o};
    if (BZ_CUDA::bf16_weights)
      ZOPH_CALL(zr_lstm_pack_weights_bf16(ctx, M, Wh, nullptr, b, LSTM_size, &packed));
    else
      ZOPH_CALL(zr_lstm_pack_weights(ctx, M, Wh, nullptr, b, LSTM_size, &packed));
  }
  // ---- training.  clear_gradients(true) allocates the training buffers (src/Hidden_To_Hidden_Layer.hpp:158-232
  // allocates them in the init call) and zeroes; clear_gradients(false) zeroes (:283-316).
  void clear_gradients(bool init) {
    zr_ctx* ctx = hh_layer_info.ctx;
    if (init || !this->train_weights) {
      if (!this->train_weights) {
        this->alloc_training(ctx, LSTM_size, minibatch_size);
        const dType* M[4] = {d_M_i, d_M_f, d_M_c, d_M_o};
        const dType* Wh[4] = {d_W_hi, d_W_hf, d_W_hc, d_W_ho};
        ZOPH_CALL(zr_lstm_train_create(ctx, M, Wh, LSTM_size, &this->train_weights));
      }
    }
    this->zero_gradients(ctx, LSTM_size);
  }
  void clear_gradients_GPU(bool init) { clear_gradients(init); }
  void calculate_global_norm() { this->add_gradient_norms(hh_layer_info.ctx, LSTM_size, minibatch_size); }
  void update_global_params() { update_weights(); }  // src/Hidden_To_Hidden_Layer.hpp:353-382
  // src/Hidden_To_Hidden_Layer.hpp:497-560, then the snapshots the kernels read are rebuilt
  void update_weights() {
    zr_ctx* ctx = hh_layer_info.ctx;
    dType* M[4] = {d_M_i, d_M_f, d_M_c, d_M_o};
    dType* Wh[4] = {d_W_hi, d_W_hf, d_W_hc, d_W_ho};
    dType* b[4] = {d_b_i, d_b_f, d_b_c, d_b_o};
    this->apply_gradients(ctx, LSTM_size, minibatch_size, M, Wh, b);
    repack();
    ZOPH_CALL(zr_lstm_train_refresh(ctx, this->train_weights, M, Wh));
  }
  void update_weights_GPU() { update_weights(); }
  void update_learning_rate(dType lr) { this->learning_rate = lr; }
  // src/Hidden_To_Hidden_Layer.hpp:748-774
  void prep_GPU_vocab_indices(int* h_input_vocab_indicies, int current_length) {
    zr_ctx* ctx = hh_layer_info.ctx;
    const int n = minibatch_size * current_length;
    ZOPH_CALL(zr_h2d(ctx, d_input_vocab_indices_full, h_input_vocab_indicies, (size_t)n * sizeof(int)));
    ZOPH_CALL(zr_vocab_prep(ctx, d_input_vocab_indices_full, n, 0, nullptr, d_input_vocab_indices_01_full));
  }
  // model-file order (src/Hidden_To_Hidden_Layer.hpp:669-692)
  void dump_weights(std::ofstream& output) {
    zr_ctx* ctx = hh_layer_info.ctx;
    write_matrix_GPU(ctx, d_W_hi, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_b_i, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_W_hf, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_b_f, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_W_hc, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_b_c, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_W_ho, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_b_o, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_M_i, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_M_f, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_M_o, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_M_c, LSTM_size, LSTM_size, output);
    if (attent_layer) attent_layer->dump_weights(output);
  }
  void load_weights(std::ifstream& input) {
    zr_ctx* ctx = hh_layer_info.ctx;
    read_matrix_GPU(ctx, d_W_hi, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_b_i, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_W_hf, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_b_f, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_W_hc, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_b_c, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_W_ho, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_b_o, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_M_i, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_M_f, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_M_o, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_M_c, LSTM_size, LSTM_size, input);
    if (attent_layer) attent_layer->load_weights(input);
    repack();
  }
  // src/Hidden_To_Hidden_Layer.hpp:780-791: reorder the columns of node 0's h and c by the beam back-pointers
  void swap_states_decoding(const int* d_indicies, int /*index*/, dType* d_temp_swap_vals) {
    zr_ctx* ctx = hh_layer_info.ctx;
    const size_t bytes = (size_t)LSTM_size * minibatch_size * sizeof(dType);
    ZOPH_CALL(zr_gather_columns(ctx, nodes[0].d_h_t, LSTM_size, d_indicies, minibatch_size, d_temp_swap_vals));
    ZOPH_CALL(zr_d2d(ctx, nodes[0].d_h_t, d_temp_swap_vals, bytes));
    ZOPH_CALL(zr_gather_columns(ctx, nodes[0].d_c_t, LSTM_size, d_indicies, minibatch_size, d_temp_swap_vals));
    ZOPH_CALL(zr_d2d(ctx, nodes[0].d_c_t, d_temp_swap_vals, bytes));
  }
  // src/Hidden_To_Hidden_Layer.hpp:801-813: one source column replicated over the beam
  void transfer_decoding_states_GPU(dType* d_h_t, dType* d_c_t) {
    zr_ctx* ctx = hh_layer_info.ctx;
    ZOPH_CALL(zr_broadcast_column(ctx, d_h_t, LSTM_size, minibatch_size, d_init_hidden_vector));
    ZOPH_CALL(zr_broadcast_column(ctx, d_c_t, LSTM_size, minibatch_size, d_init_cell_vector));
    nodes[0].d_h_t_prev = d_init_hidden_vector;
    nodes[0].d_c_t_prev = d_init_cell_vector;
  }
  // the reference's own parameter list (src/Hidden_To_Hidden_Layer.h:282): a host-side index vector
  int* d_swap_indices = nullptr;
  template <typename IndexVector>
  void swap_states_decoding(const IndexVector& indicies, int index, dType* d_temp_swap_vals) {
    swap_states_decoding((const int*)zoph_detail::upload_indices(hh_layer_info.ctx, indicies, minibatch_size, &d_swap_indices),
                         index, d_temp_swap_vals);
  }
  // src/Hidden_To_Hidden_Layer.hpp (init_attention): the top target layer owns the attention layer
  void init_attention(attention_layer<dType>* layer) {
    attent_layer = layer;
    for (size_t i = 0; i < nodes.size(); i++) {
      nodes[i].attention_model = true;
      attent_layer->nodes[i].d_indicies_mask = &nodes[i].d_input_vocab_indices_01;
      attent_layer->nodes[i].d_h_t = nodes[i].d_h_t;
    }
  }
  // The reference's own parameter list (src/Hidden_To_Hidden_Layer.h:290, body src/Hidden_To_Hidden_Layer.hpp:160-186):
  // the layer builds its attention layer itself, from the model's source states (model->source_top_h_t).
  void init_attention(int device_number, int D, bool feed_input, neuralMT_model<dType>* model, global_params& params) {
    cublasHandle_t handle = hh_layer_info.ctx;
    init_attention(new attention_layer<dType>(LSTM_size, minibatch_size, device_number, D, longest_sent, handle, model,
                                              feed_input, this->clip_gradients, this->norm_clip, params.dropout,
                                              params.dropout_rate, params, false));
  }
};

template <typename dType>
class Input_To_Hidden_Layer : public lstm_layer_training<dType> {  // src/Input_To_Hidden_Layer.h:11-368
 public:
  layer_gpu_info ih_layer_info;
  std::vector<LSTM_IH_Node<dType>> nodes;
  dType* d_W = nullptr;  // embedding, LSTM_size x input_vocab_size
  dType *d_W_hi = nullptr, *d_W_hf = nullptr, *d_W_hc = nullptr, *d_W_ho = nullptr;
  dType *d_b_i = nullptr, *d_b_f = nullptr, *d_b_c = nullptr, *d_b_o = nullptr;
  dType *d_M_i = nullptr, *d_M_f = nullptr, *d_M_o = nullptr, *d_M_c = nullptr;
  dType *d_Q_i = nullptr, *d_Q_f = nullptr, *d_Q_o = nullptr, *d_Q_c = nullptr;
  dType *d_init_hidden_vector = nullptr, *d_init_cell_vector = nullptr, *d_zeros = nullptr;
  int *d_input_vocab_indices_full = nullptr, *d_input_vocab_indices_01_full = nullptr;
  int LSTM_size = 0, minibatch_size = 0, input_vocab_size = 0, longest_sent = 0;
  bool feed_input = false;
  neuralMT_model<precision>* model = nullptr;
  upper_transfer_layer<dType> upper_layer;
  attention_layer<dType>* attent_layer = nullptr;
  zr_lstm_weights* packed = nullptr;

  // src/Input_To_Hidden_Layer.hpp:171-202 (and :3-159 for the device side)
  void init_Input_To_Hidden_Layer(int LSTM_size, int minibatch_size, int vocab_size, int longest_sent,
                                  bool /*debug_temp*/, dType learning_rate, bool clip_gradients,
                                  dType norm_clip, struct neuralMT_model<precision>* model, int /*seed*/,
                                  bool dropout, dType dropout_rate, bool /*is_bi_dir*/, bool share_embeddings,
                                  dType* d_embedding_ptr, bool /*combine_embeddings*/, global_params& /*params*/,
                                  bool /*source*/) {
    this->learning_rate = learning_rate;
    this->clip_gradients = clip_gradients;
    this->norm_clip = norm_clip;
    this->LSTM_size = LSTM_size;
    this->minibatch_size = minibatch_size;
    this->input_vocab_size = vocab_size;
    this->longest_sent = longest_sent;
    this->model = model;
    zr_ctx* ctx = ih_layer_info.ctx;
    dType* h = nullptr;
    dType** mats[] = {&d_W_hi, &d_W_hf, &d_W_hc, &d_W_ho, &d_M_i, &d_M_f, &d_M_o, &d_M_c};
    for (dType** m : mats) full_matrix_setup(ctx, &h, m, LSTM_size, LSTM_size);
    dType** vecs[] = {&d_b_i, &d_b_f, &d_b_c, &d_b_o};
    for (dType** v : vecs) full_matrix_setup(ctx, &h, v, LSTM_size, 1);
    device_fill(ctx, d_b_f, LSTM_size, (dType)1);  // forget bias 1 (:33-36)
    if (share_embeddings)
      d_W = d_embedding_ptr;
    else
      full_matrix_setup(ctx, &h, &d_W, LSTM_size, vocab_size);
    full_matrix_setup_0(ctx, &d_init_hidden_vector, LSTM_size, minibatch_size);
    full_matrix_setup_0(ctx, &d_init_cell_vector, LSTM_size, minibatch_size);
    full_matrix_setup_0(ctx, &d_zeros, LSTM_size, minibatch_size);
    const size_t nt = (size_t)minibatch_size * longest_sent;
    ZOPH_CALL(zr_malloc(ctx, nt * sizeof(int), (void**)&d_input_vocab_indices_full));
    ZOPH_CALL(zr_malloc(ctx, nt * sizeof(int), (void**)&d_input_vocab_indices_01_full));
    for (int i = 0; i < longest_sent; i++)
      nodes.push_back(LSTM_IH_Node<dType>(LSTM_size, minibatch_size, vocab_size, this, i, d_zeros, dropout, dropout_rate));
  }
  void repack() {
    zr_ctx* ctx = ih_layer_info.ctx;
    if (packed) ZOPH_CALL(zr_lstm_weights_destroy(ctx, packed));
    const dType* M[4] = {d_M_i, d_M_f, d_M_c, d_M_o};
    const dType* Wh[4] = {d_W_hi, d_W_hf, d_W_hc, d_W_ho};
    const dType* Q[4] = {d_Q_i, d_Q_f, d_Q_c, d_Q_o};
    const dType* b[4] = {d_b_i, d_b_f, d_b_c, d_b_o};
    if (BZ_CUDA::bf16_weights)
      ZOPH_CALL(zr_lstm_pack_weights_bf16(ctx, M, Wh, feed_input ? Q : nullptr, b, LSTM_size, &packed));
    else
      ZOPH_CALL(zr_lstm_pack_weights(ctx, M, Wh, feed_input ? Q : nullptr, b, LSTM_size, &packed));
  }
  // ---- training: as in Hidden_To_Hidden_Layer plus the embedding gradient d_W_grad (dense LSTM_size x vocabulary;
  // the reference keeps the same matrix and touches only the minibatch's columns, src/custom_kernels.h:1346-1368)
  dType* d_W_grad = nullptr;
  void clear_gradients(bool init) {
    zr_ctx* ctx = ih_layer_info.ctx;
    if (init || !this->train_weights) {
      if (!this->train_weights) {
        this->alloc_training(ctx, LSTM_size, minibatch_size);
        full_matrix_setup_0(ctx, &d_W_grad, LSTM_size, input_vocab_size);
        if (feed_input) this->alloc_feed_training(ctx, LSTM_size, minibatch_size);
        const dType* M[4] = {d_M_i, d_M_f, d_M_c, d_M_o};
        const dType* Wh[4] = {d_W_hi, d_W_hf, d_W_hc, d_W_ho};
        ZOPH_CALL(zr_lstm_train_create(ctx, M, Wh, LSTM_size, &this->train_weights));
      }
    }
    this->zero_gradients(ctx, LSTM_size);
    ZOPH_CALL(zr_memset_zero(ctx, d_W_grad, (size_t)LSTM_size * input_vocab_size * sizeof(dType)));
  }
  void clear_gradients_GPU(bool init) { clear_gradients(init); }
  void calculate_global_norm() {  // src/Input_To_Hidden_Layer.hpp calculate_global_norm (norm_clip_W_GPU_v2_p1 for W)
    zr_ctx* ctx = ih_layer_info.ctx;
    BZ_CUDA::add_to_global_norm(ctx, d_W_grad, (long long)LSTM_size * input_vocab_size, 1.0f / (float)minibatch_size);
    this->add_gradient_norms(ctx, LSTM_size, minibatch_size);
  }
  void update_global_params() { update_weights(); }
  void update_weights() {  // src/Input_To_Hidden_Layer.hpp:690-790
    zr_ctx* ctx = ih_layer_info.ctx;
    dType* M[4] = {d_M_i, d_M_f, d_M_c, d_M_o};
    dType* Wh[4] = {d_W_hi, d_W_hf, d_W_hc, d_W_ho};
    dType* b[4] = {d_b_i, d_b_f, d_b_c, d_b_o};
    BZ_CUDA::apply_update(ctx, d_W, d_W_grad, (long long)LSTM_size * input_vocab_size, 1.0f / (float)minibatch_size,
                          this->clip_gradients ? (float)this->norm_clip : 0.0f, (float)this->norm_clip, this->learning_rate);
    this->apply_gradients(ctx, LSTM_size, minibatch_size, M, Wh, b);
    if (feed_input && this->d_Q_grad_stack) {
      dType* Q[4] = {d_Q_i, d_Q_f, d_Q_c, d_Q_o};
      this->apply_feed_gradients(ctx, LSTM_size, minibatch_size, Q);
    }
    repack();
    ZOPH_CALL(zr_lstm_train_refresh(ctx, this->train_weights, M, Wh));
  }
  void update_weights_GPU() { update_weights(); }
  void update_learning_rate(dType lr) { this->learning_rate = lr; }
  // src/Input_To_Hidden_Layer.hpp:1178-1225 (the *_Wgrad arguments serve the embedding gradient only)
  void prep_GPU_vocab_indices(int* h_input_vocab_indicies, int* /*h_input_vocab_indicies_Wgrad*/, int current_length,
                              int /*len_W*/) {
    zr_ctx* ctx = ih_layer_info.ctx;
    const int n = minibatch_size * current_length;
    ZOPH_CALL(zr_h2d(ctx, d_input_vocab_indices_full, h_input_vocab_indicies, (size_t)n * sizeof(int)));
    // mask first, then -1 -> 0 in place (vocab_to_01 then vocab_to_nonM1, :1199-1202)
    ZOPH_CALL(zr_vocab_prep(ctx, d_input_vocab_indices_full, n, input_vocab_size, d_input_vocab_indices_full,
                            d_input_vocab_indices_01_full));
  }
  // src/Input_To_Hidden_Layer.hpp:242-317: Q matrices and per-node d_h_tild; attention node i feeds node i+1
  void init_feed_input(Hidden_To_Hidden_Layer<dType>* hidden_layer, bool /*multi_attention*/) {
    zr_ctx* ctx = ih_layer_info.ctx;
    feed_input = true;
    dType* h = nullptr;
    dType** mats[] = {&d_Q_i, &d_Q_f, &d_Q_o, &d_Q_c};
    for (dType** m : mats) full_matrix_setup(ctx, &h, m, LSTM_size, LSTM_size);
    attention_layer<dType>* att = hidden_layer ? hidden_layer->attent_layer : attent_layer;
    for (size_t i = 0; i < nodes.size(); i++) nodes[i].attention_extra();
    if (att)
      for (size_t i = 0; i + 1 < nodes.size(); i++) {
        att->nodes[i].feed_input_init(nodes[i + 1].d_h_tild);
        nodes[i + 1].d_ERRnTOt_h_tild_cpy = att->nodes[i].d_ERRtTOn_htild_below;  // :253, :272
      }
    repack();
  }
  void decoder_init_feed_input() {  // :300-317: decode keeps a single node; h~ is copied in by the driver
    zr_ctx* ctx = ih_layer_info.ctx;
    feed_input = true;
    dType* h = nullptr;
    dType** mats[] = {&d_Q_i, &d_Q_f, &d_Q_o, &d_Q_c};
    for (dType** m : mats) full_matrix_setup(ctx, &h, m, LSTM_size, LSTM_size);
    nodes[0].attention_extra();
    repack();
  }
  void init_attention(attention_layer<dType>* layer) {
    attent_layer = layer;
    for (size_t i = 0; i < nodes.size(); i++) {
      nodes[i].attention_model = true;
      attent_layer->nodes[i].d_indicies_mask = &nodes[i].d_input_vocab_indices_01;
      attent_layer->nodes[i].d_h_t = nodes[i].d_h_t;
    }
  }
  // The reference's own parameter list (src/Input_To_Hidden_Layer.h:353, body src/Input_To_Hidden_Layer.hpp:230-260):
  // the layer builds its attention layer itself, from the model's source states (model->source_top_h_t).
  void init_attention(int device_number, int D, bool feed_input, neuralMT_model<dType>* model, global_params& params) {
    cublasHandle_t handle = ih_layer_info.ctx;
    init_attention(new attention_layer<dType>(LSTM_size, minibatch_size, device_number, D, longest_sent, handle, model,
                                              feed_input, this->clip_gradients, this->norm_clip, params.dropout,
                                              params.dropout_rate, params, false));
  }
  // the reference's own parameter list (src/Input_To_Hidden_Layer.h:345): a host-side index vector
  int* d_swap_indices = nullptr;
  template <typename IndexVector>
  void swap_states_decoding(const IndexVector& indicies, int index, dType* d_temp_swap_vals) {
    swap_states_decoding((const int*)zoph_detail::upload_indices(ih_layer_info.ctx, indicies, minibatch_size, &d_swap_indices),
                         index, d_temp_swap_vals);
  }
  // model-file order (src/Input_To_Hidden_Layer.hpp:1050-1159)
  void dump_weights(std::ofstream& output) {
    zr_ctx* ctx = ih_layer_info.ctx;
    write_matrix_GPU(ctx, d_W_hi, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_b_i, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_W_hf, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_b_f, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_W_hc, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_b_c, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_W_ho, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_b_o, LSTM_size, 1, output);
    write_matrix_GPU(ctx, d_W, LSTM_size, input_vocab_size, output);
    write_matrix_GPU(ctx, d_M_i, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_M_f, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_M_o, LSTM_size, LSTM_size, output);
    write_matrix_GPU(ctx, d_M_c, LSTM_size, LSTM_size, output);
    if (feed_input) {
      write_matrix_GPU(ctx, d_Q_i, LSTM_size, LSTM_size, output);
      write_matrix_GPU(ctx, d_Q_f, LSTM_size, LSTM_size, output);
      write_matrix_GPU(ctx, d_Q_o, LSTM_size, LSTM_size, output);
      write_matrix_GPU(ctx, d_Q_c, LSTM_size, LSTM_size, output);
    }
    if (attent_layer) attent_layer->dump_weights(output);
  }
  void load_weights(std::ifstream& input) {
    zr_ctx* ctx = ih_layer_info.ctx;
    read_matrix_GPU(ctx, d_W_hi, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_b_i, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_W_hf, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_b_f, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_W_hc, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_b_c, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_W_ho, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_b_o, LSTM_size, 1, input);
    read_matrix_GPU(ctx, d_W, LSTM_size, input_vocab_size, input);
    read_matrix_GPU(ctx, d_M_i, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_M_f, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_M_o, LSTM_size, LSTM_size, input);
    read_matrix_GPU(ctx, d_M_c, LSTM_size, LSTM_size, input);
    if (feed_input) {
      read_matrix_GPU(ctx, d_Q_i, LSTM_size, LSTM_size, input);
      read_matrix_GPU(ctx, d_Q_f, LSTM_size, LSTM_size, input);
      read_matrix_GPU(ctx, d_Q_o, LSTM_size, LSTM_size, input);
      read_matrix_GPU(ctx, d_Q_c, LSTM_size, LSTM_size, input);
    }
    if (attent_layer) attent_layer->load_weights(input);
    repack();
  }
  // src/Input_To_Hidden_Layer.hpp:1231-1242
  void swap_states_decoding(const int* d_indicies, int /*index*/, dType* d_temp_swap_vals) {
    zr_ctx* ctx = ih_layer_info.ctx;
    const size_t bytes = (size_t)LSTM_size * minibatch_size * sizeof(dType);
    ZOPH_CALL(zr_gather_columns(ctx, nodes[0].d_h_t, LSTM_size, d_indicies, minibatch_size, d_temp_swap_vals));
    ZOPH_CALL(zr_d2d(ctx, nodes[0].d_h_t, d_temp_swap_vals, bytes));
    ZOPH_CALL(zr_gather_columns(ctx, nodes[0].d_c_t, LSTM_size, d_indicies, minibatch_size, d_temp_swap_vals));
    ZOPH_CALL(zr_d2d(ctx, nodes[0].d_c_t, d_temp_swap_vals, bytes));
  }
  // src/Input_To_Hidden_Layer.hpp:1252-1266
  void transfer_decoding_states_GPU(dType* d_h_t, dType* d_c_t) {
    zr_ctx* ctx = ih_layer_info.ctx;
    ZOPH_CALL(zr_broadcast_column(ctx, d_h_t, LSTM_size, minibatch_size, d_init_hidden_vector));
    ZOPH_CALL(zr_broadcast_column(ctx, d_c_t, LSTM_size, minibatch_size, d_init_cell_vector));
    nodes[0].d_h_t_prev = d_init_hidden_vector;
    nodes[0].d_c_t_prev = d_init_cell_vector;
  }
};

// ------------------------------------------------------------------------------------------------ node bodies
template <typename dType>
LSTM_HH_Node<dType>::LSTM_HH_Node(int LSTM_size, int minibatch_size, Hidden_To_Hidden_Layer<dType>* m, int index,
                                  dType* d_zeros, bool dropout, dType dropout_rate) {
  model = m;
  this->dropout = dropout;
  this->dropout_rate = dropout_rate;
  this->minibatch_size = minibatch_size;
  this->LSTM_size = LSTM_size;
  this->index = index;
  this->d_zeros = d_zeros;
  zr_ctx* ctx = m->hh_layer_info.ctx;
  dType** bufs[] = {&d_o_t, &d_c_t, &d_f_t, &d_c_prime_t_tanh, &d_i_t, &d_h_t};  // init_LSTM_GPU, src/LSTM_HH.hpp:21-39
  for (dType** b : bufs) full_matrix_setup_0(ctx, b, LSTM_size, minibatch_size);
}

template <typename dType>
void LSTM_HH_Node<dType>::forward_prop_GPU() {  // src/LSTM_HH.hpp:103-333
  zr_ctx* ctx = model->hh_layer_info.ctx;
  if (!model->packed) model->repack();
  dType* gates[4] = {d_i_t, d_f_t, d_c_prime_t_tanh, d_o_t};
  d_input = d_h_t_below;
  if (dropout && model->model && model->model->train) {  // src/LSTM_HH.hpp:111-126
    const size_t n = (size_t)LSTM_size * minibatch_size;
    if (!d_dropout_mask) {
      ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&d_dropout_mask));
      ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&d_h_t_below_drop));
    }
    if (!model->model->grad_check_flag) {
      const int stream = (model->upper_layer.source_side ? BZ_CUDA::DROPOUT_STREAM_SOURCE_HIDDEN
                                                         : BZ_CUDA::DROPOUT_STREAM_TARGET_HIDDEN) + model->layer_number;
      ZOPH_CALL(zr_uniform_fill(ctx, BZ_CUDA::dropout_seed + BZ_CUDA::dropout_minibatch,
                                BZ_CUDA::dropout_call(stream, index), d_dropout_mask, (long long)n));
    }
    ZOPH_CALL(zr_d2d(ctx, d_h_t_below_drop, d_h_t_below, n * sizeof(dType)));
    ZOPH_CALL(zr_dropout_apply(ctx, d_dropout_mask, dropout_rate, d_h_t_below_drop, (long long)n));
    d_input = d_h_t_below_drop;
  }
  ZOPH_CALL(zr_lstm_step(ctx, model->packed, d_input, d_h_t_prev, d_c_t_prev, nullptr, d_input_vocab_indices_01,
                         BZ_CUDA::clip_cell ? BZ_CUDA::cell_clip_threshold : 0.0f, minibatch_size, d_h_t, d_c_t, gates));
  send_h_t_above();
}

template <typename dType>
void LSTM_HH_Node<dType>::send_h_t_above() {  // src/LSTM_HH.hpp:337-423, pointer-passing branch
  int idx = (model->model && model->model->decode) ? 0 : index;
  dType* out = d_h_t;
  if (attention_model && model->attent_layer) {
    model->attent_layer->nodes[idx].d_h_t = d_h_t;
    model->attent_layer->nodes[idx].forward_prop();
    out = model->attent_layer->nodes[idx].d_final_temp_2;
  }
  if (model->upper_layer.upper_softmax) {
    if (!model->upper_layer.source_side && model->upper_layer.softmax) model->upper_layer.softmax->set_ht_ptr(idx, out);
  } else if (model->upper_layer.hidden_layer) {
    model->upper_layer.hidden_layer->nodes[idx].d_h_t_below = out;
  }
}

template <typename dType>
LSTM_IH_Node<dType>::LSTM_IH_Node(int LSTM_size, int minibatch_size, int /*vocab_size*/,
                                  Input_To_Hidden_Layer<dType>* m, int index, dType* d_zeros, bool dropout,
                                  dType dropout_rate) {
  model = m;
  this->dropout = dropout;
  this->dropout_rate = dropout_rate;
  this->minibatch_size = minibatch_size;
  this->LSTM_size = LSTM_size;
  this->index = index;
  this->d_zeros = d_zeros;
  zr_ctx* ctx = m->ih_layer_info.ctx;
  dType** bufs[] = {&d_o_t, &d_c_t, &d_f_t, &d_c_prime_t_tanh, &d_i_t, &d_sparse_lookup, &d_h_t};  // src/LSTM.hpp:23-42
  for (dType** b : bufs) full_matrix_setup_0(ctx, b, LSTM_size, minibatch_size);
}

template <typename dType>
void LSTM_IH_Node<dType>::attention_extra() {
  full_matrix_setup_0(model->ih_layer_info.ctx, &d_h_tild, LSTM_size, minibatch_size);
  feed_input = true;
}

template <typename dType>
void LSTM_IH_Node<dType>::forward_prop_GPU() {  // src/LSTM.hpp:76-421
  zr_ctx* ctx = model->ih_layer_info.ctx;
  if (!model->packed) model->repack();
  ZOPH_CALL(zr_embed_gather(ctx, model->d_W, LSTM_size, model->input_vocab_size, d_input_vocab_indices, minibatch_size,
                            d_sparse_lookup));
  if (dropout && model->model && model->model->train) {  // src/LSTM.hpp:112-119
    const size_t n = (size_t)LSTM_size * minibatch_size;
    if (!d_dropout_mask) ZOPH_CALL(zr_malloc(ctx, n * sizeof(dType), (void**)&d_dropout_mask));
    if (!model->model->grad_check_flag) {
      const int stream = model->upper_layer.source_side ? BZ_CUDA::DROPOUT_STREAM_SOURCE_INPUT
                                                        : BZ_CUDA::DROPOUT_STREAM_TARGET_INPUT;
      ZOPH_CALL(zr_uniform_fill(ctx, BZ_CUDA::dropout_seed + BZ_CUDA::dropout_minibatch,
                                BZ_CUDA::dropout_call(stream, index), d_dropout_mask, (long long)n));
    }
    ZOPH_CALL(zr_dropout_apply(ctx, d_dropout_mask, dropout_rate, d_sparse_lookup, (long long)n));
  }
  dType* gates[4] = {d_i_t, d_f_t, d_c_prime_t_tanh, d_o_t};
  const bool use_q = feed_input && index != 0;  // src/LSTM.hpp:154
  ZOPH_CALL(zr_lstm_step(ctx, model->packed, d_sparse_lookup, d_h_t_prev, d_c_t_prev, use_q ? d_h_tild : nullptr,
                         d_input_vocab_indices_01, BZ_CUDA::clip_cell ? BZ_CUDA::cell_clip_threshold : 0.0f,
                         minibatch_size, d_h_t, d_c_t, gates));
  send_h_t_above();
}

template <typename dType>
void LSTM_IH_Node<dType>::send_h_t_above() {  // src/LSTM.hpp:424-520, pointer-passing branch
  int idx = (model->model && model->model->decode) ? 0 : index;
  dType* out = d_h_t;
  if (attention_model && model->attent_layer) {
    model->attent_layer->nodes[idx].d_h_t = d_h_t;
    model->attent_layer->nodes[idx].forward_prop();
    out = model->attent_layer->nodes[idx].d_final_temp_2;
  }
  if (model->upper_layer.upper_softmax) {
    if (!model->upper_layer.source_side && model->upper_layer.softmax) model->upper_layer.softmax->set_ht_ptr(idx, out);
  } else if (model->upper_layer.hidden_layer) {
    model->upper_layer.hidden_layer->nodes[idx].d_h_t_below = out;
  }
}

// ------------------------------------------------------------------------------------------------ backward
template <typename dType>
void lower_transfer_layer<dType>::send_error(int index, dType* d_err) {
  if (lower_input) {
    if (input_layer) input_layer->nodes[index].d_d_ERRt_ht = d_err;
  } else if (hidden_layer) {
    hidden_layer->nodes[index].d_d_ERRt_ht = d_err;
  }
}

// One node of back-propagation through time.  The reference runs nine element-wise kernels and eight products per
// node; here the node is one element-wise kernel and one batched product (zr_lstm_node_backward), followed by the
// node's share of the weight gradients.  The errors for step t-1 land in the layer's d_d_ERRnTOt_htM1 / _ctM1, which
// the driver passes to the next backprop_prep_GPU call, and the error for the layer below is handed down by pointer.
template <typename dType>
void LSTM_HH_Node<dType>::back_prop_GPU(int index) {
  zr_ctx* ctx = model->hh_layer_info.ctx;
  if (!model->train_weights) model->clear_gradients(true);
  if (attention_model && model->attent_layer) {  // src/LSTM_HH.hpp:470-482: the error of h~ becomes the error of h_t
    auto& an = model->attent_layer->nodes[index];
    an.d_d_ERRt_ht_tild = d_d_ERRt_ht;
    an.back_prop();
  }
  const dType* gates[4] = {d_i_t, d_f_t, d_c_prime_t_tanh, d_o_t};
  ZOPH_CALL(zr_lstm_node_backward(ctx, model->train_weights, minibatch_size, gates, d_c_t, d_c_t_prev,
                                  d_input_vocab_indices_01, d_d_ERRt_ht, d_d_ERRnTOtp1_ht, d_d_ERRnTOtp1_ct,
                                  model->d_d_ERRnTOt_gates, model->d_d_ERRnTOt_htM1, model->d_d_ERRnTOt_ctM1,
                                  model->d_d_ERRnTOt_h_Below));
  BZ_CUDA::clip_error(ctx, model->d_d_ERRnTOt_htM1, (long long)LSTM_size * minibatch_size);     // src/LSTM_HH.hpp:755-757
  BZ_CUDA::clip_error(ctx, model->d_d_ERRnTOt_h_Below, (long long)LSTM_size * minibatch_size);  // src/LSTM_HH.hpp:665-667
  compute_gradients_GPU();
  if (d_input == d_h_t_below_drop && d_dropout_mask)  // src/LSTM_HH.hpp:673-675
    ZOPH_CALL(zr_dropout_apply(ctx, d_dropout_mask, dropout_rate, model->d_d_ERRnTOt_h_Below,
                               (long long)LSTM_size * minibatch_size));
  model->lower_layer.send_error(index, model->d_d_ERRnTOt_h_Below);
}

template <typename dType>
void LSTM_HH_Node<dType>::compute_gradients_GPU() {
  ZOPH_CALL(zr_lstm_node_gradients(model->hh_layer_info.ctx, LSTM_size, minibatch_size, model->d_d_ERRnTOt_gates,
                                   d_input ? d_input : d_h_t_below, d_h_t_prev, model->d_M_grad_stack,
                                   model->d_W_h_grad_stack, model->d_b_grad_stack));
}

template <typename dType>
void LSTM_IH_Node<dType>::back_prop_GPU(int /*index*/) {
  zr_ctx* ctx = model->ih_layer_info.ctx;
  if (!model->train_weights) model->clear_gradients(true);
  if (attention_model && model->attent_layer) {  // src/LSTM.hpp:587-599: a one-layer model's attention sits on this layer
    auto& an = model->attent_layer->nodes[index];
    an.d_d_ERRt_ht_tild = d_d_ERRt_ht;
    an.back_prop();
  }
  const dType* gates[4] = {d_i_t, d_f_t, d_c_prime_t_tanh, d_o_t};
  ZOPH_CALL(zr_lstm_node_backward(ctx, model->train_weights, minibatch_size, gates, d_c_t, d_c_t_prev,
                                  d_input_vocab_indices_01, d_d_ERRt_ht, d_d_ERRnTOtp1_ht, d_d_ERRnTOtp1_ct,
                                  model->d_d_ERRnTOt_gates, model->d_d_ERRnTOt_htM1, model->d_d_ERRnTOt_ctM1,
                                  model->d_d_ERRnTOt_h_Below));
  // src/LSTM.hpp:792-794 (the error that reaches the embedding through d_d_ERRnTOt_h_Below is not clamped there)
  BZ_CUDA::clip_error(ctx, model->d_d_ERRnTOt_htM1, (long long)LSTM_size * minibatch_size);
  if (feed_input && index != 0) {  // src/LSTM.hpp:804-866 and :1014-1050
    const dType* Q[4] = {model->d_Q_i, model->d_Q_f, model->d_Q_c, model->d_Q_o};
    ZOPH_CALL(zr_lstm_feed_backward(ctx, Q, LSTM_size, minibatch_size, model->d_d_ERRnTOt_gates, d_h_tild,
                                    model->d_ERRnTOt_h_tild, model->d_Q_grad_stack));
    BZ_CUDA::clip_error(ctx, model->d_ERRnTOt_h_tild, (long long)LSTM_size * minibatch_size);  // src/LSTM.hpp:861-863
    if (d_ERRnTOt_h_tild_cpy)
      ZOPH_CALL(zr_d2d(ctx, d_ERRnTOt_h_tild_cpy, model->d_ERRnTOt_h_tild,
                       (size_t)LSTM_size * minibatch_size * sizeof(dType)));
  }
  compute_gradients_GPU();
}

template <typename dType>
void LSTM_IH_Node<dType>::compute_gradients_GPU() {
  zr_ctx* ctx = model->ih_layer_info.ctx;
  ZOPH_CALL(zr_lstm_node_gradients(ctx, LSTM_size, minibatch_size, model->d_d_ERRnTOt_gates, d_sparse_lookup,
                                   d_h_t_prev, model->d_M_grad_stack, model->d_W_h_grad_stack, model->d_b_grad_stack));
  // the sparse W gradient (src/custom_kernels.h:353-378): the error at the node's input, added into the columns of
  // the minibatch's words; with dropout the error passes the node's mask first (W_small_dropout_gradient_kernel,
  // src/LSTM.hpp:1196)
  if (dropout && d_dropout_mask && model->model && model->model->train)
    ZOPH_CALL(zr_dropout_apply(ctx, d_dropout_mask, dropout_rate, model->d_d_ERRnTOt_h_Below,
                               (long long)LSTM_size * minibatch_size));
  ZOPH_CALL(zr_embed_gradient(ctx, LSTM_size, model->input_vocab_size, model->d_d_ERRnTOt_h_Below,
                              d_input_vocab_indices, d_input_vocab_indices_01, minibatch_size, model->d_W_grad));
}

#endif  // ZOPH_LAYERS_H
