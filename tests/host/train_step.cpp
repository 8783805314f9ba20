// Test driver: SGD steps of model_trainer (zoph_rnn_amd/host/zoph_model.h) on the minibatches of an integerized file.
//   train_step [--sequence] [--node-level] [--abandon-sweeps] [--whole-clip | --ind-clip=T] [--clip-cell=C,E] [--attention-D=N] [--dropout=KEEP_RATE] [--dropout-seed=S]
//              model.nn data.int minibatch longest_sent learning_rate norm_clip steps
// Every step trains on the next minibatch of the file (wrapping around) and prints "loss <step> <log-likelihood>";
// the updated model is written to <model.nn>.trained as a complete model file.  --node-level: the step is
// forward_model::compute_gradients, i.e. the layer objects' own back_prop_GPU / update_weights members in the
// reference's node-by-node order, instead of model_trainer's stack-level calls.  --abandon-sweeps: the forward pass is
// forced onto the single-launch sweep with a wait limit of one poll, so its workgroups give up (and leave the kernel
// normally); model_trainer must notice and repeat the forward pass; prints "abandoned <count>" at the end.
// --whole-clip: norm_clip bounds the L2 norm of all gradients together (prints "global_norm <step> <norm>");
// --ind-clip=THRESHOLD: every gradient element is clamped to +-THRESHOLD instead (norm_clip is then unused).
// --clip-cell=C,E: the cell is clamped to +-C in the forward pass and back-propagated errors to +-E (node-level path).
// Models with attention (and feed-input) and dropout train through the node-level path only; --attention-D sets the
// window half-width (the model file does not store it), --dropout the probability of keeping a value.
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <string>
#include <vector>

#include "../../zoph_rnn_amd/host/zoph_model.h"

int main(int argc, char** argv) {
  bool LM = false, node_level = false, abandon = false;
  int attention_D = 10;
  float dropout_rate = 1.0f;
  std::vector<std::string> pos;
  for (int i = 1; i < argc; i++) {
    const std::string a = argv[i];
    if (a.rfind("--attention-D=", 0) == 0)
      attention_D = std::atoi(a.c_str() + 14);
    else if (a.rfind("--dropout=", 0) == 0)
      dropout_rate = (float)std::atof(a.c_str() + 10);
    else if (a.rfind("--dropout-seed=", 0) == 0)
      BZ_CUDA::dropout_seed = std::strtoull(a.c_str() + 15, nullptr, 10);
    else if (std::string(argv[i]) == "--sequence")
      LM = true;
    else if (std::string(argv[i]) == "--node-level")
      node_level = true;
    else if (std::string(argv[i]) == "--abandon-sweeps")
      abandon = true;
    else if (a.rfind("--clip-cell=", 0) == 0) {  // --clip-cell of the reference: <cell threshold>,<error threshold>
      BZ_CUDA::clip_cell = true;
      BZ_CUDA::cell_clip_threshold = (float)std::atof(a.c_str() + 12);
      const size_t comma = a.find(',');
      if (comma != std::string::npos) BZ_CUDA::error_clip_threshold = (float)std::atof(a.c_str() + comma + 1);
    } else if (a == "--whole-clip")  // --whole-clip-gradients of the reference: norm_clip bounds the whole model's norm
      BZ_CUDA::global_clip_flag = true;
    else if (a.rfind("--ind-clip=", 0) == 0) {  // --ind-clip-gradients: every element clamped to +-threshold
      BZ_CUDA::individual_grad_clip = true;
      BZ_CUDA::ind_norm_clip_thres = (float)std::atof(a.c_str() + 11);
    }
    else
      pos.push_back(argv[i]);
  }
  if (pos.size() != 7) {
    std::fprintf(stderr, "usage: %s [--sequence] [--node-level] [--whole-clip | --ind-clip=THRESHOLD] model.nn data.int minibatch longest_sent learning_rate norm_clip steps\n", argv[0]);
    return 2;
  }
  const int minibatch = std::atoi(pos[2].c_str()), longest = std::atoi(pos[3].c_str()), steps = std::atoi(pos[6].c_str());
  const float lr = (float)std::atof(pos[4].c_str()), clip = (float)std::atof(pos[5].c_str());
  std::ifstream model(pos[0]);
  model_file_info info;
  std::string err;
  if (!model || !read_model_file_info(model, LM, info, err)) {
    std::fprintf(stderr, "%s: %s\n", pos[0].c_str(), err.c_str());
    return 1;
  }
  layer_gpu_info gpu;
  gpu.init(0);
  forward_model<precision> m;
  m.params.learning_rate = lr;
  m.params.norm_clip = clip;
  m.params.clip_gradient = clip > 0 && !BZ_CUDA::global_clip_flag && !BZ_CUDA::individual_grad_clip;
  m.initModel(gpu, info, minibatch, longest, attention_D, dropout_rate);
  m.load_weights(model);
  model_trainer<precision>* trainer = node_level ? nullptr : new model_trainer<precision>(m);
  if (abandon && trainer) {
    ZOPH_CALL(zr_ctx_set_option(gpu.ctx, ZR_OPT_LSTM_SWEEP, 2));
    ZOPH_CALL(zr_ctx_set_option(gpu.ctx, ZR_OPT_LSTM_SWEEP_SPIN, 1));
    trainer->lstm_sweep_option = 2;
  }
  minibatch_reader reader;
  if (!reader.open(pos[1], minibatch, longest, LM)) {
    std::fprintf(stderr, "cannot open %s\n", pos[1].c_str());
    return 1;
  }
  std::cout << std::setprecision(15);
  for (int s = 0; s < steps; s++) {
    if (!reader.read_minibatch(err)) {
      if (!err.empty()) {
        std::fprintf(stderr, "%s\n", err.c_str());
        return 1;
      }
      reader.input_file.clear();
      reader.input_file.seekg(0, std::ios::beg);
      if (!reader.read_minibatch(err)) return 1;
    }
    double loss;
    if (node_level) {
      loss = m.getError(reader);
      m.compute_gradients(reader);
    } else {
      loss = trainer->train_minibatch(reader, lr, clip);
    }
    std::cout << "loss " << s << " " << loss << "\n";
    if (BZ_CUDA::global_clip_flag) std::cout << "global_norm " << s << " " << BZ_CUDA::read_global_norm(gpu.ctx) << "\n";
  }
  if (trainer) std::cout << "abandoned " << trainer->abandoned_sweeps << "\n";
  devSynchAll(gpu.ctx);
  std::ofstream out(pos[0] + ".trained");
  m.dump_weights(out);
  return 0;
}
