// Force-decode / perplexity driver over text files: what `ZOPH_RNN --force-decode` does with a trained model
// (src/main.cu force-decode branch -> neuralMT_model::get_perplexity, src/model.hpp:2281-2355), on the MI355X path.
//
//   force_decode [options] model.nn source.txt target.txt scores.txt
//   force_decode --sequence [options] model.nn target.txt scores.txt
//
// The text files hold one tokenised sentence per line.  They are integerized with the model's own vocabulary
// (source reversed, <UNK> for unknown words, <START> / <EOF> on the target side), run through the layer classes
// minibatch by minibatch, and scores.txt receives one natural-log probability per minibatch (per sentence with the
// default --minibatch 1), as the reference's force-decode output does.  The perplexity is printed at the end.
//
// Options: --minibatch N (1)  --longest-sent L (100)  --attention-width D (10; the model file does not store it)
//          --bf16 (stream the matrices as bf16)  --int-file PATH (where to keep the integerized data)
//          --integerize-only (stop after writing the integerized file; needs no GPU)
//          --dump PATH (write the loaded model back out as a complete model file: header, vocabularies, matrices)
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <string>
#include <vector>

#include "zoph_model.h"

static int usage(const char* argv0) {
  std::fprintf(stderr,
               "usage: %s [--sequence] [--minibatch N] [--longest-sent L] [--attention-width D] [--bf16]\n"
               "          [--int-file PATH] [--integerize-only] [--dump PATH] model.nn [source.txt] target.txt scores.txt\n",
               argv0);
  return 2;
}

int main(int argc, char** argv) {
  bool LM = false, bf16 = false, integerize_only = false;
  int minibatch = 1, longest = 100, D = 10;
  std::string int_file, dump_path;
  std::vector<std::string> pos;
  for (int i = 1; i < argc; i++) {
    const std::string a = argv[i];
    auto need = [&](int& dst) {
      if (i + 1 >= argc) return false;
      dst = std::atoi(argv[++i]);
      return dst > 0;
    };
    if (a == "--sequence") LM = true;
    else if (a == "--bf16") bf16 = true;
    else if (a == "--integerize-only") integerize_only = true;
    else if (a == "--minibatch") { if (!need(minibatch)) return usage(argv[0]); }
    else if (a == "--longest-sent") { if (!need(longest)) return usage(argv[0]); }
    else if (a == "--attention-width") { if (!need(D)) return usage(argv[0]); }
    else if (a == "--int-file") { if (i + 1 >= argc) return usage(argv[0]); int_file = argv[++i]; }
    else if (a == "--dump") { if (i + 1 >= argc) return usage(argv[0]); dump_path = argv[++i]; }
    else if (a.rfind("--", 0) == 0) return usage(argv[0]);
    else pos.push_back(a);
  }
  if (pos.size() != (LM ? 3u : 4u)) return usage(argv[0]);
  const std::string model_path = pos[0], source_path = LM ? "" : pos[1], target_path = pos[LM ? 1 : 2],
                    out_path = pos[LM ? 2 : 3];
  if (int_file.empty()) int_file = out_path + ".int";

  std::ifstream model(model_path);
  if (!model) {
    std::fprintf(stderr, "cannot open %s\n", model_path.c_str());
    return 1;
  }
  model_file_info info;
  std::string err;
  if (!read_model_file_info(model, LM, info, err)) {
    std::fprintf(stderr, "%s: %s\n", model_path.c_str(), err.c_str());
    return 1;
  }
  long long total_target_words = 0;
  const int n_sent = LM ? integerize_target_text(info, target_path, int_file, minibatch, longest, total_target_words, err)
                        : integerize_parallel_text(info, source_path, target_path, int_file, minibatch, longest,
                                                   total_target_words, err);
  if (n_sent < 0) {
    std::fprintf(stderr, "integerization failed: %s\n", err.c_str());
    return 1;
  }
  std::cout << "Sentences: " << n_sent << "\n";
  std::cout << "Total target words: " << total_target_words << "\n";
  if (integerize_only) return 0;

  BZ_CUDA::bf16_weights = bf16;
  BZ_CUDA::force_decode = true;
  layer_gpu_info gpu;
  gpu.init(0);
  forward_model<precision> m;
  m.initModel(gpu, info, minibatch, longest, D);
  m.load_weights(model);
  if (!dump_path.empty()) {
    std::ofstream d(dump_path);
    if (!d) {
      std::fprintf(stderr, "cannot write %s\n", dump_path.c_str());
      return 1;
    }
    m.dump_weights(d);
  }
  std::ofstream out(out_path);
  if (!out) {
    std::fprintf(stderr, "cannot write %s\n", out_path.c_str());
    return 1;
  }
  double log_prob = 0;
  const double ppl = m.get_perplexity(int_file, total_target_words, &out, log_prob, err);
  if (!err.empty()) {
    std::fprintf(stderr, "%s\n", err.c_str());
    return 1;
  }
  devSynchAll(gpu.ctx);
  std::cout << std::setprecision(15) << "Perplexity: " << ppl << "\n";
  std::cout << std::setprecision(15) << "P_data (bits): " << log_prob / std::log(2.0) << "\n";
  return 0;
}
