// Beam-search translation driver over text files: what `ZOPH_RNN --decode` does for one model
// (ensemble_factory::decode_file_batch, src/ensemble_factory.hpp:583-765; k-best selection and output
// decoder::output_k_best_hypotheses, src/decoder.h:1386-1480), on the MI355X path, several sentences at a time.
//
//   beam_decode [options] model.nn source.txt output.txt
//
// source.txt holds one tokenised sentence per line.  Sentences are integerized with the model's source vocabulary
// (reversed, <UNK> for unknown words), grouped by source length (sentences decoded side by side must have one
// length, so that every sentence gets exactly the number of steps the reference would give it: min(max-ratio *
// source length, longest-sent - 2)) and written in input order.
// Default output: the best hypothesis of each sentence as words, one line per sentence, <START> / <EOF> stripped.
// With --num-best K > 1 or --print-score: the reference's block layout, a line of dashes per sentence, then per
// hypothesis an optional "-Score: s" line and the hypothesis (ids with --ids, <START> and <EOF> included, as the
// reference's integer output; words otherwise).
//
// model.nn may be a comma-separated list of model files: an ensemble (src/ensemble_factory.hpp:767-793).  Every model
// integerizes the source with its own source vocabulary; the target vocabularies must be the same size (the first
// model's words are printed); the models' output distributions are averaged and renormalised before the one beam picks
// from them.  At most 8 models.  With --UNK-decode the alignments written are the models' vote (their alignment weights
// summed per source position, src/ensemble_factory.hpp:797-834).
// --UNK-decode FILE (attention models): the reference's unk-replacement side file (src/decoder.h:1452-1459) -- per
// output hypothesis one line with, for every <UNK> (id 2) at position j of the hypothesis, the Viterbi alignment stored
// at position j+1, i.e. a position in the reversed source sentence as the attention layer counts them.
//
// Options: --beam B (12)  --batch N (16 sentences side by side)  --longest-sent L (100)  --attention-width D (10)
//          --penalty P (0)  --min-ratio R (0.5)  --max-ratio R (1.5)  --num-best K (1)  --print-score  --ids  --bf16
//          --UNK-decode FILE
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <map>
#include <string>
#include <vector>

#include "zoph_model.h"

static int usage(const char* argv0) {
  std::fprintf(stderr,
               "usage: %s [--beam B] [--batch N] [--longest-sent L] [--attention-width D] [--penalty P]\n"
               "          [--min-ratio R] [--max-ratio R] [--num-best K] [--print-score] [--ids] [--bf16]\n"
               "          [--UNK-decode FILE] model.nn source.txt output.txt\n",
               argv0);
  return 2;
}

int main(int argc, char** argv) {
  int beam = 12, batch = 16, longest = 100, D = 10, num_best = 1;
  double penalty = 0, min_ratio = 0.5, max_ratio = 1.5;
  bool print_score = false, ids_out = false, bf16 = false;
  std::string unk_file;
  std::vector<std::string> pos;
  for (int i = 1; i < argc; i++) {
    const std::string a = argv[i];
    auto geti = [&](int& dst) {
      if (i + 1 >= argc) return false;
      dst = std::atoi(argv[++i]);
      return dst > 0;
    };
    auto getd = [&](double& dst) {
      if (i + 1 >= argc) return false;
      dst = std::atof(argv[++i]);
      return true;
    };
    if (a == "--beam") { if (!geti(beam)) return usage(argv[0]); }
    else if (a == "--batch") { if (!geti(batch)) return usage(argv[0]); }
    else if (a == "--longest-sent") { if (!geti(longest)) return usage(argv[0]); }
    else if (a == "--attention-width") { if (!geti(D)) return usage(argv[0]); }
    else if (a == "--num-best") { if (!geti(num_best)) return usage(argv[0]); }
    else if (a == "--penalty") { if (!getd(penalty)) return usage(argv[0]); }
    else if (a == "--min-ratio") { if (!getd(min_ratio)) return usage(argv[0]); }
    else if (a == "--max-ratio") { if (!getd(max_ratio)) return usage(argv[0]); }
    else if (a == "--print-score") print_score = true;
    else if (a == "--ids") ids_out = true;
    else if (a == "--bf16") bf16 = true;
    else if (a == "--UNK-decode") {
      if (i + 1 >= argc) return usage(argv[0]);
      unk_file = argv[++i];
    }
    else if (a.rfind("--", 0) == 0) return usage(argv[0]);
    else pos.push_back(a);
  }
  if (pos.size() != 3 || beam > 31) return usage(argv[0]);

  std::vector<std::string> model_paths;
  for (size_t from = 0; from <= pos[0].size();) {
    const size_t comma = pos[0].find(',', from);
    const size_t to = comma == std::string::npos ? pos[0].size() : comma;
    if (to > from) model_paths.push_back(pos[0].substr(from, to - from));
    from = to + 1;
  }
  const int K = (int)model_paths.size();
  if (K < 1 || K > 8) return usage(argv[0]);

  std::vector<std::ifstream> model_files(K);
  std::vector<model_file_info> infos(K);
  std::string err;
  for (int k = 0; k < K; k++) {
    model_files[k].open(model_paths[k]);
    if (!model_files[k]) {
      std::fprintf(stderr, "cannot open %s\n", model_paths[k].c_str());
      return 1;
    }
    if (!read_model_file_info(model_files[k], false, infos[k], err)) {
      std::fprintf(stderr, "%s: %s\n", model_paths[k].c_str(), err.c_str());
      return 1;
    }
    if (infos[k].target_vocab_size != infos[0].target_vocab_size) {
      std::fprintf(stderr, "%s: the models of an ensemble must have target vocabularies of one size\n",
                   model_paths[k].c_str());
      return 1;
    }
  }
  const model_file_info& info = infos[0];
  // integerize the source side once per model: vocabulary lookup, reversed (src/input_file_prep.h:405-416)
  std::vector<std::vector<std::vector<int>>> sents(K);  // [model][sentence]
  for (int k = 0; k < K; k++) {
    std::unordered_map<std::string, int> smap;
    for (size_t i = 0; i < infos[k].source_vocab.size(); i++) smap[infos[k].source_vocab[i]] = (int)i;
    const int unk = smap.count("<UNK>") ? smap["<UNK>"] : 0;
    std::ifstream src(pos[1]);
    if (!src) {
      std::fprintf(stderr, "cannot open %s\n", pos[1].c_str());
      return 1;
    }
    std::string line;
    while (std::getline(src, line)) {
      std::vector<int> v;
      for (const auto& w : zoph_split_words(line)) v.push_back(smap.count(w) ? smap[w] : unk);
      std::reverse(v.begin(), v.end());
      if (v.empty() || (int)v.size() > longest - 2) {
        std::fprintf(stderr, "source sentence %zu is empty or longer than longest-sent - 2\n", sents[k].size() + 1);
        return 1;
      }
      sents[k].push_back(v);
    }
  }
  const size_t n_sents = sents[0].size();
  std::map<int, std::vector<int>> by_len;  // source length -> sentence numbers, in input order
  for (size_t i = 0; i < n_sents; i++) by_len[(int)sents[0][i].size()].push_back((int)i);

  BZ_CUDA::bf16_weights = bf16;
  BZ_CUDA::unk_replacement = !unk_file.empty();  // src/main.cu:410-412
  layer_gpu_info gpu;
  gpu.init(0);
  std::vector<forward_model<precision>> models(K);
  std::vector<beam_decoder<precision>*> decs;
  for (int k = 0; k < K; k++) {
    models[k].initModel(gpu, infos[k], 1, longest, D);
    models[k].load_weights(model_files[k]);
    decs.push_back(new beam_decoder<precision>(models[k], beam, batch, longest, D, penalty));
    decs.back()->min_decoding_ratio = min_ratio;
    decs.back()->max_decoding_ratio = max_ratio;
  }
  beam_decoder<precision>& dec = *decs[0];
  for (auto* d : decs)
    if (BZ_CUDA::unk_replacement && !d->track_viterbi) {
      std::fprintf(stderr, "--UNK-decode needs an attention model\n");
      return 1;
    }
  ensemble_beam_decoder<precision>* ensemble = K > 1 ? new ensemble_beam_decoder<precision>(decs) : nullptr;

  std::vector<std::vector<decoded_hypothesis>> results(n_sents);
  for (const auto& kv : by_len) {
    const auto& idx = kv.second;
    for (size_t base = 0; base < idx.size(); base += batch) {
      const size_t end = std::min(idx.size(), base + (size_t)batch);
      std::vector<std::vector<decoded_hypothesis>> out;
      if (ensemble) {
        std::vector<std::vector<std::vector<int>>> group(K);
        for (int k = 0; k < K; k++)
          for (size_t j = base; j < end; j++) group[k].push_back(sents[k][idx[j]]);
        ensemble->decode_batch(group, num_best, out);
      } else {
        std::vector<std::vector<int>> group;
        for (size_t j = base; j < end; j++) group.push_back(sents[0][idx[j]]);
        dec.decode_batch(group, num_best, out);
      }
      for (size_t j = 0; j < end - base; j++) results[idx[base + j]] = out[j];
    }
  }

  std::ofstream out(pos[2]);
  if (!out) {
    std::fprintf(stderr, "cannot write %s\n", pos[2].c_str());
    return 1;
  }
  auto put = [&](const decoded_hypothesis& h, bool strip) {
    bool first = true;
    for (int w : h.words) {
      if (strip && (w == 0 || w == 1)) continue;
      if (!first) out << " ";
      first = false;
      if (ids_out)
        out << w;
      else
        out << (w >= 0 && w < (int)info.target_vocab.size() ? info.target_vocab[w] : "<UNK>");
    }
    out << "\n";
  };
  std::ofstream unk_out;
  if (BZ_CUDA::unk_replacement) {
    unk_out.open(unk_file);
    if (!unk_out) {
      std::fprintf(stderr, "cannot write %s\n", unk_file.c_str());
      return 1;
    }
  }
  auto put_unk = [&](const decoded_hypothesis& h) {  // src/decoder.h:1452-1459
    if (!BZ_CUDA::unk_replacement) return;
    for (size_t j = 0; j + 1 < h.words.size(); j++)
      if (h.words[j] == 2) unk_out << h.viterbi[j + 1] << " ";
    unk_out << "\n";
  };
  const bool blocks = num_best > 1 || print_score;
  for (const auto& r : results) {
    if (!blocks) {
      if (r.empty()) {
        out << "\n";
        if (BZ_CUDA::unk_replacement) unk_out << "\n";
      } else {
        put(r[0], true);
        put_unk(r[0]);
      }
      continue;
    }
    out << "------------------------------------------------\n";
    for (const auto& h : r) {
      if (print_score) out << "-Score: " << h.score << "\n";
      put(h, false);
      put_unk(h);
    }
    out << "\n";
  }
  std::cout << "Sentences: " << n_sents << "\n";
  if (dec.abandoned_launches)
    std::cout << "Batches decoded again after a single-launch schedule gave up a wait: " << dec.abandoned_launches << "\n";
  return 0;
}
