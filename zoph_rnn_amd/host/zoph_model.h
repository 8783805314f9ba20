// Model files, integerized data files and the forward (force-decode / perplexity) schedule on top of the layer
// classes of zoph_layers.h.
//
//  * model_file_info, read_model_file_info, write_model_file_info: the text model file of the reference -- header
//    line, vocabulary blocks between "====" lines, then the matrices (written by src/input_file_prep.h:304-357 and
//    src/add_model_info.h:7-23, skipped over by neuralMT_model::load_weights, src/model.hpp:2172-2195).
//  * integerize_parallel_text / integerize_target_text: raw tokenised text -> the 4-lines-per-sentence integer file
//    (src/input_file_prep.h:403-500 for source/target pairs, :1590-1670 for the sequence model): vocabulary lookup
//    with <UNK>, source reversed and left padded with -1, target input <START> + words, target output words + <EOF>,
//    right padded with -1, padding per minibatch.
//  * minibatch_reader: file_helper::read_minibatch (src/fileHelper.h:367-518) -- fills the time-major host arrays
//    idx[b + t*minibatch] and batch_info.
//  * forward_model: the layers wired as neuralMT_model::initModel does (src/model.hpp:300-420), load_weights /
//    dump_weights in file order (src/model.hpp:2172-2241, 2058-2070), getError(GPU) (src/model.hpp:1463-1802) and
//    get_perplexity with the force-decode output of one log-probability line per minibatch (src/model.hpp:2281-2355).
#ifndef ZOPH_MODEL_H
#define ZOPH_MODEL_H

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <functional>
#include <iomanip>
#include <limits>
#include <map>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "zoph_layers.h"

struct model_file_info {
  int num_layers = 1, LSTM_size = 0, target_vocab_size = 0, source_vocab_size = 0;
  bool attention_model = false, feed_input = false, multi_source = false, combine_LSTM = false, char_cnn = false;
  bool LM = false;                         // sequence model: no source side, one vocabulary block
  std::vector<std::string> source_vocab;   // index -> word ("<UNK>" at 0)
  std::vector<std::string> target_vocab;   // index -> word ("<START>", "<EOF>", "<UNK>" at 0, 1, 2)
};

inline bool zoph_is_separator(const std::string& s) { return s.size() > 3 && s[0] == '=' && s[1] == '=' && s[2] == '='; }

// Reads the header and the vocabulary block(s) and leaves the stream at the first matrix.  Returns false and
// fills err on a malformed file or a model kind the forward path does not cover.
inline bool read_model_file_info(std::istream& in, bool LM, model_file_info& info, std::string& err) {
  std::string line;
  if (!std::getline(in, line)) {
    err = "empty model file";
    return false;
  }
  std::vector<std::string> f;
  {
    std::istringstream iss(line);
    std::string w;
    while (iss >> w) f.push_back(w);
  }
  // 9 fields after training (add_model_info); 3 or 4 straight after data preparation
  if (f.size() != 9 && f.size() != 4 && f.size() != 3) {
    err = "model header has " + std::to_string(f.size()) + " fields (expected 9, 4 or 3)";
    return false;
  }
  try {
    info.num_layers = std::stoi(f[0]);
    info.LSTM_size = std::stoi(f[1]);
    info.target_vocab_size = std::stoi(f[2]);
    info.source_vocab_size = f.size() >= 4 ? std::stoi(f[3]) : 0;
    if (f.size() == 9) {
      info.attention_model = std::stoi(f[4]) != 0;
      info.feed_input = std::stoi(f[5]) != 0;
      info.multi_source = std::stoi(f[6]) != 0;
      info.combine_LSTM = std::stoi(f[7]) != 0;
      info.char_cnn = std::stoi(f[8]) != 0;
    }
  } catch (const std::exception&) {
    err = "model header is not numeric: " + line;
    return false;
  }
  info.LM = LM;
  if (info.multi_source || info.char_cnn) {
    err = "multi-source and character-CNN models are outside the forward path built here";
    return false;
  }
  if (info.num_layers < 1 || info.LSTM_size < 1 || info.target_vocab_size < 3) {
    err = "implausible model header: " + line;
    return false;
  }
  if (!std::getline(in, line) || !zoph_is_separator(line)) {
    err = "missing separator after the model header";
    return false;
  }
  auto read_block = [&](std::vector<std::string>& vocab, const char* what) {
    while (std::getline(in, line)) {
      if (zoph_is_separator(line)) return true;
      std::istringstream iss(line);
      long long id;
      std::string word;
      if (!(iss >> id >> word) || id != (long long)vocab.size()) {
        err = std::string("bad ") + what + " vocabulary line: " + line;
        return false;
      }
      vocab.push_back(word);
    }
    err = std::string("unterminated ") + what + " vocabulary block";
    return false;
  };
  info.source_vocab.clear();
  info.target_vocab.clear();
  if (!LM && !read_block(info.source_vocab, "source")) return false;
  if (!read_block(info.target_vocab, "target")) return false;
  if ((int)info.target_vocab.size() != info.target_vocab_size ||
      (!LM && (int)info.source_vocab.size() != info.source_vocab_size)) {
    err = "vocabulary blocks do not match the sizes in the header";
    return false;
  }
  return true;
}

inline void write_model_file_info(std::ostream& out, const model_file_info& info) {
  const char* sep = "==========================================================\n";
  out << info.num_layers << " " << info.LSTM_size << " " << info.target_vocab_size << " " << info.source_vocab_size
      << " " << (int)info.attention_model << " " << (int)info.feed_input << " " << (int)info.multi_source << " "
      << (int)info.combine_LSTM << " " << (int)info.char_cnn << "\n";
  out << sep;
  if (!info.LM) {
    for (size_t i = 0; i < info.source_vocab.size(); i++) out << i << " " << info.source_vocab[i] << "\n";
    out << sep;
  }
  for (size_t i = 0; i < info.target_vocab.size(); i++) out << i << " " << info.target_vocab[i] << "\n";
  out << sep;
}

// ------------------------------------------------------------------------------------------------ integerization
inline std::vector<std::string> zoph_split_words(const std::string& line) {
  std::istringstream iss(line);
  std::vector<std::string> w;
  std::string t;
  while (iss >> t) w.push_back(t);
  return w;
}

struct integerized_sentence {
  std::vector<int> src, minus_two, tgt_in, tgt_out;
};

inline void zoph_write_int_line(std::ostream& out, const std::vector<int>& v) {
  for (int x : v) out << x << " ";
  out << "\n";
}

// Source / target text (one sentence per line, same number of lines) -> the integer file.  Sentences longer than
// longest_sent - 2 words on either side are an error here (the reference's force-decode path refuses them too).
// Returns the number of sentence pairs written, or -1 with err set.  total_target_words counts the target output
// tokens (words + <EOF>), the denominator of the perplexity.
inline int integerize_parallel_text(const model_file_info& info, const std::string& source_path,
                                    const std::string& target_path, const std::string& out_path, int minibatch_size,
                                    int longest_sent, long long& total_target_words, std::string& err) {
  std::ifstream fs(source_path), ft(target_path);
  if (!fs || !ft) {
    err = "cannot open " + (fs ? target_path : source_path);
    return -1;
  }
  std::unordered_map<std::string, int> smap, tmap;
  for (size_t i = 0; i < info.source_vocab.size(); i++) smap[info.source_vocab[i]] = (int)i;
  for (size_t i = 0; i < info.target_vocab.size(); i++) tmap[info.target_vocab[i]] = (int)i;
  const int src_unk = smap.count("<UNK>") ? smap["<UNK>"] : 0;
  const int tgt_unk = tmap.count("<UNK>") ? tmap["<UNK>"] : (tmap.count("<UNK>NULL") ? tmap["<UNK>NULL"] : 2);
  std::vector<integerized_sentence> data;
  std::string ls, lt;
  total_target_words = 0;
  while (std::getline(fs, ls)) {
    if (!std::getline(ft, lt)) {
      err = "target file has fewer lines than the source file";
      return -1;
    }
    const auto sw = zoph_split_words(ls), tw = zoph_split_words(lt);
    if ((int)sw.size() > longest_sent - 2 || (int)tw.size() > longest_sent - 2 || sw.empty() || tw.empty()) {
      err = "sentence pair " + std::to_string(data.size() + 1) + " is empty or longer than longest_sent - 2";
      return -1;
    }
    integerized_sentence s;
    for (const auto& w : sw) s.src.push_back(smap.count(w) ? smap[w] : src_unk);
    std::reverse(s.src.begin(), s.src.end());
    s.minus_two.assign(s.src.size(), -2);
    for (const auto& w : tw) s.tgt_in.push_back(tmap.count(w) ? tmap[w] : tgt_unk);
    s.tgt_out = s.tgt_in;
    s.tgt_in.insert(s.tgt_in.begin(), 0);  // <START>
    s.tgt_out.push_back(1);                // <EOF>
    total_target_words += (long long)s.tgt_out.size();
    data.push_back(s);
  }
  if (std::getline(ft, lt) && !zoph_split_words(lt).empty()) {
    err = "target file has more lines than the source file";
    return -1;
  }
  for (size_t base = 0; base < data.size(); base += minibatch_size) {
    const size_t end = std::min(data.size(), base + (size_t)minibatch_size);
    size_t max_s = 0, max_t = 0;
    for (size_t i = base; i < end; i++) {
      max_s = std::max(max_s, data[i].src.size());
      max_t = std::max(max_t, data[i].tgt_in.size());
    }
    for (size_t i = base; i < end; i++) {
      auto& d = data[i];
      d.src.insert(d.src.begin(), max_s - d.src.size(), -1);  // source: left padded
      d.minus_two.insert(d.minus_two.begin(), max_s - d.minus_two.size(), -1);
      d.tgt_in.resize(max_t, -1);                             // target: right padded
      d.tgt_out.resize(max_t, -1);
    }
  }
  std::ofstream out(out_path);
  if (!out) {
    err = "cannot write " + out_path;
    return -1;
  }
  for (const auto& d : data) {
    zoph_write_int_line(out, d.src);
    zoph_write_int_line(out, d.minus_two);
    zoph_write_int_line(out, d.tgt_in);
    zoph_write_int_line(out, d.tgt_out);
  }
  return (int)data.size();
}

// Sequence-model variant (target side only): two empty lines, then target input and output; every sentence of a
// minibatch is padded to one MORE than the longest (the reference pads `while size <= max`,
// src/input_file_prep.h:1622-1627), which adds a fully masked last step.
inline int integerize_target_text(const model_file_info& info, const std::string& target_path,
                                  const std::string& out_path, int minibatch_size, int longest_sent,
                                  long long& total_target_words, std::string& err) {
  std::ifstream ft(target_path);
  if (!ft) {
    err = "cannot open " + target_path;
    return -1;
  }
  std::unordered_map<std::string, int> tmap;
  for (size_t i = 0; i < info.target_vocab.size(); i++) tmap[info.target_vocab[i]] = (int)i;
  const int tgt_unk = tmap.count("<UNK>") ? tmap["<UNK>"] : 2;
  std::vector<integerized_sentence> data;
  std::string lt;
  total_target_words = 0;
  while (std::getline(ft, lt)) {
    const auto tw = zoph_split_words(lt);
    if (tw.empty() || (int)tw.size() > longest_sent - 3) {
      err = "sentence " + std::to_string(data.size() + 1) + " is empty or longer than longest_sent - 3";
      return -1;
    }
    integerized_sentence s;
    for (const auto& w : tw) s.tgt_in.push_back(tmap.count(w) ? tmap[w] : tgt_unk);
    s.tgt_out = s.tgt_in;
    s.tgt_in.insert(s.tgt_in.begin(), 0);
    s.tgt_out.push_back(1);
    total_target_words += (long long)s.tgt_out.size();
    data.push_back(s);
  }
  for (size_t base = 0; base < data.size(); base += minibatch_size) {
    const size_t end = std::min(data.size(), base + (size_t)minibatch_size);
    size_t max_t = 0;
    for (size_t i = base; i < end; i++) max_t = std::max(max_t, data[i].tgt_in.size());
    for (size_t i = base; i < end; i++) {
      data[i].tgt_in.resize(max_t + 1, -1);
      data[i].tgt_out.resize(max_t + 1, -1);
    }
  }
  std::ofstream out(out_path);
  if (!out) {
    err = "cannot write " + out_path;
    return -1;
  }
  for (const auto& d : data) {
    out << "\n\n";
    zoph_write_int_line(out, d.tgt_in);
    zoph_write_int_line(out, d.tgt_out);
  }
  return (int)data.size();
}

// ------------------------------------------------------------------------------------------------ minibatch reader
struct minibatch_reader {
  int minibatch_size = 1, longest_sent = 100;
  bool LM = false;
  std::ifstream input_file;
  // time-major host arrays, idx[b + t*minibatch_size], as the layers' prep_GPU_vocab_indices expect them
  std::vector<int> h_input_vocab_indicies_source, h_output_vocab_indicies_source, h_input_vocab_indicies_target,
      h_output_vocab_indicies_target, h_batch_info;
  int current_source_length = 0, current_target_length = 0;
  int sentences_in_minibatch = 0;  // fewer than minibatch_size at the end of the file (the rest is padding)
  int words_in_minibatch = 0;

  bool open(const std::string& path, int minibatch, int longest, bool lm) {
    minibatch_size = minibatch;
    longest_sent = longest;
    LM = lm;
    input_file.open(path);
    const size_t n = (size_t)minibatch * longest;
    h_input_vocab_indicies_source.assign(n, -1);
    h_output_vocab_indicies_source.assign(n, -1);
    h_input_vocab_indicies_target.assign(n, -1);
    h_output_vocab_indicies_target.assign(n, -1);
    h_batch_info.assign(2 * (size_t)minibatch, 0);
    return (bool)input_file;
  }

  static std::vector<int> ints(const std::string& line) {
    std::istringstream iss(line);
    std::vector<int> v;
    std::string w;
    while (iss >> w) v.push_back(std::stoi(w));
    return v;
  }

  // Reads up to minibatch_size sentences (4 lines each).  Returns false when nothing was left.  A short last
  // minibatch is completed with fully padded (-1) columns, which contribute nothing to the loss.
  bool read_minibatch(std::string& err) {
    std::vector<std::vector<int>> si, so, ti, to;
    std::string a, b, c, d;
    while ((int)si.size() < minibatch_size && std::getline(input_file, a)) {
      if (!std::getline(input_file, b) || !std::getline(input_file, c) || !std::getline(input_file, d)) {
        err = "integer file ends in the middle of a sentence (4 lines per sentence)";
        return false;
      }
      si.push_back(ints(a));
      so.push_back(ints(b));
      ti.push_back(ints(c));
      to.push_back(ints(d));
    }
    sentences_in_minibatch = (int)si.size();
    if (si.empty()) return false;
    current_source_length = (int)si.back().size();
    current_target_length = (int)ti.back().size();
    for (size_t i = 0; i < si.size(); i++) {
      if ((int)si[i].size() != current_source_length || (int)ti[i].size() != current_target_length ||
          to[i].size() != ti[i].size()) {
        err = "sentences of one minibatch differ in padded length (was the file made for another minibatch size?)";
        return false;
      }
    }
    if (current_source_length > longest_sent || current_target_length > longest_sent) {
      err = "a sentence is longer than longest_sent";
      return false;
    }
    words_in_minibatch = 0;
    for (int i = 0; i < minibatch_size; i++) {
      const bool real = i < (int)si.size();
      int len = 0;
      for (int j = 0; j < current_source_length; j++) {
        const int v = real ? si[i][j] : -1;
        if (v != -1) len++;
        h_input_vocab_indicies_source[i + (size_t)j * minibatch_size] = v;
        h_output_vocab_indicies_source[i + (size_t)j * minibatch_size] = real && j < (int)so[i].size() ? so[i][j] : -1;
      }
      // a padding column still needs one readable source position for the attention window
      h_batch_info[i] = real ? len : (current_source_length > 0 ? 1 : 0);
      h_batch_info[i + minibatch_size] = current_source_length - h_batch_info[i];
      for (int j = 0; j < current_target_length; j++) {
        h_input_vocab_indicies_target[i + (size_t)j * minibatch_size] = real ? ti[i][j] : -1;
        h_output_vocab_indicies_target[i + (size_t)j * minibatch_size] = real ? to[i][j] : -1;
        if (real && to[i][j] != -1) words_in_minibatch++;
      }
    }
    return true;
  }
};

// ------------------------------------------------------------------------------------------------ the model
template <typename dType>
class forward_model {
 public:
  model_file_info info;
  global_params params;
  layer_gpu_info gpu;
  neuralMT_model<precision> flags;
  Input_To_Hidden_Layer<dType> input_layer_source, input_layer_target;
  std::vector<Hidden_To_Hidden_Layer<dType>> source_hidden_layers, target_hidden_layers;
  softmax_layer<dType> softmax_obj;
  base_loss_layer<dType>* softmax = nullptr;
  attention_layer<dType>* att = nullptr;

  // neuralMT_model::initModel (src/model.hpp:35-420) for the forward path on one device.  attention_D: the window
  // half-width; the model file does not store it and the reference's decoder uses its default of 10.
  // dropout_rate < 1: dropout with that probability of KEEPING a value, applied in compute_gradients only
  // (global_params::dropout / dropout_rate, src/global_params.h:86-87).
  void initModel(const layer_gpu_info& g, const model_file_info& mi, int minibatch_size, int longest_sent,
                 int attention_D = 10, float dropout_rate = 1.0f) {
    gpu = g;
    info = mi;
    params.dropout = dropout_rate < 1.0f;
    params.dropout_rate = dropout_rate;
    const bool dr = params.dropout;
    const bool seq2seq = !mi.LM;
    const int H = mi.LSTM_size, L = mi.num_layers;
    params.LSTM_size = H;
    params.minibatch_size = minibatch_size;
    params.longest_sent = longest_sent;
    params.target_vocab_size = mi.target_vocab_size;
    params.source_vocab_size = mi.source_vocab_size;
    params.attent_params.attention_model = seq2seq && mi.attention_model;
    params.attent_params.D = attention_D;
    params.attent_params.feed_input = seq2seq && mi.attention_model && mi.feed_input;
    flags.attent_params = params.attent_params;
    source_hidden_layers.resize(seq2seq ? L - 1 : 0);
    target_hidden_layers.resize(L - 1);
    softmax = &softmax_obj;
    softmax_obj.share_gpu(gpu);
    softmax->init_loss_layer(&flags, params);
    if (seq2seq) {
      input_layer_source.ih_layer_info.share(gpu);
      input_layer_source.init_Input_To_Hidden_Layer(H, minibatch_size, mi.source_vocab_size, longest_sent, false,
                                                    params.learning_rate, params.clip_gradient, params.norm_clip,
                                                    &flags, 0, dr, dropout_rate, false, false, nullptr, false, params, true);
      for (int l = 0; l < L - 1; l++) {
        source_hidden_layers[l].hh_layer_info.share(gpu);
        source_hidden_layers[l].init_Hidden_To_Hidden_Layer(H, minibatch_size, longest_sent, false, params.learning_rate,
                                                             params.clip_gradient, params.norm_clip, &flags, 0, dr,
                                                             dropout_rate, false, l);
      }
    }
    input_layer_target.ih_layer_info.share(gpu);
    input_layer_target.init_Input_To_Hidden_Layer(H, minibatch_size, mi.target_vocab_size, longest_sent, false,
                                                  params.learning_rate, params.clip_gradient, params.norm_clip, &flags,
                                                  0, dr, dropout_rate, false, false, nullptr, false, params, false);
    for (int l = 0; l < L - 1; l++) {
      target_hidden_layers[l].hh_layer_info.share(gpu);
      target_hidden_layers[l].init_Hidden_To_Hidden_Layer(H, minibatch_size, longest_sent, false, params.learning_rate,
                                                           params.clip_gradient, params.norm_clip, &flags, 0, dr,
                                                           dropout_rate, false, l);
    }
    // upper transfer (h_t upwards) and lower transfer (error downwards) wiring, src/model.hpp:191-290
    auto wire = [&](Input_To_Hidden_Layer<dType>& in, std::vector<Hidden_To_Hidden_Layer<dType>>& hid, bool source) {
      if (hid.empty()) {
        in.upper_layer.init_upper_transfer_layer(true, false, source, softmax, nullptr);
        if (!source) softmax->init_lower_transfer_layer(true, false, &in, nullptr);
      } else {
        in.upper_layer.init_upper_transfer_layer(false, false, source, nullptr, &hid[0]);
        hid[0].lower_layer.init_lower_transfer_layer(true, false, &in, nullptr);
        for (size_t l = 0; l + 1 < hid.size(); l++) {
          hid[l].upper_layer.init_upper_transfer_layer(false, false, source, nullptr, &hid[l + 1]);
          hid[l + 1].lower_layer.init_lower_transfer_layer(false, false, nullptr, &hid[l]);
        }
        hid.back().upper_layer.init_upper_transfer_layer(true, false, source, softmax, nullptr);
        if (!source) softmax->init_lower_transfer_layer(false, false, nullptr, &hid.back());
      }
    };
    if (seq2seq) wire(input_layer_source, source_hidden_layers, true);
    wire(input_layer_target, target_hidden_layers, false);
    if (params.attent_params.attention_model) {
      // the top target layer builds the attention layer from the model's source states, as in the reference
      // (src/model.hpp:330-345: init_attention(device, D, feed_input, this, params))
      flags.source_top_h_t.resize(longest_sent);
      for (int i = 0; i < longest_sent; i++)
        flags.source_top_h_t[i] = (L == 1) ? input_layer_source.nodes[i].d_h_t : source_hidden_layers[L - 2].nodes[i].d_h_t;
      params.attent_params.D = attention_D;
      if (L == 1)
        input_layer_target.init_attention(0, attention_D, params.attent_params.feed_input, &flags, params);
      else
        target_hidden_layers[L - 2].init_attention(0, attention_D, params.attent_params.feed_input, &flags, params);
      att = (L == 1) ? input_layer_target.attent_layer : target_hidden_layers[L - 2].attent_layer;
      if (params.attent_params.feed_input)
        input_layer_target.init_feed_input(L == 1 ? nullptr : &target_hidden_layers[L - 2], false);
    }
  }

  // matrices only: the stream must stand at the first matrix (after read_model_file_info)
  void load_weights(std::ifstream& w) {
    if (!info.LM) {
      input_layer_source.load_weights(w);
      for (auto& l : source_hidden_layers) l.load_weights(w);
    }
    input_layer_target.load_weights(w);
    for (auto& l : target_hidden_layers) l.load_weights(w);
    softmax->load_weights(w);
  }
  // header, vocabulary blocks and matrices: a complete model file
  void dump_weights(std::ofstream& o, bool with_header = true) {
    if (with_header) write_model_file_info(o, info);
    o << std::setprecision(std::numeric_limits<dType>::digits10 + 2);
    if (!info.LM) {
      input_layer_source.dump_weights(o);
      for (auto& l : source_hidden_layers) l.dump_weights(o);
    }
    input_layer_target.dump_weights(o);
    for (auto& l : target_hidden_layers) l.dump_weights(o);
    softmax->dump_weights(o);
  }

  // neuralMT_model::getError(GPU = true), src/model.hpp:1463-1802: natural-log probability of the minibatch's
  // target words.  per_step, if given, is called after each target step with (step, loss of the step).
  double getError(minibatch_reader& mb, const std::function<void(int, double)>& per_step = nullptr) {
    return forward_pass(mb, true, per_step);
  }

  // The forward half shared by getError and compute_gradients: every node of the (layer, time) grid in the
  // reference's order; with_loss adds the loss layer's log-probability of every step.
  double forward_pass(minibatch_reader& mb, bool with_loss, const std::function<void(int, double)>& per_step = nullptr) {
    const bool seq2seq = !info.LM;
    const int S = seq2seq ? mb.current_source_length : 0, T = mb.current_target_length;
    const int mbs = params.minibatch_size;
    if (seq2seq) {
      input_layer_source.prep_GPU_vocab_indices(mb.h_input_vocab_indicies_source.data(), nullptr, S, 0);
      for (auto& l : source_hidden_layers) l.prep_GPU_vocab_indices(mb.h_input_vocab_indicies_source.data(), S);
      if (att) att->prep_minibatch_info(mb.h_batch_info.data());
    }
    input_layer_target.prep_GPU_vocab_indices(mb.h_input_vocab_indicies_target.data(), nullptr, T, 0);
    for (auto& l : target_hidden_layers) l.prep_GPU_vocab_indices(mb.h_input_vocab_indicies_target.data(), T);
    softmax->prep_GPU_vocab_indices(mb.h_output_vocab_indicies_target.data(), T);

    for (int i = 0; i < S; i++) {
      const int step = i * mbs;
      auto& n0 = input_layer_source.nodes[i];
      n0.update_vectors_forward_GPU(
          input_layer_source.d_input_vocab_indices_full + step, input_layer_source.d_input_vocab_indices_01_full + step,
          i == 0 ? input_layer_source.d_init_hidden_vector : input_layer_source.nodes[i - 1].d_h_t,
          i == 0 ? input_layer_source.d_init_cell_vector : input_layer_source.nodes[i - 1].d_c_t);
      n0.forward_prop();
      for (auto& l : source_hidden_layers) {
        l.nodes[i].update_vectors_forward_GPU(l.d_input_vocab_indices_01_full + step,
                                              i == 0 ? l.d_init_hidden_vector : l.nodes[i - 1].d_h_t,
                                              i == 0 ? l.d_init_cell_vector : l.nodes[i - 1].d_c_t);
        l.nodes[i].forward_prop();
      }
    }
    double total = 0;
    for (int i = 0; i < T; i++) {
      const int step = i * mbs;
      dType *hp, *cp;
      if (i > 0) {
        hp = input_layer_target.nodes[i - 1].d_h_t;
        cp = input_layer_target.nodes[i - 1].d_c_t;
      } else if (seq2seq) {  // start from the encoder's last state (src/model.hpp:1714-1724)
        hp = input_layer_source.nodes[S - 1].d_h_t;
        cp = input_layer_source.nodes[S - 1].d_c_t;
      } else {
        hp = input_layer_target.d_init_hidden_vector;
        cp = input_layer_target.d_init_cell_vector;
      }
      input_layer_target.nodes[i].update_vectors_forward_GPU(input_layer_target.d_input_vocab_indices_full + step,
                                                             input_layer_target.d_input_vocab_indices_01_full + step,
                                                             hp, cp);
      input_layer_target.nodes[i].forward_prop();
      for (size_t l = 0; l < target_hidden_layers.size(); l++) {
        auto& ly = target_hidden_layers[l];
        if (i > 0) {
          hp = ly.nodes[i - 1].d_h_t;
          cp = ly.nodes[i - 1].d_c_t;
        } else if (seq2seq) {
          hp = source_hidden_layers[l].nodes[S - 1].d_h_t;
          cp = source_hidden_layers[l].nodes[S - 1].d_c_t;
        } else {
          hp = ly.d_init_hidden_vector;
          cp = ly.d_init_cell_vector;
        }
        ly.nodes[i].update_vectors_forward_GPU(ly.d_input_vocab_indices_01_full + step, hp, cp);
        ly.nodes[i].forward_prop();
      }
      if (!with_loss) continue;
      softmax->backprop_prep_GPU(softmax->get_ht_ptr(i), step);
      const double loss = softmax->compute_loss_GPU(i);
      total += loss;
      if (per_step) per_step(i, loss);
    }
    return total;
  }

  // neuralMT_model::compute_gradients (src/model.hpp:813-1230) through the layer objects' own members in the
  // reference's order: forward over the grid (training mode: dropout where it is on), then per target step (last
  // first) the loss layer's back_prop1 and the nodes' backprop_prep_GPU / back_prop_GPU from the top layer down -- the
  // top node runs its attention node's back_prop first, the bottom node sends the feed-input error to the previous
  // step's attention node -- then the source side, started from the errors the target side left at its first step and
  // with the attention layer's source-state errors arriving at its top layer, then update_weights and clear_gradients.
  void compute_gradients(minibatch_reader& mb) {
    const bool seq2seq = !info.LM;
    const int S = seq2seq ? mb.current_source_length : 0, T = mb.current_target_length;
    const int mbs = params.minibatch_size;
    if (!trained_before) {
      clear_gradients(true);
      trained_before = true;
    }
    flags.train = true;
    forward_pass(mb, false);
    for (int i = T - 1; i >= 0; i--) {
      const bool last = i == T - 1;
      softmax->backprop_prep_GPU(softmax->get_ht_ptr(i), i * mbs);
      softmax->back_prop1(i);
      for (int j = (int)target_hidden_layers.size() - 1; j >= 0; j--) {
        auto& ly = target_hidden_layers[j];
        ly.nodes[i].backprop_prep_GPU(last ? ly.d_init_d_ERRnTOtp1_ht : ly.d_d_ERRnTOt_htM1,
                                      last ? ly.d_init_d_ERRnTOtp1_ct : ly.d_d_ERRnTOt_ctM1);
        ly.nodes[i].back_prop_GPU(i);
      }
      auto& in = input_layer_target;
      in.nodes[i].backprop_prep_GPU(last ? in.d_init_d_ERRnTOtp1_ht : in.d_d_ERRnTOt_htM1,
                                    last ? in.d_init_d_ERRnTOtp1_ct : in.d_d_ERRnTOt_ctM1);
      in.nodes[i].back_prop_GPU(i);
      softmax->back_prop2(i);
    }
    for (int i = S - 1; i >= 0; i--) {
      const bool last = i == S - 1;  // the source's last step continues from the target's first (:1097-1126)
      if (att) {  // the error of source state i, collected by the attention nodes, arrives from above
        if (source_hidden_layers.empty())
          input_layer_source.nodes[i].d_d_ERRt_ht = att->h_total_hs_error[i];
        else
          source_hidden_layers.back().nodes[i].d_d_ERRt_ht = att->h_total_hs_error[i];
      }
      for (int j = (int)source_hidden_layers.size() - 1; j >= 0; j--) {
        auto& ly = source_hidden_layers[j];
        ly.nodes[i].backprop_prep_GPU(last ? target_hidden_layers[j].d_d_ERRnTOt_htM1 : ly.d_d_ERRnTOt_htM1,
                                      last ? target_hidden_layers[j].d_d_ERRnTOt_ctM1 : ly.d_d_ERRnTOt_ctM1);
        ly.nodes[i].back_prop_GPU(i);
      }
      auto& in = input_layer_source;
      in.nodes[i].backprop_prep_GPU(last ? input_layer_target.d_d_ERRnTOt_htM1 : in.d_d_ERRnTOt_htM1,
                                    last ? input_layer_target.d_d_ERRnTOt_ctM1 : in.d_d_ERRnTOt_ctM1);
      in.nodes[i].back_prop_GPU(i);
    }
    flags.train = false;
    BZ_CUDA::dropout_minibatch++;
    update_weights();
    clear_gradients(false);
  }
  bool trained_before = false;
  // learning rate and per-matrix norm clip (0: none) of every layer's update_weights
  void set_training_rates(float learning_rate, float norm_clip) {
    auto set = [&](auto& ly) {
      ly.learning_rate = learning_rate;
      ly.norm_clip = norm_clip;
      ly.clip_gradients = norm_clip > 0;
    };
    if (!info.LM) {
      set(input_layer_source);
      for (auto& l : source_hidden_layers) set(l);
    }
    set(input_layer_target);
    for (auto& l : target_hidden_layers) set(l);
    set(softmax_obj);
    if (att) set(*att);
  }

  void clear_gradients(bool init) {  // src/model.hpp:1431-1460
    if (!info.LM) {
      input_layer_source.clear_gradients(init);
      for (auto& l : source_hidden_layers) l.clear_gradients(init);
    }
    input_layer_target.clear_gradients(init);
    for (auto& l : target_hidden_layers) l.clear_gradients(init);
    softmax->clear_gradients();
    if (att) att->clear_gradients();
  }
  // src/model.hpp:1845-1955.  With BZ_CUDA::global_clip_flag every layer first adds its gradients' squared norms to the
  // whole-model sum (calculate_global_norm, :1850-1892), which the updates then read on the device.
  void update_weights() {
    if (BZ_CUDA::global_clip_flag && !BZ_CUDA::individual_grad_clip) {
      BZ_CUDA::reset_global_norm(gpu.ctx);
      softmax_obj.calculate_global_norm();
      if (!info.LM) {
        input_layer_source.calculate_global_norm();
        for (auto& l : source_hidden_layers) l.calculate_global_norm();
      }
      input_layer_target.calculate_global_norm();
      for (auto& l : target_hidden_layers) l.calculate_global_norm();
      if (att) att->calculate_global_norm();
    }
    softmax->update_weights();
    if (!info.LM) {
      input_layer_source.update_weights();
      for (auto& l : source_hidden_layers) l.update_weights();
    }
    input_layer_target.update_weights();
    for (auto& l : target_hidden_layers) l.update_weights();
    if (att) att->update_weights();
  }

  // neuralMT_model::get_perplexity (src/model.hpp:2281-2355): one getError per minibatch; with force_decode the
  // minibatch's log-probability (natural log) goes to fd_stream, one line per minibatch.  Returns the perplexity
  // 2^(-log2 P(data) / total_target_words).
  double get_perplexity(const std::string& int_file, long long total_target_words, std::ostream* fd_stream,
                        double& log_prob_total, std::string& err) {
    minibatch_reader reader;
    if (!reader.open(int_file, params.minibatch_size, params.longest_sent, info.LM)) {
      err = "cannot open " + int_file;
      return -1;
    }
    log_prob_total = 0;
    while (reader.read_minibatch(err)) {
      const double lp = getError(reader);
      if (fd_stream) *fd_stream << std::setprecision(15) << lp << "\n";
      log_prob_total += lp;
    }
    if (!err.empty()) return -1;
    const double bits = log_prob_total / std::log(2.0);
    return std::pow(2.0, -bits / (double)total_target_words);
  }
};

// ------------------------------------------------------------------------------------------------ training
// One SGD step on a minibatch: neuralMT_model::compute_gradients (src/model.hpp:1823-2000) followed by update_weights
// (:2002-2040).  Models without attention and without dropout (language models and plain encoder-decoder models) go
// through the stack-level training entry points of the library instead of node-by-node back_prop_GPU calls; models
// with attention (feed-input makes every target step depend on the one before, so there is no sweep to batch) or
// dropout go through forward_model::compute_gradients, the layer objects' own members.
// Gradients are those of the log-likelihood and are ADDED (the reference ascends), scaled by 1/minibatch_size and
// clipped per matrix to norm_clip in L2 norm (norm_clip_GPU_v2), as the reference does without --global-clip.
template <typename dType>
class model_trainer {
 public:
  forward_model<dType>& m;
  zr_ctx* ctx;
  int H, L, mb, longest, Vs, Vt;
  bool seq2seq;
  struct side {
    std::vector<zr_lstm_train*> train;
    std::vector<dType*> h_all, c_all, g_all, dg_all, eh0, ec0, dM, dWh, db;
    dType *below0 = nullptr, *x_all = nullptr, *dW = nullptr;
    int *d_ids = nullptr, *d_nn = nullptr, *d_mask = nullptr;
  } src, tgt;
  dType *zeros = nullptr, *err_top = nullptr, *prob = nullptr, *dD = nullptr, *dbd = nullptr, *unst[4] = {};
  int *d_tout = nullptr, *d_tmask = nullptr;
  float* d_tmaskf = nullptr;

  template <typename T>
  T* dmalloc(size_t n) {
    T* p = nullptr;
    ZOPH_CALL(zr_malloc(ctx, n * sizeof(T), (void**)&p));
    return p;
  }
  template <typename LayerT>
  static void gate_ptrs(LayerT& ly, const dType* M[4], const dType* Wh[4]) {
    M[0] = ly.d_M_i; M[1] = ly.d_M_f; M[2] = ly.d_M_c; M[3] = ly.d_M_o;
    Wh[0] = ly.d_W_hi; Wh[1] = ly.d_W_hf; Wh[2] = ly.d_W_hc; Wh[3] = ly.d_W_ho;
  }
  void init_side(side& s, Input_To_Hidden_Layer<dType>& in, std::vector<Hidden_To_Hidden_Layer<dType>>& hid, int V) {
    const size_t n = (size_t)H * mb, nT = n * longest;
    for (int l = 0; l < L; l++) {
      const dType *M[4], *Wh[4];
      if (l == 0) gate_ptrs(in, M, Wh); else gate_ptrs(hid[l - 1], M, Wh);
      zr_lstm_train* t = nullptr;
      ZOPH_CALL(zr_lstm_train_create(ctx, M, Wh, H, &t));
      s.train.push_back(t);
      s.h_all.push_back(dmalloc<dType>(nT));
      s.c_all.push_back(dmalloc<dType>(nT));
      s.g_all.push_back(dmalloc<dType>(4 * nT));
      s.dg_all.push_back(dmalloc<dType>(4 * nT));
      s.eh0.push_back(dmalloc<dType>(n));
      s.ec0.push_back(dmalloc<dType>(n));
      s.dM.push_back(dmalloc<dType>(4 * (size_t)H * H));
      s.dWh.push_back(dmalloc<dType>(4 * (size_t)H * H));
      s.db.push_back(dmalloc<dType>(4 * (size_t)H));
    }
    s.below0 = dmalloc<dType>(nT);
    s.x_all = dmalloc<dType>(nT);
    s.dW = dmalloc<dType>((size_t)H * V);
    s.d_ids = dmalloc<int>((size_t)mb * longest);
    s.d_nn = dmalloc<int>((size_t)mb * longest);
    s.d_mask = dmalloc<int>((size_t)mb * longest);
  }

  explicit model_trainer(forward_model<dType>& model) : m(model), ctx(model.gpu.ctx) {
    node_level = m.params.attent_params.attention_model || m.params.dropout;
    H = m.info.LSTM_size;
    L = m.info.num_layers;
    mb = m.params.minibatch_size;
    longest = m.params.longest_sent;
    Vs = m.info.source_vocab_size;
    Vt = m.info.target_vocab_size;
    seq2seq = !m.info.LM;
    if (node_level) return;
    if ((long long)mb * longest > 65535) {
      std::fprintf(stderr, "model_trainer: minibatch_size * longest_sent must not exceed 65535\n");
      std::exit(EXIT_FAILURE);
    }
    if (seq2seq) init_side(src, m.input_layer_source, m.source_hidden_layers, Vs);
    init_side(tgt, m.input_layer_target, m.target_hidden_layers, Vt);
    const size_t n = (size_t)H * mb;
    zeros = dmalloc<dType>(n);
    ZOPH_CALL(zr_memset_zero(ctx, zeros, n * sizeof(dType)));
    err_top = dmalloc<dType>(n * longest);
    prob = dmalloc<dType>((size_t)Vt * mb * longest);
    dD = dmalloc<dType>((size_t)Vt * H);
    dbd = dmalloc<dType>(Vt);
    for (auto& u : unst) u = dmalloc<dType>((size_t)H * H);
    d_tout = dmalloc<int>((size_t)mb * longest);
    d_tmask = dmalloc<int>((size_t)mb * longest);
    d_tmaskf = dmalloc<float>((size_t)mb * longest);
  }

  void forward_side(side& s, Input_To_Hidden_Layer<dType>& in, std::vector<Hidden_To_Hidden_Layer<dType>>& hid,
                    const int* h_ids, int T, int V, const std::vector<const dType*>& h0, const std::vector<const dType*>& c0) {
    ZOPH_CALL(zr_h2d(ctx, s.d_ids, h_ids, (size_t)T * mb * sizeof(int)));
    ZOPH_CALL(zr_vocab_prep(ctx, s.d_ids, T * mb, V, s.d_nn, s.d_mask));
    std::vector<const zr_lstm_weights*> w;
    if (!in.packed) in.repack();
    w.push_back(in.packed);
    for (auto& l : hid) {
      if (!l.packed) l.repack();
      w.push_back(l.packed);
    }
    ZOPH_CALL(zr_lstm_stack_forward_train(ctx, L, w.data(), in.d_W, V, s.d_nn, s.d_mask, T, mb, h0.data(), c0.data(),
                                          BZ_CUDA::clip_cell ? BZ_CUDA::cell_clip_threshold : 0.0f, s.h_all.data(),
                                          s.c_all.data(), s.g_all.data()));
  }

  template <typename LayerT>
  void update_layer(LayerT& ly, side& s, int l, float scale, float norm_clip, float lr) {
    const size_t hh = (size_t)H * H;
    dType* M[4] = {ly.d_M_i, ly.d_M_f, ly.d_M_c, ly.d_M_o};
    dType* Wh[4] = {ly.d_W_hi, ly.d_W_hf, ly.d_W_hc, ly.d_W_ho};
    dType* b[4] = {ly.d_b_i, ly.d_b_f, ly.d_b_c, ly.d_b_o};
    ZOPH_CALL(zr_unstack_gates(ctx, s.dM[l], H, unst));
    for (int g = 0; g < 4; g++) BZ_CUDA::apply_update(ctx, M[g], unst[g], (long long)hh, scale, norm_clip, norm_clip, lr);
    ZOPH_CALL(zr_unstack_gates(ctx, s.dWh[l], H, unst));
    for (int g = 0; g < 4; g++) BZ_CUDA::apply_update(ctx, Wh[g], unst[g], (long long)hh, scale, norm_clip, norm_clip, lr);
    for (int g = 0; g < 4; g++)
      BZ_CUDA::apply_update(ctx, b[g], s.db[l] + (size_t)g * H, H, scale, norm_clip, norm_clip, lr);
    ly.repack();
    const dType *Mc[4], *Whc[4];
    gate_ptrs(ly, Mc, Whc);
    ZOPH_CALL(zr_lstm_train_refresh(ctx, s.train[l], Mc, Whc));
  }

  void backward_side(side& s, Input_To_Hidden_Layer<dType>& in, std::vector<Hidden_To_Hidden_Layer<dType>>& hid, int T,
                     int V, const std::vector<const dType*>& h0, const std::vector<const dType*>& c0, const dType* top,
                     const std::vector<const dType*>* ehT, const std::vector<const dType*>* ecT) {
    std::vector<const dType*> c_all(s.c_all.begin(), s.c_all.end()), g_all(s.g_all.begin(), s.g_all.end());
    // with BZ_CUDA::clip_cell the back-propagated errors are clamped as the node classes clamp them
    ZOPH_CALL(zr_lstm_stack_backward_clamped(ctx, L, s.train.data(), T, mb, s.d_mask, c0.data(), c_all.data(), g_all.data(),
                                             top, ehT ? ehT->data() : nullptr, ecT ? ecT->data() : nullptr,
                                             s.dg_all.data(), s.below0, s.eh0.data(), s.ec0.data(),
                                             BZ_CUDA::clip_cell ? BZ_CUDA::error_clip_threshold : 0.0f));
    ZOPH_CALL(zr_embed_gather(ctx, in.d_W, H, V, s.d_nn, T * mb, s.x_all));
    for (int l = 0; l < L; l++)
      ZOPH_CALL(zr_lstm_weight_gradients(ctx, H, T, mb, s.dg_all[l], l == 0 ? s.x_all : s.h_all[l - 1], h0[l],
                                         s.h_all[l], s.dM[l], s.dWh[l], s.db[l]));
    ZOPH_CALL(zr_memset_zero(ctx, s.dW, (size_t)H * V * sizeof(dType)));
    ZOPH_CALL(zr_embed_gradient(ctx, H, V, s.below0, s.d_nn, s.d_mask, T * mb, s.dW));
  }

  bool node_level = false;    // attention or dropout: the step runs through forward_model::compute_gradients
  int lstm_sweep_option = 0;  // the context's ZR_OPT_LSTM_SWEEP setting, restored after a repeated forward pass
  int abandoned_sweeps = 0;   // forward passes that had to be repeated (see train_minibatch)

  // Forward, backward and update on the minibatch the reader holds.  Returns the minibatch's log-likelihood (natural
  // log) under the weights BEFORE the update.
  double train_minibatch(minibatch_reader& r, float learning_rate, float norm_clip) {
    if (node_level) {
      m.set_training_rates(learning_rate, norm_clip);
      const double ll = m.getError(r);
      m.compute_gradients(r);
      return ll;
    }
    const int S = seq2seq ? r.current_source_length : 0, T = r.current_target_length;
    const size_t n = (size_t)H * mb;
    std::vector<const dType*> z(L, zeros);
    std::vector<const dType*> th0 = z, tc0 = z;
    auto& sm = m.softmax_obj;
    double loss = 0;  // from the same probabilities the error is formed from (train_perplexity_kernel)
    auto forward_and_loss = [&]() {
      if (seq2seq) {
        forward_side(src, m.input_layer_source, m.source_hidden_layers, r.h_input_vocab_indicies_source.data(), S, Vs, z, z);
        for (int l = 0; l < L; l++) {  // the decoder starts from the encoder's last state (src/model.hpp:1714-1724)
          th0[l] = src.h_all[l] + (size_t)(S - 1) * n;
          tc0[l] = src.c_all[l] + (size_t)(S - 1) * n;
        }
      }
      forward_side(tgt, m.input_layer_target, m.target_hidden_layers, r.h_input_vocab_indicies_target.data(), T, Vt, th0, tc0);
      // loss layer over all T * mb columns at once
      ZOPH_CALL(zr_h2d(ctx, d_tout, r.h_output_vocab_indicies_target.data(), (size_t)T * mb * sizeof(int)));
      ZOPH_CALL(zr_vocab_prep_softmax(ctx, d_tout, T * mb, Vt, d_tmask, d_tmaskf));
      ZOPH_CALL(zr_softmax_backward_loss(ctx, sm.d_D, sm.d_b_d, Vt, H, tgt.h_all[L - 1], T * mb, d_tout, d_tmask, prob,
                                         err_top, dD, dbd, &loss));
    };
    forward_and_loss();
    // A single-launch forward sweep that gave up a wait (another process or stream holding compute units) leaves NaN
    // in its outputs; nothing of it may reach the weights.  The loss call above has already waited for the stream, so
    // the look costs one small copy.  Run the forward pass again with one launch per diagonal, which cannot stall.
    int gave_up = 0;
    ZOPH_CALL(zr_ctx_query(ctx, ZR_QUERY_LSTM_SWEEP_ABANDONED, &gave_up));
    if (gave_up) {
      ++abandoned_sweeps;
      ZOPH_CALL(zr_ctx_set_option(ctx, ZR_OPT_LSTM_SWEEP, 1));
      forward_and_loss();
      ZOPH_CALL(zr_ctx_set_option(ctx, ZR_OPT_LSTM_SWEEP, lstm_sweep_option));
    }
    backward_side(tgt, m.input_layer_target, m.target_hidden_layers, T, Vt, th0, tc0, err_top, nullptr, nullptr);
    if (seq2seq) {
      // no attention: the encoder receives error only through its final states
      ZOPH_CALL(zr_memset_zero(ctx, err_top, (size_t)S * n * sizeof(dType)));
      std::vector<const dType*> ehT(tgt.eh0.begin(), tgt.eh0.end()), ecT(tgt.ec0.begin(), tgt.ec0.end());
      backward_side(src, m.input_layer_source, m.source_hidden_layers, S, Vs, z, z, err_top, &ehT, &ecT);
    }
    // update_weights (src/model.hpp:1845-1955) under the clipping mode BZ_CUDA names: norm_clip per matrix, or over the
    // whole model (the squared norms of all gradients are summed on the device first), or a clamp per element
    const float scale = 1.0f / (float)mb;
    if (BZ_CUDA::global_clip_flag && !BZ_CUDA::individual_grad_clip) {
      BZ_CUDA::reset_global_norm(ctx);
      BZ_CUDA::add_to_global_norm(ctx, dD, (long long)Vt * H, scale);
      BZ_CUDA::add_to_global_norm(ctx, dbd, Vt, scale);
      auto norm_side = [&](side& s, int V) {
        BZ_CUDA::add_to_global_norm(ctx, s.dW, (long long)H * V, scale);
        for (int l = 0; l < L; l++) {
          BZ_CUDA::add_to_global_norm(ctx, s.dM[l], 4LL * H * H, scale);
          BZ_CUDA::add_to_global_norm(ctx, s.dWh[l], 4LL * H * H, scale);
          BZ_CUDA::add_to_global_norm(ctx, s.db[l], 4LL * H, scale);
        }
      };
      norm_side(tgt, Vt);
      if (seq2seq) norm_side(src, Vs);
    }
    BZ_CUDA::apply_update(ctx, sm.d_D, dD, (long long)Vt * H, scale, norm_clip, norm_clip, learning_rate);
    BZ_CUDA::apply_update(ctx, sm.d_b_d, dbd, Vt, scale, norm_clip, norm_clip, learning_rate);
    sm.prepare_weights();
    auto update_side = [&](side& s, Input_To_Hidden_Layer<dType>& in, std::vector<Hidden_To_Hidden_Layer<dType>>& hid, int V) {
      BZ_CUDA::apply_update(ctx, in.d_W, s.dW, (long long)H * V, scale, norm_clip, norm_clip, learning_rate);
      update_layer(in, s, 0, scale, norm_clip, learning_rate);
      for (int l = 1; l < L; l++) update_layer(hid[l - 1], s, l, scale, norm_clip, learning_rate);
    };
    update_side(tgt, m.input_layer_target, m.target_hidden_layers, Vt);
    if (seq2seq) update_side(src, m.input_layer_source, m.source_hidden_layers, Vs);
    return loss;
  }
};

// ------------------------------------------------------------------------------------------------ beam decoding
// Batched beam-search decode on top of a loaded forward_model: what ensemble_factory::decode_file_batch
// (src/ensemble_factory.hpp:583-765) does with decoder_model_wrapper::forward_prop_source / forward_prop_target /
// swap_decoding_states (src/decoder_model_wrapper.hpp, src/model.hpp:2367-2726) and decoder<dType>
// (src/decoder.h:1158-1413), for n_sent sentences of equal source length side by side.  Columns
// [s*beam, (s+1)*beam) of every LSTM_size x (n_sent*beam) activation belong to sentence s; the logits feed the
// device-side beam directly (it normalises the entries it selects), so nothing vocabulary-sized is copied to the host.  As in the reference's decode path
// every column runs with mask 1 and a dead beam slot (-1) is fed as word 0.
struct decoded_hypothesis {
  std::vector<int> words;    // target ids, <START> ... <EOF>
  std::vector<int> viterbi;  // with BZ_CUDA::unk_replacement: one source position per word (entry 0 is -20)
  float score = 0;
};

template <typename dType>
class beam_decoder {
 public:
  forward_model<dType>& m;
  zr_ctx* ctx;
  int beam, n_sent, cols, longest_sent, D, H, L, Vs, Vt;
  double penalty, min_decoding_ratio = 0.5, max_decoding_ratio = 1.5;
  bool attention, feed_input;
  zr_attn* attn = nullptr;
  zr_beam* bm = nullptr;
  std::vector<dType*> tables;                 // longest_sent source top-layer states, H x cols
  std::vector<dType*> h[2], c[2];             // ping-pong: previous / new state per layer
  dType *h_tild[2] = {nullptr, nullptr}, *x = nullptr, *logits = nullptr, *zeros = nullptr;
  std::vector<dType*> enc_h, enc_c;           // encoder sweep outputs per layer, longest_sent * H * n_sent
  int *d_words = nullptr, *d_words_nn = nullptr, *d_back = nullptr, *d_ones = nullptr, *d_batch_info = nullptr,
      *d_src = nullptr, *d_src_nn = nullptr, *d_src_mask = nullptr, *d_rep = nullptr;
  // unk replacement (BZ_CUDA::unk_replacement, attention models): the attention step's alignment weights and source
  // indices of every column, and the Viterbi alignment taken from them (src/attention_node.hpp:225-234)
  dType* d_align = nullptr;
  int *d_align_idx = nullptr, *d_viterbi = nullptr;
  bool track_viterbi = false;
  std::vector<const zr_lstm_weights*> src_w, tgt_w;
  int abandoned_launches = 0;  // batches decoded a second time because a single-launch sweep or step gave up a wait

  template <typename T>
  T* dmalloc(size_t n) {
    T* p = nullptr;
    ZOPH_CALL(zr_malloc(ctx, n * sizeof(T), (void**)&p));
    return p;
  }

  beam_decoder(forward_model<dType>& model, int beam, int n_sent, int longest_sent, int attention_D, double penalty)
      : m(model), ctx(model.gpu.ctx), beam(beam), n_sent(n_sent), cols(beam * n_sent), longest_sent(longest_sent),
        D(attention_D), penalty(penalty) {
    // "to make sure beam search does halt": the beam is silently capped at floor(sqrt(target vocabulary))
    // (src/ensemble_factory.hpp:19-21)
    {
      const int cap = std::max(1, (int)std::sqrt((double)m.info.target_vocab_size));
      if (this->beam > cap) {
        this->beam = cap;
        cols = this->beam * n_sent;
      }
      beam = this->beam;
    }
    if (m.info.LM) {
      std::fprintf(stderr, "beam_decoder: a sequence model has no source side to decode from\n");
      std::exit(EXIT_FAILURE);
    }
    H = m.info.LSTM_size;
    L = m.info.num_layers;
    Vs = m.info.source_vocab_size;
    Vt = m.info.target_vocab_size;
    attention = m.params.attent_params.attention_model;
    feed_input = m.params.attent_params.feed_input;
    m.input_layer_source.repack();
    m.input_layer_target.repack();
    src_w.push_back(m.input_layer_source.packed);
    tgt_w.push_back(m.input_layer_target.packed);
    for (int l = 0; l + 1 < L; l++) {
      m.source_hidden_layers[l].repack();
      m.target_hidden_layers[l].repack();
      src_w.push_back(m.source_hidden_layers[l].packed);
      tgt_w.push_back(m.target_hidden_layers[l].packed);
    }
    const size_t n = (size_t)H * cols;
    for (int i = 0; i < 2; i++) {
      for (int l = 0; l < L; l++) {
        h[i].push_back(dmalloc<dType>(n));
        c[i].push_back(dmalloc<dType>(n));
      }
      h_tild[i] = dmalloc<dType>(n);
    }
    x = dmalloc<dType>(n);
    // logits, then the output product's (max, sum exp) pair per 32-row block and column (ZR_SOFTMAX_LOGITS_BLOCKS): the
    // beam folds the pairs, reads only the blocks that can hold one of a column's beam + 1 largest entries and
    // normalises only what it selects (a member of an ensemble writes V x cols probabilities there instead)
    logits = dmalloc<dType>((size_t)zr_softmax_blocks_offset(Vt, cols) + 2 * (size_t)zr_softmax_block_count(Vt) * cols);
    zeros = dmalloc<dType>((size_t)H * n_sent);
    ZOPH_CALL(zr_memset_zero(ctx, zeros, (size_t)H * n_sent * sizeof(dType)));
    for (int l = 0; l < L; l++) {
      enc_h.push_back(dmalloc<dType>((size_t)longest_sent * H * n_sent));
      enc_c.push_back(dmalloc<dType>((size_t)longest_sent * H * n_sent));
    }
    d_words = dmalloc<int>(cols);
    d_words_nn = dmalloc<int>(cols);
    d_back = dmalloc<int>(cols);
    d_ones = dmalloc<int>(cols);
    d_batch_info = dmalloc<int>(2 * (size_t)cols);
    d_src = dmalloc<int>((size_t)longest_sent * n_sent);
    d_src_nn = dmalloc<int>((size_t)longest_sent * n_sent);
    d_src_mask = dmalloc<int>((size_t)longest_sent * n_sent);
    d_rep = dmalloc<int>(cols);
    std::vector<int> ones(cols, 1), rep(cols);
    for (int i = 0; i < cols; i++) rep[i] = i / beam;
    ZOPH_CALL(zr_h2d(ctx, d_ones, ones.data(), cols * sizeof(int)));
    ZOPH_CALL(zr_h2d(ctx, d_rep, rep.data(), cols * sizeof(int)));
    if (attention) {
      std::vector<const dType*> tp;
      for (int t = 0; t < longest_sent; t++) {
        tables.push_back(dmalloc<dType>(n));
        tp.push_back(tables.back());
      }
      auto* a = m.att;
      ZOPH_CALL(zr_attn_create(ctx, H, cols, D, a->d_W_a, a->d_W_p, a->d_v_p, a->d_output_bias, a->d_W_c_p1,
                               a->d_W_c_p2, tp.data(), longest_sent, &attn));
      if (BZ_CUDA::bf16_weights)
        ZOPH_CALL(zr_attn_use_bf16_weights(ctx, attn));
      else
        ZOPH_CALL(zr_attn_prepare(ctx, attn));
    }
    ZOPH_CALL(zr_beam_create(ctx, beam, Vt, n_sent, longest_sent + 3, (float)penalty, &bm));
    ZOPH_CALL(zr_beam_set_input_ids(ctx, bm, d_words_nn));
    track_viterbi = BZ_CUDA::unk_replacement && attention;
    if (track_viterbi) {
      const size_t W = 2 * (size_t)D + 1;
      d_align = dmalloc<dType>(W * cols);
      d_align_idx = dmalloc<int>(W * cols);
      d_viterbi = dmalloc<int>(cols);
      ZOPH_CALL(zr_beam_set_viterbi(ctx, bm, 1, d_viterbi));
    }
  }

  // An ensemble member hands its output distribution on as probabilities (they are averaged over the models before the
  // beam sees them); a decoder on its own leaves logits and their per-block pairs for the beam to select from and normalise what it picks.
  bool prob_mode = false;

  // forward_prop_target (src/model.hpp:2573-2688): state half p -> half q, logits and their per-block pairs into logits
  void forward_target(int p, int step_index) {
    const int q = 1 - p;
    // (d_words_nn, the input ids, are written by the beam call that chose the words: zr_beam_set_input_ids)
    // the whole step in one call: all LSTM layers (layer 0 looks its input columns up in the embedding itself), the
    // attention step on the top layer's h_t, the output distribution of h~
    const dType* feed = (feed_input && step_index > 0) ? h_tild[p] : nullptr;
    std::vector<const dType*> hp(h[p].begin(), h[p].end()), cp(c[p].begin(), c[p].end());
    ZOPH_CALL(zr_decoder_step(ctx, L, tgt_w.data(), m.input_layer_target.d_W, Vt, d_words_nn, hp.data(), cp.data(), feed,
                              d_ones, 0.0f, cols, h[q].data(), c[q].data(), attention ? attn : nullptr, d_batch_info,
                              attention ? h_tild[q] : nullptr, d_align, d_align_idx, nullptr, nullptr, m.softmax_obj.d_D,
                              m.softmax_obj.d_b_d, Vt, prob_mode ? ZR_SOFTMAX_PROB : ZR_SOFTMAX_LOGITS_BLOCKS, logits));
    // The alignment of every column, read by the beam call that follows.  The reference's driver passes every step
    // through ensembles_models, also with one model, and that overwrites the attention layer's own Viterbi alignment
    // (get_viterbi_alignment_kernel) with the vote over the window weights (src/ensemble_factory.hpp:797-834): the same
    // position wherever a weight is positive, -1 instead of the first slot's position where none is.  A member of an
    // ensemble leaves this to the ensemble's vote.
    if (track_viterbi && !prob_mode) {
      const dType* al[1] = {d_align};
      const int* ix[1] = {d_align_idx};
      ZOPH_CALL(zr_attn_viterbi_ensemble(ctx, 1, al, ix, 2 * D + 1, cols, longest_sent, d_viterbi));
    }
  }

  // forward_prop_source (src/model.hpp:2367-2452) for up to n_sent sentences whose integerized sources (reversed, no
  // padding) all have the same length: the encoder sweep, every sentence's states replicated over its beam columns,
  // <START> in every column.  Returns the source length.
  int encode(const std::vector<std::vector<int>>& sources) {
    const int real = (int)sources.size();
    const int S = real > 0 ? (int)sources[0].size() : 0;
    if (real < 1 || real > n_sent || S < 1 || S > longest_sent) {
      std::fprintf(stderr, "beam_decoder::decode_batch: %d sentences of source length %d do not fit\n", real, S);
      std::exit(EXIT_FAILURE);
    }
    // time-major ids; a short batch is completed with copies of its first sentence (results ignored)
    std::vector<int> ids((size_t)S * n_sent);
    for (int s = 0; s < n_sent; s++) {
      const auto& src = sources[s < real ? s : 0];
      if ((int)src.size() != S) {
        std::fprintf(stderr, "beam_decoder::decode_batch: sentences of one batch must have one source length\n");
        std::exit(EXIT_FAILURE);
      }
      for (int t = 0; t < S; t++) ids[s + (size_t)t * n_sent] = src[t];
    }
    ZOPH_CALL(zr_h2d(ctx, d_src, ids.data(), ids.size() * sizeof(int)));
    ZOPH_CALL(zr_vocab_prep(ctx, d_src, (int)ids.size(), Vs, d_src_nn, d_src_mask));
    std::vector<const dType*> z(L, zeros);
    ZOPH_CALL(zr_lstm_stack_forward(ctx, L, src_w.data(), m.input_layer_source.d_W, Vs, d_src_nn, d_src_mask, S, n_sent,
                                    z.data(), z.data(), 0.0f, enc_h.data(), enc_c.data()));
    // every sentence's states replicated over its beam columns (forward_prop_source, src/model.hpp:2394-2445, and
    // transfer_decoding_states_GPU for the final state of each layer)
    const size_t hn = (size_t)H * n_sent;
    if (attention)
      for (int t = 0; t < S; t++) ZOPH_CALL(zr_gather_columns(ctx, enc_h[L - 1] + t * hn, H, d_rep, cols, tables[t]));
    for (int l = 0; l < L; l++) {
      ZOPH_CALL(zr_gather_columns(ctx, enc_h[l] + (S - 1) * hn, H, d_rep, cols, h[0][l]));
      ZOPH_CALL(zr_gather_columns(ctx, enc_c[l] + (S - 1) * hn, H, d_rep, cols, c[0][l]));
    }
    std::vector<int> binfo(2 * (size_t)cols);
    for (int i = 0; i < cols; i++) {
      binfo[i] = S;  // unpadded sources of equal length: full length, no offset
      binfo[i + cols] = 0;
    }
    ZOPH_CALL(zr_h2d(ctx, d_batch_info, binfo.data(), binfo.size() * sizeof(int)));
    std::vector<int> start(cols, 0);  // <START>
    ZOPH_CALL(zr_h2d(ctx, d_words, start.data(), cols * sizeof(int)));
    ZOPH_CALL(zr_h2d(ctx, d_words_nn, start.data(), cols * sizeof(int)));
    return S;
  }

  // swap_decoding_states + target_copy_prev_states (src/model.hpp:2691-2726): the new states (half 1 - p), reordered by
  // the beam's back-pointers, become the previous states (half p) of the next step
  void reorder_states(int p, const int* d_backptr) {
    const int q = 1 - p;
    std::vector<const dType*> from(h[q].begin(), h[q].end());
    from.insert(from.end(), c[q].begin(), c[q].end());
    std::vector<dType*> to(h[p].begin(), h[p].end());
    to.insert(to.end(), c[p].begin(), c[p].end());
    if (attention) {
      from.push_back(h_tild[q]);
      to.push_back(h_tild[p]);
    }
    ZOPH_CALL(zr_gather_columns_multi(ctx, (int)from.size(), from.data(), H, d_backptr, cols, cols, to.data()));
  }

  int decode_steps(int S) const { return std::min((int)(max_decoding_ratio * S), longest_sent - 2); }

  // True when a single-launch encoder sweep or decoder step gave up a wait (its outputs hold NaN): every later launch of
  // this context then goes out one per node, and the caller decodes the batch again.
  bool launches_abandoned() {
    int abandoned = 0;
    ZOPH_CALL(zr_ctx_query(ctx, ZR_QUERY_LSTM_SWEEP_ABANDONED, &abandoned));
    if (!abandoned) return false;
    abandoned_launches++;
    ZOPH_CALL(zr_ctx_set_option(ctx, ZR_OPT_LSTM_SWEEP, 1));
    return true;
  }

  // output_k_best_hypotheses (src/decoder.h:1386-1413) for the first `real` sentences of beam object b: length ratio
  // filter, then the num_best best scores, best first
  void collect(zr_beam* b, int real, int S, int steps, int num_best, std::vector<std::vector<decoded_hypothesis>>& out) {
    out.assign(real, {});
    const int cap = 4 * beam * (steps + 2), max_len = longest_sent + 3;
    std::vector<int> words((size_t)cap * max_len), lens(cap), vit(track_viterbi ? (size_t)cap * max_len : 0);
    std::vector<float> scores(cap);
    for (int s = 0; s < real; s++) {
      int n = zr_beam_hypotheses(ctx, b, s, cap, words.data(), lens.data(), scores.data());
      if (n >= 0 && track_viterbi) n = std::min(n, zr_beam_hypotheses_viterbi(ctx, b, s, cap, vit.data()));
      if (n < 0) {
        std::fprintf(stderr, "zr_beam_hypotheses failed: %s\n", zr_last_error());
        std::exit(EXIT_FAILURE);
      }
      n = std::min(n, cap);
      std::vector<int> order;
      for (int i = 0; i < n; i++)
        if ((float)lens[i] / (float)S > (float)min_decoding_ratio) order.push_back(i);
      std::stable_sort(order.begin(), order.end(), [&](int a, int b2) { return scores[a] > scores[b2]; });
      if ((int)order.size() > num_best) order.resize(num_best);
      for (int i : order) {
        decoded_hypothesis hyp;
        hyp.words.assign(words.begin() + (size_t)i * max_len, words.begin() + (size_t)i * max_len + lens[i]);
        if (track_viterbi) hyp.viterbi.assign(vit.begin() + (size_t)i * max_len, vit.begin() + (size_t)i * max_len + lens[i]);
        hyp.score = scores[i];
        out[s].push_back(hyp);
      }
    }
  }

  // Decodes up to n_sent sentences whose integerized sources (reversed, no padding) all have the same length S.
  // out[s] receives the num_best best finished hypotheses of sentence s, best first
  // (decoder::output_k_best_hypotheses, src/decoder.h:1386-1413).
  void decode_batch(const std::vector<std::vector<int>>& sources, int num_best,
                    std::vector<std::vector<decoded_hypothesis>>& out) {
    const int real = (int)sources.size();
    const int S = encode(sources);
    ZOPH_CALL(zr_beam_init(ctx, bm));
    const int steps = decode_steps(S);
    int p = 0, index = 0;
    bool again = false;
    for (; index < steps && !again; index++) {
      forward_target(p, index);
      // (a look costs a wait for the stream: after the first step, which has then run the encoder sweep and one decoder
      // step, and every 32 steps after that -- a launch that gives up takes about a second per step)
      if (index % 32 == 0 && launches_abandoned()) again = true;
      if (again) break;
      ZOPH_CALL(zr_beam_expand_blocks(ctx, bm, logits, logits + zr_softmax_blocks_offset(Vt, cols), index, d_words, d_back));
      reorder_states(p, d_back);
    }
    if (!again) {
      // one last step and forced <EOF> on every live hypothesis (src/ensemble_factory.hpp:727-743)
      forward_target(p, index);
      ZOPH_CALL(zr_beam_finish_blocks(ctx, bm, logits, logits + zr_softmax_blocks_offset(Vt, cols)));
      again = launches_abandoned();
    }
    if (again) {  // the batch is decoded again with one launch per node (launches_abandoned has switched the context over)
      decode_batch(sources, num_best, out);
      return;
    }
    ZOPH_CALL(zr_ctx_sync(ctx));
    collect(bm, real, S, steps, num_best, out);
  }
};

// Several models decoded together (ensemble_factory::decode_file_batch with more than one model,
// src/ensemble_factory.hpp:583-765): every model runs its own encoder and decoder step on its own weights and states,
// the output distributions are averaged and renormalised (ensembles_models, :767-793), ONE beam picks the words from
// the average, and every model reorders its states by that beam's back-pointers.  The members are beam_decoders over
// one context with the same beam, batch and target vocabulary; each has its own source vocabulary, so a sentence
// arrives integerized once per member.  Under unk replacement the column's alignment is the members' vote: their
// alignment weights summed per source position, the first largest sum wins (:797-834; zr_attn_viterbi_ensemble), and
// the shared beam carries that alignment.
template <typename dType>
class ensemble_beam_decoder {
 public:
  std::vector<beam_decoder<dType>*> members;
  zr_ctx* ctx;
  dType* mean = nullptr;  // V x cols: the averaged distribution

  explicit ensemble_beam_decoder(const std::vector<beam_decoder<dType>*>& mem) : members(mem), ctx(mem.at(0)->ctx) {
    auto& first = *members[0];
    for (auto* d : members) {
      if (d->ctx != ctx || d->beam != first.beam || d->n_sent != first.n_sent || d->Vt != first.Vt ||
          d->longest_sent != first.longest_sent || d->track_viterbi != first.track_viterbi ||
          (first.track_viterbi && d->D != first.D)) {
        std::fprintf(stderr, "ensemble_beam_decoder: the members must share the context, beam, batch, longest_sent and "
                     "target vocabulary size (and, under unk replacement, all have attention of one width)\n");
        std::exit(EXIT_FAILURE);
      }
      d->prob_mode = true;
    }
    ZOPH_CALL(zr_malloc(ctx, (size_t)first.Vt * first.cols * sizeof(dType), (void**)&mean));
  }

  // sources[k]: the batch's sentences integerized with member k's source vocabulary (reversed, equal lengths)
  void decode_batch(const std::vector<std::vector<std::vector<int>>>& sources, int num_best,
                    std::vector<std::vector<decoded_hypothesis>>& out) {
    auto& first = *members[0];
    const int K = (int)members.size(), real = (int)sources.at(0).size();
    int S = 0;
    for (int k = 0; k < K; k++) S = members[k]->encode(sources.at(k));
    ZOPH_CALL(zr_beam_init(ctx, first.bm));
    const int steps = first.decode_steps(S);
    std::vector<const dType*> dists(K), aligns(K);
    std::vector<const int*> align_idx(K);
    for (int k = 0; k < K; k++) {
      dists[k] = members[k]->logits;
      aligns[k] = members[k]->d_align;
      align_idx[k] = members[k]->d_align_idx;
    }
    auto step = [&](int index) {
      for (int k = 0; k < K; k++) {
        // every member is fed the words the shared beam chose
        if (k > 0) ZOPH_CALL(zr_d2d(ctx, members[k]->d_words_nn, first.d_words_nn, (size_t)first.cols * sizeof(int)));
        members[k]->forward_target(0, index);
      }
      ZOPH_CALL(zr_ensemble_average(ctx, K, dists.data(), first.Vt, first.cols, mean));
      // the beam call that follows reads first.d_viterbi: the members' vote replaces the first member's own alignment
      if (first.track_viterbi)
        ZOPH_CALL(zr_attn_viterbi_ensemble(ctx, K, aligns.data(), align_idx.data(), 2 * first.D + 1, first.cols,
                                           first.longest_sent, first.d_viterbi));
    };
    int index = 0;
    bool again = false;
    for (; index < steps; index++) {
      step(index);
      if (index % 32 == 0 && first.launches_abandoned()) {
        again = true;
        break;
      }
      ZOPH_CALL(zr_beam_expand(ctx, first.bm, mean, index, first.d_words, first.d_back));
      for (int k = 0; k < K; k++) members[k]->reorder_states(0, first.d_back);
    }
    if (!again) {
      step(index);
      ZOPH_CALL(zr_beam_finish(ctx, first.bm, mean));
      again = first.launches_abandoned();
    }
    if (again) {
      decode_batch(sources, num_best, out);
      return;
    }
    ZOPH_CALL(zr_ctx_sync(ctx));
    first.collect(first.bm, real, S, steps, num_best, out);
  }
};

#endif
