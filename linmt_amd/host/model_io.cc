// Text model file of the reference: reader and writer.
#include <fstream>
#include <limits>
#include <sstream>

#include "nmt.h"

namespace linmt {
namespace {

const char kRule[] = "==========================================================";

bool IsRule(const std::string &line) {
  return line.size() > 3 && line[0] == '=' && line[1] == '=' && line[2] == '=';
}

// ReadMatrixGpu (src/deep_rnn_kernel.h:1543-1561): `rows` lines of `cols` numbers, then one line
// that is skipped; element (i, j) goes to column-major position i + j * rows.
void ReadMatrix(std::ifstream &in, int rows, int cols, std::vector<float> *out, const std::string &name) {
  out->assign((size_t)rows * cols, 0.f);
  std::string line, token;
  for (int i = 0; i < rows; ++i) {
    if (!std::getline(in, line)) throw LinmtError("LoadWeights: the file ends inside " + name);
    std::istringstream iss(line);
    for (int j = 0; j < cols; ++j) {
      if (!(iss >> token))
        throw LinmtError("LoadWeights: row " + std::to_string(i) + " of " + name + " has fewer than " +
                         std::to_string(cols) + " numbers");
      (*out)[(size_t)i + (size_t)j * rows] = (float)std::stod(token);
    }
  }
  std::getline(in, line);
}

// WriteMatrixGpu (src/deep_rnn_kernel.h:1564-1578)
void WriteMatrix(std::ofstream &out, int rows, int cols, const std::vector<float> &m) {
  for (int i = 0; i < rows; ++i) {
    for (int j = 0; j < cols; ++j) {
      out << m[(size_t)i + (size_t)j * rows];
      if (j != cols - 1) out << " ";
    }
    out << "\n";
  }
  out << "\n";
}

}  // namespace

ModelInformation ReadModelInformation(const std::string &model_file) {
  std::ifstream in(model_file.c_str());
  if (!in) throw LinmtError("cannot open model file " + model_file);
  std::string line;
  std::getline(in, line);
  std::istringstream iss(line);
  ModelInformation m;
  if (!(iss >> m.num_layers >> m.lstm_size >> m.target_vocab_size >> m.source_vocab_size))
    throw LinmtError("model file " + model_file + ": malformed first line");
  // older files stop after the sizes; the flags default to 0
  iss >> m.attention_model >> m.feed_input >> m.multi_source >> m.combine_lstm >> m.char_cnn;
  return m;
}

// Order of InputToHiddenLayer / HiddenToHiddenLayer::DumpWeightsGpu
// (layer_input_to_hidden.h:1556-1590, layer_hidden_to_hidden.h:989-1014: note M_o before M_c and
// Q_o before Q_c), AttentionLayer::DumpWeights (layer_attention.h:1264-1273, attached to the top
// target layer, i.e. written after every target LSTM matrix) and SoftmaxLayer::DumpWeightsGpu
// (layer_loss.h:1213-1218).
std::vector<NeuralMachineTranslation::ParamShape> NeuralMachineTranslation::ModelFileOrder() const {
  std::vector<ParamShape> v;
  const int H = cfg_.lstm_size_, E = cfg_.embedding_size_;
  auto layer = [&](const std::string &prefix, int l, int vocab, bool feed) {
    const std::string p = prefix + "." + std::to_string(l) + ".";
    const int in = l == 0 ? E : H;
    for (char g : {'i', 'f', 'c', 'o'}) {
      v.push_back({p + "W_h" + g, H, H});
      v.push_back({p + "b_" + g, H, 1});
    }
    if (l == 0) v.push_back({p + "W", E, vocab});
    for (char g : {'i', 'f', 'o', 'c'}) v.push_back({p + "M_" + g, H, in});
    if (feed)
      for (char g : {'i', 'f', 'o', 'c'}) v.push_back({p + "Q_" + g, H, H});
  };
  if (cfg_.sequence_to_sequence_mode_)
    for (int l = 0; l < cfg_.num_layers_; ++l) layer("src", l, cfg_.source_vocab_size_, false);
  for (int l = 0; l < cfg_.num_layers_; ++l)
    layer("tgt", l, cfg_.target_vocab_size_, l == 0 && cfg_.attention_mode_ && cfg_.feed_input_mode_);
  if (cfg_.attention_mode_) {
    v.push_back({"attn.W_a", H, H});
    v.push_back({"attn.W_p", H, H});
    v.push_back({"attn.v_p", H, 1});
    v.push_back({"attn.b_out", H, 1});
    v.push_back({"attn.W_c1", H, H});
    v.push_back({"attn.W_c2", H, H});
  }
  v.push_back({"softmax.D", cfg_.target_vocab_size_, H});
  v.push_back({"softmax.b_d", cfg_.target_vocab_size_, 1});
  return v;
}

void NeuralMachineTranslation::LoadWeights(const std::string &input_weight_file) {
  const ModelInformation info = ReadModelInformation(input_weight_file);
  if (info.num_layers != cfg_.num_layers_ || info.lstm_size != cfg_.lstm_size_ ||
      info.target_vocab_size != cfg_.target_vocab_size_ ||
      (cfg_.sequence_to_sequence_mode_ && info.source_vocab_size != cfg_.source_vocab_size_) ||
      (info.attention_model != 0) != (cfg_.attention_mode_ != 0) ||
      (info.feed_input != 0) != (cfg_.attention_mode_ && cfg_.feed_input_mode_))
    throw LinmtError("LoadWeights: " + input_weight_file + " describes a different model (layers " +
                     std::to_string(info.num_layers) + ", lstm size " + std::to_string(info.lstm_size) +
                     ", vocabularies " + std::to_string(info.source_vocab_size) + "/" +
                     std::to_string(info.target_vocab_size) + ", attention " +
                     std::to_string(info.attention_model) + ", feed input " +
                     std::to_string(info.feed_input) + ")");
  if (info.multi_source || info.combine_lstm || info.char_cnn)
    throw LinmtError("LoadWeights: multi-source / tree-LSTM / char-CNN models are not supported");
  if (cfg_.embedding_size_ != cfg_.lstm_size_)
    throw LinmtError("LoadWeights: the reference's model file has embedding size = lstm size");
  std::ifstream in(input_weight_file.c_str());
  std::string line;
  std::getline(in, line);  // sizes
  std::getline(in, line);  // first rule
  while (std::getline(in, line))
    if (IsRule(line)) break;  // end of the source mapping
  if (cfg_.sequence_to_sequence_mode_)
    while (std::getline(in, line))
      if (IsRule(line)) break;  // end of the target mapping
  std::vector<float> m;
  for (const ParamShape &p : ModelFileOrder()) {
    ReadMatrix(in, p.rows, p.cols, &m, p.name);
    if (!SetParam(p.name, m.data(), m.size())) throw LinmtError("LoadWeights: cannot set " + p.name);
  }
  Synchronize();
}

void NeuralMachineTranslation::DumpWeights(const std::string &output_weight_file) {
  std::ofstream out(output_weight_file.c_str(), std::ios_base::app);
  if (!out) throw LinmtError("DumpWeights: cannot open " + output_weight_file);
  out.precision(std::numeric_limits<float>::digits10 + 2);
  std::vector<float> m;
  for (const ParamShape &p : ModelFileOrder()) {
    if (!GetParam(p.name, &m) || m.size() != (size_t)p.rows * p.cols)
      throw LinmtError("DumpWeights: cannot read " + p.name);
    WriteMatrix(out, p.rows, p.cols, m);
  }
}

void NeuralMachineTranslation::DumpModel(const std::string &output_weight_file,
                                         const std::vector<std::string> *source_words,
                                         const std::vector<std::string> *target_words) {
  {
    std::ofstream out(output_weight_file.c_str());
    if (!out) throw LinmtError("DumpModel: cannot open " + output_weight_file);
    const bool feed = cfg_.attention_mode_ && cfg_.feed_input_mode_;
    out << cfg_.num_layers_ << " " << cfg_.lstm_size_ << " " << cfg_.target_vocab_size_ << " "
        << (cfg_.sequence_to_sequence_mode_ ? cfg_.source_vocab_size_ : -1) << " "
        << (cfg_.attention_mode_ ? 1 : 0) << " " << (feed ? 1 : 0) << " 0 0 0\n";
    // mappings as the corpus preprocessor writes them (input_file_preprocess.cc:545-575)
    out << kRule << "\n";
    auto mapping = [&](int n, const std::vector<std::string> *words, std::initializer_list<const char *> reserved) {
      for (int i = 0; i < n; ++i) {
        out << i << " ";
        if (words && i < (int)words->size()) out << (*words)[i];
        else if (i < (int)reserved.size()) out << *(reserved.begin() + i);
        else out << "w" << i;
        out << "\n";
      }
      out << kRule << "\n";
    };
    if (cfg_.sequence_to_sequence_mode_) mapping(cfg_.source_vocab_size_, source_words, {"<UNK>"});
    mapping(cfg_.target_vocab_size_, target_words, {"<START>", "<EOF>", "<UNK>"});
  }
  DumpWeights(output_weight_file);
}

}  // namespace linmt
