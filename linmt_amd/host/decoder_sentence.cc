#include "decoder_sentence.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <fstream>
#include <sstream>

namespace linmt {

namespace {

// BasicMethod::Split (src/utility_cc.cc:132-153): pieces between single characters, empty ones dropped.
std::vector<std::string> SplitAt(const std::string &text, char separator) {
  std::vector<std::string> pieces;
  std::string piece;
  std::istringstream in(text);
  while (std::getline(in, piece, separator))
    if (!piece.empty()) pieces.push_back(piece);
  return pieces;
}

// The text between the quotes that follow `tag` ("" and false when a quote is missing).
bool QuotedAfter(const std::string &line, const std::string &tag, std::string *value) {
  const std::string::size_type begin = line.find(tag);
  if (begin == std::string::npos) return false;
  const std::string::size_type first = begin + tag.size();
  const std::string::size_type last = line.find('"', first);
  if (last == std::string::npos) return false;
  *value = line.substr(first, last - first);
  return true;
}

}  // namespace

// src/decoder_sentence.cu:272-325.  Lines "param="KEY" value="VALUE""; '#' starts a comment line;
// a later line with the same key wins; lines without both fields are skipped.
bool DecoderSentence::ReadConfigFile(const std::string &config_file_name,
                                     std::map<std::string, std::string> &m_parameters) {
  std::ifstream in_config_file(config_file_name.c_str());
  if (!in_config_file) throw LinmtError("Config File " + config_file_name + " does not exist");
  std::string line;
  while (std::getline(in_config_file, line)) {
    line.erase(std::remove(line.begin(), line.end(), '\r'), line.end());
    const std::string::size_type first = line.find_first_not_of(' ');
    if (first == std::string::npos) continue;
    line = line.substr(first, line.find_last_not_of(' ') - first + 1);
    if (line[0] == '#') continue;
    std::string key, value;
    if (!QuotedAfter(line, "param=\"", &key) || !QuotedAfter(line, "value=\"", &value)) continue;
    m_parameters[key] = value;
  }
  return true;
}

// src/decoder_sentence.cu:108-269.  Keys without a meaning here are accepted and ignored:
// --tmp-dir-location (no temporary files are written), --log, --log-level.
bool DecoderSentence::GeneralSettings(std::map<std::string, std::string> &m_parameters) {
  DecodingConfiguration &c = configuration_;
  c = DecodingConfiguration();
  c.sentences_per_batch_ = 1;
  auto has = [&](const char *key) { return m_parameters.find(key) != m_parameters.end(); };

  c.longest_sentence_ = 100;  // src/global_configuration.h:298; no doubling on this path
  if (has("--longest-sent")) c.longest_sentence_ = std::atoi(m_parameters["--longest-sent"].c_str());
  c.longest_sentence_ += 4;
  if (has("--beam-size")) c.beam_size_ = std::atoi(m_parameters["--beam-size"].c_str());
  if (has("--attention-width")) c.attention_width_ = std::stoi(m_parameters["--attention-width"]);
  if (has("--print-decoding-info")) {
    c.print_decoding_information_mode_ = std::atoi(m_parameters["--print-decoding-info"].c_str()) != 0;
    if (c.print_decoding_information_mode_) c.unk_replacement_mode_ = true;
  }
  if (has("--print-align-scores"))
    c.print_alignments_scores_mode_ = std::atoi(m_parameters["--print-align-scores"].c_str()) != 0;

  if (!has("--nmt-model")) throw LinmtError("you must assign --nmt-model in config file!");
  const std::vector<std::string> model_names = SplitAt(m_parameters["--nmt-model"], ' ');
  if (model_names.empty()) throw LinmtError("you must assign --nmt-model in config file!");
  // several files: an ensemble; sentences are integerised with the first model's vocabulary
  // (src/decoder_sentence.cu:21)
  c.model_name_ = model_names[0];
  c.ensemble_model_names_.assign(model_names.begin() + 1, model_names.end());
  // --nbest is read by the reference and handed to its decoder, but a sentence always comes back
  // as its one best hypothesis (Decoder::ObtainOneBestHypothesis, src/decoder.h:703): accepted,
  // without effect
  if (has("--multi-gpu") && SplitAt(m_parameters["--multi-gpu"], ' ').size() != model_names.size())
    throw LinmtError("for decoding, each model must be specified a gpu");

  if (c.beam_size_ <= 0) throw LinmtError("--beam-size cannot be <= 0!");
  if (has("--decoding-ratio")) {
    const std::vector<std::string> ratio = SplitAt(m_parameters["--decoding-ratio"], ' ');
    if (ratio.size() != 2)
      throw LinmtError("only two inputs for --decoding-ratio, now is " + std::to_string(ratio.size()));
    // the reference converts both with integer routines ("1.0 2.0" is the shipped setting)
    c.min_decoding_ratio_ = (float)std::atoi(ratio[0].c_str());
    c.max_decoding_ratio_ = (float)std::stoi(ratio[1]);
    if (c.min_decoding_ratio_ >= c.max_decoding_ratio_)
      throw LinmtError("min decoding ratio must be less than max decoding ratio!");
  }
  if (has("--lp-alpha")) c.decoding_lp_alpha_ = (float)std::atof(m_parameters["--lp-alpha"].c_str());
  if (has("--cp-beta")) c.decoding_cp_beta_ = (float)std::atof(m_parameters["--cp-beta"].c_str());
  if (has("--diversity")) c.decoding_diversity_ = (float)std::atof(m_parameters["--diversity"].c_str());
  return true;
}

// src/decoder_sentence.cu:328-391: header line, a rule of '=', "id word" lines of the source side,
// a rule, the same for the target side, a rule.
bool DecoderSentence::LoadParallelVocabulary(const std::string &nmt_model_file, int &target_vocab_size) {
  std::ifstream in_nmt_model(nmt_model_file.c_str());
  if (!in_nmt_model) throw LinmtError("can not open " + nmt_model_file + " file!");
  target_vocab_size = ReadModelInformation(nmt_model_file).target_vocab_size;
  uno_source_mapping_word_int_.clear();
  uno_target_mapping_int_word_.clear();
  auto rule = [](const std::string &s) { return s.size() > 3 && s[0] == '=' && s[1] == '=' && s[2] == '='; };
  std::string str, word;
  std::getline(in_nmt_model, str);  // model information
  std::getline(in_nmt_model, str);  // rule
  for (int side = 0; side < 2; ++side) {
    while (std::getline(in_nmt_model, str)) {
      if (rule(str)) break;
      std::istringstream iss(str);
      int index;
      if (!(iss >> index >> word)) continue;
      if (side == 0) uno_source_mapping_word_int_[word] = index;
      else uno_target_mapping_int_word_[index] = word;
    }
    if (side == 0) std::getline(in_nmt_model, str);  // the rule that opens the target side
  }
  return true;
}

// src/decoder_sentence.cu:50-69.  A word outside the vocabulary takes the id stored under the key
// "UNK"; as in the reference a vocabulary without that key gains it with id 0, the id of <UNK>.
bool DecoderSentence::IntegerizeSentence(const std::string &input_sentence,
                                         std::vector<int> &v_input_sentence_int) {
  const std::string::size_type bar = input_sentence.find(" |||| ");
  std::istringstream iss_src(bar == std::string::npos ? input_sentence : input_sentence.substr(0, bar));
  std::string word;
  while (iss_src >> word) {
    auto it = uno_source_mapping_word_int_.find(word);
    v_input_sentence_int.push_back(it == uno_source_mapping_word_int_.end()
                                       ? uno_source_mapping_word_int_["UNK"]
                                       : it->second);
  }
  std::reverse(v_input_sentence_int.begin(), v_input_sentence_int.end());
  return true;
}

// src/decoder_sentence.cu:71-105: ids up to the first "||||" become words, the rest is kept.
bool DecoderSentence::UnintSentence(std::string &sentence) {
  std::istringstream iss(sentence);
  std::vector<int> sentence_int;
  std::string other_information, word;
  bool other_information_flag = false;
  while (iss >> word) {
    if (other_information_flag) other_information += " " + word;
    else if ("||||" != word) sentence_int.push_back(std::stoi(word));
    else {
      other_information_flag = true;
      other_information += " " + word;
    }
  }
  const size_t n = other_information.size();
  if (n >= 4 && other_information.compare(n - 4, 4, "||||") == 0) other_information += " ";
  sentence.clear();
  for (size_t i = 0; i < sentence_int.size(); ++i) {
    sentence += uno_target_mapping_int_word_[sentence_int[i]];
    if (i + 1 != sentence_int.size()) sentence += " ";
  }
  sentence += other_information;
  return true;
}

// src/decoder_sentence.cu:14-38
bool DecoderSentence::Init(const std::string &config, bool load_model) {
  std::map<std::string, std::string> m_parameters;
  ReadConfigFile(config, m_parameters);
  GeneralSettings(m_parameters);
  LoadParallelVocabulary(configuration_.model_name_, target_vocab_size_);

  std::vector<std::string> names(1, configuration_.model_name_);
  names.insert(names.end(), configuration_.ensemble_model_names_.begin(),
               configuration_.ensemble_model_names_.end());
  attention_model_mode_ = true;
  std::vector<GlobalConfiguration> configs;
  for (const std::string &name : names) {
    const ModelInformation info = ReadModelInformation(name);
    attention_model_mode_ = attention_model_mode_ && info.attention_model != 0;
    GlobalConfiguration g;
    g.num_layers_ = info.num_layers;
    g.lstm_size_ = info.lstm_size;
    g.embedding_size_ = info.lstm_size;
    g.source_vocab_size_ = info.source_vocab_size;
    g.target_vocab_size_ = info.target_vocab_size;
    g.longest_sentence_ = configuration_.longest_sentence_;
    g.attention_mode_ = info.attention_model ? 1 : 0;
    g.attention_width_ = configuration_.attention_width_;
    g.feed_input_mode_ = info.feed_input != 0;
    g.sequence_to_sequence_mode_ = true;
    if (!configs.empty() && (g.target_vocab_size_ != configs[0].target_vocab_size_ ||
                             g.source_vocab_size_ != configs[0].source_vocab_size_))
      throw LinmtError("--nmt-model: the models of an ensemble must share both vocabularies");
    configs.push_back(g);
  }
  if (!load_model) return true;
  int beam = configuration_.beam_size_;
  const int Vt = configs[0].target_vocab_size_;
  if (beam > (int)std::sqrt((double)Vt)) beam = (int)std::sqrt((double)Vt);
  ensemble_.clear();
  for (size_t k = 0; k < names.size(); ++k) {
    std::unique_ptr<NeuralMachineTranslation> m(new NeuralMachineTranslation(configs[k]));
    m->InitModelDecoding(1, beam);
    m->LoadWeights(names[k]);
    if (k == 0) neural_ = std::move(m);
    else ensemble_.push_back(std::move(m));
  }
  return true;
}

// src/decoder_sentence.cu:40-48.  A sentence without words comes back empty, and so does one that
// does not fit the buffers sized by --longest-sent (the reference does not check either).
bool DecoderSentence::Process(const std::string &input_sentence, std::string &output_sentence) {
  if (!neural_) throw LinmtError("DecoderSentence::Process before Init");
  std::vector<int> v_input_sentence_int;
  IntegerizeSentence(input_sentence, v_input_sentence_int);
  output_sentence.clear();
  const int source_length = (int)v_input_sentence_int.size();
  if (source_length == 0 || source_length > configuration_.longest_sentence_) return true;

  const DecodingConfiguration &c = configuration_;
  DecodeOptions o;
  o.beam_size_ = c.beam_size_;
  o.max_decoding_ratio_ = c.max_decoding_ratio_;
  o.min_decoding_ratio_ = c.min_decoding_ratio_;
  o.penalty_ = c.penalty_;
  o.diversity_ = c.decoding_diversity_;
  o.lp_alpha_ = c.decoding_lp_alpha_;
  o.cp_beta_ = c.decoding_cp_beta_;
  o.unk_replacement_mode_ = c.unk_replacement_mode_ && attention_model_mode_;

  // DecodeBatch takes reading order and reverses by itself
  std::vector<std::vector<int>> batch(1, std::vector<int>(v_input_sentence_int.rbegin(), v_input_sentence_int.rend()));
  std::vector<SentenceResult> results;
  std::vector<NeuralMachineTranslation *> others;
  for (auto &m : ensemble_) others.push_back(m.get());
  neural_->DecodeBatch(batch, o, &results, others);
  std::ostringstream ids;
  WriteHypothesis(ids, results[0], source_length, c.print_decoding_information_mode_,
                  c.print_alignments_scores_mode_);
  output_sentence = ids.str();
  UnintSentence(output_sentence);
  return true;
}

}  // namespace linmt
