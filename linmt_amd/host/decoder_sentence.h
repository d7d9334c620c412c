// DecoderSentence (src/decoder_sentence.h:22-52, src/decoder_sentence.cu:14-391): the translation
// service's decoder.  Init reads a "param=... value=..." configuration file, the vocabularies and
// the weights of ONE model file; Process translates one tokenised sentence with beam search
// (EnsembleFactory::DecodeSentence, src/decoder.h:1780-1840, one model) and returns the words of the
// best hypothesis, optionally followed by the decoding-information fields.  The two C functions at
// the end are the ones the reference's Python server binds (src/decoder_sentence.h:94-97).
#ifndef LINMT_AMD_HOST_DECODER_SENTENCE_H_
#define LINMT_AMD_HOST_DECODER_SENTENCE_H_

#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "dispatcher.h"
#include "nmt.h"

namespace linmt {

class DecoderSentence {
 public:
  std::unordered_map<std::string, int> uno_source_mapping_word_int_;
  std::unordered_map<int, std::string> uno_target_mapping_int_word_;

  // Throws LinmtError where the reference prints a message and exits.  load_model = false stops
  // after the configuration and the vocabularies (no GPU needed): Process is then unavailable.
  bool Init(const std::string &config, bool load_model = true);
  bool Process(const std::string &input_sentence, std::string &output_sentence);

  // What Init read: the fields of GlobalConfiguration / AttentionConfiguration the path uses.
  const DecodingConfiguration &configuration() const { return configuration_; }

  // The pieces of Process, public so that they can be checked on their own (host only).
  bool ReadConfigFile(const std::string &config_file_name, std::map<std::string, std::string> &m_parameters);
  bool GeneralSettings(std::map<std::string, std::string> &m_parameters);
  bool LoadParallelVocabulary(const std::string &nmt_model_file, int &target_vocab_size);
  // ids in the order the reference hands them to its encoder: reversed
  bool IntegerizeSentence(const std::string &input_sentence, std::vector<int> &v_input_sentence_int);
  bool UnintSentence(std::string &sentence);

 private:
  DecodingConfiguration configuration_;
  int target_vocab_size_ = 0;
  bool attention_model_mode_ = false;
  std::unique_ptr<NeuralMachineTranslation> neural_;
  std::vector<std::unique_ptr<NeuralMachineTranslation>> ensemble_;  // --nmt-model files 2..n
};

}  // namespace linmt

#endif
