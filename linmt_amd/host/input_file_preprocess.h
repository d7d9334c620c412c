// The text side of decoding (src/input_file_preprocess.cc:1312-1581): source sentences to ids with
// the source vocabulary of a model file, decoder output ids back to words with its target
// vocabulary.  Pure host code.
#ifndef LINMT_AMD_HOST_INPUT_FILE_PREPROCESS_H_
#define LINMT_AMD_HOST_INPUT_FILE_PREPROCESS_H_

#include <string>
#include <unordered_map>
#include <vector>

namespace linmt {

class InputFilePreprocess {
 public:
  std::unordered_map<std::string, int> uno_source_mapping_;
  std::unordered_map<int, std::string> uno_target_reverse_mapping_;

  // IntegerizeFileDecoding (input_file_preprocess.cc:1312-1482).  Every line of source_file_name:
  // the text before " |||| ", split at blanks, words outside the model's source vocabulary become
  // <UNK>.  `sentences` receives the ids in READING order (the reference stores them reversed, the
  // order its encoder consumes; DecodeBatch reverses by itself).  A sentence with
  // size + 1 >= max_sent_cutoff - 2 is thrown away as the reference does: kept_lines (optional)
  // receives the 0-based input line of every sentence kept.  Returns the target vocabulary size
  // read from the model file.
  int IntegerizeFileDecoding(const std::string &output_weights_name, const std::string &source_file_name,
                             int max_sent_cutoff, std::vector<std::vector<int>> *sentences,
                             std::vector<int> *kept_lines = nullptr);
  // UnintFile (input_file_preprocess.cc:1485-1581): ids of every line of unint_file up to a
  // "||||" field become the words of the target mapping; the rest of the line is copied.
  void UnintFile(const std::string &output_weights_name, const std::string &unint_file,
                 const std::string &output_final_name, bool sequence_to_sequence_mode, bool decoder_mode);
};

}  // namespace linmt
#endif
