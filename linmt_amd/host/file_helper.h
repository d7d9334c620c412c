// FileHelper (src/file_helper.h:28-112, src/file_helper.cc:20-381): reader of the reference's
// integerised training file.  Four lines per sentence pair, written by its corpus preprocessor
// with every pair of one minibatch already padded to common lengths:
//   source ids, reversed and LEFT-padded with -1      (input_file_preprocess.cc:633)
//   a line the source side does not use
//   target input ids  (<START> w1 .. wn), right-padded with -1
//   target output ids (w1 .. wn <EOF>),   right-padded with -1
// ReadMinibatch() turns minibatch_size_ pairs into the column-major [column + step * minibatch]
// id blocks the model takes, the batch information [length.., padding..] of the attention layer
// and the lists of distinct input ids (the columns of the embedding gradient).
// Pure host code: nothing here touches the GPU.
#ifndef LINMT_AMD_HOST_FILE_HELPER_H_
#define LINMT_AMD_HOST_FILE_HELPER_H_

#include <fstream>
#include <string>
#include <vector>

namespace linmt {

class FileHelper {
 public:
  std::string file_name_;
  int minibatch_size_ = 0;
  int current_line_in_file_ = 1;
  int nums_lines_in_file_ = 0;
  int words_in_minibatch_ = 0;  // non-pad source input + non-pad target output ids
  int max_sentence_length_ = 0;
  int current_source_length_ = 0, current_target_length_ = 0;
  int source_vocab_size_ = 0, target_vocab_size_ = 0;
  int total_words_ = 0, total_target_words_ = 0;  // non-pad ids of the whole file (GetFileStats)

  // minibatch_size_ x length, column-major
  std::vector<int> p_host_input_vocab_indices_source_, p_host_output_vocab_indices_source_;
  std::vector<int> p_host_input_vocab_indices_target_, p_host_output_vocab_indices_target_;
  // distinct non-pad input ids first, -1 after them
  std::vector<int> p_host_input_vocab_indices_source_wgrad_, p_host_input_vocab_indices_target_wgrad_;
  int length_source_wgrad_ = 0, length_target_wgrad_ = 0;
  std::vector<int> p_host_batch_information_;  // [source length per column.., left padding..]

  // source_vocab_size = -1: target-side language model (src/file_helper.cc:66-70)
  FileHelper(const std::string &file_name, int minibatch_size, int longest_sentence,
             int source_vocab_size, int target_vocab_size);
  // false when the read reached the end of the file: the next call starts the next epoch
  bool ReadMinibatch();

 private:
  void PreprocessInputWgrad();
  std::ifstream input_file_;
  std::vector<int> source_in_tmp_, source_out_tmp_, target_in_tmp_, target_out_tmp_;  // row-major
  std::vector<char> bitmap_source_, bitmap_target_;
};

}  // namespace linmt
#endif
