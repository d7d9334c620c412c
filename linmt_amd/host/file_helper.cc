#include "file_helper.h"

#include <sstream>

#include "hip_util.h"

namespace linmt {
namespace {

// appends the integers of one line; returns how many
int ParseIds(const std::string &line, std::vector<int> *out, size_t *cursor, const char *what) {
  std::istringstream iss(line);
  std::string word;
  int n = 0;
  while (iss >> word) {
    if (*cursor >= out->size())
      throw LinmtError(std::string("FileHelper: a minibatch holds more ") + what +
                       " ids than minibatch_size x longest_sentence");
    (*out)[(*cursor)++] = std::stoi(word);
    ++n;
  }
  return n;
}

// The reference's in-place partition (src/file_helper.cc:322-378): ids to the left, -1 to the
// right, by swapping the leftmost -1 with the rightmost id.  Returns the number of ids.
int PartitionIdsLeft(std::vector<int> *v, int n) {
  if (n <= 0) return 0;
  int left = 0, right = n - 1;
  while (left < right) {
    if ((*v)[left] == -1) {
      if ((*v)[right] != -1) {
        std::swap((*v)[left], (*v)[right]);
        ++left;
        --right;
      } else {
        --right;
      }
      continue;
    }
    ++left;
  }
  if ((*v)[left] != -1) ++left;
  return left;
}

}  // namespace

FileHelper::FileHelper(const std::string &file_name, int minibatch_size, int longest_sentence,
                       int source_vocab_size, int target_vocab_size)
    : file_name_(file_name), minibatch_size_(minibatch_size), max_sentence_length_(longest_sentence),
      source_vocab_size_(source_vocab_size), target_vocab_size_(target_vocab_size) {
  if (minibatch_size <= 0 || longest_sentence <= 0 || target_vocab_size <= 0)
    throw LinmtError("FileHelper: minibatch_size, longest_sentence and target_vocab_size must be positive");
  input_file_.open(file_name_.c_str(), std::ifstream::in);
  if (!input_file_) throw LinmtError("FileHelper: cannot open " + file_name_);
  // GetFileStats (src/utility_cc.cc:17-58): lines, then non-pad ids of the two input lines
  std::string str, word;
  while (std::getline(input_file_, str)) ++nums_lines_in_file_;
  input_file_.clear();
  input_file_.seekg(0, std::ios::beg);
  for (int i = 0; i < nums_lines_in_file_; i += 4) {
    for (int k = 0; k < 4; ++k) {
      if (!std::getline(input_file_, str)) break;
      if (k == 1 || k == 3) continue;
      std::istringstream iss(str);
      while (iss >> word)
        if (std::stoi(word) != -1) {
          ++total_words_;
          total_target_words_ += k == 2 ? 1 : 0;
        }
    }
  }
  input_file_.clear();
  input_file_.seekg(0, std::ios::beg);

  const size_t cap = (size_t)minibatch_size * longest_sentence;
  for (std::vector<int> *v :
       {&p_host_input_vocab_indices_source_, &p_host_output_vocab_indices_source_,
        &p_host_input_vocab_indices_target_, &p_host_output_vocab_indices_target_,
        &p_host_input_vocab_indices_source_wgrad_, &p_host_input_vocab_indices_target_wgrad_,
        &source_in_tmp_, &source_out_tmp_, &target_in_tmp_, &target_out_tmp_})
    v->assign(cap, -1);
  p_host_batch_information_.assign(2 * (size_t)minibatch_size, 0);
  bitmap_source_.assign(source_vocab_size > 0 ? source_vocab_size : 2, 0);
  bitmap_target_.assign(target_vocab_size, 0);
}

bool FileHelper::ReadMinibatch() {
  bool same_epoch = true;
  size_t si = 0, so = 0, ti = 0, to = 0;
  std::string l0, l1, l2, l3;
  for (int i = 0; i < minibatch_size_; ++i) {
    if (current_line_in_file_ > nums_lines_in_file_) {
      // fewer pairs than a minibatch were left: the reference rewinds and keeps whatever the
      // buffers held (src/file_helper.cc:136-145); training files hold whole minibatches
      input_file_.clear();
      input_file_.seekg(0, std::ios::beg);
      current_line_in_file_ = 1;
      same_epoch = false;
      break;
    }
    std::getline(input_file_, l0);
    std::getline(input_file_, l1);
    std::getline(input_file_, l2);
    std::getline(input_file_, l3);
    current_source_length_ = ParseIds(l0, &source_in_tmp_, &si, "source");
    ParseIds(l1, &source_out_tmp_, &so, "source");
    current_target_length_ = ParseIds(l2, &target_in_tmp_, &ti, "target");
    ParseIds(l3, &target_out_tmp_, &to, "target");
    current_line_in_file_ += 4;
  }
  if (current_line_in_file_ > nums_lines_in_file_) {
    current_line_in_file_ = 1;
    input_file_.clear();
    input_file_.seekg(0, std::ios::beg);
    same_epoch = false;
  }

  // row-major [pair][step] -> column-major [pair + step * minibatch]
  const int B = minibatch_size_, S = current_source_length_, T = current_target_length_;
  words_in_minibatch_ = 0;
  for (int i = 0; i < B; ++i) {
    int length = 0;
    for (int j = 0; j < S; ++j) {
      const int id = source_in_tmp_[(size_t)j + (size_t)S * i];
      p_host_input_vocab_indices_source_[(size_t)i + (size_t)j * B] = id;
      p_host_output_vocab_indices_source_[(size_t)i + (size_t)j * B] =
          source_out_tmp_[(size_t)j + (size_t)S * i];
      length += id != -1 ? 1 : 0;
    }
    words_in_minibatch_ += length;
    p_host_batch_information_[i] = length;
    p_host_batch_information_[(size_t)i + B] = S - length;
  }
  for (int i = 0; i < B; ++i)
    for (int j = 0; j < T; ++j) {
      p_host_input_vocab_indices_target_[(size_t)i + (size_t)j * B] =
          target_in_tmp_[(size_t)j + (size_t)T * i];
      const int out = target_out_tmp_[(size_t)j + (size_t)T * i];
      p_host_output_vocab_indices_target_[(size_t)i + (size_t)j * B] = out;
      words_in_minibatch_ += out != -1 ? 1 : 0;
    }
  PreprocessInputWgrad();
  return same_epoch;
}

// First occurrence of every id in column-major order, then the reference's partition
// (src/file_helper.cc:276-381).
void FileHelper::PreprocessInputWgrad() {
  std::fill(bitmap_source_.begin(), bitmap_source_.end(), 0);
  std::fill(bitmap_target_.begin(), bitmap_target_.end(), 0);
  const int ns = minibatch_size_ * current_source_length_;
  for (int i = 0; i < ns; ++i) {
    const int id = p_host_input_vocab_indices_source_[i];
    if (id >= (int)bitmap_source_.size() || id < -1)
      throw LinmtError("FileHelper: source id " + std::to_string(id) + " outside the vocabulary");
    const bool first = id != -1 && !bitmap_source_[id];
    if (first) bitmap_source_[id] = 1;
    p_host_input_vocab_indices_source_wgrad_[i] = first ? id : -1;
  }
  const int nt = minibatch_size_ * current_target_length_;
  for (int i = 0; i < nt; ++i) {
    const int id = p_host_input_vocab_indices_target_[i];
    if (id >= target_vocab_size_ || id < -1)
      throw LinmtError("FileHelper: target id " + std::to_string(id) + " outside the vocabulary");
    const bool first = id != -1 && !bitmap_target_[id];
    if (first) bitmap_target_[id] = 1;
    p_host_input_vocab_indices_target_wgrad_[i] = first ? id : -1;
  }
  length_source_wgrad_ = PartitionIdsLeft(&p_host_input_vocab_indices_source_wgrad_, ns);
  length_target_wgrad_ = PartitionIdsLeft(&p_host_input_vocab_indices_target_wgrad_, nt);
}

}  // namespace linmt
