#include "input_file_preprocess.h"

#include <algorithm>
#include <fstream>
#include <sstream>

#include "hip_util.h"

namespace linmt {
namespace {
bool IsRule(const std::string &s) { return s.size() > 3 && s[0] == '=' && s[1] == '=' && s[2] == '='; }
}  // namespace

int InputFilePreprocess::IntegerizeFileDecoding(const std::string &output_weights_name,
                                                const std::string &source_file_name, int max_sent_cutoff,
                                                std::vector<std::vector<int>> *sentences,
                                                std::vector<int> *kept_lines) {
  std::ifstream weights_file(output_weights_name.c_str());
  if (!weights_file) throw LinmtError("IntegerizeFileDecoding: cannot open " + output_weights_name);
  std::string str, word;
  std::getline(weights_file, str);
  std::vector<std::string> header;
  {
    std::istringstream iss(str);
    while (iss >> word) header.push_back(word);
  }
  if (header.size() < 3) throw LinmtError("IntegerizeFileDecoding: malformed model file header");
  const int target_vocab_size = std::stoi(header[2]);
  uno_source_mapping_.clear();
  std::getline(weights_file, str);  // the first rule
  while (std::getline(weights_file, str)) {
    if (IsRule(str)) break;  // end of the source mapping
    std::istringstream iss(str);
    int index;
    if (iss >> index >> word) uno_source_mapping_[word] = index;
  }
  if (!uno_source_mapping_.count("<UNK>"))
    throw LinmtError("IntegerizeFileDecoding: the source mapping of " + output_weights_name + " has no <UNK>");
  const int unk = uno_source_mapping_["<UNK>"];

  std::ifstream source_input(source_file_name.c_str());
  if (!source_input) throw LinmtError("IntegerizeFileDecoding: cannot open " + source_file_name);
  sentences->clear();
  if (kept_lines) kept_lines->clear();
  int line = 0;
  while (std::getline(source_input, str)) {
    const size_t bar = str.find(" |||| ");
    if (bar != std::string::npos) str.resize(bar);
    std::vector<int> ids;
    std::istringstream iss(str);
    while (iss >> word) {
      auto it = uno_source_mapping_.find(word);
      ids.push_back(it == uno_source_mapping_.end() ? unk : it->second);
    }
    if (!((int)ids.size() + 1 >= max_sent_cutoff - 2)) {
      sentences->push_back(std::move(ids));
      if (kept_lines) kept_lines->push_back(line);
    }
    ++line;
  }
  return target_vocab_size;
}

void InputFilePreprocess::UnintFile(const std::string &output_weights_name, const std::string &unint_file,
                                    const std::string &output_final_name, bool sequence_to_sequence_mode,
                                    bool decoder_mode) {
  std::ifstream weights_file(output_weights_name.c_str());
  if (!weights_file) throw LinmtError("UnintFile: cannot open " + output_weights_name);
  std::string str, word;
  std::getline(weights_file, str);
  std::getline(weights_file, str);
  if (sequence_to_sequence_mode)
    while (std::getline(weights_file, str))
      if (IsRule(str)) break;
  uno_target_reverse_mapping_.clear();
  while (std::getline(weights_file, str)) {
    if (IsRule(str)) break;
    std::istringstream iss(str);
    int index;
    if (iss >> index >> word) uno_target_reverse_mapping_[index] = word;
  }

  std::ifstream unint(unint_file.c_str());
  if (!unint) throw LinmtError("UnintFile: cannot open " + unint_file);
  std::ofstream final_output(output_final_name.c_str());
  if (!final_output) throw LinmtError("UnintFile: cannot open " + output_final_name);
  while (std::getline(unint, str)) {
    if (decoder_mode && (str.empty() || str[0] == '=' || str[0] == ' ')) {
      final_output << str << "\n";
      continue;
    }
    std::istringstream iss(str);
    std::vector<int> sentence_int;
    bool other = false;
    std::string other_information;
    while (iss >> word) {
      if (other) {
        other_information += " " + word;
      } else if (word != "||||") {
        sentence_int.push_back(std::stoi(word));
      } else {
        other = true;
        other_information += " " + word;
      }
    }
    // a line that ends in a field separator keeps its trailing blank
    if (other_information.size() >= 4 &&
        other_information.compare(other_information.size() - 4, 4, "||||") == 0)
      other_information += " ";
    for (size_t i = 0; i < sentence_int.size(); ++i) {
      final_output << uno_target_reverse_mapping_[sentence_int[i]];
      if (i + 1 != sentence_int.size()) final_output << " ";
    }
    final_output << other_information << "\n";
  }
}

}  // namespace linmt
