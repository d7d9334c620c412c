#include "dispatcher.h"

#include <chrono>
#include <cmath>
#include <fstream>

#include "file_helper.h"

namespace linmt {

// GetPerplexity (src/deep_rnn.h:1490-1568): one pass over an integerised file,
// 2^(-(sum of log2 p(target)) / target words of the file).
double NeuralMachineTranslation::GetPerplexity(const std::string &test_file_name) {
  FileHelper file_information(test_file_name, cfg_.minibatch_size_, cfg_.longest_sentence_,
                              cfg_.sequence_to_sequence_mode_ ? cfg_.source_vocab_size_ : -1,
                              cfg_.target_vocab_size_);
  double p_data = 0.0;
  bool success = true;
  while (success) {
    success = file_information.ReadMinibatch();
    p_data += GetError(file_information.p_host_input_vocab_indices_source_.data(),
                       file_information.current_source_length_,
                       file_information.p_host_input_vocab_indices_target_.data(),
                       file_information.p_host_output_vocab_indices_target_.data(),
                       file_information.current_target_length_,
                       file_information.p_host_batch_information_.data(), cfg_.minibatch_size_);
  }
  p_data /= std::log(2.0);
  return std::pow(2.0, -p_data / file_information.total_target_words_);
}

void NeuralMachineTranslation::UpdateLearningRate(float new_learning_rate) {
  cfg_.learning_rate_ = new_learning_rate;
}

// DumpBestModel (src/deep_rnn.h:1971-2040): header and vocabulary mappings copied from the model
// file the corpus preprocessor started, then the current matrices.
void NeuralMachineTranslation::DumpBestModel(const std::string &best_model_name,
                                             const std::string &const_model_name) {
  std::ifstream const_model(const_model_name.c_str());
  if (!const_model) {  // no file to take the mappings from: placeholder words
    DumpModel(best_model_name, nullptr, nullptr);
    return;
  }
  {
    std::ofstream best(best_model_name.c_str());
    if (!best) throw LinmtError("DumpBestModel: cannot open " + best_model_name);
    std::string str;
    std::getline(const_model, str);
    best << str << "\n";
    std::getline(const_model, str);
    best << str << "\n";
    for (int part = 0; part < (cfg_.sequence_to_sequence_mode_ ? 2 : 1); ++part)
      while (std::getline(const_model, str)) {
        best << str << "\n";
        if (str.size() > 3 && str[0] == '=' && str[1] == '=' && str[2] == '=') break;
      }
  }
  DumpWeights(best_model_name);
}

TuningReport Dispatcher::Tuning(NeuralMachineTranslation &neural, TuningConfiguration &configuration,
                                const std::function<void(const TuningEvent &)> &log) {
  using Clock = std::chrono::steady_clock;
  const GlobalConfiguration &cfg = neural.cfg_;
  TuningReport report;
  auto emit = [&](TuningEvent::Kind kind, int epoch, int minibatch, double value) {
    report.events.push_back({kind, epoch, minibatch, value});
    if (log) log(report.events.back());
  };

  FileHelper file_information(configuration.train_file_name_, cfg.minibatch_size_, cfg.longest_sentence_,
                              cfg.sequence_to_sequence_mode_ ? cfg.source_vocab_size_ : -1,
                              cfg.target_vocab_size_);
  const long long half_way_count = file_information.total_words_ / 2;

  int current_batch_num_speed = 0, current_batch_num = 0, current_epoch = 1;
  long long total_words_batch_speed = 0, total_words = 0;
  double total_batch_time_speed = 0.0;
  float tmp_learning_rate = cfg.learning_rate_;
  bool learning_rate_flag = true;
  double old_perplexity = 0.0, train_loglik = 0.0;

  // dev perplexity, the stall rule and the best-model dump: the same block at the half epoch and
  // at the epoch's end (src/dispatcher.cu:240-272 and :306-337)
  auto evaluate = [&](TuningEvent::Kind kind) {
    const double new_perplexity = neural.GetPerplexity(configuration.test_file_name_);
    emit(kind, current_epoch, current_batch_num, new_perplexity);
    if (new_perplexity + configuration.margin_ >= old_perplexity && current_epoch != 1) {
      tmp_learning_rate *= configuration.decrease_factor_;
      neural.UpdateLearningRate(tmp_learning_rate);
      emit(TuningEvent::kLearningRate, current_epoch, current_batch_num, tmp_learning_rate);
    }
    if (configuration.best_model_mode_ && configuration.best_model_perp_ > new_perplexity) {
      if (!configuration.best_model_file_name_.empty())
        neural.DumpBestModel(configuration.best_model_file_name_, configuration.output_weight_file_);
      configuration.best_model_perp_ = new_perplexity;
      emit(TuningEvent::kDumpBestModel, current_epoch, current_batch_num, new_perplexity);
    }
    old_perplexity = new_perplexity;
  };
  auto halve = [&] {
    tmp_learning_rate /= 2;
    neural.UpdateLearningRate(tmp_learning_rate);
    emit(TuningEvent::kLearningRate, current_epoch, current_batch_num, tmp_learning_rate);
  };

  while (current_epoch <= configuration.epochs_number_) {
    const auto begin_minibatch = Clock::now();
    const bool success_flag = file_information.ReadMinibatch();
    train_loglik += neural.ComputeGradients(
        file_information.p_host_input_vocab_indices_source_.data(), file_information.current_source_length_,
        file_information.p_host_input_vocab_indices_target_.data(),
        file_information.p_host_output_vocab_indices_target_.data(), file_information.current_target_length_,
        file_information.p_host_input_vocab_indices_source_wgrad_.data(), file_information.length_source_wgrad_,
        file_information.p_host_input_vocab_indices_target_wgrad_.data(), file_information.length_target_wgrad_,
        file_information.p_host_batch_information_.data(), cfg.minibatch_size_);
    neural.UpdateWeights();
    neural.Synchronize();
    const double seconds = std::chrono::duration<double>(Clock::now() - begin_minibatch).count();
    total_batch_time_speed += seconds;
    report.seconds += seconds;
    total_words_batch_speed += file_information.words_in_minibatch_;
    ++current_batch_num_speed;
    ++current_batch_num;
    ++report.minibatches;
    total_words += file_information.words_in_minibatch_;
    report.words += file_information.words_in_minibatch_;

    if (current_batch_num_speed >= configuration.screen_print_rate_ || !success_flag) {
      emit(TuningEvent::kSpeed, current_epoch, current_batch_num,
           total_words_batch_speed / std::max(total_batch_time_speed, 1e-12));
      total_words_batch_speed = 0;
      total_batch_time_speed = 0.0;
      current_batch_num_speed = 0;
    }

    if (configuration.google_learning_rate_ && current_epoch >= configuration.epoch_to_start_halving_ &&
        total_words >= half_way_count && learning_rate_flag) {
      halve();
      learning_rate_flag = false;
    }
    if (configuration.learning_rate_schedule_ && total_words >= half_way_count && learning_rate_flag) {
      learning_rate_flag = false;
      evaluate(TuningEvent::kHalfEpochPerplexity);
    }

    if (!success_flag) {
      emit(TuningEvent::kEpochEnd, current_epoch, current_batch_num, train_loglik);
      train_loglik = 0.0;
      current_epoch += 1;
      current_batch_num = 0;
      if (configuration.google_learning_rate_ && current_epoch >= configuration.epoch_to_start_halving_) {
        halve();
        learning_rate_flag = true;
      }
      if (configuration.stanford_learning_rate_ && current_epoch >= configuration.epoch_to_start_halving_full_) {
        halve();
        learning_rate_flag = true;
      }
      if (configuration.learning_rate_schedule_) {
        evaluate(TuningEvent::kEpochPerplexity);
        learning_rate_flag = true;
      }
      total_words = 0;
    }
  }
  if (!configuration.output_weight_file_.empty()) {
    // the reference appends the matrices to the file its corpus preprocessor started; without such
    // a file a complete one is written
    std::ifstream started(configuration.output_weight_file_.c_str());
    if (started) {
      started.close();
      neural.DumpWeights(configuration.output_weight_file_);
    } else {
      neural.DumpModel(configuration.output_weight_file_, nullptr, nullptr);
    }
    emit(TuningEvent::kDumpFinal, current_epoch - 1, 0, 0.0);
  }
  report.final_learning_rate = tmp_learning_rate;
  return report;
}

}  // namespace linmt
