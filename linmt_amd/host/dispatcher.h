// Dispatcher::Tuning (src/dispatcher.cu:96-384): the training loop around
// NeuralMachineTranslation::ComputeGradients -- minibatches from a FileHelper, the three
// learning-rate schedules, dev-set perplexity at the half epoch and at the epoch's end,
// best-model dumping, words-per-second accounting.  Host logic only; the GPU work is the model's.
#ifndef LINMT_AMD_HOST_DISPATCHER_H_
#define LINMT_AMD_HOST_DISPATCHER_H_

#include <cfloat>
#include <functional>
#include <string>
#include <vector>

#include "nmt.h"

namespace linmt {

// The fields of GlobalConfiguration that Tuning reads (src/global_configuration.h:182-290), same
// names and defaults.
struct TuningConfiguration {
  std::string train_file_name_, test_file_name_;           // integerised training / dev files
  std::string output_weight_file_, best_model_file_name_;  // model files ("" = do not write)
  int epochs_number_ = 10;
  bool google_learning_rate_ = false;    // halve at the half epoch and after every epoch ...
  int epoch_to_start_halving_ = 6;       // ... from this epoch on
  bool stanford_learning_rate_ = false;  // halve after every epoch ...
  int epoch_to_start_halving_full_ = 6;  // ... from this epoch on
  bool learning_rate_schedule_ = false;  // multiply by decrease_factor_ when dev perplexity stalls
  float decrease_factor_ = 0.5f;
  double margin_ = 0.0;
  bool best_model_mode_ = false;
  double best_model_perp_ = DBL_MAX;
  int screen_print_rate_ = 20;
};

struct TuningEvent {
  enum Kind { kSpeed, kHalfEpochPerplexity, kEpochPerplexity, kLearningRate, kDumpBestModel, kEpochEnd, kDumpFinal };
  Kind kind;
  int epoch, minibatch;  // 1-based epoch, minibatches done in it
  double value;          // words/s, perplexity, new learning rate, perplexity of the dumped model, train log-lik
};

struct TuningReport {
  int minibatches = 0;
  long long words = 0;          // FileHelper::words_in_minibatch_ summed
  double seconds = 0.0;         // reading + ComputeGradients, as the reference accounts it
  float final_learning_rate = 0.f;
  std::vector<TuningEvent> events;
};

class Dispatcher {
 public:
  // `neural` must have been created for training with cfg.minibatch_size_ columns.  `log`
  // (optional) receives every event as it happens.
  static TuningReport Tuning(NeuralMachineTranslation &neural, TuningConfiguration &configuration,
                             const std::function<void(const TuningEvent &)> &log = nullptr);
};

}  // namespace linmt
#endif
