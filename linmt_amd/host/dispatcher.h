// Dispatcher::Tuning (src/dispatcher.cu:96-384): the training loop around
// NeuralMachineTranslation::ComputeGradients -- minibatches from a FileHelper, the three
// learning-rate schedules, dev-set perplexity at the half epoch and at the epoch's end,
// best-model dumping, words-per-second accounting.  Host logic only; the GPU work is the model's.
#ifndef LINMT_AMD_HOST_DISPATCHER_H_
#define LINMT_AMD_HOST_DISPATCHER_H_

#include <cfloat>
#include <functional>
#include <ostream>
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

// The fields of GlobalConfiguration that Decoding reads (src/global_configuration.h:228-262,298),
// same names and defaults, plus the batch size of this implementation.
struct DecodingConfiguration {
  std::string model_name_;           // the reference's text model file
  // further models of an ensemble (the reference's model_names_[1..]): the source text is
  // integerised once per model with the model's own source vocabulary; the target vocabulary and
  // the un-integerisation are the first model's
  std::vector<std::string> ensemble_model_names_;
  std::string decode_user_file_;     // source sentences, one per line, tokenised text
  std::string decoder_output_file_;  // ids of the translations ("" = decoder_final_file_ + ".ids")
  std::string decoder_final_file_;   // the translations as words
  int beam_size_ = 12;
  int hypotheses_number_ = 1;  // k-best list per sentence, closed by a line of '=' when != 1
  float penalty_ = 0.f, max_decoding_ratio_ = 1.5f, min_decoding_ratio_ = 0.5f;
  float decoding_lp_alpha_ = 0.65f, decoding_cp_beta_ = 0.20f, decoding_diversity_ = 0.f;
  int longest_sentence_ = 200;  // src/global_configuration.h:298: 100, doubled for translation
  int attention_width_ = 10;    // D of the local-p window: not stored in the model file, the
                                // reference takes it from its configuration too
  bool print_decoding_information_mode_ = false;  // " |||| score |||| alignments |||| <UNK> alignments"
  bool print_alignments_scores_mode_ = false;     // ... " |||| " alignment scores per token
  bool unk_replacement_mode_ = false;             // export alignments (what the two prints show)
  int sentences_per_batch_ = 64;  // no counterpart: the reference decodes one sentence at a time
};

struct DecodingReport {
  int sentences = 0, sentences_thrown_away = 0;
  long long source_words = 0, target_words = 0;
  double seconds = 0.0;  // decoding only (model loading and file conversion excluded)
};

// The text of one translation as the reference prints it: ids, then (print_decoding_information)
// " |||| score |||| Viterbi alignments |||| <UNK> alignments" and (print_alignments_scores)
// " |||| " the alignment scores of every token; no line end (src/decoder.h:602-681, 788-856).
// rank: which of the kept hypotheses (0 = best).
void WriteHypothesis(std::ostream &out, const SentenceResult &r, int source_length,
                     bool print_decoding_information, bool print_alignments_scores, int rank = 0);

class Dispatcher {
 public:
  // Dispatcher::Decoding (src/dispatcher.cu:387-436): model file -> decoder, source text -> ids
  // (InputFilePreprocess::IntegerizeFileDecoding), beam search (EnsembleFactory::DecodeFile with
  // one model), id output (Decoder::OutputKBestHypotheses) -> words
  // (UnintFile).
  static DecodingReport Decoding(const DecodingConfiguration &configuration);

  // `neural` must have been created for training with cfg.minibatch_size_ columns.  `log`
  // (optional) receives every event as it happens.
  static TuningReport Tuning(NeuralMachineTranslation &neural, TuningConfiguration &configuration,
                             const std::function<void(const TuningEvent &)> &log = nullptr);
};

}  // namespace linmt
#endif
