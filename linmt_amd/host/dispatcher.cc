#include "dispatcher.h"

#include <chrono>
#include <cmath>
#include <fstream>

#include "file_helper.h"
#include "input_file_preprocess.h"

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

// One line of Decoder::OutputKBestHypotheses (src/decoder.h:609-681) without its line end;
// Decoder::ObtainOneBestHypothesis (src/decoder.h:788-856) builds the same text as a string.
void WriteHypothesis(std::ostream &out, const SentenceResult &r, int source_length,
                     bool print_decoding_information, bool print_alignments_scores, int rank) {
  if (rank < 0 || rank >= (int)r.kbest.size()) return;  // nothing passed the length filter
  const Hypothesis &h = r.hypotheses[r.kbest[rank]];
  const size_t size = h.tokens.size();
  for (size_t j = 1; j + 1 < size; ++j) out << (j > 1 ? " " : "") << h.tokens[j];
  if (print_decoding_information) {
    auto viterbi = [&](size_t j) { return h.viterbi.empty() ? -1 : h.viterbi[j]; };
    out << " |||| " << r.kbest_score[rank] << " ||||";
    for (size_t j = 1; j + 1 < size; ++j) out << " " << viterbi(j);
    if (size <= 2) out << " ";
    out << " ||||";
    int unk_number = 0;
    for (size_t j = 1; j + 1 < size; ++j)
      if (h.tokens[j] == 2) {
        ++unk_number;
        out << " " << viterbi(j);
      }
    if (0 == unk_number) out << " -1";
    if (print_alignments_scores) {
      out << " ||||";
      for (size_t j = 1; j + 1 < size; ++j) {
        out << " ";
        for (int k = 0; k < source_length; ++k) {
          if (k) out << "/";
          out << (h.alignments_scores.empty() ? 0.f : h.alignments_scores[j][k]);
        }
      }
      if (size <= 2) out << " ";
    }
  }
}

// What OutputKBestHypotheses writes for one sentence (src/decoder.h:609-696): a line per kept
// hypothesis, best first, and a rule after the list unless a single hypothesis was asked for.  A
// sentence without a hypothesis that passes the length filter writes no line in the reference;
// an empty line stands for it here, so that line k of the output is always sentence k when one
// hypothesis is asked for.
static void WriteHypothesisLines(std::ostream &out, const SentenceResult &r, int source_length,
                                 const DecodingConfiguration &c) {
  const int n = (int)r.kbest.size();
  for (int rank = 0; rank < n; ++rank) {
    WriteHypothesis(out, r, source_length, c.print_decoding_information_mode_,
                    c.print_alignments_scores_mode_, rank);
    out << "\n";
  }
  if (1 != c.hypotheses_number_) out << "================\n";
  else if (n == 0) out << "\n";
}

static GlobalConfiguration DecodingModelConfiguration(const std::string &model_name,
                                                      const DecodingConfiguration &c) {
  const ModelInformation info = ReadModelInformation(model_name);
  GlobalConfiguration g;
  g.num_layers_ = info.num_layers;
  g.lstm_size_ = info.lstm_size;
  g.embedding_size_ = info.lstm_size;
  g.source_vocab_size_ = info.source_vocab_size;
  g.target_vocab_size_ = info.target_vocab_size;
  g.longest_sentence_ = c.longest_sentence_;
  g.attention_mode_ = info.attention_model ? 1 : 0;
  g.attention_width_ = c.attention_width_;
  g.feed_input_mode_ = info.feed_input != 0;
  g.sequence_to_sequence_mode_ = true;
  return g;
}

DecodingReport Dispatcher::Decoding(const DecodingConfiguration &c) {
  DecodingReport report;
  const GlobalConfiguration g = DecodingModelConfiguration(c.model_name_, c);

  InputFilePreprocess input_helper;
  std::vector<std::vector<int>> sentences;
  std::vector<int> kept;
  input_helper.IntegerizeFileDecoding(c.model_name_, c.decode_user_file_, c.longest_sentence_, &sentences,
                                      &kept);
  {
    std::ifstream count(c.decode_user_file_.c_str());
    std::string line;
    int lines = 0;
    while (std::getline(count, line)) ++lines;
    report.sentences_thrown_away = lines - (int)sentences.size();
  }
  report.sentences = (int)sentences.size();

  int beam = c.beam_size_;
  if (beam > (int)std::sqrt((double)g.target_vocab_size_)) beam = (int)std::sqrt((double)g.target_vocab_size_);
  const int n_sent = std::max(1, std::min(c.sentences_per_batch_, (int)sentences.size()));
  NeuralMachineTranslation neural(g);
  neural.InitModelDecoding(n_sent, beam);
  neural.LoadWeights(c.model_name_);
  // the other models of an ensemble, each with its own integerised copy of the text
  std::vector<std::unique_ptr<NeuralMachineTranslation>> others;
  std::vector<NeuralMachineTranslation *> ensemble;
  std::vector<std::vector<std::vector<int>>> other_sentences;
  bool all_attention = g.attention_mode_ != 0;
  for (const std::string &name : c.ensemble_model_names_) {
    const GlobalConfiguration gk = DecodingModelConfiguration(name, c);
    if (gk.target_vocab_size_ != g.target_vocab_size_)
      throw LinmtError("Decoding: the models of an ensemble must share the target vocabulary");
    all_attention = all_attention && gk.attention_mode_ != 0;
    other_sentences.emplace_back();
    std::vector<int> kept_k;
    input_helper.IntegerizeFileDecoding(name, c.decode_user_file_, c.longest_sentence_,
                                        &other_sentences.back(), &kept_k);
    if (kept_k != kept) throw LinmtError("Decoding: the models of an ensemble keep different sentences");
    others.emplace_back(new NeuralMachineTranslation(gk));
    others.back()->InitModelDecoding(n_sent, beam);
    others.back()->LoadWeights(name);
    ensemble.push_back(others.back().get());
  }

  DecodeOptions o;
  o.beam_size_ = c.beam_size_;
  o.max_decoding_ratio_ = c.max_decoding_ratio_;
  o.min_decoding_ratio_ = c.min_decoding_ratio_;
  o.penalty_ = c.penalty_;
  o.diversity_ = c.decoding_diversity_;
  o.lp_alpha_ = c.decoding_lp_alpha_;
  o.cp_beta_ = c.decoding_cp_beta_;
  o.unk_replacement_mode_ = c.unk_replacement_mode_ && all_attention;
  o.hypotheses_number_ = std::max(1, c.hypotheses_number_);
  o.all_hypotheses_tokens_ = false;  // only the kept hypotheses are written to the file

  const std::string ids_file =
      c.decoder_output_file_.empty() ? c.decoder_final_file_ + ".ids" : c.decoder_output_file_;
  {
    std::ofstream output(ids_file.c_str());
    if (!output) throw LinmtError("Decoding: cannot open " + ids_file);
    const auto begin = std::chrono::steady_clock::now();
    // Models with local-p attention (one, or an ensemble in lockstep): the sentences go through
    // DecodeStream, a few thousand at a time, with every beam column kept busy; everything else
    // is decoded batch by batch.  (Debug().no_stream: measurement and test aid.)
    bool stream = neural.cfg_.attention_mode_ && neural.attention_layer_.ProjectedMemoryPossible() &&
                  !Debug().no_stream && (ensemble.empty() || g.target_vocab_size_ % 4 == 0);
    for (NeuralMachineTranslation *m : ensemble)
      stream = stream && m->cfg_.attention_mode_ && m->attention_layer_.ProjectedMemoryPossible();
    const size_t chunk = stream ? (size_t)n_sent * 32 : (size_t)n_sent;
    for (size_t first = 0; stream && first < sentences.size(); first += chunk) {
      std::vector<std::vector<int>> list;
      std::vector<std::vector<std::vector<int>>> other_lists(ensemble.size());
      std::vector<size_t> where;
      const size_t last = std::min(sentences.size(), first + chunk);
      for (size_t i = first; i < last; ++i)
        if (!sentences[i].empty()) {  // an empty source line cannot be encoded: it translates to an empty line
          list.push_back(sentences[i]);
          for (size_t k = 0; k < ensemble.size(); ++k) other_lists[k].push_back(other_sentences[k][i]);
          where.push_back(i - first);
        }
      std::vector<SentenceResult> results, ordered(last - first);
      if (!list.empty()) neural.DecodeStream(list, o, &results, ensemble, other_lists);
      for (size_t b = 0; b < list.size(); ++b) ordered[where[b]] = std::move(results[b]);
      for (size_t i = first; i < last; ++i) {
        WriteHypothesisLines(output, ordered[i - first], (int)sentences[i].size(), c);
        report.source_words += (long long)sentences[i].size();
        report.target_words += (long long)ordered[i - first].best.size();
      }
    }
    for (size_t first = 0; !stream && first < sentences.size(); first += n_sent) {
      // an empty source line cannot be encoded: it translates to an empty line
      std::vector<std::vector<int>> batch;
      std::vector<std::vector<std::vector<int>>> other_batches(ensemble.size());
      std::vector<size_t> where;
      const size_t last = std::min(sentences.size(), first + n_sent);
      for (size_t i = first; i < last; ++i)
        if (!sentences[i].empty()) {
          batch.push_back(sentences[i]);
          for (size_t k = 0; k < ensemble.size(); ++k) other_batches[k].push_back(other_sentences[k][i]);
          where.push_back(i - first);
        }
      std::vector<SentenceResult> results, ordered(last - first);
      if (!batch.empty()) neural.DecodeBatch(batch, o, &results, ensemble, other_batches);
      for (size_t b = 0; b < batch.size(); ++b) ordered[where[b]] = std::move(results[b]);
      for (size_t i = first; i < last; ++i) {
        WriteHypothesisLines(output, ordered[i - first], (int)sentences[i].size(), c);
        report.source_words += (long long)sentences[i].size();
        report.target_words += (long long)ordered[i - first].best.size();
      }
    }
    report.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - begin).count();
  }
  input_helper.UnintFile(c.model_name_, ids_file, c.decoder_final_file_, true, true);
  return report;
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
