// C facade over the C++ layer classes (declared in include/linmt_host.h).
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>

#include "../../include/linmt_host.h"
#include "decoder_sentence.h"
#include "dispatcher.h"
#include "file_helper.h"
#include "input_file_preprocess.h"
#include "nmt.h"

using namespace linmt;

struct lnmt_model {
  std::unique_ptr<NeuralMachineTranslation> nmt;
};

namespace {

thread_local std::string g_error;

GlobalConfiguration ToConfig(const lnmt_config *c) {
  GlobalConfiguration g;
  g.num_layers_ = c->num_layers;
  g.lstm_size_ = c->lstm_size;
  g.embedding_size_ = c->embedding_size;
  g.source_vocab_size_ = c->source_vocab_size;
  g.target_vocab_size_ = c->target_vocab_size;
  g.minibatch_size_ = c->minibatch_size;
  g.longest_sentence_ = c->longest_sentence;
  g.attention_mode_ = c->attention_mode;
  g.attention_width_ = c->attention_width;
  g.feed_input_mode_ = c->feed_input != 0;
  g.sequence_to_sequence_mode_ = c->sequence_to_sequence != 0;
  g.clip_cell_mode_ = c->clip_cell != 0;
  g.cell_clip_threshold_ = c->cell_clip_threshold;
  return g;
}

template <typename F>
int Guard(F &&f) {
  try {
    f();
    return 0;
  } catch (const std::exception &e) {
    g_error = e.what();
    return -1;
  } catch (...) {  // nothing may unwind into a C caller
    g_error = "unknown C++ exception";
    return -1;
  }
}

}  // namespace

extern "C" const char *lnmt_last_error(void) { return g_error.c_str(); }

extern "C" lnmt_model *lnmt_model_create_scoring(const lnmt_config *cfg) {
  lnmt_model *m = nullptr;
  if (Guard([&] {
        std::unique_ptr<lnmt_model> p(new lnmt_model());
        p->nmt.reset(new NeuralMachineTranslation(ToConfig(cfg)));
        p->nmt->InitModel();
        m = p.release();
      }) != 0)
    return nullptr;
  return m;
}

extern "C" lnmt_model *lnmt_model_create_decoding(const lnmt_config *cfg, int n_sent,
                                                  int beam_size) {
  lnmt_model *m = nullptr;
  if (Guard([&] {
        if (n_sent < 1 || beam_size < 1) throw LinmtError("n_sent and beam_size must be positive");
        std::unique_ptr<lnmt_model> p(new lnmt_model());
        p->nmt.reset(new NeuralMachineTranslation(ToConfig(cfg)));
        p->nmt->InitModelDecoding(n_sent, beam_size);
        m = p.release();
      }) != 0)
    return nullptr;
  return m;
}

extern "C" lnmt_model *lnmt_model_create_training(const lnmt_config *cfg,
                                                  const lnmt_train_options *t) {
  lnmt_model *m = nullptr;
  if (Guard([&] {
        GlobalConfiguration g = ToConfig(cfg);
        g.train_mode_ = true;
        g.learning_rate_ = t->learning_rate;
        g.grad_clip_mode_ = t->grad_clip_mode;
        g.norm_clip_ = t->norm_clip;
        g.individual_norm_clip_threshold_ = t->individual_clip;
        g.error_clip_threshold_ = t->error_clip_threshold;
        g.dropout_mode_ = t->dropout_keep > 0.f && t->dropout_keep < 1.f;
        g.dropout_rate_ = g.dropout_mode_ ? t->dropout_keep : 1.f;
        g.dropout_seed_ = t->dropout_seed;
        if (g.grad_clip_mode_ < 0 || g.grad_clip_mode_ > 3) throw LinmtError("grad_clip_mode outside [0,3]");
        if ((g.grad_clip_mode_ == 1 || g.grad_clip_mode_ == 2) && !(g.norm_clip_ > 0.f))
          throw LinmtError("norm_clip must be positive");
        std::unique_ptr<lnmt_model> p(new lnmt_model());
        p->nmt.reset(new NeuralMachineTranslation(g));
        p->nmt->InitModel();
        m = p.release();
      }) != 0)
    return nullptr;
  return m;
}

extern "C" void lnmt_model_destroy(lnmt_model *m) { delete m; }

extern "C" int lnmt_compute_gradients(lnmt_model *m, const int *source, int source_length,
                                      const int *target_in, const int *target_out,
                                      int target_length, const int *source_wgrad,
                                      int len_source_wgrad, const int *target_wgrad,
                                      int len_target_wgrad, const int *batch_information,
                                      int minibatch_size, double *loss) {
  return Guard([&] {
    *loss = m->nmt->ComputeGradients(source, source_length, target_in, target_out, target_length,
                                     source_wgrad, len_source_wgrad, target_wgrad,
                                     len_target_wgrad, batch_information, minibatch_size);
  });
}

extern "C" int lnmt_compute_gradients_stepwise(lnmt_model *m, const int *source, int source_length,
                                               const int *target_in, const int *target_out,
                                               int target_length, const int *source_wgrad,
                                               int len_source_wgrad, const int *target_wgrad,
                                               int len_target_wgrad, const int *batch_information,
                                               int minibatch_size, double *loss) {
  return Guard([&] {
    *loss = m->nmt->ComputeGradientsStepwise(source, source_length, target_in, target_out,
                                             target_length, source_wgrad, len_source_wgrad,
                                             target_wgrad, len_target_wgrad, batch_information,
                                             minibatch_size);
  });
}

extern "C" int lnmt_model_get_grad(lnmt_model *m, const char *name, float *data, long long n) {
  return Guard([&] {
    std::vector<float> v;
    if (!m->nmt->GetGrad(name, &v) || (long long)v.size() != n)
      throw LinmtError(std::string("unknown gradient or wrong size: ") + name);
    memcpy(data, v.data(), sizeof(float) * v.size());
  });
}

extern "C" int lnmt_update_weights(lnmt_model *m, double *global_norm) {
  return Guard([&] {
    m->nmt->UpdateWeights();
    if (global_norm) *global_norm = m->nmt->last_global_norm_;
  });
}

extern "C" int lnmt_get_dropout_mask(lnmt_model *m, int kind, int side, int layer, float *data,
                                     long long n) {
  return Guard([&] {
    NeuralMachineTranslation &M = *m->nmt;
    if (layer < 0 || layer >= M.cfg_.num_layers_) throw LinmtError("layer out of range");
    LstmLayer &L = side == 0 ? M.SourceLayer(layer) : M.TargetLayer(layer);
    const DeviceArray<float> &a = kind == 0 ? L.dropout_mask_all_ : L.out_dropout_mask_all_;
    if (a.size() == 0) throw LinmtError("this layer has no such dropout mask");
    const size_t count = std::min<size_t>((size_t)n, a.size());
    a.Download(data, count, M.stream_);
    M.Synchronize();
  });
}

extern "C" int lnmt_clear_gradients(lnmt_model *m) {
  return Guard([&] {
    m->nmt->ClearGradients();
    m->nmt->Synchronize();
  });
}

extern "C" int lnmt_set_dropout_seed(lnmt_model *m, unsigned long long seed) {
  return Guard([&] {
    if (!m->nmt->cfg_.train_mode_) throw LinmtError("lnmt_set_dropout_seed: not a training model");
    m->nmt->cfg_.dropout_seed_ = seed;
    m->nmt->minibatch_counter_ = 0;
  });
}

extern "C" int lnmt_set_train_modes(lnmt_model *m, int source_input_embedding, int target_input_embedding,
                                    int target_output_embedding, int source_rnn, int target_rnn,
                                    int attention_target_rnn) {
  return Guard([&] {
    GlobalConfiguration &c = m->nmt->cfg_;
    if (!c.train_mode_) throw LinmtError("lnmt_set_train_modes: not a training model");
    c.train_source_input_embedding_mode_ = source_input_embedding != 0;
    c.train_target_input_embedding_mode_ = target_input_embedding != 0;
    c.train_target_output_embedding_mode_ = target_output_embedding != 0;
    c.train_source_rnn_mode_ = source_rnn != 0;
    c.train_target_rnn_mode_ = target_rnn != 0;
    c.train_attention_target_rnn_mode_ = attention_target_rnn != 0;
  });
}

extern "C" int lnmt_model_set_param(lnmt_model *m, const char *name, const float *data,
                                    long long n) {
  return Guard([&] {
    if (!m->nmt->SetParam(name, data, (size_t)n))
      throw LinmtError(std::string("unknown parameter or wrong size: ") + name);
    m->nmt->Synchronize();
  });
}

extern "C" int lnmt_model_get_param(lnmt_model *m, const char *name, float *data, long long n) {
  return Guard([&] {
    std::vector<float> v;
    if (!m->nmt->GetParam(name, &v) || (long long)v.size() != n)
      throw LinmtError(std::string("unknown parameter or wrong size: ") + name);
    memcpy(data, v.data(), sizeof(float) * v.size());
  });
}

extern "C" int lnmt_get_error(lnmt_model *m, const int *source, int source_length,
                              const int *target_in, const int *target_out, int target_length,
                              const int *batch_information, int minibatch_size, double *loss) {
  return Guard([&] {
    *loss = m->nmt->GetError(source, source_length, target_in, target_out, target_length,
                             batch_information, minibatch_size);
  });
}

extern "C" int lnmt_get_state(lnmt_model *m, int kind, int side, int layer, int timestep,
                              float *data, long long n) {
  return Guard([&] {
    NeuralMachineTranslation &M = *m->nmt;
    const float *src = nullptr;
    size_t count = 0;
    if (kind == 0 || kind == 1) {
      if (layer < 0 || layer >= M.cfg_.num_layers_) throw LinmtError("layer out of range");
      LstmLayer &L = side == 0 ? M.SourceLayer(layer) : M.TargetLayer(layer);
      if (timestep < 0 || timestep >= L.num_nodes_) throw LinmtError("timestep out of range");
      src = kind == 0 ? L.v_nodes_[timestep].p_device_h_t_ : L.v_nodes_[timestep].p_device_c_t_;
      count = (size_t)L.lstm_size_ * L.minibatch_size_;
    } else if (kind == 2 || kind == 3) {
      AttentionLayer &A = M.attention_layer_;
      if (timestep < 0 || timestep >= A.num_nodes_) throw LinmtError("timestep out of range");
      src = kind == 2 ? A.v_nodes_[timestep].p_device_final_tmp_2_
                      : A.v_nodes_[timestep].p_device_alignments_;
      count = kind == 2 ? (size_t)A.lstm_size_ * A.minibatch_size_
                        : (size_t)A.window_ * A.minibatch_size_;
    } else {
      throw LinmtError("unknown state kind");
    }
    if ((size_t)n < count) count = (size_t)n;
    HipErrorWrapper(hipMemcpyAsync(data, src, sizeof(float) * count, hipMemcpyDeviceToHost,
                                   M.stream_),
                    "state download failed");
    M.Synchronize();
  });
}

extern "C" int lnmt_decode_batch(lnmt_model *m, const int *sentences, const int *lengths, int n,
                                 const lnmt_decode_options *o, int *best, int cap, int *best_len,
                                 float *best_score, int *steps, int *hyp_tokens, int *hyp_len,
                                 float *hyp_score, int hyp_cap, int *n_hyp, int *best_viterbi,
                                 int *kbest_index, float *kbest_score) {
  lnmt_model *one[1] = {m};
  return lnmt_decode_batch_ensemble(one, 1, sentences, lengths, n, o, best, cap, best_len,
                                    best_score, steps, hyp_tokens, hyp_len, hyp_score, hyp_cap,
                                    n_hyp, best_viterbi, kbest_index, kbest_score);
}

extern "C" int lnmt_decode_history(lnmt_model *m, int sentence, int *tok, int *backptr, float *score,
                                   int cap_steps, int *steps) {
  return Guard([&] {
    if (!m || !tok || !backptr || !steps) throw LinmtError("lnmt_decode_history: NULL argument");
    const auto &h = m->nmt->last_history_;
    if (sentence < 0 || sentence >= h.n) throw LinmtError("lnmt_decode_history: no such sentence in the last batch");
    const int k = h.slot_of_sentence[sentence], B = h.n * h.beam;
    const int n_steps = std::min(h.limit[k], cap_steps);  // expansion steps 0 .. limit-1
    if (!h.offset.empty()) {  // DecodeStream: the sentence's rows are contiguous, back-pointers local
      const size_t at = h.offset[sentence];
      for (int e = 0; e < n_steps * h.beam; ++e) {
        tok[e] = h.tok[at + e];
        backptr[e] = h.backptr[at + e];
        if (score) score[e] = h.score[at + e];
      }
      *steps = n_steps;
      return;
    }
    for (int t = 0; t < n_steps; ++t)
      for (int j = 0; j < h.beam; ++j) {
        tok[(size_t)t * h.beam + j] = h.tok[(size_t)t * B + (size_t)k * h.beam + j];
        backptr[(size_t)t * h.beam + j] = h.backptr[(size_t)t * B + (size_t)k * h.beam + j] - k * h.beam;
        if (score) score[(size_t)t * h.beam + j] = h.score[(size_t)t * B + (size_t)k * h.beam + j];
      }
    *steps = n_steps;
  });
}

// What the two decode entry points share: sentences in, results out.  stream selects
// DecodeStream (every beam column kept busy over a list of any length) instead of DecodeBatch.
static int DecodeThroughFacade(bool stream, lnmt_model *const *models, int n_models,
                               const int *sentences, const int *lengths, int n,
                               const lnmt_decode_options *o, int *best, int cap, int *best_len,
                               float *best_score, int *steps, int *hyp_tokens, int *hyp_len,
                               float *hyp_score, int hyp_cap, int *n_hyp, int *best_viterbi,
                               int *kbest_index, float *kbest_score) {
  return Guard([&] {
    if (!models || n_models < 1 || !models[0]) throw LinmtError("no model");
    if (!sentences || !lengths || !o || !best || !best_len || !best_score || n < 0 || cap < 1)
      throw LinmtError("decode: NULL argument or negative count");
    lnmt_model *m = models[0];
    std::vector<NeuralMachineTranslation *> others;
    for (int k = 1; k < n_models; ++k) {
      if (!models[k]) throw LinmtError("ensemble model is NULL");
      others.push_back(models[k]->nmt.get());
    }
    std::vector<std::vector<int>> sents(n);
    size_t off = 0;
    for (int i = 0; i < n; ++i) {
      if (lengths[i] < 0) throw LinmtError("negative sentence length");
      sents[i].assign(sentences + off, sentences + off + lengths[i]);
      off += lengths[i];
    }
    DecodeOptions d;
    d.beam_size_ = o->beam_size;
    d.max_decoding_ratio_ = o->max_decoding_ratio;
    d.min_decoding_ratio_ = o->min_decoding_ratio;
    d.penalty_ = o->penalty;
    d.diversity_ = o->diversity;
    d.lp_alpha_ = o->lp_alpha;
    d.cp_beta_ = o->cp_beta;
    d.unk_replacement_mode_ = o->unk_replacement_mode != 0;
    d.hypotheses_number_ = std::max(1, o->num_hypotheses);
    d.all_hypotheses_tokens_ = hyp_tokens != nullptr;
    std::vector<SentenceResult> res;
    if (stream)
      m->nmt->DecodeStream(sents, d, &res, others);
    else
      m->nmt->DecodeBatch(sents, d, &res, others);
    for (int i = 0; i < n; ++i) {
      const SentenceResult &r = res[i];
      const int bl = std::min((int)r.best.size(), cap);
      for (int j = 0; j < bl; ++j) best[(size_t)i * cap + j] = r.best[j];
      if (best_viterbi)
        for (int j = 0; j < bl; ++j)
          best_viterbi[(size_t)i * cap + j] = j < (int)r.best_viterbi.size() ? r.best_viterbi[j] : -1;
      best_len[i] = bl;
      best_score[i] = r.best_score;
      if (steps) steps[i] = r.steps;
      if (n_hyp) n_hyp[i] = (int)r.hypotheses.size();
      for (int k = 0; k < d.hypotheses_number_; ++k) {
        const bool have = k < (int)r.kbest.size();
        if (kbest_index) kbest_index[(size_t)i * d.hypotheses_number_ + k] = have ? r.kbest[k] : -1;
        if (kbest_score) kbest_score[(size_t)i * d.hypotheses_number_ + k] = have ? r.kbest_score[k] : 0.f;
      }
      if (hyp_tokens) {
        const int nh = std::min((int)r.hypotheses.size(), hyp_cap);
        for (int h = 0; h < nh; ++h) {
          const Hypothesis &hy = r.hypotheses[h];
          const int len = std::min((int)hy.tokens.size(), cap);
          for (int j = 0; j < len; ++j)
            hyp_tokens[((size_t)i * hyp_cap + h) * cap + j] = hy.tokens[j];
          hyp_len[(size_t)i * hyp_cap + h] = (int)hy.tokens.size();
          hyp_score[(size_t)i * hyp_cap + h] = hy.score;
        }
      }
    }
  });
}

extern "C" int lnmt_decode_batch_ensemble(lnmt_model *const *models, int n_models,
                                          const int *sentences, const int *lengths, int n,
                                          const lnmt_decode_options *o, int *best, int cap,
                                          int *best_len, float *best_score, int *steps,
                                          int *hyp_tokens, int *hyp_len, float *hyp_score,
                                          int hyp_cap, int *n_hyp, int *best_viterbi,
                                          int *kbest_index, float *kbest_score) {
  return DecodeThroughFacade(false, models, n_models, sentences, lengths, n, o, best, cap, best_len,
                             best_score, steps, hyp_tokens, hyp_len, hyp_score, hyp_cap, n_hyp,
                             best_viterbi, kbest_index, kbest_score);
}

extern "C" int lnmt_decode_stream(lnmt_model *m, const int *sentences, const int *lengths, int n,
                                  const lnmt_decode_options *o, int *best, int cap, int *best_len,
                                  float *best_score, int *steps, int *hyp_tokens, int *hyp_len,
                                  float *hyp_score, int hyp_cap, int *n_hyp, int *best_viterbi,
                                  int *kbest_index, float *kbest_score, int *ticks) {
  const int rc = DecodeThroughFacade(true, &m, m ? 1 : 0, sentences, lengths, n, o, best, cap, best_len, best_score,
                                     steps, hyp_tokens, hyp_len, hyp_score, hyp_cap, n_hyp, best_viterbi,
                                     kbest_index, kbest_score);
  if (rc == 0 && ticks) *ticks = m->nmt->stream_ticks_;
  return rc;
}

extern "C" int lnmt_decode_stream_ensemble(lnmt_model *const *models, int n_models, const int *sentences,
                                           const int *lengths, int n, const lnmt_decode_options *o,
                                           int *best, int cap, int *best_len, float *best_score,
                                           int *steps, int *hyp_tokens, int *hyp_len, float *hyp_score,
                                           int hyp_cap, int *n_hyp, int *best_viterbi, int *kbest_index,
                                           float *kbest_score, int *ticks) {
  const int rc = DecodeThroughFacade(true, models, n_models, sentences, lengths, n, o, best, cap, best_len,
                                     best_score, steps, hyp_tokens, hyp_len, hyp_score, hyp_cap, n_hyp,
                                     best_viterbi, kbest_index, kbest_score);
  if (rc == 0 && ticks) *ticks = models[0]->nmt->stream_ticks_;
  return rc;
}

extern "C" void *lnmt_model_stream(lnmt_model *m) { return m->nmt->stream_; }

extern "C" int lnmt_profile_set_level(lnmt_model *m, int level) {
  return Guard([&] {
    m->nmt->Synchronize();
    m->nmt->profiler_.Collect();
    m->nmt->profiler_.Reset();
    m->nmt->profiler_.level_ = level;
  });
}

namespace linmt {
DebugOptions &Debug() {
  static DebugOptions options;
  return options;
}
}  // namespace linmt

extern "C" int lnmt_set_debug_option(const char *name, int value) {
  return Guard([&] {
    if (!name) throw LinmtError("lnmt_set_debug_option: NULL name");
    DebugOptions &d = linmt::Debug();
    const std::string n(name);
    if (n == "no_stream") d.no_stream = value;
    else if (n == "no_projected_memory") d.no_projected_memory = value;
    else if (n == "no_lanes") d.no_lanes = value;
    else if (n == "grouped_gates") d.grouped_gates = value;
    else if (n == "separate_beam_launches") d.separate_beam_launches = value;
    else throw LinmtError("lnmt_set_debug_option: unknown option " + n);
  });
}

extern "C" int lnmt_set_split_products(lnmt_model *m, int on, int min_columns) {
  return Guard([&] {
    if (on && m->nmt->decode_mode_ && m->nmt->cfg_.lstm_size_ % 8)
      throw linmt::LinmtError("lnmt_set_split_products: decoding needs a hidden size that is a multiple of 8");
    m->nmt->split_products_ = on != 0;
    if (min_columns > 0) m->nmt->split_min_columns_ = min_columns;
  });
}

extern "C" int lnmt_profile_count(lnmt_model *m) { return (int)m->nmt->profiler_.totals_.size(); }

extern "C" int lnmt_profile_entry(lnmt_model *m, int index, char *name, int name_cap, double *ms,
                                  double *work, long long *launches) {
  return Guard([&] {
    const auto &tot = m->nmt->profiler_.totals_;
    if (index < 0 || index >= (int)tot.size()) throw LinmtError("profile entry out of range");
    auto it = tot.begin();
    std::advance(it, index);
    snprintf(name, name_cap, "%s", it->first.c_str());
    *ms = it->second.ms;
    *work = it->second.work;
    *launches = it->second.launches;
  });
}

// ---- files either side of the path -------------------------------------------------------------
extern "C" int lnmt_read_model_information(const char *model_file, int info[9]) {
  return Guard([&] {
    const ModelInformation m = ReadModelInformation(model_file);
    const int v[9] = {m.num_layers,  m.lstm_size,    m.target_vocab_size, m.source_vocab_size, m.attention_model,
                      m.feed_input,  m.multi_source, m.combine_lstm,      m.char_cnn};
    std::copy(v, v + 9, info);
  });
}

extern "C" int lnmt_model_load_weights(lnmt_model *m, const char *model_file) {
  return Guard([&] { m->nmt->LoadWeights(model_file); });
}

extern "C" int lnmt_model_dump_model(lnmt_model *m, const char *model_file) {
  return Guard([&] { m->nmt->DumpModel(model_file, nullptr, nullptr); });
}

extern "C" int lnmt_model_file_param(lnmt_model *m, int index, char *name, int name_cap, int *rows,
                                     int *cols) {
  int count = -1;
  Guard([&] {
    const auto order = m->nmt->ModelFileOrder();
    if (index >= 0 && index < (int)order.size() && name && name_cap > 0) {
      snprintf(name, name_cap, "%s", order[index].name.c_str());
      if (rows) *rows = order[index].rows;
      if (cols) *cols = order[index].cols;
    }
    count = (int)order.size();
  });
  return count;
}

struct lnmt_file_helper {
  std::unique_ptr<FileHelper> fh;
};

extern "C" lnmt_file_helper *lnmt_file_helper_create(const char *file_name, int minibatch_size,
                                                     int longest_sentence, int source_vocab_size,
                                                     int target_vocab_size) {
  lnmt_file_helper *f = nullptr;
  Guard([&] {
    std::unique_ptr<lnmt_file_helper> p(new lnmt_file_helper());
    p->fh.reset(new FileHelper(file_name, minibatch_size, longest_sentence, source_vocab_size,
                               target_vocab_size));
    f = p.release();
  });
  return f;
}

extern "C" void lnmt_file_helper_destroy(lnmt_file_helper *f) { delete f; }

extern "C" int lnmt_file_helper_read_minibatch(lnmt_file_helper *f) {
  int same_epoch = 0;
  if (Guard([&] { same_epoch = f->fh->ReadMinibatch() ? 1 : 0; }) != 0) return -1;
  return same_epoch;
}

extern "C" int lnmt_file_helper_get(lnmt_file_helper *f, int what, int *data, long long n) {
  int valid = -1;
  Guard([&] {
    const FileHelper &h = *f->fh;
    const std::vector<int> *v = nullptr;
    long long count = 0;
    const long long B = h.minibatch_size_;
    switch (what) {
      case 0: v = &h.p_host_input_vocab_indices_source_; count = B * h.current_source_length_; break;
      case 1: v = &h.p_host_output_vocab_indices_source_; count = B * h.current_source_length_; break;
      case 2: v = &h.p_host_input_vocab_indices_target_; count = B * h.current_target_length_; break;
      case 3: v = &h.p_host_output_vocab_indices_target_; count = B * h.current_target_length_; break;
      case 4: v = &h.p_host_input_vocab_indices_source_wgrad_; count = h.length_source_wgrad_; break;
      case 5: v = &h.p_host_input_vocab_indices_target_wgrad_; count = h.length_target_wgrad_; break;
      case 6: v = &h.p_host_batch_information_; count = 2 * B; break;
      default: throw LinmtError("lnmt_file_helper_get: unknown array " + std::to_string(what));
    }
    if (count > n) throw LinmtError("lnmt_file_helper_get: the buffer is too small");
    std::copy(v->begin(), v->begin() + count, data);
    valid = (int)count;
  });
  return valid;
}

extern "C" int lnmt_file_helper_info(lnmt_file_helper *f, int info[8]) {
  return Guard([&] {
    const FileHelper &h = *f->fh;
    const int v[8] = {h.current_source_length_, h.current_target_length_, h.words_in_minibatch_,
                      h.length_source_wgrad_,   h.length_target_wgrad_,   h.nums_lines_in_file_,
                      h.total_words_,           h.total_target_words_};
    std::copy(v, v + 8, info);
  });
}

extern "C" int lnmt_tuning(lnmt_model *m, const lnmt_tuning_options *o, lnmt_tuning_event *events,
                           int event_cap, int *n_events, long long *words, double *seconds,
                           float *final_learning_rate) {
  return Guard([&] {
    if (!o || !o->train_file) throw LinmtError("lnmt_tuning: no training file");
    TuningConfiguration c;
    c.train_file_name_ = o->train_file;
    c.test_file_name_ = o->dev_file ? o->dev_file : "";
    c.output_weight_file_ = o->output_weight_file ? o->output_weight_file : "";
    c.best_model_file_name_ = o->best_model_file ? o->best_model_file : "";
    c.epochs_number_ = o->epochs;
    c.google_learning_rate_ = o->google_learning_rate != 0;
    c.epoch_to_start_halving_ = o->epoch_to_start_halving;
    c.stanford_learning_rate_ = o->stanford_learning_rate != 0;
    c.epoch_to_start_halving_full_ = o->epoch_to_start_halving_full;
    c.learning_rate_schedule_ = o->learning_rate_schedule != 0;
    c.decrease_factor_ = o->decrease_factor;
    c.margin_ = o->margin;
    c.best_model_mode_ = o->best_model_mode != 0;
    c.screen_print_rate_ = o->screen_print_rate > 0 ? o->screen_print_rate : 20;
    if (c.learning_rate_schedule_ && c.test_file_name_.empty())
      throw LinmtError("lnmt_tuning: the perplexity schedule needs a dev file");
    const TuningReport r = Dispatcher::Tuning(*m->nmt, c);
    const int n = (int)r.events.size();
    for (int i = 0; i < n && i < event_cap; ++i)
      events[i] = {(int)r.events[i].kind, r.events[i].epoch, r.events[i].minibatch, r.events[i].value};
    if (n_events) *n_events = n;
    if (words) *words = r.words;
    if (seconds) *seconds = r.seconds;
    if (final_learning_rate) *final_learning_rate = r.final_learning_rate;
  });
}

extern "C" int lnmt_get_perplexity(lnmt_model *m, const char *file_name, double *perplexity) {
  return Guard([&] { *perplexity = m->nmt->GetPerplexity(file_name); });
}

extern "C" int lnmt_decoding(const lnmt_decoding_options *o, int *sentences, int *sentences_thrown_away,
                             long long *source_words, long long *target_words, double *seconds) {
  return Guard([&] {
    if (!o || !o->model_file || !o->source_file || !o->final_file)
      throw LinmtError("lnmt_decoding: model_file, source_file and final_file are required");
    DecodingConfiguration c;
    c.model_name_ = o->model_file;
    c.decode_user_file_ = o->source_file;
    c.decoder_output_file_ = o->ids_file ? o->ids_file : "";
    c.decoder_final_file_ = o->final_file;
    c.beam_size_ = o->beam_size;
    c.penalty_ = o->penalty;
    c.max_decoding_ratio_ = o->max_decoding_ratio;
    c.min_decoding_ratio_ = o->min_decoding_ratio;
    c.decoding_lp_alpha_ = o->lp_alpha;
    c.decoding_cp_beta_ = o->cp_beta;
    c.decoding_diversity_ = o->diversity;
    if (o->longest_sentence > 0) c.longest_sentence_ = o->longest_sentence;
    if (o->attention_width > 0) c.attention_width_ = o->attention_width;
    c.print_decoding_information_mode_ = o->print_decoding_information != 0;
    c.print_alignments_scores_mode_ = o->print_alignments_scores != 0;
    c.unk_replacement_mode_ = o->unk_replacement_mode != 0;
    if (o->sentences_per_batch > 0) c.sentences_per_batch_ = o->sentences_per_batch;
    if (o->num_hypotheses > 0) c.hypotheses_number_ = o->num_hypotheses;
    for (int k = 0; k < o->n_ensemble_models; ++k) {
      if (!o->ensemble_model_files || !o->ensemble_model_files[k])
        throw LinmtError("lnmt_decoding: ensemble model file is NULL");
      c.ensemble_model_names_.push_back(o->ensemble_model_files[k]);
    }
    const DecodingReport r = Dispatcher::Decoding(c);
    if (sentences) *sentences = r.sentences;
    if (sentences_thrown_away) *sentences_thrown_away = r.sentences_thrown_away;
    if (source_words) *source_words = r.source_words;
    if (target_words) *target_words = r.target_words;
    if (seconds) *seconds = r.seconds;
  });
}

extern "C" int lnmt_integerize_file_decoding(const char *model_file, const char *source_file,
                                             int max_sent_cutoff, int *ids, long long ids_cap,
                                             int *lengths, int *lines, int max_sentences,
                                             int *n_sentences, int *target_vocab_size) {
  return Guard([&] {
    InputFilePreprocess helper;
    std::vector<std::vector<int>> sentences;
    std::vector<int> kept;
    const int v = helper.IntegerizeFileDecoding(model_file, source_file, max_sent_cutoff, &sentences, &kept);
    if (target_vocab_size) *target_vocab_size = v;
    if (n_sentences) *n_sentences = (int)sentences.size();
    long long at = 0;
    for (size_t i = 0; i < sentences.size() && (int)i < max_sentences; ++i) {
      if (at + (long long)sentences[i].size() > ids_cap) throw LinmtError("lnmt_integerize_file_decoding: ids buffer too small");
      std::copy(sentences[i].begin(), sentences[i].end(), ids + at);
      at += (long long)sentences[i].size();
      lengths[i] = (int)sentences[i].size();
      if (lines) lines[i] = kept[i];
    }
  });
}

extern "C" int lnmt_unint_file(const char *model_file, const char *unint_file, const char *final_file,
                               int sequence_to_sequence, int decoder_mode) {
  return Guard([&] {
    InputFilePreprocess helper;
    helper.UnintFile(model_file, unint_file, final_file, sequence_to_sequence != 0, decoder_mode != 0);
  });
}

struct lnmt_decoder_sentence {
  DecoderSentence decoder;
};

extern "C" lnmt_decoder_sentence *lnmt_decoder_sentence_create(const char *config_file, int load_model) {
  lnmt_decoder_sentence *d = nullptr;
  if (Guard([&] {
        if (!config_file) throw LinmtError("lnmt_decoder_sentence_create: config_file is required");
        std::unique_ptr<lnmt_decoder_sentence> p(new lnmt_decoder_sentence());
        p->decoder.Init(config_file, load_model != 0);
        d = p.release();
      }) != 0)
    return nullptr;
  return d;
}

extern "C" void lnmt_decoder_sentence_destroy(lnmt_decoder_sentence *d) { delete d; }

namespace {
void CopyText(const std::string &text, char *out, size_t cap, size_t *needed) {
  if (needed) *needed = text.size() + 1;
  if (text.size() + 1 > cap) throw LinmtError("output buffer too small");
  std::memcpy(out, text.c_str(), text.size() + 1);
}
}  // namespace

extern "C" int lnmt_decoder_sentence_process(lnmt_decoder_sentence *d, const char *sentence, char *out,
                                             size_t cap, size_t *needed) {
  return Guard([&] {
    std::string output;
    d->decoder.Process(sentence, output);
    CopyText(output, out, cap, needed);
  });
}

extern "C" int lnmt_decoder_sentence_integerize(lnmt_decoder_sentence *d, const char *sentence, int *ids,
                                                int cap, int *n) {
  return Guard([&] {
    std::vector<int> v;
    d->decoder.IntegerizeSentence(sentence, v);
    if (n) *n = (int)v.size();
    if ((int)v.size() > cap) throw LinmtError("lnmt_decoder_sentence_integerize: ids buffer too small");
    std::copy(v.begin(), v.end(), ids);
  });
}

extern "C" int lnmt_decoder_sentence_unint(lnmt_decoder_sentence *d, const char *sentence, char *out,
                                           size_t cap, size_t *needed) {
  return Guard([&] {
    std::string text(sentence);
    d->decoder.UnintSentence(text);
    CopyText(text, out, cap, needed);
  });
}

extern "C" int lnmt_decoder_sentence_settings(lnmt_decoder_sentence *d, lnmt_decoding_options *o,
                                              char *model_file, size_t cap) {
  return Guard([&] {
    const DecodingConfiguration &c = d->decoder.configuration();
    std::memset(o, 0, sizeof(*o));
    o->beam_size = c.beam_size_;
    o->penalty = c.penalty_;
    o->max_decoding_ratio = c.max_decoding_ratio_;
    o->min_decoding_ratio = c.min_decoding_ratio_;
    o->lp_alpha = c.decoding_lp_alpha_;
    o->cp_beta = c.decoding_cp_beta_;
    o->diversity = c.decoding_diversity_;
    o->longest_sentence = c.longest_sentence_;
    o->attention_width = c.attention_width_;
    o->print_decoding_information = c.print_decoding_information_mode_;
    o->print_alignments_scores = c.print_alignments_scores_mode_;
    o->unk_replacement_mode = c.unk_replacement_mode_;
    o->sentences_per_batch = c.sentences_per_batch_;
    o->num_hypotheses = c.hypotheses_number_;
    if (model_file) CopyText(c.model_name_, model_file, cap, nullptr);
  });
}

// The process-wide decoder of the reference's translation server (src/decoder_sentence.cu:844-874):
// one instance, the returned text is owned by the library and released by the next call, errors
// end the process as the reference's do.
namespace {
char *decoder_result__ = nullptr;
DecoderSentence *decoder_sentence__ = nullptr;

[[noreturn]] void Fatal(const char *where, const std::exception &e) {
  std::fprintf(stderr, "   Error: %s: %s\n", where, e.what());
  std::exit(EXIT_FAILURE);
}
}  // namespace

extern "C" void python_decoder_init(char *msg) {
  try {
    std::unique_ptr<DecoderSentence> fresh(new DecoderSentence());
    fresh->Init(msg ? msg : "");
    delete decoder_sentence__;
    decoder_sentence__ = fresh.release();
  } catch (const std::exception &e) {
    Fatal("python_decoder_init", e);
  } catch (...) {  // nothing may unwind through an extern "C" frame into a ctypes caller
    Fatal("python_decoder_init", LinmtError("unknown exception"));
  }
}

extern "C" char *python_decoder_do_job(char *sentence) {
  // the previous result stays valid until the new one has been built
  try {
    std::string output_sentence;
    if (!decoder_sentence__) throw LinmtError("python_decoder_init has not been called");
    const std::string input_sentence(sentence ? sentence : "");
    if (!input_sentence.empty()) decoder_sentence__->Process(input_sentence, output_sentence);
    char *fresh = new char[output_sentence.size() + 1];
    std::memcpy(fresh, output_sentence.c_str(), output_sentence.size() + 1);
    delete[] decoder_result__;
    decoder_result__ = fresh;
  } catch (const std::exception &e) {
    Fatal("python_decoder_do_job", e);
  } catch (...) {
    Fatal("python_decoder_do_job", LinmtError("unknown exception"));
  }
  return decoder_result__;
}
