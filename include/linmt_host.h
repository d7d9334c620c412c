/*
 * linmt_host.h -- C facade of liblinmt_host.so, the C++ layer classes (InputToHiddenLayer,
 * HiddenToHiddenLayer, AttentionLayer, SoftmaxLayer, Decoder, NeuralMachineTranslation) that sit on
 * top of the kernel ABI of linmt_hip.h.  C++ callers use the classes of linmt_amd/host/nmt.h
 * directly; this facade exists for callers without a C++ toolchain (the Python tests and the
 * benchmark drive the classes through it), in the style of the reference's own C entry points
 * python_decoder_init / python_decoder_do_job (src/decoder_sentence.h:94-97,
 * src/decoder_sentence.cu:844-874).
 *
 * All pointers are HOST pointers.  Matrices are column-major; token arrays are int32 with -1 padding.
 * Every function returns 0 on success and -1 on failure; lnmt_last_error() describes the failure.
 */
#ifndef LINMT_HOST_H_
#define LINMT_HOST_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct lnmt_config {
  int num_layers;
  int lstm_size;
  int embedding_size;       /* 0 = lstm_size */
  int source_vocab_size;
  int target_vocab_size;
  int minibatch_size;       /* scoring: columns; decoding: ignored */
  int longest_sentence;     /* reference's longest_sentence_ (with its +4) */
  int attention_mode;       /* 0 none, 1 local-p, 2 global general */
  int attention_width;      /* D */
  int feed_input;
  int sequence_to_sequence; /* 0 = target-side language model */
  int clip_cell;
  float cell_clip_threshold;
} lnmt_config;

typedef struct lnmt_decode_options {
  int beam_size;
  float max_decoding_ratio, min_decoding_ratio, penalty, diversity, lp_alpha, cp_beta;
  int unk_replacement_mode; /* the reference's unk_replacement_mode__: export alignment scores per
                               step, Viterbi alignments per token, coverage penalty on the scores */
  int num_hypotheses;       /* the reference's hypotheses_number_: hypotheses kept per sentence
                               (<= 0: 1) */
} lnmt_decode_options;

/* Training options (src/global_configuration.h:107-123, src/utility_cu.cu:82-96). */
typedef struct lnmt_train_options {
  float learning_rate;
  int grad_clip_mode;          /* 0 none, 1 per-matrix norm (reference default), 2 global norm
                                  (--whole-clip-gradients), 3 element clamp (--ind-clip-gradients) */
  float norm_clip;             /* threshold of modes 1 and 2 */
  float individual_clip;       /* threshold of mode 3 */
  float error_clip_threshold;  /* clamp of the errors handed back in time when clip_cell is set */
  float dropout_keep;          /* probability of KEEPING a unit (the reference's dropout_rate_);
                                  <= 0 or >= 1 switches dropout off */
  unsigned long long dropout_seed;
} lnmt_train_options;

typedef struct lnmt_model lnmt_model;

const char *lnmt_last_error(void);

/* NeuralMachineTranslation + InitModel (scoring, one node per timestep). */
lnmt_model *lnmt_model_create_scoring(const lnmt_config *cfg);
/* NeuralMachineTranslation + InitModelDecoding for up to n_sent sentences x beam hypotheses. */
lnmt_model *lnmt_model_create_decoding(const lnmt_config *cfg, int n_sent, int beam_size);
/* NeuralMachineTranslation + InitModel with stored activations and gradient buffers. */
lnmt_model *lnmt_model_create_training(const lnmt_config *cfg, const lnmt_train_options *t);
void lnmt_model_destroy(lnmt_model *m);

/* Parameters by reference name ("src.0.W", "src.1.M_i", "tgt.0.Q_c", "tgt.2.b_f", "attn.W_a",
 * "softmax.D", ...), each a column-major matrix as the reference stores it. */
int lnmt_model_set_param(lnmt_model *m, const char *name, const float *data, long long n);
int lnmt_model_get_param(lnmt_model *m, const char *name, float *data, long long n);

/* NeuralMachineTranslation::GetError: sum of log p(target) over the non-pad target positions. */
int lnmt_get_error(lnmt_model *m, const int *source, int source_length, const int *target_in,
                   const int *target_out, int target_length, const int *batch_information,
                   int minibatch_size, double *loss);

/* NeuralMachineTranslation::ComputeGradients up to (not including) its UpdateWeights call: forward
 * with stored activations and the backward pass of one minibatch of exactly cfg.minibatch_size
 * columns.  source_wgrad / target_wgrad: the unique non-pad input ids of the minibatch
 * (FileHelper's *_wgrad lists).  *loss receives the summed log p(target).  Gradients are of the
 * log-likelihood and unscaled; they accumulate until lnmt_update_weights or lnmt_clear_gradients. */
int lnmt_compute_gradients(lnmt_model *m, const int *source, int source_length,
                           const int *target_in, const int *target_out, int target_length,
                           const int *source_wgrad, int len_source_wgrad, const int *target_wgrad,
                           int len_target_wgrad, const int *batch_information, int minibatch_size,
                           double *loss);
/* The same minibatch driven node by node with the reference's own calls and in its order
 * (src/deep_rnn.h:1137-1273): BackPropPreprocessGpu / BackProp1 / BackProp2 on the loss layer,
 * the attention node's BackProp, BackPropPreprocessGpu + BackPropGpu(index) on every LSTM node.
 * Same gradients as lnmt_compute_gradients up to the order of the sums over steps; not with
 * dropout.  It exists to show (and test) that the layer classes answer to the reference's calls. */
int lnmt_compute_gradients_stepwise(lnmt_model *m, const int *source, int source_length,
                                    const int *target_in, const int *target_out, int target_length,
                                    const int *source_wgrad, int len_source_wgrad,
                                    const int *target_wgrad, int len_target_wgrad,
                                    const int *batch_information, int minibatch_size, double *loss);
/* Gradient by parameter name; "src.0.W" / "tgt.0.W" are E x len_wgrad (column k = id wgrad[k]). */
int lnmt_model_get_grad(lnmt_model *m, const char *name, float *data, long long n);
/* NeuralMachineTranslation::UpdateWeights + ClearGradients.  *global_norm (may be NULL) receives
 * the norm the global clip used (0 in the other modes). */
int lnmt_update_weights(lnmt_model *m, double *global_norm);
/* Which parameter groups lnmt_update_weights moves, the reference's train_*_mode__ switches
 * (src/utility_cu.cu:17-22, read by UpdateParams: src/layer_input_to_hidden.h:1154,1257,1263,
 * src/layer_hidden_to_hidden.h:765,831, src/layer_loss.h:1144).  All 1 at first; --finetune is
 * (0, 0, 0, 1, 1, 1) (src/global_configuration.cc:647-656).  A frozen group's gradients are
 * computed, count in the global norm and are cleared like the others; only the step is left out. */
int lnmt_set_train_modes(lnmt_model *m, int source_input_embedding, int target_input_embedding,
                         int target_output_embedding, int source_rnn, int target_rnn,
                         int attention_target_rnn);
/* The dropout masks the last lnmt_compute_gradients call drew (uniform numbers, kept when
 * < dropout_keep): kind 0 = embeddings of side (0 src / 1 tgt), kind 1 = the mask under which the
 * consumer above `layer` read that layer's h.  Layout rows x minibatch x steps column-major;
 * n = floats the buffer holds (copies min(n, available)).  For parity checks. */
int lnmt_get_dropout_mask(lnmt_model *m, int kind, int side, int layer, float *data, long long n);
int lnmt_clear_gradients(lnmt_model *m);
/* Restarts the sequence of dropout masks: the masks of the n-th lnmt_compute_gradients call after
 * this one are a fixed function of (seed, n), so a run can be repeated mask for mask (the
 * reference seeds each layer's cuRAND generator once, when the layer is initialised:
 * src/layer_input_to_hidden.h:603-605,744-747, src/layer_hidden_to_hidden.h:460-463). */
int lnmt_set_dropout_seed(lnmt_model *m, unsigned long long seed);

/* Copies a state of the last lnmt_get_error call: kind 0 = h, 1 = c of (side 0 src / 1 tgt, layer,
 * timestep); kind 2 = attention output h~ of target timestep; kind 3 = alignments (B x W) of target
 * timestep.  n = number of floats the caller's buffer holds. */
int lnmt_get_state(lnmt_model *m, int kind, int side, int layer, int timestep, float *data,
                   long long n);

/* Batched EnsembleFactory::DecodeFile.  sentences: concatenated source ids in ORIGINAL order,
 * lengths[n].  Outputs: best (n x cap, row-major), best_len[n], best_score[n], steps[n]; if
 * hyp_tokens != NULL also every finished hypothesis: hyp_tokens (n x hyp_cap x cap), hyp_len and
 * hyp_score (n x hyp_cap), n_hyp[n].  best_viterbi (n x cap, may be NULL; filled when
 * o->unk_replacement_mode is set): the source position (original order) aligned to each token of
 * the 1-best, -1 where no alignment score was positive.  kbest_index / kbest_score (n x
 * o->num_hypotheses, may be NULL): the hypotheses Decoder::OutputKBestHypotheses keeps
 * (src/decoder.h:587-607), best first, as indices into the sentence's finished hypotheses (the
 * order of hyp_tokens) with their final scores; -1 / 0 where fewer pass the length filter. */
int lnmt_decode_batch(lnmt_model *m, const int *sentences, const int *lengths, int n,
                      const lnmt_decode_options *o, int *best, int cap, int *best_len,
                      float *best_score, int *steps, int *hyp_tokens, int *hyp_len,
                      float *hyp_score, int hyp_cap, int *n_hyp, int *best_viterbi,
                      int *kbest_index, float *kbest_score);
/* The beam of one sentence of the last lnmt_decode_batch call, step by step: tok / backptr / score
 * hold beam entries per expansion step (entry j of step t: the token chosen, the beam entry of
 * step t-1 it extends, beam-local, and its path score), what the reference keeps in
 * eigen_top_sentences_, new_indices_changes_ and top_sentences_scores_ (src/decoder.h:128-199,
 * 436-479).  score may be NULL.  *steps receives the number of expansion steps copied (at most
 * cap_steps).  For parity checks against a step-by-step reference. */
int lnmt_decode_history(lnmt_model *m, int sentence, int *tok, int *backptr, float *score,
                        int cap_steps, int *steps);

/* The same with an ensemble of n_models models decoded in lockstep (EnsembleFactory::DecodeFile
 * with several models, src/decoder.h:1778-1931): before every beam step the models' distributions
 * are averaged and renormalised (EnsemblesModels, :1910-1931), and with o->unk_replacement_mode
 * their alignment scores are added up (:1933-1962).  models[0] runs the beam search; all were
 * created by lnmt_model_create_decoding with the same n_sent and beam_size and have the same target
 * vocabulary (a multiple of 4) and longest sentence.  n_models = 1 is lnmt_decode_batch. */
int lnmt_decode_batch_ensemble(lnmt_model *const *models, int n_models, const int *sentences,
                               const int *lengths, int n, const lnmt_decode_options *o, int *best,
                               int cap, int *best_len, float *best_score, int *steps,
                               int *hyp_tokens, int *hyp_len, float *hyp_score, int hyp_cap,
                               int *n_hyp, int *best_viterbi, int *kbest_index, float *kbest_score);

/* lnmt_decode_batch over ANY number of sentences with every beam column kept busy (no counterpart
 * in the reference, whose EnsembleFactory::DecodeFile translates one sentence at a time,
 * src/decoder.h:1702-1776): the model's n_sent groups of beam columns are slots; a sentence that has
 * taken its last step hands its slot to the next sentence of the list, so every step runs
 * n_sent * beam_size hypotheses until the list runs out.  Every sentence goes through the steps
 * lnmt_decode_batch takes it through and gives the same kind of result, exported alignments
 * (o->unk_replacement_mode, best_viterbi) and k-best lists (o->num_hypotheses, kbest_index,
 * kbest_score) included.  One model with local-p attention.  The tokens of all finished hypotheses
 * are written out only when hyp_tokens is given.  *ticks (may be NULL) receives the number of
 * steps taken in all.  lnmt_decode_history afterwards addresses the sentences by their position in
 * the list. */
int lnmt_decode_stream(lnmt_model *m, const int *sentences, const int *lengths, int n,
                       const lnmt_decode_options *o, int *best, int cap, int *best_len,
                       float *best_score, int *steps, int *hyp_tokens, int *hyp_len, float *hyp_score,
                       int hyp_cap, int *n_hyp, int *best_viterbi, int *kbest_index,
                       float *kbest_score, int *ticks);

/* lnmt_decode_stream for an ensemble: the models decode in lockstep, models[0] runs the schedule
 * and the beam search on the mean of their distributions (EnsembleFactory::EnsemblesModels,
 * src/decoder.h:1910-1931), as lnmt_decode_batch_ensemble does batch by batch.  Every model needs
 * local-p attention and the same n_sent, beam, target vocabulary and longest sentence. */
int lnmt_decode_stream_ensemble(lnmt_model *const *models, int n_models, const int *sentences,
                                const int *lengths, int n, const lnmt_decode_options *o, int *best,
                                int cap, int *best_len, float *best_score, int *steps,
                                int *hyp_tokens, int *hyp_len, float *hyp_score, int hyp_cap,
                                int *n_hyp, int *best_viterbi, int *kbest_index, float *kbest_score,
                                int *ticks);

/* The model's HIP stream (hipStream_t as void*), for callers that time with HIP events. */
void *lnmt_model_stream(lnmt_model *m);

/* Opt-in arithmetic of a decoding model's largest matrix products (no counterpart in the
 * reference, whose products are cuBLAS SGEMM calls).  on != 0: while at least min_columns
 * hypotheses are alive (min_columns <= 0 keeps the current value, 84 at first), a step's stacked
 * gate products and its output projection are formed from three-way bf16 splits of their fp32
 * operands on the bf16 matrix pipe (lh_gemm_split_f32, lh_gate_gemm_split_lstm_cell_f32 in
 * linmt_hip.h): every fp32 product a*x becomes six exact bf16 products added in fp32, which leaves
 * out less than one fp32 rounding per product.  Everything else -- the encoder, attention, steps
 * with fewer columns, scoring and training -- keeps the fp32 MFMA products, as does the default.
 * On a model created for training the same switch makes the large batched products of a minibatch
 * (weight gradients accumulated over all steps, the output projection and its two backward products,
 * the layer-major input products) split products, both operands packed per call; the per-step
 * products keep the fp32 MFMA path (min_columns == 1 there takes every product: a test aid). */
int lnmt_set_split_products(lnmt_model *m, int on, int min_columns);
/* Measurement and test aids of the decode path, process-wide, all 0 by default (no counterpart in
 * the reference).  Each switches one part back to the form it replaced, with the same results up
 * to the rounding order of the products, so that a test can demand that and a benchmark can time
 * one form against the other:
 *   "no_stream"               lnmt_decoding decodes batch by batch instead of as a stream;
 *   "no_projected_memory"     decoding attends over the encoder states instead of W_a hs / W_c1 hs;
 *   "no_lanes"                the encoder of a decoding batch runs on the model's one stream;
 *   "grouped_gates"           what the previous step fixes of every layer's gate product runs as
 *                             one grouped launch (lh_gate_gemm_group_f32);
 *   "separate_beam_launches"  beam merge and state gather as two launches instead of one.
 * An unknown name is an error.  Set them before a model is created or between calls, not while
 * another thread decodes. */
int lnmt_set_debug_option(const char *name, int value);

/* Live kernel timing with HIP events on the model's stream.  level 0 = off, 1 = the output
 * projection (the dominant matrix product), 2 = every launch of the path.  Totals accumulate
 * over lnmt_decode_batch / lnmt_get_error calls until the level is set again.  Entries are keyed "<call site>" or, for matrix products,
 * "<call site>|<kernel instance>"; work = algorithmic flop (matrix products) or bytes (others). */
int lnmt_profile_set_level(lnmt_model *m, int level);
int lnmt_profile_count(lnmt_model *m);
int lnmt_profile_entry(lnmt_model *m, int index, char *name, int name_cap, double *ms, double *work,
                       long long *launches);

/* ------------------------------------------------------------------------------------------
 * Files either side of the path.
 *
 * Model file: the reference's text checkpoint (first line "layers lstm_size target_vocab
 * source_vocab attention feed_input multi_source combine_lstm char_cnn", the two vocabulary
 * mappings between lines of '=', then every matrix as rows of numbers and an empty line).
 * lnmt_read_model_information = the first-line parse the reference does before it builds a
 * decoder (DecoderModelWrapper::ExtractModelInformation, src/decoder.h:1182-1210; info[9] in the
 * order above); lnmt_model_load_weights =
 * NeuralMachineTranslation::LoadWeights (src/deep_rnn.h:1878-1968) and fails when the header does
 * not describe the model; lnmt_model_dump_model writes a complete file (header, placeholder
 * vocabulary mappings, DumpWeights src/deep_rnn.h:2124-2146) that the reference can load. */
int lnmt_read_model_information(const char *model_file, int info[9]);
int lnmt_model_load_weights(lnmt_model *m, const char *model_file);
int lnmt_model_dump_model(lnmt_model *m, const char *model_file);
/* Parameter names in model-file order: returns the count; name i is copied into `name`. */
int lnmt_model_file_param(lnmt_model *m, int index, char *name, int name_cap, int *rows, int *cols);

/* FileHelper (src/file_helper.h:28-112): reader of the reference's integerised training file
 * (four lines per sentence pair, all pairs of a minibatch padded to common lengths).
 * source_vocab_size = -1 for a target-side language model.  lnmt_file_helper_read_minibatch =
 * ReadMinibatch (src/file_helper.cc:113-272): returns 1 while the epoch continues, 0 when this
 * read reached the end of the file, -1 on error.  After it, lnmt_file_helper_get copies one of the
 * arrays (what: 0 source input, 1 source output, 2 target input, 3 target output -- all
 * minibatch x length column-major --, 4 / 5 source / target *_wgrad lists, 6 batch information)
 * into `data` (n = capacity in ints) and returns the number of valid entries;
 * lnmt_file_helper_info fills {current_source_length, current_target_length,
 * words_in_minibatch, length_source_wgrad, length_target_wgrad, nums_lines_in_file, total_words,
 * total_target_words}. */
typedef struct lnmt_file_helper lnmt_file_helper;
lnmt_file_helper *lnmt_file_helper_create(const char *file_name, int minibatch_size,
                                          int longest_sentence, int source_vocab_size,
                                          int target_vocab_size);
void lnmt_file_helper_destroy(lnmt_file_helper *f);
int lnmt_file_helper_read_minibatch(lnmt_file_helper *f);
int lnmt_file_helper_get(lnmt_file_helper *f, int what, int *data, long long n);
int lnmt_file_helper_info(lnmt_file_helper *f, int info[8]);

/* Dispatcher::Tuning (src/dispatcher.cu:96-384): the training loop -- minibatches from the
 * training file, ComputeGradients + UpdateWeights, the reference's learning-rate schedules
 * (google: halve at the half epoch and after every epoch from epoch_to_start_halving on; stanford:
 * halve after every epoch from epoch_to_start_halving_full on; schedule: multiply by
 * decrease_factor when dev perplexity + margin >= the previous one), best-model dumping, final
 * model file.  The model must have been created with lnmt_model_create_training.  Events
 * (kind: 0 words/s over the last screen_print_rate minibatches, 1 dev perplexity at the half
 * epoch, 2 dev perplexity at the epoch's end, 3 new learning rate, 4 best model dumped (its
 * perplexity), 5 epoch end (summed training log-likelihood), 6 final model written) are copied
 * into `events` up to event_cap; *n_events receives how many happened. */
typedef struct lnmt_tuning_options {
  const char *train_file, *dev_file;               /* integerised files (dev_file may be NULL) */
  const char *output_weight_file, *best_model_file; /* NULL = not written */
  int epochs;
  int google_learning_rate, epoch_to_start_halving;
  int stanford_learning_rate, epoch_to_start_halving_full;
  int learning_rate_schedule;
  float decrease_factor;
  double margin;
  int best_model_mode;
  int screen_print_rate;
} lnmt_tuning_options;
typedef struct lnmt_tuning_event {
  int kind, epoch, minibatch;
  double value;
} lnmt_tuning_event;
int lnmt_tuning(lnmt_model *m, const lnmt_tuning_options *o, lnmt_tuning_event *events,
                int event_cap, int *n_events, long long *words, double *seconds,
                float *final_learning_rate);
/* NeuralMachineTranslation::GetPerplexity (src/deep_rnn.h:1490-1568) over an integerised file. */
int lnmt_get_perplexity(lnmt_model *m, const char *file_name, double *perplexity);

/* Dispatcher::Decoding (src/dispatcher.cu:387-436): translate a text file with a reference model
 * file.  Source lines -> ids with the model's source vocabulary (IntegerizeFileDecoding,
 * src/input_file_preprocess.cc:1312-1482; sentences with length + 1 >= longest_sentence - 2 are
 * thrown away as the reference does), batched beam search, one line of ids per sentence in the
 * format of Decoder::OutputKBestHypotheses (src/decoder.h:602-681; with print_decoding_information:
 * " |||| score |||| Viterbi alignments |||| alignments of the <UNK> tokens", with
 * print_alignments_scores also the alignment scores), then ids -> words (UnintFile,
 * src/input_file_preprocess.cc:1485-1581).  seconds covers the search only. */
typedef struct lnmt_decoding_options {
  const char *model_file, *source_file;
  const char *ids_file;   /* NULL: final_file + ".ids" */
  const char *final_file;
  int beam_size;
  float penalty, max_decoding_ratio, min_decoding_ratio, lp_alpha, cp_beta, diversity;
  int longest_sentence;
  int attention_width; /* D of the local-p window (not stored in the model file); <= 0: 10 */
  int print_decoding_information, print_alignments_scores, unk_replacement_mode;
  int sentences_per_batch;
  int num_hypotheses; /* k-best list per sentence, closed by a line of '=' when != 1; <= 0: 1 */
  /* further model files of an ensemble (the reference's several --decoding models,
   * src/global_configuration.cc:964-1005): the source text is integerised once per model with
   * the model's own source vocabulary; the target vocabulary must be model_file's.  NULL / 0: none */
  const char *const *ensemble_model_files;
  int n_ensemble_models;
} lnmt_decoding_options;
int lnmt_decoding(const lnmt_decoding_options *o, int *sentences, int *sentences_thrown_away,
                  long long *source_words, long long *target_words, double *seconds);
/* The two file conversions on their own (host only, no GPU).  lnmt_integerize_file_decoding:
 * ids (concatenated, reading order) / lengths / input line numbers of the sentences kept;
 * *n_sentences receives their number, which may exceed max_sentences (then call again). */
int lnmt_integerize_file_decoding(const char *model_file, const char *source_file,
                                  int max_sent_cutoff, int *ids, long long ids_cap, int *lengths,
                                  int *lines, int max_sentences, int *n_sentences,
                                  int *target_vocab_size);
int lnmt_unint_file(const char *model_file, const char *unint_file, const char *final_file,
                    int sequence_to_sequence, int decoder_mode);

/* ---- one sentence at a time: the decoder of the translation service ---------------------------
 * DecoderSentence (src/decoder_sentence.h:22-52, src/decoder_sentence.cu:14-391).  create reads a
 * configuration file of lines `param="--key" value="..."` (keys: --nmt-model (required; several
 * files separated by blanks are decoded as an ensemble, the first one's vocabularies serving all,
 * src/decoder_sentence.cu:21-28), --beam-size, --longest-sent, --attention-width, --decoding-ratio "min max", --lp-alpha,
 * --cp-beta, --diversity, --print-decoding-info, --print-align-scores, --nbest (accepted, a sentence always comes back as its one best hypothesis,
 * src/decoder.h:703), --multi-gpu),
 * the vocabularies and, with load_model != 0, the weights (GPU).  NULL on error.  process
 * translates one tokenised sentence (text after " |||| " is ignored): words of the best
 * hypothesis, then with --print-decoding-info " |||| score |||| alignments |||| <UNK> alignments".
 * *needed receives the size of the text including its terminator; a buffer that is too small is
 * an error.  integerize / unint are the two text conversions alone (host only; integerize returns
 * the ids reversed, the order the reference's encoder reads them in).  settings reports what
 * create read (file names in *o are NULL; the model file goes to model_file). */
typedef struct lnmt_decoder_sentence lnmt_decoder_sentence;
lnmt_decoder_sentence *lnmt_decoder_sentence_create(const char *config_file, int load_model);
void lnmt_decoder_sentence_destroy(lnmt_decoder_sentence *d);
int lnmt_decoder_sentence_process(lnmt_decoder_sentence *d, const char *sentence, char *out,
                                  size_t cap, size_t *needed);
int lnmt_decoder_sentence_integerize(lnmt_decoder_sentence *d, const char *sentence, int *ids,
                                     int cap, int *n);
int lnmt_decoder_sentence_unint(lnmt_decoder_sentence *d, const char *sentence, char *out,
                                size_t cap, size_t *needed);
int lnmt_decoder_sentence_settings(lnmt_decoder_sentence *d, lnmt_decoding_options *o,
                                   char *model_file, size_t cap);

/* The C interface the reference's Python server binds (src/decoder_sentence.h:94-97,
 * src/decoder_sentence.cu:844-874), same names and behaviour: one decoder per process, msg is the
 * path of the configuration file, the returned text belongs to the library until the next call,
 * "" for an empty sentence, an error prints a message and ends the process.  Not re-entrant. */
void python_decoder_init(char *msg);
char *python_decoder_do_job(char *sentence);

#ifdef __cplusplus
}
#endif
#endif
