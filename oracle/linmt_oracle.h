/*
 * CPU oracle for the LiNMT per-timestep LSTM / attention / softmax / beam path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a host restatement of the reference's CUDA kernels and host
 * beam search, written from its sources (each function cites the file:line it follows).  Only the
 * tests, the smoke check and the cpu_baseline leg of the benchmark may load it; the product path
 * (liblinmt_hip.so and the C++ layer classes) never calls into it.
 *
 * Layout conventions are the reference's: column-major, activations H x B, int32 ids, -1 padding.
 *
 * Parity pins (what fixes each function besides this restatement) are listed next to the
 * functions in linmt_oracle.cpp; functions that only our reading of the source pins say so.
 */
#ifndef LINMT_ORACLE_H_
#define LINMT_ORACLE_H_

#ifdef __cplusplus
extern "C" {
#endif

/* ---- elementwise / lookup ------------------------------------------------------------------ */
void orc_preprocess_indices(const int *idx, int n, int *idx0, int *mask01, float *mask01_f);
void orc_setup_reverse_indices(const int *unique, int n_unique, int *rev);
void orc_embed_lookup(const float *W, int E, int V, const int *idx0, int B, const float *drop_mask,
                      float keep, float *out);
void orc_dropout(float *x, const float *mask, float keep, long long n);

/* C = alpha * op(A) op(X) + beta * C, fp32 accumulation (column-major, flags as in cuBLAS). */
void orc_gemm(int M, int N, int K, const float *A, int lda, int transA, const float *X, int ldx,
              int transX, float alpha, float beta, float *C, int ldc);

/* LSTM cell, stacked 4H x B pre-activations (rows i,f,g,o); feed != 0 selects the kernels of the
 * feed-input branch (double-precision sigmoid). */
void orc_lstm_cell_fwd(int H, int B, const float *pre1, const float *pre2, const float *pre3,
                       const float *bias4h, const float *c_prev, const int *mask01, int feed,
                       float cell_clip, float *gates, float *c, float *h);

/* Attention core with the argument meaning of lh_attn_core_fwd_f32. */
void orc_attn_core_fwd(int H, int B, int D, int max_len, int hs_steps, const float *tanh1,
                       const float *v_p, const float *wa, const float *hs,
                       long long hs_step_stride, long long hs_col_stride, const int *hs_col,
                       const int *batch_info, const int *mask01, float *p_t, float *sigma,
                       int *indices, float *align, float *cached_exp, float *ctx, int *viterbi);

/* Whole attention node forward (dropout excluded: ha = h_t). Writes h_tild (H x B); the other
 * outputs may be NULL. Scratch is allocated inside. */
void orc_attn_node_fwd(int H, int B, int D, int max_len, int hs_steps, const float *h_t,
                       const float *W_a, const float *W_p, const float *v_p, const float *b_out,
                       const float *W_c1, const float *W_c2, const float *hs,
                       long long hs_step_stride, long long hs_col_stride, const int *hs_col,
                       const int *batch_info, const int *mask01, float *h_tild, float *p_t,
                       int *indices, float *align, float *ctx);

/* ---- softmax / loss -------------------------------------------------------------------------- */
void orc_softmax_fwd(const float *logits, int ldl, const float *bias, int V, int B, float *p,
                     int ldp);
void orc_train_loglik(const float *p, int ldp, int V, int B, const int *tgt0, const int *mask01,
                      double *accum);
void orc_logsoftmax_xent(const float *logits, int ldl, const float *bias, int V, int B,
                         const int *tgt0, const int *mask01, double *logp_tgt, double *loss_accum);

/* ---- beam ------------------------------------------------------------------------------------ */
/* One ExpandHypothesis call for one sentence, from the V x beam probability matrix p (column-major),
 * including the host renormalisation of EnsemblesModels (one model).  Outputs as lh_beam_merge_f32
 * (backptr is the LOCAL beam column here). */
void orc_beam_expand(const float *p, int V, int beam, int step, const float *prev_score,
                     float diversity, float penalty, int start_id, int eof_id, int *tok,
                     int *backptr, float *score, int *fin_count, int *fin_beam, float *fin_score);
/* The same from the distributions of several models: EnsemblesModels (src/decoder.h:1910-1931)
 * averages them in double, rounds to float and renormalises each column in float before the
 * expansion.  pin: equals orc_beam_expand for num_models identical distributions; the averaged
 * distribution against numpy (tests/test_oracle_pins.py). */
void orc_beam_expand_ensemble(const float *const *p, int num_models, int V, int beam, int step,
                              const float *prev_score, float diversity, float penalty, int start_id,
                              int eof_id, int *tok, int *backptr, float *score, int *fin_count,
                              int *fin_beam, float *fin_score);
void orc_beam_gather(const float *src, float *dst, int H, int B, const int *backptr);

/* ---- whole model ----------------------------------------------------------------------------- */
typedef struct orc_model_config {
  int layers;        /* LSTM layers per side */
  int H;             /* lstm_size (and the embedding size when E == 0) */
  int V_src, V_tgt;
  int attention;     /* 0 none, 1 local-p, 2 global-general (build-defined) */
  int D;             /* attention window half-width */
  int feed_input;
  int longest_sent;  /* longest_sentence_ of the reference (already including its +4) */
  int E;             /* embedding size; 0 = H, the reference's only case
                        (src/global_configuration.h:220).  E != H is a generalisation: "*.0.W" is
                        E x V and "*.0.M_*" are H x E.  pin: E == H gives the same bits as E = 0,
                        and the gradients at E != H agree with central differences of the
                        independent numpy model (tests/test_oracle_train_pins.py). */
} orc_model_config;

typedef struct orc_model orc_model;
orc_model *orc_model_create(const orc_model_config *cfg);
void orc_model_destroy(orc_model *m);
/* Host pointer to a parameter, reference names: "src.0.W", "src.0.M_i", "src.1.W_hi", "tgt.0.Q_c",
 * "tgt.0.b_f", "attn.W_a", "attn.v_p", "attn.b_out", "attn.W_c1", "softmax.D", "softmax.b_d" ...;
 * *n_elems receives the element count.  NULL if the name is unknown. */
float *orc_model_param(orc_model *m, const char *name, long long *n_elems);
/* Must be called after parameters were written (refreshes cached transposes). */
void orc_model_commit(orc_model *m);

typedef struct orc_decode_opts {
  int beam;
  float max_ratio, min_ratio, penalty, diversity, lp_alpha, cp_beta;
  int num_threads; /* 0 = leave OpenMP default */
} orc_decode_opts;

/* Beam-decodes ONE sentence the way EnsembleFactory::DecodeFile does (src_ids in ORIGINAL order,
 * the function reverses them like the preprocessing does).  best_tokens receives the 1-best without
 * <START>/<EOF> (capacity cap), *best_len its length, *best_score its rescored value.  If
 * hyp_tokens != NULL it receives every finished hypothesis (row-major, hyp_cap rows x cap tokens,
 * including <START>/<EOF>), hyp_len / hyp_score their lengths and RAW scores, *n_hyp the count.
 * Returns the number of target steps that were run (forward passes of the decoder). */
int orc_decode_sentence(orc_model *m, const int *src_ids, int S, const orc_decode_opts *o,
                        int *best_tokens, int cap, int *best_len, float *best_score,
                        int *hyp_tokens, int *hyp_len, float *hyp_score, int hyp_cap, int *n_hyp);

/* How close the decisions of one orc_beam_expand_ensemble call were: the smallest gap (in
 * log-probability, on the fp32 values the expansion compared) between the last kept and the first
 * dropped probability of a live column, and between neighbours of the score-ordered candidate
 * list down to the first candidate left without a slot.  0 = an exact tie.  Test infrastructure
 * (no counterpart in the reference): it tells a near-tie from a real difference. */
float orc_beam_step_margin(const float *const *p, int num_models, int V, int beam, int step,
                           const float *prev_score, float diversity, int start_id, int eof_id);
/* orc_decode_sentence that also records the beam after every expansion step (beam tokens,
 * beam-local back-pointers and scores per step) and the step's orc_beam_step_margin.
 * trace_window_margin (may be NULL), one value per step: the smallest distance of a live column's
 * window position p_t from an integer -- the local-p window is cut at (int)p_t
 * (LowerUpperKernel, src/deep_rnn_kernel.h:1095-1098), so two fp32 evaluations of a p_t that
 * close to an integer may read windows one position apart; 0.5 for models without local-p
 * attention. */
int orc_decode_sentence_trace(orc_model *m, const int *src_ids, int S, const orc_decode_opts *o,
                              int *best_tokens, int cap, int *best_len, float *best_score,
                              int *trace_tok, int *trace_backptr, float *trace_score,
                              float *trace_margin, int cap_steps, int *n_steps,
                              float *trace_window_margin);

/* The same with the reference's unk_replacement_mode__ on: alignment scores exported at every
 * step, Viterbi alignments carried by the hypotheses, coverage penalty on the real scores.
 * best_viterbi (capacity cap) receives the source position aligned to each token of the 1-best. */
int orc_decode_sentence_alignments(orc_model *m, const int *src_ids, int S, const orc_decode_opts *o,
                                   int *best_tokens, int cap, int *best_len, float *best_score,
                                   int *best_viterbi, int *hyp_tokens, int *hyp_len,
                                   float *hyp_score, int hyp_cap, int *n_hyp);
/* EnsembleFactory::DecodeFile with several models (src/decoder.h:1778-1931): every model runs every
 * step on the shared hypotheses; their distributions are averaged before the expansion and, with
 * alignments != 0 (and attention in every model), their alignment scores added up.  ms[0] supplies
 * the target vocabulary size and the longest sentence.  Outputs as orc_decode_sentence_alignments
 * (best_viterbi may be NULL).  pin: two copies of one model decode exactly like the model alone;
 * two different models against the numpy beam search on the averaged distribution
 * (tests/test_oracle_pins.py). */
int orc_decode_sentence_ensemble(orc_model *const *ms, int num_models, const int *src_ids, int S,
                                 const orc_decode_opts *o, int alignments, int *best_tokens, int cap,
                                 int *best_len, float *best_score, int *best_viterbi,
                                 int *hyp_tokens, int *hyp_len, float *hyp_score, int hyp_cap,
                                 int *n_hyp);

/* Teacher-forced forward + cross-entropy (GetError): src B x S and tgt_in/tgt_out B x T, all
 * column-major with -1 padding (source reversed + left-padded, target right-padded).
 * Returns sum over non-pad target positions of log p(target) (natural log, double). */
double orc_forward_xent(orc_model *m, const int *src, int S, const int *tgt_in, const int *tgt_out,
                        int T, int B, const int *batch_info, int num_threads);

/* ---- training: gradients and update (linmt_oracle_train.cpp) ------------------------------------ */
/* Kernel-granularity functions with the argument meaning of lh_lstm_cell_bwd_f32,
 * lh_softmax_xent_grad_f32, lh_attn_delta_f32 and lh_attn_core_bwd_f32. */
void orc_lstm_cell_bwd(int H, int B, const float *dh_above, const float *dh_next,
                       const float *dc_next, const float *gates, const float *c,
                       const float *c_prev, const int *mask01, float clip_above, float clip_next,
                       const float *above_drop_mask, float keep, float *dgates, float *dc_prev);
void orc_softmax_xent_grad(const float *logits, int ldl, const float *bias, int V, int B,
                           const int *tgt0, const int *mask01, float *dz, int ldz,
                           double *logp_tgt, double *loss_accum);
void orc_attn_delta(int H, int B, const float *dht, const float *dht_feed, const float *h_tild,
                    const int *mask01, float clip_feed, float *delta);
void orc_attn_core_bwd(int H, int B, int D, int max_len, int hs_steps, const float *dctx,
                       const float *tanh1, const float *v_p, const float *wa, const float *hs,
                       long long hs_step_stride, long long hs_col_stride, const int *batch_info,
                       const float *p_t, const float *sigma, const int *indices,
                       const float *align, const float *cached_exp, float *dhs, float *hsum,
                       float *u, float *w);

typedef struct orc_trainer orc_trainer;
orc_trainer *orc_trainer_create(orc_model *m, const orc_model_config *cfg);
void orc_trainer_destroy(orc_trainer *t);
/* Dropout for the following orc_compute_gradients calls (keep <= 0 switches it off).  Masks are
 * uniform numbers, an element survives when mask < keep and is scaled by 1/keep (DropoutKernel,
 * src/deep_rnn_kernel.h:1059-1063).  src_embed / tgt_embed: H x B x steps masks of the looked-up
 * embeddings (src/node_input_to_hidden.h:264-272); src_out / tgt_out: layers x (H x B x steps),
 * mask (l, step) is the one under which the consumer above layer l reads that layer's h: the next
 * layer (src/node_hidden_to_hidden.h:208-226), the attention node (src/layer_attention.h:253-261)
 * or, without attention, the softmax (src/layer_loss.h:501-507).  The top source layer's mask is
 * unused (the attention nodes read its states undropped). */
void orc_trainer_set_dropout(orc_trainer *t, float keep, const float *src_embed,
                             const float *tgt_embed, const float *src_out, const float *tgt_out,
                             int S, int T, int B);
/* The reference's --clip-cell (cell_clip_mode__) for the following orc_compute_gradients calls:
 * c_t clamped to +-cell_clip in the forward pass (src/node_input_to_hidden.h:599-601) and the
 * errors a node hands on -- to step t-1, to the LSTM layer below, to the attention node through
 * feed input -- clamped to +-error_clip (src/node_input_to_hidden.h:876-878, 950-952,
 * src/node_hidden_to_hidden.h:774-776, 877-879).  0 switches a clamp off.
 * pin: thresholds that never bind give the bits of the unclamped run; with binding thresholds the
 * gradients agree with central differences of the numpy forward wherever no clamp was active
 * (tests/test_oracle_train_pins.py). */
void orc_trainer_set_clip(orc_trainer *t, float cell_clip, float error_clip);
void orc_trainer_set_train_modes(orc_trainer *t, const int *modes);
/* NeuralMachineTranslation::ComputeGradients without its final UpdateWeights: forward with stored
 * activations, then the backward pass.  Arguments as orc_forward_xent; src_unique / tgt_unique are
 * the unique non-pad input ids of the minibatch (the reference's *_wgrad lists).  Returns the summed
 * log-likelihood.  Gradients are of the log-likelihood (ascent convention), unscaled. */
double orc_compute_gradients(orc_trainer *t, const int *src, int S, const int *tgt_in,
                             const int *tgt_out, int T, int B, const int *batch_info,
                             const int *src_unique, int n_src_unique, const int *tgt_unique,
                             int n_tgt_unique);
/* Gradient by parameter name; "src.0.W" / "tgt.0.W" are the H x n_unique small gradients whose
 * column k belongs to vocabulary id unique[k]. */
float *orc_trainer_grad(orc_trainer *t, const char *name, long long *n_elems);
/* NeuralMachineTranslation::UpdateWeights: scale by 1/minibatch_size, clip (0 none, 1 per matrix,
 * 2 global norm, 3 element clamp), theta += learning_rate * g, clear.  Returns the global norm
 * (mode 2) or 0. */
float orc_update_weights(orc_trainer *t, float learning_rate, int clip_mode, float norm_clip,
                         float individual_clip, int minibatch_size);

#ifdef __cplusplus
}
#endif
#endif
