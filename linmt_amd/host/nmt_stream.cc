// NeuralMachineTranslation::DecodeStream: beam search over a list of sentences with every beam
// column kept busy.  DecodeBatch starts a batch's sentences together and lets them end one by
// one, so its products shrink from n_sent*beam columns to beam columns over a batch; here a
// sentence that has taken its last step hands its beam columns ("slot") to the next sentence of
// the list, so every step runs n_sent*beam columns until the list runs out.  Every sentence goes
// through exactly the steps DecodeBatch (and Decoder::ExpandHypothesis, src/decoder.h:355-525)
// takes it through; only which sentences share a launch differs.
//
// The number of steps of a sentence is fixed by its length (decoder.h:1734), so the whole
// schedule -- which sentence enters which slot at which tick, and when a group of sentences has
// to be encoded -- is laid out on the host before the first launch, and nothing is read back
// until the end.  Sentences are taken longest first and encoded in groups of up to n_sent (ForwardPropSource as in
// DecodeBatch); what decoding needs of a group -- the projected attention memories W_a*hs and
// W_c1*hs and the encoder's final states -- is kept in one of kRing slabs until the group's last
// sentence has finished.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <exception>
#include <numeric>
#include <thread>

#include "nmt.h"

namespace linmt {

namespace {
constexpr int kRing = 4;  // groups whose encoder outputs are held at once

struct Admission {
  int sentence, group, column, slot, tick, limit;
};
}  // namespace

void NeuralMachineTranslation::DecodeStream(const std::vector<std::vector<int>> &sentences,
                                            const DecodeOptions &o,
                                            std::vector<SentenceResult> *results,
                                            const std::vector<NeuralMachineTranslation *> &ensemble,
                                            const std::vector<std::vector<std::vector<int>>> &ensemble_sentences) {
  if (!decode_mode_) throw LinmtError("DecodeStream: call InitModelDecoding first");
  // EnsembleFactory (decoder.h:1702-1931): every model runs the same columns in lockstep, each on
  // its own streams; this model owns the schedule and the beam search, the others hand it their
  // distributions (as in DecodeBatch).
  std::vector<NeuralMachineTranslation *> models{this};
  for (NeuralMachineTranslation *m : ensemble) {
    if (!m || m == this) throw LinmtError("DecodeStream: ensemble entries must be other models");
    if (!m->decode_mode_ || m->n_sent_ != n_sent_ || m->beam_size_ != beam_size_ ||
        m->cfg_.target_vocab_size_ != cfg_.target_vocab_size_ ||
        m->cfg_.longest_sentence_ != cfg_.longest_sentence_)
      throw LinmtError("DecodeStream: ensemble models must be initialised for decoding with the same "
                       "n_sent, beam, target vocabulary and longest sentence");
    models.push_back(m);
  }
  const int n_models = (int)models.size();
  if (n_models > LH_ENSEMBLE_MAX_MODELS) throw LinmtError("DecodeStream: too many models");
  if (n_models > 1 && cfg_.target_vocab_size_ % 4 != 0)
    throw LinmtError("DecodeStream: an ensemble needs a target vocabulary that is a multiple of 4");
  for (NeuralMachineTranslation *m : models) {
    if (!m->cfg_.attention_mode_ || !m->attention_layer_.ProjectedMemoryPossible())
      throw LinmtError("DecodeStream: needs local-p attention over a projected memory");
    if (2 * m->cfg_.num_layers_ + 1 > LH_GATHER_MAX_TENSORS) throw LinmtError("DecodeStream: too many layers");
  }
  const int n = (int)sentences.size();
  if (!ensemble_sentences.empty()) {
    if (ensemble_sentences.size() != ensemble.size())
      throw LinmtError("DecodeStream: one set of source ids per ensemble model");
    for (const auto &set : ensemble_sentences) {
      if ((int)set.size() != n) throw LinmtError("DecodeStream: ensemble source ids: sentence count differs");
      for (int i = 0; i < n; ++i)
        if (set[i].size() != sentences[i].size())
          throw LinmtError("DecodeStream: ensemble source ids: sentence length differs");
    }
  }
  int beam = o.beam_size_;
  if (beam > (int)std::sqrt((double)cfg_.target_vocab_size_))  // decoder.h:1662-1664
    beam = (int)std::sqrt((double)cfg_.target_vocab_size_);
  if (n < 1 || beam != beam_size_) throw LinmtError("DecodeStream: beam does not match InitModelDecoding");
  const int longest = cfg_.longest_sentence_, slots = n_sent_, B = slots * beam, K = beam + 1;
  const int V = cfg_.target_vocab_size_;
  for (const auto &w : sentences)
    if (w.empty() || (int)w.size() > longest) throw LinmtError("DecodeStream: source sentence length out of range");

  // ---- groups of n_sent sentences, the longest sentences of the whole list first: the sentences of
  // a group are about as long as each other (little padding in the encoder), and the list ends with
  // its shortest sentences, so the slots run empty over a few ticks instead of a long sentence's
  // ninety.  (Results are stored by position in the list; the order of work is free.)
  const int G = (n + slots - 1) / slots;
  std::vector<int> by_length(n);
  std::iota(by_length.begin(), by_length.end(), 0);
  std::stable_sort(by_length.begin(), by_length.end(),
                   [&](int a, int b) { return sentences[a].size() > sentences[b].size(); });
  std::vector<std::vector<int>> group_order(G);  // encoder column -> sentence
  std::vector<int> group_S(G), limit(n);
  for (int g = 0; g < G; ++g) {
    group_order[g].assign(by_length.begin() + (size_t)g * slots,
                          by_length.begin() + std::min((size_t)n, (size_t)(g + 1) * slots));
    group_S[g] = (int)sentences[group_order[g][0]].size();
  }
  for (int i = 0; i < n; ++i)
    limit[i] = std::min((int)(o.max_decoding_ratio_ * (int)sentences[i].size()), longest - 2);  // decoder.h:1734

  // ---- the schedule -----------------------------------------------------------------------------------
  std::vector<Admission> adm;                       // in admission order
  std::vector<std::vector<int>> adm_at, encode_at;  // per tick: indices into adm / groups to encode
  std::vector<int> free_at(slots, 0), group_done(G, 0), start_of(n, 0), slot_of(n, 0);
  {
    int g = 0, k = 0, tick = 0, encoded = 0;
    while (g < G) {
      if ((int)adm_at.size() <= tick) adm_at.resize(tick + 1), encode_at.resize(tick + 1);
      for (int s = 0; s < slots && g < G; ++s) {
        if (free_at[s] > tick) continue;
        if (g >= encoded) {
          // the group's slab is free once the group that held it has finished completely (all of
          // that group's sentences were admitted before this one, so its last tick is known)
          if (g >= kRing && group_done[g - kRing] > tick) break;
          encode_at[tick].push_back(g);
          encoded = g + 1;
        }
        const int i = group_order[g][k];
        adm_at[tick].push_back((int)adm.size());
        adm.push_back(Admission{i, g, k, s, tick, limit[i]});
        start_of[i] = tick, slot_of[i] = s;
        free_at[s] = tick + limit[i] + 1;  // steps 0 .. limit
        group_done[g] = std::max(group_done[g], free_at[s]);
        if (++k == (int)group_order[g].size()) ++g, k = 0;
      }
      ++tick;
    }
  }
  const int ticks = *std::max_element(free_at.begin(), free_at.end());
  adm_at.resize(ticks), encode_at.resize(ticks);

  // ---- device state of the stream ------------------------------------------------------------------
  // rows of the histories: row t+1 is written by tick t, row t holds what tick t reads (tokens
  // chosen and path scores of the tick before; a fresh slot's entries are set by its admission)
  StreamState &ss = stream_state_;
  DeviceArray<int> &tok_hist = ss.tok_hist, &bp_hist = ss.bp_hist, &fcount_hist = ss.fcount_hist,
                   &fbeam_hist = ss.fbeam_hist, &start_dev = ss.start_dev, &limit_dev = ss.limit_dev;
  DeviceArray<float> &score_hist = ss.score_hist, &fscore_hist = ss.fscore_hist;
  const size_t rows = (size_t)ticks + 1;
  tok_hist.Reserve(rows * B), bp_hist.Reserve(rows * B), score_hist.Reserve(rows * B);
  fcount_hist.Reserve((size_t)ticks * slots), fbeam_hist.Reserve((size_t)ticks * B), fscore_hist.Reserve((size_t)ticks * B);
  start_dev.Reserve(slots), limit_dev.Reserve(slots);
  // unk_replacement_mode_: the attention core writes every tick's alignments and window indices
  // into its own slice of a history ([tick][column + B * slot]) instead of the one reused buffer
  const bool capture = o.unk_replacement_mode_;
  std::vector<int> minus_one(slots, -1), zeros(slots, 0);

  // What each model of the ensemble brings: its own encoder, attention memories, decoder states.
  struct ModelState {
    NeuralMachineTranslation *M;
    int H, L, W;
    size_t slab_floats, final_slab, align_slice;
    long long T_cap;
    const float *swap_src[LH_GATHER_MAX_TENSORS];
    float *swap_dst[LH_GATHER_MAX_TENSORS];
    int n_swap;
    float *state_dst[LH_GATHER_MAX_TENSORS], *zero_dst[1];
    bool has_tild;
    float *node_alignments;  // the attention node's own buffers, put back at the end
    int *node_indices;
    std::vector<std::vector<int>> src_blocks;  // the encoder's id block of every group
    std::vector<float> ahist;
    std::vector<int> ihist;
  };
  // host arrays that asynchronous copies read or write are declared before the guard, so however
  // this function is left every stream has drained before any of them is destroyed
  std::vector<ModelState> ms(n_models);
  std::vector<int> binfo0(2 * (size_t)B, 0);
  std::fill(binfo0.begin(), binfo0.begin() + B, 1);  // length 1, offset 0: a column without a sentence
  for (int k = 0; k < n_models; ++k) {
    ModelState &m = ms[k];
    m.M = models[k];
    m.H = m.M->cfg_.lstm_size_, m.L = m.M->cfg_.num_layers_, m.W = m.M->attention_layer_.window_;
    m.slab_floats = m.M->SourceLayer(m.L - 1).h_all_.size();
    m.T_cap = (long long)(m.slab_floats / ((size_t)m.H * slots));
    m.final_slab = (size_t)2 * m.L * m.H * slots;  // [layer][h, c][H x n_sent]
    m.align_slice = (size_t)B * m.W;
    m.node_alignments = m.M->attention_layer_.v_nodes_[0].p_device_alignments_;
    m.node_indices = m.M->attention_layer_.v_nodes_[0].p_device_indices_;
    m.src_blocks.resize(G);
    if (m.T_cap != ms[0].T_cap) throw LinmtError("DecodeStream: the models hold different numbers of encoder steps");
  }
  struct Restore {
    std::vector<ModelState> &ms;
    int B;
    ~Restore() {
      for (ModelState &m : ms) {
        if (!m.M) continue;
        NeuralMachineTranslation &M = *m.M;
        M.attention_layer_.v_nodes_[0].p_device_alignments_ = m.node_alignments;
        M.attention_layer_.v_nodes_[0].p_device_indices_ = m.node_indices;
        if (M.encoder_stream_) (void)hipStreamSynchronize(M.encoder_stream_);
        // DecodeBatch reads the encoder states of column b's sentence through hs_col[b] = b / beam
        (void)hipMemcpyAsync(M.attention_layer_.p_device_hs_col_.get(), M.p_device_sentence_of_column_.get(),
                             sizeof(int) * B, hipMemcpyDeviceToDevice, M.stream_);
        (void)hipStreamSynchronize(M.stream_);
        M.stream_layer0_mask_ = nullptr;
      }
    }
  } restore{ms, B};

  start_dev.Upload(zeros.data(), slots, stream_);
  limit_dev.Upload(minus_one.data(), slots, stream_);
  tok_hist.Zero(stream_, rows * B);  // a slot that never held a sentence feeds <START> = 0
  score_hist.Zero(stream_, rows * B);
  constexpr int kEncoderLead = 24;  // a group is encoded this many ticks ahead of its first admission
  for (ModelState &m : ms) {
    NeuralMachineTranslation &M = *m.M;
    StreamState &st = M.stream_state_;
    st.finals.Reserve(m.final_slab * kRing);
    // what the first target layer reads as its column mask: 1, and for a feed-input model
    // 1 + LH_MASK_F32_GATES on a sentence's first step (the reference runs that step through the
    // kernels without the feed terms, node_input_to_hidden.h:325-621)
    st.mask_host.Reserve((size_t)ticks * B);
    int *mask_host = st.mask_host.get();
    std::fill(mask_host, mask_host + (size_t)ticks * B, 1);
    if (M.cfg_.feed_input_mode_)
      for (const Admission &a : adm)
        for (int j = 0; j < beam; ++j) mask_host[(size_t)a.tick * B + (size_t)a.slot * beam + j] = 1 + LH_MASK_F32_GATES;
    st.mask_table.Reserve((size_t)ticks * B);
    st.mask_table.Upload(mask_host, (size_t)ticks * B, M.stream_);
    if (capture) {
      st.align_hist.Reserve(m.align_slice * ticks);
      st.index_hist.Reserve(m.align_slice * ticks);
    }
    if (&M != this) {
      // the small arrays an admission writes besides the states: this model's own scratch copies
      st.start_dev.Reserve(slots), st.limit_dev.Reserve(slots);
      st.tok_hist.Reserve(B), st.score_hist.Reserve(B);
      if (M.p_device_ensemble_dist_.size() < (size_t)V * B) M.p_device_ensemble_dist_.Alloc((size_t)V * B);
    } else if (n_models > 1 && p_device_ensemble_dist_.size() < (size_t)V * B) {
      p_device_ensemble_dist_.Alloc((size_t)V * B);
    }
    // the attention memories of kRing groups side by side: slab r starts T_cap * n_sent columns
    // after slab 0, which an entry of hs_col can express
    AttentionLayer &A = M.attention_layer_;
    if (A.score_mem_.size() < m.slab_floats * kRing) {
      A.score_mem_.Alloc(m.slab_floats * kRing);
      A.ctx_mem_.Alloc(m.slab_floats * kRing);
    }
    A.hs_step_stride_ = (long long)m.H * slots;
    A.hs_steps_ = (int)m.T_cap;
    A.projected_memory_ = true;
    // A column without a sentence still runs every step: it starts from zero states and attends to
    // the first state of the first sentence of slab 0 (always an encoded sentence), so that nothing
    // it computes is undefined; nothing reads what it computes.
    A.PreprocessMinibatchInformation(binfo0.data(), B);
    A.p_device_hs_col_.Zero(M.stream_);
    for (int l = 0; l < m.L; ++l) {
      M.TargetLayer(l).p_device_h_t_previous_.Zero(M.stream_);
      M.TargetLayer(l).p_device_c_t_previous_.Zero(M.stream_);
      m.state_dst[2 * l] = M.TargetLayer(l).p_device_h_t_previous_.get();
      m.state_dst[2 * l + 1] = M.TargetLayer(l).p_device_c_t_previous_.get();
    }
    if (M.p_device_h_tild_previous_.size()) M.p_device_h_tild_previous_.Zero(M.stream_);
    m.n_swap = M.DecodingStateTensors(m.swap_src, m.swap_dst);
    m.has_tild = M.cfg_.feed_input_mode_ && M.p_device_h_tild_previous_.size();
    m.zero_dst[0] = m.has_tild ? M.p_device_h_tild_previous_.get() : nullptr;
    // The encoder of a group runs on a stream of its own from the tick at which the group's slab
    // is free (at once for the first kRing groups), beside the decoding steps, whose large
    // launches leave room at their ends for its small ones; the decoding stream waits for it
    // right before the group's first sentence enters.
    if (!M.encoder_stream_) HipErrorWrapper(hipStreamCreate(&M.encoder_stream_), "DecodeStream: stream creation failed");
    if (!M.encoder_workspace_.size()) M.encoder_workspace_.Alloc(kGemmWorkspaceBytes);
    while (M.stream_events_.size() < 2 * (size_t)G) {
      hipEvent_t e;
      HipErrorWrapper(hipEventCreateWithFlags(&e, hipEventDisableTiming), "DecodeStream: event creation failed");
      M.stream_events_.push_back(e);
    }
  }
  // ordering between the models' streams: event 0 = "tokens, back-pointers and admissions of this
  // tick are in place" (this model's stream), event k = "model k's distribution is ready"
  if (n_models > 1)
    while (ensemble_events_.size() < (size_t)n_models + 1) {
      hipEvent_t e;
      HipErrorWrapper(hipEventCreateWithFlags(&e, hipEventDisableTiming), "ensemble event creation failed");
      ensemble_events_.push_back(e);
    }
  std::vector<int> first_tick(G, 0);
  for (int t = 0; t < ticks; ++t)
    for (int g : encode_at[t]) first_tick[g] = t;
  std::vector<std::vector<int>> ready_at(ticks);  // groups to encode at this tick
  for (int g = 0; g < G; ++g)
    ready_at[std::max(g < kRing ? 0 : group_done[g - kRing], first_tick[g] - kEncoderLead)].push_back(g);

  // one group through one model's encoder, on that model's encoder stream and workspace
  auto encode_group = [&](ModelState &m, int k, int g) {
    NeuralMachineTranslation &M = *m.M;
    AttentionLayer &A = M.attention_layer_;
    HipErrorWrapper(hipEventRecord(M.stream_events_[2 * g], M.stream_), "DecodeStream: event record failed");
    HipErrorWrapper(hipStreamWaitEvent(M.encoder_stream_, M.stream_events_[2 * g], 0), "DecodeStream: wait failed");
    struct Swap {  // the encoder's launches go to its own stream and workspace
      NeuralMachineTranslation &m;
      hipStream_t s;
      char *ws;
      size_t ws_bytes;
      ~Swap() {
        m.stream_ = s, m.profiler_.stream_ = s;
        m.gemm_ws_ptr_ = ws, m.gemm_ws_bytes_ = ws_bytes;
      }
    } swap{M, M.stream_, M.gemm_ws_ptr_, M.gemm_ws_bytes_};
    M.stream_ = M.encoder_stream_, M.profiler_.stream_ = M.encoder_stream_;
    M.gemm_ws_ptr_ = M.encoder_workspace_.get(), M.gemm_ws_bytes_ = M.encoder_workspace_.size();
    const std::vector<int> &ord = group_order[g];
    const int ng = (int)ord.size(), S = group_S[g], r = g % kRing, H = m.H;
    // this model's own ids of the words when the caller gave them (decoder.h:1749-1761)
    const std::vector<std::vector<int>> &ids = k > 0 && !ensemble_sentences.empty() ? ensemble_sentences[k - 1] : sentences;
    std::vector<int> &src_block = m.src_blocks[g];
    src_block.assign((size_t)ng * S, -1);  // reversed, left-padded (input_file_preprocess.cc:633)
    for (int c = 0; c < ng; ++c) {
      const std::vector<int> &w = ids[ord[c]];
      const int len = (int)w.size();
      for (int q = 0; q < len; ++q) src_block[(size_t)(S - len + q) * ng + c] = w[len - 1 - q];
    }
    M.ForwardPropSource(src_block.data(), S, ng);
    const int cols = slots * S;  // the encoder's slices hold n_sent columns per step
    lh_gemm_seg sa{A.p_device_w_a_.get(), H, A.p_device_total_hs_, H, H};
    M.Gemm(kTagAttnProjGemm, H, cols, &sa, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
           A.score_mem_.get() + m.slab_floats * r, H, "DecodeStream W_a hs");
    lh_gemm_seg sc{A.p_device_w_c_p1_.get(), H, A.p_device_total_hs_, H, H};
    M.Gemm(kTagAttnOutGemm, H, cols, &sc, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
           A.ctx_mem_.get() + m.slab_floats * r, H, "DecodeStream W_c1 hs");
    float *finals = M.stream_state_.finals.get();
    for (int l = 0; l < m.L; ++l) {
      const LstmNode &last = M.SourceLayer(l).v_nodes_[S - 1];
      float *dst = finals + m.final_slab * r + (size_t)2 * l * H * slots;
      HipErrorWrapper(hipMemcpyAsync(dst, last.p_device_h_t_, sizeof(float) * H * ng, hipMemcpyDeviceToDevice, M.stream_),
                      "DecodeStream: copy of the encoder's final h failed");
      HipErrorWrapper(hipMemcpyAsync(dst + (size_t)H * slots, last.p_device_c_t_, sizeof(float) * H * ng,
                                     hipMemcpyDeviceToDevice, M.stream_),
                      "DecodeStream: copy of the encoder's final c failed");
    }
    HipErrorWrapper(hipEventRecord(M.stream_events_[2 * g + 1], M.stream_), "DecodeStream: event record failed");
  };
  // the sentences that enter at tick t, into model k's states and small arrays
  auto admit = [&](ModelState &m, int k, int t) {
    NeuralMachineTranslation &M = *m.M;
    AttentionLayer &A = M.attention_layer_;
    StreamState &st = M.stream_state_;
    const std::vector<int> &now = adm_at[t];
    for (size_t at = 0; at < now.size();) {
      // one launch per group of the ring (the state tensors of a launch come from one slab)
      lh_stream_admission q[LH_STREAM_ADMIT_MAX];
      const int r = adm[now[at]].group % kRing;
      int cnt = 0;
      while (at < now.size() && cnt < LH_STREAM_ADMIT_MAX && adm[now[at]].group % kRing == r) {
        const Admission &a = adm[now[at++]];
        const int len = (int)sentences[a.sentence].size();
        q[cnt++] = lh_stream_admission{a.slot, a.column, (int)(a.column + r * m.T_cap * slots), len,
                                       group_S[a.group] - len, a.limit, a.tick};
      }
      const float *state_src[LH_GATHER_MAX_TENSORS];
      for (int l = 0; l < m.L; ++l) {
        state_src[2 * l] = st.finals.get() + m.final_slab * r + (size_t)2 * l * m.H * slots;
        state_src[2 * l + 1] = state_src[2 * l] + (size_t)m.H * slots;
      }
      // this model: the slots' start ticks and limits, <START> and score 0 in the history row the
      // tick reads; the others: scratch copies of those
      LhErrorWrapper(lh_stream_admit_f32(q, cnt, beam, B, k == 0 ? start_dev.get() : st.start_dev.get(),
                                         k == 0 ? limit_dev.get() : st.limit_dev.get(),
                                         A.p_device_hs_col_.get(), A.p_device_batch_information_.get(),
                                         state_src, m.state_dst, 2 * m.L, m.zero_dst, m.has_tild ? 1 : 0, m.H,
                                         slots, k == 0 ? tok_hist.get() + (size_t)t * B : st.tok_hist.get(),
                                         Decoder::start_symbol_,
                                         k == 0 ? score_hist.get() + (size_t)t * B : st.score_hist.get(),
                                         M.stream_),
                     "DecodeStream admission");
    }
  };

  for (int t = 0; t < ticks; ++t) {
    // ---- groups to encode from this tick on, beside the steps ------------------------------------------
    for (int g : ready_at[t])
      for (int k = 0; k < n_models; ++k) encode_group(ms[k], k, g);
    // ---- groups whose first sentence enters at this tick: their encoder has to be done -----------
    for (int g : encode_at[t])
      for (ModelState &m : ms)
        HipErrorWrapper(hipStreamWaitEvent(m.M->stream_, m.M->stream_events_[2 * g + 1], 0), "DecodeStream: wait failed");
    // ---- sentences that enter at this tick --------------------------------------------------------
    admit(ms[0], 0, t);
    if (n_models > 1) {
      // the other models' streams: the tick before's merge and this tick's admissions are in place
      HipErrorWrapper(hipEventRecord(ensemble_events_[0], stream_), "ensemble event record failed");
      for (int k = 1; k < n_models; ++k) {
        ModelState &m = ms[k];
        HipErrorWrapper(hipStreamWaitEvent(m.M->stream_, ensemble_events_[0], 0), "ensemble wait failed");
        // the survivors' states of the tick before, then the newcomers' (a slot that finished has
        // the identity as back-pointers)
        if (t > 0)
          LhErrorWrapper(lh_beam_gather_f32(m.swap_src, m.swap_dst, m.n_swap, m.H, B, B,
                                            bp_hist.get() + (size_t)t * B, m.M->stream_),
                         "DecodeStream state swap");
        admit(m, k, t);
      }
    }
    // ---- one step of every slot ------------------------------------------------------------------------
    for (int k = n_models - 1; k >= 0; --k) {  // the other models first: this one's stream waits for them
      ModelState &m = ms[k];
      NeuralMachineTranslation &M = *m.M;
      M.stream_layer0_mask_ = M.stream_state_.mask_table.get() + (size_t)t * B;
      if (capture) {
        AttentionNode &node = M.attention_layer_.v_nodes_[0];
        node.p_device_alignments_ = M.stream_state_.align_hist.get() + m.align_slice * t;
        node.p_device_indices_ = M.stream_state_.index_hist.get() + m.align_slice * t;
      }
      M.ForwardPropTarget(1, tok_hist.get() + (size_t)t * B, B);
      M.stream_layer0_mask_ = nullptr;
      if (n_models > 1) {
        LhErrorWrapper(lh_softmax_fwd_f32(M.softmax_layer_.GetDistPtr(), V, nullptr, V, B,
                                          M.p_device_ensemble_dist_.get(), V, M.stream_),
                       "ensemble: model distribution");
        if (k > 0) {
          HipErrorWrapper(hipEventRecord(ensemble_events_[k], M.stream_), "ensemble event record failed");
          HipErrorWrapper(hipStreamWaitEvent(stream_, ensemble_events_[k], 0), "ensemble wait failed");
        }
      }
    }
    if (n_models == 1) {
      ProfileScope ps(profiler_, kTagBeamTopK, 4.0 * V * B);
      LhErrorWrapper(lh_beam_topk_f32(softmax_layer_.GetDistPtr(), V, nullptr, V, B, K, Decoder::end_symbol_,
                                      decoder_.cand_logp_.get(), decoder_.cand_id_.get(),
                                      decoder_.logp_eof_.get(), stream_),
                     "DecodeStream beam top-k");
    } else {
      // EnsemblesModels (decoder.h:1910-1931) + the per-column selection of ExpandHypothesis
      const float *dist[LH_ENSEMBLE_MAX_MODELS];
      for (int k = 0; k < n_models; ++k) dist[k] = models[k]->p_device_ensemble_dist_.get();
      ProfileScope ps(profiler_, kTagBeamTopK, 4.0 * n_models * V * B);
      LhErrorWrapper(lh_beam_topk_ensemble_f32(dist, n_models, V, V, B, K, Decoder::end_symbol_,
                                               decoder_.cand_logp_.get(), decoder_.cand_id_.get(),
                                               decoder_.logp_eof_.get(), stream_),
                     "DecodeStream ensemble beam top-k");
    }
    {
      ProfileScope pm(profiler_, kTagBeamMergeGather, 8.0 * K * B + 8.0 * ms[0].n_swap * ms[0].H * B);
      LhErrorWrapper(lh_beam_merge_gather_stream_f32(
                         slots, beam, K, t, start_dev.get(), limit_dev.get(), decoder_.cand_logp_.get(),
                         decoder_.cand_id_.get(), decoder_.logp_eof_.get(), score_hist.get() + (size_t)t * B,
                         o.diversity_, o.penalty_, Decoder::start_symbol_, Decoder::end_symbol_,
                         tok_hist.get() + (size_t)(t + 1) * B, bp_hist.get() + (size_t)(t + 1) * B,
                         score_hist.get() + (size_t)(t + 1) * B, fcount_hist.get() + (size_t)t * slots,
                         fbeam_hist.get() + (size_t)t * B, fscore_hist.get() + (size_t)t * B, ms[0].swap_src,
                         ms[0].swap_dst, ms[0].n_swap, ms[0].H, stream_),
                     "DecodeStream beam merge and state swap");
    }
  }

  // ---- one read-back -----------------------------------------------------------------------------------
  ss.tok.Reserve(rows * B), ss.bp.Reserve(rows * B), ss.bscore.Reserve(rows * B);
  ss.fcount.Reserve((size_t)ticks * slots), ss.fbeam.Reserve((size_t)ticks * B), ss.fscore.Reserve((size_t)ticks * B);
  const int *tok = ss.tok.get(), *bp = ss.bp.get(), *fcount = ss.fcount.get(), *fbeam = ss.fbeam.get();
  const float *fscore = ss.fscore.get(), *bscore = ss.bscore.get();
  tok_hist.Download(ss.tok.get(), rows * B, stream_);
  bp_hist.Download(ss.bp.get(), rows * B, stream_);
  score_hist.Download(ss.bscore.get(), rows * B, stream_);
  fcount_hist.Download(ss.fcount.get(), (size_t)ticks * slots, stream_);
  fbeam_hist.Download(ss.fbeam.get(), (size_t)ticks * B, stream_);
  fscore_hist.Download(ss.fscore.get(), (size_t)ticks * B, stream_);
  for (int k = 0; k < n_models; ++k) {
    ModelState &m = ms[k];
    if (capture) {
      m.ahist.resize(m.align_slice * ticks), m.ihist.resize(m.align_slice * ticks);
      m.M->stream_state_.align_hist.Download(m.ahist.data(), m.ahist.size(), m.M->stream_);
      m.M->stream_state_.index_hist.Download(m.ihist.data(), m.ihist.size(), m.M->stream_);
    }
    // every model's streams have drained before its host arrays and shared buffers are reused
    if (k > 0) HipErrorWrapper(hipStreamSynchronize(m.M->stream_), "ensemble stream synchronisation failed");
  }
  Synchronize();
  profiler_.Collect();

  // ---- hypotheses by walking the back-pointers, as DecodeBatch does; the search of every sentence
  // in the compact layout lnmt_decode_history reads.  Sentences are independent: a few host threads
  // share them (a list of a thousand sentences is tens of milliseconds of this on one thread).
  results->assign(n, SentenceResult());
  DecodeHistory &hist = last_history_;
  hist.n = n, hist.beam = beam;
  hist.slot_of_sentence.resize(n);
  std::iota(hist.slot_of_sentence.begin(), hist.slot_of_sentence.end(), 0);
  hist.limit = limit;
  hist.offset.assign(n, 0);
  size_t hist_rows = 0;
  int max_limit = 0;
  for (int i = 0; i < n; ++i) {
    hist.offset[i] = hist_rows * beam;
    hist_rows += (size_t)limit[i] + 1;
    max_limit = std::max(max_limit, limit[i]);
  }
  hist.steps = max_limit + 1;
  hist.tok.resize(hist_rows * beam), hist.backptr.resize(hist_rows * beam), hist.score.resize(hist_rows * beam);
  auto build = [&](int i) {
    SentenceResult &r = (*results)[i];
    const int t0 = start_of[i], c0 = slot_of[i] * beam, s = slot_of[i];
    r.steps = limit[i] + 1;
    const int source_length = (int)sentences[i].size();
    // alignment scores over the source positions of `column` at the sentence's step q, and their
    // arg-max as EnsemblesModels takes it (decoder.h:1946-1961): first strictly largest score above 0
    auto alignment_row = [&](int q, int column, std::vector<float> *scores, int *viterbi) {
      scores->assign(source_length, 0.f);
      for (const ModelState &m : ms)  // the models' scores are added up (decoder.h:1933-1945)
        for (int j = 0; j < m.W; ++j) {
          const size_t at = m.align_slice * (size_t)(t0 + q) + column + (size_t)B * j;
          const int idx = m.ihist[at];
          if (idx >= 0 && idx < source_length) (*scores)[idx] += m.ahist[at];
        }
      float max_val = 0;
      *viterbi = -1;
      for (int j = 0; j < source_length; ++j)
        if ((*scores)[j] > max_val) {
          max_val = (*scores)[j];
          *viterbi = j;
        }
    };
    auto prefix = [&](int step, int column, Hypothesis *h) {
      // token q+1 was produced by the forward pass of its PARENT column at step q, whose
      // alignments it carries (decoder.h:452-456)
      h->tokens.assign(step + 1, Decoder::start_symbol_);
      if (capture) {
        h->viterbi.assign(step + 2, -20);
        h->alignments_scores.assign(step + 2, std::vector<float>());
      }
      int col = column;
      for (int q = step - 1; q >= 0; --q) {
        h->tokens[q + 1] = tok[(size_t)(t0 + q + 1) * B + col];
        col = bp[(size_t)(t0 + q + 1) * B + col];
        if (capture) alignment_row(q, col, &h->alignments_scores[q + 1], &h->viterbi[q + 1]);
      }
    };
    // the finished hypotheses in the order the reference's v_hypotheses_ holds them: where each
    // one ended, its score and its length; the tokens are written out for all of them or, when the
    // caller only reads the kept ones, for those
    std::vector<int> at_step, parent_of, sizes;
    for (int step = 0; step <= limit[i]; ++step) {
      const int nf = fcount[(size_t)(t0 + step) * slots + s];
      for (int f = 0; f < nf; ++f) {
        at_step.push_back(step);
        parent_of.push_back(c0 + fbeam[(size_t)(t0 + step) * B + c0 + f]);
        sizes.push_back(step + 2);  // <START>, `step` words, <EOF>
      }
    }
    r.hypotheses.resize(at_step.size());
    auto write_out = [&](int k) {
      Hypothesis &h = r.hypotheses[k];
      if (!h.tokens.empty()) return;
      prefix(at_step[k], parent_of[k], &h);
      h.tokens.push_back(Decoder::end_symbol_);
      if (capture)  // <EOF> itself comes out of the parent's forward pass at this step
        alignment_row(at_step[k], parent_of[k], &h.alignments_scores[at_step[k] + 1], &h.viterbi[at_step[k] + 1]);
    };
    for (size_t k = 0, f = 0; k < at_step.size(); ++k) {
      f = k > 0 && at_step[k] == at_step[k - 1] ? f + 1 : 0;
      r.hypotheses[k].score = fscore[(size_t)(t0 + at_step[k]) * B + c0 + f];
      // the coverage penalty reads every hypothesis' exported alignments
      if (o.all_hypotheses_tokens_ || capture) write_out((int)k);
    }
    Decoder::OutputKBestHypotheses(r.hypotheses, source_length, o, &r, &sizes, write_out);
    if (capture)  // only the hypotheses kept hold on to their score rows (what a printout shows)
      for (size_t h = 0; h < r.hypotheses.size(); ++h)
        if (std::find(r.kbest.begin(), r.kbest.end(), (int)h) == r.kbest.end())
          std::vector<std::vector<float>>().swap(r.hypotheses[h].alignments_scores);
    for (int step = 0; step <= limit[i]; ++step)
      for (int j = 0; j < beam; ++j) {
        const size_t from = (size_t)(t0 + step + 1) * B + c0 + j, to = hist.offset[i] + (size_t)step * beam + j;
        if (step == limit[i]) {
          // the row a sentence's last step writes is the row the slot's next sentence is admitted
          // into: what the step stored there (<EOF>, the column itself, the final score) is taken
          // from the finished-hypothesis record of the same step instead
          hist.tok[to] = Decoder::end_symbol_;
          hist.backptr[to] = j;
          hist.score[to] = fscore[(size_t)(t0 + step) * B + c0 + j];
          continue;
        }
        hist.tok[to] = tok[from];
        hist.backptr[to] = bp[from] - c0;
        hist.score[to] = bscore[from];
      }
  };
  {
    const int workers = std::max(1, std::min({8, n / 32, (int)std::thread::hardware_concurrency()}));
    std::atomic<int> next{0};
    std::vector<std::exception_ptr> failed(workers);
    auto run = [&](int w) {
      try {
        for (int i = next.fetch_add(1); i < n; i = next.fetch_add(1)) build(i);
      } catch (...) {
        failed[w] = std::current_exception();
      }
    };
    std::vector<std::thread> pool;
    for (int w = 1; w < workers; ++w) pool.emplace_back(run, w);
    run(0);
    for (std::thread &t : pool) t.join();
    for (const std::exception_ptr &e : failed)
      if (e) std::rethrow_exception(e);
  }
  stream_ticks_ = ticks;
}

}  // namespace linmt
