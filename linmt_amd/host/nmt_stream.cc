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
                                            std::vector<SentenceResult> *results) {
  if (!decode_mode_) throw LinmtError("DecodeStream: call InitModelDecoding first");
  if (!cfg_.attention_mode_ || !attention_layer_.ProjectedMemoryPossible())
    throw LinmtError("DecodeStream: needs local-p attention over a projected memory");
  const int n = (int)sentences.size(), L = cfg_.num_layers_, H = cfg_.lstm_size_;
  int beam = o.beam_size_;
  if (beam > (int)std::sqrt((double)cfg_.target_vocab_size_))  // decoder.h:1662-1664
    beam = (int)std::sqrt((double)cfg_.target_vocab_size_);
  if (n < 1 || beam != beam_size_) throw LinmtError("DecodeStream: beam does not match InitModelDecoding");
  if (2 * L + 1 > LH_GATHER_MAX_TENSORS) throw LinmtError("DecodeStream: too many layers");
  const int longest = cfg_.longest_sentence_, slots = n_sent_, B = slots * beam, K = beam + 1;
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
                   &fbeam_hist = ss.fbeam_hist, &start_dev = ss.start_dev, &limit_dev = ss.limit_dev,
                   &mask_table = ss.mask_table;
  DeviceArray<float> &score_hist = ss.score_hist, &fscore_hist = ss.fscore_hist, &finals = ss.finals;
  const size_t rows = (size_t)ticks + 1;
  tok_hist.Reserve(rows * B), bp_hist.Reserve(rows * B), score_hist.Reserve(rows * B);
  fcount_hist.Reserve((size_t)ticks * slots), fbeam_hist.Reserve((size_t)ticks * B), fscore_hist.Reserve((size_t)ticks * B);
  start_dev.Reserve(slots), limit_dev.Reserve(slots);
  const size_t final_slab = (size_t)2 * L * H * slots;  // [layer][h, c][H x n_sent]
  finals.Reserve(final_slab * kRing);
  // what the first target layer reads as its column mask: 1, and for a feed-input model
  // 1 + LH_MASK_F32_GATES on a sentence's first step (the reference runs that step through the
  // kernels without the feed terms, node_input_to_hidden.h:325-621)
  ss.mask_host.Reserve((size_t)ticks * B);
  int *mask_host = ss.mask_host.get();
  std::fill(mask_host, mask_host + (size_t)ticks * B, 1);
  std::vector<int> minus_one(slots, -1), zeros(slots, 0);
  if (cfg_.feed_input_mode_)
    for (const Admission &a : adm)
      for (int j = 0; j < beam; ++j) mask_host[(size_t)a.tick * B + (size_t)a.slot * beam + j] = 1 + LH_MASK_F32_GATES;
  mask_table.Reserve((size_t)ticks * B);
  // unk_replacement_mode_: the attention core writes every tick's alignments and window indices
  // into its own slice of a history ([tick][column + B * slot]) instead of the one reused buffer
  const bool capture = o.unk_replacement_mode_;
  const int W = attention_layer_.window_;
  const size_t align_slice = (size_t)B * W;
  if (capture) {
    ss.align_hist.Reserve(align_slice * ticks);
    ss.index_hist.Reserve(align_slice * ticks);
  }
  // host arrays that asynchronous copies read or write: declared before the guard, so however this
  // function is left the stream has drained before any of them is destroyed
  std::vector<std::vector<int>> src_blocks(G);  // the encoder's id block of every group
  std::vector<int> binfo0(2 * (size_t)B, 0);
  std::fill(binfo0.begin(), binfo0.begin() + B, 1);  // length 1, offset 0: a column without a sentence
  AttentionNode &attention_node = attention_layer_.v_nodes_[0];
  struct Restore {
    NeuralMachineTranslation &m;
    int B;
    float *node_alignments;
    int *node_indices;
    ~Restore() {
      m.attention_layer_.v_nodes_[0].p_device_alignments_ = node_alignments;
      m.attention_layer_.v_nodes_[0].p_device_indices_ = node_indices;
      if (m.encoder_stream_) (void)hipStreamSynchronize(m.encoder_stream_);
      // DecodeBatch reads the encoder states of column b's sentence through hs_col[b] = b / beam
      (void)hipMemcpyAsync(m.attention_layer_.p_device_hs_col_.get(), m.p_device_sentence_of_column_.get(),
                           sizeof(int) * B, hipMemcpyDeviceToDevice, m.stream_);
      (void)hipStreamSynchronize(m.stream_);
      m.stream_layer0_mask_ = nullptr;
    }
  } restore{*this, B, attention_node.p_device_alignments_, attention_node.p_device_indices_};
  mask_table.Upload(mask_host, (size_t)ticks * B, stream_);
  start_dev.Upload(zeros.data(), slots, stream_);
  limit_dev.Upload(minus_one.data(), slots, stream_);
  tok_hist.Zero(stream_, rows * B);  // a slot that never held a sentence feeds <START> = 0
  score_hist.Zero(stream_, rows * B);

  // the attention memories of kRing groups side by side: slab r starts T_cap * n_sent columns
  // after slab 0, which an entry of hs_col can express
  AttentionLayer &A = attention_layer_;
  const size_t slab_floats = SourceLayer(L - 1).h_all_.size();
  const long long T_cap = (long long)(slab_floats / ((size_t)H * slots));
  if (A.score_mem_.size() < slab_floats * kRing) {
    A.score_mem_.Alloc(slab_floats * kRing);
    A.ctx_mem_.Alloc(slab_floats * kRing);
  }
  A.hs_step_stride_ = (long long)H * slots;
  A.hs_steps_ = (int)T_cap;
  A.projected_memory_ = true;
  // A column without a sentence still runs every step: it starts from zero states and attends to
  // the first state of the first sentence of slab 0 (always an encoded sentence), so that nothing
  // it computes is undefined; nothing reads what it computes.
  A.PreprocessMinibatchInformation(binfo0.data(), B);
  A.p_device_hs_col_.Zero(stream_);
  for (int l = 0; l < L; ++l) {
    TargetLayer(l).p_device_h_t_previous_.Zero(stream_);
    TargetLayer(l).p_device_c_t_previous_.Zero(stream_);
  }
  if (p_device_h_tild_previous_.size()) p_device_h_tild_previous_.Zero(stream_);

  const float *state_src[LH_GATHER_MAX_TENSORS];
  float *state_dst[LH_GATHER_MAX_TENSORS], *zero_dst[1];
  const float *swap_src[LH_GATHER_MAX_TENSORS];
  float *swap_dst[LH_GATHER_MAX_TENSORS];
  const int n_swap = DecodingStateTensors(swap_src, swap_dst);
  for (int l = 0; l < L; ++l) {
    state_dst[2 * l] = TargetLayer(l).p_device_h_t_previous_.get();
    state_dst[2 * l + 1] = TargetLayer(l).p_device_c_t_previous_.get();
  }
  const bool has_tild = cfg_.feed_input_mode_ && p_device_h_tild_previous_.size();
  zero_dst[0] = has_tild ? p_device_h_tild_previous_.get() : nullptr;

  // The encoder of a group runs on a stream of its own from the tick at which the group's slab is
  // free (at once for the first kRing groups), beside the decoding steps, whose large launches
  // leave room at their ends for its small ones; the decoding stream waits for it right before the
  // group's first sentence enters.
  if (!encoder_stream_) HipErrorWrapper(hipStreamCreate(&encoder_stream_), "DecodeStream: stream creation failed");
  if (!encoder_workspace_.size()) encoder_workspace_.Alloc(kGemmWorkspaceBytes);
  while (stream_events_.size() < 2 * (size_t)G) {
    hipEvent_t e;
    HipErrorWrapper(hipEventCreateWithFlags(&e, hipEventDisableTiming), "DecodeStream: event creation failed");
    stream_events_.push_back(e);
  }
  // a group is encoded kEncoderLead ticks ahead of its first admission, or as soon as its slab is free
  constexpr int kEncoderLead = 24;
  std::vector<int> first_tick(G, 0);
  for (int t = 0; t < ticks; ++t)
    for (int g : encode_at[t]) first_tick[g] = t;
  std::vector<std::vector<int>> ready_at(ticks);  // groups to encode at this tick
  for (int g = 0; g < G; ++g)
    ready_at[std::max(g < kRing ? 0 : group_done[g - kRing], first_tick[g] - kEncoderLead)].push_back(g);

  for (int t = 0; t < ticks; ++t) {
    // ---- groups to encode from this tick on, beside the steps ------------------------------------------
    for (int g : ready_at[t]) {
      HipErrorWrapper(hipEventRecord(stream_events_[2 * g], stream_), "DecodeStream: event record failed");
      HipErrorWrapper(hipStreamWaitEvent(encoder_stream_, stream_events_[2 * g], 0), "DecodeStream: wait failed");
      struct Swap {  // the encoder's launches go to its own stream and workspace
        NeuralMachineTranslation &m;
        hipStream_t s;
        char *ws;
        size_t ws_bytes;
        ~Swap() {
          m.stream_ = s, m.profiler_.stream_ = s;
          m.gemm_ws_ptr_ = ws, m.gemm_ws_bytes_ = ws_bytes;
        }
      } swap{*this, stream_, gemm_ws_ptr_, gemm_ws_bytes_};
      stream_ = encoder_stream_, profiler_.stream_ = encoder_stream_;
      gemm_ws_ptr_ = encoder_workspace_.get(), gemm_ws_bytes_ = encoder_workspace_.size();
      const std::vector<int> &ord = group_order[g];
      const int ng = (int)ord.size(), S = group_S[g], r = g % kRing;
      std::vector<int> &src_block = src_blocks[g];
      src_block.assign((size_t)ng * S, -1);  // reversed, left-padded (input_file_preprocess.cc:633)
      for (int k = 0; k < ng; ++k) {
        const std::vector<int> &w = sentences[ord[k]];
        const int len = (int)w.size();
        for (int q = 0; q < len; ++q) src_block[(size_t)(S - len + q) * ng + k] = w[len - 1 - q];
      }
      ForwardPropSource(src_block.data(), S, ng);
      const int cols = slots * S;  // the encoder's slices hold n_sent columns per step
      lh_gemm_seg sa{A.p_device_w_a_.get(), H, A.p_device_total_hs_, H, H};
      Gemm(kTagAttnProjGemm, H, cols, &sa, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
           A.score_mem_.get() + slab_floats * r, H, "DecodeStream W_a hs");
      lh_gemm_seg sc{A.p_device_w_c_p1_.get(), H, A.p_device_total_hs_, H, H};
      Gemm(kTagAttnOutGemm, H, cols, &sc, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
           A.ctx_mem_.get() + slab_floats * r, H, "DecodeStream W_c1 hs");
      for (int l = 0; l < L; ++l) {
        const LstmNode &last = SourceLayer(l).v_nodes_[S - 1];
        float *dst = finals.get() + final_slab * r + (size_t)2 * l * H * slots;
        HipErrorWrapper(hipMemcpyAsync(dst, last.p_device_h_t_, sizeof(float) * H * ng, hipMemcpyDeviceToDevice, stream_),
                        "DecodeStream: copy of the encoder's final h failed");
        HipErrorWrapper(hipMemcpyAsync(dst + (size_t)H * slots, last.p_device_c_t_, sizeof(float) * H * ng,
                                       hipMemcpyDeviceToDevice, stream_),
                        "DecodeStream: copy of the encoder's final c failed");
      }
      HipErrorWrapper(hipEventRecord(stream_events_[2 * g + 1], stream_), "DecodeStream: event record failed");
    }
    // ---- groups whose first sentence enters at this tick: their encoder has to be done -----------
    for (int g : encode_at[t])
      HipErrorWrapper(hipStreamWaitEvent(stream_, stream_events_[2 * g + 1], 0), "DecodeStream: wait failed");
    // ---- sentences that enter at this tick --------------------------------------------------------
    const std::vector<int> &now = adm_at[t];
    for (size_t at = 0; at < now.size();) {
      // one launch per group of the ring (the state tensors of a launch come from one slab)
      lh_stream_admission q[LH_STREAM_ADMIT_MAX];
      const int r = adm[now[at]].group % kRing;
      int m = 0;
      while (at < now.size() && m < LH_STREAM_ADMIT_MAX && adm[now[at]].group % kRing == r) {
        const Admission &a = adm[now[at++]];
        const int len = (int)sentences[a.sentence].size();
        q[m++] = lh_stream_admission{a.slot, a.column, (int)(a.column + r * T_cap * slots), len,
                                     group_S[a.group] - len, a.limit, a.tick};
      }
      for (int l = 0; l < L; ++l) {
        state_src[2 * l] = finals.get() + final_slab * r + (size_t)2 * l * H * slots;
        state_src[2 * l + 1] = state_src[2 * l] + (size_t)H * slots;
      }
      LhErrorWrapper(lh_stream_admit_f32(q, m, beam, B, start_dev.get(), limit_dev.get(),
                                         A.p_device_hs_col_.get(), A.p_device_batch_information_.get(),
                                         state_src, state_dst, 2 * L, zero_dst, has_tild ? 1 : 0, H, slots,
                                         tok_hist.get() + (size_t)t * B, Decoder::start_symbol_,
                                         score_hist.get() + (size_t)t * B, stream_),
                     "DecodeStream admission");
    }
    // ---- one step of every slot ------------------------------------------------------------------------
    stream_layer0_mask_ = mask_table.get() + (size_t)t * B;
    if (capture) {
      attention_node.p_device_alignments_ = ss.align_hist.get() + align_slice * t;
      attention_node.p_device_indices_ = ss.index_hist.get() + align_slice * t;
    }
    ForwardPropTarget(1, tok_hist.get() + (size_t)t * B, B);
    stream_layer0_mask_ = nullptr;
    {
      ProfileScope ps(profiler_, kTagBeamTopK, 4.0 * cfg_.target_vocab_size_ * B);
      LhErrorWrapper(lh_beam_topk_f32(softmax_layer_.GetDistPtr(), cfg_.target_vocab_size_, nullptr,
                                      cfg_.target_vocab_size_, B, K, Decoder::end_symbol_,
                                      decoder_.cand_logp_.get(), decoder_.cand_id_.get(),
                                      decoder_.logp_eof_.get(), stream_),
                     "DecodeStream beam top-k");
    }
    {
      ProfileScope pm(profiler_, kTagBeamMergeGather, 8.0 * K * B + 8.0 * n_swap * H * B);
      LhErrorWrapper(lh_beam_merge_gather_stream_f32(
                         slots, beam, K, t, start_dev.get(), limit_dev.get(), decoder_.cand_logp_.get(),
                         decoder_.cand_id_.get(), decoder_.logp_eof_.get(), score_hist.get() + (size_t)t * B,
                         o.diversity_, o.penalty_, Decoder::start_symbol_, Decoder::end_symbol_,
                         tok_hist.get() + (size_t)(t + 1) * B, bp_hist.get() + (size_t)(t + 1) * B,
                         score_hist.get() + (size_t)(t + 1) * B, fcount_hist.get() + (size_t)t * slots,
                         fbeam_hist.get() + (size_t)t * B, fscore_hist.get() + (size_t)t * B, swap_src,
                         swap_dst, n_swap, H, stream_),
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
  std::vector<float> ahist;
  std::vector<int> ihist;
  if (capture) {
    ahist.resize(align_slice * ticks), ihist.resize(align_slice * ticks);
    ss.align_hist.Download(ahist.data(), ahist.size(), stream_);
    ss.index_hist.Download(ihist.data(), ihist.size(), stream_);
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
      for (int j = 0; j < W; ++j) {
        const size_t at = align_slice * (size_t)(t0 + q) + column + (size_t)B * j;
        const int idx = ihist[at];
        if (idx >= 0 && idx < source_length) (*scores)[idx] += ahist[at];
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
