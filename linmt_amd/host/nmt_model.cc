// NeuralMachineTranslation: model wiring and the forward drivers (scoring and batched beam decode).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <numeric>

#include <cstdlib>

#include "nmt.h"

namespace linmt {

NeuralMachineTranslation::NeuralMachineTranslation(const GlobalConfiguration &cfg) : cfg_(cfg) {
  if (cfg_.embedding_size_ <= 0) cfg_.embedding_size_ = cfg_.lstm_size_;
  HipErrorWrapper(hipStreamCreate(&stream_), "stream creation failed");
  profiler_.stream_ = stream_;
  gemm_workspace_.Alloc(kGemmWorkspaceBytes);
  gemm_ws_ptr_ = gemm_workspace_.get();
  gemm_ws_bytes_ = gemm_workspace_.size();
}

void NeuralMachineTranslation::Gemm(int tag, int rows, int cols, const lh_gemm_seg *segs, int nseg,
                                    int trans_a, int trans_x, float beta, const float *bias, int act,
                                    const int *colmask, float *C, int ldc, const char *what,
                                    int act_rows) {
  if (split_products_ && cfg_.train_mode_ &&
      GemmAsSplitProduct(tag, rows, cols, segs, nseg, trans_a, trans_x, beta, bias, act, colmask, C, ldc,
                         what, act_rows))
    return;
  ProfileScope ps(profiler_, tag, gemm_ws_bytes_, 0, rows, cols, segs, nseg, trans_a, trans_x);
  LhErrorWrapper(lh_gemm_ws_f32(rows, cols, segs, nseg, trans_a, trans_x, 1.f, beta, bias, act,
                                act_rows < 0 ? rows : act_rows,
                                colmask, C, ldc, gemm_ws_ptr_, gemm_ws_bytes_,
                                stream_),
                 what);
}

// A large product as a split product: both operands packed into the model's two scratch buffers by
// one launch, then lh_gemm_split_f32.  false = not worthwhile or not expressible; the caller runs
// the fp32 MFMA product.
bool NeuralMachineTranslation::GemmAsSplitProduct(int tag, int rows, int cols, const lh_gemm_seg *segs,
                                                  int nseg, int trans_a, int trans_x, float beta,
                                                  const float *bias, int act, const int *colmask,
                                                  float *C, int ldc, const char *what, int act_rows) {
  if ((trans_a && trans_x) || nseg < 1 || nseg > 3) return false;
  double k_sum = 0;
  int groups = 0;
  for (int i = 0; i < nseg; ++i) {
    if (i + 1 < nseg && segs[i].K % 8) return false;  // segments sit side by side in whole k-groups
    k_sum += segs[i].K;
    groups += lh_split_kgroups(segs[i].K);
  }
  // packing costs about 10 bytes of traffic per operand element against 2*rows*cols*K flop:
  // 160 * (1/rows + 1/cols) is its share of the product's time at the rates of this GPU
  // (split_min_columns_ == 1, a test aid, takes every product)
  if (split_min_columns_ != 1 &&
      (2.0 * rows * cols * k_sum < 2e10 || 160.0 * (1.0 / rows + 1.0 / cols) > 0.2))
    return false;
  const int total = lh_split_kgroups_padded(groups);
  const size_t a_bytes = lh_split_bytes(rows, total), x_bytes = lh_split_bytes(cols, total);
  if (a_bytes >= (size_t(1) << 32) || x_bytes >= (size_t(1) << 32)) return false;
  if (split_scratch_a_.size() * sizeof(unsigned) < a_bytes || split_scratch_x_.size() * sizeof(unsigned) < x_bytes) {
    Synchronize();  // earlier products may still read the buffers about to be replaced
    if (split_scratch_a_.size() * sizeof(unsigned) < a_bytes) split_scratch_a_.Alloc(a_bytes / sizeof(unsigned));
    if (split_scratch_x_.size() * sizeof(unsigned) < x_bytes) split_scratch_x_.Alloc(x_bytes / sizeof(unsigned));
  }
  lh_split_source src[6];
  int n = 0, off = 0;
  for (int i = 0; i < nseg; ++i) {
    const int g = lh_split_kgroups(segs[i].K), written = i + 1 == nseg ? total - off : g;
    lh_split_source a{}, x{};
    // A is rows x K: stored column by column (rows contiguous) unless transposed
    a.src = segs[i].A, a.ld = segs[i].lda, a.k_contiguous = trans_a ? 1 : 0, a.D = rows, a.K = segs[i].K;
    a.planes = split_scratch_a_.get(), a.kgroups_total = total, a.kg_offset = off, a.kgroups = written;
    // X is K x cols: stored column by column (k contiguous) unless transposed
    x.src = segs[i].X, x.ld = segs[i].ldx, x.k_contiguous = trans_x ? 0 : 1, x.D = cols, x.K = segs[i].K;
    x.planes = split_scratch_x_.get(), x.kgroups_total = total, x.kg_offset = off, x.kgroups = written;
    src[n++] = a;
    src[n++] = x;
    off += g;
  }
  {
    ProfileScope ps(profiler_, kTagSplitPack, 10.0 * ((double)rows + cols) * k_sum);
    LhErrorWrapper(lh_split_pack_f32(src, n, stream_), what);
  }
  char name[160] = {0};
  if (profiler_.Wants(tag))
    LhErrorWrapper(lh_gemm_split_kernel_name(0, rows, cols, name, sizeof(name)), "lh_gemm_split_kernel_name");
  ProfileScope ps(profiler_, tag, name, 2.0 * rows * cols * k_sum);
  LhErrorWrapper(lh_gemm_split_f32(rows, cols, total, split_scratch_a_.get(), split_scratch_x_.get(), 1.f, beta,
                                   bias, act, act_rows < 0 ? rows : act_rows, colmask, C, ldc, stream_),
                 what);
  return true;
}

NeuralMachineTranslation::~NeuralMachineTranslation() {
  if (stream_) (void)hipStreamSynchronize(stream_);
  for (hipEvent_t e : lane_events_) (void)hipEventDestroy(e);
  for (hipEvent_t e : ensemble_events_) (void)hipEventDestroy(e);
  for (size_t l = 1; l < lane_streams_.size(); ++l) {  // lane 0 is stream_
    (void)hipStreamSynchronize(lane_streams_[l]);
    (void)hipStreamDestroy(lane_streams_[l]);
  }
  for (hipEvent_t e : stream_events_) (void)hipEventDestroy(e);
  if (encoder_stream_) {
    (void)hipStreamSynchronize(encoder_stream_);
    (void)hipStreamDestroy(encoder_stream_);
  }
  if (stream_) {
    (void)hipStreamSynchronize(stream_);
    (void)hipStreamDestroy(stream_);
  }
}

void NeuralMachineTranslation::Synchronize() {
  HipErrorWrapper(hipStreamSynchronize(stream_), "stream synchronize failed");
}

// One node per timestep on both sides, minibatch = cfg.minibatch_size_ (deep_rnn.h:249-692).
void NeuralMachineTranslation::InitModel() {
  decode_mode_ = false;
  const int B = cfg_.minibatch_size_, T = cfg_.longest_sentence_, L = cfg_.num_layers_;
  const bool seq2seq = cfg_.sequence_to_sequence_mode_;
  const bool keep = cfg_.train_mode_;  // training keeps i,f,g,o and the looked-up embeddings per step
  if (seq2seq) {
    input_layer_source_.Init(this, true, true, 0, B, T, keep, false);
    for (int l = 1; l < L; ++l) {
      v_hidden_layers_source_.emplace_back(new LstmLayer());
      v_hidden_layers_source_.back()->Init(this, false, true, l, B, T, keep, false);
    }
  }
  input_layer_target_.Init(this, true, false, 0, B, T, keep, false);
  for (int l = 1; l < L; ++l) {
    v_hidden_layers_target_.emplace_back(new LstmLayer());
    v_hidden_layers_target_.back()->Init(this, false, false, l, B, T, keep, false);
  }
  if (cfg_.attention_mode_ && seq2seq) {
    attention_layer_.Init(this, B, T, T);
    LstmLayer &top_src = SourceLayer(L - 1);
    attention_layer_.p_device_total_hs_ = top_src.h_all_.get();
    attention_layer_.hs_step_stride_ = (long long)cfg_.lstm_size_ * B;
    attention_layer_.hs_col_stride_ = cfg_.lstm_size_;
    attention_layer_.use_hs_col_ = false;
    if (cfg_.feed_input_mode_) input_layer_target_.InitFeedInput();
    if (cfg_.train_mode_) attention_layer_.InitTraining();
  }
  softmax_layer_.Init(this, B, T);
  if (cfg_.train_mode_) {
    softmax_layer_.InitTraining();
    p_device_norm_workspace_.Alloc(LH_SUMSQ_WORKSPACE);
    p_device_norms_.Alloc(512);
  }
  // wiring that does not change between minibatches: h_below and h~ pointers
  for (int side = 0; side < (seq2seq ? 2 : 1); ++side) {
    for (int l = 1; l < L; ++l) {
      LstmLayer &below = side == 0 && seq2seq ? SourceLayer(l - 1) : TargetLayer(l - 1);
      LstmLayer &cur = side == 0 && seq2seq ? SourceLayer(l) : TargetLayer(l);
      for (int t = 0; t < T; ++t) cur.v_nodes_[t].p_device_h_t_below_ = below.v_nodes_[t].p_device_h_t_;
    }
  }
  Synchronize();
}

// Source side: n_sent columns, one node per source position (the states are needed by attention);
// target side: ONE node, n_sent*beam columns, previous-state buffers (deep_rnn.h:697-922).
void NeuralMachineTranslation::InitModelDecoding(int n_sent, int beam_size) {
  decode_mode_ = true;
  n_sent_ = n_sent;
  beam_size_ = beam_size;
  const int L = cfg_.num_layers_, T = cfg_.longest_sentence_, H = cfg_.lstm_size_;
  const int B = n_sent * beam_size;
  input_layer_source_.Init(this, true, true, 0, n_sent, T, false, false);
  for (int l = 1; l < L; ++l) {
    v_hidden_layers_source_.emplace_back(new LstmLayer());
    v_hidden_layers_source_.back()->Init(this, false, true, l, n_sent, T, false, false);
    for (int t = 0; t < T; ++t)
      v_hidden_layers_source_.back()->v_nodes_[t].p_device_h_t_below_ =
          SourceLayer(l - 1).v_nodes_[t].p_device_h_t_;
  }
  input_layer_target_.Init(this, true, false, 0, B, 1, false, true);
  for (int l = 1; l < L; ++l) {
    v_hidden_layers_target_.emplace_back(new LstmLayer());
    v_hidden_layers_target_.back()->Init(this, false, false, l, B, 1, false, true);
    v_hidden_layers_target_.back()->v_nodes_[0].p_device_h_t_below_ =
        TargetLayer(l - 1).v_nodes_[0].p_device_h_t_;
  }
  if (cfg_.attention_mode_) {
    attention_layer_.Init(this, B, 1, T);
    LstmLayer &top_src = SourceLayer(L - 1);
    attention_layer_.p_device_total_hs_ = top_src.h_all_.get();
    attention_layer_.hs_step_stride_ = (long long)H * n_sent;
    attention_layer_.hs_col_stride_ = H;
    attention_layer_.use_hs_col_ = true;
    if (cfg_.feed_input_mode_) {
      input_layer_target_.InitFeedInput();
      p_device_h_tild_previous_.Alloc((size_t)H * B);
      p_device_h_tild_previous_.Zero(stream_);
      input_layer_target_.v_nodes_[0].p_device_h_tild_ = p_device_h_tild_previous_.get();
    }
  }
  softmax_layer_.Init(this, B, 1);
  std::vector<int> ones(B, 1), sent(B);
  for (int b = 0; b < B; ++b) sent[b] = b / beam_size;
  p_device_ones_.Alloc(B);
  p_device_ones_.Upload(ones.data(), B, stream_);
  p_device_sentence_of_column_.Alloc(B);
  p_device_sentence_of_column_.Upload(sent.data(), B, stream_);
  if (cfg_.attention_mode_) attention_layer_.p_device_hs_col_.Upload(sent.data(), B, stream_);
  decoder_.Init(beam_size, n_sent, T);
  Synchronize();
}

int NeuralMachineTranslation::GemmAddends(int tag, int rows, int cols, const lh_gemm_seg *segs,
                                          int nseg, float beta, float *C, int ldc,
                                          const float *addend[3], const char *what) {
  if (beta != 0.f && beta != 1.f) throw LinmtError("GemmAddends: beta must be 0 or 1");
  // planes can only replace C when they have C's leading dimension
  const bool can_split = ldc == rows && rows % 4 == 0;
  const int max_planes = !can_split ? 1 : (beta == 0.f ? 3 : 2);
  ProfileScope ps(profiler_, tag, gemm_ws_bytes_, max_planes, rows, cols, segs, nseg, 0, 0);
  int planes = 1;
  LhErrorWrapper(lh_gemm_planes_f32(rows, cols, segs, nseg, 0, 0, beta, C, ldc, gemm_ws_ptr_,
                                    gemm_ws_bytes_, max_planes, &planes, stream_),
                 what);
  int n = 0;
  if (planes == 1 || beta != 0.f) addend[n++] = C;
  if (planes > 1) {
    const float *ws = reinterpret_cast<const float *>(gemm_ws_ptr_);
    for (int p = 0; p < planes; ++p) addend[n++] = ws + (size_t)p * rows * cols;
  }
  for (int i = n; i < 3; ++i) addend[i] = nullptr;
  return n;
}

bool NeuralMachineTranslation::SetParam(const std::string &name, const float *host, size_t n) {
  // "src.<l>.<leaf>", "tgt.<l>.<leaf>", "attn.<leaf>", "softmax.<leaf>"
  const size_t d1 = name.find('.');
  if (d1 == std::string::npos) return false;
  const std::string head = name.substr(0, d1);
  if (head == "attn") return cfg_.attention_mode_ && attention_layer_.SetParam(name.substr(d1 + 1), host, n);
  if (head == "softmax") return softmax_layer_.SetParam(name.substr(d1 + 1), host, n);
  const size_t d2 = name.find('.', d1 + 1);
  if (d2 == std::string::npos) return false;
  const int l = std::atoi(name.substr(d1 + 1, d2 - d1 - 1).c_str());
  if (l < 0 || l >= cfg_.num_layers_) return false;
  const std::string leaf = name.substr(d2 + 1);
  if (head == "src") return cfg_.sequence_to_sequence_mode_ && SourceLayer(l).SetParam(leaf, host, n);
  if (head == "tgt") return TargetLayer(l).SetParam(leaf, host, n);
  return false;
}

bool NeuralMachineTranslation::GetParam(const std::string &name, std::vector<float> *out) {
  const size_t d1 = name.find('.');
  if (d1 == std::string::npos) return false;
  const std::string head = name.substr(0, d1);
  if (head == "attn") return cfg_.attention_mode_ && attention_layer_.GetParam(name.substr(d1 + 1), out);
  if (head == "softmax") return softmax_layer_.GetParam(name.substr(d1 + 1), out);
  const size_t d2 = name.find('.', d1 + 1);
  if (d2 == std::string::npos) return false;
  const int l = std::atoi(name.substr(d1 + 1, d2 - d1 - 1).c_str());
  if (l < 0 || l >= cfg_.num_layers_) return false;
  const std::string leaf = name.substr(d2 + 1);
  if (head == "src") return cfg_.sequence_to_sequence_mode_ && SourceLayer(l).GetParam(leaf, out);
  if (head == "tgt") return TargetLayer(l).GetParam(leaf, out);
  return false;
}

// Teacher-forced forward + log-likelihood of the targets (deep_rnn.h:2173-2317).  Index arrays are
// B x length column-major with -1 padding; source reversed and left-padded, target right-padded
// (input_file_preprocess.cc:633,684-690).
double NeuralMachineTranslation::GetError(const int *p_host_source, int source_length,
                                          const int *p_host_target_in,
                                          const int *p_host_target_out, int target_length,
                                          const int *p_host_batch_information, int minibatch_size) {
  ForwardTeacherForced(p_host_source, source_length, p_host_target_in, p_host_target_out,
                       target_length, p_host_batch_information, minibatch_size, true);
  double loss = 0;
  softmax_layer_.p_device_loss_.Download(&loss, 1, stream_);
  Synchronize();
  profiler_.Collect();
  return loss;
}

void NeuralMachineTranslation::ForwardTeacherForced(const int *p_host_source, int source_length,
                                                    const int *p_host_target_in,
                                                    const int *p_host_target_out, int target_length,
                                                    const int *p_host_batch_information,
                                                    int minibatch_size, bool per_step_loss) {
  if (decode_mode_) throw LinmtError("GetError: model was initialised for decoding");
  const int L = cfg_.num_layers_, B = minibatch_size;
  if (B > cfg_.minibatch_size_ || source_length > cfg_.longest_sentence_ ||
      target_length > cfg_.longest_sentence_)
    throw LinmtError("GetError: minibatch exceeds the allocated size");
  const bool seq2seq = cfg_.sequence_to_sequence_mode_;
  if (seq2seq) {
    for (int l = 0; l < L; ++l)
      SourceLayer(l).PreprocessGpuVocabIndices(p_host_source, source_length, B);
  }
  for (int l = 0; l < L; ++l) TargetLayer(l).PreprocessGpuVocabIndices(p_host_target_in, target_length, B);
  softmax_layer_.PreprocessGpuVocabIndices(p_host_target_out, target_length, B);
  const bool attention = cfg_.attention_mode_ && seq2seq;
  if (attention) {
    attention_layer_.PreprocessMinibatchInformation(p_host_batch_information, B);
    // the batch information is uploaded for B columns: lengths at [0,B), offsets at [B,2B)
    attention_layer_.hs_step_stride_ = (long long)cfg_.lstm_size_ * SourceLayer(L - 1).minibatch_size_;
    attention_layer_.hs_steps_ = source_length;
    attention_layer_.projected_memory_ = false;  // a decoding batch's memory is not this pass's
  }
  softmax_layer_.p_device_loss_.Zero(stream_);

  if (seq2seq) RunSourceSide(source_length, B);
  {
    LstmLayer &L0 = input_layer_target_;
    L0.input_hoisted_ = L0.input_hoistable_ && B == L0.minibatch_size_;
    if (L0.input_hoisted_) L0.ForwardPropInputAllSteps(target_length);
  }
  for (int t = 0; t < target_length; ++t) {
    const size_t step = (size_t)t * B;
    for (int l = 0; l < L; ++l) {
      LstmLayer &Lt = TargetLayer(l);
      LstmNode &n = Lt.v_nodes_[t];
      n.minibatch_size_ = B;
      float *hp, *cp;
      if (t == 0) {
        if (seq2seq) {  // encoder layer l at the last source step (deep_rnn.h:2259-2265)
          hp = SourceLayer(l).v_nodes_[source_length - 1].p_device_h_t_;
          cp = SourceLayer(l).v_nodes_[source_length - 1].p_device_c_t_;
        } else {
          hp = Lt.p_device_init_hidden_vec_.get();
          cp = Lt.p_device_init_cell_vec_.get();
        }
      } else {
        hp = Lt.v_nodes_[t - 1].p_device_h_t_;
        cp = Lt.v_nodes_[t - 1].p_device_c_t_;
      }
      if (l == 0) {
        n.UpdateVectorsForwardGpu(Lt.p_device_input_vocab_indices_full_.get() + step,
                                  Lt.p_device_input_vocab_indices_01_full_.get() + step, hp, cp);
        if (attention && cfg_.feed_input_mode_ && t > 0)
          n.p_device_h_tild_ = attention_layer_.v_nodes_[t - 1].p_device_final_tmp_2_;
      } else {
        n.UpdateVectorsForwardGpu(Lt.p_device_input_vocab_indices_01_full_.get() + step, hp, cp);
        n.p_device_h_t_below_ = UpwardState(TargetLayer(l - 1), t);
      }
      n.ForwardProp();
    }
    float *top = UpwardState(TargetLayer(L - 1), t);
    if (attention) {
      AttentionNode &an = attention_layer_.v_nodes_[t];
      an.minibatch_size_ = B;
      an.p_device_h_t_ = top;
      an.p_device_indices_mask_ = TargetLayer(L - 1).p_device_input_vocab_indices_01_full_.get() + step;
      an.ForwardProp();
      top = an.p_device_final_tmp_2_;
    }
    softmax_layer_.SetHTPtr(t, top);
    softmax_layer_.BackPropPreprocessGpu(top, (int)step);
    if (!per_step_loss) continue;
    // ComputeLossGpu without the per-step host read-back: accumulate on the device
    softmax_layer_.ComputeLogits(top, B);
    ProfileScope px(profiler_, kTagXent, 4.0 * cfg_.target_vocab_size_ * B);
    LhErrorWrapper(
        lh_logsoftmax_xent_f32(softmax_layer_.p_device_outputdist_.get(), cfg_.target_vocab_size_,
                               nullptr, cfg_.target_vocab_size_, B,
                               softmax_layer_.p_device_output_vocab_indices_single_,
                               softmax_layer_.p_device_output_vocab_indices_01_single_,
                               softmax_layer_.p_device_logp_tgt_.get(),
                               softmax_layer_.p_device_loss_.get(), stream_),
        "GetError loss");
  }
}

// Encoder for n_sent sentences at once; ids are n_sent x source_length column-major, reversed and
// left-padded with -1, so that every sentence ends at the last step and padded prefixes keep the
// state at exactly zero (deep_rnn.h:1572-1646 runs one sentence with B = 1).
// Layer l on lane l.  The work is issued layer by layer (so every event is recorded before the
// wait that names it is issued); on the GPU layer l+1 follows layer l one block of timesteps behind.
void NeuralMachineTranslation::RunSourceSideLanes(int source_length, int B) {
  const int L = cfg_.num_layers_, C = kLaneChunkSteps;
  const int chunks = (source_length + C - 1) / C;
  if (lane_streams_.empty()) {
    lane_streams_.assign(L, stream_);
    for (int l = 1; l < L; ++l)
      HipErrorWrapper(hipStreamCreate(&lane_streams_[l]), "encoder lane stream creation failed");
  }
  while (lane_events_.size() < (size_t)L * (chunks + 1) + 1) {
    hipEvent_t e;
    HipErrorWrapper(hipEventCreateWithFlags(&e, hipEventDisableTiming), "encoder lane event creation failed");
    lane_events_.push_back(e);
  }
  auto event = [&](int l, int c) { return lane_events_[1 + (size_t)l * (chunks + 1) + c]; };

  // everything queued so far (index upload, the previous batch) precedes every lane
  HipErrorWrapper(hipEventRecord(lane_events_[0], stream_), "encoder lane fork failed");
  for (int l = 1; l < L; ++l)
    HipErrorWrapper(hipStreamWaitEvent(lane_streams_[l], lane_events_[0], 0), "encoder lane fork failed");

  // lane 0 is the stream the caller is on (DecodeStream runs the encoder beside the decoding
  // steps, on a stream and a workspace of its own); the lanes share the caller's workspace
  hipStream_t const main_stream = stream_;
  char *const ws = gemm_ws_ptr_;
  const size_t ws_bytes = gemm_ws_bytes_;
  const size_t ws_slice = (ws_bytes / L) & ~size_t(255);
  struct Restore {
    NeuralMachineTranslation &m;
    hipStream_t s;
    char *ws;
    size_t ws_bytes;
    ~Restore() {
      m.stream_ = s;
      m.profiler_.stream_ = s;
      m.gemm_ws_ptr_ = ws;
      m.gemm_ws_bytes_ = ws_bytes;
    }
  } restore{*this, main_stream, ws, ws_bytes};

  for (int l = 0; l < L; ++l) {
    LstmLayer &Ls = SourceLayer(l);
    stream_ = l == 0 ? main_stream : lane_streams_[l];
    profiler_.stream_ = stream_;
    gemm_ws_ptr_ = ws + ws_slice * l;
    gemm_ws_bytes_ = ws_slice;
    for (int t = 0; t < source_length; ++t) {
      const size_t step = (size_t)t * B;
      LstmNode &n = Ls.v_nodes_[t];
      n.minibatch_size_ = B;
      float *hp = t == 0 ? Ls.p_device_init_hidden_vec_.get() : Ls.v_nodes_[t - 1].p_device_h_t_;
      float *cp = t == 0 ? Ls.p_device_init_cell_vec_.get() : Ls.v_nodes_[t - 1].p_device_c_t_;
      if (l == 0) {
        n.UpdateVectorsForwardGpu(Ls.p_device_input_vocab_indices_full_.get() + step,
                                  Ls.p_device_input_vocab_indices_01_full_.get() + step, hp, cp);
      } else {
        n.UpdateVectorsForwardGpu(Ls.p_device_input_vocab_indices_01_full_.get() + step, hp, cp);
        n.p_device_h_t_below_ = UpwardState(SourceLayer(l - 1), t);
      }
    }
    Ls.input_hoisted_ = true;
    if (l == 0) Ls.ForwardPropInputAllSteps(source_length);  // embeddings: no layer below to wait for
    for (int c = 0; c < chunks; ++c) {
      const int t0 = c * C, nt = std::min(C, source_length - t0);
      if (l > 0) {
        HipErrorWrapper(hipStreamWaitEvent(stream_, event(l - 1, c), 0), "encoder lane wait failed");
        Ls.ForwardPropInputSteps(t0, nt);
      }
      for (int t = t0; t < t0 + nt; ++t) Ls.v_nodes_[t].ForwardProp();
      HipErrorWrapper(hipEventRecord(event(l, c), stream_), "encoder lane record failed");
    }
  }
  // join: the caller's stream continues after the last block of every layer
  for (int l = 1; l < L; ++l)
    HipErrorWrapper(hipStreamWaitEvent(main_stream, event(l, chunks - 1), 0), "encoder lane join failed");
}

void NeuralMachineTranslation::ForwardPropSource(const int *p_host_source, int source_length,
                                                 int n_sent) {
  const int L = cfg_.num_layers_;
  for (int l = 0; l < L; ++l) SourceLayer(l).PreprocessGpuVocabIndices(p_host_source, source_length, n_sent);
  RunSourceSide(source_length, n_sent);
}

// The source side has no coupling from a layer's step t to the layer above's step t-1, so it runs
// one layer at a time: the layer's input products for all steps in one GEMM, then the recurrence.
void NeuralMachineTranslation::RunSourceSide(int source_length, int B) {
  const int L = cfg_.num_layers_;
  const bool lanes_off = Debug().no_lanes != 0;  // measurement and test aid
  bool lanes = !lanes_off && decode_mode_ && L > 1 && L <= 4 && profiler_.level_ < 2 &&
               source_length > kLaneChunkSteps;
  for (int l = 0; l < L && lanes; ++l)
    lanes = SourceLayer(l).input_hoistable_ && B == SourceLayer(l).minibatch_size_;
  if (lanes) {
    RunSourceSideLanes(source_length, B);
    return;
  }
  for (int l = 0; l < L; ++l) {
    LstmLayer &Ls = SourceLayer(l);
    for (int t = 0; t < source_length; ++t) {
      const size_t step = (size_t)t * B;
      LstmNode &n = Ls.v_nodes_[t];
      n.minibatch_size_ = B;
      float *hp = t == 0 ? Ls.p_device_init_hidden_vec_.get() : Ls.v_nodes_[t - 1].p_device_h_t_;
      float *cp = t == 0 ? Ls.p_device_init_cell_vec_.get() : Ls.v_nodes_[t - 1].p_device_c_t_;
      if (l == 0) {
        n.UpdateVectorsForwardGpu(Ls.p_device_input_vocab_indices_full_.get() + step,
                                  Ls.p_device_input_vocab_indices_01_full_.get() + step, hp, cp);
      } else {
        n.UpdateVectorsForwardGpu(Ls.p_device_input_vocab_indices_01_full_.get() + step, hp, cp);
        n.p_device_h_t_below_ = UpwardState(SourceLayer(l - 1), t);
      }
    }
    // the hoisted GEMM reads / writes the node slices as one matrix: every allocated column in use
    Ls.input_hoisted_ = Ls.input_hoistable_ && B == Ls.minibatch_size_;
    if (Ls.input_hoisted_) Ls.ForwardPropInputAllSteps(source_length);
    for (int t = 0; t < source_length; ++t) Ls.v_nodes_[t].ForwardProp();
  }
}

bool NeuralMachineTranslation::SplitProductsUsable(int curr_index, int minibatch) const {
  if (!split_products_ || !decode_mode_ || apply_dropout_ || cfg_.lstm_size_ % 8) return false;
  if (minibatch < split_min_columns_) return false;
  // the first step of a feed-input model has no h~_{t-1} segment: another operand shape, once per batch
  if (cfg_.feed_input_mode_ && curr_index == 0) return false;
  return true;
}

void NeuralMachineTranslation::ForwardPropTarget(int curr_index, int *p_device_current_indices,
                                                 int minibatch) {
  const int L = cfg_.num_layers_;
  input_layer_target_.v_nodes_[0].index_ = curr_index;  // deep_rnn.h:1760
  split_step_ = SplitProductsUsable(curr_index, minibatch);
  for (int l = 0; l < L; ++l) {
    LstmLayer &Lt = TargetLayer(l);
    LstmNode &n = Lt.v_nodes_[0];
    n.minibatch_size_ = minibatch;
    n.recurrent_hoisted_ = false;
    if (l == 0)
      n.UpdateVectorsForwardGpu(p_device_current_indices,
                                stream_layer0_mask_ ? const_cast<int *>(stream_layer0_mask_) : p_device_ones_.get(),
                                Lt.p_device_h_t_previous_.get(), Lt.p_device_c_t_previous_.get());
    else
      n.UpdateVectorsForwardGpu(p_device_ones_.get(), Lt.p_device_h_t_previous_.get(),
                                Lt.p_device_c_t_previous_.get());
  }
  // Optional regrouping (debug option "grouped_gates"): everything of this step's gate products that the
  // previous step already fixes goes out as one grouped launch -- the first layer whole (its input
  // is a column of the folded embedding table), W_h*h_{t-1} of the layers above -- and each upper
  // layer then only adds M*h_t of the layer below.  Measured on MI355X at H = 1000 it runs at the
  // same rate per flop as the layer-by-layer launches from 192 live columns up and 5-15% faster
  // below 128, which is under 1% of a batch: it stays off unless asked for.
  int first_on_chain = 0;
  if (split_step_) {
    // what the previous step fixes of every layer's packed input: h_{t-1} (and h~_{t-1} for the
    // first layer), in launches of up to LH_SPLIT_PACK_MAX matrices
    const int H = cfg_.lstm_size_, g0 = lh_split_kgroups(H);
    lh_split_source src[LH_SPLIT_PACK_MAX];
    int n = 0;
    auto flush = [&]() {
      if (!n) return;
      ProfileScope ps(profiler_, kTagSplitPack, 10.0 * H * minibatch * n);
      LhErrorWrapper(lh_split_pack_f32(src, n, stream_), "ForwardPropTarget packing the step's inputs");
      n = 0;
    };
    auto add = [&](LstmLayer &Lt, const float *x, int kg_offset, bool last) {
      if (n == LH_SPLIT_PACK_MAX) flush();
      lh_split_source &q = src[n++];
      q = lh_split_source{};
      q.src = x, q.ld = H, q.k_contiguous = 1, q.D = minibatch, q.K = H;
      q.planes = Lt.split_x_planes_.get(), q.kgroups_total = Lt.split_kgroups_;
      q.kg_offset = kg_offset, q.kgroups = last ? Lt.split_kgroups_ - kg_offset : g0;
    };
    for (int l = 0; l < L; ++l) {
      LstmLayer &Lt = TargetLayer(l);
      if (Lt.split_dirty_) Lt.BuildSplitWeights();
      LstmNode &nd = Lt.v_nodes_[0];
      if (l == 0) {
        add(Lt, nd.p_device_h_t_prev_, 0, !Lt.feed_input_mode_);
        if (Lt.feed_input_mode_) add(Lt, nd.p_device_h_tild_, g0, true);
      } else {
        add(Lt, nd.p_device_h_t_prev_, g0, true);
      }
    }
    flush();
  }
  if (!split_step_ && decode_mode_ && !apply_dropout_ && L >= 2 && L <= LH_GATE_GROUP_MAX &&
      Debug().grouped_gates) {
    lh_gate_problem problems[LH_GATE_GROUP_MAX];
    for (int l = 0; l < L; ++l) TargetLayer(l).v_nodes_[0].DescribeRecurrentProblem(l == 0, &problems[l]);
    int runnable = 0;
    char name[160] = {0};
    LhErrorWrapper(lh_gate_gemm_group_plan(cfg_.lstm_size_, minibatch, problems, L, &runnable, name,
                                           sizeof(name)),
                   "lh_gate_gemm_group_plan");
    if (runnable) {
      double k = 0;
      for (int l = 0; l < L; ++l)
        for (int i = 0; i < problems[l].nseg; ++i) k += problems[l].segs[i].K;
      ProfileScope ps(profiler_, kTagGateGemm, name, 2.0 * 4 * cfg_.lstm_size_ * (double)minibatch * k);
      LhErrorWrapper(lh_gate_gemm_group_f32(cfg_.lstm_size_, minibatch, problems, L, stream_),
                     "ForwardPropTarget grouped recurrent gate products");
      first_on_chain = 1;
      for (int l = 1; l < L; ++l) TargetLayer(l).v_nodes_[0].recurrent_hoisted_ = true;
    }
  }
  for (int l = first_on_chain; l < L; ++l) TargetLayer(l).v_nodes_[0].ForwardProp();
  float *top = TargetLayer(L - 1).v_nodes_[0].p_device_h_t_;
  if (cfg_.attention_mode_) {
    AttentionNode &an = attention_layer_.v_nodes_[0];
    an.minibatch_size_ = minibatch;
    an.p_device_h_t_ = top;
    an.p_device_indices_mask_ = p_device_ones_.get();
    an.ForwardProp();
    top = an.p_device_final_tmp_2_;
  }
  softmax_layer_.SetHTPtr(0, top);
  if (split_step_)
    softmax_layer_.ComputeLogitsSplit(top, minibatch);
  else
    softmax_layer_.ComputeLogits(top, minibatch);
  split_step_ = false;
}

int NeuralMachineTranslation::DecodingStateTensors(const float **src, float **dst) {
  const int L = cfg_.num_layers_;
  int n = 0;
  for (int l = 0; l < L; ++l) {
    LstmLayer &Lt = TargetLayer(l);
    src[n] = Lt.v_nodes_[0].p_device_h_t_;
    dst[n++] = Lt.p_device_h_t_previous_.get();
    src[n] = Lt.v_nodes_[0].p_device_c_t_;
    dst[n++] = Lt.p_device_c_t_previous_.get();
  }
  if (cfg_.attention_mode_ && cfg_.feed_input_mode_) {
    src[n] = attention_layer_.v_nodes_[0].p_device_final_tmp_2_;
    dst[n++] = p_device_h_tild_previous_.get();
  }
  return n;
}

void NeuralMachineTranslation::SwapDecodingStates(const int *p_device_backptr, int minibatch) {
  const float *src[LH_GATHER_MAX_TENSORS];
  float *dst[LH_GATHER_MAX_TENSORS];
  const int n = DecodingStateTensors(src, dst);
  ProfileScope ps(profiler_, kTagBeamGather, 8.0 * n * cfg_.lstm_size_ * minibatch);
  LhErrorWrapper(lh_beam_gather_f32(src, dst, n, cfg_.lstm_size_, minibatch, minibatch,
                                    p_device_backptr, stream_),
                 "SwapDecodingStates");
}

// ---------------------------------------------------------------------------------------------
void Decoder::Init(int beam_size, int n_sent, int max_steps) {
  beam_size_ = beam_size;
  n_sent_ = n_sent;
  max_steps_ = max_steps;
  const size_t B = (size_t)beam_size * n_sent, K = beam_size + 1, T = max_steps;
  cand_logp_.Alloc(K * B);
  cand_id_.Alloc(K * B);
  logp_eof_.Alloc(B);
  score_[0].Alloc(B);
  score_[1].Alloc(B);
  limit_.Alloc(n_sent);
  current_indices_.Alloc(B);
  tok_hist_.Alloc(T * B);
  backptr_hist_.Alloc(T * B);
  score_hist_.Alloc(T * B);
  fin_count_hist_.Alloc(T * n_sent);
  fin_beam_hist_.Alloc(T * B);
  fin_score_hist_.Alloc(T * B);
}

// Length normalisation, coverage penalty, minimum-ratio filter, best-first (decoder.h:529-600).
// With alignment export off every alignment-score row is the all-zero vector the reference starts
// from (decoder.h:364-370); with it on the rows are the exported scores, smoothed and normalised in
// place as the reference does (so a later print shows the normalised values).
void Decoder::OutputKBestHypotheses(std::vector<Hypothesis> &hyps, int source_length,
                                    const DecodeOptions &o, SentenceResult *out,
                                    const std::vector<int> *sizes,
                                    const std::function<void(int)> &materialise) {
  // the kept set, worst first: a hypothesis enters while there is room, afterwards only by beating
  // the worst kept one strictly (decoder.h:589-600; which of two exactly equal scores the
  // reference's heap drops first is not defined by its source)
  const size_t keep = (size_t)std::max(1, o.hypotheses_number_);
  std::vector<std::pair<float, int>> kept;
  auto worse = [](const std::pair<float, int> &a, const std::pair<float, int> &b) {
    return a.first != b.first ? a.first < b.first : a.second > b.second;
  };
  for (size_t i = 0; i < hyps.size(); ++i) {
    float s = hyps[i].score;
    const int size = sizes ? (*sizes)[i] : (int)hyps[i].tokens.size();
    if (0 != o.lp_alpha_) {
      const float lp = powf((float)(5 + size), o.lp_alpha_) / powf((float)(5 + 1), o.lp_alpha_);
      s /= lp;
    }
    if (0 != o.cp_beta_) {
      float cp_x_y = 0;
      if (!hyps[i].alignments_scores.empty()) {
        std::vector<std::vector<float>> &as = hyps[i].alignments_scores;
        for (int j = 1; j < size - 1; ++j) {
          float sum = 0;
          for (int k = 0; k < source_length; ++k) {
            as[j][k] += 0.01f;
            sum += as[j][k];
          }
          for (int k = 0; k < source_length; ++k) as[j][k] /= sum;
        }
        for (int k = 0; k < source_length; ++k) {
          float col = 0;
          for (int j = 1; j < size - 1; ++j) col += as[j][k];
          cp_x_y += std::log(std::min(col, 1.0f));
        }
      } else {
        float sum = 0;
        for (int k = 0; k < source_length; ++k) sum += 0.01f;
        const float unit = 0.01f / sum;
        for (int k = 0; k < source_length; ++k) {
          float col = 0;
          for (int j = 1; j < size - 1; ++j) col += unit;
          cp_x_y += std::log(std::min(col, 1.0f));
        }
      }
      cp_x_y *= o.cp_beta_;
      if (cp_x_y < -20) cp_x_y = -20;
      s += cp_x_y;
    }
    const float len_ratio = ((float)size) / source_length;
    if (len_ratio > o.min_decoding_ratio_) {
      if (kept.size() < keep) {
        kept.emplace_back(s, (int)i);
      } else {
        auto lowest = std::min_element(kept.begin(), kept.end(), worse);
        if (lowest->first < s) *lowest = std::make_pair(s, (int)i);
      }
    }
  }
  std::sort(kept.begin(), kept.end(), [&](const std::pair<float, int> &a, const std::pair<float, int> &b) {
    return worse(b, a);
  });
  out->kbest.clear();
  out->kbest_score.clear();
  for (const auto &k : kept) {
    out->kbest.push_back(k.second);
    out->kbest_score.push_back(k.first);
    if (materialise) materialise(k.second);
  }
  const int best = kept.empty() ? -1 : kept[0].second;
  const float best_score = kept.empty() ? 0.f : kept[0].first;
  out->best.clear();
  out->best_viterbi.clear();
  out->best_index = best;
  out->best_score = 0.f;
  if (best >= 0) {
    const std::vector<int> &t = hyps[best].tokens;
    out->best.assign(t.begin() + 1, t.end() - 1);
    if (!hyps[best].viterbi.empty())
      out->best_viterbi.assign(hyps[best].viterbi.begin() + 1, hyps[best].viterbi.end() - 1);
    out->best_score = best_score;
  }
}

void NeuralMachineTranslation::DecodeBatch(const std::vector<std::vector<int>> &sentences,
                                           const DecodeOptions &o,
                                           std::vector<SentenceResult> *results,
                                           const std::vector<NeuralMachineTranslation *> &ensemble,
                                           const std::vector<std::vector<std::vector<int>>> &ensemble_sentences) {
  if (!decode_mode_) throw LinmtError("DecodeBatch: call InitModelDecoding first");
  // EnsembleFactory (decoder.h:1702-1931): every model runs the same columns in lockstep, each on
  // its own stream; this model owns the beam search, the others hand it their distributions.
  std::vector<NeuralMachineTranslation *> models{this};
  for (NeuralMachineTranslation *m : ensemble) {
    if (!m || m == this) throw LinmtError("DecodeBatch: ensemble entries must be other models");
    if (!m->decode_mode_ || m->n_sent_ != n_sent_ || m->beam_size_ != beam_size_ ||
        m->cfg_.target_vocab_size_ != cfg_.target_vocab_size_ ||
        m->cfg_.longest_sentence_ != cfg_.longest_sentence_ ||
        m->cfg_.num_layers_ > LH_GATHER_MAX_TENSORS / 2 - 1)
      throw LinmtError("DecodeBatch: ensemble models must be initialised for decoding with the same "
                       "n_sent, beam, target vocabulary and longest sentence");
    models.push_back(m);
  }
  const int n_models = (int)models.size();
  if (n_models > LH_ENSEMBLE_MAX_MODELS) throw LinmtError("DecodeBatch: too many models");
  if (!ensemble_sentences.empty()) {
    if (ensemble_sentences.size() != ensemble.size())
      throw LinmtError("DecodeBatch: one set of source ids per ensemble model");
    for (const auto &set : ensemble_sentences) {
      if (set.size() != sentences.size()) throw LinmtError("DecodeBatch: ensemble source ids: sentence count differs");
      for (size_t i = 0; i < set.size(); ++i)
        if (set[i].size() != sentences[i].size())
          throw LinmtError("DecodeBatch: ensemble source ids: sentence length differs");
    }
  }
  if (n_models > 1 && cfg_.target_vocab_size_ % 4 != 0)
    throw LinmtError("DecodeBatch: an ensemble needs a target vocabulary that is a multiple of 4");
  const int n = (int)sentences.size();
  int beam = o.beam_size_;
  if (beam > (int)std::sqrt((double)cfg_.target_vocab_size_))  // decoder.h:1662-1664
    beam = (int)std::sqrt((double)cfg_.target_vocab_size_);
  if (n < 1 || n > n_sent_ || beam != beam_size_)
    throw LinmtError("DecodeBatch: batch does not match InitModelDecoding(n_sent, beam)");
  const int longest = cfg_.longest_sentence_;
  std::vector<int> order(n);
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) {
    return sentences[a].size() > sentences[b].size();
  });
  const int S = (int)sentences[order[0]].size();
  if (S < 1 || S > longest) throw LinmtError("DecodeBatch: source sentence length out of range");
  if (sentences[order[n - 1]].empty()) throw LinmtError("DecodeBatch: empty source sentence");

  // reversed, left-padded source block; per-sentence step limits; attention batch information
  std::vector<int> src((size_t)n * S, -1), limit(n), binfo(2 * (size_t)n * beam);
  int max_limit = 0;
  for (int k = 0; k < n; ++k) {
    const std::vector<int> &w = sentences[order[k]];
    const int len = (int)w.size();
    for (int t = 0; t < len; ++t) src[(size_t)(S - len + t) * n + k] = w[len - 1 - t];
    limit[k] = std::min((int)(o.max_decoding_ratio_ * len), longest - 2);  // decoder.h:1734
    max_limit = std::max(max_limit, limit[k]);
    for (int j = 0; j < beam; ++j) {
      binfo[(size_t)k * beam + j] = len;
      binfo[(size_t)n * beam + (size_t)k * beam + j] = S - len;
    }
  }
  const int B = n * beam, K = beam + 1;
  // Host arrays that asynchronous uploads read (together with src, limit and binfo above).  They
  // are declared before the guard below, so however this function is left, every model's stream
  // has drained before any of them is destroyed.
  std::vector<std::vector<int>> src_own, bi_keep;
  std::vector<int> start(B, Decoder::start_symbol_);
  // ... and the host arrays that asynchronous downloads write at the end
  std::vector<int> tok, bp, fcount, fbeam;
  std::vector<float> fscore, bscore;
  std::vector<std::vector<float>> ahists(n_models);
  std::vector<std::vector<int>> ihists(n_models);
  struct DrainStreams {
    std::vector<NeuralMachineTranslation *> &models;
    ~DrainStreams() {
      for (NeuralMachineTranslation *m : models) (void)hipStreamSynchronize(m->stream_);
    }
  } drain_streams{models};
  Decoder &d = decoder_;
  if (max_limit + 1 > d.max_steps_) throw LinmtError("DecodeBatch: too many decoding steps");

  // InitDecoder (decoder.h:334-350): <START> everywhere, scores 0
  d.current_indices_.Upload(start.data(), B, stream_);
  d.score_[0].Zero(stream_);
  d.limit_.Upload(limit.data(), n, stream_);

  // unk_replacement_mode_: the attention node writes every step's alignments and window indices
  // into its own slice of a history instead of the one reused buffer.  (With several models the
  // scores of all of them are added up, decoder.h:1933-1945, so all of them must have attention.)
  bool capture = o.unk_replacement_mode_;
  for (NeuralMachineTranslation *m : models) capture = capture && m->cfg_.attention_mode_;
  struct NodeBuffers {
    float *alignments;
    int *indices;
  };
  std::vector<NodeBuffers> node_buffers(n_models, NodeBuffers{nullptr, nullptr});
  std::vector<size_t> hist_slices(n_models, 0);

  for (int k = 0; k < n_models; ++k) {
    NeuralMachineTranslation &M = *models[k];
    const int H = M.cfg_.lstm_size_, L = M.cfg_.num_layers_;
    if (M.cfg_.attention_mode_) {
      M.attention_layer_.PreprocessMinibatchInformation(binfo.data(), B);
      M.attention_layer_.hs_step_stride_ = (long long)H * M.SourceLayer(L - 1).minibatch_size_;
      M.attention_layer_.hs_steps_ = S;
      if (M.attention_layer_.global_mode_ && S > M.attention_layer_.window_)
        throw LinmtError("DecodeBatch: source longer than the attention window");
    }
    // the encoder layers were allocated for n_sent_ columns; run them on n (ld is lstm_size_, so a
    // smaller batch simply uses the first n columns of every step's buffer)
    if (n != n_sent_ && M.cfg_.attention_mode_)
      M.attention_layer_.hs_step_stride_ = (long long)H * n_sent_;
    if (k > 0 && !ensemble_sentences.empty()) {
      // this model's own ids of the same words, laid out like `src`
      src_own.emplace_back((size_t)n * S, -1);  // kept alive until the streams have been synchronised
      std::vector<int> &own = src_own.back();
      for (int q = 0; q < n; ++q) {
        const std::vector<int> &w = ensemble_sentences[k - 1][order[q]];
        const int len = (int)w.size();
        for (int t = 0; t < len; ++t) own[(size_t)(S - len + t) * n + q] = w[len - 1 - t];
      }
      M.ForwardPropSource(own.data(), S, n);
    } else {
      M.ForwardPropSource(src.data(), S, n);
    }
    if (M.cfg_.attention_mode_)
      M.attention_layer_.BuildProjectedMemory(S, M.SourceLayer(L - 1).h_all_.size());

    // TransferDecodingStatesGpu (layer_input_to_hidden.h:1536-1545): encoder's final (h, c) of
    // layer l, sentence s -> every beam column of s.
    {
      const float *gs[LH_GATHER_MAX_TENSORS];
      float *gd[LH_GATHER_MAX_TENSORS];
      int g = 0;
      for (int l = 0; l < L; ++l) {
        gs[g] = M.SourceLayer(l).v_nodes_[S - 1].p_device_h_t_;
        gd[g++] = M.TargetLayer(l).p_device_h_t_previous_.get();
        gs[g] = M.SourceLayer(l).v_nodes_[S - 1].p_device_c_t_;
        gd[g++] = M.TargetLayer(l).p_device_c_t_previous_.get();
      }
      LhErrorWrapper(lh_beam_gather_f32(gs, gd, g, H, B, n, M.p_device_sentence_of_column_.get(),
                                        M.stream_),
                     "TransferDecodingStatesGpu");
    }
    if (M.cfg_.attention_mode_) {
      AttentionNode &node = M.attention_layer_.v_nodes_[0];
      node_buffers[k] = NodeBuffers{node.p_device_alignments_, node.p_device_indices_};
      hist_slices[k] = (size_t)n_sent_ * beam * M.attention_layer_.window_;
      Decoder &dm = M.decoder_;
      if (capture && dm.align_hist_.size() < hist_slices[k] * d.max_steps_) {
        dm.align_hist_.Alloc(hist_slices[k] * d.max_steps_);
        dm.index_hist_.Alloc(hist_slices[k] * d.max_steps_);
      }
    }
    if (n_models > 1 && M.p_device_ensemble_dist_.size() < (size_t)M.cfg_.target_vocab_size_ * B)
      M.p_device_ensemble_dist_.Alloc((size_t)M.cfg_.target_vocab_size_ * n_sent_ * beam);
  }
  // the nodes get their own buffers back however this function is left
  struct RestoreNodes {
    std::vector<NeuralMachineTranslation *> &models;
    std::vector<NodeBuffers> &buffers;
    ~RestoreNodes() {
      for (size_t k = 0; k < models.size(); ++k)
        if (buffers[k].alignments) {
          AttentionNode &node = models[k]->attention_layer_.v_nodes_[0];
          node.p_device_alignments_ = buffers[k].alignments;
          node.p_device_indices_ = buffers[k].indices;
        }
    }
  } restore_nodes{models, node_buffers};
  // ordering between the models' streams: one event per model ("distribution of this step is
  // ready") and one for the beam step ("tokens and back-pointers of this step are ready")
  if (n_models > 1) {
    while (ensemble_events_.size() < (size_t)n_models + 1) {
      hipEvent_t e;
      HipErrorWrapper(hipEventCreateWithFlags(&e, hipEventDisableTiming), "ensemble event creation failed");
      ensemble_events_.push_back(e);
    }
    // the uploads above (start tokens, scores) precede every model's first step
    HipErrorWrapper(hipEventRecord(ensemble_events_[0], stream_), "ensemble event record failed");
    for (int k = 1; k < n_models; ++k)
      HipErrorWrapper(hipStreamWaitEvent(models[k]->stream_, ensemble_events_[0], 0), "ensemble wait failed");
  }

  std::vector<int> active_at(max_limit + 1);
  int *p_device_step_indices = d.current_indices_.get();  // <START> for every column
  const bool separate_beam_launches = Debug().separate_beam_launches != 0;  // measurement and test aid
  for (int step = 0; step <= max_limit; ++step) {
    int n_active = 0;
    while (n_active < n && limit[n_active] >= step) ++n_active;  // limits are non-increasing
    active_at[step] = n_active;
    const int Ba = n_active * beam;
    if (step == 0 || n_active != active_at[step - 1]) {
      // the batch information is [len_0..len_{Ba-1}, off_0..off_{Ba-1}] for the columns in use, so
      // it is laid out again whenever the number of active columns changes
      bi_keep.emplace_back(2 * (size_t)Ba);  // kept alive until the streams have been synchronised
      std::vector<int> &bi = bi_keep.back();
      for (int b = 0; b < Ba; ++b) {
        bi[b] = binfo[b];
        bi[(size_t)Ba + b] = binfo[(size_t)B + b];
      }
      for (NeuralMachineTranslation *m : models)
        if (m->cfg_.attention_mode_) m->attention_layer_.PreprocessMinibatchInformation(bi.data(), Ba);
    }
    const int V = cfg_.target_vocab_size_;
    for (int k = n_models - 1; k >= 0; --k) {  // the other models first: this one's stream waits for them
      NeuralMachineTranslation &M = *models[k];
      if (capture) {
        AttentionNode &node = M.attention_layer_.v_nodes_[0];
        node.p_device_alignments_ = M.decoder_.align_hist_.get() + hist_slices[k] * step;
        node.p_device_indices_ = M.decoder_.index_hist_.get() + hist_slices[k] * step;
      }
      M.ForwardPropTarget(step, p_device_step_indices, Ba);
      if (n_models > 1) {
        LhErrorWrapper(lh_softmax_fwd_f32(M.softmax_layer_.GetDistPtr(), V, nullptr, V, Ba,
                                          M.p_device_ensemble_dist_.get(), V, M.stream_),
                       "ensemble: model distribution");
        if (k > 0) {
          HipErrorWrapper(hipEventRecord(ensemble_events_[k], M.stream_), "ensemble event record failed");
          HipErrorWrapper(hipStreamWaitEvent(stream_, ensemble_events_[k], 0), "ensemble wait failed");
        }
      }
    }
    if (n_models == 1) {
      ProfileScope ps(profiler_, kTagBeamTopK, 4.0 * cfg_.target_vocab_size_ * Ba);
      LhErrorWrapper(lh_beam_topk_f32(softmax_layer_.GetDistPtr(), cfg_.target_vocab_size_, nullptr,
                                    cfg_.target_vocab_size_, Ba, K, Decoder::end_symbol_,
                                    d.cand_logp_.get(), d.cand_id_.get(), d.logp_eof_.get(), stream_),
                   "beam top-k");
    } else {
      // EnsemblesModels (decoder.h:1910-1931) + the per-column selection of ExpandHypothesis
      const float *dist[LH_ENSEMBLE_MAX_MODELS];
      for (int k = 0; k < n_models; ++k) dist[k] = models[k]->p_device_ensemble_dist_.get();
      ProfileScope ps(profiler_, kTagBeamTopK, 4.0 * n_models * V * Ba);
      LhErrorWrapper(lh_beam_topk_ensemble_f32(dist, n_models, V, V, Ba, K, Decoder::end_symbol_,
                                               d.cand_logp_.get(), d.cand_id_.get(),
                                               d.logp_eof_.get(), stream_),
                     "ensemble beam top-k");
    }
    const size_t off = (size_t)step * B;
    // One model: the merge and the move of the surviving hypotheses' states are one launch.
    const bool merge_and_swap = n_models == 1 && step < max_limit && beam <= 256 && !separate_beam_launches;
    if (merge_and_swap) {
      const float *gs[LH_GATHER_MAX_TENSORS];
      float *gd[LH_GATHER_MAX_TENSORS];
      const int g = DecodingStateTensors(gs, gd);
      ProfileScope pm(profiler_, kTagBeamMergeGather, 8.0 * K * Ba + 8.0 * g * cfg_.lstm_size_ * Ba);
      LhErrorWrapper(
          lh_beam_merge_gather_f32(n_active, beam, K, step, d.limit_.get(), d.cand_logp_.get(),
                                   d.cand_id_.get(), d.logp_eof_.get(),
                                   step == 0 ? d.score_[0].get() : d.score_hist_.get() + off - B,
                                   o.diversity_, o.penalty_, Decoder::start_symbol_,
                                   Decoder::end_symbol_, d.tok_hist_.get() + off,
                                   d.backptr_hist_.get() + off, d.score_hist_.get() + off,
                                   d.fin_count_hist_.get() + (size_t)step * n,
                                   d.fin_beam_hist_.get() + off, d.fin_score_hist_.get() + off, gs, gd,
                                   g, cfg_.lstm_size_, stream_),
          "beam merge and state swap");
      p_device_step_indices = d.tok_hist_.get() + off;
      continue;
    }
    {
      ProfileScope pm(profiler_, kTagBeamMerge, 8.0 * K * Ba);
      LhErrorWrapper(
          lh_beam_merge_f32(n_active, beam, K, step, d.limit_.get(), d.cand_logp_.get(),
                            d.cand_id_.get(), d.logp_eof_.get(),
                            step == 0 ? d.score_[0].get() : d.score_hist_.get() + off - B, o.diversity_,
                            o.penalty_, Decoder::start_symbol_, Decoder::end_symbol_,
                            d.tok_hist_.get() + off, d.backptr_hist_.get() + off,
                            d.score_hist_.get() + off, d.fin_count_hist_.get() + (size_t)step * n,
                            d.fin_beam_hist_.get() + off, d.fin_score_hist_.get() + off, stream_),
          "beam merge");
    }
    if (step < max_limit) {
      if (n_models > 1) {
        HipErrorWrapper(hipEventRecord(ensemble_events_[0], stream_), "ensemble event record failed");
        for (int k = 1; k < n_models; ++k)
          HipErrorWrapper(hipStreamWaitEvent(models[k]->stream_, ensemble_events_[0], 0), "ensemble wait failed");
      }
      for (NeuralMachineTranslation *m : models) m->SwapDecodingStates(d.backptr_hist_.get() + off, Ba);
      // the tokens just chosen are the next step's input ids, read in place from the history
      p_device_step_indices = d.tok_hist_.get() + off;
    }
  }

  // one read-back for the whole batch
  const size_t steps = (size_t)max_limit + 1;
  tok.resize(steps * B), bp.resize(steps * B), fcount.resize(steps * n), fbeam.resize(steps * B);
  fscore.resize(steps * B), bscore.resize(steps * B);
  d.score_hist_.Download(bscore.data(), bscore.size(), stream_);
  d.tok_hist_.Download(tok.data(), tok.size(), stream_);
  d.backptr_hist_.Download(bp.data(), bp.size(), stream_);
  d.fin_count_hist_.Download(fcount.data(), fcount.size(), stream_);
  d.fin_beam_hist_.Download(fbeam.data(), fbeam.size(), stream_);
  d.fin_score_hist_.Download(fscore.data(), fscore.size(), stream_);
  for (int k = 0; k < n_models; ++k) {
    NeuralMachineTranslation &M = *models[k];
    if (capture) {
      ahists[k].resize(hist_slices[k] * steps);
      ihists[k].resize(hist_slices[k] * steps);
      M.decoder_.align_hist_.Download(ahists[k].data(), ahists[k].size(), M.stream_);
      M.decoder_.index_hist_.Download(ihists[k].data(), ihists[k].size(), M.stream_);
    } else if (k > 0) {
      // nothing of this model is read back: wait for its stream so that the host arrays it was
      // handed (batch information) and the shared device buffers can be reused
      HipErrorWrapper(hipStreamSynchronize(M.stream_), "ensemble stream synchronisation failed");
    }
  }
  Synchronize();
  profiler_.Collect();

  // Rebuild v_hypotheses_ by walking the back-pointers (equivalent to the row copies of
  // eigen_top_sentences_ in decoder.h:440-471).
  results->assign(n, SentenceResult());
  for (int k = 0; k < n; ++k) {
    SentenceResult &r = (*results)[order[k]];
    r.steps = limit[k] + 1;
    const int c0 = k * beam;
    const int source_length = (int)sentences[order[k]].size();
    // alignment scores over the source positions of `column` at step t, and their arg-max as
    // EnsemblesModels takes it (decoder.h:1946-1961): first strictly largest score above 0
    auto alignment_row = [&](int t, int column, std::vector<float> *scores, int *viterbi) {
      // (the reference's rows have longest_sentence_ entries; those past the sentence stay zero
      // and are never read)
      scores->assign(source_length, 0.f);
      const size_t Ba_t = (size_t)active_at[t] * beam;
      for (int k = 0; k < n_models; ++k) {  // the models' scores are added up (decoder.h:1933-1945)
        const int Wk = models[k]->attention_layer_.window_;
        for (int j = 0; j < Wk; ++j) {
          const size_t at = hist_slices[k] * t + column + Ba_t * j;
          const int idx = ihists[k][at];
          if (idx >= 0 && idx < source_length) (*scores)[idx] += ahists[k][at];
        }
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
      // tokens chosen at steps 0..step-1 along the path that ends in `column` before step `step`;
      // token t+1 was produced by the forward pass of its PARENT column at step t, whose
      // alignments it carries (decoder.h:452-456)
      h->tokens.assign(step + 1, Decoder::start_symbol_);
      if (capture) {
        h->viterbi.assign(step + 2, -20);
        h->alignments_scores.assign(step + 2, std::vector<float>());
      }
      int col = column;
      for (int t = step - 1; t >= 0; --t) {
        h->tokens[t + 1] = tok[(size_t)t * B + col];
        col = bp[(size_t)t * B + col];
        if (capture) alignment_row(t, col, &h->alignments_scores[t + 1], &h->viterbi[t + 1]);
      }
    };
    for (int step = 0; step <= limit[k]; ++step) {
      const int nf = fcount[(size_t)step * n + k];
      for (int f = 0; f < nf; ++f) {
        Hypothesis h;
        const int parent = c0 + fbeam[(size_t)step * B + c0 + f];
        prefix(step, parent, &h);
        h.tokens.push_back(Decoder::end_symbol_);
        if (capture)  // <EOF> itself comes out of the parent's forward pass at this step
          alignment_row(step, parent, &h.alignments_scores[step + 1], &h.viterbi[step + 1]);
        h.score = fscore[(size_t)step * B + c0 + f];
        r.hypotheses.push_back(std::move(h));
      }
    }
    Decoder::OutputKBestHypotheses(r.hypotheses, source_length, o, &r);
    if (capture)  // only the hypotheses kept hold on to their score rows (what a printout shows)
      for (size_t h = 0; h < r.hypotheses.size(); ++h)
        if (std::find(r.kbest.begin(), r.kbest.end(), (int)h) == r.kbest.end())
          std::vector<std::vector<float>>().swap(r.hypotheses[h].alignments_scores);
  }
  // the streams have been synchronised: the histories are complete and no copy is in flight
  last_history_.offset.clear();
  last_history_.n = n;
  last_history_.beam = beam;
  last_history_.steps = (int)steps;
  last_history_.slot_of_sentence.assign(n, 0);
  for (int k = 0; k < n; ++k) last_history_.slot_of_sentence[order[k]] = k;
  last_history_.limit = limit;
  last_history_.tok = std::move(tok);
  last_history_.backptr = std::move(bp);
  last_history_.score = std::move(bscore);
}

}  // namespace linmt
