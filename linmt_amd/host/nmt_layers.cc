// LSTM, attention and softmax layer classes: parameter storage and the per-node forward bodies,
// each a short ordered list of launches into liblinmt_hip.so on the model's single stream.
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "nmt.h"

namespace linmt {

namespace {

int GateIndex(char g) {  // stacked order i, f, c', o
  switch (g) {
    case 'i': return 0;
    case 'f': return 1;
    case 'c': return 2;
    case 'o': return 3;
    default: return -1;
  }
}

// Host H x K column-major block <-> rows [gate*H, (gate+1)*H) of a stacked 4H x K device matrix.
void UploadGateBlock(DeviceArray<float> &stack, int gate, int H, int K, const float *host,
                     hipStream_t s) {
  HipErrorWrapper(hipMemcpy2DAsync(stack.get() + (size_t)gate * H, sizeof(float) * 4 * H, host,
                                   sizeof(float) * H, sizeof(float) * H, K, hipMemcpyHostToDevice, s),
                  "parameter upload failed");
}
void DownloadGateBlock(const DeviceArray<float> &stack, int gate, int H, int K, float *host,
                       hipStream_t s) {
  HipErrorWrapper(hipMemcpy2DAsync(host, sizeof(float) * H, stack.get() + (size_t)gate * H,
                                   sizeof(float) * 4 * H, sizeof(float) * H, K,
                                   hipMemcpyDeviceToHost, s),
                  "parameter download failed");
}

bool SetFlat(DeviceArray<float> &a, const float *host, size_t n, hipStream_t s) {
  if (n != a.size()) return false;
  a.Upload(host, n, s);
  return true;
}
bool GetFlat(const DeviceArray<float> &a, std::vector<float> *out, hipStream_t s) {
  out->resize(a.size());
  a.Download(out->data(), a.size(), s);
  HipErrorWrapper(hipStreamSynchronize(s), "parameter download failed");
  return true;
}

}  // namespace

// ---------------------------------------------------------------------------------------------
void LstmLayer::Init(NeuralMachineTranslation *model, bool input_layer, bool source_side,
                     int layer_number, int minibatch_size, int num_nodes, bool keep_gates,
                     bool with_previous_state) {
  p_neural_mt_ = model;
  const GlobalConfiguration &cfg = model->cfg_;
  hipStream_t s = model->stream_;
  input_layer_mode_ = input_layer;
  source_side_mode_ = source_side;
  layer_number_ = layer_number;
  lstm_size_ = cfg.lstm_size_;
  const int E = cfg.embedding_size_ > 0 ? cfg.embedding_size_ : cfg.lstm_size_;
  input_size_ = input_layer ? E : lstm_size_;
  vocab_size_ = source_side ? cfg.source_vocab_size_ : cfg.target_vocab_size_;
  minibatch_size_ = minibatch_size;
  num_nodes_ = num_nodes;
  keep_gates_ = keep_gates;
  const size_t H = lstm_size_, B = minibatch_size;

  if (input_layer) p_device_w_.Alloc((size_t)input_size_ * vocab_size_);
  p_device_m_stack_.Alloc(4 * H * input_size_);
  p_device_w_h_stack_.Alloc(4 * H * H);
  p_device_b_stack_.Alloc(4 * H);
  p_device_m_stack_.Zero(s);
  p_device_w_h_stack_.Zero(s);
  p_device_b_stack_.Zero(s);

  p_device_init_hidden_vec_.Alloc(H * B);
  p_device_init_cell_vec_.Alloc(H * B);
  p_device_init_hidden_vec_.Zero(s);
  p_device_init_cell_vec_.Zero(s);
  h_all_.Alloc(H * B * num_nodes);
  c_all_.Alloc(H * B * num_nodes);
  if (keep_gates) gates_all_.Alloc(4 * H * B * num_nodes);
  // every step's input is known up front on the source side and for the teacher-forced target
  // input layer (num_nodes > 1); a decoding target layer has a single node
  input_hoistable_ = num_nodes > 1 && (source_side || input_layer);
  if (input_layer)
    lookup_all_.Alloc((size_t)input_size_ * B * (keep_gates || input_hoistable_ ? num_nodes : 1));
  if (input_hoistable_) pre_x_all_.Alloc(4 * H * B * num_nodes);
  preact_.Alloc(4 * H * B);
  if (with_previous_state) {
    p_device_h_t_previous_.Alloc(H * B);
    p_device_c_t_previous_.Alloc(H * B);
  }
  p_device_input_vocab_indices_full_.Alloc(B * (size_t)cfg.longest_sentence_);
  p_device_input_vocab_indices_01_full_.Alloc(B * (size_t)cfg.longest_sentence_);

  v_nodes_.assign(num_nodes, LstmNode());
  for (int i = 0; i < num_nodes; ++i) {
    LstmNode &n = v_nodes_[i];
    n.index_ = i;
    n.p_layer_ = this;
    n.minibatch_size_ = minibatch_size;
    n.p_device_h_t_ = h_all_.get() + H * B * i;
    n.p_device_c_t_ = c_all_.get() + H * B * i;
    n.p_device_gates_ = keep_gates ? gates_all_.get() + 4 * H * B * i : nullptr;
    if (input_layer)
      n.p_device_sparse_lookup_ =
          lookup_all_.get() + (keep_gates || input_hoistable_ ? (size_t)input_size_ * B * i : 0);
    if (input_hoistable_) n.p_device_pre_x_ = pre_x_all_.get() + 4 * H * B * i;
  }
  if (cfg.train_mode_ && keep_gates) InitTraining();
}

void LstmLayer::InitFeedInput() {
  feed_input_mode_ = true;
  p_device_q_stack_.Alloc(4 * (size_t)lstm_size_ * lstm_size_);
  p_device_q_stack_.Zero(p_neural_mt_->stream_);
  if (p_neural_mt_->cfg_.train_mode_ && keep_gates_) {
    p_device_q_grad_.Alloc(4 * (size_t)lstm_size_ * lstm_size_);
    p_device_q_grad_.Zero(p_neural_mt_->stream_);
    p_device_errn_to_t_h_tild_.Alloc((size_t)lstm_size_ * minibatch_size_);
  }
}

void LstmLayer::PreprocessGpuVocabIndices(const int *p_host_input_vocab_indices, int current_length,
                                          int minibatch_size) {
  const size_t n = (size_t)minibatch_size * current_length;
  if (n > p_device_input_vocab_indices_full_.size())
    throw LinmtError("PreprocessGpuVocabIndices: sentence longer than longest_sentence_");
  hipStream_t s = p_neural_mt_->stream_;
  p_device_input_vocab_indices_full_.Upload(p_host_input_vocab_indices, n, s);
  LhErrorWrapper(lh_preprocess_indices_i32(p_device_input_vocab_indices_full_.get(), (int)n,
                                           p_device_input_vocab_indices_full_.get(),
                                           p_device_input_vocab_indices_01_full_.get(), nullptr, s),
                 "PreprocessGpuVocabIndices");
}

bool LstmLayer::SetParam(const std::string &name, const float *host, size_t n) {
  hipStream_t s = p_neural_mt_->stream_;
  const int H = lstm_size_;
  if (name == "W" || name[0] == 'M') mw_fold_dirty_ = true;
  split_dirty_ = true;
  if (name == "W") return input_layer_mode_ && SetFlat(p_device_w_, host, n, s);
  if (name.size() == 3 && name[0] == 'M' && name[1] == '_') {
    const int g = GateIndex(name[2]);
    if (g < 0 || n != (size_t)H * input_size_) return false;
    UploadGateBlock(p_device_m_stack_, g, H, input_size_, host, s);
    return true;
  }
  if (name.size() == 4 && name.compare(0, 3, "W_h") == 0) {
    const int g = GateIndex(name[3]);
    if (g < 0 || n != (size_t)H * H) return false;
    UploadGateBlock(p_device_w_h_stack_, g, H, H, host, s);
    return true;
  }
  if (name.size() == 3 && name[0] == 'Q' && name[1] == '_') {
    const int g = GateIndex(name[2]);
    if (g < 0 || !feed_input_mode_ || n != (size_t)H * H) return false;
    UploadGateBlock(p_device_q_stack_, g, H, H, host, s);
    return true;
  }
  if (name.size() == 3 && name[0] == 'b' && name[1] == '_') {
    const int g = GateIndex(name[2]);
    if (g < 0 || n != (size_t)H) return false;
    p_device_b_stack_.Upload(host, H, s, (size_t)g * H);
    return true;
  }
  return false;
}

bool LstmLayer::GetParam(const std::string &name, std::vector<float> *out) {
  hipStream_t s = p_neural_mt_->stream_;
  const int H = lstm_size_;
  if (name == "W") return input_layer_mode_ && GetFlat(p_device_w_, out, s);
  const DeviceArray<float> *stack = nullptr;
  int g = -1, K = 0;
  if (name.size() == 3 && name[0] == 'M' && name[1] == '_') { stack = &p_device_m_stack_; g = GateIndex(name[2]); K = input_size_; }
  else if (name.size() == 4 && name.compare(0, 3, "W_h") == 0) { stack = &p_device_w_h_stack_; g = GateIndex(name[3]); K = H; }
  else if (name.size() == 3 && name[0] == 'Q' && name[1] == '_' && feed_input_mode_) { stack = &p_device_q_stack_; g = GateIndex(name[2]); K = H; }
  else if (name.size() == 3 && name[0] == 'b' && name[1] == '_') {
    g = GateIndex(name[2]);
    if (g < 0) return false;
    out->resize(H);
    p_device_b_stack_.Download(out->data(), H, s, (size_t)g * H);
    HipErrorWrapper(hipStreamSynchronize(s), "parameter download failed");
    return true;
  }
  if (!stack || g < 0) return false;
  out->resize((size_t)H * K);
  DownloadGateBlock(*stack, g, H, K, out->data(), s);
  HipErrorWrapper(hipStreamSynchronize(s), "parameter download failed");
  return true;
}

void LstmNode::UpdateVectorsForwardGpu(int *p_device_input_vocab_indices,
                                       int *p_device_input_vocab_indices_01,
                                       float *p_device_h_t_prev, float *p_device_c_t_prev) {
  p_device_input_vocab_indices_ = p_device_input_vocab_indices;
  p_device_input_vocab_indices_01_ = p_device_input_vocab_indices_01;
  p_device_h_t_prev_ = p_device_h_t_prev;
  p_device_c_t_prev_ = p_device_c_t_prev;
}

void LstmNode::UpdateVectorsForwardGpu(int *p_device_input_vocab_indices_01,
                                       float *p_device_h_t_prev, float *p_device_c_t_prev) {
  p_device_input_vocab_indices_01_ = p_device_input_vocab_indices_01;
  p_device_h_t_prev_ = p_device_h_t_prev;
  p_device_c_t_prev_ = p_device_c_t_prev;
}

// ---- decoding with split products ---------------------------------------------------------------
// The stacked gate matrices of a target step, side by side in the order of the packed input:
// [M | W_h] for a layer that reads the layer below, [W_h | Q] (or [W_h]) for the first layer, whose
// input product is a column of the folded embedding table.
void LstmLayer::BuildSplitWeights() {
  NeuralMachineTranslation &M = *p_neural_mt_;
  const int H = lstm_size_;
  if (source_side_mode_ || H % 8 || (!input_layer_mode_ && input_size_ != H))
    throw LinmtError("LstmLayer::BuildSplitWeights: a target layer with H a multiple of 8");
  const float *mat[2] = {input_layer_mode_ ? p_device_w_h_stack_.get() : p_device_m_stack_.get(),
                         input_layer_mode_ ? p_device_q_stack_.get() : p_device_w_h_stack_.get()};
  const int n = input_layer_mode_ && !feed_input_mode_ ? 1 : 2;
  const int g0 = lh_split_kgroups(H);
  split_kgroups_ = lh_split_kgroups_padded(n * g0);
  const size_t wn = lh_split_bytes(lh_split_gate_rows(H), split_kgroups_) / sizeof(unsigned);
  const size_t xn = lh_split_bytes(minibatch_size_, split_kgroups_) / sizeof(unsigned);
  if (split_w_planes_.size() != wn) split_w_planes_.Alloc(wn);
  if (split_x_planes_.size() != xn) {
    split_x_planes_.Alloc(xn);
    split_x_planes_.Zero(M.stream_);
  }
  lh_split_source src[2];
  for (int i = 0; i < n; ++i) {
    src[i] = lh_split_source{};
    src[i].src = mat[i], src[i].ld = 4 * H, src[i].k_contiguous = 0, src[i].D = 4 * H, src[i].K = H;
    src[i].gate_H = H, src[i].planes = split_w_planes_.get(), src[i].kgroups_total = split_kgroups_;
    src[i].kg_offset = i * g0, src[i].kgroups = i == n - 1 ? split_kgroups_ - i * g0 : g0;
  }
  LhErrorWrapper(lh_split_pack_f32(src, n, M.stream_), "LstmLayer::BuildSplitWeights");
  split_dirty_ = false;
}

// ForwardProp of a target node whose step runs on split products: the packed input of the layer
// is complete (h_{t-1}, h~_{t-1} packed at the start of the step, h of the layer below written as
// planes by that layer's kernel); one launch does the product, the cell and the planes of h for
// the layer above.
static void ForwardPropSplit(LstmNode &n) {
  LstmLayer &L = *n.p_layer_;
  NeuralMachineTranslation &M = *L.p_neural_mt_;
  const int H = L.lstm_size_, B = n.minibatch_size_;
  const bool feed = L.feed_input_mode_ && 0 != n.index_;
  const float *addend = nullptr;
  if (L.input_layer_mode_) {
    if (L.mw_fold_dirty_) L.BuildEmbeddingFold();
    addend = L.mw_fold_.get();
  }
  LstmLayer *up = L.layer_number_ + 1 < M.cfg_.num_layers_ ? &M.TargetLayer(L.layer_number_ + 1) : nullptr;
  // the layer above reads this layer's h as the first segment of its packed input
  unsigned *h_planes = up ? up->split_x_planes_.get() : nullptr;
  const int hp_total = up ? up->split_kgroups_ : 0, hp_groups = lh_split_kgroups(H);
  const float cell_clip = M.cfg_.clip_cell_mode_ ? M.cfg_.cell_clip_threshold_ : 0.f;
  char name[160] = {0};
  if (M.profiler_.Wants(kTagGateGemm))
    LhErrorWrapper(lh_gemm_split_kernel_name(1, H, B, name, sizeof(name)), "lh_gemm_split_kernel_name");
  const double k = (L.input_layer_mode_ ? (feed ? 2.0 : 1.0) : 2.0) * H;
  ProfileScope ps(M.profiler_, kTagGateGemm, name, 2.0 * 4 * H * (double)B * k);
  LhErrorWrapper(lh_gate_gemm_split_lstm_cell_f32(
                     H, B, L.split_kgroups_, L.split_w_planes_.get(), L.split_x_planes_.get(), addend,
                     4 * H, addend ? n.p_device_input_vocab_indices_ : nullptr, addend ? L.vocab_size_ : 0,
                     L.p_device_b_stack_.get(), n.p_device_c_t_prev_, n.p_device_input_vocab_indices_01_,
                     feed ? 1 : 0, cell_clip, n.p_device_c_t_, n.p_device_h_t_, h_planes, hp_total, 0,
                     hp_groups, M.stream_),
                 "LstmNode::ForwardPropGpu split gate product with cell");
}

// One cell-step: [embedding lookup] -> ONE stacked multi-segment GEMM (x, h_{t-1}[, h~_{t-1}]) ->
// ONE fused cell kernel.  The reference runs 1 + 8..12 SGEMMs + 7 elementwise kernels on 9 streams
// here (src/node_input_to_hidden.h:218-636).
void LstmNode::ForwardProp() {
  LstmLayer &L = *p_layer_;
  NeuralMachineTranslation &M = *L.p_neural_mt_;
  hipStream_t s = M.stream_;
  const int H = L.lstm_size_, B = minibatch_size_;
  // feed input only from the second target step on (node_input_to_hidden.h:325)
  const bool feed = L.feed_input_mode_ && 0 != index_;
  const bool folded = M.decode_mode_ && L.input_layer_mode_ && !L.source_side_mode_;
  if (M.split_step_ && !L.source_side_mode_) {
    ForwardPropSplit(*this);
    return;
  }
  float *pre = L.preact_.get();
  lh_gemm_seg segs[3];
  int nseg = 0;
  float beta = 0.f;
  const float *x = nullptr;  // input operand of the product, when the input term is not an addend
  if (recurrent_hoisted_) {
    // W_h*h_{t-1} is already in preact_ (grouped launch at the start of the step): add M*x
    if (L.input_layer_mode_ || feed || !p_device_h_t_below_)
      throw LinmtError("LstmNode::ForwardProp: a hoisted recurrent product needs an upper layer");
    beta = 1.f;
    x = p_device_h_t_below_;
  } else if (L.input_hoisted_) {
    // M*x of every step is already in pre_x_all_: this step only adds the recurrent products
    pre = p_device_pre_x_;
    beta = 1.f;
  } else if (folded) {
    // M*W[:,token] is a column of the precomputed 4H x V product
    if (L.mw_fold_dirty_) L.BuildEmbeddingFold();
    beta = 1.f;
  } else if (L.input_layer_mode_) {
    const bool drop = M.apply_dropout_ && p_device_dropout_mask_;
    ProfileScope ps(M.profiler_, kTagEmbedLookup, (drop ? 12.0 : 8.0) * L.input_size_ * B);
    LhErrorWrapper(lh_embed_lookup_f32(L.p_device_w_.get(), L.input_size_, L.vocab_size_,
                                       p_device_input_vocab_indices_, B,
                                       drop ? p_device_dropout_mask_ : nullptr,
                                       drop ? M.cfg_.dropout_rate_ : 1.f, p_device_sparse_lookup_, s),
                   "LstmInputHiddenNode::ForwardPropGpu sparse lookup");
    x = p_device_sparse_lookup_;
  } else {
    x = p_device_h_t_below_;
  }
  if (x) segs[nseg++] = {L.p_device_m_stack_.get(), 4 * H, x, L.input_size_, L.input_size_};
  if (!recurrent_hoisted_) segs[nseg++] = {L.p_device_w_h_stack_.get(), 4 * H, p_device_h_t_prev_, H, H};
  if (feed) segs[nseg++] = {L.p_device_q_stack_.get(), 4 * H, p_device_h_tild_, H, H};
  const bool drop_out = M.apply_dropout_ && L.out_dropout_;
  const float cell_clip = M.cfg_.clip_cell_mode_ ? M.cfg_.cell_clip_threshold_ : 0.f;

  // Product and cell in ONE kernel whenever the product runs unsplit; in the inference form (no
  // gate values kept, no dropout) the folded embedding table is read by that kernel too, the
  // training form also stores the gate values and the dropped copy of h for the layer above.
  {
    int fusable = 0;
    char name[160] = {0};
    LhErrorWrapper(lh_gate_gemm_lstm_cell_plan(H, B, segs, nseg, beta != 0.f, M.gemm_ws_bytes_, &fusable,
                                               name, sizeof(name)),
                   "lh_gate_gemm_lstm_cell_plan");
    if (fusable && (p_device_gates_ || drop_out) && !folded) {
      double k = 0;
      for (int i = 0; i < nseg; ++i) k += segs[i].K;
      ProfileScope ps(M.profiler_, kTagGateGemm, name, 2.0 * 4 * H * (double)B * k);
      LhErrorWrapper(lh_gate_gemm_lstm_cell_train_f32(
                         H, B, segs, nseg, beta != 0.f ? pre : nullptr, 4 * H, L.p_device_b_stack_.get(),
                         p_device_c_t_prev_, p_device_input_vocab_indices_01_, feed ? 1 : 0, cell_clip,
                         p_device_gates_, p_device_c_t_, p_device_h_t_,
                         drop_out ? p_device_out_dropout_mask_ : nullptr,
                         drop_out ? M.cfg_.dropout_rate_ : 1.f, drop_out ? p_device_h_t_dropped_ : nullptr,
                         M.gemm_ws_bytes_, s),
                     "LstmNode::ForwardPropGpu gate product with cell (training form)");
      return;
    }
    if (fusable && !p_device_gates_ && !drop_out) {
      double k = 0;
      for (int i = 0; i < nseg; ++i) k += segs[i].K;
      ProfileScope ps(M.profiler_, kTagGateGemm, name, 2.0 * 4 * H * (double)B * k);
      LhErrorWrapper(lh_gate_gemm_lstm_cell_f32(
                         H, B, segs, nseg, beta != 0.f ? (folded ? L.mw_fold_.get() : pre) : nullptr,
                         4 * H, folded ? p_device_input_vocab_indices_ : nullptr,
                         folded ? L.vocab_size_ : 0, L.p_device_b_stack_.get(), p_device_c_t_prev_,
                         p_device_input_vocab_indices_01_, feed ? 1 : 0, cell_clip, p_device_c_t_,
                         p_device_h_t_, M.gemm_ws_bytes_, s),
                     "LstmNode::ForwardPropGpu gate product with cell");
      return;
    }
  }
  if (folded) {
    ProfileScope ps(M.profiler_, kTagEmbedLookup, 8.0 * 4 * H * B);
    LhErrorWrapper(lh_embed_lookup_f32(L.mw_fold_.get(), 4 * H, L.vocab_size_,
                                       p_device_input_vocab_indices_, B, nullptr, 1.f, pre, s),
                   "LstmInputHiddenNode::ForwardPropGpu folded lookup");
  }
  // a split product stays in partial planes: the cell kernel adds them up (no reduction pass)
  const float *addend[3];
  const int n_add = M.GemmAddends(kTagGateGemm, 4 * H, B, segs, nseg, beta, pre, 4 * H, addend,
                                  "LstmNode::ForwardPropGpu stacked gate product");
  ProfileScope pc(M.profiler_, kTagLstmCell,
                  ((p_device_gates_ ? 44.0 : 28.0) + (drop_out ? 8.0 : 0.0) + 16.0 * (n_add - 1)) * H * B);
  LhErrorWrapper(lh_lstm_cell_fwd_f32(H, B, addend[0], addend[1], addend[2],
                                      L.p_device_b_stack_.get(), p_device_c_t_prev_,
                                      p_device_input_vocab_indices_01_, feed ? 1 : 0, cell_clip,
                                      p_device_gates_, p_device_c_t_, p_device_h_t_,
                                      drop_out ? p_device_out_dropout_mask_ : nullptr,
                                      drop_out ? M.cfg_.dropout_rate_ : 1.f,
                                      drop_out ? p_device_h_t_dropped_ : nullptr, s),
                 "LstmNode::ForwardPropGpu fused cell");
}

void LstmNode::DescribeRecurrentProblem(bool complete, lh_gate_problem *q) {
  LstmLayer &L = *p_layer_;
  NeuralMachineTranslation &M = *L.p_neural_mt_;
  const int H = L.lstm_size_;
  *q = lh_gate_problem{};
  q->segs[q->nseg++] = {L.p_device_w_h_stack_.get(), 4 * H, p_device_h_t_prev_, H, H};
  if (!complete) {
    q->out = L.preact_.get();
    q->ld_out = 4 * H;
    return;
  }
  const bool feed = L.feed_input_mode_ && 0 != index_;
  if (!(M.decode_mode_ && L.input_layer_mode_ && !L.source_side_mode_))
    throw LinmtError("DescribeRecurrentProblem: only the first target layer is complete at step start");
  if (L.mw_fold_dirty_) L.BuildEmbeddingFold();
  if (feed) q->segs[q->nseg++] = {L.p_device_q_stack_.get(), 4 * H, p_device_h_tild_, H, H};
  q->cell = 1;
  q->addend = L.mw_fold_.get();
  q->ld_addend = 4 * H;
  q->addend_col = p_device_input_vocab_indices_;
  q->addend_ncols = L.vocab_size_;
  q->bias4h = L.p_device_b_stack_.get();
  q->c_prev = p_device_c_t_prev_;
  q->mask01 = p_device_input_vocab_indices_01_;
  q->sigmoid_f64 = feed ? 1 : 0;
  q->cell_clip = M.cfg_.clip_cell_mode_ ? M.cfg_.cell_clip_threshold_ : 0.f;
  q->c = p_device_c_t_;
  q->h = p_device_h_t_;
}

// M*[x_0 .. x_{steps-1}] in one GEMM (input layer: after ONE lookup of all steps' embeddings).
// Needs the node slices to be contiguous, i.e. the pass must use every allocated column.
void LstmLayer::ForwardPropInputAllSteps(int steps) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  hipStream_t s = M.stream_;
  const int H = lstm_size_, N = minibatch_size_ * steps;
  const float *x_all = nullptr;
  if (input_layer_mode_) {
    const bool drop = M.apply_dropout_ && dropout_mask_all_.size();
    ProfileScope ps(M.profiler_, kTagEmbedLookup, (drop ? 12.0 : 8.0) * input_size_ * N);
    LhErrorWrapper(lh_embed_lookup_f32(p_device_w_.get(), input_size_, vocab_size_,
                                       p_device_input_vocab_indices_full_.get(), N,
                                       drop ? dropout_mask_all_.get() : nullptr,
                                       drop ? M.cfg_.dropout_rate_ : 1.f, lookup_all_.get(), s),
                   "InputToHiddenLayer sparse lookup, all steps");
    x_all = lookup_all_.get();
  } else {
    x_all = v_nodes_[0].p_device_h_t_below_;
  }
  lh_gemm_seg seg{p_device_m_stack_.get(), 4 * H, x_all, input_size_, input_size_};
  M.Gemm(kTagGateGemm, 4 * H, N, &seg, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr, pre_x_all_.get(),
         4 * H, "LstmLayer input products, all steps");
}

// The same for the timesteps [first, first + steps) of a layer above the input layer.
void LstmLayer::ForwardPropInputSteps(int first, int steps) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  if (input_layer_mode_) throw LinmtError("ForwardPropInputSteps: not for the input layer");
  const int H = lstm_size_, N = minibatch_size_ * steps;
  lh_gemm_seg seg{p_device_m_stack_.get(), 4 * H, v_nodes_[first].p_device_h_t_below_, input_size_,
                  input_size_};
  M.Gemm(kTagGateGemm, 4 * H, N, &seg, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
         v_nodes_[first].p_device_pre_x_, 4 * H, "LstmLayer input products, a block of steps");
}

// mw_fold_ = M_stack * W (4H x V): the input product of every vocabulary entry, for decoding.
void LstmLayer::BuildEmbeddingFold() {
  NeuralMachineTranslation &M = *p_neural_mt_;
  const int H = lstm_size_;
  if (mw_fold_.size() == 0) mw_fold_.Alloc((size_t)4 * H * vocab_size_);
  lh_gemm_seg seg{p_device_m_stack_.get(), 4 * H, p_device_w_.get(), input_size_, input_size_};
  M.Gemm(kTagGateGemm, 4 * H, vocab_size_, &seg, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
         mw_fold_.get(), 4 * H, "LstmLayer embedding fold");
  mw_fold_dirty_ = false;
}

// ---------------------------------------------------------------------------------------------
void AttentionLayer::Init(NeuralMachineTranslation *model, int minibatch_size, int num_nodes,
                          int longest_sent) {
  p_neural_mt_ = model;
  const GlobalConfiguration &cfg = model->cfg_;
  hipStream_t s = model->stream_;
  lstm_size_ = cfg.lstm_size_;
  minibatch_size_ = minibatch_size;
  num_nodes_ = num_nodes;
  global_mode_ = cfg.attention_mode_ == 2;
  d_ = cfg.attention_width_;
  window_ = global_mode_ ? longest_sent : 2 * d_ + 1;
  const size_t H = lstm_size_, B = minibatch_size, W = window_;
  p_device_w_a_.Alloc(H * H);
  p_device_w_p_.Alloc(H * H);
  p_device_v_p_.Alloc(H);
  p_device_output_bias_.Alloc(H);
  p_device_w_c_p1_.Alloc(H * H);
  p_device_w_c_p2_.Alloc(H * H);
  for (DeviceArray<float> *a : {&p_device_w_a_, &p_device_w_p_, &p_device_v_p_,
                                &p_device_output_bias_, &p_device_w_c_p1_, &p_device_w_c_p2_})
    a->Zero(s);
  tanh_1_all_.Alloc(H * B * num_nodes);
  sigma_1_all_.Alloc(B * num_nodes);
  p_t_all_.Alloc(B * num_nodes);
  wa_all_.Alloc(H * B * num_nodes);
  alignments_all_.Alloc(B * W * num_nodes);
  cached_exp_all_.Alloc(B * W * num_nodes);
  c_t_all_.Alloc(H * B * num_nodes);
  final_all_.Alloc(H * B * num_nodes);
  indices_all_.Alloc(B * W * num_nodes);
  p_device_batch_information_.Alloc(2 * B);
  p_device_hs_col_.Alloc(B);
  v_nodes_.assign(num_nodes, AttentionNode());
  for (int i = 0; i < num_nodes; ++i) {
    AttentionNode &n = v_nodes_[i];
    n.index_ = i;
    n.p_attention_layer_ = this;
    n.minibatch_size_ = minibatch_size;
    n.p_device_tanh_1_ = tanh_1_all_.get() + H * B * i;
    n.p_device_sigma_1_ = sigma_1_all_.get() + B * i;
    n.p_device_p_t_ = p_t_all_.get() + B * i;
    n.p_device_h_t_wa_cache_ = wa_all_.get() + H * B * i;
    n.p_device_alignments_ = alignments_all_.get() + B * W * i;
    n.p_device_cached_exp_ = cached_exp_all_.get() + B * W * i;
    n.p_device_c_t_ = c_t_all_.get() + H * B * i;
    n.p_device_final_tmp_2_ = final_all_.get() + H * B * i;
    n.p_device_indices_ = indices_all_.get() + B * W * i;
  }
}

void AttentionLayer::PreprocessMinibatchInformation(const int *p_host_batch_information,
                                                    int minibatch_size) {
  // host layout [len_0..len_{B-1}, off_0..off_{B-1}] for the columns in use
  hipStream_t s = p_neural_mt_->stream_;
  if ((size_t)2 * minibatch_size > p_device_batch_information_.size())
    throw LinmtError("PreprocessMinibatchInformation: too many columns");
  p_device_batch_information_.Upload(p_host_batch_information, 2 * (size_t)minibatch_size, s);
}

bool AttentionLayer::SetParam(const std::string &name, const float *host, size_t n) {
  hipStream_t s = p_neural_mt_->stream_;
  if (name == "W_a" || name == "W_p") pa_stack_dirty_ = true;
  if (name == "W_p" || name == "W_c2") pc_stack_dirty_ = true;
  if (name == "W_a") return SetFlat(p_device_w_a_, host, n, s);
  if (name == "W_p") return SetFlat(p_device_w_p_, host, n, s);
  if (name == "v_p") return SetFlat(p_device_v_p_, host, n, s);
  if (name == "b_out") return SetFlat(p_device_output_bias_, host, n, s);
  if (name == "W_c1") return SetFlat(p_device_w_c_p1_, host, n, s);
  if (name == "W_c2") return SetFlat(p_device_w_c_p2_, host, n, s);
  return false;
}

void AttentionLayer::BuildProjectionStack() {
  const size_t H = lstm_size_;
  hipStream_t s = p_neural_mt_->stream_;
  std::vector<float> wa, wp, stack(2 * H * H);
  if (!GetFlat(p_device_w_a_, &wa, s) || !GetFlat(p_device_w_p_, &wp, s))
    throw LinmtError("AttentionLayer::BuildProjectionStack: cannot read W_a / W_p");
  for (size_t k = 0; k < H; ++k)      // column k of the 2H x H stack
    for (size_t i = 0; i < H; ++i) {  // W_p[i,k] above W_a^T[i,k] = W_a[k,i]
      stack[i + k * 2 * H] = wp[i + k * H];
      stack[H + i + k * 2 * H] = wa[k + i * H];
    }
  if (p_device_w_pa_stack_.size() == 0) {
    p_device_w_pa_stack_.Alloc(2 * H * H);
    proj_out_.Alloc(2 * H * (size_t)minibatch_size_);
  }
  p_device_w_pa_stack_.Upload(stack.data(), stack.size(), s);
  HipErrorWrapper(hipStreamSynchronize(s), "projection stack upload failed");  // `stack` is a local
  pa_stack_dirty_ = false;
}

bool AttentionLayer::ProjectedMemoryPossible() const {
  return use_hs_col_ && !global_mode_ && !p_neural_mt_->cfg_.train_mode_ &&
         window_ <= LH_ATTN_PROJECTED_MAX_WINDOW && lstm_size_ <= LH_ATTN_PROJECTED_MAX_H &&
         lstm_size_ % 4 == 0 && hs_col_stride_ == lstm_size_ && hs_step_stride_ % lstm_size_ == 0 &&
         !Debug().no_projected_memory;  // measurement aid: the step's own products
}

void AttentionLayer::BuildOutputStack() {
  const size_t H = lstm_size_;
  hipStream_t s = p_neural_mt_->stream_;
  std::vector<float> wp, wc2, stack(2 * H * H);
  if (!GetFlat(p_device_w_p_, &wp, s) || !GetFlat(p_device_w_c_p2_, &wc2, s))
    throw LinmtError("AttentionLayer::BuildOutputStack: cannot read W_p / W_c2");
  for (size_t k = 0; k < H; ++k) {  // column k of the 2H x H stack: W_p above W_c2
    std::copy(wp.begin() + k * H, wp.begin() + (k + 1) * H, stack.begin() + k * 2 * H);
    std::copy(wc2.begin() + k * H, wc2.begin() + (k + 1) * H, stack.begin() + k * 2 * H + H);
  }
  if (p_device_w_pc_stack_.size() == 0) {
    p_device_w_pc_stack_.Alloc(2 * H * H);
    pc_out_.Alloc(2 * H * (size_t)minibatch_size_);
  }
  p_device_w_pc_stack_.Upload(stack.data(), stack.size(), s);
  HipErrorWrapper(hipStreamSynchronize(s), "output stack upload failed");  // `stack` is a local
  pc_stack_dirty_ = false;
}

// W_a * hs and W_c1 * hs for the source_length timesteps the encoder has just written, every
// allocated column (columns beyond the batch hold older, finite states nobody reads).
void AttentionLayer::BuildProjectedMemory(int source_length, size_t capacity) {
  projected_memory_ = false;
  if (!ProjectedMemoryPossible()) return;
  const int H = lstm_size_;
  const long long cols = hs_step_stride_ / H * source_length;
  if ((size_t)cols * H > capacity)
    throw LinmtError("AttentionLayer::BuildProjectedMemory: more states than the encoder holds");
  if (score_mem_.size() < capacity) {
    score_mem_.Alloc(capacity);
    ctx_mem_.Alloc(capacity);
  }
  NeuralMachineTranslation &M = *p_neural_mt_;
  lh_gemm_seg sa{p_device_w_a_.get(), H, p_device_total_hs_, H, H};
  M.Gemm(kTagAttnProjGemm, H, (int)cols, &sa, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
         score_mem_.get(), H, "AttentionLayer::BuildProjectedMemory W_a hs");
  lh_gemm_seg sc{p_device_w_c_p1_.get(), H, p_device_total_hs_, H, H};
  M.Gemm(kTagAttnOutGemm, H, (int)cols, &sc, 1, 0, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
         ctx_mem_.get(), H, "AttentionLayer::BuildProjectedMemory W_c1 hs");
  projected_memory_ = true;
}

bool AttentionLayer::GetParam(const std::string &name, std::vector<float> *out) {
  hipStream_t s = p_neural_mt_->stream_;
  if (name == "W_a") return GetFlat(p_device_w_a_, out, s);
  if (name == "W_p") return GetFlat(p_device_w_p_, out, s);
  if (name == "v_p") return GetFlat(p_device_v_p_, out, s);
  if (name == "b_out") return GetFlat(p_device_output_bias_, out, s);
  if (name == "W_c1") return GetFlat(p_device_w_c_p1_, out, s);
  if (name == "W_c2") return GetFlat(p_device_w_c_p2_, out, s);
  return false;
}

// Four launches instead of the reference's 5 SGEMMs + 12 kernels (src/layer_attention.h:243-483):
// tanh(W_p ha) [GEMM + tanh epilogue], W_a^T ha [GEMM], the fused core, and
// tanh(W_c1 ctx + W_c2 ha + b_out) * mask [two-segment GEMM + bias/tanh/mask epilogue].
void AttentionNode::ForwardProp() {
  AttentionLayer &A = *p_attention_layer_;
  hipStream_t s = A.p_neural_mt_->stream_;
  const int H = A.lstm_size_, B = minibatch_size_;
  const float *ha = p_device_h_t_;  // no dropout outside training
  Profiler &prof = A.p_neural_mt_->profiler_;
  const float *tanh1 = p_device_tanh_1_, *wa = p_device_h_t_wa_cache_;
  long long proj_col_stride = H;
  if (A.projected_memory_) {
    // decoding over the projected memory: one product, one kernel, h~ out
    if (A.pc_stack_dirty_) A.BuildOutputStack();
    lh_gemm_seg seg{A.p_device_w_pc_stack_.get(), 2 * H, ha, H, H};
    A.p_neural_mt_->Gemm(kTagAttnProjGemm, 2 * H, B, &seg, 1, 0, 0, 0.f, nullptr, LH_ACT_TANH, nullptr,
                         A.pc_out_.get(), 2 * H, "AttentionNode::ForwardProp [W_p ; W_c2] h_t", H);
    ProfileScope ps(prof, kTagAttnCore, 4.0 * B * (2.0 * A.window_ * H + 4.0 * H + 2.0 * A.window_));
    LhErrorWrapper(lh_attn_core_projected_fwd_f32(
                       H, B, A.d_, A.hs_steps_, A.pc_out_.get(), 2 * H, A.p_device_v_p_.get(), ha, H,
                       A.score_mem_.get(), A.ctx_mem_.get(), A.hs_step_stride_, A.hs_col_stride_,
                       A.p_device_hs_col_.get(), A.p_device_batch_information_.get(),
                       p_device_indices_mask_, A.pc_out_.get() + H, 2 * H,
                       A.p_device_output_bias_.get(), p_device_p_t_, p_device_sigma_1_,
                       p_device_indices_, p_device_alignments_, p_device_cached_exp_,
                       p_device_final_tmp_2_, nullptr, s),
                   "AttentionNode::ForwardProp attention over the projected memory");
    return;
  }
  if (!A.global_mode_ && !A.p_neural_mt_->cfg_.train_mode_) {
    if (A.pa_stack_dirty_) A.BuildProjectionStack();
    lh_gemm_seg seg{A.p_device_w_pa_stack_.get(), 2 * H, ha, H, H};
    A.p_neural_mt_->Gemm(kTagAttnProjGemm, 2 * H, B, &seg, 1, 0, 0, 0.f, nullptr, LH_ACT_TANH, nullptr,
                         A.proj_out_.get(), 2 * H, "AttentionNode::ForwardProp [W_p ; W_a^T] h_t", H);
    tanh1 = A.proj_out_.get();
    wa = A.proj_out_.get() + H;
    proj_col_stride = 2 * H;
  } else {
    if (!A.global_mode_) {
      lh_gemm_seg seg{A.p_device_w_p_.get(), H, ha, H, H};
      A.p_neural_mt_->Gemm(kTagAttnProjGemm, H, B, &seg, 1, 0, 0, 0.f, nullptr, LH_ACT_TANH, nullptr,
                           p_device_tanh_1_, H, "AttentionNode::ForwardProp p_device_tanh_1_");
    }
    lh_gemm_seg seg{A.p_device_w_a_.get(), H, ha, H, H};
    A.p_neural_mt_->Gemm(kTagAttnProjGemm, H, B, &seg, 1, 1, 0, 0.f, nullptr, LH_ACT_NONE, nullptr,
                         p_device_h_t_wa_cache_, H,
                         "AttentionNode::ForwardProp p_device_h_t_wa_cache_");
  }
  {
  ProfileScope ps(prof, kTagAttnCore, 4.0 * B * ((double)A.window_ * H + 2.0 * H + 2.0 * A.window_));
  LhErrorWrapper(
      lh_attn_core_fwd_f32(H, B, A.global_mode_ ? -1 : A.d_, A.window_, A.hs_steps_,
                           tanh1, A.p_device_v_p_.get(), wa, proj_col_stride,
                           A.p_device_total_hs_, A.hs_step_stride_, A.hs_col_stride_,
                           A.use_hs_col_ ? A.p_device_hs_col_.get() : nullptr,
                           A.p_device_batch_information_.get(), p_device_indices_mask_,
                           p_device_p_t_, p_device_sigma_1_, p_device_indices_,
                           p_device_alignments_, p_device_cached_exp_, p_device_c_t_, nullptr, s),
      "AttentionNode::ForwardProp attention core");
  }
  lh_gemm_seg segs[2] = {{A.p_device_w_c_p1_.get(), H, p_device_c_t_, H, H},
                         {A.p_device_w_c_p2_.get(), H, ha, H, H}};
  A.p_neural_mt_->Gemm(kTagAttnOutGemm, H, B, segs, 2, 0, 0, 0.f, A.p_device_output_bias_.get(),
                       LH_ACT_TANH, p_device_indices_mask_, p_device_final_tmp_2_, H,
                       "AttentionNode::ForwardProp p_device_final_tmp_2_");
}

// ---------------------------------------------------------------------------------------------
void SoftmaxLayer::Init(NeuralMachineTranslation *model, int minibatch_size, int num_nodes) {
  p_neural_mt_ = model;
  const GlobalConfiguration &cfg = model->cfg_;
  hipStream_t s = model->stream_;
  lstm_size_ = cfg.lstm_size_;
  output_vocab_size_ = cfg.target_vocab_size_;
  minibatch_size_ = minibatch_size;
  current_minibatch_ = minibatch_size;
  num_nodes_ = num_nodes;
  const size_t H = lstm_size_, V = output_vocab_size_, B = minibatch_size;
  p_device_d_.Alloc(V * H);
  p_device_b_d_.Alloc(V);
  p_device_d_.Zero(s);
  p_device_b_d_.Zero(s);
  p_device_outputdist_.Alloc(V * B);
  p_device_logp_tgt_.Alloc(B);
  p_device_loss_.Alloc(1);
  p_device_train_perplexity_.Alloc(1);
  p_device_loss_.Zero(s);
  p_device_train_perplexity_.Zero(s);
  const size_t T = cfg.longest_sentence_;
  p_device_output_vocab_indices_.Alloc(B * T);
  p_device_output_vocab_indices_01_.Alloc(B * T);
  p_device_output_vocab_indices_01_float_.Alloc(B * T);
  v_h_t_.assign(num_nodes, nullptr);
}

void SoftmaxLayer::PreprocessGpuVocabIndices(const int *p_host_output_vocab_indices_target,
                                             int current_target_length, int minibatch_size) {
  const size_t n = (size_t)minibatch_size * current_target_length;
  if (n > p_device_output_vocab_indices_.size())
    throw LinmtError("SoftmaxLayer::PreprocessGpuVocabIndices: target longer than longest_sentence_");
  hipStream_t s = p_neural_mt_->stream_;
  p_device_output_vocab_indices_.Upload(p_host_output_vocab_indices_target, n, s);
  // VocabSoftmaxKernel rewrites -1 -> 0 in place and builds both masks (deep_rnn_kernel.h:144-155)
  LhErrorWrapper(lh_preprocess_indices_i32(p_device_output_vocab_indices_.get(), (int)n,
                                           p_device_output_vocab_indices_.get(),
                                           p_device_output_vocab_indices_01_.get(),
                                           p_device_output_vocab_indices_01_float_.get(), s),
                 "SoftmaxLayer::PreprocessGpuVocabIndices");
  current_minibatch_ = minibatch_size;
}

void SoftmaxLayer::BackPropPreprocessGpu(float *p_device_h_t, int step) {
  // layer_loss.h:630-650: select the target ids / masks of this step (step = t * minibatch)
  p_device_h_t_step_ = p_device_h_t;
  p_device_output_vocab_indices_single_ = p_device_output_vocab_indices_.get() + step;
  p_device_output_vocab_indices_01_single_ = p_device_output_vocab_indices_01_.get() + step;
}

void SoftmaxLayer::ComputeLogits(float *p_device_h_t, int minibatch) {
  // D*h with the bias of MatrixBiasKernel (deep_rnn_kernel.h:525) folded into the epilogue
  lh_gemm_seg seg{p_device_d_.get(), output_vocab_size_, p_device_h_t, lstm_size_, lstm_size_};
  p_neural_mt_->Gemm(kTagLogitsGemm, output_vocab_size_, minibatch, &seg, 1, 0, 0, 0.f,
                     p_device_b_d_.get(), LH_ACT_NONE, nullptr, p_device_outputdist_.get(),
                     output_vocab_size_, "SoftmaxLayer::GetDistributionGpu p_device_outputdist");
}

void SoftmaxLayer::BuildSplitWeights() {
  const int H = lstm_size_, V = output_vocab_size_;
  split_kgroups_ = lh_split_kgroups_padded(lh_split_kgroups(H));
  const size_t dn = lh_split_bytes(V, split_kgroups_) / sizeof(unsigned);
  const size_t hn = lh_split_bytes(minibatch_size_, split_kgroups_) / sizeof(unsigned);
  if (split_d_planes_.size() != dn) split_d_planes_.Alloc(dn);
  if (split_h_planes_.size() != hn) split_h_planes_.Alloc(hn);
  lh_split_source src{};
  src.src = p_device_d_.get(), src.ld = V, src.k_contiguous = 0, src.D = V, src.K = H;
  src.planes = split_d_planes_.get(), src.kgroups_total = split_kgroups_, src.kgroups = split_kgroups_;
  LhErrorWrapper(lh_split_pack_f32(&src, 1, p_neural_mt_->stream_), "SoftmaxLayer::BuildSplitWeights");
  split_dirty_ = false;
}

// ComputeLogits on split products: h~ is packed (one small launch), D was packed when it was set.
void SoftmaxLayer::ComputeLogitsSplit(float *p_device_h_t, int minibatch) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  const int H = lstm_size_, V = output_vocab_size_;
  if (split_dirty_) BuildSplitWeights();
  if (minibatch > minibatch_size_) throw LinmtError("SoftmaxLayer::ComputeLogitsSplit: more columns than allocated");
  {
    lh_split_source src{};
    src.src = p_device_h_t, src.ld = H, src.k_contiguous = 1, src.D = minibatch, src.K = H;
    src.planes = split_h_planes_.get(), src.kgroups_total = split_kgroups_, src.kgroups = split_kgroups_;
    ProfileScope ps(M.profiler_, kTagSplitPack, 10.0 * H * minibatch);
    LhErrorWrapper(lh_split_pack_f32(&src, 1, M.stream_), "SoftmaxLayer::ComputeLogitsSplit packing h");
  }
  char name[160] = {0};
  if (M.profiler_.Wants(kTagLogitsGemm))
    LhErrorWrapper(lh_gemm_split_kernel_name(0, V, minibatch, name, sizeof(name)), "lh_gemm_split_kernel_name");
  ProfileScope ps(M.profiler_, kTagLogitsGemm, name, 2.0 * V * (double)minibatch * H);
  LhErrorWrapper(lh_gemm_split_f32(V, minibatch, split_kgroups_, split_d_planes_.get(), split_h_planes_.get(),
                                   1.f, 0.f, p_device_b_d_.get(), LH_ACT_NONE, 0, nullptr,
                                   p_device_outputdist_.get(), V, M.stream_),
                 "SoftmaxLayer::GetDistributionGpu p_device_outputdist (split products)");
}

void SoftmaxLayer::GetDistributionGpu(float *p_device_h_t) {
  hipStream_t s = p_neural_mt_->stream_;
  const int V = output_vocab_size_, B = current_minibatch_;
  ComputeLogits(p_device_h_t, B);
  ProfileScope ps(p_neural_mt_->profiler_, kTagSoftmax, 8.0 * V * B);
  LhErrorWrapper(lh_softmax_fwd_f32(p_device_outputdist_.get(), V, nullptr, V, B,
                                    p_device_outputdist_.get(), V, s),
                 "SoftmaxLayer::GetDistributionGpu softmax");
  if (training_perplexity_mode_)
    LhErrorWrapper(lh_train_loglik_f32(p_device_outputdist_.get(), V, V, B,
                                       p_device_output_vocab_indices_single_,
                                       p_device_output_vocab_indices_01_single_,
                                       p_device_train_perplexity_.get(), s),
                   "SoftmaxLayer::GetDistributionGpu train perplexity");
}

void SoftmaxLayer::ForwardProp(int index) { GetDistributionGpu(v_h_t_[index]); }

void SoftmaxLayer::GetDistributionGpuDecoderWrapper() { GetDistributionGpu(v_h_t_[0]); }

// GetPerplexityGpu + the host loop of ComputeLossGpu (layer_loss.h:673-750) as one fused pass; the
// masked sum is accumulated on the device into p_device_loss_ and also returned for this step.
double SoftmaxLayer::ComputeLossGpu(int index) {
  hipStream_t s = p_neural_mt_->stream_;
  const int V = output_vocab_size_, B = current_minibatch_;
  double before = 0, after = 0;
  p_device_loss_.Download(&before, 1, s);
  ComputeLogits(v_h_t_[index], B);
  LhErrorWrapper(lh_logsoftmax_xent_f32(p_device_outputdist_.get(), V, nullptr, V, B,
                                        p_device_output_vocab_indices_single_,
                                        p_device_output_vocab_indices_01_single_,
                                        p_device_logp_tgt_.get(), p_device_loss_.get(), s),
                 "SoftmaxLayer::ComputeLossGpu");
  p_device_loss_.Download(&after, 1, s);
  HipErrorWrapper(hipStreamSynchronize(s), "SoftmaxLayer::ComputeLossGpu");
  return after - before;
}

double SoftmaxLayer::GetTrainPerplexity() {
  hipStream_t s = p_neural_mt_->stream_;
  double v = 0;
  p_device_train_perplexity_.Download(&v, 1, s);
  HipErrorWrapper(hipStreamSynchronize(s), "SoftmaxLayer::GetTrainPerplexity");
  p_device_train_perplexity_.Zero(s);
  return v;
}

bool SoftmaxLayer::SetParam(const std::string &name, const float *host, size_t n) {
  hipStream_t s = p_neural_mt_->stream_;
  if (name == "D") {
    split_dirty_ = true;
    return SetFlat(p_device_d_, host, n, s);
  }
  if (name == "b_d") return SetFlat(p_device_b_d_, host, n, s);
  return false;
}

bool SoftmaxLayer::GetParam(const std::string &name, std::vector<float> *out) {
  hipStream_t s = p_neural_mt_->stream_;
  if (name == "D") return GetFlat(p_device_d_, out, s);
  if (name == "b_d") return GetFlat(p_device_b_d_, out, s);
  return false;
}

}  // namespace linmt
