// Training half of the layer classes: backward bodies, gradients over all timesteps, the update.
//
// What changed against the reference, by design:
//   * every gradient that does not sit on the recurrence is computed ONCE per minibatch over all
//     timesteps: the weight gradients d [x;h;h~]^T (K = minibatch x steps instead of `steps` GEMMs
//     with K = minibatch), the bias gradients, the softmax projection and its three gradient
//     products, the attention weight gradients, the error into the embeddings and, on the encoder
//     (which has no feed-input coupling and therefore runs layer by layer), the error handed to
//     the layer below;
//   * per step only the recurrence remains: fused cell backward -> W_h^T d (and M^T d / Q^T d where
//     the next consumer sits inside the same step);
//   * the embedding gradient is a deterministic gather over a per-id position list instead of an
//     atomicAdd scatter; norm, clip, update and clearing are one pass per tensor with the norm read
//     on the device.
#include <algorithm>
#include <unordered_map>

#include "nmt.h"

namespace linmt {

namespace {

int GateIndex(char g) {
  switch (g) {
    case 'i': return 0;
    case 'f': return 1;
    case 'c': return 2;
    case 'o': return 3;
    default: return -1;
  }
}

void Gemm(NeuralMachineTranslation &M, int tag, int rows, int cols, const lh_gemm_seg *segs, int nseg,
          int tA, int tX, float beta, float *C, int ldc, const char *what) {
  M.Gemm(tag, rows, cols, segs, nseg, tA, tX, beta, nullptr, LH_ACT_NONE, nullptr, C, ldc, what);
}

const lh_error_term kNoError{nullptr, 1, 0, 0};

void RowSum(NeuralMachineTranslation &M, const float *A, long long lda, int rows, long long cols,
            float *out) {
  ProfileScope ps(M.profiler_, kTagRowSum, 4.0 * rows * (double)cols);
  LhErrorWrapper(lh_rowsum_acc_f32(A, lda, rows, cols, 1.f, out, M.stream_), "bias gradient");
}

bool DownloadAll(const DeviceArray<float> &a, size_t n, std::vector<float> *out, hipStream_t s) {
  out->resize(n);
  a.Download(out->data(), n, s);
  HipErrorWrapper(hipStreamSynchronize(s), "gradient download failed");
  return true;
}

bool DownloadGate(const DeviceArray<float> &stack, int gate, int H, int K, std::vector<float> *out,
                  hipStream_t s) {
  out->resize((size_t)H * K);
  HipErrorWrapper(hipMemcpy2DAsync(out->data(), sizeof(float) * H, stack.get() + (size_t)gate * H,
                                   sizeof(float) * 4 * H, sizeof(float) * H, K,
                                   hipMemcpyDeviceToHost, s),
                  "gradient download failed");
  HipErrorWrapper(hipStreamSynchronize(s), "gradient download failed");
  return true;
}

}  // namespace

// ---------------------------------------------------------------------------------------------
void LstmLayer::InitTraining() {
  hipStream_t s = p_neural_mt_->stream_;
  const size_t H = lstm_size_, B = minibatch_size_, T = num_nodes_, in = input_size_;
  p_device_m_grad_.Alloc(4 * H * in);
  p_device_w_h_grad_.Alloc(4 * H * H);
  p_device_b_grad_.Alloc(4 * H);
  d_gates_all_.Alloc(4 * H * B * T);
  d_x_all_.Alloc(in * B * T);
  p_device_d_errn_to_t_ht_m1_.Alloc(H * B);
  p_device_d_errn_to_t_ct_m1_.Alloc(H * B);
  d_h_prev_planes_.Alloc(kErrorPlanes * ((H + 3) & ~size_t(3)) * B);
  if (!input_layer_mode_) d_x_planes_.Alloc(kErrorPlanes * ((in + 3) & ~size_t(3)) * B);
  if (input_layer_mode_) {
    p_device_small_w_grad_.Alloc(in * B * T);
    p_device_input_vocab_indices_wgrad_.Alloc(B * T);
    p_device_wgrad_seg_start_.Alloc(B * T + 1);
    p_device_wgrad_seg_cols_.Alloc(B * T);
    p_device_small_w_grad_.Zero(s);
  }
  p_device_m_grad_.Zero(s);
  p_device_w_h_grad_.Zero(s);
  p_device_b_grad_.Zero(s);
  const GlobalConfiguration &cfg = p_neural_mt_->cfg_;
  if (cfg.dropout_mode_) {
    // every layer's h is read through a mask by the consumer above, except the top source layer,
    // whose states the attention nodes read undropped
    out_dropout_ = !(source_side_mode_ && layer_number_ == cfg.num_layers_ - 1);
    if (input_layer_mode_) dropout_mask_all_.Alloc(in * B * T);
    if (out_dropout_) {
      out_dropout_mask_all_.Alloc(H * B * T);
      h_dropped_all_.Alloc(H * B * T);
    }
  }
  for (int i = 0; i < num_nodes_; ++i) {
    v_nodes_[i].p_device_d_gates_ = d_gates_all_.get() + 4 * H * B * i;
    v_nodes_[i].p_device_d_x_ = d_x_all_.get() + in * B * i;
    if (dropout_mask_all_.size()) v_nodes_[i].p_device_dropout_mask_ = dropout_mask_all_.get() + in * B * i;
    if (out_dropout_) {
      v_nodes_[i].p_device_out_dropout_mask_ = out_dropout_mask_all_.get() + H * B * i;
      v_nodes_[i].p_device_h_t_dropped_ = h_dropped_all_.get() + H * B * i;
    }
  }
}

void LstmLayer::GenerateDropoutMasks(int steps, unsigned long long seed) {
  hipStream_t s = p_neural_mt_->stream_;
  const long long B = minibatch_size_;
  if (dropout_mask_all_.size())
    LhErrorWrapper(lh_uniform_f32(dropout_mask_all_.get(), (long long)input_size_ * B * steps,
                                  seed * 2 + 0, s),
                   "dropout mask (embeddings)");
  if (out_dropout_)
    LhErrorWrapper(lh_uniform_f32(out_dropout_mask_all_.get(), (long long)lstm_size_ * B * steps,
                                  seed * 2 + 1, s),
                   "dropout mask (upward output)");
}

void LstmLayer::PreprocessWGrad(const int *p_host_indices, int current_length, int minibatch_size,
                                const int *p_host_wgrad, int len_wgrad) {
  hipStream_t s = p_neural_mt_->stream_;
  const size_t n = (size_t)minibatch_size * current_length;
  if ((size_t)len_wgrad > p_device_input_vocab_indices_wgrad_.size())
    throw LinmtError("PreprocessWGrad: more unique ids than positions");
  std::unordered_map<int, int> slot;
  for (int k = 0; k < len_wgrad; ++k) {
    if (p_host_wgrad[k] < 0 || p_host_wgrad[k] >= vocab_size_ || !slot.emplace(p_host_wgrad[k], k).second)
      throw LinmtError("PreprocessWGrad: the unique-id list holds an invalid or repeated id");
  }
  std::vector<int> count(len_wgrad + 1, 0);
  for (size_t i = 0; i < n; ++i) {
    if (p_host_indices[i] == -1) continue;
    const auto it = slot.find(p_host_indices[i]);
    if (it == slot.end()) throw LinmtError("PreprocessWGrad: an input id is missing from the unique-id list");
    ++count[it->second + 1];
  }
  for (int k = 0; k < len_wgrad; ++k) count[k + 1] += count[k];
  std::vector<int> cols(count[len_wgrad]), fill(count.begin(), count.end() - 1);
  for (size_t i = 0; i < n; ++i)
    if (p_host_indices[i] != -1) cols[fill[slot[p_host_indices[i]]]++] = (int)i;
  w_grad_length_ = len_wgrad;
  p_device_input_vocab_indices_wgrad_.Upload(p_host_wgrad, len_wgrad, s);
  p_device_wgrad_seg_start_.Upload(count.data(), count.size(), s);
  p_device_wgrad_seg_cols_.Upload(cols.data(), cols.size(), s);
  // the uploads read pageable host vectors that die with this call
  HipErrorWrapper(hipStreamSynchronize(s), "PreprocessWGrad");
}

namespace {
// W^T d of one step (rows x B, K = 4H) for a consumer that adds partial planes itself: the product
// goes to C, or stays in up to LstmLayer::kErrorPlanes planes of `planes`; returns what to read.
lh_error_term ErrorProduct(NeuralMachineTranslation &M, const float *W, const float *d_gates, int rows,
                           int B, int H, float *C, DeviceArray<float> &planes, bool leave_planes,
                           const char *what) {
  lh_gemm_seg seg{W, 4 * H, d_gates, 4 * H, 4 * H};
  // (with split products switched on, the model's Gemm() decides which kernel forms the product)
  if (!leave_planes || planes.size() == 0 || M.split_products_) {
    Gemm(M, kTagErrorGemm, rows, B, &seg, 1, 1, 0, 0.f, C, rows, what);
    return lh_error_term{C, 1, 0, rows};
  }
  const size_t bytes = planes.size() * sizeof(float);
  int S = 1;
  {
    ProfileScope ps(M.profiler_, kTagErrorGemm, bytes, LstmLayer::kErrorPlanes, rows, B, &seg, 1, 1, 0);
    LhErrorWrapper(lh_gemm_planes_f32(rows, B, &seg, 1, 1, 0, 0.f, C, rows, planes.get(), bytes,
                                      LstmLayer::kErrorPlanes, &S, M.stream_),
                   what);
  }
  if (S == 1) return lh_error_term{C, 1, 0, rows};
  const int ld = (rows + 3) & ~3;
  return lh_error_term{planes.get(), S, (long long)ld * B, ld};
}
}  // namespace

void LstmNode::BackPropGpu(const lh_error_term &dh_above, bool above_is_lstm, const lh_error_term &dh_next,
                           const float *dc_next, bool batched_dx, bool leave_planes) {
  LstmLayer &L = *p_layer_;
  NeuralMachineTranslation &M = *L.p_neural_mt_;
  hipStream_t s = M.stream_;
  const int H = L.lstm_size_, B = minibatch_size_;
  const float clip = M.cfg_.clip_cell_mode_ ? M.cfg_.error_clip_threshold_ : 0.f;
  const bool drop = M.apply_dropout_ && L.out_dropout_ && dh_above.p != nullptr;
  {
    const int reads = (dh_above.p ? dh_above.planes : 0) + (dh_next.p ? dh_next.planes : 0);
    ProfileScope ps(M.profiler_, kTagLstmCellBwd, ((drop ? 52.0 : 48.0) + 4.0 * reads) * H * B);
    LhErrorWrapper(lh_lstm_cell_bwd_terms_f32(H, B, &dh_above, &dh_next, dc_next, p_device_gates_,
                                              p_device_c_t_, p_device_c_t_prev_,
                                              p_device_input_vocab_indices_01_, above_is_lstm ? clip : 0.f,
                                              clip, drop ? p_device_out_dropout_mask_ : nullptr,
                                              M.cfg_.dropout_rate_, p_device_d_gates_,
                                              L.p_device_d_errn_to_t_ct_m1_.get(), s),
                   "LstmNode::BackPropGpu fused cell backward");
  }
  // the planes the cell kernel has just read are free again
  L.d_h_prev_term_ = ErrorProduct(M, L.p_device_w_h_stack_.get(), p_device_d_gates_, H, B, H,
                                  L.p_device_d_errn_to_t_ht_m1_.get(), L.d_h_prev_planes_, leave_planes,
                                  "LstmNode::BackPropGpu p_device_d_errn_to_t_ht_m1_");
  if (!batched_dx) {
    d_x_term_ = ErrorProduct(M, L.p_device_m_stack_.get(), p_device_d_gates_, L.input_size_, B, H,
                             p_device_d_x_, L.d_x_planes_, leave_planes,
                             "LstmNode::BackPropGpu p_device_d_errn_to_t_h_below_");
  }
  if (L.feed_input_mode_ && 0 != index_) {
    lh_gemm_seg sq{L.p_device_q_stack_.get(), 4 * H, p_device_d_gates_, 4 * H, 4 * H};
    Gemm(M, kTagErrorGemm, H, B, &sq, 1, 1, 0, 0.f, L.p_device_errn_to_t_h_tild_.get(), H,
         "LstmNode::BackPropGpu p_device_errn_to_t_h_tild_");
  }
}

void LstmNode::BackPropPreprocessGpu(float *p_device_d_errn_to_tp1_ht,
                                     float *p_device_d_errn_to_tp1_ct) {
  p_device_d_errn_to_tp1_ht_ = p_device_d_errn_to_tp1_ht;
  p_device_d_errn_to_tp1_ct_ = p_device_d_errn_to_tp1_ct;
}

void LstmNode::BackPropGpu(int index) {
  if (index != index_) throw LinmtError("LstmNode::BackPropGpu: index does not name this node");
  LstmLayer &L = *p_layer_;
  const bool above_is_lstm = L.layer_number_ < L.p_neural_mt_->cfg_.num_layers_ - 1;  // 0 = input layer
  const int H = L.lstm_size_;
  BackPropGpu(lh_error_term{p_device_d_errt_ht_, 1, 0, H}, above_is_lstm,
              lh_error_term{p_device_d_errn_to_tp1_ht_, 1, 0, H}, p_device_d_errn_to_tp1_ct_, false, false);
}

void LstmLayer::BackPropInputAllSteps(int steps) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  const int H = lstm_size_, N = minibatch_size_ * steps;
  lh_gemm_seg sm{p_device_m_stack_.get(), 4 * H, d_gates_all_.get(), 4 * H, 4 * H};
  Gemm(M, kTagErrorGemm, input_size_, N, &sm, 1, 1, 0, 0.f, d_x_all_.get(), input_size_,
       "LstmLayer::BackPropInputAllSteps");
}

void LstmLayer::ComputeGradientsAllSteps(int steps, const float *p_device_h_prev0,
                                         const float *p_device_h_tild_all) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  hipStream_t s = M.stream_;
  const int H = lstm_size_, B = minibatch_size_, in = input_size_;
  const int N = B * steps;
  const float *dG = d_gates_all_.get();
  const float *x_all = input_layer_mode_ ? lookup_all_.get() : v_nodes_[0].p_device_h_t_below_;
  {
    lh_gemm_seg sg{dG, 4 * H, x_all, in, N};
    Gemm(M, kTagWeightGradGemm, 4 * H, in, &sg, 1, 0, 1, 1.f, p_device_m_grad_.get(), 4 * H,
         "LstmLayer::ComputeGradients M");
  }
  {
    // h_{t-1} of step t is h of step t-1: one segment over steps 1.., one for step 0
    lh_gemm_seg sg[2];
    int n = 0;
    if (steps > 1) sg[n++] = {dG + (size_t)4 * H * B, 4 * H, h_all_.get(), H, B * (steps - 1)};
    if (p_device_h_prev0) sg[n++] = {dG, 4 * H, p_device_h_prev0, H, B};
    if (n)
      Gemm(M, kTagWeightGradGemm, 4 * H, H, sg, n, 0, 1, 1.f, p_device_w_h_grad_.get(), 4 * H,
           "LstmLayer::ComputeGradients W_h");
  }
  if (feed_input_mode_ && steps > 1) {
    lh_gemm_seg sg{dG + (size_t)4 * H * B, 4 * H, p_device_h_tild_all, H, B * (steps - 1)};
    Gemm(M, kTagWeightGradGemm, 4 * H, H, &sg, 1, 0, 1, 1.f, p_device_q_grad_.get(), 4 * H,
         "LstmLayer::ComputeGradients Q");
  }
  RowSum(M, dG, 4 * H, 4 * H, N, p_device_b_grad_.get());
  if (input_layer_mode_) {
    BackPropInputAllSteps(steps);
    ProfileScope ps(M.profiler_, kTagEmbedGrad, 4.0 * in * N + 4.0 * in * w_grad_length_);
    const bool drop = M.apply_dropout_ && dropout_mask_all_.size();
    LhErrorWrapper(lh_embed_gather_grad_f32(d_x_all_.get(), in, in, w_grad_length_,
                                            p_device_wgrad_seg_start_.get(),
                                            p_device_wgrad_seg_cols_.get(),
                                            drop ? dropout_mask_all_.get() : nullptr,
                                            M.cfg_.dropout_rate_, 1.f,
                                            p_device_small_w_grad_.get(), in, s),
                   "LstmLayer::ComputeGradients small_w_grad");
  }
}

void LstmLayer::ClearGradients() {
  hipStream_t s = p_neural_mt_->stream_;
  p_device_m_grad_.Zero(s);
  p_device_w_h_grad_.Zero(s);
  p_device_b_grad_.Zero(s);
  if (feed_input_mode_) p_device_q_grad_.Zero(s);
  if (input_layer_mode_) p_device_small_w_grad_.Zero(s);
}

bool LstmLayer::GetGrad(const std::string &name, std::vector<float> *out) {
  hipStream_t s = p_neural_mt_->stream_;
  const int H = lstm_size_;
  if (name == "W")
    return input_layer_mode_ &&
           DownloadAll(p_device_small_w_grad_, (size_t)input_size_ * w_grad_length_, out, s);
  if (name.size() == 3 && name[0] == 'M' && name[1] == '_' && GateIndex(name[2]) >= 0)
    return DownloadGate(p_device_m_grad_, GateIndex(name[2]), H, input_size_, out, s);
  if (name.size() == 4 && name.compare(0, 3, "W_h") == 0 && GateIndex(name[3]) >= 0)
    return DownloadGate(p_device_w_h_grad_, GateIndex(name[3]), H, H, out, s);
  if (name.size() == 3 && name[0] == 'Q' && name[1] == '_' && feed_input_mode_ && GateIndex(name[2]) >= 0)
    return DownloadGate(p_device_q_grad_, GateIndex(name[2]), H, H, out, s);
  if (name.size() == 3 && name[0] == 'b' && name[1] == '_' && GateIndex(name[2]) >= 0) {
    out->resize(H);
    p_device_b_grad_.Download(out->data(), H, s, (size_t)GateIndex(name[2]) * H);
    HipErrorWrapper(hipStreamSynchronize(s), "gradient download failed");
    return true;
  }
  return false;
}

// ---------------------------------------------------------------------------------------------
void AttentionLayer::InitTraining() {
  hipStream_t s = p_neural_mt_->stream_;
  const size_t H = lstm_size_, B = minibatch_size_, T = num_nodes_;
  p_device_w_a_grad_.Alloc(H * H);
  p_device_w_p_grad_.Alloc(H * H);
  p_device_v_p_grad_.Alloc(H);
  p_device_output_bias_grad_.Alloc(H);
  p_device_w_c_p1_grad_.Alloc(H * H);
  p_device_w_c_p2_grad_.Alloc(H * H);
  delta_all_.Alloc(H * B * T);
  h_s_sum_all_.Alloc(H * B * T);
  u_all_.Alloc(H * B * T);
  w_all_.Alloc(H * B * T);
  p_device_errn_to_t_ct_.Alloc(H * B);
  p_device_errn_to_t_ht_p1_.Alloc(H * B);
  p_device_total_hs_error_.Alloc(H * B * T);
  ClearGradients();
  p_device_total_hs_error_.Zero(s);
  for (int i = 0; i < num_nodes_; ++i) {
    AttentionNode &n = v_nodes_[i];
    n.p_device_d_errt_ht_tild_ = delta_all_.get() + H * B * i;
    n.p_device_h_s_sum_ = h_s_sum_all_.get() + H * B * i;
    n.p_device_u_ = u_all_.get() + H * B * i;
    n.p_device_w_ = w_all_.get() + H * B * i;
  }
}

void AttentionLayer::ClearGradients() {
  hipStream_t s = p_neural_mt_->stream_;
  for (DeviceArray<float> *a : {&p_device_w_a_grad_, &p_device_w_p_grad_, &p_device_v_p_grad_,
                                &p_device_output_bias_grad_, &p_device_w_c_p1_grad_,
                                &p_device_w_c_p2_grad_})
    a->Zero(s);
}

// Five launches + the two GEMMs into dha instead of the reference's 9 SGEMM/SGEMV + 8 + 3(2D+1)
// kernels per step; the weight gradients wait for ComputeGradientsAllSteps.
void AttentionNode::BackProp(const float *dht, const float *dht_feed) {
  AttentionLayer &A = *p_attention_layer_;
  NeuralMachineTranslation &M = *A.p_neural_mt_;
  hipStream_t s = M.stream_;
  const int H = A.lstm_size_, B = minibatch_size_;
  const float clip = M.cfg_.clip_cell_mode_ ? M.cfg_.error_clip_threshold_ : 0.f;
  const float *ha = p_device_h_t_;
  {
    ProfileScope ps(M.profiler_, kTagAttnBwd, 16.0 * H * B);
    LhErrorWrapper(lh_attn_delta_f32(H, B, dht, dht_feed, p_device_final_tmp_2_,
                                     p_device_indices_mask_, clip, p_device_d_errt_ht_tild_, s),
                   "AttentionNode::BackProp p_device_d_errt_ht_tild_");
  }
  lh_gemm_seg s1{A.p_device_w_c_p1_.get(), H, p_device_d_errt_ht_tild_, H, H};
  Gemm(M, kTagErrorGemm, H, B, &s1, 1, 1, 0, 0.f, A.p_device_errn_to_t_ct_.get(), H,
       "AttentionNode::BackProp p_device_errn_to_t_ct_");
  lh_gemm_seg s2{A.p_device_w_c_p2_.get(), H, p_device_d_errt_ht_tild_, H, H};
  Gemm(M, kTagErrorGemm, H, B, &s2, 1, 1, 0, 0.f, A.p_device_errn_to_t_ht_p1_.get(), H,
       "AttentionNode::BackProp p_device_errn_to_t_ht_p1_");
  {
    ProfileScope ps(M.profiler_, kTagAttnBwd, 4.0 * B * (3.0 * A.window_ * H + 6.0 * H));
    LhErrorWrapper(
        lh_attn_core_bwd_f32(H, B, A.global_mode_ ? -1 : A.d_, A.window_, A.hs_steps_,
                             A.p_device_errn_to_t_ct_.get(), p_device_tanh_1_, A.p_device_v_p_.get(),
                             p_device_h_t_wa_cache_, A.p_device_total_hs_, A.hs_step_stride_,
                             A.hs_col_stride_, A.p_device_batch_information_.get(), p_device_p_t_,
                             p_device_sigma_1_, p_device_indices_, p_device_alignments_,
                             p_device_cached_exp_, A.p_device_total_hs_error_.get(),
                             p_device_h_s_sum_, p_device_u_, p_device_w_, s),
        "AttentionNode::BackProp attention core");
  }
  if (!A.global_mode_) {
    lh_gemm_seg sp{A.p_device_w_p_.get(), H, p_device_w_, H, H};
    Gemm(M, kTagErrorGemm, H, B, &sp, 1, 1, 0, 1.f, A.p_device_errn_to_t_ht_p1_.get(), H,
         "AttentionNode::BackProp W_p^T");
  }
  lh_gemm_seg sa{A.p_device_w_a_.get(), H, p_device_h_s_sum_, H, H};
  Gemm(M, kTagErrorGemm, H, B, &sa, 1, 0, 0, 1.f, A.p_device_errn_to_t_ht_p1_.get(), H,
       "AttentionNode::BackProp W_a");
  (void)ha;
}

void AttentionLayer::ComputeGradientsAllSteps(int steps, const float *p_device_h_t_all) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  const int H = lstm_size_, N = minibatch_size_ * steps;
  const float *ha = p_device_h_t_all;
  lh_gemm_seg g1{delta_all_.get(), H, c_t_all_.get(), H, N};
  Gemm(M, kTagWeightGradGemm, H, H, &g1, 1, 0, 1, 1.f, p_device_w_c_p1_grad_.get(), H, "attention W_c1 grad");
  lh_gemm_seg g2{delta_all_.get(), H, ha, H, N};
  Gemm(M, kTagWeightGradGemm, H, H, &g2, 1, 0, 1, 1.f, p_device_w_c_p2_grad_.get(), H, "attention W_c2 grad");
  RowSum(M, delta_all_.get(), H, H, N, p_device_output_bias_grad_.get());
  if (!global_mode_) {
    RowSum(M, u_all_.get(), H, H, N, p_device_v_p_grad_.get());
    lh_gemm_seg g3{w_all_.get(), H, ha, H, N};
    Gemm(M, kTagWeightGradGemm, H, H, &g3, 1, 0, 1, 1.f, p_device_w_p_grad_.get(), H, "attention W_p grad");
  }
  lh_gemm_seg g4{ha, H, h_s_sum_all_.get(), H, N};
  Gemm(M, kTagWeightGradGemm, H, H, &g4, 1, 0, 1, 1.f, p_device_w_a_grad_.get(), H, "attention W_a grad");
}

bool AttentionLayer::GetGrad(const std::string &name, std::vector<float> *out) {
  hipStream_t s = p_neural_mt_->stream_;
  const DeviceArray<float> *a = nullptr;
  if (name == "W_a") a = &p_device_w_a_grad_;
  else if (name == "W_p") a = &p_device_w_p_grad_;
  else if (name == "v_p") a = &p_device_v_p_grad_;
  else if (name == "b_out") a = &p_device_output_bias_grad_;
  else if (name == "W_c1") a = &p_device_w_c_p1_grad_;
  else if (name == "W_c2") a = &p_device_w_c_p2_grad_;
  return a && DownloadAll(*a, a->size(), out, s);
}

// ---------------------------------------------------------------------------------------------
void SoftmaxLayer::InitTraining() {
  hipStream_t s = p_neural_mt_->stream_;
  const size_t H = lstm_size_, V = output_vocab_size_, B = minibatch_size_, T = num_nodes_;
  p_device_d_grad_.Alloc(V * H);
  p_device_b_d_grad_.Alloc(V);
  p_device_d_errt_ht_all_.Alloc(H * B * T);
  const size_t budget = (size_t)1 << 29;  // floats: 2 GiB of logits / output errors at a time
  chunk_steps_ = (int)std::max<size_t>(1, std::min<size_t>(T, budget / (V * B)));
  dz_chunk_.Alloc(V * B * chunk_steps_);
  p_device_logp_tgt_.Alloc(B * T);
  ClearGradients();
  (void)s;
}

void SoftmaxLayer::ClearGradients() {
  p_device_d_grad_.Zero(p_neural_mt_->stream_);
  p_device_b_d_grad_.Zero(p_neural_mt_->stream_);
}

void SoftmaxLayer::ForwardBackwardAllSteps(const float *p_device_h_t_all, int steps) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  hipStream_t s = M.stream_;
  const int H = lstm_size_, V = output_vocab_size_, B = current_minibatch_;
  for (int c0 = 0; c0 < steps; c0 += chunk_steps_) {
    const int n = std::min(chunk_steps_, steps - c0), N = B * n;
    const float *h = p_device_h_t_all + (size_t)H * B * c0;
    float *dz = dz_chunk_.get();
    {
      lh_gemm_seg seg{p_device_d_.get(), V, h, H, H};
      M.Gemm(kTagLogitsGemm, V, N, &seg, 1, 0, 0, 0.f, p_device_b_d_.get(), LH_ACT_NONE, nullptr, dz, V,
             "SoftmaxLayer::ForwardProp logits");
    }
    {
      ProfileScope ps(M.profiler_, kTagSoftmaxGrad, 8.0 * V * N);
      LhErrorWrapper(lh_softmax_xent_grad_f32(dz, V, nullptr, V, N,
                                              p_device_output_vocab_indices_.get() + (size_t)B * c0,
                                              p_device_output_vocab_indices_01_.get() + (size_t)B * c0,
                                              dz, V, p_device_logp_tgt_.get(), p_device_loss_.get(), s),
                     "SoftmaxLayer output error");
    }
    lh_gemm_seg sh{p_device_d_.get(), V, dz, V, V};
    Gemm(M, kTagErrorGemm, H, N, &sh, 1, 1, 0, 0.f, p_device_d_errt_ht_all_.get() + (size_t)H * B * c0, H,
         "SoftmaxLayer::GetHTGradientGpu");
    lh_gemm_seg sd{dz, V, h, H, N};
    Gemm(M, kTagWeightGradGemm, V, H, &sd, 1, 0, 1, 1.f, p_device_d_grad_.get(), V,
         "SoftmaxLayer::ComputeDGradientGpu");
    RowSum(M, dz, V, V, N, p_device_b_d_grad_.get());
  }
}

void SoftmaxLayer::BackProp1(int index) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  const int H = lstm_size_, V = output_vocab_size_, B = current_minibatch_;
  if (!p_device_h_t_step_ || p_device_d_errt_ht_all_.size() == 0)
    throw LinmtError("SoftmaxLayer::BackProp1: needs InitTraining and BackPropPreprocessGpu");
  float *dz = p_device_outputdist_.get();
  ComputeLogits(p_device_h_t_step_, B);
  {
    ProfileScope ps(M.profiler_, kTagSoftmaxGrad, 8.0 * V * B);
    LhErrorWrapper(lh_softmax_xent_grad_f32(dz, V, nullptr, V, B, p_device_output_vocab_indices_single_,
                                            p_device_output_vocab_indices_01_single_, dz, V,
                                            p_device_logp_tgt_.get(), p_device_loss_.get(), M.stream_),
                   "SoftmaxLayer::BackProp1 output error");
  }
  lh_gemm_seg sh{p_device_d_.get(), V, dz, V, V};
  Gemm(M, kTagErrorGemm, H, B, &sh, 1, 1, 0, 0.f,
       p_device_d_errt_ht_all_.get() + (size_t)H * minibatch_size_ * index, H,
       "SoftmaxLayer::GetHTGradientGpu");
  dz_index_ = index;
}

void SoftmaxLayer::BackProp2(int index) {
  NeuralMachineTranslation &M = *p_neural_mt_;
  const int H = lstm_size_, V = output_vocab_size_, B = current_minibatch_;
  if (index != dz_index_)
    throw LinmtError("SoftmaxLayer::BackProp2: call it after BackProp1 of the same step");
  const float *dz = p_device_outputdist_.get();
  lh_gemm_seg sd{dz, V, p_device_h_t_step_, H, B};
  Gemm(M, kTagWeightGradGemm, V, H, &sd, 1, 0, 1, 1.f, p_device_d_grad_.get(), V,
       "SoftmaxLayer::ComputeDGradientGpu");
  RowSum(M, dz, V, V, B, p_device_b_d_grad_.get());
  dz_index_ = -1;
}

bool SoftmaxLayer::GetGrad(const std::string &name, std::vector<float> *out) {
  hipStream_t s = p_neural_mt_->stream_;
  if (name == "D") return DownloadAll(p_device_d_grad_, p_device_d_grad_.size(), out, s);
  if (name == "b_d") return DownloadAll(p_device_b_d_grad_, p_device_b_d_grad_.size(), out, s);
  return false;
}

// ---------------------------------------------------------------------------------------------
double NeuralMachineTranslation::ComputeGradients(
    const int *p_host_source, int source_length, const int *p_host_target_in,
    const int *p_host_target_out, int target_length, const int *p_host_source_wgrad,
    int len_source_wgrad, const int *p_host_target_wgrad, int len_target_wgrad,
    const int *p_host_batch_information, int minibatch_size) {
  if (decode_mode_ || !cfg_.train_mode_)
    throw LinmtError("ComputeGradients: model was not initialised for training");
  if (minibatch_size != cfg_.minibatch_size_)
    throw LinmtError("ComputeGradients: the minibatch must have exactly minibatch_size_ columns "
                     "(gradients are taken over all timesteps of contiguous activations)");
  const int L = cfg_.num_layers_, B = minibatch_size, H = cfg_.lstm_size_;
  const int S = source_length, T = target_length;
  const bool seq2seq = cfg_.sequence_to_sequence_mode_;
  const bool attention = cfg_.attention_mode_ && seq2seq;
  const bool feed = attention && cfg_.feed_input_mode_;
  if (T < 1 || (seq2seq && S < 1)) throw LinmtError("ComputeGradients: empty minibatch");

  apply_dropout_ = cfg_.dropout_mode_;
  if (apply_dropout_) {
    ++minibatch_counter_;
    for (int l = 0; l < L; ++l) {
      const unsigned long long base = cfg_.dropout_seed_ * 0x100000001b3ULL + minibatch_counter_ * 4096;
      if (seq2seq) SourceLayer(l).GenerateDropoutMasks(S, base + 2 * l);
      TargetLayer(l).GenerateDropoutMasks(T, base + 2 * l + 1);
    }
  }
  struct DropoutOff {
    bool &flag;
    ~DropoutOff() { flag = false; }
  } dropout_off{apply_dropout_};
  ForwardTeacherForced(p_host_source, S, p_host_target_in, p_host_target_out, T,
                       p_host_batch_information, B, false);
  if (seq2seq) input_layer_source_.PreprocessWGrad(p_host_source, S, B, p_host_source_wgrad, len_source_wgrad);
  input_layer_target_.PreprocessWGrad(p_host_target_in, T, B, p_host_target_wgrad, len_target_wgrad);

  // softmax over all steps: log-likelihood, D^T dz for every step, D and b_d gradients
  LstmLayer &top_tgt = TargetLayer(L - 1);
  // what the attention nodes / the softmax read of the top decoder layer, all steps
  const float *top_up_all = UpwardState(top_tgt, 0);
  const float *h_for_softmax = attention ? attention_layer_.final_all_.get() : top_up_all;
  softmax_layer_.ForwardBackwardAllSteps(h_for_softmax, T);
  const float *dht_all = softmax_layer_.p_device_d_errt_ht_all_.get();

  // target side, last step first; layers top to bottom inside a step (feed input couples layer 1 of
  // step t+1 to the attention node of step t)
  if (attention) {
    HipErrorWrapper(hipMemsetAsync(attention_layer_.p_device_total_hs_error_.get(), 0,
                                   sizeof(float) * (size_t)H * B * S, stream_),
                    "ZeroAttentionError");
  }
  for (int t = T - 1; t >= 0; --t) {
    const float *dh_top = dht_all + (size_t)H * B * t;
    if (attention) {
      AttentionNode &an = attention_layer_.v_nodes_[t];
      an.BackProp(dh_top, (feed && t < T - 1) ? input_layer_target_.p_device_errn_to_t_h_tild_.get()
                                              : nullptr);
      dh_top = attention_layer_.p_device_errn_to_t_ht_p1_.get();
    }
    for (int l = L - 1; l >= 0; --l) {
      LstmLayer &Lt = TargetLayer(l);
      const lh_error_term above =
          l == L - 1 ? lh_error_term{dh_top, 1, 0, H} : TargetLayer(l + 1).v_nodes_[t].d_x_term_;
      const bool last = t == T - 1;
      Lt.v_nodes_[t].BackPropGpu(above, l < L - 1, last ? kNoError : Lt.d_h_prev_term_,
                                 last ? nullptr : Lt.p_device_d_errn_to_t_ct_m1_.get(), l == 0, true);
    }
  }
  for (int l = 0; l < L; ++l) {
    const float *h0 = seq2seq ? SourceLayer(l).v_nodes_[S - 1].p_device_h_t_ : nullptr;
    TargetLayer(l).ComputeGradientsAllSteps(T, h0, attention ? attention_layer_.final_all_.get() : nullptr);
  }
  if (attention) attention_layer_.ComputeGradientsAllSteps(T, top_up_all);

  // source side, one layer at a time (nothing couples a layer's step t to the layer above's t-1)
  if (seq2seq) {
    for (int l = L - 1; l >= 0; --l) {
      LstmLayer &Ls = SourceLayer(l);
      for (int t = S - 1; t >= 0; --t) {
        lh_error_term above = kNoError;
        if (l == L - 1) {
          if (attention) above.p = attention_layer_.p_device_total_hs_error_.get() + (size_t)H * B * t;
        } else {
          above.p = SourceLayer(l + 1).v_nodes_[t].p_device_d_x_;  // of BackPropInputAllSteps
        }
        above.ld = H;
        const bool last = t == S - 1;  // the decoder's step 0 hands its errors to this layer
        const lh_error_term dhn = last ? TargetLayer(l).d_h_prev_term_ : Ls.d_h_prev_term_;
        const float *dcn = last ? TargetLayer(l).p_device_d_errn_to_t_ct_m1_.get()
                                : Ls.p_device_d_errn_to_t_ct_m1_.get();
        Ls.v_nodes_[t].BackPropGpu(above, l < L - 1, dhn, dcn, true, true);
      }
      if (l > 0) Ls.BackPropInputAllSteps(S);
      Ls.ComputeGradientsAllSteps(S, nullptr, nullptr);
    }
  }
  double loss = 0;
  softmax_layer_.p_device_loss_.Download(&loss, 1, stream_);
  Synchronize();
  profiler_.Collect();
  return loss;
}

double NeuralMachineTranslation::ComputeGradientsStepwise(
    const int *p_host_source, int source_length, const int *p_host_target_in,
    const int *p_host_target_out, int target_length, const int *p_host_source_wgrad,
    int len_source_wgrad, const int *p_host_target_wgrad, int len_target_wgrad,
    const int *p_host_batch_information, int minibatch_size) {
  if (decode_mode_ || !cfg_.train_mode_)
    throw LinmtError("ComputeGradientsStepwise: model was not initialised for training");
  if (minibatch_size != cfg_.minibatch_size_)
    throw LinmtError("ComputeGradientsStepwise: the minibatch must have exactly minibatch_size_ columns");
  if (cfg_.dropout_mode_) throw LinmtError("ComputeGradientsStepwise: not with dropout");
  const int L = cfg_.num_layers_, B = minibatch_size, H = cfg_.lstm_size_;
  const int S = source_length, T = target_length;
  const bool seq2seq = cfg_.sequence_to_sequence_mode_;
  const bool attention = cfg_.attention_mode_ && seq2seq;
  const bool feed = attention && cfg_.feed_input_mode_;
  if (T < 1 || (seq2seq && S < 1)) throw LinmtError("ComputeGradientsStepwise: empty minibatch");
  ForwardTeacherForced(p_host_source, S, p_host_target_in, p_host_target_out, T,
                       p_host_batch_information, B, false);
  if (seq2seq) input_layer_source_.PreprocessWGrad(p_host_source, S, B, p_host_source_wgrad, len_source_wgrad);
  input_layer_target_.PreprocessWGrad(p_host_target_in, T, B, p_host_target_wgrad, len_target_wgrad);
  if (attention)
    HipErrorWrapper(hipMemsetAsync(attention_layer_.p_device_total_hs_error_.get(), 0,
                                   sizeof(float) * (size_t)H * B * S, stream_),
                    "ZeroAttentionError");
  LstmLayer &top_tgt = TargetLayer(L - 1);
  float *dht_all = softmax_layer_.p_device_d_errt_ht_all_.get();
  // target side (deep_rnn.h:1160-1200)
  for (int t = T - 1; t >= 0; --t) {
    float *h_in = attention ? attention_layer_.v_nodes_[t].p_device_final_tmp_2_
                            : top_tgt.v_nodes_[t].p_device_h_t_;
    p_softmax_layer_->BackPropPreprocessGpu(h_in, t * B);
    p_softmax_layer_->BackProp1(t);
    p_softmax_layer_->BackProp2(t);
    float *dh_top = dht_all + (size_t)H * B * t;
    if (attention) {
      attention_layer_.v_nodes_[t].BackProp(
          dh_top, (feed && t < T - 1) ? input_layer_target_.p_device_errn_to_t_h_tild_.get() : nullptr);
      dh_top = attention_layer_.p_device_errn_to_t_ht_p1_.get();
    }
    const bool last = t == T - 1;
    for (int l = L - 1; l >= 0; --l) {
      LstmLayer &Lt = TargetLayer(l);
      LstmNode &n = Lt.v_nodes_[t];
      n.p_device_d_errt_ht_ = l == L - 1 ? dh_top : TargetLayer(l + 1).v_nodes_[t].p_device_d_x_;
      n.BackPropPreprocessGpu(last ? nullptr : Lt.p_device_d_errn_to_t_ht_m1_.get(),
                              last ? nullptr : Lt.p_device_d_errn_to_t_ct_m1_.get());
      n.BackPropGpu(t);
    }
  }
  // source side (deep_rnn.h:1218-1246): the decoder's first step hands its errors to the encoder
  if (seq2seq) {
    for (int t = S - 1; t >= 0; --t) {
      const bool last = t == S - 1;
      for (int l = L - 1; l >= 0; --l) {
        LstmLayer &Ls = SourceLayer(l);
        LstmNode &n = Ls.v_nodes_[t];
        n.p_device_d_errt_ht_ =
            l == L - 1 ? (attention ? attention_layer_.p_device_total_hs_error_.get() + (size_t)H * B * t
                                    : nullptr)
                       : SourceLayer(l + 1).v_nodes_[t].p_device_d_x_;
        LstmLayer &from = last ? TargetLayer(l) : Ls;
        n.BackPropPreprocessGpu(from.p_device_d_errn_to_t_ht_m1_.get(),
                                from.p_device_d_errn_to_t_ct_m1_.get());
        n.BackPropGpu(t);
      }
    }
  }
  // the weight gradients of the LSTM and attention layers, which the reference accumulates node
  // by node (ComputeGradientsGpu), are taken over all steps at once
  const float *top_up_all = UpwardState(top_tgt, 0);
  for (int l = 0; l < L; ++l) {
    const float *h0 = seq2seq ? SourceLayer(l).v_nodes_[S - 1].p_device_h_t_ : nullptr;
    TargetLayer(l).ComputeGradientsAllSteps(T, h0, attention ? attention_layer_.final_all_.get() : nullptr);
    if (seq2seq) SourceLayer(l).ComputeGradientsAllSteps(S, nullptr, nullptr);
  }
  if (attention) attention_layer_.ComputeGradientsAllSteps(T, top_up_all);
  double loss = 0;
  softmax_layer_.p_device_loss_.Download(&loss, 1, stream_);
  Synchronize();
  profiler_.Collect();
  return loss;
}

void NeuralMachineTranslation::ClearGradients() {
  const int L = cfg_.num_layers_;
  for (int l = 0; l < L; ++l) {
    if (cfg_.sequence_to_sequence_mode_) SourceLayer(l).ClearGradients();
    TargetLayer(l).ClearGradients();
  }
  if (cfg_.attention_mode_ && cfg_.sequence_to_sequence_mode_) attention_layer_.ClearGradients();
  softmax_layer_.ClearGradients();
}

namespace {
struct UpdateItem {
  float *theta;
  long long ld_theta;
  float *grad;
  long long ld_grad, rows, cols;
  const int *col_index;
  bool in_global_norm;
  bool frozen;  // UpdateParams leaves the parameters alone; the gradient is only cleared
};
}  // namespace

void NeuralMachineTranslation::UpdateWeights() {
  if (!cfg_.train_mode_) throw LinmtError("UpdateWeights: model was not initialised for training");
  const int L = cfg_.num_layers_, H = cfg_.lstm_size_;
  const int mode = cfg_.grad_clip_mode_;
  std::vector<UpdateItem> items;
  // Stacked parameters are one tensor when the norm is global or absent; the per-matrix clip of
  // the reference norms W_hi, W_hf, ... separately, i.e. per gate block.
  auto add_stack = [&](DeviceArray<float> &theta, DeviceArray<float> &grad, int K, bool frozen) {
    if (mode == 1) {
      for (int g = 0; g < 4; ++g)
        items.push_back({theta.get() + (size_t)g * H, 4LL * H, grad.get() + (size_t)g * H, 4LL * H, H, K,
                         nullptr, true, frozen});
    } else {
      items.push_back({theta.get(), 4LL * H, grad.get(), 4LL * H, 4LL * H, K, nullptr, true, frozen});
    }
  };
  // the switches of InputToHiddenLayer / HiddenToHiddenLayer::UpdateParams
  // (src/layer_input_to_hidden.h:1154,1257,1263, src/layer_hidden_to_hidden.h:765,831)
  auto add_layer = [&](LstmLayer &Ly, bool source_side) {
    const bool rnn_frozen = source_side ? !cfg_.train_source_rnn_mode_ : !cfg_.train_target_rnn_mode_;
    const bool emb_frozen = source_side ? !cfg_.train_source_input_embedding_mode_
                                        : !cfg_.train_target_input_embedding_mode_;
    add_stack(Ly.p_device_w_h_stack_, Ly.p_device_w_h_grad_, H, rnn_frozen);
    add_stack(Ly.p_device_b_stack_, Ly.p_device_b_grad_, 1, rnn_frozen);
    add_stack(Ly.p_device_m_stack_, Ly.p_device_m_grad_, Ly.input_size_, rnn_frozen);
    if (Ly.feed_input_mode_) add_stack(Ly.p_device_q_stack_, Ly.p_device_q_grad_, H, rnn_frozen);
    if (Ly.input_layer_mode_ && Ly.w_grad_length_ > 0)
      items.push_back({Ly.p_device_w_.get(), Ly.input_size_, Ly.p_device_small_w_grad_.get(),
                       Ly.input_size_, Ly.input_size_, Ly.w_grad_length_,
                       Ly.p_device_input_vocab_indices_wgrad_.get(), false, emb_frozen});
  };
  auto add_flat = [&](DeviceArray<float> &theta, DeviceArray<float> &grad, bool frozen) {
    items.push_back({theta.get(), (long long)theta.size(), grad.get(), (long long)theta.size(),
                     (long long)theta.size(), 1, nullptr, true, frozen});
  };
  // SoftmaxLayer::UpdateWeightsGpu (src/layer_loss.h:1144)
  const bool out_frozen = !cfg_.train_target_output_embedding_mode_;
  add_flat(softmax_layer_.p_device_d_, softmax_layer_.p_device_d_grad_, out_frozen);
  add_flat(softmax_layer_.p_device_b_d_, softmax_layer_.p_device_b_d_grad_, out_frozen);
  for (int side = cfg_.sequence_to_sequence_mode_ ? 0 : 1; side < 2; ++side)
    for (int l = 0; l < L; ++l) add_layer(side == 0 ? SourceLayer(l) : TargetLayer(l), side == 0);
  if (cfg_.attention_mode_ && cfg_.sequence_to_sequence_mode_) {
    AttentionLayer &A = attention_layer_;
    const bool f = !cfg_.train_attention_target_rnn_mode_;
    add_flat(A.p_device_w_a_, A.p_device_w_a_grad_, f);
    add_flat(A.p_device_w_c_p1_, A.p_device_w_c_p1_grad_, f);
    add_flat(A.p_device_w_c_p2_, A.p_device_w_c_p2_grad_, f);
    add_flat(A.p_device_output_bias_, A.p_device_output_bias_grad_, f);
    if (!A.global_mode_) {
      add_flat(A.p_device_w_p_, A.p_device_w_p_grad_, f);
      add_flat(A.p_device_v_p_, A.p_device_v_p_grad_, f);
    }
  }
  if (items.size() > p_device_norms_.size()) p_device_norms_.Alloc(items.size() + 64);
  p_device_norms_.Zero(stream_);
  const float scale = 1.0f / (float)cfg_.minibatch_size_;  // ScaleGradients
  if (mode == 1 || mode == 2) {
    for (size_t i = 0; i < items.size(); ++i) {
      const UpdateItem &it = items[i];
      if (mode == 2 && !it.in_global_norm) continue;  // the embedding gradients are not in the norm
      ProfileScope ps(profiler_, kTagUpdate, 4.0 * it.rows * it.cols);
      LhErrorWrapper(lh_grad_sumsq_f32(it.grad, it.rows, it.cols, it.ld_grad, scale,
                                       p_device_norm_workspace_.get(),
                                       p_device_norms_.get() + (mode == 2 ? 0 : i), stream_),
                     "CalculateGlobalNorm");
    }
  }
  for (size_t i = 0; i < items.size(); ++i) {
    const UpdateItem &it = items[i];
    const double *nrm = mode == 2 ? p_device_norms_.get() : (mode == 1 ? p_device_norms_.get() + i : nullptr);
    if (it.frozen) {
      // the gradient is dropped, row block by row block (columns are ld_grad apart)
      HipErrorWrapper(hipMemset2DAsync(it.grad, sizeof(float) * it.ld_grad, 0, sizeof(float) * it.rows,
                                       (size_t)it.cols, stream_),
                      "UpdateParams: clearing a frozen group's gradient failed");
      continue;
    }
    ProfileScope ps(profiler_, kTagUpdate, 16.0 * it.rows * it.cols);
    LhErrorWrapper(lh_sgd_step_f32(it.theta, it.ld_theta, it.grad, it.ld_grad, it.rows, it.cols,
                                   it.col_index, cfg_.learning_rate_, scale, nrm, cfg_.norm_clip_,
                                   mode == 3 ? cfg_.individual_norm_clip_threshold_ : 0.f, stream_),
                   "UpdateParams");
  }
  double ss = 0;
  if (mode == 2) p_device_norms_.Download(&ss, 1, stream_);
  Synchronize();
  last_global_norm_ = std::sqrt(ss);
  profiler_.Collect();
}

bool NeuralMachineTranslation::GetGrad(const std::string &name, std::vector<float> *out) {
  if (!cfg_.train_mode_) return false;
  const size_t d1 = name.find('.');
  if (d1 == std::string::npos) return false;
  const std::string head = name.substr(0, d1);
  if (head == "attn") return cfg_.attention_mode_ && attention_layer_.GetGrad(name.substr(d1 + 1), out);
  if (head == "softmax") return softmax_layer_.GetGrad(name.substr(d1 + 1), out);
  const size_t d2 = name.find('.', d1 + 1);
  if (d2 == std::string::npos) return false;
  const int l = std::atoi(name.substr(d1 + 1, d2 - d1 - 1).c_str());
  if (l < 0 || l >= cfg_.num_layers_) return false;
  const std::string leaf = name.substr(d2 + 1);
  if (head == "src") return cfg_.sequence_to_sequence_mode_ && SourceLayer(l).GetGrad(leaf, out);
  if (head == "tgt") return TargetLayer(l).GetGrad(leaf, out);
  return false;
}

}  // namespace linmt
