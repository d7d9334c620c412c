// C++ layer classes of the LSTM / attention / softmax / beam path, keeping the reference's class and
// method names (src/layer_input_to_hidden.h, src/layer_hidden_to_hidden.h, src/layer_attention.h,
// src/layer_loss.h, src/deep_rnn.h, src/decoder.h) on top of the C ABI of liblinmt_hip.so.
//
// What changed against the reference, by design:
//   * one HIP stream per model instead of 28 streams + ~45 events per layer: every node's
//     ForwardProp() is a short, ordered list of launches (stacked gate GEMM -> fused cell);
//   * the four gate matrices of an operand are stored stacked (4H x K, rows i,f,c',o) so that the
//     8-12 SGEMMs of a cell are one multi-segment MFMA GEMM; M_i, W_hi, ... remain addressable as
//     strided views (ld = 4H) and by their reference names through SetParam/GetParam;
//   * "send h_t above" is pointer passing (the reference memcpy's because of `&& false`,
//     src/deep_rnn.h:544,586);
//   * decoding runs many sentences at once: the target-side minibatch is n_sent*beam columns,
//     sentence s owns columns [s*beam,(s+1)*beam); beam selection, back-pointers and the state swap
//     stay on the device, the host only reads the per-step (token, back-pointer, score) history.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "hip_util.h"
#include "profiler.h"

namespace linmt {

// Subset of GlobalConfiguration (src/global_configuration.h:93-310) that the path reads.
struct GlobalConfiguration {
  int num_layers_ = 1;
  int lstm_size_ = 100;
  int embedding_size_ = 0;  // 0: same as lstm_size_ (the reference's only case, global_configuration.h:220)
  int source_vocab_size_ = 0;
  int target_vocab_size_ = 0;
  int minibatch_size_ = 1;        // training / scoring columns
  int longest_sentence_ = 100;    // already including the reference's +4 (global_configuration.cc:290)
  int attention_mode_ = 0;        // 0 none, 1 local-p (reference), 2 global general (build-defined)
  int attention_width_ = 10;      // D
  bool feed_input_mode_ = false;
  bool sequence_to_sequence_mode_ = true;  // false: target-side language model (--nlm)
  bool clip_cell_mode_ = false;
  float cell_clip_threshold_ = 50.f;
  float error_clip_threshold_ = 1000.f;  // utility_cu.cu:91, active with clip_cell_mode_
  // training (global_configuration.h:107-123)
  bool train_mode_ = false;               // keep the activations and allocate gradients
  float learning_rate_ = 0.7f;
  // The reference's three mutually exclusive flags (global_configuration.cc:780-797):
  // 1 = clip_gradient_mode_ (per-matrix norm clip, the default), 2 = global_grad_clip_mode__
  // (--whole-clip-gradients), 3 = individual_grad_clip_mode__ (--ind-clip-gradients), 0 = none.
  int grad_clip_mode_ = 1;
  float norm_clip_ = 5.f;
  float individual_norm_clip_threshold_ = 0.1f;
  // dropout (global_configuration.h:129-130): dropout_rate_ is the probability of KEEPING a unit
  bool dropout_mode_ = false;
  float dropout_rate_ = 1.0f;
  unsigned long long dropout_seed_ = 1;
  // Which parameter groups UpdateParams moves (src/utility_cu.cu:17-22; --finetune switches the
  // three embedding groups off, src/global_configuration.cc:647-656).  A frozen group's gradients
  // are still computed, still count in the global norm, and are cleared as usual.
  bool train_source_input_embedding_mode_ = true;
  bool train_target_input_embedding_mode_ = true;
  bool train_target_output_embedding_mode_ = true;
  bool train_source_rnn_mode_ = true;
  bool train_target_rnn_mode_ = true;
  bool train_attention_target_rnn_mode_ = true;
};

class NeuralMachineTranslation;

// Measurement and test aids (lnmt_set_debug_option), process-wide, all off by default: each one
// switches a part of the decode path back to the form it replaced, so that a test can demand the
// same results of both forms and a benchmark can time them against each other.
struct DebugOptions {
  int no_stream = 0;               // Dispatcher::Decoding decodes batch by batch, never as a stream
  int no_projected_memory = 0;     // decoding attends over the encoder states themselves (the step's own products)
  int no_lanes = 0;                // the encoder of a decoding batch runs on the model's one stream
  int grouped_gates = 0;           // what the previous step fixes of every layer's gate product in one grouped launch
  int separate_beam_launches = 0;  // beam merge and state gather as the two launches the fused one replaces
};
DebugOptions &Debug();
class LstmLayer;
class AttentionLayer;

// A strided view of one gate block of a stacked parameter (reference: p_device_m_i_, p_device_w_hi_ ...).
struct MatrixView {
  float *ptr;
  int ld;
};

// ---------------------------------------------------------------------------------------------
// LstmInputHiddenNode (src/node_input_to_hidden.h:33-150) and LstmHiddenHiddenNode
// (src/node_hidden_to_hidden.h:34-131): one object per timestep (one in all when decoding).
class LstmNode {
 public:
  int index_ = 0;
  LstmLayer *p_layer_ = nullptr;
  int minibatch_size_ = 0;  // columns processed by ForwardProp (<= the layer's allocation)

  // inputs: aliases of buffers owned elsewhere, as in the reference
  int *p_device_input_vocab_indices_ = nullptr;     // layer 1 only: ids of this step, -1 -> 0
  int *p_device_input_vocab_indices_01_ = nullptr;  // 0/1 padding mask of this step
  float *p_device_h_t_prev_ = nullptr;
  float *p_device_c_t_prev_ = nullptr;
  float *p_device_h_tild_ = nullptr;     // attention output of step t-1 (feed input, layer 1 target)
  float *p_device_h_t_below_ = nullptr;  // layers >= 2

  // buffers owned by the layer, one slice per node
  float *p_device_sparse_lookup_ = nullptr;  // layer 1: E x B embedding columns
  float *p_device_pre_x_ = nullptr;  // 4H x B: M*x of this step when the layer computed it for all steps
  // decoding: W_h*h_{t-1} of this step already sits in the layer's preact_ (the step's grouped
  // launch put it there); ForwardProp only adds M*x of the layer below
  bool recurrent_hoisted_ = false;
  float *p_device_gates_ = nullptr;          // 4H x B: i_t, f_t, c_prime_t_tanh, o_t (NULL when not kept)
  float *p_device_c_t_ = nullptr;
  float *p_device_h_t_ = nullptr;
  float *p_device_dropout_mask_ = nullptr;      // layer 1: mask of the looked-up embeddings
  float *p_device_out_dropout_mask_ = nullptr;  // mask under which the consumer above reads h_t
  float *p_device_h_t_dropped_ = nullptr;       // that dropped copy (the recurrence keeps h_t)
  float *p_device_d_gates_ = nullptr;  // training: 4H x B gate errors of this step
  float *p_device_d_x_ = nullptr;      // training: error w.r.t. this step's input (M^T d)

  // BackPropGpu (node_input_to_hidden.h:647-983, node_hidden_to_hidden.h:537-900): fused cell
  // backward and W_h^T d; upper layers and the feed-input branch also produce M^T d / Q^T d here.
  // dh_above: error from the layer above (above_is_lstm) or from the attention node / softmax
  // (NULL = none); dh_next / dc_next: errors from step t+1 (NULL = none).  The errors for step t-1
  // land in the layer's p_device_d_errn_to_t_ht_m1_ / _ct_m1_.  batched_dx: M^T d is left to one
  // GEMM over all steps (BackPropInputAllSteps).
  // leave_planes: a W^T d product whose K range is split over workgroups stays in partial planes
  // (the layer's error_planes_ buffers), described by the layer's d_h_prev_term_ and this node's
  // d_x_term_, which the cell kernels of step t-1 / of the layer below add up as they read them;
  // otherwise the products are reduced into p_device_d_errn_to_t_ht_m1_ / p_device_d_x_ and the
  // terms name those.
  void BackPropGpu(const lh_error_term &dh_above, bool above_is_lstm, const lh_error_term &dh_next,
                   const float *dc_next, bool batched_dx, bool leave_planes);
  lh_error_term d_x_term_{nullptr, 1, 0, 0};
  // The reference's own two-call form (node_input_to_hidden.h:139-140, node_hidden_to_hidden.h:
  // 133-134), same signatures: BackPropPreprocessGpu hands in the errors of step t+1,
  // BackPropGpu(index) runs the node's backward step on them and on p_device_d_errt_ht_, the
  // error from above, which the upper layer / attention node / softmax left there (a pointer the
  // caller wires, as deep_rnn.h:470-520 does; NULL = none).  The error to the layer below is
  // written to p_device_d_x_ (the reference's p_device_d_errn_to_t_h_below_); weight gradients
  // are taken over all steps afterwards (LstmLayer::ComputeGradientsAllSteps), where the
  // reference's node calls ComputeGradientsGpu per step.
  float *p_device_d_errn_to_tp1_ht_ = nullptr;
  float *p_device_d_errn_to_tp1_ct_ = nullptr;
  float *p_device_d_errt_ht_ = nullptr;
  void BackPropPreprocessGpu(float *p_device_d_errn_to_tp1_ht, float *p_device_d_errn_to_tp1_ct);
  void BackPropGpu(int index);

  // InputToHidden: UpdateVectorsForwardGpu(idx0, mask01, h_prev, c_prev) (node_input_to_hidden.h:100);
  // HiddenToHidden: UpdateVectorsForwardGpu(mask01, h_prev, c_prev) (node_hidden_to_hidden.h:94).
  void UpdateVectorsForwardGpu(int *p_device_input_vocab_indices, int *p_device_input_vocab_indices_01,
                               float *p_device_h_t_prev, float *p_device_c_t_prev);
  void UpdateVectorsForwardGpu(int *p_device_input_vocab_indices_01, float *p_device_h_t_prev,
                               float *p_device_c_t_prev);
  // ForwardPropGpu of both node kinds (node_input_to_hidden.h:218-636, node_hidden_to_hidden.h:194-444).
  void ForwardProp();
  // The node's step as one problem of a grouped launch (lh_gate_gemm_group_f32): complete = the
  // whole pre-activation with the cell (first target layer while decoding: nothing in it depends
  // on this step), otherwise only W_h*h_{t-1} into the layer's preact_.
  void DescribeRecurrentProblem(bool complete, lh_gate_problem *q);
};

// InputToHiddenLayer (src/layer_input_to_hidden.h:37-378) / HiddenToHiddenLayer
// (src/layer_hidden_to_hidden.h:33-317) share everything but the source of x.
class LstmLayer {
 public:
  NeuralMachineTranslation *p_neural_mt_ = nullptr;
  bool input_layer_mode_ = true;  // true: InputToHiddenLayer (owns the embedding W)
  bool source_side_mode_ = true;
  int layer_number_ = 0;
  int lstm_size_ = 0;
  int input_size_ = 0;  // E for layer 1, H above
  int vocab_size_ = 0;
  int minibatch_size_ = 0;
  int num_nodes_ = 0;
  bool feed_input_mode_ = false;
  bool keep_gates_ = false;

  // parameters (stacked: rows [g*H,(g+1)*H) belong to gate g in the order i, f, c', o)
  DeviceArray<float> p_device_w_;        // E x V embedding (layer 1)
  DeviceArray<float> p_device_m_stack_;  // 4H x input_size : M_i, M_f, M_c, M_o
  DeviceArray<float> p_device_w_h_stack_;  // 4H x H : W_hi, W_hf, W_hc, W_ho
  DeviceArray<float> p_device_q_stack_;    // 4H x H : Q_i, Q_f, Q_c, Q_o (feed input)
  DeviceArray<float> p_device_b_stack_;    // 4H     : b_i, b_f, b_c, b_o
  MatrixView p_device_m(int gate) { return {p_device_m_stack_.get() + (size_t)gate * lstm_size_, 4 * lstm_size_}; }
  MatrixView p_device_w_h(int gate) { return {p_device_w_h_stack_.get() + (size_t)gate * lstm_size_, 4 * lstm_size_}; }
  MatrixView p_device_q(int gate) { return {p_device_q_stack_.get() + (size_t)gate * lstm_size_, 4 * lstm_size_}; }

  // activations
  DeviceArray<float> p_device_init_hidden_vec_, p_device_init_cell_vec_;  // zeros
  DeviceArray<float> h_all_, c_all_, gates_all_, lookup_all_, preact_;
  // Input products hoisted off the recurrence.  Whenever every step's input is known before the
  // recurrence starts (the whole source side, run layer by layer; the teacher-forced target input
  // layer), M*[x_0 .. x_{T-1}] is ONE GEMM over B*T columns into pre_x_all_ and a step only adds
  // W_h*h_{t-1} (+ Q*h~_{t-1}).  When decoding, the target input layer reads M*W[:,token] from the
  // precomputed 4H x V product mw_fold_ instead (a 4H-row "embedding" lookup).
  DeviceArray<float> pre_x_all_, mw_fold_;
  bool input_hoistable_ = false;  // buffers exist
  bool input_hoisted_ = false;    // this pass uses them
  bool mw_fold_dirty_ = true;
  // Decoding with split products (NeuralMachineTranslation::split_products_): the stacked gate
  // matrices of a target step side by side, [M | W_h] (first layer: [W_h | Q]), as packed bf16
  // planes, and the step's packed input [h_below; h_{t-1}] ([h_{t-1}; h~_{t-1}]).
  DeviceArray<unsigned> split_w_planes_, split_x_planes_;
  int split_kgroups_ = 0;  // k-groups of both operands, padding included
  bool split_dirty_ = true;
  void BuildSplitWeights();
  void ForwardPropInputAllSteps(int steps);
  void ForwardPropInputSteps(int first, int steps);
  void BuildEmbeddingFold();
  DeviceArray<float> p_device_h_t_previous_, p_device_c_t_previous_;  // decode: PreviousTargetState
  DeviceArray<int> p_device_input_vocab_indices_full_, p_device_input_vocab_indices_01_full_;
  std::vector<LstmNode> v_nodes_;

  void Init(NeuralMachineTranslation *model, bool input_layer, bool source_side, int layer_number,
            int minibatch_size, int num_nodes, bool keep_gates, bool with_previous_state);
  // InitFeedInput (layer_input_to_hidden.h:299): allocates Q and switches the nodes to feed input.
  void InitFeedInput();

  // ---- training --------------------------------------------------------------------------------
  DeviceArray<float> p_device_m_grad_, p_device_w_h_grad_, p_device_q_grad_, p_device_b_grad_;
  DeviceArray<float> p_device_small_w_grad_;  // E x (number of unique ids), layer 1
  DeviceArray<float> d_gates_all_, d_x_all_;  // per-step gate errors / input errors
  DeviceArray<float> p_device_d_errn_to_t_ht_m1_, p_device_d_errn_to_t_ct_m1_;  // recurrent errors
  // partial planes of W_h^T d and M^T d of the step in flight (kErrorPlanes each)
  static constexpr int kErrorPlanes = 4;
  DeviceArray<float> d_h_prev_planes_, d_x_planes_;
  lh_error_term d_h_prev_term_{nullptr, 1, 0, 0};  // the error for step t-1, as the last BackPropGpu left it
  DeviceArray<float> p_device_errn_to_t_h_tild_;  // Q^T d: error into the attention node of t-1
  DeviceArray<int> p_device_input_vocab_indices_wgrad_, p_device_wgrad_seg_start_,
      p_device_wgrad_seg_cols_;
  int w_grad_length_ = 0;  // unique ids of the current minibatch
  // dropout: uniform masks for every step, regenerated per minibatch (the reference draws them
  // with cuRAND inside each node's forward, node_input_to_hidden.h:264-272, node_hidden_to_hidden.h:208-226)
  DeviceArray<float> dropout_mask_all_, out_dropout_mask_all_, h_dropped_all_;
  bool out_dropout_ = false;  // the consumer above reads a dropped copy of this layer's h
  void GenerateDropoutMasks(int steps, unsigned long long seed);
  void InitTraining();
  // Unique-id list of the minibatch (the reference's *_wgrad arrays, file_helper.cc:281-380) plus,
  // per unique id, the (timestep, column) positions that carry it.
  void PreprocessWGrad(const int *p_host_indices, int current_length, int minibatch_size,
                       const int *p_host_wgrad, int len_wgrad);
  // ComputeGradientsGpu over all steps at once (node_input_to_hidden.h:997-1300): weight / bias
  // gradients as GEMMs with K = minibatch x steps, and the embedding gradient.
  // h_prev0 / c-less: state fed to step 0 (NULL = zeros).
  void ComputeGradientsAllSteps(int steps, const float *p_device_h_prev0,
                                const float *p_device_h_tild_all);
  // d_x_all_ = M^T d for every step in one GEMM.
  void BackPropInputAllSteps(int steps);
  void ClearGradients();
  bool GetGrad(const std::string &name, std::vector<float> *out);

  // PreprocessGpuVocabIndices (layer_input_to_hidden.h:1478-1513, layer_hidden_to_hidden.h:541-560):
  // host ids (B x T column-major, -1 padding) -> device idx0 / mask01 for all T steps.
  void PreprocessGpuVocabIndices(const int *p_host_input_vocab_indices, int current_length,
                                 int minibatch_size);
  // Reference parameter names: "W", "M_i".."M_c", "W_hi".."W_ho", "b_i".."b_o", "Q_i".."Q_c".
  bool SetParam(const std::string &name, const float *host, size_t n);
  bool GetParam(const std::string &name, std::vector<float> *out);
};

// ---------------------------------------------------------------------------------------------
// AttentionNode / AttentionLayer (src/layer_attention.h:28-131, 704-845).
class AttentionNode {
 public:
  int index_ = 0;
  AttentionLayer *p_attention_layer_ = nullptr;
  int minibatch_size_ = 0;
  float *p_device_h_t_ = nullptr;           // input: top decoder layer state
  int *p_device_indices_mask_ = nullptr;    // 0/1 mask of the target step
  float *p_device_tanh_1_ = nullptr, *p_device_sigma_1_ = nullptr, *p_device_p_t_ = nullptr;
  float *p_device_h_t_wa_cache_ = nullptr, *p_device_alignments_ = nullptr;
  float *p_device_cached_exp_ = nullptr, *p_device_c_t_ = nullptr, *p_device_final_tmp_2_ = nullptr;
  int *p_device_indices_ = nullptr;
  float *p_device_d_errt_ht_tild_ = nullptr;  // training: delta of this step (H x B)
  float *p_device_h_s_sum_ = nullptr, *p_device_u_ = nullptr, *p_device_w_ = nullptr;
  void ForwardProp();  // layer_attention.h:243-483
  // layer_attention.h:487-698.  dht: error from the softmax; dht_feed: Q^T d of step t+1 (or NULL).
  // Leaves the error for the top decoder layer in the layer's p_device_errn_to_t_ht_p1_.
  void BackProp(const float *dht, const float *dht_feed);
};

class AttentionLayer {
 public:
  NeuralMachineTranslation *p_neural_mt_ = nullptr;
  int lstm_size_ = 0, minibatch_size_ = 0, d_ = 0, num_nodes_ = 0, window_ = 0;
  bool global_mode_ = false;  // build-defined global "general" attention
  DeviceArray<float> p_device_w_a_, p_device_w_p_, p_device_v_p_, p_device_output_bias_,
      p_device_w_c_p1_, p_device_w_c_p2_;
  DeviceArray<float> tanh_1_all_, sigma_1_all_, p_t_all_, wa_all_, alignments_all_, cached_exp_all_,
      c_t_all_, final_all_;
  DeviceArray<int> indices_all_, p_device_batch_information_, p_device_hs_col_;
  // encoder top-layer states (owned by the top source layer): state(tau, col) = base + tau*step + col*colstride
  const float *p_device_total_hs_ = nullptr;
  long long hs_step_stride_ = 0, hs_col_stride_ = 0;
  int hs_steps_ = 0;       // timesteps currently held
  bool use_hs_col_ = false;  // decode: beam columns share their sentence's states
  std::vector<AttentionNode> v_nodes_;
  // Outside training the two projections of h_t share one launch: [W_p ; W_a^T] (2H x H) * h_t
  // with tanh on the upper half (src/layer_attention.h:272-275 and :327).  The stack is rebuilt
  // when W_p or W_a is set; training updates them on the device and keeps the two products apart.
  DeviceArray<float> p_device_w_pa_stack_, proj_out_;
  bool pa_stack_dirty_ = true;
  void BuildProjectionStack();
  // Decoding: a sentence's encoder states serve every step of its beam, so the two products that
  // involve them are taken out of the step.  Once per batch score_mem_ = W_a * hs and
  // ctx_mem_ = W_c1 * hs over all source positions (laid out like the states); per step one
  // product [W_p ; W_c2] (2H x H) * h_t and one kernel that scores against score_mem_, sums
  // ctx_mem_ with the alignment weights and finishes h~ = tanh(. + W_c2 h_t + b).  The context
  // vector itself is never formed.  Local-p attention with a window the kernel holds in registers.
  DeviceArray<float> score_mem_, ctx_mem_, p_device_w_pc_stack_, pc_out_;
  bool pc_stack_dirty_ = true;
  bool projected_memory_ = false;  // the two memories hold this batch's states
  bool ProjectedMemoryPossible() const;
  // capacity = floats of the encoder's state slab (the memories are allocated once, that large)
  void BuildProjectedMemory(int source_length, size_t capacity);
  void BuildOutputStack();

  // ---- training --------------------------------------------------------------------------------
  DeviceArray<float> p_device_w_a_grad_, p_device_w_p_grad_, p_device_v_p_grad_,
      p_device_output_bias_grad_, p_device_w_c_p1_grad_, p_device_w_c_p2_grad_;
  DeviceArray<float> delta_all_, h_s_sum_all_, u_all_, w_all_;
  DeviceArray<float> p_device_errn_to_t_ct_, p_device_errn_to_t_ht_p1_;
  DeviceArray<float> p_device_total_hs_error_;  // layout of the encoder's top-layer states
  void InitTraining();
  void ComputeGradientsAllSteps(int steps, const float *p_device_h_t_all);
  void ClearGradients();
  bool GetGrad(const std::string &name, std::vector<float> *out);

  void Init(NeuralMachineTranslation *model, int minibatch_size, int num_nodes, int longest_sent);
  // PreprocessMinibatchInformation (layer_attention.h:977): [len_0.., offset_0..] for B columns.
  void PreprocessMinibatchInformation(const int *p_host_batch_information, int minibatch_size);
  bool SetParam(const std::string &name, const float *host, size_t n);
  bool GetParam(const std::string &name, std::vector<float> *out);
};

// ---------------------------------------------------------------------------------------------
// BaseLossLayer (src/layer_loss.h:42-103) and SoftmaxLayer (:150-360).
class BaseLossLayer {
 public:
  virtual ~BaseLossLayer() {}
  virtual void ForwardProp(int index) = 0;
  virtual double ComputeLossGpu(int index) = 0;
  virtual void BackPropPreprocessGpu(float *p_device_h_t, int step) = 0;
  virtual void BackProp1(int index) = 0;  // layer_loss.h:60: error to h_t of step index
  virtual void BackProp2(int index) = 0;  // layer_loss.h:61: D and b_d gradients of step index
  virtual void GetDistributionGpuDecoderWrapper() = 0;
  virtual float *GetDistPtr() = 0;
  virtual void SetHTPtr(int index, float *p_device_h_t) = 0;
  virtual float *GetHTPtr(int index) = 0;
  virtual double GetTrainPerplexity() = 0;
  virtual void PreprocessGpuVocabIndices(const int *p_host_output_vocab_indices_target,
                                         int current_target_length, int minibatch_size) = 0;
};

class SoftmaxLayer : public BaseLossLayer {
 public:
  NeuralMachineTranslation *p_neural_mt_ = nullptr;
  int lstm_size_ = 0, output_vocab_size_ = 0, minibatch_size_ = 0, num_nodes_ = 0;
  int current_minibatch_ = 0;
  bool training_perplexity_mode_ = false;
  DeviceArray<float> p_device_d_, p_device_b_d_;
  // split products: D and the step's h~ as packed bf16 planes
  DeviceArray<unsigned> split_d_planes_, split_h_planes_;
  int split_kgroups_ = 0;
  bool split_dirty_ = true;
  void BuildSplitWeights();
  void ComputeLogitsSplit(float *p_device_h_t, int minibatch);
  DeviceArray<float> p_device_outputdist_;           // V x B logits / probabilities (one step)
  DeviceArray<double> p_device_logp_tgt_, p_device_loss_, p_device_train_perplexity_;
  DeviceArray<int> p_device_output_vocab_indices_, p_device_output_vocab_indices_01_;
  DeviceArray<float> p_device_output_vocab_indices_01_float_;
  std::vector<float *> v_h_t_;  // per node: input of the softmax (SetHTPtr)
  int *p_device_output_vocab_indices_single_ = nullptr, *p_device_output_vocab_indices_01_single_ = nullptr;

  void Init(NeuralMachineTranslation *model, int minibatch_size, int num_nodes);
  void ForwardProp(int index) override;                     // layer_loss.h:480-516
  void GetDistributionGpu(float *p_device_h_t);             // layer_loss.h:797-883
  double ComputeLossGpu(int index) override;                // layer_loss.h:673-704 (+ GetPerplexityGpu :708)
  void BackPropPreprocessGpu(float *p_device_h_t, int step) override;  // layer_loss.h:630-650
  // One step at a time, as the reference drives the loss layer (deep_rnn.h:1166-1273):
  // BackProp1 = GetHTGradientGpu (layer_loss.h:547-626): forward of step `index` on the h_t and
  // the targets BackPropPreprocessGpu selected, log-likelihood into p_device_loss_, and the error
  // D^T dz into step index's slice of p_device_d_errt_ht_all_; BackProp2 = ComputeDGradientGpu +
  // ComputeBDGradientGpu (layer_loss.h:887-972) from the same dz, so it follows BackProp1 of the
  // same index.  ForwardBackwardAllSteps is the batched form of the two.
  void BackProp1(int index) override;
  void BackProp2(int index) override;
  float *p_device_h_t_step_ = nullptr;  // BackPropPreprocessGpu's h_t
  int dz_index_ = -1;                   // step whose output error p_device_outputdist_ holds
  void GetDistributionGpuDecoderWrapper() override;
  float *GetDistPtr() override { return p_device_outputdist_.get(); }
  void SetHTPtr(int index, float *p) override { v_h_t_[index] = p; }
  float *GetHTPtr(int index) override { return v_h_t_[index]; }
  double GetTrainPerplexity() override;
  void PreprocessGpuVocabIndices(const int *p_host_output_vocab_indices_target,
                                 int current_target_length, int minibatch_size) override;
  // logits only (D*h + b_d), used by the on-device beam step
  void ComputeLogits(float *p_device_h_t, int minibatch);

  // ---- training --------------------------------------------------------------------------------
  DeviceArray<float> p_device_d_grad_, p_device_b_d_grad_;
  DeviceArray<float> p_device_d_errt_ht_all_;  // D^T dz for every step (H x B x steps)
  DeviceArray<float> dz_chunk_;                // V x (B x chunk steps) logits, then output errors
  int chunk_steps_ = 0;
  void InitTraining();
  // ForwardProp + BackProp1 + BackProp2 of every step (layer_loss.h:480-516, 547-626, 887-972) as
  // chunked GEMMs over B x steps columns; accumulates the log-likelihood into p_device_loss_.
  void ForwardBackwardAllSteps(const float *p_device_h_t_all, int steps);
  void ClearGradients();
  bool GetGrad(const std::string &name, std::vector<float> *out);
  bool SetParam(const std::string &name, const float *host, size_t n);
  bool GetParam(const std::string &name, std::vector<float> *out);
};

// ---------------------------------------------------------------------------------------------
// Decoder (src/decoder.h:148-245): hypothesis bookkeeping.  The selection itself
// (ExpandHypothesis / FinishCurrentHypotheses) runs on the device; this class owns the device-side
// beam buffers and rebuilds the hypotheses from the recorded history.
struct Hypothesis {
  std::vector<int> tokens;  // <START> ... <EOF>
  float score = 0.f;        // log-probability (+ penalties), before length / coverage rescoring
  // unk_replacement_mode_ only (decoder.h:129-130): per token the source position with the largest
  // alignment score (-20 at <START>) and the alignment scores over the source positions
  std::vector<int> viterbi;
  std::vector<std::vector<float>> alignments_scores;
};

struct DecodeOptions {
  int beam_size_ = 12;
  float max_decoding_ratio_ = 1.5f, min_decoding_ratio_ = 0.5f;
  float penalty_ = 0.f, diversity_ = 0.f, lp_alpha_ = 0.65f, cp_beta_ = 0.20f;
  // the reference's unk_replacement_mode__ (layer_attention.h:342-386): export the alignment
  // scores of every step; hypotheses carry Viterbi alignments and the coverage penalty is computed
  // from the exported scores instead of zeros
  bool unk_replacement_mode_ = false;
  // the reference's hypotheses_number_ (global_configuration.h:229): how many of the finished
  // hypotheses OutputKBestHypotheses keeps, best first
  int hypotheses_number_ = 1;
  // DecodeStream: write out the tokens of every finished hypothesis (SentenceResult::hypotheses),
  // not only of the ones OutputKBestHypotheses keeps.  A caller that reads only the kept ones
  // switches it off: a list of a thousand sentences has a few hundred thousand finished hypotheses.
  bool all_hypotheses_tokens_ = true;
};

struct SentenceResult {
  std::vector<int> best;  // 1-best without <START>/<EOF>
  std::vector<int> best_viterbi;  // unk_replacement_mode_: source position aligned to each token
  int best_index = -1;            // index of the 1-best in hypotheses
  float best_score = 0.f;
  // the hypotheses_number_ best (fewer when fewer pass the length filter): indices into
  // hypotheses, best first, with their final scores; kbest[0] == best_index
  std::vector<int> kbest;
  std::vector<float> kbest_score;
  std::vector<Hypothesis> hypotheses;  // in the order the reference's v_hypotheses_ would hold them
  int steps = 0;                       // decoder forward passes this sentence took part in
};

// First line of a model file: written by AddModelInformation (src/utility_cc.cc:76-98), parsed by
// DecoderModelWrapper::ExtractModelInformation (src/decoder.h:1182-1210).
struct ModelInformation {
  int num_layers = 0, lstm_size = 0, target_vocab_size = 0, source_vocab_size = 0;
  int attention_model = 0, feed_input = 0, multi_source = 0, combine_lstm = 0, char_cnn = 0;
};
ModelInformation ReadModelInformation(const std::string &model_file);

class Decoder {
 public:
  static constexpr int start_symbol_ = 0, end_symbol_ = 1;
  int beam_size_ = 0, n_sent_ = 0, max_steps_ = 0;
  DeviceArray<float> cand_logp_, logp_eof_, score_[2], fin_score_hist_, score_hist_;
  DeviceArray<int> cand_id_, limit_, tok_hist_, backptr_hist_, fin_count_hist_, fin_beam_hist_,
      current_indices_;
  // unk_replacement_mode_: the attention core's alignments / window indices of every step
  // ([step][column + columns_of_that_step * slot]), allocated on first use
  DeviceArray<float> align_hist_;
  DeviceArray<int> index_hist_;
  void Init(int beam_size, int n_sent, int max_steps);
  // OutputKBestHypotheses (decoder.h:529-699) for one sentence: the selection, not the printing.
  // sizes (optional): token counts of hypotheses whose tokens have not been written out yet;
  // materialise(i) is then called for every hypothesis that is kept, before its tokens are read.
  static void OutputKBestHypotheses(std::vector<Hypothesis> &hyps, int source_length,
                                    const DecodeOptions &o, SentenceResult *out,
                                    const std::vector<int> *sizes = nullptr,
                                    const std::function<void(int)> &materialise = nullptr);
};

// ---------------------------------------------------------------------------------------------
// NeuralMachineTranslation (src/deep_rnn.h): wiring and the forward drivers.
class NeuralMachineTranslation {
 public:
  GlobalConfiguration cfg_;
  hipStream_t stream_ = nullptr;
  bool decode_mode_ = false;
  int beam_size_ = 0, n_sent_ = 0;
  // Opt-in (lnmt_set_split_products): a
  // decoding step's gate products and output projection run as products of three-way bf16 splits
  // (lh_gemm_split_f32 / lh_gate_gemm_split_lstm_cell_f32) while at least split_min_columns_
  // hypotheses are alive; below that, and everywhere else, the fp32 MFMA products run.
  bool split_products_ = false;
  int split_min_columns_ = 84;
  bool split_step_ = false;  // the step being run uses them
  bool SplitProductsUsable(int curr_index, int minibatch) const;
  // The same switch on a model created for training: Gemm() forms its large batched products
  // (weight gradients over all steps, the output projection and its backward products, the
  // layer-major input products) this way, packing both operands on the fly into these buffers;
  // worthwhile while the packing is a small part of the product (both extents in the thousands).
  DeviceArray<unsigned> split_scratch_a_, split_scratch_x_;
  bool GemmAsSplitProduct(int tag, int rows, int cols, const lh_gemm_seg *segs, int nseg, int trans_a,
                          int trans_x, float beta, const float *bias, int act, const int *colmask,
                          float *C, int ldc, const char *what, int act_rows);
  Profiler profiler_;  // live HIP-event timing on stream_, off by default
  // Scratch of lh_gemm_ws_f32 (split-K partial sums); every product of the model runs on
  // stream_, which is the ordering that sharing it requires.
  static constexpr size_t kGemmWorkspaceBytes = size_t(64) << 20;
  DeviceArray<char> gemm_workspace_;
  // the part of it the products launched right now may use (all of it on the single stream; one
  // slice per layer while the encoder's layers run side by side)
  char *gemm_ws_ptr_ = nullptr;
  size_t gemm_ws_bytes_ = 0;
  // Encoder of a decoding batch: layer l+1 can start on a block of timesteps as soon as layer l
  // has finished it, so every layer gets a stream of its own (layer 0: stream_) and the L
  // recurrences overlap instead of queueing 2*L*S small launches behind each other.
  std::vector<hipStream_t> lane_streams_;
  std::vector<hipEvent_t> lane_events_;
  static constexpr int kLaneChunkSteps = 8;
  // Every dense product of the model: profiling key, workspace, error text.
  void Gemm(int tag, int rows, int cols, const lh_gemm_seg *segs, int nseg, int trans_a, int trans_x,
            float beta, const float *bias, int act, const int *colmask, float *C, int ldc,
            const char *what, int act_rows = -1);  // act_rows < 0: the activation covers every row
  // The plain product for a consumer that adds partial sums itself (the LSTM cell kernel takes
  // three addends).  Returns the number of addends n and fills addend[0..n): either {C} with
  // C = beta * C + product, or the partial planes of a split product preceded by C when beta = 1.
  int GemmAddends(int tag, int rows, int cols, const lh_gemm_seg *segs, int nseg, float beta,
                  float *C, int ldc, const float *addend[3], const char *what);

  LstmLayer input_layer_source_, input_layer_target_;
  std::vector<std::unique_ptr<LstmLayer>> v_hidden_layers_source_, v_hidden_layers_target_;
  AttentionLayer attention_layer_;
  SoftmaxLayer softmax_layer_;
  BaseLossLayer *p_softmax_layer_ = &softmax_layer_;
  Decoder decoder_;
  // Host copy of the beam histories of the last DecodeBatch (what the reference keeps in
  // eigen_top_sentences_ / new_indices_changes_, src/decoder.h:128-199, step by step): token and
  // GLOBAL back-pointer column of beam entry (step, column), columns in the batch's internal
  // order (sentences longest first); slot_of_sentence maps a caller's sentence to its column block.
  struct DecodeHistory {
    int n = 0, beam = 0, steps = 0;
    std::vector<int> slot_of_sentence, limit, tok, backptr;
    std::vector<float> score;  // path score of beam entry (step, column)
    // DecodeBatch: entry (step, sentence k, j) at step * n * beam + slot_of_sentence[k] * beam + j,
    // back-pointers as batch columns.  DecodeStream (offset not empty): sentence i's rows are
    // contiguous, entry (step, j) at offset[i] + step * beam + j, back-pointers beam-local.
    std::vector<size_t> offset;
  } last_history_;
  // What DecodeStream keeps between calls (device buffers and page-locked host buffers that only
  // grow): a call allocates nothing once a longer list has been decoded.
  struct StreamState {
    DeviceArray<int> tok_hist, bp_hist, fcount_hist, fbeam_hist, start_dev, limit_dev, mask_table;
    DeviceArray<float> score_hist, fscore_hist, finals, align_hist;
    DeviceArray<int> index_hist;
    PinnedArray<int> tok, bp, fcount, fbeam, mask_host;
    PinnedArray<float> fscore, bscore;
  } stream_state_;
  DeviceArray<float> p_device_h_tild_previous_;  // decode: gathered h~ of the previous step
  DeviceArray<float> p_device_ensemble_dist_;    // decode in an ensemble: this model's probabilities
  std::vector<hipEvent_t> ensemble_events_;      // owned by the model that runs the beam search
  DeviceArray<int> p_device_ones_, p_device_sentence_of_column_;

  explicit NeuralMachineTranslation(const GlobalConfiguration &cfg);
  ~NeuralMachineTranslation();
  // InitModel (deep_rnn.h:249-692): one node per timestep, B = cfg.minibatch_size_.
  void InitModel();
  // InitModelDecoding (deep_rnn.h:697-922), batched: n_sent sentences x beam hypotheses.
  void InitModelDecoding(int n_sent, int beam_size);

  LstmLayer &SourceLayer(int l) { return l == 0 ? input_layer_source_ : *v_hidden_layers_source_[l - 1]; }
  LstmLayer &TargetLayer(int l) { return l == 0 ? input_layer_target_ : *v_hidden_layers_target_[l - 1]; }

  // GetError (deep_rnn.h:2173-2317): teacher-forced forward + sum of log p(target).
  double GetError(const int *p_host_source, int source_length, const int *p_host_target_in,
                  const int *p_host_target_out, int target_length, const int *p_host_batch_information,
                  int minibatch_size);
  // ForwardPropSource (deep_rnn.h:1572-1721) for n_sent sentences (B x S ids, reversed, left-padded).
  void ForwardPropSource(const int *p_host_source, int source_length, int n_sent);
  // ForwardPropTarget (deep_rnn.h:1754-1836) on the first `minibatch` beam columns.
  void ForwardPropTarget(int curr_index, int *p_device_current_indices, int minibatch);
  // SwapDecodingStates + TargetCopyPrevStates (deep_rnn.h:1842-1872) in one gather launch.
  void SwapDecodingStates(const int *p_device_backptr, int minibatch);
  // the (source, destination) pairs SwapDecodingStates moves: h and c of every target layer and,
  // with input feeding, h~; returns their number
  int DecodingStateTensors(const float **src, float **dst);
  // EnsembleFactory::DecodeFile (decoder.h:1702-1776) for a batch of sentences (ids in ORIGINAL
  // order, ragged).  Results come back in input order.
  // `ensemble`: further models decoded in lockstep with this one (EnsembleFactory,
  // decoder.h:1778-1931): their distributions are averaged with this model's before every beam
  // step.  They must be initialised for decoding with the same n_sent, beam, target vocabulary
  // and longest sentence; hidden size, depth and attention may differ.  ensemble_sentences: the
  // same sentences integerised with the source vocabulary of each further model (the reference
  // integerises the text once per model, global_configuration.cc:985); empty = they share this
  // model's source ids.
  void DecodeBatch(const std::vector<std::vector<int>> &sentences, const DecodeOptions &o,
                   std::vector<SentenceResult> *results,
                   const std::vector<NeuralMachineTranslation *> &ensemble = {},
                   const std::vector<std::vector<std::vector<int>>> &ensemble_sentences = {});
  // The same search over any number of sentences with every beam column kept busy: a sentence
  // that has taken its last step hands its beam columns to the next sentence of the list, so the
  // sentences in flight are at different steps (nmt_stream.cc).  Local-p attention; ensembles,
  // alignment export and k-best lists as in DecodeBatch.  Every sentence goes through the steps
  // DecodeBatch takes it through.
  void DecodeStream(const std::vector<std::vector<int>> &sentences, const DecodeOptions &o,
                    std::vector<SentenceResult> *results,
                    const std::vector<NeuralMachineTranslation *> &ensemble = {},
                    const std::vector<std::vector<std::vector<int>>> &ensemble_sentences = {});
  const int *stream_layer0_mask_ = nullptr;  // DecodeStream: the first target layer's column mask of this tick
  // DecodeStream runs the encoder of the coming groups beside the decoding steps: a stream, a GEMM
  // workspace and events (two per group: "its slab is free", "it is encoded") of its own
  hipStream_t encoder_stream_ = nullptr;
  DeviceArray<char> encoder_workspace_;
  std::vector<hipEvent_t> stream_events_;
  int stream_ticks_ = 0;                     // steps the last DecodeStream took

  // ---- training --------------------------------------------------------------------------------
  DeviceArray<double> p_device_norm_workspace_, p_device_norms_;
  double last_global_norm_ = 0;
  bool apply_dropout_ = false;          // true only inside ComputeGradients
  unsigned long long minibatch_counter_ = 0;
  // What the consumer above layer `L` reads at step t: the dropped copy while training with
  // dropout, h_t otherwise.
  float *UpwardState(LstmLayer &L, int t) {
    return apply_dropout_ && L.out_dropout_ ? L.v_nodes_[t].p_device_h_t_dropped_
                                            : L.v_nodes_[t].p_device_h_t_;
  }
  // ComputeGradients (deep_rnn.h:984-1299) without its final UpdateWeights(): forward with stored
  // activations, backward, gradients left in the layers.  *_wgrad are the unique non-pad input ids
  // of the minibatch.  Returns the summed log-likelihood of the targets.
  double ComputeGradients(const int *p_host_source, int source_length, const int *p_host_target_in,
                          const int *p_host_target_out, int target_length,
                          const int *p_host_source_wgrad, int len_source_wgrad,
                          const int *p_host_target_wgrad, int len_target_wgrad,
                          const int *p_host_batch_information, int minibatch_size);
  // The same minibatch driven the reference's way (deep_rnn.h:1137-1273): after the forward pass,
  // target step by target step BackPropPreprocessGpu / BackProp1 / BackProp2 on the loss layer,
  // the attention node's BackProp, then BackPropPreprocessGpu + BackPropGpu(index) on every
  // LSTM node from the top layer down, and the same over the source side.  Same gradients as
  // ComputeGradients up to the order of the sums over steps.
  double ComputeGradientsStepwise(const int *p_host_source, int source_length,
                                  const int *p_host_target_in, const int *p_host_target_out,
                                  int target_length, const int *p_host_source_wgrad,
                                  int len_source_wgrad, const int *p_host_target_wgrad,
                                  int len_target_wgrad, const int *p_host_batch_information,
                                  int minibatch_size);
  // UpdateWeights (deep_rnn.h:1326-1412) + ClearGradients: scale, clip, theta += lr * g, zero.
  void UpdateWeights();
  void ClearGradients();
  bool GetGrad(const std::string &name, std::vector<float> *out);

  bool SetParam(const std::string &name, const float *host, size_t n);
  bool GetParam(const std::string &name, std::vector<float> *out);
  void Synchronize();

  // ---- model file (host/model_io.cc) -------------------------------------------------------------
  // The reference's text model file: header line, the two vocabulary mappings between lines of
  // '=', then every matrix as rows of numbers followed by an empty line, in the order of
  // DumpWeights (deep_rnn.h:2124-2146).  LoadWeights (deep_rnn.h:1878-1968) checks the header
  // against cfg_ and fills the parameters; DumpWeights appends the matrices to a file that already
  // holds the header part; DumpModel writes header, mappings (null: placeholder words) and matrices.
  void LoadWeights(const std::string &input_weight_file);
  void DumpWeights(const std::string &output_weight_file);
  // DumpBestModel (deep_rnn.h:1971-2040): header + mappings of const_model_name, current matrices.
  void DumpBestModel(const std::string &best_model_name, const std::string &const_model_name);
  // GetPerplexity (deep_rnn.h:1490-1568) over an integerised file (host/dispatcher.cc).
  double GetPerplexity(const std::string &test_file_name);
  void UpdateLearningRate(float new_learning_rate);
  void DumpModel(const std::string &output_weight_file, const std::vector<std::string> *source_words,
                 const std::vector<std::string> *target_words);
  // every parameter name in the order the model file stores them, with its (rows, cols)
  struct ParamShape {
    std::string name;
    int rows, cols;
  };
  std::vector<ParamShape> ModelFileOrder() const;

 private:
  // encoder + decoder + attention of a teacher-forced minibatch (shared by GetError and
  // ComputeGradients); per_step_loss: also run the loss of every step as GetError does.
  void RunSourceSide(int source_length, int minibatch_size);
  void RunSourceSideLanes(int source_length, int minibatch_size);
  void ForwardTeacherForced(const int *p_host_source, int source_length,
                            const int *p_host_target_in, const int *p_host_target_out,
                            int target_length, const int *p_host_batch_information,
                            int minibatch_size, bool per_step_loss);
};

// The reference's class names.  Its layer classes are templates over the precision with float the
// only instantiation (precision = float, src/utility_cu.h:42); both node kinds and both layer kinds
// are one class each here, so code written against the reference's names compiles against these.
template <typename T>
using LstmInputHiddenNode = LstmNode;
template <typename T>
using LstmHiddenHiddenNode = LstmNode;
template <typename T>
using InputToHiddenLayer = LstmLayer;
template <typename T>
using HiddenToHiddenLayer = LstmLayer;

}  // namespace linmt
