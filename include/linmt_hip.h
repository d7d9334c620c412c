/*
 * linmt_hip.h -- C ABI of liblinmt_hip.so: hand-written gfx950 (MI355X) HIP kernels for the
 * per-timestep LSTM / attention / softmax / beam path of LiNMT (liqiangnlp/LiNMT).
 *
 * Conventions (all taken from the reference so that its layer classes can call these directly):
 *   - every matrix is COLUMN-MAJOR, element (i,j) at j*ld+i  (reference: IDX2C, src/utility_cu.h:37);
 *   - activations are H x B (hidden index fastest, one column per sentence / hypothesis);
 *   - token / mask arrays are int32, -1 is padding before preprocessing, masks are 0/1;
 *   - every pointer is a DEVICE pointer owned by the caller unless a comment says "host";
 *   - nothing here allocates, frees or synchronises; work is queued on `stream` (a hipStream_t
 *     passed as void*, NULL = the default stream);
 *   - return value: 0 on success, LH_ERR_ARG for an argument the entry point rejects, otherwise
 *     the positive hipError_t of the failed launch.  lh_last_error() gives a text for the
 *     calling thread's last failure.  (The reference prints and exit()s instead,
 *     src/utility_cu.cu:171-214; the C++ layer classes built on this ABI keep that behaviour.)
 *
 * Gate stacking: wherever a 4H x B "stacked" matrix appears, rows [0,H) are the input gate i,
 * [H,2H) the forget gate f, [2H,3H) the candidate g = c' and [3H,4H) the output gate o.
 */
#ifndef LINMT_HIP_H_
#define LINMT_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LH_OK 0
#define LH_ERR_ARG (-1)

typedef void *lh_stream_t;

/* Library identification: returns LH_ABI_VERSION of the build. */
#define LH_ABI_VERSION 1
int lh_abi_version(void);
/* Text for the last non-zero status returned to the calling thread ("" if none). */
const char *lh_last_error(void);

/* ------------------------------------------------------------------------------------------
 * a1. Index preprocessing.
 * Replaces VocabTo01Kernel + VocabToNonMinus1Kernel (src/deep_rnn_kernel.cu:49-70) as launched by
 * InputToHiddenLayer::PreprocessGpuVocabIndices (src/layer_input_to_hidden.h:1478-1513) and
 * VocabSoftmaxKernel (src/deep_rnn_kernel.h:144-155): idx0 = idx==-1 ? 0 : idx,
 * mask01 = idx!=-1, mask01_f = (float)mask01.  idx0 may alias idx; mask01_f may be NULL.
 */
int lh_preprocess_indices_i32(const int *idx, int n, int *idx0, int *mask01, float *mask01_f,
                              lh_stream_t stream);

/* Replaces SetupReverseIndices (src/deep_rnn_kernel.cu:348-352): rev[unique[k]] = k, k < n_unique.
 * rev has (at least) vocab-size entries; entries of ids not in `unique` are left untouched. */
int lh_setup_reverse_indices_i32(const int *unique, int n_unique, int *rev, int vocab,
                                 lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a2. Sparse embedding lookup (+ dropout).
 * Replaces SparseLookupKernel (src/deep_rnn_kernel.h:249-255) followed by DropoutKernel
 * (src/deep_rnn_kernel.h:1059-1063) in LstmInputHiddenNode::ForwardPropGpu
 * (src/node_input_to_hidden.h:236-272).  W is E x V, idx0 has B entries in [0,V), out is E x B:
 *   out[:,b] = W[:,idx0[b]]            and, when drop_mask != NULL,
 *   out[i,b] = (drop_mask[i,b] < keep) * (1/keep) * out[i,b]      (keep = probability of KEEPING).
 */
int lh_embed_lookup_f32(const float *W, int E, int V, const int *idx0, int B,
                        const float *drop_mask, float keep, float *out, lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a4. Dense contractions on MFMA (v_mfma_f32_32x32x2_f32), fp32 in / fp32 accumulate.
 * Replaces CublasGemmWrapper (src/utility_cu.h:153-169) at the call sites of the gate products
 * (src/node_input_to_hidden.h:297-556, src/node_hidden_to_hidden.h:248-386), the attention
 * projections (src/layer_attention.h:272,327,441,448) and the output projection
 * (src/layer_loss.h:820), plus the elementwise kernels the reference launches right after them
 * (MatrixBiasKernel deep_rnn_kernel.h:525, TanhKernel deep_rnn_kernel.cu:277,
 * TanhAttentionForwardKernel + ZeroHT deep_rnn_kernel.h:1282-1295), which become the epilogue.
 *
 *   acc      = sum_{s < nseg} op(A_s) (M x K_s) * op(X_s) (K_s x N)
 *   v        = alpha * acc + (beta != 0 ? beta * C : 0) + (bias ? bias[m] : 0)
 *   v        = act == LH_ACT_TANH ? tanhf(v) : v
 *   C[m,n]   = colmask ? v * colmask[n] : v
 *
 * Several segments give the stacked product W*[x;h;h~] without materialising [x;h;h~].
 * transA: A_s is stored K_s x M (lda >= K_s) and used transposed; transX: X_s is stored N x K_s.
 * Both flags apply to every segment.  `segs` is a HOST array, nseg <= LH_GEMM_MAX_SEGS.
 */
#define LH_GEMM_MAX_SEGS 3
#define LH_ACT_NONE 0
#define LH_ACT_TANH 1
typedef struct lh_gemm_seg {
  const float *A; /* device */
  int lda;
  const float *X; /* device */
  int ldx;
  int K;
} lh_gemm_seg;
int lh_gemm_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX,
                float alpha, float beta, const float *bias, int act, const int *colmask, float *C,
                int ldc, lh_stream_t stream);
/* Same, with the activation applied only to rows m < act_rows.  Lets two products that share X
 * run as one launch on row-stacked weights, e.g. [W_p ; W_a^T] * ha with tanh on the W_p half
 * (src/layer_attention.h:272-275 and :327). */
int lh_gemm_act_rows_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX,
                         float alpha, float beta, const float *bias, int act, int act_rows,
                         const int *colmask, float *C, int ldc, lh_stream_t stream);
/* Same product, allowed to split the K dimension across workgroups when the output alone has
 * too few tiles to fill the GPU (the recurrent gate and attention products of a decoding step;
 * no counterpart in the reference, where cuBLAS makes that choice internally).  Each share
 * writes its partial sums into a plane of `workspace`; a second launch adds the planes in a fixed
 * order and applies the epilogue, so results do not depend on scheduling.  `workspace` is device
 * memory, 16-byte aligned, `workspace_bytes` long; its contents before and after a call mean
 * nothing.  Calls that share a workspace must be ordered on one stream.  A null or small
 * workspace only limits the split (a plane is M x N floats); 64 MiB covers every product here. */
int lh_gemm_ws_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX,
                   float alpha, float beta, const float *bias, int act, int act_rows,
                   const int *colmask, float *C, int ldc, void *workspace, size_t workspace_bytes,
                   lh_stream_t stream);
/* lh_gemm_ws_f32 for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc) and so have no workspace to hand over.  It
 * has no counterpart in the reference.  The partial planes go into an array of
 * LH_GEMM_NOALLOC_WS_BYTES that is part of the library's device code: each GPU the library runs
 * on holds its own copy until the process ends.  The limit: a product of which two partial planes
 * (((M + 3) & ~3) x N floats each) do not fit the array is rejected with LH_ERR_ARG, whether or
 * not it would be split.  For every product it accepts: same arguments, same choice of tile and
 * split and bit for bit the same result as lh_gemm_ws_f32 with a workspace of
 * LH_GEMM_NOALLOC_WS_BYTES.  No hipMalloc / hipFree and no allocating library routine is called.
 * Every call on a GPU shares that GPU's array (its contents between calls mean nothing, nothing
 * in it has to be cleared): calls that overlap in time on one GPU -- from different streams or
 * threads -- race on it; order them on one stream.
 * The first call on a device asks the runtime for the array's address on that device and raises
 * the LDS limit of the kernel instance it picks (neither is a stream operation, neither
 * allocates); a caller under graph capture does that ahead of the capture with
 * lh_gemm_noalloc_init, once per device with that device current, and by running each product
 * shape once before capturing it. */
#define LH_GEMM_NOALLOC_WS_BYTES (32u << 20)
int lh_gemm_noalloc_init(void);
int lh_gemm_noalloc_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX,
                        float alpha, float beta, const float *bias, int act, int act_rows,
                        const int *colmask, float *C, int ldc, lh_stream_t stream);
/* The plain product for a consumer that can add up partial sums itself (the LSTM cell kernel takes
 * three addends): like lh_gemm_ws_f32 with alpha = 1 and no bias / activation / mask, but a split
 * product is left unreduced.  *planes receives S, 1 <= S <= max_planes:
 *   S == 1: C = beta * C + product, as usual;
 *   S  > 1: C is NOT touched; plane s (0 <= s < S) is the ((M + 3) & ~3) x N column-major block at
 *           (float *)workspace + s * ((M + 3) & ~3) * N, and product = sum of the planes (the
 *           caller adds beta * C).
 * No counterpart in the reference. */
int lh_gemm_planes_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX,
                       float beta, float *C, int ldc, void *workspace, size_t workspace_bytes,
                       int max_planes, int *planes, lh_stream_t stream);
/* The stacked gate product of one LSTM step AND the cell, in one kernel (inference form: no gate
 * values kept, no dropout):
 *   pre = sum_s A_s X_s (+ addend[:, addend_col ? addend_col[b] : b]) + bias4h     (4H x B, never stored)
 *   c, h = cell(pre, c_prev, mask01)                        exactly as lh_lstm_cell_fwd_f32 computes them
 * Replaces, for one node, the 8-12 SGEMMs and the gate / cell / hidden-state kernels of
 * LstmInputHiddenNode::ForwardPropGpu (src/node_input_to_hidden.h:218-636) and
 * LstmHiddenHiddenNode::ForwardPropGpu (src/node_hidden_to_hidden.h:194-444).  A_s are the stacked
 * 4H x K_s gate matrices (rows g*H .. g*H+H-1 = gate g in the order i, f, c', o), X_s the K_s x B
 * inputs, all as stored (no transposes).  addend (4H x anything, leading dimension ld_addend, may
 * be NULL) holds pre-activation terms computed elsewhere: the input product of every step done
 * ahead of the recurrence, or -- with addend_col = the token of each column -- a table of input
 * products per vocabulary entry (addend_ncols of them; ids are clamped into that range like
 * lh_embed_lookup_f32 does), which makes the embedding lookup part of this kernel.
 * c may be c_prev; c and h must not overlap an X operand.
 * Only products that lh_gemm_planes_f32 would run as one unsplit launch of a tile whose LDS can
 * hold the whole tile are run this way: lh_gate_gemm_lstm_cell_plan says whether that is so
 * (*fusable) and names the kernel instance; when it is not, lh_gate_gemm_lstm_cell_f32 fails and
 * the caller uses lh_gemm_planes_f32 + lh_lstm_cell_fwd_f32.  workspace_bytes is what the caller
 * would hand lh_gemm_planes_f32 (it only steers the choice; no workspace is used). */
int lh_gate_gemm_lstm_cell_plan(int H, int B, const lh_gemm_seg *segs, int nseg, int has_addend,
                                size_t workspace_bytes, int *fusable, char *name, int name_cap);
int lh_gate_gemm_lstm_cell_f32(int H, int B, const lh_gemm_seg *segs, int nseg, const float *addend,
                               int ld_addend, const int *addend_col, int addend_ncols,
                               const float *bias4h,
                               const float *c_prev, const int *mask01, int sigmoid_f64,
                               float cell_clip, float *c, float *h, size_t workspace_bytes,
                               lh_stream_t stream);
/* The same kernel in the training form of the same reference code (the forward half of
 * src/node_input_to_hidden.h:218-636 and src/node_hidden_to_hidden.h:194-444 with train on): it also
 * stores what the backward pass and the layer above need, exactly as lh_lstm_cell_fwd_f32 does:
 *   gates  (4H x B, ld 4H, optional) receives i, f, g, o
 *   h_drop (H x B, optional)  = (next_drop_mask < keep) * (1/keep) * h
 * No addend_col (training looks embeddings up).  Same condition on when it runs
 * (lh_gate_gemm_lstm_cell_plan), same aliasing rules; gates and h_drop must not overlap an X
 * operand either. */
int lh_gate_gemm_lstm_cell_train_f32(int H, int B, const lh_gemm_seg *segs, int nseg,
                                     const float *addend, int ld_addend, const float *bias4h,
                                     const float *c_prev, const int *mask01, int sigmoid_f64,
                                     float cell_clip, float *gates, float *c, float *h,
                                     const float *next_drop_mask, float keep, float *h_drop,
                                     size_t workspace_bytes, lh_stream_t stream);
/* Several stacked gate products of one step in ONE launch (no counterpart in the reference, which
 * issues every layer's 8-12 SGEMMs one after the other, src/node_input_to_hidden.h:297-556,
 * src/node_hidden_to_hidden.h:248-386).  While decoding, what a step needs from the previous one is
 * known when the step starts: every layer's recurrent product W_h h_{t-1} and, for the first
 * target layer, the whole pre-activation (W_h h_{t-1} + Q h~_{t-1} + the folded embedding column).
 * Handing all of them over together gives the GPU a few thousand tiles at once; the products
 * that do depend on the step (M h_t of the layer below) then run with half the depth and take the
 * stored product as their addend (lh_gate_gemm_lstm_cell_f32).
 * Each problem is sum_s A_s X_s over the 4H x K_s stacked gate matrices and K_s x B inputs, as
 * stored.  cell != 0: the problem's pre-activations are complete and it ends in the LSTM cell,
 * fields as the arguments of the same name of lh_gate_gemm_lstm_cell_f32.  cell == 0: the 4H x B
 * product is stored to out (leading dimension ld_out >= 4H, 16-byte aligned).  No output may
 * overlap an X operand of any problem of the group.  lh_gate_gemm_group_plan says whether the group
 * runs this way (*runnable; aligned operands, H a multiple of 4) and names the kernel instance;
 * when it does not, lh_gate_gemm_group_f32 fails and the caller issues the products one by one. */
#define LH_GATE_GROUP_MAX 8
typedef struct lh_gate_problem {
  lh_gemm_seg segs[LH_GEMM_MAX_SEGS];
  int nseg;
  int cell;
  const float *addend;
  int ld_addend;
  const int *addend_col;
  int addend_ncols;
  const float *bias4h;
  const float *c_prev;
  const int *mask01;
  int sigmoid_f64;
  float cell_clip;
  float *c;
  float *h;
  float *out;
  int ld_out;
} lh_gate_problem;
int lh_gate_gemm_group_plan(int H, int B, const lh_gate_problem *problems, int n_problems,
                            int *runnable, char *name, int name_cap);
int lh_gate_gemm_group_f32(int H, int B, const lh_gate_problem *problems, int n_problems,
                           lh_stream_t stream);
/* Name of the kernel instance lh_gemm_ws_f32 (max_planes = 0) or lh_gemm_planes_f32 would launch
 * for this problem (tile shape and operand flags), as profilers print it; no counterpart in the
 * reference.  Pointers in `segs` are only inspected for alignment; workspace_bytes = 0 describes
 * lh_gemm_f32 / lh_gemm_act_rows_f32. */
int lh_gemm_kernel_name(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX,
                        size_t workspace_bytes, int max_planes, char *name, int name_cap);
/* Tuning and test aids (no counterpart in the reference).  Both overrides belong to the CALLING
 * THREAD: they change nothing for lh_gemm_* calls made from other host threads.
 * lh_gemm_set_config_override: forces tile configuration `config` for every later lh_gemm_* call
 * of this thread, config < 0 restores the built-in choice.  Returns the number of configurations
 * (so 0 <= config < return value), LH_ERR_ARG if config is too large.
 * lh_gemm_set_splits_override: likewise forces the K split of lh_gemm_ws_f32 (as far as the
 * workspace allows), splits <= 0 restores the built-in choice; returns the largest split.
 * lh_gemm_config_info: info = {BM, BN, WM, WN, WK, BK, workgroups resident per CU, LDS bytes} of a
 * configuration for the given operand flags. */
int lh_gemm_set_config_override(int config);
int lh_gemm_set_splits_override(int splits);
int lh_gemm_config_info(int config, int transA, int transX, int info[8]);

/* ------------------------------------------------------------------------------------------
 * a4 (second form). The same fp32 products on the bf16 matrix pipe, for callers that opt in.  No
 * counterpart in the reference (its products are cuBLAS SGEMM calls, src/utility_cu.h:153).
 * Every fp32 operand value a is held as three bf16 values a1 + a2 + a3 = a (a1 = bf16(a),
 * a2 = bf16(a - a1), a3 = bf16(a - a1 - a2)); a product a*x is formed as the six bf16 products
 * a1x1, a1x2, a2x1, a1x3, a2x2, a3x1 -- each exact -- added into an fp32 accumulator.  What is left
 * out is below 2^-23 |a x| per product, the size of one fp32 rounding; measured against float64 the
 * results are as close as those of lh_gemm_f32.  v_mfma_f32_32x32x16_bf16 issues at eight times
 * the fp32 MFMA rate, so six products take 3/8 of the matrix-pipe time.
 *
 * Operands are packed ahead of the product ("split planes", opaque to the caller):
 *   - lh_split_kgroups(K): k-groups (8 k each) a K-deep segment needs, ceil(K / 8);
 *   - lh_split_kgroups_padded(kgroups): the k-groups of a whole operand, the sum over its segments
 *     rounded up to whole slabs (a multiple of 16); the groups of padding must hold zeros;
 *   - lh_split_bytes(D, kgroups): bytes of a packed operand with D rows (A) or columns (X);
 *   - lh_split_gate_rows(H): the D to size a packed stacked gate matrix with (its rows are stored
 *     eight of gate i, eight of f, eight of c', eight of o, and so on);
 *   - lh_split_pack_f32 packs up to LH_SPLIT_PACK_MAX segments in one launch.  A segment is a D x K
 *     fp32 matrix (k_contiguous: element (d, k) at src[d * ld + k], the layout of an H x B
 *     activation used as X; otherwise src[k * ld + d], the layout of a stored weight matrix used
 *     as A) that becomes k-groups [kg_offset, kg_offset + kgroups) of an operand of kgroups_total
 *     k-groups, kgroups >= lh_split_kgroups(K); rows / columns up to the padded extent and k beyond
 *     K are written as zeros (give the last segment the operand's groups of padding as well).
 *     Several segments side by side give the operand of a multi-segment product ([x; h; h~]
 *     against [M | W_h | Q]; every segment but the last needs K % 8 == 0).  gate_H > 0: src is a stacked 4*gate_H x K gate matrix
 *     (D = 4 * gate_H) whose rows are laid out in cell-tile order for
 *     lh_gate_gemm_split_lstm_cell_f32.
 * A packed X depends on its column count: pack and product must be given the same N / B.
 * Operand values must be finite and below 3.3e38 in magnitude: the first bf16 term of a larger one
 * rounds to infinity, and where an fp32 product would give an infinity these give a NaN.
 * lh_gemm_split_f32: C = epilogue(alpha * A X + beta * C), epilogue exactly as lh_gemm_act_rows_f32.
 * lh_gate_gemm_split_lstm_cell_f32: lh_gate_gemm_lstm_cell_f32 on packed operands; H must be a
 * multiple of 8; addend, bias4h, c_prev, c, h 16-byte aligned.  h_planes != NULL: h is also
 * written as k-groups [hp_kg_offset, hp_kg_offset + hp_kgroups) of a packed X operand of
 * hp_kgroups_total k-groups and B columns (the input of the layer above, or of the next step; groups
 * beyond H / 8 are written as zeros), which saves the separate packing launch.
 * lh_gemm_split_set_config_override: test / tuning aid of the calling thread, like
 * lh_gemm_set_config_override. */
#define LH_SPLIT_PACK_MAX 8
typedef struct lh_split_source {
  const float *src;
  int ld;
  int k_contiguous;
  int D, K;
  int gate_H;
  void *planes;
  int kgroups_total;
  int kg_offset;
  int kgroups;
} lh_split_source;
int lh_split_kgroups(int K);
int lh_split_kgroups_padded(int kgroups);
int lh_split_padded(int D);
int lh_split_gate_rows(int H);
size_t lh_split_bytes(int D, int kgroups);
int lh_split_pack_f32(const lh_split_source *srcs, int n, lh_stream_t stream);
int lh_gemm_split_f32(int M, int N, int kgroups, const void *A_planes, const void *X_planes,
                      float alpha, float beta, const float *bias, int act, int act_rows,
                      const int *colmask, float *C, int ldc, lh_stream_t stream);
int lh_gate_gemm_split_lstm_cell_f32(int H, int B, int kgroups, const void *W_planes,
                                     const void *X_planes, const float *addend, int ld_addend,
                                     const int *addend_col, int addend_ncols, const float *bias4h,
                                     const float *c_prev, const int *mask01, int sigmoid_f64,
                                     float cell_clip, float *c, float *h, void *h_planes,
                                     int hp_kgroups_total, int hp_kg_offset, int hp_kgroups,
                                     lh_stream_t stream);
/* Name of the kernel instance the two products above would launch (cell != 0: M = H), as profilers
 * print it. */
int lh_gemm_split_kernel_name(int cell, int M, int N, char *name, int name_cap);
int lh_gemm_split_set_config_override(int config);

/* ------------------------------------------------------------------------------------------
 * a3. Fused LSTM cell forward: bias add, gate nonlinearities, c_t / h_t update, padding mask,
 * optional cell clip and the dropout mask of the layer above, in one pass over HBM.
 * Replaces ForwardSigmoidKernel / ForwardSigmoidKernelFeed / ForwardTanhKernel(/Feed)
 * (src/deep_rnn_kernel.cu:78-117, src/deep_rnn_kernel.h:64-88), ForwardCTKernel (.h:93),
 * ClipMatKernel (.h:1528), ForwardHTKernel (.cu:121), ZeroCTAndHT (.h:123) as sequenced in
 * LstmInputHiddenNode::ForwardPropGpu (src/node_input_to_hidden.h:350-621) and
 * LstmHiddenHiddenNode::ForwardPropGpu (src/node_hidden_to_hidden.h:270-430), and the
 * DropoutKernel the layer above applies to its copy of h (src/node_hidden_to_hidden.h:208-226).
 *
 *   s      = ((pre1 + pre2) + pre3) + bias            (4H x B stacked; pre2 / pre3 may be NULL)
 *   i,f,o  = 1/(1+exp(-s)), g = tanh(s)               fp32 expf/tanhf; with sigmoid_f64 != 0 the
 *                                                     three sigmoids are evaluated in double, as
 *                                                     ForwardSigmoidKernelFeed does
 *   c      = f*c_prev + i*g ; cell_clip > 0: c = clamp(c, +-cell_clip)
 *   h      = o*tanhf(c) ; h *= mask01[b] ; c *= mask01[b]        (i,f,g,o are not masked)
 *   gates  (4H x B, optional) receives i,f,g,o for the backward pass
 *   h_drop (H x B, optional)  = (next_drop_mask < keep) * (1/keep) * h
 * ld of every 4H x B operand is 4H, of every H x B operand H.  c may alias c_prev.
 * mask01[b] is 0 or 1; with LH_MASK_F32_GATES added to it, column b takes the fp32 sigmoids even
 * when sigmoid_f64 != 0 (a decoder that runs columns at different steps in one launch: the
 * reference evaluates the first step of a sentence with the plain kernels and every later one with
 * the Feed kernels, src/node_input_to_hidden.h:350-621).  lh_gate_gemm_lstm_cell_f32 reads its mask
 * the same way.
 */
#define LH_MASK_F32_GATES 2
int lh_lstm_cell_fwd_f32(int H, int B, const float *pre1, const float *pre2, const float *pre3,
                         const float *bias4h, const float *c_prev, const int *mask01,
                         int sigmoid_f64, float cell_clip, float *gates, float *c, float *h,
                         const float *next_drop_mask, float keep, float *h_drop,
                         lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a6. Attention core: alignment position, window, scores, max-subtracted exp, normalisation,
 * Gaussian weighting and context vector in one kernel (one workgroup per column).
 * Replaces SigmoidKernel, AlignmentPosKernel, LowerUpperKernel (src/deep_rnn_kernel.h:1076-1100),
 * CreateIndicesKernel (src/deep_rnn_kernel.cu:294-316), LoadInHSKernel (.h:1142-1164),
 * ElemReduceKernelLarge (.h:1309-1342), AlignmentReductionKernel (.h:1198-1241),
 * GetViterbiAlignmentKernel (.h:1105-1117) and CreateCTKernel (.h:1251-1260) as sequenced in
 * AttentionNode::ForwardProp (src/layer_attention.h:282-392).
 *
 * Inputs:  tanh1 = tanh(W_p*ha) (H x B), v_p (H), wa = W_a^T*ha (H x B), mask01 (B),
 *          batch_info = [len_0..len_{B-1}, off_0..off_{B-1}]  (src/file_helper.cc:242-243),
 *          encoder top-layer states: state of encoder timestep tau, column c, is the H floats at
 *          hs + tau*hs_step_stride + c*hs_col_stride; column c = hs_col ? hs_col[b] : b
 *          (hs_col lets the beam columns of one sentence share that sentence's states instead
 *          of the reference's per-beam replicas, src/deep_rnn.h:1633-1643).
 * Local-p (D >= 0), W = 2D+1:
 *   sig_b = 1/(1+exp(-(double)(v_p . tanh1[:,b])))  ; p_b = len_b * sig_b
 *   lo = max(0,(int)p_b - D) ; hi = min(len_b-1,(int)p_b + D)
 *   idx[b,j] = (mask01[b]==1 && lo+j <= hi) ? lo+j : -1                (B x W, at b + B*j)
 *   hs_j = idx>=0 ? state(tau = len_b-1-idx + off_b) : 0 ; sc_j = hs_j . wa[:,b]
 *   mx = max(0, max_valid sc_j) ; e_j = exp(sc_j - mx) ; Z = sum e_j
 *   g_j = valid ? exp(-(p_b-idx)^2 / (2*sigma^2)) : 1,  sigma^2 = D*D/4.0        (W x B, at j + W*b)
 *   a_j = valid ? (Z != 0 ? e_j/Z : e_j) * g_j : 0                             (B x W, at b + B*j)
 *   ctx[:,b] = sum_j a_j * hs_j ; viterbi[b] = idx of the first maximal a_j (-1 if none > -1)
 * Global "general" (D < 0; not in the reference, the textbook Luong global attention):
 *   window = all len_b source positions (W = max_len slots, idx = j for j < len_b when
 *   mask01[b]==1), no p_b / Gaussian (g = 1, p_t/sigma outputs untouched), mx = true maximum.
 * Outputs p_t (B), sigma (B), indices (B x W), align (B x W), cached_exp (W x B), ctx (H x B),
 * viterbi (B, optional).  max_len (= the W of the global variant) is ignored for D >= 0.
 * hs_steps = number of encoder timesteps held in hs; a slot whose tau falls outside [0,hs_steps)
 * reads as a zero vector instead of touching memory outside the buffer.
 * proj_col_stride = distance in floats between the columns of tanh1 and of wa (0 = H): both may be
 * halves of one 2H x B product of row-stacked [W_p ; W_a^T] (lh_gemm_act_rows_f32).
 */
int lh_attn_core_fwd_f32(int H, int B, int D, int max_len, int hs_steps, const float *tanh1,
                         const float *v_p, const float *wa, long long proj_col_stride,
                         const float *hs, long long hs_step_stride,
                         long long hs_col_stride, const int *hs_col, const int *batch_info,
                         const int *mask01, float *p_t, float *sigma, int *indices, float *align,
                         float *cached_exp, float *ctx, int *viterbi, lh_stream_t stream);

/* The same attention step over a PROJECTED memory, for decoding, where one sentence's encoder
 * states serve every step of its beam: with score_mem = W_a * hs and ctx_mem = W_c1 * hs computed
 * once per sentence (two plain lh_gemm_f32 calls over all source positions),
 *   score_j = h_t . score_mem_j            (= (W_a^T h_t) . hs_j of AttentionNode::ForwardProp)
 *   h~      = tanh(sum_j a_j ctx_mem_j + out_add + out_bias) * mask01
 *           (= tanh(W_c1 c_t + W_c2 h_t + b) with out_add = W_c2 h_t, src/layer_attention.h:447-478),
 * so the per-step products W_a^T h_t and W_c1 c_t are gone and the context vector never exists.
 * tanh1 = tanh(W_p h_t) as in lh_attn_core_fwd_f32; tanh1, h_t and out_add are H x B with the given
 * column strides (0 = H); the memories are addressed like hs there (mem_col = hs_col).  Everything
 * else (p_t, sigma, indices, align, cached_exp, viterbi) is written exactly as
 * lh_attn_core_fwd_f32 writes it.  Local-p only, window 2D+1 <= LH_ATTN_PROJECTED_MAX_WINDOW,
 * H <= LH_ATTN_PROJECTED_MAX_H and a multiple of 4, 16-byte aligned operands: other cases use
 * lh_attn_core_fwd_f32 and the two products.  No counterpart in the reference (an algebraic
 * regrouping of its step). */
#define LH_ATTN_PROJECTED_MAX_WINDOW 21
#define LH_ATTN_PROJECTED_MAX_H 2048
int lh_attn_core_projected_fwd_f32(int H, int B, int D, int hs_steps, const float *tanh1,
                                   long long tanh1_col_stride, const float *v_p, const float *h_t,
                                   long long h_t_col_stride, const float *score_mem,
                                   const float *ctx_mem, long long mem_step_stride,
                                   long long mem_col_stride, const int *mem_col,
                                   const int *batch_info, const int *mask01, const float *out_add,
                                   long long out_add_col_stride, const float *out_bias, float *p_t,
                                   float *sigma, int *indices, float *align, float *cached_exp,
                                   float *h_tild, int *viterbi, lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a8 / a9. Vocabulary softmax and log-likelihood, one pass over the V x B logits.
 *
 * lh_softmax_fwd_f32 replaces MatrixBiasKernel + OutputdistOverflowPreventionKernel
 * (src/deep_rnn_kernel.h:525-530,353-429) in SoftmaxLayer::GetDistributionGpu
 * (src/layer_loss.h:822-868): p[:,b] = softmax(logits[:,b] + bias), fp32.  p may alias logits.
 * bias may be NULL (already added by the GEMM epilogue).
 *
 * lh_train_loglik_f32 replaces TrainPerplexityKernel (src/deep_rnn_kernel.h:336-342):
 *   *accum += sum_{b: mask01[b]==1} log((double)p[tgt0[b], b]).
 *
 * lh_logsoftmax_xent_f32 replaces OutputdistPerplexityKernel (src/deep_rnn_kernel.h:433-519) and
 * the host loop of SoftmaxLayer::ComputeLossGpu (src/layer_loss.h:693-701) without the V x B
 * double buffer: logp_tgt[b] = log(exp(z_t - mx)) - log(sum_v exp(z_v - mx)) in double with
 * z = logits + bias, where the V exponentials under the sum are single-precision values added up
 * in double (the reference takes them in double too; the result differs by ~1e-7, against a
 * tolerance of 1e-5 on a log-probability); *loss_accum += sum_{b: mask01[b]==1} logp_tgt[b].
 * logp_tgt may be NULL.
 */
int lh_softmax_fwd_f32(const float *logits, int ldl, const float *bias, int V, int B, float *p,
                       int ldp, lh_stream_t stream);
int lh_train_loglik_f32(const float *p, int ldp, int V, int B, const int *tgt0, const int *mask01,
                        double *accum, lh_stream_t stream);
int lh_logsoftmax_xent_f32(const float *logits, int ldl, const float *bias, int V, int B,
                           const int *tgt0, const int *mask01, double *logp_tgt,
                           double *loss_accum, lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a10. Beam search step on the device.
 *
 * lh_beam_topk_f32: fused log-softmax + per-column top-K.  Replaces the V x beam distribution
 * copy (src/decoder.h:1413), CopyDistToEigen (:1429-1436), EnsemblesModels' renormalisation
 * (:1910-1931) and the per-column bounded heap of Decoder::ExpandHypothesis (:398-427).
 * For each column b < B: mx, lse = log(sum exp(z - mx)), the K largest z (ties: lowest vocab id
 * wins, as the strict `<` of decoder.h:405 keeps the earlier entry), best first:
 *   cand_logp[k + K*b] = z_k - mx - lse ; cand_id[k + K*b] = vocab id ; logp_eof[b] = logp of id
 *   `eof_id` (used by FinishCurrentHypotheses, decoder.h:506).  K <= LH_BEAM_MAX_K, K <= V.
 *
 * lh_beam_merge_f32: per-sentence merge of the candidates.  Replaces the global heap walk of
 * Decoder::ExpandHypothesis (src/decoder.h:429-480) and FinishCurrentHypotheses (:502-525) for
 * n_sent sentences at once (sentence s owns columns [s*beam, (s+1)*beam)).
 *   expansion (step < limit[s]): candidates of column i (only i = 0 when step == 0) get
 *     score = cand_logp + prev_score[i] - rank*diversity (rank 1 = best of its column); walk all
 *     candidates by (score desc, beam column asc, vocab id asc): id == start_id is dropped;
 *     id == eof_id is recorded as finished (fin_beam, fin_score = score + penalty) and takes no
 *     slot; otherwise slot k gets tok, backptr (GLOBAL column index s*beam + i), score + penalty.
 *     If the candidates run out (the reference pops an empty heap there) the remaining slots get
 *     tok = eof_id, backptr = s*beam, score = -FLT_MAX.
 *   finish (step == limit[s]): every column i is recorded as finished with
 *     fin_score = prev_score[i] + logp_eof[i] + penalty; tok/backptr/score keep column i
 *     (tok = eof_id, backptr = own column).
 *   idle (step > limit[s]): tok = eof_id, backptr = own column, score unchanged, no finished.
 * Outputs per step: tok, backptr, score (n_sent*beam each; score may alias prev_score is NOT
 * allowed), fin_count (n_sent), fin_beam / fin_score (n_sent*beam, first fin_count[s] valid, in
 * walk order).  K = beam + 1 in the reference.
 */
#define LH_BEAM_MAX_K 64
int lh_beam_topk_f32(const float *logits, int ldl, const float *bias, int V, int B, int K,
                     int eof_id, float *cand_logp, int *cand_id, float *logp_eof,
                     lh_stream_t stream);
/* The same selection over the combined distribution of several models.  Replaces
 * EnsembleFactory::EnsemblesModels (src/decoder.h:1910-1931) in front of ExpandHypothesis:
 *   q[v,b] = (float)((sum over models, in double, of p[m][v + ldp*b]) / n_models),
 *   cand_logp = log(q / sum_v q[v,b]) for the K largest q of column b (ties: lowest id), likewise
 *   logp_eof.  p[m] are the models' probabilities (lh_softmax_fwd_f32), V x B each with leading
 *   dimension ldp.  Needs V % 4 == 0, ldp % 4 == 0, 16-byte aligned p[m], V <= 65536,
 *   n_models <= LH_ENSEMBLE_MAX_MODELS.  p is a HOST array of device pointers. */
#define LH_ENSEMBLE_MAX_MODELS 8
int lh_beam_topk_ensemble_f32(const float *const *p, int n_models, int ldp, int V, int B, int K,
                              int eof_id, float *cand_logp, int *cand_id, float *logp_eof,
                              lh_stream_t stream);
int lh_beam_merge_f32(int n_sent, int beam, int K, int step, const int *limit,
                      const float *cand_logp, const int *cand_id, const float *logp_eof,
                      const float *prev_score, float diversity, float penalty, int start_id,
                      int eof_id, int *tok, int *backptr, float *score, int *fin_count,
                      int *fin_beam, float *fin_score, lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a11. Hypothesis state gather: dst_t[:,k] = src_t[:,backptr[k]], k < B, for n_tensors tensors in
 * one launch (dst_t is H x B, src_t is H x B_src; a backptr outside [0,B_src) is clamped into it).  Replaces the per-column cudaMemcpy loops of SwapStatesDecoding
 * (src/layer_input_to_hidden.h:1517-1531, src/layer_hidden_to_hidden.h:569-584), the h~ swap of
 * NeuralMachineTranslation::SwapDecodingStates (src/deep_rnn.h:1842-1857) and the whole-matrix
 * copies of TargetCopyPrevStates (src/deep_rnn.h:1861-1872).  src/dst are HOST arrays of device
 * pointers, n_tensors <= LH_GATHER_MAX_TENSORS; dst_t must not alias any src.
 * With backptr[k] = sentence of beam column k and B_src = number of sentences this is also
 * TransferDecodingStatesGpu (src/layer_input_to_hidden.h:1536-1545), the broadcast of the encoder's
 * final state to the beam columns.
 */
#define LH_GATHER_MAX_TENSORS 24
int lh_beam_gather_f32(const float *const *src, float *const *dst, int n_tensors, int H, int B,
                       int B_src, const int *backptr, lh_stream_t stream);

/* a10 + a11 in one launch: lh_beam_merge_f32 followed by lh_beam_gather_f32 over the n_sent*beam
 * columns with the back-pointers just chosen (B = B_src = n_sent*beam), i.e. the tail of
 * Decoder::ExpandHypothesis (src/decoder.h:430-480) and NeuralMachineTranslation::
 * SwapDecodingStates (src/deep_rnn.h:1842-1857) behind it.  Same arguments, same outputs bit for
 * bit as the two calls; several workgroups per sentence repeat the (cheap) merge so that the
 * copies of a sentence's columns start without a second launch.  beam <= 256. */
int lh_beam_merge_gather_f32(int n_sent, int beam, int K, int step, const int *limit,
                             const float *cand_logp, const int *cand_id, const float *logp_eof,
                             const float *prev_score, float diversity, float penalty, int start_id,
                             int eof_id, int *tok, int *backptr, float *score, int *fin_count,
                             int *fin_beam, float *fin_score, const float *const *src,
                             float *const *dst, int n_tensors, int H, lh_stream_t stream);

/* A decoder that keeps every beam column busy (no counterpart in the reference, whose
 * Decoder works on one sentence at a time): the beam columns of a sentence ("slot") are handed to
 * the next sentence of the input as soon as the sentence has taken its last step, so the sentences
 * in flight are at different steps.
 *
 * lh_beam_merge_gather_stream_f32 is lh_beam_merge_gather_f32 with sentence s at step
 * tick - start[s] (limit[s] counts from the sentence's own first step; a slot without a sentence
 * has limit -1 and idles).
 *
 * lh_stream_admit_f32 puts n_adm <= LH_STREAM_ADMIT_MAX sentences into slots, in one launch.  For
 * admission q (a HOST array): start[slot] = tick, limit[slot] = limit; for the slot's beam columns
 * c: hs_col[c] = hs_col_value, batch_info[c] = len, batch_info[B + c] = off (either array may be
 * NULL), tok_prev[c] = start_id, score_prev[c] = 0; dst_t[:, c] = src_t[:, sentence_col] for the
 * n_tensors state tensors (src_t is H x n_src: the encoder's final states, what
 * TransferDecodingStatesGpu broadcasts, src/layer_input_to_hidden.h:1536-1545) and zero_t[:, c] = 0
 * for the n_zero tensors that start a sentence at zero (h~ of the step before).  src / dst / zero
 * are HOST arrays of device pointers.  The admissions of a call name different slots. */
#define LH_STREAM_ADMIT_MAX 16
typedef struct {
  int slot, sentence_col, hs_col_value, len, off, limit, tick;
} lh_stream_admission;
int lh_beam_merge_gather_stream_f32(int n_sent, int beam, int K, int tick, const int *start,
                                    const int *limit, const float *cand_logp, const int *cand_id,
                                    const float *logp_eof, const float *prev_score, float diversity,
                                    float penalty, int start_id, int eof_id, int *tok, int *backptr,
                                    float *score, int *fin_count, int *fin_beam, float *fin_score,
                                    const float *const *src, float *const *dst, int n_tensors, int H,
                                    lh_stream_t stream);
int lh_stream_admit_f32(const lh_stream_admission *adm, int n_adm, int beam, int B, int *start,
                        int *limit, int *hs_col, int *batch_info, const float *const *src,
                        float *const *dst, int n_tensors, float *const *zero, int n_zero, int H,
                        int n_src, int *tok_prev, int start_id, float *score_prev, lh_stream_t stream);

/* ==========================================================================================
 * Training half of the path (backward pass and update).
 * ========================================================================================== */

/* Uniform numbers in (0, 1] for the dropout masks: out[i] is a fixed function of (seed, i).
 * Replaces curandGenerateUniform (src/utility_cu.cu:218-226) at the mask sites
 * (src/node_input_to_hidden.h:268, src/node_hidden_to_hidden.h:220, src/layer_attention.h:259,
 * src/layer_loss.h:504); the values differ from cuRAND's XORWOW stream, the distribution and the
 * (0, 1] range do not.  A mask keeps an element when mask < keep. */
int lh_uniform_f32(float *out, long long n, unsigned long long seed, lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a16. Softmax output error and log-likelihood in one pass over the V x B logits.
 * Replaces, for one step, the forward OutputdistOverflowPreventionKernel
 * (src/deep_rnn_kernel.h:353-429), TrainPerplexityKernel (:336-342) and the elementwise part of
 * SoftmaxLayer::GetHTGradientGpu / ComputeDGradientGpu / ComputeBDGradientGpu
 * (src/layer_loss.h:547-626, 887-972), which all consume p and the one-hot target:
 *   p        = softmax(logits[:,b] + bias)
 *   dz[:,b]  = mask01[b] * (onehot(tgt0[b]) - p)               (may alias logits)
 *   logp_tgt[b] = log((double)p[tgt0[b]]) ; *loss_accum += sum_{b: mask01[b]==1} logp_tgt[b]
 * With dz the three gradient products of the reference are plain GEMMs / row sums:
 *   dh~ = D^T dz ; dD += dz h~^T ; db_d += dz 1.
 */
int lh_softmax_xent_grad_f32(const float *logits, int ldl, const float *bias, int V, int B,
                             const int *tgt0, const int *mask01, float *dz, int ldz,
                             double *logp_tgt, double *loss_accum, lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a13. Fused LSTM cell backward: everything between the incoming errors and the four gate errors.
 * Replaces the two geam sums, DErrtCTKernel (src/deep_rnn_kernel.h:152), ZeroColumnsKernel,
 * DErrnToTOTKernel, DErrnToTFTITKernel (twice), DErrnToTTanhcptKernel, ElementwiseMultKernel and
 * the ClipMatKernel calls on incoming errors, as sequenced in LstmInputHiddenNode::BackPropGpu
 * (src/node_input_to_hidden.h:647-983) and LstmHiddenHiddenNode::BackPropGpu
 * (src/node_hidden_to_hidden.h:537-900):
 *   dh  = clamp(dh_next, clip_next) + clamp(dh_above, clip_above)     (NULL = 0; clip <= 0 = off)
 *   dc  = dc_next + dh * o * (1 - tanh(c)^2) ; dh *= mask01[b] ; dc *= mask01[b]
 *   do  = dh * tanh(c) * o(1-o) ; df = dc * c_prev * f(1-f) ; di = dc * g * i(1-i)
 *   dg  = dc * i * (1 - g^2) ; dc_prev = dc * f
 * gates (4H x B: i,f,g,o as written by lh_lstm_cell_fwd_f32), c, c_prev are the stored forward
 * values; dgates (4H x B) receives di,df,dg,do in the same stacking, so that
 *   [dx ; dh_prev ; dh~_prev] = [M | W_h | Q]^T dgates   and   d[M | W_h | Q] += dgates [x;h;h~]^T
 * are single GEMMs on the stacked weights.  dc_prev may alias dc_next.
 * The reference clamps the errors it hands back (dh_{t-1}, dh~_{t-1}, dx) to +-error_clip when
 * --clip-cell is on; here the consumer clamps on read, which is the same values.
 * above_drop_mask (H x B, optional): the consumer above (next layer, attention node or softmax) read
 * a dropped copy of this node's h, so its error comes back through the same mask, as the
 * DropoutKernel calls on d_errn_to_t_h_below (src/node_hidden_to_hidden.h:782), errn_to_t_ht_p1
 * (src/layer_attention.h:683) and d_errt_ht (src/layer_loss.h:598) do:
 *   dh_above <- clamp(dh_above) * (above_drop_mask < keep) * (1/keep).
 */
int lh_lstm_cell_bwd_f32(int H, int B, const float *dh_above, const float *dh_next,
                         const float *dc_next, const float *gates, const float *c,
                         const float *c_prev, const int *mask01, float clip_above, float clip_next,
                         const float *above_drop_mask, float keep, float *dgates, float *dc_prev,
                         lh_stream_t stream);
/* The same step with each incoming error given as a sum of partial planes: a W^T d product whose
 * K range was split over workgroups (lh_gemm_planes_f32) can be consumed as it lies, without the
 * launch that adds its planes.  A term is `planes` (1..LH_ERROR_TERM_MAX_PLANES) column-major
 * H x B blocks of leading dimension ld >= H, plane s at p + s * plane_stride; its value is
 * ((plane 0 + plane 1) + plane 2) ..., the order in which lh_gemm_ws_f32's second launch adds them,
 * so the results are bit for bit those of lh_lstm_cell_bwd_f32 on the reduced product.  The clamp
 * and the dropout mask apply to the sum.  above / next == NULL or p == NULL: no such error.
 * No counterpart in the reference (cuBLAS splits and reduces inside cublasSgemm). */
#define LH_ERROR_TERM_MAX_PLANES 8
typedef struct lh_error_term {
  const float *p;
  int planes;
  long long plane_stride; /* floats between planes; ignored when planes == 1 */
  int ld;
} lh_error_term;
int lh_lstm_cell_bwd_terms_f32(int H, int B, const lh_error_term *above, const lh_error_term *next,
                               const float *dc_next, const float *gates, const float *c,
                               const float *c_prev, const int *mask01, float clip_above,
                               float clip_next, const float *above_drop_mask, float keep,
                               float *dgates, float *dc_prev, lh_stream_t stream);

/* out[r] = beta*out[r] + sum_c A[r,c] for a column-major rows x cols matrix.  Replaces the
 * cublasSgemv-with-ones bias gradients (src/node_input_to_hidden.h:1215-1240,
 * src/layer_attention.h:541, :600, src/layer_loss.h:938-972).  Fixed summation order. */
int lh_rowsum_acc_f32(const float *A, long long lda, int rows, long long cols, float beta,
                      float *out, lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a14. Embedding gradient.  Replaces WSmallGradientKernel (src/deep_rnn_kernel.h:270-285), whose
 * atomicAdd scatter makes the sum order vary from run to run: here the caller lists, per unique
 * id k, the dx columns that carry that id (seg_cols[seg_start[k] .. seg_start[k+1])), and
 *   small_grad[:,k] = beta*small_grad[:,k] + sum_{s} dx[:, seg_cols[s]]       (E rows)
 * added up in an order that the list alone fixes (16 interleaved partial sums, then those in
 * order), so the result does not vary from run to run.  Padding columns are simply not listed.  drop_mask (laid out like dx, optional):
 * every dx element is first multiplied by (drop_mask < keep) * (1/keep), the embedding dropout of
 * WSmallGradientKernelDropout (src/deep_rnn_kernel.h:288-303).
 */
int lh_embed_gather_grad_f32(const float *dx, long long ldx, int E, int n_unique,
                             const int *seg_start, const int *seg_cols, const float *drop_mask,
                             float keep, float beta, float *small_grad, long long ldg,
                             lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a15. Attention backward.
 * lh_attn_delta_f32 replaces AddTwoMatsKernel (feed-input error), ZeroHT and TanhGradKernel at the
 * top of AttentionNode::BackProp (src/layer_attention.h:490-512):
 *   delta = (dht + clamp(dht_feed, clip_feed)) * mask01[b] * (1 - h_tild^2)    (dht_feed may be NULL)
 * lh_attn_core_bwd_f32 replaces ErrorAlignmentsKernelLarge, ErrorHSAndCTKernelLarge, ErrorPTKernel,
 * AttentionVPErrorKernel, GradWPKernel, GetHTScalingsWaGradKernel and the 2D+1 rounds of
 * ScaleHTKernel / AddTwoMatsKernel / CopyErrorsSource (src/layer_attention.h:572-660,
 * src/deep_rnn_kernel.h:1348-1520), one workgroup per column; the stored forward values come from
 * lh_attn_core_fwd_f32 (same layouts), dctx = W_c1^T delta:
 *   das_j  = dctx[:,b] . hs_j
 *   dp     = sum_j das_j a_j (idx_j - p_b)/sigma^2                               (local-p only)
 *   r_j    = das_j a_j - (a_j/g_j) * sum_k das_k a_k
 *   hsum[:,b] = sum_j r_j hs_j
 *   dhs(tau_j)[:,b] += dctx[:,b] a_j + wa[:,b] r_j        (valid slots; dhs has the layout of hs)
 *   u[:,b] = dp sig(1-sig) len tanh1[:,b] ; w[:,b] = dp len sig(1-sig) v_p (1 - tanh1[:,b]^2)
 * after which dv_p += u 1, dW_p += w ha^T, dW_a += ha hsum^T and dha = W_c2^T delta + W_p^T w +
 * W_a hsum are row sums / GEMMs.  Every column must own its states (no hs_col sharing).
 */
int lh_attn_delta_f32(int H, int B, const float *dht, const float *dht_feed, const float *h_tild,
                      const int *mask01, float clip_feed, float *delta, lh_stream_t stream);
int lh_attn_core_bwd_f32(int H, int B, int D, int max_len, int hs_steps, const float *dctx,
                         const float *tanh1, const float *v_p, const float *wa, const float *hs,
                         long long hs_step_stride, long long hs_col_stride, const int *batch_info,
                         const float *p_t, const float *sigma, const int *indices,
                         const float *align, const float *cached_exp, float *dhs, float *hsum,
                         float *u, float *w, lh_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * a17. Gradient norm and the fused scale / clip / SGD / clear step.
 * lh_grad_sumsq_f32 replaces BasicComputeNormP1/P2 + the blocking copy of NormClipGpuV2P1
 * (src/deep_rnn_kernel.h:618-708): *accum += sum (scale*g)^2 over a rows x cols view (leading
 * dimension ld), accumulated in double on the device; workspace holds LH_SUMSQ_WORKSPACE doubles.
 * lh_sgd_step_f32 replaces ScaleFunctor (ScaleGradients), ReScaleNormFunctor (NormClipGpuV2 /
 * NormClipGpuV2P2), ClipMatKernel (individual clip), the geam / AddGradVecs / UpdateSparseGradient
 * updates (src/layer_input_to_hidden.h:1145-1276, src/deep_rnn_kernel.h:883-894) and the
 * cudaMemset of ClearGradients, in one pass:
 *   v = grad_scale * g ; f = sumsq ? (sqrt(*sumsq) > norm_clip ? norm_clip/sqrt(*sumsq) : 1) : 1
 *   v = f*v ; individual_clip > 0: v = clamp(v, +-individual_clip)
 *   theta[:, col_index ? col_index[c] : c] += learning_rate * v ; g = 0
 * sumsq is read on the device, so no host synchronisation sits between norm and update.
 */
#define LH_SUMSQ_WORKSPACE 1024
int lh_grad_sumsq_f32(const float *g, long long rows, long long cols, long long ld, float scale,
                      double *workspace, double *accum, lh_stream_t stream);
int lh_sgd_step_f32(float *theta, long long ld_theta, float *g, long long ld_g, long long rows,
                    long long cols, const int *col_index, float learning_rate, float grad_scale,
                    const double *sumsq, float norm_clip, float individual_clip,
                    lh_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LINMT_HIP_H_ */
