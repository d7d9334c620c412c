// CPU oracle, training half: teacher-forced forward with stored activations, the reference's
// backward pass and its weight update.  TEST INFRASTRUCTURE ONLY (see linmt_oracle.h).
//
// Follows NeuralMachineTranslation::ComputeGradients (src/deep_rnn.h:984-1299) node by node, in the
// reference's order (target steps last to first, layers top to bottom, then the source side), with
// every gradient accumulated per step in fp32 as the reference's beta = 1 SGEMMs do:
//   softmax        src/layer_loss.h:547-626 (GetHTGradientGpu), :887-972 (D and b_d gradients)
//   attention      src/layer_attention.h:487-698 and the kernels of src/deep_rnn_kernel.h:1348-1520
//   LSTM cell      src/node_input_to_hidden.h:647-983, :997-1300; src/node_hidden_to_hidden.h:537-1108
//   embedding      WSmallGradientKernel, src/deep_rnn_kernel.h:270-285
//   update         src/deep_rnn.h:1326-1412; src/layer_input_to_hidden.h:1062-1276,1283-1360,1428-1470
//
// pin: tests compare every gradient with central differences of an independent float64 numpy
// restatement of the forward pass (the reference's own check, src/layer_input_to_hidden.h:1016-1051,
// is the same method), and the update with its closed form.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "linmt_oracle.h"

// from linmt_oracle.cpp: the transposed copy the model keeps of a matrix after orc_model_commit,
// and the product on such a copy (what orc_gemm does after transposing A itself)
const float *orc_model_rowmajor(orc_model *m, const char *name);
void orc_gemm_rowmajor_a(int M, int N, int K, const float *At, const float *X, int ldx, float alpha,
                         float beta, float *C, int ldc);

namespace {

inline size_t idx2c(size_t i, size_t j, size_t ld) { return j * ld + i; }
const char *kGate[4] = {"i", "f", "c", "o"};  // stacked order i, f, c' (tanh), o

typedef std::vector<float> Vec;

struct CellTape {
  Vec x, h_prev, c_prev, h_tild_prev, gates, c, h;
  std::vector<int> idx0, mask;
  bool feed = false;
};

struct AttnTape {
  Vec tanh1, sigma, p_t, wa, align, cached_exp, ctx, h_tild;
  std::vector<int> indices;
};

}  // namespace

struct orc_trainer {
  orc_model *m = nullptr;
  orc_model_config cfg;
  std::map<std::string, Vec> grads;
  std::vector<int> uniq[2];  // unique vocabulary ids of the minibatch, source / target input side
  // dropout (keep <= 0: off): uniform masks, an element is kept when mask < keep.
  // embed[side]: H x B x steps; out[side]: layers x (H x B x steps), the mask under which the
  // consumer above layer l (next layer, attention node, or softmax) reads that layer's h.
  float keep = 0.f;
  Vec drop_embed[2], drop_out[2];
  // --clip-cell (cell_clip_mode__): c_t clamped to +-cell_clip in the forward pass
  // (src/node_input_to_hidden.h:599-601, src/node_hidden_to_hidden.h:416-418) and the errors a node
  // hands on clamped to +-error_clip (below).  0 = off.
  float cell_clip = 0.f, error_clip = 0.f;
  // train_*_mode__ switches of UpdateParams, see orc_trainer_set_train_modes
  bool train_modes[6] = {true, true, true, true, true, true};
};

namespace {

float *P(orc_trainer *t, const std::string &name) {
  long long n = 0;
  float *p = orc_model_param(t->m, name.c_str(), &n);
  if (!p) {
    fprintf(stderr, "orc_trainer: unknown parameter %s\n", name.c_str());
    exit(EXIT_FAILURE);
  }
  return p;
}

Vec &G(orc_trainer *t, const std::string &name, size_t n) {
  Vec &g = t->grads[name];
  if (g.size() != n) g.assign(n, 0.f);
  return g;
}

// Embedding size: the LSTM size unless the configuration names another (a generalisation, the
// reference has E == H, src/global_configuration.h:220).  Only the first layer of a side reads
// an embedding: its x is E x B and its M_* are H x E.
int emb(const orc_trainer *t) { return t->cfg.E > 0 ? t->cfg.E : t->cfg.H; }
int in_rows(const orc_trainer *t, const std::string &pfx) {
  return pfx == "src.0." || pfx == "tgt.0." ? emb(t) : t->cfg.H;
}

// y = P x for the H x K parameter `name` (col-major): y is H x B, x is K x B; transposed: y is
// K x B, x is H x B.  K = H for every matrix but the first layer's M_*.
void apply(orc_trainer *t, const std::string &name, int transA, const float *x, int B, float beta,
           float *y, int K = 0) {
  const int H = t->cfg.H;
  if (K <= 0) K = H;
  if (transA) {
    orc_gemm(K, B, H, P(t, name), H, 1, x, H, 0, 1.f, beta, y, K);
    return;
  }
  // same arithmetic as orc_gemm, without transposing the matrix again on every call
  const float *rm = orc_model_rowmajor(t->m, name.c_str());
  if (rm) orc_gemm_rowmajor_a(H, B, K, rm, x, K, 1.f, beta, y, H);
  else orc_gemm(H, B, K, P(t, name), H, 0, x, K, 0, 1.f, beta, y, H);
}

// grad(name) += a b^T  (a: H x B, b: K x B)
void outer_acc(orc_trainer *t, const std::string &name, const float *a, const float *b, int B,
               int K = 0) {
  const int H = t->cfg.H;
  if (K <= 0) K = H;
  Vec &g = G(t, name, (size_t)H * K);
  orc_gemm(H, K, B, a, H, 0, b, K, 1, 1.f, 1.f, g.data(), H);
}

// grad(name) += a 1
void rowsum_acc(orc_trainer *t, const std::string &name, const float *a, int rows, int B) {
  Vec &g = G(t, name, rows);
  for (int r = 0; r < rows; ++r) {
    float s = 0.f;
    for (int b = 0; b < B; ++b) s += a[idx2c(r, b, rows)];
    g[r] += s;
  }
}

// Forward of one LSTM node with its tape.
void cell_forward(orc_trainer *t, const std::string &pfx, int B, CellTape &tp) {
  const int H = t->cfg.H;
  Vec p1((size_t)4 * H * B), p2((size_t)4 * H * B), p3, tmp((size_t)H * B), bias((size_t)4 * H);
  if (tp.feed) p3.resize((size_t)4 * H * B);
  for (int g = 0; g < 4; ++g) {
    const std::string gn = kGate[g];
    auto put = [&](Vec &dst) {
      for (int b = 0; b < B; ++b)
        memcpy(&dst[idx2c((size_t)g * H, b, (size_t)4 * H)], &tmp[(size_t)b * H], sizeof(float) * H);
    };
    apply(t, pfx + "M_" + gn, 0, tp.x.data(), B, 0.f, tmp.data(), in_rows(t, pfx));
    put(p1);
    apply(t, pfx + "W_h" + gn, 0, tp.h_prev.data(), B, 0.f, tmp.data());
    put(p2);
    if (tp.feed) {
      apply(t, pfx + "Q_" + gn, 0, tp.h_tild_prev.data(), B, 0.f, tmp.data());
      put(p3);
    }
    memcpy(&bias[(size_t)g * H], P(t, pfx + "b_" + gn), sizeof(float) * H);
  }
  tp.gates.assign((size_t)4 * H * B, 0.f);
  tp.c.assign((size_t)H * B, 0.f);
  tp.h.assign((size_t)H * B, 0.f);
  orc_lstm_cell_fwd(H, B, p1.data(), p2.data(), tp.feed ? p3.data() : nullptr, bias.data(),
                    tp.c_prev.data(), tp.mask.data(), tp.feed ? 1 : 0, t->cell_clip, tp.gates.data(),
                    tp.c.data(), tp.h.data());
}

// Backward of one LSTM node.  dh_above may be NULL (zero).  dh_next / dc_next are the errors handed
// back by node t+1 and are replaced by the ones for node t-1.  dx receives M^T d (H x B, E x B in
// a first layer);
// dh_tild_below (feed input, t > 0) receives Q^T d.
void cell_backward(orc_trainer *t, const std::string &pfx, int B, const CellTape &tp,
                   const float *dh_above, const float *above_drop_mask, Vec &dh_next, Vec &dc_next,
                   Vec &dx, Vec *dh_tild_below) {
  const int H = t->cfg.H;
  const size_t n = (size_t)H * B;
  Vec dg((size_t)4 * n, 0.f), dc_prev(n, 0.f);
  orc_lstm_cell_bwd(H, B, dh_above, dh_next.data(), dc_next.data(), tp.gates.data(), tp.c.data(),
                    tp.c_prev.data(), tp.mask.data(), 0.f, 0.f, above_drop_mask, t->keep, dg.data(),
                    dc_prev.data());
  Vec d[4];  // unstack: the reference keeps one H x B error per gate
  for (int g = 0; g < 4; ++g) {
    d[g].resize(n);
    for (int b = 0; b < B; ++b)
      memcpy(&d[g][(size_t)b * H], &dg[idx2c((size_t)g * H, b, (size_t)4 * H)], sizeof(float) * H);
  }
  Vec dh_prev(n, 0.f);
  const int Kx = in_rows(t, pfx);
  dx.assign((size_t)Kx * B, 0.f);
  for (int g = 0; g < 4; ++g) {
    const std::string gn = kGate[g];
    apply(t, pfx + "W_h" + gn, 1, d[g].data(), B, 1.f, dh_prev.data());
    apply(t, pfx + "M_" + gn, 1, d[g].data(), B, 1.f, dx.data(), Kx);
  }
  if (tp.feed && dh_tild_below) {
    dh_tild_below->assign(n, 0.f);
    for (int g = 0; g < 4; ++g)
      apply(t, pfx + std::string("Q_") + kGate[g], 1, d[g].data(), B, 1.f, dh_tild_below->data());
  }
  // ClipMatKernel on the errors handed on when cell_clip_mode__ is set: d_errn_to_t_ht_m1
  // (src/node_input_to_hidden.h:876-878, src/node_hidden_to_hidden.h:877-879), the error to the
  // layer below of a hidden layer (src/node_hidden_to_hidden.h:774-776, before its dropout; the
  // input layer's error to the embedding is not clamped) and the feed-input error
  // (src/node_input_to_hidden.h:950-952).  The clamp of d_errn_to_t_ct at :974 / :898 comes after
  // that buffer's last use and changes nothing.
  if (t->error_clip > 0.f) {
    const float lim = t->error_clip;
    auto clamp_all = [lim](Vec &v) {
      for (float &x : v) x = x > lim ? lim : (x < -lim ? -lim : x);
    };
    clamp_all(dh_prev);
    if (pfx != "src.0." && pfx != "tgt.0.") clamp_all(dx);
    if (tp.feed && dh_tild_below) clamp_all(*dh_tild_below);
  }
  // ComputeGradientsGpu
  for (int g = 0; g < 4; ++g) {
    const std::string gn = kGate[g];
    outer_acc(t, pfx + "W_h" + gn, d[g].data(), tp.h_prev.data(), B);
    outer_acc(t, pfx + "M_" + gn, d[g].data(), tp.x.data(), B, Kx);
    if (tp.feed) outer_acc(t, pfx + "Q_" + gn, d[g].data(), tp.h_tild_prev.data(), B);
    rowsum_acc(t, pfx + "b_" + gn, d[g].data(), H, B);
  }
  dh_next = dh_prev;
  dc_next = dc_prev;
}

// WSmallGradientKernel: small_grad[:, rev[idx0_b]] += dx[:, b].  Pad columns carry dx = 0.
void scatter_embedding(orc_trainer *t, const std::string &name, int side, const Vec &dx,
                       const CellTape &tp, int B, const float *drop_mask) {
  const int H = emb(t);  // rows of an embedding
  const std::vector<int> &u = t->uniq[side];
  Vec &g = G(t, name, (size_t)H * u.size());
  for (int b = 0; b < B; ++b) {
    if (!tp.mask[b]) continue;
    int k = -1;
    for (size_t j = 0; j < u.size(); ++j)
      if (u[j] == tp.idx0[b]) {
        k = (int)j;
        break;
      }
    if (k < 0) {
      fprintf(stderr, "orc_trainer: id %d missing from the unique list\n", tp.idx0[b]);
      exit(EXIT_FAILURE);
    }
    for (int r = 0; r < H; ++r) {
      float sum = dx[idx2c(r, b, H)];
      // WSmallGradientKernelDropout, deep_rnn_kernel.h:300
      if (drop_mask) sum = sum * (t->keep > drop_mask[idx2c(r, b, H)]) * (1 / t->keep);
      g[idx2c(r, k, H)] += sum;
    }
  }
}

}  // namespace

// ---- kernel-granularity restatements (argument meaning of the lh_* entry points) ------------------

// LstmInputHiddenNode::BackPropGpu up to the four gate errors (src/node_input_to_hidden.h:694-860):
// geam sums, DErrtCTKernel (deep_rnn_kernel.h:152), ZeroColumnsKernel, DErrnToTOTKernel,
// DErrnToTFTITKernel, DErrnToTTanhcptKernel, ElementwiseMultKernel; ClipMatKernel (:876,:951) on
// the errors handed back is applied where they are consumed.
extern "C" void orc_lstm_cell_bwd(int H, int B, const float *dh_above, const float *dh_next,
                                  const float *dc_next, const float *gates, const float *c,
                                  const float *c_prev, const int *mask01, float clip_above,
                                  float clip_next, const float *above_drop_mask, float keep,
                                  float *dgates, float *dc_prev) {
  auto clamp = [](float x, float lim) {
    return lim > 0.f ? (x > lim ? lim : (x < -lim ? -lim : x)) : x;
  };
  for (int b = 0; b < B; ++b)
    for (int r = 0; r < H; ++r) {
      const size_t o = idx2c(r, b, H);
      const float it = gates[idx2c(0 * (size_t)H + r, b, (size_t)4 * H)];
      const float ft = gates[idx2c(1 * (size_t)H + r, b, (size_t)4 * H)];
      const float gt = gates[idx2c(2 * (size_t)H + r, b, (size_t)4 * H)];
      const float ot = gates[idx2c(3 * (size_t)H + r, b, (size_t)4 * H)];
      float above = dh_above ? clamp(dh_above[o], clip_above) : 0.f;
      // DropoutKernel (deep_rnn_kernel.h:1059) on the error handed down by the consumer above
      if (dh_above && above_drop_mask) above = (keep > above_drop_mask[o]) * (1 / keep) * above;
      float dh = (dh_next ? clamp(dh_next[o], clip_next) : 0.f) + above;
      const float tc = tanhf(c[o]);
      float dc = (dc_next ? dc_next[o] : 0.f) + dh * ot * (1.0f - tc * tc);
      dh = dh * mask01[b];
      dc = dc * mask01[b];
      dgates[idx2c(3 * (size_t)H + r, b, (size_t)4 * H)] = dh * tc * ot * (1 - ot);
      dgates[idx2c(1 * (size_t)H + r, b, (size_t)4 * H)] = dc * c_prev[o] * ft * (1 - ft);
      dgates[idx2c(2 * (size_t)H + r, b, (size_t)4 * H)] = dc * it * (1 - gt * gt);
      dgates[idx2c(0 * (size_t)H + r, b, (size_t)4 * H)] = dc * gt * it * (1 - it);
      dc_prev[o] = dc * ft;
    }
}

// Output error of SoftmaxLayer::GetHTGradientGpu / ComputeDGradientGpu (src/layer_loss.h:547-626,
// 887-972) on top of the forward softmax: dz = mask * (onehot - p).
extern "C" void orc_softmax_xent_grad(const float *logits, int ldl, const float *bias, int V, int B,
                                      const int *tgt0, const int *mask01, float *dz, int ldz,
                                      double *logp_tgt, double *loss_accum) {
  Vec p((size_t)V * B);
  orc_softmax_fwd(logits, ldl, bias, V, B, p.data(), V);
  orc_train_loglik(p.data(), V, V, B, tgt0, mask01, loss_accum);
  for (int b = 0; b < B; ++b) {
    if (logp_tgt) logp_tgt[b] = log((double)p[idx2c(tgt0[b], b, V)]);
    for (int v = 0; v < V; ++v) dz[idx2c(v, b, ldz)] = -p[idx2c(v, b, V)] * mask01[b];
    dz[idx2c(tgt0[b], b, ldz)] += (float)mask01[b];
  }
}

// AddTwoMatsKernel + ZeroHT + TanhGradKernel, src/layer_attention.h:490-512.
extern "C" void orc_attn_delta(int H, int B, const float *dht, const float *dht_feed,
                               const float *h_tild, const int *mask01, float clip_feed,
                               float *delta) {
  for (int b = 0; b < B; ++b)
    for (int r = 0; r < H; ++r) {
      const size_t o = idx2c(r, b, H);
      float v = dht[o];
      if (dht_feed) {
        float f = dht_feed[o];
        if (clip_feed > 0.f) f = f > clip_feed ? clip_feed : (f < -clip_feed ? -clip_feed : f);
        v += f;
      }
      v = v * mask01[b];
      delta[o] = v * (1 - h_tild[o] * h_tild[o]);
    }
}

// src/layer_attention.h:572-660 with ErrorAlignmentsKernelLarge, ErrorHSAndCTKernelLarge,
// ErrorPTKernel, AttentionVPErrorKernel, GradWPKernel, GetHTScalingsWaGradKernel, ScaleHTKernel,
// AddTwoMatsKernel and CopyErrorsSource (src/deep_rnn_kernel.h:1348-1520).
extern "C" void orc_attn_core_bwd(int H, int B, int D, int max_len, int hs_steps, const float *dctx,
                                  const float *tanh1, const float *v_p, const float *wa,
                                  const float *hs, long long hs_step_stride,
                                  long long hs_col_stride, const int *batch_info, const float *p_t,
                                  const float *sigma, const int *indices, const float *align,
                                  const float *cached_exp, float *dhs, float *hsum, float *u,
                                  float *w) {
  const int W = D >= 0 ? 2 * D + 1 : max_len;
  const float sigma_sq = (float)((D * D) / 4.0);
  for (int b = 0; b < B; ++b) {
    const int len = batch_info[b], off = batch_info[B + b];
    std::vector<float> das(W, 0.f), r(W, 0.f);
    std::vector<long long> at(W, -1);
    for (int j = 0; j < W; ++j) {
      const int idx = indices[idx2c(b, j, B)];
      if (idx == -1) continue;
      const int tau = len - 1 - idx + off;
      if (tau < 0 || tau >= hs_steps) continue;
      at[j] = (long long)tau * hs_step_stride + (long long)b * hs_col_stride;
      float acc = 0.f;  // ErrorAlignmentsKernelLarge
      for (int k = 0; k < H; ++k) acc += dctx[idx2c(k, b, H)] * hs[at[j] + k];
      das[j] = acc;
    }
    for (int j = 0; j < W; ++j)  // ErrorHSAndCTKernelLarge
      if (at[j] >= 0)
        for (int k = 0; k < H; ++k) dhs[at[j] + k] += dctx[idx2c(k, b, H)] * align[idx2c(b, j, B)];
    if (D >= 0) {
      float dp = 0.f;  // ErrorPTKernel (all slots; invalid ones carry alignment 0)
      for (int j = 0; j < W; ++j)
        dp += das[j] * align[idx2c(b, j, B)] * ((indices[idx2c(b, j, B)] - p_t[b]) / sigma_sq);
      const float sg = sigma[b];
      for (int k = 0; k < H; ++k) {
        const size_t o = idx2c(k, b, H);
        u[o] = dp * sg * (1 - sg) * len * tanh1[o];                               // AttentionVPErrorKernel
        w[o] = dp * len * v_p[k] * sg * (1 - sg) * (1 - tanh1[o] * tanh1[o]);     // GradWPKernel
      }
    }
    for (int j = 0; j < W; ++j) {  // GetHTScalingsWaGradKernel
      const float aj = align[idx2c(b, j, B)], gj = cached_exp[idx2c(j, b, W)];
      float v = das[j] * aj * (1 - aj / gj);
      for (int k = 0; k < W; ++k)
        if (k != j) v += -1 * das[k] * align[idx2c(b, k, B)] * aj / gj;
      r[j] = v;
    }
    for (int k = 0; k < H; ++k) hsum[idx2c(k, b, H)] = 0.f;
    for (int j = 0; j < W; ++j) {
      if (at[j] < 0) continue;  // hs_mat holds zeros there; CopyErrorsSource skips index -1
      for (int k = 0; k < H; ++k) {
        hsum[idx2c(k, b, H)] += hs[at[j] + k] * r[j];   // ScaleHTKernel + AddTwoMatsKernel
        dhs[at[j] + k] += wa[idx2c(k, b, H)] * r[j];    // ScaleHTKernel + CopyErrorsSource
      }
    }
  }
}

extern "C" orc_trainer *orc_trainer_create(orc_model *m, const orc_model_config *cfg) {
  orc_trainer *t = new orc_trainer();
  t->m = m;
  t->cfg = *cfg;
  return t;
}

extern "C" void orc_trainer_destroy(orc_trainer *t) { delete t; }

extern "C" void orc_trainer_set_dropout(orc_trainer *t, float keep, const float *src_embed,
                                        const float *tgt_embed, const float *src_out,
                                        const float *tgt_out, int S, int T, int B) {
  t->keep = keep;
  const size_t n = (size_t)t->cfg.H * B, ne = (size_t)emb(t) * B, L = t->cfg.layers;
  if (!(keep > 0.f)) return;
  t->drop_embed[0].assign(src_embed, src_embed + ne * S);
  t->drop_embed[1].assign(tgt_embed, tgt_embed + ne * T);
  t->drop_out[0].assign(src_out, src_out + n * S * L);
  t->drop_out[1].assign(tgt_out, tgt_out + n * T * L);
}

extern "C" void orc_trainer_set_clip(orc_trainer *t, float cell_clip, float error_clip) {
  t->cell_clip = cell_clip;
  t->error_clip = error_clip;
}

extern "C" float *orc_trainer_grad(orc_trainer *t, const char *name, long long *n_elems) {
  const auto it = t->grads.find(name);
  if (it == t->grads.end()) return nullptr;
  if (n_elems) *n_elems = (long long)it->second.size();
  return it->second.data();
}

extern "C" double orc_compute_gradients(orc_trainer *t, const int *src, int S, const int *tgt_in,
                                        const int *tgt_out, int T, int B, const int *batch_info,
                                        const int *src_unique, int n_src_unique,
                                        const int *tgt_unique, int n_tgt_unique) {
  const orc_model_config &cfg = t->cfg;
  const int H = cfg.H, L = cfg.layers, V = cfg.V_tgt, E = emb(t);
  const size_t n = (size_t)H * B, ne = (size_t)E * B;
  const bool attn = cfg.attention != 0;
  const bool feed_cfg = attn && cfg.feed_input;
  const int D = cfg.attention == 1 ? cfg.D : -1;
  const int W = D >= 0 ? 2 * D + 1 : S;
  t->uniq[0].assign(src_unique, src_unique + n_src_unique);
  t->uniq[1].assign(tgt_unique, tgt_unique + n_tgt_unique);
  for (auto &kv : t->grads) std::fill(kv.second.begin(), kv.second.end(), 0.f);
  G(t, "src.0.W", (size_t)E * n_src_unique);
  G(t, "tgt.0.W", (size_t)E * n_tgt_unique);

  const bool drop = t->keep > 0.f;
  if (drop && (t->drop_embed[0].size() != ne * S || t->drop_embed[1].size() != ne * T ||
               t->drop_out[0].size() != n * S * L || t->drop_out[1].size() != n * T * L)) {
    fprintf(stderr, "orc_trainer: dropout masks do not match this minibatch\n");
    exit(EXIT_FAILURE);
  }
  auto out_mask = [&](int side, int l, int s) -> const float * {
    if (!drop) return nullptr;
    const int steps = side == 0 ? S : T;
    return t->drop_out[side].data() + ((size_t)l * steps + s) * n;
  };
  auto embed_mask = [&](int side, int s) -> const float * {
    return drop ? t->drop_embed[side].data() + (size_t)s * ne : nullptr;
  };
  auto dropped = [&](const Vec &h, const float *mask) {
    Vec r = h;
    if (mask) orc_dropout(r.data(), mask, t->keep, (long long)n);
    return r;
  };

  // ------------------------------------------------------------------------------ forward
  std::vector<std::vector<CellTape>> enc(S, std::vector<CellTape>(L)), dec(T, std::vector<CellTape>(L));
  std::vector<Vec> ha_all(T);  // what the attention node / softmax reads of the top decoder layer
  std::vector<AttnTape> att(T);
  Vec zeros(n, 0.f);
  Vec hs((size_t)S * n);
  for (int s = 0; s < S; ++s)
    for (int l = 0; l < L; ++l) {
      CellTape &tp = enc[s][l];
      tp.idx0.resize(B);
      tp.mask.resize(B);
      orc_preprocess_indices(src + (size_t)s * B, B, tp.idx0.data(), tp.mask.data(), nullptr);
      tp.x.assign(l == 0 ? ne : n, 0.f);
      if (l == 0)
        orc_embed_lookup(P(t, "src.0.W"), E, cfg.V_src, tp.idx0.data(), B, embed_mask(0, s),
                         drop ? t->keep : 1.f, tp.x.data());
      else
        tp.x = dropped(enc[s][l - 1].h, out_mask(0, l - 1, s));
      tp.h_prev = s ? enc[s - 1][l].h : zeros;
      tp.c_prev = s ? enc[s - 1][l].c : zeros;
      cell_forward(t, "src." + std::to_string(l) + ".", B, tp);
      if (l == L - 1) memcpy(&hs[(size_t)s * n], tp.h.data(), sizeof(float) * n);
    }
  double loglik = 0;
  std::vector<Vec> dz(T);           // (onehot - p) * mask, V x B per step
  std::vector<std::vector<int>> tgt_mask(T);
  for (int s = 0; s < T; ++s) {
    for (int l = 0; l < L; ++l) {
      CellTape &tp = dec[s][l];
      tp.idx0.resize(B);
      tp.mask.resize(B);
      orc_preprocess_indices(tgt_in + (size_t)s * B, B, tp.idx0.data(), tp.mask.data(), nullptr);
      tp.x.assign(l == 0 ? ne : n, 0.f);
      if (l == 0)
        orc_embed_lookup(P(t, "tgt.0.W"), E, V, tp.idx0.data(), B, embed_mask(1, s),
                         drop ? t->keep : 1.f, tp.x.data());
      else
        tp.x = dropped(dec[s][l - 1].h, out_mask(1, l - 1, s));
      tp.h_prev = s ? dec[s - 1][l].h : (S ? enc[S - 1][l].h : zeros);
      tp.c_prev = s ? dec[s - 1][l].c : (S ? enc[S - 1][l].c : zeros);
      tp.feed = l == 0 && feed_cfg && s != 0;
      if (tp.feed) tp.h_tild_prev = att[s - 1].h_tild;
      cell_forward(t, "tgt." + std::to_string(l) + ".", B, tp);
    }
    // the attention node (layer_attention.h:253-261) or, without attention, the softmax
    // (layer_loss.h:501-507) works on a dropped copy of the top layer's h
    ha_all[s] = dropped(dec[s][L - 1].h, out_mask(1, L - 1, s));
    const float *top = ha_all[s].data();
    if (attn) {
      AttnTape &a = att[s];
      a.tanh1.assign(n, 0.f);
      a.wa.assign(n, 0.f);
      a.sigma.assign(B, 0.f);
      a.p_t.assign(B, 0.f);
      a.align.assign((size_t)B * W, 0.f);
      a.cached_exp.assign((size_t)B * W, 1.f);
      a.indices.assign((size_t)B * W, -1);
      a.ctx.assign(n, 0.f);
      a.h_tild.assign(n, 0.f);
      if (D >= 0) {
        apply(t, "attn.W_p", 0, top, B, 0.f, a.tanh1.data());
        for (auto &v : a.tanh1) v = tanhf(v);
      }
      apply(t, "attn.W_a", 1, top, B, 0.f, a.wa.data());
      orc_attn_core_fwd(H, B, D, S, S, a.tanh1.data(), P(t, "attn.v_p"), a.wa.data(), hs.data(),
                        (long long)n, H, nullptr, batch_info, dec[s][L - 1].mask.data(),
                        a.p_t.data(), a.sigma.data(), a.indices.data(), a.align.data(),
                        a.cached_exp.data(), a.ctx.data(), nullptr);
      Vec t1(n), t2(n);
      apply(t, "attn.W_c1", 0, a.ctx.data(), B, 0.f, t1.data());
      apply(t, "attn.W_c2", 0, top, B, 0.f, t2.data());
      const float *b_out = P(t, "attn.b_out");
      for (int b = 0; b < B; ++b)
        for (int r = 0; r < H; ++r) {
          const size_t o = idx2c(r, b, H);
          a.h_tild[o] = tanhf(t1[o] + t2[o] + b_out[r]) * dec[s][L - 1].mask[b];
        }
      top = a.h_tild.data();
    }
    // softmax: p, log-likelihood, and the output error (onehot - p) * mask of GetHTGradientGpu
    Vec logits((size_t)V * B);
    orc_gemm_rowmajor_a(V, B, H, orc_model_rowmajor(t->m, "softmax.D"), top, H, 1.f, 0.f,
                        logits.data(), V);
    std::vector<int> t0(B);
    tgt_mask[s].resize(B);
    orc_preprocess_indices(tgt_out + (size_t)s * B, B, t0.data(), tgt_mask[s].data(), nullptr);
    dz[s].assign((size_t)V * B, 0.f);
    orc_softmax_xent_grad(logits.data(), V, P(t, "softmax.b_d"), V, B, t0.data(),
                          tgt_mask[s].data(), dz[s].data(), V, nullptr, &loglik);
  }

  // ------------------------------------------------------------------------------ backward, target
  std::vector<Vec> dh_next(L, Vec(n, 0.f)), dc_next(L, Vec(n, 0.f));
  Vec dHS((size_t)S * n, 0.f);  // error into the top source layer, laid out like hs
  Vec dh_tild_feed;                      // Q^T d from the input layer of step t+1
  bool have_feed = false;
  Vec &gD = G(t, "softmax.D", (size_t)V * H);
  for (int s = T - 1; s >= 0; --s) {
    const float *h_in = attn ? att[s].h_tild.data() : ha_all[s].data();
    Vec dht(n, 0.f);
    orc_gemm(H, B, V, P(t, "softmax.D"), V, 1, dz[s].data(), V, 0, 1.f, 0.f, dht.data(), H);
    orc_gemm(V, H, B, dz[s].data(), V, 0, h_in, H, 1, 1.f, 1.f, gD.data(), V);
    rowsum_acc(t, "softmax.b_d", dz[s].data(), V, B);

    Vec dh_top;  // error into the top decoder layer
    if (attn) {
      const AttnTape &a = att[s];
      const CellTape &topc = dec[s][L - 1];
      const float *ha = ha_all[s].data();
      Vec delta(n, 0.f);
      orc_attn_delta(H, B, dht.data(), (feed_cfg && have_feed) ? dh_tild_feed.data() : nullptr,
                     a.h_tild.data(), topc.mask.data(), 0.f, delta.data());
      outer_acc(t, "attn.W_c1", delta.data(), a.ctx.data(), B);
      outer_acc(t, "attn.W_c2", delta.data(), ha, B);
      rowsum_acc(t, "attn.b_out", delta.data(), H, B);
      Vec dctx(n, 0.f), dha(n, 0.f);
      apply(t, "attn.W_c1", 1, delta.data(), B, 0.f, dctx.data());
      apply(t, "attn.W_c2", 1, delta.data(), B, 0.f, dha.data());
      Vec hsum(n, 0.f), u(n, 0.f), w(n, 0.f);
      orc_attn_core_bwd(H, B, D, S, S, dctx.data(), a.tanh1.data(), D >= 0 ? P(t, "attn.v_p") : nullptr,
                        a.wa.data(), hs.data(), (long long)n, H, batch_info, a.p_t.data(),
                        a.sigma.data(), a.indices.data(), a.align.data(), a.cached_exp.data(),
                        dHS.data(), hsum.data(), u.data(), w.data());
      if (D >= 0) {
        rowsum_acc(t, "attn.v_p", u.data(), H, B);
        outer_acc(t, "attn.W_p", w.data(), ha, B);
        apply(t, "attn.W_p", 1, w.data(), B, 1.f, dha.data());
      }
      outer_acc(t, "attn.W_a", ha, hsum.data(), B);
      apply(t, "attn.W_a", 0, hsum.data(), B, 1.f, dha.data());
      dh_top = dha;
    } else {
      dh_top = dht;
    }

    Vec dx, dh_above = dh_top;
    for (int l = L - 1; l >= 0; --l) {
      Vec feed_out;
      cell_backward(t, "tgt." + std::to_string(l) + ".", B, dec[s][l], dh_above.data(),
                    out_mask(1, l, s), dh_next[l], dc_next[l], dx,
                    dec[s][l].feed ? &feed_out : nullptr);
      if (l == 0) {
        scatter_embedding(t, "tgt.0.W", 1, dx, dec[s][0], B, embed_mask(1, s));
        have_feed = dec[s][0].feed;
        if (have_feed) dh_tild_feed = feed_out;
      } else {
        dh_above = dx;
      }
    }
  }
  // ------------------------------------------------------------------------------ backward, source
  for (int s = S - 1; s >= 0; --s) {
    Vec dx, dh_above = attn ? Vec(dHS.begin() + (size_t)s * n, dHS.begin() + (size_t)(s + 1) * n) : zeros;
    for (int l = L - 1; l >= 0; --l) {
      // the top source layer is read undropped by the attention nodes
      cell_backward(t, "src." + std::to_string(l) + ".", B, enc[s][l], dh_above.data(),
                    l == L - 1 ? nullptr : out_mask(0, l, s), dh_next[l], dc_next[l], dx, nullptr);
      if (l == 0)
        scatter_embedding(t, "src.0.W", 0, dx, enc[s][0], B, embed_mask(0, s));
      else
        dh_above = dx;
    }
  }
  return loglik;
}

// NeuralMachineTranslation::UpdateWeights.  Every gradient is first divided by the minibatch size
// (ScaleGradients); then
//   clip_mode 2 (global, --whole-clip-gradients): norm over every gradient EXCEPT the two embedding
//     small gradients (they are absent from CalculateGlobalNorm, layer_input_to_hidden.h:1062-1098),
//     and if it exceeds the threshold every gradient INCLUDING those two is rescaled
//     (UpdateGlobalParams, :1102-1141);
//   clip_mode 1 (per matrix, NormClipGpuV2): each named matrix is rescaled to the threshold alone;
//   clip_mode 3 (individual): every element clamped to +-individual_clip;
//   clip_mode 0: nothing.
// Then theta += learning_rate * g (embeddings: only the columns of the unique ids) and the gradients
// are cleared.  Returns the global norm (clip_mode 2) or 0.
// The train_*_mode__ switches read by UpdateParams (src/layer_input_to_hidden.h:1154,1257,1263,
// src/layer_hidden_to_hidden.h:765,831, src/layer_loss.h:1144): modes[0..5] = source input
// embedding, target input embedding, target output embedding (D, b_d), source LSTM matrices,
// target LSTM matrices, attention.  The norms above them are taken over every gradient all the same
// (CalculateGlobalNorm has no such switch).
extern "C" void orc_trainer_set_train_modes(orc_trainer *t, const int *modes) {
  for (int i = 0; i < 6; ++i) t->train_modes[i] = modes[i] != 0;
}
static bool frozen(const orc_trainer *t, const std::string &name) {
  if (name == "src.0.W") return !t->train_modes[0];
  if (name == "tgt.0.W") return !t->train_modes[1];
  if (name.compare(0, 8, "softmax.") == 0) return !t->train_modes[2];
  if (name.compare(0, 4, "src.") == 0) return !t->train_modes[3];
  if (name.compare(0, 4, "tgt.") == 0) return !t->train_modes[4];
  if (name.compare(0, 5, "attn.") == 0) return !t->train_modes[5];
  return false;
}

extern "C" float orc_update_weights(orc_trainer *t, float learning_rate, int clip_mode,
                                    float norm_clip, float individual_clip, int minibatch_size) {
  const int H = emb(t);  // only the embedding columns are addressed by row below
  for (auto &kv : t->grads)
    for (auto &v : kv.second) v = (1.0f / minibatch_size) * v;
  float global = 0.f;
  // BasicComputeNormP1 <<<256, 256>>> + BasicComputeNormP2 (src/deep_rnn_kernel.h:616-676): thread
  // (block, tid) sums the squares of elements block*256 + tid, + 65536, ... in fp32; every block
  // folds its 256 sums with the shared-memory tree (strides 128, 64, then WarpReduceSum's 32 ... 1,
  // src/deep_rnn_kernel.h:313-320), and one more such tree folds the 256 block results.
  auto tree256 = [](std::vector<float> &buf) {
    for (int stride = 128; stride > 32; stride >>= 1)
      for (int tid = 0; tid < stride; ++tid) buf[tid] += buf[stride + tid];
    // WarpReduceSum runs on 32 lanes in lockstep: every lane adds the value the lane 32, 16, ...
    // above it held BEFORE this step (lanes >= the step width read stale sums that never reach
    // lane 0; the buffer is padded so that those reads stay in range)
    for (int off = 32; off >= 1; off >>= 1) {
      float next[32];
      for (int tid = 0; tid < 32; ++tid) next[tid] = buf[tid] + buf[tid + off];
      for (int tid = 0; tid < 32; ++tid) buf[tid] = next[tid];
    }
    return buf[0];
  };
  auto sumsq = [&](const Vec &g) {
    constexpr int NT = 256;
    std::vector<float> part((size_t)NT * NT, 0.f);
    const size_t n = g.size();
#pragma omp parallel for schedule(static)
    for (int t = 0; t < NT * NT; ++t) {
      float acc = 0.f;
      for (size_t i = (size_t)t; i < n; i += (size_t)NT * NT) acc += g[i] * g[i];
      part[t] = acc;
    }
    std::vector<float> blocks(NT + 64, 0.f), buf(NT + 64, 0.f);
    for (int b = 0; b < NT; ++b) {
      std::fill(buf.begin(), buf.end(), 0.f);
      std::copy(part.begin() + (size_t)b * NT, part.begin() + (size_t)(b + 1) * NT, buf.begin());
      blocks[b] = tree256(buf);
    }
    return tree256(blocks);
  };
  if (clip_mode == 2) {
    for (auto &kv : t->grads)
      if (kv.first != "src.0.W" && kv.first != "tgt.0.W") global += sumsq(kv.second);
    global = std::sqrt(global);
    if (global > norm_clip)
      for (auto &kv : t->grads)
        for (auto &v : kv.second) v = (norm_clip / global) * v;
  } else if (clip_mode == 1) {
    for (auto &kv : t->grads) {
      const float nrm = std::sqrt(sumsq(kv.second));
      if (nrm > norm_clip)
        for (auto &v : kv.second) v = (norm_clip / nrm) * v;
    }
  } else if (clip_mode == 3) {
    for (auto &kv : t->grads)
      for (auto &v : kv.second)
        v = v > individual_clip ? individual_clip : (v < -individual_clip ? -individual_clip : v);
  }
  for (auto &kv : t->grads) {
    long long n = 0;
    float *p = orc_model_param(t->m, kv.first.c_str(), &n);
    if (!p) continue;
    if (frozen(t, kv.first)) {  // UpdateParams skips the group; ClearGradients still runs
      std::fill(kv.second.begin(), kv.second.end(), 0.f);
      continue;
    }
    if (kv.first == "src.0.W" || kv.first == "tgt.0.W") {
      const std::vector<int> &u = t->uniq[kv.first == "src.0.W" ? 0 : 1];
      for (size_t k = 0; k < u.size(); ++k)  // UpdateSparseGradient
        for (int r = 0; r < H; ++r)
          p[idx2c(r, u[k], H)] += learning_rate * kv.second[idx2c(r, k, H)];
    } else {
      for (long long i = 0; i < n; ++i) p[i] += learning_rate * kv.second[i];
    }
    std::fill(kv.second.begin(), kv.second.end(), 0.f);
  }
  orc_model_commit(t->m);
  return global;
}
