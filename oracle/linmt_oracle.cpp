// CPU oracle for the LiNMT LSTM / attention / softmax / beam path.  TEST INFRASTRUCTURE ONLY:
// loaded by tests/, by the smoke check and by the benchmark's cpu_baseline leg, never by the
// product path.  Every function restates the reference source it cites (paths relative to the
// reference checkout).  The reference itself cannot be built here (CUDA + cuBLAS + cuRAND + Boost),
// and ships no tests or golden vectors, so each function is additionally pinned by an independent
// check in tests/test_oracle_*.py, named in its comment ("pin:").
//
// Functions whose behaviour is fixed only by our reading of the source ("parity unpinned"):
//   - the order in which std::priority_queue pops exactly equal scores in orc_beam_expand (the
//     reference's result depends on libstdc++'s heap there; fixtures avoid exact ties);
//   - the empty-heap pop at step 0 when <START> and <EOF> are both among the beam+1 candidates
//     (undefined behaviour in the reference; this restatement stops popping instead).
#include "linmt_oracle.h"

#include <immintrin.h>

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <queue>
#include <string>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

inline size_t idx2c(size_t i, size_t j, size_t ld) { return j * ld + i; }  // src/utility_cu.h:37

// Dot products with 8 independent fp32 partial sums (vectorisable, deterministic).
inline float dot8(const float *a, const float *b, int n) {
  __m256 acc = _mm256_setzero_ps();
  int k = 0;
  for (; k + 8 <= n; k += 8)
    acc = _mm256_fmadd_ps(_mm256_loadu_ps(a + k), _mm256_loadu_ps(b + k), acc);
  float q[8];
  _mm256_storeu_ps(q, acc);
  float tail = 0.f;
  for (; k < n; ++k) tail = std::fma(a[k], b[k], tail);
  return ((q[0] + q[4]) + (q[1] + q[5])) + ((q[2] + q[6]) + (q[3] + q[7])) + tail;
}

// C (col-major M x N) = alpha * At (row-major M x K, row stride lda) * X (col-major K x N) + beta*C.
// Every element is one dot product with the summation order of dot8; the two loop nests below
// differ only in which elements a thread visits in which order.
void gemm_rowA(int M, int N, int K, const float *At, int lda, const float *X, int ldx, float alpha,
               float beta, float *C, int ldc) {
  if (K <= 64 && N >= 64) {
    // Short dot products into a large C (weight gradients d x^T over a small minibatch): walk C
    // column by column so that the read-modify-write of C is contiguous.
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
      const float *x = X + (size_t)n * ldx;
      float *c = C + (size_t)n * ldc;
      for (int m = 0; m < M; ++m) {
        const float d = dot8(At + (size_t)m * lda, x, K);
        c[m] = beta == 0.f ? alpha * d : alpha * d + beta * c[m];
      }
    }
    return;
  }
  // Register tile of 4 rows x 4 columns: each element keeps the 8 lane sums of dot8 in one
  // vector register, so a loaded piece of a row serves 4 columns and a piece of a column 4 rows.
  const int Mb = (M + 3) / 4;
#pragma omp parallel for schedule(static)
  for (int mb = 0; mb < Mb; ++mb) {
    const int m0 = mb * 4, mr = std::min(4, M - m0);
    const float *a[4];
    for (int i = 0; i < 4; ++i) a[i] = At + (size_t)(m0 + (i < mr ? i : 0)) * lda;
    for (int n0 = 0; n0 < N; n0 += 4) {
      const int nr = std::min(4, N - n0);
      const float *x[4];
      for (int j = 0; j < 4; ++j) x[j] = X + (size_t)(n0 + (j < nr ? j : 0)) * ldx;
      __m256 acc[4][4];
      for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j) acc[i][j] = _mm256_setzero_ps();
      int k = 0;
      for (; k + 8 <= K; k += 8) {
        const __m256 x0 = _mm256_loadu_ps(x[0] + k), x1 = _mm256_loadu_ps(x[1] + k),
                     x2 = _mm256_loadu_ps(x[2] + k), x3 = _mm256_loadu_ps(x[3] + k);
        for (int i = 0; i < 4; ++i) {
          const __m256 av = _mm256_loadu_ps(a[i] + k);
          acc[i][0] = _mm256_fmadd_ps(av, x0, acc[i][0]);
          acc[i][1] = _mm256_fmadd_ps(av, x1, acc[i][1]);
          acc[i][2] = _mm256_fmadd_ps(av, x2, acc[i][2]);
          acc[i][3] = _mm256_fmadd_ps(av, x3, acc[i][3]);
        }
      }
      for (int i = 0; i < mr; ++i)
        for (int j = 0; j < nr; ++j) {
          float q[8];
          _mm256_storeu_ps(q, acc[i][j]);
          float tail = 0.f;
          for (int kk = k; kk < K; ++kk) tail = std::fma(a[i][kk], x[j][kk], tail);
          const float d = ((q[0] + q[4]) + (q[1] + q[5])) + ((q[2] + q[6]) + (q[3] + q[7])) + tail;
          float *c = C + idx2c(m0 + i, n0 + j, ldc);
          *c = beta == 0.f ? alpha * d : alpha * d + beta * *c;
        }
    }
  }
}

void transpose_to(const float *src, int rows, int cols, int ld, float *dst) {
  // src col-major rows x cols (ld) -> dst row-major rows x cols (i.e. col-major cols x rows),
  // in 32 x 32 blocks so that both sides stay in cache
  constexpr int T = 32;
  const int bi = (rows + T - 1) / T, bj = (cols + T - 1) / T;
#pragma omp parallel for schedule(static) if ((size_t)rows * cols > 65536)
  for (int blk = 0; blk < bi * bj; ++blk) {
    const int i0 = (blk / bj) * T, j0 = (blk % bj) * T;
    const int i1 = std::min(rows, i0 + T), j1 = std::min(cols, j0 + T);
    for (int i = i0; i < i1; ++i)
      for (int j = j0; j < j1; ++j) dst[(size_t)i * cols + j] = src[idx2c(i, j, ld)];
  }
}

inline float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-1.0f * x)); }          // deep_rnn_kernel.cu:83
inline float sigmoid_f64(float x) { return (float)(1.0 / (1.0 + exp(-1.0 * (double)x))); }  // deep_rnn_kernel.h:69

}  // namespace

// ------------------------------------------------------------------------------------------------
// src/deep_rnn_kernel.cu:49-70 (VocabTo01Kernel, VocabToNonMinus1Kernel), deep_rnn_kernel.h:144-155.
// pin: exact integer semantics, brute-forced in tests/test_oracle_pins.py.
extern "C" void orc_preprocess_indices(const int *idx, int n, int *idx0, int *mask01,
                                       float *mask01_f) {
  for (int i = 0; i < n; ++i) {
    const int v = idx[i];
    if (-1 == v) {
      idx0[i] = 0;
      mask01[i] = 0;
      if (mask01_f) mask01_f[i] = 0;
    } else {
      idx0[i] = v;
      mask01[i] = 1;
      if (mask01_f) mask01_f[i] = 1;
    }
  }
}

// src/deep_rnn_kernel.cu:348-352.
extern "C" void orc_setup_reverse_indices(const int *unique, int n_unique, int *rev) {
  for (int i = 0; i < n_unique; ++i) rev[unique[i]] = i;
}

// src/deep_rnn_kernel.h:249-255 (SparseLookupKernel) + :1059-1063 (DropoutKernel).
// pin: numpy fancy indexing W[:, idx] and the closed form of inverted dropout.
extern "C" void orc_embed_lookup(const float *W, int E, int V, const int *idx0, int B,
                                 const float *drop_mask, float keep, float *out) {
  (void)V;
  for (int b = 0; b < B; ++b)
    for (int i = 0; i < E; ++i) out[idx2c(i, b, E)] = W[idx2c(i, idx0[b], E)];
  if (drop_mask) orc_dropout(out, drop_mask, keep, (long long)E * B);
}

// src/deep_rnn_kernel.h:1059-1063: final = (mask < rate) * (1/rate) * final.
extern "C" void orc_dropout(float *x, const float *mask, float keep, long long n) {
  for (long long i = 0; i < n; ++i) x[i] = (mask[i] < keep) * (1 / keep) * x[i];
}

// cuBLAS SGEMM as used through CublasGemmWrapper (src/utility_cu.h:153-169); the summation order
// inside cuBLAS is not specified, fp32 accumulation is.  pin: numpy float64 matmul within fp32 bounds.
extern "C" void orc_gemm(int M, int N, int K, const float *A, int lda, int transA, const float *X,
                         int ldx, int transX, float alpha, float beta, float *C, int ldc) {
  std::vector<float> at, xn;
  const float *At = A;
  int ldat = lda;
  if (!transA) {  // A col-major M x K -> row-major copy
    at.resize((size_t)M * K);
    transpose_to(A, M, K, lda, at.data());
    At = at.data();
    ldat = K;
  }
  const float *Xn = X;
  int ldxn = ldx;
  if (transX) {  // X stored N x K col-major -> K x N col-major copy
    xn.resize((size_t)K * N);
    for (int n = 0; n < N; ++n)
      for (int k = 0; k < K; ++k) xn[idx2c(k, n, K)] = X[idx2c(n, k, ldx)];
    Xn = xn.data();
    ldxn = K;
  }
  gemm_rowA(M, N, K, At, ldat, Xn, ldxn, alpha, beta, C, ldc);
}

// LSTM cell forward.  Kernel order of src/node_input_to_hidden.h:350-621 (and the hidden-to-hidden
// twin src/node_hidden_to_hidden.h:270-430): ForwardSigmoidKernel(.cu:78) / ...Feed(.h:64) for i,f,o;
// ForwardTanhKernel(.cu:100) / ...Feed(.h:80); ForwardCTKernel(.h:93); ClipMatKernel(.h:1528);
// ForwardHTKernel(.cu:121); ZeroCTAndHT(.h:123).
// pin: torch.nn.functional LSTM-cell math in float64 with re-packed weights; mask01 = 0 => h = c = 0.
extern "C" void orc_lstm_cell_fwd(int H, int B, const float *pre1, const float *pre2,
                                  const float *pre3, const float *bias4h, const float *c_prev,
                                  const int *mask01, int feed, float cell_clip, float *gates,
                                  float *c, float *h) {
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    for (int r = 0; r < H; ++r) {
      float s[4];
      for (int g = 0; g < 4; ++g) {
        const size_t o = idx2c((size_t)g * H + r, b, (size_t)4 * H);
        float v = pre1[o];
        if (pre2) v = v + pre2[o];
        if (pre3) v = v + pre3[o];
        s[g] = v + bias4h[(size_t)g * H + r];
      }
      const float it = feed ? sigmoid_f64(s[0]) : sigmoid_f32(s[0]);
      const float ft = feed ? sigmoid_f64(s[1]) : sigmoid_f32(s[1]);
      const float gt = tanhf(s[2]);
      const float ot = feed ? sigmoid_f64(s[3]) : sigmoid_f32(s[3]);
      float ct = ft * c_prev[idx2c(r, b, H)] + it * gt;
      if (cell_clip > 0.f) ct = ct > cell_clip ? cell_clip : (ct < -cell_clip ? -cell_clip : ct);
      float ht = ot * tanhf(ct);
      ht = ht * mask01[b];
      ct = ct * mask01[b];
      if (gates) {
        gates[idx2c(0 * (size_t)H + r, b, (size_t)4 * H)] = it;
        gates[idx2c(1 * (size_t)H + r, b, (size_t)4 * H)] = ft;
        gates[idx2c(2 * (size_t)H + r, b, (size_t)4 * H)] = gt;
        gates[idx2c(3 * (size_t)H + r, b, (size_t)4 * H)] = ot;
      }
      c[idx2c(r, b, H)] = ct;
      h[idx2c(r, b, H)] = ht;
    }
  }
}

// Attention core, src/layer_attention.h:282-392 with SigmoidKernel (deep_rnn_kernel.h:1076),
// AlignmentPosKernel (:1086), LowerUpperKernel (:1095), CreateIndicesKernel (.cu:294),
// LoadInHSKernel (:1142), ElemReduceKernelLarge (:1309), AlignmentReductionKernel (:1198),
// GetViterbiAlignmentKernel (:1105), CreateCTKernel (:1251).  D < 0 = global-general variant
// (not in the reference; textbook Luong global attention with the "general" score).
// pin: window bounds brute-forced against their definition; sum_j a_j/g_j = 1 over valid slots;
// with the Gaussian forced to 1 equals a float64 softmax attention; global variant vs float64 softmax.
extern "C" void orc_attn_core_fwd(int H, int B, int D, int max_len, int hs_steps,
                                  const float *tanh1, const float *v_p, const float *wa,
                                  const float *hs, long long hs_step_stride,
                                  long long hs_col_stride, const int *hs_col,
                                  const int *batch_info, const int *mask01, float *p_t,
                                  float *sigma, int *indices, float *align, float *cached_exp,
                                  float *ctx, int *viterbi) {
  const int W = D >= 0 ? 2 * D + 1 : max_len;
  const float sigma_sq = (float)((D * D) / 4.0);  // layer_attention.h:226
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    const int len = batch_info[b], off = batch_info[B + b];
    const int col = hs_col ? hs_col[b] : b;
    float p = 0.f;
    int lo = 0, hi = len - 1;
    if (D >= 0) {
      const float dot = dot8(v_p, tanh1 + (size_t)b * H, H);
      const float sig = (float)(1.0 / (1.0 + exp(-1.0 * (double)dot)));
      p = len * sig;
      lo = (0 > (int)p - D) ? 0 : ((int)p - D);
      hi = ((len - 1) < (int)p + D) ? (len - 1) : ((int)p + D);
      p_t[b] = p;
      sigma[b] = sig;
    }
    std::vector<const float *> hsp(W, nullptr);
    std::vector<float> sc(W, 0.f);
    int cur = lo;
    for (int j = 0; j < W; ++j) {
      int idx = -1;
      if (1 == mask01[b] && cur <= hi) idx = cur;
      ++cur;
      indices[idx2c(b, j, B)] = idx;
      if (idx != -1) {
        const int tau = len - 1 - idx + off;
        if (tau >= 0 && tau < hs_steps)
          hsp[j] = hs + (size_t)tau * hs_step_stride + (size_t)col * hs_col_stride;
      }
      sc[j] = hsp[j] ? dot8(hsp[j], wa + (size_t)b * H, H) : 0.f;
    }
    float mx = D >= 0 ? 0.f : -FLT_MAX;  // deep_rnn_kernel.h:1203 initialises the max to 0
    for (int j = 0; j < W; ++j)
      if (indices[idx2c(b, j, B)] != -1 && sc[j] > mx) mx = sc[j];
    float sum = 0.f;
    std::vector<float> al(W, 0.f);
    for (int j = 0; j < W; ++j)
      if (indices[idx2c(b, j, B)] != -1) {
        al[j] = expf(sc[j] - mx);
        sum += al[j];
      }
    for (int j = 0; j < W; ++j) {
      const int idx = indices[idx2c(b, j, B)];
      float g = 1.f;
      if (idx != -1) {
        if (D >= 0) g = expf((-1 * powf(p - idx, 2.0f)) / (2 * sigma_sq));
        if (0 != sum) al[j] = (al[j] / sum) * g;
      } else {
        al[j] = 0.f;
      }
      align[idx2c(b, j, B)] = al[j];
      cached_exp[idx2c(j, b, W)] = g;
    }
    if (viterbi) {
      float best = -1.f;
      int best_idx = -1;
      for (int j = 0; j < W; ++j)
        if (best < al[j]) {
          best = al[j];
          best_idx = indices[idx2c(b, j, B)];
        }
      viterbi[b] = best_idx;
    }
    for (int r = 0; r < H; ++r) {
      float acc = 0.f;
      for (int j = 0; j < W; ++j) acc += al[j] * (hsp[j] ? hsp[j][r] : 0.f);
      ctx[idx2c(r, b, H)] = acc;
    }
  }
}

// Whole node: src/layer_attention.h:243-483 without dropout (ha = h_t).
extern "C" void orc_attn_node_fwd(int H, int B, int D, int max_len, int hs_steps, const float *h_t,
                                  const float *W_a, const float *W_p, const float *v_p,
                                  const float *b_out, const float *W_c1, const float *W_c2,
                                  const float *hs, long long hs_step_stride,
                                  long long hs_col_stride, const int *hs_col,
                                  const int *batch_info, const int *mask01, float *h_tild,
                                  float *p_t, int *indices, float *align, float *ctx) {
  const int W = D >= 0 ? 2 * D + 1 : max_len;
  std::vector<float> tanh1((size_t)H * B, 0.f), wa((size_t)H * B), sig(B), pt(B), al((size_t)B * W),
      ce((size_t)B * W), cx((size_t)H * B), t1((size_t)H * B), t2((size_t)H * B);
  std::vector<int> ind((size_t)B * W);
  if (D >= 0) {
    orc_gemm(H, B, H, W_p, H, 0, h_t, H, 0, 1.f, 0.f, tanh1.data(), H);
    for (auto &v : tanh1) v = tanhf(v);
  }
  orc_gemm(H, B, H, W_a, H, 1, h_t, H, 0, 1.f, 0.f, wa.data(), H);
  orc_attn_core_fwd(H, B, D, max_len, hs_steps, tanh1.data(), v_p, wa.data(), hs, hs_step_stride,
                    hs_col_stride, hs_col, batch_info, mask01, pt.data(), sig.data(), ind.data(),
                    al.data(), ce.data(), cx.data(), nullptr);
  orc_gemm(H, B, H, W_c1, H, 0, cx.data(), H, 0, 1.f, 0.f, t1.data(), H);
  orc_gemm(H, B, H, W_c2, H, 0, h_t, H, 0, 1.f, 0.f, t2.data(), H);
  for (int b = 0; b < B; ++b)
    for (int r = 0; r < H; ++r) {
      const size_t o = idx2c(r, b, H);
      float v = tanhf(t1[o] + t2[o] + b_out[r]);  // deep_rnn_kernel.h:1284
      v *= mask01[b];                             // ZeroHT, deep_rnn_kernel.h:1293
      h_tild[o] = v;
    }
  if (p_t && D >= 0) memcpy(p_t, pt.data(), sizeof(float) * B);
  if (indices) memcpy(indices, ind.data(), sizeof(int) * ind.size());
  if (align) memcpy(align, al.data(), sizeof(float) * al.size());
  if (ctx) memcpy(ctx, cx.data(), sizeof(float) * cx.size());
}

// MatrixBiasKernel (deep_rnn_kernel.h:525) + OutputdistOverflowPreventionKernel (:353-429): the
// 256-thread strided partial max / sums and the LDS tree are followed literally.
// pin: scipy.special.softmax in float64; columns sum to 1; shift invariance.
extern "C" void orc_softmax_fwd(const float *logits, int ldl, const float *bias, int V, int B,
                                float *p, int ldp) {
  const int T = 256;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    const float *in = logits + (size_t)b * ldl;
    float *out = p + (size_t)b * ldp;
    std::vector<float> z(V);
    for (int i = 0; i < V; ++i) z[i] = bias ? in[i] + bias[i] : in[i];
    float buf[256];
    for (int t = 0; t < T; ++t) {
      buf[t] = -FLT_MAX;
      for (int i = t; i < V; i += T)
        if (buf[t] < z[i]) buf[t] = z[i];
    }
    for (int stride = T / 2; stride > 0; stride >>= 1)
      for (int t = 0; t < stride; ++t) buf[t] = (buf[t] > buf[stride + t]) ? buf[t] : buf[stride + t];
    const float max_k = buf[0];
    for (int t = 0; t < T; ++t) {
      buf[t] = 0;
      for (int i = t; i < V; i += T) {
        const float e = expf(z[i] - max_k);
        buf[t] += e;
        out[i] = e;
      }
    }
    for (int stride = T / 2; stride > 0; stride >>= 1)
      for (int t = 0; t < stride; ++t) buf[t] += buf[stride + t];
    const float sum_k = buf[0];
    for (int i = 0; i < V; ++i) out[i] = out[i] / sum_k;
  }
}

// TrainPerplexityKernel, deep_rnn_kernel.h:336-342.
extern "C" void orc_train_loglik(const float *p, int ldp, int V, int B, const int *tgt0,
                                 const int *mask01, double *accum) {
  (void)V;
  for (int i = 0; i < B; ++i)
    if (1 == mask01[i]) accum[0] += log((double)p[idx2c(tgt0[i], i, ldp)]);
}

// OutputdistPerplexityKernel (deep_rnn_kernel.h:433-519) + the host loop of
// SoftmaxLayer::ComputeLossGpu (src/layer_loss.h:693-701).
// pin: scipy.special.log_softmax in float64 gathered at the target rows.
extern "C" void orc_logsoftmax_xent(const float *logits, int ldl, const float *bias, int V, int B,
                                    const int *tgt0, const int *mask01, double *logp_tgt,
                                    double *loss_accum) {
  const int T = 256;
  double loss = 0;
  for (int b = 0; b < B; ++b) {
    const float *in = logits + (size_t)b * ldl;
    std::vector<float> z(V);
    for (int i = 0; i < V; ++i) z[i] = bias ? in[i] + bias[i] : in[i];
    double buf[256];
    for (int t = 0; t < T; ++t) {
      buf[t] = -DBL_MAX;
      for (int i = t; i < V; i += T)
        if (buf[t] < (double)z[i]) buf[t] = z[i];
    }
    for (int stride = T / 2; stride > 0; stride >>= 1)
      for (int t = 0; t < stride; ++t) buf[t] = (buf[t] > buf[stride + t]) ? buf[t] : buf[stride + t];
    const double max_k = buf[0];
    for (int t = 0; t < T; ++t) {
      buf[t] = 0;
      for (int i = t; i < V; i += T) buf[t] += exp(z[i] - max_k);
    }
    for (int stride = T / 2; stride > 0; stride >>= 1)
      for (int t = 0; t < stride; ++t) buf[t] += buf[stride + t];
    const double sum_k = buf[0];
    const double lp = log(exp(z[tgt0[b]] - max_k)) - log(sum_k);
    if (logp_tgt) logp_tgt[b] = lp;
    if (1 == mask01[b]) loss += lp;
  }
  loss_accum[0] += loss;
}

// ------------------------------------------------------------------------------------------------
// Beam step: EnsembleFactory::EnsemblesModels (src/decoder.h:1910-1931, one model) followed by
// Decoder::ExpandHypothesis (src/decoder.h:355-480); same priority queues, same comparators.
// pin: brute-force full sort on tiny vocabularies (tests/test_oracle_pins.py); <START> never
// emitted; <EOF> never occupies a slot.
namespace {
struct DecObj {
  float val;
  int vocab;
};
struct DecCmp {
  bool operator()(const DecObj &a, const DecObj &b) const { return a.val < b.val; }
};
struct GlobObj {
  float val;
  int beam, vocab;
};
struct GlobCmp {
  bool operator()(const GlobObj &a, const GlobObj &b) const { return a.val < b.val; }
};

// p[k] (V x cols, col-major, one per model) -> averaged, renormalised row-major copy, as
// CopyDistToEigen + EnsemblesModels (src/decoder.h:1910-1931) do.
void renormalise(const float *const *p, int num_models, int V, int cols, std::vector<float> &out) {
  out.resize((size_t)V * cols);
  std::vector<float> norm(cols, 0.f);
  for (int i = 0; i < V; ++i)
    for (int j = 0; j < cols; ++j) {
      double tmp_sum = 0;
      for (int k = 0; k < num_models; ++k) tmp_sum += p[k][idx2c(i, j, V)];
      out[(size_t)i * cols + j] = (float)(tmp_sum / num_models);
    }
  for (int i = 0; i < V; ++i)
    for (int j = 0; j < cols; ++j) norm[j] += out[(size_t)i * cols + j];
  for (int i = 0; i < V; ++i)
    for (int j = 0; j < cols; ++j) out[(size_t)i * cols + j] = out[(size_t)i * cols + j] / norm[j];
}
}  // namespace

extern "C" void orc_beam_expand(const float *p, int V, int beam, int step, const float *prev_score,
                                float diversity, float penalty, int start_id, int eof_id, int *tok,
                                int *backptr, float *score, int *fin_count, int *fin_beam,
                                float *fin_score) {
  orc_beam_expand_ensemble(&p, 1, V, beam, step, prev_score, diversity, penalty, start_id, eof_id,
                           tok, backptr, score, fin_count, fin_beam, fin_score);
}

extern "C" void orc_beam_expand_ensemble(const float *const *p, int num_models, int V, int beam,
                                         int step, const float *prev_score, float diversity,
                                         float penalty, int start_id, int eof_id, int *tok,
                                         int *backptr, float *score, int *fin_count, int *fin_beam,
                                         float *fin_score) {
  std::vector<float> dist;
  renormalise(p, num_models, V, beam, dist);
  int cols = beam;
  if (step == 0) cols = 1;
  std::priority_queue<DecObj, std::vector<DecObj>, DecCmp> pq;
  std::priority_queue<GlobObj, std::vector<GlobObj>, GlobCmp> pq_global;
  for (int i = 0; i < cols; ++i) {
    while (!pq.empty()) pq.pop();
    for (int j = 0; j < V; ++j) {
      const float v = dist[(size_t)j * beam + i];
      if ((int)pq.size() < beam + 1) {
        pq.push(DecObj{-v, j});
      } else if (-v < pq.top().val) {
        pq.pop();
        pq.push(DecObj{-v, j});
      }
    }
    while (!pq.empty()) {
      const int rank = (int)pq.size();
      const float rank_penalty = (float)rank * diversity;
      const DecObj tmp = pq.top();
      pq.pop();
      const float s = std::log(-tmp.val) + prev_score[i] - rank_penalty;
      pq_global.push(GlobObj{s, i, tmp.vocab});
    }
  }
  int i = 0, nfin = 0;
  while (i < beam && !pq_global.empty()) {  // the reference has no emptiness test (UB when drained)
    const GlobObj tmp = pq_global.top();
    pq_global.pop();
    if (tmp.vocab != start_id) {
      if (tmp.vocab == eof_id) {
        fin_beam[nfin] = tmp.beam;
        fin_score[nfin] = tmp.val + penalty;
        ++nfin;
      } else {
        tok[i] = tmp.vocab;
        backptr[i] = tmp.beam;
        score[i] = tmp.val + penalty;
        ++i;
      }
    }
  }
  for (; i < beam; ++i) {
    tok[i] = eof_id;
    backptr[i] = 0;
    score[i] = -FLT_MAX;
  }
  *fin_count = nfin;
}

// How close the decisions of one orc_beam_expand_ensemble call were, on the fp32 numbers it
// compared: the smallest gap, in log-probability, between
//   - the last kept (rank beam+1) and the first dropped probability of a live column, and
//   - two neighbours of the score-ordered candidate list, from its head down to the first
//     candidate that no longer found a slot (<START> drops and <EOF> finishes included).
// A step whose margin is 0 holds an exact fp32 tie; one whose margin is below the rounding
// difference between two summation orders can come out differently on another fp32
// implementation of the same mathematics.  Not part of the reference: test infrastructure that
// tells a near-tie from a real difference.  pin: brute force by full sort (this is one).
extern "C" float orc_beam_step_margin(const float *const *p, int num_models, int V, int beam,
                                      int step, const float *prev_score, float diversity,
                                      int start_id, int eof_id) {
  std::vector<float> dist;
  renormalise(p, num_models, V, beam, dist);
  const int cols = step == 0 ? 1 : beam;
  const int K = beam + 1;
  float margin = FLT_MAX;
  std::vector<GlobObj> cands;
  std::vector<std::pair<float, int>> col(V);
  for (int i = 0; i < cols; ++i) {
    for (int j = 0; j < V; ++j) col[j] = {dist[(size_t)j * beam + i], j};
    const int keep = std::min(K + 1, V);
    std::partial_sort(col.begin(), col.begin() + keep, col.end(),
                      [](const std::pair<float, int> &a, const std::pair<float, int> &b) {
                        return a.first != b.first ? a.first > b.first : a.second < b.second;
                      });
    if (V > K) margin = std::min(margin, std::log(col[K - 1].first) - std::log(col[K].first));
    for (int r = 0; r < std::min(K, V); ++r)
      cands.push_back(GlobObj{std::log(col[r].first) + prev_score[i] - (float)(r + 1) * diversity, i,
                              col[r].second});
  }
  std::stable_sort(cands.begin(), cands.end(),
                   [](const GlobObj &a, const GlobObj &b) { return a.val > b.val; });
  int slots = 0;
  for (size_t q = 0; q < cands.size(); ++q) {
    if (q + 1 < cands.size()) margin = std::min(margin, cands[q].val - cands[q + 1].val);
    if (cands[q].vocab != start_id && cands[q].vocab != eof_id && ++slots == beam) {
      // the neighbour below the last slot was compared too (it is the first one left out)
      break;
    }
  }
  return margin;
}

// SwapStatesDecoding, src/layer_input_to_hidden.h:1517-1531.
extern "C" void orc_beam_gather(const float *src, float *dst, int H, int B, const int *backptr) {
  for (int k = 0; k < B; ++k)
    memcpy(dst + (size_t)k * H, src + (size_t)backptr[k] * H, sizeof(float) * H);
}

// ------------------------------------------------------------------------------------------------
// Whole model (forward only).
struct orc_model {
  orc_model_config cfg;
  std::map<std::string, std::vector<float>> params;
  std::map<std::string, std::vector<float>> rowmajor;  // cached transposes for gemm_rowA
  bool committed = false;
};

namespace {

const char *kGateNames[4] = {"i", "f", "c", "o"};  // stacked order i,f,g(=c'),o

// Embedding size.  The reference fixes it to the LSTM size (src/global_configuration.h:220); a
// configuration with E > 0 generalises the two places that touch an embedding: the tables W are
// E x V and the first layer's input matrices M_* are H x E.
inline int emb_size(const orc_model_config &cfg) { return cfg.E > 0 ? cfg.E : cfg.H; }
// rows of the vector a layer reads from below
inline int in_size(const orc_model_config &cfg, int layer) { return layer == 0 ? emb_size(cfg) : cfg.H; }

void add_param(orc_model *m, const std::string &name, size_t n) { m->params[name].assign(n, 0.f); }

// y (rows x B) = P (rows x K, named parameter) * x (K x B)
void mat_apply(orc_model *m, const std::string &name, int rows, int K, const float *x, int B,
               float *y) {
  const auto it = m->rowmajor.find(name);
  if (it == m->rowmajor.end()) {
    fprintf(stderr, "orc_model: parameter %s not committed\n", name.c_str());
    exit(EXIT_FAILURE);
  }
  gemm_rowA(rows, B, K, it->second.data(), K, x, K, 1.f, 0.f, y, rows);
}

struct LayerState {
  std::vector<float> h, c;
};

// One LSTM layer step (node ForwardPropGpu): x is K x B (looked up: K = E; from below: K = H).
// Writes the stacked 4H x B products per operand and runs the cell.
void lstm_layer_step(orc_model *m, const std::string &pfx, int K, int B, const float *x,
                     const float *h_prev, const float *c_prev, const float *h_tild,
                     const int *mask01, float *h, float *c) {
  const int H = m->cfg.H;
  std::vector<float> p1((size_t)4 * H * B), p2((size_t)4 * H * B), p3;
  std::vector<float> tmp((size_t)H * B);
  const bool feed = h_tild != nullptr;
  if (feed) p3.resize((size_t)4 * H * B);
  std::vector<float> bias((size_t)4 * H);
  for (int g = 0; g < 4; ++g) {
    const std::string gn = kGateNames[g];
    mat_apply(m, pfx + "M_" + gn, H, K, x, B, tmp.data());
    for (int b = 0; b < B; ++b)
      memcpy(&p1[idx2c((size_t)g * H, b, (size_t)4 * H)], &tmp[(size_t)b * H], sizeof(float) * H);
    mat_apply(m, pfx + "W_h" + gn, H, H, h_prev, B, tmp.data());
    for (int b = 0; b < B; ++b)
      memcpy(&p2[idx2c((size_t)g * H, b, (size_t)4 * H)], &tmp[(size_t)b * H], sizeof(float) * H);
    if (feed) {
      mat_apply(m, pfx + "Q_" + gn, H, H, h_tild, B, tmp.data());
      for (int b = 0; b < B; ++b)
        memcpy(&p3[idx2c((size_t)g * H, b, (size_t)4 * H)], &tmp[(size_t)b * H], sizeof(float) * H);
    }
    memcpy(&bias[(size_t)g * H], m->params[pfx + "b_" + gn].data(), sizeof(float) * H);
  }
  orc_lstm_cell_fwd(H, B, p1.data(), p2.data(), feed ? p3.data() : nullptr, bias.data(), c_prev,
                    mask01, feed ? 1 : 0, 0.f, nullptr, c, h);
}

}  // namespace

extern "C" orc_model *orc_model_create(const orc_model_config *cfg) {
  orc_model *m = new orc_model();
  m->cfg = *cfg;
  const size_t H = cfg->H, E = emb_size(*cfg);
  for (int side = 0; side < 2; ++side) {
    const std::string s = side == 0 ? "src." : "tgt.";
    const size_t V = side == 0 ? cfg->V_src : cfg->V_tgt;
    for (int l = 0; l < cfg->layers; ++l) {
      const std::string pfx = s + std::to_string(l) + ".";
      for (int g = 0; g < 4; ++g) {
        const std::string gn = kGateNames[g];
        add_param(m, pfx + "W_h" + gn, H * H);
        add_param(m, pfx + "M_" + gn, H * (l == 0 ? E : H));
        add_param(m, pfx + "b_" + gn, H);
        if (side == 1 && l == 0 && cfg->feed_input && cfg->attention)
          add_param(m, pfx + "Q_" + gn, H * H);
      }
      if (l == 0) add_param(m, pfx + "W", E * V);
    }
  }
  if (cfg->attention) {
    add_param(m, "attn.W_a", H * H);
    add_param(m, "attn.W_p", H * H);
    add_param(m, "attn.v_p", H);
    add_param(m, "attn.b_out", H);
    add_param(m, "attn.W_c1", H * H);
    add_param(m, "attn.W_c2", H * H);
  }
  add_param(m, "softmax.D", (size_t)cfg->V_tgt * H);
  add_param(m, "softmax.b_d", cfg->V_tgt);
  return m;
}

extern "C" void orc_model_destroy(orc_model *m) { delete m; }

extern "C" float *orc_model_param(orc_model *m, const char *name, long long *n_elems) {
  const auto it = m->params.find(name);
  if (it == m->params.end()) return nullptr;
  if (n_elems) *n_elems = (long long)it->second.size();
  return it->second.data();
}

// Internal to the oracle (used by linmt_oracle_train.cpp): the row-major copy orc_model_commit
// keeps of a matrix parameter, or NULL when none is kept under that name.
const float *orc_model_rowmajor(orc_model *m, const char *name) {
  const auto it = m->rowmajor.find(name);
  if (it == m->rowmajor.end() || std::string(name) == "attn.W_a") return nullptr;
  return it->second.data();
}
void orc_gemm_rowmajor_a(int M, int N, int K, const float *At, const float *X, int ldx, float alpha,
                         float beta, float *C, int ldc) {
  gemm_rowA(M, N, K, At, K, X, ldx, alpha, beta, C, ldc);
}

extern "C" void orc_model_commit(orc_model *m) {
  const int H = m->cfg.H;
  m->rowmajor.clear();
  for (auto &kv : m->params) {
    const std::string &n = kv.first;
    const size_t dot = n.rfind('.');
    const std::string leaf = n.substr(dot + 1);
    if (leaf.rfind("W_h", 0) == 0 || leaf.rfind("M_", 0) == 0 || leaf.rfind("Q_", 0) == 0 ||
        leaf == "W_p" || leaf == "W_c1" || leaf == "W_c2") {
      auto &dst = m->rowmajor[n];
      dst.resize(kv.second.size());
      const int cols = (int)(kv.second.size() / (size_t)H);  // H, or E for the first layer's M_*
      transpose_to(kv.second.data(), H, cols, H, dst.data());
    } else if (leaf == "W_a") {
      m->rowmajor[n] = kv.second;  // used transposed: W_a^T row-major == W_a column-major
    } else if (leaf == "D") {
      auto &dst = m->rowmajor[n];
      dst.resize(kv.second.size());
      transpose_to(kv.second.data(), m->cfg.V_tgt, H, m->cfg.V_tgt, dst.data());
    }
  }
  m->committed = true;
}

namespace {

// Attention node on top of the decoder stack (ha = h_t, no dropout), writing h_tild.
void attention_step(orc_model *m, int B, const float *h_t, const float *hs, long long step_stride,
                    long long col_stride, const int *hs_col, int hs_steps, const int *batch_info,
                    const int *mask01, int max_len, float *h_tild, std::vector<int> *out_indices = nullptr,
                    std::vector<float> *out_align = nullptr, std::vector<float> *out_pt = nullptr) {
  const int H = m->cfg.H;
  const int D = m->cfg.attention == 1 ? m->cfg.D : -1;
  const int W = D >= 0 ? 2 * D + 1 : max_len;
  std::vector<float> tanh1((size_t)H * B, 0.f), wa((size_t)H * B), sig(B), pt(B), al((size_t)B * W),
      ce((size_t)B * W), cx((size_t)H * B), t1((size_t)H * B), t2((size_t)H * B);
  std::vector<int> ind((size_t)B * W);
  if (D >= 0) {
    mat_apply(m, "attn.W_p", H, H, h_t, B, tanh1.data());
    for (auto &v : tanh1) v = tanhf(v);
  }
  mat_apply(m, "attn.W_a", H, H, h_t, B, wa.data());
  orc_attn_core_fwd(H, B, D, max_len, hs_steps, tanh1.data(), m->params["attn.v_p"].data(),
                    wa.data(), hs, step_stride, col_stride, hs_col, batch_info, mask01, pt.data(),
                    sig.data(), ind.data(), al.data(), ce.data(), cx.data(), nullptr);
  if (out_indices) *out_indices = ind;
  if (out_align) *out_align = al;
  if (out_pt) *out_pt = pt;
  mat_apply(m, "attn.W_c1", H, H, cx.data(), B, t1.data());
  mat_apply(m, "attn.W_c2", H, H, h_t, B, t2.data());
  const float *b_out = m->params["attn.b_out"].data();
  for (int b = 0; b < B; ++b)
    for (int r = 0; r < H; ++r) {
      const size_t o = idx2c(r, b, H);
      float v = tanhf(t1[o] + t2[o] + b_out[r]);
      v *= mask01[b];
      h_tild[o] = v;
    }
}

struct Hyp {
  std::vector<int> tokens;  // with <START> ... <EOF>
  float score;
  // unk_replacement_mode__ only: per token the source position with the largest alignment score
  // and the alignment scores over the source positions (decoder.h:129-130)
  std::vector<int> viterbi;
  std::vector<std::vector<float>> align_scores;
};

// Per-step record of the search for orc_decode_sentence_trace: the beam after every expansion
// (tokens, LOCAL back-pointers, scores; beam entries per step) and the step's margin.
struct DecodeTrace {
  int *tok, *backptr;
  float *score, *margin;
  int cap_steps, steps;
  // optional, one value per step: how far the closest window position p_t of the step's live
  // columns was from an integer (the window is cut at (int)p_t, LowerUpperKernel
  // deep_rnn_kernel.h:1095-1098, so two fp32 evaluations of a p_t that close to an integer may
  // read different windows); 0.5 when the model has no local-p attention
  float *window_margin = nullptr;
};

int decode_impl(orc_model *const *ms, int num_models, const int *src_ids, int S,
                const orc_decode_opts *o, bool unk_mode, int *best_tokens, int cap, int *best_len,
                float *best_score, int *hyp_tokens, int *hyp_len, float *hyp_score, int hyp_cap,
                int *n_hyp, int *best_viterbi, DecodeTrace *trace = nullptr);

}  // namespace

// EnsembleFactory::DecodeFile for one sentence and one model (src/decoder.h:1702-1776) on top of
// NeuralMachineTranslation::ForwardPropSource / ForwardPropTarget / SwapDecodingStates /
// TargetCopyPrevStates (src/deep_rnn.h:1572-1872) and Decoder::{InitDecoder, ExpandHypothesis,
// FinishCurrentHypotheses, OutputKBestHypotheses} (src/decoder.h:334-699).  Alignment export is
// off, so every alignment-score row used by the coverage penalty is the all-zero vector the
// reference starts from (decoder.h:364-370).
extern "C" int orc_decode_sentence(orc_model *m, const int *src_ids, int S,
                                   const orc_decode_opts *o, int *best_tokens, int cap,
                                   int *best_len, float *best_score, int *hyp_tokens, int *hyp_len,
                                   float *hyp_score, int hyp_cap, int *n_hyp) {
  return decode_impl(&m, 1, src_ids, S, o, false, best_tokens, cap, best_len, best_score,
                     hyp_tokens, hyp_len, hyp_score, hyp_cap, n_hyp, nullptr);
}

// orc_decode_sentence that also records the beam after every expansion step and how close that
// step's decisions were (orc_beam_step_margin): trace_tok / trace_backptr / trace_score hold beam
// entries per step (back-pointers are beam-local), trace_margin one value per step; *n_steps
// receives the number of expansion steps recorded (at most cap_steps).
extern "C" int orc_decode_sentence_trace(orc_model *m, const int *src_ids, int S,
                                         const orc_decode_opts *o, int *best_tokens, int cap,
                                         int *best_len, float *best_score, int *trace_tok,
                                         int *trace_backptr, float *trace_score,
                                         float *trace_margin, int cap_steps, int *n_steps,
                                         float *trace_window_margin) {
  DecodeTrace tr{trace_tok, trace_backptr, trace_score, trace_margin, cap_steps, 0};
  tr.window_margin = trace_window_margin;
  const int rc = decode_impl(&m, 1, src_ids, S, o, false, best_tokens, cap, best_len, best_score,
                             nullptr, nullptr, nullptr, 0, nullptr, nullptr, &tr);
  *n_steps = tr.steps;
  return rc;
}

// The same with unk_replacement_mode__ on (layer_attention.h:342-386, decoder.h:1930-1962): every
// step exports the alignment scores over the source positions, the Viterbi alignment is their
// arg-max, both travel with the hypotheses, and the coverage penalty of OutputKBestHypotheses sees
// real scores.  best_viterbi (capacity cap) receives the alignments of the 1-best's tokens.
extern "C" int orc_decode_sentence_alignments(orc_model *m, const int *src_ids, int S,
                                              const orc_decode_opts *o, int *best_tokens, int cap,
                                              int *best_len, float *best_score, int *best_viterbi,
                                              int *hyp_tokens, int *hyp_len, float *hyp_score,
                                              int hyp_cap, int *n_hyp) {
  return decode_impl(&m, 1, src_ids, S, o, m->cfg.attention != 0, best_tokens, cap, best_len,
                     best_score, hyp_tokens, hyp_len, hyp_score, hyp_cap, n_hyp, best_viterbi);
}

// The same for an ensemble (EnsembleFactory with several models, src/decoder.h:1778-1931): every
// model runs every step, EnsemblesModels averages their distributions (and, with alignments, adds
// up their alignment scores) before ExpandHypothesis.  All models share the target vocabulary and
// the longest sentence; ms[0]'s configuration supplies them.
extern "C" int orc_decode_sentence_ensemble(orc_model *const *ms, int num_models, const int *src_ids,
                                            int S, const orc_decode_opts *o, int alignments,
                                            int *best_tokens, int cap, int *best_len,
                                            float *best_score, int *best_viterbi, int *hyp_tokens,
                                            int *hyp_len, float *hyp_score, int hyp_cap, int *n_hyp) {
  bool unk = alignments != 0;
  for (int k = 0; k < num_models; ++k) unk = unk && ms[k]->cfg.attention != 0;
  return decode_impl(ms, num_models, src_ids, S, o, unk, best_tokens, cap, best_len, best_score,
                     hyp_tokens, hyp_len, hyp_score, hyp_cap, n_hyp, unk ? best_viterbi : nullptr);
}

namespace {
int decode_impl(orc_model *const *ms, int num_models, const int *src_ids, int S,
                const orc_decode_opts *o, bool unk_mode,
                int *best_tokens, int cap, int *best_len, float *best_score, int *hyp_tokens,
                int *hyp_len, float *hyp_score, int hyp_cap, int *n_hyp, int *best_viterbi,
                DecodeTrace *trace) {
#ifdef _OPENMP
  if (o->num_threads > 0) omp_set_num_threads(o->num_threads);
#endif
  const int V = ms[0]->cfg.V_tgt;
  int beam = o->beam;
  if (beam > (int)std::sqrt((double)V)) beam = (int)std::sqrt((double)V);  // decoder.h:1662-1664
  const int start_symbol = 0, end_symbol = 1;
  const int longest = ms[0]->cfg.longest_sent;
  const int B = beam;
  const int one = 1;

  // what one model of the ensemble carries through the sentence
  struct Run {
    orc_model *m;
    int H, L;
    std::vector<LayerState> enc, prev, cur;
    std::vector<float> top_states, h_tild, h_tild_prev, xb, logits, dist, ascore;
  };
  std::vector<Run> runs(num_models);
  std::vector<int> ones(B, 1), batch_info(2 * B), hs_col(B, 0);
  for (int b = 0; b < B; ++b) {
    batch_info[b] = S;      // decoder.h:1277-1291: (len, 0) replicated over the beam
    batch_info[B + b] = 0;
  }
  for (int k = 0; k < num_models; ++k) {
    Run &r = runs[k];
    orc_model *m = r.m = ms[k];
    const orc_model_config &cfg = m->cfg;
    const int H = r.H = cfg.H, L = r.L = cfg.layers;
    // ---- ForwardPropSource: B = 1, source reversed (input_file_preprocess.cc:633) ---------------
    r.enc.resize(L);
    for (auto &s : r.enc) {
      s.h.assign(H, 0.f);
      s.c.assign(H, 0.f);
    }
    r.top_states.resize((size_t)S * H);
    const int E = emb_size(cfg);
    std::vector<float> x(std::max(E, H)), hn(H), cn(H);
    for (int t = 0; t < S; ++t) {
      int id = src_ids[S - 1 - t];
      int id0, m01;
      orc_preprocess_indices(&id, 1, &id0, &m01, nullptr);
      x.resize(E);
      orc_embed_lookup(m->params["src.0.W"].data(), E, cfg.V_src, &id0, 1, nullptr, 1.f, x.data());
      for (int l = 0; l < L; ++l) {
        const std::string pfx = "src." + std::to_string(l) + ".";
        lstm_layer_step(m, pfx, in_size(cfg, l), 1, x.data(), r.enc[l].h.data(), r.enc[l].c.data(),
                        nullptr, &one, hn.data(), cn.data());
        r.enc[l].h = hn;
        r.enc[l].c = cn;
        x = hn;
      }
      memcpy(&r.top_states[(size_t)t * H], r.enc[L - 1].h.data(), sizeof(float) * H);
    }
    // ---- decoder state: TransferDecodingStatesGpu broadcasts the encoder's final (h,c) ----------
    r.prev.resize(L);
    r.cur.resize(L);
    for (int l = 0; l < L; ++l) {
      r.prev[l].h.resize((size_t)H * B);
      r.prev[l].c.resize((size_t)H * B);
      r.cur[l].h.resize((size_t)H * B);
      r.cur[l].c.resize((size_t)H * B);
      for (int b = 0; b < B; ++b) {
        memcpy(&r.prev[l].h[(size_t)b * H], r.enc[l].h.data(), sizeof(float) * H);
        memcpy(&r.prev[l].c[(size_t)b * H], r.enc[l].c.data(), sizeof(float) * H);
      }
    }
    r.h_tild.assign((size_t)H * B, 0.f);
    r.h_tild_prev.assign((size_t)H * B, 0.f);
    r.xb.resize((size_t)E * B);
    r.logits.resize((size_t)V * B);
    r.dist.resize((size_t)V * B);
    r.ascore.assign((size_t)longest * B, 0.f);
  }

  // ---- Decoder::InitDecoder -----------------------------------------------------------------------
  int current_index = 0;
  std::vector<int> top_sentences((size_t)B * longest, start_symbol), top_tmp((size_t)B * longest);
  std::vector<float> top_scores(B, 0.f), top_scores_tmp(B, 0.f);
  std::vector<int> current_indices(B, start_symbol), new_indices_changes(B, 0);
  std::vector<Hyp> hyps;
  // viterbi_alignments__ / alignment_scores__ (utility_cu.h:91-93) and the per-beam histories
  // eigen_top_sentences_viterbi_ (initialised to -20, decoder.h:347) / _alignments_scores_
  std::vector<int> vit(B, -1), top_vit((size_t)B * longest, -20), top_vit_tmp;
  std::vector<float> ascore((size_t)longest * B, 0.f);
  std::vector<std::vector<float>> top_as((size_t)B * longest), top_as_tmp;
  auto column_scores = [&](int b) {
    return std::vector<float>(ascore.begin() + (size_t)longest * b,
                              ascore.begin() + (size_t)longest * (b + 1));
  };

  std::vector<int> tok(B), bp(B), fin_beam(B);
  std::vector<float> sc(B), fin_score(B);
  std::vector<const float *> dists(num_models);
  for (int k = 0; k < num_models; ++k) dists[k] = runs[k].dist.data();
  float step_window_margin = 0.5f;  // of the last forward_target call

  auto forward_target = [&](int curr_index) {
    step_window_margin = 0.5f;
    for (Run &r : runs) {
      orc_model *m = r.m;
      const orc_model_config &cfg = m->cfg;
      const int H = r.H, L = r.L;
      std::vector<int> id0(B), m01(B);
      orc_preprocess_indices(current_indices.data(), B, id0.data(), m01.data(), nullptr);
      orc_embed_lookup(m->params["tgt.0.W"].data(), emb_size(cfg), V, id0.data(), B, nullptr, 1.f,
                       r.xb.data());
      const float *below = r.xb.data();
      for (int l = 0; l < L; ++l) {
        const std::string pfx = "tgt." + std::to_string(l) + ".";
        const bool feed = l == 0 && cfg.feed_input && cfg.attention && curr_index != 0;
        lstm_layer_step(m, pfx, in_size(cfg, l), B, below, r.prev[l].h.data(), r.prev[l].c.data(),
                        feed ? r.h_tild_prev.data() : nullptr, ones.data(), r.cur[l].h.data(),
                        r.cur[l].c.data());
        below = r.cur[l].h.data();
      }
      const float *top = r.cur[L - 1].h.data();
      if (cfg.attention) {
        std::vector<int> ind;
        std::vector<float> al, pt;
        attention_step(m, B, top, r.top_states.data(), H, 0, hs_col.data(), S, batch_info.data(),
                       ones.data(), S, r.h_tild.data(), &ind, &al, &pt);
        top = r.h_tild.data();
        if (cfg.attention == 1)
          for (int b = 0; b < (curr_index == 0 ? 1 : B); ++b)  // step 0: the columns are copies
            step_window_margin = std::min(step_window_margin, std::fabs(pt[b] - std::nearbyint(pt[b])));
        if (unk_mode) {
          // layer_attention.h:360-385: scores of the window's valid slots, zero elsewhere
          std::fill(r.ascore.begin(), r.ascore.end(), 0.f);
          const int W = (int)(ind.size() / B);
          for (int j = 0; j < W; ++j)
            for (int b = 0; b < B; ++b) {
              const int idx = ind[idx2c(b, j, B)];
              if (idx != -1) r.ascore[(size_t)idx + (size_t)longest * b] = al[idx2c(b, j, B)];
            }
        }
      }
      mat_apply(m, "softmax.D", V, H, top, B, r.logits.data());
      orc_softmax_fwd(r.logits.data(), V, m->params["softmax.b_d"].data(), V, B, r.dist.data(), V);
    }
    if (unk_mode) {
      // EnsemblesModels (decoder.h:1933-1961): the models' scores added up, then the first
      // strictly largest score above 0
      for (size_t i = 0; i < ascore.size(); ++i) {
        float tmp_sum = 0;
        for (const Run &r : runs) tmp_sum += r.ascore[i];
        ascore[i] = tmp_sum;
      }
      for (int b = 0; b < B; ++b) {
        float max_val = 0;
        int max_index = -1;
        for (int j = 0; j < longest; ++j) {
          const float v = ascore[(size_t)j + (size_t)longest * b];
          if (v > max_val) {
            max_val = v;
            max_index = j;
          }
        }
        vit[b] = max_index;
      }
    }
  };

  int steps_run = 0;
  int last_index = 0;
  const int limit = std::min((int)(o->max_ratio * S), longest - 2);
  for (int curr_index = 0; curr_index < limit; ++curr_index) {
    forward_target(curr_index);
    ++steps_run;
    int nfin = 0;
    orc_beam_expand_ensemble(dists.data(), num_models, V, B, curr_index, top_scores.data(),
                             o->diversity, o->penalty, start_symbol, end_symbol, tok.data(),
                             bp.data(), sc.data(), &nfin, fin_beam.data(), fin_score.data());
    if (trace && curr_index < trace->cap_steps) {
      for (int i = 0; i < B; ++i) {
        trace->tok[(size_t)curr_index * B + i] = tok[i];
        trace->backptr[(size_t)curr_index * B + i] = bp[i];
        trace->score[(size_t)curr_index * B + i] = sc[i];
      }
      trace->margin[curr_index] =
          orc_beam_step_margin(dists.data(), num_models, V, B, curr_index, top_scores.data(),
                               o->diversity, start_symbol, end_symbol);
      if (trace->window_margin) trace->window_margin[curr_index] = step_window_margin;
      trace->steps = curr_index + 1;
    }
    // bookkeeping of decoder.h:436-479
    for (int f = 0; f < nfin; ++f) {
      Hyp h;
      h.tokens.assign(current_index + 2, 0);
      for (int j = 0; j < current_index + 2; ++j)
        h.tokens[j] = top_sentences[(size_t)fin_beam[f] * longest + j];
      h.tokens[current_index + 1] = end_symbol;
      h.score = fin_score[f];
      if (unk_mode) {
        const size_t row = (size_t)fin_beam[f] * longest;
        h.viterbi.assign(top_vit.begin() + row, top_vit.begin() + row + current_index + 2);
        h.viterbi[current_index + 1] = vit[fin_beam[f]];
        h.align_scores.assign(top_as.begin() + row, top_as.begin() + row + current_index + 2);
        h.align_scores[current_index + 1] = column_scores(fin_beam[f]);
      }
      hyps.push_back(h);
    }
    if (unk_mode) {
      top_vit_tmp = top_vit;
      top_as_tmp = top_as;
      for (int i = 0; i < B; ++i) {
        for (int j = 0; j < longest; ++j) {
          top_vit_tmp[(size_t)i * longest + j] = top_vit[(size_t)bp[i] * longest + j];
          top_as_tmp[(size_t)i * longest + j] = top_as[(size_t)bp[i] * longest + j];
        }
        top_vit_tmp[(size_t)i * longest + current_index + 1] = vit[bp[i]];
        top_as_tmp[(size_t)i * longest + current_index + 1] = column_scores(bp[i]);
      }
      top_vit.swap(top_vit_tmp);
      top_as.swap(top_as_tmp);
    }
    for (int i = 0; i < B; ++i) {
      memcpy(&top_tmp[(size_t)i * longest], &top_sentences[(size_t)bp[i] * longest],
             sizeof(int) * longest);
      top_tmp[(size_t)i * longest + current_index + 1] = tok[i];
      current_indices[i] = tok[i];
      new_indices_changes[i] = bp[i];
      top_scores_tmp[i] = sc[i];
    }
    top_sentences = top_tmp;
    top_scores = top_scores_tmp;
    current_index += 1;
    // SwapDecodingStates + TargetCopyPrevStates
    for (Run &r : runs) {
      for (int l = 0; l < r.L; ++l) {
        orc_beam_gather(r.cur[l].h.data(), r.prev[l].h.data(), r.H, B, new_indices_changes.data());
        orc_beam_gather(r.cur[l].c.data(), r.prev[l].c.data(), r.H, B, new_indices_changes.data());
      }
      if (r.m->cfg.attention && r.m->cfg.feed_input)
        orc_beam_gather(r.h_tild.data(), r.h_tild_prev.data(), r.H, B, new_indices_changes.data());
    }
    last_index = curr_index;
  }
  forward_target(last_index + 1);
  ++steps_run;
  // FinishCurrentHypotheses (decoder.h:502-525): row-major dist(1, i) = p(<EOF> | column i) after
  // the host renormalisation.
  {
    std::vector<float> rn;
    renormalise(dists.data(), num_models, V, B, rn);
    for (int i = 0; i < B; ++i) {
      top_sentences[(size_t)i * longest + current_index + 1] = end_symbol;
      top_scores[i] += std::log(rn[(size_t)1 * B + i]) + o->penalty;
      Hyp h;
      h.tokens.assign(top_sentences.begin() + (size_t)i * longest,
                      top_sentences.begin() + (size_t)i * longest + current_index + 2);
      h.score = top_scores[i];
      if (unk_mode) {
        const size_t row = (size_t)i * longest;
        h.viterbi.assign(top_vit.begin() + row, top_vit.begin() + row + current_index + 2);
        h.viterbi[current_index + 1] = vit[i];
        h.align_scores.assign(top_as.begin() + row, top_as.begin() + row + current_index + 2);
        h.align_scores[current_index + 1] = column_scores(i);
      }
      hyps.push_back(h);
    }
    current_index += 1;
  }

  if (n_hyp) *n_hyp = (int)hyps.size();
  if (hyp_tokens) {
    for (int i = 0; i < (int)hyps.size() && i < hyp_cap; ++i) {
      const int n = std::min((int)hyps[i].tokens.size(), cap);
      for (int j = 0; j < n; ++j) hyp_tokens[(size_t)i * cap + j] = hyps[i].tokens[j];
      hyp_len[i] = (int)hyps[i].tokens.size();
      hyp_score[i] = hyps[i].score;
    }
  }

  // ---- OutputKBestHypotheses (decoder.h:529-699), num_hypotheses = 1 ------------------------------
  std::vector<float> rs(hyps.size());
  for (size_t i = 0; i < hyps.size(); ++i) {
    float s = hyps[i].score;
    const int size = (int)hyps[i].tokens.size();
    if (0 != o->lp_alpha) {
      const float lp = powf((float)(5 + size), o->lp_alpha) / powf((float)(5 + 1), o->lp_alpha);
      s /= lp;
    }
    if (0 != o->cp_beta && unk_mode) {
      // decoder.h:541-583 on the exported scores: +0.01, rows normalised over the source, then
      // the log of each source position's capped total
      std::vector<std::vector<float>> &as = hyps[i].align_scores;
      for (int j = 1; j < size - 1; ++j) {
        float sum = 0;
        for (int k = 0; k < S; ++k) {
          as[j][k] += 0.01f;
          sum += as[j][k];
        }
        for (int k = 0; k < S; ++k) as[j][k] /= sum;
      }
      float cp = 0;
      for (int k = 0; k < S; ++k) {
        float sum = 0;
        for (int j = 1; j < size - 1; ++j) sum += as[j][k];
        cp += std::log(std::min(sum, 1.0f));
      }
      cp *= o->cp_beta;
      if (cp < -20) cp = -20;
      s += cp;
    } else if (0 != o->cp_beta) {
      // alignment-score rows are all zero: +0.01 each, normalised to 0.01/sum(0.01 x S)
      float unit;
      {
        float sum = 0;
        for (int k = 0; k < S; ++k) sum += 0.01f;
        unit = 0.01f / sum;
      }
      float cp = 0;
      for (int k = 0; k < S; ++k) {
        float sum = 0;
        for (int j = 1; j < size - 1; ++j) sum += unit;
        cp += std::log(std::min(sum, 1.0f));
      }
      cp *= o->cp_beta;
      if (cp < -20) cp = -20;
      s += cp;
    }
    rs[i] = s;
  }
  int best = -1;
  {
    // size-1 bounded heap of decoder.h:588-600: the first hypothesis passing the ratio filter is
    // kept until a strictly better one arrives.
    for (size_t i = 0; i < hyps.size(); ++i) {
      const float len_ratio = ((float)hyps[i].tokens.size()) / S;
      if (len_ratio > o->min_ratio) {
        if (best < 0 || rs[best] < rs[i]) best = (int)i;
      }
    }
  }
  *best_len = 0;
  *best_score = 0.f;
  if (best >= 0) {
    const auto &t = hyps[best].tokens;
    int n = 0;
    for (size_t j = 1; j + 1 < t.size() && n < cap; ++j) {
      if (best_viterbi) best_viterbi[n] = unk_mode ? hyps[best].viterbi[j] : -1;
      best_tokens[n++] = t[j];
    }
    *best_len = n;
    *best_score = rs[best];
  }
  return steps_run;
}
}  // namespace

// NeuralMachineTranslation::GetError (src/deep_rnn.h:2173-2317) with SoftmaxLayer::ComputeLossGpu.
extern "C" double orc_forward_xent(orc_model *m, const int *src, int S, const int *tgt_in,
                                   const int *tgt_out, int T, int B, const int *batch_info,
                                   int num_threads) {
#ifdef _OPENMP
  if (num_threads > 0) omp_set_num_threads(num_threads);
#endif
  const orc_model_config &cfg = m->cfg;
  const int H = cfg.H, L = cfg.layers, V = cfg.V_tgt, E = emb_size(cfg);
  std::vector<LayerState> st(L);
  for (auto &s : st) {
    s.h.assign((size_t)H * B, 0.f);
    s.c.assign((size_t)H * B, 0.f);
  }
  std::vector<float> hs((size_t)S * H * B);
  std::vector<float> x((size_t)std::max(E, H) * B), hn((size_t)H * B), cn((size_t)H * B);
  std::vector<int> id0(B), m01(B);
  for (int t = 0; t < S; ++t) {
    orc_preprocess_indices(src + (size_t)t * B, B, id0.data(), m01.data(), nullptr);
    x.resize((size_t)E * B);
    orc_embed_lookup(m->params["src.0.W"].data(), E, cfg.V_src, id0.data(), B, nullptr, 1.f,
                     x.data());
    for (int l = 0; l < L; ++l) {
      const std::string pfx = "src." + std::to_string(l) + ".";
      lstm_layer_step(m, pfx, in_size(cfg, l), B, x.data(), st[l].h.data(), st[l].c.data(), nullptr, m01.data(),
                      hn.data(), cn.data());
      st[l].h = hn;
      st[l].c = cn;
      x = hn;
    }
    memcpy(&hs[(size_t)t * H * B], st[L - 1].h.data(), sizeof(float) * H * B);
  }
  double loss = 0;
  std::vector<float> h_tild((size_t)H * B, 0.f), logits((size_t)V * B);
  std::vector<int> t0(B), tm(B);
  for (int t = 0; t < T; ++t) {
    orc_preprocess_indices(tgt_in + (size_t)t * B, B, id0.data(), m01.data(), nullptr);
    x.resize((size_t)E * B);
    orc_embed_lookup(m->params["tgt.0.W"].data(), E, V, id0.data(), B, nullptr, 1.f, x.data());
    for (int l = 0; l < L; ++l) {
      const std::string pfx = "tgt." + std::to_string(l) + ".";
      const bool feed = l == 0 && cfg.feed_input && cfg.attention && t != 0;
      lstm_layer_step(m, pfx, in_size(cfg, l), B, x.data(), st[l].h.data(), st[l].c.data(),
                      feed ? h_tild.data() : nullptr, m01.data(), hn.data(), cn.data());
      st[l].h = hn;
      st[l].c = cn;
      x = hn;
    }
    const float *top = st[L - 1].h.data();
    if (cfg.attention) {
      attention_step(m, B, top, hs.data(), (long long)H * B, H, nullptr, S, batch_info,
                     m01.data(), S, h_tild.data());
      top = h_tild.data();
    }
    mat_apply(m, "softmax.D", V, H, top, B, logits.data());
    orc_preprocess_indices(tgt_out + (size_t)t * B, B, t0.data(), tm.data(), nullptr);
    orc_logsoftmax_xent(logits.data(), V, m->params["softmax.b_d"].data(), V, B, t0.data(),
                        tm.data(), nullptr, &loss);
  }
  return loss;
}
