// Attention core (Luong local-p, and the textbook global "general" variant): alignment position,
// window indices, scores, max-subtracted exp, normalisation, Gaussian weighting and the context
// vector in ONE kernel.  One workgroup (4 wavefronts) per column b:
//   phase 1  v_p . tanh1[:,b]  -> sigmoid -> p_b -> window [lo,hi]           (block reduction)
//   phase 2  score_j = hs_j . wa[:,b]; wavefront w takes slots j = w, w+4, ...  (DPP/shuffle sums)
//   phase 3  max / exp / sum / Gaussian over the <= W slots, kept in LDS
//   phase 4  ctx[:,b] = sum_j a_j hs_j, thread-per-row-quad; the second read of the window comes
//            from L2 (the W x H window was just streamed by this very workgroup).
// The reference materialises the window (LoadInHSKernel) and launches eight kernels for this.
#include "lh_common.h"

namespace {

constexpr int kMaxSlots = 512;
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / lh::kWave;

struct AttnArgs {
  int H, B, D, W;
  const float *tanh1, *v_p, *wa, *hs;
  long long proj_col_stride;  // distance between columns of tanh1 and of wa (>= H)
  long long step_stride, col_stride;
  int hs_steps;
  const int *hs_col, *batch_info, *mask01;
  float *p_t, *sigma;
  int *indices;
  float *align, *cached_exp, *ctx;
  int *viterbi;
  // Projected memory (register kernel only).  ctx_mem != NULL: the context sum runs over ctx_mem
  // (laid out like hs) instead of hs.  out_add / out_bias != NULL are added to that sum (out_add
  // per column, out_add_col_stride apart) and out_tanh applies tanh and the column mask: the
  // output is then the attention layer's h~ rather than the context vector.
  long long wa_col_stride;  // distance between columns of wa
  const float *ctx_mem, *out_add, *out_bias;
  long long out_add_col_stride;
  int out_tanh;
};

template <bool VEC>
__device__ __forceinline__ float dot_wave(const float *__restrict__ x, const float *__restrict__ y,
                                          int H, int lane) {
  float acc = 0.f;
  if constexpr (VEC) {
    for (int r = lane * 4; r < H; r += lh::kWave * 4) {
      const float4 a = *reinterpret_cast<const float4 *>(x + r);
      const float4 b = *reinterpret_cast<const float4 *>(y + r);
      acc += a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
    }
  } else {
    for (int r = lane; r < H; r += lh::kWave) acc += x[r] * y[r];
  }
  return lh::wave_sum(acc);
}

template <bool VEC>
__global__ __launch_bounds__(kThreads) void attn_core_kernel(const AttnArgs a) {
  __shared__ float s_val[kMaxSlots];   // scores, then alignment weights
  __shared__ int s_tau[kMaxSlots];     // encoder timestep of slot j, -1 = no state to read
  __shared__ int s_idx[kMaxSlots];     // source position of slot j, -1 = invalid slot
  __shared__ float s_red[kWaves];
  __shared__ float s_scalar[2];

  const int b = lh::xcd_contiguous(blockIdx.x, gridDim.x);  // a sentence's columns on one XCD
  const int tid = threadIdx.x, wave = tid / lh::kWave, lane = tid % lh::kWave;
  const int H = a.H, B = a.B, W = a.W, D = a.D;
  const int len = a.batch_info[b];
  const int off = a.batch_info[B + b];
  const int m = a.mask01[b];
  const int col = a.hs_col ? a.hs_col[b] : b;
  const float *wa = a.wa + (size_t)b * a.proj_col_stride;
  const float *hs_c = a.hs + (size_t)col * a.col_stride;

  float p = 0.f;
  int lo = 0, hi = len - 1;
  if (D >= 0) {
    float part = 0.f;
    const float *t1 = a.tanh1 + (size_t)b * a.proj_col_stride;
    for (int r = tid; r < H; r += kThreads) part += a.v_p[r] * t1[r];
    const float dot = lh::block_sum<kWaves>(part, s_red);
    const float sig = (float)(1.0 / (1.0 + exp(-1.0 * (double)dot)));
    p = (float)len * sig;
    lo = (0 > (int)p - D) ? 0 : ((int)p - D);
    hi = ((len - 1) < (int)p + D) ? (len - 1) : ((int)p + D);
    if (tid == 0) {
      a.p_t[b] = p;
      a.sigma[b] = sig;
    }
  }

  // window indices (reference layout B x W, element (b,j) at b + B*j)
  for (int j = tid; j < W; j += kThreads) {
    int idx = -1;
    if (m == 1 && lo + j <= hi) idx = lo + j;
    a.indices[b + (size_t)B * j] = idx;
    s_idx[j] = idx;
    int tau = -1;
    if (idx >= 0) {
      tau = len - 1 - idx + off;
      if (tau < 0 || tau >= a.hs_steps) tau = -1;  // outside the caller's state buffer: zero vector
    }
    s_tau[j] = tau;
  }
  __syncthreads();

  // scores
  for (int j = wave; j < W; j += kWaves) {
    const int tau = s_tau[j];
    float sc = 0.f;
    if (tau >= 0) sc = dot_wave<VEC>(hs_c + (size_t)tau * a.step_stride, wa, H, lane);
    if (lane == 0) s_val[j] = sc;
  }
  __syncthreads();

  // normalisation: every thread reduces the (few) slots redundantly out of LDS
  float mx = D >= 0 ? 0.f : -FLT_MAX;
  for (int j = 0; j < W; ++j) {
    if (s_idx[j] != -1 && s_val[j] > mx) mx = s_val[j];
  }
  float Z = 0.f;
  for (int j = 0; j < W; ++j) {
    if (s_idx[j] != -1) Z += expf(s_val[j] - mx);
  }
  __syncthreads();
  const float sigma_sq = (float)((D * D) / 4.0);
  for (int j = tid; j < W; j += kThreads) {
    const int idx = s_idx[j];
    float al = 0.f, g = 1.f;
    if (idx != -1) {
      const float e = expf(s_val[j] - mx);
      if (D >= 0) {
        const float dlt = p - (float)idx;
        g = expf((-1.f * (dlt * dlt)) / (2.f * sigma_sq));
      }
      al = (Z != 0.f) ? (e / Z) * g : e;
    }
    a.align[b + (size_t)B * j] = al;
    a.cached_exp[j + (size_t)W * b] = g;
    s_val[j] = al;
  }
  __syncthreads();

  if (a.viterbi && tid == 0) {
    float best = -1.f;
    int best_idx = -1;
    for (int j = 0; j < W; ++j) {
      if (best < s_val[j]) {
        best = s_val[j];
        best_idx = s_idx[j];
      }
    }
    a.viterbi[b] = best_idx;
  }

  // context vector
  float *ctx = a.ctx + (size_t)b * H;
  if constexpr (VEC) {
    for (int r = tid * 4; r < H; r += kThreads * 4) {
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int j = 0; j < W; ++j) {
        const int tau = s_tau[j];
        if (tau < 0) continue;
        const float w = s_val[j];
        const float4 v = *reinterpret_cast<const float4 *>(hs_c + (size_t)tau * a.step_stride + r);
        acc.x += w * v.x; acc.y += w * v.y; acc.z += w * v.z; acc.w += w * v.w;
      }
      *reinterpret_cast<float4 *>(ctx + r) = acc;
    }
  } else {
    for (int r = tid; r < H; r += kThreads) {
      float acc = 0.f;
      for (int j = 0; j < W; ++j) {
        const int tau = s_tau[j];
        if (tau < 0) continue;
        acc += s_val[j] * hs_c[(size_t)tau * a.step_stride + r];
      }
      ctx[r] = acc;
    }
  }
}

// The same computation for windows of at most WCAP slots (local-p with D <= 10) and 16-byte
// aligned operands: the whole W x H window of the column is read ONCE, straight into registers
// (thread t holds rows 4t..4t+3 -- and 4(t+256).. when H > 1024 -- of every slot, all loads in
// flight together), the scores are block-reduced from per-thread partial dot products, and the
// context vector is accumulated from the same registers.
template <int NQ, int WCAP>
__global__ __launch_bounds__(kThreads) void attn_core_regs_kernel(const AttnArgs a) {
  __shared__ float s_part[kWaves][WCAP];
  __shared__ float s_val[WCAP];
  __shared__ int s_tau[WCAP];
  __shared__ int s_idx[WCAP];
  __shared__ float s_red[kWaves];

  const int b = lh::xcd_contiguous(blockIdx.x, gridDim.x);  // a sentence's columns on one XCD
  const int tid = threadIdx.x, wave = tid / lh::kWave, lane = tid % lh::kWave;
  const int H = a.H, B = a.B, W = a.W, D = a.D;
  const int len = a.batch_info[b];
  const int off = a.batch_info[B + b];
  const int m = a.mask01[b];
  const int col = a.hs_col ? a.hs_col[b] : b;
  const float *wa = a.wa + (size_t)b * a.wa_col_stride;
  const float *hs_c = a.hs + (size_t)col * a.col_stride;

  // everything that does not depend on the window position is requested first
  float4 w4[NQ], oadd[NQ], obias[NQ];
  bool row_ok[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int r = (tid + q * kThreads) * 4;
    row_ok[q] = r < H;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    w4[q] = row_ok[q] ? *reinterpret_cast<const float4 *>(wa + r) : zero;
    oadd[q] = (row_ok[q] && a.out_add)
                  ? *reinterpret_cast<const float4 *>(a.out_add + (size_t)b * a.out_add_col_stride + r)
                  : zero;
    obias[q] = (row_ok[q] && a.out_bias) ? *reinterpret_cast<const float4 *>(a.out_bias + r) : zero;
  }

  float p = 0.f;
  int lo = 0, hi = len - 1;
  if (D >= 0) {
    float part = 0.f;
    const float *t1 = a.tanh1 + (size_t)b * a.proj_col_stride;
    // rows tid, tid + 256, ... in that order (H <= NQ * 1024), all loads in flight together
    float vv[4 * NQ], tt[4 * NQ];
#pragma unroll
    for (int k = 0; k < 4 * NQ; ++k) {
      const int r = tid + k * kThreads;
      vv[k] = r < H ? a.v_p[r] : 0.f;
      tt[k] = r < H ? t1[r] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < 4 * NQ; ++k)
      if (tid + k * kThreads < H) part += vv[k] * tt[k];
    const float dot = lh::block_sum<kWaves>(part, s_red);
    const float sig = (float)(1.0 / (1.0 + exp(-1.0 * (double)dot)));
    p = (float)len * sig;
    lo = (0 > (int)p - D) ? 0 : ((int)p - D);
    hi = ((len - 1) < (int)p + D) ? (len - 1) : ((int)p + D);
    if (tid == 0) {
      a.p_t[b] = p;
      a.sigma[b] = sig;
    }
  }
  for (int j = tid; j < WCAP; j += kThreads) {
    int idx = -1, tau = -1;
    if (j < W) {
      if (m == 1 && lo + j <= hi) idx = lo + j;
      a.indices[b + (size_t)B * j] = idx;
      if (idx >= 0) {
        tau = len - 1 - idx + off;
        if (tau < 0 || tau >= a.hs_steps) tau = -1;
      }
    }
    s_idx[j] = idx;
    s_tau[j] = tau;
  }
  __syncthreads();

  // the window, once
  float4 h[WCAP][NQ];
#pragma unroll
  for (int j = 0; j < WCAP; ++j) {
    const int tau = s_tau[j];  // the same for every thread: a scalar branch
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      h[j][q] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (tau >= 0 && row_ok[q])
        h[j][q] = *reinterpret_cast<const float4 *>(hs_c + (size_t)tau * a.step_stride +
                                                    (size_t)(tid + q * kThreads) * 4);
    }
  }
  // scores: per-thread partial dot products, wavefront sums, then the four wavefronts in order
#pragma unroll
  for (int j = 0; j < WCAP; ++j) {
    float sc = 0.f;
#pragma unroll
    for (int q = 0; q < NQ; ++q)
      sc += h[j][q].x * w4[q].x + h[j][q].y * w4[q].y + h[j][q].z * w4[q].z + h[j][q].w * w4[q].w;
    sc = lh::wave_sum(sc);
    if (lane == 0) s_part[wave][j] = sc;
  }
  if (a.ctx_mem) {
    // the scores are done with the window: the same registers take the window of ctx_mem, whose
    // loads fly while the scores are normalised
    const float *cm = a.ctx_mem + (size_t)col * a.col_stride;
#pragma unroll
    for (int j = 0; j < WCAP; ++j) {
      const int tau = s_tau[j];
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        h[j][q] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (tau >= 0 && row_ok[q])
          h[j][q] = *reinterpret_cast<const float4 *>(cm + (size_t)tau * a.step_stride +
                                                      (size_t)(tid + q * kThreads) * 4);
      }
    }
  }
  __syncthreads();
  for (int j = tid; j < WCAP; j += kThreads) {
    float sc = s_part[0][j];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sc += s_part[w][j];
    s_val[j] = s_tau[j] >= 0 ? sc : 0.f;
  }
  __syncthreads();

  float mx = D >= 0 ? 0.f : -FLT_MAX;
  for (int j = 0; j < W; ++j) {
    if (s_idx[j] != -1 && s_val[j] > mx) mx = s_val[j];
  }
  // one exponential per slot, taken by the slot's thread; the sum then runs over the slots in
  // order as before
  __shared__ float s_exp[WCAP];
  for (int j = tid; j < WCAP; j += kThreads)
    s_exp[j] = (j < W && s_idx[j] != -1) ? expf(s_val[j] - mx) : 0.f;
  __syncthreads();
  float Z = 0.f;
  for (int j = 0; j < W; ++j) {
    if (s_idx[j] != -1) Z += s_exp[j];
  }
  const float sigma_sq = (float)((D * D) / 4.0);
  for (int j = tid; j < WCAP; j += kThreads) {
    float al = 0.f, g = 1.f;
    if (j < W) {
      const int idx = s_idx[j];
      if (idx != -1) {
        const float e = s_exp[j];
        if (D >= 0) {
          const float dlt = p - (float)idx;
          g = expf((-1.f * (dlt * dlt)) / (2.f * sigma_sq));
        }
        al = (Z != 0.f) ? (e / Z) * g : e;
      }
      a.align[b + (size_t)B * j] = al;
      a.cached_exp[j + (size_t)W * b] = g;
    }
    s_val[j] = al;
  }
  __syncthreads();

  if (a.viterbi && tid == 0) {
    float best = -1.f;
    int best_idx = -1;
    for (int j = 0; j < W; ++j) {
      if (best < s_val[j]) {
        best = s_val[j];
        best_idx = s_idx[j];
      }
    }
    a.viterbi[b] = best_idx;
  }

  float *ctx = a.ctx + (size_t)b * H;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int j = 0; j < WCAP; ++j) {
      if (s_tau[j] < 0) continue;  // the general kernel skips these slots too
      const float w = s_val[j];
      acc.x += w * h[j][q].x; acc.y += w * h[j][q].y; acc.z += w * h[j][q].z; acc.w += w * h[j][q].w;
    }
    if (!row_ok[q]) continue;
    const size_t r = (size_t)(tid + q * kThreads) * 4;
    if (a.out_add) {
      acc.x += oadd[q].x; acc.y += oadd[q].y; acc.z += oadd[q].z; acc.w += oadd[q].w;
    }
    if (a.out_bias) {
      acc.x += obias[q].x; acc.y += obias[q].y; acc.z += obias[q].z; acc.w += obias[q].w;
    }
    if (a.out_tanh) {
      const float mf = (float)m;
      acc.x = tanhf(acc.x) * mf; acc.y = tanhf(acc.y) * mf;
      acc.z = tanhf(acc.z) * mf; acc.w = tanhf(acc.w) * mf;
    }
    *reinterpret_cast<float4 *>(ctx + r) = acc;
  }
}

constexpr int kRegsSlots = 21;  // the reference's default window: D = 10

}  // namespace

extern "C" int lh_attn_core_fwd_f32(int H, int B, int D, int max_len, int hs_steps,
                                    const float *tanh1, const float *v_p, const float *wa,
                                    long long proj_col_stride, const float *hs,
                                    long long hs_step_stride,
                                    long long hs_col_stride, const int *hs_col,
                                    const int *batch_info, const int *mask01, float *p_t,
                                    float *sigma, int *indices, float *align, float *cached_exp,
                                    float *ctx, int *viterbi, lh_stream_t stream) {
  if (H <= 0 || B <= 0 || hs_steps <= 0)
    return lh::fail_arg("lh_attn_core_fwd_f32: H=%d B=%d hs_steps=%d", H, B, hs_steps);
  const int W = D >= 0 ? 2 * D + 1 : max_len;
  if (W <= 0 || W > kMaxSlots)
    return lh::fail_arg("lh_attn_core_fwd_f32: window of %d slots outside [1,%d]", W, kMaxSlots);
  if (!wa || !hs || !batch_info || !mask01 || !indices || !align || !cached_exp || !ctx)
    return lh::fail_arg("lh_attn_core_fwd_f32: a required pointer is NULL");
  if (D >= 0 && (!tanh1 || !v_p || !p_t || !sigma))
    return lh::fail_arg("lh_attn_core_fwd_f32: local-p needs tanh1, v_p, p_t and sigma");
  if (hs_step_stride < 0 || hs_col_stride < 0)
    return lh::fail_arg("lh_attn_core_fwd_f32: negative stride");
  if (proj_col_stride == 0) proj_col_stride = H;
  if (proj_col_stride < H)
    return lh::fail_arg("lh_attn_core_fwd_f32: proj_col_stride %lld < H", proj_col_stride);

  AttnArgs a{H, B, D, W, tanh1, v_p, wa, hs, proj_col_stride, hs_step_stride, hs_col_stride, hs_steps, hs_col,
             batch_info, mask01, p_t, sigma, indices, align, cached_exp, ctx, viterbi,
             proj_col_stride, nullptr, nullptr, nullptr, 0, 0};
  const bool vec = H % 4 == 0 && lh::aligned16(wa) && lh::aligned16(hs) && lh::aligned16(ctx) &&
                   hs_step_stride % 4 == 0 && hs_col_stride % 4 == 0 && proj_col_stride % 4 == 0;
  hipStream_t st = lh::as_stream(stream);
  if (vec && W <= kRegsSlots && H <= 4 * kThreads)
    hipLaunchKernelGGL((attn_core_regs_kernel<1, kRegsSlots>), dim3(B), dim3(kThreads), 0, st, a);
  else if (vec && W <= kRegsSlots && H <= 8 * kThreads)
    hipLaunchKernelGGL((attn_core_regs_kernel<2, kRegsSlots>), dim3(B), dim3(kThreads), 0, st, a);
  else if (vec) hipLaunchKernelGGL(attn_core_kernel<true>, dim3(B), dim3(kThreads), 0, st, a);
  else hipLaunchKernelGGL(attn_core_kernel<false>, dim3(B), dim3(kThreads), 0, st, a);
  return lh::check_launch("lh_attn_core_fwd_f32");
}

extern "C" int lh_attn_core_projected_fwd_f32(int H, int B, int D, int hs_steps, const float *tanh1,
                                              long long tanh1_col_stride, const float *v_p,
                                              const float *h_t, long long h_t_col_stride,
                                              const float *score_mem, const float *ctx_mem,
                                              long long mem_step_stride, long long mem_col_stride,
                                              const int *mem_col, const int *batch_info,
                                              const int *mask01, const float *out_add,
                                              long long out_add_col_stride, const float *out_bias,
                                              float *p_t, float *sigma, int *indices, float *align,
                                              float *cached_exp, float *h_tild, int *viterbi,
                                              lh_stream_t stream) {
  if (H <= 0 || B <= 0 || hs_steps <= 0)
    return lh::fail_arg("lh_attn_core_projected_fwd_f32: H=%d B=%d hs_steps=%d", H, B, hs_steps);
  const int W = 2 * D + 1;
  if (D < 0 || W > LH_ATTN_PROJECTED_MAX_WINDOW || H > LH_ATTN_PROJECTED_MAX_H || H % 4 != 0)
    return lh::fail_arg("lh_attn_core_projected_fwd_f32: D=%d H=%d outside what the kernel holds in "
                        "registers (window <= %d, H <= %d, H %% 4 == 0)", D, H,
                        LH_ATTN_PROJECTED_MAX_WINDOW, LH_ATTN_PROJECTED_MAX_H);
  if (!tanh1 || !v_p || !h_t || !score_mem || !ctx_mem || !batch_info || !mask01 || !out_add ||
      !out_bias || !p_t || !sigma || !indices || !align || !cached_exp || !h_tild)
    return lh::fail_arg("lh_attn_core_projected_fwd_f32: a required pointer is NULL");
  if (tanh1_col_stride == 0) tanh1_col_stride = H;
  if (h_t_col_stride == 0) h_t_col_stride = H;
  if (out_add_col_stride == 0) out_add_col_stride = H;
  if (tanh1_col_stride < H || h_t_col_stride < H || out_add_col_stride < H || mem_step_stride < 0 ||
      mem_col_stride < 0)
    return lh::fail_arg("lh_attn_core_projected_fwd_f32: a stride is too small");
  if (!lh::aligned16(h_t) || !lh::aligned16(score_mem) || !lh::aligned16(ctx_mem) ||
      !lh::aligned16(out_add) || !lh::aligned16(out_bias) || !lh::aligned16(h_tild) ||
      h_t_col_stride % 4 != 0 || out_add_col_stride % 4 != 0 || mem_step_stride % 4 != 0 ||
      mem_col_stride % 4 != 0)
    return lh::fail_arg("lh_attn_core_projected_fwd_f32: operands must be 16-byte aligned with "
                        "strides that are multiples of 4");
  static_assert(LH_ATTN_PROJECTED_MAX_WINDOW == kRegsSlots && LH_ATTN_PROJECTED_MAX_H == 8 * kThreads,
                "limits published in the header");
  AttnArgs a{H, B, D, W, tanh1, v_p, h_t, score_mem, tanh1_col_stride, mem_step_stride, mem_col_stride,
             hs_steps, mem_col, batch_info, mask01, p_t, sigma, indices, align, cached_exp, h_tild,
             viterbi, h_t_col_stride, ctx_mem, out_add, out_bias, out_add_col_stride, 1};
  hipStream_t st = lh::as_stream(stream);
  if (H <= 4 * kThreads)
    hipLaunchKernelGGL((attn_core_regs_kernel<1, kRegsSlots>), dim3(B), dim3(kThreads), 0, st, a);
  else
    hipLaunchKernelGGL((attn_core_regs_kernel<2, kRegsSlots>), dim3(B), dim3(kThreads), 0, st, a);
  return lh::check_launch("lh_attn_core_projected_fwd_f32");
}
