// Training-side kernels: fused LSTM cell backward, attention backward, bias-gradient row sums,
// deterministic embedding-gradient gather, gradient norm and the fused clip + SGD step.
// All of them are HBM-bound passes: one coalesced read of every input, one write of every output.
#include "lh_common.h"

namespace {

template <int VW>
struct Vec;
template <>
struct Vec<4> {
  float v[4];
  __device__ __forceinline__ void load(const float *p) {
    const float4 t = *reinterpret_cast<const float4 *>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ __forceinline__ void store(float *p) const {
    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <>
struct Vec<1> {
  float v[1];
  __device__ __forceinline__ void load(const float *p) { v[0] = *p; }
  __device__ __forceinline__ void store(float *p) const { *p = v[0]; }
};

__device__ __forceinline__ float clampf(float x, float lim) {
  return lim > 0.f ? fminf(fmaxf(x, -lim), lim) : x;
}

// ---------------------------------------------------------------------------------------------
// LSTM cell backward
struct CellBwdArgs {
  int H, B;
  lh_error_term above, next;  // p == NULL: none
  const float *dc_next, *gates, *c, *c_prev;
  const int *mask01;
  float clip_above, clip_next;
  const float *above_drop_mask;
  float keep;
  float *dgates, *dc_prev;
};

// an incoming error: the sum of the term's planes, in plane order
template <int VW>
__device__ __forceinline__ void load_term(const lh_error_term &e, int b, int r, Vec<VW> *out) {
  const float *p = e.p + (size_t)b * e.ld + r;
  out->load(p);
  if (e.planes > 1) {  // the reduction launch starts from +0: a plane's -0 comes out as +0
#pragma unroll
    for (int i = 0; i < VW; ++i) out->v[i] = 0.f + out->v[i];
  }
  for (int s = 1; s < e.planes; ++s) {
    Vec<VW> u;
    u.load(p + (size_t)s * e.plane_stride);
#pragma unroll
    for (int i = 0; i < VW; ++i) out->v[i] += u.v[i];
  }
}

template <int VW>
__global__ __launch_bounds__(256) void lstm_cell_bwd_kernel(const CellBwdArgs a) {
  const int HQ = a.H / VW;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)HQ * a.B) return;
  const int b = (int)(idx / HQ);
  const int r = (int)(idx % HQ) * VW;
  const size_t o4 = (size_t)b * 4 * a.H + r;
  const size_t o1 = (size_t)b * a.H + r;

  Vec<VW> g[4], c, cp, dh, dc, t;
#pragma unroll
  for (int k = 0; k < 4; ++k) g[k].load(a.gates + o4 + (size_t)k * a.H);
  c.load(a.c + o1);
  cp.load(a.c_prev + o1);
#pragma unroll
  for (int i = 0; i < VW; ++i) dh.v[i] = 0.f, dc.v[i] = 0.f;
  if (a.next.p) {
    load_term<VW>(a.next, b, r, &t);
#pragma unroll
    for (int i = 0; i < VW; ++i) dh.v[i] = clampf(t.v[i], a.clip_next);
  }
  if (a.above.p) {
    load_term<VW>(a.above, b, r, &t);
    if (a.above_drop_mask) {  // the layer above saw a dropped copy of h: same mask on the way back
      Vec<VW> u;
      u.load(a.above_drop_mask + o1);
      const float inv = 1.0f / a.keep;
#pragma unroll
      for (int i = 0; i < VW; ++i)
        dh.v[i] += clampf(t.v[i], a.clip_above) * (float)(a.keep > u.v[i]) * inv;
    } else {
#pragma unroll
      for (int i = 0; i < VW; ++i) dh.v[i] += clampf(t.v[i], a.clip_above);
    }
  }
  if (a.dc_next) dc.load(a.dc_next + o1);
  const float m = (float)a.mask01[b];

  Vec<VW> d[4], dcp;
#pragma unroll
  for (int i = 0; i < VW; ++i) {
    const float it = g[0].v[i], ft = g[1].v[i], gt = g[2].v[i], ot = g[3].v[i];
    const float tc = tanhf(c.v[i]);
    float dhv = dh.v[i];
    float dcv = dc.v[i] + dhv * ot * (1.0f - tc * tc);
    dhv *= m;
    dcv *= m;
    d[3].v[i] = dhv * tc * ot * (1.f - ot);
    d[1].v[i] = dcv * cp.v[i] * ft * (1.f - ft);
    d[2].v[i] = dcv * it * (1.f - gt * gt);
    d[0].v[i] = dcv * gt * it * (1.f - it);
    dcp.v[i] = dcv * ft;
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) d[k].store(a.dgates + o4 + (size_t)k * a.H);
  dcp.store(a.dc_prev + o1);
}

// ---------------------------------------------------------------------------------------------
// out[r] = beta * out[r] + sum_c A[r, c]   (A column-major rows x cols, leading dimension lda).
// A workgroup owns 16 rows: 16 x 16 threads, the 16 column phases are folded through LDS in a fixed
// order, so the result does not depend on scheduling.
constexpr int kRsRows = 16, kRsPhases = 16;
__global__ __launch_bounds__(256) void rowsum_kernel(const float *__restrict__ A, long long lda,
                                                     int rows, long long cols, float beta,
                                                     float *__restrict__ out) {
  __shared__ float s[kRsPhases][kRsRows + 1];
  const int lr = threadIdx.x % kRsRows, ph = threadIdx.x / kRsRows;
  const int r = blockIdx.x * kRsRows + lr;
  float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
  if (r < rows) {
    long long cidx = ph;
    for (; cidx + 3 * kRsPhases < cols; cidx += 4 * kRsPhases) {
      acc0 += A[cidx * lda + r];
      acc1 += A[(cidx + kRsPhases) * lda + r];
      acc2 += A[(cidx + 2 * kRsPhases) * lda + r];
      acc3 += A[(cidx + 3 * kRsPhases) * lda + r];
    }
    for (; cidx < cols; cidx += kRsPhases) acc0 += A[cidx * lda + r];
  }
  s[ph][lr] = (acc0 + acc1) + (acc2 + acc3);
  __syncthreads();
  if (ph == 0 && r < rows) {
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < kRsPhases; ++k) t += s[k][lr];
    out[r] = (beta != 0.f ? beta * out[r] : 0.f) + t;
  }
}

// ---------------------------------------------------------------------------------------------
// Embedding gradient: small_grad[:, k] (+)= sum over the dx columns listed for unique id k.
// Token frequencies are Zipfian: a few ids own thousands of columns, most own one.  A workgroup
// takes one id and a slab of 16 * VW rows; its 256 threads are 16 row lanes x 16 column phases,
// phase p adding up columns p, p + 16, ... of the id's list (four loads in flight per thread), and
// the 16 partial sums meet in LDS in phase order.  The order of the additions is fixed by the
// list alone (no atomics), so the result is the same from run to run.
constexpr int kEgLanes = 16, kEgPhases = 16;
template <int VW>
__global__ __launch_bounds__(256) void embed_gather_grad_kernel(
    const float *__restrict__ dx, long long ldx, int E, const int *__restrict__ seg_start,
    const int *__restrict__ seg_cols, const float *__restrict__ drop_mask, float keep, float beta,
    float *__restrict__ small_grad, long long ldg) {
  __shared__ float part[kEgPhases][kEgLanes * VW + 1];
  const int k = blockIdx.x;
  const int lane = threadIdx.x % kEgLanes, ph = threadIdx.x / kEgLanes;
  const int r = (blockIdx.y * kEgLanes + lane) * VW;
  const bool row_ok = r < E;
  const int s0 = seg_start[k], s1 = seg_start[k + 1];
  const float inv = drop_mask ? 1.0f / keep : 1.0f;
  Vec<VW> acc;
#pragma unroll
  for (int i = 0; i < VW; ++i) acc.v[i] = 0.f;
  if (row_ok) {
    auto add = [&](const Vec<VW> &t, const Vec<VW> &u) {
#pragma unroll
      for (int i = 0; i < VW; ++i)
        acc.v[i] += drop_mask ? t.v[i] * (float)(keep > u.v[i]) * inv : t.v[i];
    };
    int s = s0 + ph;
    for (; s + 3 * kEgPhases < s1; s += 4 * kEgPhases) {
      long long o[4];
      Vec<VW> t[4], u[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) o[q] = (long long)seg_cols[s + q * kEgPhases] * ldx + r;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        t[q].load(dx + o[q]);
        if (drop_mask) u[q].load(drop_mask + o[q]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) add(t[q], u[q]);
    }
    for (; s < s1; s += kEgPhases) {
      const long long o = (long long)seg_cols[s] * ldx + r;
      Vec<VW> t, u;
      t.load(dx + o);
      if (drop_mask) u.load(drop_mask + o);
      add(t, u);
    }
  }
#pragma unroll
  for (int i = 0; i < VW; ++i) part[ph][lane * VW + i] = acc.v[i];
  __syncthreads();
  if (ph != 0 || !row_ok) return;
#pragma unroll
  for (int i = 0; i < VW; ++i) {
    float t = 0.f;
#pragma unroll
    for (int q = 0; q < kEgPhases; ++q) t += part[q][lane * VW + i];
    acc.v[i] = t;
  }
  float *o = small_grad + (long long)k * ldg + r;
  if (beta != 0.f) {
    Vec<VW> t;
    t.load(o);
#pragma unroll
    for (int i = 0; i < VW; ++i) acc.v[i] += beta * t.v[i];
  }
  acc.store(o);
}

// ---------------------------------------------------------------------------------------------
// delta = (dht + clamp(dht_feed)) * mask * (1 - h_tild^2)
template <int VW>
__global__ __launch_bounds__(256) void attn_delta_kernel(int H, int B, const float *dht,
                                                         const float *dht_feed, const float *h_tild,
                                                         const int *mask01, float clip_feed,
                                                         float *delta) {
  const int HQ = H / VW;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)HQ * B) return;
  const int b = (int)(idx / HQ);
  const size_t o = (size_t)b * H + (size_t)(idx % HQ) * VW;
  Vec<VW> d, f, h;
  d.load(dht + o);
  h.load(h_tild + o);
  if (dht_feed) {
    f.load(dht_feed + o);
#pragma unroll
    for (int i = 0; i < VW; ++i) d.v[i] += clampf(f.v[i], clip_feed);
  }
  const float m = (float)mask01[b];
#pragma unroll
  for (int i = 0; i < VW; ++i) d.v[i] = (d.v[i] * m) * (1.f - h.v[i] * h.v[i]);
  d.store(delta + o);
}

// ---------------------------------------------------------------------------------------------
// Attention core backward, one workgroup (4 wavefronts) per column b.
constexpr int kMaxSlots = 512;
constexpr int kAT = 256;
constexpr int kAW = kAT / lh::kWave;

struct AttnBwdArgs {
  int H, B, D, W;
  const float *dctx, *tanh1, *v_p, *wa, *hs;
  long long step_stride, col_stride;
  int hs_steps;
  const int *batch_info;
  const float *p_t, *sigma;
  const int *indices;
  const float *align, *cached_exp;
  float *dhs, *hsum, *u, *w;
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
__global__ __launch_bounds__(kAT) void attn_core_bwd_kernel(const AttnBwdArgs a) {
  __shared__ int s_tau[kMaxSlots];
  __shared__ int s_idx[kMaxSlots];
  __shared__ float s_das[kMaxSlots];  // d alignment score, then das * a
  __shared__ float s_al[kMaxSlots];
  __shared__ float s_g[kMaxSlots];
  __shared__ float s_r[kMaxSlots];
  __shared__ float s_red[kAW];

  const int b = blockIdx.x, tid = threadIdx.x, wave = tid / lh::kWave, lane = tid % lh::kWave;
  const int H = a.H, B = a.B, W = a.W, D = a.D;
  const int len = a.batch_info[b], off = a.batch_info[B + b];
  const float *dctx = a.dctx + (size_t)b * H;
  const float *wa = a.wa + (size_t)b * H;
  const float *hs_c = a.hs + (size_t)b * a.col_stride;
  float *dhs_c = a.dhs + (size_t)b * a.col_stride;

  for (int j = tid; j < W; j += kAT) {
    const int idx = a.indices[b + (size_t)B * j];
    int tau = -1;
    if (idx >= 0) {
      tau = len - 1 - idx + off;
      if (tau < 0 || tau >= a.hs_steps) tau = -1;
    }
    s_idx[j] = idx;
    s_tau[j] = tau;
    s_al[j] = a.align[b + (size_t)B * j];
    s_g[j] = a.cached_exp[j + (size_t)W * b];
  }
  __syncthreads();

  // d score_j = dctx . hs_j
  for (int j = wave; j < W; j += kAW) {
    const int tau = s_tau[j];
    float v = 0.f;
    if (tau >= 0) v = dot_wave<VEC>(hs_c + (size_t)tau * a.step_stride, dctx, H, lane);
    if (lane == 0) s_das[j] = v;
  }
  __syncthreads();

  // d p_t and the softmax-with-Gaussian Jacobian
  float dp = 0.f;
  float sg = 0.f;
  if (D >= 0) {
    const float sigma_sq = (float)((D * D) / 4.0);
    const float p = a.p_t[b];
    float part = 0.f;
    for (int j = tid; j < W; j += kAT)
      part += s_das[j] * s_al[j] * (((float)s_idx[j] - p) / sigma_sq);
    dp = lh::block_sum<kAW>(part, s_red);
    sg = a.sigma[b];
  }
  // total = sum_k das_k a_k; r_j = das_j a_j - (a_j / g_j) * total
  float part = 0.f;
  for (int j = tid; j < W; j += kAT) part += s_das[j] * s_al[j];
  const float total = lh::block_sum<kAW>(part, s_red);
  for (int j = tid; j < W; j += kAT) {
    const float aj = s_al[j];
    s_r[j] = s_das[j] * aj - (aj / s_g[j]) * total;
  }
  __syncthreads();

  const float pcoef = dp * sg * (1.f - sg) * (float)len;
  constexpr int VW = VEC ? 4 : 1;
  for (int r = tid * VW; r < H; r += kAT * VW) {
    Vec<VW> dc, wv, hsum, t;
    dc.load(dctx + r);
    wv.load(wa + r);
#pragma unroll
    for (int i = 0; i < VW; ++i) hsum.v[i] = 0.f;
    for (int j = 0; j < W; ++j) {
      const int tau = s_tau[j];
      if (tau < 0) continue;
      const float rj = s_r[j], aj = s_al[j];
      t.load(hs_c + (size_t)tau * a.step_stride + r);
#pragma unroll
      for (int i = 0; i < VW; ++i) hsum.v[i] += t.v[i] * rj;
      float *dst = dhs_c + (size_t)tau * a.step_stride + r;
      t.load(dst);
#pragma unroll
      for (int i = 0; i < VW; ++i) t.v[i] += dc.v[i] * aj + wv.v[i] * rj;
      t.store(dst);
    }
    hsum.store(a.hsum + (size_t)b * H + r);
    if (D >= 0) {
      Vec<VW> t1, vp, uo, wo;
      t1.load(a.tanh1 + (size_t)b * H + r);
      vp.load(a.v_p + r);
#pragma unroll
      for (int i = 0; i < VW; ++i) {
        uo.v[i] = pcoef * t1.v[i];
        wo.v[i] = pcoef * vp.v[i] * (1.f - t1.v[i] * t1.v[i]);
      }
      uo.store(a.u + (size_t)b * H + r);
      wo.store(a.w + (size_t)b * H + r);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// accum[0] += sum (scale * g)^2 over a rows x cols view.  Each thread sums runs of up to 64 squares
// in float and adds the runs in double; a workgroup's threads are combined through a fixed-order
// LDS fold, and the workgroups' partials by one more workgroup, again in a fixed order: the result
// depends on the shape of the launch only.  VEC: the view is one contiguous, 16-byte aligned run,
// read as four-float vectors with four loads in flight per thread.
constexpr int kNT = 1024;
constexpr int kFoldNT = 256;
template <bool VEC>
__global__ __launch_bounds__(kNT) void sumsq_kernel(const float *__restrict__ g, long long rows,
                                                    long long cols, long long ld, float scale,
                                                    double *__restrict__ partial) {
  __shared__ double red[kNT / lh::kWave];
  const long long n = rows * cols;
  double acc = 0.0;
  if constexpr (VEC) {
    const long long n4 = n / 4, stride = (long long)gridDim.x * kNT;
    const float4 *g4 = reinterpret_cast<const float4 *>(g);
    long long i = (long long)blockIdx.x * kNT + threadIdx.x;
    for (; i + 3 * stride < n4; i += 4 * stride) {
      const float4 a = g4[i], b = g4[i + stride], c = g4[i + 2 * stride], d = g4[i + 3 * stride];
      float f = 0.f;
      const float va[16] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w, c.x, c.y, c.z, c.w, d.x, d.y, d.z, d.w};
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const float v = scale * va[k];
        f += v * v;
      }
      acc += (double)f;
    }
    float f = 0.f;
    for (; i < n4; i += stride) {
      const float4 a = g4[i];
      const float va[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float v = scale * va[k];
        f += v * v;
      }
    }
    if (blockIdx.x == 0 && threadIdx.x < (int)(n - 4 * n4)) {
      const float v = scale * g[4 * n4 + threadIdx.x];
      f += v * v;
    }
    acc += (double)f;
  } else {
    float facc = 0.f;
    int cnt = 0;
    for (long long i = (long long)blockIdx.x * kNT + threadIdx.x; i < n; i += (long long)gridDim.x * kNT) {
      long long o = i;
      if (cols != 1) {
        const long long c = i / rows;
        o = c * ld + (i - c * rows);
      }
      const float v = scale * g[o];
      facc += v * v;
      if (++cnt == 64) {
        acc += (double)facc;
        facc = 0.f;
        cnt = 0;
      }
    }
    acc += (double)facc;
  }
  const double s = lh::block_sum<kNT / lh::kWave>(acc, red);
  if (threadIdx.x == 0) partial[blockIdx.x] = s;
}
__global__ __launch_bounds__(kFoldNT) void sumsq_fold_kernel(const double *partial, int n, double *accum) {
  __shared__ double red[kFoldNT / lh::kWave];
  double s = 0.0;
  for (int i = threadIdx.x; i < n; i += kFoldNT) s += partial[i];
  s = lh::block_sum<kFoldNT / lh::kWave>(s, red);
  if (threadIdx.x == 0) accum[0] += s;
}

// theta(:, col(c)) += lr * f * clamp(scale * g(:, c)),  g = 0
//   f = sumsq ? (sqrt(*sumsq) > norm_clip ? norm_clip / sqrt(*sumsq) : 1) : 1
__global__ __launch_bounds__(256) void sgd_step_kernel(float *__restrict__ theta, long long ld_theta,
                                                       float *__restrict__ g, long long ld_g,
                                                       long long rows, long long cols,
                                                       const int *__restrict__ col_index, float lr,
                                                       float scale, const double *sumsq,
                                                       float norm_clip, float individual_clip) {
  float f = 1.f;
  if (sumsq) {
    const float nrm = (float)sqrt(sumsq[0]);
    if (nrm > norm_clip) f = norm_clip / nrm;
  }
  const long long n = rows * cols;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    long long og = i, ot = i;
    if (cols != 1 || col_index) {
      const long long c = i / rows, r = i - c * rows;
      const long long tc = col_index ? (long long)col_index[c] : c;
      og = c * ld_g + r;
      ot = tc * ld_theta + r;
    }
    float v = scale * g[og];
    v = f * v;
    v = clampf(v, individual_clip);
    theta[ot] += lr * v;
    g[og] = 0.f;
  }
}

// ---------------------------------------------------------------------------------------------
// Counter-based uniform numbers in (0, 1]: element i is a fixed function of (seed, i), so a mask can
// be regenerated and does not depend on the launch shape.
__device__ __forceinline__ unsigned long long mix64(unsigned long long z) {
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
  return z ^ (z >> 31);
}
__global__ __launch_bounds__(256) void uniform_kernel(float *out, long long n,
                                                      unsigned long long seed) {
  const unsigned long long base = mix64(seed + 0x9e3779b97f4a7c15ULL);
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const unsigned long long r = mix64(base + (unsigned long long)i * 0x9e3779b97f4a7c15ULL);
    out[i] = ((float)(unsigned)(r >> 40) + 1.0f) * (1.0f / 16777216.0f);  // 24 bits -> (0, 1]
  }
}

}  // namespace

extern "C" int lh_uniform_f32(float *out, long long n, unsigned long long seed, lh_stream_t stream) {
  if (n < 0 || (n > 0 && !out)) return lh::fail_arg("lh_uniform_f32: n=%lld or NULL pointer", n);
  if (n == 0) return LH_OK;
  long long blocks = (n + 256 * 8 - 1) / (256 * 8);
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(uniform_kernel, dim3((unsigned)blocks), dim3(256), 0, lh::as_stream(stream), out,
                     n, seed);
  return lh::check_launch("lh_uniform_f32");
}

namespace {
// NULL / empty terms become {NULL}; false = malformed
bool normal_term(const lh_error_term *in, int H, lh_error_term *out, bool *vec) {
  *out = lh_error_term{nullptr, 1, 0, H};
  if (!in || !in->p) return true;
  if (in->planes < 1 || in->planes > LH_ERROR_TERM_MAX_PLANES || in->ld < H) return false;
  if (in->planes > 1 && in->plane_stride <= 0) return false;
  *out = *in;
  if (in->planes == 1) out->plane_stride = 0;
  if (!lh::aligned16(in->p) || in->ld % 4 || (in->planes > 1 && in->plane_stride % 4)) *vec = false;
  return true;
}
}  // namespace

extern "C" int lh_lstm_cell_bwd_terms_f32(int H, int B, const lh_error_term *above,
                                          const lh_error_term *next, const float *dc_next,
                                          const float *gates, const float *c, const float *c_prev,
                                          const int *mask01, float clip_above, float clip_next,
                                          const float *above_drop_mask, float keep, float *dgates,
                                          float *dc_prev, lh_stream_t stream) {
  if (H <= 0 || B <= 0) return lh::fail_arg("lh_lstm_cell_bwd_f32: H=%d B=%d", H, B);
  if (!gates || !c || !c_prev || !mask01 || !dgates || !dc_prev)
    return lh::fail_arg("lh_lstm_cell_bwd_f32: a required pointer is NULL");
  bool vec = H % 4 == 0 && lh::aligned16(dc_next) && lh::aligned16(gates) && lh::aligned16(c) &&
             lh::aligned16(c_prev) && lh::aligned16(dgates) && lh::aligned16(dc_prev) &&
             lh::aligned16(above_drop_mask);
  lh_error_term ta, tn;
  if (!normal_term(above, H, &ta, &vec) || !normal_term(next, H, &tn, &vec))
    return lh::fail_arg("lh_lstm_cell_bwd_f32: an error term needs 1..%d planes, ld >= H and a positive plane stride",
                        LH_ERROR_TERM_MAX_PLANES);
  if (above_drop_mask && (!ta.p || !(keep > 0.f)))
    return lh::fail_arg("lh_lstm_cell_bwd_f32: above_drop_mask needs dh_above and keep > 0");
  CellBwdArgs a{H, B, ta, tn, dc_next, gates, c, c_prev, mask01, clip_above, clip_next,
                above_drop_mask, keep, dgates, dc_prev};
  const long long work = (long long)(vec ? H / 4 : H) * B;
  const dim3 grid((unsigned)((work + 255) / 256)), block(256);
  hipStream_t st = lh::as_stream(stream);
  if (vec) hipLaunchKernelGGL(lstm_cell_bwd_kernel<4>, grid, block, 0, st, a);
  else hipLaunchKernelGGL(lstm_cell_bwd_kernel<1>, grid, block, 0, st, a);
  return lh::check_launch("lh_lstm_cell_bwd_f32");
}

extern "C" int lh_lstm_cell_bwd_f32(int H, int B, const float *dh_above, const float *dh_next,
                                    const float *dc_next, const float *gates, const float *c,
                                    const float *c_prev, const int *mask01, float clip_above,
                                    float clip_next, const float *above_drop_mask, float keep,
                                    float *dgates, float *dc_prev, lh_stream_t stream) {
  const lh_error_term above{dh_above, 1, 0, H}, next{dh_next, 1, 0, H};
  return lh_lstm_cell_bwd_terms_f32(H, B, &above, &next, dc_next, gates, c, c_prev, mask01, clip_above,
                                    clip_next, above_drop_mask, keep, dgates, dc_prev, stream);
}

extern "C" int lh_rowsum_acc_f32(const float *A, long long lda, int rows, long long cols,
                                 float beta, float *out, lh_stream_t stream) {
  if (rows <= 0 || cols < 0 || !A || !out || lda < rows)
    return lh::fail_arg("lh_rowsum_acc_f32: rows=%d cols=%lld lda=%lld or NULL pointer", rows, cols,
                        lda);
  hipLaunchKernelGGL(rowsum_kernel, dim3((rows + kRsRows - 1) / kRsRows), dim3(256), 0,
                     lh::as_stream(stream), A, lda, rows, cols, beta, out);
  return lh::check_launch("lh_rowsum_acc_f32");
}

extern "C" int lh_embed_gather_grad_f32(const float *dx, long long ldx, int E, int n_unique,
                                        const int *seg_start, const int *seg_cols,
                                        const float *drop_mask, float keep, float beta,
                                        float *small_grad, long long ldg, lh_stream_t stream) {
  if (E <= 0 || n_unique < 0 || !dx || !seg_start || !seg_cols || !small_grad || ldx < E || ldg < E)
    return lh::fail_arg("lh_embed_gather_grad_f32: E=%d n_unique=%d ldx=%lld ldg=%lld or NULL pointer",
                        E, n_unique, ldx, ldg);
  if (n_unique == 0) return LH_OK;
  if (drop_mask && !(keep > 0.f)) return lh::fail_arg("lh_embed_gather_grad_f32: keep must be > 0");
  const bool vec = E % 4 == 0 && ldx % 4 == 0 && ldg % 4 == 0 && lh::aligned16(dx) &&
                   lh::aligned16(small_grad) && lh::aligned16(drop_mask);
  hipStream_t st = lh::as_stream(stream);
  if (vec)
    hipLaunchKernelGGL(embed_gather_grad_kernel<4>, dim3(n_unique, (E / 4 + kEgLanes - 1) / kEgLanes),
                       dim3(256), 0, st, dx, ldx, E, seg_start, seg_cols, drop_mask, keep, beta, small_grad, ldg);
  else
    hipLaunchKernelGGL(embed_gather_grad_kernel<1>, dim3(n_unique, (E + kEgLanes - 1) / kEgLanes),
                       dim3(256), 0, st, dx, ldx, E, seg_start, seg_cols, drop_mask, keep, beta, small_grad, ldg);
  return lh::check_launch("lh_embed_gather_grad_f32");
}

extern "C" int lh_attn_delta_f32(int H, int B, const float *dht, const float *dht_feed,
                                 const float *h_tild, const int *mask01, float clip_feed,
                                 float *delta, lh_stream_t stream) {
  if (H <= 0 || B <= 0 || !dht || !h_tild || !mask01 || !delta)
    return lh::fail_arg("lh_attn_delta_f32: H=%d B=%d or NULL pointer", H, B);
  const bool vec = H % 4 == 0 && lh::aligned16(dht) && lh::aligned16(dht_feed) &&
                   lh::aligned16(h_tild) && lh::aligned16(delta);
  const long long work = (long long)(vec ? H / 4 : H) * B;
  const dim3 grid((unsigned)((work + 255) / 256)), block(256);
  hipStream_t st = lh::as_stream(stream);
  if (vec)
    hipLaunchKernelGGL(attn_delta_kernel<4>, grid, block, 0, st, H, B, dht, dht_feed, h_tild, mask01,
                       clip_feed, delta);
  else
    hipLaunchKernelGGL(attn_delta_kernel<1>, grid, block, 0, st, H, B, dht, dht_feed, h_tild, mask01,
                       clip_feed, delta);
  return lh::check_launch("lh_attn_delta_f32");
}

extern "C" int lh_attn_core_bwd_f32(int H, int B, int D, int max_len, int hs_steps,
                                    const float *dctx, const float *tanh1, const float *v_p,
                                    const float *wa, const float *hs, long long hs_step_stride,
                                    long long hs_col_stride, const int *batch_info,
                                    const float *p_t, const float *sigma, const int *indices,
                                    const float *align, const float *cached_exp, float *dhs,
                                    float *hsum, float *u, float *w, lh_stream_t stream) {
  if (H <= 0 || B <= 0 || hs_steps <= 0)
    return lh::fail_arg("lh_attn_core_bwd_f32: H=%d B=%d hs_steps=%d", H, B, hs_steps);
  const int W = D >= 0 ? 2 * D + 1 : max_len;
  if (W <= 0 || W > kMaxSlots)
    return lh::fail_arg("lh_attn_core_bwd_f32: window of %d slots outside [1,%d]", W, kMaxSlots);
  if (!dctx || !wa || !hs || !batch_info || !indices || !align || !cached_exp || !dhs || !hsum)
    return lh::fail_arg("lh_attn_core_bwd_f32: a required pointer is NULL");
  if (D >= 0 && (!tanh1 || !v_p || !p_t || !sigma || !u || !w))
    return lh::fail_arg("lh_attn_core_bwd_f32: local-p needs tanh1, v_p, p_t, sigma, u and w");
  if (hs_step_stride < 0 || hs_col_stride < H)
    return lh::fail_arg("lh_attn_core_bwd_f32: columns of the state buffer must not overlap");
  AttnBwdArgs a{H, B, D, W, dctx, tanh1, v_p, wa, hs, hs_step_stride, hs_col_stride, hs_steps,
                batch_info, p_t, sigma, indices, align, cached_exp, dhs, hsum, u, w};
  const bool vec = H % 4 == 0 && lh::aligned16(dctx) && lh::aligned16(wa) && lh::aligned16(hs) &&
                   lh::aligned16(dhs) && lh::aligned16(hsum) && lh::aligned16(tanh1) &&
                   lh::aligned16(v_p) && lh::aligned16(u) && lh::aligned16(w) &&
                   hs_step_stride % 4 == 0 && hs_col_stride % 4 == 0;
  hipStream_t st = lh::as_stream(stream);
  if (vec) hipLaunchKernelGGL(attn_core_bwd_kernel<true>, dim3(B), dim3(kAT), 0, st, a);
  else hipLaunchKernelGGL(attn_core_bwd_kernel<false>, dim3(B), dim3(kAT), 0, st, a);
  return lh::check_launch("lh_attn_core_bwd_f32");
}

extern "C" int lh_grad_sumsq_f32(const float *g, long long rows, long long cols, long long ld,
                                 float scale, double *workspace, double *accum,
                                 lh_stream_t stream) {
  if (rows <= 0 || cols < 0 || !g || !workspace || !accum || ld < rows)
    return lh::fail_arg("lh_grad_sumsq_f32: rows=%lld cols=%lld ld=%lld or NULL pointer", rows, cols,
                        ld);
  if (cols == 0) return LH_OK;
  const long long n = rows * cols;
  if (ld == rows) {  // contiguous: one long column, no index arithmetic in the kernel
    rows = n;
    cols = 1;
    ld = n;
  }
  long long blocks = (n + (long long)kNT * 16 - 1) / ((long long)kNT * 16);
  if (blocks > LH_SUMSQ_WORKSPACE) blocks = LH_SUMSQ_WORKSPACE;
  hipStream_t st = lh::as_stream(stream);
  if (cols == 1 && lh::aligned16(g))
    hipLaunchKernelGGL(sumsq_kernel<true>, dim3((unsigned)blocks), dim3(kNT), 0, st, g, rows, cols, ld,
                       scale, workspace);
  else
    hipLaunchKernelGGL(sumsq_kernel<false>, dim3((unsigned)blocks), dim3(kNT), 0, st, g, rows, cols, ld,
                       scale, workspace);
  int rc = lh::check_launch("lh_grad_sumsq_f32");
  if (rc != LH_OK) return rc;
  hipLaunchKernelGGL(sumsq_fold_kernel, dim3(1), dim3(kFoldNT), 0, st, workspace, (int)blocks, accum);
  return lh::check_launch("lh_grad_sumsq_f32 (fold)");
}

extern "C" int lh_sgd_step_f32(float *theta, long long ld_theta, float *g, long long ld_g,
                               long long rows, long long cols, const int *col_index,
                               float learning_rate, float grad_scale, const double *sumsq,
                               float norm_clip, float individual_clip, lh_stream_t stream) {
  if (rows <= 0 || cols < 0 || !theta || !g || ld_theta < rows || ld_g < rows)
    return lh::fail_arg("lh_sgd_step_f32: rows=%lld cols=%lld ld_theta=%lld ld_g=%lld or NULL pointer",
                        rows, cols, ld_theta, ld_g);
  if (sumsq && !(norm_clip > 0.f)) return lh::fail_arg("lh_sgd_step_f32: norm_clip must be > 0");
  if (cols == 0) return LH_OK;
  const long long n = rows * cols;
  if (!col_index && ld_theta == rows && ld_g == rows) {
    rows = n;
    cols = 1;
    ld_theta = ld_g = n;
  }
  long long blocks = (n + 256 * 8 - 1) / (256 * 8);
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(sgd_step_kernel, dim3((unsigned)blocks), dim3(256), 0, lh::as_stream(stream),
                     theta, ld_theta, g, ld_g, rows, cols, col_index, learning_rate, grad_scale,
                     sumsq, norm_clip, individual_clip);
  return lh::check_launch("lh_sgd_step_f32");
}
