// Vocabulary softmax / log-likelihood / fused log-softmax + top-K.
//
// One workgroup of 1024 threads (16 wavefronts) owns one column of the V x B logits.  The column is
// read from HBM exactly once with 16-byte loads and stays in registers (NV float4 per thread, chosen
// so that 4096*NV >= V) through the max, exp-sum and the final normalisation / selection, so the
// traffic is the algorithmic minimum: V*B*4 bytes in, plus V*B*4 out only for the kernel that has to
// hand back probabilities.  Columns that are not 16-byte aligned or longer than 65536 rows take a
// generic strided kernel that re-reads the column (from L2) instead.
#include "lh_common.h"

namespace {

constexpr int kT = 1024;
constexpr int kNW = kT / lh::kWave;
constexpr float kNegInf = -__builtin_huge_valf();

__device__ __forceinline__ float &comp(float4 &v, int c) {
  return c == 0 ? v.x : (c == 1 ? v.y : (c == 2 ? v.z : v.w));
}

// Loads column `col` (+bias) into registers; rows >= V read as -inf.
template <int NV>
__device__ __forceinline__ void load_column(float4 (&x)[NV], const float *__restrict__ col,
                                            const float *__restrict__ bias, int V, int tid) {
  const int V4 = V / 4;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int f = tid + i * kT;
    float4 v = make_float4(kNegInf, kNegInf, kNegInf, kNegInf);
    if (f < V4) {
      v = reinterpret_cast<const float4 *>(col)[f];
      if (bias) {
        const float4 bb = reinterpret_cast<const float4 *>(bias)[f];
        v.x += bb.x; v.y += bb.y; v.z += bb.z; v.w += bb.w;
      }
    }
    x[i] = v;
  }
}

template <int NV>
__device__ __forceinline__ float local_max(const float4 (&x)[NV]) {
  float m = kNegInf;
#pragma unroll
  for (int i = 0; i < NV; ++i) m = fmaxf(fmaxf(fmaxf(m, x[i].x), fmaxf(x[i].y, x[i].z)), x[i].w);
  return m;
}

// exp for the bandwidth-bound passes: one multiply + v_exp_f32 instead of expf's range handling.
// The argument is <= 0 here (max already subtracted), so there is no overflow; the result is within
// ~|x| * 2^-24 relative of expf, far inside the tolerance of the probabilities and log-sums.
__device__ __forceinline__ float exp_neg(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269504088896341f);
}

// ---- probabilities out ----------------------------------------------------------------------
template <int NV>
__global__ __launch_bounds__(kT, (NV <= 8 ? 8 : 4)) void softmax_fwd_kernel(const float *__restrict__ logits, int ldl,
                                                         const float *__restrict__ bias, int V,
                                                         float *__restrict__ p, int ldp) {
  __shared__ float red[kNW];
  const int b = blockIdx.x, tid = threadIdx.x;
  float4 x[NV];
  load_column<NV>(x, logits + (size_t)b * ldl, bias, V, tid);
  const float mx = lh::block_max<kNW>(local_max<NV>(x), red);
  float part = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    x[i].x = exp_neg(x[i].x - mx); x[i].y = exp_neg(x[i].y - mx);
    x[i].z = exp_neg(x[i].z - mx); x[i].w = exp_neg(x[i].w - mx);
    part += (x[i].x + x[i].y) + (x[i].z + x[i].w);
  }
  const float sum = lh::block_sum<kNW>(part, red);
  float4 *out = reinterpret_cast<float4 *>(p + (size_t)b * ldp);
  const int V4 = V / 4;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int f = tid + i * kT;
    if (f < V4) out[f] = make_float4(x[i].x / sum, x[i].y / sum, x[i].z / sum, x[i].w / sum);
  }
}

// Generic fallback: any V / alignment, column re-read twice.
__global__ __launch_bounds__(kT) void softmax_fwd_generic_kernel(const float *logits, int ldl,
                                                                 const float *bias, int V, float *p,
                                                                 int ldp) {
  __shared__ float red[kNW];
  const int b = blockIdx.x, tid = threadIdx.x;
  const float *col = logits + (size_t)b * ldl;
  float *out = p + (size_t)b * ldp;
  float m = kNegInf;
  for (int r = tid; r < V; r += kT) m = fmaxf(m, col[r] + (bias ? bias[r] : 0.f));
  const float mx = lh::block_max<kNW>(m, red);
  float part = 0.f;
  for (int r = tid; r < V; r += kT) {
    const float e = expf(col[r] + (bias ? bias[r] : 0.f) - mx);
    out[r] = e;  // p may alias logits: row r is only ever touched by this thread
    part += e;
  }
  const float sum = lh::block_sum<kNW>(part, red);
  for (int r = tid; r < V; r += kT) out[r] = out[r] / sum;
}

// ---- training log-likelihood from probabilities (serial, column order, like the reference) ------
__global__ void train_loglik_kernel(const float *p, int ldp, int B, const int *tgt0,
                                    const int *mask01, double *accum) {
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  double acc = accum[0];
  for (int b = 0; b < B; ++b)
    if (mask01[b] == 1) acc += log((double)p[(size_t)b * ldp + tgt0[b]]);
  accum[0] = acc;
}

// ---- double-precision log-softmax of the target row -----------------------------------------
template <int NV>
__global__ __launch_bounds__(kT, (NV <= 8 ? 8 : 4)) void logsoftmax_tgt_kernel(const float *__restrict__ logits,
                                                            int ldl, const float *__restrict__ bias,
                                                            int V, const int *__restrict__ tgt0,
                                                            double *__restrict__ logp_tgt) {
  __shared__ float redf[kNW];
  __shared__ double redd[kNW];
  const int b = blockIdx.x, tid = threadIdx.x;
  float4 x[NV];
  load_column<NV>(x, logits + (size_t)b * ldl, bias, V, tid);
  const float mxf = lh::block_max<kNW>(local_max<NV>(x), redf);
  const double mx = (double)mxf;
  // Every exponential is taken in single precision (one v_exp_f32; a double exp per element made
  // this kernel compute-bound at a third of the memory rate) and the sum is carried in double:
  // four terms are added in float, then the partial sums in double.  Each term is within 2^-23
  // relative of the double value and the errors are independent, so log(sum) moves by ~1e-7,
  // two orders inside the 1e-5 tolerance of a log-probability.
  double part = 0.0;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    // rows >= V hold -inf and add exp(-inf) = 0
    const float e = (exp_neg(x[i].x - mxf) + exp_neg(x[i].y - mxf)) +
                    (exp_neg(x[i].z - mxf) + exp_neg(x[i].w - mxf));
    part += (double)e;
  }
  const double sum = lh::block_sum<kNW>(part, redd);
  const int t = tgt0[b];
  const int f = t / 4, c = t % 4;
  if (f % kT == tid && t < V) {
    const int i = f / kT;
    float zt = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k)
      if (k == i) zt = comp(x[k], c);
    logp_tgt[b] = log(exp((double)zt - mx)) - log(sum);
  }
}

__global__ __launch_bounds__(kT) void logsoftmax_tgt_generic_kernel(const float *logits, int ldl,
                                                                    const float *bias, int V,
                                                                    const int *tgt0,
                                                                    double *logp_tgt) {
  __shared__ float redf[kNW];
  __shared__ double redd[kNW];
  const int b = blockIdx.x, tid = threadIdx.x;
  const float *col = logits + (size_t)b * ldl;
  float m = kNegInf;
  for (int r = tid; r < V; r += kT) m = fmaxf(m, col[r] + (bias ? bias[r] : 0.f));
  const double mx = (double)lh::block_max<kNW>(m, redf);
  double part = 0.0;
  for (int r = tid; r < V; r += kT) part += exp((double)(col[r] + (bias ? bias[r] : 0.f)) - mx);
  const double sum = lh::block_sum<kNW>(part, redd);
  if (tid == 0) {
    const int t = tgt0[b];
    if (t >= 0 && t < V) {
      const float zt = col[t] + (bias ? bias[t] : 0.f);
      logp_tgt[b] = log(exp((double)zt - mx)) - log(sum);
    }
  }
}

// ---- training: output error (onehot - p) * mask and log p(target) in one pass ---------------
// dz may alias logits: a column is fully in registers (or each row is owned by one thread) before
// anything is written.
template <int NV>
__global__ __launch_bounds__(kT, (NV <= 8 ? 8 : 4)) void softmax_xent_grad_kernel(
    const float *__restrict__ logits, int ldl, const float *__restrict__ bias, int V,
    const int *__restrict__ tgt0, const int *__restrict__ mask01, float *dz, int ldz,
    double *__restrict__ logp_tgt) {
  __shared__ float red[kNW];
  const int b = blockIdx.x, tid = threadIdx.x;
  float4 x[NV];
  load_column<NV>(x, logits + (size_t)b * ldl, bias, V, tid);
  const float mx = lh::block_max<kNW>(local_max<NV>(x), red);
  float part = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    x[i].x = exp_neg(x[i].x - mx); x[i].y = exp_neg(x[i].y - mx);
    x[i].z = exp_neg(x[i].z - mx); x[i].w = exp_neg(x[i].w - mx);
    part += (x[i].x + x[i].y) + (x[i].z + x[i].w);
  }
  const float sum = lh::block_sum<kNW>(part, red);
  const float m = (float)mask01[b];
  const int t = tgt0[b];
  float4 *out = reinterpret_cast<float4 *>(dz + (size_t)b * ldz);
  const int V4 = V / 4;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int f = tid + i * kT;
    if (f < V4) {
      float4 p = make_float4(x[i].x / sum, x[i].y / sum, x[i].z / sum, x[i].w / sum);
      float4 d = make_float4(-p.x * m, -p.y * m, -p.z * m, -p.w * m);
      if (t / 4 == f) {
        const int c = t % 4;
        const float pt = c == 0 ? p.x : (c == 1 ? p.y : (c == 2 ? p.z : p.w));
        logp_tgt[b] = log((double)pt);
        d.x += c == 0 ? m : 0.f;
        d.y += c == 1 ? m : 0.f;
        d.z += c == 2 ? m : 0.f;
        d.w += c == 3 ? m : 0.f;
      }
      out[f] = d;
    }
  }
}

__global__ __launch_bounds__(kT) void softmax_xent_grad_generic_kernel(
    const float *logits, int ldl, const float *bias, int V, const int *tgt0, const int *mask01,
    float *dz, int ldz, double *logp_tgt) {
  __shared__ float red[kNW];
  const int b = blockIdx.x, tid = threadIdx.x;
  const float *col = logits + (size_t)b * ldl;
  float *out = dz + (size_t)b * ldz;
  float mxl = kNegInf;
  for (int r = tid; r < V; r += kT) mxl = fmaxf(mxl, col[r] + (bias ? bias[r] : 0.f));
  const float mx = lh::block_max<kNW>(mxl, red);
  float part = 0.f;
  for (int r = tid; r < V; r += kT) {
    const float e = expf(col[r] + (bias ? bias[r] : 0.f) - mx);
    out[r] = e;
    part += e;
  }
  const float sum = lh::block_sum<kNW>(part, red);
  const float m = (float)mask01[b];
  const int t = tgt0[b];
  for (int r = tid; r < V; r += kT) {
    const float p = out[r] / sum;
    float d = -p * m;
    if (r == t) {
      logp_tgt[b] = log((double)p);
      d += m;
    }
    out[r] = d;
  }
}

// accum[0] += sum of logp_tgt over unmasked columns: one 1024-thread workgroup, strided partial
// sums folded in a fixed order (double, so the order is immaterial at the tolerance of the loss).
__global__ __launch_bounds__(kT) void masked_sum_kernel(const double *logp_tgt, const int *mask01,
                                                        int B, double *accum) {
  __shared__ double redd[kNW];
  double acc = 0.0;
  for (int b = threadIdx.x; b < B; b += kT)
    if (mask01[b] == 1) acc += logp_tgt[b];
  const double s = lh::block_sum<kNW>(acc, redd);
  if (threadIdx.x == 0) accum[0] += s;
}

// ---- fused log-softmax + per-column top-K ---------------------------------------------------
struct Best {
  float v;
  int id;
};
__device__ __forceinline__ bool beats(float v1, int i1, float v2, int i2) {
  return v1 > v2 || (v1 == v2 && i1 < i2);
}
__device__ __forceinline__ Best wave_argmax(Best x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(x.v, o, lh::kWave);
    const int oi = __shfl_xor(x.id, o, lh::kWave);
    if (beats(ov, oi, x.v, x.id)) {
      x.v = ov;
      x.id = oi;
    }
  }
  return x;
}

constexpr int kIdNone = 0x7fffffff;

// Selection without arg-max rounds over the whole column.  Any threshold tau with at least K
// elements >= tau contains the true top K among the elements >= tau; those are collected into a
// short LDS list and ranked by counting (rank r < K is output slot r) under the strict total order
// (value desc, vocab id asc), which is what K rounds of arg-max with lowest-id tie breaking give.
//   fast path: tau = K-th largest of G group maxima (G = 16 wavefronts for K <= 16, else 64
//     quarter-wavefronts): K groups hold an element >= tau.  Values only, a few instructions per
//     element; the list has a few dozen entries on ordinary logits.
//   exact path (list overflow: massive ties, winners packed into one group): per-thread bests with
//     ids, the K best of each wavefront's 64 thread-bests, tau = K-th best of those 16*K survivors
//     as a (value, id) pair.  Never more than K*NV*4 <= kListCap elements pass it.
constexpr int kListCap = 4096;

template <int NV>
__device__ __forceinline__ void collect(const float4 (&x)[NV], int tid, int V, float tv, int ti,
                                        float *l_v, int *l_id, int *count) {
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int base = (tid + i * kT) * 4;
    const float m4 = fmaxf(fmaxf(x[i].x, x[i].y), fmaxf(x[i].z, x[i].w));
    if (m4 >= tv) {  // rare: most float4 hold nothing near the threshold
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float v = c == 0 ? x[i].x : (c == 1 ? x[i].y : (c == 2 ? x[i].z : x[i].w));
        const int id = base + c;
        if (id < V && !beats(tv, ti, v, id)) {
          const int pos = atomicAdd(count, 1);
          if (pos < kListCap) {
            l_v[pos] = v;
            l_id[pos] = id;
          }
        }
      }
    }
  }
}

// The distributions of several models, for EnsembleFactory::EnsemblesModels (src/decoder.h:1910-1931).
struct EnsembleArgs {
  const float *p[LH_ENSEMBLE_MAX_MODELS];
  int n_models;
};

// ENS = false: the column is logits (+bias) of one model and a candidate's score is its
// log-softmax.  ENS = true: the column is the mean over the models of their probabilities (summed
// in double, like the reference) and a candidate's score is log(mean / sum of the column's means).
template <int NV, bool ENS>
__device__ __forceinline__ void beam_topk_body(
    const float *__restrict__ logits, int ldl, const float *__restrict__ bias,
    const EnsembleArgs &ens, int V, int K, int eof_id, float *__restrict__ cand_logp,
    int *__restrict__ cand_id, float *__restrict__ logp_eof) {
  __shared__ float red[kNW];
  __shared__ float s_v[kT];
  __shared__ int s_id[kT];
  __shared__ float q_v[kT];  // exact path: survivors, kNW * K <= kT entries
  __shared__ int q_id[kT];
  __shared__ float l_v[kListCap];
  __shared__ int l_id[kListCap];
  __shared__ int s_count, s_tau_id;
  __shared__ float s_tau_v;
  const int b = blockIdx.x, tid = threadIdx.x;
  const int wave = tid / lh::kWave;
  float4 x[NV];
  float tmax, mx = 0.f, lse = 0.f, norm = 1.f;
  if constexpr (!ENS) {
    load_column<NV>(x, logits + (size_t)b * ldl, bias, V, tid);
    tmax = local_max<NV>(x);
    mx = lh::block_max<kNW>(tmax, red);
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
      part += (exp_neg(x[i].x - mx) + exp_neg(x[i].y - mx)) + (exp_neg(x[i].z - mx) + exp_neg(x[i].w - mx));
    lse = logf(lh::block_sum<kNW>(part, red));
  } else {
    const int V4 = V / 4;
    const double n = (double)ens.n_models;
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int f = tid + i * kT;
      float4 v = make_float4(kNegInf, kNegInf, kNegInf, kNegInf);  // rows >= V are never candidates
      if (f < V4) {
        double s0 = 0, s1 = 0, s2 = 0, s3 = 0;
        for (int m = 0; m < ens.n_models; ++m) {
          const float4 t = reinterpret_cast<const float4 *>(ens.p[m] + (size_t)b * ldl)[f];
          s0 += t.x, s1 += t.y, s2 += t.z, s3 += t.w;
        }
        v = make_float4((float)(s0 / n), (float)(s1 / n), (float)(s2 / n), (float)(s3 / n));
        part += (v.x + v.y) + (v.z + v.w);
      }
      x[i] = v;
    }
    tmax = local_max<NV>(x);
    norm = lh::block_sum<kNW>(part, red);
  }
  // a candidate's score from its value in x
  auto score_of = [&](float v) { return ENS ? logf(v / norm) : (v - mx) - lse; };

  if (eof_id >= 0 && eof_id < V && (eof_id / 4) % kT == tid) {
    const int i = (eof_id / 4) / kT, c = eof_id % 4;
    float z = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k)
      if (k == i) z = comp(x[k], c);
    logp_eof[b] = score_of(z);
  }

  // ---- fast path: threshold from group maxima ----------------------------------------------
  {
    const int G = K <= 16 ? kNW : 64;
    const int gs = kT / G;  // 64 or 16 lanes
    float gm = tmax;
    for (int o = gs / 2; o > 0; o >>= 1) gm = fmaxf(gm, __shfl_xor(gm, o, lh::kWave));
    if (tid % gs == 0) s_v[tid / gs] = gm;
    if (tid == 0) s_count = 0;
    __syncthreads();
    if (tid < G) {
      const float mine = s_v[tid];
      int rank = 0;
      for (int q = 0; q < G; ++q) rank += (s_v[q] > mine || (s_v[q] == mine && q < tid)) ? 1 : 0;
      if (rank == K - 1) s_tau_v = mine;
    }
    __syncthreads();
    collect<NV>(x, tid, V, s_tau_v, kIdNone, l_v, l_id, &s_count);  // every element >= tau
    __syncthreads();
  }
  if (s_count > kListCap) {
    // ---- exact path ---------------------------------------------------------------------------
    // thread best; a thread without a finite value gets a unique id above every vocabulary id so
    // that the order stays strict
    Best me{kNegInf, 0x40000000 + tid};
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int base = (tid + i * kT) * 4;  // ids grow with i and c: strict > keeps the lowest id
      if (x[i].x > me.v) { me.v = x[i].x; me.id = base; }
      if (x[i].y > me.v) { me.v = x[i].y; me.id = base + 1; }
      if (x[i].z > me.v) { me.v = x[i].z; me.id = base + 2; }
      if (x[i].w > me.v) { me.v = x[i].w; me.id = base + 3; }
    }
    __syncthreads();
    s_v[tid] = me.v;
    s_id[tid] = me.id;
    if (tid == 0) s_count = 0;
    __syncthreads();
    {  // rank inside the wavefront, keep ranks < K
      int rank = 0;
      const int w0 = wave * lh::kWave;
#pragma unroll 8
      for (int q = 0; q < lh::kWave; ++q) rank += beats(s_v[w0 + q], s_id[w0 + q], me.v, me.id) ? 1 : 0;
      if (rank < K) {
        q_v[wave * K + rank] = me.v;
        q_id[wave * K + rank] = me.id;
      }
    }
    __syncthreads();
    {  // the K-th best of the kNW*K survivors, comparisons of one survivor split over `parts` threads
      const int total = kNW * K;
      const int parts = kT / total;  // >= 1 because K <= 64
      if (tid < total) s_id[tid] = 0;  // thread bests no longer needed: reuse as rank counters
      __syncthreads();
      const int e = tid / parts, p = tid - e * parts;
      if (e < total) {
        const float v = q_v[e];
        const int id = q_id[e];
        int cnt = 0;
#pragma unroll 4
        for (int q = p; q < total; q += parts) cnt += beats(q_v[q], q_id[q], v, id) ? 1 : 0;
        if (cnt) atomicAdd(&s_id[e], cnt);
      }
      __syncthreads();
      if (tid < total && s_id[tid] == K - 1) {
        s_tau_v = q_v[tid];
        s_tau_id = q_id[tid];
      }
    }
    __syncthreads();
    collect<NV>(x, tid, V, s_tau_v, s_tau_id, l_v, l_id, &s_count);
    __syncthreads();
  }
  const int n = s_count < kListCap ? s_count : kListCap;
  for (int e = tid; e < n; e += kT) {
    const float v = l_v[e];
    const int id = l_id[e];
    int rank = 0;
#pragma unroll 4
    for (int q = 0; q < n; ++q) rank += beats(l_v[q], l_id[q], v, id) ? 1 : 0;
    if (rank < K) {
      cand_logp[(size_t)b * K + rank] = score_of(v);
      cand_id[(size_t)b * K + rank] = id;
    }
  }
}

// Up to NV = 8 the register budget is held to 64 per thread so that two workgroups share a CU and
// one column's selection overlaps the other's loads.
template <int NV>
__global__ __launch_bounds__(kT, (NV <= 8 ? 8 : 4)) void beam_topk_kernel(
    const float *__restrict__ logits, int ldl, const float *__restrict__ bias, int V, int K,
    int eof_id, float *__restrict__ cand_logp, int *__restrict__ cand_id,
    float *__restrict__ logp_eof) {
  beam_topk_body<NV, false>(logits, ldl, bias, EnsembleArgs{}, V, K, eof_id, cand_logp, cand_id,
                            logp_eof);
}

template <int NV>
__global__ __launch_bounds__(kT, 4) void beam_topk_ensemble_kernel(
    const EnsembleArgs ens, int ldp, int V, int K, int eof_id, float *__restrict__ cand_logp,
    int *__restrict__ cand_id, float *__restrict__ logp_eof) {
  beam_topk_body<NV, true>(nullptr, ldp, nullptr, ens, V, K, eof_id, cand_logp, cand_id, logp_eof);
}

// Generic fallback for the fused top-K: K sweeps over the column with an exclusion threshold.
__global__ __launch_bounds__(kT) void beam_topk_generic_kernel(const float *logits, int ldl,
                                                               const float *bias, int V, int K,
                                                               int eof_id, float *cand_logp,
                                                               int *cand_id, float *logp_eof) {
  __shared__ float red[kNW];
  __shared__ float s_v[kNW];
  __shared__ int s_id[kNW];
  const int b = blockIdx.x, tid = threadIdx.x;
  const int wave = tid / lh::kWave, lane = tid % lh::kWave;
  const float *col = logits + (size_t)b * ldl;
  float m = kNegInf;
  for (int r = tid; r < V; r += kT) m = fmaxf(m, col[r] + (bias ? bias[r] : 0.f));
  const float mx = lh::block_max<kNW>(m, red);
  float part = 0.f;
  for (int r = tid; r < V; r += kT) part += expf(col[r] + (bias ? bias[r] : 0.f) - mx);
  const float lse = logf(lh::block_sum<kNW>(part, red));
  if (tid == 0 && eof_id >= 0 && eof_id < V)
    logp_eof[b] = ((col[eof_id] + (bias ? bias[eof_id] : 0.f)) - mx) - lse;
  // (pv, pi) = previously selected entry; round r picks the best entry that it beats.
  float pv = __builtin_huge_valf();
  int pi = -1;
  for (int r = 0; r < K; ++r) {
    Best me{kNegInf, kIdNone};
    for (int q = tid; q < V; q += kT) {
      const float z = col[q] + (bias ? bias[q] : 0.f);
      if (beats(pv, pi, z, q) && beats(z, q, me.v, me.id)) { me.v = z; me.id = q; }
    }
    Best w = wave_argmax(me);
    __syncthreads();
    if (lane == 0) { s_v[wave] = w.v; s_id[wave] = w.id; }
    __syncthreads();
    w.v = s_v[0]; w.id = s_id[0];
    for (int q = 1; q < kNW; ++q)
      if (beats(s_v[q], s_id[q], w.v, w.id)) { w.v = s_v[q]; w.id = s_id[q]; }
    if (tid == 0) {
      cand_logp[(size_t)b * K + r] = (w.v - mx) - lse;
      cand_id[(size_t)b * K + r] = w.id;
    }
    pv = w.v;
    pi = w.id;
  }
}

int pick_nv(const float *base, int ld, const float *bias, int V) {
  if (V % 4 != 0 || ld % 4 != 0 || !lh::aligned16(base) || !lh::aligned16(bias)) return 0;
  for (int nv = 2; nv <= 16; nv *= 2)
    if (V <= kT * 4 * nv) return nv;
  return 0;
}

}  // namespace

extern "C" int lh_softmax_fwd_f32(const float *logits, int ldl, const float *bias, int V, int B,
                                  float *p, int ldp, lh_stream_t stream) {
  if (V <= 0 || B <= 0 || !logits || !p || ldl < V || ldp < V)
    return lh::fail_arg("lh_softmax_fwd_f32: V=%d B=%d ldl=%d ldp=%d or NULL pointer", V, B, ldl,
                        ldp);
  hipStream_t st = lh::as_stream(stream);
  int nv = pick_nv(logits, ldl, bias, V);
  if (ldp % 4 != 0 || !lh::aligned16(p)) nv = 0;
  const dim3 grid(B), block(kT);
  switch (nv) {
    case 2: hipLaunchKernelGGL(softmax_fwd_kernel<2>, grid, block, 0, st, logits, ldl, bias, V, p, ldp); break;
    case 4: hipLaunchKernelGGL(softmax_fwd_kernel<4>, grid, block, 0, st, logits, ldl, bias, V, p, ldp); break;
    case 8: hipLaunchKernelGGL(softmax_fwd_kernel<8>, grid, block, 0, st, logits, ldl, bias, V, p, ldp); break;
    case 16: hipLaunchKernelGGL(softmax_fwd_kernel<16>, grid, block, 0, st, logits, ldl, bias, V, p, ldp); break;
    default: hipLaunchKernelGGL(softmax_fwd_generic_kernel, grid, block, 0, st, logits, ldl, bias, V, p, ldp);
  }
  return lh::check_launch("lh_softmax_fwd_f32");
}

extern "C" int lh_train_loglik_f32(const float *p, int ldp, int V, int B, const int *tgt0,
                                   const int *mask01, double *accum, lh_stream_t stream) {
  if (V <= 0 || B <= 0 || !p || !tgt0 || !mask01 || !accum || ldp < V)
    return lh::fail_arg("lh_train_loglik_f32: V=%d B=%d ldp=%d or NULL pointer", V, B, ldp);
  hipLaunchKernelGGL(train_loglik_kernel, dim3(1), dim3(64), 0, lh::as_stream(stream), p, ldp, B,
                     tgt0, mask01, accum);
  return lh::check_launch("lh_train_loglik_f32");
}

extern "C" int lh_logsoftmax_xent_f32(const float *logits, int ldl, const float *bias, int V, int B,
                                      const int *tgt0, const int *mask01, double *logp_tgt,
                                      double *loss_accum, lh_stream_t stream) {
  if (V <= 0 || B <= 0 || !logits || !tgt0 || !mask01 || !logp_tgt || !loss_accum || ldl < V)
    return lh::fail_arg("lh_logsoftmax_xent_f32: V=%d B=%d ldl=%d or NULL pointer", V, B, ldl);
  hipStream_t st = lh::as_stream(stream);
  const dim3 grid(B), block(kT);
  switch (pick_nv(logits, ldl, bias, V)) {
    case 2: hipLaunchKernelGGL(logsoftmax_tgt_kernel<2>, grid, block, 0, st, logits, ldl, bias, V, tgt0, logp_tgt); break;
    case 4: hipLaunchKernelGGL(logsoftmax_tgt_kernel<4>, grid, block, 0, st, logits, ldl, bias, V, tgt0, logp_tgt); break;
    case 8: hipLaunchKernelGGL(logsoftmax_tgt_kernel<8>, grid, block, 0, st, logits, ldl, bias, V, tgt0, logp_tgt); break;
    case 16: hipLaunchKernelGGL(logsoftmax_tgt_kernel<16>, grid, block, 0, st, logits, ldl, bias, V, tgt0, logp_tgt); break;
    default: hipLaunchKernelGGL(logsoftmax_tgt_generic_kernel, grid, block, 0, st, logits, ldl, bias, V, tgt0, logp_tgt);
  }
  int rc = lh::check_launch("lh_logsoftmax_xent_f32");
  if (rc != LH_OK) return rc;
  hipLaunchKernelGGL(masked_sum_kernel, dim3(1), dim3(kT), 0, st, logp_tgt, mask01, B, loss_accum);
  return lh::check_launch("lh_logsoftmax_xent_f32 (sum)");
}

extern "C" int lh_softmax_xent_grad_f32(const float *logits, int ldl, const float *bias, int V,
                                        int B, const int *tgt0, const int *mask01, float *dz,
                                        int ldz, double *logp_tgt, double *loss_accum,
                                        lh_stream_t stream) {
  if (V <= 0 || B <= 0 || !logits || !tgt0 || !mask01 || !dz || !logp_tgt || !loss_accum ||
      ldl < V || ldz < V)
    return lh::fail_arg("lh_softmax_xent_grad_f32: V=%d B=%d ldl=%d ldz=%d or NULL pointer", V, B,
                        ldl, ldz);
  hipStream_t st = lh::as_stream(stream);
  int nv = pick_nv(logits, ldl, bias, V);
  if (ldz % 4 != 0 || !lh::aligned16(dz)) nv = 0;
  const dim3 grid(B), block(kT);
  switch (nv) {
    case 2: hipLaunchKernelGGL(softmax_xent_grad_kernel<2>, grid, block, 0, st, logits, ldl, bias, V, tgt0, mask01, dz, ldz, logp_tgt); break;
    case 4: hipLaunchKernelGGL(softmax_xent_grad_kernel<4>, grid, block, 0, st, logits, ldl, bias, V, tgt0, mask01, dz, ldz, logp_tgt); break;
    case 8: hipLaunchKernelGGL(softmax_xent_grad_kernel<8>, grid, block, 0, st, logits, ldl, bias, V, tgt0, mask01, dz, ldz, logp_tgt); break;
    case 16: hipLaunchKernelGGL(softmax_xent_grad_kernel<16>, grid, block, 0, st, logits, ldl, bias, V, tgt0, mask01, dz, ldz, logp_tgt); break;
    default: hipLaunchKernelGGL(softmax_xent_grad_generic_kernel, grid, block, 0, st, logits, ldl, bias, V, tgt0, mask01, dz, ldz, logp_tgt);
  }
  int rc = lh::check_launch("lh_softmax_xent_grad_f32");
  if (rc != LH_OK) return rc;
  hipLaunchKernelGGL(masked_sum_kernel, dim3(1), dim3(kT), 0, st, logp_tgt, mask01, B, loss_accum);
  return lh::check_launch("lh_softmax_xent_grad_f32 (sum)");
}

extern "C" int lh_beam_topk_ensemble_f32(const float *const *p, int n_models, int ldp, int V, int B,
                                         int K, int eof_id, float *cand_logp, int *cand_id,
                                         float *logp_eof, lh_stream_t stream) {
  if (V <= 0 || B <= 0 || !p || !cand_logp || !cand_id || !logp_eof || ldp < V)
    return lh::fail_arg("lh_beam_topk_ensemble_f32: V=%d B=%d ldp=%d or NULL pointer", V, B, ldp);
  if (n_models < 1 || n_models > LH_ENSEMBLE_MAX_MODELS)
    return lh::fail_arg("lh_beam_topk_ensemble_f32: n_models=%d outside [1,%d]", n_models,
                        LH_ENSEMBLE_MAX_MODELS);
  if (K < 1 || K > LH_BEAM_MAX_K || K > V)
    return lh::fail_arg("lh_beam_topk_ensemble_f32: K=%d outside [1,min(%d,V=%d)]", K,
                        LH_BEAM_MAX_K, V);
  EnsembleArgs ens{};
  ens.n_models = n_models;
  int nv = -1;
  for (int m = 0; m < n_models; ++m) {
    if (!p[m]) return lh::fail_arg("lh_beam_topk_ensemble_f32: distribution %d is NULL", m);
    ens.p[m] = p[m];
    const int nv_m = pick_nv(p[m], ldp, nullptr, V);
    nv = m == 0 ? nv_m : (nv_m == nv ? nv : 0);
  }
  if (nv != 2 && nv != 4 && nv != 8 && nv != 16)
    return lh::fail_arg("lh_beam_topk_ensemble_f32: needs V %% 4 == 0, ldp %% 4 == 0, 16-byte "
                        "aligned distributions and V <= %d (V=%d ldp=%d)", 16 * 4 * kT, V, ldp);
  hipStream_t st = lh::as_stream(stream);
  const dim3 grid(B), block(kT);
  switch (nv) {
    case 2: hipLaunchKernelGGL(beam_topk_ensemble_kernel<2>, grid, block, 0, st, ens, ldp, V, K, eof_id, cand_logp, cand_id, logp_eof); break;
    case 4: hipLaunchKernelGGL(beam_topk_ensemble_kernel<4>, grid, block, 0, st, ens, ldp, V, K, eof_id, cand_logp, cand_id, logp_eof); break;
    case 8: hipLaunchKernelGGL(beam_topk_ensemble_kernel<8>, grid, block, 0, st, ens, ldp, V, K, eof_id, cand_logp, cand_id, logp_eof); break;
    default: hipLaunchKernelGGL(beam_topk_ensemble_kernel<16>, grid, block, 0, st, ens, ldp, V, K, eof_id, cand_logp, cand_id, logp_eof); break;
  }
  return lh::check_launch("lh_beam_topk_ensemble_f32");
}

extern "C" int lh_beam_topk_f32(const float *logits, int ldl, const float *bias, int V, int B, int K,
                                int eof_id, float *cand_logp, int *cand_id, float *logp_eof,
                                lh_stream_t stream) {
  if (V <= 0 || B <= 0 || !logits || !cand_logp || !cand_id || !logp_eof || ldl < V)
    return lh::fail_arg("lh_beam_topk_f32: V=%d B=%d ldl=%d or NULL pointer", V, B, ldl);
  if (K < 1 || K > LH_BEAM_MAX_K || K > V)
    return lh::fail_arg("lh_beam_topk_f32: K=%d outside [1,min(%d,V=%d)]", K, LH_BEAM_MAX_K, V);
  hipStream_t st = lh::as_stream(stream);
  const dim3 grid(B), block(kT);
  switch (pick_nv(logits, ldl, bias, V)) {
    case 2: hipLaunchKernelGGL(beam_topk_kernel<2>, grid, block, 0, st, logits, ldl, bias, V, K, eof_id, cand_logp, cand_id, logp_eof); break;
    case 4: hipLaunchKernelGGL(beam_topk_kernel<4>, grid, block, 0, st, logits, ldl, bias, V, K, eof_id, cand_logp, cand_id, logp_eof); break;
    case 8: hipLaunchKernelGGL(beam_topk_kernel<8>, grid, block, 0, st, logits, ldl, bias, V, K, eof_id, cand_logp, cand_id, logp_eof); break;
    case 16: hipLaunchKernelGGL(beam_topk_kernel<16>, grid, block, 0, st, logits, ldl, bias, V, K, eof_id, cand_logp, cand_id, logp_eof); break;
    default: hipLaunchKernelGGL(beam_topk_generic_kernel, grid, block, 0, st, logits, ldl, bias, V, K, eof_id, cand_logp, cand_id, logp_eof);
  }
  return lh::check_launch("lh_beam_topk_f32");
}
