// fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32) with a fused epilogue.
//
// Layout: everything column-major.  A workgroup of 4 wavefronts owns a BM x BN tile of C and walks
// K in slabs of 16.  Both operand slabs are staged in LDS k-major ([k][m] and [k][n]) so that the
// 64 lanes of an MFMA operand read are one contiguous 128-byte run per k (no bank conflicts).
// The MFMA is issued "swapped" (its 32x2 operand comes from X, its 2x32 operand from A), which makes
// the 32 lanes of an accumulator register hold 32 consecutive m of one column n: stores to the
// column-major C are full 128-byte segments.
// Global loads of slab s+1 are issued before the MFMAs of slab s and land in the second LDS buffer
// afterwards (one barrier per slab).
// Workgroup ids are remapped so that each of the 8 XCDs (ids are dealt round-robin to XCDs) owns a
// contiguous range of tiles with n fastest: the tiles that share a slice of A (the large operand:
// stacked gate weights, the V x H output embedding) hit the same XCD's L2.
#include "lh_common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 16;
constexpr int PAD = 4;
constexpr int NT = 256;

struct GemmArgs {
  const float *A[LH_GEMM_MAX_SEGS];
  const float *X[LH_GEMM_MAX_SEGS];
  int lda[LH_GEMM_MAX_SEGS];
  int ldx[LH_GEMM_MAX_SEGS];
  int K[LH_GEMM_MAX_SEGS];
  int nseg;
  int M, N;
  float alpha, beta;
  const float *bias;
  int act;
  const int *colmask;
  float *C;
  int ldc;
  int tiles_m, tiles_n;
};

// Stages one BK x BD operand slab: global -> registers (load), registers -> LDS [BK][BD+PAD] (store).
// KC = false: the operand is contiguous along the tile's outer dimension d (m or n);
// KC = true : the operand is contiguous along k (one run of BK floats per d).
template <int BD, bool KC, bool VEC>
struct SlabStage {
  static constexpr int kVecTotal = BD * BK / 4;
  static constexpr int NV = (kVecTotal + NT - 1) / NT;
  static constexpr int NS = BD * BK / NT;
  float4 v[VEC ? NV : 1];
  float s[VEC ? 1 : NS];

  __device__ __forceinline__ void load(const float *__restrict__ base, int ld, int d0, int k0,
                                       int dlim, int klim, int tid) {
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int f = tid + i * NT;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (f < kVecTotal) {
          if constexpr (!KC) {
            const int k = k0 + f / (BD / 4);
            const int d = d0 + (f % (BD / 4)) * 4;
            if (k < klim && d < dlim)
              val = *reinterpret_cast<const float4 *>(base + (size_t)k * ld + d);
          } else {
            const int d = d0 + f / (BK / 4);
            const int k = k0 + (f % (BK / 4)) * 4;
            if (d < dlim && k < klim)
              val = *reinterpret_cast<const float4 *>(base + (size_t)d * ld + k);
          }
        }
        v[i] = val;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const int e = tid + i * NT;
        int k, d;
        if constexpr (!KC) {
          k = k0 + e / BD;
          d = d0 + e % BD;
        } else {
          d = d0 + e / BK;
          k = k0 + e % BK;
        }
        float val = 0.f;
        if (k < klim && d < dlim)
          val = KC ? base[(size_t)d * ld + k] : base[(size_t)k * ld + d];
        s[i] = val;
      }
    }
  }

  __device__ __forceinline__ void store(float *__restrict__ lds, int tid) const {
    constexpr int LD = BD + PAD;
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int f = tid + i * NT;
        if (f < kVecTotal) {
          if constexpr (!KC) {
            const int k = f / (BD / 4);
            const int d = (f % (BD / 4)) * 4;
            *reinterpret_cast<float4 *>(lds + k * LD + d) = v[i];
          } else {
            const int d = f / (BK / 4);
            const int k = (f % (BK / 4)) * 4;
            lds[(k + 0) * LD + d] = v[i].x;
            lds[(k + 1) * LD + d] = v[i].y;
            lds[(k + 2) * LD + d] = v[i].z;
            lds[(k + 3) * LD + d] = v[i].w;
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const int e = tid + i * NT;
        int k, d;
        if constexpr (!KC) {
          k = e / BD;
          d = e % BD;
        } else {
          d = e / BK;
          k = e % BK;
        }
        lds[k * LD + d] = s[i];
      }
    }
  }
};

template <int BM, int BN, int WM, int WN, bool TA, bool TX, bool VEC>
__global__ __launch_bounds__(NT) void gemm_kernel(const GemmArgs g) {
  static_assert(WM * WN == NT / lh::kWave, "4 wavefronts per workgroup");
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int FM = TM / 32, FN = TN / 32;
  static_assert(FM >= 1 && FN >= 1, "wave tile must hold at least one 32x32 MFMA tile");
  constexpr int LDA = BM + PAD, LDX = BN + PAD;

  __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
  __shared__ __attribute__((aligned(16))) float Xs[2][BK * LDX];

  // XCD-aware tile assignment.
  const int nwg = gridDim.x, id = blockIdx.x;
  const int xcd = id % 8, within = id / 8;
  const int per = nwg / 8, rem = nwg % 8;
  const int logical = xcd * per + (xcd < rem ? xcd : rem) + within;
  const int m0 = (logical / g.tiles_n) * BM;
  const int n0 = (logical % g.tiles_n) * BN;

  const int tid = threadIdx.x;
  const int wave = tid / lh::kWave, lane = tid % lh::kWave;
  const int wm = wave % WM, wn = wave / WM;
  const int l32 = lane % 32, lhi = lane / 32;

  floatx16 acc[FN][FM];
#pragma unroll
  for (int a = 0; a < FN; ++a)
#pragma unroll
    for (int b = 0; b < FM; ++b)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[a][b][j] = 0.f;

  SlabStage<BM, TA, VEC> sa;
  SlabStage<BN, !TX, VEC> sx;

  int total = 0;
  for (int s = 0; s < g.nseg; ++s) total += (g.K[s] + BK - 1) / BK;

  int seg = 0, k0 = 0;
  sa.load(g.A[0], g.lda[0], m0, 0, g.M, g.K[0], tid);
  sx.load(g.X[0], g.ldx[0], n0, 0, g.N, g.K[0], tid);
  sa.store(As[0], tid);
  sx.store(Xs[0], tid);
  __syncthreads();

  for (int s = 0; s < total; ++s) {
    int nseg = seg, nk0 = k0 + BK;
    if (nk0 >= g.K[seg]) {
      nseg = seg + 1;
      nk0 = 0;
    }
    const bool has_next = s + 1 < total;
    if (has_next) {
      sa.load(g.A[nseg], g.lda[nseg], m0, nk0, g.M, g.K[nseg], tid);
      sx.load(g.X[nseg], g.ldx[nseg], n0, nk0, g.N, g.K[nseg], tid);
    }
    const float *as = As[s & 1] + wm * TM + l32;
    const float *xs = Xs[s & 1] + wn * TN + l32;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      float fa[FM], fx[FN];
#pragma unroll
      for (int b = 0; b < FM; ++b) fa[b] = as[(kk + lhi) * LDA + b * 32];
#pragma unroll
      for (int a = 0; a < FN; ++a) fx[a] = xs[(kk + lhi) * LDX + a * 32];
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fx[a], fa[b], acc[a][b], 0, 0, 0);
    }
    if (has_next) {
      sa.store(As[(s + 1) & 1], tid);
      sx.store(Xs[(s + 1) & 1], tid);
    }
    __syncthreads();
    seg = nseg;
    k0 = nk0;
  }

  // Epilogue: accumulator register j of lane l is C[m = .. + l%32][n = .. + 8*(j/4) + 4*(l/32) + j%4].
  const float alpha = g.alpha, beta = g.beta;
#pragma unroll
  for (int a = 0; a < FN; ++a) {
#pragma unroll
    for (int b = 0; b < FM; ++b) {
      const int m = m0 + wm * TM + b * 32 + l32;
      if (m >= g.M) continue;
      const float bv = g.bias ? g.bias[m] : 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int n = n0 + wn * TN + a * 32 + (j / 4) * 8 + lhi * 4 + (j % 4);
        if (n >= g.N) continue;
        float *cp = g.C + (size_t)n * g.ldc + m;
        float v = alpha * acc[a][b][j];
        if (beta != 0.f) v += beta * *cp;
        v += bv;
        if (g.act == LH_ACT_TANH) v = tanhf(v);
        if (g.colmask) v *= (float)g.colmask[n];
        *cp = v;
      }
    }
  }
}

template <int BM, int BN, int WM, int WN>
int launch_cfg(const GemmArgs &g0, bool ta, bool tx, bool vec, hipStream_t st) {
  GemmArgs g = g0;
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  const dim3 grid(g.tiles_m * g.tiles_n), block(NT);
#define LH_GEMM_LAUNCH(TA, TX, VEC) \
  hipLaunchKernelGGL((gemm_kernel<BM, BN, WM, WN, TA, TX, VEC>), grid, block, 0, st, g)
  if (!ta && !tx) {
    if (vec) LH_GEMM_LAUNCH(false, false, true); else LH_GEMM_LAUNCH(false, false, false);
  } else if (ta && !tx) {
    if (vec) LH_GEMM_LAUNCH(true, false, true); else LH_GEMM_LAUNCH(true, false, false);
  } else {
    if (vec) LH_GEMM_LAUNCH(false, true, true); else LH_GEMM_LAUNCH(false, true, false);
  }
#undef LH_GEMM_LAUNCH
  return lh::check_launch("lh_gemm_f32");
}

// Tile choice.  256 CUs: prefer the largest tile that still gives every CU about two workgroups;
// if none does, take the shape with the most workgroups that does not over-pad N.
int pick_tile(int M, int N) {
  struct Cand { int bm, bn; };
  static const Cand cands[4] = {{128, 128}, {128, 64}, {64, 64}, {128, 32}};
  int best = 3, best_wg = -1;
  for (int c = 0; c < 4; ++c) {
    const int bm = cands[c].bm, bn = cands[c].bn;
    if (bn > 32 && N <= bn / 2) continue;  // more than half of every n-tile would be padding
    const int wg = ((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    if (wg >= 448) return c;
    if (wg > best_wg) {
      best_wg = wg;
      best = c;
    }
  }
  return best;
}

}  // namespace

extern "C" int lh_gemm_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX,
                           float alpha, float beta, const float *bias, int act, const int *colmask,
                           float *C, int ldc, lh_stream_t stream) {
  if (M <= 0 || N <= 0) return lh::fail_arg("lh_gemm_f32: M=%d N=%d must be positive", M, N);
  if (!segs || nseg < 1 || nseg > LH_GEMM_MAX_SEGS)
    return lh::fail_arg("lh_gemm_f32: nseg=%d outside [1,%d]", nseg, LH_GEMM_MAX_SEGS);
  if (transA && transX) return lh::fail_arg("lh_gemm_f32: transA && transX is not supported");
  if (act != LH_ACT_NONE && act != LH_ACT_TANH) return lh::fail_arg("lh_gemm_f32: act=%d", act);
  if (!C || ldc < M) return lh::fail_arg("lh_gemm_f32: C=%p ldc=%d (M=%d)", (void *)C, ldc, M);

  GemmArgs g{};
  bool vec = true;
  for (int s = 0; s < nseg; ++s) {
    const lh_gemm_seg &e = segs[s];
    if (!e.A || !e.X || e.K <= 0)
      return lh::fail_arg("lh_gemm_f32: segment %d has A=%p X=%p K=%d", s, (const void *)e.A,
                          (const void *)e.X, e.K);
    const int min_lda = transA ? e.K : M, min_ldx = transX ? N : e.K;
    if (e.lda < min_lda || e.ldx < min_ldx)
      return lh::fail_arg("lh_gemm_f32: segment %d lda=%d (min %d) ldx=%d (min %d)", s, e.lda,
                          min_lda, e.ldx, min_ldx);
    g.A[s] = e.A;
    g.X[s] = e.X;
    g.lda[s] = e.lda;
    g.ldx[s] = e.ldx;
    g.K[s] = e.K;
    // 16-byte loads need aligned bases / leading dimensions and a contiguous extent that is a
    // multiple of 4 (the guards test only the first element of a float4).
    const int a_extent = transA ? e.K : M, x_extent = transX ? N : e.K;
    vec = vec && lh::aligned16(e.A) && lh::aligned16(e.X) && e.lda % 4 == 0 && e.ldx % 4 == 0 &&
          a_extent % 4 == 0 && x_extent % 4 == 0;
  }
  g.nseg = nseg;
  g.M = M;
  g.N = N;
  g.alpha = alpha;
  g.beta = beta;
  g.bias = bias;
  g.act = act;
  g.colmask = colmask;
  g.C = C;
  g.ldc = ldc;

  const bool ta = transA != 0, tx = transX != 0;
  hipStream_t st = lh::as_stream(stream);
  switch (pick_tile(M, N)) {
    case 0: return launch_cfg<128, 128, 2, 2>(g, ta, tx, vec, st);
    case 1: return launch_cfg<128, 64, 2, 2>(g, ta, tx, vec, st);
    case 2: return launch_cfg<64, 64, 2, 2>(g, ta, tx, vec, st);
    default: return launch_cfg<128, 32, 4, 1>(g, ta, tx, vec, st);
  }
}
