// fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32) with a fused epilogue.
//
// Layout: everything column-major.  A workgroup of WM x WN x WK wavefronts owns a BM x BN tile of C
// and walks K in slabs of BK.  Both operand slabs are staged in LDS k-major ([k][m] and [k][n]) so
// that the 64 lanes of an MFMA operand read are contiguous runs (no bank conflicts).  The MFMA is
// issued "swapped" (its 32x2 operand comes from X, its 2x32 operand from A), which makes the 32
// lanes of an accumulator register hold 32 consecutive m of one column n: stores to the
// column-major C are full 128-byte segments.
// Pipelining: the global loads of slab s+1 are issued before the MFMAs of slab s and land in the
// second LDS buffer afterwards (one barrier per slab); inside a slab the LDS operand reads of
// k-step i+1 are issued before the MFMAs of k-step i.  A slab's load latency (about a microsecond
// from HBM) is therefore hidden only by that slab's own MFMAs plus whatever other workgroups the CU
// holds: products with few workgroups per CU use deep slabs (BK up to 128, LDS up to 139 KB) so
// that the latency is paid per 128 k instead of per 16.
// WK > 1 splits every slab's k range over WK wavefront groups (intra-workgroup split-K) and reduces
// the partial accumulators through LDS in a fixed order: this is what keeps skinny products
// (few columns, or M around 1000) from leaving most of the 256 CUs' matrix pipes idle.
// Workgroup ids are remapped so that each of the 8 XCDs (ids are dealt round-robin to XCDs) owns a
// contiguous range of tiles with n fastest: the tiles that share a slice of A (the large operand:
// stacked gate weights, the V x H output embedding) hit the same XCD's L2.
#include "lh_common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int PAD = 4;

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
  int act_rows;  // tanh applies to rows < act_rows
  const int *colmask;
  float *C;
  int ldc;
  int tiles_m, tiles_n;
  // K split across workgroups (main kernel only): workgroup (tile, split) takes slabs
  // [split * slabs_per_split, ...) of the concatenated segments and writes its raw partial tile
  // into plane `split` of the workspace (ws_ld x N floats each, column-major like C); a second
  // kernel adds the planes up in split order and applies the epilogue.
  int splits, slabs_per_split;
  float *ws_part;
  int ws_ld;
  int leave_partial;  // host only: the caller sums the planes itself, no reduction launch
  // Gate product with the LSTM cell in its epilogue (gate_gemm_cell_kernel): M = 4 * cell_H rows
  // in gate order i, f, c', o; C (ldc) is a read-only addend to the pre-activations when beta = 1,
  // taken from column addend_col[n] when that is given; bias and colmask are the stacked gate bias
  // and the 0/1 column mask; the kernel writes c_out and h_out (cell_H x N) and nothing else.
  int cell_H;
  const float *c_prev;
  float *c_out, *h_out;
  float cell_clip;
  int sigmoid_f64;
  const int *addend_col;
  int addend_ncols;  // entries of addend_col are clamped to [0, addend_ncols)
};

// Stages one BK x BD operand slab: global -> registers (load), registers -> LDS [BK][BD+PAD] (store).
// KC = false: the operand is contiguous along the tile's outer dimension d (m or n);
// KC = true : the operand is contiguous along k (one run of BK floats per d).
// The loads are branch-free: an element outside the operand is fetched from a clamped (valid)
// address and replaced by zero when it is written to LDS.
template <int BD, int BK, int NT, bool KC, bool VEC>
struct SlabStage {
  static constexpr int kVecTotal = BD * BK / 4;
  static constexpr int kTotal = BD * BK;
  static constexpr int NV = (kVecTotal + NT - 1) / NT;
  static constexpr int NS = (kTotal + NT - 1) / NT;
  static_assert((VEC ? NV : NS) <= 32, "validity mask is 32 bits");
  float4 v[VEC ? NV : 1];
  float s[VEC ? 1 : NS];
  unsigned ok;  // bit i: element i of this thread lies inside the operand

  __device__ __forceinline__ void load(const float *__restrict__ base, int ld, int d0, int k0,
                                       int dlim, int klim, int tid) {
    ok = 0u;
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int f = tid + i * NT;
        int k, d;
        if constexpr (!KC) {
          k = k0 + f / (BD / 4);
          d = d0 + (f % (BD / 4)) * 4;
        } else {
          d = d0 + f / (BK / 4);
          k = k0 + (f % (BK / 4)) * 4;
        }
        const bool in = f < kVecTotal && k < klim && d < dlim;
        const size_t off = KC ? (size_t)d * ld + k : (size_t)k * ld + d;
        v[i] = *reinterpret_cast<const float4 *>(base + (in ? off : (size_t)0));
        ok |= in ? (1u << i) : 0u;
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
        const bool in = e < kTotal && k < klim && d < dlim;
        const size_t off = KC ? (size_t)d * ld + k : (size_t)k * ld + d;
        s[i] = base[in ? off : (size_t)0];
        ok |= in ? (1u << i) : 0u;
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
          const bool in = (ok >> i) & 1u;
          const float4 val = in ? v[i] : make_float4(0.f, 0.f, 0.f, 0.f);
          if constexpr (!KC) {
            const int k = f / (BD / 4);
            const int d = (f % (BD / 4)) * 4;
            *reinterpret_cast<float4 *>(lds + k * LD + d) = val;
          } else {
            const int d = f / (BK / 4);
            const int k = (f % (BK / 4)) * 4;
            lds[(k + 0) * LD + d] = val.x;
            lds[(k + 1) * LD + d] = val.y;
            lds[(k + 2) * LD + d] = val.z;
            lds[(k + 3) * LD + d] = val.w;
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const int e = tid + i * NT;
        if (e < kTotal) {
          int k, d;
          if constexpr (!KC) {
            k = e / BD;
            d = e % BD;
          } else {
            d = e / BK;
            k = e % BK;
          }
          lds[k * LD + d] = ((ok >> i) & 1u) ? s[i] : 0.f;
        }
      }
    }
  }
};

constexpr int cmax(int a, int b) { return a > b ? a : b; }

template <int BM, int BN, int WK, int BK>
constexpr int smem_floats() {
  return cmax(2 * BK * (BM + PAD + BN + PAD), (WK - 1) * BM * BN);
}

extern __shared__ __attribute__((aligned(16))) float smem[];

template <int BM, int BN, int WM, int WN, int WK, int BK, bool TA, bool TX, bool VEC>
__global__ __launch_bounds__(64 * WM * WN * WK) void gemm_generic_kernel(const GemmArgs g) {
  constexpr int NT = 64 * WM * WN * WK;
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int FM = TM / 32, FN = TN / 32;
  static_assert(FM >= 1 && FN >= 1 && TM % 32 == 0 && TN % 32 == 0, "wave tile = 32x32 MFMA tiles");
  constexpr int KPW = BK / WK;  // k values one wavefront group consumes per slab
  static_assert(KPW >= 2 && KPW % 2 == 0 && BK % 4 == 0, "slab depth");
  constexpr int NSTEP = KPW / 2;
  constexpr int LDA = BM + PAD, LDX = BN + PAD;
  constexpr int kSlabFloats = BK * (LDA + LDX);
  static_assert(smem_floats<BM, BN, WK, BK>() * 4 <= 160 * 1024, "LDS capacity of a CU");

  float *const As0 = smem, *const Xs0 = smem + BK * LDA;
  float *const As1 = smem + kSlabFloats, *const Xs1 = As1 + BK * LDA;

  // XCD-aware tile assignment.
  const int nwg = gridDim.x, id = blockIdx.x;
  const int xcd = id % 8, within = id / 8;
  const int per = nwg / 8, rem = nwg % 8;
  const int logical = xcd * per + (xcd < rem ? xcd : rem) + within;
  const int m0 = (logical / g.tiles_n) * BM;
  const int n0 = (logical % g.tiles_n) * BN;

  const int tid = threadIdx.x;
  const int wave = tid / lh::kWave, lane = tid % lh::kWave;
  const int wk = wave / (WM * WN), wmn = wave % (WM * WN);
  const int wm = wmn % WM, wn = wmn / WM;
  const int l32 = lane % 32, lhi = lane / 32;

  floatx16 acc[FN][FM];
#pragma unroll
  for (int a = 0; a < FN; ++a)
#pragma unroll
    for (int b = 0; b < FM; ++b)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[a][b][j] = 0.f;

  SlabStage<BM, BK, NT, TA, VEC> sa;
  SlabStage<BN, BK, NT, !TX, VEC> sx;

  // segment descriptors live in scalar registers; the cursor selects among them without touching
  // the kernel-argument memory again inside the loop
  const float *const A0 = g.A[0], *const A1 = g.A[1], *const A2 = g.A[2];
  const float *const X0 = g.X[0], *const X1 = g.X[1], *const X2 = g.X[2];
  const int lda0 = g.lda[0], lda1 = g.lda[1], lda2 = g.lda[2];
  const int ldx0 = g.ldx[0], ldx1 = g.ldx[1], ldx2 = g.ldx[2];
  const int K0 = g.K[0], K1 = g.K[1], K2 = g.K[2];
  const int M = g.M, N = g.N;
  int total = (K0 + BK - 1) / BK;
  if (g.nseg > 1) total += (K1 + BK - 1) / BK;
  if (g.nseg > 2) total += (K2 + BK - 1) / BK;

  int lseg = 0, lk0 = 0;  // cursor of the next slab to load
#define LH_ISSUE()                                                  \
  do {                                                              \
    const float *Ab = lseg == 0 ? A0 : (lseg == 1 ? A1 : A2);       \
    const float *Xb = lseg == 0 ? X0 : (lseg == 1 ? X1 : X2);       \
    const int la = lseg == 0 ? lda0 : (lseg == 1 ? lda1 : lda2);    \
    const int lx = lseg == 0 ? ldx0 : (lseg == 1 ? ldx1 : ldx2);    \
    const int Ks = lseg == 0 ? K0 : (lseg == 1 ? K1 : K2);          \
    sa.load(Ab, la, m0, lk0, M, Ks, tid);                           \
    sx.load(Xb, lx, n0, lk0, N, Ks, tid);                           \
    lk0 += BK;                                                      \
    if (lk0 >= Ks) {                                                \
      ++lseg;                                                       \
      lk0 = 0;                                                      \
    }                                                               \
  } while (0)

  LH_ISSUE();
  sa.store(As0, tid);
  sx.store(Xs0, tid);
  __syncthreads();

  for (int s = 0; s < total; ++s) {
    const bool has_next = s + 1 < total;
    if (has_next) LH_ISSUE();
    const float *as = ((s & 1) ? As1 : As0) + (wk * KPW + lhi) * LDA + wm * TM + l32;
    const float *xs = ((s & 1) ? Xs1 : Xs0) + (wk * KPW + lhi) * LDX + wn * TN + l32;
    float fa[2][FM], fx[2][FN];
#pragma unroll
    for (int b = 0; b < FM; ++b) fa[0][b] = as[b * 32];
#pragma unroll
    for (int a = 0; a < FN; ++a) fx[0][a] = xs[a * 32];
#pragma unroll
    for (int i = 0; i < NSTEP; ++i) {
      const int cur = i & 1, nxt = cur ^ 1;
      if (i + 1 < NSTEP) {
#pragma unroll
        for (int b = 0; b < FM; ++b) fa[nxt][b] = as[(2 * (i + 1)) * LDA + b * 32];
#pragma unroll
        for (int a = 0; a < FN; ++a) fx[nxt][a] = xs[(2 * (i + 1)) * LDX + a * 32];
      }
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fx[cur][a], fa[cur][b], acc[a][b], 0, 0, 0);
    }
    if (has_next) {
      sa.store((s & 1) ? As0 : As1, tid);
      sx.store((s & 1) ? Xs0 : Xs1, tid);
    }
    __syncthreads();
  }
#undef LH_ISSUE

  if constexpr (WK > 1) {
    // Fixed-order reduction of the WK partial tiles through LDS (the slab buffers are dead now).
    constexpr int kPerWave = FN * FM * 16 * 64;
    if (wk > 0) {
      float *dst = smem + ((wk - 1) * (WM * WN) + wmn) * kPerWave + lane;
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b)
#pragma unroll
          for (int j = 0; j < 16; ++j) dst[((a * FM + b) * 16 + j) * 64] = acc[a][b][j];
    }
    __syncthreads();
    if (wk > 0) return;
#pragma unroll
    for (int p = 0; p < WK - 1; ++p) {
      const float *src = smem + (p * (WM * WN) + wmn) * kPerWave + lane;
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b)
#pragma unroll
          for (int j = 0; j < 16; ++j) acc[a][b][j] += src[((a * FM + b) * 16 + j) * 64];
    }
  }

  // Epilogue: accumulator register j of lane l is C[m = .. + l%32][n = .. + 8*(j/4) + 4*(l/32) + j%4].
  // Everything the epilogue reads (old C for beta, the column mask, the bias) is fetched for a whole
  // 32x32 accumulator tile with independent loads before any of it is used, so the loads of one tile
  // overlap instead of costing one memory round trip each.
  const float alpha = g.alpha, beta = g.beta;
  const bool use_beta = beta != 0.f;
  const int *const colmask = g.colmask;
#pragma unroll
  for (int a = 0; a < FN; ++a) {
#pragma unroll
    for (int b = 0; b < FM; ++b) {
      const int m = m0 + wm * TM + b * 32 + l32;
      const bool m_ok = m < g.M;
      const int mc = m_ok ? m : 0;
      const float bv = g.bias ? g.bias[mc] : 0.f;
      const bool do_tanh = g.act == LH_ACT_TANH && m < g.act_rows;
      const int nb = n0 + wn * TN + a * 32 + lhi * 4;
      if constexpr (BM * BN <= 32 * 64) {
        // Small tiles run with few workgroups per CU, where a serial chain of loads in the epilogue
        // is a visible part of the launch: fetch four columns' worth before using any.
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float old[4], cm[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int n = nb + q * 8 + r;
            const int nc = n < g.N ? n : 0;
            old[r] = use_beta ? g.C[(size_t)nc * g.ldc + mc] : 0.f;
            cm[r] = colmask ? (float)colmask[nc] : 1.f;
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int n = nb + q * 8 + r;
            float v = alpha * acc[a][b][q * 4 + r];
            if (use_beta) v += beta * old[r];
            v += bv;
            if (do_tanh) v = tanhf(v);
            if (colmask) v *= cm[r];
            if (m_ok && n < g.N) g.C[(size_t)n * g.ldc + m] = v;
          }
        }
      } else {
        // Large tiles: many workgroups share a CU and hide each other's epilogue; keep the register
        // footprint (and with it the number of resident workgroups) minimal.
        if (!m_ok) continue;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int n = nb + (j / 4) * 8 + (j % 4);
          if (n >= g.N) continue;
          float *cp = g.C + (size_t)n * g.ldc + m;
          float v = alpha * acc[a][b][j];
          if (use_beta) v += beta * *cp;
          v += bv;
          if (do_tanh) v = tanhf(v);
          if (colmask) v *= (float)colmask[n];
          *cp = v;
        }
      }
    }
  }
}


// =============================================================================================
// Main kernel (16-byte aligned operands).  What shapes it:
//   * On CDNA a VALU instruction and an MFMA do not overlap inside a SIMD: every non-MFMA vector
//     instruction in the loop costs about four cycles of matrix-pipe time.  The loop therefore
//     carries almost none.  Global addresses are a uniform base (scalar registers) plus
//     per-thread 32-bit byte offsets computed once per K segment; bounds along M / N are folded
//     into those offsets (out-of-range rows re-read the tile origin: they only feed rows and
//     columns of C that are never written); the K tail of a segment, one slab at most, is the only
//     place that masks data.  Staging is 16-byte copies global -> registers -> LDS with no
//     shuffling, for either memory order:
//   * an operand that is contiguous along k in memory lives in LDS as [k/4][d][4], and an MFMA
//     operand fragment for four k-steps is one ds_read_b128 per lane;
//   * an operand that is contiguous along d lives in LDS as [k][d], and a fragment is one
//     ds_read_b32 per k-step.
//     In both, lanes 0-31 take k = 8g+q and lanes 32-63 k = 8g+4+q for step q of group g: the K
//     order inside a slab is a fixed permutation applied to both operands, which leaves the dot
//     products unchanged.
__device__ __forceinline__ float4 keep_if(float4 w, bool c) {
  // per component: a select between two float4 objects makes the compiler pick an address
  w.x = c ? w.x : 0.f;
  w.y = c ? w.y : 0.f;
  w.z = c ? w.z : 0.f;
  w.w = c ? w.w : 0.f;
  return w;
}

template <int BD, int BK, int NT, bool KC>
struct Stage {
  static constexpr int KQ = BK / 4;
  // KC: 16-byte units per k-quad row.  A staging store walks k-quads first, and LDS takes 16-byte
  // stores eight lanes (128 bytes) at a time: the row stride keeps those eight on distinct
  // 16-byte bank groups (measured: 8 conflict cycles per store otherwise).
  static constexpr int LDQ = BD + (KQ == 4 ? 2 : 1);
  // !KC: floats per k row.  Stores are contiguous and fragment reads (32 consecutive floats per
  // lane half) are conflict-free for any stride; the pad only keeps rows 16-byte aligned.
  static constexpr int LDD = BD + 8;
  static constexpr int kFloats = KC ? KQ * LDQ * 4 : BK * LDD;
  static constexpr int kUnits = KQ * BD;  // 16-byte units in a slab
  static constexpr int NU = (kUnits + NT - 1) / NT;
  // every thread owns NU whole units: no per-unit guard (and no exec-mask bookkeeping in the K loop)
  static constexpr bool kExact = kUnits % NT == 0;
  static_assert(NU <= 32, "validity mask is 32 bits");
  static_assert(BD % 16 == 0 && BK % 16 == 0, "tile extents");

  float4 v[NU];
  unsigned goff[NU];  // byte offset of each unit from the slab origin
  unsigned ok;        // K-tail validity, one bit per unit

  // unit u of the slab: (d, k) of its first element and its float offset in LDS
  static __device__ __forceinline__ int unit_d(int u) { return KC ? u / KQ : (u % (BD / 4)) * 4; }
  static __device__ __forceinline__ int unit_k(int u) { return KC ? (u % KQ) * 4 : u / (BD / 4); }
  static __device__ __forceinline__ int unit_lds(int u) {
    return KC ? ((u % KQ) * LDQ + u / KQ) * 4 : (u / (BD / 4)) * LDD + (u % (BD / 4)) * 4;
  }
  // dn = rows/columns of the operand that exist from the tile origin on
  __device__ __forceinline__ void set_ld(int ld, int tid, int dn) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = tid + i * NT;
      const int d = unit_d(u), k = unit_k(u);
      const unsigned off = KC ? (unsigned)(d * ld + k) * 4u : (unsigned)(k * ld + d) * 4u;
      goff[i] = d < dn ? off : 0u;
    }
  }
  // The same for a tile of a stacked gate matrix that holds BD/4 rows of each of the four gates:
  // tile row d is row (d % (BD/4)) of gate d / (BD/4); gates are H rows apart; rows_left = rows of
  // a gate that exist from the tile origin on.
  __device__ __forceinline__ void set_ld_gates(int ld, int tid, int H, int rows_left) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = tid + i * NT;
      const int d = unit_d(u), k = unit_k(u);
      const int r = d % (BD / 4), row = (d / (BD / 4)) * H + r;
      const unsigned off = KC ? (unsigned)(row * ld + k) * 4u : (unsigned)(k * ld + row) * 4u;
      goff[i] = r < rows_left ? off : 0u;
    }
  }
  // kn (< BK) = k values left in the segment: units past it re-read the slab origin and are
  // zeroed before they reach LDS.
  __device__ __forceinline__ void clamp_tail(int tid, int kn) {
    ok = 0u;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const bool in = unit_k(tid + i * NT) < kn;
      goff[i] = in ? goff[i] : 0u;
      ok |= in ? (1u << i) : 0u;
    }
  }
  __device__ __forceinline__ void load(const float *__restrict__ base, int tid) {
    const char *b = reinterpret_cast<const char *>(base);
#pragma unroll
    for (int i = 0; i < NU; ++i)
      if (kExact || tid + i * NT < kUnits) v[i] = *reinterpret_cast<const float4 *>(b + goff[i]);
  }
  __device__ __forceinline__ void zero_tail() {
#pragma unroll
    for (int i = 0; i < NU; ++i) v[i] = keep_if(v[i], (ok >> i) & 1u);
  }
  __device__ __forceinline__ void store(float *__restrict__ buf, int tid) const {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = tid + i * NT;
      if (kExact || u < kUnits) *reinterpret_cast<float4 *>(buf + unit_lds(u)) = v[i];
    }
  }
  // Fragment reads.  origin = float offset for (first k of the wavefront's share, lane half, row d).
  static __device__ __forceinline__ int frag_origin(int k0, int lhi, int d) {
    return KC ? ((k0 / 4 + lhi) * LDQ + d) * 4 : (k0 + 4 * lhi) * LDD + d;
  }
  static __device__ __forceinline__ void read_frag(const float *__restrict__ origin, int grp,
                                                   int frag, float (&out)[4]) {
    if constexpr (KC) {
      const float4 t =
          *reinterpret_cast<const float4 *>(origin + (2 * grp * LDQ + frag * 32) * 4);
      out[0] = t.x, out[1] = t.y, out[2] = t.z, out[3] = t.w;
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) out[q] = origin[(8 * grp + q) * LDD + frag * 32];
    }
  }
};

template <int BM, int BN, int WM, int WN, int WK, int BK, bool TA, bool TX>
constexpr int smem2_floats() {
  constexpr int NT = 64 * WM * WN * WK;
  return cmax(2 * (Stage<BM, BK, NT, TA>::kFloats + Stage<BN, BK, NT, !TX>::kFloats),
              (WK - 1) * BM * BN);
}

// The rare paths of the K loop (a new K segment, a short last slab) are a few dozen selects each.
// Left alone the compiler turns those branches into straight-line selects that every iteration
// executes, and vector ALU instructions take issue time from the matrix pipe; an empty statement
// the optimiser must keep makes each of them a real, normally untaken, branch.
#define LH_KEEP_BRANCH() asm volatile("" ::: "memory")

// CELL: the rows of a tile are BM/4 rows of each LSTM gate and the epilogue is the LSTM cell.
template <int BM, int BN, int WM, int WN, int WK, int BK, bool TA, bool TX, bool CELL>
__device__ __forceinline__ void gemm_body(const GemmArgs &g) {
  constexpr int NT = 64 * WM * WN * WK;
  constexpr int TM = BM / WM, TN = BN / WN;
  constexpr int FM = TM / 32, FN = TN / 32;
  static_assert(FM >= 1 && FN >= 1 && TM % 32 == 0 && TN % 32 == 0, "wave tile = 32x32 MFMA tiles");
  constexpr int KPW = BK / WK;  // k values one wavefront group consumes per slab
  static_assert(KPW % 8 == 0, "a fragment group covers 8 k (4 per lane half)");
  constexpr int NG = KPW / 8;
  using SA = Stage<BM, BK, NT, TA>;
  using SX = Stage<BN, BK, NT, !TX>;
  constexpr int kAF = SA::kFloats, kSlab = SA::kFloats + SX::kFloats;
  static_assert(smem2_floats<BM, BN, WM, WN, WK, BK, TA, TX>() * 4 <= 160 * 1024,
                "LDS capacity of a CU");

  // XCD-aware tile assignment.
  const int nwg = gridDim.x, id = blockIdx.x;
  const int xcd = id % 8, within = id / 8;
  const int per = nwg / 8, rem = nwg % 8;
  const int logical = xcd * per + (xcd < rem ? xcd : rem) + within;
  // the splits of a tile are neighbours: same XCD, so the partial tiles meet in its L2
  const int splits = g.splits;
  const int tile = splits == 1 ? logical : logical / splits;
  const int split = splits == 1 ? 0 : logical % splits;
  // CELL: m0 counts rows of ONE gate
  const int m0 = (tile / g.tiles_n) * (CELL ? BM / 4 : BM);
  const int n0 = (tile % g.tiles_n) * BN;

  const int tid = threadIdx.x;
  const int wave = tid / lh::kWave, lane = tid % lh::kWave;
  const int wk = wave / (WM * WN), wmn = wave % (WM * WN);
  const int wm = wmn % WM, wn = wmn / WM;
  const int l32 = lane % 32, lhi = lane / 32;

  floatx16 acc[FN][FM];
#pragma unroll
  for (int a = 0; a < FN; ++a)
#pragma unroll
    for (int b = 0; b < FM; ++b)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[a][b][j] = 0.f;

  SA sa;
  SX sx;
  const int fa_off = SA::frag_origin(wk * KPW, lhi, wm * TM + l32);
  const int fx_off = kAF + SX::frag_origin(wk * KPW, lhi, wn * TN + l32);

  const float *const A0 = g.A[0], *const A1 = g.A[1], *const A2 = g.A[2];
  const float *const X0 = g.X[0], *const X1 = g.X[1], *const X2 = g.X[2];
  const int lda0 = g.lda[0], lda1 = g.lda[1], lda2 = g.lda[2];
  const int ldx0 = g.ldx[0], ldx1 = g.ldx[1], ldx2 = g.ldx[2];
  const int K0 = g.K[0], K1 = g.K[1], K2 = g.K[2];
  const int M = g.M, N = g.N;
  const int slabs0 = (K0 + BK - 1) / BK;
  const int slabs1 = g.nseg > 1 ? (K1 + BK - 1) / BK : 0;
  const int slabs2 = g.nseg > 2 ? (K2 + BK - 1) / BK : 0;
  // this workgroup's share of the slab sequence (the host never makes an empty share)
  const int first = split * g.slabs_per_split;
  const int total = min(g.slabs_per_split, slabs0 + slabs1 + slabs2 - first);
  int lseg = 0, lk0 = first;  // cursor of the next slab to load: segment, k offset inside it
  if (lk0 >= slabs0) {
    lk0 -= slabs0;
    lseg = 1;
    if (lk0 >= slabs1) {
      lk0 -= slabs1;
      lseg = 2;
    }
  }
  lk0 *= BK;
  // The K loop's scalar work is a few additions: the origin of the next slab in each operand
  // advances by a fixed step, and everything that depends on the segment (base pointers, leading
  // dimensions, the per-thread offsets) is set up only when a segment begins.  Both wavefronts of
  // a SIMD run this code at the same time, right behind the barrier, so every scalar instruction
  // here is time the matrix pipe stands still.
  bool new_seg = true;  // the next slab opens a segment (or the first one of this share)
  bool tail = false;    // the slab in the staging registers ends its segment short of BK
  const float *pa = nullptr, *px = nullptr;  // origin of the next slab inside A / X
  int step_a = 0, step_x = 0;                // floats from one slab to the next
  int kleft = 0;                             // k values of the segment not yet loaded
#define LH_ISSUE()                                                                 \
  do {                                                                             \
    if (new_seg) {                                                                 \
      LH_KEEP_BRANCH();                                                            \
      const float *Ab = lseg == 0 ? A0 : (lseg == 1 ? A1 : A2);                    \
      const float *Xb = lseg == 0 ? X0 : (lseg == 1 ? X1 : X2);                    \
      const int la = lseg == 0 ? lda0 : (lseg == 1 ? lda1 : lda2);                 \
      const int lx = lseg == 0 ? ldx0 : (lseg == 1 ? ldx1 : ldx2);                 \
      const int Ks = lseg == 0 ? K0 : (lseg == 1 ? K1 : K2);                       \
      if constexpr (CELL) sa.set_ld_gates(la, tid, g.cell_H, g.cell_H - m0);       \
      else sa.set_ld(la, tid, M - m0);                                             \
      sx.set_ld(lx, tid, N - n0);                                                  \
      pa = TA ? Ab + (size_t)m0 * la + lk0 : Ab + (size_t)lk0 * la + m0;           \
      px = !TX ? Xb + (size_t)n0 * lx + lk0 : Xb + (size_t)lk0 * lx + n0;          \
      step_a = TA ? BK : BK * la;                                                  \
      step_x = !TX ? BK : BK * lx;                                                 \
      kleft = Ks - lk0;                                                            \
    }                                                                              \
    tail = kleft < BK;                                                             \
    if (tail) {                                                                    \
      LH_KEEP_BRANCH();                                                            \
      sa.clamp_tail(tid, kleft);                                                   \
      sx.clamp_tail(tid, kleft);                                                   \
    }                                                                              \
    sa.load(pa, tid);                                                              \
    sx.load(px, tid);                                                              \
    pa += step_a;                                                                  \
    px += step_x;                                                                  \
    kleft -= BK;                                                                   \
    new_seg = kleft <= 0; /* a short last slab has clamped the offsets as well */  \
    if (new_seg) {                                                                 \
      ++lseg;                                                                      \
      lk0 = 0;                                                                     \
    }                                                                              \
  } while (0)
#define LH_STASH(BUF)         \
  do {                        \
    float *sb = (BUF);        \
    if (tail) {               \
      LH_KEEP_BRANCH();       \
      sa.zero_tail();         \
      sx.zero_tail();         \
    }                         \
    sa.store(sb, tid);        \
    sx.store(sb + kAF, tid);  \
  } while (0)

  // Software pipeline, two slabs deep: LDS holds slab s (being consumed) and slab s+1, the
  // staging registers hold slab s+2 in flight.  A slab goes to LDS at the START of the iteration
  // before it is consumed -- its buffer was released by the barrier that ended the previous
  // iteration -- so neither the global loads nor the LDS stores sit between two slabs of MFMAs.
  LH_ISSUE();
  LH_STASH(smem);
  if (total > 1) LH_ISSUE();
  __syncthreads();
  int cur = 0;  // float offset of the slab buffer being consumed
  // Fragments are read one group (8 k) ahead of the MFMAs that use them.  Deep slabs (one
  // workgroup per CU, nobody else to cover a stall) keep that up across slab boundaries: the
  // barrier that releases a slab sits BEFORE the MFMAs of its last group, whose fragments are in
  // registers by then, and the first group of the next slab is read right behind it, under those
  // MFMAs.  Shallow slabs run several workgroups per CU, which hide the one exposed read per slab
  // better than the dozen registers the carried fragments cost would (they lower the occupancy).
  constexpr bool kCarry = BK >= 64 && NG % 2 == 0;
  float fa[2][FM][4], fx[2][FN][4];
  if constexpr (kCarry) {
#pragma unroll
    for (int b = 0; b < FM; ++b) SA::read_frag(smem + fa_off, 0, b, fa[0][b]);
#pragma unroll
    for (int a = 0; a < FN; ++a) SX::read_frag(smem + fx_off, 0, a, fx[0][a]);
  }
  for (int s = 0; s < total; ++s) {
    const float *as = smem + cur + fa_off;
    const float *xs = smem + cur + fx_off;
    if constexpr (!kCarry) {
#pragma unroll
      for (int b = 0; b < FM; ++b) SA::read_frag(as, 0, b, fa[0][b]);
#pragma unroll
      for (int a = 0; a < FN; ++a) SX::read_frag(xs, 0, a, fx[0][a]);
    }
#pragma unroll
    for (int grp = 0; grp < NG; ++grp) {
      const int c = grp & 1, n = c ^ 1;
      if (grp + 1 < NG) {
#pragma unroll
        for (int b = 0; b < FM; ++b) SA::read_frag(as, grp + 1, b, fa[n][b]);
#pragma unroll
        for (int a = 0; a < FN; ++a) SX::read_frag(xs, grp + 1, a, fx[n][a]);
      } else if constexpr (kCarry) {
        // nothing moves across: the MFMAs of the groups before stay ahead of the barrier, where
        // they cover the latency of the fragment reads the barrier has to wait for
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        cur = kSlab - cur;
        if (s + 1 < total) {
#pragma unroll
          for (int b = 0; b < FM; ++b) SA::read_frag(smem + cur + fa_off, 0, b, fa[n][b]);
#pragma unroll
          for (int a = 0; a < FN; ++a) SX::read_frag(smem + cur + fx_off, 0, a, fx[n][a]);
        }
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int a = 0; a < FN; ++a)
#pragma unroll
          for (int b = 0; b < FM; ++b)
            // operands swapped on purpose: the transposed product puts consecutive m in
            // consecutive lanes of every accumulator register
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fx[c][a][q], fa[c][b][q],
                                                             acc[a][b], 0, 0, 0);
        // the staging work of the slab rides behind MFMAs that are already in the pipe instead
        // of standing between two groups of them
        if (grp == 0 && q == 0 && s + 1 < total) LH_STASH(smem + (kSlab - cur));
        if (grp == 0 && q == 1 && s + 2 < total) LH_ISSUE();
      }
    }
    if constexpr (!kCarry) {
      __syncthreads();
      cur = kSlab - cur;
    }
  }
#undef LH_ISSUE
#undef LH_STASH

  if constexpr (WK > 1) {
    // Fixed-order reduction of the WK partial tiles through LDS (the slab buffers are dead now).
    constexpr int kPerWave = FN * FM * 16 * 64;
    if (wk > 0) {
      float *dst = smem + ((wk - 1) * (WM * WN) + wmn) * kPerWave + lane;
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b)
#pragma unroll
          for (int j = 0; j < 16; ++j) dst[((a * FM + b) * 16 + j) * 64] = acc[a][b][j];
    }
    __syncthreads();
    if (wk == 0) {
#pragma unroll
      for (int p = 0; p < WK - 1; ++p) {
        const float *src = smem + (p * (WM * WN) + wmn) * kPerWave + lane;
#pragma unroll
        for (int a = 0; a < FN; ++a)
#pragma unroll
          for (int b = 0; b < FM; ++b)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[a][b][j] += src[((a * FM + b) * 16 + j) * 64];
      }
    }
  }

  if constexpr (CELL) {
    // The four gates of a cell sit in different wavefronts: the tile goes through LDS as
    // S[n][m] (the slab buffers and the partial tiles are dead), then every thread of the
    // workgroup takes cells.
    constexpr int GQ = BM / 4;
    static_assert(smem2_floats<BM, BN, WM, WN, WK, BK, TA, TX>() >= BM * BN, "tile does not fit LDS");
    if constexpr (WK > 1) __syncthreads();  // the partial tiles have been read
    if (wk == 0) {
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b)
#pragma unroll
          for (int j = 0; j < 16; ++j)
            smem[(wn * TN + a * 32 + lhi * 4 + (j / 4) * 8 + (j % 4)) * BM + wm * TM + b * 32 + l32] =
                acc[a][b][j];
    }
    __syncthreads();
    const int H = g.cell_H;
    const bool add = g.beta != 0.f;
    // A thread's cells: everything they read from memory is fetched first, with independent
    // loads (the outputs may alias c_prev, so loads interleaved with the stores would wait for
    // one another, a memory latency per cell), then the arithmetic, then the stores.
    constexpr int kCells = GQ * BN, kPer = (kCells + NT - 1) / NT;
    float cprev[kPer], mask[kPer], pre[kPer][4];
    bool ok[kPer];
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int idx = tid + i * NT;
      const int rl = idx % GQ, nl = idx / GQ;
      const int r = m0 + rl, n = n0 + nl;
      ok[i] = idx < kCells && r < H && n < g.N;
      cprev[i] = 0.f, mask[i] = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) pre[i][q] = 0.f;
      if (ok[i]) {
        int col = n;
        if (g.addend_col) col = min(max(g.addend_col[n], 0), g.addend_ncols - 1);
        const float *ad = g.C + (size_t)col * g.ldc + r;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float v = smem[nl * BM + q * GQ + rl];
          const float t = add ? ad[(size_t)q * H] : 0.f;
          pre[i][q] = (add ? v + t : v) + g.bias[q * H + r];
        }
        cprev[i] = g.c_prev[(size_t)n * H + r];
        mask[i] = (float)g.colmask[n];
      }
    }
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int idx = tid + i * NT;
      const int r = m0 + idx % GQ, n = n0 + idx / GQ;
      float c, h;
      if (g.sigmoid_f64)
        lh::lstm_cell_point<true>(pre[i][0], pre[i][1], pre[i][2], pre[i][3], cprev[i], mask[i],
                                  g.cell_clip, c, h);
      else
        lh::lstm_cell_point<false>(pre[i][0], pre[i][1], pre[i][2], pre[i][3], cprev[i], mask[i],
                                   g.cell_clip, c, h);
      if (ok[i]) {
        const size_t o = (size_t)n * H + r;
        g.c_out[o] = c;
        g.h_out[o] = h;
      }
    }
    return;
  }

  if (wk > 0) return;

  // Epilogue: accumulator register j of lane l is C[m = .. + l%32][n = .. + 8*(j/4) + 4*(l/32) + j%4].
  // A split product stores the bare partial sums in its plane of the workspace instead.
  const bool partial = splits > 1;
  const float alpha = partial ? 1.f : g.alpha, beta = g.beta;
  const bool use_beta = !partial && beta != 0.f;
  const int *const colmask = partial ? nullptr : g.colmask;
  const float *const bias = partial ? nullptr : g.bias;
  const int act_rows = partial || g.act != LH_ACT_TANH ? 0 : g.act_rows;
  float *const Cb = partial ? g.ws_part + (size_t)split * g.ws_ld * g.N : g.C;
  const int ldc = partial ? g.ws_ld : g.ldc;
#pragma unroll
  for (int a = 0; a < FN; ++a) {
#pragma unroll
    for (int b = 0; b < FM; ++b) {
      const int m = m0 + wm * TM + b * 32 + l32;
      if (m >= g.M) continue;
      const float bv = bias ? bias[m] : 0.f;
      const bool do_tanh = m < act_rows;
      const int nb = n0 + wn * TN + a * 32 + lhi * 4;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int n = nb + (j / 4) * 8 + (j % 4);
        if (n >= g.N) continue;
        float *cp = Cb + (size_t)n * ldc + m;
        float v = alpha * acc[a][b][j];
        if (use_beta) v += beta * *cp;
        v += bv;
        if (do_tanh) v = tanhf(v);
        if (colmask) v *= (float)colmask[n];
        *cp = v;
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, int WK, int BK, bool TA, bool TX>
__global__ __launch_bounds__(64 * WM * WN * WK) void gemm_kernel(const GemmArgs g) {
  gemm_body<BM, BN, WM, WN, WK, BK, TA, TX, false>(g);
}

// Stacked gate product W*[x; h; h~] (both operands as stored, no transposes) + LSTM cell.
template <int BM, int BN, int WM, int WN, int WK, int BK>
__global__ __launch_bounds__(64 * WM * WN * WK) void gate_gemm_cell_kernel(const GemmArgs g) {
  gemm_body<BM, BN, WM, WN, WK, BK, false, false, true>(g);
}

// Whether a configuration's LDS holds a whole tile, which the cell epilogue needs.
template <int BM, int BN, int WM, int WN, int WK, int BK>
constexpr bool cell_capable() {
  return smem2_floats<BM, BN, WM, WN, WK, BK, false, false>() >= BM * BN;
}

// Second half of a split product: C = epilogue(sum of the partial planes, in split order).
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmArgs g) {
  const size_t plane = (size_t)g.ws_ld * g.N;
  const size_t total = (size_t)g.M * g.N;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    const int n = (int)(i / g.M), m = (int)(i % g.M);
    const float *p = g.ws_part + (size_t)n * g.ws_ld + m;
    float acc = 0.f;
    for (int s = 0; s < g.splits; ++s) acc += p[s * plane];
    float *cp = g.C + (size_t)n * g.ldc + m;
    float v = g.alpha * acc;
    if (g.beta != 0.f) v += g.beta * *cp;
    if (g.bias) v += g.bias[m];
    if (g.act == LH_ACT_TANH && m < g.act_rows) v = tanhf(v);
    if (g.colmask) v *= (float)g.colmask[n];
    *cp = v;
  }
}

// ---- configurations -----------------------------------------------------------------------
struct Config {
  int bm, bn, wm, wn, wk, bk;
};
// X(index, BM, BN, WM, WN, WK, BK)
#define LH_GEMM_CONFIGS(X)                                                     \
  X(0, 128, 128, 2, 2, 1, 16)  /* large products: output projection         */ \
  X(1, 128, 128, 2, 2, 1, 32)                                                  \
  X(2, 128, 96, 4, 1, 1, 16)                                                   \
  X(3, 128, 64, 2, 2, 1, 16)                                                   \
  X(4, 128, 64, 2, 2, 1, 32)                                                   \
  X(5, 64, 96, 2, 1, 2, 32)    /* stacked gate products at a few hundred columns */ \
  X(6, 64, 96, 2, 1, 2, 64)                                                    \
  X(7, 64, 64, 2, 2, 1, 16)    /* also the only shape built for unaligned operands */ \
  X(8, 64, 64, 2, 2, 1, 64)                                                    \
  X(9, 64, 64, 2, 2, 1, 128)                                                   \
  X(10, 32, 96, 1, 3, 2, 32)   /* M around 1000 */                             \
  X(11, 32, 96, 1, 3, 2, 128)                                                  \
  X(12, 32, 64, 1, 2, 4, 32)   /* skinny */                                    \
  X(13, 32, 64, 1, 2, 4, 128)                                                  \
  X(14, 32, 32, 1, 1, 8, 64)   /* very skinny */                               \
  X(15, 32, 32, 1, 1, 8, 128)                                                  \
  X(16, 128, 32, 4, 1, 1, 16)                                                  \
  X(17, 128, 32, 4, 1, 1, 64)                                                  \
  X(18, 64, 32, 2, 1, 4, 32)                                                   \
  X(19, 64, 32, 2, 1, 4, 128)                                                  \
  X(20, 128, 128, 2, 2, 1, 64) /* deep slabs: one workgroup per CU hides its own latency */ \
  X(21, 128, 64, 2, 2, 1, 64)                                                  \
  X(22, 128, 128, 2, 2, 2, 64) /* ... or two wavefronts per SIMD inside the workgroup */ \
  X(23, 128, 64, 2, 2, 2, 64)                                                  \
  X(24, 128, 96, 4, 1, 2, 64)                                                  \
  X(25, 64, 64, 2, 2, 2, 128)                                                  \
  X(26, 256, 128, 4, 2, 1, 16) /* the batched products of training */          \
  X(27, 256, 128, 4, 2, 1, 32)

#define LH_CFG_ENTRY(I, BM, BN, WM, WN, WK, BK) {BM, BN, WM, WN, WK, BK},
const Config kConfigs[] = {LH_GEMM_CONFIGS(LH_CFG_ENTRY)};
#undef LH_CFG_ENTRY
constexpr int kNumConfigs = sizeof(kConfigs) / sizeof(kConfigs[0]);
constexpr int kUnalignedConfig = 7;

template <typename KernelT>
int launch_kernel(KernelT kernel, int smem_bytes, dim3 grid, dim3 block, hipStream_t st,
                  const GemmArgs &g) {
  if (smem_bytes > 64 * 1024) {
    // more dynamic LDS than the default limit: raised once per kernel instance
    static thread_local const void *raised[64];
    static thread_local int n_raised = 0;
    bool done = false;
    for (int i = 0; i < n_raised; ++i) done = done || raised[i] == (const void *)kernel;
    if (!done) {
      hipError_t e = hipFuncSetAttribute((const void *)kernel,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem_bytes);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        return lh::fail_arg("lh_gemm_f32: cannot reserve %d bytes of LDS: %s", smem_bytes,
                            hipGetErrorString(e));
      }
      if (n_raised < 64) raised[n_raised++] = (const void *)kernel;
    }
  }
  hipLaunchKernelGGL(kernel, grid, block, smem_bytes, st, g);
  return lh::check_launch("lh_gemm_f32");
}

template <int BM, int BN, int WM, int WN, int WK, int BK, bool ALLOW_UNALIGNED>
int launch_cfg(const GemmArgs &g0, bool ta, bool tx, bool vec, hipStream_t st) {
  GemmArgs g = g0;
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  if (!vec) g.splits = 1;
  int slabs = 0;
  for (int s = 0; s < g.nseg; ++s) slabs += (g.K[s] + BK - 1) / BK;
  g.slabs_per_split = (slabs + g.splits - 1) / g.splits;
  g.splits = (slabs + g.slabs_per_split - 1) / g.slabs_per_split;  // no empty share
  const dim3 grid(g.tiles_m * g.tiles_n * g.splits), block(64 * WM * WN * WK);
  if (vec) {
    int rc;
#define LH_GEMM_LAUNCH(TA, TX)                                                              \
  rc = launch_kernel(gemm_kernel<BM, BN, WM, WN, WK, BK, TA, TX>,                           \
                     smem2_floats<BM, BN, WM, WN, WK, BK, TA, TX>() * 4, grid, block, st, g)
    if (!ta && !tx) LH_GEMM_LAUNCH(false, false);
    else if (ta) LH_GEMM_LAUNCH(true, false);
    else LH_GEMM_LAUNCH(false, true);
#undef LH_GEMM_LAUNCH
    if (rc != LH_OK || g.splits == 1 || g.leave_partial) return rc;
    const size_t total = (size_t)g.M * g.N;
    const size_t blocks = (total + 1023) / 1024;  // four elements per thread
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)(blocks < 8192 ? blocks : 8192)),
                       dim3(256), 0, st, g);
    return lh::check_launch("lh_gemm_ws_f32 split reduction");
  }
  if constexpr (ALLOW_UNALIGNED) {
    constexpr int bytes = smem_floats<BM, BN, WK, BK>() * 4;
#define LH_GEMM_LAUNCH(TA, TX) \
  return launch_kernel(gemm_generic_kernel<BM, BN, WM, WN, WK, BK, TA, TX, false>, bytes, grid, block, st, g)
    if (!ta && !tx) LH_GEMM_LAUNCH(false, false);
    else if (ta) LH_GEMM_LAUNCH(true, false);
    else LH_GEMM_LAUNCH(false, true);
#undef LH_GEMM_LAUNCH
  }
  return lh::fail_arg("lh_gemm_f32: internal error, unaligned operands reached an aligned-only tile");
}

int launch_index(int c, const GemmArgs &g, bool ta, bool tx, bool vec, hipStream_t st) {
  switch (c) {
#define LH_CFG_CASE(I, BM, BN, WM, WN, WK, BK) \
  case I:                                      \
    return launch_cfg<BM, BN, WM, WN, WK, BK, I == kUnalignedConfig>(g, ta, tx, vec, st);
    LH_GEMM_CONFIGS(LH_CFG_CASE)
#undef LH_CFG_CASE
    default: return lh::fail_arg("lh_gemm_f32: configuration %d does not exist", c);
  }
}

template <int BM, int BN, int WM, int WN, int WK, int BK>
int launch_cell_cfg(const GemmArgs &g0, hipStream_t st) {
  if constexpr (cell_capable<BM, BN, WM, WN, WK, BK>()) {
    GemmArgs g = g0;
    g.tiles_m = (g.cell_H + BM / 4 - 1) / (BM / 4);
    g.tiles_n = (g.N + BN - 1) / BN;
    g.splits = 1;
    g.slabs_per_split = 0;
    for (int s = 0; s < g.nseg; ++s) g.slabs_per_split += (g.K[s] + BK - 1) / BK;
    const dim3 grid(g.tiles_m * g.tiles_n), block(64 * WM * WN * WK);
    return launch_kernel(gate_gemm_cell_kernel<BM, BN, WM, WN, WK, BK>,
                         smem2_floats<BM, BN, WM, WN, WK, BK, false, false>() * 4, grid, block, st, g);
  } else {
    return lh::fail_arg("lh_gate_gemm_lstm_cell_f32: internal error, tile %dx%d cannot hold the cell", BM, BN);
  }
}

int launch_cell_index(int c, const GemmArgs &g, hipStream_t st) {
  switch (c) {
#define LH_CFG_CASE(I, BM, BN, WM, WN, WK, BK) \
  case I: return launch_cell_cfg<BM, BN, WM, WN, WK, BK>(g, st);
    LH_GEMM_CONFIGS(LH_CFG_CASE)
#undef LH_CFG_CASE
    default: return lh::fail_arg("lh_gate_gemm_lstm_cell_f32: configuration %d does not exist", c);
  }
}

bool cell_capable_index(int c) {
  switch (c) {
#define LH_CFG_CASE(I, BM, BN, WM, WN, WK, BK) \
  case I: return cell_capable<BM, BN, WM, WN, WK, BK>();
    LH_GEMM_CONFIGS(LH_CFG_CASE)
#undef LH_CFG_CASE
    default: return false;
  }
}

template <int BM, int BN, int WM, int WN, int WK, int BK>
int occupancy_cfg(bool ta, bool tx, int *blocks_per_cu, int *lds_bytes) {
  constexpr int block = 64 * WM * WN * WK;
  hipError_t e;
#define LH_GEMM_OCC(TA, TX)                                                                       \
  do {                                                                                            \
    constexpr int bytes = smem2_floats<BM, BN, WM, WN, WK, BK, TA, TX>() * 4;                     \
    *lds_bytes = bytes;                                                                           \
    auto kernel = gemm_kernel<BM, BN, WM, WN, WK, BK, TA, TX>;                                    \
    if (bytes > 64 * 1024)                                                                        \
      (void)hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                bytes);                                                           \
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(blocks_per_cu, kernel, block, bytes);        \
  } while (0)
  if (!ta && !tx) LH_GEMM_OCC(false, false);
  else if (ta) LH_GEMM_OCC(true, false);
  else LH_GEMM_OCC(false, true);
#undef LH_GEMM_OCC
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return lh::fail_arg("lh_gemm_config_info: occupancy query failed: %s", hipGetErrorString(e));
  }
  return LH_OK;
}

int occupancy_index(int c, bool ta, bool tx, int *blocks_per_cu, int *lds_bytes) {
  switch (c) {
#define LH_CFG_CASE(I, BM, BN, WM, WN, WK, BK) \
  case I: return occupancy_cfg<BM, BN, WM, WN, WK, BK>(ta, tx, blocks_per_cu, lds_bytes);
    LH_GEMM_CONFIGS(LH_CFG_CASE)
#undef LH_CFG_CASE
    default: return lh::fail_arg("lh_gemm_config_info: configuration %d does not exist", c);
  }
}

int g_config_override = -1;  // tuning / test aids, see lh_gemm_set_config_override
int g_splits_override = 0;

constexpr int kMaxSplits = 16;

// Leading dimension of a partial plane, and the largest split count <= want whose planes fit.
int plane_ld(int M) { return (M + 3) & ~3; }
int fit_splits(int M, int N, int want, size_t workspace_bytes) {
  if (want <= 1) return 1;
  const size_t plane = (size_t)plane_ld(M) * N * sizeof(float);
  const size_t fit = workspace_bytes / plane;
  const size_t s = fit < (size_t)want ? fit : (size_t)want;
  return s < 1 ? 1 : (int)(s > kMaxSplits ? kMaxSplits : s);
}

// ---- choice of tile configuration and K split ------------------------------------------------
// Cost model over a measured table.  For one configuration, T1(K) is the time of a launch that
// gives every CU a single workgroup and Tocc(K) of one that gives every CU as many as fit at once
// (both linear in the K depth of a workgroup's share).  A product whose fullest CU receives n
// workgroups then takes about (n / occ) * Tocc + T(n % occ), T interpolated between T1 and Tocc;
// a split adds the pass that sums the partial planes.  The cheapest (configuration, split) wins.
struct Tuning {
  int occ;           // workgroups resident per CU
  float f1, s1;      // one workgroup per CU: fixed us, us per k
  float focc, socc;  // CU full
};
#include "gemm_tuning.inc"
constexpr int kCUs = 256;
constexpr float kReduceFixedUs = 2.5f, kReduceBytesPerUs = 3.0e6f;
constexpr float kCellFixedUs = 4.0f;  // a launch of the LSTM cell kernel behind its product

float predict_us(const Tuning &t, const Config &k, int M, int N, const int *K, int nseg, int want,
                 bool reduce_free, int *splits) {
  const long long tiles = (long long)((M + k.bm - 1) / k.bm) * ((N + k.bn - 1) / k.bn);
  int slabs = 0;
  for (int s = 0; s < nseg; ++s) slabs += (K[s] + k.bk - 1) / k.bk;
  const int share = (slabs + want - 1) / want;
  const int S = (slabs + share - 1) / share;
  *splits = S;
  const float depth = (float)share * k.bk;
  // Workgroups per CU: dispatch is dynamic, so a fractional load costs less than a whole extra
  // round but leaves a tail of about half a workgroup.
  const float per_cu = (float)(tiles * S) / kCUs;
  const float load = fminf(per_cu + 0.5f, ceilf(per_cu));
  const float t1 = t.f1 + t.s1 * depth, tocc = t.focc + t.socc * depth;
  const float rounds = floorf(load / (float)t.occ);
  const float rest = load - rounds * (float)t.occ;
  float us = rounds * tocc;
  if (rest > 1e-6f)
    us += rest <= 1.f || t.occ == 1 ? t1 : t1 + (tocc - t1) * (rest - 1.f) / (float)(t.occ - 1);
  if (S > 1 && !reduce_free)
    us += kReduceFixedUs + (float)(S + 1) * (float)M * (float)N * 4.f / kReduceBytesPerUs;
  if (S > 1 && reduce_free)  // the consumer reads S planes instead of one matrix
    us += (float)(S - 1) * (float)M * (float)N * 4.f / kReduceBytesPerUs;
  return us;
}

// max_planes > 0: the caller consumes up to that many partial planes itself (no reduction pass).

// only_cell: restrict the choice to unsplit launches of configurations whose LDS holds a whole
// tile (what the gate product with the cell in its epilogue can use).  *us (optional) receives
// the predicted time of the choice.
void pick_config(int M, int N, const int *K, int nseg, bool ta, bool tx, bool vec,
                 size_t workspace_bytes, int max_planes, int *config, int *splits,
                 bool only_cell = false, float *us_out = nullptr) {
  *splits = 1;
  if (us_out) *us_out = 0.f;
  if (!vec) {
    *config = kUnalignedConfig;
    return;
  }
  // The decoder repeats a handful of problems thousands of times: remember the answers.
  struct Memo {
    int M, N, K[LH_GEMM_MAX_SEGS], flags, config, splits;
    size_t workspace_bytes;
    float us;
  };
  static thread_local Memo memo[64];
  const int flags = 1 + (ta ? 2 : 0) + (tx ? 4 : 0) + 8 * nseg + 64 * (g_config_override + 1) +
                    4096 * g_splits_override + 131072 * max_planes + (only_cell ? 1048576 : 0);
  int Kk[LH_GEMM_MAX_SEGS] = {0, 0, 0};
  for (int s = 0; s < nseg; ++s) Kk[s] = K[s];
  const unsigned h = ((unsigned)M * 2654435761u) ^ ((unsigned)N * 40503u) ^ ((unsigned)Kk[0] * 97u) ^
                     ((unsigned)Kk[1] * 31u) ^ (unsigned)Kk[2] ^ ((unsigned)flags << 20);
  Memo &e = memo[(h ^ (h >> 13)) % 64];
  if (e.flags == flags && e.M == M && e.N == N && e.K[0] == Kk[0] && e.K[1] == Kk[1] &&
      e.K[2] == Kk[2] && e.workspace_bytes == workspace_bytes) {
    *config = e.config;
    *splits = e.splits;
    if (us_out) *us_out = e.us;
    return;
  }
  static const int kSplitChoices[] = {1, 2, 3, 4, 6, 8, 12, 16};
  const Tuning *table = kTuning[ta ? 1 : (tx ? 2 : 0)];
  float best = 3.0e38f;
  *config = kUnalignedConfig;
  for (int c = 0; c < kNumConfigs; ++c) {
    if (g_config_override >= 0 && c != g_config_override) continue;
    if (only_cell && !cell_capable_index(c)) continue;
    for (int want : kSplitChoices) {
      if (only_cell && want > 1) break;
      if (!only_cell && g_splits_override > 0) want = fit_splits(M, N, g_splits_override, workspace_bytes);
      if (max_planes > 0 && want > max_planes) want = max_planes;
      if (want > 1 && fit_splits(M, N, want, workspace_bytes) < want) break;
      int S;
      const float us = predict_us(table[c], kConfigs[c], M, N, K, nseg, want, max_planes > 0, &S);
      if (us < best) {
        best = us;
        *config = c;
        *splits = S;
      }
      if (g_splits_override > 0 || (max_planes > 0 && want >= max_planes)) break;
    }
  }
  if (best > 2.9e38f) *config = -1;  // only_cell: the override names a configuration that cannot
  if (us_out) *us_out = best;
  e = Memo{M, N, {Kk[0], Kk[1], Kk[2]}, flags, *config, *splits, workspace_bytes, best};
}

struct Prepared {
  GemmArgs g;
  bool ta, tx, vec;
  int config;
};

int prepare(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX, float alpha,
            float beta, const float *bias, int act, int act_rows, const int *colmask, float *C,
            int ldc, void *workspace, size_t workspace_bytes, int max_planes, Prepared *out) {
  if (M <= 0 || N <= 0) return lh::fail_arg("lh_gemm_f32: M=%d N=%d must be positive", M, N);
  if (!segs || nseg < 1 || nseg > LH_GEMM_MAX_SEGS)
    return lh::fail_arg("lh_gemm_f32: nseg=%d outside [1,%d]", nseg, LH_GEMM_MAX_SEGS);
  if (transA && transX) return lh::fail_arg("lh_gemm_f32: transA && transX is not supported");
  if (act != LH_ACT_NONE && act != LH_ACT_TANH) return lh::fail_arg("lh_gemm_f32: act=%d", act);
  if (!C || ldc < M) return lh::fail_arg("lh_gemm_f32: C=%p ldc=%d (M=%d)", (void *)C, ldc, M);

  GemmArgs &g = out->g;
  g = GemmArgs{};
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
    // ... and the main kernel keeps per-thread byte offsets inside a slab in 32 bits.
    constexpr int kMaxLd = 1 << 22;
    vec = vec && lh::aligned16(e.A) && lh::aligned16(e.X) && e.lda % 4 == 0 && e.ldx % 4 == 0 &&
          a_extent % 4 == 0 && x_extent % 4 == 0 && e.lda < kMaxLd && e.ldx < kMaxLd;
  }
  for (int s = nseg; s < LH_GEMM_MAX_SEGS; ++s) {  // unused slots mirror segment 0 (never read)
    g.A[s] = g.A[0];
    g.X[s] = g.X[0];
    g.lda[s] = g.lda[0];
    g.ldx[s] = g.ldx[0];
    g.K[s] = g.K[0];
  }
  g.nseg = nseg;
  g.M = M;
  g.N = N;
  g.alpha = alpha;
  g.beta = beta;
  g.bias = bias;
  g.act = act;
  g.act_rows = act_rows;
  g.colmask = colmask;
  g.C = C;
  g.ldc = ldc;
  out->ta = transA != 0;
  out->tx = transX != 0;
  out->vec = vec;
  if (!workspace || !lh::aligned16(workspace)) workspace_bytes = 0;
  pick_config(M, N, g.K, nseg, transA != 0, transX != 0, vec, workspace_bytes, max_planes,
              &out->config, &g.splits);
  g.leave_partial = max_planes > 0 ? 1 : 0;
  g.ws_part = static_cast<float *>(workspace);
  g.ws_ld = plane_ld(M);
  return LH_OK;
}

}  // namespace

extern "C" int lh_gemm_ws_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA,
                              int transX, float alpha, float beta, const float *bias, int act,
                              int act_rows, const int *colmask, float *C, int ldc, void *workspace,
                              size_t workspace_bytes, lh_stream_t stream) {
  if (act_rows < 0 || act_rows > M)
    return lh::fail_arg("lh_gemm_f32: act_rows=%d outside [0,M=%d]", act_rows, M);
  Prepared p;
  const int rc = prepare(M, N, segs, nseg, transA, transX, alpha, beta, bias, act, act_rows,
                         colmask, C, ldc, workspace, workspace_bytes, 0, &p);
  if (rc != LH_OK) return rc;
  return launch_index(p.config, p.g, p.ta, p.tx, p.vec, lh::as_stream(stream));
}

extern "C" int lh_gemm_planes_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA,
                                  int transX, float beta, float *C, int ldc, void *workspace,
                                  size_t workspace_bytes, int max_planes, int *planes,
                                  lh_stream_t stream) {
  if (!planes || max_planes < 1)
    return lh::fail_arg("lh_gemm_planes_f32: planes=%p max_planes=%d", (void *)planes, max_planes);
  Prepared p;
  const int rc = prepare(M, N, segs, nseg, transA, transX, 1.f, beta, nullptr, LH_ACT_NONE, M,
                         nullptr, C, ldc, workspace, workspace_bytes, max_planes, &p);
  if (rc != LH_OK) return rc;
  // the split the launch will really use (no empty share), as launch_cfg computes it
  const Config &k = kConfigs[p.config];
  int slabs = 0;
  for (int s = 0; s < p.g.nseg; ++s) slabs += (p.g.K[s] + k.bk - 1) / k.bk;
  const int want = p.vec ? p.g.splits : 1;
  const int share = (slabs + want - 1) / want;
  *planes = (slabs + share - 1) / share;
  return launch_index(p.config, p.g, p.ta, p.tx, p.vec, lh::as_stream(stream));
}

namespace {
// The choice lh_gemm_planes_f32 makes for the stacked gate product of an LSTM cell, and whether
// that choice can carry the cell in its epilogue: aligned operands, no K split, a tile that fits LDS.
int plan_cell(int H, int B, const lh_gemm_seg *segs, int nseg, bool has_addend, const float *addend,
              int ld_addend, size_t workspace_bytes, Prepared *p, bool *fusable) {
  if (H <= 0 || B <= 0) return lh::fail_arg("lh_gate_gemm_lstm_cell: H=%d B=%d", H, B);
  float dummy;
  const int rc = prepare(4 * H, B, segs, nseg, 0, 0, 1.f, has_addend ? 1.f : 0.f, nullptr, LH_ACT_NONE,
                         4 * H, nullptr, has_addend && addend ? const_cast<float *>(addend) : &dummy,
                         has_addend && addend ? ld_addend : 4 * H,
                         workspace_bytes ? (void *)(uintptr_t)256 : nullptr, workspace_bytes,
                         has_addend ? 2 : 3, p);
  if (rc != LH_OK) return rc;
  *fusable = false;
  if (!p->vec || H % 4 != 0) return LH_OK;
  // Best unsplit launch that can carry the cell against the best launch of any kind followed by
  // the cell kernel (a launch of its own that reads the pre-activations, or S planes of them, back).
  int cfg_any, splits_any, cfg_cell, splits_cell;
  float us_any, us_cell;
  const size_t ws = workspace_bytes;
  pick_config(4 * H, B, p->g.K, nseg, false, false, true, ws, has_addend ? 2 : 3, &cfg_any, &splits_any,
              false, &us_any);
  pick_config(4 * H, B, p->g.K, nseg, false, false, true, ws, has_addend ? 2 : 3, &cfg_cell,
              &splits_cell, true, &us_cell);
  if (cfg_cell < 0) return LH_OK;
  const float cell_us = kCellFixedUs + 28.f * (float)H * (float)B / kReduceBytesPerUs;
  if (us_cell <= us_any + cell_us) {
    *fusable = true;
    p->config = cfg_cell;
    p->g.splits = 1;
  }
  return LH_OK;
}
}  // namespace

extern "C" int lh_gate_gemm_lstm_cell_plan(int H, int B, const lh_gemm_seg *segs, int nseg,
                                           int has_addend, size_t workspace_bytes, int *fusable,
                                           char *name, int name_cap) {
  if (!fusable) return lh::fail_arg("lh_gate_gemm_lstm_cell_plan: fusable is NULL");
  Prepared p;
  bool f = false;
  const int rc = plan_cell(H, B, segs, nseg, has_addend != 0, nullptr, 0, workspace_bytes, &p, &f);
  if (rc != LH_OK) return rc;
  *fusable = f ? 1 : 0;
  if (name && name_cap > 0) {
    const Config &k = kConfigs[p.config];
    if (f) snprintf(name, name_cap, "gate_gemm_cell_kernel<%d, %d, %d, %d, %d, %d>", k.bm, k.bn, k.wm, k.wn, k.wk, k.bk);
    else name[0] = 0;
  }
  return LH_OK;
}

extern "C" int lh_gate_gemm_lstm_cell_f32(int H, int B, const lh_gemm_seg *segs, int nseg,
                                          const float *addend, int ld_addend, const int *addend_col,
                                          int addend_ncols, const float *bias4h, const float *c_prev,
                                          const int *mask01, int sigmoid_f64, float cell_clip,
                                          float *c, float *h, size_t workspace_bytes,
                                          lh_stream_t stream) {
  if (!bias4h || !c_prev || !mask01 || !c || !h)
    return lh::fail_arg("lh_gate_gemm_lstm_cell_f32: a required pointer is NULL");
  if (addend && ld_addend < 4 * H)
    return lh::fail_arg("lh_gate_gemm_lstm_cell_f32: ld_addend=%d < 4H=%d", ld_addend, 4 * H);
  if (addend_col && (!addend || addend_ncols < 1))
    return lh::fail_arg("lh_gate_gemm_lstm_cell_f32: addend_col needs addend and addend_ncols >= 1");
  Prepared p;
  bool f = false;
  const int rc = plan_cell(H, B, segs, nseg, addend != nullptr, addend, ld_addend, workspace_bytes, &p, &f);
  if (rc != LH_OK) return rc;
  if (!f)
    return lh::fail_arg("lh_gate_gemm_lstm_cell_f32: this product does not run fused "
                        "(ask lh_gate_gemm_lstm_cell_plan first)");
  // Other workgroups still read the operands while one writes its cells: the outputs must not
  // overlap any X operand (c may be c_prev: a cell is read and written by one thread).
  for (int s = 0; s < nseg; ++s) {
    const float *x0 = segs[s].X, *x1 = x0 + (size_t)segs[s].ldx * B;
    const float *outs[2] = {c, h};
    for (const float *o : outs)
      if (o < x1 && x0 < o + (size_t)H * B)
        return lh::fail_arg("lh_gate_gemm_lstm_cell_f32: an output overlaps operand X of segment %d", s);
  }
  GemmArgs &g = p.g;
  g.bias = bias4h;
  g.colmask = mask01;
  g.cell_H = H;
  g.c_prev = c_prev;
  g.c_out = c;
  g.h_out = h;
  g.cell_clip = cell_clip;
  g.sigmoid_f64 = sigmoid_f64;
  g.addend_col = addend_col;
  g.addend_ncols = addend_ncols;
  return launch_cell_index(p.config, g, lh::as_stream(stream));
}

extern "C" int lh_gemm_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA, int transX,
                           float alpha, float beta, const float *bias, int act, const int *colmask,
                           float *C, int ldc, lh_stream_t stream) {
  return lh_gemm_ws_f32(M, N, segs, nseg, transA, transX, alpha, beta, bias, act, M, colmask, C,
                        ldc, nullptr, 0, stream);
}

extern "C" int lh_gemm_act_rows_f32(int M, int N, const lh_gemm_seg *segs, int nseg, int transA,
                                    int transX, float alpha, float beta, const float *bias, int act,
                                    int act_rows, const int *colmask, float *C, int ldc,
                                    lh_stream_t stream) {
  return lh_gemm_ws_f32(M, N, segs, nseg, transA, transX, alpha, beta, bias, act, act_rows, colmask,
                        C, ldc, nullptr, 0, stream);
}

extern "C" int lh_gemm_set_config_override(int config) {
  if (config >= kNumConfigs)
    return lh::fail_arg("lh_gemm_set_config_override: %d >= %d", config, kNumConfigs);
  g_config_override = config < 0 ? -1 : config;
  return kNumConfigs;
}

extern "C" int lh_gemm_set_splits_override(int splits) {
  if (splits > kMaxSplits)
    return lh::fail_arg("lh_gemm_set_splits_override: %d > %d", splits, kMaxSplits);
  g_splits_override = splits < 0 ? 0 : splits;
  return kMaxSplits;
}

extern "C" int lh_gemm_config_info(int config, int transA, int transX, int info[8]) {
  if (config < 0 || config >= kNumConfigs || !info || (transA && transX))
    return lh::fail_arg("lh_gemm_config_info: config=%d of %d, info=%p", config, kNumConfigs,
                        (void *)info);
  const Config &k = kConfigs[config];
  info[0] = k.bm, info[1] = k.bn, info[2] = k.wm, info[3] = k.wn, info[4] = k.wk, info[5] = k.bk;
  return occupancy_index(config, transA != 0, transX != 0, &info[6], &info[7]);
}

extern "C" int lh_gemm_kernel_name(int M, int N, const lh_gemm_seg *segs, int nseg, int transA,
                                   int transX, size_t workspace_bytes, int max_planes, char *name,
                                   int name_cap) {
  if (!name || name_cap < 1) return lh::fail_arg("lh_gemm_kernel_name: no output buffer");
  Prepared p;
  float dummy;
  // any aligned non-null address stands in for the workspace: nothing is launched
  const int rc = prepare(M, N, segs, nseg, transA, transX, 1.f, 0.f, nullptr, LH_ACT_NONE, M,
                         nullptr, &dummy, M, workspace_bytes ? (void *)(uintptr_t)256 : nullptr,
                         workspace_bytes, max_planes, &p);
  if (rc != LH_OK) return rc;
  const Config &k = kConfigs[p.config];
  if (p.vec)
    snprintf(name, name_cap, "gemm_kernel<%d, %d, %d, %d, %d, %d, %s, %s>", k.bm, k.bn, k.wm, k.wn,
             k.wk, k.bk, p.ta ? "true" : "false", p.tx ? "true" : "false");
  else
    snprintf(name, name_cap, "gemm_generic_kernel<%d, %d, %d, %d, %d, %d, %s, %s, false>", k.bm,
             k.bn, k.wm, k.wn, k.wk, k.bk, p.ta ? "true" : "false", p.tx ? "true" : "false");
  return LH_OK;
}
