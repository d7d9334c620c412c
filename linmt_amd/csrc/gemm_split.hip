// fp32 matrix products on the bf16 matrix pipe (lh_*split* entry points of include/linmt_hip.h).
//
// Every fp32 operand a is held as three bf16 values a1 + a2 + a3 = a (a1 = bf16(a), a2 = bf16(a - a1),
// a3 = bf16(a - a1 - a2); the subtractions are exact in fp32).  A product a*x is then the sum of
// bf16 x bf16 products, each of which the matrix pipe forms exactly and adds into an fp32
// accumulator; the six of them with i + j <= 4 (a1x1, a1x2, a2x1, a1x3, a2x2, a3x1) leave out terms
// below 2^-23 |a x|, the size of one fp32 rounding.  v_mfma_f32_32x32x16_bf16 does 16 k per 32
// cycles where v_mfma_f32_32x32x2_f32 does 2 per 64, so six of them cost 3/8 of the fp32 pipe time.
//
// Operands are packed ahead of the product ("split planes"): 16-byte units of 8 consecutive k,
//   planes[(p * KG + kg) * Dp + d],  p = plane 0..2, kg = k / 8, d = row of A / column of X,
// Dp = D rounded up to 256, zero beyond D and K.  A slab (16 k) of a tile is then six contiguous
// runs of rows per operand: global -> LDS -> MFMA fragment is 16-byte copies with no shuffles, the
// LDS image of a slab is lane-linear, and the K loop carries no vector-ALU instruction.
#include <algorithm>

#include "lh_common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kPadD = 256;       // rows / columns of a packed operand are padded to this
constexpr int kGateRows = 8;     // a packed gate matrix holds 8 rows of gate i, 8 of f, 8 of c', 8 of o, and so on
constexpr int kCUs = 256;

inline int round_up(int v, int m) { return (v + m - 1) / m * m; }

// ---- packing ---------------------------------------------------------------------------------
__device__ __forceinline__ unsigned bf16_rn(float v) {
  unsigned u = __float_as_uint(v);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ float bf16_f(unsigned h) { return __uint_as_float(h << 16); }

// eight consecutive k of one row -> one unit per plane
__device__ __forceinline__ void split8(const float (&a)[8], u4v (&out)[3]) {
  unsigned h[3][8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const unsigned h1 = bf16_rn(a[j]);
    const float r1 = a[j] - bf16_f(h1);
    const unsigned h2 = bf16_rn(r1);
    const float r2 = r1 - bf16_f(h2);
    h[0][j] = h1, h[1][j] = h2, h[2][j] = bf16_rn(r2);
  }
#pragma unroll
  for (int p = 0; p < 3; ++p) {
    out[p].x = h[p][0] | (h[p][1] << 16);
    out[p].y = h[p][2] | (h[p][3] << 16);
    out[p].z = h[p][4] | (h[p][5] << 16);
    out[p].w = h[p][6] | (h[p][7] << 16);
  }
}

struct PackSrc {
  const float *src;
  long sd, sk;   // src(d, k) = src[d * sd + k * sk]
  int D, K;      // extents that exist
  int H;         // > 0: a stacked 4H x K gate matrix, rows go to cell-tile order
  u4v *planes;
  int Dp, KG, kg0, kgn;  // padded rows, k-groups of the whole operand, first k-group and count written
};
struct PackArgs {
  PackSrc s[LH_SPLIT_PACK_MAX];
};

// one thread per (k-group, packed row) of source blockIdx.y
__global__ __launch_bounds__(256) void split_pack_kernel(const PackArgs a) {
  const PackSrc &q = a.s[blockIdx.y];
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)q.Dp * q.kgn) return;
  const int dp = (int)(idx % q.Dp), kg = (int)(idx / q.Dp);
  int d = dp;
  bool have = dp < q.D;
  if (q.H > 0) {
    // packed row t*32 + g*8 + r  <-  row g*H + t*8 + r of the stacked matrix
    const int t = dp / (4 * kGateRows), g = (dp / kGateRows) % 4, r = t * kGateRows + dp % kGateRows;
    have = r < q.H;
    d = g * q.H + r;
  }
  float v[8];
  const bool vec = have && q.sk == 1 && kg * 8 + 8 <= q.K && ((q.sd | (long)(size_t)q.src / 4) % 4 == 0);
  if (vec) {
    const floatx4 *p = reinterpret_cast<const floatx4 *>(q.src + (long)d * q.sd + kg * 8);
    const floatx4 lo = p[0], hi = p[1];
    v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = kg * 8 + j;
      v[j] = have && k < q.K ? q.src[(long)d * q.sd + (long)k * q.sk] : 0.f;
    }
  }
  u4v out[3];
  split8(v, out);
#pragma unroll
  for (int p = 0; p < 3; ++p) q.planes[((long)p * q.KG + q.kg0 + kg) * q.Dp + dp] = out[p];
}

// ---- the product -----------------------------------------------------------------------------
struct SplitArgs {
  const u4v *A, *X;
  int Mp, Np, KG;  // padded rows of A, padded columns of X, k-groups (a multiple of 8)
  int M, N;        // CELL: M = H
  int tiles_n;
  // plain epilogue
  float alpha, beta;
  const float *bias;
  int act_rows;
  const int *colmask;
  float *C;
  int ldc;
  // cell epilogue
  const float *addend;
  int ld_addend;
  const int *addend_col;
  int addend_ncols;
  const float *c_prev;
  int sigmoid_f64;
  float cell_clip;
  float *c_out, *h_out;
  u4v *h_planes;   // may be null: h as split planes, k-groups hp_kg0.. of an operand with hp_KG
  int hp_KG, hp_kg0, hp_kgn, hp_Np;
};

// WK wavefront groups share a tile: a slab is 16*WK deep and group wk takes its k-groups 2wk, 2wk+1
// (a product with few tiles is bound by the chain slab -> fragments -> MFMAs -> barrier of one
// workgroup; WK shortens that chain).  The groups' partial tiles are added up through LDS.
template <int BM, int BN, int WK>
constexpr int split_lds_bytes(bool cell) {
  const int stages = 2 * 6 * WK * (BM + BN) * 16, tile = (cell || WK > 1) ? BN * (BM + 4) * 4 : 0;
  return stages > tile ? stages : tile;
}

// Waves per SIMD the register allocation must allow: three workgroups of the plain 128x128 tile
// per CU (its natural allocation sits at that step; a few registers more would halve the occupancy).
template <int BM, int BN, int WK, bool CELL>
constexpr int split_waves_per_simd() {
  return BM == 128 && BN == 128 && WK == 1 && !CELL ? 3 : 1;
}

template <int BM, int BN, int WM, int WN, int WK, bool CELL>
__global__ __launch_bounds__(64 * WM * WN * WK)
__attribute__((amdgpu_waves_per_eu(split_waves_per_simd<BM, BN, WK, CELL>()))) void gemm_split_kernel(const SplitArgs g) {
  constexpr int NT = 64 * WM * WN * WK, TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
  static_assert(FM >= 1 && FN >= 1 && TM % 32 == 0 && TN % 32 == 0, "wave tile = 32x32 MFMA tiles");
  constexpr int KGL = 2 * WK;                         // k-groups of a slab
  constexpr int UA = 3 * KGL * BM, UX = 3 * KGL * BN;  // 16-byte units of a slab: planes x k-groups x rows
  constexpr int NUA = (UA + NT - 1) / NT, NUX = (UX + NT - 1) / NT;
  constexpr bool kExactA = UA % NT == 0, kExactX = UX % NT == 0;
  constexpr int STAGE = UA + UX;
  static_assert(!CELL || BM % (4 * kGateRows) == 0, "a cell tile holds whole groups of 8 rows per gate");
  extern __shared__ u4v lds[];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wk = wave / (WM * WN), wmn = wave % (WM * WN), wm = wmn % WM, wn = wmn / WM;
  const int l32 = lane % 32, lhi = lane / 32;
  const int logical = lh::xcd_contiguous(blockIdx.x, gridDim.x);
  const int m0 = (logical / g.tiles_n) * BM, n0 = (logical % g.tiles_n) * BN;

  floatx16 acc[FN][FM];
#pragma unroll
  for (int a = 0; a < FN; ++a)
#pragma unroll
    for (int b = 0; b < FM; ++b)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[a][b][j] = 0.f;

  // Unit u of the A slab is (plane u / (KGL BM), k-group (u / BM) % KGL, row u % BM); the X units follow.
  // Scalar slab origins + per-thread byte offsets that never change: no vector ALU in the loop.
  unsigned oa[NUA], ox[NUX];
#pragma unroll
  for (int i = 0; i < NUA; ++i) {
    const int u = (tid + i * NT) % UA, p = u / (KGL * BM), kgl = (u / BM) % KGL, r = u % BM;
    oa[i] = (unsigned)((p * g.KG + kgl) * g.Mp + r) * 16u;
  }
#pragma unroll
  for (int i = 0; i < NUX; ++i) {
    const int u = (tid + i * NT) % UX, p = u / (KGL * BN), kgl = (u / BN) % KGL, r = u % BN;
    ox[i] = (unsigned)((p * g.KG + kgl) * g.Np + r) * 16u;
  }
  // Buffer loads: the descriptor and the slab origin are scalars, the unit offset a 32-bit vector
  // register -- nothing to compute per load.  (The host keeps a packed operand below 4 GiB.)
  const unsigned bytes_a = (unsigned)((size_t)3 * g.KG * g.Mp * 16 - (size_t)m0 * 16);
  const unsigned bytes_x = (unsigned)((size_t)3 * g.KG * g.Np * 16 - (size_t)n0 * 16);
  const __amdgpu_buffer_rsrc_t res_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<u4v *>(g.A + m0), 0, bytes_a, 0x00020000);
  const __amdgpu_buffer_rsrc_t res_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<u4v *>(g.X + n0), 0, bytes_x, 0x00020000);
  const unsigned step_a = (unsigned)KGL * g.Mp * 16u, step_x = (unsigned)KGL * g.Np * 16u;
  const int slabs = g.KG / KGL;
  u4v ra[2][NUA], rx[2][NUX];

  auto loads = [&](u4v (&qa)[NUA], u4v (&qx)[NUX], int sn) {
    const unsigned s = min(sn, slabs - 1);  // past the end: a harmless re-read of the last slab
    const unsigned sa = s * step_a, sx = s * step_x;
#pragma unroll
    for (int i = 0; i < NUA; ++i)
      if (kExactA || tid + i * NT < UA) qa[i] = __builtin_amdgcn_raw_buffer_load_b128(res_a, oa[i], sa, 0);
#pragma unroll
    for (int i = 0; i < NUX; ++i)
      if (kExactX || tid + i * NT < UX) qx[i] = __builtin_amdgcn_raw_buffer_load_b128(res_x, ox[i], sx, 0);
  };
  auto stores = [&](int stage, const u4v (&qa)[NUA], const u4v (&qx)[NUX]) {
    u4v *w = lds + stage * STAGE;
#pragma unroll
    for (int i = 0; i < NUA; ++i)
      if (kExactA || tid + i * NT < UA) w[tid + i * NT] = qa[i];
#pragma unroll
    for (int i = 0; i < NUX; ++i)
      if (kExactX || tid + i * NT < UX) w[UA + tid + i * NT] = qx[i];
  };
  const int fa0 = (2 * wk + lhi) * BM + wm * TM + l32, fx0 = UA + (2 * wk + lhi) * BN + wn * TN + l32;
  // One slab: its fragments, the next slab from the staging registers to the other LDS stage, the
  // loads of the slab after the next two, 6 MFMAs per 32x32 tile (smallest terms first), barrier.
  auto body = [&](int stage, u4v (&qa)[NUA], u4v (&qx)[NUX], int sn) {
    const u4v *b = lds + stage * STAGE;
    bf16x8 fa[3][FM], fx[3][FN];
#pragma unroll
    for (int p = 0; p < 3; ++p) {
#pragma unroll
      for (int f = 0; f < FM; ++f) fa[p][f] = __builtin_bit_cast(bf16x8, b[fa0 + p * KGL * BM + f * 32]);
#pragma unroll
      for (int f = 0; f < FN; ++f) fx[p][f] = __builtin_bit_cast(bf16x8, b[fx0 + p * KGL * BN + f * 32]);
    }
    stores(stage ^ 1, qa, qx);
    loads(qa, qx, sn);
    constexpr int PA[6] = {2, 1, 0, 1, 0, 0}, PX[6] = {0, 1, 2, 0, 1, 0};
#pragma unroll
    for (int t = 0; t < 6; ++t)
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int bb = 0; bb < FM; ++bb)
          // operands swapped on purpose: consecutive m in consecutive lanes of every accumulator
          acc[a][bb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fx[PX[t]][a], fa[PA[t]][bb], acc[a][bb],
                                                               0, 0, 0);
    __syncthreads();
  };
  loads(ra[0], rx[0], 0);
  loads(ra[1], rx[1], 1);
  stores(0, ra[0], rx[0]);
  loads(ra[0], rx[0], 2);
  __syncthreads();
  int s = 0;
  for (; s + 1 < slabs; s += 2) {
    body(0, ra[1], rx[1], s + 3);
    body(1, ra[0], rx[0], s + 4);
  }
  if (s < slabs) body(0, ra[1], rx[1], s + 3);

  constexpr int LDS_M = BM + 4;
  float *const S = reinterpret_cast<float *>(lds);  // the tile as S[n][m]; the slab stages are dead
  if constexpr (WK > 1) {
    // fixed order: group WK-1 stores its partial tile, the groups below add theirs one after the
    // other, group 0 keeps the sum in its registers (plain epilogue) or leaves it in S (cell)
#pragma unroll
    for (int turn = WK - 1; turn >= (CELL ? 0 : 1); --turn) {
      if (wk == turn) {
#pragma unroll
        for (int a = 0; a < FN; ++a)
#pragma unroll
          for (int b = 0; b < FM; ++b)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
              float *e = S + (wn * TN + a * 32 + lhi * 4 + (j / 4) * 8 + (j % 4)) * LDS_M + wm * TM + b * 32 + l32;
              *e = turn == WK - 1 ? acc[a][b][j] : *e + acc[a][b][j];
            }
      }
      __syncthreads();
    }
    if constexpr (!CELL) {
      if (wk > 0) return;
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b)
#pragma unroll
          for (int j = 0; j < 16; ++j)
            acc[a][b][j] += S[(wn * TN + a * 32 + lhi * 4 + (j / 4) * 8 + (j % 4)) * LDS_M + wm * TM + b * 32 + l32];
    }
  }

  if constexpr (CELL) {
    // The four gates of a cell sit in different wavefronts: the tile goes through LDS, then every
    // thread takes 8 consecutive rows of one column, which is also one 16-byte unit of h's split
    // planes.
    if constexpr (WK == 1) {
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b)
#pragma unroll
          for (int j = 0; j < 16; ++j)
            S[(wn * TN + a * 32 + lhi * 4 + (j / 4) * 8 + (j % 4)) * LDS_M + wm * TM + b * 32 + l32] = acc[a][b][j];
      __syncthreads();
    }
    const int H = g.M;
    constexpr int kGroups = BM / (4 * kGateRows);  // groups of 8 gate rows in the tile
    constexpr int kUnits = kGroups * BN;
    for (int idx = tid; idx < kUnits; idx += NT) {
      const int rq = idx % kGroups, nl = idx / kGroups;
      const int r = (m0 / 4) + rq * 8, n = n0 + nl;   // first of 8 rows of every gate
      if (r >= H || n >= g.N) continue;               // H % 8 == 0: a unit is whole or absent
      float pre[4][8];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const floatx4 *sp = reinterpret_cast<const floatx4 *>(S + nl * LDS_M + rq * 4 * kGateRows + q * kGateRows);
        const floatx4 *bp = reinterpret_cast<const floatx4 *>(g.bias + (size_t)q * H + r);
        const floatx4 s0 = sp[0], s1 = sp[1], b0 = bp[0], b1 = bp[1];
        float v[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        const float bv[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
        if (g.addend) {
          int col = n;
          if (g.addend_col) col = min(max(g.addend_col[n], 0), g.addend_ncols - 1);
          const floatx4 *ap = reinterpret_cast<const floatx4 *>(g.addend + (size_t)col * g.ld_addend + (size_t)q * H + r);
          const floatx4 a0 = ap[0], a1 = ap[1];
          const float av[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
          for (int j = 0; j < 8; ++j) v[j] += av[j];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) pre[q][j] = v[j] + bv[j];
      }
      const floatx4 *cp = reinterpret_cast<const floatx4 *>(g.c_prev + (size_t)n * H + r);
      const floatx4 c0 = cp[0], c1 = cp[1];
      const float cprev[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
      const int cm = g.colmask[n];
      const float mask = (float)(cm & 1);
      const bool f64 = g.sigmoid_f64 && !(cm & LH_MASK_F32_GATES);
      float c[8], h[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (f64)
          lh::lstm_cell_point<true>(pre[0][j], pre[1][j], pre[2][j], pre[3][j], cprev[j], mask, g.cell_clip, c[j], h[j]);
        else
          lh::lstm_cell_point<false>(pre[0][j], pre[1][j], pre[2][j], pre[3][j], cprev[j], mask, g.cell_clip, c[j], h[j]);
      }
      floatx4 *co = reinterpret_cast<floatx4 *>(g.c_out + (size_t)n * H + r);
      floatx4 *ho = reinterpret_cast<floatx4 *>(g.h_out + (size_t)n * H + r);
      co[0] = floatx4{c[0], c[1], c[2], c[3]};
      co[1] = floatx4{c[4], c[5], c[6], c[7]};
      ho[0] = floatx4{h[0], h[1], h[2], h[3]};
      ho[1] = floatx4{h[4], h[5], h[6], h[7]};
      if (g.h_planes) {
        u4v out[3];
        split8(h, out);
#pragma unroll
        for (int p = 0; p < 3; ++p)
          g.h_planes[((size_t)p * g.hp_KG + g.hp_kg0 + r / 8) * g.hp_Np + n] = out[p];
        // k-groups of padding behind the segment must read as zeros whatever an earlier step (with
        // another column count, hence another layout) left there
        if (r / 8 == H / 8 - 1) {
          for (int kg = H / 8; kg < g.hp_kgn; ++kg)
#pragma unroll
            for (int p = 0; p < 3; ++p)
              g.h_planes[((size_t)p * g.hp_KG + g.hp_kg0 + kg) * g.hp_Np + n] = u4v{0u, 0u, 0u, 0u};
        }
      }
    }
    return;
  }

  // Epilogue: accumulator register j of lane l is C[m = .. + l%32][n = .. + 8*(j/4) + 4*(l/32) + j%4].
  const bool use_beta = g.beta != 0.f;
#pragma unroll
  for (int a = 0; a < FN; ++a) {
#pragma unroll
    for (int b = 0; b < FM; ++b) {
      const int m = m0 + wm * TM + b * 32 + l32;
      if (m >= g.M) continue;
      const float bv = g.bias ? g.bias[m] : 0.f;
      const bool do_tanh = m < g.act_rows;
      const int nb = n0 + wn * TN + a * 32 + lhi * 4;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int n = nb + (j / 4) * 8 + (j % 4);
        if (n >= g.N) continue;
        float *cp = g.C + (size_t)n * g.ldc + m;
        float v = g.alpha * acc[a][b][j];
        if (use_beta) v += g.beta * *cp;
        v += bv;
        if (do_tanh) v = tanhf(v);
        if (g.colmask) v *= (float)g.colmask[n];
        *cp = v;
      }
    }
  }
}

struct SplitConfig {
  int bm, bn, wm, wn, wk;
};
// plain products (the last entry is reachable by override only)
constexpr SplitConfig kPlain[] = {{128, 128, 2, 2, 1}, {128, 64, 2, 2, 1}, {128, 96, 4, 1, 2}, {128, 64, 2, 2, 2},
                                  {64, 96, 2, 1, 4},   {64, 64, 2, 1, 4},  {64, 32, 2, 1, 4},  {256, 128, 4, 2, 1}};
constexpr int kNumPlain = sizeof(kPlain) / sizeof(kPlain[0]);
// cell products (a tile of BM rows holds BM/4 rows of each gate)
constexpr SplitConfig kCell[] = {{128, 96, 4, 1, 2}, {128, 64, 2, 2, 2}, {128, 32, 4, 1, 2}, {64, 96, 2, 1, 4},
                                 {64, 64, 2, 1, 4},  {64, 64, 2, 2, 2},  {64, 32, 2, 1, 4},  {32, 32, 1, 1, 8}};
constexpr int kNumCell = sizeof(kCell) / sizeof(kCell[0]);
constexpr int kMaxKGL = 16;  // k-groups of the deepest slab: operands are padded to a multiple of it

thread_local int g_split_override = -1;

template <int BM, int BN, int WM, int WN, int WK, bool CELL>
int launch_split(SplitArgs &g, hipStream_t s, const char *what) {
  static_assert(split_lds_bytes<BM, BN, WK>(CELL) <= 160 * 1024, "LDS capacity of a CU");
  static_assert(64 * WM * WN * WK <= 1024, "workgroup size");
  const int tiles_m = CELL ? (4 * g.M + BM - 1) / BM : (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  // The kernel reads whole tiles and whole slabs.  Rows of A are padded to whole tiles; a tile of X
  // may reach past the padded columns (BN = 96): what it reads there belongs to other k-groups or,
  // past the end of the operand, comes back as zeros from the range-checked buffer loads, and it
  // only feeds accumulator columns >= N, which are never stored.
  if (tiles_m * BM > g.Mp || g.KG % (2 * WK))
    return lh::fail_arg("%s: %d row tiles of %d exceed the %d padded rows, or %d k-groups are not whole slabs",
                        what, tiles_m, BM, g.Mp, g.KG);
  constexpr int bytes = split_lds_bytes<BM, BN, WK>(CELL);
  static thread_local bool raised[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return lh::fail_arg("%s: hipGetDevice", what);
  if (bytes > 64 * 1024 && !raised[dev]) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_split_kernel<BM, BN, WM, WN, WK, CELL>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
      return lh::fail_arg("%s: cannot raise the LDS limit to %d bytes", what, bytes);
    raised[dev] = true;
  }
  gemm_split_kernel<BM, BN, WM, WN, WK, CELL><<<tiles_m * g.tiles_n, 64 * WM * WN * WK, bytes, s>>>(g);
  return lh::check_launch(what);
}

int launch_plain_index(int c, SplitArgs &g, hipStream_t s) {
  const char *w = "lh_gemm_split_f32";
  switch (c) {
    case 0: return launch_split<128, 128, 2, 2, 1, false>(g, s, w);
    case 1: return launch_split<128, 64, 2, 2, 1, false>(g, s, w);
    case 2: return launch_split<128, 96, 4, 1, 2, false>(g, s, w);
    case 3: return launch_split<128, 64, 2, 2, 2, false>(g, s, w);
    case 4: return launch_split<64, 96, 2, 1, 4, false>(g, s, w);
    case 5: return launch_split<64, 64, 2, 1, 4, false>(g, s, w);
    case 6: return launch_split<64, 32, 2, 1, 4, false>(g, s, w);
    default: return launch_split<256, 128, 4, 2, 1, false>(g, s, w);
  }
}
int launch_cell_index(int c, SplitArgs &g, hipStream_t s) {
  const char *w = "lh_gate_gemm_split_lstm_cell_f32";
  switch (c) {
    case 0: return launch_split<128, 96, 4, 1, 2, true>(g, s, w);
    case 1: return launch_split<128, 64, 2, 2, 2, true>(g, s, w);
    case 2: return launch_split<128, 32, 4, 1, 2, true>(g, s, w);
    case 3: return launch_split<64, 96, 2, 1, 4, true>(g, s, w);
    case 4: return launch_split<64, 64, 2, 1, 4, true>(g, s, w);
    case 5: return launch_split<64, 64, 2, 2, 2, true>(g, s, w);
    case 6: return launch_split<64, 32, 2, 1, 4, true>(g, s, w);
    default: return launch_split<32, 32, 1, 1, 8, true>(g, s, w);
  }
}

// Thresholds on the number of tiles, from sweeps over 48..768 columns (M = 30000: several
// workgroups of a wide tile per CU; M = 4000 and 2000: few row tiles, a workgroup alone on its CU,
// where wave groups that split K shorten the chain of slabs each workgroup walks).
int choose(const SplitConfig *, int, int n, int rows_tiles128, int M, int N, bool cell) {
  if (g_split_override >= 0 && g_split_override < n) return g_split_override;
  const int t128 = cell ? rows_tiles128 : (M + 127) / 128, t64 = cell ? (M + 63) / 64 : (M + 63) / 64;
  auto cols = [&](int bn) { return (N + bn - 1) / bn; };
  if (cell) {  // M = 4H
    if (4 * t128 * cols(96) >= 3 * kCUs) return 0;  // 128 x 96, 2 wave groups
    if (t128 * cols(64) >= 224) return 1;           // 128 x 64, 2 wave groups
    if (t64 * cols(96) >= 160) return 3;            //  64 x 96, 4 wave groups
    if (t64 * cols(64) >= 160) return 4;            //  64 x 64, 4 wave groups
    return 6;                                       //  64 x 32, 4 wave groups
  }
  if (2 * t128 * cols(128) >= 3 * kCUs) return 0;   // 128 x 128
  if (2 * t128 * cols(64) >= 3 * kCUs) return 1;    // 128 x 64
  if (4 * t128 * cols(96) >= 3 * kCUs) return 2;    // 128 x 96, 2 wave groups
  if (t128 * cols(64) >= 224) return 3;             // 128 x 64, 2 wave groups
  if (t64 * cols(96) >= 160) return 4;              //  64 x 96, 4 wave groups
  if (t64 * cols(64) >= 160) return 5;              //  64 x 64, 4 wave groups
  return 6;                                         //  64 x 32, 4 wave groups
}

int check_planes(const char *what, const void *p, const char *name) {
  if (!p) return lh::fail_arg("%s: %s is NULL", what, name);
  if (!lh::aligned16(p)) return lh::fail_arg("%s: %s must be 16-byte aligned", what, name);
  return LH_OK;
}

}  // namespace

extern "C" int lh_split_kgroups(int K) { return K <= 0 ? 0 : (K + 7) / 8; }

extern "C" int lh_split_kgroups_padded(int kgroups) { return kgroups <= 0 ? 0 : round_up(kgroups, kMaxKGL); }

extern "C" int lh_split_padded(int D) { return D <= 0 ? 0 : round_up(D, kPadD); }

extern "C" int lh_split_gate_rows(int H) { return H <= 0 ? 0 : (H + kGateRows - 1) / kGateRows * 4 * kGateRows; }

extern "C" size_t lh_split_bytes(int D, int kgroups) {
  if (D <= 0 || kgroups <= 0) return 0;
  return (size_t)3 * kgroups * round_up(D, kPadD) * 16;
}

extern "C" int lh_split_pack_f32(const lh_split_source *srcs, int n, lh_stream_t stream) {
  if (n < 1 || n > LH_SPLIT_PACK_MAX || !srcs)
    return lh::fail_arg("lh_split_pack_f32: 1..%d sources, got %d", LH_SPLIT_PACK_MAX, n);
  PackArgs a;
  long most = 0;
  for (int i = 0; i < n; ++i) {
    const lh_split_source &q = srcs[i];
    if (!q.src || q.D < 1 || q.K < 1 || q.ld < 1)
      return lh::fail_arg("lh_split_pack_f32: source %d: src=%p D=%d K=%d ld=%d", i, (const void *)q.src, q.D, q.K, q.ld);
    if (q.ld < (q.k_contiguous ? q.K : (q.gate_H > 0 ? 4 * q.gate_H : q.D)))
      return lh::fail_arg("lh_split_pack_f32: source %d: ld=%d is smaller than the contiguous extent", i, q.ld);
    if (q.gate_H > 0 && q.D != 4 * q.gate_H)
      return lh::fail_arg("lh_split_pack_f32: source %d: a stacked gate matrix has D = 4 * gate_H rows (D=%d, gate_H=%d)", i, q.D, q.gate_H);
    const int rc = check_planes("lh_split_pack_f32", q.planes, "planes");
    if (rc != LH_OK) return rc;
    const int kgn = q.kgroups;
    if (kgn < lh_split_kgroups(q.K) || q.kgroups_total % kMaxKGL || q.kg_offset < 0 ||
        q.kg_offset + kgn > q.kgroups_total)
      return lh::fail_arg("lh_split_pack_f32: source %d: k-groups [%d, %d) must hold K=%d and fit an operand of %d "
                          "(a multiple of %d)", i, q.kg_offset, q.kg_offset + kgn, q.K, q.kgroups_total, kMaxKGL);
    const int Dp = q.gate_H > 0 ? round_up(lh_split_gate_rows(q.gate_H), kPadD) : round_up(q.D, kPadD);
    if ((size_t)3 * q.kgroups_total * Dp * 16 >= ((size_t)1 << 32))
      return lh::fail_arg("lh_split_pack_f32: source %d: the packed operand must stay below 4 GiB", i);
    PackSrc &o = a.s[i];
    o.src = q.src;
    o.sd = q.k_contiguous ? q.ld : 1;
    o.sk = q.k_contiguous ? 1 : q.ld;
    o.D = q.D, o.K = q.K, o.H = q.gate_H > 0 ? q.gate_H : 0;
    o.planes = reinterpret_cast<u4v *>(q.planes);
    o.Dp = Dp, o.KG = q.kgroups_total, o.kg0 = q.kg_offset, o.kgn = kgn;
    most = std::max(most, (long)Dp * kgn);
  }
  for (int i = n; i < LH_SPLIT_PACK_MAX; ++i) a.s[i] = a.s[0];
  const dim3 grid((unsigned)((most + 255) / 256), (unsigned)n);
  split_pack_kernel<<<grid, 256, 0, lh::as_stream(stream)>>>(a);
  return lh::check_launch("lh_split_pack_f32");
}

extern "C" int lh_gemm_split_f32(int M, int N, int kgroups, const void *A_planes, const void *X_planes,
                                 float alpha, float beta, const float *bias, int act, int act_rows,
                                 const int *colmask, float *C, int ldc, lh_stream_t stream) {
  if (M < 1 || N < 1 || kgroups < kMaxKGL || kgroups % kMaxKGL || !C || ldc < M)
    return lh::fail_arg("lh_gemm_split_f32: M=%d N=%d kgroups=%d (a multiple of %d) C=%p ldc=%d", M, N, kgroups,
                        kMaxKGL, (void *)C, ldc);
  if (act != LH_ACT_NONE && act != LH_ACT_TANH) return lh::fail_arg("lh_gemm_split_f32: act=%d", act);
  int rc = check_planes("lh_gemm_split_f32", A_planes, "A_planes");
  if (rc == LH_OK) rc = check_planes("lh_gemm_split_f32", X_planes, "X_planes");
  if (rc != LH_OK) return rc;
  SplitArgs g{};
  g.A = reinterpret_cast<const u4v *>(A_planes), g.X = reinterpret_cast<const u4v *>(X_planes);
  g.Mp = round_up(M, kPadD), g.Np = round_up(N, kPadD), g.KG = kgroups;
  if ((size_t)3 * kgroups * std::max(g.Mp, g.Np) * 16 >= ((size_t)1 << 32))
    return lh::fail_arg("lh_gemm_split_f32: a packed operand must stay below 4 GiB");
  g.M = M, g.N = N;
  g.alpha = alpha, g.beta = beta, g.bias = bias;
  g.act_rows = act == LH_ACT_TANH ? (act_rows < 0 ? M : std::min(act_rows, M)) : 0;
  g.colmask = colmask, g.C = C, g.ldc = ldc;
  return launch_plain_index(choose(kPlain, 0, kNumPlain, 0, M, N, false), g, lh::as_stream(stream));
}

extern "C" int lh_gate_gemm_split_lstm_cell_f32(int H, int B, int kgroups, const void *W_planes,
                                                const void *X_planes, const float *addend, int ld_addend,
                                                const int *addend_col, int addend_ncols,
                                                const float *bias4h, const float *c_prev,
                                                const int *mask01, int sigmoid_f64, float cell_clip,
                                                float *c, float *h, void *h_planes,
                                                int hp_kgroups_total, int hp_kg_offset, int hp_kgroups,
                                                lh_stream_t stream) {
  const char *what = "lh_gate_gemm_split_lstm_cell_f32";
  if (H < 8 || H % 8 || B < 1 || kgroups < kMaxKGL || kgroups % kMaxKGL)
    return lh::fail_arg("%s: H=%d (a multiple of 8) B=%d kgroups=%d (a multiple of %d)", what, H, B, kgroups, kMaxKGL);
  if (!bias4h || !c_prev || !mask01 || !c || !h) return lh::fail_arg("%s: a NULL operand", what);
  if (!lh::aligned16(bias4h) || !lh::aligned16(c_prev) || !lh::aligned16(c) || !lh::aligned16(h))
    return lh::fail_arg("%s: bias4h, c_prev, c and h must be 16-byte aligned", what);
  if (addend && (!lh::aligned16(addend) || ld_addend < 4 * H || ld_addend % 4))
    return lh::fail_arg("%s: addend must be 16-byte aligned with ld_addend >= 4H, a multiple of 4 (ld_addend=%d)", what, ld_addend);
  if (addend && addend_col && addend_ncols < 1) return lh::fail_arg("%s: addend_ncols=%d", what, addend_ncols);
  int rc = check_planes(what, W_planes, "W_planes");
  if (rc == LH_OK) rc = check_planes(what, X_planes, "X_planes");
  if (rc != LH_OK) return rc;
  SplitArgs g{};
  g.A = reinterpret_cast<const u4v *>(W_planes), g.X = reinterpret_cast<const u4v *>(X_planes);
  g.Mp = round_up(lh_split_gate_rows(H), kPadD), g.Np = round_up(B, kPadD), g.KG = kgroups;
  g.M = H, g.N = B;
  g.bias = bias4h, g.colmask = mask01;
  g.addend = addend, g.ld_addend = ld_addend, g.addend_col = addend ? addend_col : nullptr;
  g.addend_ncols = addend_ncols;
  g.c_prev = c_prev, g.sigmoid_f64 = sigmoid_f64, g.cell_clip = cell_clip, g.c_out = c, g.h_out = h;
  if (h_planes) {
    rc = check_planes(what, h_planes, "h_planes");
    if (rc != LH_OK) return rc;
    if (hp_kgroups < H / 8 || hp_kgroups_total % kMaxKGL || hp_kg_offset < 0 ||
        hp_kg_offset + hp_kgroups > hp_kgroups_total)
      return lh::fail_arg("%s: k-groups [%d, %d) of h must hold H=%d and fit an operand of %d", what, hp_kg_offset,
                          hp_kg_offset + hp_kgroups, H, hp_kgroups_total);
    g.h_planes = reinterpret_cast<u4v *>(h_planes);
    g.hp_KG = hp_kgroups_total, g.hp_kg0 = hp_kg_offset, g.hp_kgn = hp_kgroups, g.hp_Np = round_up(B, kPadD);
  }
  const int tiles128 = (4 * H + 127) / 128;
  return launch_cell_index(choose(kCell, 0, kNumCell, tiles128, 4 * H, B, true), g, lh::as_stream(stream));
}

extern "C" int lh_gemm_split_kernel_name(int cell, int M, int N, char *name, int name_cap) {
  if (!name || name_cap < 1 || M < 1 || N < 1) return lh::fail_arg("lh_gemm_split_kernel_name: M=%d N=%d", M, N);
  const SplitConfig &k = cell ? kCell[choose(kCell, 0, kNumCell, (4 * M + 127) / 128, 4 * M, N, true)]
                              : kPlain[choose(kPlain, 0, kNumPlain, 0, M, N, false)];
  snprintf(name, name_cap, "gemm_split_kernel<%d, %d, %d, %d, %d, %s>", k.bm, k.bn, k.wm, k.wn, k.wk,
           cell ? "true" : "false");
  return LH_OK;
}

extern "C" int lh_gemm_split_set_config_override(int config) {
  g_split_override = config < 0 ? -1 : config;
  return kNumPlain > kNumCell ? kNumPlain : kNumCell;  // an index past a table's end leaves that table's choice alone
}
