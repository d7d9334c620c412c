// Fused LSTM cell kernels (forward and backward): one coalesced pass over HBM per cell-step.
// A thread owns VW consecutive hidden rows of one column; VW = 4 (16-byte accesses) whenever
// H % 4 == 0 and the operands are 16-byte aligned, which covers every reference configuration.
#include "lh_common.h"

namespace {

struct CellFwdArgs {
  int H, B;
  const float *pre1, *pre2, *pre3, *bias, *c_prev;
  const int *mask01;
  float cell_clip;
  float *gates, *c, *h;
  const float *drop_mask;
  float keep;
  float *h_drop;
};

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

template <int VW, bool F64>
__global__ __launch_bounds__(256) void lstm_cell_fwd_kernel(const CellFwdArgs a) {
  const int HQ = a.H / VW;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)HQ * a.B) return;
  const int b = (int)(idx / HQ);
  const int r = (int)(idx % HQ) * VW;
  const size_t o4 = (size_t)b * 4 * a.H + r;  // offset inside a 4H x B operand (gate 0)
  const size_t o1 = (size_t)b * a.H + r;      // offset inside an H x B operand

  Vec<VW> s[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    s[g].load(a.pre1 + o4 + (size_t)g * a.H);
    if (a.pre2) {
      Vec<VW> t;
      t.load(a.pre2 + o4 + (size_t)g * a.H);
#pragma unroll
      for (int i = 0; i < VW; ++i) s[g].v[i] += t.v[i];
    }
    if (a.pre3) {
      Vec<VW> t;
      t.load(a.pre3 + o4 + (size_t)g * a.H);
#pragma unroll
      for (int i = 0; i < VW; ++i) s[g].v[i] += t.v[i];
    }
    Vec<VW> bv;
    bv.load(a.bias + (size_t)g * a.H + r);
#pragma unroll
    for (int i = 0; i < VW; ++i) s[g].v[i] += bv.v[i];
  }
  Vec<VW> cp;
  cp.load(a.c_prev + o1);
  const int cm = a.mask01[b];
  const float m = (float)(cm & 1);
  const bool f32_gates = (cm & LH_MASK_F32_GATES) != 0;

  Vec<VW> c, h;
#pragma unroll
  for (int i = 0; i < VW; ++i) {
    if (F64 && f32_gates)
      lh::lstm_cell_point<false>(s[0].v[i], s[1].v[i], s[2].v[i], s[3].v[i], cp.v[i], m, a.cell_clip,
                                 c.v[i], h.v[i]);
    else
      lh::lstm_cell_point<F64>(s[0].v[i], s[1].v[i], s[2].v[i], s[3].v[i], cp.v[i], m, a.cell_clip,
                               c.v[i], h.v[i]);
  }
  if (a.gates) {
#pragma unroll
    for (int g = 0; g < 4; ++g) s[g].store(a.gates + o4 + (size_t)g * a.H);
  }
  c.store(a.c + o1);
  h.store(a.h + o1);
  if (a.h_drop) {
    Vec<VW> u, hd;
    u.load(a.drop_mask + o1);
    const float inv = 1.0f / a.keep;
#pragma unroll
    for (int i = 0; i < VW; ++i) hd.v[i] = ((float)(u.v[i] < a.keep) * inv) * h.v[i];
    hd.store(a.h_drop + o1);
  }
}

}  // namespace

extern "C" int lh_lstm_cell_fwd_f32(int H, int B, const float *pre1, const float *pre2,
                                    const float *pre3, const float *bias4h, const float *c_prev,
                                    const int *mask01, int sigmoid_f64, float cell_clip,
                                    float *gates, float *c, float *h, const float *next_drop_mask,
                                    float keep, float *h_drop, lh_stream_t stream) {
  if (H <= 0 || B <= 0) return lh::fail_arg("lh_lstm_cell_fwd_f32: H=%d B=%d", H, B);
  if (!pre1 || !bias4h || !c_prev || !mask01 || !c || !h)
    return lh::fail_arg("lh_lstm_cell_fwd_f32: a required pointer is NULL");
  if (!pre2 && pre3) return lh::fail_arg("lh_lstm_cell_fwd_f32: pre3 given without pre2");
  if (h_drop && (!next_drop_mask || !(keep > 0.f)))
    return lh::fail_arg("lh_lstm_cell_fwd_f32: h_drop needs next_drop_mask and keep > 0");

  CellFwdArgs a{H, B, pre1, pre2, pre3, bias4h, c_prev, mask01, cell_clip, gates, c, h,
                next_drop_mask, keep, h_drop};
  const bool vec = H % 4 == 0 && lh::aligned16(pre1) && lh::aligned16(pre2) &&
                   lh::aligned16(pre3) && lh::aligned16(bias4h) && lh::aligned16(c_prev) &&
                   lh::aligned16(gates) && lh::aligned16(c) && lh::aligned16(h) &&
                   lh::aligned16(next_drop_mask) && lh::aligned16(h_drop);
  const long long work = (long long)(vec ? H / 4 : H) * B;
  const dim3 grid((unsigned)((work + 255) / 256)), block(256);
  hipStream_t st = lh::as_stream(stream);
  if (vec) {
    if (sigmoid_f64) hipLaunchKernelGGL((lstm_cell_fwd_kernel<4, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((lstm_cell_fwd_kernel<4, false>), grid, block, 0, st, a);
  } else {
    if (sigmoid_f64) hipLaunchKernelGGL((lstm_cell_fwd_kernel<1, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((lstm_cell_fwd_kernel<1, false>), grid, block, 0, st, a);
  }
  return lh::check_launch("lh_lstm_cell_fwd_f32");
}
