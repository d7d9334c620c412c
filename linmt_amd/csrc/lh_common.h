// Shared helpers for the gfx950 kernels behind the C ABI in include/linmt_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <cfloat>
#include <cstdarg>
#include <cstdio>

#include "../../include/linmt_hip.h"

namespace lh {

constexpr int kWave = 64;  // CDNA wavefront width

// Per-thread text of the last failure, read back through lh_last_error().
char *last_error_buffer();
int fail_arg(const char *fmt, ...);
int check_launch(const char *what);

inline hipStream_t as_stream(lh_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- wavefront reductions (64 lanes) -------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ double wave_max(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmax(v, __shfl_xor(v, o, kWave));
  return v;
}

// Block-wide reductions over NW wavefronts through a small LDS array (NW+ entries).
// Every thread of the block must call; the result is returned to every thread.
template <int NW, typename T>
__device__ __forceinline__ T block_sum(T v, T *lds) {
  v = wave_sum(v);
  const int w = threadIdx.x / kWave, l = threadIdx.x % kWave;
  __syncthreads();
  if (l == 0) lds[w] = v;
  __syncthreads();
  T r = lds[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r += lds[i];
  return r;
}
template <int NW, typename T>
__device__ __forceinline__ T block_max(T v, T *lds) {
  v = wave_max(v);
  const int w = threadIdx.x / kWave, l = threadIdx.x % kWave;
  __syncthreads();
  if (l == 0) lds[w] = v;
  __syncthreads();
  T r = lds[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = r > lds[i] ? r : lds[i];
  return r;
}

// Workgroups of a launch are dealt to the 8 XCDs (each with its own L2) round-robin.  Maps a
// workgroup id to a work item so that every XCD owns one contiguous range of the n items: items
// that read the same data (the beam columns of a sentence) then share an L2.
__device__ __forceinline__ int xcd_contiguous(int id, int n) {
  const int xcd = id % 8, within = id / 8;
  const int per = n / 8, rem = n % 8;
  return xcd * per + (xcd < rem ? xcd : rem) + within;
}

// The LSTM cell at one (row, column): gates from the four pre-activations (bias included), the new
// cell state (optionally clipped) and hidden state, both zeroed in padded columns (m = 0/1).
// F64 evaluates the logistic function in double as the reference's feed-input kernels do
// (src/deep_rnn_kernel.h:64-80).  Shared by the cell kernel and the matrix product that applies
// the cell in its epilogue, so that both give the same bits.
template <bool F64>
__device__ __forceinline__ float sigmoid_ref(float x) {
  if constexpr (F64) {
    return (float)(1.0 / (1.0 + exp(-1.0 * (double)x)));
  } else {
    return 1.0f / (1.0f + expf(-1.0f * x));
  }
}
template <bool F64>
__device__ __forceinline__ void lstm_cell_point(float &s0, float &s1, float &s2, float &s3,
                                                float c_prev, float m, float cell_clip, float &c,
                                                float &h) {
  const float it = sigmoid_ref<F64>(s0);
  const float ft = sigmoid_ref<F64>(s1);
  const float gt = tanhf(s2);
  const float ot = sigmoid_ref<F64>(s3);
  s0 = it, s1 = ft, s2 = gt, s3 = ot;
  float ct = ft * c_prev + it * gt;
  if (cell_clip > 0.f) ct = fminf(fmaxf(ct, -cell_clip), cell_clip);
  const float ht = ot * tanhf(ct);
  c = ct * m;
  h = ht * m;
}

}  // namespace lh
