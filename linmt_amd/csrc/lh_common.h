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

}  // namespace lh
