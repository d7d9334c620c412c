// Token-index preprocessing and the sparse embedding lookup.
#include "lh_common.h"

namespace {

__global__ void preprocess_indices_kernel(const int *idx, int n, int *idx0,
                                          int *mask01, float *mask01_f) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    const int v = idx[i];
    const int valid = v != -1;
    idx0[i] = valid ? v : 0;
    mask01[i] = valid;
    if (mask01_f) mask01_f[i] = (float)valid;
  }
}

__global__ void setup_reverse_kernel(const int *__restrict__ unique, int n, int *rev, int vocab) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    const int id = unique[i];
    if (id >= 0 && id < vocab) rev[id] = i;
  }
}

// One thread moves VW consecutive embedding rows of one column.
template <int VW>
__global__ __launch_bounds__(256) void embed_lookup_kernel(const float *__restrict__ W, int E,
                                                           int V, const int *__restrict__ idx0,
                                                           int B, const float *__restrict__ mask,
                                                           float keep, float *__restrict__ out) {
  const int EQ = E / VW;
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= (long long)EQ * B) return;
  const int b = (int)(t / EQ);
  const int r = (int)(t % EQ) * VW;
  int id = idx0[b];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);  // never read outside W; callers pass ids in [0,V)
  const float *src = W + (size_t)id * E + r;
  float *dst = out + (size_t)b * E + r;
  const float inv = 1.0f / keep;
  if constexpr (VW == 4) {
    float4 x = *reinterpret_cast<const float4 *>(src);
    if (mask) {
      const float4 u = *reinterpret_cast<const float4 *>(mask + (size_t)b * E + r);
      x.x = ((float)(u.x < keep) * inv) * x.x;
      x.y = ((float)(u.y < keep) * inv) * x.y;
      x.z = ((float)(u.z < keep) * inv) * x.z;
      x.w = ((float)(u.w < keep) * inv) * x.w;
    }
    *reinterpret_cast<float4 *>(dst) = x;
  } else {
    float x = *src;
    if (mask) x = ((float)(mask[(size_t)b * E + r] < keep) * inv) * x;
    *dst = x;
  }
}

}  // namespace

extern "C" int lh_preprocess_indices_i32(const int *idx, int n, int *idx0, int *mask01,
                                         float *mask01_f, lh_stream_t stream) {
  if (n < 0 || (n > 0 && (!idx || !idx0 || !mask01)))
    return lh::fail_arg("lh_preprocess_indices_i32: n=%d or NULL pointer", n);
  if (n == 0) return LH_OK;
  const int blocks = (n + 255) / 256 < 256 ? (n + 255) / 256 : 256;
  hipLaunchKernelGGL(preprocess_indices_kernel, dim3(blocks), dim3(256), 0, lh::as_stream(stream),
                     idx, n, idx0, mask01, mask01_f);
  return lh::check_launch("lh_preprocess_indices_i32");
}

extern "C" int lh_setup_reverse_indices_i32(const int *unique, int n_unique, int *rev, int vocab,
                                            lh_stream_t stream) {
  if (n_unique < 0 || vocab <= 0 || (n_unique > 0 && (!unique || !rev)))
    return lh::fail_arg("lh_setup_reverse_indices_i32: n_unique=%d vocab=%d", n_unique, vocab);
  if (n_unique == 0) return LH_OK;
  const int blocks = (n_unique + 255) / 256 < 256 ? (n_unique + 255) / 256 : 256;
  hipLaunchKernelGGL(setup_reverse_kernel, dim3(blocks), dim3(256), 0, lh::as_stream(stream),
                     unique, n_unique, rev, vocab);
  return lh::check_launch("lh_setup_reverse_indices_i32");
}

extern "C" int lh_embed_lookup_f32(const float *W, int E, int V, const int *idx0, int B,
                                   const float *drop_mask, float keep, float *out,
                                   lh_stream_t stream) {
  if (E <= 0 || V <= 0 || B <= 0 || !W || !idx0 || !out)
    return lh::fail_arg("lh_embed_lookup_f32: E=%d V=%d B=%d or NULL pointer", E, V, B);
  if (drop_mask && !(keep > 0.f)) return lh::fail_arg("lh_embed_lookup_f32: keep=%f", keep);
  const bool vec =
      E % 4 == 0 && lh::aligned16(W) && lh::aligned16(out) && lh::aligned16(drop_mask);
  const long long work = (long long)(vec ? E / 4 : E) * B;
  const dim3 grid((unsigned)((work + 255) / 256)), block(256);
  hipStream_t st = lh::as_stream(stream);
  if (vec)
    hipLaunchKernelGGL(embed_lookup_kernel<4>, grid, block, 0, st, W, E, V, idx0, B, drop_mask,
                       keep, out);
  else
    hipLaunchKernelGGL(embed_lookup_kernel<1>, grid, block, 0, st, W, E, V, idx0, B, drop_mask,
                       keep, out);
  return lh::check_launch("lh_embed_lookup_f32");
}
