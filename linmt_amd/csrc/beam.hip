// Beam-search bookkeeping on the device: per-sentence merge of the per-column candidates and the
// back-pointer gather of every recurrent state tensor in one launch.
#include "lh_common.h"

namespace {

constexpr int kMergeThreads = 1024;
constexpr int kParts = 4;  // lanes that share one candidate in the merge
constexpr int kMaxCand = 4096;

struct MergeArgs {
  int n_sent, beam, K, step;
  const int *limit;
  const float *cand_logp;
  const int *cand_id;
  const float *logp_eof;
  const float *prev_score;
  float diversity, penalty;
  int start_id, eof_id;
  int *tok, *backptr;
  float *score;
  int *fin_count, *fin_beam;
  float *fin_score;
  // optional: sentence s is at step `step - start[s]` (a decoder whose sentences start at different
  // ticks); NULL = every sentence is at `step`
  const int *start;
};

// One workgroup merges one sentence.  Candidates are ranked by counting how many others precede
// them in the total order (score desc, beam column asc, vocab id asc); slots and finished indices
// follow from prefix counts over that order, which is what Decoder::ExpandHypothesis gets by
// popping its global heap.  `write`: this workgroup stores the step's outputs (several workgroups
// may merge the same sentence, each for its own use of the result).  s_bp (LDS, beam entries)
// receives the back-pointers; valid for the whole workgroup after a barrier.
__device__ __forceinline__ void merge_sentence(const MergeArgs &a, const int s, const bool write,
                                               int *s_bp) {
  __shared__ float s_score[kMaxCand];
  __shared__ int s_id[kMaxCand];
  __shared__ short s_col[kMaxCand];
  __shared__ short s_order[kMaxCand];
  __shared__ unsigned char s_flag[kMaxCand];
  __shared__ int s_total[2];  // slot-taking candidates; finished hypotheses the walk reaches

  const int tid = threadIdx.x;
  const int beam = a.beam, K = a.K;
  const int c0 = s * beam;  // first global column of this sentence
  const int limit = a.limit[s];
  const int step = a.start ? a.step - a.start[s] : a.step;

  if (step >= limit || step < 0) {
    // finish (== limit) or idle (> limit, or a slot whose sentence starts at a later tick): no
    // expansion.
    for (int i = tid; i < beam; i += kMergeThreads) {
      s_bp[i] = c0 + i;
      if (!write) continue;
      a.tok[c0 + i] = a.eof_id;
      a.backptr[c0 + i] = c0 + i;
      float sc = a.prev_score[c0 + i];
      if (step == limit) {
        sc = sc + (a.logp_eof[c0 + i] + a.penalty);  // decoder.h:506 adds (log p + penalty)
        a.fin_beam[c0 + i] = i;
        a.fin_score[c0 + i] = sc;
      }
      a.score[c0 + i] = sc;
    }
    if (tid == 0 && write) a.fin_count[s] = step == limit ? beam : 0;
    return;
  }

  const int cols = step == 0 ? 1 : beam;
  const int C = cols * K;
  if (tid < 2) s_total[tid] = 0;
  for (int e = tid; e < C; e += kMergeThreads) {
    const int i = e / K, k = e % K;
    const float rank_penalty = (float)(k + 1) * a.diversity;
    s_score[e] = a.cand_logp[(size_t)(c0 + i) * K + k] + a.prev_score[c0 + i] - rank_penalty;
    s_id[e] = a.cand_id[(size_t)(c0 + i) * K + k];
    s_col[e] = (short)i;
  }
  __syncthreads();
  // rank of every candidate in the total order; s_order[rank] = candidate, s_flag[rank] = what the
  // walk does with it (1 takes a slot, 2 finished hypothesis, 0 dropped <START>).  Four
  // neighbouring lanes share a candidate and each compares it with a quarter of the others.
  const int part = tid % kParts;
  for (int e = tid / kParts; e < C; e += kMergeThreads / kParts) {
    const float sc = s_score[e];
    const int id = s_id[e], col = s_col[e];
    int before = 0;
#pragma unroll 4
    for (int o = part; o < C; o += kParts) {
      const float so = s_score[o];
      const bool first = so > sc || (so == sc && (s_col[o] < col || (s_col[o] == col && s_id[o] < id)));
      before += first ? 1 : 0;
    }
#pragma unroll
    for (int d = 1; d < kParts; d *= 2) before += __shfl_xor(before, d);
    if (part == 0) {
      s_order[before] = (short)e;
      s_flag[before] = id == a.start_id ? 0 : (id == a.eof_id ? 2 : 1);
    }
  }
  __syncthreads();
  // The reference pops the global heap until `beam` slots are filled.  Entry r is reached iff fewer
  // than `beam` slot-taking entries precede it; its slot / finished index is the count of such
  // entries before it -- a prefix count taken per entry (again by four lanes), so nothing walks
  // the list serially.
  for (int r = tid / kParts; r < C; r += kMergeThreads / kParts) {
    int slots = 0, fins = 0;
#pragma unroll 4
    for (int q = part; q < r; q += kParts) {
      const int f = s_flag[q];
      slots += f == 1 ? 1 : 0;
      fins += f == 2 ? 1 : 0;
    }
#pragma unroll
    for (int d = 1; d < kParts; d *= 2) {
      slots += __shfl_xor(slots, d);
      fins += __shfl_xor(fins, d);
    }
    if (part != 0) continue;
    const int f = s_flag[r];
    if (f == 1) atomicAdd(&s_total[0], 1);
    if (slots < beam && f != 0) {
      const int e = s_order[r];
      const float sc = s_score[e] + a.penalty;
      if (f == 2) {
        atomicAdd(&s_total[1], 1);
        if (fins < beam && write) {  // at most one <EOF> candidate per column exists
          a.fin_beam[c0 + fins] = s_col[e];
          a.fin_score[c0 + fins] = sc;
        }
      } else {
        s_bp[slots] = c0 + s_col[e];
        if (write) {
          a.tok[c0 + slots] = s_id[e];
          a.backptr[c0 + slots] = c0 + s_col[e];
          a.score[c0 + slots] = sc;
        }
      }
    }
  }
  __syncthreads();
  // slots left empty when the candidates run out (the reference pops an empty heap)
  for (int i = min(s_total[0], beam) + tid; i < beam; i += kMergeThreads) {
    s_bp[i] = c0;
    if (!write) continue;
    a.tok[c0 + i] = a.eof_id;
    a.backptr[c0 + i] = c0;
    a.score[c0 + i] = -FLT_MAX;
  }
  if (tid == 0 && write) a.fin_count[s] = min(s_total[1], beam);
}

constexpr int kMaxBeam = 256;  // back-pointers of a sentence kept in LDS

__global__ __launch_bounds__(kMergeThreads) void beam_merge_kernel(const MergeArgs a) {
  __shared__ int s_bp[kMaxBeam];
  merge_sentence(a, blockIdx.x, true, s_bp);
}

struct GatherArgs {
  const float *src[LH_GATHER_MAX_TENSORS];
  float *dst[LH_GATHER_MAX_TENSORS];
  int H, B_src;
  const int *backptr;
};

template <int VW>
__global__ __launch_bounds__(256) void beam_gather_kernel(const GatherArgs a) {
  const int HQ = a.H / VW;
  const int t = blockIdx.z;
  const int k = blockIdx.y;
  int from = a.backptr[k];
  from = from < 0 ? 0 : (from >= a.B_src ? a.B_src - 1 : from);
  const float *src = a.src[t] + (size_t)from * a.H;
  float *dst = a.dst[t] + (size_t)k * a.H;
  for (int q = blockIdx.x * 256 + threadIdx.x; q < HQ; q += gridDim.x * 256) {
    if constexpr (VW == 4)
      reinterpret_cast<float4 *>(dst)[q] = reinterpret_cast<const float4 *>(src)[q];
    else
      dst[q] = src[q];
  }
}

// Merge + gather in one launch.  blockIdx.y = sentence, blockIdx.x = one of gridDim.x workgroups
// that each merge the sentence (the merge reads nothing that any of them writes), the first one
// storing the step's outputs; then the workgroups share the sentence's column copies
// dst_t[:, s*beam + i] = src_t[:, backptr[s*beam + i]] between them, 256 threads per column.
template <int VW>
__global__ __launch_bounds__(kMergeThreads) void beam_merge_gather_kernel(const MergeArgs a,
                                                                          const GatherArgs ga,
                                                                          const int n_tensors) {
  __shared__ int s_bp[kMaxBeam];
  const int s = blockIdx.y;
  merge_sentence(a, s, blockIdx.x == 0, s_bp);
  __syncthreads();
  const int beam = a.beam, c0 = s * beam;
  const int HQ = ga.H / VW;
  const int sub = threadIdx.x / 256, lane = threadIdx.x % 256;
  constexpr int kSubs = kMergeThreads / 256;
  for (int it = blockIdx.x * kSubs + sub; it < n_tensors * beam; it += gridDim.x * kSubs) {
    const int t = it / beam, i = it % beam;
    int from = s_bp[i];
    from = from < 0 ? 0 : (from >= ga.B_src ? ga.B_src - 1 : from);
    const float *src = ga.src[t] + (size_t)from * ga.H;
    float *dst = ga.dst[t] + (size_t)(c0 + i) * ga.H;
    for (int q = lane; q < HQ; q += 256) {
      if constexpr (VW == 4)
        reinterpret_cast<float4 *>(dst)[q] = reinterpret_cast<const float4 *>(src)[q];
      else
        dst[q] = src[q];
    }
  }
}

// A decoder that keeps its beam columns busy: a finished sentence's columns ("slot") are handed to
// the next sentence.  One launch admits up to LH_STREAM_ADMIT_MAX sentences: blockIdx.y = admission,
// blockIdx.x = (tensor, beam column) -- the encoder's final state of the sentence into every column
// of the slot, zeros into the tensors that start at zero -- and the first block of an admission also
// writes the slot's entries of the small arrays.
struct AdmitArgs {
  lh_stream_admission adm[LH_STREAM_ADMIT_MAX];
  int beam, B, H, n_src, n_tensors, n_zero, start_id;
  int *start, *limit, *hs_col, *batch_info, *tok_prev;
  float *score_prev;
  const float *src[LH_GATHER_MAX_TENSORS];
  float *dst[LH_GATHER_MAX_TENSORS];
  float *zero[LH_GATHER_MAX_TENSORS];
};

__global__ __launch_bounds__(256) void stream_admit_kernel(const AdmitArgs a) {
  const lh_stream_admission q = a.adm[blockIdx.y];
  const int t = blockIdx.x / a.beam, j = blockIdx.x % a.beam;
  const int c = q.slot * a.beam + j;  // the column
  if (t < a.n_tensors) {
    const float *src = a.src[t] + (size_t)q.sentence_col * a.H;
    float *dst = a.dst[t] + (size_t)c * a.H;
    for (int i = threadIdx.x; i < a.H; i += 256) dst[i] = src[i];
  } else {
    float *dst = a.zero[t - a.n_tensors] + (size_t)c * a.H;
    for (int i = threadIdx.x; i < a.H; i += 256) dst[i] = 0.f;
  }
  if (blockIdx.x == 0) {
    if (threadIdx.x == 0) {
      a.start[q.slot] = q.tick;
      a.limit[q.slot] = q.limit;
    }
    for (int i = threadIdx.x; i < a.beam; i += 256) {
      const int cc = q.slot * a.beam + i;
      if (a.hs_col) a.hs_col[cc] = q.hs_col_value;
      if (a.batch_info) {
        a.batch_info[cc] = q.len;
        a.batch_info[a.B + cc] = q.off;
      }
      a.tok_prev[cc] = a.start_id;
      a.score_prev[cc] = 0.f;
    }
  }
}

int check_merge_args(const char *who, int n_sent, int beam, int K, int step, const int *limit,
                     const float *cand_logp, const int *cand_id, const float *logp_eof,
                     const float *prev_score, const int *tok, const int *backptr, const float *score,
                     const int *fin_count, const int *fin_beam, const float *fin_score) {
  if (n_sent <= 0 || beam <= 0 || K <= 0 || step < 0)
    return lh::fail_arg("%s: n_sent=%d beam=%d K=%d step=%d", who, n_sent, beam, K, step);
  if ((long long)beam * K > kMaxCand)
    return lh::fail_arg("%s: beam*K=%lld exceeds %d", who, (long long)beam * K, kMaxCand);
  if (!limit || !cand_logp || !cand_id || !logp_eof || !prev_score || !tok || !backptr || !score ||
      !fin_count || !fin_beam || !fin_score)
    return lh::fail_arg("%s: a required pointer is NULL", who);
  if (score == prev_score) return lh::fail_arg("%s: score aliases prev_score", who);
  return LH_OK;
}

// fills a (tensors, H, B_src); *vec: 16-byte copies are possible
int check_gather_args(const char *who, const float *const *src, float *const *dst, int n_tensors,
                      int H, int B, int B_src, GatherArgs *a, bool *vec) {
  if (n_tensors < 1 || n_tensors > LH_GATHER_MAX_TENSORS || H <= 0 || B <= 0 || B_src <= 0 ||
      !src || !dst)
    return lh::fail_arg("%s: n_tensors=%d H=%d B=%d B_src=%d or NULL pointer", who, n_tensors, H,
                        B, B_src);
  *vec = H % 4 == 0;
  for (int t = 0; t < n_tensors; ++t) {
    if (!src[t] || !dst[t]) return lh::fail_arg("%s: tensor %d is NULL", who, t);
    for (int u = 0; u < n_tensors; ++u)
      if (dst[t] == src[u]) return lh::fail_arg("%s: dst %d aliases src %d", who, t, u);
    a->src[t] = src[t];
    a->dst[t] = dst[t];
    *vec = *vec && lh::aligned16(src[t]) && lh::aligned16(dst[t]);
  }
  a->H = H;
  a->B_src = B_src;
  return LH_OK;
}

}  // namespace

extern "C" int lh_beam_merge_f32(int n_sent, int beam, int K, int step, const int *limit,
                                 const float *cand_logp, const int *cand_id, const float *logp_eof,
                                 const float *prev_score, float diversity, float penalty,
                                 int start_id, int eof_id, int *tok, int *backptr, float *score,
                                 int *fin_count, int *fin_beam, float *fin_score,
                                 lh_stream_t stream) {
  const int rc = check_merge_args("lh_beam_merge_f32", n_sent, beam, K, step, limit, cand_logp, cand_id,
                                  logp_eof, prev_score, tok, backptr, score, fin_count, fin_beam,
                                  fin_score);
  if (rc != LH_OK) return rc;
  if (beam > kMaxBeam) return lh::fail_arg("lh_beam_merge_f32: beam=%d exceeds %d", beam, kMaxBeam);
  MergeArgs a{n_sent, beam, K, step, limit, cand_logp, cand_id, logp_eof, prev_score, diversity,
              penalty, start_id, eof_id, tok, backptr, score, fin_count, fin_beam, fin_score};
  hipLaunchKernelGGL(beam_merge_kernel, dim3(n_sent), dim3(kMergeThreads), 0,
                     lh::as_stream(stream), a);
  return lh::check_launch("lh_beam_merge_f32");
}

extern "C" int lh_beam_gather_f32(const float *const *src, float *const *dst, int n_tensors, int H,
                                  int B, int B_src, const int *backptr, lh_stream_t stream) {
  if (!backptr) return lh::fail_arg("lh_beam_gather_f32: backptr is NULL");
  GatherArgs a{};
  bool vec;
  const int rc = check_gather_args("lh_beam_gather_f32", src, dst, n_tensors, H, B, B_src, &a, &vec);
  if (rc != LH_OK) return rc;
  a.backptr = backptr;
  const int hq = vec ? H / 4 : H;
  const dim3 grid((hq + 255) / 256, B, n_tensors), block(256);
  if (B > 65535) return lh::fail_arg("lh_beam_gather_f32: B=%d exceeds 65535", B);
  if (vec) hipLaunchKernelGGL(beam_gather_kernel<4>, grid, block, 0, lh::as_stream(stream), a);
  else hipLaunchKernelGGL(beam_gather_kernel<1>, grid, block, 0, lh::as_stream(stream), a);
  return lh::check_launch("lh_beam_gather_f32");
}

namespace {
int merge_gather(const char *who, int n_sent, int beam, int K, int step, const int *start,
                 const int *limit, const float *cand_logp, const int *cand_id, const float *logp_eof,
                 const float *prev_score, float diversity, float penalty, int start_id, int eof_id,
                 int *tok, int *backptr, float *score, int *fin_count, int *fin_beam,
                 float *fin_score, const float *const *src, float *const *dst, int n_tensors, int H,
                 lh_stream_t stream);
}

extern "C" int lh_beam_merge_gather_f32(int n_sent, int beam, int K, int step, const int *limit,
                                        const float *cand_logp, const int *cand_id,
                                        const float *logp_eof, const float *prev_score,
                                        float diversity, float penalty, int start_id, int eof_id,
                                        int *tok, int *backptr, float *score, int *fin_count,
                                        int *fin_beam, float *fin_score, const float *const *src,
                                        float *const *dst, int n_tensors, int H,
                                        lh_stream_t stream) {
  return merge_gather("lh_beam_merge_gather_f32", n_sent, beam, K, step, nullptr, limit, cand_logp,
                      cand_id, logp_eof, prev_score, diversity, penalty, start_id, eof_id, tok, backptr,
                      score, fin_count, fin_beam, fin_score, src, dst, n_tensors, H, stream);
}

extern "C" int lh_beam_merge_gather_stream_f32(int n_sent, int beam, int K, int tick, const int *start,
                                               const int *limit, const float *cand_logp,
                                               const int *cand_id, const float *logp_eof,
                                               const float *prev_score, float diversity,
                                               float penalty, int start_id, int eof_id, int *tok,
                                               int *backptr, float *score, int *fin_count,
                                               int *fin_beam, float *fin_score,
                                               const float *const *src, float *const *dst,
                                               int n_tensors, int H, lh_stream_t stream) {
  if (!start) return lh::fail_arg("lh_beam_merge_gather_stream_f32: start is NULL");
  return merge_gather("lh_beam_merge_gather_stream_f32", n_sent, beam, K, tick, start, limit, cand_logp,
                      cand_id, logp_eof, prev_score, diversity, penalty, start_id, eof_id, tok, backptr,
                      score, fin_count, fin_beam, fin_score, src, dst, n_tensors, H, stream);
}

extern "C" int lh_stream_admit_f32(const lh_stream_admission *adm, int n_adm, int beam, int B,
                                   int *start, int *limit, int *hs_col, int *batch_info,
                                   const float *const *src, float *const *dst, int n_tensors,
                                   float *const *zero, int n_zero, int H, int n_src, int *tok_prev,
                                   int start_id, float *score_prev, lh_stream_t stream) {
  const char *who = "lh_stream_admit_f32";
  if (!adm || n_adm < 1 || n_adm > LH_STREAM_ADMIT_MAX || beam < 1 || B < beam || H < 1 || n_src < 1)
    return lh::fail_arg("%s: n_adm=%d beam=%d B=%d H=%d n_src=%d", who, n_adm, beam, B, H, n_src);
  if (n_tensors < 0 || n_tensors > LH_GATHER_MAX_TENSORS || n_zero < 0 || n_zero > LH_GATHER_MAX_TENSORS ||
      n_tensors + n_zero < 1)
    return lh::fail_arg("%s: n_tensors=%d n_zero=%d", who, n_tensors, n_zero);
  if (!start || !limit || !tok_prev || !score_prev || (n_tensors && (!src || !dst)) || (n_zero && !zero))
    return lh::fail_arg("%s: a required pointer is NULL", who);
  AdmitArgs a{};
  for (int i = 0; i < n_adm; ++i) {
    const lh_stream_admission &q = adm[i];
    if (q.slot < 0 || (q.slot + 1) * beam > B || q.sentence_col < 0 || q.sentence_col >= n_src)
      return lh::fail_arg("%s: admission %d: slot %d / sentence column %d out of range", who, i, q.slot,
                          q.sentence_col);
    for (int k = 0; k < i; ++k)
      if (adm[k].slot == q.slot)
        return lh::fail_arg("%s: admissions %d and %d name the same slot %d", who, k, i, q.slot);
    a.adm[i] = q;
  }
  a.beam = beam, a.B = B, a.H = H, a.n_src = n_src, a.n_tensors = n_tensors, a.n_zero = n_zero;
  a.start_id = start_id, a.start = start, a.limit = limit, a.hs_col = hs_col, a.batch_info = batch_info;
  a.tok_prev = tok_prev, a.score_prev = score_prev;
  for (int t = 0; t < n_tensors; ++t) {
    if (!src[t] || !dst[t]) return lh::fail_arg("%s: tensor %d is NULL", who, t);
    a.src[t] = src[t], a.dst[t] = dst[t];
  }
  for (int t = 0; t < n_zero; ++t) {
    if (!zero[t]) return lh::fail_arg("%s: zero tensor %d is NULL", who, t);
    a.zero[t] = zero[t];
  }
  hipLaunchKernelGGL(stream_admit_kernel, dim3((n_tensors + n_zero) * beam, n_adm), dim3(256), 0,
                     lh::as_stream(stream), a);
  return lh::check_launch(who);
}

namespace {
int merge_gather(const char *who, int n_sent, int beam, int K, int step, const int *start,
                 const int *limit, const float *cand_logp, const int *cand_id, const float *logp_eof,
                 const float *prev_score, float diversity, float penalty, int start_id, int eof_id,
                 int *tok, int *backptr, float *score, int *fin_count, int *fin_beam,
                 float *fin_score, const float *const *src, float *const *dst, int n_tensors, int H,
                 lh_stream_t stream) {
  int rc = check_merge_args(who, n_sent, beam, K, step, limit, cand_logp, cand_id, logp_eof,
                            prev_score, tok, backptr, score, fin_count, fin_beam, fin_score);
  if (rc != LH_OK) return rc;
  if (beam > kMaxBeam) return lh::fail_arg("%s: beam=%d exceeds %d", who, beam, kMaxBeam);
  if (n_sent > 65535) return lh::fail_arg("%s: n_sent=%d exceeds 65535", who, n_sent);
  GatherArgs ga{};
  bool vec;
  rc = check_gather_args(who, src, dst, n_tensors, H, n_sent * beam, n_sent * beam, &ga, &vec);
  if (rc != LH_OK) return rc;
  MergeArgs a{n_sent, beam, K, step, limit, cand_logp, cand_id, logp_eof, prev_score, diversity,
              penalty, start_id, eof_id, tok, backptr, score, fin_count, fin_beam, fin_score, start};
  // enough workgroups per sentence to give every CU one (each of them repeats the merge)
  int per = (256 + n_sent - 1) / n_sent;
  per = per < 1 ? 1 : (per > 16 ? 16 : per);
  const dim3 grid(per, n_sent), block(kMergeThreads);
  if (vec)
    hipLaunchKernelGGL(beam_merge_gather_kernel<4>, grid, block, 0, lh::as_stream(stream), a, ga, n_tensors);
  else
    hipLaunchKernelGGL(beam_merge_gather_kernel<1>, grid, block, 0, lh::as_stream(stream), a, ga, n_tensors);
  return lh::check_launch(who);
}
}  // namespace
