// Live per-kernel timing with HIP events recorded on the model's own stream (the stream the
// kernels are launched on).  Level 0 records nothing; level 1 brackets the matrix products (the
// dominant kernels of a decode step), keyed by the kernel instance the GEMM entry point picks;
// level 2 brackets every launch of the path.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "hip_util.h"

namespace linmt {

enum ProfileTag {
  kTagEmbedLookup = 0,
  kTagGateGemm,
  kTagLstmCell,
  kTagAttnProjGemm,   // tanh(W_p ha) and W_a^T ha
  kTagAttnCore,
  kTagAttnOutGemm,    // tanh(W_c1 ctx + W_c2 ha + b)
  kTagLogitsGemm,     // D h~ + b_d
  kTagSoftmax,
  kTagXent,
  kTagBeamTopK,
  kTagBeamMerge,
  kTagBeamGather,
  kTagErrorGemm,       // W^T d: errors handed to t-1 / the layer below / the attention node
  kTagWeightGradGemm,  // d x^T accumulated over all steps
  kTagLstmCellBwd,
  kTagAttnBwd,
  kTagSoftmaxGrad,
  kTagRowSum,
  kTagEmbedGrad,
  kTagUpdate,
  kTagSplitPack,  // fp32 -> three bf16 planes, for the products on the bf16 matrix pipe
  kTagBeamMergeGather,  // merge and state gather of a step in one launch
  kTagCount
};

inline const char *ProfileTagName(int t) {
  static const char *names[kTagCount] = {"embed_lookup", "gate_gemm", "lstm_cell", "attn_proj_gemm",
                                         "attn_core", "attn_out_gemm", "logits_gemm", "softmax",
                                         "xent", "beam_topk", "beam_merge", "beam_gather",
                                         "error_gemm", "weight_grad_gemm", "lstm_cell_bwd",
                                         "attn_bwd", "softmax_grad", "row_sum", "embed_grad",
                                         "update", "split_pack", "beam_merge_gather"};
  return t >= 0 && t < kTagCount ? names[t] : "";
}

struct ProfileTotals {
  double ms = 0;     // summed launch durations
  double work = 0;   // summed algorithmic work (flop for GEMMs, bytes otherwise)
  long long launches = 0;
};

class Profiler {
 public:
  int level_ = 0;
  hipStream_t stream_ = nullptr;
  // key: "<call site>" or "<call site>|<kernel instance>" for matrix products
  std::map<std::string, ProfileTotals> totals_;

  ~Profiler() {
    for (hipEvent_t e : pool_) (void)hipEventDestroy(e);
  }
  // level 1 brackets only the output projection, the dominant product: an event pair per launch
  // costs a few microseconds of GPU idle time, which across all ~700 products of a decoding batch
  // is 6% of it
  bool Wants(int tag) const { return level_ >= 2 || (level_ == 1 && tag == kTagLogitsGemm); }
  // Returns the slot to hand back to End(); scopes may nest or overlap.
  size_t Begin(const std::string &key, double work) {
    Pending p{key, Take(), Take(), work};
    HipErrorWrapper(hipEventRecord(pool_[p.start], stream_), "profile event record failed");
    pending_.push_back(p);
    return pending_.size() - 1;
  }
  void End(size_t slot) {
    HipErrorWrapper(hipEventRecord(pool_[pending_[slot].stop], stream_),
                    "profile event record failed");
  }
  // Call after the stream has been synchronised: folds the recorded pairs into the totals.
  void Collect() {
    for (const Pending &p : pending_) {
      float ms = 0.f;
      HipErrorWrapper(hipEventElapsedTime(&ms, pool_[p.start], pool_[p.stop]),
                      "profile event elapsed failed");
      ProfileTotals &t = totals_[p.key];
      t.ms += ms;
      t.work += p.work;
      t.launches += 1;
    }
    pending_.clear();
    next_ = 0;
  }
  void Reset() { totals_.clear(); }

 private:
  struct Pending {
    std::string key;
    size_t start, stop;
    double work;
  };
  size_t Take() {
    if (next_ == pool_.size()) {
      hipEvent_t e;
      HipErrorWrapper(hipEventCreate(&e), "profile event creation failed");
      pool_.push_back(e);
    }
    return next_++;
  }
  std::vector<hipEvent_t> pool_;
  std::vector<Pending> pending_;
  size_t next_ = 0;
};

// Brackets the launches issued while it is alive.
class ProfileScope {
 public:
  ProfileScope(Profiler &p, int tag, double work) : p_(p), on_(p.Wants(tag)) {
    if (on_) slot_ = p_.Begin(ProfileTagName(tag), work);
  }
  // Matrix product: the key carries the kernel instance lh_gemm_f32 will launch for this problem.
  ProfileScope(Profiler &p, int tag, size_t workspace_bytes, int max_planes, int M, int N,
               const lh_gemm_seg *segs, int nseg, int transA,
               int transX)
      : p_(p), on_(p.Wants(tag)) {
    if (!on_) return;
    char name[160] = {0};
    LhErrorWrapper(lh_gemm_kernel_name(M, N, segs, nseg, transA, transX, workspace_bytes, max_planes,
                                       name, sizeof(name)),
                   "lh_gemm_kernel_name");
    double k = 0;
    for (int s = 0; s < nseg; ++s) k += segs[s].K;
    slot_ = p_.Begin(std::string(ProfileTagName(tag)) + "|" + name, 2.0 * M * (double)N * k);
  }
  // Matrix product whose kernel instance the caller already knows.
  ProfileScope(Profiler &p, int tag, const char *kernel_name, double flop) : p_(p), on_(p.Wants(tag)) {
    if (on_) slot_ = p_.Begin(std::string(ProfileTagName(tag)) + "|" + kernel_name, flop);
  }
  ~ProfileScope() noexcept(false) {
    if (on_) p_.End(slot_);
  }

 private:
  Profiler &p_;
  bool on_;
  size_t slot_ = 0;
};

}  // namespace linmt
