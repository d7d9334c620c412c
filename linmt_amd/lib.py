"""ctypes binding of liblinmt_hip.so (the C ABI declared in include/linmt_hip.h).

The library is the product; this module only gives Python (tests, smoke, benchmark) a way to call
it with device pointers taken from torch tensors.  There is no fallback of any kind: if the built
library is missing, loading raises, and every wrapper raises on a non-zero status.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblinmt_hip.so")

LH_ACT_NONE = 0
LH_ACT_TANH = 1
LH_GEMM_MAX_SEGS = 3
LH_BEAM_MAX_K = 64
LH_GATHER_MAX_TENSORS = 24

c_f32p = C.c_void_p  # device pointers travel as plain addresses
c_i32p = C.c_void_p
c_f64p = C.c_void_p


class StreamAdmission(C.Structure):
    _fields_ = [("slot", C.c_int), ("sentence_col", C.c_int), ("hs_col_value", C.c_int),
                ("len", C.c_int), ("off", C.c_int), ("limit", C.c_int), ("tick", C.c_int)]


class GemmSeg(C.Structure):
    _fields_ = [("A", C.c_void_p), ("lda", C.c_int), ("X", C.c_void_p), ("ldx", C.c_int),
                ("K", C.c_int)]


class GateProblem(C.Structure):
    _fields_ = [("segs", GemmSeg * LH_GEMM_MAX_SEGS), ("nseg", C.c_int), ("cell", C.c_int),
                ("addend", C.c_void_p), ("ld_addend", C.c_int), ("addend_col", C.c_void_p),
                ("addend_ncols", C.c_int), ("bias4h", C.c_void_p), ("c_prev", C.c_void_p),
                ("mask01", C.c_void_p), ("sigmoid_f64", C.c_int), ("cell_clip", C.c_float),
                ("c", C.c_void_p), ("h", C.c_void_p), ("out", C.c_void_p), ("ld_out", C.c_int)]


class SplitSource(C.Structure):
    _fields_ = [("src", C.c_void_p), ("ld", C.c_int), ("k_contiguous", C.c_int), ("D", C.c_int),
                ("K", C.c_int), ("gate_H", C.c_int), ("planes", C.c_void_p),
                ("kgroups_total", C.c_int), ("kg_offset", C.c_int), ("kgroups", C.c_int)]


# name -> (restype, argtypes); mirrors include/linmt_hip.h one to one.
SIGNATURES = {
    "lh_abi_version": (C.c_int, []),
    "lh_last_error": (C.c_char_p, []),
    "lh_preprocess_indices_i32": (C.c_int, [c_i32p, C.c_int, c_i32p, c_i32p, c_f32p, C.c_void_p]),
    "lh_setup_reverse_indices_i32": (C.c_int, [c_i32p, C.c_int, c_i32p, C.c_int, C.c_void_p]),
    "lh_embed_lookup_f32": (C.c_int, [c_f32p, C.c_int, C.c_int, c_i32p, C.c_int, c_f32p,
                                      C.c_float, c_f32p, C.c_void_p]),
    "lh_gemm_f32": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int, C.c_int, C.c_int,
                              C.c_float, C.c_float, c_f32p, C.c_int, c_i32p, c_f32p, C.c_int,
                              C.c_void_p]),
    "lh_gemm_act_rows_f32": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int, C.c_int,
                                       C.c_int, C.c_float, C.c_float, c_f32p, C.c_int, C.c_int,
                                       c_i32p, c_f32p, C.c_int, C.c_void_p]),
    "lh_gemm_ws_f32": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int, C.c_int, C.c_int,
                                 C.c_float, C.c_float, c_f32p, C.c_int, C.c_int, c_i32p, c_f32p,
                                 C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]),
    "lh_gemm_noalloc_init": (C.c_int, []),
    "lh_gemm_noalloc_f32": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int, C.c_int,
                                      C.c_int, C.c_float, C.c_float, c_f32p, C.c_int, C.c_int,
                                      c_i32p, c_f32p, C.c_int, C.c_void_p]),
    "lh_gemm_planes_f32": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int, C.c_int,
                                     C.c_int, C.c_float, c_f32p, C.c_int, C.c_void_p, C.c_size_t,
                                     C.c_int, C.POINTER(C.c_int), C.c_void_p]),
    "lh_gemm_kernel_name": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int, C.c_int,
                                      C.c_int, C.c_size_t, C.c_int, C.c_char_p, C.c_int]),
    "lh_gate_gemm_lstm_cell_plan": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int, C.c_int,
                                              C.c_size_t, C.POINTER(C.c_int), C.c_char_p, C.c_int]),
    "lh_gate_gemm_lstm_cell_f32": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int, c_f32p,
                                             C.c_int, c_i32p, C.c_int, c_f32p, c_f32p, c_i32p, C.c_int,
                                             C.c_float, c_f32p, c_f32p, C.c_size_t, C.c_void_p]),
    "lh_gate_gemm_lstm_cell_train_f32": (C.c_int, [C.c_int, C.c_int, C.POINTER(GemmSeg), C.c_int,
                                                   c_f32p, C.c_int, c_f32p, c_f32p, c_i32p, C.c_int,
                                                   C.c_float, c_f32p, c_f32p, c_f32p, c_f32p,
                                                   C.c_float, c_f32p, C.c_size_t, C.c_void_p]),
    "lh_gate_gemm_group_plan": (C.c_int, [C.c_int, C.c_int, C.POINTER(GateProblem), C.c_int,
                                          C.POINTER(C.c_int), C.c_char_p, C.c_int]),
    "lh_gate_gemm_group_f32": (C.c_int, [C.c_int, C.c_int, C.POINTER(GateProblem), C.c_int,
                                         C.c_void_p]),
    "lh_attn_core_projected_fwd_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, c_f32p,
                                                 C.c_longlong, c_f32p, c_f32p, C.c_longlong, c_f32p,
                                                 c_f32p, C.c_longlong, C.c_longlong, c_i32p, c_i32p,
                                                 c_i32p, c_f32p, C.c_longlong, c_f32p, c_f32p, c_f32p,
                                                 c_i32p, c_f32p, c_f32p, c_f32p, c_i32p, C.c_void_p]),
    "lh_gemm_set_config_override": (C.c_int, [C.c_int]),
    "lh_gemm_set_splits_override": (C.c_int, [C.c_int]),
    "lh_gemm_config_info": (C.c_int, [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int * 8)]),
    "lh_split_kgroups": (C.c_int, [C.c_int]),
    "lh_split_kgroups_padded": (C.c_int, [C.c_int]),
    "lh_split_padded": (C.c_int, [C.c_int]),
    "lh_split_gate_rows": (C.c_int, [C.c_int]),
    "lh_split_bytes": (C.c_size_t, [C.c_int, C.c_int]),
    "lh_split_pack_f32": (C.c_int, [C.POINTER(SplitSource), C.c_int, C.c_void_p]),
    "lh_gemm_split_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_float,
                                    C.c_float, c_f32p, C.c_int, C.c_int, c_i32p, c_f32p, C.c_int,
                                    C.c_void_p]),
    "lh_gate_gemm_split_lstm_cell_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                                   c_f32p, C.c_int, c_i32p, C.c_int, c_f32p, c_f32p,
                                                   c_i32p, C.c_int, C.c_float, c_f32p, c_f32p,
                                                   C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "lh_gemm_split_kernel_name": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_char_p, C.c_int]),
    "lh_gemm_split_set_config_override": (C.c_int, [C.c_int]),
    "lh_lstm_cell_fwd_f32": (C.c_int, [C.c_int, C.c_int, c_f32p, c_f32p, c_f32p, c_f32p, c_f32p,
                                       c_i32p, C.c_int, C.c_float, c_f32p, c_f32p, c_f32p, c_f32p,
                                       C.c_float, c_f32p, C.c_void_p]),
    "lh_attn_core_fwd_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, c_f32p, c_f32p,
                                       c_f32p, C.c_longlong, c_f32p, C.c_longlong, C.c_longlong,
                                       c_i32p, c_i32p,
                                       c_i32p, c_f32p, c_f32p, c_i32p, c_f32p, c_f32p, c_f32p,
                                       c_i32p, C.c_void_p]),
    "lh_softmax_fwd_f32": (C.c_int, [c_f32p, C.c_int, c_f32p, C.c_int, C.c_int, c_f32p, C.c_int,
                                     C.c_void_p]),
    "lh_train_loglik_f32": (C.c_int, [c_f32p, C.c_int, C.c_int, C.c_int, c_i32p, c_i32p, c_f64p,
                                      C.c_void_p]),
    "lh_logsoftmax_xent_f32": (C.c_int, [c_f32p, C.c_int, c_f32p, C.c_int, C.c_int, c_i32p, c_i32p,
                                         c_f64p, c_f64p, C.c_void_p]),
    "lh_beam_topk_f32": (C.c_int, [c_f32p, C.c_int, c_f32p, C.c_int, C.c_int, C.c_int, C.c_int,
                                   c_f32p, c_i32p, c_f32p, C.c_void_p]),
    "lh_beam_topk_ensemble_f32": (C.c_int, [C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_int,
                                            C.c_int, C.c_int, C.c_int, c_f32p, c_i32p, c_f32p,
                                            C.c_void_p]),
    "lh_beam_merge_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, c_i32p, c_f32p, c_i32p,
                                    c_f32p, c_f32p, C.c_float, C.c_float, C.c_int, C.c_int, c_i32p,
                                    c_i32p, c_f32p, c_i32p, c_i32p, c_f32p, C.c_void_p]),
    "lh_beam_gather_f32": (C.c_int, [C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_int,
                                     C.c_int, C.c_int, C.c_int, c_i32p, C.c_void_p]),
    "lh_beam_merge_gather_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, c_i32p, c_f32p, c_i32p,
                                           c_f32p, c_f32p, C.c_float, C.c_float, C.c_int, C.c_int,
                                           c_i32p, c_i32p, c_f32p, c_i32p, c_i32p, c_f32p,
                                           C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_int,
                                           C.c_int, C.c_void_p]),
    "lh_beam_merge_gather_stream_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, c_i32p, c_i32p,
                                                  c_f32p, c_i32p, c_f32p, c_f32p, C.c_float, C.c_float,
                                                  C.c_int, C.c_int, c_i32p, c_i32p, c_f32p, c_i32p,
                                                  c_i32p, c_f32p, C.POINTER(C.c_void_p),
                                                  C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_void_p]),
    "lh_stream_admit_f32": (C.c_int, [C.POINTER(StreamAdmission), C.c_int, C.c_int, C.c_int, c_i32p,
                                      c_i32p, c_i32p, c_i32p, C.POINTER(C.c_void_p),
                                      C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_void_p), C.c_int,
                                      C.c_int, C.c_int, c_i32p, C.c_int, c_f32p, C.c_void_p]),
    "lh_softmax_xent_grad_f32": (C.c_int, [c_f32p, C.c_int, c_f32p, C.c_int, C.c_int, c_i32p,
                                           c_i32p, c_f32p, C.c_int, c_f64p, c_f64p, C.c_void_p]),
    "lh_uniform_f32": (C.c_int, [c_f32p, C.c_longlong, C.c_ulonglong, C.c_void_p]),
    "lh_lstm_cell_bwd_f32": (C.c_int, [C.c_int, C.c_int, c_f32p, c_f32p, c_f32p, c_f32p, c_f32p,
                                       c_f32p, c_i32p, C.c_float, C.c_float, c_f32p, C.c_float,
                                       c_f32p, c_f32p, C.c_void_p]),
    "lh_lstm_cell_bwd_terms_f32": (C.c_int, [C.c_int, C.c_int, C.c_void_p, C.c_void_p, c_f32p, c_f32p,
                                             c_f32p, c_f32p, c_i32p, C.c_float, C.c_float, c_f32p,
                                             C.c_float, c_f32p, c_f32p, C.c_void_p]),
    "lh_rowsum_acc_f32": (C.c_int, [c_f32p, C.c_longlong, C.c_int, C.c_longlong, C.c_float, c_f32p,
                                    C.c_void_p]),
    "lh_embed_gather_grad_f32": (C.c_int, [c_f32p, C.c_longlong, C.c_int, C.c_int, c_i32p, c_i32p,
                                           c_f32p, C.c_float, C.c_float, c_f32p, C.c_longlong,
                                           C.c_void_p]),
    "lh_attn_delta_f32": (C.c_int, [C.c_int, C.c_int, c_f32p, c_f32p, c_f32p, c_i32p, C.c_float,
                                    c_f32p, C.c_void_p]),
    "lh_attn_core_bwd_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, c_f32p, c_f32p,
                                       c_f32p, c_f32p, c_f32p, C.c_longlong, C.c_longlong, c_i32p,
                                       c_f32p, c_f32p, c_i32p, c_f32p, c_f32p, c_f32p, c_f32p,
                                       c_f32p, c_f32p, C.c_void_p]),
    "lh_grad_sumsq_f32": (C.c_int, [c_f32p, C.c_longlong, C.c_longlong, C.c_longlong, C.c_float,
                                    c_f64p, c_f64p, C.c_void_p]),
    "lh_sgd_step_f32": (C.c_int, [c_f32p, C.c_longlong, c_f32p, C.c_longlong, C.c_longlong,
                                  C.c_longlong, c_i32p, C.c_float, C.c_float, c_f64p, C.c_float,
                                  C.c_float, C.c_void_p]),
}

LH_SUMSQ_WORKSPACE = 1024
_lib = None


class LinmtHipError(RuntimeError):
    pass


def load():
    """Loads liblinmt_hip.so and checks that it exports every declared entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LinmtHipError(
            f"{LIB_PATH} is missing: build it with `make -C linmt_amd/csrc` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    # torch brings a HIP runtime of its own; the callers here hand over torch tensors, so its
    # runtime has to be the first one the process loads
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _ptr(t):
    """Device (or host) address of a torch tensor / None."""
    if t is None:
        return None
    return C.c_void_p(t.data_ptr())


def check(status, what):
    if status != 0:
        msg = load().lh_last_error().decode("utf-8", "replace")
        raise LinmtHipError(f"{what} failed with status {status}: {msg}")


def _stream(stream):
    if stream is None:
        import torch
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)
    return C.c_void_p(stream)


# ---- thin wrappers over torch tensors (column-major data lives in whatever tensor holds it) ------
def preprocess_indices(idx, idx0, mask01, mask01_f=None, stream=None):
    check(load().lh_preprocess_indices_i32(_ptr(idx), idx.numel(), _ptr(idx0), _ptr(mask01),
                                           _ptr(mask01_f), _stream(stream)),
          "lh_preprocess_indices_i32")


def setup_reverse_indices(unique, rev, vocab, stream=None):
    check(load().lh_setup_reverse_indices_i32(_ptr(unique), unique.numel(), _ptr(rev), vocab,
                                              _stream(stream)), "lh_setup_reverse_indices_i32")


def embed_lookup(W, E, V, idx0, B, out, drop_mask=None, keep=1.0, stream=None):
    check(load().lh_embed_lookup_f32(_ptr(W), E, V, _ptr(idx0), B, _ptr(drop_mask), keep,
                                     _ptr(out), _stream(stream)), "lh_embed_lookup_f32")


def _segs(segs):
    arr = (GemmSeg * len(segs))()
    for i, (A, lda, X, ldx, K) in enumerate(segs):
        arr[i].A = A.data_ptr()
        arr[i].lda = lda
        arr[i].X = X.data_ptr()
        arr[i].ldx = ldx
        arr[i].K = K
    return arr


def gemm(M, N, segs, C_out, ldc, transA=False, transX=False, alpha=1.0, beta=0.0, bias=None,
         act=LH_ACT_NONE, colmask=None, act_rows=None, workspace=None, stream=None):
    """segs: list of (A, lda, X, ldx, K) with torch tensors A, X.  workspace: torch tensor
    whose memory the K split may use (lh_gemm_ws_f32)."""
    arr = _segs(segs)
    if workspace is not None:
        check(load().lh_gemm_ws_f32(M, N, arr, len(segs), int(transA), int(transX), alpha, beta,
                                    _ptr(bias), act, M if act_rows is None else act_rows,
                                    _ptr(colmask), _ptr(C_out), ldc, workspace.data_ptr(),
                                    workspace.numel() * workspace.element_size(),
                                    _stream(stream)), "lh_gemm_ws_f32")
    elif act_rows is None:
        check(load().lh_gemm_f32(M, N, arr, len(segs), int(transA), int(transX), alpha, beta,
                                 _ptr(bias), act, _ptr(colmask), _ptr(C_out), ldc,
                                 _stream(stream)), "lh_gemm_f32")
    else:
        check(load().lh_gemm_act_rows_f32(M, N, arr, len(segs), int(transA), int(transX), alpha,
                                          beta, _ptr(bias), act, act_rows, _ptr(colmask),
                                          _ptr(C_out), ldc, _stream(stream)),
              "lh_gemm_act_rows_f32")


LH_GEMM_NOALLOC_WS_BYTES = 32 << 20


def gemm_noalloc_init():
    check(load().lh_gemm_noalloc_init(), "lh_gemm_noalloc_init")


def gemm_noalloc(M, N, segs, C_out, ldc, transA=False, transX=False, alpha=1.0, beta=0.0,
                 bias=None, act=LH_ACT_NONE, colmask=None, act_rows=None, stream=None):
    """lh_gemm_noalloc_f32: the K-split product over the library's own scratch array."""
    check(load().lh_gemm_noalloc_f32(M, N, _segs(segs), len(segs), int(transA), int(transX), alpha,
                                     beta, _ptr(bias), act, M if act_rows is None else act_rows,
                                     _ptr(colmask), _ptr(C_out), ldc, _stream(stream)),
          "lh_gemm_noalloc_f32")


def gemm_kernel_name(M, N, segs, transA=False, transX=False, workspace_bytes=0, max_planes=0):
    buf = C.create_string_buffer(128)
    check(load().lh_gemm_kernel_name(M, N, _segs(segs), len(segs), int(transA), int(transX),
                                     workspace_bytes, max_planes, buf, 128), "lh_gemm_kernel_name")
    return buf.value.decode()


def attn_core_projected_fwd(H, B, D, hs_steps, tanh1, tanh1_col_stride, v_p, h_t, h_t_col_stride,
                            score_mem, ctx_mem, mem_step_stride, mem_col_stride, mem_col, batch_info,
                            mask01, out_add, out_add_col_stride, out_bias, p_t, sigma, indices, align,
                            cached_exp, h_tild, viterbi=None, stream=None):
    check(load().lh_attn_core_projected_fwd_f32(
        H, B, D, hs_steps, _ptr(tanh1), tanh1_col_stride, _ptr(v_p), _ptr(h_t), h_t_col_stride,
        _ptr(score_mem), _ptr(ctx_mem), mem_step_stride, mem_col_stride, _ptr(mem_col),
        _ptr(batch_info), _ptr(mask01), _ptr(out_add), out_add_col_stride, _ptr(out_bias), _ptr(p_t),
        _ptr(sigma), _ptr(indices), _ptr(align), _ptr(cached_exp), _ptr(h_tild), _ptr(viterbi),
        _stream(stream)), "lh_attn_core_projected_fwd_f32")


def gate_gemm_lstm_cell_plan(H, B, segs, has_addend=False, workspace_bytes=0):
    """(fusable, kernel instance name) for lh_gate_gemm_lstm_cell_f32 on this problem."""
    f, buf = C.c_int(), C.create_string_buffer(128)
    check(load().lh_gate_gemm_lstm_cell_plan(H, B, _segs(segs), len(segs), int(has_addend),
                                             workspace_bytes, C.byref(f), buf, 128),
          "lh_gate_gemm_lstm_cell_plan")
    return bool(f.value), buf.value.decode()


def gate_gemm_lstm_cell(H, B, segs, bias4h, c_prev, mask01, c, h, addend=None, ld_addend=0,
                        addend_col=None, addend_ncols=0, sigmoid_f64=False, cell_clip=0.0, workspace_bytes=0,
                        stream=None):
    check(load().lh_gate_gemm_lstm_cell_f32(H, B, _segs(segs), len(segs), _ptr(addend), ld_addend,
                                            _ptr(addend_col), addend_ncols, _ptr(bias4h), _ptr(c_prev),
                                            _ptr(mask01), int(sigmoid_f64), cell_clip, _ptr(c),
                                            _ptr(h), workspace_bytes, _stream(stream)),
          "lh_gate_gemm_lstm_cell_f32")


def gate_gemm_lstm_cell_train(H, B, segs, bias4h, c_prev, mask01, c, h, gates=None, addend=None,
                              ld_addend=0, sigmoid_f64=False, cell_clip=0.0, next_drop_mask=None,
                              keep=1.0, h_drop=None, workspace_bytes=0, stream=None):
    check(load().lh_gate_gemm_lstm_cell_train_f32(H, B, _segs(segs), len(segs), _ptr(addend), ld_addend,
                                                  _ptr(bias4h), _ptr(c_prev), _ptr(mask01),
                                                  int(sigmoid_f64), cell_clip, _ptr(gates), _ptr(c),
                                                  _ptr(h), _ptr(next_drop_mask), keep, _ptr(h_drop),
                                                  workspace_bytes, _stream(stream)),
          "lh_gate_gemm_lstm_cell_train_f32")


def _gate_problems(problems):
    """problems: dicts with segs=[(A, lda, X, ldx, K)] and either out/ld_out (plain product) or the
    cell fields bias4h, c_prev, mask01, c, h (+ addend, ld_addend, addend_col, addend_ncols,
    sigmoid_f64, cell_clip)."""
    arr = (GateProblem * len(problems))()
    d = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    for q, p in zip(arr, problems):
        for i, (A, lda, X, ldx, K) in enumerate(p["segs"]):
            q.segs[i].A, q.segs[i].lda, q.segs[i].X, q.segs[i].ldx, q.segs[i].K = (
                A.data_ptr(), lda, X.data_ptr(), ldx, K)
        q.nseg = len(p["segs"])
        q.cell = int("c" in p)
        q.addend, q.ld_addend = d(p.get("addend")), p.get("ld_addend", 0)
        q.addend_col, q.addend_ncols = d(p.get("addend_col")), p.get("addend_ncols", 0)
        q.bias4h, q.c_prev, q.mask01 = d(p.get("bias4h")), d(p.get("c_prev")), d(p.get("mask01"))
        q.sigmoid_f64, q.cell_clip = int(p.get("sigmoid_f64", False)), p.get("cell_clip", 0.0)
        q.c, q.h = d(p.get("c")), d(p.get("h"))
        q.out, q.ld_out = d(p.get("out")), p.get("ld_out", 0)
    return arr


def gate_gemm_group_plan(H, B, problems):
    """(runnable, kernel instance name) of lh_gate_gemm_group_f32 on these problems."""
    r, buf = C.c_int(), C.create_string_buffer(128)
    check(load().lh_gate_gemm_group_plan(H, B, _gate_problems(problems), len(problems), C.byref(r),
                                         buf, 128), "lh_gate_gemm_group_plan")
    return bool(r.value), buf.value.decode()


def gate_gemm_group(H, B, problems, stream=None):
    check(load().lh_gate_gemm_group_f32(H, B, _gate_problems(problems), len(problems),
                                        _stream(stream)), "lh_gate_gemm_group_f32")


def split_kgroups(K):
    return load().lh_split_kgroups(K)


def split_kgroups_padded(kgroups):
    return load().lh_split_kgroups_padded(kgroups)


def split_bytes(D, kgroups):
    return load().lh_split_bytes(D, kgroups)


def split_pack(sources, stream=None):
    """sources: dicts with src (tensor), ld, k_contiguous, D, K, planes (tensor), kgroups_total and
    optionally kg_offset (0), kgroups (all from kg_offset to the operand's end when the segment is
    alone, else ceil(K/8)) and gate_H (lh_split_pack_f32, up to 8 per launch)."""
    arr = (SplitSource * len(sources))()
    for i, q in enumerate(sources):
        arr[i].src = q["src"].data_ptr()
        arr[i].ld, arr[i].k_contiguous = q["ld"], int(q["k_contiguous"])
        arr[i].D, arr[i].K, arr[i].gate_H = q["D"], q["K"], q.get("gate_H", 0)
        arr[i].planes = q["planes"].data_ptr()
        arr[i].kgroups_total, arr[i].kg_offset = q["kgroups_total"], q.get("kg_offset", 0)
        arr[i].kgroups = q.get("kgroups", (q["K"] + 7) // 8)
    check(load().lh_split_pack_f32(arr, len(sources), _stream(stream)), "lh_split_pack_f32")


def gemm_split(M, N, kgroups, A_planes, X_planes, C_out, ldc, alpha=1.0, beta=0.0, bias=None,
               act=LH_ACT_NONE, act_rows=None, colmask=None, stream=None):
    check(load().lh_gemm_split_f32(M, N, kgroups, _ptr(A_planes), _ptr(X_planes), alpha, beta,
                                   _ptr(bias), act, M if act_rows is None else act_rows,
                                   _ptr(colmask), _ptr(C_out), ldc, _stream(stream)),
          "lh_gemm_split_f32")


def gate_gemm_split_lstm_cell(H, B, kgroups, W_planes, X_planes, bias4h, c_prev, mask01, c, h,
                              addend=None, ld_addend=0, addend_col=None, addend_ncols=0,
                              sigmoid_f64=False, cell_clip=0.0, h_planes=None, hp_kgroups_total=0,
                              hp_kg_offset=0, hp_kgroups=0, stream=None):
    check(load().lh_gate_gemm_split_lstm_cell_f32(
        H, B, kgroups, _ptr(W_planes), _ptr(X_planes), _ptr(addend), ld_addend, _ptr(addend_col),
        addend_ncols, _ptr(bias4h), _ptr(c_prev), _ptr(mask01), int(sigmoid_f64), cell_clip, _ptr(c),
        _ptr(h), _ptr(h_planes), hp_kgroups_total, hp_kg_offset, hp_kgroups, _stream(stream)),
        "lh_gate_gemm_split_lstm_cell_f32")


def gemm_planes(M, N, segs, C_out, ldc, workspace, max_planes, transA=False, transX=False, beta=0.0,
                stream=None):
    """lh_gemm_planes_f32: returns the number of planes S; for S > 1 the planes are the
    ((M+3)&~3) x N blocks at the start of `workspace` (a float tensor) and C_out is untouched."""
    planes = C.c_int()
    check(load().lh_gemm_planes_f32(M, N, _segs(segs), len(segs), int(transA), int(transX), beta,
                                    _ptr(C_out), ldc, workspace.data_ptr(),
                                    workspace.numel() * workspace.element_size(), max_planes,
                                    C.byref(planes), _stream(stream)), "lh_gemm_planes_f32")
    return planes.value


def gemm_config_info(config, transA=False, transX=False):
    """dict(BM, BN, WM, WN, WK, BK, occupancy, lds_bytes) of one tile configuration."""
    info = (C.c_int * 8)()
    check(load().lh_gemm_config_info(config, int(transA), int(transX), C.byref(info)),
          "lh_gemm_config_info")
    return dict(zip(("BM", "BN", "WM", "WN", "WK", "BK", "occupancy", "lds_bytes"), list(info)))


def lstm_cell_fwd(H, B, pre1, bias4h, c_prev, mask01, c, h, pre2=None, pre3=None,
                  sigmoid_f64=False, cell_clip=0.0, gates=None, next_drop_mask=None, keep=1.0,
                  h_drop=None, stream=None):
    check(load().lh_lstm_cell_fwd_f32(H, B, _ptr(pre1), _ptr(pre2), _ptr(pre3), _ptr(bias4h),
                                      _ptr(c_prev), _ptr(mask01), int(sigmoid_f64), cell_clip,
                                      _ptr(gates), _ptr(c), _ptr(h), _ptr(next_drop_mask), keep,
                                      _ptr(h_drop), _stream(stream)), "lh_lstm_cell_fwd_f32")


def attn_core_fwd(H, B, D, max_len, hs_steps, tanh1, v_p, wa, hs, hs_step_stride, hs_col_stride,
                  hs_col, batch_info, mask01, p_t, sigma, indices, align, cached_exp, ctx,
                  viterbi=None, proj_col_stride=0, stream=None):
    """proj_col_stride: distance between the columns of tanh1 / wa (0 = H)."""
    check(load().lh_attn_core_fwd_f32(H, B, D, max_len, hs_steps, _ptr(tanh1), _ptr(v_p), _ptr(wa),
                                      proj_col_stride, _ptr(hs), hs_step_stride, hs_col_stride,
                                      _ptr(hs_col),
                                      _ptr(batch_info), _ptr(mask01), _ptr(p_t), _ptr(sigma),
                                      _ptr(indices), _ptr(align), _ptr(cached_exp), _ptr(ctx),
                                      _ptr(viterbi), _stream(stream)), "lh_attn_core_fwd_f32")


def softmax_fwd(logits, ldl, bias, V, B, p, ldp, stream=None):
    check(load().lh_softmax_fwd_f32(_ptr(logits), ldl, _ptr(bias), V, B, _ptr(p), ldp,
                                    _stream(stream)), "lh_softmax_fwd_f32")


def train_loglik(p, ldp, V, B, tgt0, mask01, accum, stream=None):
    check(load().lh_train_loglik_f32(_ptr(p), ldp, V, B, _ptr(tgt0), _ptr(mask01), _ptr(accum),
                                     _stream(stream)), "lh_train_loglik_f32")


def logsoftmax_xent(logits, ldl, bias, V, B, tgt0, mask01, logp_tgt, loss_accum, stream=None):
    check(load().lh_logsoftmax_xent_f32(_ptr(logits), ldl, _ptr(bias), V, B, _ptr(tgt0),
                                        _ptr(mask01), _ptr(logp_tgt), _ptr(loss_accum),
                                        _stream(stream)), "lh_logsoftmax_xent_f32")


def beam_topk(logits, ldl, bias, V, B, K, eof_id, cand_logp, cand_id, logp_eof, stream=None):
    check(load().lh_beam_topk_f32(_ptr(logits), ldl, _ptr(bias), V, B, K, eof_id, _ptr(cand_logp),
                                  _ptr(cand_id), _ptr(logp_eof), _stream(stream)),
          "lh_beam_topk_f32")


def beam_topk_ensemble(ps, ldp, V, B, K, eof_id, cand_logp, cand_id, logp_eof, stream=None):
    """ps: the models' V x B probability tensors (lh_softmax_fwd_f32)."""
    arr = (C.c_void_p * len(ps))(*[p.data_ptr() for p in ps])
    check(load().lh_beam_topk_ensemble_f32(arr, len(ps), ldp, V, B, K, eof_id, _ptr(cand_logp),
                                           _ptr(cand_id), _ptr(logp_eof), _stream(stream)),
          "lh_beam_topk_ensemble_f32")


def beam_merge(n_sent, beam, K, step, limit, cand_logp, cand_id, logp_eof, prev_score, diversity,
               penalty, start_id, eof_id, tok, backptr, score, fin_count, fin_beam, fin_score,
               stream=None):
    check(load().lh_beam_merge_f32(n_sent, beam, K, step, _ptr(limit), _ptr(cand_logp),
                                   _ptr(cand_id), _ptr(logp_eof), _ptr(prev_score), diversity,
                                   penalty, start_id, eof_id, _ptr(tok), _ptr(backptr),
                                   _ptr(score), _ptr(fin_count), _ptr(fin_beam), _ptr(fin_score),
                                   _stream(stream)), "lh_beam_merge_f32")


def beam_gather(src, dst, H, B, backptr, B_src=None, stream=None):
    n = len(src)
    B_src = B if B_src is None else B_src
    s = (C.c_void_p * n)(*[t.data_ptr() for t in src])
    d = (C.c_void_p * n)(*[t.data_ptr() for t in dst])
    check(load().lh_beam_gather_f32(s, d, n, H, B, B_src, _ptr(backptr), _stream(stream)),
          "lh_beam_gather_f32")


def beam_merge_gather(n_sent, beam, K, step, limit, cand_logp, cand_id, logp_eof, prev_score,
                      diversity, penalty, start_id, eof_id, tok, backptr, score, fin_count, fin_beam,
                      fin_score, src, dst, H, stream=None):
    n = len(src)
    s = (C.c_void_p * n)(*[t.data_ptr() for t in src])
    d = (C.c_void_p * n)(*[t.data_ptr() for t in dst])
    check(load().lh_beam_merge_gather_f32(n_sent, beam, K, step, _ptr(limit), _ptr(cand_logp),
                                          _ptr(cand_id), _ptr(logp_eof), _ptr(prev_score), diversity,
                                          penalty, start_id, eof_id, _ptr(tok), _ptr(backptr),
                                          _ptr(score), _ptr(fin_count), _ptr(fin_beam),
                                          _ptr(fin_score), s, d, n, H, _stream(stream)),
          "lh_beam_merge_gather_f32")


def beam_merge_gather_stream(n_sent, beam, K, tick, start, limit, cand_logp, cand_id, logp_eof,
                             prev_score, diversity, penalty, start_id, eof_id, tok, backptr, score,
                             fin_count, fin_beam, fin_score, src, dst, H, stream=None):
    n = len(src)
    s = (C.c_void_p * n)(*[t.data_ptr() for t in src])
    d = (C.c_void_p * n)(*[t.data_ptr() for t in dst])
    check(load().lh_beam_merge_gather_stream_f32(n_sent, beam, K, tick, _ptr(start), _ptr(limit),
                                                 _ptr(cand_logp), _ptr(cand_id), _ptr(logp_eof),
                                                 _ptr(prev_score), diversity, penalty, start_id, eof_id,
                                                 _ptr(tok), _ptr(backptr), _ptr(score), _ptr(fin_count),
                                                 _ptr(fin_beam), _ptr(fin_score), s, d, n, H,
                                                 _stream(stream)), "lh_beam_merge_gather_stream_f32")


def stream_admit(admissions, beam, B, start, limit, hs_col, batch_info, src, dst, zero, H, n_src,
                 tok_prev, start_id, score_prev, stream=None):
    """admissions: dicts with slot, sentence_col, hs_col_value, len, off, limit, tick."""
    arr = (StreamAdmission * len(admissions))(*[StreamAdmission(**a) for a in admissions])
    ptrs = lambda ts: (C.c_void_p * max(1, len(ts)))(*[t.data_ptr() for t in ts])  # noqa: E731
    check(load().lh_stream_admit_f32(arr, len(admissions), beam, B, _ptr(start), _ptr(limit),
                                     _ptr(hs_col), _ptr(batch_info), ptrs(src), ptrs(dst), len(src),
                                     ptrs(zero), len(zero), H, n_src, _ptr(tok_prev), start_id,
                                     _ptr(score_prev), _stream(stream)), "lh_stream_admit_f32")


# ---- training half ------------------------------------------------------------------------------
def softmax_xent_grad(logits, ldl, bias, V, B, tgt0, mask01, dz, ldz, logp_tgt, loss_accum,
                      stream=None):
    check(load().lh_softmax_xent_grad_f32(_ptr(logits), ldl, _ptr(bias), V, B, _ptr(tgt0),
                                          _ptr(mask01), _ptr(dz), ldz, _ptr(logp_tgt),
                                          _ptr(loss_accum), _stream(stream)),
          "lh_softmax_xent_grad_f32")


def uniform(out, n, seed, stream=None):
    check(load().lh_uniform_f32(_ptr(out), n, seed, _stream(stream)), "lh_uniform_f32")


def lstm_cell_bwd(H, B, gates, c, c_prev, mask01, dgates, dc_prev, dh_above=None, dh_next=None,
                  dc_next=None, clip_above=0.0, clip_next=0.0, above_drop_mask=None, keep=1.0,
                  stream=None):
    check(load().lh_lstm_cell_bwd_f32(H, B, _ptr(dh_above), _ptr(dh_next), _ptr(dc_next),
                                      _ptr(gates), _ptr(c), _ptr(c_prev), _ptr(mask01), clip_above,
                                      clip_next, _ptr(above_drop_mask), keep, _ptr(dgates),
                                      _ptr(dc_prev), _stream(stream)),
          "lh_lstm_cell_bwd_f32")


class ErrorTerm(C.Structure):
    """lh_error_term: an incoming error as the sum of `planes` H x B blocks (ld, plane_stride in floats)."""
    _fields_ = [("p", C.c_void_p), ("planes", C.c_int), ("plane_stride", C.c_longlong), ("ld", C.c_int)]


def error_term(t, planes, ld, plane_stride=0):
    return ErrorTerm(t.data_ptr(), planes, plane_stride, ld)


def lstm_cell_bwd_terms(H, B, gates, c, c_prev, mask01, dgates, dc_prev, above=None, next=None,
                        dc_next=None, clip_above=0.0, clip_next=0.0, above_drop_mask=None, keep=1.0,
                        stream=None):
    """above / next: ErrorTerm or None."""
    check(load().lh_lstm_cell_bwd_terms_f32(H, B, C.byref(above) if above is not None else None,
                                            C.byref(next) if next is not None else None, _ptr(dc_next),
                                            _ptr(gates), _ptr(c), _ptr(c_prev), _ptr(mask01), clip_above,
                                            clip_next, _ptr(above_drop_mask), keep, _ptr(dgates),
                                            _ptr(dc_prev), _stream(stream)),
          "lh_lstm_cell_bwd_terms_f32")


def rowsum_acc(A, lda, rows, cols, out, beta=0.0, stream=None):
    check(load().lh_rowsum_acc_f32(_ptr(A), lda, rows, cols, beta, _ptr(out), _stream(stream)),
          "lh_rowsum_acc_f32")


def embed_gather_grad(dx, ldx, E, n_unique, seg_start, seg_cols, small_grad, ldg, beta=0.0,
                      drop_mask=None, keep=1.0, stream=None):
    check(load().lh_embed_gather_grad_f32(_ptr(dx), ldx, E, n_unique, _ptr(seg_start),
                                          _ptr(seg_cols), _ptr(drop_mask), keep, beta,
                                          _ptr(small_grad), ldg, _stream(stream)),
          "lh_embed_gather_grad_f32")


def attn_delta(H, B, dht, h_tild, mask01, delta, dht_feed=None, clip_feed=0.0, stream=None):
    check(load().lh_attn_delta_f32(H, B, _ptr(dht), _ptr(dht_feed), _ptr(h_tild), _ptr(mask01),
                                   clip_feed, _ptr(delta), _stream(stream)), "lh_attn_delta_f32")


def attn_core_bwd(H, B, D, max_len, hs_steps, dctx, tanh1, v_p, wa, hs, hs_step_stride,
                  hs_col_stride, batch_info, p_t, sigma, indices, align, cached_exp, dhs, hsum, u,
                  w, stream=None):
    check(load().lh_attn_core_bwd_f32(H, B, D, max_len, hs_steps, _ptr(dctx), _ptr(tanh1),
                                      _ptr(v_p), _ptr(wa), _ptr(hs), hs_step_stride, hs_col_stride,
                                      _ptr(batch_info), _ptr(p_t), _ptr(sigma), _ptr(indices),
                                      _ptr(align), _ptr(cached_exp), _ptr(dhs), _ptr(hsum), _ptr(u),
                                      _ptr(w), _stream(stream)), "lh_attn_core_bwd_f32")


def grad_sumsq(g, rows, cols, ld, scale, workspace, accum, stream=None):
    check(load().lh_grad_sumsq_f32(_ptr(g), rows, cols, ld, scale, _ptr(workspace), _ptr(accum),
                                   _stream(stream)), "lh_grad_sumsq_f32")


def sgd_step(theta, ld_theta, g, ld_g, rows, cols, learning_rate, grad_scale, col_index=None,
             sumsq=None, norm_clip=0.0, individual_clip=0.0, stream=None):
    check(load().lh_sgd_step_f32(_ptr(theta), ld_theta, _ptr(g), ld_g, rows, cols,
                                 _ptr(col_index), learning_rate, grad_scale, _ptr(sumsq),
                                 norm_clip, individual_clip, _stream(stream)), "lh_sgd_step_f32")
