"""numpy binding of the CPU oracle (oracle/liblinmt_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of bench.py as the checker / reported baseline.  Nothing under linmt_amd/ imports this.
All arrays are numpy, column-major data is passed as Fortran-ordered 2-D arrays (or flat arrays
holding the column-major data).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblinmt_oracle.so")
_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])


class ModelConfig(C.Structure):
    _fields_ = [("layers", C.c_int), ("H", C.c_int), ("V_src", C.c_int), ("V_tgt", C.c_int),
                ("attention", C.c_int), ("D", C.c_int), ("feed_input", C.c_int),
                ("longest_sent", C.c_int), ("E", C.c_int)]


class DecodeOpts(C.Structure):
    _fields_ = [("beam", C.c_int), ("max_ratio", C.c_float), ("min_ratio", C.c_float),
                ("penalty", C.c_float), ("diversity", C.c_float), ("lp_alpha", C.c_float),
                ("cp_beta", C.c_float), ("num_threads", C.c_int)]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.orc_model_create.restype = C.c_void_p
        _lib.orc_model_param.restype = C.c_void_p
        _lib.orc_forward_xent.restype = C.c_double
        _lib.orc_decode_sentence.restype = C.c_int
        _lib.orc_trainer_create.restype = C.c_void_p
        _lib.orc_trainer_grad.restype = C.c_void_p
        _lib.orc_compute_gradients.restype = C.c_double
        _lib.orc_update_weights.restype = C.c_float
    return _lib


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"] or a.flags["F_CONTIGUOUS"], "oracle arrays must be contiguous"
    # data_as() keeps a reference to the array, so temporaries made in the argument list stay alive
    # until the foreign call has returned.
    return a.ctypes.data_as(C.c_void_p)


def _f(v):
    return C.c_float(v)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def preprocess_indices(idx):
    idx = i32(idx).ravel()
    idx0 = np.empty_like(idx)
    m = np.empty_like(idx)
    mf = np.empty(idx.shape, np.float32)
    lib().orc_preprocess_indices(_p(idx), idx.size, _p(idx0), _p(m), _p(mf))
    return idx0, m, mf


def setup_reverse_indices(unique, vocab):
    unique = i32(unique)
    rev = np.full(vocab, -7, np.int32)
    lib().orc_setup_reverse_indices(_p(unique), unique.size, _p(rev))
    return rev


def embed_lookup(W, idx0, drop_mask=None, keep=1.0):
    """W: (E,V) Fortran; returns (E,B) Fortran."""
    E, V = W.shape
    W = np.asfortranarray(W, np.float32)
    idx0 = i32(idx0)
    out = np.empty((E, idx0.size), np.float32, order="F")
    dm = None if drop_mask is None else np.asfortranarray(drop_mask, np.float32)
    lib().orc_embed_lookup(_p(W), E, V, _p(idx0), idx0.size, _p(dm), _f(keep), _p(out))
    return out


def gemm(A, X, transA=False, transX=False, alpha=1.0, beta=0.0, C0=None):
    A = np.asfortranarray(A, np.float32)
    X = np.asfortranarray(X, np.float32)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = X.shape[0] if transX else X.shape[1]
    out = np.zeros((M, N), np.float32, order="F") if C0 is None else np.asfortranarray(
        C0, np.float32).copy(order="F")
    lib().orc_gemm(M, N, K, _p(A), A.shape[0], int(transA), _p(X), X.shape[0], int(transX),
                   _f(alpha), _f(beta), _p(out), M)
    return out


def lstm_cell_fwd(pre1, bias4h, c_prev, mask01, pre2=None, pre3=None, feed=False, cell_clip=0.0):
    """pre*: (4H,B) Fortran; returns gates (4H,B), c (H,B), h (H,B)."""
    H4, B = pre1.shape
    H = H4 // 4
    fa = lambda a: None if a is None else np.asfortranarray(a, np.float32)
    pre1, pre2, pre3, c_prev = fa(pre1), fa(pre2), fa(pre3), fa(c_prev)
    gates = np.empty((H4, B), np.float32, order="F")
    c = np.empty((H, B), np.float32, order="F")
    h = np.empty((H, B), np.float32, order="F")
    lib().orc_lstm_cell_fwd(H, B, _p(pre1), _p(pre2), _p(pre3), _p(f32(bias4h)), _p(c_prev),
                            _p(i32(mask01)), int(feed), _f(cell_clip), _p(gates), _p(c), _p(h))
    return gates, c, h


def attn_core_fwd(H, B, D, max_len, hs_steps, tanh1, v_p, wa, hs, step_stride, col_stride, hs_col,
                  batch_info, mask01):
    W = 2 * D + 1 if D >= 0 else max_len
    out = dict(p_t=np.zeros(B, np.float32), sigma=np.zeros(B, np.float32),
               indices=np.empty((B, W), np.int32, order="F"),
               align=np.empty((B, W), np.float32, order="F"),
               cached_exp=np.empty((W, B), np.float32, order="F"),
               ctx=np.empty((H, B), np.float32, order="F"), viterbi=np.empty(B, np.int32))
    fa = lambda a: None if a is None else np.asfortranarray(a, np.float32)
    lib().orc_attn_core_fwd(H, B, D, max_len, hs_steps, _p(fa(tanh1)), _p(None if v_p is None else f32(v_p)),
                            _p(fa(wa)), _p(f32(hs)), C.c_longlong(step_stride),
                            C.c_longlong(col_stride), _p(None if hs_col is None else i32(hs_col)),
                            _p(i32(batch_info)), _p(i32(mask01)), _p(out["p_t"]), _p(out["sigma"]),
                            _p(out["indices"]), _p(out["align"]), _p(out["cached_exp"]),
                            _p(out["ctx"]), _p(out["viterbi"]))
    return out


def attn_node_fwd(H, B, D, max_len, hs_steps, h_t, W_a, W_p, v_p, b_out, W_c1, W_c2, hs,
                  step_stride, col_stride, hs_col, batch_info, mask01):
    W = 2 * D + 1 if D >= 0 else max_len
    fa = lambda a: None if a is None else np.asfortranarray(a, np.float32)
    out = dict(h_tild=np.empty((H, B), np.float32, order="F"), p_t=np.zeros(B, np.float32),
               indices=np.empty((B, W), np.int32, order="F"),
               align=np.empty((B, W), np.float32, order="F"),
               ctx=np.empty((H, B), np.float32, order="F"))
    lib().orc_attn_node_fwd(H, B, D, max_len, hs_steps, _p(fa(h_t)), _p(fa(W_a)), _p(fa(W_p)),
                            _p(None if v_p is None else f32(v_p)), _p(f32(b_out)), _p(fa(W_c1)),
                            _p(fa(W_c2)), _p(f32(hs)), C.c_longlong(step_stride),
                            C.c_longlong(col_stride), _p(None if hs_col is None else i32(hs_col)),
                            _p(i32(batch_info)), _p(i32(mask01)), _p(out["h_tild"]), _p(out["p_t"]),
                            _p(out["indices"]), _p(out["align"]), _p(out["ctx"]))
    return out


def softmax_fwd(logits, bias=None):
    logits = np.asfortranarray(logits, np.float32)
    V, B = logits.shape
    p = np.empty((V, B), np.float32, order="F")
    lib().orc_softmax_fwd(_p(logits), V, _p(None if bias is None else f32(bias)), V, B, _p(p), V)
    return p


def train_loglik(p, tgt0, mask01, accum=0.0):
    p = np.asfortranarray(p, np.float32)
    V, B = p.shape
    acc = np.array([accum], np.float64)
    lib().orc_train_loglik(_p(p), V, V, B, _p(i32(tgt0)), _p(i32(mask01)), _p(acc))
    return float(acc[0])


def logsoftmax_xent(logits, bias, tgt0, mask01):
    logits = np.asfortranarray(logits, np.float32)
    V, B = logits.shape
    lp = np.empty(B, np.float64)
    acc = np.zeros(1, np.float64)
    lib().orc_logsoftmax_xent(_p(logits), V, _p(None if bias is None else f32(bias)), V, B,
                              _p(i32(tgt0)), _p(i32(mask01)), _p(lp), _p(acc))
    return lp, float(acc[0])


def beam_expand(p, step, prev_score, diversity=0.0, penalty=0.0, start_id=0, eof_id=1):
    """p: (V, beam) Fortran probabilities.  Returns dict(tok, backptr, score, fin_beam, fin_score)."""
    p = np.asfortranarray(p, np.float32)
    V, beam = p.shape
    tok = np.empty(beam, np.int32)
    bp = np.empty(beam, np.int32)
    sc = np.empty(beam, np.float32)
    fc = np.zeros(1, np.int32)
    fb = np.zeros(max(beam, 1) * 2 + 4, np.int32)
    fs = np.zeros(max(beam, 1) * 2 + 4, np.float32)
    lib().orc_beam_expand(_p(p), V, beam, step, _p(f32(prev_score)), _f(diversity), _f(penalty),
                          start_id, eof_id, _p(tok), _p(bp), _p(sc), _p(fc), _p(fb), _p(fs))
    n = int(fc[0])
    return dict(tok=tok, backptr=bp, score=sc, fin_beam=fb[:n].copy(), fin_score=fs[:n].copy())


def beam_expand_ensemble(ps, step, prev_score, diversity=0.0, penalty=0.0, start_id=0, eof_id=1):
    """ps: the models' (V, beam) probabilities.  Result as beam_expand."""
    ps = [np.asfortranarray(p, np.float32) for p in ps]
    V, beam = ps[0].shape
    tok = np.empty(beam, np.int32)
    bp = np.empty(beam, np.int32)
    sc = np.empty(beam, np.float32)
    fc = np.zeros(1, np.int32)
    fb = np.zeros(max(beam, 1) * 2 + 4, np.int32)
    fs = np.zeros(max(beam, 1) * 2 + 4, np.float32)
    arr = (C.c_void_p * len(ps))(*[p.ctypes.data for p in ps])
    lib().orc_beam_expand_ensemble(arr, len(ps), V, beam, step, _p(f32(prev_score)), _f(diversity),
                                   _f(penalty), start_id, eof_id, _p(tok), _p(bp), _p(sc), _p(fc),
                                   _p(fb), _p(fs))
    n = int(fc[0])
    return dict(tok=tok, backptr=bp, score=sc, fin_beam=fb[:n].copy(), fin_score=fs[:n].copy())


def beam_step_margin(ps, step, prev_score, diversity=0.0, start_id=0, eof_id=1):
    """ps: the models' (V, beam) probabilities; the smallest gap the expansion had to resolve."""
    ps = [np.asfortranarray(p, np.float32) for p in ps]
    V, beam = ps[0].shape
    arr = (C.c_void_p * len(ps))(*[p.ctypes.data for p in ps])
    f = lib().orc_beam_step_margin
    f.restype = C.c_float
    return float(f(arr, len(ps), V, beam, step, _p(f32(prev_score)), _f(diversity), start_id,
                   eof_id))


def beam_gather(src, backptr):
    src = np.asfortranarray(src, np.float32)
    H, B = src.shape
    dst = np.empty((H, B), np.float32, order="F")
    lib().orc_beam_gather(_p(src), _p(dst), H, B, _p(i32(backptr)))
    return dst


# ---- training kernels (argument meaning of the lh_* entry points of the same name) -----------------
def _fa(a):
    return None if a is None else np.asfortranarray(a, np.float32)


def lstm_cell_bwd(gates, c, c_prev, mask01, dh_above=None, dh_next=None, dc_next=None,
                  clip_above=0.0, clip_next=0.0, above_drop_mask=None, keep=1.0):
    """gates (4H,B), c / c_prev (H,B).  Returns dgates (4H,B), dc_prev (H,B)."""
    H4, B = gates.shape
    H = H4 // 4
    dg = np.empty((H4, B), np.float32, order="F")
    dcp = np.empty((H, B), np.float32, order="F")
    lib().orc_lstm_cell_bwd(H, B, _p(_fa(dh_above)), _p(_fa(dh_next)), _p(_fa(dc_next)),
                            _p(_fa(gates)), _p(_fa(c)), _p(_fa(c_prev)), _p(i32(mask01)),
                            _f(clip_above), _f(clip_next), _p(_fa(above_drop_mask)), _f(keep),
                            _p(dg), _p(dcp))
    return dg, dcp


def softmax_xent_grad(logits, bias, tgt0, mask01):
    """Returns dz (V,B), logp_tgt (B,) float64, masked sum of logp_tgt."""
    logits = _fa(logits)
    V, B = logits.shape
    dz = np.empty((V, B), np.float32, order="F")
    lp = np.zeros(B, np.float64)
    acc = np.zeros(1, np.float64)
    lib().orc_softmax_xent_grad(_p(logits), V, _p(None if bias is None else f32(bias)), V, B,
                                _p(i32(tgt0)), _p(i32(mask01)), _p(dz), V, _p(lp), _p(acc))
    return dz, lp, float(acc[0])


def attn_delta(dht, h_tild, mask01, dht_feed=None, clip_feed=0.0):
    H, B = dht.shape
    out = np.empty((H, B), np.float32, order="F")
    lib().orc_attn_delta(H, B, _p(_fa(dht)), _p(_fa(dht_feed)), _p(_fa(h_tild)), _p(i32(mask01)),
                         _f(clip_feed), _p(out))
    return out


def attn_core_bwd(H, B, D, max_len, hs_steps, dctx, tanh1, v_p, wa, hs, step_stride, col_stride,
                  batch_info, fwd, dhs0):
    """fwd: the dict attn_core_fwd returned.  dhs0: flat float32 array laid out like hs; a copy
    with the step's contribution added comes back as out['dhs']."""
    out = dict(dhs=f32(dhs0).copy(), hsum=np.empty((H, B), np.float32, order="F"),
               u=np.zeros((H, B), np.float32, order="F"), w=np.zeros((H, B), np.float32, order="F"))
    lib().orc_attn_core_bwd(H, B, D, max_len, hs_steps, _p(_fa(dctx)), _p(_fa(tanh1)),
                            _p(None if v_p is None else f32(v_p)), _p(_fa(wa)), _p(f32(hs)),
                            C.c_longlong(step_stride), C.c_longlong(col_stride),
                            _p(i32(batch_info)), _p(fwd["p_t"]), _p(fwd["sigma"]),
                            _p(fwd["indices"]), _p(fwd["align"]), _p(fwd["cached_exp"]),
                            _p(out["dhs"]), _p(out["hsum"]), _p(out["u"]), _p(out["w"]))
    return out


MODEL_FILE_RULE = "=" * 58


def model_file_order(layers, H, Vs, Vt, attention, feed_input):
    """[(name, rows, cols)] in the order the reference's model file holds the matrices:
    NeuralMachineTranslation::DumpWeights (src/deep_rnn.h:2124-2146) walks the source layers, the
    target layers and the softmax; a layer writes W_hi b_i W_hf b_f W_hc b_c W_ho b_o, the
    embedding table (input layer only), M_i M_f M_o M_c, Q_i Q_f Q_o Q_c (feed input) and -- the
    layer the attention is attached to, the top target layer -- W_a W_p v_p b_out W_c1 W_c2
    (src/layer_input_to_hidden.h:1556-1590, src/layer_hidden_to_hidden.h:989-1014,
    src/layer_attention.h:1264-1273); the softmax writes D and b_d (src/layer_loss.h:1213-1218)."""
    out = []
    for side, V in (("src", Vs), ("tgt", Vt)):
        for l in range(layers):
            p = f"{side}.{l}."
            for g in "ifco":
                out += [(p + "W_h" + g, H, H), (p + "b_" + g, H, 1)]
            if l == 0:
                out.append((p + "W", H, V))
            out += [(p + "M_" + g, H, H) for g in "ifoc"]
            if side == "tgt" and l == 0 and attention and feed_input:
                out += [(p + "Q_" + g, H, H) for g in "ifoc"]
            if side == "tgt" and l == layers - 1 and attention:
                out += [("attn.W_a", H, H), ("attn.W_p", H, H), ("attn.v_p", H, 1), ("attn.b_out", H, 1),
                        ("attn.W_c1", H, H), ("attn.W_c2", H, H)]
    return out + [("softmax.D", Vt, H), ("softmax.b_d", Vt, 1)]


def write_model_file(path, params, layers, H, Vs, Vt, attention=1, feed_input=1, source_words=None,
                     target_words=None):
    """A complete model file as the reference's programs leave it, written from the source: the
    first line of cc_util::AddModelInformation (src/utility_cc.cc:76-98: layers, lstm size, target
    and source vocabulary sizes, attention, feed input, three zeros), the vocabulary mappings
    between rules of 58 '=' (src/input_file_preprocess.cc:545-575: "<id> <word>" per line, source
    id 0 = <UNK>, target ids 0-2 = <START> <EOF> <UNK>), then every matrix as WriteMatrixGpu
    writes it (src/deep_rnn_kernel.h:1564-1578: a line per row, single spaces, an empty line after
    the matrix) with the stream's precision at digits10 + 2 = 8 significant digits
    (src/deep_rnn.h:2127), which for an ostream in its default float format is printf's %.8g."""
    src_words = list(source_words) if source_words else ["<UNK>"] + [f"w{i}" for i in range(1, Vs)]
    tgt_words = list(target_words) if target_words else ["<START>", "<EOF>", "<UNK>"] + [f"w{i}" for i in range(3, Vt)]
    with open(path, "w") as f:
        f.write(f"{layers} {H} {Vt} {Vs} {int(bool(attention))} {int(bool(attention and feed_input))} 0 0 0\n")
        f.write(MODEL_FILE_RULE + "\n")
        for i in range(Vs):
            f.write(f"{i} {src_words[i]}\n")
        f.write(MODEL_FILE_RULE + "\n")
        for i in range(Vt):
            f.write(f"{i} {tgt_words[i]}\n")
        f.write(MODEL_FILE_RULE + "\n")
        for name, rows, cols in model_file_order(layers, H, Vs, Vt, attention, feed_input):
            m = np.asarray(params[name], np.float32).reshape((rows, cols))
            for i in range(rows):
                f.write(" ".join("%.8g" % float(x) for x in m[i]) + "\n")
            f.write("\n")


def read_model_file(path):
    """What NeuralMachineTranslation::LoadWeights (src/deep_rnn.h:1878-1968) and ReadMatrixGpu
    (src/deep_rnn_kernel.h:1543-1561) make of a model file: the first line's numbers, the two
    vocabulary lists, and every matrix with its numbers converted as (float)stod(token)."""
    with open(path) as f:
        lines = f.read().split("\n")
    head = [int(x) for x in lines[0].split()]
    layers, H, Vt, Vs = head[:4]
    attention, feed = (head[4], head[5]) if len(head) > 5 else (0, 0)
    is_rule = lambda l: len(l) > 3 and l[:3] == "==="  # noqa: E731
    assert is_rule(lines[1])
    k, vocab = 2, [[], []]
    for part in range(2):
        while not is_rule(lines[k]):
            vocab[part].append(lines[k].split(" ", 1)[1])
            k += 1
        k += 1
    params = {}
    for name, rows, cols in model_file_order(layers, H, Vs, Vt, attention, feed):
        m = np.array([[float(t) for t in lines[k + i].split()[:cols]] for i in range(rows)], np.float64)
        assert m.shape == (rows, cols), name
        params[name] = m.astype(np.float32).reshape((rows, cols) if cols > 1 else (rows,))
        k += rows + 1
    return dict(layers=layers, H=H, Vs=Vs, Vt=Vt, attention=attention, feed_input=feed,
                source_words=vocab[0], target_words=vocab[1]), params


class TrainingFile:
    """The reference's integerised training file read the way FileHelper::ReadMinibatch does
    (src/file_helper.cc:113-381, statistics as GetFileStats, src/utility_cc.cc:17-58), written
    from the source with numpy: four lines per sentence pair (source input, source output, target
    input, target output; -1 pads; every pair of a minibatch padded to common lengths),
    minibatch_size pairs per minibatch, the file starting over after its last minibatch."""

    def __init__(self, path, minibatch_size):
        with open(path) as fh:
            lines = fh.read().split("\n")
        if lines and lines[-1] == "":
            lines.pop()
        self.lines = [np.array(l.split(), dtype=np.int64) for l in lines]
        self.B = minibatch_size
        assert len(self.lines) % (4 * minibatch_size) == 0, "whole minibatches only"
        # GetFileStats: non-pad ids of the two input lines of every pair
        self.total_words = int(sum((l != -1).sum() for k, l in enumerate(self.lines) if k % 4 in (0, 2)))
        self.total_target_words = int(sum((l != -1).sum() for k, l in enumerate(self.lines) if k % 4 == 2))
        self.cursor = 0  # index of the next pair's first line

    @staticmethod
    def _wgrad(ids_column_major):
        """PreprocessInputWgrad (:248-378): first occurrences in column-major order, every other
        position -1, then the in-place partition that swaps the leftmost -1 with the rightmost id."""
        v = ids_column_major.copy()
        seen = set()
        for i, w in enumerate(v):
            if w == -1 or w in seen:
                v[i] = -1
            else:
                seen.add(int(w))
        left, right = 0, len(v) - 1
        while left < right:
            if v[left] == -1:
                if v[right] != -1:
                    v[left], v[right] = v[right], v[left]
                    left += 1
                right -= 1
                continue
            left += 1
        if len(v) and v[left] != -1:
            left += 1
        return v[:left].astype(np.int32)

    def read_minibatch(self):
        """Returns (minibatch, same_epoch): same_epoch is False for the last minibatch of a pass."""
        B = self.B
        block = self.lines[self.cursor:self.cursor + 4 * B]
        self.cursor += 4 * B
        same_epoch = self.cursor < len(self.lines)
        if not same_epoch:
            self.cursor = 0
        src = np.stack(block[0::4]).astype(np.int32)   # (B, S): row = sentence, column = timestep
        tin = np.stack(block[2::4]).astype(np.int32)
        tout = np.stack(block[3::4]).astype(np.int32)
        lens = (src != -1).sum(axis=1)
        mb = dict(src=src, tgt_in=tin, tgt_out=tout,
                  batch_info=np.concatenate([lens, src.shape[1] - lens]).astype(np.int32),
                  src_wgrad=self._wgrad(src.ravel(order="F")), tgt_wgrad=self._wgrad(tin.ravel(order="F")),
                  words_in_minibatch=int((src != -1).sum() + (tout != -1).sum()))
        return mb, same_epoch


class Model:
    """Host model of the oracle; parameters are numpy views into the oracle's own buffers."""

    def __init__(self, layers, H, V_src, V_tgt, attention=1, D=10, feed_input=1, longest_sent=104,
                 E=0):
        """E: embedding size, 0 = H (the reference's only case)."""
        self.cfg = ModelConfig(layers, H, V_src, V_tgt, attention, D, feed_input, longest_sent, E)
        self.E = E if E > 0 else H
        self.handle = C.c_void_p(lib().orc_model_create(C.byref(self.cfg)))

    def param(self, name):
        n = C.c_longlong(0)
        ptr = lib().orc_model_param(self.handle, name.encode(), C.byref(n))
        if not ptr:
            raise KeyError(name)
        buf = (C.c_float * n.value).from_address(ptr)
        return np.frombuffer(buf, dtype=np.float32)

    def set_params(self, params):
        for name, arr in params.items():
            dst = self.param(name)
            src = np.asarray(arr, np.float32)
            assert src.size == dst.size, (name, src.shape, dst.size)
            dst[:] = src.ravel(order="F")
        lib().orc_model_commit(self.handle)

    def decode_sentence(self, src_ids, beam=12, max_ratio=1.5, min_ratio=0.5, penalty=0.0,
                        diversity=0.0, lp_alpha=0.65, cp_beta=0.20, num_threads=0, hyp_cap=4096,
                        alignments=False, ensemble=()):
        """alignments=True: the reference's unk_replacement_mode__ (exported alignment scores,
        coverage penalty on them); the result then holds best_viterbi.  ensemble: further models
        whose distributions are averaged with this one's before every beam step."""
        src_ids = i32(src_ids)
        cap = self.cfg.longest_sent + 2
        o = DecodeOpts(beam, max_ratio, min_ratio, penalty, diversity, lp_alpha, cp_beta,
                       num_threads)
        best = np.zeros(cap, np.int32)
        blen = C.c_int(0)
        bscore = C.c_float(0)
        ht = np.zeros((hyp_cap, cap), np.int32)
        hl = np.zeros(hyp_cap, np.int32)
        hs = np.zeros(hyp_cap, np.float32)
        nh = C.c_int(0)
        vit = np.full(cap, -1, np.int32)
        if ensemble:
            handles = (C.c_void_p * (1 + len(ensemble)))(self.handle, *[m.handle for m in ensemble])
            f = lib().orc_decode_sentence_ensemble
            f.restype = C.c_int
            f.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int] + \
                [C.c_void_p, C.c_int] + [C.c_void_p] * 6 + [C.c_int, C.c_void_p]
            alignments = alignments and all(m.cfg.attention for m in (self,) + tuple(ensemble))
            steps = f(handles, len(handles), _p(src_ids), src_ids.size, C.byref(o), int(alignments),
                      _p(best), cap, C.byref(blen), C.byref(bscore), _p(vit), _p(ht), _p(hl), _p(hs),
                      hyp_cap, C.byref(nh))
        elif alignments:
            steps = lib().orc_decode_sentence_alignments(
                self.handle, _p(src_ids), src_ids.size, C.byref(o), _p(best), cap, C.byref(blen),
                C.byref(bscore), _p(vit), _p(ht), _p(hl), _p(hs), hyp_cap, C.byref(nh))
        else:
            steps = lib().orc_decode_sentence(self.handle, _p(src_ids), src_ids.size, C.byref(o),
                                              _p(best), cap, C.byref(blen), C.byref(bscore),
                                              _p(ht), _p(hl), _p(hs), hyp_cap, C.byref(nh))
        n = min(nh.value, hyp_cap)
        hyps = [(ht[i, :hl[i]].copy(), float(hs[i])) for i in range(n)]
        out = dict(best=best[:blen.value].copy(), best_score=float(bscore.value), hyps=hyps,
                   steps=steps)
        if alignments:
            out["best_viterbi"] = vit[:blen.value].copy()
        return out

    def decode_sentence_trace(self, src_ids, beam=12, max_ratio=1.5, min_ratio=0.5, penalty=0.0,
                              diversity=0.0, lp_alpha=0.65, cp_beta=0.20, num_threads=0):
        """decode_sentence plus the beam after every expansion step: dict(best, best_score, steps,
        tok (n, beam), backptr (n, beam; beam-local), score (n, beam), margin (n,)) where margin is
        the smallest gap between two candidates the step had to order (orc_beam_step_margin) and
        window_margin (n,) the smallest distance of a live column's local-p window position from
        an integer."""
        src_ids = i32(src_ids)
        cap = self.cfg.longest_sent + 2
        b = min(beam, int(np.sqrt(self.cfg.V_tgt)))
        o = DecodeOpts(beam, max_ratio, min_ratio, penalty, diversity, lp_alpha, cp_beta,
                       num_threads)
        best = np.zeros(cap, np.int32)
        blen, bscore, nst = C.c_int(0), C.c_float(0), C.c_int(0)
        tok = np.zeros((cap, b), np.int32)
        bp = np.zeros((cap, b), np.int32)
        sc = np.zeros((cap, b), np.float32)
        mg = np.zeros(cap, np.float32)
        wm = np.zeros(cap, np.float32)
        f = lib().orc_decode_sentence_trace
        f.restype = C.c_int
        f.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int,
                      C.c_void_p, C.c_void_p] + [C.c_void_p] * 4 + [C.c_int, C.c_void_p, C.c_void_p]
        steps = f(self.handle, _p(src_ids), src_ids.size, C.byref(o), _p(best), cap,
                  C.byref(blen), C.byref(bscore), _p(tok), _p(bp), _p(sc), _p(mg), cap,
                  C.byref(nst), _p(wm))
        n = nst.value
        return dict(best=best[:blen.value].copy(), best_score=float(bscore.value), steps=steps,
                    tok=tok[:n].copy(), backptr=bp[:n].copy(), score=sc[:n].copy(),
                    margin=mg[:n].copy(), window_margin=wm[:n].copy())

    def forward_xent(self, src, tgt_in, tgt_out, batch_info, num_threads=0):
        """src (B,S), tgt_in/tgt_out (B,T) int arrays with -1 padding (column t = timestep t)."""
        src = np.asfortranarray(src, np.int32)
        tgt_in = np.asfortranarray(tgt_in, np.int32)
        tgt_out = np.asfortranarray(tgt_out, np.int32)
        B, S = src.shape
        T = tgt_in.shape[1]
        return lib().orc_forward_xent(self.handle, _p(src), S, _p(tgt_in), _p(tgt_out), T, B,
                                      _p(i32(batch_info)), num_threads)

    # ---- training -------------------------------------------------------------------------------
    def _trainer(self):
        if getattr(self, "trainer", None) is None:
            self.trainer = C.c_void_p(lib().orc_trainer_create(self.handle, C.byref(self.cfg)))
        return self.trainer

    def set_dropout(self, keep, B=1, src_embed=None, tgt_embed=None, src_out=None, tgt_out=None):
        """Masks as flat float32 arrays in device layout: embed (steps, B, H) C-order = H x B x steps
        column-major; out (layers, steps, B, H).  keep <= 0 switches dropout off."""
        t = self._trainer()
        if not keep > 0:
            lib().orc_trainer_set_dropout(t, _f(0.0), None, None, None, None, 0, 0, 0)
            return
        H, L = self.cfg.H, self.cfg.layers
        se, te, so, to = (f32(a).ravel() for a in (src_embed, tgt_embed, src_out, tgt_out))
        S, T = se.size // (self.E * B), te.size // (self.E * B)
        assert so.size == L * S * H * B and to.size == L * T * H * B
        lib().orc_trainer_set_dropout(t, _f(keep), _p(se), _p(te), _p(so), _p(to), S, T, B)

    def set_clip(self, cell_clip=0.0, error_clip=0.0):
        """The reference's --clip-cell for the following compute_gradients calls (0 = off)."""
        lib().orc_trainer_set_clip(self._trainer(), _f(cell_clip), _f(error_clip))

    def set_train_modes(self, source_input_embedding=True, target_input_embedding=True,
                        target_output_embedding=True, source_rnn=True, target_rnn=True,
                        attention_target_rnn=True):
        """The train_*_mode__ switches UpdateParams reads (finetune: the three embedding groups off)."""
        modes = i32([source_input_embedding, target_input_embedding, target_output_embedding,
                     source_rnn, target_rnn, attention_target_rnn])
        lib().orc_trainer_set_train_modes(self._trainer(), _p(modes))

    def compute_gradients(self, src, tgt_in, tgt_out, batch_info, src_unique, tgt_unique):
        """Forward + backward (no update).  Returns (sum log p, {name: gradient}); matrices come back
        as Fortran-ordered 2-D arrays, the embedding gradients as (E, n_unique)."""
        self._trainer()
        src = np.asfortranarray(src, np.int32)
        tgt_in = np.asfortranarray(tgt_in, np.int32)
        tgt_out = np.asfortranarray(tgt_out, np.int32)
        B, S = src.shape
        T = tgt_in.shape[1]
        su, tu = i32(src_unique), i32(tgt_unique)
        ll = lib().orc_compute_gradients(self.trainer, _p(src), S, _p(tgt_in), _p(tgt_out), T, B,
                                         _p(i32(batch_info)), _p(su), su.size, _p(tu), tu.size)
        return ll, {name: self.grad(name) for name in self.param_names()}

    def param_names(self):
        c = self.cfg
        names = []
        for side in ("src", "tgt"):
            for l in range(c.layers):
                for g in "ifco":
                    names += [f"{side}.{l}.W_h{g}", f"{side}.{l}.M_{g}", f"{side}.{l}.b_{g}"]
                    if side == "tgt" and l == 0 and c.feed_input and c.attention:
                        names.append(f"{side}.{l}.Q_{g}")
                if l == 0:
                    names.append(f"{side}.{l}.W")
        if c.attention:
            names += ["attn.W_a", "attn.W_c1", "attn.W_c2", "attn.b_out"]
            if c.attention == 1:
                names += ["attn.W_p", "attn.v_p"]
        return names + ["softmax.D", "softmax.b_d"]

    def _shape(self, name, flat):
        H = self.cfg.H
        if name == "softmax.D":
            return flat.reshape((self.cfg.V_tgt, H), order="F")
        if name.endswith(".W"):  # embedding table or its small gradient: E rows
            return flat.reshape((self.E, flat.size // self.E), order="F")
        if flat.size % H == 0 and flat.size > H and not name.endswith("b_d"):
            return flat.reshape((H, flat.size // H), order="F")
        return flat

    def grad(self, name):
        n = C.c_longlong(0)
        ptr = lib().orc_trainer_grad(self.trainer, name.encode(), C.byref(n))
        if not ptr:
            raise KeyError(name)
        flat = np.frombuffer((C.c_float * n.value).from_address(ptr), dtype=np.float32).copy()
        return self._shape(name, flat)

    def update_weights(self, learning_rate, clip_mode, norm_clip, individual_clip, minibatch_size):
        return float(lib().orc_update_weights(self.trainer, _f(learning_rate), clip_mode,
                                              _f(norm_clip), _f(individual_clip), minibatch_size))

    def get_perplexity(self, path, minibatch_size):
        """NeuralMachineTranslation::GetPerplexity (src/deep_rnn.h:1490-1568): one pass over an
        integerised file, 2^(-(sum of log2 p(target)) / target words of the file)."""
        f = TrainingFile(path, minibatch_size)
        p_data, more = 0.0, True
        while more:
            mb, more = f.read_minibatch()
            p_data += self.forward_xent(mb["src"], mb["tgt_in"], mb["tgt_out"], mb["batch_info"])
        p_data /= np.log(2.0)
        return float(2.0 ** (-p_data / f.total_target_words))

    def tuning(self, train_file, minibatch_size, learning_rate, epochs, dev_file=None, clip_mode=2,
               norm_clip=5.0, individual_clip=0.0, google_learning_rate=False,
               epoch_to_start_halving=6, stanford_learning_rate=False, epoch_to_start_halving_full=6,
               learning_rate_schedule=False, decrease_factor=0.5, margin=0.0):
        """Dispatcher::Tuning (src/dispatcher.cu:96-384), the part that decides what the model
        becomes: minibatches in file order, ComputeGradients + UpdateWeights per minibatch, the
        three learning-rate schedules (fixed halving from an epoch on at the half and the end of
        every epoch, :228-236 and :283-291; halving at the end of every epoch, :293-301; decrease by
        a factor when the dev perplexity stalls, evaluated at the half and the end of every epoch,
        :239-272 and :303-337).  Returns the list of events (kind, epoch, minibatch, value) with
        kinds learning_rate / half_epoch_perplexity / epoch_perplexity / epoch_end, and the final
        learning rate.  The learning rate is kept in single precision, as the reference's
        `precision tmp_learning_rate` is."""
        self._trainer()
        f = TrainingFile(train_file, minibatch_size)
        half_way_count = f.total_words // 2
        events = []
        lr = np.float32(learning_rate)
        epoch, batch_num, total_words = 1, 0, 0
        flag, old_perplexity, loglik = True, 0.0, 0.0

        def evaluate(kind):
            nonlocal lr, old_perplexity
            new = self.get_perplexity(dev_file, minibatch_size)
            events.append((kind, epoch, batch_num, new))
            if new + margin >= old_perplexity and epoch != 1:
                lr = np.float32(lr * np.float32(decrease_factor))
                events.append(("learning_rate", epoch, batch_num, float(lr)))
            old_perplexity = new

        def halve():
            nonlocal lr
            lr = np.float32(lr / np.float32(2))
            events.append(("learning_rate", epoch, batch_num, float(lr)))

        while epoch <= epochs:
            mb, success = f.read_minibatch()
            src, tin, tout = (np.asfortranarray(mb[k], np.int32) for k in ("src", "tgt_in", "tgt_out"))
            B, S = src.shape
            su, tu = i32(mb["src_wgrad"]), i32(mb["tgt_wgrad"])
            loglik += lib().orc_compute_gradients(self.trainer, _p(src), S, _p(tin), _p(tout), tin.shape[1],
                                                  B, _p(i32(mb["batch_info"])), _p(su), su.size, _p(tu),
                                                  tu.size)
            self.update_weights(float(lr), clip_mode, norm_clip, individual_clip, minibatch_size)
            batch_num += 1
            total_words += mb["words_in_minibatch"]
            if google_learning_rate and epoch >= epoch_to_start_halving and total_words >= half_way_count and flag:
                halve()
                flag = False
            if learning_rate_schedule and total_words >= half_way_count and flag:
                flag = False
                evaluate("half_epoch_perplexity")
            if not success:
                events.append(("epoch_end", epoch, batch_num, loglik))
                loglik = 0.0
                epoch += 1
                batch_num = 0
                if google_learning_rate and epoch >= epoch_to_start_halving:
                    halve()
                    flag = True
                if stanford_learning_rate and epoch >= epoch_to_start_halving_full:
                    halve()
                    flag = True
                if learning_rate_schedule:
                    evaluate("epoch_perplexity")
                    flag = True
                total_words = 0
        return events, float(lr)

    def get_param(self, name):
        flat = self.param(name).copy()
        return self._shape(name, flat)

    def __del__(self):
        try:
            if getattr(self, "trainer", None) is not None:
                lib().orc_trainer_destroy(self.trainer)
            lib().orc_model_destroy(self.handle)
        except Exception:
            pass
