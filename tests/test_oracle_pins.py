"""Pins the CPU oracle without the reference (which is CUDA-only and ships no test vectors):
every oracle function is checked against something independent of its own code -- brute force on
tiny inputs, closed forms, scipy/torch float64 library routines, or the float64 numpy model in
tests/ref_numpy.py."""
import numpy as np
import pytest
import scipy.special
import torch

from conftest import assert_close
import ref_numpy as R


def test_preprocess_indices_bruteforce(orc):
    idx = np.array([-1, 0, 5, -1, 7, 2, -1, -1, 3], np.int32)
    idx0, m, mf = orc.preprocess_indices(idx)
    assert idx0.tolist() == [0, 0, 5, 0, 7, 2, 0, 0, 3]
    assert m.tolist() == [0, 1, 1, 0, 1, 1, 0, 0, 1]
    assert mf.tolist() == [float(v) for v in m]
    rev = orc.setup_reverse_indices([9, 4, 6], 12)
    assert rev[9] == 0 and rev[4] == 1 and rev[6] == 2 and rev[0] == -7


def test_embed_lookup_and_dropout_closed_form(orc):
    rng = np.random.default_rng(1)
    W = rng.standard_normal((6, 11)).astype(np.float32)
    idx = np.array([3, 0, 10, 3], np.int32)
    out = orc.embed_lookup(W, idx)
    assert np.array_equal(out, W[:, idx])
    mask = rng.uniform(size=(6, 4)).astype(np.float32)
    keep = np.float32(0.8)
    out = orc.embed_lookup(W, idx, mask, keep)
    want = np.where(mask < keep, W[:, idx] * (np.float32(1) / keep), np.float32(0))
    assert_close(out, want, "inverted dropout", rtol=1e-6, atol=0)
    assert np.all(out[mask >= keep] == 0)


@pytest.mark.parametrize("tA,tX", [(False, False), (True, False), (False, True)])
def test_gemm_vs_float64(orc, tA, tX):
    rng = np.random.default_rng(2)
    M, N, K = 37, 13, 101
    A = rng.standard_normal((K, M) if tA else (M, K)).astype(np.float32)
    X = rng.standard_normal((N, K) if tX else (K, N)).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    got = orc.gemm(A, X, tA, tX, alpha=-1.0, beta=1.0, C0=C0)
    a64 = (A.T if tA else A).astype(np.float64)
    x64 = (X.T if tX else X).astype(np.float64)
    assert_close(got, -a64 @ x64 + C0, "gemm", rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("feed", [False, True])
def test_lstm_cell_vs_torch_lstmcell(orc, feed):
    """The stacked cell equals torch.nn.LSTMCell (float64) with W_ih=[M_i;M_f;M_c;M_o],
    W_hh=[W_hi;W_hf;W_hc;W_ho], bias_ih=b, bias_hh=0; mask01 = 0 forces h = c = 0."""
    rng = np.random.default_rng(3)
    H, B = 24, 7
    Wih = rng.uniform(-0.5, 0.5, (4 * H, H)).astype(np.float32)
    Whh = rng.uniform(-0.5, 0.5, (4 * H, H)).astype(np.float32)
    Q = rng.uniform(-0.5, 0.5, (4 * H, H)).astype(np.float32)
    b = rng.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
    x = rng.standard_normal((H, B)).astype(np.float32)
    h0 = rng.standard_normal((H, B)).astype(np.float32)
    c0 = rng.standard_normal((H, B)).astype(np.float32)
    ht = rng.standard_normal((H, B)).astype(np.float32)
    mask = np.array([1, 1, 0, 1, 0, 1, 1], np.int32)
    pre1, pre2 = orc.gemm(Wih, x), orc.gemm(Whh, h0)
    pre3 = orc.gemm(Q, ht) if feed else None
    gates, c, h = orc.lstm_cell_fwd(pre1, b, c0, mask, pre2, pre3, feed=feed)
    cell = torch.nn.LSTMCell(2 * H if feed else H, H, dtype=torch.float64)
    with torch.no_grad():
        wih = np.concatenate([Wih, Q], axis=1) if feed else Wih
        cell.weight_ih.copy_(torch.from_numpy(wih.astype(np.float64)))
        cell.weight_hh.copy_(torch.from_numpy(Whh.astype(np.float64)))
        cell.bias_ih.copy_(torch.from_numpy(b.astype(np.float64)))
        cell.bias_hh.zero_()
        xin = np.concatenate([x, ht], axis=0) if feed else x
        h1, c1 = cell(torch.from_numpy(xin.T.astype(np.float64)),
                      (torch.from_numpy(h0.T.astype(np.float64)),
                       torch.from_numpy(c0.T.astype(np.float64))))
    keep = mask.astype(bool)
    assert_close(h[:, keep], h1.numpy().T[:, keep], "h")
    assert_close(c[:, keep], c1.numpy().T[:, keep], "c")
    assert np.all(h[:, ~keep] == 0) and np.all(c[:, ~keep] == 0)
    # the stored gates are not masked
    s = pre1.astype(np.float64) + pre2 + (pre3 if feed else 0) + b[:, None]
    assert_close(gates[:H], R.sigmoid(s[:H]), "i")
    assert_close(gates[2 * H:3 * H], np.tanh(s[2 * H:3 * H]), "g")


def test_lstm_cell_clip(orc):
    H, B = 4, 2
    pre = np.full((4 * H, B), 5.0, np.float32)
    c0 = np.full((H, B), 40.0, np.float32)
    _, c, h = orc.lstm_cell_fwd(pre, np.zeros(4 * H, np.float32), c0, [1, 1], cell_clip=3.0)
    assert np.all(c == 3.0)
    assert_close(h, R.sigmoid(5.0) * np.tanh(3.0) * np.ones((H, B)), "h clipped")


def _attn_inputs(rng, H, B, S, lens, scale=1.0):
    hs = (rng.standard_normal((S, B, H)) * scale).astype(np.float32)  # [tau][col][H]
    tanh1 = np.tanh(rng.standard_normal((H, B))).astype(np.float32)
    v_p = rng.standard_normal(H).astype(np.float32)
    wa = (rng.standard_normal((H, B)) * 0.3).astype(np.float32)
    batch_info = np.concatenate([lens, S - np.asarray(lens)]).astype(np.int32)
    return hs, tanh1, v_p, wa, batch_info


def test_attention_window_bounds_bruteforce(orc):
    """indices must be exactly {lo..hi} & mask for lo=max(0,int(p)-D), hi=min(len-1,int(p)+D)."""
    rng = np.random.default_rng(4)
    H, S = 8, 9
    for D in (0, 1, 3, 10):
        lens = np.array([1, 2, 5, 9, 9, 7], np.int32)
        B = len(lens)
        mask = np.array([1, 1, 1, 1, 0, 1], np.int32)
        hs, tanh1, v_p, wa, bi = _attn_inputs(rng, H, B, S, lens)
        o = orc.attn_core_fwd(H, B, D, 0, S, tanh1, v_p, wa, hs, B * H, H, None, bi, mask)
        for b in range(B):
            sig = np.float32(1.0 / (1.0 + np.exp(-np.float64(np.float32(v_p @ tanh1[:, b])))))
            p = np.float32(lens[b]) * sig
            assert abs(o["p_t"][b] - p) <= 1e-5 * max(1.0, abs(p))
            pi = int(o["p_t"][b])
            want = [s for s in range(max(0, pi - D), min(lens[b] - 1, pi + D) + 1)]
            want = want if mask[b] == 1 else []
            got = [int(v) for v in o["indices"][b] if v != -1]
            assert got == want
            assert all(v == -1 for v in o["indices"][b][len(want):])


def test_attention_local_p_vs_float64(orc):
    """a_j / g_j is a softmax over the window's scores; ctx = sum_j a_j hs_j; hs of source position
    s of a reversed, left-padded sentence sits at encoder step len-1-s+off."""
    rng = np.random.default_rng(5)
    H, S, D = 16, 12, 2
    lens = np.array([12, 7, 3, 1, 12], np.int32)
    B = len(lens)
    mask = np.array([1, 1, 1, 1, 0], np.int32)
    hs, tanh1, v_p, wa, bi = _attn_inputs(rng, H, B, S, lens)
    o = orc.attn_core_fwd(H, B, D, 0, S, tanh1, v_p, wa, hs, B * H, H, None, bi, mask)
    for b in range(B):
        idx = o["indices"][b]
        valid = idx != -1
        if mask[b] == 0:
            assert not valid.any() and np.all(o["align"][b] == 0) and np.all(o["ctx"][:, b] == 0)
            continue
        pos = idx[valid]
        vecs = np.stack([hs[lens[b] - 1 - s + (S - lens[b]), b].astype(np.float64) for s in pos], 1)
        sc = wa[:, b].astype(np.float64) @ vecs
        soft = scipy.special.softmax(sc)
        g = np.exp(-((np.float64(o["p_t"][b]) - pos) ** 2) / (2 * (D * D / 4.0)))
        assert_close(o["align"][b][valid], soft * g, "alignment")
        assert_close(o["cached_exp"][:, b][valid], g, "gaussian")
        assert np.all(o["cached_exp"][:, b][~valid] == 1)
        assert_close((o["align"][b][valid] / o["cached_exp"][:, b][valid]).sum(), 1.0, "sum a/g")
        assert_close(o["ctx"][:, b], vecs @ (soft * g), "context")
        assert o["viterbi"][b] == pos[np.argmax(o["align"][b][valid])]


def test_attention_max_is_initialised_to_zero(orc):
    """All scores very negative: the reference subtracts max(0, .) = 0, so exp underflows to 0, the
    sum is 0 and the weights stay 0 (deep_rnn_kernel.h:1203,1230)."""
    rng = np.random.default_rng(6)
    H, S, D, B = 8, 6, 1, 2
    lens = np.array([6, 6], np.int32)
    hs, tanh1, v_p, wa, bi = _attn_inputs(rng, H, B, S, lens)
    hs[:] = 10.0
    wa[:] = -10.0  # score = -800 per slot
    o = orc.attn_core_fwd(H, B, D, 0, S, tanh1, v_p, wa, hs, B * H, H, None, bi, [1, 1])
    assert np.all(o["align"] == 0) and np.all(o["ctx"] == 0)


def test_attention_global_vs_float64_softmax(orc):
    rng = np.random.default_rng(7)
    H, S = 16, 10
    lens = np.array([10, 4, 1], np.int32)
    B = len(lens)
    hs, _, _, wa, bi = _attn_inputs(rng, H, B, S, lens)
    o = orc.attn_core_fwd(H, B, -1, S, S, None, None, wa, hs, B * H, H, None, bi, [1, 1, 1])
    for b in range(B):
        vecs = np.stack([hs[lens[b] - 1 - s + (S - lens[b]), b].astype(np.float64)
                         for s in range(lens[b])], 1)
        soft = scipy.special.softmax(wa[:, b].astype(np.float64) @ vecs)
        assert_close(o["align"][b][:lens[b]], soft, "global alignment")
        assert np.all(o["align"][b][lens[b]:] == 0)
        assert_close(o["ctx"][:, b], vecs @ soft, "global context")


def test_softmax_and_xent_vs_scipy(orc):
    rng = np.random.default_rng(8)
    V, B = 1003, 5
    z = (rng.standard_normal((V, B)) * 3).astype(np.float32)
    bias = rng.standard_normal(V).astype(np.float32)
    p = orc.softmax_fwd(z, bias)
    zz = (z + bias[:, None]).astype(np.float64)
    assert_close(p, scipy.special.softmax(zz, axis=0), "softmax")
    assert_close(p.sum(axis=0), np.ones(B), "columns sum to one", rtol=1e-5)
    assert_close(orc.softmax_fwd(z + np.float32(7.0), bias), p, "shift invariance")
    tgt = np.array([0, 5, 1002, 17, 3], np.int32)
    mask = np.array([1, 1, 0, 1, 1], np.int32)
    lp, loss = orc.logsoftmax_xent(z, bias, tgt, mask)
    want = scipy.special.log_softmax(zz, axis=0)[tgt, np.arange(B)]
    assert_close(lp, want, "log-softmax of target", rtol=1e-9, atol=1e-9)
    assert_close(loss, want[mask == 1].sum(), "masked loss", rtol=1e-12, atol=1e-9)
    ll = orc.train_loglik(p, tgt, mask)
    assert_close(ll, np.log(p[tgt, np.arange(B)].astype(np.float64))[mask == 1].sum(), "train ll",
                 rtol=1e-12, atol=1e-9)


def _bruteforce_expand(p, step, prev, diversity, penalty, beam):
    """Full sort instead of heaps (tie-free inputs)."""
    p = p.astype(np.float32)
    V = p.shape[0]
    norm = np.zeros(beam, np.float32)
    for v in range(V):
        norm += p[v]
    pn = p / norm
    cands = []
    for i in range(1 if step == 0 else beam):
        order = np.argsort(-pn[:, i], kind="stable")[: beam + 1]
        for rank, v in enumerate(order):
            s = np.float32(np.float32(np.log(pn[v, i])) + np.float32(prev[i])) - np.float32(
                np.float32(rank + 1) * np.float32(diversity))
            cands.append((s, i, int(v)))
    cands.sort(key=lambda t: -t[0])
    tok, bp, sc, fb, fs = [], [], [], [], []
    for s, i, v in cands:
        if len(tok) == beam:
            break
        if v == 0:
            continue
        if v == 1:
            fb.append(i)
            fs.append(s + np.float32(penalty))
        else:
            tok.append(v)
            bp.append(i)
            sc.append(s + np.float32(penalty))
    return tok, bp, sc, fb, fs


@pytest.mark.parametrize("step", [0, 3])
@pytest.mark.parametrize("diversity,penalty", [(0.0, 0.0), (0.3, 0.7)])
def test_beam_expand_vs_bruteforce(orc, step, diversity, penalty):
    rng = np.random.default_rng(9 + step)
    for trial in range(20):
        V, beam = 40, 4
        z = rng.standard_normal((V, beam)) * 2
        z[1, :] += rng.choice([0.0, 3.0], size=beam)  # make <EOF> competitive sometimes
        z[0, :] += rng.choice([0.0, 3.0], size=beam)  # and <START>
        p = scipy.special.softmax(z, axis=0).astype(np.float32)
        prev = (rng.standard_normal(beam) * 0.5).astype(np.float32)
        got = orc.beam_expand(p, step, prev, diversity, penalty)
        tok, bp, sc, fb, fs = _bruteforce_expand(p, step, prev, diversity, penalty, beam)
        if len(tok) < beam:
            continue  # candidates exhausted: undefined in the reference
        assert got["tok"].tolist() == tok and got["backptr"].tolist() == bp
        assert_close(got["score"], sc, "beam scores", rtol=1e-6, atol=1e-6)
        assert got["fin_beam"].tolist() == fb
        assert_close(got["fin_score"], fs, "finished scores", rtol=1e-6, atol=1e-6)
        assert 0 not in got["tok"] and 1 not in got["tok"]


def test_beam_step_margin_planted_gaps(orc):
    """orc_beam_step_margin on distributions whose gaps are planted: two columns with the same
    logits 0, -0.5, -0.9, -1.0, ... (beam 2, so three candidates per column) and previous scores
    0 and -0.3 give candidate scores c + {0, -0.3, -0.5, -0.8, -0.9, -1.2}; the two slots are filled
    by the first two, so the list is compared down to the third."""
    V, beam = 12, 2

    def dist(z_col):
        z = np.full((V, beam), -9.0)
        for b in range(beam):
            z[2:2 + len(z_col[b]), b] = z_col[b]
        return scipy.special.softmax(z, axis=0).astype(np.float32)

    prev = np.array([0.0, -0.3], np.float32)
    base = [0.0, -0.5, -0.9, -1.0]
    # the closest decision is rank 3 against rank 4 inside a column: 0.1
    assert abs(orc.beam_step_margin([dist([base, base])], 3, prev) - 0.1) < 1e-5
    # with the fourth entry far away the closest one is between list neighbours 2 and 3: 0.2
    far = [0.0, -0.5, -0.9, -4.0]
    assert abs(orc.beam_step_margin([dist([far, far])], 3, prev) - 0.2) < 1e-5
    # at step 0 only column 0 is expanded: neighbours 0 / -0.5 / -0.9 -> 0.4 (the third is compared
    # because it is the first candidate left without a slot)
    assert abs(orc.beam_step_margin([dist([far, far])], 0, prev) - 0.4) < 1e-5
    # <EOF> on top of column 0 takes no slot, so the walk goes one candidate further:
    # c + {0 (EOF), -0.3, -0.5, -0.8, ...}: gaps 0.3, 0.2, 0.3 -> still 0.2, but with the third
    # real candidate close to the fourth (-0.8 against -0.82) the margin drops to 0.02
    z = np.full((V, beam), -9.0)
    z[1, 0], z[2, 0], z[3, 0], z[4, 0] = 0.0, -0.5, -0.9, -4.0
    z[2, 1], z[3, 1], z[4, 1], z[5, 1] = 0.0, -0.52, -0.9, -4.0
    c0 = scipy.special.logsumexp(z[:, 0]) - scipy.special.logsumexp(z[:, 1])
    prev2 = np.array([0.0, -0.3 - c0], np.float32)  # makes both columns' constants equal
    p = scipy.special.softmax(z, axis=0).astype(np.float32)
    # list: EOF 0, col1 -0.3, col0 -0.5, col1 -0.82, col0 -0.9 ...; slots = -0.3 and -0.5; compared
    # down to -0.82: gaps 0.3, 0.2, 0.32 -> 0.2
    assert abs(orc.beam_step_margin([p], 3, prev2) - 0.2) < 1e-4
    # an exact tie between the last kept and the first dropped probability of a column
    tie = [0.0, -0.5, -0.9, -0.9]
    assert orc.beam_step_margin([dist([tie, far])], 3, prev) == 0.0
    # invariant on random inputs: never larger than the gap between two neighbouring slots
    rng = np.random.default_rng(77)
    for _ in range(20):
        zz = rng.standard_normal((40, 4)) * 2
        pp = scipy.special.softmax(zz, axis=0).astype(np.float32)
        pv = (rng.standard_normal(4) * 0.5).astype(np.float32)
        out = orc.beam_expand(pp, 2, pv)
        m = orc.beam_step_margin([pp], 2, pv)
        assert m >= 0 and m <= np.min(out["score"][:-1] - out["score"][1:]) + 1e-6


def test_decode_sentence_trace_matches_plain_decode(orc):
    """The traced decode is the plain decode plus a record: same 1-best; following the recorded
    back-pointers from the recorded tokens rebuilds a finished hypothesis of the plain decode."""
    rng = np.random.default_rng(78)
    P, m = _tiny_model(orc, rng)
    src = rng.integers(0, 30, size=7)
    plain = m.decode_sentence(src, beam=4)
    tr = m.decode_sentence_trace(src, beam=4)
    assert tr["best"].tolist() == plain["best"].tolist() and tr["best_score"] == plain["best_score"]
    n = tr["tok"].shape[0]
    assert n == plain["steps"] - 1 and tr["margin"].shape == (n,) and np.all(tr["margin"] >= 0)
    # path of beam entry 0 after the last expansion
    col, toks = 0, []
    for t in range(n - 1, -1, -1):
        toks.append(int(tr["tok"][t, col]))
        col = int(tr["backptr"][t, col])
    want = [0] + toks[::-1] + [1]
    assert any(h.tolist() == want for h, _ in plain["hyps"])


def test_decode_trace_window_margin_closed_form(orc):
    """The traced decode's window margin against a closed form: with v_p = 0 every window position
    is p_t = S * sigmoid(0) = S / 2, so the margin is 0 for an even source length and 0.5 for an odd
    one at every step; with real weights it lies in [0, 0.5] and differs between steps; a model
    without local-p attention reports 0.5."""
    rng = np.random.default_rng(79)
    P, m = _tiny_model(orc, rng)
    P0 = dict(P)
    P0["attn.v_p"] = np.zeros_like(P["attn.v_p"])
    m.set_params(P0)
    for S, want in ((6, 0.0), (7, 0.5)):
        tr = m.decode_sentence_trace(rng.integers(0, 30, size=S), beam=4)
        assert tr["window_margin"].shape == tr["margin"].shape
        assert np.all(tr["window_margin"] == want), (S, tr["window_margin"])
    m.set_params(P)
    tr = m.decode_sentence_trace(rng.integers(0, 30, size=9), beam=4)
    wm = tr["window_margin"]
    assert np.all((wm >= 0) & (wm <= 0.5)) and len(set(wm.tolist())) > 1
    g = orc.Model(2, 12, 30, 37, attention=2, D=0, feed_input=1, longest_sent=40)
    g.set_params(P)
    assert np.all(g.decode_sentence_trace(rng.integers(0, 30, size=5), beam=4)["window_margin"] == 0.5)


def test_beam_gather_composition(orc):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((5, 6)).astype(np.float32)
    p1 = np.array([3, 3, 0, 5, 1, 2], np.int32)
    p2 = np.array([5, 0, 0, 1, 4, 4], np.int32)
    assert np.array_equal(orc.beam_gather(x, p1), x[:, p1])
    assert np.array_equal(orc.beam_gather(orc.beam_gather(x, p1), p2), x[:, p1[p2]])


def _tiny_model(orc, rng, layers=2, H=12, Vs=30, Vt=37, D=2, scale=0.6):
    P = R.make_params(rng, layers, H, Vs, Vt, scale=scale)
    m = orc.Model(layers, H, Vs, Vt, attention=1, D=D, feed_input=1, longest_sent=40)
    m.set_params(P)
    return P, m


def test_decode_sentence_vs_numpy_beam_search(orc):
    """Whole-sentence beam decode of the oracle against the independent float64 numpy model:
    same 1-best tokens, same finished hypotheses, scores within fp32 tolerance."""
    rng = np.random.default_rng(11)
    checked = 0
    for trial in range(6):
        P, m = _tiny_model(orc, rng)
        S = int(rng.integers(3, 9))
        src = rng.integers(0, 30, size=S)
        margins = []
        best, best_s, hyps = R.beam_decode(P, 2, 12, 37, src, beam=3, D=2, longest=40,
                                           margins=margins)
        if min(margins) < 1e-4:
            continue  # a decision closer than fp32 resolves; not a parity case
        got = m.decode_sentence(src, beam=3)
        assert got["best"].tolist() == list(best)
        assert_close(got["best_score"], best_s, "rescored 1-best", rtol=1e-4, atol=1e-4)
        assert len(got["hyps"]) == len(hyps)
        for (gt, gs), (wt, ws) in zip(got["hyps"], hyps):
            assert gt.tolist() == list(wt)
            assert_close(gs, ws, "hypothesis score", rtol=1e-4, atol=1e-4)
        assert got["steps"] == min(int(np.float32(1.5) * S), 38) + 1
        checked += 1
    assert checked >= 3


def test_decode_sentence_with_exported_alignments_vs_numpy(orc):
    """The unk_replacement_mode__ variant: alignment scores exported per step, coverage penalty on
    them, Viterbi alignment per 1-best token -- against the numpy model, which carries the float64
    attention weights of every token and applies the definition of the penalty directly."""
    rng = np.random.default_rng(13)
    checked = differs = 0
    for trial in range(10):
        P, m = _tiny_model(orc, rng)
        S = int(rng.integers(3, 9))
        src = rng.integers(0, 30, size=S)
        margins = []
        best, best_s, hyps, vit = R.beam_decode(P, 2, 12, 37, src, beam=3, D=2, longest=40,
                                                margins=margins, alignments=True)
        if min(margins) < 1e-4:
            continue
        got = m.decode_sentence(src, beam=3, alignments=True)
        assert got["best"].tolist() == list(best)
        assert_close(got["best_score"], best_s, "rescored 1-best", rtol=1e-4, atol=1e-4)
        assert got["best_viterbi"].tolist() == vit
        assert all(-1 <= v < S for v in vit)
        plain = m.decode_sentence(src, beam=3)
        assert len(plain["hyps"]) == len(got["hyps"])  # the search itself does not change
        differs += int(abs(plain["best_score"] - got["best_score"]) > 1e-3)
        checked += 1
    assert checked >= 5 and differs >= 3  # the penalty really is computed from the scores


def test_beam_expand_ensemble_pins(orc):
    """EnsemblesModels in front of the expansion: n copies of one distribution expand exactly like
    the distribution alone; different distributions expand exactly like their float64 mean rounded
    to float32 (the averaging restated in numpy), and like the brute-force expansion of that mean."""
    rng = np.random.default_rng(41)
    V, beam = 53, 4
    for step in (0, 3):
        ps = []
        for _ in range(3):
            z = rng.normal(size=(V, beam)) * 2
            ps.append((np.exp(z) / np.exp(z).sum(axis=0)).astype(np.float32))
        prev = rng.uniform(-3, 0, size=beam).astype(np.float32)
        alone = orc.beam_expand(ps[0], step, prev, diversity=0.1, penalty=0.2)
        copies = orc.beam_expand_ensemble([ps[0]] * 3, step, prev, diversity=0.1, penalty=0.2)
        mixed = orc.beam_expand_ensemble(ps, step, prev, diversity=0.1, penalty=0.2)
        mean = (sum(p.astype(np.float64) for p in ps) / 3).astype(np.float32)
        of_mean = orc.beam_expand(mean, step, prev, diversity=0.1, penalty=0.2)
        for key in ("tok", "backptr", "score", "fin_beam", "fin_score"):
            assert np.array_equal(alone[key], copies[key]), key
            assert np.array_equal(mixed[key], of_mean[key]), key
        tok, bp, sc, fb, fs = _bruteforce_expand(mean, step, prev, 0.1, 0.2, beam)
        if len(tok) == beam:
            assert mixed["tok"].tolist() == tok and mixed["backptr"].tolist() == bp
            assert_close(mixed["score"], sc, "beam scores", rtol=1e-6, atol=1e-6)


def test_decode_sentence_ensemble_pins(orc):
    """Two copies of one model decode exactly like the model alone (tokens, hypotheses, scores,
    alignments); two different models decode like the numpy beam search over the mean of their
    distributions, with and without exported alignments."""
    rng = np.random.default_rng(43)
    checked = 0
    for trial in range(12):
        P1, m1 = _tiny_model(orc, rng)
        P2, m2 = _tiny_model(orc, rng)
        S = int(rng.integers(3, 9))
        src = rng.integers(0, 30, size=S)
        for al in (False, True):
            alone = m1.decode_sentence(src, beam=3, alignments=al)
            twice = m1.decode_sentence(src, beam=3, alignments=al, ensemble=(m1,))
            assert alone["best"].tolist() == twice["best"].tolist()
            assert len(alone["hyps"]) == len(twice["hyps"])
            for (at, as_), (tt, ts) in zip(alone["hyps"], twice["hyps"]):
                assert at.tolist() == tt.tolist() and as_ == ts
            if not al:
                assert alone["best_score"] == twice["best_score"]
            else:
                # the summed alignment scores are twice the model's own: same arg-max
                assert alone["best_viterbi"].tolist() == twice["best_viterbi"].tolist()
        margins = []
        best, best_s, hyps, vit = R.beam_decode(P1, 2, 12, 37, src, beam=3, D=2, longest=40,
                                                margins=margins, alignments=True, ensemble=[P2])
        if min(margins) < 1e-4:
            continue
        got = m1.decode_sentence(src, beam=3, alignments=True, ensemble=(m2,))
        assert got["best"].tolist() == list(best)
        assert_close(got["best_score"], best_s, "rescored 1-best", rtol=1e-4, atol=1e-4)
        assert got["best_viterbi"].tolist() == vit
        assert len(got["hyps"]) == len(hyps)
        for (gt, gs), (wt, ws) in zip(got["hyps"], hyps):
            assert gt.tolist() == list(wt)
            assert_close(gs, ws, "hypothesis score", rtol=1e-4, atol=1e-4)
        best0, s0, hyps0 = R.beam_decode(P1, 2, 12, 37, src, beam=3, D=2, longest=40, ensemble=[P2])
        got0 = m1.decode_sentence(src, beam=3, ensemble=(m2,))
        assert got0["best"].tolist() == list(best0)
        assert_close(got0["best_score"], s0, "rescored 1-best", rtol=1e-4, atol=1e-4)
        checked += 1
    assert checked >= 5


def test_forward_xent_vs_numpy(orc):
    """Teacher-forced forward + CE on a ragged minibatch (reversed, left-padded source; right-padded
    target; -1 padding) against the float64 numpy model run sentence by sentence."""
    rng = np.random.default_rng(12)
    layers, H, Vs, Vt, D = 2, 12, 30, 37, 2
    P, m = _tiny_model(orc, rng)
    lens_s, lens_t = [5, 3, 6], [4, 6, 2]
    B, S, T = 3, max(lens_s), max(lens_t)
    src = np.full((B, S), -1, np.int32)
    tin = np.full((B, T), -1, np.int32)
    tout = np.full((B, T), -1, np.int32)
    sents = []
    for b in range(B):
        s = rng.integers(0, Vs, size=lens_s[b])
        t = rng.integers(3, Vt, size=lens_t[b] - 1)
        sents.append((s, t))
        src[b, S - lens_s[b]:] = s[::-1]
        tin[b, :lens_t[b]] = np.concatenate([[0], t])
        tout[b, :lens_t[b]] = np.concatenate([t, [1]])
    bi = np.concatenate([lens_s, S - np.array(lens_s)]).astype(np.int32)
    got = m.forward_xent(src, tin, tout, bi)
    want = 0.0
    for b, (s, t) in enumerate(sents):
        he, ce, top = R.encode(P, layers, H, s)
        h, c = [x.copy() for x in he], [x.copy() for x in ce]
        h_tild = None
        for step, (wi, wo) in enumerate(zip(np.concatenate([[0], t]), np.concatenate([t, [1]]))):
            x = P["tgt.0.W"].astype(np.float64)[:, [wi]]
            for l in range(layers):
                ht = h_tild if (l == 0 and step != 0) else None
                h[l], c[l], _ = R.lstm_step(P, f"tgt.{l}.", x, h[l], c[l], ht)
                x = h[l]
            h_tild, _ = R.attention_local_p(P, x, lambda _b, pos: top[pos], [len(s)], [1], D)
            lp = R.log_softmax(P["softmax.D"].astype(np.float64) @ h_tild
                               + P["softmax.b_d"].astype(np.float64)[:, None])
            want += lp[wo, 0]
    assert_close(got, want, "sum log p(target)", rtol=1e-5, atol=1e-4)
