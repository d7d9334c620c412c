"""Pins for the training half of the CPU oracle (oracle/linmt_oracle_train.cpp).

The oracle restates the reference's backward pass from its sources; nothing in the reference holds
expected gradients.  What fixes it here is the method the reference itself uses for its gradient
check (src/layer_input_to_hidden.h:1016-1051): central differences of the forward pass -- taken on
an INDEPENDENT float64 numpy forward (tests/ref_numpy.py), so a dropped term, a transposed operand
or a wrong gate in the backward restatement fails.  The update is pinned by its closed form."""
import numpy as np
import pytest

import ref_numpy as R


def _sentences(rng, Vs, Vt, lens_s, lens_t):
    return [(rng.integers(0, Vs, size=a), rng.integers(3, Vt, size=b)) for a, b in zip(lens_s, lens_t)]


def _model(orc, rng, layers, H, Vs, Vt, attention, feed, D, scale=0.5, E=None):
    P = R.make_params(rng, layers, H, Vs, Vt, attention=bool(attention), feed_input=bool(feed),
                      scale=scale, E=E)
    m = orc.Model(layers, H, Vs, Vt, attention=attention, D=D, feed_input=feed, longest_sent=40,
                  E=E or 0)
    m.set_params(P)
    return P, m


CASES = [
    dict(layers=2, attention=1, feed=1, D=2, seed=21),
    dict(layers=1, attention=1, feed=0, D=1, seed=22),
    dict(layers=2, attention=0, feed=0, D=2, seed=23),
    dict(layers=3, attention=1, feed=1, D=3, seed=24),
    dict(layers=2, attention=2, feed=1, D=-1, seed=25),  # global attention: no window, no Gaussian
    # embedding size != LSTM size (a generalisation of the reference, which has E == H): a
    # narrower and a wider embedding
    dict(layers=2, attention=1, feed=1, D=2, seed=26, E=4),
    dict(layers=1, attention=2, feed=1, D=-1, seed=27, E=10),
]


@pytest.mark.parametrize("case", CASES,
                         ids=lambda c: f"L{c['layers']}a{c['attention']}f{c['feed']}E{c.get('E', 0)}")
def test_gradients_vs_central_differences(orc, case):
    rng = np.random.default_rng(case["seed"])
    layers, H, Vs, Vt, D = case["layers"], 7, 13, 11, case["D"]
    P, m = _model(orc, rng, layers, H, Vs, Vt, case["attention"], case["feed"], D, E=case.get("E"))
    sents = _sentences(rng, Vs, Vt, [5, 3, 7, 4], [4, 6, 2, 5])
    src, tin, tout, bi, su, tu = R.pack_minibatch(sents)
    ll, grads = m.compute_gradients(src, tin, tout, bi, su, tu)
    kw = dict(attention=bool(case["attention"]), feed_input=bool(case["feed"]))
    P64 = {k: v.astype(np.float64) for k, v in P.items()}
    want_ll = R.minibatch_loglik(P64, layers, H, D, sents, **kw)
    assert abs(ll - want_ll) < 1e-4 * max(1.0, abs(want_ll))

    def dense(name, g):
        # embedding gradients come back per unique id
        if name in ("src.0.W", "tgt.0.W"):
            full = np.zeros_like(P64[name])
            full[:, su if name == "src.0.W" else tu] = g
            return full
        return g.reshape(P64[name].shape, order="F") if g.ndim == 1 and P64[name].ndim == 1 else g

    eps = 1e-5
    checked = 0
    for name in m.param_names():
        g = dense(name, grads[name]).astype(np.float64)
        assert g.shape == P64[name].shape, name
        for _ in range(2):
            direction = rng.standard_normal(P64[name].shape)
            Pp, Pm = dict(P64), dict(P64)
            Pp[name] = P64[name] + eps * direction
            Pm[name] = P64[name] - eps * direction
            fd = (R.minibatch_loglik(Pp, layers, H, D, sents, **kw)
                  - R.minibatch_loglik(Pm, layers, H, D, sents, **kw)) / (2 * eps)
            got = float(np.sum(g * direction))
            scale = float(np.sqrt(np.sum(g * g) * np.sum(direction * direction)))
            assert abs(got - fd) <= 2e-3 * scale + 1e-5, (name, got, fd, scale)
            checked += 1
    assert checked == 2 * len(m.param_names())


@pytest.mark.parametrize("attention,E", [(1, None), (0, None), (1, 5)])
def test_gradients_with_dropout_vs_central_differences(orc, attention, E):
    """Same check with dropout masks: embeddings, every layer's upward output, the attention /
    softmax input.  keep = 0.6 so that many elements are dropped.  The last case has an embedding
    narrower than the LSTM (embedding masks of E rows)."""
    rng = np.random.default_rng(27 + attention + (E or 0))
    layers, H, Vs, Vt, D, keep = 2, 7, 13, 11, 2, 0.6
    P, m = _model(orc, rng, layers, H, Vs, Vt, attention, attention, D, E=E)
    sents = _sentences(rng, Vs, Vt, [5, 3, 7, 4], [4, 6, 2, 5])
    src, tin, tout, bi, su, tu = R.pack_minibatch(sents)
    B, S, T = len(sents), src.shape[1], tin.shape[1]
    drop = dict(keep=keep, src_embed=rng.random((S, B, E or H)).astype(np.float32),
                tgt_embed=rng.random((T, B, E or H)).astype(np.float32),
                src_out=rng.random((layers, S, B, H)).astype(np.float32),
                tgt_out=rng.random((layers, T, B, H)).astype(np.float32))
    m.set_dropout(keep, B, drop["src_embed"], drop["tgt_embed"], drop["src_out"], drop["tgt_out"])
    ll, grads = m.compute_gradients(src, tin, tout, bi, su, tu)
    kw = dict(attention=bool(attention), feed_input=bool(attention), drop=drop)
    P64 = {k: v.astype(np.float64) for k, v in P.items()}
    want_ll = R.minibatch_loglik(P64, layers, H, D, sents, **kw)
    assert abs(ll - want_ll) < 1e-4 * max(1.0, abs(want_ll))
    # dropout changes the result (the masks are really applied)
    assert abs(want_ll - R.minibatch_loglik(P64, layers, H, D, sents, attention=bool(attention),
                                            feed_input=bool(attention))) > 1e-3
    eps = 1e-5
    for name in m.param_names():
        g = grads[name].astype(np.float64)
        if name in ("src.0.W", "tgt.0.W"):
            full = np.zeros_like(P64[name])
            full[:, su if name == "src.0.W" else tu] = g
            g = full
        direction = rng.standard_normal(P64[name].shape)
        Pp, Pm = dict(P64), dict(P64)
        Pp[name] = P64[name] + eps * direction
        Pm[name] = P64[name] - eps * direction
        fd = (R.minibatch_loglik(Pp, layers, H, D, sents, **kw)
              - R.minibatch_loglik(Pm, layers, H, D, sents, **kw)) / (2 * eps)
        got = float(np.sum(g * direction))
        scale = float(np.sqrt(np.sum(g * g) * np.sum(direction * direction)))
        assert abs(got - fd) <= 2e-3 * scale + 1e-5, (name, got, fd, scale)
    m.set_dropout(0.0)


def test_embedding_rows_outside_the_minibatch_get_no_gradient(orc):
    """Dense view of the scatter: ids that do not occur have zero finite-difference gradient, and an
    id occurring several times gets the sum (compare with a per-occurrence float64 accumulation)."""
    rng = np.random.default_rng(31)
    layers, H, Vs, Vt, D = 1, 6, 9, 10, 1
    P, m = _model(orc, rng, layers, H, Vs, Vt, 1, 1, D)
    sents = [(np.array([4, 4, 2, 4]), np.array([5, 5, 5])), (np.array([2, 4]), np.array([5, 7]))]
    src, tin, tout, bi, su, tu = R.pack_minibatch(sents)
    assert su.tolist() == [4, 2] and tu.tolist() == [0, 5, 7]
    _, grads = m.compute_gradients(src, tin, tout, bi, su, tu)
    P64 = {k: v.astype(np.float64) for k, v in P.items()}
    eps = 1e-5
    for name, uniq, V in (("src.0.W", su, Vs), ("tgt.0.W", tu, Vt)):
        for k, vid in enumerate(uniq):
            for r in (0, H - 1):
                Pp, Pm = dict(P64), dict(P64)
                Pp[name] = P64[name].copy()
                Pm[name] = P64[name].copy()
                Pp[name][r, vid] += eps
                Pm[name][r, vid] -= eps
                fd = (R.minibatch_loglik(Pp, layers, H, D, sents)
                      - R.minibatch_loglik(Pm, layers, H, D, sents)) / (2 * eps)
                assert abs(grads[name][r, k] - fd) <= 2e-3 * max(1.0, abs(fd)), (name, vid, r)


def test_error_clip_pins(orc):
    """The --clip-cell clamps of the backward pass.  (i) Thresholds that never bind give the bits of
    the unclamped run.  (ii) With a binding threshold, a two-layer model without attention is a
    plain grid of LSTM cells through source and target, and its gradients must equal textbook
    backpropagation through time written here in float64 with the error to step t-1 and the error
    to the layer below clamped where the reference clamps them (src/node_input_to_hidden.h:876-878,
    src/node_hidden_to_hidden.h:774-776, 877-879; the error to the embedding is not clamped)."""
    rng = np.random.default_rng(71)
    L, H, Vs, Vt = 2, 6, 9, 10
    P, m = _model(orc, rng, L, H, Vs, Vt, 0, 0, 1, scale=0.9)
    sents = [(np.array([4, 2, 7, 1]), np.array([5, 3, 6]))]
    src, tin, tout, bi, su, tu = R.pack_minibatch(sents)
    _, base = m.compute_gradients(src, tin, tout, bi, su, tu)
    m.set_clip(1000.0, 1000.0)
    _, loose = m.compute_gradients(src, tin, tout, bi, su, tu)
    for k in base:
        assert np.array_equal(base[k], loose[k]), k
    clip = 0.02
    m.set_clip(0.0, clip)
    _, got = m.compute_gradients(src, tin, tout, bi, su, tu)
    m.set_clip(0.0, 0.0)
    assert not np.allclose(got["src.0.W_hi"], base["src.0.W_hi"], rtol=1e-3, atol=1e-7)

    # textbook BPTT, float64
    P64 = {k: v.astype(np.float64) for k, v in P.items()}
    s_ids, t_ids = sents[0]
    steps = [("src", int(w)) for w in s_ids[::-1]] + [("tgt", int(w)) for w in np.concatenate([[0], t_ids])]
    outs = [None] * len(s_ids) + [int(w) for w in np.concatenate([t_ids, [1]])]
    h = [np.zeros((H, 1)) for _ in range(L)]
    c = [np.zeros((H, 1)) for _ in range(L)]
    tape = []
    for side, w in steps:
        x = P64[f"{side}.0.W"][:, [w]]
        row = []
        for l in range(L):
            h_new, c_new, (i, f, g, o) = R.lstm_step(P64, f"{side}.{l}.", x, h[l], c[l])
            row.append(dict(x=x, h_prev=h[l], c_prev=c[l], i=i, f=f, g=g, o=o, c=c_new, h=h_new))
            h[l], c[l] = h_new, c_new
            x = h_new
        tape.append(row)
    want = {k: np.zeros_like(v) for k, v in P64.items()}
    dh_next = [np.zeros((H, 1)) for _ in range(L)]
    dc_next = [np.zeros((H, 1)) for _ in range(L)]
    for n in range(len(steps) - 1, -1, -1):
        side, w = steps[n]
        dh_above = np.zeros((H, 1))
        if outs[n] is not None:
            top = tape[n][L - 1]["h"]
            p = np.exp(R.log_softmax(P64["softmax.D"] @ top + P64["softmax.b_d"][:, None]))
            dz = -p
            dz[outs[n], 0] += 1.0
            want["softmax.D"] += dz @ top.T
            want["softmax.b_d"] += dz[:, 0]
            dh_above = P64["softmax.D"].T @ dz
        for l in range(L - 1, -1, -1):
            tp, pfx = tape[n][l], f"{side}.{l}."
            dh = dh_next[l] + dh_above
            tc = np.tanh(tp["c"])
            dc = dc_next[l] + dh * tp["o"] * (1 - tc * tc)
            d = dict(o=dh * tc * tp["o"] * (1 - tp["o"]), f=dc * tp["c_prev"] * tp["f"] * (1 - tp["f"]),
                     i=dc * tp["g"] * tp["i"] * (1 - tp["i"]), c=dc * tp["i"] * (1 - tp["g"] ** 2))
            dh_prev, dx = np.zeros((H, 1)), np.zeros((H, 1))
            for gname in R.GATES:
                want[pfx + "W_h" + gname] += d[gname] @ tp["h_prev"].T
                want[pfx + "M_" + gname] += d[gname] @ tp["x"].T
                want[pfx + "b_" + gname] += d[gname][:, 0]
                dh_prev += P64[pfx + "W_h" + gname].T @ d[gname]
                dx += P64[pfx + "M_" + gname].T @ d[gname]
            dh_next[l] = np.clip(dh_prev, -clip, clip)       # the clamps under test
            dc_next[l] = dc * tp["f"]
            if l == 0:
                want[pfx + "W"][:, [w]] += dx                 # the embedding's error: not clamped
            else:
                dh_above = np.clip(dx, -clip, clip)
    for name in m.param_names():
        g = got[name].astype(np.float64)
        if name in ("src.0.W", "tgt.0.W"):
            full = np.zeros_like(P64[name])
            full[:, su if name == "src.0.W" else tu] = g
            g = full
        np.testing.assert_allclose(g.reshape(want[name].shape, order="F"), want[name], rtol=2e-4,
                                   atol=2e-6, err_msg=name)


def test_explicit_embedding_size_equal_to_lstm_size_changes_nothing(orc):
    """E == H reduction of the embedding-size generalisation: a model created with E = H gives the
    bits of a model created the reference's way (E = 0): log-likelihood, every gradient, the
    update, a beam decode and the scoring pass."""
    layers, H, Vs, Vt, D = 2, 8, 13, 30, 2
    outs = []
    for E in (None, H):
        rng = np.random.default_rng(61)
        P, m = _model(orc, rng, layers, H, Vs, Vt, 1, 1, D, E=E)
        sents = _sentences(rng, Vs, Vt, [5, 3, 7, 4], [4, 6, 2, 5])
        src, tin, tout, bi, su, tu = R.pack_minibatch(sents)
        xent = m.forward_xent(src, tin, tout, bi)
        dec = m.decode_sentence(sents[2][0], beam=3)
        ll, grads = m.compute_gradients(src, tin, tout, bi, su, tu)
        norm = m.update_weights(0.3, 2, 0.01, 0.0, len(sents))
        outs.append((xent, dec["best"].tolist(), dec["best_score"], ll, grads, norm,
                     {k: m.get_param(k) for k in m.param_names()}))
    a, b = outs
    assert a[0] == b[0] and a[1] == b[1] and a[2] == b[2] and a[3] == b[3] and a[5] == b[5]
    for k in a[4]:
        assert np.array_equal(a[4][k], b[4][k]), k
        assert np.array_equal(a[6][k], b[6][k]), k


def test_forward_with_other_embedding_size_vs_numpy(orc):
    """Scoring pass and beam decode at E != H against the independent numpy model."""
    rng = np.random.default_rng(62)
    layers, H, E, Vs, Vt, D = 2, 8, 5, 13, 30, 2
    P, m = _model(orc, rng, layers, H, Vs, Vt, 1, 1, D, E=E)
    sents = _sentences(rng, Vs, Vt, [5, 3, 7, 4], [4, 6, 2, 5])
    src, tin, tout, bi, su, tu = R.pack_minibatch(sents)
    P64 = {k: v.astype(np.float64) for k, v in P.items()}
    want = R.minibatch_loglik(P64, layers, H, D, sents)
    assert abs(m.forward_xent(src, tin, tout, bi) - want) < 1e-4 * max(1.0, abs(want))
    margins = []
    best, score, _ = R.beam_decode(P, layers, H, Vt, sents[0][0], 3, D, margins=margins, longest=40)
    assert min(margins) > 1e-4  # no decision closer than fp32 resolves
    got = m.decode_sentence(sents[0][0], beam=3)
    assert got["best"].tolist() == list(best)
    assert abs(got["best_score"] - score) <= 1e-4 * max(1.0, abs(score))


@pytest.mark.parametrize("mode,E", [(0, None), (1, None), (2, None), (3, None), (2, 4)])
def test_update_closed_form(orc, mode, E):
    rng = np.random.default_rng(41 + mode)
    layers, H, Vs, Vt, D = 2, 6, 9, 10, 1
    P, m = _model(orc, rng, layers, H, Vs, Vt, 1, 1, D, scale=0.8, E=E)
    sents = _sentences(rng, Vs, Vt, [5, 3, 4], [4, 3, 5])
    src, tin, tout, bi, su, tu = R.pack_minibatch(sents)
    _, grads = m.compute_gradients(src, tin, tout, bi, su, tu)
    B, lr = len(sents), 0.7
    g = {k: v.astype(np.float64) / B for k, v in grads.items()}
    dense_names = [k for k in g if k not in ("src.0.W", "tgt.0.W")]
    total = np.sqrt(sum(np.sum(g[k] ** 2) for k in dense_names))
    # thresholds chosen so that the clip is active
    norm_clip = 0.5 * total if mode == 2 else 0.5 * min(np.sqrt(np.sum(g[k] ** 2)) for k in dense_names
                                                         if np.sum(g[k] ** 2) > 0) * 3
    ind = 0.25 * max(np.abs(v).max() for v in g.values())
    if mode == 2:
        g = {k: v * (norm_clip / total) for k, v in g.items()}  # embeddings rescaled too
    elif mode == 1:
        for k in g:
            n = np.sqrt(np.sum(g[k] ** 2))
            if n > norm_clip:
                g[k] = g[k] * (norm_clip / n)
    elif mode == 3:
        g = {k: np.clip(v, -ind, ind) for k, v in g.items()}
    want = {}
    for k in g:
        want[k] = P[k].astype(np.float64).copy()
        if k == "src.0.W":
            want[k][:, su] += lr * g[k]
        elif k == "tgt.0.W":
            want[k][:, tu] += lr * g[k]
        else:
            want[k] += lr * g[k].reshape(want[k].shape, order="F")
    got_norm = m.update_weights(lr, mode, norm_clip, ind, B)
    if mode == 2:
        assert abs(got_norm - total) <= 1e-5 * total
    for k in g:
        np.testing.assert_allclose(m.get_param(k).reshape(want[k].shape, order="F"), want[k],
                                   rtol=2e-5, atol=2e-6, err_msg=k)
    # gradients are cleared by the update
    for k in g:
        assert not np.any(m.grad(k)), k


@pytest.mark.parametrize("modes", [(0, 0, 0, 1, 1, 1), (1, 1, 1, 0, 1, 0), (1, 0, 1, 1, 0, 1)],
                         ids=["finetune", "source_rnn_and_attention_frozen", "target_side_frozen"])
def test_frozen_groups_closed_form(orc, modes):
    """The train_*_mode__ switches of UpdateParams (src/layer_input_to_hidden.h:1154,1257,1263,
    src/layer_hidden_to_hidden.h:765,831, src/layer_loss.h:1144): a frozen group keeps its bits,
    every other parameter gets exactly the update it gets with nothing frozen (the global norm is
    taken over all gradients either way, CalculateGlobalNorm has no switch), and every gradient
    is cleared."""
    rng = np.random.default_rng(51)
    layers, H, Vs, Vt, D = 2, 6, 9, 10, 1
    P, a = _model(orc, rng, layers, H, Vs, Vt, 1, 1, D, scale=0.8)
    _, b = _model(orc, np.random.default_rng(51), layers, H, Vs, Vt, 1, 1, D, scale=0.8)
    sents = _sentences(rng, Vs, Vt, [5, 3, 4], [4, 3, 5])
    src, tin, tout, bi, su, tu = R.pack_minibatch(sents)
    a.compute_gradients(src, tin, tout, bi, su, tu)
    _, grads = b.compute_gradients(src, tin, tout, bi, su, tu)
    B, lr = len(sents), 0.7
    total = np.sqrt(sum(np.sum((v.astype(np.float64) / B) ** 2) for k, v in grads.items()
                        if k not in ("src.0.W", "tgt.0.W")))
    norm_clip = 0.5 * total
    b.set_train_modes(*modes)
    norm_all = a.update_weights(lr, 2, norm_clip, 0.0, B)
    norm_frozen = b.update_weights(lr, 2, norm_clip, 0.0, B)
    assert norm_all == norm_frozen and abs(norm_all - total) <= 1e-5 * total

    def group(name):
        if name == "src.0.W":
            return 0
        if name == "tgt.0.W":
            return 1
        return {"softmax": 2, "src": 3, "tgt": 4, "attn": 5}[name.split(".")[0]]

    seen = set()
    for name in a.param_names():
        g = group(name)
        seen.add(g)
        if modes[g]:
            assert np.array_equal(b.get_param(name), a.get_param(name)), name
            assert not np.array_equal(b.get_param(name).reshape(P[name].shape), P[name]), name
        else:
            assert np.array_equal(b.get_param(name).reshape(P[name].shape), P[name]), name
        assert not np.any(b.grad(name)), name
    assert seen == set(range(6))
