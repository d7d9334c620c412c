"""The benchmark configurations at their own width, depth and vocabulary, GPU against the CPU oracle:

* the 4+4-layer, 1000-hidden, 30k-vocabulary encoder-decoder scoring a full minibatch of 128
  sentence pairs of 10-50 tokens (teacher-forced forward + cross-entropy), with local-p and with
  global attention -- NeuralMachineTranslation::GetError, src/deep_rnn.h:2173-2317,
  SoftmaxLayer::ComputeLossGpu, src/layer_loss.h:673-750;
* the 8+8-layer, 2048-hidden, 1024-embedding, 50k-vocabulary training step (forward with dropout
  masks, backward, global-norm clip at 5, SGD update) on a small full minibatch, so that the oracle
  finishes in about a minute -- NeuralMachineTranslation::ComputeGradients / UpdateWeights,
  src/deep_rnn.h:984-1412.

At these widths the products run on other tile configurations, K splits and fused epilogues than
in the small model tests.  Weights are uniform[-0.08, 0.08] with forget-gate bias 1, ids Zipf(1.1)."""
import time

import numpy as np
import pytest

from conftest import assert_close

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]


@pytest.fixture(scope="module")
def host():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from linmt_amd import host as h
    h.load()
    return h


def zipf_ids(rng, n, V, s=1.1, lo=0):
    ranks = np.arange(1, V - lo + 1, dtype=np.float64)
    p = ranks ** (-s)
    p /= p.sum()
    return (rng.choice(V - lo, size=n, p=p) + lo).astype(np.int32)


def make_params(rng, layers, H, Vs, Vt, E=None, scale=0.08):
    """Reference initialisation; arrays come back column-major (what both models store), so
    handing them over copies without a transposition."""
    E = H if E is None else E
    P = {}

    def u(rows, cols=None):
        if cols is None:
            return (rng.random(size=rows, dtype=np.float32) * 2 - 1) * np.float32(scale)
        return ((rng.random(size=(cols, rows), dtype=np.float32) * 2 - 1) * np.float32(scale)).T

    for side, V in (("src", Vs), ("tgt", Vt)):
        for l in range(layers):
            pfx = f"{side}.{l}."
            for g in "ifco":
                P[pfx + "W_h" + g] = u(H, H)
                P[pfx + "M_" + g] = u(H, E if l == 0 else H)
                P[pfx + "b_" + g] = u(H)
                if side == "tgt" and l == 0:
                    P[pfx + "Q_" + g] = u(H, H)
            P[pfx + "b_f"] = np.ones(H, np.float32)
            if l == 0:
                P[pfx + "W"] = u(E, V)
    for n in ("W_a", "W_p", "W_c1", "W_c2"):
        P["attn." + n] = u(H, H)
    P["attn.v_p"] = u(H)
    P["attn.b_out"] = u(H)
    P["softmax.D"] = u(Vt, H)
    P["softmax.b_d"] = u(Vt)
    return P


def minibatch(rng, B, lo, hi, Vs, Vt):
    ls = rng.integers(lo, hi + 1, size=B)
    lt = rng.integers(lo, hi + 1, size=B)
    ls[0], lt[0] = hi, hi
    S, T = int(ls.max()), int(lt.max())
    src = np.full((B, S), -1, np.int32)
    tin = np.full((B, T), -1, np.int32)
    tout = np.full((B, T), -1, np.int32)
    for b in range(B):
        src[b, S - ls[b]:] = zipf_ids(rng, ls[b], Vs)
        t = zipf_ids(rng, lt[b] - 1, Vt, lo=3)
        tin[b, :lt[b]] = np.concatenate([[0], t])
        tout[b, :lt[b]] = np.concatenate([t, [1]])
    bi = np.concatenate([ls, S - ls]).astype(np.int32)

    def uniq(a):
        _, first = np.unique(a.ravel(order="F"), return_index=True)
        ids = a.ravel(order="F")[np.sort(first)]
        return ids[ids != -1].astype(np.int32)

    return src, tin, tout, bi, uniq(src), uniq(tin), int(lt.sum())


@pytest.mark.parametrize("attention", [1, 2], ids=["local-p", "global"])
def test_config2_teacher_forced_cross_entropy_at_size(orc, host, attention):
    layers, H, V, B, D = 4, 1000, 30000, 128, 10
    rng = np.random.default_rng(1100 + attention)
    P = make_params(rng, layers, H, V, V)
    src, tin, tout, bi, _, _, n_words = minibatch(rng, B, 10, 50, V, V)
    S = src.shape[1]
    gm = host.Model(layers, H, V, V, longest_sentence=54, attention_mode=attention,
                    attention_width=D, feed_input=True, minibatch_size=B)
    gm.set_params(P)
    got = gm.get_error(src, tin, tout, bi)
    # padded source prefixes keep their state at exactly zero on every layer
    for layer in (0, layers - 1):
        for b in (1, B // 2, B - 1):
            pad = S - bi[b]
            if pad > 0:
                for kind in (0, 1):
                    st = gm.get_state(kind, 0, layer, pad - 1, H, B)
                    assert np.all(st[:, b] == 0), (layer, b, kind)
    h_gpu = gm.get_state(0, 0, layers - 1, S - 1, H, B)  # top encoder state after the last word
    gm.close()
    om = orc.Model(layers, H, V, V, attention=attention, D=D, feed_input=1, longest_sent=54)
    om.set_params(P)
    t0 = time.time()
    want = om.forward_xent(src, tin, tout, bi)
    print(f"oracle forward_xent: {time.time() - t0:.1f} s, {n_words} target words, "
          f"per-word log-lik gpu {got / n_words:.6f} oracle {want / n_words:.6f}", flush=True)
    assert np.isfinite(h_gpu).all() and np.abs(h_gpu).max() > 1e-3
    assert_close(got / n_words, want / n_words, "per-word log-likelihood", rtol=1e-4, atol=1e-5)
    assert_close(got, want, "sum log p(target)", rtol=2e-5, atol=1e-3)


def _scaled_close(got, want, what, rel=1e-4, abs_of_max=5e-5):
    """fp32 gradients of a deep, wide model.  An element is a sum of terms of the size of the
    tensor's largest entries, built from hidden states that are themselves only fixed to 1e-5
    (rounding order differs between the GPU's and the CPU's products), so the absolute part of the
    tolerance scales with the largest entry: |err| <= rel |want| + abs_of_max max|want|.  On top
    of that the whole tensor must agree to 1e-4 in the Frobenius norm, which no systematic
    difference (a dropped term, a wrong mask) survives."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, what
    top = float(np.abs(want).max()) if want.size else 0.0
    err = np.abs(got - want)
    lim = rel * np.abs(want) + abs_of_max * top + 1e-9
    if not np.all(err <= lim):
        i = np.unravel_index(np.argmax(err - lim), err.shape)
        raise AssertionError(f"{what}: at {i} got {got[i]!r} want {want[i]!r} (max |want| {top:.3e}); "
                             f"{int(np.sum(err > lim))} of {err.size} out of tolerance")
    nrm = float(np.sqrt(np.sum(want ** 2)))
    fro = float(np.sqrt(np.sum(err ** 2))) / nrm if nrm > 0 else 0.0
    assert fro <= 1e-4, f"{what}: relative Frobenius error {fro:.3e}"
    return fro, (float(err.max()) / top if top > 0 else 0.0)


def test_config5_training_step_at_width(orc, host):
    layers, H, E, V, D, keep, B = 8, 2048, 1024, 50000, 10, 0.8, 8
    rng = np.random.default_rng(1200)
    P = make_params(rng, layers, H, V, V, E=E)
    src, tin, tout, bi, su, tu, n_words = minibatch(rng, B, 4, 12, V, V)
    S, T = src.shape[1], tin.shape[1]
    lr, clip = 0.1, 5.0
    gm = host.Model(layers, H, V, V, longest_sentence=16, attention_mode=1, attention_width=D,
                    feed_input=True, minibatch_size=B, embedding_size=E,
                    training=dict(learning_rate=lr, grad_clip_mode=2, norm_clip=clip,
                                  dropout_keep=keep, dropout_seed=99))
    gm.set_params(P)
    om = orc.Model(layers, H, V, V, attention=1, D=D, feed_input=1, longest_sent=16, E=E)
    om.set_params(P)
    names = om.param_names()

    # scoring pass (no dropout) on the training model
    got_x, want_x = gm.get_error(src, tin, tout, bi), om.forward_xent(src, tin, tout, bi)
    assert_close(got_x / n_words, want_x / n_words, "GetError per word", rtol=1e-4, atol=1e-5)

    got_ll = gm.compute_gradients(src, tin, tout, bi, su, tu)
    se = gm.get_dropout_mask(0, 0, 0, E, B, S)
    te = gm.get_dropout_mask(0, 1, 0, E, B, T)
    so = np.stack([gm.get_dropout_mask(1, 0, l, H, B, S) if l < layers - 1
                   else np.ones((S, B, H), np.float32) for l in range(layers)])
    to = np.stack([gm.get_dropout_mask(1, 1, l, H, B, T) for l in range(layers)])
    assert abs((te < keep).mean() - keep) < 0.02
    om.set_dropout(keep, B, se, te, so, to)
    t0 = time.time()
    want_ll, want = om.compute_gradients(src, tin, tout, bi, su, tu)
    print(f"oracle compute_gradients: {time.time() - t0:.1f} s; log-lik per word gpu "
          f"{got_ll / n_words:.6f} oracle {want_ll / n_words:.6f}", flush=True)
    assert_close(got_ll / n_words, want_ll / n_words, "log-likelihood per word", rtol=1e-4, atol=1e-5)
    worst_fro, worst_el = (0.0, ""), (0.0, "")
    for name in names:
        w = np.asarray(want[name])
        shape = w.shape if w.ndim == 2 else (w.size,)
        fro, el = _scaled_close(gm.get_grad(name, shape), w.reshape(shape, order="F"),
                                f"gradient of {name}")
        worst_fro, worst_el = max(worst_fro, (fro, name)), max(worst_el, (el, name))
    print(f"gradients: largest relative Frobenius error {worst_fro[0]:.2e} ({worst_fro[1]}), largest "
          f"element error / max entry {worst_el[0]:.2e} ({worst_el[1]})", flush=True)

    # the same minibatch on a second model whose matrix products are split bf16 products (size
    # thresholds off: every product that goes through Gemm()); same seed, hence the same masks
    gs = host.Model(layers, H, V, V, longest_sentence=16, attention_mode=1, attention_width=D,
                    feed_input=True, minibatch_size=B, embedding_size=E,
                    training=dict(learning_rate=lr, grad_clip_mode=2, norm_clip=clip,
                                  dropout_keep=keep, dropout_seed=99))
    gs.set_params(P)
    gs.set_split_products(True, 1)
    split_ll = gs.compute_gradients(src, tin, tout, bi, su, tu)
    assert np.array_equal(gs.get_dropout_mask(0, 1, 0, E, B, T), te)
    assert_close(split_ll / n_words, want_ll / n_words, "log-likelihood per word, split products",
                 rtol=1e-4, atol=1e-5)
    worst = (0.0, "")
    for name in names:
        w = np.asarray(want[name])
        shape = w.shape if w.ndim == 2 else (w.size,)
        fro, _ = _scaled_close(gs.get_grad(name, shape), w.reshape(shape, order="F"),
                               f"gradient of {name}, split products")
        worst = max(worst, (fro, name))
    print(f"gradients with split products: largest relative Frobenius error {worst[0]:.2e} ({worst[1]})",
          flush=True)
    gs.close()
    del want

    # UpdateWeights, global-norm clip (embedding gradients outside the norm, inside the rescale)
    want_norm = om.update_weights(lr, 2, clip, 0.0, B)
    got_norm = gm.update_weights()
    print(f"global gradient norm gpu {got_norm:.5f} oracle {want_norm:.5f}", flush=True)
    assert want_norm > clip  # the clip is active
    assert_close(got_norm, want_norm, "global gradient norm", rtol=2e-4, atol=0)
    for name in names:
        w = om.get_param(name)
        shape = w.shape if w.ndim == 2 else (w.size,)
        assert_close(gm.get_param(name, shape), w.reshape(shape, order="F"), f"updated {name}",
                     rtol=1e-4, atol=2e-6)
        # and the update moved the parameter (columns of unused embeddings aside)
    assert not np.array_equal(gm.get_param("tgt.3.W_hi", (H, H)), P["tgt.3.W_hi"])
    gm.close()


def test_config3_two_layer_local_p_model_at_size(orc, host):
    """BASELINE configs[3] as a model: 2+2 layers, hidden 1000, vocabulary 30k, batch 64, source
    and target length 100 (a few columns shorter, so that padding is exercised at this length too),
    local-p attention D=10 with input feeding -- AttentionNode::ForwardProp
    (src/layer_attention.h:243-483) inside NeuralMachineTranslation::GetError
    (src/deep_rnn.h:2173-2317) at longest_sentence 104.  Teacher-forced cross-entropy against the
    oracle per word, the attention output and the alignments of single steps compared directly."""
    layers, H, V, B, D, S, T, longest = 2, 1000, 30000, 64, 10, 100, 100, 104
    rng = np.random.default_rng(1300)
    P = make_params(rng, layers, H, V, V)
    ls = np.full(B, S)
    lt = np.full(B, T)
    ls[[5, 17, 40]] = [37, 81, 99]
    lt[[5, 23, 63]] = [12, 64, 99]
    src = np.full((B, S), -1, np.int32)
    tin = np.full((B, T), -1, np.int32)
    tout = np.full((B, T), -1, np.int32)
    for b in range(B):
        src[b, S - ls[b]:] = zipf_ids(rng, ls[b], V)
        t = zipf_ids(rng, lt[b] - 1, V, lo=3)
        tin[b, :lt[b]] = np.concatenate([[0], t])
        tout[b, :lt[b]] = np.concatenate([t, [1]])
    bi = np.concatenate([ls, S - ls]).astype(np.int32)
    n_words = int(lt.sum())
    gm = host.Model(layers, H, V, V, longest_sentence=longest, attention_mode=1, attention_width=D,
                    feed_input=True, minibatch_size=B)
    gm.set_params(P)
    got = gm.get_error(src, tin, tout, bi)
    for b in (5, 17, 40):  # padded source prefixes stay at exactly zero state on both layers
        pad = S - ls[b]
        for layer in range(layers):
            for kind in (0, 1):
                st = gm.get_state(kind, 0, layer, pad - 1, H, B)
                assert np.all(st[:, b] == 0), (layer, b, kind)
                assert np.any(gm.get_state(kind, 0, layer, pad, H, B)[:, b] != 0), (layer, b, kind)
    # a target column past its sentence end: attention output masked to exactly zero
    assert np.all(gm.get_state(2, 1, 0, 50, H, B)[:, 5] == 0)
    align = np.stack([gm.get_state(3, 1, 0, t, B, 2 * D + 1) for t in (0, 49, 99)])
    live = np.stack([tin[:, t] >= 0 for t in (0, 49, 99)])
    sums = align.sum(axis=2)  # alignments carry the Gaussian factor: 0 < sum <= 1 for live columns
    assert np.all(sums[live] > 0) and np.all(sums[live] <= 1 + 1e-5)
    gm.close()
    om = orc.Model(layers, H, V, V, attention=1, D=D, feed_input=1, longest_sent=longest)
    om.set_params(P)
    t0 = time.time()
    want = om.forward_xent(src, tin, tout, bi)
    print(f"configs[3] model: oracle forward_xent {time.time() - t0:.1f} s, {n_words} target words, "
          f"per-word log-lik gpu {got / n_words:.6f} oracle {want / n_words:.6f}", flush=True)
    assert_close(got / n_words, want / n_words, "per-word log-likelihood", rtol=1e-4, atol=1e-5)
    assert_close(got, want, "sum log p(target)", rtol=2e-5, atol=1e-3)


def test_config5_full_minibatch_properties(host):
    """The configs[4] training step at its own batch (256 sentence pairs of 20-80 tokens, 8+8
    layers, hidden 2048, embedding 1024, vocabulary 50k, dropout 0.2): the oracle would need hours
    for it (its gradients are checked at this width and depth on a small minibatch above), so
    this checks what holds whatever the numbers are -- NeuralMachineTranslation::ComputeGradients /
    UpdateWeights, src/deep_rnn.h:984-1412:
      * the same seed gives the same masks and bit-identical gradients (no atomics, fixed orders);
      * the update leaves the embeddings of words that are not in the minibatch untouched bit for
        bit and moves those of every word that is in it; states of padded source positions are exactly zero;
      * the norm the global clip used equals the float64 norm of the gradients read back (the
        embedding gradients are outside it, src/deep_rnn.h:1326-1412), and the update is
        theta + lr * min(1, clip / norm) * g / B for a matrix read back before and after;
      * without dropout the training forward's log-likelihood equals GetError's."""
    layers, H, E, V, D, B, keep, lr, clip = 8, 2048, 1024, 50000, 10, 256, 0.8, 0.1, 5.0
    rng = np.random.default_rng(1400)
    P = make_params(rng, layers, H, V, V, E=E)
    src, tin, tout, bi, su, tu, n_words = minibatch(rng, B, 20, 80, V, V)
    S = src.shape[1]

    def build(keep_):
        m = host.Model(layers, H, V, V, longest_sentence=84, attention_mode=1, attention_width=D,
                       feed_input=True, minibatch_size=B, embedding_size=E,
                       training=dict(learning_rate=lr, grad_clip_mode=2, norm_clip=clip,
                                     dropout_keep=keep_, dropout_seed=99))
        m.set_params(P)
        return m

    def shape_of(name):
        a = P[name]
        if name.endswith(".W"):  # the embedding gradient holds the minibatch's words only
            return (E, len(su if name.startswith("src") else tu))
        return a.shape if a.ndim == 2 else (a.size,)

    probe = ["tgt.7.W_hi", "src.0.M_f", "tgt.0.Q_o", "attn.W_a", "attn.v_p", "softmax.b_d", "src.3.b_c",
             "tgt.0.W"]
    gm = build(keep)
    ll1 = gm.compute_gradients(src, tin, tout, bi, su, tu)
    first = {n: gm.get_grad(n, shape_of(n)).copy() for n in probe}
    mask1 = gm.get_dropout_mask(1, 1, 3, H, B, 4).copy()
    gm.clear_gradients()
    gm.set_dropout_seed(99)
    ll2 = gm.compute_gradients(src, tin, tout, bi, su, tu)
    assert np.array_equal(gm.get_dropout_mask(1, 1, 3, H, B, 4), mask1)
    assert ll1 == ll2
    for n in probe:
        assert np.array_equal(gm.get_grad(n, shape_of(n)), first[n]), f"{n}: gradients of two runs differ"
    assert abs((mask1 < keep).mean() - keep) < 0.01
    # the embedding gradient has one column per word of the minibatch, none of them empty
    for name, ids in (("src.0.W", su), ("tgt.0.W", tu)):
        g = gm.get_grad(name, (E, len(ids)))
        assert np.all(np.abs(g).max(axis=0) > 0), name
        del g
    emb_before = gm.get_param("src.0.W", (E, V)).copy()
    # the global norm: every gradient but the embeddings', scaled by 1/B
    ss, count = 0.0, 0
    for name in P:
        if name in ("src.0.W", "tgt.0.W"):
            continue
        g = gm.get_grad(name, shape_of(name)).astype(np.float64)
        assert np.isfinite(g).all(), name
        ss += float(np.sum(g * g))
        count += g.size
    want_norm = np.sqrt(ss) / B
    before = gm.get_param("tgt.7.W_hi", (H, H)).copy()
    got_norm = gm.update_weights()
    print(f"configs[4] minibatch: {n_words} target words, log-lik per word {ll1 / n_words:.5f}, "
          f"global norm gpu {got_norm:.6f} float64 of the read-back gradients {want_norm:.6f} "
          f"({count} parameters)", flush=True)
    assert abs(got_norm - want_norm) <= 2e-4 * want_norm
    assert want_norm > clip  # the clip is active
    f = min(1.0, clip / want_norm)
    want_after = before.astype(np.float64) + lr * f * first["tgt.7.W_hi"].astype(np.float64) / B
    assert_close(gm.get_param("tgt.7.W_hi", (H, H)), want_after, "updated tgt.7.W_hi", rtol=1e-5, atol=1e-7)
    assert not gm.get_grad("tgt.7.W_hi", (H, H)).any()  # gradients are cleared by the update
    # words outside the minibatch keep their embeddings bit for bit, every word inside it moves
    emb_after = gm.get_param("src.0.W", (E, V))
    used = np.zeros(V, bool)
    used[su] = True
    assert np.array_equal(emb_after[:, ~used], emb_before[:, ~used])
    assert np.all((emb_after[:, used] != emb_before[:, used]).any(axis=0))
    del emb_before, emb_after
    gm.close()
    del first, before

    g1 = build(1.0)
    ll = g1.compute_gradients(src, tin, tout, bi, su, tu)
    xent = g1.get_error(src, tin, tout, bi)
    print(f"without dropout: training forward {ll:.4f}, GetError {xent:.4f}", flush=True)
    assert abs(ll - xent) <= 1e-5 * abs(xent)
    for b in (1, B // 2, B - 1):
        pad = S - bi[b]
        if pad > 0:
            for layer in (0, layers - 1):
                assert not g1.get_state(0, 0, layer, pad - 1, H, B)[:, b].any(), (layer, b)
    g1.close()
