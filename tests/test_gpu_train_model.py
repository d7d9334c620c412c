"""GPU parity of the training path of the C++ layer classes (ComputeGradients / UpdateWeights through
the C facade) against the CPU oracle on the same seeded weights and minibatches.  The oracle's
backward is itself pinned by central differences (tests/test_oracle_train_pins.py).  fp32 results
within rtol=1e-4 / atol=2e-5 (the GPU sums over minibatch x steps in one GEMM, the oracle step by
step, so the last bits differ)."""
import numpy as np
import pytest

from conftest import assert_close
import ref_numpy as R

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def host():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from linmt_amd import host as h
    h.load()
    return h


def _minibatch(rng, Vs, Vt, lens_s, lens_t):
    sents = [(rng.integers(0, Vs, size=a), rng.integers(3, Vt, size=b)) for a, b in zip(lens_s, lens_t)]
    return sents, R.pack_minibatch(sents)


def _pair(orc, host, rng, layers, H, Vs, Vt, D, attention, feed, B, training, scale=0.5, clip_cell=False,
          E=None, cell_clip=50.0):
    P = R.make_params(rng, layers, H, Vs, Vt, attention=bool(attention), feed_input=bool(feed),
                      scale=scale, E=E)
    om = orc.Model(layers, H, Vs, Vt, attention=attention, D=D, feed_input=int(feed), longest_sent=40,
                   E=E or 0)
    om.set_params(P)
    gm = host.Model(layers, H, Vs, Vt, longest_sentence=40, attention_mode=attention,
                    attention_width=D, feed_input=bool(feed), minibatch_size=B, training=training,
                    clip_cell=clip_cell, embedding_size=E or 0, cell_clip_threshold=cell_clip)
    gm.set_params(P)
    return P, om, gm


def _grad_shape(P, name, su, tu):
    if name == "src.0.W":
        return (P[name].shape[0], len(su))
    if name == "tgt.0.W":
        return (P[name].shape[0], len(tu))
    return P[name].shape


CASES = [
    dict(layers=2, H=16, attention=1, feed=1, D=2, seed=61),
    dict(layers=1, H=13, attention=1, feed=0, D=1, seed=62),   # H % 4 != 0: scalar kernel paths
    dict(layers=2, H=16, attention=0, feed=0, D=2, seed=63),
    dict(layers=3, H=32, attention=1, feed=1, D=10, seed=64),  # window wider than the sentences
    dict(layers=2, H=16, attention=2, feed=1, D=2, seed=65),   # global attention
    # embedding size != LSTM size (the reference has E == H; the oracle's generalisation is pinned
    # by central differences): a wider, a narrower and an unaligned embedding
    dict(layers=2, H=32, E=24, attention=1, feed=1, D=2, seed=66),
    dict(layers=2, H=16, E=40, attention=1, feed=1, D=3, seed=67),
    dict(layers=1, H=16, E=13, attention=2, feed=0, D=2, seed=68),
]


@pytest.mark.parametrize("case", CASES,
                         ids=lambda c: f"L{c['layers']}H{c['H']}E{c.get('E', 0)}a{c['attention']}f{c['feed']}")
def test_compute_gradients_vs_oracle(orc, host, case):
    rng = np.random.default_rng(case["seed"])
    Vs, Vt = 29, 41
    lens_s, lens_t = [5, 3, 9, 4, 7, 1], [4, 6, 2, 8, 5, 3]
    B = len(lens_s)
    P, om, gm = _pair(orc, host, rng, case["layers"], case["H"], Vs, Vt, case["D"],
                      case["attention"], case["feed"], B, dict(grad_clip_mode=0), E=case.get("E"))
    sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, Vs, Vt, lens_s, lens_t)
    want_ll, want = om.compute_gradients(src, tin, tout, bi, su, tu)
    got_ll = gm.compute_gradients(src, tin, tout, bi, su, tu)
    assert_close(got_ll, want_ll, "sum log p(target)", rtol=1e-5, atol=1e-4)
    for name in om.param_names():
        shape = _grad_shape(P, name, su, tu)
        g = gm.get_grad(name, shape)
        assert_close(g, np.asarray(want[name]).reshape(shape, order="F"), f"gradient of {name}",
                     atol=2e-5)
    # the same minibatch again without an update accumulates (the reference clears only in
    # ClearGradients): every gradient doubles
    gm.compute_gradients(src, tin, tout, bi, su, tu)
    for name in ("softmax.D", "tgt.0.M_i", "tgt.0.W", "src.0.b_f" if True else ""):
        shape = _grad_shape(P, name, su, tu)
        assert_close(gm.get_grad(name, shape), 2 * np.asarray(want[name]).reshape(shape, order="F"),
                     f"accumulated gradient of {name}", atol=4e-5)
    gm.clear_gradients()
    assert not np.any(gm.get_grad("softmax.D", P["softmax.D"].shape))
    gm.close()


@pytest.mark.parametrize("case", [CASES[0], CASES[1], CASES[3], CASES[4], CASES[6]],
                         ids=lambda c: f"L{c['layers']}H{c['H']}E{c.get('E', 0)}a{c['attention']}f{c['feed']}")
def test_compute_gradients_with_split_products_vs_oracle(orc, host, case):
    """lnmt_set_split_products on a training model, size thresholds off (min_columns = 1): every
    matrix product that goes through the model's Gemm() -- error and weight-gradient products,
    transposed operands, several K segments, accumulation into the gradient buffers, the output
    projection, attention, unaligned sizes -- is packed into bf16 planes and formed as six exact
    products per term.  Same tolerance against the oracle as the fp32 MFMA products."""
    rng = np.random.default_rng(case["seed"])
    Vs, Vt = 29, 41
    lens_s, lens_t = [5, 3, 9, 4, 7, 1], [4, 6, 2, 8, 5, 3]
    B = len(lens_s)
    P, om, gm = _pair(orc, host, rng, case["layers"], case["H"], Vs, Vt, case["D"],
                      case["attention"], case["feed"], B, dict(grad_clip_mode=0), E=case.get("E"))
    sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, Vs, Vt, lens_s, lens_t)
    want_ll, want = om.compute_gradients(src, tin, tout, bi, su, tu)
    gm.set_split_products(True, 1)
    gm.profile(2)
    got_ll = gm.compute_gradients(src, tin, tout, bi, su, tu)
    keys = list(gm.profile_totals())
    gm.profile(0)
    # everything that goes through the model's Gemm(): only the forward gate product of a step,
    # which hands the cell kernel up to three addends (GemmAddends), keeps the fp32 MFMA kernel
    fp32 = sorted({k.split("|")[0] for k in keys if "|gemm_kernel" in k or "|gemm_generic_kernel" in k})
    # (and, when H is not a multiple of 8, products of several K segments: segments are packed
    # side by side in whole groups of 8 k)
    allowed = {"gate_gemm"} | ({"attn_out_gemm", "error_gemm"} if case["H"] % 8 else set())
    assert set(fp32) <= allowed, keys
    for site in ("weight_grad_gemm", "error_gemm", "logits_gemm"):
        assert any(k.startswith(site + "|gemm_split_kernel") for k in keys), (site, keys)
    assert_close(got_ll, want_ll, "sum log p(target)", rtol=1e-5, atol=1e-4)
    for name in om.param_names():
        shape = _grad_shape(P, name, su, tu)
        assert_close(gm.get_grad(name, shape), np.asarray(want[name]).reshape(shape, order="F"),
                     f"gradient of {name}", atol=2e-5)
    gm.close()


@pytest.mark.parametrize("case", [CASES[0], CASES[2], CASES[3], CASES[4], CASES[5]],
                         ids=lambda c: f"L{c['layers']}H{c['H']}E{c.get('E', 0)}a{c['attention']}f{c['feed']}")
def test_compute_gradients_with_error_products_left_in_planes(orc, host, case):
    """The per-step W^T d products of ComputeGradients stay in partial planes when their K range is
    split over workgroups, and the cell kernel of step t-1 / of the layer below adds the planes as
    it reads them.  At these sizes no product would be split by itself (at H = 2048 they are:
    tests/test_gpu_configs_at_size.py), so a split of 2 is forced: same gradients against the
    oracle.  (That the cell kernel gives the bits of the reduced product is
    tests/test_gpu_train_kernels.py::test_lstm_cell_bwd_error_terms_as_partial_planes.)"""
    import torch
    from linmt_amd import lib as lh
    rng = np.random.default_rng(case["seed"])
    Vs, Vt = 29, 41
    lens_s, lens_t = [5, 3, 9, 4, 7, 1], [4, 6, 2, 8, 5, 3]
    B = len(lens_s)
    P, om, gm = _pair(orc, host, rng, case["layers"], case["H"], Vs, Vt, case["D"],
                      case["attention"], case["feed"], B, dict(grad_clip_mode=0), E=case.get("E"))
    sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, Vs, Vt, lens_s, lens_t)
    want_ll, want = om.compute_gradients(src, tin, tout, bi, su, tu)
    L = lh.load()
    H = case["H"]
    try:
        L.lh_gemm_set_splits_override(2)
        # the product of a step is indeed left in two planes at this size
        ws = torch.empty(4 * ((H + 3) & ~3) * B, device="cuda")
        a = torch.zeros(4 * H * H, device="cuda")
        x = torch.zeros(4 * H * B, device="cuda")
        out = torch.zeros(H * B, device="cuda")
        assert lh.gemm_planes(H, B, [(a, 4 * H, x, 4 * H, 4 * H)], out, H, ws, 4, transA=True) == 2
        got_ll = gm.compute_gradients(src, tin, tout, bi, su, tu)
        grads = {name: gm.get_grad(name, _grad_shape(P, name, su, tu)) for name in om.param_names()}
    finally:
        L.lh_gemm_set_splits_override(0)
    assert_close(got_ll, want_ll, "sum log p(target)", rtol=1e-5, atol=1e-4)
    for name in om.param_names():
        shape = _grad_shape(P, name, su, tu)
        assert_close(grads[name], np.asarray(want[name]).reshape(shape, order="F"), f"gradient of {name}",
                     atol=2e-5)
    gm.close()


@pytest.mark.parametrize("case", [CASES[0], CASES[2], CASES[3], CASES[4], CASES[5]],
                         ids=lambda c: f"L{c['layers']}H{c['H']}E{c.get('E', 0)}a{c['attention']}f{c['feed']}")
def test_stepwise_reference_calls_give_the_same_gradients(orc, host, case):
    """The layer classes driven the reference's way -- per target and source step
    BackPropPreprocessGpu / BackProp1 / BackProp2 on the loss layer, AttentionNode::BackProp,
    BackPropPreprocessGpu + BackPropGpu(index) on every LSTM node, in the order of
    NeuralMachineTranslation::ComputeGradients (src/deep_rnn.h:1137-1273) -- against the oracle,
    and against the batched ComputeGradients of the same model."""
    rng = np.random.default_rng(case["seed"])
    Vs, Vt = 29, 41
    lens_s, lens_t = [5, 3, 9, 4, 7, 1], [4, 6, 2, 8, 5, 3]
    B = len(lens_s)
    P, om, gm = _pair(orc, host, rng, case["layers"], case["H"], Vs, Vt, case["D"],
                      case["attention"], case["feed"], B, dict(grad_clip_mode=0), E=case.get("E"))
    sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, Vs, Vt, lens_s, lens_t)
    want_ll, want = om.compute_gradients(src, tin, tout, bi, su, tu)
    got_ll = gm.compute_gradients(src, tin, tout, bi, su, tu, stepwise=True)
    assert_close(got_ll, want_ll, "sum log p(target)", rtol=1e-5, atol=1e-4)
    step = {}
    for name in om.param_names():
        shape = _grad_shape(P, name, su, tu)
        step[name] = gm.get_grad(name, shape)
        assert_close(step[name], np.asarray(want[name]).reshape(shape, order="F"),
                     f"stepwise gradient of {name}", atol=2e-5)
    gm.clear_gradients()
    gm.compute_gradients(src, tin, tout, bi, su, tu)
    for name in om.param_names():
        assert_close(gm.get_grad(name, step[name].shape), step[name], f"batched vs stepwise {name}",
                     atol=2e-5)
    gm.close()


@pytest.mark.parametrize("mode,E", [(0, None), (1, None), (2, None), (3, None), (2, 24), (1, 8)])
def test_update_weights_vs_oracle(orc, host, mode, E):
    rng = np.random.default_rng(70 + mode)
    layers, H, Vs, Vt, D = 2, 16, 29, 41, 2
    lens_s, lens_t = [5, 3, 9, 4], [4, 6, 2, 8]
    B = len(lens_s)
    lr = 0.7
    # thresholds low enough that every clip is active on these gradients
    opts = dict(learning_rate=lr, grad_clip_mode=mode, norm_clip=0.05, individual_clip=0.002)
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 1, 1, B, opts, scale=0.8, E=E)
    for it in range(2):  # the second minibatch starts from cleared gradients and updated weights
        sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, Vs, Vt, lens_s, lens_t)
        want_ll, _ = om.compute_gradients(src, tin, tout, bi, su, tu)
        got_ll = gm.compute_gradients(src, tin, tout, bi, su, tu)
        assert_close(got_ll, want_ll, f"minibatch {it}: sum log p", rtol=1e-5, atol=1e-4)
        want_norm = om.update_weights(lr, mode, opts["norm_clip"], opts["individual_clip"], B)
        got_norm = gm.update_weights()
        if mode == 2:
            assert want_norm > opts["norm_clip"]
            assert_close(got_norm, want_norm, "global gradient norm", rtol=1e-4, atol=1e-6)
        for name in om.param_names():
            assert_close(gm.get_param(name, P[name].shape),
                         om.get_param(name).reshape(P[name].shape, order="F"),
                         f"minibatch {it}: updated {name}", atol=2e-6)
        assert not np.any(gm.get_grad("tgt.1.W_ho", (H, H)))
    gm.close()


@pytest.mark.parametrize("modes,mode", [((0, 0, 0, 1, 1, 1), 2), ((1, 1, 1, 0, 1, 0), 2), ((1, 0, 1, 1, 0, 1), 1)],
                         ids=["finetune", "source_rnn_and_attention_frozen", "target_side_frozen_per_matrix_clip"])
def test_update_weights_with_frozen_groups_vs_oracle(orc, host, modes, mode):
    """lnmt_set_train_modes, the reference's train_*_mode__ switches of UpdateParams
    (src/layer_input_to_hidden.h:1154,1257,1263, src/layer_hidden_to_hidden.h:765,831,
    src/layer_loss.h:1144; --finetune = the three embedding groups off): two minibatches, the
    frozen groups keep their bits, the others and the global norm follow the oracle."""
    rng = np.random.default_rng(90)
    layers, H, Vs, Vt, D = 2, 16, 29, 41, 2
    lens_s, lens_t = [5, 3, 9, 4], [4, 6, 2, 8]
    B, lr = len(lens_s), 0.7
    opts = dict(learning_rate=lr, grad_clip_mode=mode, norm_clip=0.05, individual_clip=0.002)
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 1, 1, B, opts, scale=0.8)
    om.set_train_modes(*modes)
    gm.set_train_modes(*modes)

    def group(name):
        if name in ("src.0.W", "tgt.0.W"):
            return 0 if name[0] == "s" else 1
        return {"softmax": 2, "src": 3, "tgt": 4, "attn": 5}[name.split(".")[0]]

    for it in range(2):
        sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, Vs, Vt, lens_s, lens_t)
        om.compute_gradients(src, tin, tout, bi, su, tu)
        gm.compute_gradients(src, tin, tout, bi, su, tu)
        want_norm = om.update_weights(lr, mode, opts["norm_clip"], opts["individual_clip"], B)
        got_norm = gm.update_weights()
        if mode == 2:
            assert_close(got_norm, want_norm, "global gradient norm", rtol=1e-4, atol=1e-6)
        for name in om.param_names():
            got = gm.get_param(name, P[name].shape)
            if modes[group(name)]:
                assert_close(got, om.get_param(name).reshape(P[name].shape, order="F"),
                             f"minibatch {it}: updated {name}", atol=2e-6)
                assert not np.array_equal(got, P[name]), name
            else:
                assert np.array_equal(got, P[name]), f"minibatch {it}: frozen {name} moved"
            shape = _grad_shape(P, name, su, tu)
            assert not np.any(gm.get_grad(name, shape)), f"minibatch {it}: gradient of {name} not cleared"
    gm.close()


def test_gradients_with_error_clip(orc, host):
    """--clip-cell: cell values clamped forward, the errors a node hands on (to step t-1, to the LSTM
    layer below, to the attention node through feed input) clamped backward -- against the oracle's
    restatement of those clamps (pinned by textbook BPTT in tests/test_oracle_train_pins.py).  The
    thresholds are set low enough to bind; a clamp that never binds changes nothing."""
    rng = np.random.default_rng(81)
    layers, H, Vs, Vt, D = 3, 16, 29, 41, 2
    lens_s, lens_t = [5, 3, 9, 4], [4, 6, 2, 8]
    B = len(lens_s)
    sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, Vs, Vt, lens_s, lens_t)
    outs = []
    for clip_cell, cell, err in ((False, 50.0, 1000.0), (True, 50.0, 1000.0), (True, 0.3, 2e-3)):
        r2 = np.random.default_rng(82)
        P, om, gm = _pair(orc, host, r2, layers, H, Vs, Vt, D, 1, 1, B,
                          dict(grad_clip_mode=0, error_clip_threshold=err), clip_cell=clip_cell,
                          cell_clip=cell)
        got_ll = gm.compute_gradients(src, tin, tout, bi, su, tu)
        om.set_clip(cell if clip_cell else 0.0, err if clip_cell else 0.0)
        want_ll, want = om.compute_gradients(src, tin, tout, bi, su, tu)
        assert_close(got_ll, want_ll, "sum log p(target)", rtol=1e-5, atol=1e-4)
        for name in om.param_names():
            shape = _grad_shape(P, name, su, tu)
            assert_close(gm.get_grad(name, shape), np.asarray(want[name]).reshape(shape, order="F"),
                         f"clip_cell={clip_cell} cell={cell} err={err}: gradient of {name}", atol=2e-5)
        outs.append(gm.get_grad("src.0.M_i", (H, H)))
        gm.close()
    assert np.array_equal(outs[0], outs[1])
    assert not np.allclose(outs[0], outs[2], rtol=1e-3, atol=1e-7)


@pytest.mark.parametrize("attention,E", [(1, None), (0, None), (1, 24)])
def test_compute_gradients_with_dropout_vs_oracle(orc, host, attention, E):
    """The model draws its own masks (one uniform tensor per layer and minibatch); the test reads
    them back and hands the very same masks to the oracle."""
    rng = np.random.default_rng(95 + attention)
    layers, H, Vs, Vt, D, keep = 3, 16, 29, 41, 2, 0.7
    lens_s, lens_t = [5, 3, 9, 4, 7, 1], [4, 6, 2, 8, 5, 3]
    B = len(lens_s)
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, attention, attention, B,
                      dict(grad_clip_mode=0, dropout_keep=keep, dropout_seed=7), E=E)
    sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, Vs, Vt, lens_s, lens_t)
    S, T = src.shape[1], tin.shape[1]
    lls = []
    for it in range(2):  # a second minibatch draws new masks
        got_ll = gm.compute_gradients(src, tin, tout, bi, su, tu)
        se = gm.get_dropout_mask(0, 0, 0, E or H, B, S)
        te = gm.get_dropout_mask(0, 1, 0, E or H, B, T)
        so = np.stack([gm.get_dropout_mask(1, 0, l, H, B, S) if l < layers - 1
                       else np.ones((S, B, H), np.float32) for l in range(layers)])
        to = np.stack([gm.get_dropout_mask(1, 1, l, H, B, T) for l in range(layers)])
        assert 0.6 < (te < keep).mean() < 0.8
        om.set_dropout(keep, B, se, te, so, to)
        want_ll, want = om.compute_gradients(src, tin, tout, bi, su, tu)
        assert_close(got_ll, want_ll, "sum log p(target)", rtol=1e-5, atol=1e-4)
        for name in om.param_names():
            shape = _grad_shape(P, name, su, tu)
            assert_close(gm.get_grad(name, shape), np.asarray(want[name]).reshape(shape, order="F"),
                         f"gradient of {name}", atol=2e-5)
        gm.clear_gradients()
        lls.append(got_ll)
    assert abs(lls[0] - lls[1]) > 1e-3  # different masks, different result
    # scoring on the same model applies no dropout
    om.set_dropout(0.0)
    assert_close(gm.get_error(src, tin, tout, bi), om.forward_xent(src, tin, tout, bi),
                 "GetError on a training model", rtol=1e-5, atol=1e-4)
    gm.close()


def test_training_rejects_partial_minibatch(orc, host):
    rng = np.random.default_rng(90)
    P, om, gm = _pair(orc, host, rng, 1, 16, 29, 41, 2, 1, 1, 4, dict(grad_clip_mode=0))
    sents, (src, tin, tout, bi, su, tu) = _minibatch(rng, 29, 41, [3, 4], [2, 3])
    with pytest.raises(host.HostError):
        gm.compute_gradients(src, tin, tout, bi, su, tu)
    gm.close()
