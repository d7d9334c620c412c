"""GPU parity of the C++ layer classes (through the C facade of liblinmt_host.so) against the CPU
oracle on the same seeded weights and inputs: beam decoding (tokens, back-pointer paths and finished
hypotheses bit-exact; scores within tolerance) and teacher-forced scoring."""
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


def _pair(orc, host, rng, layers, H, Vs, Vt, D, longest, scale, decoding=None, minibatch=1,
          attention=1, feed=True, E=None):
    P = R.make_params(rng, layers, H, Vs, Vt, attention=bool(attention), feed_input=feed,
                      scale=scale, E=E)
    om = orc.Model(layers, H, Vs, Vt, attention=attention, D=D, feed_input=int(feed),
                   longest_sent=longest, E=E or 0)
    om.set_params(P)
    gm = host.Model(layers, H, Vs, Vt, longest_sentence=longest, attention_mode=attention,
                    attention_width=D, feed_input=feed, minibatch_size=minibatch,
                    decoding=decoding, embedding_size=E or 0)
    gm.set_params(P)
    return P, om, gm


def _compare_decode(orc_res, gpu_res, what):
    assert gpu_res["best"].tolist() == orc_res["best"].tolist(), f"{what}: 1-best tokens"
    assert_close(gpu_res["best_score"], orc_res["best_score"], f"{what}: 1-best score", rtol=1e-4,
                 atol=1e-4)
    assert gpu_res["steps"] == orc_res["steps"], f"{what}: decoder steps"
    assert len(gpu_res["hyps"]) == len(orc_res["hyps"]), f"{what}: number of finished hypotheses"
    for (gt, gs), (wt, ws) in zip(gpu_res["hyps"], orc_res["hyps"]):
        assert gt.tolist() == wt.tolist(), f"{what}: hypothesis tokens"
        assert_close(gs, ws, f"{what}: hypothesis score", rtol=1e-4, atol=1e-4)


def test_param_roundtrip(orc, host):
    rng = np.random.default_rng(0)
    P, om, gm = _pair(orc, host, rng, 2, 16, 20, 23, 2, 20, 0.5, decoding=(2, 3))
    for name in ("src.0.W", "src.1.M_c", "tgt.0.Q_o", "tgt.1.W_hf", "tgt.0.b_f", "attn.W_a",
                 "attn.v_p", "softmax.D", "softmax.b_d"):
        assert np.array_equal(gm.get_param(name, P[name].shape), P[name]), name
    with pytest.raises(host.HostError):
        gm.set_params({"tgt.0.nope": np.zeros(3, np.float32)})
    gm.close()


@pytest.mark.parametrize("layers,H,Vs,Vt,D,beam,n_sent,seed",
                         [(2, 64, 120, 150, 3, 4, 7, 1), (1, 32, 50, 60, 10, 5, 3, 2),
                          (4, 48, 80, 400, 2, 12, 5, 3)])
def test_decode_batch_vs_oracle_small(orc, host, layers, H, Vs, Vt, D, beam, n_sent, seed):
    """Ragged batch of sentences decoded at once equals independent single-sentence searches of the
    oracle (the reference decodes one sentence at a time, src/decoder.h:1702-1776)."""
    rng = np.random.default_rng(seed)
    longest = 40
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, longest, 0.4, decoding=(n_sent, beam))
    sents = [rng.integers(0, Vs, size=int(rng.integers(1, 16))) for _ in range(n_sent)]
    sents[0] = rng.integers(0, Vs, size=15)
    got = gm.decode_batch(sents, beam=beam, with_hyps=True)
    for i, s in enumerate(sents):
        want = om.decode_sentence(s, beam=beam)
        _compare_decode(want, got[i], f"sentence {i} (len {len(s)})")
    # a second batch with fewer sentences on the same model (state from the first must not leak)
    got2 = gm.decode_batch(sents[:2], beam=beam, with_hyps=True)
    for i in range(2):
        _compare_decode(om.decode_sentence(sents[i], beam=beam), got2[i], f"rerun sentence {i}")
    gm.close()


def test_decode_options_vs_oracle(orc, host):
    """Penalty, diversity, length normalisation and coverage penalty switched on and off."""
    rng = np.random.default_rng(4)
    P, om, gm = _pair(orc, host, rng, 2, 32, 60, 70, 2, 30, 0.5, decoding=(3, 4))
    sents = [rng.integers(0, 60, size=n) for n in (9, 4, 6)]
    for kw in (dict(penalty=0.3, diversity=0.1), dict(lp_alpha=0.0, cp_beta=0.0),
               dict(max_ratio=0.7, min_ratio=0.2), dict(lp_alpha=1.0, cp_beta=0.5, penalty=-0.2)):
        got = gm.decode_batch(sents, beam=4, with_hyps=True, **kw)
        for i, s in enumerate(sents):
            _compare_decode(om.decode_sentence(s, beam=4, **kw), got[i], f"{kw} sentence {i}")
    gm.close()


def test_decode_with_exported_alignments_vs_oracle(orc, host):
    """unk_replacement_mode__: alignment scores exported at every step (a ragged batch, so the
    number of live columns changes between steps), Viterbi alignment per 1-best token and the
    coverage penalty computed from the scores -- against the oracle's single-sentence search,
    which is pinned on the numpy model (tests/test_oracle_pins.py)."""
    rng = np.random.default_rng(14)
    for layers, H, Vs, Vt, D, beam, lens in ((2, 48, 60, 70, 2, 4, (11, 4, 7, 1, 9)),
                                             (1, 32, 40, 90, 10, 5, (6, 14, 3))):
        P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 30, 0.5, decoding=(len(lens), beam))
        sents = [rng.integers(0, Vs, size=n) for n in lens]
        for kw in (dict(), dict(cp_beta=0.6, lp_alpha=0.3)):
            got = gm.decode_batch(sents, beam=beam, with_hyps=True, alignments=True, **kw)
            plain = gm.decode_batch(sents, beam=beam, with_hyps=True, **kw)
            for i, s in enumerate(sents):
                want = om.decode_sentence(s, beam=beam, alignments=True, **kw)
                _compare_decode(want, got[i], f"{kw} sentence {i} (len {len(s)})")
                assert got[i]["best_viterbi"].tolist() == want["best_viterbi"].tolist(), (i, kw)
                assert all(-1 <= v < len(s) for v in got[i]["best_viterbi"])
                # the search itself is the same with and without the export
                assert len(plain[i]["hyps"]) == len(got[i]["hyps"])
        gm.close()


def test_decode_ensemble_vs_oracle(orc, host):
    """EnsembleFactory with several models: models of different width, depth and attention window
    decode a ragged batch in lockstep, their distributions averaged before every beam step
    (lh_beam_topk_ensemble_f32) -- against the oracle's ensemble search (pinned on the numpy model),
    with and without exported alignments, whose scores are added up over the models.  An ensemble
    of a model with itself gives the model's own translations."""
    rng = np.random.default_rng(15)
    Vs, Vt, beam, lens = 60, 72, 4, (9, 4, 12, 2, 7)
    shapes = ((2, 48, 2), (1, 32, 3), (3, 40, 10))           # layers, H, D
    pairs = [_pair(orc, host, rng, L, H, Vs, Vt, D, 30, 0.5, decoding=(len(lens), beam))
             for L, H, D in shapes]
    oms, gms = [p[1] for p in pairs], [p[2] for p in pairs]
    sents = [rng.integers(0, Vs, size=n) for n in lens]
    for n_models in (2, 3):
        for kw in (dict(), dict(alignments=True, cp_beta=0.6, lp_alpha=0.3)):
            got = gms[0].decode_batch(sents, beam=beam, with_hyps=True, ensemble=gms[1:n_models], **kw)
            for i, s in enumerate(sents):
                want = oms[0].decode_sentence(s, beam=beam, ensemble=tuple(oms[1:n_models]), **kw)
                _compare_decode(want, got[i], f"{n_models} models {kw} sentence {i} (len {len(s)})")
                if kw:
                    assert got[i]["best_viterbi"].tolist() == want["best_viterbi"].tolist(), (i, n_models)
    alone = gms[0].decode_batch(sents, beam=beam, with_hyps=True)
    # a second model with the same parameters
    L0, H0, D0 = shapes[0]
    twin = host.Model(L0, H0, Vs, Vt, longest_sentence=30, attention_mode=1, attention_width=D0,
                      feed_input=True, minibatch_size=1, decoding=(len(lens), beam))
    twin.set_params(pairs[0][0])
    both = gms[0].decode_batch(sents, beam=beam, with_hyps=True, ensemble=[twin])
    for a, b in zip(alone, both):
        assert a["best"].tolist() == b["best"].tolist()
        assert len(a["hyps"]) == len(b["hyps"])
        for (at, as_), (bt, bs) in zip(a["hyps"], b["hyps"]):
            assert at.tolist() == bt.tolist()
            assert abs(as_ - bs) <= 1e-4 * max(1.0, abs(as_))
    # and afterwards every model still decodes on its own
    again = gms[0].decode_batch(sents, beam=beam, with_hyps=True)
    for a, b in zip(alone, again):
        assert a["best"].tolist() == b["best"].tolist() and a["best_score"] == b["best_score"]
    with pytest.raises(host.HostError):
        gms[0].decode_batch(sents, beam=beam, ensemble=[gms[0]])
    twin.close()
    for g in gms:
        g.close()


def test_decode_no_attention_and_no_feed(orc, host):
    rng = np.random.default_rng(5)
    for attention, feed in ((0, False), (1, False)):
        P, om, gm = _pair(orc, host, rng, 2, 32, 60, 70, 2, 30, 0.5, decoding=(3, 3),
                          attention=attention, feed=feed)
        sents = [rng.integers(0, 60, size=n) for n in (7, 3, 5)]
        got = gm.decode_batch(sents, beam=3, with_hyps=True)
        for i, s in enumerate(sents):
            _compare_decode(om.decode_sentence(s, beam=3), got[i],
                            f"attention={attention} feed={feed} sentence {i}")
        gm.close()


@pytest.mark.parametrize("layers,H,E,Vs,Vt,beam,lens,attention,feed",
                         [(2, 64, None, 120, 150, 4, (9, 4, 12, 1, 6), 2, True),   # global attention
                          (3, 48, None, 80, 200, 6, (14, 3, 8), 2, False),
                          (2, 64, 40, 120, 150, 4, (9, 4, 12, 1, 6), 1, True),     # E != H (folded table)
                          (2, 48, 96, 80, 200, 6, (14, 3, 8), 2, True)])
def test_decode_global_attention_and_other_embedding_size(orc, host, layers, H, E, Vs, Vt, beam,
                                                          lens, attention, feed):
    """Beam decoding with Luong global attention (attention_mode 2: the window is the whole
    sentence, no projected memory) and with an embedding narrower / wider than the LSTM (the
    decoder's folded table M*W is then 4H x V from an H x E and an E x V factor), ragged batches,
    against the oracle's single-sentence searches."""
    rng = np.random.default_rng(33)
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, 3, 40, 0.4, decoding=(len(lens), beam),
                      attention=attention, feed=feed, E=E)
    sents = [rng.integers(0, Vs, size=n) for n in lens]
    for align in (False, True):
        got = gm.decode_batch(sents, beam=beam, with_hyps=True, alignments=align)
        for i, s in enumerate(sents):
            want = om.decode_sentence(s, beam=beam, alignments=align)
            _compare_decode(want, got[i], f"attention {attention} E={E} sentence {i} (len {len(s)})")
            if align:
                assert got[i]["best_viterbi"].tolist() == want["best_viterbi"].tolist(), i
    gm.close()


def test_decode_config3_architecture(orc, host):
    """The headline architecture at full width (4+4 layers, H=1000, V=30000, beam 12, local-p D=10,
    feed input) on a few short sentences the CPU oracle finishes in seconds."""
    rng = np.random.default_rng(6)
    layers, H, V, D, beam = 4, 1000, 30000, 10, 12
    P, om, gm = _pair(orc, host, rng, layers, H, V, V, D, 104, 0.08, decoding=(4, beam))
    sents = [rng.integers(0, V, size=n) for n in (6, 4, 5, 3)]
    got = gm.decode_batch(sents, beam=beam, with_hyps=True)
    for i, s in enumerate(sents):
        _compare_decode(om.decode_sentence(s, beam=beam), got[i], f"config-3 sentence {i}")
    gm.close()


def test_decode_same_with_and_without_the_regrouped_step(orc, host, monkeypatch):
    """Decoding regroups the step (encoder lanes; gate product with the cell in its epilogue;
    attention over W_a*hs / W_c1*hs computed once per batch).  With the switches that turn the
    lanes and the projected memory off, the plain step must give the same translations, with
    scores inside the floating-point tolerance, and both must match the oracle."""
    rng = np.random.default_rng(16)
    layers, H, Vs, Vt, D, beam = 3, 96, 200, 260, 4, 6
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 40, 0.35, decoding=(5, beam))
    sents = [rng.integers(0, Vs, size=n) for n in (17, 9, 12, 3, 21)]
    fast = gm.decode_batch(sents, beam=beam, with_hyps=True, alignments=True)
    host.set_debug_option("no_projected_memory", 1)
    host.set_debug_option("no_lanes", 1)
    try:
        plain = gm.decode_batch(sents, beam=beam, with_hyps=True, alignments=True)
    finally:
        host.set_debug_option("no_projected_memory", 0)
        host.set_debug_option("no_lanes", 0)
    for i, (a, b) in enumerate(zip(fast, plain)):
        assert a["best"].tolist() == b["best"].tolist(), i
        assert a["best_viterbi"].tolist() == b["best_viterbi"].tolist(), i
        assert np.isclose(a["best_score"], b["best_score"], rtol=1e-4, atol=1e-5), i
        assert a["n_hyp"] == b["n_hyp"], i
        _compare_decode(om.decode_sentence(sents[i], beam=beam, alignments=True), a,
                        f"regrouped step, sentence {i}")
    gm.close()


def test_decode_same_with_separate_beam_launches(orc, host, monkeypatch):
    """The merge and the state swap of a step as one launch (lh_beam_merge_gather_f32, the default
    with one model) and as the two launches it replaces (debug option "separate_beam_launches"): the same
    kernels' arithmetic, so every token, score and hypothesis is equal bit for bit."""
    rng = np.random.default_rng(23)
    layers, H, Vs, Vt, D, beam = 2, 64, 150, 170, 3, 5
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 40, 0.35, decoding=(6, beam))
    sents = [rng.integers(0, Vs, size=n) for n in (14, 3, 9, 20, 6, 11)]
    gm.profile(2)
    one = gm.decode_batch(sents, beam=beam, with_hyps=True)
    assert "beam_merge_gather" in gm.profile_totals(), "the single launch did not run"
    host.set_debug_option("separate_beam_launches", 1)
    try:
        gm.profile(2)
        two = gm.decode_batch(sents, beam=beam, with_hyps=True)
    finally:
        host.set_debug_option("separate_beam_launches", 0)
    assert "beam_gather" in gm.profile_totals() and "beam_merge_gather" not in gm.profile_totals()
    gm.profile(0)
    for i, (a, b) in enumerate(zip(one, two)):
        assert a["best"].tolist() == b["best"].tolist() and a["best_score"] == b["best_score"], i
        assert a["n_hyp"] == b["n_hyp"] and a["steps"] == b["steps"], i
        for (ta, sa), (tb, sb) in zip(a["hyps"], b["hyps"]):
            assert ta.tolist() == tb.tolist() and sa == sb, i
    gm.close()


def test_decode_same_with_grouped_gate_products(orc, host, monkeypatch):
    """The debug option "grouped_gates" issues what the previous step fixes of every layer's gate product as
    one grouped launch (lh_gate_gemm_group_f32) and leaves M*h of the layer below on the chain.
    Same arithmetic up to the order of two additions: same translations, scores inside the
    floating-point tolerance, both equal to the oracle's."""
    rng = np.random.default_rng(17)
    layers, H, Vs, Vt, D, beam = 4, 96, 200, 260, 4, 6
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 40, 0.35, decoding=(5, beam))
    sents = [rng.integers(0, Vs, size=n) for n in (17, 9, 12, 3, 21)]
    plain = gm.decode_batch(sents, beam=beam, with_hyps=True)
    host.set_debug_option("grouped_gates", 1)
    try:
        gm.profile(2)
        grouped = gm.decode_batch(sents, beam=beam, with_hyps=True)
    finally:
        host.set_debug_option("grouped_gates", 0)
    assert any("gate_gemm_group_kernel" in k for k in gm.profile_totals()), "the grouped launch did not run"
    gm.profile(0)
    for i, (a, b) in enumerate(zip(grouped, plain)):
        assert a["best"].tolist() == b["best"].tolist(), i
        assert np.isclose(a["best_score"], b["best_score"], rtol=1e-4, atol=1e-5), i
        assert a["n_hyp"] == b["n_hyp"], i
        _compare_decode(om.decode_sentence(sents[i], beam=beam), a, f"grouped gates, sentence {i}")
    gm.close()


@pytest.mark.parametrize("layers,H,attention,feed,seed", [(4, 96, 1, True, 18), (1, 64, 0, False, 19),
                                                          (2, 72, 2, True, 20)])
def test_decode_same_with_split_products(orc, host, layers, H, attention, feed, seed):
    """lnmt_set_split_products: the gate products and the output projection of a decoding step as
    six exact bf16 products per term on the bf16 matrix pipe (every step here: min_columns = 1;
    the first step of a feed-input model keeps the fp32 MFMA product).  As close to float64 as the
    fp32 products: same translations, scores inside the floating-point tolerance, both equal to
    the oracle's.  One to four layers, with and without attention / feed input, a ragged batch
    whose live column count changes between steps."""
    rng = np.random.default_rng(seed)
    Vs, Vt, D, beam = 200, 260, 4, 6
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 40, 0.35, decoding=(5, beam),
                      attention=attention, feed=feed)
    sents = [rng.integers(0, Vs, size=n) for n in (17, 9, 12, 3, 21)]
    plain = gm.decode_batch(sents, beam=beam, with_hyps=True)
    gm.set_split_products(True, 1)
    gm.profile(2)
    split = gm.decode_batch(sents, beam=beam, with_hyps=True)
    keys = list(gm.profile_totals())
    assert any(k.startswith("gate_gemm|gemm_split_kernel") for k in keys), "the split gate product did not run"
    assert any(k.startswith("logits_gemm|gemm_split_kernel") for k in keys), "the split output projection did not run"
    gm.profile(0)
    gm.set_split_products(False)
    again = gm.decode_batch(sents, beam=beam, with_hyps=True)
    for i, (a, b, c) in enumerate(zip(split, plain, again)):
        assert a["best"].tolist() == b["best"].tolist(), i
        assert np.isclose(a["best_score"], b["best_score"], rtol=1e-4, atol=1e-5), i
        assert a["n_hyp"] == b["n_hyp"], i
        _compare_decode(om.decode_sentence(sents[i], beam=beam), a, f"split products, sentence {i}")
        assert c["best"].tolist() == b["best"].tolist() and c["best_score"] == b["best_score"], i
    gm.close()


def test_decode_ensemble_and_alignments_with_split_products(orc, host):
    """Split products under the other decoding features: an ensemble of two models of different
    width (both with split products, each packing its own weights) with exported alignments and
    the coverage penalty -- against the oracle's ensemble search."""
    rng = np.random.default_rng(21)
    Vs, Vt, beam, lens = 60, 72, 4, (9, 4, 12, 2, 7)
    pairs = [_pair(orc, host, rng, L, H, Vs, Vt, D, 30, 0.5, decoding=(len(lens), beam))
             for L, H, D in ((2, 48, 2), (3, 40, 10))]
    oms, gms = [p[1] for p in pairs], [p[2] for p in pairs]
    sents = [rng.integers(0, Vs, size=n) for n in lens]
    for g in gms:
        g.set_split_products(True, 1)
    kw = dict(alignments=True, cp_beta=0.6, lp_alpha=0.3)
    got = gms[0].decode_batch(sents, beam=beam, with_hyps=True, ensemble=gms[1:], **kw)
    for i, s in enumerate(sents):
        want = oms[0].decode_sentence(s, beam=beam, ensemble=tuple(oms[1:]), **kw)
        _compare_decode(want, got[i], f"split products, ensemble, sentence {i} (len {len(s)})")
        assert got[i]["best_viterbi"].tolist() == want["best_viterbi"].tolist(), i
    for g in gms:
        g.close()


def test_decode_random_architectures_vs_oracle(orc, host):
    """A seeded sweep over architectures and batch shapes the fixed cases do not hit: 1-4 layers,
    hidden sizes that land on different tile configurations (and on the one- and two-quad attention
    kernels), windows from 3 to 21 slots, beams 2-12, partly filled batches, attention / feed input
    / alignment export on and off.  Weight scales stay where fp32 rounding is not amplified: with
    uniform(-0.8, 0.8) weights at H = 256 two GPU runs that differ only in the tile configuration
    of their products already disagree by 1e-3 after one step, so that regime says nothing."""
    rng = np.random.default_rng(2024)
    for trial in range(14):
        layers = int(rng.integers(1, 5))
        H = int(rng.choice([32, 48, 100, 128, 256, 1100]))
        Vs, Vt = int(rng.integers(30, 300)), int(rng.integers(40, 500))
        D, n_sent = int(rng.integers(1, 11)), int(rng.integers(1, 9))
        att = int(rng.choice([0, 1, 1, 1]))
        feed = bool(att and rng.integers(0, 2))
        align = bool(att and rng.integers(0, 2))
        beam = min(int(rng.integers(2, 13)), int(np.sqrt(Vt)))
        scale = float(rng.choice([0.2, 0.4])) * (0.25 if H > 256 else (0.5 if H == 256 else 1.0))
        P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 44, scale, decoding=(n_sent, beam),
                          attention=att, feed=feed)
        n = int(rng.integers(1, n_sent + 1))
        sents = [rng.integers(0, Vs, size=int(rng.integers(1, 25))) for _ in range(n)]
        got = gm.decode_batch(sents, beam=beam, with_hyps=True, alignments=align)
        what = (f"trial {trial}: layers={layers} H={H} V={Vs}/{Vt} D={D} beam={beam} batch {n}/{n_sent} "
                f"attention={att} feed={feed} alignments={align} scale={scale}")
        for i, s_ in enumerate(sents):
            want = om.decode_sentence(s_, beam=beam, alignments=align)
            _compare_decode(want, got[i], f"{what}, sentence {i} (len {len(s_)})")
            if align:
                assert got[i]["best_viterbi"].tolist() == want["best_viterbi"].tolist(), what
        gm.close()


def _ragged_minibatch(rng, B, S, T, Vs, Vt, min_len=1):
    lens_s = rng.integers(min_len, S + 1, size=B)
    lens_t = rng.integers(max(min_len, 2), T + 1, size=B)
    lens_s[0], lens_t[0] = S, T
    src = np.full((B, S), -1, np.int32)
    tin = np.full((B, T), -1, np.int32)
    tout = np.full((B, T), -1, np.int32)
    for b in range(B):
        s = rng.integers(0, Vs, size=lens_s[b])
        t = rng.integers(3, Vt, size=lens_t[b] - 1)
        src[b, S - lens_s[b]:] = s[::-1]
        tin[b, :lens_t[b]] = np.concatenate([[0], t])
        tout[b, :lens_t[b]] = np.concatenate([t, [1]])
    bi = np.concatenate([lens_s, S - lens_s]).astype(np.int32)
    return src, tin, tout, bi, int(lens_t.sum())


@pytest.mark.parametrize("layers,H,Vs,Vt,D,B,S,T,attention,feed,E",
                         [(2, 64, 90, 110, 3, 9, 12, 10, 1, True, None),
                          (4, 128, 300, 500, 10, 16, 20, 18, 1, True, None),
                          (2, 64, 90, 110, 3, 9, 12, 10, 2, True, None),   # global general (build-defined)
                          (2, 64, 90, 110, 3, 9, 12, 10, 0, False, None),
                          (2, 64, 90, 110, 3, 9, 12, 10, 1, True, 40),     # embedding size != LSTM size
                          (3, 96, 90, 110, 10, 9, 12, 10, 2, True, 128)])
def test_get_error_vs_oracle(orc, host, layers, H, Vs, Vt, D, B, S, T, attention, feed, E):
    rng = np.random.default_rng(7)
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 30, 0.3, minibatch=B,
                      attention=attention, feed=feed, E=E)
    src, tin, tout, bi, n_words = _ragged_minibatch(rng, B, S, T, Vs, Vt)
    want = om.forward_xent(src, tin, tout, bi)
    got = gm.get_error(src, tin, tout, bi)
    assert_close(got, want, "sum log p(target)", rtol=1e-5, atol=1e-3)
    assert_close(got / n_words, want / n_words, "per-word log-likelihood", rtol=1e-4, atol=1e-5)
    # smaller minibatch on the same allocation
    got2 = gm.get_error(src[:4], tin[:4], tout[:4], np.concatenate([bi[:4], bi[B:B + 4]]))
    want2 = om.forward_xent(src[:4], tin[:4], tout[:4], np.concatenate([bi[:4], bi[B:B + 4]]))
    assert_close(got2, want2, "sub-batch", rtol=1e-5, atol=1e-3)
    # padded source prefix keeps the state at exactly zero; padded target columns are zeroed
    for b in range(B):
        pad = S - bi[b]
        if pad > 0:
            h = gm.get_state(0, 0, layers - 1, pad - 1, H, B)
            assert np.all(h[:, b] == 0)
    gm.close()


def test_config1_single_layer_lstm(orc, host):
    """Config 1: single-layer LSTM, E=H=256, B=32, T=30, V=5000, uniform ids; language-model path
    (no encoder, no attention).  Final-step log-probs enter through the summed log-likelihood."""
    rng = np.random.default_rng(8)
    H, V, B, T = 256, 5000, 32, 30
    P = R.make_params(rng, 1, H, V, V, attention=False, feed_input=False, scale=0.08)
    gm = host.Model(1, H, V, V, longest_sentence=34, attention_mode=0, feed_input=False,
                    minibatch_size=B, sequence_to_sequence=False)
    gm.set_params({k: v for k, v in P.items() if not k.startswith("src.")})
    tin = rng.integers(0, V, size=(B, T)).astype(np.int32)
    tout = rng.integers(0, V, size=(B, T)).astype(np.int32)
    got = gm.get_error(None, tin, tout, None)
    # oracle: step the cell by hand with the oracle's kernels-level functions
    Wih = np.concatenate([P[f"tgt.0.M_{g}"] for g in R.GATES], axis=0)
    Whh = np.concatenate([P[f"tgt.0.W_h{g}"] for g in R.GATES], axis=0)
    bias = np.concatenate([P[f"tgt.0.b_{g}"] for g in R.GATES])
    h = np.zeros((H, B), np.float32)
    c = np.zeros((H, B), np.float32)
    want = 0.0
    ones = np.ones(B, np.int32)
    for t in range(T):
        x = orc.embed_lookup(P["tgt.0.W"], tin[:, t])
        gates, c, h = orc.lstm_cell_fwd(orc.gemm(Wih, x), bias, c, ones, orc.gemm(Whh, h))
        gh = gm.get_state(0, 1, 0, t, H, B)
        gc = gm.get_state(1, 1, 0, t, H, B)
        assert_close(gh, h, f"h_t at t={t}")
        assert_close(gc, c, f"c_t at t={t}")
        lp, loss = orc.logsoftmax_xent(orc.gemm(P["softmax.D"], h), P["softmax.b_d"], tout[:, t],
                                       ones)
        want += loss
    assert_close(got, want, "config-1 log-likelihood", rtol=1e-5, atol=1e-3)
    gm.close()
