"""DecodeStream (lnmt_decode_stream): any number of sentences through the model's slots of beam
columns, a finished sentence's slot going to the next one.  Every sentence must come out as the
oracle's single-sentence search gives it (Decoder::ExpandHypothesis, src/decoder.h:355-525, on top
of the step functions of src/deep_rnn.h:1572-1872): tokens and hypotheses exactly, scores within
rtol 1e-4 / atol 1e-4 -- whatever the sentences around it in the launch are doing, including the
first step of a feed-input model (plain kernels, fp32 sigmoids) next to later steps (Feed kernels)."""
import numpy as np
import pytest

from test_gpu_model import _compare_decode, _pair

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def host():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from linmt_amd import host as h
    h.load()
    return h


@pytest.mark.parametrize("layers,H,Vs,Vt,D,beam,slots,n,feed,seed", [
    (2, 64, 120, 150, 3, 4, 3, 11, True, 1),     # several groups, slots change hands many times
    (1, 32, 50, 60, 10, 5, 4, 4, True, 2),       # exactly one group
    (4, 48, 80, 400, 2, 12, 2, 13, True, 3),     # more groups than the ring of encoder slabs holds
    (2, 40, 70, 90, 4, 3, 5, 3, False, 4),       # fewer sentences than slots, no input feeding
])
def test_decode_stream_vs_oracle(orc, host, layers, H, Vs, Vt, D, beam, slots, n, feed, seed):
    rng = np.random.default_rng(seed)
    longest = 40
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, longest, 0.4, decoding=(slots, beam), feed=feed)
    sents = [rng.integers(0, Vs, size=int(rng.integers(1, 16))) for _ in range(n)]
    sents[0] = rng.integers(0, Vs, size=15)
    got = gm.decode_stream(sents, beam=beam, with_hyps=True)
    want = [om.decode_sentence(s, beam=beam) for s in sents]
    for i, s in enumerate(sents):
        _compare_decode(want[i], got[i], f"sentence {i} (len {len(s)})")
    # steps in all: far fewer than one batch after the other would take
    batches = [sents[i:i + slots] for i in range(0, n, slots)]
    assert gm.stream_ticks <= sum(max(w["steps"] for w in want[i:i + slots]) for i in range(0, n, slots))
    assert gm.stream_ticks >= max(w["steps"] for w in want)
    # the model is left as DecodeBatch needs it, and a second stream starts clean
    got_b = gm.decode_batch(batches[0], beam=beam, with_hyps=True)
    for i in range(len(batches[0])):
        _compare_decode(want[i], got_b[i], f"batch after stream, sentence {i}")
    got2 = gm.decode_stream(sents[::-1], beam=beam, with_hyps=True)
    for i, w in enumerate(want[::-1]):
        _compare_decode(w, got2[i], f"second stream, sentence {i}")
    gm.close()


def test_decode_stream_history_and_errors(orc, host):
    rng = np.random.default_rng(9)
    beam, slots = 4, 3
    P, om, gm = _pair(orc, host, rng, 2, 48, 90, 110, 3, 40, 0.4, decoding=(slots, beam))
    sents = [rng.integers(0, 90, size=int(rng.integers(2, 12))) for _ in range(7)]
    got = gm.decode_stream(sents, beam=beam)
    for i, s in enumerate(sents):
        tr = om.decode_sentence_trace(s, beam=beam)
        tok, bp, sc = gm.decode_history(i, beam)
        assert tok.tolist() == tr["tok"].tolist() and bp.tolist() == tr["backptr"].tolist(), i
        live = tr["score"] > -1e30
        assert np.allclose(sc[live], tr["score"][live], rtol=1e-4, atol=1e-4), i
        assert got[i]["best"].tolist() == tr["best"].tolist()
    with pytest.raises(host.HostError):
        gm.decode_stream(sents, beam=beam + 1)
    with pytest.raises(host.HostError):
        gm.decode_stream([np.zeros(0, np.int32)], beam=beam)
    gm.close()
    # global attention has no projected memory to stream over
    P, om, gm = _pair(orc, host, rng, 1, 32, 50, 60, 0, 20, 0.4, decoding=(2, 3), attention=2)
    with pytest.raises(host.HostError):
        gm.decode_stream([rng.integers(0, 50, size=5)], beam=3)
    gm.close()


def test_decode_stream_equals_decode_batch_bit_for_bit_on_random_shapes(host):
    """Which sentences share a launch must not matter.  With every matrix product held to one tile
    shape and one K order (otherwise the shape is chosen by the number of columns, which shrinks in
    DecodeBatch as sentences finish), a column's arithmetic does not depend on its neighbours or on
    the tick it runs at: over random layer counts, widths, beams, slot counts and list lengths (up to
    six times the slots) every sentence must come out of the stream with exactly the tokens, finished
    hypotheses and score bits DecodeBatch gives it.  DecodeBatch gets the sentences in the groups the
    stream encodes them in (longest first, n_sent at a time): a full group's encoder runs layer-major
    with the input products batched over the steps and added to the recurrent ones, a partial group's
    step by step with both in one accumulation, and the two round differently."""
    import ref_numpy as R
    from linmt_amd import lib as lh
    L = lh.load()
    rng = np.random.default_rng(7)
    sentences = 0
    try:
        L.lh_gemm_set_config_override(7)
        L.lh_gemm_set_splits_override(1)
        for trial in range(40):
            layers = int(rng.integers(1, 5)); H = int(rng.choice([32, 48, 64, 100, 128]))
            Vs = int(rng.integers(30, 300)); Vt = int(rng.integers(40, 500))
            D = int(rng.integers(1, 11)); beam = int(rng.integers(2, 13)); slots = int(rng.integers(1, 9))
            feed = bool(rng.integers(0, 2)); scale = float(rng.choice([0.2, 0.4, 0.8]))
            beam = min(beam, int(np.sqrt(Vt)))
            P = R.make_params(rng, layers, H, Vs, Vt, attention=True, feed_input=feed, scale=scale)
            n = int(rng.integers(1, 6 * slots + 2))
            sents = [rng.integers(0, Vs, size=int(rng.integers(1, 25))) for _ in range(n)]
            gm = host.Model(layers, H, Vs, Vt, longest_sentence=44, attention_mode=1, attention_width=D,
                            feed_input=feed, decoding=(slots, beam))
            gm.set_params(P)
            got = gm.decode_stream(sents, beam=beam, with_hyps=True)
            order = sorted(range(n), key=lambda i: -len(sents[i]))  # stable, as the stream's
            for g0 in range(0, n, slots):
                group = order[g0:g0 + slots]
                want = gm.decode_batch([sents[i] for i in group], beam=beam, with_hyps=True)
                for w, i in zip(want, group):
                    what = (f"trial {trial} (layers {layers}, H {H}, beam {beam}, slots {slots}, n {n}, "
                            f"feed {feed}, scale {scale}) sentence {i} (len {len(sents[i])})")
                    assert got[i]["steps"] == w["steps"], what
                    assert got[i]["best"].tolist() == w["best"].tolist(), what
                    assert got[i]["best_score"] == w["best_score"], what
                    assert len(got[i]["hyps"]) == len(w["hyps"]), what
                    for (gt, gs), (wt, ws) in zip(got[i]["hyps"], w["hyps"]):
                        assert gt.tolist() == wt.tolist() and gs == ws, what
            sentences += n
            gm.close()
    finally:
        L.lh_gemm_set_config_override(-1)
        L.lh_gemm_set_splits_override(0)
    assert sentences > 500


def test_decode_batch_equals_lone_sentences_bit_for_bit(host):
    """The same statement for DecodeBatch: a sentence decoded among others (shorter and longer ones,
    which leave the batch before and after it) gets exactly what it gets alone, one tile shape
    forced as above.  Batches stay one short of n_sent so that both runs take the encoder step by
    step."""
    import ref_numpy as R
    from linmt_amd import lib as lh
    L = lh.load()
    rng = np.random.default_rng(11)
    sentences = 0
    try:
        L.lh_gemm_set_config_override(7)
        L.lh_gemm_set_splits_override(1)
        for trial in range(20):
            layers = int(rng.integers(1, 5)); H = int(rng.choice([32, 48, 64, 100, 128]))
            Vs = int(rng.integers(30, 300)); Vt = int(rng.integers(40, 500))
            D = int(rng.integers(0, 11)); beam = int(rng.integers(2, 13)); slots = int(rng.integers(3, 9))
            att = 1 if D else 0
            feed = bool(att and rng.integers(0, 2)); scale = float(rng.choice([0.2, 0.4, 0.8]))
            beam = min(beam, int(np.sqrt(Vt)))
            P = R.make_params(rng, layers, H, Vs, Vt, attention=bool(att), feed_input=feed, scale=scale)
            n = int(rng.integers(2, slots))
            sents = [rng.integers(0, Vs, size=int(rng.integers(1, 25))) for _ in range(n)]
            gm = host.Model(layers, H, Vs, Vt, longest_sentence=44, attention_mode=att, attention_width=max(D, 1),
                            feed_input=feed, decoding=(slots, beam))
            gm.set_params(P)
            got = gm.decode_batch(sents, beam=beam, with_hyps=True)
            for i, s in enumerate(sents):
                w = gm.decode_batch([s], beam=beam, with_hyps=True)[0]
                what = (f"trial {trial} (layers {layers}, H {H}, beam {beam}, n_sent {slots}, n {n}, attention {att}, "
                        f"feed {feed}, scale {scale}) sentence {i} (len {len(s)})")
                assert got[i]["steps"] == w["steps"], what
                assert got[i]["best"].tolist() == w["best"].tolist(), what
                assert got[i]["best_score"] == w["best_score"], what
                assert len(got[i]["hyps"]) == len(w["hyps"]), what
                for (gt, gs), (wt, ws) in zip(got[i]["hyps"], w["hyps"]):
                    assert gt.tolist() == wt.tolist() and gs == ws, what
            sentences += n
            gm.close()
    finally:
        L.lh_gemm_set_config_override(-1)
        L.lh_gemm_set_splits_override(0)
    assert sentences > 50


def test_decode_batch_ensemble_and_alignments_equal_lone_sentences_bit_for_bit(host):
    """The same for two models decoded in lockstep (each on its own stream, their distributions
    averaged by the top-k kernel) with exported alignments: tokens, finished hypotheses, score
    bits and the 1-best's source positions of a sentence do not depend on its neighbours."""
    import ref_numpy as R
    from linmt_amd import lib as lh
    L = lh.load()
    rng = np.random.default_rng(12)
    sentences = 0
    try:
        L.lh_gemm_set_config_override(7)
        L.lh_gemm_set_splits_override(1)
        for trial in range(8):
            layers = int(rng.integers(1, 4)); H = int(rng.choice([32, 48, 64, 100]))
            Vs = int(rng.integers(30, 200)); Vt = 4 * int(rng.integers(10, 75))  # ensembles: a multiple of 4
            D = int(rng.integers(1, 8)); beam = int(rng.integers(2, 9)); slots = int(rng.integers(3, 7))
            feed = bool(rng.integers(0, 2)); scale = float(rng.choice([0.2, 0.4]))
            beam = min(beam, int(np.sqrt(Vt)))
            gms = []
            for _ in range(2):
                P = R.make_params(rng, layers, H, Vs, Vt, attention=True, feed_input=feed, scale=scale)
                gm = host.Model(layers, H, Vs, Vt, longest_sentence=44, attention_mode=1, attention_width=D,
                                feed_input=feed, decoding=(slots, beam))
                gm.set_params(P)
                gms.append(gm)
            n = int(rng.integers(2, slots))
            sents = [rng.integers(0, Vs, size=int(rng.integers(1, 25))) for _ in range(n)]
            got = gms[0].decode_batch(sents, beam=beam, with_hyps=True, ensemble=gms[1:], alignments=True)
            for i, s in enumerate(sents):
                w = gms[0].decode_batch([s], beam=beam, with_hyps=True, ensemble=gms[1:], alignments=True)[0]
                what = f"trial {trial} (layers {layers}, H {H}, beam {beam}, n_sent {slots}, n {n}, feed {feed}) sentence {i}"
                assert got[i]["steps"] == w["steps"], what
                assert got[i]["best"].tolist() == w["best"].tolist(), what
                assert got[i]["best_score"] == w["best_score"], what
                assert got[i]["best_viterbi"].tolist() == w["best_viterbi"].tolist(), what
                assert len(got[i]["hyps"]) == len(w["hyps"]), what
                for (gt, gs), (wt, ws) in zip(got[i]["hyps"], w["hyps"]):
                    assert gt.tolist() == wt.tolist() and gs == ws, what
            sentences += n
            for gm in gms:
                gm.close()
    finally:
        L.lh_gemm_set_config_override(-1)
        L.lh_gemm_set_splits_override(0)
    assert sentences >= 16


@pytest.mark.parametrize("feed", [False, True])
def test_decode_stream_at_the_longest_sentence_length(orc, host, feed):
    """Sentences as long as the model allows: their step count is cut at longest_sentence - 2
    (decoder.h:1734) instead of 1.5 x length, next to one-word sentences that leave their slot
    after two steps.  Against the oracle's single-sentence search."""
    rng = np.random.default_rng(5 + int(feed))
    layers, H, Vs, Vt, D, beam, slots, longest = 2, 32, 50, 60, 3, 4, 3, 20
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, longest, 0.4, decoding=(slots, beam), feed=feed)
    sents = [rng.integers(0, Vs, size=int(rng.choice([20, 20, 19, 14, 1, 13]))) for _ in range(11)]
    sents[0] = rng.integers(0, Vs, size=20)
    sents[1] = rng.integers(0, Vs, size=1)
    got = gm.decode_stream(sents, beam=beam, with_hyps=True)
    for i, s in enumerate(sents):
        want = om.decode_sentence(s, beam=beam)
        assert want["steps"] == (19 if len(s) >= 13 else 2)
        _compare_decode(want, got[i], f"sentence {i} (len {len(s)})")
    gm.close()


@pytest.mark.parametrize("layers,H,Vs,Vt,D,beam,slots,n,feed,seed", [
    (2, 64, 120, 150, 3, 4, 3, 11, True, 21),
    (1, 48, 60, 90, 10, 5, 2, 7, False, 22),
])
def test_decode_stream_exported_alignments_and_kbest_vs_oracle(orc, host, layers, H, Vs, Vt, D, beam, slots,
                                                                n, feed, seed):
    """The reference's unk_replacement_mode__ through the stream: every tick's alignments and window
    indices go into a history, hypotheses carry the Viterbi alignment of every token and the
    coverage penalty is computed from the exported scores (src/decoder.h:529-600,1933-1961,
    src/layer_attention.h:342-386).  1-best, its alignments and its rescored value must be the
    oracle's; a k-best list must be DecodeBatch's for the same sentences."""
    rng = np.random.default_rng(seed)
    P, om, gm = _pair(orc, host, rng, layers, H, Vs, Vt, D, 40, 0.4, decoding=(slots, beam), feed=feed)
    sents = [rng.integers(0, Vs, size=int(rng.integers(1, 16))) for _ in range(n)]
    got = gm.decode_stream(sents, beam=beam, with_hyps=True, alignments=True)
    for i, s in enumerate(sents):
        want = om.decode_sentence(s, beam=beam, alignments=True)
        _compare_decode(want, got[i], f"sentence {i} (len {len(s)})")
        assert got[i]["best_viterbi"].tolist() == want["best_viterbi"].tolist(), i
    # k-best lists: the same indices and scores as batch by batch, with and without alignments
    for align in (False, True):
        ks = gm.decode_stream(sents, beam=beam, alignments=align, num_hypotheses=3)
        order = sorted(range(n), key=lambda i: -len(sents[i]))
        for g0 in range(0, n, slots):
            group = order[g0:g0 + slots]
            kb = gm.decode_batch([sents[i] for i in group], beam=beam, alignments=align, num_hypotheses=3)
            for w, i in zip(kb, group):
                assert [k for k, _ in ks[i]["kbest"]] == [k for k, _ in w["kbest"]], (align, i)
                assert np.allclose([v for _, v in ks[i]["kbest"]], [v for _, v in w["kbest"]], rtol=1e-4, atol=1e-4)
                assert ks[i]["best"].tolist() == w["best"].tolist(), (align, i)
    gm.close()


def test_decode_stream_ensemble_vs_oracle(orc, host):
    """EnsembleFactory with several models through the stream: models of different width, depth,
    attention window and input feeding decode a list in lockstep, each on its own streams with its
    own encoder, attention memories and states, their distributions averaged before every beam step
    (lh_beam_topk_ensemble_f32; src/decoder.h:1702-1776,1910-1965) -- a list several times the
    slots long, against the oracle's ensemble search, with and without exported alignments (added up
    over the models).  Afterwards every model still decodes on its own, in both drivers."""
    rng = np.random.default_rng(31)
    Vs, Vt, beam, slots = 60, 72, 4, 3
    shapes = ((2, 48, 2, True), (1, 32, 3, False), (3, 40, 10, True))  # layers, H, D, input feeding
    pairs = [_pair(orc, host, rng, L, H, Vs, Vt, D, 30, 0.4, decoding=(slots, beam), feed=feed)
             for L, H, D, feed in shapes]
    oms, gms = [p[1] for p in pairs], [p[2] for p in pairs]
    sents = [rng.integers(0, Vs, size=int(rng.integers(1, 14))) for _ in range(13)]
    for n_models in (2, 3):
        for kw in (dict(), dict(alignments=True, cp_beta=0.6, lp_alpha=0.3)):
            got = gms[0].decode_stream(sents, beam=beam, with_hyps=True, ensemble=gms[1:n_models], **kw)
            for i, s in enumerate(sents):
                want = oms[0].decode_sentence(s, beam=beam, ensemble=tuple(oms[1:n_models]), **kw)
                _compare_decode(want, got[i], f"{n_models} models {kw} sentence {i} (len {len(s)})")
                if kw:
                    assert got[i]["best_viterbi"].tolist() == want["best_viterbi"].tolist(), (i, n_models)
    for om, gm in zip(oms, gms):
        alone = gm.decode_stream(sents[:5], beam=beam, with_hyps=True)
        batch = gm.decode_batch(sents[:3], beam=beam, with_hyps=True)
        for i in range(5):
            _compare_decode(om.decode_sentence(sents[i], beam=beam), alone[i], f"alone, sentence {i}")
        for i in range(3):
            _compare_decode(om.decode_sentence(sents[i], beam=beam), batch[i], f"alone, batch, sentence {i}")
    with pytest.raises(host.HostError):
        gms[0].decode_stream(sents, beam=beam, ensemble=[gms[0]])
    for g in gms:
        g.close()
