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
