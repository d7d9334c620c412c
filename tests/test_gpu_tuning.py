"""The training-loop harness (Dispatcher::Tuning, src/dispatcher.cu:96-384) end to end on the GPU:
a synthetic "copy the source with an offset" corpus written in the reference's training-file format,
the three learning-rate schedules checked against the rule stated in the reference, dev perplexity
against the model's own GetError, model files written by the loop loadable again."""
import os

import numpy as np
import pytest

import ref_numpy as R

pytestmark = pytest.mark.gpu
B, VS, VT, H = 4, 12, 15, 24


@pytest.fixture(scope="module")
def host():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from linmt_amd import host as h
    h.load()
    return h


def _write_corpus(path, rng, n_batches):
    """Each minibatch of B pairs is padded to common lengths, as the reference's preprocessor leaves
    it: source reversed + left-padded, target right-padded."""
    pairs = []
    with open(path, "w") as f:
        for _ in range(n_batches):
            lens = rng.integers(2, 6, size=B)
            S, T = int(lens.max()), int(lens.max()) + 1
            for n in lens:
                src = rng.integers(1, VS, size=n)
                tgt = src + 3  # ids >= 3 on the target side
                s_line = [-1] * (S - n) + src[::-1].tolist()
                t_in = [0] + tgt.tolist() + [-1] * (T - n - 1)
                t_out = tgt.tolist() + [1] + [-1] * (T - n - 1)
                f.write(" ".join(map(str, s_line)) + "\n" + " ".join(["-2"] * S) + "\n" +
                        " ".join(map(str, t_in)) + "\n" + " ".join(map(str, t_out)) + "\n")
                pairs.append((np.array(s_line), np.array(t_in), np.array(t_out)))
    return pairs


def _model(host, lr=0.5, scoring=False):
    kw = dict(longest_sentence=12, attention_mode=1, attention_width=2, feed_input=True, minibatch_size=B)
    if scoring:
        return host.Model(1, H, VS, VT, **kw)
    return host.Model(1, H, VS, VT, training=dict(learning_rate=lr, grad_clip_mode=2, norm_clip=5.0), **kw)


def test_perplexity_falls_and_files_round_trip(host, tmp_path):
    rng = np.random.default_rng(3)
    train, dev = str(tmp_path / "train.txt"), str(tmp_path / "dev.txt")
    _write_corpus(train, rng, 24)
    dev_pairs = _write_corpus(dev, rng, 2)
    P = R.make_params(rng, 1, H, VS, VT, attention=True, feed_input=True, scale=0.1)
    m = _model(host)
    m.set_params(P)

    # GetPerplexity = exp(-sum log p / target input words), with the sum from GetError per minibatch
    total, words = 0.0, 0
    for k in range(0, len(dev_pairs), B):
        chunk = dev_pairs[k:k + B]
        src = np.stack([c[0] for c in chunk]); tin = np.stack([c[1] for c in chunk]); tout = np.stack([c[2] for c in chunk])
        lens = (src != -1).sum(axis=1)
        total += m.get_error(src, tin, tout, np.concatenate([lens, src.shape[1] - lens]))
        words += int((tin != -1).sum())
    before = m.get_perplexity(dev)
    assert np.isclose(before, np.exp(-total / words), rtol=1e-6)

    final, best = str(tmp_path / "final.nmt"), str(tmp_path / "best.nmt")
    rep = m.tuning(train, dev_file=dev, output_weight_file=final, best_model_file=best, epochs=12,
                   learning_rate_schedule=True, best_model_mode=True, screen_print_rate=10)
    kinds = [e[0] for e in rep["events"]]
    assert kinds.count("epoch_end") == 12 and kinds.count("epoch_perplexity") == 12
    assert kinds.count("half_epoch_perplexity") == 12 and kinds[-1] == "dump_final"
    perp = [e[3] for e in rep["events"] if e[0] == "epoch_perplexity"]
    assert min(perp) < 0.7 * before, (before, perp)
    loglik = [e[3] for e in rep["events"] if e[0] == "epoch_end"]
    assert loglik[-1] > loglik[0]
    assert rep["words"] > 0 and rep["seconds"] > 0
    speed = [e for e in rep["events"] if e[0] == "speed"]
    assert len(speed) == 12 * 3  # 24 minibatches per epoch: after 10, after 20 and at the epoch's end
    # the last dump of the best model holds the parameters of that moment: its dev perplexity is
    # the one the event reports (up to the 8 digits of the file)
    dumps = [e for e in rep["events"] if e[0] == "dump_best_model"]
    assert dumps and all(b[3] < a[3] for a, b in zip(dumps, dumps[1:]))
    s = _model(host, scoring=True)
    s.load_weights(best)
    assert np.isclose(s.get_perplexity(dev), dumps[-1][3], rtol=1e-4)
    s.load_weights(final)
    assert np.isclose(s.get_perplexity(dev), m.get_perplexity(dev), rtol=1e-4)
    info = host.read_model_information(final)
    assert (info["num_layers"], info["lstm_size"], info["attention_model"], info["feed_input"]) == (1, H, 1, 1)


@pytest.mark.parametrize("mode", ["google", "stanford", "schedule_stall"])
def test_learning_rate_schedules(host, tmp_path, mode):
    rng = np.random.default_rng(4)
    train, dev = str(tmp_path / "train.txt"), str(tmp_path / "dev.txt")
    _write_corpus(train, rng, 4)
    _write_corpus(dev, rng, 1)
    lr0, epochs = 0.25, 4
    m = _model(host, lr=lr0)
    m.set_params(R.make_params(rng, 1, H, VS, VT, attention=True, feed_input=True, scale=0.1))
    if mode == "google":
        rep = m.tuning(train, epochs=epochs, google_learning_rate=True, epoch_to_start_halving=3)
        # one halving when epoch 3 starts, at its half, when epoch 4 starts, at its half, and when
        # the epoch counter passes the last epoch (the reference halves there too)
        want = [lr0 / 2 ** k for k in range(1, 6)]
    elif mode == "stanford":
        rep = m.tuning(train, epochs=epochs, stanford_learning_rate=True, epoch_to_start_halving_full=2)
        want = [lr0 / 2 ** k for k in range(1, 5)]  # when epochs 2, 3, 4 and "5" start
    else:
        # an unreachable margin makes every evaluation after epoch 1 count as a stall
        rep = m.tuning(train, dev_file=dev, epochs=epochs, learning_rate_schedule=True, margin=1e9,
                       decrease_factor=0.7)
        # evaluations: half + end of each epoch; all but the half-epoch one of epoch 1 see
        # current_epoch != 1 (the end-of-epoch one runs after the counter moved to 2)
        want = [lr0 * 0.7 ** k for k in range(1, 2 * epochs)]
    got = [e[3] for e in rep["events"] if e[0] == "learning_rate"]
    assert np.allclose(got, want, rtol=1e-6), (got, want)
    assert np.isclose(rep["final_learning_rate"], want[-1], rtol=1e-6)


@pytest.mark.parametrize("schedule", ["dev_perplexity", "google"])
def test_training_run_from_a_file_against_the_oracles_loop(orc, host, tmp_path, schedule):
    """FileHelper -> Dispatcher::Tuning -> ComputeGradients / UpdateWeights on the HIP path against
    the oracle's own loop over the same file (oracle/orc.py Model.tuning and TrainingFile, written
    from src/dispatcher.cu:96-384 and src/file_helper.cc:113-381 and pinned in
    tests/test_oracle_tuning_pins.py): three epochs of 12 minibatches.  The learning-rate events
    must be the same events at the same minibatches with the same values, every dev perplexity
    within 1e-4 relative, the summed training log-likelihood of every epoch within 1e-4 relative,
    and the parameters at the end within rtol 1e-4 / atol 2e-6."""
    rng = np.random.default_rng(8)
    train, dev = str(tmp_path / "train.txt"), str(tmp_path / "dev.txt")
    _write_corpus(train, rng, 12)
    _write_corpus(dev, rng, 2)
    P = R.make_params(rng, 1, H, VS, VT, attention=True, feed_input=True, scale=0.1)
    lr0, epochs = 0.5, 3
    if schedule == "dev_perplexity":
        # a margin that some evaluations pass and others do not: both branches of the stall rule
        kw = dict(dev_file=dev, learning_rate_schedule=True, margin=0.35, decrease_factor=0.6)
    else:
        kw = dict(google_learning_rate=True, epoch_to_start_halving=2)
    m = _model(host, lr=lr0)
    m.set_params(P)
    rep = m.tuning(train, epochs=epochs, **kw)
    om = orc.Model(1, H, VS, VT, attention=1, D=2, feed_input=1, longest_sent=12)
    om.set_params(P)
    want, want_lr = om.tuning(train, B, lr0, epochs, clip_mode=2, norm_clip=5.0, **kw)

    kinds = ("learning_rate", "half_epoch_perplexity", "epoch_perplexity", "epoch_end")
    got = [e for e in rep["events"] if e[0] in kinds]
    assert [e[:3] for e in got] == [tuple(e[:3]) for e in want], (got, want)
    for g, w in zip(got, want):
        tol = 1e-6 if g[0] == "learning_rate" else 1e-4
        assert abs(g[3] - w[3]) <= tol * abs(w[3]), (g, w)
    assert np.isclose(rep["final_learning_rate"], want_lr, rtol=1e-6)
    rates = [e[3] for e in want if e[0] == "learning_rate"]
    if schedule == "dev_perplexity":
        n_eval = sum(1 for e in want if "perplexity" in e[0])
        assert n_eval == 2 * epochs and 0 < len(rates) < n_eval - 1  # the rule fired and did not fire
    else:
        assert len(rates) == 5  # epochs 2 and 3: at the start and the half; once more past the last epoch
    for name in om.param_names():
        w = om.get_param(name)
        shape = w.shape if w.ndim == 2 else (w.size,)
        got_p = m.get_param(name, shape)
        assert np.allclose(got_p, w.reshape(shape, order="F"), rtol=1e-4, atol=2e-6), name
    assert not np.array_equal(m.get_param("tgt.0.W_hi", (H, H)), P["tgt.0.W_hi"])
    m.close()
