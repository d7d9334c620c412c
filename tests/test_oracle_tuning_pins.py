"""Pins of the oracle's training-file reader and training loop (oracle/orc.py: TrainingFile,
Model.tuning, Model.get_perplexity -- restatements of FileHelper::ReadMinibatch,
src/file_helper.cc:113-381, Dispatcher::Tuning, src/dispatcher.cu:96-384, and
NeuralMachineTranslation::GetPerplexity, src/deep_rnn.h:1490-1568).  CPU only.

  * the reader against the committed hand-made file and expectations written from the format's
    definition (transposes, counts, first occurrences), and against the host library's FileHelper,
    an independent implementation of the same format in another language;
  * the schedules against event lists written out by hand from the rule in the reference;
  * the perplexity against its definition on the independent float64 numpy model;
  * the loop's effect on the parameters against a plain "gradient step per minibatch" written here
    with the oracle's own compute_gradients / update_weights (both pinned elsewhere), i.e. that the
    loop feeds every minibatch once, in file order, with the learning rate of the moment."""
import os

import numpy as np
import pytest

import ref_numpy as R

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
B, VS, VT, H = 4, 12, 15, 24


def write_corpus(path, rng, n_batches, batch=B, vs=VS):
    """Minibatches of `batch` pairs padded to common lengths, as the reference's preprocessor leaves
    them: source reversed + left-padded, target right-padded; the task is "source + 3"."""
    pairs = []
    with open(path, "w") as f:
        for _ in range(n_batches):
            lens = rng.integers(2, 6, size=batch)
            S, T = int(lens.max()), int(lens.max()) + 1
            for n in lens:
                src = rng.integers(1, vs, size=n)
                tgt = src + 3
                s_line = [-1] * (S - n) + src[::-1].tolist()
                t_in = [0] + tgt.tolist() + [-1] * (T - n - 1)
                t_out = tgt.tolist() + [1] + [-1] * (T - n - 1)
                f.write(" ".join(map(str, s_line)) + "\n" + " ".join(["-2"] * S) + "\n" +
                        " ".join(map(str, t_in)) + "\n" + " ".join(map(str, t_out)) + "\n")
                pairs.append((np.array(s_line), np.array(t_in), np.array(t_out)))
    return pairs


def test_training_file_reader_against_the_format_and_the_host_reader(orc):
    path = os.path.join(GOLDEN, "train_minibatches.txt")
    lines = open(path).read().split("\n")
    pairs = [tuple(np.array(lines[k + d].split(), dtype=np.int64) for d in (0, 2, 3))
             for k in range(0, len(lines) - 1, 4)]
    f = orc.TrainingFile(path, 2)
    assert f.total_words == sum(int((p[0] != -1).sum() + (p[1] != -1).sum()) for p in pairs)
    assert f.total_target_words == sum(int((p[1] != -1).sum()) for p in pairs)
    from linmt_amd import host
    fh = host.FileHelper(path, 2, 12, 10, 12)
    n_batches = len(pairs) // 2
    for rep in range(2):
        for b in range(n_batches):
            mb, same = f.read_minibatch()
            chunk = pairs[2 * b:2 * b + 2]
            assert same == (b != n_batches - 1)
            assert np.array_equal(mb["src"], np.stack([p[0] for p in chunk]))
            assert np.array_equal(mb["tgt_in"], np.stack([p[1] for p in chunk]))
            assert np.array_equal(mb["tgt_out"], np.stack([p[2] for p in chunk]))
            lengths = (mb["src"] != -1).sum(axis=1)
            assert mb["batch_info"].tolist() == lengths.tolist() + (mb["src"].shape[1] - lengths).tolist()
            for key, block in (("src_wgrad", mb["src"]), ("tgt_wgrad", mb["tgt_in"])):
                flat = block.ravel(order="F")
                assert sorted(mb[key].tolist()) == sorted(set(flat[flat != -1].tolist()))
            same_h, hb = fh.read_minibatch()
            assert same_h == same
            assert np.array_equal(hb["source_in"], mb["src"]) and np.array_equal(hb["target_out"], mb["tgt_out"])
            assert hb["source_wgrad"].tolist() == mb["src_wgrad"].tolist()
            assert hb["target_wgrad"].tolist() == mb["tgt_wgrad"].tolist()
            assert hb["batch_information"].tolist() == mb["batch_info"].tolist()
            assert hb["words_in_minibatch"] == mb["words_in_minibatch"]
    fh.close()


def _oracle(orc, P):
    om = orc.Model(1, H, VS, VT, attention=1, D=2, feed_input=1, longest_sent=12)
    om.set_params(P)
    return om


@pytest.mark.parametrize("mode", ["google", "stanford", "schedule_stall"])
def test_schedules_against_the_rule_written_out_by_hand(orc, tmp_path, mode):
    rng = np.random.default_rng(4)
    train, dev = str(tmp_path / "train.txt"), str(tmp_path / "dev.txt")
    write_corpus(train, rng, 4)
    write_corpus(dev, rng, 1)
    lr0, epochs = 0.25, 4
    om = _oracle(orc, R.make_params(rng, 1, H, VS, VT, attention=True, feed_input=True, scale=0.1))
    if mode == "google":
        ev, lr = om.tuning(train, B, lr0, epochs, google_learning_rate=True, epoch_to_start_halving=3)
        # when epoch 3 starts, at its half, when epoch 4 starts, at its half, and when the counter
        # passes the last epoch (src/dispatcher.cu:228-236,283-291)
        want = [lr0 / 2 ** k for k in range(1, 6)]
    elif mode == "stanford":
        ev, lr = om.tuning(train, B, lr0, epochs, stanford_learning_rate=True, epoch_to_start_halving_full=2)
        want = [lr0 / 2 ** k for k in range(1, 5)]  # when epochs 2, 3, 4 and "5" start (:293-301)
    else:
        ev, lr = om.tuning(train, B, lr0, epochs, dev_file=dev, learning_rate_schedule=True, margin=1e9,
                           decrease_factor=0.7)
        # every evaluation but the half-epoch one of epoch 1 sees current_epoch != 1 (:253,:318)
        want = [lr0 * 0.7 ** k for k in range(1, 2 * epochs)]
        assert [e[0] for e in ev if "perplexity" in e[0]] == ["half_epoch_perplexity", "epoch_perplexity"] * epochs
    got = [e[3] for e in ev if e[0] == "learning_rate"]
    assert np.allclose(got, want, rtol=1e-6), (got, want)
    assert np.isclose(lr, want[-1], rtol=1e-6)
    assert [e[1] for e in ev if e[0] == "epoch_end"] == list(range(1, epochs + 1))


def test_perplexity_against_its_definition_on_the_numpy_model(orc, tmp_path):
    rng = np.random.default_rng(5)
    dev = str(tmp_path / "dev.txt")
    pairs = write_corpus(dev, rng, 2)
    P = R.make_params(rng, 1, H, VS, VT, attention=True, feed_input=True, scale=0.2)
    om = _oracle(orc, P)
    # the file's pairs as the numpy model takes them: source in reading order, target without
    # <START> / <EOF>
    sents = [(c[0][c[0] != -1][::-1], c[2][(c[2] != -1) & (c[2] != 1)]) for c in pairs]
    total = R.minibatch_loglik(P, 1, H, 2, sents, attention=True, feed_input=True)
    words = sum(int((c[1] != -1).sum()) for c in pairs)
    assert np.isclose(om.get_perplexity(dev, B), np.exp(-total / words), rtol=1e-5)


def test_loop_is_one_gradient_step_per_minibatch_in_file_order(orc, tmp_path):
    rng = np.random.default_rng(6)
    train = str(tmp_path / "train.txt")
    pairs = write_corpus(train, rng, 3)
    P = R.make_params(rng, 1, H, VS, VT, attention=True, feed_input=True, scale=0.1)
    a, b = _oracle(orc, P), _oracle(orc, P)
    ev, lr = a.tuning(train, B, 0.5, 2, stanford_learning_rate=True, epoch_to_start_halving_full=2)
    assert lr == 0.125
    for epoch, rate in ((1, 0.5), (2, 0.25)):
        for k in range(0, len(pairs), B):
            chunk = pairs[k:k + B]
            src = np.stack([c[0] for c in chunk]); tin = np.stack([c[1] for c in chunk]); tout = np.stack([c[2] for c in chunk])
            lens = (src != -1).sum(axis=1)
            su = np.unique(src[src != -1]).astype(np.int32)
            tu = np.unique(tin[tin != -1]).astype(np.int32)
            b.compute_gradients(src, tin, tout, np.concatenate([lens, src.shape[1] - lens]), su, tu)
            b.update_weights(rate, 2, 5.0, 0.0, B)
    for name in a.param_names():
        # the order of the unique-id lists differs (sorted here, first occurrence in the loop): the
        # embedding columns are updated independently of one another, so the result is the same
        assert np.array_equal(a.get_param(name), b.get_param(name)), name


def test_model_file_writer_and_reader_against_the_hand_made_file(orc, tmp_path):
    """oracle/orc.py write_model_file / read_model_file (written from src/deep_rnn.h:1878-2146,
    src/deep_rnn_kernel.h:1543-1578, src/layer_input_to_hidden.h:1556-1590) against
    tests/golden/tiny_model.nmt, the hand-made file whose k-th matrix holds k + i/10 + j/100: the
    reader must find every matrix where an independent walk of the order puts it, and the writer's
    file, read back token by token, must have the hand-made file's lines, mappings and numbers."""
    path = os.path.join(GOLDEN, "tiny_model.nmt")
    info, P = orc.read_model_file(path)
    assert (info["layers"], info["H"], info["Vs"], info["Vt"], info["attention"], info["feed_input"]) == (2, 3, 5, 6, 1, 1)
    assert info["source_words"] == ["<UNK>", "s1", "s2", "s3", "s4"]
    assert info["target_words"] == ["<START>", "<EOF>", "<UNK>", "t3", "t4", "t5"]
    L, H, Vt, Vs = 2, 3, 6, 5
    names = []
    for side, vocab, feed in (("src", Vs, False), ("tgt", Vt, True)):
        for l in range(L):
            p = f"{side}.{l}."
            for g in "ifco":
                names += [(p + "W_h" + g, (H, H)), (p + "b_" + g, (H, 1))]
            if l == 0:
                names.append((p + "W", (H, vocab)))
            names += [(p + "M_" + g, (H, H)) for g in "ifoc"]
            if feed and l == 0:
                names += [(p + "Q_" + g, (H, H)) for g in "ifoc"]
    names += [("attn.W_a", (H, H)), ("attn.W_p", (H, H)), ("attn.v_p", (H, 1)), ("attn.b_out", (H, 1)),
              ("attn.W_c1", (H, H)), ("attn.W_c2", (H, H)), ("softmax.D", (Vt, H)), ("softmax.b_d", (Vt, 1))]
    assert len(names) == len(P)
    for k, (name, (r, c)) in enumerate(names):
        want = (k + np.arange(r)[:, None] / 10 + np.arange(c)[None, :] / 100).astype(np.float32)
        assert np.array_equal(P[name].reshape(r, c), want), name
    out = str(tmp_path / "again.nmt")
    orc.write_model_file(out, P, 2, 3, 5, 6, 1, 1, info["source_words"], info["target_words"])
    a, b = open(path).read().split("\n"), open(out).read().split("\n")
    assert len(a) == len(b)
    for la, lb in zip(a, b):
        ta, tb = la.split(), lb.split()
        assert len(ta) == len(tb), (la, lb)
        for x, y in zip(ta, tb):
            try:
                assert np.float32(float(x)) == np.float32(float(y)), (la, lb)
            except ValueError:
                assert x == y, (la, lb)
    # eight significant digits in printf's %g form: no trailing zeros, exponent form for small numbers
    tiny = {k: v.copy() for k, v in P.items()}
    tiny["softmax.b_d"][:3] = np.float32([1.0, 0.1, 2.0 ** -23])
    orc.write_model_file(out, tiny, 2, 3, 5, 6, 1, 1)
    tail = open(out).read().split("\n")[-8:-2]
    assert tail[:3] == ["1", "0.1", "1.1920929e-07"]
