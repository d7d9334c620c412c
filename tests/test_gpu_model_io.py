"""The reference's text model file through the C++ layer classes: LoadWeights on a hand-made file
whose numbers say which matrix / row / column they are (tests/golden/tiny_model.nmt), and
DumpModel -> LoadWeights round trips.  The matrix order checked here is the one the reference's
DumpWeightsGpu functions write (layer_input_to_hidden.h:1556-1590: W_h*/b_* interleaved, W, then
M_i M_f M_o M_c, then Q_i Q_f Q_o Q_c; attention after the last target layer; softmax last).
Parity unpinned against a reference-written model file: the checkout holds none."""
import os

import numpy as np
import pytest

import ref_numpy as R

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def host():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from linmt_amd import host as h
    h.load()
    return h


def test_load_weights_puts_every_matrix_where_the_reference_order_says(host):
    L, H, Vt, Vs = 2, 3, 6, 5
    m = host.Model(L, H, Vs, Vt, longest_sentence=10, attention_mode=1, attention_width=2,
                   feed_input=True, minibatch_size=2)
    m.load_weights(os.path.join(GOLDEN, "tiny_model.nmt"))
    # the file's k-th matrix holds k + i/10 + j/100 at (i, j); walk the order independently
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
    assert [(n, r, c) for n, (r, c) in names] == m.model_file_order()
    for k, (name, (r, c)) in enumerate(names):
        want = k + np.arange(r)[:, None] / 10 + np.arange(c)[None, :] / 100
        got = m.get_param(name, (r, c))
        assert np.allclose(got, want, rtol=0, atol=1e-5), name


@pytest.mark.parametrize("layers,attention,feed,s2s", [(1, 1, True, True), (3, 1, False, True),
                                                       (2, 0, False, True), (2, 0, False, False)])
def test_dump_then_load_round_trip(host, tmp_path, layers, attention, feed, s2s):
    rng = np.random.default_rng(5)
    H, Vs, Vt = 8, 11, 13
    P = R.make_params(rng, layers, H, Vs, Vt, attention=bool(attention), feed_input=feed, scale=0.5)
    if not s2s:
        P = {k: v for k, v in P.items() if not k.startswith("src.")}
    kw = dict(longest_sentence=12, attention_mode=attention, attention_width=3, feed_input=feed,
              minibatch_size=2, sequence_to_sequence=s2s)
    a = host.Model(layers, H, Vs, Vt, **kw)
    a.set_params(P)
    path = str(tmp_path / "model.nmt")
    a.dump_model(path)
    info = host.read_model_information(path)
    assert (info["num_layers"], info["lstm_size"], info["target_vocab_size"]) == (layers, H, Vt)
    assert info["attention_model"] == int(bool(attention)) and info["feed_input"] == int(feed)
    b = host.Model(layers, H, Vs, Vt, **kw)
    b.load_weights(path)
    for name, arr in P.items():
        got = b.get_param(name, np.atleast_2d(arr.reshape(arr.shape[0], -1)).shape)
        # the reference writes digits10 + 2 = 8 significant digits
        assert np.allclose(got, arr.reshape(got.shape), rtol=1e-7, atol=0), name
    # a file for another architecture is refused
    c = host.Model(layers + 1, H, Vs, Vt, **kw)
    with pytest.raises(host.HostError):
        c.load_weights(path)


def test_decoding_a_text_file(host, tmp_path):
    """Dispatcher::Decoding end to end: model file + source text -> ids file -> words, in batches,
    with the decoding-information fields; the ids and alignments must be the ones DecodeBatch gives
    for the same sentences on a model loaded from the same file."""
    rng = np.random.default_rng(8)
    layers, H, Vs, Vt, D, beam = 2, 24, 30, 40, 2, 4
    P = R.make_params(rng, layers, H, Vs, Vt, attention=True, feed_input=True, scale=0.5)
    kw = dict(longest_sentence=24, attention_mode=1, attention_width=D, feed_input=True)
    a = host.Model(layers, H, Vs, Vt, minibatch_size=1, **kw)
    a.set_params(P)
    model = str(tmp_path / "model.nmt")
    a.dump_model(model)  # placeholder vocabularies: source <UNK> w1.., target <START> <EOF> <UNK> w3..

    lens = [5, 1, 9, 3, 7, 2, 6]
    sents = [rng.integers(0, Vs, size=n) for n in lens]
    word = lambda i: "<UNK>" if i == 0 else f"w{i}"  # noqa: E731
    lines = [" ".join(word(i) for i in s_) for s_ in sents]
    lines[3] = lines[3].replace(word(sents[3][1]), "never-seen")  # an out-of-vocabulary word
    sents[3][1] = 0
    lines.insert(2, "")                                            # an empty line
    lines.insert(5, " ".join(["w1"] * 30))                         # too long: thrown away
    src = tmp_path / "src.txt"
    src.write_text("\n".join(lines) + "\n")
    final, ids = str(tmp_path / "out.txt"), str(tmp_path / "out.ids")
    rep = host.decoding(model, str(src), final, ids_file=ids, beam=beam, longest_sentence=24,
                        attention_width=D, print_decoding_information=True, unk_replacement_mode=True,
                        sentences_per_batch=3)
    assert rep["sentences"] == len(lens) + 1 and rep["sentences_thrown_away"] == 1
    assert rep["source_words"] == sum(lens)

    # the same groups the driver forms (three kept lines at a time, the empty one not decoded), so
    # that every product has the same shape and the comparison can be exact
    b = host.Model(layers, H, Vs, Vt, decoding=(3, beam), **kw)
    b.load_weights(model)
    want = []
    for group in (sents[0:2], sents[2:5], sents[5:7]):
        want += b.decode_batch(group, beam=beam, alignments=True)
    got_ids = open(ids).read().split("\n")[:-1]
    got_txt = open(final).read().split("\n")[:-1]
    assert len(got_ids) == len(lens) + 1 and got_ids[2] == "" and got_txt[2] == ""
    del got_ids[2], got_txt[2]
    tword = lambda i: ["<START>", "<EOF>", "<UNK>"][i] if i < 3 else f"w{i}"  # noqa: E731
    for k, (line, text, w) in enumerate(zip(got_ids, got_txt, want)):
        fields = line.split(" |||| ")
        assert len(fields) == 4, line
        toks = [int(x) for x in fields[0].split()]
        assert toks == w["best"].tolist(), k
        assert np.isclose(float(fields[1]), w["best_score"], rtol=1e-4, atol=1e-5)
        assert [int(x) for x in fields[2].split()] == w["best_viterbi"].tolist(), k
        unk = [v for t, v in zip(toks, w["best_viterbi"].tolist()) if t == 2]
        assert [int(x) for x in fields[3].split()] == (unk if unk else [-1]), k
        assert text.split(" |||| ")[0].split() == [tword(t) for t in toks]
        assert text.split(" |||| ")[1:] == fields[1:]
    assert rep["target_words"] == sum(len(w["best"]) for w in want)


def test_decoding_a_text_file_with_an_ensemble(host, tmp_path):
    """Dispatcher::Decoding with two model files: the text is integerised once per model, with the
    model's own source vocabulary (the second model knows fewer words, so some of them are <UNK>
    for it only), the models decode in lockstep and the first model's target vocabulary spells the
    output.  Expected: DecodeBatch on the shared ids with a stand-in for the second model whose
    embedding table repeats the <UNK> column for the words it does not know."""
    rng = np.random.default_rng(18)
    Vt, D, beam = 40, 2, 4
    kw = dict(longest_sentence=24, attention_mode=1, attention_width=D, feed_input=True)
    PA = R.make_params(rng, 2, 24, 30, Vt, attention=True, feed_input=True, scale=0.5)
    PB30 = R.make_params(rng, 1, 16, 30, Vt, attention=True, feed_input=True, scale=0.5)
    PB30["src.0.W"][:, 20:] = PB30["src.0.W"][:, [0]]
    PB20 = dict(PB30)
    PB20["src.0.W"] = np.ascontiguousarray(PB30["src.0.W"][:, :20])
    files = []
    for name, (L, H, Vs, P) in dict(a=(2, 24, 30, PA), b=(1, 16, 20, PB20)).items():
        m = host.Model(L, H, Vs, Vt, minibatch_size=1, **kw)
        m.set_params(P)
        files.append(str(tmp_path / f"{name}.nmt"))
        m.dump_model(files[-1])
        m.close()
    lens = [5, 8, 3, 6, 2]
    sents = [rng.integers(1, 30, size=n) for n in lens]
    assert any((s_ >= 20).any() for s_ in sents)
    src = tmp_path / "src.txt"
    src.write_text("\n".join(" ".join(f"w{i}" for i in s_) for s_ in sents) + "\n")
    final, ids = str(tmp_path / "out.txt"), str(tmp_path / "out.ids")
    rep = host.decoding(files[0], str(src), final, ids_file=ids, beam=beam, longest_sentence=24,
                        attention_width=D, print_decoding_information=True, unk_replacement_mode=True,
                        sentences_per_batch=3, ensemble_model_files=files[1:])
    assert rep["sentences"] == len(lens) and rep["sentences_thrown_away"] == 0

    a = host.Model(2, 24, 30, Vt, decoding=(3, beam), **kw)
    a.load_weights(files[0])
    b = host.Model(1, 16, 30, Vt, decoding=(3, beam), **kw)
    b.set_params(PB30)
    want = []
    for group in (sents[0:3], sents[3:5]):
        want += a.decode_batch(group, beam=beam, alignments=True, ensemble=[b])
    alone = []
    for group in (sents[0:3], sents[3:5]):
        alone += a.decode_batch(group, beam=beam, alignments=True)
    got_ids = open(ids).read().split("\n")[:-1]
    assert len(got_ids) == len(lens)
    for k, (line, w) in enumerate(zip(got_ids, want)):
        fields = line.split(" |||| ")
        assert [int(x) for x in fields[0].split()] == w["best"].tolist(), k
        assert np.isclose(float(fields[1]), w["best_score"], rtol=1e-4, atol=1e-5)
        assert [int(x) for x in fields[2].split()] == w["best_viterbi"].tolist(), k
    # the second model really takes part
    assert any(x["best"].tolist() != y["best"].tolist() or abs(x["best_score"] - y["best_score"]) > 1e-3
               for x, y in zip(want, alone))
    a.close()
    b.close()


def test_k_best_lists(host, tmp_path):
    """Decoder::OutputKBestHypotheses with hypotheses_number_ > 1 (src/decoder.h:529-607, 692-694):
    the kept hypotheses are the k best final scores among those that pass the length filter, best
    first; a decoded file holds them line by line with a rule of '=' after every sentence.  The
    final scores are recomputed here from the raw hypotheses: length normalisation
    ((5+|Y|)/6)^alpha and, without exported alignments, the coverage penalty of uniform rows."""
    rng = np.random.default_rng(21)
    layers, H, Vs, Vt, D, beam, k = 2, 24, 30, 40, 2, 5, 3
    P = R.make_params(rng, layers, H, Vs, Vt, attention=True, feed_input=True, scale=0.8)
    kw = dict(longest_sentence=24, attention_mode=1, attention_width=D, feed_input=True)
    m = host.Model(layers, H, Vs, Vt, decoding=(2, beam), **kw)
    m.set_params(P)
    sents = [rng.integers(0, Vs, size=n) for n in (7, 4)]
    alpha, beta, min_ratio = np.float32(0.65), np.float32(0.2), 0.5
    res = m.decode_batch(sents, beam=beam, with_hyps=True, num_hypotheses=k)
    one = m.decode_batch(sents, beam=beam)
    for sent, r, r1 in zip(sents, res, one):
        S = len(sent)
        final = []
        for toks, raw in r["hyps"]:
            size = len(toks)
            s_ = np.float32(raw) / (np.float32(5 + size) ** alpha / np.float32(6) ** alpha)
            col = np.float32(0)
            for _ in range(1, size - 1):
                col += np.float32(0.01) / np.float32(S * 0.01)
            cp = max(np.float32(beta * S * np.log(min(col, np.float32(1)))), np.float32(-20)) if size > 2 \
                else np.float32(-20)
            final.append((float(s_ + cp), size / S > min_ratio))
        order = sorted((i for i, f in enumerate(final) if f[1]), key=lambda i: -final[i][0])[:k]
        assert len(order) == k                        # the case is sized so that k survive
        assert [i for i, _ in r["kbest"]] == order
        assert np.allclose([s_ for _, s_ in r["kbest"]], [final[i][0] for i in order], rtol=1e-4, atol=1e-5)
        # the head of the list is the single hypothesis of the default call
        assert r["hyps"][order[0]][0][1:-1].tolist() == r1["best"].tolist() == r["best"].tolist()

    a = host.Model(layers, H, Vs, Vt, minibatch_size=1, **kw)
    a.set_params(P)
    model = str(tmp_path / "model.nmt")
    a.dump_model(model)
    word = lambda i: "<UNK>" if i == 0 else f"w{i}"  # noqa: E731
    src = tmp_path / "src.txt"
    src.write_text("".join(" ".join(word(i) for i in s_) + "\n" for s_ in sents))
    final_file, ids = str(tmp_path / "out.txt"), str(tmp_path / "out.ids")
    host.decoding(model, str(src), final_file, ids_file=ids, beam=beam, longest_sentence=24,
                  attention_width=D, print_decoding_information=True, sentences_per_batch=2,
                  num_hypotheses=k)
    lines = open(ids).read().split("\n")[:-1]
    assert len(lines) == 2 * (k + 1) and lines[k] == lines[2 * k + 1] == "================"
    b = host.Model(layers, H, Vs, Vt, decoding=(2, beam), **kw)
    b.load_weights(model)
    want = b.decode_batch(sents, beam=beam, with_hyps=True, num_hypotheses=k)
    for sidx, w in enumerate(want):
        for rank, (hyp, score) in enumerate(w["kbest"]):
            fields = lines[sidx * (k + 1) + rank].split(" |||| ")
            assert [int(x) for x in fields[0].split()] == w["hyps"][hyp][0][1:-1].tolist()
            assert np.isclose(float(fields[1]), score, rtol=1e-4, atol=1e-5)
    words = open(final_file).read().split("\n")[:-1]
    assert len(words) == len(lines) and words[k] == "================"
    # that run went through DecodeStream (one model, no exported alignments); batch by batch gives
    # the same lines
    import os
    host.set_debug_option("no_stream", 1)
    try:
        ids2 = str(tmp_path / "out2.ids")
        host.decoding(model, str(src), str(tmp_path / "out2.txt"), ids_file=ids2, beam=beam,
                      longest_sentence=24, attention_width=D, print_decoding_information=True,
                      sentences_per_batch=2, num_hypotheses=k)
    finally:
        host.set_debug_option("no_stream", 0)
    lines2 = open(ids2).read().split("\n")[:-1]
    assert [l.split(" |||| ")[0] for l in lines2] == [l.split(" |||| ")[0] for l in lines]


def test_decoding_a_long_text_file_through_the_stream(host, tmp_path):
    """Dispatcher::Decoding with one model and no exported alignments hands the file to
    DecodeStream 32 batches at a time: 150 lines at two sentences per batch are three such lists
    (64 + 64 + 22), one of them with an empty line inside.  Every line must be what DecodeStream
    gives for the same list on a model loaded from the same file (same launches, so exactly), and
    the batch-by-batch path of the dispatcher must give the same tokens."""
    import os
    rng = np.random.default_rng(31)
    layers, H, Vs, Vt, D, beam, n_sent = 2, 24, 30, 40, 2, 4, 2
    P = R.make_params(rng, layers, H, Vs, Vt, attention=True, feed_input=True, scale=0.4)
    kw = dict(longest_sentence=24, attention_mode=1, attention_width=D, feed_input=True)
    a = host.Model(layers, H, Vs, Vt, minibatch_size=1, **kw)
    a.set_params(P)
    model = str(tmp_path / "model.nmt")
    a.dump_model(model)
    a.close()
    sents = [rng.integers(0, Vs, size=int(rng.integers(1, 15))) for _ in range(149)]
    word = lambda i: "<UNK>" if i == 0 else f"w{i}"  # noqa: E731
    lines = [" ".join(word(i) for i in s_) for s_ in sents]
    lines.insert(70, "")  # an empty line inside the second list
    src = tmp_path / "src.txt"
    src.write_text("\n".join(lines) + "\n")
    ids = str(tmp_path / "out.ids")
    rep = host.decoding(model, str(src), str(tmp_path / "out.txt"), ids_file=ids, beam=beam,
                        longest_sentence=24, attention_width=D, print_decoding_information=True,
                        sentences_per_batch=n_sent)
    assert rep["sentences"] == 150 and rep["sentences_thrown_away"] == 0
    got = open(ids).read().split("\n")[:-1]
    assert len(got) == 150 and got[70] == ""
    b = host.Model(layers, H, Vs, Vt, decoding=(n_sent, beam), **kw)
    b.load_weights(model)
    chunk = 32 * n_sent
    want = []
    for first in range(0, 150, chunk):
        block = [(i, lines[i]) for i in range(first, min(150, first + chunk)) if lines[i]]
        res = b.decode_stream([sents[i if i < 70 else i - 1] for i, _ in block], beam=beam)
        it = iter(res)
        want += [next(it) if lines[i] else None for i in range(first, min(150, first + chunk))]
    b.close()
    for k, (line, w) in enumerate(zip(got, want)):
        if w is None:
            assert line == "", k
            continue
        fields = line.split(" |||| ")
        assert [int(x) for x in fields[0].split()] == w["best"].tolist(), k
        assert np.isclose(float(fields[1]), w["best_score"], rtol=1e-5, atol=1e-4), k  # six digits in the file
    assert rep["target_words"] == sum(len(w["best"]) for w in want if w is not None)
    host.set_debug_option("no_stream", 1)
    try:
        ids2 = str(tmp_path / "out2.ids")
        host.decoding(model, str(src), str(tmp_path / "out2.txt"), ids_file=ids2, beam=beam,
                      longest_sentence=24, attention_width=D, print_decoding_information=True,
                      sentences_per_batch=n_sent)
    finally:
        host.set_debug_option("no_stream", 0)
    got2 = open(ids2).read().split("\n")[:-1]
    same = sum(x.split(" |||| ")[0] == y.split(" |||| ")[0] for x, y in zip(got, got2))
    assert len(got2) == 150 and same >= 147, same  # a near-tie may fall the other way between the two modes


@pytest.mark.parametrize("layers,attention,feed", [(2, 1, True), (1, 1, False), (3, 0, False)])
def test_model_file_written_independently_loads_decodes_and_is_dumped_byte_for_byte(orc, host, tmp_path,
                                                                                    layers, attention, feed):
    """The model file against a writer that is not the path's own: oracle/orc.py write_model_file
    follows NeuralMachineTranslation::DumpWeights and WriteMatrixGpu line by line
    (src/deep_rnn.h:2124-2146, src/deep_rnn_kernel.h:1564-1578, src/layer_input_to_hidden.h:1556-1590;
    pinned on the hand-made file in tests/test_oracle_tuning_pins.py).
      * LoadWeights of that file must give a model that decodes what the oracle decodes with the
        file's numbers (read back by the oracle's own reader: eight digits do not always
        reproduce an fp32 value, so the file's numbers are the model);
      * DumpModel of a model holding the same parameters must write that file byte for byte;
      * so must the training loop's final DumpWeights onto a file that so far holds the header
        and the mappings, which is how the reference's trainer finds it."""
    rng = np.random.default_rng(40 + layers)
    H, Vs, Vt, D, beam = 16, 23, 31, 3, 4
    P = R.make_params(rng, layers, H, Vs, Vt, attention=bool(attention), feed_input=feed, scale=0.4)
    src_words = ["<UNK>"] + [f"w{i}" for i in range(1, Vs)]
    tgt_words = ["<START>", "<EOF>", "<UNK>"] + [f"w{i}" for i in range(3, Vt)]
    want_file = str(tmp_path / "oracle_written.nmt")
    orc.write_model_file(want_file, P, layers, H, Vs, Vt, attention, feed)
    info, P_file = orc.read_model_file(want_file)
    assert info["source_words"] == src_words and info["target_words"] == tgt_words
    assert max(float(np.abs(P_file[k] - np.asarray(P[k]).reshape(P_file[k].shape)).max()) for k in P) < 1e-7

    kw = dict(longest_sentence=24, attention_mode=attention, attention_width=D, feed_input=feed)
    gm = host.Model(layers, H, Vs, Vt, decoding=(3, beam), **kw)
    gm.load_weights(want_file)
    for name, arr in P_file.items():
        shape = arr.shape if arr.ndim == 2 else (arr.size,)
        assert np.array_equal(gm.get_param(name, shape), arr), name
    om = orc.Model(layers, H, Vs, Vt, attention=attention, D=D, feed_input=int(feed), longest_sent=24)
    om.set_params(P_file)
    sents = [rng.integers(0, Vs, size=n) for n in (7, 2, 11)]
    got = gm.decode_batch(sents, beam=beam, with_hyps=True)
    for i, s in enumerate(sents):
        want = om.decode_sentence(s, beam=beam)
        assert got[i]["best"].tolist() == want["best"].tolist(), i
        assert [h[0].tolist() for h in got[i]["hyps"]] == [h[0].tolist() for h in want["hyps"]], i
        assert np.allclose([h[1] for h in got[i]["hyps"]], [h[1] for h in want["hyps"]], rtol=1e-4, atol=1e-4)
    gm.close()

    tm = host.Model(layers, H, Vs, Vt, minibatch_size=2,
                    training=dict(learning_rate=0.1, grad_clip_mode=2, norm_clip=5.0), **kw)
    tm.set_params(P)
    dumped = str(tmp_path / "dumped.nmt")
    tm.dump_model(dumped)
    assert open(dumped, "rb").read() == open(want_file, "rb").read()
    # a file the corpus preprocessor has started (first line + mappings): zero epochs of the loop
    # append the matrices
    head = open(want_file).read().split("\n")
    n_head = 1 + 1 + Vs + 1 + Vt + 1
    started = str(tmp_path / "started.nmt")
    open(started, "w").write("\n".join(head[:n_head]) + "\n")
    train = str(tmp_path / "train.txt")
    open(train, "w").write("1 2\n-2 -2\n0 3\n3 1\n" * 2)
    tm.tuning(train, output_weight_file=started, epochs=0)
    assert open(started, "rb").read() == open(want_file, "rb").read()
    tm.close()
