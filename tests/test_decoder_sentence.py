"""The one-sentence decoder of the reference's translation server (DecoderSentence,
src/decoder_sentence.cu:14-391, and the two C functions of src/decoder_sentence.cu:844-874).
Host part (no GPU): configuration file, vocabularies, sentence <-> ids, with expected values
written out by hand from the reference's rules.  GPU part: the text of a translation against
DecodeBatch on the same sentence.  Parity unpinned against the reference's own output: the
checkout holds no model file and no server transcript."""
import os

import numpy as np
import pytest

import ref_numpy as R

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MODEL = os.path.join(GOLDEN, "tiny_model.nmt")  # source: <UNK> s1..s4; target: <START> <EOF> <UNK> t3..t5


def write_config(path, model, extra=""):
    path.write_text(
        "# * a comment line *\n"
        "\n"
        f'param="--nmt-model"                   value="{model}"\r\n'
        '   param="--beam-size"                  value="7"   \n'
        'param="--beam-size"                  value="3"\n'          # a later line wins
        'param="--broken                      value="5"\n'          # read as one odd key, harmless
        'value-less line\n'
        + extra)
    return str(path)


def test_config_file_and_settings(tmp_path):
    from linmt_amd import host
    cfg = write_config(tmp_path / "a.config", MODEL,
                       'param="--longest-sent" value="50"\nparam="--decoding-ratio" value="1.0 2.9"\n'
                       'param="--lp-alpha" value="0.5"\nparam="--cp-beta" value="0.1"\n'
                       'param="--diversity" value="0.25"\nparam="--attention-width" value="4"\n'
                       'param="--print-decoding-info" value="1"\nparam="--log-level" value="2"\n')
    d = host.DecoderSentence(cfg, load_model=False)
    s = d.settings()
    assert s["model_file"] == MODEL and s["beam_size"] == 3
    assert s["longest_sentence"] == 54            # + 4 as in GeneralSettings
    # both ratios go through integer conversions in the reference
    assert (s["min_decoding_ratio"], s["max_decoding_ratio"]) == (1.0, 2.0)
    assert np.allclose([s["lp_alpha"], s["cp_beta"], s["diversity"]], [0.5, 0.1, 0.25])
    assert s["attention_width"] == 4
    assert s["print_decoding_information"] == 1 and s["unk_replacement_mode"] == 1
    assert s["print_alignments_scores"] == 0 and s["sentences_per_batch"] == 1
    # defaults (src/global_configuration.h:228-235,298; attention window 10)
    d2 = host.DecoderSentence(write_config(tmp_path / "b.config", MODEL), load_model=False)
    s2 = d2.settings()
    assert (s2["longest_sentence"], s2["attention_width"]) == (104, 10)
    assert np.allclose([s2["min_decoding_ratio"], s2["max_decoding_ratio"], s2["lp_alpha"], s2["cp_beta"],
                        s2["penalty"], s2["diversity"]], [0.5, 1.5, 0.65, 0.2, 0, 0])
    assert s2["print_decoding_information"] == 0 and s2["unk_replacement_mode"] == 0


@pytest.mark.parametrize("text,why", [
    ('param="--beam-size" value="4"\n', "no --nmt-model"),
    ('param="--nmt-model" value="{m}"\nparam="--beam-size" value="0"\n', "beam 0"),
    ('param="--nmt-model" value="{m}"\nparam="--decoding-ratio" value="1"\n', "one ratio"),
    ('param="--nmt-model" value="{m}"\nparam="--decoding-ratio" value="2 1"\n', "min >= max"),
    ('param="--nmt-model" value="{m} /no/such/second.nmt"\n', "an ensemble with a missing file"),
    ('param="--nmt-model" value="{m}"\nparam="--multi-gpu" value="0 1"\n', "gpus != models"),
    ('param="--nmt-model" value="/no/such/model.nmt"\n', "missing model file"),
])
def test_settings_the_reference_exits_on(tmp_path, text, why):
    from linmt_amd import host
    p = tmp_path / "bad.config"
    p.write_text(text.replace("{m}", MODEL))
    with pytest.raises(host.HostError):
        host.DecoderSentence(str(p), load_model=False)
    with pytest.raises(host.HostError):
        host.DecoderSentence(str(tmp_path / "absent.config"), load_model=False)


def test_sentence_to_ids_and_back(tmp_path):
    from linmt_amd import host
    d = host.DecoderSentence(write_config(tmp_path / "a.config", MODEL), load_model=False)
    # reversed, unknown word -> 0, text after " |||| " dropped, any run of blanks separates
    assert d.integerize("s1 s2   never-seen s4 |||| s3 s3").tolist() == [4, 0, 2, 1]
    assert d.integerize("").tolist() == [] and d.integerize("   ").tolist() == []
    assert d.unint("3 4 5") == "t3 t4 t5"
    assert d.unint("2 5 |||| -1.25 |||| 0 1 |||| 0") == "<UNK> t5 |||| -1.25 |||| 0 1 |||| 0"
    assert d.unint("5 ||||") == "t5 |||| "      # a trailing field mark gains a blank
    assert d.unint("") == ""
    with pytest.raises(host.HostError):
        d.process("s1 s2")                      # no model was loaded


@pytest.mark.gpu
def test_translations_match_decode_batch(tmp_path):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from linmt_amd import host
    rng = np.random.default_rng(12)
    layers, H, Vs, Vt, D, beam = 2, 24, 30, 40, 3, 4
    P = R.make_params(rng, layers, H, Vs, Vt, attention=True, feed_input=True, scale=0.5)
    kw = dict(longest_sentence=34, attention_mode=1, attention_width=D, feed_input=True)
    a = host.Model(layers, H, Vs, Vt, minibatch_size=1, **kw)
    a.set_params(P)
    model = str(tmp_path / "model.nmt")
    a.dump_model(model)  # placeholder vocabularies: source <UNK> w1.., target <START> <EOF> <UNK> w3..
    cfg = tmp_path / "server.config"
    cfg.write_text(f'param="--nmt-model" value="{model}"\nparam="--beam-size" value="{beam}"\n'
                   f'param="--attention-width" value="{D}"\nparam="--longest-sent" value="30"\n'
                   'param="--decoding-ratio" value="0 2"\nparam="--print-decoding-info" value="1"\n'
                   'param="--print-align-scores" value="1"\n')
    d = host.DecoderSentence(str(cfg))
    b = host.Model(layers, H, Vs, Vt, decoding=(1, beam), **kw)
    b.load_weights(model)
    # a second model file: the service then decodes with the ensemble of the two
    P2 = R.make_params(rng, 1, 16, Vs, Vt, attention=True, feed_input=True, scale=0.5)
    a2 = host.Model(1, 16, Vs, Vt, minibatch_size=1, **kw)
    a2.set_params(P2)
    model2 = str(tmp_path / "model2.nmt")
    a2.dump_model(model2)
    cfg2 = tmp_path / "ensemble.config"
    cfg2.write_text(cfg.read_text().replace(f'value="{model}"', f'value="{model} {model2}"'))
    d2 = host.DecoderSentence(str(cfg2))
    b2 = host.Model(1, 16, Vs, Vt, decoding=(1, beam), **kw)
    b2.load_weights(model2)
    word = lambda i: "<UNK>" if i == 0 else f"w{i}"  # noqa: E731
    tword = lambda i: ["<START>", "<EOF>", "<UNK>"][i] if i < 3 else f"w{i}"  # noqa: E731
    for n in (6, 1, 11, 3):
        sent = rng.integers(0, Vs, size=n)
        text = d.process(" ".join(word(i) for i in sent) + " |||| not part of the sentence")
        w = b.decode_batch([sent], beam=beam, alignments=True, min_ratio=0.0, max_ratio=2.0)[0]
        text2 = d2.process(" ".join(word(i) for i in sent))
        w2 = b.decode_batch([sent], beam=beam, alignments=True, min_ratio=0.0, max_ratio=2.0,
                            ensemble=[b2])[0]
        assert text2.split(" |||| ")[0].split() == [tword(t) for t in w2["best"].tolist()]
        assert np.isclose(float(text2.split(" |||| ")[1]), w2["best_score"], rtol=1e-4, atol=1e-5)
        fields = text.split(" |||| ")
        assert len(fields) == 5, text
        assert fields[0].split() == [tword(t) for t in w["best"].tolist()]
        assert np.isclose(float(fields[1]), w["best_score"], rtol=1e-4, atol=1e-5)
        assert [int(x) for x in fields[2].split()] == w["best_viterbi"].tolist()
        unk = [v for t, v in zip(w["best"].tolist(), w["best_viterbi"].tolist()) if t == 2]
        assert [int(x) for x in fields[3].split()] == (unk if unk else [-1])
        rows = [[float(x) for x in tok.split("/")] for tok in fields[4].split()]
        assert len(rows) == len(w["best"]) and all(len(r) == n for r in rows)
    assert d.process("") == "" and d.process("   ") == ""
    assert d.process(" ".join(["w1"] * 40)) == ""       # longer than the buffers of --longest-sent

    # the process-wide pair the server binds: same text, result owned by the library
    host.python_decoder_init(str(cfg))
    sent = rng.integers(1, Vs, size=5)
    line = " ".join(word(i) for i in sent)
    assert host.python_decoder_do_job(line) == d.process(line)
    assert host.python_decoder_do_job("") == ""
    assert host.python_decoder_do_job(line) == d.process(line)
