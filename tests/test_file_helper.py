"""FileHelper (the reference's training-file reader, src/file_helper.cc:113-381) on a hand-made
file in the reference's four-lines-per-pair format (tests/golden/train_minibatches.txt, written by
tests/golden/make_file_fixtures.py).  Expected values come from the definition -- transposes,
counts, sets -- written here with numpy, not from the reader's code.  Parity unpinned against a
reference-written file: the checkout holds none.  Host-only: runs without a GPU."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _pairs():
    lines = open(os.path.join(GOLDEN, "train_minibatches.txt")).read().split("\n")
    out = []
    for k in range(0, len(lines) - 1, 4):
        out.append(tuple(np.array(lines[k + d].split(), dtype=np.int64) for d in (0, 2, 3)))
    return out


def _partition_order(first_seen):
    """ids to the left, -1 to the right, by the two-pointer swap the reference uses
    (src/file_helper.cc:322-378) -- restated only to state the ORDER of the unique-id list."""
    v = list(first_seen)
    left, right = 0, len(v) - 1
    while left < right:
        if v[left] == -1:
            if v[right] != -1:
                v[left], v[right] = v[right], v[left]
                left += 1
            right -= 1
            continue
        left += 1
    if v and v[left] != -1:
        left += 1
    return v[:left]


def test_read_minibatch_layout_and_counts():
    from linmt_amd import host
    pairs = _pairs()
    B = 2
    fh = host.FileHelper(os.path.join(GOLDEN, "train_minibatches.txt"), B, 12, 10, 12)
    n_batches = len(pairs) // B
    for rep in range(2):  # second pass: the reader has rewound to the start of the file
        for b in range(n_batches):
            same_epoch, mb = fh.read_minibatch()
            chunk = pairs[b * B:(b + 1) * B]
            src = np.stack([p[0] for p in chunk])
            tin = np.stack([p[1] for p in chunk])
            tout = np.stack([p[2] for p in chunk])
            assert same_epoch == (b != n_batches - 1)
            assert mb["current_source_length"] == src.shape[1]
            assert mb["current_target_length"] == tin.shape[1]
            assert np.array_equal(mb["source_in"], src)
            assert np.array_equal(mb["target_in"], tin)
            assert np.array_equal(mb["target_out"], tout)
            # [length per column .., left padding per column ..]
            lengths = (src != -1).sum(axis=1)
            assert mb["batch_information"].tolist() == lengths.tolist() + (src.shape[1] - lengths).tolist()
            assert mb["words_in_minibatch"] == int((src != -1).sum() + (tout != -1).sum())
            for key, block in (("source_wgrad", src), ("target_wgrad", tin)):
                flat = block.ravel(order="F")  # the reader walks the column-major block
                want = sorted(set(flat[flat != -1].tolist()))
                assert sorted(mb[key].tolist()) == want and len(mb[key]) == len(want)
                seen, first = set(), []
                for x in flat.tolist():
                    first.append(x if x != -1 and x not in seen else -1)
                    seen.add(x)
                assert mb[key].tolist() == _partition_order(first)
            assert mb["nums_lines_in_file"] == 4 * len(pairs)
            assert mb["total_words"] == sum(int((p[0] != -1).sum() + (p[1] != -1).sum()) for p in pairs)
            assert mb["total_target_words"] == sum(int((p[1] != -1).sum()) for p in pairs)
    fh.close()


def test_errors():
    from linmt_amd import host
    with pytest.raises(host.HostError):
        host.FileHelper(os.path.join(GOLDEN, "no_such_file.txt"), 2, 12, 10, 12)
    fh = host.FileHelper(os.path.join(GOLDEN, "train_minibatches.txt"), 2, 12, 10, 10)
    fh.read_minibatch()
    fh.read_minibatch()
    with pytest.raises(host.HostError):  # target id 11 with a vocabulary of 10
        fh.read_minibatch()
    with pytest.raises(host.HostError):  # a minibatch longer than minibatch x longest_sentence
        host.FileHelper(os.path.join(GOLDEN, "train_minibatches.txt"), 2, 2, 10, 12).read_minibatch()


def test_model_information():
    from linmt_amd import host
    info = host.read_model_information(os.path.join(GOLDEN, "tiny_model.nmt"))
    assert info == dict(num_layers=2, lstm_size=3, target_vocab_size=6, source_vocab_size=5,
                        attention_model=1, feed_input=1, multi_source=0, combine_lstm=0, char_cnn=0)
    with pytest.raises(host.HostError):
        host.read_model_information(os.path.join(GOLDEN, "no_such_model.nmt"))


def test_integerize_source_text_and_unintegerize_output(tmp_path):
    """IntegerizeFileDecoding / UnintFile (src/input_file_preprocess.cc:1312-1581) with the
    vocabularies of tests/golden/tiny_model.nmt (source: <UNK> s1..s4; target: <START> <EOF> <UNK>
    t3..t5).  Expected values written out by hand from the rules: text before " |||| ", unknown
    words -> <UNK> (id 0), a sentence with length + 1 >= cutoff - 2 is dropped, ids up to the first
    "||||" become words, separator lines and the rest of a line are copied."""
    from linmt_amd import host
    model = os.path.join(GOLDEN, "tiny_model.nmt")
    src = tmp_path / "src.txt"
    src.write_text("s1 s2 s3\ns4 nope s1 |||| ignored tail\n\ns2 s2 s2 s2 s2 s2 s2 s2 s2\n  s3  \n")
    sents, lines, vt = host.integerize_file_decoding(model, str(src), 12)
    assert [x.tolist() for x in sents] == [[1, 2, 3], [4, 0, 1], [], [3]]
    assert lines == [0, 1, 2, 4] and vt == 6   # the nine-word line is thrown away (9 + 1 >= 10)
    ids = tmp_path / "out.ids"
    ids.write_text("3 4 5\n2 |||| -1.5 |||| 0 |||| 0\n\n================\n5 ||||\n1 0\n")
    final = tmp_path / "final.txt"
    host.unint_file(model, str(ids), str(final))
    assert final.read_text() == ("t3 t4 t5\n<UNK> |||| -1.5 |||| 0 |||| 0\n\n================\n"
                                 "t5 |||| \n<EOF> <START>\n")
    with pytest.raises(host.HostError):
        host.integerize_file_decoding(os.path.join(GOLDEN, "nope.nmt"), str(src), 12)
