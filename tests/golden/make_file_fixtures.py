"""Writes the two hand-made fixtures of the file formats either side of the path.

No reference-written training file or model file exists in the reference checkout (its corpus
preprocessor and trainer are CUDA programs), so these follow the formats as the reference's
readers parse them: FileHelper::ReadMinibatch (src/file_helper.cc:113-272) and
NeuralMachineTranslation::LoadWeights / ReadMatrixGpu (src/deep_rnn.h:1878-1968,
src/deep_rnn_kernel.h:1543-1561).  Run from the repository root: python tests/golden/make_file_fixtures.py
"""
import os

HERE = os.path.dirname(os.path.abspath(__file__))

# ---- training file: 3 minibatches of 2 pairs (the third one ragged against the others) ----------
PAIRS = [
    # source (reversed, left-padded), target input, target output
    ("-1 5 4 3", "0 7 8 -1", "7 8 1 -1"),
    ("9 6 5 4", "0 3 4 5", "3 4 5 1"),
    ("-1 -1 2 1 7", "0 9 -1", "9 1 -1"),
    ("3 3 3 3 3", "0 3 3", "3 3 1"),
    ("8", "0 2", "2 1"),
    ("0", "0 11", "11 1"),
]
with open(os.path.join(HERE, "train_minibatches.txt"), "w") as f:
    for src, tin, tout in PAIRS:
        f.write(src + "\n" + " ".join(["-2"] * len(src.split())) + "\n" + tin + "\n" + tout + "\n")

# ---- model file: 2 layers, H = 3, vocabularies 5 / 6, local-p attention with input feeding -------
# Element (i, j) of the k-th matrix of the file is k + i / 10 + j / 100, so a test can tell which
# matrix, row and column every parameter came from.
L, H, VT, VS = 2, 3, 6, 5
shapes = []
def layer(vocab, first, feed):
    for _ in range(4):
        shapes.extend([(H, H), (H, 1)])          # W_hi b_i W_hf b_f W_hc b_c W_ho b_o
    if first:
        shapes.append((H, vocab))                # W
    shapes.extend([(H, H)] * 4)                  # M_i M_f M_o M_c
    if feed:
        shapes.extend([(H, H)] * 4)              # Q_i Q_f Q_o Q_c
for l in range(L):
    layer(VS, l == 0, False)
for l in range(L):
    layer(VT, l == 0, l == 0)
shapes.extend([(H, H), (H, H), (H, 1), (H, 1), (H, H), (H, H)])   # W_a W_p v_p b_out W_c1 W_c2
shapes.extend([(VT, H), (VT, 1)])                                  # D b_d
RULE = "=" * 58
with open(os.path.join(HERE, "tiny_model.nmt"), "w") as f:
    f.write(f"{L} {H} {VT} {VS} 1 1 0 0 0\n{RULE}\n")
    f.write("0 <UNK>\n" + "".join(f"{i} s{i}\n" for i in range(1, VS)) + RULE + "\n")
    f.write("0 <START>\n1 <EOF>\n2 <UNK>\n" + "".join(f"{i} t{i}\n" for i in range(3, VT)) + RULE + "\n")
    for k, (r, c) in enumerate(shapes):
        for i in range(r):
            f.write(" ".join(f"{k + i / 10 + j / 100:.2f}" for j in range(c)) + "\n")
        f.write("\n")
print(len(shapes), "matrices")
