"""GPU tests of the fp32 products formed on the bf16 matrix pipe (lh_split_pack_f32,
lh_gemm_split_f32, lh_gate_gemm_split_lstm_cell_f32): the packed planes reproduce every fp32 input
exactly, the products are as close to float64 as those of lh_gemm_f32 (tolerance: 4e-7 of the sum
of the magnitudes of a result's terms, which is what fp32 accumulation over a few thousand terms
gives), the cell form agrees with the oracle's cell within rtol=1e-4, atol=1e-5."""
import numpy as np
import pytest
import torch

from conftest import assert_close
from test_gpu_kernels import dev, host, uni

pytestmark = pytest.mark.gpu

PAD = 256


def planes_tensor(lh, D, kg):
    # filled with a pattern that is a NaN in every bf16 lane: what the packing must overwrite
    return torch.full((lh.split_bytes(D, kg) // 4,), -1, dtype=torch.int32, device="cuda")


def unpack(planes, Dp, KG):
    """planes tensor -> float64 array [3][KG*8][Dp] of the bf16 values."""
    torch.cuda.synchronize()
    raw = planes.cpu().numpy().view(np.uint16).reshape(3, KG, Dp, 8)
    f = (raw.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return f.transpose(0, 1, 3, 2).reshape(3, KG * 8, Dp)


def test_packing_is_exact_and_zero_padded(lh):
    rng = np.random.default_rng(5)
    D, K = 300, 70
    a = uni(rng, D, K)
    a[0, :8] = [0.0, -0.0, 1.0, -1.0, 1e38, -1e-30, 1.0 + 2.0 ** -23, 0.1]
    kg = lh.split_kgroups(K)
    total = lh.split_kgroups_padded(kg + 4)
    assert kg == 9 and total == 16 and lh.load().lh_split_padded(D) == 512
    for k_contig in (True, False):
        src = a if k_contig else a.T                      # (D, K) row-major or (K, D) row-major
        t = torch.from_numpy(np.ascontiguousarray(src)).cuda()
        p = planes_tensor(lh, D, total)
        p2 = planes_tensor(lh, D, total)
        lh.split_pack([dict(src=t, ld=K if k_contig else D, k_contiguous=k_contig, D=D, K=K, planes=p,
                            kgroups_total=total, kg_offset=2),
                       dict(src=t, ld=K if k_contig else D, k_contiguous=k_contig, D=D, K=K, planes=p2,
                            kgroups_total=total, kg_offset=4, kgroups=total - 4)])
        for planes, off, n in ((p, 2, kg), (p2, 4, total - 4)):
            f = unpack(planes, 512, total)[:, off * 8:(off + n) * 8]
            both = f[0] + f[1] + f[2]
            assert np.array_equal(both[:K, :D], a.T.astype(np.float64)), "a1 + a2 + a3 != a"
            assert np.all(f[:, K:, :] == 0) and np.all(f[:, :, D:] == 0), "padding is not zero"
            assert np.all(np.abs(f[1, :K, :D]) <= np.abs(f[0, :K, :D]) * 2.0 ** -8 + 1e-45)


@pytest.mark.parametrize("M,N,K", [(1003, 37, 70), (130, 300, 1000), (5000, 768, 1000), (4096, 129, 48)])
def test_split_product_against_float64(lh, M, N, K):
    rng = np.random.default_rng(M + N)
    L = lh.load()
    A = uni(rng, M, K, s=0.08)            # element (m, k)
    X = uni(rng, K, N)                    # element (k, n)
    b = uni(rng, M, s=0.08)
    want = A.astype(np.float64) @ X + b[:, None]
    mag = np.abs(A).astype(np.float64) @ np.abs(X) + np.abs(b)[:, None]
    Ad, Xd, bd = dev(A), dev(X), dev(b)   # column-major: A m-contiguous, X k-contiguous
    kg = lh.split_kgroups_padded(lh.split_kgroups(K))
    Ap, Xp = planes_tensor(lh, M, kg), planes_tensor(lh, N, kg)
    lh.split_pack([dict(src=Ad, ld=M, k_contiguous=False, D=M, K=K, planes=Ap, kgroups_total=kg, kgroups=kg)])
    lh.split_pack([dict(src=Xd, ld=K, k_contiguous=True, D=N, K=K, planes=Xp, kgroups_total=kg, kgroups=kg)])
    ref = torch.empty(M * N, device="cuda")
    lh.gemm(M, N, [(Ad, M, Xd, K, K)], ref, M, bias=bd)
    ref_err = float((np.abs(host(ref, (M, N)) - want) / mag).max())
    n_cfg = L.lh_gemm_split_set_config_override(-1)
    try:
        for cfg in range(-1, n_cfg):
            L.lh_gemm_split_set_config_override(cfg)
            out = torch.full((M * N,), float("nan"), device="cuda")
            lh.gemm_split(M, N, kg, Ap, Xp, out, M, bias=bd)
            err = float((np.abs(host(out, (M, N)) - want) / mag).max())
            assert err <= 4e-7, f"config {cfg}: {err}"
            assert err <= 1.5 * ref_err + 1e-7, f"config {cfg}: {err} against {ref_err} of lh_gemm_f32"
            # the epilogue's options
            cm = (rng.uniform(size=N) < 0.7).astype(np.int32)
            base = uni(rng, M, N)
            out = dev(base)
            lh.gemm_split(M, N, kg, Ap, Xp, out, M, alpha=0.5, beta=2.0, bias=bd, act=lh.LH_ACT_TANH,
                          act_rows=M // 2, colmask=dev(cm))
            w = 0.5 * (A.astype(np.float64) @ X) + 2.0 * base + b[:, None]
            w[: M // 2] = np.tanh(w[: M // 2])
            w *= cm[None, :]
            assert_close(host(out, (M, N)), w.astype(np.float32), f"config {cfg} epilogue")
    finally:
        L.lh_gemm_split_set_config_override(-1)


def test_split_arguments_are_checked(lh):
    kg = lh.split_kgroups_padded(lh.split_kgroups(64))
    P = planes_tensor(lh, 64, kg)
    out = torch.empty(64 * 64, device="cuda")
    with pytest.raises(lh.LinmtHipError):
        lh.gemm_split(64, 64, kg + 1, P, P, out, 64)          # not whole slabs
    with pytest.raises(lh.LinmtHipError):
        lh.gemm_split(64, 64, kg, P, P, out, 32)              # ldc < M
    with pytest.raises(lh.LinmtHipError):
        lh.split_pack([dict(src=out, ld=64, k_contiguous=True, D=64, K=64, planes=P, kgroups_total=kg,
                            kg_offset=kg - 4)])               # segment does not fit
    with pytest.raises(lh.LinmtHipError):
        lh.gate_gemm_split_lstm_cell(36, 8, kg, P, P, out, out, out, out, out)   # H not a multiple of 8


CELL_CASES = [  # H, B, Ks, addend: None / "plain" / "table", f64, clip
    (112, 76, (112, 40), None, False, 0.0),
    (40, 37, (68,), "plain", True, 0.0),
    (72, 132, (24, 12, 136), "table", False, 0.5),
    (1000, 300, (1000, 1000), "table", True, 0.0),
]


@pytest.mark.parametrize("H,B,Ks,addend,f64,clip", CELL_CASES)
def test_split_gate_product_with_cell(lh, orc, H, B, Ks, addend, f64, clip):
    """Against the oracle's cell on float64 pre-activations; multi-segment operands packed side by
    side; the addend read straight or through a column index; masked columns; cell state in place;
    h as split planes equal to packing h afterwards, over a buffer full of stale values."""
    rng = np.random.default_rng(H + B)
    L = lh.load()
    As = [uni(rng, 4 * H, K, s=0.3) for K in Ks]
    Xs = [uni(rng, K, B) for K in Ks]
    bias, c_prev = uni(rng, 4 * H, s=0.5), uni(rng, H, B)
    mask = (rng.uniform(size=B) < 0.8).astype(np.int32)
    kgs = [lh.split_kgroups(K) for K in Ks]
    KG = lh.split_kgroups_padded(sum(kgs))
    kgs[-1] = KG - sum(kgs[:-1])                              # the last segment carries the padding
    Wp = planes_tensor(lh, L.lh_split_gate_rows(H), KG)
    Xp = planes_tensor(lh, B, KG)
    off = 0
    keep = []
    for A, X, K, kg in zip(As, Xs, Ks, kgs):
        a_d, x_d = dev(A), dev(X)
        keep += [a_d, x_d]
        lh.split_pack([dict(src=a_d, ld=4 * H, k_contiguous=False, D=4 * H, K=K, gate_H=H, planes=Wp,
                            kgroups_total=KG, kg_offset=off, kgroups=kg),
                       dict(src=x_d, ld=K, k_contiguous=True, D=B, K=K, planes=Xp, kgroups_total=KG,
                            kg_offset=off, kgroups=kg)])
        off += kg
    table = cols = add_np = None
    ld, V = 4 * H, 0
    if addend == "plain":
        add_np = uni(rng, 4 * H, B)
        table = dev(add_np)
    elif addend == "table":
        V = 23
        full = uni(rng, 4 * H + 4, V)
        ld = 4 * H + 4
        cols_np = rng.integers(0, V, size=B).astype(np.int32)
        cols_np[0], cols_np[-1] = -3, V + 5                 # clamped like the embedding lookup
        table, cols = dev(full), dev(cols_np)
        add_np = full[: 4 * H, np.clip(cols_np, 0, V - 1)]
    pre = sum(A.astype(np.float64) @ X for A, X in zip(As, Xs))
    if add_np is not None:
        pre = pre + add_np
    _, wc, wh = orc.lstm_cell_fwd(pre.astype(np.float32), bias, c_prev, mask, feed=f64, cell_clip=clip)
    hkg = lh.split_kgroups_padded(H // 8 + 2)
    n_cfg = L.lh_gemm_split_set_config_override(-1)
    try:
        for cfg in range(-1, n_cfg):
            L.lh_gemm_split_set_config_override(cfg)
            what = f"config {cfg} H={H} B={B} K={Ks} addend={addend}"
            c = dev(c_prev)                                  # in place
            h = torch.full((H * B,), float("nan"), device="cuda")
            hp = planes_tensor(lh, B, hkg)                   # stale values everywhere
            lh.gate_gemm_split_lstm_cell(H, B, KG, Wp, Xp, dev(bias), c, dev(mask), c, h, addend=table,
                                         ld_addend=ld if table is not None else 0, addend_col=cols,
                                         addend_ncols=V, sigmoid_f64=f64, cell_clip=clip, h_planes=hp,
                                         hp_kgroups_total=hkg, hp_kg_offset=2, hp_kgroups=hkg - 2)
            assert_close(host(c, (H, B)), wc, what + " c")
            assert_close(host(h, (H, B)), wh, what + " h")
            assert np.all(host(h, (H, B))[:, mask == 0] == 0), what
            # h's planes: exactly what packing h gives, in the k-groups asked for
            hp2 = planes_tensor(lh, B, hkg)
            lh.split_pack([dict(src=h, ld=H, k_contiguous=True, D=B, K=H, planes=hp2,
                                kgroups_total=hkg, kg_offset=2, kgroups=hkg - 2)])
            Bp = L.lh_split_padded(B)
            got = unpack(hp, Bp, hkg)[:, 16:, :B]
            exp = unpack(hp2, Bp, hkg)[:, 16:, :B]
            assert np.array_equal(got, exp), what + ": planes of h"
    finally:
        L.lh_gemm_split_set_config_override(-1)
