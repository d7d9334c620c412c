"""GPU parity tests of the training-side entry points of liblinmt_hip.so against the CPU oracle
(kernel granularity) on the same seeded inputs; fp32 within rtol=1e-4 / atol=1e-5 unless a test
states a wider bound for a long fp32 reduction."""
import numpy as np
import pytest
import torch

from conftest import assert_close
from test_gpu_kernels import dev, host, uni

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("H,B", [(256, 32), (1000, 96), (7, 5)])
@pytest.mark.parametrize("clip", [0.0, 0.05])
def test_lstm_cell_bwd(lh, orc, H, B, clip):
    rng = np.random.default_rng(50)
    pre = uni(rng, 4 * H, B, s=2.0)
    bias = uni(rng, 4 * H)
    c_prev = uni(rng, H, B)
    mask = (rng.random(B) > 0.2).astype(np.int32)
    gates, c, _ = orc.lstm_cell_fwd(pre, bias, c_prev, mask)
    dha, dhn, dcn = uni(rng, H, B, s=0.1), uni(rng, H, B, s=0.1), uni(rng, H, B, s=0.1)
    for above, nxt, cn in ((dha, dhn, dcn), (None, dhn, dcn), (dha, None, None)):
        want_dg, want_dc = orc.lstm_cell_bwd(gates, c, c_prev, mask, above, nxt, cn, clip, clip)
        dg = torch.empty(4 * H * B, device="cuda")
        dc = torch.empty(H * B, device="cuda")
        opt = lambda a: None if a is None else dev(a)
        lh.lstm_cell_bwd(H, B, dev(gates), dev(c), dev(c_prev), dev(mask), dg, dc, opt(above),
                         opt(nxt), opt(cn), clip, clip)
        assert_close(host(dg, (4 * H, B)), want_dg, "dgates")
        assert_close(host(dc, (H, B)), want_dc, "dc_prev")
        assert not np.any(host(dg, (4 * H, B))[:, mask == 0])
    # the consumer above read a dropped copy of h: its error returns through the same mask
    u = rng.random((H, B)).astype(np.float32)
    want_dg, want_dc = orc.lstm_cell_bwd(gates, c, c_prev, mask, dha, dhn, dcn, clip, clip, u, 0.7)
    dg = torch.empty(4 * H * B, device="cuda")
    dc = torch.empty(H * B, device="cuda")
    lh.lstm_cell_bwd(H, B, dev(gates), dev(c), dev(c_prev), dev(mask), dg, dc, dev(dha), dev(dhn),
                     dev(dcn), clip, clip, dev(u), 0.7)
    assert_close(host(dg, (4 * H, B)), want_dg, "dgates (dropout)")
    assert_close(host(dc, (H, B)), want_dc, "dc_prev (dropout)")


@pytest.mark.parametrize("H,B,ld,planes_above,planes_next", [(64, 12, 64, 2, 3), (100, 7, 100, 3, 1),
                                                             (48, 5, 52, 1, 2), (33, 4, 36, 2, 2),
                                                             (2048, 256, 2048, 2, 2)])
def test_lstm_cell_bwd_error_terms_as_partial_planes(lh, H, B, ld, planes_above, planes_next):
    """lh_lstm_cell_bwd_terms_f32 on the planes of a split product gives the bits lh_lstm_cell_bwd_f32
    gives on their sum, added in plane order from +0 as the product's reduction launch adds them
    (a -0 in the first plane included), with clamp and dropout mask on the sum."""
    rng = np.random.default_rng(52)
    gates = rng.random((4 * H, B)).astype(np.float32)
    gates[2 * H:3 * H] = 2 * gates[2 * H:3 * H] - 1
    c, c_prev = uni(rng, H, B), uni(rng, H, B)
    mask = (rng.random(B) > 0.2).astype(np.int32)
    dcn = uni(rng, H, B, s=0.1)
    u = rng.random((H, B)).astype(np.float32)

    def planes_of(n):
        p = np.zeros((n, B, ld), np.float32)
        p[:, :, :H] = rng.uniform(-0.1, 0.1, size=(n, B, H)).astype(np.float32)
        p[:, :, H:] = np.nan  # padding rows of a plane are never read
        p[0, 0, 0] = -0.0
        if n > 1:
            p[1:, 0, 0] = 0.0
        total = np.zeros((B, H), np.float32)
        for k in range(n):
            total = total + p[k, :, :H]
        return p, np.ascontiguousarray(total.T)  # H x B, as the plain entry point takes it

    pa, sum_a = planes_of(planes_above)
    pn, sum_n = planes_of(planes_next)
    for clip, drop in ((0.0, False), (0.05, True)):
        want_dg = torch.empty(4 * H * B, device="cuda")
        want_dc = torch.empty(H * B, device="cuda")
        lh.lstm_cell_bwd(H, B, dev(gates), dev(c), dev(c_prev), dev(mask), want_dg, want_dc, dev(sum_a),
                         dev(sum_n), dev(dcn), clip, clip, dev(u) if drop else None, 0.7)
        dg = torch.empty(4 * H * B, device="cuda")
        dc = torch.empty(H * B, device="cuda")
        da, dn = torch.from_numpy(pa).cuda(), torch.from_numpy(pn).cuda()
        lh.lstm_cell_bwd_terms(H, B, dev(gates), dev(c), dev(c_prev), dev(mask), dg, dc,
                               lh.error_term(da, planes_above, ld, B * ld), lh.error_term(dn, planes_next, ld, B * ld),
                               dev(dcn), clip, clip, dev(u) if drop else None, 0.7)
        torch.cuda.synchronize()
        assert torch.equal(dg.view(torch.int32), want_dg.view(torch.int32)), "dgates bits"
        assert torch.equal(dc.view(torch.int32), want_dc.view(torch.int32)), "dc_prev bits"
    with pytest.raises(lh.LinmtHipError):
        lh.lstm_cell_bwd_terms(H, B, dev(gates), dev(c), dev(c_prev), dev(mask), dg, dc,
                               lh.error_term(da, 9, ld, B * ld), None)
    with pytest.raises(lh.LinmtHipError):
        lh.lstm_cell_bwd_terms(H, B, dev(gates), dev(c), dev(c_prev), dev(mask), dg, dc,
                               lh.error_term(da, 1, H - 1), None)


@pytest.mark.parametrize("V,B", [(5000, 32), (30000, 24), (37, 5), (50000, 8)])
def test_softmax_xent_grad(lh, orc, V, B):
    rng = np.random.default_rng(51)
    z = uni(rng, V, B, s=4.0)
    bias = uni(rng, V)
    tgt = rng.integers(0, V, size=B).astype(np.int32)
    mask = (rng.random(B) > 0.25).astype(np.int32)
    tgt[mask == 0] = 0
    want_dz, want_lp, want_sum = orc.softmax_xent_grad(z, bias, tgt, mask)
    dz = torch.empty(V * B, device="cuda")
    lp = torch.zeros(B, dtype=torch.float64, device="cuda")
    acc = torch.zeros(1, dtype=torch.float64, device="cuda")
    lh.softmax_xent_grad(dev(z), V, dev(bias), V, B, dev(tgt), dev(mask), dz, V, lp, acc)
    assert_close(host(dz, (V, B)), want_dz, "dz", atol=1e-6)
    live = mask == 1
    assert_close(host(lp, (B,))[live], want_lp[live], "log p(target)", rtol=1e-5, atol=1e-5)
    assert_close(host(acc, (1,))[0], want_sum, "sum log p", rtol=1e-5, atol=1e-5)
    # columns of dz sum to zero, masked columns are zero, in place gives the same
    got = host(dz, (V, B))
    assert np.all(np.abs(got.sum(axis=0)) < 1e-4) and not np.any(got[:, ~live])
    zz = dev(z)
    acc.zero_()
    lh.softmax_xent_grad(zz, V, dev(bias), V, B, dev(tgt), dev(mask), zz, V, lp, acc)
    assert np.array_equal(host(zz, (V, B)), got)


@pytest.mark.parametrize("rows,cols,lda", [(4000, 777, 4000), (30000, 130, 30004), (5, 3, 5), (16, 1, 16)])
def test_rowsum_acc(lh, rows, cols, lda):
    rng = np.random.default_rng(52)
    A = uni(rng, lda, cols)
    out0 = uni(rng, rows)
    for beta in (0.0, 1.0):
        out = dev(out0)
        lh.rowsum_acc(dev(A), lda, rows, cols, out, beta)
        want = A[:rows].astype(np.float64).sum(axis=1) + beta * out0
        assert_close(host(out, (rows,)), want, "row sums", rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("E,U,N,zipf", [(1000, 300, 2000, False), (6, 3, 10, False),
                                        (512, 1, 40, False), (1024, 400, 9000, True),
                                        (37, 50, 3000, True)])
def test_embed_gather_grad(lh, E, U, N, zipf):
    """Against the dense per-id sum in float64 (the definition of the scatter).  zipf: token
    frequencies as in text, a few ids own thousands of columns and most own one or two."""
    rng = np.random.default_rng(53)
    dx = uni(rng, E, N)
    if zipf:
        p = np.arange(1, U + 1, dtype=np.float64) ** -1.1
        owner = rng.choice(U, size=N, p=p / p.sum())
        owner[rng.random(N) < 0.1] = -1
    else:
        owner = rng.integers(-1, U, size=N)  # -1: padding column, listed nowhere
    owner[:U] = np.arange(U)
    cols = [np.flatnonzero(owner == k) for k in range(U)]
    seg_start = np.concatenate([[0], np.cumsum([len(c) for c in cols])]).astype(np.int32)
    seg_cols = np.concatenate(cols).astype(np.int32)
    g0 = uni(rng, E, U)
    for beta in (0.0, 1.0):
        g = dev(g0)
        lh.embed_gather_grad(dev(dx), E, E, U, dev(seg_start), dev(seg_cols), g, E, beta)
        want = np.stack([dx[:, c].astype(np.float64).sum(axis=1) for c in cols], axis=1) + beta * g0
        assert_close(host(g, (E, U)), want, "small gradient", rtol=1e-4, atol=1e-5)
        g2 = dev(g0)
        lh.embed_gather_grad(dev(dx), E, E, U, dev(seg_start), dev(seg_cols), g2, E, beta)
        assert torch.equal(g, g2), "the sum must not depend on scheduling"
    # embedding dropout: each dx element passes through (mask < keep) / keep first
    u, keep = rng.random((E, N)).astype(np.float32), 0.8
    g = dev(g0)
    lh.embed_gather_grad(dev(dx), E, E, U, dev(seg_start), dev(seg_cols), g, E, 0.0, dev(u), keep)
    dxm = dx.astype(np.float64) * (u < keep) / keep
    want = np.stack([dxm[:, c].sum(axis=1) for c in cols], axis=1)
    assert_close(host(g, (E, U)), want, "small gradient (dropout)", rtol=1e-4, atol=1e-5)


def test_uniform_generator(lh):
    """Own design (the reference draws from cuRAND): values in (0, 1], reproducible per seed,
    independent of n, different across seeds, uniform to within sampling error."""
    n = 1 << 22
    a, b, c = (torch.empty(n, device="cuda") for _ in range(3))
    lh.uniform(a, n, 1234)
    lh.uniform(b, n, 1234)
    lh.uniform(c, n // 3, 1235)
    A, B_, C_ = host(a, (n,)), host(b, (n,)), host(c, (n,))[: n // 3]
    assert np.array_equal(A, B_)
    assert A.min() > 0.0 and A.max() <= 1.0
    assert not np.array_equal(A[: n // 3], C_)
    assert abs(A.mean() - 0.5) < 1e-3 and abs((A < 0.8).mean() - 0.8) < 1e-3
    hist = np.histogram(A, bins=64, range=(0, 1))[0] / n
    assert np.all(np.abs(hist - 1 / 64) < 5e-4)
    assert abs(np.corrcoef(A[:-1], A[1:])[0, 1]) < 3e-3
    d = torch.empty(1000, device="cuda")
    lh.uniform(d, 1000, 1234)
    assert np.array_equal(host(d, (1000,)), A[:1000])


@pytest.mark.parametrize("H,B", [(1000, 64), (9, 4)])
def test_attn_delta(lh, orc, H, B):
    rng = np.random.default_rng(54)
    dht, feed, ht = uni(rng, H, B), uni(rng, H, B), np.tanh(uni(rng, H, B, s=2))
    mask = (rng.random(B) > 0.3).astype(np.int32)
    for f, clip in ((None, 0.0), (feed, 0.0), (feed, 0.3)):
        want = orc.attn_delta(dht, ht, mask, f, clip)
        out = torch.empty(H * B, device="cuda")
        lh.attn_delta(H, B, dev(dht), dev(ht), dev(mask), out, None if f is None else dev(f), clip)
        assert_close(host(out, (H, B)), want, "delta")


@pytest.mark.parametrize("H,B,S,D", [(256, 16, 30, 10), (1000, 12, 60, 10), (12, 5, 9, 2), (64, 6, 20, -1)])
def test_attn_core_bwd(lh, orc, H, B, S, D):
    rng = np.random.default_rng(55)
    lens = rng.integers(max(2, S // 3), S + 1, size=B)
    lens[0] = S
    bi = np.concatenate([lens, S - lens]).astype(np.int32)
    mask = np.ones(B, np.int32)
    mask[-1] = 0
    hs = uni(rng, S * B * H, s=0.5)
    tanh1 = np.tanh(uni(rng, H, B))
    v_p = uni(rng, H, s=0.3)
    wa = uni(rng, H, B, s=0.3)
    dctx = uni(rng, H, B, s=0.2)
    fwd = orc.attn_core_fwd(H, B, D, S, S, tanh1, v_p, wa, hs, B * H, H, None, bi, mask)
    dhs0 = uni(rng, S * B * H, s=0.1)
    want = orc.attn_core_bwd(H, B, D, S, S, dctx, tanh1, v_p, wa, hs, B * H, H, bi, fwd, dhs0)
    dhs = dev(dhs0)
    hsum, u, w = (torch.zeros(H * B, device="cuda") for _ in range(3))
    lh.attn_core_bwd(H, B, D, S, S, dev(dctx), dev(tanh1), dev(v_p), dev(wa), dev(hs), B * H, H,
                     dev(bi), dev(fwd["p_t"]), dev(fwd["sigma"]), dev(fwd["indices"]),
                     dev(fwd["align"]), dev(fwd["cached_exp"]), dhs, hsum, u, w)
    assert_close(host(hsum, (H, B)), want["hsum"], "hsum", atol=2e-5)
    assert_close(host(dhs, (S * B * H,)), want["dhs"], "dhs", atol=2e-5)
    if D >= 0:
        assert_close(host(u, (H, B)), want["u"], "u", atol=2e-5)
        assert_close(host(w, (H, B)), want["w"], "w", atol=2e-5)


def test_grad_sumsq_and_sgd_step(lh):
    """Closed forms: sum of squares of the scaled gradient; clipped, scaled SGD step; cleared
    gradient; strided gate views and the indexed (embedding) update."""
    rng = np.random.default_rng(56)
    rows, cols, ld = 1000, 700, 4000
    G = uni(rng, ld, cols)
    T0 = uni(rng, ld, cols)
    ws = torch.zeros(lh.LH_SUMSQ_WORKSPACE, dtype=torch.float64, device="cuda")
    acc = torch.zeros(1, dtype=torch.float64, device="cuda")
    scale = 1.0 / 64
    g = dev(G)
    lh.grad_sumsq(g[1000:], rows, cols, ld, scale, ws, acc)       # one gate block of a stacked matrix
    lh.grad_sumsq(g, ld * cols, 1, ld * cols, scale, ws, acc)      # plus the whole matrix, contiguous
    want = (np.sum((G[1000:2000].astype(np.float64) * scale) ** 2)
            + np.sum((G.astype(np.float64) * scale) ** 2))
    assert_close(host(acc, (1,))[0], want, "sum of squares", rtol=1e-6, atol=0)
    # contiguous runs of every length class: a ragged tail, fewer than four values, many blocks'
    # worth, and a start that is not 16-byte aligned
    flat = G.ravel(order="F")
    for start, n in ((0, 3), (0, 4), (0, 16385), (4, 1000003), (1, 70001), (2, 2799998)):
        acc1 = torch.zeros(1, dtype=torch.float64, device="cuda")
        lh.grad_sumsq(g[start:], n, 1, n, scale, ws, acc1)
        want1 = np.sum((flat[start:start + n].astype(np.float64) * scale) ** 2)
        assert_close(host(acc1, (1,))[0], want1, f"sum of squares of {n} from {start}", rtol=1e-6, atol=0)
    nrm = np.sqrt(want)
    for clip, ind in ((0.5 * nrm, 0.0), (2 * nrm, 0.0), (0.5 * nrm, 1e-3)):
        theta, g = dev(T0), dev(G)
        lh.sgd_step(theta[1000:], ld, g[1000:], ld, rows, cols, 0.7, scale, sumsq=acc,
                    norm_clip=float(clip), individual_clip=ind)
        f = min(1.0, clip / nrm)
        v = G[1000:2000].astype(np.float64) * scale * f
        if ind > 0:
            v = np.clip(v, -ind, ind)
        want_t = T0.astype(np.float64).copy()
        want_t[1000:2000] += 0.7 * v
        assert_close(host(theta, (ld, cols)), want_t, "theta", rtol=1e-5, atol=1e-7)
        got_g = host(g, (ld, cols))
        assert not np.any(got_g[1000:2000]) and np.array_equal(got_g[:1000], G[:1000])
    # indexed columns (sparse embedding update), one and several unique ids
    for U in (1, 37):
        E, V = 64, 200
        W0, SG = uni(rng, E, V), uni(rng, E, U)
        uniq = rng.permutation(V)[:U].astype(np.int32)
        W, sg = dev(W0), dev(SG)
        lh.sgd_step(W, E, sg, E, E, U, 0.5, 0.25, col_index=dev(uniq))
        want_w = W0.astype(np.float64).copy()
        want_w[:, uniq] += 0.5 * 0.25 * SG
        assert_close(host(W, (E, V)), want_w, "embedding", rtol=1e-6, atol=1e-7)
        assert not np.any(host(sg, (E, U)))
