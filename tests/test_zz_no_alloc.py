"""lh_gemm_noalloc_f32 -- the K-split product over the library's own device scratch array, for
callers that cannot allocate -- against lh_gemm_ws_f32 with a caller workspace of the same size.
Both take the same tile / split decision, so the results must agree bit for bit.  Two calls in a
row, the second on a smaller product, so that whatever the first call left in the shared array
is there when the second runs."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(np.asarray(a).T)).cuda().reshape(-1)


def host(t, shape):
    return t.cpu().numpy().reshape(shape[::-1]).T


def _case(lh, rng, M, N, Ks, tA, tX, epilogue, check_memory=True):
    As = [rng.uniform(-0.5, 0.5, size=((K, M) if tA else (M, K))).astype(np.float32) for K in Ks]
    Xs = [rng.uniform(-1, 1, size=((N, K) if tX else (K, N))).astype(np.float32) for K in Ks]
    segs = [(dev(A), A.shape[0], dev(X), X.shape[0], K) for A, X, K in zip(As, Xs, Ks)]
    acc = sum((A.T if tA else A).astype(np.float64) @ (X.T if tX else X) for A, X in zip(As, Xs))
    C0 = rng.uniform(-1, 1, size=(M, N)).astype(np.float32)
    kw, want = {}, acc
    if epilogue:
        bias = rng.uniform(-1, 1, size=M).astype(np.float32)
        cmask = rng.integers(0, 2, size=N).astype(np.int32)
        kw = dict(alpha=-0.5, beta=0.25, bias=dev(bias), act=lh.LH_ACT_TANH, colmask=dev(cmask))
        want = np.tanh(-0.5 * acc + 0.25 * C0 + bias[:, None]) * cmask[None, :]
    ws = torch.full((lh.LH_GEMM_NOALLOC_WS_BYTES // 4,), float("nan"), device="cuda")
    ref = dev(C0)
    lh.gemm(M, N, segs, ref, M, transA=tA, transX=tX, workspace=ws, **kw)
    got = dev(C0)
    # nothing is allocated by the call: the caching allocator's books and the device's free memory
    # are the same before and after it (the first call on the device has already happened: init)
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
    lh.gemm_noalloc(M, N, segs, got, M, transA=tA, transX=tX, **kw)
    torch.cuda.synchronize()
    after = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
    if check_memory:
        assert after[:2] == before[:2] and after[2] >= before[2], (before, after)
    return host(got, (M, N)), host(ref, (M, N)), want


def test_noalloc_gemm_equals_workspace_gemm(lh):
    from conftest import assert_close
    rng = np.random.default_rng(77)
    L = lh.load()
    # (4000, 96, K 2000): a decoding step's recurrent gate product, which the cost model splits;
    # then smaller products (one of them forced to split, one with a ragged scalar-path shape)
    calls = [((4000, 96, (1000, 1000), False, False, True), 0),
             ((1000, 48, (1000,), True, False, False), 0),
             ((200, 76, (100, 36), False, False, True), 3),
             ((37, 13, (101,), False, False, True), 0)]
    split_seen = False
    lh.gemm_noalloc_init()
    # each kernel instance's one-time set-up (the LDS limit) happens on a first, unchecked round
    try:
        for (M, N, Ks, tA, tX, epi), forced in calls:
            L.lh_gemm_set_splits_override(forced)
            _case(lh, np.random.default_rng(1), M, N, Ks, tA, tX, epi, check_memory=False)
    finally:
        L.lh_gemm_set_splits_override(0)
    try:
        for (M, N, Ks, tA, tX, epi), forced in calls:
            L.lh_gemm_set_splits_override(forced)
            got, ref, want = _case(lh, rng, M, N, Ks, tA, tX, epi)
            what = f"{(M, N, Ks, tA, tX)} forced split {forced}"
            assert np.array_equal(got, ref), what + ": differs from lh_gemm_ws_f32"
            assert_close(got, want, what)
            split_seen = split_seen or forced > 1
    finally:
        L.lh_gemm_set_splits_override(0)
    assert split_seen


def test_noalloc_gemm_rejects_oversize(lh):
    # two planes of a 4096 x 2048 product are 64 MiB: beyond the 32 MiB array
    a = torch.zeros(16, device="cuda")
    with pytest.raises(lh.LinmtHipError, match="LH_GEMM_NOALLOC_WS_BYTES"):
        lh.gemm_noalloc(4096, 2048, [(a, 4096, a, 4, 4)], a, 4096)
