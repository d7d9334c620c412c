"""The tile configuration the GEMM cost model picks for the three matrix products of a decoding
step, at the column counts a stream of 64 sentences x beam 12 runs them (768) and at two counts
below it (672, 576), against a sweep over every configuration the library has: the stacked gate
product that ends in the LSTM cell (4000 x N x (1000 + 1000), replaces the eight cuBLAS calls per
cell of src/node_hidden_to_hidden.h:248-430), the output projection (30000 x N x 1000,
src/layer_loss.h:797-806) and the attention projections (2000 x N x 1000,
src/layer_attention.h:282-330).  The choice must be within 8% of the best configuration of the sweep
(measured: 0-5%; launch times on one GPU repeat to about 3%; the table the model reads was measured on the same
kernels by csrc/tune_gemm.py).  Collected late on purpose: a timing assertion must not hide the
parity tests behind it."""
import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]
H, V = 1000, 30000


def _time(fn, launches=20, reps=3):
    fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3 / launches)
    return best


@pytest.mark.parametrize("N", [768, 672, 576])
def test_cost_model_choice_is_close_to_the_best_of_the_sweep(lh, N):
    L = lh.load()
    n_cfg = L.lh_gemm_set_config_override(-1)
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(N)
    r = lambda n, s=1.0: (torch.rand(n, device=dev, generator=g) * 2 - 1) * s  # noqa: E731
    Wx, Wh, x, h = r(4 * H * H, 0.08), r(4 * H * H, 0.08), r(H * N), r(H * N)
    bias, cp = r(4 * H, 0.08), r(H * N)
    mask = torch.ones(N, dtype=torch.int32, device=dev)
    c, ho = torch.empty(H * N, device=dev), torch.empty(H * N, device=dev)
    segs = [(Wx, 4 * H, x, H, H), (Wh, 4 * H, h, H, H)]
    D, logits = r(V * H, 0.08), torch.empty(V * N, device=dev)
    Wpc, pc = r(2 * H * H, 0.08), torch.empty(2 * H * N, device=dev)
    ws = torch.empty(16 << 20, device=dev)
    shapes = {
        "gate product + LSTM cell": lambda: lh.gate_gemm_lstm_cell(H, N, segs, bias, cp, mask, c, ho,
                                                                   workspace_bytes=64 << 20),
        "output projection": lambda: lh.gemm(V, N, [(D, V, x, H, H)], logits, V, workspace=ws),
        "attention projections": lambda: lh.gemm(2 * H, N, [(Wpc, 2 * H, h, H, H)], pc, 2 * H,
                                                 act=lh.LH_ACT_TANH, act_rows=H, workspace=ws),
    }
    try:
        for _ in range(100):  # the GPU's clocks settle under matrix load before anything is timed
            shapes["output projection"]()
        for name, fn in shapes.items():
            times = {}
            for cfg in range(n_cfg):
                L.lh_gemm_set_config_override(cfg)
                try:
                    times[cfg] = _time(fn)
                except lh.LinmtHipError:  # a configuration this product cannot use (e.g. no room for the cell)
                    pass
                if cfg == n_cfg // 2:
                    L.lh_gemm_set_config_override(-1)
                    chosen = _time(fn)
            best_cfg = min(times, key=times.get)
            ratio = chosen / times[best_cfg]
            for attempt in range(3):  # a second and third look before a timing difference counts
                if ratio <= 1.08:
                    break
                L.lh_gemm_set_config_override(best_cfg)
                best_again = _time(fn, launches=50, reps=5)
                L.lh_gemm_set_config_override(-1)
                ratio = _time(fn, launches=50, reps=5) / best_again
            print(f"N={N} {name}: chosen {chosen:.1f} us, best of the sweep {times[best_cfg]:.1f} us "
                  f"(configuration {best_cfg} = {lh.gemm_config_info(best_cfg)}), ratio {ratio:.3f}", flush=True)
            assert ratio <= 1.08, (name, N, ratio, best_cfg)
    finally:
        L.lh_gemm_set_config_override(-1)
