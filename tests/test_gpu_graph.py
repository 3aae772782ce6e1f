"""HIP-graph capture of the ops: a captured forward+backward must reproduce the eager result on every
replay, with eager work and synchronisations between replays."""
import numpy as np
import pytest
import torch

from helpers import conv_case, dense_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = fn()
    torch.cuda.synchronize()
    return g, out


def test_dense_forward_backward_graph_replays_match_eager():
    import snntc_amd as snn
    x, w, p, g = dense_case(0, 64, 300, 130, True, "baseline")
    X, W, G = t(x), t(w), t(g)

    def step():
        y = snn.snnfc(X, W, p)
        dx, dw, _ = snn.snnfc_grad(G, X, W, p, y, want_dparams=False)
        return y, dx, dw

    ref = [v.clone() for v in step()]
    graph, out = _capture(step)
    for i in range(4):
        for o in out:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for o, r in zip(out, ref):
            assert torch.equal(o, r), f"replay {i} differs from the eager result"
        # eager work of the same ops (different input) between replays
        snn.snnfc(X * 1.5, W, p)
        torch.cuda.synchronize()
        X.copy_(t(x))


def test_conv_forward_backward_graph_replays_match_eager():
    import snntc_amd as snn
    _, xpad, w, p, g = conv_case(1, 2, 12, 12, 32, 32, 3, 3, 1, 1, True, True, "baseline")
    X, W, G = t(xpad), t(w), t(g)

    def step():
        y = snn.snncv(X, W, p)
        dx, dw, _ = snn.snncv_grad(G, X, W, p, y, want_dparams=False)
        return y, dx, dw

    ref = [v.clone() for v in step()]
    graph, out = _capture(step)
    for i in range(3):
        for o in out:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for o, r in zip(out, ref):
            assert torch.equal(o, r), f"replay {i} differs from the eager result"
        snn.snncv(X + 0.25, W, p)
        torch.cuda.synchronize()


def test_optional_gradient_outputs():
    import snntc_amd as snn
    x, w, p, g = dense_case(2, 16, 70, 20, True, "baseline")
    X, W, G = t(x), t(w), t(g)
    y = snn.snnfc(X, W, p)
    dx, dw, dp = snn.snnfc_grad(G, X, W, p, y)
    dx2, none_w, none_p = snn.snnfc_grad(G, X, W, p, y, want_dparams=False, want_dw=False)
    none_x, dw2, _ = snn.snnfc_grad(G, X, W, p, y, want_dparams=False, want_dx=False)
    assert none_w is None and none_p is None and none_x is None
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2) and torch.all(dp == 0)


def test_workspace_of_a_captured_graph_survives_a_later_larger_capture():
    """Two graphs that share one memory pool: the second needs a larger scratch buffer than the first.
    The first graph's scratch must stay its own, so replaying it after the second capture (and after
    the second graph has run) still gives the eager result."""
    import snntc_amd as snn
    xs, ws, ps, _ = dense_case(3, 8, 100, 40, True, "baseline")
    xl, wl, pl, _ = dense_case(4, 96, 900, 120, True, "baseline")
    Xs, Ws, Xl, Wl = t(xs), t(ws), t(xl), t(wl)
    ref_s = snn.snnfc(Xs, Ws, ps).clone()
    ref_l = snn.snnfc(Xl, Wl, pl).clone()
    torch.cuda.synchronize()

    pool = torch.cuda.graph_pool_handle()
    g1 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1, pool=pool):
        out_s = snn.snnfc(Xs, Ws, ps)
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2, pool=pool):
        out_l = snn.snnfc(Xl, Wl, pl)
        keep = [torch.full((1 << 16,), 7.0, device=DEV) for _ in range(4)]   # more tensors from the shared pool
    torch.cuda.synchronize()
    for i in range(3):
        g2.replay()
        g1.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_s, ref_s), f"round {i}: the first graph's result changed"
        g2.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_l, ref_l), f"round {i}: the second graph's result changed"
        assert all(bool((k == 7.0).all()) for k in keep), "scratch of the first graph overwrote live tensors"
        snn.snnfc(Xl, Wl, pl)                                                 # eager work between replays
        torch.cuda.synchronize()
