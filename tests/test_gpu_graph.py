"""The three passes recorded into a HIP graph and replayed: every launch of the
library is an ordinary kernel launch on the caller's stream (no allocation, no
memset node, no host synchronisation), so a training step can be captured once
and replayed.  Each replay is checked against the eager result on the same
inputs, with eager work and synchronisations between replays."""
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def cp4():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import paralleltnnlayers_amd as p
    p.lib()
    return p


# (N, C, H, W, T, Y, R): matrix-core kernels / odd channel counts (backward-filter by the dense
# gradient) / channels above 256 / few channels on a wide plane (the few-channel forward kernel,
# backward-filter by the dense gradient over several tiles per workgroup)
SHAPES = [(2, 64, 28, 28, 64, 3, 16), (3, 5, 9, 9, 7, 3, 3), (1, 320, 14, 14, 64, 3, 32),
          (4, 16, 192, 320, 16, 3, 16)]


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_replays_match_eager(cp4, dims):
    N, C, H, W, T, Y, R = dims
    pad = Y // 2
    gen = torch.Generator(device="cuda").manual_seed(sum(dims))
    mk = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    x, dy = mk(N, C, H, W), mk(N, T, H, W)
    fac = [mk(d, R) / R ** 0.25 for d in (T, C, Y, Y)]
    s = cp4.capi.shape_for(x.shape, *fac, pad)
    ws = torch.empty(cp4.backward_filter_workspace_bytes(s) // 4 + 1, device="cuda")
    y, dx = torch.empty(N, T, H, W, device="cuda"), torch.empty(N, C, H, W, device="cuda")

    def step():
        cp4.conv2d_forward(x, *fac, pad, out=y)
        cp4.conv2d_backward_data(dy, *fac, pad, out=dx)
        return cp4.conv2d_backward_filter(x, dy, *fac, pad, workspace=ws)

    step()                      # eager warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        grads = step()
    torch.cuda.synchronize()

    for replay in range(3):
        x.copy_(mk(N, C, H, W))
        dy.copy_(mk(N, T, H, W))
        for f, d in zip(fac, (T, C, Y, Y)):
            f.copy_(mk(d, R) / R ** 0.25)
        graph.replay()
        torch.cuda.synchronize()
        got = [y.clone(), dx.clone()] + [g.clone() for g in grads]
        y.zero_(), dx.zero_()
        want_grads = step()     # eager, same inputs
        torch.cuda.synchronize()
        want = [y.clone(), dx.clone()] + list(want_grads)
        for name, a, b in zip(("y", "dx", "dFK", "dFC", "dFH", "dFW"), got, want):
            scale = b.abs().max().item()
            assert (a - b).abs().max().item() <= 1e-6 * scale, (replay, name)


def test_empty_batch_gradients_capture(cp4):
    """N == 0 writes zero gradients with a fill kernel, which a graph may hold."""
    x, dy = torch.empty(0, 8, 6, 6, device="cuda"), torch.empty(0, 4, 6, 6, device="cuda")
    fac = [torch.randn(d, 2, device="cuda") for d in (4, 8, 3, 3)]
    ws = torch.empty(16, device="cuda")
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        grads = cp4.conv2d_backward_filter(x, dy, *fac, 1, workspace=ws)
    for _ in range(2):
        for g in grads:
            g.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        assert all(float(g.abs().max()) == 0.0 for g in grads)


@pytest.mark.parametrize("dims", [(2, 64, 28, 28, 64, 3, 12), (2, 24, 14, 14, 24, 5, 6)],
                         ids=lambda d: "x".join(map(str, d)))
def test_cp3_passes_replay(cp4, dims):
    """The 3-factor CP passes (factor rewriting kernels included) with a caller-owned
    workspace: one-pass kernel with the depthwise tap step / expanded factors."""
    N, C, H, W, T, Y, R = dims
    pad = Y // 2
    gen = torch.Generator(device="cuda").manual_seed(sum(dims))
    mk = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    x, dy = mk(N, C, H, W), mk(N, T, H, W)
    K = [mk(C, R), mk(Y, Y, R), mk(R, T)]
    s = cp4.cp3_shape_for(x.shape, *K, pad)
    import ctypes
    nbytes = cp4.lib().cp3_conv2d_forward_workspace_bytes(ctypes.byref(s))
    ws = [torch.empty(nbytes, device="cuda", dtype=torch.uint8) for _ in range(2)]
    y, dx = torch.empty(N, T, H, W, device="cuda"), torch.empty(N, C, H, W, device="cuda")

    def step():
        cp4.cp3_conv2d_forward(x, *K, pad=pad, out=y, workspace=ws[0])
        cp4.cp3_conv2d_backward_data(dy, *K, pad=pad, out=dx, workspace=ws[1])

    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    torch.cuda.synchronize()
    for replay in range(3):
        x.copy_(mk(N, C, H, W))
        dy.copy_(mk(N, T, H, W))
        for k in K:
            k.copy_(mk(*k.shape))
        graph.replay()
        torch.cuda.synchronize()
        got = [y.clone(), dx.clone()]
        y.zero_(), dx.zero_()
        step()
        torch.cuda.synchronize()
        for name, a, b in zip(("y", "dx"), got, (y, dx)):
            assert (a - b).abs().max().item() <= 1e-6 * b.abs().max().item(), (replay, name)
