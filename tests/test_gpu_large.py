"""Tensors past 2^31 elements (8 GiB each): element offsets no longer fit 32 bits,
so every kernel has to carry 64-bit image bases.  The CPU oracle would take
minutes at this size; the checks use properties that do not depend on it:
images are independent in forward / backward-data (an image of the big batch
equals the same image run alone), and the factor gradients are a sum over
images (a batch whose x is zero except in the last image has that image's
gradients)."""
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

N, C, K, H, W, Y, R = 680, 256, 256, 112, 112, 3, 32      # 680*256*112*112 = 2.18e9 > 2^31


@pytest.fixture(scope="module")
def cp4():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    if torch.cuda.get_device_properties(0).total_memory < 64 * 2 ** 30:
        pytest.skip("needs 64 GiB of device memory")
    import paralleltnnlayers_amd as p
    p.lib()
    return p


@pytest.fixture(scope="module")
def operands(cp4):
    gen = torch.Generator(device="cuda").manual_seed(20)
    x = torch.randn(N, C, H, W, device="cuda", generator=gen)
    fac = [torch.randn(d, R, device="cuda", generator=gen) / (R * C) ** 0.25 for d in (K, C, Y, Y)]
    n_elements = x.numel()
    assert n_elements > 2 ** 31
    yield x, fac
    del x
    torch.cuda.empty_cache()


def close(a, b, tol):
    return (a - b).abs().max().item() <= tol * b.abs().max().item()


def test_forward_images_past_4gib(cp4, operands):
    x, fac = operands
    y = cp4.conv2d_forward(x, *fac, pad=1)
    for n in (0, N // 2, N - 1):
        alone = cp4.conv2d_forward(x[n:n + 1].contiguous(), *fac, pad=1)
        assert close(y[n:n + 1], alone, 1e-5), n


def test_backward_data_images_past_4gib(cp4, operands):
    dy, fac = operands          # K == C: the same tensor serves as the upstream gradient
    dx = cp4.conv2d_backward_data(dy, *fac, pad=1)
    for n in (0, N // 2, N - 1):
        alone = cp4.conv2d_backward_data(dy[n:n + 1].contiguous(), *fac, pad=1)
        assert close(dx[n:n + 1], alone, 1e-5), n


def test_backward_filter_last_image_past_4gib(cp4, operands):
    dy, fac = operands
    x = torch.zeros_like(dy)
    gen = torch.Generator(device="cuda").manual_seed(21)
    x[N - 1] = torch.randn(C, H, W, device="cuda", generator=gen)
    got = cp4.conv2d_backward_filter(x, dy, *fac, pad=1)
    want = cp4.conv2d_backward_filter(x[N - 1:].contiguous(), dy[N - 1:].contiguous(), *fac, pad=1)
    for name, a, b in zip(("dFK", "dFC", "dFH", "dFW"), got, want):
        assert close(a, b, 1e-4), name
