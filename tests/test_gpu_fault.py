"""Failure handling of the device code, through the C ABI.

The producer / consumer kernels wait for each other's LDS counters with a
bounded number of polls.  A wait that runs out must never end in a silently
wrong result: the wave records the fault and stops, and the host sees
CP4_ERR_DEVICE from cp4_device_status and from the timing loops.  The test
forces that from the host by setting the bound to one poll
(cp4_set_spin_limit): every wave still ends normally, nothing hangs.

Also here: argument errors that need device tensors (an undersized workspace of
another dtype) and the documented behaviour on non-finite inputs.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from paralleltnnlayers_amd.configs import WORKLOADS, make_inputs  # noqa: E402

FACTORS = ("FK", "FC", "FH", "FW")


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def pipe_variant(cp4, s):
    for v, name, ok in cp4.forward_variants(s):
        if name == "mfma_bf16x3_pipe":
            assert ok, "the workload must run on the producer / consumer kernel"
            return v
    raise AssertionError("variant missing")


@pytest.mark.parametrize("name", ["C2", "C3"])
def test_wait_timeout_is_reported_not_silent(cp4, oracle, name):
    w = WORKLOADS[name]
    a = make_inputs(w, seed=0)
    f = [dev(a[k]) for k in FACTORS]
    x = dev(a["x"])
    s = cp4.capi.shape_for(x.shape, *f, w.pad)
    v = pipe_variant(cp4, s)
    assert cp4.device_status_detail()[0] == cp4.capi.OK      # clean before
    cp4.set_spin_limit(1)
    try:
        y = torch.zeros((w.N, w.T, w.H, w.W), device="cuda")
        cp4.conv2d_forward(x, *f, pad=w.pad, out=y, variant=v)   # asynchronous: returns OK
        st, detail = cp4.device_status_detail()
        assert st == cp4.capi.ERR_DEVICE, "a wait that ran out must be reported"
        assert detail[0] != 0 and 1 <= detail[3] <= 7 and 0 <= detail[2] < 16
        assert b"wait" in cp4.lib().cp4_last_error_message()
        # the record is cleared by reading it
        assert cp4.device_status_detail()[0] == cp4.capi.OK
        # the timed loop synchronises and reports the fault itself
        with pytest.raises(cp4.Cp4Error) as ei:
            cp4.time_forward(x, *f, y, w.pad, warmup=0, profcount=2)
        assert ei.value.status == cp4.capi.ERR_DEVICE
        assert cp4.device_status_detail()[0] == cp4.capi.OK
    finally:
        cp4.set_spin_limit(0)
    # with the default bound the same call is complete and correct again
    y = cp4.conv2d_forward(x, *f, pad=w.pad, variant=v)
    cp4.device_status()
    want = oracle.forward(a["x"], a["FK"], a["FC"], a["FH"], a["FW"], w.pad)
    err = np.abs(y.cpu().numpy() - want).max() / np.abs(want).max()
    assert err <= 1e-4


def test_undersized_workspace_of_another_dtype_is_rejected(cp4):
    w = WORKLOADS["C1"]
    a = make_inputs(w, seed=0)
    f = [dev(a[k]) for k in FACTORS]
    x, dy = dev(a["x"]), dev(a["dy"])
    s = cp4.capi.shape_for(x.shape, *f, w.pad)
    need = cp4.backward_filter_workspace_bytes(s)
    assert need > 16
    # need / 4 BYTES: enough elements if they were counted as floats, a quarter of the bytes
    small = torch.empty(need // 4 + 1, device="cuda", dtype=torch.uint8)
    with pytest.raises(cp4.Cp4Error) as ei:
        cp4.conv2d_backward_filter(x, dy, *f, pad=w.pad, workspace=small)
    assert ei.value.status == cp4.capi.ERR_WORKSPACE
    with pytest.raises(cp4.Cp4Error) as ei:
        cp4.time_backward_filter(x, dy, *f, w.pad, warmup=0, profcount=1, workspace=small)
    assert ei.value.status == cp4.capi.ERR_WORKSPACE
    # a byte workspace of the full size is accepted and gives the same gradients
    full = torch.empty(need + 8, device="cuda", dtype=torch.uint8)
    got = cp4.conv2d_backward_filter(x, dy, *f, pad=w.pad, workspace=full)
    ref = cp4.conv2d_backward_filter(x, dy, *f, pad=w.pad)
    for g, r in zip(got, ref):
        assert torch.equal(g, r)


@pytest.mark.parametrize("name", ["C1", "C2"])
@pytest.mark.parametrize("bad", [float("inf"), float("-inf"), float("nan")])
def test_non_finite_activation_poisons_only_what_it_touches(cp4, name, bad):
    """An Inf or NaN in x gives NaN in every output whose sum it enters (the exact
    three-way split of Inf leaves Inf - Inf) and leaves every other output
    bit-identical to the run on finite data."""
    w = WORKLOADS[name]
    a = make_inputs(w, seed=0)
    f = [dev(a[k]) for k in FACTORS]
    x = dev(a["x"])
    s = cp4.capi.shape_for(x.shape, *f, w.pad)
    n0, c0, h0, w0 = w.N - 1, w.C // 2, 7, 11
    for v in [v for v, _, ok in cp4.forward_variants(s) if ok]:
        clean = cp4.conv2d_forward(x, *f, pad=w.pad, variant=v).cpu().numpy()
        xb = x.clone()
        xb[n0, c0, h0, w0] = bad
        y = cp4.conv2d_forward(xb, *f, pad=w.pad, variant=v).cpu().numpy()
        touched = np.zeros(y.shape, dtype=bool)
        q = w.Y - 1 - w.pad
        touched[n0, :, max(h0 - q, 0):h0 + w.pad + 1, max(w0 - q, 0):w0 + w.pad + 1] = True
        assert not np.isfinite(y[touched]).any(), f"variant {v}: a touched output stayed finite"
        assert np.array_equal(y[~touched], clean[~touched]), f"variant {v}: untouched outputs changed"
    cp4.device_status()


def _factors(rng, T, C, Y, R):
    return [(rng.standard_normal((d, R)) / np.sqrt(R)).astype(np.float32) for d in (T, C, Y, Y)]


def _build_cases(cp4, oracle):
    """(name, launch() -> device tensor, want() -> numpy reference, tolerance): one shape
    per build of the producer / consumer kernel, each through the entry point that
    reaches it."""
    rng = np.random.default_rng(5)
    cases = []

    def add(name, launch, want, tol=1e-4):
        cases.append((name, launch, want, tol))

    # wide plane -> the tiled build (the variant is named, so the route is certain)
    x = rng.standard_normal((2, 32, 12, 320)).astype(np.float32)
    f = _factors(rng, 32, 32, 3, 16)
    s = cp4.capi.shape_for(x.shape, *[dev(v) for v in f], 1)
    tiled = [v for v, n, ok in cp4.forward_variants(s) if n == "mfma_bf16x3_pipe_tiled" and ok]
    assert tiled, "the wide plane must be taken by the tiled build"
    add("tiled", lambda x=x, f=f: cp4.conv2d_forward(dev(x), *[dev(v) for v in f], pad=1, variant=tiled[0]),
        lambda x=x, f=f: oracle.forward(x, *f, 1))
    # 48 ranks -> two rank passes
    x2 = rng.standard_normal((2, 32, 16, 16)).astype(np.float32)
    f2 = _factors(rng, 32, 32, 3, 48)
    s2 = cp4.capi.shape_for(x2.shape, *[dev(v) for v in f2], 1)
    rp = [v for v, n, ok in cp4.forward_variants(s2) if n == "mfma_bf16x3_pipe_rank_passes" and ok]
    assert rp
    add("rank passes", lambda: cp4.conv2d_forward(dev(x2), *[dev(v) for v in f2], pad=1, variant=rp[0]),
        lambda: oracle.forward(x2, *f2, 1))
    # bias + ReLU -> the epilogue build
    x3 = rng.standard_normal((4, 64, 32, 32)).astype(np.float32)
    f3 = _factors(rng, 64, 64, 3, 16)
    b3 = rng.standard_normal(64).astype(np.float32)
    add("epilogue", lambda: cp4.conv2d_forward_bias_act(dev(x3), *[dev(v) for v in f3], dev(b3), "relu", pad=1),
        lambda: np.maximum(oracle.forward(x3, *f3, 1) + b3[None, :, None, None], 0))
    # 16-bit activations
    xb = torch.from_numpy(x3).cuda().to(torch.bfloat16)
    add("bfloat16", lambda: cp4.conv2d_forward_bf16(xb, *[dev(v) for v in f3], pad=1).float(),
        lambda: oracle.forward(xb.float().cpu().numpy(), *f3, 1), 1e-2)
    xh = torch.from_numpy(x3).cuda().half()
    add("float16", lambda: cp4.conv2d_forward_f16(xh, *[dev(v) for v in f3], pad=1).float(),
        lambda: oracle.forward(xh.float().cpu().numpy(), *f3, 1), 2e-3)
    # stride 2: forward, and the adjoint mode behind backward-data
    g = cp4.geometry(cp4.capi.shape_for(x3.shape, *[dev(v) for v in f3], 0), 2, "same")
    og = oracle.geometry_same(32, 32, 3, 3, 2)
    add("strided", lambda: cp4.conv2d_forward_ex(dev(x3), *[dev(v) for v in f3], g),
        lambda: oracle.forward_geom(x3, *f3, og))
    dy = rng.standard_normal((4, 64, og.out_h, og.out_w)).astype(np.float32)
    add("strided adjoint", lambda: cp4.conv2d_backward_data_ex(dev(dy), (32, 32), *[dev(v) for v in f3], g),
        lambda: oracle.backward_data_geom(dy, (32, 32), *f3, og))
    # the 3-factor op -> the 2-D-tap build
    K0 = (rng.standard_normal((64, 16)) / 4).astype(np.float32)
    K1 = (rng.standard_normal((3, 3, 16)) / 3).astype(np.float32)
    K2 = (rng.standard_normal((16, 64)) / 4).astype(np.float32)
    add("2-D taps", lambda: cp4.cp3_conv2d_forward(dev(x3), dev(K0), dev(K1), dev(K2), pad=1),
        lambda: oracle.cp3_forward(x3, K0, K1, K2, 1))
    return cases


def test_wait_timeout_is_reported_in_every_build(cp4, oracle):
    """The wait code is compiled into ten builds of the producer / consumer kernel:
    with the bound at one poll each of them must report the fault (every wave still
    ends normally), and with the default bound give the right answer again."""
    for name, launch, want, tol in _build_cases(cp4, oracle):
        assert cp4.device_status_detail()[0] == cp4.capi.OK, name
        cp4.set_spin_limit(1)
        try:
            launch()
            st, detail = cp4.device_status_detail()
        finally:
            cp4.set_spin_limit(0)
        assert st == cp4.capi.ERR_DEVICE, f"{name}: a wait that ran out was not reported"
        assert detail[0] != 0, name
        got = launch().cpu().numpy()
        cp4.device_status()
        ref = want()
        err = np.abs(got - ref).max() / np.abs(ref).max()
        assert err <= tol, f"{name}: {err:.2e} after the fault"


def test_layer_reports_a_wait_timeout(cp4):
    """The autograd layer launches asynchronously: check_device() where the loop
    synchronises - or set_device_checks(True) - turns an incomplete output into an error."""
    from paralleltnnlayers_amd import torch_ops
    layer = torch_ops.CP4Conv2d(64, 64, 3, 16)
    x = torch.randn(4, 64, 32, 32, device="cuda", requires_grad=True)
    layer(x).sum().backward()
    layer.check_device()                        # clean
    cp4.set_spin_limit(1)
    try:
        y = layer(x)
        with pytest.raises(cp4.Cp4Error) as ei:
            layer.check_device()
        assert ei.value.status == cp4.capi.ERR_DEVICE
        torch_ops.set_device_checks(True)
        y = layer(x)
        with pytest.raises(cp4.Cp4Error) as ei:
            y.sum().backward()                  # the backward pass ends with the check
        assert ei.value.status == cp4.capi.ERR_DEVICE
    finally:
        torch_ops.set_device_checks(False)
        cp4.set_spin_limit(0)
    layer.check_device()
    layer(x).sum().backward()
    layer.check_device()
