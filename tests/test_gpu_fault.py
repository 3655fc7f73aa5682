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
