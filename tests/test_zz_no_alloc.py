"""The backward-filter entry point that allocates nothing
(cp4_conv2d_backward_filter_noalloc: static device scratch inside the library)
against the entry point with a caller's workspace, through the C ABI.

Two calls in a row, the second on a smaller input: the shared scratch keeps the
first call's contents, and the second result must not depend on them.  Both
entry points run the same kernels in the same order, so the bar is bit equality.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from paralleltnnlayers_amd.configs import WORKLOADS, Workload, make_inputs  # noqa: E402

FACTORS = ("FK", "FC", "FH", "FW")


@pytest.fixture(scope="module")
def cp4():
    import paralleltnnlayers_amd as p
    p.lib()
    assert torch.cuda.is_available()
    return p


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def run_both(cp4, w, seed):
    a = make_inputs(w, seed=seed)
    f = [dev(a[k]) for k in FACTORS]
    x, dy = dev(a["x"]), dev(a["dy"])
    outs = [torch.full_like(t, float("nan")) for t in f]      # allocated by the caller, before the call
    torch.cuda.synchronize()
    got = cp4.conv2d_backward_filter_noalloc(x, dy, *f, outs, pad=w.pad)
    want = cp4.conv2d_backward_filter(x, dy, *f, pad=w.pad)
    torch.cuda.synchronize()
    return got, want, a


def test_noalloc_backward_filter_matches_workspace_entry_twice(cp4, oracle):
    big = WORKLOADS["C5"]                                       # 23.6 MB of scratch: matrix-core path
    small = Workload("small", "backward_filter", 3, 20, 9, 11, 1, 12, 3, 3, 5, "uniform")  # general path
    mid = Workload("mid", "backward_filter", 8, 64, 14, 14, 1, 32, 3, 3, 16, "uniform")    # matrix cores, smaller
    s = cp4.capi.shape_for((big.N, big.C, big.H, big.W), *[torch.empty(d, big.R) for d in
                                                            (big.T, big.C, big.Y, big.X)], big.pad)
    assert cp4.backward_filter_workspace_bytes(s) <= cp4.lib().cp4_noalloc_scratch_bytes()
    for w, seed in ((big, 0), (mid, 1), (small, 2), (big, 3)):
        got, want, a = run_both(cp4, w, seed)
        for g, r, k in zip(got, want, FACTORS):
            assert torch.equal(g, r), f"{w.name} d{k}: differs from the workspace entry point"
        if w is not big:
            ref = oracle.backward_filter(a["x"], a["dy"], a["FK"], a["FC"], a["FH"], a["FW"], w.pad)
            for g, r, k in zip(got, ref, FACTORS):
                err = np.abs(g.cpu().numpy() - r).max() / np.abs(r).max()
                assert err <= 1e-3, f"{w.name} d{k}: {err:.2e} against the oracle"


def test_noalloc_leaves_device_memory_untouched(cp4, oracle):
    """The property that names the entry point: after a first call (which loads the
    code object and looks the scratch array up) a call allocates and frees nothing -
    neither through the runtime (free device memory unchanged) nor through torch's
    caching allocator.  Checked on a shape of each route: general kernels, matrix
    cores, and more than 64 ranks (rank tiles on compact factor copies in the scratch)."""
    shapes = [Workload("general", "backward_filter", 3, 20, 9, 11, 1, 12, 3, 3, 5, "uniform"),
              Workload("matrix", "backward_filter", 8, 64, 14, 14, 1, 32, 3, 3, 16, "uniform"),
              Workload("tiles", "backward_filter", 4, 32, 12, 12, 1, 48, 3, 3, 80, "uniform")]
    for w in shapes:
        a = make_inputs(w, seed=4)
        f = [dev(a[k]) for k in FACTORS]
        x, dy = dev(a["x"]), dev(a["dy"])
        outs = [torch.empty_like(t) for t in f]
        cp4.conv2d_backward_filter_noalloc(x, dy, *f, outs, pad=w.pad)      # warm-up
        torch.cuda.synchronize()
        free0, torch0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
        reserved0 = torch.cuda.memory_reserved()
        cp4.conv2d_backward_filter_noalloc(x, dy, *f, outs, pad=w.pad)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0, f"{w.name}: device memory changed"
        assert torch.cuda.memory_allocated() == torch0 and torch.cuda.memory_reserved() == reserved0
        ref = oracle.backward_filter(a["x"], a["dy"], a["FK"], a["FC"], a["FH"], a["FW"], w.pad)
        for g, r, k in zip(outs, ref, FACTORS):
            err = np.abs(g.cpu().numpy() - r).max() / np.abs(r).max()
            assert err <= 1e-3, f"{w.name} d{k}: {err:.2e} against the oracle"


def test_noalloc_rejects_shapes_beyond_its_scratch(cp4):
    L = cp4.lib()
    s = cp4.capi.Shape(N=32, H=56, W=56, pad=1, T=256, C=256, Y=3, X=3, Rank=32)
    assert cp4.backward_filter_workspace_bytes(s) > L.cp4_noalloc_scratch_bytes()
    one = ctypes.c_void_p(256)      # never dereferenced: the size check comes first
    rc = L.cp4_conv2d_backward_filter_noalloc(ctypes.byref(s), *([one] * 10), None)
    assert rc == cp4.capi.ERR_WORKSPACE
    assert b"static scratch" in L.cp4_last_error_message()
