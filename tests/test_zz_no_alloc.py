"""dq8_minmax_static -- the entry point that allocates nothing -- against dq8_minmax, through
the C ABI: same running minimum / maximum bit for bit, on two calls in a row (the second
with a smaller tensor, so that stale pairs of the first call sit in the shared scratch), for
the three layouts, with NaNs, and with the size limit enforced."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu


def _state(n):
    return (torch.full((n,), float("inf"), device="cuda"),
            torch.full((n,), float("-inf"), device="cuda"))


def _both(L, x, outer, nch, inner):
    """(min, max) from dq8_minmax with a caller workspace and from dq8_minmax_static."""
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: C.c_void_p(t.data_ptr())  # noqa: E731
    need = L.dq8_minmax_workspace_bytes(outer, nch, inner)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    lo_a, hi_a = _state(nch)
    lo_b, hi_b = _state(nch)
    assert L.dq8_minmax(p(x), outer, nch, inner, p(lo_a), p(hi_a), p(ws), need, st) == 0, \
        L.dq8_last_error()
    assert L.dq8_minmax_static(p(x), outer, nch, inner, p(lo_b), p(hi_b), st) == 0, \
        L.dq8_last_error()
    torch.cuda.synchronize()
    return (lo_a.cpu().numpy(), hi_a.cpu().numpy()), (lo_b.cpu().numpy(), hi_b.cpu().numpy())


@pytest.mark.parametrize("layout", ["per_tensor", "last_axis", "axis0", "middle_axis"])
def test_static_scratch_matches_workspace_form_twice(layout):
    from bladedisc_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(77)
    # first call large, second smaller: the scratch still holds the first call's pairs
    shapes = {"per_tensor": [(1, 1, 3_000_017), (1, 1, 4099)],
              "last_axis": [(4099, 516, 1), (130, 36, 1)],
              "axis0": [(1, 2050, 8192), (1, 7, 100)],
              "middle_axis": [(6, 33, 5000), (2, 5, 16)]}[layout]
    for outer, nch, inner in shapes:
        x = rng.standard_normal(outer * nch * inner).astype(np.float32)
        x[rng.integers(0, x.size, 3)] *= 50.0
        if layout == "last_axis":
            x[5 * nch + 3] = np.nan                      # poisons channel 3 only
        dx = torch.from_numpy(x).cuda()
        (lo_a, hi_a), (lo_b, hi_b) = _both(L, dx, outer, nch, inner)
        np.testing.assert_array_equal(lo_a, lo_b)        # NaN == NaN position-wise here
        np.testing.assert_array_equal(hi_a, hi_b)
        v = x.reshape(outer, nch, inner)
        with np.errstate(invalid="ignore"):
            np.testing.assert_array_equal(lo_b, v.min(axis=(0, 2)))
            np.testing.assert_array_equal(hi_b, v.max(axis=(0, 2)))


def test_static_scratch_folds_into_running_state_and_rejects_oversize():
    from bladedisc_amd import _lib
    L = _lib.lib()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: C.c_void_p(t.data_ptr())  # noqa: E731
    lo = torch.tensor([-7.0], device="cuda")
    hi = torch.tensor([0.5], device="cuda")
    x = torch.linspace(-1.0, 3.0, 1001, device="cuda")
    assert L.dq8_minmax_static(p(x), 1, 1, 1001, p(lo), p(hi), st) == 0
    torch.cuda.synchronize()
    assert lo.item() == -7.0 and hi.item() == 3.0
    # an empty tensor leaves the state alone
    assert L.dq8_minmax_static(None, 0, 1, 5, p(lo), p(hi), st) == 0
    # more pairs than the built-in array holds: refused before anything is launched
    cap = L.dq8_minmax_static_max_bytes()
    assert cap == 4 << 20
    nch = 1 << 20                              # one pair per (channel) row of 16 elements
    assert L.dq8_minmax_workspace_bytes(1, nch, 16) == 8 * nch > cap
    assert L.dq8_minmax_static(p(x), 1, nch, 16, p(lo), p(hi), st) != 0
    assert b"more than the built-in" in L.dq8_last_error()
    torch.cuda.synchronize()
    assert lo.item() == -7.0 and hi.item() == 3.0


def test_static_scratch_under_graph_capture_and_without_allocation():
    """The callers this entry is for: code under HIP graph capture.  After one warm call (the
    per-device address lookup), the call is captured into a graph and replayed on fresh data
    several times, with eager work and synchronisations in between, each replay against
    dq8_minmax; and a call leaves the device's free memory as it found it."""
    from bladedisc_amd import _lib
    L = _lib.lib()
    p = lambda t: C.c_void_p(t.data_ptr())  # noqa: E731
    outer, nch, inner = 300, 64, 257
    rng = np.random.default_rng(5)
    x = torch.zeros(outer * nch * inner, device="cuda")
    lo, hi = _state(nch)
    warm = torch.from_numpy(rng.standard_normal(x.numel()).astype(np.float32)).cuda()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert L.dq8_minmax_static(p(warm), outer, nch, inner, p(lo), p(hi), st) == 0   # warm the lookup
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert L.dq8_minmax_static(p(warm), outer, nch, inner, p(lo), p(hi), st) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before

    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        g.capture_begin()
        rc = L.dq8_minmax_static(p(x), outer, nch, inner, p(lo), p(hi), C.c_void_p(side.cuda_stream))
        g.capture_end()
    assert rc == 0, L.dq8_last_error()
    torch.cuda.synchronize()
    need = L.dq8_minmax_workspace_bytes(outer, nch, inner)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    for rep in range(3):
        data = rng.standard_normal(x.numel()).astype(np.float32) * (rep + 1)
        x.copy_(torch.from_numpy(data))
        lo.fill_(float("inf"))
        hi.fill_(float("-inf"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        lo_ref, hi_ref = _state(nch)
        assert L.dq8_minmax(p(x), outer, nch, inner, p(lo_ref), p(hi_ref), p(ws), need, st) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(lo.cpu().numpy(), lo_ref.cpu().numpy())
        np.testing.assert_array_equal(hi.cpu().numpy(), hi_ref.cpu().numpy())
        v = data.reshape(outer, nch, inner)
        np.testing.assert_array_equal(lo.cpu().numpy(), v.min(axis=(0, 2)))
