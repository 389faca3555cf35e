"""Calibration statistics and observers on the GPU: dq8_minmax against numpy (min and max are
exact operations, so the comparison is bit for bit), the observer classes against the oracle's
restatement of the reference's qparams arithmetic, fake quantization against the oracle's
quantize -> dequantize."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
import oracle as O  # noqa: E402
from oracle import observer_oracle as OB  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from bladedisc_amd import kernels
    return kernels


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def fresh(n):
    return (torch.full((n,), float("inf"), device="cuda"),
            torch.full((n,), float("-inf"), device="cuda"))


@pytest.mark.parametrize("n", [1, 3, 7, 255, 4095, 4096, 4097, 12289, (1 << 20) + 3])
def test_minmax_per_tensor_sizes(K, n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    lo, hi = fresh(1)
    K.minmax(dev(x), lo, hi)
    assert lo.item() == x.min() and hi.item() == x.max()


def test_minmax_unaligned_pointer_and_running_state(K):
    rng = np.random.default_rng(3)
    a = rng.standard_normal(5001).astype(np.float32)
    b = (rng.standard_normal(9000) * 2).astype(np.float32)
    lo, hi = fresh(1)
    K.minmax(dev(a)[1:], lo, hi)                 # 4-byte aligned only
    assert lo.item() == a[1:].min() and hi.item() == a[1:].max()
    K.minmax(dev(b), lo, hi)                     # folds into the state
    want_lo, want_hi = OB.running_min_max([a[1:], b])
    assert lo.item() == want_lo and hi.item() == want_hi
    K.minmax(torch.empty(0, device="cuda"), lo, hi)   # nothing observed: state kept
    assert lo.item() == want_lo and hi.item() == want_hi


@pytest.mark.parametrize("shape,axis", [
    ((768, 768), 0), ((300, 770), 0), ((5, 9000), 0), ((64, 3, 3, 32), 0),     # rows layout
    ((1000, 768), 1), ((777, 10), 1), ((4099, 4), 1), ((3, 5), 1), ((70000, 8), 1),  # last axis
    ((2, 5, 64), 1), ((3, 8, 7), 1), ((4, 6, 1, 1), 1),                         # middle axis
])
def test_minmax_per_channel(K, shape, axis):
    rng = np.random.default_rng(sum(shape) + axis)
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    y = (rng.standard_normal(shape) * 3 + 1).astype(np.float32)
    nch = shape[axis]
    lo, hi = fresh(nch)
    K.minmax(dev(x), lo, hi, axis=axis)
    K.minmax(dev(y), lo, hi, axis=axis)
    want_lo, want_hi = OB.running_min_max([x, y], ch_axis=axis)
    np.testing.assert_array_equal(lo.cpu().numpy(), want_lo)
    np.testing.assert_array_equal(hi.cpu().numpy(), want_hi)


def test_minmax_nan_marks_its_channel_only(K):
    x = np.arange(4 * 1000, dtype=np.float32).reshape(4, 1000)
    x[2, 517] = np.nan
    lo, hi = fresh(4)
    K.minmax(dev(x), lo, hi, axis=0)
    lo, hi = lo.cpu().numpy(), hi.cpu().numpy()
    assert np.isnan(lo[2]) and np.isnan(hi[2])
    np.testing.assert_array_equal(lo[[0, 1, 3]], [0, 1000, 3000])
    np.testing.assert_array_equal(hi[[0, 1, 3]], [999, 1999, 3999])
    xt = np.ascontiguousarray(x.T)                # the same with the channel as last axis
    lo, hi = fresh(4)
    K.minmax(dev(xt), lo, hi, axis=1)
    assert np.isnan(lo[2].item()) and np.isnan(hi[2].item()) and lo[3].item() == 3000
    lo, hi = fresh(1)                             # per tensor: one NaN poisons the result,
    K.minmax(dev(x), lo, hi)                      # as torch.aminmax does
    assert np.isnan(lo.item()) and np.isnan(hi.item())


def test_minmax_argument_checks(K):
    x = torch.zeros((4, 8), device="cuda")
    lo, hi = fresh(3)
    with pytest.raises(ValueError):
        K.minmax(x, lo, hi, axis=0)
    with pytest.raises(TypeError):
        K.minmax(x.double(), *fresh(1))
    from bladedisc_amd import _lib
    import ctypes as C
    L = _lib.lib()
    lo, hi = fresh(1)
    st = L.dq8_minmax(C.c_void_p(x.data_ptr()), 1, 1, 32, C.c_void_p(lo.data_ptr()),
                      C.c_void_p(hi.data_ptr()), None, 0, None)
    assert st != 0 and b"workspace" in L.dq8_last_error()


def test_minmax_full_size_against_the_library_reduction(K):
    """[65536, 4096] f32, 1 GiB: per tensor and per last-axis channel, equal to torch's own
    reductions (exact operations: any correct implementation gives the same bits)."""
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn((65536, 4096), device="cuda", generator=g)
    lo, hi = fresh(1)
    K.minmax(x, lo, hi)
    assert lo.item() == x.min().item() and hi.item() == x.max().item()
    lo, hi = fresh(4096)
    K.minmax(x, lo, hi, axis=1)
    assert torch.equal(lo, x.amin(dim=0)) and torch.equal(hi, x.amax(dim=0))
    lo, hi = fresh(65536)
    K.minmax(x, lo, hi, axis=0)
    assert torch.equal(lo, x.amin(dim=1)) and torch.equal(hi, x.amax(dim=1))


# ------------------------------------------------------------------ observers
def test_min_max_observer_qparams_and_fake_quant(K):
    from bladedisc_amd import observer as ob
    rng = np.random.default_rng(11)
    a = rng.standard_normal((64, 768)).astype(np.float32)
    b = (rng.standard_normal((32, 768)) * 1.5).astype(np.float32)
    o = ob.MinMaxObserver()                                       # qint8, per tensor, symmetric
    o.set_mode(observe=True, fake_quant=False)
    assert o(dev(a)).data_ptr() and o(dev(b)) is not None
    lo, hi = OB.running_min_max([a, b])
    s, z = OB.calculate_qparams(lo, hi, -128, 127, symmetric=True)
    assert o.scale.item() == s and o.zero_point.item() == z
    o.set_mode(observe=False, fake_quant=True)
    got = o(dev(a)).cpu().numpy()
    zp = np.array([z], np.int32).reshape(1)
    want = O.dequantize(O.quantize(a, np.float32(s), zp), np.float32(s), zp)
    np.testing.assert_array_equal(got, want)

    o = ob.MinMaxObserver(dtype=torch.quint8, qscheme=torch.per_tensor_affine)
    o.set_mode(observe=True, fake_quant=True)
    got = o(dev(a)).cpu().numpy()
    s, z = OB.calculate_qparams(a.min(), a.max(), 0, 255, symmetric=False)
    assert o.scale.item() == s and o.zero_point.item() == z
    zp = np.array([z], np.int32).reshape(1)
    want = O.dequantize(O.quantize(a, np.float32(s), zp, qmin=0, qmax=255, dtype=np.uint8),
                        np.float32(s), zp)
    np.testing.assert_array_equal(got, want)

    with pytest.raises(ValueError):                               # observer.py:105-106
        ob.MinMaxObserver(dtype=torch.quint8, qscheme=torch.per_tensor_symmetric)
    fresh_ob = ob.MinMaxObserver()                                # nothing observed yet
    s0, z0 = fresh_ob._calculate_qparams(fresh_ob.min_val, fresh_ob.max_val)
    assert s0.item() == 1.0 and z0.item() == 0


def test_per_channel_and_bias_observers(K):
    from bladedisc_amd import observer as ob
    rng = np.random.default_rng(12)
    w = (rng.standard_normal((96, 768)) * 0.02).astype(np.float32)
    w[5] = 0                                                       # an all-zero channel: eps floor
    x = rng.standard_normal((16, 768)).astype(np.float32)
    bias = (rng.standard_normal(96) * 0.01).astype(np.float32)
    w_ob = ob.PerChannelMinMaxObserver(ch_axis=0)
    got_w = w_ob(dev(w)).cpu().numpy()
    lo, hi = OB.running_min_max([w], ch_axis=0)
    s, z = OB.calculate_qparams(lo, hi, -128, 127, symmetric=True)
    np.testing.assert_array_equal(w_ob.scale.cpu().numpy(), s)
    np.testing.assert_array_equal(w_ob.zero_point.cpu().numpy(), z)
    assert s[5] == np.finfo(np.float32).eps
    want = O.dequantize(O.quantize(w, s, z, axis=0), s, z, axis=0)
    np.testing.assert_array_equal(got_w, want)
    assert w_ob(torch.empty((0, 768), device="cuda")).numel() == 0      # observer.py:263-264

    a_ob = ob.MinMaxObserver()
    a_ob(dev(x))
    b_ob = ob.BiasObserver(w_ob, a_ob)
    got_b = b_ob(dev(bias)).cpu().numpy()
    bs = OB.bias_scale(s, a_ob.scale.item())
    np.testing.assert_array_equal(b_ob.scale.cpu().numpy(), bs)
    want_b = (np.clip(np.rint(bias / bs), -2.0 ** 31, 2.0 ** 31 - 1) * bs).astype(np.float32)
    np.testing.assert_array_equal(got_b, want_b)
