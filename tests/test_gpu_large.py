"""Operands and results beyond 2^31 bytes / elements: the kernels' 64-bit addressing.

The oracle checks seeded slices (the first rows, the rows either side of the 2^31-byte and
2^32-byte marks, the last rows); size-independent properties cover the rest (every row block of
a GEMM against a second call on that block alone; quantize -> dequantize within half a step).
"""
import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu


def slices_around(rows, row_bytes, marks=(1 << 31, 1 << 32), width=3):
    """Row ranges at the start, the end and either side of each byte mark."""
    out = [(0, width), (rows - width, rows)]
    for mk in marks:
        r = mk // row_bytes
        if width <= r < rows - width:
            out.append((r - width, r + width))
    return out


def test_qgemm_operand_larger_than_4_gib():
    """A is [1.1 M, 4096] int8 (4.5 GB); N = 64 takes the 256x64 tile, N = 256 a square one."""
    from bladedisc_amd import kernels as K
    m, k = 1_100_000, 4096
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda", generator=g)
    for n in (64, 256):
        w = torch.randint(-128, 128, (n, k), dtype=torch.int8, device="cuda", generator=g)
        sx = torch.full((1,), 0.02, device="cuda")
        sw = torch.rand(n, device="cuda", generator=g) * 0.05 + 0.001
        so = torch.full((1,), 20.0, device="cuda")
        bias = torch.randn(n, device="cuda", generator=g) * 50
        out = K.qgemm(a, w, K.EPI_REQUANT_CPU, sx=sx, sw=sw, so=so, bias=bias)
        acc = K.qgemm(a, w, K.EPI_ACC_S32)
        torch.cuda.synchronize()
        w_h = w.cpu().numpy()
        b32 = O.bias_f32_to_s32(bias.cpu().numpy(), np.float32(0.02), sw.cpu().numpy())
        for lo, hi in slices_around(m, k):
            a_h = a[lo:hi].cpu().numpy()
            want_acc = O.gemm_s32(a_h, w_h, tp_b=True)
            assert np.array_equal(acc[lo:hi].cpu().numpy(), want_acc), (n, lo)
            want = O.requant_cpu(want_acc, np.float32(0.02), sw.cpu().numpy(), np.float32(20.0), b32=b32)
            assert np.array_equal(out[lo:hi].cpu().numpy(), want), (n, lo)
        # every block of rows equals the same call on that block alone
        step = 131072
        for lo in range(0, m, step):
            hi = min(m, lo + step)
            part = K.qgemm(a[lo:hi], w, K.EPI_REQUANT_CPU, sx=sx, sw=sw, so=so, bias=bias)
            assert torch.equal(part, out[lo:hi]), (n, lo)
        sat = float(((out == 127) | (out == -128)).float().mean())
        assert sat < 0.5
        del out, acc


def test_qgemm_result_larger_than_4_gib():
    """[40000, 512] x [512, 30000] -> int32: 4.8 GB of results."""
    from bladedisc_amd import kernels as K
    m, n, k = 40000, 30000, 512
    g = torch.Generator(device="cuda").manual_seed(6)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda", generator=g)
    w = torch.randint(-128, 128, (n, k), dtype=torch.int8, device="cuda", generator=g)
    acc = K.qgemm(a, w, K.EPI_ACC_S32)
    torch.cuda.synchronize()
    w_h = w.cpu().numpy()
    for lo, hi in slices_around(m, n * 4):
        want = O.gemm_s32(a[lo:hi].cpu().numpy(), w_h, tp_b=True)
        assert np.array_equal(acc[lo:hi].cpu().numpy(), want), lo
    # column sums of the whole result against (sum of A's rows) . W, in int64
    a_sum = a.to(torch.float64).sum(0)                                  # exact: |.| < 2^53
    want_cols = (w.to(torch.float64) @ a_sum).to(torch.int64)
    got_cols = torch.zeros(n, dtype=torch.int64, device="cuda")
    for lo in range(0, m, 4096):
        got_cols += acc[lo:lo + 4096].sum(0, dtype=torch.int64)
    assert torch.equal(got_cols, want_cols)


@pytest.mark.parametrize("axis", [None, 1])
def test_quantize_dequantize_more_than_2_31_elements(axis):
    """[524289, 4100] f32: 2.15 G elements, 8.6 GB in, per tensor and per last-axis channel."""
    from bladedisc_amd import kernels as K
    rows, cols = 524289, 4100
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.empty((rows, cols), device="cuda")
    for lo in range(0, rows, 65536):                    # (randn's own temporaries stay small)
        x[lo:lo + 65536].normal_(0, 1, generator=g)
    nq = cols if axis is not None else 1
    scale = torch.rand(nq, device="cuda", generator=g) * 0.02 + 0.02
    zp = torch.randint(-5, 6, (nq,), dtype=torch.int32, device="cuda", generator=g)
    q = K.quantize(x, scale, zp, axis=axis)
    y = K.dequantize(q, scale, zp, axis=axis)
    torch.cuda.synchronize()
    s_h, z_h = scale.cpu().numpy(), zp.cpu().numpy()
    for lo, hi in slices_around(rows, cols * 4, marks=(1 << 31, 1 << 32, 1 << 33)):
        x_h = x[lo:hi].cpu().numpy()
        want_q = O.quantize(x_h, s_h, z_h, axis=axis)
        assert np.array_equal(q[lo:hi].cpu().numpy(), want_q), lo
        want_y = O.dequantize(want_q, s_h, z_h, axis=axis)
        assert np.array_equal(y[lo:hi].cpu().numpy().view(np.uint32), want_y.view(np.uint32)), lo
    # whole tensor: inside the representable range the round trip is within half a step
    for lo in range(0, rows, 65536):
        xs, ys = x[lo:lo + 65536], y[lo:lo + 65536]
        lim_lo = (-128 - zp).float() * scale
        lim_hi = (127 - zp).float() * scale
        err = (ys - torch.maximum(torch.minimum(xs, lim_hi), lim_lo)).abs()
        assert bool((err <= scale * 0.5001).all()), lo


def test_qconv_input_larger_than_2_gib():
    """NHWC input of 2.2 GB (33 x 256 x 256 x 1024), 1x1 filter with stride 2: beyond the 32-bit
    buffer offsets of the pipelined kernels, so the implicit GEMM must take the path with
    64-bit image bases.  The oracle convolves the first and the last image, and the image
    that straddles the 2^31-byte mark."""
    from bladedisc_amd import kernels as K
    nb, h, ci, co = 33, 256, 1024, 16
    g = torch.Generator(device="cuda").manual_seed(8)
    x = torch.randint(-128, 128, (nb, h, h, ci), dtype=torch.int8, device="cuda", generator=g)
    w = torch.randint(-128, 128, (co, 1, 1, ci), dtype=torch.int8, device="cuda", generator=g)
    md = list(O.NHWC_OHWI_METADATA) + [2, 2, 1, 1, 1]
    out_shape = [nb, h // 2, h // 2, co]
    sx = torch.full((1,), 0.02, device="cuda")
    sw = torch.rand(co, device="cuda", generator=g) * 0.05 + 0.001
    so = torch.full((1,), 8.0, device="cuda")
    acc = K.qconv2d(x, w, [0, 0, 0, 0], md, out_shape, K.EPI_ACC_S32)
    y = K.qconv2d(x, w, [0, 0, 0, 0], md, out_shape, K.EPI_REQUANT_CPU, sx=sx, sw=sw, so=so)
    torch.cuda.synchronize()
    w_h = w.cpu().numpy()
    straddling = (1 << 31) // (h * h * ci)
    for b in (0, straddling, nb - 1):
        want = O.conv_s32(x[b:b + 1].cpu().numpy(), w_h, [0, 0, 0, 0], md, [1] + out_shape[1:])
        assert np.array_equal(acc[b:b + 1].cpu().numpy(), want), b
        want_q = O.requant_cpu(want.reshape(-1, co), np.float32(0.02), sw.cpu().numpy(),
                               np.float32(8.0)).reshape(want.shape)
        assert np.array_equal(y[b:b + 1].cpu().numpy(), want_q), b
    # every image equals the convolution of that image alone
    for b in range(nb):
        one = K.qconv2d(x[b:b + 1], w, [0, 0, 0, 0], md, [1] + out_shape[1:], K.EPI_REQUANT_CPU,
                        sx=sx, sw=sw, so=so)
        assert torch.equal(one, y[b:b + 1]), b
    assert float(((y == 127) | (y == -128)).float().mean()) < 0.5
