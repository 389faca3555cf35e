"""Synthetic inputs of the five benchmark configurations of the quantized hot path.

Everything is generated on the host with ``numpy.random.Generator(PCG64(1234 + config))``
so that the GPU path and the CPU checker see identical bytes.  Scales follow the
benchmark's definition (symmetric, ``max|x| / 127``); the reference's own observers use
``/ 127.5`` (tools/torch_quant/torch_quant/observer.py:134-163), which only changes the
numbers, not the arithmetic under test.
"""
import numpy as np

BERT_LINEARS = ((768, 768), (768, 3072), (3072, 768))          # (K, N)
SWEEP_M = (1, 16, 128, 1000, 4096, 16384)
RESNET_CONVS = (                                                # NHWC x OHWI
    dict(name="56x56x64_3x3x64", nb=32, h=56, w=56, ci=64, co=64, k=3, stride=1, pad=1),
    dict(name="28x28x128_3x3x128", nb=32, h=28, w=28, ci=128, co=128, k=3, stride=1, pad=1),
    dict(name="14x14x256_1x1x1024", nb=32, h=14, w=14, ci=256, co=1024, k=1, stride=1, pad=0),
)
# Every distinct convolution of ResNet-50 (h = w: input size; batch 32 in the sweep): the layers
# around the three above, timed on the GPU only.  (h, ci, co, k, stride, pad)
RESNET50_LAYERS = (
    (224, 3, 64, 7, 2, 3),
    (56, 64, 64, 1, 1, 0), (56, 64, 64, 3, 1, 1), (56, 64, 256, 1, 1, 0), (56, 256, 64, 1, 1, 0),
    (56, 256, 128, 1, 1, 0), (56, 128, 128, 3, 2, 1), (56, 256, 512, 1, 2, 0),
    (28, 128, 512, 1, 1, 0), (28, 512, 128, 1, 1, 0), (28, 128, 128, 3, 1, 1),
    (28, 512, 256, 1, 1, 0), (28, 256, 256, 3, 2, 1), (28, 512, 1024, 1, 2, 0),
    (14, 256, 1024, 1, 1, 0), (14, 1024, 256, 1, 1, 0), (14, 256, 256, 3, 1, 1),
    (14, 1024, 512, 1, 1, 0), (14, 512, 512, 3, 2, 1), (14, 1024, 2048, 1, 2, 0),
    (7, 512, 2048, 1, 1, 0), (7, 2048, 512, 1, 1, 0), (7, 512, 512, 3, 1, 1),
)
BERT_SEQ_LENS = (32, 128, 384)


def _rng(config):
    return np.random.Generator(np.random.PCG64(1234 + config))


def sym_scale(x, axis=None):
    """Symmetric int8 scale max|x|/127 (per tensor, or per slice along `axis`)."""
    if axis is None:
        s = np.float32(np.abs(x).max() / 127.0)
        return s if s > 0 else np.float32(1.0)
    red = tuple(i for i in range(x.ndim) if i != axis)
    s = (np.abs(x).max(axis=red) / 127.0).astype(np.float32)
    s[s == 0] = 1.0
    return s


def quantize_host(x, scale, axis=None):
    """Input synthesis only (numpy): round-half-even of x/scale, clamped to int8."""
    if axis is not None:
        shape = [1] * x.ndim
        shape[axis] = -1
        scale = np.asarray(scale, np.float32).reshape(shape)
    q = np.rint(x.astype(np.float32) / np.asarray(scale, np.float32))
    return np.clip(q, -128, 127).astype(np.int8)


def output_scale(a_q, w_q, sx, sw, bias=None, rows=256):
    """Per-tensor output scale max|y|/127 of y = (sx*a_q) @ (sw*w_q)^T + bias, estimated
    on the first `rows` rows."""
    a = a_q[:rows].astype(np.float32) * np.float32(sx)
    w = w_q.astype(np.float32) * np.asarray(sw, np.float32).reshape(-1, 1)
    y = a @ w.T
    if bias is not None:
        y = y + bias
    return sym_scale(y)


def config1():
    """One quantized linear, 64 x 768 -> 768, f32 in / f32 out."""
    r = _rng(1)
    x = r.standard_normal((64, 768)).astype(np.float32)
    w = (r.standard_normal((768, 768)) * 0.02).astype(np.float32)
    bias = (r.standard_normal(768) * 0.01).astype(np.float32)
    sx = sym_scale(x)
    sw = sym_scale(w, axis=0)
    w_q = quantize_host(w, sw, axis=0)
    y = x @ w.T + bias
    so = sym_scale(y)
    return dict(x=x, w=w, w_q=w_q, bias=bias, sx=sx, sw=sw, so=so, y_fp32=y)


def config2(m, k, n):
    """One shape of the dynamic-M sweep: int8 activations [m,k], weights [n,k]."""
    r = np.random.Generator(np.random.PCG64([1236, m, k, n]))
    x = r.standard_normal((m, k)).astype(np.float32)
    w = (r.standard_normal((n, k)) * 0.02).astype(np.float32)
    sx = sym_scale(x)
    sw = sym_scale(w, axis=0)
    a_q = quantize_host(x, sx)
    w_q = quantize_host(w, sw, axis=0)
    so = output_scale(a_q, w_q, sx, sw)
    return dict(a_q=a_q, w_q=w_q, sx=sx, sw=sw, so=so)


def config3(size):
    """Large square GEMM: uniform int8 operands, per-channel scales uniform in
    [0.001, 0.05], f32 bias in output units.  The output scale is chosen so that the
    result is not degenerate (std of about 40 LSB at the mean channel)."""
    r = _rng(2)   # same stream as the benchmark's headline problem
    m = n = k = size
    a = r.integers(-127, 128, (m, k), dtype=np.int8)
    w = r.integers(-127, 128, (n, k), dtype=np.int8)
    sw = r.uniform(0.001, 0.05, n).astype(np.float32)
    sx = np.float32(0.02)
    std_acc = np.sqrt(k) * (127.0 * 128.0 / 3.0)
    so = np.float32(float(sx) * float(sw.mean()) * std_acc / 40.0)
    bias_q = (r.standard_normal(n) * 10.0).astype(np.float32)
    return dict(a_q=a, w_q=w, sx=sx, sw=sw, so=so, bias_q=bias_q)


def config4(conv):
    """One ResNet-50-like int8 NHWC convolution."""
    r = np.random.Generator(np.random.PCG64([1238, conv["h"], conv["ci"], conv["co"]]))
    x = np.maximum(r.standard_normal((conv["nb"], conv["h"], conv["w"], conv["ci"])), 0).astype(np.float32)
    w = (r.standard_normal((conv["co"], conv["k"], conv["k"], conv["ci"])) * 0.05).astype(np.float32)
    sx = sym_scale(x)
    sw = sym_scale(w, axis=0)
    x_q = quantize_host(x, sx)
    w_q = quantize_host(w, sw, axis=0)
    # output scale from the centre of the first image (full receptive fields only)
    k, ci = conv["k"], conv["ci"]
    patch = x_q[0, 8:8 + k, 8:8 + k, :].astype(np.float32).reshape(-1)
    y = (w_q.reshape(conv["co"], -1).astype(np.float32) @ patch) * sw * sx
    so = np.float32(max(np.abs(y).max() * 1.5 / 127.0, 1e-6))
    return dict(x_q=x_q, w_q=w_q, sx=sx, sw=sw, so=so)


def config5_weights(hidden=768, ffn=3072, vocab=30522, max_seq=512):
    """Random-init BERT-base encoder layer (weights ~ N(0, 0.02)) with its embedding
    tables."""
    r = _rng(5)
    g = lambda *s: (r.standard_normal(s) * 0.02).astype(np.float32)  # noqa: E731
    return dict(
        tok_emb=g(vocab, hidden), pos_emb=g(max_seq, hidden),
        emb_ln_g=np.ones(hidden, np.float32), emb_ln_b=np.zeros(hidden, np.float32),
        wq=g(hidden, hidden), wk=g(hidden, hidden), wv=g(hidden, hidden),
        bq=g(hidden), bk=g(hidden), bv=g(hidden),
        wo=g(hidden, hidden), bo=g(hidden),
        ln1_g=np.ones(hidden, np.float32), ln1_b=np.zeros(hidden, np.float32),
        w1=g(ffn, hidden), b1=g(ffn), w2=g(hidden, ffn), b2=g(hidden),
        ln2_g=np.ones(hidden, np.float32), ln2_b=np.zeros(hidden, np.float32))


def config5_tokens(batch, seq, vocab=30522):
    r = np.random.Generator(np.random.PCG64([1239, batch, seq]))
    return r.integers(0, vocab, (batch, seq), dtype=np.int64)
