"""Quantized BERT-base encoder layer on the quantized RAL entries.

The counterpart of what the reference's post-training-quantization example produces
for one encoder layer (examples/PyTorch/Quantization/bert_ptq.py, pytorch_blade/tests/
quantization): the four linears (merged QKV, attention output, FFN1, FFN2) run as
int8 GEMMs with per-tensor activation scales, per-output-channel weight scales and a
fused bias + requantisation; ``quantize`` / ``dequantize`` sit between them and the
fp32 LayerNorm / softmax / GELU, which PyTorch computes.  Scales come from a min/max
calibration pass, as the reference's observers produce them.

Two backends execute the quantized operators:
  RalBackend  through ``tao_ral_call_impl`` by mangled name (what a compiled program does),
  RawBackend  through the raw kernel C ABI (``dq8_*``), the cheaper path for timing.
Both run the same HIP kernels.
"""
import math

import numpy as np
import torch

from . import baseline_configs as cfg
from . import kernels as K
from . import ral_ops

LINEARS = ("qkv", "out", "ffn1", "ffn2")


class RawBackend:
    name = "raw"

    def __init__(self, device="cuda"):
        self.z1 = torch.zeros(1, dtype=torch.int32, device=device)

    def quantize(self, x, scale):
        return K.quantize(x, scale, self.z1)

    def dequantize(self, q, scale):
        return K.dequantize(q, scale, self.z1)

    def qlinear(self, x_q, w_q, bias, sx, sw, so):
        """E1: sat8(rne((acc + b32) * (sx*sw/so))) with the f32 bias folded to int32."""
        return K.qgemm(x_q, w_q, K.EPI_REQUANT_CPU, sx=sx, sw=sw, so=so, bias=bias)

    def qlinear_dequantized(self, x_q, w_q, bias, sx, sw, so):
        """qlinear followed by dequantize(., so), in the GEMM's epilogue: f32 out."""
        return K.qgemm(x_q, w_q, K.EPI_REQUANT_CPU_DEQUANT_F32, sx=sx, sw=sw, so=so, bias=bias)

    def qlinear_table(self, x_q, w_q, bias, sx, sw, so, table):
        """qlinear followed by a 256-entry table lookup on its int8 result, in the epilogue."""
        post = K.make_postops(table=table)
        return K.qgemm(x_q, w_q, K.EPI_REQUANT_CPU, sx=sx, sw=sw, so=so, bias=bias, post=post)

    def qlinear_dequantized_residual(self, x_q, w_q, bias, sx, sw, so, residual):
        """qlinear, dequantize(., so) and the addition of an f32 tensor of the result's
        shape, in the epilogue: f32 out."""
        post = K.make_postops(residual=residual)
        return K.qgemm(x_q, w_q, K.EPI_REQUANT_CPU_DEQUANT_F32, sx=sx, sw=sw, so=so, bias=bias,
                       post=post)

    def lut8(self, q, table):
        return K.lut8(q, table)


class RalBackend:
    name = "ral"

    def __init__(self, execution, device="cuda"):
        self.ex = execution
        self.z1 = torch.zeros(1, dtype=torch.int32, device=device)

    def quantize(self, x, scale):
        return ral_ops.quantize(self.ex, x, scale, self.z1)

    def dequantize(self, q, scale):
        return ral_ops.dequantize(self.ex, q, scale, self.z1)

    def qlinear(self, x_q, w_q, bias, sx, sw, so):
        return ral_ops.pdll_qgemm_cpu_style(self.ex, x_q, w_q, bias, sx, sw, so,
                                            transpose_b=True, weight_is_const=True)

    def qlinear_dequantized(self, x_q, w_q, bias, sx, sw, so):
        return ral_ops.pdll_qgemm_fused(self.ex, x_q, w_q, bias, sx, sw, so, transpose_b=True,
                                        weight_is_const=True)

    def qlinear_table(self, x_q, w_q, bias, sx, sw, so, table):
        return ral_ops.pdll_qgemm_fused(self.ex, x_q, w_q, bias, sx, sw, so, transpose_b=True,
                                        weight_is_const=True, table=table)

    def qlinear_dequantized_residual(self, x_q, w_q, bias, sx, sw, so, residual):
        return ral_ops.pdll_qgemm_fused(self.ex, x_q, w_q, bias, sx, sw, so, transpose_b=True,
                                        weight_is_const=True, residual=residual)

    def lut8(self, q, table):
        # a compiled program would carry this as one of its own generated kernels; the
        # runtime has no entry for it
        return K.lut8(q, table)


def _layer_norm(x, g, b):
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), g, b, 1e-12)


class QuantBertLayer:
    """One encoder layer; hidden 768, 12 heads, FFN 3072 by default."""

    def __init__(self, weights, backend, heads=12, device="cuda", fuse_gelu=False,
                 fuse_dequant=False, fuse_epilogue=False):
        """fuse_dequant: a linear whose int8 result is only dequantized writes
        the dequantized f32 from the GEMM's epilogue (same bits, no int8 round trip).
        fuse_gelu: run dequantize -> GELU -> quantize between the two FFN linears as one
        256-entry table lookup on the int8 tensor (what the compiler's fusion of those three
        elementwise operators amounts to); the result is bit-identical to the three separate
        operators because the table is built by running exactly them on all 256 inputs.
        fuse_epilogue: the operators behind three of the linears run in the
        GEMM's epilogue -- the residual additions behind the attention output and FFN2
        (dequantize + add, f32 out) and the GELU table behind FFN1 -- again the same bits."""
        self.fuse_gelu = fuse_gelu or fuse_epilogue
        self.fuse_dequant = fuse_dequant or fuse_epilogue
        self.fuse_epilogue = fuse_epilogue
        self.gelu_table = None
        self.be = backend
        self.heads = heads
        self.device = device
        d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
        w = weights
        self.f = {k: d(v) for k, v in w.items()}          # fp32 master copies
        merged_w = np.concatenate([w["wq"], w["wk"], w["wv"]], axis=0)
        merged_b = np.concatenate([w["bq"], w["bk"], w["bv"]], axis=0)
        self.fw = {"qkv": merged_w, "out": w["wo"], "ffn1": w["w1"], "ffn2": w["w2"]}
        self.fb = {"qkv": merged_b, "out": w["bo"], "ffn1": w["b1"], "ffn2": w["b2"]}
        self.w_q, self.sw, self.bias = {}, {}, {}
        for name in LINEARS:
            # per-output-channel symmetric weight scales; the weights are quantized by
            # the same GPU kernel that serves mhlo_disc.quantize
            self.sw[name] = d(cfg.sym_scale(self.fw[name], axis=0))
            zeros = torch.zeros(self.sw[name].numel(), dtype=torch.int32, device=device)
            self.w_q[name] = K.quantize(d(self.fw[name]), self.sw[name], zeros, axis=0)
            self.bias[name] = d(self.fb[name])
        self.s_in, self.s_out = {}, {}

    # ---------------------------------------------------------------- fp32 parts
    def embed(self, tokens):
        t = torch.as_tensor(tokens, device=self.device)
        pos = torch.arange(t.shape[1], device=self.device)
        h = self.f["tok_emb"][t] + self.f["pos_emb"][pos][None]
        return _layer_norm(h, self.f["emb_ln_g"], self.f["emb_ln_b"])

    def attention(self, qkv):
        """softmax(q k^T / sqrt(d)) v in fp32, PyTorch's fused kernel.  qkv: [B, S, 3H] -> [B, S, H].
        (Written out as two batched products, a scale and a softmax the same arithmetic is nine
        launches, half of them copies into head-major layout: 73 -> 53 us for the whole layer at
        batch 8 x seq 32, 248 -> 178 us at seq 384.)"""
        b, s, h3 = qkv.shape
        h = h3 // 3
        dh = h // self.heads
        q, k, v = (t.reshape(b, s, self.heads, dh).transpose(1, 2) for t in qkv.split(h, dim=-1))
        o = torch.nn.functional.scaled_dot_product_attention(q, k, v)
        return o.transpose(1, 2).reshape(b, s, h)

    def _linear_fp32(self, name, x):
        return x @ torch.from_numpy(self.fw[name]).to(self.device).T + self.bias[name]

    def forward_fp32(self, h, record=None):
        """The unquantized layer; `record` collects the inputs / outputs of the linears."""
        rec = record if record is not None else {}
        rec["qkv_in"] = h
        rec["qkv_out"] = self._linear_fp32("qkv", h)
        rec["out_in"] = self.attention(rec["qkv_out"])
        rec["out_out"] = self._linear_fp32("out", rec["out_in"])
        rec["ffn1_in"] = _layer_norm(h + rec["out_out"], self.f["ln1_g"], self.f["ln1_b"])
        rec["ffn1_out"] = self._linear_fp32("ffn1", rec["ffn1_in"])
        rec["ffn2_in"] = torch.nn.functional.gelu(rec["ffn1_out"])
        rec["ffn2_out"] = self._linear_fp32("ffn2", rec["ffn2_in"])
        return _layer_norm(rec["ffn1_in"] + rec["ffn2_out"], self.f["ln2_g"], self.f["ln2_b"])

    def calibrate(self, h):
        """Min/max calibration: symmetric per-tensor scale max|x|/127 for the input and
        the output of each linear, from one fp32 pass."""
        rec = {}
        self.forward_fp32(h, rec)
        for name in LINEARS:
            for which, store in (("in", self.s_in), ("out", self.s_out)):
                amax = rec["%s_%s" % (name, which)].abs().max().clamp_min(1e-12)
                store[name] = (amax / 127.0).reshape(1).float()
        self.gelu_table = K.activation_table(torch.nn.functional.gelu, self.s_out["ffn1"],
                                             self.be.z1, self.s_in["ffn2"], self.be.z1)
        return rec

    # ----------------------------------------------------------- quantized layer
    def _gemm(self, name, x_q):
        return self.be.qlinear(x_q, self.w_q[name], self.bias[name], self.s_in[name],
                               self.sw[name], self.s_out[name])

    def _gemm_dequantized(self, name, x_q):
        """(y_q or None, y): the linear's int8 result and its dequantized form."""
        if self.fuse_dequant:
            return None, self.be.qlinear_dequantized(x_q, self.w_q[name], self.bias[name],
                                                     self.s_in[name], self.sw[name],
                                                     self.s_out[name])
        y_q = self._gemm(name, x_q)
        return y_q, self.be.dequantize(y_q, self.s_out[name])

    def _qlinear(self, name, x, rec):
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        x_q = self.be.quantize(x2, self.s_in[name])
        y_q, y = self._gemm_dequantized(name, x_q)
        if rec is not None:
            rec[name] = dict(x=x2, x_q=x_q, y_q=y_q, y=y)
        return y.reshape(*shape[:-1], y.shape[-1])

    def _qlinear_residual(self, name, x, residual, rec):
        """residual + dequantize(linear(quantize(x))) with everything behind the GEMM fused."""
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        x_q = self.be.quantize(x2, self.s_in[name])
        r2 = residual.reshape(-1, residual.shape[-1])
        y = self.be.qlinear_dequantized_residual(x_q, self.w_q[name], self.bias[name],
                                                 self.s_in[name], self.sw[name],
                                                 self.s_out[name], r2)
        if rec is not None:
            rec[name] = dict(x=x2, x_q=x_q, y_plus_residual=y)
        return y.reshape(*shape[:-1], y.shape[-1])

    def _ffn_fused(self, h1, rec):
        """quantize -> ffn1 -> [table: dequantize, GELU, quantize] -> ffn2 -> dequantize."""
        shape = h1.shape
        x2 = h1.reshape(-1, shape[-1])
        x_q = self.be.quantize(x2, self.s_in["ffn1"])
        if self.fuse_epilogue:
            y1_q = None
            x2_q = self.be.qlinear_table(x_q, self.w_q["ffn1"], self.bias["ffn1"],
                                         self.s_in["ffn1"], self.sw["ffn1"],
                                         self.s_out["ffn1"], self.gelu_table)
            r2 = x2
            y2 = self.be.qlinear_dequantized_residual(
                x2_q, self.w_q["ffn2"], self.bias["ffn2"], self.s_in["ffn2"], self.sw["ffn2"],
                self.s_out["ffn2"], r2)
            if rec is not None:
                rec["ffn1"] = dict(x=x2, x_q=x_q)
                rec["ffn2"] = dict(x_q=x2_q, y_plus_residual=y2)
            return y2.reshape(*shape[:-1], y2.shape[-1])
        y1_q = self._gemm("ffn1", x_q)
        x2_q = self.be.lut8(y1_q, self.gelu_table)
        y2_q, y2 = self._gemm_dequantized("ffn2", x2_q)
        if rec is not None:
            rec["ffn1"] = dict(x=x2, x_q=x_q, y_q=y1_q)
            rec["ffn2"] = dict(x_q=x2_q, y_q=y2_q, y=y2)
        return y2.reshape(*shape[:-1], y2.shape[-1])

    def capture(self, h, stream=None):
        """Records one forward pass on `h`'s shape into a HIP graph and returns
        (replay, static_input, static_output): copy new activations into static_input,
        call replay(), read static_output.  A BERT layer at small batch x seq is a few
        dozen short kernels, and launching them one by one from the host takes longer
        than running them; a graph replays them back to back.  With the RAL backend the
        context must be bound to `stream` (pass the stream it was created on): its entries
        allocate their results from the context's pool, which the warm-up passes fill, so
        nothing is allocated from the device while capturing; the execution must stay open
        for as long as the graph is replayed (it owns the buffers the graph writes)."""
        static_in = h.clone()
        if isinstance(self.be, RalBackend) and stream is None:
            raise RuntimeError("capture with the RAL backend needs the stream its context is bound to")
        side = stream if stream is not None else torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):        # warm-up on the capture stream
            if isinstance(self.be, RalBackend):
                # in an execution of its own: when it ends, its buffers go back to the
                # context's pool, where the captured pass finds them
                keep = self.be.ex
                self.be.ex = keep.ctx.execution()
                try:
                    for _ in range(2):
                        self.forward(static_in)
                    side.synchronize()
                finally:
                    self.be.ex.close()
                    self.be.ex = keep
            else:
                for _ in range(2):
                    self.forward(static_in)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            static_out = self.forward(static_in)
        return graph.replay, static_in, static_out

    def forward(self, h, record=None):
        if not self.s_in:
            raise RuntimeError("calibrate() first")
        qkv = self._qlinear("qkv", h, record)
        ctx = self.attention(qkv)
        if self.fuse_epilogue:
            pre1 = self._qlinear_residual("out", ctx, h, record)
            h1 = _layer_norm(pre1, self.f["ln1_g"], self.f["ln1_b"])
            pre2 = self._ffn_fused(h1, record)       # h1 + ffn2(gelu(ffn1(h1)))
            return _layer_norm(pre2, self.f["ln2_g"], self.f["ln2_b"])
        attn = self._qlinear("out", ctx, record)
        h1 = _layer_norm(h + attn, self.f["ln1_g"], self.f["ln1_b"])
        if self.fuse_gelu:
            f2 = self._ffn_fused(h1, record)
        else:
            f1 = self._qlinear("ffn1", h1, record)
            g = torch.nn.functional.gelu(f1)
            f2 = self._qlinear("ffn2", g, record)
        return _layer_norm(h1 + f2, self.f["ln2_g"], self.f["ln2_b"])
