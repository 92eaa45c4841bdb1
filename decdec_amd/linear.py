"""nn.Module front ends of the ops, with the interface of the reference's end-to-end modules.

``DECLinear`` / ``APLinear`` / ``LUTGEMMLinear`` follow the reference's end-to-end/DECLinear.py,
APLinear.py and LUTGEMMLinear.py (same constructor arguments, buffers, ``load_dec_data`` /
``create_dec_config`` / ``update_dec_config`` methods, decode path = zero the persistent output
buffer and call the fused op, prefill path = dequantise + matmul).  ``SQLLMLinear`` is the same
pattern for the ``dec_sqllm`` op, for which the reference ships no module.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import ext, formats


class DECLinear(nn.Module):
    """Holds the DEC side data of a quantised linear layer (reference DECLinear.py:6-53)."""

    def __init__(self):
        super().__init__()
        self.dec_config = None
        self.k_chunk = None
        self.q_residual = None
        self.scales = None
        self.thresholds = None
        self.external_zero = False      # True: the owner of `output` clears it before every decode step

    def load_dec_data(self, q_residual, scales, thresholds):
        assert q_residual.dtype == torch.int
        assert q_residual.shape == (self.in_features, self.out_features // 8)
        assert scales.dtype == self.dtype
        assert scales.shape == (self.out_features,)
        assert thresholds.dtype == self.dtype
        assert thresholds.shape == (self.in_features,)
        self.q_residual = q_residual
        self.scales = scales
        self.thresholds = thresholds

    def create_dec_config(self, dec_context, k_chunk):
        self.k_chunk = k_chunk
        assert self.q_residual is not None and self.scales is not None and self.thresholds is not None
        self.dec_config = ext.create_dec_config(dec_context, k_chunk, self.q_residual, self.scales, self.thresholds)

    def update_dec_config(self, dec_context, k_chunk):
        """New context / k_chunk without copying the residual again."""
        self.k_chunk = k_chunk
        assert self.dec_config is not None
        ext.update_dec_config(self.dec_config, dec_context, k_chunk)

    def _finish(self):
        if self.bias is not None:
            self.output += self.bias
        return self.output


class APLinear(DECLinear):
    """Any-precision bitplane layer (reference APLinear.py:7-58)."""

    def __init__(self, in_features, out_features, bitwidth, bias=False, dtype=torch.half, device="cuda"):
        super().__init__()
        self.in_features, self.out_features, self.bitwidth, self.dtype = in_features, out_features, bitwidth, dtype
        self.register_buffer("qweight", torch.empty((bitwidth, out_features, in_features // 32),
                                                    dtype=torch.int32, device=device))
        self.register_buffer("lut", torch.empty((out_features, 2 ** bitwidth), dtype=dtype, device=device))
        if bias:
            self.register_buffer("bias", torch.empty((out_features,), dtype=dtype, device=device))
        else:
            self.bias = None
        self.output = torch.zeros((1, 1, out_features), dtype=dtype, device=device)

    def gemm(self, x):
        weight = ext.anyprec_dequant(self.qweight, self.lut, self.bitwidth)
        return torch.matmul(x, weight.T)

    def forward(self, x, **kwargs):
        assert x.shape[0] == 1
        if x.shape[1] > 1:
            out = self.gemm(x)
            if self.bias is not None:
                out += self.bias
            return out
        if not self.external_zero:
            self.output.zero_()
        if self.dec_config is None:
            ext.anyprec_gemv(x, self.output, self.qweight, self.lut, self.bitwidth)
        else:
            ext.dec_anyprec(self.dec_config, x, self.output, self.qweight, self.lut, self.bitwidth)
        return self._finish()


class LUTGEMMLinear(DECLinear):
    """LUT-GEMM binary-coding layer (reference LUTGEMMLinear.py:6-102)."""

    def __init__(self, in_features, out_features, bitwidth, group_size, bias=False, dtype=torch.half, device="cuda"):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.bitwidth, self.group_size, self.dtype = bitwidth, group_size, dtype
        self.register_buffer("qweight", torch.empty((in_features // 32, bitwidth, out_features),
                                                    dtype=torch.int32, device=device))
        self.register_buffer("alpha", torch.empty((in_features // group_size, bitwidth, out_features),
                                                  dtype=dtype, device=device))
        self.register_buffer("q_bias", torch.empty((in_features // group_size, out_features),
                                                   dtype=dtype, device=device))
        if bias:
            self.register_buffer("bias", torch.empty((out_features,), dtype=dtype, device=device))
        else:
            self.bias = None
        self.output = torch.zeros((1, 1, out_features), dtype=dtype, device=device)

    def gemm(self, x):
        weight = formats.dequant_bcq(self.qweight, self.alpha, self.q_bias, self.group_size).to(x.dtype)
        return torch.matmul(x, weight.T)

    def forward(self, x, **kwargs):
        assert x.shape[0] == 1
        if x.shape[1] > 1:
            out = self.gemm(x)
            if self.bias is not None:
                out += self.bias
            return out
        if not self.external_zero:
            self.output.zero_()
        if self.dec_config is None:
            ext.lutgemm_gemv(x, self.output, self.qweight, self.alpha, self.q_bias, self.bitwidth, self.group_size)
        else:
            ext.dec_lutgemm(self.dec_config, x, self.output, self.qweight, self.alpha, self.q_bias,
                            self.bitwidth, self.group_size)
        return self._finish()


class SQLLMLinear(DECLinear):
    """SqueezeLLM per-channel LUT layer over the ``sqllm_gemv`` / ``dec_sqllm`` ops."""

    def __init__(self, in_features, out_features, bitwidth, bias=False, dtype=torch.half, device="cuda"):
        super().__init__()
        self.in_features, self.out_features, self.bitwidth, self.dtype = in_features, out_features, bitwidth, dtype
        self.register_buffer("qweight", torch.empty((in_features * bitwidth // 32, out_features),
                                                    dtype=torch.int32, device=device))
        self.register_buffer("lut", torch.empty((out_features, 2 ** bitwidth), dtype=dtype, device=device))
        if bias:
            self.register_buffer("bias", torch.empty((out_features,), dtype=dtype, device=device))
        else:
            self.bias = None
        self.output = torch.zeros((1, 1, out_features), dtype=dtype, device=device)

    def gemm(self, x):
        weight = formats.dequant_sqllm(self.qweight, self.lut, self.bitwidth)
        return torch.matmul(x, weight.T)

    def forward(self, x, **kwargs):
        assert x.shape[0] == 1
        if x.shape[1] > 1:
            out = self.gemm(x)
            if self.bias is not None:
                out += self.bias
            return out
        if not self.external_zero:
            self.output.zero_()
        if self.dec_config is None:
            ext.sqllm_gemv(x, self.output, self.qweight, self.lut, self.bitwidth)
        else:
            ext.dec_sqllm(self.dec_config, x, self.output, self.qweight, self.lut, self.bitwidth)
        return self._finish()
