"""Caller-side module: a linear layer whose weight lives in the packed formats.

The reference is driven by an out-of-tree caller (reduced-kobold, README.md:1)
that keeps, per layer, the packed matrix, scales, zeros and optional 16:32 mask
and calls ``int4matmul.quant_matmul`` (int4matmul.cpp:26-48) with a freshly
zeroed output.  ``QuantLinear`` is that holder: buffers in the layouts the
kernels read, the call convention of kernel_test.py:254-259, and two ways to
fill it -- from already packed tensors, or by round-to-nearest quantisation of
an fp16 ``[in, out]`` weight, packed on the device by the library's packers.
"""
from __future__ import annotations

from typing import Optional

import torch

import int4matmul_kernels_amd as pkg
from int4matmul_kernels_amd import capi


class QuantLinear(torch.nn.Module):
    """y = x @ W_q (+ bias); x is fp16 ``[batch, seq, in_features]``.

    ``matrix``: int32 ``[in * bits / 32, out]`` (dense) or ``[in / 16, out]``
    (16:32 sparse, int4 only); ``scales`` / ``zeros``: fp16 ``[groups, out]``
    (``[out]`` when ``group_size < 0``); ``sparse_mask``: int32 ``[in / 32, out]``.
    """

    def __init__(self, bits: int, in_features: int, out_features: int, group_size: int = 128,
                 sparse: bool = False, bias: bool = False, device="cuda"):
        super().__init__()
        if bits not in (4, 3, 2):
            raise ValueError("bits must be 4, 3 or 2")
        if sparse and bits != 4:
            raise ValueError("16:32 sparsity is supported for int4 only")
        if in_features % 64 or out_features % 64:
            raise ValueError("in_features and out_features must be multiples of 64")
        if group_size == 0 or (group_size > 0 and group_size % 64):
            raise ValueError("group_size must be negative or a positive multiple of 64")
        self.bits, self.in_features, self.out_features = bits, in_features, out_features
        self.group_size, self.sparse = group_size, sparse
        rows = in_features // 16 if sparse else in_features * bits // 32
        groups = 1 if group_size < 0 else (in_features + group_size - 1) // group_size
        sz_shape = (out_features,) if group_size < 0 else (groups, out_features)
        self.register_buffer("matrix", torch.zeros((rows, out_features), dtype=torch.int32, device=device))
        self.register_buffer("scales", torch.ones(sz_shape, dtype=torch.float16, device=device))
        self.register_buffer("zeros", torch.zeros(sz_shape, dtype=torch.float16, device=device))
        self.register_buffer("sparse_mask", torch.zeros((in_features // 32, out_features), dtype=torch.int32,
                                                        device=device) if sparse else None)
        self.register_buffer("bias", torch.zeros((out_features,), dtype=torch.float16, device=device) if bias else None)

    # ------------------------------------------------------------------ filling
    @classmethod
    def from_packed(cls, bits: int, matrix, scales, zeros, group_size: int, sparse_mask=None, bias=None):
        out_features = matrix.shape[1]
        in_features = matrix.shape[0] * 16 if sparse_mask is not None else matrix.shape[0] * 32 // bits
        m = cls(bits, in_features, out_features, group_size, sparse_mask is not None, bias is not None,
                device=matrix.device)
        m.matrix.copy_(matrix)
        m.scales.copy_(scales.reshape(m.scales.shape))
        m.zeros.copy_(zeros.reshape(m.zeros.shape))
        if sparse_mask is not None:
            m.sparse_mask.copy_(sparse_mask)
        if bias is not None:
            m.bias.copy_(bias)
        return m

    @classmethod
    def from_float(cls, weight: torch.Tensor, bits: int = 4, group_size: int = 128, keep: Optional[torch.Tensor] = None,
                   bias=None):
        """Round-to-nearest asymmetric quantisation of ``weight`` (``[in, out]``) per
        (group, column): scale = (max - min) / (2^bits - 1), zero = -min / scale, code =
        clamp(round(w / scale + zero)).  ``keep`` (bool ``[in, out]``, exactly 16 of every 32
        consecutive inputs per column) selects the 16:32 format; dropped weights become 0."""
        K, S = weight.shape
        dev = weight.device
        m = cls(bits, K, S, group_size, keep is not None, bias is not None, device=dev)
        g = K if group_size < 0 else group_size
        w = weight.float()
        if keep is not None:
            w = torch.where(keep, w, torch.full_like(w, float("nan")))       # dropped weights do not shape the range
        pad = (-K) % g
        wp = torch.nn.functional.pad(w, (0, 0, 0, pad), value=float("nan")).reshape(-1, g, S)
        lo = torch.nan_to_num(wp, nan=float("inf")).amin(dim=1)
        hi = torch.nan_to_num(wp, nan=float("-inf")).amax(dim=1)
        lo = torch.where(torch.isfinite(lo), lo, torch.zeros_like(lo))
        hi = torch.where(torch.isfinite(hi), hi, torch.zeros_like(hi))
        qmax = float((1 << bits) - 1)
        scale = ((hi - lo) / qmax).clamp_min(1e-8).half()
        zero = (-lo / scale.float()).clamp(0, qmax).half()
        rows = torch.arange(K, device=dev) // g
        codes = torch.round(torch.nan_to_num(w) / scale.float()[rows] + zero.float()[rows]).clamp(0, qmax).to(torch.uint8)
        if keep is not None:
            capi.sparse_pack(m.matrix, m.sparse_mask, codes.t().contiguous(), keep.t().contiguous().to(torch.uint8))
        else:
            capi.dense_pack(bits, m.matrix, codes.contiguous())
        m.scales.copy_(scale.reshape(m.scales.shape))
        m.zeros.copy_(zero.reshape(m.zeros.shape))
        if bias is not None:
            m.bias.copy_(bias)
        return m

    # ------------------------------------------------------------------ forward
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        ext = pkg.load_extension()
        lead = x.shape[:-1]
        x3 = x.reshape(1, -1, self.in_features) if x.dim() != 3 else x
        x3 = x3.contiguous().half()
        outs = torch.zeros((x3.shape[0], x3.shape[1], self.out_features), dtype=torch.float16, device=x3.device)
        ext.quant_matmul(self.bits, outs, self.matrix, x3, self.scales, self.zeros, self.group_size, self.sparse_mask)
        y = outs.reshape(*lead, self.out_features)
        return y + self.bias if self.bias is not None else y

    def dequantized_weight(self) -> torch.Tensor:
        """fp16 ``[in, out]`` weights exactly as the kernels decode them"""
        w = torch.empty((self.in_features, self.out_features), dtype=torch.float16, device=self.matrix.device)
        capi.dequantize(self.bits, w, self.matrix, self.scales, self.zeros, self.group_size, self.sparse_mask)
        return w

    def extra_repr(self) -> str:
        return (f"bits={self.bits}, in_features={self.in_features}, out_features={self.out_features}, "
                f"group_size={self.group_size}, sparse={self.sparse}")
