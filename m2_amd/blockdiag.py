"""BlockdiagLinear / blockdiag_multiply with the reference's interface, on bf16 MFMA.

Reference: bert/src/mm/blockdiag_linear.py:12-48, bert/src/mm/structured_linear.py:11-69,
bert/src/mm/blockdiag_multiply.py:19-60.  Under CUDA autocast, or with bf16 input, the arithmetic is
bf16 x bf16 with fp32 accumulation and a bf16 result (the reference's `custom_fwd(cast_inputs=bf16)`);
with fp32 input outside autocast it is fp32 throughout, as in the reference.  Inputs are zero-padded
to `in_features_extended` and outputs cropped to `out_features` like the reference's preprocess /
postprocess.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops


def _fp32_path(x: torch.Tensor) -> bool:
    """fp32 arithmetic exactly when the reference would use it: fp32 input and no CUDA autocast."""
    return x.dtype == torch.float32 and not torch.is_autocast_enabled()


def blockdiag_multiply(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x (..., nblocks*p), weight (nblocks, q, p) -> (..., nblocks*q)."""
    if not x.is_cuda:
        raise RuntimeError("blockdiag_multiply (m2_amd) runs on the GPU only")
    nb, q, p = weight.shape
    if x.shape[-1] != nb * p:
        raise ValueError(f"last dim {x.shape[-1]} != nblocks*p = {nb * p}")
    if _fp32_path(x) and p % 8 == 0:
        out = ops.blockdiag_linear_f32(x.reshape(-1, nb * p).contiguous(), weight.detach().float().contiguous())
        return out.view(*x.shape[:-1], nb * q)
    x2 = x.reshape(-1, nb * p).to(torch.bfloat16).contiguous()
    w = weight.detach().to(torch.bfloat16).contiguous()
    out_dtype = torch.bfloat16 if (x.dtype == torch.bfloat16 or torch.is_autocast_enabled()) else torch.float32
    out = ops.blockdiag_linear(x2, w, None, None, out_dtype=out_dtype)
    return out.view(*x.shape[:-1], nb * q)


class BlockdiagLinear(nn.Module):
    def __init__(self, in_features, out_features, bias=True, nblocks=4, shuffle=False, device=None, dtype=None):
        super().__init__()
        if shuffle:
            raise NotImplementedError("shuffle=True is not used by M2-BERT and is not built")
        self.in_features = in_features
        self.out_features = out_features
        in_blksz = int(math.ceil(in_features / nblocks))
        out_blksz = int(math.ceil(out_features / nblocks))
        self.in_features_extended = in_blksz * nblocks
        self.out_features_extended = out_blksz * nblocks
        self.shuffle = shuffle
        kw = {"device": device, "dtype": dtype}
        self.weight = nn.Parameter(torch.empty(nblocks, out_blksz, in_blksz, **kw))
        if bias:
            self.bias = nn.Parameter(torch.zeros(out_features, **kw))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()
        self._w16 = None

    def reset_parameters(self) -> None:
        # first block-row of a dense Kaiming-uniform matrix, rescaled for the sparsity
        # (bert/src/mm/blockdiag_linear.py:26-36, bert/src/mm/structured_linear.py:30-38)
        nb, q, p = self.weight.shape
        dense = torch.empty(self.out_features_extended, self.in_features_extended, dtype=self.weight.dtype)
        nn.init.kaiming_uniform_(dense, a=math.sqrt(5))
        dense *= math.sqrt(dense.numel() / self.weight.numel())
        with torch.no_grad():
            self.weight.copy_(dense[:q].reshape(q, nb, p).permute(1, 0, 2))
            if self.bias is not None:
                bound = 1 / math.sqrt(self.bias.shape[-1])
                nn.init.uniform_(self.bias, -bound, bound)

    @property
    def saving(self):
        return self.weight.numel() / (self.in_features * self.out_features)

    def weight_bf16(self) -> torch.Tensor:
        tag = (self.weight.data_ptr(), self.weight._version, self.weight.device)
        if self._w16 is None or self._w16[0] != tag:
            self._w16 = (tag, self.weight.detach().to(torch.bfloat16).contiguous())
        return self._w16[1]

    def forward(self, x):
        if not x.is_cuda:
            raise RuntimeError("BlockdiagLinear (m2_amd) runs on the GPU only")
        if x.shape[-1] < self.in_features_extended:
            x = F.pad(x, (0, self.in_features_extended - x.shape[-1]))
        bias = None
        if self.bias is not None:
            bias = self.bias.detach().float()
            if self.out_features_extended > self.out_features:
                bias = F.pad(bias, (0, self.out_features_extended - self.out_features))
            bias = bias.contiguous()
        nb, q, p = self.weight.shape
        if _fp32_path(x) and p % 8 == 0:
            out = ops.blockdiag_linear_f32(x.reshape(-1, self.in_features_extended).contiguous(),
                                           self.weight.detach().float().contiguous(), bias)
        else:
            x2 = x.reshape(-1, self.in_features_extended).to(torch.bfloat16).contiguous()
            out_dtype = torch.bfloat16 if (x.dtype == torch.bfloat16 or torch.is_autocast_enabled()) else torch.float32
            out = ops.blockdiag_linear(x2, self.weight_bf16(), bias, None, out_dtype=out_dtype)
        out = out.view(*x.shape[:-1], self.out_features_extended)
        if self.out_features_extended > self.out_features:
            out = out[..., :self.out_features]
        return out
