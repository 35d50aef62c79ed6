"""HyenaFilter and its parts with the reference's constructor arguments and state-dict names, the
arithmetic done by the HIP kernels of libm2_amd.so.

Reference: bert/src/mm/hyena_utils.py:50-63 (Sin), :66-88 (PositionalEmbedding), :91-112
(ExponentialModulation), :115-248 (HyenaFilter), bert/src/utils/train.py:4-17 (OptimModule).
The submodules hold parameters and buffers under the same names.  The hot path does not call their
`forward`s (the whole filter is produced by `m2_hyena_filter_fwd`); a caller that evaluates them directly, as
bert/src/mm/flash_mm.py:141-149 does with `filter_fn.implicit_filter(z)`, gets the reference's own expressions
as plain torch ops on whatever device the tensors live on.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from . import ops
from .init import modulation_deltas, positional_embedding_buffers


class OptimModule(nn.Module):
    """`register(name, tensor, lr)`: a buffer when lr == 0.0, else a parameter carrying `_optim`
    hyper-parameters (bert/src/utils/train.py:7-17)."""

    def register(self, name, tensor, lr=None, wd=0.0):
        if lr == 0.0:
            self.register_buffer(name, tensor)
        else:
            self.register_parameter(name, nn.Parameter(tensor))
            optim = {}
            if lr is not None:
                optim["lr"] = lr
            if wd is not None:
                optim["weight_decay"] = wd
            setattr(getattr(self, name), "_optim", optim)


class Sin(nn.Module):
    """sin(w_mod * freq * x) (bert/src/mm/hyena_utils.py:50-63); one instance, hence one `freq`, is shared by every
    activation slot of both implicit-filter MLPs."""

    def __init__(self, dim, w=10, w_mod=1, train_freq=True):
        super().__init__()
        init = w * torch.ones(1, dim)
        self.freq = nn.Parameter(init) if train_freq else init
        self.w_mod = w_mod

    def forward(self, x):
        return torch.sin(self.w_mod * self.freq * x)


class PositionalEmbedding(OptimModule):
    def __init__(self, emb_dim: int, seq_len: int, lr_pos_emb: float = 1e-5, **kwargs):
        super().__init__()
        self.seq_len = seq_len
        z, t = positional_embedding_buffers(emb_dim, seq_len)
        self.register("z", z, lr=lr_pos_emb)
        self.register("t", t, lr=0.0)

    def forward(self, L):
        return self.z[:, :L], self.t[:, :L]


class ExponentialModulation(OptimModule):
    def __init__(self, d_model, fast_decay_pct=0.3, slow_decay_pct=1.5, target=1e-2, modulation_lr=0.0,
                 shift: float = 0.0, **kwargs):
        super().__init__()
        self.shift = shift
        self.register("deltas", modulation_deltas(d_model, fast_decay_pct, slow_decay_pct, target), lr=modulation_lr)

    def forward(self, t, x):
        """x * (exp(-t |deltas|) + shift) (bert/src/mm/hyena_utils.py:110-112)."""
        decay = torch.exp(-t * self.deltas.abs())
        return x * (decay + self.shift)


class HyenaFilter(OptimModule):
    """Implicit long filter with exponential-decay modulation (bert/src/mm/hyena_utils.py:115-248)."""

    def __init__(self, d_model, emb_dim=3, order=16, seq_len=1024, lr=1e-3, lr_pos_emb=1e-5, dropout=0.0, w=1,
                 w_mod=1, wd=0, bias=True, num_inner_mlps=2, linear_mixer=False, modulate: bool = True,
                 normalized=False, bidirectional=False, **kwargs):
        super().__init__()
        if linear_mixer or not modulate or normalized or num_inner_mlps != 2:
            raise NotImplementedError("the HIP filter kernel covers the M2-BERT setting: sin-MLP with two inner layers, "
                                      "modulate=True, normalized=False, linear_mixer=False")
        assert emb_dim % 2 != 0 and emb_dim >= 3, "emb_dim must be odd and greater or equal to 3 (time, sine and cosine)"
        self.d_model = d_model
        self.emb_dim = emb_dim
        self.order = order
        self.seq_len = seq_len
        self.modulate = modulate
        self.use_bias = bias
        self.bidirectional = bidirectional
        self.normalized = normalized
        self.w_mod = w_mod

        self.bias = nn.Parameter(torch.randn(self.d_model))
        self.dropout = nn.Dropout(dropout)
        act = Sin(dim=order, w=w, w_mod=w_mod)
        self.pos_emb = PositionalEmbedding(emb_dim, seq_len, lr_pos_emb)

        def mlp():
            return nn.Sequential(nn.Linear(emb_dim, order), act, nn.Linear(order, order), act,
                                 nn.Linear(order, order), act, nn.Linear(order, d_model, bias=False))

        self.implicit_filter = mlp()
        if self.bidirectional:
            self.implicit_filter_rev = mlp()
        self.modulation = ExponentialModulation(d_model, **kwargs)
        for c in self.implicit_filter.children():
            for name, _ in c.state_dict().items():
                setattr(getattr(c, name), "_optim", {"weight_decay": wd, "lr": lr})
        self.flashfft = None

    # -- kernel plumbing -------------------------------------------------------------------
    def _mlp_tensors(self, seq: nn.Sequential):
        return [seq[0].weight, seq[0].bias, seq[2].weight, seq[2].bias, seq[4].weight, seq[4].bias, seq[6].weight]

    def kernel_params(self, which: str = "both") -> dict:
        """Tensor bundle for `ops.hyena_filter_taps`; `which` in {'both', 'fwd', 'rev'}."""
        p = {"z": self.pos_emb.z, "t": self.pos_emb.t, "freq": self.implicit_filter[1].freq,
             "deltas": self.modulation.deltas}
        if which == "rev":
            p["fwd"] = self._mlp_tensors(self.implicit_filter_rev)
        else:
            p["fwd"] = self._mlp_tensors(self.implicit_filter)
            if which == "both" and self.bidirectional:
                p["rev"] = self._mlp_tensors(self.implicit_filter_rev)
        def plain(t):      # the kernels read fp32, contiguous tensors; parameters normally are, and then this is a view
            t = t.detach()
            return t if (t.dtype == torch.float32 and t.is_contiguous()) else t.float().contiguous()
        return {k: ([plain(t) for t in v] if isinstance(v, list) else plain(v)) for k, v in p.items()}

    def _taps(self, L: int, which: str) -> torch.Tensor:
        if L > self.seq_len:
            raise ValueError(f"L={L} exceeds the filter's seq_len={self.seq_len}")
        return ops.hyena_filter_taps([self.kernel_params(which)], L, self.d_model, self.order, self.emb_dim,
                                     w_mod=float(self.w_mod), shift=float(self.modulation.shift))[0]

    # -- reference API ---------------------------------------------------------------------
    def filter(self, L, *args, **kwargs):
        """(1, L, d) forward taps."""
        return self._taps(L, "fwd")[:, :L].transpose(0, 1).unsqueeze(0)

    def filter_rev(self, L, *args, **kwargs):
        """(1, L, d) reverse taps."""
        return self._taps(L, "rev")[:, :L].transpose(0, 1).unsqueeze(0)

    def bidirectional_taps(self, L: int) -> torch.Tensor:
        """(d, 2L): forward taps then the flipped reverse taps, as the long convolution consumes them."""
        return self._taps(L, "both")

    def forward(self, x, L, k_fwd=None, k_rev=None, bias=None, *args, **kwargs):
        """y = fftconv(x, k) + x * bias for x (B, d, L); k_fwd / k_rev (d, L) or (1, L, d)-style tuples."""
        B, d, Lx = x.shape
        if k_fwd is None:
            taps = self.bidirectional_taps(L)
        else:
            k_fwd = k_fwd[0] if type(k_fwd) is tuple else k_fwd
            if self.bidirectional:
                k_rev = k_rev[0] if type(k_rev) is tuple else k_rev
                taps = torch.cat([k_fwd.float(), k_rev.float().flip(-1)], dim=-1).contiguous()
            else:
                taps = torch.cat([k_fwd.float(), torch.zeros_like(k_fwd, dtype=torch.float32)], dim=-1).contiguous()
        if bias is None:
            bias = self.bias
        D = bias.detach().float().reshape(-1).contiguous()
        if not self.use_bias:
            D = torch.zeros_like(D)
        spec = ops.filter_spectrum(taps, None, D, None)
        act = x if x.dtype in (torch.float32, torch.bfloat16) else x.float()
        xc = act.permute(1, 0, 2).contiguous()                       # (d, B, L)
        y = ops.fftconv(xc, spec, B, Lx, d)
        return y.permute(1, 0, 2).contiguous().to(dtype=x.dtype)
