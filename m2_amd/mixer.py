"""MonarchMixerSequenceMixing with the reference's constructor and state dict, computed by the fused
HIP mixer core (bert/src/mm/monarch_mixer_sequence_mixer.py:12-154).

Data flow of `forward(u)`, u (B, L, d):

    xproj (3d, B*L) = in_linear.weight @ u^T + bias       one library GEMM, written CHANNEL-major
    spec            = spectra of the two bidirectional implicit filters (skip weights folded in)
    y (d, B*L)      = m2_mixer_core_fwd(xproj, u^T, short_filter, spec)
    out (B*L, d)    = y^T @ out_linear.weight^T + bias     one library GEMM

so the three `transpose` passes of the reference disappear into GEMM operand orientation.  With fp32
input outside autocast everything is fp32; with bf16 input or under CUDA autocast the projections
and the stored activations are bf16 while the FFT convolution stays fp32.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from . import ops
from .hyena import HyenaFilter


class MonarchMixerSequenceMixing(nn.Module):
    def __init__(self, d_model, l_max=128, dropout=0.0, hyena_kernel_lr=None, bidirectional=False,
                 hyena_lr_pos_emb=1e-5, hyena_w=10, hyena_w_mod=1, hyena_wd=0.1, hyena_emb_dim=3,
                 hyena_filter_dropout=0.0, hyena_filter_order=16, residual_long_conv=False,
                 hyena_training_additions=False):
        super().__init__()
        self.d_model = d_model
        self.l_max = l_max
        self.kernel_lr = hyena_kernel_lr
        self.channels = 1
        self.bidirectional = bidirectional
        self.residual_long_conv = residual_long_conv
        self.NUM_PROJECTIONS = 3
        self.hyena_training_additions = hyena_training_additions

        def make_filter():
            return HyenaFilter(self.d_model, order=hyena_filter_order, seq_len=self.l_max, dropout=hyena_filter_dropout,
                               bidirectional=self.bidirectional, lr=hyena_kernel_lr, lr_pos_emb=hyena_lr_pos_emb,
                               w=hyena_w, w_mod=hyena_w_mod, wd=hyena_wd, emb_dim=hyena_emb_dim)

        self.filter_fn = make_filter()
        if self.residual_long_conv:
            self.filter_fn2 = make_filter()
        self.in_linear = nn.Linear(d_model, 3 * d_model)
        self.out_linear = nn.Linear(d_model, d_model)
        if self.hyena_training_additions:
            # extra pre-LayerNorm; the dropouts and the Identity activation do nothing in a forward-only path
            # (bert/src/mm/monarch_mixer_sequence_mixer.py:84-87,102-103,118-119,150-151)
            self.act = nn.Identity()
            self.drop = nn.Dropout(dropout)
            self.layernorm = nn.LayerNorm(d_model)
        total_width = self.d_model * self.NUM_PROJECTIONS
        self.short_filter = nn.Conv1d(in_channels=total_width, out_channels=total_width, kernel_size=3,
                                      groups=total_width, padding=2)
        self._cast_cache = {}
        self.cache_filters = False
        self._spec_cache = None
        self._filter_table = None

    # -- helpers -----------------------------------------------------------------------------
    def _cast(self, name: str, p: torch.Tensor, dtype) -> torch.Tensor:
        """Cached cast of a parameter (re-done when the parameter changes)."""
        key = (name, dtype)
        tag = (p.data_ptr(), p._version, p.device)
        hit = self._cast_cache.get(key)
        if hit is None or hit[0] != tag:
            hit = (tag, p.detach().to(dtype).contiguous())
            self._cast_cache[key] = hit
        return hit[1]

    def filter_spectrum(self, L: int) -> torch.Tensor:
        """Spectra of filter_fn (and filter_fn2) for sequence length L, generated from the weights.

        The reference regenerates its filters in every forward and so does this by default.  With
        `self.cache_filters = True` (inference with frozen weights) the spectra are kept and reused until a
        filter parameter or buffer changes (in-place updates bump the tensor version; re-assignment changes
        the storage pointer)."""
        fns = [self.filter_fn] + ([self.filter_fn2] if self.residual_long_conv else [])
        if self.cache_filters:
            tag = (L,) + tuple((t.data_ptr(), t._version) for f in fns
                               for t in list(f.parameters()) + list(f.buffers()))
            hit = self._spec_cache
            if hit is not None and hit[0] == tag:
                return hit[1]
            spec = self._generate_spectrum(L, fns)
            self._spec_cache = (tag, spec)
            return spec
        return self._generate_spectrum(L, fns)

    def filter_table_entry(self):
        """(filters, skip weights) of this mixer for an `ops.FilterTable`: filter_fn, then filter_fn2 if present."""
        fns = [self.filter_fn] + ([self.filter_fn2] if self.residual_long_conv else [])
        filters = [f.kernel_params("both") for f in fns]
        skips = []
        for f in fns:
            b = f.bias.detach()
            skips.append(b if (b.dtype == torch.float32 and b.is_contiguous()) else b.float().contiguous())
        return filters, skips

    def _generate_spectrum(self, L: int, fns) -> torch.Tensor:
        """All of filter generation in one library call: hidden layers, projection + decay, window, skip weight,
        transform (for L <= 512 the taps never reach memory)."""
        f0 = self.filter_fn
        filters, skips = self.filter_table_entry()
        table = self._filter_table
        key_probe = (L,) + tuple(t.data_ptr() for f in filters for v in f.values()
                                 for t in (v if isinstance(v, list) else [v])) + tuple(b.data_ptr() for b in skips)
        if table is None or table[0] != key_probe:
            table = (key_probe, ops.FilterTable([filters], [skips], L, self.d_model, f0.order, f0.emb_dim))
            self._filter_table = table
        return ops.mixer_filter_spectra(table[1], w_mod=float(f0.w_mod), shift=float(f0.modulation.shift))[0]

    def core(self, xproj: torch.Tensor, u_cm: Optional[torch.Tensor], B: int, L: int,
             spec: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Channel-major core: xproj (3d, B, L) = in_linear.weight @ u^T WITHOUT the bias (the kernel adds
        in_linear.bias as it loads), u_cm (d, B, L) fp32 -> y (d, B, L)."""
        if spec is None:
            spec = self.filter_spectrum(L)
        sw = self._cast("short_w", self.short_filter.weight, torch.float32).view(3 * self.d_model, 3)
        sb = self._cast("short_b", self.short_filter.bias, torch.float32)
        pb = self._cast("in_b32", self.in_linear.bias, torch.float32)
        return ops.mixer_core(xproj, u_cm, sw, sb, spec, B, L, self.d_model, proj_bias=pb)

    def pre_norm(self, h32: torch.Tensor, want_f32: bool, want_bf16: bool):
        """The extra input LayerNorm of hyena_training_additions: (M, d) fp32 -> (f32 | None, bf16 | None,
        channel-major f32 (d, M) | None when there is no residual long convolution)."""
        ln = self.layernorm
        return ops.layernorm(h32, ln.weight.detach().float(), ln.bias.detach().float(), ln.eps, want_f32=want_f32,
                             want_bf16=want_bf16, want_channel_major=self.residual_long_conv)

    # -- reference API -----------------------------------------------------------------------
    def forward(self, u, **kwargs):
        if not u.is_cuda:
            raise RuntimeError("MonarchMixerSequenceMixing (m2_amd) runs on the GPU only")
        B, L, d = u.shape
        if d != self.d_model:
            raise ValueError(f"expected last dim {self.d_model}, got {d}")
        low = u.dtype == torch.bfloat16 or torch.is_autocast_enabled()
        act = torch.bfloat16 if low else torch.float32
        u2 = u.reshape(B * L, d)
        w_in = self._cast("in_w", self.in_linear.weight, act)
        w_out = self._cast("out_w", self.out_linear.weight, act)
        b_out = self._cast("out_b", self.out_linear.bias, act)
        with torch.autocast("cuda", enabled=False):
            u_cm = None
            if self.hyena_training_additions:
                if self.training and self.drop.p > 0:
                    raise NotImplementedError("m2_amd is a forward/inference path: call .eval() first")
                u2, u16, u_cm = self.pre_norm(u2.float().contiguous(), want_f32=not low, want_bf16=low)
                if low:
                    u2 = u16
            xproj = torch.empty(3 * d, B * L, dtype=act, device=u.device)               # (3d, B*L), bias added in the core
            torch.mm(u2.to(act), w_in.t(), out=xproj.t())
            if u_cm is None and self.residual_long_conv:
                u_cm = u2.float().t().contiguous()                                       # (d, B*L)
            if not self.residual_long_conv:
                u_cm = None
            y = self.core(xproj.view(3 * d, B, L), None if u_cm is None else u_cm.view(d, B, L), B, L)
            out = torch.addmm(b_out, y.view(d, B * L).t(), w_out.t())                   # (B*L, d)
        return out.view(B, L, d), None
