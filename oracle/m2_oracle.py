"""CPU oracle for the M2-BERT Monarch-Mixer forward path.

THIS IS TEST INFRASTRUCTURE.  It is a plain-PyTorch restatement, on the CPU, of the
reference's `use_flash_mm=False, use_flash_fft=False` forward path.  Only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import it, and only
as the checker; nothing in the shipped `m2_amd` package imports, calls or falls back to it.

Every function takes plain tensors or a flat ``{name: tensor}`` state dict whose keys are the
reference's own parameter / buffer names, so that the same weights can be loaded into the HIP
modules with ``load_state_dict`` and handed to this file unchanged.  All arithmetic runs in the
dtype of the tensors handed in (fp32 for parity runs, fp64 when a test wants a tighter pin).  The functions
are plain torch ops with the reference's own expressions and dtype flow (`.to(k.dtype)` before the FFT,
`bias.to(out.dtype)` in the structured linear), so a test may also run them on GPU tensors under
`torch.autocast("cuda", dtype=torch.bfloat16)` to obtain the reference's mixed-precision numerics as PyTorch
itself defines them.

What pins each function (tests/test_oracle_*.py; no reference code is imported or run):

  positional_embedding   closed form + spot values           (bert/src/mm/hyena_utils.py:66-88)
  modulation_deltas      closed form, two constants          (bert/src/mm/hyena_utils.py:91-112)
  hyena_filter_taps      independent float64 numpy MLP       (bert/src/mm/hyena_utils.py:50-63,168-217)
  bidirectional_kernel   index identities                    (bert/src/mm/hyena_utils.py:231-236)
  fftconv                O(L^2) float64 direct sum, scipy.signal.fftconvolve, linearity,
                         causality, delta filter             (bert/src/mm/hyena_utils.py:16-42)
  short_conv             3-tap direct sum vs F.conv1d        (bert/src/mm/monarch_mixer_sequence_mixer.py:90-97,112)
  mixer_forward          composition of the above            (bert/src/mm/monarch_mixer_sequence_mixer.py:100-154)
  blockdiag_multiply     dense block_diag matmul             (bert/src/mm/blockdiag_multiply.py:9-34,49-60)
  blockdiag_linear       dense F.linear                      (bert/src/mm/structured_linear.py:52-69)
  glu_mlp_forward        dense equivalent + library GELU/LN  (bert/src/bert_layers.py:482-508)
  layer_forward          composition                         (bert/src/bert_layers.py:575-599)
  encoder_forward        composition, mask independence      (bert/src/bert_layers.py:691-813)
  embeddings_forward     gather + library LayerNorm          (bert/src/bert_layers.py:191-252)

The reference holds no golden vectors for this path (its only test-like file prints diffs of
random data), so nothing here is pinned by a reference fixture; everything is pinned by the
mathematics as listed.  State-dict key names and ordering are taken from reading the reference
and are not checked against an import: "parity unpinned" applies to the *naming* only.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch
import torch.nn.functional as F

Tensor = torch.Tensor
StateDict = Dict[str, Tensor]


# --------------------------------------------------------------------------------------
# HyenaFilter pieces
# --------------------------------------------------------------------------------------
def positional_embedding(emb_dim: int, seq_len: int, dtype=torch.float32):
    """z (1, seq_len, emb_dim) and t (1, seq_len, 1) of the implicit-filter positional embedding.

    Follows bert/src/mm/hyena_utils.py:66-88: t = linspace(0, 1, L); w_l = 2*pi*l/L;
    bands = (emb_dim-1)//2; f = linspace(1e-4, bands-1, bands);
    z = [t, Re exp(-i f w), Im exp(-i f w)] = [t, cos(f w), -sin(f w)].
    The reference builds these in fp32; we build in fp32 and cast so that fp64 runs see the
    same constants the model would hold.
    """
    assert emb_dim % 2 == 1 and emb_dim >= 3
    t = torch.linspace(0, 1, seq_len, dtype=torch.float32)[None, :, None]
    bands = (emb_dim - 1) // 2
    t_rescaled = torch.linspace(0, seq_len - 1, seq_len, dtype=torch.float32)[None, :, None]
    w = 2 * math.pi * t_rescaled / seq_len
    f = torch.linspace(1e-4, bands - 1, bands, dtype=torch.float32)[None, None]
    ang = f * w
    z = torch.cat([t, torch.cos(ang), -torch.sin(ang)], dim=-1)
    return z.to(dtype), t.to(dtype)


def modulation_deltas(d_model: int, fast_decay_pct: float = 0.3, slow_decay_pct: float = 1.5,
                      target: float = 1e-2, dtype=torch.float32) -> Tensor:
    """deltas (1, 1, d) of ExponentialModulation (bert/src/mm/hyena_utils.py:102-107)."""
    max_decay = math.log(target) / fast_decay_pct
    min_decay = math.log(target) / slow_decay_pct
    return torch.linspace(min_decay, max_decay, d_model, dtype=torch.float32)[None, None].to(dtype)


def hyena_filter_taps(sd: StateDict, prefix: str, L: int, rev: bool = False,
                      w_mod: float = 1.0, shift: float = 0.0) -> Tensor:
    """Implicit filter h (1, L, d): sin-MLP over the positional embedding, then decay.

    bert/src/mm/hyena_utils.py:201-217 (`filter` / `filter_rev`), :50-63 (`Sin`),
    :110-112 (`ExponentialModulation.forward`).  One `freq` tensor is shared by all
    activation slots of both MLPs (:160), so it is read from `implicit_filter.1.freq`.
    """
    mlp = prefix + ("implicit_filter_rev." if rev else "implicit_filter.")
    z = sd[prefix + "pos_emb.z"][:, :L]
    t = sd[prefix + "pos_emb.t"][:, :L]
    freq = sd[prefix + "implicit_filter.1.freq"]
    h = z
    idx = 0
    while (mlp + f"{idx}.weight") in sd:
        w = sd[mlp + f"{idx}.weight"]
        b = sd.get(mlp + f"{idx}.bias")
        h = F.linear(h, w, None if b is None else b)
        if (mlp + f"{idx + 2}.weight") in sd:      # every Linear but the last is followed by Sin
            h = torch.sin(w_mod * freq * h)
        idx += 2
    deltas = sd[prefix + "modulation.deltas"]
    decay = torch.exp(-t * deltas.abs())
    return h * (decay + shift)


def bidirectional_kernel(k_fwd: Tensor, k_rev: Optional[Tensor], L: int) -> Tensor:
    """(d, L),(d, L) -> (d, 2L): pad(k_fwd,(0,L)) + pad(flip(k_rev),(L,0)).

    bert/src/mm/hyena_utils.py:231-236.
    """
    if k_rev is None:
        return k_fwd
    return F.pad(k_fwd, (0, L)) + F.pad(k_rev.flip(-1), (L, 0))


def fftconv(u: Tensor, k: Tensor, D: Tensor) -> Tensor:
    """y = irfft(rfft(u, 2L) * rfft(k, 2L) / 2L, norm='forward')[..., :L] + u * D.

    u (B, d, L), k (d, Lk) with Lk <= 2L, D broadcastable to u.
    bert/src/mm/hyena_utils.py:16-42 with gelu=False, dropout_mask=None, k_rev=None.
    """
    L = u.shape[-1]
    n = 2 * L
    k_f = torch.fft.rfft(k, n=n) / n
    u_f = torch.fft.rfft(u.to(k.dtype), n=n)
    y = torch.fft.irfft(u_f * k_f, n=n, norm="forward")[..., :L]
    return (y + u * D).to(u.dtype)


def hyena_filter_forward(x: Tensor, L: int, k_fwd: Tensor, k_rev: Optional[Tensor], bias: Tensor) -> Tensor:
    """HyenaFilter.forward (bert/src/mm/hyena_utils.py:219-248) with explicit taps."""
    return fftconv(x, bidirectional_kernel(k_fwd, k_rev, L), bias)


# --------------------------------------------------------------------------------------
# Sequence mixer
# --------------------------------------------------------------------------------------
def short_conv(u: Tensor, weight: Tensor, bias: Tensor) -> Tensor:
    """Depthwise Conv1d(kernel 3, padding 2)[..., :L] on u (B, C, L).

    bert/src/mm/monarch_mixer_sequence_mixer.py:90-97,112; closed form
    out[b,c,t] = bias[c] + sum_j w[c,0,j] * u[b,c,t-2+j] (zero for negative index).
    """
    L = u.shape[-1]
    ksz = weight.shape[-1]
    return F.conv1d(u, weight, bias, padding=ksz - 1, groups=u.shape[1])[..., :L]


def mixer_filters(sd: StateDict, prefix: str, L: int, bidirectional: bool = True,
                  residual_long_conv: bool = True, w_mod: float = 1.0):
    """The (up to) four tap sets of one mixer, each (d, L): k, k_rev, k2, k2_rev."""
    out = []
    for fn in (["filter_fn."] + (["filter_fn2."] if residual_long_conv else [])):
        k = hyena_filter_taps(sd, prefix + fn, L, rev=False, w_mod=w_mod)[0].transpose(0, 1)
        kr = hyena_filter_taps(sd, prefix + fn, L, rev=True, w_mod=w_mod)[0].transpose(0, 1) if bidirectional else None
        out += [k, kr]
    return out


def mixer_forward(sd: StateDict, prefix: str, u: Tensor, bidirectional: bool = True,
                  residual_long_conv: bool = True, w_mod: float = 1.0,
                  training_additions: bool = False) -> Tensor:
    """MonarchMixerSequenceMixing.forward in eval mode, u (B, L, d) -> (B, L, d).

    bert/src/mm/monarch_mixer_sequence_mixer.py:100-154.  With hyena_training_additions the input goes through
    an extra nn.LayerNorm(d_model) (default eps 1e-5, :84-87, :102-103) and that normalised input is also what
    the residual long convolution sees (:107); the two dropouts and the Identity activation (:118-119,
    :150-151) do nothing in eval mode.
    """
    B, L, d = u.shape
    if training_additions:
        u = F.layer_norm(u, (d,), sd[prefix + "layernorm.weight"], sd[prefix + "layernorm.bias"], 1e-5)
    u_orig = u
    x = F.linear(u, sd[prefix + "in_linear.weight"], sd[prefix + "in_linear.bias"])
    x = x.transpose(1, 2)                                             # (B, 3d, L)
    uc = short_conv(x, sd[prefix + "short_filter.weight"], sd[prefix + "short_filter.bias"])
    x1, x2, v = uc.split(d, dim=1)
    v = v * x1
    filt = mixer_filters(sd, prefix, L, bidirectional, residual_long_conv, w_mod)
    y = hyena_filter_forward(v, L, filt[0], filt[1], sd[prefix + "filter_fn.bias"][None, :, None])
    y = y * x2
    if residual_long_conv:
        yu = hyena_filter_forward(u_orig.transpose(1, 2), L, filt[2], filt[3],
                                  sd[prefix + "filter_fn2.bias"][None, :, None])
        y = y + yu
    y = y.transpose(1, 2)
    return F.linear(y, sd[prefix + "out_linear.weight"], sd[prefix + "out_linear.bias"])


# --------------------------------------------------------------------------------------
# Block-diagonal ("Monarch") linear and the GLU MLP
# --------------------------------------------------------------------------------------
def blockdiag_multiply(x: Tensor, weight: Tensor) -> Tensor:
    """out[..., k*q + j] = sum_i x[..., k*p + i] * weight[k, j, i].

    bert/src/mm/blockdiag_multiply.py:19-34 (einsum reference) and :49-60 (bmm form).
    """
    nb, q, p = weight.shape
    assert x.shape[-1] == nb * p
    xs = x.reshape(*x.shape[:-1], nb, p)
    return torch.einsum("...kp,kqp->...kq", xs, weight).reshape(*x.shape[:-1], nb * q)


def blockdiag_linear(x: Tensor, weight: Tensor, bias: Optional[Tensor], in_features: int,
                     out_features: int) -> Tensor:
    """BlockdiagLinear.forward: pad input, multiply, crop, add bias.

    bert/src/mm/structured_linear.py:52-69, bert/src/mm/blockdiag_linear.py:42-48.
    """
    nb, q, p = weight.shape
    if x.shape[-1] < nb * p:
        x = F.pad(x, (0, nb * p - x.shape[-1]))
    out = blockdiag_multiply(x, weight)[..., :out_features]
    return out + bias.to(out.dtype) if bias is not None else out


def glu_mlp_forward(sd: StateDict, prefix: str, x: Tensor, intermediate_size: int,
                    layer_norm_eps: float = 1e-12) -> Tensor:
    """BertGatedLinearUnitMLP.forward with BlockdiagLinear layers, x (B, L, d).

    bert/src/bert_layers.py:482-508: h = gated_layers(x); gelu_erf(h[..., :I]) * h[..., I:];
    wo; LayerNorm(wo_out + x).  Dropout is the identity in eval mode.
    """
    d = x.shape[-1]
    I = intermediate_size
    h = blockdiag_linear(x, sd[prefix + "gated_layers.weight"], None, d, 2 * I)
    a = F.gelu(h[..., :I]) * h[..., I:]
    o = blockdiag_linear(a, sd[prefix + "wo.weight"], sd[prefix + "wo.bias"], I, d)
    return F.layer_norm(o + x, (d,), sd[prefix + "layernorm.weight"], sd[prefix + "layernorm.bias"],
                        layer_norm_eps)


# --------------------------------------------------------------------------------------
# Layer / encoder / embeddings
# --------------------------------------------------------------------------------------
def layer_forward(sd: StateDict, prefix: str, x: Tensor, cfg) -> Tensor:
    """BertLayer.forward, M2 branch: mlp(attention(x)); no norm/residual around the mixer.

    bert/src/bert_layers.py:575-599.
    """
    a = mixer_forward(sd, prefix + "attention.", x, cfg.bidirectional, cfg.residual_long_conv,
                      cfg.hyena_w_mod, getattr(cfg, "hyena_training_additions", False))
    return glu_mlp_forward(sd, prefix + "mlp.", a, cfg.intermediate_size, cfg.layer_norm_eps)


def encoder_forward(sd: StateDict, prefix: str, x: Tensor, attention_mask: Optional[Tensor], cfg,
                    output_all_encoded_layers: bool = False) -> List[Tensor]:
    """BertEncoder.forward, M2 branch (bert/src/bert_layers.py:691-813).

    The attention mask never reaches an M2 layer (:577, :721-726): pad positions are
    convolved like real tokens.  It is accepted and ignored here on purpose.
    """
    outs = []
    for i in range(cfg.num_hidden_layers):
        x = layer_forward(sd, f"{prefix}layer.{i}.", x, cfg)
        if output_all_encoded_layers:
            outs.append(x)
    if not output_all_encoded_layers:
        outs.append(x)
    return outs


def embeddings_forward(sd: StateDict, prefix: str, input_ids: Tensor, cfg,
                       token_type_ids: Optional[Tensor] = None) -> Tensor:
    """BertEmbeddings.forward (bert/src/bert_layers.py:191-252), eval mode."""
    B, L = input_ids.shape
    e = F.embedding(input_ids, sd[prefix + "word_embeddings.weight"])
    if token_type_ids is None:
        token_type_ids = torch.zeros_like(input_ids)
    e = e + F.embedding(token_type_ids, sd[prefix + "token_type_embeddings.weight"])
    if cfg.use_positional_encodings:
        e = e + sd[prefix + "position_embeddings.weight"][:L][None]
    return F.layer_norm(e, (e.shape[-1],), sd[prefix + "LayerNorm.weight"], sd[prefix + "LayerNorm.bias"],
                        cfg.layer_norm_eps)


def pooler_forward(sd: StateDict, prefix: str, hidden: Tensor, mask: Optional[Tensor], pool_all: bool) -> Tensor:
    """BertPooler.forward (bert/src/bert_layers.py:816-859) without sequence_token_planting:
    tanh(dense(first token)), or with pool_all tanh(dense(mean over the positions whose mask is 1))."""
    if not pool_all:
        pooled = hidden[:, 0]
    else:
        m = mask.to(hidden.dtype)
        pooled = (hidden * m.unsqueeze(-1)).sum(dim=1) / m.sum(dim=1, keepdim=True)
    return torch.tanh(F.linear(pooled, sd[prefix + "dense.weight"], sd[prefix + "dense.bias"]))


def model_forward(sd: StateDict, input_ids: Tensor, attention_mask: Optional[Tensor], cfg,
                  prefix: str = "", pooled: bool = False):
    """BertModel.forward: embeddings -> encoder, last hidden state (B, L, d); with pooled=True also the
    pooler's output, as a pair.

    bert/src/bert_layers.py:948-1010.
    """
    x = embeddings_forward(sd, prefix + "embeddings.", input_ids, cfg)
    seq = encoder_forward(sd, prefix + "encoder.", x, attention_mask, cfg)[-1]
    if not pooled:
        return seq
    if attention_mask is None:
        attention_mask = torch.ones_like(input_ids)
    return seq, pooler_forward(sd, prefix + "pooler.", seq, attention_mask, getattr(cfg, "pool_all", False))


def cast_state_dict(sd: StateDict, dtype) -> StateDict:
    return {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in sd.items()}
