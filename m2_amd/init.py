"""Seeded weights by parameter name.

`seeded_state_dict` returns CPU fp32 tensors keyed by the reference's state-dict names, drawn from
one `torch.Generator`.  The same dict is loaded into the HIP modules (`load_state_dict`) and handed
to the CPU oracle, so both sides see identical bits without depending on module construction order.
Recipe (mirrors the N(0, initializer_range) init Hugging Face `post_init` applies in the reference,
bert/src/bert_layers.py:939): Linear / Conv1d / Embedding / BlockdiagLinear weights and
`filter_fn*.bias` ~ N(0, 0.02); other biases 0; LayerNorm weight 1, bias 0; Sin.freq = hyena_w;
pos_emb.z, pos_emb.t, modulation.deltas from their closed forms.
"""
from __future__ import annotations

import math
from typing import Dict

import torch

from .config import M2BertConfig


def positional_embedding_buffers(emb_dim: int, seq_len: int):
    """(z (1, L, emb), t (1, L, 1)) as bert/src/mm/hyena_utils.py:66-88 builds them."""
    t = torch.linspace(0, 1, seq_len)[None, :, None]
    bands = (emb_dim - 1) // 2
    t_rescaled = torch.linspace(0, seq_len - 1, seq_len)[None, :, None]
    w = 2 * math.pi * t_rescaled / seq_len
    f = torch.linspace(1e-4, bands - 1, bands)[None, None]
    z = torch.exp(-1j * f * w)
    return torch.cat([t, z.real, z.imag], dim=-1), t


def modulation_deltas(d_model: int, fast_decay_pct: float = 0.3, slow_decay_pct: float = 1.5, target: float = 1e-2):
    """(1, 1, d) as bert/src/mm/hyena_utils.py:102-107."""
    max_decay = math.log(target) / fast_decay_pct
    min_decay = math.log(target) / slow_decay_pct
    return torch.linspace(min_decay, max_decay, d_model)[None, None]


def _normal(gen, *shape, std):
    return torch.empty(*shape).normal_(0.0, std, generator=gen)


def hyena_filter_state(prefix: str, cfg: M2BertConfig, gen, std: float) -> Dict[str, torch.Tensor]:
    d, order, emb, L = cfg.hidden_size, cfg.hyena_filter_order, cfg.hyena_emb_dim, cfg.long_conv_l_max
    sd = {prefix + "bias": _normal(gen, d, std=std)}
    z, t = positional_embedding_buffers(emb, L)
    sd[prefix + "pos_emb.z"] = z
    sd[prefix + "pos_emb.t"] = t
    freq = float(cfg.hyena_w) * torch.ones(1, order)
    for mlp in (["implicit_filter"] + (["implicit_filter_rev"] if cfg.bidirectional else [])):
        dims = [(order, emb), (order, order), (order, order)]
        for i, (o, k) in enumerate(dims):
            sd[f"{prefix}{mlp}.{2 * i}.weight"] = _normal(gen, o, k, std=std)
            sd[f"{prefix}{mlp}.{2 * i}.bias"] = torch.zeros(o)
            sd[f"{prefix}{mlp}.{2 * i + 1}.freq"] = freq      # one shared tensor in the reference
        sd[f"{prefix}{mlp}.6.weight"] = _normal(gen, d, order, std=std)
    sd[prefix + "modulation.deltas"] = modulation_deltas(d)
    return sd


def mixer_state(prefix: str, cfg: M2BertConfig, gen, std: float) -> Dict[str, torch.Tensor]:
    d = cfg.hidden_size
    sd = {}
    sd.update(hyena_filter_state(prefix + "filter_fn.", cfg, gen, std))
    if cfg.residual_long_conv:
        sd.update(hyena_filter_state(prefix + "filter_fn2.", cfg, gen, std))
    sd[prefix + "in_linear.weight"] = _normal(gen, 3 * d, d, std=std)
    sd[prefix + "in_linear.bias"] = torch.zeros(3 * d)
    sd[prefix + "out_linear.weight"] = _normal(gen, d, d, std=std)
    sd[prefix + "out_linear.bias"] = torch.zeros(d)
    sd[prefix + "short_filter.weight"] = _normal(gen, 3 * d, 1, 3, std=std)
    sd[prefix + "short_filter.bias"] = torch.zeros(3 * d)
    if cfg.hyena_training_additions:       # the extra pre-LayerNorm (monarch_mixer_sequence_mixer.py:84-87)
        sd[prefix + "layernorm.weight"] = torch.ones(d) + _normal(gen, d, std=std)
        sd[prefix + "layernorm.bias"] = _normal(gen, d, std=std)
    return sd


def mlp_state(prefix: str, cfg: M2BertConfig, gen, std: float) -> Dict[str, torch.Tensor]:
    d, I, nb = cfg.hidden_size, cfg.intermediate_size, cfg.monarch_mlp_nblocks
    return {
        prefix + "gated_layers.weight": _normal(gen, nb, 2 * I // nb, d // nb, std=std),
        prefix + "wo.weight": _normal(gen, nb, d // nb, I // nb, std=std),
        prefix + "wo.bias": torch.zeros(d),
        prefix + "layernorm.weight": torch.ones(d),
        prefix + "layernorm.bias": torch.zeros(d),
    }


def seeded_state_dict(cfg: M2BertConfig, seed: int, std: float | None = None, what: str = "model",
                      pooler: bool = True) -> Dict[str, torch.Tensor]:
    """`what`: 'model' (BertModel keys, with the pooler's unless pooler=False), 'mixer' (one
    MonarchMixerSequenceMixing), 'mlp' (one GLU MLP)."""
    gen = torch.Generator().manual_seed(seed)
    std = cfg.initializer_range if std is None else std
    if what == "mixer":
        return mixer_state("", cfg, gen, std)
    if what == "mlp":
        return mlp_state("", cfg, gen, std)
    d = cfg.hidden_size
    sd = {
        "embeddings.word_embeddings.weight": _normal(gen, cfg.vocab_size, d, std=std),
        "embeddings.token_type_embeddings.weight": _normal(gen, cfg.type_vocab_size, d, std=std),
        "embeddings.LayerNorm.weight": torch.ones(d),
        "embeddings.LayerNorm.bias": torch.zeros(d),
    }
    if cfg.use_positional_encodings:
        sd["embeddings.position_embeddings.weight"] = _normal(gen, cfg.max_position_embeddings, d, std=std)
        sd["embeddings.position_ids"] = torch.arange(cfg.max_position_embeddings).expand((1, -1)).clone()
    for i in range(cfg.num_hidden_layers):
        sd.update(mixer_state(f"encoder.layer.{i}.attention.", cfg, gen, std))
        sd.update(mlp_state(f"encoder.layer.{i}.mlp.", cfg, gen, std))
    if pooler:      # drawn last, so the other tensors do not depend on it
        sd["pooler.dense.weight"] = _normal(gen, d, d, std=std)
        sd["pooler.dense.bias"] = _normal(gen, d, std=std)
    return sd
