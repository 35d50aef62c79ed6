"""Loading reference-style checkpoints (Composer nesting, `model.bert.` prefixes, head keys, context extension).
Runs on the CPU: modules can be built and loaded without a GPU, only their forward needs one."""
import os

import pytest
import torch

import m2_amd
from m2_amd import checkpoint as ck


def _reference_style(sd, extra_heads=True):
    out = {"model.bert." + k: v.clone() for k, v in sd.items()}
    if extra_heads:
        out["model.cls.predictions.decoder.weight"] = torch.zeros(4, 4)
        out["model.cls.predictions.bias"] = torch.zeros(4)
    return {"state": {"model": out}, "rng": [torch.zeros(1)]}


def test_composer_checkpoint_round_trip(tmp_path):
    cfg = m2_amd.m2_bert_80m(128)
    cfg.num_hidden_layers = 2
    sd = m2_amd.seeded_state_dict(cfg, 21)
    path = os.path.join(tmp_path, "ckpt.pt")
    torch.save(_reference_style(sd), path)
    model = m2_amd.BertModel(cfg)
    missing, unexpected = m2_amd.load_reference_checkpoint(model, path)
    assert missing == []
    assert sorted(unexpected) == ["model.cls.predictions.bias", "model.cls.predictions.decoder.weight"]
    got = model.state_dict()
    assert set(got) == set(sd)
    for k in sd:
        assert torch.equal(got[k], sd[k]), k


def test_plain_and_prefixed_state_dicts_and_errors():
    cfg = m2_amd.m2_bert_80m(128)
    cfg.num_hidden_layers = 1
    sd = m2_amd.seeded_state_dict(cfg, 22)
    for obj in (sd, {"model": {"bert." + k: v for k, v in sd.items()}}, {"state_dict": sd}):
        model = m2_amd.BertModel(cfg)
        missing, unexpected = m2_amd.load_reference_checkpoint(model, obj)
        assert missing == [] and unexpected == []
        assert torch.equal(model.state_dict()["encoder.layer.0.mlp.wo.weight"], sd["encoder.layer.0.mlp.wo.weight"])
    # a checkpoint without a pooler is fine for a model with one (2 missing keys <= 5) ...
    nop = {k: v for k, v in sd.items() if not k.startswith("pooler.")}
    missing, _ = m2_amd.load_reference_checkpoint(m2_amd.BertModel(cfg), nop)
    assert sorted(missing) == ["pooler.dense.bias", "pooler.dense.weight"]
    # ... one that lacks a whole mixer is not
    broken = {k: v for k, v in sd.items() if ".attention." not in k}
    with pytest.raises(RuntimeError, match="not in the checkpoint"):
        m2_amd.load_reference_checkpoint(m2_amd.BertModel(cfg), broken)
    # wrong shape: clear message
    bad = dict(sd)
    bad["encoder.layer.0.mlp.wo.weight"] = torch.zeros(4, 192, 100)
    with pytest.raises(ValueError, match="expects"):
        m2_amd.load_reference_checkpoint(m2_amd.BertModel(cfg), bad)
    with pytest.raises(ValueError, match="not a state dict"):
        ck.unwrap_state_dict({"a": 1})


@pytest.mark.parametrize("tile_z", [False, True])
def test_context_extension_128_to_512(tile_z):
    short = m2_amd.m2_bert_80m(128)
    short.num_hidden_layers = 1
    long = m2_amd.m2_bert_80m(512)
    long.num_hidden_layers = 1
    sd = m2_amd.seeded_state_dict(short, 23)
    model = m2_amd.BertModel(long)
    fresh = {k: v.clone() for k, v in model.state_dict().items()}
    with pytest.raises(ValueError, match="extend_to"):
        m2_amd.load_reference_checkpoint(m2_amd.BertModel(long), sd)
    missing, unexpected = m2_amd.load_reference_checkpoint(model, _reference_style(sd), extend_to=512,
                                                           tile_pos_emb_z=tile_z, max_missing=16)
    got = model.state_dict()
    pe = got["embeddings.position_embeddings.weight"]
    assert pe.shape[0] == 512
    for r in range(4):
        assert torch.equal(pe[128 * r:128 * (r + 1)], sd["embeddings.position_embeddings.weight"])
    p = "encoder.layer.0.attention.filter_fn."
    assert torch.equal(got["embeddings.position_ids"], torch.arange(512)[None])
    assert torch.equal(got[p + "pos_emb.t"], fresh[p + "pos_emb.t"])             # the long model's own time axis
    if tile_z:
        assert torch.equal(got[p + "pos_emb.z"], sd[p + "pos_emb.z"].repeat(1, 4, 1))
        assert p + "pos_emb.z" not in missing
    else:
        assert torch.equal(got[p + "pos_emb.z"], fresh[p + "pos_emb.z"])
        assert p + "pos_emb.z" in missing
    assert torch.equal(got[p + "implicit_filter.0.weight"], sd[p + "implicit_filter.0.weight"])
    assert "embeddings.position_ids" in missing and p + "pos_emb.t" in missing


def test_context_extension_reference_mode_writes_the_old_table_into_slots_of_a_zero_tensor():
    """mode="reference": `z_new = zeros(new_len); for k in range(2, R): z_new[(k-1) L_old : k L_old] = z_old`
    (bert/src/bert_layers.py:1141-1151) -- slot 0 stays zero, slots 1 .. R - 2 hold copies, the rest stays zero.
    Built here from that formula for the reference's own cases 8192 -> 32768 (R = 5) and 128 -> 2048 (R = 17),
    and for a length the reference has no entry for (every slot but the first)."""
    for old, new, R in ((8192, 32768, 5), (128, 2048, 17), (128, 1024, 17), (256, 1024, None)):
        z_old = torch.randn(1, old, 5, generator=torch.Generator().manual_seed(old))
        sd = {"encoder.layer.0.attention.filter_fn.pos_emb.z": z_old,
              "encoder.layer.0.attention.filter_fn.pos_emb.t": torch.zeros(1, old, 1),
              "embeddings.position_embeddings.weight": torch.randn(old, 8),
              "embeddings.position_ids": torch.arange(old)[None]}
        out = m2_amd.extend_context(sd, new, mode="reference")
        want = torch.zeros(1, new, 5)
        ks = range(2, R) if R is not None else range(2, new // old + 1)
        for k in ks:
            if k * old <= new:
                want[:, (k - 1) * old:k * old, :] = z_old
        got = out["encoder.layer.0.attention.filter_fn.pos_emb.z"]
        assert torch.equal(got, want), (old, new)
        assert not got[:, :old].any() and torch.equal(got[:, old:2 * old], z_old)
        assert "encoder.layer.0.attention.filter_fn.pos_emb.t" not in out and "embeddings.position_ids" not in out
        assert out["embeddings.position_embeddings.weight"].shape[0] == new
    with pytest.raises(ValueError, match="unknown"):
        m2_amd.extend_context(sd, 1024, mode="zeros")
    # through the loader: the model's z becomes the zero-slotted table
    short = m2_amd.m2_bert_80m(128)
    short.num_hidden_layers = 1
    long = m2_amd.m2_bert_80m(512)
    long.num_hidden_layers = 1
    sd = m2_amd.seeded_state_dict(short, 29)
    model = m2_amd.BertModel(long)
    m2_amd.load_reference_checkpoint(model, sd, extend_to=512, z_mode="reference", max_missing=16)
    z = model.state_dict()["encoder.layer.0.attention.filter_fn2.pos_emb.z"]
    zo = sd["encoder.layer.0.attention.filter_fn2.pos_emb.z"]
    assert not z[:, :128].any() and all(torch.equal(z[:, 128 * s:128 * (s + 1)], zo) for s in (1, 2, 3))


def test_filter_submodules_compute_the_reference_expressions():
    """Sin, ExponentialModulation and the implicit-filter Sequential evaluate on their own (plain torch ops), so that a
    caller doing `filter_fn.implicit_filter(z)` and `filter_fn.modulation(t, h)` gets the filter the kernel produces."""
    from oracle import m2_oracle as O
    cfg = m2_amd.m2_bert_80m(64)
    cfg.hidden_size = 64
    sd = m2_amd.seeded_state_dict(cfg, 3, std=0.2, what="mixer")
    fn = m2_amd.HyenaFilter(64, emb_dim=5, order=128, seq_len=64, bidirectional=True, w=10)
    fn.load_state_dict({k[len("filter_fn."):]: v for k, v in sd.items() if k.startswith("filter_fn.")})
    z, t = fn.pos_emb(64)
    h = fn.modulation(t, fn.implicit_filter(z))
    hr = fn.modulation(t, fn.implicit_filter_rev(z))
    assert torch.allclose(h, O.hyena_filter_taps(sd, "filter_fn.", 64, rev=False), atol=1e-6)
    assert torch.allclose(hr, O.hyena_filter_taps(sd, "filter_fn.", 64, rev=True), atol=1e-6)
    assert fn.implicit_filter[1] is fn.implicit_filter[3] is fn.implicit_filter_rev[5]      # one shared Sin
