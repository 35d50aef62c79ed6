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
