"""The C-ABI library loads on a machine without a GPU and exports every symbol include/m2_amd.h
declares; argument validation that happens before any launch is exercised (no compute calls)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "m2_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(m2_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for s in ("m2_version", "m2_last_error", "m2_hyena_filter_fwd", "m2_filter_spectrum_fwd", "m2_mixer_core_fwd",
              "m2_fftconv_fwd", "m2_blockdiag_glu_fwd", "m2_blockdiag_linear_fwd", "m2_layernorm_fwd"):
        assert s in syms


def test_library_exports_every_declared_symbol():
    from m2_amd import _lib
    for s in declared_symbols():
        assert hasattr(_lib.lib, s), f"{s} is declared in include/m2_amd.h but not exported"
    assert sorted(_lib.EXPORTS) == declared_symbols()
    assert _lib.lib.m2_version() == 100


def test_size_queries_and_argument_checks_without_gpu():
    from m2_amd import _lib
    lib = _lib.lib
    assert lib.m2_fftconv_supported_seqlen(128) == 1
    assert lib.m2_fftconv_supported_seqlen(8192) == 1
    assert lib.m2_fftconv_supported_seqlen(32768) == 1
    assert lib.m2_fftconv_supported_seqlen(16384) == 1
    assert lib.m2_fftconv_supported_seqlen(64) == 0 and lib.m2_fftconv_supported_seqlen(65536) == 0
    assert lib.m2_fftconv_supported_seqlen(65536) == 0
    assert lib.m2_fftconv_supported_seqlen(64) == 0
    assert lib.m2_fftconv_supported_seqlen(100) == 0
    assert lib.m2_filter_spectrum_bytes(768, 8192) == 768 * 8192 * 16
    assert lib.m2_hyena_filter_workspace_bytes(2, 8192, 768, 128) == (2 * 2 * 8192 * 128 * 4 + 2 * 2 * 2 * 3 * 128 * 128 * 2
                                                                      + 2 * 2 * 2 * 768 * 128 * 2)
    # null pointers and unsupported sizes are refused before anything is launched
    assert lib.m2_mixer_core_fwd(None, None, None, None, None, None, None, 1, 128, 64, 0, None) == -1
    assert b"null" in lib.m2_last_error()
    one = ctypes.c_void_p(16)
    assert lib.m2_mixer_core_fwd(one, None, None, one, one, one, one, 1, 100, 64, 0, None) == -2
    assert b"L=100" in lib.m2_last_error()
    assert lib.m2_mixer_core_fwd(one, None, None, one, one, one, one, 1, 128, 64, 7, None) == -1
    assert lib.m2_blockdiag_glu_fwd(one, one, one, 8, 768, 3072, 3, None) == -2
    assert lib.m2_blockdiag_linear_fwd(one, one, None, None, one, 8, 100, 64, 4, 1, None) == -2
    assert lib.m2_layernorm_fwd(one, one, one, 1e-12, None, None, None, 4, 100, None) == -2
    # the MLPs of a batch of mixers are one grid dimension: 16384 mixers with two filters each would be 65536 of them
    assert lib.m2_mixer_filters_fwd(one, None, 16384, 2, 128, 768, 128, 5, 1.0, 0.0, one, one, None) == -1
    assert b"65535" in lib.m2_last_error()
    assert lib.m2_mixer_filters_fwd(one, None, 4, 3, 128, 768, 128, 5, 1.0, 0.0, one, one, None) == -1
    with pytest.raises(RuntimeError):
        _lib.check(-2)


def test_modules_refuse_cpu_tensors():
    """There is no CPU fallback: the product modules raise on CPU input instead of computing."""
    import torch
    import m2_amd
    mix = m2_amd.MonarchMixerSequenceMixing(64, l_max=128, bidirectional=True, hyena_emb_dim=5,
                                            hyena_filter_order=128, residual_long_conv=True)
    with pytest.raises(RuntimeError):
        mix(torch.randn(1, 128, 64))
    lin = m2_amd.BlockdiagLinear(64, 128, nblocks=4)
    with pytest.raises(RuntimeError):
        lin(torch.randn(2, 64))
    with pytest.raises(RuntimeError):
        m2_amd.ops.layernorm(torch.randn(4, 64), torch.ones(64), torch.zeros(64), 1e-12)


def test_state_dict_names_match_the_reference_layout():
    """Key names as read from the reference sources (bert/src/bert_layers.py, bert/src/mm/*.py)."""
    import m2_amd
    cfg = m2_amd.m2_bert_80m(128)
    cfg.num_hidden_layers = 1
    keys = set(m2_amd.BertModel(cfg).state_dict().keys())
    p = "encoder.layer.0."
    expect = {"embeddings.word_embeddings.weight", "embeddings.position_embeddings.weight",
              "embeddings.token_type_embeddings.weight", "embeddings.LayerNorm.weight", "embeddings.LayerNorm.bias",
              "embeddings.position_ids", "pooler.dense.weight", "pooler.dense.bias",
              p + "attention.in_linear.weight", p + "attention.in_linear.bias", p + "attention.out_linear.weight",
              p + "attention.out_linear.bias", p + "attention.short_filter.weight", p + "attention.short_filter.bias",
              p + "mlp.gated_layers.weight", p + "mlp.wo.weight", p + "mlp.wo.bias", p + "mlp.layernorm.weight",
              p + "mlp.layernorm.bias"}
    for fn in ("filter_fn.", "filter_fn2."):
        q = p + "attention." + fn
        expect |= {q + "bias", q + "pos_emb.z", q + "pos_emb.t", q + "modulation.deltas"}
        for mlp in ("implicit_filter.", "implicit_filter_rev."):
            expect |= {q + mlp + f"{i}.weight" for i in (0, 2, 4, 6)}
            expect |= {q + mlp + f"{i}.bias" for i in (0, 2, 4)}
            expect |= {q + mlp + f"{i}.freq" for i in (1, 3, 5)}
    assert keys == expect
    assert set(m2_amd.BertModel(cfg, add_pooling_layer=False).state_dict().keys()) == \
        expect - {"pooler.dense.weight", "pooler.dense.bias"}
    # hyena_training_additions adds the mixer's own LayerNorm (bert/src/mm/monarch_mixer_sequence_mixer.py:84-87)
    cfg2 = m2_amd.m2_bert_80m(128)
    cfg2.num_hidden_layers = 1
    cfg2.hyena_training_additions = True
    keys2 = set(m2_amd.BertModel(cfg2).state_dict().keys())
    assert keys2 == expect | {p + "attention.layernorm.weight", p + "attention.layernorm.bias"}
    assert set(m2_amd.seeded_state_dict(cfg2, 1).keys()) == keys2
    m = m2_amd.BertModel(cfg)
    sd = m.state_dict()
    assert tuple(sd[p + "attention.short_filter.weight"].shape) == (3 * 768, 1, 3)
    assert tuple(sd[p + "mlp.gated_layers.weight"].shape) == (4, 1536, 192)
    assert tuple(sd[p + "mlp.wo.weight"].shape) == (4, 192, 768)
    assert tuple(sd[p + "attention.filter_fn.pos_emb.z"].shape) == (1, 128, 5)
    # buffers vs parameters as the reference registers them (lr == 0.0 -> buffer)
    params = {n for n, _ in m.named_parameters()}
    assert p + "attention.filter_fn.pos_emb.z" in params
    assert p + "attention.filter_fn.pos_emb.t" not in params
    assert p + "attention.filter_fn.modulation.deltas" not in params


def test_static_scratch_covers_what_its_documentation_promises():
    """m2_hyena_filter_fwd_static: both filters of a mixer up to L = 8192, or one filter up to L = 16384, for d <= 1536."""
    from m2_amd._lib import M2_HYENA_FILTER_STATIC_SCRATCH_BYTES, lib
    import re
    header = open(os.path.join(ROOT, "include", "m2_amd.h")).read()
    m = re.search(r"#define M2_HYENA_FILTER_STATIC_SCRATCH_BYTES \((\d+)u << (\d+)\)", header)
    assert m and (int(m.group(1)) << int(m.group(2))) == M2_HYENA_FILTER_STATIC_SCRATCH_BYTES
    for nf, L in ((2, 8192), (1, 16384), (2, 128), (1, 32)):
        for d in (768, 1536):
            assert lib.m2_hyena_filter_workspace_bytes(nf, L, d, 128) <= M2_HYENA_FILTER_STATIC_SCRATCH_BYTES, (nf, L, d)
    assert lib.m2_hyena_filter_workspace_bytes(2, 16384, 768, 128) > M2_HYENA_FILTER_STATIC_SCRATCH_BYTES
