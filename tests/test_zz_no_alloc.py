"""The allocation-free filter-generation entry point (m2_hyena_filter_fwd_static, scratch in a device array of the
library) against m2_hyena_filter_fwd (caller workspace), through the C ABI: two calls in a row, the second with a
shorter sequence, must give bit-identical taps; sizes beyond the static array are refused."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _filters(cfg, seed, gpu):
    import m2_amd
    sd = m2_amd.seeded_state_dict(cfg, seed, std=0.1, what="mixer")
    mix = m2_amd.MonarchMixerSequenceMixing(cfg.hidden_size, l_max=cfg.long_conv_l_max, bidirectional=True, hyena_emb_dim=5,
                                            hyena_filter_order=128, residual_long_conv=True, hyena_w=10)
    mix.load_state_dict(sd)
    mix = mix.to(gpu)
    return [mix.filter_fn.kernel_params("both"), mix.filter_fn2.kernel_params("both")], mix


def test_static_scratch_entry_point_matches_workspace_entry_point(gpu):
    import m2_amd
    from m2_amd import ops
    from m2_amd._lib import M2_HYENA_FILTER_STATIC_SCRATCH_BYTES, lib
    d = 768                                       # the benchmark's own width: both filters of a mixer at L = 8192
    cfg = m2_amd.m2_bert_80m(8192)
    filters, _ = _filters(cfg, 3, gpu)
    for L in (8192, 1024):                       # the second call is shorter: stale scratch beyond it must not matter
        assert lib.m2_hyena_filter_workspace_bytes(2, L, d, 128) <= M2_HYENA_FILTER_STATIC_SCRATCH_BYTES
        want = ops.hyena_filter_taps(filters, L, d, 128, 5)
        out = torch.full((2, d, 2 * L), float("nan"), device=gpu)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        stats_before = torch.cuda.memory_stats()
        got = ops.hyena_filter_taps(filters, L, d, 128, 5, static_scratch=True, out=out)
        torch.cuda.synchronize()
        stats_after = torch.cuda.memory_stats()
        assert torch.cuda.mem_get_info()[0] == free_before           # no device allocation behind the call ...
        for key in ("allocation.all.allocated", "allocated_bytes.all.allocated", "segment.all.allocated"):
            assert stats_after[key] == stats_before[key], key         # ... and none served from torch's cache either
        assert got is out and torch.equal(got, want), L
    # against the oracle as well (fp64), the shorter length
    from conftest import rel_err
    from oracle import m2_oracle as O
    sd = m2_amd.seeded_state_dict(cfg, 3, std=0.1, what="mixer")
    sd64 = O.cast_state_dict(sd, torch.float64)
    kf = O.hyena_filter_taps(sd64, "filter_fn.", 1024, rev=False)[0].T
    kr = O.hyena_filter_taps(sd64, "filter_fn.", 1024, rev=True)[0].T
    assert rel_err(got[0], O.bidirectional_kernel(kf, kr, 1024))[0] < 2e-5
    # two filters of 16384 positions do not fit the static array: refused, nothing launched
    cfg_long = m2_amd.m2_bert_80m(16384)
    long_filters, _ = _filters(cfg_long, 3, gpu)
    with pytest.raises(RuntimeError, match="static array"):
        ops.hyena_filter_taps(long_filters, 16384, d, 128, 5, static_scratch=True)
    one = ops.hyena_filter_taps(long_filters[:1], 16384, d, 128, 5, static_scratch=True)      # one filter just fits
    assert torch.equal(one, ops.hyena_filter_taps(long_filters[:1], 16384, d, 128, 5))
