"""GPU parity of each C-ABI entry point against the CPU oracle (same seeded inputs).

Tolerances: fp32 long-convolution path 1e-4 relative (max-abs error over max-abs reference);
bf16 GEMM paths 2e-2 relative.
"""
import math

import pytest
import torch

from conftest import rel_err

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-4
TOL_BF16 = 2e-2


def _cfg(L, d=128, layers=1, I=None):
    import m2_amd
    cfg = m2_amd.M2BertConfig(hidden_size=d, intermediate_size=I or 4 * d, num_hidden_layers=layers).with_seq_len(L)
    return cfg


@pytest.mark.parametrize("L", [128, 256, 1024])
@pytest.mark.parametrize("std", [0.02, 0.3])
def test_hyena_filter_taps(gpu, L, std):
    """K1 vs oracle.hyena_filter_taps; std=0.3 drives the sin arguments far outside [-pi, pi]."""
    import m2_amd
    from oracle import m2_oracle as O
    cfg = _cfg(L, d=192)
    sd = m2_amd.seeded_state_dict(cfg, 7, std=std, what="mixer")
    mix = m2_amd.MonarchMixerSequenceMixing(cfg.hidden_size, l_max=L, bidirectional=True, hyena_emb_dim=5,
                                            hyena_filter_order=128, residual_long_conv=True, hyena_w=10)
    mix.load_state_dict(sd)
    mix = mix.to(gpu)
    sd64 = O.cast_state_dict(sd, torch.float64)
    for fn, name in ((mix.filter_fn, "filter_fn."), (mix.filter_fn2, "filter_fn2.")):
        taps = fn.bidirectional_taps(L).cpu()
        kf = O.hyena_filter_taps(sd64, name, L, rev=False)[0].T
        kr = O.hyena_filter_taps(sd64, name, L, rev=True)[0].T
        ref = O.bidirectional_kernel(kf, kr, L)
        e, _ = rel_err(taps, ref)
        # yardstick: how far the fp32 CPU oracle itself is from fp64 (sin(10 x) amplifies rounding)
        ref32 = O.bidirectional_kernel(O.hyena_filter_taps(sd, name, L, rev=False)[0].T,
                                       O.hyena_filter_taps(sd, name, L, rev=True)[0].T, L)
        e32, _ = rel_err(ref32, ref)
        assert e < max(2e-5, 4 * e32), (name, e, e32)
        # reference API shapes
        h = fn.filter(L)
        assert h.shape == (1, L, cfg.hidden_size)
        assert rel_err(h.cpu(), kf.T[None])[0] < max(2e-5, 4 * e32)
        hr = fn.filter_rev(L)
        assert rel_err(hr.cpu(), kr.T[None])[0] < max(2e-5, 4 * e32)


@pytest.mark.parametrize("L,emb_dim,w,w_mod,shift", [(256, 3, 4, 2, 0.05), (256, 7, 14, 1, 0.0), (2048, 3, 10, 2, 0.05),
                                                     (2048, 7, 1, 1, -0.02)])
def test_hyena_filter_settings_off_the_default(gpu, L, emb_dim, w, w_mod, shift):
    """The filter with the other settings its constructor takes (bert/src/mm/hyena_utils.py:115-166): emb_dim 3 and 7
    (one and three frequency bands), the Sin frequency w, the multiplier w_mod and a modulation shift -- taps of
    HyenaFilter.filter / filter_rev against the fp64 oracle (fp32 yardstick as above), and the spectra of the batched
    call (one-kernel route at L = 256, fused hidden + projection at L = 2048) against the two-step route."""
    import m2_amd
    from m2_amd import ops
    from oracle import m2_oracle as O
    d = 192
    torch.manual_seed(L + emb_dim)
    fn = m2_amd.HyenaFilter(d, emb_dim=emb_dim, order=128, seq_len=L, bidirectional=True, w=w, w_mod=w_mod, shift=shift)
    with torch.no_grad():
        for prm in fn.parameters():
            if prm.dim() == 2:
                prm.normal_(0.0, 0.05)
    fn = fn.to(gpu)
    sd = {"f." + k: v.detach().cpu() for k, v in fn.state_dict().items()}
    sd64 = O.cast_state_dict(sd, torch.float64)
    taps = fn.bidirectional_taps(L)
    for rev, got in ((False, fn.filter(L)), (True, fn.filter_rev(L))):
        ref = O.hyena_filter_taps(sd64, "f.", L, rev=rev, w_mod=w_mod, shift=shift)
        e32 = rel_err(O.hyena_filter_taps(sd, "f.", L, rev=rev, w_mod=w_mod, shift=shift), ref)[0]
        assert rel_err(got.cpu(), ref)[0] < max(2e-5, 4 * e32), (rev, e32)
    params = fn.kernel_params("both")
    skip = fn.bias.detach().float().contiguous()
    table = ops.FilterTable([[params]], [[skip]], L, d, 128, emb_dim)
    spec = ops.mixer_filter_spectra(table, w_mod=float(w_mod), shift=float(shift))[0]
    two_step = ops.filter_spectrum(taps, None, skip, None)
    assert rel_err(spec, two_step)[0] < TOL_F32


@pytest.mark.parametrize("L", [128, 256, 512, 1024, 2048])
@pytest.mark.parametrize("bidirectional,residual", [(True, True), (False, True), (True, False)])
def test_mixer_filter_spectra_batched(gpu, L, bidirectional, residual):
    """m2_mixer_filters_fwd (all filters of three mixers -> spectra in one call; for L <= 512 projection, decay and
    transform are one kernel and the taps never exist) against the fp64 oracle's taps pushed through the stand-alone
    spectrum kernel, with the two-step path (m2_hyena_filter_fwd + m2_filter_spectrum_fwd, itself pinned against the
    oracle above) as the yardstick; also sub-ranges of the table."""
    import m2_amd
    from m2_amd import ops
    from oracle import m2_oracle as O
    d, nm = 192, 3
    mixers, sds = [], []
    for i in range(nm):
        cfg = _cfg(L, d=d)
        cfg.bidirectional, cfg.residual_long_conv = bidirectional, residual
        sd = m2_amd.seeded_state_dict(cfg, 70 + i, std=0.1, what="mixer")
        mix = m2_amd.MonarchMixerSequenceMixing(d, l_max=L, bidirectional=bidirectional, hyena_emb_dim=5,
                                                hyena_filter_order=128, residual_long_conv=residual, hyena_w=10)
        mix.load_state_dict(sd)
        mixers.append(mix.to(gpu))
        sds.append(sd)
    entries = [m.filter_table_entry() for m in mixers]
    table = ops.FilterTable([e[0] for e in entries], [e[1] for e in entries], L, d, 128, 5)
    got = ops.mixer_filter_spectra(table)
    assert got.shape == (nm, ops.lib.m2_filter_spectrum_bytes(d, L) // 4)
    names = ["filter_fn."] + (["filter_fn2."] if residual else [])
    for i, (mix, sd) in enumerate(zip(mixers, sds)):
        sd64 = O.cast_state_dict(sd, torch.float64)
        taps64, taps_gpu = [], []
        for name in names:
            kf = O.hyena_filter_taps(sd64, name, L, rev=False)[0].T
            kr = O.hyena_filter_taps(sd64, name, L, rev=True)[0].T if bidirectional else torch.zeros_like(kf)
            taps64.append(O.bidirectional_kernel(kf, kr, L).float().to(gpu).contiguous())
        fns = [mix.filter_fn] + ([mix.filter_fn2] if residual else [])
        taps_gpu = [f.bidirectional_taps(L) for f in fns]
        D = [f.bias.detach().float() for f in fns]
        want = ops.filter_spectrum(taps64[0], taps64[1] if residual else None, D[0], D[1] if residual else None)
        two_step = ops.filter_spectrum(taps_gpu[0], taps_gpu[1] if residual else None, D[0], D[1] if residual else None)
        e, e2 = rel_err(got[i], want)
        y, _ = rel_err(two_step, want)
        assert e < max(2e-5, 3 * y), (i, e, e2, y)
    # a sub-range of the table, into a caller's buffer
    part = torch.full((2, got.shape[1]), float("nan"), device=gpu)
    assert ops.mixer_filter_spectra(table, first=1, count=2, out=part) is part
    assert torch.equal(part, got[1:])


@pytest.mark.parametrize("L", [8192, 32768])
def test_hyena_filter_taps_at_benchmark_lengths(gpu, L):
    """Filter taps at the benchmark's own sizes (d = 768, L = 8192 and 32768: the 64-position hidden tiles and the
    256-position projection runs) against the fp64 oracle, with the fp32 CPU oracle's own distance from fp64 as the
    yardstick, both filters of a mixer, N(0, 0.02) weights as in the benchmark."""
    import m2_amd
    from oracle import m2_oracle as O
    cfg = m2_amd.m2_bert_80m(L)
    sd = m2_amd.seeded_state_dict(cfg, 1234, what="mixer")
    mix = m2_amd.MonarchMixerSequenceMixing(768, l_max=L, bidirectional=True, hyena_emb_dim=5, hyena_filter_order=128,
                                            residual_long_conv=True, hyena_w=10)
    mix.load_state_dict(sd)
    mix = mix.to(gpu)
    sd64 = O.cast_state_dict(sd, torch.float64)
    for fn, name in ((mix.filter_fn, "filter_fn."), (mix.filter_fn2, "filter_fn2.")):
        taps = fn.bidirectional_taps(L).cpu()
        ref = O.bidirectional_kernel(O.hyena_filter_taps(sd64, name, L, rev=False)[0].T,
                                     O.hyena_filter_taps(sd64, name, L, rev=True)[0].T, L)
        ref32 = O.bidirectional_kernel(O.hyena_filter_taps(sd, name, L, rev=False)[0].T,
                                       O.hyena_filter_taps(sd, name, L, rev=True)[0].T, L)
        e32, _ = rel_err(ref32, ref)
        e, e2 = rel_err(taps, ref)
        print(f"taps L={L} {name}: max-rel {e:.2e} L2-rel {e2:.2e} (fp32 CPU oracle vs fp64: {e32:.2e})")
        assert e < max(2e-5, 4 * e32), (name, e, e32)


@pytest.mark.parametrize("L", [128, 256, 512, 1024, 2048, 4096, 8192, 16384, 32768])
@pytest.mark.parametrize("act", ["f32", "bf16"])
def test_mixer_core(gpu, L, act):
    """K1c + K2 vs the oracle's short conv / gating / two fftconvs, every FFT plan."""
    import m2_amd
    from m2_amd import ops
    from oracle import m2_oracle as O
    d, B = (64, 3) if L <= 16384 else (16, 2)
    g = torch.Generator().manual_seed(100 + L)
    dt = torch.float32 if act == "f32" else torch.bfloat16
    xproj = torch.randn(3 * d, B, L, generator=g).to(dt)
    u = torch.randn(d, B, L, generator=g)
    sw = torch.randn(3 * d, 3, generator=g) * 0.5
    sb = torch.randn(3 * d, generator=g) * 0.1
    t = torch.linspace(0, 1, 2 * L)
    taps = [torch.randn(d, 2 * L, generator=g) * torch.exp(-4 * torch.minimum(t, 1 - t)) for _ in range(2)]
    D = [torch.randn(d, generator=g) for _ in range(2)]
    spec = ops.filter_spectrum(taps[0].to(gpu), taps[1].to(gpu), D[0].to(gpu), D[1].to(gpu))
    pb = torch.randn(3 * d, generator=g) * 0.3
    y = ops.mixer_core(xproj.to(gpu), u.to(gpu), sw.to(gpu), sb.to(gpu), spec, B, L, d, proj_bias=pb.to(gpu))
    # oracle in float64 on the same (possibly bf16-rounded) inputs
    x64 = (xproj.double() + pb.double()[:, None, None]).permute(1, 0, 2)      # (B, 3d, L)
    uc = O.short_conv(x64, sw.double().view(3 * d, 1, 3), sb.double())
    x1, x2, v = uc.split(d, dim=1)
    y1 = O.fftconv(v * x1, taps[0].double(), D[0].double()[None, :, None])
    y2 = O.fftconv(u.double().permute(1, 0, 2), taps[1].double(), D[1].double()[None, :, None])
    ref = (y1 * x2 + y2).permute(1, 0, 2)
    e, e2 = rel_err(y.float(), ref)
    tol = TOL_F32 if act == "f32" else 6e-3        # bf16 output rounding is 2^-9
    assert e < tol, (L, act, e, e2)


def test_plain_fftconv_module_api(gpu):
    """HyenaFilter.forward(x, L, k_fwd, k_rev, bias) keeps the reference call shape."""
    import m2_amd
    from oracle import m2_oracle as O
    L, d, B = 256, 64, 2
    g = torch.Generator().manual_seed(5)
    fn = m2_amd.HyenaFilter(d, emb_dim=5, order=128, seq_len=L, bidirectional=True, w=10).to(gpu)
    x = torch.randn(B, d, L, generator=g)
    kf = torch.randn(d, L, generator=g) * 0.1
    kr = torch.randn(d, L, generator=g) * 0.1
    bias = torch.randn(d, generator=g)
    y = fn(x.to(gpu), L, k_fwd=kf.to(gpu), k_rev=kr.to(gpu), bias=bias.to(gpu)[None, :, None])
    ref = O.hyena_filter_forward(x.double(), L, kf.double(), kr.double(), bias.double()[None, :, None])
    assert rel_err(y, ref)[0] < TOL_F32


@pytest.mark.parametrize("M,d,I", [(256, 768, 3072), (200, 256, 512), (4096, 1536, 6144), (300, 512, 2048),
                                   (300, 1024, 4096), (130, 256, 768), (1100, 768, 3072),
                                   # block sizes off the 64-wide tile grid: the 960-wide model of the reference
                                   # (bert/yamls/pretrain/monarch-mixer-pretrain-960dim-parameter-matched.yaml: 240-wide
                                   # blocks), the 1792-wide one, and small multiples of 8
                                   (4096, 960, 3840), (333, 960, 3840), (300, 1792, 7168), (200, 32, 64), (130, 96, 352),
                                   (70, 544, 1120)])
def test_blockdiag_glu_and_linear(gpu, M, d, I):
    """K3 vs oracle.blockdiag_* on bf16-rounded operands (fp64 reference)."""
    from m2_amd import ops
    from oracle import m2_oracle as O
    nb = 4
    g = torch.Generator().manual_seed(11)
    x = torch.randn(M, d, generator=g).bfloat16()
    wg = (torch.randn(nb, 2 * I // nb, d // nb, generator=g) * 0.05).bfloat16()
    wo = (torch.randn(nb, d // nb, I // nb, generator=g) * 0.05).bfloat16()
    bias = torch.randn(d, generator=g)
    got = ops.blockdiag_glu(x.to(gpu), wg.to(gpu))
    h = O.blockdiag_multiply(x.double(), wg.double())
    ref = torch.nn.functional.gelu(h[:, :I]) * h[:, I:]
    assert rel_err(got.float(), ref)[0] < TOL_BF16
    a = ref.bfloat16()
    got2 = ops.blockdiag_linear(a.to(gpu), wo.to(gpu), bias.to(gpu), x.to(gpu), out_dtype=torch.float32)
    ref2 = O.blockdiag_multiply(a.double(), wo.double()) + bias.double() + x.double()
    assert rel_err(got2, ref2)[0] < 1e-3        # fp32 accumulate of exact bf16 products
    got3 = ops.blockdiag_linear(a.to(gpu), wo.to(gpu), None, None, out_dtype=torch.bfloat16)
    assert rel_err(got3.float(), O.blockdiag_multiply(a.double(), wo.double()))[0] < TOL_BF16


def test_blockdiag_linear_full_size_ragged(gpu):
    """wo at the benchmark's M with a ragged last tile (the shape that selects the 128-row tiles, two workgroups
    per compute unit), bias + bf16 residual, fp32 and bf16 outputs; fp32 oracle on the CPU."""
    from m2_amd import ops
    from oracle import m2_oracle as O
    M, d, I, nb = 32768 - 70, 768, 3072, 4
    g = torch.Generator().manual_seed(21)
    a = torch.randn(M, I, generator=g).bfloat16()
    wo = (torch.randn(nb, d // nb, I // nb, generator=g) * 0.05).bfloat16()
    bias = torch.randn(d, generator=g)
    res = torch.randn(M, d, generator=g).bfloat16()
    ref = O.blockdiag_multiply(a.float(), wo.float()) + bias + res.float()
    got = ops.blockdiag_linear(a.to(gpu), wo.to(gpu), bias.to(gpu), res.to(gpu), out_dtype=torch.float32)
    assert rel_err(got, ref)[0] < 1e-3
    got16 = ops.blockdiag_linear(a.to(gpu), wo.to(gpu), bias.to(gpu), res.to(gpu), out_dtype=torch.bfloat16)
    assert rel_err(got16.float(), ref)[0] < TOL_BF16


@pytest.mark.parametrize("M,d", [(300, 768), (64, 1536), (1000, 128)])
def test_layernorm_three_outputs(gpu, M, d):
    from m2_amd import ops
    g = torch.Generator().manual_seed(3)
    x = torch.randn(M, d, generator=g) * 3 + 1
    gamma = torch.randn(d, generator=g)
    beta = torch.randn(d, generator=g)
    o32, o16, ot = ops.layernorm(x.to(gpu), gamma.to(gpu), beta.to(gpu), 1e-12, True, True, True)
    ref = torch.nn.functional.layer_norm(x.double(), (d,), gamma.double(), beta.double(), 1e-12)
    assert rel_err(o32, ref)[0] < 1e-5
    assert rel_err(ot.T, ref)[0] < 1e-5
    assert rel_err(o16.float(), ref)[0] < 6e-3
    # rows stored as bf16 (what the reference's LayerNorm receives under autocast): the same statistics in fp32 on
    # the rounded values
    x16 = x.bfloat16()
    p32, p16, pt = ops.layernorm(x16.to(gpu), gamma.to(gpu), beta.to(gpu), 1e-12, True, True, True)
    ref16 = torch.nn.functional.layer_norm(x16.double(), (d,), gamma.double(), beta.double(), 1e-12)
    assert rel_err(p32, ref16)[0] < 1e-5
    assert rel_err(pt.T, ref16)[0] < 1e-5
    assert rel_err(p16.float(), ref16)[0] < 6e-3


def test_config1_mixer_fp32(gpu):
    """BASELINE config 1: one MonarchMixerSequenceMixing layer, fp32, B=16 L=128 d=768, tol 1e-4."""
    import m2_amd
    from oracle import m2_oracle as O
    cfg = m2_amd.m2_bert_80m(128)
    sd = m2_amd.seeded_state_dict(cfg, 1234, what="mixer")
    mix = m2_amd.MonarchMixerSequenceMixing(768, l_max=128, bidirectional=True, hyena_emb_dim=5, hyena_filter_order=128,
                                            residual_long_conv=True, hyena_w=10, hyena_w_mod=1)
    mix.load_state_dict(sd)
    mix = mix.to(gpu).eval()
    u = torch.randn(16, 128, 768, generator=torch.Generator().manual_seed(1234))
    y, none = mix(u.to(gpu))
    assert none is None and y.dtype == torch.float32 and y.shape == u.shape
    ref = O.mixer_forward(sd, "", u)
    e, e2 = rel_err(y, ref)
    assert e < TOL_F32 and e2 < TOL_F32, (e, e2)


def test_input_shorter_than_l_max(gpu):
    """A model built for l_max = 1024 run on 256 positions: the filters are the first 256 rows of the positional
    embedding and of t, the transform length follows the input (bert/src/mm/hyena_utils.py:201-211,
    bert/src/mm/monarch_mixer_sequence_mixer.py:104,120-139).  The mixer alone in fp32 at 1e-4, then two encoder layers."""
    import m2_amd
    from oracle import m2_oracle as O
    cfg = m2_amd.m2_bert_80m(1024)
    cfg.num_hidden_layers = 2
    sd = m2_amd.seeded_state_dict(cfg, 31, what="mixer")
    mix = m2_amd.MonarchMixerSequenceMixing(768, l_max=1024, bidirectional=True, hyena_emb_dim=5, hyena_filter_order=128,
                                            residual_long_conv=True, hyena_w=10, hyena_w_mod=1)
    mix.load_state_dict(sd)
    mix = mix.to(gpu).eval()
    u = torch.randn(3, 256, 768, generator=torch.Generator().manual_seed(8))
    y, _ = mix(u.to(gpu))
    e, e2 = rel_err(y, O.mixer_forward(sd, "", u))
    assert y.shape == u.shape and e < TOL_F32 and e2 < TOL_F32, (e, e2)
    sd = m2_amd.seeded_state_dict(cfg, 32)
    model = m2_amd.BertModel(cfg)
    model.load_state_dict(sd)
    model = model.to(gpu).eval()
    ids = torch.randint(0, cfg.vocab_size, (3, 256), generator=torch.Generator().manual_seed(9))
    mask = torch.ones(3, 256, dtype=torch.long)
    out, _ = model(ids.to(gpu), attention_mask=mask.to(gpu))
    e, e2 = rel_err(out, O.model_forward(sd, ids, mask, cfg))
    assert out.shape == (3, 256, 768) and e < TOL_BF16 and e2 < TOL_BF16, (e, e2)


@pytest.mark.parametrize("L,B,layers", [(128, 4, 2), (1024, 2, 2), (16384, 1, 1), (32768, 1, 1)])
def test_encoder_small(gpu, L, B, layers):
    """Fused encoder schedule and the module-by-module path agree with the oracle (bf16 tolerance)."""
    import m2_amd
    from oracle import m2_oracle as O
    cfg = m2_amd.m2_bert_80m(L)
    cfg.num_hidden_layers = layers
    sd = m2_amd.seeded_state_dict(cfg, 99)
    model = m2_amd.BertModel(cfg)
    model.load_state_dict(sd)
    model = model.to(gpu).eval()
    ids = torch.randint(0, cfg.vocab_size, (B, L), generator=torch.Generator().manual_seed(5))
    mask = torch.ones(B, L, dtype=torch.long)
    out, _ = model(ids.to(gpu), attention_mask=mask.to(gpu))
    ref = O.model_forward(sd, ids, mask, cfg)
    e, e2 = rel_err(out, ref)
    assert e < TOL_BF16 and e2 < TOL_BF16, (e, e2)
    # layer-by-layer module path
    x = model.embeddings(ids.to(gpu))
    for layer in model.encoder.layer:
        x = layer(x)
    e, e2 = rel_err(x, ref)
    assert e < TOL_BF16 and e2 < TOL_BF16, (e, e2)
    # wo + LayerNorm as one kernel (an option; two kernels are the default)
    for layer in model.encoder.layer:
        layer.mlp.fuse_wo_layernorm = True
    out1, _ = model(ids.to(gpu), attention_mask=mask.to(gpu))
    e, e2 = rel_err(out1, ref)
    assert e < TOL_BF16 and e2 < TOL_BF16, (e, e2)
    # the MLP as two kernels with an fp32 sum into the LayerNorm (the default is one kernel and a bf16 sum)
    for layer in model.encoder.layer:
        layer.mlp.fuse_wo_layernorm = False
        layer.mlp.fuse_mlp = False
        layer.mlp.bf16_presum = False
    out2, _ = model(ids.to(gpu), attention_mask=mask.to(gpu))
    e, e2 = rel_err(out2, ref)
    assert e < TOL_BF16 and e2 < TOL_BF16, (e, e2)
    # one kernel, fp32 sum
    for layer in model.encoder.layer:
        layer.mlp.fuse_mlp = True
    out3, _ = model(ids.to(gpu), attention_mask=mask.to(gpu))
    e, e2 = rel_err(out3, ref)
    assert e < TOL_BF16 and e2 < TOL_BF16, (e, e2)


def test_encoder_hip_graph_replays_match_eager(gpu):
    """The captured encoder graph is replayed several times, with eager work and synchronisations in
    between and with new inputs, and every replay must equal the eager result bit for bit."""
    import m2_amd
    cfg = m2_amd.m2_bert_80m(128)
    cfg.num_hidden_layers = 3
    sd = m2_amd.seeded_state_dict(cfg, 41)
    eager = m2_amd.BertModel(cfg)
    eager.load_state_dict(sd)
    eager = eager.to(gpu).eval()
    graphed = m2_amd.BertModel(cfg, use_hip_graph=True)
    graphed.load_state_dict(sd)
    graphed = graphed.to(gpu).eval()
    gen = torch.Generator().manual_seed(9)
    for it in range(5):
        ids = torch.randint(0, cfg.vocab_size, (4, 128), generator=gen).to(gpu)
        want, _ = eager(ids)
        torch.cuda.synchronize()
        scratch = torch.randn(1024, 1024, device=gpu) @ torch.randn(1024, 1024, device=gpu)     # unrelated eager work
        got, _ = graphed(ids)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (it, (got - want).abs().max().item())
        del scratch
    # all layers, second shape -> second graph
    ids = torch.randint(0, cfg.vocab_size, (2, 128), generator=gen).to(gpu)
    want, _ = eager(ids, output_all_encoded_layers=True)
    for _ in range(2):
        got, _ = graphed(ids, output_all_encoded_layers=True)
        assert len(got) == 3 and all(torch.equal(a, b) for a, b in zip(got, want))
    assert len(graphed.encoder._graphs) == 2
    graphed.encoder.reset_graphs()
    assert len(graphed.encoder._graphs) == 0


def test_cached_filter_spectra_follow_the_weights(gpu):
    """cache_filters=True reuses the spectra and regenerates them when a filter weight changes."""
    import m2_amd
    cfg = m2_amd.m2_bert_80m(128)
    sd = m2_amd.seeded_state_dict(cfg, 3, what="mixer")
    mix = m2_amd.MonarchMixerSequenceMixing(768, l_max=128, bidirectional=True, hyena_emb_dim=5, hyena_filter_order=128,
                                            residual_long_conv=True, hyena_w=10)
    mix.load_state_dict(sd)
    mix = mix.to(gpu).eval()
    u = torch.randn(2, 128, 768, generator=torch.Generator().manual_seed(1)).to(gpu)
    y0, _ = mix(u)
    mix.cache_filters = True
    y1, _ = mix(u)
    spec_a = mix._spec_cache[1]
    y2, _ = mix(u)
    assert mix._spec_cache[1] is spec_a and torch.equal(y0, y1) and torch.equal(y1, y2)
    with torch.no_grad():
        mix.filter_fn.bias.add_(1.0)                       # the skip weight D1 is part of the spectrum
    y3, _ = mix(u)
    assert mix._spec_cache[1] is not spec_a and not torch.equal(y3, y2)
    mix.cache_filters = False
    y4, _ = mix(u)
    assert torch.equal(y3, y4)


def test_encoder_overlapped_filter_generation_matches_sequential(gpu):
    """Generating the filter spectra on a second stream (next layer's behind the mixer core, or all layers' from the
    start) must not change a bit, eagerly or as a captured graph."""
    import m2_amd
    cfg = m2_amd.m2_bert_80m(256)
    cfg.num_hidden_layers = 3
    model = m2_amd.BertModel(cfg)
    model.load_state_dict(m2_amd.seeded_state_dict(cfg, 43))
    model = model.to(gpu).eval()
    ids = torch.randint(0, cfg.vocab_size, (2, 256), generator=torch.Generator().manual_seed(10)).to(gpu)
    for batch in (True, False):                     # all layers' filters by batched calls / layer by layer
        model.encoder.batch_filters = batch
        model.encoder.overlap_filters = False          # on the main stream
        want, _ = model(ids)
        for mode in (True, "upfront", None):            # None picks "upfront" at this length
            model.encoder.overlap_filters = mode
            for _ in range(3):
                got, _ = model(ids)
                torch.cuda.synchronize()
                assert torch.equal(got, want), (batch, mode)
        if batch:
            batched = want
    # at this length the batched path runs projection + transform as one kernel: same numbers to fp32 rounding
    assert rel_err(batched, want)[0] < 1e-4
    model.encoder.batch_filters = True
    # and inside a captured graph (the side stream becomes a parallel branch), replayed with eager work between
    graphed = m2_amd.BertModel(cfg, use_hip_graph=True)
    graphed.load_state_dict(m2_amd.seeded_state_dict(cfg, 43))
    graphed = graphed.to(gpu).eval()
    graphed.encoder.overlap_filters = "upfront"
    for it in range(4):
        ids2 = torch.randint(0, cfg.vocab_size, (2, 256), generator=torch.Generator().manual_seed(20 + it)).to(gpu)
        model.encoder.overlap_filters = False
        want2, _ = model(ids2)
        got2, _ = graphed(ids2)
        torch.cuda.synchronize()
        assert torch.equal(got2, want2), it


def test_embed_layernorm_matches_oracle(gpu):
    """Gather + sum + LayerNorm kernel against the oracle's BertEmbeddings, with and without explicit
    token-type / position ids, and against the unfused path (sum by torch ops, then the LayerNorm kernel)."""
    import m2_amd
    from oracle import m2_oracle as orc
    cfg = m2_amd.m2_bert_80m(128)
    sd = m2_amd.seeded_state_dict(cfg, 17)
    emb = m2_amd.BertModel(cfg).embeddings
    emb.load_state_dict({k[len("embeddings."):]: v for k, v in sd.items() if k.startswith("embeddings.")})
    emb = emb.to(gpu).eval()
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, cfg.vocab_size, (3, 100), generator=g)
    tt = torch.randint(0, cfg.type_vocab_size, (3, 100), generator=g)
    for use_tt in (False, True):
        want = orc.embeddings_forward({k: v.double() for k, v in sd.items()}, "embeddings.", ids, cfg,
                                      token_type_ids=tt if use_tt else None)
        o32, o16, oT = emb.forward_forms(ids.to(gpu), tt.to(gpu) if use_tt else None)
        e, e2 = rel_err(o32, want)
        assert e < 1e-5 and e2 < 1e-5, (use_tt, e, e2)
        assert torch.equal(oT, o32.reshape(-1, o32.shape[-1]).t())
        assert torch.equal(o16, o32.reshape(-1, o32.shape[-1]).to(torch.bfloat16))
        # unfused path: explicit inputs_embeds
        o32b, _, _ = emb.forward_forms(None, tt.to(gpu) if use_tt else None, None,
                                       inputs_embeds=emb.word_embeddings(ids.to(gpu)), want_bf16=False, want_channel_major=False)
        assert (o32b - o32).abs().max().item() < 1e-5
    if cfg.use_positional_encodings:
        pos = torch.arange(100).flip(0)[None]
        o32, _, _ = emb.forward_forms(ids.to(gpu), None, pos.to(gpu), want_bf16=False, want_channel_major=False)
        e = emb.summed(ids.to(gpu), None, pos.to(gpu)).double().cpu()
        want = torch.nn.functional.layer_norm(e, (e.shape[-1],), sd["embeddings.LayerNorm.weight"].double(),
                                              sd["embeddings.LayerNorm.bias"].double(), cfg.layer_norm_eps)
        err, err2 = rel_err(o32, want)
        assert err < 1e-5 and err2 < 1e-5


def test_mixer_and_encoder_with_training_additions(gpu):
    """hyena_training_additions=True (the extra input LayerNorm of the mixer): one fp32 mixer at 1e-4, and a
    two-layer encoder (fused schedule, graph replay, module-by-module path) at the bf16 tolerance."""
    import m2_amd
    from oracle import m2_oracle as O
    cfg = m2_amd.m2_bert_80m(128)
    cfg.hyena_training_additions = True
    cfg.num_hidden_layers = 2
    sdm = m2_amd.seeded_state_dict(cfg, 77, what="mixer")
    mix = m2_amd.MonarchMixerSequenceMixing(768, l_max=128, bidirectional=True, hyena_emb_dim=5, hyena_filter_order=128,
                                            residual_long_conv=True, hyena_w=10, hyena_w_mod=1,
                                            hyena_training_additions=True)
    mix.load_state_dict(sdm)
    mix = mix.to(gpu).eval()
    u = torch.randn(4, 128, 768, generator=torch.Generator().manual_seed(8)) * 2 + 0.5
    y, _ = mix(u.to(gpu))
    e, e2 = rel_err(y, O.mixer_forward(sdm, "", u, training_additions=True))
    assert e < TOL_F32 and e2 < TOL_F32, (e, e2)

    sd = m2_amd.seeded_state_dict(cfg, 78)
    model = m2_amd.BertModel(cfg)
    model.load_state_dict(sd)
    model = model.to(gpu).eval()
    ids = torch.randint(0, cfg.vocab_size, (3, 128), generator=torch.Generator().manual_seed(6))
    ref = O.model_forward(sd, ids, None, cfg)
    out, _ = model(ids.to(gpu))
    e, e2 = rel_err(out, ref)
    assert e < TOL_BF16 and e2 < TOL_BF16, (e, e2)
    model.encoder.use_hip_graph = True
    for _ in range(2):
        got, _ = model(ids.to(gpu))
        torch.cuda.synchronize()
        assert torch.equal(got, out)
    model.encoder.use_hip_graph = False
    x = model.embeddings(ids.to(gpu))
    for layer in model.encoder.layer:
        x = layer(x)
    e, e2 = rel_err(x, ref)
    assert e < TOL_BF16 and e2 < TOL_BF16, (e, e2)


@pytest.mark.parametrize("pool_all", [False, True])
def test_pooled_output_and_text_encoder_loop(gpu, pool_all):
    """BertModel's pooled output against the oracle, and the embedding caller's batching loop (ragged and empty
    texts, padding, truncation, last partial batch) against one-at-a-time oracle results."""
    import m2_amd
    from oracle import m2_oracle as O
    cfg = m2_amd.m2_bert_80m(128)
    cfg.num_hidden_layers = 1
    cfg.pool_all = pool_all
    sd = m2_amd.seeded_state_dict(cfg, 61)
    model = m2_amd.BertModel(cfg)
    model.load_state_dict(sd)
    model = model.to(gpu).eval()
    g = torch.Generator().manual_seed(12)
    lengths = [5, 128, 0 if not pool_all else 1, 200, 64]       # an empty text has no mean: only with CLS pooling
    texts = [torch.randint(1, cfg.vocab_size, (n,), generator=g) for n in lengths]
    enc = m2_amd.M2BertTextEncoder(model, max_seq_len=128)
    got = enc.encode_token_ids(texts, batch_size=2)
    assert got.shape == (len(texts), cfg.hidden_size) and got.dtype.name == "float32"
    for k, ids in enumerate(texts):
        row = torch.zeros(1, 128, dtype=torch.long)
        n = min(len(ids), 128)
        row[0, :n] = ids[:n]
        mask = torch.zeros(1, 128, dtype=torch.long)
        mask[0, :n] = 1
        _, want = O.model_forward(sd, row, mask, cfg, pooled=True)
        err = (torch.from_numpy(got[k]) - want[0]).abs().max().item()
        assert err < 2e-2, (k, err)

    class WordTokenizer:                      # stands in for a Hugging Face tokenizer (same calling convention)
        def __call__(self, batch, return_tensors="pt"):
            ids = torch.tensor([[101] + [1000 + (hash(w) % 20000) for w in batch[0].split()] + [102]])
            return {"input_ids": ids, "attention_mask": torch.ones_like(ids)}
    enc = m2_amd.M2BertTextEncoder(model, max_seq_len=128, tokenizer=WordTokenizer())
    q = enc.encode_queries(["monarch mixer", "a longer query about sub-quadratic sequence models", "x"], batch_size=2)
    c = enc.encode_corpus([{"title": "T", "text": "some passage"}, {"title": "U", "text": "another"}], batch_size=8)
    assert q.shape == (3, cfg.hidden_size) and c.shape == (2, cfg.hidden_size)
    again = enc.encode_queries(["x"], batch_size=1)
    assert abs(again[0] - q[2]).max() < 2e-2          # same text alone or inside a batch


def test_model_loaded_from_reference_style_checkpoint_runs_identically(gpu, tmp_path):
    """A Composer-style checkpoint file (state/model nesting, `model.bert.` prefixes, head keys) loaded through
    the checkpoint loader gives bit-identical outputs to loading the plain state dict."""
    import os
    import m2_amd
    cfg = m2_amd.m2_bert_80m(128)
    cfg.num_hidden_layers = 1
    sd = m2_amd.seeded_state_dict(cfg, 31)
    path = os.path.join(tmp_path, "ckpt.pt")
    wrapped = {"model.bert." + k: v for k, v in sd.items()}
    wrapped["model.cls.predictions.bias"] = torch.zeros(8)
    torch.save({"state": {"model": wrapped}}, path)
    a = m2_amd.BertModel(cfg)
    a.load_state_dict(sd)
    b = m2_amd.BertModel(cfg)
    missing, unexpected = m2_amd.load_reference_checkpoint(b, path)
    assert missing == [] and unexpected == ["model.cls.predictions.bias"]
    a, b = a.to(gpu).eval(), b.to(gpu).eval()
    ids = torch.randint(0, cfg.vocab_size, (2, 128), generator=torch.Generator().manual_seed(4)).to(gpu)
    (sa, pa), (sb, pb) = a(ids), b(ids)
    assert torch.equal(sa, sb) and torch.equal(pa, pb)


@pytest.mark.parametrize("M,d,I", [(256, 768, 3072), (1000, 768, 3072), (64, 256, 1024), (130, 512, 768)])
def test_blockdiag_linear_layernorm_fused(gpu, M, d, I):
    """wo + bias + residual + LayerNorm as one kernel against fp64 on the bf16-rounded operands, all three output
    forms, ragged M, and against the two separate kernels."""
    from m2_amd import ops
    nb = 4
    assert ops.blockdiag_linear_layernorm_supported(I, d, nb)
    assert not ops.blockdiag_linear_layernorm_supported(6144, 1536, nb)        # d > 768: separate kernels
    assert not ops.blockdiag_linear_layernorm_supported(3072, 768, 8)
    g = torch.Generator().manual_seed(M + d)
    x = torch.randn(M, I, generator=g).bfloat16()
    w = (torch.randn(nb, d // nb, I // nb, generator=g) * 0.05).bfloat16()
    bias = torch.randn(d, generator=g)
    resid = torch.randn(M, d, generator=g).bfloat16()
    gamma = 1 + 0.1 * torch.randn(d, generator=g)
    beta = 0.1 * torch.randn(d, generator=g)
    xs = x.double().reshape(M, nb, I // nb)
    s = torch.einsum("mkp,kqp->mkq", xs, w.double()).reshape(M, d) + bias.double() + resid.double()
    want = torch.nn.functional.layer_norm(s, (d,), gamma.double(), beta.double(), 1e-12)
    o32, o16, ot = ops.blockdiag_linear_layernorm(x.to(gpu), w.to(gpu), bias.to(gpu), resid.to(gpu), gamma.to(gpu),
                                                  beta.to(gpu), 1e-12, want_f32=True, want_bf16=True, want_channel_major=True)
    e, e2 = rel_err(o32, want)
    assert e < 1e-3 and e2 < 1e-3, (e, e2)
    assert torch.equal(ot, o32.t())
    assert torch.equal(o16, o32.to(torch.bfloat16))
    # the two separate kernels
    s2 = ops.blockdiag_linear(x.to(gpu), w.to(gpu), bias.to(gpu), resid.to(gpu), out_dtype=torch.float32)
    ref32, _, _ = ops.layernorm(s2, gamma.to(gpu), beta.to(gpu), 1e-12)
    assert (ref32 - o32).abs().max().item() < 1e-4
    # no bias, no residual, only the channel-major output
    _, _, ot2 = ops.blockdiag_linear_layernorm(x.to(gpu), w.to(gpu), None, None, gamma.to(gpu), beta.to(gpu), 1e-5,
                                               want_f32=False, want_bf16=False, want_channel_major=True)
    s3 = torch.einsum("mkp,kqp->mkq", xs, w.double()).reshape(M, d)
    want3 = torch.nn.functional.layer_norm(s3, (d,), gamma.double(), beta.double(), 1e-5)
    e, e2 = rel_err(ot2.t(), want3)
    assert e < 1e-3 and e2 < 1e-3, (e, e2)


@pytest.mark.parametrize("L", [128, 4096])
@pytest.mark.parametrize("bidirectional,residual", [(False, True), (True, False), (False, False)])
def test_mixer_variants_without_reverse_filter_or_residual_conv(gpu, L, bidirectional, residual):
    """The module with bidirectional=False (reverse half of the window is zero) and / or residual_long_conv=False
    (no second convolution, no u input), B = 1, on the whole-row (L = 128) and the split (L = 4096) kernels."""
    import m2_amd
    from oracle import m2_oracle as O
    d = 64
    cfg = m2_amd.m2_bert_80m(L)
    cfg.hidden_size, cfg.bidirectional, cfg.residual_long_conv = d, bidirectional, residual
    sd = m2_amd.seeded_state_dict(cfg, 500 + L, std=0.1, what="mixer")
    sd["in_linear.bias"] = torch.randn(3 * d, generator=torch.Generator().manual_seed(1)) * 0.1
    mix = m2_amd.MonarchMixerSequenceMixing(d, l_max=L, bidirectional=bidirectional, hyena_emb_dim=5,
                                            hyena_filter_order=128, residual_long_conv=residual, hyena_w=10, hyena_w_mod=1)
    mix.load_state_dict(sd)
    mix = mix.to(gpu).eval()
    u = torch.randn(1, L, d, generator=torch.Generator().manual_seed(3))
    y, _ = mix(u.to(gpu))
    assert ("filter_fn2.bias" in sd) == residual
    ref = O.mixer_forward(sd, "", u, bidirectional, residual)
    e, e2 = rel_err(y, ref)
    assert e < TOL_F32 and e2 < TOL_F32, (e, e2)


def test_plain_fftconv_long_rows(gpu):
    """m2_fftconv_fwd (one filter, no short conv, no gates) on the half-transform kernels (L = 2048 .. 16384) and the
    real-signal kernel (L = 32768), fp32 and bf16 storage."""
    from m2_amd import ops
    from oracle import m2_oracle as O
    for L in (2048, 4096, 8192, 16384, 32768):
        d, B = 16, 2
        g = torch.Generator().manual_seed(L)
        x = torch.randn(d, B, L, generator=g)
        t = torch.linspace(0, 1, 2 * L)
        taps = torch.randn(d, 2 * L, generator=g) * torch.exp(-6 * torch.minimum(t, 1 - t))
        D = torch.randn(d, generator=g)
        spec = ops.filter_spectrum(taps.to(gpu), None, D.to(gpu), None)
        ref = O.fftconv(x.double().permute(1, 0, 2), taps.double(), D.double()[None, :, None]).permute(1, 0, 2)
        y = ops.fftconv(x.to(gpu), spec, B, L, d)
        assert rel_err(y, ref)[0] < TOL_F32
        y16 = ops.fftconv(x.bfloat16().to(gpu), spec, B, L, d)
        ref16 = O.fftconv(x.bfloat16().double().permute(1, 0, 2), taps.double(), D.double()[None, :, None]).permute(1, 0, 2)
        assert rel_err(y16.float(), ref16)[0] < 6e-3


def test_mixer_core_full_size_impulse_and_linearity(gpu):
    """At the benchmark's own size (L = 8192, B = 4, d = 768), properties that need no CPU transform:
    (1) with the projections zeroed the core is the second bidirectional convolution alone, so a unit impulse at
        position n0 must return the filter itself: y[t] = k_fwd[t - n0] for t >= n0, k_rev[n0 - t - 1] for t < n0
        (+ D at t = n0);
    (2) the core is affine in u: y(u1 + u2) - y(u1) - y(u2) + y(0) = 0."""
    from m2_amd import ops
    L, B, d = 8192, 4, 768
    g = torch.Generator().manual_seed(77)
    t = torch.linspace(0, 1, 2 * L)
    taps = [(torch.randn(d, 2 * L, generator=g) * torch.exp(-5 * torch.minimum(t, 1 - t))).to(gpu) for _ in range(2)]
    D = [torch.randn(d, generator=g).to(gpu) for _ in range(2)]
    spec = ops.filter_spectrum(taps[0], taps[1], D[0], D[1])
    sw = (torch.randn(3 * d, 3, generator=g) * 0.5).to(gpu)
    sb = (torch.randn(3 * d, generator=g) * 0.1).to(gpu)
    zero_x = torch.zeros(3 * d, B, L, device=gpu)
    zero_b = torch.zeros(3 * d, device=gpu)
    n0s = [0, 1, 4095, 8191]
    u = torch.zeros(d, B, L, device=gpu)
    for b, n0 in enumerate(n0s):
        u[:, b, n0] = 1.0
    y = ops.mixer_core(zero_x, u, sw, zero_b, spec, B, L, d)      # short conv of zeros with zero bias: a = 0, gate = 0
    k = taps[1]
    for b, n0 in enumerate(n0s):
        want = torch.empty(d, L, device=gpu)
        want[:, n0:] = k[:, :L - n0]                                 # causal taps k_fwd[t - n0]
        if n0 > 0:
            want[:, :n0] = k[:, 2 * L - n0:]                         # window position 2L - (n0 - t) holds k_rev[n0 - t - 1]
        want[:, n0] += D[1]
        err = (y[:, b] - want).abs().max().item() / want.abs().max().item()
        assert err < TOL_F32, (n0, err)
    # affinity in u with everything switched on
    xproj = torch.randn(3 * d, B, L, generator=g).to(gpu)
    u1 = torch.randn(d, B, L, generator=g).to(gpu)
    u2 = torch.randn(d, B, L, generator=g).to(gpu)
    f = lambda uu: ops.mixer_core(xproj, uu, sw, sb, spec, B, L, d)
    resid = f(u1 + u2) - f(u1) - f(u2) + f(torch.zeros_like(u1))
    scale = f(u1).abs().max().item()
    assert resid.abs().max().item() / scale < 5e-5


def test_unsupported_sizes_fail_loudly(gpu):
    from m2_amd import ops
    d = 64
    taps = torch.zeros(d, 2 * 192, device=gpu)
    with pytest.raises(RuntimeError, match="unsupported"):
        ops.filter_spectrum(taps, None, None, None)                 # L = 192 is not a power of two
    taps = torch.zeros(d, 2 * 64, device=gpu)
    with pytest.raises(RuntimeError, match="unsupported"):
        ops.filter_spectrum(taps, None, None, None)                 # L = 64 is below the shortest plan
    with pytest.raises(RuntimeError):
        ops.layernorm(torch.zeros(4, 100, device=gpu), torch.ones(100, device=gpu), torch.zeros(100, device=gpu), 1e-5)


@pytest.mark.parametrize("extra", [["--config", "c3"], ["--config", "c2", "--eager"]])
def test_bench_prints_its_json_line(gpu, extra):
    """bench.py as a child process (2 timed steps, no CPU leg): one JSON line with the fields the contract names."""
    import json, os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--steps", "2", "--warmup", "1",
                        "--no-cpu-baseline"] + extra, capture_output=True, text=True, timeout=110, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert line["n_gpus"] == 1 and line["steps"] == 2 and line["value"] > 0 and line["unit"] == "seq/s"
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and 0 < roof["frac"] < 1 and roof["peak"] == 8000.0
    assert abs(roof["achieved"] / roof["peak"] - roof["frac"]) < 1e-9
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=60, cwd=root)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_bench_reference_benchmark_form(gpu):
    """bench.py --reference-benchmark (random hidden states into the encoder, masked-LM head on top: the form of
    bert/benchmark_fwd.py:38-80) at the shortest length of the reference's grid: one JSON line, tokens per ms."""
    import json, os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--steps", "2", "--warmup", "1", "--config", "l512",
                        "--reference-benchmark"], capture_output=True, text=True, timeout=110, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert line["unit"] == "tokens/ms" and line["value"] > 0, line


@pytest.mark.parametrize("M,I", [(1, 3072), (100, 3072), (128, 3072), (300, 1536), (4096, 3072), (32768 - 70, 3072),
                                 (130, 256)])
def test_mlp_fused_matches_oracle_and_the_two_kernel_path(gpu, M, I):
    """gated_layers -> GLU -> wo + bias + residual as one kernel (d = 768) against fp64 on the bf16-rounded operands
    (the gated values rounded to bf16 between the two products, as the two-kernel path and the reference's autocast
    do), ragged M, both output dtypes, and against m2_blockdiag_glu_fwd + m2_blockdiag_linear_fwd."""
    from m2_amd import ops
    from oracle import m2_oracle as O
    d, nb = 768, 4
    assert ops.mlp_fused_supported(d, I, nb) and not ops.mlp_fused_supported(1536, 6144, nb)
    g = torch.Generator().manual_seed(M + I)
    x = torch.randn(M, d, generator=g).bfloat16()
    wg = (torch.randn(nb, 2 * I // nb, d // nb, generator=g) * 0.07).bfloat16()
    wo = (torch.randn(nb, d // nb, I // nb, generator=g) * 0.05).bfloat16()
    bias = torch.randn(d, generator=g)
    got = ops.mlp_fused(x.to(gpu), wg.to(gpu), wo.to(gpu), bias.to(gpu), x.to(gpu), out_dtype=torch.float32)
    h = O.blockdiag_multiply(x.float(), wg.float()).double()
    a = (torch.nn.functional.gelu(h[:, :I]) * h[:, I:])
    ref = O.blockdiag_multiply(a.float(), wo.float()).double() + bias.double() + x.double()
    e, e2 = rel_err(got, ref)
    assert e < 5e-3 and e2 < 3e-3, (e, e2)          # the only rounding inside is that of the gated values to bf16
    # the two-kernel path rounds at the same place: agreement to accumulation order
    g2 = ops.blockdiag_glu(x.to(gpu), wg.to(gpu))
    two = ops.blockdiag_linear(g2, wo.to(gpu), bias.to(gpu), x.to(gpu), out_dtype=torch.float32)
    assert rel_err(got, two)[0] < 1e-3
    got16 = ops.mlp_fused(x.to(gpu), wg.to(gpu), wo.to(gpu), None, None, out_dtype=torch.bfloat16)
    ref16 = O.blockdiag_multiply(a.float(), wo.float()).double()
    assert rel_err(got16.float(), ref16)[0] < TOL_BF16
    with pytest.raises(RuntimeError, match="768"):
        ops.mlp_fused(torch.zeros(8, 512, device=gpu, dtype=torch.bfloat16),
                      torch.zeros(4, 256, 128, device=gpu, dtype=torch.bfloat16),
                      torch.zeros(4, 128, 128, device=gpu, dtype=torch.bfloat16))


@pytest.mark.parametrize("M,in_f,out_f,nb", [(300, 768, 6144, 4), (65, 256, 100, 4), (1, 64, 8, 2), (1000, 3072, 768, 4)])
def test_blockdiag_linear_fp32_outside_autocast(gpu, M, in_f, out_f, nb):
    """BlockdiagLinear / blockdiag_multiply with fp32 input and no autocast compute in fp32 (1e-4 against fp64), as
    the reference does on that call; under autocast the same module rounds its operands to bf16."""
    import m2_amd
    from oracle import m2_oracle as O
    g = torch.Generator().manual_seed(M + out_f)
    lin = m2_amd.BlockdiagLinear(in_f, out_f, bias=True, nblocks=nb)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(lin.weight.shape, generator=g) * 0.05)
        lin.bias.copy_(torch.randn(out_f, generator=g))
    x = torch.randn(2, M, in_f, generator=g)
    ref = O.blockdiag_linear(x.double(), lin.weight.detach().double(), lin.bias.detach().double(), in_f, out_f)
    lin = lin.to(gpu)
    got = lin(x.to(gpu))
    assert got.dtype == torch.float32 and got.shape == (2, M, out_f)
    e, e2 = rel_err(got, ref)
    assert e < 2e-6 and e2 < 2e-6, (e, e2)
    got_mul = m2_amd.blockdiag_multiply(x.to(gpu), lin.weight)
    assert rel_err(got_mul, O.blockdiag_multiply(x.double(), lin.weight.detach().double().cpu()))[0] < 2e-6
    if (in_f // nb) % 64 == 0 and (out_f // nb) % 64 == 0:
        with torch.autocast("cuda", dtype=torch.bfloat16):
            low = lin(x.to(gpu))
        assert low.dtype == torch.bfloat16
        e = rel_err(low.float(), ref)[0]
        assert 1e-4 < e < TOL_BF16, e


@pytest.mark.gpu
@pytest.mark.parametrize("M,I,d", [(1, 6144, 1536), (100, 6144, 1536), (128, 6144, 1536), (300, 1536, 1536), (8192, 6144, 1536),
                                   (8192 - 70, 6144, 1536), (130, 256, 1536), (520, 128, 1536),
                                   (1, 3840, 960), (8192 - 70, 3840, 960), (300, 128, 960), (200, 3840, 896), (200, 1024, 992),
                                   (1, 7168, 1792), (8192 - 70, 7168, 1792), (300, 128, 1792), (33000, 256, 1792)])
def test_glu_stream_matches_oracle_and_the_tiled_kernel(gpu, M, I, d):
    """gated_layers -> GLU for 384-wide blocks (d = 1536), 448-wide ones (d = 1792: two LDS stages instead of three) and
    blocks of 224 .. 248 (d = 960: 240 wide, computed as 256 with zeros beyond) from packed weights, against fp64 on the bf16-rounded operands and against
    m2_blockdiag_glu_fwd (same arithmetic: bit-close, the accumulation order differs), ragged M, one chunk per r
    (I = 128), more rows than one round of workgroups."""
    from m2_amd import ops
    from oracle import m2_oracle as O
    nb = 4
    assert ops.glu_stream_supported(d, I, nb) and not ops.glu_stream_supported(768, 3072, nb)
    assert not ops.glu_stream_supported(1024, 4096, nb) and not ops.glu_stream_supported(2048, 8192, nb)
    g = torch.Generator().manual_seed(7 * M + I)
    x = torch.randn(M, d, generator=g).bfloat16()
    wg = (torch.randn(nb, 2 * I // nb, d // nb, generator=g) * 0.05).bfloat16()
    got = ops.glu_stream(x.to(gpu), wg.to(gpu))
    h = O.blockdiag_multiply(x.float(), wg.float()).double()
    ref = torch.nn.functional.gelu(h[:, :I]) * h[:, I:]
    assert got.shape == (M, I) and got.dtype == torch.bfloat16
    assert rel_err(got.float(), ref)[0] < TOL_BF16
    tiled = ops.blockdiag_glu(x.to(gpu), wg.to(gpu))
    assert rel_err(got.float(), tiled.float().double())[0] < 1e-2      # both rounded to bf16: an ulp apart at most
    # the packed weight can be computed once and handed in
    pk = ops.glu_stream_pack(wg.to(gpu))
    again = ops.glu_stream(x.to(gpu), wg.to(gpu), packed=pk)
    assert torch.equal(again, got)
    with pytest.raises(RuntimeError, match="384"):
        ops.glu_stream(torch.zeros(8, 768, device=gpu, dtype=torch.bfloat16),
                       torch.zeros(4, 256, 192, device=gpu, dtype=torch.bfloat16))

