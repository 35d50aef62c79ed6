"""Pins of the CPU oracle (oracle/m2_oracle.py) that do not retype its formulas.

The reference ships no golden vectors for this path, so each oracle function is checked against
something independent: a closed form with spot values worked out by hand, an O(L^2) float64 direct
sum, a scipy / numpy library routine, a dense-matrix equivalent, or an invariant (linearity,
causality, mask independence).  A dropped term, a wrong sign, an off-by-one in the anti-causal
branch or a transposed operand fails at least one of them.
"""
import math

import numpy as np
import pytest
import scipy.signal
import torch
import torch.nn.functional as F

from oracle import m2_oracle as O

torch.manual_seed(0)
DT = torch.float64


# ---------------------------------------------------------------------------- positional embedding
def test_positional_embedding_spot_values():
    """L=16, emb_dim=5: row l=1 is [1/15, cos(1e-4 w), cos(w), -sin(1e-4 w), -sin(w)], w = 2 pi/16."""
    z, t = O.positional_embedding(5, 16)
    assert z.shape == (1, 16, 5) and t.shape == (1, 16, 1)
    expect = [1 / 15, 1.0, 0.9238795325, -3.9269908e-05, -0.3826834324]
    assert np.allclose(z[0, 1].numpy(), expect, atol=2e-7)
    assert np.allclose(z[0, 0].numpy(), [0, 1, 1, 0, 0], atol=1e-7)
    assert np.allclose(t[0, :, 0].numpy(), np.linspace(0, 1, 16), atol=1e-7)
    # emb_dim = 3: one band at frequency 1e-4 only
    z3, _ = O.positional_embedding(3, 8)
    assert z3.shape == (1, 8, 3)
    assert np.allclose(z3[0, :, 1].numpy(), np.cos(1e-4 * 2 * np.pi * np.arange(8) / 8), atol=1e-7)


def test_positional_embedding_is_what_the_modules_hold():
    """The product modules build z/t with their own code (complex exponential form): same numbers."""
    from m2_amd.init import positional_embedding_buffers
    for emb, L in [(5, 128), (3, 64), (7, 32)]:
        z, t = O.positional_embedding(emb, L)
        z2, t2 = positional_embedding_buffers(emb, L)
        assert torch.allclose(z, z2, atol=1e-6) and torch.equal(t, t2)


def test_modulation_deltas_closed_form():
    dl = O.modulation_deltas(768)
    assert dl.shape == (1, 1, 768)
    assert abs(dl[0, 0, 0].item() - math.log(0.01) / 1.5) < 1e-6      # -3.0701
    assert abs(dl[0, 0, -1].item() - math.log(0.01) / 0.3) < 1e-5     # -15.3506
    assert abs(dl[0, 0, 0].item() + 3.0701134) < 1e-5 and abs(dl[0, 0, -1].item() + 15.3505673) < 1e-5
    steps = dl[0, 0, 1:] - dl[0, 0, :-1]
    assert torch.allclose(steps, steps[0].expand_as(steps), atol=1e-5)


# ---------------------------------------------------------------------------- implicit filter MLP
def _filter_sd(d=12, order=8, emb=5, L=32, seed=0, std=0.5):
    g = torch.Generator().manual_seed(seed)
    z, t = O.positional_embedding(emb, L, DT)
    sd = {"pos_emb.z": z, "pos_emb.t": t, "modulation.deltas": O.modulation_deltas(d, dtype=DT),
          "implicit_filter.1.freq": 10 * torch.ones(1, order, dtype=DT) + torch.randn(1, order, generator=g).to(DT)}
    for mlp in ("implicit_filter.", "implicit_filter_rev."):
        for i, (o, k) in enumerate([(order, emb), (order, order), (order, order)]):
            sd[f"{mlp}{2 * i}.weight"] = (torch.randn(o, k, generator=g) * std).to(DT)
            sd[f"{mlp}{2 * i}.bias"] = (torch.randn(o, generator=g) * std).to(DT)
        sd[f"{mlp}6.weight"] = (torch.randn(d, order, generator=g) * std).to(DT)
    return sd


def test_hyena_filter_taps_vs_numpy_loops():
    """Independent evaluation with explicit numpy loops over positions and layers."""
    d, order, emb, L = 12, 8, 5, 32
    sd = _filter_sd(d, order, emb, L)
    for rev in (False, True):
        got = O.hyena_filter_taps(sd, "", L, rev=rev, w_mod=1.0, shift=0.0)[0].numpy()
        mlp = "implicit_filter_rev." if rev else "implicit_filter."
        W = [sd[f"{mlp}{i}.weight"].numpy() for i in (0, 2, 4, 6)]
        b = [sd[f"{mlp}{i}.bias"].numpy() for i in (0, 2, 4)]
        f = sd["implicit_filter.1.freq"].numpy()[0]
        z = sd["pos_emb.z"].numpy()[0]
        t = sd["pos_emb.t"].numpy()[0, :, 0]
        dl = np.abs(sd["modulation.deltas"].numpy()[0, 0])
        want = np.zeros((L, d))
        for l in range(L):
            h = z[l]
            for layer in range(3):
                h = np.sin(f * (W[layer] @ h + b[layer]))
            want[l] = (W[3] @ h) * np.exp(-t[l] * dl)
        assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    # forward and reverse MLPs are different functions of the same embedding
    assert not torch.allclose(O.hyena_filter_taps(sd, "", L, rev=False), O.hyena_filter_taps(sd, "", L, rev=True))


def test_hyena_filter_w_mod_and_shift():
    sd = _filter_sd()
    base = O.hyena_filter_taps(sd, "", 32)
    sd2 = dict(sd)
    sd2["implicit_filter.1.freq"] = sd["implicit_filter.1.freq"] * 2
    assert torch.allclose(O.hyena_filter_taps(sd, "", 32, w_mod=2.0), O.hyena_filter_taps(sd2, "", 32), atol=1e-12)
    # shift adds the undecayed MLP output
    sd3 = dict(sd)
    sd3["modulation.deltas"] = torch.zeros_like(sd["modulation.deltas"])      # decay == 1
    raw = O.hyena_filter_taps(sd3, "", 32)
    assert torch.allclose(O.hyena_filter_taps(sd, "", 32, shift=0.25), base + 0.25 * raw, atol=1e-12)


# ---------------------------------------------------------------------------- long convolution
def _direct_bidirectional(u, k_fwd, k_rev, D):
    """y[t] = sum_{s<=t} k_fwd[s] u[t-s] + sum_{j>t} k_rev[j-t-1] u[j] + D u[t], plain loops."""
    B, C, L = u.shape
    y = np.zeros((B, C, L))
    for b in range(B):
        for c in range(C):
            for t in range(L):
                acc = D[c] * u[b, c, t]
                for s in range(t + 1):
                    acc += k_fwd[c, s] * u[b, c, t - s]
                for j in range(t + 1, L):
                    acc += k_rev[c, j - t - 1] * u[b, c, j]
                y[b, c, t] = acc
    return y


@pytest.mark.parametrize("L", [1, 2, 7, 16, 33])
def test_fftconv_bidirectional_vs_direct_sum(L):
    g = torch.Generator().manual_seed(L)
    B, C = 2, 3
    u = torch.randn(B, C, L, generator=g, dtype=DT)
    kf = torch.randn(C, L, generator=g, dtype=DT)
    kr = torch.randn(C, L, generator=g, dtype=DT)
    D = torch.randn(C, generator=g, dtype=DT)
    got = O.hyena_filter_forward(u, L, kf, kr, D[None, :, None]).numpy()
    want = _direct_bidirectional(u.numpy(), kf.numpy(), kr.numpy(), D.numpy())
    assert np.allclose(got, want, atol=1e-10)


def test_fftconv_vs_scipy_fftconvolve():
    """Full linear convolution with the two-sided kernel [flip(k_rev), k_fwd], then the right slice."""
    L, C = 40, 2
    g = torch.Generator().manual_seed(3)
    u = torch.randn(1, C, L, generator=g, dtype=DT)
    kf = torch.randn(C, L, generator=g, dtype=DT)
    kr = torch.randn(C, L, generator=g, dtype=DT)
    got = O.hyena_filter_forward(u, L, kf, kr, torch.zeros(1, C, 1, dtype=DT))[0].numpy()
    for c in range(C):
        # two-sided kernel h[m], m = -L..L-1: h[m] = k_fwd[m] (m >= 0), h[-m'] = k_rev[m'-1] (m' >= 1); k_rev[L-1] is lag -L
        h = np.concatenate([kr[c].numpy()[::-1], kf[c].numpy()])          # index i <-> lag i - L
        full = scipy.signal.fftconvolve(u[0, c].numpy(), h)               # index n <-> output t = n - L
        assert np.allclose(got[c], full[L:2 * L], atol=1e-10)
        assert np.allclose(got[c], np.convolve(u[0, c].numpy(), h)[L:2 * L], atol=1e-10)


def test_fftconv_causal_only_and_delta():
    L, C = 24, 2
    g = torch.Generator().manual_seed(4)
    u = torch.randn(1, C, L, generator=g, dtype=DT)
    k = torch.randn(C, L, generator=g, dtype=DT)
    zero = torch.zeros(C, L, dtype=DT)
    D0 = torch.zeros(1, C, 1, dtype=DT)
    y = O.hyena_filter_forward(u, L, k, zero, D0)
    for c in range(C):
        assert np.allclose(y[0, c].numpy(), np.convolve(u[0, c].numpy(), k[c].numpy())[:L], atol=1e-10)
    # causality: changing inputs after t0 leaves outputs up to t0 alone; anti-causal filter is strictly so
    u2 = u.clone()
    u2[..., 10:] += 1.0
    assert torch.allclose(O.hyena_filter_forward(u2, L, k, zero, D0)[..., :10], y[..., :10], atol=1e-10)
    ya = O.hyena_filter_forward(u, L, zero, k, D0)
    ya2 = O.hyena_filter_forward(u2, L, zero, k, D0)
    assert not torch.allclose(ya2[..., :10], ya[..., :10])
    u3 = u.clone()
    u3[..., :10] += 1.0                                            # the past (and the present) do not matter
    assert torch.allclose(O.hyena_filter_forward(u3, L, zero, k, D0)[..., 10:], ya[..., 10:], atol=1e-10)
    # delta filter is the identity; D is a per-channel skip
    delta = torch.zeros(C, L, dtype=DT)
    delta[:, 0] = 1
    Dv = torch.tensor([0.5, -2.0], dtype=DT)[None, :, None]
    assert torch.allclose(O.hyena_filter_forward(u, L, delta, zero, Dv), u * (1 + Dv), atol=1e-10)
    # k_rev = delta picks the next sample
    assert torch.allclose(O.hyena_filter_forward(u, L, zero, delta, D0)[..., :-1], u[..., 1:], atol=1e-10)


def test_fftconv_linearity_and_unidirectional():
    L, C = 16, 3
    g = torch.Generator().manual_seed(6)
    u, v = (torch.randn(2, C, L, generator=g, dtype=DT) for _ in range(2))
    kf, kr = (torch.randn(C, L, generator=g, dtype=DT) for _ in range(2))
    D = torch.randn(1, C, 1, generator=g, dtype=DT)
    f = lambda x: O.hyena_filter_forward(x, L, kf, kr, D)
    assert torch.allclose(f(2 * u - 3 * v), 2 * f(u) - 3 * f(v), atol=1e-10)
    # not bidirectional: the kernel is just k_fwd (L taps)
    assert torch.allclose(O.hyena_filter_forward(u, L, kf, None, D),
                          O.hyena_filter_forward(u, L, kf, torch.zeros_like(kf), D), atol=1e-10)
    assert O.bidirectional_kernel(kf, kr, L).shape == (C, 2 * L)
    assert torch.equal(O.bidirectional_kernel(kf, kr, L)[:, L:], kr.flip(-1))


# ---------------------------------------------------------------------------- short conv + mixer
def test_short_conv_three_tap_sum():
    B, C, L = 2, 6, 9
    g = torch.Generator().manual_seed(8)
    u = torch.randn(B, C, L, generator=g, dtype=DT)
    w = torch.randn(C, 1, 3, generator=g, dtype=DT)
    b = torch.randn(C, generator=g, dtype=DT)
    got = O.short_conv(u, w, b).numpy()
    un, wn, bn = u.numpy(), w.numpy(), b.numpy()
    want = np.zeros((B, C, L))
    for t in range(L):
        for j in range(3):
            s = t - 2 + j
            if s >= 0:
                want[:, :, t] += wn[None, :, 0, j] * un[:, :, s]
        want[:, :, t] += bn
    assert np.allclose(got, want, atol=1e-12)


def _tiny_cfg(L=16, d=8, layers=2, I=16):
    import m2_amd
    return m2_amd.M2BertConfig(hidden_size=d, intermediate_size=I, num_hidden_layers=layers, vocab_size=50,
                               hyena_filter_order=8).with_seq_len(L)


def test_mixer_forward_is_the_composition_written_with_loops():
    """Whole mixer on a tiny case against an independent numpy restatement that uses the direct-sum
    convolution and explicit channel slicing (x1 = [0,d), x2 = [d,2d), v = [2d,3d))."""
    import m2_amd
    cfg = _tiny_cfg(L=12, d=4)
    sd = O.cast_state_dict(m2_amd.seeded_state_dict(cfg, 3, std=0.4, what="mixer"), DT)
    B, L, d = 2, cfg.long_conv_l_max, cfg.hidden_size
    u = torch.randn(B, L, d, generator=torch.Generator().manual_seed(1), dtype=DT)
    got = O.mixer_forward(sd, "", u).numpy()
    un = u.numpy()
    proj = un @ sd["in_linear.weight"].numpy().T + sd["in_linear.bias"].numpy()       # (B, L, 3d)
    pc = np.transpose(proj, (0, 2, 1))                                                 # (B, 3d, L)
    sw, sb = sd["short_filter.weight"].numpy()[:, 0], sd["short_filter.bias"].numpy()
    uc = np.zeros_like(pc)
    for t in range(L):
        uc[:, :, t] = sb + sum(sw[:, j] * pc[:, :, t - 2 + j] for j in range(3) if t - 2 + j >= 0)
    x1, x2, v = uc[:, :d], uc[:, d:2 * d], uc[:, 2 * d:]
    k = [O.hyena_filter_taps(sd, p, L, rev=r)[0].numpy().T for p in ("filter_fn.", "filter_fn2.") for r in (False, True)]
    y1 = _direct_bidirectional(v * x1, k[0], k[1], sd["filter_fn.bias"].numpy())
    y2 = _direct_bidirectional(np.transpose(un, (0, 2, 1)), k[2], k[3], sd["filter_fn2.bias"].numpy())
    y = np.transpose(y1 * x2 + y2, (0, 2, 1))
    want = y @ sd["out_linear.weight"].numpy().T + sd["out_linear.bias"].numpy()
    assert np.allclose(got, want, atol=1e-9)
    # without the residual long conv the second term is absent
    got_nores = O.mixer_forward(sd, "", u, residual_long_conv=False).numpy()
    want_nores = np.transpose(y1 * x2, (0, 2, 1)) @ sd["out_linear.weight"].numpy().T + sd["out_linear.bias"].numpy()
    assert np.allclose(got_nores, want_nores, atol=1e-9)


# ---------------------------------------------------------------------------- block-diagonal MLP
def test_blockdiag_multiply_is_block_diag_matmul():
    g = torch.Generator().manual_seed(9)
    nb, q, p = 4, 5, 3
    w = torch.randn(nb, q, p, generator=g, dtype=DT)
    x = torch.randn(2, 7, nb * p, generator=g, dtype=DT)
    dense = torch.block_diag(*w.unbind(0))                         # (nb q, nb p)
    assert torch.allclose(O.blockdiag_multiply(x, w), F.linear(x, dense), atol=1e-12)
    # the bmm form of the reference's fast path
    xr = x.reshape(-1, nb, p).transpose(0, 1)
    bm = torch.bmm(xr, w.transpose(-1, -2)).transpose(0, 1).reshape(2, 7, nb * q)
    assert torch.allclose(O.blockdiag_multiply(x, w), bm, atol=1e-12)


def test_blockdiag_linear_pad_crop_bias():
    g = torch.Generator().manual_seed(10)
    nb, in_f, out_f = 4, 10, 9                     # not divisible: p = 3 (pad to 12), q = 3 (crop 12 -> 9)
    w = torch.randn(nb, 3, 3, generator=g, dtype=DT)
    b = torch.randn(out_f, generator=g, dtype=DT)
    x = torch.randn(5, in_f, generator=g, dtype=DT)
    dense = torch.block_diag(*w.unbind(0))[:out_f, :in_f]
    assert torch.allclose(O.blockdiag_linear(x, w, b, in_f, out_f), F.linear(x, dense, b), atol=1e-12)
    assert torch.allclose(O.blockdiag_linear(x, w, None, in_f, out_f), F.linear(x, dense), atol=1e-12)


def test_glu_mlp_dense_equivalent_and_pairing():
    """Gate column j pairs with value column I + j, i.e. gate block k with value block k + nb/2."""
    import m2_amd
    cfg = _tiny_cfg(d=8, I=16)
    sd = O.cast_state_dict(m2_amd.seeded_state_dict(cfg, 5, std=0.5, what="mlp"), DT)
    sd["layernorm.weight"] = torch.randn(8, dtype=DT)
    sd["layernorm.bias"] = torch.randn(8, dtype=DT)
    sd["wo.bias"] = torch.randn(8, dtype=DT)
    x = torch.randn(2, 5, 8, dtype=DT)
    got = O.glu_mlp_forward(sd, "", x, 16, 1e-12)
    Wg = torch.block_diag(*sd["gated_layers.weight"].unbind(0))    # (32, 8)
    Wo = torch.block_diag(*sd["wo.weight"].unbind(0))              # (8, 16)
    h = x @ Wg.T
    gate, val = h[..., :16], h[..., 16:]
    a = 0.5 * gate * (1 + torch.erf(gate / math.sqrt(2))) * val
    o = a @ Wo.T + sd["wo.bias"] + x
    mu = o.mean(-1, keepdim=True)
    var = ((o - mu) ** 2).mean(-1, keepdim=True)
    want = (o - mu) / torch.sqrt(var + 1e-12) * sd["layernorm.weight"] + sd["layernorm.bias"]
    assert torch.allclose(got, want, atol=1e-10)
    # block structure: gate columns [0, 8) read only input block 0, value columns [16, 24) only block 2
    x2 = x.clone()
    x2[..., 2:4] += 1.0                                            # input block 1
    h2 = O.blockdiag_multiply(x2, sd["gated_layers.weight"])
    assert torch.allclose(h2[..., :8], h[..., :8]) and torch.allclose(h2[..., 16:24], h[..., 16:24])
    assert not torch.allclose(h2[..., 8:16], h[..., 8:16])


# ---------------------------------------------------------------------------- layer / encoder / embeddings
def test_encoder_ignores_attention_mask_and_stacks_layers():
    import m2_amd
    cfg = _tiny_cfg(L=16, d=8, layers=3)
    sd = O.cast_state_dict(m2_amd.seeded_state_dict(cfg, 6, std=0.3), DT)
    x = torch.randn(2, 16, 8, dtype=DT)
    m1 = torch.ones(2, 16, dtype=torch.long)
    m0 = m1.clone()
    m0[:, 8:] = 0
    a = O.encoder_forward(sd, "encoder.", x, m1, cfg, output_all_encoded_layers=True)
    b = O.encoder_forward(sd, "encoder.", x, m0, cfg, output_all_encoded_layers=True)
    assert len(a) == 3 and all(torch.equal(p, q) for p, q in zip(a, b))
    # layer i output is layer_forward of layer i-1 output; no residual around the mixer
    y = x
    for i in range(3):
        mix = O.mixer_forward(sd, f"encoder.layer.{i}.attention.", y)
        y = O.glu_mlp_forward(sd, f"encoder.layer.{i}.mlp.", mix, cfg.intermediate_size, cfg.layer_norm_eps)
        assert torch.allclose(a[i], y, atol=1e-10)
    assert torch.equal(O.encoder_forward(sd, "encoder.", x, None, cfg)[-1], a[-1])


def test_embeddings_gather_and_layernorm():
    import m2_amd
    cfg = _tiny_cfg(L=16, d=8, layers=1)
    sd = O.cast_state_dict(m2_amd.seeded_state_dict(cfg, 7, std=0.5), DT)
    ids = torch.randint(0, cfg.vocab_size, (3, 16), generator=torch.Generator().manual_seed(2))
    got = O.embeddings_forward(sd, "embeddings.", ids, cfg)
    W, T, P = (sd[f"embeddings.{n}.weight"] for n in ("word_embeddings", "token_type_embeddings", "position_embeddings"))
    e = torch.stack([torch.stack([W[ids[b, l]] + T[0] + P[l] for l in range(16)]) for b in range(3)])
    want = F.layer_norm(e, (8,), sd["embeddings.LayerNorm.weight"], sd["embeddings.LayerNorm.bias"], 1e-12)
    assert torch.allclose(got, want, atol=1e-12)
    # shorter sequences use the first L position rows
    got8 = O.embeddings_forward(sd, "embeddings.", ids[:, :8], cfg)
    assert torch.allclose(got8, got[:, :8], atol=1e-12)
    tt = torch.ones_like(ids)
    assert not torch.allclose(O.embeddings_forward(sd, "embeddings.", ids, cfg, tt), got)


def test_mixer_training_additions_is_a_pre_layernorm_seen_by_both_convolutions():
    """hyena_training_additions in eval mode: the input LayerNorm (eps 1e-5) feeds the projections AND the
    residual long convolution (monarch_mixer_sequence_mixer.py:102-107); everything else is unchanged.  Checked
    by composing the plain mixer with an explicitly computed LayerNorm, and by showing that normalising only the
    projection input (the plausible mistake) gives a different answer."""
    import m2_amd
    cfg = m2_amd.m2_bert_80m(64)
    cfg.hidden_size = 64
    cfg.hyena_training_additions = True
    sd = {k: v.double() for k, v in m2_amd.seeded_state_dict(cfg, 5, std=0.3, what="mixer").items()}
    u = torch.randn(2, 64, 64, dtype=torch.float64, generator=torch.Generator().manual_seed(2)) * 3 + 1.5
    got = O.mixer_forward(sd, "", u, True, True, 1.0, True)
    mu = u.mean(-1, keepdim=True)
    var = ((u - mu) ** 2).mean(-1, keepdim=True)
    un = (u - mu) / torch.sqrt(var + 1e-5) * sd["layernorm.weight"] + sd["layernorm.bias"]
    want = O.mixer_forward(sd, "", un, True, True, 1.0, False)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    # the residual convolution must see the normalised input: feeding it the raw input changes the result
    plain = O.mixer_forward(sd, "", u, True, True, 1.0, False)
    assert (got - plain).abs().max() > 1e-3


def test_pooler_first_token_and_masked_mean():
    """BertPooler (bert/src/bert_layers.py:816-859): tanh(W h[:, 0] + b), and with pool_all the mean over the
    positions whose mask is 1 only -- checked against explicit per-example loops."""
    g = torch.Generator().manual_seed(11)
    B, L, d = 3, 7, 5
    h = torch.randn(B, L, d, dtype=torch.float64, generator=g)
    sd = {"dense.weight": torch.randn(d, d, dtype=torch.float64, generator=g),
          "dense.bias": torch.randn(d, dtype=torch.float64, generator=g)}
    mask = torch.tensor([[1, 1, 1, 0, 0, 0, 0], [1, 1, 1, 1, 1, 1, 1], [1, 0, 0, 0, 0, 0, 0]])
    cls = O.pooler_forward(sd, "", h, mask, pool_all=False)
    mean = O.pooler_forward(sd, "", h, mask, pool_all=True)
    for b in range(B):
        want = torch.tanh(sd["dense.weight"] @ h[b, 0] + sd["dense.bias"])
        assert torch.allclose(cls[b], want, atol=1e-14)
        n = int(mask[b].sum())
        avg = sum(h[b, l] for l in range(L) if mask[b, l] == 1) / n
        assert torch.allclose(mean[b], torch.tanh(sd["dense.weight"] @ avg + sd["dense.bias"]), atol=1e-14)
    # one real token: both poolings coincide
    assert torch.allclose(cls[2], mean[2], atol=1e-14)
