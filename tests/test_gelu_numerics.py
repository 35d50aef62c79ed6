"""CPU pins of the GLU kernels' x Phi(x) polynomial (m2_amd/csrc/mfma_stream.h, blockdiag_kernels.hip), element by
element on the distribution the GPU test uses (tests/test_gpu_configs.py::test_glu_at_benchmark_sizes_and_gelu_tails):

  * the clamped odd degree-13 polynomial evaluated in float32, as the kernels do, stays inside the bound
    |ref| 2^-7 + 2.5e-4 (|value| + 1) against erf-GELU in float64 (bert/src/bert_layers.py:475,494-502);
  * the same polynomial evaluated in IEEE half precision (what packed-half instructions would compute, x^2 range-scaled
    so that nothing overflows) does not: 0.5 + x p(x^2) cancels in the negative tail, where half precision leaves an
    absolute error of about 2^-11 |x| -- which is why the kernels evaluate the gate in float32.
"""
import torch

COEF = [2.7693410957e-08, -1.8473178272e-06, 5.2869800351e-05, -8.6171873090e-04, 9.0065851481e-03, -6.5103946404e-02,
        3.9828952833e-01]


def _gelu_poly(x, dt):
    xc = x.clamp(-3.9, 3.9).to(dt)
    x2 = (xc * xc / 16.0).to(dt)                       # <= 0.95; coefficients rescaled by 16^k
    c = [torch.tensor(COEF[i] * 16.0 ** (6 - i), dtype=dt) for i in range(7)]
    p = c[0]
    for k in range(1, 7):
        p = torch.addcmul(c[k], p, x2).to(dt)          # one fused multiply-add rounded to dt
    p = torch.addcmul(torch.tensor(0.5, dtype=dt), p, xc).to(dt)
    return (x.to(dt) * p).to(dt)


def _violations(sigma, dt):
    g = torch.Generator().manual_seed(17)
    gate = torch.randn(1_000_000, generator=g, dtype=torch.float64) * sigma
    val = torch.randn(1_000_000, generator=g, dtype=torch.float64) * sigma
    ref = torch.nn.functional.gelu(gate) * val
    out = (_gelu_poly(gate.float(), dt).double() * val).float().bfloat16().double()
    err = (out - ref).abs()
    bound = ref.abs() * 2.0 ** -7 + 2.5e-4 * (val.abs() + 1)
    return (err > bound).double().mean().item(), (err / bound).max().item()


def test_float32_polynomial_meets_the_element_wise_bound():
    for sigma in (0.7, 3.0):
        frac, worst = _violations(sigma, torch.float32)
        assert frac == 0.0 and worst < 0.8, (sigma, frac, worst)


def test_half_precision_polynomial_misses_it():
    frac, worst = _violations(3.0, torch.float16)
    assert frac > 0.05 and worst > 10.0, (frac, worst)
