"""Pins the oracle's optimizer-side functions (Adam(W) step, sum of squares,
clip coefficient, scale) without a GPU: against torch's own ops and optimizers
on CPU, against binary64 evaluation, and against closed forms.

torch's CPU square root is not correctly rounded (about 0.6 % of results are
one ulp off), the oracle's is; whole Adam steps therefore agree with
torch.optim to one ulp per step, while every other tensor of the step (both
moments) must agree bit for bit.
"""

import math

import numpy as np
import pytest
import torch

from oracle import cref, torch_ops

from helpers import assert_bits_equal

F32 = np.float32
HP = dict(lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


def _fma(a, b, c):
    """fused multiply-add of binary32 arrays through binary64 (the product is exact there)."""
    a, b, c = (np.asarray(x, F32).astype(np.float64) for x in (a, b, c))
    return (a * b + c).astype(F32)


def _bits(x):
    return np.asarray(x).view(np.uint32)


def _state(n, seed):
    g = torch.Generator().manual_seed(seed)
    p = torch.randn(n, generator=g) * 0.02
    grad = torch.randn(n, generator=g) * 1e-3
    m = torch.randn(n, generator=g) * 1e-3
    v = (torch.randn(n, generator=g) * 1e-3) ** 2
    return p, grad, m, v


def _param_agreement(got: torch.Tensor, want: torch.Tensor, before: torch.Tensor, steps: int = 1) -> None:
    """Updated parameters agree to two ulps of max(|p|, |update|) per step, and almost all bit for bit."""
    scale = torch.maximum(want.abs(), (want - before).abs()).double()
    err = (got.double() - want.double()).abs()
    assert bool((err <= steps * 2.0**-22 * scale).all()), float((err / scale.clamp_min(1e-300)).max())
    differing = (got.view(torch.int32) != want.view(torch.int32)).float().mean().item()
    assert differing < 0.01 * steps, differing


# --------------------------------------------------- where torch fuses multiply-adds --
def test_torch_cpu_ops_fuse_where_the_oracle_says():
    n = 200_003
    p, g, m, v = _state(n, 1)
    pn, gn, mn, vn = (x.numpy() for x in (p, g, m, v))
    # lerp_, small and large weight
    for w in (0.1, 0.7):
        got = m.clone().lerp_(g, w).numpy()
        wf = F32(w)
        fused = _fma(np.full(n, wf), gn - mn, mn) if w < 0.5 else _fma(np.full(n, wf - F32(1)), gn - mn, gn)
        plain = mn + wf * (gn - mn) if w < 0.5 else gn - (gn - mn) * (F32(1) - wf)
        assert (_bits(got) != _bits(fused)).sum() == 0
        assert (_bits(got) != _bits(plain)).sum() > n // 100
    # addcmul_: fma((value*g), g, v)
    a = F32(0.05)
    got = v.clone().addcmul_(g, g, value=0.05).numpy()
    assert (_bits(got) != _bits(_fma(a * gn, gn, vn))).sum() == 0
    assert (_bits(got) != _bits(vn + (a * gn) * gn)).sum() > n // 100
    assert (_bits(got) != _bits(_fma(np.full(n, a), gn * gn, vn))).sum() > n // 100
    # add(alpha): fma(p, wd, g)
    got = g.add(p, alpha=0.1).numpy()
    assert (_bits(got) != _bits(_fma(pn, np.full(n, F32(0.1)), gn))).sum() == 0
    # addcdiv_: p + (value*m)/den, not fused
    den = (v.sqrt() / 0.3).add_(1e-8)
    s = F32(-2.5e-3)
    got = p.clone().addcdiv_(m, den, value=-2.5e-3).numpy()
    assert (_bits(got) != _bits(pn + (s * mn) / den.numpy())).sum() == 0
    assert (_bits(got) != _bits(pn + s * (mn / den.numpy()))).sum() > n // 100
    # mul_ by a Python scalar: plain product with the scalar rounded to binary32
    got = p.clone().mul_(1 - 3e-4 * 0.1).numpy()
    assert (_bits(got) != _bits(pn * F32(1 - 3e-4 * 0.1))).sum() == 0


# ----------------------------------------------------------- one step vs torch's ops --
@pytest.mark.parametrize("decoupled", [True, False])
@pytest.mark.parametrize("beta1", [0.9, 0.3])
@pytest.mark.parametrize("step", [1, 7, 1000])
def test_step_matches_torch_op_sequence(decoupled, beta1, step):
    n = 100_003
    hp = dict(HP, beta1=beta1)
    p, g, m, v = _state(n, 2 + step)
    tp, tm, tv = p.clone(), m.clone(), v.clone()
    torch_ops.adam_step_torch_ops(tp, g.clone(), tm, tv, step=step, decoupled=decoupled, **hp)
    op, og, om, ov = p.clone(), g.clone(), m.clone(), v.clone()
    out16 = torch.empty(n, dtype=torch.bfloat16)
    cref.adamw_step(op, og, om, ov, out16, step=step, decoupled=decoupled, **hp)
    assert_bits_equal(om, tm, "exp_avg")
    assert_bits_equal(ov, tv, "exp_avg_sq")
    _param_agreement(op, tp, p)
    assert_bits_equal(out16, op.bfloat16(), "16-bit copy of the updated parameters")
    assert_bits_equal(og, g, "gradient untouched without zero_grad")


@pytest.mark.parametrize("foreach", [False, True])
@pytest.mark.parametrize("cls", [torch.optim.AdamW, torch.optim.Adam])
def test_five_steps_match_torch_optim(cls, foreach):
    n = 50_001
    p0, _, _, _ = _state(n, 11)
    param = torch.nn.Parameter(p0.clone())
    opt = cls([param], lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]), eps=HP["eps"],
              weight_decay=HP["weight_decay"], foreach=foreach)
    op, om, ov = p0.clone(), torch.zeros(n), torch.zeros(n)
    gen = torch.Generator().manual_seed(12)
    for step in range(1, 6):
        grad = torch.randn(n, generator=gen) * 1e-3
        param.grad = grad.clone()
        opt.step()
        cref.adamw_step(op, grad.clone(), om, ov, None, step=step, decoupled=cls is torch.optim.AdamW, **HP)
        st = opt.state[param]
        if cls is torch.optim.AdamW:  # the moments depend on the gradient only
            assert_bits_equal(om, st["exp_avg"], f"exp_avg step {step}")
            assert_bits_equal(ov, st["exp_avg_sq"], f"exp_avg_sq step {step}")
        _param_agreement(op, param.detach(), p0, steps=step)


def test_step_against_binary64_and_closed_forms():
    n = 20_000
    p, g, m, v = _state(n, 21)
    hp = dict(HP)
    step = 3
    op, om, ov = p.clone(), m.clone(), v.clone()
    cref.adamw_step(op, g.clone(), om, ov, None, step=step, **hp)
    P, G, M, V = (x.double() for x in (p, g, m, v))
    P = P * (1 - hp["lr"] * hp["weight_decay"])
    M = M + (1 - hp["beta1"]) * (G - M)
    V = V * hp["beta2"] + (1 - hp["beta2"]) * G * G
    den = V.sqrt() / math.sqrt(1 - hp["beta2"] ** step) + hp["eps"]
    P = P - hp["lr"] / (1 - hp["beta1"] ** step) * M / den
    assert torch.allclose(om.double(), M, rtol=3e-7, atol=1e-9)
    assert torch.allclose(ov.double(), V, rtol=3e-7, atol=1e-12)
    assert torch.allclose(op.double(), P, rtol=3e-7, atol=1e-8)
    # first step from zero moments, |g| >> eps: the update is -lr * sign(g)
    p1, m1, v1 = p.clone(), torch.zeros(n), torch.zeros(n)
    big = torch.where(g.abs() < 1e-4, torch.full_like(g, 1e-3), g)
    cref.adamw_step(p1, big.clone(), m1, v1, None, step=1, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0)
    assert torch.allclose(p1 - p, -1e-3 * big.sign(), rtol=1e-3, atol=1e-9)
    # zero learning rate and no decay: parameters unchanged bit for bit, moments still move
    p2, m2, v2 = p.clone(), m.clone(), v.clone()
    cref.adamw_step(p2, g.clone(), m2, v2, None, step=2, lr=0.0, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.0)
    assert_bits_equal(p2, p, "lr = 0")
    assert not torch.equal(m2, m)
    # all-zero state and gradient (pad lanes): everything stays zero
    z = [torch.zeros(64) for _ in range(4)]
    cref.adamw_step(z[0], z[1], z[2], z[3], None, step=1, **hp)
    assert all(torch.equal(t, torch.zeros(64)) for t in z)
    # gradient scale == a preceding grad.mul_(scale); zero_grad clears the gradient
    p3, g3, m3, v3 = p.clone(), g.clone(), m.clone(), v.clone()
    cref.adamw_step(p3, g3, m3, v3, None, step=4, grad_scale=0.37, zero_grad=True, **hp)
    p4, m4, v4 = p.clone(), m.clone(), v.clone()
    cref.adamw_step(p4, g.clone().mul_(torch.tensor(0.37)), m4, v4, None, step=4, **hp)
    assert_bits_equal(p3, p4, "grad_scale"), assert_bits_equal(m3, m4, "grad_scale m"), assert_bits_equal(v3, v4, "v")
    assert torch.equal(g3, torch.zeros(n))


# ------------------------------------------------------------------ norm and clipping --
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_sumsq_exact_on_small_inputs(dtype):
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(4097, generator=g) * 3e-2).to(dtype)
    exact = math.fsum(float(t) ** 2 for t in x.float().tolist())
    got = cref.sumsq(x)
    assert abs(got - exact) <= 1e-13 * exact
    assert cref.sumsq(x[:0]) == 0.0


@pytest.mark.parametrize("max_norm", [0.5, 1.0, 1e6])
def test_clip_matches_the_reference_op_sequence(max_norm):
    g = torch.Generator().manual_seed(32)
    bufs = [torch.randn(70_001, generator=g) * 1e-2, (torch.randn(513, generator=g) * 0.1)]
    want = [b.clone() for b in bufs]
    total = torch_ops.clip_grad_norm_(want, max_norm)
    norm, coef = cref.clip_coef(sum(cref.sumsq(b) for b in bufs), max_norm)
    # torch sums in binary32 in an order of its choosing; the oracle's norm is the exact one rounded
    assert abs(norm - float(total)) <= 2e-6 * norm
    exact = math.sqrt(math.fsum(float(t) ** 2 for b in bufs for t in b.tolist()))
    assert abs(norm - exact) <= 6e-8 * exact
    assert coef == min(np.float32(max_norm) / (np.float32(norm) + np.float32(1e-6)), np.float32(1.0))
    got = [b.clone() for b in bufs]
    for b in got:
        cref.flat_scale(b, coef)
    for a, b in zip(got, want):
        assert torch.allclose(a, b, rtol=3e-6, atol=0)
    if max_norm == 1e6:  # no clipping: coefficient exactly 1, buffers untouched
        assert coef == 1.0
        for a, b in zip(got, bufs):
            assert_bits_equal(a, b, "coef 1")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_scale_is_torch_mul_by_a_float32_scalar_tensor(dtype):
    g = torch.Generator().manual_seed(33)
    x = (torch.randn(10_001, generator=g) * 1e-2).to(dtype)
    c = torch.tensor(0.7334219)
    want = x.clone().mul_(c)
    got = x.clone()
    cref.flat_scale(got, float(c))
    assert_bits_equal(got, want, "scale")


def test_clip_coef_keeps_nan():
    norm, coef = cref.clip_coef(float("nan"), 1.0)
    assert math.isnan(norm) and math.isnan(coef)
    norm, coef = cref.clip_coef(0.0, 1.0)
    assert norm == 0.0 and coef == 1.0
