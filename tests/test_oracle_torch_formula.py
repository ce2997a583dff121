"""Pins the oracle's restatement of the reference's torch-formula branch
(oracle.torch_formula_update / oracle_torch_adam_span).

The branch (patrickstar/ops/fp16_cpu_adam.py:245-277, reached from :429-443 for optimizer state
held in GPU memory) delegates all arithmetic to PyTorch's element-wise kernels.  PyTorch is here,
so the strongest pin is PyTorch itself: `reference_call_sequence` below issues the very calls of
those lines on torch tensors, and the oracle (plain C, one rounding step per torch kernel) has
to reproduce the result.  On CPU tensors torch rounds two of the kernels differently from its
GPU kernels (`x / python_scalar` is a true division on the CPU and a multiplication by the
reciprocal on the GPU; the CPU's vectorised addcdiv associates as (value * b) / c), so the bar
here is an ulp of m and v and a bound of 1e-5 * lr on the parameter; the bit-for-bit comparison against
torch's GPU kernels, which are what the branch really runs on, is in
tests/test_gpu_torch_arithmetic.py.  Independent checks: torch.optim.Adam / AdamW, the textbook
recurrences in float64, first-step closed forms, and the invariants of a zero-padded tail.
"""
import math

import numpy as np
import pytest
import torch

import oracle


def reference_call_sequence(data, grad16, exp_avg, exp_avg_sq, step, lr, beta1, beta2, eps, weight_decay,
                            use_adamw, loss_scale, gradient_clipping=-1):
    """The calls of fp16_chunk_adam_ops (:364-379 GPU branch, :412-413, :430) and
    torch_adam_update (:259-277) on torch tensors, in place on data / exp_avg / exp_avg_sq."""
    if gradient_clipping > 0:
        max_fp16 = torch.finfo(torch.half).max
        if loss_scale is not None:
            gradient_clipping *= loss_scale
        gradient_clipping = min(max_fp16, gradient_clipping)
        grad16 = grad16.clone().clamp_(-gradient_clipping, gradient_clipping)
    bias_correction1 = 1 - beta1**step
    bias_correction2 = 1 - beta2**step
    grad = grad16.float()
    if loss_scale is not None:
        grad.div_(loss_scale)
    if weight_decay != 0:
        if use_adamw:
            data.mul_(1 - lr * weight_decay)
        else:
            grad = grad.add(data, alpha=weight_decay)
    exp_avg.mul_(beta1).add_(grad, alpha=1 - beta1)
    exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    denom = (exp_avg_sq.sqrt() / math.sqrt(bias_correction2)).add_(eps)
    step_size = lr / bias_correction1
    data.addcdiv_(exp_avg, denom, value=-step_size)


def _state(n, seed, scale, history=True):
    r = np.random.default_rng(seed)
    p = r.normal(0, 0.02, n).astype(np.float32)
    g = (r.normal(0, 1e-3, n) * scale).astype(np.float16)
    m = r.normal(0, 1e-4, n).astype(np.float32) if history else np.zeros(n, np.float32)
    v = np.abs(r.normal(0, 1e-6, n)).astype(np.float32) if history else np.zeros(n, np.float32)
    return p, g, m, v


def _ulps(a, b):
    """Distance in units of the last place between two float32 arrays of equal sign pattern."""
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia)
    ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    return np.abs(ia - ib)


CASES = [
    # step, lr, betas, eps, wd, adamw, loss_scale
    (1, 1e-3, (0.9, 0.999), 1e-6, 0.0, False, 8),
    (100, 1e-4, (0.9, 0.999), 1e-8, 0.01, True, 2**16),
    (100, 1e-4, (0.9, 0.999), 1e-8, 0.01, False, 2**12),
    (7, 3e-4, (0.8, 0.95), 1e-8, 0.1, True, None),
    (2500, 1e-3, (0.9, 0.98), 1e-9, 0.0, True, 4096.0),
    (13, 1e-3, (0.9, 0.999), 1e-8, 0.01, True, 1000.0),  # a scale that is not a power of two
]


@pytest.mark.parametrize("case", CASES)
def test_against_the_literal_torch_calls(case):
    step, lr, (b1, b2), eps, wd, adamw, scale = case
    n = 4096 + 37
    p, g, m, v = _state(n, step, scale or 1.0, history=step > 1)
    po, mo, vo = p.copy(), m.copy(), v.copy()
    oracle.torch_formula_update(po, g, mo, vo, step, lr, b1, b2, eps, wd, adamw, scale)
    tp, tm, tv = (torch.from_numpy(x.copy()) for x in (p, m, v))
    reference_call_sequence(tp, torch.from_numpy(g.copy()), tm, tv, step, lr, b1, b2, eps, wd, adamw, scale)
    # m and v: mul + one fused multiply-add; identical unless the scale is not a power of two, where
    # the CPU kernel's true division puts g (and so g*g) an ulp away
    pow2 = scale is None or math.log2(scale) == int(math.log2(scale))
    if pow2:
        assert _ulps(mo, tm.numpy()).max() <= 1
        assert _ulps(vo, tv.numpy()).max() <= 1
    else:
        np.testing.assert_allclose(mo, tm.numpy(), rtol=1e-6, atol=1e-10)  # m ~ 1e-4: a few of its ulps
        np.testing.assert_allclose(vo, tv.numpy(), rtol=1e-6, atol=1e-14)
    # the update term is O(lr): an ulp or two of the quotient moves p by ~1e-7 * lr, usually below p's own ulp
    np.testing.assert_allclose(po, tp.numpy(), rtol=1.2e-7, atol=1e-5 * lr)


@pytest.mark.parametrize("adamw", [False, True])
def test_against_torch_optim(adamw):
    n, lr, b1, b2, eps, wd = 2048, 1e-3, 0.9, 0.999, 1e-8, 0.01
    p, g16, m, v = _state(n, 5, 1.0)
    step = 11
    po, mo, vo = p.copy(), m.copy(), v.copy()
    oracle.torch_formula_update(po, g16, mo, vo, step, lr, b1, b2, eps, wd, adamw, None)
    param = torch.nn.Parameter(torch.from_numpy(p.copy()))
    opt = (torch.optim.AdamW if adamw else torch.optim.Adam)([param], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd)
    param.grad = torch.from_numpy(g16.astype(np.float32))
    opt.state[param] = {
        "step": torch.tensor(float(step - 1)),
        "exp_avg": torch.from_numpy(m.copy()),
        "exp_avg_sq": torch.from_numpy(v.copy()),
    }
    opt.step()
    np.testing.assert_allclose(po, param.detach().numpy(), rtol=2e-6, atol=2e-9)
    np.testing.assert_allclose(mo, opt.state[param]["exp_avg"].numpy(), rtol=2e-6, atol=1e-10)
    np.testing.assert_allclose(vo, opt.state[param]["exp_avg_sq"].numpy(), rtol=2e-6, atol=1e-14)


@pytest.mark.parametrize("adamw", [False, True])
def test_against_textbook_float64(adamw):
    n, lr, b1, b2, eps, wd, step, scale = 3000, 1e-3, 0.9, 0.999, 1e-8, 0.01, 40, 1024
    p, g16, m, v = _state(n, 9, scale)
    po, mo, vo = p.copy(), m.copy(), v.copy()
    oracle.torch_formula_update(po, g16, mo, vo, step, lr, b1, b2, eps, wd, adamw, scale)
    P, G, M, V = (x.astype(np.float64) for x in (p, g16, m, v))
    G = G / scale
    if adamw:
        P = P * (1 - lr * wd)
    else:
        G = G + wd * P
    M = b1 * M + (1 - b1) * G
    V = b2 * V + (1 - b2) * G * G
    P = P - lr / (1 - b1**step) * M / (np.sqrt(V) / math.sqrt(1 - b2**step) + eps)
    np.testing.assert_allclose(po, P, rtol=1e-6, atol=1e-9)
    np.testing.assert_allclose(mo, M, rtol=1e-6, atol=1e-10)
    np.testing.assert_allclose(vo, V, rtol=1e-6, atol=1e-14)


def test_first_step_closed_forms():
    """From m = v = 0 without decay: m' = (1-b1) g and v' = (1-b2) g^2 exactly (one rounding each),
    and p' = p - lr * g / (|g| + eps) to float accuracy."""
    n, lr, b1, b2, eps = 1000, 1e-3, 0.9, 0.999, 1e-6
    p, g16, m, v = _state(n, 3, 8.0, history=False)
    po, mo, vo = p.copy(), m.copy(), v.copy()
    oracle.torch_formula_update(po, g16, mo, vo, 1, lr, b1, b2, eps, 0.0, False, 8)
    g = g16.astype(np.float32) * np.float32(1.0 / 8)
    np.testing.assert_array_equal(mo, np.float32(1 - b1) * g)
    np.testing.assert_array_equal(vo, np.float32(1 - b2) * (g * g))
    G = g.astype(np.float64)
    expect = p - lr * G / (np.abs(G) + eps)  # m'/bc1 = g and sqrt(v')/sqrt(bc2) = |g| at step 1
    np.testing.assert_allclose(po, expect, rtol=2e-6, atol=1e-9)


def test_zero_padding_stays_zero_and_decay_is_a_plain_product():
    z = np.zeros(64, np.float32)
    for adamw in (False, True):
        p, m, v = z.copy(), z.copy(), z.copy()
        oracle.torch_formula_update(p, np.zeros(64, np.float16), m, v, 5, 1e-3, 0.9, 0.999, 1e-8, 0.01, adamw, 2**10)
        assert not p.any() and not m.any() and not v.any()
    # decoupled decay with a zero gradient and zero moments: p' = p * float(1 - lr*wd), nothing else
    p = np.linspace(-1, 1, 64).astype(np.float32)
    q = p.copy()
    oracle.torch_formula_update(q, np.zeros(64, np.float16), z.copy(), z.copy(), 5, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, None)
    np.testing.assert_array_equal(q, p * np.float32(1 - 1e-3 * 0.01))


def test_differs_from_the_operator_by_its_float_constants():
    """Same inputs through both arithmetics of the reference.  The operator forms 1 - beta in float
    (1.0f - 0.999f = 0.0010000467, 4.7e-5 above float(1 - 0.999)) where the torch formula narrows
    the Python double, so the second moment differs by up to that relative amount and the
    parameter by a fraction of it: close, but far from bit-equal."""
    n, step, lr, b1, b2, eps, wd, scale = 1 << 14, 100, 1e-4, 0.9, 0.999, 1e-8, 0.01, 2**12
    p, g16, m, v = _state(n, 21, scale)
    pt, mt, vt = p.copy(), m.copy(), v.copy()
    oracle.torch_formula_update(pt, g16, mt, vt, step, lr, b1, b2, eps, wd, True, scale)
    o = oracle.AdamOracle(lr, b1, b2, eps, wd, True)
    po, mo, vo = p.copy(), m.copy(), v.copy()
    o.update(step, lr, b1, b2, eps, wd, True, po, g16, mo, vo, float(scale))
    np.testing.assert_allclose(pt, po, rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(mt, mo, rtol=1e-6, atol=1e-10)
    np.testing.assert_allclose(vt, vo, rtol=5e-5, atol=1e-14)
    assert np.float32(1.0) - np.float32(0.999) != np.float32(1 - 0.999)
    assert (mt.view(np.uint32) != mo.view(np.uint32)).mean() > 0.1
    assert (vt.view(np.uint32) != vo.view(np.uint32)).mean() > 0.1


def test_clamp_bound_and_order():
    """The clamp acts on the fp16 gradient before the unscale, with the bound narrowed to fp16."""
    n, scale, clip = 4096, 1024, 0.0017
    p, g16, m, v = _state(n, 33, scale * 2.0)
    bound = np.float16(np.float32(min(65504.0, clip * scale)))
    assert (np.abs(g16) > bound).mean() > 0.05
    a = [x.copy() for x in (p, m, v)]
    oracle.torch_formula_update(a[0], g16, a[1], a[2], 3, 1e-3, 0.9, 0.999, 1e-8, 0.0, False, scale, gradient_clipping=clip)
    b = [x.copy() for x in (p, m, v)]
    oracle.torch_formula_update(b[0], np.clip(g16, -bound, bound), b[1], b[2], 3, 1e-3, 0.9, 0.999, 1e-8, 0.0, False, scale)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x, y)
    tp, tm, tv = (torch.from_numpy(x.copy()) for x in (p, m, v))
    reference_call_sequence(tp, torch.from_numpy(g16.copy()), tm, tv, 3, 1e-3, 0.9, 0.999, 1e-8, 0.0, False, scale, clip)
    assert _ulps(a[1], tm.numpy()).max() <= 1
    np.testing.assert_allclose(a[0], tp.numpy(), rtol=1.2e-7, atol=1e-8)


def test_step_oracle_takes_the_torch_branch():
    chunks = []
    for s in range(2):
        p, g16, m, v = _state(512, 40 + s, 16.0, history=False)
        chunks.append({"p32": p, "m": m, "v": v, "p16": g16})
    ref = [{k: x.copy() for k, x in c.items()} for c in chunks]
    opt = oracle.OptimizerStepOracle(chunks, oracle.StaticScalerOracle(16), lr=1e-3, weight_decay=0.01, use_adamw=True,
                                     arithmetic="torch")
    assert opt.step() is False and opt.step_count == 1
    for c, r in zip(chunks, ref):
        oracle.torch_formula_update(r["p32"], r["p16"], r["m"], r["v"], 1, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, 16)
        np.testing.assert_array_equal(c["p32"], r["p32"])
        np.testing.assert_array_equal(c["p16"], oracle.cast_fp32_to_fp16(r["p32"]))
