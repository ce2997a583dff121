"""Pins the CPU oracle of the Adam arithmetic (oracle/adam_oracle.c).

The reference holds no golden vectors for this path (its only numeric check,
unitest/test_ds_cpu_adam.py:141-155, is "within 1e-4 absolute of a torch
formula on unseeded inputs"), so the oracle is pinned against
  * a library routine: torch.optim.Adam / torch.optim.AdamW single steps,
  * the textbook recurrences evaluated in float64,
  * closed forms of the first step,
  * invariants (zero padding, power-of-two scales, permutation, code paths),
chosen so that a dropped term, a wrong sign or a swapped beta fails.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import AdamOracle

RNG = np.random.default_rng(1234)


def F32(x):
    """The double that a C float parameter holds after pybind narrows a Python float."""
    return float(np.float32(x))


def _isas():
    out = [oracle.ISA_SCALAR]
    probe = AdamOracle()
    z = np.zeros(16, dtype=np.float32)
    for isa in (oracle.ISA_AVX2, oracle.ISA_AVX512):
        try:
            probe.update(1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, z.copy(), z.copy(), z.copy(), z.copy(), -1.0, isa)
            out.append(isa)
        except RuntimeError:
            pass
    return out


ISAS = _isas()


def _state(n, with_history=True, seed=0):
    r = np.random.default_rng(seed)
    p = r.normal(0, 0.02, n).astype(np.float32)
    g = r.normal(0, 1e-3, n).astype(np.float32)
    if with_history:
        m = r.normal(0, 1e-4, n).astype(np.float32)
        v = np.abs(r.normal(0, 1e-6, n)).astype(np.float32)
    else:
        m = np.zeros(n, np.float32)
        v = np.zeros(n, np.float32)
    return p, g, m, v


def _textbook_f64(p, g, m, v, step, lr, b1, b2, eps, wd, adamw):
    """Kingma & Ba recurrences (L2 form) / Loshchilov & Hutter (decoupled), in float64."""
    p, g, m, v = (x.astype(np.float64) for x in (p, g, m, v))
    if wd and not adamw:
        g = g + wd * p
    m = b1 * m + (1 - b1) * g
    v = b2 * v + (1 - b2) * g * g
    mhat = m / (1 - b1**step)
    denom = np.sqrt(v) / math.sqrt(1 - b2**step) + eps
    if wd and adamw:
        p = p * (1 - lr * wd)
    p = p - lr * mhat / denom
    return p, m, v


@pytest.mark.parametrize("adamw", [False, True])
@pytest.mark.parametrize("wd", [0.0, 0.01])
@pytest.mark.parametrize("step", [1, 2, 100])
def test_matches_torch_optim(adamw, wd, step):
    n = 4099
    p, g, m, v = _state(n, with_history=step > 1, seed=step)
    # the native operator receives its betas as C floats: compare against the library fed the same values
    lr, b1, b2, eps = 1e-3, F32(0.9), F32(0.999), 1e-8

    tp = torch.nn.Parameter(torch.from_numpy(p.copy()))
    cls = torch.optim.AdamW if adamw else torch.optim.Adam
    opt = cls([tp], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd, foreach=False)
    tp.grad = torch.from_numpy(g.copy())
    if step > 1:
        opt.state[tp]["step"] = torch.tensor(float(step - 1))
        opt.state[tp]["exp_avg"] = torch.from_numpy(m.copy())
        opt.state[tp]["exp_avg_sq"] = torch.from_numpy(v.copy())
    opt.step()

    o = AdamOracle(lr, b1, b2, eps, wd, adamw)
    po, mo, vo = p.copy(), m.copy(), v.copy()
    o.update(step, lr, b1, b2, eps, wd, True, po, g, mo, vo, -1.0)

    np.testing.assert_allclose(mo, opt.state[tp]["exp_avg"].numpy(), rtol=2e-6, atol=1e-10)  # m can cancel: atol = 1e-6 of its scale
    np.testing.assert_allclose(vo, opt.state[tp]["exp_avg_sq"].numpy(), rtol=2e-6, atol=1e-18)
    np.testing.assert_allclose(po, tp.detach().numpy(), rtol=2e-6, atol=2e-9)


@pytest.mark.parametrize("adamw,wd", [(False, 0.0), (False, 0.001), (True, 0.001), (True, 0.01)])
@pytest.mark.parametrize("step", [1, 7, 100, 5000])
@pytest.mark.parametrize("half_scale", [None, 32.0, 2.0**12])
def test_matches_float64_textbook(adamw, wd, step, half_scale):
    n = 1023
    p, g, m, v = _state(n, with_history=step > 1, seed=step + 17)
    lr, b1, b2, eps = 0.01, F32(0.9), F32(0.999), 1e-8
    if half_scale is None:
        grads, scale, g_true = g, -1.0, g
    else:
        grads = (g * half_scale).astype(np.float16)
        scale = half_scale
        g_true = grads.astype(np.float32) / np.float32(half_scale)
    pr, mr, vr = _textbook_f64(p, g_true, m, v, step, lr, b1, b2, eps, wd, adamw)
    o = AdamOracle(lr, b1, b2, eps, wd, adamw)
    po, mo, vo = p.copy(), m.copy(), v.copy()
    o.update(step, lr, b1, b2, eps, wd, True, po, grads, mo, vo, scale)
    # float32 evaluation of a ~10-op chain: a few ulp.  m can cancel, hence the atol.
    np.testing.assert_allclose(mo, mr, rtol=1e-6, atol=1e-10)
    np.testing.assert_allclose(vo, vr, rtol=1e-6, atol=1e-16)
    # bias-correction scalars are float32 in the reference: relative error of
    # 1-beta2^t at t=1 is ~6e-5 (beta2 rounded to float32), which carries into p's increment.
    np.testing.assert_allclose(po - p, pr - p.astype(np.float64), rtol=2e-4, atol=5e-9)  # atol: half an ulp of p (|p| < 0.125)
    np.testing.assert_allclose(po, pr, rtol=1e-5, atol=1e-7)


def test_first_step_closed_forms():
    """m=v=0, wd=0, t=1: m' = (1-b1) g, v' = (1-b2) g^2, p' = p - lr*g/(|g| + eps) (to float32 accuracy),
    and exactly: sign(p'-p) = -sign(g), |p'-p| <= lr."""
    n = 2048
    p, g, m, v = _state(n, with_history=False, seed=5)
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-6
    o = AdamOracle(lr, b1, b2, eps, 0.0, False)
    po, mo, vo = p.copy(), m.copy(), v.copy()
    o.update(1, lr, b1, b2, eps, 0.0, True, po, g, mo, vo, -1.0)
    b1m = np.float32(1.0) - np.float32(b1)
    b2m = np.float32(1.0) - np.float32(b2)
    # with m=v=0 the fused ops have an exact zero addend: results are single roundings
    assert np.array_equal(mo, g * b1m)
    assert np.array_equal(vo, (g * g) * b2m)
    big = np.abs(g) > 1e-4
    d = po.astype(np.float64) - p
    assert np.all(np.sign(d[big]) == -np.sign(g[big]))
    assert np.all(np.abs(d) <= lr * (1 + 1e-5))
    expect = -lr * g.astype(np.float64) / (np.abs(g.astype(np.float64)) + eps)  # mhat = g, sqrt(vhat) = |g| at t = 1
    np.testing.assert_allclose(d[big], expect[big], rtol=1e-4, atol=5e-9)  # float32 bc scalars: 6e-5 rel; half an ulp of p


def test_zero_padding_invariants():
    """The unused tail of a chunk holds zeros in all four lists and must stay so
    (L2, or no decay); under decoupled decay p' = p*(1 - lr*wd) exactly as fma(p, -lr*wd, p)."""
    n = 64
    z = np.zeros(n, np.float32)
    for adamw, wd in [(False, 0.0), (False, 0.01), (True, 0.01)]:
        o = AdamOracle(1e-4, 0.9, 0.999, 1e-8, wd, adamw)
        p, m, v = z.copy(), z.copy(), z.copy()
        o.update(100, 1e-4, 0.9, 0.999, 1e-8, wd, True, p, np.zeros(n, np.float16), m, v, 65536.0)
        assert not p.any() and not m.any() and not v.any()
    p0 = RNG.normal(0, 0.02, n).astype(np.float32)
    p = p0.copy()
    o = AdamOracle(1e-4, 0.9, 0.999, 1e-8, 0.01, True)
    m, v = z.copy(), z.copy()
    o.update(3, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, p, z.copy(), m, v, -1.0)
    wdec = np.float32(-1e-4) * np.float32(0.01)
    expect = (p0.astype(np.float64) * np.float64(wdec) + p0.astype(np.float64)).astype(np.float32)
    assert np.array_equal(p, expect)
    assert not m.any() and not v.any()


@pytest.mark.parametrize("k", [3, 12, 16])
def test_power_of_two_scale_is_exact(k):
    """(g*2^k as fp16, scale 2^k) is bit-identical to (g as fp16 -> fp32, no scale) while nothing overflows."""
    n = 4096
    p, g, m, v = _state(n, seed=k)
    g16 = g.astype(np.float16)
    scaled = (g16.astype(np.float32) * np.float32(2.0**k)).astype(np.float16)
    assert np.isfinite(scaled).all()
    a = [x.copy() for x in (p, m, v)]
    b = [x.copy() for x in (p, m, v)]
    AdamOracle(1e-4, 0.9, 0.999, 1e-8, 0.01, True).update(100, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, a[0], scaled, a[1], a[2], 2.0**k)
    AdamOracle(1e-4, 0.9, 0.999, 1e-8, 0.01, True).update(100, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, b[0], g16.astype(np.float32), b[1], b[2], -1.0)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)


def test_scale_must_divide_not_multiply():
    n = 256
    p, g, m, v = _state(n, seed=9)
    a = [x.copy() for x in (p, m, v)]
    b = [x.copy() for x in (p, m, v)]
    AdamOracle().update(1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, a[0], g * 8, a[1], a[2], 8.0)
    AdamOracle().update(1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, b[0], g, b[1], b[2], -1.0)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)
    # scale <= 0 means "do not unscale" (cpu_adam.cpp:101)
    c = [x.copy() for x in (p, m, v)]
    AdamOracle().update(1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, c[0], g, c[1], c[2], 0.0)
    for x, y in zip(c, b):
        assert np.array_equal(x, y)


def test_code_paths_bit_identical_and_permutation_equivariant():
    n = 16384 * 3 + 77  # crosses work-item boundaries and leaves a vector remainder
    p, g, m, v = _state(n, seed=3)
    g16 = (g * 4096).astype(np.float16)
    results = []
    for isa in ISAS:
        po, mo, vo = p.copy(), m.copy(), v.copy()
        took = AdamOracle(1e-4, 0.9, 0.999, 1e-8, 0.01, True).update(100, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, po, g16, mo, vo, 4096.0, isa)
        assert took == isa
        results.append((po, mo, vo))
    for r in results[1:]:
        for x, y in zip(results[0], r):
            assert np.array_equal(x, y)
    perm = RNG.permutation(n)
    po, mo, vo = p[perm].copy(), m[perm].copy(), v[perm].copy()
    AdamOracle(1e-4, 0.9, 0.999, 1e-8, 0.01, True).update(100, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, po, g16[perm].copy(), mo, vo, 4096.0)
    for x, y in zip(results[0], (po, mo, vo)):
        assert np.array_equal(x[perm], y)


def test_beta_power_state_machine():
    """cpu_adam.h:143-162: consecutive steps multiply in float32; a jump or a beta change uses pow()."""
    b1, b2 = np.float32(0.9), np.float32(0.999)
    o = AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.0, False)
    run1, run2 = np.float32(1.0), np.float32(1.0)
    for t in range(1, 11):
        o.advance(t, 0.9, 0.999)
        o.set(1e-3, 1e-8, 0.0, True)
        run1 = np.float32(run1 * b1)
        run2 = np.float32(run2 * b2)
        c = o.consts()
        bc1 = np.float32(1.0) - run1
        assert c[5] == bc1
        assert c[2] == np.float32(1.0) / np.sqrt(np.float32(1.0) - run2, dtype=np.float32)
        assert c[3] == np.float32(-1e-3) / bc1
    # the running product is NOT what pow gives at t=10 for beta1 (float32 drift): the branch matters
    cold = AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.0, False)
    cold.advance(100, 0.9, 0.999)
    cold.set(1e-3, 1e-8, 0.0, True)
    p1 = np.float32(math.pow(float(b1), 100.0))
    p2 = np.float32(math.pow(float(b2), 100.0))
    c = cold.consts()
    assert c[5] == np.float32(1.0) - p1
    assert c[2] == np.float32(1.0) / np.sqrt(np.float32(1.0) - p2, dtype=np.float32)
    # then 101 continues by multiplication from the pow value
    cold.advance(101, 0.9, 0.999)
    cold.set(1e-3, 1e-8, 0.0, True)
    assert cold.consts()[5] == np.float32(1.0) - np.float32(p1 * b1)
    # same step number again (a second tensor of the same step in the reference's per-tensor loop): pow branch
    cold.advance(101, 0.9, 0.999)
    cold.set(1e-3, 1e-8, 0.0, True)
    assert cold.consts()[5] == np.float32(1.0) - np.float32(math.pow(float(b1), 101.0))
    # beta change: pow with the new betas
    cold.advance(102, 0.8, 0.99)
    cold.set(1e-3, 1e-8, 0.0, True)
    assert cold.consts()[5] == np.float32(1.0) - np.float32(math.pow(float(np.float32(0.8)), 102.0))
    # bias_correction off
    cold.set(1e-3, 1e-8, 0.0, False)
    c = cold.consts()
    assert c[5] == 1.0 and c[2] == 1.0 and c[3] == np.float32(-1e-3)
    # 1 - beta as float32 differs from float32(0.1): the constant is computed in float32
    assert c[0] == np.float32(1.0) - np.float32(0.8)
    assert AdamOracle(1e-3, 0.9, 0.999).consts()[0] != np.float32(0.1)


def test_fp16_cast_is_rne_everywhere():
    L = oracle.lib()
    # every fp16 value, its fp32 image, the fp32 neighbours and the midpoints between adjacent fp16 values
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
    f = h.astype(np.float32)
    for i in range(0, 65536, 257):
        assert L.oracle_f16_to_f32(int(h.view(np.uint16)[i])) == f[i] or np.isnan(f[i])
    finite = np.isfinite(f)
    cand = [f[finite]]
    bits = f[finite].view(np.uint32)
    cand.append((bits + 1).view(np.float32))
    cand.append((bits - 1).view(np.float32))
    nxt = np.nextafter(h[finite], np.float16(np.inf)).astype(np.float32)
    mid = ((f[finite].astype(np.float64) + nxt.astype(np.float64)) / 2).astype(np.float32)
    cand.append(mid[np.isfinite(mid)])
    mb = mid[np.isfinite(mid)].view(np.uint32)
    cand.append((mb + 1).view(np.float32))
    cand.append((mb - 1).view(np.float32))
    cand.append(np.array([65519.99, 65520.0, 65520.01, 7e4, 1e38, np.inf, -np.inf, 2.0**-25, 2.0**-25 * 1.0001, 2.0**-24 * 1.5, 0.0, -0.0, 1e-45], np.float32))
    cand.append(RNG.normal(0, 1, 200000).astype(np.float32) * np.float32(10.0) ** RNG.integers(-9, 5, 200000).astype(np.float32))
    x = np.concatenate(cand).astype(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    got = oracle.cast_fp32_to_fp16(np.ascontiguousarray(x))
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    nan = oracle.cast_fp32_to_fp16(np.array([np.nan, -np.nan], np.float32))
    assert np.isnan(nan).all()


def test_has_inf_or_nan_forms_agree():
    for n in (1, 7, 1000):
        x = RNG.normal(0, 100, n).astype(np.float16)
        assert not oracle.has_inf_or_nan(x)
        for bad in (np.inf, -np.inf, np.nan):
            y = x.copy()
            y[RNG.integers(0, n)] = bad
            assert oracle.has_inf_or_nan(y)
            assert oracle.has_inf_or_nan(y.astype(np.float32))  # the float32-sum form
    both = np.zeros(8, np.float16)
    both[1], both[5] = np.inf, -np.inf  # sums to NaN: still an overflow
    assert oracle.has_inf_or_nan(both) and oracle.has_inf_or_nan(both.astype(np.float32))
    big = np.full(4096, 65504.0, np.float16)  # finite elements, finite float32 sum
    assert not oracle.has_inf_or_nan(big) and not oracle.has_inf_or_nan(big.astype(np.float32))
    assert not oracle.has_inf_or_nan(np.zeros(0, np.float16))
