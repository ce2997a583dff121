"""Pins the oracle's restatement of FP16Adam.step's sequencing (patrickstar/ops/fp16_cpu_adam.py:472-628) and of the
element-wise gradient clamp (:364-379) through invariants and a library routine; CPU only."""
import numpy as np
import torch

import oracle


def _chunks(n_chunks=3, n=300, seed=0):
    r = np.random.default_rng(seed)
    out = []
    for _ in range(n_chunks):
        p = r.normal(0, 0.02, n).astype(np.float32)
        out.append({"p32": p, "m": r.normal(0, 1e-4, n).astype(np.float32), "v": np.abs(r.normal(0, 1e-6, n)).astype(np.float32),
                    "p16": (r.normal(0, 1e-3, n) * 256).astype(np.float16)})
    return out


def _copy(chunks):
    return [{k: v.copy() for k, v in c.items()} for c in chunks]


def test_skipped_step_leaves_state_alone_and_restores_fp16():
    cs = _chunks()
    cs[1]["p16"][17] = np.inf
    before = _copy(cs)
    s = oracle.ScalerOracle(init_scale=256, scale_factor=2, scale_window=1000)
    opt = oracle.OptimizerStepOracle(cs, s, lr=1e-3, weight_decay=0.01, use_adamw=True)
    opt.check_overflow()
    assert opt.has_overflow is True
    assert opt.step() is True
    assert opt.step_count == 0 and opt.has_overflow is False
    assert s.loss_scale == 128.0 and s.cur_iter == 1 and s.last_overflow_iter == 0
    for c, b in zip(cs, before):
        for k in ("p32", "m", "v"):
            assert np.array_equal(c[k], b[k])
        assert np.array_equal(c["p16"].view(np.uint16), oracle.cast_fp32_to_fp16(b["p32"]).view(np.uint16))
    # the native object did not see the skipped step: the next clean step is t = 1 by the running product
    for c in cs:
        c["p16"][...] = np.float16(0.25)
    opt.check_overflow()
    assert opt.step() is False and opt.step_count == 1 and s.cur_iter == 2
    assert opt.native.consts()[5] == np.float32(1.0) - np.float32(0.9)


def test_clean_step_equals_one_operator_call_per_chunk_plus_cast():
    cs = _chunks(seed=3)
    ref = _copy(cs)
    s = oracle.StaticScalerOracle(256)
    opt = oracle.OptimizerStepOracle(cs, s, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=False)
    assert opt.step() is False and opt.step_count == 1
    for c, r in zip(cs, ref):
        o = oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.01, False)
        o.update(1, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, r["p32"], r["p16"], r["m"], r["v"], 256.0)
        for k in ("p32", "m", "v"):
            assert np.array_equal(c[k], r[k])
        assert np.array_equal(c["p16"].view(np.uint16), oracle.cast_fp32_to_fp16(r["p32"]).view(np.uint16))
    # no scaler at all: loss_scale -1 (no unscale); inf gradients are not looked at
    cs2 = _chunks(seed=4)
    cs2[0]["p16"][0] = np.inf
    opt2 = oracle.OptimizerStepOracle(cs2, None, lr=1e-3)
    opt2.check_overflow()
    assert opt2.has_overflow is False and opt2.step() is False
    assert np.isnan(cs2[0]["p32"][0]) or np.isinf(cs2[0]["p32"][0]) or cs2[0]["p32"][0] != cs2[0]["p32"][0]


def test_clamp_restatement_equals_tensor_clamp():
    """The reference clamps with Tensor.clamp_(-c, c) on the fp16 gradient tensor, c = min(65504, clipping * loss_scale)."""
    for clipping, scale in [(1.0, 8), (0.3, 1000.0), (0.1, None), (5.0, 2**16), (1.0001, 8)]:
        cs = _chunks(n_chunks=1, n=4000, seed=11)
        bound = min(65504.0, clipping * (scale if scale is not None else 1))
        g = (np.random.default_rng(5).normal(0, bound, 4000)).astype(np.float16)
        g[:3] = [np.inf, -np.inf, np.nan]
        cs[0]["p16"][...] = g
        want = torch.from_numpy(g.copy()).clamp_(-bound, bound).numpy()
        twin = _copy(cs)
        twin[0]["p16"][...] = want
        sc = None if scale is None else oracle.StaticScalerOracle(scale)
        a = oracle.OptimizerStepOracle(cs, sc, lr=1e-3, gradient_clipping=clipping)
        b = oracle.OptimizerStepOracle(twin, sc, lr=1e-3)
        a.step()
        b.step()
        for k in ("p32", "m", "v", "p16"):
            x, y = cs[0][k], twin[0][k]
            nan = np.isnan(x.astype(np.float32))
            assert np.array_equal(nan, np.isnan(y.astype(np.float32)))
            assert np.array_equal(x[~nan], y[~nan]), (clipping, scale, k)
        assert 0 < (np.abs(g[3:].astype(np.float32)) > bound).mean() < 1
