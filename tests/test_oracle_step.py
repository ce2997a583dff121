"""Pins the oracle's restatement of FP16Adam.step's sequencing (patrickstar/ops/fp16_cpu_adam.py:472-628) and of the
element-wise gradient clamp (:364-379) through invariants and a library routine; CPU only."""
import math

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


# ---- the per-tensor call pattern of one step (fp16_cpu_adam.py:336-428 -> cpu_adam.h:143-162) -----------------
#
# The reference calls adam_update once per tensor with the same `step`.  IncrementStep does `_step++` and
# compares: only the first call of a step can continue the running float product; every later call of the
# step finds `_step + 1 != step` and evaluates pow.  Expected values below are built WITHOUT the step-level
# oracle: from math.pow / numpy float32 arithmetic and from fresh single-call operator objects whose branch
# is forced by hand (those branches are pinned in test_oracle_adam.py::test_beta_power_state_machine).

B1, B2 = np.float32(0.9), np.float32(0.999)


def _beta_powers(t, first, single_tensor_history=False):
    """float32 beta^t as IncrementStep leaves it for the first / a later call of step t (steps 1..t-1 all ran)."""
    if first:
        if single_tensor_history:
            r1 = r2 = np.float32(1.0)
            for _ in range(t):
                r1, r2 = np.float32(r1 * B1), np.float32(r2 * B2)
            return r1, r2
        return (np.float32(np.float32(math.pow(float(B1), t - 1)) * B1),
                np.float32(np.float32(math.pow(float(B2), t - 1)) * B2))
    return np.float32(math.pow(float(B1), t)), np.float32(math.pow(float(B2), t))


def _probe_update_f64(g, m, v, lr, eps, b1t, b2t):
    """Textbook Adam on a zero parameter in float64 with the given float32 beta powers: p' = -lr/bc1 * m'/(sqrt(v')*bc2inv + eps)."""
    b1, b2 = float(B1), float(B2)
    m1 = b1 * m + (1.0 - b1) * g
    v1 = b2 * v + (1.0 - b2) * g * g
    bc1 = float(np.float32(1.0) - b1t)
    bc2inv = float(np.float32(1.0) / np.sqrt(np.float32(1.0) - b2t, dtype=np.float32))
    return -(lr / bc1) * m1 / (math.sqrt(v1) * bc2inv + eps)


def _three_tensor_layout():
    # two chunks of 600 elements: tensors at (0, 0, 250), (0, 250, 300), (1, 0, 400); the tails are padding
    return [(0, 0, 250), (0, 250, 300), (1, 0, 400)]


def test_first_tensor_of_a_step_multiplies_and_every_later_tensor_takes_pow():
    lr, eps = 1e-3, 1e-8
    tensors = _three_tensor_layout()
    cs = _chunks(n_chunks=2, n=600, seed=21)
    for c in cs:
        c["p16"][...] = 0
    opt = oracle.OptimizerStepOracle(cs, None, lr=lr, betas=(0.9, 0.999), eps=eps, tensors=tensors)
    rng = np.random.default_rng(22)
    differing = 0
    for t in range(1, 21):
        # element 0 of every tensor is a probe: parameter and moments 0, so the new parameter IS
        # step_size * m'/denominator with no cancellation anywhere
        probes = []
        for ci, off, numel in tensors:
            g = rng.normal(0, 1e-2, numel).astype(np.float16)
            g[0] = np.float16(0.0123)
            cs[ci]["p16"][off : off + numel] = g
            cs[ci]["p32"][off] = cs[ci]["m"][off] = cs[ci]["v"][off] = 0.0
            probes.append((float(g[0]), 0.0, 0.0))
        assert opt.step() is False
        for k, ((ci, off, _), (g, m, v)) in enumerate(zip(tensors, probes)):
            got = float(cs[ci]["p32"][off])
            right = _probe_update_f64(g, m, v, lr, eps, *_beta_powers(t, first=(k == 0)))
            wrong = _probe_update_f64(g, m, v, lr, eps, *_beta_powers(t, first=(k != 0)))
            assert abs(got - right) <= 4e-7 * abs(right), (t, k, got, right)
            if abs(right - wrong) > 2e-6 * abs(right):
                differing += 1
                assert abs(got - wrong) > 1e-6 * abs(right), (t, k, "took the other branch of IncrementStep")
    # the two branches really are different numbers on most early steps (bc2inv differs by up to 1e-5)
    assert differing >= 8


def test_step_oracle_equals_hand_sequenced_operator_calls():
    """Bit-exact: every tensor against a FRESH operator object driven into the branch the reference takes."""
    kw = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    tensors = _three_tensor_layout()
    cs = _chunks(n_chunks=2, n=600, seed=31)
    s = oracle.StaticScalerOracle(64)
    opt = oracle.OptimizerStepOracle(cs, s, tensors=tensors, **kw)
    rng = np.random.default_rng(32)

    def hand(t, k, ref_chunk, off, numel):
        o = oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.01, True)
        if k == 0 and t > 1:
            o.advance(t - 1, 0.9, 0.999)  # a cold call: pow(beta, t-1), as the LAST tensor of step t-1 left it
        elif k > 0:
            o.advance(t, 0.9, 0.999)  # the first tensor of this step came before: _step is already t
        sl = slice(off, off + numel)
        o.update(t, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, ref_chunk["p32"][sl], ref_chunk["p16"][sl],
                 ref_chunk["m"][sl], ref_chunk["v"][sl], 64.0)

    steps = list(range(1, 13))
    for t in steps:
        for c in cs:
            c["p16"][...] = (rng.normal(0, 1e-3, c["p16"].size) * 64).astype(np.float16)
        ref = _copy(cs)
        opt.step()
        for k, (ci, off, numel) in enumerate(tensors):
            hand(t, k, ref[ci], off, numel)
        for c, r in zip(cs, ref):
            for key in ("p32", "m", "v"):
                assert np.array_equal(c[key].view(np.uint32), r[key].view(np.uint32)), (t, key)
            assert np.array_equal(c["p16"].view(np.uint16), oracle.cast_fp32_to_fp16(r["p32"]).view(np.uint16))
    assert opt.step_count == 12

    # a jump (optimizer reloaded at step 99 with a fresh native object): the first tensor of step 100 finds
    # _step + 1 = 1 != 100 and takes pow like the others; step 101 then multiplies for its first tensor again
    opt2 = oracle.OptimizerStepOracle(cs, s, tensors=tensors, **kw)
    opt2.step_count = 99
    for t in (100, 101):
        for c in cs:
            c["p16"][...] = (rng.normal(0, 1e-3, c["p16"].size) * 64).astype(np.float16)
        ref = _copy(cs)
        opt2.step()
        for k, (ci, off, numel) in enumerate(tensors):
            o = oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.01, True)
            if t == 101 and k == 0:
                o.advance(100, 0.9, 0.999)
            elif t == 101:
                o.advance(101, 0.9, 0.999)
            sl = slice(off, off + numel)
            o.update(t, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, ref[ci]["p32"][sl], ref[ci]["p16"][sl], ref[ci]["m"][sl],
                     ref[ci]["v"][sl], 64.0)
        for c, r in zip(cs, ref):
            for key in ("p32", "m", "v"):
                assert np.array_equal(c[key].view(np.uint32), r[key].view(np.uint32)), (t, key)


def test_a_skipped_step_does_not_touch_the_native_object_and_single_tensor_lists_keep_the_running_product():
    # one tensor per step: the running float product on every step (the one-chunk reference configuration)
    cs = _chunks(n_chunks=1, n=64, seed=41)
    opt = oracle.OptimizerStepOracle(cs, None, lr=1e-3)
    for t in range(1, 31):
        cs[0]["p16"][...] = np.float16(0.01)
        opt.step()
        b1t, _ = _beta_powers(t, first=True, single_tensor_history=True)
        assert opt.native.consts()[5] == np.float32(1.0) - b1t
    # two tensors, dynamic scaler, step 3 poisoned: the skipped step makes no operator call, so step 3 is retried
    # and its first tensor multiplies from pow(beta, 2)
    cs = _chunks(n_chunks=2, n=64, seed=42)
    s = oracle.ScalerOracle(init_scale=4, scale_factor=2, scale_window=1000)
    opt = oracle.OptimizerStepOracle(cs, s, lr=1e-3)
    skipped = []
    for i in range(5):
        for c in cs:
            c["p16"][...] = np.float16(0.01)
        if i == 2:
            cs[1]["p16"][5] = np.nan
        cs[0]["p32"][0] = cs[0]["m"][0] = cs[0]["v"][0] = 0.0
        m0, v0 = 0.0, 0.0
        scale = s.loss_scale
        opt.check_overflow()
        skipped.append(opt.step())
        if not skipped[-1]:
            t = opt.step_count
            right = _probe_update_f64(float(np.float16(0.01)) / scale, m0, v0, 1e-3, 1e-8, *_beta_powers(t, first=True))
            assert abs(float(cs[0]["p32"][0]) - right) <= 4e-7 * abs(right), (i, t)
    assert skipped == [False, False, True, False, False] and opt.step_count == 4


def test_frozen_tensors_are_not_listed_and_not_touched():
    cs = _chunks(n_chunks=1, n=500, seed=51)
    cs[0]["p16"][...] = cs[0]["p32"].astype(np.float16)  # the slot of a frozen parameter holds the parameter
    before = _copy(cs)
    live = [(0, 0, 100), (0, 300, 200)]  # elements 100..299 belong to a frozen parameter
    cs[0]["p16"][:100] = np.float16(0.5)
    cs[0]["p16"][300:] = np.float16(-0.5)
    opt = oracle.OptimizerStepOracle(cs, None, lr=1e-2, weight_decay=0.1, use_adamw=True, tensors=live)
    opt.step()
    for key in ("p32", "m", "v"):
        assert np.array_equal(cs[0][key][100:300], before[0][key][100:300])
        assert not np.array_equal(cs[0][key][:100], before[0][key][:100])
    assert np.array_equal(cs[0]["p16"][100:300].view(np.uint16), before[0]["p32"][100:300].astype(np.float16).view(np.uint16))


def _pow32(b, t):
    return np.float32(math.pow(float(b), t))


def test_every_tensor_carries_its_own_step_number():
    """state[p]["step"] is counted per parameter and every operator call gets its tensor's own
    (fp16_cpu_adam.py:571-574,603,406).  Tensor 1 is frozen during steps 3..5 and comes back standing at 2 while the
    others stand at 5.  Which branch of IncrementStep (cpu_adam.h:143-162) each call then takes follows from the
    step numbers of consecutive calls alone, and is worked out by hand here:
      6th step  T0(6): the object stands at 5 (T2's call of the 5th step, a pow) -> pow(b,5)*b
                T1(3): the object stands at 6 -> pow(b,3);   T2(6): the object stands at 3 -> pow(b,6)
      7th step  T0(7): the object stands at 6 -> pow(b,6)*b; T1(4): pow(b,4); T2(7): pow(b,7)
    Probe elements (parameter and moments zero) are compared with the float64 textbook value for that beta^t."""
    lr, eps = 1e-3, 1e-8
    tensors = _three_tensor_layout()
    cs = _chunks(n_chunks=2, n=600, seed=61)
    opt = oracle.OptimizerStepOracle(cs, None, lr=lr, betas=(0.9, 0.999), eps=eps, tensors=tensors)
    rng = np.random.default_rng(62)

    def one_step(active, expect):
        opt.tensors = [tensors[k] for k in active]
        for k in active:
            ci, off, numel = tensors[k]
            g = rng.normal(0, 1e-2, numel).astype(np.float16)
            g[0] = np.float16(0.0123)
            cs[ci]["p16"][off : off + numel] = g
            cs[ci]["p32"][off] = cs[ci]["m"][off] = cs[ci]["v"][off] = 0.0
        frozen_before = {k: cs[tensors[k][0]]["p32"][tensors[k][1] : tensors[k][1] + tensors[k][2]].copy()
                         for k in range(len(tensors)) if k not in active}
        assert opt.step() is False
        for k, (b1t, b2t) in expect.items():
            ci, off, _ = tensors[k]
            right = _probe_update_f64(float(np.float16(0.0123)), 0.0, 0.0, lr, eps, b1t, b2t)
            got = float(cs[ci]["p32"][off])
            assert abs(got - right) <= 4e-7 * abs(right), (k, got, right)
        for k, before in frozen_before.items():
            ci, off, numel = tensors[k]
            assert np.array_equal(cs[ci]["p32"][off : off + numel], before)

    both = lambda f: (f(B1), f(B2))
    one_step([0, 1, 2], {})
    one_step([0, 1, 2], {1: both(lambda b: _pow32(b, 2)), 2: both(lambda b: _pow32(b, 2))})
    for t in (3, 4, 5):
        one_step([0, 2], {0: both(lambda b: np.float32(_pow32(b, t - 1) * b)), 2: both(lambda b: _pow32(b, t))})
    assert [opt.state(s)["step"] for s in tensors] == [5, 2, 5]
    one_step([0, 1, 2], {0: both(lambda b: np.float32(_pow32(b, 5) * b)), 1: both(lambda b: _pow32(b, 3)),
                         2: both(lambda b: _pow32(b, 6))})
    one_step([0, 1, 2], {0: both(lambda b: np.float32(_pow32(b, 6) * b)), 1: both(lambda b: _pow32(b, 4)),
                         2: both(lambda b: _pow32(b, 7))})
    assert [opt.state(s)["step"] for s in tensors] == [7, 4, 7]
    # the branches are different numbers: tensor 1 updated with the others' step number would be off by far more
    wrong = _probe_update_f64(0.0123, 0.0, 0.0, lr, eps, _pow32(B1, 7), _pow32(B2, 7))
    right = _probe_update_f64(0.0123, 0.0, 0.0, lr, eps, _pow32(B1, 4), _pow32(B2, 4))
    assert abs(wrong - right) > 1e-3 * abs(right)

    # a call whose step number is the previous call's plus one continues the product in the MIDDLE of a step:
    # T0 sits out one step and then stands one behind T1, which is called right after it
    cs = _chunks(n_chunks=2, n=600, seed=63)
    opt = oracle.OptimizerStepOracle(cs, None, lr=lr, betas=(0.9, 0.999), eps=eps, tensors=tensors[:2])
    two = tensors[:2]

    def step_two(active, expect):
        nonlocal tensors
        saved, tensors = tensors, two
        try:
            one_step(active, expect)
        finally:
            tensors = saved

    step_two([0, 1], {})
    step_two([1], {1: both(lambda b: np.float32(_pow32(b, 1) * b))})  # the object stood at 1 (T1's pow of step 1)
    # T0(2): the object stands at 2 -> 3 != 2 -> pow(b,2);  T1(3): the object stands at 2 -> multiplies T0's value
    step_two([0, 1], {0: both(lambda b: _pow32(b, 2)), 1: both(lambda b: np.float32(_pow32(b, 2) * b))})


def test_every_tensor_carries_its_own_hyper_parameters():
    """lr / betas / eps / weight_decay are read from state[p] per parameter (fp16_cpu_adam.py:596-601) and handed to
    the tensor's own call (:407-410,416-428).  Bit for bit against fresh operator objects driven by hand; betas that
    differ from the object's restart beta^t from pow on that call AND, because the object keeps them, on the next."""
    tensors = _three_tensor_layout()
    cs = _chunks(n_chunks=2, n=600, seed=71)
    s = oracle.StaticScalerOracle(32)
    opt = oracle.OptimizerStepOracle(cs, s, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True,
                                     tensors=tensors)
    opt.state(tensors[1])["lr"] = 5e-4
    opt.state(tensors[1])["weight_decay"] = 0.0
    opt.state(tensors[2])["betas"] = (0.8, 0.99)
    opt.state(tensors[2])["eps"] = 1e-6
    hyper = [(1e-3, 0.9, 0.999, 1e-8, 0.01), (5e-4, 0.9, 0.999, 1e-8, 0.0), (1e-3, 0.8, 0.99, 1e-6, 0.01)]
    rng = np.random.default_rng(72)
    for t in range(1, 6):
        for c in cs:
            c["p16"][...] = (rng.normal(0, 1e-3, c["p16"].size) * 32).astype(np.float16)
        ref = _copy(cs)
        opt.step()
        for k, ((ci, off, numel), (lr, b1, b2, eps, wd)) in enumerate(zip(tensors, hyper)):
            o = oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.01, True)
            # by hand: T0 follows T2's call of the step before, whose betas were others -> pow; T1 follows T0 in the
            # same step -> pow; T2's betas differ from T1's -> pow.  A fresh object at step 0 takes pow for t > 1 and
            # multiplies 1 * beta for t == 1, which is the same float as pow(beta, 1).
            sl = slice(off, off + numel)
            o.update(t, lr, b1, b2, eps, wd, True, ref[ci]["p32"][sl], ref[ci]["p16"][sl], ref[ci]["m"][sl],
                     ref[ci]["v"][sl], 32.0)
        for c, r in zip(cs, ref):
            for key in ("p32", "m", "v"):
                assert np.array_equal(c[key].view(np.uint32), r[key].view(np.uint32)), (t, key)
    # decoupled decay really was off for tensor 1 and on for the others: with zero gradient and moments only the
    # decay moves a parameter
    cs2 = _chunks(n_chunks=2, n=600, seed=73)
    for c in cs2:
        c["p16"][...] = 0
        c["m"][...] = 0
        c["v"][...] = 0
    before = _copy(cs2)
    opt2 = oracle.OptimizerStepOracle(cs2, None, lr=1e-2, weight_decay=0.1, use_adamw=True, tensors=tensors)
    opt2.state(tensors[1])["weight_decay"] = 0.0
    opt2.step()
    assert np.array_equal(cs2[0]["p32"][250:550], before[0]["p32"][250:550])
    want = before[0]["p32"][:250].astype(np.float64) * (1 - 1e-2 * 0.1)
    assert np.allclose(cs2[0]["p32"][:250], want, rtol=1e-6, atol=0)


def test_torch_managed_tensors_go_through_the_operator_with_their_fp32_gradients():
    """A chunk dict with `g32` in place of `p16` (the reference's TORCH_BASED parameters, fp16_cpu_adam.py:345-353):
    listed first, its tensor is the step's first operator call and takes the multiplying branch; its fp32 gradient
    reaches the operator unrounded (a gradient of 1e-9 * scale, which fp16 cannot hold after scaling by 1/64, still
    moves the state); it is the operator's arithmetic also when the chunk tensors take the torch formula; an inf in
    it is NOT seen by the overflow probe; a skipped step leaves it alone; no fp16 copy exists.  Every tensor against
    a fresh operator object driven into the branch by hand, and the fp32 path against float64 textbook Adam."""
    kw = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, use_adamw=True)
    rng = np.random.default_rng(41)
    for arithmetic in ("operator", "torch"):
        cs = _chunks(n_chunks=1, n=300, seed=42)
        managed = {"p32": rng.normal(0, 0.02, 200).astype(np.float32), "m": np.zeros(200, np.float32),
                   "v": np.zeros(200, np.float32), "g32": np.zeros(200, np.float32)}
        tensors = [(1, 0, 120), (0, 0, 300), (1, 120, 80)]
        s = oracle.ScalerOracle(init_scale=64, scale_factor=2, scale_window=1000)
        opt = oracle.OptimizerStepOracle(cs + [managed], s, tensors=tensors, arithmetic=arithmetic, **kw)
        for t in (1, 2, 3):
            cs[0]["p16"][...] = (rng.normal(0, 1e-3, 300) * 64).astype(np.float16)
            managed["g32"][...] = (rng.normal(0, 1e-9, 200) * 64).astype(np.float32)
            ref = _copy(cs + [managed])
            opt.check_overflow()
            assert opt.step() is False
            for k, (ci, off, numel) in enumerate(tensors):
                if ci == 0 and arithmetic == "torch":
                    continue  # the torch formula is pinned elsewhere; it leaves the operator object alone
                o = oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.0, True)
                if k == 0 and t > 1:
                    o.advance(t - 1, 0.9, 0.999)
                elif k > 0:
                    o.advance(t, 0.9, 0.999)
                sl = slice(off, off + numel)
                o.update(t, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, ref[ci]["p32"][sl], ref[ci]["g32" if ci == 1 else "p16"][sl],
                         ref[ci]["m"][sl], ref[ci]["v"][sl], 64.0)
            for ci, (c, r) in enumerate(zip(cs + [managed], ref)):
                if ci == 0 and arithmetic == "torch":
                    continue
                for key in ("p32", "m", "v"):
                    assert np.array_equal(c[key].view(np.uint32), r[key].view(np.uint32)), (arithmetic, t, ci, key)
            assert "p16" not in managed
        # float64 textbook Adam from zero state over the same three gradients would need the history; one step is enough:
        fresh = {"p32": np.zeros(4, np.float32), "m": np.zeros(4, np.float32), "v": np.zeros(4, np.float32),
                 "g32": (np.array([1e-9, -3e-9, 2e-7, 5e-4]) * 64).astype(np.float32)}
        one = oracle.OptimizerStepOracle([fresh], oracle.StaticScalerOracle(64), tensors=[(0, 0, 4)], arithmetic=arithmetic, **kw)
        one.step()
        g = fresh["g32"].astype(np.float64) / 64
        expect = -1e-3 * (0.1 * g / 0.1) / (np.sqrt(0.001 * g * g / 0.001) + 1e-8)
        np.testing.assert_allclose(fresh["p32"], expect, rtol=2e-5)
        assert abs(fresh["p32"][0]) > 5e-5  # g = 1e-9 is far below eps after fp16 rounding would have lost it; here it counts
        # an inf in the fp32 gradient is not probed (core/hook.py:202-203); an inf in the chunk is, and the skipped step
        # leaves the torch-managed tensors as they are
        managed["g32"][3] = np.inf
        cs[0]["p16"][...] = np.float16(0.5)
        opt.check_overflow()
        assert opt.has_overflow is False
        cs[0]["p16"][7] = np.inf
        before = _copy([managed])[0]
        opt.check_overflow()
        assert opt.step() is True and s.loss_scale == 32.0
        for key in ("p32", "m", "v", "g32"):
            assert np.array_equal(managed[key].view(np.uint32), before[key].view(np.uint32))
