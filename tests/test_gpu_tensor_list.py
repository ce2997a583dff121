"""GPU parity of ps_adam_step_tensors: the per-tensor loop of the reference as one call, for chunk layouts in which
momentum and variance tensors are NOT at their parameter's own offset (the reference's own packing of optimizer-state
tensors, patrickstar/core/client.py:282-309).  Bit-exact against the CPU restatements, both arithmetics, host-decided
and device-gated."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from patrickstar_amd import _lib
from _harness import assert_bits_equal

pytestmark = pytest.mark.gpu

SIZES = [1, 3, 255, 256, 257, 768, 1000, 4096 + 3, 2304 * 64, 100_000, 5, 64] * 5 + [300_001]  # 61 tensors: two launches


class PermutedLayout:
    """Parameters packed in order into an fp16 and an fp32 payload; momentum packed in REVERSE order and variance
    in a rotated order into theirs, so no two lists share offsets."""

    def __init__(self, sizes, seed, scale):
        rng = np.random.default_rng(seed)
        self.sizes = sizes
        total = sum(sizes)
        rot = 7 % len(sizes)
        order = {"p": list(range(len(sizes))), "m": list(reversed(range(len(sizes)))),
                 "v": list(range(rot, len(sizes))) + list(range(rot))}
        self.off = {}
        for key, seq in order.items():
            cur, offs = 0, {}
            for i in seq:
                offs[i] = cur
                cur += sizes[i]
            self.off[key] = offs
        self.host = {
            "p": rng.normal(0, 0.02, total).astype(np.float32),
            "m": rng.normal(0, 1e-4, total).astype(np.float32),
            "v": np.abs(rng.normal(0, 1e-6, total)).astype(np.float32),
            "h": (rng.normal(0, 1e-3, total) * scale).astype(np.float16),
        }
        self.dev = {k: torch.from_numpy(a.copy()).cuda() for k, a in self.host.items()}
        rows = []
        for i, n in enumerate(sizes):
            rows.append([
                self.dev["p"][self.off["p"][i]:].data_ptr(), self.dev["m"][self.off["m"][i]:].data_ptr(),
                self.dev["v"][self.off["v"][i]:].data_ptr(), self.dev["h"][self.off["p"][i]:].data_ptr(),
            ])
        self.table = _lib.chunk_array(rows)
        self.numels = (ctypes.c_size_t * len(sizes))(*sizes)

    def views(self, i):
        n = self.sizes[i]
        return (self.host["p"][self.off["p"][i]:][:n], self.host["h"][self.off["p"][i]:][:n],
                self.host["m"][self.off["m"][i]:][:n], self.host["v"][self.off["v"][i]:][:n])

    def new_grads(self, rng, scale):
        g = (rng.normal(0, 1e-3, self.host["h"].size) * scale).astype(np.float16)
        self.host["h"][...] = g
        self.dev["h"].copy_(torch.from_numpy(g))

    def compare(self, what):
        for k in "pmvh":
            assert_bits_equal(self.dev[k].cpu().numpy(), self.host[k], f"{what}: {k}")


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
@pytest.mark.parametrize("adamw,wd,scale", [(True, 0.01, 2**12), (False, 0.01, 1000.0), (False, 0.0, None)])
def test_host_decided_steps_over_a_permuted_layout(arithmetic, adamw, wd, scale):
    lib = _lib.load()
    lr, b1, b2, eps = 1e-4, 0.9, 0.999, 1e-8
    L = PermutedLayout(SIZES, seed=len(arithmetic) + int(adamw), scale=scale or 1.0)
    rng = np.random.default_rng(9)
    oid = 820
    _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, int(adamw), 0), "create")
    if arithmetic == "torch":
        _lib.check(lib.ps_adam_set_arithmetic(oid, _lib.PS_ARITH_TORCH), "arith")
    native = oracle.AdamOracle(lr, b1, b2, eps, wd, adamw)
    # steps 1..3 from a fresh operator object, a jump to 100, then 101: per tensor the reference makes one operator
    # call, so tensor 0 multiplies the running product where it can and every other tensor evaluates pow
    for step in (1, 2, 3, 100, 101):
        if step > 1:
            L.new_grads(rng, scale or 1.0)
        _lib.check(
            lib.ps_adam_step_tensors(oid, step, lr, b1, b2, eps, wd, 1, L.table, L.numels, len(SIZES), None,
                                     float(scale) if scale is not None else -1.0, None, _lib.current_stream_handle()),
            "ps_adam_step_tensors",
        )
        torch.cuda.synchronize()
        for i, n in enumerate(SIZES):
            p, h, m, v = L.views(i)
            if arithmetic == "torch":
                pc, mc, vc, hc = p.copy(), m.copy(), v.copy(), h.copy()
                oracle.torch_formula_update(pc, hc, mc, vc, step, lr, b1, b2, eps, wd, adamw, scale)
                p[...], m[...], v[...] = pc, mc, vc
            else:
                pc, mc, vc, hc = p.copy(), m.copy(), v.copy(), h.copy()
                native.update(step, lr, b1, b2, eps, wd, True, pc, hc, mc, vc, float(scale) if scale is not None else -1.0)
                p[...], m[...], v[...] = pc, mc, vc
            h[...] = oracle.cast_fp32_to_fp16(np.ascontiguousarray(p))
        L.compare(f"{arithmetic} step {step}")
    lib.ps_adam_destroy(oid)


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
def test_device_gated_steps_over_a_permuted_layout(arithmetic):
    """Scale, step and flag from the device state; iteration 1 is poisoned and must restore the fp16 slots only."""
    lib = _lib.load()
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.01
    kw = dict(init_scale=2**10, scale_factor=2, scale_window=2, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw)
    scaler.materialize("cuda:0", betas=(b1, b2))
    oscaler = oracle.ScalerOracle(**kw)
    L = PermutedLayout(SIZES[:50], seed=4, scale=2.0**10)
    rng = np.random.default_rng(10)
    oid = 821
    _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, 1, 0), "create")
    if arithmetic == "torch":
        _lib.check(lib.ps_adam_set_arithmetic(oid, _lib.PS_ARITH_TORCH), "arith")
    native = oracle.AdamOracle(lr, b1, b2, eps, wd, True)
    adam_step = 0
    for it in range(5):
        L.new_grads(rng, float(oscaler.loss_scale))
        if it == 1:
            L.host["h"][L.off["p"][9] + 2] = np.float16("inf")
            L.dev["h"].copy_(torch.from_numpy(L.host["h"]))
        scaler.scan(L.dev["h"])
        _lib.check(
            lib.ps_adam_step_tensors(oid, 0, lr, b1, b2, eps, wd, 1, L.table, L.numels, 50, None, -1.0, scaler.state_ptr,
                                     _lib.current_stream_handle()),
            "ps_adam_step_tensors",
        )
        scaler.update_scale(None, operator_calls=0 if arithmetic == "torch" else 50)
        torch.cuda.synchronize()
        if it == 1:
            oscaler.update_scale(True)
            for i in range(50):
                p, h, m, v = L.views(i)
                h[...] = oracle.cast_fp32_to_fp16(np.ascontiguousarray(p))
        else:
            adam_step += 1
            scale = oscaler.loss_scale
            for i, n in enumerate(SIZES[:50]):
                p, h, m, v = L.views(i)
                pc, mc, vc, hc = p.copy(), m.copy(), v.copy(), h.copy()
                if arithmetic == "torch":
                    oracle.torch_formula_update(pc, hc, mc, vc, adam_step, lr, b1, b2, eps, wd, True, scale)
                else:
                    native.update(adam_step, lr, b1, b2, eps, wd, True, pc, hc, mc, vc, float(scale))
                p[...], m[...], v[...] = pc, mc, vc
                h[...] = oracle.cast_fp32_to_fp16(pc)
            oscaler.update_scale(False)
        L.compare(f"{arithmetic} iteration {it}")
        assert scaler.loss_scale == oscaler.loss_scale
    assert scaler.adam_step == 4
    lib.ps_adam_destroy(oid)


def test_tensor_list_argument_checks_and_empty_lists():
    lib = _lib.load()
    lib.ps_adam_create(822, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0)
    s = _lib.current_stream_handle()
    assert lib.ps_adam_step_tensors(822, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, None, 0, None, -1.0, None, s) == 0
    assert lib.ps_adam_step_tensors(822, 2, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, None, 3, None, -1.0, None, s) == _lib.PS_ERR_BAD_ARG
    assert lib.ps_adam_step_tensors(822, 2, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, None, -1, None, -1.0, None, s) == _lib.PS_ERR_BAD_ARG
    x = torch.ones(8, device="cuda")
    h = torch.zeros(8, dtype=torch.half, device="cuda")
    rows = _lib.chunk_array([[x.data_ptr(), x.data_ptr(), 0, h.data_ptr()], [x.data_ptr(), 0, 0, 0]])
    numels = (ctypes.c_size_t * 2)(8, 0)
    assert lib.ps_adam_step_tensors(822, 2, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, rows, numels, 2, None, -1.0, None, s) == _lib.PS_ERR_BAD_ARG
    assert b"tensor 0" in lib.ps_last_error()
    numels = (ctypes.c_size_t * 2)(0, 0)  # zero-length tensors may carry NULL addresses and are skipped
    assert lib.ps_adam_step_tensors(822, 2, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, rows, numels, 2, None, -1.0, None, s) == 0
    assert lib.ps_adam_step_tensors(4711, 2, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, rows, numels, 2, None, -1.0, None, s) == _lib.PS_ERR_UNKNOWN_ID
    torch.cuda.synchronize()
    assert torch.equal(x, torch.ones(8, device="cuda"))
    lib.ps_adam_destroy(822)


@pytest.mark.parametrize("gated", [False, True])
def test_one_step_spread_over_two_tensor_list_calls_under_one_call_pattern(gated):
    """A step of 20 operator calls made through two entry-point calls: the first list holds the step's first call
    (reference tensor 0, here at index 2 of a shuffled list) and names it; the second list says that the first call is
    not among its tensors.  Tensor 0 takes the running product, all 19 others pow, as in one call over all 20."""
    lib = _lib.load()
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.01
    sizes = SIZES[:20]
    L = PermutedLayout(sizes, seed=21, scale=2.0**8)
    rng = np.random.default_rng(22)
    oid = 823
    _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, 1, 0), "create")
    first_list = [7, 3, 0, 12, 19, 8]
    second_list = [i for i in range(20) if i not in first_list]

    def sub(indices):
        rows = _lib.chunk_array([[L.table[i].param_fp32, L.table[i].exp_avg, L.table[i].exp_avg_sq, L.table[i].param_fp16] for i in indices])
        return rows, (ctypes.c_size_t * len(indices))(*[sizes[i] for i in indices]), len(indices)

    a, b = sub(first_list), sub(second_list)
    kw = dict(init_scale=2**8, scale_factor=2, scale_window=1000)
    scaler = ps.DynamicLossScaler(**kw)
    scaler.materialize("cuda:0", betas=(b1, b2))
    state = scaler.state_ptr if gated else None
    native = oracle.AdamOracle(lr, b1, b2, eps, wd, True)
    s = _lib.current_stream_handle()
    steps = (1, 2, 3, 4) if gated else (1, 2, 3, 50, 51)
    for step in steps:
        if step > 1:
            L.new_grads(rng, 2.0**8)
        for (rows, numels, n), pat in ((a, _lib.call_pattern(20, 2, 0, sizes[0])), (b, _lib.call_pattern(20, 0, 0, 0))):
            _lib.check(lib.ps_adam_step_tensors(oid, 0 if gated else step, lr, b1, b2, eps, wd, 1, rows, numels, n, pat,
                                                -1.0 if gated else 2.0**8, state, s), "ps_adam_step_tensors")
        if gated:
            scaler.update_scale(None, operator_calls=20)
        torch.cuda.synchronize()
        for i in range(20):
            p, h, m, v = L.views(i)
            pc, mc, vc, hc = p.copy(), m.copy(), v.copy(), h.copy()
            native.update(step, lr, b1, b2, eps, wd, True, pc, hc, mc, vc, 2.0**8)
            p[...], m[...], v[...] = pc, mc, vc
            h[...] = oracle.cast_fp32_to_fp16(pc)
        L.compare(f"gated={gated} step {step}")
    # a pattern that does not describe a whole tensor of the list is refused before anything is queued
    rows, numels, n = a
    E = _lib.PS_ERR_BAD_ARG
    for bad in (_lib.call_pattern(0, 2, 0, sizes[0]), _lib.call_pattern(20, 6, 0, 5), _lib.call_pattern(20, -1, 0, 5),
                _lib.call_pattern(20, 2, 1, sizes[0]), _lib.call_pattern(20, 2, 0, sizes[0] + 1)):
        assert lib.ps_adam_step_tensors(oid, 60, lr, b1, b2, eps, wd, 1, rows, numels, n, bad, 2.0**8, None, s) == E
    torch.cuda.synchronize()
    L.compare("after the refused calls")
    lib.ps_adam_destroy(oid)


def test_long_tensors_through_the_tensor_list_entry_points():
    """Tensors of up to 51 M elements (launch grids hundreds of thousands of tiles wide, one launch per long tensor) in
    the permuted layout, whole lists compared: ps_adam_step_tensors, then ps_adam_step_tensors_each host-decided and
    device-decided with three sets of numbers among the tensors."""
    lib = _lib.load()
    sizes = [50257 * 1024, 4096 * 1600, 1600, 2_000_001, 1600 * 1600, 7]
    scale = 2.0**10
    L = PermutedLayout(sizes, seed=3, scale=scale)
    rng = np.random.default_rng(4)
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.01
    _lib.check(lib.ps_adam_create(871, lr, b1, b2, eps, wd, 1, 0), "create")
    native = oracle.AdamOracle(lr, b1, b2, eps, wd, True)
    stream = _lib.current_stream_handle()
    for step in (1, 2):
        if step > 1:
            L.new_grads(rng, scale)
        _lib.check(lib.ps_adam_step_tensors(871, step, lr, b1, b2, eps, wd, 1, L.table, L.numels, len(sizes), None, scale, None, stream),
                   "ps_adam_step_tensors")
        for i in range(len(sizes)):
            p, g, m, v = L.views(i)
            native.update(step, lr, b1, b2, eps, wd, True, p, g, m, v, scale)
            g[...] = oracle.cast_fp32_to_fp16(p)
        L.compare(f"tensor list, step {step}")
    # every tensor its own numbers: the long one two steps behind, two at another learning rate
    made = [0, 2, 2, 2, 2, 2]
    lrs = [lr, lr, 5e-4, lr, 5e-4, lr]
    each = (_lib.ps_tensor_call * len(sizes))()
    for gated in (False, True):
        if gated:
            kw = dict(init_scale=2**10, scale_factor=2, scale_window=1000, min_scale=1)
            scaler = ps.DynamicLossScaler(**kw)
            scaler.materialize("cuda:0", betas=(b1, b2))
            scaler._seed_step(made[1])  # the counter of the steps made so far, behind it a fresh operator object
            native = oracle.AdamOracle(lr, b1, b2, eps, wd, True)  # ... on both sides
            workspace = torch.empty(lib.ps_tensors_each_workspace_bytes(len(sizes)), dtype=torch.uint8, device="cuda")
        for it in range(2):
            L.new_grads(rng, scale)
            for i, e in enumerate(each):
                e.lr, e.beta1, e.beta2, e.eps, e.weight_decay, e.arithmetic = lrs[i], b1, b2, eps, wd, -1
                e.step = made[i] - made[1] if gated else made[i] + 1
            if gated:
                _lib.check(lib.ps_adam_step_tensors_each(871, 1, L.table, L.numels, each, len(sizes), -1.0, scaler.state_ptr,
                                                         workspace.data_ptr(), workspace.numel(), stream), "each")
                scaler.update_scale(None, operator_calls=len(sizes))
            else:
                _lib.check(lib.ps_adam_step_tensors_each(871, 1, L.table, L.numels, each, len(sizes), scale, None, None, 0, stream), "each")
            for i in range(len(sizes)):
                made[i] += 1
                p, g, m, v = L.views(i)
                native.update(made[i], lrs[i], b1, b2, eps, wd, True, p, g, m, v, scale)
                g[...] = oracle.cast_fp32_to_fp16(p)
            L.compare(f"per-tensor numbers, gated={gated}, iteration {it}")
        if gated:
            assert scaler.adam_step == made[1] and scaler.loss_scale == 2**10
    lib.ps_adam_destroy(871)
