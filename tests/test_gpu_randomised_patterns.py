"""Seeded randomised parity of the fused steps under random operator-call patterns.

Every case draws a chunk list (1 to 70 chunks, so that some lists need two launches), cuts every chunk into tensors at random
places, visits the tensors in a random order (the first of them is the step's first operator call, wherever it lies), picks
hyper-parameters, decay form, clamp, scale kind and base misalignments, sprinkles zeros, subnormals and huge values over
the state, and runs a few steps (consecutive and jumping step numbers; device-decided cases get poisoned iterations).
Bar: bit-exact against the step-level oracle, which makes one operator call per tensor."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from patrickstar_amd import _lib
from _harness import assert_bits_equal
from test_gpu_call_pattern import RawChunks
from test_gpu_tensor_list import PermutedLayout

pytestmark = pytest.mark.gpu


def _sprinkle(a, rng, kinds):
    idx = rng.integers(0, a.size, max(1, a.size // 50))
    a[idx] = rng.choice(kinds, idx.size).astype(a.dtype)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_chunk_lists_under_random_call_patterns(seed):
    lib = _lib.load()
    rng = np.random.default_rng(seed)
    for case in range(40):
        C = int(rng.choice([1, 2, 3, 5, 65, 70])) if rng.random() < 0.8 else int(rng.integers(1, 9))
        n = int(rng.choice([1, 2, 255, 256, 257, 511, 1024, int(rng.integers(1, 2500))]))
        offs = tuple(int(x) for x in rng.integers(0, 4, 4)) if rng.random() < 0.5 else (0, 0, 0, 0)
        R = RawChunks(C, n, seed=int(rng.integers(1 << 30)), offs=offs)
        for c, bufs in zip(R.host, R.dev):
            if rng.random() < 0.5:
                _sprinkle(c["p32"], rng, [0.0, -0.0, 1e-41, -3e-42, 1e30, -1e-30, 65504.0, 1.0])
                _sprinkle(c["m"], rng, [0.0, 1e-42, -1e-41, 1e20, -1e-25])
                _sprinkle(c["v"], rng, [0.0, 1e-44, 1e-38, 1e25, 3e-41])
                for key, t, off in zip(("p32", "m", "v"), bufs, R.offs):
                    t[off:off + n].copy_(torch.from_numpy(c[key]))
        tensors = []
        for ci in range(C):
            cuts = sorted(set([0, n] + [int(x) for x in rng.integers(0, n + 1, int(rng.integers(0, 4)))]))
            tensors += [(ci, a, b - a) for a, b in zip(cuts[:-1], cuts[1:])]
        tensors = [tensors[i] for i in rng.permutation(len(tensors))]
        lr, eps = float(rng.choice([1e-3, 1e-4, 0.1])), float(rng.choice([1e-8, 1e-6, 1e-3]))
        b1, b2 = float(rng.choice([0.9, 0.0, 0.5])), float(rng.choice([0.999, 0.9, 0.99]))
        wd, adamw = float(rng.choice([0.0, 0.01, 0.3])), bool(rng.integers(0, 2))
        gated = bool(rng.integers(0, 2))
        clip = float(rng.choice([-1, -1, 0.5, 1e-3]))
        oid = 5000 + case
        _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, int(adamw), 0), "create")
        if clip > 0:
            _lib.check(lib.ps_adam_set_grad_clamp(oid, clip), "clamp")
        calls = _lib.call_pattern(len(tensors), *tensors[0])
        what = (f"seed {seed} case {case}: C={C} n={n} offs={offs} tensors={len(tensors)} first={tensors[0]} lr={lr} eps={eps} "
                f"betas=({b1},{b2}) wd={wd} adamw={adamw} gated={gated} clip={clip}")
        stream = _lib.current_stream_handle()
        if gated:
            kw = dict(init_scale=float(rng.choice([2.0**10, 1000.0, 3.0])), scale_factor=2, scale_window=int(rng.integers(1, 4)), min_scale=1)
            scaler = ps.DynamicLossScaler(**kw)
            scaler.materialize("cuda:0", betas=(b1, b2))
            oscaler = oracle.ScalerOracle(**kw)
            oopt = oracle.OptimizerStepOracle(R.host, oscaler, lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd, use_adamw=adamw,
                                              tensors=tensors, gradient_clipping=clip)
            for it in range(int(rng.integers(2, 6))):
                poison = (int(rng.integers(0, C)), int(rng.integers(0, n))) if rng.random() < 0.25 else None
                R.new_grads(rng, float(oscaler.loss_scale), poison=poison)
                _lib.check(lib.ps_overflow_scan_chunks(R.table, C, n, None, scaler.state_ptr, stream), "scan")
                _lib.check(lib.ps_adam_step_chunks_gated(oid, lr, eps, wd, 1, R.table, C, n, None, calls, scaler.state_ptr, stream), "gated")
                scaler.update_scale(None, operator_calls=len(tensors))
                oopt.check_overflow()
                assert oopt.step() == (poison is not None), what
                R.compare(f"{what} iteration {it}")
                assert scaler.loss_scale == oscaler.loss_scale, what
        else:
            scale = [None, 8.0, 2.0**12, 1000.0, 12345.678][int(rng.integers(0, 5))]
            oopt = oracle.OptimizerStepOracle(R.host, oracle.StaticScalerOracle(scale) if scale else None, lr=lr, betas=(b1, b2), eps=eps,
                                              weight_decay=wd, use_adamw=adamw, tensors=tensors, gradient_clipping=clip)
            step = 0
            for _ in range(int(rng.integers(2, 6))):
                step = step + 1 if rng.random() < 0.7 else int(rng.integers(1, 3000))
                R.new_grads(rng, scale or 1.0)
                oopt.step_count = step - 1
                _lib.check(lib.ps_adam_step_chunks(oid, step, lr, b1, b2, eps, wd, 1, R.table, C, n, None, calls, scale if scale else -1.0, stream),
                           "chunks")
                oopt.step()
                R.compare(f"{what} step {step}")
        lib.ps_adam_destroy(oid)


@pytest.mark.parametrize("seed", [4, 5])
def test_tensor_lists_in_any_order_and_over_two_calls(seed):
    """The tensor-list entry point with tensors of random lengths (zero and one element included) whose momentum and
    variance sit at other element phases than the parameters, listed in another order than the reference visits them and
    split over one or two calls under one call pattern."""
    lib = _lib.load()
    rng = np.random.default_rng(seed)
    pool = [1, 2, 3, 63, 64, 255, 256, 257, 300, 1000, 4099, 65536, 70001]
    for case in range(25):
        k = int(rng.choice([7, 8, 20, 64, 65, 130]))
        sizes = [int(rng.choice(pool)) if rng.random() < 0.8 else int(rng.integers(1, 5000)) for _ in range(k)]
        scale = [None, 8.0, 2.0**12, 1000.0][int(rng.integers(0, 4))]
        L = PermutedLayout(sizes, seed=int(rng.integers(1 << 30)), scale=scale or 1.0)
        lr, eps, wd = float(rng.choice([1e-3, 1e-4])), float(rng.choice([1e-8, 1e-6])), float(rng.choice([0.0, 0.01]))
        adamw, b1, b2 = bool(rng.integers(0, 2)), 0.9, float(rng.choice([0.999, 0.95]))
        torch_arith = rng.random() < 0.3
        oid = 7000 + case
        _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, int(adamw), 0), "create")
        if torch_arith:
            _lib.check(lib.ps_adam_set_arithmetic(oid, _lib.PS_ARITH_TORCH), "arithmetic")
        ref_order = [int(i) for i in rng.permutation(k)]  # the order of the reference's operator calls
        listed = [int(i) for i in rng.permutation(k)]     # the order of the list(s) handed over
        cut = int(rng.integers(1, k)) if rng.random() < 0.5 else k
        first = ref_order[0]
        parts = sorted([part for part in (listed[:cut], listed[cut:]) if part], key=lambda part: first not in part)
        native = oracle.AdamOracle(lr, b1, b2, eps, wd, adamw)
        what = f"seed {seed} case {case}: k={k} scale={scale} torch={torch_arith} adamw={adamw} wd={wd} parts={[len(x) for x in parts]}"
        step = 0
        for it in range(int(rng.integers(1, 4))):
            step = step + 1 if rng.random() < 0.7 else int(rng.integers(1, 3000))
            if it:
                L.new_grads(rng, scale or 1.0)
            for part in parts:
                rows = _lib.chunk_array([[L.table[i].param_fp32, L.table[i].exp_avg, L.table[i].exp_avg_sq, L.table[i].param_fp16] for i in part])
                numels = (ctypes.c_size_t * len(part))(*[sizes[i] for i in part])
                pattern = _lib.call_pattern(k, part.index(first), 0, sizes[first]) if first in part else _lib.call_pattern(k, 0, 0, 0)
                _lib.check(lib.ps_adam_step_tensors(oid, step, lr, b1, b2, eps, wd, 1, rows, numels, len(part), pattern,
                                                    float(scale) if scale else -1.0, None, _lib.current_stream_handle()), what)
            torch.cuda.synchronize()
            for i in ref_order:
                p, h, m, v = L.views(i)
                pc, mc, vc, hc = p.copy(), m.copy(), v.copy(), h.copy()
                if torch_arith:
                    oracle.torch_formula_update(pc, hc, mc, vc, step, lr, b1, b2, eps, wd, adamw, scale)
                else:
                    native.update(step, lr, b1, b2, eps, wd, True, pc, hc, mc, vc, float(scale) if scale else -1.0)
                p[...], m[...], v[...] = pc, mc, vc
                h[...] = oracle.cast_fp32_to_fp16(np.ascontiguousarray(pc))
            L.compare(f"{what} step {step}")
        lib.ps_adam_destroy(oid)


@pytest.mark.parametrize("seed", [6, 7])
def test_engine_with_random_frozen_sets_and_host_placements(seed):
    """initialize_engine over small random MLPs: layer widths (some odd), chunk size (one to several layers per chunk),
    frozen parameters, which positions keep their optimizer state in pinned host memory, arithmetic, optimizer type and
    scaler kind are drawn per case; dynamic cases overflow now and then.  Whatever combination of entry points one
    step turns into (whole chunks, tensor list, streamed chunks, staged tensor lists), every payload matches the oracle
    that makes one operator call per trainable tensor under the same placement."""
    from _harness import tensor_spans

    def snap(t):
        return t.detach().to("cpu", copy=True).numpy().copy()

    rng = np.random.default_rng(seed)
    seen = set()
    for case in range(30):
        widths = [int(rng.choice([8, 12, 16, 24, 33])) for _ in range(int(rng.integers(3, 8)))]
        with_gain = rng.random() < 0.5

        class Net(torch.nn.Module):
            def __init__(self):
                super().__init__()
                self.layers = torch.nn.ModuleList([torch.nn.Linear(a, b) for a, b in zip(widths[:-1], widths[1:])])
                if with_gain:
                    self.gain = torch.nn.Parameter(torch.ones(widths[-1]))

            def forward(self, x):
                for layer in self.layers:
                    x = torch.tanh(layer(x))
                if with_gain:
                    x = x * self.gain
                return x.float().pow(2).mean()

        names = [n for n, _ in Net().named_parameters()]
        per_module = max(a * b + b for a, b in zip(widths[:-1], widths[1:]))
        chunk = int(per_module * rng.choice([1.0, 1.3, 2.2, 3.5])) + int(rng.integers(0, 20))
        frozen = set(n for n in names if rng.random() < 0.3)
        if len(frozen) == len(names):
            frozen.pop()
        arithmetic = "operator" if rng.random() < 0.6 else "torch"
        loss_scale = int(rng.choice([0, 64]))
        optim_type = "AdamW" if rng.random() < 0.5 else "Adam"
        host_share, host_draw = float(rng.choice([0.0, 0.3, 0.6, 1.0])), rng.random(64)

        def model_func():
            torch.manual_seed(1000 * seed + case)
            m = Net()
            for n, p in m.named_parameters():
                if n in frozen:
                    p.requires_grad_(False)
            return m

        config = {
            "optimizer": {"type": optim_type, "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.05,
                                                         "arithmetic": arithmetic}},
            "fp16": {"enabled": True, "loss_scale": loss_scale, "initial_scale_power": 7, "loss_scale_window": 3, "hysteresis": 2, "min_loss_scale": 1},
            "default_chunk_size": chunk,
            "client": {"host_chunk_policy": lambda position: host_draw[position % 64] < host_share},
        }
        what = f"seed {seed} case {case}: widths={widths} chunk={chunk} frozen={sorted(frozen)} {arithmetic} {optim_type} loss_scale={loss_scale}"
        engine, optimizer = ps.initialize_engine(model_func=model_func, local_rank=0, config=config)
        client = engine.client
        cl, pos = client.chunk_list, client.positions()
        host = [i for i, q in enumerate(pos) if q.on_host]
        mirror = [{"p32": snap(cl[q.fp32].payload), "m": snap(cl[q.exp_avg].payload), "v": snap(cl[q.exp_avg_sq].payload),
                   "p16": snap(cl[q.fp16].payload)} for q in pos]
        oscaler = oracle.scaler_from_config(config["fp16"])
        oopt = oracle.OptimizerStepOracle(mirror, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.05,
                                          use_adamw=(optim_type == "AdamW"), tensors=tensor_spans(client, optimizer),
                                          arithmetic=arithmetic, operator_chunks=host)
        x = torch.randn(8, widths[0], device="cuda").half()
        for it in range(4):
            blow_up = loss_scale == 0 and rng.random() < 0.25
            loss = engine(x * (6e4 if blow_up else 1.0))
            engine.backward(loss)
            for q, c in zip(pos, mirror):
                c["p16"][...] = snap(cl[q.fp16].payload)
            optimizer.step()
            torch.cuda.synchronize()
            oopt.check_overflow()
            oopt.step()
            for i, (q, c) in enumerate(zip(pos, mirror)):
                for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                    assert_bits_equal(snap(cl[cid].payload), c[key], f"{what} host={host} iteration {it} position {i} {key}")
            assert optimizer.loss_scaler.loss_scale == oscaler.loss_scale, what
        seen.update([s[0] for s in optimizer._stages] if optimizer._stages else
                    ["one tensor list" if optimizer._tensor_table else "whole chunks"])
    # the draw covers every way a step can be put together
    assert {"tensors", "stream", "staged", "one tensor list", "whole chunks"} <= seen, seen


@pytest.mark.parametrize("seed", [6, 7, 8])
def test_per_tensor_step_numbers_and_hyper_parameters_under_random_sequences(seed):
    """ps_adam_step_tensors_each through the C ABI: tensors cut at random places out of two chunks (momentum and variance
    at other element phases than the parameters in half of the cases), visited in a random order, every tensor with its
    own step number (drawn so that "the previous call's plus one" happens often), betas / lr / eps / weight decay from
    small pools, some tensors sitting out some steps; operator arithmetic everywhere, or the torch formula for the
    tensors of chunk 0 and the operator for those of chunk 1; host-decided and device-decided (with poisoned steps).
    Bar: bit-exact against the oracle, whose operator object walks through the same calls."""
    lib = _lib.load()
    rng = np.random.default_rng(seed)
    for case in range(24):
        n = int(rng.choice([700, 1500, 4099, 6000]))
        offs = tuple(int(x) for x in rng.integers(0, 4, 4)) if rng.random() < 0.5 else (0, 0, 0, 0)
        R = RawChunks(2, n, seed=int(rng.integers(1 << 30)), offs=offs)
        spans = []
        for ci in range(2):
            cuts = sorted(set([0, n] + [int(x) for x in rng.integers(0, n + 1, int(rng.integers(1, 5)))]))
            spans += [(ci, a, b - a) for a, b in zip(cuts[:-1], cuts[1:])]
            if rng.random() < 0.3:
                spans.append((ci, int(rng.integers(0, n)), 0))  # the reference calls the operator for empty tensors too
        spans = [spans[i] for i in rng.permutation(len(spans))]
        torch_arith = rng.random() < 0.4
        gated = bool(rng.integers(0, 2))
        adamw = bool(rng.integers(0, 2))
        clip = float(rng.choice([-1, -1, 0.5]))
        betas0 = (0.9, 0.999)
        beta_pool = [(0.9, 0.999), (0.9, 0.999), (0.8, 0.99), (0.0, 0.9)]
        base = int(rng.integers(0, 50))
        oid = 9000 + case
        _lib.check(lib.ps_adam_create(oid, 1e-3, betas0[0], betas0[1], 1e-8, 0.0, int(adamw), 0), "create")
        if clip > 0:
            _lib.check(lib.ps_adam_set_grad_clamp(oid, clip), "clamp")
        if torch_arith:
            _lib.check(lib.ps_adam_set_arithmetic(oid, _lib.PS_ARITH_TORCH), "arithmetic")
        if gated:
            kw = dict(init_scale=float(rng.choice([2.0**10, 1000.0])), scale_factor=2, scale_window=int(rng.integers(1, 4)), min_scale=1)
            scaler = ps.DynamicLossScaler(**kw)
            scaler.materialize("cuda:0", betas=betas0)
            scaler._seed_step(base)
            oscaler = oracle.ScalerOracle(**kw)
        else:
            scale = [None, 8.0, 2.0**12, 1000.0][int(rng.integers(0, 4))]
            oscaler = oracle.StaticScalerOracle(scale) if scale else None
        oopt = oracle.OptimizerStepOracle(R.host, oscaler, lr=1e-3, betas=betas0, eps=1e-8, weight_decay=0.0, use_adamw=adamw,
                                          tensors=spans, gradient_clipping=clip, arithmetic="torch" if torch_arith else "operator",
                                          operator_chunks=(1,))
        for span in spans:
            st = oopt.state(span)
            st["step"] = base + int(rng.integers(0, 4))  # steps made so far: neighbours often differ by exactly one
            st["betas"] = beta_pool[int(rng.integers(0, len(beta_pool)))]
            st["lr"] = float(rng.choice([1e-3, 1e-3, 5e-4]))
            st["eps"] = float(rng.choice([1e-8, 1e-8, 1e-6]))
            st["weight_decay"] = float(rng.choice([0.0, 0.01, 0.01]))
        device_step = base  # adam_step of the device-resident state
        what = (f"seed {seed} case {case}: n={n} offs={offs} tensors={len(spans)} torch={torch_arith} gated={gated} adamw={adamw} "
                f"clip={clip} base={base}")
        workspace = torch.empty(64 * len(spans), dtype=torch.uint8, device="cuda")
        stream = _lib.current_stream_handle()
        for it in range(int(rng.integers(3, 6))):
            active = [s for s in spans if rng.random() < 0.8] or spans[:1]
            oopt.tensors = active
            rows, numels = [], []
            each = (_lib.ps_tensor_call * len(active))()
            n_operator = 0
            for k, (ci, off, numel) in enumerate(active):
                rows.append([t[o + off:].data_ptr() for t, o in zip(R.dev[ci], R.offs)])
                numels.append(numel)
                st = oopt.state((ci, off, numel))
                e = each[k]
                e.lr, (e.beta1, e.beta2), e.eps, e.weight_decay = st["lr"], st["betas"], st["eps"], st["weight_decay"]
                e.step = st["step"] + 1 - (device_step + 1) if gated else st["step"] + 1
                e.arithmetic = _lib.PS_ARITH_OPERATOR if ci == 1 else -1
                n_operator += not (torch_arith and ci == 0)
            table, sizes = _lib.chunk_array(rows), (ctypes.c_size_t * len(numels))(*numels)

            def idle_slots_hold_parameters():
                # the slot of a tensor that sits out a step holds its fp16 parameter (nothing wrote a gradient over
                # it), which is what the reference's whole-chunk write-back puts there again
                for ci, off, numel in spans:
                    if (ci, off, numel) not in active and numel:
                        R.host[ci]["p16"][off:off + numel] = oracle.cast_fp32_to_fp16(np.ascontiguousarray(R.host[ci]["p32"][off:off + numel]))
                        o = R.offs[3] + off
                        R.dev[ci][3][o:o + numel].copy_(torch.from_numpy(R.host[ci]["p16"][off:off + numel]))

            if gated:
                poison = None
                filled = [s for s in active if s[2]]
                if rng.random() < 0.25 and filled:  # an inf in the gradient of a tensor that takes part in the step
                    ci, off, numel = filled[int(rng.integers(0, len(filled)))]
                    poison = (ci, off + int(rng.integers(0, numel)))
                R.new_grads(rng, float(oscaler.loss_scale), poison=None)
                idle_slots_hold_parameters()
                if poison is not None:
                    R.host[poison[0]]["p16"][poison[1]] = np.float16("inf")
                    R.dev[poison[0]][3][R.offs[3] + poison[1]] = float("inf")
                _lib.check(lib.ps_overflow_scan_chunks(R.table, 2, n, None, scaler.state_ptr, stream), "scan")
                _lib.check(lib.ps_adam_step_tensors_each(oid, 1, table, sizes, each, len(active), -1.0, scaler.state_ptr,
                                                         workspace.data_ptr(), workspace.numel(), stream), "each")
                scaler.update_scale(None, operator_calls=n_operator)
                oopt.check_overflow()
                skipped = oopt.step()
                assert skipped == (poison is not None), what
                device_step += not skipped
                R.compare(f"{what} iteration {it}")
                assert scaler.loss_scale == oscaler.loss_scale and scaler.adam_step == device_step, what
            else:
                R.new_grads(rng, oscaler.loss_scale if oscaler else 1.0)
                idle_slots_hold_parameters()
                _lib.check(lib.ps_adam_step_tensors_each(oid, 1, table, sizes, each, len(active),
                                                         float(oscaler.loss_scale) if oscaler else -1.0, None, None, 0, stream), "each")
                oopt.step()
                R.compare(f"{what} iteration {it}")
        lib.ps_adam_destroy(oid)


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("torch_arith", [False, True])
def test_more_distinct_calls_in_a_step_than_one_launch_carries(gated, torch_arith):
    """ps_adam_step_tensors_each over 150 tensors (two of them long enough to get launches of their own) of which nearly
    every one has its own learning rate and step number, with three weight decays (one of them zero: another kernel
    form) and two epsilons: far more distinct calls than the constants one launch brings along, in launches that mix
    them.  Bar: bit-exact against the oracle, three steps, host- and device-decided, both arithmetics (the tensors of
    chunk 1 stay with the operator)."""
    lib = _lib.load()
    rng = np.random.default_rng(77 + 2 * gated + torch_arith)
    n = 150000
    R = RawChunks(2, n, seed=5, offs=(0, 0, 0, 0))
    spans = []
    for ci in range(2):
        cuts = [0, 90001] + sorted(set(int(x) for x in rng.integers(90001, n, 73))) + [n]
        spans += [(ci, a, b - a) for a, b in zip(cuts[:-1], cuts[1:]) if b > a]
    spans = [spans[i] for i in rng.permutation(len(spans))]
    oid = 9100 + 2 * gated + torch_arith
    _lib.check(lib.ps_adam_create(oid, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0), "create")
    if torch_arith:
        _lib.check(lib.ps_adam_set_arithmetic(oid, _lib.PS_ARITH_TORCH), "arithmetic")
    base = 40
    if gated:
        kw = dict(init_scale=2.0**10, scale_factor=2, scale_window=2, min_scale=1)
        scaler = ps.DynamicLossScaler(**kw)
        scaler.materialize("cuda:0", betas=(0.9, 0.999))
        scaler._seed_step(base)
        oscaler = oracle.ScalerOracle(**kw)
    else:
        oscaler = oracle.StaticScalerOracle(2.0**12)
    oopt = oracle.OptimizerStepOracle(R.host, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, use_adamw=True,
                                      tensors=spans, arithmetic="torch" if torch_arith else "operator", operator_chunks=(1,))
    for k, span in enumerate(spans):
        st = oopt.state(span)
        st["step"] = base + int(rng.integers(0, 30))
        st["lr"] = 1e-3 * (1.0 + 0.01 * k)
        st["eps"] = float(rng.choice([1e-8, 1e-6]))
        st["weight_decay"] = float(rng.choice([0.0, 0.01, 0.1]))
    assert len({(oopt.state(s)["lr"], oopt.state(s)["step"]) for s in spans}) > 100
    device_step = base
    workspace = torch.empty(lib.ps_tensors_each_workspace_bytes(len(spans)), dtype=torch.uint8, device="cuda")
    stream = _lib.current_stream_handle()
    rows = [[t[o + off:].data_ptr() for t, o in zip(R.dev[ci], R.offs)] for ci, off, _ in spans]
    table = _lib.chunk_array(rows)
    sizes = (ctypes.c_size_t * len(spans))(*[s[2] for s in spans])
    each = (_lib.ps_tensor_call * len(spans))()
    for it in range(3):
        for e, span in zip(each, spans):
            st = oopt.state(span)
            e.lr, (e.beta1, e.beta2), e.eps, e.weight_decay = st["lr"], st["betas"], st["eps"], st["weight_decay"]
            e.step = st["step"] + 1 - (device_step + 1) if gated else st["step"] + 1
            e.arithmetic = _lib.PS_ARITH_OPERATOR if span[0] == 1 else -1
        what = f"gated={gated} torch={torch_arith} iteration {it}"
        if gated:
            poisoned = it == 1
            R.new_grads(rng, float(oscaler.loss_scale), poison=(1, 12345) if poisoned else None)
            _lib.check(lib.ps_overflow_scan_chunks(R.table, 2, n, None, scaler.state_ptr, stream), "scan")
            _lib.check(lib.ps_adam_step_tensors_each(oid, 1, table, sizes, each, len(spans), -1.0, scaler.state_ptr,
                                                     workspace.data_ptr(), workspace.numel(), stream), "each")
            scaler.update_scale(None, operator_calls=sum(1 for s in spans if not (torch_arith and s[0] == 0)))
            oopt.check_overflow()
            assert oopt.step() == poisoned, what
            device_step += not poisoned
            R.compare(what)
            assert scaler.loss_scale == oscaler.loss_scale and scaler.adam_step == device_step, what
        else:
            R.new_grads(rng, oscaler.loss_scale)
            _lib.check(lib.ps_adam_step_tensors_each(oid, 1, table, sizes, each, len(spans), float(oscaler.loss_scale), None, None, 0,
                                                     stream), "each")
            oopt.step()
            R.compare(what)
    lib.ps_adam_destroy(oid)


@pytest.mark.parametrize("gated", [False, True])
def test_more_distinct_calls_than_sixteen_bits_number(gated):
    """66,000 one- to three-element tensors, every one with a learning rate of its own: a launch names its tensors'
    calls in 16 bits, so a device-decided step hands its launches windows of the table of constants, and a host-decided
    one cuts its launches by the 24 sets of constants each brings along.  Bit-exact against the oracle, one step."""
    lib = _lib.load()
    rng = np.random.default_rng(91 + gated)
    lengths = rng.integers(1, 4, 66000)
    starts = np.concatenate([[0], np.cumsum(lengths)[:-1]])
    n = int(lengths.sum())
    R = RawChunks(1, n, seed=6, offs=(0, 0, 0, 0))
    spans = [(0, int(a), int(k)) for a, k in zip(starts, lengths)]
    oid = 9200 + gated
    _lib.check(lib.ps_adam_create(oid, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, 0), "create")
    base = 6
    if gated:
        kw = dict(init_scale=2.0**10, scale_factor=2, scale_window=1000, min_scale=1)
        scaler = ps.DynamicLossScaler(**kw)
        scaler.materialize("cuda:0", betas=(0.9, 0.999))
        scaler._seed_step(base)
        oscaler = oracle.ScalerOracle(**kw)
    else:
        oscaler = oracle.StaticScalerOracle(2.0**10)
    oopt = oracle.OptimizerStepOracle(R.host, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True,
                                      tensors=spans)
    each = (_lib.ps_tensor_call * len(spans))()
    for k, (e, span) in enumerate(zip(each, spans)):
        st = oopt.state(span)
        st["step"] = base
        st["lr"] = 1e-3 * (1.0 + 1e-5 * k)
        e.lr, e.beta1, e.beta2, e.eps, e.weight_decay, e.arithmetic = st["lr"], 0.9, 0.999, 1e-8, 0.01, -1
        e.step = 0 if gated else base + 1
    table = _lib.chunk_array([[t[o + off:].data_ptr() for t, o in zip(R.dev[0], R.offs)] for _, off, _ in spans])
    sizes = (ctypes.c_size_t * len(spans))(*[s[2] for s in spans])
    stream = _lib.current_stream_handle()
    R.new_grads(rng, float(oscaler.loss_scale))
    if gated:
        workspace = torch.empty(lib.ps_tensors_each_workspace_bytes(len(spans)), dtype=torch.uint8, device="cuda")
        _lib.check(lib.ps_overflow_scan_chunks(R.table, 1, n, None, scaler.state_ptr, stream), "scan")
        _lib.check(lib.ps_adam_step_tensors_each(oid, 1, table, sizes, each, len(spans), -1.0, scaler.state_ptr, workspace.data_ptr(),
                                                 workspace.numel(), stream), "each")
        scaler.update_scale(None, operator_calls=len(spans))
        oopt.check_overflow()
        assert oopt.step() is False
        assert scaler.adam_step == base + 1
    else:
        _lib.check(lib.ps_adam_step_tensors_each(oid, 1, table, sizes, each, len(spans), float(oscaler.loss_scale), None, None, 0, stream),
                   "each")
        oopt.step()
    R.compare(f"gated={gated}")
    lib.ps_adam_destroy(oid)


class _TorchManaged:
    """fp32 tensors that PyTorch manages itself (the reference's TORCH_BASED parameters): fp32 parameter, momentum,
    variance and a fp32 gradient, on the device (element offset `skew` into their buffers) and mirrored as an
    oracle chunk without a `p16` entry."""

    def __init__(self, n, seed, skew=0):
        rng = np.random.default_rng(seed)
        self.n, self.skew = n, skew
        self.host = {"p32": rng.normal(0, 0.02, n).astype(np.float32), "m": rng.normal(0, 1e-4, n).astype(np.float32),
                     "v": np.abs(rng.normal(0, 1e-6, n)).astype(np.float32), "g32": np.zeros(n, np.float32)}
        self.dev = {}
        for key, arr in self.host.items():
            self.dev[key] = torch.zeros(n + 8, dtype=torch.float, device="cuda")
            self.dev[key][skew:skew + n].copy_(torch.from_numpy(arr))

    def row(self, off):
        return [self.dev[key][self.skew + off:].data_ptr() for key in ("p32", "m", "v", "g32")]

    def new_grads(self, rng, scale):
        self.host["g32"][...] = (rng.normal(0, 1e-3, self.n) * scale).astype(np.float32)
        self.dev["g32"][self.skew:self.skew + self.n].copy_(torch.from_numpy(self.host["g32"]))

    def compare(self, what):
        torch.cuda.synchronize()
        for key in ("p32", "m", "v", "g32"):
            assert_bits_equal(self.dev[key][self.skew:self.skew + self.n].cpu().numpy(), self.host[key], f"{what}: torch-managed {key}")


@pytest.mark.parametrize("seed", [11, 12])
def test_torch_managed_fp32_tensors_take_their_place_in_the_call_sequence(seed):
    """ps_adam_step_tensors_each with PS_TENSOR_GRAD_F32 tensors among the chunk tensors (the reference's TORCH_BASED
    parameters: fp32 gradient handed to the operator as it is, no fp16 copy, no overflow probe, nothing restored on
    a skipped step; fp16_cpu_adam.py:345-353,301-302,459-460): any of them may be the step's first call, they carry
    their own step numbers and hyper-parameters like every tensor, whole aligned tiles and ragged / unaligned ones,
    with and without the gradient clamp, host- and device-decided, under both arithmetics of the chunk tensors.
    Bar: bit-exact against the oracle."""
    lib = _lib.load()
    rng = np.random.default_rng(seed)
    for case in range(16):
        n = int(rng.choice([700, 1500, 4099]))
        R = RawChunks(2, n, seed=int(rng.integers(1 << 30)))
        nt = int(rng.choice([3000, 5000]))
        T = _TorchManaged(nt, seed=int(rng.integers(1 << 30)), skew=int(rng.choice([0, 0, 1, 4])))
        spans = []
        for ci in range(2):
            cuts = sorted(set([0, n] + [int(x) for x in rng.integers(0, n + 1, int(rng.integers(1, 4)))]))
            spans += [(ci, a, b - a) for a, b in zip(cuts[:-1], cuts[1:])]
        cuts = sorted(set([0, 2048, nt] + [int(x) for x in rng.integers(2048, nt + 1, int(rng.integers(0, 3)))]))
        spans += [(2, a, b - a) for a, b in zip(cuts[:-1], cuts[1:])]
        spans = [spans[i] for i in rng.permutation(len(spans))]
        torch_arith = rng.random() < 0.4
        gated = bool(rng.integers(0, 2))
        adamw = bool(rng.integers(0, 2))
        clip = float(rng.choice([-1, -1, 0.5]))
        base = int(rng.integers(0, 50))
        oid = 9300 + case
        _lib.check(lib.ps_adam_create(oid, 1e-3, 0.9, 0.999, 1e-8, 0.0, int(adamw), 0), "create")
        if clip > 0:
            _lib.check(lib.ps_adam_set_grad_clamp(oid, clip), "clamp")
        if torch_arith:
            _lib.check(lib.ps_adam_set_arithmetic(oid, _lib.PS_ARITH_TORCH), "arithmetic")
        if gated:
            kw = dict(init_scale=float(rng.choice([2.0**10, 1000.0])), scale_factor=2, scale_window=int(rng.integers(1, 4)), min_scale=1)
            scaler = ps.DynamicLossScaler(**kw)
            scaler.materialize("cuda:0", betas=(0.9, 0.999))
            scaler._seed_step(base)
            oscaler = oracle.ScalerOracle(**kw)
        else:
            scale = [None, 8.0, 2.0**12, 1000.0][int(rng.integers(0, 4))]
            oscaler = oracle.StaticScalerOracle(scale) if scale else None
        oopt = oracle.OptimizerStepOracle(R.host + [T.host], oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0,
                                          use_adamw=adamw, tensors=spans, gradient_clipping=clip,
                                          arithmetic="torch" if torch_arith else "operator")
        uniform = rng.random() < 0.4  # every tensor with the same numbers: what an ordinary run looks like
        for span in spans:
            st = oopt.state(span)
            st["step"] = base if uniform else base + int(rng.integers(0, 3))
            if not uniform:
                st["lr"] = float(rng.choice([1e-3, 5e-4]))
                st["weight_decay"] = float(rng.choice([0.0, 0.01]))
                st["betas"] = [(0.9, 0.999), (0.8, 0.99)][int(rng.integers(0, 2))]
        device_step = base
        what = (f"seed {seed} case {case}: n={n} nt={nt} skew={T.skew} tensors={len(spans)} first={spans[0]} torch={torch_arith} "
                f"gated={gated} adamw={adamw} clip={clip} uniform={uniform}")
        workspace = torch.empty(64 * len(spans), dtype=torch.uint8, device="cuda")
        stream = _lib.current_stream_handle()
        rows = [T.row(off) if ci == 2 else [t[o + off:].data_ptr() for t, o in zip(R.dev[ci], R.offs)] for ci, off, _ in spans]
        table, sizes = _lib.chunk_array(rows), (ctypes.c_size_t * len(spans))(*[s[2] for s in spans])
        each = (_lib.ps_tensor_call * len(spans))()
        n_operator = sum(1 for ci, _, _ in spans if ci == 2 or not torch_arith)
        for it in range(int(rng.integers(3, 6))):
            for e, span in zip(each, spans):
                st = oopt.state(span)
                e.lr, (e.beta1, e.beta2), e.eps, e.weight_decay = st["lr"], st["betas"], st["eps"], st["weight_decay"]
                e.step = st["step"] + 1 - (device_step + 1) if gated else st["step"] + 1
                e.arithmetic = _lib.PS_ARITH_OPERATOR if span[0] == 2 else -1
                e.flags = _lib.PS_TENSOR_GRAD_F32 if span[0] == 2 else 0
            cur = float(oscaler.loss_scale) if oscaler else 1.0
            T.new_grads(rng, cur)
            if gated:
                poison = (int(rng.integers(0, 2)), int(rng.integers(0, n))) if rng.random() < 0.3 else None
                R.new_grads(rng, cur, poison=poison)
                _lib.check(lib.ps_overflow_scan_chunks(R.table, 2, n, None, scaler.state_ptr, stream), "scan")
                _lib.check(lib.ps_adam_step_tensors_each(oid, 1, table, sizes, each, len(spans), -1.0, scaler.state_ptr,
                                                         workspace.data_ptr(), workspace.numel(), stream), "each")
                scaler.update_scale(None, operator_calls=n_operator)
                oopt.check_overflow()
                assert oopt.step() == (poison is not None), what
                device_step += poison is None
                assert scaler.loss_scale == oscaler.loss_scale and scaler.adam_step == device_step, what
            else:
                R.new_grads(rng, cur)
                _lib.check(lib.ps_adam_step_tensors_each(oid, 1, table, sizes, each, len(spans), float(oscaler.loss_scale) if oscaler else -1.0,
                                                         None, None, 0, stream), "each")
                oopt.step()
            R.compare(f"{what} iteration {it}")
            T.compare(f"{what} iteration {it}")
        lib.ps_adam_destroy(oid)
