"""GPU parity of the overflow probe, the device-resident loss scaler and the device-gated step.

Bar: skipped-step flags and the loss-scale sequence BIT-EXACT (value and Python type) against the
oracle state machine; on a skipped step fp32 param / m / v / step untouched and fp16 == RNE(fp32).
"""
import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from patrickstar_amd import _lib
from _harness import N_FULL, ChunkHarness

pytestmark = pytest.mark.gpu


def same_typed(a, b):
    return len(a) == len(b) and all(x == y and type(x) is type(y) for x, y in zip(a, b))


# ---------------------------------------------------------------- probe

@pytest.mark.parametrize("n", [1, 7, 2047, 2048, 4095, 4096, 4097, 8192, 8192 * 3 + 5, 1 << 20])
def test_overflow_scan_positions_and_values(n):
    base = (torch.randn(n, device="cuda") * 100).half()
    assert ps.DynamicLossScaler._has_inf_or_nan(base) is False
    assert oracle.has_inf_or_nan(base.cpu().numpy()) is False
    for pos in sorted({0, n - 1, n // 2, max(0, n - 9)}):
        for bad in (float("inf"), float("-inf"), float("nan")):
            x = base.clone()
            x[pos] = bad
            assert ps.DynamicLossScaler._has_inf_or_nan(x) is True
            assert oracle.has_inf_or_nan(x.cpu().numpy()) is True
            if n > 1:  # unaligned view (2-byte offset) must see the same thing
                assert ps.DynamicLossScaler._has_inf_or_nan(x[1:]) is (pos != 0)
    # largest finite fp16 values are not an overflow; +inf and -inf together are
    big = torch.full((n,), 65504.0, dtype=torch.half, device="cuda")
    assert ps.DynamicLossScaler._has_inf_or_nan(big) is False
    f32 = base.float()
    assert ps.DynamicLossScaler._has_inf_or_nan(f32) is False
    f32[n // 2] = float("nan")
    assert ps.DynamicLossScaler._has_inf_or_nan(f32) is True


@pytest.mark.parametrize("n", [1, 5, 2047, 2048, 2049, 4096 + 3, 2048 * 5, 2048 * 37 + 11, 1 << 20])
def test_overflow_scan_of_binary32_gradients_positions_and_values(n):
    """The probe on fp32 gradients (what check_overflow sees when backward leaves binary32 .grad tensors): 16-byte loads
    on whole tiles, element by element on the ragged end and on views that do not start on a 16-byte boundary."""
    probe = ps.DynamicLossScaler._has_inf_or_nan
    base = torch.randn(n, device="cuda") * 1e3
    base[::7] = torch.finfo(torch.float32).max   # the largest finite values and subnormals are not an overflow
    base[3::11] = 1e-45
    assert probe(base) is False
    for pos in sorted({0, n - 1, n // 2, max(0, n - 9), min(n - 1, 2047), min(n - 1, 2048)}):
        for bad in (float("inf"), float("-inf"), float("nan")):
            x = base.clone()
            x[pos] = bad
            assert probe(x) is True, (n, pos, bad)
            for skip in (1, 3, 4):  # views at a 4-, 12- and 16-byte offset
                if n > skip:
                    assert probe(x[skip:]) is (pos >= skip), (n, pos, bad, skip)
    # a quiet nan with payload bits and a negative nan
    x = base.clone().view(torch.int32)
    x[n // 3] = 0x7FC12345
    assert probe(x.view(torch.float32)) is True
    x[n // 3] = -1  # 0xFFFFFFFF
    assert probe(x.view(torch.float32)) is True


def test_overflow_scan_empty_and_sticky_flag():
    s = ps.DynamicLossScaler(init_scale=2**16)
    s.scan(torch.zeros(0, dtype=torch.half, device="cuda"))
    assert s.overflow_flag is False
    bad = torch.tensor([1.0, float("inf")], dtype=torch.half, device="cuda")
    good = torch.ones(5000, dtype=torch.half, device="cuda")
    s.scan(good)
    assert s.overflow_flag is False
    s.scan(bad)
    s.scan(good)  # sticky: a later clean gradient does not clear it
    assert s.overflow_flag is True
    s.update_scale(None)  # consumes and clears the device flag
    assert s.overflow_flag is False and s.loss_scale == 2**16 / 2 and s.last_step_skipped is True


# ---------------------------------------------------------------- state machine

CASES = [
    dict(init_scale=2**16, scale_factor=2, scale_window=3, min_scale=1),
    dict(init_scale=2**16, scale_factor=2, scale_window=1000, min_scale=1),
    dict(init_scale=4, scale_factor=2, scale_window=2, min_scale=1),
    dict(init_scale=2**16, scale_factor=2, scale_window=1000, min_scale=2**10),
    dict(init_scale=16, scale_factor=2, scale_window=1000, delayed_shift=2),
    dict(init_scale=16, scale_factor=2, scale_window=2, delayed_shift=2),
    dict(init_scale=16, scale_factor=2, scale_window=1000, delayed_shift=2, consecutive_hysteresis=True),
    dict(init_scale=16, scale_factor=2.0, scale_window=5, delayed_shift=3, consecutive_hysteresis=True),
    dict(init_scale=1000.0, scale_factor=3, scale_window=2),
    dict(init_scale=2**32, scale_factor=2.0, scale_window=7, min_scale=0.5),
    # beyond 2**53: powers of two stay exact in the device's binary64, as ints (2**60 -> 2**120) and as floats
    dict(init_scale=2**60, scale_factor=2, scale_window=2, min_scale=2**55),
    dict(init_scale=2**100, scale_factor=2.0, scale_window=3),
    dict(init_scale=3 * 2**70, scale_factor=4, scale_window=2, min_scale=3 * 2**60),
]


@pytest.mark.parametrize("kwargs", CASES)
def test_device_scaler_matches_oracle_state_machine(kwargs):
    rng = np.random.default_rng(len(str(kwargs)))
    for density in (0.0, 0.1, 0.5, 1.0):
        flags = (rng.random(120) < density).tolist()
        dev = ps.DynamicLossScaler(**kwargs)
        dev.enable_log(256)
        ora = oracle.ScalerOracle(**kwargs)
        want = []
        for f in flags:
            dev.update_scale(bool(f))  # asynchronous: nothing is read back in this loop
            ora.update_scale(bool(f))
            want.append(ora.loss_scale)
        log = dev.read_log()
        assert [f for f, _ in log] == [bool(f) for f in flags]
        got = [s for _, s in log]
        assert same_typed(got, want), (kwargs, density, got[:12], want[:12])
        assert dev.cur_iter == ora.cur_iter and dev.last_overflow_iter == ora.last_overflow_iter
        assert dev.cur_hysteresis == ora.cur_hysteresis
        assert same_typed([dev.loss_scale], [ora.loss_scale])


def test_hand_trajectory_on_device():
    s = ps.DynamicLossScaler(init_scale=2**16, scale_factor=2, scale_window=3, min_scale=1)
    got = []
    for f in [0, 0, 0, 1, 0, 0, 0, 1, 1]:
        s.update_scale(bool(f))
        got.append(s.loss_scale)
    assert same_typed(got, [65536, 65536, 131072, 65536.0, 65536.0, 65536.0, 131072.0, 65536.0, 32768.0])


# ---------------------------------------------------------------- device-gated step, small, vs oracle

def _inject(h, rng, step_chunks, chunk_size):
    """Write 1..16 non-finite values into the fp16 gradient payloads at seeded positions."""
    k = int(rng.integers(1, 17))
    for _ in range(k):
        c = int(rng.choice(step_chunks))
        pos = int(rng.choice([0, chunk_size - 1, int(rng.integers(0, chunk_size))]))
        val = [float("inf"), float("-inf"), float("nan")][int(rng.integers(0, 3))]
        h.payloads(c)[3][pos] = val


@pytest.mark.parametrize("window,factor,delayed", [(1000, 2, 1), (5, 2, 1), (4, 2, 2)])
def test_gated_step_small_bit_exact_200_steps(window, factor, delayed):
    """Config-3 shape at a size the oracle can follow: 8 chunks, 200 steps, 5 % of the steps poisoned.
    Every step: flags, scale, fp32/m/v/fp16 bit-exact against the oracle's optimizer step."""
    n_chunks, chunk_size, steps = 8, 2048 * 2 + 300, 200
    kw = dict(init_scale=2**16, scale_factor=factor, scale_window=window, min_scale=1, delayed_shift=delayed)
    scaler = ps.DynamicLossScaler(**kw)
    h = ChunkHarness(n_chunks, chunk_size, scaler, seed=3, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    scaler.enable_log(steps)
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    rng = np.random.default_rng(0)
    bad_steps = set(rng.choice(steps, size=steps // 20, replace=False).tolist())
    want_flags, want_scales = [], []
    for step in range(steps):
        h.fill_grads(1e-3, float(oscaler.loss_scale))
        if step in bad_steps:
            _inject(h, rng, list(range(n_chunks)), chunk_size)
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        oopt.check_overflow()
        skipped = oopt.step()
        want_flags.append(skipped)
        want_scales.append(oscaler.loss_scale)
        if step in bad_steps or step % 25 == 0 or step == steps - 1:
            h.compare(oc, what=f"step {step} (skipped={skipped})")
    log = scaler.read_log()
    assert [f for f, _ in log] == want_flags
    assert all(want_flags[s] for s in bad_steps)
    if window == 1000:  # no growth in 200 steps: only the poisoned steps overflow
        assert want_flags == [s in bad_steps for s in range(steps)]
    else:  # a growing scale also drives honest gradients over the fp16 range now and then
        assert sum(want_flags) > len(bad_steps)
    assert same_typed([s for _, s in log], want_scales)
    assert h.opt.state[h.params[0]]["step"] == oopt.step_count == steps - sum(want_flags)
    assert scaler.skipped_steps == sum(want_flags)
    h.compare(oc, what="final")


def test_gated_step_non_power_of_two_scale_uses_true_division():
    kw = dict(init_scale=3000.0, scale_factor=3, scale_window=2, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw)
    h = ChunkHarness(2, 2048 + 13, scaler, seed=8, lr=1e-3, weight_decay=0.001)
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-3, weight_decay=0.001)
    for step in range(6):
        h.fill_grads(1e-3, min(float(oscaler.loss_scale), 3e4))
        if step == 3:
            h.payloads(1)[3][5] = float("nan")
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        oopt.check_overflow()
        oopt.step()
        h.compare(oc, what=f"step {step}")
        assert same_typed([scaler.loss_scale], [oscaler.loss_scale])


# ---------------------------------------------------------------- the overflow / loss-scale configuration at full size

def test_config3_full_size_flags_and_scale_trajectory():
    """8 chunks of 64 Mi elements, 200 steps, a seeded 5 % of them poisoned with +-inf/nan at 1..16 positions
    (first / last element of a chunk included).  Dynamic scaler 2^16, window 1000, "hysteresis" 2 (the engine hands it
    over as scale_factor), min 1.  Nothing is read back inside the loop.  Checked: flags exactly on the poisoned
    steps, scale sequence bit-exact with the oracle (ten halvings, no growth), step counter 190, and on a skipped
    step fp32 param/m/v untouched (checksum) with fp16 == RNE(fp32)."""
    n_chunks, steps = 8, 200
    cfg = {"enabled": True, "loss_scale": 0, "initial_scale_power": 16, "loss_scale_window": 1000, "hysteresis": 2, "min_loss_scale": 1}
    _, _, scaler, _ = ps.parse_config({"fp16": cfg})
    oscaler = oracle.scaler_from_config(cfg)
    h = ChunkHarness(n_chunks, N_FULL, scaler, seed=5, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    scaler.enable_log(steps)
    h.fill_state()
    rng = np.random.default_rng(0)
    bad_steps = sorted(rng.choice(steps, size=10, replace=False).tolist())
    checks = {}
    sums = torch.zeros(steps, 3, dtype=torch.int64, device="cuda")
    fp16_ok = torch.ones(steps, dtype=torch.bool, device="cuda")

    def checksum():
        return torch.stack([sum(h.payloads(i)[k].view(torch.int32).sum(dtype=torch.int64) for i in range(n_chunks)) for k in range(3)])

    # gradients are drawn at a fixed magnitude so that they stay finite in fp16 for every scale on the trajectory
    grad_pool = [(torch.randn(N_FULL, device="cuda") * 1e-3 * 64).half() for _ in range(2)]
    for step in range(steps):
        for i in range(n_chunks):
            h.payloads(i)[3].copy_(grad_pool[(step + i) % 2])
        if step in bad_steps:
            _inject(h, rng, [0, n_chunks - 1, int(rng.integers(0, n_chunks))], N_FULL)
            before = checksum()
        h.opt.step()
        if step in bad_steps:
            sums[step] = checksum() - before
            ok = torch.tensor(True, device="cuda")
            for i in range(n_chunks):
                p, _, _, hh = h.payloads(i)
                ok = ok & torch.equal(p.half(), hh)
            fp16_ok[step] = ok
    want_scales = []
    for step in range(steps):
        oscaler.update_scale(step in bad_steps)
        want_scales.append(oscaler.loss_scale)
    log = scaler.read_log()
    assert [i for i, (f, _) in enumerate(log) if f] == bad_steps
    assert same_typed([s for _, s in log], want_scales)
    assert want_scales[-1] == 2.0**6
    assert h.opt.state[h.params[0]]["step"] == steps - len(bad_steps) == 190
    assert not sums.any().item(), "a skipped step must leave fp32 param / m / v untouched"
    assert fp16_ok.all().item(), "a skipped step must restore fp16 == RNE(fp32)"


# ---------------------------------------------------------------- checkpoint

def test_state_dict_round_trip_continues_bit_exact():
    """Semantics of the reference's checkpoint test (unitest/test_checkpoint.py:44-180): save, keep training,
    reload, replay the same gradients, incl. step and (an addition) the scaler state.

    What "identical" can mean is set by the operator object (cpu_adam.h:143-162), which a checkpoint does not carry:
    reloading into the SAME optimizer right at the saved step leaves it in step with the counter, and training
    continues exactly as if nothing had happened; a NEW optimizer starts with a new operator object, whose first call
    (the first tensor of the first step after the reload) evaluates pow(beta, t) where the uninterrupted run
    multiplied pow(beta, t-1) by beta.  Every other tensor is the same bit for bit in all three runs."""
    kw = dict(init_scale=2**10, scale_factor=2, scale_window=4, min_scale=1)
    akw = dict(lr=1e-3, weight_decay=0.01, use_adamw=True)
    n = 2048 + 99
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    grads = [[(torch.randn(n, device="cuda", generator=gen) * 1e-3 * 512).half() for _ in range(2)] for _ in range(8)]
    grads[5][1][7] = float("inf")

    def run(h, lo, hi, oopt=None):
        for s in range(lo, hi):
            for i in range(2):
                h.payloads(i)[3].copy_(grads[s][i])
                if oopt is not None:
                    oopt.chunks[i]["p16"][...] = grads[s][i].cpu().numpy()
            h.opt.step()
            if oopt is not None:
                oopt.check_overflow()
                oopt.step()

    def bits(t):
        return t.view(torch.int16 if t.dtype == torch.half else torch.int32)

    # run A: uninterrupted
    a = ChunkHarness(2, n, ps.DynamicLossScaler(**kw), seed=21, **akw)
    a.fill_state()
    run(a, 0, 3)
    sd = a.opt.state_dict()
    master = [a.payloads(i)[0].clone() for i in range(2)]
    assert sd["state"][0]["step"] == 3 and sd["state"][0]["exp_avg"].device.type == "cpu"
    # run B: the same optimizer reloads its own checkpoint at once, then continues
    b = ChunkHarness(2, n, ps.DynamicLossScaler(**kw), seed=21, **akw)
    b.fill_state()
    run(b, 0, 3)
    b.opt.load_state_dict(b.opt.state_dict())
    run(a, 3, 8)
    run(b, 3, 8)
    final = [tuple(t.clone() for t in a.payloads(i)) for i in range(2)]
    final_scale, final_step = a.opt.loss_scaler.loss_scale, a.opt.state[a.params[0]]["step"]
    for i in range(2):
        for x, y in zip(b.payloads(i), final[i]):
            assert torch.equal(bits(x), bits(y)), "an immediate reload into the same optimizer changed the run"

    # run C: a new optimizer (new operator object) loads the checkpoint and replays steps 3..7
    c = ChunkHarness(2, n, ps.DynamicLossScaler(**kw), seed=99, **akw)
    for i in range(2):
        c.payloads(i)[0].copy_(master[i])  # the model checkpoint restores the fp32 master params
    c.opt.load_state_dict(sd)
    assert c.opt.state[c.params[0]]["step"] == 3
    oc = c.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    for f in (False, False, False):
        oscaler.update_scale(f)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    oopt.step_count = 3  # with a fresh native object behind it, like the new optimizer
    run(c, 3, 8, oopt)
    c.compare(oc, what="reloaded into a new optimizer")
    for x, y in zip(c.payloads(1), final[1]):
        assert torch.equal(bits(x), bits(y)), "chunk 1 is never the first operator call: must not notice the reload"
    p_c, p_a = c.payloads(0)[0], final[0][0]
    # chunk 0 took one step with pow(beta, 4) in place of pow(beta, 3) * beta: 1 / sqrt(1 - beta2^t) moves by up to 1e-5
    # relative at such small t, i.e. the parameter by about lr * 1e-5
    assert not torch.equal(bits(p_c), bits(p_a)) and torch.allclose(p_c, p_a, rtol=0, atol=1e-3 * 5e-5)
    assert c.opt.loss_scaler.loss_scale == final_scale and c.opt.state[c.params[0]]["step"] == final_step == 7


def test_fused_gradient_clamp_follows_the_device_resident_scale():
    """With a dynamic scaler the clamp bound min(65504, clipping * loss_scale) moves with the scale, on the device."""
    kw = dict(init_scale=2**8, scale_factor=2, scale_window=2, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw)
    akw = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    h = ChunkHarness(2, 2048 + 17, scaler, seed=31, gradient_clipping=0.002, **akw)
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, gradient_clipping=0.002, **akw)
    for step in range(7):
        h.fill_grads(2e-3, float(oscaler.loss_scale))  # sigma == the clamp bound before scaling
        if step == 4:
            h.payloads(0)[3][9] = float("inf")
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        oopt.check_overflow()
        oopt.step()
        h.compare(oc, what=f"clamp, dynamic scale, step {step}")
    assert same_typed([scaler.loss_scale], [oscaler.loss_scale])


# ---------------------------------------------------------------- backward-side producer

@pytest.mark.parametrize("src_dtype", [torch.half, torch.float])
def test_grad_to_chunk_all_alignments_and_probe(src_dtype):
    """ps_grad_to_chunk == slot.copy_(grad) (RNE for fp32 sources) for every relative alignment of gradient and chunk
    slot, short (element-wise) and long (vector) gradients; the fused probe sees a non-finite value wherever it sits."""
    lib = _lib.load()
    stream = _lib.current_stream_handle()
    for n in (1, 37, 4095, 4096, 4096 + 8 * 300 + 5):
        for src_off in range(0, 9):
            for dst_off in (0, 1, 3, 7, 8, 13):
                if n < 4096 and (src_off > 2 or dst_off > 3):
                    continue
                g_all = (torch.randn(n + 16, device="cuda") * 50).to(src_dtype)
                slot_all = torch.full((n + 32,), 7.0, dtype=torch.half, device="cuda")
                g, slot = g_all[src_off:src_off + n], slot_all[dst_off:dst_off + n]
                scaler = ps.DynamicLossScaler(init_scale=2**4)
                rc = lib.ps_grad_to_chunk(g.data_ptr(), int(src_dtype == torch.half), slot.data_ptr(), n, scaler.state_ptr, stream)
                assert rc == 0
                want = torch.full_like(slot_all, 7.0)
                want[dst_off:dst_off + n].copy_(g)
                assert torch.equal(slot_all.view(torch.int16), want.view(torch.int16)), (n, src_off, dst_off)
                assert scaler.overflow_flag is False
    # the probe: positions in the head, the vector body and the tail, for a misaligned pair
    n = 4096 + 8 * 300 + 5
    for pos in (0, 2, 9, n // 2, n - 9, n - 1):
        for bad in (float("inf"), float("nan")):
            g_all = (torch.randn(n + 16, device="cuda") * 50).to(src_dtype)
            slot_all = torch.zeros(n + 32, dtype=torch.half, device="cuda")
            g, slot = g_all[3:3 + n], slot_all[5:5 + n]
            g[pos] = bad
            scaler = ps.DynamicLossScaler(init_scale=2**4)
            assert lib.ps_grad_to_chunk(g.data_ptr(), int(src_dtype == torch.half), slot.data_ptr(), n, scaler.state_ptr, stream) == 0
            assert scaler.overflow_flag is True, (pos, bad)
    if src_dtype == torch.float:  # a finite fp32 gradient beyond the fp16 range lands as inf in the chunk: flagged
        g = torch.full((5000,), 1e6, device="cuda")
        slot = torch.zeros(5000, dtype=torch.half, device="cuda")
        scaler = ps.DynamicLossScaler(init_scale=2**4)
        assert lib.ps_grad_to_chunk(g.data_ptr(), 0, slot.data_ptr(), 5000, scaler.state_ptr, stream) == 0
        assert scaler.overflow_flag is True and torch.isinf(slot).all()
    # without a state pointer it is a plain copy
    g = torch.randn(6000, device="cuda").half()
    slot = torch.zeros(6001, dtype=torch.half, device="cuda")
    assert lib.ps_grad_to_chunk(g.data_ptr(), 1, slot[1:].data_ptr(), 6000, None, stream) == 0
    assert torch.equal(slot[1:], g)


def test_device_gated_step_replays_from_a_hip_graph():
    """Scale, overflow flag, step counter and bias corrections live on the device, so the whole dynamic step (probe,
    gated update, scale update) is a fixed sequence of kernel launches: captured once into a HIP graph, it is replayed
    for later iterations, clean and poisoned alike.  Every replay is compared with the oracle, with eager work and
    synchronisation in between."""
    kw = dict(init_scale=2**10, scale_factor=2, scale_window=3, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw)
    h = ChunkHarness(3, 256 * 9 + 7, scaler, seed=77, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)

    def one_iteration(run_step, it):
        h.fill_grads(1e-3, float(oscaler.loss_scale))
        if it in (2, 5):
            h.payloads(it % 3)[3][it] = float("inf") if it == 2 else float("nan")
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        run_step()
        torch.cuda.synchronize()
        oopt.check_overflow()
        assert oopt.step() is (it in (2, 5))
        h.compare(oc, what=f"iteration {it}")
        assert scaler.loss_scale == oscaler.loss_scale and type(scaler.loss_scale) is type(oscaler.loss_scale)

    one_iteration(h.opt.step, 0)  # eager: builds the descriptor tables, nothing is allocated afterwards
    graph = torch.cuda.CUDAGraph()
    h.fill_grads(1e-3, float(oscaler.loss_scale))
    for i, c in enumerate(oc):
        c["p16"][...] = h.download(i)[3]
    with torch.cuda.graph(graph):
        h.opt.step()
    # capture records, it does not run: the state is untouched until the first replay
    assert scaler.cur_iter == 1
    graph.replay()
    torch.cuda.synchronize()
    oopt.check_overflow()
    assert oopt.step() is False
    h.compare(oc, what="first replay")
    for it in range(2, 9):
        one_iteration(graph.replay, it)
    assert scaler.cur_iter == 9 and h.opt.state[h.params[0]]["step"] == 7 == oopt.step_count
