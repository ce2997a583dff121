"""GPU tests of (a) host-resident chunk positions streamed through HBM staging and (b) the engine front-end.

Bar as everywhere: bit-exact against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from _harness import HybridHarness, assert_bits_equal, tensor_spans

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("host_keeps_fp16", [True, False])
@pytest.mark.parametrize("host_positions", [[1, 3, 4], [0, 1, 2, 3, 4], [4]])
@pytest.mark.parametrize("chunk_size", [2048 * 3, 2048 + 77])
def test_hybrid_static_bit_exact(host_positions, chunk_size, host_keeps_fp16):
    h = HybridHarness(5, chunk_size, host_positions, ps.LossScaler(2**12), seed=chunk_size + len(host_positions),
                      host_keeps_fp16=host_keeps_fp16,
                      lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    for i in range(5):
        on_host = h.payloads(i)[0].device.type == "cpu"
        assert on_host == (i in host_positions)
        assert (not on_host) or all(t.is_pinned() for t in h.payloads(i)[:3])
        # the fp16 payload follows the state to the host only when asked to
        assert (h.payloads(i)[3].device.type == "cpu") == (on_host and host_keeps_fp16)
    h.fill_state()
    oc = h.oracle_chunks()
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(2**12), lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    for step in range(3):  # consecutive steps: resident and host halves must see the same running-product beta^t
        h.fill_grads(1e-3, 2**12)
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        torch.cuda.synchronize()
        oopt.step()
        h.compare(oc, what=f"hybrid step {step}")


@pytest.mark.parametrize("host_keeps_fp16", [True, False])
def test_hybrid_dynamic_skips_and_restores_host_chunks_too(host_keeps_fp16):
    kw = dict(init_scale=2**10, scale_factor=2, scale_window=3, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw)
    h = HybridHarness(4, 2048 * 2 + 9, [1, 2], scaler, seed=12, host_keeps_fp16=host_keeps_fp16, lr=1e-3, weight_decay=0.01)
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-3, weight_decay=0.01)
    skipped = []
    for step in range(7):
        h.fill_grads(1e-3, float(oscaler.loss_scale))
        if step == 2:
            h.payloads(2)[3][5] = float("inf")  # in a HOST-resident chunk: only the streamed probe can see it
        if step == 5:
            h.payloads(0)[3][0] = float("nan")  # in a resident chunk
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        torch.cuda.synchronize()
        oopt.check_overflow()
        skipped.append(oopt.step())
        h.compare(oc, what=f"hybrid dynamic step {step}")
        assert scaler.loss_scale == oscaler.loss_scale and type(scaler.loss_scale) is type(oscaler.loss_scale)
    assert skipped == [False, False, True, False, False, True, False]
    assert h.opt.state[h.params[0]]["step"] == 5


class _MLP(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = torch.nn.Linear(24, 40)
        self.fc2 = torch.nn.Linear(40, 8)
        self.gain = torch.nn.Parameter(torch.ones(8))

    def forward(self, x):
        return (self.fc2(torch.tanh(self.fc1(x))) * self.gain).float().pow(2).mean()


def _snap(t):
    """A private host copy (a host-resident payload would otherwise be aliased by ".cpu()")."""
    return t.detach().to("cpu", copy=True).numpy()


@pytest.mark.parametrize("host_positions", [(), (1,), (0, 1)])
@pytest.mark.parametrize("loss_scale", [0, 128])
def test_engine_end_to_end_against_oracle(loss_scale, host_positions):
    """initialize_engine -> forward -> backward -> step on a small fp16 model.  After backward the fp16 chunk payloads
    hold the gradients; the oracle is fed exactly those and must agree bit for bit with what step() leaves behind.
    With a host-chunk policy the selected positions keep fp32 param / m / v in pinned host memory and the fp16
    payload (the module's parameters) in HBM; where the state lives must not change a bit."""
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.01}},
        "fp16": {"enabled": True, "loss_scale": loss_scale, "initial_scale_power": 7, "loss_scale_window": 4, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 1100,
    }
    if host_positions:
        config["client"] = {"host_chunk_policy": lambda pos: pos in host_positions}
    engine, optimizer = ps.initialize_engine(model_func=_MLP, local_rank=0, config=config)
    client = engine.client
    assert engine.optimizer is optimizer and isinstance(optimizer, ps.FP16Adam)
    assert all(p.dtype == torch.half and p.is_cuda for p in engine.module.parameters())
    pos = client.positions()
    assert len(pos) == 2  # fc1 fills 1000 of 1100; fc2 (328) does not fit behind it -> second chunk, which also takes gain
    cl = client.chunk_list
    for i, q in enumerate(pos):
        assert q.on_host == (i in host_positions)
        assert cl[q.fp16].payload.is_cuda
        for cid in (q.fp32, q.exp_avg, q.exp_avg_sq):
            assert cl[cid].payload.is_cuda != q.on_host and (cl[cid].payload.is_pinned() or not q.on_host)
    mirror = [{"p32": _snap(cl[q.fp32].payload), "m": _snap(cl[q.exp_avg].payload),
               "v": _snap(cl[q.exp_avg_sq].payload), "p16": _snap(cl[q.fp16].payload)} for q in pos]
    oscaler = oracle.scaler_from_config(config["fp16"])
    # The reference calls the operator once per parameter in parameters() order: `gain` (the module's own parameter,
    # which sits in the SECOND chunk) comes first and is the one call of a step that may continue the running beta^t.
    spans = tensor_spans(client, optimizer)
    assert spans[0] == (1, 328, 8) and len(spans) == 5
    oopt = oracle.OptimizerStepOracle(mirror, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True,
                                      tensors=spans)
    x = torch.randn(16, 24, device="cuda").half()
    losses = []
    for it in range(6):
        loss = engine(x * (1.0 if it != 3 else 3e4))  # iteration 3 overflows fp16 activations -> inf/nan gradients
        engine.backward(loss)
        assert all(p.grad is None for p in engine.module.parameters())
        for q, c in zip(pos, mirror):
            c["p16"][...] = _snap(cl[q.fp16].payload)  # the gradients, as backward left them in the chunks
        optimizer.step()
        torch.cuda.synchronize()  # host-resident state is written by copies the host does not otherwise wait for
        oopt.check_overflow()
        skipped = oopt.step()
        if loss_scale == 0:
            assert skipped == (it == 3)
        for q, c in zip(pos, mirror):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                got = _snap(cl[cid].payload)
                if loss_scale != 0 and it >= 3:
                    assert np.array_equal(np.isnan(got), np.isnan(c[key]))  # static scale: the poison spreads, same places
                else:
                    assert_bits_equal(got, c[key], f"iteration {it} {key}")
        losses.append(float(loss.detach()))
        if loss_scale == 0:
            assert optimizer.loss_scaler.loss_scale == oscaler.loss_scale
    if loss_scale == 0:
        assert optimizer.state[next(engine.module.parameters())]["step"] == 5
        assert losses[5] < losses[0]  # it trains
    # parameters are views of the chunk payloads: the model sees what the optimizer wrote
    w = engine.module.fc1.weight
    info = client.chunk_tensor_index.get_tensor_info(w.ps_attr.data_id())
    assert w.data_ptr() == cl[info.chunk_id].payload.data_ptr() + 2 * info.start_offset


def test_hybrid_full_size_placement_invariance():
    """At the real chunk size (64 Mi elements): where a chunk lives must not change a single bit.  The same seeded
    state and gradients are stepped twice, once with every chunk in HBM and once with half of them in pinned host
    memory; the oracle checks one resident and one host-resident chunk."""
    from _harness import N_FULL

    kw = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    host = [1, 2, 5]
    a = HybridHarness(6, N_FULL, host, ps.LossScaler(2**12), seed=42, **kw)
    b = HybridHarness(6, N_FULL, [], ps.LossScaler(2**12), seed=42, **kw)
    for h in (a, b):
        h.fill_state()
        h.fill_grads(1e-3, 2**12)
        for prm in h.params:
            dict.__setitem__(h.opt.state[prm], "step", 99)
    idx = [0, 5]
    oc = a.oracle_chunks(idx)
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(2**12), **kw)
    oopt.step_count = 99
    for h in (a, b):
        h.opt.step()
    torch.cuda.synchronize()
    oopt.step()
    a.compare(oc, idx, what="hybrid full size vs oracle")
    for i in range(6):
        for x, y in zip(a.payloads(i), b.payloads(i)):
            y = y.cpu() if x.device.type == "cpu" else y
            assert torch.equal(x.view(torch.int16 if x.dtype == torch.half else torch.int32),
                               y.view(torch.int16 if y.dtype == torch.half else torch.int32)), f"chunk {i}"


@pytest.mark.parametrize("host_keeps_fp16", [True, False])
@pytest.mark.parametrize("slots", [1, 3, 8])
def test_hybrid_slot_counts_and_slot_reuse(slots, host_keeps_fp16):
    """More host-resident positions than staging slots, for 1, 3 and 8 slots: every slot is reused, and a chunk's
    write-back must have left its slot before the next occupant is copied in.  Dynamic scaler, one poisoned step."""
    kw = dict(init_scale=2**12, scale_factor=2, scale_window=1000, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw)
    host = [0, 2, 3, 4, 5, 6, 8, 9, 10]
    h = HybridHarness(11, 256 * 40 + 3, host, scaler, seed=slots, host_keeps_fp16=host_keeps_fp16,
                      lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    h.opt.staging_slots = slots
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    for step in range(4):
        h.fill_grads(1e-3, float(oscaler.loss_scale))
        if step == 1:
            h.payloads(9)[3][-1] = float("-inf")  # last element of a host-resident position
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        torch.cuda.synchronize()
        oopt.check_overflow()
        assert oopt.step() is (step == 1)
        h.compare(oc, what=f"{slots} slots, step {step}")
    assert h.opt._streamer.n_slots == slots and scaler.loss_scale == oscaler.loss_scale


class _Tied(torch.nn.Module):
    """One weight used twice (as embedding and as output projection), one parameter that gets no gradient."""

    def __init__(self):
        super().__init__()
        self.emb = torch.nn.Embedding(50, 16)
        self.mid = torch.nn.Linear(16, 16)
        self.unused = torch.nn.Parameter(torch.ones(7))

    def forward(self, ids):
        h = torch.tanh(self.mid(self.emb(ids)))
        logits = h @ self.emb.weight.t()
        return logits.float().logsumexp(-1).mean()


def test_gradients_reach_their_slots_during_backward():
    """The copy into the chunk slot runs from a post-accumulate-grad hook.  It must see the COMPLETE gradient of a
    parameter that is used twice, must not disturb the rest of backward (the slot is the parameter's own storage),
    must leave no .grad behind, and a parameter without a gradient must present a zero gradient to step()."""
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "Adam", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0}},
        "fp16": {"enabled": True, "loss_scale": 64},
        "default_chunk_size": 4096,
    }
    engine, optimizer = ps.initialize_engine(model_func=_Tied, local_rank=0, config=config)
    client = engine.client
    ids = torch.randint(0, 50, (8, 5), device="cuda")
    params = [p for p in engine.module.parameters()]
    loss = engine(ids)
    used = [p for p in params if p is not engine.module.unused]
    expected = torch.autograd.grad(loss * 64, used, retain_graph=True)  # no hooks fire for autograd.grad
    before = {p: client.access_data(p).clone() for p in params}
    for p, b in before.items():
        assert torch.equal(p.data, b)  # the slot IS the parameter
    engine.backward(loss)
    torch.cuda.synchronize()
    assert all(p.grad is None for p in params)
    for p, g in zip(used, expected):
        assert g.dtype == torch.half
        assert torch.equal(client.access_data(p), g), f"slot of {p.ps_attr.name} does not hold its gradient"
    assert not client.access_data(engine.module.unused).any()
    # step() turns the slots back into parameters; the model keeps training through the same storage
    optimizer.step()
    torch.cuda.synchronize()
    for p in used:
        assert not torch.equal(p.data, before[p]) and torch.isfinite(p.data.float()).all()
    loss2 = engine(ids)
    engine.backward(loss2)
    optimizer.step()
    assert float(loss2.detach()) < float(loss.detach())


def test_config5_full_shape_180_chunks_60_on_the_host():
    """The hybrid configuration at its real shape: 180 chunks of 64 Mi elements (12.08 G elements), 120 resident in HBM
    (113 GB) and 60 in pinned host memory (56 GB) streamed through two staging slots.  One AdamW step at t = 100.
    The oracle checks one resident chunk and the first and last host-resident chunks; size-independent properties
    cover the rest: every chunk's fp32 parameters changed, and fp16 == RNE(fp32) everywhere."""
    from _harness import N_FULL

    import gc

    gc.collect()
    torch.cuda.empty_cache()  # hand cached blocks of earlier tests back before asking for 113 GB
    free, _ = torch.cuda.mem_get_info()
    if free < 130e9:
        pytest.skip("needs 130 GB of free HBM")
    kw = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    host = list(range(120, 180))
    try:
        h = HybridHarness(180, N_FULL, host, ps.LossScaler(2**12), seed=5, **kw)
    except RuntimeError as e:  # the box cannot pin 56 GB
        pytest.skip(f"cannot allocate the configuration: {e}")
    # seeded contents, cheaper than 720 random fills: a few distinct random chunks, rotated
    base = []
    for _ in range(3):
        p = torch.empty(N_FULL, device="cuda").normal_(0, 0.02, generator=h.gen)
        m = torch.empty(N_FULL, device="cuda").normal_(0, 1e-4, generator=h.gen)
        v = torch.empty(N_FULL, device="cuda").normal_(0, 1e-6, generator=h.gen).abs_()
        g = torch.empty(N_FULL, device="cuda").normal_(0, 1e-3, generator=h.gen).mul_(2.0**12).half()
        base.append((p, m, v, g))
    for i in range(180):
        for dst, src in zip(h.payloads(i), base[i % 3]):
            dst.copy_(src)
    torch.cuda.synchronize()
    before = [t[0].view(torch.int32).sum(dtype=torch.int64).item() for t in base]
    for prm in h.params:
        dict.__setitem__(h.opt.state[prm], "step", 99)
    idx = [7, 120, 179]
    oc = h.oracle_chunks(idx)
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(2**12), **kw)
    oopt.step_count = 99
    del base
    h.opt.step()
    torch.cuda.synchronize()
    oopt.step()
    h.compare(oc, idx, what="hybrid configuration")
    # identical inputs give identical outputs wherever the chunk lives: all chunks of one residue class agree
    ref = {}
    for i in range(180):
        p, _, _, hh = h.payloads(i)
        pd = p if p.is_cuda else p.cuda()
        hd = hh if hh.is_cuda else hh.cuda()
        assert torch.equal(pd.half(), hd), f"chunk {i}: fp16 copy is not RNE(fp32)"
        s = pd.view(torch.int32).sum(dtype=torch.int64).item()
        assert s != before[i % 3], f"chunk {i} was not updated"
        assert ref.setdefault(i % 3, s) == s, f"chunk {i} differs from its twins"


class _PartlyFrozen(torch.nn.Module):
    """fc1 is frozen before the engine sees the model; fc2 and `gain` train.  With 1100-element chunks fc1 has the
    first chunk to itself (a position that drops out of the step) and the trainable tensors share the second; with
    2000-element chunks all five tensors share ONE chunk, frozen and trainable side by side."""

    def __init__(self):
        super().__init__()
        self.fc1 = torch.nn.Linear(24, 40)
        self.fc2 = torch.nn.Linear(40, 8)
        self.gain = torch.nn.Parameter(torch.ones(8))
        for p in self.fc1.parameters():
            p.requires_grad_(False)

    def forward(self, x):
        return (self.fc2(torch.tanh(self.fc1(x))) * self.gain).float().pow(2).mean()


@pytest.mark.parametrize("chunk_size", [1100, 2000])
@pytest.mark.parametrize("optim_type,loss_scale", [("AdamW", 0), ("Adam", 128)])
def test_frozen_parameters_are_skipped_like_the_reference_skips_them(optim_type, loss_scale, chunk_size):
    """requires_grad=False parameters are not updated, not decayed and not counted (fp16_cpu_adam.py:566-569), even with
    weight decay and when they share a chunk with trainable ones; the trainable ones match the oracle bit for bit."""
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": optim_type, "params": {"lr": 1e-2, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.1}},
        "fp16": {"enabled": True, "loss_scale": loss_scale, "initial_scale_power": 7, "loss_scale_window": 3, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": chunk_size,
    }
    engine, optimizer = ps.initialize_engine(model_func=_PartlyFrozen, local_rank=0, config=config)
    client = engine.client
    cl = client.chunk_list
    pos = client.positions()
    assert len(pos) == (2 if chunk_size == 1100 else 1)
    frozen = list(engine.module.fc1.parameters())
    masters = [client.access_data(client.param_fp16_to_param_fp32_map[p]) for p in frozen]
    frozen_before = [(p.detach().clone(), m.clone()) for p, m in zip(frozen, masters)]
    spans = tensor_spans(client, optimizer)
    assert len(spans) == 3  # gain, fc2.weight, fc2.bias
    mirror = [{"p32": _snap(cl[q.fp32].payload), "m": _snap(cl[q.exp_avg].payload),
               "v": _snap(cl[q.exp_avg_sq].payload), "p16": _snap(cl[q.fp16].payload)} for q in pos]
    oscaler = oracle.scaler_from_config(config["fp16"])
    oopt = oracle.OptimizerStepOracle(mirror, oscaler, lr=1e-2, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.1,
                                      use_adamw=(optim_type == "AdamW"), tensors=spans)
    x = torch.randn(16, 24, device="cuda").half()
    for it in range(6):
        loss = engine(x * (1.0 if it != 2 or loss_scale else 3e4))  # dynamic scaler: iteration 2 overflows
        engine.backward(loss)
        for q, c in zip(pos, mirror):
            c["p16"][...] = _snap(cl[q.fp16].payload)
        # the slots of frozen parameters still hold the parameters, not zeros
        for p, (p0, _) in zip(frozen, frozen_before):
            assert torch.equal(client.access_data(p), p0)
        optimizer.step()
        torch.cuda.synchronize()
        oopt.check_overflow()
        skipped = oopt.step()
        if loss_scale == 0:
            assert skipped == (it == 2)
        for p, m, (p0, m0) in zip(frozen, masters, frozen_before):
            assert torch.equal(p.detach(), p0) and torch.equal(m, m0), "a frozen parameter moved"
        for q, c in zip(pos, mirror):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                assert_bits_equal(_snap(cl[cid].payload), c[key], f"iteration {it} {key}")
    live = [p for p in engine.module.parameters() if p.requires_grad]
    assert optimizer.state[live[0]]["step"] == (5 if loss_scale == 0 else 6)
    assert optimizer.state[frozen[0]]["step"] == 0


def test_training_loop_never_reads_the_step_state_back(monkeypatch):
    """engine.backward multiplies the loss by the device-resident scale; optimizer.step only queues work.  Over eight
    iterations, one of them poisoned, nothing may call ps_state_read (the one synchronising entry point), and the
    result must still be the oracle's bit for bit, scale sequence included."""
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.01}},
        "fp16": {"enabled": True, "loss_scale": 0, "initial_scale_power": 7, "loss_scale_window": 3, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 1100,
    }
    engine, optimizer = ps.initialize_engine(model_func=_MLP, local_rank=0, config=config)
    client = engine.client
    cl = client.chunk_list
    pos = client.positions()
    scaler = optimizer.loss_scaler
    scaler.enable_log(16)
    mirror = [{"p32": _snap(cl[q.fp32].payload), "m": _snap(cl[q.exp_avg].payload),
               "v": _snap(cl[q.exp_avg_sq].payload), "p16": _snap(cl[q.fp16].payload)} for q in pos]
    oscaler = oracle.scaler_from_config(config["fp16"])
    oopt = oracle.OptimizerStepOracle(mirror, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01,
                                      use_adamw=True, tensors=tensor_spans(client, optimizer))
    reads = []
    real_read = ps.DynamicLossScaler._read
    monkeypatch.setattr(ps.DynamicLossScaler, "_read", lambda self: reads.append(1) or real_read(self))
    x = torch.randn(16, 24, device="cuda").half()
    grads_per_iteration, expected_scales = [], []
    for it in range(8):
        loss = engine(x * (1.0 if it != 4 else 3e4))
        engine.backward(loss)
        grads_per_iteration.append([cl[q.fp16].payload.clone() for q in pos])  # device-side copies: no host sync
        optimizer.step()
    assert reads == [], "the training loop read the device-resident step state back"
    monkeypatch.undo()
    torch.cuda.synchronize()
    for it, grads in enumerate(grads_per_iteration):
        for c, g in zip(mirror, grads):
            c["p16"][...] = g.cpu().numpy()
        oopt.check_overflow()
        assert oopt.step() == (it == 4)
        expected_scales.append((it == 4, oscaler.loss_scale))
    for i, (q, c) in enumerate(zip(pos, mirror)):
        for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
            assert_bits_equal(_snap(cl[cid].payload), c[key], f"position {i} {key}")
    log = scaler.read_log()
    assert [(f, s) for f, s in log] == expected_scales and [type(s) for _, s in log] == [type(s) for _, s in expected_scales]
    assert optimizer.state[next(engine.module.parameters())]["step"] == 7
    # the aliasing scale tensor tracks the state
    assert float(scaler.scale_tensor) == scaler.loss_scale == oscaler.loss_scale


class _Deep(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.layers = torch.nn.ModuleList([torch.nn.Linear(16, 16) for _ in range(6)])

    def forward(self, x):
        for layer in self.layers:
            x = torch.tanh(layer(x))
        return x.float().pow(2).mean()


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
def test_engine_places_optimizer_state_by_the_hbm_budget(arithmetic):
    """No policy given, an artificially small HBM budget: initialize_engine keeps the first two positions' optimizer
    state in HBM and puts the other four in pinned host memory (use_hybrid_adam), and training is bit for bit what the
    reference computes under that placement: the operator everywhere, or (arithmetic="torch") the torch formula on the
    resident positions and the operator on the host ones."""
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.01,
                                                  "use_hybrid_adam": True, "arithmetic": arithmetic}},
        "fp16": {"enabled": True, "loss_scale": 0, "initial_scale_power": 7, "loss_scale_window": 3, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 300,
        "client": {"hbm_budget_bytes": 28000},
    }
    engine, optimizer = ps.initialize_engine(model_func=_Deep, local_rank=0, config=config)
    client = engine.client
    assert client.placement["host_positions"] == [2, 3, 4, 5]
    cl = client.chunk_list
    pos = client.positions()
    assert [q.on_host for q in pos] == [False, False, True, True, True, True]
    for q in pos:
        assert cl[q.fp16].payload.is_cuda
        for cid in (q.fp32, q.exp_avg, q.exp_avg_sq):
            assert cl[cid].payload.is_pinned() == q.on_host and cl[cid].payload.is_cuda != q.on_host
    mirror = [{"p32": _snap(cl[q.fp32].payload), "m": _snap(cl[q.exp_avg].payload),
               "v": _snap(cl[q.exp_avg_sq].payload), "p16": _snap(cl[q.fp16].payload)} for q in pos]
    oscaler = oracle.scaler_from_config(config["fp16"])
    oopt = oracle.OptimizerStepOracle(mirror, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01,
                                      use_adamw=True, tensors=tensor_spans(client, optimizer), arithmetic=arithmetic,
                                      operator_chunks=(2, 3, 4, 5))
    x = torch.randn(8, 16, device="cuda").half()
    for it in range(6):
        loss = engine(x * (1.0 if it != 2 else 6e4))
        engine.backward(loss)
        for q, c in zip(pos, mirror):
            c["p16"][...] = _snap(cl[q.fp16].payload)
        optimizer.step()
        torch.cuda.synchronize()
        oopt.check_overflow()
        assert oopt.step() == (it == 2)
        for i, (q, c) in enumerate(zip(pos, mirror)):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                assert_bits_equal(_snap(cl[cid].payload), c[key], f"{arithmetic} iteration {it} position {i} {key}")
        assert optimizer.loss_scaler.loss_scale == oscaler.loss_scale


def test_engine_refuses_host_placement_without_hybrid_adam():
    config = {
        "optimizer": {"type": "Adam", "params": {"lr": 1e-3, "use_hybrid_adam": False}},
        "default_chunk_size": 300,
        "client": {"hbm_budget_bytes": 28000},
    }
    with pytest.raises(RuntimeError, match="use_hybrid_adam is False"):
        ps.initialize_engine(model_func=_Deep, local_rank=0, config=config)
    # with room for everything the switch changes nothing
    config["client"] = {"hbm_budget_bytes": 10**9}
    engine, optimizer = ps.initialize_engine(model_func=_Deep, local_rank=0, config=config)
    assert not any(q.on_host for q in engine.client.positions())


def test_two_host_threads_stream_host_chunks_on_one_gpu_at_the_same_time():
    """Two optimizers with host-resident positions, stepped by two host threads on two streams of the same GPU at the
    same moment (a barrier in front of every step; ctypes drops the GIL inside the call).  Both use the library's
    one set of side streams for that GPU: the calls take turns there, and both must match the oracle bit for bit."""
    import threading

    n, steps = 256 * 1024 + 77, 4
    cases = [
        dict(host=[1, 2, 4], keeps=True, scaler=lambda: ps.LossScaler(2**10), oscaler=lambda: oracle.StaticScalerOracle(2**10),
             kw=dict(lr=1e-3, weight_decay=0.01, use_adamw=True)),
        dict(host=[0, 3], keeps=False, scaler=lambda: ps.DynamicLossScaler(init_scale=2**8, scale_factor=2, scale_window=2),
             oscaler=lambda: oracle.ScalerOracle(init_scale=2**8, scale_factor=2, scale_window=2), kw=dict(lr=1e-4, weight_decay=0.0)),
    ]
    hs = [HybridHarness(5, n, c["host"], c["scaler"](), seed=31 + i, host_keeps_fp16=c["keeps"], **c["kw"]) for i, c in enumerate(cases)]
    for h in hs:
        h.opt.staging_slots = 2
        h.fill_state()
    start = [h.oracle_chunks() for h in hs]
    grads = [[] for _ in hs]  # per harness, per step: the fp16 payloads as the step found them
    barrier = threading.Barrier(2)
    errors = []

    def worker(t):
        try:
            h, stream = hs[t], torch.cuda.Stream()
            scale = 2.0**10 if t == 0 else 2.0**8
            for step in range(steps):
                with torch.cuda.stream(stream):
                    h.fill_grads(1e-3, scale)
                    if t == 1 and step == 1:
                        h.payloads(3)[3][n - 1] = float("inf")  # last element of a host position's fp16 payload
                    grads[t].append([h.download(i)[3] for i in range(5)])
                    barrier.wait(timeout=60)
                    h.opt.step()
            stream.synchronize()
        except Exception as e:  # surfaced by the main thread
            errors.append((t, repr(e)))
            barrier.abort()

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    torch.cuda.synchronize()
    for t, (h, c) in enumerate(zip(hs, cases)):
        oc = start[t]
        oscaler = c["oscaler"]()
        oopt = oracle.OptimizerStepOracle(oc, oscaler, **c["kw"])
        for step in range(steps):
            for i, ch in enumerate(oc):
                ch["p16"][...] = grads[t][step][i]
            oopt.check_overflow()
            assert oopt.step() == (t == 1 and step == 1)
        h.compare(oc, what=f"thread {t}")
        if t == 1:
            assert h.opt.loss_scaler.loss_scale == oscaler.loss_scale and h.opt.loss_scaler.cur_iter == steps


class _DeepPartlyFrozen(_Deep):
    """Six 272-element layers, one per 300-element chunk position.  Frozen: layer 0's weight (so the step's first
    operator call is a bias in the middle of a chunk that also holds a frozen tensor), the biases of layers 1 and 4,
    and all of layer 2 (a position that drops out of the step)."""

    def __init__(self):
        super().__init__()
        for p in (self.layers[0].weight, self.layers[1].bias, self.layers[4].bias, *self.layers[2].parameters()):
            p.requires_grad_(False)


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
@pytest.mark.parametrize("loss_scale", [0, 64])
@pytest.mark.parametrize("host", [(0, 1), (3, 5), (1, 3, 4), (0, 3), (0, 1, 2, 3, 4, 5)])
def test_frozen_parameters_together_with_host_resident_positions(host, loss_scale, arithmetic):
    """Chunks that mix frozen and trainable tensors, some of them with their optimizer state in host memory: the step
    is spread over a tensor-list call (resident tensors), the streamed whole-chunk form (host positions without frozen
    tensors) and staged tensor-list calls (host positions with frozen tensors), under ONE call pattern.  Bit for bit
    what the reference computes under that placement; frozen tensors do not move."""
    torch.manual_seed(1)
    config = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.05,
                                                  "arithmetic": arithmetic}},
        "fp16": {"enabled": True, "loss_scale": loss_scale, "initial_scale_power": 7, "loss_scale_window": 3, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 300,
        "client": {"host_chunk_policy": lambda position: position in host},
    }
    engine, optimizer = ps.initialize_engine(model_func=_DeepPartlyFrozen, local_rank=0, config=config)
    client = engine.client
    cl = client.chunk_list
    pos = client.positions()
    assert [q.on_host for q in pos] == [i in host for i in range(6)]
    frozen = [p for p in engine.module.parameters() if not p.requires_grad]
    assert len(frozen) == 5
    masters = [client.access_data(client.param_fp16_to_param_fp32_map[p]) for p in frozen]
    frozen_before = [(p.detach().clone(), m.clone()) for p, m in zip(frozen, masters)]
    spans = tensor_spans(client, optimizer)
    assert len(spans) == 7 and spans[0] == (0, 256, 16)  # layer 0's bias comes first
    mirror = [{"p32": _snap(cl[q.fp32].payload), "m": _snap(cl[q.exp_avg].payload),
               "v": _snap(cl[q.exp_avg_sq].payload), "p16": _snap(cl[q.fp16].payload)} for q in pos]
    oscaler = oracle.scaler_from_config(config["fp16"])
    oopt = oracle.OptimizerStepOracle(mirror, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.05,
                                      use_adamw=True, tensors=spans, arithmetic=arithmetic, operator_chunks=host)
    x = torch.randn(8, 16, device="cuda").half()
    for it in range(6):
        loss = engine(x * (1.0 if it != 2 or loss_scale else 6e4))  # dynamic scaler: iteration 2 overflows
        engine.backward(loss)
        for q, c in zip(pos, mirror):
            c["p16"][...] = _snap(cl[q.fp16].payload)
        optimizer.step()
        torch.cuda.synchronize()
        oopt.check_overflow()
        assert oopt.step() == (it == 2 and loss_scale == 0)
        for p, m, (p0, m0) in zip(frozen, masters, frozen_before):
            assert torch.equal(p.detach(), p0) and torch.equal(m, m0), "a frozen parameter moved"
        for i, (q, c) in enumerate(zip(pos, mirror)):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                assert_bits_equal(_snap(cl[cid].payload), c[key], f"host={host} iteration {it} position {i} {key}")
        assert optimizer.loss_scaler.loss_scale == oscaler.loss_scale
    kinds = [s[0] for s in optimizer._stages]
    whole_on_host = [i for i in host if i in (3, 5)]
    part_on_host = [i for i in host if i in (0, 1, 4)]
    assert kinds.count("stream") == bool(whole_on_host) and kinds.count("staged") == len(part_on_host)
    assert kinds.count("tensors") == (len(host) < 6)
    # the stage that holds the step's first operator call goes first: the first trainable tensor (position 0), or,
    # with the torch formula on resident state, the first one whose state lives in host memory
    first = 0 if arithmetic == "operator" else min(i for i in host if i != 2)
    assert kinds[0] == ("tensors" if first not in host else "staged" if first in part_on_host else "stream")


def test_freezing_and_unfreezing_parameters_between_steps():
    """requires_grad is looked at every step (fp16_cpu_adam.py:569-571).  Unfreezing before the first step and freezing
    later both follow the reference (oracle with the matching tensor list); a parameter that comes back after it missed
    steps is updated with its own step number, as the reference counts it (fp16_cpu_adam.py:571-574,603)."""
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-2, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.1}},
        "fp16": {"enabled": True, "loss_scale": 128},
        "default_chunk_size": 2000,
    }
    engine, optimizer = ps.initialize_engine(model_func=_PartlyFrozen, local_rank=0, config=config)
    client = engine.client
    cl = client.chunk_list
    pos = client.positions()
    module = engine.module
    for p in module.fc1.parameters():  # frozen when the engine was built (no backward hook): trainable from step 1 on
        p.requires_grad_(True)
    mirror = [{"p32": _snap(cl[q.fp32].payload), "m": _snap(cl[q.exp_avg].payload),
               "v": _snap(cl[q.exp_avg_sq].payload), "p16": _snap(cl[q.fp16].payload)} for q in pos]
    oopt = oracle.OptimizerStepOracle(mirror, oracle.StaticScalerOracle(128), lr=1e-2, betas=(0.9, 0.999), eps=1e-8,
                                      weight_decay=0.1, use_adamw=True, tensors=tensor_spans(client, optimizer))
    assert len(oopt.tensors) == 5
    x = torch.randn(16, 24, device="cuda").half()

    def iterate(what):
        loss = engine(x)
        engine.backward(loss)
        for q, c in zip(pos, mirror):
            c["p16"][...] = _snap(cl[q.fp16].payload)
        optimizer.step()
        torch.cuda.synchronize()
        oopt.step()
        for q, c in zip(pos, mirror):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                assert_bits_equal(_snap(cl[cid].payload), c[key], f"{what} {key}")

    iterate("all five trainable, step 1")
    iterate("all five trainable, step 2")
    module.gain.requires_grad_(False)  # the first tensor of the step drops out: the call pattern moves on
    module.fc2.bias.requires_grad_(False)
    oopt.tensors = tensor_spans(client, optimizer)
    assert len(oopt.tensors) == 3 and optimizer.state[module.gain]["step"] == 2
    gain_before = client.access_data(module.gain).clone()
    iterate("two frozen, step 3")
    iterate("two frozen, step 4")
    assert torch.equal(client.access_data(module.gain), gain_before)
    assert optimizer.state[module.gain]["step"] == 2 and optimizer.state[module.fc2.weight]["step"] == 4
    module.gain.requires_grad_(True)  # stands at 2 steps, the others at 4
    oopt.tensors = tensor_spans(client, optimizer)
    iterate("gain back: its step 3 beside the others' step 5")
    iterate("step 4 beside step 6")
    assert optimizer.state[module.gain]["step"] == 4 and optimizer.state[module.fc2.weight]["step"] == 6
    assert optimizer.state[module.fc2.bias]["step"] == 2


def test_a_failed_launch_in_the_streamed_step_leaves_the_pipeline_usable():
    """ps_adam_step_hybrid makes its side streams wait for the caller's stream before it queues anything; if queuing then
    stops half way (here: the resident chunks' launch reports an error) the caller's stream must still be put behind
    the side streams before the call returns.  The failure is forced from outside, without any fault on the GPU: the
    library asks hipGetLastError after every launch, and an error left in the calling thread's HIP error state by a
    harmless refused call (hipSetDevice of a device that does not exist) is what it then finds.  Afterwards the same
    process streams host chunks again and gets the oracle's bits."""
    import ctypes

    hip = ctypes.CDLL("libamdhip64.so")
    akw = dict(lr=1e-3, weight_decay=0.01, use_adamw=True)
    h = HybridHarness(4, 2048 * 2 + 9, [1, 3], ps.LossScaler(2**8), seed=31, **akw)
    h.fill_state()
    h.fill_grads(1e-3, 2**8)
    h.opt.step()  # a good step first: the side streams exist and have been used
    torch.cuda.synchronize()
    h.fill_grads(1e-3, 2**8)
    torch.cuda.synchronize()
    assert hip.hipSetDevice(9999) != 0
    try:
        h.opt.step()
        forced = False
    except RuntimeError as e:
        forced = True
        assert "ps_adam_step_hybrid" in str(e)
    torch.cuda.synchronize()  # nothing is left waiting on anything
    if not forced:
        pytest.skip("this HIP runtime forgets a refused call's error at the next successful call: a launch failure "
                    "cannot be forced from outside")
    # the pipeline of this process (one per device) goes on working
    g = HybridHarness(4, 2048 * 2 + 9, [0, 2], ps.LossScaler(2**8), seed=32, **akw)
    g.fill_state()
    oc = g.oracle_chunks()
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(2**8), lr=1e-3, weight_decay=0.01, use_adamw=True)
    for step in range(2):
        g.fill_grads(1e-3, 2**8)
        for i, c in enumerate(oc):
            c["p16"][...] = g.download(i)[3]
        g.opt.step()
        torch.cuda.synchronize()
        oopt.step()
        g.compare(oc, what=f"after a failed call, step {step}")
