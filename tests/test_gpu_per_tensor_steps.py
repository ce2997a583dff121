"""GPU tests of what the reference keeps PER PARAMETER: the step number (``state[p]["step"]``, counted only while the
parameter is trainable, fp16_cpu_adam.py:571-574) and the hyper-parameters (``state[p]["lr" | "betas" | "eps" |
"weight_decay"]``, :596-601), each operator call getting its own tensor's numbers (:403-428); and of resuming from a
checkpoint that holds them (:660-694).

Bar as everywhere: bit-exact against the CPU oracle, whose per-tensor sequence is pinned in tests/test_oracle_step.py."""
import logging

import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from _harness import ChunkHarness, assert_bits_equal, tensor_spans

pytestmark = pytest.mark.gpu


class _Net(torch.nn.Module):
    """parameters() order (the order of the reference's operator calls): gain, fc1.weight, fc1.bias, fc2.weight,
    fc2.bias, fc3.weight, fc3.bias.  With 700-element chunks: fc1 (24*20+20 = 500) has the first position, fc2
    (20*12+12 = 252) and fc3 (12*8+8 = 104) share the second and `gain` (the parent's own parameter, registered when
    its children are done) follows them there: the step's first call is a tensor at the end of the SECOND chunk."""

    def __init__(self):
        super().__init__()
        self.fc1 = torch.nn.Linear(24, 20)
        self.fc2 = torch.nn.Linear(20, 12)
        self.fc3 = torch.nn.Linear(12, 8)
        self.gain = torch.nn.Parameter(torch.ones(8))

    def forward(self, x):
        h = torch.tanh(self.fc2(torch.tanh(self.fc1(x))))
        return (self.fc3(h) * self.gain).float().pow(2).mean()


def _snap(t):
    return t.detach().to("cpu", copy=True).numpy()


def _config(loss_scale, arithmetic, host=(), chunk=700, betas=(0.9, 0.999)):
    cfg = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-3, "betas": betas, "eps": 1e-8, "weight_decay": 0.05,
                                                  "arithmetic": arithmetic}},
        "fp16": {"enabled": True, "loss_scale": loss_scale, "initial_scale_power": 7, "loss_scale_window": 4,
                 "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": chunk,
    }
    if host:
        cfg["client"] = {"host_chunk_policy": lambda position: position in host}
    return cfg


class _Run:
    """An engine over `_Net` and the oracle fed with the same gradients, compared bit for bit after every step."""

    def __init__(self, loss_scale, arithmetic, host=(), seed=0, betas=(0.9, 0.999), model=_Net):
        torch.manual_seed(seed)
        self.config = _config(loss_scale, arithmetic, host, betas=betas)
        self.engine, self.opt = ps.initialize_engine(model_func=model, local_rank=0, config=self.config)
        self.client = self.engine.client
        self.cl = self.client.chunk_list
        self.pos = self.client.positions()
        self.module = self.engine.module
        self.arithmetic, self.host, self.dynamic = arithmetic, tuple(host), loss_scale == 0
        self.x = torch.randn(16, 24, device="cuda").half()
        self.oscaler = oracle.scaler_from_config(self.config["fp16"])
        self.new_oracle(betas=betas)

    def mirror(self):
        return [{"p32": _snap(self.cl[q.fp32].payload), "m": _snap(self.cl[q.exp_avg].payload),
                 "v": _snap(self.cl[q.exp_avg_sq].payload), "p16": _snap(self.cl[q.fp16].payload)} for q in self.pos]

    def new_oracle(self, betas=(0.9, 0.999), step=0):
        """A new optimizer on the oracle's side: a FRESH operator object behind it."""
        self.chunks = self.mirror()
        self.oopt = oracle.OptimizerStepOracle(
            self.chunks, self.oscaler, lr=1e-3, betas=betas, eps=1e-8, weight_decay=0.05, use_adamw=True,
            tensors=tensor_spans(self.client, self.opt), arithmetic=self.arithmetic, operator_chunks=self.host)
        self.oopt.step_count = step

    def span(self, p):
        info = self.client.chunk_tensor_index.get_tensor_info(p.ps_attr.data_id())
        position_of = {q.fp16: i for i, q in enumerate(self.pos)}
        return (position_of[info.chunk_id], info.start_offset, info.numel)

    def set(self, p, key, value):
        """Write one state[p] entry on both sides."""
        self.opt.state[p][key] = value
        self.oopt.state(self.span(p))[key] = value

    def trainable_changed(self):
        self.oopt.tensors = tensor_spans(self.client, self.opt)

    def iterate(self, what, poison=False):
        """`poison`: overflowing activations -> inf / nan gradients (only with a dynamic scaler, which then skips the
        step; a static scaler would let the nan spread)."""
        poison = poison and self.dynamic
        loss = self.engine(self.x * (6e4 if poison else 1.0))
        self.engine.backward(loss)
        for q, c in zip(self.pos, self.chunks):
            c["p16"][...] = _snap(self.cl[q.fp16].payload)
        self.opt.step()
        torch.cuda.synchronize()
        self.oopt.check_overflow()
        skipped = self.oopt.step()
        assert skipped == poison, what
        for i, (q, c) in enumerate(zip(self.pos, self.chunks)):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                assert_bits_equal(_snap(self.cl[cid].payload), c[key], f"{what}: position {i} {key}")
        if self.dynamic:
            assert self.opt.loss_scaler.loss_scale == self.oscaler.loss_scale, what

    def steps(self):
        return [self.opt.state[p]["step"] for p in self.module.parameters()]

    def oracle_steps(self):
        return [self.oopt.state(self.span(p))["step"] for p in self.module.parameters()]


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
@pytest.mark.parametrize("loss_scale", [0, 128])
def test_a_thawed_parameter_is_updated_with_its_own_step_number(loss_scale, arithmetic):
    """freeze -> k steps -> thaw: the parameter that sat out stands k steps behind and its operator call (or its torch
    formula) gets ITS step number, the others theirs; a skipped step in between advances nobody; freezing the
    parameter that defined the common counter changes nothing for the rest."""
    r = _Run(loss_scale, arithmetic)
    m = r.module
    r.iterate("all trainable, step 1")
    r.iterate("all trainable, step 2")
    m.fc2.weight.requires_grad_(False)
    m.gain.requires_grad_(False)
    r.trainable_changed()
    for k in (3, 4, 5):
        r.iterate(f"fc2.weight and gain frozen, step {k}")
    assert r.steps() == [2, 5, 5, 2, 5, 5, 5] == r.oracle_steps()
    m.fc2.weight.requires_grad_(True)  # stands at 2, the others at 5; gain stays frozen
    r.trainable_changed()
    r.iterate("fc2.weight back, its step 3 beside step 6")
    assert r.opt._plan["kind"] == "each"
    r.iterate("poisoned", poison=True)
    r.iterate("fc2.weight at 4 beside 7")
    assert r.steps() == ([2, 7, 7, 4, 7, 7, 7] if r.dynamic else [2, 8, 8, 5, 8, 8, 8]) == r.oracle_steps()
    m.fc1.weight.requires_grad_(False)  # the parameter the common counter was taken from
    m.gain.requires_grad_(True)  # now the first trainable parameter: the counter is its own, the others stand ahead
    r.trainable_changed()
    r.iterate("fc1.weight frozen, gain back at step 3")
    r.iterate("one more")
    want = [4, 7, 9, 6, 9, 9, 9] if r.dynamic else [4, 8, 10, 7, 10, 10, 10]
    assert r.steps() == want == r.oracle_steps()
    # everybody in step again (by hand): back to one fused call over whole chunks
    for p in m.parameters():
        r.set(p, "step", 20)
    m.fc1.weight.requires_grad_(True)
    r.trainable_changed()
    r.iterate("all at 21")
    assert r.opt._plan["kind"] == "uniform" and r.steps() == [21] * 7


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
@pytest.mark.parametrize("loss_scale", [0, 128])
def test_hyper_parameters_written_for_some_parameters_only(loss_scale, arithmetic):
    """state[p]["lr"] for one layer, no decay for `gain`, other betas and eps for fc3: every tensor is updated with its
    own numbers; betas that differ from the previous call's restart beta^t from pow (cpu_adam.h:145-150)."""
    r = _Run(loss_scale, arithmetic, seed=1)
    m = r.module
    r.iterate("uniform, step 1")
    for p in m.fc2.parameters():
        r.set(p, "lr", 5e-4)
    r.set(m.gain, "weight_decay", 0.0)
    for p in m.fc3.parameters():
        r.set(p, "betas", (0.8, 0.99))
        r.set(p, "eps", 1e-6)
    for k in (2, 3):
        r.iterate(f"three hyper-parameter sets, step {k}")
    assert r.opt._plan["kind"] == "each"
    r.iterate("poisoned", poison=True)
    r.iterate("after the skipped step")
    # gain's decay really is off: its fp32 master moved by the Adam term only (checked against the oracle above);
    # now make everything agree again, with the NEW numbers everywhere
    for p in m.parameters():
        for key, value in (("lr", 5e-4), ("weight_decay", 0.0), ("betas", (0.8, 0.99)), ("eps", 1e-6)):
            r.set(p, key, value)
    r.iterate("uniform again, other betas than the optimizer was built with")
    assert r.opt._plan["kind"] == "uniform"
    r.iterate("and once more")
    assert r.steps() == r.oracle_steps()


@pytest.mark.parametrize("layerwise", [False, True])
def test_a_learning_rate_schedule_waits_for_nothing(layerwise):
    """The reference's step reads the learning rate from state[p]["lr"] (fp16_cpu_adam.py:596-601; param_groups is
    copied once, :111-116), so a schedule writes state[p]["lr"] of every parameter before every step.  With a dynamic
    scaler the step numbers live on the device: re-planning after such writes must not read them back (no host
    synchronisation inside the training loop), with one rate for all parameters or one per layer, one layer standing
    two steps behind in the second case.  Bit-exact against the oracle under the same schedule."""
    r = _Run(0, "operator", seed=5)
    m = r.module
    scaler = r.opt.loss_scaler
    watched, reads = [False], []
    read = scaler._read

    def counting_read(notify=True):
        if watched[0]:
            reads.append(1)
        return read(notify)

    scaler._read = counting_read
    step = r.opt.step

    def watched_step(*a, **k):
        watched[0] = True
        try:
            return step(*a, **k)
        finally:
            watched[0] = False

    r.opt.step = watched_step
    if layerwise:
        m.fc2.weight.requires_grad_(False)
        r.trainable_changed()
        r.iterate("fc2.weight sits out, step 1")
        r.iterate("fc2.weight sits out, step 2")
        m.fc2.weight.requires_grad_(True)
        r.trainable_changed()
        r.iterate("thawed: this plan reads the counter back once")
        reads.clear()
    decay = {id(p): (0.8 ** i if layerwise else 1.0) for i, p in enumerate(m.parameters())}
    for k in range(1, 7):
        watched[0] = True
        for p in m.parameters():
            r.set(p, "lr", 1e-3 * decay[id(p)] * min(1.0, k / 4))  # warm-up, then flat
        watched[0] = False
        r.iterate(f"scheduled step {k}", poison=(k == 3))
        assert r.opt._plan["kind"] == ("each" if layerwise else "uniform")
    assert not reads, f"{len(reads)} read-backs of the device state inside the loop"
    assert r.steps() == r.oracle_steps()


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
@pytest.mark.parametrize("loss_scale", [0, 128])
def test_betas_changed_after_construction_reach_the_step(loss_scale, arithmetic):
    """The reference hands state[p]["betas"] to the operator on every call (fp16_cpu_adam.py:404-407).  A whole-list,
    device-decided step takes no betas as arguments: the device-resident state must be given the new ones."""
    r = _Run(loss_scale, arithmetic, seed=2)
    for k in (1, 2, 3):
        r.iterate(f"step {k}")
    for p in r.module.parameters():
        r.set(p, "betas", (0.85, 0.98))
    r.iterate("new betas: beta^t restarts from pow")
    assert r.opt._plan["kind"] == "uniform"
    r.iterate("poisoned", poison=True)
    r.iterate("the running product continues with the new betas")
    r.iterate("and again")


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
@pytest.mark.parametrize("loss_scale", [0, 128])
def test_resume_with_a_frozen_last_parameter_and_other_betas(loss_scale, arithmetic):
    """Save at t = 7 with the LAST parameter frozen and betas that are not the constructor's, load into a NEW engine
    and optimizer, take one more step: the trainable parameters go on with step 8 (not 1: the frozen parameter's own
    count of 0 plays no part) and the saved betas; the new optimizer's operator object is fresh, so every call
    evaluates pow."""
    a = _Run(loss_scale, arithmetic, seed=3)
    assert list(a.module.parameters())[-1] is a.module.fc3.bias
    a.module.fc3.bias.requires_grad_(False)
    a.trainable_changed()
    for p in a.module.parameters():
        a.set(p, "betas", (0.85, 0.98))
    for k in range(1, 8):
        a.iterate(f"run A step {k}", poison=(k == 4 and a.dynamic))
    n_clean = 6 if a.dynamic else 7
    assert a.steps() == [n_clean] * 6 + [0]
    model_sd, optim_sd = a.engine.state_dict(), a.opt.state_dict()
    assert [optim_sd["state"][i]["step"] for i in range(7)] == [n_clean] * 6 + [0]

    b = _Run(loss_scale, arithmetic, seed=77)  # other initial weights, the constructor's betas
    b.module.fc3.bias.requires_grad_(False)
    b.engine.load_state_dict(model_sd)
    b.opt.load_state_dict(optim_sd)
    assert b.steps() == [n_clean] * 6 + [0]
    for p, q in zip(a.module.parameters(), b.module.parameters()):
        assert torch.equal(a.client.access_data(a.client.param_fp16_to_param_fp32_map[p]),
                           b.client.access_data(b.client.param_fp16_to_param_fp32_map[q]))
    if b.dynamic:
        for k in range(7):
            b.oscaler.update_scale(k == 3)  # the scaler travelled with the checkpoint
        assert b.opt.loss_scaler.loss_scale == b.oscaler.loss_scale
    b.new_oracle(betas=(0.85, 0.98), step=n_clean)
    b.oopt.state(b.span(b.module.fc3.bias))["step"] = 0
    b.iterate("first step after the reload")
    assert b.steps() == [n_clean + 1] * 6 + [0] == b.oracle_steps()
    b.iterate("second step after the reload")
    # the same checkpoint into the optimizer that wrote it: it stays in step with its own operator object
    a.opt.load_state_dict(optim_sd)
    a.iterate("run A continues after loading its own checkpoint")


@pytest.mark.parametrize("loss_scale", [0, 128])
def test_thaw_with_optimizer_state_in_host_memory(loss_scale):
    """Per-tensor step numbers when the second position's optimizer state lives in pinned host memory: those tensors
    take the operator's arithmetic, read and written over the link in place, in the same call order."""
    for arithmetic in ("operator", "torch"):
        r = _Run(loss_scale, arithmetic, host=(1,), seed=4)
        m = r.module
        assert [q.on_host for q in r.pos] == [False, True]
        r.iterate("step 1")
        m.fc3.bias.requires_grad_(False)
        m.fc1.bias.requires_grad_(False)
        r.trainable_changed()
        r.iterate("step 2 without two biases")
        r.iterate("step 3 without two biases")
        m.fc3.bias.requires_grad_(True)
        m.fc1.bias.requires_grad_(True)
        r.trainable_changed()
        r.iterate("both back")
        assert r.opt._plan["kind"] == "each"
        r.iterate("poisoned", poison=True)
        r.iterate("and on")
        assert r.steps() == r.oracle_steps()


def test_a_call_whose_step_is_the_previous_calls_plus_one_continues_the_product():
    """Three flat chunks through FP16Adam; chunk 0 sits out one step, so that afterwards it stands one behind chunk 1,
    which is called right after it: chunk 1's call then MULTIPLIES chunk 0's pow(beta, t) by beta in the middle of
    the step (IncrementStep looks only at the call before).  Host- and device-decided."""
    for dynamic in (False, True):
        kw = dict(init_scale=2**8, scale_factor=2, scale_window=1000, min_scale=1)
        scaler = ps.DynamicLossScaler(**kw) if dynamic else ps.LossScaler(2**8)
        h = ChunkHarness(3, 2048 + 300, scaler, seed=5, lr=1e-3, weight_decay=0.01)
        h.fill_state()
        oc = h.oracle_chunks()
        oscaler = oracle.ScalerOracle(**kw) if dynamic else oracle.StaticScalerOracle(2**8)
        oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-3, weight_decay=0.01)
        spans = list(oopt.tensors)

        def step(what, active):
            for i, p in enumerate(h.params):
                p.requires_grad_(i in active)
            oopt.tensors = [spans[i] for i in active]
            h.fill_grads(1e-3, 2**8)
            for i, c in enumerate(oc):
                c["p16"][...] = h.download(i)[3]
            h.opt.step()
            torch.cuda.synchronize()
            oopt.check_overflow()
            assert oopt.step() is False
            h.compare(oc, what=f"{'device' if dynamic else 'host'}-decided, {what}")

        step("step 1", [0, 1, 2])
        step("chunk 0 sits out", [1, 2])
        step("chunk 0 at 2, chunk 1 at 3 multiplies, chunk 2 at 3 takes pow", [0, 1, 2])
        step("the same relation again", [0, 1, 2])
        assert [h.opt.state[p]["step"] for p in h.params] == [3, 4, 4]


def test_overflow_warning_is_written_when_the_scaler_is_next_read(caplog):
    """fp16_cpu_adam.py:551-556 logs "Gradient overflow! Update loss scale from X to Y." on every skipped step.  A
    device-decided step does not tell the host; the lines appear at the next read-back, one per skipped step, with the
    oracle's numbers (and Python types: the first halving turns the int 128 into a float)."""
    r = _Run(0, "operator", seed=6)
    scales = []
    with caplog.at_level(logging.WARNING, logger="patrickstar_amd"):
        for k in range(6):
            before = r.oscaler.loss_scale
            r_poison = k in (1, 4)
            loss = r.engine(r.x * (6e4 if r_poison else 1.0))
            r.engine.backward(loss)
            for q, c in zip(r.pos, r.chunks):
                c["p16"][...] = _snap(r.cl[q.fp16].payload)
            r.opt.step()
            r.oopt.check_overflow()
            assert r.oopt.step() == r_poison
            if r_poison:
                scales.append((before, r.oscaler.loss_scale))
        assert not [rec for rec in caplog.records if "Gradient overflow" in rec.getMessage()], "nothing was read back yet"
        assert r.opt.loss_scaler.loss_scale == r.oscaler.loss_scale  # ONE read-back
        lines = [rec.getMessage() for rec in caplog.records if "Gradient overflow" in rec.getMessage()]
        assert lines == [f"Gradient overflow! Update loss scale from {a} to {b}." for a, b in scales]
        assert lines[0] == "Gradient overflow! Update loss scale from 128 to 64.0."
        caplog.clear()
        r.opt.loss_scaler.loss_scale
        r.opt.state_dict()
        assert not caplog.records, "every skipped step is reported once"


def test_padding_is_skipped_only_while_zeros_stay_zeros():
    """The zeros behind a chunk's last tensor are left alone (they are a fixed point of the update).  With eps = 0 they
    are not: the reference's arithmetic writes 0 / 0 into the padding, and then so does the step."""
    n, used = 4096 + 512, 3000
    for dynamic in (False, True):
        for eps in (1e-8, 0.0):
            kw = dict(init_scale=2**8, scale_factor=2, scale_window=1000, min_scale=1)
            scaler = ps.DynamicLossScaler(**kw) if dynamic else ps.LossScaler(2**8)
            h = ChunkHarness(2, n, scaler, used_numel_last=used, seed=8, lr=1e-3, eps=eps, weight_decay=0.01, use_adamw=True)
            h.fill_state()
            assert h.opt._build_tables() and list(h.opt._used) == [n, used]
            oc = h.oracle_chunks()
            oscaler = oracle.ScalerOracle(**kw) if dynamic else oracle.StaticScalerOracle(2**8)
            oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-3, eps=eps, weight_decay=0.01, use_adamw=True)
            for step in range(2):
                h.fill_grads(1e-3, 2**8)
                for i, c in enumerate(oc):
                    c["p16"][...] = h.download(i)[3]
                h.opt.step()
                torch.cuda.synchronize()
                oopt.check_overflow()
                oopt.step()
                what = f"dynamic={dynamic} eps={eps} step {step}"
                if eps > 0:
                    h.compare(oc, what=what)
                else:
                    # a NaN's sign and payload are not part of the bar: same bits in front of the padding, NaNs in
                    # the same places behind it
                    h.compare(oc[:1], indices=[0], what=what)
                    for got, key in zip(h.download(1), ("p32", "m", "v", "p16")):
                        assert_bits_equal(got[:used], oc[1][key][:used], f"{what} chunk 1 {key}")
                        assert np.array_equal(np.isnan(got[used:]), np.isnan(oc[1][key][used:])), (what, key)
                        keep = ~np.isnan(got[used:])
                        assert np.array_equal(got[used:][keep], oc[1][key][used:][keep]), (what, key)
            tail = h.download(1)[0][used:]
            assert np.all(tail == 0) if eps > 0 else np.all(np.isnan(tail))


@pytest.mark.parametrize("seed", [21, 22, 23])
@pytest.mark.parametrize("loss_scale", [0, 128])
def test_random_schedules_of_freezing_and_state_writes(loss_scale, seed):
    """Thirty iterations in which, before each step, something a user may do to the optimizer happens at random:
    parameters are frozen and thawed, learning rates are written for all parameters (a schedule) or for one, weight
    decay, eps or betas for one or for all, step numbers are read (a read-back) or written by hand, the whole state goes
    through state_dict() / load_state_dict(); with a dynamic scaler some iterations overflow.  After every step every
    payload must equal the oracle's bit for bit, and every parameter's step number the reference's count."""
    rng = np.random.default_rng(seed)
    arithmetic = "torch" if seed == 23 else "operator"
    r = _Run(loss_scale, arithmetic, seed=seed)
    params = list(r.module.parameters())
    number = {id(p): i for i, p in enumerate(params)}
    for it in range(30):
        what = f"seed {seed} iteration {it}"
        for _ in range(int(rng.integers(0, 3))):
            action = int(rng.integers(0, 8))
            if action == 0:  # freeze or thaw one parameter (never the last trainable one)
                p = params[int(rng.integers(0, len(params)))]
                if not p.requires_grad or sum(q.requires_grad for q in params) > 1:
                    p.requires_grad_(not p.requires_grad)
                    r.trainable_changed()
                    what += f"; requires_grad[{number[id(p)]}]={p.requires_grad}"
            elif action == 1:  # a learning-rate schedule
                lr = float(rng.choice([1e-3, 8e-4, 5e-4]))
                for p in params:
                    r.set(p, "lr", lr)
                what += f"; lr={lr} for all"
            elif action == 2:
                p = params[int(rng.integers(0, len(params)))]
                r.set(p, "lr", float(rng.choice([1e-3, 2e-3])))
                what += f"; lr[{number[id(p)]}]"
            elif action == 3:
                p = params[int(rng.integers(0, len(params)))]
                key, value = [("weight_decay", 0.0), ("weight_decay", 0.05), ("eps", 1e-6), ("eps", 1e-8)][int(rng.integers(0, 4))]
                r.set(p, key, value)
                what += f"; {key}[{number[id(p)]}]={value}"
            elif action == 4:
                betas = [(0.9, 0.999), (0.85, 0.98)][int(rng.integers(0, 2))]
                targets = params if rng.random() < 0.5 else [params[int(rng.integers(0, len(params)))]]
                for p in targets:
                    r.set(p, "betas", betas)
                what += f"; betas={betas} for {len(targets)}"
            elif action == 5:  # somebody looks at the step numbers
                assert r.steps() == r.oracle_steps(), what
            elif action == 6:  # ... or writes one
                p = params[int(rng.integers(0, len(params)))]
                r.set(p, "step", int(rng.integers(0, 40)))
                what += f"; step[{number[id(p)]}] written"
            else:  # the optimizer's state out and in again (the same optimizer: its operator object runs on)
                r.opt.load_state_dict(r.opt.state_dict())
                what += "; state reloaded"
        r.iterate(what, poison=rng.random() < 0.15)
    assert r.steps() == r.oracle_steps()


def test_a_step_with_per_tensor_numbers_replays_from_a_hip_graph():
    """The device-decided per-tensor step (probe, the small kernel that forms every call's constants from the
    device-resident state, the update kernels, the scale update) is a fixed sequence of launches too: tensors stand at
    fixed DISTANCES from the device's counter, so one captured graph serves later iterations, clean and poisoned.
    Every replay is compared with the oracle, with eager work and synchronisation in between."""
    kw = dict(init_scale=2**10, scale_factor=2, scale_window=3, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw)
    h = ChunkHarness(3, 256 * 9 + 7, scaler, seed=78, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    spans = list(oopt.tensors)
    # the second tensor at another learning rate, the third four steps ahead of the others
    h.opt.state[h.params[1]]["lr"] = 5e-4
    oopt.state(spans[1])["lr"] = 5e-4
    h.opt.state[h.params[2]]["step"] = 4
    oopt.state(spans[2])["step"] = 4

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
        assert scaler.loss_scale == oscaler.loss_scale

    one_iteration(h.opt.step, 0)  # eager: makes the plan, the tensor table and the workspace; nothing is allocated afterwards
    assert h.opt._plan["kind"] == "each"
    graph = torch.cuda.CUDAGraph()
    h.fill_grads(1e-3, float(oscaler.loss_scale))
    for i, c in enumerate(oc):
        c["p16"][...] = h.download(i)[3]
    with torch.cuda.graph(graph):
        h.opt.step()
    graph.replay()
    torch.cuda.synchronize()
    oopt.check_overflow()
    assert oopt.step() is False
    h.compare(oc, what="first replay")
    for it in range(2, 9):
        one_iteration(graph.replay, it)
    assert [h.opt.state[p]["step"] for p in h.params] == [7, 7, 11] == [oopt.state(s)["step"] for s in spans]
