"""GPU tests of ``"use_cpu_embedding": True``: the weights of ``nn.Embedding`` modules stay fp32 parameters that
PyTorch manages itself (the reference's ``ParamType.TORCH_BASED``, ``patrickstar/core/preprocess.py:351-364``), the
lookup's output is cast to half (``patrickstar/ops/embedding.py:94-104``), and ``FP16Adam.step`` updates them through the
operator from their fp32 ``.grad`` (``patrickstar/ops/fp16_cpu_adam.py:345-353,415-428``), in ``parameters()`` order
with every other tensor: no overflow probe on them (``patrickstar/core/hook.py:202-203``), nothing restored for them
on a skipped step (``fp16_cpu_adam.py:301-302``), no fp16 copy (``:459-460``).  The reference keeps them in host
memory; here they stay in HBM.

Bar: bit-exact against the CPU oracle fed with the same gradients."""
import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from patrickstar_amd.chunk_layout import ParamType
from _harness import assert_bits_equal

pytestmark = pytest.mark.gpu


class _EmbNet(torch.nn.Module):
    """parameters() order: emb.dummy (empty, fp16, not trainable), emb.weight (fp32, PyTorch's own: the step's FIRST
    operator call), pos.dummy, pos.weight, fc1.weight, fc1.bias, fc2.weight, fc2.bias."""

    def __init__(self):
        super().__init__()
        self.emb = torch.nn.Embedding(40, 24)
        self.pos = torch.nn.Embedding(6, 24)
        self.fc1 = torch.nn.Linear(24, 20)
        self.fc2 = torch.nn.Linear(20, 8)

    def forward(self, idx, amplify=1.0):
        h = self.emb(idx) + self.pos(torch.arange(idx.shape[1], device=idx.device))[None]
        assert h.dtype == torch.half
        h = torch.tanh(self.fc1(h * amplify))
        return self.fc2(h).float().pow(2).mean()


def _snap(t):
    return t.detach().to("cpu", copy=True).numpy()


def _config(loss_scale, arithmetic, clip=None, host=()):
    cfg = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.05,
                                                  "arithmetic": arithmetic}},
        "fp16": {"enabled": True, "loss_scale": loss_scale, "initial_scale_power": 7, "loss_scale_window": 3,
                 "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 700,
        "use_cpu_embedding": True,
    }
    if clip is not None:
        cfg["gradient_clipping"] = clip
    if host:
        cfg["client"] = {"host_chunk_policy": lambda position: position in host}
        cfg["default_chunk_size"] = 520  # fc1 (500 elements) fills the first position, fc2 (168) goes to a second
    return cfg


class _Run:
    def __init__(self, loss_scale, arithmetic, clip=None, seed=0, host=()):
        torch.manual_seed(seed)
        self.config = _config(loss_scale, arithmetic, clip, host)
        self.engine, self.opt = ps.initialize_engine(model_func=_EmbNet, local_rank=0, config=self.config)
        self.client, self.module = self.engine.client, self.engine.module
        self.cl, self.pos = self.client.chunk_list, self.client.positions()
        self.dynamic = loss_scale == 0
        self.idx = torch.randint(0, 40, (5, 6), device="cuda")
        self.managed = [p for p in self.module.parameters() if p.ps_attr.param_type == ParamType.TORCH_BASED and p.requires_grad]
        self.oscaler = oracle.scaler_from_config(self.config["fp16"])
        self.chunks = [{"p32": _snap(self.cl[q.fp32].payload), "m": _snap(self.cl[q.exp_avg].payload),
                        "v": _snap(self.cl[q.exp_avg_sq].payload), "p16": _snap(self.cl[q.fp16].payload)} for q in self.pos]
        # one oracle "chunk" per parameter that PyTorch manages itself, behind the chunk positions
        self.own = [{"p32": _snap(p).ravel(), "m": _snap(self.opt.state[p]["exp_avg"]).ravel(),
                     "v": _snap(self.opt.state[p]["exp_avg_sq"]).ravel(), "g32": np.zeros(p.numel(), np.float32)}
                    for p in self.managed]
        index = self.client.chunk_tensor_index
        position_of = {q.fp16: i for i, q in enumerate(self.pos)}
        spans = []
        for p in self.module.parameters():
            if not p.requires_grad:
                continue
            if p.ps_attr.param_type == ParamType.TORCH_BASED:
                spans.append((len(self.pos) + [id(q) for q in self.managed].index(id(p)), 0, p.numel()))
            else:
                info = index.get_tensor_info(p.ps_attr.data_id())
                spans.append((position_of[info.chunk_id], info.start_offset, info.numel))
        self.spans = spans
        self.oopt = oracle.OptimizerStepOracle(
            self.chunks + self.own, self.oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.05, use_adamw=True,
            tensors=spans, arithmetic=arithmetic, gradient_clipping=clip if clip is not None else -1, operator_chunks=tuple(host))

    def iterate(self, what, poison=False):
        poison = poison and self.dynamic
        loss = self.engine(self.idx, amplify=6e4 if poison else 1.0)
        self.engine.backward(loss)
        for q, c in zip(self.pos, self.chunks):
            c["p16"][...] = _snap(self.cl[q.fp16].payload)
        for p, c in zip(self.managed, self.own):
            if p.requires_grad:
                assert p.grad is not None and p.grad.dtype == torch.float
                c["g32"][...] = _snap(p.grad).ravel()
        self.opt.step()
        torch.cuda.synchronize()
        self.oopt.check_overflow()
        assert self.oopt.step() == poison, what
        for i, (q, c) in enumerate(zip(self.pos, self.chunks)):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                assert_bits_equal(_snap(self.cl[cid].payload), c[key], f"{what}: position {i} {key}")
        for k, (p, c) in enumerate(zip(self.managed, self.own)):
            assert_bits_equal(_snap(p).ravel(), c["p32"], f"{what}: own parameter {k}")
            assert_bits_equal(_snap(self.opt.state[p]["exp_avg"]).ravel(), c["m"], f"{what}: own parameter {k} exp_avg")
            assert_bits_equal(_snap(self.opt.state[p]["exp_avg_sq"]).ravel(), c["v"], f"{what}: own parameter {k} exp_avg_sq")
        if self.dynamic:
            assert self.opt.loss_scaler.loss_scale == self.oscaler.loss_scale, what


def test_the_layout_is_the_references():
    r = _Run(128, "operator")
    names = [n for n, _ in r.module.named_parameters()]
    assert names[:4] == ["emb.dummy", "emb.weight", "pos.dummy", "pos.weight"]
    assert r.module.emb.weight.dtype == torch.float and r.module.emb.weight.is_cuda
    assert r.module.emb.dummy.dtype == torch.half and r.module.emb.dummy.numel() == 0 and not r.module.emb.dummy.requires_grad
    assert next(r.module.parameters()).dtype == torch.half
    assert len(r.managed) == 2 and r.spans[0][0] == len(r.pos)  # the step's first operator call is emb.weight
    # the embedding weights are in no chunk: the chunk lists hold the two linear layers only
    assert sum(s[2] for s in r.spans if s[0] < len(r.pos)) == 24 * 20 + 20 + 20 * 8 + 8
    assert r.opt.state[r.module.emb.dummy].get("exp_avg") is None


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
@pytest.mark.parametrize("loss_scale", [0, 128])
def test_training_steps_with_fp32_embeddings(loss_scale, arithmetic):
    r = _Run(loss_scale, arithmetic, seed=1)
    for k in (1, 2, 3):
        r.iterate(f"step {k}")
    assert r.opt._plan["kind"] == "each"
    r.iterate("poisoned", poison=True)
    for k in (4, 5, 6, 7):
        r.iterate(f"step {k}")
    steps = [r.opt.state[p]["step"] for p in r.module.parameters() if p.requires_grad]
    assert steps == [7 if r.dynamic else 8] * len(steps)  # a static scaler skips nothing


@pytest.mark.parametrize("loss_scale", [0, 128])
def test_per_parameter_numbers_and_freezing_apply_to_them_too(loss_scale):
    r = _Run(loss_scale, "operator", seed=2)
    m = r.module
    r.iterate("step 1")
    m.pos.weight.requires_grad_(False)
    r.oopt.tensors = [s for s in r.spans if s != r.spans[1]]
    r.iterate("pos.weight frozen, step 2")
    r.iterate("pos.weight frozen, step 3")
    m.pos.weight.requires_grad_(True)
    r.oopt.tensors = r.spans
    r.opt.state[m.emb.weight]["lr"] = 2e-3
    r.oopt.state(r.spans[0])["lr"] = 2e-3
    r.iterate("thawed two steps behind, emb.weight at another learning rate")
    r.iterate("poisoned", poison=True)
    r.iterate("and on")
    skipped = 1 if r.dynamic else 0
    assert r.opt.state[m.pos.weight]["step"] == 4 - skipped and r.opt.state[m.emb.weight]["step"] == 6 - skipped


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
def test_with_optimizer_state_of_a_chunk_position_in_host_memory(arithmetic):
    """The second chunk position keeps fp32 master, momentum and variance in pinned host memory (hybrid Adam): its
    tensors take the operator's arithmetic whatever the optimizer's, the embeddings theirs, the first position the
    optimizer's."""
    r = _Run(0, arithmetic, seed=6, host=(1,))
    assert len(r.pos) == 2 and r.pos[1].on_host and not r.pos[0].on_host
    for k in (1, 2):
        r.iterate(f"step {k}")
    r.iterate("poisoned", poison=True)
    r.iterate("step 3")


def test_gradient_clamp_reaches_the_fp32_gradients():
    r = _Run(128, "operator", clip=1e-4, seed=3)
    for k in (1, 2, 3):
        r.iterate(f"clamped step {k}")


def test_checkpoint_round_trip_with_fp32_embeddings():
    """Optimizer and model state of a run with fp32 embeddings reloaded into a new engine: the two runs continue
    bit for bit (but for what a fresh operator object changes in the first call of the first step: compared against
    the oracle, whose new optimizer has a fresh object too)."""
    r = _Run(0, "operator", seed=4)
    for k in (1, 2, 3):
        r.iterate(f"step {k}")
    osd, msd = r.opt.state_dict(), r.engine.state_dict()
    assert "emb.weight" in msd and msd["emb.weight"].dtype == torch.float and "emb.dummy" in msd
    r2 = _Run(0, "operator", seed=9)
    r2.engine.load_state_dict(msd)
    r2.opt.load_state_dict(osd)
    for p, q in zip(r.module.parameters(), r2.module.parameters()):
        assert torch.equal(p.detach().float(), q.detach().float())
    for p, q in zip(r.managed, r2.managed):
        assert torch.equal(r.opt.state[p]["exp_avg"], r2.opt.state[q]["exp_avg"])
        assert r2.opt.state[q]["step"] == 3
    # the oracle of the resumed run: present state, step counts and scaler as saved, a fresh operator object
    r2.idx = r.idx
    r2.oscaler.cur_scale, r2.oscaler.cur_iter = r.oscaler.cur_scale, r.oscaler.cur_iter
    r2.oscaler.last_overflow_iter, r2.oscaler.cur_hysteresis = r.oscaler.last_overflow_iter, r.oscaler.cur_hysteresis
    for c, q in zip(r2.chunks, r2.pos):
        for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
            c[key][...] = _snap(r2.cl[cid].payload)
    for p, c in zip(r2.managed, r2.own):
        c["p32"][...] = _snap(p).ravel()
        c["m"][...] = _snap(r2.opt.state[p]["exp_avg"]).ravel()
        c["v"][...] = _snap(r2.opt.state[p]["exp_avg_sq"]).ravel()
    r2.oopt.step_count = 3
    for span in r2.spans:
        r2.oopt.state(span)["step"] = 3
    for k in (4, 5):
        r2.iterate(f"resumed step {k}")
