"""GPU parity of the torch-formula arithmetic (arithmetic="torch", PS_ARITH_TORCH).

The reference's branch for optimizer state held in GPU memory (FP16Adam.torch_adam_update,
patrickstar/ops/fp16_cpu_adam.py:245-277) is a sequence of PyTorch element-wise kernels.  Two
independent checks, both BIT-EXACT on fp32 param / m / v and the fp16 copy:
  * against PyTorch itself: the literal call sequence of those lines run on torch's GPU kernels,
    on the same GPU, from the same inputs;
  * against the CPU oracle (oracle.torch_formula_update), through the C ABI.
"""
import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from patrickstar_amd import _lib
from _harness import ChunkHarness, HybridHarness
from test_oracle_torch_formula import reference_call_sequence

pytestmark = pytest.mark.gpu


def same_bits(a, b):
    ia = a.view(torch.int32) if a.dtype == torch.float32 else a.view(torch.int16)
    ib = b.view(torch.int32) if b.dtype == torch.float32 else b.view(torch.int16)
    return bool(torch.equal(ia, ib))


class TorchMirror:
    """fp32 param / m / v of every chunk kept a second time on the GPU and advanced by the
    reference's own torch calls."""

    def __init__(self, harness):
        self.h = harness
        self.state = [tuple(t.clone() for t in harness.payloads(i)[:3]) for i in range(harness.n_chunks)]

    def step(self, step, lr, betas, eps, wd, adamw, loss_scale, clip=-1):
        for i, (p, m, v) in enumerate(self.state):
            g16 = self.h.payloads(i)[3].clone()  # the gradients, before the product overwrites them
            reference_call_sequence(p, g16, m, v, step, lr, betas[0], betas[1], eps, wd, adamw, loss_scale, clip)

    def compare(self, what):
        for i, (p, m, v) in enumerate(self.state):
            gp, gm, gv, gh = self.h.payloads(i)
            assert same_bits(gp, p), f"{what}: chunk {i} fp32 param differs from torch in {(gp != p).sum().item()} elements"
            assert same_bits(gm, m), f"{what}: chunk {i} exp_avg differs from torch in {(gm != m).sum().item()} elements"
            assert same_bits(gv, v), f"{what}: chunk {i} exp_avg_sq differs from torch in {(gv != v).sum().item()} elements"
            assert same_bits(gh, p.half()), f"{what}: chunk {i} fp16 param differs from torch's .half()"


CASES = [
    # lr, betas, eps, wd, adamw, static scale (None: no scaler), grad std multiplier
    (1e-3, (0.9, 0.999), 1e-6, 0.0, False, 8),
    (1e-4, (0.9, 0.999), 1e-8, 0.01, True, 2**12),
    (1e-4, (0.9, 0.999), 1e-8, 0.01, False, 2**16),
    (3e-4, (0.8, 0.95), 1e-8, 0.1, True, None),
    (1e-3, (0.9, 0.999), 1e-8, 0.01, True, 1000.0),  # x / 1000.0 is x * float(1 / 1000.0) on the GPU
    (1e-3, (0.95, 0.98), 1e-9, 0.003, False, 12345.678),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("chunk_size", [256 * 12, 256 * 5 + 19])
def test_static_steps_match_torch_and_oracle_bitwise(case, chunk_size):
    lr, betas, eps, wd, adamw, scale = case
    scaler = ps.LossScaler(scale) if scale is not None else None
    h = ChunkHarness(3, chunk_size, scaler, seed=chunk_size, lr=lr, betas=betas, eps=eps, weight_decay=wd,
                     use_adamw=adamw, arithmetic="torch")
    h.fill_state(m_std=0, v_std=0)
    mirror = TorchMirror(h)
    oc = h.oracle_chunks()
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(scale) if scale is not None else None, lr=lr,
                                      betas=betas, eps=eps, weight_decay=wd, use_adamw=adamw, arithmetic="torch")
    for step in range(1, 6):
        h.fill_grads(1e-3, float(scale or 1.0))
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        mirror.step(step, lr, betas, eps, wd, adamw, scale)
        h.opt.step()
        torch.cuda.synchronize()
        oopt.step()
        mirror.compare(f"step {step}")
        h.compare(oc, what=f"step {step}")
    assert h.opt.state[h.params[0]]["step"] == 5


def test_cold_step_from_a_checkpoint_matches_torch():
    """state["step"] = 99 restored, then step 100: bias corrections 1 - beta ** 100 from pow."""
    lr, betas, eps, wd = 1e-4, (0.9, 0.999), 1e-8, 0.01
    h = ChunkHarness(2, 256 * 9 + 3, ps.LossScaler(2**12), seed=3, lr=lr, betas=betas, eps=eps, weight_decay=wd,
                     use_adamw=True, arithmetic="torch")
    h.fill_state()
    sd = h.opt.state_dict()
    for st in sd["state"].values():
        st["step"] = 99
    h.opt.load_state_dict(sd)
    mirror = TorchMirror(h)
    h.fill_grads(1e-3, 2.0**12)
    mirror.step(100, lr, betas, eps, wd, True, 2**12)
    oc = h.oracle_chunks()
    h.opt.step()
    torch.cuda.synchronize()
    mirror.compare("step 100")
    for c in oc:
        oracle.torch_formula_update(c["p32"], c["p16"], c["m"], c["v"], 100, lr, betas[0], betas[1], eps, wd, True, 2**12)
        c["p16"][...] = oracle.cast_fp32_to_fp16(c["p32"])
    h.compare(oc, what="step 100")


@pytest.mark.parametrize("adamw", [True, False])
def test_device_gated_steps_match_torch_and_oracle_bitwise(adamw):
    """Dynamic scaler: scale, step counter and bias corrections come from the device-resident state;
    flagged steps are skipped.  The torch mirror is told what the oracle state machine decided."""
    kw = dict(init_scale=2**14, scale_factor=2, scale_window=4, min_scale=1)
    lr, betas, eps, wd = 1e-3, (0.9, 0.999), 1e-8, 0.01
    scaler = ps.DynamicLossScaler(**kw)
    h = ChunkHarness(3, 256 * 7 + 5, scaler, seed=5, lr=lr, betas=betas, eps=eps, weight_decay=wd, use_adamw=adamw,
                     arithmetic="torch")
    h.fill_state(m_std=0, v_std=0)
    mirror = TorchMirror(h)
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=lr, betas=betas, eps=eps, weight_decay=wd, use_adamw=adamw,
                                      arithmetic="torch")
    poisoned = {3: float("inf"), 8: float("nan")}
    for it in range(14):
        h.fill_grads(1e-3, float(oscaler.loss_scale))
        if it in poisoned:
            h.payloads(1)[3][17] = poisoned[it]
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        if it not in poisoned:
            mirror.step(oopt.step_count + 1, lr, betas, eps, wd, adamw, oscaler.loss_scale)
        h.opt.step()
        torch.cuda.synchronize()
        oopt.check_overflow()
        assert oopt.step() is (it in poisoned)
        mirror.compare(f"iteration {it}")
        h.compare(oc, what=f"iteration {it}")
        assert scaler.loss_scale == oscaler.loss_scale and type(scaler.loss_scale) is type(oscaler.loss_scale)
    assert h.opt.state[h.params[0]]["step"] == 12 == oopt.step_count


def test_gradient_clamp_matches_torch():
    lr, betas, eps, clip, scale = 1e-3, (0.9, 0.999), 1e-8, 0.0017, 1024
    h = ChunkHarness(2, 256 * 6 + 1, ps.LossScaler(scale), seed=8, gradient_clipping=clip, lr=lr, betas=betas, eps=eps,
                     arithmetic="torch")
    h.fill_state()
    mirror = TorchMirror(h)
    h.fill_grads(2e-3, float(scale))
    bound = min(65504.0, clip * scale)
    assert (h.payloads(0)[3].float().abs() > bound).float().mean().item() > 0.05
    oc = h.oracle_chunks()
    mirror.step(1, lr, betas, eps, 0.0, False, scale, clip)
    h.opt.step()
    torch.cuda.synchronize()
    mirror.compare("clamped step")
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(scale), lr=lr, betas=betas, eps=eps, gradient_clipping=clip,
                                      arithmetic="torch")
    oopt.step()
    h.compare(oc, what="clamped step")


@pytest.mark.parametrize("dynamic", [False, True])
def test_hybrid_placement_resident_chunks_torch_host_chunks_operator(dynamic):
    """What the reference computes under a hybrid placement: torch formula for chunks whose state is in GPU memory,
    the native operator for chunks whose state is in host memory."""
    lr, betas, eps, wd = 1e-4, (0.9, 0.999), 1e-8, 0.01
    kw = dict(init_scale=2**12, scale_factor=2, scale_window=1000, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw) if dynamic else ps.LossScaler(2**12)
    host = [1, 3]
    h = HybridHarness(4, 2048 + 77, host, scaler, seed=31, lr=lr, betas=betas, eps=eps, weight_decay=wd, use_adamw=True,
                      arithmetic="torch")
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = oracle.ScalerOracle(**kw) if dynamic else oracle.StaticScalerOracle(2**12)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=lr, betas=betas, eps=eps, weight_decay=wd, use_adamw=True,
                                      arithmetic="torch", operator_chunks=host)
    for step in range(3):
        h.fill_grads(1e-3, 2.0**12)
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        torch.cuda.synchronize()
        oopt.check_overflow()
        oopt.step()
        h.compare(oc, what=f"hybrid step {step}")


def test_device_bias_corrections_follow_python_pow():
    """1 - beta ** t held in the device state for t = adam_step + 1, against Python's own float ** int, over
    3000 consecutive clean steps for two beta pairs; the float constants derived from them must be identical."""
    lib = _lib.load()
    for betas in ((0.9, 0.999), (0.95, 0.98)):
        s = ps.DynamicLossScaler(init_scale=2**10, scale_window=10**9)
        s.materialize("cuda:0", betas=betas)
        worst = 0
        for t in range(1, 3001):
            st = s._read()
            assert st.adam_step == t - 1
            bc1, bc2 = 1 - betas[0] ** t, 1 - betas[1] ** t
            assert np.float32(-(1e-3 / st.bias_correction1_next)) == np.float32(-(1e-3 / bc1))
            assert np.float32(1.0 / np.sqrt(st.bias_correction2_next)) == np.float32(1.0 / np.sqrt(bc2))
            worst = max(worst, abs(st.bias_correction1_next - bc1) / bc1, abs(st.bias_correction2_next - bc2) / bc2)
            s.update_scale(False)
        assert worst < 4e-16


def test_nonfinite_gradients_propagate_like_torch():
    """A static scaler never skips: inf / nan gradients poison exactly the elements torch's kernels poison (NaN payload
    bits are not compared, positions and every finite element are), and the subnormal range behaves the same."""
    lr, betas, eps, wd, scale = 1e-3, (0.9, 0.999), 1e-8, 0.01, 8
    h = ChunkHarness(2, 256 * 4 + 9, ps.LossScaler(scale), seed=13, lr=lr, betas=betas, eps=eps, weight_decay=wd,
                     use_adamw=True, arithmetic="torch")
    h.fill_state()
    h.fill_grads(1e-3, float(scale))
    g = h.payloads(0)[3]
    g[3], g[64], g[300], g[1000] = float("inf"), float("-inf"), float("nan"), 65504.0
    p, m, v, _ = h.payloads(1)
    m[:4] = torch.tensor([1e-41, -3e-42, 0.0, 1e-30])
    v[:4] = torch.tensor([2e-42, 1e-41, 0.0, 1e-35])
    h.payloads(1)[3][:4] = torch.tensor([6e-8, -6e-8, 0.0, 1e-7]).half()  # subnormal fp16 gradients
    mirror = TorchMirror(h)
    mirror.step(1, lr, betas, eps, wd, True, scale)
    h.opt.step()
    torch.cuda.synchronize()
    for i, (tp, tm, tv) in enumerate(mirror.state):
        for got, want in zip(h.payloads(i)[:3], (tp, tm, tv)):
            assert torch.equal(torch.isnan(got), torch.isnan(want))
            ok = ~torch.isnan(want)
            assert torch.equal(got[ok].view(torch.int32), want[ok].view(torch.int32))
        hh, th = h.payloads(i)[3], tp.half()
        assert torch.equal(torch.isnan(hh), torch.isnan(th))
        ok = ~torch.isnan(th)
        assert torch.equal(hh[ok].view(torch.int16), th[ok].view(torch.int16))
    assert torch.isnan(h.payloads(0)[0][300])
