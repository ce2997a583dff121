"""GPU parity of the per-tensor operator-call pattern inside ONE fused step.

The reference calls the native operator once per tensor with the same step number
(patrickstar/ops/fp16_cpu_adam.py:336-428); Adam_Optimizer::IncrementStep (cpu_adam.h:143-162) lets only the first call
of a step continue the running float product beta^t and makes every later call evaluate pow.  The fused entry points
take a ps_call_pattern that says which elements the first call covered; everything here is bit-exact against the
step-level oracle, which literally makes one operator call per tensor."""
import ctypes
import math

import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from patrickstar_amd import _lib
from _harness import ChunkHarness, assert_bits_equal

pytestmark = pytest.mark.gpu


class RawChunks:
    """C chunks of n elements on the device (optionally at unaligned bases) with a host mirror in oracle form."""

    def __init__(self, C, n, seed, offs=(0, 0, 0, 0)):
        rng = np.random.default_rng(seed)
        self.C, self.n, self.offs = C, n, offs
        self.host = [
            {"p32": rng.normal(0, 0.02, n).astype(np.float32), "m": rng.normal(0, 1e-4, n).astype(np.float32),
             "v": np.abs(rng.normal(0, 1e-6, n)).astype(np.float32), "p16": np.zeros(n, np.float16)}
            for _ in range(C)
        ]
        self.dev = []
        rows = []
        for c in self.host:
            bufs = []
            for key, off in zip(("p32", "m", "v", "p16"), offs):
                t = torch.zeros(n + 8, dtype=torch.half if key == "p16" else torch.float, device="cuda")
                t[off:off + n].copy_(torch.from_numpy(c[key]))
                bufs.append(t)
            self.dev.append(bufs)
            rows.append([t[off:].data_ptr() for t, off in zip(bufs, offs)])
        self.table = _lib.chunk_array(rows)

    def new_grads(self, rng, scale, poison=None):
        for ci, (c, bufs) in enumerate(zip(self.host, self.dev)):
            c["p16"][...] = (rng.normal(0, 1e-3, self.n) * scale).astype(np.float16)
            if poison is not None and poison[0] == ci:
                c["p16"][poison[1]] = np.float16("inf")
            bufs[3][self.offs[3]:self.offs[3] + self.n].copy_(torch.from_numpy(c["p16"]))

    def compare(self, what):
        torch.cuda.synchronize()
        for ci, (c, bufs) in enumerate(zip(self.host, self.dev)):
            for key, t, off in zip(("p32", "m", "v", "p16"), bufs, self.offs):
                assert_bits_equal(t[off:off + self.n].cpu().numpy(), c[key], f"{what}: chunk {ci} {key}")


# the first call's tensor starts and ends inside tiles (256 elements), in the middle of the SECOND chunk
N = 256 * 9 + 37
TENSORS = [(1, 300, 1000), (0, 0, 700), (0, 700, N - 700), (1, 0, 300), (1, 1300, N - 1300), (2, 0, N)]


@pytest.mark.parametrize("offs", [(0, 0, 0, 0), (1, 2, 3, 4)])
@pytest.mark.parametrize("adamw,wd,scale", [(True, 0.01, 2.0**12), (False, 0.01, 1000.0)])
def test_host_decided_steps_follow_the_per_tensor_pattern(adamw, wd, scale, offs):
    lib = _lib.load()
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    R = RawChunks(3, N, seed=1, offs=offs)
    rng = np.random.default_rng(2)
    oopt = oracle.OptimizerStepOracle(R.host, oracle.StaticScalerOracle(scale), lr=lr, betas=(b1, b2), eps=eps,
                                      weight_decay=wd, use_adamw=adamw, tensors=TENSORS)
    oid = 840
    _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, int(adamw), 0), "create")
    calls = _lib.call_pattern(len(TENSORS), *TENSORS[0])
    for step in (1, 2, 3, 4, 5, 6, 100, 101):
        R.new_grads(rng, scale)
        oopt.step_count = step - 1
        _lib.check(
            lib.ps_adam_step_chunks(oid, step, lr, b1, b2, eps, wd, 1, R.table, 3, N, None, calls, scale,
                                    _lib.current_stream_handle()),
            "ps_adam_step_chunks",
        )
        oopt.step()
        R.compare(f"step {step}")
    lib.ps_adam_destroy(oid)


def test_the_pattern_changes_bits_and_a_missing_pattern_means_one_call():
    """Same inputs through calls=NULL (the whole list is one operator call) and through a 6-call pattern at step 3,
    where the two branches of IncrementStep give different bias corrections: the results must differ, and each must
    match its own oracle."""
    lib = _lib.load()
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    outs = []
    for tensors in (None, TENSORS):
        R = RawChunks(3, N, seed=5)
        rng = np.random.default_rng(6)
        one_call = [(0, 0, N)]  # a single native call cannot span chunks in the oracle: drive its object by hand below
        oid = 841
        _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, 0.0, 0, 0), "create")
        native = oracle.AdamOracle(lr, b1, b2, eps, 0.0, False)
        oopt = oracle.OptimizerStepOracle(R.host, None, lr=lr, betas=(b1, b2), eps=eps, tensors=tensors or one_call)
        for step in (1, 2, 3):
            R.new_grads(rng, 1.0)
            calls = _lib.call_pattern(len(tensors), *tensors[0]) if tensors else None
            _lib.check(
                lib.ps_adam_step_chunks(oid, step, lr, b1, b2, eps, 0.0, 1, R.table, 3, N, None, calls, -1.0,
                                        _lib.current_stream_handle()),
                "ps_adam_step_chunks",
            )
            if tensors:
                oopt.step()
            else:
                native.advance(step, b1, b2)
                native.set(lr, eps, 0.0, True)
                for c in R.host:
                    assert oracle.lib().oracle_adam_span(native._buf, c["p32"].ctypes.data, c["p16"].ctypes.data, 1,
                                                         c["m"].ctypes.data, c["v"].ctypes.data, N, -1.0, 0) > 0
                    c["p16"][...] = oracle.cast_fp32_to_fp16(c["p32"])
            R.compare(f"{'pattern' if tensors else 'one call'} step {step}")
        outs.append(np.concatenate([c["p32"] for c in R.host]))
        lib.ps_adam_destroy(oid)
    differ = (outs[0].view(np.uint32) != outs[1].view(np.uint32)).mean()
    assert differ > 0.05, differ  # the call pattern is not a no-op


def test_device_gated_steps_follow_the_per_tensor_pattern():
    lib = _lib.load()
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 0.01
    kw = dict(init_scale=2**10, scale_factor=2, scale_window=3, min_scale=1)
    scaler = ps.DynamicLossScaler(**kw)
    scaler.materialize("cuda:0", betas=(b1, b2))
    oscaler = oracle.ScalerOracle(**kw)
    R = RawChunks(3, N, seed=11)
    rng = np.random.default_rng(12)
    oopt = oracle.OptimizerStepOracle(R.host, oscaler, lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd, use_adamw=True,
                                      tensors=TENSORS)
    oid = 842
    _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, 1, 0), "create")
    calls = _lib.call_pattern(len(TENSORS), *TENSORS[0])
    skipped = []
    for it in range(9):
        R.new_grads(rng, float(oscaler.loss_scale), poison=(2, N - 1) if it in (2, 6) else None)
        s = _lib.current_stream_handle()
        _lib.check(lib.ps_overflow_scan_chunks(R.table, 3, N, None, scaler.state_ptr, s), "scan")
        _lib.check(lib.ps_adam_step_chunks_gated(oid, lr, eps, wd, 1, R.table, 3, N, None, calls, scaler.state_ptr, s), "gated")
        scaler.update_scale(None, operator_calls=len(TENSORS))
        oopt.check_overflow()
        skipped.append(oopt.step())
        R.compare(f"iteration {it}")
        assert scaler.loss_scale == oscaler.loss_scale
    assert skipped == [False, False, True, False, False, False, True, False, False]
    assert scaler.adam_step == 7 == oopt.step_count
    # a reloaded optimizer (fresh operator object behind step 7): the first call of step 8 evaluates pow as well
    scaler._seed_step(7)
    oopt2 = oracle.OptimizerStepOracle(R.host, oscaler, lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd, use_adamw=True,
                                       tensors=TENSORS)
    oopt2.step_count = 7
    for it in range(2):
        R.new_grads(rng, float(oscaler.loss_scale))
        s = _lib.current_stream_handle()
        _lib.check(lib.ps_adam_step_chunks_gated(oid, lr, eps, wd, 1, R.table, 3, N, None, calls, scaler.state_ptr, s), "gated")
        scaler.update_scale(None, operator_calls=len(TENSORS))
        oopt2.step()
        R.compare(f"after reload, iteration {it}")
    lib.ps_adam_destroy(oid)


@pytest.mark.parametrize("betas", [(0.9, 0.999), (0.8, 0.99), (0.95, 0.9999)])
@pytest.mark.parametrize("calls", [1, 3])
def test_device_beta_powers_equal_the_operator_objects_over_2500_steps(betas, calls):
    """The device keeps the operator object's state machine (running product for the first call of a step, pow for the
    others) without a host in the loop; read back after every step it must equal what IncrementStep computes, where pow
    is the C library's on the host and a double-double squaring loop on the device."""
    lib = _lib.load()
    b1, b2 = (np.float32(b) for b in betas)
    scaler = ps.DynamicLossScaler(init_scale=2**10, scale_factor=2, scale_window=10**6)
    scaler.materialize("cuda:0", betas=betas)
    cur1 = cur2 = np.float32(1.0)
    for t in range(1, 2501):
        # before step t: what its first call and its later calls will use
        if calls == 1:
            first1, first2 = np.float32(cur1 * b1), np.float32(cur2 * b2)
        else:
            first1 = np.float32(np.float32(math.pow(float(b1), t - 1)) * b1)
            first2 = np.float32(np.float32(math.pow(float(b2), t - 1)) * b2)
        rest1, rest2 = np.float32(math.pow(float(b1), t)), np.float32(math.pow(float(b2), t))
        st = scaler._read()
        assert (st.adam_step, st.beta1_t_next, st.beta2_t_next) == (t - 1, first1, first2), (t, st.beta1_t_next, first1)
        assert (st.beta1_t_rest, st.beta2_t_rest) == (rest1, rest2), t
        cur1, cur2 = (first1, first2) if calls == 1 else (rest1, rest2)
        scaler.update_scale(False, operator_calls=calls)
    st = scaler._read()
    assert st.operator_step == 2500 and st.beta1_t_cur == cur1 and st.beta2_t_cur == cur2


def test_steps_without_operator_calls_leave_the_operator_object_alone():
    """With the torch formula on every chunk the operator is never called: its step stays where it was, and the
    first call that does come takes the cold (pow) branch."""
    scaler = ps.DynamicLossScaler(init_scale=4, scale_factor=2, scale_window=10**6)
    scaler.materialize("cuda:0", betas=(0.9, 0.999))
    for _ in range(5):
        scaler.update_scale(False, operator_calls=0)
    st = scaler._read()
    assert st.adam_step == 5 and st.operator_step == 0 and st.beta1_t_cur == 1.0
    assert st.beta1_t_next == st.beta1_t_rest == np.float32(math.pow(float(np.float32(0.9)), 6))
    scaler.update_scale(False, operator_calls=1)  # step 6 through the operator, cold
    st = scaler._read()
    assert st.operator_step == 6 and st.beta1_t_cur == np.float32(math.pow(float(np.float32(0.9)), 6))
    assert st.beta1_t_next == np.float32(st.beta1_t_cur * np.float32(0.9))


def test_call_pattern_argument_checks():
    lib = _lib.load()
    lib.ps_adam_create(843, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0)
    buf = torch.zeros(1024, device="cuda")
    h = torch.zeros(1024, dtype=torch.half, device="cuda")
    rows = _lib.chunk_array([[buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), h.data_ptr()]] * 2)
    s = _lib.current_stream_handle()
    E = _lib.PS_ERR_BAD_ARG

    def step(calls):
        return lib.ps_adam_step_chunks(843, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, rows, 2, 512, None, calls, -1.0, s)

    assert step(_lib.call_pattern(0)) == E and b"n_calls" in lib.ps_last_error()
    assert step(_lib.call_pattern(2, 2, 0, 8)) == E and b"first_chunk" in lib.ps_last_error()
    assert step(_lib.call_pattern(2, -1, 0, 8)) == E
    assert step(_lib.call_pattern(2, 0, 500, 13)) == E and b"does not fit" in lib.ps_last_error()
    assert step(_lib.call_pattern(2, 0, 513, 0)) == 0  # a first call without elements: nothing to place
    assert lib.ps_adam_step_chunks_gated(843, 1e-3, 1e-8, 0.0, 1, rows, 2, 512, None, _lib.call_pattern(3, 5, 0, 1),
                                         ctypes.c_void_p(buf.data_ptr()), s) == E
    torch.cuda.synchronize()
    lib.ps_adam_destroy(843)


def test_fp16adam_derives_the_pattern_from_its_parameters():
    """Four flat parameters (one per chunk), ten consecutive steps from step 1 with a static scale: FP16Adam has to
    hand the pattern "4 calls, the first one is chunk 0" to the library by itself."""
    h = ChunkHarness(4, 256 * 20 + 3, loss_scaler=ps.LossScaler(8), lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    h.fill_state(m_std=0, v_std=0)
    oc = h.oracle_chunks()
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(8), lr=1e-3, betas=(0.9, 0.999), eps=1e-8)
    for step in range(10):
        h.fill_grads(1e-3, 8)
        for i, c in enumerate(oc):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        oopt.step()
        h.compare(oc, what=f"step {step + 1}")
    assert h.opt._operator_calls == 4 and h.opt.state[h.params[0]]["step"] == 10
