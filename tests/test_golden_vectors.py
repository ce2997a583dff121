"""Committed fixtures (tests/golden/): the oracle must reproduce them on the CPU, the HIP path on the GPU, bit for bit.
The fixtures come from the repository's pinned oracle (see tests/golden/make_vectors.py), not from the reference,
which holds no vectors for this path."""
import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
VEC = np.load(os.path.join(HERE, "golden", "adam_vectors.npz"))
META = json.load(open(os.path.join(HERE, "golden", "scaler_trajectories.json")))
CASES = [tuple(c) for c in META["cases"]]


def _same(a, b):
    va = a.view(np.uint16 if a.dtype == np.float16 else np.uint32)
    vb = b.view(np.uint16 if b.dtype == np.float16 else np.uint32)
    return np.array_equal(va, vb)


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_oracle_reproduces_golden_vectors(case):
    name, n, adamw, wd, lr, eps, scale, gdt, t0, steps = case
    p, m, v = (VEC[f"{name}/{k}0"].copy() for k in "pmv")
    o = oracle.AdamOracle(lr, 0.9, 0.999, eps, wd, adamw)
    for k in range(steps):
        o.update(t0 + k, lr, 0.9, 0.999, eps, wd, True, p, VEC[f"{name}/g{k}"].copy(), m, v, scale)
        assert _same(p, VEC[f"{name}/p{k + 1}"]) and _same(m, VEC[f"{name}/m{k + 1}"]) and _same(v, VEC[f"{name}/v{k + 1}"])
        assert _same(oracle.cast_fp32_to_fp16(p), VEC[f"{name}/h{k + 1}"])


def test_oracle_reproduces_golden_scale_trajectories():
    for t in META["trajectories"]:
        s = oracle.ScalerOracle(**t["kwargs"])
        for f, (want, typ) in zip(t["flags"], t["scales"]):
            s.update_scale(f)
            assert s.loss_scale == want and ("int" if isinstance(s.loss_scale, int) else "float") == typ


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_hip_operator_reproduces_golden_vectors(case):
    import torch

    from patrickstar_amd import _lib

    name, n, adamw, wd, lr, eps, scale, gdt, t0, steps = case
    lib = _lib.load()
    dp, dm, dv = (torch.from_numpy(VEC[f"{name}/{k}0"].copy()).cuda() for k in "pmv")
    h = torch.zeros(n, dtype=torch.half, device="cuda")
    oid = 950
    _lib.check(lib.ps_adam_create(oid, lr, 0.9, 0.999, eps, wd, int(adamw), 0), "create")
    for k in range(steps):
        g = torch.from_numpy(VEC[f"{name}/g{k}"].copy()).cuda()
        _lib.check(
            lib.ps_adam_update(oid, t0 + k, lr, 0.9, 0.999, eps, wd, 1, dp.data_ptr(), g.data_ptr(), int(gdt == "f16"),
                               dm.data_ptr(), dv.data_ptr(), n, float(scale), h.data_ptr(), _lib.current_stream_handle()),
            "update",
        )
        torch.cuda.synchronize()
        for t, key in ((dp, "p"), (dm, "m"), (dv, "v"), (h, "h")):
            assert _same(t.cpu().numpy(), VEC[f"{name}/{key}{k + 1}"]), f"{name} step {k} {key}"
    lib.ps_adam_destroy(oid)


@pytest.mark.gpu
@pytest.mark.parametrize("case", [c for c in CASES if c[7] == "f16"], ids=[c[0] for c in CASES if c[7] == "f16"])
def test_hip_chunk_step_reproduces_golden_vectors(case):
    """The same vectors through FP16Adam.step(): each case is a one-chunk list (ragged against the 256-element tile)."""
    import torch

    import patrickstar_amd as ps

    name, n, adamw, wd, lr, eps, scale, gdt, t0, steps = case
    client = ps.PatrickStarClient(0, n)
    params = client.append_flat_chunks(1)
    scaler = ps.LossScaler(scale) if scale > 0 else None
    opt = ps.FP16Adam(client, params, loss_scaler=scaler, lr=lr, betas=(0.9, 0.999), eps=eps, weight_decay=wd, use_adamw=adamw)
    q = client.positions()[0]
    cl = client.chunk_list
    for key, cid in (("p", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq)):
        cl[cid].payload.copy_(torch.from_numpy(VEC[f"{name}/{key}0"].copy()))
    dict.__setitem__(opt.state[params[0]], "step", t0 - 1)
    for k in range(steps):
        cl[q.fp16].payload.copy_(torch.from_numpy(VEC[f"{name}/g{k}"].copy()))
        opt.step()
        torch.cuda.synchronize()
        for key, cid in (("p", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("h", q.fp16)):
            assert _same(cl[cid].payload.cpu().numpy(), VEC[f"{name}/{key}{k + 1}"]), f"{name} step {k} {key}"


@pytest.mark.gpu
def test_device_scaler_reproduces_golden_scale_trajectories():
    import patrickstar_amd as ps

    for t in META["trajectories"]:
        s = ps.DynamicLossScaler(**t["kwargs"])
        s.enable_log(len(t["flags"]))
        for f in t["flags"]:
            s.update_scale(f)
        for (flag, got), f, (want, typ) in zip(s.read_log(), t["flags"], t["scales"]):
            assert flag == f and got == want and ("int" if isinstance(got, int) else "float") == typ


# ---- the torch-formula branch: vectors written by PyTorch's own GPU kernels (tests/golden/make_torch_branch_vectors.py)

TVEC = np.load(os.path.join(HERE, "golden", "torch_branch_vectors.npz"))
TCASES = [tuple(c) for c in json.loads(bytes(TVEC["meta"]).decode())["cases"]]


@pytest.mark.parametrize("case", TCASES, ids=[c[0] for c in TCASES])
def test_oracle_reproduces_torch_gpu_kernels_bitwise(case):
    name, n, t0, steps, lr, b1, b2, eps, wd, adamw, scale, clip = case
    p, m, v = (TVEC[f"{name}/{k}0"].copy() for k in "pmv")
    for k in range(steps):
        oracle.torch_formula_update(p, TVEC[f"{name}/g{k}"].copy(), m, v, t0 + k, lr, b1, b2, eps, wd, adamw, scale, clip)
        assert _same(p, TVEC[f"{name}/p{k + 1}"]) and _same(m, TVEC[f"{name}/m{k + 1}"]) and _same(v, TVEC[f"{name}/v{k + 1}"])
        assert _same(oracle.cast_fp32_to_fp16(p), TVEC[f"{name}/h{k + 1}"])


@pytest.mark.gpu
@pytest.mark.parametrize("case", TCASES, ids=[c[0] for c in TCASES])
def test_hip_torch_arithmetic_reproduces_torch_gpu_kernels_bitwise(case):
    import torch

    from patrickstar_amd import _lib

    name, n, t0, steps, lr, b1, b2, eps, wd, adamw, scale, clip = case
    lib = _lib.load()
    dp, dm, dv = (torch.from_numpy(TVEC[f"{name}/{k}0"].copy()).cuda() for k in "pmv")
    oid = 951
    _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, int(adamw), 0), "create")
    _lib.check(lib.ps_adam_set_arithmetic(oid, _lib.PS_ARITH_TORCH), "set_arithmetic")
    if clip > 0:
        _lib.check(lib.ps_adam_set_grad_clamp(oid, clip), "set_grad_clamp")
    for k in range(steps):
        h = torch.from_numpy(TVEC[f"{name}/g{k}"].copy()).cuda()  # gradients in, fp16 parameters out
        rows = _lib.chunk_array([[dp.data_ptr(), dm.data_ptr(), dv.data_ptr(), h.data_ptr()]])
        _lib.check(
            lib.ps_adam_step_chunks(oid, t0 + k, lr, b1, b2, eps, wd, 1, rows, 1, n, None, None,
                                    float(scale) if scale is not None else -1.0, _lib.current_stream_handle()),
            "ps_adam_step_chunks",
        )
        torch.cuda.synchronize()
        for got, key in ((dp, "p"), (dm, "m"), (dv, "v"), (h, "h")):
            assert _same(got.cpu().numpy(), TVEC[f"{name}/{key}{k + 1}"]), (name, key, k)
    lib.ps_adam_destroy(oid)
