"""Writes torch_branch_vectors.npz: inputs and outputs of the reference's torch-formula branch
(patrickstar/ops/fp16_cpu_adam.py:245-277 with :364-379, :412-413, :430) as computed by PyTorch's own GPU
kernels, which are what that branch runs on.  Needs a GPU; the call sequence is the one in
tests/test_oracle_torch_formula.py: reference_call_sequence (the statements of those lines, issued on torch tensors).

The fixture lets the CPU test suite hold the oracle's restatement of that branch to the bits torch's GPU kernels
produce, on machines without a GPU.

Run on a GPU machine from the repository root:
    python tests/golden/make_torch_branch_vectors.py --out tests/golden/torch_branch_vectors.npz
"""
import argparse
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))  # tests/
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))  # repository root
from test_oracle_torch_formula import reference_call_sequence  # noqa: E402

CASES = [
    # name, n, first step, steps, lr, beta1, beta2, eps, wd, adamw, loss_scale (None: no scaler), clipping
    ("l2_nodecay_scale8_t1", 1023, 1, 3, 1e-3, 0.9, 0.999, 1e-6, 0.0, False, 8, -1),
    ("adamw_scale2p16_t100", 1023, 100, 2, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, 2**16, -1),
    ("l2_decay_scale2p12_t100", 515, 100, 1, 1e-4, 0.9, 0.999, 1e-8, 0.01, False, 2**12, -1),
    ("adamw_noscaler_t7", 515, 7, 2, 3e-4, 0.8, 0.95, 1e-8, 0.1, True, None, -1),
    ("adamw_scale1000_t13", 515, 13, 2, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, 1000.0, -1),
    ("l2_scale12345_t2500", 257, 2500, 1, 1e-3, 0.95, 0.98, 1e-9, 0.003, False, 12345.678, -1),
    ("adamw_clamped_scale1024_t3", 1023, 3, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, 1024, 0.0017),
]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", required=True)
    args = ap.parse_args()
    assert torch.cuda.is_available(), "the branch runs on torch's GPU kernels: a GPU is needed"
    out = {}
    rng = np.random.default_rng(20240611)
    for name, n, t0, steps, lr, b1, b2, eps, wd, adamw, scale, clip in CASES:
        p = rng.normal(0, 0.02, n).astype(np.float32)
        m = rng.normal(0, 1e-4, n).astype(np.float32) if t0 > 1 else np.zeros(n, np.float32)
        v = np.abs(rng.normal(0, 1e-6, n)).astype(np.float32) if t0 > 1 else np.zeros(n, np.float32)
        if t0 > 1:
            m[:4] = [1e-41, -3e-42, 0.0, 1e-30]  # subnormals and tiny values
            v[:4] = [2e-42, 1e-41, 0.0, 1e-35]
        out[f"{name}/p0"], out[f"{name}/m0"], out[f"{name}/v0"] = p.copy(), m.copy(), v.copy()
        tp, tm, tv = (torch.from_numpy(x).cuda() for x in (p, m, v))
        for k in range(steps):
            s = float(scale) if scale is not None else 1.0
            g = (rng.normal(0, 2e-3 if clip > 0 else 1e-3, n).astype(np.float32) * np.float32(s)).astype(np.float16)
            out[f"{name}/g{k}"] = g.copy()
            reference_call_sequence(tp, torch.from_numpy(g).cuda(), tm, tv, t0 + k, lr, b1, b2, eps, wd, adamw, scale, clip)
            out[f"{name}/p{k + 1}"] = tp.cpu().numpy().copy()
            out[f"{name}/m{k + 1}"] = tm.cpu().numpy().copy()
            out[f"{name}/v{k + 1}"] = tv.cpu().numpy().copy()
            out[f"{name}/h{k + 1}"] = tp.half().cpu().numpy().copy()
    out["meta"] = np.frombuffer(
        json.dumps({"cases": CASES, "torch": torch.__version__, "device": torch.cuda.get_device_name(0)}).encode(),
        dtype=np.uint8,
    )
    np.savez_compressed(args.out, **out)
    print("wrote", args.out, "with", len(out), "arrays from torch", torch.__version__, "on", torch.cuda.get_device_name(0))


if __name__ == "__main__":
    main()
