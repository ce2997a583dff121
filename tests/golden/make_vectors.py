"""Writes tests/golden/adam_vectors.npz and tests/golden/scaler_trajectories.json.

The reference ships no golden vectors for this path and its native operator cannot be built in this image, so
these fixtures are produced by the repository's own CPU oracle AFTER it has been pinned (tests/test_oracle_adam.py,
tests/test_oracle_scaler.py).  They freeze inputs and expected outputs so that (a) a later change of the oracle,
the compiler or libm that alters a single bit is noticed, and (b) the HIP path can be checked against data that
does not depend on running the oracle on the GPU box.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

CASES = [
    # name, n, adamw, wd, lr, eps, loss_scale, grad dtype, first step, consecutive steps
    ("l2_nodecay_scale8_t1", 1023, False, 0.0, 1e-3, 1e-6, 8.0, "f16", 1, 3),
    ("l2_decay_noscale_t1", 1023, False, 0.001, 0.01, 1e-8, -1.0, "f32", 1, 1),
    ("l2_decay_scale32_t1", 515, False, 0.001, 0.01, 1e-8, 32.0, "f16", 1, 1),
    ("adamw_scale2p16_t100_cold", 1023, True, 0.01, 1e-4, 1e-8, 65536.0, "f16", 100, 2),
    ("adamw_scale2p12_t100_cold", 515, True, 0.01, 1e-4, 1e-8, 4096.0, "f16", 100, 1),
    ("adamw_scale1000_truediv_t7", 515, True, 0.01, 1e-3, 1e-8, 1000.0, "f16", 7, 2),
    ("adamw_f32grad_noscale_t5000", 257, True, 0.1, 1e-3, 1e-8, -1.0, "f32", 5000, 1),
]


def main():
    out = {}
    rng = np.random.default_rng(20240607)
    for name, n, adamw, wd, lr, eps, scale, gdt, t0, steps in CASES:
        p = rng.normal(0, 0.02, n).astype(np.float32)
        m = rng.normal(0, 1e-4, n).astype(np.float32) if t0 > 1 else np.zeros(n, np.float32)
        v = np.abs(rng.normal(0, 1e-6, n)).astype(np.float32) if t0 > 1 else np.zeros(n, np.float32)
        m[:4] = [1e-41, -3e-42, 0.0, 1e-30]  # subnormals and tiny values
        v[:4] = [2e-42, 1e-41, 0.0, 1e-35]
        out[f"{name}/p0"], out[f"{name}/m0"], out[f"{name}/v0"] = p.copy(), m.copy(), v.copy()
        o = oracle.AdamOracle(lr, 0.9, 0.999, eps, wd, adamw)
        for k in range(steps):
            s = abs(scale) if scale > 0 else 1.0
            g = rng.normal(0, 1e-3, n).astype(np.float32) * np.float32(s)
            g = g.astype(np.float16) if gdt == "f16" else g
            out[f"{name}/g{k}"] = g.copy()
            o.update(t0 + k, lr, 0.9, 0.999, eps, wd, True, p, g, m, v, scale)
            out[f"{name}/p{k + 1}"], out[f"{name}/m{k + 1}"], out[f"{name}/v{k + 1}"] = p.copy(), m.copy(), v.copy()
            out[f"{name}/h{k + 1}"] = oracle.cast_fp32_to_fp16(p)
    np.savez_compressed(os.path.join(HERE, "adam_vectors.npz"), **out)

    traj = []
    rng = np.random.default_rng(7)
    for kw in (
        dict(init_scale=2**16, scale_factor=2, scale_window=1000, min_scale=1),
        dict(init_scale=2**16, scale_factor=2, scale_window=3, min_scale=1),
        dict(init_scale=4, scale_factor=2, scale_window=2, min_scale=1),
        dict(init_scale=16, scale_factor=2, scale_window=2, min_scale=1, delayed_shift=2),
        dict(init_scale=16, scale_factor=2.0, scale_window=5, min_scale=1, delayed_shift=3, consecutive_hysteresis=True),
        dict(init_scale=1000.0, scale_factor=3, scale_window=2, min_scale=1),
    ):
        flags = [bool(x) for x in (rng.random(60) < 0.25)]
        s = oracle.ScalerOracle(**kw)
        scales = []
        for f in flags:
            s.update_scale(f)
            scales.append([s.loss_scale, "int" if isinstance(s.loss_scale, int) else "float"])
        traj.append({"kwargs": kw, "flags": flags, "scales": scales})
    with open(os.path.join(HERE, "scaler_trajectories.json"), "w") as f:
        json.dump({"cases": CASES, "trajectories": traj}, f, indent=1)
    print("wrote", len(out), "arrays and", len(traj), "trajectories")


if __name__ == "__main__":
    main()
