"""Pins the loss-scale state machine of the oracle (patrickstar/fp16/loss_scaler.py:107-182).

The reference asserts its loss-scale sequence nowhere (unitest/test_loss_scale.py:242-250
only prints), so the trajectories below are derived by hand from the rules:
  overflow:   shrink now if delayed_shift == 1 or the hysteresis counter is at 1,
              else spend one hysteresis credit; remember the iteration
  clean step: grow when (iteration - last overflow iteration) is a multiple of the window
  always:     iteration += 1
"""
import numpy as np
import pytest

from oracle import ScalerOracle, StaticScalerOracle, scaler_from_config


def run(scaler, flags):
    out = []
    for f in flags:
        scaler.update_scale(bool(f))
        out.append(scaler.loss_scale)
    return out


def same(a, b):
    """Equal values AND equal Python types (int stays int until the first true division)."""
    return len(a) == len(b) and all(x == y and type(x) is type(y) for x, y in zip(a, b))


def test_hand_trajectory_window3():
    s = ScalerOracle(init_scale=2**16, scale_factor=2, scale_window=3, min_scale=1)
    flags = [0, 0, 0, 1, 0, 0, 0, 1, 1]
    # iter 0,1: (it+1)%3 != 0; iter 2: grow; iter 3: shrink (last=3); iter 4,5: no; iter 6: (6-3)%3==0 grow;
    # iter 7, 8: shrink twice
    want = [65536, 65536, 131072, 65536.0, 65536.0, 65536.0, 131072.0, 65536.0, 32768.0]
    assert same(run(s, flags), want)
    assert s.cur_iter == 9 and s.last_overflow_iter == 8


def test_first_growth_is_on_the_window_th_clean_step():
    for w in (1, 2, 5, 1000):
        s = ScalerOracle(init_scale=4, scale_factor=2, scale_window=w)
        traj = run(s, [0] * (2 * w))
        assert traj[: w - 1] == [4] * (w - 1)
        assert traj[w - 1] == 8 and traj[2 * w - 1] == 16
        assert all(type(x) is int for x in traj)


def test_overflow_on_a_due_growth_suppresses_it():
    s = ScalerOracle(init_scale=8, scale_factor=2, scale_window=3)
    # growth is due at iter 2; an overflow there halves instead, and the next growth is 3 clean iterations later
    assert same(run(s, [0, 0, 1, 0, 0, 0, 0]), [8, 8, 4.0, 4.0, 4.0, 8.0, 8.0])


def test_min_scale_clamp_returns_the_min_scale_object():
    s = ScalerOracle(init_scale=4, scale_factor=2, scale_window=2, min_scale=1)
    # 4/2=2.0, 2.0/2=1.0 (max(1.0, 1) keeps the first of equals), max(0.5, 1) -> the int 1, stays; then growth 1*2 = 2 (int)
    # iter 3: overflow, last=3; iter 4: 1; iter 5: (5-3)%2==0 -> grow
    assert same(run(s, [1, 1, 1, 1, 0, 0]), [2.0, 1.0, 1, 1, 1, 2])
    t = ScalerOracle(init_scale=2**16, scale_factor=2, scale_window=1000, min_scale=2**10)
    traj = run(t, [1] * 8)
    assert same(traj, [32768.0, 16384.0, 8192.0, 4096.0, 2048.0, 1024.0, 1024, 1024])


def test_delayed_shift_hysteresis():
    s = ScalerOracle(init_scale=16, scale_factor=2, scale_window=1000, delayed_shift=2)
    # first overflow spends the credit, later ones shrink (credit is only restored by a growth)
    assert same(run(s, [1, 1, 1, 0, 1]), [16, 8.0, 4.0, 4.0, 2.0])
    assert s.cur_hysteresis == 1
    c = ScalerOracle(init_scale=16, scale_factor=2, scale_window=1000, delayed_shift=2, consecutive_hysteresis=True)
    # a clean step restores the credit
    assert same(run(c, [1, 0, 1, 1, 1]), [16, 16, 16, 8.0, 4.0])
    g = ScalerOracle(init_scale=16, scale_factor=2, scale_window=2, delayed_shift=2)
    # T: credit 2->1; F (iter1: 1-0=1 no); F (iter2: 2%2==0: grow, credit back to 2); T: credit 2->1; T: shrink
    assert same(run(g, [1, 0, 0, 1, 1]), [16, 16, 32, 32, 16.0])


def test_non_power_of_two_factor_and_float_init():
    s = ScalerOracle(init_scale=1000.0, scale_factor=3, scale_window=2)
    assert same(run(s, [0, 0, 1, 1]), [1000.0, 3000.0, 1000.0, 1000.0 / 3])


def test_scale_is_init_times_power_of_factor_property():
    rng = np.random.default_rng(7)
    for trial in range(20):
        w = int(rng.integers(1, 9))
        s = ScalerOracle(init_scale=2**16, scale_factor=2, scale_window=w, min_scale=1)
        flags = rng.random(300) < 0.2
        prev = s.loss_scale
        for it, f in enumerate(flags):
            before_last = s.last_overflow_iter
            s.update_scale(bool(f))
            cur = s.loss_scale
            assert cur >= 1
            assert float(cur) == 2.0 ** round(np.log2(float(cur)))
            if f:
                assert cur == max(prev / 2, 1)
            elif (it - before_last) % w == 0:
                assert cur == prev * 2
            else:
                assert cur == prev
            prev = cur
        assert s.cur_iter == 300


def test_config3_expectation():
    """The overflow / loss-scale configuration: 10 overflows in 200 steps, window 1000 -> ten halvings, no growth."""
    rng = np.random.default_rng(0)
    bad = set(rng.choice(200, size=10, replace=False).tolist())
    s = scaler_from_config({"enabled": True, "loss_scale": 0, "initial_scale_power": 16, "loss_scale_window": 1000, "hysteresis": 2, "min_loss_scale": 1})
    traj = run(s, [i in bad for i in range(200)])
    assert traj[-1] == 2.0**6
    halvings = sum(1 for a, b in zip([2**16] + traj[:-1], traj) if b == a / 2)
    assert halvings == 10 and all(b <= a for a, b in zip([2**16] + traj[:-1], traj))


def test_engine_wiring_quirks():
    # "hysteresis" is the scale FACTOR; delayed_shift stays 1; window defaults to 2000 (runtime/engine.py:90-97)
    s = scaler_from_config({"enabled": True, "loss_scale": 0, "hysteresis": 4})
    assert s.scale_factor == 4 and s.delayed_shift == 1 and s.scale_window == 2000
    assert s.loss_scale == 2**16 and s.min_scale == 1 and s.consecutive_hysteresis is False
    s.update_scale(True)
    assert s.loss_scale == 2**16 / 4
    st = scaler_from_config({"enabled": True, "loss_scale": 128})
    assert isinstance(st, StaticScalerOracle) and st.loss_scale == 128
    st.update_scale(True)
    assert st.loss_scale == 128 and st.has_overflow(np.array([np.inf], np.float16)) is False
    assert scaler_from_config(None) is None
    for bad in ({"enabled": False, "loss_scale": 0}, {"enabled": True}):
        try:
            scaler_from_config(bad)
        except AssertionError:
            pass
        else:
            raise AssertionError("expected an assertion")


@pytest.mark.parametrize("window", [1, 2, 3, 7, 1000])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_matches_torch_amp_scale_update(window, seed):
    """A library routine with the same contract: torch's AMP scale update (the kernel behind
    torch.amp.GradScaler.update, which the reference's own loss-scale test runs beside PatrickStar,
    unitest/test_loss_scale.py:114-120): back off on a step that saw inf/nan, grow after `growth_interval`
    consecutive clean steps.  With delayed_shift = 1 and no min-scale clamp in reach the reference's state machine
    ("grow when (cur_iter - last_overflow_iter) % window == 0") is the same function of the overflow history."""
    import torch

    rng = np.random.default_rng(seed)
    flags = rng.random(2000 if window > 100 else 300) < 1.0 / (window + 1)  # growth and back-off roughly in balance
    s = ScalerOracle(init_scale=2**20, scale_factor=2, scale_window=window, min_scale=2**-200)
    scale = torch.tensor([float(2**20)])
    tracker = torch.zeros(1, dtype=torch.int32)
    compared = 0
    for f in flags:
        s.update_scale(bool(f))
        torch._amp_update_scale_(scale, tracker, torch.tensor([float(f)]), 2.0, 0.5, window)
        if not 2.0**-100 < s.loss_scale < 2.0**100:
            break  # torch keeps the scale in a float32 tensor (and refuses to grow it to inf); stay inside its range
        assert float(s.loss_scale) == scale.item()
        compared += 1
    assert compared >= 100
