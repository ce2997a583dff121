"""GPU data tests of the stand-alone fp32 -> fp16 write-back entry points, ps_cast_fp32_to_fp16 and
ps_restore_fp16_chunks: what FP16ChunkWriteBuffer does with `payload_fp16.copy_(payload_fp32)`
(patrickstar/ops/chunk_io_buff.py:116-126,143-146), bit for bit against the oracle's round-to-nearest-even cast."""
import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from patrickstar_amd import _lib
from _harness import assert_bits_equal

pytestmark = pytest.mark.gpu


def _awkward_values(n, rng):
    """fp32 values that exercise every rounding case of the cast: ordinary values over many binades, every kind of
    special value, ties, the fp16 overflow threshold, fp16 subnormals and values that round to zero."""
    x = (rng.normal(0, 1, n) * 10.0 ** rng.integers(-9, 6, n)).astype(np.float32)
    special = np.array(
        [np.inf, -np.inf, np.nan, 0.0, -0.0, 65504.0, 65519.996, 65520.0, 65520.004, -65520.0, 7e4, -1e38, 3.4e38,
         2.0**-24, 2.0**-25, 2.0**-25 * 1.0000001, 2.0**-26, 2.0**-14, 2.0**-14 * 0.9999, 6.1e-5, 5.96e-8, 1e-45,
         1.0 + 2.0**-11, 1.0 + 2.0**-11 + 2.0**-23, 1.0 + 3 * 2.0**-11, 2049.0, 2051.0, -2049.0],
        dtype=np.float32,
    )
    reps = max(1, n // (8 * special.size))
    where = rng.choice(n, size=min(n, reps * special.size), replace=False)
    x[where] = np.tile(special, reps)[: where.size]
    # ties between neighbouring fp16 values (exactly representable in fp32)
    h = rng.integers(0, 0x7BFF, size=n // 16).astype(np.uint16).view(np.float16).astype(np.float64)
    nxt = np.nextafter(h.astype(np.float16), np.float16(np.inf)).astype(np.float64)
    ties = ((h + nxt) / 2).astype(np.float32)
    x[rng.choice(n, size=ties.size, replace=False)] = ties
    return x


@pytest.mark.parametrize("n", [1, 7, 255, 256, 257, 4099, 256 * 4096 + 123, 5_000_001])
@pytest.mark.parametrize("src_off,dst_off", [(0, 0), (1, 0), (0, 1), (3, 5), (4, 8)])
def test_cast_matches_the_oracle_on_ragged_lengths_and_unaligned_bases(n, src_off, dst_off):
    lib = _lib.load()
    rng = np.random.default_rng(n + 17 * src_off + dst_off)
    x = _awkward_values(n, rng)
    src = torch.zeros(n + 16, dtype=torch.float, device="cuda")
    src[src_off:src_off + n].copy_(torch.from_numpy(x))
    dst = torch.full((n + 32,), 7.0, dtype=torch.half, device="cuda")
    _lib.check(
        lib.ps_cast_fp32_to_fp16(src[src_off:].data_ptr(), dst[dst_off:].data_ptr(), n, _lib.current_stream_handle()),
        "ps_cast_fp32_to_fp16",
    )
    torch.cuda.synchronize()
    got = dst.cpu().numpy()
    want = oracle.cast_fp32_to_fp16(x)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got[dst_off:dst_off + n]), nan)
    assert_bits_equal(got[dst_off:dst_off + n][~nan], want[~nan], f"cast n={n} offsets {src_off},{dst_off}")
    # nothing outside the destination span was written
    assert (got[:dst_off] == 7.0).all() and (got[dst_off + n:] == 7.0).all()
    # torch's own cast-copy (what the reference runs) agrees as well
    assert torch.equal(dst[dst_off:dst_off + n].isnan(), src[src_off:src_off + n].half().isnan())
    both = ~dst[dst_off:dst_off + n].isnan()
    assert torch.equal(dst[dst_off:dst_off + n][both].view(torch.int16), src[src_off:src_off + n].half()[both].view(torch.int16))


def _state_with_flag(flag):
    s = ps.DynamicLossScaler(init_scale=2**8)
    s.materialize("cuda:0")
    off = _lib.ps_step_state.overflow.offset
    s._state[off:off + 4].view(torch.int32).fill_(flag)
    return s


@pytest.mark.parametrize("n_chunks,n", [(1, 256 * 3 + 5), (3, 256 * 40), (70, 777), (130, 256)])
@pytest.mark.parametrize("mode", ["unconditional", "flag set", "flag clear"])
def test_restore_chunks_with_and_without_the_device_flag(n_chunks, n, mode):
    """ps_restore_fp16_chunks: d_state NULL restores always; with a state it restores only when the sticky overflow
    flag is set (FP16Adam.has_overflow_and_reset_param, fp16_cpu_adam.py:298-309).  More than 64 chunks take several
    launches.  fp32 / m / v payloads are never written."""
    lib = _lib.load()
    rng = np.random.default_rng(n_chunks * 1000 + n)
    stride32 = -(-n // 4) * 4 + 4
    stride16 = -(-n // 8) * 8 + 8
    p32 = torch.zeros(n_chunks * stride32, dtype=torch.float, device="cuda")
    h16 = torch.zeros(n_chunks * stride16, dtype=torch.half, device="cuda")
    host = []
    rows = []
    for c in range(n_chunks):
        x = _awkward_values(n, rng)
        host.append(x)
        p32[c * stride32:c * stride32 + n].copy_(torch.from_numpy(x))
        rows.append([p32[c * stride32:].data_ptr(), p32.data_ptr(), p32.data_ptr(), h16[c * stride16:].data_ptr()])
    garbage = torch.from_numpy(rng.integers(0, 0x7BFF, h16.numel()).astype(np.int16)).cuda()
    h16.view(torch.int16).copy_(garbage)
    before32 = p32.clone()
    state = None if mode == "unconditional" else _state_with_flag(1 if mode == "flag set" else 0)
    _lib.check(
        lib.ps_restore_fp16_chunks(_lib.chunk_array(rows), n_chunks, n, state.state_ptr if state else None,
                                   _lib.current_stream_handle()),
        "ps_restore_fp16_chunks",
    )
    torch.cuda.synchronize()
    assert torch.equal(p32.view(torch.int32), before32.view(torch.int32))
    got = h16.cpu().numpy()
    old = garbage.cpu().numpy().view(np.float16)
    for c in range(n_chunks):
        span = slice(c * stride16, c * stride16 + n)
        if mode == "flag clear":
            assert_bits_equal(got[span], old[span], f"chunk {c} must be untouched")
        else:
            want = oracle.cast_fp32_to_fp16(host[c])
            nan = np.isnan(want)
            assert np.array_equal(np.isnan(got[span]), nan)
            assert_bits_equal(got[span][~nan], want[~nan], f"chunk {c} restored")
        # the gap behind every chunk is never written
        gap = slice(c * stride16 + n, (c + 1) * stride16)
        assert_bits_equal(got[gap], old[gap], f"gap behind chunk {c}")
    if state is not None:
        assert state.overflow_flag == (mode == "flag set")  # the restore does not consume the flag


@pytest.mark.parametrize("host_positions,host_keeps_fp16", [((), True), ((1, 3), True), ((0, 2), False)])
def test_has_overflow_and_reset_param_restores_every_chunk(host_positions, host_keeps_fp16):
    """FP16Adam.has_overflow_and_reset_param (fp16_cpu_adam.py:287-310) as a call of its own: a set flag rewrites the
    fp16 payload of EVERY position from its fp32 master (RNE, padding included), clears the flag and reports True; a
    clear flag changes nothing.  Positions in pinned host memory are rewritten in place by the same kernel."""
    import oracle
    import patrickstar_amd as ps
    from _harness import HybridHarness, assert_bits_equal

    h = HybridHarness(4, 2048 + 77, list(host_positions), ps.DynamicLossScaler(init_scale=2**8), seed=3,
                      host_keeps_fp16=host_keeps_fp16, lr=1e-3)
    h.fill_state()
    h.fill_grads(1e-3, 2.0**8)
    before = [h.download(i) for i in range(4)]
    assert h.opt.has_overflow_and_reset_param() is False
    torch.cuda.synchronize()
    for i in range(4):
        assert_bits_equal(h.download(i)[3], before[i][3], f"clear flag: position {i} fp16 untouched")
    h.payloads(2)[3][17] = float("nan")
    h.opt.check_overflow_chunks()
    assert h.opt.has_overflow is True
    assert h.opt.has_overflow_and_reset_param() is True
    torch.cuda.synchronize()
    assert h.opt.has_overflow is False
    for i in range(4):
        p, m, v, f16 = h.download(i)
        assert_bits_equal(f16, oracle.cast_fp32_to_fp16(before[i][0]), f"position {i} fp16 = RNE(fp32 master)")
        for got, want, name in ((p, before[i][0], "fp32"), (m, before[i][1], "exp_avg"), (v, before[i][2], "exp_avg_sq")):
            assert_bits_equal(got, want, f"position {i} {name} untouched")
    assert h.opt.has_overflow_and_reset_param() is False
    # a static scaler never reports overflow (loss_scaler.py:63-65)
    s = HybridHarness(2, 512, [], ps.LossScaler(8), seed=4, lr=1e-3)
    assert s.opt.has_overflow_and_reset_param() is False
