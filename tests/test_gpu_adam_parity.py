"""GPU parity of the fused chunk-list Adam step against the CPU oracle, through the C ABI.

Bar: fp32 param / exp_avg / exp_avg_sq and the fp16 param copy BIT-EXACT against the
oracle (the stated tolerance of 1e-6 relative / 1 fp16 ulp is met with zero slack),
because the kernel performs the same IEEE binary32 operations in the same order.
"""
import math

import numpy as np
import pytest
import torch

import oracle
import patrickstar_amd as ps
from patrickstar_amd import _lib
from _harness import N_FULL, ChunkHarness, assert_bits_equal

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(a).cuda()


# ---------------------------------------------------------------- native operator

def torch_adam_update(step, lr, beta1, beta2, eps, weight_decay, bias_correction, param, grad, exp_avg, exp_avg_sq,
                      loss_scale, use_adamw):
    """The comparison formula of the reference's operator test (unitest/test_ds_cpu_adam.py:37-71), on torch tensors."""
    if loss_scale > 0:
        grad.div_(loss_scale)
    bias_correction1 = 1 - beta1**step
    bias_correction2 = 1 - beta2**step
    if weight_decay != 0:
        if use_adamw:
            param.mul_(1 - lr * weight_decay)
        else:
            grad = grad.add(param, alpha=weight_decay)
    exp_avg.mul_(beta1).add_(grad, alpha=1 - beta1)
    exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    denom = (exp_avg_sq.sqrt() / math.sqrt(bias_correction2)).add_(eps)
    param.addcdiv_(exp_avg, denom, value=-(lr / bias_correction1))


@pytest.mark.parametrize("use_adamw", [False, True])
@pytest.mark.parametrize("shape", [(1023,), (1024, 32)])
@pytest.mark.parametrize("grad_dtype", [torch.float, torch.half])
@pytest.mark.parametrize("loss_scale", [-1, 2**5])
def test_adam_update_reference_test_grid(use_adamw, shape, grad_dtype, loss_scale):
    """The reference's own operator test (unitest/test_ds_cpu_adam.py:77-192), with the operator module under its
    reference names (create_adam / adam_update / destroy_adam on flat tensors): step 1, lr .01, betas (.9,.999),
    eps 1e-8, wd .001, uniform [0,1) inputs.  Its bar is 1e-4 absolute against the torch formula; ours is additionally
    bit-exactness against the CPU restatement of the operator, and the gradients must come back untouched."""
    cpu_adam_op = ps.adam_op
    step, lr, eps, beta1, beta2, weight_decay = 1, 0.01, 1e-8, 0.9, 0.999, 0.001
    torch.manual_seed(abs(hash((use_adamw, shape, str(grad_dtype), loss_scale))) % 2**31)
    opt_id = 900
    p_data = torch.rand(shape)
    p_grad = torch.rand(shape, dtype=grad_dtype)
    if loss_scale > 0:
        p_grad.mul_(loss_scale)
    exp_avg = torch.rand(shape)
    exp_avg_sq = torch.rand(shape)
    p_data_copy, exp_avg_copy, exp_avg_sq_copy = p_data.clone(), exp_avg.clone(), exp_avg_sq.clone()
    p_grad_copy = p_grad.clone().float()
    host = [t.clone().view(-1).numpy() for t in (p_data, p_grad, exp_avg, exp_avg_sq)]

    d_data, d_grad, d_avg, d_sq = (t.cuda() for t in (p_data, p_grad, exp_avg, exp_avg_sq))
    cpu_adam_op.create_adam(opt_id, lr, beta1, beta2, eps, weight_decay, use_adamw, False)
    cpu_adam_op.adam_update(opt_id, step, lr, beta1, beta2, eps, weight_decay, True, d_data.view(-1), d_grad.view(-1),
                            d_avg.view(-1), d_sq.view(-1), loss_scale)
    torch.cuda.synchronize()
    cpu_adam_op.destroy_adam(opt_id)

    # the reference's check: within 1e-4 of the torch formula
    torch_adam_update(step, lr, beta1, beta2, eps, weight_decay, True, p_data_copy, p_grad_copy, exp_avg_copy,
                      exp_avg_sq_copy, loss_scale, use_adamw)
    assert torch.max(torch.abs(p_data_copy - d_data.cpu())) < 1e-4
    assert torch.max(torch.abs(exp_avg_copy - d_avg.cpu())) < 1e-4
    assert torch.max(torch.abs(exp_avg_sq_copy - d_sq.cpu())) < 1e-4

    # ours: the gradients are read only, and every bit equals the CPU restatement of the operator
    assert_bits_equal(d_grad.cpu().view(-1).numpy(), host[1], "grads must not be written")
    po, g, mo, vo = host
    oracle.AdamOracle(lr, beta1, beta2, eps, weight_decay, use_adamw).update(
        step, lr, beta1, beta2, eps, weight_decay, True, po, g, mo, vo, float(loss_scale))
    assert_bits_equal(d_data.cpu().view(-1).numpy(), po, "param")
    assert_bits_equal(d_avg.cpu().view(-1).numpy(), mo, "exp_avg")
    assert_bits_equal(d_sq.cpu().view(-1).numpy(), vo, "exp_avg_sq")


def test_operator_module_argument_checks():
    op = ps.adam_op
    op.create_adam(901, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, False)
    x = torch.zeros(8, device="cuda")
    with pytest.raises(RuntimeError, match="GPU tensor"):
        op.adam_update(901, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, torch.zeros(8), x, x, x, -1)
    with pytest.raises(RuntimeError, match="flat and contiguous"):
        op.adam_update(901, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, x.view(2, 4), x, x, x, -1)
    with pytest.raises(TypeError, match="float32"):
        op.adam_update(901, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, x.half(), x, x, x, -1)
    with pytest.raises(RuntimeError, match="differ in length"):
        op.adam_update(901, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, x, x[:4], x, x, -1)
    op.destroy_adam(901)
    with pytest.raises(RuntimeError, match="never created"):
        op.adam_update(901, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, x, x, x, x, -1)


def test_ds_cpu_adam_update_method_hands_the_scalers_scale_to_the_operator():
    """FP16Adam.ds_cpu_adam_update (fp16_cpu_adam.py:205-243): one operator call on 2-D tensors, flattened, with the
    loss scaler's scale or -1; two calls with the same step number take the two branches of IncrementStep."""
    rng = np.random.default_rng(17)
    for scaler, scale in ((None, -1.0), (ps.LossScaler(32), 32.0)):
        client = ps.PatrickStarClient(0, 64)
        opt = ps.FP16Adam(client, client.append_flat_chunks(1), loss_scaler=scaler, lr=1e-2, weight_decay=0.001, use_adamw=True)
        native = oracle.AdamOracle(1e-2, 0.9, 0.999, 1e-8, 0.001, True)
        for call, shape in enumerate([(1024, 32), (1023,), (7, 9)]):
            host = [rng.normal(0, 0.02, shape).astype(np.float32), (rng.normal(0, 1e-3, shape) * abs(scale)).astype(np.float16),
                    rng.normal(0, 1e-4, shape).astype(np.float32), np.abs(rng.normal(0, 1e-6, shape)).astype(np.float32)]
            dev = [_dev(x.copy()) for x in host]
            step = 1 if call < 2 else 2  # same step twice (running product, then pow), then the next step (running product)
            opt.ds_cpu_adam_update(dev[0], dev[1], dev[2], dev[3], step, 1e-2, 0.9, 0.999, 1e-8, 0.001, True)
            torch.cuda.synchronize()
            p, g, m, v = (x.reshape(-1).copy() for x in host)
            native.update(step, 1e-2, 0.9, 0.999, 1e-8, 0.001, True, p, g, m, v, scale)
            assert_bits_equal(dev[0].cpu().numpy().reshape(-1), p, f"call {call} param")
            assert_bits_equal(dev[2].cpu().numpy().reshape(-1), m, f"call {call} exp_avg")
            assert_bits_equal(dev[3].cpu().numpy().reshape(-1), v, f"call {call} exp_avg_sq")
            assert_bits_equal(dev[1].cpu().numpy().reshape(-1), g, f"call {call} gradient untouched")
    with pytest.raises(AssertionError, match="GPU"):
        opt.ds_cpu_adam_update(torch.zeros(4), dev[1], dev[2], dev[3], 3, 1e-2, 0.9, 0.999, 1e-8, 0.0, True)


def test_adam_update_unaligned_views_fp16_out_and_errors():
    lib = _lib.load()
    rng = np.random.default_rng(5)
    n, off = 5003, 3  # views that start 3 elements into their buffers: 12-byte / 6-byte misalignment
    p, m, v = (rng.normal(0, 0.02, n + off).astype(np.float32) for _ in range(3))
    v = np.abs(v) * 1e-4
    g = (rng.normal(0, 1e-3, n + off) * 1000).astype(np.float16)
    dp, dm, dv, dg = _dev(p.copy()), _dev(m.copy()), _dev(v.copy()), _dev(g.copy())
    out16 = torch.zeros(n + off, dtype=torch.half, device="cuda")
    oid = 901
    lib.ps_adam_create(oid, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0, 0)
    s = _lib.current_stream_handle()
    rc = lib.ps_adam_update(oid, 7, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, dp[off:].data_ptr(), dg[off:].data_ptr(), 1,
                            dm[off:].data_ptr(), dv[off:].data_ptr(), n, 1000.0, out16[off:].data_ptr(), s)
    assert rc == 0
    torch.cuda.synchronize()
    po, mo, vo = p[off:].copy(), m[off:].copy(), v[off:].copy()
    oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.0, False).update(7, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, po, g[off:].copy(), mo, vo, 1000.0)
    assert_bits_equal(dp.cpu().numpy()[off:], po, "param")
    assert_bits_equal(dm.cpu().numpy()[off:], mo, "exp_avg")
    assert_bits_equal(dv.cpu().numpy()[off:], vo, "exp_avg_sq")
    assert_bits_equal(out16.cpu().numpy()[off:], oracle.cast_fp32_to_fp16(po), "fp16 out")
    assert_bits_equal(dp.cpu().numpy()[:off], p[:off], "elements before the view")
    # numel == 0 still advances the host state and succeeds
    assert lib.ps_adam_update(oid, 8, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, None, 1, None, None, 0, -1.0, None, s) == 0
    # unknown id: an error code, not a crash
    assert lib.ps_adam_update(4242, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, dp.data_ptr(), dg.data_ptr(), 1, dm.data_ptr(),
                              dv.data_ptr(), n, -1.0, None, s) == _lib.PS_ERR_UNKNOWN_ID
    assert b"4242" in lib.ps_last_error()
    assert lib.ps_adam_update(oid, 9, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, dg.data_ptr(), 1, dm.data_ptr(), dv.data_ptr(),
                              n, -1.0, None, s) == _lib.PS_ERR_BAD_ARG
    lib.ps_adam_destroy(oid)
    assert lib.ps_adam_destroy(oid) == 0  # unknown ids are ignored


# ---------------------------------------------------------------- chunk-list step, small shapes

@pytest.mark.parametrize("use_adamw,wd", [(False, 0.0), (False, 0.01), (True, 0.01)])
@pytest.mark.parametrize("scale", [None, 8, 2**16, 1000.0])
@pytest.mark.parametrize("chunk_size", [2048 * 3, 2048 * 2 + 77, 100])
def test_chunk_step_small_bit_exact(use_adamw, wd, scale, chunk_size):
    """Whole and ragged tiles, every weight-decay form, no / power-of-two / non-power-of-two static scale,
    three consecutive steps (running-product branch of the step scalars)."""
    scaler = None if scale is None else ps.LossScaler(scale)
    h = ChunkHarness(3, chunk_size, scaler, seed=chunk_size, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd, use_adamw=use_adamw)
    h.fill_state()
    oc = h.oracle_chunks()
    oscaler = None if scale is None else oracle.StaticScalerOracle(scale)
    oopt = oracle.OptimizerStepOracle(oc, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd, use_adamw=use_adamw)
    for step in range(3):
        h.fill_grads(1e-3, scale or 1.0)
        for c, i in zip(oc, range(3)):
            c["p16"][...] = h.download(i)[3]
        h.opt.step()
        assert oopt.step() is False
        h.compare(oc, what=f"step {step + 1}")
    assert h.opt.state[h.params[0]]["step"] == 3


def test_chunk_step_cold_start_and_subnormals():
    """t=100 on a fresh optimizer takes the pow() branch; subnormal m/v/g and huge/small magnitudes keep their bits."""
    n = 2048 * 4
    h = ChunkHarness(2, n, ps.LossScaler(2**12), seed=11, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    h.fill_state()
    p, m, v, g = h.payloads(0)
    m[:64] = 1e-41  # subnormal
    v[:64] = 3e-42
    v[64:128] = 0.0
    m[64:128] = 0.0
    p[128:192] = 1e30
    p[192:256] = 1e-30
    h.fill_grads(1e-3, 2**12)
    g[:32] = 6e-8  # fp16 subnormal gradients
    g[64:96] = 0.0
    g[256:260] = 65504.0
    for prm in h.params:
        dict.__setitem__(h.opt.state[prm], "step", 99)
    oc = h.oracle_chunks()
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(2**12), lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    oopt.step_count = 99
    h.opt.step()
    oopt.step()
    h.compare(oc, what="cold t=100")


def test_empty_and_zero_sized_chunk_lists():
    lib = _lib.load()
    s = _lib.current_stream_handle()
    lib.ps_adam_create(902, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0)
    assert lib.ps_adam_step_chunks(902, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, 0, 1024, None, None, -1.0, s) == 0
    buf = torch.zeros(64, dtype=torch.float, device="cuda")
    one = _lib.chunk_array([[buf.data_ptr()] * 4])
    assert lib.ps_adam_step_chunks(902, 2, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, one, 1, 0, None, None, -1.0, s) == 0
    assert lib.ps_adam_step_chunks(902, 3, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, 2, 16, None, None, -1.0, s) == _lib.PS_ERR_BAD_ARG
    assert lib.ps_adam_step_chunks(902, 3, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, one, -1, 16, None, None, -1.0, s) == _lib.PS_ERR_BAD_ARG
    null_payload = _lib.chunk_array([[buf.data_ptr(), 0, buf.data_ptr(), buf.data_ptr()]])
    assert lib.ps_adam_step_chunks(902, 3, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, null_payload, 1, 16, None, None, -1.0, s) == _lib.PS_ERR_BAD_ARG
    assert b"NULL payload" in lib.ps_last_error()
    assert lib.ps_cast_fp32_to_fp16(None, None, 0, s) == 0
    lib.ps_adam_destroy(902)
    torch.cuda.synchronize()
    assert not buf.any()


def test_more_chunks_than_one_launch_carries():
    """Descriptors travel 64 per launch: a 150-chunk list takes three launches and every chunk is updated."""
    n = 2048 + 5
    h = ChunkHarness(150, n, ps.LossScaler(16), seed=6, lr=1e-3, weight_decay=0.01, use_adamw=True)
    h.fill_state()
    h.fill_grads(1e-3, 16)
    idx = [0, 63, 64, 127, 128, 149]
    oc = h.oracle_chunks(idx)
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(16), lr=1e-3, weight_decay=0.01, use_adamw=True)
    before = [h.payloads(i)[1].abs().sum().item() for i in range(150)]
    h.opt.step()
    oopt.step()
    h.compare(oc, idx, what="150 chunks")
    after = [h.payloads(i)[1].abs().sum().item() for i in range(150)]
    assert all(a != b for a, b in zip(after, before))


def test_nonfinite_gradients_with_static_scale_propagate_like_the_oracle():
    """A static scaler never checks overflow (loss_scaler.py:60-61): inf/nan flow into the state.
    NaN payload bits are implementation-defined, so NaN positions are compared as positions."""
    n = 2048
    h = ChunkHarness(1, n, ps.LossScaler(8), seed=2, lr=1e-3)
    h.fill_state()
    h.fill_grads(1e-3, 8)
    g = h.payloads(0)[3]
    g[5], g[9], g[100] = float("inf"), float("-inf"), float("nan")
    oc = h.oracle_chunks()
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(8), lr=1e-3)
    h.opt.step()
    oopt.step()
    p, m, v, hh = h.download(0)
    for got, want in ((p, oc[0]["p32"]), (m, oc[0]["m"]), (v, oc[0]["v"]), (hh.astype(np.float32), oc[0]["p16"].astype(np.float32))):
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok], want[ok])
    assert np.isnan(p[[5, 9, 100]]).all() and h.opt.has_overflow is False


# ---------------------------------------------------------------- the benchmark's named configurations

def test_config1_one_full_chunk_ten_steps():
    """Configuration "one chunk on the reference CPU path": one 64 Mi-element chunk, p~N(0,.02), m=v=0, g16=(N(0,1e-3)*8).half(), static scale 8,
    Adam lr 1e-3 betas (.9,.999) eps 1e-6 wd 0, steps 1..10.  Bit-exact against the oracle after every step."""
    h = ChunkHarness(1, N_FULL, ps.LossScaler(8), seed=0, lr=1e-3, betas=(0.9, 0.999), eps=1e-6, weight_decay=0)
    h.fill_state(m_std=0, v_std=0)
    oc = h.oracle_chunks()
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(8), lr=1e-3, betas=(0.9, 0.999), eps=1e-6, weight_decay=0.0)
    for step in range(1, 11):
        h.fill_grads(1e-3, 8)
        oc[0]["p16"][...] = h.download(0)[3]
        h.opt.step()
        oopt.step()
        h.compare(oc, what=f"config 1 step {step}")
    # step-1 closed form spot check is in the oracle's own tests; here: the update moved every parameter with a
    # non-zero gradient history
    assert h.opt.state[h.params[0]]["step"] == 10


def test_config2_padded_two_chunks_cold_t100():
    """Configuration "GPT-2-small-sized": 124,439,808 parameters in 2 chunks of 64 Mi, zero tail; m~N(0,1e-4), v=|N(0,1e-6)|,
    g16=(N(0,1e-3)*2^16).half(), AdamW wd .01 lr 1e-4, t=100 cold."""
    real = 124_439_808
    h = ChunkHarness(2, N_FULL, ps.LossScaler(2**16), used_numel_last=real - N_FULL, seed=1,
                     lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    h.fill_state()
    h.fill_grads(1e-3, 2**16)
    for prm in h.params:
        dict.__setitem__(h.opt.state[prm], "step", 99)
    oc = h.oracle_chunks()
    assert np.isfinite(oc[1]["p16"].astype(np.float32)).all()
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(2**16), lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    oopt.step_count = 99
    h.opt.step()
    oopt.step()
    h.compare(oc, what="config 2")
    used = real - N_FULL
    for t in h.download(1):
        assert not t[used:].any(), "the zero-padded tail must stay exactly zero"


@pytest.mark.parametrize("arithmetic", ["operator", "torch"])
def test_config4_first_and_last_chunk_of_24(arithmetic):
    """Configuration "GPT-2-1.5B-sized" (the timed one): 24 chunks resident in HBM, AdamW lr 1e-4 eps 1e-8 wd .01, static scale 2^12,
    t=100.  The oracle checks the first and the last chunk; a checksum guards the ones in between against being skipped.
    Under the torch arithmetic one chunk in the middle is also compared with the reference's torch calls run by torch."""
    h = ChunkHarness(24, N_FULL, ps.LossScaler(2**12), seed=4, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True,
                     arithmetic=arithmetic)
    h.fill_state()
    h.fill_grads(1e-3, 2**12)
    for prm in h.params:
        dict.__setitem__(h.opt.state[prm], "step", 99)
    idx = [0, 23]
    oc = h.oracle_chunks(idx)
    before = [h.payloads(i)[0].view(torch.int32).sum(dtype=torch.int64).item() for i in range(24)]
    oopt = oracle.OptimizerStepOracle(oc, oracle.StaticScalerOracle(2**12), lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True,
                                      arithmetic=arithmetic)
    oopt.step_count = 99
    if arithmetic == "torch":
        from test_oracle_torch_formula import reference_call_sequence

        tp, tm, tv, tg = (t.clone() for t in h.payloads(11))
        reference_call_sequence(tp, tg, tm, tv, 100, 1e-4, 0.9, 0.999, 1e-8, 0.01, True, 2**12)
        del tg
    h.opt.step()
    oopt.step()
    h.compare(oc, idx, what="config 4")
    if arithmetic == "torch":
        for got, want in zip(h.payloads(11)[:3], (tp, tm, tv)):
            assert torch.equal(got.view(torch.int32), want.view(torch.int32))
        del tp, tm, tv
    after = [h.payloads(i)[0].view(torch.int32).sum(dtype=torch.int64).item() for i in range(24)]
    assert all(a != b for a, b in zip(after, before)), "every chunk must have been updated"
    # fp16 copy == RNE(fp32) everywhere (size-independent property, checked on the device)
    for i in range(24):
        p, _, _, hh = h.payloads(i)
        assert torch.equal(p.half(), hh)


# ---------------------------------------------------------------- element-wise gradient clamp

@pytest.mark.parametrize("clipping,scale", [(1.0, 8), (0.3, 1000.0), (0.1, None), (5.0, 2**16), (1.0001, 8), (1e-3, 2**12)])
def test_fused_gradient_clamp_matches_oracle_and_torch_clamp(clipping, scale):
    """FP16Adam's "gradient clipping" is an element-wise clamp of the fp16 gradients to +-min(65504, clipping*scale)
    (fp16_cpu_adam.py:364-379).  The fused form must equal (a) the oracle's restatement and (b) the library call the
    reference itself makes: Tensor.clamp_ on the fp16 gradient tensor followed by an unclamped step."""
    n = 2048 * 2 + 31
    kw = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True)
    mk = lambda: None if scale is None else ps.LossScaler(scale)
    a = ChunkHarness(2, n, mk(), seed=77, gradient_clipping=clipping, **kw)
    b = ChunkHarness(2, n, mk(), seed=77, **kw)  # same seed -> same state and gradients
    for h in (a, b):
        h.fill_state()
    oc = a.oracle_chunks()
    oopt = oracle.OptimizerStepOracle(oc, None if scale is None else oracle.StaticScalerOracle(scale), gradient_clipping=clipping, **kw)
    bound = min(65504.0, clipping * (scale if scale is not None else 1))
    for step in range(2):
        for h in (a, b):
            h.fill_grads(bound / (scale or 1.0), scale or 1.0)  # scaled gradients ~ N(0, bound): about a third is clamped
            g = h.payloads(1)[3]
            g[3], g[4], g[5] = float("inf"), float("-inf"), float("nan")  # static scale: nothing is skipped
        for i, c in enumerate(oc):
            c["p16"][...] = a.download(i)[3]
        clipped_fraction = float((a.payloads(0)[3].float().abs() > bound).float().mean())
        assert 0.0 < clipped_fraction < 1.0, "the case must actually clamp something, and not everything"
        for i in range(2):
            b.payloads(i)[3].clamp_(-bound, bound)  # what the reference calls
        a.opt.step()
        b.opt.step()
        oopt.step()
        for i in range(2):
            for x, y, key in zip(a.download(i), b.download(i), ("p32", "m", "v", "p16")):
                nan = np.isnan(x.astype(np.float32))
                assert np.array_equal(nan, np.isnan(y.astype(np.float32))) and np.array_equal(nan, np.isnan(oc[i][key].astype(np.float32)))
                assert_bits_equal(x[~nan], y[~nan], f"step {step} chunk {i} {key}: fused clamp vs Tensor.clamp_")
                assert_bits_equal(x[~nan], oc[i][key][~nan], f"step {step} chunk {i} {key}: fused clamp vs oracle")
        # +-inf were clamped to the bound (finite), the NaN stayed a NaN
        assert np.isfinite(a.download(1)[0][[3, 4]]).all() and np.isnan(a.download(1)[0][5])


@pytest.mark.parametrize("phase", [0, 1, 2, 3])
@pytest.mark.parametrize("grad_dtype", [np.float16, np.float32])
def test_adam_update_vector_path_all_phases(phase, grad_dtype):
    """Large tensors take the operator's vector path: views starting 0..3 elements into their buffers (the phase a
    tensor has inside its chunks), fp16 and fp32 gradients, fp16 output aliasing the fp16 gradients or absent."""
    lib = _lib.load()
    rng = np.random.default_rng(100 + phase)
    n = 256 * 40 + 131  # 40 whole tiles + a remainder, beyond the 4096-element threshold
    tot = n + phase
    p = rng.normal(0, 0.02, tot).astype(np.float32)
    m = rng.normal(0, 1e-4, tot).astype(np.float32)
    v = np.abs(rng.normal(0, 1e-6, tot)).astype(np.float32)
    g = (rng.normal(0, 1e-3, tot) * 64).astype(grad_dtype)
    dp, dm, dv, dg = _dev(p.copy()), _dev(m.copy()), _dev(v.copy()), _dev(g.copy())
    half = grad_dtype == np.float16
    out = dg if half else None  # fp16 parameters overwrite the fp16 gradients, as in the chunk layout
    oid = 903
    lib.ps_adam_create(oid, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, 0)
    rc = lib.ps_adam_update(oid, 5, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, dp[phase:].data_ptr(), dg[phase:].data_ptr(), int(half),
                            dm[phase:].data_ptr(), dv[phase:].data_ptr(), n, 64.0, out[phase:].data_ptr() if out is not None else None,
                            _lib.current_stream_handle())
    assert rc == 0
    torch.cuda.synchronize()
    lib.ps_adam_destroy(oid)
    po, mo, vo = p[phase:].copy(), m[phase:].copy(), v[phase:].copy()
    oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.01, True).update(5, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, po, g[phase:].copy(), mo, vo, 64.0)
    assert_bits_equal(dp.cpu().numpy()[phase:], po, "param")
    assert_bits_equal(dm.cpu().numpy()[phase:], mo, "exp_avg")
    assert_bits_equal(dv.cpu().numpy()[phase:], vo, "exp_avg_sq")
    if half:
        assert_bits_equal(dg.cpu().numpy()[phase:], oracle.cast_fp32_to_fp16(po), "fp16 params over the gradients")
    else:
        assert_bits_equal(dg.cpu().numpy(), g, "fp32 gradients untouched")
    for t, ref in ((dp, p), (dm, m), (dv, v)):
        assert_bits_equal(t.cpu().numpy()[:phase], ref[:phase], "elements before the view")


def test_adam_update_with_parameter_and_gradient_at_different_phases_goes_elementwise():
    lib = _lib.load()
    rng = np.random.default_rng(9)
    n = 9000
    p = rng.normal(0, 0.02, n + 3).astype(np.float32)
    m = rng.normal(0, 1e-4, n + 3).astype(np.float32)
    v = np.abs(rng.normal(0, 1e-6, n + 3)).astype(np.float32)
    g = (rng.normal(0, 1e-3, n + 3)).astype(np.float16)
    dp, dm, dv, dg = _dev(p.copy()), _dev(m.copy()), _dev(v.copy()), _dev(g.copy())
    oid = 904
    lib.ps_adam_create(oid, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0, 0)
    rc = lib.ps_adam_update(oid, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, dp[1:].data_ptr(), dg[3:].data_ptr(), 1, dm[2:].data_ptr(),
                            dv.data_ptr(), n, -1.0, None, _lib.current_stream_handle())
    assert rc == 0
    torch.cuda.synchronize()
    lib.ps_adam_destroy(oid)
    po, mo, vo = p[1:1 + n].copy(), m[2:2 + n].copy(), v[:n].copy()
    oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.0, False).update(1, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, po, g[3:3 + n].copy(), mo, vo, -1.0)
    assert_bits_equal(dp.cpu().numpy()[1:1 + n], po, "param")
    assert_bits_equal(dm.cpu().numpy()[2:2 + n], mo, "exp_avg")
    assert_bits_equal(dv.cpu().numpy()[:n], vo, "exp_avg_sq")


@pytest.mark.parametrize("grads_half", [True, False])
@pytest.mark.parametrize("po,mo,vo", [(0, 1, 2), (3, 0, 1), (2, 2, 5), (1, 6, 3)])
def test_adam_update_with_state_at_other_phases_than_the_parameter(po, mo, vo, grads_half):
    """The reference packs momentum / variance tensors in another order than the parameters, so the views handed to one
    operator call may start at different element phases: parameter and gradient share one (they share a layout), the
    two state tensors have their own.  Long enough for the vector path; everything around the views stays untouched."""
    lib = _lib.load()
    rng = np.random.default_rng(90 + po + 4 * mo + 16 * vo)
    n, pad = 256 * 40 + 77, 8
    p = rng.normal(0, 0.02, n + 2 * pad).astype(np.float32)
    m = rng.normal(0, 1e-4, n + 2 * pad).astype(np.float32)
    v = np.abs(rng.normal(0, 1e-6, n + 2 * pad)).astype(np.float32)
    g = (rng.normal(0, 1e-3, n + 2 * pad) * 64).astype(np.float16 if grads_half else np.float32)
    out = np.zeros(n + 2 * pad, np.float16)
    dp, dm, dv, dg, dout = (_dev(x.copy()) for x in (p, m, v, g, out))
    oid = 906
    lib.ps_adam_create(oid, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, 0)
    rc = lib.ps_adam_update(oid, 3, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, dp[po:].data_ptr(), dg[po:].data_ptr(), int(grads_half),
                            dm[mo:].data_ptr(), dv[vo:].data_ptr(), n, 64.0, dout[po:].data_ptr(), _lib.current_stream_handle())
    assert rc == 0, lib.ps_last_error()
    torch.cuda.synchronize()
    lib.ps_adam_destroy(oid)
    pw, mw, vw = p[po:po + n].copy(), m[mo:mo + n].copy(), v[vo:vo + n].copy()
    oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.01, True).update(3, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, pw, g[po:po + n].copy(), mw, vw, 64.0)
    for got, src, off, want, name in ((dp, p, po, pw, "param"), (dm, m, mo, mw, "exp_avg"), (dv, v, vo, vw, "exp_avg_sq"),
                                      (dout, out, po, oracle.cast_fp32_to_fp16(pw), "fp16 out")):
        got = got.cpu().numpy()
        assert_bits_equal(got[off:off + n], want, name)
        assert_bits_equal(got[:off], src[:off], f"{name}: before the view")
        assert_bits_equal(got[off + n:], src[off + n:], f"{name}: behind the view")
    assert_bits_equal(dg.cpu().numpy(), g, "gradients are never written")


def test_randomised_call_sequences_match_the_oracle_state_machine():
    """Random hyper-parameters, step patterns (consecutive, repeated, jumping), beta changes, bias correction on/off,
    weight-decay forms, scales (none, powers of two, arbitrary) and sizes: the operator's host state machine and the
    kernels must track the oracle call for call, through both the flat-tensor and the chunk-list entry points."""
    lib = _lib.load()
    stream = _lib.current_stream_handle()
    rng = np.random.default_rng(2024)
    for trial in range(40):
        adamw = bool(rng.integers(0, 2))
        wd = float(rng.choice([0.0, 0.01, 0.3]))
        lr = float(10 ** rng.uniform(-5, -1))
        eps = float(10 ** rng.uniform(-10, -5))
        betas = [float(rng.choice([0.9, 0.8, 0.0, 0.95])), float(rng.choice([0.999, 0.99, 0.5]))]
        n = int(rng.choice([1, 63, 256, 257, 1000, 4096, 5000]))
        use_chunks = bool(rng.integers(0, 2))
        oid = 1000 + trial
        lib.ps_adam_create(oid, lr, betas[0], betas[1], eps, wd, int(adamw), 0)
        o = oracle.AdamOracle(lr, betas[0], betas[1], eps, wd, adamw)
        p = rng.normal(0, 0.05, n).astype(np.float32)
        m = rng.normal(0, 1e-3, n).astype(np.float32)
        v = np.abs(rng.normal(0, 1e-5, n)).astype(np.float32)
        dp, dm, dv = _dev(p.copy()), _dev(m.copy()), _dev(v.copy())
        step = int(rng.choice([0, 0, 10, 1000]))
        for call in range(5):
            step = {0: step + 1, 1: step + 1, 2: step, 3: step + int(rng.integers(2, 50))}[int(rng.integers(0, 4))]
            step = max(step, 1)
            if rng.random() < 0.2:
                betas[int(rng.integers(0, 2))] = float(rng.choice([0.85, 0.97, 0.9]))
            if rng.random() < 0.3:
                lr = float(10 ** rng.uniform(-5, -1))
            scale = float(rng.choice([-1.0, 0.0, 1.0, 8.0, 2.0**16, 1000.0, 3.3]))
            bias_correction = int(rng.random() < 0.8)
            g = (rng.normal(0, 1e-2, n) * (scale if scale > 0 else 1.0)).astype(np.float16)
            dg = _dev(g.copy())
            if use_chunks:
                table = _lib.chunk_array([[dp.data_ptr(), dm.data_ptr(), dv.data_ptr(), dg.data_ptr()]])
                rc = lib.ps_adam_step_chunks(oid, step, lr, betas[0], betas[1], eps, wd, bias_correction, table, 1, n, None, None, scale, stream)
            else:
                rc = lib.ps_adam_update(oid, step, lr, betas[0], betas[1], eps, wd, bias_correction, dp.data_ptr(), dg.data_ptr(), 1,
                                        dm.data_ptr(), dv.data_ptr(), n, scale, None, stream)
            assert rc == 0
            o.update(step, lr, betas[0], betas[1], eps, wd, bool(bias_correction), p, g, m, v, scale)
            torch.cuda.synchronize()
            what = f"trial {trial} call {call} (n={n}, step={step}, scale={scale}, chunks={use_chunks}, adamw={adamw}, wd={wd}, bc={bias_correction})"
            assert_bits_equal(dp.cpu().numpy(), p, what + " param")
            assert_bits_equal(dm.cpu().numpy(), m, what + " exp_avg")
            assert_bits_equal(dv.cpu().numpy(), v, what + " exp_avg_sq")
            if use_chunks:
                assert_bits_equal(dg.cpu().numpy(), oracle.cast_fp32_to_fp16(p), what + " fp16 param")
        lib.ps_adam_destroy(oid)


@pytest.mark.parametrize("offsets", [(1, 1, 1, 1), (0, 2, 0, 4), (3, 0, 1, 7), (0, 0, 0, 4)])
def test_chunk_step_with_unaligned_payload_bases(offsets):
    """Chunk payloads handed over at bases that are not 16-byte aligned (or aligned differently per list) take the
    element-wise tile path and must produce the same bits."""
    lib = _lib.load()
    rng = np.random.default_rng(sum(offsets))
    n, C = 256 * 5 + 19, 3
    op, om, ov, oh = offsets
    host = []
    dev = []
    rows = []
    for c in range(C):
        p = rng.normal(0, 0.02, n + 8).astype(np.float32)
        m = rng.normal(0, 1e-4, n + 8).astype(np.float32)
        v = np.abs(rng.normal(0, 1e-6, n + 8)).astype(np.float32)
        g = (rng.normal(0, 1e-3, n + 8) * 16).astype(np.float16)
        host.append((p, m, v, g))
        d = tuple(_dev(x.copy()) for x in (p, m, v, g))
        dev.append(d)
        rows.append([d[0][op:].data_ptr(), d[1][om:].data_ptr(), d[2][ov:].data_ptr(), d[3][oh:].data_ptr()])
    oid = 905
    lib.ps_adam_create(oid, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, 0)
    assert lib.ps_adam_step_chunks(oid, 3, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, _lib.chunk_array(rows), C, n, None, None, 16.0,
                                   _lib.current_stream_handle()) == 0
    torch.cuda.synchronize()
    lib.ps_adam_destroy(oid)
    o = oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-8, 0.01, True)
    o.advance(3, 0.9, 0.999)
    o.set(1e-3, 1e-8, 0.01, True)
    for (p, m, v, g), d in zip(host, dev):
        po, mo, vo, go = p[op:op + n].copy(), m[om:om + n].copy(), v[ov:ov + n].copy(), g[oh:oh + n].copy()
        assert oracle.lib().oracle_adam_span(o._buf, po.ctypes.data, go.ctypes.data, 1, mo.ctypes.data, vo.ctypes.data, n, 16.0, 0) > 0
        assert_bits_equal(d[0].cpu().numpy()[op:op + n], po, "param")
        assert_bits_equal(d[1].cpu().numpy()[om:om + n], mo, "exp_avg")
        assert_bits_equal(d[2].cpu().numpy()[ov:ov + n], vo, "exp_avg_sq")
        assert_bits_equal(d[3].cpu().numpy()[oh:oh + n], oracle.cast_fp32_to_fp16(po), "fp16 param")
        # nothing outside the views was touched
        assert_bits_equal(d[0].cpu().numpy()[:op], p[:op], "before")
        assert_bits_equal(d[0].cpu().numpy()[op + n:], p[op + n:], "after")
        assert_bits_equal(d[3].cpu().numpy()[oh + n:], g[oh + n:], "after fp16")


def test_randomised_shapes_hyperparameters_and_arithmetics():
    """Forty seeded random cases through ps_adam_step_chunks: list length, chunk length (down to one element),
    per-list base misalignment, step number, betas, decay form, scale kind and arithmetic all vary.  Each case is one
    cold step compared bit for bit with the matching CPU restatement."""
    lib = _lib.load()
    rng = np.random.default_rng(20240612)
    for case in range(40):
        C = int(rng.integers(1, 6))
        n = int(rng.choice([1, 3, 64, 255, 256, 257, 1000, int(rng.integers(300, 3000))]))
        offs = [int(o) for o in (rng.integers(0, 4, 4) if rng.random() < 0.5 else np.zeros(4, int))]
        offs[3] *= 2  # keep the fp16 list's phase comparable now and then
        step = int(rng.choice([1, 2, 17, 100, 5000]))
        b1, b2 = float(rng.choice([0.9, 0.8, 0.95])), float(rng.choice([0.999, 0.98, 0.95]))
        lr, eps = float(rng.choice([1e-3, 1e-4, 3e-5])), float(rng.choice([1e-8, 1e-6]))
        wd = float(rng.choice([0.0, 0.01, 0.1]))
        adamw = bool(rng.integers(0, 2))
        scale = [None, 8, 2**12, 2**16, 1000.0, 12345.678][int(rng.integers(0, 6))]
        torch_arith = bool(rng.integers(0, 2))
        what = f"case {case}: C={C} n={n} offs={offs} step={step} betas=({b1},{b2}) lr={lr} eps={eps} wd={wd} adamw={adamw} scale={scale} torch={torch_arith}"
        host, dev, rows = [], [], []
        for _ in range(C):
            p = rng.normal(0, 0.02, n + 16).astype(np.float32)
            m = rng.normal(0, 1e-4, n + 16).astype(np.float32)
            v = np.abs(rng.normal(0, 1e-6, n + 16)).astype(np.float32)
            g = (rng.normal(0, 1e-3, n + 16) * (scale or 1.0)).astype(np.float16)
            host.append((p, m, v, g))
            d = tuple(_dev(x.copy()) for x in (p, m, v, g))
            dev.append(d)
            rows.append([d[k][offs[k]:].data_ptr() for k in range(4)])
        oid = 3000 + case
        _lib.check(lib.ps_adam_create(oid, lr, b1, b2, eps, wd, int(adamw), 0), "create")
        if torch_arith:
            _lib.check(lib.ps_adam_set_arithmetic(oid, _lib.PS_ARITH_TORCH), "set_arithmetic")
        _lib.check(
            lib.ps_adam_step_chunks(oid, step, lr, b1, b2, eps, wd, 1, _lib.chunk_array(rows), C, n, None, None,
                                    float(scale) if scale is not None else -1.0, _lib.current_stream_handle()),
            what,
        )
        torch.cuda.synchronize()
        lib.ps_adam_destroy(oid)
        for (p, m, v, g), d in zip(host, dev):
            po, mo, vo, go = (np.ascontiguousarray(x[o:o + n]) for x, o in zip((p, m, v, g), offs))
            if torch_arith:
                oracle.torch_formula_update(po, go, mo, vo, step, lr, b1, b2, eps, wd, adamw, scale)
            else:
                oracle.AdamOracle(lr, b1, b2, eps, wd, adamw).update(
                    step, lr, b1, b2, eps, wd, True, po, go, mo, vo, float(scale) if scale is not None else -1.0)
            for k, (want, name) in enumerate(((po, "param"), (mo, "exp_avg"), (vo, "exp_avg_sq"), (oracle.cast_fp32_to_fp16(po), "fp16"))):
                got = d[k].cpu().numpy()
                assert_bits_equal(got[offs[k]:offs[k] + n], want, f"{what} {name}")
                # nothing outside the view was touched
                src = (p, m, v, g)[k]
                assert_bits_equal(got[:offs[k]], src[:offs[k]], f"{what} {name} before")
                assert_bits_equal(got[offs[k] + n:], src[offs[k] + n:], f"{what} {name} after")


def test_two_host_threads_step_their_own_optimizers_concurrently():
    """Entry points may be called from any host thread: two threads, each with its own optimizer id, chunk list and
    stream, step at the same time (ctypes drops the GIL during the calls); both must match the oracle."""
    import threading

    lib = _lib.load()
    n, C, steps = 256 * 30 + 11, 4, 25
    results, errors = {}, []

    def worker(tid):
        try:
            rng = np.random.default_rng(100 + tid)
            stream = torch.cuda.Stream()
            lr, wd = (1e-3, 0.0) if tid == 0 else (1e-4, 0.01)
            host = [(rng.normal(0, 0.02, n).astype(np.float32), np.zeros(n, np.float32), np.zeros(n, np.float32)) for _ in range(C)]
            grads = [[(rng.normal(0, 1e-3, n) * 8).astype(np.float16) for _ in range(C)] for _ in range(steps)]
            with torch.cuda.stream(stream):
                dev = [tuple(_dev(x.copy()) for x in h) + (torch.zeros(n, dtype=torch.half, device="cuda"),) for h in host]
                rows = _lib.chunk_array([[d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr()] for d in dev])
                oid = 700 + tid
                lib.ps_adam_create(oid, lr, 0.9, 0.999, 1e-8, wd, tid, 0)
                handle = _lib.current_stream_handle()
                for s in range(steps):
                    for c in range(C):
                        dev[c][3].copy_(torch.from_numpy(grads[s][c]), non_blocking=False)
                    assert lib.ps_adam_step_chunks(oid, s + 1, lr, 0.9, 0.999, 1e-8, wd, 1, rows, C, n, None, None, 8.0, handle) == 0
                stream.synchronize()
                lib.ps_adam_destroy(oid)
            o = oracle.AdamOracle(lr, 0.9, 0.999, 1e-8, wd, bool(tid))
            for s in range(steps):
                o.advance(s + 1, 0.9, 0.999)
                o.set(lr, 1e-8, wd, True)
                for c in range(C):
                    p, m, v = host[c]
                    assert oracle.lib().oracle_adam_span(o._buf, p.ctypes.data, grads[s][c].ctypes.data, 1, m.ctypes.data, v.ctypes.data, n, 8.0, 0) > 0
            results[tid] = (host, [tuple(t.cpu().numpy() for t in d) for d in dev])
        except Exception as e:  # surfaced by the main thread
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for tid in range(2):
        host, got = results[tid]
        for c in range(C):
            assert_bits_equal(got[c][0], host[c][0], f"thread {tid} chunk {c} param")
            assert_bits_equal(got[c][1], host[c][1], f"thread {tid} chunk {c} exp_avg")
            assert_bits_equal(got[c][2], host[c][2], f"thread {tid} chunk {c} exp_avg_sq")
            assert_bits_equal(got[c][3], oracle.cast_fp32_to_fp16(host[c][0]), f"thread {tid} chunk {c} fp16")
