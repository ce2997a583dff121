"""CPU-only tests of the host side: chunk layout known answers, config parsing, argument checks,
and that the C-ABI library loads and exports every symbol the header declares (no compute calls)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import patrickstar_amd as ps
from patrickstar_amd import _lib
from patrickstar_amd.chunk_layout import AccessType, ChunkTensorIndex, ChunkType, ParamType, register_param

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _param(n, name):
    p = torch.nn.Parameter(torch.zeros(n))
    register_param(p, ParamType.CHUNK_BASED, torch.float, name)
    return p


def test_first_fit_known_answers():
    """The expectations of the reference's unitest/test_chunk_data.py:51-102: sizes 10, 15, 5 in a 40-element chunk
    land at 0, 10, 25; 100 is rejected; re-inserting is a no-op; a second chunk starts at 0."""
    idx = ChunkTensorIndex(40)
    p1 = _param(10, "param1")
    idx.add_tensor(0, p1.ps_attr.data_id(), 0, p1.numel(), p1, AccessType.DATA)
    assert idx.tensor_id_to_chunk_id(p1.ps_attr.data_id()) == 0
    assert idx.get_chunk_id(p1, AccessType.DATA) == 0
    p2 = _param(15, "param2")
    assert idx.get_chunk_id(p2, AccessType.DATA) is None
    assert idx.try_insert_tensor(0, p2, AccessType.DATA)
    assert idx.get_tensor_info(p2.ps_attr.data_id()).start_offset == 10
    p3 = _param(5, "param3")
    assert idx.try_insert_tensor(0, p3, AccessType.DATA)
    assert idx.get_tensor_info(p3.ps_attr.data_id()).start_offset == 25
    p4 = _param(100, "param4")
    assert not idx.try_insert_tensor(0, p4, AccessType.DATA)
    p5 = _param(13, "param5")
    assert idx.try_insert_tensor(1, p5, AccessType.DATA)
    assert idx.get_tensor_info(p5.ps_attr.data_id()).start_offset == 0
    assert idx.try_insert_tensor(1, p5, AccessType.DATA)
    assert idx.get_tensor_info(p5.ps_attr.data_id()).start_offset == 0
    assert not idx.try_insert_tensor(1, _param(1000, "param6"), AccessType.DATA)
    assert [i.start_offset for i in idx.generate_tensor_info_in_order(0)] == [0, 10, 25]
    assert idx.used_numel(0) == 30


def test_first_fit_fills_gaps_and_list_insert_is_atomic():
    idx = ChunkTensorIndex(40)
    a, b, c = _param(10, "a"), _param(10, "b"), _param(10, "c")
    for p in (a, b, c):
        assert idx.try_insert_tensor(0, p, AccessType.DATA)
    idx.delete_tensor(0, b, AccessType.DATA)  # hole at [10, 20)
    big, small = _param(11, "big"), _param(6, "small")
    assert idx.try_insert_tensor(0, big, AccessType.DATA) is False or idx.get_tensor_info(big.ps_attr.data_id()).start_offset == 30
    assert idx.try_insert_tensor(0, small, AccessType.DATA)
    assert idx.get_tensor_info(small.ps_attr.data_id()).start_offset == 10
    # atomic list insert: the second member does not fit -> the first is rolled back
    idx2 = ChunkTensorIndex(20)
    x, y = _param(15, "x"), _param(10, "y")
    assert not idx2.try_insert_tensor_list(0, [x, y], AccessType.DATA)
    assert idx2.get_chunk_id(x, AccessType.DATA) is None and idx2.used_numel(0) == 0
    assert idx2.try_insert_tensor_list(0, [x], AccessType.DATA)


class _Tiny(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.a = torch.nn.Linear(4, 6)  # 24 + 6
        self.b = torch.nn.Linear(6, 2)  # 12 + 2
        self.scale = torch.nn.Parameter(torch.ones(3))


def test_client_packs_modules_in_construction_order_and_mirrors_offsets():
    client = ps.PatrickStarClient(0, 32, device="cpu")
    model = _Tiny()
    w0 = model.a.weight.detach().clone()
    client.register_model(model)
    idx = client.chunk_tensor_index
    ids16 = list(client.chunk_ids_generator(ChunkType.PARAM_FP16))
    ids32 = list(client.chunk_ids_generator(ChunkType.PARAM_FP32))
    assert len(ids16) == len(ids32) == 2
    # children first (a: 30 elements fills chunk 0 up to 30; b: 14 does not fit behind it -> chunk 1), then the parent's own (3)
    info = lambda p: idx.get_tensor_info(p.ps_attr.data_id())
    assert (info(model.a.weight).chunk_id, info(model.a.weight).start_offset) == (ids16[0], 0)
    assert (info(model.a.bias).chunk_id, info(model.a.bias).start_offset) == (ids16[0], 24)
    assert (info(model.b.weight).chunk_id, info(model.b.weight).start_offset) == (ids16[1], 0)
    assert (info(model.b.bias).chunk_id, info(model.b.bias).start_offset) == (ids16[1], 12)
    assert (info(model.scale).chunk_id, info(model.scale).start_offset) == (ids16[1], 14)
    # fp32 shadows share the layout; payloads hold the initial values, the tail is zero
    sh = client.param_fp16_to_param_fp32_map[model.a.weight]
    assert (info(sh).chunk_id, info(sh).start_offset) == (ids32[0], 0)
    assert torch.equal(client.access_data(sh), w0)
    assert torch.equal(client.access_data(model.a.weight), w0.half())
    assert not client.chunk_list[ids16[0]].payload[30:].any()
    assert client.chunk_list[ids16[0]].payload.dtype == torch.half and client.chunk_list[ids32[0]].payload.dtype == torch.float

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("HIP library not built")
    opt = ps.FP16Adam(client, model.parameters(), lr=1e-3)
    # optimizer() walks parameters in definition order (scale first), yet m/v sit at their parameter's own offset
    for p in model.parameters():
        for key, ctype in (("exp_avg", ChunkType.MOMENTUM), ("exp_avg_sq", ChunkType.VARIANCE)):
            sp = dict.__getitem__(opt.state[p], key)
            assert info(sp).start_offset == info(p).start_offset
            assert info(sp).chunk_id == idx.get_optimizer_state_chunk_id(p, AccessType.DATA, ctype)
            assert not client.access_data(sp).any()
    pos = client.positions()
    assert len(pos) == 2 and all(x.exp_avg is not None and x.exp_avg_sq is not None and not x.on_host for x in pos)
    assert opt.state[model.scale]["step"] == 0 and opt.state[model.scale]["lr"] == 1e-3
    sd = opt.state_dict()
    assert set(sd) == {"state", "param_groups"} and sd["state"][0]["exp_avg"].shape == model.scale.shape


def test_oversized_module_is_rejected():
    client = ps.PatrickStarClient(0, 16, device="cpu")
    with pytest.raises(RuntimeError, match="larger than the default chunk size"):
        client.register_model(torch.nn.Linear(8, 8))


def test_config_parsing_defaults_and_quirks():
    t, p, scaler, clip = ps.parse_config(None)
    assert (t, scaler, clip) == ("Adam", None, -1)
    assert p == {"lr": 0.01, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0, "use_hybrid_adam": True}
    t, p, scaler, clip = ps.parse_config({"optimizer": {"type": "AdamW", "params": {"lr": 1e-4}}, "gradient_clipping": 1.0})
    assert t == "AdamW" and p["lr"] == 1e-4 and p["betas"] == (0.9, 0.999) and scaler is None and clip == 1.0
    # the README configuration of the reference (README.md:59-92)
    cfg = {
        "optimizer": {"type": "Adam", "params": {"lr": 0.001, "betas": (0.9, 0.999), "eps": 1e-6, "weight_decay": 0, "use_hybrid_adam": True}},
        "fp16": {"enabled": True, "loss_scale": 0, "initial_scale_power": 2**3, "loss_scale_window": 1000, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 64 * 1024 * 1024, "release_after_init": True, "use_cpu_embedding": False,
    }
    t, p, scaler, clip = ps.parse_config(cfg)
    assert isinstance(scaler, ps.DynamicLossScaler)
    assert scaler.loss_scale == 2**8 and scaler.scale_factor == 2 and scaler.scale_window == 1000
    assert scaler.delayed_shift == 1 and scaler.consecutive_hysteresis is False and scaler.min_scale == 1
    # "hysteresis" feeds the scale FACTOR; the window defaults to 2000
    _, _, s2, _ = ps.parse_config({"fp16": {"enabled": True, "loss_scale": 0, "hysteresis": 4}})
    assert s2.scale_factor == 4 and s2.delayed_shift == 1 and s2.scale_window == 2000 and s2.loss_scale == 2**16
    _, _, s3, _ = ps.parse_config({"fp16": {"enabled": True, "loss_scale": 128}})
    assert isinstance(s3, ps.LossScaler) and s3.loss_scale == 128 and s3.has_overflow(None) is False
    s3.update_scale(True)
    assert s3.loss_scale == 128
    with pytest.raises(ValueError, match="Only support Adam and AdamW"):
        ps.parse_config({"optimizer": {"type": "SGD"}})
    with pytest.raises(AssertionError, match="Must enable fp16"):
        ps.parse_config({"fp16": {"enabled": False, "loss_scale": 0}})
    with pytest.raises(AssertionError, match="loss_scale"):
        ps.parse_config({"fp16": {"enabled": True}})


@pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="HIP library not built")
def test_fp16adam_argument_checks():
    client = ps.PatrickStarClient(0, 64, device="cpu")
    params = client.append_flat_chunks(1)
    for kw, msg in [
        (dict(lr=-1.0), "Invalid learning rate"),
        (dict(eps=-1e-8), "Invalid epsilon value"),
        (dict(betas=(1.0, 0.999)), "Invalid beta parameter at index 0"),
        (dict(betas=(0.9, -0.1)), "Invalid beta parameter at index 1"),
        (dict(weight_decay=-0.1), "Invalid weight_decay value"),
        (dict(arithmetic="fast"), "Invalid arithmetic"),
    ]:
        with pytest.raises(ValueError, match=msg):
            ps.FP16Adam(client, params, **kw)
    with pytest.raises(AssertionError, match="one param group"):
        ps.FP16Adam(client, [{"params": params[:1]}, {"params": [torch.nn.Parameter(torch.zeros(1))]}])
    first = ps.FP16Adam.optimizer_id
    a = ps.FP16Adam(client, params)
    assert a.opt_id == first and ps.FP16Adam.optimizer_id == first + 1
    assert a.has_overflow is False and a.loss_scaler is None
    del a


def test_library_loads_and_exports_every_declared_symbol():
    """Every function declared in include/ps_adam.h is exported by libps_adam.so and bound by the Python loader."""
    header = open(os.path.join(ROOT, "include", "ps_adam.h")).read()
    body = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ps_[a-z0-9_]+)\s*\(", body))
    assert len(declared) >= 17
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    assert os.path.exists(_lib.LIB_PATH), "build the HIP library first (python -m patrickstar_amd.build)"
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.ps_abi_version() == _lib.PS_ABI_VERSION == 5
    # host-only entry points: registry and argument checks work without a GPU
    assert lib.ps_adam_create(77, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0) == 0
    assert lib.ps_adam_destroy(77) == 0
    assert lib.ps_scaler_update(None, 0, None, 0, 1, None) == _lib.PS_ERR_BAD_ARG
    assert b"d_state" in lib.ps_last_error()
    assert lib.ps_state_init(None, 1.0, 1, 2.0, 1, 10, 1.0, 1, 1, 0, 0.9, 0.999, None) == _lib.PS_ERR_BAD_ARG
    assert ctypes.sizeof(_lib.ps_step_state) == 256 and ctypes.sizeof(_lib.ps_chunk) == 32


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.HipLibraryMissing, match="no CPU fallback"):
        _lib.load()
    client = ps.PatrickStarClient(0, 64, device="cpu")
    with pytest.raises(_lib.HipLibraryMissing):
        ps.FP16Adam(client, client.append_flat_chunks(1))


def test_dynamic_scaler_needs_a_gpu_for_anything_but_its_configuration():
    s = ps.DynamicLossScaler(init_scale=2**8, scale_window=10)
    assert s.loss_scale == 2**8 and s.cur_iter == 0 and s.last_overflow_iter == -1 and s.cur_hysteresis == 1
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="GPU"):
            s.update_scale(True)


def test_dynamic_scaler_refuses_int_scales_a_binary64_cannot_hold():
    # the device keeps the scale as a binary64; Python ints are exact at any size, so an int that would be rounded on
    # its way to the device is refused rather than changed silently
    for bad in (dict(init_scale=2**53 + 1), dict(min_scale=2**60 + 2**5), dict(scale_factor=2**53 + 1), dict(init_scale=2**2000)):
        with pytest.raises(ValueError, match="binary64"):
            ps.DynamicLossScaler(**bad)
    for good in (dict(init_scale=2**53), dict(init_scale=2**200), dict(init_scale=3 * 2**70, min_scale=5 * 2**60), dict(init_scale=2.0**60 + 1.0)):
        assert ps.DynamicLossScaler(**good).loss_scale == good["init_scale"]


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_registered_module_keeps_fp16_payloads_in_hbm_under_a_host_policy():
    client = ps.PatrickStarClient(0, 64, device="cpu", config={"host_chunk_policy": lambda pos: False})
    assert client.host_keeps_fp16 is True  # directly driven chunk lists: whole positions go to the host
    client.register_model(torch.nn.Linear(4, 4))
    assert client.host_keeps_fp16 is False  # a module computes with its fp16 payloads: only p32 / m / v may leave
    assert ps.PatrickStarClient(0, 64, device="cpu", config={"host_keeps_fp16": False}).host_keeps_fp16 is False


def test_plan_host_positions():
    n = 64 * 1024 * 1024
    per = 14 * n
    # everything fits: nothing goes to the host
    assert ps.plan_host_positions(24, n, free_bytes=288e9) == set()
    # the 12 B-parameter shape on a 160 GB budget: the last positions are the ones that leave
    planned = ps.plan_host_positions(180, n, free_bytes=160e9, staging_slots=2, margin_use_ratio=0.8)
    resident = 180 - len(planned)
    assert planned == set(range(resident, 180)) and 0 < resident < 180
    assert (resident + 2) * per <= 160e9 * 0.8 < (resident + 3) * per
    # nothing fits: all on the host
    assert ps.plan_host_positions(5, n, free_bytes=1e9) == set(range(5))
    policy = planned.__contains__
    assert policy(179) and not policy(0)
    # fp16 payloads of host positions stay in HBM: they cost 2 B/element there, and a staging slot 12
    planned12 = ps.plan_host_positions(180, n, free_bytes=160e9, staging_slots=2, margin_use_ratio=0.8, host_keeps_fp16=False)
    r12 = 180 - len(planned12)
    used = lambda r: r * per + (180 - r) * 2 * n + 2 * 12 * n
    assert planned12 == set(range(r12, 180)) and used(r12) <= 160e9 * 0.8 < used(r12 + 1) and r12 < resident


def test_product_never_touches_the_oracle():
    """The oracle is test infrastructure: nothing under patrickstar_amd/ may import, load or name it."""
    pkg = os.path.join(ROOT, "patrickstar_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


@pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="HIP library not built")
def test_argument_checks_happen_before_any_gpu_work():
    """Bad arguments are rejected on the host with a code and a message (no GPU is needed to see that)."""
    lib = _lib.load()
    lib.ps_adam_create(88, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0)
    fake = _lib.chunk_array([[16, 32, 48, 64]])  # never dereferenced: every call below fails validation first
    bad_slot = _lib.chunk_array([[16, 0, 48, 64]])
    E = _lib.PS_ERR_BAD_ARG
    assert lib.ps_adam_step_hybrid(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, 0, fake, 1, 1024, None, None, 2, None, 1.0, None, None) == E
    assert b"staging" in lib.ps_last_error()
    assert lib.ps_adam_step_hybrid(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, 0, fake, 1, 1024, None, fake, 0, None, 1.0, None, None) == E
    assert lib.ps_adam_step_hybrid(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, 0, fake, 1, 1024, None, fake, 9, None, 1.0, None, None) == E
    assert lib.ps_adam_step_hybrid(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, 0, fake, 1, 1024, None, bad_slot, 1, None, 1.0, None, None) == E
    assert lib.ps_adam_step_hybrid(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, 0, bad_slot, 1, 1024, None, fake, 1, None, 1.0, None, None) == E
    assert b"host chunk 0" in lib.ps_last_error()
    assert lib.ps_adam_step_hybrid(4711, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, None, 0, fake, 1, 1024, None, fake, 1, None, 1.0, None, None) == _lib.PS_ERR_UNKNOWN_ID
    assert lib.ps_adam_step_chunks_gated(88, 1e-3, 1e-8, 0.0, 1, fake, 1, 1024, None, None, None, None) == E
    assert lib.ps_overflow_scan_host_chunks(fake, 1, 1024, None, fake, 1, None, None) == E
    assert lib.ps_overflow_scan(None, 10, None, None) == E
    assert lib.ps_adam_set_grad_clamp(4711, 1.0) == _lib.PS_ERR_UNKNOWN_ID
    assert lib.ps_adam_set_grad_clamp(88, 1.0) == 0
    assert lib.ps_adam_set_arithmetic(88, 7) == E
    assert lib.ps_adam_set_arithmetic(88, _lib.PS_ARITH_TORCH) == 0
    assert lib.ps_adam_set_arithmetic(88, _lib.PS_ARITH_OPERATOR) == 0
    assert lib.ps_adam_set_arithmetic(4711, _lib.PS_ARITH_TORCH) == _lib.PS_ERR_UNKNOWN_ID
    # descriptors are validated before the operator's step scalars advance or anything is enqueued
    assert lib.ps_adam_step_chunks(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, bad_slot, 1, 1024, None, None, 1.0, None) == E
    assert b"chunk 0 has a NULL payload" in lib.ps_last_error()
    assert lib.ps_state_init(ctypes.c_void_p(16), 1.0, 1, 2.0, 1, 0, 1.0, 1, 1, 0, 0.9, 0.999, None) == E  # window 0
    assert b"scale_window" in lib.ps_last_error()
    assert lib.ps_scaler_update(ctypes.c_void_p(16), 3, None, 0, 1, None) == E
    assert lib.ps_scaler_update(ctypes.c_void_p(16), 0, None, 0, -1, None) == E
    assert lib.ps_state_seed_step(ctypes.c_void_p(16), -1, 0.9, 0.999, 1, None) == E
    # sizes beyond what one launch grid can cover (the runtime refuses 2^32 threads in a dimension: 2^26 - 1 tiles of 256
    # elements per chunk) are refused by every chunk-list entry point; 2^62 elements is beyond the limit of each of them,
    # whatever its tile size
    assert lib.ps_adam_step_chunks(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, fake, 1, 2**34, None, None, 1.0, None) == E
    assert b"beyond the launch grid" in lib.ps_last_error()
    huge = 2**62
    flag = ctypes.c_void_p(16)
    assert lib.ps_adam_step_chunks(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, fake, 1, huge, None, None, 1.0, None) == E
    assert b"beyond the launch grid" in lib.ps_last_error()
    assert lib.ps_adam_step_chunks_gated(88, 1e-3, 1e-8, 0.0, 1, fake, 1, huge, None, None, flag, None) == E
    assert lib.ps_overflow_scan_chunks(fake, 1, huge, None, flag, None) == E
    assert lib.ps_overflow_scan_chunks_noalloc(fake, 1, huge, flag, None) == E
    assert lib.ps_restore_fp16_chunks(fake, 1, huge, None, None) == E
    assert lib.ps_adam_step_hybrid(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, fake, 1, None, 0, huge, None, None, 0, None, 1.0, None, None) == E
    one = (ctypes.c_size_t * 1)(huge)
    assert lib.ps_adam_step_tensors(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, fake, one, 1, None, 1.0, None, None) == E
    assert b"beyond the launch grid" in lib.ps_last_error()
    # the per-tensor form: every record is looked at before the operator object moves or anything is queued
    numels = (ctypes.c_size_t * 2)(100, 200)
    two = _lib.chunk_array([[16, 16, 16, 16], [16, 16, 16, 16]])
    each = (_lib.ps_tensor_call * 2)()
    for e in each:
        e.lr, e.beta1, e.beta2, e.eps, e.weight_decay, e.step, e.arithmetic = 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, -1
    assert lib.ps_adam_step_tensors_each(4711, 1, two, numels, each, 2, 1.0, None, None, 0, None) == _lib.PS_ERR_UNKNOWN_ID
    assert lib.ps_adam_step_tensors_each(88, 1, two, numels, None, 2, 1.0, None, None, 0, None) == E
    each[1].arithmetic = 7
    assert lib.ps_adam_step_tensors_each(88, 1, two, numels, each, 2, 1.0, None, None, 0, None) == E
    assert b"each[1].arithmetic" in lib.ps_last_error()
    each[1].arithmetic, each[1].step = _lib.PS_ARITH_TORCH, 0
    assert lib.ps_adam_step_tensors_each(88, 1, two, numels, each, 2, 1.0, None, None, 0, None) == E
    assert b"at least 1" in lib.ps_last_error()
    # device-decided: a distance of 0 or less is fine, a workspace that is missing, short or misaligned is not
    assert lib.ps_tensors_each_workspace_bytes(2) == 128 and lib.ps_tensors_each_workspace_bytes(0) == 0
    assert lib.ps_adam_step_tensors_each(88, 1, two, numels, each, 2, 1.0, flag, None, 0, None) == E
    assert lib.ps_adam_step_tensors_each(88, 1, two, numels, each, 2, 1.0, flag, ctypes.c_void_p(4096), 127, None) == E
    assert b"needs 128" in lib.ps_last_error()
    assert lib.ps_adam_step_tensors_each(88, 1, two, numels, each, 2, 1.0, flag, ctypes.c_void_p(4104), 128, None) == E
    assert b"16-byte aligned" in lib.ps_last_error()
    numels[1] = huge
    assert lib.ps_adam_step_tensors_each(88, 1, two, numels, each, 2, 1.0, flag, ctypes.c_void_p(4096), 128, None) == E
    # used lengths beyond the chunk
    used = (ctypes.c_size_t * 1)(1025)
    assert lib.ps_adam_step_chunks(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, fake, 1, 1024, used, None, 1.0, None) == E
    assert b"used_numel" in lib.ps_last_error()
    # negative counts and a call pattern that does not fit the list
    assert lib.ps_adam_step_chunks(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, fake, -1, 1024, None, None, 1.0, None) == E
    assert lib.ps_adam_step_chunks(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, fake, 1, 1024, None, _lib.call_pattern(2, 1, 0, 10), 1.0, None) == E
    assert b"first_chunk" in lib.ps_last_error()
    assert lib.ps_adam_step_chunks(88, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, fake, 1, 1024, None, _lib.call_pattern(2, 0, 1000, 25), 1.0, None) == E
    assert b"does not fit a chunk" in lib.ps_last_error()
    lib.ps_adam_destroy(88)


def test_build_entry_point_compiles_and_loads():
    """__graft_entry__.build() in a fresh process: hipcc cross-compiles the library for gfx950 without a GPU, the CPU
    checker is rebuilt, the package imports and the ABI version matches the binding."""
    import subprocess
    import sys

    r = subprocess.run([sys.executable, "-c", "import __graft_entry__ as g; g.build()"], cwd=ROOT, capture_output=True,
                       text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "built" in r.stdout and os.path.exists(_lib.LIB_PATH)


def test_chunk_tensor_index_known_answers_of_the_reference_test():
    """The expectations of unitest/test_chunk_tensor_index.py:82-170: which of 10, 20, 30, 20, 7, 2 fit into a
    20-element chunk, and the insert / delete / insert sequence on tensor lists (7, 2 | 6, 5 | delete 6 | 8 | 7 | 1, 2, 3)."""
    idx = ChunkTensorIndex(20)
    fits = [idx.try_insert_tensor(0, _param(n, f"param_{i}"), AccessType.DATA) for i, n in enumerate([10, 20, 30, 20, 7, 2])]
    assert fits == [True, False, False, False, True, True]
    offsets = [i.start_offset for i in idx.generate_tensor_info_in_order(0)]
    assert offsets == sorted(offsets) == [0, 10, 17]

    idx = ChunkTensorIndex(20)
    first = [_param(7, "a"), _param(2, "b")]
    assert idx.try_insert_tensor_list(0, first, AccessType.DATA)
    second = [_param(6, "c"), _param(5, "d")]
    assert idx.try_insert_tensor_list(0, second, AccessType.DATA)  # 7, 2, 6, 5
    idx.delete_tensor(0, second[0], AccessType.DATA)  # 7, 2, (6), 5
    assert not idx.try_insert_tensor_list(0, [_param(8, "e")], AccessType.DATA)
    assert not idx.try_insert_tensor_list(0, [_param(7, "f")], AccessType.DATA)
    assert idx.try_insert_tensor_list(0, [_param(1, "g"), _param(2, "h"), _param(3, "i")], AccessType.DATA)
    assert [(t.start_offset, t.numel) for t in idx.generate_tensor_info_in_order(0)] == [(0, 7), (7, 2), (9, 1), (10, 2), (12, 3), (15, 5)]


def test_optimizer_state_chunk_map_known_answer():
    """unitest/test_chunk_tensor_index.py:172-213: two fp16 chunks (10, 5) and (6, 9); the momentum chunk of the first
    is unknown until registered, then it is the registered id for every parameter of that fp16 chunk only."""
    idx = ChunkTensorIndex(20)
    params = []
    for chunk_id, sizes in ((0, (10, 5)), (1, (6, 9))):
        for n in sizes:
            p = _param(n, f"param_{n}")
            assert idx.try_insert_tensor(chunk_id, p, AccessType.DATA)
            params.append(p)
    assert idx.get_optimizer_state_chunk_id(params[0], AccessType.DATA, ChunkType.MOMENTUM) is None
    idx.register_optimizer_state_chunk_id(params[0], AccessType.DATA, ChunkType.MOMENTUM, 3)
    assert idx.get_optimizer_state_chunk_id(params[0], AccessType.DATA, ChunkType.MOMENTUM) == 3
    assert idx.get_optimizer_state_chunk_id(params[1], AccessType.DATA, ChunkType.MOMENTUM) == 3
    assert idx.get_optimizer_state_chunk_id(params[2], AccessType.DATA, ChunkType.MOMENTUM) is None
    assert idx.get_optimizer_state_chunk_id(params[0], AccessType.DATA, ChunkType.VARIANCE) is None


def test_client_append_and_access_known_answer():
    """unitest/test_client.py:45-78: tensors of 10, 11, 12, 13 elements appended one by one to 40-element chunks
    (the fourth opens a second chunk), written through access_data and read back later."""
    client = ps.PatrickStarClient(rank=0, default_chunk_size=40, device="cpu")
    params, refs = [], []
    for i, n in enumerate([10, 11, 12, 13]):
        param = torch.nn.Parameter(torch.rand(n))
        refs.append(param.data.clone())
        register_param(param, ParamType.CHUNK_BASED, torch.float, f"param_{i}")
        client.append_tensor([param], torch.float, AccessType.DATA, ChunkType.PARAM_FP32)
        client.access_data(param, torch.device("cpu:0")).copy_(param.data)
        client.release_data(param)
        params.append(param)
    idx = client.chunk_tensor_index
    infos = [idx.get_tensor_info(p.ps_attr.data_id()) for p in params]
    assert [(t.chunk_id, t.start_offset) for t in infos] == [(0, 0), (0, 10), (0, 21), (1, 0)]
    for param, ref in zip(params, refs):
        assert torch.max(client.access_data(param, torch.device("cpu:0")) - ref) == 0
        client.release_data(param)


@pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="HIP library not built")
def test_step_tables_follow_the_reference_call_order_and_skip_frozen_parameters():
    """What FP16Adam hands to the library for one step (no GPU needed to build it).  The reference visits
    parameters in param_groups order and skips those with requires_grad=False (fp16_cpu_adam.py:566-605): the first
    operator call of a step is the first TRAINABLE parameter, wherever its chunk is; a chunk that also holds a frozen
    parameter cannot be updated as a whole."""
    def build(freeze=(), arithmetic="operator"):
        client = ps.PatrickStarClient(0, 32, device="cpu")
        model = _Tiny()
        for name in freeze:
            dict(model.named_parameters())[name].requires_grad_(False)
        client.register_model(model)
        opt = ps.FP16Adam(client, model.parameters(), lr=1e-3, weight_decay=0.1, arithmetic=arithmetic)
        opt._build_tables()
        return client, model, opt

    # parameters() order: scale (the parent's own, chunk 1 offset 14), a.weight, a.bias, b.weight, b.bias
    client, model, opt = build()
    assert opt._tensor_table is None and opt._tables[1] == 2 and opt._operator_calls == 5
    pat = opt._calls._obj
    assert (pat.n_calls, pat.first_chunk, pat.first_offset, pat.first_numel) == (5, 1, 14, 3)

    # the torch formula never calls the operator for HBM-resident state
    _, _, opt = build(arithmetic="torch")
    assert opt._calls is None and opt._operator_calls == 0

    # scale frozen: the first call moves to a.weight; chunk 1 now mixes frozen and trainable -> tensor by tensor
    client, model, opt = build(freeze=("scale",))
    rows, numels, n = opt._tensor_table
    assert n == 4 and list(numels) == [24, 6, 12, 2] and opt._operator_calls == 4
    want = [client.access_data(p).data_ptr() for p in (model.a.weight, model.a.bias, model.b.weight, model.b.bias)]
    assert [rows[i].param_fp16 for i in range(4)] == want
    for i, p in enumerate((model.a.weight, model.a.bias, model.b.weight, model.b.bias)):
        assert rows[i].param_fp32 == client.access_data(client.param_fp16_to_param_fp32_map[p]).data_ptr()
        assert rows[i].exp_avg == client.access_data(dict.__getitem__(opt.state[p], "exp_avg")).data_ptr()

    # a whole chunk frozen (a.weight and a.bias are all of chunk 0): that position simply drops out
    client, model, opt = build(freeze=("a.weight", "a.bias"))
    assert opt._tensor_table is None and opt._tables[1] == 1 and opt._operator_calls == 3
    pat = opt._calls._obj
    assert (pat.n_calls, pat.first_chunk, pat.first_offset, pat.first_numel) == (3, 0, 14, 3)


@pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="HIP library not built")
def test_hyper_parameters_are_read_from_the_state_entries_per_parameter():
    """The reference reads lr / betas / eps / weight_decay from state[p] per tensor (fp16_cpu_adam.py:593-598), not
    from param_groups, and hands each operator call its own (:403-428).  While every trainable parameter agrees the
    whole chunk list goes to one fused call; entries that differ send the step tensor by tensor, each with its own
    numbers; frozen parameters are not looked at."""
    client = ps.PatrickStarClient(0, 32, device="cpu")
    model = _Tiny()
    model.a.bias.requires_grad_(False)
    client.register_model(model)
    opt = ps.FP16Adam(client, model.parameters(), lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=0.1)
    assert opt._hyper() == (1e-3, (0.9, 0.99), 1e-6, 0.1)
    opt.param_groups[0]["lr"] = 7.0  # ignored, as in the reference
    assert opt._plan is not None and opt._hyper()[0] == 1e-3
    opt.state[model.b.weight]["lr"] = 5e-4
    assert opt._plan is None and opt._hyper() == "each"
    rows, numels, n, each, workspace, operator_calls, offsets, managed = opt._each_table(opt._plan)
    trainable = [model.scale, model.a.weight, model.b.weight, model.b.bias]  # parameters() order without a.bias
    assert n == 4 == operator_calls and workspace is None and list(numels) == [p.numel() for p in trainable]
    assert [each[i].lr for i in range(4)] == [1e-3, 1e-3, 5e-4, 1e-3]
    assert all((each[i].beta1, each[i].beta2, each[i].eps, each[i].weight_decay) == (0.9, 0.99, 1e-6, 0.1) for i in range(4))
    assert all(each[i].arithmetic == _lib.PS_ARITH_OPERATOR for i in range(4))
    assert [rows[i].param_fp16 for i in range(4)] == [client.access_data(p).data_ptr() for p in trainable]
    for p in model.parameters():
        if p.requires_grad:
            opt.state[p]["lr"] = 5e-4
    assert opt._hyper()[0] == 5e-4
    opt.state[model.a.bias]["weight_decay"] = 0.5  # frozen: never handed to the operator
    assert opt._hyper() == (5e-4, (0.9, 0.99), 1e-6, 0.1)


def _tiny_optimizer(freeze=(), **kw):
    client = ps.PatrickStarClient(0, 32, device="cpu")
    model = _Tiny()
    for name in freeze:
        dict(model.named_parameters())[name].requires_grad_(False)
    client.register_model(model)
    return client, model, ps.FP16Adam(client, model.parameters(), lr=1e-3, **kw)


@pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="HIP library not built")
def test_a_checkpoint_with_a_frozen_last_parameter_resumes_at_its_step_count():
    """load_state_dict restores `step` per parameter (fp16_cpu_adam.py:660-694).  The counter the next step continues
    from is that of the TRAINABLE parameters: the last parameter in parameters() order is frozen here and stands at 0
    steps while the others have made 7; a resumed optimizer must go on with step 8, not with step 1."""
    _, model, opt = _tiny_optimizer(freeze=("b.bias",))
    opt._make_plan()
    opt._common_step, opt._steps_dirty = 7, True  # as seven host-decided steps leave it
    sd = opt.state_dict()
    assert [sd["state"][i]["step"] for i in range(5)] == [7, 7, 7, 7, 0]
    _, model2, opt2 = _tiny_optimizer(freeze=("b.bias",))
    opt2.load_state_dict(sd)
    assert [dict.__getitem__(opt2.state[p], "step") for p in model2.parameters()] == [7, 7, 7, 7, 0]
    opt2._make_plan()
    assert opt2._plan["kind"] == "uniform" and opt2._common_step == 7 and opt2._offsets == {}
    assert opt2.state[model2.scale]["step"] == 7 and opt2.state[model2.b.bias]["step"] == 0
    # betas and the other entries come from the checkpoint too
    sd["state"][0]["betas"] = sd["state"][1]["betas"] = sd["state"][2]["betas"] = sd["state"][3]["betas"] = (0.8, 0.9)
    opt2.load_state_dict(sd)
    assert opt2._hyper()[1] == (0.8, 0.9)


@pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="HIP library not built")
def test_a_parameter_that_missed_steps_keeps_its_own_step_number():
    """The reference counts state[p]["step"] per parameter (fp16_cpu_adam.py:571-574): a parameter that was frozen for
    some steps stands behind the others when it becomes trainable again, and each operator call gets its tensor's own
    step number (:406,603).  The plan keeps such a parameter's distance from the common counter."""
    _, model, opt = _tiny_optimizer()
    opt._make_plan()
    opt._common_step, opt._steps_dirty = 2, True  # two steps with everything trainable
    model.b.weight.requires_grad_(False)
    opt._make_plan()
    assert opt._plan["kind"] == "uniform" and opt.state[model.b.weight]["step"] == 2
    opt._common_step, opt._steps_dirty = 5, True  # three more without b.weight
    assert opt.state[model.scale]["step"] == 5 and opt.state[model.b.weight]["step"] == 2
    model.b.weight.requires_grad_(True)
    opt._make_plan()
    assert opt._plan["kind"] == "each" and opt._common_step == 5 and opt._offsets == {model.b.weight: -3}
    opt._common_step, opt._steps_dirty = 6, True  # one step together: both advance
    assert opt.state[model.scale]["step"] == 6 and opt.state[model.b.weight]["step"] == 3
    # the first trainable parameter defines the common counter: freeze it and the counter moves to the next one's
    model.scale.requires_grad_(False)
    opt._make_plan()
    assert opt._common_step == 6 and opt._offsets == {model.b.weight: -3} and opt.state[model.scale]["step"] == 6
    # writing an entry by hand is picked up like any other change
    opt.state[model.b.weight]["step"] = 6
    opt._make_plan()
    assert opt._plan["kind"] == "uniform" and opt._offsets == {}


def test_placement_is_decided_from_the_free_hbm_when_the_model_is_registered():
    """use_hybrid_adam + a memory margin decide where optimizer state lives (fp16_cpu_adam.py:523-528,
    memtracer.py:190-214, chunk_io_buff.py:234-239): everything resident when it fits, the FIRST positions resident
    when it does not, an error when it does not and hybrid Adam is off; an explicit policy is left alone."""
    def client_with(n_layers=6, **cfg):
        client = ps.PatrickStarClient(0, 300, device="cpu", config=cfg or None)
        for _ in range(n_layers):
            client.register_module_params(torch.nn.Linear(16, 16))  # 272 elements: one position each
        return client

    per = 14 * 300
    c = client_with()
    c.plan_placement(free_bytes=6 * per / 0.8)
    assert c.host_chunk_policy is None and c.placement["host_positions"] == []
    # 22,400 usable bytes: 6 fp16 payloads (3,600) + 3 staging slots (10,800) leave room for 2 resident states (3,600 each)
    c = client_with(hbm_budget_bytes=28000)
    c.plan_placement()
    assert c.placement["host_positions"] == [2, 3, 4, 5] and c.placement["free_bytes"] == 28000
    assert [c.host_chunk_policy(i) for i in range(6)] == [False, False, True, True, True, True]
    c = client_with(hbm_budget_bytes=28000)
    c.use_hybrid_adam = False
    with pytest.raises(RuntimeError, match="use_hybrid_adam is False"):
        c.plan_placement()
    keep = lambda pos: pos == 0
    c = client_with(hbm_budget_bytes=1, host_chunk_policy=keep)
    c.plan_placement()
    assert c.host_chunk_policy is keep and c.placement == {"source": "host_chunk_policy"}
    # no budget and no GPU to ask: nothing is moved
    c = client_with()
    c.plan_placement()
    assert c.host_chunk_policy is None


@pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="HIP library not built")
def test_layout_invariants_hold_for_random_models():
    """Random stacks of Linear layers (with and without bias, some with a parameter of the parent's own) and random chunk
    sizes: every parameter gets a span inside one chunk, spans of a chunk do not overlap and appear in insertion order,
    the parameters of one module share a chunk (first-fit by module, core/client.py:246-280), the fp32 master and
    both optimizer states of a parameter sit at the parameter's own chunk position and offset, payloads start with the
    initial values and are zero behind the last tensor, and what FP16Adam hands to the library names every trainable
    tensor exactly once."""
    from hypothesis import given, settings, strategies as st

    @settings(max_examples=40, deadline=None)
    @given(widths=st.lists(st.integers(1, 9), min_size=2, max_size=7), slack=st.integers(0, 40), biases=st.integers(0, 127),
           own=st.booleans(), frozen=st.integers(0, 1 << 14))
    def check(widths, slack, biases, own, frozen):
        ran.append(1)

        class Net(torch.nn.Module):
            def __init__(self):
                super().__init__()
                self.layers = torch.nn.ModuleList(
                    [torch.nn.Linear(a, b, bias=bool((biases >> i) & 1)) for i, (a, b) in enumerate(zip(widths[:-1], widths[1:]))])
                if own:
                    self.own = torch.nn.Parameter(torch.arange(3.0))

        torch.manual_seed(0)
        model = Net()
        params = list(model.parameters())
        for i, p in enumerate(params):
            if (frozen >> i) & 1 and i:  # the first parameter stays trainable
                p.requires_grad_(False)
        chunk = max(sum(q.numel() for q in layer.parameters()) for layer in model.layers) + slack
        chunk = max(chunk, 3)
        init = {n: p.detach().clone() for n, p in model.named_parameters()}
        client = ps.PatrickStarClient(0, chunk, device="cpu")
        client.register_model(model)
        opt = ps.FP16Adam(client, model.parameters(), lr=1e-3)
        idx = client.chunk_tensor_index
        info = lambda p: idx.get_tensor_info(p.ps_attr.data_id())
        position_of = {q.fp16: i for i, q in enumerate(client.positions())}
        # spans: inside the chunk, disjoint, in insertion order
        for q in client.positions():
            end = 0
            for t in idx.generate_tensor_info_in_order(q.fp16):
                assert t.start_offset >= end and t.start_offset + t.numel <= chunk
                end = t.start_offset + t.numel
            assert not client.chunk_list[q.fp16].payload[end:].any() and not client.chunk_list[q.fp32].payload[end:].any()
        for layer in model.layers:
            assert len({info(p).chunk_id for p in layer.parameters()}) == 1
        for name, p in model.named_parameters():
            assert torch.equal(client.access_data(p), init[name].half())
            master = client.param_fp16_to_param_fp32_map[p]
            assert torch.equal(client.access_data(master), init[name])
            pos = client.positions()[position_of[info(p).chunk_id]]
            for shadow, cid in ((master, pos.fp32), (dict.__getitem__(opt.state[p], "exp_avg"), pos.exp_avg),
                                (dict.__getitem__(opt.state[p], "exp_avg_sq"), pos.exp_avg_sq)):
                assert (info(shadow).chunk_id, info(shadow).start_offset, info(shadow).numel) == (cid, info(p).start_offset, p.numel())
        # what one step covers: every trainable element exactly once, no frozen one
        table, n_dev, host_positions = opt._build_tables()
        assert not host_positions
        trainable = [p for p in params if p.requires_grad]
        if opt._tensor_table is not None:
            rows, numels, n = opt._tensor_table
            assert n == len(trainable) and list(numels) == [p.numel() for p in trainable]
            assert [rows[i].param_fp16 for i in range(n)] == [client.access_data(p).data_ptr() for p in trainable]
        else:
            live = {info(p).chunk_id for p in trainable}
            assert n_dev == len(live)
            for cid in live:  # a whole-chunk step is only taken when nothing frozen shares a live chunk
                assert all(t.param.requires_grad for t in idx.generate_tensor_info_in_order(cid))
        assert opt._operator_calls == len(trainable)
        first = opt._calls._obj
        live_positions = [q for q in client.positions() if any(t.param.requires_grad for t in idx.generate_tensor_info_in_order(q.fp16))]
        assert live_positions[first.first_chunk].fp16 == info(trainable[0]).chunk_id
        assert (first.n_calls, first.first_offset, first.first_numel) == (len(trainable), info(trainable[0]).start_offset, trainable[0].numel())

    ran = []
    check()
    assert len(ran) >= 20


@pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="HIP library not built")
def test_per_parameter_step_counts_follow_the_reference_under_random_schedules():
    """state[p]["step"] under random sequences of steps, freezing, thawing, hand-written entries and checkpoint reloads,
    against the reference's rule written out plainly (fp16_cpu_adam.py:569-574: every step adds one to the count of every
    parameter that is trainable at that moment).  No GPU: a host-decided step is stood in for by what it does to the
    common counter."""
    rng = np.random.default_rng(0)
    for case in range(30):
        client, model, opt = _tiny_optimizer()
        params = list(model.parameters())
        want = {p: 0 for p in params}

        def host_decided_step():
            if opt._plan is None or tuple(p.requires_grad for p in params) != opt._trainable_seen:
                opt._make_plan()
            if opt._plan["kind"] != "empty":
                opt._common_step += 1
                opt._steps_dirty = True
            for p in params:
                if p.requires_grad:
                    want[p] += 1

        for _ in range(40):
            op = rng.integers(0, 10)
            if op < 5:
                host_decided_step()
            elif op < 7:
                params[int(rng.integers(0, len(params)))].requires_grad_(bool(rng.integers(0, 2)))
            elif op == 7:
                p = params[int(rng.integers(0, len(params)))]
                value = int(rng.integers(0, 20))
                opt.state[p]["step"] = value
                want[p] = value
            elif op == 8:
                sd = opt.state_dict()
                assert [sd["state"][i]["step"] for i in range(len(params))] == [want[p] for p in params]
                client, model2, opt2 = _tiny_optimizer()
                params2 = list(model2.parameters())
                for p, q in zip(params, params2):
                    q.requires_grad_(p.requires_grad)
                opt2.load_state_dict(sd)
                want = {q: want[p] for p, q in zip(params, params2)}
                model, opt, params = model2, opt2, params2
            else:
                assert [opt.state[p]["step"] for p in params] == [want[p] for p in params], case
            if opt._plan is not None and opt._plan["kind"] == "uniform":
                trainable = [p for p in params if p.requires_grad]
                assert len({want[p] for p in trainable}) <= 1 or tuple(p.requires_grad for p in params) != opt._trainable_seen
        assert [opt.state[p]["step"] for p in params] == [want[p] for p in params], case
