"""ctypes binding of libps_adam.so (the C ABI declared in include/ps_adam.h).

There is no CPU fallback: if the library has not been built, loading raises.
"""
import ctypes
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libps_adam.so")

PS_FLAG_FALSE, PS_FLAG_TRUE, PS_FLAG_FROM_DEVICE = 0, 1, 2
PS_ERR_BAD_ARG, PS_ERR_UNKNOWN_ID, PS_ERR_NO_DEVICE = -10001, -10002, -10003
PS_ARITH_OPERATOR, PS_ARITH_TORCH = 0, 1
PS_TENSOR_GRAD_F32 = 1
PS_ABI_VERSION = 5


class ps_chunk(ctypes.Structure):
    _fields_ = [
        ("param_fp32", ctypes.c_void_p),
        ("exp_avg", ctypes.c_void_p),
        ("exp_avg_sq", ctypes.c_void_p),
        ("param_fp16", ctypes.c_void_p),
    ]


class ps_step_state(ctypes.Structure):
    _fields_ = [
        ("cur_scale", ctypes.c_double),
        ("scale_factor", ctypes.c_double),
        ("min_scale", ctypes.c_double),
        ("cur_iter", ctypes.c_int64),
        ("last_overflow_iter", ctypes.c_int64),
        ("scale_window", ctypes.c_int64),
        ("adam_step", ctypes.c_int64),
        ("skipped_steps", ctypes.c_int64),
        ("delayed_shift", ctypes.c_int32),
        ("cur_hysteresis", ctypes.c_int32),
        ("consecutive_hysteresis", ctypes.c_int32),
        ("scale_is_int", ctypes.c_int32),
        ("factor_is_int", ctypes.c_int32),
        ("min_is_int", ctypes.c_int32),
        ("overflow", ctypes.c_uint32),
        ("last_skipped", ctypes.c_uint32),
        ("beta1", ctypes.c_float),
        ("beta2", ctypes.c_float),
        ("beta1_t_next", ctypes.c_float),
        ("beta2_t_next", ctypes.c_float),
        ("reserved", ctypes.c_uint32 * 4),
        ("beta1_f64", ctypes.c_double),
        ("beta2_f64", ctypes.c_double),
        ("bias_correction1_next", ctypes.c_double),
        ("bias_correction2_next", ctypes.c_double),
        ("operator_step", ctypes.c_int64),
        ("beta1_t_cur", ctypes.c_float),
        ("beta2_t_cur", ctypes.c_float),
        ("beta1_t_rest", ctypes.c_float),
        ("beta2_t_rest", ctypes.c_float),
        ("reserved2", ctypes.c_uint32 * 2),
        ("operator_beta1", ctypes.c_float),
        ("operator_beta2", ctypes.c_float),
        ("pending_operator_step", ctypes.c_int64),
        ("pending_beta1_t", ctypes.c_float),
        ("pending_beta2_t", ctypes.c_float),
        ("pending_beta1", ctypes.c_float),
        ("pending_beta2", ctypes.c_float),
        ("reserved3", ctypes.c_uint32 * 8),
    ]


class ps_call_pattern(ctypes.Structure):
    _fields_ = [
        ("n_calls", ctypes.c_int64),
        ("first_chunk", ctypes.c_int64),
        ("first_offset", ctypes.c_uint64),
        ("first_numel", ctypes.c_uint64),
    ]


class ps_tensor_call(ctypes.Structure):
    _fields_ = [
        ("lr", ctypes.c_double),
        ("beta1", ctypes.c_double),
        ("beta2", ctypes.c_double),
        ("eps", ctypes.c_double),
        ("weight_decay", ctypes.c_double),
        ("step", ctypes.c_int64),
        ("arithmetic", ctypes.c_int32),
        ("flags", ctypes.c_int32),
    ]


class ps_scale_record(ctypes.Structure):
    _fields_ = [
        ("scale_after", ctypes.c_double),
        ("overflow", ctypes.c_uint32),
        ("scale_is_int", ctypes.c_uint32),
    ]


assert ctypes.sizeof(ps_chunk) == 32
assert ctypes.sizeof(ps_step_state) == 256
assert ctypes.sizeof(ps_call_pattern) == 32
assert ctypes.sizeof(ps_scale_record) == 16
assert ctypes.sizeof(ps_tensor_call) == 56

_f, _d, _i, _i64, _sz, _vp = (
    ctypes.c_float,
    ctypes.c_double,
    ctypes.c_int,
    ctypes.c_int64,
    ctypes.c_size_t,
    ctypes.c_void_p,
)

# name -> (restype, argtypes); one entry per declaration in include/ps_adam.h
SIGNATURES = {
    "ps_abi_version": (_i, []),
    "ps_last_error": (ctypes.c_char_p, []),
    "ps_adam_create": (_i, [_i, _f, _f, _f, _f, _f, _i, _i]),
    "ps_adam_set_grad_clamp": (_i, [_i, _d]),
    "ps_adam_set_arithmetic": (_i, [_i, _i]),
    "ps_adam_destroy": (_i, [_i]),
    "ps_adam_update": (_i, [_i, _sz, _f, _f, _f, _f, _f, _i, _vp, _vp, _i, _vp, _vp, _sz, _f, _vp, _vp]),
    "ps_adam_step_chunks": (_i, [_i, _sz, _d, _d, _d, _d, _d, _i, _vp, _i, _sz, _vp, _vp, _d, _vp]),
    "ps_adam_step_chunks_gated": (_i, [_i, _d, _d, _d, _i, _vp, _i, _sz, _vp, _vp, _vp, _vp]),
    "ps_adam_step_tensors": (_i, [_i, _sz, _d, _d, _d, _d, _d, _i, _vp, _vp, _i, _vp, _d, _vp, _vp]),
    "ps_tensors_each_workspace_bytes": (_sz, [_i]),
    "ps_adam_step_tensors_each": (_i, [_i, _i, _vp, _vp, _vp, _i, _d, _vp, _vp, _sz, _vp]),
    "ps_adam_step_hybrid": (_i, [_i, _sz, _d, _d, _d, _d, _d, _i, _vp, _i, _vp, _i, _sz, _vp, _vp, _i, _vp, _d, _vp, _vp]),
    "ps_overflow_scan_host_chunks": (_i, [_vp, _i, _sz, _vp, _vp, _i, _vp, _vp]),
    "ps_restore_fp16_chunks": (_i, [_vp, _i, _sz, _vp, _vp]),
    "ps_cast_fp32_to_fp16": (_i, [_vp, _vp, _sz, _vp]),
    "ps_state_init": (_i, [_vp, _d, _i, _d, _i, _i64, _d, _i, _i, _i, _d, _d, _vp]),
    "ps_state_seed_step": (_i, [_vp, _i64, _d, _d, _i, _vp]),
    "ps_state_set_scaler": (_i, [_vp, _d, _i, _i64, _i64, _i, _vp]),
    "ps_overflow_scan": (_i, [_vp, _sz, _vp, _vp]),
    "ps_overflow_scan_f32": (_i, [_vp, _sz, _vp, _vp]),
    "ps_overflow_scan_chunks": (_i, [_vp, _i, _sz, _vp, _vp, _vp]),
    "ps_overflow_scan_chunks_noalloc": (_i, [_vp, _i, _sz, _vp, _vp]),
    "ps_grad_to_chunk": (_i, [_vp, _i, _vp, _sz, _vp, _vp]),
    "ps_scaler_update": (_i, [_vp, _i, _vp, _i64, _i64, _vp]),
    "ps_state_read": (_i, [_vp, ctypes.POINTER(ps_step_state), _vp]),
}

_lib = None


class HipLibraryMissing(RuntimeError):
    pass


def load():
    """Load libps_adam.so once; raise HipLibraryMissing if it was never built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipLibraryMissing(
            f"{LIB_PATH} not found: build it with `python -m patrickstar_amd.build` "
            "(hipcc, --offload-arch=gfx950). There is no CPU fallback for this path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.ps_abi_version() != PS_ABI_VERSION:
        raise HipLibraryMissing(
            f"{LIB_PATH} has ABI version {lib.ps_abi_version()}, expected {PS_ABI_VERSION}; rebuild it"
        )
    _lib = lib
    return lib


def check(rc, what):
    """Map a non-zero return code of the C ABI to RuntimeError with the library's text."""
    if rc != 0:
        msg = load().ps_last_error()
        raise RuntimeError(f"{what} failed (code {rc}): {msg.decode() if msg else ''}")


def current_stream_handle():
    import torch

    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def call_pattern(n_calls, first_chunk=0, first_offset=0, first_numel=0):
    """A ps_call_pattern, by reference, for the `calls` argument of the step entry points."""
    return ctypes.byref(ps_call_pattern(int(n_calls), int(first_chunk), int(first_offset), int(first_numel)))


def size_array(values):
    """Host array of size_t, or None for an empty / absent list."""
    return (ctypes.c_size_t * len(values))(*values) if values else None


def chunk_array(rows):
    """Host array of ps_chunk descriptors from rows of (fp32, exp_avg, exp_avg_sq, fp16) addresses."""
    arr = (ps_chunk * len(rows))()
    for i, (p32, m, v, p16) in enumerate(rows):
        arr[i].param_fp32, arr[i].exp_avg, arr[i].exp_avg_sq, arr[i].param_fp16 = p32, m, v, p16
    return arr
