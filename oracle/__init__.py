"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

CPU restatement of the reference's chunk-wise mixed-precision optimizer step,
used only as the parity checker by ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``.  ``patrickstar_amd`` never imports it.

Contents
--------
``AdamOracle``            ctypes front-end of ``adam_oracle.c`` (the native operator,
                          ``patrickstar/ops/csrc/adam/cpu_adam.cpp:33-185,700-742`` and
                          ``csrc/includes/cpu_adam.h:143-175``).
``torch_formula_update``  ``FP16Adam.torch_adam_update`` (``patrickstar/ops/fp16_cpu_adam.py:245-277``
                          with the scalars of ``:412-413``), the branch the reference takes for
                          optimizer state in GPU memory; scalars formed here in Python arithmetic as
                          there, per-element rounding in ``adam_oracle.c: oracle_torch_adam_span``.
``cast_fp32_to_fp16``     whole-chunk RNE write-back (``patrickstar/ops/chunk_io_buff.py:116-126``).
``has_inf_or_nan``        ``patrickstar/fp16/loss_scaler.py:133-155``.
``ScalerOracle``          ``patrickstar/fp16/loss_scaler.py:107-182`` state machine.
``StaticScalerOracle``    ``patrickstar/fp16/loss_scaler.py:46-76``.
``scaler_from_config``    ``patrickstar/runtime/engine.py:79-99`` wiring (``hysteresis`` feeds
                          ``scale_factor``; ``delayed_shift`` is always 1 through the engine).
``OptimizerStepOracle``   sequencing of ``patrickstar/ops/fp16_cpu_adam.py:472-628`` over a
                          chunk list held as numpy arrays.

Pinning: see the header of ``adam_oracle.c`` for the Adam arithmetic and
``tests/test_oracle_scaler.py`` for the state machine (torch's AMP scale-update
routine on random overflow histories, hand-derived trajectories, invariants).  The reference's own tests hold no golden vectors for this
path; its loss-scale sequence is asserted nowhere in the reference.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_adam.so")
_lib = None

ISA_AUTO, ISA_SCALAR, ISA_AVX2, ISA_AVX512 = 0, 1, 2, 3


def build(force=False):
    """Compile ``adam_oracle.c`` with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        f, u64, sz, vp, ci = (
            ctypes.c_float,
            ctypes.c_uint64,
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_int,
        )
        L.oracle_sizeof_state.restype = ci
        L.oracle_adam_init.argtypes = [vp, f, f, f, f, f, ci]
        L.oracle_adam_init.restype = None
        L.oracle_adam_advance.argtypes = [vp, u64, f, f]
        L.oracle_adam_advance.restype = None
        L.oracle_adam_set.argtypes = [vp, f, f, f, ci]
        L.oracle_adam_set.restype = None
        L.oracle_adam_consts.argtypes = [vp, f, vp]
        L.oracle_adam_consts.restype = None
        L.oracle_adam_span.argtypes = [vp, vp, vp, ci, vp, vp, sz, f, ci]
        L.oracle_adam_span.restype = ci
        L.oracle_adam_update.argtypes = [vp, u64, f, f, f, f, f, ci, vp, vp, ci, vp, vp, sz, f, ci]
        L.oracle_adam_update.restype = ci
        L.oracle_f32_to_f16.argtypes = [f]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = f
        L.oracle_cast_f32_to_f16.argtypes = [vp, vp, sz]
        L.oracle_cast_f32_to_f16.restype = None
        L.oracle_any_nonfinite_f16.argtypes = [vp, sz]
        L.oracle_any_nonfinite_f16.restype = ci
        L.oracle_torch_adam_span.argtypes = [vp, ci, ci, vp, vp, vp, vp, sz]
        L.oracle_torch_adam_span.restype = None
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _check(a, dtype):
    assert isinstance(a, np.ndarray) and a.dtype == dtype and a.flags["C_CONTIGUOUS"], (
        type(a),
        getattr(a, "dtype", None),
    )


class AdamOracle:
    """One native optimizer object of the reference (``create_adam`` ... ``adam_update``)."""

    def __init__(self, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, adamw_mode=True):
        self._L = lib()
        self._buf = ctypes.create_string_buffer(self._L.oracle_sizeof_state())
        self._L.oracle_adam_init(self._buf, lr, beta1, beta2, eps, weight_decay, int(adamw_mode))

    def advance(self, step, beta1, beta2):
        self._L.oracle_adam_advance(self._buf, step, beta1, beta2)

    def set(self, lr, eps, weight_decay, bias_correction=True):
        self._L.oracle_adam_set(self._buf, lr, eps, weight_decay, int(bias_correction))

    def consts(self, loss_scale=-1.0):
        """(1-beta1, 1-beta2, bc2inv, step_size, wd_term, bc1) as float32."""
        out = np.zeros(6, dtype=np.float32)
        self._L.oracle_adam_consts(self._buf, loss_scale, _ptr(out))
        return out

    def update(
        self,
        step,
        lr,
        beta1,
        beta2,
        eps,
        weight_decay,
        bias_correction,
        params,
        grads,
        exp_avg,
        exp_avg_sq,
        loss_scale=-1.0,
        isa=ISA_AUTO,
    ):
        """``adam_update`` of the reference on flat numpy arrays, in place.

        ``grads`` is float32 or float16 (read only); the others are float32.
        """
        _check(params, np.float32)
        _check(exp_avg, np.float32)
        _check(exp_avg_sq, np.float32)
        assert grads.dtype in (np.float16, np.float32) and grads.flags["C_CONTIGUOUS"]
        n = params.size
        assert grads.size == n and exp_avg.size == n and exp_avg_sq.size == n
        took = self._L.oracle_adam_update(
            self._buf,
            int(step),
            lr,
            beta1,
            beta2,
            eps,
            weight_decay,
            int(bool(bias_correction)),
            _ptr(params),
            _ptr(grads),
            int(grads.dtype == np.float16),
            _ptr(exp_avg),
            _ptr(exp_avg_sq),
            n,
            float(loss_scale),
            isa,
        )
        if took < 0:
            raise RuntimeError(f"oracle code path {isa} is not supported by this CPU")
        return took


def torch_formula_update(params, grads_fp16, exp_avg, exp_avg_sq, step, lr, beta1, beta2, eps, weight_decay,
                         use_adamw, loss_scale=None, gradient_clipping=-1):
    """The reference's torch-formula branch on flat numpy arrays, in place.

    Follows ``fp16_chunk_adam_ops`` / ``torch_adam_update`` statement by statement
    (``patrickstar/ops/fp16_cpu_adam.py``): ``:364-379`` element-wise clamp of the fp16 gradient (GPU
    branch), ``:412-413`` bias corrections in Python arithmetic, ``:430`` ``.float()``, ``:259-277`` the
    update.  ``loss_scale`` is the Python number of the scaler (None: no scaler).  Every scalar is
    computed here with Python floats exactly as the reference's Python does; narrowing to float32 is
    what torch does where a kernel takes a Python scalar.
    """
    _check(params, np.float32)
    _check(exp_avg, np.float32)
    _check(exp_avg_sq, np.float32)
    _check(grads_fp16, np.float16)
    f32 = np.float32
    bias_correction1 = 1 - beta1**step
    bias_correction2 = 1 - beta2**step
    step_size = lr / bias_correction1
    k = np.zeros(10, dtype=np.float32)
    if loss_scale is not None:
        k[0] = f32(1.0 / loss_scale)
    wd_mode = 0
    if weight_decay != 0:
        if use_adamw:
            wd_mode, k[1] = 2, f32(1 - lr * weight_decay)
        else:
            wd_mode, k[1] = 1, f32(weight_decay)
    k[2], k[3] = f32(beta1), f32(1 - beta1)
    k[4], k[5] = f32(beta2), f32(1 - beta2)
    k[6] = f32(1.0 / math.sqrt(bias_correction2))
    k[7] = f32(eps)
    k[8] = f32(-step_size)
    if gradient_clipping > 0:
        bound = gradient_clipping
        if loss_scale is not None:
            bound = bound * loss_scale
        bound = min(65504.0, bound)
        k[9] = f32(np.float16(f32(bound)))
    lib().oracle_torch_adam_span(
        _ptr(k), wd_mode, int(loss_scale is not None), _ptr(params), _ptr(grads_fp16), _ptr(exp_avg),
        _ptr(exp_avg_sq), params.size,
    )


def cast_fp32_to_fp16(src):
    """Whole-array fp32 -> fp16 round-to-nearest-even (the write-back cast)."""
    _check(src, np.float32)
    dst = np.empty(src.shape, dtype=np.float16)
    lib().oracle_cast_f32_to_f16(_ptr(src), _ptr(dst), src.size)
    return dst


def has_inf_or_nan(x):
    """``DynamicLossScaler._has_inf_or_nan``: the float32 sum of ``x`` is +-inf or NaN.

    For fp16 inputs of any realistic length this is "some element is not
    finite" (a finite fp16 sum cannot reach the float32 range), which is the
    form the C helper evaluates; both forms are compared in the tests.
    """
    if x.dtype == np.float16 and x.flags["C_CONTIGUOUS"]:
        return bool(lib().oracle_any_nonfinite_f16(_ptr(x), x.size))
    s = float(np.asarray(x, dtype=np.float32).sum(dtype=np.float32))
    return s == float("inf") or s == -float("inf") or s != s


class StaticScalerOracle:
    """Static scale: never reports overflow, never changes."""

    def __init__(self, scale=1):
        self.cur_scale = scale

    def has_overflow(self, grad):
        return False

    def update_scale(self, overflow):
        return None

    @property
    def loss_scale(self):
        return self.cur_scale


class ScalerOracle:
    """Dynamic loss-scale state machine, restated as one transition function.

    Python number semantics are kept on purpose: ``cur_scale`` stays an ``int``
    until the first true division, and ``max(x / f, min_scale)`` hands back the
    ``min_scale`` object itself when the clamp bites.
    """

    def __init__(
        self,
        init_scale=2**32,
        scale_factor=2.0,
        scale_window=1000,
        min_scale=1,
        delayed_shift=1,
        consecutive_hysteresis=False,
    ):
        self.cur_scale = init_scale
        self.cur_iter = 0
        self.last_overflow_iter = -1
        self.scale_factor = scale_factor
        self.scale_window = scale_window
        self.min_scale = min_scale
        self.delayed_shift = delayed_shift
        self.cur_hysteresis = delayed_shift
        self.consecutive_hysteresis = consecutive_hysteresis

    def has_overflow(self, grad):
        return has_inf_or_nan(grad)

    def update_scale(self, overflow):
        if overflow:
            shrink_now = self.delayed_shift == 1 or self.cur_hysteresis == 1
            if shrink_now:
                self.cur_scale = max(self.cur_scale / self.scale_factor, self.min_scale)
            else:
                self.cur_hysteresis -= 1
            self.last_overflow_iter = self.cur_iter
        else:
            if self.consecutive_hysteresis:
                self.cur_hysteresis = self.delayed_shift
            since = self.cur_iter - self.last_overflow_iter
            if since % self.scale_window == 0:
                if not self.consecutive_hysteresis:
                    self.cur_hysteresis = self.delayed_shift
                self.cur_scale *= self.scale_factor
        self.cur_iter += 1

    @property
    def loss_scale(self):
        return self.cur_scale


def scaler_from_config(fp16_config):
    """Scaler the reference engine builds from ``config["fp16"]`` (None if the block is absent)."""
    if fp16_config is None:
        return None
    assert fp16_config["enabled"], "Must enable fp16 training."
    assert "loss_scale" in fp16_config, "Must have `loss_scale` field set."
    if fp16_config["loss_scale"] == 0:
        return ScalerOracle(
            init_scale=2 ** fp16_config.get("initial_scale_power", 16),
            scale_factor=fp16_config.get("hysteresis", 2),
            scale_window=fp16_config.get("loss_scale_window", 2000),
            min_scale=fp16_config.get("min_loss_scale", 1),
        )
    return StaticScalerOracle(fp16_config["loss_scale"])


class OptimizerStepOracle:
    """``FP16Adam.step`` over a chunk list, one ``adam_update`` per TENSOR as the reference makes them.

    Each chunk is a dict of flat numpy arrays ``p32``, ``m``, ``v`` (float32)
    and ``p16`` (float16; holds the gradients on entry to ``step`` and the
    refreshed fp16 parameters on exit, as in the reference where backward
    overwrites the fp16 parameter slot with the gradient).

    A dict with ``g32`` (float32) in place of ``p16`` stands for parameters
    that PyTorch manages itself (``ParamType.TORCH_BASED``: the fp32 embedding
    weights under ``use_cpu_embedding``): their ``.grad`` is float32 and is
    handed to the operator as it is (``fp16_cpu_adam.py:345-353``; they live
    on the CPU there, so it is always the operator, ``:415-428``), they are not
    probed for overflow (``core/hook.py:202-203``), nothing is restored for
    them on a skipped step (``fp16_cpu_adam.py:301-302``) and no fp16 copy is
    written (``:459-460``).

    ``tensors`` lists the trainable parameters in ``param_groups`` order as
    ``(chunk index, element offset, numel)``; by default every chunk is one
    tensor, in chunk order (what a synthetic chunk list of one flat parameter
    per chunk is).  Parameters that are not listed (``requires_grad=False``)
    are skipped like ``fp16_cpu_adam.py:566-569`` skips them.

    Sequencing restated from ``fp16_cpu_adam.py``: overflow gate first
    (``:549-558``: on overflow restore fp16 from fp32, ``update_scale(True)``,
    leave ``step`` alone), else ``step += 1`` (``:574``), then the loop of
    ``fp16_chunk_adam_ops`` (``:336-468``): for every tensor in turn clamp its
    gradient (``:364-379``), run the operator (``:415-428``) or the torch
    formula (``:430-443``) with the scaler's current scale or -1 (``:227``);
    whole-chunk cast fp32 -> fp16 of every chunk that was visited
    (``chunk_io_buff.py:116-126,143-146``); ``update_scale(False)`` (``:624-625``).

    Every operator call carries the same ``step``, so inside
    ``Adam_Optimizer::IncrementStep`` (``cpu_adam.h:143-162``) only the FIRST
    call of a step can find ``_step + 1 == step`` and multiply the running
    float product; every later call of the step sees ``_step + 1 != step`` and
    evaluates ``pow``.  With two or more tensors the first tensor of step t is
    therefore updated with ``float(pow(beta, t-1)) * beta`` and all others
    with ``float(pow(beta, t))``.  ``AdamOracle.update`` is that call, state
    machine included; nothing about the branch is decided here.
    """

    def __init__(self, chunks, loss_scaler=None, lr=1e-3, betas=(0.9, 0.999), eps=1e-8,
                 weight_decay=0.0, use_adamw=False, isa=ISA_AUTO, gradient_clipping=-1, arithmetic="operator",
                 operator_chunks=(), tensors=None):
        self.chunks = chunks
        self.loss_scaler = loss_scaler
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        self.use_adamw = use_adamw
        self.has_overflow = False
        self.isa = isa
        self.gradient_clipping = gradient_clipping
        # The reference picks per tensor by where its optimizer state lives (:415-443):
        # "operator": every tensor through the native operator (state in host memory);
        # "torch": tensors through torch_adam_update (state in GPU memory), except those of the chunks
        # listed in operator_chunks (indices of chunks whose state is in host memory).
        assert arithmetic in ("operator", "torch")
        self.arithmetic = arithmetic
        self.operator_chunks = set(operator_chunks)
        if tensors is None:
            tensors = [(i, 0, c["p32"].size) for i, c in enumerate(chunks)]
        for ci, off, numel in tensors:
            assert 0 <= ci < len(chunks) and 0 <= off and off + numel <= chunks[ci]["p32"].size, (ci, off, numel)
        self.tensors = list(tensors)
        # state[p] of the reference (fp16_cpu_adam.py:111-131): every parameter carries its OWN step number and
        # its own copy of the hyper-parameters, and step() hands each operator call its tensor's own numbers
        # (:571-606, :406-410).  Keyed by the tensor's span; made on first use with the constructor's values.
        self._default_step = 0
        self._state = {}
        self.native = AdamOracle(lr, betas[0], betas[1], eps, weight_decay, use_adamw)

    def state(self, span):
        """The reference's ``state[p]`` entries of the tensor at ``span = (chunk, offset, numel)``: ``step``, ``lr``,
        ``betas``, ``eps``, ``weight_decay``.  Writable, like the reference's."""
        span = tuple(span)
        if span not in self._state:
            self._state[span] = {"step": self._default_step, "lr": self.lr, "betas": self.betas, "eps": self.eps,
                                 "weight_decay": self.weight_decay}
        return self._state[span]

    @property
    def step_count(self):
        """``state[p]["step"]`` of the first listed tensor (every tensor's, while all of them are stepped together)."""
        return self.state(self.tensors[0])["step"] if self.tensors else self._default_step

    @step_count.setter
    def step_count(self, value):
        self._default_step = value
        for st in self._state.values():
            st["step"] = value

    def check_overflow(self):
        """Sticky OR over every chunk's gradients (``fp16_cpu_adam.py:279-285``)."""
        if self.loss_scaler is None:
            return
        for c in self.chunks:
            if self.has_overflow:
                break
            if "p16" in c and self.loss_scaler.has_overflow(c["p16"]):
                self.has_overflow = True

    def _clamp(self, g):
        # fp16_cpu_adam.py:364-379, GPU branch: clamp_ of the fp16 gradient tensor to
        # +-min(65504, clipping * loss_scale); the Python float bound narrows to float, then to half
        bound = self.gradient_clipping
        if self.loss_scaler is not None:
            bound = bound * self.loss_scaler.loss_scale
        bound = min(65504.0, bound)
        # (a float32 gradient tensor takes the bound as a float: this restatement keeps the bound of the GPU branch
        # for it too, not the CPU branch's, which multiplies its bound tensor by the loss scale in place on every call)
        b = np.float16(np.float32(bound)) if g.dtype == np.float16 else np.float32(bound)
        g[g < -b] = -b
        g[g > b] = b

    def step(self):
        """Returns True when the step was skipped."""
        if self.has_overflow:
            for c in self.chunks:
                if "p16" in c:
                    c["p16"][...] = cast_fp32_to_fp16(c["p32"])
            self.has_overflow = False
            self.loss_scaler.update_scale(True)
            return True
        scaler_scale = self.loss_scaler.loss_scale if self.loss_scaler is not None else None
        if not self.tensors:
            self._default_step += 1
        # :569-606: every trainable parameter's own step advances, then the lists are built
        calls = []
        for span in self.tensors:
            st = self.state(span)
            st["step"] += 1
            calls.append((span, st["step"], st["lr"], st["betas"], st["eps"], st["weight_decay"]))
        visited = []
        for (ci, off, numel), step, lr, (beta1, beta2), eps, weight_decay in calls:
            c = self.chunks[ci]
            torch_managed = "g32" in c
            p, g, m, v = (c[k][off : off + numel] for k in ("p32", "g32" if torch_managed else "p16", "m", "v"))
            if self.gradient_clipping > 0:
                self._clamp(g)
            if self.arithmetic == "torch" and ci not in self.operator_chunks and not torch_managed:
                torch_formula_update(p, g, m, v, step, lr, beta1, beta2, eps, weight_decay, self.use_adamw, scaler_scale)
            else:
                # one adam_update of the native operator: IncrementStep, update_state, Step
                self.native.update(
                    step, lr, beta1, beta2, eps, weight_decay, True,
                    p, g, m, v, float(scaler_scale if scaler_scale is not None else -1), self.isa,
                )
            if ci not in visited and not torch_managed:
                visited.append(ci)
        # the gradients of a chunk have all been read by now: whole-chunk write-back, padding included
        for ci in visited:
            c = self.chunks[ci]
            c["p16"][...] = cast_fp32_to_fp16(c["p32"])
        if self.loss_scaler:
            self.loss_scaler.update_scale(False)
        return False
