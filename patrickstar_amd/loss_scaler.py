"""Loss scalers with the reference's interface, the dynamic one resident on the GPU.

``LossScaler`` (static) and ``DynamicLossScaler`` keep the constructor
arguments, methods and semantics of ``patrickstar/fp16/loss_scaler.py:46-190``.
The dynamic scaler's state (current scale, iteration, last overflow iteration,
hysteresis credit) lives in a 256-byte device struct (``ps_step_state``) that the
HIP kernels read and update, so the optimizer step never has to ask the host
whether gradients overflowed.  Reading a field from Python
(``loss_scale``, ``cur_iter``, ...) copies the struct back, which is the only
synchronisation point.
"""
import ctypes
import weakref

import torch

from . import _lib


class LossScaler:
    """Static loss scale: never reports overflow, never changes
    (``patrickstar/fp16/loss_scaler.py:46-76``)."""

    def __init__(self, scale=1):
        self.cur_scale = scale

    def has_overflow(self, param):
        return False

    def _has_inf_or_nan(x):
        return False

    def update_scale(self, overflow):
        pass

    @property
    def loss_scale(self):
        return self.cur_scale

    def backward(self, loss, retain_graph=False):
        scaled_loss = loss * self.loss_scale
        scaled_loss.backward(retain_graph=retain_graph)


def _is_int(x):
    return isinstance(x, int) and not isinstance(x, bool)


class DynamicLossScaler:
    """Dynamic loss scale (``patrickstar/fp16/loss_scaler.py:79-190``), device resident.

    Number semantics follow Python's, as in the reference: ``loss_scale`` is an
    ``int`` until the first halving (a true division) and the ``min_scale``
    object's own type when the clamp bites.  The device keeps the scale as a
    binary64: an ``int`` argument that a binary64 cannot hold exactly (beyond
    2**53 only powers of two times a 53-bit integer can) is refused here
    instead of being rounded silently; an ``int`` scale that GROWS past 2**53
    by a factor that is not a power of two is rounded like a float from there on.
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
        self._init = dict(
            init_scale=init_scale,
            scale_factor=scale_factor,
            scale_window=scale_window,
            min_scale=min_scale,
            delayed_shift=delayed_shift,
            consecutive_hysteresis=consecutive_hysteresis,
        )
        for name, x in (("init_scale", init_scale), ("scale_factor", scale_factor), ("min_scale", min_scale)):
            if _is_int(x):
                try:
                    exact = int(float(x)) == x
                except OverflowError:
                    exact = False
                if not exact:
                    raise ValueError(f"{name} = {x} is an int that a binary64 cannot hold exactly; pass a representable value")
        self.scale_factor = scale_factor
        self.scale_window = scale_window
        self.min_scale = min_scale
        self.delayed_shift = delayed_shift
        self.consecutive_hysteresis = consecutive_hysteresis
        self._state = None  # device tensor holding one ps_step_state
        self._log = None  # optional device tensor of ps_scale_record
        self._log_capacity = 0
        self._log_start = 0  # the iteration the ring has been recording from
        self._log_seen = 0  # iterations below this one have been handed to on_read
        self._scale_seen = init_scale  # loss scale after iteration _log_seen - 1
        # Called with (records, lost) whenever a field is read back from the device and update_scale calls have
        # completed since the last time: records = [(iteration, overflow, scale before, scale after)], lost = how
        # many iterations fell out of the ring unseen.  A callable, or a weak reference to one.  Needs enable_log.
        self.on_read = None
        self._betas = (0.9, 0.999)

    # -- device state ---------------------------------------------------------
    def materialize(self, device=None, betas=None):
        """Create the device-resident state (idempotent).  ``betas`` seeds the Adam beta^t products."""
        if betas is not None:
            self._betas = (float(betas[0]), float(betas[1]))
        if self._state is not None:
            if betas is not None:
                self._seed_step(self.adam_step)
            return self
        if not torch.cuda.is_available():
            raise RuntimeError("DynamicLossScaler keeps its state on the GPU; no GPU is available")
        lib = _lib.load()
        device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        self._state = torch.zeros(ctypes.sizeof(_lib.ps_step_state), dtype=torch.uint8, device=device)
        i = self._init
        if not i["scale_window"] > 0:
            raise ValueError(f"scale_window must be positive, got {i['scale_window']}")
        with torch.cuda.device(device):
            _lib.check(
                lib.ps_state_init(
                    self._state.data_ptr(),
                    float(i["init_scale"]),
                    int(_is_int(i["init_scale"])),
                    float(i["scale_factor"]),
                    int(_is_int(i["scale_factor"])),
                    int(i["scale_window"]),
                    float(i["min_scale"]),
                    int(_is_int(i["min_scale"])),
                    int(i["delayed_shift"]),
                    int(bool(i["consecutive_hysteresis"])),
                    self._betas[0],
                    self._betas[1],
                    _lib.current_stream_handle(),
                ),
                "ps_state_init",
            )
        return self

    def _seed_step(self, adam_step, fresh_operator=True, betas=None):
        """Set the Adam step counter and, if given, the betas of the steps to come.  ``fresh_operator``: a newly
        created operator object stands behind it (a new optimizer); False keeps the running one, as the reference's
        ``load_state_dict`` does: its first call then continues the running beta^t product only if the object stands
        at ``adam_step`` with the same betas (``cpu_adam.h:143-162``)."""
        if betas is not None:
            self._betas = (float(betas[0]), float(betas[1]))
        with torch.cuda.device(self._state.device):
            _lib.check(
                _lib.load().ps_state_seed_step(
                    self._state.data_ptr(), int(adam_step), self._betas[0], self._betas[1], int(bool(fresh_operator)),
                    _lib.current_stream_handle(),
                ),
                "ps_state_seed_step",
            )

    def enable_log(self, capacity):
        """Record (overflow flag, scale after) of every ``update_scale`` in a device ring of ``capacity`` entries,
        from the present iteration on."""
        fresh = self._state is None
        self.materialize()
        if not fresh:
            s = self._read()  # settle what the old ring (if any) still holds
            self._log_start = self._log_seen = int(s.cur_iter)
            self._scale_seen = int(s.cur_scale) if s.scale_is_int else float(s.cur_scale)
        self._log = torch.zeros(capacity * ctypes.sizeof(_lib.ps_scale_record), dtype=torch.uint8, device=self._state.device)
        self._log_capacity = capacity

    def _records(self, first, last):
        """Ring entries of iterations [first, last) as (overflow, typed scale after); the ring must still hold them."""
        raw = self._log.cpu().numpy().tobytes()
        recs = (_lib.ps_scale_record * self._log_capacity).from_buffer_copy(raw)
        out = []
        for it in range(first, last):
            r = recs[it % self._log_capacity]
            out.append((bool(r.overflow), int(r.scale_after) if r.scale_is_int else float(r.scale_after)))
        return out

    def read_log(self):
        """[(overflow: bool, loss_scale)] for the iterations the ring still holds (synchronises)."""
        cur = int(self._read(notify=False).cur_iter)
        return self._records(max(self._log_start, cur - self._log_capacity), cur)

    def _read(self, notify=True):
        host = _lib.ps_step_state()
        with torch.cuda.device(self._state.device):
            _lib.check(
                _lib.load().ps_state_read(self._state.data_ptr(), ctypes.byref(host), _lib.current_stream_handle()),
                "ps_state_read",
            )
        if notify and self._log is not None and self.on_read is not None and host.cur_iter > self._log_seen:
            self._notify(int(host.cur_iter))
        return host

    def _notify(self, cur_iter):
        """Hand the outcomes of the iterations completed since the last read-back to ``on_read``."""
        hook = self.on_read
        if isinstance(hook, weakref.ReferenceType):
            hook = hook()
        first = max(self._log_seen, self._log_start, cur_iter - self._log_capacity)
        lost = first - max(self._log_seen, self._log_start)
        got = self._records(first, cur_iter)
        records, before = [], self._scale_seen
        for k, (overflow, after) in enumerate(got):
            # (the scale in front of an iteration that fell out of the ring is not known)
            records.append((first + k, overflow, None if (lost and k == 0) else before, after))
            before = after
        self._log_seen = cur_iter
        if got:
            self._scale_seen = got[-1][1]
        if hook is not None and (records or lost):
            hook(records, lost)

    @property
    def state_ptr(self):
        self.materialize()
        return self._state.data_ptr()

    # -- reference attributes (read back lazily) --------------------------------
    @property
    def cur_scale(self):
        if self._state is None:
            return self._init["init_scale"]
        s = self._read()
        return int(s.cur_scale) if s.scale_is_int else float(s.cur_scale)

    @property
    def cur_iter(self):
        return 0 if self._state is None else int(self._read().cur_iter)

    @property
    def last_overflow_iter(self):
        return -1 if self._state is None else int(self._read().last_overflow_iter)

    @property
    def cur_hysteresis(self):
        return self.delayed_shift if self._state is None else int(self._read().cur_hysteresis)

    @property
    def adam_step(self):
        return 0 if self._state is None else int(self._read().adam_step)

    @property
    def skipped_steps(self):
        return 0 if self._state is None else int(self._read().skipped_steps)

    @property
    def overflow_flag(self):
        """The sticky device flag of the step being assembled (synchronises)."""
        return False if self._state is None else bool(self._read().overflow)

    @property
    def last_step_skipped(self):
        return False if self._state is None else bool(self._read().last_skipped)

    @property
    def loss_scale(self):
        return self.cur_scale

    # -- overflow probe -----------------------------------------------------------
    def scan(self, x):
        """OR "x holds an inf or nan" into the device flag; asynchronous."""
        self.materialize(x.device)
        if x.numel() == 0:
            return
        if not x.is_contiguous():
            x = x.contiguous()
        lib = _lib.load()
        with torch.cuda.device(x.device):
            if x.dtype == torch.half:
                rc = lib.ps_overflow_scan(x.data_ptr(), x.numel(), self._state.data_ptr(), _lib.current_stream_handle())
            elif x.dtype == torch.float:
                rc = lib.ps_overflow_scan_f32(x.data_ptr(), x.numel(), self._state.data_ptr(), _lib.current_stream_handle())
            else:
                raise TypeError(f"overflow probe supports fp16 and fp32 gradients, got {x.dtype}")
        _lib.check(rc, "ps_overflow_scan")

    def has_overflow(self, param):
        """True if ``param.grad`` holds an inf or nan (synchronises, like the reference's ``float(sum)``).
        The sticky flag of the optimizer is left as it was."""
        return DynamicLossScaler._has_inf_or_nan(param.grad)

    _probes = {}  # device -> a scaler kept only for its flag word (one small device state per GPU, made once)

    @staticmethod
    def _has_inf_or_nan(x):
        if not x.is_cuda:
            raise RuntimeError("the overflow probe runs on the GPU; got a tensor on " + str(x.device))
        probe = DynamicLossScaler._probes.get(x.device)
        if probe is None:
            probe = DynamicLossScaler._probes[x.device] = DynamicLossScaler(init_scale=1).materialize(x.device)
        off = _lib.ps_step_state.overflow.offset
        probe._state[off : off + 4].zero_()
        probe.scan(x)
        return probe.overflow_flag

    # -- state machine ----------------------------------------------------------------
    def update_scale(self, overflow, operator_calls=1):
        """``overflow`` is a bool, or None to consume the sticky device flag; asynchronous.
        ``operator_calls``: how many tensors the optimizer step behind this call handed to the native operator in the
        reference's terms; a clean step takes the operator's step / beta^t state through that many calls."""
        self.materialize()
        mode = _lib.PS_FLAG_FROM_DEVICE if overflow is None else (_lib.PS_FLAG_TRUE if overflow else _lib.PS_FLAG_FALSE)
        log_ptr = self._log.data_ptr() if self._log is not None else None
        with torch.cuda.device(self._state.device):
            _lib.check(
                _lib.load().ps_scaler_update(
                    self._state.data_ptr(), mode, log_ptr, self._log_capacity, int(operator_calls),
                    _lib.current_stream_handle()
                ),
                "ps_scaler_update",
            )

    @property
    def scale_tensor(self):
        """The current loss scale as a 0-dim float64 tensor that ALIASES the device-resident state: it always holds
        what the latest queued ``update_scale`` leaves there, and reading it on the device needs no host round trip."""
        self.materialize()
        off = _lib.ps_step_state.cur_scale.offset
        return self._state[off : off + 8].view(torch.float64).reshape(())

    def backward(self, loss, retain_graph=False):
        """``(loss * loss_scale).backward()`` (``patrickstar/fp16/loss_scaler.py:188-190``) with the scale taken from
        the device: the host does not wait for the previous optimizer step to learn it.  The product is formed as
        torch forms ``tensor * python_number``: in float for half and float losses, the scale narrowed to float."""
        scale = self.scale_tensor
        if loss.dtype == torch.float64:
            scaled_loss = loss * scale
        else:
            scaled_loss = (loss.float() * scale.float()).to(loss.dtype)
        scaled_loss.backward(retain_graph=retain_graph)

    # -- checkpointing (the reference does not save its scaler; this is an addition) ----
    def state_dict(self):
        if self._state is None:
            return {"cur_scale": self._init["init_scale"], "cur_iter": 0, "last_overflow_iter": -1,
                    "cur_hysteresis": self.delayed_shift}
        s = self._read()
        return {
            "cur_scale": int(s.cur_scale) if s.scale_is_int else float(s.cur_scale),
            "cur_iter": int(s.cur_iter),
            "last_overflow_iter": int(s.last_overflow_iter),
            "cur_hysteresis": int(s.cur_hysteresis),
        }

    def load_state_dict(self, sd):
        self.materialize()
        if self._log is not None:
            self._read()  # outcomes recorded so far belong to the run that is being replaced: hand them on now
            self._log_start = self._log_seen = int(sd["cur_iter"])
            self._scale_seen = sd["cur_scale"]
        with torch.cuda.device(self._state.device):
            _lib.check(
                _lib.load().ps_state_set_scaler(
                    self._state.data_ptr(), float(sd["cur_scale"]), int(_is_int(sd["cur_scale"])), int(sd["cur_iter"]),
                    int(sd["last_overflow_iter"]), int(sd["cur_hysteresis"]), _lib.current_stream_handle(),
                ),
                "ps_state_set_scaler",
            )
