"""FP16Adam: the chunk-wise mixed-precision Adam/AdamW step on MI355X.

Keeps the constructor, attributes and ``step()`` / ``state_dict()`` /
``load_state_dict()`` behaviour of ``patrickstar/ops/fp16_cpu_adam.py:61-694``.
Where the reference walks the chunk lists tensor by tensor (staging each fp16
gradient chunk, calling a CPU operator or ~10 torch kernels per tensor, then
casting each fp32 chunk back to fp16), this implementation hands the whole
chunk list to ONE fused HIP kernel per step through the C ABI in
``include/ps_adam.h``.

With a dynamic loss scaler the step is decided on the device: the overflow flag,
the loss scale and the step counter live in a device struct, a flagged step
restores the fp16 parameters from the fp32 master copy and halves the scale,
and ``step()`` returns without synchronising.  ``state[p]["step"]`` and
``has_overflow`` read that struct back on demand.

The reference has two arithmetics and picks per tensor by where the optimizer
state lives (``fp16_cpu_adam.py:415-443``): the native operator for state in host
memory, ``torch_adam_update`` (a sequence of torch kernels) for state in GPU
memory.  They agree to about 1e-6 on the parameters and the first moment and
to 5e-5 on the second moment (the operator forms ``1 - beta2`` in float).
``arithmetic="operator"``
(default) runs the operator's order of operations on every chunk;
``arithmetic="torch"`` runs the torch formula, with the rounding of torch's GPU
kernels, on chunks resident in HBM and keeps the operator's for host-resident
chunks -- bit for bit what the reference computes under the same placement.
"""
import ctypes
import logging
import weakref
from copy import deepcopy

import torch

from . import _lib, adam_op
from .chunk_layout import AccessType, ChunkType, ParamType, register_param
from .loss_scaler import DynamicLossScaler


logger = logging.getLogger("patrickstar_amd")


def _empty_fp32_param():
    return torch.nn.Parameter(torch.tensor([], dtype=torch.float), requires_grad=False)


class _ParamState(dict):
    """Per-parameter optimizer state whose ``step`` entry may live on the device."""

    def __init__(self, owner):
        super().__init__()
        self._owner = weakref.ref(owner)

    def _sync(self):
        owner = self._owner()
        if owner is not None:
            owner._sync_steps()

    def __getitem__(self, key):
        if key == "step":
            self._sync()
        return super().__getitem__(key)

    def __setitem__(self, key, value):
        if key == "step":
            self._sync()  # settle every parameter's entry before one of them is overwritten
        super().__setitem__(key, value)
        if key in ("lr", "betas", "eps", "weight_decay", "step"):
            owner = self._owner()
            if owner is not None:
                owner._plan = None  # the next step() looks at every parameter's entries again
                if key == "step":
                    owner._steps_written = True  # ... and at how the step numbers relate to one another

    def items(self):
        self._sync()
        return super().items()

    def values(self):
        self._sync()
        return super().values()


class FP16Adam(torch.optim.Optimizer):
    optimizer_id = 0

    def __init__(
        self,
        client,
        params,
        loss_scaler=None,
        gradient_clipping=-1,
        lr=1e-3,
        betas=(0.9, 0.999),
        eps=1e-8,
        weight_decay=0,
        use_adamw=False,
        amsgrad=False,
        use_hybrid_adam=True,
        scan_in_step=True,
        arithmetic="operator",
    ):
        if not 0.0 <= lr:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if not 0.0 <= eps:
            raise ValueError("Invalid epsilon value: {}".format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError("Invalid beta parameter at index 0: {}".format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError("Invalid beta parameter at index 1: {}".format(betas[1]))
        if not 0.0 <= weight_decay:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        if arithmetic not in ("operator", "torch"):
            raise ValueError("Invalid arithmetic: {} (expected 'operator' or 'torch')".format(arithmetic))
        # fail now, not at the first step, if the HIP library was never built
        self._lib = _lib.load()
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad)
        super().__init__(params, defaults)
        self.client = client
        self.loss_scaler = loss_scaler
        self.gradient_clipping = gradient_clipping
        self.use_hybrid_adam = use_hybrid_adam
        self.use_adamw = use_adamw
        # True: step() itself probes every fp16 gradient chunk for inf/nan (one extra 2 B/element
        # pass).  False: the caller has already fed the flag through check_overflow().
        self.scan_in_step = scan_in_step
        self.arithmetic = arithmetic
        self._dynamic = isinstance(loss_scaler, DynamicLossScaler)
        self._host_overflow = False
        self._steps_dirty = False
        # What one step does, derived from requires_grad and the state[p] entries of every parameter (_make_plan);
        # None: look again.  The reference reads all of it per parameter on every step (fp16_cpu_adam.py:569-606).
        self._plan = None
        # The common step counter: every trainable parameter's state[p]["step"] is this number plus the parameter's
        # own distance (0 for all of them in the ordinary case).  Host-decided steps count here; device-decided steps
        # count in the loss scaler's device state (adam_step) and this is what it was seeded with.
        self._common_step = 0
        self._offsets = {}  # parameter -> its distance from the common counter (only parameters that have one)
        self._steps_written = True  # some state[p]["step"] was written since the plan was last made (or none was made yet)
        self._each_static = None  # what the tensor table of a step with per-tensor numbers keeps between plans
        # HBM staging slots for host-resident chunks (one being filled, one computed on, one drained); the client has
        # budgeted that many when it placed the payloads
        self.staging_slots = getattr(client, "staging_slots", 3)

        assert len(self.param_groups) == 1, "Only support one param group at the moment."
        # Eager state initialisation: m and v are chunk tensors shadowing the fp16 parameter chunks.
        for group in self.param_groups:
            for p in group["params"]:
                st = _ParamState(self)
                self.state[p] = st
                dict.__setitem__(st, "betas", group["betas"])
                dict.__setitem__(st, "lr", group["lr"])
                dict.__setitem__(st, "weight_decay", group["weight_decay"])
                dict.__setitem__(st, "eps", group["eps"])
                dict.__setitem__(st, "step", 0)
                if p.ps_attr.param_type == ParamType.TORCH_BASED:
                    # a parameter PyTorch manages itself (fp32 embedding weights under use_cpu_embedding): plain fp32
                    # moments beside it (fp16_cpu_adam.py:122-131)
                    if p.requires_grad:
                        for key in ("exp_avg", "exp_avg_sq"):
                            sp = torch.nn.Parameter(torch.zeros_like(p.data, dtype=torch.float), requires_grad=False)
                            register_param(sp, ParamType.TORCH_BASED, torch.float, f"{p.ps_attr.name}.{key}")
                            dict.__setitem__(st, key, sp)
                    continue
                if not p.ps_attr.is_local():
                    continue
                name = p.ps_attr.name
                for key, ctype in (("exp_avg", ChunkType.MOMENTUM), ("exp_avg_sq", ChunkType.VARIANCE)):
                    sp = _empty_fp32_param()
                    register_param(sp, ParamType.CHUNK_BASED, torch.float, f"{name}.{key}")
                    sp.ps_attr.reset_shape(p.ps_attr.shape)
                    sp.ps_attr._is_local = p.ps_attr.is_local()
                    dict.__setitem__(st, key, sp)
                    # the layout of momentum and variance chunks follows the fp16 parameter chunks
                    self.client.append_tensor_as_ref(sp, torch.float, AccessType.DATA, ctype, p)
        self.client.allocate_payloads()
        if not use_hybrid_adam and self.client.host_fp16_chunk_ids:
            raise ValueError(
                "use_hybrid_adam=False keeps every optimizer state in HBM, but the client placed chunk positions "
                f"{sorted(self.client.host_fp16_chunk_ids)} in host memory"
            )

        self.opt_id = FP16Adam.optimizer_id
        FP16Adam.optimizer_id = FP16Adam.optimizer_id + 1
        self.ds_opt_adam = adam_op  # the operator module, under the attribute name the reference uses
        self.ds_opt_adam.create_adam(self.opt_id, lr, betas[0], betas[1], eps, weight_decay, self.use_adamw, False)
        self._created = True
        if gradient_clipping is not None and gradient_clipping > 0:
            # element-wise clamp of the fp16 gradients to +-min(65504, clipping * loss_scale), fused into the kernels
            _lib.check(self._lib.ps_adam_set_grad_clamp(self.opt_id, float(gradient_clipping)), "ps_adam_set_grad_clamp")
        if arithmetic == "torch":
            _lib.check(self._lib.ps_adam_set_arithmetic(self.opt_id, _lib.PS_ARITH_TORCH), "ps_adam_set_arithmetic")
        self._tables = None
        self._tensor_table = None  # (ps_chunk rows, numels, count) when the step has to go tensor by tensor
        self._calls = None  # ps_call_pattern of one step (None: no operator call at all)
        self._stages = None  # the entry-point calls of a step that cannot be made as one (see _plan_stages)
        self._trainable_seen = None  # requires_grad of every parameter when the plan was made
        self._operator_calls = 0
        if self._dynamic and torch.cuda.is_available():
            self.loss_scaler.materialize(self.client.device, betas=betas)
            self.loss_scaler.enable_log(self.OVERFLOW_LOG_CAPACITY)
            self.loss_scaler.on_read = weakref.WeakMethod(self._warn_about_overflows)

    def __del__(self):
        # the native object is per id and process-global: drop it with the optimizer
        if getattr(self, "_created", False):
            self._created = False
            try:
                self._lib.ps_adam_destroy(self.opt_id)
            except Exception:  # interpreter shutdown: the library handle may already be gone
                pass

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault("amsgrad", False)

    # -- the operator on one tensor ------------------------------------------------
    def ds_cpu_adam_update(self, data, grad, momentum, variance, step, lr, beta1, beta2, eps, weight_decay,
                           bias_correction):
        """One operator call on one tensor, in place on ``data``, ``momentum`` and ``variance``, with the loss scaler's
        current scale (or -1): ``fp16_cpu_adam.py:205-243`` under its own name.  The reference asserts CPU tensors
        here; these are GPU tensors.  ``step()`` does not go through this method (it hands whole chunk lists to the
        library); it is the per-tensor form for callers that drive the operator themselves."""
        for name, t in (("data", data), ("grad", grad), ("momentum", momentum), ("variance", variance)):
            assert t.device.type == "cuda", f"{name} must live on the GPU"
        loss_scale = self.loss_scaler.loss_scale if self.loss_scaler is not None else -1
        self.ds_opt_adam.adam_update(
            self.opt_id, step, lr, beta1, beta2, eps, weight_decay, bias_correction,
            data.view(-1), grad.view(-1), momentum.view(-1), variance.view(-1), loss_scale,
        )

    # -- chunk descriptor tables -------------------------------------------------
    def _trainable(self):
        """The parameters ``step()`` updates, in the order the reference visits them (``fp16_cpu_adam.py:566-605``)."""
        return [p for group in self.param_groups for p in group["params"] if p.requires_grad and p.ps_attr.is_local()]

    @staticmethod
    def _torch_managed(p):
        return p.ps_attr.param_type == ParamType.TORCH_BASED

    def _build_tables(self):
        """Descriptors of what one step covers, and how the reference would have cut it into operator calls.

        Whole-chunk form (the normal case): an array of ps_chunk descriptors for HBM-resident positions and a list of
        host-resident ones.  If some tensor of a chunk is NOT updated (``requires_grad=False``, or not handed to the
        optimizer) the whole-chunk pass does not apply; the step then goes tensor by tensor through
        ``ps_adam_step_tensors`` over the trainable tensors only, as the reference's loop skips the others.
        """
        cl = self.client.chunk_list
        index = self.client.chunk_tensor_index
        trainable = [p for p in self._trainable() if not self._torch_managed(p)]  # the chunk lists' part of the step
        live_ids = {p.ps_attr.data_id() for p in trainable}
        chunk_of = {p: index.get_tensor_info(p.ps_attr.data_id()).chunk_id for p in trainable}
        live_chunks = set(chunk_of.values())
        partly_frozen = any(
            info.tensor_id not in live_ids for cid in live_chunks for info in index.generate_tensor_info_in_order(cid)
        )
        dev_rows, host_positions, where = [], [], {}
        dev_used, host_used = [], []
        for pos in self.client.positions():
            if pos.fp16 not in live_chunks or pos.exp_avg is None or pos.exp_avg_sq is None:
                continue  # a chunk position without trainable parameters
            # elements in front of the chunk's zero padding: where its last tensor ends
            used = max((info.start_offset + info.numel for info in index.generate_tensor_info_in_order(pos.fp16)), default=0)
            if pos.on_host:
                where[pos.fp16] = ("host", len(host_positions))
                host_positions.append(pos)
                host_used.append(used)
            else:
                where[pos.fp16] = ("hbm", len(dev_rows))
                dev_used.append(used)
                dev_rows.append(
                    [
                        cl[pos.fp32].payload.data_ptr(),
                        cl[pos.exp_avg].payload.data_ptr(),
                        cl[pos.exp_avg_sq].payload.data_ptr(),
                        cl[pos.fp16].payload.data_ptr(),
                    ]
                )
        self._tensor_table = None
        if partly_frozen and not host_positions:
            self._tensor_table = self._tensor_rows(trainable)
        # The operator calls of one step: with the operator's arithmetic every trainable tensor is one, with the torch
        # arithmetic only those whose optimizer state lives in host memory (fp16_cpu_adam.py:415-443).
        if self.arithmetic == "torch":
            called = [p for p in trainable if where[chunk_of[p]][0] == "host"]
        else:
            called = trainable
        self._operator_calls = len(called)
        self._calls = None
        if called:
            first = called[0]
            info = index.get_tensor_info(first.ps_attr.data_id())
            kind, k = where[info.chunk_id]
            self._calls = _lib.call_pattern(
                len(called), k if kind == "hbm" else len(dev_rows) + k, info.start_offset, info.numel
            )
        table = _lib.chunk_array(dev_rows) if dev_rows else None
        self._tables = (table, len(dev_rows), host_positions)
        # the padding behind a chunk's last tensor is zeros in all four lists and stays zeros: the kernels skip it
        full = self.client.default_chunk_size
        self._used = _lib.size_array(dev_used) if any(u != full for u in dev_used) else None
        self._used_all = _lib.size_array(dev_used + host_used) if any(u != full for u in dev_used + host_used) else None
        self._stages = None
        if host_positions:
            from .hybrid import HostChunkStreamer

            if partly_frozen:
                self._plan_stages(trainable, chunk_of, where, host_positions, called, live_ids, host_used)
            else:
                self._streamer = HostChunkStreamer(self.client, host_positions, n_slots=self.staging_slots, used=host_used)
        return self._tables

    def _tensor_rows(self, params, slot=None):
        """(ps_chunk rows, numels, count) of a tensor list for ``ps_adam_step_tensors``: the four addresses of every
        parameter's fp32 master, exp_avg, exp_avg_sq and fp16 slot.  ``slot``: (payloads of the parameters' chunk
        position, staging tensors) when the step works on a staged copy of a host-resident position: addresses are then
        taken at the tensors' offsets inside the staging tensors (inside the real fp16 payload if that one lives in HBM)."""
        index = self.client.chunk_tensor_index
        rows, numels = [], []
        for p in params:
            st = self.state[p]
            if self._torch_managed(p):
                # the parameter itself is the fp32 master; the fourth address is its fp32 gradient's, which is a new
                # tensor after every backward: _step_each writes it in before every step
                rows.append([p.data_ptr(), dict.__getitem__(st, "exp_avg").data_ptr(), dict.__getitem__(st, "exp_avg_sq").data_ptr(),
                             p.data_ptr()])
                numels.append(p.numel())
                continue
            quad = (self.client.param_fp16_to_param_fp32_map[p], dict.__getitem__(st, "exp_avg"),
                    dict.__getitem__(st, "exp_avg_sq"), p)
            if slot is None:
                rows.append([self.client.access_data(q).data_ptr() for q in quad])
            else:
                payloads, staging = slot
                row = []
                for k, q in enumerate(quad):
                    base = staging[k] if payloads[k].device.type == "cpu" else payloads[k]
                    row.append(base.data_ptr() + index.get_tensor_info(q.ps_attr.data_id()).start_offset * base.element_size())
                rows.append(row)
            numels.append(p.ps_attr.numel)
        return _lib.chunk_array(rows), (ctypes.c_size_t * len(numels))(*numels), len(numels)

    def _plan_stages(self, trainable, chunk_of, where, host_positions, called, live_ids, host_used):
        """Chunks that mix trainable and frozen tensors TOGETHER WITH host-resident positions: the step is spread over
        several entry-point calls, all under one call pattern (the stage that holds the step's first operator call
        goes first and names it):
          * the trainable tensors of HBM-resident chunks: one tensor-list call;
          * host-resident positions whose tensors are all trainable: streamed as whole chunks;
          * host-resident positions that hold frozen tensors too: copied into a staging slot, their trainable tensors
            updated there by a tensor-list call with the operator's arithmetic, and copied back, on the caller's stream.
        """
        from .hybrid import HostChunkStreamer

        cl, index = self.client.chunk_list, self.client.chunk_tensor_index
        whole, part = [], []
        for k, pos in enumerate(host_positions):
            frozen_here = any(info.tensor_id not in live_ids for info in index.generate_tensor_info_in_order(pos.fp16))
            (part if frozen_here else whole).append(k)
        self._streamer = HostChunkStreamer(self.client, host_positions, n_slots=self.staging_slots, step_indices=whole,
                                           used=host_used)
        n_calls = len(called)
        first = called[0] if called else None
        first_info = index.get_tensor_info(first.ps_attr.data_id()) if first is not None else None

        def pattern():
            """For a stage that does not hold the step's first operator call."""
            return _lib.call_pattern(n_calls, 0, 0, 0) if n_calls else None

        def position_of(params, wanted):
            for i, q in enumerate(params):
                if q is wanted:
                    return i
            return None

        stages = []  # (holds the first call, stage)
        resident = [p for p in trainable if where[chunk_of[p]][0] == "hbm"]
        if resident:
            i = position_of(resident, first)
            pat = pattern() if i is None else _lib.call_pattern(n_calls, i, 0, first.ps_attr.numel)
            stages.append((i is not None, ("tensors", self._tensor_rows(resident), pat)))
        if whole:
            i = None
            if first is not None and where[first_info.chunk_id][0] == "host" and where[first_info.chunk_id][1] in whole:
                i = whole.index(where[first_info.chunk_id][1])
            pat = pattern() if i is None else _lib.call_pattern(n_calls, i, first_info.start_offset, first_info.numel)
            stages.append((i is not None, ("stream", pat)))
        for k in part:
            pos = host_positions[k]
            here = [p for p in trainable if chunk_of[p] == pos.fp16]
            payloads = [cl[c].payload for c in (pos.fp32, pos.exp_avg, pos.exp_avg_sq, pos.fp16)]
            staging = self._streamer._slots[0]
            i = position_of(here, first)
            pat = pattern() if i is None else _lib.call_pattern(n_calls, i, 0, first.ps_attr.numel)
            stages.append((i is not None, ("staged", payloads, staging, self._tensor_rows(here, (payloads, staging)), pat)))
        stages.sort(key=lambda e: not e[0])  # stable: the stage with the first call moves to the front
        self._stages = [stage for _, stage in stages]

    def _run_stages(self, step_no, hyper, loss_scale, scaler, stream):
        """Queue the stages of a step that is spread over several entry-point calls (see ``_plan_stages``).
        ``scaler``: the device-resident scaler of a device-decided step, else None."""
        lr, (beta1, beta2), eps, weight_decay = hyper
        state_ptr = scaler.state_ptr if scaler is not None else None

        def tensors(table, pat):
            rows, numels, n = table
            _lib.check(
                self._lib.ps_adam_step_tensors(
                    self.opt_id, step_no, lr, beta1, beta2, eps, weight_decay, 1, rows, numels, n, pat, float(loss_scale),
                    state_ptr, stream,
                ),
                "ps_adam_step_tensors",
            )

        for stage in self._stages:
            if stage[0] == "tensors":
                tensors(stage[1], stage[2])
            elif stage[0] == "stream":
                self._streamer.step(self.opt_id, step_no, lr, beta1, beta2, eps, weight_decay, loss_scale, None, 0,
                                    stage[1], scaler, self._streamer.host_used_of_step)
            else:
                _, payloads, staging, table, pat = stage
                moved = [(s, h) for s, h in zip(staging, payloads) if h.device.type == "cpu"]
                for s, h in moved:
                    s.copy_(h, non_blocking=True)
                # a host-resident position is updated with the operator's arithmetic whatever the optimizer's own is
                # (the reference runs its CPU operator on it, fp16_cpu_adam.py:415-428)
                if self.arithmetic == "torch":
                    _lib.check(self._lib.ps_adam_set_arithmetic(self.opt_id, _lib.PS_ARITH_OPERATOR), "ps_adam_set_arithmetic")
                try:
                    tensors(table, pat)
                finally:
                    if self.arithmetic == "torch":
                        _lib.check(self._lib.ps_adam_set_arithmetic(self.opt_id, _lib.PS_ARITH_TORCH), "ps_adam_set_arithmetic")
                for s, h in moved:
                    h.copy_(s, non_blocking=True)

    def invalidate_tables(self):
        """Call after re-allocating chunk payloads."""
        self._tables = None
        self._each_static = None
        if self._plan is not None and self._plan["kind"] == "each":
            self._plan["table"] = None

    # -- overflow flag ------------------------------------------------------------
    @property
    def has_overflow(self):
        if self._dynamic:
            return self.loss_scaler.overflow_flag
        return self._host_overflow

    @has_overflow.setter
    def has_overflow(self, value):
        if self._dynamic:
            self.loss_scaler.materialize(self.client.device)
            off = _lib.ps_step_state.overflow.offset
            self.loss_scaler._state[off : off + 4].view(torch.int32).fill_(1 if value else 0)
        else:
            self._host_overflow = bool(value)

    def check_overflow(self, param):
        """OR "param.grad holds an inf/nan" into the sticky flag (no-op for static or absent scalers).
        Asynchronous: nothing is read back."""
        if self._dynamic and param.grad is not None:
            self.loss_scaler.scan(param.grad)

    def has_overflow_and_reset_param(self, write_chunk_buff=None):
        """``fp16_cpu_adam.py:287-310`` under its own name: if the sticky flag is set, rewrite every chunk's fp16
        parameters from the fp32 masters (frozen parameters included, as the reference rewrites every chunk-based
        parameter), clear the flag and return True.  ``step()`` does not come through here (its gate is decided on the
        device); this form reads the flag back, i.e. it synchronises.  ``write_chunk_buff`` is accepted and ignored."""
        if not self.has_overflow:
            return False
        cl = self.client.chunk_list
        rows = [
            [cl[pos.fp32].payload.data_ptr(), 16, 16, cl[pos.fp16].payload.data_ptr()]  # m and v are not touched
            for pos in self.client.positions()
            if pos.fp32 is not None and cl[pos.fp32].payload is not None
        ]
        if rows:
            with torch.cuda.device(self.client.device):
                # pinned host payloads of host-resident positions are device-accessible: the kernel reads / writes them in place
                _lib.check(
                    self._lib.ps_restore_fp16_chunks(
                        _lib.chunk_array(rows), len(rows), self.client.default_chunk_size, None, _lib.current_stream_handle()
                    ),
                    "ps_restore_fp16_chunks",
                )
        self.has_overflow = False
        return True

    def check_overflow_chunks(self):
        """Probe the fp16 gradient payload of every chunk (asynchronous)."""
        if not self._dynamic:
            return
        table, n_dev, host_positions = self._tables or self._build_tables()
        stream = _lib.current_stream_handle()
        if n_dev:
            _lib.check(
                self._lib.ps_overflow_scan_chunks(
                    table, n_dev, self.client.default_chunk_size, self._used, self.loss_scaler.state_ptr, stream
                ),
                "ps_overflow_scan_chunks",
            )
        if host_positions:
            self._streamer.scan_gradients(self.loss_scaler)

    # -- the step -----------------------------------------------------------------
    def _entries(self, p):
        """(lr, betas, eps, weight_decay, step) of one parameter as its ``state[p]`` holds them."""
        g, st = dict.__getitem__, self.state[p]
        return g(st, "lr"), tuple(g(st, "betas")), g(st, "eps"), g(st, "weight_decay"), g(st, "step")

    def _hyper(self):
        """(lr, betas, eps, weight_decay) of the step when every trainable parameter's ``state[p]`` holds the same
        (None when nothing is trainable, ``"each"`` when they differ)."""
        plan = self._plan or self._make_plan()
        return plan["hyper"] if plan["kind"] == "uniform" else (None if plan["kind"] == "empty" else "each")

    def _make_plan(self):
        """What one step does, from ``requires_grad`` and the ``state[p]`` entries of every parameter.

        The reference counts ``state[p]["step"]`` per parameter and reads lr / betas / eps / weight_decay per
        parameter, on every step (``fp16_cpu_adam.py:569-606``), and hands each operator call its tensor's own
        numbers (``:403-428``); ``param_groups[0]["lr"]`` is copied into ``state[p]`` once, by the constructor
        (``:111-116``), and not looked at again, here as there.  Ordinarily all trainable parameters agree: then ONE
        counter (on the host, or in the device-resident state of a dynamic loss scaler) stands for all of them and
        the whole chunk list goes to one fused call ("uniform").  If they do not (a parameter that was frozen for some
        steps stands behind; somebody wrote ``state[p]["lr"]`` for some parameters; a checkpoint said so) the step goes
        tensor by tensor through ``ps_adam_step_tensors_each``, every tensor with its own numbers ("each"): its step
        number is kept as a distance from the common counter, which is all a device-decided step needs to know on
        the host.  Made again whenever ``requires_grad`` of some parameter or a ``state[p]`` entry has changed.

        How the step numbers relate to one another changes only when the set of trainable parameters changes or a
        ``state[p]["step"]`` is written; only then is the device's counter read back.  Writing hyper-parameters (a
        learning-rate schedule writes ``state[p]["lr"]`` of every parameter before every step) keeps the distances
        and waits for nothing.
        """
        params = self.param_groups[0]["params"]
        flags = tuple(p.requires_grad for p in params)
        resettle = self._steps_written or flags != self._trainable_seen
        if resettle:
            self._sync_steps()  # every state[p]["step"] is now what the steps so far made it
            self._tables = None
            self._each_static = None
        self._trainable_seen = flags
        self._steps_written = False
        trainable = self._trainable()
        if not trainable:
            self._offsets = {}
            self._plan = {"kind": "empty"}
            return self._plan
        common = self._common_step
        if resettle:
            # the common counter moves to the first trainable parameter's step number (a checkpoint was loaded, or
            # the parameters that defined it were frozen)
            steps = [dict.__getitem__(self.state[p], "step") for p in trainable]
            common = steps[0]
            self._offsets = {p: t - common for p, t in zip(trainable, steps) if t != common}
        entries = [self._entries(p)[:4] + (self._offsets.get(p, 0),) for p in trainable]
        # parameters that PyTorch manages itself (fp32, with fp32 gradients) are tensors of their own kind: with them
        # the step always goes tensor by tensor
        if all(e == entries[0] for e in entries) and not any(self._torch_managed(p) for p in trainable):
            self._plan = {"kind": "uniform", "hyper": entries[0][:4]}
        else:
            self._plan = {"kind": "each", "trainable": trainable, "entries": entries, "table": None}
        # a device-decided step keeps the counter and the betas of the whole-list kernels on the device
        betas = entries[0][1]
        if self._dynamic and self.loss_scaler._state is not None:
            new_betas = (float(betas[0]), float(betas[1])) != self.loss_scaler._betas
            if new_betas and not resettle:
                self._sync_steps()  # seeding needs the counter as it stands
                common = self._common_step
            if new_betas or common != self._common_step:
                # the operator object behind this optimizer stays the one it was (the reference's load_state_dict,
                # fp16_cpu_adam.py:660-694, does not touch it): whether its running beta^t product continues is
                # decided on the device, as Adam_Optimizer::IncrementStep would (cpu_adam.h:143-162)
                self.loss_scaler._seed_step(common, fresh_operator=False, betas=betas)
        self._common_step = common
        return self._plan

    def _stepped_params(self):
        """The parameters the steps so far have updated: those that were trainable when the plan was last made
        (before the first step: those that are trainable now)."""
        params = self.param_groups[0]["params"]
        flags = self._trainable_seen if self._trainable_seen is not None else [p.requires_grad for p in params]
        return [p for p, on in zip(params, flags) if on]

    def _sync_steps(self):
        """Write the step counter (device-resident or host-side) into state[p]["step"] of every parameter that
        the steps so far have updated: the common count plus the parameter's own distance from it."""
        if not self._steps_dirty:
            return
        self._steps_dirty = False
        if self._dynamic:
            self._common_step = self.loss_scaler.adam_step
        for p in self._stepped_params():
            dict.__setitem__(self.state[p], "step", self._common_step + self._offsets.get(p, 0))

    def _each_table(self, plan):
        """Tensor rows and per-tensor call records of a step whose tensors carry their own numbers."""
        if plan["table"] is None:
            trainable = plan["trainable"]
            if self._each_static is None:
                # addresses, lengths, where the state lives and the workspace stay as they are while the same
                # parameters are trainable (a learning-rate schedule makes a new plan before every step)
                rows, numels, n = self._tensor_rows(trainable)
                on_host = {pos.fp16 for pos in self.client.positions() if pos.on_host}
                index = self.client.chunk_tensor_index
                host = [not self._torch_managed(p) and index.get_tensor_info(p.ps_attr.data_id()).chunk_id in on_host
                        for p in trainable]
                workspace = None
                if self._dynamic:
                    nbytes = self._lib.ps_tensors_each_workspace_bytes(n)
                    workspace = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=self.client.device)
                self._each_static = (rows, numels, n, host, workspace)
            rows, numels, n, host, workspace = self._each_static
            each = (_lib.ps_tensor_call * n)()
            operator_calls = 0
            offsets = [e[4] for e in plan["entries"]]
            managed = []  # (row, parameter) of the tensors PyTorch manages itself
            for i, (lr, (beta1, beta2), eps, weight_decay, d) in enumerate(plan["entries"]):
                e = each[i]
                e.lr, e.beta1, e.beta2, e.eps, e.weight_decay = lr, beta1, beta2, eps, weight_decay
                # optimizer state in host memory is updated by the operator whatever the optimizer's arithmetic
                # (fp16_cpu_adam.py:415-443); the kernel reads and writes such pinned payloads over the link.  The
                # reference keeps the parameters PyTorch manages itself on the CPU, so theirs is the operator's too.
                own = self._torch_managed(trainable[i])
                e.arithmetic = _lib.PS_ARITH_OPERATOR if (host[i] or own or self.arithmetic == "operator") else _lib.PS_ARITH_TORCH
                operator_calls += e.arithmetic == _lib.PS_ARITH_OPERATOR
                if own:
                    e.flags = _lib.PS_TENSOR_GRAD_F32
                    managed.append((i, trainable[i]))
                if self._dynamic:
                    e.step = d  # a device-decided step is told every tensor's distance from the device's counter
            plan["table"] = (rows, numels, n, each, workspace, operator_calls, offsets, managed)
        return plan["table"]

    def _step_each(self, plan, stream):
        """One step through ``ps_adam_step_tensors_each``."""
        rows, numels, n, each, workspace, operator_calls, offsets, managed = self._each_table(plan)
        for i, p in managed:
            # fp16_cpu_adam.py:345-353: the gradient PyTorch left on the parameter, fp32, read where it is
            g = p.grad
            if g is None or g.dtype != torch.float or not g.is_contiguous() or g.device != p.device:
                raise RuntimeError(
                    f"{p.ps_attr.name}: a parameter that PyTorch manages itself needs a contiguous fp32 .grad on "
                    f"{p.device} when step() runs (got {None if g is None else (g.dtype, g.device, g.is_contiguous())})"
                )
            rows[i].param_fp16 = g.data_ptr()
        if self._dynamic:
            scaler = self.loss_scaler
            _lib.check(
                self._lib.ps_adam_step_tensors_each(
                    self.opt_id, 1, rows, numels, each, n, -1.0, scaler.state_ptr, workspace.data_ptr(),
                    workspace.numel(), stream,
                ),
                "ps_adam_step_tensors_each",
            )
            scaler.update_scale(None, operator_calls=operator_calls)
            return
        self._common_step += 1
        for i, d in enumerate(offsets):
            each[i].step = self._common_step + d
        loss_scale = self.loss_scaler.loss_scale if self.loss_scaler is not None else -1
        _lib.check(
            self._lib.ps_adam_step_tensors_each(self.opt_id, 1, rows, numels, each, n, float(loss_scale), None, None, 0, stream),
            "ps_adam_step_tensors_each",
        )
        if self.loss_scaler:
            self.loss_scaler.update_scale(False)

    @torch.no_grad()
    def step(self, closure=None):
        """One optimizer step over the whole chunk list.  Returns the closure's loss (or None)."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        # which parameters are trainable is looked at every step, as the reference does (fp16_cpu_adam.py:569-571):
        # freezing or unfreezing a parameter between steps makes a new plan (descriptor tables, call pattern, and
        # whether every tensor can still share one step number)
        if self._plan is None or tuple(p.requires_grad for p in self.param_groups[0]["params"]) != self._trainable_seen:
            self._make_plan()
        plan = self._plan
        if plan["kind"] == "empty":
            # nothing is trainable: the reference still runs its scale update (fp16_cpu_adam.py:549-558,624-625)
            if self._dynamic:
                self.loss_scaler.update_scale(None, operator_calls=0)
            return loss
        with torch.cuda.device(self.client.device):
            stream = _lib.current_stream_handle()
            if plan["kind"] == "each":
                if self._dynamic and self.scan_in_step:
                    self.check_overflow_chunks()
                self._step_each(plan, stream)
                self._steps_dirty = True
                return loss
            hyper = plan["hyper"]
            lr, (beta1, beta2), eps, weight_decay = hyper
            table, n_dev, host_positions = self._tables or self._build_tables()
            chunk_numel = self.client.default_chunk_size
            if self._dynamic:
                scaler = self.loss_scaler
                if self.scan_in_step:
                    self.check_overflow_chunks()
                if self._stages is not None:
                    self._run_stages(0, hyper, -1.0, scaler, stream)
                elif self._tensor_table is not None:
                    rows, numels, n_tensors = self._tensor_table
                    _lib.check(
                        self._lib.ps_adam_step_tensors(
                            self.opt_id, 0, lr, beta1, beta2, eps, weight_decay, 1, rows, numels, n_tensors, None, -1.0,
                            scaler.state_ptr, stream,
                        ),
                        "ps_adam_step_tensors",
                    )
                elif host_positions:
                    self._streamer.step(self.opt_id, 0, lr, beta1, beta2, eps, weight_decay, -1.0, table, n_dev,
                                        self._calls, scaler, self._used_all)
                elif n_dev:
                    _lib.check(
                        self._lib.ps_adam_step_chunks_gated(
                            self.opt_id, lr, eps, weight_decay, 1, table, n_dev, chunk_numel, self._used, self._calls,
                            scaler.state_ptr, stream,
                        ),
                        "ps_adam_step_chunks_gated",
                    )
                # consume the device flag; a clean step advances state["step"] and takes the operator object
                # through this step's calls
                scaler.update_scale(None, operator_calls=self._operator_calls)
                self._steps_dirty = True
                return loss

            # Static or absent scaler: the host knows every scalar (the static scaler never reports overflow).
            # every parameter's "step" advances together: one host counter, written back to the per-parameter
            # entries only when somebody reads them
            self._common_step += 1
            self._steps_dirty = True
            step_no = self._common_step
            loss_scale = self.loss_scaler.loss_scale if self.loss_scaler is not None else -1
            if self._stages is not None:
                self._run_stages(step_no, hyper, loss_scale, None, stream)
            elif self._tensor_table is not None:
                rows, numels, n_tensors = self._tensor_table
                _lib.check(
                    self._lib.ps_adam_step_tensors(
                        self.opt_id, step_no, lr, beta1, beta2, eps, weight_decay, 1, rows, numels, n_tensors, None,
                        float(loss_scale), None, stream,
                    ),
                    "ps_adam_step_tensors",
                )
            elif host_positions:
                self._streamer.step(self.opt_id, step_no, lr, beta1, beta2, eps, weight_decay, loss_scale, table, n_dev,
                                    self._calls, None, self._used_all)
            elif n_dev:
                _lib.check(
                    self._lib.ps_adam_step_chunks(
                        self.opt_id, step_no, lr, beta1, beta2, eps, weight_decay, 1, table, n_dev,
                        chunk_numel, self._used, self._calls, float(loss_scale), stream,
                    ),
                    "ps_adam_step_chunks",
                )
            if self.loss_scaler:
                self.loss_scaler.update_scale(False)
        return loss

    # -- the reference's overflow warning ----------------------------------------------
    OVERFLOW_LOG_CAPACITY = 1024

    def _warn_about_overflows(self, records, lost):
        """``fp16_cpu_adam.py:551-556`` logs every skipped step as it happens.  Here a step is skipped on the device
        and the host does not wait to learn of it; the loss scaler's device log keeps (flag, scale after) of every
        iteration, and the lines are written when the scaler's state is next read back (``loss_scale``,
        ``has_overflow``, ``state[p]["step"]``, ``state_dict()``), one per skipped step, with the reference's text."""
        if lost:
            logger.warning(
                f"Gradient overflow! {lost} loss-scale updates were not read back in time to be reported one by one "
                f"(the device log holds {self.OVERFLOW_LOG_CAPACITY})."
            )
        for _, overflow, before, after in records:
            if overflow:
                logger.warning(f"Gradient overflow! Update loss scale from {before} to {after}.")

    # -- checkpointing --------------------------------------------------------------
    def state_dict(self):
        """``{"state": ..., "param_groups": ...}`` with chunk-backed m and v cloned to CPU tensors.
        A ``"loss_scaler"`` entry is added (the reference loses its scaler state on resume)."""
        self._sync_steps()
        raw = super().state_dict()
        assert len(raw["param_groups"]) == 1
        packed = {}
        for idx, entries in raw["state"].items():
            packed[idx] = {}
            for k, v in dict.items(entries):
                if isinstance(v, torch.nn.Parameter):
                    packed[idx][k] = self.client.access_data(v).detach().to("cpu", copy=True)
                else:
                    packed[idx][k] = v
        out = {"state": packed, "param_groups": raw["param_groups"]}
        if self.loss_scaler is not None and hasattr(self.loss_scaler, "state_dict"):
            out["loss_scaler"] = self.loss_scaler.state_dict()
        return out

    def load_state_dict(self, state_dict):
        """``fp16_cpu_adam.py:660-694``: every parameter gets its saved ``step``, hyper-parameters and moments back.
        The next ``step()`` derives the common counter from the parameters that are trainable then (a frozen
        parameter's own count plays no part) and hands loaded betas to the device-resident state."""
        state_dict = deepcopy(state_dict)
        saved_groups = state_dict["param_groups"]
        saved_state = state_dict["state"]
        assert len(saved_groups) == 1
        assert len(saved_groups[0]["params"]) == len(self.param_groups[0]["params"])
        assert len(saved_state) == len(self.state)
        self._sync_steps()
        for old_id, p in zip(saved_groups[0]["params"], self.param_groups[0]["params"]):
            saved = saved_state[old_id]
            mine = self.state[p]
            assert len(saved) == len(mine)
            for k, v in list(dict.items(mine)):
                if isinstance(v, torch.nn.Parameter):
                    self.client.access_data(v).copy_(saved[k])
                else:
                    dict.__setitem__(mine, k, saved[k])
        self._plan = None
        self._steps_written = True
        if self._dynamic:
            self.loss_scaler.materialize(self.client.device)
            if "loss_scaler" in state_dict:
                self.loss_scaler.load_state_dict(state_dict["loss_scaler"])
