"""Host-resident chunk positions: streamed through HBM staging slots by the C ABI.

The reference's hybrid Adam keeps some chunks' optimizer state in host memory and
updates them with the CPU operator (``patrickstar/ops/fp16_cpu_adam.py:415-428``,
``patrickstar/ops/chunk_io_buff.py:214-255``).  On MI355X those chunks are instead
copied into double-buffered HBM staging by ``hipMemcpyAsync`` on side streams,
updated by the same fused kernel as resident chunks, and copied back, all ordered
by events inside ``ps_adam_step_hybrid``; the Python side only owns the
staging buffers.  A position's fp16 payload may stay in HBM (where forward and
backward use it, as in the reference); it is then updated in place and only the
optimizer state (12 B/element each way) crosses the link.
"""
import torch

from . import _lib


class HostChunkStreamer:
    def __init__(self, client, host_positions, n_slots=3, step_indices=None, used=None):
        """``step_indices``: which of ``host_positions`` ``step()`` streams (default: all of them); the gradient probe
        always covers every position.  ``used``: per position, the elements in front of its zero padding (only those
        cross the link); default: whole chunks."""
        self.client = client
        self.n_slots = n_slots
        self.chunk_numel = client.default_chunk_size
        cl = client.chunk_list
        rows = []
        stage_fp16 = False  # does any position keep its fp16 payload in host memory?
        for pos in host_positions:
            payloads = [cl[c].payload for c in (pos.fp32, pos.exp_avg, pos.exp_avg_sq, pos.fp16)]
            for t in payloads[:3]:
                if t.device.type != "cpu" or not t.is_pinned():
                    raise RuntimeError("host-resident optimizer state must be pinned host memory")
            p16 = payloads[3]
            if p16.device.type == "cpu":
                if not p16.is_pinned():
                    raise RuntimeError("a host-resident fp16 payload must be pinned host memory")
                stage_fp16 = True
            rows.append([t.data_ptr() for t in payloads])
        self.host_table = _lib.chunk_array(rows)
        self.n_host = len(rows)
        used = list(used) if used is not None else [self.chunk_numel] * len(rows)
        self.host_used = _lib.size_array(used) if any(u != self.chunk_numel for u in used) else None
        if step_indices is None:
            self.step_table, self.n_step, self.step_used = self.host_table, self.n_host, used
        else:
            picked = [rows[k] for k in step_indices]
            self.step_table, self.n_step = (_lib.chunk_array(picked) if picked else None), len(picked)
            self.step_used = [used[k] for k in step_indices]
        # for a step() that streams these positions and updates no resident chunk beside them
        self.host_used_of_step = _lib.size_array(self.step_used) if any(u != self.chunk_numel for u in self.step_used) else None
        dev = client.device
        n = self.chunk_numel
        # staging lives for the life of the optimizer: allocating it per step (as the reference does with
        # its per-step buffers, fp16_cpu_adam.py:530-547) would serialise against the streams that use it
        self._slots = [
            (
                torch.empty(n, dtype=torch.float, device=dev),
                torch.empty(n, dtype=torch.float, device=dev),
                torch.empty(n, dtype=torch.float, device=dev),
                torch.empty(n if stage_fp16 else 0, dtype=torch.half, device=dev),
            )
            for _ in range(n_slots)
        ]
        self.staging = _lib.chunk_array(
            [[t.data_ptr() if t.numel() else None for t in slot] for slot in self._slots]
        )
        self._lib = _lib.load()

    def step(self, opt_id, step_no, lr, beta1, beta2, eps, weight_decay, loss_scale, resident, n_resident, calls=None,
             scaler=None, used=None):
        """One optimizer step over the resident chunk array AND the host-resident chunks.
        ``calls``: the step's ps_call_pattern over both lists (resident positions counted first).
        ``scaler`` (a device-resident DynamicLossScaler) selects the device-gated form.
        ``used``: size_t array over the resident positions followed by the streamed ones (None: whole chunks)."""
        _lib.check(
            self._lib.ps_adam_step_hybrid(
                opt_id, step_no, lr, beta1, beta2, eps, weight_decay, 1, resident, n_resident, self.step_table,
                self.n_step, self.chunk_numel, used, self.staging, self.n_slots, calls, float(loss_scale),
                scaler.state_ptr if scaler is not None else None, _lib.current_stream_handle(),
            ),
            "ps_adam_step_hybrid",
        )

    def scan_gradients(self, scaler):
        _lib.check(
            self._lib.ps_overflow_scan_host_chunks(
                self.host_table, self.n_host, self.chunk_numel, self.host_used, self.staging, self.n_slots, scaler.state_ptr,
                _lib.current_stream_handle(),
            ),
            "ps_overflow_scan_host_chunks",
        )
