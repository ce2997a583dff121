"""Chunk client for one GPU: builds the four chunk lists and hands out views.

MI355X has 288 GB of HBM, so by default every chunk is resident in HBM and a
tensor "access" is just a view into its chunk payload: there is nothing to
move, evict or fetch.  Chunks may instead be placed in pinned host memory
(``host_chunk_policy``) to be streamed through HBM staging buffers by the
optimizer step.

Reference for the rules: ``patrickstar/core/client.py:187-309`` (append_chunk,
append_tensor, append_tensor_as_ref), ``patrickstar/core/preprocess.py:341-435``
(per-module registration of fp16 params and their fp32 shadows, in module
construction order) and ``:289-320`` (initial values copied into both payloads).
"""
from typing import Callable, Dict, List, Optional

import torch

from .chunk_layout import (
    AccessType,
    ChunkList,
    ChunkTensorIndex,
    ChunkType,
    ParamType,
    is_param_registered,
    register_param,
)

class ChunkPosition:
    """The four chunks that sit at the same place of the four lists."""

    __slots__ = ("fp16", "fp32", "exp_avg", "exp_avg_sq", "on_host")

    def __init__(self, fp16, fp32, exp_avg, exp_avg_sq, on_host):
        self.fp16, self.fp32, self.exp_avg, self.exp_avg_sq, self.on_host = fp16, fp32, exp_avg, exp_avg_sq, on_host


def plan_host_positions(n_positions, chunk_size, free_bytes, staging_slots=3, margin_use_ratio=0.8,
                        host_keeps_fp16=True):
    """Which chunk positions to keep in pinned host memory when ``free_bytes`` of HBM are available.

    The reference sizes its GPU share of the optimizer state from a memory margin measured during warm-up,
    ``margin / (chunk_size * 12) * margin_use_ratio`` chunks (``patrickstar/core/memtracer/memtracer.py:190-214``),
    and gives the FIRST chunks to the GPU (``patrickstar/ops/chunk_io_buff.py:234-239``).  Here a resident position
    costs 14 B/element (fp16 + fp32 + m + v) and the streaming path needs ``staging_slots`` more positions' worth of
    HBM; positions that do not fit go to the host, last positions first.  With ``host_keeps_fp16=False`` a host
    position still keeps its fp16 payload (2 B/element) in HBM and a staging slot holds 12 B/element.  Returns a
    ``set`` of position indices, usable as ``host_chunk_policy = planned.__contains__``.
    """
    per_position = 14 * chunk_size
    per_host_position = 0 if host_keeps_fp16 else 2 * chunk_size
    per_slot = per_position - per_host_position
    budget = free_bytes * margin_use_ratio
    if budget >= n_positions * per_position:
        return set()
    # resident * per_position + (n - resident) * per_host_position + slots * per_slot <= budget
    resident = int((budget - staging_slots * per_slot - n_positions * per_host_position) // (per_position - per_host_position))
    resident = max(0, min(n_positions, resident))
    return set(range(resident, n_positions))


class PatrickStarClient:
    def __init__(self, rank: int, default_chunk_size: int, config=None, device=None):
        self.local_rank = rank
        self.device = torch.device(device) if device is not None else torch.device(f"cuda:{rank}")
        self.default_chunk_size = default_chunk_size
        self.chunk_list = ChunkList(rank)
        self.chunk_tensor_index = ChunkTensorIndex(default_chunk_size)
        self.param_fp16_to_param_fp32_map: Dict[torch.nn.Parameter, torch.nn.Parameter] = {}
        self.chunk_based_param_fp16: List[torch.nn.Parameter] = []
        self.torch_managed_params: List[torch.nn.Parameter] = []  # fp32 parameters outside the chunk lists (use_cpu_embedding)
        self.module = None
        self.optimizer = None
        self._param_idx = 0
        # fp16 chunk ids of the positions whose fp32 / m / v chunks are kept in pinned host memory
        self.host_fp16_chunk_ids = set()
        # True: such a position's fp16 payload is in pinned host memory as well (the whole position is streamed);
        # False: it stays in HBM, where forward and backward use it (the only form a registered module can have)
        self.host_keeps_fp16 = True
        self._slabs = []  # the allocations HBM-resident payloads are views of
        # called with (position index among fp16 chunks) -> True to keep that position in host memory
        self.host_chunk_policy: Optional[Callable[[int], bool]] = None
        default_opts = {"with_mem_saving_comm": False, "with_mem_cache": False, "with_async_move": False}
        self.opt_config = dict(default_opts)
        # Placement when no policy is given: decided once, from the HBM that is free when the model is registered.
        self.use_hybrid_adam = True  # the optimizer's switch (fp16_cpu_adam.py:523-528); initialize_engine sets it
        self.hbm_budget_bytes = None  # None: ask the device (torch.cuda.mem_get_info)
        self.margin_use_ratio = 0.8  # the reference's default share of the margin (memtracer.py:190-214)
        self.staging_slots = 3  # what the optimizer streams host-resident positions through (FP16Adam.staging_slots)
        self.placement = None  # what plan_placement decided, for inspection
        if config is not None:
            self.opt_config.update(config.get("opts", {}))
            if "host_chunk_policy" in config:
                self.host_chunk_policy = config["host_chunk_policy"]
            self.host_keeps_fp16 = bool(config.get("host_keeps_fp16", True))
            self.hbm_budget_bytes = config.get("hbm_budget_bytes", None)
            self.margin_use_ratio = config.get("margin_use_ratio", 0.8)

    # -- building the lists -----------------------------------------------
    def append_chunk(self, data_type, chunk_type):
        chunk_id = self.chunk_list.generate_chunk_id()
        self.chunk_list.new_chunk(chunk_id, self.default_chunk_size, data_type, chunk_type)
        self.chunk_tensor_index.add_chunk(chunk_id, chunk_type)
        return chunk_id

    def append_tensor(self, param_list, data_type, access_type, chunk_type):
        """All of ``param_list`` goes into the last chunk of the list, or, if it does not fit, into a new one."""
        assert isinstance(data_type, torch.dtype)
        assert isinstance(access_type, AccessType)
        if not self.chunk_list.is_empty(chunk_type):
            last = self.chunk_list.last_chunk_id(chunk_type)
            if self.chunk_tensor_index.try_insert_tensor_list(last, param_list, access_type):
                return
        chunk_id = self.append_chunk(data_type, chunk_type)
        if not self.chunk_tensor_index.try_insert_tensor_list(chunk_id, param_list, access_type):
            raise RuntimeError(
                f"Can not append a tensor to chunk_tensor_index. "
                f"Overall size of param list is larger than the default chunk size {self.default_chunk_size}."
            )

    def append_tensor_as_ref(self, param, data_type, access_type, chunk_type, ref_param):
        """Place an optimizer-state tensor in the state chunk that shadows ``ref_param``'s fp16 chunk,
        at ``ref_param``'s own offset, so that all four lists share one layout and a whole chunk
        can be updated by a single pass."""
        index = self.chunk_tensor_index
        chunk_id = index.get_optimizer_state_chunk_id(ref_param, access_type, chunk_type)
        if chunk_id is None:
            chunk_id = self.append_chunk(data_type, chunk_type)
        ref_info = index.get_tensor_info(ref_param.ps_attr.get_tensor_id(access_type))
        if ref_info.numel != param.ps_attr.numel:
            raise RuntimeError("Failed to insert optimizer param w.r.t its ref_param.")
        tensor_id = param.ps_attr.get_tensor_id(access_type)
        if index.tensor_id_to_chunk_id(tensor_id) is None:
            index.add_tensor(chunk_id, tensor_id, ref_info.start_offset, ref_info.numel, param, access_type)
        index.register_optimizer_state_chunk_id(ref_param, access_type, chunk_type, chunk_id)

    def register_module_params(self, module):
        """Register the parameters a module owns directly as fp16 chunk tensors with fp32 shadows."""
        fp16_list, fp32_list = [], []
        for name, param in module.named_parameters(recurse=False):
            if is_param_registered(param):
                continue
            full = f"{module.__class__.__name__}.{name}_{self._param_idx}"
            self._param_idx += 1
            register_param(param, ParamType.CHUNK_BASED, torch.half, full)
            shadow = torch.nn.Parameter(torch.tensor([], dtype=torch.float), requires_grad=False)
            register_param(shadow, ParamType.CHUNK_BASED, torch.float, f"{full}_fp32")
            shadow.ps_attr.reset_shape(param.shape)
            self.param_fp16_to_param_fp32_map[param] = shadow
            self.chunk_based_param_fp16.append(param)
            fp16_list.append(param)
            fp32_list.append(shadow)
        if fp16_list:
            self.append_tensor(fp16_list, torch.half, AccessType.DATA, ChunkType.PARAM_FP16)
            self.append_tensor(fp32_list, torch.float, AccessType.DATA, ChunkType.PARAM_FP32)

    def plan_placement(self, free_bytes=None):
        """Decide which chunk positions keep their optimizer state (fp32 param, m, v) in pinned host memory.

        The reference measures a memory margin during its warm-up iteration, turns it into a number of chunks,
        ``margin / (chunk_size * 12) * margin_use_ratio`` (``patrickstar/core/memtracer/memtracer.py:190-214``), hands the
        FIRST that many chunks to the GPU and updates the rest on the CPU (``patrickstar/ops/chunk_io_buff.py:234-239``),
        all of it only when ``use_hybrid_adam`` is set (``patrickstar/ops/fp16_cpu_adam.py:523-528``).  Here the margin is
        the HBM that is free when the model is registered (or ``config["client"]["hbm_budget_bytes"]``); the fp16 payloads
        of all positions stay in HBM (2 B/element), a resident position costs 12 B/element more and the streaming path
        needs ``staging_slots`` positions' worth of staging.  Everything fits -> every position is resident (the normal
        case with 288 GB).  It does not fit -> the LAST positions go to the host if ``use_hybrid_adam``, else an error.
        An explicit ``host_chunk_policy`` is left alone.  Called by ``register_model`` before any payload exists.
        """
        if self.host_chunk_policy is not None:
            self.placement = {"source": "host_chunk_policy"}
            return
        n_positions = self.chunk_tensor_index.chunk_num(ChunkType.PARAM_FP16)
        if free_bytes is None:
            free_bytes = self.hbm_budget_bytes
        if free_bytes is None:
            if self.device.type != "cuda" or not torch.cuda.is_available():
                self.placement = {"source": "no device to ask", "host_positions": []}
                return
            free_bytes = torch.cuda.mem_get_info(self.device)[0]
        planned = plan_host_positions(
            n_positions, self.default_chunk_size, free_bytes, staging_slots=self.staging_slots,
            margin_use_ratio=self.margin_use_ratio, host_keeps_fp16=False,
        )
        self.placement = {"source": "free HBM", "free_bytes": free_bytes, "positions": n_positions,
                          "host_positions": sorted(planned)}
        if not planned:
            return
        if not self.use_hybrid_adam:
            need = 14 * self.default_chunk_size * n_positions
            raise RuntimeError(
                f"{n_positions} chunk positions of {self.default_chunk_size} elements need {need} bytes of HBM for fp16 + "
                f"fp32 + momentum + variance; {free_bytes} are free (x {self.margin_use_ratio}) and use_hybrid_adam is "
                "False, so no optimizer state may live in host memory"
            )
        self.host_chunk_policy = planned.__contains__

    def register_torch_managed_embedding(self, module):
        """``use_cpu_embedding`` of the reference (``patrickstar/core/preprocess.py:351-364``,
        ``patrickstar/ops/embedding.py:81-104``): the weights of an ``nn.Embedding`` stay fp32 parameters that PyTorch
        manages itself (``ParamType.TORCH_BASED``), outside the chunk lists; the lookup runs in fp32 and its output
        is cast to half.  The reference keeps such weights in host memory and looks them up on the CPU; here they
        stay in HBM (this package has no CPU compute path), which changes where the work runs, not its numbers.
        The optimizer updates them with the operator's arithmetic from their fp32 gradients
        (``patrickstar/ops/fp16_cpu_adam.py:345-353``).  As in the reference (``preprocess.py:260-282``) an empty
        fp16 parameter is put in front of the module's own, so that code which takes a model's dtype from its
        first parameter still sees half."""
        for name, param in module.named_parameters(recurse=False):
            if is_param_registered(param):
                continue
            register_param(param, ParamType.TORCH_BASED, torch.float, f"embedding_{name}")
            param.data = param.data.to(self.device, torch.float)
            self.torch_managed_params.append(param)
        if "dummy" not in module._parameters:
            module.dummy = torch.nn.Parameter(torch.tensor([], dtype=torch.half, device=self.device), requires_grad=False)
            register_param(module.dummy, ParamType.TORCH_BASED, torch.half, "embedding_dummy")
            others = [(k, module._parameters.pop(k)) for k in list(module._parameters) if k != "dummy"]
            module._parameters.update(others)  # "dummy" is now the first entry
        # the lookup itself runs in fp32; what the rest of the model sees is half (ops/embedding.py:104)
        module.register_forward_hook(lambda mod, args, output: output.to(torch.half))

    def register_model(self, model, use_cpu_embedding=False):
        """Register every module's own parameters in module CONSTRUCTION order (children finish
        constructing before their parent does), copy the initial values into the fp16 and fp32
        payloads and re-point each parameter at its fp16 chunk slot.  ``use_cpu_embedding``: the
        weights of ``nn.Embedding`` modules stay fp32 parameters of PyTorch's own (see
        ``register_torch_managed_embedding``)."""
        self.module = model
        # a module's parameters are views of the fp16 payloads, which forward and backward need in HBM:
        # positions selected by the host-chunk policy keep only their optimizer state in host memory
        self.host_keeps_fp16 = False

        def visit(m):
            for child in m.children():
                visit(child)
            if use_cpu_embedding and isinstance(m, torch.nn.Embedding):
                self.register_torch_managed_embedding(m)
            else:
                self.register_module_params(m)

        visit(model)
        self.plan_placement()
        self.allocate_payloads()
        for p16 in self.chunk_based_param_fp16:
            init = p16.data
            slot16 = self.access_data(p16)
            slot32 = self.access_data(self.param_fp16_to_param_fp32_map[p16])
            slot32.copy_(init.to(slot32.device, torch.float))
            slot16.copy_(slot32)
            p16.data = slot16  # the module now computes with the chunk's own memory
        return model

    def append_flat_chunks(self, n_chunks: int, used_numel_last: Optional[int] = None):
        """Synthetic chunk lists: one flat fp16 parameter per chunk (the last may be shorter; its tail
        stays zero).  Returns the fp16 parameters."""
        params = []
        for c in range(n_chunks):
            numel = self.default_chunk_size if (c < n_chunks - 1 or used_numel_last is None) else used_numel_last
            p16 = torch.nn.Parameter(torch.tensor([], dtype=torch.half), requires_grad=True)
            register_param(p16, ParamType.CHUNK_BASED, torch.half, f"flat_{self._param_idx}")
            p16.ps_attr.reset_shape(torch.Size([numel]))
            shadow = torch.nn.Parameter(torch.tensor([], dtype=torch.float), requires_grad=False)
            register_param(shadow, ParamType.CHUNK_BASED, torch.float, f"flat_{self._param_idx}_fp32")
            shadow.ps_attr.reset_shape(torch.Size([numel]))
            self._param_idx += 1
            self.param_fp16_to_param_fp32_map[p16] = shadow
            self.chunk_based_param_fp16.append(p16)
            # a new chunk per parameter, also when a short one would still fit behind the previous
            for plist, dt, ct in (([p16], torch.half, ChunkType.PARAM_FP16), ([shadow], torch.float, ChunkType.PARAM_FP32)):
                cid = self.append_chunk(dt, ct)
                assert self.chunk_tensor_index.try_insert_tensor_list(cid, plist, AccessType.DATA)
            params.append(p16)
        self.allocate_payloads()
        return params

    # -- payloads -------------------------------------------------------------
    def _fp16_chunk_of_position(self, chunk_id):
        """The fp16 chunk id whose list position a chunk of any list shares."""
        ctype = self.chunk_tensor_index.chunk_id_to_chunk_type_map[chunk_id]
        ids16 = self.chunk_tensor_index.chunk_type_to_chunk_id_list_map.get(ChunkType.PARAM_FP16, [])
        if ctype == ChunkType.PARAM_FP16:
            return chunk_id
        if ctype == ChunkType.PARAM_FP32:
            ids32 = self.chunk_tensor_index.chunk_type_to_chunk_id_list_map[ChunkType.PARAM_FP32]
            pos = ids32.index(chunk_id)
            return ids16[pos] if pos < len(ids16) else None  # an fp32 list driven on its own has no fp16 twin
        for ref_id, os_map in self.chunk_tensor_index.param_chunk_id_to_os_chunk_id_map.items():
            if os_map.get(ctype) == chunk_id:
                return ref_id
        raise KeyError(chunk_id)

    def allocate_payloads(self):
        """Give every chunk that has none a zero-filled payload.  Safe to call repeatedly.

        HBM-resident chunks of one list are carved out of ONE allocation per call (a slab): a few large
        allocations are backed by large physical fragments, which the streaming kernels need when few waves
        are in flight (measured: 6.30 TB/s from slabs vs 6.01 TB/s from one allocation per chunk; skewing the
        slabs' start addresses against each other by a few KiB made no measurable difference).
        Positions selected by the host-chunk policy get their own pinned host allocations instead.
        """
        ids16 = self.chunk_tensor_index.chunk_type_to_chunk_id_list_map.get(ChunkType.PARAM_FP16, [])
        if self.host_chunk_policy is not None:
            for pos, cid in enumerate(ids16):
                if self.host_chunk_policy(pos):
                    self.host_fp16_chunk_ids.add(cid)
        pending = {}
        for chunk_id, chunk in self.chunk_list.generate_chunk():
            if chunk.payload is not None:
                continue
            on_host = bool(self.host_fp16_chunk_ids) and self._fp16_chunk_of_position(chunk_id) in self.host_fp16_chunk_ids
            if on_host and (self.host_keeps_fp16 or chunk.chunk_type != ChunkType.PARAM_FP16):
                chunk.allocate_payload("cpu", pin_memory=True)
            else:
                pending.setdefault(chunk.chunk_type, []).append(chunk)
        for chunk_type, chunks in pending.items():
            if self.device.type == "cpu":
                for chunk in chunks:
                    chunk.allocate_payload(self.device)
                continue
            # every payload starts on a 512-element boundary of its slab (>= 1 KiB for every dtype), so that odd
            # chunk sizes do not push later chunks off the alignment the vector kernels want
            def stride(c):
                return -(-c.capacity // 512) * 512

            slab = torch.zeros(sum(stride(c) for c in chunks), dtype=chunks[0].data_type, device=self.device)
            self._slabs.append(slab)
            cursor = 0
            for chunk in chunks:
                chunk.payload = slab.narrow(0, cursor, chunk.capacity)
                cursor += stride(chunk)

    def chunk_ids_generator(self, chunk_type):
        for cid in self.chunk_tensor_index.chunk_type_to_chunk_id_list_map.get(chunk_type, []):
            yield cid

    def positions(self) -> List[ChunkPosition]:
        """Chunk ids of the four lists, position by position (needs the optimizer-state lists)."""
        idx = self.chunk_tensor_index
        ids16 = idx.chunk_type_to_chunk_id_list_map.get(ChunkType.PARAM_FP16, [])
        ids32 = idx.chunk_type_to_chunk_id_list_map.get(ChunkType.PARAM_FP32, [])
        out = []
        for c16, c32 in zip(ids16, ids32):
            os_map = idx.param_chunk_id_to_os_chunk_id_map.get(c16, {})
            out.append(
                ChunkPosition(
                    c16, c32, os_map.get(ChunkType.MOMENTUM), os_map.get(ChunkType.VARIANCE),
                    c16 in self.host_fp16_chunk_ids,
                )
            )
        return out

    # -- tensor views -----------------------------------------------------------
    def access_data(self, param, device=None):
        """The tensor of ``param`` inside its chunk payload (a view; nothing moves)."""
        if param.ps_attr.param_type == ParamType.TORCH_BASED:
            return param.data  # PyTorch's own tensor (patrickstar/core/client.py:552-553)
        info = self.chunk_tensor_index.get_tensor_info(param.ps_attr.data_id())
        payload = self.chunk_list[info.chunk_id].payload
        if payload is None:
            # first access: give every chunk that has none its (zero-filled) payload, as the reference does
            # on the first access of a chunk (patrickstar/core/client.py:350-420)
            self.allocate_payloads()
            payload = self.chunk_list[info.chunk_id].payload
        view = payload.narrow(0, info.start_offset, info.numel).view(param.ps_attr.shape)
        if device is not None and torch.device(device).type != view.device.type:
            # a copy would silently detach the caller from the chunk
            raise RuntimeError(
                f"{param.ps_attr.name} lives on {view.device}; this client does not move chunks (asked for {device})"
            )
        return view

    def release_data(self, param, reset_state=None):
        return None

    def is_local_param(self, param, access_type):
        return True

    def init(self, model, optimizer):
        self.module = model
        self.optimizer = optimizer

    def start_mem_tracer(self):
        return None
