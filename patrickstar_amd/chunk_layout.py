"""Chunk layout: the data model the optimizer step runs over.

Four parallel chunk lists (fp16 params/grads, fp32 master params, momentum,
variance) of ``default_chunk_size`` elements each; tensors are packed
first-fit, module by module; the unused tail of a chunk stays zero.

Only the layout and the 1-GPU "a tensor is a view into its chunk payload"
semantics are here.  The reference's eviction / movement / communication
machinery is not part of this path.

Reference for the rules (not for the code): ``patrickstar/core/const.py:76-86``
(types), ``core/parameter.py`` (``ps_attr``), ``core/tensor_stub.py``
(``TensorInfo``), ``core/chunk_tensor_index.py:69-113,266-320`` (optimizer-state
chunk map, first-fit insertion), ``core/chunk_data.py:122-176`` (zero-filled
payload), ``core/chunk_list.py:128-132,344-392``.
"""
import bisect
from enum import Enum
from typing import Dict, Iterator, List, Optional

import torch


class AccessType(Enum):
    DATA = 1
    GRAD = 2


class ChunkType(Enum):
    PARAM_FP16 = 0
    PARAM_FP32 = 1
    MOMENTUM = 2
    VARIANCE = 3
    UNDEF = 4


class ParamType(Enum):
    CHUNK_BASED = 0
    TORCH_BASED = 1


class _TensorSlot:
    """Identity of one tensor (data or grad) of a registered parameter."""

    _next_id = 0

    def __init__(self):
        self.id = _TensorSlot._next_id
        _TensorSlot._next_id += 1
        self.tensor = None


class PSParameter:
    """What ``param.ps_attr`` holds: the chunk-side description of a parameter.

    ``data_type`` may differ from ``param.dtype`` (an fp16 chunk parameter is
    created from an fp32 module parameter).
    """

    def __init__(self, param, param_type, data_type, name=None):
        self.name = name
        self.numel = param.numel()
        self.shape = param.shape
        self.data_type = data_type
        self.param_type = param_type
        self.data_chunk_id = None
        self.grad_chunk_id = None
        self._is_local = True
        if param_type == ParamType.CHUNK_BASED:
            self.data_tensor = _TensorSlot()
            self.grad_tensor = _TensorSlot() if param.requires_grad else None

    def is_local(self):
        return self._is_local

    def reset_shape(self, new_shape):
        self.shape = new_shape
        self.numel = new_shape.numel()

    def get_tensor_id(self, access_type):
        if self.param_type == ParamType.TORCH_BASED:
            return -1
        if not isinstance(access_type, AccessType):
            raise ValueError(access_type)
        slot = self.data_tensor if access_type == AccessType.DATA else self.grad_tensor
        return slot.id

    def data_id(self):
        return self.get_tensor_id(AccessType.DATA)

    def grad_id(self):
        return self.get_tensor_id(AccessType.GRAD)

    def __str__(self):
        return (
            f"name: {self.name}, numel: {self.numel}, shape: {self.shape}, data_type: {self.data_type}, "
            f"param_type: {self.param_type}, is_local: {self.is_local()}"
        )


def register_param(param, param_type, data_type, name=None):
    assert isinstance(param, torch.nn.Parameter)
    if not hasattr(param, "ps_attr"):
        param.ps_attr = PSParameter(param, param_type, data_type, name)


def is_param_registered(param) -> bool:
    assert isinstance(param, torch.nn.Parameter)
    return hasattr(param, "ps_attr")


class TensorInfo:
    """Where one tensor lives: chunk id, element offset, length."""

    def __init__(self, chunk_id, tensor_id, start_offset, numel, param, access_type, param_name=""):
        self.chunk_id = chunk_id
        self.tensor_id = tensor_id
        self.start_offset = start_offset
        self.numel = numel
        self.param = param
        self.access_type = access_type
        suffix = "data" if access_type == AccessType.DATA else "grad"
        self.tensor_name = f"{param_name}.{suffix}"

    def __str__(self):
        return (
            f"tensor_id: {self.tensor_id}, name: {self.tensor_name}, chunk_id: {self.chunk_id}, "
            f"start_offset: {self.start_offset}, numel: {self.numel}"
        )


class ChunkTensorIndex:
    """tensor id -> (chunk, offset) and chunk id -> tensors ordered by offset.

    Insertion is first-fit inside ONE chunk: the first gap between already
    placed tensors that is large enough, else the space after the last one,
    else failure.  A list of tensors (the parameters of one module) is placed
    atomically: if any member fails, the members placed so far are removed.
    """

    def __init__(self, default_chunk_size: int = 0):
        self.default_chunk_size = default_chunk_size
        self.tensor_id_to_info_map: Dict[int, TensorInfo] = {}
        self.chunk_id_to_tensor_id_list_map: Dict[int, List[int]] = {}
        self.chunk_type_to_chunk_id_list_map: Dict[ChunkType, List[int]] = {}
        self.chunk_id_to_chunk_type_map: Dict[int, ChunkType] = {}
        # fp16 param chunk id -> {ChunkType -> chunk id of that optimizer-state list}
        self.param_chunk_id_to_os_chunk_id_map: Dict[int, Dict[ChunkType, int]] = {}

    # -- chunks ---------------------------------------------------------
    def add_chunk(self, chunk_id, chunk_type: ChunkType):
        self.chunk_type_to_chunk_id_list_map.setdefault(chunk_type, []).append(chunk_id)
        self.chunk_id_to_chunk_type_map[chunk_id] = chunk_type
        self.chunk_id_to_tensor_id_list_map.setdefault(chunk_id, [])

    def chunk_num(self, list_type: ChunkType) -> int:
        return len(self.chunk_type_to_chunk_id_list_map.get(list_type, []))

    def is_local_chunk(self, chunk_id) -> bool:
        return True  # one GPU: every chunk is local

    # -- lookup -----------------------------------------------------------
    def get_tensor_info(self, tensor_id) -> TensorInfo:
        return self.tensor_id_to_info_map[tensor_id]

    def tensor_id_to_chunk_id(self, tensor_id) -> Optional[int]:
        info = self.tensor_id_to_info_map.get(tensor_id)
        return None if info is None else info.chunk_id

    def get_chunk_id(self, param, access_type) -> Optional[int]:
        return self.tensor_id_to_chunk_id(param.ps_attr.get_tensor_id(access_type))

    def generate_tensor_info_in_order(self, chunk_id) -> Iterator[TensorInfo]:
        for tid in self.chunk_id_to_tensor_id_list_map.get(chunk_id, []):
            yield self.tensor_id_to_info_map[tid]

    def params_generator(self, chunk_id):
        for tid in self.chunk_id_to_tensor_id_list_map[chunk_id]:
            yield self.tensor_id_to_info_map[tid].param

    def used_numel(self, chunk_id) -> int:
        """End offset of the last tensor in the chunk (0 for an empty chunk)."""
        ids = self.chunk_id_to_tensor_id_list_map.get(chunk_id, [])
        if not ids:
            return 0
        last = self.tensor_id_to_info_map[ids[-1]]
        return last.start_offset + last.numel

    # -- placement ----------------------------------------------------------
    def _record(self, chunk_id, position, tensor_id, start, numel, param, access_type):
        name = param.ps_attr.name if is_param_registered(param) else None
        self.tensor_id_to_info_map[tensor_id] = TensorInfo(
            chunk_id, tensor_id, start, numel, param, access_type, name
        )
        self.chunk_id_to_tensor_id_list_map.setdefault(chunk_id, []).insert(position, tensor_id)
        if is_param_registered(param):
            if access_type == AccessType.DATA:
                param.ps_attr.data_chunk_id = chunk_id
            elif access_type == AccessType.GRAD:
                param.ps_attr.grad_chunk_id = chunk_id

    def add_tensor(self, chunk_id, tensor_id, start_offset, numel, param, access_type):
        """Place a tensor at a GIVEN offset (kept ordered by offset)."""
        ids = self.chunk_id_to_tensor_id_list_map.setdefault(chunk_id, [])
        starts = [self.tensor_id_to_info_map[t].start_offset for t in ids]
        self._record(
            chunk_id, bisect.bisect_right(starts, start_offset), tensor_id, start_offset, numel, param, access_type
        )

    def try_insert_tensor(self, chunk_id, param, access_type) -> bool:
        assert is_param_registered(param)
        tensor_id = param.ps_attr.get_tensor_id(access_type)
        ids = self.chunk_id_to_tensor_id_list_map.setdefault(chunk_id, [])
        if tensor_id in ids:
            return True  # already placed here: nothing to do
        need = param.ps_attr.numel
        cursor = 0
        for position, other in enumerate(ids):
            info = self.tensor_id_to_info_map[other]
            if info.start_offset - cursor >= need:
                self._record(chunk_id, position, tensor_id, cursor, need, param, access_type)
                return True
            cursor = info.start_offset + info.numel
        if self.default_chunk_size - cursor >= need:
            self._record(chunk_id, len(ids), tensor_id, cursor, need, param, access_type)
            return True
        return False

    def try_insert_tensor_list(self, chunk_id, param_list, access_type) -> bool:
        placed = []
        for param in param_list:
            placed.append(param)
            if not self.try_insert_tensor(chunk_id, param, access_type):
                for p in placed:
                    self.delete_tensor(chunk_id, p, access_type)
                return False
        return True

    def delete_tensor(self, chunk_id, param, access_type):
        assert is_param_registered(param)
        tensor_id = param.ps_attr.get_tensor_id(access_type)
        if tensor_id not in self.tensor_id_to_info_map:
            return
        del self.tensor_id_to_info_map[tensor_id]
        self.chunk_id_to_tensor_id_list_map[chunk_id].remove(tensor_id)

    # -- optimizer-state chunks follow their fp16 parameter chunk ------------
    def register_optimizer_state_chunk_id(self, ref_param, access_type, chunk_type, chunk_id):
        ref_chunk_id = self.get_chunk_id(ref_param, access_type)
        self.param_chunk_id_to_os_chunk_id_map.setdefault(ref_chunk_id, {})[chunk_type] = chunk_id

    def get_optimizer_state_chunk_id(self, ref_param, access_type, chunk_type) -> Optional[int]:
        ref_chunk_id = self.get_chunk_id(ref_param, access_type)
        return self.param_chunk_id_to_os_chunk_id_map.get(ref_chunk_id, {}).get(chunk_type)


class Chunk:
    """One payload of ``capacity`` elements; zero-filled on allocation."""

    def __init__(self, capacity: int, data_type: torch.dtype, chunk_id: int, chunk_type: ChunkType):
        self.capacity = capacity
        self.data_type = data_type
        self.chunk_id = chunk_id
        self.chunk_type = chunk_type
        self.payload: Optional[torch.Tensor] = None

    def allocate_payload(self, device, pin_memory=False):
        device = torch.device(device)
        if device.type == "cpu":
            self.payload = torch.zeros(self.capacity, dtype=self.data_type, pin_memory=pin_memory)
        else:
            self.payload = torch.zeros(self.capacity, dtype=self.data_type, device=device)
        return self.payload

    def release_payload(self):
        self.payload = None

    def get_device(self):
        return None if self.payload is None else self.payload.device

    def get_chunk_space(self) -> int:
        return self.capacity * torch.empty((), dtype=self.data_type).element_size()


class ChunkList:
    """All chunks by id, and the ids of each list in creation order."""

    def __init__(self, local_rank: int = 0):
        self.local_rank = local_rank
        self.id_to_chunk_map: Dict[int, Chunk] = {}
        self.chunk_type_to_id_list_map: Dict[ChunkType, List[int]] = {}
        self._next_chunk_id = 0

    def __getitem__(self, chunk_id) -> Chunk:
        return self.id_to_chunk_map.get(chunk_id)

    def __len__(self):
        return len(self.id_to_chunk_map)

    def size(self):
        return len(self.id_to_chunk_map)

    def generate_chunk_id(self) -> int:
        cid = self._next_chunk_id
        self._next_chunk_id += 1
        return cid

    def new_chunk(self, chunk_id, chunk_size, data_type, chunk_type: ChunkType):
        if chunk_id in self.id_to_chunk_map:
            raise RuntimeError(f"chunk list new chunk with chunk_id {chunk_id} already existed")
        self.id_to_chunk_map[chunk_id] = Chunk(chunk_size, data_type, chunk_id, chunk_type)
        self.chunk_type_to_id_list_map.setdefault(chunk_type, []).append(chunk_id)
        return chunk_type

    def is_empty(self, chunk_type: ChunkType) -> bool:
        return len(self.chunk_type_to_id_list_map.get(chunk_type, [])) == 0

    def last_chunk_id(self, chunk_type: ChunkType) -> int:
        if self.is_empty(chunk_type):
            raise RuntimeError(f"Call last_chunk_id on an empty {chunk_type} chunk list")
        return self.chunk_type_to_id_list_map[chunk_type][-1]

    def generate_chunk(self):
        for chunk_id, chunk in self.id_to_chunk_map.items():
            yield chunk_id, chunk

    def max_chunk_size(self) -> int:
        return max((c.capacity for c in self.id_to_chunk_map.values()), default=0)
