"""MI355X-native chunk-wise mixed-precision Adam step with fp16 loss scaling.

A drop-in for ONE path of PatrickStar: ``initialize_engine(config)`` /
``optimizer.step()`` over the four-list chunk layout, executed by hand-written
HIP kernels (gfx950) behind the C ABI of ``include/ps_adam.h``.
"""
from . import adam_op  # noqa: F401
from .chunk_layout import (  # noqa: F401
    AccessType,
    Chunk,
    ChunkList,
    ChunkTensorIndex,
    ChunkType,
    ParamType,
    TensorInfo,
    is_param_registered,
    register_param,
)
from .client import PatrickStarClient, plan_host_positions  # noqa: F401
from .engine import PatrickStarEngine, initialize_engine, parse_config  # noqa: F401
from .fp16_adam import FP16Adam  # noqa: F401
from .loss_scaler import DynamicLossScaler, LossScaler  # noqa: F401

__version__ = "0.1.0"
