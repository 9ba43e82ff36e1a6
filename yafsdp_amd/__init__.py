"""MI355X-native per-rank buffer path of YaFSDP-style sharded data parallelism.

Host side (Python) mirrors the reference's interface for this path
(``ya_fsdp/_collectives.py``, ``_param_group.py``, ``_param.py``, ``_api.py``);
every tensor op on the path is a hand-written gfx950 kernel reached through the
C ABI of ``libyafsdp_hip.so`` (``include/yafsdp_hip.h``).  Importing the package
does not load the library; the modules that launch kernels do, and fail loudly
if it has not been built (``python -m yafsdp_amd._build``).
"""

from ._api import MixedPrecisionPolicy
from ._common import FSDPMeshInfo, LogicalShardGroup, ShardedState, TrainingState
from ._layout import RaggedShard, ShardLayout, make_layout

__all__ = [
    "MixedPrecisionPolicy",
    "FSDPMeshInfo",
    "LogicalShardGroup",
    "ShardedState",
    "TrainingState",
    "RaggedShard",
    "ShardLayout",
    "make_layout",
    "YaFSDPParamGroup",
    "YaFSDPBufferContext",
    "YaFSDPCommContext",
    "init_shared_state",
    "all_gather",
    "reduce_scatter",
    "AllGatherResult",
    "fully_shard",
    "YaFSDPModule",
    "UnshardHandle",
    "RaggedShardDTensor",
    "connect_logical_ranks",
]

_LAZY = {
    "YaFSDPParamGroup": "_param_group",
    "YaFSDPBufferContext": "_param_group",
    "YaFSDPCommContext": "_param_group",
    "init_shared_state": "_param_group",
    "all_gather": "_collectives",
    "reduce_scatter": "_collectives",
    "AllGatherResult": "_collectives",
    "fully_shard": "fully_shard",
    "YaFSDPModule": "fully_shard",
    "UnshardHandle": "fully_shard",
    "RaggedShardDTensor": "_tensor",
    "connect_logical_ranks": "_tensor",
}


def __getattr__(name):
    if name in _LAZY:
        import importlib

        value = getattr(importlib.import_module(f"{__name__}.{_LAZY[name]}"), name)
        globals()[name] = value  # also replaces the submodule of the same name (fully_shard)
        return value
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
