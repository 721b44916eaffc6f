"""MatrixFSDP's per-rank data-parallel hot path on MI355X (gfx950).

Flat-buffer copy-in / copy-out (pack, unpack, gradient chunk-cat with
bf16->fp32 cast) and the owner-rank Muon / AdamW update as hand-written HIP
kernels behind a C ABI (``include/mfsdp_hip.h``), with a host side that keeps
the reference's shard metadata and operator signatures.
"""
from .core.layout import LayoutSegment, ShardPlan, validate_shard_plan
from .core.managed_param import ManagedParam, ParamShardHint, managed_params_from_module, managed_params_from_named
from .api import MixedPrecisionPolicy, fully_shard, matrix_fully_shard
from .optim.wrapper import MatrixOptimizerConfig, MixedMuonAdamWOptimizer, configure_optimizer
from .runtime.param_group import FSDPLifecycleState, MatrixFSDPParamGroup

__all__ = [
    "LayoutSegment",
    "ShardPlan",
    "validate_shard_plan",
    "ManagedParam",
    "ParamShardHint",
    "managed_params_from_module",
    "managed_params_from_named",
    "MixedPrecisionPolicy",
    "fully_shard",
    "matrix_fully_shard",
    "MatrixOptimizerConfig",
    "MixedMuonAdamWOptimizer",
    "configure_optimizer",
    "FSDPLifecycleState",
    "MatrixFSDPParamGroup",
]
