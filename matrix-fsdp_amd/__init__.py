"""MatrixFSDP's per-rank data-parallel hot path on MI355X (gfx950).

Flat-buffer copy-in / copy-out (pack, unpack, gradient chunk-cat with
bf16->fp32 cast) and the owner-rank Muon / AdamW update as hand-written HIP
kernels behind a C ABI (``include/mfsdp_hip.h``), with a host side that keeps
the reference's shard metadata and operator signatures.
"""
from .core.layout import LayoutSegment, ShardPlan, validate_shard_plan
from .core.managed_param import ManagedParam, ParamShardHint, managed_params_from_module, managed_params_from_named
from .api import MixedPrecisionPolicy, fully_shard, matrix_fully_shard
from .core.placement import MatrixShard
from .core.state import MatrixShardedState
from .optim.state import MatrixFSDPOptimizerStateManager
from .policy.wrap import and_policy, module_type_policy, not_policy, or_policy, size_based_policy
from .optim.wrapper import MatrixFSDPOptimizer, MatrixOptimizerConfig, MixedMuonAdamWOptimizer, configure_optimizer
from .runtime.param_group import FSDPLifecycleState, MatrixFSDPParamGroup
from .checkpoint import (
    get_model_state_dict,
    get_optimizer_state_dict,
    get_state_dict,
    load_matrix_dcp,
    load_matrix_dcp_full_state,
    load_matrix_state_dict,
    matrix_get_state_dict,
    matrix_set_state_dict,
    matrix_state_dict,
    patch_model_state_dict,
    patch_optimizer_state_dict,
    save_matrix_dcp,
    save_matrix_dcp_simulated_world,
    set_model_state_dict,
    set_optimizer_state_dict,
    set_state_dict,
)

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
    "MatrixShard",
    "MatrixShardedState",
    "MatrixFSDPOptimizer",
    "MatrixFSDPOptimizerStateManager",
    "and_policy",
    "module_type_policy",
    "not_policy",
    "or_policy",
    "size_based_policy",
    "get_model_state_dict",
    "get_optimizer_state_dict",
    "get_state_dict",
    "load_matrix_dcp",
    "load_matrix_dcp_full_state",
    "load_matrix_state_dict",
    "matrix_get_state_dict",
    "matrix_set_state_dict",
    "matrix_state_dict",
    "patch_model_state_dict",
    "patch_optimizer_state_dict",
    "save_matrix_dcp",
    "save_matrix_dcp_simulated_world",
    "set_model_state_dict",
    "set_optimizer_state_dict",
    "set_state_dict",
]
