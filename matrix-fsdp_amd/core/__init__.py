from .layout import LayoutSegment, ShardPlan, validate_shard_plan
from .managed_param import ManagedParam, ParamShardHint, managed_params_from_module, managed_params_from_named

__all__ = [
    "LayoutSegment",
    "ShardPlan",
    "validate_shard_plan",
    "ManagedParam",
    "ParamShardHint",
    "managed_params_from_module",
    "managed_params_from_named",
]
