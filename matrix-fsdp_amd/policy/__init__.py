"""Which modules of a tree become units: predicates over ``nn.Module`` and their combinators."""
from .wrap import WrapPolicy, and_policy, module_type_policy, not_policy, or_policy, size_based_policy

__all__ = ["WrapPolicy", "and_policy", "module_type_policy", "not_policy", "or_policy", "size_based_policy"]
