"""Wrap policies: predicates over modules that say which submodules become
flat-buffer units of their own (matrix_fsdp/policy/wrap.py:10-68).  A policy
is any ``callable(module) -> bool``; these are the stock ones and their
combinators."""
from __future__ import annotations

from collections.abc import Callable, Iterable

from torch import nn

WrapPolicy = Callable[[nn.Module], bool]


def module_type_policy(module_types: type[nn.Module] | Iterable[type[nn.Module]]) -> WrapPolicy:
    types = (module_types,) if isinstance(module_types, type) else tuple(module_types)
    if not types:
        raise ValueError("module_type_policy() expects at least one module type.")
    if not all(isinstance(t, type) and issubclass(t, nn.Module) for t in types):
        raise TypeError("module_type_policy() expects nn.Module types.")
    return lambda module: isinstance(module, types)


def size_based_policy(min_num_params: int, *, recurse: bool = False) -> WrapPolicy:
    """Modules holding at least ``min_num_params`` parameter elements, counting
    only their own parameters unless ``recurse``."""
    if min_num_params < 0:
        raise ValueError("min_num_params must be non-negative.")
    return lambda module: sum(p.numel() for p in module.parameters(recurse=recurse)) >= min_num_params


def _callables(policies: tuple) -> None:
    if not policies:
        raise ValueError("Expected at least one wrap policy.")
    if not all(callable(p) for p in policies):
        raise TypeError("Wrap policies must be callable.")


def or_policy(*policies: WrapPolicy) -> WrapPolicy:
    _callables(policies)
    return lambda module: any(p(module) for p in policies)


def and_policy(*policies: WrapPolicy) -> WrapPolicy:
    _callables(policies)
    return lambda module: all(p(module) for p in policies)


def not_policy(policy: WrapPolicy) -> WrapPolicy:
    if not callable(policy):
        raise TypeError("not_policy() expects a callable policy.")
    return lambda module: not policy(module)
