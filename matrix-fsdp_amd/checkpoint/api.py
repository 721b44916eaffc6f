"""``(model_state_dict, optim_state_dict)``-shaped access to MatrixFSDP state,
for training code written against
``torch.distributed.checkpoint.state_dict.get_state_dict`` / ``set_state_dict``
(matrix_fsdp/checkpoint/_api.py:15-277).  The model half is a
``matrix_state_dict``; the optimizer half is the optimizer's own
``state_dict()`` (a dict of them, keyed ``"0"``, ``"1"``, ..., for several
optimizers).  ``options`` may carry ``full_state_dict`` and ``cpu_offload``.
"""
from __future__ import annotations

import functools
from typing import Any

import torch
from torch import nn

from .state_dict import load_matrix_state_dict, matrix_state_dict

_PATCHED_CALLS: set[Any] = set()


def _optimizers(optimizers) -> tuple[Any, ...]:
    if hasattr(optimizers, "state_dict") and hasattr(optimizers, "load_state_dict"):
        return (optimizers,)
    return tuple(optimizers)


def _unpatched(obj, name: str):
    """``obj.<name>`` -- the class's own method when ``patch_*`` replaced it, so
    that a patched ``state_dict`` does not call itself."""
    call = getattr(obj, name)
    return functools.partial(getattr(type(obj), name), obj) if call in _PATCHED_CALLS else call


def _snapshot(value, *, to_host: bool, _memo: dict | None = None):
    """Copies of every tensor (on the host if asked); containers that occur
    twice stay one object.  An optimizer's ``state_dict()`` hands out its live
    tensors; a counter shared between the saved state and the running
    optimizer would keep counting in both."""
    memo = {} if _memo is None else _memo
    if id(value) in memo:
        return memo[id(value)]
    if torch.is_tensor(value):
        out = value.detach().cpu() if to_host and value.is_cuda else value.detach().clone()
    elif isinstance(value, dict):
        out = memo[id(value)] = {}
        out.update((key, _snapshot(item, to_host=to_host, _memo=memo)) for key, item in value.items())
    elif isinstance(value, list):
        out = memo[id(value)] = []
        out.extend(_snapshot(item, to_host=to_host, _memo=memo) for item in value)
    elif isinstance(value, tuple):
        out = tuple(_snapshot(item, to_host=to_host, _memo=memo) for item in value)
    else:
        return value
    memo[id(value)] = out
    return out


def _no_submodules(submodules) -> None:
    if submodules:
        raise NotImplementedError("MatrixFSDP state_dict submodule filtering is not supported yet.")


def matrix_get_state_dict(module: nn.Module, optimizers=None, *, options=None) -> tuple[dict[str, Any], dict[str, Any]]:
    model_state = matrix_state_dict(module, full_state=bool(getattr(options, "full_state_dict", False)), clone=True)
    optim_state: dict[str, Any] = {}
    if optimizers is not None:
        many = _optimizers(optimizers)
        if len(many) == 1:
            optim_state = _unpatched(many[0], "state_dict")()
        else:
            optim_state = {str(i): _unpatched(opt, "state_dict")() for i, opt in enumerate(many)}
    to_host = bool(getattr(options, "cpu_offload", False))
    if to_host:
        model_state = _snapshot(model_state, to_host=True)
    return model_state, _snapshot(optim_state, to_host=to_host)


def _load_optimizers(optimizers, optim_state_dict: dict[str, Any]) -> None:
    many = _optimizers(optimizers)
    for index, optimizer in enumerate(many):
        if len(many) == 1:
            state = optim_state_dict
        elif str(index) in optim_state_dict:
            state = optim_state_dict[str(index)]
        else:
            raise ValueError(f"Missing optimizer state for optimizer index {index}.")
        _unpatched(optimizer, "load_state_dict")(state)
        refresh = getattr(optimizer, "refresh_state_dtensors", None)
        if refresh is not None:
            refresh()


def matrix_set_state_dict(module: nn.Module, optimizers=None, *, model_state_dict: dict[str, Any], optim_state_dict: dict[str, Any] | None = None, options=None) -> None:
    """Loads what ``matrix_get_state_dict`` returned (same layout)."""
    del options  # the same-layout loader is strict by construction
    load_matrix_state_dict(module, model_state_dict)
    if optimizers is not None and optim_state_dict is not None:
        _load_optimizers(optimizers, optim_state_dict)


def get_state_dict(model: nn.Module, optimizers=None, *, submodules=None, options=None):
    _no_submodules(submodules)
    return matrix_get_state_dict(model, optimizers, options=options)


def get_model_state_dict(model: nn.Module, *, submodules=None, options=None) -> dict[str, Any]:
    _no_submodules(submodules)
    return matrix_get_state_dict(model, None, options=options)[0]


def get_optimizer_state_dict(model: nn.Module, optimizers, *, submodules=None, options=None) -> dict[str, Any]:
    _no_submodules(submodules)
    return matrix_get_state_dict(model, optimizers, options=options)[1]


def set_state_dict(model: nn.Module, optimizers=None, *, model_state_dict: dict[str, Any], optim_state_dict: dict[str, Any] | None = None, options=None) -> None:
    matrix_set_state_dict(model, optimizers, model_state_dict=model_state_dict, optim_state_dict=optim_state_dict, options=options)


def set_model_state_dict(model: nn.Module, model_state_dict: dict[str, Any], *, options=None) -> None:
    matrix_set_state_dict(model, None, model_state_dict=model_state_dict, options=options)


def set_optimizer_state_dict(model: nn.Module, optimizers, optim_state_dict: dict[str, Any], *, options=None) -> None:
    del model, options
    _load_optimizers(optimizers, optim_state_dict)


def patch_model_state_dict(model: nn.Module, *, options=None) -> nn.Module:
    """``model.state_dict()`` / ``model.load_state_dict()`` become the MatrixFSDP
    calls, for code that insists on the methods."""

    def load(state_dict, strict: bool = True, assign: bool = False):
        del strict, assign
        set_model_state_dict(model, state_dict, options=options)
        return torch.nn.modules.module._IncompatibleKeys([], [])

    model.state_dict = functools.partial(get_model_state_dict, model, options=options)  # type: ignore[method-assign]
    model.load_state_dict = load  # type: ignore[method-assign]
    _PATCHED_CALLS.update((model.state_dict, model.load_state_dict))
    return model


def patch_optimizer_state_dict(model: nn.Module, optimizers, *, options=None):
    for optimizer in _optimizers(optimizers):
        optimizer.state_dict = functools.partial(get_optimizer_state_dict, model, optimizer, options=options)  # type: ignore[method-assign]
        optimizer.load_state_dict = functools.partial(set_optimizer_state_dict, model, optimizer, options=options)  # type: ignore[method-assign]
        _PATCHED_CALLS.update((optimizer.state_dict, optimizer.load_state_dict))
    return optimizers
