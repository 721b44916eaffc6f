"""Optimizer construction for flat-buffer managed parameters.

Mirrors the Muon / AdamW wiring of matrix_fsdp/optim/wrapper.py
(``MixedMuonAdamWOptimizer`` :353-612, ``classify_matrix_optimizer_params``
:687-737, ``configure_optimizer`` :763-821, ``_optimizer_type_for_param``
:827-846) with the inner optimizers replaced by the HIP-backed ``Muon`` and
``FusedAdamW`` of this package.  The "units" handed in are ``MatrixFlatBuffer``
objects (or a module carrying them as ``_matrix_fsdp_flat_buffers``); the
prefetch-scheduler arguments of the reference have no counterpart on one
device: they are accepted by name and dropped, anything else is a ``TypeError``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Iterable

import torch
from torch import nn

from ..core.managed_param import ManagedParam
from .adamw import FusedAdamW
from .adamw_state import initialize_flat_adamw_state
from .muon import Muon
from .state import MatrixFSDPOptimizerStateManager

DEFAULT_MUON_ADJUST_LR_FN = "match_rms_adamw"


@dataclass(frozen=True)
class MatrixOptimizerParamGroupSummary:
    name: str
    optimizer_type: str
    param_fqns: tuple[str, ...]
    numel: int

    def as_dict(self) -> dict[str, Any]:
        return {"name": self.name, "optimizer_type": self.optimizer_type, "param_fqns": self.param_fqns, "numel": self.numel}


@dataclass(frozen=True)
class ClassifiedMatrixOptimizerParams:
    muon_params: tuple[nn.Parameter, ...]
    adamw_params: tuple[nn.Parameter, ...]
    group_summaries: tuple[MatrixOptimizerParamGroupSummary, ...]


@dataclass(frozen=True)
class MatrixOptimizerConfig:
    optimizer: str = "adamw"
    kwargs: dict[str, Any] = field(default_factory=dict)
    default_matrix_optimizer: str = "muon"
    default_other_optimizer: str = "adamw"


def collect_flat_buffers(module_or_units) -> list:
    if isinstance(module_or_units, nn.Module):
        found = []
        for module in module_or_units.modules():
            found.extend(getattr(module, "_matrix_fsdp_flat_buffers", ()))
        return found
    if hasattr(module_or_units, "local_param_views"):
        return [module_or_units]
    if hasattr(module_or_units, "flat_buffer"):  # one unit
        return [] if module_or_units.flat_buffer is None else [module_or_units.flat_buffer]
    found = []
    for item in module_or_units:
        buffer = getattr(item, "flat_buffer", item)  # a unit or a flat buffer
        if buffer is not None:
            found.append(buffer)
    return found


def collect_param_groups(module_or_units) -> list:
    """The ``MatrixFSDPParamGroup`` units of a module (in ``named_modules``
    order), of one unit, or of an iterable of units."""
    if isinstance(module_or_units, nn.Module):
        units, seen = [], set()
        for module in module_or_units.modules():
            unit = getattr(module, "_matrix_fsdp_param_group", None)
            if unit is not None and id(unit) not in seen:
                seen.add(id(unit))
                units.append(unit)
        return units
    if hasattr(module_or_units, "flat_buffer"):
        return [module_or_units]
    return list(module_or_units)


def _optimizer_type_for_param(managed_param: ManagedParam, param: nn.Parameter, *, default_matrix_optimizer: str, default_other_optimizer: str) -> str:
    """Muon only for parameters whose *local view* is the whole 2-D matrix."""
    hint = managed_param.shard_hint.optimizer_type
    if hint == "muon":
        if len(managed_param.shape) != 2 or param.ndim != 2:
            raise ValueError(
                f"Param {managed_param.fqn!r} is marked for Muon, but its local view is not a full 2D matrix. "
                f"Use matrix_owner planning for Muon parameters."
            )
        return "muon"
    if hint == "adamw":
        return "adamw"
    if len(managed_param.shape) == 2 and param.ndim == 2:
        return default_matrix_optimizer
    return default_other_optimizer


def classify_matrix_optimizer_params(module_or_units, *, default_matrix_optimizer: str = "muon", default_other_optimizer: str = "adamw") -> ClassifiedMatrixOptimizerParams:
    flat_buffers = collect_flat_buffers(module_or_units)
    if not flat_buffers:
        raise ValueError("Expected a module wrapped by matrix_fully_shard().")
    if default_matrix_optimizer not in ("muon", "adamw"):
        raise ValueError("default_matrix_optimizer must be 'muon' or 'adamw'.")
    if default_other_optimizer not in ("muon", "adamw"):
        raise ValueError("default_other_optimizer must be 'muon' or 'adamw'.")
    grouped: dict[str, list[tuple[ManagedParam, nn.Parameter]]] = {"muon": [], "adamw": []}
    seen: set[int] = set()
    for fb in flat_buffers:
        for view in fb.local_param_views:
            mp = view.managed_param
            param = mp.param
            if id(param) in seen or param.numel() == 0:
                continue
            seen.add(id(param))
            kind = _optimizer_type_for_param(mp, param, default_matrix_optimizer=default_matrix_optimizer, default_other_optimizer=default_other_optimizer)
            grouped[kind].append((mp, param))
    if not grouped["muon"] and not grouped["adamw"]:
        raise RuntimeError("No non-empty local MatrixFSDP parameters were found for optimizer construction.")
    summaries = tuple(
        MatrixOptimizerParamGroupSummary(kind, kind, tuple(mp.fqn for mp, _ in entries), sum(p.numel() for _, p in entries))
        for kind, entries in grouped.items()
        if entries
    )
    return ClassifiedMatrixOptimizerParams(
        tuple(p for _, p in grouped["muon"]), tuple(p for _, p in grouped["adamw"]), summaries
    )


_SCHEDULER_KWARG_NAMES = frozenset(
    {
        "max_unsharded_prefetch_units",
        "max_forward_prefetch_units",
        "max_backward_prefetch_units",
        "backward_prefetch_timing",
        "prefetch_policy",
        "max_cached_full_param_buffers_per_key",
        "max_cached_elastic_workspaces_per_key",
        "max_active_full_param_buffers",
        "max_active_full_param_numel",
        "max_active_full_param_memory_mb",
        "max_pending_backward_reduces",
        "owner_backward_prefetch_with_pending_reduce",
        "trim_cuda_cache",
        "cuda_cache_trim_threshold_mb",
        "scheduler_config",
    }
)


class LazyMuon:
    """``Muon`` built at the first ``step()`` (matrix_fsdp/optim/wrapper.py:615-684, ``_LazyMuonOptimizer``).

    The reference delays ``torch.optim.Muon`` because an optimizer that allocates its momentum buffers up front can
    push the first forward of a large model out of memory.  Until the first step this object answers with what an
    optimizer without any state would: ``state == {}``, ``state_dict()["state"] == {}``, one parameter group holding
    the constructor's keywords.  ``load_state_dict`` and ``add_param_group`` build the optimizer first."""

    def __init__(self, params: Iterable[nn.Parameter], **kwargs: Any) -> None:
        self.params = tuple(params)
        self.kwargs = dict(kwargs)
        self._built: Muon | None = None
        self._pending_groups = [dict(self.kwargs, params=list(self.params))]

    def _materialize(self) -> Muon:
        if self._built is None:
            with _without_auto_prepare():
                self._built = Muon(self.params, **self.kwargs)
        return self._built

    @property
    def param_groups(self) -> list[dict[str, Any]]:
        return self._pending_groups if self._built is None else self._built.param_groups

    @property
    def state(self) -> dict[Any, Any]:
        return {} if self._built is None else self._built.state

    @property
    def defaults(self) -> dict[str, Any]:
        return dict(self.kwargs) if self._built is None else self._built.defaults

    def step(self, closure=None):
        built = self._materialize()
        return built.step() if closure is None else built.step(closure=closure)

    def zero_grad(self, set_to_none: bool = True) -> None:
        if self._built is not None:
            self._built.zero_grad(set_to_none=set_to_none)
            return
        for p in self.params:
            if p.grad is None:
                continue
            if set_to_none:
                p.grad = None
            else:
                p.grad.detach_()
                p.grad.zero_()

    def state_dict(self) -> dict[str, Any]:
        if self._built is not None:
            return self._built.state_dict()
        groups = [dict({k: v for k, v in g.items() if k != "params"}, params=list(range(len(g["params"])))) for g in self._pending_groups]
        return {"state": {}, "param_groups": groups}

    def load_state_dict(self, state_dict: dict[str, Any]) -> None:
        self._materialize().load_state_dict(state_dict)

    def add_param_group(self, param_group: dict[str, Any]) -> None:
        self._materialize().add_param_group(param_group)


_LazyMuonOptimizer = LazyMuon  # the reference's name for it


class MixedMuonAdamWOptimizer:
    """Muon on local full 2-D matrices, AdamW on everything else; the two inner
    optimizers stay separate objects.  Defaults follow the reference
    (``muon_momentum=0.5``, ``muon_ns_steps=2``, ``muon_adjust_lr_fn="match_rms_adamw"``)."""

    def __init__(
        self,
        muon_params: Iterable[nn.Parameter],
        adamw_params: Iterable[nn.Parameter],
        *,
        group_summaries: Iterable[MatrixOptimizerParamGroupSummary] = (),
        lr: float = 0.001,
        weight_decay: float = 0.01,
        muon_lr: float | None = None,
        adamw_lr: float | None = None,
        adamw_betas: tuple[float, float] = (0.9, 0.999),
        adamw_eps: float = 1e-8,
        adamw_weight_decay: float | None = None,
        adamw_foreach: bool | None = None,
        muon_weight_decay: float | None = None,
        muon_momentum: float = 0.5,
        muon_ns_steps: int = 2,
        muon_adjust_lr_fn: str | None = DEFAULT_MUON_ADJUST_LR_FN,
        lazy_muon_init: bool = False,
        flat_adamw_state: bool = False,
        flat_buffers: Iterable | None = None,
        fsdp_param_groups: Iterable | None = None,
        **scheduler_kwargs: Any,
    ) -> None:
        # The reference's constructor also takes its prefetch scheduler's settings (matrix_fsdp/optim/wrapper.py:384-399);
        # one device has nothing to schedule, so exactly those names are accepted and dropped.  ``adamw_foreach`` picks
        # between torch's two AdamW loops there; here AdamW is one fused launch per contiguous run either way.
        unknown = sorted(set(scheduler_kwargs) - _SCHEDULER_KWARG_NAMES)
        if unknown:
            raise TypeError(f"MixedMuonAdamWOptimizer.__init__() got an unexpected keyword argument {unknown[0]!r}")
        self.adamw_foreach = adamw_foreach
        self.lazy_muon_init = bool(lazy_muon_init)
        self.fsdp_param_groups = list(fsdp_param_groups or ())
        self.muon_params = tuple(p for p in muon_params if p.numel() > 0)
        self.adamw_params = tuple(p for p in adamw_params if p.numel() > 0)
        self.group_summaries = tuple(group_summaries)
        self.flat_adamw_state = flat_adamw_state
        self.flat_buffers = list(flat_buffers or ())
        self.muon = None
        self.adamw = None
        with _without_auto_prepare():  # this wrapper drives the units' lifecycle itself
            self._build(lr, weight_decay, muon_lr, adamw_lr, adamw_betas, adamw_eps, adamw_weight_decay, muon_weight_decay, muon_momentum, muon_ns_steps, muon_adjust_lr_fn)
        if self.muon is None and self.adamw is None:
            raise RuntimeError("MixedMuonAdamWOptimizer requires at least one non-empty parameter.")

    def _build(self, lr, weight_decay, muon_lr, adamw_lr, adamw_betas, adamw_eps, adamw_weight_decay, muon_weight_decay, muon_momentum, muon_ns_steps, muon_adjust_lr_fn) -> None:
        if self.muon_params:
            muon_kwargs = dict(
                lr=lr if muon_lr is None else muon_lr,
                momentum=muon_momentum,
                ns_steps=muon_ns_steps,
                weight_decay=weight_decay if muon_weight_decay is None else muon_weight_decay,
                adjust_lr_fn=muon_adjust_lr_fn,
            )
            self.muon = LazyMuon(self.muon_params, **muon_kwargs) if self.lazy_muon_init else Muon(self.muon_params, **muon_kwargs)
        if self.adamw_params:
            self.adamw = FusedAdamW(
                self.adamw_params,
                lr=lr if adamw_lr is None else adamw_lr,
                betas=adamw_betas,
                eps=adamw_eps,
                weight_decay=weight_decay if adamw_weight_decay is None else adamw_weight_decay,
            )

    @property
    def param_groups(self) -> list[dict[str, Any]]:
        groups = []
        for opt in (self.muon, self.adamw):
            if opt is not None:
                groups.extend(opt.param_groups)
        return groups

    @property
    def state(self) -> dict[Any, Any]:
        state = {}
        for opt in (self.muon, self.adamw):
            if opt is not None:
                state.update(opt.state)
        return state

    @property
    def defaults(self) -> dict[str, Any]:
        return {
            "muon": dict(self.muon.defaults) if self.muon is not None else None,
            "adamw": dict(self.adamw.defaults) if self.adamw is not None else None,
        }

    def step(self, closure=None):
        if closure is not None:
            raise NotImplementedError("MixedMuonAdamWOptimizer does not support closures.")
        prepare_units_for_step(self.fsdp_param_groups)
        if self.flat_adamw_state and self.adamw is not None and self.flat_buffers:
            initialize_flat_adamw_state(self.adamw, self.flat_buffers)
        result = None
        if self.muon is not None:
            result = self.muon.step()
        if self.adamw is not None:
            adamw_result = self.adamw.step()
            result = result if result is not None else adamw_result
        return result

    def zero_grad(self, *args: Any, **kwargs: Any) -> None:
        for opt in (self.muon, self.adamw):
            if opt is not None:
                opt.zero_grad(*args, **kwargs)

    def state_dict(self) -> dict[str, Any]:
        return {
            "muon": self.muon.state_dict() if self.muon is not None else None,
            "adamw": self.adamw.state_dict() if self.adamw is not None else None,
            "group_summaries": tuple(g.as_dict() for g in self.group_summaries),
        }

    def load_state_dict(self, state_dict: dict[str, Any]) -> None:
        if self.muon is not None and state_dict.get("muon") is not None:
            self.muon.load_state_dict(state_dict["muon"])
        if self.adamw is not None and state_dict.get("adamw") is not None:
            self.adamw.load_state_dict(state_dict["adamw"])

    def iter_named_optimizers(self) -> tuple[tuple[str, Any], ...]:
        return tuple((name, opt) for name, opt in (("muon", self.muon), ("adamw", self.adamw)) if opt is not None)

    def add_param_group(self, param_group: dict[str, Any]) -> None:
        raise NotImplementedError("MixedMuonAdamWOptimizer does not support adding param groups after construction.")

    def optimizer_group_summary(self) -> dict[str, Any]:
        return {
            "optimizer": "mixed_muon_adamw",
            "has_muon": self.muon is not None,
            "has_adamw": self.adamw is not None,
            "groups": tuple(g.as_dict() for g in self.group_summaries),
        }


def units_of(module_or_units) -> list:
    """The lifecycle units behind ``module_or_units`` (none for bare flat buffers)."""
    if isinstance(module_or_units, nn.Module) or hasattr(module_or_units, "finalize_backward"):
        return collect_param_groups(module_or_units)
    if hasattr(module_or_units, "local_param_views"):
        return []
    return [item for item in module_or_units if hasattr(item, "finalize_backward")]


def prepare_units_for_step(units, operation: str = "optimizer.step") -> None:
    for unit in units:
        unit.prepare_for_optimizer_step(operation)


class PreparedMatrixOptimizer:
    """Lifecycle hooks of the units on a regular ``torch.optim`` optimizer, which
    stays the object the user holds (matrix_fsdp/optim/wrapper.py:99-247):
    ``step()`` refuses closures and ``no_sync()``, finishes pending backwards,
    insists on sharded parameters and (opt-in) lays AdamW state out flat;
    ``zero_grad()`` refuses ``no_sync()`` and afterwards releases the units'
    reduced gradient shards.  The optimizer gains ``matrix_fsdp`` (this object),
    ``state_manager``, ``no_sync``, ``refresh_state_dtensors`` and
    ``validate_local_state_shapes``; ``remove()`` takes everything off again.
    The reference's scheduler arguments have no counterpart on one device."""

    _ATTRS = ("matrix_fsdp", "state_manager", "no_sync", "refresh_state_dtensors", "validate_local_state_shapes")

    def __init__(self, optimizer: torch.optim.Optimizer, module_or_units, *, flat_adamw_state: bool = False) -> None:
        self.optimizer = optimizer
        self._fsdp_param_groups = units_of(module_or_units)
        self.flat_adamw_state = flat_adamw_state
        self.state_manager = MatrixFSDPOptimizerStateManager(optimizer, self._fsdp_param_groups)
        self._original_zero_grad = optimizer.zero_grad
        self._removed = False
        self._handles = [optimizer.register_step_pre_hook(self._step_pre_hook)]
        optimizer.zero_grad = self._zero_grad  # type: ignore[method-assign]
        optimizer.matrix_fsdp = self  # type: ignore[attr-defined]
        optimizer.state_manager = self.state_manager  # type: ignore[attr-defined]
        optimizer.no_sync = self.no_sync  # type: ignore[attr-defined]
        optimizer.refresh_state_dtensors = self.refresh_state_dtensors  # type: ignore[attr-defined]
        optimizer.validate_local_state_shapes = self.validate_local_state_shapes  # type: ignore[attr-defined]

    @property
    def fsdp_param_groups(self) -> list:
        return self._fsdp_param_groups

    runtime_param_groups = fsdp_param_groups

    def no_sync(self):
        from ..runtime.param_group import MatrixFSDPNoSync

        return MatrixFSDPNoSync(self._fsdp_param_groups)

    def _refuse_inside_no_sync(self, operation: str) -> None:
        if any(unit.is_no_sync_active() for unit in self._fsdp_param_groups):
            raise RuntimeError(f"{operation} cannot run inside no_sync().")

    def _step_pre_hook(self, optimizer, args, kwargs) -> None:
        if kwargs.get("closure") is not None or (len(args) > 1 and args[1] is not None):
            raise NotImplementedError("MatrixFSDP prepared optimizers do not support optimizer closures yet.")
        self._refuse_inside_no_sync("optimizer.step")
        prepare_units_for_step(self._fsdp_param_groups)
        if self.flat_adamw_state:
            initialize_flat_adamw_state(self.optimizer, collect_flat_buffers(self._fsdp_param_groups))

    def _zero_grad(self, *args: Any, **kwargs: Any) -> None:
        self._refuse_inside_no_sync("optimizer.zero_grad")
        for unit in self._fsdp_param_groups:
            if unit.has_pending_backward_reduce:
                unit.finalize_backward()
        self._original_zero_grad(*args, **kwargs)
        for unit in self._fsdp_param_groups:
            if unit.flat_buffer is not None:
                unit.flat_buffer.clear_local_grad_shard()

    def remove(self) -> None:
        if self._removed:
            return
        for handle in self._handles:
            handle.remove()
        self.optimizer.zero_grad = self._original_zero_grad  # type: ignore[method-assign]
        for attr in self._ATTRS:
            if attr in vars(self.optimizer):
                delattr(self.optimizer, attr)
        self._removed = True

    # state placement metadata
    def local_state_summary(self) -> dict[str, Any]:
        return self.state_manager.local_state_summary()

    def local_state_objects(self):
        return self.state_manager.local_state_objects()

    def local_state_dtensors(self) -> dict[str, dict[str, Any]]:
        return self.state_manager.local_state_dtensors()

    @property
    def state_objects(self):
        if not self.state_manager.state_objects:
            self.state_manager.refresh_state_dtensors()
        return self.state_manager.state_objects

    @property
    def state_dtensors(self) -> dict[str, dict[str, Any]]:
        return self.state_manager.refresh_state_dtensors()

    def refresh_state_dtensors(self) -> dict[str, dict[str, Any]]:
        return self.state_manager.refresh_state_dtensors()

    def validate_local_state_shapes(self) -> None:
        self.state_manager.validate_local_state_shapes()


def prepare_matrix_optimizer(optimizer: torch.optim.Optimizer, module_or_units, **kwargs: Any) -> PreparedMatrixOptimizer:
    """Hooks the units' lifecycle onto ``optimizer`` (a second call replaces the
    first; matrix_fsdp/optim/wrapper.py:250-268)."""
    existing = getattr(optimizer, "matrix_fsdp", None)
    if isinstance(existing, PreparedMatrixOptimizer):
        existing.remove()
    return PreparedMatrixOptimizer(optimizer, module_or_units, **kwargs)


_original_optimizer_init = None
_auto_prepare_suppressed = 0


def install_matrix_optimizer_auto_prepare() -> None:
    """From now on every ``torch.optim.Optimizer`` built over parameters that a
    unit manages is prepared as by ``prepare_matrix_optimizer`` (the parameters
    carry a weak reference to their unit).  Installed once per process, by the
    first unit (matrix_fsdp/optim/wrapper.py:271-322)."""
    global _original_optimizer_init
    if _original_optimizer_init is not None:
        return
    _original_optimizer_init = torch.optim.Optimizer.__init__

    def optimizer_init(self, *args: Any, **kwargs: Any) -> None:
        _original_optimizer_init(self, *args, **kwargs)
        if _auto_prepare_suppressed or isinstance(getattr(self, "matrix_fsdp", None), PreparedMatrixOptimizer):
            return
        units, seen = [], set()
        for group in self.param_groups:
            for param in group.get("params", ()):
                ref = getattr(param, "_matrix_fsdp_param_group_ref", None)
                unit = ref() if ref is not None else None
                if unit is not None and id(unit) not in seen:
                    seen.add(id(unit))
                    units.append(unit)
        if units:
            prepare_matrix_optimizer(self, units)

    torch.optim.Optimizer.__init__ = optimizer_init  # type: ignore[method-assign]


def uninstall_matrix_optimizer_auto_prepare() -> None:
    global _original_optimizer_init
    if _original_optimizer_init is not None:
        torch.optim.Optimizer.__init__ = _original_optimizer_init  # type: ignore[method-assign]
        _original_optimizer_init = None


class _without_auto_prepare:
    """Optimizers built inside belong to a wrapper that manages the lifecycle itself."""

    def __enter__(self) -> None:
        global _auto_prepare_suppressed
        _auto_prepare_suppressed += 1

    def __exit__(self, *exc) -> None:
        global _auto_prepare_suppressed
        _auto_prepare_suppressed -= 1


def make_mixed_muon_adamw_optimizer(module_or_units, *, default_matrix_optimizer: str = "muon", default_other_optimizer: str = "adamw", **optimizer_kwargs: Any) -> MixedMuonAdamWOptimizer:
    flat_buffers = collect_flat_buffers(module_or_units)
    optimizer_kwargs.setdefault("fsdp_param_groups", units_of(module_or_units))
    classified = classify_matrix_optimizer_params(
        flat_buffers, default_matrix_optimizer=default_matrix_optimizer, default_other_optimizer=default_other_optimizer
    )
    return MixedMuonAdamWOptimizer(
        classified.muon_params, classified.adamw_params, group_summaries=classified.group_summaries, flat_buffers=flat_buffers, **optimizer_kwargs
    )


def _local_params(module_or_units) -> list[nn.Parameter]:
    params, seen = [], set()
    for fb in collect_flat_buffers(module_or_units):
        for view in fb.local_param_views:
            p = view.managed_param.param
            if id(p) not in seen and p.numel() > 0:
                seen.add(id(p))
                params.append(p)
    return params


def configure_optimizer(module_or_units, optimizer: str | MatrixOptimizerConfig = "adamw", **kwargs: Any):
    """``'adamw'`` / ``'sgd'`` / ``'muon'`` / ``'mixed_muon_adamw'`` (aliases
    ``'muon_adamw'``, ``'mixed'``) over the local parameters of the given
    flat buffers (matrix_fsdp/optim/wrapper.py:763-821)."""
    default_matrix_optimizer, default_other_optimizer = "muon", "adamw"
    optimizer_kwargs: dict[str, Any] = {}
    if isinstance(optimizer, MatrixOptimizerConfig):
        kind = optimizer.optimizer
        optimizer_kwargs.update(optimizer.kwargs)
        default_matrix_optimizer = optimizer.default_matrix_optimizer
        default_other_optimizer = optimizer.default_other_optimizer
    else:
        kind = optimizer
    optimizer_kwargs.update(kwargs)
    default_matrix_optimizer = optimizer_kwargs.pop("default_matrix_optimizer", default_matrix_optimizer)
    default_other_optimizer = optimizer_kwargs.pop("default_other_optimizer", default_other_optimizer)
    # the reference routes these to its prefetch scheduler (matrix_fsdp/optim/wrapper.py:32-51, 939-942); one device
    # has nothing to schedule, so they are taken and dropped -- all but flat_adamw_state, which is a layout choice
    flat_adamw_state = bool(optimizer_kwargs.pop("flat_adamw_state", False))
    for name in _SCHEDULER_KWARG_NAMES:
        optimizer_kwargs.pop(name, None)
    kind = kind.lower()
    if kind in ("mixed_muon_adamw", "muon_adamw", "mixed"):
        return make_mixed_muon_adamw_optimizer(
            module_or_units, default_matrix_optimizer=default_matrix_optimizer, default_other_optimizer=default_other_optimizer,
            flat_adamw_state=flat_adamw_state, **optimizer_kwargs
        )
    params = _local_params(module_or_units)
    with _without_auto_prepare():  # prepared below, for the units of module_or_units
        if kind == "adamw":
            built = FusedAdamW(params, **optimizer_kwargs)
        elif kind == "sgd":
            built = torch.optim.SGD(params, **optimizer_kwargs)
        elif kind == "muon":
            built = Muon(params, **optimizer_kwargs)
        else:
            built = None
    if built is not None:
        units = units_of(module_or_units)
        if units:
            prepare_matrix_optimizer(built, units, flat_adamw_state=flat_adamw_state and kind == "adamw")
        return built
    raise ValueError(f"optimizer must be one of 'adamw', 'sgd', 'muon', or 'mixed_muon_adamw', got {kind!r}.")


configure_matrix_optimizer = configure_optimizer


class MatrixFSDPOptimizer:
    """An optimizer together with the units whose local parameters it steps:
    the wrapper the reference hands to checkpointing
    (matrix_fsdp/optim/wrapper.py:1002-1229).  On one device the units finish
    their backward inside the autograd pass, so ``step`` has no lifecycle work
    left; what remains is the opt-in flat AdamW state and the placement
    metadata of the state tensors (``state_manager``).  The reference's
    scheduler arguments have no counterpart and are not accepted."""

    def __init__(self, optimizer, module_or_units, *, flat_adamw_state: bool = False) -> None:
        self.optimizer = optimizer
        self._fsdp_param_groups = collect_param_groups(module_or_units)
        self.flat_adamw_state = flat_adamw_state
        self.state_manager = MatrixFSDPOptimizerStateManager(optimizer, self._fsdp_param_groups)

    @classmethod
    def from_shard_hints(cls, module_or_units, *, default_matrix_optimizer: str = "muon", default_other_optimizer: str = "adamw", flat_adamw_state: bool = False, **optimizer_kwargs: Any) -> "MatrixFSDPOptimizer":
        inner = make_mixed_muon_adamw_optimizer(
            module_or_units,
            default_matrix_optimizer=default_matrix_optimizer,
            default_other_optimizer=default_other_optimizer,
            flat_adamw_state=flat_adamw_state,
            **optimizer_kwargs,
        )
        return cls(inner, module_or_units, flat_adamw_state=flat_adamw_state)

    @property
    def fsdp_param_groups(self) -> list:
        return self._fsdp_param_groups

    runtime_param_groups = fsdp_param_groups

    @property
    def param_groups(self) -> list[dict[str, Any]]:
        return self.optimizer.param_groups

    @property
    def state(self) -> dict[Any, Any]:
        return self.optimizer.state

    @property
    def defaults(self) -> dict[str, Any]:
        return self.optimizer.defaults

    def step(self, closure=None):
        if closure is not None:
            raise NotImplementedError("MatrixFSDPOptimizer V0 does not support optimizer closures.")
        prepare_units_for_step(self._fsdp_param_groups, "MatrixFSDPOptimizer.step()")
        if self.flat_adamw_state and isinstance(self.optimizer, torch.optim.Optimizer):
            initialize_flat_adamw_state(self.optimizer, collect_flat_buffers(self._fsdp_param_groups))
        result = self.optimizer.step()
        self.state_manager.refresh_state_dtensors()
        return result

    def zero_grad(self, *args: Any, **kwargs: Any) -> None:
        self.optimizer.zero_grad(*args, **kwargs)

    def state_dict(self) -> dict[str, Any]:
        return self.optimizer.state_dict()

    def load_state_dict(self, state_dict: dict[str, Any]) -> None:
        self.optimizer.load_state_dict(state_dict)

    def add_param_group(self, param_group: dict[str, Any]) -> None:
        self.optimizer.add_param_group(param_group)

    def optimizer_group_summary(self) -> dict[str, Any]:
        """wrapper.py:1172-1195."""
        if hasattr(self.optimizer, "optimizer_group_summary"):
            return self.optimizer.optimizer_group_summary()
        kind = type(self.optimizer).__name__
        groups = []
        for index, group in enumerate(self.optimizer.param_groups):
            numel = sum(p.numel() for p in group["params"] if torch.is_tensor(p))
            groups.append(
                {
                    "name": f"group_{index}",
                    "optimizer_type": kind,
                    "fqns": (),
                    "num_params": sum(1 for p in group["params"] if torch.is_tensor(p)),
                    "param_numel": numel,
                    "local_numel": numel,
                }
            )
        return {"optimizer": kind, "has_muon": False, "has_adamw": kind.lower().endswith("adamw"), "groups": tuple(groups)}

    # ------------------------------------------------------------------ state placement metadata
    def local_state_summary(self) -> dict[str, Any]:
        return self.state_manager.local_state_summary()

    def local_state_objects(self):
        return self.state_manager.local_state_objects()

    def local_state_dtensors(self) -> dict[str, dict[str, Any]]:
        return self.state_manager.local_state_dtensors()

    @property
    def state_objects(self):
        if not self.state_manager.state_objects:
            self.state_manager.refresh_state_dtensors()
        return self.state_manager.state_objects

    @property
    def state_dtensors(self) -> dict[str, dict[str, Any]]:
        return self.state_manager.refresh_state_dtensors()

    def refresh_state_dtensors(self) -> dict[str, dict[str, Any]]:
        return self.state_manager.refresh_state_dtensors()

    def validate_local_state_shapes(self) -> None:
        self.state_manager.validate_local_state_shapes()
