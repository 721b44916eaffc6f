"""``MatrixFSDPParamGroup``: the forward / backward lifecycle of one unit on a single HIP device.

A unit is a module whose parameters share one ``MatrixFlatBuffer``.  Between
steps the parameters are views of the rank's local shard (what the optimizer
updates); around the unit's forward and backward they are views of the full
buffer.  The hooks below drive that swap the way the reference's unit does
(matrix_fsdp/runtime/fsdp_unit.py:250-310 registration, :1024-1192 forward
hooks, :1384-1421 post-accumulate-grad counting, :1470-1560 backward
finalisation), with everything that needs more than one process left out:
no process group (a world of size ``W`` is simulated in memory by the flat
buffer), no prefetch scheduler, no communication streams, no offload.

States (matrix_fsdp/runtime/fsdp_unit.py:63-66):
``SHARDED`` -> pre-forward -> ``UNSHARDED`` -> post-forward ->
``FORWARD_RESHARDED`` (only with ``reshard_after_forward``) -> pre-backward ->
``UNSHARDED`` -> last gradient accumulated -> ``SHARDED`` with ``param.grad``
pointing into the reduced local gradient shard.
"""
from __future__ import annotations

import weakref
from enum import Enum
from itertools import count
from typing import Callable, Iterable, Mapping

import torch
from torch import nn
from torch.autograd import Variable

from ..core.layout import MatrixGroupLayout, ParamSegment, ShardPlan
from ..core.managed_param import ManagedParam, ManagedParamRegistry, ParamShardHint, managed_params_from_module
from ..core.plans import contiguous_even_plan, fsdp2_chunk_plan
from .flat_buffer import MatrixFlatBuffer
from .grad_bucket import BucketParamGrad, MatrixGradBucket

Planner = Callable[[list[ManagedParam], int], ShardPlan]

_MANAGED_ATTR = "_matrix_fsdp_managed"
_PARAM_GROUP_COUNTER = count()


class FSDPLifecycleState(str, Enum):
    SHARDED = "sharded"
    UNSHARDED = "unsharded"
    FORWARD_RESHARDED = "forward_resharded"


def default_planner(managed_params: list[ManagedParam], world_size: int) -> ShardPlan:
    """Per-parameter even chunks when every parameter divides by the world
    size (matrix_fsdp/planning/planner.py:428-487), otherwise the rank-contiguous
    even split of the flat buffer (planner.py:46-56)."""
    if all(mp.numel % world_size == 0 for mp in managed_params):
        return fsdp2_chunk_plan(managed_params, world_size)
    return contiguous_even_plan(managed_params[-1].end, world_size)


def _floating_tensors_to(obj, dtype: torch.dtype):
    """Floating-point tensors anywhere in ``obj`` cast to ``dtype``
    (the reference's ``cast_floating_tensors``)."""
    if isinstance(obj, torch.Tensor):
        return obj.to(dtype) if obj.is_floating_point() and obj.dtype != dtype else obj
    if isinstance(obj, (list, tuple)):
        return type(obj)(_floating_tensors_to(o, dtype) for o in obj)
    if isinstance(obj, dict):
        return {k: _floating_tensors_to(v, dtype) for k, v in obj.items()}
    return obj


def _tensors_requiring_grad(obj) -> Iterable[torch.Tensor]:
    if isinstance(obj, torch.Tensor):
        if obj.requires_grad:
            yield obj
    elif isinstance(obj, (list, tuple)):
        for o in obj:
            yield from _tensors_requiring_grad(o)
    elif isinstance(obj, dict):
        for o in obj.values():
            yield from _tensors_requiring_grad(o)


class _FullBufferView:
    """What autograd keeps in place of a tensor that lives in a unit's full
    buffer: the view's geometry relative to the buffer's first element."""

    __slots__ = ("shape", "stride", "offset")

    def __init__(self, shape: tuple[int, ...], stride: tuple[int, ...], offset: int) -> None:
        self.shape, self.stride, self.offset = shape, stride, offset


class MatrixFSDPNoSync:
    """``with model.no_sync():`` -- micro-batches whose gradients are to be
    accumulated before the next optimizer step (matrix_fsdp/runtime/fsdp_unit.py:70-97).
    On one device the "reduce" of a backward is a local copy-in, so nothing is
    deferred: every backward adds its reduced shard to the accumulated one, in
    and out of this context, and the result is what the reference reaches at
    the first backward outside it.  What the context keeps is the rule that
    ``optimizer.step()`` may not run inside it."""

    def __init__(self, units: Iterable["MatrixFSDPParamGroup"]) -> None:
        self.units = list(units)

    def __enter__(self) -> "MatrixFSDPNoSync":
        for unit in self.units:
            unit._no_sync_depth += 1
        return self

    def __exit__(self, *exc) -> None:
        for unit in self.units:
            unit._no_sync_depth -= 1


def _units_below(module: nn.Module) -> list["MatrixFSDPParamGroup"]:
    found, seen = [], set()
    for sub in module.modules():
        unit = getattr(sub, "_matrix_fsdp_param_group", None)
        if unit is not None and id(unit) not in seen:
            seen.add(id(unit))
            found.append(unit)
    return found


class MatrixFSDPParamGroup:
    def __init__(
        self,
        module: nn.Module,
        *,
        world_size: int = 1,
        rank: int = 0,
        planner: Planner | None = None,
        shard_hints: Mapping[str, ParamShardHint] | None = None,
        ignored_params: set[nn.Parameter] | None = None,
        reshard_after_forward: bool = True,
        param_dtype: torch.dtype | None = None,
        reduce_dtype: torch.dtype | None = None,
        output_dtype: torch.dtype | None = None,
        cast_forward_inputs: bool = True,
        use_saved_tensor_hooks: bool = True,
        full_param_buffer_pool=None,
        use_zero_copy_grad_bucket: bool = False,
    ) -> None:
        if world_size < 1 or not 0 <= rank < world_size:
            raise ValueError(f"rank {rank} is outside a world of {world_size}.")
        if full_param_buffer_pool is not None and full_param_buffer_pool.max_cached_per_key > 0 and not use_saved_tensor_hooks:
            # a view autograd saved in the forward would read another unit's values from the shared storage
            raise ValueError("a full_param_buffer_pool that keeps buffers needs use_saved_tensor_hooks=True.")
        self.module = module
        self.world_size = world_size
        self.rank = rank
        self.planner = planner or default_planner
        self.shard_hints = shard_hints
        self.ignored_params = set(ignored_params or ())
        self.reshard_after_forward_enabled = bool(reshard_after_forward)
        self.param_dtype = param_dtype
        self.reduce_dtype = reduce_dtype
        self.output_dtype = output_dtype
        self.cast_forward_inputs = cast_forward_inputs
        self.use_saved_tensor_hooks = use_saved_tensor_hooks
        self.full_param_buffer_pool = full_param_buffer_pool
        self.use_zero_copy_grad_bucket = use_zero_copy_grad_bucket
        self._saved_tensor_contexts: list = []
        self.saved_full_param_views = 0
        self.managed_params: list[ManagedParam] = []
        self.flat_buffer: MatrixFlatBuffer | None = None
        self.shard_plan: ShardPlan | None = None
        self.group_layout: MatrixGroupLayout | None = None
        # identifiers and mesh fields a checkpoint records (matrix_fsdp/runtime/runtime.py:47-53); one device has no
        # mesh and no replicas
        self.runtime_param_group_id = f"param_group_{next(_PARAM_GROUP_COUNTER)}"
        self.replicate_world_size = 1
        self.dp_shard_mesh_dim = 0
        self.dp_replicate_mesh_dim = None
        self.device_mesh_metadata = None
        self.lifecycle_state = FSDPLifecycleState.SHARDED
        self.events: list[str] = []
        self._handles: list = []
        self._seen_param_ids: set[int] = set()
        self._expected_param_ids: set[int] = set()
        self._backward_callback_queued = False
        self._finalized_after_backward = True
        self._in_backward = False
        self._no_sync_depth = 0
        self.init()

    # ------------------------------------------------------------------ set-up
    def init(self) -> None:
        # parameters a nested unit already manages stay with that unit
        taken = {p for p in self.module.parameters() if getattr(p, _MANAGED_ATTR, False)}
        self.managed_params = list(
            managed_params_from_module(self.module, shard_hints=self.shard_hints, ignored_params=self.ignored_params | taken)
        )
        # frozen parameters would be handed zero gradients by the reduced shard and then decayed by the optimizer;
        # the reference refuses them (fsdp_unit.py:1694-1703): pass them as ignored_params instead
        if any(not mp.param.requires_grad for mp in self.managed_params):
            raise NotImplementedError("MatrixFSDP V0 expects all managed parameters to require grad.")
        self.module._matrix_fsdp_param_group = self  # type: ignore[attr-defined]
        module = self.module
        self.module.no_sync = lambda: MatrixFSDPNoSync(_units_below(module))  # type: ignore[attr-defined]
        if not self.managed_params:
            return
        plan = self.planner(self.managed_params, self.world_size)
        if isinstance(plan, MatrixGroupLayout):  # the group planners hand back the layout form
            plan = plan.to_shard_plan()
        if len(plan.shard_sizes) != self.world_size:
            raise ValueError(f"planner returned a plan for {len(plan.shard_sizes)} ranks, expected {self.world_size}.")
        self.shard_plan = plan
        self.group_layout = MatrixGroupLayout.from_shard_plan(plan, self.managed_params)
        self.flat_buffer = MatrixFlatBuffer(
            self.managed_params, plan, self.rank, param_dtype=self.param_dtype, reduce_dtype=self.reduce_dtype,
            full_param_buffer_pool=self.full_param_buffer_pool,
        )
        buffers = list(getattr(self.module, "_matrix_fsdp_flat_buffers", ()))
        self.module._matrix_fsdp_flat_buffers = (*buffers, self.flat_buffer)  # type: ignore[attr-defined]
        me = weakref.ref(self)
        for mp in self.managed_params:
            setattr(mp.param, _MANAGED_ATTR, True)
            mp.param._matrix_fsdp_param_group_ref = me  # lets optimizers built over the parameter find their unit
            self._expected_param_ids.add(id(mp.param))
            self._handles.append(mp.param.register_post_accumulate_grad_hook(self._post_accumulate_grad))
        self._handles.append(self.module.register_forward_pre_hook(self._pre_forward, with_kwargs=True))
        # leaves the saved-tensor hooks first, and also when the forward raises
        self._handles.append(self.module.register_forward_hook(self._leave_saved_tensor_hooks, always_call=True))
        self._handles.append(self.module.register_forward_hook(self._post_forward, with_kwargs=True))
        self._record("init")
        from ..optim.wrapper import install_matrix_optimizer_auto_prepare

        install_matrix_optimizer_auto_prepare()

    def _record(self, event: str) -> None:
        self.events.append(event)
        if len(self.events) > 256:
            del self.events[:128]

    # ------------------------------------------------------------------ layout queries (fsdp_unit.py:822-850)
    @property
    def global_layout(self) -> MatrixGroupLayout | None:
        """The planner's layout.  The unit runs the plan as it comes (several
        segments per rank included), so it equals ``group_layout``: nothing is
        flat-reordered."""
        return self.group_layout

    @property
    def param_registry(self) -> ManagedParamRegistry:
        return ManagedParamRegistry(tuple(self.managed_params))

    @property
    def runtime_layout_compatibility(self):
        """How the reference's runtime would classify this unit's layout:
        ``mode`` is ``matrix_shard``, ``segment_runtime``, ``flat_reorder`` or
        ``unsupported`` (matrix_fsdp/planning/layout_validator.py:33-88).  This
        runtime executes every valid plan through one segment program, so the
        verdict is information, not a gate."""
        from ..planning.layout_validator import explain_runtime_layout_compatibility

        if self.group_layout is None:
            return None
        return explain_runtime_layout_compatibility(self.group_layout, self.managed_params, self.world_size)

    def owner_ranks(self, fqn: str) -> tuple[int, ...]:
        return self.group_layout.owner_ranks(fqn)

    def rank_segments_for_param(self, fqn: str, rank: int) -> tuple[ParamSegment, ...]:
        return self.group_layout.rank_segments_for_param(rank, fqn)

    def mixed_precision_metadata(self) -> dict[str, object]:
        """matrix_fsdp/core/mixed_precision.py:11-17."""
        name = lambda dtype: None if dtype is None else str(dtype)  # noqa: E731
        return {
            "param_dtype": name(self.param_dtype),
            "reduce_dtype": name(self.reduce_dtype),
            "output_dtype": name(self.output_dtype),
            "cast_forward_inputs": bool(self.cast_forward_inputs),
        }

    def no_sync(self) -> MatrixFSDPNoSync:
        return MatrixFSDPNoSync([self])

    @property
    def has_pending_backward_reduce(self) -> bool:
        """A backward has started on this unit and its gradients have not been reduced into the local shard yet."""
        return self._in_backward

    def is_no_sync_active(self) -> bool:
        return self._no_sync_depth > 0

    def assert_optimizer_ready(self, operation: str = "optimizer.step") -> None:
        """An optimizer may only touch the parameters while they are views of
        the local shard (matrix_fsdp/runtime/fsdp_unit.py:905-915)."""
        if self.flat_buffer is not None and self.lifecycle_state != FSDPLifecycleState.SHARDED:
            raise RuntimeError(
                f"{operation} expects MatrixFSDP parameters to be sharded, "
                f"but found lifecycle state {self.lifecycle_state.value}."
            )

    def prepare_for_optimizer_step(self, operation: str = "optimizer.step") -> None:
        """Finishes a backward that has not been finalised yet, then checks
        that the unit is sharded.  A forward whose backward has not started
        leaves the unit forward-resharded: stepping there is refused."""
        if self._no_sync_depth > 0:
            raise RuntimeError(f"{operation} cannot run inside MatrixFSDP no_sync().")
        if self.flat_buffer is None:
            return
        if self.lifecycle_state == FSDPLifecycleState.FORWARD_RESHARDED:
            raise RuntimeError(f"{operation} cannot run on a forward-resharded MatrixFSDP unit: run backward first.")
        if self._in_backward:
            self.finalize_backward()
        self.assert_optimizer_ready(operation)

    def reset_after_load(self) -> None:
        """A checkpoint load leaves the unit sharded with no backward pending."""
        self.lifecycle_state = FSDPLifecycleState.SHARDED
        self._seen_param_ids.clear()
        self._backward_callback_queued = False
        self._finalized_after_backward = True
        self._in_backward = False

    def remove_hooks(self) -> None:
        for handle in self._handles:
            handle.remove()
        self._handles.clear()

    # ------------------------------------------------------------------ shard / unshard
    def _single_rank_alias(self) -> bool:
        """A world of one with no compute-dtype cast: the local shard *is* the
        full buffer (matrix_fsdp/runtime/flat_buffer.py:320-327)."""
        fb = self.flat_buffer
        return self.world_size == 1 and fb.layout.packed_rank_shards_are_full_tensor_order and fb._param_compute_dtype() == fb.local_shard.dtype

    def unshard(self, reason: str = "manual") -> None:
        if self.flat_buffer is None or self.lifecycle_state == FSDPLifecycleState.UNSHARDED:
            return
        fb = self.flat_buffer
        if self._single_rank_alias():
            fb.full_buffer = fb.local_shard
            fb.use_full_param_buffer()
        else:
            fb.unshard()
        self.lifecycle_state = FSDPLifecycleState.UNSHARDED
        self._record(f"unshard:{reason}")

    def reshard(self, reason: str = "manual") -> None:
        if self.flat_buffer is None:
            return
        self.flat_buffer.use_local_shards()
        self.lifecycle_state = FSDPLifecycleState.SHARDED
        self._record(f"reshard:{reason}")

    # ------------------------------------------------------------------ saved tensors (fsdp_unit.py:1325-1382)
    # Autograd saves views of the parameters for the backward (``linear`` keeps ``weight.t()``), and such a view
    # pins the storage it was cut from: a full buffer "freed" after the forward would stay allocated until the
    # backward, and one handed to another unit through a buffer pool would be read back with that unit's values.
    # While the unit's forward runs, tensors that live in its full buffer are therefore saved as their geometry
    # only and rebuilt on the buffer the backward has gathered.  (torch applies only the innermost pair of
    # saved-tensor hooks, so activation checkpointing around the *inside* of a unit's forward is shadowed there.)
    def _enter_saved_tensor_hooks(self) -> None:
        context = None
        if self.use_saved_tensor_hooks and torch.is_grad_enabled() and not self._single_rank_alias():
            context = torch.autograd.graph.saved_tensors_hooks(self._pack_saved_tensor, self._unpack_saved_tensor)
            context.__enter__()
        self._saved_tensor_contexts.append(context)  # one entry per forward call, so that leaving pairs up

    def _leave_saved_tensor_hooks(self, *unused) -> None:
        if self.flat_buffer is not None and self._saved_tensor_contexts:
            context = self._saved_tensor_contexts.pop()
            if context is not None:
                context.__exit__(None, None, None)

    def _pack_saved_tensor(self, tensor: torch.Tensor):
        full = self.flat_buffer.full_buffer
        if full is None or tensor.dtype != full.dtype or tensor.device != full.device:
            return tensor
        if tensor.untyped_storage().data_ptr() != full.untyped_storage().data_ptr():
            return tensor
        self.saved_full_param_views += 1
        return _FullBufferView(tuple(tensor.shape), tuple(tensor.stride()), tensor.storage_offset() - full.storage_offset())

    def _unpack_saved_tensor(self, saved):
        if not isinstance(saved, _FullBufferView):
            return saved
        if self.lifecycle_state != FSDPLifecycleState.UNSHARDED:
            self.unshard("saved_tensor")
        full = self.flat_buffer.full_buffer
        if full is None:
            raise RuntimeError("Saved full parameter view was unpacked before full parameters were available.")
        return full.as_strided(saved.shape, saved.stride, full.storage_offset() + saved.offset)

    # ------------------------------------------------------------------ forward hooks
    def _pre_forward(self, module, args, kwargs):
        if self.flat_buffer is None:
            return args, kwargs
        self._enter_saved_tensor_hooks()  # first, so that the always-called leave hook pairs up even if this hook raises
        if self._in_backward:
            # activation checkpointing re-runs the forward in the middle of this unit's backward: the parameters
            # are (or become) full again and the bookkeeping of the backward in flight is left alone
            self.unshard("recompute")
            if self.cast_forward_inputs and self.param_dtype is not None:
                args = _floating_tensors_to(args, self.param_dtype)
                kwargs = _floating_tensors_to(kwargs, self.param_dtype)
            return args, kwargs
        if not self._finalized_after_backward and self.lifecycle_state == FSDPLifecycleState.FORWARD_RESHARDED:
            raise RuntimeError(
                "reshard_after_forward=True does not support running another forward before the previous forward has entered backward."
            )
        self._seen_param_ids.clear()
        self._record("pre_forward")
        self.unshard("pre_forward")
        if self.cast_forward_inputs and self.param_dtype is not None:
            args = _floating_tensors_to(args, self.param_dtype)
            kwargs = _floating_tensors_to(kwargs, self.param_dtype)
        return args, kwargs

    def _post_forward(self, module, args, kwargs, output):
        if self.flat_buffer is None:
            return output
        if self._in_backward:  # a recomputed forward: no reshard, no new backward hooks
            return output if self.output_dtype is None else _floating_tensors_to(output, self.output_dtype)
        grad_enabled = torch.is_grad_enabled()
        outputs_with_grad = list(_tensors_requiring_grad(output)) if grad_enabled else []
        if outputs_with_grad:
            self._finalized_after_backward = False
            for tensor in outputs_with_grad:
                tensor.register_hook(self._pre_backward)
        if self.reshard_after_forward_enabled or not outputs_with_grad:
            self.flat_buffer.use_local_shards()
            self.lifecycle_state = FSDPLifecycleState.FORWARD_RESHARDED if outputs_with_grad else FSDPLifecycleState.SHARDED
            self._record("reshard:post_forward")
        if self.output_dtype is not None:
            output = _floating_tensors_to(output, self.output_dtype)
        return output

    # ------------------------------------------------------------------ backward
    def _stash_local_grads(self) -> None:
        """Before autograd writes this backward's full gradients: the reduced
        shard of an earlier backward stays with the flat buffer if the
        parameters still point at it (this backward then adds to it, as
        ``.grad`` accumulates everywhere in torch) and is dropped if
        ``zero_grad`` has cleared them; either way ``param.grad`` is emptied, a
        local-shard view cannot receive a full gradient."""
        fb = self.flat_buffer
        if fb.local_grad_shard is not None and not fb.local_grads_are_live():
            fb.clear_local_grad_shard()
        fb.detach_param_grads()

    def _pre_backward(self, grad: torch.Tensor) -> torch.Tensor:
        if not self._backward_callback_queued:
            self._backward_callback_queued = True
            Variable._execution_engine.queue_callback(self._post_backward_callback)
        entering = not self._in_backward and not self._finalized_after_backward
        if entering:
            self._in_backward = True  # until finalize_backward
            self._stash_local_grads()
        if self.lifecycle_state != FSDPLifecycleState.UNSHARDED and not self._finalized_after_backward:
            self._record("pre_backward")
            self.unshard("pre_backward")
        if entering and self.use_zero_copy_grad_bucket and self.flat_buffer.prepare_grad_bucket():
            # the parameters are full again, so full-shaped views of the workspace can stand in as their grads:
            # autograd accumulates into the reduce-scatter input directly and no copy-in launch is needed
            self._record("zero_copy_grad_bucket")
        return grad

    def _post_accumulate_grad(self, param: torch.Tensor) -> None:
        if id(param) not in self._expected_param_ids:
            return
        self._seen_param_ids.add(id(param))
        if len(self._seen_param_ids) == len(self._expected_param_ids) and self.lifecycle_state == FSDPLifecycleState.UNSHARDED:
            self.finalize_backward()

    def _post_backward_callback(self) -> None:
        """End of the autograd pass: units whose parameters did not all receive
        a gradient are finalised here."""
        self._backward_callback_queued = False
        if not self._finalized_after_backward:
            self.finalize_backward()

    def finalize_backward(self) -> None:
        """Per-parameter grads -> reduce-scatter input -> this rank's reduced
        gradient shard; parameters and their grads become local-shard views
        again."""
        fb = self.flat_buffer
        if fb is None or self._finalized_after_backward:
            return
        bucket = fb.collect_grad_bucket()
        if bucket.has_grads:
            missing = [mp for mp in self.managed_params if all(pg.managed_param is not mp for pg in bucket.param_grads)] if bucket.param_grads else []
            if missing:
                # parameters without a gradient contribute zeros, as a reduce-scatter of an untouched workspace would
                zeros = [(mp, torch.zeros(mp.numel, dtype=bucket.param_grads[0].grad.dtype, device=fb.device)) for mp in missing]
                by_fqn = {pg.managed_param.fqn: pg for pg in bucket.param_grads}
                by_fqn.update({mp.fqn: BucketParamGrad(mp, z) for mp, z in zeros})
                ordered = tuple(by_fqn[mp.fqn] for mp in self.managed_params)
                bucket = MatrixGradBucket(ordered, bucket.total_numel, bucket.shard_sizes, bucket.rank_segments)
            accumulated = fb.local_grad_shard is not None
            fb.reduce_grad_bucket_to_local_shard(bucket, accumulate=True)
            fb.use_local_shards()
            fb.use_local_grad_shard()
            if accumulated:
                self._record("accumulate_local_grad_shard")
        else:
            fb.use_local_shards()
            if fb.local_grad_shard is not None:
                fb.use_local_grad_shard()  # nothing new: the stashed shard goes back to the parameters
        self.lifecycle_state = FSDPLifecycleState.SHARDED
        self._finalized_after_backward = True
        self._in_backward = False
        self._seen_param_ids.clear()
        self._record("finalize_backward")
