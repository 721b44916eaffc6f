"""``MatrixFlatBuffer``: one unit's flat parameter buffer on a single HIP device.

Host-side mirror of the copy / view half of the reference's
``MatrixFlatBuffer`` (matrix_fsdp/runtime/flat_buffer.py:95-1480): it owns the
local shard, materialises the full buffer, swaps ``param.data`` between
local-shard views and full-buffer views and turns per-parameter grads into
the rank's reduced grad shard.  Every byte is moved by a segment program (one
HIP launch per buffer); there is no slice-loop fallback.

The world of size ``W`` is *simulated in memory*: no process group exists, so
the gathered buffer an all-gather would deliver is built from ``world_shards``
(every rank's shard, kept by this object) and the reduce-scatter of the
gradient workspace degrades to taking this rank's chunk, exactly as the
reference does without a process group
(matrix_fsdp/runtime/collectives.py:216-219, 939-946).  Scheduling, buffer
pools, collectives and the lifecycle state machine are not part of this
object.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..core.layout import LayoutSegment, ShardPlan, validate_shard_plan
from ..core.managed_param import ManagedParam
from ..core.placement import MatrixShard, explain_matrix_shard_compatibility, shard_sizes_to_matrix_local_units
from ..core.state import MatrixShardedState
from ..kernels import native
from ..kernels.segment_program import (
    SegmentProgram,
    compact_owner_program,
    pack_program,
    take_local_segments_program,
    unpack_program,
)
from .grad_bucket import (
    BucketParamGrad,
    CopyInBackend,
    CopyInProgramCache,
    MatrixGradBucket,
    classify_copy_in_layout,
    fill_reduce_scatter_input,
)
from .param_buffer_layout import ParamBufferLayout, rank_chunk_shard_sizes


@dataclass
class LocalParamView:
    """The part of a parameter this rank holds
    (matrix_fsdp/runtime/flat_buffer.py:54-64)."""

    managed_param: ManagedParam
    param_start: int
    param_end: int
    shard_start: int
    shard_end: int

    @property
    def numel(self) -> int:
        return self.param_end - self.param_start


class MatrixFlatBuffer:
    def __init__(
        self,
        managed_params: list[ManagedParam],
        plan: ShardPlan,
        rank: int,
        *,
        divide_grads_by_world: bool = True,
        param_dtype: torch.dtype | None = None,
        reduce_dtype: torch.dtype | None = None,
        keep_world_shards: bool = True,
        full_param_buffer_pool=None,
    ) -> None:
        if not managed_params:
            raise ValueError("MatrixFlatBuffer needs at least one parameter.")
        validate_shard_plan(plan)
        if not 0 <= rank < len(plan.shard_sizes):
            raise ValueError(f"rank {rank} is outside the plan's world of {len(plan.shard_sizes)}.")
        first = managed_params[0]
        for mp in managed_params:
            if mp.dtype != first.dtype:
                raise NotImplementedError("MatrixFSDP V0 only supports one dtype per unit.")
            if mp.device != first.device:
                raise NotImplementedError("MatrixFSDP V0 only supports one device per unit.")
        if first.device.type != "cuda":
            raise RuntimeError("MatrixFlatBuffer runs on a HIP device; move the module there first.")
        if managed_params[-1].end != plan.total_numel:
            raise RuntimeError(f"Full tensor has {managed_params[-1].end} elements, expected {plan.total_numel}.")
        self.managed_params = list(managed_params)
        self.plan = plan
        self.rank = rank
        self.device = first.device
        self.divide_grads_by_world = divide_grads_by_world
        self.param_dtype = param_dtype
        self.reduce_dtype = reduce_dtype
        self.shard_sizes = tuple(plan.shard_sizes)
        self.layout = ParamBufferLayout.from_plan(plan)
        self.local_start = plan.rank_packed_offset(rank)
        self.local_end = self.local_start + self.shard_sizes[rank]
        self.local_segments: tuple[LayoutSegment, ...] = plan.local_segments(rank)
        self._programs: dict[tuple, SegmentProgram] = {}
        self._copy_in_cache = CopyInProgramCache()
        self._packed_grad_offset_cache: dict[bool, dict[str, int | None]] = {}

        # initial pack: cat(params) -> compact rank-major shards (flat_buffer.py:240-243)
        full = torch.cat([mp.param.detach().reshape(-1) for mp in self.managed_params])
        world = torch.empty(sum(self.shard_sizes), dtype=full.dtype, device=self.device)
        self._program("pack_compact", full.dtype).run((full,), world)
        self.world_shards: torch.Tensor | None = world if keep_world_shards else None
        self.local_shard = world[self.local_start : self.local_end] if keep_world_shards else world[self.local_start : self.local_end].clone()
        self.full_buffer: torch.Tensor | None = None
        self.full_param_buffer_pool = full_param_buffer_pool
        self._full_buffer_pooled = False
        self.local_grad_shard: torch.Tensor | None = None
        self.grad_bucket_input: torch.Tensor | None = None
        self.grad_bucket_input_is_compact = False
        self.local_param_views = self._build_local_param_views()
        # placement of the local shard in the flat buffer; plans a MatrixShard cannot express (several segments per
        # rank) keep the shard sizes in lowest terms, as the reference does (flat_buffer.py:143-165)
        self.matrix_shard_compatibility = explain_matrix_shard_compatibility(plan)
        self.matrix_shard = MatrixShard((0,), shard_sizes_to_matrix_local_units(self.shard_sizes))
        self.param_state = self._make_sharded_state("param", self.local_shard, self.matrix_shard, (plan.total_numel,))
        self.use_local_shards()

    # ------------------------------------------------------------------ sharded-state metadata
    @property
    def local_numel(self) -> int:
        return self.local_end - self.local_start

    @property
    def placement(self) -> MatrixShard:
        return self.matrix_shard

    @property
    def grad_state(self) -> MatrixShardedState | None:
        if self.local_grad_shard is None:
            return None
        return self._make_sharded_state("grad", self.local_grad_shard, self.matrix_shard, (self.plan.total_numel,))

    def _make_sharded_state(self, name: str, local_tensor: torch.Tensor, placement: MatrixShard | None, global_shape: tuple[int, ...]) -> MatrixShardedState:
        return MatrixShardedState(name, local_tensor, placement=placement, global_shape=global_shape, global_stride=(1,), requires_grad=local_tensor.requires_grad)

    def param_shard_sizes(self, mp: ManagedParam) -> tuple[int, ...]:
        """Elements of ``mp`` each rank holds (flat_buffer.py:1441-1451)."""
        return tuple(
            sum(max(0, min(mp.end, seg.global_end) - max(mp.offset, seg.global_start)) for seg in segments)
            for segments in self.plan.rank_segments
        )

    def param_matrix_shard(self, mp: ManagedParam) -> MatrixShard | None:
        """The parameter's own placement, when the ranks hold it as rank-ordered
        contiguous pieces (flat_buffer.py:1433-1471)."""
        cursor = 0
        for segments in self.plan.rank_segments:
            pieces = [(max(mp.offset, seg.global_start), min(mp.end, seg.global_end)) for seg in segments]
            pieces = [(a - mp.offset, b - mp.offset) for a, b in pieces if a < b]
            if not pieces:
                continue
            if len(pieces) != 1 or pieces[0][0] != cursor:
                return None
            cursor = pieces[0][1]
        if cursor != mp.numel or mp.numel == 0:
            return None
        return MatrixShard((0,), shard_sizes_to_matrix_local_units(self.param_shard_sizes(mp)))

    def make_param_state(self, mp: ManagedParam, name: str, local_tensor: torch.Tensor) -> MatrixShardedState | None:
        """Metadata view of a shard-shaped tensor that belongs to ``mp`` (an
        optimizer moment, say); ``None`` when the parameter has no placement
        (flat_buffer.py:1417-1427)."""
        placement = self.param_matrix_shard(mp)
        if placement is None:
            return None
        return self._make_sharded_state(name, local_tensor.view(-1), placement, (mp.numel,))

    # ------------------------------------------------------------------ programs
    def _program(self, kind: str, dtype: torch.dtype, out_dtype: torch.dtype | None = None) -> SegmentProgram:
        key = (kind, dtype, out_dtype)
        program = self._programs.get(key)
        if program is None:
            if kind == "pack_compact":
                program = pack_program(self.plan, dtype, padded=False, out_dtype=out_dtype, device=self.device)
            elif kind == "pack_padded":
                program = pack_program(self.plan, dtype, padded=True, out_dtype=out_dtype, device=self.device)
            elif kind == "unpack_compact":
                program = unpack_program(self.plan, dtype, padded=False, out_dtype=out_dtype, device=self.device)
            elif kind == "unpack_padded":
                program = unpack_program(self.plan, dtype, padded=True, out_dtype=out_dtype, device=self.device)
            elif kind == "take_local":
                program = take_local_segments_program(
                    self.local_segments, self.plan.total_numel, self.local_numel, dtype, out_dtype=out_dtype, device=self.device
                )
            else:
                raise KeyError(kind)
            self._programs[key] = program
        return program

    # ------------------------------------------------------------------ dtypes (flat_buffer.py:1186-1206)
    def _param_compute_dtype(self) -> torch.dtype:
        return self.param_dtype or self.local_shard.dtype

    def _maybe_to_param_dtype(self, tensor: torch.Tensor) -> torch.Tensor:
        return native.cast(tensor, self._param_compute_dtype())

    def _maybe_to_reduce_dtype(self, tensor: torch.Tensor) -> torch.Tensor:
        return tensor if self.reduce_dtype is None else native.cast(tensor, self.reduce_dtype)

    def _maybe_to_local_dtype(self, tensor: torch.Tensor) -> torch.Tensor:
        return native.cast(tensor, self.local_shard.dtype)

    # ------------------------------------------------------------------ views
    def _build_local_param_views(self) -> list[LocalParamView]:
        views = []
        for mp in self.managed_params:
            for seg in self.local_segments:
                start, end = max(mp.offset, seg.global_start), min(mp.end, seg.global_end)
                if start < end:
                    shard_start = seg.local_start + start - seg.global_start
                    views.append(LocalParamView(mp, start - mp.offset, end - mp.offset, shard_start, shard_start + end - start))
        return views

    def _local_views_by_param(self) -> dict[str, list[LocalParamView]]:
        by_param: dict[str, list[LocalParamView]] = {}
        for view in self.local_param_views:
            by_param.setdefault(view.managed_param.fqn, []).append(view)
        return by_param

    def use_local_shards(self) -> None:
        """``param.data`` -> view of the local shard: whole parameters keep
        their shape, partial ones are 1-D slices, absent ones are empty
        (flat_buffer.py:269-299)."""
        by_param = self._local_views_by_param()
        for mp in self.managed_params:
            views = by_param.get(mp.fqn)
            if views is None:
                mp.param.data = self.local_shard.new_empty(0)
            elif len(views) != 1:
                raise NotImplementedError("MatrixFSDP V0 cannot expose multi-segment parameters yet.")
            else:
                view = views[0]
                data = self.local_shard[view.shard_start : view.shard_end]
                mp.param.data = data.view(mp.shape) if view.numel == mp.numel else data
        self.clear_full_params()

    def use_full_param_buffer(self) -> None:
        """``param.data`` -> zero-copy view of the full buffer (flat_buffer.py:413-425)."""
        if self.full_buffer is None:
            raise RuntimeError("Full parameter buffer is not materialized.")
        for mp in self.managed_params:
            mp.param.data = self.full_buffer[mp.offset : mp.end].view(mp.shape)

    def param_data_alias_full_buffer(self) -> bool:
        if self.full_buffer is None:
            return False
        base, size = self.full_buffer.data_ptr(), self.full_buffer.element_size()
        return all(mp.param.data.data_ptr() == base + mp.offset * size for mp in self.managed_params)

    def param_data_alias_local_shard(self) -> bool:
        base, size = self.local_shard.data_ptr(), self.local_shard.element_size()
        by_param = self._local_views_by_param()
        return all(mp.param.data.data_ptr() == base + by_param[mp.fqn][0].shard_start * size for mp in self.managed_params if mp.fqn in by_param)

    # ------------------------------------------------------------------ copy-out
    def gathered_padded_shards(self, out: torch.Tensor | None = None) -> torch.Tensor:
        """What the padded all-gather would deliver: ``[W*max_shard]`` in the
        parameter compute dtype, slot ``r`` holding rank ``r``'s shard and a
        zero tail (runtime/collectives.py:236-241).  Built in one launch from
        the simulated world's shards."""
        if self.world_shards is None:
            raise RuntimeError("world shards were not kept; construct with keep_world_shards=True.")
        dtype = self._param_compute_dtype()
        if out is None:
            out = torch.empty(self.layout.padded_numel, dtype=dtype, device=self.device)
        key = ("pad_world", self.world_shards.dtype, dtype)
        program = self._programs.get(key)
        if program is None:
            contiguous = ShardPlan(sum(self.shard_sizes), self.shard_sizes, tuple(self.plan.rank_packed_offset(r) for r in range(len(self.shard_sizes))))
            program = pack_program(contiguous, self.world_shards.dtype, padded=True, out_dtype=dtype, device=self.device)
            self._programs[key] = program
        return program.run((self.world_shards,), out)

    def unshard(self, gathered_padded: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
        """Materialises the full buffer from the gathered padded shards
        (un-pad + unpack fused, one launch) and points every parameter at
        it."""
        pool = self.full_param_buffer_pool
        if gathered_padded is None:
            gathered_padded = self.gathered_padded_shards()
        dtype = gathered_padded.dtype
        self.clear_full_params()
        pooled = False
        if out is None:
            if pool is not None:
                out, pooled = pool.acquire(gathered_padded, self.plan.total_numel), True
            else:
                out = torch.empty(self.plan.total_numel, dtype=dtype, device=self.device)
        self._program("unpack_padded", dtype).run((gathered_padded,), out)
        self.full_buffer = out
        self._full_buffer_pooled = pooled
        self.use_full_param_buffer()
        return out

    def gather_full_params(self) -> torch.Tensor:
        """The full flat buffer in the local shard's dtype, assembled from the
        current shards without touching ``param.data`` or ``full_buffer``
        (what a checkpoint's ``full_state`` stores)."""
        if self.world_shards is None:
            raise RuntimeError("world shards were not kept; construct with keep_world_shards=True.")
        return self._unpack_rank_shards_to_full_tensor(self.world_shards)

    def gather_full_grads(self) -> torch.Tensor:
        """The reduced gradient over the full flat buffer.  Only this rank's
        gradient shard exists in a simulated world, so the other ranks' slots
        are zero; with one rank this is the whole gradient."""
        if self.local_grad_shard is None:
            raise RuntimeError("Cannot build full gradients before local grad shard exists.")
        packed = self.local_grad_shard.new_zeros(sum(self.shard_sizes))
        if self.local_numel:
            native.copy_range(self.local_grad_shard, packed[self.local_start : self.local_end], 0)
        return self._unpack_rank_shards_to_full_tensor(packed)

    def local_shard_from_full(self, full_tensor: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """This rank's shard of a full flat tensor, cast to the local dtype in
        the same launch when the dtypes differ (bf16 or fp16 <-> fp32)."""
        full_tensor = full_tensor.reshape(-1)
        if full_tensor.numel() != self.plan.total_numel:
            raise ValueError(f"Full tensor has {full_tensor.numel()} elements, expected {self.plan.total_numel}.")
        if out is None:
            out = torch.empty(self.local_numel, dtype=self.local_shard.dtype, device=self.device)
        if self.local_numel == 0:
            return out
        out_dtype = None if out.dtype == full_tensor.dtype else out.dtype
        return self._program("take_local", full_tensor.dtype, out_dtype).run((full_tensor,), out)

    def load_full_params(self, full_tensor: torch.Tensor) -> None:
        """Re-shards a full flat tensor into this buffer: every simulated
        rank's shard when the world is kept, else this rank's."""
        full_tensor = full_tensor.reshape(-1)
        if full_tensor.numel() != self.plan.total_numel:
            raise ValueError(f"Full tensor has {full_tensor.numel()} elements, expected {self.plan.total_numel}.")
        if self.world_shards is None:
            self.local_shard_from_full(full_tensor, out=self.local_shard)
            return
        out_dtype = None if full_tensor.dtype == self.world_shards.dtype else self.world_shards.dtype
        self._program("pack_compact", full_tensor.dtype, out_dtype).run((full_tensor,), self.world_shards)

    def clear_full_params(self) -> None:
        """Drops the full buffer; one that came from the pool goes back to it.
        The parameters must not point into it any more."""
        if self.full_buffer is not None and self._full_buffer_pooled and self.full_param_buffer_pool is not None:
            self.full_param_buffer_pool.release(self.full_buffer)
        self.full_buffer = None
        self._full_buffer_pooled = False

    def clear_local_grad_shard(self) -> None:
        self.local_grad_shard = None
        self.grad_bucket_input = None

    def _pack_full_tensor_by_rank_segments(self, full_tensor: torch.Tensor) -> torch.Tensor:
        """flat_buffer.py:1304-1316."""
        full_tensor = full_tensor.reshape(-1)
        if full_tensor.numel() != self.plan.total_numel:
            raise RuntimeError(f"Full tensor has {full_tensor.numel()} elements, expected {self.plan.total_numel}.")
        packed = full_tensor.new_empty(sum(self.shard_sizes))
        return self._program("pack_compact", full_tensor.dtype).run((full_tensor,), packed)

    def _unpack_rank_shards_to_full_tensor(self, rank_shards: torch.Tensor) -> torch.Tensor:
        """flat_buffer.py:1318-1333, including the identity shortcut that
        returns the input itself."""
        rank_shards = rank_shards.reshape(-1)
        expected = sum(self.shard_sizes)
        if rank_shards.numel() != expected:
            raise RuntimeError(f"Packed rank shards have {rank_shards.numel()} elements, expected {expected}.")
        if self.layout.packed_rank_shards_are_full_tensor_order:
            return rank_shards
        full = rank_shards.new_empty(self.plan.total_numel)
        return self._program("unpack_compact", rank_shards.dtype).run((rank_shards,), full)

    # ------------------------------------------------------------------ grad copy-in
    def collect_grad_bucket(self) -> MatrixGradBucket:
        """Takes every parameter's ``.grad`` (flat_buffer.py:589-621).  The
        reduce-dtype cast is folded into the copy-in launch instead of being
        applied per grad."""
        workspace = self.grad_bucket_input
        if workspace is not None:
            # zero-copy bucket: autograd has accumulated into views of the workspace, which then already is the
            # reduce-scatter input (flat_buffer.py:447-486, 589-621).  A grad that was replaced instead of added to
            # (create_graph, a hook) sends everything down the copy path.
            offsets = self._packed_grad_offsets(compact=self.grad_bucket_input_is_compact)
            base, size = workspace.data_ptr(), workspace.element_size()
            in_place = all(
                mp.param.grad is not None and mp.param.grad.dtype == workspace.dtype and mp.param.grad.data_ptr() == base + offsets[mp.fqn] * size
                for mp in self.managed_params
            )
            self.grad_bucket_input = None
            if in_place:
                for mp in self.managed_params:
                    mp.param.grad = None
                return MatrixGradBucket((), self.plan.total_numel, self.shard_sizes, self.plan.rank_segments, packed_input=workspace, packed_input_is_compact=self.grad_bucket_input_is_compact)
        param_grads = []
        for mp in self.managed_params:
            grad = mp.param.grad
            if grad is None:
                continue
            param_grads.append(BucketParamGrad(mp, grad.detach().reshape(-1)))
            mp.param.grad = None
        return MatrixGradBucket(tuple(param_grads), self.plan.total_numel, self.shard_sizes, self.plan.rank_segments)

    def fill_reduce_scatter_input(self, bucket: MatrixGradBucket, packed: torch.Tensor | None = None, *, backend: CopyInBackend = "auto") -> torch.Tensor:
        if packed is None:
            dtype = self.reduce_dtype or bucket.param_grads[0].grad.dtype
            packed = torch.empty(self.layout.padded_numel, dtype=dtype, device=self.device)
        return fill_reduce_scatter_input(bucket, packed, backend=backend, cache=self._copy_in_cache)

    def _compute_packed_grad_offset_for_param(self, mp: ManagedParam, *, compact: bool = False) -> int | None:
        """flat_buffer.py:1274-1302."""
        max_shard = self.layout.max_shard_size
        cursor, start, end = 0, None, None
        for rank, segments in enumerate(self.plan.rank_segments):
            for seg in segments:
                g0, g1 = max(mp.offset, seg.global_start), min(mp.end, seg.global_end)
                if g0 >= g1:
                    continue
                if g0 - mp.offset != cursor:
                    return None
                base = self.plan.rank_packed_offset(rank) if compact else rank * max_shard
                cur = base + seg.local_start + g0 - seg.global_start
                if start is None:
                    start = cur
                elif end != cur:
                    return None
                end = cur + (g1 - g0)
                cursor = g1 - mp.offset
        if start is None or cursor != mp.numel:
            return None
        return start

    def _packed_grad_offsets(self, *, compact: bool) -> dict[str, int | None]:
        cached = self._packed_grad_offset_cache.get(compact)
        if cached is None:
            cached = {mp.fqn: self._compute_packed_grad_offset_for_param(mp, compact=compact) for mp in self.managed_params}
            self._packed_grad_offset_cache[compact] = cached
        return cached

    def is_whole_param_owner_layout(self) -> bool:
        """Every rank holds one contiguous chunk made of whole parameters."""
        return rank_chunk_shard_sizes(self.plan.rank_segments) is not None and all(
            off is not None for off in self._packed_grad_offsets(compact=True).values()
        )

    def _fill_compact_owner_reduce_scatter_input(self, bucket: MatrixGradBucket, packed_rank_chunks: torch.Tensor) -> torch.Tensor:
        """flat_buffer.py:1232-1252 as one launch (zero fill included)."""
        expected = self.layout.rank_chunk_workspace_numel(compact=True)
        if packed_rank_chunks.ndim != 1:
            raise ValueError(f"packed_rank_chunks must be 1D, got shape {tuple(packed_rank_chunks.shape)}.")
        if packed_rank_chunks.numel() != expected:
            raise ValueError(f"packed_rank_chunks has {packed_rank_chunks.numel()} elements, expected {expected}.")
        offsets = self._packed_grad_offsets(compact=True)
        params, grads, offs = [], [], []
        for pg in bucket.param_grads:
            mp, grad = pg.managed_param, pg.grad.reshape(-1)
            if grad.numel() != mp.numel:
                raise RuntimeError(f"Gradient for {mp.fqn} has {grad.numel()} elements, expected {mp.numel}.")
            if offsets.get(mp.fqn) is None:
                raise RuntimeError(f"Gradient for {mp.fqn} cannot be packed into compact owner rank chunks.")
            params.append(mp)
            grads.append(grad)
            offs.append(offsets[mp.fqn])
        if not grads:
            return packed_rank_chunks.zero_()
        key = ("compact_owner", grads[0].dtype, packed_rank_chunks.dtype, tuple(mp.fqn for mp in params))
        program = self._programs.get(key)
        if program is None:
            program = compact_owner_program(params, offs, expected, grads[0].dtype, packed_rank_chunks.dtype, device=self.device)
            self._programs[key] = program
        return program.run(grads, packed_rank_chunks)

    def reduce_grad_bucket_to_local_shard(self, bucket: MatrixGradBucket, *, backend: CopyInBackend = "auto", accumulate: bool = False) -> torch.Tensor:
        """Copy-in, then this rank's chunk of the workspace as the local grad
        shard in the local dtype.  Without a process group the reduce-scatter
        is the identity on the rank's chunk (runtime/collectives.py:939-946);
        grads are therefore not divided by the world size.  ``accumulate`` adds
        the result to the shard a previous backward left
        (flat_buffer.py:886-900) instead of replacing it."""
        reduce_dtype = self.reduce_dtype or (bucket.param_grads[0].grad.dtype if bucket.param_grads else self.local_shard.dtype)
        compact = self.is_whole_param_owner_layout() and backend == "auto"
        if bucket.packed_input is not None:
            packed, compact = bucket.packed_input, bucket.packed_input_is_compact
        elif compact:
            packed = torch.empty(self.layout.rank_chunk_workspace_numel(compact=True), dtype=reduce_dtype, device=self.device)
            self._fill_compact_owner_reduce_scatter_input(bucket, packed)
        else:
            packed = torch.empty(self.layout.padded_numel, dtype=reduce_dtype, device=self.device)
            fill_reduce_scatter_input(bucket, packed, backend=backend, cache=self._copy_in_cache)
        offset = self.plan.rank_packed_offset(self.rank) if compact else self.rank * self.layout.max_shard_size
        if offset == 0 and packed.numel() == self.shard_sizes[self.rank]:
            chunk = packed  # a world of one: the workspace is the shard, no second pass over the gradients
        else:
            chunk = torch.empty(self.shard_sizes[self.rank], dtype=packed.dtype, device=self.device)
            native.copy_range(packed, chunk, offset)
        reduced = self._maybe_to_local_dtype(chunk)
        if accumulate and self.local_grad_shard is not None:
            self.accumulate_local_grad_shard(reduced)
        else:
            self.local_grad_shard = reduced
        return self.local_grad_shard

    def accumulate_local_grad_shard(self, local_grad_shard: torch.Tensor) -> bool:
        """Adds a freshly reduced shard to the one already held; returns
        whether there was one (flat_buffer.py:886-900)."""
        existing = self.local_grad_shard
        if existing is None:
            self.local_grad_shard = local_grad_shard.reshape(-1)
            return False
        if existing.numel() != local_grad_shard.numel():
            raise RuntimeError(f"Accumulated local grad shard has {existing.numel()} elements, new local grad shard has {local_grad_shard.numel()}.")
        if existing.dtype != local_grad_shard.dtype:
            local_grad_shard = native.cast(local_grad_shard.contiguous(), existing.dtype)
        if existing.numel():
            native.accumulate(existing, local_grad_shard.reshape(-1).contiguous())
        return True

    def local_grads_are_live(self) -> bool:
        """Whether some local parameter's ``.grad`` still is a view of the local
        grad shard (``zero_grad`` has not dropped them)."""
        if self.local_grad_shard is None:
            return False
        storage = self.local_grad_shard.untyped_storage().data_ptr()
        return any(
            mp.param.grad is not None and mp.param.grad.untyped_storage().data_ptr() == storage
            for mp in self.managed_params
        )

    def detach_param_grads(self) -> None:
        """``param.grad = None`` everywhere; the shard itself stays with the buffer."""
        for mp in self.managed_params:
            mp.param.grad = None

    def use_local_grad_shard(self, local_grad_shard: torch.Tensor | None = None) -> None:
        """``param.grad`` -> views of the reduced local grad shard, which a
        caller may hand in (flat_buffer.py:860-884)."""
        if local_grad_shard is not None:
            if local_grad_shard.numel() != self.local_numel:
                raise ValueError(f"Local grad shard has {local_grad_shard.numel()} elements, expected {self.local_numel}.")
            self.local_grad_shard = local_grad_shard.reshape(-1)
        if self.local_grad_shard is None:
            raise RuntimeError("Local gradient shard is not available.")
        by_param = self._local_views_by_param()
        for mp in self.managed_params:
            views = by_param.get(mp.fqn)
            if views is None:
                mp.param.grad = None
                continue
            view = views[0]
            grad = self.local_grad_shard[view.shard_start : view.shard_end]
            mp.param.grad = grad.view(mp.shape) if view.numel == mp.numel else grad

    def prepare_grad_bucket(self) -> bool:
        """Zero-copy bucket: allocate the workspace and point ``param.grad`` at
        views of it so that autograd writes in place; declined when the
        parameter dtype differs from the local shard's or a parameter is not
        one contiguous run of the workspace (flat_buffer.py:447-486)."""
        if self._param_compute_dtype() != self.local_shard.dtype or self.layout.max_shard_size == 0:
            return False
        if self.reduce_dtype is not None and self.reduce_dtype != self.local_shard.dtype:
            return False  # the workspace would have to be in the reduce dtype, which autograd cannot write into
        compact = self.is_whole_param_owner_layout()
        offsets = self._packed_grad_offsets(compact=compact)
        if any(off is None for off in offsets.values()):
            return False
        numel = self.layout.rank_chunk_workspace_numel(compact=compact)
        self.grad_bucket_input = torch.zeros(numel, dtype=self.local_shard.dtype, device=self.device)
        self.grad_bucket_input_is_compact = compact
        for mp in self.managed_params:
            off = offsets[mp.fqn]
            mp.param.grad = self.grad_bucket_input[off : off + mp.numel].view(mp.shape)
        return True

    def communication_summary(self) -> dict[str, object]:
        summary = self.layout.as_summary()
        summary["copy_in_layout_kind"] = classify_copy_in_layout(
            MatrixGradBucket(
                tuple(BucketParamGrad(mp, torch.empty(mp.numel, device="meta")) for mp in self.managed_params),
                self.plan.total_numel,
                self.shard_sizes,
                self.plan.rank_segments,
            )
        )
        return summary
