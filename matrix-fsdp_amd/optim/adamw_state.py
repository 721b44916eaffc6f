"""Flat AdamW state: both moments of every local parameter are views into
two flat buffers of ``sum(local shard numel)`` elements, laid out exactly like
the local shards themselves (matrix_fsdp/optim/adamw_state.py:44-122, 177-218).

With this layout a parameter's ``exp_avg`` / ``exp_avg_sq`` sit at
``flat_buffer_base + shard_start``, so parameters that are neighbours in a
local shard have neighbouring state and the fused kernel can take a whole
shard in one launch.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
from torch.optim.optimizer import Optimizer


@dataclass(frozen=True)
class FlatAdamWStateBuffers:
    total_numel: int
    exp_avg: torch.Tensor
    exp_avg_sq: torch.Tensor
    max_exp_avg_sq: torch.Tensor | None = None  # with amsgrad


def local_param_state_layout(flat_buffers) -> tuple[dict[int, tuple[int, int]], int]:
    """``id(param) -> (state_start, state_end)`` over the concatenation of the
    given flat buffers' local shards, and the total length.  Parameters held
    only partially, or by more than one view, get no entry
    (matrix_fsdp/optim/adamw_state.py:90-122)."""
    spans: dict[int, tuple[int, int]] = {}
    ambiguous: set[int] = set()
    base = 0
    for fb in flat_buffers:
        fb_base = base
        base += fb.local_shard.numel()
        for view in fb.local_param_views:
            param = view.managed_param.param
            pid = id(param)
            if param.numel() == 0 or view.numel != param.numel() or pid in spans:
                ambiguous.add(pid)
                continue
            spans[pid] = (fb_base + view.shard_start, fb_base + view.shard_start + view.numel)
    for pid in ambiguous:
        spans.pop(pid, None)
    return spans, base


def initialize_flat_adamw_state(optimizer: Optimizer, flat_buffers) -> bool:
    """Pre-creates ``state[p] = {step, exp_avg, exp_avg_sq[, max_exp_avg_sq]}``
    as views of flat buffers for every parameter that has a grad and no state
    yet.  Returns whether anything was initialised
    (matrix_fsdp/optim/adamw_state.py:44-87, 133-175)."""
    spans, total = local_param_state_layout(flat_buffers)
    if not spans:
        return False
    buffers: dict[tuple, FlatAdamWStateBuffers] = getattr(optimizer, "_matrix_fsdp_flat_adamw_state_buffers", None) or {}
    optimizer._matrix_fsdp_flat_adamw_state_buffers = buffers
    initialised = False
    for group in optimizer.param_groups:
        amsgrad = bool(group.get("amsgrad", False))
        for param in group["params"]:
            if param.grad is None or param.numel() == 0 or param.grad.is_sparse:
                continue
            span = spans.get(id(param))
            if span is None or len(optimizer.state[param]) != 0:
                continue
            key = (param.device.type, param.device.index, param.dtype)
            buf = buffers.get(key)
            if buf is None:
                buf = FlatAdamWStateBuffers(
                    total,
                    torch.zeros(total, device=param.device, dtype=param.dtype),
                    torch.zeros(total, device=param.device, dtype=param.dtype),
                )
                buffers[key] = buf
            elif buf.total_numel != total:
                raise RuntimeError(
                    f"Existing flat AdamW state has {buf.total_numel} elements, "
                    f"but the current MatrixFSDP optimizer layout expects {total}."
                )
            if amsgrad and buf.max_exp_avg_sq is None:
                buf = buffers[key] = FlatAdamWStateBuffers(
                    total, buf.exp_avg, buf.exp_avg_sq, torch.zeros(total, device=param.device, dtype=param.dtype)
                )
            start, end = span
            state = optimizer.state[param]
            state["step"] = torch.tensor(0.0, dtype=torch.float32)
            state["exp_avg"] = buf.exp_avg[start:end].view_as(param)
            state["exp_avg_sq"] = buf.exp_avg_sq[start:end].view_as(param)
            if amsgrad:
                state["max_exp_avg_sq"] = buf.max_exp_avg_sq[start:end].view_as(param)
            initialised = True
    return initialised
