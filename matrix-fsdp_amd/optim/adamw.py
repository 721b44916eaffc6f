"""``FusedAdamW``: AdamW on the HIP kernel, one launch per contiguous run of parameters.

Hyper-parameters, parameter-group keys and state keys (``step``, ``exp_avg``,
``exp_avg_sq``) are those of ``torch.optim.AdamW`` (``amsgrad`` and ``maximize`` included), the optimizer the reference
builds for everything Muon does not take (matrix_fsdp/optim/wrapper.py:431-439);
the arithmetic is the single-tensor path of torch/optim/adam.py:347-547.  When
the parameters are views of one flat shard and their grads views of one local
grad shard, neighbouring parameters are merged and the run is updated by a
single launch: the moments this optimizer creates for such a run are laid out
back to back as well (``initialize_flat_adamw_state`` does the same for a whole
flat buffer up front and keeps the buffers addressable).
"""
from __future__ import annotations

import torch
from torch import Tensor

from . import functional as F


class FusedAdamW(torch.optim.AdamW):
    """A ``torch.optim.AdamW`` (same constructor checks, defaults, parameter-group and state keys, so state dicts
    are interchangeable) whose ``step`` runs on the HIP kernel."""

    def __init__(
        self,
        params,
        lr: float = 1e-3,
        betas: tuple[float, float] = (0.9, 0.999),
        eps: float = 1e-8,
        weight_decay: float = 1e-2,
        amsgrad: bool = False,
        *,
        maximize: bool = False,
    ) -> None:
        if isinstance(lr, Tensor):
            raise ValueError("FusedAdamW takes a float lr")
        super().__init__(params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=bool(amsgrad), maximize=bool(maximize), foreach=False)

    def _init_states(self, params: list[Tensor], amsgrad: bool) -> None:
        """First step: parameters that follow each other in memory (views of one local shard) get moments that
        follow each other too, so that the run can be updated by one launch.  Every parameter still has its own
        ``exp_avg`` / ``exp_avg_sq`` tensors of its own shape."""
        fresh = sorted((p for p in params if len(self.state[p]) == 0), key=lambda p: p.data_ptr())
        names = ("exp_avg", "exp_avg_sq") + (("max_exp_avg_sq",) if amsgrad else ())
        start = 0
        while start < len(fresh):
            end = start + 1
            while end < len(fresh) and _follows(fresh[end - 1].data, fresh[end].data):
                end += 1
            run = fresh[start:end]
            flats = {name: torch.zeros(sum(p.numel() for p in run), dtype=run[0].dtype, device=run[0].device) for name in names}
            cursor = 0
            for p in run:
                state = self.state[p]
                state["step"] = torch.tensor(0.0, dtype=torch.float32)
                for name in names:
                    state[name] = flats[name][cursor : cursor + p.numel()].view(p.shape)
                cursor += p.numel()
            start = end

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            amsgrad = bool(group.get("amsgrad", False))
            entries = []
            active = [p for p in group["params"] if p.grad is not None and p.numel() > 0]
            for p in active:
                if p.grad.is_sparse:
                    raise RuntimeError("AdamW does not support sparse gradients")
                if p.dtype != torch.float32:
                    raise RuntimeError(f"FusedAdamW updates float32 parameters, got {p.dtype}")
            self._init_states(active, amsgrad)
            for p in active:
                state = self.state[p]
                if amsgrad and "max_exp_avg_sq" not in state:  # amsgrad switched on after the first step
                    state["max_exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                state["step"] += 1
                tensors = [p.data, p.grad.contiguous(), state["exp_avg"], state["exp_avg_sq"]]
                if amsgrad:
                    tensors.append(state["max_exp_avg_sq"])
                entries.append((*tensors, int(state["step"].item())))
            for *tensors, step in _merge_contiguous(entries):
                F.adamw_step(
                    *tensors[:4], step,
                    lr=group["lr"], betas=group["betas"], eps=group["eps"], weight_decay=group["weight_decay"],
                    max_exp_avg_sq=tensors[4] if amsgrad else None, maximize=bool(group.get("maximize", False)),
                )
        return loss


def _follows(prev: Tensor, nxt: Tensor) -> bool:
    return (
        prev.dtype == nxt.dtype
        and prev.device == nxt.device
        and prev.is_contiguous()
        and nxt.is_contiguous()
        and prev.untyped_storage().data_ptr() == nxt.untyped_storage().data_ptr()
        and prev.data_ptr() + prev.numel() * prev.element_size() == nxt.data_ptr()
    )


def _merge_contiguous(entries):
    """Merges neighbours whose parameter, grad and moments each continue the
    previous entry's memory inside one storage (and share a step count) into
    one flat update.  Yields ``(param, grad, exp_avg, exp_avg_sq[, max_exp_avg_sq], step)``
    as 1-D spans."""
    runs: list[dict] = []
    for tensors_and_step in sorted(entries, key=lambda e: e[0].data_ptr()):
        tensors, step = tensors_and_step[:-1], tensors_and_step[-1]
        if runs:
            run = runs[-1]
            if run["step"] == step and all(_follows(a, b) for a, b in zip(run["last"], tensors)):
                run["numel"] += tensors[0].numel()
                run["last"] = tensors
                continue
        runs.append({"first": tensors, "last": tensors, "numel": tensors[0].numel(), "step": step})
    for run in runs:
        yield (*(_flat_span(t, run["numel"]) for t in run["first"]), run["step"])


def _flat_span(first: Tensor, numel: int) -> Tensor:
    """1-D view of ``numel`` elements starting at ``first``'s first element."""
    if first.numel() == numel:
        return first.reshape(-1)
    return torch.as_strided(first, (numel,), (1,), first.storage_offset())
