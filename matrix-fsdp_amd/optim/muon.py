"""``Muon``: drop-in for ``torch.optim.Muon`` running on the HIP kernels.

Constructor arguments, validation messages, parameter-group keys and the
per-parameter state (``momentum_buffer = zeros_like(grad)``) follow
torch/optim/_muon.py:87-202, which is the optimizer the reference
instantiates for owner-rank matrices (matrix_fsdp/optim/wrapper.py:416-429).
``step()`` runs momentum, Newton-Schulz and the parameter update of every
matrix through ``mfsdp_muon_step_ex`` (independent matrices side by side where
that pays); nothing falls back to torch arithmetic.
"""
from __future__ import annotations

import torch

from . import functional as F

EPS = F.NS_EPS
DEFAULT_A, DEFAULT_B, DEFAULT_C = F.NS_COEFFICIENTS
DEFAULT_NS_STEPS = F.NS_STEPS


class Muon(torch.optim.Muon):
    """A ``torch.optim.Muon`` (same constructor checks, defaults and state) whose ``step`` runs on the HIP kernels."""

    def __init__(
        self,
        params,
        lr: float = 1e-3,
        weight_decay: float = 0.1,
        momentum: float = 0.95,
        nesterov: bool = True,
        ns_coefficients: tuple[float, float, float] = (DEFAULT_A, DEFAULT_B, DEFAULT_C),
        eps: float = EPS,
        ns_steps: int = DEFAULT_NS_STEPS,
        adjust_lr_fn: str | None = None,
    ) -> None:
        super().__init__(
            params, lr=lr, weight_decay=weight_decay, momentum=momentum, nesterov=nesterov, ns_coefficients=ns_coefficients,
            eps=eps, ns_steps=ns_steps, adjust_lr_fn=adjust_lr_fn,
        )
        self._workspace: F.MuonWorkspace | None = None

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        jobs = []
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None:
                    continue
                if torch.is_complex(p):
                    raise RuntimeError("Muon does not support complex parameters")
                if p.grad.is_sparse:
                    raise RuntimeError("Muon does not support sparse gradients")
                grad = p.grad
                if grad.ndim != 2:
                    raise ValueError("Param gradient must be a 2D matrix")
                state = self.state[p]
                if "momentum_buffer" not in state:
                    state["momentum_buffer"] = torch.zeros_like(grad, memory_format=torch.preserve_format)
                keywords = dict(
                    lr=float(group["lr"]),
                    weight_decay=group["weight_decay"],
                    momentum=group["momentum"],
                    nesterov=group["nesterov"],
                    ns_coefficients=group["ns_coefficients"],
                    ns_steps=group["ns_steps"],
                    eps=group["eps"],
                    adjust_lr_fn=group["adjust_lr_fn"],
                )
                jobs.append((p.data, grad.contiguous(), state["momentum_buffer"], keywords))
        # the matrices are independent: one device's share goes to muon_step_many, which runs small ones side by side
        by_device: dict[torch.device, list] = {}
        for job in jobs:
            by_device.setdefault(job[0].device, []).append(job)
        for device, device_jobs in by_device.items():
            if self._workspace is None or self._workspace.device != device:
                self._workspace = F.MuonWorkspace(device)
            F.muon_step_many(device_jobs, workspace=self._workspace)
        return loss
