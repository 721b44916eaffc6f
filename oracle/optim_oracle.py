"""CPU oracle for the owner-rank Muon update and the AdamW tail.  TEST INFRASTRUCTURE.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product never routes through it.

The reference delegates this arithmetic to a third-party dependency that is
not under its source tree: PyTorch (``torch==2.10.0``, requirements.txt:2;
call sites matrix_fsdp/optim/wrapper.py:416-429, 439, 497-516).  The functions
below restate the published algorithm of ``torch/optim/_muon.py`` and
``torch/optim/adam.py`` in plain tensor operations.

Pinning (tests/test_oracle_optim.py):
  * ``muon_step`` / ``newton_schulz`` against ``torch.optim.Muon.step`` of
    the installed torch on seeded inputs (bit-exact on CPU: same operations in
    the same order);
  * ``newton_schulz_scalar`` (the quintic map every singular value follows)
    against ``newton_schulz`` on diagonal matrices, and a float64 SVD-based
    evaluation of the same polynomial on random matrices;
  * ``adamw_step`` against ``torch.optim.AdamW(foreach=False).step``;
  * The reference's own tests compare torch with torch at this boundary
    (test/fsdp/test_matrix_fsdp_distributed.py:1417-1470), so they pin
    ownership plumbing, not Newton-Schulz arithmetic; the pin is torch itself.
"""
from __future__ import annotations

import math

import torch

NS_EPS = 1e-7
NS_COEFFICIENTS = (3.4445, -4.7750, 2.0315)


def newton_schulz(update: torch.Tensor, coefficients=NS_COEFFICIENTS, steps: int = 5, eps: float = NS_EPS) -> torch.Tensor:
    """Quintic Newton-Schulz in bf16 (torch/optim/_muon.py:31-70): work on the
    short side, divide by ``max(||X||_F, eps)`` in bf16, then per step
    ``A = X X^T``, ``B = b A + c A A``, ``X = a X + B X`` with every product
    rounded to bf16."""
    a, b, c = coefficients
    x = update.bfloat16()
    tall = update.size(0) > update.size(1)
    if tall:
        x = x.T
    x = x / x.norm().clamp(min=eps)
    for _ in range(steps):
        gram = x @ x.T
        poly = torch.addmm(gram, gram, gram, beta=b, alpha=c)
        x = torch.addmm(x, poly, x, beta=a)
    return x.T if tall else x


def newton_schulz_scalar(sigma: float, coefficients=NS_COEFFICIENTS, steps: int = 5) -> float:
    """What one singular value becomes: ``s <- a s + b s^3 + c s^5`` per step."""
    a, b, c = coefficients
    for _ in range(steps):
        sigma = a * sigma + b * sigma**3 + c * sigma**5
    return sigma


def adjust_lr(lr: float, adjust_lr_fn: str | None, shape) -> float:
    """torch/optim/_muon.py:73-84."""
    rows, cols = shape[:2]
    if adjust_lr_fn is None or adjust_lr_fn == "original":
        ratio = math.sqrt(max(1, rows / cols))
    elif adjust_lr_fn == "match_rms_adamw":
        ratio = 0.2 * math.sqrt(max(rows, cols))
    else:
        ratio = 1.0
    return lr * ratio


def muon_step(
    param: torch.Tensor,
    grad: torch.Tensor,
    momentum_buf: torch.Tensor,
    *,
    lr: float,
    weight_decay: float = 0.1,
    momentum: float = 0.95,
    nesterov: bool = True,
    coefficients=NS_COEFFICIENTS,
    steps: int = 5,
    eps: float = NS_EPS,
    adjust_lr_fn: str | None = None,
) -> torch.Tensor:
    """One matrix of ``_single_tensor_muon`` (torch/optim/_muon.py:285-318),
    in place on ``param`` and ``momentum_buf``; returns the orthogonalised
    update ``O``."""
    momentum_buf.lerp_(grad, 1 - momentum)
    update = grad.lerp(momentum_buf, momentum) if nesterov else momentum_buf
    ortho = newton_schulz(update, coefficients, steps, eps)
    param.mul_(1 - lr * weight_decay)
    param.add_(ortho, alpha=-adjust_lr(lr, adjust_lr_fn, param.shape))
    return ortho


def adamw_step(
    param: torch.Tensor,
    grad: torch.Tensor,
    exp_avg: torch.Tensor,
    exp_avg_sq: torch.Tensor,
    step: int,
    *,
    lr: float,
    betas=(0.9, 0.999),
    eps: float = 1e-8,
    weight_decay: float = 1e-2,
    max_exp_avg_sq: torch.Tensor | None = None,
    maximize: bool = False,
) -> None:
    """Single-tensor AdamW, ``step`` being the 1-based count *after* this
    update (torch/optim/adam.py:347-547: maximize :397, decoupled decay
    :417-419, moments :457 and :476, bias corrections and the update :530-546
    with the amsgrad maximum :537-541 when ``max_exp_avg_sq`` is given)."""
    beta1, beta2 = betas
    if maximize:
        grad = -grad
    param.mul_(1 - lr * weight_decay)
    exp_avg.lerp_(grad, 1 - beta1)
    exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    bc1 = 1 - beta1**step
    bc2 = 1 - beta2**step
    step_size = lr / bc1
    second = exp_avg_sq
    if max_exp_avg_sq is not None:
        torch.maximum(max_exp_avg_sq, exp_avg_sq, out=max_exp_avg_sq)
        second = max_exp_avg_sq
    denom = (second.sqrt() / math.sqrt(bc2)).add_(eps)
    param.addcdiv_(exp_avg, denom, value=-step_size)
