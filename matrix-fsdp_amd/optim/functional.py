"""Tensor-level entry points of the HIP optimizer kernels (current stream, no synchronisation)."""
from __future__ import annotations

import math
import os

import torch

from .. import _lib

NS_COEFFICIENTS = (3.4445, -4.7750, 2.0315)
NS_EPS = 1e-7
NS_STEPS = 5

_DTYPE_CODES = {torch.float32: _lib.DT_F32, torch.bfloat16: _lib.DT_BF16}


def adjust_lr(lr: float, adjust_lr_fn: str | None, param_shape) -> float:
    """Muon's shape-dependent learning-rate factor (torch/optim/_muon.py:73-84)."""
    rows, cols = param_shape[:2]
    if adjust_lr_fn is None or adjust_lr_fn == "original":
        ratio = math.sqrt(max(1, rows / cols))
    elif adjust_lr_fn == "match_rms_adamw":
        ratio = 0.2 * math.sqrt(max(rows, cols))
    else:
        ratio = 1.0
    return lr * ratio


def muon_workspace_bytes(rows: int, cols: int) -> int:
    n = int(_lib.lib().mfsdp_muon_workspace_bytes(rows, cols))
    if n <= 0:
        raise ValueError("Param gradient must be a 2D matrix")
    return n


class MuonWorkspace:
    """Scratch memory for the Newton-Schulz iteration, grown on demand and
    reused across matrices (the kernels themselves never allocate)."""

    def __init__(self, device) -> None:
        self.device = torch.device(device)
        self.buffer: torch.Tensor | None = None

    def get(self, rows: int, cols: int) -> torch.Tensor:
        need = muon_workspace_bytes(rows, cols)
        if self.buffer is None or self.buffer.numel() < need:
            self.buffer = None  # release before growing
            self.buffer = torch.empty(need, dtype=torch.uint8, device=self.device)
        return self.buffer


def _check_matrix(t: torch.Tensor, what: str) -> None:
    if t.ndim != 2:
        raise ValueError("Param gradient must be a 2D matrix" if what == "grad" else f"{what} must be a 2D matrix")
    if not t.is_cuda or not t.is_contiguous():
        raise RuntimeError(f"{what} must be a contiguous CUDA tensor")
    if t.dtype not in _DTYPE_CODES:
        raise RuntimeError(f"{what} must be float32 or bfloat16, got {t.dtype}")


def newton_schulz(
    update: torch.Tensor,
    ns_coefficients=NS_COEFFICIENTS,
    ns_steps: int = NS_STEPS,
    eps: float = NS_EPS,
    *,
    workspace: MuonWorkspace | None = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """bf16 orthogonalisation of ``update`` (torch/optim/_muon.py:31-70)."""
    if ns_steps >= 100:
        raise ValueError("Number of steps must be less than 100 for computational efficiency")
    if update.ndim != 2:
        raise ValueError("Input tensor gradient must be a 2D matrix")
    if len(ns_coefficients) != 3:
        raise ValueError("Coefficients must be a tuple of exactly 3 values")
    _check_matrix(update, "update")
    rows, cols = update.shape
    workspace = workspace or MuonWorkspace(update.device)
    ws = workspace.get(rows, cols)
    if out is None:
        out = torch.empty((rows, cols), dtype=torch.bfloat16, device=update.device)
    a, b, c = ns_coefficients
    stream = torch.cuda.current_stream(update.device).cuda_stream
    with torch.cuda.device(update.device):
        _lib.check(
            _lib.lib().mfsdp_newton_schulz(
                update.data_ptr(), _DTYPE_CODES[update.dtype], rows, cols, a, b, c, ns_steps, eps,
                out.data_ptr(), ws.data_ptr(), ws.numel(), stream,
            )
        )
    return out


def muon_step(
    param: torch.Tensor,
    grad: torch.Tensor,
    momentum_buf: torch.Tensor,
    *,
    lr: float,
    weight_decay: float,
    momentum: float,
    nesterov: bool,
    ns_coefficients=NS_COEFFICIENTS,
    ns_steps: int = NS_STEPS,
    eps: float = NS_EPS,
    adjust_lr_fn: str | None = None,
    workspace: MuonWorkspace | None = None,
    shared_machine: bool = False,
) -> None:
    """One matrix of ``_single_tensor_muon`` (torch/optim/_muon.py:285-318), in
    place on ``param`` and ``momentum_buf``.  ``shared_machine`` tells the
    kernels that other matrices are updated on other streams at the same time
    (``muon_step_many`` sets it)."""
    if grad.ndim != 2:
        raise ValueError("Param gradient must be a 2D matrix")
    for t, what in ((param, "param"), (grad, "grad"), (momentum_buf, "momentum buffer")):
        _check_matrix(t, what)
    if not (param.dtype == grad.dtype == momentum_buf.dtype):
        # Tensor.lerp_ rejects mixed dtypes; the reference's local shard, grad shard and state share one dtype
        raise RuntimeError(f"param, grad and momentum buffer must share a dtype, got {param.dtype}, {grad.dtype}, {momentum_buf.dtype}")
    if not (param.shape == grad.shape == momentum_buf.shape):
        raise RuntimeError("param, grad and momentum buffer must share a shape")
    if ns_steps >= 100:
        raise ValueError("Number of steps must be less than 100 for computational efficiency")
    rows, cols = param.shape
    workspace = workspace or MuonWorkspace(param.device)
    ws = workspace.get(rows, cols)
    a, b, c = ns_coefficients
    stream = torch.cuda.current_stream(param.device).cuda_stream
    with torch.cuda.device(param.device):
        _lib.check(
            _lib.lib().mfsdp_muon_step_ex(
                param.data_ptr(), grad.data_ptr(), momentum_buf.data_ptr(), _DTYPE_CODES[param.dtype], rows, cols,
                lr, weight_decay, momentum, int(bool(nesterov)), a, b, c, ns_steps, eps,
                adjust_lr(lr, adjust_lr_fn, param.shape), _lib.MUON_SHARED_MACHINE if shared_machine else 0,
                ws.data_ptr(), ws.numel(), stream,
            )
        )


class MuonStreamPool:
    """Side streams (default priority) with one Newton-Schulz workspace each, for updating independent matrices at
    the same time."""

    def __init__(self, device, n_streams: int = 3) -> None:
        self.device = torch.device(device)
        self.streams = [torch.cuda.Stream(device=self.device) for _ in range(n_streams)]
        self.workspaces = [MuonWorkspace(self.device) for _ in range(n_streams)]


_STREAM_POOLS: dict[torch.device, MuonStreamPool] = {}


def _underfills_the_machine(shape, compute_units: int) -> bool:
    """Would the 256 x 256 tiles of this matrix's symmetric products (the lower triangle of an m x m result, m the
    short side) occupy less than three quarters of the CUs?"""
    t = -(-min(shape) // 256)
    return 4 * (t * (t + 1) // 2) < 3 * compute_units


def side_by_side_default() -> bool | None:
    """``MATRIX_FSDP_MUON_SIDE_BY_SIDE``: ``0`` keeps every matrix on the calling stream (result bits that do not
    depend on which other parameters the optimizer holds), ``1`` forces the side streams, unset / ``auto`` decides
    per call."""
    value = os.environ.get("MATRIX_FSDP_MUON_SIDE_BY_SIDE", "auto").strip().lower()
    if value in ("0", "false", "off", "no"):
        return False
    if value in ("1", "true", "on", "yes"):
        return True
    return None


def muon_step_many(jobs, *, workspace: MuonWorkspace | None = None, pool: MuonStreamPool | None = None,
                   side_by_side: bool | None = None) -> None:
    """Updates several matrices; ``jobs`` is a sequence of ``(param, grad, momentum_buf, keywords of muon_step)``.

    The matrices of a rank are independent of each other.  When at least two of them are so small that the triangle
    of their symmetric products leaves CUs idle (a hidden4096 layer on 256 CUs: 136 tiles), those are spread over up
    to three side streams, longest first, so that the idle CUs work for another matrix (three hidden4096 matrices:
    7.3 against 7.5 ms); the calling stream waits for the side streams before anything enqueued later runs.  Matrices
    that keep the machine busy on their own run first, one after the other on the calling stream, as every matrix does
    when fewer than two are small.

    Reproducibility: a matrix updated on a side stream takes 256 x 256 tiles in its symmetric products where it would
    take 128 x 128 tiles alone, so the order of its fp32 sums, and with it the last bits of the update, depends on
    whether other small matrices are updated in the same call.  Both forms meet the same parity bar; a caller that
    needs bits independent of the optimizer's other parameters passes ``side_by_side=False`` (or sets
    ``MATRIX_FSDP_MUON_SIDE_BY_SIDE=0``), which keeps everything on the calling stream; ``True`` sends every 2-D
    matrix to the side streams whatever its size."""
    jobs = list(jobs)
    if not jobs:
        return
    device = jobs[0][0].device
    for param, *_ in jobs:
        if param.device != device:
            raise RuntimeError("muon_step_many updates the matrices of one device")
    if side_by_side is None:
        side_by_side = side_by_side_default()
    compute_units = torch.cuda.get_device_properties(device).multi_processor_count
    if side_by_side is False:
        small = []
    elif side_by_side:
        small = [job for job in jobs if job[0].ndim == 2]
    else:
        small = [job for job in jobs if job[0].ndim == 2 and _underfills_the_machine(job[0].shape, compute_units)]
        if len(small) < 2:
            small = []
    small_ids = {id(job) for job in small}
    alone = [job for job in jobs if id(job) not in small_ids]
    if alone:
        workspace = workspace or MuonWorkspace(device)
        for param, grad, buf, kw in alone:
            muon_step(param, grad, buf, workspace=workspace, **kw)
    jobs = small
    if not jobs:
        return
    if pool is None:
        pool = _STREAM_POOLS.get(device)
        if pool is None:
            pool = _STREAM_POOLS[device] = MuonStreamPool(device)
    n = min(len(pool.streams), len(jobs))
    # longest first onto the least loaded stream (flops of the products: 4 m^2 n + 2 m^3 per step)
    def cost(job):
        m, k = min(job[0].shape), max(job[0].shape)
        return 4 * m * m * k + 2 * m**3

    loads, assigned = [0] * n, [[] for _ in range(n)]
    for job in sorted(jobs, key=cost, reverse=True):
        s = loads.index(min(loads))
        assigned[s].append(job)
        loads[s] += cost(job)
    current = torch.cuda.current_stream(device)
    fork = torch.cuda.Event()
    fork.record(current)
    for s in range(n):
        side = pool.streams[s]
        side.wait_event(fork)
        with torch.cuda.stream(side):
            for param, grad, buf, kw in assigned[s]:
                for t in (param, grad, buf):
                    t.record_stream(side)
                muon_step(param, grad, buf, workspace=pool.workspaces[s], shared_machine=True, **kw)
        join = torch.cuda.Event()
        join.record(side)
        current.wait_event(join)


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
    """Fused AdamW over flat fp32 tensors; ``step`` is the 1-based count after
    this update (torch/optim/adam.py:347-547).  ``max_exp_avg_sq`` turns on
    amsgrad, ``maximize`` negates the gradient."""
    state = [(param, "param"), (exp_avg, "exp_avg"), (exp_avg_sq, "exp_avg_sq")]
    if max_exp_avg_sq is not None:
        state.append((max_exp_avg_sq, "max_exp_avg_sq"))
    for t, what in state:
        if not t.is_cuda or not t.is_contiguous() or t.dtype != torch.float32:
            raise RuntimeError(f"{what} must be a contiguous float32 CUDA tensor")
        if t.numel() != param.numel():
            raise RuntimeError(f"{what} has {t.numel()} elements, param has {param.numel()}")
    if not grad.is_cuda or not grad.is_contiguous() or grad.dtype not in _DTYPE_CODES or grad.numel() != param.numel():
        raise RuntimeError("grad must be a contiguous float32 or bfloat16 CUDA tensor of the param's size")
    stream = torch.cuda.current_stream(param.device).cuda_stream
    with torch.cuda.device(param.device):
        _lib.check(
            _lib.lib().mfsdp_adamw_step_ex(
                param.data_ptr(), grad.data_ptr(), _DTYPE_CODES[grad.dtype], exp_avg.data_ptr(), exp_avg_sq.data_ptr(),
                None if max_exp_avg_sq is None else max_exp_avg_sq.data_ptr(),
                param.numel(), int(step), lr, betas[0], betas[1], eps, weight_decay, int(bool(maximize)), stream,
            )
        )
