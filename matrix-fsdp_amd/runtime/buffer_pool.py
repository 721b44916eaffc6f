"""Reusable full-parameter buffers (matrix_fsdp/runtime/buffer_pool.py:10-206).

A unit that reshards gives its full buffer back; the next unit with the same
element count, dtype and device unshards into the same storage (identical
transformer layers then share one 400 MB buffer instead of holding one each,
and the buffer's address stays fixed, which captured graphs need).  At most
``max_cached_per_key`` buffers are kept per (device, dtype, numel); ``0`` keeps
none.

A released buffer may still be read by kernels already queued.  The pool
records an event on the releasing stream and hands the buffer out again only
once that event has completed -- except to a caller on the very stream the
event was recorded on, where stream order already guarantees it.
"""
from __future__ import annotations

from dataclasses import dataclass
from threading import Lock
from typing import Any

import torch


@dataclass(frozen=True)
class FullParamBufferKey:
    device_type: str
    device_index: int | None
    dtype: torch.dtype
    numel: int

    @property
    def nbytes(self) -> int:
        return self.numel * torch.empty((), dtype=self.dtype).element_size()


@dataclass(frozen=True)
class FullParamBufferAcquire:
    tensor: torch.Tensor
    reused: bool


@dataclass(frozen=True)
class FullParamBufferRelease:
    kind: str  # "none" | "cached" | "pending_event" | "dropped"
    numel: int = 0
    bytes: int = 0


@dataclass
class _Waiting:
    key: FullParamBufferKey
    tensor: torch.Tensor
    event: Any
    stream: Any  # the stream the event was recorded on, when the pool recorded it


def _done(event: Any) -> bool:
    query = getattr(event, "query", None)
    return True if query is None else bool(query())


class FullParamBufferPool:
    def __init__(self, *, max_cached_per_key: int = 0) -> None:
        if max_cached_per_key < 0:
            raise ValueError("max_cached_per_key must be non-negative.")
        self.max_cached_per_key = max_cached_per_key
        self._free: dict[FullParamBufferKey, list[torch.Tensor]] = {}
        self._waiting: list[_Waiting] = []
        self._lock = Lock()  # forward hooks and the autograd thread both come here
        self.allocations = 0
        self.reuses = 0
        self.releases = 0
        self.pending_releases = 0
        self.drops = 0

    @staticmethod
    def _key(reference: torch.Tensor, numel: int) -> FullParamBufferKey:
        return FullParamBufferKey(reference.device.type, reference.device.index, reference.dtype, int(numel))

    def _held(self, key: FullParamBufferKey) -> int:
        return len(self._free.get(key, ())) + sum(1 for w in self._waiting if w.key == key)

    def _settle(self) -> None:
        """Waiting buffers whose event has completed become free."""
        still = []
        for w in self._waiting:
            if _done(w.event):
                self._free.setdefault(w.key, []).append(w.tensor)
                self.releases += 1
            else:
                still.append(w)
        self._waiting = still

    # ------------------------------------------------------------------ acquire
    def acquire_with_stats(self, reference: torch.Tensor, numel: int) -> FullParamBufferAcquire:
        key = self._key(reference, numel)
        with self._lock:
            self._settle()
            free = self._free.get(key)
            if free:
                self.reuses += 1
                return FullParamBufferAcquire(free.pop(), True)
            if reference.is_cuda and self._waiting:
                here = torch.cuda.current_stream(reference.device)
                for i, w in enumerate(self._waiting):
                    if w.key == key and w.stream is not None and w.stream == here:
                        del self._waiting[i]
                        self.releases += 1
                        self.reuses += 1
                        return FullParamBufferAcquire(w.tensor, True)
            self.allocations += 1
        return FullParamBufferAcquire(reference.new_empty(numel), False)

    def acquire(self, reference: torch.Tensor, numel: int) -> torch.Tensor:
        return self.acquire_with_stats(reference, numel).tensor

    def can_cache(self, buffer: torch.Tensor | None) -> bool:
        if buffer is None or self.max_cached_per_key == 0:
            return False
        key = self._key(buffer, buffer.numel())
        with self._lock:
            self._settle()
            return self._held(key) < self.max_cached_per_key

    # ------------------------------------------------------------------ release
    def release(self, buffer: torch.Tensor | None, *, cuda_stream: "torch.cuda.Stream | None" = None, cuda_event: Any | None = None) -> FullParamBufferRelease:
        if buffer is None:
            return FullParamBufferRelease("none")
        buffer = buffer.detach().reshape(-1)
        key = self._key(buffer, buffer.numel())
        described = dict(numel=key.numel, bytes=key.nbytes)
        stream = None
        if cuda_event is None and buffer.is_cuda and self.max_cached_per_key > 0:
            stream = cuda_stream if cuda_stream is not None else torch.cuda.current_stream(buffer.device)
            cuda_event = torch.cuda.Event()
            cuda_event.record(stream)
        with self._lock:
            self._settle()
            if self._held(key) >= self.max_cached_per_key:
                self.drops += 1
                return FullParamBufferRelease("dropped", **described)
            if cuda_event is not None and not _done(cuda_event):
                self._waiting.append(_Waiting(key, buffer, cuda_event, stream))
                self.pending_releases += 1
                return FullParamBufferRelease("pending_event", **described)
            self._free.setdefault(key, []).append(buffer)
            self.releases += 1
            return FullParamBufferRelease("cached", **described)

    def clear(self) -> None:
        with self._lock:
            self._free.clear()
            self._waiting.clear()

    def stats(self) -> dict[str, Any]:
        with self._lock:
            self._settle()
            return {
                "allocations": self.allocations,
                "reuses": self.reuses,
                "releases": self.releases,
                "pending_releases": self.pending_releases,
                "drops": self.drops,
                "cached_buffers": sum(len(b) for b in self._free.values()),
                "cached_numel": sum(k.numel * len(b) for k, b in self._free.items()),
                "cached_bytes": sum(k.nbytes * len(b) for k, b in self._free.items()),
                "pending_buffers": len(self._waiting),
                "pending_numel": sum(w.key.numel for w in self._waiting),
                "pending_bytes": sum(w.key.nbytes for w in self._waiting),
                "keys": len(self._free),
                "max_cached_per_key": self.max_cached_per_key,
            }


def clear_global_full_param_buffer_pool() -> None:
    """Pools belong to the units they are handed to; there is no process-wide
    one to clear.  Kept for callers of the reference's function of this name."""
