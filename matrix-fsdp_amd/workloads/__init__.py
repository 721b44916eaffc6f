"""Synthetic parameter sets and shard plans of the measured workloads.

Each workload names one flat buffer (an FSDP unit: one transformer layer, or a
small MLP) by the shapes of its parameters, the seed its values are drawn
with and the simulated world it is sharded for.  Values are drawn in fp32 on
the CPU with a seeded generator and then cast, so that every device sees the
same bits.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..core.layout import ShardPlan
from ..core.plans import block_grid_plan, flat_reordered_owner_layout, fsdp2_chunk_plan


@dataclass(frozen=True)
class ParamSpec:
    """Stand-in for a ``ManagedParam`` when only extents matter."""

    fqn: str
    shape: tuple[int, ...]
    offset: int
    end: int

    @property
    def numel(self) -> int:
        return self.end - self.offset


def param_specs(shapes: list[tuple[str, tuple[int, ...]]]) -> tuple[ParamSpec, ...]:
    specs, cursor = [], 0
    for name, shape in shapes:
        n = 1
        for d in shape:
            n *= d
        specs.append(ParamSpec(name, tuple(shape), cursor, cursor + n))
        cursor += n
    return tuple(specs)


def mlp_shapes() -> list[tuple[str, tuple[int, ...]]]:
    """2-block MLP: 512x256, 256, 256x512, 512."""
    return [("fc1.weight", (512, 256)), ("fc1.bias", (256,)), ("fc2.weight", (256, 512)), ("fc2.bias", (512,))]


def transformer_layer_shapes(hidden: int, ffn: int, *, gated: bool) -> list[tuple[str, tuple[int, ...]]]:
    """One decoder layer: fused QKV, output projection, MLP (with a gate
    projection W3 when ``gated``) and two RMSNorm vectors."""
    shapes = [("attn.wqkv.weight", (3 * hidden, hidden)), ("attn.wo.weight", (hidden, hidden)), ("mlp.w1.weight", (ffn, hidden))]
    if gated:
        shapes.append(("mlp.w3.weight", (ffn, hidden)))
    shapes += [("mlp.w2.weight", (hidden, ffn)), ("attn_norm.weight", (hidden,)), ("mlp_norm.weight", (hidden,))]
    return shapes


@dataclass(frozen=True)
class Workload:
    name: str
    shapes: list
    layers: int
    world_size: int
    layout: str  # "fsdp2_chunk" or "block2x2"
    seed: int
    grad_seed: int

    @property
    def specs(self) -> tuple[ParamSpec, ...]:
        return param_specs(self.shapes)

    @property
    def total_numel(self) -> int:
        return self.specs[-1].end

    def plan(self) -> ShardPlan:
        if self.layout == "fsdp2_chunk":
            return fsdp2_chunk_plan(self.specs, self.world_size)
        if self.layout == "block2x2":
            return block_grid_plan(self.specs, (2, 2))
        if self.layout == "owner":
            return self.owner_layout(0)[2]
        raise ValueError(self.layout)

    def owner_ranks(self, layer: int) -> list[int]:
        """Whole-parameter owners of one layer's parameters: matrix number ``k`` of the model (five per
        layer, in layer order) lives on rank ``k % W``; the two norm vectors go to ranks ``layer % W`` and
        ``(layer + 1) % W``."""
        owners, matrix, vector = [], 0, 0
        n_matrices = sum(1 for _, shape in self.shapes if len(shape) == 2)
        for _, shape in self.shapes:
            if len(shape) == 2:
                owners.append((layer * n_matrices + matrix) % self.world_size)
                matrix += 1
            else:
                owners.append((layer + vector) % self.world_size)
                vector += 1
        return owners

    def owner_layout(self, layer: int):
        """``(order, offsets, plan)`` of the rank-major flat layout of one layer (see
        ``flat_reordered_owner_layout``)."""
        return flat_reordered_owner_layout(self.specs, self.world_size, self.owner_ranks(layer))


MLP_W2 = Workload("mlp_w2", mlp_shapes(), 1, 2, "fsdp2_chunk", seed=0, grad_seed=1000)
HIDDEN2048_W4 = Workload("hidden2048_w4_rows", transformer_layer_shapes(2048, 8192, gated=False), 8, 4, "fsdp2_chunk", seed=1, grad_seed=1001)
HIDDEN4096_W4_BLOCK = Workload("hidden4096_w4_block2x2", transformer_layer_shapes(4096, 11008, gated=True), 32, 4, "block2x2", seed=3, grad_seed=1003)
HIDDEN5120 = Workload("hidden5120_owner", transformer_layer_shapes(5120, 13824, gated=True), 40, 4, "owner", seed=4, grad_seed=1004)

MUON_HIDDEN4096_SHAPES = ((4096, 4096), (12288, 4096), (11008, 4096))
HIDDEN5120_TAIL_NUMEL = (40 * 2 * 5120 + 32000 * 5120) // 4  # one rank's fp32 AdamW shard: norm vectors + embedding
MUON_SEED = 4


def normal_flat(numel: int, std: float, seed: int, dtype: torch.dtype, device="cpu", chunk: int = 1 << 24) -> torch.Tensor:
    """``numel`` values N(0, std) drawn in fp32 on the CPU from ``seed`` in
    fixed-size chunks (so the stream does not depend on the device), cast to
    ``dtype`` and moved to ``device``."""
    gen = torch.Generator().manual_seed(seed)
    out = torch.empty(numel, dtype=dtype, device=device)
    for start in range(0, numel, chunk):
        n = min(chunk, numel - start)
        out[start : start + n] = (torch.randn(n, generator=gen, dtype=torch.float32) * std).to(dtype).to(device)
    return out
