"""The kernels under HIP graph capture: once their programs / workspaces exist, pack, unpack, gradient copy-in, the
Muon step and the AdamW step enqueue nothing but kernels (no allocation, no memset, no synchronisation), so a caller
may capture them.  Every replay is checked against the eager result, with eager work between the replays."""
import pytest
import torch

from matrix_fsdp_amd.kernels.segment_program import grad_fill_program, pack_program, unpack_program
from matrix_fsdp_amd.optim import functional as F
from matrix_fsdp_amd.workloads import MLP_W2, normal_flat
from oracle import copy_oracle as CO

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_copy_programs_replay_bit_exact():
    w = MLP_W2
    plan = w.plan()
    pack = pack_program(plan, torch.bfloat16, device=DEV)
    unpack = unpack_program(plan, torch.bfloat16, device=DEV)
    fill = grad_fill_program(w.specs, plan.shard_sizes, plan.rank_segments, torch.bfloat16, torch.float32, device=DEV)
    full = torch.empty(w.total_numel, dtype=torch.bfloat16, device=DEV)
    grads = [torch.empty(s.numel, dtype=torch.bfloat16, device=DEV) for s in w.specs]
    padded = torch.empty(w.world_size * plan.max_shard_size, dtype=torch.bfloat16, device=DEV)
    out = torch.empty_like(full)
    packed32 = torch.empty(w.world_size * plan.max_shard_size, dtype=torch.float32, device=DEV)

    def enqueue():
        pack.run((full,), padded)
        unpack.run((padded,), out)
        fill.run(grads, packed32)

    full.copy_(normal_flat(w.total_numel, 0.02, 1, torch.bfloat16))
    for g, s in zip(grads, w.specs):
        g.copy_(normal_flat(s.numel, 1e-3, 2, torch.bfloat16))
    enqueue()  # programs pick their table variant for these pointers before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for seed in (10, 20, 30):
        host_full = normal_flat(w.total_numel, 0.02, seed, torch.bfloat16)
        host_grads = [normal_flat(s.numel, 1e-3, seed + 1 + k, torch.bfloat16) for k, s in enumerate(w.specs)]
        full.copy_(host_full)
        for g, h in zip(grads, host_grads):
            g.copy_(h)
        padded.fill_(7)
        out.fill_(9)
        packed32.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(padded.cpu().view(torch.int16), CO.pack_to_padded(host_full, plan).view(torch.int16))
        assert torch.equal(out.cpu().view(torch.int16), host_full.view(torch.int16))
        want = torch.zeros(w.world_size, plan.max_shard_size)
        CO.chunk_cat([g.float() for g in host_grads], w.world_size, want)
        assert torch.equal(packed32.cpu(), want.reshape(-1))
        # eager work of the program itself between replays
        (full.float() * 2).sum().item()


def test_muon_and_adamw_steps_replay_like_eager():
    shape = (384, 640)
    ws = F.MuonWorkspace(DEV)
    kw = dict(lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True)
    akw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    p, g, buf = (torch.empty(shape, device=DEV) for _ in range(3))
    n = 100_003
    ap, ag, am, av = (torch.empty(n, device=DEV) for _ in range(4))

    def load(seed: int) -> None:
        p.copy_(normal_flat(p.numel(), 0.02, seed, torch.float32).view(shape))
        g.copy_(normal_flat(p.numel(), 1e-3, seed + 1, torch.bfloat16).float().view(shape))
        buf.copy_(normal_flat(p.numel(), 1e-3, seed + 2, torch.float32).view(shape))
        ap.copy_(normal_flat(n, 0.02, seed + 3, torch.float32))
        ag.copy_(normal_flat(n, 1e-3, seed + 4, torch.float32))
        am.copy_(normal_flat(n, 1e-3, seed + 5, torch.float32))
        av.copy_(normal_flat(n, 1e-3, seed + 6, torch.float32).square())

    def enqueue() -> None:
        F.muon_step(p, g, buf, workspace=ws, **kw)
        F.adamw_step(ap, ag, am, av, 3, **akw)

    load(0)
    enqueue()  # sizes the workspace and configures the kernels before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for seed in (100, 200, 300):
        load(seed)
        enqueue()
        torch.cuda.synchronize()
        eager = [t.clone() for t in (p, buf, ap, am, av)]
        load(seed)
        graph.replay()
        torch.cuda.synchronize()
        for have, want in zip((p, buf, ap, am, av), eager):
            assert torch.equal(have, want)  # same kernels on the same inputs: bit-identical
