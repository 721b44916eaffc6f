"""``fully_shard`` + ``configure_optimizer`` driving the HIP kernels through a training loop on one device.

The twin of every sharded model is the same module trained eagerly on the same GPU with torch's own optimizers:
forward and backward then run the very same library kernels on the same values, so the only difference left is
the path under test (flat-buffer copies, casts, gradient copy-in, HIP optimizer kernels)."""
import copy

import pytest
import torch
from torch import nn

from matrix_fsdp_amd import (
    FSDPLifecycleState,
    MixedMuonAdamWOptimizer,
    MixedPrecisionPolicy,
    ParamShardHint,
    configure_optimizer,
    fully_shard,
)
from matrix_fsdp_amd.core.plans import fsdp2_chunk_plan, whole_param_owner_plan
from matrix_fsdp_amd.optim.wrapper import collect_flat_buffers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class Block(nn.Module):
    def __init__(self, dim: int, hidden: int) -> None:
        super().__init__()
        self.norm = nn.LayerNorm(dim)
        self.up = nn.Linear(dim, hidden, bias=False)
        self.down = nn.Linear(hidden, dim, bias=True)

    def forward(self, x):
        return x + self.down(torch.nn.functional.gelu(self.up(self.norm(x))))


class Net(nn.Module):
    def __init__(self, dim: int = 64, hidden: int = 128, blocks: int = 2, out: int = 16) -> None:
        super().__init__()
        self.blocks = nn.ModuleList(Block(dim, hidden) for _ in range(blocks))
        self.head = nn.Linear(dim, out)

    def forward(self, x):
        for block in self.blocks:
            x = block(x)
        return self.head(x)


def make_pair(seed: int = 0, **net_kwargs):
    torch.manual_seed(seed)
    model = Net(**net_kwargs).to(DEV)
    return model, copy.deepcopy(model)


def batches(n: int, dim: int = 64, out: int = 16, seed: int = 1):
    gen = torch.Generator().manual_seed(seed)
    return [(torch.randn(32, dim, generator=gen).to(DEV), torch.randn(32, out, generator=gen).to(DEV)) for _ in range(n)]


def shard_all(model: Net, **kwargs) -> None:
    for block in model.blocks:
        fully_shard(block, **kwargs)
    fully_shard(model, **kwargs)


def named_full_params(model: nn.Module) -> dict[str, torch.Tensor]:
    return {name: p.detach().float().cpu().clone() for name, p in model.named_parameters()}


def rel(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30))


def test_single_rank_adamw_training_matches_eager():
    model, twin = make_pair()
    shard_all(model)
    units = [m._matrix_fsdp_param_group for m in [*model.blocks, model]]
    assert len(collect_flat_buffers(model)) == 3
    assert [len(u.managed_params) for u in units] == [5, 5, 2]  # the root keeps only what no block manages
    opt = configure_optimizer(model, "adamw", lr=1e-3, betas=(0.9, 0.95), weight_decay=0.1)
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-3, betas=(0.9, 0.95), weight_decay=0.1, foreach=False)
    for x, y in batches(3):
        loss = torch.nn.functional.mse_loss(model(x), y)
        assert all(u.lifecycle_state == FSDPLifecycleState.FORWARD_RESHARDED for u in units)
        loss.backward()
        assert all(u.lifecycle_state == FSDPLifecycleState.SHARDED for u in units)
        for u in units:
            fb = u.flat_buffer
            assert fb.param_data_alias_local_shard()
            assert all(mp.param.grad.data_ptr() >= fb.local_grad_shard.data_ptr() for mp in u.managed_params)
        opt.step()
        opt.zero_grad()
        ref_loss = torch.nn.functional.mse_loss(twin(x), y)
        ref_loss.backward()
        ref.step()
        ref.zero_grad()
        assert abs(loss.item() - ref_loss.item()) <= 1e-5 * abs(ref_loss.item())
    have, want = named_full_params(model), named_full_params(twin)
    for name in want:
        assert rel(have[name], want[name]) < 2e-6, name


def test_wrap_policy_units_train_like_eager():
    """``wrap_policy`` picks the blocks and the head as units (top-down, a selected module is not descended into);
    with ``auto_shard_hints`` and the owner planner the matrices go to Muon."""
    from matrix_fsdp_amd import matrix_fully_shard
    from matrix_fsdp_amd.policy import module_type_policy, or_policy, size_based_policy

    model, twin = make_pair(seed=3)
    policy = or_policy(module_type_policy(Block), size_based_policy(64 * 16))  # Block would also pass the size test via its Linears, but is taken whole
    assert matrix_fully_shard(model, wrap_policy=policy, auto_shard_hints=True, auto_planner_policy="muon_shard_aware") is model
    units = {name: m._matrix_fsdp_param_group for name, m in model.named_modules() if hasattr(m, "_matrix_fsdp_param_group")}
    assert sorted(units) == ["blocks.0", "blocks.1", "head"]
    assert [len(u.managed_params) for u in units.values()] == [5, 5, 2]
    assert len({id(u.planner) for u in units.values()}) == 1  # one owner planner balances the ranks across the units
    assert units["blocks.0"].managed_params[2].shard_hint.optimizer_type == "muon"  # up.weight
    opt = configure_optimizer(model, "mixed_muon_adamw", lr=2e-3, weight_decay=0.05)
    muon_names = {fqn for g in opt.optimizer_group_summary()["groups"] if g["optimizer_type"] == "muon" for fqn in g["param_fqns"]}
    assert muon_names == {"up.weight", "down.weight", "weight"}
    matrices = [p for p in twin.parameters() if p.ndim == 2]
    others = [p for p in twin.parameters() if p.ndim != 2]
    defaults = opt.defaults
    ref_muon = torch.optim.Muon(matrices, **{k: defaults["muon"][k] for k in ("lr", "weight_decay", "momentum", "nesterov", "ns_coefficients", "eps", "ns_steps", "adjust_lr_fn")})
    ref_adamw = torch.optim.AdamW(others, **{k: defaults["adamw"][k] for k in ("lr", "betas", "eps", "weight_decay")}, foreach=False)
    start = named_full_params(twin)
    (x, y), = batches(1, seed=6)
    torch.nn.functional.mse_loss(model(x), y).backward()
    opt.step()
    torch.nn.functional.mse_loss(twin(x), y).backward()
    ref_muon.step()
    ref_adamw.step()
    have, want = named_full_params(model), named_full_params(twin)
    for name in want:
        assert rel(have[name] - start[name], want[name] - start[name]) < (1e-2 if want[name].ndim == 2 else 1e-5), name


def test_single_rank_mixed_muon_adamw_training_matches_eager():
    model, twin = make_pair(seed=2)
    shard_all(model, reshard_after_forward=False)
    opt = configure_optimizer(model, "mixed_muon_adamw", lr=2e-3, weight_decay=0.05)
    assert isinstance(opt, MixedMuonAdamWOptimizer)
    matrices = [p for p in twin.parameters() if p.ndim == 2]
    others = [p for p in twin.parameters() if p.ndim != 2]
    defaults = opt.defaults
    ref_muon = torch.optim.Muon(matrices, **{k: defaults["muon"][k] for k in ("lr", "weight_decay", "momentum", "nesterov", "ns_coefficients", "eps", "ns_steps", "adjust_lr_fn")})
    ref_adamw = torch.optim.AdamW(others, **{k: defaults["adamw"][k] for k in ("lr", "betas", "eps", "weight_decay")}, foreach=False)
    start = named_full_params(twin)
    for step, (x, y) in enumerate(batches(3, seed=5)):
        torch.nn.functional.mse_loss(model(x), y).backward()
        opt.step()
        opt.zero_grad()
        torch.nn.functional.mse_loss(twin(x), y).backward()
        ref_muon.step()
        ref_adamw.step()
        ref_muon.zero_grad()
        ref_adamw.zero_grad()
        have, want = named_full_params(model), named_full_params(twin)
        for name in want:
            # the orthogonalised update is a bf16 iteration: 1e-2 per step of the parameter change; vectors follow
            # AdamW exactly in the first step and afterwards see gradients through slightly different matrices
            tol = 1e-2 * (step + 1) if want[name].ndim == 2 else (1e-5 if step == 0 else 2e-3)
            assert rel(have[name] - start[name], want[name] - start[name]) < tol, (step, name)


@pytest.mark.parametrize("low", [torch.bfloat16, torch.float16])
def test_mixed_precision_low_precision_compute_fp32_master(low):
    model, twin = make_pair(seed=3)
    policy = MixedPrecisionPolicy(param_dtype=low, reduce_dtype=torch.float32)
    for block in model.blocks:
        fully_shard(block, mp_policy=policy)
    fully_shard(model, mp_policy=MixedPrecisionPolicy(param_dtype=low, reduce_dtype=torch.float32, output_dtype=torch.float32))
    opt = configure_optimizer(model, "adamw", lr=1e-3, betas=(0.9, 0.95), weight_decay=0.0)
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-3, betas=(0.9, 0.95), weight_decay=0.0, foreach=False)
    seen_dtypes = []
    model.blocks[0].up.register_forward_pre_hook(lambda mod, args: seen_dtypes.append((mod.weight.dtype, args[0].dtype)))
    for x, y in batches(2, seed=7):
        out = model(x)
        assert out.dtype == torch.float32
        torch.nn.functional.mse_loss(out, y).backward()
        for unit in [*model.blocks, model]:
            fb = unit._matrix_fsdp_param_group.flat_buffer
            assert fb.local_shard.dtype == torch.float32 and fb.local_grad_shard.dtype == torch.float32
            assert all(mp.param.dtype == torch.float32 and mp.param.grad.dtype == torch.float32 for mp in fb.managed_params)
        # eager twin: low-precision working copy of the fp32 master weights, grads cast up
        work = copy.deepcopy(twin).to(low)
        torch.nn.functional.mse_loss(work(x.to(low)).float(), y).backward()
        for master, w in zip(twin.parameters(), work.parameters()):
            master.grad = w.grad.float()
        for (name, p), master in zip(model.named_parameters(), twin.parameters()):
            assert torch.equal(p.grad.reshape(-1).cpu(), master.grad.reshape(-1).cpu()), name  # cast + copy-in are exact
        opt.step()
        opt.zero_grad()
        ref.step()
        ref.zero_grad()
    assert seen_dtypes and all(w == low and a == low for w, a in seen_dtypes)
    have, want = named_full_params(model), named_full_params(twin)
    for name in want:
        assert rel(have[name], want[name]) < 2e-6, name


@pytest.mark.parametrize("world, rank", [(1, 0), (4, 1)])
def test_gradients_accumulate_over_backwards_until_zero_grad(world, rank):
    """Micro-batches: every backward reduces its gradients into the local shard and adds them to what the
    previous one left, ``zero_grad`` (dropping or zeroing the grads) starts over.  The twin accumulates full
    gradients in ``.grad`` the ordinary way; the rank's shard of them is compared bit for bit (fp32 adds of the
    same numbers in the same order)."""
    model, twin = make_pair(seed=5)
    shard_all(model, world_size=world, rank=rank, planner=fsdp2_chunk_plan)
    units = [m._matrix_fsdp_param_group for m in [*model.blocks, model]]
    opt = configure_optimizer(model, "adamw", lr=1e-3)

    def twin_local_grads(unit):
        full = torch.cat([dict(twin.named_parameters())[prefix + mp.fqn].grad.reshape(-1) for prefix, u in prefixed if u is unit for mp in u.managed_params])
        return torch.cat([full[s.global_start : s.global_end] for s in unit.flat_buffer.local_segments])

    prefixed = [(f"blocks.{i}.", u) for i, u in enumerate(units[:-1])] + [("", units[-1])]
    data = batches(6, seed=9)
    zeroed_in_place = False
    for round_, zero in enumerate(("none", "zeros", "none")):
        for micro, (x, y) in enumerate(data[2 * round_ : 2 * round_ + 2]):
            torch.nn.functional.mse_loss(model(x), y).backward()
            torch.nn.functional.mse_loss(twin(x), y).backward()
            for unit in units:
                fb = unit.flat_buffer
                assert torch.equal(fb.local_grad_shard, twin_local_grads(unit)), (round_, micro)
                assert all(v.managed_param.param.grad.data_ptr() == fb.local_grad_shard.data_ptr() + v.shard_start * 4 for v in fb.local_param_views)
                # a shard zeroed in place is still live: the next backward adds to the zeros
                assert ("accumulate_local_grad_shard" in unit.events[-3:]) == (micro == 1 or zeroed_in_place)
            zeroed_in_place = False
        # no step: the parameters of the two models stay identical, so the gradients can be compared bit for bit
        twin.zero_grad(set_to_none=(zero == "none"))
        if zero == "none":  # through the optimizer: grads dropped and the reduced shards released
            opt.zero_grad()
            assert all(p.grad is None for p in model.parameters())
            assert all(u.flat_buffer.local_grad_shard is None for u in units)
        else:  # through the module: grads zeroed where they are
            model.zero_grad(set_to_none=False)
            assert all(float(u.flat_buffer.local_grad_shard.abs().sum()) == 0.0 for u in units)
            zeroed_in_place = True


class CheckpointedNet(Net):
    """Every block runs under activation checkpointing: its forward is re-run in the middle of the backward."""

    use_reentrant = False

    def forward(self, x):
        from torch.utils.checkpoint import checkpoint

        for block in self.blocks:
            x = checkpoint(block, x, use_reentrant=self.use_reentrant)
        return self.head(x)


@pytest.mark.parametrize("use_reentrant", [False, True])
@pytest.mark.parametrize("reshard_after_forward", [True, False])
@pytest.mark.parametrize("world, rank", [(1, 0), (4, 2)])
def test_activation_checkpointing_recomputes_inside_the_backward(use_reentrant, reshard_after_forward, world, rank):
    torch.manual_seed(6)
    model = CheckpointedNet().to(DEV)
    model.use_reentrant = use_reentrant
    twin = Net().to(DEV)
    twin.load_state_dict(model.state_dict())
    shard_all(model, world_size=world, rank=rank, planner=fsdp2_chunk_plan, reshard_after_forward=reshard_after_forward)
    units = [m._matrix_fsdp_param_group for m in [*model.blocks, model]]
    names = [(f"blocks.{i}.", u) for i, u in enumerate(units[:-1])] + [("", units[-1])]
    for x, y in batches(2, seed=11):
        for unit in units:
            unit.events.clear()
        x = x.requires_grad_(use_reentrant)  # the reentrant form needs an input that requires grad
        torch.nn.functional.mse_loss(model(x), y).backward()
        torch.nn.functional.mse_loss(twin(x.detach()), y).backward()
        for prefix, unit in names:
            assert unit.lifecycle_state == FSDPLifecycleState.SHARDED and not unit._in_backward
            fb = unit.flat_buffer
            full = torch.cat([dict(twin.named_parameters())[prefix + mp.fqn].grad.reshape(-1) for mp in unit.managed_params])
            want = torch.cat([full[s.global_start : s.global_end] for s in fb.local_segments])
            assert torch.equal(fb.local_grad_shard, want), prefix
        if not use_reentrant:  # the re-run forward neither reshards nor counts as a new forward
            assert units[0].events.count("pre_forward") == 1
            assert units[0].events.count("reshard:post_forward") == int(reshard_after_forward)
        for p in [*model.parameters(), *twin.parameters()]:
            p.grad = None


def test_a_unit_called_twice_in_one_forward_and_an_unused_unit():
    """Weight sharing in time: the same block applied twice before one backward (``reshard_after_forward=False``,
    with resharding the second forward is refused), and a unit that takes no part in the step at all."""
    model, twin = make_pair(seed=8)
    shard_all(model, reshard_after_forward=False)
    units = [m._matrix_fsdp_param_group for m in [*model.blocks, model]]
    (x, y), = batches(1, seed=12)

    def twice(net, x):
        return net.head(net.blocks[0](net.blocks[0](x)))  # blocks[1] unused; the root's own forward is bypassed too

    torch.nn.functional.mse_loss(twice(model, x), y).backward()
    torch.nn.functional.mse_loss(twice(twin, x), y).backward()
    assert units[0].lifecycle_state == FSDPLifecycleState.SHARDED
    for (name, p), q in zip(model.blocks[0].named_parameters(), twin.blocks[0].parameters()):
        assert torch.equal(p.grad, q.grad), name
    assert all(p.grad is None for p in model.blocks[1].parameters())  # nothing reduced, nothing to step
    assert units[1].flat_buffer.local_grad_shard is None

    strict, _ = make_pair(seed=8)
    fully_shard(strict.blocks[0])
    with pytest.raises(RuntimeError, match="another forward"):
        strict.blocks[0](strict.blocks[0](x))


def test_simulated_world_of_four_updates_only_the_rank_shard():
    """Rank 1 of a simulated world of 4 (per-parameter chunks): parameters are packed, gathered and unpacked
    through the segment programs every step, and the optimizer sees quarter-parameter views.  The twin trains
    the whole model and then puts back every element the rank does not hold, which is what a world whose other
    ranks never step looks like."""
    world, rank = 4, 1
    model, twin = make_pair(seed=4)
    shard_all(model, world_size=world, rank=rank, planner=fsdp2_chunk_plan)
    opt = configure_optimizer(model, "adamw", lr=1e-3, weight_decay=0.1)
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-3, weight_decay=0.1, foreach=False)
    for name, p in model.named_parameters():
        assert p.ndim == 1 and p.numel() * world == dict(twin.named_parameters())[name].numel()
    for x, y in batches(3, seed=9):
        torch.nn.functional.mse_loss(model(x), y).backward()
        opt.step()
        opt.zero_grad()
        before = [p.detach().clone() for p in twin.parameters()]
        torch.nn.functional.mse_loss(twin(x), y).backward()
        ref.step()
        ref.zero_grad()
        with torch.no_grad():
            for p, old in zip(twin.parameters(), before):
                flat, keep = p.view(-1), old.view(-1)
                chunk = flat.numel() // world
                mine = flat[rank * chunk : (rank + 1) * chunk].clone()
                flat.copy_(keep)
                flat[rank * chunk : (rank + 1) * chunk] = mine
    twin_params = dict(twin.named_parameters())
    for name, p in model.named_parameters():
        full = twin_params[name].detach().view(-1)
        chunk = full.numel() // world
        assert rel(p.detach().cpu(), full[rank * chunk : (rank + 1) * chunk].cpu()) < 2e-6, name
    # and the full parameters the forward sees are the twin's
    unit = model.blocks[0]._matrix_fsdp_param_group
    unit.unshard()
    assert unit.flat_buffer.param_data_alias_full_buffer()
    assert rel(model.blocks[0].up.weight.detach().cpu(), twin.blocks[0].up.weight.detach().cpu()) < 2e-6
    unit.reshard()


def test_owner_layout_unit_runs_muon_on_owned_matrices():
    """Whole-parameter owners in a simulated world of 2: rank 0 owns ``up``, rank 1 owns ``down``; the hint puts
    Muon on the owned matrix and the unit still trains."""
    torch.manual_seed(6)
    block = Block(64, 128).to(DEV)
    hints = {"up.weight": ParamShardHint(optimizer_type="muon")}
    owners = {"norm.weight": 0, "norm.bias": 0, "up.weight": 0, "down.weight": 1, "down.bias": 1}
    fully_shard(
        block,
        world_size=2,
        rank=0,
        planner=lambda mps, w: whole_param_owner_plan(mps, w, [owners[mp.fqn] for mp in mps]),
        shard_placement_fn=lambda p: ParamShardHint(optimizer_type="muon") if tuple(p.shape) == (128, 64) else None,
    )
    assert hints  # the hint table above documents what shard_placement_fn produces
    opt = configure_optimizer(block, "mixed_muon_adamw", lr=1e-3)
    assert [tuple(p.shape) for p in opt.muon_params] == [(128, 64)]
    assert block.down.weight.numel() == 0  # not this rank's
    x = torch.randn(8, 64, device=DEV)
    before = block.up.weight.detach().clone()
    block(x).square().mean().backward()
    assert block.up.weight.grad is not None and block.down.weight.grad is None
    opt.step()
    assert not torch.equal(block.up.weight.detach(), before)


def test_lifecycle_rules():
    model, _ = make_pair(seed=8)
    shard_all(model)
    unit = model.blocks[0]._matrix_fsdp_param_group
    x, _ = batches(1)[0]
    with torch.no_grad():
        model(x)
    assert unit.lifecycle_state == FSDPLifecycleState.SHARDED and unit.flat_buffer.param_data_alias_local_shard()
    opt = configure_optimizer(model, "adamw", lr=1e-3)
    mixed = configure_optimizer(model, "mixed_muon_adamw", lr=1e-3)
    out = model(x)
    assert unit.lifecycle_state == FSDPLifecycleState.FORWARD_RESHARDED
    with pytest.raises(RuntimeError, match="another forward"):
        model(x)
    for optimizer in (opt, mixed):  # between forward and backward there is nothing to step
        with pytest.raises(RuntimeError, match="forward-resharded"):
            optimizer.step()
    out.sum().backward()
    assert unit.lifecycle_state == FSDPLifecycleState.SHARDED
    assert "unshard:pre_backward" in unit.events and unit.events[-1] == "finalize_backward"
    unit.unshard()
    with pytest.raises(RuntimeError, match="expects MatrixFSDP parameters to be sharded"):
        opt.step()
    with pytest.raises(RuntimeError, match="expects MatrixFSDP parameters to be sharded"):
        unit.assert_optimizer_ready("test")
    unit.reshard()
    with model.no_sync():  # covers every unit below the module it is called on
        assert unit.is_no_sync_active()
        with pytest.raises(RuntimeError, match="no_sync"):
            opt.step()
    assert not unit.is_no_sync_active()
    before = unit.flat_buffer.local_shard.clone()
    opt.step()
    assert not torch.equal(unit.flat_buffer.local_shard, before)
    with pytest.raises(ValueError, match="already wrapped"):
        fully_shard(model)
    with pytest.raises(ValueError, match="floating-point"):
        fully_shard(nn.Linear(4, 4).to(DEV), mp_policy=MixedPrecisionPolicy(param_dtype=torch.int32))


def test_muon_optimizer_policy_in_a_simulated_world_of_two():
    """``optimizer_policy="muon"``: hints from the module structure, whole-parameter owners balanced over the
    units by one shared planner, Muon on the matrices rank 0 owns and AdamW on its vectors.  The twin trains
    everything and puts back what rank 0 does not own."""
    from matrix_fsdp_amd.planning import MuonOwnerPlanner, owner_ranks

    world, rank = 2, 0
    model, twin = make_pair(seed=10)
    planner = MuonOwnerPlanner()
    for unit in [*model.blocks, model]:
        fully_shard(unit, world_size=world, rank=rank, optimizer_policy="muon", planner=planner, reshard_after_forward=False)
    owned = {}
    for prefix, unit in [("blocks.0.", model.blocks[0]), ("blocks.1.", model.blocks[1]), ("", model)]:
        group = unit._matrix_fsdp_param_group
        for mp in group.managed_params:
            ranks = owner_ranks(group.shard_plan, mp)
            assert len(ranks) == 1  # never cut
            owned[prefix + mp.fqn] = ranks[0] == rank
    assert 0 < sum(owned.values()) < len(owned)
    assert abs(planner.rank_units[0] - planner.rank_units[1]) <= max(p.numel() for p in twin.parameters())
    opt = configure_optimizer(model, "mixed_muon_adamw", lr=1e-3, weight_decay=0.0)
    assert all(p.ndim == 2 for p in opt.muon_params) and len(opt.muon_params) == sum(owned[n] and p.ndim == 2 for n, p in twin.named_parameters())
    twin_named = dict(twin.named_parameters())
    defaults = opt.defaults
    ref_muon = torch.optim.Muon([p for n, p in twin_named.items() if p.ndim == 2], **{k: defaults["muon"][k] for k in ("lr", "weight_decay", "momentum", "nesterov", "ns_coefficients", "eps", "ns_steps", "adjust_lr_fn")})
    ref_adamw = torch.optim.AdamW([p for n, p in twin_named.items() if p.ndim != 2], **{k: defaults["adamw"][k] for k in ("lr", "betas", "eps", "weight_decay")}, foreach=False)
    start = named_full_params(twin)
    for x, y in batches(2, seed=11):
        torch.nn.functional.mse_loss(model(x), y).backward()
        opt.step()
        opt.zero_grad()
        before = {n: p.detach().clone() for n, p in twin_named.items()}
        torch.nn.functional.mse_loss(twin(x), y).backward()
        ref_muon.step()
        ref_adamw.step()
        ref_muon.zero_grad()
        ref_adamw.zero_grad()
        with torch.no_grad():
            for n, p in twin_named.items():
                if not owned[n]:
                    p.copy_(before[n])
    for n, p in model.named_parameters():
        if owned[n]:
            want = twin_named[n].detach().float().cpu()
            tol = 2e-2 if want.ndim == 2 else 2e-3
            assert rel(p.detach().float().cpu() - start[n], want - start[n]) < tol, n
        else:
            assert p.numel() == 0, n


def test_shard0_placement_maps_to_leading_dimension_hints():
    """The expectations of the reference's test (test/fsdp/test_matrix_fsdp_e2e.py:252-291): a matrix may be cut
    between rows, a vector between elements, ignored parameters are not asked about, the layout is one stretch per
    rank."""
    from torch.distributed.tensor import Shard

    model = nn.Sequential(nn.Linear(4, 2), nn.LayerNorm(2)).to(DEV)
    assert fully_shard(model, shard_placement_fn=lambda p: Shard(0)) is model
    unit = model._matrix_fsdp_param_group
    assert unit.param_registry.param("0.weight").shard_hint == ParamShardHint(split_granularity="row_block", block_shape=(1, 4))
    assert unit.param_registry.param("0.bias").shard_hint == ParamShardHint(split_granularity="block", block_shape=(1,))
    assert unit.group_layout is not None and unit.runtime_layout_compatibility.mode == "matrix_shard"

    model = nn.Sequential(nn.Linear(4, 2), nn.LayerNorm(2)).to(DEV)
    ignored, asked = model[1].weight, []

    def placement(param):
        asked.append(id(param))
        return Shard(0)

    fully_shard(model, shard_placement_fn=placement, ignored_params={ignored}, world_size=2, rank=1)
    unit = model._matrix_fsdp_param_group
    assert id(ignored) not in asked and "1.weight" not in unit.param_registry.fqns
    assert unit.param_registry.param("1.bias").shard_hint == ParamShardHint(split_granularity="block", block_shape=(1,))
    assert unit.shard_plan.shard_sizes == (8, 4)  # 12 elements: the cut nearest to 6 that takes a block on a tie

    seen = []
    model = nn.Sequential(nn.Linear(4, 2), nn.Linear(2, 1)).to(DEV)
    fully_shard(model, shard_placement_fn=lambda p: seen.append(id(p)))
    assert seen == [id(p) for p in model.parameters()]


@pytest.mark.parametrize("rank", [0, 1, 2])
def test_shard0_units_train_like_eager_in_a_simulated_world_of_three(rank):
    """Every unit is cut at row boundaries into three rank-contiguous stretches (``hinted_ordered_group_plan``);
    parameters straddling a cut are 1-D slices for the optimizer.  The twin trains whole and then takes back
    every element outside the rank's stretch."""
    from torch.distributed.tensor import Shard

    world = 3
    model, twin = make_pair(seed=11)
    shard_all(model, world_size=world, rank=rank, shard_placement_fn=lambda p: Shard(0))
    units = [m._matrix_fsdp_param_group for m in [*model.blocks, model]]
    twin_params = dict(twin.named_parameters())
    prefixes = [f"blocks.{i}." for i in range(len(model.blocks))] + [""]
    for unit in units:
        assert unit.runtime_layout_compatibility.mode == "matrix_shard"
        for mp in unit.managed_params:  # cuts fall between rows
            for piece in unit.group_layout.param(mp.fqn).segments:
                row = mp.shape[-1] if len(mp.shape) == 2 else 1
                assert (piece.global_start - mp.offset) % row == 0 and (piece.global_end - mp.offset) % row == 0
    opt = configure_optimizer(model, "adamw", lr=1e-3, weight_decay=0.1)
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-3, weight_decay=0.1, foreach=False)

    def stretch(unit, prefix):
        """(twin parameter, first, last) for the part of each parameter inside the rank's stretch."""
        lo, hi = unit.shard_plan.local_range(rank)
        for mp in unit.managed_params:
            a, b = max(lo, mp.offset), min(hi, mp.end)
            yield twin_params[prefix + mp.fqn], mp, max(a - mp.offset, 0), max(b - mp.offset, 0)

    for x, y in batches(3, seed=12):
        torch.nn.functional.mse_loss(model(x), y).backward()
        opt.step()
        opt.zero_grad()
        before = {name: p.detach().clone() for name, p in twin_params.items()}
        torch.nn.functional.mse_loss(twin(x), y).backward()
        ref.step()
        ref.zero_grad()
        with torch.no_grad():
            for unit, prefix in zip(units, prefixes):
                for p, mp, a, b in stretch(unit, prefix):
                    mine = p.view(-1)[a:b].clone()
                    p.copy_(before[prefix + mp.fqn])
                    p.view(-1)[a:b] = mine
    for unit, prefix in zip(units, prefixes):
        for p, mp, a, b in stretch(unit, prefix):
            local = mp.param.detach().view(-1)
            assert local.numel() == max(b - a, 0), mp.fqn
            if b > a:
                assert rel(local.cpu(), p.detach().view(-1)[a:b].cpu()) < 2e-6, mp.fqn
        unit.unshard()
        assert unit.flat_buffer.param_data_alias_full_buffer()
        for mp in unit.managed_params:
            assert rel(mp.param.detach().cpu(), twin_params[prefix + mp.fqn].detach().cpu()) < 2e-6, mp.fqn
        unit.reshard()


def test_plain_torch_optimizers_are_prepared_automatically():
    """A ``torch.optim`` optimizer built over a unit's parameters gets the unit's lifecycle hooks by itself
    (the reference's behaviour, test/fsdp/test_matrix_fsdp_e2e.py:1818-1893, 2006-2022)."""
    from matrix_fsdp_amd import PreparedMatrixOptimizer, matrix_fully_shard, prepare_matrix_optimizer

    torch.manual_seed(0)
    model = matrix_fully_shard(nn.Linear(4, 2).to(DEV))
    unit = model._matrix_fsdp_param_group
    optimizer = torch.optim.AdamW(model.parameters(), lr=0.01)
    prepared = optimizer.matrix_fsdp
    assert isinstance(prepared, PreparedMatrixOptimizer) and optimizer.state_manager is prepared.state_manager
    model(torch.randn(3, 4, device=DEV)).sum().backward()
    optimizer.step()
    assert prepared.state_objects and optimizer.matrix_fsdp.state_objects
    prepared.validate_local_state_shapes()
    assert unit.flat_buffer.local_grad_shard is not None
    optimizer.zero_grad()
    assert unit.flat_buffer.local_grad_shard is None
    with pytest.raises(NotImplementedError, match="closures"):
        optimizer.step(lambda: None)
    again = prepare_matrix_optimizer(optimizer, model)  # replaces the first preparation
    assert optimizer.matrix_fsdp is again and prepared._removed
    again.remove()
    assert not hasattr(optimizer, "matrix_fsdp") and not hasattr(optimizer, "state_manager")
    optimizer.zero_grad()  # the class's own method again

    # no_sync on the optimizer: neither step nor zero_grad inside it
    optimizer = torch.optim.SGD(model.parameters(), lr=0.1)
    with optimizer.no_sync():
        with pytest.raises(RuntimeError, match="cannot run inside no_sync"):
            optimizer.step()
        with pytest.raises(RuntimeError, match="cannot run inside no_sync"):
            optimizer.zero_grad()
    assert not unit.is_no_sync_active()

    # optimizers over foreign parameters are left alone; wrappers keep their inner optimizers unprepared
    assert not hasattr(torch.optim.SGD(nn.Linear(2, 2).parameters(), lr=0.1), "matrix_fsdp")
    mixed = configure_optimizer(model, "mixed_muon_adamw", lr=0.01)
    assert all(not hasattr(opt, "matrix_fsdp") for _, opt in mixed.iter_named_optimizers())
    assert isinstance(configure_optimizer(model, "adamw", lr=0.01).matrix_fsdp, PreparedMatrixOptimizer)

    muon = torch.optim.Muon(matrix_fully_shard(nn.Linear(4, 2, bias=False).to(DEV)).parameters(), lr=0.01)
    assert isinstance(muon.matrix_fsdp, PreparedMatrixOptimizer)


@pytest.mark.parametrize("set_to_none", [True, False])
def test_auto_prepared_sgd_matches_eager_over_several_steps(set_to_none):
    from matrix_fsdp_amd import PreparedMatrixOptimizer

    model, twin = make_pair(seed=21)
    shard_all(model, world_size=1, rank=0)
    opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9)
    ref = torch.optim.SGD(twin.parameters(), lr=0.1, momentum=0.9)
    assert isinstance(opt.matrix_fsdp, PreparedMatrixOptimizer) and len(opt.matrix_fsdp.fsdp_param_groups) == 3
    for x, y in batches(3, seed=22):
        for net, optimizer in ((model, opt), (twin, ref)):
            torch.nn.functional.mse_loss(net(x), y).backward()
            optimizer.step()
            optimizer.zero_grad(set_to_none=set_to_none)
        assert all(unit.flat_buffer.local_grad_shard is None for unit in opt.matrix_fsdp.fsdp_param_groups)
    ours, theirs = named_full_params(model), named_full_params(twin)
    for name in theirs:
        assert rel(ours[name], theirs[name]) < 2e-6, name


class TransposedLinear(nn.Module):
    """``x @ w.t()`` spelled out: autograd saves the view ``w.t()``, not the parameter."""

    def __init__(self, dim: int) -> None:
        super().__init__()
        self.w = nn.Parameter(torch.randn(dim, dim) / dim**0.5)

    def forward(self, x):
        return torch.tanh(x @ self.w.t())


def _stack(dim: int, depth: int, seed: int):
    torch.manual_seed(seed)
    model = nn.Sequential(*[TransposedLinear(dim) for _ in range(depth)]).to(DEV)
    return model, copy.deepcopy(model)


def test_saved_tensor_hooks_free_full_buffers_between_forward_and_backward():
    """Without the hooks the views autograd saved keep every layer's full buffer alive until the backward; with them
    a resharded layer's buffer is really gone (matrix_fsdp/runtime/fsdp_unit.py:1355-1382).  Gradients are the same
    either way, and the same as the eager twin's."""
    from matrix_fsdp_amd import matrix_fully_shard

    dim, depth, world = 512, 6, 4
    full_bytes = dim * dim * 4
    held, grads = {}, {}
    x = torch.randn(8, dim, device=DEV)
    for hooks in (False, True, False):  # the first pass also pays for the libraries' one-time workspaces
        model, twin = _stack(dim, depth, seed=3)
        for layer in model:
            matrix_fully_shard(layer, world_size=world, rank=1, use_saved_tensor_hooks=hooks)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        out = model(x)
        held[hooks] = torch.cuda.memory_allocated() - before
        out.square().mean().backward()
        units = [layer._matrix_fsdp_param_group for layer in model]
        assert all(u.lifecycle_state == FSDPLifecycleState.SHARDED for u in units)
        # the first layer's input needs no gradient, so its product keeps no view of the weight
        assert sum(u.saved_full_param_views for u in units) == (depth - 1 if hooks else 0)
        twin(x).square().mean().backward()
        for unit, ref_layer in zip(units, twin):
            want = ref_layer.w.grad.view(-1).chunk(world)[1]  # the other ranks of the simulated world contribute nothing
            assert rel(unit.flat_buffer.local_grad_shard, want) < 1e-6
        grads[hooks] = torch.cat([u.flat_buffer.local_grad_shard for u in units])
    assert torch.equal(grads[True], grads[False])
    assert held[False] - held[True] >= (depth - 2) * full_bytes, held  # every pinned buffer but (at most) the last layer's
    assert held[True] < 2 * full_bytes + depth * 8 * dim * 4 * 4, held


def test_full_param_buffer_pool_shares_one_buffer_between_equal_units():
    """Equal layers unshard into the same storage, forward and backward, and still train like the eager twin: what
    autograd saved of a layer's parameters is rebuilt on the buffer gathered for that layer's backward."""
    from matrix_fsdp_amd import FullParamBufferPool, matrix_fully_shard

    dim, depth, world = 256, 4, 2
    pool = FullParamBufferPool(max_cached_per_key=1)
    model, twin = _stack(dim, depth, seed=4)
    for layer in model:
        matrix_fully_shard(layer, world_size=world, rank=0, full_param_buffer_pool=pool)
    units = [layer._matrix_fsdp_param_group for layer in model]
    seen = set()
    for unit in units:
        unit.unshard()
        seen.add(unit.flat_buffer.full_buffer.data_ptr())
        assert unit.flat_buffer.param_data_alias_full_buffer()
        unit.reshard()
        assert unit.flat_buffer.full_buffer is None
    assert len(seen) == 1 and pool.stats()["allocations"] == 1 and pool.stats()["reuses"] == depth - 1
    opt = configure_optimizer(model, "adamw", lr=1e-2, weight_decay=0.0)
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-2, weight_decay=0.0, foreach=False)
    gen = torch.Generator().manual_seed(5)
    for _ in range(3):
        x = torch.randn(16, dim, generator=gen).to(DEV)
        model(x).square().mean().backward()
        opt.step()
        opt.zero_grad()
        before = [p.detach().clone() for p in twin.parameters()]
        twin(x).square().mean().backward()
        ref.step()
        ref.zero_grad()
        with torch.no_grad():  # the other rank of the simulated world never steps
            for p, old in zip(twin.parameters(), before):
                half = p.numel() // world
                p.view(-1)[half:] = old.view(-1)[half:]
    for unit, ref_layer in zip(units, twin):
        assert rel(unit.flat_buffer.local_shard, ref_layer.w.detach().view(-1)[: dim * dim // world]) < 2e-6
    stats = pool.stats()
    assert stats["allocations"] <= 2 and stats["reuses"] >= 3 * 2 * depth - 1, stats


class SkippableTail(nn.Module):
    def __init__(self) -> None:
        super().__init__()
        self.body = nn.Sequential(nn.Linear(32, 48), nn.GELU(), nn.Linear(48, 16))
        self.tail = nn.Linear(16, 16)

    def forward(self, x, use_tail: bool = True):
        x = self.body(x)
        return self.tail(x) if use_tail else x


@pytest.mark.parametrize("world, rank, planner, applies", [(1, 0, None, True), (3, 1, "owner", True), (4, 2, fsdp2_chunk_plan, False)])
def test_zero_copy_grad_bucket_through_the_lifecycle(world, rank, planner, applies):
    """``use_zero_copy_grad_bucket``: autograd accumulates into views of the reduce-scatter workspace, the backward
    has no copy-in launch, and the reduced shard equals the copy-in path's bit for bit -- also over two
    accumulated backwards and with an unused parameter.  Per-parameter chunks scatter a parameter over the
    workspace's rows, so there the bucket declines and the copy-in path runs (test/fsdp/test_flat_buffer.py:1049-1063)."""
    from matrix_fsdp_amd import matrix_fully_shard

    shards = {}
    for zero_copy in (False, True):
        torch.manual_seed(7)
        model = SkippableTail().to(DEV)
        kwargs = {}
        if planner == "owner":
            kwargs["planner"] = lambda mps, w: whole_param_owner_plan(mps, w, [i % w for i in range(len(mps))])
        elif planner is not None:
            kwargs["planner"] = planner
        matrix_fully_shard(model, world_size=world, rank=rank, use_zero_copy_grad_bucket=zero_copy, **kwargs)
        unit = model._matrix_fsdp_param_group
        gen = torch.Generator().manual_seed(8)
        for micro in range(2):
            x = torch.randn(8, 32, generator=gen).to(DEV)
            out = model(x, use_tail=micro == 1)  # the first micro-batch leaves the last layer unused
            out.square().mean().backward()
            assert unit.lifecycle_state == FSDPLifecycleState.SHARDED and unit.flat_buffer.grad_bucket_input is None
        assert ("zero_copy_grad_bucket" in unit.events) == (zero_copy and applies)
        shards[zero_copy] = unit.flat_buffer.local_grad_shard.clone()
        assert all(p.grad is None or p.grad.untyped_storage().data_ptr() == unit.flat_buffer.local_grad_shard.untyped_storage().data_ptr() for p in model.parameters())
    assert torch.equal(shards[True], shards[False])


def test_zero_copy_grad_bucket_declines_under_mixed_precision():
    from matrix_fsdp_amd import matrix_fully_shard

    model = nn.Linear(16, 16).to(DEV)
    matrix_fully_shard(model, world_size=2, rank=0, use_zero_copy_grad_bucket=True, mp_policy=MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.float32))
    model(torch.randn(4, 16, device=DEV)).float().square().mean().backward()
    unit = model._matrix_fsdp_param_group
    assert "zero_copy_grad_bucket" not in unit.events and unit.flat_buffer.local_grad_shard.dtype == torch.float32


class TinyExpert(nn.Module):
    def __init__(self, dim: int, hidden: int) -> None:
        super().__init__()
        self.w1 = nn.Linear(dim, hidden, bias=True)
        self.w2 = nn.Linear(hidden, dim, bias=False)

    def forward(self, x):
        return self.w2(torch.nn.functional.silu(self.w1(x)))


class TinyMoE(nn.Module):
    """Dense soft routing (every expert sees every token, weighted by the router): all parameters get gradients."""

    def __init__(self, dim: int = 32, hidden: int = 64, experts: int = 4) -> None:
        super().__init__()
        self.router = nn.Linear(dim, experts, bias=False)
        self.experts = nn.ModuleList(TinyExpert(dim, hidden) for _ in range(experts))
        self.norm = nn.LayerNorm(dim)

    def forward(self, x):
        gates = torch.softmax(self.router(x), dim=-1)
        mixed = sum(gates[:, i : i + 1] * expert(x) for i, expert in enumerate(self.experts))
        return self.norm(x + mixed)


@pytest.mark.parametrize("rank", [0, 1])
def test_expert_owner_layout_trains_like_eager(rank):
    """Structure-derived hints mark every expert's parameters as one group; ``expert_owner_tail_plan`` keeps each
    group on one rank of a simulated world of 2 and fills up with the router and the norm.  The unit runs that
    layout as planned (several whole-parameter segments per rank, not in flat order) and AdamW on the owned
    parameters matches the eager twin."""
    from matrix_fsdp_amd import expert_owner_tail_plan, matrix_fully_shard, validate_group_layout

    world = 2
    torch.manual_seed(31)
    model = TinyMoE().to(DEV)
    twin = copy.deepcopy(model)
    matrix_fully_shard(model, world_size=world, rank=rank, auto_shard_hints=True, planner=expert_owner_tail_plan)
    unit = model._matrix_fsdp_param_group
    validate_group_layout(unit.group_layout, unit.managed_params, world)  # one owner rank per expert group
    owners = {mp.fqn: unit.owner_ranks(mp.fqn) for mp in unit.managed_params}
    assert all(len(ranks) == 1 for ranks in owners.values())
    for e in range(4):
        assert len({owners[f"experts.{e}.{name}"] for name in ("w1.weight", "w1.bias", "w2.weight")}) == 1
    assert {owners[f"experts.{e}.w1.weight"][0] for e in range(4)} == {0, 1}
    assert unit.runtime_layout_compatibility.mode in ("flat_reorder", "matrix_shard")
    opt = configure_optimizer(model, "adamw", lr=1e-2, weight_decay=0.01)
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-2, weight_decay=0.01, foreach=False)
    twin_named = dict(twin.named_parameters())
    gen = torch.Generator().manual_seed(32)
    for _ in range(3):
        x, y = torch.randn(16, 32, generator=gen).to(DEV), torch.randn(16, 32, generator=gen).to(DEV)
        torch.nn.functional.mse_loss(model(x), y).backward()  # (a loss of the normalised output alone would be constant)
        opt.step()
        opt.zero_grad()
        before = {n: p.detach().clone() for n, p in twin_named.items()}
        torch.nn.functional.mse_loss(twin(x), y).backward()
        ref.step()
        ref.zero_grad()
        with torch.no_grad():
            for n, p in twin_named.items():
                if owners[n] != (rank,):
                    p.copy_(before[n])
    for n, p in model.named_parameters():
        if owners[n] == (rank,):
            assert p.shape == twin_named[n].shape and rel(p.detach().cpu(), twin_named[n].detach().cpu()) < 2e-6, n
        else:
            assert p.numel() == 0, n
