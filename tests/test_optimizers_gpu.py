"""Optimizer classes on a HIP device: same surface and state as the torch optimizers the reference
instantiates, results within the Muon / AdamW tolerances of those optimizers run on the CPU."""
import pytest
import torch
from torch import nn

from matrix_fsdp_amd import ParamShardHint, managed_params_from_named
from matrix_fsdp_amd.core.plans import whole_param_owner_plan
from matrix_fsdp_amd.optim.adamw import FusedAdamW
from matrix_fsdp_amd.optim.adamw_state import initialize_flat_adamw_state
from matrix_fsdp_amd.optim.muon import Muon
from matrix_fsdp_amd.optim.wrapper import (
    MixedMuonAdamWOptimizer,
    classify_matrix_optimizer_params,
    configure_optimizer,
)
from matrix_fsdp_amd.runtime.flat_buffer import MatrixFlatBuffer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rel_fro(have, want):
    have, want = have.detach().double().cpu(), want.detach().double().cpu()
    return float(torch.linalg.norm(have - want) / torch.linalg.norm(want))


def test_muon_class_matches_torch_muon_over_steps():
    gen = torch.Generator().manual_seed(0)
    p0 = torch.randn(256, 384, generator=gen) * 0.02
    ref = nn.Parameter(p0.clone())
    ours = nn.Parameter(p0.clone().to(DEV))
    kw = dict(lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True, ns_steps=5, adjust_lr_fn="match_rms_adamw")
    opt_ref, opt = torch.optim.Muon([ref], **kw), Muon([ours], **kw)
    assert opt.defaults == opt_ref.defaults
    for step in range(3):
        g = (torch.randn(256, 384, generator=gen) * 1e-3).bfloat16().float()
        before = ref.detach().clone()
        ref.grad, ours.grad = g.clone(), g.to(DEV)
        opt_ref.step()
        ours.data.copy_(before)  # compare one step at a time from identical parameters
        opt.state[ours].get("momentum_buffer", torch.zeros(0)).numel() and opt.state[ours]["momentum_buffer"].copy_(prev_buf)
        opt.step()
        prev_buf = opt_ref.state[ref]["momentum_buffer"].clone()
        assert rel_fro(ours.detach().cpu() - before, ref.detach() - before) < 1e-2
        assert torch.allclose(opt.state[ours]["momentum_buffer"].cpu(), prev_buf, rtol=1e-5, atol=1e-9)
    assert set(opt.state[ours]) == {"momentum_buffer"}
    sd = opt.state_dict()
    assert sd["param_groups"][0]["ns_steps"] == 5 and sd["param_groups"][0]["adjust_lr_fn"] == "match_rms_adamw"
    with pytest.raises(ValueError, match="2D"):
        Muon([nn.Parameter(torch.zeros(3, device=DEV))])
    with pytest.raises(ValueError, match="not supported"):
        Muon([ours], adjust_lr_fn="bogus")


def test_fused_adamw_merges_flat_views_into_one_launch_and_matches_torch():
    gen = torch.Generator().manual_seed(1)
    sizes = [(12, 5), (7,), (3, 3)]
    total = sum(torch.Size(s).numel() for s in sizes)
    flat_p = (torch.randn(total, generator=gen) * 0.02).to(DEV)
    flat_g = (torch.randn(total, generator=gen) * 1e-3).to(DEV)
    ours, refs, off = [], [], 0
    for s in sizes:
        n = torch.Size(s).numel()
        p = nn.Parameter(flat_p[off : off + n].view(s))
        p.grad = flat_g[off : off + n].view(s)
        ours.append(p)
        r = nn.Parameter(flat_p[off : off + n].view(s).cpu().clone())
        r.grad = flat_g[off : off + n].view(s).cpu().clone()
        refs.append(r)
        off += n
    kw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    opt, opt_ref = FusedAdamW(ours, **kw), torch.optim.AdamW(refs, foreach=False, **kw)
    # flat state: the moments of neighbouring parameters are neighbours too
    exp_avg, exp_avg_sq = torch.zeros(total, device=DEV), torch.zeros(total, device=DEV)
    off = 0
    for p in ours:
        n = p.numel()
        opt.state[p] = {"step": torch.tensor(0.0), "exp_avg": exp_avg[off : off + n].view_as(p), "exp_avg_sq": exp_avg_sq[off : off + n].view_as(p)}
        off += n
    from matrix_fsdp_amd.optim import adamw as adamw_module

    entries = [(p.data, p.grad, opt.state[p]["exp_avg"], opt.state[p]["exp_avg_sq"], 1) for p in ours]
    assert len(list(adamw_module._merge_contiguous(entries))) == 1
    for _ in range(2):
        opt.step()
        opt_ref.step()
    for p, r in zip(ours, refs):
        assert torch.allclose(p.detach().cpu(), r.detach(), rtol=1e-6, atol=1e-8)
        assert torch.allclose(opt.state[p]["exp_avg"].cpu(), opt_ref.state[r]["exp_avg"], rtol=1e-5, atol=1e-10)
        assert float(opt.state[p]["step"]) == 2.0
    with pytest.raises(ValueError, match="Invalid beta"):
        FusedAdamW(ours, betas=(1.0, 0.9))


def test_fused_adamw_lays_out_its_own_moments_for_contiguous_parameters(monkeypatch):
    """Without any flat-state set-up: parameters that are views of one shard get back-to-back moments at the first
    step, so the whole run is one launch per step; a parameter elsewhere in memory keeps its own launch; amsgrad
    adds its running maximum to the same layout.  Results as ``torch.optim.AdamW``."""
    from matrix_fsdp_amd.optim import adamw as adamw_module

    gen = torch.Generator().manual_seed(3)
    sizes = [(6, 4), (5,), (2, 8)]
    total = sum(torch.Size(s).numel() for s in sizes)
    flat_p = (torch.randn(total, generator=gen) * 0.02).to(DEV)
    ours, refs, off = [], [], 0
    for s in sizes + [(9,)]:
        n = torch.Size(s).numel()
        p = nn.Parameter(flat_p[off : off + n].view(s)) if s != (9,) else nn.Parameter((torch.randn(9, generator=gen) * 0.02).to(DEV))
        ours.append(p)
        refs.append(nn.Parameter(p.detach().cpu().clone()))
        off += n
    kw = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-8, weight_decay=0.05, amsgrad=True)
    opt, opt_ref = FusedAdamW(ours, **kw), torch.optim.AdamW(refs, foreach=False, **kw)
    launches = []
    real = adamw_module.F.adamw_step
    monkeypatch.setattr(adamw_module.F, "adamw_step", lambda *a, **k: (launches.append(a[0].numel()), real(*a, **k))[1])
    for step in range(3):
        flat_g = (torch.randn(total + 9, generator=gen) * 1e-3).to(DEV)  # one grad shard, as after a backward
        off = 0
        for p, r in zip(ours, refs):
            p.grad = flat_g[off : off + p.numel()].view(p.shape)
            r.grad = p.grad.cpu().clone()
            off += p.numel()
        launches.clear()
        opt.step()
        opt_ref.step()
        assert sorted(launches) == [9, total], launches
    first, second = opt.state[ours[0]], opt.state[ours[1]]
    for name in ("exp_avg", "exp_avg_sq", "max_exp_avg_sq"):
        assert second[name].data_ptr() == first[name].data_ptr() + ours[0].numel() * 4 and first[name].shape == ours[0].shape
    for p, r in zip(ours, refs):
        assert torch.allclose(p.detach().cpu(), r.detach(), rtol=1e-6, atol=1e-8)
        for name in ("exp_avg", "exp_avg_sq", "max_exp_avg_sq"):
            assert torch.allclose(opt.state[p][name].cpu(), opt_ref.state[r][name], rtol=1e-5, atol=1e-12), name
    # a state dict loaded back gives every parameter its own tensors again: still correct, one launch each
    opt.load_state_dict(opt.state_dict())
    launches.clear()
    opt.step()
    opt_ref.step()
    assert len(launches) in (2, 4)
    for p, r in zip(ours, refs):
        assert torch.allclose(p.detach().cpu(), r.detach(), rtol=1e-6, atol=1e-8)


def build_owner_buffers():
    """Two units; every matrix whole on its owner, rank 0 owning every second parameter."""
    gen = torch.Generator().manual_seed(2)
    buffers, all_named = [], []
    for unit in range(2):
        named = [
            (f"l{unit}.w_a", nn.Parameter((torch.randn(64, 128, generator=gen) * 0.02).to(DEV))),
            (f"l{unit}.norm", nn.Parameter(torch.ones(128, device=DEV))),
            (f"l{unit}.w_b", nn.Parameter((torch.randn(128, 64, generator=gen) * 0.02).to(DEV))),
            (f"l{unit}.bias", nn.Parameter(torch.zeros(64, device=DEV))),
        ]
        # flat order after the runtime's rank-major reorder: rank 0's parameters first
        owners = [0, 0, 1, 1]
        mps = list(managed_params_from_named(named, shard_hints={f"l{unit}.w_a": ParamShardHint(optimizer_type="muon")}))
        buffers.append(MatrixFlatBuffer(mps, whole_param_owner_plan(mps, 2, owners), rank=0))
        all_named.extend(named)
    return buffers, all_named


def test_classify_and_mixed_optimizer_step_with_flat_adamw_state():
    buffers, named = build_owner_buffers()
    classified = classify_matrix_optimizer_params(buffers)
    assert [tuple(p.shape) for p in classified.muon_params] == [(64, 128), (64, 128)]
    assert [tuple(p.shape) for p in classified.adamw_params] == [(128,), (128,)]
    assert {g.name for g in classified.group_summaries} == {"muon", "adamw"}
    opt = configure_optimizer(buffers, "mixed_muon_adamw", lr=1e-3, flat_adamw_state=True)
    assert isinstance(opt, MixedMuonAdamWOptimizer)
    assert opt.defaults["muon"]["momentum"] == 0.5 and opt.defaults["muon"]["ns_steps"] == 2
    assert opt.defaults["muon"]["adjust_lr_fn"] == "match_rms_adamw" and opt.defaults["adamw"]["weight_decay"] == 0.01
    # eager twins on the CPU
    twins = {}
    for fb in buffers:
        for view in fb.local_param_views:
            p = view.managed_param.param
            twins[id(p)] = nn.Parameter(p.detach().cpu().clone())
    ref_muon = torch.optim.Muon([twins[id(p)] for p in classified.muon_params], lr=1e-3, momentum=0.5, ns_steps=2, weight_decay=0.01, adjust_lr_fn="match_rms_adamw")
    ref_adamw = torch.optim.AdamW([twins[id(p)] for p in classified.adamw_params], lr=1e-3, weight_decay=0.01, foreach=False)
    gen = torch.Generator().manual_seed(3)
    for _ in range(2):
        for p in classified.muon_params + classified.adamw_params:
            g = (torch.randn(p.shape, generator=gen) * 1e-3).bfloat16().float()
            p.grad, twins[id(p)].grad = g.to(DEV), g.clone()
        befores = {id(p): twins[id(p)].detach().clone() for p in classified.muon_params}
        for p in classified.muon_params:  # identical starting points each step
            p.data.copy_(befores[id(p)])
        opt.step()
        ref_muon.step()
        ref_adamw.step()
        for p in classified.muon_params:
            assert rel_fro(p.detach().cpu() - befores[id(p)], twins[id(p)].detach() - befores[id(p)]) < 1e-2
            twins_buf = ref_muon.state[twins[id(p)]]["momentum_buffer"]
            opt.state[p]["momentum_buffer"].copy_(twins_buf)
        for p in classified.adamw_params:
            assert torch.allclose(p.detach().cpu(), twins[id(p)].detach(), rtol=1e-6, atol=1e-8)
    # flat AdamW state: views into one buffer sized to the sum of local shards, at flat_base + shard_start
    state_buffers = opt.adamw._matrix_fsdp_flat_adamw_state_buffers
    (buf,) = state_buffers.values()
    assert buf.total_numel == sum(fb.local_shard.numel() for fb in buffers)
    base = 0
    for fb in buffers:
        for view in fb.local_param_views:
            p = view.managed_param.param
            if p.ndim == 1:
                assert opt.state[p]["exp_avg"].data_ptr() == buf.exp_avg.data_ptr() + 4 * (base + view.shard_start)
        base += fb.local_shard.numel()
    sd = opt.state_dict()
    assert set(sd) == {"muon", "adamw", "group_summaries"}
    opt.load_state_dict(sd)
    opt.zero_grad()
    with pytest.raises(NotImplementedError):
        opt.add_param_group({})
    with pytest.raises(NotImplementedError):
        opt.step(closure=lambda: None)
    assert opt.optimizer_group_summary()["optimizer"] == "mixed_muon_adamw"
    assert [name for name, _ in opt.iter_named_optimizers()] == ["muon", "adamw"]


def test_muon_hint_on_partial_parameter_is_rejected():
    named = [("w", nn.Parameter(torch.zeros(8, 8, device=DEV)))]
    mps = list(managed_params_from_named(named, shard_hints={"w": ParamShardHint(optimizer_type="muon")}))
    from matrix_fsdp_amd.core.plans import contiguous_even_plan

    fb = MatrixFlatBuffer(mps, contiguous_even_plan(64, 2), rank=0)
    with pytest.raises(ValueError, match="not a full 2D matrix"):
        classify_matrix_optimizer_params([fb])
    with pytest.raises(ValueError, match="optimizer must be one of"):
        configure_optimizer([fb], "lion")
    assert isinstance(configure_optimizer([fb], "adamw", lr=1e-3), FusedAdamW)


def test_hip_optimizers_are_torch_optimizers_of_the_same_kind():
    """``configure_optimizer(..., "adamw")`` is a ``torch.optim.AdamW`` in the reference
    (test/fsdp/test_matrix_fsdp_e2e.py:1911-1912); the HIP optimizers subclass torch's, share their constructor
    checks and their state-dict layout, and take the reference's scheduler keywords without effect."""
    from matrix_fsdp_amd import configure_optimizer, fully_shard
    from matrix_fsdp_amd.optim.muon import Muon

    model = nn.Sequential(nn.Linear(8, 8), nn.Linear(8, 4)).to(DEV)
    fully_shard(model)
    opt = configure_optimizer(model, "adamw", lr=1e-2, max_forward_prefetch_units=2, prefetch_policy="static", trim_cuda_cache=True)
    assert isinstance(opt, torch.optim.AdamW) and isinstance(opt, FusedAdamW)
    twin = torch.optim.AdamW([nn.Parameter(p.detach().clone()) for p in model.parameters()], lr=1e-2, foreach=False)
    assert set(opt.param_groups[0]) == set(twin.param_groups[0])
    model(torch.randn(4, 8, device=DEV)).sum().backward()
    opt.step()
    twin.load_state_dict(opt.state_dict())  # interchangeable state dicts
    assert float(twin.state[twin.param_groups[0]["params"][0]]["step"]) == 1.0
    muon = Muon([p for p in model.parameters() if p.ndim == 2], lr=1e-2)
    assert isinstance(muon, torch.optim.Muon)
    with pytest.raises(ValueError, match="only supports 2D"):
        Muon(list(model.parameters()))
    with pytest.raises(ValueError, match="Learning rate should be >= 0"):
        Muon([p for p in model.parameters() if p.ndim == 2], lr=-1.0)
    flat = configure_optimizer(model, "adamw", lr=1e-2, flat_adamw_state=True)
    model(torch.randn(4, 8, device=DEV)).sum().backward()
    flat.step()
    first, second = (flat.state[p]["exp_avg"] for p in list(model.parameters())[:2])
    assert second.data_ptr() == first.data_ptr() + first.numel() * 4


def test_mixed_optimizer_takes_the_reference_constructor_and_delays_muon_state():
    """test/fsdp/test_bench_fsdp2_compare.py:406-424 and the construction of bench_fsdp2_compare.py:2648:
    ``MixedMuonAdamWOptimizer(muon_params, adamw_params, lazy_muon_init=True)`` holds no state before the first step,
    and steps like the eager optimizer afterwards."""
    from matrix_fsdp_amd.optim.wrapper import DEFAULT_MUON_ADJUST_LR_FN, LazyMuon

    matrix = nn.Parameter(torch.ones(4, 4, device=DEV))
    eager = MixedMuonAdamWOptimizer([matrix], [])
    assert DEFAULT_MUON_ADJUST_LR_FN == "match_rms_adamw"
    assert eager.muon is not None and eager.muon.param_groups[0]["adjust_lr_fn"] == DEFAULT_MUON_ADJUST_LR_FN
    lazy = MixedMuonAdamWOptimizer([matrix], [], lazy_muon_init=True)
    assert lazy.state == {}
    assert lazy.muon.state_dict()["state"] == {}
    assert lazy.muon.param_groups[0]["adjust_lr_fn"] == DEFAULT_MUON_ADJUST_LR_FN
    assert isinstance(lazy.muon, LazyMuon) and lazy.muon.state_dict()["param_groups"][0]["params"] == [0]

    # the bench's construction: every 2-D parameter to Muon, the rest to AdamW, built lazily
    gen = torch.Generator().manual_seed(11)
    shapes = [(128, 256), (256,), (256, 128), (128,)]
    params = [nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(DEV)) for s in shapes]
    twins = [nn.Parameter(p.detach().clone()) for p in params]
    split = lambda ps: ([p for p in ps if p.ndim == 2 and p.numel() > 0], [p for p in ps if p.ndim != 2 and p.numel() > 0])
    opt = MixedMuonAdamWOptimizer(*split(params), lazy_muon_init=True, adamw_foreach=False, max_forward_prefetch_units=2,
                                  prefetch_policy="static", scheduler_config=None, trim_cuda_cache=False)
    ref = MixedMuonAdamWOptimizer(*split(twins))
    assert opt.state == {} and opt.defaults["muon"] == {k: v for k, v in ref.defaults["muon"].items() if k in opt.defaults["muon"]}
    opt.zero_grad()  # nothing to clear yet, and nothing gets built by it
    assert opt.muon.state == {}
    for step in range(2):
        for p, t in zip(params, twins):
            g = (torch.randn(p.shape, generator=gen) * 1e-3).to(DEV)
            p.grad, t.grad = g.clone(), g.clone()
        opt.step()
        ref.step()
        for p, t in zip(params, twins):
            assert torch.equal(p.detach(), t.detach())  # same kernels, same order: bit-identical to the eager construction
    assert set(opt.muon.state[params[0]]) == {"momentum_buffer"}
    assert opt.state_dict()["muon"]["state"].keys() == ref.state_dict()["muon"]["state"].keys()
    opt.load_state_dict(ref.state_dict())
    fresh = MixedMuonAdamWOptimizer(*split(params), lazy_muon_init=True)
    fresh.load_state_dict(ref.state_dict())  # loading builds the optimizer
    assert torch.equal(fresh.muon.state[params[0]]["momentum_buffer"], ref.muon.state[twins[0]]["momentum_buffer"])
    with pytest.raises(TypeError, match="unexpected keyword argument 'bogus'"):
        MixedMuonAdamWOptimizer([matrix], [], bogus=1)
