"""MatrixFSDP state dicts and DCP checkpoints on one HIP device.

The cases of the reference's own checkpoint and optimizer-state tests (test/fsdp/test_checkpoint.py:129-787,
test/fsdp/test_optim_state.py:22-242) for the features this runtime has, followed by loads into other layouts,
which the simulated world makes checkable on one device: every rank of the saved world and every rank of the target
world is built here, and whatever the target ranks hold afterwards must be, bit for bit, the matching slice of what
a one-rank run of the same model holds."""
import copy

import pytest
import torch
from torch import nn
from torch.distributed.checkpoint.state_dict import StateDictOptions

from matrix_fsdp_amd import FSDPLifecycleState, ParamShardHint, configure_optimizer, fully_shard, matrix_fully_shard
from matrix_fsdp_amd.checkpoint import (
    get_model_state_dict,
    get_optimizer_state_dict,
    get_state_dict,
    load_matrix_dcp,
    load_matrix_dcp_full_state,
    load_matrix_state_dict,
    matrix_get_state_dict,
    matrix_set_state_dict,
    matrix_state_dict,
    patch_model_state_dict,
    patch_optimizer_state_dict,
    save_matrix_dcp,
    save_matrix_dcp_simulated_world,
    set_model_state_dict,
    set_optimizer_state_dict,
    set_state_dict,
)
from matrix_fsdp_amd.core.plans import contiguous_even_plan, fsdp2_chunk_plan, whole_param_owner_plan
from matrix_fsdp_amd.optim.adamw import FusedAdamW
from matrix_fsdp_amd.optim.state import MatrixFSDPOptimizerStateManager
from matrix_fsdp_amd.optim.wrapper import MatrixFSDPOptimizer
from oracle import copy_oracle as CO

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def small_model() -> nn.Module:
    return nn.Sequential(nn.Linear(4, 8), nn.ReLU(), nn.Linear(8, 2)).to(DEV)


def linear() -> nn.Module:
    return nn.Linear(4, 2).to(DEV)


def one_step(model, optimizer, seed: int = 7) -> None:
    x = torch.randn(3, 4, generator=torch.Generator().manual_seed(seed)).to(DEV)
    optimizer.zero_grad()
    model(x).sum().backward()
    optimizer.step()


def global_metadata(folder) -> dict:
    return torch.load(folder / "matrix_metadata.pt", map_location="cpu", weights_only=True)


def rewrite_rank_metadata(folder, metadata: dict, rank: int = 0) -> None:
    payload = global_metadata(folder)
    payload["ranks"][rank] = metadata
    torch.save(payload, folder / "matrix_metadata.pt")


def assert_optimizer_state_equal(actual: dict, expected: dict) -> None:
    assert actual["param_groups"] == expected["param_groups"]
    assert set(actual["state"]) == set(expected["state"])
    for state_id, want in expected["state"].items():
        have = actual["state"][state_id]
        assert set(have) == set(want)
        for name, value in want.items():
            if torch.is_tensor(value):
                assert torch.equal(have[name].cpu(), value.cpu()), name
            else:
                assert have[name] == value


def tensor_devices(value) -> list[torch.device]:
    if torch.is_tensor(value):
        return [value.device]
    if isinstance(value, dict):
        return [d for item in value.values() for d in tensor_devices(item)]
    if isinstance(value, (list, tuple)):
        return [d for item in value for d in tensor_devices(item)]
    return []


# ------------------------------------------------------------------------------------------------ state dicts


def test_sharded_state_dict_describes_and_restores_the_local_shard():
    torch.manual_seed(0)
    model = small_model()
    eager = copy.deepcopy(model)
    matrix_fully_shard(model)
    unit = model._matrix_fsdp_param_group
    fb = unit.flat_buffer

    state = matrix_state_dict(model)
    assert state["metadata"] == {"version": 1, "state_dict_type": "matrix_sharded", "num_param_groups": 1, "num_units": 1, "include_grads": False}
    assert len(state["param_groups"]) == 1 and state["param_groups"][0] is state["units"][0]
    saved = state["units"][0]
    assert saved["param_group_index"] == 0 and saved["module_fqn"] == ""
    assert saved["param_fqns"] == ("0.weight", "0.bias", "2.weight", "2.bias")
    assert saved["matrix_shard"] == {"dims": (0,), "local_units": (1,)}
    assert saved["param_shard_state"]["name"] == "param"
    assert saved["param_shard_state"]["local_numel"] == fb.local_numel == 58
    assert saved["param_shard_state"]["matrix_shard"] == {"type": "MatrixShard", "dims": (0,), "local_units": (1,)}
    assert saved["layout"]["total_numel"] == 58 and saved["layout"]["shard_sizes"] == (58,)
    assert saved["params"]["2.weight"]["offset"] == 40 and saved["params"]["2.weight"]["shape"] == (2, 8)
    assert saved["params"]["2.weight"]["owner_ranks"] == (0,) and saved["params"]["2.weight"]["shard_sizes"] == (16,)
    assert saved["mixed_precision"] == {"param_dtype": None, "reduce_dtype": None, "output_dtype": None, "cast_forward_inputs": True}
    assert saved["param_shard"].data_ptr() != fb.local_shard.data_ptr()  # a copy by default

    fb.local_shard.add_(10.0)
    load_matrix_state_dict(model, state)
    assert unit.lifecycle_state == FSDPLifecycleState.SHARDED
    assert torch.equal(fb.local_shard, saved["param_shard"])
    unit.unshard()
    for want, have in zip(eager.parameters(), model.parameters()):
        assert torch.equal(want, have)


def test_state_dict_tuple_apis_round_trip_model_and_optimizer():
    torch.manual_seed(0)
    model = matrix_fully_shard(small_model())
    optimizer = configure_optimizer(model, "adamw", lr=0.01)
    one_step(model, optimizer)

    model_state, optim_state = matrix_get_state_dict(model, optimizer, options=StateDictOptions(cpu_offload=True))
    assert model_state["metadata"]["state_dict_type"] == "matrix_sharded"
    assert tensor_devices(model_state) and all(d.type == "cpu" for d in tensor_devices(model_state) + tensor_devices(optim_state))
    model_only = get_model_state_dict(model, options=StateDictOptions(cpu_offload=True))
    assert torch.equal(model_state["param_groups"][0]["param_shard"], model_only["param_groups"][0]["param_shard"])
    assert get_state_dict(model, optimizer)[1]["param_groups"] == get_optimizer_state_dict(model, optimizer)["param_groups"] == optim_state["param_groups"]

    torch.manual_seed(1234)
    restored = matrix_fully_shard(small_model())
    restored_optimizer = configure_optimizer(restored, "adamw", lr=0.2)
    matrix_set_state_dict(restored, restored_optimizer, model_state_dict=model_state, optim_state_dict=optim_state)
    want = model._matrix_fsdp_param_group.flat_buffer.local_shard
    have = restored._matrix_fsdp_param_group.flat_buffer.local_shard
    assert torch.equal(have, want)
    assert_optimizer_state_equal(restored_optimizer.state_dict(), optimizer.state_dict())

    have.add_(1.0)
    set_model_state_dict(restored, model_state)
    assert torch.equal(have, want)
    restored_optimizer.param_groups[0]["lr"] = 0.2
    set_optimizer_state_dict(restored, restored_optimizer, optim_state)
    assert restored_optimizer.state_dict()["param_groups"] == optimizer.state_dict()["param_groups"]
    have.add_(1.0)
    set_state_dict(restored, restored_optimizer, model_state_dict=model_state, optim_state_dict=optim_state)
    assert torch.equal(have, want)

    # after the load both copies train on identically
    one_step(model, optimizer, seed=8)
    one_step(restored, restored_optimizer, seed=8)
    assert torch.equal(have, want)
    with pytest.raises(NotImplementedError, match="submodule"):
        get_state_dict(model, optimizer, submodules={model[0]})


def test_patched_state_dict_methods():
    torch.manual_seed(0)
    model = matrix_fully_shard(small_model())
    optimizer = configure_optimizer(model, "adamw", lr=0.01)
    one_step(model, optimizer)
    patch_model_state_dict(model)
    patch_optimizer_state_dict(model, optimizer)
    model_state, optim_state = model.state_dict(), optimizer.state_dict()
    assert model_state["metadata"]["state_dict_type"] == "matrix_sharded" and "param_groups" in optim_state

    torch.manual_seed(1234)
    restored = matrix_fully_shard(small_model())
    restored_optimizer = configure_optimizer(restored, "adamw", lr=0.2)
    patch_model_state_dict(restored)
    patch_optimizer_state_dict(restored, restored_optimizer)
    incompatible = restored.load_state_dict(model_state)
    restored_optimizer.load_state_dict(optim_state)
    assert incompatible.missing_keys == [] and incompatible.unexpected_keys == []
    assert torch.equal(restored._matrix_fsdp_param_group.flat_buffer.local_shard, model._matrix_fsdp_param_group.flat_buffer.local_shard)
    assert restored_optimizer.state_dict()["param_groups"] == optimizer.state_dict()["param_groups"]


def test_state_dict_load_checks_layout_metadata():
    torch.manual_seed(0)
    model = matrix_fully_shard(linear())
    fb = model._matrix_fsdp_param_group.flat_buffer
    state = matrix_state_dict(model)

    without_legacy_key = copy.deepcopy(state)
    without_legacy_key.pop("units")
    fb.local_shard.add_(1.0)
    load_matrix_state_dict(model, without_legacy_key)
    assert torch.equal(fb.local_shard, state["param_groups"][0]["param_shard"])

    for mutate, match in (
        (lambda s: s["param_groups"][0].__setitem__("dp_shard_mesh_dim", 1), "dp_shard_mesh_dim"),
        (lambda s: s["param_groups"][0]["layout"].__setitem__("total_numel", 11), "layout"),
        (lambda s: s["param_groups"][0].__setitem__("world_size", 2), "world_size"),
        (lambda s: s["param_groups"][0].__setitem__("rank", 1), "rank"),
        (lambda s: s["param_groups"][0]["params"]["weight"].__setitem__("shape", (4, 2)), "shape"),
        (lambda s: s["metadata"].__setitem__("version", 2), "version"),
        (lambda s: s["param_groups"].append(s["param_groups"][0]), "2 param groups"),
    ):
        broken = copy.deepcopy(state)
        mutate(broken)
        with pytest.raises(ValueError, match=match):
            load_matrix_state_dict(model, broken)
    broken = copy.deepcopy(state)
    broken["param_groups"][0]["param_shard"] = torch.zeros(3, device=DEV)
    with pytest.raises(ValueError, match="3 elements"):
        load_matrix_state_dict(model, broken)


def test_full_state_dict_holds_the_full_parameters():
    torch.manual_seed(0)
    model = small_model()
    eager = copy.deepcopy(model)
    matrix_fully_shard(model)
    state = matrix_state_dict(model, full_state=True)
    assert state["metadata"]["state_dict_type"] == "matrix_full"
    assert set(state["params"]) == set(eager.state_dict())
    for name, want in eager.state_dict().items():
        assert torch.equal(state["params"][name], want)
    assert "param_shard" in state["units"][0]
    model._matrix_fsdp_param_group.flat_buffer.local_shard.zero_()
    assert state["params"]["0.weight"].abs().sum() > 0  # copies, not views of the live shard

    # one unit per Linear, and a simulated world of 2 with per-parameter chunks (which needs the unpack)
    torch.manual_seed(0)
    model = small_model()
    eager = copy.deepcopy(model)
    for layer in (model[0], model[2]):
        matrix_fully_shard(layer, world_size=2, rank=1, planner=fsdp2_chunk_plan)
    state = matrix_state_dict(model, full_state=True)
    assert [u["module_fqn"] for u in state["units"]] == ["0", "2"]
    assert set(state["params"]) == set(eager.state_dict())
    for name, want in eager.state_dict().items():
        assert torch.equal(state["params"][name], want)


def test_state_dict_can_carry_the_local_grad_shard():
    torch.manual_seed(0)
    model = matrix_fully_shard(linear())
    fb = model._matrix_fsdp_param_group.flat_buffer
    model(torch.randn(3, 4, device=DEV)).sum().backward()
    assert fb.local_grad_shard is not None
    state = matrix_state_dict(model, include_grads=True)
    saved = state["units"][0]
    assert saved["grad_shard_state"]["name"] == "grad" and saved["grad_shard_state"]["local_numel"] == fb.local_numel
    assert saved["grad_shard_state"]["matrix_shard"] == {"type": "MatrixShard", "dims": (0,), "local_units": (1,)}
    want = fb.local_grad_shard.clone()
    fb.clear_local_grad_shard()
    for param in model.parameters():
        param.grad = None
    load_matrix_state_dict(model, state)
    assert torch.equal(fb.local_grad_shard, want)
    assert model.weight.grad.data_ptr() == fb.local_grad_shard.data_ptr()
    full = matrix_state_dict(model, include_grads=True, full_state=True)
    assert torch.equal(full["grads"]["weight"], want[:8].view(2, 4)) and torch.equal(full["grads"]["bias"], want[8:])


# ------------------------------------------------------------------------------------------------ DCP, same layout


def test_dcp_round_trip_and_metadata_files(tmp_path):
    torch.manual_seed(0)
    model = small_model()
    eager = copy.deepcopy(model)
    matrix_fully_shard(model)
    unit = model._matrix_fsdp_param_group
    fb = unit.flat_buffer
    save_matrix_dcp(model, tmp_path, no_dist=True)

    payload = global_metadata(tmp_path)
    assert payload["metadata"]["format"] == "matrix_dcp_global_metadata" and payload["metadata"]["ranks"] == (0,)
    assert set(payload["ranks"]) == {0} and not list(tmp_path.glob("matrix_metadata_rank_*.pt"))
    saved = payload["ranks"][0]
    assert saved["metadata"]["state_dict_type"] == "matrix_dcp_sharded" and saved["metadata"]["dcp_rank"] == 0
    assert saved["param_groups"][0]["param_shard_key"] == "rank_0.unit_0.param_shard"
    assert saved["param_groups"][0]["grad_shard_key"] is None and "param_shard" not in saved["param_groups"][0]

    fb.local_shard.add_(10.0)
    load_matrix_dcp(model, tmp_path, no_dist=True)
    assert unit.lifecycle_state == FSDPLifecycleState.SHARDED
    unit.unshard()
    for want, have in zip(eager.parameters(), model.parameters()):
        assert torch.equal(want, have)
    unit.reshard()

    # the per-rank sidecar of older checkpoints
    (tmp_path / "matrix_metadata.pt").unlink()
    torch.save(saved, tmp_path / "matrix_metadata_rank_0.pt")
    want = fb.local_shard.clone()
    fb.local_shard.add_(10.0)
    load_matrix_dcp(model, tmp_path, no_dist=True)
    assert torch.equal(fb.local_shard, want)

    with pytest.raises(NotImplementedError, match="one process"):
        save_matrix_dcp(model, tmp_path, no_dist=False)


def test_dcp_load_rejects_a_layout_mismatch_before_touching_tensors(tmp_path):
    torch.manual_seed(0)
    model = matrix_fully_shard(linear())
    fb = model._matrix_fsdp_param_group.flat_buffer
    save_matrix_dcp(model, tmp_path)
    saved = global_metadata(tmp_path)["ranks"][0]
    saved["units"][0]["local_end"] += 1
    rewrite_rank_metadata(tmp_path, saved)
    fb.local_shard.fill_(3.0)
    with pytest.raises(ValueError, match="local_end"):
        load_matrix_dcp(model, tmp_path)
    assert torch.all(fb.local_shard == 3.0)


def test_dcp_grad_shard_and_full_state(tmp_path):
    torch.manual_seed(0)
    model = small_model()
    eager = copy.deepcopy(model)
    matrix_fully_shard(model)
    fb = model._matrix_fsdp_param_group.flat_buffer
    model(torch.randn(3, 4, device=DEV)).sum().backward()
    want_grad = fb.local_grad_shard.clone()
    save_matrix_dcp(model, tmp_path / "a", include_grads=True, full_state=True)
    fb.clear_local_grad_shard()
    load_matrix_dcp(model, tmp_path / "a")
    assert torch.equal(fb.local_grad_shard, want_grad)
    full = load_matrix_dcp_full_state(tmp_path / "a")
    assert set(full["params"]) == set(eager.state_dict()) == set(full["grads"])
    for name, want in eager.state_dict().items():
        assert torch.equal(full["params"][name], want.cpu())
    assert torch.equal(full["grads"]["0.weight"], want_grad[:32].view(8, 4).cpu())
    save_matrix_dcp(model, tmp_path / "b")
    with pytest.raises(ValueError, match="full_state"):
        load_matrix_dcp_full_state(tmp_path / "b")


def test_dcp_optimizer_state_round_trip_and_its_metadata(tmp_path):
    torch.manual_seed(0)
    model = matrix_fully_shard(linear())
    optimizer = MatrixFSDPOptimizer(FusedAdamW(model.parameters(), lr=0.01), model)
    one_step(model, optimizer)
    want = copy.deepcopy(optimizer.state_dict())
    save_matrix_dcp(model, tmp_path, optimizer=optimizer)

    saved = global_metadata(tmp_path)["ranks"][0]["optimizer"]
    assert saved["kind"] == "FusedAdamW" and saved["optimizer_format_version"] == 2 and set(saved["components"]) == {"optimizer"}
    assert saved["state"] == saved["components"]["optimizer"]["state"] and saved["param_groups"] == saved["components"]["optimizer"]["param_groups"]
    assert saved["state"][0]["fqn"] == "weight"
    assert saved["state"][0]["entries"]["exp_avg"]["key"] == "rank_0.unit_0.optimizer.optimizer.weight.exp_avg"
    entries = [entry for state in saved["state"].values() for entry in state["entries"].values() if entry["kind"] == "tensor"]
    shard_shaped = [e for e in entries if tuple(e["shape"]) != ()]
    assert len(shard_shaped) == 4 and len(entries) == 6
    for entry in shard_shaped:
        numel = int(torch.Size(entry["shape"]).numel())
        assert entry["matrix_state"]["matrix_shard"] == {"type": "MatrixShard", "dims": (0,), "local_units": (1,)}
        assert entry["matrix_state"]["local_numel"] == numel and entry["matrix_state"]["global_shape"] == (numel,)
    assert all("matrix_state" not in e for e in entries if tuple(e["shape"]) == ())

    torch.manual_seed(1234)
    restored = matrix_fully_shard(linear())
    restored_optimizer = MatrixFSDPOptimizer(FusedAdamW(restored.parameters(), lr=0.2), restored)
    load_matrix_dcp(restored, tmp_path, optimizer=restored_optimizer)
    assert_optimizer_state_equal(restored_optimizer.state_dict(), want)
    assert restored_optimizer.state_objects["weight"]["exp_avg"].local_tensor.numel() == 8
    one_step(model, optimizer, seed=9)
    one_step(restored, restored_optimizer, seed=9)
    assert torch.equal(restored._matrix_fsdp_param_group.flat_buffer.local_shard, model._matrix_fsdp_param_group.flat_buffer.local_shard)

    # a plain optimizer gets the same placement metadata
    save_matrix_dcp(model, tmp_path / "plain", optimizer=optimizer.optimizer)
    plain = global_metadata(tmp_path / "plain")["ranks"][0]["optimizer"]
    assert all("matrix_state" in e for s in plain["state"].values() for e in s["entries"].values() if e["kind"] == "tensor" and tuple(e["shape"]) != ())

    # component bookkeeping
    saved_rank = global_metadata(tmp_path)["ranks"][0]
    saved_rank["optimizer"]["components"] = {}
    rewrite_rank_metadata(tmp_path, saved_rank)
    with pytest.raises(ValueError, match="missing component"):
        load_matrix_dcp(restored, tmp_path, optimizer=restored_optimizer)
    saved_rank = global_metadata(tmp_path / "plain")["ranks"][0]
    saved_rank["optimizer"]["components"]["extra"] = copy.deepcopy(saved_rank["optimizer"]["components"]["optimizer"])
    rewrite_rank_metadata(tmp_path / "plain", saved_rank)
    with pytest.raises(ValueError, match="unknown component"):
        load_matrix_dcp(restored, tmp_path / "plain", optimizer=restored_optimizer)
    save_matrix_dcp(model, tmp_path / "none")
    with pytest.raises(ValueError, match="does not contain optimizer state"):
        load_matrix_dcp(restored, tmp_path / "none", optimizer=restored_optimizer)


def mixed_model() -> nn.Module:
    return nn.Sequential(nn.Linear(4, 8), nn.LayerNorm(8), nn.Linear(8, 2, bias=False)).to(DEV)


def test_dcp_mixed_muon_adamw_round_trip(tmp_path):
    torch.manual_seed(0)
    model = fully_shard(mixed_model(), optimizer_policy="mixed_muon_adamw")
    optimizer = MatrixFSDPOptimizer.from_shard_hints(model)
    one_step(model, optimizer)
    want = copy.deepcopy(optimizer.state_dict())
    torch.manual_seed(1234)
    restored = fully_shard(mixed_model(), optimizer_policy="mixed_muon_adamw")
    restored_optimizer = MatrixFSDPOptimizer.from_shard_hints(restored)
    save_matrix_dcp(model, tmp_path, optimizer=optimizer)
    load_matrix_dcp(restored, tmp_path, optimizer=restored_optimizer)

    saved = global_metadata(tmp_path)["ranks"][0]["optimizer"]
    assert saved["kind"] == "mixed_muon_adamw" and saved["group_summary"]["optimizer"] == "mixed_muon_adamw"
    assert set(saved["components"]) == {"muon", "adamw"} and "state" not in saved
    assert [state["fqn"] for state in saved["components"]["muon"]["state"].values()] == ["0.weight", "2.weight"]
    hint = global_metadata(tmp_path)["ranks"][0]["param_groups"][0]["params"]["0.weight"]["shard_hint"]
    assert hint["optimizer_type"] == "muon"
    have = restored_optimizer.state_dict()
    assert have["group_summaries"] == want["group_summaries"]
    for component in ("muon", "adamw"):
        assert_optimizer_state_equal(have[component], want[component])
    restored_optimizer.validate_local_state_shapes()
    one_step(model, optimizer, seed=9)
    one_step(restored, restored_optimizer, seed=9)
    assert torch.equal(restored._matrix_fsdp_param_group.flat_buffer.local_shard, model._matrix_fsdp_param_group.flat_buffer.local_shard)


# ------------------------------------------------------------------------------------------------ optimizer state manager


def test_state_manager_describes_shard_shaped_state():
    torch.manual_seed(0)
    model = matrix_fully_shard(nn.Sequential(nn.Linear(4, 8), nn.LayerNorm(8), nn.Linear(8, 2)).to(DEV))
    unit = model._matrix_fsdp_param_group
    optimizer = MatrixFSDPOptimizer(FusedAdamW(model.parameters(), lr=0.01), model, flat_adamw_state=True)
    one_step(model, optimizer)
    assert isinstance(optimizer.state_manager, MatrixFSDPOptimizerStateManager)
    entries = optimizer.state_manager.iter_local_state_tensors()
    assert {e.name for e in entries} == {"exp_avg", "exp_avg_sq"} and len(entries) == 12
    for entry in entries:
        assert tuple(entry.sharded_state.global_shape) == (entry.tensor.numel(),)
        assert not entry.sharded_state.uses_dtensor and entry.sharded_state.shares_storage_with(entry.tensor)
        assert entry.sharded_state.local_tensor.data_ptr() == entry.tensor.data_ptr()
    assert set(optimizer.local_state_objects()["0.weight"]) == {"exp_avg", "exp_avg_sq"}

    # flat state: both moments of every parameter are views of two buffers of the local shard's length
    (flat,) = optimizer.optimizer._matrix_fsdp_flat_adamw_state_buffers.values()
    assert flat.exp_avg.numel() == flat.exp_avg_sq.numel() == unit.flat_buffer.local_numel
    states = [s for p, s in optimizer.optimizer.state.items() if p.numel()]
    assert {s["exp_avg"].untyped_storage().data_ptr() for s in states} == {flat.exp_avg.untyped_storage().data_ptr()}
    assert {s["exp_avg_sq"].untyped_storage().data_ptr() for s in states} == {flat.exp_avg_sq.untyped_storage().data_ptr()}

    described = optimizer.state_manager.local_state_metadata()["0.weight"]["exp_avg"]
    assert described["name"] == "exp_avg" and described["global_shape"] == (32,) and described["global_stride"] == (1,)
    assert described["local_shape"] == (32,) and described["local_numel"] == 32 and described["dtype"] == "torch.float32"
    assert described["matrix_shard"] == {"type": "MatrixShard", "dims": (0,), "local_units": (1,)}
    assert described["device_mesh"] is None and described["dtensor_spec"] is None and not described["uses_dtensor"]

    summary = optimizer.state_manager.summarize()
    assert summary.param_numel == unit.flat_buffer.local_numel
    assert summary.tensor_state_numel_by_name == {"exp_avg": unit.flat_buffer.local_numel, "exp_avg_sq": unit.flat_buffer.local_numel}
    assert summary.scalar_state_tensor_numel == 6 and summary.as_dict() == optimizer.local_state_summary()
    assert optimizer.state_objects and optimizer.state_dtensors == {} and optimizer.refresh_state_dtensors() == {}

    # amsgrad: the running maximum is flat too, and the optimizer follows torch.optim.AdamW(amsgrad=True, maximize=True)
    torch.manual_seed(0)
    model = small_model()
    twin = copy.deepcopy(model)
    matrix_fully_shard(model)
    optimizer = MatrixFSDPOptimizer(FusedAdamW(model.parameters(), lr=0.01, amsgrad=True, maximize=True), model, flat_adamw_state=True)
    reference = torch.optim.AdamW(twin.parameters(), lr=0.01, amsgrad=True, maximize=True, foreach=False)
    for seed in (7, 8, 9):
        one_step(model, optimizer, seed=seed)
        x = torch.randn(3, 4, generator=torch.Generator().manual_seed(seed)).to(DEV)
        reference.zero_grad()
        twin(x).sum().backward()
        reference.step()
    (flat,) = optimizer.optimizer._matrix_fsdp_flat_adamw_state_buffers.values()
    assert flat.max_exp_avg_sq is not None and flat.max_exp_avg_sq.numel() == 58
    states = [s for p, s in optimizer.optimizer.state.items() if p.numel()]
    assert {s["max_exp_avg_sq"].untyped_storage().data_ptr() for s in states} == {flat.max_exp_avg_sq.untyped_storage().data_ptr()}
    for have, want in zip(model.parameters(), twin.parameters()):
        assert torch.allclose(have.detach(), want.detach(), rtol=0, atol=2e-6 * float(want.detach().abs().max()))
        assert torch.allclose(optimizer.state[have]["max_exp_avg_sq"], reference.state[want]["max_exp_avg_sq"], rtol=1e-5, atol=1e-10)

    # opt-in only
    torch.manual_seed(0)
    model = matrix_fully_shard(linear())
    optimizer = MatrixFSDPOptimizer(FusedAdamW(model.parameters(), lr=0.01), model)
    one_step(model, optimizer)
    assert not hasattr(optimizer.optimizer, "_matrix_fsdp_flat_adamw_state_buffers")
    param, state = next(iter(optimizer.optimizer.state.items()))
    state["mismatched"] = torch.zeros(param.numel() + 1, device=DEV)
    state["scalar_ok"] = torch.tensor(1.0)
    objects = next(iter(optimizer.local_state_objects().values()))
    assert "mismatched" not in objects and "scalar_ok" not in objects
    with pytest.raises(RuntimeError, match="mismatched"):
        optimizer.validate_local_state_shapes()


# ------------------------------------------------------------------------------------------------ other layouts


class Wide(nn.Module):
    """Every parameter divides by 4; the flat buffer (13 684 elements) does not split evenly into 3."""

    def __init__(self) -> None:
        super().__init__()
        self.up = nn.Linear(64, 128)
        self.norm = nn.LayerNorm(128)
        self.down = nn.Linear(128, 32, bias=False)
        self.scale = nn.Parameter(torch.ones(4, 253))

    def forward(self, x):
        return self.down(self.norm(torch.relu(self.up(x)))) * self.scale[:, :32].sum(0)


def wide_world(world_size: int, planner, seed: int = 0, lr: float = 0.01):
    """The same model as every rank of a simulated world holds it, each with an AdamW and one step taken."""
    ranks = []
    for rank in range(world_size):
        torch.manual_seed(seed)
        model = matrix_fully_shard(Wide().to(DEV), world_size=world_size, rank=rank, planner=planner)
        optimizer = configure_optimizer(model, "adamw", lr=lr)
        ranks.append((model, optimizer))
    return ranks


def wide_step(model, optimizer, seed: int = 3) -> None:
    x = torch.randn(16, 64, generator=torch.Generator().manual_seed(seed)).to(DEV)
    optimizer.zero_grad()
    model(x).square().sum().backward()
    optimizer.step()


def even(managed_params, world_size):
    return contiguous_even_plan(managed_params[-1].end, world_size)


@pytest.mark.parametrize(
    "source_world, source_planner, target_world, target_planner",
    [
        (4, fsdp2_chunk_plan, 2, even),  # several segments per source rank: the packed order is not the flat order
        (2, even, 4, fsdp2_chunk_plan),
        (3, even, 1, even),  # uneven source shards
        (1, even, 3, even),
        (4, fsdp2_chunk_plan, 4, even),  # same world, same sizes, other elements
    ],
)
def test_dcp_load_into_another_layout(tmp_path, source_world, source_planner, target_world, target_planner):
    # what one rank alone holds after the same step: full parameters, gradient and moments
    ((whole, whole_optimizer),) = wide_world(1, even)
    wide_step(whole, whole_optimizer)
    whole_fb = whole._matrix_fsdp_param_group.flat_buffer
    full_param, full_grad = whole_fb.local_shard.clone(), whole_fb.local_grad_shard.clone()
    full_state = {name: torch.cat([whole_optimizer.state[p][name].reshape(-1) for p in whole.parameters()]) for name in ("exp_avg", "exp_avg_sq")}

    source = wide_world(source_world, source_planner)
    for model, optimizer in source:
        wide_step(model, optimizer)
    save_matrix_dcp_simulated_world([m for m, _ in source], tmp_path, optimizers=[o for _, o in source], include_grads=True)
    payload = global_metadata(tmp_path)
    assert payload["metadata"]["ranks"] == tuple(range(source_world))
    assert payload["ranks"][source_world - 1]["param_groups"][0]["param_shard_key"] == f"rank_{source_world - 1}.unit_0.param_shard"

    for rank, (model, optimizer) in enumerate(wide_world(target_world, target_planner, seed=99, lr=0.5)):
        unit = model._matrix_fsdp_param_group
        fb = unit.flat_buffer
        if (source_world, source_planner) != (target_world, target_planner) and source_world == target_world and rank == 0:
            with pytest.raises(ValueError):  # without allow_reshard the mismatch is an error
                load_matrix_dcp(model, tmp_path, optimizer=optimizer)
        load_matrix_dcp(model, tmp_path, optimizer=optimizer, allow_reshard=True)
        assert unit.lifecycle_state == FSDPLifecycleState.SHARDED
        assert torch.equal(fb.local_shard, CO.target_local_shard_from_full(full_param, fb.local_segments))
        assert torch.equal(fb.local_grad_shard, CO.target_local_shard_from_full(full_grad, fb.local_segments))
        assert torch.equal(fb.gather_full_params(), full_param)  # every simulated rank's shard was refilled
        assert optimizer.param_groups[0]["lr"] == 0.01
        seen = 0
        for view in fb.local_param_views:
            mp = view.managed_param
            state = optimizer.state[mp.param]
            assert int(state["step"].item()) == 1
            for name in ("exp_avg", "exp_avg_sq"):
                want = CO.target_local_param_tensor_from_full(full_state[name][mp.offset : mp.end], unit.rank_segments_for_param(mp.fqn, rank), mp.offset)
                assert state[name].shape == mp.param.shape and torch.equal(state[name].reshape(-1), want), (rank, mp.fqn, name)
            seen += 1
        assert seen == len([p for p in model.parameters() if p.numel()])
        # and training goes on as the one-rank run does
        wide_step(model, optimizer, seed=4)
        if rank == 0:
            wide_step(whole, whole_optimizer, seed=4)
        assert torch.equal(fb.local_shard, CO.target_local_shard_from_full(whole_fb.local_shard, fb.local_segments))


def test_dcp_owner_layout_with_mixed_optimizer_into_another_world(tmp_path):
    """Whole parameters on owner ranks, Muon on the matrices: momentum buffers follow their matrices."""

    def owners(assignment):
        return lambda managed_params, world_size: whole_param_owner_plan(managed_params, world_size, assignment)

    def hint(param):
        return ParamShardHint(optimizer_type="muon" if param.ndim == 2 and param.shape[0] > 4 else "adamw")

    def world(world_size, assignment, seed=0):
        ranks = []
        for rank in range(world_size):
            torch.manual_seed(seed)
            model = fully_shard(Wide().to(DEV), world_size=world_size, rank=rank, planner=owners(assignment), shard_placement_fn=hint)
            optimizer = None
            if any(p.numel() for p in model.parameters()):
                optimizer = configure_optimizer(model, "mixed_muon_adamw", lr=0.01, muon_momentum=0.9)
            ranks.append((model, optimizer))
        return ranks

    # parameters in order: scale, up.weight, up.bias, norm.weight, norm.bias, down.weight
    ((whole, whole_optimizer),) = world(1, [0] * 6)
    wide_step(whole, whole_optimizer)
    names = [n for n, _ in whole.named_parameters()]
    whole_state = {n: whole_optimizer.state[p] for n, p in whole.named_parameters()}
    whole_params = {n: p.detach().clone() for n, p in whole.named_parameters()}

    source = world(4, [0, 2, 0, 0, 1, 1])  # rank 0 runs AdamW only, rank 2 Muon only, rank 1 both, rank 3 owns nothing
    for model, optimizer in source:
        if optimizer is not None:
            wide_step(model, optimizer)
    assert source[3][1] is None and source[3][0]._matrix_fsdp_param_group.flat_buffer.local_numel == 0
    save_matrix_dcp_simulated_world([m for m, _ in source], tmp_path, optimizers=[o for _, o in source])
    assert names == ["scale", "up.weight", "up.bias", "norm.weight", "norm.bias", "down.weight"]
    saved = global_metadata(tmp_path)["ranks"]
    assert [set(saved[r]["optimizer"]["components"]) for r in range(3)] == [{"adamw"}, {"muon", "adamw"}, {"muon"}]
    assert "optimizer" not in saved[3] and saved[3]["param_groups"][0]["shard_sizes"][3] == 0

    for rank, (model, optimizer) in enumerate(world(2, [1, 1, 1, 0, 0, 0], seed=5)):
        load_matrix_dcp(model, tmp_path, optimizer=optimizer, allow_reshard=True)
        local = {n: p for n, p in model.named_parameters() if p.numel()}
        assert set(local) == {n for n, owner in zip(names, [1, 1, 1, 0, 0, 0]) if owner == rank}
        for name, param in local.items():
            assert torch.equal(param, whole_params[name])
            have, want = optimizer.state[param], whole_state[name]
            assert set(have) == set(want), name
            for key, value in want.items():
                if torch.is_tensor(value):
                    assert torch.equal(have[key].cpu(), value.cpu()), (name, key)
                else:
                    assert have[key] == value


# ------------------------------------------------------------------------------------------------ full-size buffers


def test_rank_shard_of_a_full_layer_buffer():
    """The program a load into another layout ends with, at the size of one hidden4096 layer buffer (202 M bf16
    elements), for the row split (a few segments per rank) and the 2x2 block split (~85 k segments): taking each
    rank's shard of the full buffer one by one gives what packing all ranks at once gives, and unpacking that gives
    the buffer back."""
    from matrix_fsdp_amd.core.plans import block_grid_plan
    from matrix_fsdp_amd.kernels.segment_program import pack_program, take_local_segments_program, unpack_program
    from matrix_fsdp_amd.workloads import HIDDEN4096_W4_BLOCK

    specs = HIDDEN4096_W4_BLOCK.specs
    total = specs[-1].end
    gen = torch.Generator(device=DEV).manual_seed(11)
    full = torch.empty(total, dtype=torch.int16, device=DEV).random_(-(2**15), 2**15, generator=gen)
    for plan in (fsdp2_chunk_plan(specs, 4), block_grid_plan(specs, (2, 2))):
        packed = torch.empty(sum(plan.shard_sizes), dtype=torch.int16, device=DEV)
        pack_program(plan, torch.int16, padded=False, device=DEV).run((full,), packed)
        for rank in range(4):
            local = torch.full((plan.shard_sizes[rank],), 7, dtype=torch.int16, device=DEV)
            take_local_segments_program(plan.local_segments(rank), total, plan.shard_sizes[rank], torch.int16, device=DEV).run((full,), local)
            start = plan.rank_packed_offset(rank)
            assert torch.equal(local, packed[start : start + plan.shard_sizes[rank]])
            # spot checks against plain slicing: first, last and a middle segment of the rank
            segments = plan.local_segments(rank)
            for seg in (segments[0], segments[len(segments) // 2], segments[-1]):
                assert torch.equal(local[seg.local_start : seg.local_end], full[seg.global_start : seg.global_end])
            del local
        back = torch.empty_like(full)
        unpack_program(plan, torch.int16, padded=False, device=DEV).run((packed,), back)
        assert torch.equal(back, full)
        del packed, back
