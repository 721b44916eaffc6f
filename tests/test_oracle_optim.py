"""Pins the optimizer oracle against the installed torch (the library that holds the reference's
arithmetic) and against closed forms."""
import math

import pytest
import torch

from oracle import optim_oracle as O


def make(shape, seed, std=1e-3):
    gen = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=gen) * std


@pytest.mark.parametrize("shape", [(48, 32), (32, 48), (40, 40)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nesterov,adjust", [(True, None), (True, "match_rms_adamw"), (False, "original")])
def test_muon_step_equals_torch_muon(shape, dtype, nesterov, adjust):
    p0 = make(shape, 1, 0.02).to(dtype)
    grads = [make(shape, 10 + i).to(dtype) for i in range(3)]
    p_ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.Muon([p_ref], lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=nesterov, adjust_lr_fn=adjust)
    p = p0.clone()
    buf = torch.zeros_like(p)
    for g in grads:
        p_ref.grad = g.clone()
        opt.step()
        # torch normalises the update in place; for bf16 without Nesterov that update IS the momentum
        # buffer, so the comparison of later steps is only meaningful where torch leaves the buffer alone
        O.muon_step(p, g.clone(), buf, lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=nesterov, adjust_lr_fn=adjust)
        if dtype == torch.bfloat16 and not nesterov:
            break
        assert torch.equal(p, p_ref.detach())
        assert torch.equal(buf, opt.state[p_ref]["momentum_buffer"])
    assert torch.equal(p, p_ref.detach())


def test_newton_schulz_equals_torch_routine():
    from torch.optim._muon import _zeropower_via_newtonschulz

    for shape in [(64, 32), (32, 64), (16, 16)]:
        u = make(shape, 3)
        for steps in (0, 1, 5):
            assert torch.equal(O.newton_schulz(u, steps=steps), _zeropower_via_newtonschulz(u, O.NS_COEFFICIENTS, steps, O.NS_EPS))


def bf16_round(v: float) -> float:
    return float(torch.tensor(v, dtype=torch.float32).bfloat16())


def scalar_quintic_bf16(s: float, steps: int) -> float:
    """The quintic on one value with the matrix iteration's rounding points: A, B and X in bf16."""
    a, b, c = O.NS_COEFFICIENTS
    s = bf16_round(s)
    for _ in range(steps):
        gram = bf16_round(s * s)
        poly = bf16_round(b * gram + c * (gram * gram))
        s = bf16_round(a * s + poly * s)
    return s


def test_newton_schulz_on_diagonal_follows_the_scalar_quintic():
    """For a diagonal matrix every product is diagonal, so each entry follows s <- a s + b s^3 + c s^5
    (with bf16 rounding of A, B and X).  A dropped term or a wrong sign misses by far more than the 2 %
    allowed here; the unrounded quintic is checked to be close as well."""
    sigma = torch.tensor([0.9, 0.5, 0.25, 0.1, 0.01, 0.0])
    x = torch.diag(sigma)
    norm = float(x.bfloat16().norm())
    out = O.newton_schulz(x, steps=5).float()
    assert torch.count_nonzero(out - torch.diag(torch.diag(out))) == 0
    for s, got in zip(sigma.tolist(), torch.diag(out).tolist()):
        rounded = scalar_quintic_bf16(bf16_round(s) / norm, 5)
        assert abs(got - rounded) <= 0.02 * max(1.0, abs(rounded))
        assert abs(got - O.newton_schulz_scalar(s / norm, steps=5)) <= 0.08


def test_newton_schulz_matches_float64_polynomial_of_singular_values():
    gen = torch.Generator().manual_seed(7)
    g = torch.randn(24, 40, generator=gen, dtype=torch.float64)
    u, s, vh = torch.linalg.svd(g, full_matrices=False)
    s = s / torch.linalg.norm(g)
    want = (u * torch.tensor([O.newton_schulz_scalar(float(v)) for v in s], dtype=torch.float64)) @ vh
    got = O.newton_schulz(g.float(), steps=5).double()
    assert torch.linalg.norm(got - want) / torch.linalg.norm(want) < 2e-2
    sv = torch.linalg.svdvals(got)
    assert sv.max() < 1.3 and sv.min() > 0.3


def test_adjust_lr():
    assert O.adjust_lr(0.02, None, (12288, 4096)) == 0.02 * math.sqrt(3)
    assert O.adjust_lr(0.02, "original", (4096, 11008)) == 0.02
    assert O.adjust_lr(0.02, "match_rms_adamw", (4096, 11008)) == 0.02 * 0.2 * math.sqrt(11008)


@pytest.mark.parametrize("wd", [0.0, 0.1])
def test_adamw_step_equals_torch_adamw(wd):
    p0, grads = make((1000,), 2, 0.02), [make((1000,), 20 + i) for i in range(3)]
    p_ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([p_ref], lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=wd, foreach=False)
    p, m, v = p0.clone(), torch.zeros(1000), torch.zeros(1000)
    for t, g in enumerate(grads, start=1):
        p_ref.grad = g.clone()
        opt.step()
        O.adamw_step(p, g, m, v, t, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=wd)
        assert torch.equal(p, p_ref.detach())
        assert torch.equal(m, opt.state[p_ref]["exp_avg"]) and torch.equal(v, opt.state[p_ref]["exp_avg_sq"])


@pytest.mark.parametrize("amsgrad,maximize", [(True, False), (False, True), (True, True)])
def test_adamw_step_amsgrad_and_maximize_equal_torch_adamw(amsgrad, maximize):
    """Gradients shrink after the first step, so the running maximum of the second moment differs from the moment
    itself and a wrong (or missing) maximum changes the result."""
    p0 = make((1000,), 3, 0.02)
    grads = [make((1000,), 40 + i) * scale for i, scale in enumerate((1.0, 0.05, 0.2, 0.01))]
    p_ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([p_ref], lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1, amsgrad=amsgrad, maximize=maximize, foreach=False)
    p, m, v = p0.clone(), torch.zeros(1000), torch.zeros(1000)
    vmax = torch.zeros(1000) if amsgrad else None
    for t, g in enumerate(grads, start=1):
        p_ref.grad = g.clone()
        opt.step()
        O.adamw_step(p, g, m, v, t, lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1, max_exp_avg_sq=vmax, maximize=maximize)
        assert torch.equal(p, p_ref.detach())
        assert torch.equal(m, opt.state[p_ref]["exp_avg"]) and torch.equal(v, opt.state[p_ref]["exp_avg_sq"])
        if amsgrad:
            assert torch.equal(vmax, opt.state[p_ref]["max_exp_avg_sq"])
    if amsgrad:
        assert not torch.equal(vmax, v)
