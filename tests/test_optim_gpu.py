"""Parity of the HIP Muon / AdamW kernels (through the C ABI) with the CPU oracle.

Tolerances: the Muon update must be within rel-Frobenius 1e-2 of the reference arithmetic on the
same seeded inputs (bf16 products, fp32 accumulation; only the summation order differs); AdamW is
fp32 element-wise and must agree to 1e-6 relative."""
import pytest
import torch

from matrix_fsdp_amd.optim import functional as F
from oracle import optim_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MUON_TOL = 1e-2


def rel_fro(have: torch.Tensor, want: torch.Tensor) -> float:
    have, want = have.detach().double().cpu(), want.detach().double().cpu()
    return float(torch.linalg.norm(have - want) / torch.linalg.norm(want))


def max_err_over_scale(have: torch.Tensor, want: torch.Tensor) -> float:
    """Largest element error relative to the tensor's largest magnitude (fp32 element-wise kernels
    differ from the CPU only by fused multiply-adds: a few 1e-7 of the operand scale)."""
    want = want.detach().double().cpu()
    return float((have.detach().double().cpu() - want).abs().max() / want.abs().max().clamp(min=1e-300))


def make(shape, seed, std=1e-3):
    gen = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=gen) * std


@pytest.mark.parametrize("shape", [(256, 256), (256, 512), (512, 256), (64, 96), (100, 36), (300, 520), (1, 7), (1024, 1024)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_newton_schulz_parity(shape, dtype):
    u = make(shape, 11).to(dtype)
    for steps in (0, 1, 5):
        want = O.newton_schulz(u, steps=steps)
        have = F.newton_schulz(u.to(DEV), ns_steps=steps)
        assert have.dtype == torch.bfloat16 and have.shape == want.shape
        assert rel_fro(have, want) < MUON_TOL, (shape, dtype, steps)


def test_newton_schulz_diagonal_closed_form():
    sigma = torch.tensor([0.9, 0.5, 0.25, 0.1, 0.01, 0.0])
    x = torch.diag(sigma)
    have = F.newton_schulz(x.to(DEV)).float().cpu()
    want = O.newton_schulz(x).float()
    assert torch.count_nonzero(have - torch.diag(torch.diag(have))) == 0
    assert torch.allclose(torch.diag(have), torch.diag(want), atol=0.02)


def test_newton_schulz_singular_values_land_near_one():
    u = make((384, 640), 12)
    sv = torch.linalg.svdvals(F.newton_schulz(u.to(DEV)).float().cpu())
    assert sv.max() < 1.3 and sv.min() > 0.3


@pytest.mark.parametrize("coefficients", [(1.5, -0.5, 0.0), (2.0, -1.5, 0.5), (0.0, 1.0, 1.0)])
def test_newton_schulz_other_polynomials(coefficients):
    """torch.optim.Muon takes any three coefficients; with c = 0 (the cubic iteration) addmm leaves b * A, with a = 0
    the update product has no X term."""
    for shape in ((256, 256), (300, 520), (512, 256)):
        u = make(shape, 17)
        want = O.newton_schulz(u, coefficients=coefficients, steps=3)
        have = F.newton_schulz(u.to(DEV), ns_coefficients=coefficients, ns_steps=3)
        assert rel_fro(have, want) < MUON_TOL, (shape, coefficients)
    p, g, buf = make((256, 384), 18, 0.02), make((256, 384), 19).bfloat16().float(), make((256, 384), 20)
    p_dev, buf_dev = p.to(DEV), buf.to(DEV)
    kw = dict(lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True)
    F.muon_step(p_dev, g.to(DEV), buf_dev, ns_coefficients=coefficients, ns_steps=3, **kw)
    p_ref, buf_ref = p.clone(), buf.clone()
    O.muon_step(p_ref, g, buf_ref, coefficients=coefficients, steps=3, **kw)
    assert rel_fro(p_dev.cpu() - p, p_ref - p) < MUON_TOL


@pytest.mark.parametrize("shape", [(192, 320), (320, 192), (100, 36), (37, 101)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("steps", [0, 1])
def test_muon_step_with_no_or_one_newton_schulz_step(shape, dtype, steps):
    """Without a Newton-Schulz step there is no product whose epilogue could carry the parameter update (the separate
    update kernel runs on the normalised update); with one step the only update product is also the last one.  Wide,
    tall and unaligned shapes (tall parameters are updated from the transposed tile)."""
    p = make(shape, 31, 0.02).to(dtype)
    g, buf = make(shape, 32).to(dtype), make(shape, 33).to(dtype)
    kw = dict(lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True)
    p_dev, buf_dev = p.to(DEV), buf.to(DEV)
    F.muon_step(p_dev, g.to(DEV), buf_dev, ns_steps=steps, **kw)
    p_ref, buf_ref = p.clone(), buf.clone()
    O.muon_step(p_ref, g, buf_ref, steps=steps, **kw)
    tol = MUON_TOL if dtype == torch.float32 else 0.05  # a bf16 parameter moves in steps of its own last bit
    assert rel_fro(p_dev.cpu().float() - p.float(), p_ref.float() - p.float()) < tol
    if dtype == torch.float32:
        assert torch.allclose(buf_dev.cpu(), buf_ref, rtol=1e-6, atol=1e-9)
    else:
        assert (buf_dev.cpu().view(torch.int16).int() - buf_ref.view(torch.int16).int()).abs().max() <= 1


def test_non_finite_coefficients_are_refused_before_anything_runs():
    p, g, buf = make((64, 64), 21, 0.02).to(DEV), make((64, 64), 22).to(DEV), make((64, 64), 23).to(DEV)
    before = (p.clone(), buf.clone())
    for bad in ((float("nan"), -4.775, 2.0315), (3.4445, float("inf"), 2.0315), (3.4445, -4.775, 1e-45)):
        with pytest.raises(RuntimeError, match="coefficients must be finite"):
            F.muon_step(p, g, buf, lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True, ns_coefficients=bad)
        with pytest.raises(RuntimeError, match="coefficients must be finite"):
            F.newton_schulz(g, ns_coefficients=bad)
    torch.cuda.synchronize()
    assert torch.equal(p, before[0]) and torch.equal(buf, before[1])  # the momentum buffer was not touched


def test_zero_update_stays_zero():
    have = F.newton_schulz(torch.zeros(64, 128, device=DEV))
    assert torch.count_nonzero(have) == 0


@pytest.mark.parametrize("shape", [(256, 512), (512, 256), (192, 192)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nesterov,adjust", [(True, None), (True, "match_rms_adamw"), (False, "original")])
def test_muon_step_parity(shape, dtype, nesterov, adjust):
    p0 = make(shape, 1, 0.02).to(dtype)
    kw = dict(lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=nesterov, adjust_lr_fn=adjust)
    p_cpu, buf_cpu = p0.clone(), make(shape, 2).to(dtype)
    p_dev, buf_dev = p_cpu.to(DEV), buf_cpu.to(DEV)
    ws = F.MuonWorkspace(DEV)
    for step in range(2):
        g = make(shape, 20 + step).to(dtype)
        before = p_cpu.clone()
        O.muon_step(p_cpu, g.clone(), buf_cpu, **kw)
        before_dev = p_dev.clone()
        F.muon_step(p_dev, g.to(DEV), buf_dev, workspace=ws, **kw)
        # the parameter delta, which the orthogonalised update dominates
        # bf16 parameters move by whole bf16 steps (2^-8 relative), so their delta and value carry that grain
        delta_err = rel_fro(p_dev.float().cpu() - before_dev.float().cpu(), p_cpu.float() - before.float())
        buf_ok = bool(torch.allclose(buf_dev.cpu(), buf_cpu, rtol=1e-6, atol=1e-9)) if dtype == torch.float32 else rel_fro(buf_dev.float(), buf_cpu.float()) < 4e-3
        value_err = rel_fro(p_dev.float(), p_cpu.float())
        assert delta_err < (MUON_TOL if dtype == torch.float32 else 0.05), delta_err
        assert buf_ok
        assert value_err < MUON_TOL, value_err
        p_cpu, buf_cpu = p_dev.cpu().clone(), buf_dev.cpu().clone()  # re-sync so that steps are compared one at a time


def test_muon_step_matches_torch_optim_muon_on_device_inputs():
    """Same check against the optimizer class the reference instantiates (CPU execution)."""
    shape = (512, 768)
    p0, g, buf0 = make(shape, 1, 0.02), make(shape, 3).bfloat16().float(), make(shape, 4)
    p_ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.Muon([p_ref], lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True)
    opt.state[p_ref]["momentum_buffer"] = buf0.clone()
    p_ref.grad = g.clone()
    opt.step()
    p, buf = p0.to(DEV), buf0.to(DEV)
    F.muon_step(p, g.to(DEV), buf, lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True)
    assert rel_fro(p.cpu() - p0, p_ref.detach() - p0) < MUON_TOL
    assert torch.allclose(buf.cpu(), opt.state[p_ref]["momentum_buffer"], rtol=1e-6, atol=1e-9)


def test_muon_step_many_matches_one_matrix_at_a_time():
    """Independent matrices spread over side streams: the same bits as one call per matrix on the calling stream (for
    matrices this small the flag does not change the tiling), work enqueued afterwards sees the updates, and an
    optimizer over several parameter groups goes the same way."""
    shapes = [(512, 768), (768, 512), (256, 256), (320, 200), (1024, 512)]
    hypers = [dict(lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True), dict(lr=0.01, weight_decay=0.0, momentum=0.9, nesterov=False, adjust_lr_fn="match_rms_adamw")]
    params = [make(sh, 100 + i, 0.02) for i, sh in enumerate(shapes)]
    grads = [make(sh, 200 + i).bfloat16().float() for i, sh in enumerate(shapes)]
    bufs = [make(sh, 300 + i) for i, sh in enumerate(shapes)]
    one_p, one_b = [p.to(DEV) for p in params], [b.to(DEV) for b in bufs]
    ws = F.MuonWorkspace(DEV)
    for i in range(len(shapes)):
        F.muon_step(one_p[i], grads[i].to(DEV), one_b[i], workspace=ws, **hypers[i % 2])
    many_p, many_b = [p.to(DEV) for p in params], [b.to(DEV) for b in bufs]
    dev_grads = [g.to(DEV) for g in grads]
    F.muon_step_many([(many_p[i], dev_grads[i], many_b[i], hypers[i % 2]) for i in range(len(shapes))])
    total = sum(p.sum() for p in many_p)  # enqueued on the calling stream right behind the batch
    for i in range(len(shapes)):
        assert torch.equal(many_p[i], one_p[i]) and torch.equal(many_b[i], one_b[i])
        p_ref, b_ref = params[i].clone(), bufs[i].clone()
        O.muon_step(p_ref, grads[i], b_ref, **hypers[i % 2])
        assert rel_fro(many_p[i].cpu() - params[i], p_ref - params[i]) < MUON_TOL
    assert float(total) == float(sum(p.sum() for p in one_p))
    F.muon_step_many([])
    F.muon_step_many([(many_p[0], dev_grads[0], many_b[0], hypers[0])])  # a single matrix stays on the calling stream
    F.muon_step(one_p[0], dev_grads[0], one_b[0], workspace=ws, **hypers[0])
    assert torch.equal(many_p[0], one_p[0])


def test_muon_step_many_side_by_side_switch(monkeypatch):
    """Matrices large enough that the side-by-side form changes the tiling of their symmetric products (m = 3072: the
    triangle of 256 x 256 tiles occupies 78 of the CUs): with ``side_by_side=False`` (argument or environment) every
    matrix gets the bits of a call of its own, whatever else the batch holds; the side-by-side form stays within the
    parity bar of the same result."""
    shapes = [(3072, 3072), (3072, 3328), (3072, 3072)]
    kw = dict(lr=0.02, weight_decay=0.1, momentum=0.95, nesterov=True)
    params = [make(sh, 400 + i, 0.02).to(DEV) for i, sh in enumerate(shapes)]
    grads = [make(sh, 500 + i).bfloat16().float().to(DEV) for i, sh in enumerate(shapes)]
    ws = F.MuonWorkspace(DEV)
    alone_p, alone_b = [p.clone() for p in params], [torch.zeros_like(p) for p in params]
    for i in range(len(shapes)):
        F.muon_step(alone_p[i], grads[i], alone_b[i], workspace=ws, **kw)

    def batch(**how):
        ps, bs = [p.clone() for p in params], [torch.zeros_like(p) for p in params]
        F.muon_step_many([(ps[i], grads[i], bs[i], kw) for i in range(len(shapes))], **how)
        torch.cuda.synchronize()
        return ps, bs

    ps, bs = batch(side_by_side=False)
    assert all(torch.equal(a, b) for a, b in zip(ps, alone_p)) and all(torch.equal(a, b) for a, b in zip(bs, alone_b))
    monkeypatch.setenv("MATRIX_FSDP_MUON_SIDE_BY_SIDE", "0")
    ps, bs = batch()
    assert all(torch.equal(a, b) for a, b in zip(ps, alone_p))
    monkeypatch.delenv("MATRIX_FSDP_MUON_SIDE_BY_SIDE")
    for how in (dict(), dict(side_by_side=True)):
        ps, bs = batch(**how)
        for i in range(len(shapes)):
            assert rel_fro((ps[i] - params[i]).cpu(), (alone_p[i] - params[i]).cpu()) < MUON_TOL
            assert torch.equal(bs[i], alone_b[i])  # the momentum does not depend on the tiling


def test_muon_argument_errors():
    p = torch.zeros(8, 8, device=DEV)
    with pytest.raises(ValueError, match="2D"):
        F.muon_step(p.view(-1), p.view(-1), p.view(-1), lr=0.1, weight_decay=0.0, momentum=0.9, nesterov=True)
    with pytest.raises(RuntimeError, match="dtype"):
        F.muon_step(p, p.bfloat16(), p, lr=0.1, weight_decay=0.0, momentum=0.9, nesterov=True)
    with pytest.raises(ValueError, match="less than 100"):
        F.newton_schulz(p, ns_steps=100)
    with pytest.raises(ValueError, match="2D"):
        F.newton_schulz(p.view(-1))
    with pytest.raises(RuntimeError, match="Learning rate"):
        F.muon_step(p, p.clone(), p.clone(), lr=-1.0, weight_decay=0.0, momentum=0.9, nesterov=True)


@pytest.mark.parametrize("n", [1, 3, 1000, 4099, 1 << 20])
@pytest.mark.parametrize("grad_dtype", [torch.float32, torch.bfloat16])
def test_adamw_parity(n, grad_dtype):
    p_cpu, m_cpu, v_cpu = make((n,), 5, 0.02), torch.zeros(n), torch.zeros(n)
    p, m, v = p_cpu.to(DEV), m_cpu.to(DEV), v_cpu.to(DEV)
    kw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    for t in (1, 2, 3):
        g = make((n,), 30 + t).to(grad_dtype)
        O.adamw_step(p_cpu, g.float(), m_cpu, v_cpu, t, **kw)
        F.adamw_step(p, g.to(DEV), m, v, t, **kw)
        assert max_err_over_scale(p, p_cpu) < 1e-6
        assert max_err_over_scale(m, m_cpu) < 1e-6
        assert max_err_over_scale(v, v_cpu) < 1e-6


@pytest.mark.parametrize("amsgrad,maximize", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("n", [1000, 4099])
def test_adamw_amsgrad_and_maximize_parity(n, amsgrad, maximize):
    p_cpu, m_cpu, v_cpu = make((n,), 5, 0.02), torch.zeros(n), torch.zeros(n)
    x_cpu = torch.zeros(n) if amsgrad else None
    p, m, v = p_cpu.to(DEV), m_cpu.to(DEV), v_cpu.to(DEV)
    x = torch.zeros(n, device=DEV) if amsgrad else None
    kw = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1, maximize=maximize)
    for t, scale in enumerate((1.0, 0.05, 0.2, 0.01), start=1):  # shrinking grads: the running maximum matters
        g = make((n,), 30 + t) * scale
        O.adamw_step(p_cpu, g, m_cpu, v_cpu, t, max_exp_avg_sq=x_cpu, **kw)
        F.adamw_step(p, g.to(DEV), m, v, t, max_exp_avg_sq=x, **kw)
        assert max_err_over_scale(p, p_cpu) < 1e-6
        assert max_err_over_scale(m, m_cpu) < 1e-6
        assert max_err_over_scale(v, v_cpu) < 1e-6
        if amsgrad:
            assert max_err_over_scale(x, x_cpu) < 1e-6
    if amsgrad:
        assert not torch.equal(x, v)


def test_optimizer_scalars_are_formed_in_double():
    """``1 - beta2`` for beta2 = 0.999 is 1.3e-5 off when it is formed from an fp32 beta2, and ``1 - momentum``
    for 0.95 is 2.4e-7 off: the entry points take doubles and round once, as the tensor operations of torch do, so
    the moments agree with the oracle to an fp32 rounding or two element by element."""
    n = 5000
    p_cpu, m_cpu, v_cpu = make((n,), 5, 0.02), torch.zeros(n), torch.zeros(n)
    p, m, v = p_cpu.to(DEV), m_cpu.to(DEV), v_cpu.to(DEV)
    kw = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    for t in (1, 2, 3):
        g = make((n,), 50 + t)
        O.adamw_step(p_cpu, g, m_cpu, v_cpu, t, **kw)
        F.adamw_step(p, g.to(DEV), m, v, t, **kw)
        # the same operations in the same order as torch's single-tensor path, each rounded once; torch's CPU
        # kernels fuse some multiply-adds depending on the host's vector ISA, so the last bit may differ
        assert float(((v.cpu() - v_cpu).abs() / v_cpu.abs().clamp_min(1e-30)).max()) < 4e-7
        assert float((m.cpu() - m_cpu).abs().max()) <= 1.2e-7 * float(m_cpu.abs().max())
        assert float((p.cpu() - p_cpu).abs().max()) <= 1.2e-7 * float(p_cpu.abs().max())
    # Muon's momentum buffer (fp32 lerp with weight 1 - 0.95)
    shape = (64, 128)
    grad, buf = make(shape, 60), make(shape, 61)
    param = make(shape, 62, 0.02)
    buf_cpu = buf.clone()
    O.muon_step(param.clone(), grad, buf_cpu, lr=0.02, weight_decay=0.0, momentum=0.95, nesterov=True)
    buf_dev = buf.to(DEV)
    F.muon_step(param.to(DEV), grad.to(DEV), buf_dev, lr=0.02, weight_decay=0.0, momentum=0.95, nesterov=True)
    assert float((buf_dev.cpu() - buf_cpu).abs().max()) <= 1.2e-7 * float(buf_cpu.abs().max())


def test_adamw_unaligned_views_and_errors():
    n = 1001
    base = [torch.zeros(n + 1, device=DEV) for _ in range(3)]
    p, m, v = (b[1:] for b in base)
    p.copy_(make((n,), 6, 0.02))
    g = make((n,), 7).to(DEV)
    p_cpu, m_cpu, v_cpu = p.cpu().clone(), torch.zeros(n), torch.zeros(n)
    O.adamw_step(p_cpu, g.cpu(), m_cpu, v_cpu, 1, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    F.adamw_step(p, g, m, v, 1, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    assert max_err_over_scale(p, p_cpu) < 1e-6
    assert all(float(b[0]) == 0.0 for b in base)
    with pytest.raises(RuntimeError, match="step"):
        F.adamw_step(p, g, m, v, 0, lr=1e-3)
    with pytest.raises(RuntimeError, match="float32"):
        F.adamw_step(p.bfloat16(), g, m, v, 1, lr=1e-3)
