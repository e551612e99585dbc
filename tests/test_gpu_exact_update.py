"""The exact form of the parameter update on the GPU: the reference's expression
(optim/cuda_adamw_kernels.cu:334,351: p * wdu - step_size * (m / (sqrtf(v) / c2s + eps))) with
every operation rounded as IEEE 754 rounds it, so that parameters agree with the oracles BIT
FOR BIT, step after step without re-basing either side -- for every element type, with
stochastic rounding and with rank-1 scaling when asked for, and by itself (update_form "auto")
for fp32 parameters in the block-scaled step with nearest rounding."""
import numpy as np
import pytest
import torch

import quantfour_adamw_cuda_amd as q4
from oracle import q4_oracle as oc
from oracle import q4_oracle_torch as ot
from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
from quantfour_adamw_cuda_amd import quantfour_hip as q
from tests.q4_testlib import (HP, HP_DRIVER, DeviceTensor, OracleTensor, bits, grads_config1, grads_config3,
                              grads_student_t, p_close, p_mismatches, to_np)

pytestmark = pytest.mark.gpu

DT = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}
HPA = (HP["beta1"], HP["beta2"], HP["lr"], HP["weight_decay"], HP["eps"])


def say(msg):
    print(msg, flush=True)


def same_params(dev_p, ref_p):
    """mismatch count: fp32 by bit pattern (NaN == NaN), 16-bit types by stored pattern"""
    if dev_p.dtype == torch.float32:
        return p_mismatches(to_np(dev_p), np.asarray(ref_p, np.float32))
    a = dev_p.detach().contiguous().view(torch.int16).cpu().numpy().reshape(-1)
    b = ref_p if isinstance(ref_p, np.ndarray) else ref_p.detach().contiguous().view(torch.int16).cpu().numpy()
    return int(np.count_nonzero(a.view(np.uint16) != np.asarray(b).reshape(-1).view(np.uint16)))


def test_rounding_selfcheck_of_this_gpu(cuda):
    """every fp32 pattern of the short forms' domains: square roots, refined reciprocals (the
    hardware property the short division rests on) and quotients all correctly rounded, and so
    are the general expansions that lanes outside the domains take"""
    c = q.rounding_selfcheck(cuda)
    say(f"[selfcheck] {c}")
    assert c["walked"] == (186 + 120) * (1 << 23) + 2      # [2^-96, 2^90] and [2^-60, 2^60], ends included
    assert (c["sqrt"], c["reciprocal"], c["quotient"], c["general_sqrt"], c["general_quotient"]) == (0, 0, 0, 0, 0)


@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "fp32"), ("fp32", "bf16"), ("fp32", "fp16"), ("bf16", "bf16"),
                                       ("bf16", "fp32"), ("fp16", "fp16"), ("fp16", "bf16")])
@pytest.mark.parametrize("n", [100003, 4097, 1 << 20])
def test_exact_form_bit_for_bit_every_dtype(cuda, p_dt, g_dt, n):
    """update_form "exact" against the C oracle, six steps, neither side re-based: zeros,
    denormals, +-1e3 outliers, Student-t tails; full tiles and the ragged last one"""
    gen = torch.Generator().manual_seed(n % 977 + len(p_dt) + 3 * len(g_dt))
    p0 = (torch.randn(n, generator=gen) * 0.02).to(DT[p_dt])
    dev, ref = DeviceTensor(p0, cuda), OracleTensor(p0)
    makers = (grads_config1, grads_config3, grads_student_t, grads_config3, grads_config1, grads_student_t)
    for step, maker in enumerate(makers, start=1):
        g = maker(gen, n).to(DT[g_dt])
        q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, *HPA, step, update_form="exact")
        torch.cuda.synchronize()
        ref.step(g, step)
        assert np.array_equal(dev.m.cpu().numpy(), ref.m) and np.array_equal(dev.v.cpu().numpy(), ref.v)
        bad = same_params(dev.p, ref.p)
        assert bad == 0, f"{p_dt}/{g_dt} n={n} step {step}: {bad} parameters differ"


@pytest.mark.parametrize("hp", [HP, HP_DRIVER, dict(beta1=0.5, beta2=0.9999999, lr=3.0, weight_decay=0.5, eps=1e-3),
                                dict(beta1=0.99, beta2=0.5, lr=1e-7, weight_decay=0.0, eps=1e-12)],
                         ids=["baseline", "driver", "extreme-a", "extreme-b"])
def test_config1_ten_steps_cumulative(cuda, hp):
    """BASELINE configs[0] at its hyper-parameters (and three other sets): after ten steps of
    the default call on fp32 parameters, device and oracle hold the same bits -- a cumulative
    bound of zero"""
    gen = torch.Generator().manual_seed(0)
    n = 4096 * 4096 if hp is HP else 1 << 20
    p0 = torch.randn(n, generator=gen) * 0.02
    dev, ref = DeviceTensor(p0, cuda), OracleTensor(p0)
    for step in range(1, 11):
        g = grads_config1(gen, n)
        q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, hp["beta1"], hp["beta2"], hp["lr"],
                      hp["weight_decay"], hp["eps"], step)
        ref.step(g, step, hp)
    torch.cuda.synchronize()
    assert np.array_equal(dev.m.cpu().numpy(), ref.m) and np.array_equal(dev.v.cpu().numpy(), ref.v)
    assert same_params(dev.p, ref.p) == 0


def test_auto_rule_and_the_folded_form(cuda):
    """"auto" is the exact form for fp32 parameters and the folded one for 16-bit parameters;
    the folded form is a tolerance (and really another computation: some parameters differ)"""
    n = 1 << 22
    gen = torch.Generator().manual_seed(5)
    p0 = torch.randn(n, generator=gen) * 0.02
    g = grads_student_t(gen, n).to(torch.bfloat16)
    runs = {}
    for p_dt in ("fp32", "bf16"):
        for form in ("auto", "exact", "folded"):
            dev = DeviceTensor(p0.to(DT[p_dt]), cuda)
            for step in (1, 2):
                q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, *HPA, step, update_form=form)
            runs[p_dt, form] = dev
    torch.cuda.synchronize()
    for p_dt in ("fp32", "bf16"):
        for form in ("exact", "folded"):      # codes and scales never depend on the form
            assert torch.equal(runs[p_dt, form].m, runs[p_dt, "auto"].m) and torch.equal(runs[p_dt, form].v, runs[p_dt, "auto"].v)
    assert torch.equal(runs["fp32", "auto"].p, runs["fp32", "exact"].p)
    assert torch.equal(runs["bf16", "auto"].p, runs["bf16", "folded"].p)
    differing = int((runs["fp32", "folded"].p != runs["fp32", "exact"].p).sum())
    say(f"[forms] fp32: {differing} of {n} parameters differ between the folded and the exact form after two steps")
    assert 0 < differing < n
    # the folded form's tolerance, one step from identical inputs
    dev, ref = DeviceTensor(p0, cuda), OracleTensor(p0)
    q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, *HPA, 1, update_form="folded")
    prev = ref.step(g, 1)
    ok, worst = p_close(to_np(dev.p), ref.p, prev)
    assert ok, worst
    with pytest.raises(ValueError, match="update_form"):
        q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, *HPA, 2, update_form="fast")


def test_values_outside_the_short_forms(cuda):
    """zeros of either sign in parameters, gradients and state, denormal and tiny moments, huge
    and infinite and NaN gradients, eps and betas at the edges of what the short sequences
    take: those lanes go through the general expansions and still match the oracle's bits"""
    n = 128 * 64
    inf, nan = float("inf"), float("nan")
    cases = [
        ("baseline hp", HP),
        ("eps below the short forms", dict(HP, eps=1e-30)),
        ("eps above the short forms", dict(HP, eps=1e25)),
        ("beta2 next to 1 (small c2s)", dict(HP, beta2=0.99999994)),
        ("huge lr", dict(HP, lr=1e20, weight_decay=0.0)),
    ]
    for label, hp in cases:
        gen = torch.Generator().manual_seed(len(label))
        p0 = torch.randn(n, generator=gen) * 0.02
        p0[0:8] = torch.tensor([0.0, -0.0, 0.0, -0.0, 1e-45, -1e-45, 1e-38, -1e-38])
        dev, ref = DeviceTensor(p0, cuda), OracleTensor(p0)
        for step in (1, 2, 3):
            g = grads_config3(gen, n)
            g[0:8] = torch.tensor([0.0, -0.0, -0.0, 0.0, 1e-45, 1e-30, -1e-22, 1e-19])
            g[128:256] = 0.0                          # an all-zero block
            g[256:264] = torch.tensor([1e-18, -1e-17, 3e-16, 1e-12, 1e15, -1e18, 3e19, -1e19])
            if step == 2:
                g[384], g[385], g[512], g[640:768] = inf, -inf, nan, 1e30
            hpa = (hp["beta1"], hp["beta2"], hp["lr"], hp["weight_decay"], hp["eps"])
            q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, *hpa, step)
            torch.cuda.synchronize()
            ref.step(g, step, hp)
            assert np.array_equal(dev.m.cpu().numpy(), ref.m) and np.array_equal(dev.v.cpu().numpy(), ref.v), label
            pd = to_np(dev.p)
            bad = np.flatnonzero(~((bits(pd) == bits(ref.p)) | (np.isnan(pd) & np.isnan(ref.p))))
            assert bad.size == 0, f"{label}, step {step}: {bad.size} parameters differ, first {bad[:5]}: {pd[bad[:5]]} vs {ref.p[bad[:5]]}"


@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16"), ("fp32", "fp32")])
def test_exact_form_with_stochastic_rounding(cuda, p_dt, g_dt):
    n = 128 * 300 + 77
    gen = torch.Generator().manual_seed(21)
    p0 = (torch.randn(n, generator=gen) * 0.05).to(DT[p_dt])
    dev = DeviceTensor(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.sv.cpu())
    for step, maker in enumerate((grads_config1, grads_config3, grads_student_t, grads_config1), start=1):
        g = maker(gen, n).to(DT[g_dt])
        ref = ot.step_quant_sr(ref[0], g, *ref[1:], seed=99, tensor_salt=11, step=step, **HP)
        q.fused_4bit_multi_sr([dev.p], [g.to(cuda)], [dev.m], [dev.v], [dev.sm], [dev.sv], *HPA, step, 99,
                              salts=[11], update_form="exact")
        assert torch.equal(dev.m.cpu(), ref[1]) and torch.equal(dev.v.cpu(), ref[2])
        assert same_params(dev.p, ref[0] if p_dt != "fp32" else ref[0].numpy()) == 0, f"step {step}"


@pytest.mark.parametrize("shape", [(66, 1024), (257, 768), (300, 16), (70, 2560), (66, 2432), (257, 77), (64, 2501)])
@pytest.mark.parametrize("p_dt,g_dt,sr", [("fp32", "bf16", False), ("bf16", "bf16", False), ("fp32", "fp32", True)])
def test_exact_form_with_rank1_scaling(cuda, shape, p_dt, g_dt, sr):
    """the four rank-1 update kernels (row-aligned, wide, narrow, rows of any length), with and without stochastic rounding"""
    rows, cols = shape
    gen = torch.Generator().manual_seed(rows + cols)
    p0 = (torch.randn(rows, cols, generator=gen) * 0.05).to(DT[p_dt])
    n = rows * cols
    p = p0.clone().to(cuda)
    m = torch.zeros((n + 1) // 2, dtype=torch.uint8, device=cuda)
    v, sm = torch.zeros_like(m), torch.zeros((n + 127) // 128, device=cuda)
    r, c, rn, cn = (torch.zeros(k, device=cuda) for k in (rows, cols, rows, cols))
    ref = (p0.clone(), m.cpu(), v.cpu(), sm.cpu(), r.cpu(), c.cpu())
    kw = dict(seed=5, salts=[2]) if sr else {}
    for step in range(1, 5):
        g = (grads_config1 if step & 1 else grads_config3)(gen, n).view(rows, cols).to(DT[g_dt])
        if sr:
            ref = ot.step_quant_rank1_sr(ref[0], g, *ref[1:], seed=5, tensor_salt=2, step=step, **HP)
        else:
            ref = ot.step_quant_rank1(ref[0], g, *ref[1:], step=step, **HP)
        q.fused_4bit_rank1_multi([p], [g.to(cuda)], [m], [v], [sm], [r], [c], [rn], [cn], *HPA, step,
                                 update_form="exact", **kw)
        assert torch.equal(m.cpu(), ref[1]) and torch.equal(v.cpu(), ref[2]), f"step {step}: codes"
        assert same_params(p, ref[0] if p_dt != "fp32" else ref[0].numpy()) == 0, f"{shape} {p_dt}/{g_dt} step {step}"


@pytest.mark.parametrize("dtype,form", [(torch.float32, "auto"), (torch.bfloat16, "exact"), (torch.float32, "folded")])
def test_optimizer_param_update_option(cuda, dtype, form):
    """AdamWFused_QuantFour(param_update=...): fp32 parameters bit-identical by default, bf16
    ones on request; "folded" stays within the tolerance; the option travels in the param
    groups and survives a state_dict round trip"""
    gen = torch.Generator().manual_seed(8)
    shapes = [(300, 257), (4096,), (129, 33), (64, 512)]
    ps = [(torch.randn(s, generator=gen) * 0.02).to(dtype) for s in shapes]
    params = [torch.nn.Parameter(p.clone().to(cuda)) for p in ps]
    kw = dict(lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]), eps=HP["eps"], weight_decay=HP["weight_decay"])
    opt = AdamWFused_QuantFour(params, param_update=form, **kw)
    assert opt.param_groups[0]["param_update"] == form
    refs = [OracleTensor(p) if p.numel() > 4096 else None for p in ps]
    small = [[to_np(p), np.zeros(p.numel(), np.float32), np.zeros(p.numel(), np.float32)] if p.numel() <= 4096 else None
             for p in ps]
    for step in (1, 2, 3):
        gs = [(torch.randn(s, generator=gen) * 1e-3).to(dtype) for s in shapes]
        for p, g in zip(params, gs):
            p.grad = g.to(cuda)
        opt.step()
        torch.cuda.synchronize()
        if step == 2:       # resume from a state_dict: the option comes back with the groups
            sd = opt.state_dict()
            opt = AdamWFused_QuantFour(params, **kw)
            opt.load_state_dict(sd)
            assert opt.param_groups[0]["param_update"] == form
        for p, g, r, s in zip(params, gs, refs, small):
            if r is None:
                if dtype == torch.float32:
                    oc.step_unquant(s[0], to_np(g), s[1], s[2], step=step, **HP)
                    assert p_mismatches(to_np(p.detach()), s[0]) == 0
                continue
            prev = r.step(g, step)
            if form == "folded":
                ok, worst = p_close(to_np(p.detach()), r.p, prev)
                assert ok, worst
                r.resync(p.detach())
            else:
                assert same_params(p.detach(), r.p) == 0, f"{tuple(p.shape)} step {step}"
    with pytest.raises(ValueError, match="param_update"):
        AdamWFused_QuantFour(params, param_update="nearest", **kw)
