"""GPU parity of the fused step with stochastic rounding, through the C ABI, against
oracle/q4_oracle_torch.py step_quant_sr (pinned in tests/test_oracle_pins.py): the noise is a
function of (seed, step, tensor salt, element), so codes and scales must agree bit for bit."""
import numpy as np
import pytest
import torch

from oracle import q4_oracle_torch as ot
from quantfour_adamw_cuda_amd import _lib
from quantfour_adamw_cuda_amd import quantfour_hip as q
from tests.q4_testlib import HP, DeviceTensor, grads_config1, grads_config3, grads_student_t, p_close, to_np

pytestmark = pytest.mark.gpu

DT = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}
HPA = (HP["beta1"], HP["beta2"], HP["lr"], HP["weight_decay"], HP["eps"])
SEED = 0x1234_5678_9ABC_DEF0


def _check(dev, ref, prev, what):
    for name, d, r in (("m codes", dev.m, ref[1]), ("v codes", dev.v, ref[2])):
        d = d.cpu()
        bad = torch.nonzero(d != r).reshape(-1)
        assert bad.numel() == 0, f"{what}: {name} differ at bytes {bad[:5].tolist()}: {d[bad[:5]].tolist()} vs {r[bad[:5]].tolist()} ({bad.numel()} bytes)"
    for name, d, r in (("m scales", dev.sm, ref[3]), ("v scales", dev.sv, ref[4])):
        assert torch.equal(d.cpu().view(torch.int32), r.view(torch.int32)), f"{what}: {name} differ"
    ok, worst = p_close(to_np(dev.p), to_np(ref[0]), to_np(prev), bf16=dev.p.dtype == torch.bfloat16)
    assert ok, f"{what}: parameters out of tolerance (worst {worst})"


def test_salt_function_matches_oracle():
    L = _lib.load()
    for seed, step, salt in ((0, 1, 0), (SEED, 7, 3), (2 ** 64 - 1, 123456, 2 ** 32 - 1), (1 << 32, 2, 5)):
        assert L.q4adamw_sr_tensor_salt(seed, float(step), salt) == ot.sr_tensor_salt(seed, step, salt)


@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16"), ("fp32", "fp32"), ("bf16", "fp32"),
                                       ("fp16", "fp16"), ("fp32", "fp16")])
@pytest.mark.parametrize("n", [128 * 300 + 77, 4097, 1 << 18])
def test_sr_against_oracle(cuda, p_dt, g_dt, n):
    gen = torch.Generator().manual_seed(n % 1000)
    p0 = (torch.randn(n, generator=gen) * 0.05).to(DT[p_dt])
    dev = DeviceTensor(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.sv.cpu())
    makers = (grads_config1, grads_config3, grads_student_t, grads_config1)
    for step in range(1, 5):
        g = makers[step - 1](gen, n).to(DT[g_dt])
        prev = ref[0]
        ref = ot.step_quant_sr(ref[0], g, *ref[1:], seed=SEED, tensor_salt=11, step=step, **HP)
        q.fused_4bit_multi_sr([dev.p], [g.to(cuda)], [dev.m], [dev.v], [dev.sm], [dev.sv], *HPA, step,
                              SEED, salts=[11])
        _check(dev, ref, prev, f"{p_dt}/{g_dt} n={n} step {step}")
        ref = (dev.p.cpu().clone(),) + tuple(ref[1:])


def test_sr_against_oracle_at_scale(cuda):
    """16.8M elements, three steps: about a thousand elements per step fall into the fast
    path's guard bands (2^-16 of the elements per moment), so both the bands' width and the
    exact path behind them are exercised; every code must still agree."""
    n = (1 << 24) + 12345
    gen = torch.Generator().manual_seed(77)
    p0 = torch.randn(n, generator=gen) * 0.05
    dev = DeviceTensor(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.sv.cpu())
    for step, maker in enumerate((grads_config1, grads_student_t, grads_config3), start=1):
        g = maker(gen, n).to(torch.bfloat16)
        prev = ref[0]
        ref = ot.step_quant_sr(ref[0], g, *ref[1:], seed=SEED + step, tensor_salt=3, step=step, **HP)
        q.fused_4bit_multi_sr([dev.p], [g.to(cuda)], [dev.m], [dev.v], [dev.sm], [dev.sv], *HPA, step,
                              SEED + step, salts=[3])
        _check(dev, ref, prev, f"n={n} step {step}")
        ref = (dev.p.cpu().clone(),) + tuple(ref[1:])


def test_sr_multi_tensor_salts_reproducibility_and_options(cuda):
    gen = torch.Generator().manual_seed(5)
    sizes = [5000 + 131 * i for i in range(60)]          # more than one launch batch
    ps = [torch.randn(n, generator=gen) * 0.05 for n in sizes]
    gs = [grads_config1(gen, n).to(torch.bfloat16) for n in sizes]

    def run(seed, salts, **kw):
        devs = [DeviceTensor(p, cuda) for p in ps]
        q.fused_4bit_multi_sr([d.p for d in devs], [g.to(cuda) for g in gs], [d.m for d in devs],
                              [d.v for d in devs], [d.sm for d in devs], [d.sv for d in devs], *HPA, 1, seed,
                              salts=salts, **kw)
        return devs

    a = run(SEED, None)
    for i in (0, 1, 47, 48, 59):                          # default salt = position in the list
        z8 = torch.zeros((sizes[i] + 1) // 2, dtype=torch.uint8)
        zs = torch.zeros((sizes[i] + 127) // 128)
        ref = ot.step_quant_sr(ps[i], gs[i], z8, z8.clone(), zs, zs.clone(), seed=SEED, tensor_salt=i, step=1, **HP)
        _check(a[i], ref, ps[i], f"tensor {i}")
    b = run(SEED, list(range(60)))
    assert all(torch.equal(x.m, y.m) and torch.equal(x.v, y.v) for x, y in zip(a, b)), "a call must be reproducible"
    c = run(SEED + 1, None)
    assert all(not torch.equal(x.m, y.m) for x, y in zip(a, c)), "another seed must draw other noise"
    d = run(SEED, [7] * 60)
    assert not torch.equal(a[3].m, d[3].m)
    # gradient multiplier: same as pre-multiplied fp32 gradients
    e = run(SEED, None, grad_scale_dev=torch.tensor([0.5], device=cuda))
    z8 = torch.zeros((sizes[2] + 1) // 2, dtype=torch.uint8)
    zs = torch.zeros((sizes[2] + 127) // 128)
    ref = ot.step_quant_sr(ps[2], gs[2].float() * 0.5, z8, z8.clone(), zs, zs.clone(), seed=SEED, tensor_salt=2,
                           step=1, **HP)
    _check(e[2], ref, ps[2], "with multiplier")


def test_sr_is_unbiased_at_scale(cuda):
    """one step from zero state on 2^24 elements: inside the code book's range (values beyond its
    ends clamp under either rounding) the dequantized moments average to the exact moments,
    which nearest rounding does not achieve"""
    n = 1 << 24
    gen = torch.Generator(device=cuda).manual_seed(6)
    g = torch.randn(n, generator=gen, device=cuda) * 1e-3
    p = torch.zeros(n, device=cuda)
    m_exact = (1 - np.float32(HP["beta1"])) * g
    v_exact = (1 - np.float32(HP["beta2"])) * (g * g)
    out = {}
    for name in ("sr", "nearest"):
        d = DeviceTensor(p, cuda)
        if name == "sr":
            q.fused_4bit_multi_sr([d.p], [g], [d.m], [d.v], [d.sm], [d.sv], *HPA, 1, SEED)
        else:
            q.fused_4bit_multi([d.p], [g], [d.m], [d.v], [d.sm], [d.sv], *HPA, 1)
        m = q.dequantize_state(d.m, d.sm, n, 0)
        v = q.dequantize_state(d.v, d.sv, n, 1)
        sm = d.sm.repeat_interleave(128)[:n]
        sv = d.sv.repeat_interleave(128)[:n]
        in_m = (m_exact / sm >= -0.8875)
        in_v = (v_exact / sv >= 0.0625)
        # signed error relative to the block scale, averaged over the in-range elements: bias
        out[name] = (float((((m - m_exact) / sm)[in_m]).double().mean()),
                     float((((v - v_exact) / sv)[in_v]).double().mean()))
    assert abs(out["sr"][0]) < 1e-4 and abs(out["sr"][1]) < 1e-4, out
    assert abs(out["nearest"][0]) > 5 * abs(out["sr"][0]) or abs(out["nearest"][1]) > 5 * abs(out["sr"][1]), out


def test_optimizer_stochastic_rounding(cuda):
    """round_type="stochastic": the class passes the group's seed and the parameters' positions;
    same seed -> same run, bit for bit; a resumed run continues the sequence; the result tracks
    torch.optim.AdamW within the draft's own bar (tests/driver.py:70-71)"""
    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour

    def mlp(seed):
        torch.manual_seed(seed)
        return torch.nn.Sequential(torch.nn.Linear(256, 200), torch.nn.Tanh(), torch.nn.Linear(200, 64)).to(cuda)

    def run(opt_fn, steps, model=None, opt=None, data_seed=0):
        model = model or mlp(1)
        opt = opt or opt_fn(model.parameters())
        gen = torch.Generator(device=cuda).manual_seed(data_seed)
        for _ in range(steps):
            x = torch.randn(32, 256, generator=gen, device=cuda)
            opt.zero_grad(set_to_none=True)
            model(x).square().mean().backward()
            opt.step()
        return model, opt

    sr = lambda ps: AdamWFused_QuantFour(ps, lr=1e-3, weight_decay=0.01, round_type="stochastic", seed=99)
    m1, o1 = run(sr, 8)
    m2, _ = run(sr, 8)
    assert all(torch.equal(a, b) for a, b in zip(m1.parameters(), m2.parameters()))
    m3, _ = run(lambda ps: AdamWFused_QuantFour(ps, lr=1e-3, weight_decay=0.01, round_type="stochastic", seed=100), 8)
    assert any(not torch.equal(a, b) for a, b in zip(m1.parameters(), m3.parameters()))
    # the first weight's codes against the oracle for the last step is covered by the functional
    # tests; here: the salt is the parameter's position (weight of layer 2 = position 2)
    ref_model, _ = run(lambda ps: torch.optim.AdamW(ps, lr=1e-3, weight_decay=0.01), 8)
    for a, b in zip(m1.parameters(), ref_model.parameters()):
        torch.testing.assert_close(a, b, atol=0.025, rtol=1e-5)
    # resume after 5 steps == 8 steps straight through
    m5, o5 = run(sr, 5)
    m_res = mlp(2)
    m_res.load_state_dict(m5.state_dict())
    o_res = AdamWFused_QuantFour(m_res.parameters())
    o_res.load_state_dict(o5.state_dict())
    gen = torch.Generator(device=cuda).manual_seed(0)
    for i in range(8):
        x = torch.randn(32, 256, generator=gen, device=cuda)
        if i < 5:
            continue
        o_res.zero_grad(set_to_none=True)
        m_res(x).square().mean().backward()
        o_res.step()
    assert all(torch.equal(a, b) for a, b in zip(m1.parameters(), m_res.parameters()))


def test_sr_non_finite_gradients(cuda):
    """inf and NaN gradients: a NaN moment gets code 0, an infinite block scale sends finite
    values to the code of zero, as the oracle has it"""
    n = 128 * 40 + 9
    gen = torch.Generator().manual_seed(18)
    p0 = torch.randn(n, generator=gen) * 0.05
    dev = DeviceTensor(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.sv.cpu())
    for step in (1, 2, 3):
        g = grads_config1(gen, n)
        if step == 2:
            g[5] = float("inf")
            g[128 + 7] = float("-inf")
            g[256 + 9] = float("nan")
            g[384:512] = float("nan")
            g[512 + 1], g[512 + 2] = float("inf"), float("nan")
        with np.errstate(invalid="ignore"):
            ref = ot.step_quant_sr(ref[0], g, *ref[1:], seed=SEED, tensor_salt=0, step=step, **HP)
        q.fused_4bit_multi_sr([dev.p], [g.to(cuda)], [dev.m], [dev.v], [dev.sm], [dev.sv], *HPA, step, SEED)
        for name, d, r in (("m codes", dev.m, ref[1]), ("v codes", dev.v, ref[2])):
            bad = torch.nonzero(d.cpu() != r).reshape(-1)
            assert bad.numel() == 0, f"step {step}: {name} differ at bytes {bad[:8].tolist()}: {d.cpu()[bad[:8]].tolist()} vs {r[bad[:8]].tolist()}"
        for name, d, r in (("m scales", dev.sm, ref[3]), ("v scales", dev.sv, ref[4])):
            assert torch.equal(d.cpu().view(torch.int32), r.view(torch.int32)), f"step {step}: {name}"
        ref = (dev.p.cpu().clone(),) + tuple(ref[1:])


@pytest.mark.parametrize("rank1", [False, True])
@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16")])
def test_variants_against_the_scalar_c_oracle(cuda, p_dt, g_dt, stochastic, rank1):
    """the HIP step's variants against q4o_step_quant_variants, the scalar C loops, directly
    (the other tests of this file and of test_gpu_rank1.py go through the vectorised torch
    restatement): codes, scales and statistics bit for bit over four steps of a 96 x 2432 matrix"""
    from oracle import q4_oracle as oc
    rows, cols = 96, 2432
    n = rows * cols
    gen = torch.Generator().manual_seed(99)
    p0 = (torch.randn(rows, cols, generator=gen) * 0.05).to(DT[p_dt])
    as_np = lambda t: (t.view(torch.int16).numpy().view(np.uint16).copy() if t.dtype == torch.bfloat16
                       else t.numpy().copy())
    nbytes, nblk = oc.state_sizes(n)
    cm, cv = np.zeros(nbytes, np.uint8), np.zeros(nbytes, np.uint8)
    csm, csv = np.zeros(nblk, np.float32), np.zeros(nblk, np.float32)
    cr, cc = np.zeros(rows, np.float32), np.zeros(cols, np.float32)
    p = p0.clone().to(cuda)
    m = torch.zeros(nbytes, dtype=torch.uint8, device=cuda)
    v = torch.zeros_like(m)
    sm, sv = torch.zeros(nblk, device=cuda), torch.zeros(nblk, device=cuda)
    r, c, rn, cn = (torch.zeros(k, device=cuda) for k in (rows, cols, rows, cols))
    kw = dict(seed=SEED, tensor_salt=4) if stochastic else {}
    for step in range(1, 5):
        g = (grads_config1 if step % 2 else grads_config3)(gen, n).view(rows, cols).to(DT[g_dt])
        cp = as_np(p.cpu())                     # the oracle starts every step from the device's parameters
        prev = cp.copy()
        if rank1:
            oc.step_quant_variants(cp, as_np(g), cm, cv, csm, None, cr, cc, step=step, **kw, **HP)
            q.fused_4bit_rank1_multi([p], [g.to(cuda)], [m], [v], [sm], [r], [c], [rn], [cn], *HPA, step,
                                     **(dict(seed=SEED, salts=[4]) if stochastic else {}))
        else:
            oc.step_quant_variants(cp.reshape(-1), as_np(g).reshape(-1), cm, cv, csm, csv, step=step, **kw, **HP)
            if stochastic:
                q.fused_4bit_multi_sr([p.view(-1)], [g.to(cuda).view(-1)], [m], [v], [sm], [sv], *HPA, step, SEED, salts=[4])
            else:
                q.fused_4bit(p.view(-1), g.to(cuda).view(-1), m, v, sm, sv, *HPA, step)
        torch.cuda.synchronize()
        what = f"{p_dt}/{g_dt} sr={stochastic} rank1={rank1} step {step}"
        assert np.array_equal(m.cpu().numpy(), cm) and np.array_equal(v.cpu().numpy(), cv), f"{what}: codes"
        assert np.array_equal(sm.cpu().numpy().view(np.uint32), csm.view(np.uint32)), f"{what}: first-moment scales"
        if rank1:
            assert np.array_equal(r.cpu().numpy().view(np.uint32), cr.view(np.uint32)), f"{what}: row maxima"
            assert np.array_equal(c.cpu().numpy().view(np.uint32), cc.view(np.uint32)), f"{what}: column maxima"
        else:
            assert np.array_equal(sv.cpu().numpy().view(np.uint32), csv.view(np.uint32)), f"{what}: second-moment scales"
        ok, worst = p_close(to_np(p), cp.reshape(-1), prev.reshape(-1), bf16=p_dt == "bf16")
        assert ok, f"{what}: parameters out of tolerance (worst {worst})"
