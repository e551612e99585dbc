"""Seeded sweep over sizes, dtypes, hyper-parameters, step numbers and gradient magnitudes:
the HIP step against the C oracle (block-scaled path) on configurations no hand-written test
names.  Deterministic: every case derives from its index.  Q4ADAMW_SWEEP_EXTRA=N in the
environment adds the indices 1000 .. 1000+N-1 to every sweep (a longer hunt, same rules)."""
import os

import numpy as np
import pytest
import torch

import quantfour_adamw_cuda_amd as q4
from tests.q4_testlib import DeviceTensor, OracleTensor, assert_state_equal

pytestmark = pytest.mark.gpu

EXTRA = list(range(1000, 1000 + int(os.environ.get("Q4ADAMW_SWEEP_EXTRA", "0"))))

DTYPES = [(torch.float32, torch.float32), (torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16),
          (torch.bfloat16, torch.float32), (torch.float16, torch.float16), (torch.float32, torch.float16)]


def _as_grad(g, g_dt):
    """numpy fp32 -> torch gradient of type g_dt; fp16 gradients are kept finite (the
    non-finite cases have tests of their own)"""
    if g_dt == torch.float16:
        g = np.clip(g, -6.0e4, 6.0e4)
    return torch.from_numpy(g).to(g_dt)


def _case(i):
    rng = np.random.default_rng(1000 + i)
    n = int(rng.choice([rng.integers(1, 300), rng.integers(300, 5000), rng.integers(5000, 400000)]))
    p_dt, g_dt = DTYPES[i % len(DTYPES)]
    hp = dict(beta1=float(rng.choice([0.5, 0.8, 0.9, 0.95, 0.99])),
              beta2=float(rng.choice([0.88, 0.95, 0.99, 0.999, 0.9999])),
              lr=float(10.0 ** rng.uniform(-6, -1)), weight_decay=float(rng.choice([0.0, 1e-4, 0.01, 0.1, 0.5])),
              eps=float(rng.choice([1e-12, 1e-8, 1e-6, 1e-3])))
    first_step = int(rng.choice([1, 2, 10, 1000, 100000]))
    g_scale = float(10.0 ** rng.uniform(-9, 3))
    return rng, n, p_dt, g_dt, hp, first_step, g_scale


@pytest.mark.parametrize("i", list(range(48)) + EXTRA)
def test_random_configuration(cuda, i):
    rng, n, p_dt, g_dt, hp, first_step, g_scale = _case(i)
    print(f"[sweep {i}] n={n} p={p_dt} g={g_dt} hp={hp} step0={first_step} g_scale={g_scale:.3g}", flush=True)
    p0 = torch.from_numpy((rng.standard_normal(n) * 10.0 ** rng.uniform(-4, 1)).astype(np.float32)).to(p_dt)
    dev, ref = DeviceTensor(p0, cuda), OracleTensor(p0)
    for k in range(3):
        g = rng.standard_normal(n).astype(np.float32) * np.float32(g_scale)
        u = rng.uniform(size=n)
        g[u < 0.1] = 0.0
        g[u > 0.999] *= np.float32(1e3)
        if k == 1:
            g[: n // 2] = 0.0                      # long runs of zero blocks
        g = _as_grad(g, g_dt)
        step = first_step + k
        q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, hp["beta1"], hp["beta2"], hp["lr"],
                      hp["weight_decay"], hp["eps"], step)
        prev = ref.step(g, step, hp)
        assert_state_equal(dev, ref, prev, f"sweep {i} step {step}")
        ref.resync(dev.p)


@pytest.mark.parametrize("i", list(range(16)) + EXTRA)
def test_random_configuration_stochastic_rounding(cuda, i):
    from oracle import q4_oracle_torch as ot
    from quantfour_adamw_cuda_amd import quantfour_hip as q
    from tests.q4_testlib import p_close, to_np
    rng, n, p_dt, g_dt, hp, first_step, g_scale = _case(100 + i)
    seed, salt = int(rng.integers(0, 2 ** 63)), int(rng.integers(0, 2 ** 32))
    print(f"[sweep sr {i}] n={n} p={p_dt} g={g_dt} hp={hp} step0={first_step} seed={seed} salt={salt}", flush=True)
    p0 = torch.from_numpy((rng.standard_normal(n) * 0.05).astype(np.float32)).to(p_dt)
    dev = DeviceTensor(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.sv.cpu())
    for k in range(2):
        g = _as_grad(rng.standard_normal(n).astype(np.float32) * np.float32(g_scale), g_dt)
        step = first_step + k
        prev = ref[0]
        ref = ot.step_quant_sr(ref[0], g, *ref[1:], seed=seed, tensor_salt=salt, step=step, **hp)
        q.fused_4bit_multi_sr([dev.p], [g.to(cuda)], [dev.m], [dev.v], [dev.sm], [dev.sv], hp["beta1"], hp["beta2"],
                              hp["lr"], hp["weight_decay"], hp["eps"], step, seed, salts=[salt])
        assert torch.equal(dev.m.cpu(), ref[1]) and torch.equal(dev.v.cpu(), ref[2]), f"sr sweep {i} step {step}: codes"
        assert torch.equal(dev.sm.cpu().view(torch.int32), ref[3].view(torch.int32))
        assert torch.equal(dev.sv.cpu().view(torch.int32), ref[4].view(torch.int32))
        ok, worst = p_close(to_np(dev.p), to_np(ref[0]), to_np(prev), bf16=p_dt == torch.bfloat16)
        assert ok, f"sr sweep {i} step {step}: parameters (worst {worst})"
        ref = (dev.p.cpu().clone(),) + tuple(ref[1:])


@pytest.mark.parametrize("i", list(range(24)) + EXTRA)
def test_random_configuration_rank1(cuda, i):
    """every third case adds stochastic rounding (random seed and salt), every fourth has rows
    of whole tiles, every eighth rows of whole blocks that end in a partial tile"""
    from oracle import q4_oracle_torch as ot
    from quantfour_adamw_cuda_amd import quantfour_hip as q
    from tests.q4_testlib import p_close, to_np
    rng, _, p_dt, g_dt, hp, first_step, g_scale = _case(200 + i)
    rows, cols = int(rng.integers(1, 90)), 8 * int(rng.integers(2, 300))     # narrow matrices included
    if i % 4 == 1:      # rows of whole tiles, enough of them: the update kernel that shares column maxima
        rows, cols = rows + 63, 256 * (2 + cols % 7)
    elif i % 8 == 3:    # the same kernel with a partial last tile: 17 to 63 blocks of 128 columns
        rows, cols = 64 + rows % 8, 128 * (17 + cols % 47)
    sr = dict(seed=int(rng.integers(0, 2 ** 63)), tensor_salt=int(rng.integers(0, 2 ** 32))) if i % 3 == 2 else None
    print(f"[sweep rank1 {i}] {rows}x{cols} p={p_dt} g={g_dt} hp={hp} step0={first_step} sr={sr}", flush=True)
    n = rows * cols
    p0 = torch.from_numpy((rng.standard_normal((rows, cols)) * 0.05).astype(np.float32)).to(p_dt)
    z = lambda k, dt=torch.float32: torch.zeros(k, dtype=dt, device=cuda)
    p, m, v, sm = p0.clone().to(cuda), z((n + 1) // 2, torch.uint8), z((n + 1) // 2, torch.uint8), z((n + 127) // 128)
    r, c, rn, cn = z(rows), z(cols), z(rows), z(cols)
    ref = (p0.clone(), m.cpu(), v.cpu(), sm.cpu(), r.cpu(), c.cpu())
    for k in range(2):
        g = rng.standard_normal((rows, cols)).astype(np.float32) * np.float32(g_scale)
        g *= rng.uniform(0.01, 1.0, (rows, 1)).astype(np.float32) * rng.uniform(0.01, 1.0, (1, cols)).astype(np.float32)
        g = _as_grad(g, g_dt)
        step = first_step + k
        prev = ref[0]
        if sr is None:
            ref = ot.step_quant_rank1(ref[0], g, *ref[1:], step=step, **hp)
            kw = {}
        else:
            ref = ot.step_quant_rank1_sr(ref[0], g, *ref[1:], step=step, **sr, **hp)
            kw = dict(seed=sr["seed"], salts=[sr["tensor_salt"]])
        q.fused_4bit_rank1_multi([p], [g.to(cuda)], [m], [v], [sm], [r], [c], [rn], [cn], hp["beta1"], hp["beta2"],
                                 hp["lr"], hp["weight_decay"], hp["eps"], step, **kw)
        for name, d, x in (("m", m, ref[1]), ("v", v, ref[2])):
            assert torch.equal(d.cpu(), x), f"rank1 sweep {i} step {step}: {name} codes"
        for name, d, x in (("sm", sm, ref[3]), ("r", r, ref[4]), ("c", c, ref[5])):
            assert torch.equal(d.cpu().view(torch.int32), x.view(torch.int32)), f"rank1 sweep {i} step {step}: {name}"
        ok, worst = p_close(to_np(p), to_np(ref[0]), to_np(prev), bf16=p_dt == torch.bfloat16)
        assert ok, f"rank1 sweep {i} step {step}: parameters (worst {worst})"
        ref = (p.cpu().clone(),) + tuple(ref[1:])


@pytest.mark.parametrize("p_dt,g_dt", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16)])
def test_long_run_stays_bit_exact(cuda, p_dt, g_dt):
    """120 consecutive steps of one tensor: the packed state feeds back into itself, so any
    difference from the oracle would persist and grow.  The gradient regime changes every few
    steps (decaying magnitude, sparse steps, spikes, all-zero steps, a sign flip), which walks
    the block scales up and down; codes and scales are compared bit for bit after every step."""
    rng = np.random.default_rng(4242)
    n = 128 * 1500 + 77
    p0 = torch.from_numpy((rng.standard_normal(n) * 0.05).astype(np.float32)).to(p_dt)
    dev, ref = DeviceTensor(p0, cuda), OracleTensor(p0)
    hp = dict(beta1=0.9, beta2=0.95, lr=3e-3, weight_decay=0.05, eps=1e-8)   # short memory: scales move fast
    base = rng.standard_normal(n).astype(np.float32)
    for step in range(1, 121):
        regime = (step // 6) % 5
        g = base * np.float32(0.7) + rng.standard_normal(n).astype(np.float32) * np.float32(0.3)
        g *= np.float32(1e-2 * 0.97 ** step)
        if regime == 1:
            g[rng.uniform(size=n) < 0.9] = 0.0
        elif regime == 2:
            g[rng.uniform(size=n) > 0.9995] *= np.float32(300.0)
        elif regime == 3 and step % 2:
            g[:] = 0.0
        elif regime == 4:
            g = -g
        g = _as_grad(g, g_dt)
        if step % 20 == 1:
            print(f"[long run {p_dt}/{g_dt}] step {step}", flush=True)
        q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, hp["beta1"], hp["beta2"], hp["lr"],
                      hp["weight_decay"], hp["eps"], step)
        prev = ref.step(g, step, hp)
        assert_state_equal(dev, ref, prev, f"long run step {step}")
        ref.resync(dev.p)
    assert ref.m.any() and ref.v.any() and len(np.unique(ref.sm)) > 100
