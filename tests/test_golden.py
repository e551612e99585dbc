"""Replays the committed golden fixtures (tests/golden/*.npz, written by
tests/golden/make_golden.py): on the CPU through both oracle restatements, on the GPU
through the C ABI."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import q4_oracle as oc
from oracle import q4_oracle_torch as ot
from tests.q4_testlib import p_close

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "quant_*.npz")))
SR_FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "sr_*.npz")))
RANK1_FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "rank1_*.npz")))


def load(path):
    z = np.load(path, allow_pickle=False)
    b1, b2, lr, wd, eps = z["hp"].tolist()
    hp = dict(beta1=b1, beta2=b2, lr=lr, weight_decay=wd, eps=eps)
    steps = sum(1 for k in z.files if k.startswith("sm"))
    return z, hp, steps


def test_fixtures_exist():
    assert len(FIXTURES) >= 4 and len(SR_FIXTURES) >= 2 and len(RANK1_FIXTURES) >= 2


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_oracles_replay_fixture(path):
    z, hp, steps = load(path)
    p = z["p0"].copy()
    n = p.size
    nb, nk = oc.state_sizes(n)
    m, v = np.zeros(nb, np.uint8), np.zeros(nb, np.uint8)
    sm, sv = np.zeros(nk, np.float32), np.zeros(nk, np.float32)
    bf16_p = p.dtype == np.uint16
    pbits = np.uint16 if p.dtype.itemsize == 2 else np.uint32      # bf16 bit patterns and fp16 are 2 bytes
    tp = torch.from_numpy(p.view(np.int16).copy()).view(torch.bfloat16) if bf16_p else torch.from_numpy(p.copy())
    tm, tv, tsm, tsv = (torch.from_numpy(x.copy()) for x in (m, v, sm, sv))
    for t in range(1, steps + 1):
        g = z[f"g{t}"]
        oc.step_quant(p, g, m, v, sm, sv, step=t, **hp)
        assert np.array_equal(p.view(pbits), z[f"p{t}"].view(pbits))
        assert np.array_equal(m, z[f"m{t}"]) and np.array_equal(v, z[f"v{t}"])
        assert np.array_equal(sm.view(np.uint32), z[f"sm{t}"]) and np.array_equal(sv.view(np.uint32), z[f"sv{t}"])
        tg = torch.from_numpy(g.view(np.int16).copy()).view(torch.bfloat16) if g.dtype == np.uint16 else torch.from_numpy(g.copy())
        tp, tm, tv, tsm, tsv = ot.step_quant(tp, tg, tm, tv, tsm, tsv, step=t, **hp)
        assert np.array_equal(tm.numpy(), m) and np.array_equal(tv.numpy(), v)
        assert np.array_equal(tsm.numpy().view(np.uint32), z[f"sm{t}"])
        assert np.array_equal(tsv.numpy().view(np.uint32), z[f"sv{t}"])
        got = tp.view(torch.int16).numpy().view(np.uint16) if bf16_p else tp.numpy().view(pbits)
        assert np.array_equal(got, z[f"p{t}"].view(got.dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_device_replays_fixture(path, cuda):
    import quantfour_adamw_cuda_amd as q4
    z, hp, steps = load(path)
    p0 = z["p0"]
    bf16_p = p0.dtype == np.uint16
    n = p0.size
    nb, nk = oc.state_sizes(n)
    to_t = lambda a: (torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
                      if a.dtype == np.uint16 else torch.from_numpy(a.copy()))
    p = to_t(p0).to(cuda)
    m = torch.zeros(nb, dtype=torch.uint8, device=cuda)
    v = torch.zeros(nb, dtype=torch.uint8, device=cuda)
    sm = torch.zeros(nk, device=cuda)
    sv = torch.zeros(nk, device=cuda)
    prev = p0
    for t in range(1, steps + 1):
        print(f"[golden {os.path.basename(path)}] step {t}", flush=True)
        q4.fused_4bit(p, to_t(z[f"g{t}"]).to(cuda), m, v, sm, sv, hp["beta1"], hp["beta2"], hp["lr"],
                      hp["weight_decay"], hp["eps"], t)
        torch.cuda.synchronize()
        assert np.array_equal(m.cpu().numpy(), z[f"m{t}"]) and np.array_equal(v.cpu().numpy(), z[f"v{t}"])
        assert np.array_equal(sm.cpu().numpy().view(np.uint32), z[f"sm{t}"])
        assert np.array_equal(sv.cpu().numpy().view(np.uint32), z[f"sv{t}"])
        got = p.view(torch.int16).cpu().numpy().view(np.uint16) if bf16_p else p.cpu().numpy()
        ok, worst = p_close(got, z[f"p{t}"], prev, bf16=bf16_p, exact=not bf16_p)   # fp32: bit for bit
        assert ok, worst
        # continue from the fixture's parameters so that the bound stays a per-step bound
        prev = z[f"p{t}"]
        p.copy_(to_t(prev).to(cuda))


# ---------------------------------------------------------------------------
# stochastic rounding and rank-1 fixtures (written from oracle/q4_oracle_torch.py)
# ---------------------------------------------------------------------------
def _t(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16) if a.dtype == np.uint16 else torch.from_numpy(a.copy())


def _bits(t):
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1)
    if t.dtype == torch.float32:
        return t.contiguous().cpu().numpy().view(np.uint32).reshape(-1)
    return t.cpu().numpy().reshape(-1)


@pytest.mark.parametrize("path", SR_FIXTURES, ids=[os.path.basename(p) for p in SR_FIXTURES])
def test_oracle_replays_sr_fixture(path):
    z, hp, steps = load(path)
    seed, salt = (int(x) for x in z["sr"])
    n = z["p0"].size
    nb, nk = oc.state_sizes(n)
    st = (_t(z["p0"]), torch.zeros(nb, dtype=torch.uint8), torch.zeros(nb, dtype=torch.uint8), torch.zeros(nk), torch.zeros(nk))
    for t in range(1, steps + 1):
        st = ot.step_quant_sr(st[0], _t(z[f"g{t}"]), *st[1:], seed=seed, tensor_salt=salt, step=t, **hp)
        for key, got in zip(("p", "m", "v", "sm", "sv"), st):
            assert np.array_equal(_bits(got), z[f"{key}{t}"].view(_bits(got).dtype)), (key, t)


@pytest.mark.gpu
@pytest.mark.parametrize("path", SR_FIXTURES, ids=[os.path.basename(p) for p in SR_FIXTURES])
def test_device_replays_sr_fixture(path, cuda):
    from quantfour_adamw_cuda_amd import quantfour_hip as q
    z, hp, steps = load(path)
    seed, salt = (int(x) for x in z["sr"])
    n = z["p0"].size
    nb, nk = oc.state_sizes(n)
    p = _t(z["p0"]).to(cuda)
    m, v = torch.zeros(nb, dtype=torch.uint8, device=cuda), torch.zeros(nb, dtype=torch.uint8, device=cuda)
    sm, sv = torch.zeros(nk, device=cuda), torch.zeros(nk, device=cuda)
    prev = z["p0"]
    for t in range(1, steps + 1):
        q.fused_4bit_multi_sr([p], [_t(z[f"g{t}"]).to(cuda)], [m], [v], [sm], [sv], hp["beta1"], hp["beta2"], hp["lr"],
                              hp["weight_decay"], hp["eps"], t, seed, salts=[salt])
        for key, got in (("m", m), ("v", v), ("sm", sm), ("sv", sv)):
            assert np.array_equal(_bits(got), z[f"{key}{t}"].view(_bits(got).dtype)), (key, t)
        ok, worst = p_close(_bits(p).view(z["p0"].dtype), z[f"p{t}"], prev, bf16=z["p0"].dtype == np.uint16)
        assert ok, worst
        prev = z[f"p{t}"]
        p.copy_(_t(prev).to(cuda))


@pytest.mark.parametrize("path", RANK1_FIXTURES, ids=[os.path.basename(p) for p in RANK1_FIXTURES])
def test_oracle_replays_rank1_fixture(path):
    z, hp, steps = load(path)
    rows, cols = (int(x) for x in z["shape"])
    nb, nk = oc.state_sizes(rows * cols)
    st = (_t(z["p0"]).view(rows, cols), torch.zeros(nb, dtype=torch.uint8), torch.zeros(nb, dtype=torch.uint8),
          torch.zeros(nk), torch.zeros(rows), torch.zeros(cols))
    sr = dict(seed=int(z["sr"][0]), tensor_salt=int(z["sr"][1])) if "sr" in z else None
    for t in range(1, steps + 1):
        if sr is None:
            st = ot.step_quant_rank1(st[0], _t(z[f"g{t}"]).view(rows, cols), *st[1:], step=t, **hp)
        else:
            st = ot.step_quant_rank1_sr(st[0], _t(z[f"g{t}"]).view(rows, cols), *st[1:], step=t, **sr, **hp)
        for key, got in zip(("p", "m", "v", "sm", "r", "c"), st):
            assert np.array_equal(_bits(got), z[f"{key}{t}"].view(_bits(got).dtype)), (key, t)


@pytest.mark.gpu
@pytest.mark.parametrize("path", RANK1_FIXTURES, ids=[os.path.basename(p) for p in RANK1_FIXTURES])
def test_device_replays_rank1_fixture(path, cuda):
    from quantfour_adamw_cuda_amd import quantfour_hip as q
    z, hp, steps = load(path)
    rows, cols = (int(x) for x in z["shape"])
    nb, nk = oc.state_sizes(rows * cols)
    p = _t(z["p0"]).view(rows, cols).to(cuda)
    m, v = torch.zeros(nb, dtype=torch.uint8, device=cuda), torch.zeros(nb, dtype=torch.uint8, device=cuda)
    sm = torch.zeros(nk, device=cuda)
    r, c, rn, cn = (torch.zeros(k, device=cuda) for k in (rows, cols, rows, cols))
    prev = z["p0"]
    for t in range(1, steps + 1):
        sr = dict(seed=int(z["sr"][0]), salts=[int(z["sr"][1])]) if "sr" in z else {}
        q.fused_4bit_rank1_multi([p], [_t(z[f"g{t}"]).view(rows, cols).to(cuda)], [m], [v], [sm], [r], [c], [rn], [cn],
                                 hp["beta1"], hp["beta2"], hp["lr"], hp["weight_decay"], hp["eps"], t, **sr)
        for key, got in (("m", m), ("v", v), ("sm", sm), ("r", r), ("c", c)):
            assert np.array_equal(_bits(got), z[f"{key}{t}"].view(_bits(got).dtype)), (key, t)
        ok, worst = p_close(_bits(p).view(z["p0"].dtype), z[f"p{t}"], prev, bf16=z["p0"].dtype == np.uint16)
        assert ok, worst
        prev = z[f"p{t}"]
        p.copy_(_t(prev).view(rows, cols).to(cuda))
