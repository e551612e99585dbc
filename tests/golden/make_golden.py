"""Writes the golden fixtures of the 4-bit AdamW step (tests/golden/*.npz).

The reference ships no golden vectors, known-answer tests or fixtures for this path
(its tests/assets/ directory does not exist), so these vectors come from this build's
CPU oracle (oracle/q4_oracle.c; oracle/q4_oracle_torch.py for stochastic rounding and the
rank-1 scaled second moment), after that oracle has been pinned by
tests/test_oracle_pins.py.  They freeze the arithmetic: a later change to the oracle or
to the kernel that alters a single bit of the packed states shows up against them.

    python tests/golden/make_golden.py

Each fixture holds the inputs themselves (no RNG is needed to replay it) and, for every
step, the expected parameters, packed codes and block scales as raw bit patterns.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import torch  # noqa: E402

from oracle import q4_oracle as oc  # noqa: E402
from oracle import q4_oracle_torch as ot  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_round(x):
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return u.astype(np.uint16)


def make(name, n, steps, hp, p_bf16=False, g_bf16=False, seed=0, special=None, p_f16=False, g_f16=False):
    """bf16 tensors are stored as uint16 bit patterns, fp16 tensors as numpy float16"""
    rng = np.random.default_rng(seed)
    p = (rng.standard_normal(n) * 0.02).astype(np.float32)
    grads = []
    for _ in range(steps):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        u = rng.uniform(size=n)
        g[u < 0.15] = 0.0
        g[(u >= 0.15) & (u < 0.17)] = np.float32(1e-41)          # fp32 denormal
        g[(u >= 0.17) & (u < 0.171)] = np.float32(1e3)
        if special is not None:
            special(g)
        grads.append(g)
    p_in = bf16_round(p) if p_bf16 else (p.astype(np.float16) if p_f16 else p)
    g_in = [bf16_round(g) if g_bf16 else (g.astype(np.float16) if g_f16 else g) for g in grads]
    nb, nk = oc.state_sizes(n)
    m, v = np.zeros(nb, np.uint8), np.zeros(nb, np.uint8)
    sm, sv = np.zeros(nk, np.float32), np.zeros(nk, np.float32)
    cur = p_in.copy()
    out = dict(p0=p_in, hp=np.array([hp["beta1"], hp["beta2"], hp["lr"], hp["weight_decay"], hp["eps"]],
                                    np.float64))
    for t, g in enumerate(g_in, 1):
        oc.step_quant(cur, g, m, v, sm, sv, step=t, **hp)
        out[f"g{t}"] = g
        out[f"p{t}"] = cur.copy()
        out[f"m{t}"] = m.copy()
        out[f"v{t}"] = v.copy()
        out[f"sm{t}"] = sm.view(np.uint32).copy()
        out[f"sv{t}"] = sv.view(np.uint32).copy()
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
    print(name, n, "elements,", steps, "steps")


def _grads(rng, n, steps):
    out = []
    for _ in range(steps):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        u = rng.uniform(size=n)
        g[u < 0.15] = 0.0
        g[(u >= 0.17) & (u < 0.171)] = np.float32(1e3)
        out.append(g)
    return out


def _to_torch(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16) if a.dtype == np.uint16 else torch.from_numpy(a.copy())


def _to_numpy(t):
    return t.view(torch.int16).numpy().view(np.uint16).copy() if t.dtype == torch.bfloat16 else t.numpy().copy()


def make_sr(name, n, steps, hp, seed, sr_seed, tensor_salt, g_bf16=False):
    """stochastic rounding (oracle/q4_oracle_torch.py step_quant_sr): noise seed and tensor
    salt travel in the fixture"""
    rng = np.random.default_rng(seed)
    p = (rng.standard_normal(n) * 0.02).astype(np.float32)
    gs = [bf16_round(g) if g_bf16 else g for g in _grads(rng, n, steps)]
    nb, nk = oc.state_sizes(n)
    state = (torch.from_numpy(p.copy()), torch.zeros(nb, dtype=torch.uint8), torch.zeros(nb, dtype=torch.uint8),
             torch.zeros(nk), torch.zeros(nk))
    out = dict(p0=p, hp=np.array([hp[k] for k in ("beta1", "beta2", "lr", "weight_decay", "eps")], np.float64),
               sr=np.array([sr_seed, tensor_salt], np.uint64))
    for t, g in enumerate(gs, 1):
        state = ot.step_quant_sr(state[0], _to_torch(g), *state[1:], seed=sr_seed, tensor_salt=tensor_salt,
                                 step=t, **hp)
        out[f"g{t}"] = g
        out[f"p{t}"], out[f"m{t}"], out[f"v{t}"] = _to_numpy(state[0]), state[1].numpy().copy(), state[2].numpy().copy()
        out[f"sm{t}"], out[f"sv{t}"] = state[3].numpy().view(np.uint32).copy(), state[4].numpy().view(np.uint32).copy()
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
    print(name, n, "elements,", steps, "steps")


def make_rank1(name, rows, cols, steps, hp, seed, p_bf16=False, g_bf16=False, sr=None):
    """rank-1 scaled second moment (oracle/q4_oracle_torch.py step_quant_rank1); with
    sr = (noise seed, tensor salt) both moments are rounded stochastically
    (step_quant_rank1_sr) and the pair travels in the fixture"""
    rng = np.random.default_rng(seed)
    n = rows * cols
    p = (rng.standard_normal(n) * 0.02).astype(np.float32)
    p_in = bf16_round(p) if p_bf16 else p
    gs = _grads(rng, n, steps)
    gs[1].reshape(rows, cols)[rows // 2] = 0.0
    gs[1].reshape(rows, cols)[:, 16:24] = 0.0
    gs = [bf16_round(g) if g_bf16 else g for g in gs]
    nb, nk = oc.state_sizes(n)
    state = (_to_torch(p_in).view(rows, cols), torch.zeros(nb, dtype=torch.uint8), torch.zeros(nb, dtype=torch.uint8),
             torch.zeros(nk), torch.zeros(rows), torch.zeros(cols))
    out = dict(p0=p_in, shape=np.array([rows, cols], np.int64),
               hp=np.array([hp[k] for k in ("beta1", "beta2", "lr", "weight_decay", "eps")], np.float64))
    if sr is not None:
        out["sr"] = np.array(sr, np.uint64)
    for t, g in enumerate(gs, 1):
        if sr is None:
            state = ot.step_quant_rank1(state[0], _to_torch(g).view(rows, cols), *state[1:], step=t, **hp)
        else:
            state = ot.step_quant_rank1_sr(state[0], _to_torch(g).view(rows, cols), *state[1:], seed=sr[0],
                                           tensor_salt=sr[1], step=t, **hp)
        out[f"g{t}"] = g
        out[f"p{t}"] = _to_numpy(state[0].reshape(-1))
        out[f"m{t}"], out[f"v{t}"] = state[1].numpy().copy(), state[2].numpy().copy()
        out[f"sm{t}"] = state[3].numpy().view(np.uint32).copy()
        out[f"r{t}"], out[f"c{t}"] = state[4].numpy().view(np.uint32).copy(), state[5].numpy().view(np.uint32).copy()
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
    print(name, rows, "x", cols, ",", steps, "steps")


def zero_blocks(g):
    g[128:384] = 0.0


if __name__ == "__main__":
    hp = dict(beta1=0.9, beta2=0.999, lr=1e-3, weight_decay=0.01, eps=1e-8)
    hp_driver = dict(beta1=0.8, beta2=0.88, lr=5e-3, weight_decay=0.03, eps=1e-8)   # tests/driver.py:28-31
    make("quant_fp32_fp32_n1027", 1027, 3, hp, seed=1, special=zero_blocks)
    make("quant_fp32_bf16_n4099", 4099, 3, hp, g_bf16=True, seed=2)
    make("quant_bf16_bf16_n2050", 2050, 3, hp, p_bf16=True, g_bf16=True, seed=3)
    make("quant_driver_hp_n640", 640, 4, hp_driver, seed=4)
    make("quant_fp16_fp16_n2309", 2309, 3, hp, p_f16=True, g_f16=True, seed=10)
    make("quant_fp32_fp16_n1500", 1500, 3, hp, g_f16=True, seed=11)
    make_sr("sr_fp32_bf16_n3001", 3001, 3, hp, seed=5, sr_seed=0x0123456789ABCDEF, tensor_salt=7, g_bf16=True)
    make_sr("sr_fp32_fp32_n1100", 1100, 3, hp_driver, seed=6, sr_seed=42, tensor_salt=0)
    make_rank1("rank1_fp32_bf16_5x520", 5, 520, 3, hp, seed=7, g_bf16=True)
    make_rank1("rank1_bf16_bf16_3x1024", 3, 1024, 3, hp, seed=8, p_bf16=True, g_bf16=True)
    make_rank1("rank1_sr_fp32_bf16_6x768", 6, 768, 3, hp, seed=9, g_bf16=True, sr=(0xFEDCBA9876543210, 11))
