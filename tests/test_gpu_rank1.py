"""GPU parity of the fused step with a rank-1-scaled second moment, through the C ABI,
against the torch restatement in oracle/q4_oracle_torch.py (itself pinned by brute force and
closed forms in tests/test_oracle_pins.py): codes, block scales and row / column maxima bit
for bit, parameters within the step's tolerance."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import q4_oracle_torch as ot
from quantfour_adamw_cuda_amd import _lib
from quantfour_adamw_cuda_amd import quantfour_hip as q
from tests.q4_testlib import HP, grads_config1, grads_config3, p_close, to_np

pytestmark = pytest.mark.gpu

DT = {"fp32": torch.float32, "bf16": torch.bfloat16}
HPA = (HP["beta1"], HP["beta2"], HP["lr"], HP["weight_decay"], HP["eps"])


class Rank1State:
    def __init__(self, p, device):
        rows, cols = p.shape
        n = p.numel()
        self.p = p.clone().to(device)
        self.m = torch.zeros((n + 1) // 2, dtype=torch.uint8, device=device)
        self.v = torch.zeros_like(self.m)
        self.sm = torch.zeros((n + 127) // 128, device=device)
        self.r = torch.zeros(rows, device=device)
        self.c = torch.zeros(cols, device=device)
        self.rn = torch.zeros(rows, device=device)
        self.cn = torch.zeros(cols, device=device)

    def step(self, g, step, **kw):
        q.fused_4bit_rank1_multi([self.p], [g], [self.m], [self.v], [self.sm], [self.r], [self.c],
                                 [self.rn], [self.cn], *HPA, step, **kw)

    def tensors(self):
        return (self.p, self.m, self.v, self.sm, self.r, self.c)


def _check(dev, ref, prev, what):
    """ref = (p, m_codes, v_codes, m_scale, row_max, col_max) from the oracle, on any device"""
    names = ("p", "m codes", "v codes", "m scales", "row maxima", "column maxima")
    for name, d, r in list(zip(names, dev.tensors(), ref))[1:]:
        d, r = d.cpu(), r.cpu()
        if d.dtype == torch.float32:
            same = torch.equal(d.view(torch.int32), r.view(torch.int32))
        else:
            same = torch.equal(d, r)
        if not same:
            bad = torch.nonzero(d != r).reshape(-1)[:5]
            raise AssertionError(f"{what}: {name} differ at {bad.tolist()}: {d[bad].tolist()} vs {r[bad].tolist()} "
                                 f"({int((d != r).sum())} of {d.numel()})")
    assert not dev.rn.any() and not dev.cn.any(), f"{what}: scratch must be zero after the step"
    ok, worst = p_close(to_np(dev.p), to_np(ref[0]), to_np(prev), bf16=dev.p.dtype == torch.bfloat16)
    assert ok, f"{what}: parameters out of tolerance (worst {worst})"


SHAPES = [(64, 512), (3, 4096), (100, 520), (257, 768), (130, 1032), (1, 512), (70, 2048 + 512), (5, 8200)]


@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16"), ("fp32", "fp32"), ("bf16", "fp32")])
@pytest.mark.parametrize("shape", SHAPES)
def test_rank1_against_oracle(cuda, p_dt, g_dt, shape):
    rows, cols = shape
    gen = torch.Generator().manual_seed(rows * 131 + cols)
    p0 = (torch.randn(rows, cols, generator=gen) * 0.05).to(DT[p_dt])
    dev = Rank1State(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.r.cpu(), dev.c.cpu())
    make = (grads_config1, grads_config3, grads_config1, grads_config3)
    for step in range(1, 5):
        g = make[step - 1](gen, rows * cols).view(rows, cols)
        if step == 2:
            g[rows // 2] = 0.0          # a row and a column without gradient
            g[:, 8:16] = 0.0
        g = g.to(DT[g_dt])
        prev = ref[0]
        ref = ot.step_quant_rank1(ref[0], g, *ref[1:], step=step, **HP)
        dev.step(g.to(cuda), step)
        _check(dev, ref, prev, f"{p_dt}/{g_dt} {shape} step {step}")
        ref = (dev.p.cpu().clone(),) + tuple(ref[1:])   # per-step parameter bound


def test_rank1_multi_tensor_and_options(cuda):
    """several matrices in one call (more than one launch batch), with a multiplier"""
    gen = torch.Generator().manual_seed(9)
    shapes = [(8 + i % 5, 512 + 8 * (i % 7)) for i in range(37)]
    ps = [(torch.randn(s, generator=gen) * 0.05) for s in shapes]
    devs = [Rank1State(p, cuda) for p in ps]
    refs = [(p.clone(), d.m.cpu(), d.v.cpu(), d.sm.cpu(), d.r.cpu(), d.c.cpu()) for p, d in zip(ps, devs)]
    dev_s = torch.tensor([0.125], device=cuda)
    for step in (1, 2):
        gs = [(grads_config1(gen, s[0] * s[1]) * 8).view(s).to(torch.bfloat16) for s in shapes]
        dgs = [g.to(cuda) for g in gs]
        q.fused_4bit_rank1_multi([d.p for d in devs], dgs, [d.m for d in devs], [d.v for d in devs],
                                 [d.sm for d in devs], [d.r for d in devs], [d.c for d in devs],
                                 [d.rn for d in devs], [d.cn for d in devs], *HPA, step,
                                 grad_scale_dev=dev_s, zero_grad=(step == 2))
        for i, (d, g) in enumerate(zip(devs, gs)):
            prev = refs[i][0]
            refs[i] = ot.step_quant_rank1(prev, g.float() * np.float32(0.125), *refs[i][1:], step=step, **HP)
            _check(d, refs[i], prev, f"tensor {i} step {step}")
            refs[i] = (d.p.cpu().clone(),) + tuple(refs[i][1:])
            assert bool(dgs[i].any()) == (step == 1)


def test_rank1_found_inf_leaves_everything(cuda):
    gen = torch.Generator().manual_seed(10)
    p0 = torch.randn(40, 1024, generator=gen) * 0.05
    dev = Rank1State(p0, cuda)
    g = grads_config1(gen, p0.numel()).view(p0.shape).to(torch.bfloat16).to(cuda)
    dev.step(g, 1)
    before = [t.clone() for t in dev.tensors()]
    flag = torch.ones(1, device=cuda)
    dev.step(g, 2, found_inf=flag)
    assert all(torch.equal(a, b) for a, b in zip(before, dev.tensors()))
    assert not dev.rn.any() and not dev.cn.any()


def test_rank1_full_size_matrix(cuda):
    """a Llama-3-8B MLP matrix, three steps, against the same oracle on the GPU (plain torch
    kernels); the oracle's GPU form is checked against its CPU form on a slice first"""
    gen = torch.Generator(device=cuda).manual_seed(11)
    small = torch.randn(64, 1024, generator=gen, device=cuda) * 0.05
    gs = (torch.randn(64, 1024, generator=gen, device=cuda) * 1e-3).to(torch.bfloat16)
    z = lambda n, dt=torch.float32: torch.zeros(n, dtype=dt, device=cuda)
    a = ot.step_quant_rank1(small, gs, z(32768, torch.uint8), z(32768, torch.uint8), z(512), z(64), z(1024), step=1, **HP)
    b = ot.step_quant_rank1(small.cpu(), gs.cpu(), z(32768, torch.uint8).cpu(), z(32768, torch.uint8).cpu(),
                            z(512).cpu(), z(64).cpu(), z(1024).cpu(), step=1, **HP)
    assert all(torch.equal(x.cpu(), y) for x, y in zip(a[1:], b[1:]))
    rows, cols = 4096, 14336
    p0 = torch.randn(rows, cols, generator=gen, device=cuda) * 0.02
    dev = Rank1State(p0, cuda)
    ref = (p0.clone(), dev.m.clone(), dev.v.clone(), dev.sm.clone(), dev.r.clone(), dev.c.clone())
    for step in (1, 2, 3):
        g = (torch.randn(rows, cols, generator=gen, device=cuda) * 1e-3 *
             torch.rand(rows, 1, generator=gen, device=cuda) * torch.rand(1, cols, generator=gen, device=cuda)
             ).to(torch.bfloat16)
        prev = ref[0]
        ref = ot.step_quant_rank1(ref[0], g, *ref[1:], step=step, **HP)
        dev.step(g, step)
        _check(dev, ref, prev, f"4096x14336 step {step}")
        ref = (dev.p.clone(),) + tuple(ref[1:])


def test_rank1_argument_errors(cuda):
    L = _lib.load()
    p = torch.zeros(4, 512, device=cuda)
    d = Rank1State(p, cuda)
    g = torch.zeros_like(p)
    arr = q.make_rank1_table([d.p], [g], [d.m], [d.v], [d.sm], [d.r], [d.c], [d.rn], [d.cn])
    call = lambda a: L.q4adamw_fused_4bit_rank1_multi(a, 1, 0, 0, *HPA, 1.0, None, None)
    arr[0].cols = 500
    assert call(arr) == -1 and b"cols" in L.q4adamw_last_error()
    arr[0].cols = 512
    arr[0].col_max = d.c.data_ptr() + 4
    assert call(arr) == -2
    arr[0].col_max = None
    assert call(arr) == -1
    with pytest.raises(AssertionError, match="rank-1"):
        q.make_rank1_table([torch.zeros(4, 100, device=cuda)], [torch.zeros(4, 100, device=cuda)], [d.m], [d.v],
                           [d.sm], [d.r], [d.c], [d.rn], [d.cn])
