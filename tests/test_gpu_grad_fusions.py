"""GPU parity of the gradient-side operations folded into the step (multiplier, overflow
flag, zeroing) and of the global gradient norm, through the C ABI.

The oracle for a step with multiplier s is the ordinary oracle step on the gradient
fp32(g) * s (oracle.q4_oracle.scale_grad).  Two size-independent properties tie the
extended kernels to the plain ones: a multiplier of exactly 1 changes no bit, and with
fp32 gradients a step with multiplier s equals, bit for bit, a plain step on g * s."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import q4_oracle as oc
from quantfour_adamw_cuda_amd import AdamWFused_QuantFour, _lib
from quantfour_adamw_cuda_amd import quantfour_hip as q
from tests.q4_testlib import (HP, DeviceTensor, OracleTensor, assert_state_equal, grads_config1,
                              grads_config3, to_np)

pytestmark = pytest.mark.gpu

DT = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}
HPA = (HP["beta1"], HP["beta2"], HP["lr"], HP["weight_decay"], HP["eps"])


def _step(d, g, step, **kw):
    q.fused_4bit_multi([d.p], [g], [d.m], [d.v], [d.sm], [d.sv], *HPA, step, **kw)


def _state_bits(d):
    return [t.clone() for t in (d.p, d.m, d.v, d.sm, d.sv)]


def _same(a, b):
    return all(torch.equal(x.view(torch.uint8), y.view(torch.uint8)) for x, y in zip(a, b))


@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16"), ("fp32", "fp32"), ("bf16", "fp32"),
                                       ("fp16", "fp16"), ("fp32", "fp16")])
@pytest.mark.parametrize("n", [128 * 1024 + 77, 4097])
def test_multiplier_against_oracle(cuda, p_dt, g_dt, n):
    """host multiplier, device multiplier and their product, three steps, ragged sizes"""
    gen = torch.Generator().manual_seed(100 + n % 7)
    p0 = (torch.randn(n, generator=gen) * 0.05).to(DT[p_dt])
    dev, ref = DeviceTensor(p0, cuda), OracleTensor(p0)
    dev_scalar = torch.tensor([1.0 / 1024.0], device=cuda)
    for step, (host_s, use_dev) in enumerate([(0.37, False), (1.0, True), (-3.0, True)], start=1):
        g = (grads_config1(gen, n) * 1024.0).to(DT[g_dt])
        s = np.float32(host_s) * (np.float32(1.0 / 1024.0) if use_dev else np.float32(1.0))
        prev = ref.p.copy()
        oc.step_quant(ref.p, oc.scale_grad(to_np(g), s), ref.m, ref.v, ref.sm, ref.sv, step=step, **HP)
        gd = g.to(cuda)
        _step(dev, gd, step, grad_scale=host_s, grad_scale_dev=dev_scalar if use_dev else None)
        assert torch.equal(gd.cpu(), g), "gradients must stay as they are"
        assert_state_equal(dev, ref, prev, f"{p_dt}/{g_dt} n={n} step {step}")
        ref.resync(dev.p)


@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16")])
def test_unit_multiplier_changes_no_bit(cuda, p_dt, g_dt):
    """the extended kernel with s = 1 (forced by a device scalar) equals the plain kernel"""
    n = 300_001
    gen = torch.Generator().manual_seed(3)
    p0 = (torch.randn(n, generator=gen) * 0.05).to(DT[p_dt])
    a, b = DeviceTensor(p0, cuda), DeviceTensor(p0, cuda)
    one = torch.ones(1, device=cuda)
    for step in (1, 2, 3):
        g = grads_config3(gen, n).to(DT[g_dt]).to(cuda)
        _step(a, g, step)
        _step(b, g, step, grad_scale_dev=one)
        assert _same(_state_bits(a), _state_bits(b)), f"step {step}"


def test_fp32_multiplier_equals_prescaled_gradient(cuda):
    """fp32 gradients: step(g, s) == step(g * s), every bit, at a full-size tensor"""
    n = 64 * 1024 * 1024 + 5
    gen = torch.Generator(device=cuda).manual_seed(4)
    p0 = torch.randn(n, generator=gen, device=cuda) * 0.05
    for p_dt in ("fp32", "bf16"):
        a, b = DeviceTensor(p0.to(DT[p_dt]), cuda), DeviceTensor(p0.to(DT[p_dt]), cuda)
        for step, s in ((1, 1.0 / 65536.0), (2, 0.3)):
            g = torch.randn(n, generator=gen, device=cuda) * 1e-3 / s
            _step(a, g, step, grad_scale=s)
            _step(b, g * np.float32(s), step)
            assert _same(_state_bits(a), _state_bits(b)), f"{p_dt} step {step}"


@pytest.mark.parametrize("g_dt", ["bf16", "fp32"])
def test_zero_grad_and_found_inf(cuda, g_dt):
    n = 200_003
    gen = torch.Generator().manual_seed(5)
    p0 = torch.randn(n, generator=gen) * 0.05
    a, b = DeviceTensor(p0, cuda), DeviceTensor(p0, cuda)
    flag = torch.zeros(1, device=cuda)
    for step in (1, 2):
        g = grads_config1(gen, n).to(DT[g_dt]).to(cuda)
        ga, gb = g.clone(), g.clone()
        _step(a, ga, step)
        _step(b, gb, step, zero_grad=True, found_inf=flag)
        assert _same(_state_bits(a), _state_bits(b)), f"step {step}"
        assert torch.equal(ga, g)
        assert not gb.any(), "gradients must be zero after a zeroing step"
    # overflow flag set: parameters and state stay; the gradients stay too unless the call
    # was to clear them (an overflowed gradient must not reach the next accumulation)
    before = _state_bits(b)
    flag.fill_(1.0)
    g = grads_config1(gen, n).to(DT[g_dt]).to(cuda)
    g[::1000] = float("inf")
    g0 = g.clone()
    _step(b, g, 3, found_inf=flag, grad_scale=0.5)
    assert _same(before, _state_bits(b)) and torch.equal(g, g0)
    _step(b, g, 3, zero_grad=True, found_inf=flag, grad_scale=0.5)
    assert _same(before, _state_bits(b))
    assert not g.any(), "a cancelled step still clears the gradients"


def test_small_tensor_kernel_options(cuda):
    """non-quantized kernel: multiplier against the oracle, zeroing, overflow flag"""
    gen = torch.Generator().manual_seed(6)
    sizes = [1, 5, 1023, 4096]
    ps = [(torch.randn(n, generator=gen) * 0.1) for n in sizes]
    dp = [p.clone().to(cuda) for p in ps]
    dm = [torch.zeros(n, device=cuda) for n in sizes]
    dv = [torch.zeros(n, device=cuda) for n in sizes]
    rp = [p.numpy().copy() for p in ps]
    rm = [np.zeros(n, np.float32) for n in sizes]
    rv = [np.zeros(n, np.float32) for n in sizes]
    flag = torch.zeros(1, device=cuda)
    dev_s = torch.tensor([0.25], device=cuda)
    for step in (1, 2):
        gs = [grads_config1(gen, n).to(torch.bfloat16) for n in sizes]
        dg = [g.to(cuda) for g in gs]
        q.fused_single_tensor_multi(dp, dg, dm, dv, *HPA, step, grad_scale=2.0, grad_scale_dev=dev_s,
                                    found_inf=flag, zero_grad=(step == 2))
        for i, g in enumerate(gs):
            oc.step_unquant(rp[i], oc.scale_grad(to_np(g), np.float32(2.0) * np.float32(0.25)), rm[i], rv[i],
                            step=step, **HP)
            assert np.array_equal(dm[i].cpu().numpy().view(np.uint32), rm[i].view(np.uint32))
            assert np.array_equal(dv[i].cpu().numpy().view(np.uint32), rv[i].view(np.uint32))
            np.testing.assert_allclose(dp[i].cpu().numpy(), rp[i], rtol=1e-6, atol=1e-9)
            assert bool(dg[i].any()) == (step == 1)
            rp[i][:] = dp[i].cpu().numpy()
    flag.fill_(3.0)
    before = [t.clone() for t in dp + dm + dv]
    dg = [grads_config1(gen, n).to(torch.bfloat16).to(cuda) for n in sizes]
    dg0 = [g.clone() for g in dg]
    q.fused_single_tensor_multi(dp, dg, dm, dv, *HPA, 3, found_inf=flag)
    assert all(torch.equal(x, y) for x, y in zip(before + dg0, dp + dm + dv + dg))
    q.fused_single_tensor_multi(dp, dg, dm, dv, *HPA, 3, found_inf=flag, zero_grad=True)
    assert all(torch.equal(x, y) for x, y in zip(before, dp + dm + dv))
    assert not any(bool(g.any()) for g in dg), "a cancelled step still clears the gradients"


def test_option_argument_errors(cuda):
    L = _lib.load()
    d = DeviceTensor(torch.zeros(4097), cuda)
    g = torch.zeros(4097, device=cuda)
    arr = q.make_table([d.p], [g], [d.m], [d.v], [d.sm], [d.sv])
    o = _lib.Q4GradOptions(1.0, 0, d.sm.data_ptr() + 2, None)
    rc = L.q4adamw_fused_4bit_multi_ex(arr, 1, 0, 0, *HPA, 1.0, ctypes.byref(o), None)
    assert rc == -2 and b"grad_scale_dev" in L.q4adamw_last_error()
    with pytest.raises(AssertionError, match="one float32"):
        q.grad_options(cuda, grad_scale_dev=torch.ones(2, device=cuda))
    with pytest.raises(AssertionError, match="device"):
        q.grad_options(cuda, found_inf=torch.ones(1))


# ---------------------------------------------------------------------------
# global gradient norm
# ---------------------------------------------------------------------------
def _f32(x):
    return np.float32(x)


@pytest.mark.parametrize("g_dt", ["bf16", "fp32"])
def test_grad_norm_against_oracle(cuda, g_dt):
    """ragged tensor list (more tensors than one launch holds), tails, empty tensors"""
    gen = torch.Generator().manual_seed(7)
    sizes = [0, 1, 7, 127, 4096, 8191, 8192, 8193, 16384, 16385, 70001, 1 << 20, (1 << 21) + 3]
    sizes += [int(x) for x in torch.randint(1, 3000, (170,), generator=gen)]
    gs = [grads_config1(gen, n).to(DT[g_dt]) for n in sizes]
    dg = [g.to(cuda) for g in gs]
    dev_s = torch.tensor([1.0 / 512.0], device=cuda)
    for host_s, sd, max_norm in ((1.0, None, 0.0), (1.0, None, 0.01), (-2.0, dev_s, 1e-4), (1.0, None, 1e6)):
        out = q.grad_norm(dg, grad_scale=host_s, grad_scale_dev=sd, max_norm=max_norm).cpu().numpy()
        s = _f32(host_s) * (_f32(1.0 / 512.0) if sd is not None else _f32(1.0))
        norm, coef, mult = oc.grad_norm([to_np(g) for g in gs], s, max_norm)
        # fp64 sums in two different orders, rounded to fp32: at most one fp32 ulp apart
        assert abs(out[0] - norm) <= np.spacing(norm), (out, norm)
        assert abs(out[1] - coef) <= 2 * np.spacing(coef), (out, coef)
        assert abs(out[2] - mult) <= 2 * np.spacing(abs(mult)), (out, mult)
        assert (out[1] == 1.0) == (coef == 1.0)


def test_grad_norm_closed_forms_and_determinism(cuda):
    ones = torch.ones((1 << 24) + 3, dtype=torch.bfloat16, device=cuda)
    out = q.grad_norm([ones, ones[:8]], grad_scale=0.5, max_norm=1.0).cpu().numpy()
    norm = _f32(0.5) * _f32(np.sqrt((1 << 24) + 11))
    assert out[0] == norm and out[1] == _f32(1.0) / (norm + _f32(1e-6)) and out[2] == _f32(0.5) * out[1]
    # the same input gives the same bits, whatever the workspace held before
    gen = torch.Generator(device=cuda).manual_seed(8)
    g = [torch.randn(n, generator=gen, device=cuda) for n in (1 << 22, 12345, 1 << 18)]
    ws = torch.full((_lib.NORM_WORKSPACE_BYTES // 8,), float("nan"), dtype=torch.float64, device=cuda)
    a = q.grad_norm(g, max_norm=1.0, workspace=ws).clone()
    ws.fill_(7.0)
    b = q.grad_norm(g, max_norm=1.0, workspace=ws)
    assert torch.equal(a, b)
    want = torch.linalg.vector_norm(torch.cat(g).double()).float()
    assert abs(float(a[0]) - float(want)) <= float(np.spacing(_f32(float(want))))
    # views at odd element offsets into a flat buffer give the bits of tensors of their own
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        flat = torch.randn((1 << 20) + 77, generator=gen, device=cuda).to(dt)
        views = [flat[1:300001], flat[300003:]]
        assert any(v.data_ptr() % 16 for v in views)
        a = q.grad_norm(views, max_norm=1.0).clone()
        assert torch.equal(a, q.grad_norm([v.clone() for v in views], max_norm=1.0)) and float(a[0]) > 0
    bad = torch.tensor([1.0, float("inf")], device=cuda)
    out = q.grad_norm([bad], max_norm=1.0).cpu().numpy()
    assert np.isinf(out[0]) and out[1] == 0.0
    out = q.grad_norm([torch.tensor([float("nan")], device=cuda)], max_norm=1.0).cpu().numpy()
    assert np.isnan(out[0]) and np.isnan(out[1])
    # no elements at all
    out = q.grad_norm([torch.zeros(0, device=cuda)], max_norm=1.0).cpu().numpy()
    assert out[0] == 0.0 and out[1] == 1.0


def test_grad_norm_argument_errors(cuda):
    L = _lib.load()
    g = torch.zeros(64, device=cuda)
    arr = q.make_grad_table([g])
    out = torch.zeros(3, device=cuda)
    ws = torch.zeros(_lib.NORM_WORKSPACE_BYTES // 8, dtype=torch.float64, device=cuda)
    call = lambda a, cnt, tag, w, wb, o: L.q4adamw_grad_norm(a, cnt, tag, 1.0, None, 0.0, w, wb, o, None)
    assert call(arr, 1, 0, ws.data_ptr(), 100, out.data_ptr()) == -1
    assert b"workspace" in L.q4adamw_last_error()
    assert call(arr, 1, 0, None, 16384, out.data_ptr()) == -1
    assert call(arr, 1, 7, ws.data_ptr(), 16384, out.data_ptr()) == -1
    assert call(arr, -1, 0, ws.data_ptr(), 16384, out.data_ptr()) == -1
    off = q.make_grad_table([g[1:]])
    off[0].g += 2                                              # half an element
    assert call(off, 1, 0, ws.data_ptr(), 16384, out.data_ptr()) == -2


# ---------------------------------------------------------------------------
# optimizer level
# ---------------------------------------------------------------------------
def _model(cuda, seed):
    torch.manual_seed(seed)
    return torch.nn.Sequential(torch.nn.Linear(96, 128), torch.nn.Tanh(), torch.nn.Linear(128, 64)).to(cuda)


def test_optimizer_clip_and_scale_equal_separate_passes(cuda):
    """step(grad_scale, max_grad_norm) == unscale pass + clip_grad_norm_ + plain step, up to the
    rounding of multiplying once by the product instead of twice (fp32 gradients: the moments'
    codes may differ only where a value sits within an ulp of a threshold, so compare the
    parameters)"""
    a, b = _model(cuda, 1), _model(cuda, 1)
    oa = AdamWFused_QuantFour(a.parameters(), lr=1e-3, weight_decay=0.01)
    ob = AdamWFused_QuantFour(b.parameters(), lr=1e-3, weight_decay=0.01)
    scale, max_norm = 1024.0, 0.05
    for it in range(4):
        x = torch.randn(32, 96, device=cuda)
        (a(x).square().mean() * scale).backward()
        (b(x).square().mean() * scale).backward()
        oa.step(grad_scale=1.0 / scale, max_grad_norm=max_norm, zero_grad=True)
        for p in b.parameters():
            p.grad.mul_(1.0 / scale)
        total = torch.nn.utils.clip_grad_norm_(b.parameters(), max_norm)
        ob.step()
        ob.zero_grad(set_to_none=False)
        assert abs(float(oa.last_grad_norm) - float(total)) <= 2e-6 * float(total)
        assert float(total) > max_norm, "the test must actually clip"
        for pa, pb in zip(a.parameters(), b.parameters()):
            assert not pa.grad.any()
            torch.testing.assert_close(pa, pb, rtol=0, atol=2e-4)  # lr * O(1) per differing code


def test_grad_scaler_drives_the_fused_path(cuda):
    """torch.amp.GradScaler.step(): the scale reaches the kernels as a device scalar, a step
    with an overflow changes nothing, and the scaler backs off"""
    m = _model(cuda, 2)
    opt = AdamWFused_QuantFour(m.parameters(), lr=1e-3)
    ref = _model(cuda, 2)
    ropt = AdamWFused_QuantFour(ref.parameters(), lr=1e-3)
    scaler = torch.amp.GradScaler("cuda", init_scale=2.0 ** 12)
    for it in range(3):
        x = torch.randn(16, 96, device=cuda)
        scaler.scale(m(x).square().mean()).backward()
        scaler.step(opt)
        scaler.update()
        opt.zero_grad(set_to_none=True)
        ref(x).square().mean().backward()
        ropt.step()
        ropt.zero_grad(set_to_none=True)
        for pa, pb in zip(m.parameters(), ref.parameters()):
            # power-of-two scale: scaling and unscaling are exact, so the runs are identical
            assert torch.equal(pa, pb)
    before = [p.detach().clone() for p in m.parameters()]
    x = torch.randn(16, 96, device=cuda)
    scaler.scale(m(x).square().mean()).backward()
    next(m.parameters()).grad[0, 0] = float("inf")
    s0 = scaler.get_scale()
    scaler.step(opt)
    scaler.update()
    assert all(torch.equal(p, q0) for p, q0 in zip(m.parameters(), before))
    assert scaler.get_scale() == s0 * 0.5
    # the skipped step does not count: state_dict() (and the next step) take its advance back
    assert all(float(st["step"]) == 3.0 for st in opt.state_dict()["state"].values())
    opt.zero_grad(set_to_none=True)
    ref.zero_grad(set_to_none=True)
    x = torch.randn(16, 96, device=cuda)
    scaler.scale(m(x).square().mean()).backward()
    scaler.step(opt)
    scaler.update()
    ref(x).square().mean().backward()
    ropt.step()
    assert all(float(st["step"]) == 4.0 for st in opt.state.values())
    for pa, pb in zip(m.parameters(), ref.parameters()):
        assert torch.equal(pa, pb)       # same bias corrections as the run that never overflowed


@pytest.mark.parametrize("variance", ["group", "rank1"])
def test_optimizer_cancelled_step_clears_gradients(cuda, variance):
    """an overflowed step changes neither parameters nor state nor step counters, and with
    zero_grad=True the overflowed gradients are gone afterwards: the next backward
    accumulates onto zeros and the run continues like one that never saw the overflow"""
    torch.manual_seed(3)
    mk = lambda: torch.nn.Sequential(torch.nn.Linear(512, 64), torch.nn.Tanh(), torch.nn.Linear(64, 8)).to(cuda)
    a, b = mk(), mk()
    b.load_state_dict(a.state_dict())
    oa = AdamWFused_QuantFour(a.parameters(), lr=1e-3, variance_scale_type=variance)
    ob = AdamWFused_QuantFour(b.parameters(), lr=1e-3, variance_scale_type=variance)
    flag = torch.zeros(1, device=cuda)
    for it in range(4):
        x = torch.randn(16, 512, device=cuda)
        if it == 2:    # a's extra, overflowed iteration
            a(x).square().mean().backward()
            next(a.parameters()).grad[0, :7] = float("nan")
            flag.fill_(1.0)
            oa.step(found_inf=flag, zero_grad=True)
            assert all(not p.grad.any() for p in a.parameters())
            flag.zero_()
        a(x).square().mean().backward()
        b(x).square().mean().backward()
        oa.step(found_inf=flag, zero_grad=True)
        ob.step(zero_grad=True)
        for pa, pb in zip(a.parameters(), b.parameters()):
            assert torch.equal(pa, pb), f"iteration {it}"
    sa, sb = oa.state_dict()["state"], ob.state_dict()["state"]
    assert all(float(sa[k]["step"]) == float(sb[k]["step"]) == 4.0 for k in sa)


def test_clip_pipeline_and_rank1_replay_under_graph_capture(cuda):
    """norm kernel -> step with the device multiplier -> rank-1 step (atomics, three launches):
    nothing allocates, synchronises or uses a memset, so the sequence can be captured; replays
    with refreshed gradients and eager work in between must equal eager launches bit for bit"""
    gen = torch.Generator().manual_seed(31)
    sizes = [70001, 4097, 128 * 40]
    ps = [torch.randn(n, generator=gen) * 0.02 for n in sizes]
    mat = torch.randn(24, 1024, generator=gen) * 0.02

    class Rank1:
        def __init__(self):
            self.p = mat.clone().to(cuda)
            n = mat.numel()
            self.m = torch.zeros(n // 2, dtype=torch.uint8, device=cuda)
            self.v = torch.zeros_like(self.m)
            self.sm = torch.zeros(n // 128, device=cuda)
            self.r, self.c = torch.zeros(24, device=cuda), torch.zeros(1024, device=cuda)
            self.rn, self.cn = torch.zeros(24, device=cuda), torch.zeros(1024, device=cuda)

        def all(self):
            return (self.p, self.m, self.v, self.sm, self.r, self.c, self.rn, self.cn)

    def fresh():
        return [DeviceTensor(p, cuda) for p in ps], Rank1()

    eager, graphed = fresh(), fresh()
    gbuf = [torch.zeros(n, device=cuda) for n in sizes] + [torch.zeros(24, 1024, device=cuda)]
    out = [torch.zeros(3, device=cuda) for _ in range(2)]
    ws = [torch.zeros(_lib.NORM_WORKSPACE_BYTES // 8, dtype=torch.float64, device=cuda) for _ in range(2)]

    def launch(state, gs, which):
        ts, r1 = state
        q.grad_norm(gs, grad_scale=0.5, max_norm=1e-3, out=out[which], workspace=ws[which])
        mult = out[which][2:3]
        q.fused_4bit_multi([x.p for x in ts], gs[:3], [x.m for x in ts], [x.v for x in ts], [x.sm for x in ts],
                           [x.sv for x in ts], *HPA, 2, grad_scale_dev=mult)
        q.fused_4bit_rank1_multi([r1.p], gs[3:], [r1.m], [r1.v], [r1.sm], [r1.r], [r1.c], [r1.rn], [r1.cn],
                                 *HPA, 2, grad_scale_dev=mult)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(graphed, gbuf, 1)                   # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graphed = fresh()                              # new state: re-capture against its pointers
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch(graphed, gbuf, 1)
    for rep in range(4):
        gs = [grads_config1(gen, n).to(cuda) for n in sizes] + [grads_config1(gen, 24 * 1024).view(24, 1024).to(cuda)]
        for b, g in zip(gbuf, gs):
            b.copy_(g)
        graph.replay()
        launch(eager, gs, 0)
        torch.cuda.synchronize()
        assert torch.equal(out[0].view(torch.int32), out[1].view(torch.int32)), f"replay {rep}: norm outputs"
        assert float(out[0][1]) < 1.0, "the pipeline must actually clip"
        for x, y in zip(graphed[0], eager[0]):
            for a, b in ((x.p, y.p), (x.m, y.m), (x.v, y.v), (x.sm, y.sm), (x.sv, y.sv)):
                assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"replay {rep}"
        for a, b in zip(graphed[1].all(), eager[1].all()):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"replay {rep}: rank-1 state"
