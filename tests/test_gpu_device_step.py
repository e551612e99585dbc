"""A step whose number lives on the device: q4adamw_bias_table + q4adamw_device_step +
q4adamw_grad_options.step_consts.  The derived scalars are made on the device with the host's
own operations, so a step made this way must equal, bit for bit, the step made with the same
step number on the host -- also when the whole sequence is a captured graph that is replayed."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import q4_oracle as oc
from quantfour_adamw_cuda_amd import _lib
from quantfour_adamw_cuda_amd import quantfour_hip as q
from tests.q4_testlib import HP, DeviceTensor, grads_config1

HPA = (HP["beta1"], HP["beta2"], HP["lr"], HP["weight_decay"], HP["eps"])


def test_bias_table_is_the_launchers_arithmetic():
    """host only: every entry equals what the step's launcher derives for that step number
    (oracle: q4o_derive_scalars, optim/cuda_adamw_kernels.cu:435-436); bad arguments are refused"""
    L = _lib.load()
    for b1, b2, first, count in ((0.9, 0.999, 1, 300), (0.8, 0.88, 1, 64), (0.95, 0.9999, 5000, 100)):
        out = (ctypes.c_float * (2 * count))()
        assert L.q4adamw_bias_table(b1, b2, first, count, out) == 0
        got = np.frombuffer(out, np.float32).reshape(count, 2)
        for k in (0, 1, count // 2, count - 1):
            sc = oc.derive_scalars(b1, b2, 1e-3, 0.01, first + k)
            assert got[k, 0].view(np.uint32) == np.float32(sc[0]).view(np.uint32)
            assert got[k, 1].view(np.uint32) == np.float32(sc[1]).view(np.uint32)
    one = (ctypes.c_float * 2)()
    assert L.q4adamw_bias_table(1.0, 0.999, 1, 1, one) == -3
    assert L.q4adamw_bias_table(0.9, 0.999, 0, 1, one) == -1
    assert L.q4adamw_bias_table(0.9, 0.999, 1, 1, None) == -1
    assert L.q4adamw_bias_table(0.9, 0.999, 1, 0, None) == 0


def _same(a, b):
    return all(torch.equal(x, y) for x, y in zip((a.p, a.m, a.v, a.sm, a.sv), (b.p, b.m, b.v, b.sm, b.sv)))


@pytest.mark.gpu
@pytest.mark.parametrize("p_dt,g_dt", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16),
                                       (torch.float32, torch.float32)])
def test_device_step_equals_host_step(cuda, p_dt, g_dt):
    """quantized and non-quantized kernels, a learning rate that changes every step and comes
    from device memory, a start in the middle of training, an overflow flag"""
    gen = torch.Generator().manual_seed(3)
    n = 100_003
    p0 = (torch.randn(n, generator=gen) * 0.05).to(p_dt)
    a, b = DeviceTensor(p0, cuda), DeviceTensor(p0, cuda)
    s0 = (torch.randn(900, generator=gen) * 0.05).to(p_dt)
    small = [s0.clone().to(cuda) for _ in range(2)]
    sm_state = [[torch.zeros(900, device=cuda) for _ in range(2)] for _ in range(2)]
    table = q.make_bias_table(HP["beta1"], HP["beta2"], cuda)
    assert table.shape[0] >= 32768 and float(table[-1, 0]) == 1.0 and float(table[-1, 1]) == 1.0
    consts, flag = q.new_step_consts(cuda), torch.zeros(1, device=cuda)
    lr_dev = torch.zeros(1, device=cuda)
    for first in (0, 4999):                     # the counter holds the number of steps taken
        counter = torch.full((1,), float(first), device=cuda)
        for k in range(1, 5):
            lr = 1e-3 * (1.0 + 0.25 * k)
            lr_dev.fill_(lr)
            lr32 = float(lr_dev)                  # the fp32 value both sides use
            g = grads_config1(gen, n).to(g_dt).to(cuda)
            gs = grads_config1(gen, 900).to(g_dt).to(cuda)
            q.fused_4bit_multi([a.p], [g], [a.m], [a.v], [a.sm], [a.sv], HP["beta1"], HP["beta2"], lr32,
                               HP["weight_decay"], HP["eps"], first + k)
            q.fused_single_tensor_multi([small[0]], [gs], [sm_state[0][0]], [sm_state[0][1]], HP["beta1"], HP["beta2"],
                                        lr32, HP["weight_decay"], HP["eps"], first + k)
            q.device_step(counter, table, consts, HP["beta1"], HP["beta2"], 123.0, HP["weight_decay"], HP["eps"],
                          lr_dev=lr_dev, found_inf=flag)
            q.fused_4bit_multi([b.p], [g], [b.m], [b.v], [b.sm], [b.sv], HP["beta1"], HP["beta2"], 123.0,
                               HP["weight_decay"], HP["eps"], 1, step_consts=consts, found_inf=flag)
            q.fused_single_tensor_multi([small[1]], [gs], [sm_state[1][0]], [sm_state[1][1]], HP["beta1"], HP["beta2"],
                                        123.0, HP["weight_decay"], HP["eps"], 1, step_consts=consts)
            assert float(counter) == first + k
            assert _same(a, b), f"start {first} step {k}"
            assert torch.equal(small[0], small[1]) and all(torch.equal(x, y) for x, y in zip(*sm_state))
    # overflow: the counter stays, the scalars stay, nothing is stepped
    flag.fill_(1.0)
    before = [t.clone() for t in (b.p, b.m, b.v, b.sm, b.sv, counter, consts)]
    q.device_step(counter, table, consts, *HPA, found_inf=flag)
    q.fused_4bit_multi([b.p], [g], [b.m], [b.v], [b.sm], [b.sv], *HPA, 1, step_consts=consts, found_inf=flag)
    assert all(torch.equal(x, y) for x, y in zip(before, (b.p, b.m, b.v, b.sm, b.sv, counter, consts)))
    # far past the table both corrections are 1, as they are on the host
    flag.zero_()
    far = table.shape[0] + 12345
    counter.fill_(float(far - 1))
    q.device_step(counter, table, consts, *HPA)
    q.fused_4bit_multi([b.p], [g], [b.m], [b.v], [b.sm], [b.sv], *HPA, 1, step_consts=consts)
    q.fused_4bit_multi([a.p], [g], [a.m], [a.v], [a.sm], [a.sv], *HPA, far)
    assert _same(a, b)
    # stochastic rounding: the noise's salt is finished on the device from the step number there
    arr = q.make_table([b.p], [g], [b.m], [b.v], [b.sm], [b.sv])
    salts = q.make_salts([77])
    for k in (1, 2):
        q.device_step(counter, table, consts, *HPA)
        q.launch_table_sr(arr, salts, 0xABCDEF0123456789, cuda, q._tag(b.p, "param"), q._tag(g, "grad"), *HPA, 1,
                          q.grad_options(cuda, step_consts=consts))
        q.fused_4bit_multi_sr([a.p], [g], [a.m], [a.v], [a.sm], [a.sv], *HPA, far + k, 0xABCDEF0123456789, salts=[77])
        assert float(counter) == far + k and _same(a, b), f"stochastic rounding, step {far + k}"


@pytest.mark.gpu
def test_training_steps_replayed_from_one_captured_graph(cuda):
    """step counter, block-scaled step, non-quantized step and rank-1 step captured once; every
    replay is the next training step (fresh gradients in the same buffers, a new learning rate
    in device memory) and equals the eager step with that step number on the host"""
    gen = torch.Generator().manual_seed(9)
    n, rows, cols = 70_001, 70, 1024      # rows of whole tiles: the update kernel that shares column maxima
    p0, s0, m0 = (torch.randn(k, generator=gen) * 0.05 for k in (n, 777, rows * cols))

    class State:
        def __init__(self):
            self.big = DeviceTensor(p0, cuda)
            self.small = s0.clone().to(cuda)
            self.small_m, self.small_v = torch.zeros(777, device=cuda), torch.zeros(777, device=cuda)
            self.mat = DeviceTensor(m0, cuda)
            self.mat.p = self.mat.p.view(rows, cols)
            self.r, self.c, self.rn, self.cn = (torch.zeros(k, device=cuda) for k in (rows, cols, rows, cols))

        def tensors(self):
            return (self.big.p, self.big.m, self.big.v, self.big.sm, self.big.sv, self.small, self.small_m, self.small_v,
                    self.mat.p, self.mat.m, self.mat.v, self.mat.sm, self.r, self.c)

        def step(self, g_big, g_small, g_mat, lr, step, **kw):
            hp = (HP["beta1"], HP["beta2"], lr, HP["weight_decay"], HP["eps"])
            q.fused_4bit_multi([self.big.p], [g_big], [self.big.m], [self.big.v], [self.big.sm], [self.big.sv], *hp, step, **kw)
            q.fused_single_tensor_multi([self.small], [g_small], [self.small_m], [self.small_v], *hp, step, **kw)
            q.fused_4bit_rank1_multi([self.mat.p], [g_mat], [self.mat.m], [self.mat.v], [self.mat.sm], [self.r], [self.c],
                                     [self.rn], [self.cn], *hp, step, **kw)

    eager, replayed = State(), State()
    table = q.make_bias_table(HP["beta1"], HP["beta2"], cuda)
    consts, counter, lr_dev = q.new_step_consts(cuda), torch.zeros(1, device=cuda), torch.full((1,), 1e-3, device=cuda)
    bufs = [torch.zeros(n, dtype=torch.bfloat16, device=cuda), torch.zeros(777, dtype=torch.bfloat16, device=cuda),
            torch.zeros(rows, cols, dtype=torch.bfloat16, device=cuda)]

    def one_step():
        q.device_step(counter, table, consts, HP["beta1"], HP["beta2"], 1.0, HP["weight_decay"], HP["eps"], lr_dev=lr_dev)
        replayed.step(*bufs, 1.0, 1, step_consts=consts)

    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            one_step()
    torch.cuda.current_stream(cuda).wait_stream(side)
    torch.cuda.synchronize()
    assert float(counter) == 0.0, "capture must not run the kernels"
    for step in range(1, 7):
        lr = 1e-3 / step
        lr_dev.fill_(lr)
        gs = [grads_config1(gen, b.numel()).view(b.shape).to(torch.bfloat16).to(cuda) for b in bufs]
        for b, g in zip(bufs, gs):
            b.copy_(g)
        graph.replay()
        eager.step(*gs, float(lr_dev), step)
        torch.cuda.synchronize()
        _ = torch.randn(1000, device=cuda).sum().item()      # eager work between replays
        assert float(counter) == step
        for i, (x, y) in enumerate(zip(eager.tensors(), replayed.tensors())):
            assert torch.equal(x, y), f"step {step}: tensor {i}"


@pytest.mark.gpu
def test_device_step_argument_errors(cuda):
    L = _lib.load()
    t = torch.zeros(64, device=cuda)
    ok = (t.data_ptr(), t.data_ptr() + 64, 1, 4, None, 0.9, 0.999, 1e-3, 0.01, 1e-8, None, t.data_ptr() + 128, None)
    call = lambda *args: L.q4adamw_device_step(*args)
    assert call(None, *ok[1:]) == -1
    assert call(ok[0], None, *ok[2:]) == -1
    assert call(*ok[:3], 0, *ok[4:]) == -1
    assert call(*ok[:5], 1.5, *ok[6:]) == -3
    assert call(*ok[:11], t.data_ptr() + 132, None) == -2
    assert call(ok[0] + 2, *ok[1:]) == -2
    o = _lib.Q4GradOptions()
    o.grad_scale, o.step_consts = 1.0, t.data_ptr() + 4
    arr = (_lib.Q4Tensor * 1)()
    assert L.q4adamw_fused_4bit_multi_ex(arr, 1, 0, 0, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, ctypes.byref(o), None) == -2


@pytest.mark.gpu
@pytest.mark.parametrize("variance,rounding", [("group", "real-nearest"), ("rank1", "real-nearest"),
                                               ("group", "stochastic"), ("rank1", "stochastic")])
def test_capturable_optimizer_replays_equal_the_eager_optimizer(cuda, variance, rounding):
    """AdamWFused_QuantFour(capturable=True): one warm-up step, then step(zero_grad=True) is
    captured once and replayed; every replay is the next step (device counter, tensor lr) and
    equals, bit for bit, a second optimizer stepping eagerly with the step number on the host;
    state_dict() reports the device's step count; a resumed optimizer continues identically"""
    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
    gen = torch.Generator().manual_seed(12)
    shapes = [(40, 1024), (68, 768), (300, 33), (64,), (5000,), (16, 520)]
    init = [torch.randn(s, generator=gen) * 0.05 for s in shapes]
    pc = [torch.nn.Parameter(t.clone().to(cuda)) for t in init]
    pe = [torch.nn.Parameter(t.clone().to(cuda)) for t in init]
    lr_t = torch.full((), 1e-3, device=cuda)
    kw = dict(weight_decay=0.01, variance_scale_type=variance, round_type=rounding, seed=31)
    oc_ = AdamWFused_QuantFour(pc, lr=lr_t, capturable=True, **kw)
    oe = AdamWFused_QuantFour(pe, lr=1e-3, **kw)
    static = [torch.zeros_like(p) for p in pc]
    for p, g in zip(pc, static):
        p.grad = g

    def fresh_grads(step):
        gs = [(grads_config1(gen, p.numel()).view(p.shape)).to(cuda) for p in pc]
        for buf, g, p in zip(static, gs, pe):
            buf.copy_(g)
            p.grad = g.clone()
        lr = 1e-3 / step
        lr_t.fill_(lr)
        oe.param_groups[0]["lr"] = float(lr_t)

    def check(step):
        for i, (a, b) in enumerate(zip(pc, pe)):
            assert torch.equal(a, b), f"step {step}: parameter {i}"
            sa, sb = oc_.state[a], oe.state[b]
            assert torch.equal(sa["exp_avg"], sb["exp_avg"]) and torch.equal(sa["exp_avg_sq"], sb["exp_avg_sq"]), (step, i)
            assert not a.grad.any(), "zero_grad inside the captured step"

    fresh_grads(1)
    oc_.step(zero_grad=True)            # warm-up: state and descriptor tables exist before the capture
    oe.step()
    check(1)
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    graph = torch.cuda.CUDAGraph()
    fresh_grads(2)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            oc_.step(zero_grad=True)
    torch.cuda.current_stream(cuda).wait_stream(side)
    torch.cuda.synchronize()
    for step in range(2, 8):
        if step > 2:
            fresh_grads(step)
        graph.replay()
        oe.step()
        torch.cuda.synchronize()
        check(step)
    sd = oc_.state_dict()
    assert all(float(s["step"]) == 7.0 for s in sd["state"].values())
    assert all(float(s["step"]) == 7.0 for s in oe.state_dict()["state"].values())
    # resume (eagerly) from the captured run's state: the counter restarts from the loaded number
    p2 = [torch.nn.Parameter(p.detach().clone()) for p in pc]
    o2 = AdamWFused_QuantFour(p2, lr=1e-3, capturable=True, **kw)
    o2.load_state_dict(sd)
    assert torch.is_tensor(o2.param_groups[0]["lr"])      # a copy of the saved tensor
    o2.param_groups[0]["lr"] = lr_t
    fresh_grads(8)
    for p, g in zip(p2, pe):
        p.grad = g.grad.clone()
    o2.step()
    oe.step()
    for a, b in zip(p2, pe):
        assert torch.equal(a, b)
    # a parameter without a gradient is refused: the group shares one counter
    p2[0].grad = None
    with pytest.raises(ValueError, match="every parameter"):
        o2.step()


@pytest.mark.gpu
def test_capturable_optimizer_overflow_flag_and_float_lr(cuda):
    """a set overflow flag leaves the device counter where it is (state_dict() reports it); a
    float lr that changes between eager steps is picked up"""
    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
    gen = torch.Generator().manual_seed(13)
    init = [torch.randn(s, generator=gen) * 0.05 for s in ((70, 130), (33,))]
    pc = [torch.nn.Parameter(t.clone().to(cuda)) for t in init]
    pe = [torch.nn.Parameter(t.clone().to(cuda)) for t in init]
    a = AdamWFused_QuantFour(pc, lr=1e-3, capturable=True)
    b = AdamWFused_QuantFour(pe, lr=1e-3)
    flag = torch.zeros(1, device=cuda)
    for it in range(5):
        gs = [grads_config1(gen, p.numel()).view(p.shape).to(cuda) for p in pc]
        for opt, ps in ((a, pc), (b, pe)):
            opt.param_groups[0]["lr"] = 1e-3 * (it + 1)
            for p, g in zip(ps, gs):
                p.grad = g.clone()
        if it == 2:      # an overflowed iteration for the capturable optimizer only
            flag.fill_(1.0)
            a.step(found_inf=flag)
            flag.zero_()
            assert all(float(s["step"]) == 2.0 for s in a.state_dict()["state"].values())
        a.step(found_inf=flag)
        b.step()
        for x, y in zip(pc, pe):
            assert torch.equal(x, y), f"iteration {it}"
    assert all(float(s["step"]) == 5.0 for s in a.state_dict()["state"].values())
