"""GPU parity of the fused step with a rank-1-scaled second moment, through the C ABI,
against the torch restatement in oracle/q4_oracle_torch.py (itself pinned by brute force and
closed forms in tests/test_oracle_pins.py): codes, block scales and row / column maxima bit
for bit, parameters within the step's tolerance."""
import numpy as np
import pytest
import torch

from oracle import q4_oracle_torch as ot
from quantfour_adamw_cuda_amd import _lib
from quantfour_adamw_cuda_amd import quantfour_hip as q
from tests.q4_testlib import HP, grads_config1, grads_config3, p_close, to_np

pytestmark = pytest.mark.gpu

DT = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}
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


SHAPES = [(66, 1024), (128, 1536), (64, 4096), (64, 512), (3, 4096), (100, 520), (257, 768), (130, 1032), (1, 512), (70, 2048 + 512), (5, 8200),
          # rows of whole blocks whose last tile is a partial one (384, 256 and 128 of a 512-element
          # tile, 128 of a 256-element one), row counts that are and are not multiples of four
          (66, 2432), (64, 4352), (65, 6272), (67, 2176),
          # narrow matrices: a tile spans several rows (fewer than 256 columns, or than 512 when
          # parameters and gradients are 16-bit types)
          (300, 16), (77, 64), (1000, 24), (513, 248), (40, 504), (9, 256), (2000, 136),
          # rows of any length: no multiple of 8, or shorter than 16; rows then start at any
          # element of the packed codes and an access of 4 or 8 elements crosses rows
          (130, 1031), (257, 77), (33, 129), (4500, 2), (700, 9), (64, 2501), (3, 4099), (1, 5001), (100, 12)]


@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16"), ("fp32", "fp32"), ("bf16", "fp32"),
                                       ("fp16", "fp16"), ("fp32", "fp16"), ("fp16", "fp32")])
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


@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16"), ("fp32", "fp32"), ("bf16", "fp32"),
                                       ("fp16", "fp16")])
@pytest.mark.parametrize("shape", [(64, 512), (70, 2048 + 512), (100, 520), (130, 1032), (5, 8200), (333, 40), (50, 264),
                                   (65, 2432), (66, 4352)])     # rows whose last tile is a partial one
def test_rank1_stochastic_rounding_against_oracle(cuda, p_dt, g_dt, shape):
    """rank-1 scaling and stochastic rounding together: codes, scales and statistics bit for
    bit against step_quant_rank1_sr; the noise follows seed, step and the tensor's salt"""
    rows, cols = shape
    gen = torch.Generator().manual_seed(rows * 137 + cols)
    p0 = (torch.randn(rows, cols, generator=gen) * 0.05).to(DT[p_dt])
    dev = Rank1State(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.r.cpu(), dev.c.cpu())
    seed, salt = 0x1234_5678_9ABC_DEF0 + rows, cols % 13
    make = (grads_config1, grads_config3, grads_config1, grads_config3)
    for step in range(1, 5):
        g = make[step - 1](gen, rows * cols).view(rows, cols)
        if step == 2:
            g[rows // 2] = 0.0
            g[:, 8:16] = 0.0
        g = g.to(DT[g_dt])
        prev = ref[0]
        ref = ot.step_quant_rank1_sr(ref[0], g, *ref[1:], seed=seed, tensor_salt=salt, step=step, **HP)
        dev.step(g.to(cuda), step, seed=seed, salts=[salt])
        _check(dev, ref, prev, f"sr {p_dt}/{g_dt} {shape} step {step}")
        ref = (dev.p.cpu().clone(),) + tuple(ref[1:])


@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16")])
def test_rank1_long_run_stays_bit_exact(cuda, p_dt, g_dt, stochastic):
    """60 consecutive steps of one matrix (rows that end in a partial tile): codes, scales and
    statistics feed back into themselves and are compared bit for bit after every step, while
    the gradients' magnitude decays, rows and columns fall silent and come back, and spikes
    move the row and column maxima"""
    rows, cols = 96, 2432
    gen = torch.Generator().manual_seed(777)
    p0 = (torch.randn(rows, cols, generator=gen) * 0.05).to(DT[p_dt])
    dev = Rank1State(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.r.cpu(), dev.c.cpu())
    seed, salt = 0x0BAD_CAFE_1234, 5
    for step in range(1, 61):
        g = torch.randn(rows, cols, generator=gen) * (1e-2 * 0.95 ** step)
        regime = (step // 5) % 4
        if regime == 1:
            g[step % rows] = 0.0
            g[:, (step * 8) % cols:(step * 8) % cols + 64] = 0.0
        elif regime == 2:
            g[torch.rand(rows, cols, generator=gen) > 0.9995] *= 200.0
        elif regime == 3 and step % 2:
            g.zero_()
        g = g.to(DT[g_dt])
        prev = ref[0]
        if stochastic:
            ref = ot.step_quant_rank1_sr(ref[0], g, *ref[1:], seed=seed, tensor_salt=salt, step=step, **HP)
            dev.step(g.to(cuda), step, seed=seed, salts=[salt])
        else:
            ref = ot.step_quant_rank1(ref[0], g, *ref[1:], step=step, **HP)
            dev.step(g.to(cuda), step)
        _check(dev, ref, prev, f"long run {p_dt}/{g_dt} sr={stochastic} step {step}")
        ref = (dev.p.cpu().clone(),) + tuple(ref[1:])
    assert ref[1].any() and ref[2].any() and ref[4].min() > 0 and ref[5].min() > 0


def test_rank1_stochastic_rounding_many_tensors_and_options(cuda):
    """40 matrices in one call (two launch batches): default salts are the positions in the
    list, the call is reproducible, another seed changes codes; gradient multiplier on top"""
    gen = torch.Generator().manual_seed(19)
    shapes = [(6 + i % 4, 512 + 8 * (i % 5)) for i in range(40)]
    ps = [(torch.randn(s, generator=gen) * 0.05) for s in shapes]
    gs = [(grads_config1(gen, s[0] * s[1]) * 4).view(s).to(torch.bfloat16) for s in shapes]
    dev_s = torch.tensor([0.25], device=cuda)

    def run(seed):
        devs = [Rank1State(p, cuda) for p in ps]
        q.fused_4bit_rank1_multi([d.p for d in devs], [g.to(cuda) for g in gs], [d.m for d in devs],
                                 [d.v for d in devs], [d.sm for d in devs], [d.r for d in devs],
                                 [d.c for d in devs], [d.rn for d in devs], [d.cn for d in devs], *HPA, 1,
                                 grad_scale_dev=dev_s, seed=seed)
        return devs

    a, b, c = run(5), run(5), run(6)
    for i, (d, p, g) in enumerate(zip(a, ps, gs)):
        z8, zs = torch.zeros_like(d.m).cpu(), torch.zeros_like(d.sm).cpu()
        ref = ot.step_quant_rank1_sr(p, g.float() * np.float32(0.25), z8, z8.clone(), zs, torch.zeros(p.shape[0]),
                                     torch.zeros(p.shape[1]), seed=5, tensor_salt=i, step=1, **HP)
        _check(d, ref, p, f"tensor {i}")
        assert all(torch.equal(x, y) for x, y in zip(d.tensors(), b[i].tensors()))
    assert any(not torch.equal(x.v, y.v) for x, y in zip(a, c))
    assert all(torch.equal(x.r, y.r) and torch.equal(x.c, y.c) for x, y in zip(a, c))   # statistics do not depend on the noise


ND_SHAPES = [(4, 6, 64), (3, 5, 520), (2, 3, 4, 32), (8, 16, 1024), (1, 7, 16), (5, 1, 2, 264), (6, 7, 101), (3, 4, 5, 7)]


@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("p_dt,g_dt", [("fp32", "bf16"), ("bf16", "bf16"), ("fp32", "fp32")])
@pytest.mark.parametrize("shape", ND_SHAPES)
def test_rank1_more_than_two_dimensions_against_oracle(cuda, shape, p_dt, g_dt, stochastic):
    """tensors of three and four dimensions: one statistic per dimension (maximum over all
    others), scale = their minimum; codes, first-moment scales, every dimension's statistic
    and the derived row scales bit for bit against step_quant_rank1_nd over four steps"""
    gen = torch.Generator().manual_seed(sum(shape) * 7 + len(shape))
    n, cols, k = int(np.prod(shape)), shape[-1], len(shape) - 1
    rows = n // cols
    p0 = (torch.randn(shape, generator=gen) * 0.05).to(DT[p_dt])
    z = lambda m, dt=torch.float32: torch.zeros(m, dtype=dt, device=cuda)
    p, m, v, sm = p0.clone().to(cuda), z((n + 1) // 2, torch.uint8), z((n + 1) // 2, torch.uint8), z((n + 127) // 128)
    lead, lead_next = [z(shape[j]) for j in range(k)], [z(shape[j]) for j in range(k)]
    rs, rn, c, cn = z(rows), z(rows), z(cols), z(cols)
    ref = (p0.clone(), m.cpu(), v.cpu(), sm.cpu(),
           [torch.zeros([shape[j] if d == j else 1 for d in range(len(shape))]) for j in range(len(shape))])
    sr = dict(seed=0x5151_0000_ABCD + n, tensor_salt=3) if stochastic else {}
    make = (grads_config1, grads_config3, grads_config1, grads_config3)
    for step in range(1, 5):
        g = make[step - 1](gen, n).view(shape)
        if step == 2:
            g[shape[0] // 2] = 0.0          # a slice of the first dimension and some columns without gradient
            g[..., 8:16] = 0.0
        g = g.to(DT[g_dt])
        prev = ref[0]
        ref = ot.step_quant_rank1_nd(ref[0], g, *ref[1:], step=step, **sr, **HP)
        kw = dict(seed=sr["seed"], salts=[sr["tensor_salt"]]) if stochastic else {}
        q.fused_4bit_rank1_multi([p], [g.to(cuda)], [m], [v], [sm], [rs], [c], [rn], [cn], *HPA, step,
                                 leads=[(lead, lead_next)], **kw)
        what = f"{shape} {p_dt}/{g_dt} sr={stochastic} step {step}"
        assert torch.equal(m.cpu(), ref[1]), f"{what}: m codes"
        assert torch.equal(sm.cpu().view(torch.int32), ref[3].view(torch.int32)), f"{what}: m scales"
        for j in range(k):
            assert torch.equal(lead[j].cpu().view(torch.int32), ref[4][j].reshape(-1).view(torch.int32)), f"{what}: statistic {j}"
            assert not lead_next[j].any()
        assert torch.equal(c.cpu().view(torch.int32), ref[4][k].reshape(-1).view(torch.int32)), f"{what}: last statistic"
        assert torch.equal(rs, q.rank1_row_scale(lead, shape[:-1])), f"{what}: row scales"
        assert not rn.any() and not cn.any(), f"{what}: scratch"
        bad = torch.nonzero(v.cpu() != ref[2]).reshape(-1)
        assert bad.numel() == 0, f"{what}: v codes differ at bytes {bad[:5].tolist()} ({bad.numel()})"
        ok, worst = p_close(to_np(p), to_np(ref[0]), to_np(prev), bf16=DT[p_dt] == torch.bfloat16)
        assert ok, f"{what}: parameters (worst {worst})"
        ref = (p.cpu().clone(),) + tuple(ref[1:])


def test_rank1_multi_tensor_and_options(cuda):
    """several matrices in one call (more than one launch batch), with a multiplier"""
    gen = torch.Generator().manual_seed(9)
    shapes = [(8 + i % 5, 512 + 8 * (i % 7)) for i in range(37)]
    shapes += [(65, 512), (70, 768), (64, 1024)]      # rows of whole tiles: the kernel that shares column maxima
    shapes += [(66, 2176), (65, 2432)]                # the same with a partial last tile in every row
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


@pytest.mark.parametrize("rows,cols", [(40, 1024), (66, 1024),     # 66 rows of four tiles: the kernel that shares column maxima
                                       (66, 2176)])                # and with a partial last tile in every row
def test_rank1_found_inf_leaves_everything(cuda, rows, cols):
    gen = torch.Generator().manual_seed(10)
    p0 = torch.randn(rows, cols, generator=gen) * 0.05
    dev = Rank1State(p0, cuda)
    g = grads_config1(gen, p0.numel()).view(p0.shape).to(torch.bfloat16).to(cuda)
    dev.step(g, 1)
    before = [t.clone() for t in dev.tensors()]
    flag = torch.ones(1, device=cuda)
    g0 = g.clone()
    dev.step(g, 2, found_inf=flag)
    assert all(torch.equal(a, b) for a, b in zip(before, dev.tensors()))
    assert not dev.rn.any() and not dev.cn.any() and torch.equal(g, g0)
    dev.step(g, 2, found_inf=flag, zero_grad=True)   # cancelled, but the gradients are cleared
    assert all(torch.equal(a, b) for a, b in zip(before, dev.tensors()))
    assert not dev.rn.any() and not dev.cn.any() and not g.any()


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
    arr[0].cols = 1
    assert call(arr) == -1 and b"columns" in L.q4adamw_last_error()
    arr[0].rows, arr[0].cols = 1 << 20, 4100           # rows of any length: fewer than 2^32 elements
    assert call(arr) == -4 and b"2^32" in L.q4adamw_last_error()
    arr[0].rows, arr[0].cols = 4, 512
    arr[0].col_max = d.c.data_ptr() + 4
    assert call(arr) == -2
    arr[0].col_max = None
    assert call(arr) == -1
    with pytest.raises(AssertionError, match="rank-1"):
        q.make_rank1_table([torch.zeros(400, 1, device=cuda)], [torch.zeros(400, 1, device=cuda)], [d.m], [d.v],
                           [d.sm], [d.r], [d.c], [d.rn], [d.cn])


# ---------------------------------------------------------------------------
# interchange kernels and the optimizer class
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(1, 8), (7, 24), (64, 512), (130, 1032), (300, 264), (33, 129), (257, 77), (5, 5), (4001, 1)])
def test_rank1_quantize_dequantize_against_oracle(cuda, shape):
    gen = torch.Generator().manual_seed(shape[0] + shape[1])
    x = torch.rand(shape, generator=gen) ** 6
    x[shape[0] // 2] = 0.0
    x[:, min(3, shape[1] - 1)] = 0.0
    codes, rmax, cmax = q.quantize_state_rank1(x.to(cuda))
    rc, rr, rcm = ot.quantize_rank1(x)
    assert torch.equal(codes.cpu(), rc) and torch.equal(rmax.cpu(), rr) and torch.equal(cmax.cpu(), rcm)
    back = q.dequantize_state_rank1(codes, rmax, cmax)
    want = ot.dequantize_rank1(rc, rr, rcm)
    assert torch.equal(back.cpu().view(torch.int32), want.view(torch.int32))
    # signed input: statistics are maxima of magnitudes
    y = x.clone()
    y[0] = -y[0]
    _, r2, c2 = q.quantize_state_rank1(y.to(cuda))
    assert torch.equal(r2.cpu(), rr) and torch.equal(c2.cpu(), rcm)


def _mlp(cuda, seed):
    torch.manual_seed(seed)
    return torch.nn.Sequential(torch.nn.Linear(512, 96), torch.nn.Tanh(), torch.nn.Linear(96, 1024),
                               torch.nn.Tanh(), torch.nn.Linear(1024, 16)).to(cuda)


def test_optimizer_rank1_layout_tracking_and_resume(cuda):
    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
    with pytest.raises(ValueError, match="variance_scale_type"):
        AdamWFused_QuantFour([torch.nn.Parameter(torch.zeros(2, device=cuda))], variance_scale_type="rank2")
    model, twin = _mlp(cuda, 3), _mlp(cuda, 3)
    opt = AdamWFused_QuantFour(model.parameters(), lr=1e-3, weight_decay=0.01, variance_scale_type="rank1")
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-3, weight_decay=0.01)
    for it in range(10):
        x = torch.randn(32, 512, device=cuda)
        for m_, o_ in ((model, opt), (twin, ref)):
            o_.zero_grad(set_to_none=True)
            m_(x).square().mean().backward()
            o_.step()
    # layout: all three weight matrices are rank-1 scaled ([1024, 96] through the narrow path)
    w0, w1, w2 = model[0].weight, model[2].weight, model[4].weight
    ov = lambda p: opt.state[p]["variance_qstate"]["overhead"]
    assert [tuple(t.shape) for t in ov(w0)["max_dims"]] == [(96, 1), (1, 512)] and ov(w0)["max1"] is None
    assert [tuple(t.shape) for t in ov(w2)["max_dims"]] == [(16, 1), (1, 1024)]
    assert [tuple(t.shape) for t in ov(w1)["max_dims"]] == [(1024, 1), (1, 96)] and ov(w1)["max1"] is None
    assert all(not t.any() for t in ov(w0)["scratch_dims"])
    assert opt.state[model[0].bias]["exp_avg_sq"].dtype == torch.float32      # below the threshold
    # the draft's own bar against AdamW (tests/driver.py:70-71)
    for a, b in zip(model.parameters(), twin.parameters()):
        torch.testing.assert_close(a, b, atol=0.025, rtol=1e-5)
    # export: dequantized second moment is close to AdamW's (4-bit resolution of its scale)
    exported = opt.adamw_state_dict()["state"]
    v4 = exported[0]["exp_avg_sq"]
    v32 = ref.state[twin[0].weight]["exp_avg_sq"]
    scale = torch.minimum(v32.amax(1, keepdim=True), v32.amax(0, keepdim=True))
    assert float(((v4 - v32).abs() / scale).max()) < 0.2
    # resume from a state_dict: bit-identical continuation
    sd = opt.state_dict()
    model2 = _mlp(cuda, 4)
    model2.load_state_dict(model.state_dict())
    opt2 = AdamWFused_QuantFour(model2.parameters(), lr=1e-3, weight_decay=0.01, variance_scale_type="rank1")
    opt2.load_state_dict(sd)
    x = torch.randn(32, 512, device=cuda)
    for m_, o_ in ((model, opt), (model2, opt2)):
        o_.zero_grad(set_to_none=True)
        m_(x).square().mean().backward()
        o_.step()
    for a, b in zip(model.parameters(), model2.parameters()):
        assert torch.equal(a, b)
    for pa, pb in zip(model.parameters(), model2.parameters()):
        sa, sb = opt.state[pa], opt2.state[pb]
        assert torch.equal(sa["exp_avg_sq"], sb["exp_avg_sq"]) and torch.equal(sa["exp_avg"], sb["exp_avg"])
    # adopting torch.optim.AdamW's state quantizes the second moment with rank-1 statistics
    opt3 = AdamWFused_QuantFour(_mlp(cuda, 3).parameters(), lr=1e-3, variance_scale_type="rank1")
    opt3.load_state_dict(ref.state_dict())
    p3 = opt3.param_groups[0]["params"][0]
    md = opt3.state[p3]["variance_qstate"]["overhead"]["max_dims"]
    assert torch.equal(md[0].reshape(-1), v32.amax(1)) and torch.equal(md[1].reshape(-1), v32.amax(0))
    want_codes, _, _ = ot.quantize_rank1(v32.cpu())
    assert torch.equal(opt3.state[p3]["exp_avg_sq"].cpu(), want_codes)


def test_optimizer_rank1_with_stochastic_rounding(cuda):
    """variance_scale_type="rank1" with round_type="stochastic": same seed -> identical run,
    another seed -> another run, resume continues the noise sequence, and the run tracks
    torch.optim.AdamW within the draft's bar (tests/driver.py:70-71)"""
    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour

    def run(seed, steps, model=None, opt=None):
        model = model or _mlp(cuda, 3)
        opt = opt or (AdamWFused_QuantFour(model.parameters(), lr=1e-3, weight_decay=0.01,
                                           variance_scale_type="rank1", round_type="stochastic", seed=seed)
                      if seed is not None else torch.optim.AdamW(model.parameters(), lr=1e-3, weight_decay=0.01))
        gen = torch.Generator(device=cuda).manual_seed(0)
        for i in range(steps):
            x = torch.randn(32, 512, generator=gen, device=cuda)
            if i < int(getattr(opt, "_skip_first", 0)):
                continue
            opt.zero_grad(set_to_none=True)
            model(x).square().mean().backward()
            opt.step()
        return model, opt

    m1, o1 = run(7, 8)
    m2, _ = run(7, 8)
    m3, _ = run(8, 8)
    assert all(torch.equal(a, b) for a, b in zip(m1.parameters(), m2.parameters()))
    assert any(not torch.equal(a, b) for a, b in zip(m1.parameters(), m3.parameters()))
    w0 = m1[0].weight
    assert "max_dims" in o1.state[w0]["variance_qstate"]["overhead"]
    ref, _ = run(None, 8)
    for a, b in zip(m1.parameters(), ref.parameters()):
        torch.testing.assert_close(a, b, atol=0.025, rtol=1e-5)
    # resume after 5 steps == 8 steps straight through
    m5, o5 = run(7, 5)
    m_res = _mlp(cuda, 4)
    m_res.load_state_dict(m5.state_dict())
    o_res = AdamWFused_QuantFour(m_res.parameters(), variance_scale_type="rank1")
    o_res.load_state_dict(o5.state_dict())
    assert o_res.param_groups[0]["round_type"] == "stochastic" and o_res.param_groups[0]["seed"] == 7
    o_res._skip_first = 5
    run(7, 8, m_res, o_res)
    assert all(torch.equal(a, b) for a, b in zip(m1.parameters(), m_res.parameters()))


def test_optimizer_rank1_with_tensors_of_more_than_two_dimensions(cuda):
    """a stack of expert matrices [experts, in, out] and a 4-D kernel in one model: layout,
    tracking of torch.optim.AdamW within the draft's bar, bit-identical resume, adoption of
    AdamW state (codes equal the oracle's N-D quantizer) and fp32 export"""
    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour

    class Net(torch.nn.Module):
        def __init__(self, seed):
            super().__init__()
            g_ = torch.Generator().manual_seed(seed)
            self.experts = torch.nn.Parameter(torch.randn(4, 96, 512, generator=g_) * 0.05)
            self.kernel = torch.nn.Parameter(torch.randn(16, 8, 3, 32, generator=g_) * 0.05)
            self.out = torch.nn.Linear(512, 16)

        def forward(self, x):                                    # x: [batch, 96]
            h = torch.einsum("bi,eio->beo", x, self.experts).mean(1)           # [batch, 512]
            k = self.kernel.sum(dim=(1, 2))                                      # [16, 32]
            return self.out(torch.tanh(h)) + torch.tanh(h[:, :32] @ k.t())

    def make(seed):
        return Net(seed).to(cuda)

    model, twin = make(5), make(5)
    twin.load_state_dict(model.state_dict())          # the Linear layer draws from the global generator
    opt = AdamWFused_QuantFour(model.parameters(), lr=1e-3, weight_decay=0.01, variance_scale_type="rank1")
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-3, weight_decay=0.01)
    gen = torch.Generator(device=cuda).manual_seed(1)
    for it in range(10):
        x = torch.randn(32, 96, generator=gen, device=cuda)
        for m_, o_ in ((model, opt), (twin, ref)):
            o_.zero_grad(set_to_none=True)
            m_(x).square().mean().backward()
            o_.step()
    ov = lambda p: opt.state[p]["variance_qstate"]["overhead"]
    assert [tuple(t.shape) for t in ov(model.experts)["max_dims"]] == [(4, 1, 1), (1, 96, 1), (1, 1, 512)]
    assert [tuple(t.shape) for t in ov(model.kernel)["max_dims"]] == [(16, 1, 1, 1), (1, 8, 1, 1), (1, 1, 3, 1), (1, 1, 1, 32)]
    assert ov(model.experts)["row_scale"].numel() == 4 * 96 and not ov(model.experts)["row_scratch"].any()
    assert all(not t.any() for t in ov(model.kernel)["scratch_dims"])
    for a, b in zip(model.parameters(), twin.parameters()):
        torch.testing.assert_close(a, b, atol=0.025, rtol=1e-5)
    # export: the dequantized second moment is AdamW's to the 4-bit resolution of its scale
    v32 = ref.state[twin.experts]["exp_avg_sq"]
    exported = opt.adamw_state_dict()["state"][0]["exp_avg_sq"]
    assert exported.shape == v32.shape and exported.dtype == torch.float32
    stats = [v32.amax(dim=[d for d in range(3) if d != j], keepdim=True) for j in range(3)]
    scale = torch.minimum(torch.minimum(stats[0], stats[1]), stats[2])
    assert float(((exported - v32).abs() / scale).max()) < 0.3        # ten requantizations at 1/16 resolution
    # resume: bit-identical continuation
    model2 = make(6)
    model2.load_state_dict(model.state_dict())
    opt2 = AdamWFused_QuantFour(model2.parameters(), lr=1e-3, weight_decay=0.01, variance_scale_type="rank1")
    opt2.load_state_dict(opt.state_dict())
    x = torch.randn(32, 96, generator=gen, device=cuda)
    for m_, o_ in ((model, opt), (model2, opt2)):
        o_.zero_grad(set_to_none=True)
        m_(x).square().mean().backward()
        o_.step()
    for a, b in zip(model.parameters(), model2.parameters()):
        assert torch.equal(a, b)
    for pa, pb in zip(model.parameters(), model2.parameters()):
        assert torch.equal(opt.state[pa]["exp_avg_sq"], opt2.state[pb]["exp_avg_sq"])
    # adopting torch.optim.AdamW's state
    opt3 = AdamWFused_QuantFour(make(5).parameters(), lr=1e-3, variance_scale_type="rank1")
    opt3.load_state_dict(ref.state_dict())
    p3 = opt3.param_groups[0]["params"][0]
    want_codes, want_dims = ot.quantize_rank1_nd(v32.cpu())
    assert torch.equal(opt3.state[p3]["exp_avg_sq"].cpu(), want_codes)
    for a, b in zip(opt3.state[p3]["variance_qstate"]["overhead"]["max_dims"], want_dims):
        assert torch.equal(a.cpu(), b)


def test_rank1_more_than_2_to_32_elements(cuda):
    """a matrix of 2 x 33000 x 65536 elements (4.3e9) whose lower half repeats the upper half:
    row and column maxima of the whole equal those of a half, so the run on the whole matrix
    must reproduce, in both halves, the run on one half -- rows whose flat indices lie beyond
    2^32 included"""
    half_rows, cols = 33000, 65536
    gen = torch.Generator(device=cuda).manual_seed(14)
    p_half = torch.empty(half_rows, cols, dtype=torch.bfloat16, device=cuda).normal_(0, 0.05, generator=gen)
    half, whole = Rank1State(p_half, cuda), Rank1State(torch.cat([p_half, p_half]), cuda)
    for step in (1, 2):
        g_half = torch.empty(half_rows, cols, dtype=torch.bfloat16, device=cuda).normal_(0, 1e-3, generator=gen)
        g_half *= torch.rand(half_rows, 1, device=cuda, generator=gen).to(torch.bfloat16)
        half.step(g_half, step)
        whole.step(torch.cat([g_half, g_half]), step)
        n2 = half_rows * cols // 2
        for name, w, h in (("p", whole.p.view(-1), half.p.view(-1)), ("m", whole.m, half.m), ("v", whole.v, half.v),
                           ("sm", whole.sm, half.sm), ("r", whole.r, half.r)):
            k = h.numel()
            assert torch.equal(w[:k].view(torch.uint8), h.view(torch.uint8)), f"step {step}: upper half {name}"
            assert torch.equal(w[k:].view(torch.uint8), h.view(torch.uint8)), f"step {step}: lower half {name}"
        assert torch.equal(whole.c, half.c)
    assert whole.v.any() and whole.r.min() > 0


def test_rank1_non_finite_gradients(cuda):
    """inf and NaN gradients: maxima are taken over the non-NaN values, an infinite scale sends
    finite values to code 0 (x / inf = 0), NaN and inf / inf get code 0"""
    rows, cols = 40, 1024
    gen = torch.Generator().manual_seed(19)
    p0 = torch.randn(rows, cols, generator=gen) * 0.05
    dev = Rank1State(p0, cuda)
    ref = (p0.clone(), dev.m.cpu(), dev.v.cpu(), dev.sm.cpu(), dev.r.cpu(), dev.c.cpu())
    for step in (1, 2, 3):
        g = grads_config1(gen, rows * cols).view(rows, cols)
        if step == 2:
            g[3, 5] = float("inf")
            g[7, 100] = float("nan")
            g[9] = float("nan")
            g[11, 5], g[11, 6] = float("-inf"), float("nan")
        ref = ot.step_quant_rank1(ref[0], g, *ref[1:], step=step, **HP)
        dev.step(g.to(cuda), step)
        for name, d, r in list(zip(("p", "m codes", "v codes", "m scales", "row maxima", "column maxima"),
                                   dev.tensors(), ref))[1:]:
            d = d.cpu()
            same = torch.equal(d.view(torch.int32), r.view(torch.int32)) if d.dtype == torch.float32 else torch.equal(d, r)
            assert same, f"step {step}: {name} differ at {torch.nonzero(d != r).reshape(-1)[:6].tolist()}"
        ref = (dev.p.cpu().clone(),) + tuple(ref[1:])
