"""Full-size checks of benchmark configuration 3 (Llama-3-8B: fp32 params, bf16 grads) and
configs[4] (Llama-2-13B-shaped: bf16 params and grads): every tensor of the whole parameter
set, every step, against the vectorised oracle run with plain torch ops on the GPU -- after
that GPU run of the oracle has itself been checked against the C oracle -- plus format
properties that hold at any size."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import q4_oracle as oc
from oracle import q4_oracle_torch as ot
from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
from tests.q4_testlib import HP, bits, strict_param_metrics, to_np

pytestmark = pytest.mark.gpu
KW = dict(lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]), eps=HP["eps"], weight_decay=HP["weight_decay"])


def say(msg):
    print(msg, flush=True)


def student_t(shape, gen, device, scale=1e-4):
    z = torch.randn(shape, generator=gen, device=device)
    c = torch.zeros(shape, device=device)
    for _ in range(3):
        c += torch.randn(shape, generator=gen, device=device).square_()
    return (z * torch.rsqrt(c / 3.0) * scale).to(torch.bfloat16)


def test_gpu_run_of_the_torch_oracle_matches_the_c_oracle(cuda):
    """The checker used below: torch element-wise ops on the GPU must give the C oracle's
    bits (IEEE division and individually rounded multiplies and adds on the device)."""
    gen = torch.Generator().manual_seed(3)
    n = 3 * 1000003
    p = torch.randn(n, generator=gen) * 0.02
    nb, nk = oc.state_sizes(n)
    m, v = np.zeros(nb, np.uint8), np.zeros(nb, np.uint8)
    sm, sv = np.zeros(nk, np.float32), np.zeros(nk, np.float32)
    pc = p.numpy().copy()
    dp = p.to(cuda)
    dm, dv, dsm, dsv = (torch.from_numpy(x.copy()).to(cuda) for x in (m, v, sm, sv))
    for step in range(1, 4):
        z = torch.randn(n, generator=gen)
        g = (z / (torch.randn(3, n, generator=gen).square().sum(0) / 3).sqrt() * 1e-4).to(torch.bfloat16)
        if step == 2:
            g[1000:3000] = 0
        oc.step_quant(pc, to_np(g), m, v, sm, sv, step=step, **HP)
        dp, dm, dv, dsm, dsv = ot.step_quant(dp, g.to(cuda), dm, dv, dsm, dsv, step=step, **HP)
        assert np.array_equal(dm.cpu().numpy(), m) and np.array_equal(dv.cpu().numpy(), v)
        assert np.array_equal(bits(dsm.cpu().numpy()), bits(sm)) and np.array_equal(bits(dsv.cpu().numpy()), bits(sv))
        # parameters too, and cumulatively: neither side is re-based on the other
        assert np.array_equal(bits(dp.cpu().numpy()), bits(pc)), f"step {step}: the GPU run's parameters"


def llama3_8b_shapes():
    shapes = [(128256, 4096), (128256, 4096)]
    for _ in range(32):
        shapes += [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096),
                   (4096, 14336), (4096,), (4096,)]
    return shapes + [(4096,)]


def llama2_13b_shapes():
    shapes = [(32000, 5120), (32000, 5120)]
    for _ in range(40):
        shapes += [(5120, 5120)] * 4 + [(13824, 5120), (13824, 5120), (5120, 13824), (5120,), (5120,)]
    return shapes


def _check_tensor(p, st, before, g, step):
    """One tensor after a step against the oracle applied to its state before the step."""
    p0, m0, v0, sm0, sv0 = before
    if st["momentum_qstate"]["enable"]:
        rp, rm, rv, rsm, rsv = ot.step_quant(p0.reshape(-1), g.reshape(-1), m0, v0, sm0, sv0, step=step, **HP)
        assert torch.equal(st["exp_avg"], rm), f"first-moment codes, shape {tuple(p.shape)}"
        assert torch.equal(st["exp_avg_sq"], rv), f"second-moment codes, shape {tuple(p.shape)}"
        assert torch.equal(st["momentum_qstate"]["overhead"]["max1"].view(torch.int32), rsm.view(torch.int32))
        assert torch.equal(st["variance_qstate"]["overhead"]["max1"].view(torch.int32), rsv.view(torch.int32))
        # format properties: a non-zero block holds code 15 (second moment) resp. 15 or 0
        # (first moment) where its abs-max sits, an all-zero block holds only zero codes
        n = p.numel()
        if n % 256 == 0:
            vcodes = torch.maximum(st["exp_avg_sq"] & 15, st["exp_avg_sq"] >> 4).view(-1, 64).amax(1)
            sv = st["variance_qstate"]["overhead"]["max1"]
            assert torch.equal(vcodes == 15, sv > 0) and bool((vcodes[sv == 0] == 0).all())
    else:
        rp, rm, rv = ot.step_unquant(p0, g, m0, v0, step=step, **HP)
        assert torch.equal(st["exp_avg"].reshape(-1).view(torch.int32), rm.view(torch.int32))
        assert torch.equal(st["exp_avg_sq"].reshape(-1).view(torch.int32), rv.view(torch.int32))
    if p.dtype == torch.bfloat16:
        d = (p.detach().reshape(-1).float() - rp.reshape(-1).float()).abs()
        scale = torch.maximum(rp.reshape(-1).float().abs(), (rp.reshape(-1).float() - p0.reshape(-1).float()).abs())
        ulp = torch.exp2(torch.floor(torch.log2(scale.clamp_min(1e-30))) - 7)
        assert bool((d <= ulp).all()), f"bf16 params, shape {tuple(p.shape)}"
    else:
        # fp32 parameters come from the exact form of the update: bit for bit (and so within
        # the 1e-6 relative bound; the session summary reports the strict metrics as zeros)
        bad = int((p.detach().reshape(-1).view(torch.int32) != rp.reshape(-1).view(torch.int32)).sum())
        assert bad == 0, f"params, shape {tuple(p.shape)}: {bad} differ from the oracle's"
        strict = strict_param_metrics(p.detach(), rp, p0)
        assert strict["above"] == 0 and strict["max_rel"] == 0.0, f"params, shape {tuple(p.shape)}: {strict}"


def _run_config(shapes, p_dtype, cuda, steps, label):
    gen = torch.Generator(device=cuda).manual_seed(0)
    params = []
    for s in shapes:
        p = nn.Parameter((torch.randn(s, generator=gen, device=cuda) * 0.02).to(p_dtype))
        if p_dtype != torch.bfloat16:
            p.grad_dtype = torch.bfloat16
        params.append(p)
    total = sum(p.numel() for p in params)
    opt = AdamWFused_QuantFour(params, **KW)
    for step in range(1, steps + 1):
        grads = [student_t(s, gen, cuda) for s in shapes]
        if step == 2:
            grads[0][5000:6000] = 0       # embedding rows without gradient: all-zero blocks
        before = []
        for p in params:
            st = opt.state.get(p, {})
            if st:
                if st["momentum_qstate"]["enable"]:
                    before.append((p.detach().clone(), st["exp_avg"].clone(), st["exp_avg_sq"].clone(),
                                   st["momentum_qstate"]["overhead"]["max1"].clone(),
                                   st["variance_qstate"]["overhead"]["max1"].clone()))
                else:
                    before.append((p.detach().clone(), st["exp_avg"].clone(), st["exp_avg_sq"].clone(), None, None))
            else:
                n = p.numel()
                if n > 4096:
                    nb, nk = oc.state_sizes(n)
                    before.append((p.detach().clone(), torch.zeros(nb, dtype=torch.uint8, device=cuda),
                                   torch.zeros(nb, dtype=torch.uint8, device=cuda),
                                   torch.zeros(nk, device=cuda), torch.zeros(nk, device=cuda)))
                else:
                    before.append((p.detach().clone(), torch.zeros(n, device=cuda), torch.zeros(n, device=cuda), None, None))
        for p, g in zip(params, grads):
            p.grad = g
        say(f"[{label}] step {step}: {len(params)} tensors, {total / 1e9:.2f} G params")
        opt.step()
        torch.cuda.synchronize()
        for i, (p, g) in enumerate(zip(params, grads)):
            _check_tensor(p, opt.state[p], before[i], g, step)
            before[i] = None
        say(f"[{label}] step {step}: all tensors match the oracle")
        del before, grads
    return total


def test_llama3_8b_full_parameter_set(cuda):
    shapes = llama3_8b_shapes()
    assert len(shapes) == 291
    total = _run_config(shapes, torch.float32, cuda, 3, "llama3-8b fp32/bf16")
    assert total == 8030261248
    torch.cuda.empty_cache()


def test_llama2_13b_shaped_parameter_set_bf16(cuda):
    shapes = llama2_13b_shapes()
    assert len(shapes) == 362
    total = _run_config(shapes, torch.bfloat16, cuda, 3, "llama2-13b bf16/bf16")
    assert 13.0e9 < total < 13.1e9
    torch.cuda.empty_cache()


def test_more_than_2_to_32_elements_in_one_tensor(cuda):
    """element indices and byte offsets beyond 32 bits: a tensor of 2^32 + 2^20 + 77 elements in one
    call equals, bit for bit, the same data stepped as two tensors split at a block boundary
    (blocks are independent), for the plain step and for stochastic rounding with the salts and
    element offsets that make the noise line up only where it must"""
    from quantfour_adamw_cuda_amd import quantfour_hip as q
    n = (1 << 32) + (1 << 20) + 77
    cut = (1 << 32) - 5 * 128 * 1024            # multiple of 128 and of both chunk sizes
    gen = torch.Generator(device=cuda).manual_seed(12)
    hp = (0.9, 0.999, 1e-3, 0.01, 1e-8)

    def fresh():
        g_ = torch.Generator(device=cuda).manual_seed(13)
        p = torch.empty(n, dtype=torch.bfloat16, device=cuda).normal_(0, 0.05, generator=g_)
        m = torch.zeros((n + 1) // 2, dtype=torch.uint8, device=cuda)
        v = torch.zeros_like(m)
        sm = torch.zeros((n + 127) // 128, device=cuda)
        sv = torch.zeros_like(sm)
        return p, m, v, sm, sv

    g = torch.empty(n, dtype=torch.bfloat16, device=cuda).normal_(0, 1e-3, generator=gen)
    whole, parts = fresh(), fresh()
    for step in (1, 2):
        q.fused_4bit_multi([whole[0]], [g], [whole[1]], [whole[2]], [whole[3]], [whole[4]], *hp, step)
        a = [t[:c] for t, c in zip(parts, (cut, cut // 2, cut // 2, cut // 128, cut // 128))]
        b = [t[c:] for t, c in zip(parts, (cut, cut // 2, cut // 2, cut // 128, cut // 128))]
        q.fused_4bit_multi([a[0], b[0]], [g[:cut], g[cut:]], [a[1], b[1]], [a[2], b[2]], [a[3], b[3]],
                           [a[4], b[4]], *hp, step)
        for name, x, y in zip(("p", "m", "v", "sm", "sv"), whole, parts):
            assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), f"step {step}: {name} differs"
    assert whole[1][-1] < 16 and whole[1][cut // 2:].any()      # odd tail: high nibble stays clear
    # stochastic rounding: the noise of element e depends on e itself, so only the first part
    # of a split run sees the same noise; check that part, and that the tail beyond 2^32 is not
    # a repeat of the head (its hash mixes the high half of the index)
    sr_whole, sr_head = fresh(), fresh()
    q.fused_4bit_multi_sr([sr_whole[0]], [g], [sr_whole[1]], [sr_whole[2]], [sr_whole[3]], [sr_whole[4]],
                          *hp, 1, 42, salts=[3])
    h = [t[:c] for t, c in zip(sr_head, (cut, cut // 2, cut // 2, cut // 128, cut // 128))]
    q.fused_4bit_multi_sr([h[0]], [g[:cut]], [h[1]], [h[2]], [h[3]], [h[4]], *hp, 1, 42, salts=[3])
    assert torch.equal(sr_whole[1][:cut // 2], h[1]) and torch.equal(sr_whole[2][:cut // 2], h[2])
    # elements 2^32 .. 2^32 + 2^20 carry the gradients and parameters of elements 0 .. 2^20 in a
    # second run; with identical inputs only the noise can make their codes differ
    g2, rep = g.clone(), fresh()
    g2[1 << 32:(1 << 32) + (1 << 20)] = g[:1 << 20]
    rep[0][1 << 32:(1 << 32) + (1 << 20)] = rep[0][:1 << 20]
    q.fused_4bit_multi_sr([rep[0]], [g2], [rep[1]], [rep[2]], [rep[3]], [rep[4]], *hp, 1, 42, salts=[3])
    lo, hi = rep[1][:1 << 19], rep[1][1 << 31:(1 << 31) + (1 << 19)]
    assert torch.equal(rep[3][:1 << 13], rep[3][1 << 25:(1 << 25) + (1 << 13)])      # same block scales
    assert 0.01 < float((lo != hi).float().mean()) < 0.9


@pytest.mark.parametrize("rows_half,cols,form", [(131080, 16384, 0), (130056, 16512, 1)])
def test_more_than_2_to_32_elements_in_one_rank1_matrix(cuda, rows_half, cols, form):
    """Rank-1 scaling couples a matrix's rows through the column maxima, so a split run is not
    the same computation -- unless both halves hold the same data: the matrix [A; A] has A's
    column maxima and A's row maxima twice, so its step must equal, bit for bit, the step of A
    alone, in its upper half (elements below 2^32) and in its lower half (offsets beyond 2^32).
    Both update forms that a matrix of this size can take: tiles aligned to the rows, and rows
    that end in a partial tile (which such a matrix leaves to the kernel with tiles anywhere)."""
    from quantfour_adamw_cuda_amd import _lib, quantfour_hip as q
    half = rows_half * cols
    assert 2 * half > 1 << 32 and half > 1 << 31
    assert _lib.load().q4adamw_rank1_form(2 * rows_half, cols, 1) == form
    hp = (0.9, 0.999, 1e-3, 0.01, 1e-8)

    def state(rows):
        n = rows * cols
        g_ = torch.Generator(device=cuda).manual_seed(21)
        p = torch.empty(half, dtype=torch.bfloat16, device=cuda).normal_(0, 0.05, generator=g_)
        if rows != rows_half:
            p = torch.cat([p, p])
        return [p.view(rows, cols), torch.zeros((n + 1) // 2, dtype=torch.uint8, device=cuda),
                torch.zeros((n + 1) // 2, dtype=torch.uint8, device=cuda), torch.zeros((n + 127) // 128, device=cuda),
                torch.zeros(rows, device=cuda), torch.zeros(cols, device=cuda),
                torch.zeros(rows, device=cuda), torch.zeros(cols, device=cuda)]

    one, two = state(rows_half), state(2 * rows_half)
    gen = torch.Generator(device=cuda).manual_seed(22)
    for step in (1, 2):
        g = torch.empty(half, dtype=torch.bfloat16, device=cuda).normal_(0, 1e-3, generator=gen)
        g[:cols] *= 8.0                     # a loud first row and a silent column: maxima that matter
        g.view(rows_half, cols)[:, 5] = 0
        gg = torch.cat([g, g])
        for st, grad in ((one, g.view(rows_half, cols)), (two, gg.view(2 * rows_half, cols))):
            q.fused_4bit_rank1_multi([st[0]], [grad], [st[1]], [st[2]], [st[3]], [st[4]], [st[5]], [st[6]], [st[7]],
                                     *hp, step)
        del gg
        names = ("p", "m codes", "v codes", "m scales", "row maxima")
        for name, a, b in zip(names, one[:5], two[:5]):
            a8, b8 = a.reshape(-1).view(torch.uint8), b.reshape(-1).view(torch.uint8)
            k = a8.numel()
            assert torch.equal(b8[:k], a8), f"step {step}: {name}, upper half"
            assert torch.equal(b8[k:], a8), f"step {step}: {name}, lower half (offsets beyond 2^32)"
        assert torch.equal(one[5].view(torch.int32), two[5].view(torch.int32)), f"step {step}: column maxima"
        assert not one[6].any() and not two[6].any() and not two[7].any(), "scratch maxima return to zero"
    assert one[1].any() and one[2].any() and float(one[5][5]) == 0.0
