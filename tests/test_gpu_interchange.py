"""Checkpoint interchange: stand-alone quantize / dequantize against the oracle, taking over
the state of torch.optim.AdamW (quantize on load) and handing state back as fp32."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import quantfour_adamw_cuda_amd as q4
from oracle import q4_oracle as oc
from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
from tests.q4_testlib import HP, bits, grads_config3, p_close, to_np

pytestmark = pytest.mark.gpu
KW = dict(lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]), eps=HP["eps"], weight_decay=HP["weight_decay"])


@pytest.mark.parametrize("n", [1, 2, 127, 128, 129, 255, 4097, 1000003])
@pytest.mark.parametrize("which", [0, 1])
def test_quantize_dequantize_match_oracle(cuda, n, which):
    gen = torch.Generator().manual_seed(n + which)
    x = grads_config3(gen, n)
    if n > 1000:
        x[128:384] = 0                       # all-zero blocks: scale 0, codes 0
        qmid = torch.from_numpy(oc.tables(which)[1])
        x[512:512 + 15] = qmid * x[384:512].abs().max()   # ties
    if which:
        x = x * x
    print(f"[quantize] n={n} which={which}", flush=True)
    codes, scales = q4.quantize_state(x.to(cuda), which)
    torch.cuda.synchronize()
    rc, rs = oc.quant(x.numpy(), which)
    assert np.array_equal(codes.cpu().numpy(), rc)
    assert np.array_equal(bits(scales.cpu().numpy()), bits(rs))
    back = q4.dequantize_state(codes, scales, n, which)
    torch.cuda.synchronize()
    assert np.array_equal(bits(back.cpu().numpy()), bits(oc.dequant(rc, rs, n, which)))


def test_take_over_adamw_state_and_hand_it_back(cuda):
    gen = torch.Generator().manual_seed(17)
    shapes = [(130, 257), (4096,), (5000,), (33, 129)]
    host = [torch.randn(s, generator=gen) * 0.02 for s in shapes]
    ref_params = [nn.Parameter(h.clone().to(cuda)) for h in host]
    adamw = torch.optim.AdamW(ref_params, **KW)
    for _ in range(3):
        for p in ref_params:
            p.grad = (torch.randn(p.shape, generator=gen) * 1e-3).to(cuda)
        adamw.step()
    sd = adamw.state_dict()

    params = [nn.Parameter(p.detach().clone()) for p in ref_params]
    opt = AdamWFused_QuantFour(params, **KW)
    opt.load_state_dict(sd)
    torch.cuda.synchronize()
    twins = []
    for p, rp in zip(params, ref_params):
        st, rst = opt.state[p], adamw.state[rp]
        assert float(st["step"]) == 3.0 and st["step"].device.type == "cpu"
        m32, v32 = rst["exp_avg"].cpu().numpy().reshape(-1), rst["exp_avg_sq"].cpu().numpy().reshape(-1)
        if p.numel() > 4096:
            mc, ms = oc.quant(m32, 0)
            vc, vs = oc.quant(v32, 1)
            assert st["exp_avg"].dtype == torch.uint8 and np.array_equal(st["exp_avg"].cpu().numpy(), mc)
            assert np.array_equal(st["exp_avg_sq"].cpu().numpy(), vc)
            assert np.array_equal(bits(st["momentum_qstate"]["overhead"]["max1"].cpu().numpy()), bits(ms))
            assert np.array_equal(bits(st["variance_qstate"]["overhead"]["max1"].cpu().numpy()), bits(vs))
            twins.append(("q", to_np(p.detach()), mc, vc, ms, vs))
        else:
            assert st["exp_avg"].dtype == torch.float32 and not st["momentum_qstate"]["enable"]
            assert np.array_equal(bits(st["exp_avg"].cpu().numpy().reshape(-1)), bits(m32))
            twins.append(("s", to_np(p.detach()), m32.copy(), v32.copy()))
    # training goes on from step 4, in step with the oracle
    for step in (4, 5):
        grads = [torch.randn(s, generator=gen) * 1e-3 for s in shapes]
        for p, g in zip(params, grads):
            p.grad = g.to(cuda)
        opt.step()
        torch.cuda.synchronize()
        for tw, p, g in zip(twins, params, grads):
            prev = tw[1].copy()
            if tw[0] == "q":
                oc.step_quant(tw[1], g.numpy().reshape(-1), tw[2], tw[3], tw[4], tw[5], step=step, **HP)
                assert np.array_equal(opt.state[p]["exp_avg"].cpu().numpy(), tw[2])
                assert np.array_equal(opt.state[p]["exp_avg_sq"].cpu().numpy(), tw[3])
            else:
                oc.step_unquant(tw[1], g.numpy().reshape(-1), tw[2], tw[3], step=step, **HP)
                assert np.array_equal(bits(opt.state[p]["exp_avg"].cpu().numpy().reshape(-1)), bits(tw[2]))
            ok, worst = p_close(to_np(p.detach()), tw[1], prev, exact=True)   # fp32 parameters: bit for bit
            assert ok, worst
            tw[1][:] = to_np(p.detach())
    # and back: fp32 state that torch.optim.AdamW accepts
    back = opt.adamw_state_dict()
    fresh = [nn.Parameter(p.detach().clone()) for p in params]
    adamw2 = torch.optim.AdamW(fresh, **KW)
    adamw2.load_state_dict(back)
    for tw, p, f in zip(twins, params, fresh):
        st = adamw2.state[f]
        assert float(st["step"]) == 5.0 and st["exp_avg"].shape == p.shape
        if tw[0] == "q":
            want_m = oc.dequant(tw[2], tw[4], p.numel(), 0)
            want_v = oc.dequant(tw[3], tw[5], p.numel(), 1)
        else:
            want_m, want_v = tw[2], tw[3]
        assert np.array_equal(bits(st["exp_avg"].cpu().numpy().reshape(-1)), bits(want_m))
        assert np.array_equal(bits(st["exp_avg_sq"].cpu().numpy().reshape(-1)), bits(want_v))
    for f in fresh:
        f.grad = torch.zeros_like(f)
    adamw2.step()                                # the library routine runs on it


@pytest.mark.parametrize("which", [0, 1])
def test_quantize_non_finite_values(cuda, which):
    """a NaN never becomes a block's scale (the oracle's running maximum skips it) and gets code 0;
    an infinite scale sends the block's finite values to x / inf = 0"""
    from oracle import q4_oracle_torch as ot
    from quantfour_adamw_cuda_amd import quantfour_hip as q
    gen = torch.Generator().manual_seed(23 + which)
    x = torch.randn(128 * 12, generator=gen)
    x = x * x if which else x
    x[3] = float("nan")
    x[128:256] = float("nan")
    x[256 + 4] = float("inf")
    x[384 + 5], x[384 + 6] = float("inf"), float("nan")
    x[512 + 64], x[512 + 65] = float("nan"), float("nan")          # one lane's both values
    codes, scales = q4.quantize_state(x.to(cuda), which)
    rc, rs = oc.quant(x.numpy(), which)
    assert np.array_equal(bits(scales.cpu().numpy()), bits(rs)), (scales.cpu().numpy(), rs)
    assert np.array_equal(codes.cpu().numpy(), rc)
    if which:
        m = x.view(12, 128).clone()
        m = torch.cat([m] * 5, dim=1)[:, :512].contiguous()           # 12 x 512 with the same oddities
        c1, r1, k1 = q.quantize_state_rank1(m.to(cuda))
        c2, r2, k2 = ot.quantize_rank1(m)
        assert torch.equal(r1.cpu().view(torch.int32), r2.view(torch.int32))
        assert torch.equal(k1.cpu().view(torch.int32), k2.view(torch.int32))
        assert torch.equal(c1.cpu(), c2)
