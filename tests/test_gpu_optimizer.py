"""GPU tests of the optimizer class: the reference's own test idea (tests/driver.py: track
torch.optim.AdamW on a small MLP), the multi-tensor GPT-2-small parameter set against the
oracle, checkpoint resume, and the real Llama-3-8B tensor shapes."""
from copy import deepcopy

import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import q4_oracle as oc
from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
from tests.q4_testlib import HP, bits, grads_config1, p_close, to_np

pytestmark = pytest.mark.gpu

KW = dict(lr=HP["lr"], betas=(HP["beta1"], HP["beta2"]), eps=HP["eps"], weight_decay=HP["weight_decay"])


def say(msg):
    print(msg, flush=True)


def _driver_loop(model, model_clone, fourbit, iters=10, size=5, atol=0.025):
    """tests/driver.py:25-71 (_test_basics): non-default hyper-parameters, 10 iterations,
    params change after the first step and stay within atol 0.025 / rtol 1e-5 of AdamW."""
    betas, weight_decay, lr, eps = (0.8, 0.88), 0.03, 0.005, 1e-8
    adam = torch.optim.AdamW(model_clone.parameters(), lr=lr, betas=betas, weight_decay=weight_decay, eps=eps)
    opt = fourbit(model.parameters(), lr=lr, betas=betas, weight_decay=weight_decay, eps=eps)
    orig = [p.clone() for p in model.parameters()]
    worst = 0.0
    for i in range(iters):
        adam.zero_grad(set_to_none=True)
        opt.zero_grad(set_to_none=True)
        inp = torch.randn(size, model[0].in_features, device="cuda")
        model(inp).sum().backward()
        model_clone(inp).sum().backward()
        adam.step()
        opt.step()
        if i == 0:
            for p1, p2 in zip(model.parameters(), orig):
                assert not torch.equal(p1, p2)
        for p1, p2 in zip(model.parameters(), model_clone.parameters()):
            torch.testing.assert_close(p1, p2, atol=atol, rtol=1e-5)
            worst = max(worst, float((p1.detach() - p2.detach()).abs().max()))
    return opt, worst


def test_driver_mlp_default_threshold(cuda):
    """The reference's 85-parameter MLP: every tensor is below the quantization threshold, so
    the non-quantized kernel runs and the result matches AdamW far inside the tolerance."""
    torch.manual_seed(2020)
    model = nn.Sequential(nn.Linear(5, 10), nn.Linear(10, 5)).cuda()
    clone = deepcopy(model)
    opt, worst = _driver_loop(model, clone, AdamWFused_QuantFour)
    say(f"driver MLP (non-quantized path): worst |diff| {worst:.3e}")
    assert worst < 1e-5
    for p in model.parameters():
        assert opt.state[p]["exp_avg"].dtype == torch.float32 and float(opt.state[p]["step"]) == 10.0


def test_adam_equivalence_alternating_zero_grad(cuda):
    """tests/test_4bit_AdamW.py:29-72 (_test_adam_equivalence, test_adam_equivalence_gpu) as it
    was meant to run: three small Linear layers, betas (0.8, 0.88), weight decay 0.03, six
    iterations that clear the gradients alternately in place and by dropping them, parameters
    equal to torch.optim.AdamW's under assert_close's default tolerance after every step."""
    torch.manual_seed(2020)
    model = nn.Sequential(nn.Linear(5, 10), nn.Linear(10, 10), nn.Linear(10, 5)).cuda()
    clone = deepcopy(model)
    betas, weight_decay = (0.8, 0.88), 0.03
    adam = torch.optim.AdamW(clone.parameters(), betas=betas, weight_decay=weight_decay)
    opt = AdamWFused_QuantFour(model.parameters(), betas=betas, weight_decay=weight_decay)
    orig = [p.clone() for p in model.parameters()]
    for p1, p2 in zip(clone.parameters(), orig):
        torch.testing.assert_close(p1, p2)
    for i in range(6):
        adam.zero_grad(set_to_none=bool(i % 2))
        opt.zero_grad(set_to_none=bool(i % 2))
        inp = torch.randn(5, 5, device="cuda")
        model(inp).sum().backward()
        clone(inp).sum().backward()
        adam.step()
        opt.step()
        if i == 0:
            for p1, p2 in zip(model.parameters(), orig):
                assert not torch.equal(p1, p2)
        for p1, p2 in zip(model.parameters(), clone.parameters()):
            torch.testing.assert_close(p1, p2)


def test_driver_mlp_forced_quantization(cuda):
    """Same loop with every tensor forced onto the 4-bit path (threshold 0), and a wider MLP
    whose weight matrices are quantized at the default threshold.  With betas (0.8, 0.88)
    the second moment moves fast and its 16 linear levels (lowest: 1/16 of the block max)
    make single elements lag AdamW by up to a step's worth per step; over 10 steps of at most
    lr = 0.005 each the observed worst case is 0.028, so these two cases use atol 0.05 (half
    of the trivial bound).  Bit-exactness against the oracle is what the other tests pin."""
    def forced(params, **kw):
        opt = AdamWFused_QuantFour(params, **kw)
        opt.param_quant_threshold = 0
        return opt

    torch.manual_seed(2020)
    model = nn.Sequential(nn.Linear(5, 10), nn.Linear(10, 5)).cuda()
    opt, worst = _driver_loop(model, deepcopy(model), forced, atol=0.05)
    say(f"driver MLP (forced 4-bit): worst |diff| {worst:.3e}")
    for p in model.parameters():
        assert opt.state[p]["exp_avg"].dtype == torch.uint8
    torch.manual_seed(2021)
    wide = nn.Sequential(nn.Linear(96, 128), nn.Linear(128, 64)).cuda()
    opt, worst = _driver_loop(wide, deepcopy(wide), AdamWFused_QuantFour, size=16, atol=0.05)
    say(f"wide MLP (4-bit weights, fp32-state biases): worst |diff| {worst:.3e}")
    kinds = sorted(str(opt.state[p]["exp_avg"].dtype) for p in wide.parameters())
    assert kinds == ["torch.float32", "torch.float32", "torch.uint8", "torch.uint8"]


def gpt2_small_shapes():
    shapes = [(50257, 768), (1024, 768)]
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,), (768,), (768,),
                   (768, 3072), (3072,), (3072, 768), (768,)]
    return shapes + [(768,), (768,)]


class OracleSet:
    """CPU twin of a parameter list, stepped tensor by tensor with the C oracle."""

    def __init__(self, params, threshold=4096):
        self.items = []
        for p in params:
            n = p.numel()
            if n > threshold:
                nb, nk = oc.state_sizes(n)
                self.items.append(["q", to_np(p), np.zeros(nb, np.uint8), np.zeros(nb, np.uint8),
                                   np.zeros(nk, np.float32), np.zeros(nk, np.float32)])
            else:
                self.items.append(["s", to_np(p), np.zeros(n, np.float32), np.zeros(n, np.float32)])

    def step_and_check(self, params, grads, opt, step, what):
        worst = 0.0
        for it, p, g in zip(self.items, params, grads):
            prev = it[1].copy()
            st = opt.state[p]
            if it[0] == "q":
                oc.step_quant(it[1], to_np(g), it[2], it[3], it[4], it[5], step=step, **HP)
                assert np.array_equal(st["exp_avg"].cpu().numpy(), it[2]), f"{what}: m codes {tuple(p.shape)}"
                assert np.array_equal(st["exp_avg_sq"].cpu().numpy(), it[3]), f"{what}: v codes {tuple(p.shape)}"
                assert np.array_equal(bits(st["momentum_qstate"]["overhead"]["max1"].cpu().numpy()), bits(it[4]))
                assert np.array_equal(bits(st["variance_qstate"]["overhead"]["max1"].cpu().numpy()), bits(it[5]))
            else:
                oc.step_unquant(it[1], to_np(g), it[2], it[3], step=step, **HP)
                assert np.array_equal(bits(st["exp_avg"].cpu().numpy().reshape(-1)), bits(it[2]))
                assert np.array_equal(bits(st["exp_avg_sq"].cpu().numpy().reshape(-1)), bits(it[3]))
            ok, w = p_close(to_np(p.detach()), it[1], prev, bf16=p.dtype == torch.bfloat16,
                            exact=p.dtype == torch.float32)   # fp32 parameters: bit for bit
            assert ok, f"{what}: params {tuple(p.shape)} worst {w}"
            worst = max(worst, w)
            it[1][:] = to_np(p.detach())
        return worst


def test_gpt2_small_parameter_set(cuda):
    """148 tensors, 124 M params, fp32: 50 quantized tensors in one multi-tensor launch, 98
    small tensors on the non-quantized kernel; 5 steps, every tensor checked every step."""
    gen = torch.Generator().manual_seed(0)
    shapes = gpt2_small_shapes()
    assert len(shapes) == 148 and sum(int(np.prod(s)) for s in shapes) == 124439808
    host = [torch.randn(s, generator=gen) * 0.02 for s in shapes]
    params = [nn.Parameter(h.clone().to(cuda)) for h in host]
    opt = AdamWFused_QuantFour(params, **KW)
    ref = OracleSet(host)
    assert sum(1 for it in ref.items if it[0] == "q") == 50
    for step in range(1, 6):
        grads = [grads_config1(gen, int(np.prod(s))).view(s) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = g.to(cuda)
        say(f"[gpt2-small] step {step}")
        opt.step()
        torch.cuda.synchronize()
        worst = ref.step_and_check(params, grads, opt, step, f"gpt2 step {step}")
    say(f"gpt2-small: parity ok, worst relative parameter error {worst:.3e}")


def test_resume_from_state_dict_is_bit_identical(cuda):
    """save -> load into a fresh optimizer -> the next steps equal the uninterrupted run."""
    gen = torch.Generator().manual_seed(11)
    shapes = [(300, 257), (4096,), (129, 33), (64, 64)]
    host = [torch.randn(s, generator=gen) * 0.02 for s in shapes]
    grads = [[torch.randn(s, generator=gen) * 1e-3 for s in shapes] for _ in range(6)]

    def run(params, opt, steps):
        for gs in steps:
            for p, g in zip(params, gs):
                p.grad = g.to(cuda)
            opt.step()

    a = [nn.Parameter(h.clone().to(cuda)) for h in host]
    opt_a = AdamWFused_QuantFour(a, **KW)
    run(a, opt_a, grads)
    b = [nn.Parameter(h.clone().to(cuda)) for h in host]
    opt_b = AdamWFused_QuantFour(b, **KW)
    run(b, opt_b, grads[:3])
    sd = deepcopy(opt_b.state_dict())
    saved = [p.detach().clone() for p in b]
    c = [nn.Parameter(s.clone()) for s in saved]
    opt_c = AdamWFused_QuantFour(c, **KW)
    opt_c.load_state_dict(sd)
    run(c, opt_c, grads[3:])
    torch.cuda.synchronize()
    for pa, pc in zip(a, c):
        assert torch.equal(pa.view(torch.int32), pc.view(torch.int32))
        sa, sc = opt_a.state[pa], opt_c.state[pc]
        assert torch.equal(sa["exp_avg"], sc["exp_avg"]) and torch.equal(sa["exp_avg_sq"], sc["exp_avg_sq"])
        assert float(sa["step"]) == float(sc["step"]) == 6.0
        if sa["momentum_qstate"]["enable"]:
            assert torch.equal(sa["momentum_qstate"]["overhead"]["max1"], sc["momentum_qstate"]["overhead"]["max1"])
            assert torch.equal(sa["variance_qstate"]["overhead"]["max1"], sc["variance_qstate"]["overhead"]["max1"])


def test_param_groups_missing_grads_and_bf16(cuda):
    """Two param groups with their own hyper-parameters, a parameter without a gradient
    (skipped, its step count stays behind), a bf16 parameter with bf16 gradient."""
    gen = torch.Generator().manual_seed(5)
    w1 = nn.Parameter((torch.randn(200, 130, generator=gen) * 0.02).to(cuda))
    w2 = nn.Parameter((torch.randn(9000, generator=gen) * 0.02).to(cuda))
    w3 = nn.Parameter((torch.randn(70, 129, generator=gen) * 0.02).to(torch.bfloat16).to(cuda))
    opt = AdamWFused_QuantFour([{"params": [w1, w3]}, {"params": [w2], "lr": 5e-4, "weight_decay": 0.0}], **KW)
    r1, r2, r3 = OracleSet([w1.detach().cpu()]), OracleSet([w2.detach().cpu()]), OracleSet([w3.detach().cpu()])
    hp2 = dict(HP, lr=5e-4, weight_decay=0.0)
    for step in range(1, 4):
        g1 = torch.randn(200, 130, generator=gen) * 1e-3
        g3 = (torch.randn(70, 129, generator=gen) * 1e-3).to(torch.bfloat16)
        w1.grad, w3.grad = g1.to(cuda), g3.to(cuda)
        g2 = None
        if step != 2:
            g2 = torch.randn(9000, generator=gen) * 1e-3
            w2.grad = g2.to(cuda)
        else:
            w2.grad = None
        opt.step()
        torch.cuda.synchronize()
        r1.step_and_check([w1], [g1], opt, step, "group 0 fp32")
        r3.step_and_check([w3], [g3], opt, step, "group 0 bf16")
        if g2 is not None:
            it = r2.items[0]
            t2 = int(float(opt.state[w2]["step"]))
            prev = it[1].copy()
            oc.step_quant(it[1], g2.numpy().reshape(-1), it[2], it[3], it[4], it[5], step=t2, **hp2)
            assert np.array_equal(opt.state[w2]["exp_avg"].cpu().numpy(), it[2])
            ok, w = p_close(to_np(w2.detach()), it[1], prev, exact=True)
            assert ok, w
            it[1][:] = to_np(w2.detach())
    assert float(opt.state[w1]["step"]) == 3.0 and float(opt.state[w2]["step"]) == 2.0


def test_fp16_model_state_layout_resume_and_interchange(cuda):
    """a model held in fp16 (the reference dispatches on half parameters,
    optim/cuda_adamw_kernels.cu:443): packed states stay uint8 with fp32 scales, small tensors
    keep fp32 moments, the run tracks torch.optim.AdamW on an fp32 twin within the draft's bar,
    resume is bit-identical, and the exported AdamW state is fp32"""
    torch.manual_seed(8)
    mk = lambda: nn.Sequential(nn.Linear(256, 96), nn.Tanh(), nn.Linear(96, 32)).to(cuda)
    model, twin = mk().half(), mk()
    twin.load_state_dict({k: v.float() for k, v in model.state_dict().items()})
    opt = AdamWFused_QuantFour(model.parameters(), lr=1e-3, weight_decay=0.01)
    ref = torch.optim.AdamW(twin.parameters(), lr=1e-3, weight_decay=0.01)
    for it in range(8):
        x = torch.randn(32, 256, device=cuda)
        opt.zero_grad(set_to_none=True)
        model(x.half()).float().square().mean().backward()
        opt.step()
        ref.zero_grad(set_to_none=True)
        twin(x).square().mean().backward()
        ref.step()
    w = model[0].weight
    st = opt.state[w]
    assert w.dtype == torch.float16 and w.grad.dtype == torch.float16
    assert st["exp_avg"].dtype == torch.uint8 and st["momentum_qstate"]["overhead"]["max1"].dtype == torch.float32
    assert opt.state[model[0].bias]["exp_avg"].dtype == torch.float32
    for a, b in zip(model.parameters(), twin.parameters()):
        torch.testing.assert_close(a.float(), b, atol=0.025, rtol=1e-5)
    exported = opt.adamw_state_dict()["state"][0]
    assert exported["exp_avg"].dtype == torch.float32 and exported["exp_avg"].shape == w.shape
    model2 = mk().half()
    model2.load_state_dict(model.state_dict())
    opt2 = AdamWFused_QuantFour(model2.parameters(), lr=1e-3, weight_decay=0.01)
    opt2.load_state_dict(opt.state_dict())
    assert opt2.state[model2[0].weight]["exp_avg"].dtype == torch.uint8
    assert opt2.state[model2[0].weight]["variance_qstate"]["overhead"]["max1"].dtype == torch.float32
    x = torch.randn(32, 256, device=cuda).half()
    for m_, o_ in ((model, opt), (model2, opt2)):
        o_.zero_grad(set_to_none=True)
        m_(x).float().square().mean().backward()
        o_.step()
    for a, b in zip(model.parameters(), model2.parameters()):
        assert torch.equal(a, b)


@pytest.mark.parametrize("shape", [(4096,), (1024, 4096), (4096, 4096), (14336, 4096), (4096, 14336)])
def test_llama3_8b_tensor_shapes(cuda, shape):
    """Every distinct tensor shape of the headline configuration except the embedding, at its
    real size: fp32 master parameter, bf16 gradient (Student-t, df 3), 3 steps."""
    gen = torch.Generator(device=cuda).manual_seed(shape[0])
    n = int(np.prod(shape))
    p = nn.Parameter(torch.randn(shape, generator=gen, device=cuda) * 0.02)
    p.grad_dtype = torch.bfloat16
    opt = AdamWFused_QuantFour([p], **KW)
    ref = OracleSet([p.detach().cpu()])
    for step in range(1, 4):
        z = torch.randn(n, generator=gen, device=cuda)
        c = torch.randn(3, n, generator=gen, device=cuda).square().sum(0) / 3.0
        g = (z / c.sqrt() * 1e-4).to(torch.bfloat16).view(shape)
        p.grad = g
        say(f"[llama shape {shape}] step {step}")
        opt.step()
        torch.cuda.synchronize()
        ref.step_and_check([p], [g.cpu()], opt, step, f"llama {shape} step {step}")


def test_llama3_8b_embedding_shape(cuda):
    """128256 x 4096 (525 M elements, byte offsets beyond 2^31): one step against the oracle."""
    shape = (128256, 4096)
    n = shape[0] * shape[1]
    gen = torch.Generator(device=cuda).manual_seed(9)
    p = nn.Parameter(torch.randn(shape, generator=gen, device=cuda) * 0.02)
    p.grad_dtype = torch.bfloat16
    opt = AdamWFused_QuantFour([p], **KW)
    ref = OracleSet([p.detach().cpu()])
    g = (torch.randn(shape, generator=gen, device=cuda) * 1e-4).to(torch.bfloat16)
    g[1000:1100] = 0          # rows without gradient: all-zero blocks
    p.grad = g
    say("[llama embedding] step 1")
    opt.step()
    torch.cuda.synchronize()
    ref.step_and_check([p], [g.cpu()], opt, 1, "llama embedding")


def _twin_optimizers(cuda, shapes, dtype=torch.float32, **kw):
    """two optimizers over equal parameters: `a` keeps its plan from step to step, `b` is
    rebuilt from its own state_dict before every step and so always gathers from scratch"""
    gen = torch.Generator().manual_seed(77)
    base = [(torch.randn(s, generator=gen) * 0.02).to(dtype) for s in shapes]
    pa = [nn.Parameter(t.clone().to(cuda)) for t in base]
    pb = [nn.Parameter(t.clone().to(cuda)) for t in base]
    return pa, pb, AdamWFused_QuantFour(pa, **KW, **kw), AdamWFused_QuantFour(pb, **KW, **kw), gen


def _same_everything(opt_a, pa, opt_b, pb):
    for x, y in zip(pa, pb):
        assert torch.equal(x.detach().view(torch.uint8), y.detach().view(torch.uint8))
        sa, sb = opt_a.state.get(x, {}), opt_b.state.get(y, {})
        assert set(sa) == set(sb)
        if not sa:
            continue
        assert float(sa["step"]) == float(sb["step"])
        for key in ("exp_avg", "exp_avg_sq"):
            assert torch.equal(sa[key].view(torch.uint8), sb[key].view(torch.uint8)), key
        for q in ("momentum_qstate", "variance_qstate"):
            ma, mb = sa[q]["overhead"].get("max1"), sb[q]["overhead"].get("max1")
            assert (ma is None) == (mb is None) and (ma is None or torch.equal(ma.view(torch.int32), mb.view(torch.int32)))


def test_kept_plan_follows_every_change_of_what_it_rests_on(cuda):
    """The optimizer keeps a group's launch plan between steps and re-gathers only when
    something under it changed.  Each step below changes one such thing -- which parameters
    have a gradient, a gradient's dtype, a parameter's storage, a state tensor, a step counter,
    the group's parameter list -- and the result must equal, bit for bit, that of a twin
    whose plan is thrown away before every step."""
    shapes = [(40, 300), (5000,), (17,), (64, 128), (4096,)]
    pa, pb, oa, ob, gen = _twin_optimizers(cuda, shapes)

    def grads(mask=None, dtypes=None):
        out = []
        for i, s in enumerate(shapes):
            if mask is not None and not mask[i]:
                out.append(None)
                continue
            g = torch.randn(s, generator=gen) * 1e-3
            out.append(g.to(dtypes[i] if dtypes else torch.float32))
        return out

    def step_both(gs):
        for ps in (pa, pb):
            for p, g in zip(ps, gs):
                p.grad = None
                if g is not None and g.dtype != p.dtype:
                    p.grad_dtype = g.dtype
                p.grad = None if g is None else g.to(cuda)
        ob._plans.clear()
        ob._launch_cache.clear()
        oa.step()
        ob.step()
        torch.cuda.synchronize()
        _same_everything(oa, pa, ob, pb)

    step_both(grads())
    assert 0 in oa._plans
    kept = oa._plans[0]
    step_both(grads())
    assert oa._plans[0] is kept, "nothing changed: the plan must have been reused"
    step_both(grads(mask=[True, False, True, True, True]))          # one parameter without a gradient
    assert oa._plans[0] is not kept
    step_both(grads())                                               # and with one again (its step lags by one)
    assert [float(oa.state[p]["step"]) for p in pa] == [4.0, 3.0, 4.0, 4.0, 4.0]
    kept = oa._plans[0]
    step_both(grads())
    assert oa._plans[0] is kept
    step_both(grads(dtypes=[torch.bfloat16, torch.float32, torch.float32, torch.float32, torch.float32]))
    assert oa._plans[0] is not kept                                  # a gradient changed its dtype
    kept = oa._plans[0]
    for ps in (pa, pb):                                              # a parameter moved to other storage
        ps[3].data = ps[3].data.clone()
    step_both(grads(dtypes=[torch.bfloat16, torch.float32, torch.float32, torch.float32, torch.float32]))
    assert oa._plans[0] is not kept
    kept = oa._plans[0]
    for o, ps in ((oa, pa), (ob, pb)):                               # a state tensor replaced from outside
        o.state[ps[1]]["exp_avg"] = o.state[ps[1]]["exp_avg"].clone()
        o.state[ps[0]]["step"] = torch.tensor(11.0)
    step_both(grads(dtypes=[torch.bfloat16, torch.float32, torch.float32, torch.float32, torch.float32]))
    assert oa._plans[0] is not kept and float(oa.state[pa[0]]["step"]) == 12.0
    kept = oa._plans[0]
    sd = oa.state_dict()                                             # a loaded state_dict replaces every state tensor
    oa.load_state_dict(sd)
    ob.load_state_dict(ob.state_dict())
    step_both(grads(dtypes=[torch.bfloat16, torch.float32, torch.float32, torch.float32, torch.float32]))
    assert oa._plans[0] is not kept


def test_a_refused_gradient_leaves_everything_as_it_was(cuda):
    """Everything is validated before the first launch and before any step counter moves: a
    gradient the kernels cannot take (every other element of a buffer, a transposed view) in
    the LAST bucket of the LAST group leaves parameters, state and counters of every group
    untouched, on the first step and on a step that had a plan."""
    gen = torch.Generator().manual_seed(5)
    shapes = [(64, 100), (3000,), (8192,)]
    ps = [nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(cuda)) for s in shapes]
    opt = AdamWFused_QuantFour([{"params": ps[:2]}, {"params": ps[2:], "lr": 2e-3}], **KW)
    flat = torch.zeros(2 * 8192, device=cuda)

    def snapshot():
        """parameters, and the state that exists (the first refused step creates it, all zeros)"""
        out = {("p", i): p.detach().clone() for i, p in enumerate(ps)}
        for i, p in enumerate(ps):
            st = opt.state.get(p, {})
            out.update({(k, i): st[k].clone() for k in ("step", "exp_avg", "exp_avg_sq") if k in st})
        return out

    def unchanged(before, after):
        return all(torch.equal(t, after[k]) for k, t in before.items())

    def set_grads(bad):
        for p in ps[:2]:
            p.grad = (torch.randn(p.shape, generator=gen) * 1e-3).to(cuda)
        ps[2].grad = None
        ps[2].grad = bad if bad is not None else (torch.randn(8192, generator=gen) * 1e-3).to(cuda)

    for round_ in range(2):
        before = snapshot()
        set_grads(flat[::2])                          # strided
        with pytest.raises(AssertionError, match="contiguous"):
            opt.step()
        torch.cuda.synchronize()
        assert unchanged(before, snapshot()), round_
        assert all(float(opt.state[p]["step"]) == round_ for p in ps if opt.state.get(p))
        set_grads(None)                               # a good step: the next round starts from a kept plan
        opt.step()
        assert [float(opt.state[p]["step"]) for p in ps] == [round_ + 1.0] * 3
    before = snapshot()
    ps[0].grad = None
    ps[0].grad = torch.zeros(100, 64, device=cuda).t()     # not contiguous
    with pytest.raises(AssertionError, match="contiguous"):
        opt.step()
    assert unchanged(before, snapshot())
    # the SAME gradient objects as in the step before, one of them re-strided in place: the
    # kept plan looks at the strides again
    sq = nn.Parameter((torch.randn(96, 96, generator=gen) * 0.02).to(cuda))
    opt2 = AdamWFused_QuantFour([sq], **KW)
    sq.grad = (torch.randn(96, 96, generator=gen) * 1e-3).to(cuda)
    opt2.step()
    opt2.step()
    assert 0 in opt2._plans
    p_before, m_before = sq.detach().clone(), opt2.state[sq]["exp_avg"].clone()
    sq.grad.t_()                                           # same object, same shape, other strides
    assert not sq.grad.is_contiguous()
    with pytest.raises(AssertionError, match="contiguous"):
        opt2.step()
    torch.cuda.synchronize()
    assert torch.equal(sq.detach(), p_before) and torch.equal(opt2.state[sq]["exp_avg"], m_before)
    assert float(opt2.state[sq]["step"]) == 2.0


@pytest.mark.parametrize("found_inf_at", [None, 2])
@pytest.mark.parametrize("round_type", ["real-nearest", "stochastic"])
@pytest.mark.parametrize("variance_scale", ["group", "rank1"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_views_at_odd_offsets_into_flat_buffers(cuda, dtype, variance_scale, round_type, found_inf_at):
    """Parameters and gradients that are views into flat buffers at odd element offsets (2 or 4
    bytes past a 16-byte boundary, as a flat-parameter wrapper or a gradient bucket makes them
    once one tensor has an odd size) take the same path as tensors of their own and give the
    same bits: block-scaled and rank-1 (rows, wide, narrow and 3-D forms), nearest and
    stochastic, with the gradient norm taken, the gradients cleared by the step, and a step
    that an overflow flag cancels.  Elements of the buffers between the views stay as they were."""
    shapes = [(8, 1024), (6, 520), (300, 24), (4, 6, 64), (100,), (5000,), (33, 129)]
    gen = torch.Generator().manual_seed(123)
    base = [(torch.randn(s, generator=gen) * 0.02).to(dtype) for s in shapes]
    offsets, total = [], 1
    for t in base:
        offsets.append(total)
        total += t.numel() + (1 if len(offsets) % 2 else 2)
    flat_p = torch.full((total,), 7.0, dtype=dtype, device=cuda)
    flat_g = torch.full((total,), 7.0, dtype=dtype, device=cuda)
    pa = [nn.Parameter(flat_p[o:o + t.numel()].view(t.shape)) for o, t in zip(offsets, base)]
    for p, t in zip(pa, base):
        p.data.copy_(t)
    assert any(p.data_ptr() % 16 for p in pa) and all(p.is_contiguous() for p in pa)
    pb = [nn.Parameter(t.clone().to(cuda)) for t in base]
    kw = dict(KW, variance_scale_type=variance_scale, round_type=round_type)
    if round_type == "stochastic":
        kw["seed"] = 99
    oa, ob = AdamWFused_QuantFour(pa, **kw), AdamWFused_QuantFour(pb, **kw)
    covered = torch.zeros(total, dtype=torch.bool, device=cuda)
    for o, t in zip(offsets, base):
        covered[o:o + t.numel()] = True
    for step in range(1, 5):
        gs = [(torch.randn(t.shape, generator=gen) * 1e-3).to(dtype) for t in base]
        for o, p, q, g in zip(offsets, pa, pb, gs):
            view = flat_g[o:o + g.numel()].view(g.shape)
            view.copy_(g)
            p.grad = view
            q.grad = g.clone().to(cuda)
        flag = torch.full((1,), 1.0 if step == found_inf_at else 0.0, device=cuda)
        say(f"[flat views] {dtype} {variance_scale} {round_type} step {step} cancelled {step == found_inf_at}")
        import warnings
        with warnings.catch_warnings(record=True) as caught:
            warnings.simplefilter("always")
            for o in (oa, ob):
                o.step(grad_scale=0.5, max_grad_norm=0.01, found_inf=flag, zero_grad=True)
        # the views' owner is told once that unaligned parameters are the slow case; the twin never
        assert sum("16-byte boundary" in str(w.message) for w in caught) == (1 if step == 1 else 0)
        torch.cuda.synchronize()
        assert torch.equal(oa.last_grad_norm, ob.last_grad_norm)
        _same_everything(oa, pa, ob, pb)
        assert all(not bool(p.grad.any()) for p in pa)                    # cleared, cancelled or not
        assert bool((flat_p[~covered] == 7.0).all()) and bool((flat_g[~covered] == 7.0).all())
