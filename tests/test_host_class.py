"""Host-side behaviour of AdamWFused_QuantFour that needs no GPU: constructor validation
(optim/fused_quantfour.py:38-47), state layout (:61-70, :110-120, :180-204), routing by
size (optim/adamw_fourbit_triton.py:131-134), error paths, state_dict handling."""
import pytest
import torch

import quantfour_adamw_cuda_amd as q4
from quantfour_adamw_cuda_amd import AdamWFused_QuantFour, enable_param_quantization


def params(*shapes):
    return [torch.nn.Parameter(torch.randn(s)) for s in shapes]


@pytest.mark.parametrize("kwargs,msg", [
    (dict(lr=0.0), "Invalid learning rate"), (dict(lr=-1e-3), "Invalid learning rate"),
    (dict(eps=0.0), "Invalid eps value"), (dict(betas=(1.0, 0.999)), r"Invalid Beta\[0\]"),
    (dict(betas=(0.0, 0.999)), r"Invalid Beta\[0\]"), (dict(betas=(0.9, 1.0)), r"Invalid Beta\[1\]"),
    (dict(betas=(0.9, -0.1)), r"Invalid Beta\[1\]"), (dict(weight_decay=-0.1), "Invalid weight_decay value")])
def test_constructor_validation(kwargs, msg):
    with pytest.raises(ValueError, match=msg):
        AdamWFused_QuantFour(params((4, 4)), **kwargs)


def test_constructor_defaults_and_api():
    opt = AdamWFused_QuantFour(params((4, 4)))
    g = opt.param_groups[0]
    assert g["lr"] == 1e-3 and g["betas"] == (0.9, 0.999) and g["eps"] == 1e-8
    assert g["weight_decay"] == 1e-2 and g["fused"] is False
    assert opt.param_quant_threshold == 4096
    assert isinstance(opt, torch.optim.Optimizer)
    AdamWFused_QuantFour(params((4, 4)), 3e-4, (0.8, 0.88), 1e-6, 0.03, fused=True)   # positional order
    with pytest.raises(TypeError):
        AdamWFused_QuantFour(params((4, 4)), 3e-4, (0.8, 0.88), 1e-6, 0.03, True)      # fused is keyword-only


def test_enable_param_quantization_rule():
    p = torch.zeros(4096)
    assert enable_param_quantization(p, 4096) is False       # numel <= threshold: not quantized
    assert enable_param_quantization(torch.zeros(4097), 4096) is True
    assert enable_param_quantization(p, 0) is True            # a zero threshold disables the rule
    assert enable_param_quantization(torch.zeros(1), None) is True


def test_state_layout():
    big, small, odd = params((70, 129), (64, 64), (4097,))
    opt = AdamWFused_QuantFour([big, small, odd])
    for p in (big, small, odd):
        opt._init_state(p)
    sb, ss, so = opt.state[big], opt.state[small], opt.state[odd]
    for st in (sb, ss, so):
        assert set(st) == {"step", "exp_avg", "exp_avg_sq", "momentum_qstate", "variance_qstate"}
        assert st["step"].dtype == torch.float32 and st["step"].dim() == 0 and float(st["step"]) == 0.0
        for q in ("momentum_qstate", "variance_qstate"):
            assert set(st[q]) == {"enable", "overhead", "qmap"} and st[q]["qmap"] is None
    n = 70 * 129
    assert sb["momentum_qstate"]["enable"] and sb["variance_qstate"]["enable"]
    assert sb["exp_avg"].dtype == torch.uint8 and sb["exp_avg"].shape == ((n + 1) // 2,)
    assert sb["exp_avg_sq"].dtype == torch.uint8 and sb["exp_avg_sq"].shape == ((n + 1) // 2,)
    for q in ("momentum_qstate", "variance_qstate"):
        max1 = sb[q]["overhead"]["max1"]
        assert max1.dtype == torch.float32 and max1.shape == ((n + 127) // 128,) and not max1.any()
    assert not sb["exp_avg"].any() and not sb["exp_avg_sq"].any()
    assert so["exp_avg"].shape == (2049,) and so["momentum_qstate"]["overhead"]["max1"].shape == (33,)
    # 64*64 = 4096 elements: not quantized, fp32 moments shaped like the parameter
    assert not ss["momentum_qstate"]["enable"] and ss["momentum_qstate"]["overhead"] == {}
    assert ss["exp_avg"].dtype == torch.float32 and ss["exp_avg"].shape == (64, 64)
    assert q4.state_sizes(n) == ((n + 1) // 2, (n + 127) // 128)


def test_threshold_override_routes_small_tensors_to_the_quantized_path():
    (p,) = params((100,))
    opt = AdamWFused_QuantFour([p])
    opt.param_quant_threshold = 0
    opt._init_state(p)
    assert opt.state[p]["momentum_qstate"]["enable"] and opt.state[p]["exp_avg"].dtype == torch.uint8


def test_step_refuses_cpu_parameters_and_sparse_grads():
    (p,) = params((8, 8))
    opt = AdamWFused_QuantFour([p])
    p.grad = torch.zeros_like(p)
    with pytest.raises(AssertionError, match="param must be on cuda"):
        opt.step()
    (e,) = params((10, 4))
    opt2 = AdamWFused_QuantFour([e])
    e.grad = torch.sparse_coo_tensor(torch.tensor([[1], [2]]), torch.tensor([1.0]), (10, 4))
    with pytest.raises(RuntimeError, match="does not support sparse gradients"):
        opt2.step()


def test_step_without_grads_is_a_noop_and_closure_runs():
    (p,) = params((8, 8))
    opt = AdamWFused_QuantFour([p])
    calls = []

    def closure():
        calls.append(torch.is_grad_enabled())
        return torch.tensor(3.0)

    assert float(opt.step(closure)) == 3.0 and calls == [True]
    assert len(opt.state) == 0


def test_step_fails_loudly_without_the_library(monkeypatch):
    from quantfour_adamw_cuda_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libq4adamw.so")
    (p,) = params((8, 8))
    p.grad = torch.zeros_like(p)
    with pytest.raises(RuntimeError, match="is missing"):
        AdamWFused_QuantFour([p]).step()


def test_state_dict_round_trip_keeps_dtypes():
    big, small = [torch.nn.Parameter(torch.randn(s).to(torch.bfloat16)) for s in ((50, 130), (10, 10))]
    opt = AdamWFused_QuantFour([big, small], lr=2e-3)
    for p in (big, small):
        opt._init_state(p)
    opt.state[big]["exp_avg"].fill_(0x5A)
    opt.state[big]["momentum_qstate"]["overhead"]["max1"].fill_(1.0 + 2.0 ** -20)   # not a bf16 value
    opt.state[small]["exp_avg_sq"].fill_(1.0 + 2.0 ** -20)
    opt.state[big]["step"] += 7
    sd = opt.state_dict()
    assert sd["param_groups"][0]["lr"] == 2e-3
    big2, small2 = [torch.nn.Parameter(p.detach().clone()) for p in (big, small)]
    opt2 = AdamWFused_QuantFour([big2, small2])
    opt2.load_state_dict(sd)
    s_big, s_small = opt2.state[big2], opt2.state[small2]
    assert s_big["exp_avg"].dtype == torch.uint8 and bool((s_big["exp_avg"] == 0x5A).all())
    max1 = s_big["momentum_qstate"]["overhead"]["max1"]
    assert max1.dtype == torch.float32 and bool((max1 == 1.0 + 2.0 ** -20).all())
    assert s_small["exp_avg_sq"].dtype == torch.float32 and bool((s_small["exp_avg_sq"] == 1.0 + 2.0 ** -20).all())
    assert float(s_big["step"]) == 7.0 and opt2.param_groups[0]["lr"] == 2e-3
    assert s_big["momentum_qstate"]["enable"] is True and s_small["momentum_qstate"]["enable"] is False


def test_loaded_state_shares_nothing_with_its_source():
    """load_state_dict(opt.state_dict()) must not leave the two optimizers advancing one step
    counter or writing one moment buffer"""
    (big,) = params((50, 130))
    opt = AdamWFused_QuantFour([big])
    opt._init_state(big)
    big2 = torch.nn.Parameter(big.detach().clone())
    opt2 = AdamWFused_QuantFour([big2])
    opt2.load_state_dict(opt.state_dict())
    a, b = opt.state[big], opt2.state[big2]
    assert a["step"].data_ptr() != b["step"].data_ptr()
    assert a["exp_avg"].data_ptr() != b["exp_avg"].data_ptr()
    assert (a["momentum_qstate"]["overhead"]["max1"].data_ptr()
            != b["momentum_qstate"]["overhead"]["max1"].data_ptr())


def test_step_counters_share_one_buffer_and_follow_replacements():
    """the step counters of a group are views of one host buffer (one addition per step);
    a counter replaced from outside is picked up by identity and keeps its own value"""
    ps = [torch.nn.Parameter(torch.zeros(n)) for n in (5000, 3, 8192)]
    opt = AdamWFused_QuantFour(ps)
    for p in ps:
        opt._init_state(p)
    steps = [opt.state[p]["step"] for p in ps]
    assert opt._advance_steps(0, ps, steps) == [1.0, 1.0, 1.0]
    assert all(opt.state[p]["step"] is s for p, s in zip(ps, steps))
    buf = opt._step_buffers[0][0]
    assert all(s.dim() == 0 and s.dtype == torch.float32 and s.untyped_storage().data_ptr() ==
               buf.untyped_storage().data_ptr() for s in steps)
    assert opt._advance_steps(0, ps, steps) == [2.0, 2.0, 2.0] and opt._step_buffers[0][0] is buf
    opt.state[ps[1]]["step"] = torch.tensor(7.0)
    steps = [opt.state[p]["step"] for p in ps]
    assert opt._advance_steps(0, ps, steps) == [3.0, 8.0, 3.0]
    assert [float(opt.state[p]["step"]) for p in ps] == [3.0, 8.0, 3.0]
    # a subset of the parameters (the others had no gradient this time)
    steps = [opt.state[p]["step"] for p in ps[:2]]
    assert opt._advance_steps(0, ps[:2], steps) == [4.0, 9.0]
    assert [float(opt.state[p]["step"]) for p in ps] == [4.0, 9.0, 3.0]
    sd = opt.state_dict()
    assert [float(sd["state"][i]["step"]) for i in range(3)] == [4.0, 9.0, 3.0]


def test_rank1_state_layout_and_round_trip():
    """variance_scale_type="rank1": matrices keep row and column maxima (the draft's max_dims,
    keepdim shapes) instead of block scales, whatever their sizes; vectors and matrices of one
    column keep block scales; a state_dict round trip keeps layout, values and dtypes"""
    wide, narrow, vec = [torch.nn.Parameter(torch.randn(s).to(torch.bfloat16))
                         for s in ((12, 1024), (8192, 1), (8192,))]
    odd = torch.nn.Parameter(torch.randn(1024, 101).to(torch.bfloat16))
    opt = AdamWFused_QuantFour([wide, narrow, vec, odd], variance_scale_type="rank1")
    for p in (wide, narrow, vec, odd):
        opt._init_state(p)
    oo = opt.state[odd]["variance_qstate"]["overhead"]
    assert oo["max1"] is None and [tuple(t.shape) for t in oo["max_dims"]] == [(1024, 1), (1, 101)]
    ov = opt.state[wide]["variance_qstate"]["overhead"]
    assert ov["max1"] is None and ov["dim"] == 2
    assert [tuple(t.shape) for t in ov["max_dims"]] == [(12, 1), (1, 1024)]
    assert [tuple(t.shape) for t in ov["scratch_dims"]] == [(12, 1), (1, 1024)]
    assert all(t.dtype == torch.float32 and not t.any() for t in ov["max_dims"] + ov["scratch_dims"])
    assert opt.state[wide]["momentum_qstate"]["overhead"]["max1"].shape == (12 * 1024 // 128,)
    for p in (narrow, vec):
        o = opt.state[p]["variance_qstate"]["overhead"]
        assert "max_dims" not in o and o["max1"].shape == (p.numel() // 128,)
    ov["max_dims"][0].fill_(1.0 + 2.0 ** -20)            # not a bf16 value
    ov["max_dims"][1].fill_(3.0)
    ov["scratch_dims"][1].fill_(9.0)                     # scratch is not state: it restarts from zero
    wide2, narrow2, vec2, odd2 = [torch.nn.Parameter(p.detach().clone()) for p in (wide, narrow, vec, odd)]
    opt2 = AdamWFused_QuantFour([wide2, narrow2, vec2, odd2])  # the layout follows the checkpoint
    opt2.load_state_dict(opt.state_dict())
    o2 = opt2.state[wide2]["variance_qstate"]["overhead"]
    assert o2["max_dims"][0].dtype == torch.float32 and bool((o2["max_dims"][0] == 1.0 + 2.0 ** -20).all())
    assert bool((o2["max_dims"][1] == 3.0).all()) and tuple(o2["max_dims"][1].shape) == (1, 1024)
    assert all(not t.any() for t in o2["scratch_dims"])
    assert o2["max_dims"][0].data_ptr() != ov["max_dims"][0].data_ptr()
    with pytest.raises(ValueError, match="variance_scale_type"):
        AdamWFused_QuantFour([wide], variance_scale_type="rank2")


def test_rank1_state_layout_of_tensors_with_more_than_two_dimensions():
    """one statistic per dimension in keepdim shape (the draft's max_dims), plus the derived
    scale of every flattened row; a state_dict round trip restores statistics and recomputes
    the row scales; five dimensions, or a last dimension of 1, keep block scales"""
    t3, t4, t5, odd = [torch.nn.Parameter(torch.randn(s)) for s in ((4, 6, 256), (3, 2, 5, 160), (2, 2, 2, 2, 512), (80, 80, 1))]
    last_odd = torch.nn.Parameter(torch.randn(8, 8, 100))
    o_odd = AdamWFused_QuantFour([last_odd], variance_scale_type="rank1")
    o_odd._init_state(last_odd)
    assert [tuple(t.shape) for t in o_odd.state[last_odd]["variance_qstate"]["overhead"]["max_dims"]] == [(8, 1, 1), (1, 8, 1), (1, 1, 100)]
    opt = AdamWFused_QuantFour([t3, t4, t5, odd], variance_scale_type="rank1")
    for p in (t3, t4, t5, odd):
        opt._init_state(p)
    o3, o4 = (opt.state[p]["variance_qstate"]["overhead"] for p in (t3, t4))
    assert o3["dim"] == 3 and [tuple(t.shape) for t in o3["max_dims"]] == [(4, 1, 1), (1, 6, 1), (1, 1, 256)]
    assert o4["dim"] == 4 and [tuple(t.shape) for t in o4["scratch_dims"]] == [(3, 1, 1, 1), (1, 2, 1, 1), (1, 1, 5, 1), (1, 1, 1, 160)]
    assert o3["row_scale"].shape == (24,) and o4["row_scale"].shape == (30,) and o4["row_scratch"].shape == (30,)
    for p in (t5, odd):
        assert "max_dims" not in opt.state[p]["variance_qstate"]["overhead"]
    o3["max_dims"][0].copy_(torch.tensor([4.0, 1.0, 3.0, 2.0]).view(4, 1, 1))
    o3["max_dims"][1].fill_(2.5)
    o3["max_dims"][2].fill_(9.0)
    opt2 = AdamWFused_QuantFour([torch.nn.Parameter(p.detach().clone()) for p in (t3, t4, t5, odd)],
                                variance_scale_type="rank1")
    opt2.load_state_dict(opt.state_dict())
    n3 = opt2.state[opt2.param_groups[0]["params"][0]]["variance_qstate"]["overhead"]
    assert all(torch.equal(a, b) and a.data_ptr() != b.data_ptr() for a, b in zip(n3["max_dims"], o3["max_dims"]))
    want = torch.tensor([2.5, 1.0, 2.5, 2.0]).repeat_interleave(6)      # min(statistic of dim 0, 2.5) per row
    assert torch.equal(n3["row_scale"], want) and not n3["row_scratch"].any()


def test_round_type_and_seed_travel_in_the_param_groups():
    (p,) = params((64, 130))
    with pytest.raises(ValueError, match="round_type"):
        AdamWFused_QuantFour([p], round_type="nearest-even")
    both = AdamWFused_QuantFour([p], round_type="stochastic", variance_scale_type="rank1", seed=3)
    assert both.variance_scale_type == "rank1" and both.param_groups[0]["round_type"] == "stochastic"
    assert AdamWFused_QuantFour([p]).param_groups[0]["round_type"] == "real-nearest"
    torch.manual_seed(5)
    a = AdamWFused_QuantFour([p], round_type="stochastic")
    torch.manual_seed(5)
    b = AdamWFused_QuantFour([p], round_type="stochastic")
    seed = a.param_groups[0]["seed"]
    assert isinstance(seed, int) and 0 <= seed < 1 << 31 and seed == b.param_groups[0]["seed"]
    assert AdamWFused_QuantFour([p], round_type="stochastic", seed=77).param_groups[0]["seed"] == 77
    # a resumed optimizer continues with the checkpoint's seed and rounding
    c = AdamWFused_QuantFour([torch.nn.Parameter(p.detach().clone())])
    c.load_state_dict(a.state_dict())
    assert c.param_groups[0]["seed"] == seed and c.param_groups[0]["round_type"] == "stochastic"
    q0, q1 = params((8, 8), (9, 9))
    d = AdamWFused_QuantFour([{"params": [q0]}, {"params": [q1]}])
    assert d._param_position(q0) == 0 and d._param_position(q1) == 1


def test_capturable_option():
    (p,) = params((64, 130))
    assert AdamWFused_QuantFour([p]).param_groups[0]["capturable"] is False
    opt = AdamWFused_QuantFour([p], capturable=True)
    assert opt.param_groups[0]["capturable"] is True and opt.state_dict()["param_groups"][0]["capturable"] is True


def test_setstate_backfills():
    (p,) = params((4, 4))
    opt = AdamWFused_QuantFour([p])
    opt._init_state(p)
    state = opt.__getstate__()
    state["param_groups"][0].pop("fused")
    state["state"][p]["step"] = 3          # a plain number, as older checkpoints hold it
    opt.__setstate__(state)
    assert opt.param_groups[0]["fused"] is None
    assert torch.is_tensor(opt.state[p]["step"]) and float(opt.state[p]["step"]) == 3.0


def test_pickle_and_deepcopy_keep_the_settings():
    import copy
    import pickle
    ps = params((64, 136), (8,))
    opt = AdamWFused_QuantFour(ps, lr=2e-3, variance_scale_type="rank1", round_type="stochastic", seed=5)
    for p in ps:
        opt._init_state(p)
    opt._launch_cache["x"] = object()        # caches hold ctypes arrays: they must not travel
    for twin in (pickle.loads(pickle.dumps(opt)), copy.deepcopy(opt)):
        assert twin.variance_scale_type == "rank1" and twin.param_quant_threshold == 4096
        g = twin.param_groups[0]
        assert g["lr"] == 2e-3 and g["round_type"] == "stochastic" and g["seed"] == 5
        assert twin._launch_cache == {} and twin._device_steps == {} and twin.kernel_timing is None
        big = twin.param_groups[0]["params"][0]
        assert "max_dims" in twin.state[big]["variance_qstate"]["overhead"]
        assert twin.state[big]["exp_avg"].dtype == torch.uint8


def test_functional_wrappers_validate():
    p = torch.zeros(300)
    with pytest.raises(AssertionError, match="param must be on cuda"):
        q4.fused_4bit(p, p, torch.zeros(150, dtype=torch.uint8), torch.zeros(150, dtype=torch.uint8),
                      torch.zeros(3), torch.zeros(3), 0.9, 0.999, 1e-3, 0.01, 1e-8, 1)
    q4.fused_4bit_multi([], [], [], [], [], [], 0.9, 0.999, 1e-3, 0.01, 1e-8, 1)       # nothing to do
    q4.fused_single_tensor_multi([], [], [], [], 0.9, 0.999, 1e-3, 0.01, 1e-8, 1)


def test_fp64_parameters_and_gradients_are_refused():
    """The reference's launchers dispatch on double as well (AT_DISPATCH_FLOATING_TYPES_AND_HALF,
    optim/cuda_adamw_kernels.cu:147, :443); this build's kernels take fp32, bf16 and fp16
    storage (the arithmetic is fp32 either way) and say so before anything is launched."""
    from quantfour_adamw_cuda_amd import quantfour_hip as qh
    with pytest.raises(TypeError, match="param must be float32, bfloat16 or float16, got torch.float64"):
        qh._tag(torch.zeros(4, dtype=torch.float64), "param")
    with pytest.raises(TypeError, match="grad must be float32, bfloat16 or float16, got torch.float64"):
        qh._tag(torch.zeros(4, dtype=torch.float64), "grad")
    assert [qh._tag(torch.zeros(1, dtype=d), "param") for d in (torch.float32, torch.bfloat16, torch.float16)] == [0, 1, 2]
