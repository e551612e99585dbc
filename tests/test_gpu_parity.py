"""GPU parity tests: the HIP step, called through the C ABI, against the CPU oracle
on identical seeded inputs.  Packed codes and block scales must be bit-exact;
parameters within 1e-6 relative (fp32) or one bf16 ulp (bf16 parameters)."""
import numpy as np
import pytest
import torch

import quantfour_adamw_cuda_amd as q4
from oracle import q4_oracle as oc
from tests.q4_testlib import (HP, HP_DRIVER, DeviceTensor, OracleTensor, assert_state_equal, bits,
                              grads_config1, grads_config3, grads_student_t, p_close, to_np,
                              BASELINE_ATOL, STRICT_LOG, strict_atol_since)

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)


def run_steps(p0, grad_fn, steps, device, hp=HP, g_dtype=torch.float32, what=""):
    """Steps one tensor on the device and in the oracle; checks after every step.  fp32
    parameters come from the exact form of the update and are compared bit for bit, the two
    sides never re-based on each other: the last step's equality is the cumulative bound.
    16-bit parameters (folded form, one ulp per step) continue from the device's values."""
    dev = DeviceTensor(p0, device)
    ref = OracleTensor(p0)
    exact = p0.dtype == torch.float32
    worst = 0.0
    for t in range(1, steps + 1):
        g = grad_fn(t).to(g_dtype)
        say(f"[{what}] step {t} numel {p0.numel()} p {p0.dtype} g {g_dtype}")
        q4.fused_4bit(dev.p, g.to(device).reshape(-1), dev.m, dev.v, dev.sm, dev.sv,
                      hp["beta1"], hp["beta2"], hp["lr"], hp["weight_decay"], hp["eps"], t)
        torch.cuda.synchronize()
        prev = ref.step(g, t, hp)
        worst = max(worst, assert_state_equal(dev, ref, prev, f"{what} step {t}"))
        if not exact:
            ref.resync(dev.p)
    return worst


def test_config1_single_tensor(cuda):
    """4096x4096 fp32, seed 0, outlier-laden grads, 10 steps."""
    gen = torch.Generator().manual_seed(0)
    n = 4096 * 4096
    p0 = torch.randn(n, generator=gen) * 0.02
    mark = len(STRICT_LOG)
    worst = run_steps(p0, lambda t: grads_config1(gen, n), 10, cuda, what="config1")
    say(f"config1 worst relative parameter error {worst:.3e}")
    assert strict_atol_since(mark) <= BASELINE_ATOL        # |dev - ref| <= 5e-10 + 1e-6 |ref| every step


@pytest.mark.parametrize("n", [1, 2, 127, 128, 129, 511, 512, 513, 4095, 4097, 1000003, 3 * 1000003])
def test_ragged_lengths(cuda, n):
    """Tail blocks, odd lengths (half-filled last byte), zeros and denormals in the grads."""
    gen = torch.Generator().manual_seed(1000 + n % 997)
    p0 = torch.randn(n, generator=gen) * 0.02
    run_steps(p0, lambda t: grads_config3(gen, n), 3, cuda, what=f"ragged n={n}")


@pytest.mark.parametrize("n", [1, 3, 127, 129, 513, 4097, 100003])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_ragged_lengths_16_bit(cuda, n, dt):
    """tail tiles of the 8-elements-per-lane geometry: element-wise conversions, half-filled
    last byte, values that overflow fp16 (+-1e3 gradients stay finite; parameters near the top
    of the fp16 range round to infinity in the oracle and on the device alike)"""
    gen = torch.Generator().manual_seed(2000 + n)
    p0 = (torch.randn(n, generator=gen) * 0.02).to(dt)
    if dt == torch.float16 and n > 3:
        p0[1], p0[2] = 65504.0, -65504.0
    run_steps(p0, lambda t: grads_config3(gen, n), 3, cuda, g_dtype=dt, what=f"ragged {dt} n={n}")


@pytest.mark.parametrize("offsets", [(1, 0), (0, 1), (1, 1), (3, 5), (7, 2)])
@pytest.mark.parametrize("p_dtype,g_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                             (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                             (torch.float16, torch.float16)])
def test_views_at_odd_element_offsets(cuda, p_dtype, g_dtype, offsets):
    """Parameters and gradients that start 2 to 28 bytes past a 16-byte boundary (views into a
    flat buffer): the 16-byte accesses of the full tiles and the element-wise ones of the last
    tile give the oracle's results, and nothing outside the views is written."""
    po, go = offsets
    for n in (1000003, 4096 * 33):
        gen = torch.Generator().manual_seed(n + 17 * po + go)
        p0 = (torch.randn(n, generator=gen) * 0.02).to(p_dtype)
        p_big = torch.full((n + 64,), 3.0, dtype=p_dtype, device=cuda)
        g_big = torch.full((n + 64,), 5.0, dtype=g_dtype, device=cuda)
        dev = DeviceTensor(p0, cuda)
        dev.p = p_big[po:po + n]
        dev.p.copy_(p0)
        assert dev.p.data_ptr() % 16 or not po
        g_view = g_big[go:go + n]
        ref = OracleTensor(p0)
        for t in range(1, 4):
            g = (torch.randn(n, generator=gen) * 1e-3).to(g_dtype)
            g_view.copy_(g)
            say(f"[odd offsets] p {p_dtype}+{po} g {g_dtype}+{go} n {n} step {t}")
            q4.fused_4bit(dev.p, g_view, dev.m, dev.v, dev.sm, dev.sv, HP["beta1"], HP["beta2"], HP["lr"],
                          HP["weight_decay"], HP["eps"], t)
            torch.cuda.synchronize()
            prev = ref.step(g, t)
            assert_state_equal(dev, ref, prev, f"odd offsets step {t}")
            ref.resync(dev.p)
        assert (p_big[:po] == 3.0).all() and (p_big[po + n:] == 3.0).all()
        assert (g_big[:go] == 5.0).all() and (g_big[go + n:] == 5.0).all() and torch.equal(g_view.cpu(), g)


def test_all_zero_blocks_and_guard_bytes(cuda):
    """Blocks whose grads stay zero keep zero codes and zero scales; bytes past the
    packed length and scales past the last block are never written."""
    n = 128 * 9 + 37
    gen = torch.Generator().manual_seed(7)
    p0 = torch.randn(n, generator=gen) * 0.02
    g = torch.randn(n, generator=gen) * 1e-3
    g[128:384] = 0.0          # two all-zero blocks
    g[640:768] = 0.0
    nbytes, nblk = oc.state_sizes(n)
    pad = 64
    dev = DeviceTensor(p0, cuda)
    m_big = torch.full((nbytes + pad,), 0xA5, dtype=torch.uint8, device=cuda)
    v_big = torch.full((nbytes + pad,), 0x5A, dtype=torch.uint8, device=cuda)
    sm_big = torch.full((nblk + pad,), 123.0, device=cuda)
    sv_big = torch.full((nblk + pad,), 321.0, device=cuda)
    p_big = torch.full((n + pad,), 9.0, device=cuda)
    m_big[:nbytes] = 0
    v_big[:nbytes] = 0
    sm_big[:nblk] = 0
    sv_big[:nblk] = 0
    p_big[:n] = p0.to(cuda)
    ref = OracleTensor(p0)
    for t in range(1, 4):
        say(f"[zero blocks] step {t}")
        q4.fused_4bit(p_big[:n], g.to(cuda), m_big[:nbytes], v_big[:nbytes], sm_big[:nblk],
                      sv_big[:nblk], HP["beta1"], HP["beta2"], HP["lr"], HP["weight_decay"],
                      HP["eps"], t)
        torch.cuda.synchronize()
        prev = ref.step(g, t)
        dev.p, dev.m, dev.v, dev.sm, dev.sv = p_big[:n], m_big[:nbytes], v_big[:nbytes], sm_big[:nblk], sv_big[:nblk]
        assert_state_equal(dev, ref, prev, f"zero blocks step {t}")
        ref.resync(dev.p)
        for b in (1, 2, 5):
            assert ref.sm[b] == 0 and ref.sv[b] == 0
            assert not ref.m[b * 64:(b + 1) * 64].any() and not ref.v[b * 64:(b + 1) * 64].any()
    assert (m_big[nbytes:] == 0xA5).all() and (v_big[nbytes:] == 0x5A).all()
    assert (sm_big[nblk:] == 123.0).all() and (sv_big[nblk:] == 321.0).all()
    assert (p_big[n:] == 9.0).all()


def _nudge(x, d):
    """x moved by d ulps away from (d > 0) or towards (d < 0) zero."""
    u = np.float32(x).view(np.uint32)
    return np.uint32(int(u) + d).view(np.float32)


def _threshold_probe_grads(n_blocks, rng):
    """Gradients that, from zero state, put the normalised moments exactly on and
    within a few ulps of every quantization threshold.  From zero state
    m' = r1*g and v' = r2*g*g, so the block's largest |g| fixes the scale and the
    others are chosen as threshold * largest, nudged by -3..+3 ulps."""
    qm_mid = oc.tables(0)[1]
    qv_mid = oc.tables(1)[1]
    g = np.zeros((n_blocks, 128), np.float32)
    for b in range(n_blocks):
        big = np.float32(10.0 ** rng.uniform(-6, 0))
        row = []
        for mid in qm_mid:
            base = np.float32(np.float32(mid) * big)
            row += [_nudge(base, d) for d in range(-3, 4)]
        for mid in qv_mid:
            base = np.float32(np.sqrt(np.float64(mid)) * big)
            row += [_nudge(base, d) for d in (-1, 0, 1)]
        row = np.array(row, np.float32)
        rng.shuffle(row)
        row = row[:127]
        g[b, 0] = big
        g[b, 1:1 + row.size] = row
    return g.reshape(-1)


def test_threshold_neighbourhoods(cuda):
    """Binary-search boundary ties: values on and next to every threshold."""
    rng = np.random.default_rng(3)
    n_blocks = 4096
    g_np = _threshold_probe_grads(n_blocks, rng)
    n = g_np.size
    gen = torch.Generator().manual_seed(3)
    p0 = torch.randn(n, generator=gen) * 0.02
    g = torch.from_numpy(g_np)
    run_steps(p0, lambda t: g if t == 1 else g * float(1 + 0.37 * t), 3, cuda, what="thresholds")


def test_dense_threshold_sweep(cuda):
    """Every block holds one element of magnitude 1 and 127 elements spread over a
    narrow band around one threshold, so that many quotients fall inside the
    kernel's guard bands and take its exact path."""
    qm_mid, qv_mid = oc.tables(0)[1], oc.tables(1)[1]
    rng = np.random.default_rng(11)
    rows = []
    for mid in list(qm_mid) + [float(np.sqrt(x)) for x in qv_mid]:
        for _ in range(64):
            big = np.float32(10.0 ** rng.uniform(-5, -1))
            band = np.float32(mid) * big * (1.0 + rng.uniform(-4e-6, 4e-6, 127))
            rows.append(np.concatenate(([big], band)).astype(np.float32))
    g_np = np.concatenate(rows)
    n = g_np.size
    gen = torch.Generator().manual_seed(5)
    p0 = torch.randn(n, generator=gen) * 0.02
    g = torch.from_numpy(g_np)
    run_steps(p0, lambda t: g, 2, cuda, what="dense thresholds")


def test_extreme_scales(cuda):
    """Blocks whose abs-max is denormal, tiny, huge: the kernel's reciprocal path does
    not apply there and the exact path must take over."""
    rng = np.random.default_rng(5)
    rows = []
    for e in (-44, -40, -38, -36, -34, -30, -20, -10, 0, 10, 15, 17):
        for _ in range(8):
            rows.append((rng.standard_normal(128) * 10.0 ** e).astype(np.float32))
    g_np = np.concatenate(rows)
    n = g_np.size
    gen = torch.Generator().manual_seed(9)
    p0 = torch.randn(n, generator=gen) * 0.02
    g = torch.from_numpy(g_np)
    run_steps(p0, lambda t: g * float(t), 3, cuda, what="extreme scales")


@pytest.mark.parametrize("p_dtype,g_dtype", [(torch.float32, torch.bfloat16),
                                             (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float32),
                                             (torch.float16, torch.float16),
                                             (torch.float32, torch.float16),
                                             (torch.float16, torch.float32),
                                             (torch.float16, torch.bfloat16),
                                             (torch.bfloat16, torch.float16)])
def test_bf16_io(cuda, p_dtype, g_dtype):
    """16-bit gradient and parameter variants, bf16 and fp16 (Llama-shaped distributions)."""
    gen = torch.Generator().manual_seed(21)
    n = 1024 * 4096 + 777
    p0 = (torch.randn(n, generator=gen) * 0.02).to(p_dtype)
    run_steps(p0, lambda t: grads_student_t(gen, n), 3, cuda, g_dtype=g_dtype,
              what=f"bf16 io p={p_dtype} g={g_dtype}")


def test_driver_hyperparameters(cuda):
    """The reference test's non-default hyper-parameters (tests/driver.py:28-31)."""
    gen = torch.Generator().manual_seed(2020)
    n = 300000
    p0 = torch.randn(n, generator=gen) * 0.1
    run_steps(p0, lambda t: torch.randn(n, generator=gen) * 1e-2, 10, cuda, hp=HP_DRIVER,
              what="driver hp")


def test_multi_tensor_matches_single(cuda):
    """One multi-tensor launch equals per-tensor launches bit for bit (params too)."""
    gen = torch.Generator().manual_seed(31)
    sizes = [5000, 4097, 128 * 300, 1000003, 9, 70001, 512 * 64, 512 * 64 + 1]
    ps = [torch.randn(n, generator=gen) * 0.02 for n in sizes]
    a = [DeviceTensor(p, cuda) for p in ps]
    b = [DeviceTensor(p, cuda) for p in ps]
    for t in range(1, 4):
        gs = [grads_config3(gen, n).to(cuda) for n in sizes]
        say(f"[multi] step {t}")
        q4.fused_4bit_multi([x.p for x in a], gs, [x.m for x in a], [x.v for x in a],
                            [x.sm for x in a], [x.sv for x in a], HP["beta1"], HP["beta2"],
                            HP["lr"], HP["weight_decay"], HP["eps"], t)
        for x, g in zip(b, gs):
            q4.fused_4bit(x.p, g, x.m, x.v, x.sm, x.sv, HP["beta1"], HP["beta2"], HP["lr"],
                          HP["weight_decay"], HP["eps"], t)
        torch.cuda.synchronize()
        for x, y in zip(a, b):
            assert torch.equal(x.m, y.m) and torch.equal(x.v, y.v)
            assert torch.equal(x.sm.view(torch.int32), y.sm.view(torch.int32))
            assert torch.equal(x.sv.view(torch.int32), y.sv.view(torch.int32))
            assert torch.equal(x.p.view(torch.int32), y.p.view(torch.int32))


def test_unquantized_step_vs_oracle(cuda):
    """Small-tensor path: fp32 moments bit-exact, params within tolerance."""
    gen = torch.Generator().manual_seed(41)
    sizes = [1, 768, 2304, 3072, 4096, 10000]
    ps = [torch.randn(n, generator=gen) * 0.02 for n in sizes]
    dp = [p.clone().to(cuda) for p in ps]
    dm = [torch.zeros(n, device=cuda) for n in sizes]
    dv = [torch.zeros(n, device=cuda) for n in sizes]
    rp = [p.numpy().copy() for p in ps]
    rm = [np.zeros(n, np.float32) for n in sizes]
    rv = [np.zeros(n, np.float32) for n in sizes]
    for t in range(1, 6):
        gs = [grads_config3(gen, n) for n in sizes]
        say(f"[unquant] step {t}")
        q4.fused_single_tensor_multi(dp, [g.to(cuda) for g in gs], dm, dv, HP["beta1"], HP["beta2"],
                                     HP["lr"], HP["weight_decay"], HP["eps"], t)
        torch.cuda.synchronize()
        for i, g in enumerate(gs):
            prev = rp[i].copy()
            oc.step_unquant(rp[i], g.numpy(), rm[i], rv[i], step=t, **HP)
            assert np.array_equal(bits(dm[i].cpu().numpy()), bits(rm[i]))
            assert np.array_equal(bits(dv[i].cpu().numpy()), bits(rv[i]))
            ok, worst = p_close(dp[i].cpu().numpy(), rp[i], prev, exact=True)   # this kernel's update is the exact form
            assert ok, f"unquant params: {worst} mismatches"
            rp[i][:] = dp[i].cpu().numpy()


def test_replay_under_graph_capture(cuda):
    """The library allocates nothing and only launches kernels, so a step can be captured
    into a graph; replays (same step number, refreshed inputs) must equal eager launches."""
    gen = torch.Generator().manual_seed(77)
    sizes = [70001, 4097, 128 * 40]
    ps = [torch.randn(n, generator=gen) * 0.02 for n in sizes]
    eager = [DeviceTensor(p, cuda) for p in ps]
    graphed = [DeviceTensor(p, cuda) for p in ps]
    gbuf = [torch.zeros(n, device=cuda) for n in sizes]
    args = (HP["beta1"], HP["beta2"], HP["lr"], HP["weight_decay"], HP["eps"], 3)

    def launch(ts, gs):
        q4.fused_4bit_multi([x.p for x in ts], gs, [x.m for x in ts], [x.v for x in ts],
                            [x.sm for x in ts], [x.sv for x in ts], *args)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(graphed, gbuf)                      # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for x, p in zip(graphed, ps):                  # undo the warm-up step
        x.p.copy_(p.to(cuda)); x.m.zero_(); x.v.zero_(); x.sm.zero_(); x.sv.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch(graphed, gbuf)
    for x, p in zip(graphed, ps):                  # capture does not execute, but be explicit
        x.p.copy_(p.to(cuda)); x.m.zero_(); x.v.zero_(); x.sm.zero_(); x.sv.zero_()
    for rep in range(4):
        gs = [grads_config3(gen, n).to(cuda) for n in sizes]
        for b, g in zip(gbuf, gs):
            b.copy_(g)
        say(f"[graph] replay {rep}")
        graph.replay()
        launch(eager, gs)
        torch.cuda.synchronize()
        for x, y in zip(graphed, eager):
            assert torch.equal(x.m, y.m) and torch.equal(x.v, y.v)
            assert torch.equal(x.sm.view(torch.int32), y.sm.view(torch.int32))
            assert torch.equal(x.sv.view(torch.int32), y.sv.view(torch.int32))
            assert torch.equal(x.p.view(torch.int32), y.p.view(torch.int32))


def test_concurrent_threads_and_streams(cuda):
    """the library keeps no state between calls (descriptors travel in the kernel arguments,
    the error text is per thread): four host threads, each on a stream of its own, step their
    own tensors at the same time -- ctypes drops the interpreter lock during the calls -- and
    every result equals the same steps made one after the other; a refusal in one thread
    leaves its message in that thread only"""
    import threading
    from quantfour_adamw_cuda_amd import _lib
    gen = torch.Generator().manual_seed(77)
    nthreads, steps = 4, 12
    sizes = [150_001 + 4096 * i for i in range(nthreads)]
    p0s = [torch.randn(n, generator=gen) * 0.02 for n in sizes]
    gs = [[grads_config1(gen, n).to(torch.bfloat16).to(cuda) for _ in range(steps)] for n in sizes]
    seq = [DeviceTensor(p0, cuda) for p0 in p0s]
    for d, g_list in zip(seq, gs):
        for t, g in enumerate(g_list, 1):
            q4.fused_4bit(d.p, g, d.m, d.v, d.sm, d.sv, *[HP[k] for k in ("beta1", "beta2", "lr", "weight_decay", "eps")], t)
    torch.cuda.synchronize()
    par = [DeviceTensor(p0, cuda) for p0 in p0s]
    errors, messages = [], [None] * nthreads
    barrier = threading.Barrier(nthreads)

    def worker(i):
        try:
            stream = torch.cuda.Stream(device=cuda)
            L = _lib.load()
            barrier.wait()
            with torch.cuda.stream(stream):
                d = par[i]
                for t, g in enumerate(gs[i], 1):
                    q4.fused_4bit(d.p, g, d.m, d.v, d.sm, d.sv,
                                  *[HP[k] for k in ("beta1", "beta2", "lr", "weight_decay", "eps")], t)
                    if i == 0 and t == 3:      # a refusal: nothing launched, message stays in this thread
                        rc = L.q4adamw_fused_4bit(d.p.data_ptr() + 2, g.data_ptr(), d.m.data_ptr(), d.v.data_ptr(),
                                                  d.sm.data_ptr(), d.sv.data_ptr(), 1000, 0, 1, 0.9, 0.999, 1e-3,
                                                  0.01, 1e-8, 1.0, stream.cuda_stream)
                        assert rc == -2
                messages[i] = L.q4adamw_last_error().decode()
            stream.synchronize()
        except Exception as e:   # noqa: BLE001
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(nthreads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=120)
    assert not errors, errors
    torch.cuda.synchronize()
    for a, b in zip(seq, par):
        for x, y in zip((a.p, a.m, a.v, a.sm, a.sv), (b.p, b.m, b.v, b.sm, b.sv)):
            assert torch.equal(x, y)
    assert "aligned" in messages[0] and all(m == "" for m in messages[1:]), messages


@pytest.mark.parametrize("p_dtype,g_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                             (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16)])
def test_non_finite_gradients(cuda, p_dtype, g_dtype):
    """inf, -inf and NaN gradients in some blocks: codes and scales still match the oracle bit
    for bit (a block's scale is the maximum over its non-NaN magnitudes, an infinite scale sends
    finite values to the code of zero, inf/inf and NaN get code 0); the blocks without such
    values are untouched by their neighbours; parameters agree where the oracle's are finite
    and are non-finite where the oracle's are"""
    n = 128 * 64 + 50
    gen = torch.Generator().manual_seed(17)
    p0 = (torch.randn(n, generator=gen) * 0.05).to(p_dtype)
    dev, ref = DeviceTensor(p0, cuda), OracleTensor(p0)
    inf, nan = float("inf"), float("nan")
    for step in (1, 2, 3):
        g = grads_config1(gen, n)
        if step == 2:
            g[5] = inf                     # one inf in block 0
            g[128 + 7] = -inf              # block 1
            g[256 + 9] = nan               # block 2
            g[384:512] = nan               # block 3: nothing but NaN
            g[512 + 1], g[512 + 2] = inf, nan   # block 4: both
            g[n - 3] = inf                 # the ragged last block
        g = g.to(g_dtype)
        q4.fused_4bit(dev.p, g.to(cuda), dev.m, dev.v, dev.sm, dev.sv, HP["beta1"], HP["beta2"], HP["lr"],
                      HP["weight_decay"], HP["eps"], step)
        prev = ref.step(g, step)
        for name, d, r in (("sm", dev.sm, ref.sm), ("sv", dev.sv, ref.sv)):
            assert np.array_equal(bits(d.cpu().numpy()), bits(r)), f"step {step}: {name}: {d.cpu().numpy()[:6]} vs {r[:6]}"
        assert np.array_equal(dev.m.cpu().numpy(), ref.m), f"step {step}: m codes"
        assert np.array_equal(dev.v.cpu().numpy(), ref.v), f"step {step}: v codes"
        p_dev = dev.p.float().cpu().numpy()
        p_ref = (ref.p.astype(np.float32) if ref.p.dtype != np.uint16
                 else (ref.p.astype(np.uint32) << 16).view(np.float32))
        finite = np.isfinite(p_ref)
        assert np.array_equal(np.isfinite(p_dev), finite), f"step {step}: finiteness of the parameters"
        ok, worst = p_close(to_np(dev.p)[finite], ref.p[finite], prev[finite], bf16=p_dtype == torch.bfloat16,
                            exact=p_dtype == torch.float32)
        assert ok, f"step {step}: parameters out of tolerance (worst {worst})"
        ref.resync(dev.p)


def test_batches_and_tensors_larger_than_a_grid(cuda):
    """With the grid size lowered to 64 workgroups (q4adamw_set_grid_limit), a tensor of 300
    chunks spans five grids and a list of tensors is cut in the middle of one: every entry point
    that launches one workgroup per chunk still gives the oracle's bits -- the block-scaled step
    (plain, with gradient options, stochastic rounding), rank-1 scaling (statistics and update),
    the non-quantized step, and the checkpoint quantizers."""
    from oracle import q4_oracle_torch as ot
    from quantfour_adamw_cuda_amd import _lib
    from quantfour_adamw_cuda_amd import quantfour_hip as qh
    L = _lib.load()
    hpa = (HP["beta1"], HP["beta2"], HP["lr"], HP["weight_decay"], HP["eps"])
    gen = torch.Generator().manual_seed(99)
    sizes = [1024 * 300 + 77, 5000, 1024 * 70, 129]
    try:
        L.q4adamw_set_grid_limit(64)
        # block-scaled, one call over the list; then the same with options and with noise
        ps = [torch.randn(n, generator=gen) * 0.02 for n in sizes]
        for variant in ("plain", "options", "stochastic"):
            devs = [DeviceTensor(p, cuda) for p in ps]
            refs = [(p.clone(),) + tuple(t.cpu() for t in (d.m, d.v, d.sm, d.sv)) for p, d in zip(ps, devs)]
            for step in (1, 2):
                gs = [grads_config3(gen, n) for n in sizes]
                dg = [g.to(cuda) for g in gs]
                lists = ([d.p for d in devs], dg, [d.m for d in devs], [d.v for d in devs], [d.sm for d in devs], [d.sv for d in devs])
                if variant == "stochastic":
                    qh.fused_4bit_multi_sr(*lists, *hpa, step, 7, salts=[5, 6, 7, 8], update_form="exact")
                    refs = [ot.step_quant_sr(r[0], g, *r[1:], seed=7, tensor_salt=s, step=step, **HP)
                            for r, g, s in zip(refs, gs, (5, 6, 7, 8))]
                else:
                    kw = dict(grad_scale=0.5, zero_grad=True) if variant == "options" else {}
                    qh.fused_4bit_multi(*lists, *hpa, step, **kw)
                    refs = [ot.step_quant(r[0], g * 0.5 if kw else g, *r[1:], step=step, **HP) for r, g in zip(refs, gs)]
                    if kw:
                        assert all(not g.any() for g in dg), "gradients cleared in every grid"
                for d, r, n in zip(devs, refs, sizes):
                    assert torch.equal(d.m.cpu(), r[1]) and torch.equal(d.v.cpu(), r[2]), f"{variant} n={n} step {step}: codes"
                    assert torch.equal(d.sm.cpu().view(torch.int32), r[3].view(torch.int32))
                    assert torch.equal(d.p.cpu().view(torch.int32), r[0].view(torch.int32)), f"{variant} n={n} step {step}: parameters"
        # rank-1: 300 x 1024 (rows form: 75 row groups x 4 tiles = 300 chunks; 2 statistics tiles... and a
        # 1300 x 520 matrix in the wide form (660 chunks, 12 statistics tiles)
        for rows, cols in ((300, 1024), (1300, 520)):
            p0 = torch.randn(rows, cols, generator=gen) * 0.05
            n = rows * cols
            p = p0.clone().to(cuda)
            m = torch.zeros((n + 1) // 2, dtype=torch.uint8, device=cuda)
            v, sm = torch.zeros_like(m), torch.zeros((n + 127) // 128, device=cuda)
            r, c, rn, cn = (torch.zeros(k, device=cuda) for k in (rows, cols, rows, cols))
            ref = (p0.clone(), m.cpu(), v.cpu(), sm.cpu(), r.cpu(), c.cpu())
            for step in (1, 2, 3):
                g = grads_config1(gen, n).view(rows, cols)
                ref = ot.step_quant_rank1(ref[0], g, *ref[1:], step=step, **HP)
                qh.fused_4bit_rank1_multi([p], [g.to(cuda)], [m], [v], [sm], [r], [c], [rn], [cn], *hpa, step,
                                          update_form="exact")
                assert torch.equal(m.cpu(), ref[1]) and torch.equal(v.cpu(), ref[2]), f"rank-1 {rows}x{cols} step {step}"
                assert torch.equal(r.cpu().view(torch.int32), ref[4].view(torch.int32))
                assert torch.equal(c.cpu().view(torch.int32), ref[5].view(torch.int32))
                assert torch.equal(p.cpu().view(torch.int32), ref[0].view(torch.int32))
        # non-quantized step: 100 tensors of 3000 elements = 300 chunks of 1024
        small = [torch.randn(3000, generator=gen) * 0.02 for _ in range(100)]
        dp = [p.clone().to(cuda) for p in small]
        dm, dv = [torch.zeros(3000, device=cuda) for _ in small], [torch.zeros(3000, device=cuda) for _ in small]
        rp, rm, rv = [p.numpy().copy() for p in small], [np.zeros(3000, np.float32) for _ in small], [np.zeros(3000, np.float32) for _ in small]
        gs = [torch.randn(3000, generator=gen) * 1e-3 for _ in small]
        q4.fused_single_tensor_multi(dp, [g.to(cuda) for g in gs], dm, dv, *hpa, 1)
        for i, g in enumerate(gs):
            oc.step_unquant(rp[i], g.numpy(), rm[i], rv[i], step=1, **HP)
            assert np.array_equal(bits(dp[i].cpu().numpy()), bits(rp[i])) and np.array_equal(bits(dm[i].cpu().numpy()), bits(rm[i]))
        # checkpoint quantizers: 128 * 4 * 200 elements = 200 workgroups of four blocks
        x = torch.randn(128 * 4 * 200 + 50, generator=gen)
        for which in (0, 1):
            xx = x.abs() if which else x
            codes, scales = qh.quantize_state(xx.to(cuda), which)
            rc, rs = oc.quant(xx.numpy(), which)
            assert np.array_equal(codes.cpu().numpy(), rc) and np.array_equal(bits(scales.cpu().numpy()), bits(rs))
            back = qh.dequantize_state(codes, scales, xx.numel(), which)
            assert np.array_equal(bits(back.cpu().numpy()), bits(oc.dequant(rc, rs, xx.numel(), which)))
    finally:
        L.q4adamw_set_grid_limit(0)
