"""Pins of the CPU oracle (no GPU): tables against known-answer bit patterns and closed
forms, the quantizer against brute force and a library routine, the derived scalars
against known answers, the two independent restatements against each other, the
non-quantized step against torch.optim.AdamW, and the quantized step against
invariants of the format."""

import numpy as np
import pytest
import torch

from oracle import q4_oracle as oc
from oracle import q4_oracle_torch as ot
from tests.q4_testlib import HP, HP_DRIVER, bits, grads_config1, grads_config3, grads_student_t

# fp32 bit patterns of the reference's literal tables (optim/cuda_adamw_kernels.cu:25-98)
QMAP_M_HEX = ("bf633333 bf29999a bee00000 be59999a bd9eb852 bd051eb8 bbb43958 00000000 "
              "3bb43958 3d051eb8 3d9eb852 3e59999a 3ee00000 3f29999a 3f633333 3f800000").split()
QMID_M_HEX = ("bf466666 bf0ccccd bea66666 be147ae1 bd6147ae bc9ba5e3 bb343958 3b343958 "
              "3c9ba5e3 3d6147ae 3e147ae1 3ea66666 3f0ccccd 3f466666 3f71999a").split()


def hexes(a):
    return [f"{x:08x}" for x in bits(a)]


def test_tables_known_answers():
    qm, mid = oc.tables(0)
    assert hexes(qm) == QMAP_M_HEX
    assert hexes(mid) == QMID_M_HEX
    qv, midv = oc.tables(1)
    assert np.array_equal(qv, np.arange(1, 17, dtype=np.float32) / 16)
    assert np.array_equal(midv, (2 * np.arange(1, 16, dtype=np.float32) + 1) / 32)
    for which in (0, 1):
        assert np.array_equal(oc.tables(which)[0], ot.QMAP[which].numpy())
        assert np.array_equal(oc.tables(which)[1], ot.QMID[which].numpy())


def test_tables_closed_forms():
    """The first-moment map is the dynamic-exponent construction of quant_opt_base.py:55-86;
    the thresholds are the means of neighbouring entries, except that the literal table
    is one ulp below the fp32 mean at entries 3 and 10 (+-0.145)."""
    qm_cf, mid_cf, qv_cf, midv_cf = ot.closed_form_tables()
    qm, mid = oc.tables(0)
    assert np.array_equal(np.asarray(qm_cf, np.float32), qm)
    assert np.array_equal(np.asarray(mid_cf, np.float32), mid)      # double means, rounded once
    fp32_means = (qm[:-1] + qm[1:]) * np.float32(0.5)
    differ = np.flatnonzero(bits(fp32_means) != bits(mid))
    assert differ.tolist() == [3, 10]
    assert (bits(fp32_means)[differ].astype(np.int64) - bits(mid)[differ].astype(np.int64)).tolist() == [1, 1]
    for which in (0, 1):
        q, m = oc.tables(which)
        assert np.all(q[:-1] < m) and np.all(m < q[1:])              # strictly between neighbours


def _neighbourhood(values, radius):
    out = []
    for v in values:
        u = int(np.float32(v).view(np.uint32))
        for d in range(-radius, radius + 1):
            w = u + d
            if 0 <= (w & 0x7fffffff) < 0x7f800000:
                out.append(np.uint32(w & 0xffffffff).view(np.float32))
    return np.array(out, np.float32)


@pytest.mark.parametrize("which", [0, 1])
def test_quantizer_search_equals_count_and_library(which):
    """Binary search restated from the reference == number of thresholds strictly below x
    == numpy.searchsorted(mid, x, 'left'), on every fp32 within 64 ulps of every table
    entry and threshold, on +-0, on the range ends and on two million random values."""
    qmap, mid = oc.tables(which)
    rng = np.random.default_rng(which)
    xs = np.concatenate([
        _neighbourhood(np.concatenate([qmap, mid, [0.0, -0.0, 1.0, -1.0]]), 64),
        rng.uniform(-1.2, 1.2, 2_000_000).astype(np.float32),
        (rng.standard_normal(200_000) * 1e-3).astype(np.float32),
        np.array([np.inf, -np.inf, 3e38, -3e38, 1e-45, -1e-45], np.float32),
    ])
    lib = oc.lib()
    search = np.fromiter((lib.q4o_quantize_search(which, float(x)) for x in xs[:300_000]), np.int32)
    count = np.fromiter((lib.q4o_quantize_count(which, float(x)) for x in xs[:300_000]), np.int32)
    assert np.array_equal(search, count)
    ss = np.searchsorted(mid, xs, side="left").astype(np.int32)
    assert np.array_equal(ss[:300_000], count)
    # the vectorised restatement uses torch.bucketize
    tb = torch.bucketize(torch.from_numpy(xs), ot.QMID[which], right=False).numpy().astype(np.int32)
    assert np.array_equal(tb, ss)


@pytest.mark.parametrize("which", [0, 1])
def test_quantizer_special_cases(which):
    qmap, mid = oc.tables(which)
    for k, q in enumerate(qmap):                       # a code-book entry maps to itself
        assert oc.quantize_count(which, q) == k and oc.quantize_search(which, q) == k
    for j, m in enumerate(mid):                        # a tie goes DOWN
        assert oc.quantize_count(which, m) == j
        assert oc.quantize_count(which, np.nextafter(m, np.float32(2))) == j + 1
        assert oc.quantize_search(which, m) == j
    assert oc.quantize_count(which, np.float32(-5)) == 0 and oc.quantize_count(which, np.float32(5)) == 15
    assert oc.quantize_count(which, np.float32("nan")) == 0 and oc.quantize_search(which, np.float32("nan")) == 0
    if which == 0:
        assert oc.quantize_count(0, np.float32(-1.0)) == 0    # x <= -0.8875
        assert oc.quantize_count(0, np.float32(0.0)) == 7 and oc.quantize_count(0, np.float32(-0.0)) == 7
    else:
        assert oc.quantize_count(1, np.float32(0.0)) == 0


def test_derived_scalars_known_answers():
    s = oc.derive_scalars(0.9, 0.999, 1e-3, 0.01, 1)
    # 1 - f32(0.999) is NOT f32(0.001): 0x3a831200 vs 0x3a83126f
    assert f"{bits(s)[4]:08x}" == "3dccccd0" and f"{bits(s)[5]:08x}" == "3a831200"
    assert f"{bits(s)[3]:08x}" == "3f7fff58"
    assert f"{int(np.float32(0.001).view(np.uint32)):08x}" == "3a83126f"
    for b1, b2, lr, wd in [(0.9, 0.999, 1e-3, 0.01), (0.8, 0.88, 5e-3, 0.03), (0.95, 0.99, 3e-4, 0.1)]:
        f32 = np.float32
        one = f32(1)
        for t in [1, 2, 3, 10, 100, 1000, 5000]:
            s = oc.derive_scalars(b1, b2, lr, wd, t)
            # the same chain in numpy fp32 scalars, pow taken in double and rounded once
            c1 = one - f32(float(f32(b1)) ** t)
            c2s = np.sqrt(one - f32(float(f32(b2)) ** t))
            want = np.array([c1, c2s, f32(lr) / c1, one - f32(lr) * f32(wd), one - f32(b1),
                             one - f32(b2)], f32)
            assert np.array_equal(bits(want), bits(s))
            # and against double precision: the fp32 chain loses at most the cancellation
            # error of 1 - beta**t, i.e. half an ulp of 1.0 relative to the difference
            c1d = 1 - float(f32(b1)) ** t
            assert abs(float(s[0]) - c1d) <= 2.0 ** -24 and abs(float(s[2]) * c1d - float(f32(lr))) < 1e-9
            st = ot.derive_scalars(b1, b2, lr, wd, t)
            got = np.array([st["c1"], st["c2s"], st["ss"], st["wdu"], st["r1"], st["r2"]], np.float32)
            assert np.array_equal(bits(got), bits(s))


def _zero_state(n):
    nb, nk = oc.state_sizes(n)
    return (np.zeros(nb, np.uint8), np.zeros(nb, np.uint8), np.zeros(nk, np.float32), np.zeros(nk, np.float32))


@pytest.mark.parametrize("n,gradfn,hp", [
    (300_007, grads_config1, HP), (128 * 11 + 1, grads_config3, HP), (127, grads_config3, HP),
    (1, grads_config3, HP), (4097, grads_config3, HP), (200_000, grads_student_t, HP),
    (50_001, grads_config1, HP_DRIVER)])
def test_two_restatements_agree_bit_for_bit(n, gradfn, hp):
    """Scalar C oracle == vectorised torch oracle: params, codes, scales, every step."""
    gen = torch.Generator().manual_seed(n)
    p = torch.randn(n, generator=gen) * 0.02
    pc = p.numpy().copy()
    m, v, sm, sv = _zero_state(n)
    tm, tv, tsm, tsv = (torch.from_numpy(x.copy()) for x in (m, v, sm, sv))
    for step in range(1, 5):
        g = gradfn(gen, n)
        oc.step_quant(pc, g.numpy(), m, v, sm, sv, step=step, **hp)
        p, tm, tv, tsm, tsv = ot.step_quant(p, g, tm, tv, tsm, tsv, step=step, **hp)
        assert np.array_equal(bits(p.numpy()), bits(pc))
        assert np.array_equal(tm.numpy(), m) and np.array_equal(tv.numpy(), v)
        assert np.array_equal(bits(tsm.numpy()), bits(sm)) and np.array_equal(bits(tsv.numpy()), bits(sv))


def test_bf16_restatements_agree():
    """bf16 gradients widen exactly; bf16 parameters are rounded to nearest even on store."""
    gen = torch.Generator().manual_seed(5)
    n = 70_003
    for p_dtype in (torch.float32, torch.bfloat16):
        p = (torch.randn(n, generator=gen) * 0.02).to(p_dtype)
        pc = (p.view(torch.int16).numpy().view(np.uint16).copy() if p_dtype == torch.bfloat16
              else p.numpy().copy())
        m, v, sm, sv = _zero_state(n)
        tm, tv, tsm, tsv = (torch.from_numpy(x.copy()) for x in (m, v, sm, sv))
        for step in range(1, 4):
            g = grads_student_t(gen, n).to(torch.bfloat16)
            gb = g.view(torch.int16).numpy().view(np.uint16).copy()
            oc.step_quant(pc, gb, m, v, sm, sv, step=step, **HP)
            p, tm, tv, tsm, tsv = ot.step_quant(p, g, tm, tv, tsm, tsv, step=step, **HP)
            got = p.view(torch.int16).numpy().view(np.uint16) if p_dtype == torch.bfloat16 else bits(p.numpy())
            assert np.array_equal(got, pc if p_dtype == torch.bfloat16 else bits(pc))
            assert np.array_equal(tm.numpy(), m) and np.array_equal(tv.numpy(), v)


def test_format_invariants():
    """scale == max |x| of the block; the arg-max gets code 15 (or 0 for a negative first
    moment); pack/unpack round trip; unused high nibble of an odd tail is zero; an
    all-zero block is closed under the step (zero codes, zero scales, stays so)."""
    rng = np.random.default_rng(0)
    n = 128 * 7 + 77
    x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    x[256:384] = 0
    for which, data in ((0, x), (1, x * x)):
        codes, scale = oc.quant(data, which)
        blocks = np.pad(np.abs(data), (0, 128 * 8 - n)).reshape(8, 128)
        assert np.array_equal(bits(scale), bits(blocks.max(axis=1)))
        unpacked = ot.unpack(torch.from_numpy(codes), n).numpy()
        assert np.array_equal(ot.pack(torch.from_numpy(unpacked), n).numpy(), codes)
        assert codes[-1] >> 4 == 0                                      # odd tail
        for b in range(8):
            seg = slice(b * 128, min((b + 1) * 128, n))
            if scale[b] == 0:
                assert not unpacked[seg].any()
                continue
            k = int(np.argmax(np.abs(data[seg])))
            assert unpacked[seg][k] == (15 if data[seg][k] > 0 else 0)
        deq = oc.dequant(codes, scale, n, which)
        codes2, scale2 = oc.quant(deq, which)
        # requantizing a dequantized state changes nothing when the block's arg-max sits on
        # +1.0 (always true for the second moment)
        if which == 1:
            assert np.array_equal(codes2, codes) and np.array_equal(bits(scale2), bits(scale))
    # all-zero block: zero state, zero grads
    p = (rng.standard_normal(256) * 0.02).astype(np.float32)
    m, v, sm, sv = _zero_state(256)
    for step in (1, 2, 3):
        oc.step_quant(p, np.zeros(256, np.float32), m, v, sm, sv, step=step, **HP)
        assert not m.any() and not v.any() and not sm.any() and not sv.any()
    assert np.all(np.signbit(oc.dequant(m, sm, 256, 0)))               # -0.8875 * 0 = -0.0


def test_unquantized_step_is_adamw():
    """With fp32 moments the step is textbook AdamW with decoupled weight decay: it must
    track torch.optim.AdamW (library routine).  The bound is set by the reference's fp32
    derived scalars: 1.0f - 0.999f is 1.3e-5 (relative) away from the 0.001 that torch
    uses, so the second moment may differ by that much and the parameters by a few 1e-6."""
    gen = torch.Generator().manual_seed(2020)
    n = 4096
    for hp in (HP, HP_DRIVER):
        p0 = torch.randn(n, generator=gen) * 0.1
        ref = torch.nn.Parameter(p0.clone())
        opt = torch.optim.AdamW([ref], lr=hp["lr"], betas=(hp["beta1"], hp["beta2"]), eps=hp["eps"],
                                weight_decay=hp["weight_decay"])
        p = p0.numpy().copy()
        m = np.zeros(n, np.float32)
        v = np.zeros(n, np.float32)
        for step in range(1, 11):
            g = torch.randn(n, generator=gen) * 1e-2
            ref.grad = g.clone()
            opt.step()
            oc.step_unquant(p, g.numpy(), m, v, step=step, **hp)
            st = opt.state[ref]
            for got, want, tol in ((p, ref.detach().numpy(), 1e-5), (m, st["exp_avg"].numpy(), 1e-6),
                                   (v, st["exp_avg_sq"].numpy(), 1e-4)):
                assert np.abs(got - want).max() <= tol * np.abs(want).max()


def test_quantized_step_tracks_adamw_like_the_reference_test():
    """The reference's only live test (tests/driver.py:28-31, :70-71): 10 steps with betas
    (0.8, 0.88), lr 5e-3, wd 0.03 stay within atol 0.025 / rtol 1e-5 of torch.optim.AdamW."""
    gen = torch.Generator().manual_seed(2020)
    n = 5000
    p0 = torch.randn(n, generator=gen) * 0.3
    ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([ref], lr=5e-3, betas=(0.8, 0.88), eps=1e-8, weight_decay=0.03)
    p = p0.numpy().copy()
    m, v, sm, sv = _zero_state(n)
    for step in range(1, 11):
        g = torch.randn(n, generator=gen)
        ref.grad = g.clone()
        opt.step()
        oc.step_quant(p, g.numpy(), m, v, sm, sv, step=step, **HP_DRIVER)
        torch.testing.assert_close(torch.from_numpy(p), ref.detach(), atol=0.025, rtol=1e-5)
    assert not np.array_equal(p, p0.numpy())


# ---------------------------------------------------------------------------
# gradient-side operations: pinned against torch's own routines on the CPU
# ---------------------------------------------------------------------------
def test_grad_norm_matches_torch_clip_grad_norm():
    gen = torch.Generator().manual_seed(11)
    for max_norm in (0.05, 1.0, 1e3):
        params = [torch.nn.Parameter(torch.zeros(n)) for n in (1, 127, 4096, 100003)]
        for p in params:
            p.grad = torch.randn(p.numel(), generator=gen) * 1e-2
        before = [p.grad.clone() for p in params]
        total = torch.nn.utils.clip_grad_norm_(params, max_norm)
        norm, coef, mult = oc.grad_norm([g.numpy() for g in before], 1.0, max_norm)
        assert abs(float(norm) - float(total)) <= 2e-6 * float(total)
        assert mult == coef
        # what the routine did to the gradients is a multiplication by the coefficient
        for p, g0 in zip(params, before):
            want = g0 * float(coef)
            assert torch.allclose(p.grad, want, rtol=3e-6, atol=0.0)
        assert (float(coef) == 1.0) == (float(total) + 1e-6 <= max_norm)


def test_grad_norm_closed_forms():
    ones = np.ones(1 << 20, np.float32)
    norm, coef, mult = oc.grad_norm([ones, ones[:3]], s=-0.5, max_norm=0.0)
    assert norm == np.float32(0.5 * np.sqrt((1 << 20) + 3)) and coef == 1.0 and mult == np.float32(-0.5)
    # bf16 bit patterns: 0x4000 = 2.0
    twos = np.full(9, 0x4000, np.uint16)
    norm, coef, mult = oc.grad_norm([twos], s=1.0, max_norm=3.0)
    assert norm == np.float32(6.0)
    assert coef == np.float32(3.0) / (np.float32(6.0) + np.float32(1e-6)) and mult == coef
    assert oc.grad_norm([np.zeros(5, np.float32)], 1.0, 1.0)[1] == 1.0      # 1 / 1e-6 clamps to 1
    n, c, _ = oc.grad_norm([np.array([np.inf], np.float32)], 1.0, 1.0)
    assert np.isinf(n) and c == 0.0
    n, c, _ = oc.grad_norm([np.array([np.nan], np.float32)], 1.0, 1.0)
    assert np.isnan(n) and np.isnan(c)


def test_scale_grad_is_unscale():
    """GradScaler.unscale_ multiplies by the fp32 reciprocal of the scale; for the power-of-two
    scales it uses that equals dividing, and for bf16 bit patterns the widening is exact."""
    gen = torch.Generator().manual_seed(12)
    g = torch.randn(5000, generator=gen)
    for scale in (65536.0, 2.0 ** 10):
        inv = torch.tensor(scale).double().reciprocal().float()
        want = (g * inv).numpy()
        assert np.array_equal(oc.scale_grad(g.numpy(), float(inv)), want)
        assert np.array_equal(want, (g / scale).numpy())
    gb = g.to(torch.bfloat16)
    got = oc.scale_grad(gb.view(torch.int16).numpy().view(np.uint16), 0.3)
    assert np.array_equal(got, (gb.float() * np.float32(0.3)).numpy())


# ---------------------------------------------------------------------------
# rank-1 scaling of the second moment
# ---------------------------------------------------------------------------
def test_rank1_quantizer_brute_force():
    """small matrices, plain Python loops: scale_ij = min(max of row i, max of column j), code =
    number of thresholds strictly below x_ij / scale_ij, 0/0 -> 0; dequantize multiplies back"""
    gen = torch.Generator().manual_seed(21)
    _, mid = oc.tables(1)
    qmap, _ = oc.tables(1)
    for rows, cols in ((1, 8), (8, 1), (5, 6), (7, 16)):
        x = torch.rand(rows, cols, generator=gen) ** 4
        x[rows // 2] = 0.0                                  # a zero row
        if cols > 2:
            x[:, 1] = 0.0                                   # a zero column
        codes, rmax, cmax = ot.quantize_rank1(x)
        un = ot.unpack(codes, rows * cols).view(rows, cols)
        back = ot.dequantize_rank1(codes, rmax, cmax)
        for i in range(rows):
            for j in range(cols):
                r = max(float(x[i, k]) for k in range(cols))
                c = max(float(x[k, j]) for k in range(rows))
                s = np.float32(min(r, c))
                assert float(rmax[i]) == r and float(cmax[j]) == c
                if s == 0:
                    want = 0
                else:
                    q = np.float32(x[i, j].item()) / s
                    want = sum(1 for t in mid if t < q)
                assert int(un[i, j]) == want, (rows, cols, i, j)
                assert float(back[i, j]) == float(np.float32(qmap[want]) * s)


def test_rank1_closed_forms():
    # one row: every column maximum is the element itself, so every non-zero element gets the
    # top code; one column likewise
    x = torch.tensor([[0.3, 0.0, 7.0, 1e-20]])
    codes, _, _ = ot.quantize_rank1(x)
    assert ot.unpack(codes, 4).tolist() == [15, 0, 15, 15]
    codes, _, _ = ot.quantize_rank1(x.t().contiguous())
    assert ot.unpack(codes, 4).tolist() == [15, 0, 15, 15]
    # outer product of powers of two a_i * b_j: scale_ij = min(a_i * max b, b_j * max a) and
    # the quotient is max(b_j / max b, a_i / max a) exactly
    a = torch.tensor([1.0, 0.5, 0.25, 0.125])
    b = torch.tensor([1.0, 0.5, 0.25, 2.0 ** -5, 2.0 ** -6, 0.125])
    x = a[:, None] * b[None, :]
    codes, rmax, cmax = ot.quantize_rank1(x)
    assert torch.equal(rmax, a) and torch.equal(cmax, b)
    q = torch.maximum((b / b.max())[None, :].expand(4, 6), (a / a.max())[:, None].expand(4, 6))
    want = torch.bucketize(q, ot.QMID[1], right=False)
    assert torch.equal(ot.unpack(codes, 24).view(4, 6), want)
    # the step on an all-zero state keeps the arg-max of every row and column at code 15
    gen = torch.Generator().manual_seed(22)
    rows, cols = 16, 128
    g = torch.randn(rows, cols, generator=gen)
    p = torch.zeros(rows, cols)
    z8 = torch.zeros(rows * cols // 2, dtype=torch.uint8)
    out = ot.step_quant_rank1(p, g, z8, z8.clone(), torch.zeros(rows * cols // 128), torch.zeros(rows),
                              torch.zeros(cols), step=1, **HP)
    vc = ot.unpack(out[2], rows * cols).view(rows, cols)
    v_new = (1 - np.float32(HP["beta2"])) * (g * g)
    assert torch.equal(out[4], v_new.amax(1)) and torch.equal(out[5], v_new.amax(0))
    # an element that is the maximum of its row or of its column has quotient >= ... 1 only
    # when it is the smaller of the two maxima; the global maximum always is
    i, j = divmod(int(v_new.argmax()), cols)
    assert int(vc[i, j]) == 15
    # m-part and parameters agree with the block-scaled step (same first moment arithmetic)
    ref = ot.step_quant(p.reshape(-1), g.reshape(-1), z8, z8.clone(), torch.zeros(rows * cols // 128),
                        torch.zeros(rows * cols // 128), step=1, **HP)
    assert torch.equal(out[1], ref[1]) and torch.equal(out[3], ref[3])
    assert torch.equal(out[0].reshape(-1), ref[0])


def test_fp16_conversions_against_numpy():
    """the C oracle's binary16 conversions against numpy's: every one of the 65536 patterns
    widened; narrowing of every pattern's value, of the midpoints between neighbouring values
    (ties go to even), of values one fp32 ulp either side of them, of the overflow boundary
    (65520 rounds to infinity) and of random fp32 bit patterns"""
    L = oc.lib()
    h = np.arange(65536, dtype=np.uint16)
    wide = h.view(np.float16).astype(np.float32)
    got = np.array([L.q4o_f16_to_f32(int(x)) for x in h], np.float32)
    nan = np.isnan(wide)
    assert np.array_equal(got[~nan].view(np.uint32), wide[~nan].view(np.uint32)) and np.isnan(got[nan]).all()
    finite = wide[np.isfinite(wide)]
    srt = np.sort(finite.astype(np.float64))
    mids = ((srt[:-1] + srt[1:]) / 2).astype(np.float32)       # exact in fp32
    rng = np.random.default_rng(3)
    rand = rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    special = np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e9, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                        np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -14, 0.0, -0.0], np.float32)
    xs = np.concatenate([finite, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
                         rand[~np.isnan(rand)], special, -special]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.q4o_f32_to_f16(float(x)) for x in xs], np.uint16)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, (xs[bad[:5]], got[bad[:5]], want[bad[:5]])
    assert (L.q4o_f32_to_f16(float("nan")) & 0x7c00) == 0x7c00 and (L.q4o_f32_to_f16(float("nan")) & 0x3ff) != 0


def test_c_and_torch_oracles_agree_on_fp16_tensors():
    """fp16 parameters and gradients through both restatements, three steps on an odd size"""
    gen = torch.Generator().manual_seed(44)
    n = 128 * 5 + 77
    p = (torch.randn(n, generator=gen) * 0.05).to(torch.float16)
    nb, nk = oc.state_sizes(n)
    pc = p.numpy().copy()
    cm, cv, csm, csv = np.zeros(nb, np.uint8), np.zeros(nb, np.uint8), np.zeros(nk, np.float32), np.zeros(nk, np.float32)
    ts = (p.clone(), torch.zeros(nb, dtype=torch.uint8), torch.zeros(nb, dtype=torch.uint8), torch.zeros(nk), torch.zeros(nk))
    for step in (1, 2, 3):
        g = (torch.randn(n, generator=gen) * 1e-3).to(torch.float16)
        oc.step_quant(pc, g.numpy(), cm, cv, csm, csv, step=step, **HP)
        ts = ot.step_quant(ts[0], g, *ts[1:], step=step, **HP)
        assert np.array_equal(cm, ts[1].numpy()) and np.array_equal(cv, ts[2].numpy())
        assert np.array_equal(csm.view(np.uint32), ts[3].numpy().view(np.uint32))
        assert np.array_equal(csv.view(np.uint32), ts[4].numpy().view(np.uint32))
        assert ts[0].dtype == torch.float16
        assert np.array_equal(pc.view(np.uint16), ts[0].numpy().view(np.uint16)), f"step {step}"


def test_rank1_nd_brute_force_and_reduction_to_matrices():
    """statistics per dimension and their broadcast minimum on small 3-D and 4-D tensors, by
    plain loops; on a matrix the N-D functions, quantizer and step, are the 2-D ones"""
    rng = np.random.default_rng(51)
    f32 = np.float32
    mid = [f32((2 * k + 1) / 32) for k in range(1, 16)]
    for shape in ((3, 4, 8), (2, 3, 2, 8), (5, 1, 16)):
        x = (np.abs(rng.standard_normal(shape)) ** 3).astype(np.float32)
        x[1] = 0.0 if len(shape) == 3 else x[1]
        x[..., 2] = 0.0
        codes, dims = ot.quantize_rank1_nd(torch.from_numpy(x))
        got = ot.unpack(codes, x.size).numpy().reshape(shape)
        back = ot.dequantize_rank1_nd(codes, dims).numpy()
        for d, st in enumerate(dims):
            want = x.max(axis=tuple(k for k in range(len(shape)) if k != d))
            assert st.shape == tuple(n if k == d else 1 for k, n in enumerate(shape))
            assert np.array_equal(st.numpy().reshape(-1), want)
        for idx in np.ndindex(*shape):
            s = min(f32(np.take(x, idx[d], axis=d).max()) for d in range(len(shape)))
            if s == 0:
                want = 0
            else:
                q = f32(x[idx] / s)
                want = sum(1 for t in mid if t < q)
            assert got[idx] == want, (shape, idx)
            assert back[idx] == f32(f32((want + 1) / 16) * s)
    m = torch.from_numpy((np.abs(rng.standard_normal((6, 24))) ** 2).astype(np.float32))
    c2, r, c = ot.quantize_rank1(m)
    cn, dims = ot.quantize_rank1_nd(m)
    assert torch.equal(c2, cn) and torch.equal(dims[0].reshape(-1), r) and torch.equal(dims[1].reshape(-1), c)
    # the step: a matrix through the N-D step equals the 2-D step, nearest and stochastic
    gen = torch.Generator().manual_seed(24)
    p, g = torch.randn(8, 128, generator=gen) * 0.02, torch.randn(8, 128, generator=gen)
    z8, zs = torch.zeros(512, dtype=torch.uint8), torch.zeros(8)
    a = ot.step_quant_rank1(p, g, z8, z8.clone(), zs, torch.zeros(8), torch.zeros(128), step=1, **HP)
    b = ot.step_quant_rank1_nd(p, g, z8, z8.clone(), zs, [torch.zeros(8, 1), torch.zeros(1, 128)], step=1, **HP)
    assert all(torch.equal(x, y) for x, y in zip(a[:4], b[:4]))
    assert torch.equal(a[4], b[4][0].reshape(-1)) and torch.equal(a[5], b[4][1].reshape(-1))
    a = ot.step_quant_rank1_sr(p, g, z8, z8.clone(), zs, torch.zeros(8), torch.zeros(128), seed=9, tensor_salt=2, step=1, **HP)
    b = ot.step_quant_rank1_nd(p, g, z8, z8.clone(), zs, [torch.zeros(8, 1), torch.zeros(1, 128)], seed=9,
                               tensor_salt=2, step=1, **HP)
    assert all(torch.equal(x, y) for x, y in zip(a[:4], b[:4]))


# ---------------------------------------------------------------------------
# stochastic rounding
# ---------------------------------------------------------------------------
def test_sr_quantizer_brute_force_and_exact_values():
    """scalar restatement with plain Python floats rounded through numpy.float32; code-book
    values themselves are never moved, whatever the noise"""
    rng = np.random.default_rng(31)
    f32 = np.float32
    for which in (0, 1):
        Q, _ = oc.tables(which)
        x = (rng.standard_normal(1024) * (0.3 if which == 0 else 1.0)).astype(np.float32)
        if which:
            x = np.abs(x)
        x[5] = 0.0
        x[128:256] = 0.0                                     # an all-zero block
        x[300] = -x[256:384].max() if which == 0 else x[300]  # the most negative value of a block
        u = ((2 * rng.integers(0, 65536, 1024) + 1) / 2.0 ** 17).astype(np.float32)
        codes, scales = ot.quantize_sr(torch.from_numpy(x), which, u)
        got = ot.unpack(codes, 1024).numpy()
        for i in range(1024):
            s = f32(np.abs(x[i // 128 * 128:(i // 128 + 1) * 128]).max())
            assert scales[i // 128] == s
            if s == 0:
                want = 0
            else:
                q = f32(x[i] / s)
                if q <= Q[0]:
                    want = 0
                elif q >= Q[15]:
                    want = 15
                else:
                    k = max(j for j in range(16) if Q[j] <= q)
                    want = k + (1 if f32(u[i] * f32(Q[k + 1] - Q[k])) < f32(q - Q[k]) else 0)
            assert got[i] == want, (which, i)
        # exact code-book values times a power-of-two scale
        blk = np.tile(Q, 8).astype(np.float32) * f32(0.25)
        codes, _ = ot.quantize_sr(torch.from_numpy(blk), which, u[:128])
        assert ot.unpack(codes, 128).tolist() == list(range(16)) * 8


def test_rank1_sr_quantizer_brute_force_and_reductions():
    """rank-1 scaling with stochastic rounding: scalar restatement on small matrices (zero
    rows and columns included); a one-row matrix reduces to 'every non-zero element gets the
    top code' whatever the noise; in the step, only the second moment's codes depend on how
    the second moment is rounded"""
    rng = np.random.default_rng(41)
    f32 = np.float32
    Q, _ = oc.tables(1)
    for rows, cols in ((3, 8), (7, 16), (16, 24)):
        x = np.abs(rng.standard_normal((rows, cols))).astype(np.float32) ** 2
        x[1, :] = 0.0                                   # a zero row
        x[:, 2] = 0.0                                   # a zero column
        u = ((2 * rng.integers(0, 65536, rows * cols) + 1) / 2.0 ** 17).astype(np.float32)
        codes, rmax, cmax = ot.quantize_rank1_sr(torch.from_numpy(x), u)
        got = ot.unpack(codes, rows * cols).numpy().reshape(rows, cols)
        assert np.array_equal(rmax.numpy(), x.max(1)) and np.array_equal(cmax.numpy(), x.max(0))
        for i in range(rows):
            for j in range(cols):
                s = min(f32(x[i].max()), f32(x[:, j].max()))
                if s == 0:
                    want = 0
                else:
                    q = f32(x[i, j] / s)
                    if q < Q[0]:
                        want = 0          # below the first entry: code -1 + 1
                    elif q >= Q[15]:
                        want = 15
                    else:
                        k = max(t for t in range(16) if Q[t] <= q)
                        want = k + (1 if f32(u[i * cols + j] * f32(Q[k + 1] - Q[k])) < f32(q - Q[k]) else 0)
                assert got[i, j] == want, (rows, cols, i, j)
    x = torch.tensor([[0.3, 0.0, 7.0, 1e-20]])
    for noise in (2.0 ** -17, 0.5, 1 - 2.0 ** -17):
        codes, _, _ = ot.quantize_rank1_sr(x, np.full(4, noise, np.float32))
        assert ot.unpack(codes, 4).tolist() == [15, 0, 15, 15]
    # the step: statistics, first moment and parameters do not depend on how the second
    # moment is rounded; the first moment's codes are those of the block-scaled SR step
    gen = torch.Generator().manual_seed(23)
    rows, cols = 16, 128
    g = torch.randn(rows, cols, generator=gen)
    p = torch.randn(rows, cols, generator=gen) * 0.02
    z8 = torch.zeros(rows * cols // 2, dtype=torch.uint8)
    zs = torch.zeros(rows * cols // 128)
    kw = dict(seed=77, tensor_salt=5, step=1, **HP)
    out = ot.step_quant_rank1_sr(p, g, z8, z8.clone(), zs, torch.zeros(rows), torch.zeros(cols), **kw)
    near = ot.step_quant_rank1(p, g, z8, z8.clone(), zs, torch.zeros(rows), torch.zeros(cols), step=1, **HP)
    sr = ot.step_quant_sr(p.reshape(-1), g.reshape(-1), z8, z8.clone(), zs, zs.clone(), **kw)
    assert torch.equal(out[0], near[0]) and torch.equal(out[4], near[4]) and torch.equal(out[5], near[5])
    assert torch.equal(out[1], sr[1]) and torch.equal(out[3], sr[3])
    a, b = ot.unpack(out[2], rows * cols), ot.unpack(near[2], rows * cols)
    assert int((a - b).abs().max()) <= 1 and bool((a != b).any())     # a neighbouring code, not always the nearest


def test_sr_is_unbiased_and_noise_is_uniform():
    um, uv = ot.sr_noise(1 << 20, ot.sr_tensor_salt(1234567890123, 7, 3))
    for u in (um, uv):
        assert u.min() >= 2.0 ** -17 and u.max() <= 1.0 - 2.0 ** -17
        assert abs(float(u.astype(np.float64).mean()) - 0.5) < 2e-3
        hist = np.histogram(u, bins=64, range=(0.0, 1.0))[0]
        assert hist.min() > 0.9 * (1 << 20) / 64 and hist.max() < 1.1 * (1 << 20) / 64
    assert abs(np.corrcoef(um, uv)[0, 1]) < 5e-3 and abs(np.corrcoef(um[:-1], um[1:])[0, 1]) < 5e-3
    # different steps, tensors and seeds draw different noise
    salts = {ot.sr_tensor_salt(s, t, k) for s in (1, 2, 1 << 40) for t in (1, 2) for k in (0, 1)}
    assert len(salts) == 12
    # the dequantized mean of many roundings of one value is that value (nearest rounding would
    # be off by up to half a gap)
    for which, x0 in ((0, 0.1234), (0, -0.5), (1, 0.4321)):
        n = 1 << 18
        x = np.full(n, x0, np.float32)
        x[::128] = 1.0                                       # every block's scale is 1
        u = ot.sr_noise(n, 99)[which]
        codes, scales = ot.quantize_sr(torch.from_numpy(x), which, u)
        back = ot.dequantize(codes, scales, n, which).numpy().astype(np.float64)
        keep = np.arange(n) % 128 != 0
        assert abs(back[keep].mean() - x0) < 2e-3 * abs(x0) + 1e-4


@pytest.mark.parametrize("which", [0, 1])
def test_quantizer_search_equals_count_on_every_fp32(which):
    """the literal search of the reference (cuda_adamw_kernels.cu:167-194) and the closed form
    the kernels use agree on all 2^32 fp32 bit patterns, NaN and infinities included; along the
    number line the code never decreases, never jumps by more than one, and steps exactly 15
    times"""
    bad, first, steps = oc.exhaustive_search_vs_count(which)
    assert bad == 0, f"{bad} patterns disagree, first {first:#010x}"
    assert steps == 15


# ---------------------------------------------------------------------------
# rank-1 scaling and stochastic rounding: the scalar C restatement against the vectorised one
# ---------------------------------------------------------------------------
def _np_elem(t):
    """torch tensor -> the numpy form the C oracle takes (bf16 as uint16 bit patterns)"""
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def _variant_inputs(rows, cols, p_dt, g_dt, seed):
    gen = torch.Generator().manual_seed(seed)
    n = rows * cols
    p = (torch.randn(rows, cols, generator=gen) * 0.05).to(p_dt)
    make = (grads_config1, grads_config3, grads_student_t)
    grads = []
    for k in range(3):
        g = make[k](gen, n).view(rows, cols).clone()
        if k == 1:
            g[rows // 2] = 0.0                      # a silent row and silent columns
            g[:, : max(1, cols // 7)] = 0.0
        if k == 2 and n > 40:
            g.view(-1)[5] = float("inf")            # non-finite gradients reach the statistics
            g.view(-1)[37] = float("nan")
        grads.append(g.to(g_dt))
    return p, grads


@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("rank1", [False, True])
@pytest.mark.parametrize("p_dt,g_dt", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                       (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16)])
@pytest.mark.parametrize("shape", [(1, 1), (3, 50), (7, 129), (40, 264), (130, 96), (5, 1031)])
def test_c_and_torch_restatements_of_the_variants_agree(shape, p_dt, g_dt, rank1, stochastic):
    """q4o_step_quant_variants (scalar loops) and step_quant / step_quant_sr / step_quant_rank1 /
    step_quant_rank1_sr (vectorised) are written apart from each other and must give the same
    bits -- codes, block scales, row and column maxima and parameters -- over three steps that
    feed back into each other, with silent rows and columns and non-finite gradients."""
    rows, cols = shape
    n = rows * cols
    p, grads = _variant_inputs(rows, cols, p_dt, g_dt, 31 * rows + cols)
    nbytes, nblk = oc.state_sizes(n)
    seed, salt = 0x1234_5678_9ABC_DEF0 ^ (rows << 40), cols % 11
    # C side (in place)
    cp = _np_elem(p)
    cm, cv = np.zeros(nbytes, np.uint8), np.zeros(nbytes, np.uint8)
    csm, csv = np.zeros(nblk, np.float32), np.zeros(nblk, np.float32)
    cr, cc = np.zeros(rows, np.float32), np.zeros(cols, np.float32)
    # torch side (functional)
    if rank1:
        ref = (p.clone(), torch.zeros(nbytes, dtype=torch.uint8), torch.zeros(nbytes, dtype=torch.uint8),
               torch.zeros(nblk), torch.zeros(rows), torch.zeros(cols))
    else:
        ref = (p.clone().reshape(-1), torch.zeros(nbytes, dtype=torch.uint8), torch.zeros(nbytes, dtype=torch.uint8),
               torch.zeros(nblk), torch.zeros(nblk))
    hp = dict(HP)
    for step, g in enumerate(grads, 1):
        kw = dict(seed=seed, tensor_salt=salt) if stochastic else {}
        if rank1:
            oc.step_quant_variants(cp, _np_elem(g), cm, cv, csm, None, cr, cc, step=step, **kw, **hp)
            fn = ot.step_quant_rank1_sr if stochastic else ot.step_quant_rank1
            ref = fn(ref[0], g, *ref[1:], step=step, **kw, **hp)
        else:
            oc.step_quant_variants(cp.reshape(-1), _np_elem(g).reshape(-1), cm, cv, csm, csv, step=step, **kw, **hp)
            fn = ot.step_quant_sr if stochastic else ot.step_quant
            ref = fn(ref[0], g.reshape(-1), *ref[1:], step=step, **kw, **hp)
        what = f"{shape} {p_dt}/{g_dt} rank1={rank1} sr={stochastic} step {step}"
        assert np.array_equal(cm, ref[1].numpy()), f"{what}: first-moment codes"
        assert np.array_equal(cv, ref[2].numpy()), f"{what}: second-moment codes"
        assert np.array_equal(bits(csm), bits(ref[3].numpy())), f"{what}: first-moment scales"
        if rank1:
            assert np.array_equal(bits(cr), bits(ref[4].numpy())), f"{what}: row maxima"
            assert np.array_equal(bits(cc), bits(ref[5].numpy())), f"{what}: column maxima"
        else:
            assert np.array_equal(bits(csv), bits(ref[4].numpy())), f"{what}: second-moment scales"
        # parameters: the same arithmetic on both sides (numpy's correctly rounded sqrt, IEEE
        # division), so the same bits; a NaN (from a non-finite gradient) is a NaN whatever its payload
        got, want = cp.reshape(-1), _np_elem(ref[0]).reshape(-1)
        as_f32 = lambda a: ((a.astype(np.uint32) << 16).view(np.float32) if a.dtype == np.uint16
                            else a.astype(np.float32))
        nan = np.isnan(as_f32(want))
        assert np.array_equal(nan, np.isnan(as_f32(got))), f"{what}: NaN parameters"
        assert np.array_equal(got[~nan].view(np.uint8), want[~nan].view(np.uint8)), f"{what}: parameters"


def test_c_variants_without_options_is_the_fused_step():
    """with neither option q4o_step_quant_variants must be q4o_step_quant, bit for bit"""
    gen = torch.Generator().manual_seed(3)
    n = 128 * 37 + 19
    p0 = (torch.randn(n, generator=gen) * 0.02).numpy()
    nbytes, nblk = oc.state_sizes(n)
    a = [p0.copy(), np.zeros(nbytes, np.uint8), np.zeros(nbytes, np.uint8), np.zeros(nblk, np.float32), np.zeros(nblk, np.float32)]
    b = [x.copy() for x in a]
    for step in range(1, 5):
        g = grads_config1(gen, n).numpy()
        oc.step_quant(a[0], g, *a[1:], step=step, **HP)
        oc.step_quant_variants(b[0], g, *b[1:], step=step, **HP)
        for x, y in zip(a, b):
            assert np.array_equal(x.view(np.uint8), y.view(np.uint8)), step


def test_c_noise_and_salt_are_the_vectorised_ones():
    for seed, step, salt in ((0, 1, 0), (2 ** 64 - 1, 123456, 2 ** 32 - 1), (0x1234_5678_9ABC_DEF0, 7, 3)):
        s = ot.sr_tensor_salt(seed, step, salt)
        assert oc.sr_tensor_salt(seed, step, salt) == s
        um, uv = ot.sr_noise(300, s)
        for e in (0, 1, 2, 17, 255, 299):
            assert oc.sr_noise(e, s) == (float(um[e]), float(uv[e]))
    # beyond 2^32 elements the high half of the index enters the hash
    e = (1 << 32) + 12345
    key = (np.uint64(e) & ot._M32) ^ np.uint64(77) ^ ((np.uint64(e >> 32) * np.uint64(0x9E3779B9)) & ot._M32)
    h = int(ot.lowbias32(key))
    assert oc.sr_noise(e, 77) == ((2 * (h >> 16) + 1) / 2 ** 17, (2 * (h & 0xFFFF) + 1) / 2 ** 17)


@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("p_dt,g_dt", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("shape", [(4, 6, 64), (3, 5, 24), (2, 3, 4, 32), (5, 1, 2, 40), (7, 33)])
def test_c_and_torch_restatements_agree_on_more_than_two_dimensions(shape, p_dt, g_dt, stochastic):
    """one statistic per dimension, scale = their minimum: q4o_step_quant_variants against
    step_quant_rank1_nd, every dimension's statistic bit for bit over three steps"""
    n = int(np.prod(shape))
    p, grads = _variant_inputs(n // shape[-1], shape[-1], p_dt, g_dt, sum(shape))
    p = p.view(shape)
    nbytes, nblk = oc.state_sizes(n)
    cp = _np_elem(p)
    cm, cv, csm = np.zeros(nbytes, np.uint8), np.zeros(nbytes, np.uint8), np.zeros(nblk, np.float32)
    cdims = [np.zeros(d, np.float32) for d in shape]
    ref = (p.clone(), torch.zeros(nbytes, dtype=torch.uint8), torch.zeros(nbytes, dtype=torch.uint8), torch.zeros(nblk),
           [torch.zeros([d if j == i else 1 for j, d in enumerate(shape)]) for i in range(len(shape))])
    kw = dict(seed=0xFEED_FACE_0000_0001, tensor_salt=9) if stochastic else {}
    for step, g in enumerate(grads, 1):
        g = g.view(shape)
        oc.step_quant_variants(cp, _np_elem(g), cm, cv, csm, max_dims=cdims, step=step, **kw, **HP)
        ref = ot.step_quant_rank1_nd(ref[0], g, *ref[1:], step=step, **kw, **HP)
        what = f"{shape} {p_dt}/{g_dt} sr={stochastic} step {step}"
        assert np.array_equal(cm, ref[1].numpy()) and np.array_equal(cv, ref[2].numpy()), f"{what}: codes"
        assert np.array_equal(bits(csm), bits(ref[3].numpy())), f"{what}: first-moment scales"
        for k, (mine, theirs) in enumerate(zip(cdims, ref[4])):
            assert np.array_equal(bits(mine), bits(theirs.reshape(-1).numpy())), f"{what}: statistic of dimension {k}"
