"""The fused step's quantizers at EVERY block-scale mantissa.

The fast path of the quantizers multiplies by a reciprocal of the block scale instead of
dividing (a Newton-refined one for block scales, the bare hardware estimate for rank-1
scales) and hands every quotient inside a guard band around a threshold to IEEE division.
The reciprocal's error depends on the scale's mantissa, so this walk takes all 2^23 of them,
at three exponents, and for each one places values on and around every threshold times the
scale: 0, +-1, 2, 3, 4, 6, 8, 12 ulps for the first moment, the squares of gradients that far
from the one whose square lands on the threshold for the second moment (second moments are
made of squares, so neighbouring reachable values are about two ulps apart).  That reaches
from inside the guard bands to well outside them, where the fast path decides on its own.

tests/test_gpu_every_quotient.py walks every value at a few scales; this file walks every
scale at the values that matter.  Expected codes: the torch oracle run on the device (IEEE
division and torch.bucketize; tests/test_gpu_full_size.py checks that run against the C
oracle), for stochastic rounding the device restatement of the oracle's rounding rule that
test_gpu_every_quotient.py checks against the oracle.

How the inputs choose the moments: beta1 = beta2 = 0.5 and step 1.  First moment: old code 7
(value 0), so the new moment is g / 2 exactly; a block's last element holds g = 2 s and pins
the scale s.  Second moment: old code 0 under an old scale 2 s gives an old value s / 8, the
new one is s / 16 + g^2 / 2; the pinned element holds old code 15 (old value 2 s) and g = 0,
which makes it exactly s.
"""
import pytest
import torch

from oracle import q4_oracle as oc
from oracle import q4_oracle_torch as ot
from quantfour_adamw_cuda_amd import quantfour_hip as qh
from tests.test_gpu_every_quotient import _packed, _sr_codes, _sr_noise

pytestmark = pytest.mark.gpu

HP = dict(beta1=0.5, beta2=0.5, lr=1e-3, weight_decay=0.0, eps=1e-8)
HPA = (0.5, 0.5, 1e-3, 0.0, 1e-8)
OFFSETS = [0, 1, -1, 2, -2, 3, -3, 4, -4, 6, -6, 8, -8, 12, -12]          # ulps, 15 per threshold
MANTISSAS = 1 << 23
SEED = 0x5EED_0F_5CA1E5


def _scales(k0, count, exponent, device):
    """count consecutive scales 2^exponent * (1 + k 2^-23), k = k0 ..."""
    bits = ((127 + exponent) << 23) + torch.arange(k0, k0 + count, device=device, dtype=torch.int32)
    return bits.view(torch.float32)


def _nudged(x, offsets):
    """x[..., None] moved by each offset in units in the last place (of its magnitude)"""
    return (x.view(torch.int32).unsqueeze(-1) + offsets).view(torch.float32)


def _first_moment_targets(s, device):
    """[K, 15, 15]: for each scale, threshold and offset the value RN(threshold * s) moved by
    the offset"""
    mid = torch.tensor(oc.tables(0)[1], device=device)
    offs = torch.tensor(OFFSETS, device=device, dtype=torch.int32)
    return _nudged(s.unsqueeze(1) * mid.unsqueeze(0), offs)


def _second_moment_gradients(s, offsets, device):
    """[K, 15, len(offsets)]: gradients g whose second moment s / 16 + g^2 / 2 lands on
    threshold * s, moved by the offsets"""
    mid = torch.tensor(oc.tables(1)[1], device=device, dtype=torch.float64)
    offs = torch.tensor(offsets, device=device, dtype=torch.int32)
    g = torch.sqrt(2.0 * s.double().unsqueeze(1) * (mid.unsqueeze(0) - 0.0625)).float()
    return _nudged(g, offs)


def _block_scaled_inputs(k0, count, exponent, device):
    """Four blocks per scale: two whose first moment walks the thresholds (8 and 7 of them),
    two whose second moment does.  Returns g, m codes, v codes, m scales, v scales (old state)
    and the scales walked."""
    s = _scales(k0, count, exponent, device)
    g = torch.zeros(count, 4, 128, device=device)
    tm = _first_moment_targets(s, device) * 2.0                              # m' = g / 2
    g[:, 0, :120] = tm[:, :8].reshape(count, 120)
    g[:, 1, :105] = tm[:, 8:].reshape(count, 105)
    g[:, 0:2, 127] = (s * 2.0).unsqueeze(1)
    tv = _second_moment_gradients(s, OFFSETS, device)
    g[:, 2, :120] = tv[:, :8].reshape(count, 120)
    g[:, 3, :105] = tv[:, 8:].reshape(count, 105)
    del tm, tv
    m_codes = torch.full((count * 4 * 64,), 0x77, dtype=torch.uint8, device=device)    # code 7: zero
    v_codes = torch.zeros(count, 4, 64, dtype=torch.uint8, device=device)
    v_codes[:, 2:4, 63] = 0xF0                                                # last element: code 15
    m_scale = torch.zeros(count * 4, device=device)
    v_scale = torch.zeros(count, 4, device=device)
    v_scale[:, 2:4] = (s * 2.0).unsqueeze(1)
    return g.reshape(-1), m_codes, v_codes.reshape(-1), m_scale, v_scale.reshape(-1), s


def _compare(name, got, want, what):
    if not torch.equal(got, want):
        bad = torch.nonzero(got != want).reshape(-1)
        i = int(bad[0])
        raise AssertionError(f"{what}: {name} differ in {bad.numel()} places; first at {i}: "
                             f"got {got[i].item()}, want {want[i].item()}")


@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("exponent", [-20, 0, 20])
def test_every_block_scale_mantissa(cuda, exponent, stochastic):
    count = 1 << 19                       # scales per launch: 2^28 elements
    for launch, k0 in enumerate(range(0, MANTISSAS, count)):
        g, m, v, sm, sv, s = _block_scaled_inputs(k0, count, exponent, cuda)
        n = g.numel()
        p = torch.zeros(n, device=cuda)
        what = f"exponent {exponent} scales from {k0} stochastic {stochastic}"
        # expected, from the state before the step
        if stochastic:
            sc = ot.derive_scalars(step=1, **{k: HP[k] for k in ("beta1", "beta2", "lr", "weight_decay")})
            _, m_new, v_new = ot.adamw_update(p, g, ot.dequantize(m, sm, n, 0), ot.dequantize(v, sv, n, 1), sc, HP["eps"])
            want_sm = m_new.abs().view(-1, 128).amax(dim=1)
            want_sv = v_new.view(-1, 128).amax(dim=1)
            um, uv = _sr_noise(n, ot.sr_tensor_salt(SEED, 1, launch), cuda)
            want_m = _packed(_sr_codes(m_new / want_sm.repeat_interleave(128), 0, um))     # no all-zero block here
            want_v = _packed(_sr_codes(v_new / want_sv.repeat_interleave(128), 1, uv))
            del m_new, v_new, um, uv
            qh.fused_4bit_multi_sr([p], [g], [m], [v], [sm], [sv], *HPA, 1, SEED, salts=[launch])
        else:
            _, want_m, want_v, want_sm, want_sv = ot.step_quant(p, g, m, v, sm, sv, step=1, **HP)
            qh.fused_4bit_multi([p], [g], [m], [v], [sm], [sv], *HPA, 1)
        # the walk is what it claims to be: the pinned elements fix the scales
        assert torch.equal(want_sm.view(-1, 4)[:, 0], s) and torch.equal(want_sm.view(-1, 4)[:, 1], s), what
        assert torch.equal(want_sv.view(-1, 4)[:, 2], s) and torch.equal(want_sv.view(-1, 4)[:, 3], s), what
        _compare("first-moment scales", sm.view(torch.int32), want_sm.view(torch.int32), what)
        _compare("second-moment scales", sv.view(torch.int32), want_sv.view(torch.int32), what)
        _compare("first-moment codes", m, want_m, what)
        _compare("second-moment codes", v, want_v, what)
        del g, m, v, sm, sv, s, p, want_m, want_v, want_sm, want_sv


# second-moment offsets for a row of 512 columns: 15 thresholds x 33 offsets = 495 values
ROW_OFFSETS = [0] + [d * sgn for d in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28, 32) for sgn in (1, -1)]
COLS = 512


@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("exponent", [-20, 0, 20])
def test_every_rank1_scale_mantissa(cuda, exponent, stochastic):
    """Rank-1 scaling: a row per scale.  Row 0 holds a large value in every column, so that
    every column maximum exceeds every row maximum and the scale of element (i, j) is row i's
    maximum; the row's first element pins that maximum.  512 columns: the update kernel whose
    workgroups share the columns' maxima of four rows."""
    rows = 1 << 19
    big_old = float(2.0 ** (exponent + 4))
    for launch, k0 in enumerate(range(0, MANTISSAS, rows - 1)):
        count = min(rows - 1, MANTISSAS - k0)
        if count < 63:                      # the last launch of the walk: keep the matrix in this kernel's range
            k0, count = MANTISSAS - 63, 63
        s = _scales(k0, count, exponent, cuda)
        g = torch.zeros(count + 1, COLS, device=cuda)
        g[1:, 1:496] = _second_moment_gradients(s, ROW_OFFSETS, cuda).reshape(count, 495)
        n = g.numel()
        p = torch.zeros(count + 1, COLS, device=cuda)
        m = torch.full((n // 2,), 0x77, dtype=torch.uint8, device=cuda)
        v = torch.zeros(count + 1, COLS // 2, dtype=torch.uint8, device=cuda)
        v[0, :] = 0xFF
        v[1:, 0] = 0x0F                                                      # first element: code 15
        v = v.reshape(-1)
        sm = torch.zeros(n // 128, device=cuda)
        r = torch.cat([torch.full((1,), big_old, device=cuda), s * 2.0])
        c = torch.full((COLS,), big_old, device=cuda)
        rn, cn = torch.zeros_like(r), torch.zeros_like(c)
        what = f"exponent {exponent} scales from {k0} stochastic {stochastic}"
        if stochastic:
            sc = ot.derive_scalars(step=1, **{k: HP[k] for k in ("beta1", "beta2", "lr", "weight_decay")})
            v_old = ot.dequantize_rank1(v, r, c).reshape(-1)
            _, m_new, v_new = ot.adamw_update(p.reshape(-1), g.reshape(-1), ot.dequantize(m, sm, n, 0), v_old, sc, HP["eps"])
            want_sm = m_new.abs().view(-1, 128).amax(dim=1)
            v_new = v_new.view(count + 1, COLS)
            want_r, want_c = v_new.amax(dim=1), v_new.amax(dim=0)
            um, uv = _sr_noise(n, ot.sr_tensor_salt(SEED, 1, launch), cuda)
            q_m = m_new / want_sm.repeat_interleave(128)                      # 0 / 0 = NaN -> code 0
            nan = torch.isnan(q_m)
            want_m = _sr_codes(torch.where(nan, torch.zeros_like(q_m), q_m), 0, um)
            want_m[nan] = 0
            want_m = _packed(want_m)
            want_v = _packed(_sr_codes((v_new / ot.rank1_scale(want_r, want_c)).reshape(-1), 1, uv))
            del v_old, m_new, v_new, um, uv, q_m, nan
        else:
            _, want_m, want_v, want_sm, want_r, want_c = ot.step_quant_rank1(p, g, m, v, sm, r, c, step=1, **HP)
        assert torch.equal(want_r[1:], s) and bool((want_c == big_old / 2).all()), what
        qh.fused_4bit_rank1_multi([p], [g], [m], [v], [sm], [r], [c], [rn], [cn], *HPA, 1,
                                  seed=SEED if stochastic else None, salts=[launch] if stochastic else None)
        _compare("row maxima", r.view(torch.int32), want_r.view(torch.int32), what)
        _compare("column maxima", c.view(torch.int32), want_c.view(torch.int32), what)
        _compare("first-moment scales", sm.view(torch.int32), want_sm.view(torch.int32), what)
        _compare("first-moment codes", m, want_m, what)
        _compare("second-moment codes", v, want_v, what)
        assert not bool(rn.any()) and not bool(cn.any()), f"{what}: scratch statistics must be zero again"
        del g, p, m, v, sm, r, c, rn, cn, s, want_m, want_v, want_sm, want_r, want_c
