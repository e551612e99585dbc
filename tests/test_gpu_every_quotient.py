"""The fused step's quantizers on EVERY fp32 value a block can hold, at several block scales.

With beta1 = beta2 = 0.5, zero state and step 1 the new first moment is exactly g / 2 and the
new second moment RN(g * g) / 2, so the gradients choose the moments: every block gets 127
enumerated values and one pinned element that fixes the block's scales.  All fp32 patterns of
magnitude up to the scale are walked (2.1e9 per scale of 1.0), which covers every quotient the
first moment's quantizer can see and the squares among the second moment's.  Expected codes:
IEEE division and torch.bucketize with right=False (the count of thresholds below the value;
tests/test_oracle_pins.py pins that form against the reference's search loop on every fp32),
with the thresholds of oracle/q4_oracle.py.  Codes and scales must agree bit for bit.

Stochastic rounding takes the same walk with one noise value per position; its expected codes
come from a torch restatement of oracle/q4_oracle_torch.py's sr_noise and sr_codes that runs
on the device (the numpy one would need minutes per scale), checked against them first."""
import numpy as np
import pytest
import torch

import quantfour_adamw_cuda_amd as q4
from oracle import q4_oracle as oc
from oracle import q4_oracle_torch as ot
from quantfour_adamw_cuda_amd import quantfour_hip as qh

pytestmark = pytest.mark.gpu

BLOCKS_PER_CHUNK = 1 << 21          # 2^28 elements per launch


def _bits(x):
    return int(np.float32(x).view(np.uint32))


def _enumerated_gradients(start, per_sign, pin, cuda):
    """One launch's gradients: 127 values 2 x per block, x walking the patterns start ..., and
    the pinned element last."""
    chunk = BLOCKS_PER_CHUNK * 127
    idx = torch.arange(start, start + chunk, device=cuda, dtype=torch.int64)
    idx = torch.where(idx < 2 * per_sign, idx, torch.zeros_like(idx))         # tail: zeros
    pat = torch.where(idx < per_sign, idx, (idx - per_sign) | 0x80000000)
    x = (pat - ((pat >> 31) << 32)).to(torch.int32).view(torch.float32)      # the pattern as two's complement
    return torch.cat([(x * 2.0).view(-1, 127), torch.full((BLOCKS_PER_CHUNK, 1), pin, device=cuda)], dim=1).reshape(-1)


def _packed(codes):
    codes = codes.to(torch.uint8)
    return codes[0::2] | (codes[1::2] << 4)


# pinned gradient -> first-moment scale pin / 2: an exact reciprocal (1.0), inexact ones, a small one
@pytest.mark.parametrize("pin", [2.0, 3.0, 1.3333334, 0.0033203125])
def test_every_value_of_a_block(cuda, pin):
    pin = float(np.float32(pin))
    am = float(np.float32(pin) * np.float32(0.5))
    av = float(np.float32(0.5) * (np.float32(pin) * np.float32(pin)))
    mid_m = torch.tensor(oc.tables(0)[1], device=cuda)
    mid_v = torch.tensor(oc.tables(1)[1], device=cuda)
    per_sign = _bits(am) + 1                      # patterns 0 .. bits(am): every 0 <= x <= am
    total = 2 * per_sign
    chunk = BLOCKS_PER_CHUNK * 127
    n = BLOCKS_PER_CHUNK * 128
    p = torch.zeros(n, device=cuda)
    m = torch.zeros(n // 2, dtype=torch.uint8, device=cuda)
    v = torch.zeros_like(m)
    sm = torch.zeros(n // 128, device=cuda)
    sv = torch.zeros_like(sm)
    for start in range(0, total, chunk):
        g = _enumerated_gradients(start, per_sign, pin, cuda)
        p.zero_(); m.zero_(); v.zero_(); sm.zero_(); sv.zero_()
        q4.fused_4bit(p, g, m, v, sm, sv, 0.5, 0.5, 1e-3, 0.0, 1e-8, 1)
        assert bool((sm == am).all()) and bool((sv == av).all()), f"pin {pin} chunk {start}: scales"
        for name, codes, new, scale, mid in (("first", m, g * 0.5, am, mid_m), ("second", v, (g * g) * 0.5, av, mid_v)):
            # a device tensor as divisor: torch divides by a host scalar through its reciprocal
            want = _packed(torch.bucketize(new / torch.full((1,), scale, device=cuda), mid, right=False))
            bad = torch.nonzero(codes != want).reshape(-1)
            if bad.numel():
                e = int(bad[0]) * 2
                raise AssertionError(f"pin {pin} chunk {start}: {name}-moment codes differ in {bad.numel()} bytes; first at "
                                     f"element {e}: g = {g[e:e + 2].tolist()}, got byte {int(codes[bad[0]])}, want {int(want[bad[0]])}")
            del want, bad
        del g


_M32 = 0xFFFFFFFF


def _lowbias32(x):
    """oracle/q4_oracle_torch.py lowbias32 on int64 tensors holding 32-bit values (a product's
    low 32 bits survive the wrap of int64)."""
    x = x ^ (x >> 16)
    x = (x * 0x7FEB352D) & _M32
    x = x ^ (x >> 15)
    x = (x * 0x846CA68B) & _M32
    return x ^ (x >> 16)


def _sr_noise(numel, salt, device):
    e = torch.arange(numel, device=device, dtype=torch.int64)
    h = _lowbias32((e & _M32) ^ salt ^ (((e >> 32) * 0x9E3779B9) & _M32))
    to_u = lambda k: (2 * k + 1).to(torch.float32) * 2.0 ** -17                # exact: 17-bit integers
    return to_u(h >> 16), to_u(h & 0xFFFF)


def _sr_codes(q, which, noise):
    Q = torch.tensor(oc.tables(which)[0], device=q.device)
    k_raw = torch.searchsorted(Q, q, right=True)                              # code-book values <= q
    big = torch.tensor([torch.finfo(torch.float32).max], device=q.device)
    lower = torch.cat([-big, Q])
    gap = torch.cat([torch.zeros(1, device=q.device), Q[1:] - Q[:-1], torch.full((1,), float("inf"), device=q.device)])
    d = q - lower[k_raw]
    t = noise * gap[k_raw]
    return (k_raw - 1 + (t < d)).clamp(0, 15)


def test_device_restatement_of_the_rounding_matches_the_oracle(cuda):
    n = (1 << 20) + 3
    salt = ot.sr_tensor_salt(99, 4, 17)
    um, uv = _sr_noise(n, salt, cuda)
    rm, rv = ot.sr_noise(n, salt)
    assert np.array_equal(um.cpu().numpy(), rm) and np.array_equal(uv.cpu().numpy(), rv)
    gen = torch.Generator().manual_seed(3)
    for which, x in ((0, torch.rand(n, generator=gen) * 2.2 - 1.1), (1, torch.rand(n, generator=gen) * 1.1)):
        x[:32] = torch.tensor(oc.tables(which)[0]).repeat(2)                      # code-book values themselves
        want = ot.sr_codes(x.numpy(), which, (rm, rv)[which])
        got = _sr_codes(x.to(cuda), which, (um, uv)[which]).cpu().numpy()
        assert np.array_equal(got, want), f"moment {which}"


@pytest.mark.parametrize("pin", [2.0, 3.0, 1.3333334, 0.0033203125])
def test_every_value_of_a_block_stochastic(cuda, pin):
    pin = float(np.float32(pin))
    am = float(np.float32(pin) * np.float32(0.5))
    av = float(np.float32(0.5) * (np.float32(pin) * np.float32(pin)))
    per_sign = _bits(am) + 1
    total = 2 * per_sign
    chunk = BLOCKS_PER_CHUNK * 127
    n = BLOCKS_PER_CHUNK * 128
    p = torch.zeros(n, device=cuda)
    m = torch.zeros(n // 2, dtype=torch.uint8, device=cuda)
    v = torch.zeros_like(m)
    sm = torch.zeros(n // 128, device=cuda)
    sv = torch.zeros_like(sm)
    seed = 0x0123_4567_89AB_CDEF
    for launch, start in enumerate(range(0, total, chunk)):
        g = _enumerated_gradients(start, per_sign, pin, cuda)
        p.zero_(); m.zero_(); v.zero_(); sm.zero_(); sv.zero_()
        # step 1 every time (zero state); the launches differ in their salt
        qh.fused_4bit_multi_sr([p], [g], [m], [v], [sm], [sv], 0.5, 0.5, 1e-3, 0.0, 1e-8, 1, seed, salts=[launch])
        assert bool((sm == am).all()) and bool((sv == av).all()), f"pin {pin} chunk {start}: scales"
        noise = _sr_noise(n, ot.sr_tensor_salt(seed, 1, launch), cuda)
        for which, name, codes, new, scale in ((0, "first", m, g * 0.5, am), (1, "second", v, (g * g) * 0.5, av)):
            want = _packed(_sr_codes(new / torch.full((1,), scale, device=cuda), which, noise[which]))
            bad = torch.nonzero(codes != want).reshape(-1)
            if bad.numel():
                e = int(bad[0]) * 2
                raise AssertionError(f"pin {pin} chunk {start}: {name}-moment codes differ in {bad.numel()} bytes; first at "
                                     f"element {e}: g = {g[e:e + 2].tolist()}, got byte {int(codes[bad[0]])}, want {int(want[bad[0]])}")
            del want, bad
        del g, noise


ROWS = 1 << 16


# 4096 columns: rows of whole tiles, the kernel whose workgroups share the columns' maxima of
# four rows; 4104: the kernel whose tiles run across row ends
@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("pin,COLS", [(2.0, 4096), (3.0, 4096), (1.3333334, 4096), (3.0, 4104)])
def test_every_square_under_rank1_scaling(cuda, pin, COLS, stochastic):
    """Rank-1 scaling divides by min(row maximum, column maximum) per element, through an
    unrefined hardware reciprocal in the fast path.  A matrix whose first row and first column
    hold the pinned gradient has every row and column maximum equal, so the interior walks
    every fp32 gradient 0 <= g <= pin (the second moment sees every square) at one scale.  The
    first moment keeps its block scales, which vary here; it is checked as well."""
    pin = float(np.float32(pin))
    av = float(np.float32(0.5) * (np.float32(pin) * np.float32(pin)))
    mid_m = torch.tensor(oc.tables(0)[1], device=cuda)
    mid_v = torch.tensor(oc.tables(1)[1], device=cuda)
    count = _bits(pin) + 1
    inner = (ROWS - 1) * (COLS - 1)
    n = ROWS * COLS
    p = torch.zeros(ROWS, COLS, device=cuda)
    m = torch.zeros(n // 2, dtype=torch.uint8, device=cuda)
    v = torch.zeros_like(m)
    sm = torch.zeros(n // 128, device=cuda)
    r, rn = torch.zeros(ROWS, device=cuda), torch.zeros(ROWS, device=cuda)
    c, cn = torch.zeros(COLS, device=cuda), torch.zeros(COLS, device=cuda)
    seed = 0x0FED_CBA9_8765_4321
    for launch, start in enumerate(range(0, count, inner)):
        idx = torch.arange(start, start + inner, device=cuda, dtype=torch.int64)
        idx = torch.where(idx < count, idx, torch.zeros_like(idx))
        g = torch.full((ROWS, COLS), pin, device=cuda)
        g[1:, 1:] = idx.to(torch.int32).view(torch.float32).view(ROWS - 1, COLS - 1)
        del idx
        p.zero_(); m.zero_(); v.zero_(); sm.zero_(); r.zero_(); c.zero_()
        qh.fused_4bit_rank1_multi([p], [g], [m], [v], [sm], [r], [c], [rn], [cn], 0.5, 0.5, 1e-3, 0.0, 1e-8, 1,
                                  seed=seed if stochastic else None, salts=[launch] if stochastic else None)
        what = f"pin {pin} launch {launch}"
        assert bool((r == av).all()) and bool((c == av).all()), f"{what}: row / column maxima"
        assert not bool(rn.any()) and not bool(cn.any()), f"{what}: scratch statistics must be zero again"
        flat = g.reshape(-1)
        m_new = flat * 0.5
        m_scale = m_new.abs().view(-1, 128).amax(dim=1)
        assert torch.equal(sm, m_scale), f"{what}: first-moment scales"
        q_m = m_new / m_scale.repeat_interleave(128)                     # 0 / 0 = NaN -> code 0
        q_v = ((flat * flat) * 0.5) / torch.full((1,), av, device=cuda)
        if stochastic:
            um, uv = _sr_noise(n, ot.sr_tensor_salt(seed, 1, launch), cuda)
            nan = torch.isnan(q_m)
            want_m = _sr_codes(torch.where(nan, torch.zeros_like(q_m), q_m), 0, um)
            want_m[nan] = 0
            want_v = _sr_codes(q_v, 1, uv)
            del um, uv
        else:
            want_m = torch.bucketize(q_m, mid_m, right=False)
            want_m[torch.isnan(q_m)] = 0
            want_v = torch.bucketize(q_v, mid_v, right=False)
        for name, codes, want in (("first", m, _packed(want_m)), ("second", v, _packed(want_v))):
            bad = torch.nonzero(codes != want).reshape(-1)
            if bad.numel():
                e = int(bad[0]) * 2
                raise AssertionError(f"{what}: {name}-moment codes differ in {bad.numel()} bytes; first at element {e}: "
                                     f"g = {flat[e:e + 2].tolist()}, got byte {int(codes[bad[0]])}, want {int(want[bad[0]])}")
        del g, flat, m_new, q_m, q_v, want_m, want_v


@pytest.mark.parametrize("which", [0, 1])
def test_every_value_through_the_checkpoint_quantizer(cuda, which):
    """q4adamw_quantize (checkpoint interchange: exact division, one wave per block) on every
    fp32 value of magnitude up to a block scale of 1.5; the second moment's values are not
    negative."""
    scale = 1.5
    mid = torch.tensor(oc.tables(which)[1], device=cuda)
    per_sign = _bits(scale) + 1
    total = per_sign if which else 2 * per_sign
    chunk = BLOCKS_PER_CHUNK * 127
    for start in range(0, total, chunk):
        idx = torch.arange(start, start + chunk, device=cuda, dtype=torch.int64)
        idx = torch.where(idx < total, idx, torch.zeros_like(idx))
        pat = torch.where(idx < per_sign, idx, (idx - per_sign) | 0x80000000)
        x = (pat - ((pat >> 31) << 32)).to(torch.int32).view(torch.float32)
        x = torch.cat([x.view(-1, 127), torch.full((BLOCKS_PER_CHUNK, 1), scale, device=cuda)], dim=1).reshape(-1)
        del idx, pat
        codes, scales = qh.quantize_state(x, which)
        assert bool((scales == scale).all()), f"moment {which} chunk {start}: scales"
        want = _packed(torch.bucketize(x / torch.full((1,), scale, device=cuda), mid, right=False))
        bad = torch.nonzero(codes != want).reshape(-1)
        assert bad.numel() == 0, (f"moment {which} chunk {start}: codes differ in {bad.numel()} bytes; first at element "
                                  f"{int(bad[0]) * 2}: got byte {int(codes[bad[0]])}, want {int(want[bad[0]])}")
        del x, codes, scales, want, bad


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_every_16bit_gradient(cuda, dt):
    """Parameters and gradients both in a 16-bit type take the kernel that owns eight elements
    per lane (a block is sixteen lanes).  Its gradients have only 2^16 patterns: all of them up
    to the pinned one, at 48 pinned values, with nearest and with stochastic rounding."""
    mid_m = torch.tensor(oc.tables(0)[1], device=cuda)
    mid_v = torch.tensor(oc.tables(1)[1], device=cuda)
    gen = torch.Generator().manual_seed(8)
    pins = (torch.rand(48, generator=gen) * 3.9 + 0.05).to(dt)
    for launch, pin_t in enumerate(pins):
        top = int(pin_t.view(torch.int16))                       # positive: the pattern as an integer
        pat = torch.cat([torch.arange(0, top + 1), torch.arange(0, top + 1) - 32768]).to(torch.int16)
        pad = (-pat.numel()) % 127
        x = torch.cat([pat, torch.zeros(pad, dtype=torch.int16)]).view(dt).to(cuda)
        blocks = x.numel() // 127
        g = torch.cat([x.view(-1, 127), pin_t.to(cuda).expand(blocks, 1)], dim=1).reshape(-1).contiguous()
        n = g.numel()
        gf = g.float()
        m_new, v_new = gf * 0.5, (gf * gf) * 0.5
        am, av = m_new.abs().max().reshape(1), v_new.max().reshape(1)
        for stochastic in (False, True):
            p = torch.zeros(n, dtype=dt, device=cuda)
            m = torch.zeros(n // 2, dtype=torch.uint8, device=cuda)
            v = torch.zeros_like(m)
            sm = torch.zeros(n // 128, device=cuda)
            sv = torch.zeros_like(sm)
            what = f"{dt} pin {float(pin_t)} stochastic {stochastic}"
            if stochastic:
                qh.fused_4bit_multi_sr([p], [g], [m], [v], [sm], [sv], 0.5, 0.5, 1e-3, 0.0, 1e-8, 1, 31, salts=[launch])
                um, uv = _sr_noise(n, ot.sr_tensor_salt(31, 1, launch), cuda)
                want_m, want_v = _sr_codes(m_new / am, 0, um), _sr_codes(v_new / av, 1, uv)
            else:
                q4.fused_4bit(p, g, m, v, sm, sv, 0.5, 0.5, 1e-3, 0.0, 1e-8, 1)
                want_m = torch.bucketize(m_new / am, mid_m, right=False)
                want_v = torch.bucketize(v_new / av, mid_v, right=False)
            assert bool((sm == am).all()) and bool((sv == av).all()), f"{what}: scales"
            assert torch.equal(m, _packed(want_m)), f"{what}: first-moment codes"
            assert torch.equal(v, _packed(want_v)), f"{what}: second-moment codes"
