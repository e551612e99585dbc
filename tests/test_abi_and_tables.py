"""CPU-side checks of the shipped library (no GPU work): it loads, exports every symbol
the header declares, its host-only helpers agree with the oracle, and the first-moment
bucket table has the properties the kernel's fast path relies on.  A numpy model of the
fast path shows that every code it decides on its own equals the exact code."""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import q4_oracle as oc
from quantfour_adamw_cuda_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "q4adamw.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(q4adamw_\w+)\s*\(", header))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(raw, name), name
    assert lib.q4adamw_version() >= 1000
    assert lib.q4adamw_last_error() is not None


def test_probe_library_exports_every_declared_symbol():
    """libq4probe.so (the bench's memory-system probes) against include/q4probe.h; its
    argument checks answer before any GPU call"""
    from quantfour_adamw_cuda_amd import build
    header = open(os.path.join(ROOT, "include", "q4probe.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(q4probe_\w+)\s*\(", header))
    assert declared == {"q4probe_copy", "q4probe_read", "q4probe_step_streams"}
    P = ctypes.CDLL(build.PROBE_LIB)
    for name in declared:
        assert hasattr(P, name), name
    vp, u64 = ctypes.c_void_p, ctypes.c_uint64
    P.q4probe_copy.argtypes = [vp, vp, u64, vp]
    P.q4probe_step_streams.argtypes = [vp, vp, vp, vp, vp, vp, u64, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp]
    assert P.q4probe_copy(None, None, 16, None) == -1
    assert P.q4probe_copy(16, 32, 8, None) == -1                 # bytes not a multiple of 16
    assert P.q4probe_step_streams(16, 16, 4, 4, 4, 4, 2048, 0, 7, 3, None) == -1
    assert P.q4probe_step_streams(16, 16, 4, 4, 4, 4, 2048, 0, 1, 4, None) == -1        # streams mask


def test_struct_layouts_match_header():
    assert ctypes.sizeof(_lib.Q4Tensor) == 56 and ctypes.sizeof(_lib.Q4SmallTensor) == 40
    assert _lib.Q4Tensor.numel.offset == 48 and _lib.Q4SmallTensor.numel.offset == 32
    assert ctypes.sizeof(_lib.Q4Rank1Tensor) == 168 and _lib.Q4Rank1Tensor.rows.offset == 72
    assert ctypes.sizeof(_lib.Q4GradOptions) == 40 and _lib.Q4GradOptions.grad_scale_dev.offset == 8
    assert _lib.Q4GradOptions.update_form.offset == 32
    assert (_lib.UPDATE_AUTO, _lib.UPDATE_EXACT, _lib.UPDATE_FOLDED) == (0, 1, 2)
    assert ctypes.sizeof(_lib.Q4Grad) == 16 and _lib.NORM_WORKSPACE_BYTES == 16384
    header = open(os.path.join(ROOT, "include", "q4adamw.h")).read()
    assert "#define Q4ADAMW_NORM_WORKSPACE_BYTES 16384" in header
    for name, value in (("AUTO", 0), ("EXACT", 1), ("FOLDED", 2)):
        assert f"#define Q4ADAMW_UPDATE_{name} {value}" in header


def test_grids_of_a_batch_and_the_test_hook(lib):
    """a batch beyond one grid (HIP: gridDim.x * blockDim.x < 2^32) is dealt to several grids;
    q4adamw_set_grid_limit lowers the grid size so that tests can cross the boundary"""
    u64 = ctypes.c_uint64
    bases, counts = (u64 * 8)(), (u64 * 8)()
    limit = (1 << 24) - 8

    def plan(chunks, threads=256):
        n = lib.q4adamw_grid_plan(chunks, threads, bases, counts, 8)
        return [(bases[k], counts[k]) for k in range(min(max(n, 0), 8))] if n >= 0 else n

    assert plan(0) == [] and plan(1) == [(0, 1)] and plan(limit) == [(0, limit)]
    assert plan(limit + 1) == [(0, limit), (limit, 1)]
    assert plan((1 << 24) + 1) == [(0, limit), (limit, 9)]
    assert plan(1 << 20, threads=1024) == [(0, 1 << 20)]
    assert plan((1 << 22) - 7, threads=1024) == [(0, (1 << 22) - 8), ((1 << 22) - 8, 1)]
    assert plan(3 * limit + 5) == [(0, limit), (limit, limit), (2 * limit, limit), (3 * limit, 5)]
    assert plan(0x7ffffff1) == _lib.load().q4adamw_grid_plan(0x7ffffff1, 256, bases, counts, 8) == -4
    try:
        lib.q4adamw_set_grid_limit(1000)
        assert plan(2500) == [(0, 1000), (1000, 1000), (2000, 500)]
        lib.q4adamw_set_grid_limit(1001)            # rounded down to a multiple of 8
        assert plan(2500) == [(0, 1000), (1000, 1000), (2000, 500)]
    finally:
        lib.q4adamw_set_grid_limit(0)
    assert plan(2500) == [(0, 2500)]


def test_rank1_kernel_form_by_shape(lib):
    """rows form for the Llama shapes, wide for ragged rows, narrow below a tile; a matrix of more
    than 2^32 elements whose rows are no whole number of tiles leaves the rows form (a tile
    there could straddle a multiple of 2^32, where the noise key's high half changes)"""
    form = lib.q4adamw_rank1_form
    assert form(4096, 4096, 0) == 0 and form(128256, 4096, 1) == 0 and form(4096, 14336, 0) == 0
    assert form(4096, 4480, 1) == 0                 # last tile 384 of 512: an 11th of the row idle... within a 16th
    assert form(100, 520, 0) == 1 and form(32, 4096, 0) == 1 and form(4096, 11008 + 8, 1) == 1
    assert form(1000, 248, 0) == 2 and form(1000, 504, 1) == 2 and form(1000, 504, 0) == 1
    big_rows = (1 << 32) // 4480 + 2
    assert form(big_rows, 4480, 1) == 1 and form(big_rows - 3, 4480, 1) == 0      # just above / below 2^32 elements
    assert form((1 << 32) // 4096 + 4, 4096, 1) == 0                              # whole tiles: aligned anyway
    assert form(100, 521, 0) == 3 and form(100, 12, 0) == 3 and form(5000, 2, 1) == 3 and form(64, 50257, 1) == 3
    assert form(0, 16, 0) == -1 and form(8, 1 << 31, 0) == -1


def test_new_entry_points_validate_before_any_gpu_call(lib):
    z = ctypes.c_void_p(0)
    hp = (0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0)
    t = (_lib.Q4Tensor * 1)()
    t[0].numel = 128
    assert lib.q4adamw_fused_4bit_multi_sr(t, 1, None, 7, 0, 0, *hp, None, z) == -1      # null pointers
    assert lib.q4adamw_fused_4bit_multi_ex(t, 1, 0, 5, *hp, None, z) == -1               # dtype tag
    r = (_lib.Q4Rank1Tensor * 1)()
    r[0].rows, r[0].cols = 4, 1
    assert lib.q4adamw_fused_4bit_rank1_multi(r, 1, 0, 0, *hp, None, z) == -1 and b"columns" in lib.q4adamw_last_error()
    r[0].rows, r[0].cols = 4, 500                                                        # any row length is taken: next check
    assert lib.q4adamw_fused_4bit_rank1_multi(r, 1, 0, 0, *hp, None, z) == -1 and b"null" in lib.q4adamw_last_error()
    r[0].rows, r[0].cols = 1 << 20, (1 << 12) + 4                                        # ... below 2^32 elements
    assert lib.q4adamw_fused_4bit_rank1_multi(r, 1, 0, 0, *hp, None, z) == -4 and b"2^32" in lib.q4adamw_last_error()
    r[0].cols = 1 << 31
    assert lib.q4adamw_fused_4bit_rank1_multi(r, 1, 0, 0, *hp, None, z) == -4
    r[0].rows, r[0].cols = 0, 512                                                        # empty: nothing to do
    assert lib.q4adamw_fused_4bit_rank1_multi(r, 1, 0, 0, *hp, None, z) == 0
    g = (_lib.Q4Grad * 1)()
    g[0].numel = 16
    assert lib.q4adamw_grad_norm(g, 1, 0, 1.0, None, 0.0, z, 16384, z, z) == -1
    assert lib.q4adamw_quantize_rank1(z, 4, 12, z, z, z, z) == -1 and b"null" in lib.q4adamw_last_error()
    assert lib.q4adamw_quantize_rank1(z, -4, 12, z, z, z, z) == -1 and b"negative" in lib.q4adamw_last_error()
    assert lib.q4adamw_dequantize_rank1(z, z, z, 0, 512, z, z) == 0
    # hyper-parameter domain, shared by every step entry point
    t[0].numel = 0
    assert lib.q4adamw_fused_4bit_multi_sr(t, 1, None, 7, 0, 0, 0.9, 1.0, 1e-3, 0.01, 1e-8, 1.0, None, z) == -3
    assert lib.q4adamw_sr_tensor_salt(0, 1.0, 0) != lib.q4adamw_sr_tensor_salt(0, 2.0, 0)


def test_host_helpers_match_oracle(lib):
    f = ctypes.c_float
    for which in (0, 1):
        qmap, qmid = (f * 16)(), (f * 15)()
        lib.q4adamw_tables(which, qmap, qmid)
        o_map, o_mid = oc.tables(which)
        assert np.array_equal(np.array(qmap[:], np.float32).view(np.uint32), o_map.view(np.uint32))
        assert np.array_equal(np.array(qmid[:], np.float32).view(np.uint32), o_mid.view(np.uint32))
    out = (f * 6)()
    for b1, b2, lr, wd in [(0.9, 0.999, 1e-3, 0.01), (0.8, 0.88, 5e-3, 0.03)]:
        for t in (1, 2, 7, 100, 2000):
            lib.q4adamw_derive_scalars(b1, b2, lr, wd, float(t), out)
            want = oc.derive_scalars(b1, b2, lr, wd, t)
            assert np.array_equal(np.array(out[:], np.float32).view(np.uint32), want.view(np.uint32))


def test_argument_errors_need_no_gpu(lib):
    """Validation happens before any HIP call."""
    z = ctypes.c_void_p(0)
    rc = lib.q4adamw_fused_4bit(z, z, z, z, z, z, 128, 0, 0, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, z)
    assert rc == -1 and b"null" in lib.q4adamw_last_error()
    rc = lib.q4adamw_fused_4bit(z, z, z, z, z, z, 0, 0, 0, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, z)
    assert rc == 0                                            # empty tensor: nothing to do
    rc = lib.q4adamw_fused_4bit(z, z, z, z, z, z, 128, 0, 7, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, z)
    assert rc == -1 and b"dtype" in lib.q4adamw_last_error()
    rc = lib.q4adamw_fused_4bit(z, z, z, z, z, z, 128, 0, 0, 1.5, 0.999, 1e-3, 0.01, 1e-8, 1.0, z)
    assert rc == -3
    rc = lib.q4adamw_fused_4bit(z, z, z, z, z, z, 128, 0, 0, 0.9, 0.999, 1e-3, 0.01, 1e-8, 0.0, z)
    assert rc == -3                                           # step counts from 1
    a, odd = ctypes.c_void_p(0x1004), ctypes.c_void_p(0x1002)   # fp32 tensors two bytes off
    rc = lib.q4adamw_fused_4bit(odd, a, a, a, a, a, 128, 0, 0, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, z)
    assert rc == -2 and b"element size" in lib.q4adamw_last_error()
    rc = lib.q4adamw_fused_4bit(a, odd, a, a, a, a, 128, 0, 0, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, z)
    assert rc == -2 and b"element size" in lib.q4adamw_last_error()
    rc = lib.q4adamw_fused_4bit(a, a, a, a, odd, a, 128, 0, 0, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, z)
    assert rc == -2 and b"4-byte aligned" in lib.q4adamw_last_error()
    rc = lib.q4adamw_fused_single_tensor(z, z, z, z, 16, 0, 0, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, z)
    assert rc == -1
    assert lib.q4adamw_mtable_entry(4096, (ctypes.c_uint32 * 2)()) == -1
    assert lib.q4adamw_release() == 0


# ---------------------------------------------------------------------------
# bucket table
# ---------------------------------------------------------------------------
GUARD_ULPS = 6
NO_THR = 0x7F000000


def _table(lib):
    out = (ctypes.c_uint32 * 2)()
    lo = np.zeros(2048, np.uint32)
    hi = np.zeros(2048, np.uint32)
    for i in range(2048):
        assert lib.q4adamw_mtable_entry(i, out) == 0
        lo[i], hi[i] = out[0], out[1]
    return lo, hi


def test_bucket_table_properties(lib):
    lo, hi = _table(lib)
    _, mid = oc.tables(0)
    mid_bits = mid.view(np.uint32)
    with_thr = np.flatnonzero(hi != NO_THR)
    assert with_thr.size == 15
    # every bucket that holds a threshold is one the kernel's 256-entry table carries
    held = {lib.q4adamw_mtable_half_bucket(h) for h in range(256)}
    assert set(with_thr.tolist()) <= held
    seen = []
    for i in range(2048):
        sign, mag = i >> 10, i & 1023
        base = int(lo[i] & 15)
        b_lo = np.uint32(mag << 21).view(np.float32)
        if mag >> 2 >= 255:
            continue                                           # inf / nan patterns
        b_hi = np.uint32((mag + 1) << 21).view(np.float32)
        # any value of the bucket
        probe = np.float32(-b_lo if sign else b_lo)
        exact = oc.quantize_count(0, probe)
        if hi[i] == NO_THR:
            assert (lo[i] & ~np.uint32(15)) == NO_THR
            assert base == exact, (i, base, exact)
            continue
        # exactly one threshold inside, at least 64 ulps away from both bucket edges
        inside = [j for j in range(15) if (b_lo <= mid[j] < b_hi if not sign else -b_hi < mid[j] < -b_lo)]
        assert len(inside) == 1
        j = inside[0]
        seen.append(j)
        m = int(mid_bits[j] & 0x7FFFFFFF)
        assert m - (mag << 21) >= 64 and ((mag + 1) << 21) - m >= 64
        assert base == sum(1 for k in range(15) if mid[k] < mid[j])
        lo_mag, hi_mag = int(lo[i] & 0x7FFFFFFF), int(hi[i] & 0x7FFFFFFF)
        if not sign:
            assert GUARD_ULPS <= m - lo_mag <= GUARD_ULPS + 15 and hi_mag - m == GUARD_ULPS
        else:
            assert GUARD_ULPS <= lo_mag - m <= GUARD_ULPS + 15 and m - hi_mag == GUARD_ULPS
            assert lo[i] >> 31 == 1 and hi[i] >> 31 == 1
    assert sorted(seen) == list(range(15))


def _half_index(q):
    """High byte of q converted to half precision toward zero (what v_cvt_pkrtz_f16_f32
    leaves in bits 8..15 / 24..31), for finite |q| < 65536: truncate, then convert exactly."""
    q = np.asarray(q, np.float32)
    bits = q.view(np.uint32)
    normal = (bits & np.uint32(0xFFFFE000)).view(np.float32)               # keep 10 mantissa bits
    tiny = (np.trunc(q.astype(np.float64) * 2.0 ** 24) / 2.0 ** 24).astype(np.float32)
    tz = np.where(np.abs(q) >= np.float32(2.0 ** -14), normal, tiny)
    h = tz.astype(np.float16).view(np.uint16)
    assert np.array_equal(h.view(np.float16).astype(np.float32), tz)       # the conversion was exact
    return (h >> 8).astype(np.int64) | np.where(np.signbit(q), 0x80, 0)    # -0.0 keeps its sign


def test_half_index_names_the_same_entry(lib):
    """The kernel indexes 256 entries by the high byte of the quotient as a half (round toward
    zero); that entry must be the one the top eleven fp32 bits select in the full table, for
    every magnitude a quotient can take (the approximate quotient never exceeds 1 by more than
    a few ulps) and far beyond."""
    lo, hi = _table(lib)
    bucket_of = np.array([lib.q4adamw_mtable_half_bucket(h) for h in range(256)])
    assert lib.q4adamw_mtable_half_bucket(256) < 0
    rng = np.random.default_rng(5)
    mag = np.concatenate([
        10.0 ** rng.uniform(-44, 4.5, 200000),
        2.0 ** np.arange(-30, 16, dtype=np.float64),                       # bucket edges
        np.nextafter((2.0 ** np.arange(-30, 16)).astype(np.float32), np.float32(0)).astype(np.float64),
        [0.0, 1.0, 1.0 + 2 ** -22, 65504.0, 65535.0],
    ]).astype(np.float32)
    # all four mantissa quarters of every exponent, and their lower neighbours
    quarters = (2.0 ** np.arange(-20, 3))[:, None] * np.array([1.0, 1.25, 1.5, 1.75])[None, :]
    q32 = quarters.astype(np.float32).ravel()
    mag = np.concatenate([mag, q32, np.nextafter(q32, np.float32(0))])
    q = np.concatenate([mag, -mag])
    full = (q.view(np.uint32) >> 21).astype(np.int64)
    via_half = bucket_of[_half_index(q)]
    assert np.array_equal(lo[via_half], lo[full]) and np.array_equal(hi[via_half], hi[full])
    # the buckets themselves coincide wherever the half is normal
    normal = np.abs(q) >= np.float32(2.0 ** -14)
    assert np.array_equal(via_half[normal], full[normal])


def _nudge(x, d):
    """array of fp32 moved by d ulps in magnitude (d may be an array)."""
    return (x.view(np.uint32).astype(np.int64) + d).astype(np.uint32).view(np.float32)


def _rn32(x64):
    return x64.astype(np.float32)


def test_fast_path_model_first_moment(lib):
    """Model of the kernel's first-moment fast path: q^ = RN(x * r) with r anywhere within one
    ulp of 1/s, entry lookup by the quotient's half-precision high byte, decision by the guard
    bounds.  Wherever
    the model does not ask for the exact path its code must equal the exact code
    #{j : mid_j < RN(x / s)}, for x on and around every threshold times the scale."""
    lo, hi = _table(lib)
    bucket_of = np.array([lib.q4adamw_mtable_half_bucket(h) for h in range(256)])
    _, mid = oc.tables(0)
    rng = np.random.default_rng(0)
    s = (10.0 ** rng.uniform(-25, 25, 4000)).astype(np.float32)
    d = np.arange(-40, 41)
    undecided = 0
    total = 0
    for j in range(15):
        centre = _rn32(mid[j].astype(np.float64) * s.astype(np.float64))
        x = _nudge(centre[:, None].repeat(d.size, 1), d[None, :])          # [s, d]
        exact_q = _rn32(x.astype(np.float64) / s[:, None].astype(np.float64))
        exact_code = np.searchsorted(mid, exact_q.ravel(), side="left").reshape(exact_q.shape)
        r0 = _rn32(1.0 / s.astype(np.float64))
        for dr in (-1, 0, 1):
            r = _nudge(r0, dr)
            q = _rn32(x.astype(np.float64) * r[:, None].astype(np.float64))
            a = bucket_of[_half_index(q)]
            e_lo, e_hi = lo[a], hi[a]
            above_hi = q > e_hi.view(np.float32)
            above_lo = q > (e_lo.view(np.float32))
            decided = above_hi == above_lo
            code = (e_lo & 15).astype(np.int64) + above_hi
            assert np.array_equal(code[decided], exact_code[decided])
            undecided += int((~decided).sum())
            total += decided.size
    # the guard band is a few ulps wide: most of the +-40 ulp neighbourhood is decided
    assert 0 < undecided < 0.6 * total


def _sr_tables(lib):
    thr = np.zeros(256, np.uint32)
    base = np.zeros(256, np.int64)
    out = (ctypes.c_uint32 * 2)()
    for h in range(256):
        assert lib.q4adamw_sr_bucket_entry(h, out) == 0
        thr[h], base[h] = out[0], out[1]
    slope = np.zeros(17, np.float32)
    offset = np.zeros(17, np.float32)
    pair = (ctypes.c_float * 2)()
    for k in range(17):
        assert lib.q4adamw_sr_affine_entry(k, pair) == 0
        slope[k], offset[k] = pair[0], pair[1]
    return thr.view(np.float32), base, slope, offset


def test_sr_affine_table_is_the_code_coordinate(lib):
    """Entry k of the affine table maps interval k's ends to k and k + 1 (to within the
    rounding of its two numbers), neighbouring entries meet at the code-book value between
    them, and the ends are constant."""
    _, _, slope, offset = _sr_tables(lib)
    Q = oc.tables(0)[0].astype(np.float64)
    assert (slope[0], offset[0]) == (0.0, 1.0) and (slope[16], offset[16]) == (0.0, 16.0)
    for k in range(1, 16):
        f = lambda q: float(slope[k]) * q + float(offset[k])
        assert abs(f(Q[k - 1]) - k) < 2.0 ** -20 and abs(f(Q[k]) - (k + 1)) < 2.0 ** -20
        assert max(abs(Q[k - 1]), abs(Q[k])) * float(slope[k]) < 9.0
        if k < 15:
            g = float(slope[k + 1]) * Q[k] + float(offset[k + 1])
            assert abs(f(Q[k]) - g) < 2.0 ** -20


def test_fast_path_model_first_moment_stochastic(lib):
    """Model of the first moment's fast path under stochastic rounding: q^ = RN(x * r), r
    within one ulp of 1/s; interval number from the half-indexed table; y = fma(n, -2^-16,
    fma(q^, slope, offset)); near tie iff fract(y) < 2^-16, else code trunc(y).  Wherever the
    model decides, its code must be the oracle's for the exact quotient RN(x / s) and the noise
    (2 n + 1) / 2^17 -- for positions spread over every interval and for positions within a
    few guard bands of the noise, where the decision flips."""
    from oracle import q4_oracle_torch as ot
    thr, base, slope, offset = _sr_tables(lib)
    Q = oc.tables(0)[0].astype(np.float64)
    rng = np.random.default_rng(11)
    count = 40000
    decided_total = undecided_total = 0
    for near in (False, True):
        s = (10.0 ** rng.uniform(-25, 25, count)).astype(np.float32)
        n = rng.integers(0, 1 << 16, count)
        n[:64] = 0
        n[64:128] = 65535
        u = ((2.0 * n + 1.0) / 2.0 ** 17).astype(np.float32)
        k = rng.integers(1, 16, count)
        lower, width = Q[k - 1], Q[k] - Q[k - 1]
        pos = u.astype(np.float64) + rng.uniform(-4, 4, count) * 2.0 ** -17 if near else rng.uniform(0, 1, count)
        target = np.clip(lower + np.clip(pos, 0, 1) * width, -1.0, 1.0)
        x = _rn32(target * s.astype(np.float64))
        x = np.clip(x, -s, s)                                             # |x| <= scale, as in a block
        exact_q = _rn32(x.astype(np.float64) / s.astype(np.float64))
        want = ot.sr_codes(exact_q, 0, u)
        r0 = _rn32(1.0 / s.astype(np.float64))
        for dr in (-1, 0, 1):
            q = _rn32(x.astype(np.float64) * _nudge(r0, dr).astype(np.float64))
            h = _half_index(q)
            k_raw = base[h] + (q >= thr[h])
            t = _rn32(q.astype(np.float64) * slope[k_raw].astype(np.float64) + offset[k_raw].astype(np.float64))
            y = _rn32(t.astype(np.float64) - n * 2.0 ** -16)
            decided = (y - np.floor(y)) >= np.float32(2.0 ** -16)
            assert np.all(y[decided] >= 0) and np.all(y[decided] < 16)
            code = np.trunc(y).astype(np.int64)
            bad = np.flatnonzero(decided & (code != want))
            assert bad.size == 0, (near, dr, bad[:5], q[bad[:5]], n[bad[:5]], code[bad[:5]], want[bad[:5]])
            decided_total += int(decided.sum())
            undecided_total += int((~decided).sum())
    # positions within +-4 bands of the noise: about a quarter lands inside the band
    assert 0 < undecided_total < 0.25 * (decided_total + undecided_total)


def test_fast_path_model_second_moment():
    """Same for the second moment: t = fma(x, 16 r, w - 0.5) with w = 2^-17; code = trunc(t)
    unless fract(t) < 2w."""
    _, mid = oc.tables(1)
    rng = np.random.default_rng(1)
    s = (10.0 ** rng.uniform(-25, 25, 4000)).astype(np.float32)
    d = np.arange(-40, 41)
    w = np.float32(2.0 ** -17)
    undecided = total = 0
    for j in range(15):
        centre = _rn32(mid[j].astype(np.float64) * s.astype(np.float64))
        x = _nudge(centre[:, None].repeat(d.size, 1), d[None, :])
        x = np.minimum(x, s[:, None])                                       # x <= scale always
        exact_q = _rn32(x.astype(np.float64) / s[:, None].astype(np.float64))
        exact_code = np.searchsorted(mid, exact_q.ravel(), side="left").reshape(exact_q.shape)
        r0 = _rn32(1.0 / s.astype(np.float64))
        for dr in (-1, 0, 1):
            r16 = _nudge(r0, dr) * np.float32(16)
            t = _rn32(x.astype(np.float64) * r16[:, None].astype(np.float64) + np.float64(w - np.float32(0.5)))
            fract = t - np.floor(t)
            decided = ~(fract < 2 * w)
            code = np.trunc(t).astype(np.int64)
            assert np.array_equal(code[decided], exact_code[decided])
            undecided += int((~decided).sum())
            total += decided.size
    assert 0 < undecided < 0.6 * total
    # far from thresholds nothing is flagged: uniform quotients
    q = rng.uniform(0, 1, 200000).astype(np.float32)
    t = _rn32(q.astype(np.float64) * 16 + np.float64(w - np.float32(0.5)))
    assert ((t - np.floor(t)) < 2 * w).mean() < 1e-3


def test_tables_exhaustively_on_the_host(tmp_path):
    """tests/native/check_tables.cpp walks every fp32 bit pattern in [-1, 1] (2.1e9 of them) through
    the constexpr tables of csrc/q4adamw_tables.h: decided codes are exact for every value
    within the quotient's error, and the stochastic-rounding interval numbers are exact"""
    import shutil
    import subprocess
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++")
    exe = str(tmp_path / "check_tables")
    subprocess.check_call([gxx, "-O2", "-std=c++17", "-fopenmp", "-o", exe,
                           os.path.join(ROOT, "tests", "native", "check_tables.cpp")])
    out = subprocess.run([exe], stdout=subprocess.PIPE, text=True, timeout=600)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout
    assert "0 wrong" in out.stdout


def test_device_code_holds_no_packed_fp32_instructions(tmp_path):
    """The build passes -packed-fp32-ops as a target feature.  hipcc's host pass does not
    know it (and says so); the gfx950 pass obeys it: a kernel that the compiler would
    otherwise turn into v_pk_fma_f32 compiles without packed fp32 instructions under the
    build's flags, and with them when the feature flag is left out."""
    import subprocess
    from quantfour_adamw_cuda_amd import build
    src = tmp_path / "pk.hip"
    src.write_text("#include <hip/hip_runtime.h>\n"
                   "__global__ void k(float2 *a, const float2 *b, const float2 *c) {\n"
                   "  int i = threadIdx.x; float2 x = a[i], y = b[i], z = c[i];\n"
                   "  x.x = x.x * y.x + z.x; x.y = x.y * y.y + z.y; a[i] = x; }\n")
    flags = [f for f in build.HIPCC_FLAGS if f not in ("-shared", "-fPIC", "-ffp-contract=off")]
    feature = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    assert all(f in flags for f in feature)
    bare = [f for f in flags if f not in feature]

    def packed(fl, name):
        out = tmp_path / name
        subprocess.run([build.hipcc_path()] + fl + ["--cuda-device-only", "-S", "-o", str(out), str(src)],
                       check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
        return sum(1 for ln in out.read_text().splitlines() if ln.strip().startswith(("v_pk_fma_f32", "v_pk_mul_f32", "v_pk_add_f32")))

    assert packed(bare, "bare.s") > 0, "the probe kernel no longer provokes packed instructions: pick another"
    assert packed(flags, "flagged.s") == 0


def test_assembly_block_keeps_the_wait_states_before_a_read_of_vcc(tmp_path):
    """On gfx950 a vector instruction that reads VCC needs two wait states after the vector
    instruction that wrote it.  The compiler keeps them in its own code (shown here on a plain
    compare + select) and does not look into assembly blocks, so the one block of the kernels
    that has such a pair (the stochastic-rounding select of the affine table's offset) must
    keep them itself."""
    import re
    import subprocess
    from quantfour_adamw_cuda_amd import build
    csrc = os.path.join(os.path.dirname(build.__file__), "csrc")
    src = tmp_path / "vcc.hip"
    src.write_text('#include "q4adamw_device.h"\n'
                   "__global__ void block(const float *q, const float *t, const uint32_t *h, uint32_t *o) {\n"
                   "  int i = threadIdx.x; o[i] = q4::high_half_if_ge(q[i], t[i], h[i]); }\n"
                   "__global__ void plain(const float *a, const float *b, const float *c, const float *d, float *o) {\n"
                   "  int i = threadIdx.x; o[i] = a[i] >= b[i] ? c[i] : d[i]; }\n")
    flags = [f for f in build.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    out = tmp_path / "vcc.s"
    subprocess.run([build.hipcc_path()] + flags + ["-I", csrc, "--cuda-device-only", "-S", "-o", str(out), str(src)],
                   check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    lines = [ln.strip() for ln in out.read_text().splitlines()]
    lines = [ln for ln in lines if ln and not ln.startswith((";", ".", "//")) and not ln.endswith(":")]

    def wait_states_before_read(writer_prefix, reader_prefix):
        found = []
        for i, ln in enumerate(lines):
            if ln.startswith(writer_prefix) and " vcc" in ln:
                n = 0
                for nxt in lines[i + 1:]:
                    if nxt.startswith(reader_prefix) and nxt.endswith("vcc") or ", vcc " in nxt and nxt.startswith(reader_prefix):
                        found.append(n)
                        break
                    m = re.match(r"s_nop (\d+)", nxt)
                    n += int(m.group(1)) + 1 if m else 1
        return found

    own = wait_states_before_read("v_cmp_ge_f32_e32", "v_cndmask_b32_sdwa")
    assert own and min(own) >= 2, f"the assembly block leaves {own} wait states"
    compilers = wait_states_before_read("v_cmp_ge_f32_e32", "v_cndmask_b32_e32")
    assert compilers and min(compilers) >= 2, f"the compiler's own pair: {compilers}"
