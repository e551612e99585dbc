"""Shared helpers of the parity tests: seeded inputs for the benchmark
configurations and the comparison of a device step with the CPU oracle."""
import numpy as np
import torch

from oracle import q4_oracle as oc

HP = dict(beta1=0.9, beta2=0.999, lr=1e-3, weight_decay=0.01, eps=1e-8)
HP_DRIVER = dict(beta1=0.8, beta2=0.88, lr=5e-3, weight_decay=0.03, eps=1e-8)  # tests/driver.py:28-31


def bits(a):
    """uint32 view of an fp32 numpy array (for bit-exact comparison incl. -0.0, NaN)."""
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def bf16_bits(t):
    """torch bf16 tensor -> numpy uint16 bit patterns."""
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16).copy()


def to_np(t):
    if t.dtype == torch.bfloat16:
        return bf16_bits(t).reshape(-1)
    return t.detach().cpu().contiguous().numpy().reshape(-1).copy()


def grads_config1(gen, n):
    """N(0, 1e-3^2) with 0.1 % of the entries replaced by +-1e-1 outliers."""
    g = torch.randn(n, generator=gen) * 1e-3
    mask = torch.rand(n, generator=gen) < 1e-3
    sign = torch.where(torch.rand(n, generator=gen) < 0.5, -1.0, 1.0)
    return torch.where(mask, sign * 1e-1, g)


def grads_config3(gen, n):
    """20 % exact zeros, 1 % fp32 denormals, 0.01 % +-1e3 outliers, rest N(0, 1e-3^2)."""
    g = torch.randn(n, generator=gen) * 1e-3
    u = torch.rand(n, generator=gen)
    sign = torch.where(torch.rand(n, generator=gen) < 0.5, -1.0, 1.0)
    den_bits = torch.randint(1, 1 << 23, (n,), generator=gen, dtype=torch.int32)
    den = den_bits.view(torch.float32) * sign
    g = torch.where(u < 0.20, torch.zeros(()), g)
    g = torch.where((u >= 0.20) & (u < 0.21), den, g)
    g = torch.where((u >= 0.21) & (u < 0.2101), sign * 1e3, g)
    return g


def grads_student_t(gen, n, scale=1e-4):
    """Student-t with 3 degrees of freedom, scaled."""
    z = torch.randn(n, generator=gen)
    c = torch.randn(3, n, generator=gen).square().sum(0) / 3.0
    return z / c.sqrt() * scale


class OracleTensor:
    """CPU-side twin of one quantized tensor, stepped by the C oracle."""

    def __init__(self, p):
        self.p = to_np(p)
        n = self.p.size
        nbytes, nblk = oc.state_sizes(n)
        self.m = np.zeros(nbytes, np.uint8)
        self.v = np.zeros(nbytes, np.uint8)
        self.sm = np.zeros(nblk, np.float32)
        self.sv = np.zeros(nblk, np.float32)

    def step(self, g, step, hp=HP):
        """Returns the parameters the step started from."""
        prev = self.p.copy()
        oc.step_quant(self.p, to_np(g), self.m, self.v, self.sm, self.sv, step=step, **hp)
        return prev

    def resync(self, p_dev):
        """Continue from the device's parameters, so that the parameter bound stays a
        per-step bound (the moments never depend on the parameters)."""
        self.p[:] = to_np(p_dev)


class DeviceTensor:
    """Device-side state of one quantized tensor for the functional entry points."""

    def __init__(self, p, device):
        self.p = p.detach().clone().to(device).reshape(-1).contiguous()
        n = self.p.numel()
        nbytes, nblk = oc.state_sizes(n)
        self.m = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        self.v = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        self.sm = torch.zeros(nblk, dtype=torch.float32, device=device)
        self.sv = torch.zeros(nblk, dtype=torch.float32, device=device)


# Strict parameter metrics of every fp32-parameter comparison made in this session, one entry
# per call: (test id, elements, max |dev - ref| / |ref|, elements above 1e-6 relative, max of
# that ratio where the parameter is at least as large as the step it took, max error in ulps
# of the step where the step is the larger one).  tests/conftest.py prints them per test.
STRICT_LOG = []


def _current_test():
    import os
    return os.environ.get("PYTEST_CURRENT_TEST", "?").split(" (")[0]


def strict_param_metrics(p_dev, p_ref, p_prev, label=None):
    """The parameter bound as the optimizer's users read it -- |dev - ref| <= 1e-6 * |ref| --
    measured on one step from identical inputs (fp32 parameters; numpy arrays or torch
    tensors).  An update that is not bit-identical to the oracle's cannot meet it for a
    parameter that its own step carries to (nearly) zero, so the elements are split by which
    is larger, the parameter or the step it took:
      |ref| >= |ref - prev|   the strict bound is ASSERTED by the callers (returned as `dom`)
      |ref| <  |ref - prev|   the error is reported in ulps of the step (`step_ulps`); the
                              callers assert 1e-6 relative to the step there
    `atol` is the smallest absolute tolerance that makes |dev - ref| <= atol + 1e-6 * |ref| hold
    for every element.  Returns dict(n, max_rel, above, dom, step_ulps, atol) and logs it for
    the session summary."""
    if torch.is_tensor(p_ref):
        dev, ref, prev = (t.detach().reshape(-1).double() for t in (p_dev, p_ref, p_prev))
        diff, aref, step = (dev - ref).abs(), ref.abs(), (ref - prev).abs()
        tiny = torch.finfo(torch.float32).tiny
        rel = diff / aref.clamp_min(tiny)
        rel = torch.where((aref == 0) & (diff == 0), torch.zeros_like(rel), rel)
        is_dom = aref >= step
        dom = float(torch.where(is_dom, rel, torch.zeros_like(rel)).max()) if rel.numel() else 0.0
        ulp = torch.exp2(torch.floor(torch.log2(step.clamp_min(tiny))) - 23)
        su = torch.where(is_dom, torch.zeros_like(rel), diff / ulp)
        out = dict(n=int(rel.numel()), max_rel=float(rel.max()) if rel.numel() else 0.0,
                   above=int((rel > 1e-6).sum()), dom=dom, step_ulps=float(su.max()) if rel.numel() else 0.0,
                   atol=float((diff - 1e-6 * aref).clamp_min(0).max()) if rel.numel() else 0.0)
    else:
        dev, ref, prev = (np.asarray(a, np.float32).reshape(-1).astype(np.float64) for a in (p_dev, p_ref, p_prev))
        diff, aref, step = np.abs(dev - ref), np.abs(ref), np.abs(ref - prev)
        tiny = float(np.finfo(np.float32).tiny)
        with np.errstate(invalid="ignore", divide="ignore"):
            rel = diff / np.maximum(aref, tiny)
            rel = np.where((aref == 0) & (diff == 0), 0.0, rel)
            rel = np.where(np.isnan(ref) | np.isinf(ref), 0.0, rel)     # non-finite cases are compared elsewhere
            is_dom = aref >= step
            ulp = np.exp2(np.floor(np.log2(np.maximum(step, tiny))) - 23)
            su = np.where(is_dom | ~np.isfinite(step), 0.0, diff / ulp)
        out = dict(n=int(rel.size), max_rel=float(rel.max()) if rel.size else 0.0,
                   above=int((rel > 1e-6).sum()), dom=float(np.where(is_dom, rel, 0.0).max()) if rel.size else 0.0,
                   step_ulps=float(su.max()) if rel.size else 0.0,
                   atol=float(np.nan_to_num(np.maximum(diff - 1e-6 * aref, 0.0), nan=0.0, posinf=0.0).max()) if rel.size else 0.0)
    STRICT_LOG.append((label or _current_test(), out))
    return out


# With the benchmark's hyper-parameters (lr 1e-3, betas 0.9 / 0.999, eps 1e-8, weight decay
# 0.01) the fp32 parameters of one step satisfy |dev - ref| <= ATOL + 1e-6 |ref|: the measured
# need is 3.3e-10 over 2.4e10 element-steps of the Llama-3-8B set (a step is at most about
# 3.2 lr, and the error at most 6 ulps of the step).
BASELINE_RTOL, BASELINE_ATOL = 1e-6, 5e-10


def strict_atol_since(mark):
    """largest `atol` among the strict comparisons logged since STRICT_LOG had `mark` entries"""
    return max((m["atol"] for _, m in STRICT_LOG[mark:]), default=0.0)


def p_mismatches(p_dev, p_ref):
    """Number of fp32 parameters whose bit patterns differ (a NaN on both sides counts as
    equal, whatever its payload)."""
    a, b = np.asarray(p_dev, np.float32).reshape(-1), np.asarray(p_ref, np.float32).reshape(-1)
    same = (bits(a) == bits(b)) | (np.isnan(a) & np.isnan(b))
    return int(a.size - np.count_nonzero(same))


def p_close(p_dev, p_ref, p_prev, bf16=False, exact=False):
    """exact=True (fp32 parameters from the exact form of the update, which the library takes
    by itself for fp32 parameters in the block-scaled step with nearest rounding, and anywhere
    on request): bit-identical to the oracle's; returns (ok, number of mismatches).
    Otherwise the parameter tolerance for ONE step from identical inputs (the folded form).
    fp32: |dev - ref| <= 1e-6 * |ref| wherever the parameter is at least as large as the step it
    took (the strict bound), and 1e-6 relative to the step elsewhere (parameters that their own
    step carries towards zero, where a relative bound on the parameter alone cannot hold for
    anything but bit-identical arithmetic).  Both together: 1e-6 * max(|ref|, |ref - prev|).
    bf16 parameters (uint16 bit patterns) and fp16 parameters (numpy float16): at most one
    ulp of the storage type, measured on the same scale.
    Returns (ok, worst ratio or ulps)."""
    half = np.asarray(p_ref).dtype == np.float16
    if bf16 or half:
        # one ulp of the larger of the parameter and the step it took (a parameter
        # that cancels against its update lands near zero, where its own ulp is tiny)
        if half:
            f = lambda u: np.asarray(u).astype(np.float64)
            mant, floor_ulp = 10, 2.0 ** -24          # below 2^-14 fp16 is spaced 2^-24 apart
        else:
            f = lambda u: (u.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
            mant, floor_ulp = 7, 0.0
        dev, ref, prev = f(p_dev), f(p_ref), f(p_prev)
        scale = np.maximum(np.maximum(np.abs(ref), np.abs(ref - prev)), np.finfo(np.float32).tiny)
        ulp = np.maximum(2.0 ** (np.floor(np.log2(scale)) - mant), floor_ulp)
        worst = float((np.abs(dev - ref) / ulp).max()) if dev.size else 0.0
        return worst <= 1.0, worst
    strict = strict_param_metrics(p_dev, p_ref, p_prev)
    if exact:
        bad = p_mismatches(p_dev, p_ref)
        return bad == 0, float(bad)
    ref = p_ref.astype(np.float64)
    diff = np.abs(p_dev.astype(np.float64) - ref)
    scale = np.maximum(np.abs(ref), np.abs(ref - p_prev.astype(np.float64)))
    scale = np.maximum(scale, np.finfo(np.float32).tiny)
    worst = float((diff / scale).max())
    return worst <= 1e-6 and strict["dom"] <= 1e-6, worst


def assert_state_equal(dev, ref, p_prev, what="", exact=None):
    """codes and scales bit-exact; parameters bit-exact where the exact form of the update ran
    (exact=None: fp32 parameters, what the library chooses by itself in the block-scaled step
    with nearest rounding), within tolerance otherwise; p_prev holds the parameters both sides
    started the step from."""
    m = dev.m.cpu().numpy()
    v = dev.v.cpu().numpy()
    sm = dev.sm.cpu().numpy()
    sv = dev.sv.cpu().numpy()
    bad = np.flatnonzero(bits(sm) != bits(ref.sm))
    assert bad.size == 0, f"{what}: first-moment scales differ at blocks {bad[:5]}: {sm[bad[:5]]} vs {ref.sm[bad[:5]]}"
    bad = np.flatnonzero(bits(sv) != bits(ref.sv))
    assert bad.size == 0, f"{what}: second-moment scales differ at blocks {bad[:5]}: {sv[bad[:5]]} vs {ref.sv[bad[:5]]}"
    bad = np.flatnonzero(m != ref.m)
    assert bad.size == 0, f"{what}: first-moment codes differ at bytes {bad[:5]}: {m[bad[:5]]} vs {ref.m[bad[:5]]} ({bad.size} bytes)"
    bad = np.flatnonzero(v != ref.v)
    assert bad.size == 0, f"{what}: second-moment codes differ at bytes {bad[:5]}: {v[bad[:5]]} vs {ref.v[bad[:5]]} ({bad.size} bytes)"
    is_bf16 = dev.p.dtype == torch.bfloat16
    if exact is None:
        exact = dev.p.dtype == torch.float32
    ok, worst = p_close(to_np(dev.p), ref.p, p_prev, bf16=is_bf16, exact=exact and dev.p.dtype == torch.float32)
    if exact and dev.p.dtype != torch.float32:    # 16-bit parameters from the exact form: the stored patterns
        bad = int(np.count_nonzero(to_np(dev.p) != ref.p))
        assert bad == 0, f"{what}: {bad} 16-bit parameters differ from the oracle's"
    assert ok, f"{what}: parameters differ (bit-exact expected, {worst:.0f} mismatches)" if exact else \
        f"{what}: parameters out of tolerance (worst {worst})"
    return 0.0 if exact else worst
