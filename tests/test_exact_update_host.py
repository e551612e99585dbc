"""Host-side checks of the exact parameter update's short sequences: tests/native/check_exact_update.c
runs the division on every numerator whose quotient comes within the sequence's error of a
rounding midpoint (for all 2^23 divisor mantissas: the computer-assisted part of the proof
that it is correctly rounded), and the square-root fix-up on every mantissa with the estimate
one ulp low, right, and one ulp high."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_short_division_and_square_root_round_correctly(tmp_path):
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    exe = str(tmp_path / "check_exact_update")
    subprocess.check_call([gcc, "-std=c11", "-O2", "-ffp-contract=off", "-Wall", "-Werror",
                           os.path.join(ROOT, "tests", "native", "check_exact_update.c"), "-lm", "-o", exe])
    out = subprocess.run([exe, "50000000"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert out.returncode == 0 and out.stdout.startswith("ok "), out.stdout
    near, roots = int(out.stdout.split()[1]), int(out.stdout.split()[-3])
    assert near > 50_000_000 and roots == 3 << 24, out.stdout


def test_param_update_option_is_validated():
    import torch
    from quantfour_adamw_cuda_amd import AdamWFused_QuantFour
    from quantfour_adamw_cuda_amd import quantfour_hip as q
    p = [torch.nn.Parameter(torch.zeros(8))]
    for form in ("auto", "exact", "folded"):
        assert AdamWFused_QuantFour(p, param_update=form).param_groups[0]["param_update"] == form
    with pytest.raises(ValueError, match="param_update"):
        AdamWFused_QuantFour(p, param_update="fast")
    with pytest.raises(ValueError, match="update_form"):
        q.grad_options(torch.device("cpu"), update_form="fast")
    assert q.grad_options(torch.device("cpu")) is None
    assert q.grad_options(torch.device("cpu"), update_form="exact").update_form == 1
    # an optimizer pickled before the option existed comes back with "auto"
    opt = AdamWFused_QuantFour(p)
    state = opt.__getstate__()
    for g in state["param_groups"]:
        g.pop("param_update")
    opt.__setstate__(state)
    assert opt.param_groups[0]["param_update"] == "auto"
