"""The block fp8 quantiser of the scatter divides the eight values a lane holds by one scale.  It does so with the
reciprocal of the scale refined once and one correction per quotient (DivideByShared in
tilexr_amd/csrc/ep_numerics.hip.h), not with eight full divisions.  tests/cxx/shared_division_check.hip, built from that
same header, tries it on the GPU against the correctly rounded division for every pair the quantiser can meet: all 2^16
element patterns (NaNs and infinities included) with all 2^15 non-negative block maxima, about 10^9 pairs per element
type, and passes when no e4m3 code differs.
"""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CHECK = os.path.join(ROOT, "tests", "cxx", "bin", "shared_division_check")


@pytest.mark.parametrize("element", ["bf16", "fp16"])
def test_shared_divisor_division_gives_the_codes_of_the_exact_division(element):
    if not os.path.exists(CHECK):
        pytest.fail(f"{CHECK} is missing: build it with `make -C tilexr_amd/csrc` (or __graft_entry__.build())")
    print(f"shared division check {element}", flush=True)
    run = subprocess.run([CHECK, element], capture_output=True, text=True, timeout=100)
    last = run.stdout.strip().splitlines()[-1] if run.stdout.strip() else ""
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]
    assert last.startswith(f"OK {element}:") and " 0 codes differ" in last, last
