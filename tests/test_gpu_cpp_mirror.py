"""The C++ host mirror (include/stingray_sampler.hpp) over the C ABI: tests/cpp/host_mirror_test.cpp compares
Sampler::Greedy / Sample / BuildFilteredDistribution / SampleWithDistribution / SampleFromProbs / ResampleResidual
and their exceptions with the CPU oracle.  The program is built by __graft_entry__.build()."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "host_mirror_test")


def test_cpp_host_mirror_matches_the_oracle():
    assert os.path.exists(BIN), "build with: python -c 'import __graft_entry__ as g; g.build()'"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=200)
    assert r.returncode == 0, r.stdout[-4000:] + r.stderr[-2000:]
    assert r.stdout.strip().splitlines()[-1].startswith("OK ")
