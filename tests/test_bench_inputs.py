"""bench.py generates its synthetic inputs itself (numpy); the oracle holds the same generators
for the parity tests.  They must produce the same bits."""
import os
import sys

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, REPO)
import bench  # noqa: E402


def test_mt19937_stream_is_the_standard_one():
    # the C++ standard's check value: the 10000th output of a default-seeded (5489) mt19937
    assert int(bench._mt19937_raw(5489, 10000)[-1]) == 4123659995


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_generators_match_the_oracle(orc, dtype):
    n = 70001
    assert np.array_equal(bench.gen_uniform(n, dtype, 20246, -1.0, 1.0), orc.fill_uniform(n, dtype, 20246, -1.0, 1.0))
    assert np.array_equal(bench.gen_normal(n, dtype, 20248, 0.0, 2.0), orc.fill_normal(n, dtype, 20248, 0.0, 2.0))
    assert np.array_equal(bench.gen_normal(7, dtype, 3, 1.0, 0.1), orc.fill_normal(7, dtype, 3, 1.0, 0.1))
    got, want = bench.gen_bits(n, dtype, 20244), orc.fill_bits(n, dtype, 20244)
    assert np.array_equal(got.view(np.uint32 if dtype == "f32" else np.uint16),
                          want.view(np.uint32 if dtype == "f32" else np.uint16))


def test_bench_refuses_more_than_one_gpu():
    """Every figure of this build is one GPU's: `bench.py --gpus N` with N > 1 says so and exits before it
    touches a device."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""
