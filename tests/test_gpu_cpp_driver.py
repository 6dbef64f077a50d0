"""Runs the C++ CPU-vs-GPU comparison driver (tests/cpp/compare_cpu_and_gpu.cpp): the reference's
own kind of test (Tests/test_compare_cpu_and_gpu.cpp), through the C++ header and the functors."""
import os
import subprocess

import pytest

from conftest import ROOT

BIN = os.path.join(ROOT, "tests", "cpp", "compare_cpu_and_gpu.bin")


@pytest.mark.gpu
@pytest.mark.parametrize("height,width", [(240, 320), (97, 131)])
def test_cpp_driver_cpu_and_gpu_agree(height, width):
    if not os.path.exists(BIN):
        pytest.fail("%s is missing: run __graft_entry__.build() first" % BIN)
    res = subprocess.run([BIN, str(height), str(width)], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=100)
    print(res.stdout)
    assert res.returncode == 0, res.stdout
    assert res.stdout.count("positions differing 0") == 2      # the float run and the double run
