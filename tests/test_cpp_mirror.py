"""The C++ mirror of the reference interface (include/nabla_optim.hpp) replays the
reference's own optimizer tests on the device (tests/cpp/test_reference_kats.cpp)."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "test_reference_kats.bin")


def test_cpp_replay_is_built():
    assert os.path.exists(BIN), "build it with `make -C tests/cpp` (or __graft_entry__.build())"


@pytest.mark.gpu
def test_cpp_replay_of_reference_tests(gpu):
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("ok    ") == 13 and "0 failure(s)" in r.stdout
