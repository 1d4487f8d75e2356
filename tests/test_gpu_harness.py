"""The plain-C harnesses of the fp16 entry points (tests/harness/*.c, the counterparts of the main() functions of the
reference's cuda-src/mlstm_forward.cu:192-263 and mlstm_backward.cu:561-670), each run as a fresh child process: the header
compiles and the library links from C, and the reference's own self-check prints no mismatch."""
import os
import re
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "harness")


def run(binary, *args):
    path = os.path.join(HERE, binary)
    if not os.path.exists(path):
        pytest.fail(f"{path} is not built: run `make -C tests/harness` (or __graft_entry__.build())")
    return subprocess.run([path, *args], capture_output=True, text=True, timeout=120)


@pytest.mark.gpu
@pytest.mark.parametrize("S", ["640", "1280"])       # the README's shape and the reference source's constant
def test_forward_harness_prints_no_mismatch(S):
    p = run("mlstm_forward_main", S)
    assert p.returncode == 0, p.stderr
    assert "Check H" in p.stdout
    assert re.findall(r"Non_matching count: (\d+)", p.stdout) == ["0"], p.stdout


@pytest.mark.gpu
def test_backward_harness_prints_no_mismatch():
    p = run("mlstm_backward_main")
    assert p.returncode == 0, p.stderr
    for name in ("dQ", "dK", "dV", "dF", "dI"):
        assert f"Check {name}" in p.stdout
    assert re.findall(r"Non_matching count: (\d+)", p.stdout) == ["0"] * 5, p.stdout


def test_harness_sources_use_the_public_header_only():
    # no GPU needed: the harnesses may call nothing of the library that include/mlstm_hip.h does not declare
    for name in ("mlstm_forward_main.c", "mlstm_backward_main.c"):
        src = open(os.path.join(HERE, name)).read()
        assert '#include "mlstm_hip.h"' in src
        called = set(re.findall(r"\b(mlstm_[a-z_0-9]+)\s*\(", src))
        header = open(os.path.join(HERE, "..", "..", "include", "mlstm_hip.h")).read()
        for fn in called:
            assert re.search(r"\b%s\s*\(" % fn, header), fn
