"""Runs the C++ test executables of the nz:: host layer (neuzephyr_amd/nz/tests).
test_host needs no GPU (Dimension, node shape errors, graph ordering, allocator bookkeeping,
under ASan/UBSan); test_gpu restates the reference's own tests for the path against this build."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TESTS = os.path.join(ROOT, "neuzephyr_amd", "nz", "tests")


def _run(name, timeout):
    exe = os.path.join(TESTS, name)
    assert os.path.exists(exe), f"{exe} is not built; run __graft_entry__.build()"
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0")
    p = subprocess.run([exe], capture_output=True, text=True, timeout=timeout, env=env)
    print(p.stdout[-4000:])
    print(p.stderr[-2000:])
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    assert "0 failures" in p.stdout


def test_host_layer_without_gpu():
    _run("test_host", 120)


@pytest.mark.gpu
def test_cpp_api_on_gpu():
    _run("test_gpu", 300)


@pytest.mark.gpu
def test_readme_example_runs_and_learns():
    """The reference's README network on the nz:: layer (reduced image size): finite loss that goes down."""
    import json
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "neuzephyr_amd", "nz", "examples",
                       "readme_example")
    assert os.path.exists(exe), "build the host layer first (python -m neuzephyr_amd.build)"
    p = subprocess.run([exe, "6", "1", "4", "96", "128"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr[-2000:]
    line = json.loads(p.stdout.strip().splitlines()[-1])
    assert line["fused_groups"] == 3
    assert 0.0 < line["loss_last"] < line["loss_first"]
