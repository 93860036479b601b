"""include/tenferro.hpp -- the C++ mirror of the reference's interface -- through its own test program
(tests/cpp/test_mirror.cpp): the host part needs no GPU, the gpu part runs the hot path on device 0 and checks it
against plain loops."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_mirror")


def _binary():
    if not os.path.exists(BIN):   # built by __graft_entry__.build(); compile here only if nothing is built
        import importlib.util
        spec = importlib.util.spec_from_file_location("graft_entry", os.path.join(ROOT, "__graft_entry__.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        if not os.path.exists(os.path.join(ROOT, "tenferro-rs_amd", "libtenferro_hip.so")):
            mod._build_module().build(force=False)
        mod.build_cpp_mirror_test()
    return BIN


def _run(mode):
    r = subprocess.run([_binary(), mode], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failed" in r.stdout, r.stdout
    return r.stdout


def test_header_is_self_contained_and_host_checks_pass():
    out = _run("host")
    assert out.startswith("host:") or "host:" in out


@pytest.mark.gpu
def test_hot_path_through_the_cpp_mirror():
    out = _run("gpu")
    assert "gpu:" in out
