"""The host code of the library and the oracle under AddressSanitizer + UndefinedBehaviorSanitizer
(tests/cpp/test_host_sanitized.cpp): parser and plan validation on random input, the tree optimiser and its shared cache
from several threads, every primitive and random einsum networks executed on host memory through the unchanged host code
with stand-ins for the device launchers, all checked against the oracle, and the oracle's blocked contraction against its
brute-force form.  A sanitizer report fails the run; so does a leak."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_host_sanitized")
SOURCES = [os.path.join(ROOT, "tests", "cpp", "test_host_sanitized.cpp"), os.path.join(ROOT, "tests", "cpp", "host_backend.cpp"),
           os.path.join(ROOT, "oracle", "tfo_oracle.cpp")] + \
          [os.path.join(ROOT, "tenferro-rs_amd", "csrc", f) for f in ("errors.cpp", "plan.cpp", "prims.cpp", "einsum.cpp", "internal.hpp")]


def _binary():
    stale = not os.path.exists(BIN) or any(os.path.getmtime(s) > os.path.getmtime(BIN) for s in SOURCES)
    if stale:   # built by __graft_entry__.build(); compile here when it is missing or older than its sources
        import importlib.util
        spec = importlib.util.spec_from_file_location("graft_entry", os.path.join(ROOT, "__graft_entry__.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_host_sanitized_test()
    return BIN


def test_host_code_and_oracle_run_clean_under_asan_and_ubsan():
    env = dict(os.environ)
    env["ASAN_OPTIONS"] = "detect_leaks=1:abort_on_error=0:halt_on_error=1"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    r = subprocess.run([_binary()], capture_output=True, text=True, timeout=600, env=env)
    out = r.stdout + r.stderr
    assert "AddressSanitizer" not in out and "runtime error" not in out and "LeakSanitizer" not in out, out[-4000:]
    assert r.returncode == 0, out[-4000:]
    last = r.stdout.strip().splitlines()[-1]
    assert last.endswith(" checks, 0 failed") and int(last.split()[0]) > 40000, last
