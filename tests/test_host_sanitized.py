"""The host logic of the decode path -- table builder, table patching, prefix-tree manager and the
host-only C-ABI in front of them -- rebuilt with AddressSanitizer and UndefinedBehaviorSanitizer
(chunk-attention_amd/build.py --host-sanitize) and driven through the same CPU tests that check it
bit-exactly against the oracle.  The reference has no such build; this is the cheap half of the
path to put under a sanitizer: integer work whose every index is checked by the tests already."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

TESTS = ["tests/test_tables_native.py", "tests/test_tree_native.py"]


def _runtime(name):
    try:
        path = subprocess.check_output(["gcc", "-print-file-name=" + name], text=True).strip()
    except (OSError, subprocess.CalledProcessError):
        return None
    return path if os.path.isabs(path) and os.path.exists(path) else None


def test_host_logic_under_asan_and_ubsan():
    asan = _runtime("libasan.so")
    if asan is None:
        pytest.skip("no gcc AddressSanitizer runtime on this machine")
    sys.path.insert(0, os.path.join(ROOT, "chunk-attention_amd"))
    import importlib.util
    spec = importlib.util.spec_from_file_location("ca_build", os.path.join(ROOT, "chunk-attention_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    lib = build.build_host_sanitized()
    env = dict(os.environ)
    env["CHUNK_ATTN_HIP_LIB"] = lib
    env["CHUNK_ATTN_HOST_ONLY"] = "1"
    # the sanitizer runtime must come first among the preloaded libraries, and the C++ runtime has
    # to be there when it starts (python itself does not link it, and the sanitizer looks up
    # __cxa_throw once, at start); whatever was preloaded before stays
    stdcxx = _runtime("libstdc++.so.6") or _runtime("libstdc++.so")
    env["LD_PRELOAD"] = ":".join(x for x in (asan, stdcxx, env.get("LD_PRELOAD")) if x)
    # python itself is not instrumented: its own allocations at exit are not this test's business
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1:halt_on_error=1"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"] + TESTS,
                       cwd=ROOT, env=env, capture_output=True, text=True, timeout=900)
    tail = (r.stdout + r.stderr)[-3000:]
    assert r.returncode == 0, tail
    assert " passed" in r.stdout and "AddressSanitizer" not in tail and "runtime error" not in tail, tail
