"""The host-side allocator and tiered prefix tree under the address and undefined-behaviour
sanitizers: a randomised C++ exercise (tests/cpp/tree_sanitize_test.cpp) that checks both
structures' invariants after every operation.  No GPU, no library: host sources only."""
import os
import subprocess

import pytest

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "tree_sanitize_test")


@pytest.mark.parametrize("seed", [1, 7, 42])
def test_allocator_and_prefix_tree_are_clean_under_sanitizers(seed):
    if not os.path.exists(BIN):
        # host sources only (g++, a few seconds): built here when the tree's build step has not run
        from breccia_amd.build import build_tree_sanitize_test
        build_tree_sanitize_test()
    env = dict(os.environ)
    # other preloaded libraries may come before the sanitizer runtime
    env["ASAN_OPTIONS"] = "verify_asan_link_order=0:detect_leaks=1"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    r = subprocess.run([BIN, str(seed), "5000"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert r.stdout.startswith("ok "), r.stdout
