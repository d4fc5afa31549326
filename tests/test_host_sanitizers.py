"""The host C code under AddressSanitizer + UndefinedBehaviorSanitizer: tests/sanitize/Makefile builds the input
generator, the CPU oracle and the C harness with -fsanitize=address,undefined and runs them (exact-size buffers,
odd sizes, every mask kind, bad arguments; the harness's argument parsing and its exit without a GPU).  Any
sanitizer report makes the run fail."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_host_code_runs_clean_under_asan_and_ubsan():
    lib = os.path.join(os.path.dirname(HERE), "flash-attn-rtx5060_amd", "lib", "libfa_fwd_gfx950.so")
    assert os.path.exists(lib), "build the library first (python -c 'import __graft_entry__ as g; g.build()')"
    r = subprocess.run(["make", "-C", os.path.join(HERE, "sanitize"), "run"], capture_output=True, text=True, timeout=600)
    tail = (r.stdout + r.stderr)[-4000:]
    assert r.returncode == 0, tail
    assert r.stdout.count("host self-test passed") == 2, tail
    assert "ERROR: AddressSanitizer" not in tail and "runtime error:" not in tail, tail
