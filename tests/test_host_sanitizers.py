"""The CPU-side code under the address and undefined-behaviour sanitizers (no GPU involved):

* ``oracle/_build/oracle_sanitize_check`` (``make -C oracle asan``): the oracle over small frames
  with poisoned inputs, partial tiles, an empty scene and a key buffer that is too small;
* ``flashgs_amd/lib/asan/host_checks`` (``python -m flashgs_amd.build --asan-host``): the .ply
  reader against malformed files - a header may claim any vertex count - and every C-ABI entry
  point with the arguments it must refuse before any HIP call.

Both are built by ``__graft_entry__.build()``; a missing binary is built here.  A sanitizer report
aborts the program, so a zero exit status and the closing line are the whole check.
"""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")


def _run(path):
    res = subprocess.run([path], env=ENV, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-4000:]
    return res.stdout


def test_oracle_under_sanitizers():
    exe = os.path.join(ROOT, "oracle", "_build", "oracle_sanitize_check")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "asan"])
    assert "oracle sanitize check ok" in _run(exe)


def test_library_host_code_and_ply_reader_under_sanitizers():
    from flashgs_amd import build
    if not os.path.exists(build.ASAN_CHECKS):
        subprocess.check_call([sys.executable, "-m", "flashgs_amd.build", "--asan-host"], cwd=ROOT)
    assert "host checks ok" in _run(build.ASAN_CHECKS)
