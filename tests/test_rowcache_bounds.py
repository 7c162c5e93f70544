"""The bytes that the shifted row accesses of the cross-entropy kernels touch (blackforge_amd/csrc/rowcache.hpp), checked
on the CPU: tests/cpp/rowcache_bounds_test.cpp compiles RowCache for the host over accessors that check every address
against the tensor's extent, for the group sizes, register counts, row lengths and alignments the launcher uses."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "blackforge_amd", "host", "bin", "rowcache_bounds_test")


def test_shifted_rows_touch_only_their_tensor():
    assert os.path.exists(EXE), "run `make -C blackforge_amd/host` (the driver's build() does)"
    proc = subprocess.run([EXE], capture_output=True, text=True, timeout=300)
    print(proc.stdout[-3000:])
    assert proc.returncode == 0 and " 0 failure(s)" in proc.stdout, proc.stdout[-3000:] + proc.stderr[-1000:]
    assert proc.stdout.count("[  OK  ]") >= 47
