"""Device dispatch of the HIP backend (include/blackforge/backend/hip/dispatch.hpp) through its C++ test program:
the `--device cpu|cuda[:N]|hip[:N]` parser with the reference's diagnostics, target names, listing and selection."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "blackforge_amd", "host", "bin", "dispatch_test")


def run(expected_devices):
    assert os.path.exists(EXE), "run `make -C blackforge_amd/host` (the driver's build() does)"
    proc = subprocess.run([EXE, str(expected_devices)], capture_output=True, text=True, timeout=120)
    print(proc.stdout[-3000:])
    assert proc.returncode == 0 and "0 failure(s)" in proc.stdout, proc.stdout[-3000:] + proc.stderr[-1000:]
    return proc.stdout


def test_device_spec_parser_and_refusals():
    """Runs anywhere: with no device `hip:0` must be refused, with one it must be selected (-1 = either)."""
    out = run(-1)
    assert out.count("[  OK  ]") >= 24


@pytest.mark.gpu
def test_hip0_is_selected_on_a_gpu_box(hip):
    out = run(hip.capi.device_count())
    assert "hip:0 is selected" in out and "listing names hip:0" in out
