"""The drop-in check on the GPU: oracle/_ref/hip_dropin_test hands the SAME ir::ModelIR / ast::Program objects to the
reference's CPU backend and to blackforge::backend::hip (Executor, Model(ir, seed), runTraining(program, module, ...),
checkpoint interchange) and compares the results.  The program is built from the reference's own sources by
oracle/Makefile where the reference tree exists and travels with the tree.  Where the reference build itself is absent
(a tree that never saw the reference) the test skips; where libbf_ref.so was built but the program was not, it fails."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "oracle", "_ref", "hip_dropin_test")


def test_same_program_through_cpu_and_hip_backends(hip, tmp_path):
    if not os.path.exists(EXE):
        if os.path.exists(os.path.join(ROOT, "oracle", "_ref", "libbf_ref.so")):
            pytest.fail("oracle/_ref/libbf_ref.so is present but oracle/_ref/hip_dropin_test is not: run `make -C oracle all`")
        pytest.skip("oracle/_ref was never built here (needs the reference tree at build time)")
    proc = subprocess.run([EXE, str(tmp_path)], capture_output=True, text=True, timeout=300)
    print(proc.stdout[-4000:])
    assert proc.returncode == 0, proc.stdout[-4000:] + proc.stderr[-2000:]
    assert proc.stdout.count("[  OK  ]") >= 17 and "0 failure(s)" in proc.stdout
