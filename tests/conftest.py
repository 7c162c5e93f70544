"""Shared pytest configuration.

Markers: ``gpu`` = needs a real MI355X (parity tests through the C ABI); everything else runs on CPU.
"""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X GPU")


@pytest.fixture(scope="session")
def oracle():
    """The C restatement of the reference CPU backend (test infrastructure)."""
    from oracle import bfo
    return bfo.oracle()


@pytest.fixture(scope="session")
def ref():
    """The real reference CPU backend, where oracle/_ref has been built."""
    from oracle import bfo
    r = bfo.reference()
    if r is None:
        pytest.skip("oracle/_ref/libbf_ref.so not built (reference tree absent)")
    return r


@pytest.fixture(scope="session")
def hip():
    """The shipped C-ABI library on a GPU box; fails loudly when it is missing."""
    import blackforge_amd as bf
    lib = bf.capi.load()
    if bf.capi.device_count() < 1:
        pytest.fail("no HIP device visible: gpu-marked tests need a real MI355X")
    route = os.environ.get("BF_ATTN_ROUTE")   # run the whole suite on another attention route: BF_ATTN_ROUTE=0 pytest -m gpu
    if route is not None:
        bf.capi.call("bf_hip_attention_set_route", int(route))
    return bf


@pytest.fixture
def rng():
    return np.random.default_rng(1234)
