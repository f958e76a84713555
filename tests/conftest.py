"""Shared pytest fixtures.  GPU tests carry the `gpu` marker; everything else runs on the CPU."""
import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "ref_literals.json")
    return {c["name"]: c for c in json.load(open(path))["cases"]}


@pytest.fixture(scope="session")
def orc():
    import oracle
    if not os.path.exists(oracle.LIB_ORACLE):
        oracle.build()
    return oracle.Oracle("orc")


@pytest.fixture(scope="session")
def orc64():
    import oracle
    if not os.path.exists(oracle.LIB_ORACLE):
        oracle.build()
    return oracle.Oracle("orc", f64=True)


@pytest.fixture(scope="session")
def ref():
    import oracle
    if not oracle.have_ref():
        pytest.skip("oracle/_ref/libdcgan_ref.so not built (reference tree absent)")
    return oracle.Oracle("ref")
