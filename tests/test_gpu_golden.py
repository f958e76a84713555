"""HIP kernels, through the C ABI, on the literal inputs of the reference's own operator tests."""
import pytest

from common import GOLDEN_NAMES, check_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    import __graft_entry__ as ge
    return ge.load_package().HipBackend(0)


@pytest.mark.parametrize("name", GOLDEN_NAMES)
def test_gpu_golden(be, golden, name):
    print("case", name, flush=True)
    check_case(be, golden[name])
