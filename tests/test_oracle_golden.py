"""The oracle against the literal inputs of the reference's own operator tests
(tests/golden/ref_literals.json; expected values computed in float64 by torch / numpy)."""
import pytest

from common import GOLDEN_NAMES, check_case


@pytest.mark.parametrize("name", GOLDEN_NAMES)
def test_oracle_golden(orc, golden, name):
    check_case(orc, golden[name], rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("name", GOLDEN_NAMES)
def test_oracle_f64_golden(orc64, golden, name):
    check_case(orc64, golden[name], rtol=2e-6, atol=1e-6)


# The reference's CPU transpose-gradient functions are VALID-only; the literal of
# tests/test_conv2d_transpose_grad.cu is such a shape, so the reference build covers it too.
@pytest.mark.parametrize("name", [n for n in GOLDEN_NAMES])
def test_reference_build_golden(ref, golden, name):
    check_case(ref, golden[name], rtol=2e-6, atol=1e-6)
