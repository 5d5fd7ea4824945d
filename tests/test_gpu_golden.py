"""The hip backend (through the C ABI) against the reference's own known-answer vectors."""
import pytest

from golden_recipes import RECIPES

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from providers import HipOps
    return HipOps()


@pytest.mark.parametrize("case", RECIPES, ids=[r.__name__ for r in RECIPES])
def test_hip_matches_reference_vectors(ops, case):
    print("case:", case.__name__, flush=True)
    case(ops)
