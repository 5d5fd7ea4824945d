"""The CPU oracle against the reference's own known-answer vectors (no GPU needed)."""
import pytest

from golden_recipes import RECIPES
from providers import OracleOps


@pytest.fixture(scope="module")
def ops(oracle):
    return OracleOps()


@pytest.mark.parametrize("case", RECIPES, ids=[r.__name__ for r in RECIPES])
def test_oracle_matches_reference_vectors(ops, case):
    case(ops)
