"""CPU: the oracle (and the device-free layout algebra) against every known-answer vector the reference's own documentation
and docstrings hold for this path (tests/golden/reference_vectors.json)."""
import pytest

from golden_ops import check_vector, load_vectors

VECTORS = load_vectors()


@pytest.mark.parametrize("vec", VECTORS, ids=[v["id"] for v in VECTORS])
def test_oracle_matches_reference_vector(H, vec):
    check_vector(H, vec)
