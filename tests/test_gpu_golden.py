"""GPU: the HIP backend, through the C ABI, against the reference's documentation/docstring vectors."""
import pytest

from golden_ops import check_vector, load_vectors

pytestmark = pytest.mark.gpu
VECTORS = load_vectors()


@pytest.mark.parametrize("vec", VECTORS, ids=[v["id"] for v in VECTORS])
def test_hip_matches_reference_vector(G, vec):
    check_vector(G, vec)
