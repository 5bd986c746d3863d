"""GPU: the HIP backend, through its C ABI, against the reference's own known-answer vectors."""
import pytest

import kat

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("case", kat.ALL, ids=lambda f: f.__name__)
def test_hip_matches_reference_vectors(hip, case, dt):
    case(hip, dt)
