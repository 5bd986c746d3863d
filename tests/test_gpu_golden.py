"""GPU: the HIP backend, through its C ABI, against the reference's own known-answer vectors."""
import pytest

import kat

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("case", kat.ALL, ids=lambda f: f.__name__)
def test_hip_matches_reference_vectors(hip, case, dt):
    case(hip, dt)


@pytest.mark.parametrize("dt", kat.INT_DTYPES + ["bool", "f64"])
def test_hip_matches_reference_integer_bool_and_f64_vectors(hip, dt):
    if dt == "f64":
        for case in (kat.run_binary, kat.run_compare, kat.run_inplace):
            case(hip, dt)
    else:
        kat.run_binary_wide(hip, dt)
