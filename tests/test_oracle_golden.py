"""CPU: the oracle (oracle/liboracle.so) against the reference's own known-answer vectors."""
import pytest

import kat


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16", "f64"])
@pytest.mark.parametrize("case", kat.ALL, ids=lambda f: f.__name__)
def test_oracle_matches_reference_vectors(oracle, case, dt):
    case(oracle, dt)


@pytest.mark.parametrize("dt", kat.INT_DTYPES + ["bool"])
def test_oracle_matches_reference_integer_and_bool_vectors(oracle, dt):
    kat.run_binary_wide(oracle, dt)
