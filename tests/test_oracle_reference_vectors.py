"""The CPU oracle against every known-answer vector and invariant the reference's own
backend test-suite holds for the hot path (no GPU needed)."""
import pytest

import backend_cases


@pytest.mark.parametrize("case", backend_cases.ALL_CASES, ids=lambda f: f.__name__)
def test_oracle_case(case, oracle_backend, rng):
    with oracle_backend.use():
        if "rng" in case.__code__.co_varnames[:case.__code__.co_argcount]:
            case(rng)
        else:
            case()
