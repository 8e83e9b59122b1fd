"""HIPBackend against the reference's own backend test-suite vectors (through the C ABI)."""
import pytest

import backend_cases

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", backend_cases.ALL_CASES, ids=lambda f: f.__name__)
def test_hip_case(case, hip_backend, rng):
    print("case", case.__name__, flush=True)
    with hip_backend.use():
        if "rng" in case.__code__.co_varnames[:case.__code__.co_argcount]:
            case(rng)
        else:
            case()
    hip_backend.sync()
