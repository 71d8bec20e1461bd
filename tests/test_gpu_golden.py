"""The HIP path against the literal vectors the reference's own tests hold."""
import pytest

from helpers import golden_cases, run_golden_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", golden_cases(), ids=lambda c: c["op"] + "@" + c["source"].split(" ")[0])
def test_hip_matches_reference_vectors(hip_backend, case):
    assert run_golden_case(hip_backend, case) == []
