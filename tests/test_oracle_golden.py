"""The CPU oracle against the literal vectors the reference's own tests hold."""
import pytest

from helpers import golden_cases, run_golden_case


@pytest.mark.parametrize("case", golden_cases(), ids=lambda c: c["op"] + "@" + c["source"].split(" ")[0])
def test_oracle_matches_reference_vectors(oracle_backend, case):
    assert run_golden_case(oracle_backend, case) == []


def test_reference_heap_topk_matches_vectors():
    # the restated heap algorithm (mode 0) must give the same tie-free golden answer
    from oracle.oracle import OracleBackend
    be = OracleBackend(topk_mode=0)
    for case in golden_cases():
        if case["op"] == "top_k":
            assert run_golden_case(be, case) == []
