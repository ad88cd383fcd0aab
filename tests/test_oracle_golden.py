"""Pins the CPU oracle (oracle/) against the known answers the reference's own doctests and tests
hold for the hot path (tests/golden/nx_known_answers.json, each with its file:line source)."""
import pytest

from support import check_case, load_cases

CASES = load_cases()


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_oracle_matches_reference_known_answer(case, oracle):
    from oracle.binary_backend import ReferenceRaises
    check_case(case, oracle, (ReferenceRaises, ValueError))
