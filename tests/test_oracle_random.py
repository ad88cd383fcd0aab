"""The oracle backend under the `Nx.Random` mirror against the reference's own known answers:
twenty rounds of u32 add / xor / shift / or over iota, concatenate, slice, as_type and bitcast pin
those callbacks of the oracle far beyond their doctests (one wrong bit anywhere changes every
output word)."""
import pytest

from random_support import CASES, check_random_case


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_oracle_matches_reference_random_known_answer(case, oracle):
    check_random_case(case, oracle)
