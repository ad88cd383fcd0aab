"""The reference's own known answers (tests/golden/nx_known_answers.json), run on the device
backend through the C ABI."""
import pytest

from support import check_case, load_cases

pytestmark = pytest.mark.gpu
CASES = load_cases()


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_device_matches_reference_known_answer(case, hip):
    from nx_amd._lib import HipNxArgumentError
    check_case(case, hip, (HipNxArgumentError, ValueError))
