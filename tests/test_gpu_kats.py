"""The reference's own literal cases (tests/golden/reference_kats.json) through the
C-ABI on the device."""
import pytest

import kat

pytestmark = pytest.mark.gpu
CASES = kat.load_cases()


@pytest.mark.parametrize("tc", CASES, ids=[kat.case_id(tc) for tc in CASES])
def test_reference_literals_on_device(tc):
    import cumo_amd
    t, c = tc
    kat.check(t, c, kat.run_device(t, c, cumo_amd))
