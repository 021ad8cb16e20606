"""The HIP device against the same closed forms, brute-force loops and invariants that pin the oracle."""
import pytest

import closed_form_checks as cf

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("check", cf.ALL_CHECKS, ids=lambda f: f.__name__)
def test_device_matches_closed_forms(hip, check):
    check(hip)
