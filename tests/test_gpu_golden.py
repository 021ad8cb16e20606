"""The HIP device against the reference's own known-answer vectors, through the C ABI."""
import pytest

import golden_checks

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("check", golden_checks.ALL_CHECKS, ids=lambda f: f.__name__)
def test_hip_matches_reference_vectors(hip, check):
    check(hip)
