"""The CPU oracle against the reference's own known-answer vectors (no GPU involved)."""
import pytest

import golden_checks


@pytest.mark.parametrize("check", golden_checks.ALL_CHECKS, ids=lambda f: f.__name__)
def test_oracle_matches_reference_vectors(oracle, check):
    check(oracle)


@pytest.mark.parametrize("check", golden_checks.ALL_CHECKS, ids=lambda f: f.__name__)
def test_oracle_builtin_blas_matches_reference_vectors(oracle, check):
    """Same vectors with the BLAS-free loops, the path used when no BLAS library is found."""
    oracle.force_builtin_blas(True)
    try:
        check(oracle)
    finally:
        oracle.force_builtin_blas(False)
