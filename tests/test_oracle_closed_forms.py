"""The CPU oracle against closed forms, brute force and invariants (no GPU involved), and the completeness of the
routine -> check table: every routine the oracle declares is pinned by at least one check that exists."""
import re
from pathlib import Path

import pytest

import closed_form_checks as cf
import golden_checks

ROOT = Path(__file__).resolve().parents[1]


@pytest.mark.parametrize("check", cf.ALL_CHECKS, ids=lambda f: f.__name__)
def test_oracle_matches_closed_forms(oracle, check):
    check(oracle)


@pytest.mark.parametrize("check", cf.ALL_CHECKS, ids=lambda f: f.__name__)
def test_oracle_builtin_blas_matches_closed_forms(oracle, check):
    """Same checks with the BLAS-free loops, the path taken when no BLAS library is found."""
    oracle.force_builtin_blas(True)
    try:
        check(oracle)
    finally:
        oracle.force_builtin_blas(False)


def _declared_routines():
    text = (ROOT / "oracle" / "zg_oracle.h").read_text()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return set(re.findall(r"\b(zo_\w+)\s*\(", text))


def test_every_oracle_routine_is_pinned():
    declared = _declared_routines()
    assert len(declared) >= 70
    assert cf.UNPINNED == set()  # no routine of the oracle is left without an independent check
    covered = set(cf.PINS) | cf.UNPINNED | cf.NOT_ARITHMETIC
    assert declared - covered == set(), f"routines without a pin: {sorted(declared - covered)}"
    assert set(cf.PINS) - declared == set(), f"pins for routines that do not exist: {sorted(set(cf.PINS) - declared)}"
    closed = {f.__name__ for f in cf.ALL_CHECKS}
    golden = {f.__name__ for f in golden_checks.ALL_CHECKS}
    train = set(re.findall(r"^def (test_\w+)", (ROOT / "tests" / "test_oracle_train.py").read_text(), flags=re.M))
    for routine, pins in cf.PINS.items():
        assert pins, routine
        for pin in pins:
            kind, _, name = pin.rpartition(":")
            pool = {"": closed, "golden": golden, "train": train}[kind]
            assert name in pool, f"{routine}: {pin} names no existing check"
        # at least one pin of every routine is a closed form or one of the reference's own vectors
        assert any(not p.startswith("train:") for p in pins), routine
