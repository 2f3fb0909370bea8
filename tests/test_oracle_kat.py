"""The oracle against the committed known-answer vectors (exact rational arithmetic from the
operators' definitions, tests/golden/make_golden.py).  Bit-exact."""
import os
import subprocess
import sys

import pytest

import kat_runner
from util import assert_bit_exact, load_kat

CASES = load_kat()


@pytest.mark.parametrize("case", CASES, ids=[kat_runner.case_id(c) for c in CASES])
def test_oracle_matches_known_answer(case):
    got = kat_runner.run_oracle(case)
    assert_bit_exact(got, kat_runner.expected(case), case["op"])


def test_known_answers_are_reproducible(tmp_path):
    """The committed fixture is what the committed generator writes."""
    here = os.path.dirname(os.path.abspath(__file__))
    script = os.path.join(here, "golden", "make_golden.py")
    src = open(script).read().replace('os.path.join(HERE, "kat.json")', repr(str(tmp_path / "kat.json")))
    gen = tmp_path / "gen.py"
    gen.write_text(src)
    subprocess.run([sys.executable, str(gen)], check=True, stdout=subprocess.DEVNULL)
    assert (tmp_path / "kat.json").read_text() == open(os.path.join(here, "golden", "kat.json")).read()
