"""The rational fixtures catch one-line mistakes in the oracle: every edit listed in ``tests/oracle_mutations.py`` is applied
to a copy of ``oracle/pmetal_oracle.c``, the copy is built, and at least one case of ``tests/golden/exact_cases.json`` must
then fail -- with nothing but the fixture and the edited library taking part (no other test of the suite is needed to see
the mistake).  The unedited source passes every case; the edits listed as equivalent pass every case too."""
import json
import os

import pytest

import oracle_mutations as M

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = json.load(open(os.path.join(HERE, "golden", "exact_cases.json")))


@pytest.fixture(scope="module")
def workdir(tmp_path_factory):
    return str(tmp_path_factory.mktemp("oracle_mutants"))


def test_the_unedited_oracle_passes_every_fixture_case(workdir):
    assert M.failing_cases(M.build(open(M.ORACLE_C).read(), workdir, "unedited"), CASES) == []


@pytest.mark.parametrize("name,item,ref,edits", M.MUTATIONS, ids=[m[0] for m in M.MUTATIONS])
def test_fixture_catches(workdir, name, item, ref, edits):
    bad = M.failing_cases(M.build(M.mutated_source(name), workdir, name), CASES)
    assert bad, f"no fixture case notices the edit of {ref} ({name})"


def test_every_checklist_item_has_an_edit():
    assert {m[1] for m in M.MUTATIONS} >= set(range(1, 12))


@pytest.mark.parametrize("name,ref,edits,why", M.EQUIVALENT, ids=[m[0] for m in M.EQUIVALENT])
def test_equivalent_edits_change_nothing_the_fixture_sees(workdir, name, ref, edits, why):
    assert M.failing_cases(M.build(M.edited_source(edits, name), workdir, name), CASES) == []
