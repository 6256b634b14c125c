"""What the emitter decides for the best candidates of every end-to-end case, against the stored
record (``tests/golden/codegen_snapshots.json``, written by ``tests/golden/make_codegen_snapshots.py``).

A difference here is a changed search order, tiling, parameter list, launch geometry or define
block; after a deliberate change the record is rewritten with the script.  The reference keeps
the same kind of record of its generated sources (``tests/pipeline/test_pipeline_snapshots.py``).
"""

import json

import pytest

from .golden import make_codegen_snapshots as maker


@pytest.fixture(scope="module")
def now():
    return maker.snapshot()


def stored():
    with open(maker.WHERE) as handle:
        return json.load(handle)


def test_every_case_of_the_list_is_recorded(now):
    assert sorted(now) == sorted(stored())
    assert all(now[name] for name in now), "a case the search proposes nothing for"


@pytest.mark.parametrize("name", sorted(stored()))
def test_candidates_and_their_emitted_decisions_are_the_recorded_ones(name, now):
    want, got = stored()[name], now[name]
    assert [row["label"] for row in got] == [row["label"] for row in want], "the search ranks other candidates first"
    changed = [g["label"] for g, w in zip(got, want) if g["sha256"] != w["sha256"]]
    assert not changed, f"manifest or defines differ from the record for {changed}"


def test_template_bodies_are_not_part_of_the_record():
    source = ("// CLEAVE-HIP-MANIFEST-BEGIN\n// {\n// }\n// CLEAVE-HIP-MANIFEST-END\n// ---- template: t  role: main  x\n"
              "#define CL_A 1\n// a comment of the body\n#define CL_B 2\nint body;\n")
    assert maker.decisions(source) == "// {\n// }\n// ---- template: t  role: main  x\n#define CL_A 1"
