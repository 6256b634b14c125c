"""Writes ``codegen_snapshots.json``: for every end-to-end case, what the emitter decides for the
best candidates of the search -- the manifest (parameters in call order, launches with grid, block
and LDS bytes) and the ``#define`` block in front of each template body -- as one sha256 per
candidate, with the candidate's label beside it.  Template bodies are left out on purpose: a
comment edited in a kernel is not a change of the emitter.

    python tests/golden/make_codegen_snapshots.py          # rewrite the file after a deliberate change

The reference keeps the same kind of record for its TileLang sources
(``tests/pipeline/test_pipeline_snapshots.py``, ``tests/pipeline/_pipeline.py:101-138``).
"""

import hashlib
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

WHERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "codegen_snapshots.json")
TOPK = 4
UNIT = "// ---- template:"


def decisions(source: str) -> str:
    """The manifest comment and, for every unit of the source, its header line and the defines
    that follow it directly."""
    kept, state = [], "before"
    for row in source.splitlines():
        if row.startswith("// CLEAVE-HIP-MANIFEST-BEGIN"):
            state = "manifest"
        elif row.startswith("// CLEAVE-HIP-MANIFEST-END"):
            state = "between"
        elif row.startswith(UNIT):
            state = "defines"
            kept.append(row)
        elif state == "manifest" or (state == "defines" and row.startswith("#define CL_")):
            kept.append(row)
        elif state == "defines":
            state = "between"
    return "\n".join(kept)


def snapshot() -> dict:
    from cleave_amd.codegen import HipCodeGen
    from cleave_amd.schedule import apply_tiling, search_tiling
    from tests._end2end_cases import CASES, flat_graph

    record = {}
    for name in sorted(CASES):
        rows = []
        for cand in search_tiling(flat_graph(name), topk=TOPK):
            text = decisions(HipCodeGen().gen(apply_tiling(cand)))
            rows.append({"label": f"{cand.template} {dict(cand.tiling)}", "sha256": hashlib.sha256(text.encode()).hexdigest()})
        record[name] = rows
    return record


if __name__ == "__main__":
    with open(WHERE, "w") as out:
        json.dump(snapshot(), out, indent=1, sort_keys=True)
        out.write("\n")
    print(f"wrote {WHERE}")
