"""Writes the committed fixtures under tests/golden/ from the data files the reference's own tests
hold.  Runs only in the authoring container (needs /root/reference); the reference files are read
as text and never imported or executed.

    python tests/golden/make_fixtures.py
"""
import ast
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/prefilling_dllm_engine"


def mimic_slot_mapping():
    """examples/mimic_data/mimic_slot_mapping.py: a literal slot-mapping list (−1 = skip) used by
    examples/test_dllm_kv_cache_load.py.  Stored run-length encoded."""
    src = open(os.path.join(REF, "examples/mimic_data/mimic_slot_mapping.py")).read()
    lst = ast.literal_eval(src.split("=", 1)[1].strip())
    runs, i = [], 0
    while i < len(lst):
        j = i
        if lst[i] < 0:
            assert lst[i] == -1
            while j < len(lst) and lst[j] == -1:
                j += 1
            runs.append(["skip", 0, j - i])
            i = j
        else:
            while j + 1 < len(lst) and lst[j + 1] == lst[j] + 1:
                j += 1
            runs.append(["run", lst[i], j - i + 1])
            i = j + 1
    out = {"source": "examples/mimic_data/mimic_slot_mapping.py", "length": len(lst), "runs": runs}
    with open(os.path.join(HERE, "mimic_slot_mapping.json"), "w") as f:
        json.dump(out, f, indent=1)


if __name__ == "__main__":
    mimic_slot_mapping()
    print("fixtures written to", HERE)
