"""Writes tests/golden/oracle_manifest_names.json: the tensor names, dtypes and shapes (no payloads: the reference
repository holds none) that the reference oracle's own manifests list for two of its sets, with their `state_heads`
notes. The loader's naming rules are tested against these real names.

Run from the repository root where the reference is checked out:
    python tests/golden/make_manifest_fixture.py /root/reference/oracle/goldens
"""
import json
import os
import sys

SETS = ("layer00-prefill", "layer04-decode")


def main(root):
    out = {}
    for name in SETS:
        with open(os.path.join(root, name, "manifest.json"), "r", encoding="utf-8") as f:
            doc = json.load(f)
        out[name] = {
            "state_heads": doc.get("notes", {}).get("state_heads"),
            "tensors": {k: {"dtype": v["dtype"], "shape": v["shape"]} for k, v in doc["tensors"].items()},
        }
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_manifest_names.json")
    with open(dst, "w", encoding="utf-8") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print(f"wrote {dst}: {sum(len(v['tensors']) for v in out.values())} tensor entries")


if __name__ == "__main__":
    main(sys.argv[1])
