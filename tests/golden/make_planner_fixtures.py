"""Writes tests/golden/planner_profiles.json: the per-layer measurements (forward / backward ms, activation and parameter
bytes) and the edges of two of the profile data files the reference ships under profiling_results/, as plain arrays.
Inputs of tests/test_planner.py.  Run in the build container, where the reference tree is mounted:

    python tests/golden/make_planner_fixtures.py /root/reference/profiling_results
"""
import json
import os
import sys

NAMES = ["vgg-19-pbs-32", "bert-48-pbs-2", "xlnet-36-pbs-1"]


def read(path):
    nodes, edges = [], []
    for line in open(path):
        if not line.strip():
            continue
        if line.startswith((" ", "\t")):
            a, b = line.strip().split(" -- ")
            edges.append([a, b])
        else:
            node_id, desc, meta = line.strip().split(" -- ")[:3]
            vals = [m.split("=", 1)[1] for m in meta.split(", ")]
            nodes.append([node_id, desc] + vals)          # values kept as the strings the file holds
    return {"nodes": nodes, "edges": edges}


if __name__ == "__main__":
    src = sys.argv[1]
    out = {n: read(os.path.join(src, n + ".txt")) for n in NAMES}
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "planner_profiles.json")
    with open(dst, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", dst, {n: (len(v["nodes"]), len(v["edges"])) for n, v in out.items()})
