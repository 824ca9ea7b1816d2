"""Writes tests/golden/affinity_cases.json: what the reference's
AffinityManager.parse_affinity and AffinityManager.num_cpus_for_gpu return (or
raise) for the inputs listed here.  These two are the pure parts of
tspipe/affinity_manager.py; the rest of the class shells out to nvidia-smi and
taskset and cannot run without them.

Run once in the build container, where the reference is mounted at
/root/reference; the JSON it writes is the committed fixture.
"""
import json
import os
import sys

sys.path.insert(0, "/root/reference")
from tspipe.affinity_manager import AffinityManager  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

PARSE = ["0-3,8,10-11", "5", "0-15", "16-31,48-63", "7,3,1", "3-3", "5-2", "", "a-b", "1-", "1,,2", "0-3 ", "-1", "1-2-3"]

MAPS = [
    {"0": "0-15", "1": "0-15", "2": "16-31", "3": "40-42,50-52"},
    {"0": "0-5", "1": "0-5", "2": "0-5", "3": "0-5"},
    {"0": "0-7", "1": "4-11"},
    {"0": "0-63"},
    {"0": "0-2", "1": "0-2", "2": "0-2", "3": "0-2"},
    {"0": "0-23", "1": "0-23", "2": "24-47", "3": "24-47", "4": "0-47"},
]


def attempt(fn, *args):
    try:
        return {"value": fn(*args)}
    except Exception as exc:  # the class of the exception is the recorded behaviour
        return {"raises": type(exc).__name__}


def main():
    cases = {"parse": [{"text": t, **attempt(AffinityManager.parse_affinity, t)} for t in PARSE], "demand": []}
    for spec in MAPS:
        lists = {int(g): AffinityManager.parse_affinity(t) for g, t in spec.items()}
        cases["demand"].append({"lists": spec,
                                "cores": {g: attempt(AffinityManager.num_cpus_for_gpu, int(g), lists) for g in spec}})
    with open(os.path.join(HERE, "affinity_cases.json"), "w") as fh:
        json.dump(cases, fh, indent=1, sort_keys=True)
    print(len(cases["parse"]), "parse cases,", len(cases["demand"]), "maps")


if __name__ == "__main__":
    main()
