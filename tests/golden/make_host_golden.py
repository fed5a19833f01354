"""Generate tests/golden/host_traces.json from the COMPILED REFERENCE.

Runs in the authoring container only (needs the reference checkout to build
oracle/_ref; see oracle/build_ref.py).  The fixture holds, for every scenario
in tests/scenarios.py, the scenario itself and the trace of return values the
reference's own KVStorage / BatchScheduler (csrc/memory_manager.cpp,
csrc/batch_scheduler.cpp) produced for it.  Data only: no reference source is
stored.

    python tests/golden/make_host_golden.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import build_ref  # noqa: E402
import scenarios  # noqa: E402

N_RANDOM = 24


def main():
    mm, bsm = build_ref.load()
    if mm is None:
        build_ref.build()
        mm, bsm = build_ref.load()
    out = {}
    all_sc = dict(scenarios.scripted_scenarios())
    for seed in range(N_RANDOM):
        all_sc[f"random_{seed:02d}"] = scenarios.random_scenario(seed)
    for name, sc in all_sc.items():
        trace = scenarios.run_scenario(mm.KVStorage, bsm.BatchScheduler, sc)
        out[name] = {"scenario": sc, "trace": trace}
        print(f"{name}: {len(sc['ops'])} ops, {len(trace)} trace records")
    path = os.path.join(HERE, "host_traces.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
