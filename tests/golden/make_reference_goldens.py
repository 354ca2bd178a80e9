#!/usr/bin/env python3
"""Writes tests/golden/reference_goldens.json by running oracle/_ref/ref_kv_probe, the
driver built (oracle/Makefile, target `ref`) from the reference's own host sources.

The fixture holds data only -- inputs and the values the reference's classes produced:
  * ledger: KV reservations, arena size, num_blocks, BackboneDeviceBytes for a set of
    (block_size, max_context) pairs (reference StaticArenaManager on its mock runtime);
  * arena_scripts: seeded random Reserve sequences replayed on the reference
    StaticMemoryArena (offsets, refusals, committed size);
  * arena_contract: the observable outcomes of the reference's TestStaticArena sequence
    (tests/mock_contract_smoke.cpp:533-584);
  * stats: KV diagnostics (src/pipeline/pipeline.cpp:134-136, :532-534) incl. the values
    the reference's own tests and docs hold (86 blocks @128/256; 129 tokens @ 8192).

Run in the build container (needs /root/reference):  python tests/golden/make_reference_goldens.py
"""
import json
import os
import random
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
PROBE = os.path.join(ROOT, "oracle", "_ref", "ref_kv_probe")


def probe(*args):
    out = subprocess.run([PROBE, *map(str, args)], check=True, capture_output=True, text=True).stdout
    return json.loads(out)


def main():
    if not os.path.exists(PROBE):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-j8", "ref"], check=True)
    golden = {"generator": "tests/golden/make_reference_goldens.py", "ledger": [], "arena_scripts": [], "stats": []}
    for block_size, max_context in [(64, 8192), (64, 2048), (64, 2000), (64, 32768), (128, 8192), (128, 256),
                                    (128, 32768), (16, 4096), (64, 64)]:
        golden["ledger"].append(probe("ledger", block_size, max_context))
    rng = random.Random(20251125)
    for _ in range(24):
        steps = []
        for _ in range(rng.randint(1, 12)):
            kind = rng.random()
            if kind < 0.08:
                steps.append((0, 512))                      # empty: refused
            elif kind < 0.16:
                steps.append((rng.randint(1, 5000), rng.choice([3, 6, 48, 1000])))  # non power of two: refused
            else:
                steps.append((rng.randint(1, 70000), rng.choice([1, 2, 16, 32, 64, 128, 256, 512, 1024, 4096])))
        result = probe("arena-script", len(steps), *[f"{b},{a}" for b, a in steps])
        golden["arena_scripts"].append({"script": steps, "result": result})
    golden["arena_contract"] = probe("arena-contract")
    for block_size, max_context, position in [(128, 256, 1), (128, 8192, 128), (64, 8192, 127), (64, 8192, 128),
                                              (64, 2048, 2047), (64, 2000, 0), (128, 100, 0), (0, 128, 0)]:
        golden["stats"].append({"block_size": block_size, "max_context": max_context, "position": position,
                                "result": probe("stats", block_size, max_context, position)})
    path = os.path.join(HERE, "reference_goldens.json")
    with open(path, "w") as handle:
        json.dump(golden, handle, indent=1, sort_keys=True)
        handle.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    sys.exit(main())
