#!/usr/bin/env python3
"""Writes ``schedule_tables.json``: task tables produced by the reference's
own ``src/jaxpp/schedules.py``.

Only that one file of the reference is loaded.  Its sole import from the rest
of the package (``MpmdIdx`` and ``TaskType`` from ``jaxpp.types``, which pulls
in jax) is satisfied by a stand-in module holding those two definitions, so
nothing else of the reference runs.  Run in the build container:

    python tests/golden/make_schedule_fixtures.py [/root/reference]

The fixture holds data only.  Small cases are stored as full tables; large
ones as the SHA-256 of the same canonical JSON.

Encoding: a table is a list of rows (one per rank); an entry is ``null`` for
a bubble slot, ``[stage, microbatch, KIND, latency]`` for a task, or
``{"fused": [task, ...]}`` for a fused group.
"""
from __future__ import annotations

import enum
import hashlib
import importlib.util
import json
import os
import sys
import types
from typing import NewType

HERE = os.path.dirname(os.path.abspath(__file__))


def load_reference_schedules(root: str):
    class TaskType(enum.Enum):
        FWD = 1
        BWD = 2
        BWD_I = 3
        BWD_W = 4

        @property
        def default_latency(self):
            return 2 if self is TaskType.BWD else 1

    pkg = types.ModuleType("jaxpp")
    pkg.__path__ = []
    stub = types.ModuleType("jaxpp.types")
    stub.MpmdIdx = NewType("MpmdIdx", int)
    stub.TaskType = TaskType
    sys.modules["jaxpp"] = pkg
    sys.modules["jaxpp.types"] = stub
    path = os.path.join(root, "src", "jaxpp", "schedules.py")
    spec = importlib.util.spec_from_file_location("jaxpp.schedules", path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules["jaxpp.schedules"] = mod
    spec.loader.exec_module(mod)
    return mod


def encode_entry(mod, e):
    if e is None:
        return None
    if isinstance(e, mod.FusedTask):
        return {"fused": [encode_entry(mod, t) for t in e]}
    return [e.stage_id, e.mubatch_idx, e.fwd_or_bwd.name, e.latency]


def encode_table(mod, table):
    return [[encode_entry(mod, e) for e in row] for row in table]


def digest(obj) -> str:
    blob = json.dumps(obj, separators=(",", ":"), sort_keys=True).encode()
    return hashlib.sha256(blob).hexdigest()


# (class name, constructor kwargs, n_mubatches, store full table?)
CASES = [
    # the five benchmark configurations
    ("Std1F1B", {"num_stages": 2}, 8, True),
    ("Std1F1B", {"num_stages": 4}, 16, True),
    ("Interleaved1F1B", {"num_stages": 8, "mpmd_dim": 4}, 32, True),
    ("ZeroBubble", {"num_stages": 8}, 24, True),
    ("DualPipeV", {"num_stages": 8, "mpmd_dim": 4}, 16, True),
    # the reference's own test grid (tests/test_transformations.py:140-155, :194-200)
    ("Std1F1B", {"num_stages": 1}, 4, True),
    ("Std1F1B", {"num_stages": 2}, 4, True),
    ("Eager1F1B", {"num_stages": 3}, 5, True),
    ("Interleaved1F1B", {"num_stages": 1, "mpmd_dim": 1}, 1, True),
    ("Interleaved1F1B", {"num_stages": 8, "mpmd_dim": 4}, 1, True),
    ("KimiK2", {"num_stages": 8, "mpmd_dim": 4, "fuse_steady_state": True}, 1, True),
    ("Interleaved1F1B", {"num_stages": 4, "mpmd_dim": 2}, 12, True),
    ("ZeroBubble", {"num_stages": 4}, 4, True),
    ("ZeroBubble", {"num_stages": 4}, 8, True),
    ("DualPipeV", {"num_stages": 6, "mpmd_dim": 3}, 6, True),
    ("DualPipeV", {"num_stages": 6, "mpmd_dim": 3}, 10, True),
    ("Interleaved1F1B", {"num_stages": 48, "mpmd_dim": 8}, 64, False),
    ("DualPipeV", {"num_stages": 16, "mpmd_dim": 8}, 18, False),
    # tests/test_schedules.py:35-66
    ("Eager1F1B", {"num_stages": 2}, 4, True),
    ("Interleaved1F1B", {"num_stages": 2, "mpmd_dim": 1}, 4, True),
    ("ZeroBubble", {"num_stages": 2}, 4, True),
    # the notebook's printed cases (examples/tutorial.ipynb)
    ("Interleaved1F1B", {"num_stages": 4, "mpmd_dim": 4}, 4, True),
    ("Interleaved1F1B", {"num_stages": 8, "mpmd_dim": 4}, 4, True),
    # unexported but present
    ("GPipe", {"num_stages": 3}, 5, True),
    ("KimiK2", {"num_stages": 8, "mpmd_dim": 4}, 16, False),
    ("Interleaved1F1B", {"num_stages": 8, "mpmd_dim": 4, "fuse_steady_state": True}, 8, False),
    ("Interleaved1F1B", {"num_stages": 12, "mpmd_dim": 4}, 6, False),
]

# digest-only sweeps over small shapes
for S in range(1, 7):
    for n in range(1, 11):
        CASES.append(("Std1F1B", {"num_stages": S}, n, False))
        CASES.append(("Eager1F1B", {"num_stages": S}, n, False))
        CASES.append(("GPipe", {"num_stages": S}, n, False))
        if S >= 2 and n >= S:
            CASES.append(("ZeroBubble", {"num_stages": S}, n, False))
for P in range(1, 6):
    for n in range(2 * P, 2 * P + 9):
        CASES.append(("DualPipeV", {"num_stages": 2 * P, "mpmd_dim": P}, n, False))
    for vp in (1, 2, 3):
        for n in (P, 2 * P, 3 * P, 4 * P):
            CASES.append(("Interleaved1F1B", {"num_stages": vp * P, "mpmd_dim": P}, n, False))
            CASES.append(("KimiK2", {"num_stages": vp * P, "mpmd_dim": P}, n, False))


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    mod = load_reference_schedules(root)
    out = []
    seen = set()
    for cls_name, kwargs, n, full in CASES:
        key = (cls_name, json.dumps(kwargs, sort_keys=True), n)
        if key in seen:
            continue
        seen.add(key)
        sched = getattr(mod, cls_name)(**kwargs)
        raw = encode_table(mod, sched.tasks(n))
        rec = {"schedule": cls_name, "kwargs": kwargs, "n_mubatches": n,
               "is_partial_bwd": bool(sched.is_partial_bwd),
               "mpmd_idx_of_stage": [int(sched.get_mpmd_idx(s))
                                     for s in range(kwargs["num_stages"])],
               "raw_sha256": digest(raw)}
        for unpack in (False, True):
            tag = "unpacked" if unpack else "fused"
            try:
                pre = encode_table(mod, mod.preprocess_schedule_tasks(
                    sched.tasks(n), 0, unpack))
            except NotImplementedError:
                rec[f"pre_{tag}_error"] = "NotImplementedError"
                continue
            rec[f"pre_{tag}_sha256"] = digest(pre)
            if full:
                rec[f"pre_{tag}"] = pre
        if full:
            rec["raw"] = raw
        out.append(rec)
    path = os.path.join(HERE, "schedule_tables.json")
    with open(path, "w") as f:
        json.dump({"source": "NVIDIA/jaxpp v0.9.2 src/jaxpp/schedules.py",
                   "cases": out}, f, separators=(",", ":"))
    print(f"{len(out)} cases -> {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
