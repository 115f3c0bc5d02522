"""Schedule task tables: bit-exact against tables emitted by the reference's
schedules.py (tests/golden/schedule_tables.json), the notebook's printed
vectors, and the structural / error-message checks of the reference's
tests/test_schedules.py."""
import hashlib
import json
import os

import pytest

from jaxpp_amd import schedules as S
from jaxpp_amd.types import TaskType

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "schedule_tables.json")
with open(GOLDEN) as f:
    CASES = json.load(f)["cases"]


def enc(e):
    if e is None:
        return None
    if isinstance(e, S.FusedTask):
        return {"fused": [enc(t) for t in e]}
    return [e.stage_id, e.mubatch_idx, e.fwd_or_bwd.name, e.latency]


def enc_table(t):
    return [[enc(e) for e in row] for row in t]


def digest(obj):
    return hashlib.sha256(
        json.dumps(obj, separators=(",", ":"), sort_keys=True).encode()).hexdigest()


def case_id(c):
    kw = ",".join(f"{k}={v}" for k, v in c["kwargs"].items())
    return f"{c['schedule']}({kw})x{c['n_mubatches']}"


@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_tables_match_reference(case):
    sched = getattr(S, case["schedule"])(**case["kwargs"])
    n = case["n_mubatches"]
    assert bool(sched.is_partial_bwd) == case["is_partial_bwd"]
    assert [int(sched.get_mpmd_idx(s)) for s in range(case["kwargs"]["num_stages"])] \
        == case["mpmd_idx_of_stage"]
    raw = enc_table(sched.tasks(n))
    if "raw" in case:
        assert raw == case["raw"]
    assert digest(raw) == case["raw_sha256"]
    for unpack, tag in ((False, "fused"), (True, "unpacked")):
        if f"pre_{tag}_error" in case:
            with pytest.raises(NotImplementedError):
                S.preprocess_schedule_tasks(sched.tasks(n), 0, unpack)
            continue
        pre = enc_table(S.preprocess_schedule_tasks(sched.tasks(n), 0, unpack))
        if f"pre_{tag}" in case:
            assert pre == case[f"pre_{tag}"]
        assert digest(pre) == case[f"pre_{tag}_sha256"]


def names(row):
    return [str(t) for t in row]


def test_notebook_vectors():
    # examples/tutorial.ipynb:473-480, :513-516, :630-645, :670-681
    t = S.Interleaved1F1B(num_stages=4, mpmd_dim=4).tasks(4)
    assert names(t[2]) == ["fwd_2__0", "fwd_2__1", "fwd_2__2", "bwd_2__0",
                           "fwd_2__3", "bwd_2__1", "bwd_2__2", "bwd_2__3"]
    assert names(t[3]) == [f"FusedTask(fwd_3__{i}, bwd_3__{i})" for i in range(4)]
    t = S.Interleaved1F1B(num_stages=8, mpmd_dim=4).tasks(4)
    assert names(t[0]) == ([f"fwd_0__{i}" for i in range(4)] + [f"fwd_4__{i}" for i in range(4)]
                           + [f"bwd_4__{i}" for i in range(4)] + [f"bwd_0__{i}" for i in range(4)])
    assert names(t[3]) == ([f"fwd_3__{i}" for i in range(4)]
                           + [f"FusedTask(fwd_7__{i}, bwd_7__{i})" for i in range(4)]
                           + [f"bwd_3__{i}" for i in range(4)])


def test_std1f1b_cfg1_closed_form():
    F = lambda m: S.Task.make(0, m, TaskType.FWD)
    B = lambda m: S.Task.make(0, m, TaskType.BWD)
    row0 = S.Std1F1B(2).tasks(8)[0]
    assert row0 == [F(0), F(1), None, B(0), F(2), B(1), F(3), B(2), F(4), B(3),
                    F(5), B(4), F(6), B(5), F(7), B(6), None, B(7)]


@pytest.mark.parametrize("cls,kw", [
    (S.Std1F1B, {}), (S.Eager1F1B, {}), (S.Interleaved1F1B, {"mpmd_dim": 1}),
    (S.ZeroBubble, {}),
])
def test_structure_and_errors(cls, kw):
    # mirrors the reference's tests/test_schedules.py:55-84
    res = cls(num_stages=2, **kw).tasks(4)
    assert isinstance(res, list)
    assert len(res) == (kw.get("mpmd_dim") or 2)
    assert all(isinstance(r, list) for r in res)
    with pytest.raises(ValueError, match="The argument `num_stages` must be `>= 0"):
        cls(num_stages=-1, **kw)
    if kw:
        with pytest.raises(ValueError, match="The argument `mpmd_dim` must be `>= 0"):
            cls(num_stages=2, mpmd_dim=-1)
        with pytest.raises(ValueError, match="can not be evenly divided by"):
            cls(num_stages=2, mpmd_dim=3)


def test_dualpipev_validation():
    # tests/test_schedules.py:87-113
    for ns in (4, 12):
        with pytest.raises(ValueError) as exc:
            S.DualPipeV(num_stages=ns, mpmd_dim=4)
        assert (f"DualPipeV only supports 2 * mpmd_dim stages, self.num_stages={ns}"
                f" requested with self.mpmd_dim=4") in str(exc.value)
    with pytest.raises(ValueError) as exc:
        S.DualPipeV(num_stages=6, mpmd_dim=3).tasks(5)
    assert "DualPipeV requires n_mubatches=5 >= self.num_stages=6" in str(exc.value)


def test_zero_bubble_edge_cases():
    with pytest.raises(AssertionError, match="Expect num of microbatches >= num of stages"):
        S.ZeroBubble(4).tasks(3)
    with pytest.raises(UnboundLocalError):
        S.ZeroBubble(1).tasks(2)


def test_interleaved_round_rule():
    # accepted although 6 % 4 != 0; rejected although the message names mpmd_dim
    S.Interleaved1F1B(num_stages=8, mpmd_dim=4).tasks(6)
    with pytest.raises(ValueError, match="n_microbatches must be divisible by mpmd_dim"):
        S.Interleaved1F1B(num_stages=8, mpmd_dim=4).tasks(9)


def test_task_identity_ignores_latency():
    a = S.Task.make(0, 3, TaskType.BWD_I)
    b = S.Task.make(0, 3, TaskType.BWD_I, latency=2)
    assert a == b and hash(a) == hash(b) and b.latency == 2
    assert S.FusedTask((a, b)).latency == 3
    assert S.mk_task_name(5, TaskType.BWD_W) == "bwdW_5"
    assert str(S.Task.make(1, 2, TaskType.BWD_I)) == "bwdA_1__2"


def test_first_stage_merge_rules():
    BI = lambda s, m: S.Task.make(s, m, TaskType.BWD_I)
    BW = lambda s, m: S.Task.make(s, m, TaskType.BWD_W)
    F = lambda s, m: S.Task.make(s, m, TaskType.FWD)
    out = S.check_and_strip_adjecent_bwd_a_bwd_w([F(0, 0), BI(0, 0), BW(0, 0)], 0)
    assert out == [F(0, 0), BI(0, 0)] and out[1].latency == 2
    with pytest.raises(NotImplementedError):
        S.check_and_strip_adjecent_bwd_a_bwd_w([BI(0, 0), F(0, 1), BW(0, 0)], 0)
    # a trailing first-stage BWD_I is passed through
    assert S.check_and_strip_adjecent_bwd_a_bwd_w([F(0, 0), BI(0, 0)], 0)[1].latency == 1
    fused = S.FusedTask((BI(0, 0), BW(0, 0)))
    out = S.check_and_strip_adjecent_bwd_a_bwd_w([fused, F(0, 1)], 0)
    assert isinstance(out[0], S.Task) and out[0].latency == 2
    # other stages stay split
    out = S.check_and_strip_adjecent_bwd_a_bwd_w([BI(1, 0), BW(1, 0)], 0)
    assert len(out) == 2


@pytest.mark.parametrize("case", [c for c in CASES if "raw" in c], ids=case_id)
def test_every_task_once_and_ascending(case):
    sched = getattr(S, case["schedule"])(**case["kwargs"])
    n = case["n_mubatches"]
    seen = {}
    for row in sched.tasks(n):
        for t in S.unpack_fused_tasks_fn(S.strip_nones(row)):
            key = (t.stage_id, t.fwd_or_bwd)
            assert t.mubatch_idx == seen.get(key, 0), "microbatches ascend per (stage, kind)"
            seen[key] = t.mubatch_idx + 1
    assert all(v == n for v in seen.values())
    assert {k[0] for k in seen} == set(range(case["kwargs"]["num_stages"]))
