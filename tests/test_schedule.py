"""Schedule construction: oracle vs the reference's golden vectors, hand-derived
orders and pipeline invariants; product (pfeife_amd.schedule) vs oracle; and the
single-GPU serialisation of the per-rank lists."""
import json
import os

import pytest

from oracle.schedule_oracle import rank_works as oracle_rank_works
from pfeife_amd.schedule.scheduler import (PipeSchedParams, SingleCommScheduler, Step, StepWork, serialize_ranks)

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "schedule_vectors.json")


def load_cases():
    with open(GOLDEN) as f:
        return json.load(f)


def fmt(works):
    return " ".join("%s%d%d" % ("F" if f else "B", n, b) for n, b, f in works)


def test_oracle_and_product_match_reference_golden_vectors():
    cases = load_cases()
    assert len(cases) > 300
    checked = 0
    for c in cases:
        args = c["args"]
        if "error" in c:
            with pytest.raises(Exception):
                oracle_rank_works(*args)
            with pytest.raises(Exception):
                PipeSchedParams(*args)
            continue
        want = [[(n, b, bool(f)) for n, b, f in w] for w in c["rank_works"]]
        assert oracle_rank_works(*args) == want, args
        assert PipeSchedParams(*args).rank_works == want, args
        checked += 1
    assert checked > 250


def test_hand_derived_orders():
    # device_cnt=1, node_cnt=2, batch_cnt=4, loop_batch=1
    assert fmt(oracle_rank_works(1, 4, 2, 1, 0)[0]) == (
        "F00 F10 B10 F01 B00 F11 B11 F02 B01 F12 B12 F03 B02 F13 B13 B03")
    # ViT-L shape: 2 ranks, 2 stages, 4 micro-batches, loop_batch 2
    w = oracle_rank_works(2, 4, 2, 2, 0)
    assert fmt(w[0]) == "F00 F01 B00 F02 B01 F03 B02 B03"
    assert fmt(w[1]) == "F10 B10 F11 B11 F12 B12 F13 B13"
    # Llama shape: 2 ranks, 4 stages looped, 8 micro-batches, loop_batch 2
    w = oracle_rank_works(2, 8, 4, 2, 0)
    assert fmt(w[0]).startswith("F00 F01 F20 F21 B20 F02 B21 F03 B00 F22 B01 F23 B22")
    assert fmt(w[1]).startswith("F10 F11 F30 B30 F31 B31 F12 B10 F13 B11 F32 B32")


@pytest.mark.parametrize("args", [(1, 4, 2, 1, 0), (2, 4, 2, 2, 0), (2, 8, 4, 2, 0), (2, 8, 4, 2, 1), (4, 8, 8, 4, 0),
                                  (3, 6, 3, 3, 1), (1, 1, 1, 1, 0), (2, 6, 4, 2, 0)])
def test_invariants_and_serialisation(args):
    device_cnt, batch_cnt, node_cnt, _, _ = args
    works = PipeSchedParams(*args).rank_works
    assert works == oracle_rank_works(*args)
    seen = set()
    for r, w in enumerate(works):
        for n, b, f in w:
            assert n % device_cnt == r
            assert (n, b, f) not in seen
            seen.add((n, b, f))
        # per stage, forwards and backwards each run in increasing micro-batch order
        for n in range(node_cnt):
            for f in (True, False):
                mbs = [b for nn, b, ff in w if nn == n and ff == f]
                assert mbs == sorted(mbs)
    assert len(seen) == 2 * node_cnt * batch_cnt
    order = serialize_ranks(works, node_cnt)
    assert sorted(order) == sorted(seen)
    pos = {job: i for i, job in enumerate(order)}
    for n in range(node_cnt):
        for b in range(batch_cnt):
            assert pos[(n, b, True)] < pos[(n, b, False)]
            if n > 0:
                assert pos[(n - 1, b, True)] < pos[(n, b, True)]
                assert pos[(n, b, False)] < pos[(n - 1, b, False)]
    # each rank's own order survives the merge
    for w in works:
        idx = [pos[j] for j in w]
        assert idx == sorted(idx)


def test_step_lists():
    sched = SingleCommScheduler(PipeSchedParams(2, 4, 2, 2, 0))
    r0 = sched.get_train_steps(0)
    assert [s.work for s in r0[:3]] == [StepWork.RECV_ACT, StepWork.FORWARD, StepWork.SEND_ACT]
    assert r0[-1] == Step(StepWork.OPTIMIZER_STEP, -1, -1)
    assert len(r0) == 3 * 8 + 1
    assert sched.get_train_steps(5) == []
    bwd = [s for s in r0 if s.work == StepWork.BACKWARD]
    assert [(s.node_id, s.batch_id) for s in bwd] == [(0, 0), (0, 1), (0, 2), (0, 3)]
