"""TEST INFRASTRUCTURE -- CPU restatement of the reference's schedule construction.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module.

`rank_works(device_cnt, batch_cnt, node_cnt, loop_batch, prefetch_fwd)` follows
`PipeSchedParams._build_sched` (pfeife/schedule/scheduler.py:56-111): per rank a
forward queue and a backward queue are filled group by group (:68-87), then
interleaved: after `alter_idx` forwards every further forward is followed by one
backward, and the remaining backwards drain at the end (:89-109).

Pinned by tests/test_schedule.py against tests/golden/schedule_vectors.json
(rank_works lists written by importing the reference's scheduler.py, see
tests/golden/make_schedule_vectors.py), against three hand-derived orders, and
against the dependency invariants of a pipeline schedule.
"""


def rank_works(device_cnt, batch_cnt, node_cnt, loop_batch, prefetch_fwd):
    assert batch_cnt >= loop_batch
    fwd = {r: [] for r in range(device_cnt)}
    bwd = {r: [] for r in range(device_cnt)}
    loop_start = 0
    while loop_start < batch_cnt:
        width = (loop_start - 1) % loop_batch + 1  # scheduler.py:69
        hi = min(loop_start + width, batch_cnt)
        for node in range(node_cnt):
            for mb in range(loop_start, hi):
                fwd[node % device_cnt].append((node, mb))
        for node in reversed(range(node_cnt)):
            for mb in range(loop_start, hi):
                bwd[node % device_cnt].append((node, mb))
        loop_start += loop_batch
    result = []
    for r in range(device_cnt):
        out = []
        top = max(n for n, _ in fwd[r])  # raises on an empty rank like the reference does
        last_dist = node_cnt - top
        alter_idx = (node_cnt - last_dist) // device_cnt * loop_batch + last_dist + min(last_dist - 1, prefetch_fwd) - 1
        taken = 0
        for i, (n, mb) in enumerate(fwd[r]):
            out.append((n, mb, True))
            if i >= alter_idx:
                out.append((bwd[r][taken][0], bwd[r][taken][1], False))
                taken += 1
        out += [(n, mb, False) for n, mb in bwd[r][taken:]]
        result.append(out)
    return result
