"""CPU restatement of the reference's pipeline valuation, TEST INFRASTRUCTURE ONLY.

Nothing under pfeife_amd/ may import this file; tests use it as the checker for
pfeife_amd/schedule/planner.py.

Restates
  * `PipeGraph.get_value`       (pfeife/graph/pipe_graph.py:219-314): the expected time of one
    optimisation step is the longest path through a DAG whose vertices are the jobs
    (stage, micro-batch, direction), with an edge job -> dependent job weighted by the job's own
    duration (+ the transfer time when the dependency crosses ranks) and an edge from each
    rank's job to the rank's next job weighted by the job's duration; every rank's last job
    reaches the sink after its duration plus the rank's optimizer time;
  * `PipeGraph.get_peak_memory` (pfeife/graph/pipe_graph.py:177-217): per rank, a running
    sum over the rank's job list that starts at the rank's weights, adds a stage's activation
    memory at its forward, releases it at its backward, and peaks by the stage's temporary memory.

  * `PipeSchedSet._build_set`   (pfeife/schedule/scheduler.py:130-151): the (loop_batch,
    prefetch_fwd) pairs valued per stage count, and the stage counts of
    `PipeGraphGenerator.gen_graph` (pfeife/schedule/planner.py:667-670): `loop_cnt * device_cnt`,
    else 1x, 2x, 3x `device_cnt`; pinned by hand-enumerated sets in tests/test_planner.py.

What pins it (tests/test_planner.py): closed forms of the one-forward-one-backward pipeline
with equal stages ((B + D - 1)(f + b) + optimizer), the single-stage sum, a hand-worked
two-stage case with unequal stages and a transfer time, and a hand-worked memory trace.
"""
import itertools


def pipe_value(fwd, bwd, optim, ranks, rank_works, batch_cnt, edges, return_dist=False):
    """fwd/bwd/optim: per-stage times; ranks[s]: rank of stage s; edges: [(src stage, dst stage,
    transfer time)]; rank_works[r]: ordered [(stage, micro-batch, is_forward)]."""
    n_rank = len(rank_works)
    graph = {}
    sink = (-1, -1, False)
    graph[sink] = []
    optim_times = [0.0] * n_rank
    out_edges = {s: [] for s in range(len(fwd))}
    in_edges = {s: [] for s in range(len(fwd))}
    for a, b, t in edges:
        out_edges[a].append((b, t))
        in_edges[b].append((a, t))
    for s in range(len(fwd)):
        optim_times[ranks[s]] += optim[s]
        for mb in range(batch_cnt):
            graph[(s, mb, True)] = [((d, mb, True), fwd[s] + t) for d, t in out_edges[s]]
            graph[(s, mb, False)] = [((a, mb, False), bwd[s] + t) for a, t in in_edges[s]]
    for r, works in enumerate(rank_works):
        if not works:
            continue
        for prev, nxt in zip(works, works[1:]):
            graph[prev].append((nxt, fwd[prev[0]] if prev[2] else bwd[prev[0]]))
        last = works[-1]
        graph[last].append((sink, bwd[last[0]] + optim_times[r]))

    order, seen = [], set()

    def visit(v):
        # iterative depth-first post-order
        stack = [(v, iter(graph.get(v, ())))]
        seen.add(v)
        while stack:
            node, it = stack[-1]
            for nb, _ in it:
                if nb not in seen:
                    seen.add(nb)
                    stack.append((nb, iter(graph.get(nb, ()))))
                    break
            else:
                order.append(node)
                stack.pop()

    for v in list(graph):
        if v not in seen:
            visit(v)
    order.reverse()
    dist = {v: float("-inf") for v in graph}
    dist[(0, 0, True)] = 0.0
    for v in order:
        for nb, w in graph[v]:
            if dist[v] + w > dist[nb]:
                dist[nb] = dist[v] + w
    return (dist[sink], dist) if return_dist else dist[sink]


def peak_memory(device_mem, act_mem, temp_mem, rank_works):
    out = []
    for weight, works in zip(device_mem, rank_works):
        cur = peak_max = weight
        for stage, _, is_fwd in works:
            if is_fwd:
                peak = cur + temp_mem[stage]
                cur += act_mem[stage]
            else:
                peak = cur + (temp_mem[stage] - act_mem[stage])
                cur -= act_mem[stage]
            peak_max = max(peak_max, peak)
        out.append(peak_max)
    return out


def chain_edges(n_stage, ranks, send_time):
    """Edges of a chain of stages; send_time[s]: transfer time of the boundary in front of stage s
    (counted only when the two stages sit on different ranks)."""
    return [(s - 1, s, send_time[s] if ranks[s - 1] != ranks[s] else 0.0) for s in range(1, n_stage)]


def brute_force_points(candidates, n_cuts, value_fn):
    """The best of ALL increasing choices of n_cuts split points among `candidates`."""
    best = None
    for pts in itertools.combinations(candidates, n_cuts):
        v = value_fn(list(pts))
        if best is None or v < best[0]:
            best = (v, list(pts))
    return best


def sched_set(device_cnt, batch_cnt, node_cnt):
    """[(loop_batch, prefetch_fwd)] of pfeife/schedule/scheduler.py:130-151, in its order."""
    out = []
    if node_cnt > device_cnt:
        for loop_batch in range(device_cnt, batch_cnt + 1):
            if loop_batch > device_cnt and batch_cnt % loop_batch != 0:
                continue
            for prefetch_fwd in range(0, device_cnt):
                out.append((loop_batch, prefetch_fwd))
    else:
        for prefetch_fwd in range(0, device_cnt):
            out.append((batch_cnt, prefetch_fwd))
    return out


def brute_force_plan(candidates, stage_counts, variants_of, value_fn):
    """The best of ALL (stage count, schedule variant, increasing split points): variants_of(cnt) ->
    [(loop_batch, prefetch_fwd)], value_fn(points, cnt, loop_batch, prefetch_fwd) -> time or None
    (None: the variant cannot be run)."""
    best = None
    for cnt in stage_counts:
        for lb, pf in variants_of(cnt):
            for pts in itertools.combinations(candidates, cnt - 1):
                v = value_fn(list(pts), cnt, lb, pf)
                if v is not None and (best is None or v < best[0]):
                    best = (v, list(pts), cnt, lb, pf)
    return best
