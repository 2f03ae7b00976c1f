"""Auto-partitioner: picks `split_points` when the user gives none.

Counterpart of the search branch of `PipeGraphGenerator.gen_graph`
(pfeife/schedule/planner.py:667-815) with `BeamSingleGenerator._optimize_split`
(:1624-1880) as the search and `PipeGraph.get_value` / `get_peak_memory`
(pfeife/graph/pipe_graph.py:177-314) as the objective:

  * the stage count is `loop_cnt * device_cnt` when `loop_cnt` is given, else the best of
    1x, 2x and 3x `device_cnt` (a count needs at least `count + 4` compute nodes; a looped
    count the user did not ask for is skipped when its stages would average 3 ms or less);
  * for every stage count the schedule variants of `PipeSchedSet` (`loop_batch` x
    `prefetch_fwd`, pfeife/schedule/scheduler.py:118-151) are searched, except that a
    `loop_batch` / `prefetch_fwd` the user fixed in the option is kept (planner.py:706-714).  Every
    variant is valued: the reference leaves a stage count at the first variant that improves the
    best time by less than 1 % (planner.py:778-787), a shortcut for its far costlier valuation
    that can miss the optimum by more than that;
  * a candidate split is valued by the expected time of one optimisation step: the jobs
    (stage, micro-batch, direction) run in each rank's schedule order, a job starts when its
    rank is free and the jobs it depends on have finished (plus the transfer time of the
    boundary when the two stages sit on different ranks), the step ends when every rank has
    run its optimizer;
  * a split whose peak memory on some rank exceeds the rank's budget is rejected.

The profile (pfeife_amd/graph/profile.py) gives per-node forward / backward times from HIP
events on the stage's real launch lists, so prefix sums make a stage's cost an O(1) lookup
and a candidate costs one pass over the schedule's jobs; the search is a beam over the split
points (exhaustive when there are few combinations).  Boundaries are only tried where few
bytes cross (between blocks: the residual stream), which is also where the stage lowering
keeps its fusions.
"""
import itertools
import math
from dataclasses import dataclass, field
from typing import List, Optional

from .scheduler import PipeSchedParams, PipeSchedSet

HBM_BYTES = 288 * 1024 ** 3       # MI355X
RESERVE_MEM_RATIO = 0.9           # part of a rank's memory the plan may use
ADAM_BYTES_PER_PARAM_BYTE = 7.0   # 28 bytes moved per fp32 parameter
OPTIM_GBS = 4800.0                # measured rate of the fused Adam step
FWD_AVG_MIN = 3.0                 # ms: looped stage counts nobody asked for need stages longer than this


@dataclass
class LinkModel:
    """Transfer time between two ranks.  On the one-GPU executor a boundary is a pointer and
    costs nothing; `gbs` prices it for a plan that is meant for one GPU per rank."""
    gbs: Optional[float] = None
    latency_ms: float = 0.0

    def send_ms(self, nbytes):
        if not self.gbs:
            return 0.0
        return self.latency_ms + nbytes / (self.gbs * 1e6)


@dataclass
class Plan:
    split_points: List[int]
    sched_params: PipeSchedParams
    expect_ms: float
    peak_mem: List[int]
    idle_mem: List[int]
    stage_fwd_ms: List[float] = field(default_factory=list)
    stage_bwd_ms: List[float] = field(default_factory=list)
    evaluated: int = 0

    def describe(self):
        from ..utils import fmem

        lines = ["split_points: %s, expect time: %.3f, schedule: %d ranks x %d stages, loop_batch %d, prefetch %d"
                 % (self.split_points, self.expect_ms, self.sched_params.device_cnt, self.sched_params.node_cnt,
                    self.sched_params.loop_batch, self.sched_params.prefetch_fwd)]
        for i, (idle, peak) in enumerate(zip(self.idle_mem, self.peak_mem)):
            lines.append("dev %d - idle mem: %s peak: %s" % (i, fmem(idle), fmem(peak)))
        return "\n".join(lines)


class CostModel:
    """Prefix sums over the node profile: cost of the stage [a, b) in O(1)."""

    def __init__(self, prof, link=None):
        self.prof = prof
        self.n = prof.n
        self.link = link or LinkModel()
        self.fwd = self._scan(prof.fwd_ms)
        self.bwd = self._scan(prof.bwd_ms)
        self.act = self._scan(prof.act_bytes)
        self.par = self._scan(prof.param_bytes)

    @staticmethod
    def _scan(xs):
        out = [0.0]
        for x in xs:
            out.append(out[-1] + x)
        return out

    def stages(self, points):
        """-> per-stage (fwd ms, bwd ms, optimizer ms, activation bytes, parameter bytes)."""
        bounds = [0] + list(points) + [self.n]
        rows = []
        for a, b in zip(bounds, bounds[1:]):
            par = self.par[b] - self.par[a]
            rows.append((self.fwd[b] - self.fwd[a], self.bwd[b] - self.bwd[a],
                         par * ADAM_BYTES_PER_PARAM_BYTE / (OPTIM_GBS * 1e6),
                         self.act[b] - self.act[a], par))
        return rows

    def value(self, points, sched):
        """Expected time (ms) of one step under `sched` (a PipeSchedParams)."""
        rows = self.stages(points)
        S = len(rows)
        D = sched.device_cnt
        rank_of = [s % D for s in range(S)]
        send = [0.0] * S
        for s in range(1, S):
            if rank_of[s] != rank_of[s - 1]:
                send[s] = self.link.send_ms(self.prof.cut_bytes[points[s - 1]])
        works = sched.rank_works
        pos = [0] * len(works)
        free = [0.0] * len(works)
        done = {}
        remaining = sum(len(w) for w in works)
        while remaining:
            progressed = False
            for r, w in enumerate(works):
                while pos[r] < len(w):
                    s, mb, is_fwd = w[pos[r]]
                    if is_fwd:
                        if s == 0:
                            ready = 0.0
                        else:
                            t = done.get((s - 1, mb, True))
                            if t is None:
                                break
                            ready = t + send[s]
                    else:
                        ready = done.get((s, mb, True))
                        if ready is None:
                            break
                        if s < S - 1:
                            t = done.get((s + 1, mb, False))
                            if t is None:
                                break
                            ready = max(ready, t + send[s + 1])
                    start = max(free[r], ready)
                    end = start + (rows[s][0] if is_fwd else rows[s][1])
                    done[(s, mb, is_fwd)] = end
                    free[r] = end
                    pos[r] += 1
                    remaining -= 1
                    progressed = True
            if not progressed:
                raise RuntimeError("planner: the schedule deadlocks at %s" % (pos,))
        total = 0.0
        for r in range(len(works)):
            opt = sum(rows[s][2] for s in range(S) if rank_of[s] == r)
            total = max(total, free[r] + opt)
        return total

    def memory(self, points, sched, temp_bytes=None):
        """-> (idle bytes, peak bytes) per rank, by the reference's accounting
        (pfeife/graph/pipe_graph.py:177-217): a rank starts at its idle memory (parameters, their
        gradients, two Adam moments and the 16-bit shadow); a forward job peaks at the running sum
        plus the stage's temporary memory and then keeps its activations; a backward job peaks at
        the running sum plus (temporary - activation) memory and then releases the activations.
        A stage's temporary memory is its activations plus the backward temporaries."""
        rows = self.stages(points)
        D = sched.device_cnt
        temp = self.prof.temp_bytes if temp_bytes is None else temp_bytes
        idle = [0] * D
        for s, row in enumerate(rows):
            idle[s % D] += int(row[4] * 4.5)
        peak = []
        for r, w in enumerate(sched.rank_works):
            cur = top = idle[r]
            for s, _, is_fwd in w:
                act = rows[s][3]
                if is_fwd:
                    top = max(top, cur + act + temp)
                    cur += act
                else:
                    top = max(top, cur + temp)
                    cur -= act
            peak.append(int(top))
        return idle, peak


def cut_candidates(prof, window=4):
    """Positions where a stage may start: the valleys of the crossing traffic, i.e. positions where
    no position within `window` nodes has fewer values (or as many values but fewer bytes) crossing.
    In a transformer these are the block boundaries, where only the residual stream (and values
    every block reads, such as rotary tables) crosses."""
    n = prof.n
    if n < 2:
        return []
    key = [(prof.cut_values[i], prof.cut_bytes[i]) for i in range(n + 1)]
    ok = prof.cut_ok if prof.cut_ok else [True] * (n + 1)
    out = []
    for i in range(1, n):
        lo, hi = max(1, i - window), min(n - 1, i + window)
        if ok[i] and all(key[i] <= key[j] for j in range(lo, hi + 1) if ok[j]):
            out.append(i)
    return out or [i for i in range(1, n) if ok[i]]


def _balanced_start(model, cand, n_cuts):
    total = model.fwd[-1] + model.bwd[-1]
    pts = []
    for k in range(1, n_cuts + 1):
        target = total * k / (n_cuts + 1)
        lo = pts[-1] if pts else 0
        best = None
        for c in cand:
            if c <= lo:
                continue
            d = abs(model.fwd[c] + model.bwd[c] - target)
            if best is None or d < best[0]:
                best = (d, c)
        if best is None:
            return None
        pts.append(best[1])
    return pts


def search_points(model, sched, cand, max_mem=None, beam=8, exhaustive_limit=20000, rounds=64):
    """Split points (one per stage boundary, increasing, from `cand`) with the least expected
    step time whose peak memory fits.  -> (value, points, number of candidates valued)."""
    n_cuts = sched.node_cnt - 1
    seen = {}

    def score(pts):
        key = tuple(pts)
        v = seen.get(key)
        if v is None:
            v = model.value(list(pts), sched)
            if max_mem is not None:
                _, peak = model.memory(list(pts), sched)
                if any(p > m for p, m in zip(peak, max_mem)):
                    v = math.inf
            seen[key] = v
        return v

    if n_cuts == 0:
        return score(()), [], 1
    if len(cand) < n_cuts:
        return math.inf, None, 0
    if math.comb(len(cand), n_cuts) <= exhaustive_limit:
        best = min(((score(p), p) for p in itertools.combinations(cand, n_cuts)), key=lambda x: (x[0], x[1]))
        return best[0], list(best[1]), len(seen)
    start = _balanced_start(model, cand, n_cuts)
    if start is None:
        return math.inf, None, 0
    where = {c: i for i, c in enumerate(cand)}
    front = [tuple(start)]
    best = (score(front[0]), front[0])
    stale = 0
    for _ in range(rounds):
        nxt = set()
        for pts in front:
            for k in range(n_cuts):
                i = where[pts[k]]
                step = 1
                while step < len(cand):
                    for j in (i - step, i + step):
                        if 0 <= j < len(cand):
                            lo = pts[k - 1] if k > 0 else 0
                            hi = pts[k + 1] if k + 1 < n_cuts else model.n
                            if lo < cand[j] < hi:
                                nxt.add(pts[:k] + (cand[j],) + pts[k + 1:])
                    step *= 2
        fresh = [p for p in nxt if p not in seen]
        if not fresh:
            break
        ranked = sorted(((score(p), p) for p in nxt), key=lambda x: (x[0], x[1]))
        front = [p for _, p in ranked[:beam]]
        if ranked[0][0] < best[0] - 1e-12:
            best = ranked[0]
            stale = 0
        else:
            stale += 1
            if stale >= 2:
                break
    return best[0], list(best[1]), len(seen)


def schedule_variants(option, device_cnt, batch_cnt, node_cnt):
    """(loop_batch, prefetch_fwd) pairs to value for `node_cnt` stages: the reference's set, narrowed
    to what the user fixed; when the set is empty (fewer micro-batches than ranks) the manual-split
    defaults are used (`loop_batch = device_cnt` clamped to `batch_cnt`, no prefetch)."""
    pairs = PipeSchedSet.variants(device_cnt, batch_cnt, node_cnt)
    if option.loop_batch is not None:
        pairs = [(lb, pf) for lb, pf in pairs if lb == option.loop_batch]
    if option.prefetch_fwd is not None:
        pairs = [(lb, pf) for lb, pf in pairs if pf == option.prefetch_fwd]
    if not pairs:
        lb = option.loop_batch if option.loop_batch is not None else device_cnt
        pairs = [(max(1, min(lb, batch_cnt)), option.prefetch_fwd if option.prefetch_fwd is not None else 0)]
    return pairs


def plan_split(prof, option, device_cnt, max_mem=None, link=None, beam=8):
    """-> Plan with the best (split points, schedule variant) over the stage counts tried."""
    model = CostModel(prof, link)
    batch_cnt = option.batch_cnt
    if max_mem is None:
        max_mem = [HBM_BYTES * RESERVE_MEM_RATIO] * device_cnt
    cand = cut_candidates(prof)
    counts = [option.loop_cnt * device_cnt] if option.loop_cnt else [i * device_cnt for i in range(1, 4)]
    best = None
    evaluated = 0
    total_ms = model.fwd[-1] + model.bwd[-1]
    for loop_idx, cnt in enumerate(counts):
        if cnt + 4 > prof.n or cnt - 1 > len(cand):
            break
        if loop_idx != 0 and not option.loop_cnt and total_ms / cnt <= FWD_AVG_MIN:
            continue   # stages too short to be worth another loop (planner.py:724-737)
        for loop_batch, prefetch in schedule_variants(option, device_cnt, batch_cnt, cnt):
            sched = PipeSchedParams(device_cnt, batch_cnt, cnt, loop_batch, prefetch)
            try:
                v, pts, n = search_points(model, sched, cand, max_mem, beam=beam)
            except RuntimeError:   # a variant whose rank lists cannot be merged into one order
                continue
            evaluated += n
            if pts is None or not math.isfinite(v):
                continue
            if best is None or v < best[0] - 1e-9:
                best = (v, pts, sched)
    if best is None:
        # too few compute nodes (or cut positions) for device_cnt stages: fewer stages, down to one,
        # with every legal position as a candidate
        every = [i for i in range(1, prof.n) if (prof.cut_ok[i] if prof.cut_ok else True)]
        for cnt in range(min(device_cnt, len(every) + 1, prof.n), 0, -1):
            ranks = min(device_cnt, cnt)
            lb, pf = schedule_variants(option, ranks, batch_cnt, cnt)[0]
            sched = PipeSchedParams(ranks, batch_cnt, cnt, max(1, min(lb, batch_cnt)), pf)
            v, pts, n = search_points(model, sched, every, max_mem[:ranks], beam=beam)
            evaluated += n
            if pts is not None and math.isfinite(v):
                best = (v, pts, sched)
                break
    if best is None:
        raise RuntimeError("auto-partitioner: no split of the graph's %d compute nodes into %s stages fits"
                           % (prof.n, counts))
    v, pts, sched = best
    idle, peak = model.memory(pts, sched)
    rows = model.stages(pts)
    return Plan(pts, sched, v, peak, idle, [r[0] for r in rows], [r[1] for r in rows], evaluated)
