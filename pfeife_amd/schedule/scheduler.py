"""Order of work of one optimisation step.

Restates, for the single-GPU executor, the schedule objects of the reference:
`StepWork` / `Step` (pfeife/schedule/scheduler.py:9-31), the looped one-forward-
one-backward order of `PipeSchedParams._build_sched` (:56-111) and the job
triples of `Scheduler._add_forward/_add_backward` + `SingleCommScheduler`
(:182-202, :249-274).  A schedule is drawn for `device_cnt` pipeline ranks
(stage i belongs to rank i % device_cnt); `serialize_ranks` then merges the
per-rank lists into the one order in which a single GPU executes them.
"""
from dataclasses import dataclass
from enum import Enum
from typing import List, Tuple


class StepWork(Enum):
    SEND_ACT = 1
    RECV_ACT = 2
    FORWARD = 3
    SEND_GRAD = 4
    RECV_GRAD = 5
    BACKWARD = 6
    OPTIMIZER_STEP = 7


@dataclass
class Step:
    work: StepWork
    node_id: int
    batch_id: int

    def __str__(self):
        return "%s / (node %d of batch %d)" % (self.work, self.node_id, self.batch_id)


class PipeSchedParams:
    """rank_works[r] = ordered [(stage, micro_batch, is_forward)] of pipeline rank r."""

    def __init__(self, device_cnt, batch_cnt, node_cnt, loop_batch, prefetch_fwd):
        self.device_cnt = int(device_cnt)
        self.batch_cnt = int(batch_cnt)
        self.node_cnt = int(node_cnt)
        self.loop_batch = int(loop_batch)
        self.prefetch_fwd = int(prefetch_fwd)
        assert self.batch_cnt >= self.loop_batch, "batch_cnt should be greater than loop_batch"
        self.rank_works: List[List[Tuple[int, int, bool]]] = self._build_sched()

    def _build_sched(self):
        D, B, S, L = self.device_cnt, self.batch_cnt, self.node_cnt, self.loop_batch
        fwd_q = [[] for _ in range(D)]
        bwd_q = [[] for _ in range(D)]
        for start in range(0, B, L):
            # size of this group of micro-batches, as the reference computes it
            group = (start - 1) % L + 1
            mbs = range(start, min(start + group, B))
            for stage in range(S):
                fwd_q[stage % D].extend((stage, mb) for mb in mbs)
            for stage in range(S - 1, -1, -1):
                bwd_q[stage % D].extend((stage, mb) for mb in mbs)

        works = []
        for rank in range(D):
            fwd, bwd = fwd_q[rank], bwd_q[rank]
            order = []
            if fwd:
                last_stage = max(s for s, _ in fwd)
                dist = S - last_stage  # stages from this rank's last stage to the pipeline end
                warm = (S - dist) // D * L + dist + min(dist - 1, self.prefetch_fwd) - 1
            else:
                warm = 0
            nb = 0
            for i, (stage, mb) in enumerate(fwd):
                order.append((stage, mb, True))
                if i >= warm:
                    order.append((bwd[nb][0], bwd[nb][1], False))
                    nb += 1
            order.extend((stage, mb, False) for stage, mb in bwd[nb:])
            works.append(order)
        return works

    def __str__(self):
        return "PipeSched(node_cnt=%d, loop_batch=%d, prefetch_fwd=%d)" % (
            self.node_cnt, self.loop_batch, self.prefetch_fwd)

    __repr__ = __str__


class PipeSchedSet:
    """The schedule variants the auto-partitioner values for one stage count
    (pfeife/schedule/scheduler.py:118-151): a looped pipeline (more stages than ranks) tries every
    `loop_batch` from `device_cnt` to `batch_cnt` that is `device_cnt` itself or divides
    `batch_cnt`, each with `prefetch_fwd` 0 .. device_cnt - 1; a plain pipeline takes
    `loop_batch = batch_cnt` with the same prefetch range."""

    def __init__(self, device_cnt, batch_cnt, node_cnt):
        self.device_cnt, self.batch_cnt, self.node_cnt = int(device_cnt), int(batch_cnt), int(node_cnt)
        self.scheds: List[PipeSchedParams] = [
            PipeSchedParams(self.device_cnt, self.batch_cnt, self.node_cnt, lb, pf)
            for lb, pf in self.variants(self.device_cnt, self.batch_cnt, self.node_cnt)]

    @staticmethod
    def variants(device_cnt, batch_cnt, node_cnt):
        """-> [(loop_batch, prefetch_fwd)] in the order the reference builds its set."""
        D, B, S = int(device_cnt), int(batch_cnt), int(node_cnt)
        if S > D:
            loops = [lb for lb in range(D, B + 1) if lb == D or B % lb == 0]
        else:
            loops = [B]
        return [(lb, pf) for lb in loops for pf in range(D)]


class Scheduler:
    """Expands rank_works into RECV/COMPUTE/SEND job triples per rank."""

    def __init__(self, sched_params: PipeSchedParams):
        self.sched_params = sched_params
        self.node_cnt = sched_params.node_cnt
        self.device_cnt = sched_params.device_cnt
        self.batch_cnt = sched_params.batch_cnt
        self.steps = self._build_steps()

    def _build_steps(self):
        steps = []
        for rank_job in self.sched_params.rank_works:
            rank_steps = []
            for node_idx, batch_id, is_fwd in rank_job:
                if is_fwd:
                    rank_steps += [Step(StepWork.RECV_ACT, node_idx, batch_id),
                                   Step(StepWork.FORWARD, node_idx, batch_id),
                                   Step(StepWork.SEND_ACT, node_idx, batch_id)]
                else:
                    rank_steps += [Step(StepWork.RECV_GRAD, node_idx, batch_id),
                                   Step(StepWork.BACKWARD, node_idx, batch_id),
                                   Step(StepWork.SEND_GRAD, node_idx, batch_id)]
            if rank_steps:
                rank_steps.append(Step(StepWork.OPTIMIZER_STEP, -1, -1))
            steps.append(rank_steps)
        return steps

    def get_train_steps(self, worker_id):
        return self.steps[worker_id] if worker_id < len(self.steps) else []


class SingleCommScheduler(Scheduler):
    def __init__(self, sched_params, dep_graph=None):
        self.dep_graph = dep_graph
        super().__init__(sched_params)


class BeamScheduler(Scheduler):
    pass


def serialize_ranks(rank_works, node_cnt):
    """Merge per-rank work lists into one serial order for a single GPU.

    A forward of stage s needs the forward of s-1 of the same micro-batch; a
    backward of stage s needs its own forward and the backward of s+1.  Ranks are
    visited round-robin and each contributes its next job as soon as that job's
    dependencies have run, so every rank's own order is preserved (in particular
    the per-stage micro-batch order that fixes the gradient summation order).
    """
    pos = [0] * len(rank_works)
    done = set()
    order = []
    total = sum(len(w) for w in rank_works)
    while len(order) < total:
        progressed = False
        for r, works in enumerate(rank_works):
            while pos[r] < len(works):
                stage, mb, is_fwd = works[pos[r]]
                if is_fwd:
                    ready = stage == 0 or (stage - 1, mb, True) in done
                else:
                    ready = (stage, mb, True) in done and (stage == node_cnt - 1 or (stage + 1, mb, False) in done)
                if not ready:
                    break
                done.add((stage, mb, is_fwd))
                order.append((stage, mb, is_fwd))
                pos[r] += 1
                progressed = True
                # one job per visit keeps the interleaving close to the pipelined timeline
                break
        if not progressed:
            raise RuntimeError("schedule deadlock: no rank can make progress at %s" % (pos,))
    return order
