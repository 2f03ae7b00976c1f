"""Single-GPU stage worker: owns the stage programs and runs the job loop of a step.

Counterpart of `ProcessWorker` in pfeife/mp/worker.py for one rank that holds
every stage:
  * `set_partition_graph`  (worker.py:682-758): here it lowers each (stage,
    micro-batch) to prepared launch lists on preallocated buffers instead of
    allocating per-edge copy buffers;
  * `distribute_input`     (worker.py:818-840): micro-batch slab -> stage input
    buffer through the split/gather kernel (or one H2D copy for host tensors);
  * `run_with_module`      (worker.py:912-940) + `_handle_job_with_comm`
    (:978-1006): the schedule's jobs in one serial order;
  * `send_same_node`       (worker.py:1096-1151): nothing to do, a stage reads its
    producer's output buffer and writes the gradient buffer its producer reads;
  * `_init_optimizer` / `optimizer_step` (worker.py:583-597, 1432-1436).
"""
import os

import torch

from ..executor.lowering import BufferPool, Lowerer, ParamStore, Unsupported
from ..executor.values import Val
from ..option import get_optimizer_cls
from ..schedule.scheduler import PipeSchedParams, SingleCommScheduler, StepWork, serialize_ranks
from ..utils import fmem, get_logger


class MicroBatchPrograms:
    """Everything that was built for one micro-batch slot."""

    def __init__(self):
        self.stage_programs = {}   # stage -> StageProgram
        self.input_buffers = {}    # graph placeholder index -> static device buffer
        self.input_sig = None      # shapes/dtypes the programs were built for
        self.outputs = []          # per graph output: Val | python constant
        self.loss_grads = {}       # graph output index -> static gradient buffer
        self.graph = None          # the partition graph the programs were lowered from
        self.grad_seen = set()


class StageWorker:
    def __init__(self, runner, option, device, kernels=None):
        self.runner = runner
        self.option = option
        self.device = torch.device(device)
        if kernels is None:
            from ..hip import HipKernels  # raises when the library or the GPU is missing

            kernels = HipKernels(self.device.index)
        self.kernels = kernels
        self.log = get_logger()
        self.params = ParamStore(kernels, self.device)
        self.pool = BufferPool(self.device)
        self.lowerer = self._new_lowerer()
        self.dw_jobs = {}          # stage -> [launch list, captured graph or None]: the once-per-step weight-gradient job
        self.part_graph = None
        self.static_inputs = {}
        self.mbs = {}
        self.order = []
        self.optimizer = None
        self.mem_usage_info = {}
        # every launch of a step goes to one created stream (default priority): a created
        # stream can be captured into hipGraphs, the legacy default stream cannot
        self.stream_obj = torch.cuda.Stream(self.device) if self.device.type == "cuda" else None
        self.use_graphs = (bool(getattr(kernels, "supports_graphs", False)) and self.stream_obj is not None
                           and os.environ.get("PFEIFE_NO_GRAPH", "0") != "1")
        self.graphs_ready = False
        self.steps_done = 0
        self.begin_graph = None
        self.plan = None           # the auto-partitioner's choice (split points + schedule variant), if it ran
        self.profile = None
        # One stream per pipeline rank ("lane"): the jobs of different ranks are independent by
        # construction of the schedule (that is what lets the reference run them on different
        # GPUs), so on one GPU they run side by side and fill the CUs and launch gaps that a
        # single job's kernels leave idle.  rank -> torch.cuda.Stream; None: everything on stream_obj.
        self.lanes = None
        self.lane_mode = "0"
        self._job_events = {}
        self._loss_events = {}
        # dynamic loss scaling: {scale, growth tracker, found_inf, completed steps, 4 scratch} on the device
        self.dyn_scale = option.loss_scale == "dynamic"
        self.scaler_state = None
        if self.dyn_scale:
            if not hasattr(kernels, "scaler_unscale"):
                raise RuntimeError("dynamic loss scaling needs the HIP kernel table")
            self.scaler_state = torch.tensor([option.init_scale] + [0.0] * 7, dtype=torch.float32,
                                             device=self.device)
            self._one = torch.ones((), dtype=torch.float32, device=self.device)

    def _new_lowerer(self):
        # Weight gradients of the linear layers once per step instead of once per micro-batch
        # (PFEIFE_DW_STACK=0: inside every backward job, as torch.autograd issues them); decided per
        # micro-batch slot when it is lowered: only steps whose micro-batches all have the same
        # shapes stack their buffers (`uniform_mbs`, set by the runner before the step's first job)
        self.stack_dw = os.environ.get("PFEIFE_DW_STACK", "1") != "0"
        self.uniform_mbs = getattr(self, "uniform_mbs", True)
        return Lowerer(self.kernels, self.device, self.option.mixed_precision, self.params, self.pool)

    # -- graph ---------------------------------------------------------------------
    def set_partition_graph(self, part_graph, example_inputs):
        """Register a stage partition.  The first one fixes the schedule; later ones are
        the same pipeline captured again for another micro-batch shape (TorchDynamo
        recompiles with the new sizes baked in) and must have the same stage count."""
        pg = part_graph
        static = {}
        for i, (is_static, ex) in enumerate(zip(pg.static_placeholder, example_inputs)):
            if not is_static:
                continue
            if ex.device != self.device:
                ex.data = ex.data.to(self.device)  # stage parameters live on the worker's device
            param = ex if isinstance(ex, torch.nn.Parameter) else None
            static[i] = Val(ex.detach(), req_grad=bool(ex.requires_grad), param=param,
                            name=pg.placeholder_names[i])
        pg.static_vals = static
        if self.part_graph is not None:
            if len(pg.nodes) != len(self.part_graph.nodes):
                raise RuntimeError("recaptured graph splits into %d stages, the pipeline has %d"
                                   % (len(pg.nodes), len(self.part_graph.nodes)))
            for st in pg.nodes.values():
                st.rank = self.part_graph.nodes[st.idx].rank
            return
        self.part_graph = pg
        self.static_inputs = static
        node_cnt = len(pg.nodes)
        opt = self.option
        device_cnt = max(1, min(opt.device_cnt, node_cnt))
        loop_batch = opt.loop_batch if opt.loop_batch is not None else device_cnt
        loop_batch = max(1, min(loop_batch, opt.batch_cnt))
        prefetch = opt.prefetch_fwd if opt.prefetch_fwd is not None else 0
        plan = getattr(self, "plan", None)
        if plan is not None and plan.sched_params.node_cnt == node_cnt:
            # the auto-partitioner valued its split under one schedule variant: run that one
            loop_batch, prefetch = plan.sched_params.loop_batch, plan.sched_params.prefetch_fwd
        for st in pg.nodes.values():
            st.rank = st.idx % device_cnt
        self.sched_params = PipeSchedParams(device_cnt, opt.batch_cnt, node_cnt, loop_batch, prefetch)
        self.scheduler = SingleCommScheduler(self.sched_params)
        self.order = serialize_ranks(self.sched_params.rank_works, node_cnt)
        self._setup_lanes(pg, device_cnt)
        last = {}
        for i, (stage, mb, is_fwd) in enumerate(self.order):
            if is_fwd:
                last[mb] = i
        self.last_forward = {i: mb for mb, i in last.items()}
        # the job after which a stage's once-per-step weight-gradient job runs: its last backward
        self.last_backward = {}
        for stage, mb, is_fwd in self.order:
            if not is_fwd:
                self.last_backward[stage] = mb

    def _lane_key(self, stage, is_fwd):
        rank = self.part_graph.nodes[stage].rank
        return (rank, is_fwd) if self.lane_mode == "rankdir" else (rank, False)

    def _setup_lanes(self, pg, device_cnt):
        """Decide which jobs get streams of their own.  PFEIFE_LANES = "rank": one stream per
        pipeline rank; "rankdir" (default): per rank one for its forward and one for its backward
        jobs (forward jobs read parameters only, so they may run ahead of the rank's backward jobs;
        backward jobs of a rank stay in schedule order on one stream, which fixes the order in
        which micro-batches are summed into a parameter's gradient); "0": a single stream.
        A single stream is also used when a parameter is read by stages of two ranks (its
        gradient accumulator would be updated from two streams at once)."""
        self.lanes = None
        self._job_events = {}
        self._loss_events = {}
        mode = os.environ.get("PFEIFE_LANES", "rankdir")
        if os.environ.get("PFEIFE_NO_LANES", "0") == "1":
            mode = "0"
        if mode not in ("0", "rank", "rankdir"):
            raise RuntimeError("PFEIFE_LANES must be 0, rank or rankdir, not %r" % mode)
        self.lane_mode = mode
        if self.stream_obj is None or mode == "0" or (device_cnt < 2 and mode == "rank"):
            return
        owner = {}
        for st in pg.nodes.values():
            for gi in st.input_placeholder:
                v = pg.static_vals.get(gi) if gi >= 0 else None
                if v is None or not v.req_grad:
                    continue
                key = v.buf.untyped_storage().data_ptr()
                if owner.setdefault(key, st.rank) != st.rank:
                    self.log.info("parameter %s is shared by two pipeline ranks: single-stream execution", v.name)
                    return
        # user code (loss, hooks) and the optimizer run on stream_obj, which is also the lane of
        # the last stage's backward jobs: they read the loss gradients user code writes
        main_key = self._lane_key(max(pg.nodes), False)
        keys = sorted({self._lane_key(sid, d) for sid in pg.nodes for d in (True, False)})
        self.lanes = {k: (self.stream_obj if k == main_key else torch.cuda.Stream(self.device)) for k in keys}
        # which stages hand a value to user code / receive a loss gradient from it
        self._output_stages = sorted({ref[0] for ref in pg.outputs if isinstance(ref[0], int)})

    def plan_split_points(self, gm, live_args):
        """`split_points=None`: profile the captured graph on this device and let the planner pick
        the stage boundaries (pfeife/schedule/planner.py:667-815 in the reference)."""
        from ..graph.profile import profile_graph
        from ..schedule.planner import plan_split

        opt = self.option
        prof = profile_graph(self.kernels, self.device, opt.mixed_precision, gm, live_args, stream=self.stream())
        n_nodes = prof.n
        device_cnt = max(1, min(opt.device_cnt, n_nodes))
        plan = plan_split(prof, opt, device_cnt)
        self.plan, self.profile = plan, prof
        self.log.info("auto-partitioner: %s", plan.describe().replace("\n", "; "))
        return plan

    def stage_parameters(self):
        seen, out = set(), []
        for v in self.static_inputs.values():
            if v.param is not None and id(v.param) not in seen:
                seen.add(id(v.param))
                out.append(v.param)
        return out

    @staticmethod
    def _signature(values):
        sig = []
        for v in values:
            if torch.is_tensor(v):
                sig.append((tuple(v.shape), v.dtype))
            else:
                sig.append(("const", repr(v)))
        return tuple(sig)

    def build_micro_batch(self, mb, dynamic_inputs, part_graph=None):
        """Lower every stage for micro-batch slot `mb`; `dynamic_inputs` maps graph
        placeholder index -> the value user code passed (tensor chunk or constant)."""
        pg = part_graph if part_graph is not None else self.part_graph
        slot = MicroBatchPrograms()
        slot.input_sig = self._signature([dynamic_inputs[i] for i in sorted(dynamic_inputs)])
        graph_vals = {}
        L = self.lowerer
        L.defer_dw = self.stack_dw and self.uniform_mbs
        L.stack_mbs = self.option.batch_cnt
        L.stack_tag = slot.input_sig
        for i, v in dynamic_inputs.items():
            if torch.is_tensor(v):
                if L.defer_dw:   # (a layer that reads a graph input directly: its rows of all micro-batches in one matrix)
                    buf = self.pool.stacked((L.stack_tag, "in", i), v.shape, v.dtype, mb, L.stack_mbs)
                else:
                    buf = torch.empty(v.shape, dtype=v.dtype, device=self.device)
                slot.input_buffers[i] = buf
                graph_vals[i] = Val(buf, req_grad=False, name=pg.placeholder_names[i])
            else:
                graph_vals[i] = v
        for i, v in pg.static_vals.items():
            graph_vals[i] = v
        if self.dyn_scale:     # gradients stored whole by a once-per-step product leave it unscaled and checked
            L.dw_unscale = (self.scaler_state[0:1], self.scaler_state[2:3], 1.0)
        else:
            L.dw_unscale = (None, None, 1.0 / float(self.option.loss_scale))
        stage_out = {}
        for sid in sorted(pg.nodes):
            st = pg.nodes[sid]
            ins = []
            for k, name in enumerate(st.inputs):
                gi = st.input_placeholder[k]
                if gi >= 0:
                    ins.append(graph_vals[gi])
                else:
                    src_stage, oi = st.input_source[k]
                    pv = stage_out[src_stage][oi]
                    if isinstance(pv, Val):
                        bv = Val(pv.buf, req_grad=pv.req_grad, name=name)  # same storage: the handoff is a pointer
                        bv.boundary = True
                        ins.append(bv)
                    elif isinstance(pv, (list, tuple)) and any(isinstance(e, Val) for e in pv):
                        # its gradient would have to travel back as a tuple as well; the stage
                        # programs hand over single tensors only
                        raise Unsupported("the split point in front of stage %d cuts between '%s' (a tuple of "
                                          "tensors) and its users; move it before the node that makes the tuple "
                                          "or after the nodes that take it apart" % (sid, name))
                    else:
                        ins.append(pv)
            self.pool.lane = self._lane_key(sid, True) if self.lanes is not None else 0
            prog = L.lower_forward(st, mb, ins)
            slot.stage_programs[sid] = prog
            stage_out[sid] = prog.outputs
        # graph outputs and the buffers their loss gradients arrive in
        for oi, ref in enumerate(pg.outputs):
            if ref[0] == "const":
                slot.outputs.append(ref[1])
            elif ref[0] == "input":
                slot.outputs.append(graph_vals[ref[1]])
            else:
                v = stage_out[ref[0]][ref[1]]
                slot.outputs.append(v)
                if isinstance(v, Val) and v.req_grad:
                    if L.defer_dw and v.buf.is_contiguous():
                        # (the last layer's weight gradient reads these across micro-batches as one matrix)
                        slot.loss_grads[oi] = self.pool.stacked((L.stack_tag, "loss", oi), v.buf.shape, v.buf.dtype, mb,
                                                                L.stack_mbs).zero_()
                    else:
                        slot.loss_grads[oi] = torch.zeros_like(v.buf)
        # backward, last stage first: a stage's output gradients are its consumers' input gradients
        for sid in sorted(pg.nodes, reverse=True):
            st = pg.nodes[sid]
            prog = slot.stage_programs[sid]
            out_grads = [[] for _ in st.outputs]
            for tid in sorted(pg.nodes):
                if tid <= sid:
                    continue
                tst = pg.nodes[tid]
                tprog = slot.stage_programs[tid]
                for k, src in enumerate(tst.input_source):
                    if src is not None and src[0] == sid and tprog.input_grads[k] is not None:
                        out_grads[src[1]].append(tprog.input_grads[k])
            for oi, ref in enumerate(pg.outputs):
                if ref[0] == sid and oi in slot.loss_grads:
                    out_grads[ref[1]].append(slot.loss_grads[oi])
            self.pool.lane = self._lane_key(sid, False) if self.lanes is not None else 0
            L.lower_backward(prog, out_grads)
        self.pool.lane = 0
        # gradients that lost their single storing writer in this lowering: zero them now (their backward
        # jobs, which accumulate, come later in the step)
        self._run_pending_fills(self.stream())
        if self.stream_obj is not None:
            # tables the lowering copied to the device went through torch's current stream; the jobs
            # that read them run on the lanes
            self.stream_obj.synchronize()
            torch.cuda.current_stream(self.device).synchronize()
        self._drop_graphs(self.mbs.get(mb))   # a slot rebuilt for another micro-batch shape
        self._drop_dw_jobs()
        self.mbs[mb] = slot
        self.pool.prune_stacked({s.input_sig for s in self.mbs.values()})
        self.graphs_ready = False   # new programs (and possibly new parameters): capture again
        self._drop_begin_graph()
        return slot

    def _drop_graphs(self, slot):
        """Frees the captured hipGraphs of a micro-batch slot that is being replaced or released."""
        if slot is None or not hasattr(self.kernels, "destroy_graph"):
            return
        for prog in slot.stage_programs.values():
            for attr in ("fwd_graph", "bwd_graph"):
                g = getattr(prog, attr, None)
                if g is not None:
                    self.kernels.destroy_graph(g)
                    setattr(prog, attr, None)

    def _drop_dw_jobs(self):
        for job in self.dw_jobs.values():
            if job[1] is not None and hasattr(self.kernels, "destroy_graph"):
                self.kernels.destroy_graph(job[1])
        self.dw_jobs = {}

    def _drop_begin_graph(self):
        if self.begin_graph is not None and hasattr(self.kernels, "destroy_graph"):
            self.kernels.destroy_graph(self.begin_graph)
        self.begin_graph = None

    def release(self):
        """Frees every captured graph and drops the stage programs and their buffers (the worker
        cannot run another step afterwards)."""
        if self.stream_obj is not None:
            self.stream_obj.synchronize()
        for slot in self.mbs.values():
            self._drop_graphs(slot)
        self._drop_begin_graph()
        self._drop_dw_jobs()
        self.mbs = {}
        self.graphs_ready = False
        self.static_inputs = {}
        self.part_graph = None
        self.lanes = None
        self._job_events = {}
        self._loss_events = {}
        self.optimizer = None
        self.plan = self.profile = None
        self._steps_owner = None
        self._host_steps_stale = False
        self.params = ParamStore(self.kernels, self.device)
        self.pool = BufferPool(self.device)
        self.lowerer = self._new_lowerer()
        self.__dict__.pop("_adam_tables", None)

    # -- per step --------------------------------------------------------------------
    def stream(self):
        return self.stream_obj.cuda_stream if self.stream_obj is not None else None

    def capture_graphs(self):
        """Record every job's launch list (and the per-step zero/refresh list) into hipGraphs.
        Called after one complete eager step, when every program exists and every kernel has
        run once (so one-time function attributes are set)."""
        s = self.stream()
        for slot in self.mbs.values():
            for prog in slot.stage_programs.values():
                if prog.fwd_graph is None and prog.fwd:
                    prog.fwd_graph = self.kernels.capture(prog.fwd, s)
                if prog.bwd_graph is None and prog.bwd:
                    prog.bwd_graph = self.kernels.capture(prog.bwd, s)
        for job in self.dw_jobs.values():
            if job[1] is None and job[0]:
                job[1] = self.kernels.capture(job[0], s)
        pre = self.params.zero_launches() + self.params.refresh_launches()
        self._drop_begin_graph()
        self.begin_graph = self.kernels.capture(pre, s) if pre else None
        self._begin_len = (len(self.params.zero), len(self.params.refresh))
        self.graphs_ready = True

    def distribute_input(self, mb, placeholder_idx, value):
        """Copy one micro-batch slab into the stage input buffer it was built for."""
        slot = self.mbs[mb]
        buf = slot.input_buffers.get(placeholder_idx)
        if buf is None:
            return
        if value.device == buf.device and value.is_contiguous() and buf.is_contiguous() and value.numel() > 0:
            rows = value.shape[0] if value.dim() > 0 else 1
            row_bytes = value.numel() * value.element_size() // max(rows, 1)
            self.kernels.split_gather(value, buf, row_bytes, 0, rows)(self.stream())
        elif value.numel() > 0:
            buf.copy_(value, non_blocking=True)  # host -> device (or a layout change): PyTorch plumbing

    def begin_step(self):
        s = self.stream()
        self.end_jobs()   # a step that failed half-way may have left lanes running
        self.params.rebind_grads()
        if self.use_graphs and not self.graphs_ready and self.steps_done >= 1 and len(self.mbs) == self.option.batch_cnt:
            self.capture_graphs()
        if self.graphs_ready and self.begin_graph is not None:
            self.begin_graph(s)
        else:
            for launch in self.params.zero_launches():      # optimizer.zero_grad(set_to_none=False)
                launch(s)
            for launch in self.params.refresh_launches():   # one master -> 16-bit cast per step
                launch(s)
        for slot in self.mbs.values():
            slot.grad_seen.clear()
        if self.lanes is not None:   # zeroed gradients, fresh shadows and the step's inputs are in place
            for lane in self.lanes.values():
                if lane is not self.stream_obj:
                    lane.wait_stream(self.stream_obj)

    # -- lanes -------------------------------------------------------------------------
    def _event(self, table, key):
        ev = table.get(key)
        if ev is None:
            ev = table[key] = torch.cuda.Event()
        return ev

    def outputs_ready(self, mb):
        """User code of micro-batch `mb` is about to read the graph outputs on the main stream."""
        if self.lanes is None:
            return
        for sid in self._output_stages:
            if self.lanes[self._lane_key(sid, True)] is not self.stream_obj:
                ev = self._job_events.get((sid, mb, True))
                if ev is not None:
                    self.stream_obj.wait_event(ev)

    def loss_grads_ready(self, mb):
        """The loss gradients of micro-batch `mb` have been written (on the main stream)."""
        if self.lanes is None:
            return
        if any(self.lanes[self._lane_key(sid, False)] is not self.stream_obj for sid in self._output_stages):
            self._event(self._loss_events, mb).record(self.stream_obj)

    def end_jobs(self):
        """Every lane's work precedes what follows on the main stream (the optimizer step)."""
        if self.lanes is None:
            return
        for lane in self.lanes.values():
            if lane is not self.stream_obj:
                self.stream_obj.wait_stream(lane)

    def recv_loss_grad(self, mb, out_idx, grad):
        slot = self.mbs[mb]
        buf = slot.loss_grads.get(out_idx)
        if buf is None:
            return
        slot.grad_seen.add(out_idx)
        if grad is None:
            return
        g = grad.detach()
        if g.shape != buf.shape:
            raise RuntimeError("loss gradient of output %d has shape %s, expected %s"
                               % (out_idx, tuple(g.shape), tuple(buf.shape)))
        if self.dyn_scale:
            if g.device == buf.device and g.dtype.is_floating_point and g.is_contiguous() and buf.is_contiguous():
                self.kernels.scale_by_state(g, self.scaler_state, buf, g.numel())(self.stream())
            else:
                # the kernel walks both operands as flat arrays: anything with strides of its own (an output
                # kept channels-last in memory, a permuted gradient) goes through a stride-aware copy.
                # The product is formed in fp32 (the scale itself, 65536 by default, is not an fp16 number)
                # and the scale stays on the device (a 0-dim view of the scaler state, no host read).
                buf.copy_(g.to(device=buf.device, dtype=torch.float32) * self.scaler_state[0])
            return
        scale = self.option.loss_scale
        if g.device == buf.device and g.is_contiguous() and buf.is_contiguous() and g.dtype.is_floating_point:
            if scale != 1.0:
                self.kernels.axpby(g, scale, None, 0.0, buf, g.numel())(self.stream())
            else:
                self.kernels.cast(g, buf, g.numel())(self.stream())
        else:
            buf.copy_(g * scale if scale != 1.0 else g)

    def finish_micro_batch(self, mb):
        """Outputs whose hook never fired: zero gradient, except scalars which get 1
        (the implicit gradient the reference keeps, worker.py:1568-1573)."""
        slot = self.mbs[mb]
        for oi, buf in slot.loss_grads.items():
            if oi not in slot.grad_seen:
                if self.dyn_scale and buf.dim() == 0:
                    self.kernels.scale_by_state(self._one, self.scaler_state, buf, 1)(self.stream())
                    continue
                self.kernels.fill(buf, self.option.loss_scale if buf.dim() == 0 else 0.0, buf.numel())(self.stream())

    def _run_pending_fills(self, stream):
        fills, self.params.pending_fills = self.params.pending_fills, []
        for launch in fills:
            launch(stream)

    def _run_dw_job(self, stage, stream):
        """The stage's weight-gradient products over all micro-batches of the step, after its last
        backward job and on that job's stream (built when every micro-batch slot exists)."""
        job = self.dw_jobs.get(stage)
        if job is None:
            progs = [self.mbs[m].stage_programs[stage] for m in sorted(self.mbs)]
            self.pool.lane = ("dw", stage)    # this job's temporaries are its own: jobs of two stages may overlap
            launches = self.lowerer.lower_deferred_dw(progs) if any(p.dw_deferred for p in progs) else []
            self.pool.lane = 0
            if self.stream_obj is not None:
                # the job is about to run on its lane; what its lowering put on the device through
                # torch's current stream (the table of the batched reduction) has to be there first
                torch.cuda.current_stream(self.device).synchronize()
            job = self.dw_jobs[stage] = [launches, None]
            self._run_pending_fills(stream)    # (demoted while the job was lowered: only this job writes them)
        if job[1] is not None:
            job[1](stream)
        else:
            for launch in job[0]:
                launch(stream)

    def run_job(self, stage, mb, is_fwd):
        prog = self.mbs[mb].stage_programs[stage]
        if self.lanes is None:
            if is_fwd:
                prog.run_forward(self.stream())
            else:
                prog.run_backward(self.stream())
                if self.last_backward.get(stage) == mb and self.stack_dw:
                    self._run_dw_job(stage, self.stream())
            return
        # the job goes to its rank's stream, after the jobs of other ranks whose results it reads:
        # forward after the producers of its inputs, backward after the consumers of its outputs
        pg = self.part_graph
        st = pg.nodes[stage]
        lane = self.lanes[self._lane_key(stage, is_fwd)]
        if is_fwd:
            deps = {(src[0], True) for src in st.input_source if src is not None}
        else:
            deps = {(t.idx, False) for t in pg.nodes.values()
                    if any(src is not None and src[0] == stage for src in t.input_source)}
            deps.add((stage, True))    # its own forward (which followed the producers of its inputs)
        for other, d in sorted(deps):
            if self.lanes[self._lane_key(other, d)] is not lane:
                ev = self._job_events.get((other, mb, d))
                if ev is None:
                    raise RuntimeError("job order: stage %d of micro-batch %d runs before stage %d (%s)"
                                       % (stage, mb, other, "forward" if is_fwd else "backward"))
                lane.wait_event(ev)
        if not is_fwd and lane is not self.stream_obj and stage in self._output_stages:
            ev = self._loss_events.get(mb)
            if ev is not None:
                lane.wait_event(ev)
        if is_fwd:
            prog.run_forward(lane.cuda_stream)
        else:
            prog.run_backward(lane.cuda_stream)
        self._event(self._job_events, (stage, mb, is_fwd)).record(lane)   # (the weight-gradient job feeds no other job)
        if not is_fwd and self.last_backward.get(stage) == mb and self.stack_dw:
            self._run_dw_job(stage, lane.cuda_stream)

    def init_optimizer(self, optimizer):
        if optimizer is not None:
            self.optimizer = optimizer
        elif self.optimizer is None:
            params = [p for p in self.stage_parameters() if p.requires_grad]
            if params:
                cls = get_optimizer_cls(self.option.optimizer_type)
                self.optimizer = cls(params, **self.option.optimizer_kwargs)

    def scaler_scale(self):
        """Current loss scale (synchronises; for logging and tests)."""
        return float(self.scaler_state[0].item()) if self.dyn_scale else float(self.option.loss_scale)

    def _dynamic_optimizer_step(self, opt):
        """GradScaler.unscale_ + step + update on the device (pfeife/mp/worker.py:1432-1436): the
        gradients are unscaled in place and checked; an Adam/AdamW step reads the overflow flag
        itself, any other optimizer is skipped after one host read of the flag."""
        s = self.stream()
        key = (len(self.params.params), len(self.params.zero))
        if getattr(self, "_unscale_key", None) != key:
            self._unscale = [self.kernels.scaler_unscale(buf, n, self.scaler_state)
                             for buf, n in self.params.grad_buffers()]
            self._unscale_key = key
        for launch in self._unscale:
            launch(s)
        if opt is not None:
            if self._fused_adam_applicable(opt):
                self._fused_adam_step(opt, scaled=True)
            elif float(self.scaler_state[2].item()) == 0.0:
                opt.step()
        o = self.option
        self.kernels.scaler_update(self.scaler_state, o.growth_factor, o.backoff_factor, o.growth_interval)(s)

    def optimizer_step(self):
        opt = self.optimizer
        if self.dyn_scale:
            return self._dynamic_optimizer_step(opt)
        if self.option.loss_scale != 1.0:   # gradients leave the step unscaled, with or without an optimizer
            key = (len(self.params.params), len(self.params.zero))
            if getattr(self, "_unscale_key", None) != key:
                self._unscale = self.params.scale_grads_launches(1.0 / self.option.loss_scale)
                self._unscale_key = key
            for launch in self._unscale:
                launch(self.stream())
        if opt is None:
            return
        if self._fused_adam_applicable(opt):
            self._fused_adam_step(opt)
        else:
            opt.step()

    def _fused_adam_applicable(self, opt):
        """torch.optim.Adam / AdamW in their plain configuration on fp32 GPU parameters run as one
        HIP launch per param group; anything else keeps PyTorch's own step()."""
        if not hasattr(self.kernels, "adam_step") or type(opt) not in (torch.optim.Adam, torch.optim.AdamW):
            return False
        for g in opt.param_groups:
            if g.get("amsgrad") or g.get("maximize") or g.get("capturable") or g.get("differentiable"):
                return False
            if torch.is_tensor(g["lr"]) or g.get("decoupled_weight_decay", False) and type(opt) is torch.optim.Adam:
                return False
            for p in g["params"]:
                if p.grad is None:
                    continue
                if (p.dtype != torch.float32 or p.grad.dtype != torch.float32 or not p.is_cuda
                        or not p.is_contiguous() or not p.grad.is_contiguous() or p.grad.is_sparse):
                    return False
        return True

    def _fused_adam_step(self, opt, scaled=False):
        cache = self.__dict__.setdefault("_adam_tables", {})
        s = self.stream()
        rebuilt = False
        groups = []
        for gi, g in enumerate(opt.param_groups):
            params = [p for p in g["params"] if p.grad is not None]
            if not params:
                continue
            for p in params:   # state exactly as torch.optim.Adam initialises it
                st = opt.state[p]
                if len(st) == 0:
                    st["step"] = torch.tensor(0.0, dtype=torch.float32)
                    st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
            sig = tuple((p.data_ptr(), p.grad.data_ptr(), opt.state[p]["exp_avg"].data_ptr()) for p in params)
            ent = cache.get(gi)
            if ent is None or ent[0] != sig:
                table = self.kernels.adam_table([p.data for p in params], [p.grad for p in params],
                                                [opt.state[p]["exp_avg"] for p in params],
                                                [opt.state[p]["exp_avg_sq"] for p in params])
                ent = cache[gi] = (sig, table)
                rebuilt = True
            groups.append((g, params, ent[1]))
        if scaled and rebuilt:
            self._seed_device_step_count(opt, groups)
        for g, params, (table, n_items, max_n) in groups:
            b1, b2 = g["betas"]
            if scaled:
                # skipped on overflow; the bias corrections use the device's count of completed steps.
                # The host-side `step` entries are brought up to date from that count when somebody
                # reads them (sync_optimizer_steps: optimizer.state_dict() calls it)
                self.kernels.adam_step_scaled(table, n_items, max_n, float(g["lr"]), float(b1), float(b2),
                                              float(g["eps"]), float(g["weight_decay"]),
                                              type(opt) is torch.optim.AdamW, self.scaler_state, s)
                self._host_steps_stale = True
            else:
                step = int(opt.state[params[0]]["step"].item()) + 1
                self.kernels.adam_step(table, n_items, max_n, float(g["lr"]), float(b1), float(b2), float(g["eps"]),
                                       float(g["weight_decay"]), step, type(opt) is torch.optim.AdamW, s)
                for p in params:
                    opt.state[p]["step"] += 1

    def _seed_device_step_count(self, opt, groups):
        """The fused step under dynamic loss scaling takes Adam's bias corrections from the device's
        count of completed steps (scaler_state[3]).  Whenever the optimizer's state tensors are new
        to this worker (first step, `load_state_dict`), that count is set from the optimizer's own
        `step` entries, so a resumed optimizer continues at step k + 1 against its warm moments.
        One counter serves every parameter: an optimizer whose parameters disagree is refused."""
        if getattr(self, "_host_steps_stale", False) and getattr(self, "_steps_owner", None) is opt:
            self.sync_optimizer_steps()
        steps = {int(float(opt.state[p]["step"])) for _, params, _ in groups for p in params}
        if len(steps) > 1:
            raise RuntimeError("fused Adam step with dynamic loss scaling: the optimizer's parameters are at "
                               "different step counts %s; one device-side counter serves them all" % sorted(steps))
        k = float(steps.pop()) if steps else 0.0
        if float(self.scaler_state[3].item()) != k:
            self.scaler_state[3:4].fill_(k)
        if getattr(self, "_steps_owner", None) is not opt:
            self._steps_owner = opt
            if hasattr(opt, "register_state_dict_pre_hook"):
                opt.register_state_dict_pre_hook(lambda o: self.sync_optimizer_steps())

    def sync_optimizer_steps(self):
        """Writes the device's count of completed optimizer steps into the optimizer's `step`
        entries (one host read).  torch.amp.GradScaler leaves `step` untouched on a skipped step;
        so does this, which is why the entries cannot simply be bumped on the host."""
        opt = getattr(self, "_steps_owner", None)
        if opt is None or not self.dyn_scale or not getattr(self, "_host_steps_stale", False):
            return
        done = float(self.scaler_state[3].item())
        for g in opt.param_groups:
            for p in g["params"]:
                st = opt.state.get(p)
                if st and "step" in st:
                    if torch.is_tensor(st["step"]):
                        st["step"].fill_(done)
                    else:
                        st["step"] = done
        self._host_steps_stale = False

    def scaler_state_dict(self):
        """The dynamic loss scaler's state in torch.amp.GradScaler.state_dict()'s layout (empty
        for a static scale), for checkpoints."""
        if not self.dyn_scale:
            return {}
        st = self.scaler_state.tolist()
        o = self.option
        return {"scale": st[0], "growth_factor": o.growth_factor, "backoff_factor": o.backoff_factor,
                "growth_interval": o.growth_interval, "_growth_tracker": int(st[1])}

    def load_scaler_state_dict(self, state):
        if not self.dyn_scale:
            if state:
                raise RuntimeError("this worker runs with a static loss scale; there is no scaler state to load")
            return
        self.scaler_state[0:1].fill_(float(state["scale"]))
        self.scaler_state[1:2].fill_(float(state.get("_growth_tracker", 0)))
        self.scaler_state[2:3].fill_(0.0)

    # -- reporting -----------------------------------------------------------------------
    def memory_report(self):
        fwd = sum(p.fwd_bytes for s in self.mbs.values() for p in s.stage_programs.values())
        return "forward buffers %s, backward/scratch buffers %s" % (fmem(fwd), fmem(self.pool.bytes))

    def launch_counts(self):
        out = {}
        for mb, slot in self.mbs.items():
            for sid, p in slot.stage_programs.items():
                out[(sid, mb)] = (len(p.fwd), len(p.bwd))
        return out
