"""Public front-end: `PartialRunner`, `PartialModule`, `partial_compiler`.

Same contract as pfeife/mp/partial/module.py:37-438:

    runner = PartialRunner(option, optimizer)
    model = torch.compile(model, backend=partial_compiler)
    runner.set_exec_fn(fn)            # fn(*micro_batch) calls model, computes a loss, calls loss.backward()
    losses = runner.step(*batch)      # list of fn's return values, one per micro-batch, in order

`step` splits the batch (pfeife/batch.py), runs `fn` once per micro-batch on a
helper thread that parks inside the compiled model until the schedule has
produced that micro-batch's outputs (module.py:161-166, 417-433), and executes
the stage jobs on the calling thread in the schedule's order.  Exactly one
thread is runnable at any time, as in the reference (module.py:87-89, 145-159).

What differs: the first `step` does not profile the model.  The probe call of
`fn` (module.py:168-170) only records the captured graph and the micro-batch's
input signature, builds the stage programs, and hands `fn` zero-valued outputs
of the right shape so that user code can run through its loss once; like the
reference's probe it contributes nothing to the gradients.
"""
import threading
from functools import partial
from queue import Queue
from typing import List

import torch
import torch.fx as fx
import torch.nn as nn

from ...batch import split_args_kwargs
from ...executor.values import Val
from ...graph.canonicalize import canonicalize
from ...graph.partition_graph import compute_nodes, is_static_placeholder, partition_by_split_points
from ...option import PipeOption
from ...utils import get_logger, to_device
from ..net_states import get_state
from ..worker import StageWorker

STEP_TOKEN = "###<<STEP_TOKEN>>###"


def _same_shapes(args, kwargs):
    """Do the micro-batches of a step agree in the shapes and dtypes of all their tensors?  (A batch
    that does not divide evenly gives the first micro-batches one row more, pfeife/batch.py:45.)"""
    from torch.utils._pytree import tree_flatten

    sigs = set()
    for a, k in zip(args, kwargs):
        leaves, _ = tree_flatten((a, k))
        sigs.add(tuple((tuple(t.shape), t.dtype) for t in leaves if torch.is_tensor(t)))
    return len(sigs) <= 1


class _ExecError:
    def __init__(self, exc):
        self.exc = exc


class _StepAborted(BaseException):
    """Raised inside a parked micro-batch thread when the step it belongs to has failed."""


_ABORT = object()


class PartialRunner:
    def __init__(self, option: PipeOption = None, optimizer=None, kernels=None):
        """`kernels` is for tests of the host logic only (a kernel table double);
        user code never passes it and the HIP table is the only one shipped."""
        self.option = option if option is not None else PipeOption()
        self.optimizer = optimizer
        self.exec_fn = None
        self.net_state = get_state()
        self._compiled = False
        self._probing = False
        self._train_queues = [Queue() for _ in range(self.option.batch_cnt)]
        self._return_queues = [Queue() for _ in range(self.option.batch_cnt)]
        self._batch_threads = []
        self.results = []
        self.worker = StageWorker(self, self.option, self.net_state.device, kernels)
        # stage programs are built for concrete shapes: a new micro-batch shape must give a new static
        # graph (handled as an alias of the pipelined one), not a symbolic-shape graph
        torch._dynamo.config.automatic_dynamic_shapes = False
        PartialModule.set_runner(self)
        for i in range(self.option.batch_cnt):
            t = threading.Thread(target=self._exec_loop, args=(i,), daemon=True, name="pfeife-mb%d" % i)
            self._batch_threads.append(t)
            t.start()

    def set_exec_fn(self, exec_fn):
        self.exec_fn = exec_fn

    # -- one optimisation step ---------------------------------------------------
    def step(self, *args, **kwargs):
        """One optimisation step.  All device work of the step is issued on the worker's own
        stream, ordered after the caller's current stream on entry and before it on exit."""
        so = self.worker.stream_obj
        if so is None:
            return self._step(*args, **kwargs)
        outer = torch.cuda.current_stream(so.device)
        so.wait_stream(outer)
        with torch.cuda.stream(so):
            out = self._step(*args, **kwargs)
        outer.wait_stream(so)
        return out

    def _step(self, *args, **kwargs):
        if self.exec_fn is None:
            raise RuntimeError("call set_exec_fn() before step()")
        option = self.option
        args, kwargs = split_args_kwargs(args, kwargs, option.batch_cnt)
        self.worker.uniform_mbs = _same_shapes(args, kwargs)

        if not self._compiled:
            self._probe_forward(args[0], kwargs[0])
            if option.print_graph:
                print("Found %d graphs in the main module" % len(PartialModule._all_modules))

        self.reset()
        self.results = []
        self._parked = set()
        try:
            return self._run_step(args, kwargs)
        except BaseException:
            self._abort_parked()
            raise

    def _abort_parked(self):
        """A failed step leaves the micro-batch threads that already handed their inputs over
        parked inside the compiled model; wake them with an abort so that each one unwinds out of
        exec_fn and is ready for the next step()."""
        for bid in sorted(self._parked):
            PartialModule._module_queues[bid].put(_ABORT)
            self._return_queues[bid].get()
        self._parked = set()

    def _run_step(self, args, kwargs):
        option = self.option
        pp = PartialModule._pp_modules[0] if PartialModule._pp_modules else None
        worker = self.worker

        # every micro-batch thread runs user code up to the compiled model, hands its
        # inputs to the worker and parks there
        for bid in range(option.batch_cnt):
            self._train_queues[bid].put((args[bid], kwargs[bid]))
            tok = self._return_queues[bid].get()
            if isinstance(tok, _ExecError):
                raise tok.exc
            if tok is STEP_TOKEN:
                self._parked.add(bid)
            else:
                # exec_fn returned without reaching a pipelined graph: nothing to schedule for it
                self.results.append(tok)
                if pp is not None:
                    raise RuntimeError("exec_fn finished without calling the compiled model")

        if pp is None:
            return self._take_results()

        worker.begin_step()
        for i, (stage, mb, is_fwd) in enumerate(worker.order):
            worker.run_job(stage, mb, is_fwd)
            if is_fwd and worker.last_forward.get(i) == mb:
                self.finalize_output(mb)
        worker.end_jobs()
        worker.optimizer_step()
        worker.steps_done += 1
        return self._take_results()

    def _take_results(self):
        results, self.results = self.results, []
        return results

    def finalize_output(self, batch_idx):
        """Wake micro-batch `batch_idx`: its outputs exist; wait until its exec_fn has
        returned (loss computed, backward hooks fired)."""
        self.worker.outputs_ready(batch_idx)
        PartialModule._module_queues[batch_idx].put(None)
        ret = self._return_queues[batch_idx].get()
        self._parked.discard(batch_idx)
        if isinstance(ret, _ExecError):
            raise ret.exc
        self.worker.finish_micro_batch(batch_idx)
        self.worker.loss_grads_ready(batch_idx)
        self.results.append(ret)

    def backward_hook(self, batch_idx, output_idx, grad):
        self.worker.recv_loss_grad(batch_idx, output_idx, grad)

    def reset(self):
        for pm in PartialModule._all_modules:
            pm.reset()

    def gather_params(self):
        """Parameters never leave the user's module on a single GPU; kept for API parity
        (module.py:115-117)."""
        return None

    def log_memory_usage(self):
        get_logger().info(self.worker.memory_report())

    def scaler_state_dict(self):
        """State of the dynamic loss scaler (torch.amp.GradScaler.state_dict() layout) for a
        checkpoint; the reference keeps its GradScaler inside the worker and saves nothing
        (pfeife/mp/worker.py:133-145).  `optimizer.state_dict()` already carries the count of
        completed steps in its `step` entries."""
        return self.worker.scaler_state_dict()

    def load_scaler_state_dict(self, state):
        self.worker.load_scaler_state_dict(state)

    def train(self):
        """No-op, as in the reference (pfeife/mp/partial/module.py:175-177): stage programs are built
        from the graph TorchDynamo captured, and a captured dropout with p > 0 is refused at lowering."""

    def eval(self):
        """No-op, as in the reference (pfeife/mp/partial/module.py:179-181)."""

    # -- helpers --------------------------------------------------------------------
    def _exec_loop(self, batch_idx):
        q = self._train_queues[batch_idx]
        while True:
            args, kwargs = q.get()
            try:
                if self.worker.stream_obj is not None:
                    torch.cuda.set_device(self.net_state.device)
                    with torch.cuda.stream(self.worker.stream_obj):   # user code shares the step's stream
                        ret = self.exec_fn(*args, **kwargs)
                else:
                    ret = self.exec_fn(*args, **kwargs)
            except BaseException as e:  # surfaced on the thread that called step()
                ret = _ExecError(e)
            self._return_queues[batch_idx].put(ret)

    def _probe_forward(self, args, kwargs):
        self._probing = True
        try:
            self.exec_fn(*args, **kwargs)
        finally:
            self._probing = False
        self._compiled = True
        self.worker.init_optimizer(self.optimizer)


class PartialModule(nn.Module):
    _module_queues: List[Queue] = []
    _runner: PartialRunner = None
    _all_modules: List["PartialModule"] = []
    _pp_modules: List["PartialModule"] = []
    _option: PipeOption = None

    def __init__(self, gm: fx.GraphModule, example_inputs=None):
        super().__init__()
        self.gm = gm
        self.example_inputs = list(example_inputs) if example_inputs is not None else None
        self.curr_batch = 0
        self.net_state = get_state()
        self.device = self.net_state.device
        self.probed = False
        n_compute = len(compute_nodes(gm))
        has_params = any(isinstance(e, nn.Parameter) for e in (self.example_inputs or []))
        can_pp = all(not m.should_pp for m in self._all_modules)
        # pipeline the first captured graph that has real work in it (reference: node-count test,
        # module.py:205-216)
        self.should_pp = can_pp and n_compute >= 2 * self.net_state.pp_size and has_params
        if self._option is not None and self._option.print_graph:
            print("================ GRAPH %d: %d nodes / PP enabled: %s ================"
                  % (len(self._all_modules) + 1, len(gm.graph.nodes), self.should_pp))
            gm.graph.print_tabular()
        self.partition_graph = None
        self._canonical, self._folded = False, []
        # TorchDynamo recompiles when a micro-batch arrives with a new shape (ragged last chunk);
        # a structurally identical graph is the same pipeline, run by the module that owns the programs
        self.alias_of = None
        if not self.should_pp:
            sig = self._structure(gm)
            for m in self._all_modules:
                if m.should_pp and m._sig == sig:
                    self.alias_of = m
                    break
        self._sig = self._structure(gm) if self.should_pp else None
        self._all_modules.append(self)

    @staticmethod
    def _structure(gm):
        return tuple((n.op, str(n.target)) for n in gm.graph.nodes)

    @staticmethod
    def set_runner(runner: PartialRunner):
        PartialModule._runner = runner
        PartialModule._option = runner.option
        PartialModule._module_queues = [Queue() for _ in range(runner.option.batch_cnt)]
        PartialModule._all_modules = []
        PartialModule._pp_modules = []

    def reset(self):
        self.curr_batch = 0

    # -- compilation --------------------------------------------------------------------
    def _compile(self, args):
        option = self._option
        worker = self._runner.worker
        ex = self.example_inputs if self.example_inputs is not None else list(args)
        # module state is identified on the real call arguments (they are the live tensors)
        live = list(args)
        if not self._canonical:
            # library spellings (decomposed norms, eager attention, mask / rotary-table bookkeeping)
            # -> the lowering's vocabulary; constants it evaluated become extra static inputs
            live, info = canonicalize(self.gm, live, worker.device, is_static_placeholder)
            self._canonical, self._folded = True, live[len(args):]
            if any(info.values()):
                get_logger().info("graph canonicalised: %s", info)
        else:
            live = live + self._folded
        points = option.split_points
        plan = None
        if self.alias_of is not None:
            points = self.alias_of.split_points_used      # same pipeline, another micro-batch shape
        elif points is None and option.device_cnt > 1:
            plan = worker.plan_split_points(self.gm, live)
            points = plan.split_points
        self.split_points_used = points
        self.partition_graph = partition_by_split_points(self.gm, live, points, option.device_cnt)
        if option.print_graph:
            if plan is not None:
                print(plan.describe())
            self.partition_graph.print_graph()
            for idx, st in self.partition_graph.nodes.items():
                print("================ PARTITION GRAPH %d: %d nodes ================"
                      % (idx, len(st.graph_module.graph.nodes)))
                st.graph_module.graph.print_tabular()
        worker.set_partition_graph(self.partition_graph, live)
        if self.alias_of is None:
            self._pp_modules.append(self)
        del ex

    def _dynamic_inputs(self, args):
        pg = self.partition_graph
        return {i: (to_device(a, self.device) if not torch.is_tensor(a) else a)
                for i, a in enumerate(args) if not pg.static_placeholder[i]}

    def _ensure_programs(self, mb, args):
        worker = self._runner.worker
        dyn = self._dynamic_inputs(args)
        sig = worker._signature([dyn[i] for i in sorted(dyn)])
        slot = worker.mbs.get(mb)
        if slot is None or slot.input_sig != sig or slot.graph is not self.partition_graph:
            worker.build_micro_batch(mb, dyn, self.partition_graph).graph = self.partition_graph
        return dyn

    def _outputs_for_user(self, mb, probe):
        worker = self._runner.worker
        slot = worker.mbs[mb]
        outs = []
        for oi, v in enumerate(slot.outputs):
            if isinstance(v, Val):
                if probe:
                    t = torch.zeros_like(v.buf)
                else:
                    t = v.buf.detach()
                if v.req_grad:
                    t.requires_grad_()
                    if not probe:
                        t.register_hook(partial(self._runner.backward_hook, mb, oi))
                outs.append(t)
            else:
                outs.append(v)
        spec = self.partition_graph.output_spec
        if spec == "single":
            return outs[0]
        return tuple(outs) if spec == "tuple" else outs

    # -- call ----------------------------------------------------------------------------
    def forward(self, *args):
        owner = self.alias_of if self.alias_of is not None else self
        if not owner.should_pp:
            return self.gm(*to_device(args, self.device))
        runner = self._runner
        if runner._probing:
            if self.partition_graph is None:
                self._compile(args)
            self._ensure_programs(0, args)
            return self._outputs_for_user(0, probe=True)
        if owner.partition_graph is None:
            raise RuntimeError("the compiled model was called outside PartialRunner.step()")
        if self.partition_graph is None:
            self._compile(args)  # same pipeline, captured again for another micro-batch shape

        mb = owner.curr_batch
        owner.curr_batch += 1
        if mb >= self._option.batch_cnt:
            raise RuntimeError("the compiled model was called more than batch_cnt times in one step")
        dyn = self._ensure_programs(mb, args)
        worker = runner.worker
        for i, v in dyn.items():
            if torch.is_tensor(v):
                worker.distribute_input(mb, i, v)
        runner._return_queues[mb].put(STEP_TOKEN)   # inputs are in place; main thread may schedule
        if self._module_queues[mb].get() is _ABORT:  # parked until this micro-batch's outputs exist
            raise _StepAborted()
        return self._outputs_for_user(mb, probe=False)


def partial_compiler(gm: fx.GraphModule, example_inputs: List[torch.Tensor]):
    if PartialModule._runner is None:
        raise RuntimeError("create a PartialRunner before the compiled model is first called")
    return PartialModule(gm, example_inputs)
