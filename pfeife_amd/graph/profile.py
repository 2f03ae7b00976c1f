"""Per-node time and memory profile of a captured graph, the input of the auto-partitioner.

Counterpart of `gen_local_comp_graph` (pfeife/local/graph_bench.py:390-625): the reference
runs the FX graph three times under interpreters that record, per computation node, the
forward and backward time (mean of three timed runs), the activation memory kept for
backward, the weight memory and the bytes on every edge.  Here the whole graph is lowered
ONCE as a single stage for one micro-batch (the same launch lists a real stage replays),
the lowerer says which launches belong to which graph node, and the launches are timed on
the device with events recorded between the nodes (HIP events on the worker's stream; wall
clock for a host kernel table, whose launches are synchronous).  Memory figures are the
sizes of the buffers the lowering allocated, not allocator watermarks.  While the profile runs
the single-stage copy's buffers (one micro-batch of activations, a gradient buffer and a 16-bit
shadow per parameter) exist next to the model; they are released before it returns.
"""
import time
from dataclasses import dataclass, field
from typing import List

import torch

from ..executor.lowering import BufferPool, Lowerer, ParamStore
from ..executor.values import Val
from .partition_graph import compute_nodes, partition_by_split_points


@dataclass
class GraphProfile:
    """Index i is the i-th compute node of the captured graph (the numbering integer
    `split_points` use).  cut_bytes[i] / cut_values[i]: bytes / number of activation values that
    a stage boundary in front of node i would hand over (i = 1 .. n-1; entries 0 and n are 0)."""
    names: List[str] = field(default_factory=list)
    fwd_ms: List[float] = field(default_factory=list)
    bwd_ms: List[float] = field(default_factory=list)
    act_bytes: List[int] = field(default_factory=list)     # forward buffers the node allocates (kept for backward)
    param_bytes: List[int] = field(default_factory=list)   # module state first read by the node
    cut_bytes: List[int] = field(default_factory=list)
    cut_values: List[int] = field(default_factory=list)
    cut_ok: List[bool] = field(default_factory=list)       # False: a non-tensor value (a tuple) would cross
    temp_bytes: int = 0                                    # backward temporaries of the whole graph

    @property
    def n(self):
        return len(self.names)


def _tensor_bytes(v):
    return v.numel() * v.element_size() if torch.is_tensor(v) else 0


def cut_sizes(gm):
    """(bytes, count, ok) per cut position of the values that cross it: produced by a compute node
    before the cut and used by a compute node at or after it.  ok: every one is a plain tensor."""
    nodes = compute_nodes(gm)
    index = {n: i for i, n in enumerate(nodes)}
    n = len(nodes)
    add_b = [0] * (n + 2)
    add_c = [0] * (n + 2)
    add_x = [0] * (n + 2)     # values that are not plain tensors (tuples of tensors): not handed over
    for node in nodes:
        i = index[node]
        # a value that only the graph's output node reads stays on the producing stage
        last = max([index[u] for u in node.users if u in index] + [i])
        if last > i:
            ex = node.meta.get("example_value")
            b = _tensor_bytes(ex)
            # crosses the cuts in front of nodes i+1 .. last
            add_b[i + 1] += b
            add_b[last + 1] -= b
            add_c[i + 1] += 1
            add_c[last + 1] -= 1
            if isinstance(ex, (tuple, list)):
                add_x[i + 1] += 1
                add_x[last + 1] -= 1
    cb, cc, ok, rb, rc, rx = [], [], [], 0, 0, 0
    for i in range(n + 1):
        rb += add_b[i]
        rc += add_c[i]
        rx += add_x[i]
        cb.append(rb)
        cc.append(rc)
        ok.append(rx == 0)
    cb[0] = cc[0] = 0
    cb[n] = cc[n] = 0
    return cb, cc, ok


def profile_graph(kernels, device, compute_dtype, gm, live_args, repeats=3, stream=None):
    """Lower `gm` as one stage for the micro-batch `live_args` (the captured graph's call
    arguments: module state and one micro-batch of user inputs), run it, and time every node.
    Leaves the parameters' `.grad` as it found them."""
    device = torch.device(device)
    pg = partition_by_split_points(gm, live_args, None, 1)
    st = pg.nodes[0]
    nodes = compute_nodes(gm)
    params = ParamStore(kernels, device)
    pool = BufferPool(device)
    L = Lowerer(kernels, device, compute_dtype, params, pool)
    saved_grads = []
    ins = []
    first_use_bytes = {}
    for k, gi in enumerate(st.input_placeholder):
        ex = live_args[gi]
        if pg.static_placeholder[gi]:
            if ex.device != device:
                ex.data = ex.data.to(device)
            param = ex if isinstance(ex, torch.nn.Parameter) else None
            if param is not None:
                saved_grads.append((param, param.grad))
            ins.append(Val(ex.detach(), req_grad=bool(ex.requires_grad), param=param, name=st.inputs[k]))
            first_use_bytes[st.inputs[k]] = _tensor_bytes(ex)
        elif torch.is_tensor(ex):
            ins.append(Val(ex.detach().to(device).clone(), req_grad=False, name=st.inputs[k]))
        else:
            ins.append(ex)
    try:
        prog = L.lower_forward(st, 0, ins)
        out_grads = []
        for v in prog.outputs:
            if isinstance(v, Val) and v.req_grad:
                out_grads.append([torch.zeros_like(v.buf)])
            else:
                out_grads.append(None)
        L.lower_backward(prog, out_grads)

        cuda = device.type == "cuda"
        s = stream

        def run_list(launches, ranges, acc):
            """Runs the list once, adding each node's time (ms) to acc[name]."""
            marks = []
            pos = 0
            for name, a, b in ranges:
                if a > pos:            # launches that belong to no node (none today): charged to the next one
                    a = pos
                marks.append((name, a, b))
                pos = b
            if cuda:
                evs = [torch.cuda.Event(enable_timing=True) for _ in range(len(marks) + 1)]
                # the events go to the stream the launches go to (`s` is its raw handle)
                so = torch.cuda.ExternalStream(s, device=device) if s else torch.cuda.current_stream(device)
                for (name, a, b), ev in zip(marks, evs):
                    ev.record(so)
                    for launch in launches[a:b]:
                        launch(s)
                for launch in launches[pos:]:
                    launch(s)
                evs[-1].record(so)
                evs[-1].synchronize()
                for i, (name, a, b) in enumerate(marks):
                    if b > a:
                        acc[name] = acc.get(name, 0.0) + evs[i].elapsed_time(evs[i + 1])
            else:
                for name, a, b in marks:
                    t0 = time.perf_counter()
                    for launch in launches[a:b]:
                        launch(s)
                    if b > a:
                        acc[name] = acc.get(name, 0.0) + (time.perf_counter() - t0) * 1e3
                for launch in launches[pos:]:
                    launch(s)

        fwd_ranges = [(n_, a, b) for n_, a, b, _ in prog.fwd_ranges]
        pre = params.zero_launches() + params.refresh_launches()
        f_acc, b_acc = {}, {}
        for it in range(repeats + 1):
            for launch in pre:
                launch(s)
            fa, ba = ({}, {}) if it == 0 else (f_acc, b_acc)   # first pass warms up (code objects, caches)
            run_list(prog.fwd, fwd_ranges, fa)
            run_list(prog.bwd, prog.bwd_ranges, ba)
        if cuda:
            torch.cuda.synchronize(device)

        prof = GraphProfile()
        sub_nodes = compute_nodes(st.graph_module)
        if len(sub_nodes) != len(nodes):
            raise RuntimeError("profile: the single-stage copy has %d compute nodes, the graph %d"
                               % (len(sub_nodes), len(nodes)))
        act = {n_: by for n_, _, _, by in prog.fwd_ranges}
        placeholders = {n_.name for n_ in st.graph_module.graph.nodes if n_.op == "placeholder"}
        seen_state = set()
        for sn in sub_nodes:
            prof.names.append(sn.name)
            prof.fwd_ms.append(f_acc.get(sn.name, 0.0) / repeats)
            prof.bwd_ms.append(b_acc.get(sn.name, 0.0) / repeats)
            prof.act_bytes.append(int(act.get(sn.name, 0)))
            pb = 0
            for a in sn.all_input_nodes:
                if a.name in placeholders and a.name in first_use_bytes and a.name not in seen_state:
                    seen_state.add(a.name)
                    pb += first_use_bytes[a.name]
            prof.param_bytes.append(pb)
        prof.cut_bytes, prof.cut_values, prof.cut_ok = cut_sizes(gm)
        prof.temp_bytes = int(pool.bytes)
        return prof
    finally:
        for p, g in saved_grads:
            p.grad = g
        # the single-stage copy holds a second set of activations, gradient buffers and 16-bit
        # shadows: give them back before the real stages are built
        prog = out_grads = ins = None
        L = params = pool = None
        if device.type == "cuda":
            torch.cuda.synchronize(device)
            torch.cuda.empty_cache()
