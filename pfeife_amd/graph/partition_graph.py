"""Cuts a TorchDynamo FX graph into pipeline-stage submodules.

Counterpart of pfeife/graph/partition_graph.py:53-122 (`PartitionNode`,
`PartitionGraph`) and :125-334 (`partition_module`), plus the manual-split
branch of the planner (pfeife/schedule/planner.py:635-665, 1271-1316) that turns
`split_points` into a stage per graph node and assigns stage i to pipeline rank
i % device_cnt.

Differences that follow from TorchDynamo >= 2.5: parameters and buffers arrive
as graph placeholders (not `get_attr`/`call_module`), so they are ordinary stage
inputs flagged `static`; and `split_points` integers index the graph's compute
nodes (everything except placeholders and the output node) in topological order,
which is deterministic, instead of allocator-dependent profiling nodes.  A
string entry names a module path ("blocks.12"): the stage starts at the first
compute node recorded under that path.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Set, Tuple

import torch
import torch.fx as fx
from torch.fx.passes.split_module import split_module


@dataclass
class ShapeMeta:
    size: Tuple[int, ...]
    dtype: torch.dtype
    requires_grad: bool

    @property
    def bytes(self):
        n = 1
        for s in self.size:
            n *= int(s)
        return n * torch.empty((), dtype=self.dtype).element_size()


@dataclass
class PartitionNode:
    """One pipeline stage."""
    idx: int
    rank: int = -1
    inputs: List[str] = field(default_factory=list)            # placeholder names of the stage, in order
    outputs: List[str] = field(default_factory=list)           # names of the values the stage returns, in order
    input_map: Dict[str, int] = field(default_factory=dict)    # name -> producing stage, -1 = graph input
    output_map: Dict[str, Set[int]] = field(default_factory=dict)  # name -> consuming stages, -1 = graph output
    input_shapes: List[Optional[ShapeMeta]] = field(default_factory=list)
    output_shapes: List[Optional[ShapeMeta]] = field(default_factory=list)
    graph_module: Optional[fx.GraphModule] = None
    # index into the original graph's placeholders for inputs that come from outside (-1 otherwise)
    input_placeholder: List[int] = field(default_factory=list)
    # (producing stage, index into its outputs) for inputs that come from another stage
    input_source: List[Optional[Tuple[int, int]]] = field(default_factory=list)


class PartitionGraph:
    def __init__(self):
        self.nodes: Dict[int, PartitionNode] = {}
        # for every placeholder of the captured graph: [(stage, index into stage.inputs)]
        self.inputs: List[List[Tuple[int, int]]] = []
        # for every value the captured graph returns: (stage, index into stage.outputs), or None for constants
        self.outputs: List[Optional[Tuple[int, int]]] = []
        self.output_spec = None  # structure of the original return value
        self.placeholder_names: List[str] = []
        self.static_placeholder: List[bool] = []

    # -- summary (the reference prints its PipeGraph the same way, pfeife/graph/pipe_graph.py:53-54,
    # :113-120, :145-154: one line per stage, one per stage-to-stage edge) --------------------------------
    def edges(self):
        """[(src stage, dst stage, bytes, [(value name, shape, dtype)])] for every pair of stages that
        exchange activations, in stage order."""
        out = {}
        for idx in sorted(self.nodes):
            st = self.nodes[idx]
            for name, meta in zip(st.outputs, st.output_shapes):
                for dst in sorted(d for d in st.output_map.get(name, ()) if d >= 0):
                    e = out.setdefault((idx, dst), [0, []])
                    if meta is not None:
                        e[0] += meta.bytes
                        e[1].append((name, tuple(meta.size), meta.dtype))
        return [(a, b, w, vals) for (a, b), (w, vals) in sorted(out.items())]

    def stage_summary(self, idx):
        """dict(weight, node_len, recv, send, inputs, outputs) of one stage: bytes of the module
        state it reads, number of compute nodes, bytes received from / sent to other stages."""
        st = self.nodes[idx]
        weight = recv = 0
        for meta, gi, src in zip(st.input_shapes, st.input_placeholder, st.input_source):
            if meta is None:
                continue
            if src is not None:
                recv += meta.bytes
            elif gi >= 0 and gi < len(self.static_placeholder) and self.static_placeholder[gi]:
                weight += meta.bytes
        send = sum(meta.bytes for name, meta in zip(st.outputs, st.output_shapes)
                   if meta is not None and any(d >= 0 for d in st.output_map.get(name, ())))
        n = len(compute_nodes(st.graph_module)) if st.graph_module is not None else 0
        return dict(weight=weight, node_len=n, recv=recv, send=send)

    def to_str(self):
        from ..utils import fmem

        lines = []
        edges = self.edges()
        lines.append("GRAPH: %d nodes / %d edges" % (len(self.nodes), len(edges)))
        lines.append("==== nodes ====")
        for idx in sorted(self.nodes):
            st = self.nodes[idx]
            s = self.stage_summary(idx)
            lines.append("Node [%d/%d] (weight: %s, node len: %d, recv weight: %s, send weight: %s)"
                         % (idx, st.rank, fmem(s["weight"]), s["node_len"], fmem(s["recv"]), fmem(s["send"])))
        lines.append("==== edges ====")
        for a, b, w, vals in edges:
            shapes = ", ".join("%s %s %s" % (n, list(sz), str(dt).replace("torch.", "")) for n, sz, dt in vals)
            lines.append("Edge (%d -> %d) (weight: %s, device: %d -> %d, values: %s)"
                         % (a, b, fmem(w), self.nodes[a].rank, self.nodes[b].rank, shapes))
        return "\n".join(lines)

    def print_graph(self):
        print(self.to_str())


def compute_nodes(gm: fx.GraphModule):
    return [n for n in gm.graph.nodes if n.op not in ("placeholder", "output", "get_attr")]


def _module_path(node):
    """Innermost-to-outermost module paths TorchDynamo recorded for a node, normalised to 'a.b.3.c'."""
    stack = node.meta.get("nn_module_stack")
    if not stack:
        return []
    out = []
    for _, (path, _cls) in stack.items():
        p = path
        for prefix in ("L['self'].", "L['self']", "self."):
            if p.startswith(prefix):
                p = p[len(prefix):]
                break
        p = p.replace("._modules['", ".").replace("']", "").replace("[", ".").replace("]", "").strip(".")
        out.append(p)
    return out


def resolve_split_points(gm: fx.GraphModule, split_points):
    """-> sorted list of compute-node indices at which a new stage starts."""
    nodes = compute_nodes(gm)
    resolved = []
    for sp in split_points or []:
        if isinstance(sp, int):
            if not (0 < sp < len(nodes)):
                raise RuntimeError("split point %d is outside the graph's %d compute nodes" % (sp, len(nodes)))
            resolved.append(sp)
            continue
        key = str(sp).strip(".")
        hit = None
        for i, n in enumerate(nodes):
            if any(p == key or p.startswith(key + ".") for p in _module_path(n)):
                hit = i
                break
        if hit is None:
            raise RuntimeError("split point '%s' matches no module path of the captured graph" % sp)
        if hit == 0:
            raise RuntimeError("split point '%s' is the first node of the graph; a stage would be empty" % sp)
        resolved.append(hit)
    if sorted(set(resolved)) != sorted(resolved):
        raise RuntimeError("duplicate split points: %s" % (split_points,))
    return sorted(resolved)


def stage_assignment(gm: fx.GraphModule, split_points) -> Dict[fx.Node, int]:
    starts = resolve_split_points(gm, split_points)
    stage_of = {}
    stage = 0
    for i, n in enumerate(compute_nodes(gm)):
        while stage < len(starts) and i >= starts[stage]:
            stage += 1
        stage_of[n] = stage
    return stage_of


def _shape_meta(v):
    if torch.is_tensor(v):
        return ShapeMeta(tuple(int(s) for s in v.shape), v.dtype, bool(v.requires_grad))
    return None


def is_static_placeholder(node: fx.Node, example):
    """Module state (parameters / buffers) as opposed to per-call user inputs."""
    if isinstance(example, torch.nn.Parameter):
        return True
    name = node.name
    # (constants the canonicalisation pass evaluated at compile time arrive as placeholders too)
    return torch.is_tensor(example) and ("_parameters_" in name or "_buffers_" in name or name.startswith("pf_folded_"))


def partition_module(gm: fx.GraphModule, stage_of: Dict[fx.Node, int], example_inputs=None,
                     device_cnt: int = 1) -> PartitionGraph:
    """Build the per-stage GraphModules and their IO maps."""
    n_stage = max(stage_of.values()) + 1 if stage_of else 1

    def callback(node):
        return stage_of[node]

    split = split_module(gm, None, callback, keep_original_order=True)
    pg = PartitionGraph()
    placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
    pg.placeholder_names = [n.name for n in placeholders]
    ex = list(example_inputs) if example_inputs is not None else [None] * len(placeholders)
    pg.static_placeholder = [is_static_placeholder(n, e) for n, e in zip(placeholders, ex)]
    pg.inputs = [[] for _ in placeholders]

    top_placeholders = [n for n in split.graph.nodes if n.op == "placeholder"]
    ph_index = {n: i for i, n in enumerate(top_placeholders)}
    if len(top_placeholders) != len(placeholders):
        raise RuntimeError("split_module changed the number of graph inputs")

    # value produced at top level -> (stage, out_idx)
    produced: Dict[fx.Node, Tuple[int, int]] = {}
    stage_nodes = {}
    for node in split.graph.nodes:
        if node.op == "call_module":
            sid = int(str(node.target).split("_")[-1])
            sub = getattr(split, node.target)
            pn = PartitionNode(idx=sid, rank=sid % max(1, device_cnt), graph_module=sub)
            sub_ph = [n for n in sub.graph.nodes if n.op == "placeholder"]
            if len(sub_ph) != len(node.args) or node.kwargs:
                raise RuntimeError("unexpected calling convention of stage %d" % sid)
            out_node = next(n for n in sub.graph.nodes if n.op == "output")
            res = out_node.args[0]
            outs = list(res) if isinstance(res, (tuple, list)) else [res]
            pn.outputs = [o.name if isinstance(o, fx.Node) else repr(o) for o in outs]
            pn.output_map = {name: set() for name in pn.outputs}
            pn.output_shapes = [_shape_meta(o.meta.get("example_value")) if isinstance(o, fx.Node) else None
                                for o in outs]
            pn._multi = isinstance(res, (tuple, list))
            for i, (ph, arg) in enumerate(zip(sub_ph, node.args)):
                pn.inputs.append(ph.name)
                if arg in ph_index:
                    gi = ph_index[arg]
                    pn.input_map[ph.name] = -1
                    pn.input_placeholder.append(gi)
                    pn.input_source.append(None)
                    pn.input_shapes.append(_shape_meta(ex[gi]))
                    pg.inputs[gi].append((sid, i))
                else:
                    src_stage, out_idx = produced[arg]
                    pn.input_map[ph.name] = src_stage
                    pn.input_placeholder.append(-1)
                    pn.input_source.append((src_stage, out_idx))
                    src = pg.nodes[src_stage]
                    pn.input_shapes.append(src.output_shapes[out_idx])
                    src.output_map[src.outputs[out_idx]].add(sid)
            pg.nodes[sid] = pn
            stage_nodes[node] = pn
            if not pn._multi:
                produced[node] = (sid, 0)
        elif node.op == "call_function" and node.target.__name__ == "getitem" and node.args[0] in stage_nodes:
            produced[node] = (stage_nodes[node.args[0]].idx, int(node.args[1]))
        elif node.op == "output":
            res = node.args[0]
            pg.output_spec = "tuple" if isinstance(res, tuple) else ("list" if isinstance(res, list) else "single")
            outs = list(res) if isinstance(res, (tuple, list)) else [res]
            for o in outs:
                if isinstance(o, fx.Node) and o in produced:
                    sid, oi = produced[o]
                    pg.outputs.append((sid, oi))
                    st = pg.nodes[sid]
                    st.output_map[st.outputs[oi]].add(-1)
                elif isinstance(o, fx.Node) and o in ph_index:
                    pg.outputs.append(("input", ph_index[o]))
                else:
                    pg.outputs.append(("const", o))
        elif node.op == "placeholder":
            continue
        else:
            raise RuntimeError("unexpected top-level node after the stage split: %s" % node.format_node())
    if sorted(pg.nodes) != list(range(n_stage)):
        raise RuntimeError("stage split produced stages %s, expected %d" % (sorted(pg.nodes), n_stage))
    return pg


def partition_by_split_points(gm, example_inputs, split_points, device_cnt=1) -> PartitionGraph:
    return partition_module(gm, stage_assignment(gm, split_points), example_inputs, device_cnt)
