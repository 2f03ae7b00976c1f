"""Micro-batch split of the arguments of one optimisation step.

Host-side mirror of pfeife/batch.py:30-132 (`shard_dict_of_args`,
`split_args_kwargs`): every tensor found in the (nested) arguments is cut
along dimension 0 into `batch_split` chunks with torch.tensor_split semantics
(the first N % n chunks hold one extra row), plain lists that contain no
tensor are cut into ceil(len/n)-sized runs (trailing runs may be empty), and
every other leaf is replicated.  The pytree structure of each argument is kept.

The chunks returned here are zero-copy views; `chunk_rows` gives the row
range of each chunk so that the executor can materialise a micro-batch slab
into a stage's preallocated input buffer with the pf_split_gather kernel.
"""
import torch
from torch.utils._pytree import tree_flatten, tree_map, tree_unflatten


def send_value(value, device):
    return tree_map(lambda v: v.to(device) if torch.is_tensor(v) else v, value)


def chunk_rows(n_rows, batch_split):
    """Row ranges [(start, count)] of torch.tensor_split(x, batch_split, 0)."""
    base, extra = divmod(n_rows, batch_split)
    out, start = [], 0
    for i in range(batch_split):
        cnt = base + (1 if i < extra else 0)
        out.append((start, cnt))
        start += cnt
    return out


def _keeps_whole(v):
    """Leaves of the argument pytree: everything but tuples, dicts and lists that hold tensors."""
    if isinstance(v, (tuple, dict)):
        return False
    if isinstance(v, list):
        return not any(torch.is_tensor(x) for x in v)
    return True


def _split_leaf(v, n):
    if torch.is_tensor(v):
        return list(torch.tensor_split(v, n, 0))
    if isinstance(v, list):
        step = (len(v) + n - 1) // n
        return [v[i * step:(i + 1) * step] for i in range(n)]
    return [v] * n


def shard_dict_of_args(args_dict, batch_split):
    specs = {}
    per_leaf = {}
    for key, arg in args_dict.items():
        flat, spec = tree_flatten(arg, is_leaf=_keeps_whole)
        specs[key] = spec
        per_leaf[key] = [_split_leaf(v, batch_split) for v in flat]
    chunks = []
    for ci in range(batch_split):
        chunks.append({key: tree_unflatten([leaf[ci] for leaf in per_leaf[key]], specs[key]) for key in args_dict})
    return chunks


def split_args_kwargs(args, kwargs, batch_split):
    """-> (list of `batch_split` arg tuples, list of `batch_split` kwarg dicts)"""
    if args is None:
        args_split = [(None,) for _ in range(batch_split)]
    else:
        per_chunk = shard_dict_of_args(dict(enumerate(args)), batch_split)
        args_split = [tuple(c[i] for i in range(len(c))) for c in per_chunk]
    if kwargs is None:
        kwargs_split = [dict() for _ in range(batch_split)]
    else:
        kwargs_split = shard_dict_of_args(kwargs, batch_split)
    return args_split, kwargs_split


def merge_chunks(chunks, out=None):
    """Inverse of the split for one tensor argument: stack the per-micro-batch tensors
    (`batch_cnt` chunks along dimension 0, chunk i holding the rows `chunk_rows` assigns to it)
    back into one batch-major tensor with the pf_merge_scatter kernel.  The reference returns
    the per-micro-batch values as a Python list (pfeife/mp/partial/module.py:99-102) and leaves
    any stacking to user code; this is that stacking done on the device."""
    chunks = [c for c in chunks]
    if not chunks:
        raise ValueError("merge_chunks: no chunks")
    first = chunks[0]
    if first.device.type != "cuda":
        raise RuntimeError("merge_chunks: the merge kernel needs GPU tensors (got %s)" % first.device)
    from .hip import HipKernels

    k = getattr(merge_chunks, "_k", None)
    if k is None:
        k = merge_chunks._k = HipKernels(first.device.index)
    tail = tuple(first.shape[1:])
    for c in chunks:
        if tuple(c.shape[1:]) != tail or c.dtype != first.dtype or c.device != first.device:
            raise ValueError("merge_chunks: chunks differ in trailing shape, dtype or device")
    total = sum(int(c.shape[0]) for c in chunks)
    if out is None:
        out = torch.empty((total,) + tail, dtype=first.dtype, device=first.device)
    elif tuple(out.shape) != (total,) + tail or not out.is_contiguous():
        raise ValueError("merge_chunks: bad output tensor")
    row_bytes = out[0].numel() * out.element_size() if total else 0
    start = 0
    for c in chunks:
        rows = int(c.shape[0])
        if rows:
            k.run("merge_scatter", c.contiguous(), out, row_bytes=row_bytes, row_start=start, n_rows=rows)
        start += rows
    return out
