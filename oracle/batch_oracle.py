"""TEST INFRASTRUCTURE -- CPU restatement of the reference's micro-batch split.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module.

Follows pfeife/batch.py:30-132.  Written with explicit row ranges instead of
torch.tensor_split so that the chunk boundaries are stated, not inherited:
chunk i of a tensor with N rows cut n ways starts at i*(N//n) + min(i, N % n)
and holds N//n + (1 if i < N % n else 0) rows (the documented behaviour of
torch.tensor_split with an integer `sections`, which batch.py:45 calls).
Pinned by tests/test_batch.py against torch.tensor_split itself, brute force over
N in [0, 3n], nested pytrees, list chunking (batch.py:47-53) and replication
(batch.py:55).
"""
import torch


def tensor_chunk_bounds(n_rows, n_chunks):
    q, r = divmod(n_rows, n_chunks)
    return [(i * q + min(i, r), q + (1 if i < r else 0)) for i in range(n_chunks)]


def _split_value(v, n, i):
    if torch.is_tensor(v):
        start, cnt = tensor_chunk_bounds(v.shape[0], n)[i]
        return v[start:start + cnt]
    if isinstance(v, tuple):
        return tuple(_split_value(x, n, i) for x in v)
    if isinstance(v, dict):
        return {k: _split_value(x, n, i) for k, x in v.items()}
    if isinstance(v, list):
        if any(torch.is_tensor(x) for x in v):  # batch.py:21-27: such a list is a container, not a leaf
            return [_split_value(x, n, i) for x in v]
        size = -(-len(v) // n)  # batch.py:49
        return v[i * size:(i + 1) * size]
    return v


def split_args_kwargs(args, kwargs, n):
    if args is None:
        a = [(None,) for _ in range(n)]
    else:
        a = [tuple(_split_value(x, n, i) for x in args) for i in range(n)]
    if kwargs is None:
        k = [dict() for _ in range(n)]
    else:
        k = [{key: _split_value(x, n, i) for key, x in kwargs.items()} for i in range(n)]
    return a, k
