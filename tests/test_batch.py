"""Micro-batch split: oracle pinned against torch.tensor_split and brute force;
product (pfeife_amd.batch) bit-exact against the oracle."""
import torch

from oracle.batch_oracle import split_args_kwargs as oracle_split
from oracle.batch_oracle import tensor_chunk_bounds
from pfeife_amd.batch import chunk_rows, split_args_kwargs


def same(a, b):
    if torch.is_tensor(a):
        return torch.is_tensor(b) and a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b)
    if isinstance(a, (tuple, list)):
        return type(a) == type(b) and len(a) == len(b) and all(same(x, y) for x, y in zip(a, b))
    if isinstance(a, dict):
        return isinstance(b, dict) and list(a) == list(b) and all(same(a[k], b[k]) for k in a)
    return a == b


def test_chunk_bounds_brute_force_against_tensor_split():
    for n in range(1, 9):
        for N in range(0, 3 * n + 1):
            x = torch.arange(N * 2).view(N, 2)
            ref = torch.tensor_split(x, n, 0)
            bounds = tensor_chunk_bounds(N, n)
            assert bounds == chunk_rows(N, n)
            assert sum(c for _, c in bounds) == N
            for (s, c), r in zip(bounds, ref):
                assert torch.equal(x[s:s + c], r)
            # first N % n chunks hold one extra row
            assert [c for _, c in bounds] == [N // n + (1 if i < N % n else 0) for i in range(n)]


def test_product_matches_oracle_on_nested_arguments():
    g = torch.Generator().manual_seed(0)
    img = torch.randn(10, 3, 4, 4, generator=g)
    labels = torch.randint(0, 9, (10,), generator=g)
    args = (img, [labels, (img[:, 0], 3)], "tag", [1, 2, 3, 4, 5], 7, None)
    kwargs = {"mask": torch.ones(10, 5, dtype=torch.bool), "cfg": {"a": labels.float(), "b": [True, False]},
              "empty": []}
    for n in (1, 2, 3, 4, 7, 10, 12):
        a1, k1 = split_args_kwargs(args, kwargs, n)
        a2, k2 = oracle_split(args, kwargs, n)
        assert len(a1) == len(k1) == n
        assert same(a1, a2), n
        assert same(k1, k2), n
        # tensors are views of the caller's storage (no copy)
        assert a1[0][0].untyped_storage().data_ptr() == img.untyped_storage().data_ptr()
    a, k = split_args_kwargs(args, kwargs, 4)
    assert [x[0].shape[0] for x in a] == [3, 3, 2, 2]
    assert [x[3] for x in a] == [[1, 2], [3, 4], [5], []]  # ceil-sized list runs, trailing run empty
    assert all(x[2] == "tag" and x[4] == 7 and x[5] is None for x in a)
    assert torch.equal(torch.cat([x[1][0] for x in a]), labels)
    assert [kk["cfg"]["b"] for kk in k] == [[True], [False], [], []]


def test_none_arguments_and_ragged_edges():
    a, k = split_args_kwargs(None, None, 3)
    assert a == [(None,)] * 3 and k == [{}, {}, {}]
    assert same((a, k), oracle_split(None, None, 3))
    x = torch.arange(2)
    a, _ = split_args_kwargs((x,), {}, 4)  # fewer rows than chunks: empty trailing chunks
    assert [t[0].tolist() for t in a] == [[0], [1], [], []]
    assert same(a, oracle_split((x,), {}, 4)[0])
