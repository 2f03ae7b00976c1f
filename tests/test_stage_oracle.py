"""Pins oracle/stage_oracle.py: the restated stage execution of the reference
(clone-in, copy_ handoff, autograd.backward per stage, AccumulateGrad) must be
the same computation as plain gradient accumulation on the un-partitioned model:
in fp32 on CPU losses and accumulated gradients are bit-identical, for every
schedule shape."""
import copy

import pytest
import torch
import torch.nn as nn

from oracle.stage_oracle import merge_rank_works, run_pipeline_step, run_unpipelined
from oracle.schedule_oracle import rank_works
from pfeife_amd.bench_models.vit import ViTConfig, VisionTransformer, split_stages

CFG = ViTConfig(image_size=32, patch_size=16, dim=48, depth=4, heads=4, mlp_dim=96, num_classes=7)


def _data(n, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, 3, 32, 32, generator=g), torch.randint(0, 7, (n,), generator=g)


@pytest.mark.parametrize("batch_cnt,device_cnt,n", [(4, 2, 8), (4, 1, 8), (3, 2, 7), (1, 1, 2), (6, 2, 6)])
def test_pipelined_equals_unpipelined_bit_exact(batch_cnt, device_cnt, n):
    torch.manual_seed(1)
    model = VisionTransformer(CFG)
    ref = copy.deepcopy(model)
    x, y = _data(n)
    crit = nn.CrossEntropyLoss()
    losses = run_pipeline_step(split_stages(model, 2), crit, x, y, batch_cnt, device_cnt=device_cnt)
    want = run_unpipelined(ref, crit, x, y, batch_cnt)
    assert len(losses) == batch_cnt
    for a, b in zip(losses, want):
        assert torch.equal(a, b)
    for (name, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert torch.equal(p.grad, q.grad), name


def test_loss_is_sum_of_micro_batch_means_not_divided():
    """The reference sums per-micro-batch mean losses and never divides by batch_cnt
    (bench_models/models/train_vit.py:64-65): gradients are batch_cnt x the full-batch-mean gradient."""
    torch.manual_seed(2)
    model = VisionTransformer(CFG)
    ref = copy.deepcopy(model)
    x, y = _data(8)
    crit = nn.CrossEntropyLoss()
    run_pipeline_step(split_stages(model, 2), crit, x, y, 4)
    for p in ref.parameters():
        p.grad = None
    crit(ref(x), y).backward()
    for (name, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        torch.testing.assert_close(p.grad, 4 * q.grad, rtol=2e-4, atol=1e-6, msg=name)


def test_scaler_compounds_per_stage():
    """GradScaler.scale is applied to every stage's outputs (pfeife/mp/worker.py:1580):
    with scale S the gradients of stage i of L are S^(L-i) times the true ones."""
    torch.manual_seed(3)
    model = VisionTransformer(CFG)
    ref = copy.deepcopy(model)
    x, y = _data(4)
    crit = nn.CrossEntropyLoss()
    S = 16.0
    run_pipeline_step(split_stages(model, 2), crit, x, y, 2, loss_scale=S)
    run_pipeline_step(split_stages(ref, 2), crit, x, y, 2, loss_scale=1.0)
    first = {id(p) for n, p in model.named_parameters()
             if n.startswith(("patch_embed", "cls_token", "pos_embed", "blocks.0", "blocks.1"))}
    for (name, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        factor = S * S if id(p) in first else S
        torch.testing.assert_close(p.grad, factor * q.grad, rtol=1e-5, atol=0, msg=name)


def test_merge_respects_rank_order_and_dependencies():
    works = rank_works(2, 8, 4, 2, 0)
    order = merge_rank_works(works, 4)
    pos = {j: i for i, j in enumerate(order)}
    for w in works:
        assert [pos[j] for j in w] == sorted(pos[j] for j in w)
    for n in range(4):
        for b in range(8):
            assert pos[(n, b, True)] < pos[(n, b, False)]
            if n:
                assert pos[(n - 1, b, True)] < pos[(n, b, True)] and pos[(n, b, False)] < pos[(n - 1, b, False)]
