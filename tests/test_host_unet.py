"""Host logic on CPU for the SDXL-style UNet stage (GroupNorm, 3x3 / 1x1 convolutions as
channels-last GEMMs, per-sample time-embedding add, cross attention to 77 context
tokens, GEGLU, MSE loss in user code), with the kernel oracle as the kernel table double."""
import copy

import pytest
import torch
import torch.nn.functional as F

from oracle.kernels_oracle import OracleKernels
from oracle.stage_oracle import run_unpipelined
from pfeife_amd.bench_models.unet_stage import UNetStage, UNetStageConfig
from pfeife_amd.mp import net_states
from pfeife_amd.option import PipeOption

CFG = UNetStageConfig(in_channels=32, channels=64, temb_dim=48, context_dim=40, heads=2, layers=1, groups=8)


class Wrapped(torch.nn.Module):
    """run_unpipelined feeds one tensor: pack (hidden, temb, context) along one batch-major tuple."""

    def __init__(self, m, temb, ctx):
        super().__init__()
        self.m, self.temb, self.ctx = m, temb, ctx


def run(mixed, batch=4, batch_cnt=2, hw=8):
    from pfeife_amd.mp import PartialRunner, initialize_pfeife, partial_compiler

    torch._dynamo.reset()
    net_states._reset_state_for_tests()
    initialize_pfeife(device="cpu")
    torch.manual_seed(0)
    model = UNetStage(CFG)
    ref = copy.deepcopy(model)
    option = PipeOption(device_cnt=1, batch_cnt=batch_cnt, batch_size=batch // batch_cnt, mixed_precision=mixed,
                        optimizer=dict(type="sgd", lr=0.0))
    runner = PartialRunner(option, kernels=OracleKernels("cpu"))
    cmodel = torch.compile(model, backend=partial_compiler)

    def fn(hidden, temb, ctx, target):
        out = cmodel(hidden, temb, ctx)
        loss = F.mse_loss(out.float(), target.float())
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    hidden = torch.randn(batch, CFG.in_channels, hw, hw, generator=g)
    temb = torch.randn(batch, CFG.temb_dim, generator=g)
    ctx = torch.randn(batch, 7, CFG.context_dim, generator=g)
    target = torch.randn(batch, CFG.channels, hw, hw, generator=g)
    losses = runner.step(hidden, temb, ctx, target)
    # plain gradient accumulation on the un-partitioned model (the stage oracle's pinned equivalent)
    adt = {"bf16": torch.bfloat16, "fp16": torch.float16}.get(mixed)
    for p in ref.parameters():
        p.grad = torch.zeros_like(p)
    want = []
    per = batch // batch_cnt
    for i in range(batch_cnt):
        sl = slice(i * per, (i + 1) * per)
        if adt is None:
            out = ref(hidden[sl], temb[sl], ctx[sl])
        else:
            with torch.autocast("cpu", dtype=adt):
                out = ref(hidden[sl], temb[sl], ctx[sl])
        loss = F.mse_loss(out.float(), target[sl].float())
        loss.backward()
        want.append(loss.detach())
    return model, ref, losses, want


def test_fp32():
    model, ref, losses, want = run(None)
    for a, b in zip(losses, want):
        assert abs(float(a) - float(b)) <= 1e-5 * abs(float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n


def test_bf16():
    model, ref, losses, want = run("bf16")
    for a, b in zip(losses, want):
        assert abs(float(a) - float(b)) <= 2e-2 * abs(float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        rel = (p.grad - q.grad).norm() / (q.grad.norm() + 1e-12)
        assert rel <= 5e-2, (n, float(rel))
