"""Host logic on CPU for the Llama-style decoder (RMSNorm, rotary pattern match,
SwiGLU, causal attention, embedding, in-graph shifted cross entropy, an input
that feeds two stages), with the kernel oracle as the kernel table double."""
import copy

import pytest
import torch
import torch.nn.functional as F

from oracle.kernels_oracle import OracleKernels
from oracle.stage_oracle import run_pipeline_step
from pfeife_amd.bench_models.llama import LlamaConfig, LlamaForCausalLM, split_stages
from pfeife_amd.mp import net_states
from pfeife_amd.option import PipeOption

CFG = LlamaConfig(vocab=96, dim=64, layers=4, heads=4, ffn=88, max_seq=16)


def shifted_ce(logits, ids):
    return F.cross_entropy(logits[:, :-1, :].reshape(-1, logits.shape[-1]).float(), ids[:, 1:].reshape(-1))


def run(mixed, bounds, device_cnt, batch=8, batch_cnt=4, T=16):
    from pfeife_amd.mp import PartialRunner, initialize_pfeife, partial_compiler

    torch._dynamo.reset()
    net_states._reset_state_for_tests()
    initialize_pfeife(device="cpu")
    torch.manual_seed(0)
    model = LlamaForCausalLM(CFG)
    ref = copy.deepcopy(model)
    option = PipeOption(device_cnt=device_cnt, batch_cnt=batch_cnt, batch_size=batch // batch_cnt,
                        split_points=["layers.%d" % b for b in bounds], mixed_precision=mixed,
                        optimizer=dict(type="sgd", lr=0.0))
    runner = PartialRunner(option, kernels=OracleKernels("cpu"))
    cmodel = torch.compile(model, backend=partial_compiler)

    def fn(ids):
        loss = cmodel(ids, ids)
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    ids = torch.randint(0, CFG.vocab, (batch, T), generator=g)
    losses = runner.step(ids)
    adt = {"bf16": torch.bfloat16, "fp16": torch.float16}.get(mixed)
    want = run_pipeline_step(split_stages(ref, bounds), shifted_ce, ids, ids, batch_cnt, device_cnt=device_cnt,
                             loop_batch=option.loop_batch, autocast_dtype=adt)
    return model, ref, losses, want, runner


def test_fp32_four_stages_looped_schedule():
    model, ref, losses, want, runner = run(None, [1, 2, 3], device_cnt=2)
    assert len(runner.worker.part_graph.nodes) == 4
    # the token ids reach the first stage (embedding) and the last stage (labels)
    ids_slot = runner.worker.part_graph.placeholder_names.index("l_input_ids_")
    assert sorted(s for s, _ in runner.worker.part_graph.inputs[ids_slot]) == [0, 3]
    for a, b in zip(losses, want):
        assert abs(float(a) - float(b)) <= 1e-5 * abs(float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n
    # the nine-node rotary pattern is one kernel per q and k: a middle stage (one layer) runs
    # rmsnorm, q/k/v, 2 rope, 3 attention kernels, o_proj, rmsnorm, gate, up, glu, down
    assert len(runner.worker.mbs[0].stage_programs[1].fwd) == 15


@pytest.mark.parametrize("mixed,tol", [("bf16", 4e-2), ("fp16", 6e-3)])
def test_mixed_precision(mixed, tol):
    model, ref, losses, want, _ = run(mixed, [2], device_cnt=2)
    for a, b in zip(losses, want):
        assert abs(float(a) - float(b)) <= 2e-2 * abs(float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        rel = (p.grad - q.grad).norm() / (q.grad.norm() + 1e-12)
        assert rel <= tol, (n, float(rel))


def test_causal_attention_with_unequal_lengths_is_rejected():
    """F.scaled_dot_product_attention(is_causal=True) with Tq != Tk masks top-left; the kernels
    mask bottom-right, so the lowering must refuse instead of computing something else."""
    from pfeife_amd.executor.lowering import Unsupported
    from pfeife_amd.mp import PartialRunner, initialize_pfeife, partial_compiler

    class Cross(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.Linear(16, 16)
            self.b = torch.nn.Linear(16, 16)

        def forward(self, x, ctx):
            q = self.a(x).view(x.shape[0], -1, 2, 8).transpose(1, 2)
            k = self.a(ctx).view(ctx.shape[0], -1, 2, 8).transpose(1, 2)
            o = F.scaled_dot_product_attention(q, k, k, is_causal=True)
            return self.b(o.transpose(1, 2).reshape(x.shape[0], -1, 16))

    torch._dynamo.reset()
    net_states._reset_state_for_tests()
    initialize_pfeife(device="cpu")
    torch.manual_seed(0)
    model = Cross()
    option = PipeOption(device_cnt=2, batch_cnt=2, batch_size=2, split_points=["b"],
                        optimizer=dict(type="sgd", lr=0.0))
    runner = PartialRunner(option, kernels=OracleKernels("cpu"))
    cmodel = torch.compile(model, backend=partial_compiler)

    def fn(x, ctx):
        loss = cmodel(x, ctx).float().square().mean()
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    with pytest.raises(Exception) as err:
        runner.step(torch.randn(4, 4, 16), torch.randn(4, 6, 16))
    chain, e = [], err.value
    while e is not None:
        chain.append(e)
        e = e.__cause__ or e.__context__
    assert any(isinstance(c, Unsupported) and "is_causal" in str(c) for c in chain) or "is_causal" in str(err.value)
