"""Host logic of the executor on CPU: graph capture, stage partition, lowering to
launch programs, schedule-ordered job loop, micro-batch threads.  The kernel
table is replaced by the CPU oracle of the kernels (a test double injected
through PartialRunner's `kernels` argument; the product only ships the HIP
table), so these tests check everything EXCEPT the HIP code."""
import copy

import pytest
import torch
import torch.nn as nn

from oracle.kernels_oracle import OracleKernels
from oracle.stage_oracle import run_pipeline_step, run_unpipelined
from pfeife_amd.bench_models.vit import ViTConfig, VisionTransformer, split_stages
from pfeife_amd.mp import net_states
from pfeife_amd.option import PipeOption

CFG = ViTConfig(image_size=32, patch_size=16, dim=64, depth=4, heads=4, mlp_dim=128, num_classes=10)


def make_runner(option):
    from pfeife_amd.mp import PartialRunner, initialize_pfeife

    torch._dynamo.reset()
    net_states._reset_state_for_tests()
    initialize_pfeife(device="cpu")
    return PartialRunner(option, kernels=OracleKernels("cpu"))


def run_case(mixed, batch=8, batch_cnt=4, device_cnt=2, split=("blocks.2",), steps=1, lr=0.0, opt_type="sgd"):
    from pfeife_amd.mp import partial_compiler

    torch.manual_seed(0)
    model = VisionTransformer(CFG)
    ref = copy.deepcopy(model)
    option = PipeOption(device_cnt=device_cnt, batch_cnt=batch_cnt, batch_size=batch // batch_cnt,
                        split_points=list(split) if split else None, mixed_precision=mixed,
                        optimizer=dict(type=opt_type, lr=lr))
    runner = make_runner(option)
    cmodel = torch.compile(model, backend=partial_compiler)
    crit = nn.CrossEntropyLoss()

    def fn(x, y):
        loss = crit(cmodel(x).float(), y)
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    x = torch.randn(batch, 3, 32, 32, generator=g)
    y = torch.randint(0, 10, (batch,), generator=g)
    out = [runner.step(x, y) for _ in range(steps)]
    return model, ref, out, (x, y), runner, crit


def test_fp32_matches_reference_stage_semantics():
    model, ref, out, (x, y), runner, crit = run_case(None)
    want = run_pipeline_step(split_stages(ref, 2), crit, x, y, 4, device_cnt=2)
    for a, b in zip(out[0], want):
        assert abs(float(a) - float(b)) <= 1e-5 * abs(float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n
    # the job order is the serialised looped schedule: F00 F01 | F10 ... and ends with the last backward of stage 0
    order = runner.worker.order
    assert order[0] == (0, 0, True) and order[-1] == (0, 3, False)
    assert len(order) == 2 * 2 * 4


@pytest.mark.parametrize("mixed,tol", [("bf16", 3e-2), ("fp16", 5e-3)])
def test_mixed_precision_follows_autocast(mixed, tol):
    model, ref, out, (x, y), _, crit = run_case(mixed)
    adt = {"bf16": torch.bfloat16, "fp16": torch.float16}[mixed]
    want = run_unpipelined(ref, lambda o, t: crit(o.float(), t), x, y, 4, autocast_dtype=adt)
    for a, b in zip(out[0], want):
        assert abs(float(a) - float(b)) <= 2e-2 * abs(float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        rel = (p.grad - q.grad).norm() / (q.grad.norm() + 1e-12)
        assert rel <= tol, (n, float(rel))


def test_single_stage_ragged_batch_and_repeat():
    # 7 samples over 3 micro-batches -> 3, 2, 2 rows; same result on every repetition (lr = 0)
    model, ref, out, (x, y), runner, crit = run_case(None, batch=7, batch_cnt=3, device_cnt=1, split=None, steps=3)
    want = run_unpipelined(ref, crit, x, y, 3)
    assert [float(a) for a in out[0]] == [float(a) for a in out[2]]
    for a, b in zip(out[0], want):
        assert abs(float(a) - float(b)) <= 1e-5 * abs(float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n


def test_optimizer_step_updates_parameters_like_eager_training():
    model, ref, out, (x, y), runner, crit = run_case(None, steps=2, lr=0.05)
    opt = torch.optim.SGD(ref.parameters(), lr=0.05)
    ref_losses = []
    for _ in range(2):
        ref_losses.append(run_unpipelined(ref, crit, x, y, 4))
        opt.step()
    for a, b in zip(out[1], ref_losses[1]):
        assert abs(float(a) - float(b)) <= 1e-4 * abs(float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        torch.testing.assert_close(p.detach(), q.detach(), rtol=1e-4, atol=1e-6, msg=n)


def test_three_stages_integer_split_points_and_errors():
    from pfeife_amd.graph.partition_graph import compute_nodes, resolve_split_points
    from pfeife_amd.mp import partial_compiler

    model, ref, out, (x, y), runner, crit = run_case(None, split=("blocks.1", "blocks.3"), device_cnt=3, batch_cnt=4)
    want = run_unpipelined(ref, crit, x, y, 4)
    for a, b in zip(out[0], want):
        assert abs(float(a) - float(b)) <= 1e-5 * abs(float(b))
    pg = runner.worker.part_graph
    assert sorted(pg.nodes) == [0, 1, 2]
    # each cross-stage value appears once as a producer output and once per consumer input
    for sid, st in pg.nodes.items():
        for k, src in enumerate(st.input_source):
            if src is not None:
                assert sid in pg.nodes[src[0]].output_map[pg.nodes[src[0]].outputs[src[1]]]
    assert pg.outputs == [(2, 0)]
    with pytest.raises(RuntimeError, match="matches no module path"):
        resolve_split_points(pg.nodes[0].graph_module, ["nonexistent.9"])


def test_unsupported_node_fails_loudly():
    from pfeife_amd.executor.lowering import Unsupported
    from pfeife_amd.mp import partial_compiler

    class Odd(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(8, 8)

        def forward(self, x):
            return torch.cumsum(self.fc(x), dim=1)

    option = PipeOption(device_cnt=1, batch_cnt=1, batch_size=2)
    runner = make_runner(option)
    m = torch.compile(Odd(), backend=partial_compiler)
    runner.set_exec_fn(lambda x: m(x).sum())
    with pytest.raises(Exception) as ei:
        runner.step(torch.randn(2, 8))
    assert "no HIP lowering" in str(ei.value) or isinstance(ei.value, Unsupported)


def test_static_loss_scale_is_applied_once_and_removed():
    """option.loss_scale multiplies the gradients entering the last stage and is divided out
    before the optimizer step: final gradients equal the unscaled ones (powers of two: exactly)."""
    from pfeife_amd.mp import partial_compiler

    grads = []
    for scale in (1.0, 1024.0):
        torch.manual_seed(0)
        model = VisionTransformer(CFG)
        option = PipeOption(device_cnt=2, batch_cnt=2, batch_size=2, split_points=["blocks.2"],
                            optimizer=dict(type="sgd", lr=0.0), loss_scale=scale)
        runner = make_runner(option)
        cmodel = torch.compile(model, backend=partial_compiler)
        crit = nn.CrossEntropyLoss()

        def fn(x, y):
            loss = crit(cmodel(x).float(), y)
            loss.backward()
            return loss.detach()

        runner.set_exec_fn(fn)
        g = torch.Generator().manual_seed(42)
        runner.step(torch.randn(4, 3, 32, 32, generator=g), torch.randint(0, 10, (4,), generator=g))
        grads.append({n: p.grad.clone() for n, p in model.named_parameters()})
    for n in grads[0]:
        assert torch.equal(grads[0][n], grads[1][n]), n


def test_scaler_rule_of_the_kernel_oracle_matches_torch_gradscaler():
    """scaler_unscale / scaler_update of the kernel oracle against torch.amp.GradScaler on the CPU,
    over a sequence with overflows and growth."""
    from oracle.kernels_oracle import OracleKernels

    k = OracleKernels("cpu")
    ref = torch.amp.GradScaler("cpu", init_scale=1024.0, growth_factor=2.0, backoff_factor=0.5, growth_interval=3)
    state = torch.tensor([1024.0, 0.0, 0.0, 0.0])
    p = torch.nn.Parameter(torch.zeros(4))
    opt = torch.optim.SGD([p], lr=1.0)
    done = 0
    for step, bad in enumerate([False, False, True, False, False, False, True, True, False, False, False, False]):
        ref.scale(torch.zeros(1))          # GradScaler creates its scale tensor on first use
        g = torch.tensor([1.0, -2.0, 0.5, 4.0]) * float(ref.get_scale())
        if bad:
            g[1] = float("inf")
        p.grad = g.clone()
        before = p.detach().clone()
        ref.step(opt)
        ref.update()
        mine = g.clone()
        k.scaler_unscale(mine, 4, state)(None)
        assert float(state[2]) == (1.0 if bad else 0.0)
        if not bad:
            assert torch.equal(mine, torch.tensor([1.0, -2.0, 0.5, 4.0]))
            done += 1
        assert torch.equal(p.detach(), before) == bad   # torch skipped exactly the overflowing steps
        k.scaler_update(state, 2.0, 0.5, 3)(None)
        assert float(state[0]) == float(ref.get_scale()), (step, float(state[0]), float(ref.get_scale()))
        assert float(state[3]) == done and float(state[2]) == 0.0


def test_dynamic_loss_scale_skips_overflowing_steps():
    """PipeOption(loss_scale="dynamic"): gradients leave the step unscaled, a step whose gradients
    overflow changes no parameter and halves the scale, clean steps grow it every growth_interval."""
    from pfeife_amd.mp import partial_compiler

    torch.manual_seed(0)
    model = VisionTransformer(CFG)
    ref = copy.deepcopy(model)
    option = PipeOption(device_cnt=2, batch_cnt=2, batch_size=2, split_points=["blocks.2"],
                        optimizer=dict(type="sgd", lr=0.1), loss_scale="dynamic", init_scale=256.0,
                        growth_interval=2)
    runner = make_runner(option)
    cmodel = torch.compile(model, backend=partial_compiler)
    crit = nn.CrossEntropyLoss()
    poison = [False]

    def fn(x, y):
        loss = crit(cmodel(x).float(), y)
        (loss * float("inf") if poison[0] else loss).backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    x, y = torch.randn(4, 3, 32, 32, generator=g), torch.randint(0, 10, (4,), generator=g)
    w = runner.worker
    assert w.scaler_scale() == 256.0
    runner.step(x, y)                                   # clean step 1
    # same step without scaling on the reference copy: identical gradients (power-of-two scale)
    ropt = torch.optim.SGD(ref.parameters(), lr=0.1)
    for xs, ys in zip(x.chunk(2), y.chunk(2)):
        crit(ref(xs), ys).backward()
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n
    ropt.step()
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.detach() - q.detach()).abs().max() <= 1e-5 * q.detach().abs().max() + 1e-7, n
    assert w.scaler_scale() == 256.0
    poison[0] = True
    before = {n: p.detach().clone() for n, p in model.named_parameters()}
    runner.step(x, y)                                   # overflow: skipped, scale halves
    for n, p in model.named_parameters():
        assert torch.equal(p.detach(), before[n]), n
    assert w.scaler_scale() == 128.0
    poison[0] = False
    runner.step(x, y)
    runner.step(x, y)                                   # two clean steps: scale doubles
    assert w.scaler_scale() == 256.0
    assert float(w.scaler_state[3]) == 3.0
    # the scaler's state travels in torch.amp.GradScaler's layout and loads back
    saved = runner.scaler_state_dict()
    assert saved == {"scale": 256.0, "growth_factor": 2.0, "backoff_factor": 0.5, "growth_interval": 2,
                     "_growth_tracker": 0}
    ref_scaler = torch.amp.GradScaler("cpu")
    ref_scaler.load_state_dict(saved)                   # torch accepts it as its own
    assert ref_scaler.get_growth_interval() == 2
    runner.step(x, y)                                   # one clean step: tracker 1
    assert runner.scaler_state_dict()["_growth_tracker"] == 1
    runner.load_scaler_state_dict(dict(saved, scale=64.0))
    assert w.scaler_scale() == 64.0 and runner.scaler_state_dict()["_growth_tracker"] == 0


def test_bf16_step_with_non_finite_gradients_is_skipped():
    """bf16 mixed precision runs the dynamic scaler by default, as the reference's GradScaler does
    for every mixed precision (pfeife/mp/worker.py:135): a step whose gradients are not finite
    changes no parameter and halves the scale; the next clean step is applied."""
    from pfeife_amd.mp import partial_compiler

    torch.manual_seed(0)
    model = VisionTransformer(CFG)
    option = PipeOption(device_cnt=2, batch_cnt=2, batch_size=2, split_points=["blocks.2"], mixed_precision="bf16",
                        optimizer=dict(type="sgd", lr=0.1))
    assert option.loss_scale == "dynamic"
    runner = make_runner(option)
    cmodel = torch.compile(model, backend=partial_compiler)
    crit = nn.CrossEntropyLoss()
    poison = [True]

    def fn(x, y):
        loss = crit(cmodel(x).float(), y)
        (loss * float("inf") if poison[0] else loss).backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    x, y = torch.randn(4, 3, 32, 32, generator=g), torch.randint(0, 10, (4,), generator=g)
    before = {n: p.detach().clone() for n, p in model.named_parameters()}
    runner.step(x, y)
    w = runner.worker
    assert w.dyn_scale and w.scaler_scale() == 32768.0 and float(w.scaler_state[3]) == 0.0
    for n, p in model.named_parameters():
        assert torch.equal(p.detach(), before[n]), n
    poison[0] = False
    runner.step(x, y)
    assert float(w.scaler_state[3]) == 1.0 and w.scaler_scale() == 32768.0
    assert any(not torch.equal(p.detach(), before[n]) for n, p in model.named_parameters())
    assert all(torch.isfinite(p.grad).all() for p in model.parameters())


def test_static_loss_scale_has_no_scaler_state():
    runner = make_runner(PipeOption(device_cnt=1, batch_cnt=1, batch_size=2))
    assert runner.scaler_state_dict() == {}
    runner.load_scaler_state_dict({})
    with pytest.raises(RuntimeError, match="static loss scale"):
        runner.load_scaler_state_dict({"scale": 2.0})


def test_failed_step_releases_parked_micro_batches():
    """exec_fn raising for a later micro-batch (or after the model returned) must not leave the
    earlier micro-batch threads parked: the error reaches the caller and the next step() runs."""
    from pfeife_amd.mp import partial_compiler

    torch.manual_seed(0)
    model = VisionTransformer(CFG)
    option = PipeOption(device_cnt=2, batch_cnt=2, batch_size=2, split_points=["blocks.2"],
                        optimizer=dict(type="sgd", lr=0.0))
    runner = make_runner(option)
    cmodel = torch.compile(model, backend=partial_compiler)
    crit = nn.CrossEntropyLoss()
    fail = [None]

    def fn(x, y):
        if fail[0] == "before" and float(y[0]) < 0:
            raise ValueError("bad labels")
        loss = crit(cmodel(x).float(), y.abs())
        if fail[0] == "after" and float(y[0]) < 0:
            raise ValueError("bad loss")
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    x, y = torch.randn(4, 3, 32, 32, generator=g), torch.randint(1, 10, (4,), generator=g)
    good = [float(v) for v in runner.step(x, y)]
    ybad = y.clone()
    ybad[2] = -ybad[2]                        # first sample of micro-batch 1
    for mode in ("before", "after"):
        fail[0] = mode
        with pytest.raises(ValueError):
            runner.step(x, ybad)
        fail[0] = None
        again = [float(v) for v in runner.step(x, y)]
        assert again == good, mode


def test_print_graph_lists_stages_and_edges(capsys):
    """print_graph=True prints the stage summary in the reference's layout (pfeife/graph/pipe_graph.py:145-154):
    a header, one line per stage, one per stage-to-stage edge with the boundary shapes and bytes."""
    from pfeife_amd.mp import partial_compiler

    torch.manual_seed(0)
    model = VisionTransformer(CFG)
    option = PipeOption(device_cnt=2, batch_cnt=2, batch_size=2, split_points=["blocks.1", "blocks.2", "blocks.3"],
                        optimizer=dict(type="sgd", lr=0.0), print_graph=True)
    runner = make_runner(option)
    cmodel = torch.compile(model, backend=partial_compiler)
    crit = nn.CrossEntropyLoss()

    def fn(x, y):
        loss = crit(cmodel(x).float(), y)
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    runner.step(torch.randn(4, 3, 32, 32, generator=g), torch.randint(0, 10, (4,), generator=g))
    out = capsys.readouterr().out
    assert "GRAPH: 4 nodes / 3 edges" in out
    assert "==== nodes ====" in out and "==== edges ====" in out
    pg = runner.worker.part_graph
    for idx in range(4):
        assert "Node [%d/%d] (weight: " % (idx, idx % 2) in out
    # micro-batch 2 x (4 patches + cls) x dim floats cross every boundary
    tokens = (CFG.image_size // CFG.patch_size) ** 2 + 1
    edges = pg.edges()
    assert [(a, b) for a, b, _, _ in edges] == [(0, 1), (1, 2), (2, 3)]
    for a, b, w, vals in edges:
        assert w == 2 * tokens * CFG.dim * 4 and vals[0][1] == (2, tokens, CFG.dim)
        assert "Edge (%d -> %d) (weight: " % (a, b) in out
    # the parameters are split over the stages without overlap
    total = sum(pg.stage_summary(i)["weight"] for i in range(4))
    assert total == sum(p.numel() * 4 for p in model.parameters())


def test_weights_tied_across_two_stages_accumulate_both_contributions():
    """An embedding table that is also the output projection (first and last stage, different pipeline
    ranks): its gradient is the sum of both stages' contributions over all micro-batches."""
    import copy

    from oracle.kernels_oracle import OracleKernels
    from pfeife_amd.bench_models.llama import LlamaConfig, LlamaForCausalLM
    from pfeife_amd.mp import PartialRunner, initialize_pfeife, net_states, partial_compiler
    from pfeife_amd.option import PipeOption

    cfg = LlamaConfig(vocab=256, dim=64, layers=4, heads=4, ffn=176, max_seq=32)
    torch.manual_seed(0)
    model = LlamaForCausalLM(cfg)
    model.lm_head.weight = model.embed.weight
    ref = copy.deepcopy(model)
    assert ref.lm_head.weight is ref.embed.weight
    torch._dynamo.reset()
    net_states._reset_state_for_tests()
    initialize_pfeife(device="cpu")
    option = PipeOption(device_cnt=2, batch_cnt=4, batch_size=2, split_points=["layers.2"],
                        optimizer=dict(type="sgd", lr=0.0))
    runner = PartialRunner(option, kernels=OracleKernels("cpu"))
    cmodel = torch.compile(model, backend=partial_compiler)

    def fn(tok):
        loss = cmodel(tok, tok)
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    ids = torch.randint(0, cfg.vocab, (8, 32), generator=torch.Generator().manual_seed(1))
    losses = runner.step(ids)
    for chunk, got in zip(ids.chunk(4), losses):
        want = ref(chunk, chunk)
        want.backward()
        assert abs(float(got) - float(want.detach())) <= 1e-5 * abs(float(want.detach()))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n


def test_weight_gradients_run_once_per_step_over_all_micro_batches(monkeypatch):
    """Equal micro-batches: every linear layer's weight gradient is ONE product whose reduction runs
    over the rows of all micro-batches (their activations and output gradients lie end to end in
    stacked buffers), issued after the stage's last backward job.  A ragged batch and PFEIFE_DW_STACK=0
    keep one product per micro-batch inside the backward jobs.  All three
    give the gradients of plain accumulation (checked by the callers' own comparisons above)."""
    model, ref, out, (x, y), runner, crit = run_case(None, steps=2)   # 8 samples in 4 micro-batches, 2 stages
    w = runner.worker
    assert sorted(w.dw_jobs) == [0, 1] and w.last_backward == {0: 3, 1: 3}
    # the linear layers' weight gradients are STORED by their one product (no zero fill, no unscale pass
    # over them: the second step above must not add to the first), every other gradient accumulates
    whole = [n for n, p in model.named_parameters() if w.params.stored_whole(p)]
    assert len(whole) == 8 + 9 and all(n.endswith("weight") for n in whole), whole
    swept = sum(n for _, n in w.params.grad_buffers())               # what the unscale pass walks (padded to 64)
    rest = sum(p.numel() for n, p in model.named_parameters() if n not in whole)
    assert rest <= swept < rest + 64 * len(list(model.parameters()))
    tokens = (CFG.image_size // CFG.patch_size) ** 2 + 1
    per_stage = {sid: len(w.mbs[0].stage_programs[sid].dw_deferred) for sid in (0, 1)}
    assert per_stage[0] >= 8 and per_stage[1] >= 8                    # four linear layers per block, two blocks each
    for sid, (launches, _) in w.dw_jobs.items():
        kinds = [l.__qualname__.split(".")[1] for l in launches]
        assert kinds.count("gemm") == per_stage[sid]                     # one product per layer, not per micro-batch
        # ... and one column sum per layer for its bias, over the same stacked rows, finished together
        assert kinds.count("colsum_accumulate") == per_stage[sid] and kinds.count("colreduce_finalize_batch") == 1
    # the block layers reduce over 4 micro-batches x 2 samples x tokens rows
    ks = sorted({int(r["rows"]) for r in w.mbs[0].stage_programs[0].dw_deferred})
    assert 2 * tokens in ks
    run_pipeline_step(split_stages(ref, 2), crit, x, y, 4, device_cnt=2)
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n
    # ragged: 7 samples over 3 micro-batches: nothing is stacked or deferred (no buffer is kept twice)
    model, ref, out, (x, y), runner, crit = run_case(None, batch=7, batch_cnt=3, device_cnt=1, split=None)
    w = runner.worker
    assert not any(p.dw_deferred for slot in w.mbs.values() for p in slot.stage_programs.values())
    assert all(not launches for launches, _ in w.dw_jobs.values())
    # switched off: nothing is deferred
    monkeypatch.setenv("PFEIFE_DW_STACK", "0")
    model, ref, out, (x, y), runner, crit = run_case(None)
    assert runner.worker.dw_jobs == {} and not runner.worker.mbs[0].stage_programs[0].dw_deferred
    run_unpipelined(ref, crit, x, y, 4)
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n


def test_ragged_step_after_uniform_steps_starts_from_zeroed_gradients():
    """Uniform steps store the linear weights' gradients from one product per step (no zero fill over
    them).  A later step whose micro-batches differ (7 samples over 3: 3, 2, 2) rebuilds only the slot
    whose shape changed, without the deferral: from then on those gradients are accumulated again, and
    the very step in which that happens must already start from zero, not from the previous step's
    stored values."""
    from pfeife_amd.mp import partial_compiler

    torch.manual_seed(0)
    model = VisionTransformer(CFG)
    ref = copy.deepcopy(model)
    option = PipeOption(device_cnt=1, batch_cnt=3, batch_size=2, split_points=None, optimizer=dict(type="sgd", lr=0.0))
    runner = make_runner(option)
    cmodel = torch.compile(model, backend=partial_compiler, dynamic=False)
    crit = nn.CrossEntropyLoss()

    def fn(x, y):
        loss = crit(cmodel(x).float(), y)
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    x6, y6 = torch.randn(6, 3, 32, 32, generator=g), torch.randint(0, 10, (6,), generator=g)
    x7, y7 = torch.randn(7, 3, 32, 32, generator=g), torch.randint(0, 10, (7,), generator=g)
    runner.step(x6, y6)
    runner.step(x6, y6)
    w = runner.worker
    assert any(w.params.stored_whole(p) for p in model.parameters())
    runner.step(x7, y7)
    assert not any(w.params.stored_whole(p) for p in model.parameters())
    run_unpipelined(ref, crit, x7, y7, 3)
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n
    runner.step(x6, y6)          # and back: every slot has its uniform shape again
    for q in ref.parameters():
        q.grad = None
    run_unpipelined(ref, crit, x6, y6, 3)
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-9, n
