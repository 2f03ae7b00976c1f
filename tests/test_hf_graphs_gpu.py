"""The reference scripts' own model graph forms on the HIP path: Hugging Face
`ViTForImageClassification` (bench_models/models/train_vit.py:150-169) and `LlamaForCausalLM` with
`attn_implementation="eager"` (bench_models/models/train_llama.py:486-520), built from configs,
one optimisation step under mixed precision against plain PyTorch autocast on the same GPU
(losses within 2e-2 relative, every parameter's gradient within 2.5e-2 relative L2)."""
import copy
import gc

import pytest
import torch

pytestmark = pytest.mark.gpu
transformers = pytest.importorskip("transformers")


def _fresh_runner(option):
    from pfeife_amd.mp import PartialRunner, initialize_pfeife
    from pfeife_amd.mp import net_states

    from pfeife_amd.mp.partial.module import PartialModule

    # the previous test's programs (tens of GB of preallocated buffers at the full-size
    # configurations) stay reachable through the compiled modules until they are released
    old = PartialModule._runner
    if old is not None and getattr(old, "worker", None) is not None:
        old.worker.release()
        old.exec_fn = None
    PartialModule._runner = None
    torch._dynamo.reset()
    gc.collect()
    torch.cuda.empty_cache()
    net_states._reset_state_for_tests()
    initialize_pfeife()
    return PartialRunner(option)


def _check(model, ref, losses, want, mixed):
    ltol = 1e-5 if mixed is None else 2e-2
    for a, b in zip(losses, want):
        assert abs(float(a) - float(b)) <= ltol * abs(float(b)), (float(a), float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        gp, gq = p.grad.float(), q.grad.float()
        assert torch.isfinite(gp).all(), n
        if n.endswith("k_proj.bias"):
            # zero by construction (softmax is invariant to a shift of every score of a row, which is
            # all a key bias does): both sides hold rounding noise only
            assert float(gp.abs().max()) <= 1e-2 * max(float(x.grad.abs().max()) for x in ref.parameters()), n
            continue
        if mixed is None:
            assert (gp - gq).abs().max() <= 1e-4 * gq.abs().max() + 1e-7, (n, float((gp - gq).abs().max()))
        else:
            rel = float((gp - gq).norm() / (gq.norm() + 1e-20))
            assert rel <= 2.5e-2, (n, rel)


@pytest.mark.parametrize("mixed,attn", [(None, "eager"), ("fp16", "eager"), ("bf16", "sdpa")])
def test_hf_vit_on_device(mixed, attn):
    from pfeife_amd.mp import partial_compiler
    from pfeife_amd.option import PipeOption

    cfg = transformers.ViTConfig(hidden_size=256, image_size=64, intermediate_size=512, num_attention_heads=4,
                                 qkv_bias=True, num_labels=16, num_channels=3, num_hidden_layers=4, patch_size=16,
                                 hidden_act="gelu")
    cfg._attn_implementation = attn
    torch.manual_seed(0)
    model = transformers.ViTForImageClassification(cfg)
    ref = copy.deepcopy(model).cuda()
    option = PipeOption(device_cnt=2, batch_cnt=4, batch_size=4, split_points=["vit.layers.2"], mixed_precision=mixed,
                        loss_scale=(256.0 if mixed == "fp16" else 1.0), optimizer=dict(type="sgd", lr=0.0))
    runner = _fresh_runner(option)
    model.cuda()
    cmodel = torch.compile(model, backend=partial_compiler)
    crit = torch.nn.CrossEntropyLoss()

    def fn(px, labels):
        loss = crit(cmodel(px).logits.float(), labels)
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    x = torch.randn(16, 3, 64, 64, generator=g).cuda()
    y = torch.randint(0, 16, (16,), generator=g).cuda()
    losses = runner.step(x, y)
    torch.cuda.synchronize()
    dt = {"fp16": torch.float16, "bf16": torch.bfloat16}.get(mixed)
    want = []
    for xs, ys in zip(x.chunk(4), y.chunk(4)):
        with torch.autocast("cuda", dtype=dt, enabled=dt is not None):
            loss = crit(ref(xs).logits.float(), ys)
        loss.backward()
        want.append(loss.detach())
    _check(model, ref, losses, want, mixed)


@pytest.mark.parametrize("mixed", [None, "bf16"])
def test_hf_llama_eager_on_device(mixed):
    from pfeife_amd.mp import partial_compiler
    from pfeife_amd.option import PipeOption

    cfg = transformers.LlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=688, num_attention_heads=4,
                                   num_key_value_heads=4, num_hidden_layers=4, max_position_embeddings=128,
                                   pad_token_id=0, bos_token_id=1, eos_token_id=2, use_cache=False)
    torch.manual_seed(0)
    model = transformers.AutoModelForCausalLM.from_config(cfg, attn_implementation="eager")
    ref = copy.deepcopy(model).cuda()
    option = PipeOption(device_cnt=2, batch_cnt=4, batch_size=2,
                        split_points=["model.layers.1", "model.layers.2", "model.layers.3"], mixed_precision=mixed,
                        optimizer=dict(type="sgd", lr=0.0))
    runner = _fresh_runner(option)
    model.cuda()
    cmodel = torch.compile(model, backend=partial_compiler)

    def fn(ids):
        loss = cmodel(input_ids=ids, labels=ids).loss
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    ids = torch.randint(3, 512, (8, 128), generator=torch.Generator().manual_seed(42)).cuda()
    losses = runner.step(ids)
    torch.cuda.synchronize()
    assert len(runner.worker.part_graph.nodes) == 4
    dt = {"bf16": torch.bfloat16}.get(mixed)
    want = []
    for chunk in ids.chunk(4):
        with torch.autocast("cuda", dtype=dt, enabled=dt is not None):
            loss = ref(input_ids=chunk, labels=chunk).loss
        loss.backward()
        want.append(loss.detach())
    _check(model, ref, losses, want, mixed)
    kernels = [getattr(l, "kernel", "") for slot in runner.worker.mbs.values() for prog in slot.stage_programs.values()
               for l in prog.fwd]
    assert kernels.count("pf_rmsnorm_fwd") == (2 * 4 + 1) * 4 and kernels.count("pf_rope") == 2 * 4 * 4
