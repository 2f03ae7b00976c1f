"""The model graph forms the reference's own scripts feed to the pipeline: Hugging Face
`ViTForImageClassification` (bench_models/models/train_vit.py:150-169) and `LlamaForCausalLM`
built from a config with `attn_implementation="eager"` (bench_models/models/train_llama.py:486-520:
attention as matmul + mask add + softmax + matmul, rotary embedding and RMSNorm spelled out in
elementwise operations, the shifted next-token loss inside the graph).

Host test: the graphs are captured by TorchDynamo, canonicalised, partitioned and lowered with the
kernel oracle as the kernel table double, and one optimisation step is compared with plain
gradient accumulation on the same module (fp32: losses to 1e-5, gradients to 1e-4 of their
maximum).  Needs `transformers` (present where the suite is developed; skipped elsewhere)."""
import copy

import pytest
import torch

transformers = pytest.importorskip("transformers")

from oracle.kernels_oracle import OracleKernels  # noqa: E402
from pfeife_amd.mp import net_states  # noqa: E402
from pfeife_amd.option import PipeOption  # noqa: E402


def _runner(option):
    from pfeife_amd.mp import PartialRunner, initialize_pfeife

    torch._dynamo.reset()
    net_states._reset_state_for_tests()
    initialize_pfeife(device="cpu")
    return PartialRunner(option, kernels=OracleKernels("cpu"))


def _check(model, ref, losses, want):
    for a, b in zip(losses, want):
        assert abs(float(a) - float(b)) <= 1e-5 * abs(float(b)), (float(a), float(b))
    for (n, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert p.grad is not None and q.grad is not None, n
        # (the key projection's bias has an exactly-zero true gradient, softmax being shift invariant:
        # both sides hold rounding noise of ~1e-9 there, hence the absolute floor)
        assert (p.grad - q.grad).abs().max() <= 1e-4 * q.grad.abs().max() + 1e-7, (n, float((p.grad - q.grad).abs().max()))


def _forward_kernels(runner):
    """Names of the kernel-table entries the forward launch lists call (the kernel double's
    launches are closures of the method that made them)."""
    out = []
    for slot in runner.worker.mbs.values():
        for prog in slot.stage_programs.values():
            for launch in prog.fwd:
                out.append(getattr(launch, "kernel", None) or "pf_" + launch.__qualname__.split(".")[1])
    return out


@pytest.mark.parametrize("attn", ["eager", "sdpa"])
def test_hf_vit_for_image_classification(attn):
    from pfeife_amd.mp import partial_compiler

    cfg = transformers.ViTConfig(hidden_size=64, image_size=32, intermediate_size=128, num_attention_heads=4,
                                 qkv_bias=True, num_labels=10, num_channels=3, num_hidden_layers=4, patch_size=16,
                                 hidden_act="gelu")
    cfg._attn_implementation = attn
    torch.manual_seed(0)
    model = transformers.ViTForImageClassification(cfg)
    ref = copy.deepcopy(model)
    option = PipeOption(device_cnt=2, batch_cnt=4, batch_size=2, split_points=["vit.layers.2"],
                        optimizer=dict(type="sgd", lr=0.0))
    runner = _runner(option)
    cmodel = torch.compile(model, backend=partial_compiler)
    crit = torch.nn.CrossEntropyLoss()

    def fn(px, labels):
        loss = crit(cmodel(px).logits, labels)      # the model returns an ImageClassifierOutput
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    g = torch.Generator().manual_seed(42)
    x = torch.randn(8, 3, 32, 32, generator=g)
    y = torch.randint(0, 10, (8,), generator=g)
    losses = runner.step(x, y)
    assert len(runner.worker.part_graph.nodes) == 2
    want = []
    for xs, ys in zip(x.chunk(4), y.chunk(4)):
        loss = crit(ref(xs).logits, ys)
        loss.backward()
        want.append(loss.detach())
    _check(model, ref, losses, want)
    # attention ran as the attention operation, not as loose matrix products with a softmax between
    kernels = _forward_kernels(runner)
    assert kernels.count("pf_softmax_fwd") + kernels.count("pf_attention_fwd") == 4 * 4   # layers x micro-batches


def test_hf_llama_eager_attention_four_stages_looped():
    from pfeife_amd.mp import partial_compiler

    cfg = transformers.LlamaConfig(vocab_size=256, hidden_size=64, intermediate_size=176, num_attention_heads=4,
                                   num_key_value_heads=4, num_hidden_layers=4, max_position_embeddings=64,
                                   pad_token_id=0, bos_token_id=1, eos_token_id=2, use_cache=False)
    torch.manual_seed(0)
    model = transformers.AutoModelForCausalLM.from_config(cfg, attn_implementation="eager")
    ref = copy.deepcopy(model)
    option = PipeOption(device_cnt=2, batch_cnt=4, batch_size=2,
                        split_points=["model.layers.1", "model.layers.2", "model.layers.3"],
                        optimizer=dict(type="sgd", lr=0.0))
    runner = _runner(option)
    cmodel = torch.compile(model, backend=partial_compiler)

    def fn(ids):
        loss = cmodel(input_ids=ids, labels=ids).loss    # HF computes the shifted next-token loss itself
        loss.backward()
        return loss.detach()

    runner.set_exec_fn(fn)
    ids = torch.randint(3, 256, (8, 32), generator=torch.Generator().manual_seed(42))
    losses = runner.step(ids)
    assert len(runner.worker.part_graph.nodes) == 4
    want = []
    for chunk in ids.chunk(4):
        loss = ref(input_ids=chunk, labels=chunk).loss
        loss.backward()
        want.append(loss.detach())
    _check(model, ref, losses, want)
    kernels = _forward_kernels(runner)
    assert kernels.count("pf_rmsnorm_fwd") == (2 * 4 + 1) * 4          # decomposed norms became the norm kernel
    assert kernels.count("pf_rope") == 2 * 4 * 4                       # rotary embedding of q and k per layer
    assert kernels.count("pf_softmax_fwd") + kernels.count("pf_attention_fwd") == 4 * 4
