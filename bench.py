"""Headline benchmark: train samples/sec of the pipeline-stage hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload vit_l16_fp16]

One "step" is one PartialRunner.step(): micro-batch split, forward + backward of
every stage in the looped schedule's order for every micro-batch, fp32 gradient
accumulation, loss, optimizer step.  Inputs are resident in HBM before the timed
region.  Prints ONE JSON line (the last line of stdout).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"fp16": 2500.0, "bf16": 2500.0, "fp32": 157.3}
PEAK_HBM_GBS = 8000.0
AUTO_SPLIT = False   # --auto-split: split_points=None, the planner picks the stage boundaries


def log(*a):
    print(*a, file=sys.stderr, flush=True)


WORKLOADS = {
    # name: (family, config attr, global batch, batch_cnt, split points, device_cnt, mixed precision)
    "vit_l16_fp16": ("vit", "VIT_L16", 64, 4, ["blocks.12"], 2, "fp16"),
    "vit_s16_fp32": ("vit", "VIT_S16", 16, 4, ["blocks.6"], 2, None),
    "llama_1b_bf16": ("llama", "LLAMA_1B", 16, 8, ["layers.4", "layers.8", "layers.12"], 2, "bf16"),
    "vit_g14_share_bf16": ("vit_share", "VIT_G14_SHARE", 96, 4, [], 1, "bf16"),
    "sdxl_stage_fp16": ("unet", "SDXL_STAGE", 4, 1, [], 1, "fp16"),
}


def build_workload(name, device):
    import torch

    from pfeife_amd.bench_models import llama, unet_stage, vit
    from pfeife_amd.loss import CrossEntropyLoss
    from pfeife_amd.mp import PartialRunner, initialize_pfeife, partial_compiler
    from pfeife_amd.option import PipeOption

    family, cfg_name, batch, batch_cnt, splits, device_cnt, mixed = WORKLOADS[name]
    torch.manual_seed(42)
    g = torch.Generator().manual_seed(42)
    if family == "vit":
        cfg = getattr(vit, cfg_name)
        model = vit.VisionTransformer(cfg)
        inputs = (torch.randn(batch, cfg.channels, cfg.image_size, cfg.image_size, generator=g),
                  torch.randint(0, cfg.num_classes, (batch,), generator=g))
    elif family == "vit_share":
        cfg = getattr(vit, cfg_name)
        model = vit.BlockStack(cfg)
        inputs = (torch.randn(batch, cfg.tokens, cfg.dim, generator=g),
                  torch.randn(batch, cfg.tokens, cfg.dim, generator=g) * 1e-2)
    elif family == "unet":
        cfg = getattr(unet_stage, cfg_name)
        model = unet_stage.UNetStage(cfg)
        inputs = (torch.randn(batch, cfg.in_channels, 32, 32, generator=g),
                  torch.randn(batch, cfg.temb_dim, generator=g),
                  torch.randn(batch, 77, cfg.context_dim, generator=g),
                  torch.randn(batch, cfg.channels, 32, 32, generator=g))
    else:
        cfg = getattr(llama, cfg_name)
        model = llama.LlamaForCausalLM(cfg)
        inputs = (torch.randint(0, cfg.vocab, (batch, cfg.max_seq), generator=g),)
    initialize_pfeife()
    if AUTO_SPLIT and splits:
        # same stage count, boundaries chosen by the auto-partitioner from a profile on this GPU
        option = PipeOption(device_cnt=device_cnt, batch_cnt=batch_cnt, batch_size=batch // batch_cnt,
                            split_points=None, loop_cnt=(len(splits) + 1) // device_cnt, mixed_precision=mixed,
                            optimizer=dict(type="adam", lr=1e-5))
    else:
        option = PipeOption(device_cnt=device_cnt, batch_cnt=batch_cnt, batch_size=batch // batch_cnt,
                            split_points=splits or None, mixed_precision=mixed, optimizer=dict(type="adam", lr=1e-5))
    runner = PartialRunner(option)
    model.to(device)
    cmodel = torch.compile(model, backend=partial_compiler)
    if family == "vit":
        crit = CrossEntropyLoss(cfg.num_classes)

        def exec_fn(px, labels):
            loss = crit(cmodel(px), labels)
            loss.backward()
            return loss.detach()
    elif family == "vit_share":
        def exec_fn(act, grad_out):
            out = cmodel(act)
            out.backward(grad_out.to(out.dtype))   # supplied upstream gradient of this GPU's block share
            return out.detach()[0, 0, 0]
    elif family == "unet":
        def exec_fn(hidden, temb, ctx, target):
            out = cmodel(hidden, temb, ctx)
            loss = torch.nn.functional.mse_loss(out.float(), target.float())   # as train_sdxl.py:1422-1424
            loss.backward()
            return loss.detach()
    else:
        def exec_fn(ids):
            loss = cmodel(ids, ids)                # next-token CE is inside the last stage
            loss.backward()
            return loss.detach()

    runner.set_exec_fn(exec_fn)
    info = dict(cfg=cfg, batch=batch, batch_cnt=batch_cnt, splits=splits, device_cnt=device_cnt, mixed=mixed,
                model=model, family=family)
    return runner, tuple(t.to(device) for t in inputs), info


def measured_traffic(workload):
    """HBM bytes per launch (FETCH_SIZE + WRITE_SIZE, each scaled by the same counter's reading
    for a copy kernel of known size) per kernel name, parsed from the committed rocprofv3 --pmc
    summary `profiles/<workload>_pmc_traffic.md` (table rows `| `kernel` | ... | bytes |`, last
    column = bytes per launch).  Kernels that are not in the file have no figure."""
    path = os.path.join(ROOT, "profiles", "%s_pmc_traffic.md" % workload)
    out = {}
    if not os.path.exists(path):
        return out
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) < 2 or not cells[0].startswith("`"):
            continue
        try:
            out[cells[0].strip("`")] = float(cells[-1])
        except ValueError:
            pass
    return out


def _step_launches(runner):
    for slot in runner.worker.mbs.values():
        for prog in slot.stage_programs.values():
            for launch in list(prog.fwd) + list(prog.bwd):
                yield launch
    for launches, _ in runner.worker.dw_jobs.values():   # the once-per-step weight-gradient job of each stage
        for launch in launches:
            yield launch


def _time_launches(launches, reps):
    """Replays prepared launches back-to-back between HIP events on the stream they are issued on."""
    import torch

    stream = torch.cuda.current_stream()
    sp = stream.cuda_stream
    for launch in launches:  # warm
        launch(sp)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record(stream)
    for _ in range(reps):
        for launch in launches:
            launch(sp)
    ev1.record(stream)
    ev1.synchronize()
    return ev0.elapsed_time(ev1) / reps


def gemm_roofline(runner, mixed, workload, reps=3):
    """Replays every matrix-product launch of one step, grouped by kernel
    instantiation, between HIP events on the launch stream; returns the roofline
    record of the instantiation that takes the most time plus an all-GEMM summary."""
    groups = {}
    for launch in _step_launches(runner):
        if getattr(launch, "kernel", "") in ("pf_gemm", "pf_gemm_grouped"):
            g = groups.setdefault(launch.variant, dict(launches=[], flops=0.0))
            g["launches"].append(launch)
            g["flops"] += launch.flops
    out = {}
    for name, g in groups.items():
        ms = _time_launches(g["launches"], reps)
        n = len(g["launches"])
        out[name] = dict(ms_per_step=ms, launches_per_step=n, flops_per_step=g["flops"],
                         avg_launch_us=1e3 * ms / n, tflops=g["flops"] / (ms * 1e-3) / 1e12)
    if not out:
        return None, {}
    dom = max(out, key=lambda k: out[k]["ms_per_step"])
    peak = PEAK_TFLOPS[mixed or "fp32"]
    d = out[dom]
    tot_ms = sum(v["ms_per_step"] for v in out.values())
    tot_fl = sum(v["flops_per_step"] for v in out.values())
    roof = dict(bound="mfma", achieved=round(d["tflops"], 2), peak=peak, unit="TFLOP/s",
                frac=round(d["tflops"] / peak, 4), traffic=measured_traffic(workload).get(dom), kernel=dom,
                avg_launch_us=round(d["avg_launch_us"], 2), launches_per_step=d["launches_per_step"],
                flops_per_launch=d["flops_per_step"] / d["launches_per_step"],
                all_gemm_tflops=round(tot_fl / (tot_ms * 1e-3) / 1e12, 2), all_gemm_ms_per_step=round(tot_ms, 3))
    return roof, out


def hbm_kernel_rates(runner, reps=3):
    """Achieved HBM GB/s (algorithmic bytes / HIP-event time) of the bandwidth-bound kernels the
    step really launches, replayed per entry point, plus the optimizer step; the standalone fp32
    gradient-accumulate kernel is reported too but marked off-path (accumulation is fused into
    the weight-gradient products)."""
    import torch

    groups = {}
    for launch in _step_launches(runner):
        nb = getattr(launch, "bytes", None)
        if nb:
            g = groups.setdefault(launch.kernel, dict(launches=[], bytes=0.0))
            g["launches"].append(launch)
            g["bytes"] += nb
    out = []
    w = runner.worker
    for name, g in sorted(groups.items()):
        ms = _time_launches(g["launches"], reps)
        n = len(g["launches"])
        gbs = g["bytes"] / (ms * 1e-3) / 1e9
        # what a launch of this size can reach at all: a plain copy kernel that moves the same number
        # of bytes (half read, half written), launched the same number of times back to back
        per = max(1024, int(g["bytes"] / n) // 8)
        src = torch.ones(per, device="cuda")
        dst = torch.empty(per, device="cuda")
        copy = w.kernels.axpby(src, 1.0, None, 0.0, dst, per)
        copy_ms = _time_launches([copy] * min(n, 64), reps) / min(n, 64)
        del src, dst
        out.append(dict(kernel=name, on_path=True, launches_per_step=n, ms_per_step=round(ms, 3),
                        avg_launch_us=round(1e3 * ms / n, 2), bytes_per_launch=round(g["bytes"] / n),
                        achieved=round(gbs, 1), peak=PEAK_HBM_GBS, unit="GB/s", frac=round(gbs / PEAK_HBM_GBS, 4),
                        copy_same_bytes_us=round(1e3 * copy_ms, 2),
                        frac_of_copy=round(copy_ms / (ms / n), 4)))

    opt = w.optimizer
    if opt is not None and w._fused_adam_applicable(opt):
        n_par = sum(p.numel() for g in opt.param_groups for p in g["params"] if p.grad is not None)
        stream = w.stream_obj   # the optimizer step is issued on the worker's own stream

        def timed(fn):
            fn()
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record(stream)
            for _ in range(reps):
                fn()
            ev1.record(stream)
            ev1.synchronize()
            return ev0.elapsed_time(ev1) / reps

        if w.dyn_scale:
            # the in-place unscale + overflow check over the fp32 gradient buffers that precedes the step
            w.optimizer_step()            # builds the launch list
            n_g = sum(n for _, n in w.params.grad_buffers())
            ms = timed(lambda: [launch(w.stream()) for launch in w._unscale])
            gbs = 8.0 * n_g / (ms * 1e-3) / 1e9
            out.append(dict(kernel="pf_scaler_unscale", on_path=True, launches_per_step=len(w._unscale),
                            ms_per_step=round(ms, 3), avg_launch_us=round(1e3 * ms / len(w._unscale), 2),
                            bytes_per_launch=round(8.0 * n_g / len(w._unscale)), achieved=round(gbs, 1),
                            peak=PEAK_HBM_GBS, unit="GB/s", frac=round(gbs / PEAK_HBM_GBS, 4)))
        ms = timed(lambda: w._fused_adam_step(opt, scaled=w.dyn_scale))
        nb = 28.0 * n_par   # read p, g, m, v; write p, m, v (fp32)
        gbs = nb / (ms * 1e-3) / 1e9
        out.append(dict(kernel="pf_adam_step", on_path=True, launches_per_step=len(opt.param_groups),
                        ms_per_step=round(ms, 3), avg_launch_us=round(1e3 * ms / len(opt.param_groups), 2),
                        bytes_per_launch=round(nb / len(opt.param_groups)), achieved=round(gbs, 1), peak=PEAK_HBM_GBS,
                        unit="GB/s", frac=round(gbs / PEAK_HBM_GBS, 4)))
    k = w.kernels
    n = 4096 * 1024 * 16
    acc = torch.zeros(n, device="cuda")
    g = torch.ones(n, device="cuda")
    launch = k.grad_accumulate(acc, g, n)
    _time_launches([launch], 3)
    ms = _time_launches([launch], reps * 5)
    gbs = 12.0 * n / (ms * 1e-3) / 1e9
    out.append(dict(kernel="pf_grad_accumulate_f32", on_path=False, launches_per_step=0, ms_per_step=0.0,
                    avg_launch_us=round(ms * 1e3, 2), bytes_per_launch=12 * n, achieved=round(gbs, 1),
                    peak=PEAK_HBM_GBS, unit="GB/s", frac=round(gbs / PEAK_HBM_GBS, 4)))
    return out


def gemm_ceiling(kernels, mixed, reps=20):
    """Off-path record: what the step's matrix-product kernel reaches on shapes that take the
    step's shape losses away, so that kernel loss and shape loss can be told apart.  Times (hipGraph
    replays, HIP events) the 256x256-tile direct-to-LDS kernel on 8192^3, one of the step's own
    products ([3152 x 1024] . [1024 x 4096], the MLP's first layer, plain 16-bit store) and the same
    product with a four times longer reduction, plus the 128x128 tile on the step's dominant
    shape ([3152 x 4096] . [4096 x 1024]) and on that shape with 16 times the rows.  The first entry
    is no product at all: the tile's matrix-instruction stream alone on register-resident fragments
    of the same random data (`pf_mfma_rate`, no loads, LDS or barriers), on every CU for about as
    long as the 8192^3 product runs: what the MFMA pipes sustain under the board's power limit, the
    attainable ceiling the published peak (full boost clock) overstates."""
    import torch

    dt = {"fp16": torch.float16, "bf16": torch.bfloat16}.get(mixed)
    if dt is None:
        return None
    st = torch.cuda.Stream()
    s = st.cuda_stream
    out = []
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    frags = torch.cat([torch.randn(2048, device="cuda"), torch.randn(2048, device="cuda") * 0.03]).to(dt)
    wgs, iters = 1024, 512          # 4 workgroups per CU in turn, 8192 MFMAs per wavefront: the 8192^3 product's count
    sink = torch.empty(256 * wgs, device="cuda", dtype=torch.float32)
    rate = kernels.mfma_rate(frags, iters, wgs, sink)
    torch.cuda.synchronize()        # operands were made on the current stream, the launches go to `st`
    rate(s)
    ev0.record(st)
    for _ in range(reps):
        rate(s)
    ev1.record(st)
    ev1.synchronize()
    us = 1e3 * ev0.elapsed_time(ev1) / reps
    tf = wgs * 4 * iters * 16 * 2.0 * 32 * 32 * 16 / us / 1e6
    out.append(dict(shape="MFMA instruction stream only (no operand traffic), %d workgroups x 4 wavefronts x %d MFMAs" % (wgs, iters * 16),
                    kernel="mfma_rate_kernel<%d>" % {"fp16": 1, "bf16": 2}[mixed], avg_launch_us=round(us, 2),
                    tflops=round(tf, 1), frac=round(tf / PEAK_TFLOPS[mixed], 4)))
    for label, M, N, K, variant in (("8192^3, 256x256 tile", 8192, 8192, 8192, 7),
                                    ("step shape 3152x4096x1024, 256x256 tile", 3152, 4096, 1024, 7),
                                    ("same with K x4 (3152x4096x4096), 256x256 tile", 3152, 4096, 4096, 7),
                                    ("step shape 3152x1024x4096, 128x128 tile", 3152, 1024, 4096, 8),
                                    ("same with M x16 (50432x1024x4096), 128x128 tile", 50432, 1024, 4096, 8),
                                    ("same with M x16 (50432x1024x4096), 256x256 tile", 50432, 1024, 4096, 7)):
        x = torch.randn(M, K, device="cuda", dtype=dt)
        w = torch.randn(N, K, device="cuda", dtype=dt) * 0.03
        c = torch.empty(M, N, device="cuda", dtype=dt)
        n = 4 if M * N * K > 1e11 else 16
        torch.cuda.synchronize()
        chain = [kernels.gemm(x, w, c, M=M, N=N, K=K, lda=K, ldb=K, ldc=N, variant=variant) for _ in range(n)]
        graph = kernels.capture(chain, s)
        graph(s)
        ev0.record(st)
        for _ in range(reps):
            graph(s)
        ev1.record(st)
        ev1.synchronize()
        us = 1e3 * ev0.elapsed_time(ev1) / (reps * n)
        kernels.destroy_graph(graph)
        tf = 2.0 * M * N * K / us / 1e6
        out.append(dict(shape=label, kernel=chain[0].variant, avg_launch_us=round(us, 2), tflops=round(tf, 1),
                        frac=round(tf / PEAK_TFLOPS[mixed], 4)))
        del x, w, c, chain
    return out


def cpu_baseline(name):
    """The oracle's restatement of the reference's stage execution on the host
    cores, fp32, on a bounded sample of the workload (about 10-20 s of CPU work in all)."""
    import torch
    import torch.nn as nn
    import torch.nn.functional as F

    from oracle.stage_oracle import run_pipeline_step
    from pfeife_amd.bench_models import llama, unet_stage, vit

    family, cfg_name, batch, batch_cnt, splits, device_cnt, mixed = WORKLOADS[name]
    cores = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env:
        cores = min(cores, int(env))
    torch.set_num_threads(cores)
    torch.manual_seed(42)
    g = torch.Generator().manual_seed(42)
    cnt, passes = 2, 2
    if family == "vit":
        cfg = getattr(vit, cfg_name)
        model = vit.VisionTransformer(cfg)
        stages = vit.split_stages(model, int(splits[0].split(".")[1]))
        mb, cnt = 8, 4     # the workload's four micro-batches at half their size
        x = torch.randn(mb * cnt, cfg.channels, cfg.image_size, cfg.image_size, generator=g)
        y = torch.randint(0, cfg.num_classes, (mb * cnt,), generator=g)
        loss_fn = nn.CrossEntropyLoss()
        unit, per_sample = "samples/s", 1
    elif family == "vit_share":
        cfg = getattr(vit, cfg_name)
        stages = [vit.BlockStack(cfg)]
        mb = 4
        x = torch.randn(mb * cnt, cfg.tokens, cfg.dim, generator=g)
        y = torch.randn(mb * cnt, cfg.tokens, cfg.dim, generator=g) * 1e-2
        loss_fn = lambda o, t: (o * t).sum()
        unit, per_sample = "samples/s", 1
    elif family == "unet":
        cfg = getattr(unet_stage, cfg_name)
        stage = unet_stage.UNetStage(cfg)
        mb, cnt, passes = 1, 1, 1     # one sample, one pass (2e13 FLOPs: tens of seconds on the host cores)
        temb = torch.randn(mb, cfg.temb_dim, generator=g)
        ctx = torch.randn(mb, 77, cfg.context_dim, generator=g)

        class OneInput(nn.Module):     # the stage executor hands one tensor from stage to stage
            def __init__(self):
                super().__init__()
                self.stage = stage

            def forward(self, hidden):
                return self.stage(hidden, temb, ctx)

        stages = [OneInput()]
        x = torch.randn(mb * cnt, cfg.in_channels, 32, 32, generator=g)
        y = torch.randn(mb * cnt, cfg.channels, 32, 32, generator=g)
        loss_fn = lambda o, t: F.mse_loss(o.float(), t.float())
        unit, per_sample = "samples/s", 1
    else:
        cfg = getattr(llama, cfg_name)
        model = llama.LlamaForCausalLM(cfg)
        stages = llama.split_stages(model, [int(s.split(".")[1]) for s in splits])
        mb, T = 1, 512   # bounded: 2 micro-batches of one 512-token sequence
        x = torch.randint(0, cfg.vocab, (mb * cnt, T), generator=g)
        y = x
        loss_fn = lambda lg, t: F.cross_entropy(lg[:, :-1].reshape(-1, lg.shape[-1]), t[:, 1:].reshape(-1))
        unit, per_sample = "samples/s (sequences of 2048 tokens; measured tokens/s / 2048)", T / float(cfg.max_seq)
    times = []
    for _ in range(passes):  # with two passes the first warms the allocator and the thread pool
        t0 = time.perf_counter()
        run_pipeline_step(stages, loss_fn, x, y, cnt, device_cnt=device_cnt)
        times.append(time.perf_counter() - t0)
    sps = mb * cnt * per_sample / times[-1]
    return dict(value=round(sps, 4), unit=unit, cores=cores, kind="port",
                # the CPU sample is SMALLER than the GPU step: do not divide `value` fields by each other
                # without these (GPU step: the workload's micro_batch x batch_cnt, with the optimizer step)
                micro_batch=mb, batch_cnt=cnt, optimizer_step=False, precision="fp32",
                gpu_step_micro_batch=batch // batch_cnt, gpu_step_batch_cnt=batch_cnt,
                sample="%s fp32 on CPU: %d micro-batches x %d samples, %d stages, forward+backward+grad-accumulate "
                       "(no optimizer step), oracle stage executor; %.1f s%s" % (
                           cfg_name, cnt, mb, len(stages), times[-1],
                           "" if family != "llama" else "; 512-token sequences, attention cost scaled linearly"))


def torch_eager_gpu(name, device, steps=5, warmup=2):
    """The same optimisation step in plain PyTorch on the same GPU: the un-partitioned model run
    eagerly under torch.autocast, one forward + backward per micro-batch with gradient accumulation,
    torch.amp.GradScaler for fp16 and torch.optim.Adam.  This is what the reference's stages execute
    (eager ATen modules, pfeife/mp/worker.py:1457-1494 and 1585-1587, GradScaler :135-140) when all of
    them sit on one device, without its queues and copies.  Reported beside `value`, never as it."""
    import torch
    import torch.nn.functional as F

    from pfeife_amd.bench_models import llama, vit

    from pfeife_amd.bench_models import unet_stage

    family, cfg_name, batch, batch_cnt, splits, device_cnt, mixed = WORKLOADS[name]
    if family not in ("vit", "llama", "unet", "vit_share"):
        return None
    torch.manual_seed(42)
    g = torch.Generator().manual_seed(42)
    if family == "vit_share":
        cfg = getattr(vit, cfg_name)
        model = vit.BlockStack(cfg).to(device)
        x = torch.randn(batch, cfg.tokens, cfg.dim, generator=g).to(device)
        y = (torch.randn(batch, cfg.tokens, cfg.dim, generator=g) * 1e-2).to(device)

        def loss_of(xb, yb):   # the supplied upstream gradient, written as a loss: d(sum(out * g))/d(out) = g
            out = model(xb)
            return (out.float() * yb.float()).sum()
    elif family == "unet":
        cfg = getattr(unet_stage, cfg_name)
        model = unet_stage.UNetStage(cfg).to(device)
        x = torch.randn(batch, cfg.in_channels, 32, 32, generator=g).to(device)
        temb = torch.randn(batch, cfg.temb_dim, generator=g).to(device)
        ctx = torch.randn(batch, 77, cfg.context_dim, generator=g).to(device)
        y = torch.randn(batch, cfg.channels, 32, 32, generator=g).to(device)
        per = batch // batch_cnt
        state = {"i": 0}

        def loss_of(xb, yb):
            i = state["i"] % batch_cnt
            state["i"] += 1
            sl = slice(i * per, (i + 1) * per)
            return F.mse_loss(model(xb, temb[sl], ctx[sl]).float(), yb.float())
    elif family == "vit":
        cfg = getattr(vit, cfg_name)
        model = vit.VisionTransformer(cfg).to(device)
        x = torch.randn(batch, cfg.channels, cfg.image_size, cfg.image_size, generator=g).to(device)
        y = torch.randint(0, cfg.num_classes, (batch,), generator=g).to(device)

        def loss_of(xb, yb):
            return F.cross_entropy(model(xb).float(), yb)
    else:
        cfg = getattr(llama, cfg_name)
        model = llama.LlamaForCausalLM(cfg).to(device)
        x = torch.randint(0, cfg.vocab, (batch, cfg.max_seq), generator=g).to(device)
        y = x

        def loss_of(xb, yb):
            return model(xb, yb)
    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16}.get(mixed)
    opt = torch.optim.Adam(model.parameters(), lr=1e-5)
    # the reference builds its GradScaler for every mixed precision (pfeife/mp/worker.py:135)
    scaler = torch.amp.GradScaler("cuda", enabled=mixed in ("fp16", "bf16"))
    xs, ys = x.chunk(batch_cnt), y.chunk(batch_cnt)

    def step():
        opt.zero_grad(set_to_none=False)
        for xb, yb in zip(xs, ys):
            with torch.autocast("cuda", dtype=dtype, enabled=dtype is not None):
                loss = loss_of(xb, yb)
            scaler.scale(loss).backward()
        scaler.step(opt)
        scaler.update()
        return loss

    trace = []
    for _ in range(warmup):
        trace.append(step())
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
        trace.append(loss)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    last = float(loss)
    log("[bench] torch eager: last micro-batch loss per step", [round(float(l), 4) for l in trace])
    del opt, model
    torch.cuda.empty_cache()
    return dict(value=round(batch * steps / dt, 2), unit="samples/s", ms_per_step=round(1e3 * dt / steps, 3), steps=steps,
                sample="%s in PyTorch %s eager on this GPU: autocast %s, %d micro-batches x %d with gradient "
                       "accumulation, GradScaler %s, torch.optim.Adam; last loss %.4f" % (
                           cfg_name, torch.__version__, mixed, batch_cnt, batch // batch_cnt,
                           "on" if mixed in ("fp16", "bf16") else "off", last))


def unet_stage_forward_flops(cfg, hw=32, ctx_tokens=77):
    """Algorithmic forward FLOPs per sample of bench_models/unet_stage.UNetStage, layer by layer
    (2 x rows x in x out per linear layer / convolution tap, 4 x Tq x Tk x dim per attention)."""
    T, c, cin = hw * hw, cfg.channels, cfg.in_channels
    lin = lambda rows, i, o: 2.0 * rows * i * o

    def resnet(ci, co):
        f = lin(T, 9 * ci, co) + lin(T, 9 * co, co) + lin(1, cfg.temb_dim, co)   # conv1, conv2 (3x3), time embedding
        return f + (lin(T, ci, co) if ci != co else 0.0)                          # 1x1 shortcut

    def block():
        self_attn = 4 * lin(T, c, c) + 4.0 * T * T * c                            # q, k, v, out + QK^T, PV
        cross = 2 * lin(T, c, c) + 2 * lin(ctx_tokens, cfg.context_dim, c) + 4.0 * T * ctx_tokens * c
        ff = lin(T, c, 2 * cfg.ff_mult * c) + lin(T, cfg.ff_mult * c, c)          # GEGLU projection, output
        return self_attn + cross + ff

    transformer = 2 * lin(T, c, c) + cfg.layers * block()                         # proj_in, proj_out + blocks
    return resnet(cin, c) + resnet(c, c) + 2 * transformer + resnet(c, c) + transformer + resnet(c, c)


def model_flops_per_step(info):
    cfg, samples = info["cfg"], info["batch"]
    if info["family"] in ("vit", "vit_share"):
        T, d, ff, L = cfg.tokens, cfg.dim, cfg.mlp_dim, cfg.depth
        per_block = 2 * T * d * 3 * d + 2 * T * d * d + 4 * T * d * ff + 4 * T * T * d
        extra = 0
        if info["family"] == "vit":
            extra = 2 * (T - 1) * (cfg.channels * cfg.patch_size ** 2) * d + 2 * d * cfg.num_classes
        return 3.0 * samples * (L * per_block + extra)
    if info["family"] == "unet":
        return 3.0 * samples * unet_stage_forward_flops(cfg)
    T, d, ff, L, V = cfg.max_seq, cfg.dim, cfg.ffn, cfg.layers, cfg.vocab
    per_tok = L * (8 * d * d + 6 * d * ff + 4 * T * d) + 2 * d * V
    return 3.0 * samples * T * per_tok


def run_workload(name, steps, warmup, device, roofline=True, hbm=True, ceiling=True):
    """Builds the workload, runs warm-up + `steps` timed steps, then the per-kernel replays."""
    import torch

    runner, batch, info = build_workload(name, device)
    log("[bench] workload", name, "building stage programs (first step) ...")
    t0 = time.perf_counter()
    losses = runner.step(*batch)
    torch.cuda.synchronize()
    log("[bench] first step %.1f s, losses %s" % (time.perf_counter() - t0, [round(float(l), 4) for l in losses]))
    log("[bench]", runner.worker.memory_report())
    for _ in range(max(0, warmup - 1)):
        runner.step(*batch)
    torch.cuda.synchronize()
    w = runner.worker
    applied = lambda: float(w.scaler_state[3]) if w.dyn_scale else float(w.steps_done)
    if w.dyn_scale:
        # dynamic loss scaling starts high and halves on overflow (skipping that optimizer step):
        # extra untimed steps until one is applied, so that every timed step does the full work
        for extra in range(24):
            before = applied()
            runner.step(*batch)
            torch.cuda.synchronize()
            if applied() > before:
                break
        log("[bench] dynamic loss scale settled at %g after %d extra warm-up steps" % (w.scaler_scale(), extra + 1))
    before = applied()
    t0 = time.perf_counter()
    for _ in range(steps):
        losses = runner.step(*batch)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    skipped = steps - int(round(applied() - before))
    scaling = dict(mode="dynamic" if w.dyn_scale else "static",
                   scale=w.scaler_scale() if w.dyn_scale else float(runner.option.loss_scale),
                   skipped_optimizer_steps_in_timed_region=skipped)
    if skipped:
        log("[bench] WARNING: %d of %d timed steps overflowed and skipped their optimizer step" % (skipped, steps))
    ms = 1e3 * dt / steps
    value = info["batch"] * steps / dt
    log("[bench] %.2f ms/step, %.1f samples/s, last losses %s" % (ms, value, [round(float(l), 4) for l in losses]))

    # host-side cost of a step: time to ENQUEUE it (no synchronisation inside step())
    t0 = time.perf_counter()
    for _ in range(3):
        runner.step(*batch)
    host_ms = 1e3 * (time.perf_counter() - t0) / 3
    torch.cuda.synchronize()
    log("[bench] host enqueue time %.2f ms/step" % host_ms)

    roof, per_variant = gemm_roofline(runner, info["mixed"], name) if roofline else (None, {})
    for k, v in sorted(per_variant.items(), key=lambda kv: -kv[1]["ms_per_step"]):
        log("[bench] %-66s %4d launches/step %8.3f ms/step %8.1f us/launch %7.1f TFLOP/s"
            % (k, v["launches_per_step"], v["ms_per_step"], v["avg_launch_us"], v["tflops"]))
    rates = hbm_kernel_rates(runner) if hbm else None
    for r in rates or []:
        log("[bench] %-26s %4d launches/step %8.3f ms/step %8.1f us/launch %7.1f GB/s (%.0f%% of %d)%s%s"
            % (r["kernel"], r["launches_per_step"], r["ms_per_step"], r["avg_launch_us"], r["achieved"],
               100 * r["frac"], PEAK_HBM_GBS, "" if r["on_path"] else "  [off-path micro-benchmark]",
               "" if "frac_of_copy" not in r else "  copy of the same bytes: %.1f us (kernel at %.0f%% of it)"
               % (r["copy_same_bytes_us"], 100 * r["frac_of_copy"])))
    ceiling = gemm_ceiling(w.kernels, info["mixed"]) if (roofline and hbm and ceiling) else None
    for r in ceiling or []:
        log("[bench] gemm ceiling [off-path] %-52s %8.1f us/launch %7.1f TFLOP/s (%.0f%% of peak)  %s"
            % (r["shape"], r["avg_launch_us"], r["tflops"], 100 * r["frac"], r["kernel"]))
    flops_step = model_flops_per_step(info)
    cfg = info["cfg"]
    plan = getattr(w, "plan", None)
    used = getattr(w.part_graph, "nodes", {})
    splits_txt = ("%s (compute-node indices chosen by the auto-partitioner, expected %.1f ms/step for one rank per GPU)"
                  % (plan.split_points, plan.expect_ms)) if plan is not None else str(info["splits"])
    lanes = "%d streams (%s)" % (len(w.lanes), w.lane_mode) if w.lanes else "one stream"
    res = dict(value=value, ms=ms, host_ms=host_ms, roof=roof, hbm=rates, info=info, loss_scaling=scaling,
               gemm_ceiling=ceiling,
               model_tflops=None if flops_step is None else round(flops_step / (ms * 1e-3) / 1e12, 2),
               workload="%s: %s micro-batch %d x %d, %d stages split at %s, schedule drawn for %d ranks, "
                        "all stages on one GPU on %s, Adam" % (
                            name, type(cfg).__name__, info["batch"] // info["batch_cnt"], info["batch_cnt"],
                            len(used), splits_txt, info["device_cnt"], lanes))
    return runner, res


def release(runner):
    """Drops a workload's buffers so that the next one starts from an empty device."""
    import gc

    import torch

    runner.worker.release()
    runner.exec_fn = None
    del runner
    torch._dynamo.reset()
    gc.collect()
    torch.cuda.empty_cache()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="vit_l16_fp16", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--no-gemm-ceiling", action="store_true",
                    help="skip the off-path gemm_ceiling record (profiles of the step's own kernels)")
    ap.add_argument("--no-eager-baseline", action="store_true",
                    help="skip timing the same step in plain PyTorch eager on this GPU")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the bounded runs of the other GPU workloads that follow the headline measurement")
    ap.add_argument("--no-graph", action="store_true",
                    help="issue every kernel launch individually instead of replaying captured hipGraphs "
                         "(use for rocprofv3 --pmc runs: counters are collected per dispatched kernel)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain copy kernel (ew_kernel<Scale>, 256 MiB read + 256 MiB written) three "
                         "times, as the known-size reference for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs")
    ap.add_argument("--auto-split", action="store_true",
                    help="pass split_points=None: the auto-partitioner profiles the model on the GPU and picks "
                         "the stage boundaries (same stage count as the workload's manual split)")
    args = ap.parse_args()
    global AUTO_SPLIT
    AUTO_SPLIT = args.auto_split
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs every pipeline stage on ONE GPU; --gpus %d is not supported "
              "(no collectives, no second device)." % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda", 0)
    if args.no_graph:
        os.environ["PFEIFE_NO_GRAPH"] = "1"
    t_start = time.perf_counter()
    runner, head = run_workload(args.workload, args.steps, args.warmup, device, roofline=not args.no_roofline,
                                hbm=not args.no_roofline, ceiling=not args.no_gemm_ceiling)
    if args.calibrate_copy:
        n = 64 * 1024 * 1024
        src = torch.ones(n, device=device)
        dst = torch.empty(n, device=device)
        launch = runner.worker.kernels.axpby(src, 1.0, None, 0.0, dst, n)
        for _ in range(3):
            launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        del src, dst
    eager = None
    if not args.no_eager_baseline:
        log("[bench] timing plain PyTorch eager on this GPU ...")
        try:
            eager = torch_eager_gpu(args.workload, device)
        except Exception as e:   # report, do not lose the headline line
            eager = dict(skipped="failed: %s" % (str(e)[:200],))
        log("[bench] torch eager on this GPU", eager)
    cpu = None
    if not args.no_cpu_baseline:
        log("[bench] timing the CPU baseline ...")
        try:
            cpu = cpu_baseline(args.workload)
        except Exception as e:   # report, do not lose the headline line
            cpu = dict(skipped="failed: %s" % (str(e)[:200],))
        log("[bench] cpu baseline", cpu)

    # the other single-GPU configurations, for a bounded number of steps each (reported next to the
    # headline, never as `value`); a workload is skipped once the whole run has used its time budget
    others = []
    if not args.no_others and args.workload == "vit_l16_fp16":
        release(runner)
        runner = None
        for name in ("llama_1b_bf16", "vit_g14_share_bf16", "sdxl_stage_fp16"):
            if time.perf_counter() - t_start > 240.0:
                others.append(dict(workload=name, skipped="time budget of the default run used up"))
                continue
            try:
                r2, res = run_workload(name, 3, 2, device, roofline=not args.no_roofline, hbm=False)
            except Exception as e:   # report, do not lose the headline line
                others.append(dict(workload=name, skipped="failed: %s" % (str(e)[:200],)))
                continue
            roof = res["roof"] or {}
            others.append(dict(workload=res["workload"], value=round(res["value"], 2), unit="samples/s", steps=3,
                               ms_per_step=round(res["ms"], 3), model_tflops=res["model_tflops"],
                               host_enqueue_ms_per_step=round(res["host_ms"], 3), dominant_kernel=roof.get("kernel"),
                               frac=roof.get("frac"), all_gemm_tflops=roof.get("all_gemm_tflops"),
                               loss_scaling=res["loss_scaling"]))
            release(r2)
            r2 = None
            if not args.no_eager_baseline and time.perf_counter() - t_start < 240.0:
                try:   # the same step in plain PyTorch eager, where the leg covers the model family
                    e2 = torch_eager_gpu(name, device, steps=3, warmup=2)
                except Exception as e:
                    e2 = dict(skipped="failed: %s" % (str(e)[:200],))
                if e2 is not None:
                    others[-1]["torch_eager_gpu"] = e2
                    log("[bench] torch eager on this GPU", name, e2)

    info = head["info"]
    rec = {
        "metric": "train samples/sec on 1 MI355X; MFMA util % (GEMMs), HBM GB/s % (elementwise)",
        "value": round(head["value"], 2),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms"], 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": info["mixed"] or "fp32",
        "data": "synthetic (inputs ~N(0,1) / uniform int ids, random-init weights, seed 42)",
        "config": {"workload": head["workload"], "global_batch": info["batch"], "batch_cnt": info["batch_cnt"]},
        "roofline": head["roof"],
        "hbm_kernels": head["hbm"],
        "gemm_ceiling": head["gemm_ceiling"],
        "cpu_baseline": cpu,
        "torch_eager_gpu": eager,
        "model_tflops": head["model_tflops"],
        "host_enqueue_ms_per_step": round(head["host_ms"], 3),
        "loss_scaling": head["loss_scaling"],
        "other_workloads": others,
    }
    print(json.dumps(rec), flush=True)


if __name__ == "__main__":
    main()
