"""TEST INFRASTRUCTURE -- CPU/ATen restatement of the reference's stage execution.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module.

`run_pipeline_step` executes one optimisation step the way `ProcessWorker` does
for stages that all live on one rank (pfeife/mp/worker.py):
  * inputs are split with the reference's rule (oracle/batch_oracle.py);
  * jobs run in the order of `PipeSchedParams.rank_works` merged over ranks
    (oracle/schedule_oracle.py; merge = any order that respects the rank lists);
  * FORWARD  (worker.py:1438-1502): stage inputs are CLONES of the boundary
    buffers, the stage is called under torch.autocast when mixed precision is
    on (worker.py:675-680), the result keeps its autograd graph;
  * SEND_ACT (worker.py:1096-1128): result copied with `copy_` into the
    consumer's preallocated `requires_grad` leaf buffer;
  * the loss is evaluated by user code on a detached `requires_grad` copy of the
    last stage's output and its gradient recorded by a hook
    (pfeife/mp/partial/module.py:119-143);
  * BACKWARD (worker.py:1504-1590): `torch.autograd.backward(outputs, grads)`,
    which accumulates into `param.grad` (AccumulateGrad);
  * SEND_GRAD (worker.py:1129-1151): `input_buffer.grad` copied into the
    producer's gradient buffer, zeros if there is none (worker.py:84-88);
  * gradients are zero-filled, not None, at step start (worker.py:583-597).
The GradScaler of worker.py:133-145 is represented by `loss_scale` applied at
every stage output like the reference does (worker.py:1580); 1.0 disables it.

Pinned by tests/test_stage_oracle.py: in fp32 on CPU the accumulated gradients
and the losses are bit-identical to plain gradient accumulation over the
micro-batches on the un-partitioned model.
"""
import contextlib

import torch

from .batch_oracle import split_args_kwargs
from .schedule_oracle import rank_works


def merge_rank_works(works, node_cnt):
    pos = [0] * len(works)
    done, order = set(), []
    total = sum(len(w) for w in works)
    while len(order) < total:
        moved = False
        for r, w in enumerate(works):
            if pos[r] >= len(w):
                continue
            n, b, f = w[pos[r]]
            ok = (n == 0 or (n - 1, b, True) in done) if f else (
                (n, b, True) in done and (n == node_cnt - 1 or (n + 1, b, False) in done))
            if ok:
                done.add((n, b, f))
                order.append((n, b, f))
                pos[r] += 1
                moved = True
        if not moved:
            raise RuntimeError("deadlock")
    return order


def run_pipeline_step(stages, loss_fn, inputs, targets, batch_cnt, device_cnt=1, loop_batch=None, prefetch_fwd=0,
                      autocast_dtype=None, loss_scale=1.0, zero_grads=True):
    """stages: list of nn.Module, stage i maps the previous stage's tensor to the next;
    loss_fn(output, target_chunk) -> scalar.  Returns the list of per-micro-batch losses."""
    node_cnt = len(stages)
    device_cnt = min(device_cnt, node_cnt)
    loop_batch = loop_batch or device_cnt
    order = merge_rank_works(rank_works(device_cnt, batch_cnt, node_cnt, loop_batch, prefetch_fwd), node_cnt)
    (chunks, _) = split_args_kwargs((inputs, targets), None, batch_cnt)
    dev = next(stages[0].parameters()).device
    if zero_grads:
        for st in stages:
            for p in st.parameters():
                p.grad = torch.zeros_like(p)
    ctx = (lambda: torch.autocast(dev.type, dtype=autocast_dtype)) if autocast_dtype else contextlib.nullcontext
    in_buf, results, loss_grads, grad_buf, losses = {}, {}, {}, {}, [None] * batch_cnt
    for n, b, is_fwd in order:
        if is_fwd:
            if n == 0:
                x = chunks[b][0].to(dev)
            else:
                with ctx():
                    x = in_buf[(n, b)].clone()
            with ctx():
                out = stages[n](x)
            results[(n, b)] = out
            if n + 1 < node_cnt:
                buf = torch.zeros(out.shape, dtype=out.dtype, device=dev, requires_grad=out.requires_grad)
                with torch.no_grad():
                    buf.copy_(out)
                in_buf[(n + 1, b)] = buf
            else:
                user_out = out.detach().requires_grad_()
                user_out.register_hook(lambda g, b=b: loss_grads.__setitem__(b, g))
                loss = loss_fn(user_out, chunks[b][1].to(dev))
                loss.backward()
                losses[b] = loss.detach()
        else:
            out = results.pop((n, b))
            g = loss_grads.pop(b) if n == node_cnt - 1 else grad_buf.pop((n, b))
            torch.autograd.backward([out * loss_scale] if loss_scale != 1.0 else [out], [g])
            if n > 0:
                ib = in_buf.pop((n, b))
                grad_buf[(n - 1, b)] = (ib.grad if ib.grad is not None else torch.zeros_like(ib)).clone()
    return losses


def run_unpipelined(model, loss_fn, inputs, targets, batch_cnt, autocast_dtype=None):
    """Plain gradient accumulation: for each micro-batch, forward, loss, backward."""
    (chunks, _) = split_args_kwargs((inputs, targets), None, batch_cnt)
    dev = next(model.parameters()).device
    for p in model.parameters():
        p.grad = torch.zeros_like(p)
    ctx = (lambda: torch.autocast(dev.type, dtype=autocast_dtype)) if autocast_dtype else contextlib.nullcontext
    losses = []
    for x, y in chunks:
        with ctx():
            out = model(x.to(dev))
        loss = loss_fn(out, y.to(dev))
        loss.backward()
        losses.append(loss.detach())
    return losses
