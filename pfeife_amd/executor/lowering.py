"""Turns one pipeline-stage FX graph into prepared HIP launch lists.

This module occupies the seam where the reference calls the stage submodule
(`self.mods[node.idx](*inputs)`, pfeife/mp/worker.py:1457-1494) and
`torch.autograd.backward` (pfeife/mp/worker.py:1585-1587): instead of running
ATen kernels under autograd, the stage graph is lowered ONCE per (stage,
micro-batch) to

    program.fwd : [launch, ...]     forward kernels on preallocated buffers
    program.bwd : [launch, ...]     hand-derived backward kernels

and a step replays those lists.  Stage inputs are used in place (the reference
clones them, worker.py:1442-1455) and the gradient of a stage input is written
straight into the buffer the producing stage reads as its output gradient (the
reference copies twice, worker.py:1096-1151): the handoff moves no bytes.

Numerics follow torch.autocast's policy when `compute_dtype` is fp16/bf16
(reference: `get_mp_ctx`, worker.py:675-680): matrix products take 16-bit
operands with fp32 accumulation and give 16-bit results, normalisations,
softmax and losses are computed in fp32, the residual stream stays fp32 and
parameter gradients are accumulated in fp32.
"""
import math
import operator
import os

import torch
import torch.nn.functional as F

from .values import Val, as_matrix, collapse_for_copy, dense_like, is_dense

ACT_NONE, ACT_GELU, ACT_GELU_TANH, ACT_SILU, ACT_RELU = 0, 1, 2, 3, 4
# kernel variant (pf_gemm_desc.variant) that regrouped weight-gradient products are pinned to: the 256x256
# tile the automatic choice itself uses (eight wavefronts), so that products that chose it on their own and
# products moved onto it share launches
BIG_TILE_VARIANT = int(os.environ.get("PFEIFE_BIG_TILE", "7"))


class Unsupported(RuntimeError):
    """A graph node for which no HIP lowering exists. There is no eager fallback."""


# ---------------------------------------------------------------------------
# parameter store: fp32 masters, 16-bit shadows, fp32 gradient accumulators
# ---------------------------------------------------------------------------
class ParamStore:
    def __init__(self, kernels, device):
        self.kernels = kernels
        self.device = device
        self._shadow = {}      # (id(param), dtype) -> tensor
        self._grads = {}       # id(param) -> fp32 grad tensor (== param.grad)
        self.refresh = []      # launches: master -> shadow casts (once per step)
        self.zero = []         # launches: zero-fill of every gradient accumulator (once per step)
        self.params = []       # parameters that receive gradients, in first-use order
        self._keep = []
        self.cast_pairs = []   # (fp32 master, 16-bit shadow): refreshed by ONE batched launch per step
        self.shadow_t_pairs = []   # (fp32 master, transposed 16-bit shadow) of weight matrices
        self._arena = None     # current block of the gradient arena
        self._arena_used = 0
        self.arena_block = 64 * 1024 * 1024   # fp32 elements per arena block (256 MiB)
        # Gradients that ONE once-per-step weight-gradient product writes whole (stored, already
        # unscaled and checked for overflow by that product's epilogue) need no zero fill and no
        # unscale pass: they live in blocks of their own, outside the arena those passes sweep.
        self._lazy = {}            # id(param) -> True while that holds, False once another writer appeared
        self._lazy_block = None
        self._lazy_used = 0
        self.deferred_sites = {}   # id(param) -> {(stage, node name)} of the deferred products that write it
        self.pending_fills = []    # zero fills of gradients demoted since the step's zero fill ran

    def shadow(self, tensor, dtype):
        if tensor.dtype == dtype:
            return tensor
        key = (tensor.data_ptr(), tuple(tensor.shape), tensor.dtype, dtype)
        sh = self._shadow.get(key)
        if sh is None:
            sh = torch.empty(tensor.shape, dtype=dtype, device=tensor.device)
            src = tensor.detach()
            if not src.is_contiguous():
                raise Unsupported("non-contiguous parameter %s" % (tuple(tensor.shape),))
            if hasattr(self.kernels, "cast_batch"):
                self.cast_pairs.append((src, sh))
            else:
                self.refresh.append(self.kernels.cast(src, sh, src.numel()))
            self._shadow[key] = sh
            self._keep.append(tensor)
        return sh

    def refresh_launches(self):
        """Launches that bring every shadow up to date with its master (once per step): weight
        matrices get their plain and transposed shadows from one read of the master, in one
        launch for all of them; the remaining casts share a second launch."""
        out = list(self.refresh)
        pairs = list(self.cast_pairs)
        t_of = {src.data_ptr(): (src, sh) for src, sh in self.shadow_t_pairs}
        batch = getattr(self.kernels, "shadow_batch", None)
        duals, rest = [], []
        for src, sh in pairs:
            hit = t_of.get(src.data_ptr())
            if (batch is not None and hit is not None and hit[1].dtype == sh.dtype
                    and self.kernels.shadow_batch_ok(src, sh, hit[1])):
                duals.append((src, sh, hit[1]))
                del t_of[src.data_ptr()]
            else:
                rest.append((src, sh))
        for src, sh in t_of.values():           # transposed shadow only (or not batchable)
            if batch is not None and self.kernels.shadow_batch_ok(src, None, sh):
                duals.append((src, None, sh))
            else:
                rows, cols = src.shape
                out.append(self.kernels.transpose_cast(src, cols, sh, rows, rows, cols))
        if duals:
            out.insert(0, batch(duals))
        if rest:
            out.insert(0, self.kernels.cast_batch(rest))
        return out

    def _arena_alloc(self, shape, device):
        """fp32 gradient accumulator carved out of a large block, so that one fill per block
        zeroes every gradient of the step (optimizer.zero_grad(set_to_none=False))."""
        n = 1
        for d in shape:
            n *= int(d)
        pad = (n + 63) // 64 * 64   # keep every accumulator 256-byte aligned
        if n >= self.arena_block // 4:
            t = torch.zeros(shape, dtype=torch.float32, device=device)
            self.zero.append(self.kernels.fill(t, 0.0, t.numel()))
            return t
        if self._arena is None or self._arena_used + pad > self._arena.numel():
            self._arena = torch.zeros(self.arena_block, dtype=torch.float32, device=device)
            self._arena_used = 0
            self.zero.append(None)          # placeholder: the block's fill is sized when known
            self._arena_slots = getattr(self, "_arena_slots", []) + [(len(self.zero) - 1, self._arena)]
        t = self._arena[self._arena_used:self._arena_used + n].view(shape)
        self._arena_used += pad
        return t

    def zero_launches(self):
        """Launches that zero every gradient accumulator (one fill per arena block)."""
        out = []
        slots = dict((i, a) for i, a in getattr(self, "_arena_slots", []))
        for i, launch in enumerate(self.zero):
            if launch is not None:
                out.append(launch)
            else:
                a = slots[i]
                used = self._arena_used if a is self._arena else a.numel()
                out.append(self.kernels.fill(a, 0.0, used))
        return out

    def grad_buffers(self):
        """(buffer, used elements) of every fp32 gradient accumulator: whole arenas where the
        gradients live in one, single tensors otherwise."""
        out = []
        slots = dict((i, a) for i, a in getattr(self, "_arena_slots", []))
        done = set()
        for i, launch in enumerate(self.zero):
            if launch is None:
                a = slots[i]
                used = self._arena_used if a is self._arena else a.numel()
                out.append((a, used))
                done.add(a.data_ptr())
        for p in self.params:
            g = self._grads[id(p)]
            base = g._base if g._base is not None else g
            if base.data_ptr() not in done and not self._lazy.get(id(p)):
                out.append((g, g.numel()))
        return out

    def scale_grads_launches(self, factor):
        """Launches multiplying every gradient accumulator by `factor` (loss-scale removal)."""
        out = []
        slots = dict((i, a) for i, a in getattr(self, "_arena_slots", []))
        done = set()
        for i, launch in enumerate(self.zero):
            if launch is None:
                a = slots[i]
                used = self._arena_used if a is self._arena else a.numel()
                out.append(self.kernels.axpby(a, factor, None, 0.0, a, used))
                done.add(a.data_ptr())
        for p in self.params:
            g = self._grads[id(p)]
            base = g._base if g._base is not None else g
            if base.data_ptr() not in done and not self._lazy.get(id(p)):
                out.append(self.kernels.axpby(g, factor, None, 0.0, g, g.numel()))
        return out

    def shadow_t(self, tensor, dtype):
        """Transposed copy [cols, rows] of a 2-d parameter in `dtype`, refreshed once per step."""
        key = (tensor.data_ptr(), tuple(tensor.shape), tensor.dtype, dtype, "T")
        sh = self._shadow.get(key)
        if sh is None:
            rows, cols = tensor.shape
            sh = torch.empty((cols, rows), dtype=dtype, device=tensor.device)
            src = tensor.detach()
            if not src.is_contiguous():
                raise Unsupported("non-contiguous parameter %s" % (tuple(tensor.shape),))
            self.shadow_t_pairs.append((src, sh))
            self._shadow[key] = sh
            self._keep.append(tensor)
        return sh

    def shadow_perm(self, tensor, dtype, perm):
        """Contiguous copy of tensor.permute(perm) in `dtype` (e.g. conv weights as [O, kh, kw, C]),
        refreshed once per step."""
        key = (tensor.data_ptr(), tuple(tensor.shape), tensor.dtype, dtype, tuple(perm))
        sh = self._shadow.get(key)
        if sh is None:
            src = tensor.detach().permute(*perm)
            sh = torch.empty(src.shape, dtype=dtype, device=tensor.device)
            sizes, ss, ds = collapse_for_copy(src.shape, src.stride(), sh.stride())
            self.refresh.append(self.kernels.copy_strided(src, ss, sh, ds, sizes, 0))
            self._shadow[key] = sh
            self._keep.append(tensor)
        return sh

    def _lazy_alloc(self, shape, device):
        n = 1
        for d in shape:
            n *= int(d)
        pad = (n + 63) // 64 * 64
        if n >= self.arena_block // 4:
            return torch.zeros(shape, dtype=torch.float32, device=device)
        if self._lazy_block is None or self._lazy_used + pad > self._lazy_block.numel():
            self._lazy_block = torch.zeros(self.arena_block, dtype=torch.float32, device=device)
            self._lazy_used = 0
        t = self._lazy_block[self._lazy_used:self._lazy_used + n].view(shape)
        self._lazy_used += pad
        return t

    def demote(self, param):
        """The gradient of `param` has (or may have) a writer besides its one storing product: from now
        on it is zeroed at the start of a step and swept by the unscale pass like any other."""
        if self._lazy.get(id(param)):
            self._lazy[id(param)] = False
            g = self._grads[id(param)]
            fill = self.kernels.fill(g, 0.0, g.numel())
            self.zero.append(fill)
            # this step's zero fill has already run without it, and the buffer may still hold the
            # previous step's stored gradient: the worker runs these before anything accumulates
            self.pending_fills.append(fill)

    def stored_whole(self, param):
        return bool(self._lazy.get(id(param))) and len(self.deferred_sites.get(id(param), ())) == 1

    def grad(self, param, deferred_site=None):
        """fp32 gradient accumulator of `param` (== param.grad).  deferred_site: (stage, node name) of
        a once-per-step weight-gradient product that asks for it; any other caller accumulates."""
        g = self._grads.get(id(param))
        if deferred_site is not None:
            self.deferred_sites.setdefault(id(param), set()).add(deferred_site)
        if g is None:
            if deferred_site is not None and param.grad is None and param.dim() == 2:
                param.grad = g = self._lazy_alloc(param.shape, param.device)
                self._lazy[id(param)] = True
            elif param.grad is None or param.grad.dtype != torch.float32 or not param.grad.is_contiguous():
                param.grad = self._arena_alloc(param.shape, param.device)
                g = param.grad
            else:
                g = param.grad
                self.zero.append(self.kernels.fill(g, 0.0, g.numel()))
            self._grads[id(param)] = g
            self.params.append(param)
        else:
            if deferred_site is None:
                self.demote(param)
            if param.grad is not g:
                # user code replaced .grad (e.g. zero_grad(set_to_none=True)); programs hold raw pointers
                param.grad = g
        return g

    def rebind_grads(self):
        for p in self.params:
            g = self._grads[id(p)]
            if p.grad is not g:
                p.grad = g


class BufferPool:
    """Named scratch and per-stage backward buffers, shared wherever lifetimes cannot overlap."""

    def __init__(self, device):
        self.device = device
        self._scratch = {}
        self._bwd = {}
        self._stacked = {}
        self.bytes = 0
        # Jobs of different pipeline ranks may run at the same time on streams of their own;
        # the worker sets `lane` to the rank whose stage is being lowered, and every shared
        # buffer is shared within a lane only.
        self.lane = 0

    def scratch(self, slot, shape, dtype):
        key = (self.lane, slot, tuple(shape), dtype)
        t = self._scratch.get(key)
        if t is None:
            t = torch.empty(tuple(shape), dtype=dtype, device=self.device)
            self._scratch[key] = t
            self.bytes += t.numel() * t.element_size()
        return t

    def bwd_like(self, seq, like):
        """Buffer number `seq` of a backward job.  Backward jobs of one lane never overlap in
        time (one stream, one job at a time) and their temporaries die with the
        job, so all stages and micro-batches of a lane share one set of buffers."""
        key = (self.lane, seq, tuple(like.shape), tuple(like.stride()), like.dtype)
        t = self._bwd.get(key)
        if t is None:
            t = torch.empty_like(like, device=self.device)
            self._bwd[key] = t
            self.bytes += t.numel() * t.element_size()
        return t

    def fresh_like(self, like):
        t = torch.empty_like(like, device=self.device)
        self.bytes += t.numel() * t.element_size()
        return t

    def stacked(self, key, shape, dtype, mb, count):
        """Buffer `key` of micro-batch `mb`, one of `count` equal buffers laid end to end in one
        allocation: what the micro-batches of a step write at the same place of the same stage
        (an activation, the gradient of a layer's output) then forms ONE matrix with `count` times
        the rows, which the weight-gradient product of the whole step reads in a single launch."""
        shape = tuple(int(x) for x in shape)
        if mb is None or not 0 <= mb < count:
            return torch.empty(shape, dtype=dtype, device=self.device)
        key = (key, shape, dtype, count)
        slab = self._stacked.get(key)
        if slab is None:
            slab = self._stacked[key] = torch.empty((count,) + shape, dtype=dtype, device=self.device)
            self.bytes += slab.numel() * slab.element_size()
        return slab[mb]

    def prune_stacked(self, live_tags):
        """Forget the stacked allocations made under tags no micro-batch slot uses any more (their
        memory goes when the programs that hold slices of them do)."""
        self._stacked = {k: v for k, v in self._stacked.items() if k[0][0] in live_tags}


class StageProgram:
    def __init__(self, stage, mb):
        self.stage = stage
        self.mb = mb
        self.inputs = []       # [Val] in stage-placeholder order
        self.outputs = []      # [Val or python constant]
        self.fwd = []
        self.bwd = []
        self.backward_fns = []  # build-time closures, one per lowered node, in forward order
        self.input_grads = []   # filled by lower_backward: gradient tensor (or None) per input
        self.fwd_bytes = 0
        self.tile_groups = []   # sibling regions that must all be written for the zero-fill to be skipped
        self.fwd_graph = None   # replay callables once the launch lists have been captured
        self.bwd_graph = None
        # which launches belong to which graph node (the partitioner's profiler times them):
        # (node name, first launch, one past the last launch[, forward bytes allocated])
        self.fwd_ranges = []
        self.bwd_ranges = []
        self.backward_nodes = []  # node name per entry of backward_fns
        self.alloc_seq = 0        # forward buffers handed out so far (the same sequence for every micro-batch)
        # weight-gradient products left to the stage's once-per-step job: (numel, dtype) of the layer
        # output gradients they read, and per product (dy, x, accumulator, gemm arguments)
        self.dw_sigs = set()
        self.dw_deferred = []

    def run_forward(self, stream):
        if self.fwd_graph is not None:
            self.fwd_graph(stream)
            return
        for launch in self.fwd:
            launch(stream)

    def run_backward(self, stream):
        if self.bwd_graph is not None:
            self.bwd_graph(stream)
            return
        for launch in self.bwd:
            launch(stream)


def _dtype_promote(a, b):
    return torch.promote_types(a, b)


# ---------------------------------------------------------------------------
# backward build context
# ---------------------------------------------------------------------------
class BwdCtx:
    def __init__(self, lowerer, program):
        self.L = lowerer
        self.k = lowerer.kernels
        self.program = program
        self.out = program.bwd
        self._seq = 0
        self._pending = {}
        self.reduces = []   # deferred column reductions, finished by one batched launch at the end
        self._dw = []       # held-back weight-gradient products: (launch, accumulator, tiles)
        self._dw_big = []   # open sets of issued ones that may yet share a launch on 256x256 tiles, each a list of
                            # (issued launch, its products on that tile, their accumulators, tiles)
        # 16-bit copies of fp32 gradients that a producing kernel wrote on the side, and column
        # sums of such copies left as partial rows: {data_ptr: (storage_ptr, copy, colsum or None)}
        self._lp = {}
        self._kept = {}     # (numel, dtype) -> buffers of that kind handed out so far in this job

    def emit(self, launch):
        self.out.append(launch)

    def _kept_for_dw(self, shape, dtype):
        """Gradients that a deferred weight-gradient product may read must outlive the job and lie
        end to end across micro-batches: buffers of those sizes come from stacked allocations
        (per stage and position in the job), not from the set every job of a lane shares."""
        sigs = self.program.dw_sigs
        if not sigs or not self.L.defer_dw:
            return None
        n = 1
        for d in shape:
            n *= int(d)
        if (n, dtype) not in sigs:
            return None
        i = self._kept[(n, dtype)] = self._kept.get((n, dtype), 0) + 1
        return self.L.pool.stacked((self.L.stack_tag, "g", self.program.stage, i, n), shape, dtype, self.program.mb,
                                   self.L.stack_mbs)

    # -- weight-gradient products that share a launch ---------------------------------------------
    FULL_GRID = 256     # workgroups that fill the device (one tile per CU)
    OPEN_SETS = 4       # sets of issued weight-gradient products that may yet share a launch on 256x256 tiles

    @staticmethod
    def _tiles(launch):
        bm, bn = (int(x) for x in launch.variant.split("<")[1].split(",")[1:3])
        return ((launch.desc.M + bm - 1) // bm) * ((launch.desc.N + bn - 1) // bn)

    def emit_dw(self, launch, grad):
        """A weight-gradient product: only the optimizer reads its result, and its inputs (a
        finished gradient, a saved activation) are not written again within the job, so it may
        be held back and issued together with later ones.  Products too small to give every CU a
        tile are collected until they fill the device (ViT-L: dW of the 1024x1024 attention
        projection, 64 tiles, rides with dW of the qkv projection, 192 tiles)."""
        groupable = getattr(self.k, "gemm_groupable", None)
        if groupable is None or not groupable(launch):
            self.emit(launch)
            return
        tiles = self._tiles(launch)
        if any(g.data_ptr() == grad.data_ptr() for _, g, _ in self._dw) or \
                any(g.data_ptr() == grad.data_ptr() for entries in self._dw_big for _, _, gs, _ in entries for g in gs):
            self.flush_dw()          # two products into one accumulator keep their order
            self._dw_big = []
        if tiles >= self.FULL_GRID:
            self.emit(launch)
            self._offer_big(launch, [(launch, grad)])
            return
        held = sum(t for _, _, t in self._dw)
        if self._dw and (self._dw[0][0].group_key != launch.group_key or held + tiles > self.FULL_GRID
                         or len(self._dw) == self.k.GEMM_GROUP_MAX):
            self.flush_dw()
            held = 0
        self._dw.append((launch, grad, tiles))
        if held + tiles >= self.FULL_GRID - 32:
            self.flush_dw()

    def _offer_big(self, issued, members):
        """`issued` (one launch, already in the job) computes `members`: (product, accumulator) pairs.
        Products that fill the device on 128x128 tiles, alone or a few together, run faster on 256x256
        tiles, which move half the operand bytes per FLOP through LDS, but then cover only part of it (a
        decoder's 2048x2048 attention projections and ViT-L's 1024x4096 MLP weights: 64 tiles each).  So
        every such launch is issued where it stands and remembered; once the remembered products give
        nearly every CU a 256x256 tile they all give way to ONE launch on that tile, at the place of the
        last.  Members of a set that is dropped stay as they were issued, and the sums are the same bit
        for bit either way (the tile does not change the order in which a product is summed)."""
        retile = getattr(self.k, "gemm_retiled", None)
        if retile is None or os.environ.get("PFEIFE_DW_RETILE", "1") == "0":
            return
        bigs, t256 = [], 0
        for launch, _ in members:
            d = launch.desc
            big = launch if launch.variant.startswith("gemm16x_kernel<%d, 256, 256" % d.in_dtype) else retile(launch, BIG_TILE_VARIANT)
            if d.M < 256 or d.N < 256 or big is None or not self.k.gemm_groupable(big):
                return               # less than one full tile either way: stays on the small tile
            bigs.append(big)
            t256 += ((d.M + 255) // 256) * ((d.N + 255) // 256)
        if t256 > self.FULL_GRID - 32:
            return                   # nothing worth its launch fits beside it
        # best fit over a few open sets: the fullest one that still takes it (a decoder's 5632x2048 MLP
        # weights, 176 tiles each, are each completed by one of the 64-tile attention projections)
        mine = None
        for entries in self._dw_big:
            held = sum(t for _, _, _, t in entries)
            if entries[0][1][0].group_key == bigs[0].group_key and held + t256 <= self.FULL_GRID \
                    and sum(len(b) for _, b, _, _ in entries) + len(bigs) <= self.k.GEMM_GROUP_MAX \
                    and (mine is None or held > sum(t for _, _, _, t in mine)):
                mine = entries
        if mine is None:
            mine = []
            self._dw_big.append(mine)
            if len(self._dw_big) > self.OPEN_SETS:
                self._close_set(self._dw_big[0])     # the oldest has waited long enough
        mine.append((issued, bigs, [g for _, g in members], t256))
        if sum(t for _, _, _, t in mine) >= self.FULL_GRID - 56:
            self._close_set(mine)

    def _close_set(self, entries):
        """Two or more remembered launches that cover half the device or more on 256x256 tiles give way to
        one launch on that tile, here; anything less stays as it was issued."""
        self._dw_big.remove(entries)
        if len(entries) >= 2 and sum(t for _, _, _, t in entries) >= self.FULL_GRID // 2:
            for old, _, _, _ in entries:   # blanked, not deleted: positions in the list stay valid until compact()
                self.out[next(i for i in range(len(self.out) - 1, -1, -1) if self.out[i] is old)] = None
            self.emit(self.k.gemm_group([b for _, bs, _, _ in entries for b in bs]))

    def compact(self, ranges):
        """Drop the blanked launches; `ranges` ((name, first, end) over the list) follow."""
        new, n = [], 0
        for launch in self.out:
            new.append(n)
            n += launch is not None
        new.append(n)
        self.out[:] = [launch for launch in self.out if launch is not None]
        ranges[:] = [(name, new[a], new[b]) for name, a, b in ranges]

    def close_dw(self):
        """End of the job: nothing more will arrive."""
        self.flush_dw()
        while self._dw_big:
            self._close_set(self._dw_big[0])

    def flush_dw(self):
        if len(self._dw) == 1:
            self.emit(self._dw[0][0])
            self._offer_big(self._dw[0][0], [(self._dw[0][0], self._dw[0][1])])
        elif self._dw:
            group = self.k.gemm_group([l for l, _, _ in self._dw])
            self.emit(group)
            self._offer_big(group, [(l, g) for l, g, _ in self._dw])
        self._dw = []

    def register_lp(self, full, copy, colsum=None):
        """`copy` holds the values of the fp32 gradient `full` in the compute dtype; `colsum`:
        (ws, offset, n_partials, stride) of partial rows whose sum is copy's column sum."""
        self._lp[full.data_ptr()] = (full.untyped_storage().data_ptr(), copy, colsum)

    def _written(self, t):
        """Gradient buffer t is about to be written: side copies of anything in its storage are stale."""
        if self._lp and t is not None:
            st = t.untyped_storage().data_ptr()
            for key in [k for k, v in self._lp.items() if v[0] == st]:
                del self._lp[key]

    def colsum_from_producer(self, x, rows, cols, ld, acc):
        """The kernel that produced x may already have summed its columns (partial rows on the side):
        then acc[c] += those, finished with the job's other reductions.  -> whether that was so."""
        for _, copy, cs in self._lp.values():
            if cs is not None and copy.data_ptr() == x.data_ptr() and copy.numel() == rows * cols and ld == cols:
                ws, off, nb, stride = cs
                self.reduces.append((ws, off, nb, stride, cols, acc))
                return True
        return False

    def colsum_into(self, x, rows, cols, ld, acc, at_once=False):
        """acc[c] += sum_r x[r, c] (bias gradient), reduction finished at the end of the job (the
        batched finish adds every accumulator from one workgroup column: an accumulator may appear
        in it ONCE; at_once: finish here instead, for a second sum into the same accumulator)."""
        if self.colsum_from_producer(x, rows, cols, ld, acc):
            return
        ws = self.temp((self.k.colreduce_workspace(rows, cols),), torch.float32)
        if at_once:
            self.emit(self.k.colsum_accumulate(x, rows, cols, ld, acc, ws, defer=0))
            return
        self.emit(self.k.colsum_accumulate(x, rows, cols, ld, None, ws, defer=1))
        self.reduces.append((ws, 0, self.k.colsum_partials(rows), cols, cols, acc))

    def finish_reduces(self):
        """Launches that finish the deferred column reductions.  One batched launch adds every listed
        accumulator from its own workgroups, without atomics: an accumulator that was reduced into
        twice (a parameter used by two layers of the job) goes into a later launch."""
        out, rest = [], list(self.reduces)
        while rest:
            seen, now, later = set(), [], []
            for item in rest:
                key = item[5].data_ptr()
                (later if key in seen else now).append(item)
                seen.add(key)
            out.append(self.k.colreduce_finalize_batch(now))
            rest = later
        return out

    def new_like(self, like, private=False):
        if like.is_contiguous():
            kept = self._kept_for_dw(like.shape, like.dtype)
            if kept is not None:
                return kept
        if private:
            # gradients that outlive this job (they cross a stage boundary) get their own storage
            return self.L.pool.fresh_like(like)
        self._seq += 1
        return self.L.pool.bwd_like(self._seq, like)

    def temp(self, shape, dtype):
        kept = self._kept_for_dw(shape, dtype)
        if kept is not None:
            return kept
        self._seq += 1
        return self.L.pool.bwd_like(self._seq, torch.empty(tuple(shape), dtype=dtype, device="meta"))

    # -- reading -------------------------------------------------------------
    def grad_of(self, val):
        """Accumulated gradient of `val` (None: nothing contributed, i.e. zero)."""
        if val.kind == "base":
            return val.grad
        g = self.grad_of(val.base)
        return None if g is None else val.view_fn(g)

    # -- writing -------------------------------------------------------------
    def _own_base_grad(self, val, zero_fill):
        """Make sure `val` (kind base) has a private, writable gradient buffer."""
        if val.param is not None:
            return self.L.params.grad(val.param)
        self._written(val.grad)
        if val.grad is None:
            val.grad = self.new_like(val.buf, val.boundary)
            val.grad_shared = False
            val.partial_only = True
            if zero_fill:
                self._zero(val.grad)
        elif val.grad_shared:
            fresh = self.new_like(val.buf, val.boundary)
            self.copy(val.grad, fresh)
            val.grad, val.grad_shared = fresh, False
        return val.grad

    def _zero(self, t):
        if is_dense(t):
            self.emit(self.k.fill(t, 0.0, t.numel()))
        else:
            raise Unsupported("zero-fill of a non-dense gradient buffer")

    def _writable(self, val, zero_fill):
        """Gradient tensor laid out like val.buf that may be written in place."""
        if val.kind == "base":
            return self._own_base_grad(val, zero_fill)
        return val.view_fn(self._writable(val.base, zero_fill))

    def grad_target(self, val):
        """-> (dst, prev): write the NEW TOTAL gradient of `val` into dst; prev is the
        total so far (None: nothing yet; `prev is dst`: accumulate in place)."""
        dst, prev = self._grad_target(val)
        self._written(dst)
        return dst, prev

    def _grad_target(self, val):
        if not val.req_grad:
            raise RuntimeError("gradient requested for a value that does not require one: %r" % val)
        if val.kind == "view":
            dst_b, prev_b = self._grad_target(val.base)
            self._pending[id(val)] = dst_b
            return val.view_fn(dst_b), (None if prev_b is None else val.view_fn(prev_b))
        if val.kind == "part":
            parent = val.base
            had_full = self._has_full_contribution(parent)
            pg = self._writable(parent, zero_fill=not val.tiled)
            region = val.view_fn(pg)
            if val.written or had_full:
                return region, region
            return region, None
        if val.param is not None:
            g = self.L.params.grad(val.param)  # AccumulateGrad: always += into the fp32 accumulator
            return g, g
        if val.grad is None:
            return self.new_like(val.buf, val.boundary), None
        if val.grad_shared:
            return self.new_like(val.buf, val.boundary), val.grad
        return val.grad, val.grad

    def _has_full_contribution(self, val):
        if val.kind == "base":
            return val.grad is not None and not val.partial_only
        if val.kind == "view":
            return self._has_full_contribution(val.base)
        return val.written or self._has_full_contribution(val.base)

    def commit(self, val, dst):
        if val.param is not None:
            return
        if val.kind == "view":
            self.commit(val.base, self._pending.pop(id(val)))
        elif val.kind == "part":
            val.written = True
        else:
            if val.grad is not dst:
                val.grad, val.grad_shared = dst, False
            val.partial_only = False

    # -- generic contributions -------------------------------------------------
    def copy(self, src, dst, accumulate=False):
        """dst (=|+=) src for same-shape tensors of any strides / float dtypes."""
        if src.shape != dst.shape:
            raise RuntimeError("copy: shape mismatch %s vs %s" % (tuple(src.shape), tuple(dst.shape)))
        if src.numel() == 0:
            return
        if is_dense(src) and is_dense(dst) and src.stride() == dst.stride():
            n = src.numel()
            if accumulate:
                self.emit(self.k.axpby(dst, 1.0, src, 1.0, dst, n))
            else:
                self.emit(self.k.cast(src, dst, n))
            return
        sizes, ss, ds = collapse_for_copy(src.shape, src.stride(), dst.stride())
        if len(sizes) > 6:
            raise Unsupported("strided copy over %d dimensions" % len(sizes))
        self.emit(self.k.copy_strided(src, ss, dst, ds, sizes, 1 if accumulate else 0))

    def merge(self, tmp, dst, prev):
        """dst = tmp (+ prev): finish a contribution that was computed into a temporary."""
        if prev is None:
            self.copy(tmp, dst)
        elif prev is dst:
            self.copy(tmp, dst, accumulate=True)
        else:
            self.copy(prev, dst)
            self.copy(tmp, dst, accumulate=True)

    def contribute(self, val, t):
        """Add tensor t (val's shape, any strides/dtype) to val's gradient."""
        if not val.req_grad:
            return
        if (val.kind == "base" and val.param is None and not val.boundary and val.grad is None
                and t.dtype == val.buf.dtype and t.stride() == val.buf.stride()):
            val.grad, val.grad_shared, val.partial_only = t, True, False  # alias, no bytes moved
            return
        dst, prev = self.grad_target(val)
        if prev is None:
            self.copy(t, dst)
        elif prev is dst:
            self.copy(t, dst, accumulate=True)
        else:
            if is_dense(t) and is_dense(prev) and t.stride() == prev.stride() == dst.stride():
                self.emit(self.k.axpby(prev, 1.0, t, 1.0, dst, t.numel()))
            else:
                self.copy(prev, dst)
                self.copy(t, dst, accumulate=True)
        self.commit(val, dst)

    def matrix_in(self, t, dtype):
        """t as a row-major matrix of `dtype` (cast / compact into a temp when needed)."""
        if t.dtype == dtype and as_matrix(t) is not None:
            return t
        hit = self._lp.get(t.data_ptr())
        if hit is not None and hit[1].dtype == dtype and hit[1].numel() == t.numel() and t.is_contiguous():
            return hit[1].view(t.shape)
        tmp = self.temp(t.shape, dtype)
        self.copy(t, tmp)
        return tmp


# ---------------------------------------------------------------------------
# the lowerer
# ---------------------------------------------------------------------------
class Lowerer:
    def __init__(self, kernels, device, compute_dtype=None, params=None, pool=None):
        self.kernels = kernels
        self.device = torch.device(device)
        self.cd = compute_dtype or torch.float32
        self.mixed = self.cd != torch.float32
        self.params = params or ParamStore(kernels, self.device)
        self.pool = pool or BufferPool(self.device)
        self._ws = None
        # defer_dw: weight-gradient products of linear layers are left out of the backward jobs and run
        # once per step over all `stack_mbs` micro-batches (the worker builds that job); forward buffers
        # and the gradients those products read are then laid end to end across micro-batches
        self.defer_dw = False
        self.stack_mbs = 1
        self.stack_tag = None   # micro-batch slots lowered under the same tag (input shapes) share stacked allocations
        # loss scaling as the once-per-step weight-gradient products see it: (device scale or None,
        # device overflow flag or None, constant factor); set by the worker
        self.dw_unscale = (None, None, 1.0)

    # -- buffers -------------------------------------------------------------
    def alloc(self, shape, dtype):
        if self.defer_dw:
            self.cur.alloc_seq += 1
            t = self.pool.stacked((self.stack_tag, "f", self.cur.stage, self.cur.alloc_seq), shape, dtype, self.cur.mb,
                                  self.stack_mbs)
        else:
            t = torch.empty(tuple(int(s) for s in shape), dtype=dtype, device=self.device)
        self.cur.fwd_bytes += t.numel() * t.element_size()
        return t

    def workspace(self, rows, cols):
        """fp32 scratch for the two-stage column reductions (shared by every launch of that size)."""
        need = max(1, self.kernels.colreduce_workspace(rows, cols))
        return self.pool.scratch("colreduce_ws", (need,), torch.float32)

    def emit(self, launch):
        self.cur.fwd.append(launch)

    # -- entry points ----------------------------------------------------------
    def lower_forward(self, part_node, mb, input_vals):
        """Build the forward launch list of one stage for one micro-batch.
        `input_vals` are the Vals (or constants) bound to the stage placeholders."""
        prog = StageProgram(part_node.idx, mb)
        self.cur = prog
        gm = part_node.graph_module
        self.env = {}
        self.fused = {}
        placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
        if len(placeholders) != len(input_vals):
            raise RuntimeError("stage %d expects %d inputs, got %d" % (part_node.idx, len(placeholders), len(input_vals)))
        for n, v in zip(placeholders, input_vals):
            self.env[n] = v
            if isinstance(v, Val):
                v.name = v.name or n.name
        prog.inputs = list(input_vals)
        self.patterns, self.pattern_skip = find_rope_patterns(gm)
        for node in gm.graph.nodes:
            if node.op == "placeholder":
                continue
            if node.op == "output":
                res = node.args[0]
                outs = list(res) if isinstance(res, (tuple, list)) else [res]
                prog.outputs = [self.arg(o) for o in outs]
                continue
            first, bytes0 = len(prog.fwd), prog.fwd_bytes
            self.cur_node = node.name
            if node in self.fused:
                self.env[node] = self.fused[node]
            elif node in self.pattern_skip:
                pass  # interior of a matched multi-node pattern, produced by the pattern's root
            else:
                if node in self.patterns:
                    out = lower_rope(self, node, *self.patterns[node])
                else:
                    out = self._handler(node)(self, node)
                self.env[node] = out
                if isinstance(out, Val) and not out.name:
                    out.name = node.name
            if node.op != "get_attr":
                prog.fwd_ranges.append((node.name, first, len(prog.fwd), prog.fwd_bytes - bytes0))
        self.cur = None
        return prog

    def lower_backward(self, prog, output_grads):
        """Build the backward launch list.  `output_grads[i]` is the (preallocated)
        gradient tensor of prog.outputs[i] or None; the tensors are only read."""
        B = BwdCtx(self, prog)
        for v, gs in zip(prog.outputs, output_grads):
            if gs is None or not isinstance(v, Val) or not v.req_grad:
                continue
            for g in ([gs] if torch.is_tensor(gs) else gs):  # several consumers: fan-out sum
                B.contribute(v, g)
        for fn, name in zip(reversed(prog.backward_fns), reversed(prog.backward_nodes)):
            first = len(prog.bwd)
            fn(B)
            prog.bwd_ranges.append((name, first, len(prog.bwd)))
        first = len(prog.bwd)
        B.close_dw()
        prog.bwd.extend(B.finish_reduces())
        if prog.bwd_ranges and len(prog.bwd) > first:   # held-back tail: charged to the job's last node
            prog.bwd_ranges.append((prog.bwd_ranges[-1][0], first, len(prog.bwd)))
        B.compact(prog.bwd_ranges)
        prog.input_grads = []
        for v in prog.inputs:
            if isinstance(v, Val) and v.req_grad and v.param is None:
                prog.input_grads.append(B.grad_of(v))
            else:
                prog.input_grads.append(None)
        for group in prog.tile_groups:
            w = [p.written for p in group]
            if any(w) and not all(w):
                raise RuntimeError("stage %d: a split/unbind piece received no gradient while its siblings did; "
                                   "the unwritten region would hold garbage" % prog.stage)
        prog.backward_fns = []  # closures keep build-time state alive; not needed any more
        return prog

    def lower_deferred_dw(self, progs):
        """The once-per-step weight-gradient job of one stage.  `progs`: the stage's programs, one
        per micro-batch, in micro-batch order.  Product i of every program reads that micro-batch's
        layer-output gradient and layer input; where those lie end to end in memory (equal
        micro-batches, stacked buffers) the micro-batches are ONE product over all their rows:
        one launch and one read-modify-write of the fp32 accumulator instead of one per micro-batch
        (ViT-L: a quarter of a weight-gradient launch was that pass).  Otherwise (ragged batch, an
        operand in a buffer of its own) one product per micro-batch, in micro-batch order.
        Returns the launch list."""
        job = StageProgram(progs[0].stage, None)
        B = BwdCtx(self, job)
        lists = [p.dw_deferred for p in progs]
        if len({tuple(r["name"] for r in recs) for recs in lists}) == 1:
            groups = list(zip(*lists))              # product i of every micro-batch
        else:
            # programs lowered at different times (a slot rebuilt for another shape without the
            # deferral): every program's products on their own
            groups = [(r,) for recs in lists for r in recs]
        stored = set()      # gradients this job has written so far: only the first product into one stores
        for recs in groups:
            r0 = recs[0]
            es = r0["dy"].element_size()
            same = all(r["name"] == r0["name"] and r["wg"] is r0["wg"] and
                       (r["rows"], r["n_out"], r["n_in"], r["ld_dy"], r["ld_x"]) ==
                       (r0["rows"], r0["n_out"], r0["n_in"], r0["ld_dy"], r0["ld_x"]) and
                       r["dy"].dtype == r0["dy"].dtype and r["x"].dtype == r0["x"].dtype for r in recs)
            stacked = same and len(recs) > 1 and r0["rows"] > 0 and all(
                r["dy"].untyped_storage().data_ptr() == r0["dy"].untyped_storage().data_ptr() and
                r["x"].untyped_storage().data_ptr() == r0["x"].untyped_storage().data_ptr() and
                r["dy"].data_ptr() == r0["dy"].data_ptr() + j * r0["rows"] * r0["ld_dy"] * es and
                r["x"].data_ptr() == r0["x"].data_ptr() + j * r0["rows"] * r0["ld_x"] * es
                for j, r in enumerate(recs))
            if stacked:
                n = len(recs)
                dy = torch.as_strided(r0["dy"], (n * r0["rows"], r0["n_out"]), (r0["ld_dy"], 1))
                x = torch.as_strided(r0["x"], (n * r0["rows"], r0["n_in"]), (r0["ld_x"], 1))
                products = [(dy, x, n * r0["rows"])]
            else:
                products = [(r["dy"], r["x"], r["rows"]) for r in recs if r["rows"] > 0]
            # A gradient that nothing else writes is STORED by its (first) product, unscaled and
            # checked for overflow in that product's epilogue: no zero fill, no read of the old
            # value, no unscale pass over it.  Anything else accumulates as every gradient does.
            direct = getattr(self.kernels, "gemm_stores_checked", None)
            whole = direct is not None and len(groups) > 0 and self.params.stored_whole(r0["param"])
            scale, flag, factor = self.dw_unscale
            launches = []
            for i, (dy, x, rows) in enumerate(products):
                kw = dict(M=r0["n_out"], N=r0["n_in"], K=rows, lda=r0["ld_dy"], ldb=r0["ld_x"], ldc=r0["n_in"],
                          a_trans=1, b_trans=1)
                if whole:
                    launch = self.kernels.gemm(dy, x, r0["wg"], beta=int(i > 0 or id(r0["param"]) in stored),
                                               alpha=factor, unscale_by=scale, nonfinite_flag=flag, **kw)
                    if not direct(launch):     # this product runs on a kernel without that epilogue
                        whole = False
                        launches = []
                        break
                else:
                    launch = self.kernels.gemm(dy, x, r0["wg"], beta=1, **kw)
                launches.append(launch)
            if not launches:
                self.params.demote(r0["param"])
                launches = [self.kernels.gemm(dy, x, r0["wg"], beta=1, M=r0["n_out"], N=r0["n_in"], K=rows,
                                              lda=r0["ld_dy"], ldb=r0["ld_x"], ldc=r0["n_in"], a_trans=1, b_trans=1)
                            for dy, x, rows in products]
            elif not whole:
                self.params.demote(r0["param"])
            stored.add(id(r0["param"]))
            for launch in launches:
                B.emit_dw(launch, r0["wg"])
            # the layer's bias gradient: one column sum over all micro-batches' rows where they are
            # stacked, else one per micro-batch (each finished on the spot: same accumulator)
            if len(products) == 1 and all(r.get("bias_grad") is not None for r in recs):
                B.colsum_into(products[0][0], products[0][2], r0["n_out"], r0["ld_dy"], r0["bias_grad"])
            else:
                for r in recs:
                    if r.get("bias_grad") is not None and r["rows"] > 0:
                        B.colsum_into(r["dy"], r["rows"], r["n_out"], r["ld_dy"], r["bias_grad"], at_once=True)
        B.close_dw()
        job.bwd.extend(B.finish_reduces())
        B.compact([])
        return job.bwd

    # -- helpers for handlers ----------------------------------------------------
    def arg(self, a):
        if isinstance(a, torch.fx.Node):
            return self.env[a]
        if isinstance(a, (tuple, list)):
            return type(a)(self.arg(x) for x in a)
        return a

    def add_backward(self, fn):
        self.cur.backward_fns.append(fn)
        self.cur.backward_nodes.append(getattr(self, "cur_node", ""))

    def _handler(self, node):
        if node.op == "call_function":
            h = FUNCTION_HANDLERS.get(node.target)
            if h is None:
                h = FUNCTION_HANDLERS.get(getattr(node.target, "__name__", None))
        elif node.op == "call_method":
            h = METHOD_HANDLERS.get(node.target)
        else:
            h = None
        if h is None:
            raise Unsupported("no HIP lowering for graph node %s (target %s)" % (node.format_node(), node.target))
        return h

    def sole_user(self, node):
        if len(node.users) != 1:
            return None
        return next(iter(node.users))

    def matrix_in(self, t, dtype):
        """Forward-side: t as a matrix of dtype, materialising a saved copy when needed."""
        if t.dtype == dtype and as_matrix(t) is not None:
            return t
        tmp = self.alloc(t.shape, dtype)
        self.copy(t, tmp)
        return tmp

    def copy(self, src, dst):
        if src.numel() == 0:
            return
        if src.dtype.is_floating_point and is_dense(src) and is_dense(dst) and src.stride() == dst.stride():
            self.emit(self.kernels.cast(src, dst, src.numel()))
            return
        sizes, ss, ds = collapse_for_copy(src.shape, src.stride(), dst.stride())
        if len(sizes) > 6:
            raise Unsupported("strided copy over %d dimensions" % len(sizes))
        self.emit(self.kernels.copy_strided(src, ss, dst, ds, sizes, 0))

    def consumers_cast_to_cd(self, node):
        """True when every user of `node` is an op that autocast would feed 16-bit inputs."""
        if not self.mixed or not node.users:
            return False
        for u in node.users:
            if u.op == "call_function" and u.target in CAST_TO_CD_TARGETS:
                continue
            return False
        return True


# ---------------------------------------------------------------------------
# handlers
# ---------------------------------------------------------------------------
def _kw(node, idx, name, default=None):
    if len(node.args) > idx:
        return node.args[idx]
    return node.kwargs.get(name, default)


def _act_of_node(n):
    """(act code) if node n is a supported unary activation, else None."""
    if n.op != "call_function":
        return None
    t = n.target
    if t in (F.gelu, torch._C._nn.gelu):
        approx = n.kwargs.get("approximate", "none")
        return ACT_GELU_TANH if approx == "tanh" else ACT_GELU
    if t in (F.silu,):
        return ACT_SILU
    if t in (F.relu, torch.relu):
        return ACT_RELU
    return None


def _is_add_node(n):
    return n.op == "call_function" and n.target in (operator.add, operator.iadd, torch.add)


def lower_linear(L, node):
    x = L.arg(node.args[0])
    w = L.arg(node.args[1])
    b = L.arg(_kw(node, 2, "bias"))
    cd = L.cd
    K = x.shape[-1]
    N = w.shape[0]
    if w.shape[1] != K:
        raise RuntimeError("linear: weight %s does not match input %s" % (w.shape, x.shape))
    xm = L.matrix_in(x.buf, cd)
    M, _, lda = as_matrix(xm)
    w_cd = L.params.shadow(w.buf, cd) if w.param is not None or not w.req_grad else None
    if w_cd is None:
        raise Unsupported("linear with a non-parameter weight that requires grad")
    if not w_cd.is_contiguous():
        raise Unsupported("linear with a non-contiguous weight")
    b_cd = None if b is None else L.params.shadow(b.buf, cd)
    # dx = dy W reads W along its rows; a transposed shadow keeps the reduction dimension
    # contiguous for that product too (the weight is static within a step, the copy is made once)
    w_t = L.params.shadow_t(w.buf, cd) if (x.req_grad and w.param is not None and M >= 256) else None

    # fusions: linear -> activation, or linear -> (+ residual)
    act, res, out_node = ACT_NONE, None, node
    user = L.sole_user(node)
    if user is not None:
        a = _act_of_node(user)
        gate_of_glu = False
        if a is not None and len(user.users) == 1:
            uu = next(iter(user.users))
            gate_of_glu = (uu.op == "call_function" and uu.target in (operator.mul, torch.mul)
                           and all(isinstance(x, torch.fx.Node) for x in uu.args[:2]))
        if a is not None and user.args[0] is node and not gate_of_glu:
            act, out_node = a, user
        elif _is_add_node(user) and not user.kwargs:
            other = user.args[1] if user.args[0] is node else user.args[0]
            if isinstance(other, torch.fx.Node) and other in L.env and isinstance(L.env[other], Val):
                ov = L.env[other]
                if ov.shape == tuple(x.shape[:-1]) + (N,) and as_matrix(ov.buf) is not None \
                        and ov.dtype.is_floating_point:
                    res, out_node = ov, user
    out_shape = tuple(x.shape[:-1]) + (N,)
    out_dtype = cd if res is None else _dtype_promote(cd, res.dtype)
    out = L.alloc(out_shape, out_dtype)
    h = L.alloc(out_shape, cd) if act != ACT_NONE else None
    kw = dict(M=M, N=N, K=K, lda=lda, ldb=K, ldc=N, bias=b_cd, round_mid=1 if L.mixed else 0)
    if act != ACT_NONE:
        kw.update(aux_out=h, ld_aux_out=N, act=act)
    if res is not None:
        kw.update(residual=res.buf, ld_res=as_matrix(res.buf)[2])
    L.emit(L.kernels.gemm(xm, w_cd, out, **kw))
    defer_dw = L.defer_dw and w.req_grad and w.param is not None
    if defer_dw:
        L.cur.dw_sigs.add((M * N, cd))
    req = x.req_grad or w.req_grad or (b is not None and b.req_grad) or (res is not None and res.req_grad)
    outv = Val(out, req_grad=req, name=out_node.name)
    if L.mixed and out_dtype == torch.float32 and act == ACT_NONE:
        # backward reads this value's gradient as a 16-bit matrix (and sums its columns for the
        # bias): whoever produces that gradient may write it in that form as well
        outv.lp_grad = dict(colsum=b is not None and b.req_grad and b.param is not None, cols=N)
    if act != ACT_NONE:
        outv.preact = (act, h)
    if out_node is not node:
        L.fused[out_node] = outv
    x_users = len(node.args[0].users) if isinstance(node.args[0], torch.fx.Node) else 0

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        if res is not None:
            B.contribute(res, g)
        if act != ACT_NONE and not outv.grad_is_preact:
            gm_ = B.matrix_in(g, cd)
            dy = B.temp(out_shape, cd)
            if not (gm_.is_contiguous() and h.is_contiguous()):
                raise Unsupported("activation backward on non-contiguous gradient")
            B.emit(B.k.act_bwd(gm_, h, dy, act, dy.numel()))
        else:
            dy = B.matrix_in(g, cd)
        _, _, ld_dy = as_matrix(dy)
        if w.req_grad and w.param is not None:
            # dW = dY^T X reduces over the token rows, the strided dimension of both operands: the
            # GEMM reads them with transposing LDS reads (no transposed copies in memory)
            wg = L.params.grad(w.param, (B.program.stage, node.name) if defer_dw else None)
            if defer_dw:
                # left to the stage's once-per-step job: over all micro-batches the operands form one
                # product with that many times the reduction length, and one pass over the accumulator
                B.program.dw_deferred.append(dict(name=node.name, dy=dy, x=xm, wg=wg, param=w.param, rows=M, n_out=N,
                                                  n_in=K, ld_dy=ld_dy, ld_x=lda))
            else:
                B.emit_dw(B.k.gemm(dy, xm, wg, M=N, N=K, K=M, lda=ld_dy, ldb=lda, ldc=K, a_trans=1, b_trans=1, beta=1), wg)
        if b is not None and b.req_grad and b.param is not None:
            bg = L.params.grad(b.param)
            if defer_dw and w.req_grad and w.param is not None:
                # the bias gradient is the column sum of the same dy: with the weight gradient, once per step
                if not B.colsum_from_producer(dy, M, N, ld_dy, bg):
                    B.program.dw_deferred[-1]["bias_grad"] = bg
            else:
                B.colsum_into(dy, M, N, ld_dy, bg)
        if x.req_grad:
            dst, prev = B.grad_target(x)
            dm = as_matrix(dst)
            if w_t is not None:
                wb, kw2 = w_t, dict(M=M, N=K, K=N, lda=ld_dy, ldb=N, b_trans=0)
            else:
                wb, kw2 = w_cd, dict(M=M, N=K, K=N, lda=ld_dy, ldb=K, b_trans=1)
            if x.preact is not None and x_users == 1 and prev is None:
                kw2.update(dact=x.preact[0], aux_in=x.preact[1], ld_aux_in=K)
                x.grad_is_preact = True
            if dm is not None:
                if prev is dst:
                    kw2["beta"] = 1
                elif prev is not None:
                    pm = as_matrix(prev)
                    if pm is None:
                        raise Unsupported("accumulating into a non-matrix gradient")
                    kw2.update(residual=prev, ld_res=pm[2])
                launch = B.k.gemm(dy, wb, dst, ldc=dm[2], **kw2)
                B.emit(launch)
                B.commit(x, dst)
                if ("dact" in kw2 and hasattr(B.k, "gemm_attach_colsum") and dm[2] == K
                        and os.environ.get("PFEIFE_EPILOGUE_COLSUM", "1") != "0"):
                    # dst now holds the gradient of the producing layer's pre-activation: its column sums
                    # are that layer's bias gradient, and the product's epilogue can leave them behind
                    cs = B.k.gemm_attach_colsum(launch, B.temp)
                    if cs is not None:
                        B.register_lp(dst, dst, colsum=cs)
            else:
                # target is not a plain matrix (e.g. a permuted view): go through a temp
                tmp = B.temp(tuple(x.shape), x.dtype)
                B.emit(B.k.gemm(dy, wb, tmp, ldc=K, **kw2))
                if prev is None:
                    B.copy(tmp, dst)
                elif prev is dst:
                    B.copy(tmp, dst, accumulate=True)
                else:
                    B.copy(prev, dst)
                    B.copy(tmp, dst, accumulate=True)
                B.commit(x, dst)

    if req:
        L.add_backward(bwd)
    return outv if out_node is node else outv


def lower_layer_norm(L, node, rms=False):
    x = L.arg(node.args[0])
    shape = _kw(node, 1, "normalized_shape")
    gamma = L.arg(_kw(node, 2, "weight"))
    if rms:
        beta = None
        eps = _kw(node, 3, "eps", None)
        if eps is None:
            eps = torch.finfo(torch.float32).eps
    else:
        beta = L.arg(_kw(node, 3, "bias"))
        eps = _kw(node, 4, "eps", 1e-5)
    if len(tuple(shape)) != 1 or shape[0] != x.shape[-1]:
        raise Unsupported("normalisation over other than the last dimension: %s" % (shape,))
    if gamma is None:
        raise Unsupported("normalisation without a weight")
    d = x.shape[-1]
    if not x.buf.is_contiguous():
        raise Unsupported("normalisation of a non-contiguous input")
    rows = x.buf.numel() // d
    y_dtype = L.cd if L.consumers_cast_to_cd(node) else (torch.float32 if L.mixed else x.dtype)
    y = L.alloc(x.shape, y_dtype)
    rstd = L.alloc((rows,), torch.float32)
    g32 = gamma.buf if gamma.dtype == torch.float32 else L.params.shadow(gamma.buf, torch.float32)
    if rms:
        mean = None
        L.emit(L.kernels.rmsnorm_fwd(x.buf, g32, y, rstd, rows, d, float(eps)))
    else:
        mean = L.alloc((rows,), torch.float32)
        b32 = None if beta is None else (beta.buf if beta.dtype == torch.float32 else L.params.shadow(beta.buf, torch.float32))
        L.emit(L.kernels.layernorm_fwd(x.buf, g32, b32, y, mean, rstd, rows, d, float(eps)))
    req = x.req_grad or gamma.req_grad or (beta is not None and beta.req_grad)
    outv = Val(y, req_grad=req)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        if not g.is_contiguous():
            t = B.temp(g.shape, g.dtype)
            B.copy(g, t)
            g = t
        dgamma = L.params.grad(gamma.param) if gamma.req_grad and gamma.param is not None else None
        dbeta = L.params.grad(beta.param) if beta is not None and beta.req_grad and beta.param is not None else None
        want = dgamma is not None or dbeta is not None
        ws = B.temp((B.k.colreduce_workspace(rows, d),), torch.float32) if want else None
        if x.req_grad:
            dst, prev = B.grad_target(x)
            if not dst.is_contiguous() or (prev is not None and not prev.is_contiguous()):
                raise Unsupported("normalisation backward into a non-contiguous gradient")
        else:
            dst, prev = B.temp(x.shape, x.dtype), None
        lp_info = getattr(x, "lp_grad", None)
        if (lp_info is not None and x.req_grad and L.mixed and dst.dtype == torch.float32 and d % 8 == 0
                and lp_info["cols"] == d and hasattr(B.k, "norm_bwd_fused")):
            # the layer before x reads this gradient as a 16-bit matrix and sums its columns for
            # its bias: written here, while the values are in registers
            want_cs = bool(lp_info["colsum"]) and d <= 2048
            stride = (3 if want_cs else 2) * d
            nb = B.k.norm_bwd_partials(rows)
            ws = B.temp((nb * stride,), torch.float32) if (want or want_cs) else None
            lp = B.temp(x.shape, L.cd)
            B.emit(B.k.norm_bwd_fused(g, x.buf, g32, mean, rstd, prev, dst, lp, ws, rows, d, want, want_cs))
            B.register_lp(dst, lp, (ws, 2 * d, nb, stride) if want_cs else None)
        else:
            stride = 2 * d
            nb = B.k.norm_bwd_partials(rows) if want else 0
            if rms:
                B.emit(B.k.rmsnorm_bwd(g, x.buf, g32, rstd, prev, dst, None, ws, rows, d, defer=1 if want else 0))
            else:
                B.emit(B.k.layernorm_bwd(g, x.buf, g32, mean, rstd, prev, dst, None, None, ws, rows, d,
                                         defer=1 if want else 0))
        if want:
            if dgamma is not None:
                B.reduces.append((ws, 0, nb, stride, d, dgamma))
            if dbeta is not None:
                B.reduces.append((ws, d, nb, stride, d, dbeta))
        if x.req_grad:
            B.commit(x, dst)

    if req:
        L.add_backward(bwd)
    return outv


def lower_rms_norm(L, node):
    return lower_layer_norm(L, node, rms=True)


def lower_sdpa(L, node):
    q, k, v = (L.arg(a) for a in node.args[:3])
    mask = _kw(node, 3, "attn_mask")
    drop = _kw(node, 4, "dropout_p", 0.0)
    causal = bool(_kw(node, 5, "is_causal", False))
    scale = _kw(node, 6, "scale", None)
    if mask is not None:
        raise Unsupported("scaled_dot_product_attention with an explicit mask")
    if drop:
        raise Unsupported("attention dropout")
    if node.kwargs.get("enable_gqa"):
        raise Unsupported("grouped-query attention")
    cd = L.cd
    if q.buf.dim() != 4:
        raise Unsupported("attention on %d-d tensors" % q.buf.dim())
    Bn, H, Tq, hd = q.shape
    Tk = k.shape[2]
    if k.shape != (Bn, H, Tk, hd) or v.shape[:3] != (Bn, H, Tk):
        raise Unsupported("attention with mismatched head layout %s %s %s" % (q.shape, k.shape, v.shape))
    if causal and Tq != Tk:
        # F.scaled_dot_product_attention aligns a non-square causal mask at the top-left corner
        # (tril(0)); the attention and softmax kernels align it bottom-right (key j visible to
        # query i iff j <= i + Tk - Tq, the decode convention).  They agree only when Tq == Tk.
        raise Unsupported("is_causal attention with Tq=%d != Tk=%d" % (Tq, Tk))
    hv = v.shape[3]
    scale = float(scale) if scale is not None else 1.0 / math.sqrt(hd)
    Tkp = (Tk + 7) // 8 * 8

    def head_tensor(val):
        t = val.buf
        if t.dtype != cd or t.stride(3) != 1 or any(s % 8 for s in t.stride()[:3] if cd != torch.float32):
            c = L.alloc(t.shape, cd)
            L.copy(t, c)
            return c
        return t

    qt, kt, vt = head_tensor(q), head_tensor(k), head_tensor(v)
    req = q.req_grad or k.req_grad or v.req_grad
    kern = L.kernels
    if L.mixed and hv == hd and hd % 8 == 0 and hd <= getattr(kern, "MAX_FUSED_HEAD_DIM", 0):
        return _lower_sdpa_fused(L, (q, k, v), (qt, kt, vt), (Bn, H, Tq, Tk, hd), scale, causal, req)
    S = L.pool.scratch("attn_s", (Bn, H, Tq, Tkp), torch.float32)
    P = L.alloc((Bn, H, Tq, Tkp), cd)
    O = L.alloc((Bn, Tq, H, hv), cd)           # token-major, so that transpose(1,2).reshape is a view
    Ov = O.permute(0, 2, 1, 3)
    bs = lambda t: (t.stride(0), t.stride(1))
    L.emit(kern.gemm(qt, kt, S, M=Tq, N=Tk, K=hd, lda=qt.stride(2), ldb=kt.stride(2), ldc=Tkp, batch=(Bn, H),
                     sa=bs(qt), sb=bs(kt), sc=bs(S), alpha=scale))
    L.emit(kern.softmax_fwd(S, Tkp, P, Tkp, Bn * H * Tq, Tk, Tq, 1 if causal else 0))
    L.emit(kern.gemm(P, vt, Ov, M=Tq, N=hv, K=Tk, lda=Tkp, ldb=vt.stride(2), ldc=Ov.stride(2), b_trans=1,
                     batch=(Bn, H), sa=bs(P), sb=bs(vt), sc=bs(Ov)))
    outv = Val(Ov, req_grad=req)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        if g.dtype != cd or g.stride(3) != 1:
            t = B.new_like(Ov)
            B.copy(g, t)
            g = t
        dP = L.pool.scratch("attn_dp", (Bn, H, Tq, Tkp), torch.float32)
        dS = L.pool.scratch("attn_ds", (Bn, H, Tq, Tkp), cd)
        kb = B.k
        B.emit(kb.gemm(g, vt, dP, M=Tq, N=Tk, K=hv, lda=g.stride(2), ldb=vt.stride(2), ldc=Tkp, batch=(Bn, H),
                       sa=bs(g), sb=bs(vt), sc=bs(dP)))
        B.emit(kb.softmax_bwd(dP, Tkp, P, Tkp, dS, Tkp, Bn * H * Tq, Tk, scale))

        def into(val, emit_fn):
            if not val.req_grad:
                return
            dst, prev = B.grad_target(val)
            direct = dst.dtype == cd and dst.stride(3) == 1 and (prev is None or prev is dst)
            if direct:
                emit_fn(dst, 1 if prev is dst else 0)
                B.commit(val, dst)
            else:
                tmp = B.temp(val.shape, cd)
                emit_fn(tmp, 0)
                B.merge(tmp, dst, prev)
                B.commit(val, dst)

        # dQ = dS K ; dK = dS^T Q ; dV = P^T dO
        into(q, lambda dst, beta: B.emit(kb.gemm(dS, kt, dst, M=Tq, N=hd, K=Tk, lda=Tkp, ldb=kt.stride(2),
                                                  ldc=dst.stride(2), b_trans=1, batch=(Bn, H), sa=bs(dS), sb=bs(kt),
                                                  sc=bs(dst), beta=beta)))
        into(k, lambda dst, beta: B.emit(kb.gemm(dS, qt, dst, M=Tk, N=hd, K=Tq, lda=Tkp, ldb=qt.stride(2),
                                                  ldc=dst.stride(2), a_trans=1, b_trans=1, batch=(Bn, H), sa=bs(dS),
                                                  sb=bs(qt), sc=bs(dst), beta=beta)))
        into(v, lambda dst, beta: B.emit(kb.gemm(P, g, dst, M=Tk, N=hv, K=Tq, lda=Tkp, ldb=g.stride(2),
                                                  ldc=dst.stride(2), a_trans=1, b_trans=1, batch=(Bn, H), sa=bs(P),
                                                  sb=bs(g), sc=bs(dst), beta=beta)))

    if req:
        L.add_backward(bwd)
    return outv


def _lower_sdpa_fused(L, vals, tensors, dims, scale, causal, req):
    """softmax(QK^T)V as one kernel (no score matrix in memory) and a three-kernel backward."""
    q, k, v = vals
    qt, kt, vt = tensors
    Bn, H, Tq, Tk, hd = dims
    cd = L.cd
    O = L.alloc((Bn, Tq, H, hd), cd)            # token-major, so that transpose(1,2).reshape is a view
    Ov = O.permute(0, 2, 1, 3)
    lse = L.alloc((Bn, H, Tq), torch.float32)
    L.emit(L.kernels.attention_fwd(qt, kt, vt, Ov, lse, scale, causal))
    outv = Val(Ov, req_grad=req)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        if g.dtype != cd or g.stride(3) != 1 or any(s % 8 for s in g.stride()[:3]):
            t = B.new_like(Ov)
            B.copy(g, t)
            g = t
        delta = L.pool.scratch("attn_delta", (Bn, H, Tq), torch.float32)
        plan = []
        outs = []
        for val, like in ((q, qt), (k, kt), (v, vt)):
            if val.req_grad:
                dst, prev = B.grad_target(val)
                direct = (prev is None and dst.dtype == cd and dst.stride(3) == 1
                          and all(s % 4 == 0 for s in dst.stride()[:3]))
                buf = dst if direct else B.temp(val.shape, cd)
                plan.append((val, dst, prev, buf, direct))
            else:
                buf = B.temp(val.shape, cd)
            outs.append(buf)
        B.emit(B.k.attention_bwd(qt, kt, vt, Ov, g, lse, delta, outs[0], outs[1], outs[2], scale, causal))
        for val, dst, prev, buf, direct in plan:
            if not direct:
                B.merge(buf, dst, prev)
            B.commit(val, dst)

    if req:
        L.add_backward(bwd)
    return outv


def lower_conv2d(L, node):
    x = L.arg(node.args[0])
    w = L.arg(node.args[1])
    b = L.arg(_kw(node, 2, "bias"))
    stride = _kw(node, 3, "stride", (1, 1))
    padding = _kw(node, 4, "padding", (0, 0))
    dilation = _kw(node, 5, "dilation", (1, 1))
    groups = _kw(node, 6, "groups", 1)
    pair = lambda v: (v, v) if isinstance(v, int) else tuple(v)
    stride, padding, dilation = pair(stride), pair(padding), pair(dilation)
    O, C, kh, kw_ = w.shape
    if (groups == 1 and dilation == (1, 1) and stride == (1, 1) and kh == kw_ and kh in (1, 3)
            and padding == (kh // 2, kh // 2)):
        return _lower_conv_same(L, x, w, b, kh)
    if groups != 1 or dilation != (1, 1) or padding != (0, 0) or stride != (kh, kw_):
        raise Unsupported("conv2d other than a patch projection (kernel == stride, no padding) or a 1x1 / 3x3 "
                          "stride-1 'same' convolution")
    Bn, Cx, H, W = x.shape
    if Cx != C or H % kh or W % kw_:
        raise Unsupported("conv2d patch projection with ragged image size")
    Hp, Wp = H // kh, W // kw_
    cd = L.cd
    cols = L.alloc((Bn * Hp * Wp, C * kh * kw_), cd)
    xs = x.buf.stride()
    src_strides = (xs[0], xs[2] * kh, xs[3] * kw_, xs[1], xs[2], xs[3])
    sizes = (Bn, Hp, Wp, C, kh, kw_)
    cview = cols.view(Bn, Hp, Wp, C, kh, kw_)
    s2, ss2, ds2 = collapse_for_copy(sizes, src_strides, cview.stride())
    L.emit(L.kernels.copy_strided(x.buf, ss2, cols, ds2, s2, 0))
    M, K, N = Bn * Hp * Wp, C * kh * kw_, O
    w_cd = L.params.shadow(w.buf, cd)
    b_cd = None if b is None else L.params.shadow(b.buf, cd)
    out = L.alloc((Bn, Hp, Wp, O), cd)
    L.emit(L.kernels.gemm(cols, w_cd, out, M=M, N=N, K=K, lda=K, ldb=K, ldc=N, bias=b_cd,
                          round_mid=1 if L.mixed else 0))
    req = x.req_grad or w.req_grad or (b is not None and b.req_grad)
    outv = Val(out.permute(0, 3, 1, 2), req_grad=req)   # logical NCHW, channels-last memory

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        gm_ = g.permute(0, 2, 3, 1)
        dy = B.matrix_in(gm_, cd)
        _, _, ld_dy = as_matrix(dy)
        if w.req_grad and w.param is not None:
            B.emit(B.k.gemm(dy, cols, L.params.grad(w.param), M=N, N=K, K=M, lda=ld_dy, ldb=K, ldc=K, a_trans=1,
                            b_trans=1, beta=1))
        if b is not None and b.req_grad and b.param is not None:
            B.colsum_into(dy, M, N, ld_dy, L.params.grad(b.param))
        if x.req_grad:
            dcols = B.temp((M, K), cd)
            B.emit(B.k.gemm(dy, w_cd, dcols, M=M, N=K, K=N, lda=ld_dy, ldb=K, ldc=K, b_trans=1))
            dst, prev = B.grad_target(x)
            dview = torch.as_strided(dst, sizes, tuple(
                s * m for s, m in zip((dst.stride(0), dst.stride(2), dst.stride(3), dst.stride(1), dst.stride(2),
                                       dst.stride(3)), (1, kh, kw_, 1, 1, 1))), dst.storage_offset())
            if prev is not None and prev is not dst:
                B.copy(prev, dst)
            B.copy(dcols.view(sizes), dview, accumulate=prev is not None)
            B.commit(x, dst)

    if req:
        L.add_backward(bwd)
    return outv



def as_nhwc(L, t, dtype=None):
    """Channels-last contiguous [B, H, W, C] tensor holding the logical NCHW tensor t (a view when
    t already lives in channels-last memory with the wanted dtype, a copy kernel otherwise)."""
    dtype = dtype or t.dtype
    p = t.permute(0, 2, 3, 1)
    if p.is_contiguous() and t.dtype == dtype:
        return p
    out = L.alloc(p.shape, dtype)
    L.copy(p, out)
    return out


def _grad_nhwc(B, g, dtype):
    """Gradient of a logical-NCHW value as a contiguous channels-last matrix source."""
    p = g.permute(0, 2, 3, 1)
    if p.is_contiguous() and g.dtype == dtype:
        return p
    t = B.temp(p.shape, dtype)
    B.copy(p, t)
    return t


def _lower_conv_same(L, x, w, b, k):
    """1x1 or 3x3 stride-1 'same' convolution as one GEMM over channels-last rows
    (3x3: the nine shifted windows of a zero-bordered copy are laid side by side first)."""
    cd = L.cd
    Bn, C, H, W = x.shape
    O = w.shape[0]
    M = Bn * H * W
    xn = as_nhwc(L, x.buf, cd)
    if k == 1:
        cols, Kc = xn.reshape(M, C), C
        w_cd = L.params.shadow(w.buf, cd).reshape(O, C)
    else:
        Kc = 9 * C
        padded = torch.zeros((Bn, H + 2, W + 2, C), dtype=cd, device=L.device)  # border stays zero for good
        L.cur.fwd_bytes += padded.numel() * padded.element_size()
        L.copy(xn, padded[:, 1:H + 1, 1:W + 1, :])
        cols = L.alloc((M, Kc), cd)
        ps = padded.stride()
        win = torch.as_strided(padded, (Bn, H, W, 3, 3, C), (ps[0], ps[1], ps[2], ps[1], ps[2], 1))
        L.copy(win, cols.view(Bn, H, W, 3, 3, C))
        w_cd = L.params.shadow_perm(w.buf, cd, (0, 2, 3, 1)).reshape(O, Kc)
    b_cd = None if b is None else L.params.shadow(b.buf, cd)
    out = L.alloc((Bn, H, W, O), cd)
    L.emit(L.kernels.gemm(cols, w_cd, out, M=M, N=O, K=Kc, lda=Kc, ldb=Kc, ldc=O, bias=b_cd,
                          round_mid=1 if L.mixed else 0))
    req = x.req_grad or w.req_grad or (b is not None and b.req_grad)
    outv = Val(out.permute(0, 3, 1, 2), req_grad=req)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        dy = _grad_nhwc(B, g, cd).reshape(M, O)
        if w.req_grad and w.param is not None:
            wg = L.params.grad(w.param)
            if k == 1:
                B.emit(B.k.gemm(dy, cols, wg, M=O, N=Kc, K=M, lda=O, ldb=Kc, ldc=Kc, a_trans=1, b_trans=1, beta=1))
            else:
                tmp = B.temp((O, 3, 3, C), torch.float32)
                B.emit(B.k.gemm(dy, cols, tmp, M=O, N=Kc, K=M, lda=O, ldb=Kc, ldc=Kc, a_trans=1, b_trans=1))
                B.copy(tmp, wg.permute(0, 2, 3, 1), accumulate=True)
        if b is not None and b.req_grad and b.param is not None:
            B.colsum_into(dy, M, O, O, L.params.grad(b.param))
        if x.req_grad:
            dst, prev = B.grad_target(x)
            dstn = dst.permute(0, 2, 3, 1)
            if k == 1:
                direct = prev is None and dstn.is_contiguous()
                t = dstn if direct else B.temp((Bn, H, W, C), x.dtype)
                B.emit(B.k.gemm(dy, w_cd, t, M=M, N=C, K=O, lda=O, ldb=C, ldc=C, b_trans=1))
                if not direct:
                    B.merge(t, dstn, None if prev is None else prev.permute(0, 2, 3, 1))
            else:
                dcols = B.temp((M, Kc), cd)
                B.emit(B.k.gemm(dy, w_cd, dcols, M=M, N=Kc, K=O, lda=O, ldb=Kc, ldc=Kc, b_trans=1))
                dpad = B.temp((Bn, H + 2, W + 2, C), torch.float32)
                B.emit(B.k.fill(dpad, 0.0, dpad.numel()))
                dc = dcols.view(Bn, H, W, 3, 3, C)
                for i in range(3):
                    for j in range(3):   # nine bijective shifted adds, one after the other on the stream
                        B.copy(dc[:, :, :, i, j, :], dpad[:, i:i + H, j:j + W, :], accumulate=True)
                B.merge(dpad[:, 1:H + 1, 1:W + 1, :], dstn, None if prev is None else prev.permute(0, 2, 3, 1))
            B.commit(x, dst)

    if req:
        L.add_backward(bwd)
    return outv


def lower_group_norm(L, node):
    x = L.arg(node.args[0])
    groups = int(_kw(node, 1, "num_groups"))
    gamma = L.arg(_kw(node, 2, "weight"))
    beta = L.arg(_kw(node, 3, "bias"))
    eps = float(_kw(node, 4, "eps", 1e-5))
    if x.buf.dim() != 4 or gamma is None or beta is None:
        raise Unsupported("group_norm other than affine on [B, C, H, W]")
    Bn, C, H, W = x.shape
    xn = as_nhwc(L, x.buf)
    # fp32 result under autocast; written in the compute dtype when it only feeds matrix products,
    # directly or through one activation
    users = list(node.users)
    to_cd = L.consumers_cast_to_cd(node) or (
        L.mixed and len(users) == 1 and _act_of_node(users[0]) is not None and L.consumers_cast_to_cd(users[0]))
    y_dtype = L.cd if to_cd else (torch.float32 if L.mixed else x.dtype)
    y = L.alloc((Bn, H, W, C), y_dtype)
    mean = L.alloc((Bn * groups,), torch.float32)
    rstd = L.alloc((Bn * groups,), torch.float32)
    g32 = gamma.buf if gamma.dtype == torch.float32 else L.params.shadow(gamma.buf, torch.float32)
    b32 = beta.buf if beta.dtype == torch.float32 else L.params.shadow(beta.buf, torch.float32)
    L.emit(L.kernels.groupnorm_fwd(xn, g32, b32, y, mean, rstd, Bn, H * W, C, groups, eps))
    req = x.req_grad or gamma.req_grad or beta.req_grad
    outv = Val(y.permute(0, 3, 1, 2), req_grad=req)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        gn = _grad_nhwc(B, g, g.dtype)
        ws = B.temp((B.k.groupnorm_workspace(Bn, C, groups),), torch.float32)
        if x.req_grad:
            dst, prev = B.grad_target(x)
            dstn = dst.permute(0, 2, 3, 1)
            direct = prev is None and dstn.is_contiguous()
            t = dstn if direct else B.temp((Bn, H, W, C), x.dtype)
        else:
            t = B.temp((Bn, H, W, C), x.dtype)
        B.emit(B.k.groupnorm_bwd(gn, xn, g32, mean, rstd, t, None, None, ws, Bn, H * W, C, groups, defer=1))
        if gamma.req_grad and gamma.param is not None:
            B.reduces.append((ws, 0, Bn, 2 * C, C, L.params.grad(gamma.param)))
        if beta.req_grad and beta.param is not None:
            B.reduces.append((ws, C, Bn, 2 * C, C, L.params.grad(beta.param)))
        if x.req_grad:
            if not direct:
                B.merge(t, dstn, None if prev is None else prev.permute(0, 2, 3, 1))
            B.commit(x, dst)

    if req:
        L.add_backward(bwd)
    return outv


def _view_handler(fn_of_node):
    """Builds a handler for an op that is a pure view of its first argument."""

    def handler(L, node):
        x = L.arg(node.args[0])
        if not isinstance(x, Val):
            raise Unsupported("view of a non-tensor: %s" % node.format_node())
        fn = fn_of_node(L, node)
        out = fn(x.buf)
        if out.untyped_storage().data_ptr() != x.buf.untyped_storage().data_ptr():
            # the op had to copy (reshape of a non-viewable layout): materialise with the copy kernel
            shape = tuple(out.shape)
            dense = L.alloc(x.shape, x.dtype)
            L.copy(x.buf, dense)
            outbuf = dense.view(shape)
            outv = Val(outbuf, req_grad=x.req_grad)

            def bwd(B):
                g = B.grad_of(outv)
                if g is not None:
                    B.contribute(x, g.reshape(x.shape) if g.is_contiguous() else _compact(B, g).view(x.shape))

            if x.req_grad:
                L.add_backward(bwd)
            return outv
        return Val(out, req_grad=x.req_grad, kind="view", base=x, view_fn=fn)

    return handler


def _compact(B, g):
    t = B.temp(g.shape, g.dtype)
    B.copy(g, t)
    return t


def _shape_args(L, node):
    a = [L.arg(v) for v in node.args[1:]]
    if len(a) == 1 and isinstance(a[0], (tuple, list, torch.Size)):
        a = list(a[0])
    return tuple(int(v) for v in a)


lower_reshape = _view_handler(lambda L, n: (lambda t, s=_shape_args(L, n): t.reshape(s)))
lower_view = _view_handler(lambda L, n: (lambda t, s=_shape_args(L, n): t.view(s)))
lower_permute = _view_handler(lambda L, n: (lambda t, s=_shape_args(L, n): t.permute(s)))
lower_transpose = _view_handler(lambda L, n: (lambda t, a=int(n.args[1]), b=int(n.args[2]): t.transpose(a, b)))
lower_flatten = _view_handler(
    lambda L, n: (lambda t, a=int(_kw(n, 1, "start_dim", 0)), b=int(_kw(n, 2, "end_dim", -1)): t.flatten(a, b)))
lower_unsqueeze = _view_handler(lambda L, n: (lambda t, d=int(n.args[1]): t.unsqueeze(d)))
lower_squeeze = _view_handler(
    lambda L, n: (lambda t, d=(n.args[1] if len(n.args) > 1 else None): t.squeeze() if d is None else t.squeeze(d)))


def lower_contiguous(L, node):
    x = L.arg(node.args[0])
    if x.buf.is_contiguous():
        return Val(x.buf, req_grad=x.req_grad, kind="view", base=x, view_fn=lambda t: t)
    dense = L.alloc(x.shape, x.dtype)
    L.copy(x.buf, dense)
    outv = Val(dense, req_grad=x.req_grad)

    def bwd(B):
        g = B.grad_of(outv)
        if g is not None:
            B.contribute(x, g)

    if x.req_grad:
        L.add_backward(bwd)
    return outv


def _chain_single_user(node):
    """True when node and the chain of view nodes above it each have exactly one user."""
    n = node
    while isinstance(n, torch.fx.Node) and n.op in ("call_method", "call_function"):
        if len(n.users) != 1:
            return False
        name = n.target if n.op == "call_method" else getattr(n.target, "__name__", "")
        if name not in ("reshape", "view", "permute", "transpose", "flatten", "unsqueeze", "squeeze"):
            return True
        n = n.args[0]
    return True


def lower_unbind(L, node):
    x = L.arg(node.args[0])
    dim = int(_kw(node, 1, "dim", 0))
    n = x.shape[dim]
    all_used = len(node.users) == n and all(
        u.op == "call_function" and u.target is operator.getitem and len(u.users) > 0 for u in node.users)
    tiled = all_used and _chain_single_user(node.args[0]) and len(node.args[0].users) == 1
    parts = []
    for i in range(n):
        fn = (lambda t, i=i: t.select(dim, i))
        p = Val(fn(x.buf), req_grad=x.req_grad, kind="part", base=x, view_fn=fn)
        p.tiled = tiled
        parts.append(p)
    if tiled:
        L.cur.tile_groups.append(parts)
    return parts


def lower_split_like(L, node, pieces_fn):
    x = L.arg(node.args[0])
    bufs = pieces_fn(x.buf)
    n_total = sum(1 for _ in bufs)
    all_used = len(node.users) == n_total and all(
        u.op == "call_function" and u.target is operator.getitem and len(u.users) > 0 for u in node.users)
    tiled = all_used and _chain_single_user(node.args[0]) and len(node.args[0].users) == 1
    parts = []
    for i in range(n_total):
        fn = (lambda t, i=i: pieces_fn(t)[i])
        p = Val(bufs[i], req_grad=x.req_grad, kind="part", base=x, view_fn=fn)
        p.tiled = tiled
        parts.append(p)
    if tiled:
        L.cur.tile_groups.append(parts)
    return parts


def lower_chunk(L, node):
    n = int(node.args[1])
    dim = int(_kw(node, 2, "dim", 0))
    return lower_split_like(L, node, lambda t: t.chunk(n, dim))


def lower_split(L, node):
    sz = node.args[1]
    dim = int(_kw(node, 2, "dim", 0))
    return lower_split_like(L, node, lambda t: t.split(sz, dim))


def lower_getitem(L, node):
    src = L.arg(node.args[0])
    idx = node.args[1]
    if isinstance(src, (list, tuple)):
        return src[idx]
    if not isinstance(src, Val):
        raise Unsupported("getitem on %s" % type(src))
    idx_t = idx if isinstance(idx, tuple) else (idx,)
    for i in idx_t:
        if not (isinstance(i, (int, slice)) or i is None or i is Ellipsis):
            raise Unsupported("advanced indexing is not lowered: %s" % (idx,))
    fn = (lambda t, idx=idx: t[idx])
    out = fn(src.buf)
    full = out.numel() == src.buf.numel()
    return Val(out, req_grad=src.req_grad, kind="view" if full else "part", base=src, view_fn=fn)


def lower_expand(L, node):
    x = L.arg(node.args[0])
    sizes = _shape_args(L, node)
    out = x.buf.expand(*sizes)
    if out.numel() == x.buf.numel():
        return Val(out, req_grad=x.req_grad, kind="view", base=x, view_fn=lambda t: t.expand(*sizes))
    # broadcasting view; its gradient is a sum over the expanded (leading) dimensions
    lead = out.dim() - x.buf.dim()
    exp_dims = [i for i in range(out.dim()) if i < lead or (x.buf.shape[i - lead] == 1 and out.shape[i] != 1)]
    inner_start = max(exp_dims) + 1
    if exp_dims != list(range(inner_start)) and any(out.shape[i] != 1 for i in range(inner_start) if i not in exp_dims):
        raise Unsupported("expand over non-leading dimensions: %s -> %s" % (x.shape, sizes))
    outv = Val(out, req_grad=x.req_grad)
    rows = 1
    for i in range(inner_start):
        rows *= out.shape[i]
    cols = out.numel() // rows

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        gc = B.matrix_in(g.reshape(rows, cols) if g.is_contiguous() else _compact(B, g).view(rows, cols), torch.float32)
        dst, prev = B.grad_target(x)
        if dst.dtype != torch.float32 or not dst.is_contiguous():
            raise Unsupported("expand backward into a non-fp32 gradient")
        if prev is None:
            B.emit(B.k.fill(dst, 0.0, dst.numel()))
        elif prev is not dst:
            B.copy(prev, dst)
        B.emit(B.k.colsum_accumulate(gc, rows, cols, as_matrix(gc)[2], dst, L.workspace(rows, cols)))
        B.commit(x, dst)

    if x.req_grad:
        L.add_backward(bwd)
    return outv


def lower_cat(L, node):
    tensors = L.arg(node.args[0])
    dim = int(_kw(node, 1, "dim", 0))
    vals = [t for t in tensors]
    dt = vals[0].dtype
    for v in vals[1:]:
        dt = _dtype_promote(dt, v.dtype)
    shape = list(vals[0].shape)
    if dim < 0:
        dim += len(shape)
    shape[dim] = sum(v.shape[dim] for v in vals)
    out = L.alloc(shape, dt)
    off = 0
    regions = []
    for v in vals:
        n = v.shape[dim]
        region = out.narrow(dim, off, n)
        L.copy(v.buf, region)
        regions.append((off, n))
        off += n
    req = any(v.req_grad for v in vals)
    outv = Val(out, req_grad=req)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        for v, (o, n) in zip(vals, regions):
            if v.req_grad:
                B.contribute(v, g.narrow(dim, o, n))

    if req:
        L.add_backward(bwd)
    return outv


def lower_add(L, node):
    a, b = L.arg(node.args[0]), L.arg(node.args[1])
    alpha = node.kwargs.get("alpha", 1)
    if alpha != 1:
        raise Unsupported("add with alpha")
    if not isinstance(a, Val) or not isinstance(b, Val):
        raise Unsupported("add of a tensor and a python scalar")
    if b.buf.numel() > a.buf.numel():
        a, b = b, a
    out_dtype = _dtype_promote(a.dtype, b.dtype)
    req = a.req_grad or b.req_grad
    if a.shape == b.shape:
        if not (is_dense(a.buf) and is_dense(b.buf) and a.buf.stride() == b.buf.stride()):
            raise Unsupported("add of differently laid out tensors")
        out = torch.empty_like(a.buf, dtype=out_dtype)
        L.cur.fwd_bytes += out.numel() * out.element_size()
        L.emit(L.kernels.axpby(a.buf, 1.0, b.buf, 1.0, out, out.numel()))
        outv = Val(out, req_grad=req)

        def bwd(B):
            g = B.grad_of(outv)
            if g is None:
                return
            B.contribute(a, g)
            B.contribute(b, g)

        if req:
            L.add_backward(bwd)
        return outv
    # per-sample, per-channel vector added to every pixel: [B, C, H, W] + [B, C, 1, 1]
    if (a.buf.dim() == 4 and b.buf.dim() == 4 and b.shape == (a.shape[0], a.shape[1], 1, 1)
            and a.buf.permute(0, 2, 3, 1).is_contiguous() and b.buf.reshape(-1).is_contiguous()
            and b.buf.stride(1) == 1):
        Bn, C, H, W = a.shape
        out = L.alloc((Bn, H, W, C), out_dtype)
        L.emit(L.kernels.bias_add(a.buf, b.buf, out, Bn * H * W * C, C, H * W))
        outv = Val(out.permute(0, 3, 1, 2), req_grad=req)

        def bwd_chan(B):
            g = B.grad_of(outv)
            if g is None:
                return
            B.contribute(a, g)
            if b.req_grad:
                gn = _grad_nhwc(B, g, g.dtype).reshape(Bn, H * W, C)
                acc = B.temp((Bn, C), torch.float32)
                B.emit(B.k.fill(acc, 0.0, acc.numel()))
                ws = B.temp((B.k.colreduce_workspace(H * W, C),), torch.float32)
                for i in range(Bn):
                    B.emit(B.k.colsum_accumulate(gn[i], H * W, C, C, acc[i], ws))
                B.contribute(b, acc.view(Bn, C, 1, 1))

        if req:
            L.add_backward(bwd_chan)
        return outv
    # broadcast of b over the leading dimensions of a
    bshape = tuple(b.shape)
    while bshape and bshape[0] == 1:
        bshape = bshape[1:]
    if tuple(a.shape[len(a.shape) - len(bshape):]) != bshape or not a.buf.is_contiguous() or not b.buf.is_contiguous():
        raise Unsupported("add with general broadcasting %s + %s" % (a.shape, b.shape))
    n, blen = a.buf.numel(), b.buf.numel()
    out = L.alloc(a.shape, out_dtype)
    L.emit(L.kernels.bias_add(a.buf, b.buf, out, n, blen))
    outv = Val(out, req_grad=req)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        B.contribute(a, g)
        if b.req_grad:
            gc = g if g.is_contiguous() else _compact(B, g)
            dst, prev = B.grad_target(b)
            if dst.dtype != torch.float32 or not dst.is_contiguous():
                raise Unsupported("broadcast-add backward into a non-fp32 gradient")
            if prev is None:
                B.emit(B.k.fill(dst, 0.0, dst.numel()))
            elif prev is not dst:
                B.copy(prev, dst)
            B.emit(B.k.colsum_accumulate(gc, n // blen, blen, blen, dst, L.workspace(n // blen, blen)))
            B.commit(b, dst)

    if req:
        L.add_backward(bwd)
    return outv


def lower_unary_act(L, node):
    act = _act_of_node(node)
    x = L.arg(node.args[0])
    if not is_dense(x.buf):
        raise Unsupported("activation on a non-dense tensor")
    y = torch.empty_like(x.buf)   # same (possibly permuted) dense layout: the kernel walks flat memory
    L.cur.fwd_bytes += y.numel() * y.element_size()
    L.emit(L.kernels.act_fwd(x.buf, y, act, y.numel()))
    outv = Val(y, req_grad=x.req_grad)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        if not (g.dtype == x.dtype and g.stride() == x.buf.stride()):
            t = B.new_like(y)
            B.copy(g, t)
            g = t
        dst, prev = B.grad_target(x)
        if prev is None and dst.stride() == x.buf.stride() and dst.dtype == x.dtype:
            B.emit(B.k.act_bwd(g, x.buf, dst, act, y.numel()))
        else:
            tmp = B.new_like(y)
            B.emit(B.k.act_bwd(g, x.buf, tmp, act, y.numel()))
            B.merge(tmp, dst, prev)
        B.commit(x, dst)

    if x.req_grad:
        L.add_backward(bwd)
    return outv


def lower_dropout(L, node):
    p = _kw(node, 1, "p", 0.5)
    training = _kw(node, 2, "training", True)
    if p and training:
        raise Unsupported("dropout with p > 0 in training mode")
    x = L.arg(node.args[0])
    return Val(x.buf, req_grad=x.req_grad, kind="view", base=x, view_fn=lambda t: t)


def lower_pad(L, node):
    """F.pad(x, pad, "constant", value) of a tensor that needs no gradient (label shifting:
    pfeife's language-model scripts let the model library pad the labels with -100 and slice
    them by one).  The padded buffer is filled once, when the program is built; a step only copies
    x into its interior."""
    x = L.arg(node.args[0])
    pad = tuple(_kw(node, 1, "pad"))
    mode = _kw(node, 2, "mode", "constant")
    value = _kw(node, 3, "value", None)
    if not isinstance(x, Val) or x.req_grad:
        raise Unsupported("pad of a tensor that needs a gradient")
    if mode != "constant" or len(pad) % 2 or len(pad) // 2 > x.buf.dim() or any(p < 0 for p in pad):
        raise Unsupported("pad mode %s / widths %s" % (mode, pad))
    shape = list(x.shape)
    region = []
    for i in range(len(pad) // 2):
        dim = x.buf.dim() - 1 - i
        shape[dim] += pad[2 * i] + pad[2 * i + 1]
        region.append((dim, pad[2 * i], x.shape[dim]))
    out = torch.full(shape, 0 if value is None else value, dtype=x.dtype, device=L.device)
    L.cur.fwd_bytes += out.numel() * out.element_size()
    inner = out
    for dim, start, n in region:
        inner = inner.narrow(dim, start, n)
    L.copy(x.buf, inner)
    return Val(out, req_grad=False)


def lower_cross_entropy(L, node):
    logits = L.arg(node.args[0])
    target = L.arg(node.args[1])
    if _kw(node, 2, "weight") is not None or node.kwargs.get("label_smoothing", 0.0):
        raise Unsupported("weighted / label-smoothed cross entropy")
    ignore_index = int(node.kwargs.get("ignore_index", -100))
    if node.kwargs.get("reduction", "mean") != "mean":
        raise Unsupported("cross entropy with reduction other than mean")
    if logits.buf.dim() != 2 or not logits.buf.is_contiguous() or target.dtype != torch.int64:
        raise Unsupported("cross entropy expects contiguous [rows, classes] logits and int64 targets")
    rows, classes = logits.shape
    tgt = target.buf if target.buf.is_contiguous() else None
    if tgt is None:
        raise Unsupported("non-contiguous cross entropy targets")
    row_loss = L.alloc((rows,), torch.float32)
    row_lse = L.alloc((rows,), torch.float32)
    loss2 = L.alloc((2,), torch.float32)
    L.emit(L.kernels.cross_entropy_fwd(logits.buf, tgt, row_loss, row_lse, loss2, rows, classes, ignore_index))
    outv = Val(loss2[0], req_grad=logits.req_grad)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        if g.dtype != torch.float32:
            raise Unsupported("loss gradient must be fp32")
        dst, prev = B.grad_target(logits)
        if prev is None and dst.is_contiguous() and dst.dtype == logits.dtype:
            B.emit(B.k.cross_entropy_bwd(logits.buf, tgt, row_lse, g, loss2, dst, rows, classes, ignore_index))
        else:
            # the logits already have a gradient (they are also returned to user code, as model
            # libraries' output records do): form this one aside and add it
            tmp = B.temp(logits.shape, logits.dtype)
            B.emit(B.k.cross_entropy_bwd(logits.buf, tgt, row_lse, g, loss2, tmp, rows, classes, ignore_index))
            B.merge(tmp, dst, prev)
        B.commit(logits, dst)

    if logits.req_grad:
        L.add_backward(bwd)
    return outv


def lower_float(L, node):
    """x.float() / x.to(float32): under the mixed-precision policy a no-op for fp32 values,
    a cast kernel otherwise."""
    x = L.arg(node.args[0])
    if L.mixed and node.users and all(u.op == "call_function" and u.target is F.cross_entropy for u in node.users):
        # the loss kernels read 16-bit logits and do their arithmetic in fp32: no fp32 copy of the logits
        return Val(x.buf, req_grad=x.req_grad, kind="view", base=x, view_fn=lambda t: t)
    return _lower_cast(L, x, torch.float32)


def _lower_cast(L, x, dtype):
    if x.dtype == dtype:
        return Val(x.buf, req_grad=x.req_grad, kind="view", base=x, view_fn=lambda t: t)
    out = torch.empty_like(x.buf, dtype=dtype) if is_dense(x.buf) else L.alloc(x.shape, dtype)
    L.copy(x.buf, out)
    outv = Val(out, req_grad=x.req_grad)

    def bwd(B):
        g = B.grad_of(outv)
        if g is not None:
            B.contribute(x, g)

    if x.req_grad:
        L.add_backward(bwd)
    return outv


def lower_to(L, node):
    x = L.arg(node.args[0])
    dtype = node.kwargs.get("dtype")
    for a in node.args[1:]:
        if isinstance(a, torch.dtype):
            dtype = a
    if dtype is None:
        return Val(x.buf, req_grad=x.req_grad, kind="view", base=x, view_fn=lambda t: t)
    return _lower_cast(L, x, dtype)


def lower_embedding(L, node):
    ids = L.arg(node.args[0])
    table = L.arg(node.args[1])
    pad = _kw(node, 2, "padding_idx")
    if pad is not None and not isinstance(pad, int):
        raise Unsupported("embedding with a non-constant padding_idx")
    if ids.dtype != torch.int64 or not ids.buf.is_contiguous() or not table.buf.is_contiguous():
        raise Unsupported("embedding expects contiguous int64 ids")
    vocab, dim = table.shape
    # F.embedding's convention: None = no padding row, negative values count from the end
    padding_idx = -1 if pad is None else (pad + vocab if pad < 0 else pad)
    if padding_idx >= vocab or (pad is not None and padding_idx < 0):
        raise Unsupported("embedding padding_idx out of range")
    n = ids.buf.numel()
    out_dtype = table.dtype  # autocast leaves embedding outputs in the table's dtype (fp32 residual stream)
    out = L.alloc(tuple(ids.shape) + (dim,), out_dtype)
    L.emit(L.kernels.embedding_fwd(table.buf, ids.buf, out, n, dim, vocab))
    outv = Val(out, req_grad=table.req_grad)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None or table.param is None:
            return
        gc = g if g.is_contiguous() else _compact(B, g)
        B.emit(B.k.embedding_bwd(gc, ids.buf, L.params.grad(table.param), n, dim, vocab, padding_idx))

    if table.req_grad:
        L.add_backward(bwd)
    return outv


def lower_mul(L, node):
    a, b = L.arg(node.args[0]), L.arg(node.args[1])
    if isinstance(a, Val) and isinstance(b, Val):
        # gated MLP: act(gate) * up, with the activation node fused here
        for gate_v, up_v, gate_n in ((a, b, node.args[0]), (b, a, node.args[1])):
            info = gate_v.pending_act
            if info is not None and len(gate_n.users) == 1 and gate_v.shape == up_v.shape:
                act, gsrc = info
                return _lower_glu(L, gsrc, up_v, act)
        raise Unsupported("elementwise tensor*tensor outside the gated-MLP pattern")
    v, s = (a, b) if isinstance(a, Val) else (b, a)
    if not isinstance(v, Val) or not isinstance(s, (int, float)):
        raise Unsupported("mul operands %s" % (node.format_node(),))
    if not is_dense(v.buf):
        raise Unsupported("scaling a non-dense tensor")
    out = torch.empty_like(v.buf)
    L.cur.fwd_bytes += out.numel() * out.element_size()
    L.emit(L.kernels.axpby(v.buf, float(s), None, 0.0, out, out.numel()))
    outv = Val(out, req_grad=v.req_grad)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        gc = g if is_dense(g) and g.stride() == v.buf.stride() else _compact(B, g)
        t = B.new_like(v.buf)
        B.emit(B.k.axpby(gc, float(s), None, 0.0, t, t.numel()))
        B.contribute(v, t)

    if v.req_grad:
        L.add_backward(bwd)
    return outv


def _lower_glu(L, gate, up, act):
    rows_cols = as_matrix(gate.buf), as_matrix(up.buf)
    if rows_cols[0] is None or rows_cols[1] is None or gate.dtype != up.dtype:
        raise Unsupported("gated MLP on non-matrix operands")
    rows, cols, ldg = rows_cols[0]
    _, _, ldu = rows_cols[1]
    y = L.alloc(gate.shape, gate.dtype)
    L.emit(L.kernels.glu_fwd(gate.buf, ldg, up.buf, ldu, y, cols, act, rows, cols))
    req = gate.req_grad or up.req_grad
    outv = Val(y, req_grad=req)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        gc = B.matrix_in(g, gate.dtype)
        dg_dst, dg_prev = B.grad_target(gate)
        du_dst, du_prev = B.grad_target(up)
        mg, mu = as_matrix(dg_dst), as_matrix(du_dst)
        if dg_prev is not None or du_prev is not None or mg is None or mu is None:
            raise Unsupported("gated MLP backward into already written / non-matrix gradients")
        B.emit(B.k.glu_bwd(gc, as_matrix(gc)[2], gate.buf, ldg, up.buf, ldu, dg_dst, mg[2], du_dst, mu[2], act, rows,
                           cols))
        B.commit(gate, dg_dst)
        B.commit(up, du_dst)

    if req:
        L.add_backward(bwd)
    return outv


def lower_act_maybe_gate(L, node):
    """silu/gelu whose single user is a tensor*tensor product is the gate of a gated MLP:
    defer it to the product so that one kernel computes act(gate) * up."""
    user = L.sole_user(node)
    x = L.arg(node.args[0])
    if (user is not None and user.op == "call_function" and user.target in (operator.mul, torch.mul)
            and all(isinstance(a, torch.fx.Node) for a in user.args[:2])):
        v = Val(x.buf, req_grad=x.req_grad, kind="view", base=x, view_fn=lambda t: t)
        v.pending_act = (_act_of_node(node), x)
        return v
    return lower_unary_act(L, node)


def _is(node, *targets):
    return isinstance(node, torch.fx.Node) and node.op == "call_function" and node.target in targets


def find_rope_patterns(gm):
    """Rotary embedding written the HF way,
        x * cos + cat((-x[..., h:], x[..., :h]), -1) * sin,
    is nine graph nodes; match it so that one kernel computes it.
    -> ({add_node: (x_node, cos_node, sin_node)}, {interior nodes})"""
    roots, skip = {}, set()
    for add in gm.graph.nodes:
        if not _is(add, operator.add, torch.add) or len(add.args) != 2:
            continue
        m1, m2 = add.args
        if not (_is(m1, operator.mul, torch.mul) and _is(m2, operator.mul, torch.mul)):
            continue
        for a, b in ((m1, m2), (m2, m1)):
            x, cos = a.args
            cat, sin = b.args
            if not _is(cat, torch.cat) or not isinstance(x, torch.fx.Node):
                continue
            parts = cat.args[0]
            dim = cat.kwargs.get("dim", cat.args[1] if len(cat.args) > 1 else 0)
            if dim != -1 or len(parts) != 2 or not _is(parts[0], operator.neg, torch.neg):
                continue
            hi, lo = parts[0].args[0], parts[1]
            if not (_is(hi, operator.getitem) and _is(lo, operator.getitem)):
                continue
            if hi.args[0] is not x or lo.args[0] is not x:
                continue
            ih, il = hi.args[1], lo.args[1]
            ok = (isinstance(ih, tuple) and isinstance(il, tuple) and len(ih) == 2 and len(il) == 2
                  and ih[0] is Ellipsis and il[0] is Ellipsis and isinstance(ih[1], slice) and isinstance(il[1], slice)
                  and ih[1].stop is None and il[1].start is None and ih[1].start == il[1].stop
                  and ih[1].step is None and il[1].step is None)
            interior = [a, b, cat, parts[0], hi, lo]
            if not ok or any(len(n.users) != 1 for n in interior):
                continue
            roots[add] = (x, cos, sin, ih[1].start)
            skip.update(interior)
            break
    return roots, skip


def lower_rope(L, node, x_node, cos_node, sin_node, half):
    x, cos, sin = L.arg(x_node), L.arg(cos_node), L.arg(sin_node)
    if x.buf.dim() != 4 or x.shape[-1] != 2 * half or x.buf.stride(3) != 1:
        raise Unsupported("rotary embedding on a tensor of shape %s" % (x.shape,))
    Bn, H, T, D = x.shape                      # [B, H, T, D] view of a token-major projection

    def table(t):
        """[T, D] fp32 view of a rotary table given as [T, D] or with broadcast dimensions in front
        ([1, 1, T, D] / [B, 1, T, D] with the same positions for every batch entry, the form model
        libraries hand over after `unsqueeze(1)`)."""
        if t.req_grad:
            raise Unsupported("trainable rotary tables")
        b = t.buf
        if b.dtype == torch.float32 and b.dim() > 2 and tuple(b.shape[-2:]) == (T, D) and b.stride(-1) == 1:
            lead = b.reshape(-1, T, D)
            if lead.shape[0] == 1 or bool((lead == lead[:1]).all()):   # build-time check (one host read)
                b = lead[0]
        if b.dtype != torch.float32 or b.dim() != 2 or tuple(b.shape) != (T, D) or b.stride(1) != 1:
            raise Unsupported("rotary tables must be fp32 [T, D] (or that with broadcast dimensions in front), "
                              "got %s %s" % (t.shape, t.dtype))
        return Val(b, req_grad=False, name=t.name)

    cos, sin = table(cos), table(sin)
    out_dtype = L.cd if L.mixed else x.dtype
    y = L.alloc((Bn, T, H, D), out_dtype)       # token-major like the projections
    yv = y.permute(0, 2, 1, 3)
    xs = (x.buf.stride(0), x.buf.stride(2), x.buf.stride(1))
    ys = (yv.stride(0), yv.stride(2), yv.stride(1))
    tab_ld = cos.buf.stride(0)
    if sin.buf.stride(0) != tab_ld:
        raise Unsupported("cos/sin tables with different row strides")
    if x.dtype != out_dtype:
        xin = L.alloc((Bn, T, H, D), out_dtype).permute(0, 2, 1, 3)
        L.copy(x.buf, xin)
        xs = (xin.stride(0), xin.stride(2), xin.stride(1))
    else:
        xin = x.buf
    L.emit(L.kernels.rope(xin, yv, cos.buf, sin.buf, Bn, T, H, D, xs, ys, 0, tab_ld))
    outv = Val(yv, req_grad=x.req_grad)

    def bwd(B):
        g = B.grad_of(outv)
        if g is None:
            return
        if g.dtype != out_dtype or g.stride(3) != 1:
            t = B.new_like(yv)
            B.copy(g, t)
            g = t
        gs = (g.stride(0), g.stride(2), g.stride(1))
        dst, prev = B.grad_target(x)
        if prev is None and dst.dtype == out_dtype and dst.stride(3) == 1:
            ds = (dst.stride(0), dst.stride(2), dst.stride(1))
            B.emit(B.k.rope(g, dst, cos.buf, sin.buf, Bn, T, H, D, gs, ds, 1, tab_ld))
        else:
            tmp = B.new_like(yv)
            B.emit(B.k.rope(g, tmp, cos.buf, sin.buf, Bn, T, H, D, gs, (tmp.stride(0), tmp.stride(2), tmp.stride(1)),
                            1, tab_ld))
            if prev is None:
                B.copy(tmp, dst)
            elif prev is dst:
                B.copy(tmp, dst, accumulate=True)
            else:
                B.copy(prev, dst)
                B.copy(tmp, dst, accumulate=True)
        B.commit(x, dst)

    if x.req_grad:
        L.add_backward(bwd)
    return outv


FUNCTION_HANDLERS = {
    F.linear: lower_linear, torch._C._nn.linear: lower_linear,
    F.layer_norm: lower_layer_norm, torch.layer_norm: lower_layer_norm,
    F.rms_norm: lower_rms_norm, torch.rms_norm: lower_rms_norm,
    F.group_norm: lower_group_norm, torch.group_norm: lower_group_norm,
    F.scaled_dot_product_attention: lower_sdpa, torch._C._nn.scaled_dot_product_attention: lower_sdpa,
    F.conv2d: lower_conv2d, torch.conv2d: lower_conv2d,
    F.gelu: lower_act_maybe_gate, torch._C._nn.gelu: lower_act_maybe_gate,
    F.silu: lower_act_maybe_gate,
    F.relu: lower_unary_act, torch.relu: lower_unary_act,
    F.dropout: lower_dropout,
    F.pad: lower_pad, torch._C._nn.pad: lower_pad,
    F.cross_entropy: lower_cross_entropy,
    F.embedding: lower_embedding,
    operator.add: lower_add, operator.iadd: lower_add, torch.add: lower_add,
    operator.mul: lower_mul, torch.mul: lower_mul,
    operator.getitem: lower_getitem,
    torch.cat: lower_cat,
    torch.flatten: lower_flatten, torch.transpose: lower_transpose, torch.permute: lower_permute,
    torch.reshape: lower_reshape, torch.unsqueeze: lower_unsqueeze, torch.squeeze: lower_squeeze,
    torch.unbind: lower_unbind, torch.chunk: lower_chunk, torch.split: lower_split,
}
METHOD_HANDLERS = {
    "reshape": lower_reshape, "view": lower_view, "permute": lower_permute, "transpose": lower_transpose,
    "flatten": lower_flatten, "unsqueeze": lower_unsqueeze, "squeeze": lower_squeeze,
    "contiguous": lower_contiguous, "unbind": lower_unbind, "chunk": lower_chunk, "split": lower_split,
    "expand": lower_expand, "float": lower_float, "to": lower_to, "add": lower_add, "mul": lower_mul,
}
CAST_TO_CD_TARGETS = {F.linear, torch._C._nn.linear, F.conv2d, torch.conv2d,
                      F.scaled_dot_product_attention, torch._C._nn.scaled_dot_product_attention, torch.matmul}
