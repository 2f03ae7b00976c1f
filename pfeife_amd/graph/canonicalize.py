"""Brings a captured FX graph into the forms the stage lowering knows.

The reference hands whatever TorchDynamo captured to eager ATen, so every model library's
spelling of an operation runs as it is (pfeife/mp/worker.py:1457-1494).  The HIP lowering works
on a vocabulary of fused operations instead; this pass rewrites the spellings that the model
libraries the reference's scripts use (Hugging Face `ViTForImageClassification`,
bench_models/models/train_vit.py:150-169, and `LlamaForCausalLM` with
`attn_implementation="eager"`, bench_models/models/train_llama.py:486-520) into that vocabulary
before the graph is cut into stages:

  * input-independent bookkeeping (position ids, attention masks built from `arange`
    comparisons, rotary cos/sin tables computed from `inv_freq`) is evaluated ONCE, when the
    graph is compiled, and enters the graph as constant tensors (extra static placeholders);
    nothing that depends on a per-step input or on a trainable tensor is touched;
  * the decomposed RMSNorm (`w * (x.float() * rsqrt(x.float().pow(2).mean(-1, True) + eps)).to(dt)`)
    becomes `F.rms_norm`;
  * eager attention (`softmax(q @ k^T * s + mask) @ v`, with an optional cast and a disabled
    dropout in between) becomes `F.scaled_dot_product_attention`; the additive mask must be one
    of the folded constants and either all zeros or the causal pattern; an explicit `attn_mask`
    of `F.scaled_dot_product_attention` that is such a constant is dropped / becomes `is_causal`;
  * nodes without data flow (`_set_grad_enabled`, `_log_api_usage_once`) are dropped.
"""
import math
import operator

import torch
import torch.fx as fx
import torch.nn.functional as F

FOLDED_PREFIX = "pf_folded_"

_SIDE_EFFECT_TARGETS = (torch._C._set_grad_enabled, torch._C._log_api_usage_once)
_VIEW_METHODS = ("view", "reshape", "permute", "transpose", "unsqueeze", "squeeze", "expand", "flatten", "contiguous")
_RANDOM_NAMES = ("rand", "randn", "randint", "bernoulli", "normal", "multinomial", "rand_like", "randn_like")


def _name(node):
    return node.target if node.op == "call_method" else getattr(node.target, "__name__", str(node.target))


def _is_fn(node, *targets):
    return isinstance(node, fx.Node) and node.op == "call_function" and node.target in targets


def _is_method(node, *names):
    return isinstance(node, fx.Node) and node.op == "call_method" and node.target in names


def _is_mul(node):
    return _is_fn(node, operator.mul, torch.mul) or _is_method(node, "mul")


def _is_add(node):
    return _is_fn(node, operator.add, torch.add) or _is_method(node, "add")


def _static_nograd(node, example, is_static):
    return torch.is_tensor(example) and is_static(node, example) and not example.requires_grad


def _trivial_on_placeholders(node):
    """A slice / view taken directly from graph inputs: the lowering treats it as a view already."""
    if not all(a.op == "placeholder" for a in node.all_input_nodes):
        return False
    return _is_fn(node, operator.getitem) or _is_method(node, *_VIEW_METHODS)


def fold_constants(gm, live_args, device, is_static):
    """Evaluates every node that depends only on constants, shapes and non-trainable module state
    (buffers), and replaces the values the rest of the graph reads by static placeholders.
    -> (extended live_args, number of constants)."""
    graph = gm.graph
    placeholders = [n for n in graph.nodes if n.op == "placeholder"]
    if len(placeholders) != len(live_args):
        raise RuntimeError("canonicalize: %d graph inputs, %d arguments" % (len(placeholders), len(live_args)))
    value = {}
    foldable = set()
    for ph, ex in zip(placeholders, live_args):
        if _static_nograd(ph, ex, is_static):
            value[ph] = ex.detach()
            foldable.add(ph)
    for node in graph.nodes:
        if node.op not in ("call_function", "call_method"):
            continue
        if node.op == "call_function" and node.target in _SIDE_EFFECT_TARGETS:
            continue
        if _name(node) in _RANDOM_NAMES:
            continue
        ev = node.meta.get("example_value")
        if not torch.is_tensor(ev) or ev.requires_grad:
            continue
        if all(a in foldable for a in node.all_input_nodes):
            foldable.add(node)

    def evaluate(node):
        if node in value:
            return value[node]
        args = fx.node.map_arg(node.args, evaluate)
        kwargs = fx.node.map_arg(node.kwargs, evaluate)
        with torch.no_grad():
            if node.op == "call_function":
                out = node.target(*args, **kwargs)
            else:
                out = getattr(args[0], node.target)(*args[1:], **kwargs)
        value[node] = out
        return out

    frontier = []
    for node in graph.nodes:
        if node in foldable and node.op != "placeholder":
            if any(u not in foldable for u in node.users) and not _trivial_on_placeholders(node):
                frontier.append(node)
    live = list(live_args)
    last_ph = placeholders[-1] if placeholders else None
    count = 0
    for node in frontier:
        t = evaluate(node)
        if not torch.is_tensor(t):
            continue
        t = t.detach().to(device).contiguous()
        with graph.inserting_after(last_ph):
            ph = graph.placeholder("%s%d_%s" % (FOLDED_PREFIX, count, node.name))
        ph.meta = dict(node.meta)
        ph.meta["example_value"] = t
        value[ph] = t
        node.replace_all_uses_with(ph)
        last_ph = ph
        live.append(t)
        count += 1
    return live, count


def _single_user(node):
    return len(node.users) == 1


def rewrite_rms_norm(gm):
    """w * (x32 * rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps)).to(dtype), x32 = x.to(float32)
    -> F.rms_norm(x, (d,), w, eps).  Returns the number of rewrites."""
    graph = gm.graph
    n = 0
    for root in list(graph.nodes):
        if not _is_mul(root) or len(root.args) != 2:
            continue
        for w, cast in (root.args, root.args[::-1]):
            if not (isinstance(w, fx.Node) and w.op == "placeholder"):
                continue
            h1 = cast.args[0] if _is_method(cast, "to", "type") and _single_user(cast) else cast
            if not (_is_mul(h1) and len(h1.args) == 2 and _single_user(h1)):
                continue
            hit = None
            for x32, rs in (h1.args, h1.args[::-1]):
                if not (_is_fn(rs, torch.rsqrt) and _single_user(rs)):
                    continue
                add = rs.args[0]
                if not (_is_add(add) and _single_user(add) and isinstance(add.args[1], (int, float))):
                    continue
                var = add.args[0]
                if not (_is_method(var, "mean") and _single_user(var)):
                    continue
                dims = var.args[1] if len(var.args) > 1 else var.kwargs.get("dim")
                keep = var.args[2] if len(var.args) > 2 else var.kwargs.get("keepdim", False)
                if dims not in (-1, (-1,), [-1]) or not keep:
                    continue
                pw = var.args[0]
                if not (_is_method(pw, "pow") and _single_user(pw) and pw.args[1] == 2 and pw.args[0] is x32):
                    continue
                if not isinstance(x32, fx.Node):
                    continue
                x = x32
                if _is_method(x32, "to", "float") and set(x32.users) == {pw, h1}:
                    want32 = x32.target == "float" or torch.float32 in x32.args or x32.kwargs.get("dtype") == torch.float32
                    if want32:
                        x = x32.args[0]
                hit = (x, float(add.args[1]))
                break
            if hit is None:
                continue
            x, eps = hit
            wv = w.meta.get("example_value")
            xv = x.meta.get("example_value")
            if not (torch.is_tensor(wv) and wv.dim() == 1 and torch.is_tensor(xv) and xv.shape[-1] == wv.shape[0]):
                continue
            with graph.inserting_before(root):
                new = graph.call_function(F.rms_norm, (x, (int(wv.shape[0]),), w, eps))
            new.meta = dict(root.meta)
            root.replace_all_uses_with(new)
            n += 1
            break
    return n


def _mask_kind(t):
    """For a boolean mask: 'none' when everything is visible, 'causal' for the lower triangle.
    For an additive mask: 'none' for an all-zero additive mask, 'causal' for 0 on and below the diagonal and a large
    negative number above it (the same for every batch entry and head), else None."""
    visible = t if t.dtype == torch.bool else (t == 0)
    if bool(visible.all()):
        return "none"
    if t.dim() < 2 or t.shape[-1] != t.shape[-2]:
        return None
    T = t.shape[-1]
    tril = torch.ones(T, T, dtype=torch.bool, device=t.device).tril()
    if bool((visible == tril).all()) and (t.dtype == torch.bool or bool((t[..., ~tril] <= -1e4).all())):
        return "causal"
    return None


def rewrite_sdpa_masks(gm, live_by_placeholder):
    """F.scaled_dot_product_attention(q, k, v, attn_mask=<folded constant>): a mask that hides
    nothing is dropped, the causal pattern becomes is_causal=True."""
    n = 0
    for node in gm.graph.nodes:
        if not _is_fn(node, F.scaled_dot_product_attention, torch._C._nn.scaled_dot_product_attention):
            continue
        mask = node.args[3] if len(node.args) > 3 else node.kwargs.get("attn_mask")
        if not (isinstance(mask, fx.Node) and mask.op == "placeholder" and mask.name.startswith(FOLDED_PREFIX)):
            continue
        kind = _mask_kind(live_by_placeholder[mask])
        if kind is None:
            continue
        kwargs = dict(node.kwargs)
        for i, key in enumerate(("attn_mask", "dropout_p", "is_causal", "scale")):
            if len(node.args) > 3 + i:
                kwargs[key] = node.args[3 + i]
        kwargs["attn_mask"] = None
        kwargs["is_causal"] = bool(kwargs.get("is_causal", False)) or kind == "causal"
        node.args = tuple(node.args[:3])
        node.kwargs = kwargs
        n += 1
    return n


def rewrite_eager_attention(gm, live_by_placeholder):
    """softmax(q @ k.transpose(-1, -2) * s [+ mask], -1) [.to(dt)] [dropout p = 0] @ v
    -> F.scaled_dot_product_attention(q, k, v, is_causal=..., scale=s)."""
    graph = gm.graph
    n = 0
    for root in list(graph.nodes):
        if not (_is_fn(root, torch.matmul) or _is_method(root, "matmul")):
            continue
        p, v = root.args
        chain = []
        if _is_fn(p, F.dropout, torch.dropout) and _single_user(p):
            prob = p.args[1] if len(p.args) > 1 else p.kwargs.get("p", 0.5)
            training = p.args[2] if len(p.args) > 2 else p.kwargs.get("training", True)
            if prob and training:
                continue
            chain.append(p)
            p = p.args[0]
        if _is_method(p, "to", "type") and _single_user(p):
            chain.append(p)
            p = p.args[0]
        if not (_is_fn(p, F.softmax, torch.softmax) and _single_user(p)):
            continue
        dim = p.args[1] if len(p.args) > 1 else p.kwargs.get("dim")
        if dim != -1:
            continue
        chain.append(p)
        s = p.args[0]
        mask = None
        if _is_add(s) and _single_user(s):
            a, b = s.args
            if isinstance(b, fx.Node) and b.op == "placeholder" and b.name.startswith(FOLDED_PREFIX):
                chain.append(s)
                s, mask = a, b
            elif isinstance(a, fx.Node) and a.op == "placeholder" and a.name.startswith(FOLDED_PREFIX):
                chain.append(s)
                s, mask = b, a
            else:
                continue
        scale = None
        if _is_mul(s) and _single_user(s) and isinstance(s.args[1], (int, float)):
            chain.append(s)
            scale, s = float(s.args[1]), s.args[0]
        elif _is_fn(s, operator.truediv, torch.div) and _single_user(s) and isinstance(s.args[1], (int, float)):
            chain.append(s)
            scale, s = 1.0 / float(s.args[1]), s.args[0]
        if not ((_is_fn(s, torch.matmul) or _is_method(s, "matmul")) and _single_user(s)):
            continue
        q, kt = s.args
        if not (_is_method(kt, "transpose") or _is_fn(kt, torch.transpose)):
            continue
        d0, d1 = kt.args[1], kt.args[2]
        kv = kt.args[0].meta.get("example_value")
        nd = kv.dim() if torch.is_tensor(kv) else 4
        if sorted((d0 % nd, d1 % nd)) != [nd - 2, nd - 1]:
            continue
        k = kt.args[0]
        causal = False
        if mask is not None:
            kind = _mask_kind(live_by_placeholder[mask])
            if kind is None:
                continue          # an arbitrary additive mask: left as it is (the lowering will refuse it)
            causal = kind == "causal"
        qv = q.meta.get("example_value")
        if scale is None:
            scale = 1.0          # a bare q @ k^T: no scaling was applied
        elif torch.is_tensor(qv) and abs(scale - 1.0 / math.sqrt(qv.shape[-1])) < 1e-12:
            scale = None         # the default: let the lowering derive it
        kwargs = dict(attn_mask=None, dropout_p=0.0, is_causal=causal)
        if scale is not None:
            kwargs["scale"] = scale
        with graph.inserting_before(root):
            new = graph.call_function(F.scaled_dot_product_attention, (q, k, v), kwargs)
        new.meta = dict(root.meta)
        root.replace_all_uses_with(new)
        n += 1
    return n


def canonicalize(gm, live_args, device, is_static):
    """Rewrites `gm` in place; -> (live_args extended by the folded constants, summary dict).
    `is_static(node, example)` says which placeholders are module state."""
    graph = gm.graph
    dropped = 0
    for node in list(graph.nodes):
        if node.op == "call_function" and node.target in _SIDE_EFFECT_TARGETS and not node.users:
            graph.erase_node(node)
            dropped += 1
    live, folded = fold_constants(gm, live_args, device, is_static)
    placeholders = [n for n in graph.nodes if n.op == "placeholder"]
    by_ph = dict(zip(placeholders, live))
    norms = rewrite_rms_norm(gm)
    attn = rewrite_eager_attention(gm, by_ph) + rewrite_sdpa_masks(gm, by_ph)
    graph.eliminate_dead_code()
    # constants nothing reads any more (masks that became a flag, tables of dropped branches)
    keep_live = []
    for ph, t in zip(placeholders, live):
        if ph.name.startswith(FOLDED_PREFIX) and not ph.users:
            graph.erase_node(ph)
        else:
            keep_live.append(t)
    graph.lint()
    gm.recompile()
    return keep_live, dict(folded=folded, rms_norm=norms, attention=attn, dropped=dropped)
