"""Values of a stage program and the gradient bookkeeping used while the
backward launch list is being built.

A stage program is built once per (stage, micro-batch): every value gets a
preallocated device buffer, and forward/backward become flat lists of prepared
kernel launches on those buffers.  Nothing here runs per step.

Gradient rules (all resolved at build time):
  * a gradient buffer has the shape, dtype and strides of the value's buffer;
  * views do not own gradients: the gradient of a full view is the same view of
    its base's gradient, the gradient of a partial view (slice, unbind item) is
    a region of its parent's gradient;
  * the first contribution to a value overwrites, later ones accumulate; a
    buffer that is shared with another value (alias) is never modified in
    place, the new total goes to a fresh buffer instead.
"""
import torch


def dense_like(t):
    """Uninitialised tensor with t's shape, dtype and (when dense) stride order."""
    return torch.empty_like(t)


def as_matrix(t):
    """Describe t as a row-major matrix [rows, cols] with leading dimension ld
    (last dimension contiguous, all leading dimensions collapsing into one
    stride).  Returns (rows, cols, ld) or None."""
    if t.dim() == 0:
        return None
    cols = t.shape[-1]
    if cols > 1 and t.stride(-1) != 1:
        return None
    lead = [(s, st) for s, st in zip(t.shape[:-1], t.stride()[:-1]) if s != 1]
    rows = 1
    for s, _ in lead:
        rows *= s
    if not lead:
        return (1, cols, max(cols, 1))
    ld = lead[-1][1]
    expect = ld
    for s, st in reversed(lead):
        if st != expect:
            return None
        expect = st * s
    if ld < cols:
        return None
    return (rows, cols, ld)


def is_dense(t):
    return t.is_contiguous() or t.numel() == 0 or torch.empty_like(t).stride() == t.stride()


def collapse_for_copy(shape, s_strides, d_strides):
    """Merge adjacent dimensions that are contiguous in both operands (fewer div/mod per element)."""
    dims = [(n, a, b) for n, a, b in zip(shape, s_strides, d_strides) if n != 1]
    if not dims:
        return [1], [1], [1]
    out = [dims[0]]
    for n, a, b in dims[1:]:
        pn, pa, pb = out[-1]
        if pa == a * n and pb == b * n:
            out[-1] = (pn * n, a, b)
        else:
            out.append((n, a, b))
    return [d[0] for d in out], [d[1] for d in out], [d[2] for d in out]


class Val:
    """A tensor value of a stage program."""

    __slots__ = ("buf", "req_grad", "kind", "base", "view_fn", "param", "grad", "grad_shared", "written",
                 "partial_only", "tiled", "name", "preact", "grad_is_preact", "pending_act", "boundary", "lp_grad")

    def __init__(self, buf, req_grad=False, kind="base", base=None, view_fn=None, param=None, name=""):
        self.buf = buf
        self.req_grad = bool(req_grad)
        self.kind = kind          # "base" | "view" (full view of base) | "part" (region of base)
        self.base = base
        self.view_fn = view_fn    # tensor of base's layout -> the corresponding view / region
        self.param = param        # nn.Parameter when the value is a trainable parameter
        self.grad = None
        self.grad_shared = False
        self.written = False      # part: region already holds a contribution
        self.partial_only = False  # base: gradient so far written by partial children only
        self.tiled = False        # part: siblings tile the parent and all of them receive a gradient
        self.name = name
        self.preact = None        # (act, pre-activation buffer) when this value is act(linear(...)) fused in a GEMM
        self.grad_is_preact = False
        self.lp_grad = None       # dict(colsum, cols) when backward reads this value's gradient as a 16-bit matrix
        self.boundary = False     # stage input produced by another stage: its gradient outlives the backward job
        self.pending_act = None   # (act, source value) when this is the not-yet-applied gate of a gated MLP

    @property
    def shape(self):
        return tuple(self.buf.shape)

    @property
    def dtype(self):
        return self.buf.dtype

    def __repr__(self):
        return "Val(%s %s %s%s)" % (self.name, tuple(self.buf.shape), self.buf.dtype, " grad" if self.req_grad else "")
