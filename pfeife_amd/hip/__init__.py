"""ctypes binding of libpfeife_hip.so and the tensor-level kernel table built on it.

`HipKernels` is the only kernel table the product ships: every method takes
preallocated torch tensors (device memory owned by PyTorch), resolves them to raw
pointers once, and returns a *prepared launch*: a callable `launch(stream)` that
re-issues exactly the same C call.  Stage programs are lists of prepared
launches, so a steady-state step does no argument marshalling at all.

There is no fallback: if the shared library is missing, `load()` raises.
"""
import ctypes
import os
from ctypes import POINTER, Structure, byref, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpfeife_hip.so")
ABI_VERSION = 4

PF_F32, PF_F16, PF_BF16, PF_I64, PF_I32, PF_U8 = 0, 1, 2, 3, 4, 5
ACT_NONE, ACT_GELU, ACT_GELU_TANH, ACT_SILU, ACT_RELU = 0, 1, 2, 3, 4

_DTYPE_CODE = {
    torch.float32: PF_F32,
    torch.float16: PF_F16,
    torch.bfloat16: PF_BF16,
    torch.int64: PF_I64,
    torch.int32: PF_I32,
    torch.uint8: PF_U8,
}


def dtype_code(dtype):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError("pfeife_amd: dtype %s has no HIP kernel support" % (dtype,))


class GemmDesc(Structure):
    """Mirror of `pf_gemm_desc` in include/pfeife_hip.h (field order is ABI)."""

    _fields_ = [
        ("in_dtype", c_int32), ("c_dtype", c_int32), ("a_trans", c_int32), ("b_trans", c_int32),
        ("M", c_int64), ("N", c_int64), ("K", c_int64),
        ("A", c_void_p), ("lda", c_int64),
        ("B", c_void_p), ("ldb", c_int64),
        ("C", c_void_p), ("ldc", c_int64),
        ("batch1", c_int64), ("batch2", c_int64),
        ("a_stride1", c_int64), ("a_stride2", c_int64),
        ("b_stride1", c_int64), ("b_stride2", c_int64),
        ("c_stride1", c_int64), ("c_stride2", c_int64),
        ("alpha", c_float), ("beta", c_int32),
        ("bias", c_void_p), ("bias_dtype", c_int32), ("round_mid", c_int32),
        ("aux_out", c_void_p), ("ld_aux_out", c_int64),
        ("act", c_int32), ("dact", c_int32),
        ("aux_in", c_void_p), ("ld_aux_in", c_int64),
        ("residual", c_void_p), ("ld_res", c_int64),
        ("res_dtype", c_int32), ("variant", c_int32),
        ("colsum_ws", c_void_p), ("unscale_by", c_void_p), ("nonfinite_flag", c_void_p),
    ]


class NormBwdDesc(Structure):
    """Mirror of `pf_norm_bwd_desc` in include/pfeife_hip.h."""

    _fields_ = ([(n, c_void_p) for n in ("dy", "x", "gamma", "mean", "rstd", "dx_add", "dx", "dx_lp", "workspace")]
                + [("rows", c_int64), ("d", c_int64)]
                + [(n, c_int32) for n in ("dy_dtype", "x_dtype", "add_dtype", "dx_dtype", "dx_lp_dtype", "want_wgrad",
                                          "want_colsum", "reserved")])


class AttnDesc(Structure):
    """Mirror of `pf_attn_desc` in include/pfeife_hip.h."""

    _fields_ = ([(n, c_int32) for n in ("dtype", "B", "H", "Tq", "Tk", "hd", "causal", "reserved")]
                + [("scale", c_float), ("reserved2", c_float)]
                + [(n, c_void_p) for n in ("q", "k", "v", "o", "d_o", "dq", "dk", "dv", "lse", "delta")]
                + [(n, c_int64) for n in ("q_sb", "q_sh", "q_st", "k_sb", "k_sh", "k_st", "v_sb", "v_sh", "v_st",
                                          "o_sb", "o_sh", "o_st", "do_sb", "do_sh", "do_st", "dq_sb", "dq_sh",
                                          "dq_st", "dk_sb", "dk_sh", "dk_st", "dv_sb", "dv_sh", "dv_st")])


# name -> argtypes (every function returns int unless listed in _RET_I64)
_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float
_SIGNATURES = {
    "pf_init": [_I],
    "pf_graph_capture_begin": [_P],
    "pf_graph_capture_end": [_P, POINTER(c_void_p)],
    "pf_graph_launch": [_P, _P],
    "pf_graph_destroy": [_P],
    "pf_gemm": [POINTER(GemmDesc), _P],
    "pf_gemm_grouped": [POINTER(GemmDesc), _I, _P],
    "pf_gemm_variant": [POINTER(GemmDesc), ctypes.c_char_p, _I],
    "pf_attention_fwd": [POINTER(AttnDesc), _P],
    "pf_attention_bwd": [POINTER(AttnDesc), _P],
    "pf_norm_bwd_fused": [POINTER(NormBwdDesc), _P],
    "pf_layernorm_fwd": [_P, _I, _P, _P, _P, _I, _P, _P, _L, _L, _F, _P],
    "pf_layernorm_bwd": [_P, _I, _P, _I, _P, _P, _P, _P, _I, _P, _I, _P, _P, _P, _L, _L, _I, _P],
    "pf_rmsnorm_fwd": [_P, _I, _P, _P, _I, _P, _L, _L, _F, _P],
    "pf_rmsnorm_bwd": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _I, _P, _P, _L, _L, _I, _P],
    "pf_colsum_accumulate": [_P, _I, _L, _L, _L, _P, _P, _I, _P],
    "pf_colsum_accumulate_static": [_P, _I, _L, _L, _L, _P, _P],
    "pf_colreduce_finalize_batch": [_P, _I, _L, _P],
    "pf_norm_bwd_partials": None,
    "pf_colsum_partials": None,
    "pf_softmax_fwd": [_P, _L, _P, _I, _L, _L, _L, _L, _I, _P],
    "pf_softmax_bwd": [_P, _L, _P, _I, _L, _P, _I, _L, _L, _L, _F, _P],
    "pf_cross_entropy_fwd": [_P, _I, _P, _P, _P, _P, _L, _L, _L, _P],
    "pf_cross_entropy_bwd": [_P, _I, _P, _P, _P, _P, _P, _I, _L, _L, _L, _P],
    "pf_mse_fwd": [_P, _I, _P, _I, _P, _P, _L, _P],
    "pf_mse_bwd": [_P, _I, _P, _I, _P, _P, _I, _L, _P],
    "pf_sum_fwd": [_P, _I, _P, _P, _L, _P],
    "pf_act_fwd": [_P, _P, _I, _I, _L, _P],
    "pf_act_bwd": [_P, _P, _P, _I, _I, _L, _P],
    "pf_glu_fwd": [_P, _L, _P, _L, _P, _L, _I, _I, _L, _L, _P],
    "pf_glu_bwd": [_P, _L, _P, _L, _P, _L, _P, _L, _P, _L, _I, _I, _L, _L, _P],
    "pf_axpby": [_P, _I, _F, _P, _I, _F, _P, _I, _L, _P],
    "pf_bias_add": [_P, _I, _P, _I, _P, _I, _L, _L, _L, _P],
    "pf_groupnorm_fwd": [_P, _I, _P, _P, _P, _I, _P, _P, _L, _L, _L, _I, _F, _P],
    "pf_groupnorm_bwd": [_P, _I, _P, _I, _P, _P, _P, _P, _I, _P, _P, _P, _L, _L, _L, _I, _I, _P],
    "pf_cast": [_P, _I, _P, _I, _L, _P],
    "pf_shadow_batch": [_P, _I, _L, _P],
    "pf_cast_batch": [_P, _I, _L, _P],
    "pf_transpose_cast": [_P, _I, _L, _P, _I, _L, _L, _L, _P],
    "pf_fill": [_P, _I, _F, _L, _P],
    "pf_adam_step": [_P, _I, _L, ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.c_double, _L,
                     _I, _P],
    "pf_adam_step_scaled": [_P, _I, _L, ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.c_double,
                            ctypes.c_double, _I, _P, _P],
    "pf_scale_by_state": [_P, _I, _P, _P, _I, _L, _P],
    "pf_scaler_unscale": [_P, _L, _P, _P],
    "pf_scaler_update": [_P, ctypes.c_double, ctypes.c_double, _I, _P],
    "pf_copy_strided": [_P, _I, POINTER(c_int64), _P, _I, POINTER(c_int64), POINTER(c_int64), _I, _I, _P],
    "pf_rope": [_P, _P, _I, _P, _P, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _I, _P],
    "pf_grad_accumulate_f32": [_P, _P, _I, _L, _P],
    "pf_split_gather": [_P, _P, _L, _L, _L, _P, _P],
    "pf_merge_scatter": [_P, _P, _L, _L, _L, _P, _P],
    "pf_embedding_fwd": [_P, _I, _P, _P, _I, _L, _L, _L, _P],
    "pf_embedding_bwd": [_P, _I, _P, _P, _L, _L, _L, _L, _P],
    "pf_mfma_rate": [_I, _P, _L, _I, _P, _P],
}
_RET_I64 = {"pf_colreduce_workspace": [_L, _L], "pf_reduce_workspace": [_L], "pf_groupnorm_workspace": [_L, _L, _I],
            "pf_colsum_static_capacity": []}
EXPORTED_SYMBOLS = sorted(list(_SIGNATURES) + list(_RET_I64) + ["pf_version", "pf_last_error"])

_lib = None


def load(path=None):
    """Load the shared library (once) and declare every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise RuntimeError(
            "pfeife_amd: %s is missing. Build it with `python -m pfeife_amd.hip.build` "
            "(hipcc, gfx950). There is no fallback path." % path
        )
    lib = ctypes.CDLL(path)
    lib.pf_version.restype = c_int
    lib.pf_version.argtypes = []
    lib.pf_last_error.restype = c_char_p
    lib.pf_last_error.argtypes = []
    for name, args in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = c_int
        fn.argtypes = args if args is not None else [c_int64]
    for name, args in _RET_I64.items():
        fn = getattr(lib, name)
        fn.restype = c_int64
        fn.argtypes = args
    if lib.pf_version() != ABI_VERSION:
        raise RuntimeError("pfeife_amd: library ABI %d != binding ABI %d" % (lib.pf_version(), ABI_VERSION))
    _lib = lib
    return lib


def last_error():
    return load().pf_last_error().decode("utf-8", "replace")


def _ptr(t):
    return None if t is None else t.data_ptr()


def _es(t):
    """bytes per element of a tensor operand (0 for an absent one)"""
    return 0 if t is None else t.element_size()


def _dt(t, default=PF_F32):
    return default if t is None else dtype_code(t.dtype)


def current_stream_ptr():
    return torch.cuda.current_stream().cuda_stream


class HipKernels:
    """Tensor-level kernel table backed by libpfeife_hip.so.

    Every public method returns a prepared launch `fn(stream)`; `run(name, ...)`
    prepares and immediately issues it on torch's current stream.
    """

    name = "hip"
    supports_graphs = True

    def __init__(self, device=None):
        self.lib = load()
        if not torch.cuda.is_available():
            raise RuntimeError("pfeife_amd: no GPU visible; the HIP kernel table cannot run")
        self.device = torch.device("cuda", torch.cuda.current_device() if device is None else device)
        rc = self.lib.pf_init(self.device.index or 0)
        if rc != 0:
            raise RuntimeError("pfeife_amd: pf_init failed: %s" % last_error())

    # -- helpers -------------------------------------------------------------
    def _prep(self, fname, args, keep, nbytes=None):
        """A prepared launch: `launch(stream)`.  `nbytes`: algorithmic HBM bytes of the launch (each
        operand touched once at its storage dtype), for harnesses that report achieved GB/s."""
        fn = getattr(self.lib, fname)
        lib = self.lib

        def launch(stream, _fn=fn, _args=args, _keep=keep, _name=fname):
            rc = _fn(*_args, stream)
            if rc != 0:
                raise RuntimeError("%s failed (%d): %s" % (_name, rc, lib.pf_last_error().decode()))

        launch.kernel = fname
        launch.bytes = nbytes
        return launch

    def run(self, name, *a, **kw):
        getattr(self, name)(*a, **kw)(current_stream_ptr())

    def capture(self, launches, stream):
        """Record `launches` (prepared launches) into a hipGraph on `stream`; returns a replay
        callable `fn(stream)` that issues the whole list with one host call."""
        lib = self.lib
        rc = lib.pf_graph_capture_begin(stream)
        if rc != 0:
            raise RuntimeError("graph capture: %s" % lib.pf_last_error().decode())
        try:
            for launch in launches:
                launch(stream)
        finally:
            handle = c_void_p()
            rc = lib.pf_graph_capture_end(stream, byref(handle))
        if rc != 0:
            raise RuntimeError("graph capture: %s" % lib.pf_last_error().decode())
        h = handle.value

        def replay(s, _h=h, _fn=lib.pf_graph_launch, _keep=launches):
            if _fn(_h, s) != 0:
                raise RuntimeError("graph launch: %s" % lib.pf_last_error().decode())

        replay.kernel = "pf_graph_launch"
        replay.handle = h
        return replay

    def destroy_graph(self, replay):
        """Frees the hipGraphExec behind a replay callable returned by `capture` (idempotent)."""
        h = getattr(replay, "handle", None)
        if h:
            replay.handle = None
            self.lib.pf_graph_destroy(h)

    def colreduce_workspace(self, rows, cols):
        return int(self.lib.pf_colreduce_workspace(rows, cols))

    def reduce_workspace(self, n):
        return int(self.lib.pf_reduce_workspace(n))

    # -- dense contractions ----------------------------------------------------
    def gemm(self, a, b, c, M, N, K, lda, ldb, ldc, a_trans=0, b_trans=0, batch=(1, 1), sa=(0, 0), sb=(0, 0),
             sc=(0, 0), alpha=1.0, beta=0, bias=None, round_mid=0, aux_out=None, ld_aux_out=0, act=0, dact=0,
             aux_in=None, ld_aux_in=0, residual=None, ld_res=0, variant=0, unscale_by=None, nonfinite_flag=None):
        if a.dtype != b.dtype:
            raise RuntimeError("gemm: operand dtypes differ (%s, %s)" % (a.dtype, b.dtype))
        d = GemmDesc()
        d.in_dtype, d.c_dtype = dtype_code(a.dtype), dtype_code(c.dtype)
        d.a_trans, d.b_trans = int(a_trans), int(b_trans)
        d.M, d.N, d.K = M, N, K
        d.A, d.lda, d.B, d.ldb, d.C, d.ldc = _ptr(a), lda, _ptr(b), ldb, _ptr(c), ldc
        d.batch1, d.batch2 = batch
        d.a_stride1, d.a_stride2 = sa
        d.b_stride1, d.b_stride2 = sb
        d.c_stride1, d.c_stride2 = sc
        d.alpha, d.beta = alpha, int(beta)
        d.bias, d.bias_dtype, d.round_mid = _ptr(bias), _dt(bias), int(round_mid)
        d.aux_out, d.ld_aux_out = _ptr(aux_out), ld_aux_out
        d.act, d.dact = int(act), int(dact)
        d.aux_in, d.ld_aux_in = _ptr(aux_in), ld_aux_in
        d.residual, d.ld_res, d.res_dtype = _ptr(residual), ld_res, _dt(residual)
        d.variant = int(variant)
        d.unscale_by, d.nonfinite_flag = _ptr(unscale_by), _ptr(nonfinite_flag)
        for t in (unscale_by, nonfinite_flag):
            if t is not None and t.dtype != torch.float32:
                raise RuntimeError("gemm: unscale_by / nonfinite_flag are fp32 device scalars")
        for t in (aux_out, aux_in):
            if t is not None and t.dtype != a.dtype:
                raise RuntimeError("gemm: aux tensors must have the operand dtype")
        launch = self._prep("pf_gemm", (byref(d),), (d, a, b, c, bias, aux_out, aux_in, residual, unscale_by, nonfinite_flag))
        name = ctypes.create_string_buffer(128)
        self.lib.pf_gemm_variant(byref(d), name, 128)
        launch.variant = name.value.decode()
        launch.group_key = self._group_key(launch.variant)
        launch.flops = 2.0 * M * N * K * batch[0] * batch[1]
        launch.desc = d
        return launch

    def gemm_attach_colsum(self, launch, alloc):
        """Make a prepared product with a fused GELU' epilogue on the direct-to-LDS kernel also leave the
        column sums of what it stores (the bias gradient of the layer whose pre-activation gradient it
        writes) as partial rows.  alloc(shape, dtype) -> workspace tensor that outlives the launch.
        -> (workspace, offset, partial rows, row stride) for the deferred finish, or None when the
        launch runs on another kernel."""
        v = getattr(launch, "variant", "")
        d = getattr(launch, "desc", None)
        if d is None or not (v.startswith("gemm16x_kernel<") and v.endswith(", false, false, 5>")):
            return None
        if d.batch1 * d.batch2 != 1 or d.colsum_ws:
            return None
        bm = int(v.split("<")[1].split(",")[1])
        nb = (d.M + bm - 1) // bm
        ws = alloc((nb, d.N), torch.float32)
        d.colsum_ws = ws.data_ptr()
        launch.colsum_ws = ws
        return ws, 0, nb, d.N

    def gemm_retiled(self, launch, variant):
        """The same product pinned to another kernel variant (see `pf_gemm_desc.variant`), or None when
        that variant cannot run it."""
        d = GemmDesc()
        ctypes.memmove(ctypes.byref(d), ctypes.byref(launch.desc), ctypes.sizeof(GemmDesc))
        d.variant = int(variant)
        name = ctypes.create_string_buffer(128)
        if self.lib.pf_gemm_variant(byref(d), name, 128) != 0:
            return None
        new = self._prep("pf_gemm", (byref(d),), (d, launch))
        new.variant = name.value.decode()
        new.group_key = self._group_key(new.variant)
        new.flops = launch.flops
        new.desc = d
        return new

    GEMM_GROUP_MAX = 8      # PF_GEMM_GROUP_MAX

    @staticmethod
    def _group_key(variant):
        """Weight-gradient products that store (class 1) and that accumulate (class 4) share the
        accumulate launch of their tile: one key for both."""
        if variant.startswith("gemm16x_kernel<") and variant.endswith("true, true, 1>"):
            return variant[:-3] + " 4>"
        return variant

    @staticmethod
    def gemm_groupable(launch):
        """A weight-gradient product on the direct-to-LDS kernel (fp32 C stored or accumulated):
        launches of this kind with the same `group_key` may share one launch (pf_gemm_grouped)."""
        v = getattr(launch, "group_key", "")
        return v.startswith("gemm16x_kernel<") and v.endswith("true, true, 4>")

    @staticmethod
    def gemm_stores_checked(launch):
        """Does this product run on a kernel whose epilogue honours `nonfinite_flag` (the fp32 classes
        of the direct-to-LDS kernel)?"""
        return HipKernels.gemm_groupable(launch)

    def gemm_group(self, launches):
        """One launch for 2..GEMM_GROUP_MAX independent `gemm_groupable` products of the same variant."""
        n = len(launches)
        if not (2 <= n <= self.GEMM_GROUP_MAX) or len({l.group_key for l in launches}) != 1 \
                or not all(self.gemm_groupable(l) for l in launches):
            raise RuntimeError("gemm_group: needs 2..%d groupable launches of one variant" % self.GEMM_GROUP_MAX)
        arr = (GemmDesc * n)()
        for i, l in enumerate(launches):
            ctypes.memmove(ctypes.byref(arr[i]), ctypes.byref(l.desc), ctypes.sizeof(GemmDesc))
        launch = self._prep("pf_gemm_grouped", (arr, n), (arr, launches))
        launch.variant = launches[0].group_key.replace("gemm16x_kernel<", "gemm16x_group_kernel<")
        launch.group_key = launch.variant
        launch.flops = sum(l.flops for l in launches)
        launch.members = list(launches)
        return launch

    # -- fused attention -----------------------------------------------------------
    MAX_FUSED_HEAD_DIM = 96

    @staticmethod
    def _attn_desc(q, k, v, o, lse, scale, causal, d_o=None, dq=None, dk=None, dv=None, delta=None):
        d = AttnDesc()
        Bn, H, Tq, hd = q.shape
        d.dtype, d.B, d.H, d.Tq, d.Tk, d.hd, d.causal = dtype_code(q.dtype), Bn, H, Tq, k.shape[2], hd, int(causal)
        d.scale = float(scale)
        d.q, d.k, d.v, d.o, d.lse = _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse)
        d.d_o, d.dq, d.dk, d.dv, d.delta = _ptr(d_o), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(delta)
        for name, t in (("q", q), ("k", k), ("v", v), ("o", o), ("do", d_o), ("dq", dq), ("dk", dk), ("dv", dv)):
            if t is None:
                continue
            if t.dim() != 4 or t.stride(3) != 1 or t.dtype != q.dtype:
                raise RuntimeError("attention operand %s must be a [B,H,T,hd] tensor with unit hd stride" % name)
            setattr(d, name + "_sb", t.stride(0))
            setattr(d, name + "_sh", t.stride(1))
            setattr(d, name + "_st", t.stride(2))
        return d

    def attention_fwd(self, q, k, v, o, lse, scale, causal):
        d = self._attn_desc(q, k, v, o, lse, scale, causal)
        return self._prep("pf_attention_fwd", (byref(d),), (d, q, k, v, o, lse))

    def attention_bwd(self, q, k, v, o, d_o, lse, delta, dq, dk, dv, scale, causal):
        d = self._attn_desc(q, k, v, o, lse, scale, causal, d_o, dq, dk, dv, delta)
        return self._prep("pf_attention_bwd", (byref(d),), (d, q, k, v, o, d_o, lse, delta, dq, dk, dv))

    # -- normalisation -----------------------------------------------------------
    def layernorm_fwd(self, x, gamma, beta, y, mean, rstd, rows, d, eps):
        args = (_ptr(x), _dt(x), _ptr(gamma), _ptr(beta), _ptr(y), _dt(y), _ptr(mean), _ptr(rstd), rows, d, eps)
        return self._prep("pf_layernorm_fwd", args, (x, gamma, beta, y, mean, rstd), rows * d * (_es(x) + _es(y)))

    def layernorm_bwd(self, dy, x, gamma, mean, rstd, dx_add, dx, dgamma, dbeta, ws, rows, d, defer=0):
        args = (_ptr(dy), _dt(dy), _ptr(x), _dt(x), _ptr(gamma), _ptr(mean), _ptr(rstd), _ptr(dx_add), _dt(dx_add),
                _ptr(dx), _dt(dx), _ptr(dgamma), _ptr(dbeta), _ptr(ws), rows, d, int(defer))
        return self._prep("pf_layernorm_bwd", args, (dy, x, gamma, mean, rstd, dx_add, dx, dgamma, dbeta, ws),
                          rows * d * (_es(dy) + _es(x) + _es(dx) + _es(dx_add)))

    def norm_bwd_fused(self, dy, x, gamma, mean, rstd, dx_add, dx, dx_lp, ws, rows, d, want_wgrad, want_colsum):
        """Layer/RMS-norm backward (mean None: RMS) that also writes a 16-bit copy of dx and, with
        want_colsum, its column sums; partial rows [dgamma | dbeta | colsum] go to ws."""
        n = NormBwdDesc()
        n.dy, n.x, n.gamma, n.mean, n.rstd = _ptr(dy), _ptr(x), _ptr(gamma), _ptr(mean), _ptr(rstd)
        n.dx_add, n.dx, n.dx_lp, n.workspace = _ptr(dx_add), _ptr(dx), _ptr(dx_lp), _ptr(ws)
        n.rows, n.d = rows, d
        n.dy_dtype, n.x_dtype, n.add_dtype, n.dx_dtype = _dt(dy), _dt(x), _dt(dx_add), _dt(dx)
        n.dx_lp_dtype = _dt(dx_lp)
        n.want_wgrad, n.want_colsum = int(bool(want_wgrad)), int(bool(want_colsum))
        return self._prep("pf_norm_bwd_fused", (byref(n),), (n, dy, x, gamma, mean, rstd, dx_add, dx, dx_lp, ws),
                          rows * d * (_es(dy) + _es(x) + _es(dx) + _es(dx_add) + _es(dx_lp)))

    def groupnorm_workspace(self, B, C, groups):
        return int(self.lib.pf_groupnorm_workspace(B, C, groups))

    def groupnorm_fwd(self, x, gamma, beta, y, mean, rstd, B, HW, C, groups, eps):
        args = (_ptr(x), _dt(x), _ptr(gamma), _ptr(beta), _ptr(y), _dt(y), _ptr(mean), _ptr(rstd), B, HW, C, groups,
                eps)
        return self._prep("pf_groupnorm_fwd", args, (x, gamma, beta, y, mean, rstd), B * HW * C * (2 * _es(x) + _es(y)))

    def groupnorm_bwd(self, dy, x, gamma, mean, rstd, dx, dgamma, dbeta, ws, B, HW, C, groups, defer=0):
        args = (_ptr(dy), _dt(dy), _ptr(x), _dt(x), _ptr(gamma), _ptr(mean), _ptr(rstd), _ptr(dx), _dt(dx),
                _ptr(dgamma), _ptr(dbeta), _ptr(ws), B, HW, C, groups, int(defer))
        return self._prep("pf_groupnorm_bwd", args, (dy, x, gamma, mean, rstd, dx, dgamma, dbeta, ws),
                          B * HW * C * (2 * _es(dy) + 2 * _es(x) + _es(dx)))

    def rmsnorm_fwd(self, x, gamma, y, rstd, rows, d, eps):
        args = (_ptr(x), _dt(x), _ptr(gamma), _ptr(y), _dt(y), _ptr(rstd), rows, d, eps)
        return self._prep("pf_rmsnorm_fwd", args, (x, gamma, y, rstd), rows * d * (_es(x) + _es(y)))

    def rmsnorm_bwd(self, dy, x, gamma, rstd, dx_add, dx, dgamma, ws, rows, d, defer=0):
        args = (_ptr(dy), _dt(dy), _ptr(x), _dt(x), _ptr(gamma), _ptr(rstd), _ptr(dx_add), _dt(dx_add), _ptr(dx),
                _dt(dx), _ptr(dgamma), _ptr(ws), rows, d, int(defer))
        return self._prep("pf_rmsnorm_bwd", args, (dy, x, gamma, rstd, dx_add, dx, dgamma, ws),
                          rows * d * (_es(dy) + _es(x) + _es(dx) + _es(dx_add)))

    def colsum_accumulate(self, x, rows, cols, ld, acc, ws, defer=0):
        args = (_ptr(x), _dt(x), rows, cols, ld, _ptr(acc), _ptr(ws), int(defer))
        return self._prep("pf_colsum_accumulate", args, (x, acc, ws), rows * cols * _es(x))

    def norm_bwd_partials(self, rows):
        return int(self.lib.pf_norm_bwd_partials(rows))

    def colsum_partials(self, rows):
        return int(self.lib.pf_colsum_partials(rows))

    def colreduce_finalize_batch(self, items):
        """items: [(ws_tensor, ws_offset_elems, n_partials, stride, cols, acc_tensor)]"""
        if not items:
            return lambda stream: None
        rows = []
        for ws, off, n, stride, cols, acc in items:
            rows.append([ws.data_ptr() + 4 * off, acc.data_ptr(), int(n), int(stride), int(cols)])
        table = torch.tensor(rows, dtype=torch.int64).to(items[0][0].device)
        max_cols = max(r[4] for r in rows)
        keep = (table,) + tuple(i[0] for i in items) + tuple(i[5] for i in items)
        nbytes = sum(4 * (r[2] + 2) * r[4] for r in rows)   # partial rows read, accumulator read and written
        return self._prep("pf_colreduce_finalize_batch", (table.data_ptr(), len(rows), max_cols), keep, nbytes)

    # -- softmax / losses ----------------------------------------------------------
    def softmax_fwd(self, s, ld_s, p, ld_p, rows, cols, q_len, causal):
        args = (_ptr(s), ld_s, _ptr(p), _dt(p), ld_p, rows, cols, q_len, int(causal))
        return self._prep("pf_softmax_fwd", args, (s, p), rows * cols * (_es(s) + _es(p)))

    def softmax_bwd(self, dp, ld_dp, p, ld_p, ds, ld_ds, rows, cols, scale):
        args = (_ptr(dp), ld_dp, _ptr(p), _dt(p), ld_p, _ptr(ds), _dt(ds), ld_ds, rows, cols, scale)
        return self._prep("pf_softmax_bwd", args, (dp, p, ds), rows * cols * (_es(dp) + _es(p) + _es(ds)))

    def cross_entropy_fwd(self, logits, targets, row_loss, row_lse, loss, rows, classes, ignore_index):
        args = (_ptr(logits), _dt(logits), _ptr(targets), _ptr(row_loss), _ptr(row_lse), _ptr(loss), rows, classes,
                ignore_index)
        return self._prep("pf_cross_entropy_fwd", args, (logits, targets, row_loss, row_lse, loss), rows * classes * _es(logits))

    def cross_entropy_bwd(self, logits, targets, row_lse, dloss, loss, dlogits, rows, classes, ignore_index):
        n_valid = loss.data_ptr() + 4
        args = (_ptr(logits), _dt(logits), _ptr(targets), _ptr(row_lse), _ptr(dloss), n_valid, _ptr(dlogits),
                _dt(dlogits), rows, classes, ignore_index)
        return self._prep("pf_cross_entropy_bwd", args, (logits, targets, row_lse, dloss, loss, dlogits),
                          rows * classes * (_es(logits) + _es(dlogits)))

    def mse_fwd(self, a, b, partial, loss, n):
        args = (_ptr(a), _dt(a), _ptr(b), _dt(b), _ptr(partial), _ptr(loss), n)
        return self._prep("pf_mse_fwd", args, (a, b, partial, loss))

    def mse_bwd(self, a, b, dloss, da, n):
        args = (_ptr(a), _dt(a), _ptr(b), _dt(b), _ptr(dloss), _ptr(da), _dt(da), n)
        return self._prep("pf_mse_bwd", args, (a, b, dloss, da))

    def sum_fwd(self, x, partial, loss, n):
        args = (_ptr(x), _dt(x), _ptr(partial), _ptr(loss), n)
        return self._prep("pf_sum_fwd", args, (x, partial, loss))

    # -- elementwise -----------------------------------------------------------------
    def act_fwd(self, x, y, act, n):
        return self._prep("pf_act_fwd", (_ptr(x), _ptr(y), _dt(x), int(act), n), (x, y), 2 * n * _es(x))

    def act_bwd(self, dy, x, dx, act, n):
        return self._prep("pf_act_bwd", (_ptr(dy), _ptr(x), _ptr(dx), _dt(x), int(act), n), (dy, x, dx), 3 * n * _es(x))

    def glu_fwd(self, gate, ld_gate, up, ld_up, y, ld_y, act, rows, cols):
        args = (_ptr(gate), ld_gate, _ptr(up), ld_up, _ptr(y), ld_y, _dt(gate), int(act), rows, cols)
        return self._prep("pf_glu_fwd", args, (gate, up, y), 3 * rows * cols * _es(gate))

    def glu_bwd(self, dy, ld_dy, gate, ld_gate, up, ld_up, dgate, ld_dgate, dup, ld_dup, act, rows, cols):
        args = (_ptr(dy), ld_dy, _ptr(gate), ld_gate, _ptr(up), ld_up, _ptr(dgate), ld_dgate, _ptr(dup), ld_dup,
                _dt(gate), int(act), rows, cols)
        return self._prep("pf_glu_bwd", args, (dy, gate, up, dgate, dup), 5 * rows * cols * _es(gate))

    def axpby(self, a, alpha, b, beta, out, n):
        args = (_ptr(a), _dt(a), alpha, _ptr(b), _dt(b), beta, _ptr(out), _dt(out), n)
        return self._prep("pf_axpby", args, (a, b, out), n * (_es(a) + _es(b) + _es(out)))

    def bias_add(self, x, bias, y, n, bias_len, rows_per_bias=0):
        args = (_ptr(x), _dt(x), _ptr(bias), _dt(bias), _ptr(y), _dt(y), n, bias_len, rows_per_bias)
        return self._prep("pf_bias_add", args, (x, bias, y))

    def cast(self, src, dst, n):
        return self._prep("pf_cast", (_ptr(src), _dt(src), _ptr(dst), _dt(dst), n), (src, dst), n * (_es(src) + _es(dst)))

    def cast_batch(self, pairs):
        """One launch casting every (src, dst) pair of contiguous tensors."""
        rows = []
        for src, dst in pairs:
            vec = 1 if (src.data_ptr() % 16 == 0 and dst.data_ptr() % 16 == 0) else 0
            rows.append([src.data_ptr(), dst.data_ptr(), src.numel(),
                         dtype_code(src.dtype) | (dtype_code(dst.dtype) << 32), vec])
        table = torch.tensor(rows, dtype=torch.int64).to(pairs[0][1].device)
        args = (table.data_ptr(), len(rows), max(r[2] for r in rows))
        return self._prep("pf_cast_batch", args, (table, pairs))

    @staticmethod
    def shadow_batch_ok(src, plain, transposed):
        """Can pf_shadow_batch make these shadows of the contiguous fp32 matrix `src`?"""
        if src.dim() != 2 or src.dtype != torch.float32 or not src.is_contiguous():
            return False
        if src.shape[0] % 4 or src.shape[1] % 4 or src.data_ptr() % 16:
            return False
        return all(t is None or (t.is_contiguous() and t.data_ptr() % 8 == 0 and t.dtype in (torch.float16, torch.bfloat16))
                   for t in (plain, transposed))

    def shadow_batch(self, items):
        """One launch writing the plain and/or transposed 16-bit shadow of every (src, plain, transposed)."""
        rows = []
        for src, plain, tr in items:
            r, c = src.shape
            dt = dtype_code((plain if plain is not None else tr).dtype)
            rows.append([src.data_ptr(), 0 if plain is None else plain.data_ptr(), 0 if tr is None else tr.data_ptr(),
                         r, c, dt])
        table = torch.tensor(rows, dtype=torch.int64).to(items[0][0].device)
        tiles = max(((r[3] + 63) // 64) * ((r[4] + 63) // 64) for r in rows)
        nbytes = sum(r[3] * r[4] * (4 + 2 * (r[1] != 0) + 2 * (r[2] != 0)) for r in rows)
        return self._prep("pf_shadow_batch", (table.data_ptr(), len(rows), tiles), (table, items), nbytes)

    def transpose_cast(self, src, ld_src, dst, ld_dst, rows, cols):
        args = (_ptr(src), _dt(src), ld_src, _ptr(dst), _dt(dst), ld_dst, rows, cols)
        return self._prep("pf_transpose_cast", args, (src, dst), rows * cols * (_es(src) + _es(dst)))

    def adam_table(self, params, grads, exp_avgs, exp_avg_sqs):
        """Device table of pf_adam_item for one param group (built once, pointers are static)."""
        rows = [[p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), p.numel()]
                for p, g, m, v in zip(params, grads, exp_avgs, exp_avg_sqs)]
        for r in rows:
            if any(x % 16 for x in r[:4]):
                raise RuntimeError("adam: tensors must be 16-byte aligned")
        table = torch.tensor(rows, dtype=torch.int64).to(params[0].device)
        return table, len(rows), max(r[4] for r in rows)

    def adam_step(self, table, n_items, max_n, lr, beta1, beta2, eps, weight_decay, step, adamw, stream):
        rc = self.lib.pf_adam_step(table.data_ptr(), n_items, max_n, lr, beta1, beta2, eps, weight_decay, step,
                                   int(adamw), stream)
        if rc != 0:
            raise RuntimeError("pf_adam_step failed: %s" % self.lib.pf_last_error().decode())

    def adam_step_scaled(self, table, n_items, max_n, lr, beta1, beta2, eps, weight_decay, adamw, state, stream):
        rc = self.lib.pf_adam_step_scaled(table.data_ptr(), n_items, max_n, lr, beta1, beta2, eps, weight_decay,
                                          int(adamw), state.data_ptr(), stream)
        if rc != 0:
            raise RuntimeError("pf_adam_step_scaled failed: %s" % self.lib.pf_last_error().decode())

    # -- dynamic loss scaling (state: float32[8] on the device) ----------------------------
    def scale_by_state(self, src, state, dst, n):
        return self._prep("pf_scale_by_state", (_ptr(src), _dt(src), _ptr(state), _ptr(dst), _dt(dst), n),
                          (src, state, dst), n * (_es(src) + _es(dst)))

    def scaler_unscale(self, grads, n, state):
        return self._prep("pf_scaler_unscale", (_ptr(grads), n, _ptr(state)), (grads, state), 8 * n)

    def scaler_update(self, state, growth_factor, backoff_factor, growth_interval):
        return self._prep("pf_scaler_update", (_ptr(state), float(growth_factor), float(backoff_factor),
                                               int(growth_interval)), (state,))

    def fill(self, dst, value, n):
        return self._prep("pf_fill", (_ptr(dst), _dt(dst), float(value), n), (dst,))

    def mfma_rate(self, operands, iters, workgroups, sink):
        """Measurement aid: the GEMM tile's matrix-instruction stream alone (see pf_mfma_rate)."""
        assert operands.numel() >= 4096 and sink.numel() >= 256 * workgroups and sink.dtype == torch.float32
        return self._prep("pf_mfma_rate", (_dt(operands), _ptr(operands), int(iters), int(workgroups), _ptr(sink)), (operands, sink))

    def copy_strided(self, src, src_strides, dst, dst_strides, sizes, accumulate=0):
        nd = len(sizes)
        arr = c_int64 * nd
        ss, ds, sz = arr(*src_strides), arr(*dst_strides), arr(*sizes)
        args = (_ptr(src), _dt(src), ss, _ptr(dst), _dt(dst), ds, sz, nd, int(accumulate))
        return self._prep("pf_copy_strided", args, (src, dst, ss, ds, sz))

    def rope(self, x, y, cos_t, sin_t, B, T, H, D, xs, ys, inverse, tab_ld=None):
        tab_ld = D // 2 if tab_ld is None else tab_ld
        args = (_ptr(x), _ptr(y), _dt(x), _ptr(cos_t), _ptr(sin_t), tab_ld, B, T, H, D, xs[0], xs[1], xs[2], ys[0],
                ys[1], ys[2], int(inverse))
        return self._prep("pf_rope", args, (x, y, cos_t, sin_t))

    def grad_accumulate(self, acc, g, n):
        return self._prep("pf_grad_accumulate_f32", (_ptr(acc), _ptr(g), _dt(g), n), (acc, g), n * (8 + _es(g)))

    # -- micro-batch split / merge, embedding ---------------------------------------------
    def split_gather(self, src, dst, row_bytes, row_start, n_rows, index=None):
        args = (_ptr(src), _ptr(dst), row_bytes, row_start, n_rows, _ptr(index))
        return self._prep("pf_split_gather", args, (src, dst, index))

    def merge_scatter(self, src, dst, row_bytes, row_start, n_rows, index=None):
        args = (_ptr(src), _ptr(dst), row_bytes, row_start, n_rows, _ptr(index))
        return self._prep("pf_merge_scatter", args, (src, dst, index))

    def embedding_fwd(self, table, ids, out, n_ids, dim, vocab):
        args = (_ptr(table), _dt(table), _ptr(ids), _ptr(out), _dt(out), n_ids, dim, vocab)
        return self._prep("pf_embedding_fwd", args, (table, ids, out))

    def embedding_bwd(self, dout, ids, dtable, n_ids, dim, vocab, padding_idx=-1):
        args = (_ptr(dout), _dt(dout), _ptr(ids), _ptr(dtable), n_ids, dim, vocab, int(padding_idx))
        return self._prep("pf_embedding_bwd", args, (dout, ids, dtable))
