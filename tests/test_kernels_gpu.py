"""Parity of every HIP kernel (through the C ABI) against the CPU oracle on the
same seeded inputs.  Integer / byte movers must be bit-exact; floating-point
kernels must agree within the tolerance written next to each test."""
import itertools

import pytest
import torch

pytestmark = pytest.mark.gpu

F16, BF16, F32 = torch.float16, torch.bfloat16, torch.float32


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def both(hip, oracle, name, tensors, outs, **scalars):
    """Run kernel `name` on the GPU (HIP) and on CPU (oracle) from identical
    inputs; returns {out_name: (hip_result_on_cpu, oracle_result)}."""
    print("kernel", name, {k: (tuple(v.shape), str(v.dtype)) for k, v in tensors.items() if v is not None},
          scalars, flush=True)
    dev = {k: (None if v is None else v.cuda()) for k, v in tensors.items()}
    cpu = {k: (None if v is None else v.clone()) for k, v in tensors.items()}
    hip.run(name, **dev, **scalars)
    torch.cuda.synchronize()
    oracle.run(name, **cpu, **scalars)
    return {o: (dev[o].cpu(), cpu[o]) for o in outs}


def close(pair, rtol, atol):
    a, b = pair
    assert a.dtype == b.dtype and a.shape == b.shape
    torch.testing.assert_close(a.float(), b.float(), rtol=rtol, atol=atol)


TOL = {F32: (2e-5, 2e-5), F16: (4e-3, 4e-3), BF16: (2e-2, 2e-2)}

GEMM_SHAPES = [(197, 197, 64), (130, 72, 200), (257, 1000, 88), (512, 384, 1024), (64, 64, 8), (1, 8, 8)]


@pytest.mark.parametrize("dtype", [F16, BF16, F32])
@pytest.mark.parametrize("a_trans,b_trans", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_layouts(hip, oracle, dtype, a_trans, b_trans):
    for i, (M, N, K) in enumerate(GEMM_SHAPES):
        def ld8(v):  # 16-bit operands need leading dimensions that are multiples of 8
            return (v + 7) // 8 * 8 + 8

        lda = ld8(M if a_trans else K)
        ldb = ld8(N if b_trans else K)
        ldc = N + 3
        a = rnd((K if a_trans else M, lda), dtype, 10 + i)
        b = rnd((K if b_trans else N, ldb), dtype, 20 + i)
        c = torch.zeros(M, ldc, dtype=F32)
        r = both(hip, oracle, "gemm", dict(a=a, b=b, c=c), ["c"], M=M, N=N, K=K, lda=lda, ldb=ldb, ldc=ldc,
                 a_trans=a_trans, b_trans=b_trans, alpha=0.5)
        # fp32 accumulation of the same 16-bit products: only the summation order differs
        close(r["c"], rtol=1e-4, atol=1e-4 * (K ** 0.5))
        assert torch.all(r["c"][0][:, N:] == 0), "columns beyond N were written"


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_gemm_batched_strided_heads(hip, oracle, dtype):
    # attention layout: packed qkv [B, T, 3, H, hd]; S = Q K^T per (b, h); then P V
    B, T, H, hd = 2, 197, 3, 64
    C = H * hd
    qkv = rnd((B, T, 3 * C), dtype, 1, 0.5)
    Tp = 200
    s = torch.zeros(B, H, T, Tp, dtype=F32)
    q, k, v = qkv[:, :, 0:C], qkv[:, :, C:2 * C], qkv[:, :, 2 * C:]
    res = {}
    for name, tab, dev in (("hip", hip, "cuda"), ("oracle", oracle, "cpu")):
        t = qkv.to(dev)
        S = s.to(dev)
        tab.run("gemm", t[:, :, 0:C], t[:, :, C:2 * C], S, M=T, N=T, K=hd, lda=3 * C, ldb=3 * C, ldc=Tp,
                batch=(B, H), sa=(T * 3 * C, hd), sb=(T * 3 * C, hd), sc=(H * T * Tp, T * Tp), alpha=hd ** -0.5)
        P = torch.softmax(S[..., :T].float().cpu(), -1).to(dtype)
        Pp = torch.zeros(B, H, T, Tp, dtype=dtype)
        Pp[..., :T] = P
        Pp = Pp.to(dev)
        O = torch.zeros(B, T, C, dtype=dtype, device=dev)
        tab.run("gemm", Pp, t[:, :, 2 * C:], O, M=T, N=hd, K=T, lda=Tp, ldb=3 * C, ldc=C, b_trans=1, batch=(B, H),
                sa=(H * T * Tp, T * Tp), sb=(T * 3 * C, hd), sc=(T * C, hd))
        if dev == "cuda":
            torch.cuda.synchronize()
        res[name] = (S.cpu(), O.cpu())
    close((res["hip"][0], res["oracle"][0]), rtol=1e-4, atol=1e-3)
    close((res["hip"][1], res["oracle"][1]), *TOL[dtype])
    ref = torch.nn.functional.scaled_dot_product_attention(
        *(x.reshape(B, T, H, hd).transpose(1, 2).float() for x in (q, k, v))).transpose(1, 2).reshape(B, T, C)
    torch.testing.assert_close(res["hip"][1].float(), ref, rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("dtype", [F16, BF16, F32])
def test_gemm_epilogues(hip, oracle, dtype):
    M, N, K = 300, 264, 136
    x, w = rnd((M, K), dtype, 1), rnd((N, K), dtype, 2, 0.1)
    bias = rnd((N,), dtype, 3)
    rt, at = TOL[dtype]
    # forward linear + bias + GELU, pre-activation kept
    r = both(hip, oracle, "gemm", dict(a=x, b=w, c=torch.zeros(M, N, dtype=dtype), bias=bias,
                                      aux_out=torch.zeros(M, N, dtype=dtype)), ["c", "aux_out"],
             M=M, N=N, K=K, lda=K, ldb=K, ldc=N, round_mid=1, act=1, ld_aux_out=N)
    close(r["c"], rt, at)
    close(r["aux_out"], rt, at)
    # backward through GELU: dH = (dY W) * gelu'(h)
    dy = rnd((M, N), dtype, 4)
    h = rnd((M, K), dtype, 5)
    r = both(hip, oracle, "gemm", dict(a=dy, b=w, c=torch.zeros(M, K, dtype=dtype), aux_in=h), ["c"],
             M=M, N=K, K=N, lda=N, ldb=K, ldc=K, b_trans=1, dact=1, ld_aux_in=K)
    close(r["c"], rt, at * 4)
    # residual add into an fp32 stream
    res = rnd((M, N), F32, 6)
    r = both(hip, oracle, "gemm", dict(a=x, b=w, c=torch.zeros(M, N, dtype=F32), bias=bias, residual=res), ["c"],
             M=M, N=N, K=K, lda=K, ldb=K, ldc=N, round_mid=1, ld_res=N)
    close(r["c"], rt, at)
    # weight gradient accumulated into fp32 (beta = 1)
    acc = rnd((N, K), F32, 7)
    r = both(hip, oracle, "gemm", dict(a=dy, b=x, c=acc), ["c"], M=N, N=K, K=M, lda=N, ldb=K, ldc=K, a_trans=1,
             b_trans=1, beta=1)
    close(r["c"], rtol=1e-4, atol=2e-3)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("variant,tile", [(1, "256, 256, 32, 2, 2, 1, 5"), (2, "256, 128, 64, 2, 2, 1, 3"), (3, "128, 128, 64, 2, 2, 1, 3"),
                                          (4, "192, 256, 32, 2, 2, 1, 5"), (5, "128, 128, 64, 2, 2, 2, 3"), (6, "256, 128, 64, 2, 2, 2, 3"),
                                          (7, "256, 256, 32, 2, 4, 1, 5"), (8, "128, 128, 64, 2, 4, 1, 3"), (9, "256, 128, 64, 4, 2, 1, 3")])
def test_gemm_direct_to_lds_epilogue_classes(hip, oracle, dtype, variant, tile):
    """Every straight-line epilogue class of the direct-to-LDS kernel on every tile shape, ragged in M
    (and in N against the 256- and 192-wide tiles), against the oracle; the launch names the class."""
    M, N, K = 1000, 1160, 320
    dt = {F16: 1, BF16: 2}[dtype]
    x, w = rnd((M, K), dtype, 1), rnd((N, K), dtype, 2, 0.1)
    bias = rnd((N,), dtype, 3)
    rt, at = TOL[dtype]

    def run(ec, tensors, outs, **kw):
        print("gemm variant", variant, "class", ec, flush=True)
        dev = {k: (None if v is None else v.cuda()) for k, v in tensors.items()}
        cpu = {k: (None if v is None else v.clone()) for k, v in tensors.items()}
        launch = hip.gemm(**dev, variant=variant, **kw)
        assert launch.variant == "gemm16x_kernel<%d, %s, false, false, %d>" % (dt, tile, ec), launch.variant
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        oracle.gemm(**cpu, **kw)()
        return {o: (dev[o].cpu(), cpu[o]) for o in outs}

    base = dict(M=M, N=N, K=K, lda=K, ldb=K, ldc=N)
    z16 = lambda: torch.zeros(M, N, dtype=dtype)
    r = run(0, dict(a=x, b=w, c=z16(), bias=bias), ["c"], round_mid=1, **base)
    close(r["c"], rt, at)
    r = run(1, dict(a=x, b=w, c=torch.zeros(M, N, dtype=F32), bias=bias), ["c"], **base)
    close(r["c"], 1e-3, 1e-2)
    r = run(2, dict(a=x, b=w, c=z16(), bias=bias, aux_out=z16()), ["c", "aux_out"], round_mid=1, act=1, ld_aux_out=N, **base)
    close(r["c"], rt, at)
    close(r["aux_out"], rt, at)
    r = run(3, dict(a=x, b=w, c=torch.zeros(M, N, dtype=F32), bias=bias, residual=rnd((M, N), F32, 4)), ["c"],
            round_mid=1, ld_res=N, **base)
    close(r["c"], rt, at)
    r = run(4, dict(a=x, b=w, c=rnd((M, N), F32, 5)), ["c"], beta=1, **base)
    close(r["c"], 1e-3, 1e-2)
    r = run(5, dict(a=x, b=w, c=z16(), aux_in=rnd((M, N), dtype, 6)), ["c"], dact=1, ld_aux_in=N, **base)
    close(r["c"], rt, at * 4)
    r = run(6, dict(a=x, b=w, c=rnd((M, N), dtype, 7)), ["c"], beta=1, **base)
    close(r["c"], rt, at * 2)
    # 16-bit residual stream (UNet transformer blocks under autocast): residual row stride wider than N
    res16 = rnd((M, N + 8), dtype, 8)
    r = run(7, dict(a=x, b=w, c=z16(), bias=bias, residual=res16), ["c"], round_mid=1, ld_res=N + 8, **base)
    close(r["c"], rt, at * 2)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("variant,tile", [(1, "256, 256, 32, 2, 2, 1, 5"), (2, "256, 128, 64, 2, 2, 1, 3"), (3, "128, 128, 64, 2, 2, 1, 3"),
                                          (5, "128, 128, 64, 2, 2, 2, 3"), (6, "256, 128, 64, 2, 2, 2, 3"), (7, "256, 256, 32, 2, 4, 1, 5"),
                                          (8, "128, 128, 64, 2, 4, 1, 3"), (9, "256, 128, 64, 4, 2, 1, 3")])
def test_gemm_direct_to_lds_weight_gradient_tiles(hip, oracle, dtype, variant, tile):
    """The reduction-strided (weight-gradient) form of every tile that has one: dW += dY^T X with a
    ragged reduction length (not a multiple of any stage depth) and ragged M and N, fp32 accumulate
    and fp32 store, against the oracle."""
    rows, M, N = 1000, 1160, 520
    dt = {F16: 1, BF16: 2}[dtype]
    dy, x = rnd((rows, M), dtype, 1), rnd((rows, N), dtype, 2, 0.1)
    for ec, beta in ((4, 1), (1, 0)):
        print("gemm variant", variant, "transposed class", ec, flush=True)
        c0 = rnd((M, N), F32, 3)
        dev = dict(a=dy.cuda(), b=x.cuda(), c=c0.clone().cuda())
        cpu = dict(a=dy, b=x, c=c0.clone())
        kw = dict(M=M, N=N, K=rows, lda=M, ldb=N, ldc=N, a_trans=1, b_trans=1, beta=beta)
        launch = hip.gemm(**dev, variant=variant, **kw)
        assert launch.variant == "gemm16x_kernel<%d, %s, true, true, %d>" % (dt, tile, ec), launch.variant
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        oracle.gemm(**cpu, **kw)()
        close((dev["c"].cpu(), cpu["c"]), 1e-3, 2e-2)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("variant,bm", [(1, 256), (2, 256), (3, 128), (4, 192), (5, 128), (6, 256), (7, 256), (8, 128), (9, 256)])
def test_gemm_gelu_grad_epilogue_leaves_column_sums(hip, dtype, variant, bm):
    """The GELU' epilogue of the direct-to-LDS kernel can also leave the column sums of the values it
    stores (the bias gradient of the layer whose pre-activation gradient it writes) as one partial row
    per tile row: their sum must equal the column sums of the stored 16-bit matrix (fp32 adds of the
    same numbers in another order), ragged in M and N; the output itself must not change."""
    M, N, K = 1000, 1160, 320
    x, w = rnd((M, K), dtype, 1).cuda(), rnd((N, K), dtype, 2, 0.1).cuda()
    pre = rnd((M, N), dtype, 6).cuda()
    kw = dict(M=M, N=N, K=K, lda=K, ldb=K, ldc=N, dact=1, ld_aux_in=N, variant=variant)
    plain = torch.zeros(M, N, dtype=dtype, device="cuda")
    hip.gemm(x, w, plain, aux_in=pre, **kw)(torch.cuda.current_stream().cuda_stream)
    out = torch.zeros(M, N, dtype=dtype, device="cuda")
    launch = hip.gemm(x, w, out, aux_in=pre, **kw)
    cs = hip.gemm_attach_colsum(launch, lambda shape, dt: torch.full(shape, float("nan"), dtype=dt, device="cuda"))
    assert cs is not None and launch.variant.endswith(", 5>")
    ws, off, nb, stride = cs
    assert (off, nb, stride) == (0, (M + bm - 1) // bm, N) and tuple(ws.shape) == (nb, N)
    launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(out, plain)
    got = ws.double().sum(0).cpu()
    want = out.double().sum(0).cpu()
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-4)
    # any other kernel path refuses the request loudly
    other = hip.gemm(x, w, torch.zeros(M, N, dtype=dtype, device="cuda"), M=M, N=N, K=K, lda=K, ldb=K, ldc=N, variant=variant)
    assert hip.gemm_attach_colsum(other, lambda shape, dt: torch.zeros(shape, dtype=dt, device="cuda")) is None
    other.desc.colsum_ws = ws.data_ptr()
    with pytest.raises(RuntimeError, match="colsum_ws"):
        other(torch.cuda.current_stream().cuda_stream)


def test_gemm_full_size_vit_l(hip, oracle):
    # qkv projection of ViT-L/16 at micro-batch 16: [3152 x 1024] . [1024 x 3072]
    M, N, K = 3152, 3072, 1024
    x, w = rnd((M, K), F16, 1), rnd((N, K), F16, 2, 0.03)
    r = both(hip, oracle, "gemm", dict(a=x, b=w, c=torch.zeros(M, N, dtype=F16)), ["c"], M=M, N=N, K=K, lda=K,
             ldb=K, ldc=N)
    close(r["c"], *TOL[F16])


def test_gemm_rejects_bad_arguments(hip):
    a = torch.zeros(8, 12, dtype=F16, device="cuda")
    with pytest.raises(RuntimeError, match="multiples of 8"):
        hip.run("gemm", a, a, torch.zeros(8, 8, device="cuda"), M=8, N=8, K=12, lda=12, ldb=12, ldc=8)
    with pytest.raises(RuntimeError, match="lda"):
        hip.run("gemm", a, a, torch.zeros(8, 8, device="cuda"), M=8, N=8, K=16, lda=8, ldb=16, ldc=8)


@pytest.mark.parametrize("xdt,ydt", [(F32, F16), (F32, BF16), (F32, F32), (F16, F16), (BF16, BF16)])
@pytest.mark.parametrize("rows,d", [(37, 1024), (5, 1408), (21, 1280), (9, 100), (3, 2048)])
def test_layernorm_rmsnorm(hip, oracle, xdt, ydt, rows, d):
    x = rnd((rows, d), xdt, 1) + 0.5
    gamma, beta = rnd((d,), F32, 2) + 1, rnd((d,), F32, 3)
    rt, at = TOL[ydt]
    t = dict(x=x, gamma=gamma, beta=beta, y=torch.zeros(rows, d, dtype=ydt), mean=torch.zeros(rows),
             rstd=torch.zeros(rows))
    r = both(hip, oracle, "layernorm_fwd", t, ["y", "mean", "rstd"], rows=rows, d=d, eps=1e-5)
    close(r["y"], rt, at)
    close(r["mean"], 1e-5, 1e-5)
    close(r["rstd"], 1e-5, 1e-5)
    mean, rstd = r["mean"][1], r["rstd"][1]
    dy = rnd((rows, d), ydt, 4)
    add = rnd((rows, d), xdt, 5)
    ws = torch.zeros(2 * 512 * d)
    t = dict(dy=dy, x=x, gamma=gamma, mean=mean, rstd=rstd, dx_add=add, dx=torch.zeros(rows, d, dtype=xdt),
             dgamma=rnd((d,), F32, 6), dbeta=rnd((d,), F32, 7), ws=ws)
    r = both(hip, oracle, "layernorm_bwd", t, ["dx", "dgamma", "dbeta"], rows=rows, d=d)
    close(r["dx"], *TOL[xdt])
    close(r["dgamma"], 1e-4, 1e-4 * rows ** 0.5)
    close(r["dbeta"], 1e-4, 1e-4 * rows ** 0.5)
    # RMSNorm
    t = dict(x=x, gamma=gamma, y=torch.zeros(rows, d, dtype=ydt), rstd=torch.zeros(rows))
    r = both(hip, oracle, "rmsnorm_fwd", t, ["y", "rstd"], rows=rows, d=d, eps=1e-6)
    close(r["y"], rt, at)
    close(r["rstd"], 1e-5, 1e-5)
    t = dict(dy=dy, x=x, gamma=gamma, rstd=r["rstd"][1], dx_add=None, dx=torch.zeros(rows, d, dtype=xdt),
             dgamma=rnd((d,), F32, 6), ws=ws)
    r = both(hip, oracle, "rmsnorm_bwd", t, ["dx", "dgamma"], rows=rows, d=d)
    close(r["dx"], *TOL[xdt])
    close(r["dgamma"], 1e-4, 1e-4 * rows ** 0.5)


def test_layernorm_many_rows_param_grads(hip, oracle):
    rows, d = 3152, 1024  # ViT-L residual stream at micro-batch 16: more rows than reduction workgroups
    x, dy = rnd((rows, d), F32, 1), rnd((rows, d), F16, 2)
    gamma = rnd((d,), F32, 3) + 1
    mean, rstd = x.mean(1), 1 / torch.sqrt(x.var(1, unbiased=False) + 1e-5)
    t = dict(dy=dy, x=x, gamma=gamma, mean=mean, rstd=rstd, dx_add=None, dx=torch.zeros(rows, d),
             dgamma=torch.zeros(d), dbeta=torch.zeros(d), ws=torch.zeros(2 * 512 * d))
    r = both(hip, oracle, "layernorm_bwd", t, ["dx", "dgamma", "dbeta"], rows=rows, d=d)
    close(r["dx"], 1e-4, 1e-4)
    close(r["dgamma"], 1e-4, 2e-2)
    close(r["dbeta"], 1e-4, 2e-2)


@pytest.mark.parametrize("lpdt", [F16, BF16])
@pytest.mark.parametrize("rows,d,rms,want_cs", [(3152, 1024, False, True), (37, 2048, True, True), (9, 100, False, False),
                                                (300, 4096, False, False), (5, 1408, True, True)])
def test_norm_backward_with_16bit_copy_and_column_sums(hip, oracle, lpdt, rows, d, rms, want_cs):
    """pf_norm_bwd_fused: dx as pf_layernorm_bwd / pf_rmsnorm_bwd give it (bit-exact), its 16-bit copy
    (bit-exact rounding of dx), and partial rows that reduce to dgamma, dbeta and the copy's column sums."""
    x, dy, add = rnd((rows, d), F32, 1) + 0.5, rnd((rows, d), lpdt, 2), rnd((rows, d), F32, 3)
    gamma = rnd((d,), F32, 4) + 1
    mean = None if rms else x.mean(1)
    rstd = 1 / torch.sqrt((x * x).mean(1) + 1e-6) if rms else 1 / torch.sqrt(x.var(1, unbiased=False) + 1e-5)
    nb = hip.norm_bwd_partials(rows)
    stride = (3 if want_cs else 2) * d
    dev = lambda t: None if t is None else t.cuda()
    dx, lp, ws = torch.zeros(rows, d).cuda(), torch.zeros(rows, d, dtype=lpdt).cuda(), torch.zeros(nb * stride).cuda()
    hip.run("norm_bwd_fused", dev(dy), dev(x), dev(gamma), dev(mean), dev(rstd), dev(add), dx, lp, ws, rows, d, True,
            want_cs)
    dx0, dg0, db0 = torch.zeros(rows, d).cuda(), torch.zeros(d).cuda(), torch.zeros(d).cuda()
    ws0 = torch.zeros(hip.colreduce_workspace(rows, d)).cuda()
    if rms:
        hip.run("rmsnorm_bwd", dev(dy), dev(x), dev(gamma), dev(rstd), dev(add), dx0, dg0, ws0, rows, d)
    else:
        hip.run("layernorm_bwd", dev(dy), dev(x), dev(gamma), dev(mean), dev(rstd), dev(add), dx0, dg0, db0, ws0, rows, d)
    torch.cuda.synchronize()
    assert torch.equal(dx, dx0)
    assert torch.equal(lp, dx0.to(lpdt))
    part = ws.view(nb, stride).cpu()
    torch.testing.assert_close(part[:, :d].sum(0), dg0.cpu(), rtol=1e-5, atol=1e-5 * rows ** 0.5)
    if not rms:
        torch.testing.assert_close(part[:, d:2 * d].sum(0), db0.cpu(), rtol=1e-5, atol=1e-5 * rows ** 0.5)
    if want_cs:
        torch.testing.assert_close(part[:, 2 * d:].sum(0), lp.float().sum(0).cpu(), rtol=1e-5, atol=1e-5 * rows ** 0.5)
    # and against the oracle (dx within the fp32 tolerance of the other norm tests)
    odx, olp, ows = torch.zeros(rows, d), torch.zeros(rows, d, dtype=lpdt), torch.zeros(3 * d)
    oracle.run("norm_bwd_fused", dy, x, gamma, mean, rstd, add, odx, olp, ows, rows, d, True, want_cs)
    close((dx.cpu(), odx), *TOL[F32])
    close((lp.cpu(), olp), *TOL[lpdt])


@pytest.mark.parametrize("dtype", [F16, BF16, F32])
def test_colsum(hip, oracle, dtype):
    for rows, cols, ld in [(3152, 1024, 1024), (77, 1000, 1000), (5, 13, 16), (4096, 96, 104)]:
        x = rnd((rows, ld), dtype, 1)
        t = dict(x=x, acc=rnd((cols,), F32, 2), ws=torch.zeros(2 * 512 * cols))
        r = both(hip, oracle, "colsum_accumulate", t, ["acc"], rows=rows, cols=cols, ld=ld)
        close(r["acc"], 1e-4, 1e-4 * rows ** 0.5 + 1e-3)


@pytest.mark.parametrize("pdt", [F16, BF16, F32])
@pytest.mark.parametrize("causal", [0, 1])
def test_softmax(hip, oracle, pdt, causal):
    for B, T, Tk in [(6, 197, 197), (2, 128, 128), (3, 64, 77)]:
        if causal and T != Tk:
            continue
        rows, ldp = B * T, (Tk + 7) // 8 * 8
        s = rnd((rows, Tk), F32, 1, 3.0)
        t = dict(s=s, p=torch.full((rows, ldp), 7.0, dtype=pdt))
        r = both(hip, oracle, "softmax_fwd", t, ["p"], ld_s=Tk, ld_p=ldp, rows=rows, cols=Tk, q_len=T, causal=causal)
        close(r["p"], *TOL[pdt])
        p = r["p"][1]
        dp = rnd((rows, Tk), F32, 2)
        t = dict(dp=dp, p=p, ds=torch.full((rows, ldp), 7.0, dtype=pdt))
        r = both(hip, oracle, "softmax_bwd", t, ["ds"], ld_dp=Tk, ld_p=ldp, ld_ds=ldp, rows=rows, cols=Tk, scale=0.125)
        close(r["ds"], *TOL[pdt])


@pytest.mark.parametrize("ldt", [F16, BF16, F32])
def test_cross_entropy(hip, oracle, ldt):
    for rows, classes in [(16, 1000), (37, 32000), (4, 7)]:
        logits = rnd((rows, classes), ldt, 1, 2.0)
        g = torch.Generator().manual_seed(5)
        targets = torch.randint(0, classes, (rows,), generator=g)
        targets[rows // 2] = -100
        t = dict(logits=logits, targets=targets, row_loss=torch.zeros(rows), row_lse=torch.zeros(rows),
                 loss=torch.zeros(2))
        r = both(hip, oracle, "cross_entropy_fwd", t, ["loss", "row_lse", "row_loss"], rows=rows, classes=classes,
                 ignore_index=-100)
        close(r["loss"], 1e-5, 1e-5)
        close(r["row_lse"], 1e-5, 1e-5)
        ref = torch.nn.functional.cross_entropy(logits.float(), targets, ignore_index=-100)
        torch.testing.assert_close(r["loss"][0][0], ref, rtol=1e-5, atol=1e-5)
        t = dict(logits=logits, targets=targets, row_lse=r["row_lse"][1], dloss=torch.tensor([1.7]),
                 loss=r["loss"][1], dlogits=torch.zeros(rows, classes, dtype=ldt))
        r = both(hip, oracle, "cross_entropy_bwd", t, ["dlogits"], rows=rows, classes=classes, ignore_index=-100)
        close(r["dlogits"], TOL[ldt][0], 1e-5 if ldt == F32 else 1e-3)


@pytest.mark.parametrize("dtype", [F16, BF16, F32])
def test_mse_sum(hip, oracle, dtype):
    n = 4 * 4 * 32 * 32 + 3
    a, b = rnd((n,), dtype, 1), rnd((n,), dtype, 2)
    t = dict(a=a, b=b, partial=torch.zeros(1024), loss=torch.zeros(1))
    r = both(hip, oracle, "mse_fwd", t, ["loss"], n=n)
    close(r["loss"], 1e-5, 1e-6)
    t = dict(a=a, b=b, dloss=torch.tensor([0.5]), da=torch.zeros(n, dtype=dtype))
    r = both(hip, oracle, "mse_bwd", t, ["da"], n=n)
    close(r["da"], TOL[dtype][0], 1e-6)
    t = dict(x=a, partial=torch.zeros(1024), loss=torch.zeros(1))
    r = both(hip, oracle, "sum_fwd", t, ["loss"], n=n)
    close(r["loss"], 1e-4, 1e-2)


@pytest.mark.parametrize("dtype", [F16, BF16, F32])
@pytest.mark.parametrize("act", [1, 2, 3, 4])
def test_activations_and_glu(hip, oracle, dtype, act):
    n = 8 * 1000 + 5
    x, dy = rnd((n,), dtype, 1, 2.0), rnd((n,), dtype, 2)
    rt, at = TOL[dtype]
    r = both(hip, oracle, "act_fwd", dict(x=x, y=torch.zeros(n, dtype=dtype)), ["y"], act=act, n=n)
    close(r["y"], rt, at)
    r = both(hip, oracle, "act_bwd", dict(dy=dy, x=x, dx=torch.zeros(n, dtype=dtype)), ["dx"], act=act, n=n)
    close(r["dx"], rt, at)
    rows, cols, ld = 33, 264, 2 * 264
    gu = rnd((rows, ld), dtype, 3)
    res = {}
    for name, tab, dev in (("hip", hip, "cuda"), ("oracle", oracle, "cpu")):
        t = gu.to(dev)
        y = torch.zeros(rows, cols, dtype=dtype, device=dev)
        tab.run("glu_fwd", t, ld, t[:, cols:], ld, y, cols, act=act, rows=rows, cols=cols)
        d = torch.zeros(rows, ld, dtype=dtype, device=dev)
        dyy = rnd((rows, cols), dtype, 4).to(dev)
        tab.run("glu_bwd", dyy, cols, t, ld, t[:, cols:], ld, d, ld, d[:, cols:], ld, act=act, rows=rows, cols=cols)
        res[name] = (y.cpu(), d.cpu())
    close((res["hip"][0], res["oracle"][0]), rt, at)
    close((res["hip"][1], res["oracle"][1]), rt, at * 2)


@pytest.mark.parametrize("dtype", [F16, BF16, F32])
def test_streaming_kernels(hip, oracle, dtype):
    n = 3152 * 1024 + 7
    a, b = rnd((n,), dtype, 1), rnd((n,), F32, 2)
    rt, at = TOL[dtype]
    r = both(hip, oracle, "axpby", dict(a=a, b=b, out=torch.zeros(n, dtype=F32)), ["out"], alpha=1.0, beta=1.0, n=n)
    close(r["out"], 1e-6, 1e-6)
    r = both(hip, oracle, "axpby", dict(a=b, b=None, out=torch.zeros(n, dtype=dtype)), ["out"], alpha=0.5, beta=0.0,
             n=n)
    close(r["out"], rt, at)
    r = both(hip, oracle, "cast", dict(src=b, dst=torch.zeros(n, dtype=dtype)), ["dst"], n=n)
    assert torch.equal(r["dst"][0], r["dst"][1]), "cast must round exactly like torch"
    r = both(hip, oracle, "fill", dict(dst=torch.ones(n, dtype=dtype)), ["dst"], value=0.0, n=n)
    assert torch.equal(r["dst"][0], r["dst"][1])
    # fp32 gradient accumulation: identical single additions -> bit-exact
    r = both(hip, oracle, "grad_accumulate", dict(acc=b.clone(), g=a), ["acc"], n=n)
    assert torch.equal(r["acc"][0], r["acc"][1]), "grad accumulate must be bit-exact"
    m = 1024 * 77
    x, bias = rnd((m,), dtype, 3), rnd((1024,), F32, 4)
    r = both(hip, oracle, "bias_add", dict(x=x, bias=bias, y=torch.zeros(m, dtype=F32)), ["y"], n=m, bias_len=1024)
    close(r["y"], 1e-6, 1e-6)


@pytest.mark.parametrize("dtype", [F16, F32])
def test_copy_strided_and_rope(hip, oracle, dtype):
    # patch extraction [B, C, Hp, p, Wp, p] -> [B, Hp, Wp, C, p, p]
    B, C, Hp, p = 2, 3, 4, 16
    img = rnd((B, C, Hp * p, Hp * p), F32, 1)
    sizes = (B, Hp, Hp, C, p, p)
    s = img.stride()
    ss = (s[0], s[2] * p, s[3] * p, s[1], s[2], s[3])
    out = torch.zeros(B * Hp * Hp, C * p * p, dtype=dtype)
    ds = (Hp * Hp * C * p * p, Hp * C * p * p, C * p * p, p * p, p, 1)
    r = both(hip, oracle, "copy_strided", dict(src=img, dst=out), ["dst"], src_strides=ss, dst_strides=ds, sizes=sizes)
    assert torch.equal(r["dst"][0], r["dst"][1])
    ref = img.reshape(B, C, Hp, p, Hp, p).permute(0, 2, 4, 1, 3, 5).reshape(B * Hp * Hp, -1).to(dtype)
    assert torch.equal(r["dst"][0], ref)
    # scalar path + accumulate
    src = rnd((5, 7, 3), dtype, 2)
    dst = rnd((3, 5, 7), dtype, 3)
    r = both(hip, oracle, "copy_strided", dict(src=src, dst=dst), ["dst"], src_strides=(21, 3, 1),
             dst_strides=(7, 1, 35), sizes=(5, 7, 3), accumulate=1)
    close(r["dst"], *TOL[dtype])
    # batched transposes (tiled through LDS): NCHW -> NHWC and back, ragged extents, plain and accumulating
    for (Bt, Ct, HW) in ((2, 70, 100), (3, 16, 33), (1, 128, 64)):
        nchw = rnd((Bt, Ct, HW), dtype, 6)
        nhwc = torch.zeros(Bt, HW, Ct, dtype=dtype)
        r = both(hip, oracle, "copy_strided", dict(src=nchw, dst=nhwc), ["dst"], src_strides=(Ct * HW, 1, HW),
                 dst_strides=(HW * Ct, Ct, 1), sizes=(Bt, HW, Ct))
        assert torch.equal(r["dst"][0], r["dst"][1]) and torch.equal(r["dst"][0], nchw.permute(0, 2, 1).contiguous())
        acc0 = rnd((Bt, Ct, HW), dtype, 7)
        r = both(hip, oracle, "copy_strided", dict(src=r["dst"][0], dst=acc0), ["dst"], src_strides=(HW * Ct, 1, Ct),
                 dst_strides=(Ct * HW, HW, 1), sizes=(Bt, Ct, HW), accumulate=1)
        close(r["dst"], *TOL[dtype])
        close((r["dst"][0], (acc0.float() + nchw.float()).to(dtype)), *TOL[dtype])
    # four dimensions with the source-contiguous one in the middle: [B, H, T, D] -> [B, D, H, T]
    x4 = rnd((2, 3, 40, 24), dtype, 8)
    y4 = torch.zeros(2, 24, 3, 40, dtype=dtype)
    r = both(hip, oracle, "copy_strided", dict(src=x4, dst=y4), ["dst"], src_strides=(3 * 40 * 24, 1, 40 * 24, 24),
             dst_strides=(24 * 3 * 40, 3 * 40, 40, 1), sizes=(2, 24, 3, 40))
    assert torch.equal(r["dst"][0], x4.permute(0, 3, 1, 2).contiguous())
    # convolution weight [out, in, 9] -> [out, 9, in] (a short source-contiguous dimension) and its gradient back
    wt = rnd((20, 70, 9), F32, 9)
    w9 = torch.zeros(20, 9, 70, dtype=dtype)
    r = both(hip, oracle, "copy_strided", dict(src=wt, dst=w9), ["dst"], src_strides=(630, 1, 9), dst_strides=(630, 70, 1),
             sizes=(20, 9, 70))
    assert torch.equal(r["dst"][0], r["dst"][1]) and torch.equal(r["dst"][0], wt.permute(0, 2, 1).to(dtype))
    g9, gacc = rnd((20, 9, 70), F32, 10), rnd((20, 70, 9), F32, 11)
    r = both(hip, oracle, "copy_strided", dict(src=g9, dst=gacc), ["dst"], src_strides=(630, 70, 1), dst_strides=(630, 1, 9),
             sizes=(20, 9, 70), accumulate=1)
    close(r["dst"], 1e-6, 1e-6)
    close((r["dst"][0], gacc + g9.permute(0, 2, 1)), 1e-6, 1e-6)
    # rotary embedding on q inside a packed [B, T, 3, H, D] tensor, forward then inverse = identity
    Bq, T, H, D = 2, 33, 4, 64
    qkv = rnd((Bq, T, 3 * H * D), dtype, 4)
    inv_freq = 1.0 / (10000 ** (torch.arange(0, D, 2).float() / D))
    ang = torch.arange(T).float()[:, None] * inv_freq[None, :]
    cos_t, sin_t = ang.cos().contiguous(), ang.sin().contiguous()
    xs = (T * 3 * H * D, 3 * H * D, D)
    y = torch.zeros(Bq, T, H, D, dtype=dtype)
    r = both(hip, oracle, "rope", dict(x=qkv, y=y, cos_t=cos_t, sin_t=sin_t), ["y"], B=Bq, T=T, H=H, D=D, xs=xs,
             ys=(T * H * D, H * D, D), inverse=0)
    close(r["y"], *TOL[dtype])
    back = both(hip, oracle, "rope", dict(x=r["y"][1], y=torch.zeros_like(y), cos_t=cos_t, sin_t=sin_t), ["y"], B=Bq,
                T=T, H=H, D=D, xs=(T * H * D, H * D, D), ys=(T * H * D, H * D, D), inverse=1)
    close((back["y"][0], qkv.view(Bq, T, 3, H, D)[:, :, 0].contiguous()), TOL[dtype][0] * 3, TOL[dtype][1] * 3)
    # a head dim whose half is no multiple of 8 takes the element-wise kernel
    D2 = 24
    x2 = rnd((Bq, T, H, D2), dtype, 5)
    ang2 = torch.arange(T).float()[:, None] * (1.0 / (10000 ** (torch.arange(0, D2, 2).float() / D2)))[None, :]
    r = both(hip, oracle, "rope", dict(x=x2, y=torch.zeros_like(x2), cos_t=ang2.cos().contiguous(),
                                       sin_t=ang2.sin().contiguous()), ["y"], B=Bq, T=T, H=H, D=D2,
             xs=(T * H * D2, H * D2, D2), ys=(T * H * D2, H * D2, D2), inverse=0)
    close(r["y"], *TOL[dtype])


def test_split_merge_bit_exact(hip, oracle):
    g = torch.Generator().manual_seed(3)
    for N, n, shape_tail, dtype in [(64, 4, (3, 8, 8), F32), (10, 4, (5,), torch.int64), (7, 3, (3,), torch.uint8),
                                    (5, 8, (2, 2), F16), (16, 4, (), torch.int64)]:
        if dtype in (F32, F16):
            full = torch.randn((N,) + shape_tail, generator=g).to(dtype)
        else:
            full = torch.randint(0, 200, (N,) + shape_tail, generator=g).to(dtype)
        row_bytes = full[0].numel() * full.element_size() if N else 0
        chunks = torch.tensor_split(full, n, 0)
        merged = {"hip": torch.zeros_like(full).cuda(), "oracle": torch.zeros_like(full)}
        start = 0
        for ch in chunks:
            rows = ch.shape[0]
            for name, tab, dev in (("hip", hip, "cuda"), ("oracle", oracle, "cpu")):
                slab = torch.zeros_like(ch).to(dev)
                tab.run("split_gather", full.to(dev), slab, row_bytes=row_bytes, row_start=start, n_rows=rows)
                assert torch.equal(slab.cpu(), ch), (name, N, n, start)
                tab.run("merge_scatter", slab, merged[name], row_bytes=row_bytes, row_start=start, n_rows=rows)
            start += rows
        assert start == N
        torch.cuda.synchronize()
        assert torch.equal(merged["hip"].cpu(), full) and torch.equal(merged["oracle"], full)
    # indexed gather / scatter
    full = torch.randn(33, 24, generator=g)
    idx = torch.randperm(33, generator=g)[:9]
    for name, tab, dev in (("hip", hip, "cuda"), ("oracle", oracle, "cpu")):
        out = torch.zeros(9, 24, device=dev)
        tab.run("split_gather", full.to(dev), out, row_bytes=96, row_start=0, n_rows=9, index=idx.to(dev))
        assert torch.equal(out.cpu(), full[idx]), name
        back = torch.zeros(33, 24, device=dev)
        tab.run("merge_scatter", out, back, row_bytes=96, row_start=0, n_rows=9, index=idx.to(dev))
        ref = torch.zeros(33, 24)
        ref[idx] = full[idx]
        assert torch.equal(back.cpu(), ref), name


@pytest.mark.parametrize("dtype", [F16, BF16, F32])
def test_embedding(hip, oracle, dtype):
    vocab, dim, n = 1000, 264, 300
    table = rnd((vocab, dim), F32, 1)
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 50, (n,), generator=g)  # heavy collisions
    r = both(hip, oracle, "embedding_fwd", dict(table=table, ids=ids, out=torch.zeros(n, dim, dtype=dtype)), ["out"],
             n_ids=n, dim=dim, vocab=vocab)
    assert torch.equal(r["out"][0], r["out"][1])
    dout = rnd((n, dim), dtype, 3)
    r = both(hip, oracle, "embedding_bwd", dict(dout=dout, ids=ids, dtable=rnd((vocab, dim), F32, 4)), ["dtable"],
             n_ids=n, dim=dim, vocab=vocab)
    close(r["dtable"], 1e-5, 1e-5)
    # padding row keeps its old contents; ids spread over a vocabulary that is no multiple of the
    # rows one wavefront owns, with the last row hit; same summation order as index_add: exact
    vocab2 = 1003
    ids2 = torch.randint(0, vocab2, (n,), generator=g)
    ids2[5], ids2[17], ids2[100] = vocab2 - 1, 7, 7
    r = both(hip, oracle, "embedding_bwd", dict(dout=dout, ids=ids2, dtable=rnd((vocab2, dim), F32, 5)), ["dtable"],
             n_ids=n, dim=dim, vocab=vocab2, padding_idx=7)
    assert torch.equal(*r["dtable"])
    assert torch.equal(r["dtable"][0][7], rnd((vocab2, dim), F32, 5)[7])


@pytest.mark.parametrize("dtype", [F16, BF16, F32])
def test_transpose_cast(hip, oracle, dtype):
    for rows, cols in [(1024, 4096), (1000, 1024), (37, 5), (64, 64)]:
        src = rnd((rows, cols), F32, 1)
        r = both(hip, oracle, "transpose_cast", dict(src=src, dst=torch.zeros(cols, rows, dtype=dtype)), ["dst"],
                 ld_src=cols, ld_dst=rows, rows=rows, cols=cols)
        assert torch.equal(r["dst"][0], r["dst"][1])
        assert torch.equal(r["dst"][0], src.t().to(dtype))


def test_deferred_reductions_match_immediate(hip):
    """Partials written with defer=1 and finished by one batched launch give bit-identical
    accumulators to the immediate two-kernel path (same partials, same summation order)."""
    rows, d = 3152, 1024
    x = rnd((rows, d), F32, 1).cuda()
    dy = rnd((rows, d), F16, 2).cuda()
    gamma = (rnd((d,), F32, 3) + 1).cuda()
    mean, rstd = x.mean(1), 1 / torch.sqrt(x.var(1, unbiased=False) + 1e-5)
    need = hip.colreduce_workspace(rows, d)
    outs = {}
    for defer in (0, 1):
        dx = torch.zeros(rows, d, device="cuda")
        dg, db, bias = rnd((d,), F32, 4).cuda(), rnd((d,), F32, 5).cuda(), rnd((d,), F32, 6).cuda()
        ws1, ws2 = torch.zeros(need, device="cuda"), torch.zeros(need, device="cuda")
        if defer:
            hip.run("layernorm_bwd", dy, x, gamma, mean, rstd, None, dx, None, None, ws1, rows, d, defer=1)
            hip.run("colsum_accumulate", dy, rows, d, d, None, ws2, defer=1)
            nb = hip.norm_bwd_partials(rows)
            hip.run("colreduce_finalize_batch", [(ws1, 0, nb, 2 * d, d, dg), (ws1, d, nb, 2 * d, d, db),
                                                 (ws2, 0, hip.colsum_partials(rows), d, d, bias)])
        else:
            hip.run("layernorm_bwd", dy, x, gamma, mean, rstd, None, dx, dg, db, ws1, rows, d)
            hip.run("colsum_accumulate", dy, rows, d, d, bias, ws2)
        torch.cuda.synchronize()
        outs[defer] = (dx.cpu(), dg.cpu(), db.cpu(), bias.cpu())
    for a, b in zip(outs[0], outs[1]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("case", [
    dict(B=2, H=3, Tq=197, Tk=197, hd=64, causal=0, packed=True),    # ViT block
    dict(B=1, H=2, Tq=257, Tk=257, hd=88, causal=0, packed=True),    # ViT-g head dim 88
    dict(B=2, H=4, Tq=128, Tk=128, hd=64, causal=1, packed=False),   # decoder
    dict(B=1, H=2, Tq=300, Tk=300, hd=64, causal=1, packed=False),   # ragged causal over several tiles
    dict(B=2, H=2, Tq=64, Tk=77, hd=64, causal=0, packed=False),     # cross attention (77 context tokens)
    dict(B=1, H=1, Tq=5, Tk=3, hd=8, causal=0, packed=False),        # tiny
    dict(B=2, H=2, Tq=100, Tk=130, hd=64, causal=1, packed=False),   # short causal, more keys than queries
    dict(B=1, H=3, Tq=200, Tk=40, hd=88, causal=0, packed=False),    # short, several query blocks, few keys
    dict(B=1, H=2, Tq=320, Tk=290, hd=64, causal=0, packed=False),   # beyond the whole-head-in-LDS kernels
    dict(B=2, H=2, Tq=280, Tk=280, hd=64, causal=1, packed=False),   # ninth tile: second pass of the first wavefront
    dict(B=2, H=2, Tq=600, Tk=77, hd=64, causal=0, packed=False),    # cross attention from many queries: split-query dK/dV
    dict(B=2, H=3, Tq=200, Tk=160, hd=64, causal=0, packed=False),   # one-workgroup backward, more queries than keys
    dict(B=1, H=2, Tq=150, Tk=250, hd=64, causal=1, packed=False),   # one-workgroup backward, causal with more keys
    dict(B=1, H=2, Tq=256, Tk=256, hd=40, causal=1, packed=False),   # one-workgroup backward at its largest head
    dict(B=1, H=3, Tq=200, Tk=40, hd=64, causal=0, packed=False),    # one-workgroup backward, two key tiles only
    dict(B=1, H=2, Tq=33, Tk=250, hd=16, causal=0, packed=False),    # one-workgroup backward, two query tiles only
    dict(B=1, H=2, Tq=330, Tk=40, hd=88, causal=0, packed=False),    # the same at head dim 88, ragged query blocks
    dict(B=1, H=2, Tq=160, Tk=170, hd=96, causal=0, packed=False),   # head dim 96: six key tiles in one 4-wavefront workgroup
])
def test_fused_attention(hip, oracle, dtype, case):
    B, H, Tq, Tk, hd = case["B"], case["H"], case["Tq"], case["Tk"], case["hd"]
    C = H * hd
    if case["packed"]:
        qkv = rnd((B, Tq, 3, H, hd), dtype, 1, 0.7)
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    else:
        q = rnd((B, Tq, H, hd), dtype, 1, 0.7).permute(0, 2, 1, 3)
        k = rnd((B, Tk, H, hd), dtype, 2, 0.7).permute(0, 2, 1, 3)
        v = rnd((B, Tk, H, hd), dtype, 3, 0.7).permute(0, 2, 1, 3)
    d_o = rnd((B, Tq, H, hd), dtype, 4).permute(0, 2, 1, 3)
    scale = hd ** -0.5
    res = {}
    for name, tab, dev in (("hip", hip, "cuda"), ("oracle", oracle, "cpu")):
        if case["packed"]:
            base = qkv.to(dev)
            qd, kd, vd = (base[:, :, i].permute(0, 2, 1, 3) for i in range(3))
            dbase = torch.zeros_like(base)
            dq, dk, dv = (dbase[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        else:
            qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
            dq, dk, dv = torch.zeros_like(qd), torch.zeros_like(kd), torch.zeros_like(vd)
        o = torch.zeros(B, Tq, H, hd, dtype=dtype, device=dev).permute(0, 2, 1, 3)
        lse = torch.zeros(B, H, Tq, device=dev)
        delta = torch.zeros(B, H, Tq, device=dev)
        tab.run("attention_fwd", qd, kd, vd, o, lse, scale, case["causal"])
        tab.run("attention_bwd", qd, kd, vd, o, d_o.to(dev), lse, delta, dq, dk, dv, scale, case["causal"])
        if dev == "cuda":
            torch.cuda.synchronize()
        res[name] = [t.cpu().float() for t in (o, lse, dq, dk, dv)]
    rt, at = TOL[dtype]
    for i, nm in enumerate(["o", "lse", "dq", "dk", "dv"]):
        a, b = res["hip"][i], res["oracle"][i]
        tol = (1e-4, 1e-4) if nm == "lse" else (rt * 2, at * 2)
        torch.testing.assert_close(a, b, rtol=tol[0], atol=tol[1], msg=lambda m, nm=nm: nm + ": " + m)
    # the oracle itself against torch's attention and its autograd
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    mask = None
    if case["causal"]:
        mask = torch.ones(Tq, Tk, dtype=torch.bool).tril(Tk - Tq)
    ref = torch.nn.functional.scaled_dot_product_attention(qf, kf, vf, attn_mask=mask)
    ref.backward(d_o.float())
    torch.testing.assert_close(res["oracle"][0], ref.detach(), rtol=3e-2, atol=3e-2)
    for g, r in ((res["oracle"][2], qf.grad), (res["oracle"][3], kf.grad), (res["oracle"][4], vf.grad)):
        torch.testing.assert_close(g, r, rtol=5e-2, atol=5e-2)


def test_fused_attention_long_causal_sequences(hip):
    """The decoder configuration's own attention shape: 2 x 32 heads, 2048 causal tokens, head dim 64
    (16 query blocks per head, whose work differs by a factor of 16; the kernels start the heaviest
    blocks of every head first).  Checked against torch's attention and its autograd in fp32 on the
    same bf16 inputs; also without the mask, which takes the plain block order."""
    B, H, T, hd = 2, 32, 2048, 64
    qkv = rnd((B, T, 3, H, hd), BF16, 11, 0.7)
    d_o = rnd((B, T, H, hd), BF16, 12).permute(0, 2, 1, 3)
    for causal in (1, 0):
        base = qkv.cuda()
        qd, kd, vd = (base[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        dbase = torch.zeros_like(base)
        dq, dk, dv = (dbase[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        o = torch.zeros(B, T, H, hd, dtype=BF16, device="cuda").permute(0, 2, 1, 3)
        lse = torch.zeros(B, H, T, device="cuda")
        delta = torch.zeros(B, H, T, device="cuda")
        hip.run("attention_fwd", qd, kd, vd, o, lse, hd ** -0.5, causal)
        hip.run("attention_bwd", qd, kd, vd, o, d_o.cuda(), lse, delta, dq, dk, dv, hd ** -0.5, causal)
        torch.cuda.synchronize()
        qf, kf, vf = (qkv[:, :, i].permute(0, 2, 1, 3).float().requires_grad_() for i in range(3))
        ref = torch.nn.functional.scaled_dot_product_attention(qf, kf, vf, is_causal=bool(causal))
        ref.backward(d_o.float())
        torch.testing.assert_close(o.cpu().float(), ref.detach(), rtol=3e-2, atol=3e-2)
        for got, want, nm in ((dq, qf.grad, "dq"), (dk, kf.grad, "dk"), (dv, vf.grad, "dv")):
            rel = (got.cpu().float() - want).norm() / want.norm()
            assert rel <= 2e-2, (nm, causal, float(rel))
            torch.testing.assert_close(got.cpu().float(), want, rtol=5e-2, atol=5e-2, msg=lambda m, nm=nm: nm + ": " + m)


@pytest.mark.parametrize("xdt,ydt", [(F32, F32), (F16, F16), (F32, BF16)])
def test_groupnorm_and_channel_bias(hip, oracle, xdt, ydt):
    for B, HW, C, G in [(4, 1024, 1280, 32), (2, 64, 64, 8), (3, 49, 96, 32), (2, 100, 128, 2), (1, 33, 64, 4)]:
        x = rnd((B, HW, C), xdt, 1) * 2 + 0.3
        gamma, beta = rnd((C,), F32, 2) + 1, rnd((C,), F32, 3)
        t = dict(x=x, gamma=gamma, beta=beta, y=torch.zeros(B, HW, C, dtype=ydt), mean=torch.zeros(B * G),
                 rstd=torch.zeros(B * G))
        r = both(hip, oracle, "groupnorm_fwd", t, ["y", "mean", "rstd"], B=B, HW=HW, C=C, groups=G, eps=1e-5)
        close(r["y"], *TOL[ydt])
        close(r["mean"], 1e-5, 1e-5)
        close(r["rstd"], 1e-4, 1e-5)
        ref = torch.nn.functional.group_norm(x.float().permute(0, 2, 1), G, gamma, beta, 1e-5).permute(0, 2, 1)
        torch.testing.assert_close(r["y"][1].float(), ref.to(ydt).float(), rtol=TOL[ydt][0], atol=TOL[ydt][1])
        dy = rnd((B, HW, C), ydt, 4)
        need = hip.groupnorm_workspace(B, C, G)
        t = dict(dy=dy, x=x, gamma=gamma, mean=r["mean"][1], rstd=r["rstd"][1], dx=torch.zeros(B, HW, C, dtype=xdt),
                 dgamma=rnd((C,), F32, 5), dbeta=rnd((C,), F32, 6), ws=torch.zeros(need))
        r = both(hip, oracle, "groupnorm_bwd", t, ["dx", "dgamma", "dbeta"], B=B, HW=HW, C=C, groups=G)
        close(r["dx"], TOL[xdt][0] * 2, TOL[xdt][1] * 2)
        close(r["dgamma"], 1e-3, 1e-3 * (B * HW) ** 0.5)
        close(r["dbeta"], 1e-3, 1e-3 * (B * HW) ** 0.5)
    # per-sample vector added to every row of that sample
    B, HW, C = 3, 50, 64
    x, bias = rnd((B * HW, C), xdt, 7), rnd((B, C), xdt, 8)
    r = both(hip, oracle, "bias_add", dict(x=x, bias=bias, y=torch.zeros(B * HW, C, dtype=F32)), ["y"],
             n=B * HW * C, bias_len=C, rows_per_bias=HW)
    close(r["y"], 1e-6, 1e-6)
    torch.testing.assert_close(r["y"][1], (x.float().view(B, HW, C) + bias.float()[:, None, :]).view(B * HW, C))


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_transpose_16bit_register_path(hip, oracle, dtype):
    for rows, cols, lds, ldd in [(3152, 4096, 4096, 3152), (1000, 264, 272, 1000), (8, 8, 8, 8), (77, 64, 64, 80)]:
        src = rnd((rows, lds), dtype, 1)
        dst = torch.zeros(cols, ldd, dtype=dtype)
        r = both(hip, oracle, "transpose_cast", dict(src=src, dst=dst), ["dst"], ld_src=lds, ld_dst=ldd, rows=rows,
                 cols=cols)
        assert torch.equal(r["dst"][0][:, :rows], src[:, :cols].t())
        assert torch.equal(r["dst"][1][:, :rows], src[:, :cols].t())


def test_loss_scaler_kernels(hip, oracle):
    """Dynamic loss scaling kept on the device: scale_by_state, scaler_unscale (power-of-two scale:
    bit-exact, sets found_inf on inf/NaN anywhere in a large buffer) and scaler_update over a
    sequence with two overflows against the oracle (itself pinned to torch.amp.GradScaler)."""
    n = 256 * 1024 * 3 + 5
    state0 = torch.tensor([4096.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0])
    src = rnd((n,), F16, 1)
    r = both(hip, oracle, "scale_by_state", dict(src=src, state=state0.clone(), dst=torch.zeros(n, dtype=F32)),
             ["dst"], n=n)
    assert torch.equal(*r["dst"])
    g = rnd((n,), F32, 2, scale=4096.0)
    r = both(hip, oracle, "scaler_unscale", dict(grads=g.clone(), state=state0.clone()), ["grads", "state"], n=n)
    assert torch.equal(*r["grads"]) and torch.equal(*r["state"]) and float(r["state"][0][2]) == 0.0
    for pos, bad in ((0, float("inf")), (n - 1, float("nan")), (n // 2 + 3, float("-inf"))):
        gb = g.clone()
        gb[pos] = bad
        r = both(hip, oracle, "scaler_unscale", dict(grads=gb, state=state0.clone()), ["state"], n=n)
        assert torch.equal(*r["state"]) and float(r["state"][0][2]) == 1.0, pos
    dev, cpu = state0.clone().cuda(), state0.clone()
    for found in (0, 0, 1, 0, 0, 0, 1, 1, 0, 0):
        dev[2] = float(found)
        cpu[2] = float(found)
        hip.run("scaler_update", dev, 2.0, 0.5, 3)
        oracle.run("scaler_update", cpu, 2.0, 0.5, 3)
        torch.cuda.synchronize()
        assert torch.equal(dev.cpu(), cpu), (found, dev.cpu(), cpu)


def test_adam_step_scaled_skips_on_overflow_and_counts_steps_on_device(hip):
    """pf_adam_step_scaled reads found_inf and the completed-step count from the scaler state:
    with found_inf set nothing changes; otherwise it equals pf_adam_step at step = count + 1."""
    n = 100003
    mk = lambda: [rnd((n,), F32, 3).cuda(), rnd((n,), F32, 4).cuda(), torch.zeros(n, device="cuda"),
                  torch.zeros(n, device="cuda")]
    ref, got = mk(), mk()
    state = torch.tensor([1.0, 0.0, 0.0, 2.0, 0.0, 0.0, 0.0, 0.0], device="cuda")          # two steps completed -> step 3
    s = torch.cuda.current_stream().cuda_stream
    tr, _, _ = hip.adam_table([ref[0]], [ref[1]], [ref[2]], [ref[3]])
    tg, ni, mx = hip.adam_table([got[0]], [got[1]], [got[2]], [got[3]])
    hip.adam_step(tr, ni, mx, 1e-3, 0.9, 0.999, 1e-8, 0.01, 3, True, s)
    state[2] = 1.0
    before = [t.clone() for t in got]
    hip.adam_step_scaled(tg, ni, mx, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, state, s)
    torch.cuda.synchronize()
    for a, b in zip(got, before):
        assert torch.equal(a, b)
    state[2] = 0.0
    hip.adam_step_scaled(tg, ni, mx, 1e-3, 0.9, 0.999, 1e-8, 0.01, True, state, s)
    torch.cuda.synchronize()
    for a, b in zip(got, ref):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_shadow_batch_bit_exact(hip, dtype):
    """pf_shadow_batch: plain and transposed 16-bit shadows of several fp32 matrices in one launch,
    bit-identical to torch's cast (and to its transpose), for tile-ragged shapes and for items with
    only one of the two destinations."""
    shapes = [(1024, 4096), (200, 72), (64, 64), (4, 1000), (260, 4)]
    items, keep = [], []
    for i, (r, c) in enumerate(shapes):
        src = rnd((r, c), F32, 10 + i, 3.0).cuda()
        plain = None if i == 3 else torch.zeros(r, c, dtype=dtype, device="cuda")
        tr = None if i == 4 else torch.zeros(c, r, dtype=dtype, device="cuda")
        assert hip.shadow_batch_ok(src, plain, tr)
        items.append((src, plain, tr))
    hip.shadow_batch(items)(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for src, plain, tr in items:
        if plain is not None:
            assert torch.equal(plain, src.to(dtype))
        if tr is not None:
            assert torch.equal(tr, src.t().contiguous().to(dtype))
    assert not hip.shadow_batch_ok(torch.zeros(6, 8, device="cuda"), None, None)          # rows % 4
    assert not hip.shadow_batch_ok(torch.zeros(8, 8, device="cuda").t(), None, None)      # not contiguous


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_gemm_grouped_weight_gradients_bit_exact(hip, dtype):
    """pf_gemm_grouped: several weight-gradient products (dY^T X accumulated into fp32) in one launch
    give bit-identical results to the same products launched one by one (same kernel, same tiles);
    products of different instantiations in one call fall back to separate launches, in order."""
    torch.manual_seed(0)
    K = 1576   # token rows: not a multiple of the reduction tile
    shapes = [(1024, 1024), (1024, 3072), (256, 512), (384, 1024)]
    probs = []
    for i, (M, N) in enumerate(shapes):
        dy = rnd((K, M), dtype, 20 + i).cuda()
        x = rnd((K, N), dtype, 30 + i).cuda()
        c0 = rnd((M, N), F32, 40 + i).cuda()
        probs.append((dy, x, c0))
    singles, groups = [], []
    for dy, x, c0 in probs:
        M, N = dy.shape[1], x.shape[1]
        c1, c2 = c0.clone(), c0.clone()
        singles.append((hip.gemm(dy, x, c1, M=M, N=N, K=K, lda=M, ldb=N, ldc=N, a_trans=1, b_trans=1, beta=1), c1))
        groups.append((hip.gemm(dy, x, c2, M=M, N=N, K=K, lda=M, ldb=N, ldc=N, a_trans=1, b_trans=1, beta=1), c2))
    s = torch.cuda.current_stream().cuda_stream
    for l, _ in singles:
        l(s)
    by_variant = {}
    for l, c in groups:      # the 256x512 problem runs on the register-staged kernel: not groupable
        by_variant.setdefault(l.variant if hip.gemm_groupable(l) else "single %d" % len(by_variant), []).append(l)
    grouped = 0
    for v, ls in by_variant.items():
        if len(ls) >= 2:
            g = hip.gemm_group(ls)
            assert g.variant.startswith("gemm16x_group_kernel<") and g.flops == sum(l.flops for l in ls)
            g(s)
            grouped += 1
        else:
            ls[0](s)
    assert grouped >= 1
    torch.cuda.synchronize()
    for (_, c1), (_, c2), (dy, x, c0) in zip(singles, groups, probs):
        assert torch.equal(c1, c2)
        ref = c0.double() + dy.double().t() @ x.double()
        torch.testing.assert_close(c1.double(), ref, rtol=2e-3, atol=2e-2)
    with pytest.raises(RuntimeError):
        hip.gemm_group([groups[0][0]])


def test_weight_gradients_of_mixed_sizes_regroup_on_large_tiles(hip, monkeypatch):
    """An encoder's weight gradients in backward order (two 1024x4096 MLP weights that fill the device
    alone on 128x128 tiles, then the 1024x1024 projection and the 3072x1024 qkv weight that are held
    back to fill it together, then the next layer's MLP weight): 64 + 64 + (16 + 48) + 64 tiles of
    256x256, so the fifth product completes the set and the job holds ONE launch.  Token count 1576:
    the reduction ends inside a tile.  Values equal those of the launches it replaced, bit for bit."""
    from types import SimpleNamespace
    from pfeife_amd.executor.lowering import BwdCtx
    from pfeife_amd.hip import dtype_code
    K = 1576
    shapes = [(1024, 4096), (4096, 1024), (1024, 1024), (3072, 1024), (1024, 4096), (4096, 1024)]
    probs = [(rnd((K, M), F16, 80 + i).cuda(), rnd((K, N), F16, 90 + i).cuda(), rnd((M, N), F32, 100 + i).cuda())
             for i, (M, N) in enumerate(shapes)]

    def build():
        prog = SimpleNamespace(bwd=[])
        B = BwdCtx(SimpleNamespace(kernels=hip), prog)
        outs = []
        for dy, x, c0 in probs:
            c = c0.clone()
            M, N = c.shape
            B.emit_dw(hip.gemm(dy, x, c, M=M, N=N, K=K, lda=M, ldb=N, ldc=N, a_trans=1, b_trans=1, beta=1), c)
            outs.append(c)
        B.close_dw()
        ranges = [("all", 0, len(prog.bwd))]
        B.compact(ranges)
        assert ranges == [("all", 0, len(prog.bwd))] and None not in prog.bwd
        return prog.bwd, outs

    new, c_new = build()
    assert [l.variant.split("<")[0] for l in new] == ["gemm16x_group_kernel", "gemm16x_kernel"]
    assert new[0].variant.startswith("gemm16x_group_kernel<%d, 256, 256" % dtype_code(F16))
    monkeypatch.setenv("PFEIFE_DW_RETILE", "0")
    old, c_old = build()
    assert len(old) == 5       # projection and qkv share a launch on 128x128 tiles
    s = torch.cuda.current_stream().cuda_stream
    for l in new + old:
        l(s)
    torch.cuda.synchronize()
    for a, b in zip(c_new, c_old):
        assert torch.equal(a, b)
    dy, x, c0 = probs[3]
    torch.testing.assert_close(c_new[3].double(), c0.double() + dy.double().t() @ x.double(), rtol=2e-3, atol=2e-2)


def test_weight_gradients_that_fill_the_device_together_share_a_launch_on_large_tiles(hip, monkeypatch):
    """Four 2048x2048 weight-gradient products (a decoder layer's attention projections) each fill the
    device on 128x128 tiles; the backward builder replaces them by ONE launch on 256x256 tiles once the
    fourth arrives (at the end of a job, with what has arrived if that covers half the device), and the values are those of the
    four separate launches, bit for bit.  PFEIFE_DW_RETILE=0 keeps the separate launches."""
    from types import SimpleNamespace
    from pfeife_amd.executor.lowering import BwdCtx
    from pfeife_amd.hip import dtype_code
    K, M, N = 4096, 2048, 2048
    probs = [(rnd((K, M), BF16, 50 + i).cuda(), rnd((K, N), BF16, 60 + i).cuda(), rnd((M, N), F32, 70 + i).cuda())
             for i in range(4)]

    def build(n):
        prog = SimpleNamespace(bwd=[])
        B = BwdCtx(SimpleNamespace(kernels=hip), prog)
        outs = []
        for dy, x, c0 in probs[:n]:
            c = c0.clone()
            B.emit_dw(hip.gemm(dy, x, c, M=M, N=N, K=K, lda=M, ldb=N, ldc=N, a_trans=1, b_trans=1, beta=1), c)
            outs.append(c)
        B.close_dw()
        ranges = [("all", 0, len(prog.bwd))]
        B.compact(ranges)
        assert ranges == [("all", 0, len(prog.bwd))] and None not in prog.bwd
        return prog.bwd, outs

    s = torch.cuda.current_stream().cuda_stream
    one, c_one = build(4)
    assert len(one) == 1 and one[0].variant.startswith("gemm16x_group_kernel<%d, 256, 256" % dtype_code(BF16))
    three, c_three = build(3)    # end of the job: three cover 192 CUs together, still better than one after another
    assert len(three) == 1 and three[0].variant.startswith("gemm16x_group_kernel<")
    assert [l.variant.split("<")[0] for l in build(1)[0]] == ["gemm16x_kernel"]
    monkeypatch.setenv("PFEIFE_DW_RETILE", "0")
    four, c_four = build(4)
    assert len(four) == 4
    for l in one + three + four:
        l(s)
    torch.cuda.synchronize()
    for i, (dy, x, c0) in enumerate(probs):
        assert torch.equal(c_one[i], c_four[i])
        if i < 3:
            assert torch.equal(c_three[i], c_four[i])
    torch.testing.assert_close(c_one[0].double(), probs[0][2].double() + probs[0][0].double().t() @ probs[0][1].double(),
                               rtol=2e-3, atol=5e-2)


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_mfma_rate_probe_multiplies_what_it_is_given(hip, dtype):
    """The matrix-instruction rate probe (bench.py's attainable-ceiling record) really issues
    iters * 16 MFMAs per wavefront on the fragments it is handed: every wavefront's 64 per-lane
    checksums add up to iters * sum_{i,j} sum(A_i . B_j), computed here from the fragment layout of
    v_mfma_f32_32x32x16 (lane l holds row or column l % 32 and reduction indices 8 * (l / 32) + 0..7).
    Small integers keep every fp32 sum exact."""
    g = torch.Generator().manual_seed(5)
    frags = torch.randint(-2, 3, (8, 64, 8), generator=g).to(dtype)
    iters, wgs = 7, 3
    sink = torch.full((256 * wgs,), float("nan"), device="cuda")
    hip.mfma_rate(frags.cuda(), iters, wgs, sink)(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    per_k = frags.double().reshape(8, 2, 32, 8).sum(2).reshape(8, 16)     # [fragment][k]: sum over its 32 rows / columns
    want = iters * float((per_k[:4].sum(0) * per_k[4:].sum(0)).sum())
    assert sink.cpu().double().reshape(4 * wgs, 64).sum(1).tolist() == [want] * (4 * wgs)


@pytest.mark.parametrize("variant", [0, 7, 8, 9])
def test_accumulating_products_stay_exact_next_to_other_streams(hip, variant):
    """Weight-gradient products (both operands reduction-strided, fp32 accumulate) on one stream while
    two other streams keep the compute units busy with other products.  Small integers make every
    sum exact in fp32: after n launches the accumulator is n times the product, bit for bit, or a
    launch lost, repeated or mixed up rows."""
    torch.manual_seed(0)
    M, N, K, reps = 1536, 384, 788, 12
    dy = torch.randint(-2, 3, (K, M), device="cuda").to(F16)
    x = torch.randint(-2, 3, (K, N), device="cuda").to(F16)
    want = dy.float().t() @ x.float()
    accs = [torch.zeros(M, N, device="cuda") for _ in range(6)]
    launches = [hip.gemm(dy, x, c, M=M, N=N, K=K, lda=M, ldb=N, ldc=N, a_trans=1, b_trans=1, beta=1, variant=variant)
                for c in accs]
    a2 = torch.randn(K, N, device="cuda").to(F16)
    w2 = torch.randn(M, N, device="cuda").to(F16)
    o2 = torch.empty(K, M, device="cuda", dtype=F16)
    side_a = hip.gemm(a2, w2, o2, M=K, N=M, K=N, lda=N, ldb=N, ldc=M)
    o3 = torch.zeros(M, N, device="cuda")
    side_b = hip.gemm(dy, x, o3, M=M, N=N, K=K, lda=M, ldb=N, ldc=N, a_trans=1, b_trans=1, beta=1)
    main, s1, s2 = torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for _ in range(reps):
        for launch in launches:
            launch(main.cuda_stream)
            side_a(s1.cuda_stream)
            side_b(s2.cuda_stream)
    torch.cuda.synchronize()
    for c in accs:
        assert torch.equal(c, reps * want)
    assert torch.equal(o3, reps * len(accs) * want)


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_weight_gradient_product_unscales_checks_and_stores_inside_a_group(hip, oracle, dtype):
    """A weight-gradient product can divide by a loss scale kept on the device (`unscale_by`), raise
    an overflow flag when it writes a non-finite value (`nonfinite_flag`), and STORE its result
    (beta = 0) as a member of a grouped launch whose other members accumulate.  Against the oracle:
    three products of ragged sizes in one launch (store, accumulate, store), then the same launch
    replayed with an inf planted in one operand: the flag goes up, and stays down without it."""
    rows = 520
    shapes = [(264, 392), (520, 136), (136, 264)]
    scale = torch.tensor([1024.0], device="cuda")
    flag = torch.zeros(1, device="cuda")
    devs, cpus, launches = [], [], []
    for i, (m, n) in enumerate(shapes):
        dy, x = rnd((rows, m), dtype, 10 + i), rnd((rows, n), dtype, 20 + i, 0.1)
        c0 = rnd((m, n), F32, 30 + i)
        beta = int(i == 1)
        dev = dict(a=dy.cuda(), b=x.cuda(), c=c0.clone().cuda())
        kw = dict(M=m, N=n, K=rows, lda=m, ldb=n, ldc=n, a_trans=1, b_trans=1, beta=beta, variant=8)
        launch = hip.gemm(**dev, unscale_by=scale, nonfinite_flag=flag, **kw)
        assert launch.variant.endswith("true, true, %d>" % (4 if beta else 1)) and hip.gemm_stores_checked(launch)
        kw.pop("variant")
        cpu = dict(a=dy, b=x, c=c0.clone())
        oracle.gemm(**cpu, unscale_by=scale.cpu(), **kw)()
        devs.append(dev)
        cpus.append(cpu)
        launches.append(launch)
    group = hip.gemm_group(launches)
    assert group.variant.startswith("gemm16x_group_kernel<") and group.variant.endswith("true, true, 4>")
    group(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for dev, cpu in zip(devs, cpus):
        close((dev["c"].cpu(), cpu["c"]), 1e-3, 1e-4)
    assert float(flag) == 0.0
    # each on its own as well (the store class and the accumulate class of the plain kernel)
    for dev, cpu, launch in zip(devs, cpus, launches):
        if launch.desc.beta:
            continue
        dev["c"].fill_(7.0)
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        close((dev["c"].cpu(), cpu["c"]), 1e-3, 1e-4)
    assert float(flag) == 0.0
    devs[2]["a"][3, 5] = float("inf")
    group(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert float(flag) == 1.0 and not bool(torch.isfinite(devs[2]["c"]).all())
    # kernels without that epilogue refuse the flag loudly (here: operands stored differently)
    a, b = rnd((64, 96), dtype, 1).cuda(), rnd((96, 80), dtype, 2).cuda()
    bad = hip.gemm(a, b, torch.zeros(64, 80, device="cuda"), M=64, N=80, K=96, lda=96, ldb=80, ldc=80, b_trans=1,
                   nonfinite_flag=flag)
    with pytest.raises(RuntimeError, match="nonfinite_flag"):
        bad(torch.cuda.current_stream().cuda_stream)
