"""Pins the CPU oracle of the kernels (oracle/kernels_oracle.py) against the
PyTorch library routines that the reference's stages execute through ATen, and
against torch.autograd for every backward formula.  A dropped term, a wrong sign
or a transposed operand in the oracle fails one of these."""
import math

import pytest
import torch
import torch.nn.functional as F

F32 = torch.float32


def rnd(shape, seed, scale=1.0, dtype=F32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("a_trans,b_trans", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_layouts_match_matmul(oracle, a_trans, b_trans):
    M, N, K = 13, 9, 21
    A, B = rnd((M, K), 1), rnd((K, N), 2)  # logical op(A), op(B)
    a = (A.t() if a_trans else A).contiguous()
    b = (B if b_trans else B.t()).contiguous()
    c = torch.zeros(M, N + 2)
    oracle.run("gemm", a, b, c, M=M, N=N, K=K, lda=a.shape[1], ldb=b.shape[1], ldc=N + 2, a_trans=a_trans,
               b_trans=b_trans, alpha=2.0)
    torch.testing.assert_close(c[:, :N], 2.0 * A @ B)
    assert torch.all(c[:, N:] == 0)


def test_gemm_is_linear_forward_and_backward(oracle):
    M, N, K = 10, 6, 8
    x, w, bias = rnd((M, K), 1).requires_grad_(), rnd((N, K), 2).requires_grad_(), rnd((N,), 3)
    res = rnd((M, N), 4)
    y = res + F.gelu(F.linear(x, w, bias))
    dy = rnd((M, N), 5)
    y.backward(dy)
    # forward with fused bias + gelu + residual
    c, h = torch.zeros(M, N), torch.zeros(M, N)
    oracle.run("gemm", x.detach(), w.detach(), c, M=M, N=N, K=K, lda=K, ldb=K, ldc=N, bias=bias, aux_out=h,
               ld_aux_out=N, act=1, residual=res, ld_res=N)
    torch.testing.assert_close(c, y.detach())
    torch.testing.assert_close(h, F.linear(x, w, bias).detach())
    # dH = dY * gelu'(h) then dx = dH W, dW = dH^T x (accumulated)
    dh = torch.zeros(M, N)
    oracle.run("act_bwd", dy, h, dh, act=1, n=M * N)
    dx = torch.zeros(M, K)
    oracle.run("gemm", dh, w.detach(), dx, M=M, N=K, K=N, lda=N, ldb=K, ldc=K, b_trans=1)
    torch.testing.assert_close(dx, x.grad)
    dw = torch.ones(N, K)
    oracle.run("gemm", dh, x.detach(), dw, M=N, N=K, K=M, lda=N, ldb=K, ldc=K, a_trans=1, b_trans=1, beta=1)
    torch.testing.assert_close(dw - 1, w.grad)
    # fused activation gradient in the dX product: (dY W2) * gelu'(h)
    w2 = rnd((K, N), 6)
    g = torch.zeros(M, N)
    oracle.run("gemm", rnd((M, K), 7), w2, g, M=M, N=N, K=K, lda=K, ldb=N, ldc=N, b_trans=1, dact=1, aux_in=h,
               ld_aux_in=N)
    hh = h.clone().requires_grad_()
    (F.gelu(hh) * (rnd((M, K), 7) @ w2)).sum().backward()
    torch.testing.assert_close(g, hh.grad)


def test_gemm_batched_attention_matches_sdpa(oracle):
    B, T, H, hd = 2, 5, 3, 8
    C = H * hd
    qkv = rnd((B, T, 3 * C), 1)
    s = torch.zeros(B, H, T, 8)
    oracle.run("gemm", qkv[:, :, :C], qkv[:, :, C:2 * C], s, M=T, N=T, K=hd, lda=3 * C, ldb=3 * C, ldc=8,
               batch=(B, H), sa=(T * 3 * C, hd), sb=(T * 3 * C, hd), sc=(H * T * 8, T * 8), alpha=hd ** -0.5)
    p = torch.zeros(B, H, T, 8)
    oracle.run("softmax_fwd", s, 8, p, 8, rows=B * H * T, cols=T, q_len=T, causal=1)
    o = torch.zeros(B, T, C)
    oracle.run("gemm", p, qkv[:, :, 2 * C:], o, M=T, N=hd, K=T, lda=8, ldb=3 * C, ldc=C, b_trans=1, batch=(B, H),
               sa=(H * T * 8, T * 8), sb=(T * 3 * C, hd), sc=(T * C, hd))
    q, k, v = (x.reshape(B, T, H, hd).transpose(1, 2) for x in qkv.split(C, dim=2))
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B, T, C)
    torch.testing.assert_close(o, ref)
    assert torch.all(p[..., T:] == 0)


@pytest.mark.parametrize("rms", [False, True])
def test_norms_match_torch_and_autograd(oracle, rms):
    rows, d = 7, 24
    x = (rnd((rows, d), 1) + 0.3).requires_grad_()
    gamma, beta = (rnd((d,), 2) + 1).requires_grad_(), rnd((d,), 3).requires_grad_()
    y, mean, rstd = torch.zeros(rows, d), torch.zeros(rows), torch.zeros(rows)
    if rms:
        ref = F.rms_norm(x, (d,), gamma, 1e-6)
        oracle.run("rmsnorm_fwd", x.detach(), gamma.detach(), y, rstd, rows=rows, d=d, eps=1e-6)
    else:
        ref = F.layer_norm(x, (d,), gamma, beta, 1e-5)
        oracle.run("layernorm_fwd", x.detach(), gamma.detach(), beta.detach(), y, mean, rstd, rows=rows, d=d, eps=1e-5)
    torch.testing.assert_close(y, ref.detach())
    dy, add = rnd((rows, d), 4), rnd((rows, d), 5)
    ref.backward(dy)
    dx, dg, db = torch.zeros(rows, d), torch.full((d,), 2.0), torch.full((d,), 3.0)
    if rms:
        oracle.run("rmsnorm_bwd", dy, x.detach(), gamma.detach(), rstd, add, dx, dg, None, rows=rows, d=d)
    else:
        oracle.run("layernorm_bwd", dy, x.detach(), gamma.detach(), mean, rstd, add, dx, dg, db, None, rows=rows, d=d)
        torch.testing.assert_close(db - 3.0, beta.grad)
    torch.testing.assert_close(dx, x.grad + add)
    torch.testing.assert_close(dg - 2.0, gamma.grad)
    # fused form: same dx, plus its fp16 copy, the copy's column sums and the parameter partials
    dx2, lp, ws = torch.zeros(rows, d), torch.zeros(rows, d, dtype=torch.float16), torch.zeros(3 * d)
    oracle.run("norm_bwd_fused", dy, x.detach(), gamma.detach(), None if rms else mean, rstd, add, dx2, lp, ws,
               rows=rows, d=d, want_wgrad=True, want_colsum=True)
    assert torch.equal(dx2, dx) and torch.equal(lp, dx.to(torch.float16))
    torch.testing.assert_close(ws[:d], gamma.grad)
    if not rms:
        torch.testing.assert_close(ws[d:2 * d], beta.grad)
    torch.testing.assert_close(ws[2 * d:], (x.grad + add).to(torch.float16).float().sum(0))


def test_softmax_backward_matches_autograd(oracle):
    rows, cols = 6, 11
    s = rnd((rows, cols), 1).requires_grad_()
    scale = 0.3
    p_ref = torch.softmax(s * scale, dim=1)
    dp = rnd((rows, cols), 2)
    p_ref.backward(dp)
    p = torch.zeros(rows, 16)
    oracle.run("softmax_fwd", (s * scale).detach(), cols, p, 16, rows=rows, cols=cols, q_len=1, causal=0)
    torch.testing.assert_close(p[:, :cols], p_ref.detach())
    ds = torch.ones(rows, 16)
    oracle.run("softmax_bwd", dp, cols, p, 16, ds, 16, rows=rows, cols=cols, scale=scale)
    torch.testing.assert_close(ds[:, :cols], s.grad)
    assert torch.all(ds[:, cols:] == 0)


def test_cross_entropy_matches_nn_loss(oracle):
    rows, classes = 9, 13
    logits = rnd((rows, classes), 1, 2.0).requires_grad_()
    targets = torch.tensor([0, 12, 3, -100, 5, 5, -100, 1, 2])
    ref = torch.nn.CrossEntropyLoss()(logits, targets)  # the module pfeife/loss.py:53-60 wraps
    (ref * 1.7).backward()
    row_loss, row_lse, loss = torch.zeros(rows), torch.zeros(rows), torch.zeros(2)
    oracle.run("cross_entropy_fwd", logits.detach(), targets, row_loss, row_lse, loss, rows=rows, classes=classes,
               ignore_index=-100)
    torch.testing.assert_close(loss[0], ref.detach())
    assert loss[1] == 7
    dl = torch.zeros(rows, classes)
    oracle.run("cross_entropy_bwd", logits.detach(), targets, row_lse, torch.tensor([1.7]), loss, dl, rows=rows,
               classes=classes, ignore_index=-100)
    torch.testing.assert_close(dl, logits.grad)


def test_mse_and_sum(oracle):
    a, b = rnd((37,), 1).requires_grad_(), rnd((37,), 2)
    ref = F.mse_loss(a, b)
    (ref * 0.5).backward()
    loss, da = torch.zeros(1), torch.zeros(37)
    oracle.run("mse_fwd", a.detach(), b, None, loss, n=37)
    oracle.run("mse_bwd", a.detach(), b, torch.tensor([0.5]), da, n=37)
    torch.testing.assert_close(loss[0], ref.detach())
    torch.testing.assert_close(da, a.grad)
    oracle.run("sum_fwd", b, None, loss, n=37)
    torch.testing.assert_close(loss[0], b.sum())


@pytest.mark.parametrize("act,fn", [(1, F.gelu), (2, lambda x: F.gelu(x, approximate="tanh")), (3, F.silu),
                                    (4, F.relu)])
def test_activation_and_glu_gradients(oracle, act, fn):
    x = rnd((50,), 1, 2.0).requires_grad_()
    dy = rnd((50,), 2)
    fn(x).backward(dy)
    y, dx = torch.zeros(50), torch.zeros(50)
    oracle.run("act_fwd", x.detach(), y, act=act, n=50)
    oracle.run("act_bwd", dy, x.detach(), dx, act=act, n=50)
    torch.testing.assert_close(y, fn(x).detach())
    torch.testing.assert_close(dx, x.grad)
    g, u = rnd((5, 8), 3).requires_grad_(), rnd((5, 8), 4).requires_grad_()
    d = rnd((5, 8), 5)
    (fn(g) * u).backward(d)
    out, dg, du = torch.zeros(5, 8), torch.zeros(5, 8), torch.zeros(5, 8)
    oracle.run("glu_fwd", g.detach(), 8, u.detach(), 8, out, 8, act=act, rows=5, cols=8)
    oracle.run("glu_bwd", d, 8, g.detach(), 8, u.detach(), 8, dg, 8, du, 8, act=act, rows=5, cols=8)
    torch.testing.assert_close(out, (fn(g) * u).detach())
    torch.testing.assert_close(dg, g.grad)
    torch.testing.assert_close(du, u.grad)


def test_rope_matches_rotate_half_and_its_autograd(oracle):
    B, T, H, D = 2, 5, 3, 8
    x = rnd((B, T, H, D), 1).requires_grad_()
    inv_freq = 1.0 / (10000 ** (torch.arange(0, D, 2).float() / D))
    ang = torch.arange(T).float()[:, None] * inv_freq[None, :]
    cos, sin = torch.cat([ang, ang], -1).cos()[None, :, None, :], torch.cat([ang, ang], -1).sin()[None, :, None, :]

    def rotate_half(t):
        return torch.cat([-t[..., D // 2:], t[..., :D // 2]], dim=-1)

    ref = x * cos + rotate_half(x) * sin  # HF Llama apply_rotary_pos_emb
    dy = rnd((B, T, H, D), 2)
    ref.backward(dy)
    y, dx = torch.zeros(B, T, H, D), torch.zeros(B, T, H, D)
    st = (T * H * D, H * D, D)
    oracle.run("rope", x.detach(), y, ang.cos().contiguous(), ang.sin().contiguous(), B, T, H, D, st, st, inverse=0)
    oracle.run("rope", dy, dx, ang.cos().contiguous(), ang.sin().contiguous(), B, T, H, D, st, st, inverse=1)
    torch.testing.assert_close(y, ref.detach())
    torch.testing.assert_close(dx, x.grad)


def test_byte_movers_match_tensor_split_and_embedding(oracle):
    full = torch.arange(10 * 3, dtype=torch.int64).view(10, 3)
    out = []
    start = 0
    for ch in torch.tensor_split(full, 4, 0):  # pfeife/batch.py:45
        slab = torch.zeros_like(ch)
        oracle.run("split_gather", full, slab, row_bytes=24, row_start=start, n_rows=ch.shape[0])
        assert torch.equal(slab, ch)
        out.append(slab)
        start += ch.shape[0]
    merged = torch.zeros_like(full)
    start = 0
    for slab in out:
        oracle.run("merge_scatter", slab, merged, row_bytes=24, row_start=start, n_rows=slab.shape[0])
        start += slab.shape[0]
    assert torch.equal(merged, full)
    table = rnd((20, 6), 1).requires_grad_()
    ids = torch.tensor([3, 3, 7, 0, 19, 3])
    e = F.embedding(ids, table)
    d = rnd((6, 6), 2)
    e.backward(d)
    o, dt = torch.zeros(6, 6), torch.zeros(20, 6)
    oracle.run("embedding_fwd", table.detach(), ids, o, n_ids=6, dim=6, vocab=20)
    oracle.run("embedding_bwd", d, ids, dt, n_ids=6, dim=6, vocab=20)
    assert torch.equal(o, e.detach())
    torch.testing.assert_close(dt, table.grad)
    # padding row: torch keeps its gradient at zero
    table.grad = None
    F.embedding(ids, table, padding_idx=3).backward(d)
    dt = torch.zeros(20, 6)
    oracle.run("embedding_bwd", d, ids, dt, n_ids=6, dim=6, vocab=20, padding_idx=3)
    torch.testing.assert_close(dt, table.grad)
    assert float(dt[3].abs().max()) == 0.0 and float(dt[7].abs().max()) > 0.0


def test_streaming(oracle):
    a, b = rnd((17,), 1), rnd((17,), 2)
    out = torch.zeros(17)
    oracle.run("axpby", a, 2.0, b, -1.0, out, n=17)
    torch.testing.assert_close(out, 2 * a - b)
    acc = b.clone()
    oracle.run("grad_accumulate", acc, a.half(), n=17)
    assert torch.equal(acc, b + a.half().float())
    x = rnd((4, 6), 3)
    y = torch.zeros(4, 6)
    oracle.run("bias_add", x, a[:6], y, n=24, bias_len=6)
    torch.testing.assert_close(y, x + a[:6])
    acc = torch.ones(6)
    oracle.run("colsum_accumulate", x, rows=4, cols=6, ld=6, acc=acc, ws=None)
    torch.testing.assert_close(acc, 1 + x.sum(0))


@pytest.mark.parametrize("Tq,Tk,causal", [(9, 9, 1), (7, 12, 0), (5, 5, 0), (4, 10, 1)])
def test_fused_attention_matches_sdpa_and_its_autograd(oracle, Tq, Tk, causal):
    """attention_fwd / attention_bwd against F.scaled_dot_product_attention and autograd in fp32 (where
    the oracle's 16-bit roundings of P and dS are the identity).  Causal with Tq != Tk: the oracle's
    (and the kernels') bottom-right alignment, written here as an explicit mask."""
    B, H, hd = 2, 3, 8
    q, k, v = (rnd((B, H, T, hd), i + 1).requires_grad_() for i, T in enumerate((Tq, Tk, Tk)))
    d_o = rnd((B, H, Tq, hd), 4)
    mask = torch.ones(Tq, Tk, dtype=torch.bool).tril(Tk - Tq) if causal else None
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=0.3)
    ref.backward(d_o)
    o, lse, delta = torch.zeros(B, H, Tq, hd), torch.zeros(B, H, Tq), torch.zeros(B, H, Tq)
    dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    oracle.run("attention_fwd", qd, kd, vd, o, lse, 0.3, causal)
    oracle.run("attention_bwd", qd, kd, vd, o, d_o, lse, delta, dq, dk, dv, 0.3, causal)
    torch.testing.assert_close(o, ref.detach())
    s = torch.matmul(qd, kd.transpose(-1, -2)) * 0.3
    if causal:
        s = s.masked_fill(~mask, float("-inf"))
    torch.testing.assert_close(lse, torch.logsumexp(s, -1))
    torch.testing.assert_close(delta, (d_o * ref.detach()).sum(-1))
    torch.testing.assert_close(dq, q.grad)
    torch.testing.assert_close(dk, k.grad)
    torch.testing.assert_close(dv, v.grad)
    if causal and Tq == Tk:   # the square case is also what is_causal=True means
        torch.testing.assert_close(o, F.scaled_dot_product_attention(qd, kd, vd, is_causal=True, scale=0.3))


def test_groupnorm_matches_torch_and_autograd(oracle):
    """groupnorm_fwd / groupnorm_bwd work on channels-last [B, HW, C] activations; F.group_norm on the
    [B, C, HW] view is the reference, autograd gives dx, dgamma, dbeta."""
    B, HW, C, G = 3, 10, 12, 4
    x = (rnd((B, HW, C), 1) * 2 + 0.3).requires_grad_()
    gamma, beta = (rnd((C,), 2) + 1).requires_grad_(), rnd((C,), 3).requires_grad_()
    ref = F.group_norm(x.permute(0, 2, 1), G, gamma, beta, 1e-5).permute(0, 2, 1)
    y, mean, rstd = torch.zeros(B, HW, C), torch.zeros(B * G), torch.zeros(B * G)
    oracle.run("groupnorm_fwd", x.detach(), gamma.detach(), beta.detach(), y, mean, rstd, B=B, HW=HW, C=C, groups=G,
               eps=1e-5)
    torch.testing.assert_close(y, ref.detach())
    xg = x.detach().reshape(B, HW, G, C // G)
    torch.testing.assert_close(mean.view(B, G), xg.mean(dim=(1, 3)))
    torch.testing.assert_close(rstd.view(B, G), 1 / torch.sqrt(xg.var(dim=(1, 3), unbiased=False) + 1e-5))
    dy = rnd((B, HW, C), 4)
    ref.backward(dy)
    dx, dg, db = torch.zeros(B, HW, C), torch.full((C,), 2.0), torch.full((C,), 3.0)
    ws = torch.zeros(oracle.groupnorm_workspace(B, C, G))
    oracle.run("groupnorm_bwd", dy, x.detach(), gamma.detach(), mean, rstd, dx, dg, db, ws, B=B, HW=HW, C=C, groups=G)
    torch.testing.assert_close(dx, x.grad)
    torch.testing.assert_close(dg - 2.0, gamma.grad)
    torch.testing.assert_close(db - 3.0, beta.grad)
    # deferred form: per-batch partial rows [B][2][C] that sum to the same parameter gradients
    oracle.run("groupnorm_bwd", dy, x.detach(), gamma.detach(), mean, rstd, dx, None, None, ws, B=B, HW=HW, C=C,
               groups=G, defer=1)
    part = ws[:B * 2 * C].view(B, 2, C)
    torch.testing.assert_close(part[:, 0].sum(0), gamma.grad)
    torch.testing.assert_close(part[:, 1].sum(0), beta.grad)


def test_transpose_cast_copy_strided_and_column_sums(oracle):
    src = torch.arange(5 * 8, dtype=torch.float32).view(5, 8) / 3
    dst = torch.zeros(6, 8, dtype=torch.float16)          # [cols=6][rows=5], row stride 8
    oracle.run("transpose_cast", src, 8, dst, 8, rows=5, cols=6)
    assert torch.equal(dst[:, :5], src[:, :6].t().to(torch.float16)) and torch.all(dst[:, 5:] == 0)
    # copy_strided: a permuted view into a padded destination, then accumulated once more
    a = rnd((2, 3, 4), 1)
    out = torch.zeros(4, 3, 2 + 1)
    sizes, ss, ds = (4, 3, 2), (1, 4, 12), (9, 3, 1)      # out[k, j, i] = a[i, j, k]
    oracle.run("copy_strided", a, ss, out, ds, sizes)
    assert torch.equal(out[:, :, :2], a.permute(2, 1, 0)) and torch.all(out[:, :, 2] == 0)
    oracle.run("copy_strided", a, ss, out, ds, sizes, accumulate=1)
    assert torch.equal(out[:, :, :2], 2 * a.permute(2, 1, 0))
    ids = torch.arange(6).view(2, 3)
    iout = torch.zeros(3, 2, dtype=torch.int64)
    oracle.run("copy_strided", ids, (1, 3), iout, (2, 1), (3, 2))
    assert torch.equal(iout, ids.t())
    # column sums: immediate and deferred through the batched finish
    x = rnd((7, 6), 2).to(torch.float16)
    acc = torch.full((4,), 1.5)
    oracle.run("colsum_accumulate", x, 7, 4, 6, acc, None)
    torch.testing.assert_close(acc - 1.5, x[:, :4].float().sum(0))
    ws, acc2 = torch.zeros(8), torch.zeros(4)
    oracle.run("colsum_accumulate", x, 7, 4, 6, None, ws, defer=1)
    oracle.run("colreduce_finalize_batch", [(ws, 0, oracle.colsum_partials(7), 4, 4, acc2)])
    torch.testing.assert_close(acc2, x[:, :4].float().sum(0))
