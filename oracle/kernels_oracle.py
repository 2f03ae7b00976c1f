"""TEST INFRASTRUCTURE -- CPU restatement of every kernel of libpfeife_hip.so.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the product (pfeife_amd/) never does.

`OracleKernels` has the same method table as `pfeife_amd.hip.HipKernels`
(include/pfeife_hip.h documents the semantics of each entry point) but computes
with plain PyTorch ops in fp32 on whatever device the tensors live on (CPU in
the unit tests).  Each method returns a closure `launch(stream)` like the HIP
table does, so the same stage program can be replayed on either table.

What pins this oracle (tests/test_oracle_kernels.py): every forward is checked
against the torch.nn.functional routine the reference's stages execute through
ATen (pfeife/mp/worker.py:1494), every backward against torch.autograd of that
routine (pfeife/mp/worker.py:1585-1587), the losses against
nn.CrossEntropyLoss / F.mse_loss (pfeife/loss.py:53-70), and the byte movers
against torch.tensor_split / index_select (pfeife/batch.py:45).
"""
import math

import torch
import torch.nn.functional as F

ACT_NONE, ACT_GELU, ACT_GELU_TANH, ACT_SILU, ACT_RELU = 0, 1, 2, 3, 4


def _act(act, x):
    if act == ACT_GELU:
        return F.gelu(x)
    if act == ACT_GELU_TANH:
        return F.gelu(x, approximate="tanh")
    if act == ACT_SILU:
        return F.silu(x)
    if act == ACT_RELU:
        return F.relu(x)
    return x


def _act_grad(act, x):
    if act == ACT_GELU:
        cdf = 0.5 * (1.0 + torch.erf(x * (1.0 / math.sqrt(2.0))))
        pdf = torch.exp(-0.5 * x * x) * (1.0 / math.sqrt(2.0 * math.pi))
        return cdf + x * pdf
    if act == ACT_GELU_TANH:
        k, c = math.sqrt(2.0 / math.pi), 0.044715
        u = k * (x + c * x ** 3)
        t = torch.tanh(u)
        return 0.5 * (1 + t) + 0.5 * x * (1 - t * t) * k * (1 + 3 * c * x * x)
    if act == ACT_SILU:
        s = torch.sigmoid(x)
        return s * (1 + x * (1 - s))
    if act == ACT_RELU:
        return (x > 0).to(x.dtype)
    return torch.ones_like(x)


def _strided(t, size, stride):
    return torch.as_strided(t, size, stride, t.storage_offset())


def _flat(t, n):
    """First n elements starting at t's data pointer, as a flat view."""
    return _strided(t, (n,), (1,))


def _rows(t, rows, cols, ld):
    return _strided(t, (rows, cols), (ld, 1))


class OracleKernels:
    name = "oracle"
    supports_graphs = False

    def __init__(self, device="cpu"):
        self.device = torch.device(device)

    def run(self, name, *a, **kw):
        getattr(self, name)(*a, **kw)(None)

    def colreduce_workspace(self, rows, cols):
        return 2 * max(1, cols)

    def reduce_workspace(self, n):
        return 1

    # -- dense contractions ----------------------------------------------------
    GEMM_GROUP_MAX = 4

    @staticmethod
    def gemm_groupable(launch):
        return False      # the oracle runs every product on its own

    def gemm_group(self, launches):
        def launch(stream=None):
            for l in launches:
                l(stream)

        return launch

    def gemm(self, a, b, c, M, N, K, lda, ldb, ldc, a_trans=0, b_trans=0, batch=(1, 1), sa=(0, 0), sb=(0, 0),
             sc=(0, 0), alpha=1.0, beta=0, bias=None, round_mid=0, aux_out=None, ld_aux_out=0, act=0, dact=0,
             aux_in=None, ld_aux_in=0, residual=None, ld_res=0, unscale_by=None, nonfinite_flag=None):
        b1, b2 = batch
        in_dtype = a.dtype

        def launch(stream=None):
            A = _strided(a, (b1, b2, M, K), (sa[0], sa[1], 1, lda) if a_trans else (sa[0], sa[1], lda, 1))
            # op(B) is K x N
            Bm = _strided(b, (b1, b2, K, N), (sb[0], sb[1], ldb, 1) if b_trans else (sb[0], sb[1], 1, ldb))
            C = _strided(c, (b1, b2, M, N), (sc[0], sc[1], ldc, 1))
            # unscale_by: a loss scale read when the product runs (GradScaler.unscale_ folded in)
            a_eff = alpha if unscale_by is None else alpha / float(unscale_by.reshape(-1)[0])
            v = a_eff * torch.matmul(A.float(), Bm.float())
            if bias is not None:
                v = v + _flat(bias, N).float()
            if round_mid:
                v = v.to(in_dtype).float()
            if aux_out is not None:
                _rows(aux_out, M, N, ld_aux_out).copy_(v[0, 0].to(in_dtype))
            if act:
                v = _act(act, v)
            if dact:
                v = v * _act_grad(dact, _rows(aux_in, M, N, ld_aux_in).float())
            if residual is not None:
                v = v + _rows(residual, M, N, ld_res).float()
            if beta:
                v = v + C.float()
            C.copy_(v.to(c.dtype))
            if nonfinite_flag is not None and not bool(torch.isfinite(v).all()):
                nonfinite_flag.fill_(1.0)     # the overflow check of the same unscale_

        return launch

    @staticmethod
    def gemm_stores_checked(launch):
        return True       # every product of the oracle honours unscale_by / nonfinite_flag

    # -- fused attention -----------------------------------------------------------
    MAX_FUSED_HEAD_DIM = 96

    @staticmethod
    def _attn_scores(q, k, scale, causal):
        Tq, Tk = q.shape[2], k.shape[2]
        s = torch.matmul(q.float(), k.float().transpose(-1, -2)) * scale
        if causal:
            i = torch.arange(Tq, device=s.device)[:, None]
            j = torch.arange(Tk, device=s.device)[None, :]
            s = s.masked_fill(j > i + (Tk - Tq), float("-inf"))
        return s

    def attention_fwd(self, q, k, v, o, lse, scale, causal):
        def launch(stream=None):
            s = self._attn_scores(q, k, scale, causal)
            l = torch.logsumexp(s, dim=-1)
            p = torch.exp(s - l[..., None]).to(q.dtype).float()   # probabilities enter the PV product in 16 bits
            o.copy_(torch.matmul(p, v.float()).to(o.dtype))
            lse.copy_(l)

        return launch

    def attention_bwd(self, q, k, v, o, d_o, lse, delta, dq, dk, dv, scale, causal):
        def launch(stream=None):
            s = self._attn_scores(q, k, scale, causal)
            p = torch.exp(s - lse[..., None].float())
            do = d_o.float()
            dlt = (do * o.float()).sum(dim=-1)
            delta.copy_(dlt)
            dp = torch.matmul(do, v.float().transpose(-1, -2))
            ds = (p * (dp - dlt[..., None]) * scale).to(q.dtype).float()
            p16 = p.to(q.dtype).float()
            dq.copy_(torch.matmul(ds, k.float()).to(dq.dtype))
            dk.copy_(torch.matmul(ds.transpose(-1, -2), q.float()).to(dk.dtype))
            dv.copy_(torch.matmul(p16.transpose(-1, -2), do).to(dv.dtype))

        return launch

    # -- normalisation -----------------------------------------------------------
    def layernorm_fwd(self, x, gamma, beta, y, mean, rstd, rows, d, eps):
        def launch(stream=None):
            X = _rows(x, rows, d, d).float()
            mu = X.mean(dim=1, keepdim=True)
            var = ((X - mu) ** 2).mean(dim=1, keepdim=True)
            rs = 1.0 / torch.sqrt(var + eps)
            out = (X - mu) * rs * _flat(gamma, d).float()
            if beta is not None:
                out = out + _flat(beta, d).float()
            _rows(y, rows, d, d).copy_(out.to(y.dtype))
            _flat(mean, rows).copy_(mu[:, 0])
            _flat(rstd, rows).copy_(rs[:, 0])

        return launch

    def norm_bwd_partials(self, rows):
        return 1

    def colsum_partials(self, rows):
        return 1

    def colreduce_finalize_batch(self, items):
        def launch(stream=None):
            for ws, off, n, stride, cols, acc in items:
                part = _strided(ws, (n, cols), (stride, 1)) if off == 0 else torch.as_strided(
                    ws, (n, cols), (stride, 1), ws.storage_offset() + off)
                _flat(acc, cols).add_(part.sum(dim=0))

        return launch

    def layernorm_bwd(self, dy, x, gamma, mean, rstd, dx_add, dx, dgamma, dbeta, ws, rows, d, defer=0, _rms=False):
        def launch(stream=None):
            DY = _rows(dy, rows, d, d).float()
            X = _rows(x, rows, d, d).float()
            rs = _flat(rstd, rows).float()[:, None]
            mu = torch.zeros_like(rs) if _rms else _flat(mean, rows).float()[:, None]
            xh = (X - mu) * rs
            g = DY * _flat(gamma, d).float()
            c1 = torch.zeros_like(rs) if _rms else g.mean(dim=1, keepdim=True)
            c2 = (g * xh).mean(dim=1, keepdim=True)
            out = rs * (g - c1 - xh * c2)
            if dx_add is not None:
                out = out + _rows(dx_add, rows, d, d).float()
            _rows(dx, rows, d, d).copy_(out.to(dx.dtype))
            if defer:
                _flat(ws, 2 * d)[:d].copy_((DY * xh).sum(dim=0))
                _flat(ws, 2 * d)[d:].copy_(DY.sum(dim=0))
                return
            if dgamma is not None:
                _flat(dgamma, d).add_((DY * xh).sum(dim=0))
            if dbeta is not None:
                _flat(dbeta, d).add_(DY.sum(dim=0))

        return launch

    def norm_bwd_fused(self, dy, x, gamma, mean, rstd, dx_add, dx, dx_lp, ws, rows, d, want_wgrad, want_colsum):
        """Norm backward plus a 16-bit copy of dx and (want_colsum) the column sums of that copy;
        one partial row set [dgamma | dbeta | colsum] in ws."""
        inner = self.layernorm_bwd(dy, x, gamma, mean, rstd, dx_add, dx, None, None, None, rows, d, defer=0,
                                   _rms=mean is None)

        def launch(stream=None):
            inner(None)
            out = _rows(dx, rows, d, d)
            if dx_lp is not None:
                _rows(dx_lp, rows, d, d).copy_(out.to(dx_lp.dtype))
            n = 3 if want_colsum else 2
            if want_wgrad:
                DY = _rows(dy, rows, d, d).float()
                X = _rows(x, rows, d, d).float()
                rs = _flat(rstd, rows).float()[:, None]
                mu = torch.zeros_like(rs) if mean is None else _flat(mean, rows).float()[:, None]
                _flat(ws, n * d)[:d].copy_((DY * (X - mu) * rs).sum(dim=0))
                _flat(ws, n * d)[d:2 * d].copy_(DY.sum(dim=0))
            if want_colsum:
                _flat(ws, n * d)[2 * d:].copy_(_rows(dx_lp, rows, d, d).float().sum(dim=0))

        return launch

    def groupnorm_workspace(self, B, C, groups):
        return B * 2 * C + B * groups * 2

    def groupnorm_fwd(self, x, gamma, beta, y, mean, rstd, B, HW, C, groups, eps):
        def launch(stream=None):
            X = _strided(x, (B, HW, groups, C // groups), (HW * C, C, C // groups, 1)).float()
            mu = X.mean(dim=(1, 3), keepdim=True)
            var = ((X - mu) ** 2).mean(dim=(1, 3), keepdim=True)
            rs = 1.0 / torch.sqrt(var + eps)
            out = ((X - mu) * rs).reshape(B, HW, C) * _flat(gamma, C).float() + _flat(beta, C).float()
            _strided(y, (B, HW, C), (HW * C, C, 1)).copy_(out.to(y.dtype))
            _flat(mean, B * groups).copy_(mu.reshape(-1))
            _flat(rstd, B * groups).copy_(rs.reshape(-1))

        return launch

    def groupnorm_bwd(self, dy, x, gamma, mean, rstd, dx, dgamma, dbeta, ws, B, HW, C, groups, defer=0):
        def launch(stream=None):
            Cg = C // groups
            X = _strided(x, (B, HW, groups, Cg), (HW * C, C, Cg, 1)).float()
            DY = _strided(dy, (B, HW, groups, Cg), (HW * C, C, Cg, 1)).float()
            mu = _flat(mean, B * groups).float().view(B, 1, groups, 1)
            rs = _flat(rstd, B * groups).float().view(B, 1, groups, 1)
            gm = _flat(gamma, C).float().view(1, 1, groups, Cg)
            xh = (X - mu) * rs
            g = DY * gm
            c1 = g.mean(dim=(1, 3), keepdim=True)
            c2 = (g * xh).mean(dim=(1, 3), keepdim=True)
            out = rs * (g - c1 - xh * c2)
            _strided(dx, (B, HW, C), (HW * C, C, 1)).copy_(out.reshape(B, HW, C).to(dx.dtype))
            pg = (DY * xh).sum(dim=1).reshape(B, C)
            pb = DY.sum(dim=1).reshape(B, C)
            if defer:
                w = _strided(ws, (B, 2, C), (2 * C, C, 1))
                w[:, 0].copy_(pg)
                w[:, 1].copy_(pb)
                return
            if dgamma is not None:
                _flat(dgamma, C).add_(pg.sum(0))
            if dbeta is not None:
                _flat(dbeta, C).add_(pb.sum(0))

        return launch

    def rmsnorm_fwd(self, x, gamma, y, rstd, rows, d, eps):
        def launch(stream=None):
            X = _rows(x, rows, d, d).float()
            rs = 1.0 / torch.sqrt((X * X).mean(dim=1, keepdim=True) + eps)
            _rows(y, rows, d, d).copy_((X * rs * _flat(gamma, d).float()).to(y.dtype))
            _flat(rstd, rows).copy_(rs[:, 0])

        return launch

    def rmsnorm_bwd(self, dy, x, gamma, rstd, dx_add, dx, dgamma, ws, rows, d, defer=0):
        return self.layernorm_bwd(dy, x, gamma, None, rstd, dx_add, dx, dgamma, None, ws, rows, d, defer=defer,
                                  _rms=True)

    def colsum_accumulate(self, x, rows, cols, ld, acc, ws, defer=0):
        def launch(stream=None):
            if defer:
                _flat(ws, cols).copy_(_rows(x, rows, cols, ld).float().sum(dim=0))
                return
            _flat(acc, cols).add_(_rows(x, rows, cols, ld).float().sum(dim=0))

        return launch

    # -- softmax / losses ----------------------------------------------------------
    def softmax_fwd(self, s, ld_s, p, ld_p, rows, cols, q_len, causal):
        def launch(stream=None):
            S = _rows(s, rows, cols, ld_s).float()
            if causal:
                r = torch.arange(rows, device=S.device)[:, None] % q_len
                cidx = torch.arange(cols, device=S.device)[None, :]
                S = S.masked_fill(cidx > r + (cols - q_len), float("-inf"))
            P = torch.softmax(S, dim=1)
            P = torch.nan_to_num(P, nan=0.0)
            full = _rows(p, rows, ld_p, ld_p)
            full.zero_()
            full[:, :cols].copy_(P.to(p.dtype))

        return launch

    def softmax_bwd(self, dp, ld_dp, p, ld_p, ds, ld_ds, rows, cols, scale):
        def launch(stream=None):
            DP = _rows(dp, rows, cols, ld_dp).float()
            P = _rows(p, rows, cols, ld_p).float()
            out = scale * P * (DP - (DP * P).sum(dim=1, keepdim=True))
            full = _rows(ds, rows, ld_ds, ld_ds)
            full.zero_()
            full[:, :cols].copy_(out.to(ds.dtype))

        return launch

    def cross_entropy_fwd(self, logits, targets, row_loss, row_lse, loss, rows, classes, ignore_index):
        def launch(stream=None):
            L = _rows(logits, rows, classes, classes).float()
            t = _flat(targets, rows)
            lse = torch.logsumexp(L, dim=1)
            valid = t != ignore_index
            tt = torch.where(valid, t, torch.zeros_like(t))
            rl = torch.where(valid, lse - L.gather(1, tt[:, None])[:, 0], torch.zeros_like(lse))
            _flat(row_lse, rows).copy_(lse)
            _flat(row_loss, rows).copy_(rl)
            n = valid.sum().float()
            out = _flat(loss, 2)
            out[0] = rl.sum() / n if n > 0 else float("nan")
            out[1] = n

        return launch

    def cross_entropy_bwd(self, logits, targets, row_lse, dloss, loss, dlogits, rows, classes, ignore_index):
        def launch(stream=None):
            L = _rows(logits, rows, classes, classes).float()
            t = _flat(targets, rows)
            lse = _flat(row_lse, rows).float()
            g = (1.0 if dloss is None else _flat(dloss, 1).float()[0]) / _flat(loss, 2)[1]
            valid = t != ignore_index
            sm = torch.exp(L - lse[:, None])
            tt = torch.where(valid, t, torch.zeros_like(t))
            sm.scatter_add_(1, tt[:, None], -torch.ones(rows, 1, dtype=sm.dtype, device=sm.device))
            sm = sm * g * valid[:, None].float()
            _rows(dlogits, rows, classes, classes).copy_(sm.to(dlogits.dtype))

        return launch

    def mse_fwd(self, a, b, partial, loss, n):
        def launch(stream=None):
            d = _flat(a, n).float() - _flat(b, n).float()
            _flat(loss, 1)[0] = (d * d).sum() / n

        return launch

    def mse_bwd(self, a, b, dloss, da, n):
        def launch(stream=None):
            g = 2.0 * (1.0 if dloss is None else _flat(dloss, 1).float()[0]) / n
            _flat(da, n).copy_((g * (_flat(a, n).float() - _flat(b, n).float())).to(da.dtype))

        return launch

    def sum_fwd(self, x, partial, loss, n):
        def launch(stream=None):
            _flat(loss, 1)[0] = _flat(x, n).float().sum() if n > 0 else 0.0

        return launch

    # -- elementwise -----------------------------------------------------------------
    def act_fwd(self, x, y, act, n):
        def launch(stream=None):
            _flat(y, n).copy_(_act(act, _flat(x, n).float()).to(y.dtype))

        return launch

    def act_bwd(self, dy, x, dx, act, n):
        def launch(stream=None):
            _flat(dx, n).copy_((_flat(dy, n).float() * _act_grad(act, _flat(x, n).float())).to(dx.dtype))

        return launch

    def glu_fwd(self, gate, ld_gate, up, ld_up, y, ld_y, act, rows, cols):
        def launch(stream=None):
            g = _rows(gate, rows, cols, ld_gate).float()
            u = _rows(up, rows, cols, ld_up).float()
            _rows(y, rows, cols, ld_y).copy_((_act(act, g).to(gate.dtype).float() * u).to(y.dtype))

        return launch

    def glu_bwd(self, dy, ld_dy, gate, ld_gate, up, ld_up, dgate, ld_dgate, dup, ld_dup, act, rows, cols):
        def launch(stream=None):
            d = _rows(dy, rows, cols, ld_dy).float()
            g = _rows(gate, rows, cols, ld_gate).float()
            u = _rows(up, rows, cols, ld_up).float()
            _rows(dup, rows, cols, ld_dup).copy_((d * _act(act, g).to(gate.dtype).float()).to(dup.dtype))
            _rows(dgate, rows, cols, ld_dgate).copy_((d * u * _act_grad(act, g)).to(dgate.dtype))

        return launch

    def axpby(self, a, alpha, b, beta, out, n):
        def launch(stream=None):
            v = alpha * _flat(a, n).float()
            if b is not None:
                v = v + beta * _flat(b, n).float()
            _flat(out, n).copy_(v.to(out.dtype))

        return launch

    def bias_add(self, x, bias, y, n, bias_len, rows_per_bias=0):
        def launch(stream=None):
            rows = n // bias_len
            X = _flat(x, n).float().view(rows, bias_len)
            if rows_per_bias:
                nb = rows // rows_per_bias
                bb = _strided(bias, (nb, bias_len), (bias_len, 1)).float().repeat_interleave(rows_per_bias, dim=0)
            else:
                bb = _flat(bias, bias_len).float()
            _flat(y, n).copy_((X + bb).reshape(-1).to(y.dtype))

        return launch

    def cast(self, src, dst, n):
        def launch(stream=None):
            _flat(dst, n).copy_(_flat(src, n).to(dst.dtype))

        return launch

    def cast_batch(self, pairs):
        def launch(stream=None):
            for src, dst in pairs:
                dst.copy_(src.to(dst.dtype))

        return launch

    @staticmethod
    def shadow_batch_ok(src, plain, transposed):
        return src.dim() == 2 and src.is_contiguous()

    def shadow_batch(self, items):
        def launch(stream=None):
            for src, plain, tr in items:
                if plain is not None:
                    plain.copy_(src.to(plain.dtype))
                if tr is not None:
                    tr.copy_(src.t().to(tr.dtype))

        return launch

    def transpose_cast(self, src, ld_src, dst, ld_dst, rows, cols):
        def launch(stream=None):
            _rows(dst, cols, rows, ld_dst).copy_(_rows(src, rows, cols, ld_src).t().to(dst.dtype))

        return launch

    def fill(self, dst, value, n):
        def launch(stream=None):
            _flat(dst, n).fill_(value)

        return launch

    # -- dynamic loss scaling: torch.amp.GradScaler's rule (pfeife/mp/worker.py:133-145, 1432-1436)
    # on a float32[8] state {scale, growth tracker, found_inf, completed steps, 4 unused here}
    def scale_by_state(self, src, state, dst, n):
        def launch(stream=None):
            _flat(dst, n).copy_((_flat(src, n).float() * state[0]).to(dst.dtype))

        return launch

    def scaler_unscale(self, grads, n, state):
        def launch(stream=None):
            g = _flat(grads, n)
            g.mul_(1.0 / state[0])
            if not torch.isfinite(g).all():
                state[2] = 1.0

        return launch

    def scaler_update(self, state, growth_factor, backoff_factor, growth_interval):
        def launch(stream=None):
            if float(state[2]) != 0.0:
                state[0] *= backoff_factor
                state[1] = 0.0
            else:
                state[1] += 1.0
                state[3] += 1.0
                if float(state[1]) >= growth_interval:
                    state[0] *= growth_factor
                    state[1] = 0.0
            state[2] = 0.0

        return launch

    def copy_strided(self, src, src_strides, dst, dst_strides, sizes, accumulate=0):
        def launch(stream=None):
            s = _strided(src, tuple(sizes), tuple(src_strides))
            d = _strided(dst, tuple(sizes), tuple(dst_strides))
            if not src.dtype.is_floating_point:
                assert src.dtype == dst.dtype and not accumulate
                d.copy_(s)
            elif accumulate:
                d.copy_((d.float() + s.float()).to(dst.dtype))
            else:
                d.copy_(s.to(dst.dtype))

        return launch

    def rope(self, x, y, cos_t, sin_t, B, T, H, D, xs, ys, inverse, tab_ld=None):
        def launch(stream=None):
            half = D // 2
            ld = half if tab_ld is None else tab_ld
            X = _strided(x, (B, T, H, D), (xs[0], xs[1], xs[2], 1)).float()
            c = _strided(cos_t, (T, half), (ld, 1)).float()[None, :, None, :]
            s = _strided(sin_t, (T, half), (ld, 1)).float()[None, :, None, :]
            if inverse:
                s = -s
            x1, x2 = X[..., :half], X[..., half:]
            out = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)
            _strided(y, (B, T, H, D), (ys[0], ys[1], ys[2], 1)).copy_(out.to(y.dtype))

        return launch

    def grad_accumulate(self, acc, g, n):
        def launch(stream=None):
            _flat(acc, n).add_(_flat(g, n).float())

        return launch

    # -- micro-batch split / merge, embedding ---------------------------------------------
    @staticmethod
    def _bytes(t, n):
        return _flat(t.view(torch.uint8) if t.dtype != torch.uint8 else t, n)

    def split_gather(self, src, dst, row_bytes, row_start, n_rows, index=None):
        def launch(stream=None):
            if n_rows == 0 or row_bytes == 0:
                return
            rows = (_flat(index, n_rows) if index is not None
                    else torch.arange(row_start, row_start + n_rows, device=src.device))
            total = int(rows.max().item() + 1) * row_bytes
            s = self._bytes(src, total).view(-1, row_bytes)
            self._bytes(dst, n_rows * row_bytes).view(n_rows, row_bytes).copy_(s.index_select(0, rows))

        return launch

    def merge_scatter(self, src, dst, row_bytes, row_start, n_rows, index=None):
        def launch(stream=None):
            if n_rows == 0 or row_bytes == 0:
                return
            rows = (_flat(index, n_rows) if index is not None
                    else torch.arange(row_start, row_start + n_rows, device=src.device))
            total = int(rows.max().item() + 1) * row_bytes
            d = self._bytes(dst, total).view(-1, row_bytes)
            d.index_copy_(0, rows, self._bytes(src, n_rows * row_bytes).view(n_rows, row_bytes))

        return launch

    def embedding_fwd(self, table, ids, out, n_ids, dim, vocab):
        def launch(stream=None):
            t = _rows(table, vocab, dim, dim)
            _rows(out, n_ids, dim, dim).copy_(t.index_select(0, _flat(ids, n_ids)).to(out.dtype))

        return launch

    def embedding_bwd(self, dout, ids, dtable, n_ids, dim, vocab, padding_idx=-1):
        def launch(stream=None):
            i = _flat(ids, n_ids)
            g = _rows(dout, n_ids, dim, dim).float()
            if padding_idx >= 0:      # aten::embedding_dense_backward leaves the padding row at zero
                g = g * (i != padding_idx).unsqueeze(1)
            _rows(dtable, vocab, dim, dim).index_add_(0, i, g)

        return launch
