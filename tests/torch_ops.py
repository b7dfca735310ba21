"""A stand-in kernel set in plain torch, for tests only.

It has the method names and arguments of return_amd.kernels.hip_ops.HipOps, so that
(a) the engine's host logic (cache, step, scheduler) can be exercised on the CPU,
and (b) every HIP kernel has a plain reference of the same call to be compared with
on the GPU. Formulas cite the reference like the plain model does. Nothing in
return_amd imports this file.
"""
from __future__ import annotations

import torch

from return_amd.parts.runtime import ScaledRows, Slabs


class TorchOps:
    def __init__(self, device="cpu"):
        self.device = torch.device(device)

    # rollout/monkey_patch/qwen3.py:73-75
    def embed(self, table, ids, out):
        out.copy_(table[ids.long()].float())

    # rollout/fused.py:6-17 with the residual addition of qwen3.py:63,67 in front
    def add_rmsnorm(self, h, delta, weight, eps, out, rows=None):
        if isinstance(delta, Slabs):                        # shares of a product: their sum, rounded as the product would be
            delta = delta.tensor.sum(0).to(out.dtype)
        if rows is None:
            if delta is not None:
                h += delta.float()
            v = h
        else:
            v = h[rows.long()]
            if delta is not None:
                v = v + delta[rows.long()].float()
        rstd = 1.0 / torch.sqrt((v * v).sum(-1, keepdim=True) / v.shape[-1] + eps)
        out.copy_((v * rstd * weight).to(out.dtype))

    def residual_add(self, h, delta):
        h += delta.float()

    # rollout/fused.py:36-56 on a [-1, D] view
    def head_rmsnorm(self, x, weight, eps):
        v = x.float()
        rstd = 1.0 / torch.sqrt((v * v).sum(-1, keepdim=True) / v.shape[-1] + eps)
        x.copy_((v * rstd * weight).to(x.dtype))

    # rollout/attention.py:10-25
    def rope(self, x, positions, cos, sin, rotary_dim):
        half = rotary_dim // 2
        c = cos[positions.long()][:, None, :]
        s = sin[positions.long()][:, None, :]
        v = x.float()
        x1, x2 = v[..., :half], v[..., half:rotary_dim]
        o = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, v[..., rotary_dim:]], dim=-1)
        x.copy_(o.to(x.dtype))

    def split_heads(self, qkv, n_q, n_kv, D, q, k, v):
        T = qkv.shape[0]
        q.copy_(qkv[:, :n_q * D].view(T, n_q, D))
        k.copy_(qkv[:, n_q * D:(n_q + n_kv) * D].view(T, n_kv, D))
        v.copy_(qkv[:, (n_q + n_kv) * D:].view(T, n_kv, D))

    # rollout/cache.py:334-337
    def kv_write(self, k, v, k_pool, v_pool, slot_mapping):
        P = k_pool.shape[2]                                 # pools are [pages, kv heads, rows in a page, D]
        page, row = slot_mapping.long() // P, slot_mapping.long() % P
        k_pool[page, :, row] = k
        v_pool[page, :, row] = v

    def qkv_prepare(self, qkv, n_q, n_kv, D, w_q, w_k, eps, positions, cos, sin, rotary_dim, q_out,
                    k_pool, v_pool, slot_mapping):
        T = qkv.shape[0]
        q = qkv[:, :n_q * D].reshape(T, n_q, D).float()
        k = qkv[:, n_q * D:(n_q + n_kv) * D].reshape(T, n_kv, D).float()
        v = qkv[:, (n_q + n_kv) * D:].reshape(T, n_kv, D)

        def norm(x, w):
            return x * (1.0 / torch.sqrt((x * x).sum(-1, keepdim=True) / D + eps)) * w

        def rot(x):
            half = rotary_dim // 2
            c = cos[positions.long()][:, None, :]
            s = sin[positions.long()][:, None, :]
            x1, x2 = x[..., :half], x[..., half:rotary_dim]
            return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, x[..., rotary_dim:]], dim=-1)

        if w_q is not None:
            q, k = norm(q, w_q), norm(k, w_k)
        if rotary_dim:
            q, k = rot(q), rot(k)
        q_out.copy_(q.to(q_out.dtype))
        if k_pool is not None:
            self.kv_write(k.to(qkv.dtype), v, k_pool, v_pool, slot_mapping)

    # rollout/fused.py:103-114
    def silu_mul(self, gu, out):
        I = out.shape[1]
        g, u = gu[:, :I].float(), gu[:, I:].float()
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))

    # rollout/monkey_patch/qwen3.py:21 (F.linear)
    def linear(self, x, w, out_dtype=None):
        if isinstance(x, ScaledRows):                       # rows whose norm this product finishes
            y = (x.tensor.float() @ w.float().t()) * self._rstd(x)
            return y.to(out_dtype or x.tensor.dtype)
        return (x.float() @ w.float().t()).to(out_dtype or x.dtype)

    # A norm finished inside the products around it, as HipOps offers for steps of few rows
    # (norm(h) W^T = rstd * ((h * w_norm) W^T), rollout/fused.py:6-17): here for up to 16 rows of any
    # dtype, with the sum of squares in SHARES columns so that the adding-up is exercised too.
    SHARES = 3

    @staticmethod
    def _rstd(rows):
        return 1.0 / torch.sqrt(rows.partials.sum(-1, keepdim=True) / rows.size + rows.eps)

    def linear_residual(self, x, w):
        """As HipOps: for more than 16 rows the product comes as two shares over halves of K."""
        if isinstance(x, ScaledRows) or x.shape[0] <= 16 or x.shape[1] % 2:
            return self.linear(x, w)
        half = x.shape[1] // 2
        return Slabs(torch.stack([x[:, :half].float() @ w[:, :half].float().t(),
                                  x[:, half:].float() @ w[:, half:].float().t()]))

    def can_defer_norm(self, M, w_last, w_first, gated_first):
        return 1 <= M <= 16 and w_first.shape[1] == w_last.shape[0] >= self.SHARES

    def linear_add_norm(self, x, w, h, norm_weight, eps):
        y = self.linear(x, w)                               # (rounded to the compute dtype like a stored result)
        h += y.float()
        sq = h * h
        cut = [sq[:, i::self.SHARES].sum(-1) for i in range(self.SHARES)]
        return ScaledRows((h * norm_weight).to(y.dtype), torch.stack(cut, dim=1), h.shape[1], eps)

    # rollout/monkey_patch/qwen3.py:20-22
    def linear_silu_mul(self, x, w_gate_up):
        gu = self.linear(x, w_gate_up)
        out = torch.empty(gu.shape[0], w_gate_up.shape[0] // 2, dtype=gu.dtype, device=gu.device)
        self.silu_mul(gu, out)
        return out

    # rollout/attention.py:126-139 over the tables of rollout/cache.py:282-328,
    # gathered as opd/test_parallel.py:14-42 does
    def attention(self, q, out, k_pool, v_pool, step, group, scale, window=0):
        g = step.groups[group]
        n_q, n_kv = q.shape[1], k_pool.shape[1]
        cu_q, cu_p = step.cu_q.tolist(), g.cu_pages.tolist()
        q_start, kv_start = step.q_start.tolist(), g.kv_start.tolist()
        table = g.page_table.long()
        for s in range(step.n_seqs):
            a, b = cu_q[s], cu_q[s + 1]
            pages = table[cu_p[s]:cu_p[s + 1]]
            end = q_start[s] + (b - a)                      # keys held after this step
            k = k_pool[pages].transpose(1, 2).reshape(-1, n_kv, k_pool.shape[3])[:end - kv_start[s]].float()
            v = v_pool[pages].transpose(1, 2).reshape(-1, n_kv, v_pool.shape[3])[:end - kv_start[s]].float()
            k_pos = torch.arange(kv_start[s], end, device=q.device)
            q_pos = torch.arange(q_start[s], end, device=q.device)
            kk = k.repeat_interleave(n_q // n_kv, dim=1)
            vv = v.repeat_interleave(n_q // n_kv, dim=1)
            score = torch.einsum("qhd,khd->hqk", q[a:b].float(), kk) * scale
            hide = k_pos[None, :] > q_pos[:, None]
            if window:
                hide = hide | (k_pos[None, :] <= q_pos[:, None] - window)
            score = score.masked_fill(hide[None], float("-inf"))
            out[a:b] = torch.einsum("hqk,khd->qhd", score.softmax(-1), vv).to(out.dtype)

    # rollout/model.py:15-61 with the draw made by inverse CDF in vocabulary order
    def sample(self, logits, temperature, top_k, top_p, u):
        M, V = logits.shape
        res = torch.empty(M, 2, dtype=torch.int32, device=logits.device)
        for r in range(M):
            row = logits[r].double()
            t = float(temperature[r])
            if t <= 0:
                tok = int(row.argmax())
            else:
                x = row / t
                vals, idx = torch.sort(x, descending=True, stable=True)
                k = int(top_k[r]) if int(top_k[r]) > 0 else V
                vals = vals.masked_fill(torch.arange(V, device=x.device) >= k, float("-inf"))
                cum = vals.softmax(-1).cumsum(-1)
                remove = cum > float(top_p[r])
                remove[1:] = remove[:-1].clone()
                remove[0] = False
                vals = vals.masked_fill(remove, float("-inf"))
                p = torch.zeros(V, dtype=torch.float64, device=x.device)
                p[idx] = vals.softmax(-1)
                c = p.cumsum(-1)
                tok = int((c > float(u[r]) * float(c[-1])).nonzero()[0]) if float(u[r]) < 1 else V - 1
            lp = float(row.log_softmax(-1)[tok])
            res[r, 0] = tok
            res[r, 1] = torch.tensor(lp, dtype=torch.float32).view(torch.int32)
        return res
