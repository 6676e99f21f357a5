"""A plain PyTorch twin of every kernel of the HIP library, with the same call
signatures, computing in 32-bit with elementary torch operations.

Used two ways: on the GPU, each HIP kernel is compared with its twin here on
random inputs; on the CPU, the engine's host logic (batch building, cache
manager, block tables, plan, scheduler) is run end to end with these twins in
place of the kernels, which have no CPU form. Formula sources are the same
reference lines that tests/plain_model.py cites.
"""
from __future__ import annotations

import contextlib
import math

import torch


def _f(t):
    return t.to(torch.float32)


class PlainOps:
    force_generic = False

    def together(self):
        """Independent products: nothing to gain here, they run as they are called."""
        return contextlib.nullcontext()

    beside_min_rows = 8   # low, so that the host tests walk the many-row branch too

    def wants_beside(self, rows, weight_bytes=0):
        return rows >= self.beside_min_rows

    def beside(self):
        """Work for a second stream: here it simply runs where it is called."""
        return contextlib.nullcontext()

    def join(self):
        pass

    def fill_nan_pages(self, pool, pages):
        pool.index_fill_(0, pages.long(), float("nan"))

    def embed(self, tokens, table, out, positions=None, pos_table=None):
        x = _f(table[tokens.long()])
        if pos_table is not None:
            x = x + _f(pos_table[positions.long()])
        out.copy_(x)

    def rmsnorm(self, x, gain, eps, out, delta=None, rows=None, rows_sum=None):
        extra = None
        if delta is not None:
            extra = _f(delta)
        if rows_sum is not None:
            add = torch.zeros_like(x)
            self.moe_combine(add, rows_sum.y, rows_sum.weights, rows_sum.shared, rows_sum.gate)
            extra = add if extra is None else extra + add
        if rows is None:
            if extra is not None:
                x += extra
            v = x
        else:
            v = x[rows.long()]
            if extra is not None:
                v = v + extra[rows.long()]
        ms = (v * v).sum(-1, keepdim=True) / v.shape[-1]
        out.copy_((v * torch.rsqrt(ms + eps) * gain).to(out.dtype))

    def qkv_rope(self, x, w_qkv, bias, qkv, positions, row_seq, inv_freq, rot_dim, n_q, n_kv,
                 head_dim, k_pool, v_pool, block_table, page_size, write_kv=True,
                 interleaved=False, q_norm=None, k_norm=None, norm_eps=0.0):
        self.linear(x, w_qkv, qkv)
        self.rope_kv_write(qkv, bias, positions, row_seq, inv_freq, rot_dim, n_q, n_kv, head_dim,
                           k_pool, v_pool, block_table, page_size, write_kv, interleaved,
                           q_norm, k_norm, norm_eps)

    def rope_kv_write(self, qkv, bias, positions, row_seq, inv_freq, rot_dim, n_q, n_kv, head_dim,
                      k_pool, v_pool, block_table, page_size, write_kv=True, interleaved=False,
                      q_norm=None, k_norm=None, norm_eps=0.0):
        t = qkv.shape[0]
        x = _f(qkv)
        if bias is not None:
            x = x + bias
        x = x.view(t, n_q + 2 * n_kv, head_dim).clone()
        if q_norm is not None:   # query and key heads normed over their dims before they turn
            for lo, hi, gain in ((0, n_q, q_norm), (n_q, n_q + n_kv, k_norm)):
                part = x[:, lo:hi]
                x[:, lo:hi] = part * torch.rsqrt((part * part).mean(-1, keepdim=True) + norm_eps) * gain
        if rot_dim:
            half = rot_dim // 2
            phi = positions.to(torch.float32)[:, None] * inv_freq[None, :]
            c, s = torch.cos(phi)[:, None, :], torch.sin(phi)[:, None, :]
            qk = x[:, :n_q + n_kv, :]
            if interleaved:   # pair i is dims (2i, 2i + 1)
                x1, x2 = qk[..., 0:rot_dim:2].clone(), qk[..., 1:rot_dim:2].clone()
                qk[..., 0:rot_dim:2] = x1 * c - x2 * s
                qk[..., 1:rot_dim:2] = x1 * s + x2 * c
            else:             # pair i is dims (i, i + rot_dim / 2)
                x1, x2 = qk[..., :half].clone(), qk[..., half:rot_dim].clone()
                qk[..., :half] = x1 * c - x2 * s
                qk[..., half:rot_dim] = x1 * s + x2 * c
        qkv.view(t, n_q + 2 * n_kv, head_dim)[:, :n_q] = x[:, :n_q].to(qkv.dtype)
        if not write_kv:
            return
        pos = positions.long()
        page = block_table[row_seq.long(), pos // page_size].long()
        assert (page >= 0).all(), "write into a page that is not held"
        slot = pos % page_size
        k_pool[page, :, slot, :] = x[:, n_q:n_q + n_kv].to(k_pool.dtype)
        v_pool[page, :, slot, :] = x[:, n_q + n_kv:].to(v_pool.dtype)

    def moe_combine(self, residual, y, wts, shared=None, gate=None):
        t, h = residual.shape
        k = wts.shape[1]
        acc = (_f(y).view(t, k, h) * wts[:, :, None]).sum(1)
        if shared is not None:
            g = torch.sigmoid(gate.reshape(t, 1)) if gate is not None else 1.0
            acc = acc + g * _f(shared)
        residual += acc

    def linear(self, x, w, out, bias=None):
        r = _f(x) @ _f(w).T
        if bias is not None:
            r = r + bias
        out.copy_(r.to(out.dtype))

    @staticmethod
    def _act(g, act):
        if act == "silu":
            return g / (1 + torch.exp(-g))
        assert act == "gelu_pytorch_tanh", act
        return 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3)))

    def swiglu_linear(self, x, w_gate_up, out, act="silu", bias=None):
        inner = w_gate_up.shape[0] // 2
        g = _f(x) @ _f(w_gate_up[:inner]).T
        u = _f(x) @ _f(w_gate_up[inner:]).T
        if bias is not None:
            g, u = g + bias[:inner], u + bias[inner:]
        out.copy_((self._act(g, act) * u).to(out.dtype))

    def grouped_swiglu(self, x, w_gate_up, offsets, order, top_k, out, tiles=None, act="silu"):
        e, two_i, _ = w_gate_up.shape
        inner = two_i // 2
        off = offsets.tolist()
        for g in range(e):
            rows = order[off[g]:off[g + 1]].long()
            if rows.numel() == 0:
                continue
            xs = _f(x[rows // top_k])
            gg = xs @ _f(w_gate_up[g, :inner]).T
            uu = xs @ _f(w_gate_up[g, inner:]).T
            out[off[g]:off[g + 1]] = (self._act(gg, act) * uu).to(out.dtype)

    def grouped_down(self, h, w_down, offsets, order, out, tiles=None):
        e = w_down.shape[0]
        off = offsets.tolist()
        for g in range(e):
            rows = order[off[g]:off[g + 1]].long()
            if rows.numel() == 0:
                continue
            out[rows] = (_f(h[off[g]:off[g + 1]]) @ _f(w_down[g]).T).to(out.dtype)

    def router_topk(self, logits, experts, top_k, renorm, ids, wts, score="softmax",
                    choice_bias=None, scale=1.0, n_group=0, topk_group=0):
        l = logits[:, :experts]
        if score == "sigmoid":
            p = 1 / (1 + torch.exp(-l))
        else:
            p = torch.exp(l - l.max(-1, keepdim=True).values)
            p = p / p.sum(-1, keepdim=True)
        work = p.clone() if choice_bias is None else p + choice_bias[None, :]
        rows = torch.arange(work.shape[0])
        if n_group > 1 and topk_group < n_group:
            # group-limited: the groups by their best score, a stable sort (ties: lower group)
            per = experts // n_group
            best_of = work.view(-1, n_group, per).max(-1).values
            keep = torch.sort(best_of, dim=-1, descending=True, stable=True).indices[:, :topk_group]
            is_open = torch.zeros_like(best_of, dtype=torch.bool)
            is_open.scatter_(1, keep, True)
            work = work.masked_fill(~is_open.repeat_interleave(per, dim=1), -float("inf"))
        for j in range(top_k):
            best = work.max(-1).values
            # lowest index among the maxima
            idx = torch.argmax((work == best[:, None]).to(torch.int32), dim=-1)
            ids[:, j] = idx.to(torch.int32)
            wts[:, j] = p[rows, idx]
            work[rows, idx] = -float("inf")
        if renorm:
            wts /= wts.sum(-1, keepdim=True)
        wts *= scale

    def moe_align(self, ids, experts, offsets, order, tiles=None):
        flat = ids.reshape(-1).long()
        counts = torch.bincount(flat, minlength=experts)
        offsets[0] = 0
        offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
        order.copy_(torch.sort(flat, stable=True).indices.to(torch.int32))
        if tiles is not None and tiles.tiles16 is not None:
            off = offsets.tolist()
            for size, out in ((16, tiles.tiles16), (256, tiles.tiles_big)):
                lst = [[e, r, off[e + 1], 0] for e in range(experts)
                       for r in range(off[e], off[e + 1], size)]
                if lst:
                    out[:len(lst)] = torch.tensor(lst, dtype=torch.int32, device=out.device)
                tiles.tile_counts[0 if size == 16 else 1] = len(lst)

    def moe_route(self, logits, experts, top_k, renorm, r, score="softmax", choice_bias=None,
                  scale=1.0, n_group=0, topk_group=0):
        self.router_topk(logits, experts, top_k, renorm, r.ids, r.weights, score, choice_bias,
                         scale, n_group, topk_group)
        self.moe_align(r.ids, experts, r.offsets, r.order, tiles=r)

    def paged_attention(self, qkv, k_pool, v_pool, block_table, ctx, n_q, n_kv, head_dim,
                        page_size, window, scale, out, slopes=None):
        t = qkv.shape[0]
        q = _f(qkv[:, :n_q * head_dim]).view(t, n_q, head_dim)
        group = n_q // n_kv
        pos = ctx.positions.tolist()
        seq = ctx.row_seq.tolist()
        for r in range(t):
            lo = max(0, pos[r] - window + 1) if window else 0
            js = torch.arange(lo, pos[r] + 1)
            pages = block_table[seq[r], js // page_size].long()
            assert (pages >= 0).all(), "read of a page that is not held"
            k = _f(k_pool[pages, :, js % page_size, :])  # [n, n_kv, D]
            v = _f(v_pool[pages, :, js % page_size, :])
            for h in range(n_q):
                g = h // group
                s = (k[:, g, :] @ q[r, h]) * scale
                if slopes is not None:
                    s = s + float(slopes[h]) * (js - pos[r]).float().to(s.device)
                p = torch.exp(s - s.max())
                p = p / p.sum()
                out[r, h * head_dim:(h + 1) * head_dim] = (p @ v[:, g, :]).to(out.dtype)

    def sample(self, logits, temperature, uniform, out, top_k=None, top_p=None, rep_penalty=None,
               pen_tokens=None, pen_counts=None, pen_offsets=None):
        from plain_model import sample_distribution
        r, v = logits.shape
        for i in range(r):
            recent = []
            if pen_offsets is not None:
                for e in range(int(pen_offsets[i]), int(pen_offsets[i + 1])):
                    recent += [int(pen_tokens[e])] * int(pen_counts[e])
            p = sample_distribution(
                logits[i].cpu(), float(temperature[i]), int(top_k[i]) if top_k is not None else 0,
                float(top_p[i]) if top_p is not None else 1.0,
                float(rep_penalty[i]) if rep_penalty is not None else 1.0, recent)
            cdf = torch.cumsum(p.double(), 0)
            idx = int(torch.searchsorted(cdf, torch.tensor(float(uniform[i]) * float(cdf[-1]),
                                                           dtype=torch.float64), right=True))
            out[i] = min(idx, v - 1)
