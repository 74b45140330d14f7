"""Plain torch forms of the kernel operations (tests only).

Two uses: (1) the GPU tests compare every HIP kernel with the function of the
same name here; (2) CPU tests hand an instance to the engine in place of the
HIP operations, so that the cache, the step function and the scheduler can be
exercised without a GPU.  Nothing in the package imports this file.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def v_pages(kv_layer):
    """The value half of the pages [pages, 2, nkv, P, d]: stored transposed, [pages, nkv, d, P]."""
    pages, _, nkv, P, d = kv_layer.shape
    return kv_layer[:, 1].reshape(pages, nkv, d, P)


class TorchOps:
    def __init__(self, compute_dtype=torch.float64):
        self.cd = compute_dtype

    def embedding(self, ids, table, feedback=None, token_seq=None, seq_slots=None, scale=1.0):
        ids = ids.long()
        if feedback is not None:
            ids = torch.where(ids < 0, feedback.long()[seq_slots.long()[token_seq.long()]], ids)
        return (table[ids].to(self.cd) * scale).to(torch.float32)

    def embedding_rmsnorm(self, ids, table, weight, eps, feedback=None, token_seq=None, seq_slots=None):
        hidden = self.embedding(ids, table, feedback, token_seq, seq_slots)
        x = hidden.to(self.cd)
        x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight.to(self.cd)
        return hidden, x.to(table.dtype)

    # the fused and sliced forms are the HIP kernels' own: this stand-in offers none of them
    def can_fold_norm(self, rows, width, dtype):
        return False

    def can_fuse_rope_attention(self, *sizes):
        return False

    def slices_for(self, M, N, K):
        return 0

    def add_rmsnorm(self, hidden, delta, weight, eps, out_dtype, rows=None):
        if hasattr(delta, "sums"):  # parts.base.PartialSums
            delta = delta.sums
        if delta is not None and delta.dim() == 3:  # partial sums of a product taken in slices
            delta = delta.to(self.cd).sum(0)
        if rows is None:
            if delta is not None:
                hidden += delta.to(hidden.dtype)
            h = hidden
        else:
            h = hidden[rows.long()]
            if delta is not None:
                h = h + delta[rows.long()].to(hidden.dtype)
        x = h.to(self.cd)
        y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight.to(self.cd)
        return y.to(out_dtype)

    def rmsnorm(self, x, weight, eps, out_dtype=None):
        xx = x.to(self.cd)
        y = xx / torch.sqrt((xx * xx).mean(-1, keepdim=True) + eps) * weight.to(self.cd)
        return y.to(out_dtype or x.dtype)

    def linear(self, x, weight, out_dtype=None, fold=None, sums_ok=False):
        assert fold is None, "this stand-in folds no norm (can_fold_norm says so)"
        return (x.to(self.cd) @ weight.to(self.cd).t()).to(out_dtype or x.dtype)

    def add_bias(self, x, bias):
        x += bias.to(x.dtype)
        return x

    def rope_table(self, positions, inv_freq):
        ang = (positions.to(torch.float32)[:, None] * inv_freq[None, :]).double()  # float32 product
        return torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).to(torch.float32)

    def qk_norm_rope_write(self, qkv, slots, q_weight, k_weight, cos_sin, rotary_dim, eps, kv_layer,
                           num_q_heads, num_kv_heads, head_dim, write_kv=True):
        nq, nkv, d = num_q_heads, num_kv_heads, head_dim
        N = qkv.shape[0]
        x = qkv.to(self.cd)
        q = x[:, : nq * d].reshape(N, nq, d)
        k = x[:, nq * d : (nq + nkv) * d].reshape(N, nkv, d)
        v = x[:, (nq + nkv) * d :].reshape(N, nkv, d)

        def norm(t, w):
            if w is None:
                return t
            return t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps) * w.to(self.cd)

        def rope(t):
            if rotary_dim == 0:
                return t
            half = rotary_dim // 2
            c, s = cos_sin[:, None, :, 0].to(self.cd), cos_sin[:, None, :, 1].to(self.cd)
            x1, x2 = t[..., :half], t[..., half:rotary_dim]
            return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, t[..., rotary_dim:]], dim=-1)

        q = rope(norm(q, q_weight))
        k = rope(norm(k, k_weight))
        if write_kv:
            P = kv_layer.shape[3]
            for n in range(N):
                slot = int(slots[n])
                if slot < 0:
                    continue
                page, off = slot // P, slot % P
                kv_layer[page, 0, :, off, :] = k[n].to(kv_layer.dtype)
                v_pages(kv_layer)[page, :, :, off] = v[n].to(kv_layer.dtype)
        return q.to(qkv.dtype).contiguous()

    def paged_attention(self, q, kv_layer, block_table, seq_slots, cu_tokens, kv_lens, token_seq, window, scale,
                        min_q_len=0, max_q_len=0, max_kv_len=0, sinks=None):
        N, nq, d = q.shape
        nkv, P = kv_layer.shape[2], kv_layer.shape[3]
        group = nq // nkv
        out = torch.zeros((N, nq, d), dtype=self.cd, device=q.device)
        for s in range(seq_slots.shape[0]):
            slot = int(seq_slots[s])
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            kv_len = int(kv_lens[s])
            for t in range(q0, q1):
                pos = kv_len - (q1 - q0) + (t - q0)
                lo = max(0, pos - window + 1) if window else 0
                idx = torch.arange(lo, pos + 1, device=q.device)
                pages = block_table[slot, (idx // P).long()].long()
                assert int(pages.min()) >= 0, "attention reads a page that was given back"
                offs = (idx % P).long()
                keys = kv_layer[pages, 0, :, offs, :].to(self.cd)  # [n, nkv, d]
                vals = v_pages(kv_layer)[pages, :, :, offs].to(self.cd)  # [n, nkv, d]
                keys = keys.repeat_interleave(group, dim=1)
                vals = vals.repeat_interleave(group, dim=1)
                sc = torch.einsum("hd,nhd->hn", q[t].to(self.cd), keys) * scale
                if sinks is None:
                    p = torch.softmax(sc, dim=-1)
                else:  # one more place in every head's sum, with a score of its own and no value
                    sk = sinks.to(self.cd)[:, None]
                    big = torch.maximum(sc.max(dim=1, keepdim=True).values, sk)
                    e = torch.exp(sc - big)
                    p = e / (e.sum(1, keepdim=True) + torch.exp(sk - big))
                out[t] = torch.einsum("hn,nhd->hd", p, vals)
        return out.reshape(N, nq * d).to(q.dtype)

    def silu_mul(self, gate_up):
        I = gate_up.shape[1] // 2
        g, u = gate_up[:, :I].to(self.cd), gate_up[:, I:].to(self.cd)
        return (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)

    def gate_up_silu(self, x, weight):
        return self.silu_mul(self.linear(x, weight))

    # -- arrangements that norm a sublayer's output -------------------------------------------
    def cast(self, x, dtype):
        return x.to(dtype)

    def scale_(self, x, factor):
        x.copy_((x.to(self.cd) * factor).to(x.dtype))
        return x

    def rmsnorm_add(self, hidden, y, weight, eps, out_dtype, extra=None):
        v = y.to(self.cd)
        if extra is not None:
            v = v + extra.to(self.cd)
        v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight.to(self.cd)
        hidden.copy_((hidden.to(self.cd) + v).to(hidden.dtype))
        return hidden.to(out_dtype)

    # -- gated recurrence --------------------------------------------------------------------
    def mingru_scan(self, zxg, z_bias, x_bias, state, seq_slots, cu_tokens, out_dtype, max_q_len=0):
        W = z_bias.shape[0]
        v = zxg.to(self.cd)
        z = torch.sigmoid(v[:, :W] + z_bias.to(self.cd))
        u = v[:, W : 2 * W] + x_bias.to(self.cd)
        c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        g = v[:, 2 * W :]
        g = g * torch.sigmoid(g)
        out = torch.empty((zxg.shape[0], W), dtype=self.cd, device=zxg.device)
        for s in range(seq_slots.shape[0]):
            row = int(seq_slots[s])
            S = state[row].to(self.cd)
            for t in range(int(cu_tokens[s]), int(cu_tokens[s + 1])):
                S = (1.0 - z[t]) * S + z[t] * c[t]
                out[t] = S * g[t]
            state[row] = S.to(state.dtype)
        return out.to(out_dtype)

    # -- latent attention --------------------------------------------------------------------
    @staticmethod
    def _rotate_pairs(x, cos_sin, rot_dims):
        """x [N, ..., r]: pairs (2i, 2i + 1) of the first rot_dims elements turned by cos_sin [N, rot_dims / 2, 2]."""
        if rot_dims == 0:
            return x
        y = x.clone()
        shape = [x.shape[0]] + [1] * (x.dim() - 2) + [rot_dims // 2]
        c, s = cos_sin[..., 0].to(x.dtype).view(shape), cos_sin[..., 1].to(x.dtype).view(shape)
        u, v = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
        y[..., 0:rot_dims:2] = u * c - v * s
        y[..., 1:rot_dims:2] = v * c + u * s
        return y

    def latent_kv_write(self, dkv, norm_w, eps, cos_sin, rot_dims, slots, pages, page_size, rank, rot):
        x = dkv.to(self.cd)
        c = x[:, :rank]
        c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * norm_w.to(self.cd)
        kr = self._rotate_pairs(x[:, rank:], cos_sin, rot_dims)
        c_pages, t_pages, r_pages = self._latent_pages(pages, page_size, rank, rot)
        for n in range(dkv.shape[0]):
            slot = int(slots[n])
            if slot < 0:
                continue
            c_pages[slot // page_size, slot % page_size] = c[n].to(pages.dtype)
            t_pages[slot // page_size, :, slot % page_size] = c[n].to(pages.dtype)
            r_pages[slot // page_size, slot % page_size] = kr[n].to(pages.dtype)

    @staticmethod
    def _latent_pages(pages, P, rank, rot):
        """Views of a page's three parts: latents [P, rank], the same transposed [rank, P], rotated parts [P, rot]."""
        n = pages.shape[0]
        return (pages[:, : P * rank].unflatten(1, (P, rank)), pages[:, P * rank : 2 * P * rank].unflatten(1, (rank, P)),
                pages[:, 2 * P * rank : P * (2 * rank + rot)].unflatten(1, (P, rot)))

    def latent_query_dtype(self, cache_dtype, page_size, rank, rot):
        return torch.float32

    def latent_q_rope(self, q, cos_sin, rot_dims, heads, dim, rot):
        x = q.view(q.shape[0], heads, dim + rot)[:, :, dim:].to(self.cd)
        return self._rotate_pairs(x, cos_sin, rot_dims).to(torch.float32).contiguous()

    def heads_linear(self, x, heads, col0, K, weight, out_dtype):
        """x [N, heads * xw] or [N, heads, xw]; per head: columns col0 .. col0 + K of its part times weight[h] [out, K]^T."""
        N = x.shape[0]
        xs = x.reshape(N, heads, -1)[:, :, col0 : col0 + K].to(self.cd)
        return torch.einsum("nhk,hok->nho", xs, weight.to(self.cd)).to(out_dtype).contiguous()

    def latent_attention(self, q_lat, q_rot, pages, page_size, rank, rot, block_table, seq_slots, cu_tokens, kv_lens,
                         token_seq, sink, window, scale, max_q_len, max_kv_len, out_dtype):
        N, H, _ = q_lat.shape
        c_pages, _, r_pages = self._latent_pages(pages, page_size, rank, rot)
        out = torch.zeros((N, H, rank), dtype=self.cd, device=pages.device)
        for s in range(seq_slots.shape[0]):
            row = int(seq_slots[s])
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            kv_len = int(kv_lens[s])
            for t in range(q0, q1):
                pos = kv_len - (q1 - q0) + (t - q0)
                lo = max(0, pos - window + 1) if window else 0
                idx = torch.arange(lo, pos + 1, device=pages.device)
                pg = block_table[row, (idx // page_size).long()].long()
                assert int(pg.min()) >= 0, "attention reads a page that was given back"
                off = (idx % page_size).long()
                c = c_pages[pg, off].to(self.cd)  # [n, rank]
                kr = r_pages[pg, off].to(self.cd)
                sc = (q_lat[t].to(self.cd) @ c.T + q_rot[t].to(self.cd) @ kr.T) * scale  # [H, n]
                if sink is None:
                    out[t] = torch.softmax(sc, dim=1) @ c
                    continue
                sk = sink.to(self.cd)[:, None]
                m = torch.maximum(sc.max(dim=1, keepdim=True).values, sk)
                e = torch.exp(sc - m)
                out[t] = (e @ c) / (e.sum(1, keepdim=True) + torch.exp(sk - m))
        return out.to(out_dtype)

    # -- routed feed-forward -----------------------------------------------------------------
    def moe_route(self, logits, bias, top, score="softmax_chosen", experts=None):
        v = logits.to(self.cd)[:, : experts or logits.shape[1]]
        if bias is not None:
            v = v + bias.to(self.cd)
        # (a stable sort: among equal values the lower index comes first)
        idx = torch.sort(v, dim=-1, descending=True, stable=True).indices[:, :top]
        vals = torch.gather(v, 1, idx)
        gains = torch.sigmoid(vals) if score == "sigmoid" else torch.softmax(vals, dim=-1)
        return idx.to(torch.int32), gains.to(torch.float32)

    def moe_route_grouped(self, logits, correction, top, groups=1, keep=1, score="softmax", group_top=1):
        s = torch.sigmoid(logits.to(self.cd)) if score == "sigmoid" else torch.softmax(logits.to(self.cd), dim=-1)
        c = s if correction is None else s + correction.to(self.cd)
        N, E = c.shape
        size = E // groups
        best = torch.sort(c.view(N, groups, size), dim=-1, descending=True).values[:, :, :group_top].sum(-1)
        # (a stable sort: among equal scores the lower index comes first, for groups and for experts)
        kept = torch.sort(best, dim=-1, descending=True, stable=True).indices[:, :keep]
        allowed = torch.zeros((N, groups), dtype=torch.bool, device=c.device).scatter_(1, kept, True)
        c = torch.where(allowed[:, :, None].expand(N, groups, size).reshape(N, E), c, torch.full_like(c, -math.inf))
        ids = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :top]
        chosen = torch.gather(s, 1, ids)
        return ids.to(torch.int32), (chosen / (chosen.sum(-1, keepdim=True) + 1e-20)).to(torch.float32)

    def moe_experts(self, x, ids, gains, gate_up, down, form="gated_silu", gain_on_input=False, limit=0.0):
        if form == "relu2" or gain_on_input:
            return self._moe_experts_plain(x, ids, gains, gate_up, down, form, gain_on_input)
        N, top = ids.shape
        ff = gate_up.shape[1] // 2
        out = torch.zeros((N, down.shape[1]), dtype=self.cd, device=x.device)
        xx = x.to(self.cd)
        for n in range(N):
            for k in range(top):
                e = int(ids[n, k])
                if e >= gate_up.shape[0]:  # an identity expert
                    out[n] += gains[n, k].to(self.cd) * xx[n]
                    continue
                gu = gate_up[e].to(self.cd) @ xx[n]
                if form == "gated_clamp":
                    g, u = torch.clamp(gu[:ff], max=limit), torch.clamp(gu[ff:], min=-limit, max=limit)
                    a = g * torch.sigmoid(1.702 * g) * (u + 1.0)
                else:
                    a = gu[:ff] * torch.sigmoid(gu[:ff]) * gu[ff:]
                a = a.to(x.dtype).to(self.cd)
                out[n] += gains[n, k].to(self.cd) * (down[e].to(self.cd) @ a)
        return out.to(torch.float32)

    def _moe_experts_plain(self, x, ids, gains, up, down, form, gain_on_input):
        assert form == "relu2"
        N, top = ids.shape
        out = torch.zeros((N, down.shape[1]), dtype=self.cd, device=x.device)
        xx = x.to(self.cd)
        for n in range(N):
            for k in range(top):
                e, g = int(ids[n, k]), gains[n, k].to(self.cd)
                z = up[e].to(self.cd) @ xx[n]
                if gain_on_input:
                    z = z * g
                a = (torch.clamp(z, min=0.0) ** 2).to(x.dtype).to(self.cd)
                y = down[e].to(self.cd) @ a
                out[n] += y if gain_on_input else g * y
        return out.to(torch.float32)

    def bias_act(self, z, kind, gated, bias=None, row_gate=None):
        zz = z.to(self.cd)
        if bias is not None:
            zz = zz + bias.to(self.cd)
        act = {"silu": lambda t: t * torch.sigmoid(t), "relu": lambda t: torch.clamp(t, min=0.0),
               "relu2": lambda t: torch.clamp(t, min=0.0) ** 2,
               "gelu_tanh": lambda t: 0.5 * t * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (t + 0.044715 * t ** 3)))}[kind]
        if gated:
            F = zz.shape[1] // 2
            out = act(zz[:, :F]) * zz[:, F:]
        else:
            out = act(zz)
        if row_gate is not None:
            t, col = row_gate
            out = out * torch.sigmoid(t[:, col].to(self.cd))[:, None]
        return out.to(z.dtype)

    def softcap_(self, x, cap):
        x.copy_((cap * torch.tanh(x.to(self.cd) / cap)).to(x.dtype))
        return x

    def rmsnorm_add_rmsnorm(self, hidden, y, weight, eps, next_weight, next_eps, out_dtype, extra=None):
        self.rmsnorm_add(hidden, y, weight, eps, out_dtype, extra)
        x = hidden.to(self.cd)
        return (x / torch.sqrt((x * x).mean(-1, keepdim=True) + next_eps) * next_weight.to(self.cd)).to(out_dtype)

    # -- attention behind a short convolution ------------------------------------------------------
    def conv_norm_rope_write(self, u, taps, state, token_seq, cu_tokens, seq_slots, slots, q_weight, k_weight, cos_sin,
                             rotary_dim, eps, kv_layer, num_q_heads, num_kv_heads, dim, vdim, write_kv=True):
        nq, nkv = num_q_heads, num_kv_heads
        N, cols = u.shape
        J = taps.shape[1]
        D, P = kv_layer.shape[4], kv_layer.shape[3]
        uu, tt = u.to(self.cd), taps.to(self.cd)
        c = torch.zeros_like(uu)
        for s in range(seq_slots.shape[0]):
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            if q1 <= q0:
                continue
            if J > 1:
                before = state[int(seq_slots[s]), : (J - 1) * cols].to(self.cd).view(J - 1, cols)
                rows = torch.cat([before, uu[q0:q1]], dim=0)
            else:
                rows = uu[q0:q1]
            for j in range(J):
                c[q0:q1] += rows[j : j + (q1 - q0)] * tt[:, j]

        def norm(t, w):
            return t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps) * w.to(self.cd)

        def rope(t):
            if rotary_dim == 0:
                return t
            half = rotary_dim // 2
            co, si = cos_sin[:, None, :, 0].to(self.cd), cos_sin[:, None, :, 1].to(self.cd)
            x1, x2 = t[..., :half], t[..., half:rotary_dim]
            return torch.cat([x1 * co - x2 * si, x2 * co + x1 * si, t[..., rotary_dim:]], dim=-1)

        def padded(t):
            return torch.nn.functional.pad(t, (0, D - t.shape[-1]))

        qw, kw = nq * dim, nkv * dim
        q = padded(rope(norm(c[:, :qw].reshape(N, nq, dim), q_weight)))
        if write_kv:
            k = padded(rope(norm(c[:, qw : qw + kw].reshape(N, nkv, dim), k_weight)))
            v = padded(c[:, qw + kw : qw + kw + nkv * vdim].reshape(N, nkv, vdim))
            for n in range(N):
                slot = int(slots[n])
                if slot < 0:
                    continue
                page, off = slot // P, slot % P
                kv_layer[page, 0, :, off, :] = k[n].to(kv_layer.dtype)
                v_pages(kv_layer)[page, :, :, off] = v[n].to(kv_layer.dtype)
        return q.to(u.dtype).contiguous()

    def conv_state_update(self, u, state, kept, cu_tokens, seq_slots):
        cols = u.shape[1]
        for s in range(seq_slots.shape[0]):
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            if q1 <= q0:
                continue
            slot = int(seq_slots[s])
            rows = torch.cat([state[slot, : kept * cols].view(kept, cols), u[q0:q1].to(state.dtype)], dim=0)
            state[slot, : kept * cols] = rows[-kept:].reshape(-1)

    # -- projections normed as a whole, gates per head, side-by-side sublayers -------------------
    def proj_norm_rope_write(self, qkv, bias, slots, q_weight, k_weight, cos_sin, rotary_dim, eps, kv_layer,
                             num_q_heads, num_kv_heads, dim, vdim, has_kv=True, write_kv=True, per_head=False):
        nq, nkv = num_q_heads, num_kv_heads
        N = qkv.shape[0]
        D, P = kv_layer.shape[4], kv_layer.shape[3]
        x = qkv.to(self.cd)
        if bias is not None:
            x = x + bias.to(self.cd)

        def norm(t, w):
            if per_head:
                h = t.reshape(N, -1, dim)
                t = (h / torch.sqrt((h * h).mean(-1, keepdim=True) + eps)).reshape(N, -1)
            else:
                t = t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps)
            return t if w is None else t * w.to(self.cd)

        def rope(t):
            if rotary_dim == 0:
                return t
            half = rotary_dim // 2
            c, s = cos_sin[:, None, :, 0].to(self.cd), cos_sin[:, None, :, 1].to(self.cd)
            x1, x2 = t[..., :half], t[..., half:rotary_dim]
            return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, t[..., rotary_dim:]], dim=-1)

        def padded(t):
            return torch.nn.functional.pad(t, (0, D - t.shape[-1]))

        qw, kw = nq * dim, nkv * dim
        q = padded(rope(norm(x[:, :qw], q_weight).reshape(N, nq, dim)))
        if has_kv and write_kv:
            k = padded(rope(norm(x[:, qw : qw + kw], k_weight).reshape(N, nkv, dim)))
            v = padded(x[:, qw + kw : qw + kw + nkv * vdim].reshape(N, nkv, vdim))
            for n in range(N):
                slot = int(slots[n])
                if slot < 0:
                    continue
                page, off = slot // P, slot % P
                kv_layer[page, 0, :, off, :] = k[n].to(kv_layer.dtype)
                v_pages(kv_layer)[page, :, :, off] = v[n].to(kv_layer.dtype)
        return q.to(qkv.dtype).contiguous()

    # -- the gated delta rule ------------------------------------------------------------------
    def delta_conv(self, u, taps, state, token_seq, cu_tokens, seq_slots, kv_heads, dim, heads, vdim, unit_eps, q_scale):
        N, cols = u.shape
        J = taps.shape[1]
        G, H = kv_heads, heads
        y = torch.zeros((N, cols), dtype=self.cd, device=u.device)
        for s in range(seq_slots.shape[0]):
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            if q1 <= q0:
                continue
            rows = u[q0:q1].to(self.cd)
            if J > 1:
                kept = state[int(seq_slots[s]), : (J - 1) * cols].view(J - 1, cols).to(self.cd)
                rows = torch.cat([kept, rows], dim=0)
            for j in range(J):
                y[q0:q1] += rows[j : j + (q1 - q0)] * taps[:, j].to(self.cd)
        y = y * torch.sigmoid(y)

        def unit(t):
            h = t.reshape(N, G, dim)
            return (h / torch.sqrt((h * h).sum(-1, keepdim=True) + unit_eps)).reshape(N, G * dim)

        q = unit(y[:, : G * dim]) * q_scale
        k = unit(y[:, G * dim : 2 * G * dim])
        return q.to(torch.float32), k.to(torch.float32), y[:, 2 * G * dim :].to(torch.float32).contiguous()

    def delta_scan(self, q, k, v, ba, a_log, dt_bias, state, heads, kv_heads, dim, vdim, seq_slots, cu_tokens):
        N = v.shape[0]
        H, G = heads, kv_heads
        out = torch.zeros((N, H, vdim), dtype=self.cd, device=v.device)
        qq, kk, vv = q.to(self.cd).view(N, G, dim), k.to(self.cd).view(N, G, dim), v.to(self.cd).view(N, H, vdim)
        beta = torch.sigmoid(ba[:, :H].to(self.cd))
        g = torch.exp(-torch.exp(a_log.to(self.cd)) * torch.nn.functional.softplus(ba[:, H:].to(self.cd) + dt_bias.to(self.cd)))
        for s in range(seq_slots.shape[0]):
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            if q1 <= q0:
                continue
            slot = int(seq_slots[s])
            S = state[slot, : H * vdim * dim].view(H, vdim, dim).to(self.cd).clone()  # [head][value][key]
            for t in range(q0, q1):
                for h in range(H):
                    j = h // (H // G)
                    S[h] = g[t, h] * S[h]
                    w = beta[t, h] * (vv[t, h] - S[h] @ kk[t, j])
                    S[h] = S[h] + torch.outer(w, kk[t, j])
                    out[t, h] = S[h] @ qq[t, j]
            state[slot, : H * vdim * dim] = S.reshape(-1).to(state.dtype)
        return out.reshape(N, H * vdim).to(torch.float32)

    def delta_out_norm(self, o, gate, norm_w, eps, heads, vdim):
        N = o.shape[0]
        x = o.to(self.cd).view(N, heads, vdim)
        x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * norm_w.to(self.cd)
        gg = gate.to(self.cd).view(N, heads, vdim)
        return (x * gg * torch.sigmoid(gg)).reshape(N, heads * vdim).to(gate.dtype)

    def head_gate(self, a, gates, col0, heads, vdim):
        N = a.shape[0]
        g = torch.sigmoid(gates[:, col0 : col0 + heads].to(self.cd))
        return (a.view(N, heads, -1)[:, :, :vdim].to(self.cd) * g[:, :, None]).reshape(N, heads * vdim).to(a.dtype)

    def tanh_(self, x):
        x.copy_(torch.tanh(x.to(self.cd)).to(x.dtype))
        return x

    def scaled_add_rmsnorm(self, hidden, a, b, mult, weight, eps, out_dtype, rows=None):
        d = a.to(torch.float32) if b is None else a.to(torch.float32) + b.to(torch.float32)
        if rows is None:
            hidden += mult * d
            h = hidden
        else:
            h = hidden[rows.long()] + mult * d[rows.long()]
        x = h.to(self.cd)
        return (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight.to(self.cd)).to(out_dtype)

    # -- recurrence with a matrix state ----------------------------------------------------------
    def shift_mix(self, x, state, prev_offset, mu, token_seq, cu_tokens, seq_slots):
        N, W = x.shape
        xx = x.to(self.cd)
        prev = torch.zeros_like(xx)
        prev[1:] = xx[:-1]
        for s in range(seq_slots.shape[0]):
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            if q1 > q0:
                prev[q0] = state[int(seq_slots[s]), prev_offset : prev_offset + W].to(self.cd)
        return (xx[None] + (prev - xx)[None] * mu.to(self.cd)[:, None, :]).to(x.dtype)

    def wkv_scan(self, r, k, v, wraw, w0, u, g, norm_w, eps, x, state, heads, dim, seq_slots, cu_tokens, out_dtype,
                 max_q_len=0):
        N, W = x.shape
        HD = heads * dim
        decay = torch.exp(-torch.exp(wraw.to(self.cd) + w0.to(self.cd))).view(N, heads, dim)
        rr, kk, vv = (t.to(self.cd).view(N, heads, dim) for t in (r, k, v))
        uu = u.to(self.cd).view(heads, dim)
        out = torch.zeros((N, heads, dim), dtype=self.cd, device=x.device)
        for s in range(seq_slots.shape[0]):
            slot = int(seq_slots[s])
            q0, q1 = int(cu_tokens[s]), int(cu_tokens[s + 1])
            if q1 <= q0:
                continue
            S = state[slot, : HD * dim].to(self.cd).view(heads, dim, dim).clone()
            for t in range(q0, q1):
                kv = kk[t][:, :, None] * vv[t][:, None, :]
                out[t] = torch.einsum("hi,hij->hj", rr[t], S + uu[:, :, None] * kv)
                S = decay[t][:, :, None] * S + kv
            state[slot, : HD * dim] = S.reshape(-1).to(state.dtype)
            state[slot, HD * dim : HD * dim + W] = x[q1 - 1].to(state.dtype)
        out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps)
        gg = g.to(self.cd)
        y = out.reshape(N, HD) * norm_w.to(self.cd) * (gg * torch.sigmoid(gg))
        return y.to(out_dtype)

    def argmax(self, logits, scatter=None):
        out = torch.argmax(logits, dim=-1).to(torch.int32)  # torch returns the first maximum
        if scatter is not None:
            scatter[0][scatter[1].long()] = out
        return out

    def sample(self, logits, temperature, uniform):
        out = []
        for r in range(logits.shape[0]):
            T = float(temperature[r])
            if T <= 0:
                out.append(int(torch.argmax(logits[r])))
                continue
            z = logits[r].double() / T
            p = torch.exp(z - z.max())
            cdf = torch.cumsum(p, 0)
            target = float(uniform[r]) * float(cdf[-1])
            i = int(torch.searchsorted(cdf, torch.tensor(target, dtype=cdf.dtype), right=True))
            out.append(min(i, logits.shape[1] - 1))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)
