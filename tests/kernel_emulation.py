"""A test double for the kernel library: the same calls, computed with torch on the CPU.

It exists so that the engine's own logic (step layout, paged cache, slots, generation loop)
can be tested where there is no GPU.  It is slow and lives under tests/: the product has no
CPU path, and nothing in the package imports this file.
"""

from __future__ import annotations

import torch

PAGE = 64


class TorchKernels:
    page_size = PAGE

    def __init__(self, device="cpu"):
        self.device = torch.device(device)
        self.calls = []

    def embed(self, tokens, table, out):
        self.calls.append("embed")
        out.copy_(table[tokens.long()].float())

    def rmsnorm(self, x, weight, eps, out, rows=None):
        self.calls.append("rmsnorm")
        src = x if rows is None else x[rows.long()]
        inv = 1.0 / torch.sqrt((src.double() ** 2).mean(-1, keepdim=True) + eps)
        y = src * inv.float()
        if weight is not None:
            y = y * weight.float()
        out.copy_(y.to(out.dtype))

    def gemm(self, a, w, out, accumulate=False, then_norm=None):
        self.calls.append("gemm")
        product = (a.double() @ w.double().t()).float()
        if accumulate:
            product = product + out.float()
        out.copy_(product.to(out.dtype))
        return None         # this double never prepares a following norm: the norm runs as a step of its own

    def qk_norm_rope_cache(self, qkv, q_out, q_weight, k_weight, eps, cos, sin, positions, row_seq,
                           k_pages, v_pages, page_table, n_heads, n_kv_heads, head_dim, write_kv, max_position):
        self.calls.append("qk_norm_rope_cache")
        n_rows = qkv.shape[0]
        q_width, kv_width = n_heads * head_dim, n_kv_heads * head_dim
        q = qkv[:, :q_width].float().reshape(n_rows, n_heads, head_dim)
        k = qkv[:, q_width:q_width + kv_width].float().reshape(n_rows, n_kv_heads, head_dim)
        v = qkv[:, q_width + kv_width:].reshape(n_rows, n_kv_heads, head_dim)

        def norm(x, w):
            if w is None:
                return x
            inv = 1.0 / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)
            return x * inv.float() * w.float()

        def rotate(x):
            if cos is None:
                return x
            half = cos.shape[1]
            c = cos[positions.long()][:, None, :]
            s = sin[positions.long()][:, None, :]
            a, b, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
            return torch.cat([a * c - b * s, a * s + b * c, rest], dim=-1)

        q_out.copy_(rotate(norm(q, q_weight)).reshape(n_rows, q_width).to(q_out.dtype))
        if not write_kv:
            return
        k = rotate(norm(k, k_weight))
        for row in range(n_rows):
            pos = int(positions[row])
            page = int(page_table[int(row_seq[row]), pos // PAGE])
            k_pages[page, :, pos % PAGE, :] = k[row].to(k_pages.dtype)
            v_pages[page, :, :, pos % PAGE] = v[row].to(v_pages.dtype)

    def attention(self, q, out, k_pages, v_pages, page_table, row_seq, positions, n_heads, n_kv_heads, head_dim,
                  scale, window=0, layout=None):
        self.calls.append("attention")
        n_rows = q.shape[0]
        group = n_heads // n_kv_heads
        qh = q.float().reshape(n_rows, n_heads, head_dim)
        result = torch.empty_like(qh)
        for row in range(n_rows):
            pos, seq = int(positions[row]), int(row_seq[row])
            first = max(0, pos - window + 1) if window else 0
            index = torch.arange(first, pos + 1)
            pages = page_table[seq, index // PAGE].long()
            keys = k_pages[pages, :, index % PAGE, :].float()      # [n, kv_heads, head_dim]
            values = v_pages[pages, :, :, index % PAGE].float()
            for head in range(n_heads):
                kv = head // group
                scores = (keys[:, kv, :].double() @ qh[row, head].double()).float() * scale
                probs = torch.softmax(scores, dim=0)
                result[row, head] = (probs.double() @ values[:, kv, :].double()).float()
        out.copy_(result.reshape(n_rows, n_heads * head_dim).to(out.dtype))

    def pack_weight(self, w):
        return w

    # ---- residual streams, kept-apart sublayer results ----
    def streams_open(self, x, out):
        self.calls.append("streams_open")
        out.copy_(x.unsqueeze(1).expand_as(out))

    def streams_rmsnorm(self, x, take, weight, eps, out, rows=None):
        self.calls.append("streams_rmsnorm")
        src = x if rows is None else x[rows.long()]
        share = torch.ones(x.shape[1]) if take is None else take.float()
        u = (src.double() * share.double()[None, :, None]).sum(1).float()
        y = u * (1.0 / torch.sqrt((u.double() ** 2).mean(-1, keepdim=True) + eps)).float()
        if weight is not None:
            y = y * weight.float()
        out.copy_(y.to(out.dtype))

    def streams_update(self, x, y, mix=None, give=None, scale=None):
        self.calls.append("streams_update")
        streams = x.shape[1]
        m = torch.eye(streams, dtype=torch.float64) if mix is None else mix.double()
        g = torch.ones(streams, dtype=torch.float64) if give is None else give.double()
        add = y.double() * (scale.double() if scale is not None else 1.0)
        new = torch.einsum("st,nsd->ntd", m, x.double()) + g[None, :, None] * add[:, None, :]
        x.copy_(new.float())

    def streams_update_rmsnorm(self, x, y, mix, give, scale, take, weight, eps, out):
        self.streams_update(x, y, mix, give, scale)
        self.streams_rmsnorm(x, take, weight, eps, out)

    def scale(self, x, factor):
        self.calls.append("scale")
        x.mul_(factor)

    def relu_squared(self, x, out=None):
        self.calls.append("relu_squared")
        (x if out is None else out).copy_((x.float().clamp(min=0) ** 2).to(x.dtype))

    # ---- linear attention with a decay ----
    def lightning_scan(self, proj, q_off, k_off, v_off, state, decay, seq_start, seq_slot, out, n_heads, dim, vdim,
                       max_rows_per_seq=None):
        self.calls.append("lightning_scan")
        silu = lambda z: z / (1 + torch.exp(-z))
        p = proj.float()
        for b in range(seq_slot.shape[0]):
            lo, hi, slot = int(seq_start[b]), int(seq_start[b + 1]), int(seq_slot[b])
            for row in range(lo, hi):
                q = silu(p[row, q_off:q_off + n_heads * dim]).reshape(n_heads, dim)
                k = silu(p[row, k_off:k_off + n_heads * dim]).reshape(n_heads, dim)
                v = silu(p[row, v_off:v_off + n_heads * vdim]).reshape(n_heads, vdim)
                s = state[slot] * decay.float()[:, None, None] + k[:, :, None] * v[:, None, :]
                state[slot] = s
                out[row] = torch.einsum("hdv,hd->hv", s.double(), q.double()).float().reshape(-1)

    def gated_rmsnorm(self, o, proj, gate_off, weight, eps, out):
        self.calls.append("gated_rmsnorm")
        width = o.shape[1]
        y = o * (1.0 / torch.sqrt((o.double() ** 2).mean(-1, keepdim=True) + eps)).float()
        if weight is not None:
            y = y * weight.float()
        out.copy_((y * torch.sigmoid(proj[:, gate_off:gate_off + width].float())).to(out.dtype))

    # ---- attention over a cached latent ----
    @staticmethod
    def _turn(x, freq, turned, positions):
        """x [n, ..., w]: the first `turned` of the last axis in pairs (i, i + turned/2) by the float32 angle position * freq[i]."""
        if not turned:
            return x
        half = turned // 2
        angle = (positions.float()[:, None] * freq.float()[None, :]).double()
        shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (half,)
        c, s = torch.cos(angle).reshape(shape).float(), torch.sin(angle).reshape(shape).float()
        a, b, rest = x[..., :half], x[..., half:turned], x[..., turned:]
        return torch.cat([a * c - b * s, b * c + a * s, rest], dim=-1)

    def latent_write(self, down, offset, weight, eps, freq, turned, positions, row_seq, k_pages, v_pages, page_table,
                     rank, rot_dim, write=True, query=None, query_head=0, query_first=0, source_head=0, source_first=0, n_heads=0):
        self.calls.append("latent_write")
        if query is not None:
            self.rotate_heads(down, source_head, source_first, query, query_head, query_first, freq, turned, positions, n_heads, rot_dim)
        if not write:
            return
        x = down[:, offset:offset + rank + rot_dim].float()
        c = x[:, :rank] * (1.0 / torch.sqrt((x[:, :rank].double() ** 2).mean(-1, keepdim=True) + eps)).float()
        if weight is not None:
            c = c * weight.float()
        key = torch.cat([c, self._turn(x[:, rank:], freq, turned, positions)], dim=-1)
        value = torch.cat([c, torch.zeros(x.shape[0], rot_dim)], dim=-1)
        for row in range(x.shape[0]):
            pos = int(positions[row])
            page = int(page_table[int(row_seq[row]), pos // PAGE])
            k_pages[page, 0, pos % PAGE, :] = key[row].to(k_pages.dtype)
            v_pages[page, 0, :, pos % PAGE] = value[row].to(v_pages.dtype)

    def heads_linear(self, x, x_head, x_first, w, y, y_head, y_first, n_heads):
        self.calls.append("heads_linear")
        n, n_in, n_out = x.shape[0], w.shape[1], w.shape[2]
        xs = x[:, :n_heads * x_head].reshape(n, n_heads, x_head)[:, :, x_first:x_first + n_in]
        result = torch.einsum("nhi,hio->nho", xs.double(), w.double()).float()
        y[:, :n_heads * y_head].view(n, n_heads, y_head)[:, :, y_first:y_first + n_out] = result.to(y.dtype)

    def rotate_heads(self, x, x_head, x_first, y, y_head, y_first, freq, turned, positions, n_heads, width):
        self.calls.append("rotate_heads")
        n = x.shape[0]
        xs = x[:, :n_heads * x_head].reshape(n, n_heads, x_head)[:, :, x_first:x_first + width].float()
        y[:, :n_heads * y_head].view(n, n_heads, y_head)[:, :, y_first:y_first + width] = \
            self._turn(xs, freq, turned, positions).to(y.dtype)

    def gemm_swiglu(self, a, w, out):
        self.calls.append("gemm_swiglu")
        both = torch.empty(a.shape[0], w.shape[0], dtype=a.dtype)
        self.gemm(a, w, both)
        self.swiglu(both, out)

    def swiglu(self, gate_up, out):
        self.calls.append("swiglu")
        width = out.shape[1]
        g, u = gate_up[:, :width].float(), gate_up[:, width:].float()
        out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))

    def sample(self, logits, tokens, bad, temperature=None, top_k=None, top_p=None, uniform=None):
        self.calls.append("sample")
        for row in range(logits.shape[0]):
            x = logits[row]
            if not torch.isfinite(x).all():
                tokens[row], bad[row] = -1, 1
                continue
            bad[row] = 0
            temp = float(temperature[row]) if temperature is not None else 0.0
            if temp <= 0:
                tokens[row] = int(torch.argmax(x))
                continue
            keep = torch.ones_like(x, dtype=torch.bool)
            k = int(top_k[row]) if top_k is not None else 0
            if 0 < k < x.numel():
                keep &= x >= torch.topk(x, k).values[-1]
            e = torch.where(keep, torch.exp((x - x.max()) / temp), torch.zeros_like(x)).double()
            p = float(top_p[row]) if top_p is not None else 1.0
            if 0 < p < 1:
                order = torch.argsort(e, descending=True)
                mass = torch.cumsum(e[order], 0)
                count = int(torch.searchsorted(mass, p * e.sum()).clamp(max=x.numel() - 1)) + 1
                keep &= e >= e[order][count - 1]
                e = torch.where(keep, e, torch.zeros_like(e))
            cdf = torch.cumsum(e, 0)
            target = float(uniform[row]) * float(cdf[-1])
            tokens[row] = int(torch.searchsorted(cdf, torch.tensor(target, dtype=cdf.dtype), right=True)
                              .clamp(max=x.numel() - 1))
