"""A CPU stand-in for the HIP kernel library, for tests of the engine's logic
(batching, cache pages, block tables, cutting of prompts) on machines without
a GPU.  It follows the kernels' contracts (layouts of the paged cache, what is
float32), not their code, and is installed with ``ops.install_test_double``.
It is not part of the engine and not the plain implementation either.
"""
import torch


class EmuOps:
    def embedding(self, ids, table):
        return table[ids.long()].float()

    def add_rms_norm(self, resid, delta, weight, eps, out_dtype, rows=None):
        if rows is None:
            if delta is not None:
                resid += delta.float()
            x = resid
        else:
            x = resid[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()].float()
        r = torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)
        return (x * r * weight.float()).to(out_dtype)

    def rms_norm(self, x, weight, eps):
        xf = x.float()
        r = torch.rsqrt((xf * xf).mean(dim=-1, keepdim=True) + eps)
        return (xf * r * weight.float()).to(x.dtype)

    def linear(self, x, w, out_dtype=None):
        return (x.float() @ w.float().t()).to(out_dtype or x.dtype)

    def qk_norm_rope_store(self, qkv, n_q, n_kv, d, q_norm_w, k_norm_w, eps, cos, sin, rotary_dim, positions,
                           k_cache, v_cache, page_size, slots):
        T = qkv.shape[0]
        x = qkv.float()
        q = x[:, :n_q * d].reshape(T, n_q, d)
        k = x[:, n_q * d:(n_q + n_kv) * d].reshape(T, n_kv, d)
        v = x[:, (n_q + n_kv) * d:].reshape(T, n_kv, d)
        if q_norm_w is not None:
            q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_norm_w.float()
            k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_norm_w.float()
        if cos is not None:
            half = rotary_dim // 2
            c = cos[positions.long()][:, None, :]
            s = sin[positions.long()][:, None, :]

            def rot(t):
                a, b, rest = t[..., :half], t[..., half:rotary_dim], t[..., rotary_dim:]
                return torch.cat([a * c - b * s, a * s + b * c, rest], dim=-1)
            q, k = rot(q), rot(k)
        if slots is not None:
            for t in range(T):
                sl = int(slots[t])
                if sl < 0:
                    continue
                page, off = sl // page_size, sl % page_size
                k_cache[page, :, off, :] = k[t].to(k_cache.dtype)
                v_cache[page, :, :, off] = v[t].to(v_cache.dtype)
        return q.reshape(T, n_q * d).to(qkv.dtype)

    def paged_attention(self, q, k_cache, v_cache, page_size, meta, n_q, n_kv, d, scale, window):
        T = meta.T
        out = torch.zeros((T, n_q, d), dtype=torch.float32)
        qf = q.float().reshape(T, n_q, d)
        bt = meta.block_table
        for t in range(T):
            s = int(meta.token_entry[t])
            p = int(meta.positions[t])
            lo = 0 if not window else max(0, p - window + 1)
            keys = list(range(lo, p + 1))
            pages = [int(bt[s, c // page_size]) for c in keys]
            assert all(pg >= 0 for pg in pages), "attention reads a page that is not held"
            offs = [c % page_size for c in keys]
            K = k_cache[pages, :, offs, :].float()          # [n, n_kv, d]
            V = v_cache[pages, :, :, offs].float()          # [n, n_kv, d]
            for h in range(n_q):
                g = h * n_kv // n_q
                sc = (K[:, g, :] @ qf[t, h]) * scale
                pr = torch.softmax(sc, dim=0)
                out[t, h] = pr @ V[:, g, :]
        return out.reshape(T, n_q * d).to(q.dtype)

    def swiglu(self, gate_up):
        I = gate_up.shape[1] // 2
        g, u = gate_up[:, :I].float(), gate_up[:, I:].float()
        return (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)

    def sample(self, logits, temperature, u):
        out = torch.empty(logits.shape[0], dtype=torch.int32)
        for r in range(logits.shape[0]):
            t = float(temperature[r])
            if t == 0.0:
                out[r] = int(torch.argmax(logits[r]))
            else:
                p = torch.softmax(logits[r].double() / t, dim=0)
                c = torch.cumsum(p, 0)
                idx = int(torch.searchsorted(c, torch.tensor(float(u[r]), dtype=torch.float64), right=True))
                out[r] = min(idx, logits.shape[1] - 1)
        return out
