"""A test double for the kernels: the same calls as ``celeg_amd.csrc.hip_ops.HipOps``,
written with torch on the CPU.

It exists only so that the host-side logic of the engine (batch metadata, block
tables, state slots, the step function, the scheduler) can be tested where there is
no GPU.  It is not part of the product: nothing under ``celeg_amd`` imports it, and
the engine refuses to run without its HIP kernels unless a test hands it this object.
"""
from __future__ import annotations

import torch


class CpuOps:
    device = torch.device("cpu")

    def embed(self, table, token_ids, out):
        out.copy_(table[token_ids.long()].float())

    def rmsnorm(self, x, weight, eps, out, delta=None, rows=None):
        if rows is None:
            if delta is not None:
                x.add_(delta.float())
            v = x.float()
        else:
            idx = rows.long()
            v = x[idx].float()
            if delta is not None:
                v = v + delta[idx].float()
        inv = torch.rsqrt((v * v).mean(dim=-1, keepdim=True) + eps)
        out.copy_((v * inv * weight).to(out.dtype))

    def swiglu(self, gate_up, out):
        ff = out.shape[1]
        g, u = gate_up[:, :ff].float(), gate_up[:, ff:].float()
        out.copy_(((g / (1 + torch.exp(-g))) * u).to(out.dtype))

    def add_bias(self, x, bias):
        x.copy_((x.float() + bias).to(x.dtype))

    def cast(self, src, dst):
        dst.copy_(src.reshape(dst.shape).to(dst.dtype))

    def apply_table_updates(self, table, updates, capacity):
        n = int(updates[0])
        for i in range(min(n, capacity)):
            slot, logical, page = (int(v) for v in updates[1 + 3 * i: 4 + 3 * i])
            table[slot, logical] = page

    def linear(self, x, w, out, bias=None):
        y = x.float() @ w.float().t()
        if bias is not None:
            y = y + bias
        out.copy_(y.to(out.dtype))
        return out

    def short_conv(self, bcx, weight, bias, state, out, batch):
        T, H = out.shape
        L = weight.shape[1]
        cu = batch.cu_seqlens.tolist()
        for s in range(batch.n_seqs):
            slot, start = int(batch.seq_slot[s]), int(batch.seq_start[s])
            r0, r1 = cu[s], cu[s + 1]
            rows = bcx[r0:r1].float()
            bx_new = rows[:, :H] * rows[:, 2 * H:]
            old = state[slot].clone()          # [L, H]: positions start-L .. start-1
            history = torch.cat([old, bx_new], dim=0)   # index i <-> position start-L+i
            for r in range(r1 - r0):
                pos = start + r
                conv = torch.zeros(H)
                for tap in range(L):
                    q = pos - (L - 1 - tap)
                    if q >= 0:
                        conv = conv + weight[:, tap] * history[q - start + L]
                if bias is not None:
                    conv = conv + bias
                out[r0 + r] = (rows[r, H:2 * H] * conv).to(out.dtype)
            end = start + (r1 - r0)
            new = torch.zeros(L, H)
            for j in range(L):
                q = end - L + j
                if q >= 0:
                    new[j] = history[q - start + L]
            state[slot] = new

    def qk_norm_rope_store(self, q, k, v, q_weight, k_weight, eps, inv_freq, rotary_dim,
                           heads, kv_heads, head_dim, batch, kv):
        T = q.shape[0]
        pos = batch.positions.long()

        def encode(x, n_heads, weight):
            x = x.float().reshape(T, n_heads, head_dim)
            if weight is not None:
                inv = torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)
                x = x * inv * weight
            if inv_freq is not None:
                half = rotary_dim // 2
                angle = pos.float()[:, None] * inv_freq[None, :]
                c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
                a, b = x[..., :half].clone(), x[..., half:2 * half].clone()
                x = x.clone()
                x[..., :half] = a * c - b * s
                x[..., half:2 * half] = b * c + a * s
            return x

        q.copy_(encode(q, heads, q_weight).reshape(T, -1).to(q.dtype))
        if k is None:
            return
        kk = encode(k, kv_heads, k_weight).to(kv.k.dtype)
        vv = v.reshape(T, kv_heads, head_dim)
        P = kv.page_tokens
        for t in range(T):
            p = int(pos[t])
            page = int(kv.table[int(batch.token_slot[t]), p // P])
            kv.k[page, kv.layer, :, p % P, :] = kk[t]
            kv.v[page, kv.layer, :, :, p % P] = vv[t]

    def paged_attention(self, q, out, heads, kv_heads, head_dim, scale, window, batch, kv):
        T = q.shape[0]
        P = kv.page_tokens
        group = heads // kv_heads
        qf = q.float().reshape(T, heads, head_dim)
        for t in range(T):
            p = int(batch.positions[t])
            slot = int(batch.token_slot[t])
            first = max(0, p - window + 1) if window else 0
            keys = torch.stack([kv.k[int(kv.table[slot, u // P]), kv.layer, :, u % P, :]
                                for u in range(first, p + 1)]).float()   # [n, Hkv, hd]
            vals = torch.stack([kv.v[int(kv.table[slot, u // P]), kv.layer, :, :, u % P]
                                for u in range(first, p + 1)]).float()
            for h in range(heads):
                g = h // group
                s = (keys[:, g] @ qf[t, h]) * scale
                pr = torch.softmax(s, dim=0)
                out[t, h * head_dim:(h + 1) * head_dim] = (pr @ vals[:, g]).to(out.dtype)

    def sample(self, logits, fparams, iparams, seen, out_tokens, last_tokens=None, all_greedy=False):
        import plain_lfm2 as plain   # the double may lean on the plain sampler
        R, V = logits.shape
        for r in range(R):
            t, top_p, pen, u = (float(x) for x in fparams[4 * r: 4 * r + 4])
            k, row, slot = (int(x) for x in iparams[3 * r: 3 * r + 3])
            s = seen[row].bool().tolist() if (seen is not None and row >= 0) else [False] * V
            # the draw comes from the host: walk with it instead of a generator state
            out_tokens[r] = _sample_with_draw(plain, logits[r].tolist(), t, k, top_p, pen, s, u)
            if last_tokens is not None and slot >= 0:
                last_tokens[slot] = out_tokens[r]

    def mark_seen(self, seen, token_ids, token_slot, n):
        for t, s in zip(token_ids[:n].tolist(), token_slot[:n].tolist()):
            if 0 <= s < seen.shape[0]:
                seen[s, t] = 1


def _sample_with_draw(plain, logits, temperature, top_k, top_p, penalty, seen, u):
    orig = plain.random_unit
    plain.random_unit = lambda state: (state, u)
    try:
        return plain.sample(logits, temperature, top_k, top_p, penalty, seen, 1)[0]
    finally:
        plain.random_unit = orig
