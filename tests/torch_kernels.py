"""Plain torch versions of the engine's device operations, one per kernel, with the same
signatures as nano_vllm_amd.kernels.ops.HipKernels.

Two uses, both in tests only: each HIP kernel is compared with its function here, and the
engine's host logic (batching, cache, scheduler) runs on them on the CPU, where no GPU is
present.  The product never imports this file.
"""
from __future__ import annotations

import torch


def _round(x, dtype):
    return x.to(dtype).to(torch.float32)


def v_tile(page_size: int) -> int:
    """Keys per tile of the V cache [pages, kv_heads, page / vt, head_dim, vt]."""
    return 32 if page_size % 32 == 0 else page_size


def new_caches(pages, kv_heads, head_dim, page_size, dtype, device, fill=None):
    """K [pages, kv_heads, page, head_dim] and V [pages, kv_heads, page / vt, head_dim, vt]."""
    vt = v_tile(page_size)
    k = torch.zeros((pages, kv_heads, page_size, head_dim), dtype=dtype, device=device)
    v = torch.zeros((pages, kv_heads, page_size // vt, head_dim, vt), dtype=dtype, device=device)
    if fill is not None:
        k.normal_(0, fill)
        v.normal_(0, fill)
    return k, v


class TorchKernels:
    name = "torch-plain"

    def __init__(self, device="cpu", dtype=torch.float32):
        self.device = torch.device(device)
        self.dtype = dtype
        self.fault_flag = torch.zeros(1, dtype=torch.int32, device=self.device)

    def check_faults(self):
        pass

    # rows
    def embedding(self, table, ids, out=None):
        y = table[ids.long()]
        if out is not None:
            out.copy_(y)
            return out
        return y

    gather_rows = embedding

    # norms (layernorm.py:16-40)
    def rms_norm(self, x, weight, eps, out=None):
        xf = x.float()
        y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
        y = (_round(y, x.dtype) * weight.float()).to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def add_rms_norm(self, x, residual, weight, eps, out=None):
        s = x.float() + residual.float()
        residual.copy_(s.to(x.dtype))
        y = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps)
        y = (_round(y, x.dtype) * weight.float()).to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out, residual
        return y, residual

    # feed-forward (activation.py:8-11)
    def silu_mul(self, gate_up, out=None):
        inner = gate_up.shape[1] // 2
        g, u = gate_up[:, :inner].float(), gate_up[:, inner:].float()
        y = (g * torch.sigmoid(g) * u).to(gate_up.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def linear(self, x, weight, bias=None, out_float32=False, out=None, deferred=False):
        y = x.float() @ weight.float().T
        if bias is not None:
            y = y + bias.float()
        y = y if out_float32 else y.to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def linear_silu_mul(self, x, weight):
        return self.silu_mul(self.linear(x, weight))

    # position encoding (rotary_embedding.py:29-35)
    def rotary_table(self, inv_freq, num_positions):
        t = torch.arange(num_positions, dtype=torch.float32, device=inv_freq.device)
        ang = t[:, None] * inv_freq[None, :]
        return torch.cat((ang.cos(), ang.sin()), dim=-1)

    def qk_norm_rope_store(self, qkv, num_heads, num_kv_heads, head_dim, q_weight, k_weight, eps, table,
                           positions, slots, k_cache, v_cache, max_position=None):
        if table is not None:
            assert max_position is not None and max_position <= table.shape[0], "a position has no row in the table"
        T = qkv.shape[0]
        D = head_dim
        qd, kd = num_heads * D, num_kv_heads * D
        dt = qkv.dtype

        def prepare(x, heads, w):
            x = x.float().reshape(T, heads, D)
            if w is not None:
                x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
                x = _round(_round(x, dt) * w.float(), dt)
            if table is not None:
                row = table[positions.long()]                       # [T, R]: the first R channels of a head are rotated
                R = row.shape[1]
                cos, sin = row[:, None, : R // 2], row[:, None, R // 2:]
                x1, x2 = x[..., : R // 2], x[..., R // 2:R]
                x = torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., R:]), dim=-1)
            return x.to(dt)

        q = prepare(qkv[:, :qd], num_heads, q_weight)
        qkv[:, :qd] = q.reshape(T, qd)
        if num_kv_heads:
            k = prepare(qkv[:, qd:qd + kd], num_kv_heads, k_weight)
            qkv[:, qd:qd + kd] = k.reshape(T, kd)
            if k_cache is not None:
                page_size = k_cache.shape[2]
                v = qkv[:, qd + kd:].reshape(T, num_kv_heads, D)
                s = slots.long()
                ok = s >= 0
                page, off = s[ok] // page_size, s[ok] % page_size
                vt = v_cache.shape[4]
                k_cache[page, :, off, :] = k[ok]
                v_cache[page, :, off // vt, :, off % vt] = v[ok]
        return qkv[:, :qd]

    # attention (attention.py:64-75): token by token through the block table
    def paged_attention(self, q, num_heads, num_kv_heads, head_dim, k_cache, v_cache, batch, group, scale,
                        window=None, out=None):
        T = q.shape[0]
        D, G = head_dim, num_heads // num_kv_heads
        page_size = k_cache.shape[2]
        tables = batch.groups[group].block_tables
        o = torch.zeros((T, num_heads * D), dtype=torch.float32, device=q.device)
        pos_l, seq_l = batch.positions.tolist(), batch.token_seq.tolist()
        for t in range(T):
            pos, seq = pos_l[t], seq_l[t]
            first = max(0, pos - window + 1) if window else 0
            js = torch.arange(first, pos + 1, device=q.device)
            pages = tables[seq].long()[js // page_size]
            assert bool((pages >= 0).all()), "a visible key has no page"
            offs = js % page_size
            keys = k_cache[pages, :, offs, :].float()                # [n, Hkv, D]
            vt = v_cache.shape[4]
            vals = v_cache[pages, :, offs // vt, :, offs % vt].float()   # [n, Hkv, D]
            qt = q[t].float().reshape(num_heads, D)
            for h in range(num_heads):
                s = (keys[:, h // G] @ qt[h]) * scale
                p = torch.softmax(s, dim=0)
                o[t, h * D:(h + 1) * D] = p @ vals[:, h // G]
        y = o.to(q.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    # sampling (sampler.py:8-12), same counter-based noise as the kernel
    def sample(self, logits, temperatures, keys):
        import math
        M = (1 << 64) - 1

        def mix(z):
            z = (z + 0x9E3779B97F4A7C15) & M
            z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
            z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
            return z ^ (z >> 31)

        out = []
        for r in range(logits.shape[0]):
            l = logits[r].double().cpu()
            t = float(temperatures[r])
            if t > 0:
                key = int(keys[r]) & M
                noise = torch.tensor([math.log(-math.log((((mix(key ^ i)) >> 40) + 0.5) / 16777216.0))
                                      for i in range(l.numel())], dtype=torch.float64)
                l = l / t - noise
            out.append(int(torch.argmax(l)))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)
