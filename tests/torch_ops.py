"""A test double of the kernel surface in plain torch, for tests of the engine's logic
(batching, cache, scheduler) on a machine without a GPU. It is not part of the product:
the package never selects it, and it computes each operation in the most direct way
(float32 math, loops over requests), reading the cache through the block table as the
kernels must."""

from __future__ import annotations

import math

import torch

from distie_amd.kernels.interface import Ops


class TorchOps(Ops):
    def __init__(self, device="cpu") -> None:
        self.device = torch.device(device)

    def embed(self, ids, table):
        return table[ids.long()].float()

    def rmsnorm(self, x, weight, eps, out_dtype):
        x = x.float()
        y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
        return y.to(out_dtype)

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype):
        residual += delta.float()
        return self.rmsnorm(residual, weight, eps, out_dtype)

    def linear(self, x, weight, bias=None):
        y = x.float() @ weight.float().T
        if bias is not None:
            y = y + bias.float()
        return y.to(x.dtype)

    def linear_f32out(self, x, weight):
        return x.float() @ weight.float().T

    def rope_kv_write(self, qkv, meta, group, k_cache, v_cache, inv_freq, num_heads, num_kv_heads,
                      head_dim, write):
        T = qkv.shape[0]
        view = qkv.view(T, num_heads + 2 * num_kv_heads, head_dim)
        if inv_freq is not None:
            ang = meta.positions.float()[:, None] * inv_freq.float()[None, :]
            rot = 2 * inv_freq.shape[0]
            cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
            qk = view[:, :num_heads + num_kv_heads, :rot].float()
            a, b = qk[..., :rot // 2], qk[..., rot // 2:]
            view[:, :num_heads + num_kv_heads, :rot] = torch.cat(
                [a * cos - b * sin, b * cos + a * sin], -1).to(qkv.dtype)
        if write:
            P = k_cache.shape[2]
            slots = meta.groups[group].slots.long()
            k = view[:, num_heads:num_heads + num_kv_heads]
            v = view[:, num_heads + num_kv_heads:]
            k_cache[slots // P, :, slots % P] = k.to(k_cache.dtype)
            v_cache[slots // P, :, :, slots % P] = v.to(v_cache.dtype)
        return qkv

    def paged_attention(self, qkv, meta, group, k_cache, v_cache, num_heads, num_kv_heads, head_dim,
                        scale, window, extras=None):
        T = qkv.shape[0]
        P = k_cache.shape[2]
        q_all = qkv.view(T, num_heads + 2 * num_kv_heads, head_dim)[:, :num_heads].float()
        out = torch.zeros(T, num_heads, head_dim, dtype=torch.float32, device=qkv.device)
        table = meta.groups[group].block_table.long()
        if meta.table_rows is not None:
            table = table[meta.table_rows.long()]
        cu = meta.cu_q.tolist()
        rep = num_heads // num_kv_heads
        for b in range(meta.num_requests):
            for t in range(cu[b], cu[b + 1]):
                pos = int(meta.positions[t])
                first = 0 if window is None else max(0, pos - window + 1)
                keys = torch.arange(first, pos + 1, device=qkv.device)
                pages = table[b, keys // P]
                assert (pages >= 0).all(), "attention would read a page that was given back"
                k = k_cache[pages, :, keys % P].float()          # [n, KH, D]
                v = v_cache[pages, :, :, keys % P].float()
                k = k.repeat_interleave(rep, dim=1)
                v = v.repeat_interleave(rep, dim=1)
                s = torch.einsum("hd,nhd->hn", q_all[t], k) * scale
                if extras is not None and extras.score_cap is not None:
                    s = extras.score_cap * torch.tanh(s / extras.score_cap)
                if extras is not None and extras.head_slopes is not None:
                    s = s + extras.head_slopes.float()[:, None] * (keys - pos).float()[None, :]
                out[t] = torch.einsum("hn,nhd->hd", torch.softmax(s, -1), v)
        return out.view(T, num_heads * head_dim).to(qkv.dtype)

    def silu_mul(self, gate_up):
        inter = gate_up.shape[1] // 2
        g, u = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        return (g * torch.sigmoid(g) * u).to(gate_up.dtype)

    def gather_rows(self, x, rows):
        return x[rows.long()].clone()

    def argmax(self, logits):
        return logits.argmax(-1).to(torch.int32)

    def sample(self, logits, temperature, seeds, counters):
        return plain_sample(logits, temperature, seeds, counters)


def plain_sample(logits, temperature, seeds, counters):
    """argmax where t <= 0; else the first index whose cumulative softmax weight (float64)
    exceeds u * total, u from the request's (seed, counter)."""
    from engine_util import plain_uniform as uniform_of

    out = []
    for row, t, seed, counter in zip(logits.double().cpu(), temperature.tolist(), seeds.tolist(), counters.tolist()):
        if t <= 0:
            out.append(int(row.argmax()))
            continue
        w = torch.exp((row - row.max()) / t)
        target = uniform_of(seed & ((1 << 64) - 1), counter & ((1 << 64) - 1)) * w.sum()
        hit = (torch.cumsum(w, 0) > target).nonzero()
        out.append(int(hit[0]) if len(hit) else int((w > 0).nonzero()[-1]))
    return torch.tensor(out, dtype=torch.int32, device=logits.device)
