"""Synthetic MiniCPM-style decoder used to time and check the LoRA path inside a whole decode step.

Not a served model: random-init weights, plain torch for everything that is not LoRA (RMSNorm,
rotary embedding, attention over a dense padded KV cache, SwiGLU), and this package's LoRA
linears for the four stacked projections of every layer.  The shape follows the end-to-end
benchmark configuration: 24 layers, hidden 1024, 16 query heads / 2 KV heads of 64, SwiGLU
intermediate 4096, RMSNorm; decode streams with one new token each.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .layers.lora import LoRAMergedColumnParallelLinear, LoRAQKVParallelLinear, LoRARowParallelLinear


class RMSNorm(nn.Module):
    def __init__(self, hidden: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden))
        self.eps = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        v = x.float()
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.eps)
        return (v * self.weight.float()).to(x.dtype)


def _rotary(t: torch.Tensor, positions: torch.Tensor, base: float = 10000.0) -> torch.Tensor:
    """t [B, H, D], positions [B]: rotate pairs (d, d + D/2)."""
    half = t.size(-1) // 2
    inv = base ** (-torch.arange(half, device=t.device, dtype=torch.float32) / half)
    ang = positions.float()[:, None] * inv[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = t[..., :half].float(), t[..., half:].float()
    return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1).to(t.dtype)


class DecoderLayer(nn.Module):
    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, inter: int, max_loras: int, rank: int):
        super().__init__()
        self.heads, self.kv_heads, self.head_dim = heads, kv_heads, head_dim
        kw = dict(max_loras=max_loras, max_lora_rank=rank)
        self.input_norm = RMSNorm(hidden)
        self.qkv = LoRAQKVParallelLinear(hidden, head_dim, heads, kv_heads, **kw)
        self.o = LoRARowParallelLinear(heads * head_dim, hidden, **kw)
        self.post_norm = RMSNorm(hidden)
        self.gate_up = LoRAMergedColumnParallelLinear(hidden, [inter, inter], **kw)
        self.down = LoRARowParallelLinear(inter, hidden, **kw)

    def forward(self, x, k_cache, v_cache, positions, mask):
        """x [B, hidden]; caches [B, kv_heads, S, head_dim]; positions [B] (index of the new
        token); mask [B, 1, 1, S] True where a cache entry takes part."""
        b = x.size(0)
        q, k, v = self.qkv(self.input_norm(x)).split(
            [self.heads * self.head_dim, self.kv_heads * self.head_dim, self.kv_heads * self.head_dim], dim=-1)
        q = _rotary(q.view(b, self.heads, self.head_dim), positions)
        k = _rotary(k.view(b, self.kv_heads, self.head_dim), positions)
        v = v.view(b, self.kv_heads, self.head_dim)
        index = positions.view(b, 1, 1, 1).expand(b, self.kv_heads, 1, self.head_dim).long()
        k_cache.scatter_(2, index, k.unsqueeze(2))
        v_cache.scatter_(2, index, v.unsqueeze(2))
        # grouped-query decode attention as two batched matmuls over the dense cache (the cache is
        # read once; query heads of a KV head form the rows of its matmul)
        group = self.heads // self.kv_heads
        scores = torch.matmul(q.view(b, self.kv_heads, group, self.head_dim), k_cache.transpose(-1, -2))
        scores = (scores.float() * self.head_dim ** -0.5).masked_fill(~mask, float("-inf"))
        attn = torch.matmul(torch.softmax(scores, dim=-1).to(x.dtype), v_cache)
        x = x + self.o(attn.reshape(b, self.heads * self.head_dim))
        gate, up = self.gate_up(self.post_norm(x)).chunk(2, dim=-1)
        return x + self.down(F.silu(gate) * up)


class MiniDecoder(nn.Module):
    def __init__(self, layers: int = 24, hidden: int = 1024, heads: int = 16, kv_heads: int = 2, head_dim: int = 64,
                 inter: int = 4096, max_loras: int = 32, rank: int = 32):
        super().__init__()
        self.hidden, self.kv_heads, self.head_dim = hidden, kv_heads, head_dim
        self.layers = nn.ModuleList(DecoderLayer(hidden, heads, kv_heads, head_dim, inter, max_loras, rank) for _ in range(layers))
        self.norm = RMSNorm(hidden)

    @torch.no_grad()
    def init_random(self, seed: int, adapters: int, rank: int, alpha: float = 32.0) -> None:
        """Seeded N(0, 0.02)-style base weights and `adapters` seeded adapters on every projection."""
        g = torch.Generator().manual_seed(seed)
        for layer in self.layers:
            for mod in (layer.qkv, layer.o, layer.gate_up, layer.down):
                w = mod.weight
                w.copy_((torch.randn(w.shape, generator=g) * (w.size(1) ** -0.5)).to(w.dtype))
            for slot in range(adapters):
                hid, inter = self.hidden, layer.down.input_size
                q, kv = layer.qkv.q_size, layer.qkv.kv_size

                def ab(k, n):
                    return torch.randn(rank, k, generator=g) * 0.02, torch.randn(n, rank, generator=g) * 0.02

                pairs = [ab(hid, q), ab(hid, kv), ab(hid, kv)]
                layer.qkv.set_slot_lora(slot, torch.stack([p[0] for p in pairs]).to(w.device), [p[1].to(w.device) for p in pairs], rank, alpha / rank)
                a, b2 = ab(q, hid)
                layer.o.set_slot_lora(slot, a.to(w.device), b2.to(w.device), rank, alpha / rank)
                pairs = [ab(hid, inter), ab(hid, inter)]
                layer.gate_up.set_slot_lora(slot, torch.stack([p[0] for p in pairs]).to(w.device), [p[1].to(w.device) for p in pairs], rank, alpha / rank)
                a, b2 = ab(inter, hid)
                layer.down.set_slot_lora(slot, a.to(w.device), b2.to(w.device), rank, alpha / rank)

    def make_cache(self, streams: int, max_len: int, dtype, device, seed: int):
        """Seeded KV caches [layers][2] of shape [streams, kv_heads, max_len, head_dim] (filled on
        the device: they are filler for the attention, not part of any parity claim)."""
        g = torch.Generator(device=device).manual_seed(seed)
        shape = (streams, self.kv_heads, max_len, self.head_dim)
        return [(torch.randn(shape, generator=g, device=device, dtype=dtype), torch.randn(shape, generator=g, device=device, dtype=dtype))
                for _ in self.layers]

    def forward(self, x, caches, positions):
        s = caches[0][0].size(2)
        mask = (torch.arange(s, device=x.device)[None, :] <= positions[:, None])[:, None, None, :]
        for layer, (k_cache, v_cache) in zip(self.layers, caches):
            x = layer(x, k_cache, v_cache, positions, mask)
        return self.norm(x)
