"""A two-layer Llama-shaped decoder with random weights, for end-to-end tests of the driver.

``forward_paged`` is token-major and attends through ``PagedAttentionBackend``;
``forward_naive`` recomputes full causal attention over padded ``[B, S]`` inputs with the
library's own rotary / repeat_kv / SDPA functions (the arithmetic the reference's model
file runs, compiler_fx/modeling_llama.py:560-625).
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F


class TinyLlama(nn.Module):
    def __init__(self, vocab=199, hidden=256, layers=2, hq=4, hkv=2, d=128, inter=384, rope_base=10000.0, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.hq, self.hkv, self.d, self.layers = hq, hkv, d, layers
        w = lambda *s: nn.Parameter(torch.randn(*s, generator=g) / math.sqrt(s[-1]))
        self.embed = nn.Parameter(torch.randn(vocab, hidden, generator=g))
        self.qkv = nn.ParameterList([w((hq + 2 * hkv) * d, hidden) for _ in range(layers)])
        self.o = nn.ParameterList([w(hidden, hq * d) for _ in range(layers)])
        self.gate_up = nn.ParameterList([w(2 * inter, hidden) for _ in range(layers)])
        self.down = nn.ParameterList([w(hidden, inter) for _ in range(layers)])
        self.head = w(vocab, hidden)
        self.register_buffer("inv_freq", 1.0 / (rope_base ** (torch.arange(0, d, 2, dtype=torch.float32) / d)))

    @staticmethod
    def norm(x):
        return (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(x.dtype)

    def mlp(self, i, x):
        gu = F.linear(x, self.gate_up[i])
        g_, u = gu.chunk(2, dim=-1)
        return F.linear(F.silu(g_) * u, self.down[i])

    def forward_paged(self, ids, positions, backend):
        x = self.embed[ids]                                   # [T, hidden]
        T = x.shape[0]
        hq, hkv, d = self.hq, self.hkv, self.d
        for i in range(self.layers):
            qkv = F.linear(self.norm(x), self.qkv[i])         # [T, (Hq + 2 Hkv) D]: q, k, v are column slices
            q = qkv[:, :hq * d].view(T, hq, d)
            k = qkv[:, hq * d:(hq + hkv) * d].view(T, hkv, d)
            v = qkv[:, (hq + hkv) * d:].view(T, hkv, d)
            a = backend.attend(i, q, k, v)
            x = x + F.linear(a.reshape(T, hq * d), self.o[i])
            x = x + self.mlp(i, self.norm(x))
        return F.linear(self.norm(x), self.head)

    def forward_naive(self, ids):
        """ids [B, S] -> logits [B, S, V]; plain causal attention over the whole input."""
        from transformers.models.llama.modeling_llama import apply_rotary_pos_emb, repeat_kv
        B, S = ids.shape
        hq, hkv, d = self.hq, self.hkv, self.d
        x = self.embed[ids]
        pos = torch.arange(S, device=ids.device, dtype=torch.float32)
        freqs = pos[:, None] * self.inv_freq[None, :]
        emb = torch.cat((freqs, freqs), dim=-1)
        cos, sin = emb.cos().to(x.dtype)[None], emb.sin().to(x.dtype)[None]      # [1, S, D]
        for i in range(self.layers):
            qkv = F.linear(self.norm(x), self.qkv[i])
            q = qkv[..., :hq * d].view(B, S, hq, d).transpose(1, 2)
            k = qkv[..., hq * d:(hq + hkv) * d].view(B, S, hkv, d).transpose(1, 2)
            v = qkv[..., (hq + hkv) * d:].view(B, S, hkv, d).transpose(1, 2)
            q, k = apply_rotary_pos_emb(q, k, cos, sin)
            k, v = repeat_kv(k, hq // hkv), repeat_kv(v, hq // hkv)
            a = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True).to(x.dtype)
            x = x + F.linear(a.transpose(1, 2).reshape(B, S, hq * d), self.o[i])
            x = x + self.mlp(i, self.norm(x))
        return F.linear(self.norm(x), self.head)
