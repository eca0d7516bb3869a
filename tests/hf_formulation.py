"""An independently written decoder in the formulation of the Hugging Face LLaMA / Baichuan
model code, in float64 and WITHOUT a KV cache: every call recomputes the whole sequence under a
causal mask.  It shares no code with oracle/ops.py or with the product, so a mistake made the same
way in both of those (gate and up swapped, the residual taken after the norm, a rotary position
off by one, q/k/v columns in another order, a stale cache row) shows up as a disagreement.

What it fixes, from the published model definitions:
  LLaMA      h = x + o_proj(softmax(rope(q) rope(k)^T / sqrt(dh) + causal) v),  q, k, v = *_proj(rms(x))
             out = h + down_proj(silu(gate_proj(rms(h))) * up_proj(rms(h)))
             rope(x) = x * cos + rotate_half(x) * sin, inv_freq = 10000^(-2i/dh), position = token index
  Baichuan-13B  the same without rope and with  + slope_h * j  added to the logits (ALiBi)
Weights here are nn.Linear style [out, in]; the fused EET matrix is cat(Wq^T, Wk^T, Wv^T) along the
output axis (python/eet/transformers/modeling_llama.py:85, 764-766).
"""
import math

import numpy as np

F64 = np.float64


def rms(x, gamma, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * gamma


def rotate_half(x):
    d = x.shape[-1]
    return np.concatenate([-x[..., d // 2:], x[..., : d // 2]], -1)


def rope(x, positions):
    """x [B, H, T, dh], positions [T]."""
    d = x.shape[-1]
    inv_freq = 1.0 / (10000.0 ** (np.arange(0, d, 2, dtype=F64) / d))
    ang = positions[:, None].astype(F64) * inv_freq[None, :]
    emb = np.concatenate([ang, ang], -1)
    return x * np.cos(emb)[None, None] + rotate_half(x) * np.sin(emb)[None, None]


def power_of_two_slopes(n):
    """ALiBi slopes for n a power of two: 2^(-8(i+1)/n)."""
    assert n & (n - 1) == 0
    return np.array([2.0 ** (-8.0 * (i + 1) / n) for i in range(n)])


class Layer:
    def __init__(self, wq, wk, wv, wo, wgate, wup, wdown, g_attn, g_ffn, heads, eps, alibi_slopes=None):
        self.w = [np.asarray(m, F64) for m in (wq, wk, wv, wo, wgate, wup, wdown)]
        self.g_attn, self.g_ffn = np.asarray(g_attn, F64), np.asarray(g_ffn, F64)
        self.heads, self.eps, self.slopes = heads, eps, alibi_slopes

    def attention(self, x, pad):
        wq, wk, wv, wo = self.w[:4]
        B, T, hid = x.shape
        H = self.heads
        dh = wq.shape[0] // H
        xn = rms(x, self.g_attn, self.eps)
        q, k, v = [(xn @ w.T).reshape(B, T, H, dh).transpose(0, 2, 1, 3) for w in (wq, wk, wv)]
        if self.slopes is None:
            pos = np.arange(T)
            q, k = rope(q, pos), rope(k, pos)
        s = q @ k.transpose(0, 1, 3, 2) / math.sqrt(dh)
        if self.slopes is not None:
            # the caller builds the bias in fp32 and casts it to fp16 (modeling_baichuan.py:273)
            bias = (np.float32(self.slopes)[:, None] * np.arange(T, dtype=np.float32)[None, :]).astype(np.float16)
            s = s + bias.astype(F64)[None, :, None, :]
        i, j = np.arange(T)[:, None], np.arange(T)[None, :]
        masked = (j > i)[None, None]
        if pad is not None:
            masked = masked | (j[None, None] < np.asarray(pad).reshape(B, 1, 1, 1))
        s = np.where(masked, -np.inf, s)
        m = s.max(-1, keepdims=True)
        m = np.where(np.isinf(m), 0.0, m)
        e = np.exp(s - m)
        p = e / np.maximum(e.sum(-1, keepdims=True), 1e-300)
        ctx = (p @ v).transpose(0, 2, 1, 3).reshape(B, T, H * dh)
        return x + ctx @ wo.T

    def ffn(self, h):
        wgate, wup, wdown = self.w[4:]
        hn = rms(h, self.g_ffn, self.eps)
        gate = hn @ wgate.T
        return h + ((gate / (1.0 + np.exp(-gate))) * (hn @ wup.T)) @ wdown.T

    def __call__(self, x, pad=None):
        return self.ffn(self.attention(x, pad))


class Model:
    def __init__(self, embed, layers, g_final, lm_head, eps):
        self.embed, self.layers = np.asarray(embed, F64), layers
        self.g_final, self.lm_head, self.eps = np.asarray(g_final, F64), np.asarray(lm_head, F64), eps

    def logits(self, ids, pad=None):
        """ids [B, T] -> logits [B, T, vocab] for every position (full recompute)."""
        x = self.embed[ids]
        for layer in self.layers:
            x = layer(x, pad)
        return rms(x, self.g_final, self.eps) @ self.lm_head.T
