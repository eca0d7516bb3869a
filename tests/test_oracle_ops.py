"""Pins the fp32 oracle ops by what the mathematics fixes: closed forms,
invariants, special cases and brute force.  None of these retype the oracle's
own formula."""
import math

import numpy as np
import pytest

from oracle import ops as O


def test_dequant_matmul_special_cases():
    rng = np.random.default_rng(0)
    K = 64
    x = rng.standard_normal((3, K)).astype(np.float16)
    # q = identity, scale = 1  =>  C = A
    assert np.array_equal(O.dequant_matmul(x, np.eye(K, dtype=np.int8), np.ones(K, np.float16)), x)
    # a single non-zero weight picks one activation and scales it
    q = np.zeros((K, 16), np.int8)
    q[5, 3] = -128
    s = np.full(16, 0.5, np.float16)
    c = O.dequant_matmul(x, q, s, np.float32)
    want = np.zeros((3, 16), np.float32)
    want[:, 3] = x[:, 5].astype(np.float32) * -64.0
    assert np.array_equal(c, want)
    # rows are independent: M = 1 result equals row 0 of the M = 3 result
    q = rng.integers(-128, 128, (K, 16), dtype=np.int8)
    assert np.array_equal(O.dequant_matmul(x[:1], q, s), O.dequant_matmul(x, q, s)[:1])
    # against float64 elementwise brute force
    ref = np.array([[sum(float(x[m, k]) * float(q[k, n]) * float(s[n]) for k in range(K)) for n in range(16)]
                    for m in range(3)])
    assert np.allclose(O.dequant_matmul(x, q, s, np.float32), ref, rtol=1e-5, atol=1e-4)


def test_rmsnorm_closed_forms():
    x = np.full((2, 128), 3.0, np.float16)
    g = np.full(128, 2.0, np.float16)
    # constant row c: c / sqrt(c^2 + eps) * gamma
    assert np.allclose(O.rmsnorm(x, g, 0.0).astype(np.float32), 2.0)
    y = O.rmsnorm(x, g, 9.0).astype(np.float32)          # mean x^2 = 9, eps = 9
    assert np.allclose(y, 3 / math.sqrt(18) * 2, rtol=1e-3)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((4, 256)).astype(np.float16)
    y = O.rmsnorm(x, np.ones(256, np.float16), 1e-6).astype(np.float64)
    assert np.allclose((y * y).mean(-1), 1.0, rtol=2e-3)     # unit RMS out
    assert np.allclose(O.rmsnorm(2 * x, np.ones(256, np.float16), 1e-12).astype(np.float32),
                       O.rmsnorm(x, np.ones(256, np.float16), 1e-12).astype(np.float32), atol=2e-3)  # scale invariant


def rotate_half_rope(x, pos, base=10000.0):
    """The HF formulation: x*cos + rotate_half(x)*sin with inv_freq = base^(-2i/d)."""
    d = x.shape[-1]
    inv_freq = 1.0 / (base ** (np.arange(0, d, 2, dtype=np.float64) / d))
    ang = np.concatenate([pos * inv_freq, pos * inv_freq])
    x = x.astype(np.float64)
    rot = np.concatenate([-x[..., d // 2:], x[..., : d // 2]], -1)
    return x * np.cos(ang) + rot * np.sin(ang)


@pytest.mark.parametrize("dh", [32, 64, 128])
def test_rope(dh):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((3, dh)).astype(np.float16)
    assert np.array_equal(O.rope_neox(x, 0), x)                         # pos 0 is the identity
    for pos in (1, 7, 1023):
        y = O.rope_neox(x, pos).astype(np.float64)
        assert np.allclose(y, rotate_half_rope(x, pos), atol=2e-3)       # equals rotate_half
        assert np.allclose((y * y).sum(-1), (x.astype(np.float64) ** 2).sum(-1), rtol=3e-3)  # a rotation
    # relative property: <rope(q,m), rope(k,n)> depends only on m - n
    q = rng.standard_normal(dh).astype(np.float16)
    k = rng.standard_normal(dh).astype(np.float16)
    d1 = float(O.rope_neox(q, 10).astype(np.float64) @ O.rope_neox(k, 4).astype(np.float64))
    d2 = float(O.rope_neox(q, 106).astype(np.float64) @ O.rope_neox(k, 100).astype(np.float64))
    assert abs(d1 - d2) < 0.05


def test_qkv_split_layout():
    B, S, H, dh = 2, 3, 2, 8
    qkv = np.arange(B * S * 3 * H * dh, dtype=np.float32).reshape(B * S, 3 * H * dh).astype(np.float16)
    q, k, v = O.qkv_split(qkv, B, S, H, dh, rope=False)
    # element (b, s, which, h, d) of the fused row
    for (b, s, h, d) in [(0, 0, 0, 0), (1, 2, 1, 7), (0, 1, 1, 3)]:
        row = qkv[b * S + s]
        assert q[b, h, s, d] == row[h * dh + d]
        assert k[b, h, s, d] == row[H * dh + h * dh + d]
        assert v[b, h, s, d] == row[2 * H * dh + h * dh + d]


def test_swiglu_and_residual():
    g = np.array([[0.0, 1.0, -1.0, 20.0, -20.0]], np.float16)
    u = np.array([[5.0, 2.0, 2.0, 1.0, 1.0]], np.float16)
    y = O.swiglu(g, u).astype(np.float64)
    want = [0.0, 2 * 1 / (1 + math.exp(-1)), 2 * -1 / (1 + math.exp(1)), 20.0, -20 / (1 + math.exp(20))]
    assert np.allclose(y[0], want, rtol=1e-3, atol=1e-6)
    assert np.array_equal(O.residual_add(np.float16([[1.5]]), np.float16([[2.25]])), np.float16([[3.75]]))


def brute_attention(q, K, V, scale, bias=None, pad=0):
    out = []
    l = (K.astype(np.float64) @ q.astype(np.float64)) * scale
    if bias is not None:
        l = l + bias.astype(np.float64)
    l[:pad] = -np.inf
    e = np.exp(l - l.max())
    p = e / (e.sum() + 1e-6)
    return p @ V.astype(np.float64)


@pytest.mark.parametrize("dh", [32, 128])
def test_decode_attention(dh):
    rng = np.random.default_rng(3)
    B, H, cap, step = 2, 3, 16, 9
    kc = rng.standard_normal((B, H, cap, dh)).astype(np.float16)
    vc = rng.standard_normal((B, H, cap, dh)).astype(np.float16)
    q, k, v = [rng.standard_normal((B, H, dh)).astype(np.float16) for _ in range(3)]
    scale = float(np.float16(1 / math.sqrt(dh)))
    # step = 1: the only weight is 1/(1 + 1e-6)
    k1, v1 = kc.copy(), vc.copy()
    c = O.decode_attention(q, k, v, k1, v1, 1).reshape(B, H, dh)
    assert np.allclose(c.astype(np.float32), v.astype(np.float32) / (1 + 1e-6), atol=1e-3)
    assert np.array_equal(k1[:, :, 0], k) and np.array_equal(v1[:, :, 0], v)
    # uniform keys => mean of the values
    ku = np.broadcast_to(k[:, :, None, :], (B, H, cap, dh)).copy()
    c = O.decode_attention(q, k, v, ku, vc.copy(), step).reshape(B, H, dh)
    vv = vc.copy()
    vv[:, :, step - 1] = v
    assert np.allclose(c.astype(np.float32), vv[:, :, :step].astype(np.float32).mean(2), atol=2e-3)
    # brute force, with padding and an ALiBi row
    bias = O.alibi_bias(H, step)
    pad = np.array([2, 0])
    k2, v2 = kc.copy(), vc.copy()
    c = O.decode_attention(q, k, v, k2, v2, step, pad=pad, alibi=bias).reshape(B, H, dh)
    for b in range(B):
        for h in range(H):
            want = brute_attention(q[b, h], k2[b, h, :step], v2[b, h, :step], scale, bias[h], pad[b])
            assert np.allclose(c[b, h].astype(np.float64), want, atol=2e-3)
    # the padded prefix has exactly zero weight: changing it changes nothing
    k3, v3 = kc.copy(), vc.copy()
    k3[0, :, :2] += 5
    v3[0, :, :2] -= 7
    c3 = O.decode_attention(q, k, v, k3, v3, step, pad=pad, alibi=bias).reshape(B, H, dh)
    assert np.array_equal(c3[0], c[0])
    # softmax shift invariance: adding a constant to the bias row changes nothing (beyond the 1e-6 term)
    c4 = O.decode_attention(q, k, v, kc.copy(), vc.copy(), step, alibi=bias + np.float16(3.0)).reshape(B, H, dh)
    c5 = O.decode_attention(q, k, v, kc.copy(), vc.copy(), step, alibi=bias).reshape(B, H, dh)
    assert np.allclose(c4.astype(np.float32), c5.astype(np.float32), atol=2e-3)


def test_prefill_equals_decode_row_by_row():
    rng = np.random.default_rng(4)
    B, H, S, dh = 2, 2, 6, 32
    q, k, v = [rng.standard_normal((B, H, S, dh)).astype(np.float16) for _ in range(3)]
    pad = np.array([0, 2])
    for bias in (None, O.alibi_mask(H, S)):
        ctx = O.prefill_attention(q, k, v, pad, bias).reshape(B, S, H, dh)
        for i in range(S):
            kc, vc = k.copy(), v.copy()
            row = None if bias is None else bias[:, i, : i + 1]
            c = O.decode_attention(q[:, :, i], k[:, :, i], v[:, :, i], kc, vc, i + 1, pad=pad, alibi=row)
            c = c.reshape(B, H, dh)
            for b in range(B):
                if i < pad[b]:
                    assert not ctx[b, i].any()           # padded query rows are zeroed
                else:
                    assert np.allclose(ctx[b, i].astype(np.float32), c[b].astype(np.float32), atol=2e-3)


def test_alibi_closed_form():
    s8 = O.alibi_slopes(8)
    assert np.allclose(s8, [2.0 ** -(i + 1) for i in range(8)])
    s40 = O.alibi_slopes(40)
    want = [2.0 ** (-0.25 * (i + 1)) for i in range(32)] + [2.0 ** (-0.125 * (2 * i + 1)) for i in range(8)]
    assert np.allclose(s40, want)
    b = O.alibi_bias(40, 2304)
    assert b.dtype == np.float16 and b.shape == (40, 2304)
    assert b[0, 0] == 0 and b[3, 10] == np.float16(np.float32(want[3]) * np.float32(10))
    m = O.alibi_mask(4, 5)
    assert np.isinf(m[0, 1, 2]) and m[2, 3, 1] == b[2 * 0 + 2, 1] * 0 + O.alibi_bias(4, 5)[2, 1]


def test_cpu_path_matches_numpy_oracle():
    import torch
    from oracle import cpu_path
    rng = np.random.default_rng(8)
    x = rng.standard_normal((4, 256)).astype(np.float16)
    q = rng.integers(-128, 128, (256, 48), dtype=np.int8)
    s = (rng.random(48) * 1e-2).astype(np.float16)
    got = cpu_path.dequant_matmul(torch.from_numpy(x), torch.from_numpy(q), torch.from_numpy(s)).numpy()
    want = O.dequant_matmul(x, q, s)
    assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=2e-3, atol=1e-4)


def test_reorder_cache_gather():
    """reorder_cache: element-by-element definition (brute force), a permutation undone by its
    inverse, and a repeated source -- an in-place loop over beams would fail the last two."""
    rng = np.random.default_rng(8)
    B, H, T, dh, rows = 4, 2, 6, 8, 4
    k0 = rng.standard_normal((B, H, T, dh)).astype(np.float16)
    v0 = rng.standard_normal((B, H, T, dh)).astype(np.float16)
    idx = [1, 0, 0, 2]                       # 0 <-> 1 swap (in-place order trap) + a source used twice
    k, v = k0.copy(), v0.copy()
    O.reorder_cache(k, v, idx, rows)
    for b in range(B):
        for h in range(H):
            for t in range(T):
                src = idx[b] if t < rows else b
                assert np.array_equal(k[b, h, t], k0[src, h, t]) and np.array_equal(v[b, h, t], v0[src, h, t])
    perm, inv = [2, 3, 1, 0], [3, 2, 0, 1]
    k, v = k0.copy(), v0.copy()
    O.reorder_cache(k, v, perm, T)
    O.reorder_cache(k, v, inv, T)
    assert np.array_equal(k, k0) and np.array_equal(v, v0)


def test_layernorm_closed_forms():
    """LayerNorm against the float64 textbook form; zero mean and unit variance out with gamma = 1, beta = 0;
    invariance under a shift and a scale of the input; beta passes straight through a constant row."""
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((5, 256)) * 1.7 + 0.8).astype(np.float16)
    g = (1 + 0.1 * rng.standard_normal(256)).astype(np.float16)
    b = (0.2 * rng.standard_normal(256)).astype(np.float16)
    x64 = x.astype(np.float64)
    mu, var = x64.mean(-1, keepdims=True), x64.var(-1, keepdims=True)       # population variance
    want = (x64 - mu) / np.sqrt(var + 1e-5) * g.astype(np.float64) + b.astype(np.float64)
    assert np.abs(O.layernorm(x, g, b, 1e-5).astype(np.float64) - want).max() < 3e-3
    one, zero = np.ones(256, np.float16), np.zeros(256, np.float16)
    y = O.layernorm(x, one, zero, 1e-6).astype(np.float64)
    assert np.abs(y.mean(-1)).max() < 2e-3 and np.allclose((y * y).mean(-1), 1.0, rtol=3e-3)
    y2 = O.layernorm((x.astype(np.float32) * 2 + 3).astype(np.float16), one, zero, 1e-12).astype(np.float32)
    assert np.abs(y2 - O.layernorm(x, one, zero, 1e-12).astype(np.float32)).max() < 6e-3
    const = np.full((2, 256), 4.0, np.float16)       # variance 0: only beta is left
    assert np.array_equal(O.layernorm(const, g, b, 1e-6), np.broadcast_to(b, (2, 256)))
    # a dropped mean (RMSnorm in its place) is seen: the input has mean 0.8
    assert np.abs(O.rmsnorm(x, g, 1e-5).astype(np.float64) + b.astype(np.float64) - want).max() > 0.1


def test_bias_and_post_layernorm_tail():
    rng = np.random.default_rng(4)
    out = rng.standard_normal((3, 64)).astype(np.float16)
    inp = rng.standard_normal((3, 64)).astype(np.float16)
    bias = rng.standard_normal(64).astype(np.float16)
    g = (1 + 0.1 * rng.standard_normal(64)).astype(np.float16)
    b = (0.3 * rng.standard_normal(64)).astype(np.float16)
    # the two adds are fp16 adds, one after the other: brute force, element by element
    yb = np.array([[np.float16(np.float16(out[m, n] + inp[m, n]) + bias[n]) for n in range(64)] for m in range(3)])
    assert np.array_equal(O.add_bias(O.residual_add(out, inp), bias), yb)
    y64 = yb.astype(np.float64)
    want = (y64 - y64.mean(-1, keepdims=True)) / np.sqrt(y64.var(-1, keepdims=True) + 1e-6) * g.astype(np.float64) \
        + b.astype(np.float64)
    assert np.abs(O.add_bias_residual_norm(out, inp, bias, g, b, 1e-6).astype(np.float64) - want).max() < 3e-3
    # without a bias the tail is an RMSnorm of out + inp (beta is not used)
    y = O.residual_add(out, inp).astype(np.float64)
    want = y / np.sqrt((y * y).mean(-1, keepdims=True) + 1e-6) * g.astype(np.float64)
    assert np.abs(O.add_bias_residual_norm(out, inp, None, g, b, 1e-6).astype(np.float64) - want).max() < 3e-3
