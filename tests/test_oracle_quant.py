"""Pins the quantiser three ways: the known answers recorded from the reference
(tests/golden), closed forms / invariants / brute force, and agreement of the
three implementations (numpy oracle, plain-C oracle, the shipped host packer)."""
import ctypes
import json
import os

import math

import numpy as np
import pytest
import torch

from oracle import quant as Q

import eet_amd

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = json.load(open(os.path.join(HERE, "golden", "quant_known_answers.json")))


def c_quantize(lib, w32):
    K, N = w32.shape
    w32 = np.ascontiguousarray(w32, dtype=np.float32)
    q = np.empty((K, N), np.int8)
    s = np.empty(N, np.float32)
    assert lib.oracle_quantize_ref128(w32.ctypes.data, K, N, q.ctypes.data, s.ctypes.data) == 0
    return q, s


def product_quantize(w):
    """The shipped host quantiser (eet_quantize_int8) alone, without the packing step."""
    from eet_amd.ops import _quantize
    u, s = _quantize(torch.from_numpy(np.ascontiguousarray(w)), 0)
    return u.numpy(), None, s.numpy()


def golden_matrix(case, dtype=np.float32):
    K = case["K"]
    w = np.full((K, 64), 0.25, dtype)      # other columns: arbitrary, independent
    col = np.full(K, case["column"]["fill"], dtype)
    for k, v in case["column"]["set"].items():
        col[int(k)] = v
    w[:, 5] = col
    return w


@pytest.mark.parametrize("case", GOLD["quantize"], ids=lambda c: c["name"])
def test_known_answers(case, oracle_c):
    w = golden_matrix(case)
    for name, (q, s) in {
        "numpy": Q.quantize_ref128(w),
        "c": c_quantize(oracle_c, w),
        "product": product_quantize(w)[::2],
    }.items():
        assert float(s[5]) == case["scale"], name
        if "q_all" in case:
            assert (q[:, 5] == case["q_all"]).all(), name
        for k, v in case.get("q", {}).items():
            assert int(q[int(k), 5]) == v, (name, k)


def brute_force(w):
    """Scalar loops, one numpy float32 operation at a time."""
    K, N = w.shape
    q = np.zeros((K, N), np.int8)
    s = np.zeros(N, np.float32)
    for n in range(N):
        amax = np.float32(0)
        for k in range(K):
            amax = max(amax, abs(np.float32(w[k, n])))
        s[n] = np.float32(amax * np.float32(0.0078125))
        for k in range(K):
            with np.errstate(all="ignore"):
                x = np.float32(w[k, n]) / s[n]
            if np.isnan(x):
                v = 127
            else:
                x = float(x)       # exact widening
                r = int(abs(x) + 0.5) * (1 if x >= 0 else -1) if abs(x) < 1e9 else (1e9 if x > 0 else -1e9)
                v = max(-128, min(127, r))
            q[k, n] = v
    return q, s


def test_brute_force_small():
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((4, 8)) * 0.02).astype(np.float32)
    w[:, 3] = 0
    w[1, 4] = w[:, 4].max() * 0 + 0.5
    q, s = Q.quantize_ref128(w)
    qb, sb = brute_force(w)
    assert np.array_equal(q, qb) and np.array_equal(s, sb)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("shape", [(64, 64), (128, 192), (256, 48), (1, 16), (4096, 64)])
def test_three_implementations_agree(dtype, shape, oracle_c):
    rng = np.random.default_rng(shape[0] * 31 + shape[1] + (dtype == np.float16))
    w = (rng.standard_normal(shape) * 0.02).astype(dtype)
    if shape[1] > 8:
        w[:, 1] = 0                                        # zero column
        w[:, 2] = np.linspace(-1, 1, shape[0]).astype(dtype)  # exact ties at +-absmax
        w[:, 3] = (rng.standard_normal(shape[0]) * 1e-7).astype(dtype)  # tiny / subnormal in fp16
        w[0, 4] = 60000 if dtype == np.float16 else 3e38     # huge
    q, s = Q.quantize_ref128(w)
    qc, sc32 = c_quantize(oracle_c, w.astype(np.float32))
    with np.errstate(over="ignore"):
        sc = sc32.astype(dtype)
    u, _, sp = product_quantize(w)
    assert np.array_equal(q, qc) and np.array_equal(s, sc)
    assert np.array_equal(q, u) and np.array_equal(s.view(np.uint8), sp.view(np.uint8))


def test_invariants():
    rng = np.random.default_rng(7)
    w = (rng.standard_normal((512, 96)) * 0.02).astype(np.float16)
    q, s = Q.quantize_ref128(w)
    w32 = w.astype(np.float32)
    amax = np.abs(w32).max(0)
    # closed form of the scale: fp16_rn(absmax * 2^-7) -- a power-of-two scaling, exact before rounding
    assert np.array_equal(s, (amax / 128).astype(np.float16))
    # the extreme element of every column maps to +127 (128 clamped) or -128
    k = np.abs(w32).argmax(0)
    ext = q[k, np.arange(96)].astype(int)
    sign = np.sign(w32[k, np.arange(96)])
    assert ((ext == 127) & (sign > 0) | (ext == -128) & (sign < 0)).all()
    # dequantised error is at most half a step
    err = np.abs(q.astype(np.float32) * (amax / 128)[None] - w32)
    assert (err <= (amax / 128)[None] * 0.5 * 1.0001 + (q == 127) * (amax / 128)[None]).all()
    # a dropped half-away rule would show up here: 2.5 -> 3, -2.5 -> -3, 0.5 -> 1, -0.5 -> -1
    col = np.zeros((8, 16), np.float32)
    col[:, 0] = [128, 2.5, -2.5, 0.5, -0.5, 1.5, -1.5, 0.49999997]
    qq, _ = Q.quantize_ref128(col)
    assert qq[:, 0].tolist() == [127, 3, -3, 1, -1, 2, -2, 0]


def test_sym127_scalar_brute_force():
    """quantize_sym127 against a scalar loop in C-float arithmetic (numpy float32 scalars):
    scale = absmax / 127, q = round-half-away(w / scale) in [-127, 127], zero column -> 0."""
    rng = np.random.default_rng(4)
    w = (rng.standard_normal((24, 6)) * 0.02).astype(np.float32)
    w[:, 1] = 0
    w[3, 2], w[4, 2], w[5, 2] = 127.0, 2.5, -0.5           # scale exactly 1: ties visible
    w[:3, 2] = [1.5, -1.5, 126.5]
    q, s = Q.quantize_sym127(w)
    for n in range(w.shape[1]):
        amax = np.float32(0)
        for k in range(w.shape[0]):
            amax = max(amax, np.float32(abs(w[k, n])))
        sc = np.float32(amax / np.float32(127.0))
        assert s[n] == sc
        for k in range(w.shape[0]):
            if sc == 0:
                want = 0
            else:
                r = float(np.float32(w[k, n] / sc))
                want = int(math.copysign(math.floor(abs(r) + 0.5), r))     # exact in float64
                want = max(-127, min(127, want))
            assert q[k, n] == want, (k, n)
    assert q[3, 2] == 127 and q[4, 2] == 3 and q[5, 2] == -1 and q[0, 2] == 2 and q[1, 2] == -2 and q[2, 2] == 127
    # the extreme element of a non-zero column is exactly +-127
    k = np.abs(w).argmax(0)
    assert (np.abs(q[k, np.arange(6)].astype(int))[[0, 2, 3, 4, 5]] == 127).all()


def test_sym127_generator():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((128, 32)) * 0.02).astype(np.float16)
    w[:, 0] = 0
    q, s = Q.quantize_sym127(w)
    u, p, sp = eet_amd.quant_weights(torch.from_numpy(w), torch.int8, True, mode="sym127")
    assert np.array_equal(q, u.numpy()) and np.array_equal(s, sp.numpy())
    assert np.abs(q).max() == 127 and (q[:, 0] == 0).all() and s[0] == 0


# ---------------------------------------------------------------------------
# layouts
# ---------------------------------------------------------------------------
def test_processed_sm80_known_order():
    g = GOLD["processed_sm80"]
    K = N = 64
    q = ((np.arange(K)[:, None] * 3 + np.arange(N)[None, :] * 7) % 251 - 125).astype(np.int8)
    proc = Q.preprocess_ref_sm80(q)
    for n in (0, 1, 17, 63):
        col = proc[64 * n: 64 * n + 64].astype(int) - 128
        for pos, k in enumerate(g["k_order_first_32"]):
            assert col[pos] == q[k, n]
        assert sorted(col.tolist()) == sorted(q[:, n].astype(int).tolist())


def test_processed_sm80_larger_k_order():
    # [column pair][64-row K tile][column in pair][64 rows]
    K, N = 192, 128
    idx = Q.preprocess_ref_sm80_index(K, N)
    k, n = idx // N, idx % N
    p = np.arange(K * N)
    assert np.array_equal(n // 2, p // (2 * K))
    assert np.array_equal(k // 64, (p % (2 * K)) // 128)
    assert np.array_equal(n % 2, (p % 128) // 64)
    assert sorted(idx.tolist()) == list(range(K * N))


@pytest.mark.parametrize("shape", [(64, 64), (128, 192), (256, 64)])
def test_processed_sm80_product_matches_oracle(shape):
    from eet_amd._lib import lib
    K, N = shape
    rng = np.random.default_rng(1)
    q = rng.integers(-128, 128, shape, dtype=np.int8)
    want = Q.preprocess_ref_sm80(q)
    got = np.empty(K * N, np.int8)
    back = np.empty((K, N), np.int8)
    assert lib().eet_preprocess_ref_sm80(q.ctypes.data, K, N, got.ctypes.data) == 0
    assert np.array_equal(got.view(np.uint8), want)
    assert lib().eet_unprocess_ref_sm80(got.ctypes.data, K, N, back.ctypes.data) == 0
    assert np.array_equal(back, q)
    assert np.array_equal(Q.unprocess_ref_sm80(want, K, N), q)


def gfx950_reference_pack(q):
    """The gfx950 layout from its definition, element by element."""
    K, N = q.shape
    out = np.empty(K * N, np.uint8)
    kt_n = K // 64
    for nt in range(N // 16):
        for kt in range(kt_n):
            base = (nt * kt_n + kt) * 1024
            for lane in range(64):
                g, i = lane // 16, lane % 16
                for b in range(16):
                    out[base + lane * 16 + b] = np.uint8(q[kt * 64 + g * 16 + b, nt * 16 + i]) ^ 0x80
    return out


def test_gfx950_layout_definition():
    rng = np.random.default_rng(2)
    q = rng.integers(-128, 128, (128, 48), dtype=np.int8)
    p = eet_amd.pack_weights(torch.from_numpy(q)).numpy()
    assert np.array_equal(p.reshape(-1).view(np.uint8), gfx950_reference_pack(q))


@pytest.mark.parametrize("shape", [(64, 16), (4096, 4096), (4096, 12288), (4096, 11008), (11008, 4096),
                                   (5120, 15360), (5120, 13696), (13696, 5120), (192, 80)])
def test_gfx950_roundtrip(shape):
    rng = np.random.default_rng(5)
    q = torch.from_numpy(rng.integers(-128, 128, shape, dtype=np.int8))
    p = eet_amd.pack_weights(q)
    assert p.shape == q.shape
    assert torch.equal(eet_amd.unpack_weights(p), q)
    # a pure permutation of the biased bytes
    assert np.array_equal(np.bincount(p.numpy().reshape(-1).view(np.uint8), minlength=256),
                          np.bincount((q.numpy().reshape(-1).view(np.uint8) ^ 0x80), minlength=256))


def test_pack_rejects_ragged_shapes():
    with pytest.raises(RuntimeError, match="K % 64"):
        eet_amd.pack_weights(torch.zeros(100, 16, dtype=torch.int8))
    with pytest.raises(RuntimeError, match="N % 16"):
        eet_amd.pack_weights(torch.zeros(64, 24, dtype=torch.int8))


def test_torch_packer_and_quantiser_match_the_library():
    rng = np.random.default_rng(9)
    q = torch.from_numpy(rng.integers(-128, 128, (256, 96), dtype=np.int8))
    assert torch.equal(eet_amd.pack_weights_torch(q), eet_amd.pack_weights(q))
    w = torch.from_numpy((rng.standard_normal((512, 64)) * 0.02).astype(np.float16))
    w[:, 3] = 0
    # a column whose scale is exactly 1 (ref128) with exact ties and the value just below one half,
    # where floor(|x| + 0.5) would round up and C round() does not
    w32 = w.float()
    w32[:, 5] = 0
    w32[:8, 5] = torch.tensor([128.0, 2.5, -2.5, 0.5, -0.5, 0.49999997, -0.49999997, 127.5])
    for mode in ("ref128", "sym127"):
        for mat in (w, w32):
            u, p, s = eet_amd.quant_weights(mat, torch.int8, True, mode=mode)
            ut, st = eet_amd.quant_weights_torch(mat, mode)
            assert torch.equal(ut, u) and torch.equal(st, s)
