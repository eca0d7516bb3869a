"""CPU oracle: per-output-channel symmetric int8 quantiser and the reference's
NVIDIA-specific "processed" layout.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).
"""
import numpy as np


def _round_half_away(x):
    """C round(): nearest integer, halves away from zero, NaN stays NaN.

    x - trunc(x) is exact in binary floating point, so this has no
    double-rounding error (floor(x + 0.5) does, e.g. for 0.49999997f).
    """
    t = np.trunc(x)
    frac = np.abs(x - t)
    return t + np.where(frac >= 0.5, np.sign(x), 0).astype(x.dtype)


def quantize_ref128(w):
    """Reference quantiser, int8 branch.

    Follows 3rdparty/cutlass_kernels/cutlass_preprocessors.cc:581-678:
      * quant_range_scale = 1 / (1 << 7)                                (:610)
      * per_col_max = max_k |float(w[k, n])|                            (:619-628)
      * per_col_max *= quant_range_scale (fp32); scale = ComputeType(.) (:632-635)
      * q = int8(max(-128, min(127, round(float(w) / per_col_max))))    (:643-648)
    The division uses the fp32 scale, not the stored (fp16-rounded) one.
    std::min(127.f, NaN) returns 127.f, so an all-zero column (0/0) gives 127.

    w: [K, N] float16 or float32.  Returns (q int8 [K, N], scale [N] of w's dtype).
    """
    w = np.asarray(w)
    assert w.ndim == 2 and w.dtype in (np.float16, np.float32)
    w32 = w.astype(np.float32)
    absmax = np.max(np.abs(w32), axis=0) if w.shape[0] else np.zeros(w.shape[1], np.float32)
    s32 = (absmax * np.float32(1.0 / 128.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        r = _round_half_away((w32 / s32[None, :]).astype(np.float32))
    r = np.where(np.isnan(r), np.float32(127.0), np.minimum(np.float32(127.0), r))
    r = np.maximum(np.float32(-128.0), r)
    with np.errstate(over="ignore"):
        scale = s32.astype(w.dtype)
    return r.astype(np.int8), scale


def quantize_sym127(w):
    """The synthetic benchmark's generator ("scales = max|W_col|/127, int8 in
    [-127, 127]").  Not a reference function: the reference only has the /128
    rule above.  Zero columns give q = 0, scale = 0.
    """
    w = np.asarray(w)
    w32 = w.astype(np.float32)
    absmax = np.max(np.abs(w32), axis=0)
    s32 = (absmax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        r = _round_half_away((w32 / s32[None, :]).astype(np.float32))
    r = np.where(np.isnan(r), np.float32(0.0), r)
    r = np.clip(r, -127.0, 127.0)
    return r.astype(np.int8), s32.astype(w.dtype)


# --------------------------------------------------------------------------
# The reference's processed layout for sm75/sm80 (ColumnMajorTileInterleave<64,2>).
# Never consumed on gfx950; restated so that weights saved by the reference can
# be un-processed, and as an independent check of the index maps.
# --------------------------------------------------------------------------

def _permute_rows(q):
    """cutlass_preprocessors.cc:137-195.  Within each 16-row group, output row
    r takes input row 8*((r%4)/2) + r%2 + 2*(r/4)  (:182-183, int8: ELTS_PER_REG=4)."""
    K, N = q.shape
    assert K % 16 == 0 and N % 8 == 0
    r = np.arange(16)
    src = 8 * ((r % 4) // 2) + r % 2 + 2 * (r // 4)
    rows = (np.arange(0, K, 16)[:, None] + src[None, :]).reshape(-1)
    return q[rows, :]


def _interleave_columns(qt):
    """cutlass_preprocessors.cc:432-495 on the transposed [N, K] matrix viewed as
    uint32 words of 4 consecutive k: 64-row (16-word) tiles of two adjacent
    columns are interleaved (:474-493)."""
    N, K = qt.shape
    assert K % 4 == 0 and N % 64 == 0  # the reference checks num_cols % rows_per_tile (:450-458)
    words = qt.reshape(N, K // 4, 4)
    nvr = K // 4
    out = np.empty((N // 2, nvr * 2, 4), dtype=qt.dtype)
    vr = np.arange(nvr)
    base = (vr // 16) * 16
    for c in range(N):
        wr = 2 * base + 16 * (c % 2) + vr % 16
        out[c // 2, wr, :] = words[c, vr, :]
    return out.reshape(N // 2 * nvr * 2 * 4)


def preprocess_ref_sm80(q):
    """preprocess_weights_for_mixed_gemm for arch 75..89, int8
    (cutlass_preprocessors.cc:497-534): row permute -> transpose -> column
    interleave -> +128 and swap bytes 1<->2 of every 4 (:337-358).
    Returns a flat uint8 array of K*N bytes."""
    q = np.asarray(q, dtype=np.int8)
    K, N = q.shape
    p = _permute_rows(q)
    t = np.ascontiguousarray(p.T)
    flat = _interleave_columns(t).astype(np.int16) + 128
    flat = flat.astype(np.uint8).reshape(-1, 4)
    flat = flat[:, [0, 2, 1, 3]]
    return flat.reshape(-1)


def unprocess_ref_sm80(buf, K, N):
    """Inverse of preprocess_ref_sm80 (ours; used to read reference-saved weights)."""
    idx = preprocess_ref_sm80_index(K, N)
    out = np.empty(K * N, dtype=np.int8)
    out[idx] = (np.asarray(buf, dtype=np.uint8).astype(np.int16) - 128).astype(np.int8)
    return out.reshape(K, N)


def preprocess_ref_sm80_index(K, N):
    """For every byte of the processed buffer, the flat [K, N] index it holds."""
    ids = np.arange(K * N, dtype=np.int64).reshape(K, N)
    r = np.arange(16)
    src = 8 * ((r % 4) // 2) + r % 2 + 2 * (r // 4)
    rows = (np.arange(0, K, 16)[:, None] + src[None, :]).reshape(-1)
    t = np.ascontiguousarray(ids[rows, :].T)
    flat = _interleave_columns(t).reshape(-1, 4)[:, [0, 2, 1, 3]]
    return flat.reshape(-1)
