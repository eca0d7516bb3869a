"""Helpers shared by the GPU parity tests: calls go through the C ABI."""
import numpy as np
import torch

from eet_amd._lib import check, lib

# north-star tolerance against the fp32 oracle: 1e-2 relative / 1e-3 absolute
RTOL, ATOL = 1e-2, 1e-3


def stream():
    return torch.cuda.current_stream().cuda_stream


def assert_close(got, want, rtol=RTOL, atol=ATOL, what=""):
    got = np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = np.abs(got - want)
    tol = atol + rtol * np.abs(want)
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} outside tolerance, max err {err.max():.5f}"


def measured(got, want, what, bound=None, rtol=RTOL):
    """Error of one fused launch, printed and -- with `bound` -- asserted: `excess` is the largest
    err - rtol * |want| over the elements, i.e. the absolute tolerance the launch needs at the
    north-star's relative tolerance.  `bound` is 1.5 x the excess observed on an MI355X (at least the
    north-star's 1e-3 is always allowed); returns (max_abs_err, excess)."""
    got = np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = np.abs(got - want)
    excess = float((err - rtol * np.abs(want)).max())
    print(f"ERR {what}: max_abs_err {err.max():.3e} needs atol {max(excess, 0.0):.3e} at rtol {rtol:g}"
          + (f" (bound {bound:.1e})" if bound is not None else ""), flush=True)
    if bound is not None:
        assert excess <= bound, f"{what}: needs atol {excess:.3e} at rtol {rtol:g}, bound {bound:.1e}"
    return float(err.max()), excess


def gemm_workspace(M, N, K, epi, device, min_bytes=0):
    """(pointer, bytes) of the optional split-k workspace the library asks for
    (None, 0 when it asks for none); min_bytes forces a larger one for tests
    that override the split."""
    need = max(lib().eet_gemm_w8a16_workspace(M, N, K, epi), min_bytes)
    if not need:
        return None, 0, None
    # zero-filled: the small-M k split keeps its arrival counters at the start of the workspace
    buf = torch.zeros((need + 3) // 4, dtype=torch.float32, device=device)
    return buf.data_ptr(), need, buf


def gemm(a, wp, s, M, N, K, ws_min_bytes=0):
    c = torch.empty(M, N, dtype=torch.float16, device=a.device)
    ws, ws_bytes, keep = gemm_workspace(M, N, K, 0, a.device, ws_min_bytes)
    check(lib().eet_gemm_w8a16(a.data_ptr(), wp.data_ptr(), s.data_ptr(), c.data_ptr(), M, N, K, ws, ws_bytes,
                               stream()), "eet_gemm_w8a16")
    return c


def gemm_fused(a, wp, s, M, N, K, epi, residual=None, gamma=None, eps=0.0, ws_min_bytes=0, use_ws=True):
    n_out = N // 2 if epi == 2 else N
    c = torch.empty(M, n_out, dtype=torch.float16, device=a.device)
    ws, ws_bytes, keep = gemm_workspace(M, N, K, epi, a.device, ws_min_bytes) if use_ws else (None, 0, None)
    check(lib().eet_gemm_w8a16_fused(a.data_ptr(), wp.data_ptr(), s.data_ptr(), c.data_ptr(), M, N, K, epi,
                                     residual.data_ptr() if residual is not None else None,
                                     gamma.data_ptr() if gamma is not None else None, eps, ws, ws_bytes, stream()),
          "eet_gemm_w8a16_fused")
    return c


def mmha(q, k, v, kc, vc, step, pad=None, alibi=None, stride=0, rope_row=None):
    B, H, T, dh = kc.shape
    ctx = torch.empty(B, H * dh, dtype=torch.float16, device=kc.device)
    L = lib()
    need = L.eet_mmha_decode_workspace(B, H, dh, step)
    ws = torch.empty(max(need // 4, 1), dtype=torch.float32, device=kc.device)
    check(L.eet_mmha_decode(q.data_ptr(), k.data_ptr() if k is not None else None,
                            v.data_ptr() if v is not None else None, stride, kc.data_ptr(), vc.data_ptr(),
                            ctx.data_ptr(), alibi.data_ptr() if alibi is not None else None,
                            pad.data_ptr() if pad is not None else None, B, H, dh, step, T,
                            rope_row.data_ptr() if rope_row is not None else None, ws.data_ptr(),
                            ws.numel() * 4, stream()), "eet_mmha_decode")
    return ctx
