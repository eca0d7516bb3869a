"""GPU parity of the fused dequant-GEMM against the fp32 oracle
(dequantise-then-matmul), through the C ABI.  Tolerance: 1e-2 rel / 1e-3 abs."""
import numpy as np
import pytest
import torch

import eet_amd
from oracle import ops as O

from gpu_util import assert_close, gemm

pytestmark = pytest.mark.gpu


def make(M, K, N, seed, mode="ref128"):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(K, N, generator=g) * 0.02).half()
    x = torch.randn(M, K, generator=g).half()
    u, p, s = eet_amd.quant_weights(w, torch.int8, True, mode=mode)
    return x, u, p, s


SMALL = [(1, 64, 16), (1, 256, 64), (3, 128, 48), (8, 1024, 176), (16, 1024, 1024), (17, 512, 48), (32, 576, 80),
         (5, 2752, 512), (9, 4096, 112)]


@pytest.mark.parametrize("M,K,N", SMALL)
def test_small_shapes(gpu, M, K, N):
    x, u, p, s = make(M, K, N, 100 + M + K + N)
    c = gemm(x.to(gpu), p.to(gpu), s.to(gpu), M, N, K)
    assert_close(c.cpu().numpy(), O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32), what=f"{M}x{K}x{N}")


# benchmark configurations 1 and 2: LLaMA-7B decode linears at M in {1, 4, 8, 16, 32}
@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 12288), (4096, 11008), (11008, 4096)])
def test_llama7b_shapes(gpu, K, N):
    x, u, p, s = make(32, K, N, K + N)
    pd, sd = p.to(gpu), s.to(gpu)
    ref32 = O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32)
    for M in (1, 4, 8, 16, 32):
        c = gemm(x[:M].contiguous().to(gpu), pd, sd, M, N, K)
        assert_close(c.cpu().numpy(), ref32[:M], what=f"M={M} K={K} N={N}")


def test_config1_sym127(gpu):
    """benchmark configuration 1 as worded: /127 scales, int8 in [-127, 127], M = 1."""
    x, u, p, s = make(1, 4096, 4096, 1, mode="sym127")
    c = gemm(x.to(gpu), p.to(gpu), s.to(gpu), 1, 4096, 4096)
    assert_close(c.cpu().numpy(), O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32))


def test_special_cases(gpu):
    K = N = 128
    g = torch.Generator().manual_seed(3)
    x = torch.randn(16, K, generator=g).half()
    # q = identity, scale = 1  =>  C == A exactly
    eye = torch.eye(K, dtype=torch.int8)
    c = gemm(x.to(gpu), eet_amd.pack_weights(eye).to(gpu), torch.ones(N).half().to(gpu), 16, N, K)
    assert torch.equal(c.cpu(), x)
    # a single non-zero weight (-128, the value that has no positive twin)
    q = torch.zeros(K, N, dtype=torch.int8)
    q[77, 5] = -128
    c = gemm(x.to(gpu), eet_amd.pack_weights(q).to(gpu), torch.full((N,), 0.5).half().to(gpu), 16, N, K).cpu()
    want = torch.zeros(16, N).half()
    want[:, 5] = (x[:, 77].float() * -64).half()
    assert torch.equal(c, want)
    # extremes of the int8 range everywhere
    q = torch.full((K, N), 127, dtype=torch.int8)
    q[::2] = -128
    s = torch.full((N,), 2.0 ** -7).half()
    c = gemm(x.to(gpu), eet_amd.pack_weights(q).to(gpu), s.to(gpu), 16, N, K)
    assert_close(c.cpu().numpy(), O.dequant_matmul(x.numpy(), q.numpy(), s.numpy(), np.float32))
    # zero-scale column (the all-zero-column case of the quantiser: q = 127, scale = 0) gives exact zeros
    s0 = s.clone()
    s0[9] = 0
    c = gemm(x.to(gpu), eet_amd.pack_weights(q).to(gpu), s0.to(gpu), 16, N, K).cpu()
    assert (c[:, 9] == 0).all()


def test_rows_are_independent(gpu):
    """M = 1 equals row 0 of M = 32 bit for bit (same kernel family, same summation order per row)."""
    x, u, p, s = make(32, 4096, 1024, 9)
    pd, sd = p.to(gpu), s.to(gpu)
    full = gemm(x.to(gpu), pd, sd, 32, 1024, 4096).cpu()
    for M in (1, 7, 16):
        part = gemm(x[:M].contiguous().to(gpu), pd, sd, M, 1024, 4096).cpu()
        assert_close(part.numpy(), full[:M].numpy(), rtol=2e-3, atol=2e-4)


def test_large_m_path(gpu):
    """M > 32 (prefill sizes) takes the other kernel; same oracle."""
    for (M, K, N) in [(33, 256, 64), (100, 512, 192), (129, 256, 48), (256, 1024, 256), (300, 576, 272),
                      (2048, 512, 128), (2048, 5120, 512)]:
        x, u, p, s = make(M, K, N, M + K)
        c = gemm(x.to(gpu), p.to(gpu), s.to(gpu), M, N, K)
        assert_close(c.cpu().numpy(), O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32), what=f"M={M}")


def small_m_shape(M, N, K, epi, rms):
    """(n-tiles per workgroup, wavefronts, k-tiles per batch, k split) the library runs this call with."""
    import ctypes
    from eet_amd._lib import check, lib
    v = [ctypes.c_int(0) for _ in range(4)]
    check(lib().eet_gemm_w8a16_small_m_shape(M, N, K, epi, 1 if rms else 0, *[ctypes.byref(x) for x in v]))
    return tuple(x.value for x in v)


SMALL_M_SHAPES = ["1,8,2", "1,16,2", "1,16,1", "2,8,2", "2,8,1", "3,8,1", "4,8,1", "6,8,1", "8,8,1"]   # NT, wavefronts, k-tiles per batch


@pytest.mark.parametrize("cfg", SMALL_M_SHAPES)
def test_small_m_launch_shapes(gpu, tuning, cfg):
    """Every launch shape the small-M dispatcher can pick (selected with the tuning override), for the
    three row-group counts (M <= 8, <= 16, <= 32), on channel counts that leave the last workgroup
    ragged and k ranges that leave the wavefronts uneven shares: plain, RMSnorm prologue + residual,
    RMSnorm prologue + SwiGLU (an odd NT cannot pair gate / up tiles: the dispatcher's own choice runs)."""
    from eet_amd.ops import interleave_gate_up
    tuning("EET_GEMM_SMALL_M_CONFIG", cfg)
    eps = 1e-6
    want_shape = tuple(int(v) for v in cfg.split(",")) + (1,)
    for (M, K, N) in [(5, 576, 208), (16, 2752, 1104), (27, 704, 400)]:
        # the override really selects the kernel that runs (no silent fall-back to the table's choice) ...
        nt, waves, u = want_shape[:3]
        rg = (M + 7) // 8 if M <= 16 else 4
        # ... where a kernel of that shape can exist: the activation slabs of all wavefronts within 64 KiB,
        # the reduction buffer within 144 KiB (the library's own budget), and an even NT for gate / up pairs
        exists = waves * u * rg * 1024 <= 65536 and waves * nt * ((rg + 1) // 2) * 1024 <= 147456
        assert (small_m_shape(M, N, K, 0, False) == want_shape) == exists, (cfg, M)
        assert (small_m_shape(M, N, K, 1, True) == want_shape) == exists, (cfg, M)
        assert (small_m_shape(M, 2 * (N // 2 + 8), K, 2, True) == want_shape) == (exists and nt % 2 == 0), (cfg, M)
        x, u, p, s = make(M, K, N, M + K + N)
        g = torch.Generator().manual_seed(M)
        gamma = (1 + 0.1 * torch.randn(K, generator=g)).half()
        res = torch.randn(M, N, generator=g).half()
        xd, pd, sd = x.to(gpu), p.to(gpu), s.to(gpu)
        ref = O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32)
        assert_close(gemm(xd, pd, sd, M, N, K).cpu().numpy(), ref, what=f"{cfg} plain M={M}")
        x32 = x.numpy().astype(np.float32)
        xn = x32 / np.sqrt((x32 * x32).mean(-1, keepdims=True) + np.float32(eps)) * gamma.numpy().astype(np.float32)
        deq = u.numpy().astype(np.float32) * s.numpy().astype(np.float32)[None, :]
        got = fused(xd, pd, sd, M, N, K, 1, res.to(gpu), gamma.to(gpu), eps).cpu().numpy()
        assert_close(got, O.residual_add((xn @ deq).astype(np.float16), res.numpy()), rtol=1e-2, atol=3e-3,
                     what=f"{cfg} rms+residual M={M}")
        F = N // 2 + 8
        wg = (torch.randn(K, F, generator=g) * 0.02).half()
        wu = (torch.randn(K, F, generator=g) * 0.02).half()
        ug, pg, sg = eet_amd.quant_weights(wg, torch.int8, True)
        uu, pu, su = eet_amd.quant_weights(wu, torch.int8, True)
        w01, s01 = interleave_gate_up(pg, sg, pu, su)
        got = fused(xd, w01.to(gpu), s01.to(gpu), M, 2 * F, K, 2, None, gamma.to(gpu), eps).cpu().numpy()
        gate = xn @ (ug.numpy().astype(np.float32) * sg.numpy().astype(np.float32)[None, :])
        up = xn @ (uu.numpy().astype(np.float32) * su.numpy().astype(np.float32)[None, :])
        assert_close(got, up * gate / (1 + np.exp(-gate)), rtol=1e-2, atol=3e-3, what=f"{cfg} rms+swiglu M={M}")


# absolute tolerance the RMSnorm-prologue launches may need at 1e-2 relative: 1.5 x what an MI355X run showed
# (in brackets); 1e-3, the north-star's, wherever the observed need is below it
PROLOGUE_BOUNDS = {(1, 256, 64, 0): 1e-3,          # [3.5e-6]
                   (8, 4096, 12288, 0): 1e-3,      # [8.0e-4]
                   (8, 4096, 22016, 2): 3.3e-3,    # [2.16e-3]  SwiGLU: gate and up are rounded to fp16 first
                   (16, 1024, 176, 0): 1e-3,       # [3.0e-4]
                   (32, 512, 96, 2): 1e-3,         # [6.4e-5]
                   (5, 11008, 4096, 1): 2.0e-3}    # [1.30e-3]  K = 11008 behind one moved rounding

@pytest.mark.parametrize("cfg", ["2,8,1,2", "2,8,2,2", "4,8,1,4", "5,8,1,4", "4,4,2,4"])
def test_pair_split(gpu, tuning, cfg):
    """The k split (2 or 4 workgroups share a group of n-tiles, each takes a share of the k range, the one
    that arrives last adds the others' fp32 sums and finishes): forced through the tuning override, at the
    O / down shapes of both decoders and on ragged ones (k-tile and n-tile counts that do not divide), plain
    and with the residual epilogue, twice in a row (the tickets only ever grow)."""
    tuning("EET_GEMM_SMALL_M_CONFIG", cfg)
    for (M, K, N) in [(32, 4096, 4096), (16, 11008, 4096), (8, 5120, 5120), (32, 13696, 5120), (27, 4160, 4112),
                      (3, 192, 48)]:
        assert small_m_shape(M, N, K, 1, False) == tuple(int(v) for v in cfg.split(","))
        x, u, p, s = make(M, K, N, M + K + N)
        res = torch.randn(M, N, generator=torch.Generator().manual_seed(M)).half()
        xd, pd, sd, rd = x.to(gpu), p.to(gpu), s.to(gpu), res.to(gpu)
        ref = O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32)
        print(f"pair split {cfg}: M={M} K={K} N={N}", flush=True)
        for rep in range(2):
            assert_close(gemm(xd, pd, sd, M, N, K).cpu().numpy(), ref, what=f"{cfg} plain M={M} K={K} N={N} rep {rep}")
            got = fused(xd, pd, sd, M, N, K, 1, rd).cpu().numpy()
            assert_close(got, O.residual_add(ref.astype(np.float16), res.numpy()), rtol=1e-2, atol=2e-3,
                         what=f"{cfg} residual M={M} K={K} N={N} rep {rep}")
    # not for the RMSnorm prologue or the SwiGLU epilogue: the table's choice runs
    assert small_m_shape(8, 4096, 4096, 0, True)[3] == 1 and small_m_shape(8, 4096, 4096, 2, False)[3] == 1


@pytest.mark.parametrize("cfg", ["4,8,1,4", "5,8,1,4"])
def test_pair_split_is_reproducible(gpu, tuning, cfg):
    """Four workgroups share a tile's k range and whichever arrives last adds the shares: it adds them in
    the order of the k range, not of arrival, so that repeated launches give the same bits."""
    tuning("EET_GEMM_SMALL_M_CONFIG", cfg)
    M, K, N = 32, 13696, 5120
    x, u, p, s = make(M, K, N, 5)
    xd, pd, sd = x.to(gpu), p.to(gpu), s.to(gpu)
    first = gemm(xd, pd, sd, M, N, K).clone()
    for rep in range(30):
        assert torch.equal(gemm(xd, pd, sd, M, N, K), first), f"launch {rep} differs from the first"


def test_k_split_dispatch(gpu):
    """What the table picks (no override) for a call that hands over the workspace: the k split for the O / down
    launches of both decoders at the batch sizes where it measured faster, the plain launch elsewhere; and the
    launch shapes measured for the decoders' other launches at one and two rows."""
    assert small_m_shape(32, 4096, 4096, 1, False) == (2, 8, 1, 2)       # LLaMA O, M = 32
    assert small_m_shape(16, 4096, 4096, 1, False) == (1, 8, 2, 1)       # ... up to M = 16 a plain launch measured faster
    assert small_m_shape(16, 4096, 11008, 1, False) == (4, 4, 1, 4)      # LLaMA down, M = 16 / 32
    assert small_m_shape(32, 4096, 11008, 1, False) == (4, 8, 1, 4)
    assert small_m_shape(8, 4096, 11008, 1, False)[3] == 1               # M <= 8: not on the LLaMA shapes
    assert small_m_shape(16, 5120, 5120, 1, False) == (5, 8, 1, 4)       # Baichuan O: 320 n-tiles as 64 groups x 4
    assert small_m_shape(8, 5120, 5120, 1, False) == (2, 8, 2, 1)        # ... up to M = 8 a plain launch measured faster
    assert small_m_shape(32, 5120, 5120, 1, False) == (2, 4, 2, 1)       # ... and not at M = 32 with the short k range
    assert small_m_shape(32, 5120, 13696, 1, False) == (5, 8, 1, 4)
    assert small_m_shape(8, 5120, 13696, 1, False) == (5, 8, 1, 4)
    assert small_m_shape(16, 12288, 4096, 0, True)[3] == 1               # never with the RMSnorm prologue
    assert small_m_shape(16, 4112, 4096, 1, False)[3] == 1               # other channel counts keep the table's choice
    assert small_m_shape(1, 12288, 4096, 0, True) == (3, 8, 1, 1)        # RMSnorm + QKV: one workgroup per CU from M = 1 on
    assert small_m_shape(8, 12288, 4096, 0, True) == (3, 8, 1, 1)
    assert small_m_shape(1, 15360, 5120, 0, True) == (2, 8, 2, 1)
    assert small_m_shape(16, 27392, 5120, 2, True) == (8, 8, 1, 1)
    assert small_m_shape(2, 27392, 5120, 2, True) == (4, 8, 1, 1)
    assert small_m_shape(4, 4096, 11008, 1, False) == (1, 16, 1, 1)


LARGE_M_TILES = ["8,4", "4,5", "4,4", "4,2", "2,2"]   # m-tiles, n-tiles per wavefront


@pytest.mark.parametrize("tile", LARGE_M_TILES)
def test_large_m_tiles(gpu, tuning, tile):
    """Every large-M kernel variant (selected with the tuning override), on ragged M / N edges and on
    k-loops of 1..9 tiles (prologue, unrolled body and tail of the software pipeline)."""
    tuning("EET_GEMM_LARGE_M_TILE", tile)
    for (M, K, N) in [(129, 64, 48), (300, 128, 272), (257, 192, 720), (200, 256, 336), (512, 320, 256),
                      (130, 448, 64), (333, 576, 1040)]:
        x, u, p, s = make(M, K, N, M + K + N)
        c = gemm(x.to(gpu), p.to(gpu), s.to(gpu), M, N, K)
        assert_close(c.cpu().numpy(), O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32),
                     what=f"tile {tile} M={M} K={K} N={N}")


@pytest.mark.parametrize("M,K,N,tile", [(1024, 256, 12288, "128x256"), (2048, 256, 5120, "64x320"),
                                        (512, 192, 22016, "64x256"), (512, 256, 8192, "64x128"),
                                        (256, 256, 1024, "32x128"), (100, 320, 12288, "32x128"),
                                        (64, 256, 4096, "slabs")])
def test_large_m_dispatch(gpu, M, K, N, tile):
    """Shapes on which the dispatcher itself picks each tile (named for the record) -- no override."""
    x, u, p, s = make(M, K, N, 77)
    c = gemm(x.to(gpu), p.to(gpu), s.to(gpu), M, N, K)
    assert_close(c.cpu().numpy(), O.dequant_matmul(x.numpy(), u.numpy(), s.numpy(), np.float32), what=tile)


def test_full_size_linearity(gpu):
    """Size-independent property at a benchmark shape: gemm(a + b) == gemm(a) + gemm(b) within fp16 rounding,
    and doubling the scales doubles the output exactly."""
    K, N, M = 4096, 11008, 8
    g = torch.Generator().manual_seed(11)
    q = torch.randint(-128, 128, (K, N), generator=g, dtype=torch.int8)
    p = eet_amd.pack_weights(q).to(gpu)
    s = (torch.rand(N, generator=g) * 1e-3).half()
    # multiples of 1/64 in [-1, 1): a + b is exact in fp16, so only the three output roundings differ
    a = (torch.randint(-64, 64, (M, K), generator=g).float() / 64).half()
    b = (torch.randint(-64, 64, (M, K), generator=g).float() / 64).half()
    ab = (a.float() + b.float()).half()
    ca, cb, cab = [gemm(t.to(gpu), p, s.to(gpu), M, N, K).float().cpu() for t in (a, b, ab)]
    # each of the three outputs carries one fp16 rounding (2^-11 relative to its own magnitude)
    err = (cab - (ca + cb)).abs()
    assert (err <= 1e-3 + 1e-3 * (ca.abs() + cb.abs() + cab.abs())).all(), float(err.max())
    c2 = gemm(a.to(gpu), p, (s * 2).to(gpu), M, N, K).float().cpu()
    # exact, except where the smaller result is an fp16 subnormal (one subnormal step = 2^-24)
    assert ((c2 - ca * 2).abs() <= 2.0 ** -24).all()


def fused(a, wp, s, M, N, K, epi, residual=None, gamma=None, eps=0.0, **kw):
    from gpu_util import gemm_fused
    return gemm_fused(a, wp, s, M, N, K, epi, residual, gamma, eps, **kw)


@pytest.mark.parametrize("M", [1, 8, 13, 32, 70, 300])
def test_residual_epilogue(gpu, M):
    K, N = 1024, 528
    x, u, p, s = make(M, K, N, 40 + M)
    res = torch.randn(M, N, generator=torch.Generator().manual_seed(M)).half()
    xd, pd, sd, rd = x.to(gpu), p.to(gpu), s.to(gpu), res.to(gpu)
    got = fused(xd, pd, sd, M, N, K, 1, rd).cpu()
    plain = gemm(xd, pd, sd, M, N, K).cpu()
    assert torch.equal(got, (plain + res))          # fp16 add of the rounded product, bit for bit
    want = O.residual_add(O.dequant_matmul(x.numpy(), u.numpy(), s.numpy()), res.numpy())
    assert_close(got.numpy(), want, rtol=1e-2, atol=2e-3)


@pytest.mark.parametrize("M,K,F", [(1, 256, 64), (8, 4096, 11008), (16, 512, 208), (32, 512, 704), (100, 256, 96),
                                   (260, 512, 1376)])
def test_swiglu_epilogue(gpu, M, K, F):
    from eet_amd.ops import interleave_gate_up
    g = torch.Generator().manual_seed(F + M)
    x = torch.randn(M, K, generator=g).half()
    wg = (torch.randn(K, F, generator=g) * 0.02).half()
    wu = (torch.randn(K, F, generator=g) * 0.02).half()
    ug, pg, sg = eet_amd.quant_weights(wg, torch.int8, True)
    uu, pu, su = eet_amd.quant_weights(wu, torch.int8, True)
    w01, s01 = interleave_gate_up(pg, sg, pu, su)
    got = fused(x.to(gpu), w01.to(gpu), s01.to(gpu), M, 2 * F, K, 2).cpu().numpy()
    want = O.swiglu(O.dequant_matmul(x.numpy(), ug.numpy(), sg.numpy()),
                    O.dequant_matmul(x.numpy(), uu.numpy(), su.numpy()))
    assert_close(got, want, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("tile", LARGE_M_TILES)
def test_large_m_tile_epilogues(gpu, tuning, tile):
    """Residual and SwiGLU epilogues of every large-M kernel variant (5 n-tiles per wavefront cannot
    pair gate / up tiles: there the override is ignored for SwiGLU and the dispatcher's own choice runs)."""
    from eet_amd.ops import interleave_gate_up
    tuning("EET_GEMM_LARGE_M_TILE", tile)
    M, K, N = 270, 320, 592
    x, u, p, s = make(M, K, N, 5)
    res = torch.randn(M, N, generator=torch.Generator().manual_seed(M)).half()
    xd, pd, sd, rd = x.to(gpu), p.to(gpu), s.to(gpu), res.to(gpu)
    got = fused(xd, pd, sd, M, N, K, 1, rd).cpu()
    assert torch.equal(got, gemm(xd, pd, sd, M, N, K).cpu() + res)
    assert_close(got.numpy(), O.residual_add(O.dequant_matmul(x.numpy(), u.numpy(), s.numpy()), res.numpy()),
                 rtol=1e-2, atol=2e-3)
    F = 336
    g = torch.Generator().manual_seed(F)
    wg = (torch.randn(K, F, generator=g) * 0.02).half()
    wu = (torch.randn(K, F, generator=g) * 0.02).half()
    ug, pg, sg = eet_amd.quant_weights(wg, torch.int8, True)
    uu, pu, su = eet_amd.quant_weights(wu, torch.int8, True)
    w01, s01 = interleave_gate_up(pg, sg, pu, su)
    got = fused(xd, w01.to(gpu), s01.to(gpu), M, 2 * F, K, 2).cpu().numpy()
    want = O.swiglu(O.dequant_matmul(x.numpy(), ug.numpy(), sg.numpy()),
                    O.dequant_matmul(x.numpy(), uu.numpy(), su.numpy()))
    assert_close(got, want, rtol=1e-2, atol=1e-3)


SPLIT_K = ["2,2,2", "2,2,3", "2,2,8", "4,2,4", "4,4,2", "8,4,5"]   # m-tiles, n-tiles, parts of the k range


@pytest.mark.parametrize("cfg", SPLIT_K)
@pytest.mark.parametrize("M,K,N", [(70, 1216, 400), (33, 4096, 1024), (161, 640, 528)])
def test_split_k(gpu, tuning, cfg, M, K, N):
    """Every tile with its k range shared by several workgroups (uneven shares, ragged rows and channels,
    one k-tile per part at K = 640 with 8 parts) + the second kernel that adds the fp32 parts, for all three
    epilogues, against the fp32 oracle; without the workspace the same call runs in a single pass."""
    from eet_amd.ops import interleave_gate_up
    tuning("EET_GEMM_LARGE_M_TILE", cfg)
    ws = 8 * M * max(N, 1024) * 4
    x, u, p, s = make(M, K, N, 11)
    res = torch.randn(M, N, generator=torch.Generator().manual_seed(M)).half()
    xd, pd, sd, rd = x.to(gpu), p.to(gpu), s.to(gpu), res.to(gpu)
    ref = O.dequant_matmul(x.numpy(), u.numpy(), s.numpy())
    got = gemm(xd, pd, sd, M, N, K, ws_min_bytes=ws).cpu()
    assert_close(got.numpy(), ref, rtol=1e-2, atol=1e-3)
    got_r = fused(xd, pd, sd, M, N, K, 1, rd, ws_min_bytes=ws).cpu()
    assert torch.equal(got_r, got + res)
    single = fused(xd, pd, sd, M, N, K, 0, use_ws=False).cpu()     # no workspace: one pass, same tile
    assert_close(single.numpy(), ref, rtol=1e-2, atol=1e-3)
    F = 272
    g = torch.Generator().manual_seed(F)
    wg = (torch.randn(K, F, generator=g) * 0.02).half()
    wu = (torch.randn(K, F, generator=g) * 0.02).half()
    ug, pg, sg = eet_amd.quant_weights(wg, torch.int8, True)
    uu, pu, su = eet_amd.quant_weights(wu, torch.int8, True)
    w01, s01 = interleave_gate_up(pg, sg, pu, su)
    got = fused(xd, w01.to(gpu), s01.to(gpu), M, 2 * F, K, 2, ws_min_bytes=ws).cpu().numpy()
    want = O.swiglu(O.dequant_matmul(x.numpy(), ug.numpy(), sg.numpy()),
                    O.dequant_matmul(x.numpy(), uu.numpy(), su.numpy()))
    assert_close(got, want, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("M,K,N", [(40, 4096, 4096), (64, 11008, 4096), (96, 4096, 4096), (256, 11008, 4096),
                                   (48, 4096, 12288)])
def test_split_k_dispatch(gpu, M, K, N):
    """Shapes for which the library asks for a split-k workspace: the result with it (MFMA tiles, k range
    split) and without it (32-row slabs of the small-M kernel / single-pass tiles) both match the oracle."""
    from eet_amd._lib import lib
    assert lib().eet_gemm_w8a16_workspace(M, N, K, 0) > 0
    x, u, p, s = make(M, K, N, 13)
    xd, pd, sd = x.to(gpu), p.to(gpu), s.to(gpu)
    ref = O.dequant_matmul(x.numpy(), u.numpy(), s.numpy())
    assert_close(fused(xd, pd, sd, M, N, K, 0).cpu().numpy(), ref, rtol=1e-2, atol=1e-3)
    assert_close(fused(xd, pd, sd, M, N, K, 0, use_ws=False).cpu().numpy(), ref, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("M,K,N,epi", [(1, 256, 64, 0), (8, 4096, 12288, 0), (8, 4096, 22016, 2), (16, 1024, 176, 0),
                                       (32, 512, 96, 2), (5, 11008, 4096, 1)])
def test_rmsnorm_prologue(gpu, M, K, N, epi):
    """RMSnorm folded into the GEMM against the fp32 composition rmsnorm -> GEMM (-> epilogue).

    The fused kernel rounds x * gamma to fp16 and applies 1/rms to the fp32 sum; the unfused path
    rounds x * gamma / rms to fp16.  Both carry one fp16 rounding per activation, at different
    places, so the comparison is against the composition with NO intermediate rounding; the error is
    printed and held to 1.5 x the need measured on an MI355X (PROLOGUE_BOUNDS; relative stays 1e-2)."""
    from eet_amd.ops import interleave_gate_up
    g = torch.Generator().manual_seed(M + K + N)
    x = (torch.randn(M, K, generator=g) * 1.7).half()
    gamma = (1 + 0.1 * torch.randn(K, generator=g)).half()
    eps = 1e-6
    x32 = x.numpy().astype(np.float32)
    xn = x32 / np.sqrt((x32 * x32).mean(-1, keepdims=True) + eps) * gamma.numpy().astype(np.float32)

    def mm(u, s):
        return xn @ (u.numpy().astype(np.float32) * s.numpy().astype(np.float32)[None, :])
    if epi == 2:
        F = N // 2
        ug, pg, sg = eet_amd.quant_weights((torch.randn(K, F, generator=g) * 0.02).half(), torch.int8, True)
        uu, pu, su = eet_amd.quant_weights((torch.randn(K, F, generator=g) * 0.02).half(), torch.int8, True)
        p, s = interleave_gate_up(pg, sg, pu, su)
        gate, up = mm(ug, sg), mm(uu, su)
        want = up * gate / (1 + np.exp(-gate))
        res = None
    else:
        u, p, s = eet_amd.quant_weights((torch.randn(K, N, generator=g) * 0.02).half(), torch.int8, True)
        want = mm(u, s)
        res = torch.randn(M, N, generator=g).half() if epi == 1 else None
        if epi == 1:
            want = want + res.numpy().astype(np.float32)
    rd = res.to(gpu) if res is not None else None
    got = fused(x.to(gpu), p.to(gpu), s.to(gpu), M, N, K, epi, rd, gamma.to(gpu), eps).cpu().numpy()
    # the SwiGLU epilogue adds the fp16 roundings of gate and up (as the separate kernels have them)
    from gpu_util import measured
    atol = PROLOGUE_BOUNDS[(M, K, N, epi)]
    measured(got, want, f"rmsnorm prologue M={M} K={K} N={N} epi={epi}", atol)
    # and the unfused path (eet_rmsnorm then the GEMM) agrees with the same reference
    from eet_amd._lib import check, lib
    from gpu_util import stream
    xd, gd = x.to(gpu), gamma.to(gpu)
    xnd = torch.empty_like(xd)
    check(lib().eet_rmsnorm(xd.data_ptr(), gd.data_ptr(), xnd.data_ptr(), M, K, eps, stream()))
    got2 = fused(xnd, p.to(gpu), s.to(gpu), M, N, K, epi, rd).cpu().numpy()
    # (this path rounds x * gamma / rms to fp16 before the GEMM: one rounding more than the reference form)
    assert_close(got2, want, rtol=1e-2, atol=3e-3 if epi == 2 else 2e-3)
