"""GPU parity of the glue kernels and the prompt attention against the oracle."""
import numpy as np
import pytest
import torch

from eet_amd._lib import check, lib
from oracle import ops as O

from gpu_util import assert_close, stream

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N", [(1, 64), (8, 4096), (3, 5120), (2, 16384), (5, 1000)])
def test_rmsnorm(gpu, M, N):
    g = torch.Generator().manual_seed(N)
    x = torch.randn(M, N, generator=g).half()
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).half()
    out = torch.empty(M, N, dtype=torch.float16, device=gpu)
    xd, gd = x.to(gpu), gamma.to(gpu)
    check(lib().eet_rmsnorm(xd.data_ptr(), gd.data_ptr(), out.data_ptr(), M, N, 1e-6, stream()))
    assert_close(out.cpu().numpy(), O.rmsnorm(x.numpy(), gamma.numpy(), 1e-6), rtol=2e-3, atol=1e-3)


@pytest.mark.parametrize("B,S,H,dh,rope,ts,t0", [(2, 5, 4, 128, 1, -1, 0), (3, 1, 4, 128, 1, 1030, 1030),
                                                   (2, 7, 5, 64, 0, -1, 0), (1, 1, 2, 32, 1, 17, 17),
                                                   (2, 1, 40, 128, 0, 9, 9), (2, 6, 3, 96, 1, -1, 0)])
def test_qkv_split(gpu, B, S, H, dh, rope, ts, t0):
    g = torch.Generator().manual_seed(B + S + H)
    cap = t0 + S + 3
    qkv = torch.randn(B * S, 3 * H * dh, generator=g).half()
    kc = torch.randn(B, H, cap, dh, generator=g).half()
    vc = torch.randn(B, H, cap, dh, generator=g).half()
    q_ref, k_ref, v_ref = O.qkv_split(qkv.numpy(), B, S, H, dh, bool(rope), ts)
    kcn, vcn = kc.numpy().copy(), vc.numpy().copy()
    kcn[:, :, t0:t0 + S] = k_ref
    vcn[:, :, t0:t0 + S] = v_ref
    qd = torch.empty(B, H, S, dh, dtype=torch.float16, device=gpu)
    kcd, vcd = kc.to(gpu), vc.to(gpu)
    qkvd = qkv.to(gpu)
    check(lib().eet_qkv_split(qkvd.data_ptr(), qd.data_ptr(), kcd.data_ptr(), vcd.data_ptr(), B, S, H, dh,
                              rope, ts, t0, cap, stream()))
    # rotation angles reach ~1000 rad in fp32: allow a few fp16 ulps on O(1..4) values
    assert_close(qd.cpu().numpy(), q_ref, rtol=4e-3, atol=4e-3)
    assert_close(kcd.cpu().numpy(), kcn, rtol=4e-3, atol=4e-3)
    assert np.array_equal(vcd.cpu().numpy(), vcn)          # v is a pure copy
    if not rope:
        assert np.array_equal(qd.cpu().numpy(), q_ref) and np.array_equal(kcd.cpu().numpy(), kcn)


def test_swiglu_and_residual(gpu):
    g = torch.Generator().manual_seed(1)
    M, N = 8, 11008
    gate = (torch.randn(M, N, generator=g) * 3).half()
    up = torch.randn(M, N, generator=g).half()
    gd, ud = gate.to(gpu), up.to(gpu)
    check(lib().eet_swiglu(gd.data_ptr(), ud.data_ptr(), M, N, stream()))
    assert_close(gd.cpu().numpy(), O.swiglu(gate.numpy(), up.numpy()), rtol=2e-3, atol=1e-3)
    a = torch.randn(M, 4096, generator=g).half()
    b = torch.randn(M, 4096, generator=g).half()
    ad, bd = a.to(gpu), b.to(gpu)
    check(lib().eet_residual_add(ad.data_ptr(), bd.data_ptr(), M, 4096, stream()))
    assert np.array_equal(ad.cpu().numpy(), O.residual_add(a.numpy(), b.numpy()))


@pytest.mark.parametrize("B,H,S,dh,use_pad,use_alibi", [(2, 3, 9, 128, False, False), (2, 2, 40, 64, True, False),
                                                       (1, 4, 130, 128, False, True), (2, 2, 33, 32, True, True),
                                                       (1, 1, 1, 128, False, False), (2, 2, 64, 128, False, False),
                                                       (2, 3, 300, 128, True, False), (1, 2, 257, 64, True, True),
                                                       (1, 2, 1024, 128, False, False), (1, 1, 2500, 128, False, True),
                                                       (2, 3, 200, 96, True, False), (1, 2, 77, 96, False, True),
                                                       (2, 2, 600, 128, True, True), (1, 3, 515, 128, False, True),
                                                       (1, 2, 256, 128, False, False), (2, 1, 255, 128, True, False),
                                                       (1, 2, 769, 128, False, False)])
def test_prefill_attention(gpu, B, H, S, dh, use_pad, use_alibi):
    g = torch.Generator().manual_seed(S)
    cap = S + 5
    q, k, v = [torch.randn(B, H, S, dh, generator=g).half() for _ in range(3)]
    kc = torch.zeros(B, H, cap, dh).half()
    vc = torch.zeros(B, H, cap, dh).half()
    kc[:, :, :S], vc[:, :, :S] = k, v
    pad = torch.tensor([0, min(S - 1, 70)][:B] if B > 1 else [min(S - 1, 70)]) if use_pad else None
    bias_full = O.alibi_mask(H, S) if use_alibi else None
    want = O.prefill_attention(q.numpy(), k.numpy(), v.numpy(), pad.numpy() if use_pad else None, bias_full)
    ctx = torch.empty(B, S, H * dh, dtype=torch.float16, device=gpu)
    row = torch.from_numpy(O.alibi_bias(H, S)).to(gpu) if use_alibi else None
    padd = pad.to(gpu) if use_pad else None
    qd, kcd, vcd = q.to(gpu), kc.to(gpu), vc.to(gpu)
    check(lib().eet_prefill_attention(qd.data_ptr(), kcd.data_ptr(), vcd.data_ptr(),
                                      ctx.data_ptr(), row.data_ptr() if use_alibi else None,
                                      padd.data_ptr() if use_pad else None, B, H, S, dh, cap, stream()))
    assert_close(ctx.cpu().numpy(), want, what="prefill ctx")


@pytest.mark.parametrize("dh", [128, 64])
@pytest.mark.parametrize("dominant", [1, 6, 11, 12, 37, 62])
def test_prefill_attention_one_dominant_key(gpu, dh, dominant):
    """One key whose score towers over the rest (q . k / sqrt(dh) ~ +40 against O(1)), at every position class
    of the 64-key chunk layout: the running maximum has to be taken over all keys of a chunk, or the weight of
    that key overflows fp16 (e^40) and the row comes out as NaN.  Every later query then returns that key's V row."""
    B, H, S = 1, 2, 192
    g = torch.Generator().manual_seed(dominant)
    q = torch.full((B, H, S, dh), 2.0).half()
    k = (torch.randn(B, H, S, dh, generator=g) * 0.05).half()
    v = torch.randn(B, H, S, dh, generator=g).half()
    for pos in (dominant, 64 + dominant):
        k[:, :, pos] = 40.0 * (dh ** 0.5) / (2.0 * dh)
    want = O.prefill_attention(q.numpy(), k.numpy(), v.numpy(), None, None)
    ctx = torch.empty(B, S, H * dh, dtype=torch.float16, device=gpu)
    qd, kd, vd = q.to(gpu), k.to(gpu), v.to(gpu)
    check(lib().eet_prefill_attention(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), ctx.data_ptr(), None, None,
                                      B, H, S, dh, S, stream()))
    got = ctx.cpu().numpy()
    assert np.isfinite(got).all()
    assert_close(got, want, what=f"dominant key {dominant}")


@pytest.mark.parametrize("dh", [128, 64])
@pytest.mark.parametrize("per_chunk", [0.5, 3.0, 7.0, 12.0])
def test_prefill_attention_rising_scores(gpu, dh, per_chunk):
    """Scores that rise along the keys by `per_chunk` powers of two per 64-key chunk: the running reference of the
    softmax is passed by a little in every chunk (below and above the point where the kernel re-bases its
    accumulators), by a lot in a few, and the weights of a row span the whole fp16 range.  Held to the oracle."""
    B, H, S = 1, 2, 448
    g = torch.Generator().manual_seed(int(per_chunk * 10) + dh)
    unit = torch.ones(dh) / dh ** 0.5
    q = (unit * 4.0 + torch.randn(B, H, S, dh, generator=g) * 0.05).half()
    # q . k / sqrt(dh) = 4 a_t / sqrt(dh); in powers of two: times log2(e)
    slope = per_chunk / 64.0 / 1.4427 * dh ** 0.5 / 4.0
    a = torch.arange(S).float() * slope
    k = (unit[None, None, None, :] * a[None, None, :, None] + torch.randn(B, H, S, dh, generator=g) * 0.05).half()
    v = torch.randn(B, H, S, dh, generator=g).half()
    want = O.prefill_attention(q.numpy(), k.numpy(), v.numpy(), None, None)
    ctx = torch.empty(B, S, H * dh, dtype=torch.float16, device=gpu)
    qd, kd, vd = q.to(gpu), k.to(gpu), v.to(gpu)
    check(lib().eet_prefill_attention(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), ctx.data_ptr(), None, None,
                                      B, H, S, dh, S, stream()))
    got = ctx.cpu().numpy()
    assert np.isfinite(got).all()
    assert_close(got, want, what=f"rising scores {per_chunk}/chunk")


@pytest.mark.parametrize("shape", [1, 2])
@pytest.mark.parametrize("S,use_pad,use_alibi", [(300, True, False), (1025, False, True), (64, False, False),
                                                 (515, True, True), (1700, False, False)])
def test_prefill_attention_launch_shapes_dh128(gpu, tuning, shape, S, use_pad, use_alibi):
    """Head size 128 runs in one of two launch shapes (queries per workgroup, tiles per wavefront, ring depth)
    depending on the prompt length; each is forced here at lengths on either side of the switch and held to
    the same oracle."""
    tuning("EET_PREFILL_SHAPE", shape)
    test_prefill_attention(gpu, 2, 2, S, 128, use_pad, use_alibi)


@pytest.mark.parametrize("group", [-1, 1, 2, 5])
@pytest.mark.parametrize("B,H,S,dh", [(4, 6, 700, 128), (2, 8, 1600, 128), (4, 4, 300, 64)])
def test_prefill_attention_workgroup_order(gpu, tuning, group, B, H, S, dh):
    """Which (batch, head) pair and query block a workgroup takes is a permutation chosen for the XCDs' L2
    caches (pairs in groups per XCD, long query blocks first); every forced group size -- also one that does not
    divide the pairs of an XCD, and the ungrouped order -- must cover every (pair, block) exactly once: the
    context buffer starts as NaN and is held to the oracle everywhere."""
    tuning("EET_PREFILL_GROUP", group)
    g = torch.Generator().manual_seed(S + group)
    q, k, v = [torch.randn(B, H, S, dh, generator=g).half() for _ in range(3)]
    want = O.prefill_attention(q.numpy(), k.numpy(), v.numpy(), None, None)
    ctx = torch.full((B, S, H * dh), float("nan"), dtype=torch.float16, device=gpu)
    qd, kcd, vcd = q.to(gpu), k.to(gpu).contiguous(), v.to(gpu).contiguous()
    check(lib().eet_prefill_attention(qd.data_ptr(), kcd.data_ptr(), vcd.data_ptr(), ctx.data_ptr(), None, None,
                                      B, H, S, dh, S, stream()))
    got = ctx.cpu().numpy()
    assert not np.isnan(got).any(), "a (pair, query block) was left out"
    assert_close(got, want, what=f"prefill ctx, group {group}")


@pytest.mark.parametrize("S,use_alibi", [(300, False), (130, True)])
def test_prefill_attention_register_staged_kernel_dh128(gpu, tuning, S, use_alibi):
    """Head size 128 normally takes the DMA kernel; the register-staged one (the path of the other head
    sizes, and of bias rows the DMA kernel cannot address) is selected here and held to the same oracle."""
    tuning("EET_PREFILL_LEGACY", 1)
    test_prefill_attention(gpu, 2, 3, S, 128, True, use_alibi)


@pytest.mark.parametrize("B,H,dh,rows,cap", [(4, 3, 64, 9, 16), (8, 32, 128, 100, 128), (3, 2, 32, 0, 8),
                                             (5, 4, 128, 40, 40)])
def test_kv_cache_reorder(gpu, B, H, dh, rows, cap):
    """Gather with repeated sources; rows at and after `rows` of the destination stay as they were.
    Bit-exact against the oracle's snapshot gather."""
    g = torch.Generator().manual_seed(B * 100 + rows)
    k = torch.randn(B, H, cap, dh, generator=g).half()
    v = torch.randn(B, H, cap, dh, generator=g).half()
    idx = torch.randint(0, B, (B,), generator=g)
    idx[0] = idx[-1] = B - 1                      # a source used twice, and beam 0 overwritten
    kd0 = torch.randn(B, H, cap, dh, generator=g).half()
    vd0 = torch.randn(B, H, cap, dh, generator=g).half()
    dk, dv, dkd, dvd, didx = k.to(gpu), v.to(gpu), kd0.to(gpu), vd0.to(gpu), idx.to(gpu)
    check(lib().eet_kv_cache_reorder(dk.data_ptr(), dv.data_ptr(), dkd.data_ptr(), dvd.data_ptr(), didx.data_ptr(),
                                     B, H, dh, rows, cap, stream()), "eet_kv_cache_reorder")
    torch.cuda.synchronize()
    wk, wv = k.numpy().copy(), v.numpy().copy()
    O.reorder_cache(wk, wv, idx.numpy(), rows)
    wk[:, :, rows:], wv[:, :, rows:] = kd0.numpy()[:, :, rows:], vd0.numpy()[:, :, rows:]
    assert np.array_equal(dkd.cpu().numpy().view(np.uint16), wk.view(np.uint16))
    assert np.array_equal(dvd.cpu().numpy().view(np.uint16), wv.view(np.uint16))
    # the sources are untouched
    assert torch.equal(dk.cpu(), k) and torch.equal(dv.cpu(), v)


def test_kv_cache_reorder_arguments(gpu):
    B, H, dh, cap = 2, 2, 64, 8
    k = torch.zeros(B, H, cap, dh, dtype=torch.float16, device=gpu)
    v, k2, v2 = torch.zeros_like(k), torch.zeros_like(k), torch.zeros_like(k)
    idx = torch.tensor([5, -1], device=gpu)          # out of range: the beam keeps its own rows
    k.copy_(torch.arange(k.numel(), device=gpu).view_as(k) % 97)
    L = lib()
    assert L.eet_kv_cache_reorder(k.data_ptr(), v.data_ptr(), k2.data_ptr(), v2.data_ptr(), idx.data_ptr(), B, H, dh,
                                  4, cap, stream()) == 0
    torch.cuda.synchronize()
    assert torch.equal(k2[:, :, :4], k[:, :, :4]) and not k2[:, :, 4:].any()
    # in place would race: refused
    assert L.eet_kv_cache_reorder(k.data_ptr(), v.data_ptr(), k.data_ptr(), v2.data_ptr(), idx.data_ptr(), B, H, dh,
                                  4, cap, stream()) == -1
    assert b"overlap" in L.eet_last_error()
    assert L.eet_kv_cache_reorder(k.data_ptr(), v.data_ptr(), k2.data_ptr(), v2.data_ptr(), idx.data_ptr(), B, H, dh,
                                  9, cap, stream()) == -1
    assert L.eet_kv_cache_reorder(k.data_ptr(), v.data_ptr(), k2.data_ptr(), v2.data_ptr(), idx.data_ptr(), B, H, 12,
                                  4, cap, stream()) == -2
