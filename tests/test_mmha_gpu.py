"""GPU parity of the decode attention against the fp32 oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import ops as O

from gpu_util import assert_close, mmha

pytestmark = pytest.mark.gpu


def case(B, H, dh, step, cap, seed, use_pad=False, use_alibi=False):
    g = torch.Generator().manual_seed(seed)
    kc = torch.randn(B, H, cap, dh, generator=g).half()
    vc = torch.randn(B, H, cap, dh, generator=g).half()
    q, k, v = [torch.randn(B, H, dh, generator=g).half() for _ in range(3)]
    pad = torch.randint(0, max(1, step // 2), (B,), generator=g) if use_pad else None
    alibi = torch.from_numpy(O.alibi_bias(H, step)) if use_alibi else None
    return q, k, v, kc, vc, pad, alibi


CASES = [
    # B, H, dh, step, cap, pad, alibi
    (2, 4, 128, 1, 16, False, False),
    (2, 4, 128, 2, 16, False, False),
    (2, 4, 128, 37, 64, True, False),
    (3, 5, 64, 300, 512, False, True),
    (2, 2, 32, 70, 80, True, True),
    (1, 8, 128, 4096, 4100, False, False),      # past the reference's 4096-step limit? no: exactly at it
    (1, 2, 128, 5000, 5000, True, False),       # beyond it
    (8, 32, 128, 1025, 1153, False, False),     # benchmark configuration 4, first decode step
    (8, 32, 128, 1152, 1153, False, False),     # config 4, last decode step
    (4, 40, 128, 2304, 2305, False, True),      # config 5 shape at reduced batch
    (2, 3, 96, 1, 8, False, False),             # head size 96: 12 of the 16 lanes of a row group hold a slice
    (2, 5, 96, 413, 420, True, True),
    (1, 32, 96, 2100, 2100, True, False),
]


@pytest.mark.parametrize("B,H,dh,step,cap,use_pad,use_alibi", CASES)
def test_against_oracle(gpu, B, H, dh, step, cap, use_pad, use_alibi):
    q, k, v, kc, vc, pad, alibi = case(B, H, dh, step, cap, step + B, use_pad, use_alibi)
    kcn, vcn = kc.numpy().copy(), vc.numpy().copy()
    want = O.decode_attention(q.numpy(), k.numpy(), v.numpy(), kcn, vcn, step,
                              pad.numpy() if use_pad else None, alibi.numpy() if use_alibi else None)
    kcd, vcd = kc.to(gpu), vc.to(gpu)
    ctx = mmha(q.to(gpu), k.to(gpu), v.to(gpu), kcd, vcd, step, pad.to(gpu) if use_pad else None,
               alibi.to(gpu) if use_alibi else None)
    assert_close(ctx.cpu().numpy(), want, what="ctx")
    # the new token landed in row step-1, nothing else moved
    assert np.array_equal(kcd.cpu().numpy(), kcn) and np.array_equal(vcd.cpu().numpy(), vcn)


@pytest.mark.parametrize("threads", [256, 512, 1024])
@pytest.mark.parametrize("ring", [2, 4, 8])
@pytest.mark.parametrize("nsplit", [1, 3])
def test_every_launch_shape(gpu, tuning, threads, ring, nsplit):
    """Every workgroup width / ring depth / split count the kernel is instantiated for (selected with the
    tuning overrides), with padding, ALiBi, the fused rotary append and a ragged last pass of the ring."""
    tuning("EET_MMHA_THREADS", str(threads))
    tuning("EET_MMHA_UNROLL", str(ring))
    tuning("EET_MMHA_NSPLIT", str(nsplit))
    for (B, H, dh, step, use_pad, use_alibi) in [(2, 3, 128, 333, True, False), (2, 2, 64, 1207, False, True),
                                                 (1, 2, 32, 45, True, True), (3, 2, 128, 3, False, False),
                                                 (2, 2, 96, 290, True, True)]:
        cap = step + 3
        q, k, v, kc, vc, pad, alibi = case(B, H, dh, step, cap, step + threads, use_pad, use_alibi)
        kcn, vcn = kc.numpy().copy(), vc.numpy().copy()
        want = O.decode_attention(q.numpy(), k.numpy(), v.numpy(), kcn, vcn, step,
                                  pad.numpy() if use_pad else None, alibi.numpy() if use_alibi else None)
        kcd, vcd = kc.to(gpu), vc.to(gpu)
        ctx = mmha(q.to(gpu), k.to(gpu), v.to(gpu), kcd, vcd, step, pad.to(gpu) if use_pad else None,
                   alibi.to(gpu) if use_alibi else None)
        assert_close(ctx.cpu().numpy(), want, what=f"ctx B={B} H={H} dh={dh} step={step}")
        assert np.array_equal(kcd.cpu().numpy(), kcn) and np.array_equal(vcd.cpu().numpy(), vcn)


def test_known_answers(gpu):
    B, H, dh, cap = 2, 3, 128, 300
    q, k, v, kc, vc, _, _ = case(B, H, dh, 1, cap, 5)
    # step = 1  =>  ctx = v / (1 + 1e-6)
    ctx = mmha(q.to(gpu), k.to(gpu), v.to(gpu), kc.to(gpu), vc.to(gpu), 1).cpu()
    assert_close(ctx.view(B, H, dh).numpy(), v.float().numpy() / (1 + 1e-6))
    # uniform keys  =>  ctx = mean of the values (both one block and split over several)
    for step in (17, 290):
        ku = k[:, :, None, :].expand(B, H, cap, dh).contiguous()
        vcd = vc.to(gpu)
        ctx = mmha(q.to(gpu), k.to(gpu), v.to(gpu), ku.to(gpu), vcd, step).cpu()
        vv = vc.clone()
        vv[:, :, step - 1] = v
        assert_close(ctx.view(B, H, dh).numpy(), vv[:, :, :step].float().mean(2).numpy(), atol=2e-3)


def test_fused_rows_and_no_append(gpu):
    """q, k, v as rows of a fused [B, 3*H*dh] buffer (the Baichuan call form), and k = v = NULL
    (cache already holds the new row)."""
    B, H, dh, step, cap = 3, 4, 64, 50, 64
    q, k, v, kc, vc, _, _ = case(B, H, dh, step, cap, 8)
    fused = torch.cat([q.view(B, -1), k.view(B, -1), v.view(B, -1)], 1).contiguous().to(gpu)
    kcn, vcn = kc.numpy().copy(), vc.numpy().copy()
    want = O.decode_attention(q.numpy(), k.numpy(), v.numpy(), kcn, vcn, step)
    hd = H * dh
    kcd, vcd = kc.to(gpu), vc.to(gpu)
    ctx = mmha(fused, fused[:, hd:], fused[:, 2 * hd:], kcd, vcd, step, stride=3 * hd)
    assert_close(ctx.cpu().numpy(), want)
    assert np.array_equal(kcd.cpu().numpy(), kcn)
    ctx2 = mmha(q.to(gpu), None, None, torch.from_numpy(kcn).to(gpu), torch.from_numpy(vcn).to(gpu), step)
    assert torch.equal(ctx2.cpu(), ctx.cpu())


def test_everything_padded_gives_zeros(gpu):
    B, H, dh, step, cap = 2, 2, 128, 9, 16
    q, k, v, kc, vc, _, _ = case(B, H, dh, step, cap, 3)
    pad = torch.tensor([step, 0])
    ctx = mmha(q.to(gpu), k.to(gpu), v.to(gpu), kc.to(gpu), vc.to(gpu), step, pad.to(gpu)).cpu().view(B, H, dh)
    assert not ctx[0].any() and ctx[1].any()


@pytest.mark.parametrize("dh,step", [(128, 1), (128, 77), (64, 300), (32, 40), (128, 1100), (96, 1), (96, 530)])
def test_fused_rotary(gpu, dh, step):
    """q and the appended k rotated inside the kernel == rotating them first (oracle) and then attending."""
    from eet_amd._lib import check, lib
    from gpu_util import stream
    B, H, cap = 2, 4, step + 3
    q, k, v, kc, vc, _, _ = case(B, H, dh, step, cap, 100 + step)
    pos = step - 1
    qr, kr = O.rope_neox(q.numpy(), pos), O.rope_neox(k.numpy(), pos)
    kcn, vcn = kc.numpy().copy(), vc.numpy().copy()
    want = O.decode_attention(qr, kr, v.numpy(), kcn, vcn, step)
    table = torch.empty(cap, dh, dtype=torch.float32, device=gpu)
    check(lib().eet_rope_table(table.data_ptr(), cap, dh, stream()))
    c, s = O.rope_coeff(pos, dh)
    assert_close(table[pos].cpu().numpy(), np.concatenate([c, s]), rtol=0, atol=2e-4, what="rope table row")
    kcd, vcd = kc.to(gpu), vc.to(gpu)
    ctx = mmha(q.to(gpu), k.to(gpu), v.to(gpu), kcd, vcd, step, rope_row=table[pos])
    assert_close(ctx.cpu().numpy(), want, what="ctx")
    assert_close(kcd.cpu().numpy(), kcn, rtol=4e-3, atol=4e-3, what="k cache")   # rotated k landed in row step-1
    assert np.array_equal(vcd.cpu().numpy(), vcn)


@pytest.mark.parametrize("B,H,step,cap,use_alibi", [(8, 32, 1152, 1153, False),      # benchmark configuration 4, full size
                                                    (32, 40, 2304, 2305, True)])     # config 5, full size
def test_full_size_uniform_keys(gpu, B, H, step, cap, use_alibi):
    """Size-independent property at the full benchmark shapes: when every cached key of a head equals the new
    key, q . k_t is the same for all t, so the weights are softmax(bias) alone (uniform without ALiBi) over
    the rows that are not padded away, and ctx is that weighted mean of V, whatever q is."""
    dh = 128
    g = torch.Generator(device=gpu).manual_seed(B * step)
    k0 = torch.randn(B, H, dh, generator=g, device=gpu).half()
    kc = k0[:, :, None, :].expand(B, H, cap, dh).contiguous()
    vc = torch.randn(B, H, cap, dh, generator=g, device=gpu).half()
    q = torch.randn(B, H, dh, generator=g, device=gpu).half()
    v = torch.randn(B, H, dh, generator=g, device=gpu).half()
    pad = torch.randint(0, step // 2, (B,), generator=g, device=gpu)
    bias = torch.from_numpy(O.alibi_bias(H, step)).to(gpu) if use_alibi else None
    ctx = mmha(q, k0, v, kc, vc, step, pad, bias)
    vv = vc[:, :, :step].float()
    vv[:, :, step - 1] = v.float()                                    # the appended row
    logits = bias.float()[None].expand(B, H, step).clone() if use_alibi else torch.zeros(B, H, step, device=gpu)
    logits.masked_fill_(torch.arange(step, device=gpu)[None, None, :] < pad[:, None, None], float("-inf"))
    want = torch.einsum("bht,bhtd->bhd", torch.softmax(logits, -1), vv).reshape(B, H * dh)
    assert_close(ctx.cpu().numpy(), want.cpu().numpy(), what="ctx")
    assert torch.equal(kc[:, :, step - 1], k0) and torch.equal(vc[:, :, step - 1], v)
