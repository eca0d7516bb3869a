"""The incremental decode step recorded once into a HIP graph and replayed: the replayable form of
the attention call (step read from device memory) against the by-value form through the C ABI, and
greedy decoding from graph replays against the eager loop, token for token, on tiny models.
Replays alternate with eager work and synchronisations, and every replay is checked."""
import numpy as np
import pytest
import torch

from eet_amd import decoder as D
from eet_amd._lib import check, lib

from gpu_util import mmha, stream

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,H,dh,alibi,rope", [(2, 4, 128, False, True), (3, 8, 64, True, False), (8, 32, 128, False, False)])
def test_replayable_attention_matches_by_value_form(gpu, B, H, dh, alibi, rope):
    L = lib()
    g = torch.Generator().manual_seed(B + H)
    cap, step_max = 700, 700
    kc = torch.randn(B, H, cap, dh, generator=g).half().to(gpu)
    vc = torch.randn(B, H, cap, dh, generator=g).half().to(gpu)
    kc2, vc2 = kc.clone(), vc.clone()
    bias = (torch.rand(H, cap, generator=g) * 4).half().to(gpu) if alibi else None
    table = torch.empty(cap, dh, dtype=torch.float32, device=gpu)
    check(L.eet_rope_table(table.data_ptr(), cap, dh, stream()))
    step_dev = torch.zeros(1, dtype=torch.int32, device=gpu)
    need = L.eet_mmha_decode_replayable_workspace(B, H, dh, step_max)
    ws = torch.empty(max(need // 4, 1), dtype=torch.float32, device=gpu)
    for step in (1, 2, 37, 300, 699, 700):
        q, k, v = [torch.randn(B, H, dh, generator=g).half().to(gpu) for _ in range(3)]
        step_dev.fill_(step)
        ctx = torch.empty(B, H * dh, dtype=torch.float16, device=gpu)
        check(L.eet_mmha_decode_replayable(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0, kc.data_ptr(), vc.data_ptr(),
                                           ctx.data_ptr(), bias.data_ptr() if alibi else None, cap if alibi else 0, None,
                                           B, H, dh, step_dev.data_ptr(), step_max, cap,
                                           table.data_ptr() if rope else None, ws.data_ptr(), ws.numel() * 4, stream()),
              "eet_mmha_decode_replayable")
        want = mmha(q, k, v, kc2, vc2, step, alibi=bias[:, :step].contiguous() if alibi else None,
                    rope_row=table[step - 1] if rope else None)
        torch.cuda.synchronize()
        # launch shapes can differ (the replayable call is shaped for step_max), so sums may be taken in
        # another order: same tolerance as against the oracle; the appended rows are bit-identical
        err = (ctx.float() - want.float()).abs()
        assert (err <= 1e-3 + 1e-2 * want.float().abs()).all(), (step, float(err.max()))
        assert torch.equal(kc[:, :, step - 1], kc2[:, :, step - 1]) and torch.equal(vc[:, :, step - 1], vc2[:, :, step - 1])
    # a step outside [1, step_max] is clamped into it: with step_max below the cache capacity a replay past
    # step_max repeats step_max instead of reading the rotary table and the bias rows past their end
    small_max = 300
    q, k, v = [torch.randn(B, H, dh, generator=g).half().to(gpu) for _ in range(3)]
    outs = []
    for held in (small_max, small_max + 7, 10 ** 6):
        kc3, vc3 = kc2.clone(), vc2.clone()
        step_dev.fill_(held)
        ctx = torch.empty(B, H * dh, dtype=torch.float16, device=gpu)
        check(L.eet_mmha_decode_replayable(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0, kc3.data_ptr(), vc3.data_ptr(),
                                           ctx.data_ptr(), bias.data_ptr() if alibi else None, cap if alibi else 0, None,
                                           B, H, dh, step_dev.data_ptr(), small_max, cap,
                                           table.data_ptr() if rope else None, ws.data_ptr(), ws.numel() * 4, stream()),
              "eet_mmha_decode_replayable")
        outs.append((ctx, kc3, vc3))
    torch.cuda.synchronize()
    for ctx, kc3, vc3 in outs[1:]:
        assert torch.equal(ctx, outs[0][0]) and torch.equal(kc3, outs[0][1]) and torch.equal(vc3, outs[0][2])
    step_dev.fill_(-3)          # below 1: runs as step 1
    ctx = torch.empty(B, H * dh, dtype=torch.float16, device=gpu)
    kc3, vc3 = kc2.clone(), vc2.clone()
    check(L.eet_mmha_decode_replayable(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0, kc3.data_ptr(), vc3.data_ptr(),
                                       ctx.data_ptr(), bias.data_ptr() if alibi else None, cap if alibi else 0, None,
                                       B, H, dh, step_dev.data_ptr(), small_max, cap,
                                       table.data_ptr() if rope else None, ws.data_ptr(), ws.numel() * 4, stream()),
          "eet_mmha_decode_replayable")
    want = mmha(q, k, v, kc2.clone(), vc2.clone(), 1, alibi=bias[:, :1].contiguous() if alibi else None,
                rope_row=table[0] if rope else None)
    torch.cuda.synchronize()
    assert torch.equal(ctx, want)


@pytest.mark.parametrize("alibi", [False, True])
def test_greedy_from_graph_replays_matches_eager(gpu, alibi):
    cfg = D.DecoderConfig(num_layers=2, hidden=256, heads=4, d_ff=704, vocab=512, eps=1e-6, alibi=alibi, max_batch=3,
                          max_prompt=12, max_full_seq=40)
    sd, _ = D.random_state_dict(cfg, seed=7)
    sd["lm_head.weight"] = sd["lm_head.weight"] * 8
    ids = torch.randint(0, cfg.vocab, (3, 9), generator=torch.Generator().manual_seed(3)).to(gpu)
    eager = D.Int8Decoder(cfg, sd, device="cuda:0")
    want = eager.greedy(ids, 12).cpu()
    graphed = D.Int8Decoder(cfg, sd, device="cuda:0")
    got = graphed.greedy_graph(ids, 12).cpu()
    assert torch.equal(got, want)
    assert graphed.layers[0][0].step == eager.layers[0][0].step == 9 + 11
    # replay by replay, with eager work of the same library and a synchronisation in between
    a, b = D.Int8Decoder(cfg, sd, device="cuda:0"), D.Int8Decoder(cfg, sd, device="cuda:0")
    with torch.no_grad():
        la, lb = a.logits(ids, True), b.logits(ids, True)
        nxt = torch.argmax(la[:, -1, :], dim=-1)
        replay = b.capture_decode_step(nxt)
        for t in range(10):
            want_logits = a.logits(nxt[:, None], False)          # eager step on the twin model
            torch.cuda.synchronize()
            tok = replay().clone()
            torch.cuda.synchronize()
            assert torch.equal(tok, torch.argmax(want_logits[:, -1, :], dim=-1)), t
            nxt = tok
    assert torch.equal(a.layers[1][0].k_cache[:, :, :19], b.layers[1][0].k_cache[:, :, :19])
    # the step limit still holds for replays
    small = D.DecoderConfig(num_layers=1, hidden=256, heads=4, d_ff=704, vocab=512, alibi=alibi, max_batch=1,
                            max_prompt=4, max_full_seq=6)
    sd2, _ = D.random_state_dict(small, seed=8)
    m = D.Int8Decoder(small, sd2, device="cuda:0")
    with torch.no_grad():
        lg = m.logits(ids[:1, :4], True)
        rp = m.capture_decode_step(torch.argmax(lg[:, -1, :], dim=-1))
        rp()
        rp()
        with pytest.raises(RuntimeError, match="exceeds max_full_seq"):
            rp()


def test_recorded_step_survives_workspace_regrowth_and_resyncs(gpu):
    """The graph records raw pointers of the named workspaces.  After the recording a LARGER decoder asks for
    the same names (the named buffers are replaced), the workspaces are cleared, and fresh allocations
    overwrite whatever the allocator hands out again: replays must still match the eager twin, because the
    recording keeps its buffers alive.  Then an eager call on the graphed decoder moves the host-side step:
    the next replay brings the device-side step back in line; and a decoder with a reorder state set
    refuses to replay."""
    from eet_amd import ops
    cfg = D.DecoderConfig(num_layers=2, hidden=256, heads=4, d_ff=704, vocab=512, eps=1e-6, alibi=False, max_batch=3,
                          max_prompt=12, max_full_seq=48)
    sd, _ = D.random_state_dict(cfg, seed=17)
    sd["lm_head.weight"] = sd["lm_head.weight"] * 8
    ids = torch.randint(0, cfg.vocab, (3, 9), generator=torch.Generator().manual_seed(4)).to(gpu)
    ops.workspaces.clear()
    a, b = D.Int8Decoder(cfg, sd, device="cuda:0"), D.Int8Decoder(cfg, sd, device="cuda:0")
    with torch.no_grad():
        la, lb = a.logits(ids, True), b.logits(ids, True)
        nxt = torch.argmax(la[:, -1, :], dim=-1)
        replay = b.capture_decode_step(nxt)

        def both(n, t0):
            nonlocal nxt
            for t in range(n):
                want = torch.argmax(a.logits(nxt[:, None], False)[:, -1, :], dim=-1)
                torch.cuda.synchronize()
                tok = replay().clone()
                torch.cuda.synchronize()
                assert torch.equal(tok, want), t0 + t
                nxt = tok
        both(3, 0)
        # a larger decoder under the same workspace names, then clear(), then junk over the freed memory
        big = D.DecoderConfig(num_layers=1, hidden=256, heads=4, d_ff=704, vocab=512, alibi=False, max_batch=6,
                              max_prompt=40, max_full_seq=64)
        sdb, _ = D.random_state_dict(big, seed=18)
        c = D.Int8Decoder(big, sdb, device="cuda:0")
        c.logits(torch.randint(0, big.vocab, (6, 40), generator=torch.Generator().manual_seed(1)).to(gpu), True)
        c.logits(torch.randint(0, big.vocab, (6, 1), generator=torch.Generator().manual_seed(2)).to(gpu), False)
        ops.workspaces.clear()
        torch.cuda.synchronize()
        junk = [torch.full((1 << 16,), float("nan"), dtype=torch.float16, device=gpu) for _ in range(64)]
        torch.cuda.synchronize()
        both(3, 3)          # `a` re-creates its workspaces by name; the recording still owns the old ones
        del junk
        # an eager step on the graphed decoder itself: the host-side step moves, the device-side one does not
        want = torch.argmax(a.logits(nxt[:, None], False)[:, -1, :], dim=-1)
        got = torch.argmax(b.logits(nxt[:, None], False)[:, -1, :], dim=-1)
        assert torch.equal(got, want)
        nxt = got
        want = torch.argmax(a.logits(nxt[:, None], False)[:, -1, :], dim=-1)
        tok = replay(nxt).clone()      # the previous replay's output is stale: hand the tokens over
        torch.cuda.synchronize()
        assert torch.equal(tok, want)
        nxt = tok
        both(2, 8)
        assert b.layers[0][0].step == a.layers[0][0].step
        # a new prompt on the graphed decoder, then replays again
        la, lb = a.logits(ids[:, :7], True), b.logits(ids[:, :7], True)
        nxt = torch.argmax(la[:, -1, :], dim=-1)
        want = torch.argmax(a.logits(nxt[:, None], False)[:, -1, :], dim=-1)
        tok = replay(nxt).clone()
        torch.cuda.synchronize()
        assert torch.equal(tok, want)
        # beam reorder swaps cache buffers: refused
        b.reorder_state = torch.zeros(3, dtype=torch.long, device=gpu)
        with pytest.raises(RuntimeError, match="reorder"):
            replay()
        with pytest.raises(RuntimeError, match="reorder"):
            b.capture_decode_step(nxt)
    ops.workspaces.clear()


def test_graph_replays_with_the_k_split_match_eager(gpu):
    """At batch 16 the down projection of a LLaMA-7B-width layer runs with the k split (four
    workgroups share a tile group and exchange partial sums through a named workspace whose counters must be
    zero): the recorded step replays that workspace's pointer, so replays must leave the counters as eager
    calls do.  Token for token against the eager loop, and an eager run AFTER the replays on the same
    workspace."""
    import ctypes
    from eet_amd._lib import check, lib
    v = [ctypes.c_int(0) for _ in range(4)]
    check(lib().eet_gemm_w8a16_small_m_shape(16, 4096, 11008, 1, 0, *[ctypes.byref(x) for x in v]))
    assert v[3].value > 1 and lib().eet_gemm_w8a16_workspace(16, 4096, 11008, 1) > 0, "the k split is expected here"
    cfg = D.DecoderConfig(num_layers=1, hidden=4096, heads=32, d_ff=11008, vocab=512, eps=1e-6, alibi=False, max_batch=16,
                          max_prompt=8, max_full_seq=24)
    sd, _ = D.random_state_dict(cfg, seed=11)
    sd["lm_head.weight"] = sd["lm_head.weight"] * 8
    ids = torch.randint(0, cfg.vocab, (16, 5), generator=torch.Generator().manual_seed(5)).to(gpu)
    eager = D.Int8Decoder(cfg, sd, device="cuda:0")
    want = eager.greedy(ids, 8).cpu()
    graphed = D.Int8Decoder(cfg, sd, device="cuda:0")
    got = graphed.greedy_graph(ids, 8).cpu()
    assert torch.equal(got, want)
    again = eager.greedy(ids, 8).cpu()          # the shared workspace is still usable by eager calls
    assert torch.equal(again, want)


def test_static_attention_entry_point_inside_a_graph(gpu):
    """eet_mmha_decode_static recorded into a HIP graph after one warm call outside the capture (the first
    call per device looks the scratch address up), replayed with eager work in between: every replay is
    bit-identical to eet_mmha_decode with a workspace."""
    L = lib()
    B, H, dh, cap = 1, 16, 128, 1200        # B*H < 256: the time axis is split, the partials go through the scratch
    g = torch.Generator().manual_seed(23)
    kc = torch.randn(B, H, cap, dh, generator=g).half().to(gpu)
    vc = torch.randn(B, H, cap, dh, generator=g).half().to(gpu)
    step = 1100
    assert L.eet_mmha_decode_workspace(B, H, dh, step) > 0
    q, k, v = [torch.randn(B, H, dh, generator=g).half().to(gpu) for _ in range(3)]
    ctx = torch.zeros(B, H * dh, dtype=torch.float16, device=gpu)

    def call():
        check(L.eet_mmha_decode_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0, kc.data_ptr(), vc.data_ptr(),
                                       ctx.data_ptr(), None, None, B, H, dh, step, cap, None, stream()),
              "eet_mmha_decode_static")
    call()                                   # warm call outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        q.copy_(torch.randn(B, H, dh, generator=g).half())
        k.copy_(torch.randn(B, H, dh, generator=g).half())
        kc2, vc2 = kc.clone(), vc.clone()
        want = mmha(q, k, v, kc2, vc2, step)          # eager work of the same library between the replays
        torch.cuda.synchronize()
        ctx.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(ctx, want), rep
        assert torch.equal(kc[:, :, step - 1], kc2[:, :, step - 1])
