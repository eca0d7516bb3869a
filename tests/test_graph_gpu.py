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
