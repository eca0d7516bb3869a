"""Pins the oracle's composed layer and decoder (OracleAttention, OracleFFN, OracleDecoder) with
checks that do not retype them:

  * against tests/hf_formulation.py -- float64, Hugging Face formulation, no KV cache, the whole
    sequence recomputed under a causal mask -- at every prompt row and every incremental step;
  * negative controls: the same comparison with one plausible mistake planted in the independent
    model (gate/up swapped, residual taken after the norm, rotary position off by one, K and V
    column blocks swapped) must FAIL by a wide margin, so the comparison has the power to see them;
  * closed forms: zero output-projection / down-projection weights give output == input bit for
    bit; a one-token prompt gives x + Wo . v / (1 + 1e-6); the rotary position of incremental
    step t is the prompt position t (an incremental call equals the last row of a longer prefill).
"""
import math

import numpy as np
import pytest

import hf_formulation as HF
from oracle import ops as O
from oracle import quant as Q

EPS = 1e-6


def make_model(seed, layers=2, hidden=128, heads=4, d_ff=192, vocab=96, alibi=False, cap=16, batch=2):
    """Random HF-style weights -> per-channel int8 (oracle quantiser) -> (independent float64 model
    over the dequantised weights, oracle decoder over the int8 weights)."""
    rng = np.random.default_rng(seed)
    dh = hidden // heads

    def linear(out_f, in_f):
        w = (rng.standard_normal((out_f, in_f)) * 0.08).astype(np.float16)     # nn.Linear layout [out, in]
        q, s = Q.quantize_ref128(np.ascontiguousarray(w.T))                    # EET layout [in, out]
        deq = (q.astype(np.float64) * s.astype(np.float64)[None, :]).T         # back to [out, in]
        return q, s, deq

    slopes = HF.power_of_two_slopes(heads) if alibi else None
    hf_layers, or_layers = [], []
    for _ in range(layers):
        (qq, qs, wq), (kq, ks, wk), (vq, vs, wv) = [linear(hidden, hidden) for _ in range(3)]
        oq, os_, wo = linear(hidden, hidden)
        gq, gs, wg = linear(d_ff, hidden)
        uq, us, wu = linear(d_ff, hidden)
        dq, ds, wd = linear(hidden, d_ff)
        g1 = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
        g2 = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
        hf_layers.append(HF.Layer(wq, wk, wv, wo, wg, wu, wd, g1, g2, heads, EPS, slopes))
        # fused QKV: columns [Q | K | V] (python/eet/transformers/modeling_llama.py:85)
        qkv_q, qkv_s = np.concatenate([qq, kq, vq], 1), np.concatenate([qs, ks, vs])
        or_layers.append((O.OracleAttention(batch, heads, dh, cap, qkv_q, qkv_s, oq, os_, g1, EPS, rope=not alibi),
                          O.OracleFFN(gq, gs, uq, us, dq, ds, g2, EPS)))
    embed = (rng.standard_normal((vocab, hidden)) * 0.5).astype(np.float16)
    gf = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    head = (rng.standard_normal((vocab, hidden)) * 0.08).astype(np.float16)
    hf = HF.Model(embed, hf_layers, gf, head, EPS)
    orc = O.OracleDecoder(embed, or_layers, gf, head, EPS, n_head=heads, alibi=alibi)
    return hf, orc, rng


def max_rel(got, want):
    """Largest error relative to the RMS magnitude of the expected tensor."""
    want = np.asarray(want, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - want).max() / math.sqrt((want * want).mean()))


# the oracle rounds to fp16 between ops (as the reference's buffers do); the independent model never rounds
TOL = 1.5e-2


def run_teacher_forced(hf, orc, ids, S, pad=None):
    """Oracle: prefill ids[:, :S], then one incremental call per remaining token.  Independent
    model: one full forward over all T tokens.  Returns the per-step relative errors of the logits."""
    B, T = ids.shape
    want = hf.logits(ids, pad)
    errs = [max_rel(orc.step(ids[:, :S], True, pad), want[:, S - 1])]
    for t in range(S, T):
        errs.append(max_rel(orc.step(ids[:, t:t + 1], False, pad), want[:, t]))
    return errs


@pytest.mark.parametrize("alibi", [False, True])
def test_decoder_matches_hf_formulation(alibi):
    hf, orc, rng = make_model(11, alibi=alibi)
    ids = rng.integers(0, 96, (2, 9))
    errs = run_teacher_forced(hf, orc, ids, S=5)
    assert max(errs) < TOL, errs


def test_decoder_matches_hf_formulation_left_padded():
    """Left padding: padded key columns carry no weight; rotary positions stay the raw token
    indices (csrc/core/self_add_bias.cu:393 uses the sequence index, padding included)."""
    hf, orc, rng = make_model(12)
    ids = rng.integers(0, 96, (2, 8))
    pad = np.array([0, 2])
    B, T = ids.shape
    want = hf.logits(ids, pad)
    got = orc.step(ids[:, :5], True, pad)
    assert max_rel(got, want[:, 4]) < TOL
    for t in range(5, T):
        assert max_rel(orc.step(ids[:, t:t + 1], False, pad), want[:, t]) < TOL


def test_every_prompt_row_of_a_layer():
    """One layer, all rows of the prompt (the decoder test only sees the last row of each call)."""
    hf, orc, rng = make_model(13, layers=1)
    x = rng.standard_normal((2, 6, 128)).astype(np.float16)
    attn, ffn = orc.layers[0]
    got = ffn.forward(attn.forward(x, None, True))
    want = hf.layers[0](x.astype(np.float64))
    assert max_rel(got, want) < TOL
    # and the attention sub-layer alone, so an error cannot hide behind the FFN
    hf2, orc2, _ = make_model(13, layers=1)
    assert max_rel(orc2.layers[0][0].forward(x, None, True), hf2.layers[0].attention(x.astype(np.float64), None)) < TOL


class _Mistake:
    """Plants one plausible mistake into the independent model."""

    @staticmethod
    def swap_gate_up(layer):
        layer.w[4], layer.w[5] = layer.w[5], layer.w[4]

    @staticmethod
    def residual_after_norm(layer):
        orig = layer.ffn

        def ffn(h):
            hn = HF.rms(h, layer.g_ffn, layer.eps)
            return orig(h) - h + hn
        layer.ffn = ffn

    @staticmethod
    def swap_k_v(layer):
        layer.w[1], layer.w[2] = layer.w[2], layer.w[1]

    @staticmethod
    def rotary_off_by_one(layer):
        real = HF.rope
        orig = layer.attention

        def attention(x, pad):
            HF.rope = lambda t, pos: real(t, pos + (pos >= 5))     # incremental steps shifted by one
            try:
                return orig(x, pad)
            finally:
                HF.rope = real
        layer.attention = attention

    @staticmethod
    def rotary_pairs_adjacent(layer):
        """GPT-J style pairs (2i, 2i+1) instead of NeoX pairs (i, i + dh/2)."""
        real = HF.rope
        orig = layer.attention

        def gptj(x, positions):
            d = x.shape[-1]
            inv_freq = 1.0 / (10000.0 ** (np.arange(0, d, 2, dtype=np.float64) / d))
            ang = positions[:, None] * inv_freq[None, :]
            c, s = np.cos(ang)[None, None], np.sin(ang)[None, None]
            out = np.empty_like(x)
            out[..., 0::2] = x[..., 0::2] * c - x[..., 1::2] * s
            out[..., 1::2] = x[..., 1::2] * c + x[..., 0::2] * s
            return out

        def attention(x, pad):
            HF.rope = gptj
            try:
                return orig(x, pad)
            finally:
                HF.rope = real
        layer.attention = attention


@pytest.mark.parametrize("mistake", ["swap_gate_up", "residual_after_norm", "swap_k_v", "rotary_off_by_one",
                                     "rotary_pairs_adjacent"])
def test_comparison_sees_planted_mistakes(mistake):
    hf, orc, rng = make_model(11)
    for layer in hf.layers:
        getattr(_Mistake, mistake)(layer)
    ids = rng.integers(0, 96, (2, 9))
    errs = run_teacher_forced(hf, orc, ids, S=5)
    assert max(errs) > 5 * TOL, (mistake, errs)


def test_zero_projection_is_the_identity():
    """With all-zero O-proj (down-proj) weights the sub-layer returns its input bit for bit:
    the residual is the un-normalised input and is added exactly once."""
    _, orc, rng = make_model(14, layers=1)
    attn, ffn = orc.layers[0]
    x = rng.standard_normal((2, 4, 128)).astype(np.float16)
    attn.o_q = np.zeros_like(attn.o_q)
    assert np.array_equal(attn.forward(x, None, True), x)
    x1 = rng.standard_normal((2, 1, 128)).astype(np.float16)
    assert np.array_equal(attn.forward(x1, None, False), x1)
    ffn.d_q = np.zeros_like(ffn.d_q)
    assert np.array_equal(ffn.forward(x), x)


def test_one_token_prompt_closed_form():
    """A prompt of one token attends only itself: ctx = v / (1 + 1e-6) and the sub-layer output is
    x + Wo . ctx, whatever q and k are (so also whatever the rotary position is)."""
    _, orc, rng = make_model(15, layers=1)
    attn = orc.layers[0][0]
    x = rng.standard_normal((2, 1, 128)).astype(np.float16)
    got = attn.forward(x, None, True)
    xn = HF.rms(x.astype(np.float64), attn.gamma.astype(np.float64), EPS)
    wv = attn.qkv_q[:, 256:].astype(np.float64) * attn.qkv_s[256:].astype(np.float64)
    wo = attn.o_q.astype(np.float64) * attn.o_s.astype(np.float64)
    want = x.astype(np.float64) + ((xn @ wv) / (1 + 1e-6)) @ wo
    assert max_rel(got, want) < 5e-3
    assert attn.step == 1


def test_incremental_call_equals_last_row_of_longer_prefill():
    """Rotary position and cache row of incremental step t are those of prompt position t: feeding
    tokens one by one gives what a prefill of the longer prompt gives in its last row."""
    _, orc_a, rng = make_model(16, layers=1)
    _, orc_b, _ = make_model(16, layers=1)
    x = rng.standard_normal((2, 7, 128)).astype(np.float16)
    a, b = orc_a.layers[0][0], orc_b.layers[0][0]
    a.forward(x[:, :4], None, True)
    for t in range(4, 7):
        inc = a.forward(x[:, t:t + 1], None, False)
        full = b.forward(x[:, :t + 1], None, True)
        assert np.abs(inc[:, 0].astype(np.float32) - full[:, -1].astype(np.float32)).max() < 4e-3
        assert a.step == b.step == t + 1
        assert np.array_equal(a.k_cache[:, :, :t + 1], b.k_cache[:, :, :t + 1])


def test_greedy_tokens_match_hf_formulation():
    hf, orc, rng = make_model(17)
    ids = rng.integers(0, 96, (2, 5))
    toks = orc.greedy(ids, 4)
    seq = ids
    for t in range(4):
        lg = hf.logits(seq)[:, -1]
        top2 = np.sort(lg, -1)[:, -2:]
        nxt = lg.argmax(-1)
        for b in range(2):
            if top2[b, 1] - top2[b, 0] > 0.05:        # margin above the fp16 noise of the oracle
                assert toks[b, t] == nxt[b]
        seq = np.concatenate([seq, toks[:, t:t + 1]], 1)     # follow the oracle's tokens


def test_bias_branch_one_token_closed_form():
    """The bias branch of the attention op on a one-token prompt, where attention is the identity on v:
    out = x + Wo . ((LN(x) . Wv + bv) / (1 + 1e-6)) + bo, with LayerNorm(gamma, beta) in front.  And the
    feed-forward op in its three tails against the float64 formulas."""
    rng = np.random.default_rng(21)
    hidden, heads, d_ff = 128, 4, 192

    def linear(i, o):
        q, s = Q.quantize_ref128(np.ascontiguousarray((rng.standard_normal((i, o)) * 0.08).astype(np.float16)))
        return q, s, q.astype(np.float64) * s.astype(np.float64)[None, :]
    qkv_q, qkv_s, wqkv = linear(hidden, 3 * hidden)
    o_q, o_s, wo = linear(hidden, hidden)
    g = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    beta = (0.2 * rng.standard_normal(hidden)).astype(np.float16)
    qkv_b = (0.3 * rng.standard_normal(3 * hidden)).astype(np.float16)
    o_b = (0.3 * rng.standard_normal(hidden)).astype(np.float16)
    attn = O.OracleAttention(2, heads, hidden // heads, 8, qkv_q, qkv_s, o_q, o_s, g, EPS, rope=False,
                             qkv_bias=qkv_b, o_bias=o_b, beta=beta)
    x = (rng.standard_normal((2, 1, hidden)) + 0.5).astype(np.float16)

    def ln(v):
        v = v.astype(np.float64)
        return (v - v.mean(-1, keepdims=True)) / np.sqrt(v.var(-1, keepdims=True) + EPS) * g.astype(np.float64) \
            + beta.astype(np.float64)
    v = ln(x) @ wqkv[:, 2 * hidden:] + qkv_b[2 * hidden:].astype(np.float64)
    want = x.astype(np.float64) + (v / (1 + 1e-6)) @ wo + o_b.astype(np.float64)
    assert max_rel(attn.forward(x, None, True), want) < 5e-3
    # the new token's k row in the cache carries its bias
    k = (ln(x) @ wqkv[:, hidden:2 * hidden] + qkv_b[hidden:2 * hidden].astype(np.float64)).reshape(2, heads, -1)
    assert np.abs(attn.k_cache[:, :, 0].astype(np.float64) - k).max() < 6e-3
    # without the bias terms the same formula must NOT match (the comparison sees a dropped bias)
    assert max_rel(attn.forward(x, None, True), x.astype(np.float64) + ((ln(x) @ wqkv[:, 2 * hidden:]) / (1 + 1e-6)) @ wo) > 0.05

    g_q, g_s, wg = linear(hidden, d_ff)
    u_q, u_s, wu = linear(hidden, d_ff)
    d_q, d_s, wd = linear(d_ff, hidden)
    x2 = (rng.standard_normal((2, 3, hidden)) + 0.5).astype(np.float16)

    def ffn_core(norm):
        xn = norm(x2)
        gate, up = xn @ wg, xn @ wu
        return (up * gate / (1 + np.exp(-gate))) @ wd

    def rms(v):
        v = v.astype(np.float64)
        return v / np.sqrt((v * v).mean(-1, keepdims=True) + EPS) * g.astype(np.float64)
    x64 = x2.astype(np.float64)
    ffn = O.OracleFFN(g_q, g_s, u_q, u_s, d_q, d_s, g, EPS, beta=beta, o_bias=o_b)
    assert max_rel(ffn.forward(x2, True, True), x64 + ffn_core(ln) + o_b.astype(np.float64)) < 1e-2
    assert max_rel(ffn.forward(x2, True, False), ffn_core(ln) + o_b.astype(np.float64)) < 1e-2
    assert max_rel(ffn.forward(x2, False, True), ln(x64 + ffn_core(ln) + o_b.astype(np.float64))) < 1e-2
    plain = O.OracleFFN(g_q, g_s, u_q, u_s, d_q, d_s, g, EPS)
    assert max_rel(plain.forward(x2, False, True), rms(x64 + ffn_core(rms))) < 1e-2      # RMSnorm tail without a bias
    assert max_rel(plain.forward(x2, True, False), ffn_core(rms)) < 1e-2


def test_beam_search_against_exhaustive_search():
    """The checker's beam search over a first-order table model (logits depend on the last token only), where
    the answer can be enumerated: with num_beams >= V^(T-1) every prefix survives, so the result is the
    sequence of highest total log-probability among all V^T; with one beam it is the greedy sequence; with an
    end-of-sequence token the returned score is the length-normalised log-probability of what is returned."""
    import itertools
    rng = np.random.default_rng(33)
    V, T = 5, 3
    table = rng.standard_normal((V, V)) * 2.0
    logp = table - np.log(np.exp(table).sum(-1, keepdims=True))

    def step_fn(ids, first, reorder):
        return table[ids[:, -1]]
    prompt = np.array([[1, 3], [0, 2]])
    toks, score = O.beam_search(step_fn, prompt, V ** (T - 1), T)
    for b in range(2):
        best = max(itertools.product(range(V), repeat=T),
                   key=lambda s: logp[prompt[b, -1], s[0]] + logp[s[0], s[1]] + logp[s[1], s[2]])
        assert tuple(toks[b]) == best
        total = logp[prompt[b, -1], best[0]] + logp[best[0], best[1]] + logp[best[1], best[2]]
        assert abs(score[b] - total / (2 + T)) < 1e-9            # length penalty 1: divided by prompt + generated
    toks1, _ = O.beam_search(step_fn, prompt, 1, 4)
    for b in range(2):
        last, greedy = prompt[b, -1], []
        for _ in range(4):
            last = int(np.argmax(table[last]))
            greedy.append(last)
        assert list(toks1[b]) == greedy
    # a narrow beam can miss the optimum but never beats it
    toks2, score2 = O.beam_search(step_fn, prompt, 2, T)
    assert (score2 <= score + 1e-12).all()
    # with an end token: what comes back is a closed hypothesis (scored at its length without the end token) or an
    # open beam, and its score is the one recomputed from the table
    eos = 4
    toks3, score3 = O.beam_search(step_fn, prompt, 3, 6, eos=eos, pad_token=-1)
    for b in range(2):
        seq = [t for t in toks3[b] if t != -1]
        assert eos not in seq
        last, total = prompt[b, -1], 0.0
        for t in seq:
            total += logp[last, t]
            last = t
        closed = total + logp[last, eos]
        cands = [closed / (2 + len(seq))] + ([total / (2 + len(seq))] if len(seq) == 6 else [])
        assert min(abs(score3[b] - c) for c in cands) < 1e-9


def test_beam_search_cache_reorder_matches_cacheless_model():
    """The oracle decoder under beam search (KV caches gathered by the source-beam index at every step) against
    the same search over the independent model that recomputes every beam's whole sequence without a cache."""
    hf, orc, rng = make_model(19, batch=6, cap=24)
    ids = rng.integers(0, 96, (2, 4))
    hist = {}

    def cacheless(x, first, reorder):
        hist["ids"] = x if first else np.concatenate([hist["ids"][reorder], x], axis=1)
        return hf.logits(hist["ids"])[:, -1]
    want_t, want_s = O.beam_search(cacheless, ids, 3, 6)
    got_t, got_s = orc.beam_search(ids, 3, 6)
    assert np.array_equal(got_t, want_t)
    assert np.abs(got_s - want_s).max() < 2e-2
