"""CPU oracle: fp32 restatements of every op on the int8 decode path.
TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

All functions take / return numpy arrays.  Buffers that the reference keeps in
fp16 are rounded to fp16 at the same op boundaries; arithmetic inside an op is
fp32 (float64 where noted for the brute-force variants used to pin the fp32 ones).
"""
import math

import numpy as np

F32 = np.float32
F16 = np.float16


# ----------------------------------------------------------------------------
# int8 weight-only linear
# ----------------------------------------------------------------------------
def dequant_matmul(x, q, scale, out_dtype=F16):
    """C = A . (float(q) * float(scale)), fp32 accumulate, one rounding to fp16.

    The grading form: dequantise-then-matmul in fp32.  Reference call sites:
    csrc/op/llama_mmha.cpp:313-337, 428-447; csrc/op/gated_ffn_int8.cpp:253-326
    (bias = nullptr, no activation).  The reference kernel itself rounds each
    dequantised weight to fp16 before the MMA
    (cutlass_extensions/.../mma_tensorop_dequantizer.h:258-275), which stays inside
    the tolerance of the grading form and is not restated.
    x: [M, K] fp16, q: [K, N] int8, scale: [N] fp16.
    """
    wd = q.astype(F32) * scale.astype(F32)[None, :]
    y = x.astype(F32) @ wd
    return y.astype(out_dtype)


# ----------------------------------------------------------------------------
# glue ops
# ----------------------------------------------------------------------------
def rmsnorm(x, gamma, eps):
    """x * rsqrt(mean(x^2) + eps) * gamma in fp32, fp16 out.
    csrc/core/layer_norm.cu:490-531 (T5norm1_kernel_opt, half)."""
    xf = x.astype(F32)
    var = np.mean(xf * xf, axis=-1, keepdims=True, dtype=F32)
    inv = (F32(1.0) / np.sqrt(var + F32(eps))).astype(F32)
    return (xf * inv * gamma.astype(F32)).astype(F16)


def rope_coeff(pos, dh):
    """cos/sin table row for one position.  csrc/core/common.cuh:176-180:
    angle_i = pos / 10000^(2i/dh), i in [0, dh/2), computed in fp32."""
    i = np.arange(dh // 2, dtype=F32)
    inv = (F32(pos) / np.power(F32(10000.0), (2 * i) / F32(dh), dtype=F32)).astype(F32)
    return np.cos(inv, dtype=F32), np.sin(inv, dtype=F32)


def rope_neox(x, pos):
    """NeoX-style rotation of pairs (i, i + dh/2).  csrc/core/common.cuh:209-225,
    csrc/core/self_add_bias.cu:369-403.  x: [..., dh] fp16; pos: int."""
    dh = x.shape[-1]
    c, s = rope_coeff(pos, dh)
    x1 = x[..., : dh // 2].astype(F32)
    x2 = x[..., dh // 2:].astype(F32)
    return np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], axis=-1).astype(F16)


def qkv_split(qkv, B, S, H, dh, rope, time_step=-1):
    """Split a fused [B, S, 3*H*dh] row into q, k, v [B, H, S, dh]; with
    rope=True rotate q and k at position seq index (prefill, time_step=-1) or
    time_step (decode).  self_add_bias.cu:369-403 (:393 for the position) and
    :278-301 (no rotation, Baichuan)."""
    x = qkv.reshape(B, S, 3, H, dh)
    q = np.transpose(x[:, :, 0], (0, 2, 1, 3)).copy()
    k = np.transpose(x[:, :, 1], (0, 2, 1, 3)).copy()
    v = np.transpose(x[:, :, 2], (0, 2, 1, 3)).copy()
    if rope:
        for s in range(S):
            pos = s if time_step == -1 else time_step
            q[:, :, s] = rope_neox(q[:, :, s], pos)
            k[:, :, s] = rope_neox(k[:, :, s], pos)
    return q, k, v


def layernorm(x, gamma, beta, eps):
    """(x - mean) * rsqrt(var + eps) * gamma + beta, fp32 statistics (variance of the centred
    values over n), fp16 out.  csrc/core/layer_norm.cu:384-446 (decoder_norm1_kernel_opt, half)."""
    xf = x.astype(F32)
    mean = np.mean(xf, axis=-1, keepdims=True, dtype=F32)
    d = xf - mean
    var = np.mean(d * d, axis=-1, keepdims=True, dtype=F32)
    inv = (F32(1.0) / np.sqrt(var + F32(eps))).astype(F32)
    return (d * inv * gamma.astype(F32) + beta.astype(F32)).astype(F16)


def add_bias(out, bias):
    """out + bias in fp16.  csrc/core/add_bias.cu:5-11."""
    return (out.astype(F16) + bias.astype(F16)[None, :]).astype(F16)


def add_bias_residual_norm(out, inp, bias, gamma, beta, eps):
    """Post-layernorm tail of the feed-forward op: y = (out + inp) [+ bias] with fp16 adds, then
    LayerNorm(gamma, beta) when a bias is given, RMSnorm(gamma) otherwise.
    csrc/core/layer_norm.cu:39-80 (add_bias_input_layernorm, half), :103-131 (add_input_RMSnorm,
    half); selected by bias != nullptr at :650-666."""
    y = residual_add(out, inp)
    if bias is not None:
        return layernorm(add_bias(y, bias), gamma, beta, eps)
    return rmsnorm(y, gamma, eps)


def swiglu(gate, up):
    """up * gate / (1 + exp(-gate)).  csrc/core/activation_kernel.cu:106-124.
    (The reference does the multiply / divide in half2; here once in fp32.)"""
    g = gate.astype(F32)
    return (up.astype(F32) * g / (F32(1.0) + np.exp(-g, dtype=F32))).astype(F16)


def residual_add(out, inp):
    """out + inp in fp16.  csrc/core/add_bias.cu:22-28."""
    return (out.astype(F16) + inp.astype(F16)).astype(F16)


# ----------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------
def decode_attention(q, k_new, v_new, k_cache, v_cache, step, pad=None, alibi=None, dtype=F32):
    """Masked multi-head attention for one new token over the KV cache.

    Follows csrc/core/attention_dispatch.cu:140-324 (masked_attention_kernel_opt)
    and :1155-1336 (t5_masked_attention_kernel, the ALiBi variant):
      * the new k, v are written to cache row step-1                    (:221-228, :283-291)
      * logit_t = sum_d q_d * k_td * (1/sqrt(dh))                       (:229-233); scale cast to T (:897)
      * rows t < pad get -1e20 (=> weight 0)                            (:219-220)
      * ALiBi: logit_t += bias[h, t]                                    (:1249)
      * p = exp(l - max) / (sum + 1e-6)                                 (:257-272)
      * ctx = sum_t p_t * v_t, fp16 out                                 (:279-323)
    The reference rounds each logit to fp16 (:238) and adds the ALiBi term in fp16;
    here both stay in fp32 (strictly more accurate, inside the tolerance).

    q, k_new, v_new: [B, H, dh] fp16.  k_cache, v_cache: [B, H, T, dh] fp16,
    updated in place.  pad: [B] ints or None.  alibi: [H, step] fp16 or None.
    Returns ctx [B, H*dh] fp16.
    """
    B, H, dh = q.shape
    k_cache[:, :, step - 1] = k_new
    v_cache[:, :, step - 1] = v_new
    scalar = dtype(F16(1.0 / math.sqrt(dh)))  # (T)(1/sqrtf(dh)), T = half
    K = k_cache[:, :, :step].astype(dtype)
    V = v_cache[:, :, :step].astype(dtype)
    logits = np.einsum("bhd,bhtd->bht", q.astype(dtype), K).astype(dtype) * scalar
    if alibi is not None:
        logits = logits + alibi[None, :, :step].astype(dtype)
    if pad is not None:
        t = np.arange(step)[None, None, :]
        logits = np.where(t < np.asarray(pad).reshape(B, 1, 1), dtype(-np.inf), logits)
    m = np.max(logits, axis=-1, keepdims=True)
    m = np.where(np.isinf(m), dtype(0.0), m)  # everything padded away: weights 0, ctx 0
    e = np.exp(logits - m)
    p = e / (np.sum(e, axis=-1, keepdims=True) + dtype(1e-6))
    ctx = np.einsum("bht,bhtd->bhd", p, V)
    return ctx.reshape(B, H * dh).astype(F16)


def prefill_attention(q, k, v, pad=None, alibi=None):
    """Causal attention over the prompt, fp32.

    Follows the reference's unfused prefill: QK^T * (1/sqrt(dh)) (fp16 GEMM,
    csrc/op/llama_mmha.cpp:354-373), softmax_kernel_gpt2 (causal, left-pad
    columns -1e20, left-pad query rows zeroed, denominator + 1e-6;
    csrc/core/gpt2_self_softmax.cu:8-56) or, with ALiBi, masked_softmax_kernel
    (bias[h, i, j] added, no padding handling; :161-188), then P.V
    (llama_mmha.cpp:397-416).  q, k, v: [B, H, S, dh] fp16.  alibi: [H, S, S].
    Returns ctx [B, S, H*dh] fp16.
    """
    B, H, S, dh = q.shape
    scalar = F32(F16(math.sqrt(1.0 / dh)))
    logits = np.einsum("bhid,bhjd->bhij", q.astype(F32), k.astype(F32)) * scalar
    if alibi is not None:
        a = alibi.astype(F32)
        logits = logits + np.where(np.isinf(a), F32(0.0), a)[None]
    i = np.arange(S)[:, None]
    j = np.arange(S)[None, :]
    mask = (j > i)[None, None]
    if pad is not None:
        padv = np.asarray(pad).reshape(B, 1, 1, 1)
        mask = mask | (j[None, None] < padv)
    logits = np.where(mask, F32(-np.inf), logits)
    m = np.max(logits, axis=-1, keepdims=True)
    m = np.where(np.isinf(m), F32(0.0), m)
    e = np.exp(logits - m)
    p = e / (np.sum(e, axis=-1, keepdims=True) + F32(1e-6))
    if pad is not None:
        p = np.where(i[None, None] < padv, F32(0.0), p)
    ctx = np.einsum("bhij,bhjd->bhid", p.astype(F32), v.astype(F32))
    return np.transpose(ctx, (0, 2, 1, 3)).reshape(B, S, H * dh).astype(F16)


def alibi_slopes(n):
    """python/eet/transformers/modeling_baichuan.py:51-65 (_get_interleave)."""
    def pow2(n):
        start = 2 ** (-(2 ** -(math.log2(n) - 3)))
        return [start * start ** i for i in range(n)]
    if math.log2(n).is_integer():
        return pow2(n)
    c = 2 ** math.floor(math.log2(n))
    return pow2(c) + alibi_slopes(2 * c)[0::2][: n - c]


def alibi_bias(n_head, length):
    """The decode-time bias row the Baichuan caller passes: slope_h * j for
    j < length, built in fp32 and cast to fp16
    (modeling_baichuan.py:71-80, 270-281, 308-317).  Returns [n_head, length] fp16."""
    slopes = np.asarray(alibi_slopes(n_head), dtype=F32)
    j = np.arange(length, dtype=F32)
    return (slopes[:, None] * j[None, :]).astype(F32).astype(F16)


def alibi_mask(n_head, length):
    """Prefill mask [n_head, S, S]: slope_h * j, -inf above the diagonal, fp16."""
    b = alibi_bias(n_head, length).astype(F32)
    m = np.broadcast_to(b[:, None, :], (n_head, length, length)).copy()
    iu = np.triu_indices(length, 1)
    m[:, iu[0], iu[1]] = -np.inf
    return m.astype(F16)


# ----------------------------------------------------------------------------
# layer / decoder composition
# ----------------------------------------------------------------------------
def reorder_cache(k_cache, v_cache, index, rows):
    """Beam-search gather: beam b takes over the first `rows` time steps of beam
    index[b].  csrc/core/transpose.cu:135-152 (reorderKV) as called from
    csrc/op/llama_mmha.cpp:248-252; the gather is taken from a snapshot, which is
    what that in-place kernel means to compute.  Caches [B][H][T][dh]."""
    ks, vs = k_cache.copy(), v_cache.copy()
    for b, src in enumerate(index):
        k_cache[b, :, :rows] = ks[src, :, :rows]
        v_cache[b, :, :rows] = vs[src, :, :rows]


class OracleAttention:
    """LlamaMmha / BaichuanMmha restated.  csrc/op/llama_mmha.cpp:114-266,
    csrc/op/baichuan_mmha.cpp:81-216.  Weights are the *unprocessed* int8
    [K, N] matrices plus fp16 scales."""

    def __init__(self, B, H, dh, cap, qkv_q, qkv_s, o_q, o_s, gamma, eps, rope=True, qkv_bias=None, o_bias=None,
                 beta=None):
        """qkv_bias [3 * H * dh] (q | k | v), beta: the bias branch of BaichuanMmha -- with a Q bias the op
        normalises with LayerNorm(gamma, beta) instead of RMSnorm (csrc/op/baichuan_mmha.cpp:45, 224-231)
        and adds the biases to the fused QKV rows in fp16 (:295-297, csrc/core/self_add_bias.cu:352-354);
        o_bias is added after the residual (:402, csrc/core/add_bias.cu:13-20)."""
        self.H, self.dh, self.rope, self.eps = H, dh, rope, eps
        self.qkv_q, self.qkv_s, self.o_q, self.o_s, self.gamma = qkv_q, qkv_s, o_q, o_s, gamma
        self.qkv_bias, self.o_bias, self.beta = qkv_bias, o_bias, beta
        self.k_cache = np.zeros((B, H, cap, dh), F16)
        self.v_cache = np.zeros((B, H, cap, dh), F16)
        self.step = 1

    def forward(self, x, pad, first_pass, alibi=None, reorder=None):
        B, S, hidden = x.shape
        H, dh = self.H, self.dh
        if reorder is not None and not first_pass:
            reorder_cache(self.k_cache, self.v_cache, reorder, self.step)
        if self.qkv_bias is not None:
            xn = layernorm(x.reshape(B * S, hidden), self.gamma, self.beta, self.eps)
            qkv = add_bias(dequant_matmul(xn, self.qkv_q, self.qkv_s), self.qkv_bias)
        else:
            xn = rmsnorm(x.reshape(B * S, hidden), self.gamma, self.eps)
            qkv = dequant_matmul(xn, self.qkv_q, self.qkv_s)
        if first_pass:
            q, k, v = qkv_split(qkv, B, S, H, dh, self.rope, -1)
            self.k_cache[:B, :, :S] = k
            self.v_cache[:B, :, :S] = v
            ctx = prefill_attention(q, k, v, pad, alibi)
            self.step = S
        else:
            assert S == 1
            self.step += 1
            q, k, v = qkv_split(qkv, B, 1, H, dh, self.rope, self.step - 1)
            ctx = decode_attention(q[:, :, 0], k[:, :, 0], v[:, :, 0], self.k_cache[:B], self.v_cache[:B],
                                   self.step, pad, alibi)
        out = residual_add(dequant_matmul(ctx.reshape(B * S, H * dh), self.o_q, self.o_s), x.reshape(B * S, hidden))
        if self.o_bias is not None:
            out = add_bias(out, self.o_bias)
        return out.reshape(B, S, hidden)


class OracleFFN:
    """GatedFeedForwardNetworkInt8 restated.  csrc/op/gated_ffn_int8.cpp:98-132."""

    def __init__(self, g_q, g_s, u_q, u_s, d_q, d_s, gamma, eps, beta=None, o_bias=None):
        """beta: with a layernorm bias the op normalises with LayerNorm (gated_ffn_int8.cpp:139-146);
        o_bias: the output bias (:328-357).  The two intermediate biases the constructor takes are never
        read by the reference's forward (:98-132), so they have no place here."""
        self.g_q, self.g_s, self.u_q, self.u_s, self.d_q, self.d_s = g_q, g_s, u_q, u_s, d_q, d_s
        self.gamma, self.eps, self.beta, self.o_bias = gamma, eps, beta, o_bias

    def forward(self, x, pre_layernorm=True, add_residual=True):
        B, S, hidden = x.shape
        x2 = x.reshape(B * S, hidden)
        # the norm in front is applied in both modes (:112)
        xn = layernorm(x2, self.gamma, self.beta, self.eps) if self.beta is not None else rmsnorm(x2, self.gamma, self.eps)
        act = swiglu(dequant_matmul(xn, self.g_q, self.g_s), dequant_matmul(xn, self.u_q, self.u_s))
        out = dequant_matmul(act, self.d_q, self.d_s)
        if add_residual and not pre_layernorm:       # post-layernorm mode (:335-342)
            out = add_bias_residual_norm(out, x2, self.o_bias, self.gamma, self.beta, self.eps)
        elif add_residual:                           # (:343-347)
            out = residual_add(out, x2)
            if self.o_bias is not None:
                out = add_bias(out, self.o_bias)
        elif self.o_bias is not None:                # (:349-355)
            out = add_bias(out, self.o_bias)
        return out.reshape(B, S, hidden)


class OracleDecoder:
    """Embedding -> layers -> final RMSnorm -> fp16 lm_head, greedy decode.
    python/eet/transformers/modeling_llama.py:161-297, 452-471;
    python/eet/pipelines/generation.py:1144-1218 (argmax loop)."""

    def __init__(self, embed, layers, final_gamma, lm_head, eps, n_head=None, alibi=False):
        self.embed, self.layers, self.final_gamma, self.lm_head, self.eps = embed, layers, final_gamma, lm_head, eps
        self.alibi, self.n_head, self.past = alibi, n_head, 0

    def step(self, ids, first_pass, pad=None, reorder=None):
        x = self.embed[ids]
        B, S, _ = x.shape
        bias = None
        if self.alibi:
            self.past = S if first_pass else self.past + 1
            bias = alibi_mask(self.n_head, self.past) if first_pass else alibi_bias(self.n_head, self.past)
        for attn, ffn in self.layers:
            x = ffn.forward(attn.forward(x, pad, first_pass, bias, reorder))
        x = rmsnorm(x, self.final_gamma, self.eps)
        return (x[:, -1].astype(F32) @ self.lm_head.astype(F32).T)

    def greedy(self, ids, n_new, pad=None):
        out = []
        logits = self.step(ids, True, pad)
        for _ in range(n_new):
            nxt = np.argmax(logits, axis=-1)
            out.append(nxt)
            logits = self.step(nxt[:, None], False, pad)
        return np.stack(out, axis=1)


    def beam_search(self, ids, num_beams, n_new, eos=None, pad_token=0, length_penalty=1.0):
        """python/eet/pipelines/generation.py:1379-1680 with the beam scorer of :960-975, restated for the
        checker: rows [b * num_beams + k]; scores accumulate log-softmax values; 2 * num_beams candidates per
        prompt in score order; an end-of-sequence candidate ranked inside the first num_beams closes a
        hypothesis scored sum / length ** length_penalty (length with the prompt); the source beams are
        handed to the layers as the cache reorder of the next step (:1577)."""
        return beam_search(lambda x, first, reorder: self.step(x, first, None, reorder), ids, num_beams, n_new, eos,
                           pad_token, length_penalty)


def beam_search(step_fn, ids, nb, n_new, eos=None, pad_token=0, length_penalty=1.0):
    """The search itself over any next-token function step_fn(ids [rows, S], first_pass, reorder) -> logits
    [rows, V] (so that tests can pin it with an exhaustive search over a small vocabulary)."""
    B, S = ids.shape
    rows = np.repeat(ids, nb, axis=0)
    score = np.zeros((B, nb), np.float64)
    score[:, 1:] = -1e9
    gen = np.zeros((B * nb, 0), np.int64)
    closed = [[] for _ in range(B)]
    done = np.zeros(B, bool)
    logits = step_fn(rows, True, None)
    for t in range(n_new):
        z = logits.astype(np.float64)
        z = z - z.max(-1, keepdims=True)
        logp = z - np.log(np.exp(z).sum(-1, keepdims=True)) + score.reshape(-1, 1)
        V = logp.shape[-1]
        flat = logp.reshape(B, nb * V)
        order = np.argsort(-flat, axis=1, kind="stable")[:, : 2 * nb]
        length = S + t
        new_score = np.zeros((B, nb))
        new_tok = np.full((B, nb), pad_token, np.int64)
        new_src = np.zeros((B, nb), np.int64)
        for b in range(B):
            if done[b]:
                continue
            kept = 0
            for rank, cand in enumerate(order[b]):
                beam, tok, sc = cand // V, cand % V, flat[b, cand]
                if eos is not None and tok == eos:
                    if rank < nb:
                        closed[b].append((sc / length ** length_penalty, gen[b * nb + beam].copy()))
                    continue
                new_score[b, kept], new_tok[b, kept], new_src[b, kept] = sc, tok, beam
                kept += 1
                if kept == nb:
                    break
            if len(closed[b]) >= nb:
                closed[b] = sorted(closed[b], key=lambda h: -h[0])[:nb]
                done[b] = closed[b][-1][0] >= flat[b, order[b, 0]] / (length + 1) ** length_penalty
        score = new_score
        src_rows = (np.arange(B)[:, None] * nb + new_src).reshape(-1)
        gen = np.concatenate([gen[src_rows], new_tok.reshape(-1, 1)], axis=1)
        if done.all() or t == n_new - 1:
            break
        logits = step_fn(new_tok.reshape(-1, 1), False, src_rows)
    out = np.full((B, n_new), pad_token, np.int64)
    best = np.zeros(B)
    for b in range(B):
        hyps = list(closed[b])
        if not done[b]:
            hyps += [(score[b, k] / (S + gen.shape[1]) ** length_penalty, gen[b * nb + k]) for k in range(nb)]
        sc, toks = max(hyps, key=lambda h: h[0])
        out[b, : len(toks)] = toks
        best[b] = sc
    return out, best
