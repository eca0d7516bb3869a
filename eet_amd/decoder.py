"""Caller of the operator API: a LLaMA- / Baichuan-shaped int8 decoder assembled
from the ops exactly as the reference's Python model code assembles it, plus
the greedy loop that drives it.

Counterpart of python/eet/transformers/modeling_llama.py:51-297, 452-471
(EETLlamaSelfMaskedAttention ... EETLlamaForCausalLM), modeling_baichuan.py:
51-80, 270-317 (ALiBi mask) and pipelines/generation.py:1144-1218 (greedy
search).  Embedding and lm_head stay fp16 torch ops, as in the reference
(modeling_llama.py:370-372, 471).
"""
import math
from dataclasses import dataclass

import torch

from . import convert, ops


@dataclass
class DecoderConfig:
    num_layers: int = 32
    hidden: int = 4096
    heads: int = 32
    d_ff: int = 11008
    vocab: int = 32000
    eps: float = 1e-6
    alibi: bool = False          # False: rotary (LLaMA); True: ALiBi (Baichuan-13B)
    max_batch: int = 8
    max_prompt: int = 1024
    max_full_seq: int = 1153

    @staticmethod
    def llama_7b(**kw):
        return DecoderConfig(**kw)

    @staticmethod
    def baichuan_13b(**kw):
        d = dict(num_layers=40, hidden=5120, heads=40, d_ff=13696, vocab=64000, alibi=True, max_batch=32,
                 max_prompt=2048, max_full_seq=2305)
        d.update(kw)
        return DecoderConfig(**d)


# ---- ALiBi (modeling_baichuan.py:51-80) ------------------------------------
def alibi_slopes(n):
    def pow2(n):
        start = 2 ** (-(2 ** -(math.log2(n) - 3)))
        return [start * start ** i for i in range(n)]
    if math.log2(n).is_integer():
        return pow2(n)
    c = 2 ** math.floor(math.log2(n))
    return pow2(c) + alibi_slopes(2 * c)[0::2][: n - c]


def alibi_mask(n_head, max_pos, dtype=torch.float16, device="cpu"):
    """[n_head, max_pos, max_pos]: slope_h * j, -inf above the diagonal; built
    in fp32 and cast (the `.to(tensor)` at modeling_baichuan.py:273)."""
    slopes = torch.tensor(alibi_slopes(n_head), dtype=torch.float32)
    alibi = slopes[:, None, None] * torch.arange(max_pos, dtype=torch.float32)[None, None, :]
    mask = torch.triu(torch.full((max_pos, max_pos), float("-inf")), 1)
    return (mask[None] + alibi).to(dtype).to(device)


# ---- random-init weights in the reference's state-dict naming ----------------
def random_state_dict(cfg, seed=1234, quant_mode="ref128"):
    """Seeded synthetic weights: W ~ N(0, 0.02^2) quantised per output channel,
    gamma = 1 + 0.1 N(0,1).  Keys follow convert_llama_weights
    (modeling_llama.py:739-784): 'layer.N.self_attn.qkv_proj.weight' holds the
    processed int8 [K, N], '.scale' the fp16 scales.  Also returns the
    unprocessed int8 matrices for checking."""
    g = torch.Generator().manual_seed(seed)
    H, F = cfg.hidden, cfg.d_ff
    sd, raw = {}, {}

    def lin(name, K, N):
        w = (torch.randn(K, N, generator=g) * 0.02).half()
        u, p, s = ops.quant_weights(w, torch.int8, True, mode=quant_mode)
        sd[name + ".weight"], sd[name + ".scale"] = p, s
        raw[name] = (u, s)

    for i in range(cfg.num_layers):
        pre = f"layer.{i}."
        lin(pre + "self_attn.qkv_proj", H, 3 * H)
        lin(pre + "self_attn.out_proj", H, H)
        lin(pre + "ffn.intermediate_0", H, F)
        lin(pre + "ffn.intermediate_1", H, F)
        lin(pre + "ffn.output", F, H)
        sd[pre + "self_attn.layernorm.weight"] = (1 + 0.1 * torch.randn(H, generator=g)).half()
        sd[pre + "ffn.layernorm.weight"] = (1 + 0.1 * torch.randn(H, generator=g)).half()
    sd["embed_tokens.weight"] = (torch.randn(cfg.vocab, H, generator=g) * 0.02).half()
    sd["norm.weight"] = (1 + 0.1 * torch.randn(H, generator=g)).half()
    sd["lm_head.weight"] = (torch.randn(cfg.vocab, H, generator=g) * 0.02).half()
    return sd, raw


class Int8Decoder:
    """Embedding -> num_layers x (attention op, gated-FFN op) -> final RMSnorm
    -> lm_head.  Construction order and arguments of the ops are those of
    EETLlamaSelfMaskedAttention / EETGatedFeedForward (modeling_llama.py:51-146)."""

    def __init__(self, cfg, state_dict, device="cuda:0"):
        self.cfg = cfg
        convert.check_layout(state_dict)
        dev = torch.device(device)
        self.desc = ops.MetaDesc(dtype=torch.float16, batch_size=cfg.max_batch, head_num=cfg.heads,
                                 hidden_units=cfg.hidden, layer_num=cfg.num_layers, max_seq_len=cfg.max_prompt,
                                 max_full_seq_len=cfg.max_full_seq, activation_fn="silu", d_kv=0, d_ff=cfg.d_ff,
                                 cuda_device=str(dev), layernorm_eps=cfg.eps, is_int8=True)
        e = torch.empty(0)
        attn_cls = ops.BaichuanMmha if cfg.alibi else ops.LlamaMmha
        self.layers = []
        for i in range(cfg.num_layers):
            pre = f"layer.{i}."
            t = {k: state_dict[pre + k].to(dev) for k in (
                "self_attn.qkv_proj.weight", "self_attn.qkv_proj.scale", "self_attn.out_proj.weight",
                "self_attn.out_proj.scale", "self_attn.layernorm.weight", "ffn.intermediate_0.weight",
                "ffn.intermediate_0.scale", "ffn.intermediate_1.weight", "ffn.intermediate_1.scale",
                "ffn.output.weight", "ffn.output.scale", "ffn.layernorm.weight")}
            attn = attn_cls(self.desc, t["self_attn.qkv_proj.weight"], t["self_attn.qkv_proj.scale"], e, e, e,
                            t["self_attn.out_proj.weight"], t["self_attn.out_proj.scale"], e,
                            t["self_attn.layernorm.weight"], e)
            ffn = ops.GatedFeedForwardNetworkInt8(
                self.desc, t["ffn.intermediate_0.weight"], t["ffn.intermediate_0.scale"], e,
                t["ffn.intermediate_1.weight"], t["ffn.intermediate_1.scale"], e, t["ffn.output.weight"],
                t["ffn.output.scale"], e, t["ffn.layernorm.weight"], e, "decoder_out_cache")
            self.layers.append((attn, ffn))
        self.embed = state_dict["embed_tokens.weight"].to(dev)
        self.norm_w = state_dict["norm.weight"].to(dev)
        self.final_norm = ops.LayerNorm(self.desc, self.norm_w, e)
        self.lm_head = state_dict["lm_head.weight"].to(dev)
        self.pre_padding_len = torch.empty(0, dtype=torch.long)
        self.reorder_state = torch.empty(0, dtype=torch.long)
        self.past = 0
        self._mask = None

    def _alibi(self, first_pass, like):
        cfg = self.cfg
        if self._mask is None:
            # Only rows of the [H, P, P] mask are ever used (row i is slope*j, j <= i),
            # so the table is kept as [H, P] and expanded on demand.
            slopes = torch.tensor(alibi_slopes(cfg.heads), dtype=torch.float32)
            self._mask = (slopes[:, None] * torch.arange(cfg.max_full_seq, dtype=torch.float32)[None, :]
                          ).to(torch.float16).to(like.device)
        L = self.past
        if first_pass:
            # the op reads the last row of the [H, S, S] mask; hand it that row as a [H, 1->S, S] view
            return self._mask[:, None, :L].expand(cfg.heads, L, L)
        if ops.replay_state is not None:
            return self._mask[:, None, :]         # the whole table: the kernel reads the step itself
        return self._mask[:, None, :L].contiguous()

    def __call__(self, input_ids, first_pass=True, attention_mask=None):
        """modeling_llama.py:262-297 / modeling_baichuan.py:283-333.  Returns the
        normalised hidden states [B, S, hidden]."""
        cfg = self.cfg
        B, S = input_ids.shape
        assert B <= cfg.max_batch and S <= cfg.max_prompt
        if attention_mask is None:
            pad = self.pre_padding_len
        else:
            pad = torch.sum(1 - attention_mask, 1, True).to(input_ids.device).long()
        x = ops._timed("embedding (torch)", 2 * B * S * cfg.hidden * 2,
                       lambda: torch.nn.functional.embedding(input_ids, self.embed))
        bias = torch.empty(0)
        if cfg.alibi:
            self.past = S if first_pass else self.past + S
            bias = self._alibi(first_pass, x)
        for attn, ffn in self.layers:
            x = attn.forward(x, pad, self.reorder_state, True, True, first_pass, bias)
            x = ffn.forward(x, True, True)
        return ops._timed("final_rmsnorm", 2 * B * S * cfg.hidden * 2, lambda: self.final_norm.layer_norm(x))

    def logits(self, input_ids, first_pass=True, attention_mask=None):
        h = self(input_ids, first_pass, attention_mask)
        B = h.shape[0]
        return ops._timed("lm_head fp16 (torch)", self.lm_head.numel() * 2 + B * (self.cfg.hidden + self.cfg.vocab) * 2,
                          lambda: torch.nn.functional.linear(h[:, -1:, :], self.lm_head))

    @torch.no_grad()
    def greedy(self, input_ids, max_new_tokens, attention_mask=None):
        """Prefill with the whole prompt, then one token per call: argmax of the
        last position (generation.py:1144-1218).  Returns [B, max_new_tokens]."""
        out = []
        logits = self.logits(input_ids, True, attention_mask)
        for i in range(max_new_tokens):
            nxt = torch.argmax(logits[:, -1, :], dim=-1)
            out.append(nxt)
            if i + 1 < max_new_tokens:
                logits = self.logits(nxt[:, None], False, attention_mask)
        return torch.stack(out, dim=1)

    # ---- beam search ----------------------------------------------------------------------------
    @torch.no_grad()
    def beam_search(self, input_ids, num_beams, max_new_tokens, eos_token_id=None, pad_token_id=0,
                    length_penalty=1.0):
        """Beam search over the decoder (pipelines/generation.py:1379-1680 with the stock beam scorer the
        reference instantiates at :960-975): every prompt is expanded to num_beams rows; each step takes
        the log-softmax of the last position, adds the running beam scores, keeps the best 2 * num_beams
        (beam, token) pairs per prompt in score order, turns end-of-sequence candidates among the first
        num_beams ranks into finished hypotheses (score = sum of log-probabilities / length ** length_penalty,
        the length counting the prompt) and continues with the first num_beams others.  The beam each
        continuation came from is handed to the attention ops as reorder_state with the next call
        (generation.py:1577), which gathers their KV caches (csrc/op/llama_mmha.cpp:248-252).
        Returns (tokens [B, <= max_new_tokens] padded with pad_token_id, scores [B])."""
        cfg = self.cfg
        B, S = input_ids.shape
        nb = int(num_beams)
        if nb < 1 or B * nb > cfg.max_batch:
            raise RuntimeError(f"[EET][ERROR] beam_search: batch {B} x num_beams {nb} exceeds max_batch {cfg.max_batch}")
        dev = input_ids.device
        ids = input_ids.repeat_interleave(nb, 0)                                   # [B * nb, S]
        beam_scores = torch.zeros(B, nb, dtype=torch.float32, device=dev)
        beam_scores[:, 1:] = -1e9                                                  # only the first copy counts at step 0
        gen = torch.empty(B * nb, 0, dtype=torch.long, device=dev)
        finished = [[] for _ in range(B)]                                          # per prompt: (score, tokens)
        done = [False] * B
        self.reorder_state = torch.empty(0, dtype=torch.long)
        try:
            logits = self.logits(ids, True)
            for step in range(max_new_tokens):
                logp = torch.log_softmax(logits[:, -1, :].float(), dim=-1) + beam_scores.view(-1, 1)
                V = logp.shape[-1]
                top_s, top_i = torch.topk(logp.view(B, nb * V), 2 * nb, dim=1, largest=True, sorted=True)
                top_s, src, tok = top_s.cpu(), (top_i // V).cpu(), (top_i % V).cpu()
                gen_host = gen.cpu()
                cur_len = S + step                                                 # tokens before this step's
                nxt_s = torch.zeros(B, nb)
                nxt_t = torch.full((B, nb), pad_token_id, dtype=torch.long)
                nxt_b = torch.zeros(B, nb, dtype=torch.long)
                for b in range(B):
                    if done[b]:
                        continue
                    k = 0
                    for rank in range(2 * nb):
                        sc, sb, tk = float(top_s[b, rank]), int(src[b, rank]), int(tok[b, rank])
                        if eos_token_id is not None and tk == eos_token_id:
                            if rank < nb:                                          # an end among the best num_beams
                                finished[b].append((sc / (cur_len ** length_penalty), gen_host[b * nb + sb].clone()))
                            continue
                        nxt_s[b, k], nxt_t[b, k], nxt_b[b, k] = sc, tk, sb
                        k += 1
                        if k == nb:
                            break
                    if len(finished[b]) >= nb:
                        finished[b] = sorted(finished[b], key=lambda h: -h[0])[:nb]
                        best_open = float(top_s[b].max()) / ((cur_len + 1) ** length_penalty)
                        done[b] = finished[b][-1][0] >= best_open
                beam_scores = nxt_s.to(dev)
                beam_idx = (torch.arange(B)[:, None] * nb + nxt_b).view(-1).to(dev)
                gen = torch.cat([gen[beam_idx], nxt_t.view(-1, 1).to(dev)], dim=1)
                if all(done) or step == max_new_tokens - 1:
                    break
                self.reorder_state = beam_idx                                      # the ops gather their caches
                logits = self.logits(nxt_t.view(-1, 1).to(dev), False)
        finally:
            self.reorder_state = torch.empty(0, dtype=torch.long)
        gen_host, scores_host = gen.cpu(), beam_scores.cpu()
        out = torch.full((B, max_new_tokens), pad_token_id, dtype=torch.long)
        best = torch.zeros(B)
        for b in range(B):
            hyps = list(finished[b])
            if not done[b]:                                                        # open beams count as they stand
                total = S + gen_host.shape[1]
                hyps += [(float(scores_host[b, k]) / (total ** length_penalty), gen_host[b * nb + k]) for k in range(nb)]
            sc, toks = max(hyps, key=lambda h: h[0])
            out[b, : toks.numel()] = toks
            best[b] = sc
        return out, best

    # ---- the incremental step as a HIP graph ---------------------------------------------------
    def _shift_host_steps(self, by):
        for attn, _ in self.layers:
            attn.step += by
        if self.cfg.alibi:
            self.past += by

    def capture_decode_step(self, next_ids):
        """Records one incremental step (step counter advance, embedding, all layers, final norm,
        lm_head, argmax, feeding the token back) into a HIP graph, after a prompt has been
        processed eagerly.  next_ids [B] are the tokens the first replay consumes.  Returns a
        function that replays the step and returns the new tokens [B] (a static buffer).

        The graph holds raw device pointers.  Everything they point to is kept alive with the
        graph (the named workspaces handed out while recording, the KV caches, the static
        input / output buffers); a replay refuses to run when a layer's cache tensors are no
        longer the recorded ones (a beam reorder swaps them), and brings the device-side step
        back in line when eager calls or a new prompt moved the host-side step in between."""
        cfg, dev = self.cfg, self.embed.device
        if self.reorder_state is not None and self.reorder_state.numel() != 0:
            raise RuntimeError("[EET][ERROR] capture_decode_step: a decoder that reorders its KV cache (beam search) "
                               "cannot replay a recorded step: the reorder swaps the cache buffers the graph points to")
        B = next_ids.shape[0]
        lib = ops.lib()
        step_dev = torch.tensor([self.layers[0][0].step], dtype=torch.int32, device=dev)
        ids = next_ids.reshape(B, 1).clone()
        out_tok = torch.zeros(B, dtype=torch.long, device=dev)
        ops.replay_state = ops.ReplayState(step_dev, cfg.max_full_seq)

        def one_step():
            ops.check(lib.eet_step_advance(step_dev.data_ptr(), 1, ops._stream()), "eet_step_advance")
            logits = self.logits(ids, False)
            out_tok.copy_(torch.argmax(logits[:, -1, :], dim=-1))
            ids.copy_(out_tok[:, None])
        try:
            with ops.workspaces.recording() as handed:
                # eager warm-up on a side stream (allocates every workspace), then undone: the cache row it
                # wrote is written again by the first replay
                keep = ids.clone()
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side), torch.no_grad():
                    one_step()
                    ops.check(lib.eet_step_advance(step_dev.data_ptr(), -1, ops._stream()), "eet_step_advance")
                    ids.copy_(keep)
                torch.cuda.current_stream().wait_stream(side)
                self._shift_host_steps(-1)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph), torch.no_grad():
                    one_step()
                self._shift_host_steps(-1)      # recording ran the host code once; no kernel has run
        finally:
            ops.replay_state = None
        caches = [(attn.k_cache, attn.v_cache) for attn, _ in self.layers]
        state = {"step": self.layers[0][0].step}     # what step_dev holds

        def replay(next_ids=None):
            """One recorded step.  next_ids [B]: the tokens to consume instead of the previous replay's output
            (needed after eager calls or a new prompt on this decoder)."""
            host_step = self.layers[0][0].step
            if host_step + 1 > cfg.max_full_seq:
                raise RuntimeError(f"[EET][ERROR] decode step {host_step + 1} exceeds max_full_seq "
                                   f"{cfg.max_full_seq}")
            if self.reorder_state is not None and self.reorder_state.numel() != 0:
                raise RuntimeError("[EET][ERROR] replay: reorder_state is set; a recorded step cannot reorder the cache")
            for (attn, _), (k, v) in zip(self.layers, caches):
                if attn.k_cache is not k or attn.v_cache is not v:
                    raise RuntimeError("[EET][ERROR] replay: a layer's KV cache is no longer the buffer this step was "
                                       "recorded with (beam reorder?): record the step again")
            if any(attn.step != host_step for attn, _ in self.layers):
                raise RuntimeError("[EET][ERROR] replay: the layers disagree about the current step")
            if host_step != state["step"]:
                # eager calls or a new prompt moved the host-side step since the last replay
                step_dev.fill_(host_step)
            if next_ids is not None:
                ids.copy_(next_ids.reshape(B, 1))
            graph.replay()
            self._shift_host_steps(1)
            state["step"] = host_step + 1
            return out_tok
        self._graph_keep = (graph, step_dev, ids, out_tok, handed, caches)
        replay.keep = self._graph_keep      # the closure owns what the graph points to
        return replay

    @torch.no_grad()
    def greedy_graph(self, input_ids, max_new_tokens, attention_mask=None):
        """greedy() with the incremental step replayed from a HIP graph."""
        logits = self.logits(input_ids, True, attention_mask)
        nxt = torch.argmax(logits[:, -1, :], dim=-1)
        out = [nxt]
        if max_new_tokens > 1:
            if attention_mask is not None:
                raise NotImplementedError("greedy_graph: left-padded batches run through greedy()")
            replay = self.capture_decode_step(nxt)
            for _ in range(max_new_tokens - 1):
                out.append(replay().clone())
        return torch.stack(out, dim=1)
