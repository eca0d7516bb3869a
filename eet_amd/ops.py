"""The reference's operator API (pybind module `EET`, csrc/py11/eet2py.cpp)
re-hosted on libeet_hip.so through ctypes.

Same names, positional argument order and state machine as the reference ops:
MetaDesc (eet2py.cpp:26-42), LlamaMmha (:73-86), BaichuanMmha (:58-71),
GatedFeedForwardNetworkInt8 (:126-134), LayerNorm (:143-145), quant_weights
(:152-155) and preprocess_weights (:148-150).  The ops of other model families
are exported as names that raise.

Differences that a caller can observe, all deliberate:
  * shapes and limits that the reference only `assert`s (compiled out) are
    checked and raise RuntimeError;
  * kernels run on torch's current stream, not on a private stream
    (csrc/op/meta_desc.hpp:58-60);
  * "processed" int8 weights are in the gfx950 tile layout
    (eet_pack_gfx950), not the sm80 cutlass layout;
  * outputs are views of per-process named torch buffers that own their
    storage (the reference returns from_blob views, llama_mmha.cpp:197-198).
"""
import torch

from ._lib import check, lib

_EMPTY = torch.empty(0)


def _ptr(t):
    return t.data_ptr() if t is not None and t.numel() > 0 else None


def _current_stream():
    """Handle of torch's current stream on the current device (the private
    accessor when torch has it: it costs a tenth of building a Stream object)."""
    try:
        return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())
    except AttributeError:
        return torch.cuda.current_stream().cuda_stream


def _stream():
    return _StreamScope.handle if _StreamScope.handle is not None else _current_stream()


class _StreamScope:
    """Looks torch's current stream up once per op call instead of once per kernel."""
    handle = None

    def __enter__(self):
        _StreamScope.handle = _current_stream()

    def __exit__(self, *a):
        _StreamScope.handle = None


# ----------------------------------------------------------------------------
# named persistent workspaces (the reference's MManager, csrc/op/mmanager.hpp:12-224)
# ----------------------------------------------------------------------------
class _Workspaces:
    def __init__(self):
        self._bufs = {}
        self._recorders = []

    def get(self, name, numel, dtype, device, zero=False):
        key = (name, str(device), dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < numel:
            alloc = torch.zeros if zero else torch.empty      # zero: a buffer whose first use needs zeros
            buf = alloc(max(int(numel), 1), dtype=dtype, device=device)
            self._bufs[key] = buf
        for handed in self._recorders:
            handed.append(buf)
        return buf

    def clear(self):
        self._bufs.clear()

    def recording(self):
        """Context manager that collects every buffer handed out inside it.  A HIP graph records raw
        device pointers: whoever records one keeps the collected tensors alive for as long as the
        graph lives, so that a later, larger request under the same name (which replaces the named
        buffer) or clear() cannot hand the recorded memory back to the allocator."""
        ws = self

        class _Rec:
            def __enter__(self):
                self.handed = []
                ws._recorders.append(self.handed)
                return self.handed

            def __exit__(self, *a):
                ws._recorders.remove(self.handed)
        return _Rec()


workspaces = _Workspaces()


class _SpareKV:
    """The second KV buffer of the beam-search reorder, shared by every attention op with the
    same cache shape on a device: an op gathers into the spare pair, takes it as its cache and
    leaves its old pair as the new spare.  The ops of a decoder run one after another on one
    stream, so a single spare serves all layers."""

    def __init__(self):
        self._pairs = {}

    def swap(self, k_cache, v_cache, gather):
        key = (tuple(k_cache.shape), k_cache.dtype, str(k_cache.device))
        pair = self._pairs.get(key)
        if pair is None:
            pair = (torch.zeros_like(k_cache), torch.zeros_like(v_cache))
        gather(pair[0], pair[1])
        self._pairs[key] = (k_cache, v_cache)
        return pair

    def clear(self):
        self._pairs.clear()


spare_kv = _SpareKV()


# ----------------------------------------------------------------------------
# MetaDesc
# ----------------------------------------------------------------------------
class MetaDesc:
    """csrc/op/meta_desc.hpp:9-101; constructor keywords as in eet2py.cpp:26-42."""

    def __init__(self, dtype, batch_size, head_num, hidden_units, layer_num, max_seq_len, max_full_seq_len=1,
                 activation_fn="gelu", d_kv=0, d_ff=0, cuda_device="cuda:0", requires_grad=False,
                 layernorm_eps=1e-6, is_int8=False):
        if not isinstance(dtype, torch.dtype):
            raise TypeError("MetaDesc: dtype must be a torch.dtype")
        if requires_grad:
            raise RuntimeError("[EET][ERROR] EET only supports inference (requires_grad must be False)")
        self.dtype = dtype
        self.batch_size = int(batch_size)
        self.head_num = int(head_num)
        self.hidden_units = int(hidden_units)
        self.layer_num = int(layer_num)
        self.max_seq_len = int(max_seq_len)
        self.max_full_seq_len = int(max_full_seq_len)
        self.activation_fn = activation_fn
        self.d_kv = int(d_kv)
        self.d_ff = int(d_ff)
        self.device = torch.device(cuda_device)
        self.layernorm_eps = float(layernorm_eps)
        self.is_int8 = bool(is_int8)


def _require_int8_fp16(desc, who):
    if desc.dtype != torch.float16 or not desc.is_int8:
        raise NotImplementedError(
            f"[EET][ERROR] {who}: only the int8 weight-only path with fp16 activations is implemented "
            f"(dtype={desc.dtype}, is_int8={desc.is_int8})")


def _check_weight(name, w, K, N, device):
    if w.dtype != torch.int8 or tuple(w.shape) != (K, N) or not w.is_contiguous():
        raise RuntimeError(f"[EET][ERROR] {name}: expected contiguous int8 [{K}, {N}], got {w.dtype} {tuple(w.shape)}")
    if w.device.type != "cuda":
        raise RuntimeError(f"[EET][ERROR] {name}: weight must be on the GPU")


def _check_vec(name, v, N):
    if v.dtype != torch.float16 or v.numel() != N or not v.is_contiguous() or v.device.type != "cuda":
        raise RuntimeError(f"[EET][ERROR] {name}: expected contiguous fp16 GPU tensor of {N} elements, "
                           f"got {v.dtype} {tuple(v.shape)} on {v.device}")


EPI_NONE, EPI_RESIDUAL, EPI_SWIGLU = 0, 1, 2


class LaunchTimer:
    """Per-kernel timing of the decode path for a benchmark's breakdown: while one is installed
    (`ops.launch_timer = LaunchTimer()`), the incremental calls of the ops issue their launches
    one library call at a time -- the same entry points with the same arguments that
    eet_mmha_int8_decode / eet_gated_ffn_int8_decode issue from C++ -- each bracketed by a pair
    of events on the current stream.  summary() waits for the GPU."""

    def __init__(self):
        self.records = []

    def run(self, name, nbytes, fn):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        out = fn()
        e1.record()
        self.records.append((name, nbytes, e0, e1))
        return out

    def summary(self):
        torch.cuda.synchronize()
        agg = {}
        for name, nbytes, e0, e1 in self.records:
            a = agg.setdefault(name, [0, 0.0, 0])
            a[0] += 1
            a[1] += e0.elapsed_time(e1) * 1e3
            a[2] += nbytes
        return {k: {"calls": v[0], "us_total": v[1], "bytes_total": v[2]} for k, v in agg.items()}


launch_timer = None


class ReplayState:
    """Set as `ops.replay_state` while a decoder records its incremental step into a HIP graph (and
    for the eager warm-up before it): the attention ops then issue the replayable form of their
    call, which reads the step from `step_dev` (int32 on the GPU) instead of taking it by value."""

    def __init__(self, step_dev, step_max):
        self.step_dev, self.step_max = step_dev, int(step_max)


replay_state = None


def _timed(name, nbytes, fn):
    return launch_timer.run(name, nbytes, fn) if launch_timer is not None else fn()


def linear_bytes(M, K, N, epilogue=EPI_NONE):
    """Algorithmic bytes of one int8 linear: every operand once."""
    n_out = N // 2 if epilogue == EPI_SWIGLU else N
    return K * N + 2 * N + 2 * M * K + 2 * M * n_out + (2 * M * N if epilogue == EPI_RESIDUAL else 0)


RMS_FUSE_MAX_M = 32     # the RMSnorm prologue exists in the small-M kernel only


def _k_split_ws(M, N, K, epilogue, device):
    """(pointer, bytes) of the small-M kernel's k-split workspace for this call, or (None, 0).  A buffer of its
    own, zero when created (the arrival counters at its start must start at zero; every call leaves them so).
    One buffer per device, like every named workspace here (and like the reference's MManager buffers,
    csrc/op/mmanager.hpp:141-205): the ops of a process are meant to run on one stream; launches on two
    streams that can overlap in time must not share it."""
    need = lib().eet_gemm_w8a16_workspace(M, N, K, epilogue) if M <= RMS_FUSE_MAX_M else 0
    if not need:
        return None, 0
    buf = workspaces.get("gemm_small_m_k_split", (need + 3) // 4, torch.float32, device, zero=True)
    return buf.data_ptr(), buf.numel() * 4


def _gemm(a, w, scale, out, M, N, K, epilogue=EPI_NONE, residual=None, rms_gamma=None, rms_eps=0.0):
    L = lib()
    ws, ws_bytes = None, 0
    if M > RMS_FUSE_MAX_M:    # a launch with few tiles may split its k range: fp32 partial sums
        ws_bytes = L.eet_gemm_w8a16_workspace(M, N, K, epilogue)
        if ws_bytes:
            ws = workspaces.get("gemm_split_k", ws_bytes // 4, torch.float32, a.device).data_ptr()
    elif rms_gamma is None:   # launches without a prologue may share a tile group's k range among workgroups
        ws, ws_bytes = _k_split_ws(M, N, K, epilogue, a.device)
    check(L.eet_gemm_w8a16_fused(a.data_ptr(), w.data_ptr(), scale.data_ptr(), out.data_ptr(), M, N, K,
                                 epilogue, residual.data_ptr() if residual is not None else None,
                                 rms_gamma.data_ptr() if rms_gamma is not None else None, rms_eps, ws, ws_bytes,
                                 _stream()),
          "eet_gemm_w8a16_fused")


def interleave_gate_up(gate_w, gate_s, up_w, up_s):
    """Merge two packed [K, N] weights (and their scales) tile by tile:
    16-channel tile 2i of the result is gate tile i, tile 2i+1 is up tile i.
    In the packed layout a tile is K*16 contiguous bytes."""
    K, N = gate_w.shape
    g = gate_w.reshape(N // 16, K * 16)
    u = up_w.reshape(N // 16, K * 16)
    w = torch.stack((g, u), 1).reshape(K, 2 * N).contiguous()
    s = torch.stack((gate_s.reshape(N // 16, 16), up_s.reshape(N // 16, 16)), 1).reshape(2 * N).contiguous()
    return w, s


def _rmsnorm(x, gamma, out, M, N, eps):
    check(lib().eet_rmsnorm(x.data_ptr(), gamma.data_ptr(), out.data_ptr(), M, N, eps, _stream()), "eet_rmsnorm")


# ----------------------------------------------------------------------------
# attention ops
# ----------------------------------------------------------------------------
_rope_tables = {}


def _rope_table(T, dh, device):
    """fp32 [T, dh] table (cos | sin per position), built once per (T, dh, device)."""
    key = (T, dh, str(device))
    t = _rope_tables.get(key)
    if t is None:
        t = torch.empty(T, dh, dtype=torch.float32, device=device)
        check(lib().eet_rope_table(t.data_ptr(), T, dh, _stream()), "eet_rope_table")
        _rope_tables[key] = t
    return t


class _MmhaInt8:
    """Shared body of LlamaMmha (rotary) and BaichuanMmha (ALiBi)."""

    _rope = True
    _bias_branch = False
    _name = "LlamaMmha"

    def __init__(self, desc, QKV_weights, QKV_scale, Q_bias, K_bias, V_bias, Output_weights, Output_scale,
                 Output_bias, layernorm_weights, layernorm_bias):
        _require_int8_fp16(desc, self._name)

        def given(b):
            return b is not None and b.numel() != 0
        # The bias branch: a Q bias switches the op to LayerNorm(gamma, beta) and adds Q / K / V biases to
        # the fused QKV rows (csrc/op/baichuan_mmha.cpp:45, 224-231, 295-297); the output bias follows
        # the residual add (:402).
        self.with_bias = given(Q_bias)
        if self.with_bias and not self._bias_branch:
            # for fp16 the reference's rotary split prints "Not support add bias for half" and launches
            # nothing (csrc/core/self_add_bias.cu:476-480): there is no behaviour to reproduce
            raise NotImplementedError(f"[EET][ERROR] {self._name}: Q / K / V biases are not supported with fp16 "
                                      "(the reference's rotary split refuses them for half as well)")
        if not self.with_bias and (given(K_bias) or given(V_bias) or given(layernorm_bias)):
            raise RuntimeError(f"[EET][ERROR] {self._name}: K_bias, V_bias and layernorm_bias take effect only "
                               "together with Q_bias (the reference selects the bias branch by Q_bias alone)")
        if self.with_bias and not (given(K_bias) and given(V_bias) and given(layernorm_bias)):
            raise RuntimeError(f"[EET][ERROR] {self._name}: with Q_bias the op also reads K_bias, V_bias and "
                               "layernorm_bias; all must be given")
        self.desc = desc
        H = desc.head_num
        if desc.d_kv == 0:
            self.dh, self.inner = desc.hidden_units // H, desc.hidden_units
        else:
            self.dh, self.inner = desc.d_kv, desc.d_kv * H
        if self.dh not in (32, 64, 96, 128):
            raise RuntimeError(f"[EET][ERROR] {self._name}: head size {self.dh} not supported (32, 64, 96, 128)")
        hidden = desc.hidden_units
        _check_weight("QKV_weights", QKV_weights, hidden, 3 * self.inner, desc.device)
        _check_weight("Output_weights", Output_weights, self.inner, hidden, desc.device)
        _check_vec("QKV_scale", QKV_scale, 3 * self.inner)
        _check_vec("Output_scale", Output_scale, hidden)
        _check_vec("layernorm_weights", layernorm_weights, hidden)
        # keep the tensors alive: the kernels read them through raw pointers
        self.qkv_w, self.qkv_s, self.o_w, self.o_s, self.gamma = (QKV_weights, QKV_scale, Output_weights,
                                                                  Output_scale, layernorm_weights)
        dev = QKV_weights.device
        self.t_cap = desc.max_full_seq_len
        # KV cache, private to the op (csrc/op/llama_mmha.cpp:47-48); layout [B][H][T][dh]
        self.k_cache = torch.zeros(desc.batch_size, H, self.t_cap, self.dh, dtype=torch.float16, device=dev)
        self.v_cache = torch.zeros_like(self.k_cache)
        self.step = 1
        self.first_batch = 0
        self.rope_table = _rope_table(self.t_cap, self.dh, dev) if self._rope else None
        self.qkv_bias = self.beta = self.o_bias = None
        if self.with_bias:
            for nm, b in (("Q_bias", Q_bias), ("K_bias", K_bias), ("V_bias", V_bias)):
                _check_vec(nm, b, self.inner)
            _check_vec("layernorm_bias", layernorm_bias, hidden)
            self.qkv_bias = torch.cat((Q_bias.reshape(-1), K_bias.reshape(-1), V_bias.reshape(-1))).contiguous()
            self.beta = layernorm_bias
        if given(Output_bias):
            _check_vec("Output_bias", Output_bias, hidden)
            self.o_bias = Output_bias
        self.biased = self.with_bias or self.o_bias is not None

    def forward(self, input, pre_padding_len, reorder_state, pre_layernorm, add_residual, first_pass,
                relative_attention_bias=_EMPTY):
        with _StreamScope():
            return self._forward(input, pre_padding_len, reorder_state, pre_layernorm, add_residual, first_pass,
                                 relative_attention_bias)

    def _forward(self, input, pre_padding_len, reorder_state, pre_layernorm, add_residual, first_pass,
                 relative_attention_bias):
        # pre_layernorm / add_residual are accepted and ignored exactly as in the
        # reference: it always normalises first and always adds the input back
        # (csrc/op/llama_mmha.cpp:136, 222, 462).
        desc, H, dh = self.desc, self.desc.head_num, self.dh
        if input.dtype != torch.float16 or input.dim() != 3 or input.shape[2] != desc.hidden_units:
            raise RuntimeError(f"[EET][ERROR] {self._name}: input must be fp16 [B, S, {desc.hidden_units}], got "
                               f"{input.dtype} {tuple(input.shape)}")
        if input.device.type != "cuda":
            raise RuntimeError(f"[EET][ERROR] {self._name}: input must be on the GPU")
        reorder = reorder_state if (reorder_state is not None and reorder_state.numel() != 0) else None
        if reorder is not None and not first_pass:
            if reorder.dtype != torch.int64 or reorder.device.type != "cuda" or reorder.numel() < self.first_batch:
                raise RuntimeError(f"[EET][ERROR] {self._name}: reorder_state must be an int64 GPU tensor with one "
                                   f"entry per beam ({self.first_batch})")
            reorder = reorder.contiguous()
        x = input.contiguous()
        B, S, hidden = x.shape
        if B > desc.batch_size:
            raise RuntimeError(f"[EET][ERROR] {self._name}: batch {B} exceeds batch_size {desc.batch_size}")
        dev = x.device
        pad = pre_padding_len if (pre_padding_len is not None and pre_padding_len.numel() != 0) else None
        if pad is not None:
            if pad.dtype != torch.int64 or pad.numel() < B or pad.device.type != "cuda":
                raise RuntimeError(f"[EET][ERROR] {self._name}: pre_padding_len must be an int64 GPU tensor of B elements")
            pad = pad.contiguous()
        bias = relative_attention_bias if (relative_attention_bias is not None
                                           and relative_attention_bias.numel() != 0) else None
        if self._rope and bias is not None:
            raise RuntimeError(f"[EET][ERROR] {self._name}: relative_attention_bias is not used by the rotary op")
        if first_pass:
            if S > desc.max_seq_len or S > self.t_cap:
                raise RuntimeError(f"[EET][ERROR] {self._name}: prompt length {S} exceeds max_seq_len "
                                   f"{desc.max_seq_len} / max_full_seq_len {self.t_cap}")
            self.step, self.first_batch = S, B
            t0, time_step = 0, -1
        else:
            if S != 1:
                raise RuntimeError(f"[EET][ERROR] {self._name}: incremental call needs seq_len 1, got {S}")
            if self.step + 1 > self.t_cap:
                raise RuntimeError(f"[EET][ERROR] {self._name}: step {self.step + 1} exceeds max_full_seq_len "
                                   f"{self.t_cap}")
            self.step += 1
            t0, time_step = self.step - 1, self.step - 1
        M = B * S
        L = lib()
        if reorder is not None and not first_pass:
            # beam b continues from the rows of beam reorder[b] (csrc/op/llama_mmha.cpp:248-252):
            # gather into the spare cache pair (one per cache shape, shared by all layers), then
            # take that pair as this op's cache
            def gather(k_dst, v_dst):
                check(L.eet_kv_cache_reorder(self.k_cache.data_ptr(), self.v_cache.data_ptr(), k_dst.data_ptr(),
                                             v_dst.data_ptr(), reorder.data_ptr(), self.first_batch, H, dh,
                                             self.step - 1, self.t_cap, _stream()), "eet_kv_cache_reorder")
            self.k_cache, self.v_cache = spare_kv.swap(self.k_cache, self.v_cache, gather)
        f16 = torch.float16
        xn = workspaces.get("layernorm", desc.batch_size * max(desc.max_seq_len, 1) * hidden, f16, dev)
        qkv = workspaces.get("qkv", desc.batch_size * max(desc.max_seq_len, 1) * 3 * self.inner, f16, dev)
        qbuf = workspaces.get("q_buf", desc.batch_size * max(desc.max_seq_len, 1) * self.inner, f16, dev)
        cbuf = workspaces.get("context_buf", desc.batch_size * max(desc.max_seq_len, 1) * self.inner, f16, dev)
        out = workspaces.get("self_mask_attn_cache", desc.batch_size * max(desc.max_seq_len, 1) * hidden, f16, dev)
        if self.biased and replay_state is not None:
            raise NotImplementedError(f"[EET][ERROR] {self._name}: the bias branch has no replayable (HIP graph) form")
        if not first_pass and M <= RMS_FUSE_MAX_M and not self.biased:
            # the whole incremental call from one library call: RMSnorm + QKV, rotary + append +
            # attention, output projection + residual
            alibi = None
            if bias is not None and replay_state is None:
                if bias.numel() != H * self.step:
                    raise RuntimeError(f"[EET][ERROR] {self._name}: relative_attention_bias must be [H, 1, step] "
                                       f"with step={self.step}, got {tuple(bias.shape)}")
                alibi = bias.to(f16).contiguous()
            need = L.eet_mmha_int8_decode_workspace(B, H, dh, self.step)
            ws = workspaces.get("mmha_ws", max(need // 4, 1), torch.float32, dev)
            if replay_state is not None:
                rs = replay_state
                ld = 0
                if bias is not None:
                    # the whole [H, T] table with a fixed leading dimension: the kernel reads row entries < step
                    ld = bias.shape[-1]
                    if bias.numel() != H * ld or ld < rs.step_max:
                        raise RuntimeError(f"[EET][ERROR] {self._name}: a replayable step needs the bias table "
                                           f"[H, >= {rs.step_max}], got {tuple(bias.shape)}")
                    alibi = bias.to(f16).contiguous()
                need = L.eet_mmha_decode_replayable_workspace(B, H, dh, rs.step_max)
                ws = workspaces.get("mmha_ws", max(need // 4, 1), torch.float32, dev)
                check(L.eet_mmha_int8_decode_replayable(
                    x.data_ptr(), self.gamma.data_ptr(), desc.layernorm_eps, self.qkv_w.data_ptr(),
                    self.qkv_s.data_ptr(), self.o_w.data_ptr(), self.o_s.data_ptr(), self.k_cache.data_ptr(),
                    self.v_cache.data_ptr(), _ptr(alibi), ld, _ptr(pad),
                    self.rope_table.data_ptr() if self._rope else None, qkv.data_ptr(), cbuf.data_ptr(), out.data_ptr(),
                    B, H, dh, hidden, rs.step_dev.data_ptr(), rs.step_max, self.t_cap, ws.data_ptr(), ws.numel() * 4,
                    *_k_split_ws(B, hidden, self.inner, EPI_RESIDUAL, dev), _stream()), "eet_mmha_int8_decode_replayable")
                self._keep = (x, pad, alibi, reorder)
                return out[: M * hidden].view(B, S, hidden)
            rope = self.rope_table.data_ptr() + (self.step - 1) * dh * 4 if self._rope else None
            if launch_timer is not None:
                inner, base = self.inner, qkv.data_ptr()
                _timed("qkv_gemm+rmsnorm", linear_bytes(B, hidden, 3 * inner), lambda: _gemm(
                    x, self.qkv_w, self.qkv_s, qkv, B, 3 * inner, hidden, EPI_NONE, None, self.gamma, desc.layernorm_eps))
                attn_bytes = 2 * self.step * B * inner * 2 + 6 * B * inner * 2 + (2 * H * self.step if alibi is not None else 0)
                _timed("decode_attention", attn_bytes, lambda: check(L.eet_mmha_decode(
                    base, base + 2 * inner, base + 4 * inner, 3 * inner, self.k_cache.data_ptr(), self.v_cache.data_ptr(),
                    cbuf.data_ptr(), _ptr(alibi), _ptr(pad), B, H, dh, self.step, self.t_cap, rope, ws.data_ptr(),
                    ws.numel() * 4, _stream()), "eet_mmha_decode"))
                _timed("o_gemm+residual", linear_bytes(B, inner, hidden, EPI_RESIDUAL), lambda: _gemm(
                    cbuf, self.o_w, self.o_s, out, B, hidden, inner, EPI_RESIDUAL, x))
                self._keep = (x, pad, alibi, reorder)
                return out[: M * hidden].view(B, S, hidden)
            check(L.eet_mmha_int8_decode(x.data_ptr(), self.gamma.data_ptr(), desc.layernorm_eps,
                                         self.qkv_w.data_ptr(), self.qkv_s.data_ptr(), self.o_w.data_ptr(),
                                         self.o_s.data_ptr(), self.k_cache.data_ptr(), self.v_cache.data_ptr(),
                                         _ptr(alibi), _ptr(pad), rope, qkv.data_ptr(), cbuf.data_ptr(),
                                         out.data_ptr(), B, H, dh, hidden, self.step, self.t_cap, ws.data_ptr(),
                                         ws.numel() * 4, *_k_split_ws(B, hidden, self.inner, EPI_RESIDUAL, dev),
                                         _stream()), "eet_mmha_int8_decode")
            self._keep = (x, pad, alibi, reorder)  # inputs of kernels still in flight
            return out[: M * hidden].view(B, S, hidden)
        if self.with_bias:
            # LayerNorm, QKV projection, then the three biases on the fused rows (fp16 adds, as
            # fused_add_QKV_bias makes them: csrc/core/self_add_bias.cu:352-354)
            check(L.eet_layernorm(x.data_ptr(), self.gamma.data_ptr(), self.beta.data_ptr(), xn.data_ptr(), M, hidden,
                                  desc.layernorm_eps, _stream()), "eet_layernorm")
            _gemm(xn, self.qkv_w, self.qkv_s, qkv, M, 3 * self.inner, hidden)
            check(L.eet_add_bias(qkv.data_ptr(), self.qkv_bias.data_ptr(), M, 3 * self.inner, _stream()), "eet_add_bias")
        elif M <= RMS_FUSE_MAX_M:
            # RMSnorm folded into the GEMM's activation load
            _gemm(x, self.qkv_w, self.qkv_s, qkv, M, 3 * self.inner, hidden, EPI_NONE, None, self.gamma,
                  desc.layernorm_eps)
        else:
            _rmsnorm(x, self.gamma, xn, M, hidden, desc.layernorm_eps)
            _gemm(xn, self.qkv_w, self.qkv_s, qkv, M, 3 * self.inner, hidden)
        if first_pass:
            # split (+ rotary at position s) and write K, V rows [0, S) of the cache
            check(L.eet_qkv_split(qkv.data_ptr(), qbuf.data_ptr(), self.k_cache.data_ptr(),
                                  self.v_cache.data_ptr(), B, S, H, dh, 1 if self._rope else 0, -1, 0, self.t_cap,
                                  _stream()), "eet_qkv_split")
            alibi = None
            if bias is not None:
                # [H, S, S] mask whose row i holds slope*j for j <= i: its last row is the whole table
                if bias.dim() != 3 or bias.shape[0] != H or bias.shape[2] != S:
                    raise RuntimeError(f"[EET][ERROR] {self._name}: relative_attention_bias must be [H, S, S]")
                alibi = bias[:, -1, :].to(f16).contiguous()
            check(L.eet_prefill_attention(qbuf.data_ptr(), self.k_cache.data_ptr(), self.v_cache.data_ptr(),
                                          cbuf.data_ptr(), _ptr(alibi), _ptr(pad), B, H, S, dh, self.t_cap,
                                          _stream()), "eet_prefill_attention")
        else:
            alibi = None
            if bias is not None:
                if bias.numel() != H * self.step:
                    raise RuntimeError(f"[EET][ERROR] {self._name}: relative_attention_bias must be [H, 1, step] "
                                       f"with step={self.step}, got {tuple(bias.shape)}")
                alibi = bias.to(f16).contiguous()
            need = L.eet_mmha_decode_workspace(B, H, dh, self.step)
            ws = workspaces.get("mmha_ws", max(need // 4, 1), torch.float32, dev)
            # q, k, v are read straight from the fused GEMM output; the kernel rotates q and k
            # (rotary op only) and appends k, v at row step-1
            base, hd = qkv.data_ptr(), self.inner
            rope = self.rope_table.data_ptr() + (self.step - 1) * dh * 4 if self._rope else None
            check(L.eet_mmha_decode(base, base + 2 * hd, base + 4 * hd, 3 * hd, self.k_cache.data_ptr(),
                                    self.v_cache.data_ptr(), cbuf.data_ptr(), _ptr(alibi), _ptr(pad), B, H, dh,
                                    self.step, self.t_cap, rope, ws.data_ptr(), ws.numel() * 4, _stream()),
                  "eet_mmha_decode")
        # output projection with the residual add (csrc/op/llama_mmha.cpp:428-462) in its epilogue
        _gemm(cbuf, self.o_w, self.o_s, out, M, hidden, self.inner, EPI_RESIDUAL, x)
        if self.o_bias is not None:     # (out + input) + bias, csrc/core/add_bias.cu:13-20
            check(L.eet_add_bias(out.data_ptr(), self.o_bias.data_ptr(), M, hidden, _stream()), "eet_add_bias")
        self._keep = (x, pad, alibi, reorder)  # inputs of kernels still in flight
        return out[: M * hidden].view(B, S, hidden)


class LlamaMmha(_MmhaInt8):
    """csrc/op/llama_mmha.cpp:14-266."""
    _rope = True
    _bias_branch = False
    _name = "LlamaMmha"


class BaichuanMmha(_MmhaInt8):
    """csrc/op/baichuan_mmha.cpp:81-216: no rotary; an ALiBi tensor is passed in
    ([H, S, S] for the prompt, [H, 1, step] per decode step)."""
    _rope = False
    _bias_branch = True
    _name = "BaichuanMmha"


# ----------------------------------------------------------------------------
# gated FFN
# ----------------------------------------------------------------------------
class GatedFeedForwardNetworkInt8:
    """csrc/op/gated_ffn_int8.cpp:12-132, 328-357."""

    def __init__(self, desc, Intermediate_0_weights, Intermediate_0_scale, Intermediate_0_bias,
                 Intermediate_1_weights, Intermediate_1_scale, Intermediate_1_bias, Output_weights, Output_scale,
                 Output_bias, layernorm_weights, layernorm_bias, ffn_cache_name="out_cache"):
        _require_int8_fp16(desc, "GatedFeedForwardNetworkInt8")
        if desc.activation_fn != "silu":
            # the reference prints "unsupported activation" and goes on (gated_ffn_int8.cpp:57-61)
            raise NotImplementedError(f"[EET][ERROR] GatedFeedForwardNetworkInt8: activation "
                                      f"'{desc.activation_fn}' is not implemented (silu only)")
        # Intermediate_0_bias / Intermediate_1_bias are accepted and never used, exactly as in the reference:
        # its forward passes no bias to fc1 / fc2 and gated_act takes none (gated_ffn_int8.cpp:98-132, 168-179).
        self.desc = desc
        hidden = desc.hidden_units
        self.d_ff = desc.d_ff if desc.d_ff != 0 else 4 * hidden  # gated_ffn_int8.cpp:62-68
        dev = desc.device
        _check_weight("Intermediate_0_weights", Intermediate_0_weights, hidden, self.d_ff, dev)
        _check_weight("Intermediate_1_weights", Intermediate_1_weights, hidden, self.d_ff, dev)
        _check_weight("Output_weights", Output_weights, self.d_ff, hidden, dev)
        _check_vec("Intermediate_0_scale", Intermediate_0_scale, self.d_ff)
        _check_vec("Intermediate_1_scale", Intermediate_1_scale, self.d_ff)
        _check_vec("Output_scale", Output_scale, hidden)
        _check_vec("layernorm_weights", layernorm_weights, hidden)
        self.w2, self.s2, self.gamma = Output_weights, Output_scale, layernorm_weights
        self.beta = self.o_bias = None
        if layernorm_bias is not None and layernorm_bias.numel() != 0:    # LayerNorm instead of RMSnorm (:139-146)
            _check_vec("layernorm_bias", layernorm_bias, hidden)
            self.beta = layernorm_bias
        if Output_bias is not None and Output_bias.numel() != 0:
            _check_vec("Output_bias", Output_bias, hidden)
            self.o_bias = Output_bias
        self.cache_name = ffn_cache_name
        # gate and up merged tile by tile so that one launch computes both and applies SwiGLU;
        # the op keeps only the merged copy (the caller's separate tensors can be freed)
        self.w01, self.s01 = interleave_gate_up(Intermediate_0_weights, Intermediate_0_scale,
                                                Intermediate_1_weights, Intermediate_1_scale)

    def forward(self, input, pre_layernorm, add_residual):
        with _StreamScope():
            return self._forward(input, pre_layernorm, add_residual)

    def _forward(self, input, pre_layernorm, add_residual):
        desc = self.desc
        if input.dtype != torch.float16 or input.dim() != 3 or input.shape[2] != desc.hidden_units:
            raise RuntimeError(f"[EET][ERROR] GatedFeedForwardNetworkInt8: input must be fp16 [B, S, "
                               f"{desc.hidden_units}], got {input.dtype} {tuple(input.shape)}")
        post_ln = add_residual and not pre_layernorm
        if post_ln and self.o_bias is not None and self.beta is None:
            raise RuntimeError("[EET][ERROR] GatedFeedForwardNetworkInt8: the post-layernorm tail with an output bias is "
                               "a LayerNorm and needs layernorm_bias (gated_ffn_int8.cpp:335-342)")
        x = input.contiguous()
        B, S, hidden = x.shape
        if B > desc.batch_size or S > max(desc.max_seq_len, 1):
            raise RuntimeError(f"[EET][ERROR] GatedFeedForwardNetworkInt8: input [{B}, {S}] exceeds "
                               f"[{desc.batch_size}, {desc.max_seq_len}]")
        M, dev, f16 = B * S, x.device, torch.float16
        cap = desc.batch_size * max(desc.max_seq_len, 1)
        xn = workspaces.get("layernorm_tensor", cap * hidden, f16, dev)
        act = workspaces.get("ffn_inner_act", cap * self.d_ff, f16, dev)
        out = workspaces.get(self.cache_name, cap * hidden, f16, dev)
        if post_ln or self.beta is not None or self.o_bias is not None:
            return self._forward_general(x, xn, act, out, M, hidden, post_ln, add_residual)
        # fc1, fc2 and gated_act (gated_ffn_int8.cpp:253-301, 168-179) in one launch; at decode
        # sizes the RMSnorm (:112) rides in the same launch and fc3 follows from the same library call
        if M <= RMS_FUSE_MAX_M and launch_timer is not None:
            _timed("gate_up_gemm+rmsnorm+swiglu", linear_bytes(M, hidden, 2 * self.d_ff, EPI_SWIGLU), lambda: _gemm(
                x, self.w01, self.s01, act, M, 2 * self.d_ff, hidden, EPI_SWIGLU, None, self.gamma, desc.layernorm_eps))
            epi = EPI_RESIDUAL if add_residual else EPI_NONE
            _timed("down_gemm+residual", linear_bytes(M, self.d_ff, hidden, epi), lambda: _gemm(
                act, self.w2, self.s2, out, M, hidden, self.d_ff, epi, x if add_residual else None))
            self._keep = x
            return out[: M * hidden].view(B, S, hidden)
        if M <= RMS_FUSE_MAX_M:
            check(lib().eet_gated_ffn_int8_decode(x.data_ptr(), self.gamma.data_ptr(), desc.layernorm_eps,
                                                  self.w01.data_ptr(), self.s01.data_ptr(), self.w2.data_ptr(),
                                                  self.s2.data_ptr(), act.data_ptr(), out.data_ptr(), M, hidden,
                                                  self.d_ff, 1 if add_residual else 0,
                                                  *_k_split_ws(M, hidden, self.d_ff,
                                                               EPI_RESIDUAL if add_residual else EPI_NONE, dev),
                                                  _stream()),
                  "eet_gated_ffn_int8_decode")
            self._keep = x
            return out[: M * hidden].view(B, S, hidden)
        _rmsnorm(x, self.gamma, xn, M, hidden, desc.layernorm_eps)
        _gemm(xn, self.w01, self.s01, act, M, 2 * self.d_ff, hidden, EPI_SWIGLU)
        # fc3 with add_input_bias_layernorm's residual add (:303-357) in its epilogue
        if add_residual:
            _gemm(act, self.w2, self.s2, out, M, hidden, self.d_ff, EPI_RESIDUAL, x)
        else:
            _gemm(act, self.w2, self.s2, out, M, hidden, self.d_ff)
        self._keep = x
        return out[: M * hidden].view(B, S, hidden)


    def _forward_general(self, x, xn, act, out, M, hidden, post_ln, add_residual):
        """The branches LLaMA / Baichuan never take: LayerNorm in front (layernorm_bias given), an output bias,
        and the post-layernorm tail.  Unfused: norm kernel, gate|up + SwiGLU, down, then the tail."""
        desc, L, B, S = self.desc, lib(), x.shape[0], x.shape[1]
        if self.beta is not None:
            check(L.eet_layernorm(x.data_ptr(), self.gamma.data_ptr(), self.beta.data_ptr(), xn.data_ptr(), M, hidden,
                                  desc.layernorm_eps, _stream()), "eet_layernorm")
        else:
            _rmsnorm(x, self.gamma, xn, M, hidden, desc.layernorm_eps)     # applied in both modes (:112)
        _gemm(xn, self.w01, self.s01, act, M, 2 * self.d_ff, hidden, EPI_SWIGLU)
        if post_ln:
            # add_bias + add_residual + layer_norm (:335-342): LayerNorm with a bias, RMSnorm without
            _gemm(act, self.w2, self.s2, out, M, hidden, self.d_ff)
            check(L.eet_add_bias_residual_norm(out.data_ptr(), x.data_ptr(), _ptr(self.o_bias), self.gamma.data_ptr(),
                                               self.beta.data_ptr() if self.o_bias is not None else None, M, hidden,
                                               desc.layernorm_eps, _stream()), "eet_add_bias_residual_norm")
        else:
            if add_residual:
                _gemm(act, self.w2, self.s2, out, M, hidden, self.d_ff, EPI_RESIDUAL, x)
            else:
                _gemm(act, self.w2, self.s2, out, M, hidden, self.d_ff)
            if self.o_bias is not None:
                check(L.eet_add_bias(out.data_ptr(), self.o_bias.data_ptr(), M, hidden, _stream()), "eet_add_bias")
        self._keep = x
        return out[: M * hidden].view(B, S, hidden)


class LayerNorm:
    """csrc/op/layer_norm.cpp:8-33: LayerNorm(gamma, beta), RMSnorm when beta is empty."""

    def __init__(self, desc, gamma, beta):
        if desc.dtype != torch.float16:
            raise NotImplementedError("[EET][ERROR] LayerNorm: fp16 only")
        _check_vec("gamma", gamma, desc.hidden_units)
        self.beta = None
        if beta is not None and beta.numel() != 0:
            _check_vec("beta", beta, desc.hidden_units)
            self.beta = beta
        self.desc, self.gamma = desc, gamma
        self.output = torch.zeros(desc.batch_size, max(desc.max_seq_len, 1), desc.hidden_units,
                                  dtype=torch.float16, device=gamma.device)

    def layer_norm(self, input):
        desc = self.desc
        if input.dtype != torch.float16 or input.dim() != 3 or input.shape[2] != desc.hidden_units:
            raise RuntimeError("[EET][ERROR] LayerNorm: input must be fp16 [B, S, hidden]")
        x = input.contiguous()
        B, S, hidden = x.shape
        if B * S > self.output.shape[0] * self.output.shape[1]:
            raise RuntimeError("[EET][ERROR] LayerNorm: input larger than batch_size * max_seq_len")
        if self.beta is not None:
            check(lib().eet_layernorm(x.data_ptr(), self.gamma.data_ptr(), self.beta.data_ptr(), self.output.data_ptr(),
                                      B * S, hidden, desc.layernorm_eps, _stream()), "eet_layernorm")
        else:
            _rmsnorm(x, self.gamma, self.output, B * S, hidden, desc.layernorm_eps)
        self._keep = x
        return self.output.view(-1)[: B * S * hidden].view(B, S, hidden)


# ----------------------------------------------------------------------------
# offline packer
# ----------------------------------------------------------------------------
def _quantize(weight, mode):
    K, N = weight.shape
    q = torch.empty(K, N, dtype=torch.int8)
    scale = torch.empty(N, dtype=weight.dtype)
    dt = 0 if weight.dtype == torch.float32 else 1
    check(lib().eet_quantize_int8(weight.data_ptr(), dt, K, N, mode, q.data_ptr(), scale.data_ptr()),
          "eet_quantize_int8")
    return q, scale


def pack_weights(q):
    """int8 [K, N] row-major -> gfx950 tile layout (same shape and byte count)."""
    if q.device.type != "cpu" or q.dtype != torch.int8 or q.dim() != 2 or not q.is_contiguous():
        raise RuntimeError("[EET][ERROR] pack_weights: expected a contiguous CPU int8 [K, N] tensor")
    out = torch.empty_like(q)
    check(lib().eet_pack_gfx950(q.data_ptr(), q.shape[0], q.shape[1], out.data_ptr()), "eet_pack_gfx950")
    return out


def unpack_weights(p):
    if p.device.type != "cpu" or p.dtype != torch.int8 or p.dim() != 2 or not p.is_contiguous():
        raise RuntimeError("[EET][ERROR] unpack_weights: expected a contiguous CPU int8 [K, N] tensor")
    out = torch.empty_like(p)
    check(lib().eet_unpack_gfx950(p.data_ptr(), p.shape[0], p.shape[1], out.data_ptr()), "eet_unpack_gfx950")
    return out


def pack_weights_torch(q):
    """eet_pack_gfx950 expressed as torch view / permute ops, so that a weight
    that already lives on the GPU can be packed there.  Same result, any device."""
    if q.dtype != torch.int8 or q.dim() != 2 or q.shape[0] % 64 or q.shape[1] % 16:
        raise RuntimeError("[EET][ERROR] pack_weights_torch: expected int8 [K, N] with K % 64 == 0 and N % 16 == 0")
    K, N = q.shape
    t = (q.view(torch.uint8) ^ 0x80).view(K // 64, 4, 16, N // 16, 16)   # [kt, g, b, nt, i]
    return t.permute(3, 0, 1, 4, 2).contiguous().view(torch.int8).view(K, N)


def _round_half_away(r):
    """C round(): r - trunc(r) is exact in binary floating point, so unlike
    floor(|r| + 0.5) this never rounds twice (0.49999997f stays 0)."""
    t = torch.trunc(r)
    return t + torch.where((r - t).abs() >= 0.5, torch.sign(r), torch.zeros_like(r))


def quant_weights_torch(w, mode="ref128"):
    """The quantiser as torch ops on w's device, bit-identical to
    eet_quantize_int8 (fp32 math, one correctly rounded operation per step):
    returns (unprocessed int8 [K, N], scales in w's dtype)."""
    w32 = w.float()
    amax = w32.abs().amax(0)
    if mode == "ref128":
        s32 = amax * (1.0 / 128.0)
        r = _round_half_away(w32 / s32)
        r = torch.where(torch.isnan(r), torch.full_like(r, 127.0), r).clamp(-128, 127)
    else:
        s32 = amax / 127.0
        r = _round_half_away(w32 / s32)
        r = torch.where(torch.isnan(r), torch.zeros_like(r), r).clamp(-127, 127)
    return r.to(torch.int8), s32.to(w.dtype)


def quant_weights_device(origin_weight, return_unprocessed_quantized_tensor=False, mode="ref128"):
    """quant_weights for a weight that already lives on the GPU (fp16 / fp32
    [K, N], K % 64 == 0, N % 16 == 0): two HIP kernels instead of the host
    threads, same bits.  Returns [processed, scales] or [unprocessed,
    processed, scales] like quant_weights, as GPU tensors.  The reference
    only quantises CPU tensors (fpA_intB_gemm_wrapper.cu:33)."""
    w = origin_weight
    if w.device.type != "cuda" or w.dim() != 2 or not w.is_contiguous() or w.dtype not in (torch.float16, torch.float32):
        raise RuntimeError("[EET][ERROR] quant_weights_device: expected a contiguous fp16 / fp32 GPU tensor [K, N]")
    K, N = w.shape
    L = lib()
    packed = torch.empty(K, N, dtype=torch.int8, device=w.device)
    scales = torch.empty(N, dtype=w.dtype, device=w.device)
    q = torch.empty(K, N, dtype=torch.int8, device=w.device) if return_unprocessed_quantized_tensor else None
    need = L.eet_quantize_pack_device_workspace(N)
    ws = workspaces.get("quant_absmax", max(need // 4, 1), torch.int32, w.device)
    with torch.cuda.device(w.device):
        check(L.eet_quantize_pack_device(w.data_ptr(), 0 if w.dtype == torch.float32 else 1, K, N,
                                         {"ref128": 0, "sym127": 1}[mode], q.data_ptr() if q is not None else None,
                                         packed.data_ptr(), scales.data_ptr(), ws.data_ptr(), need, _stream()),
              "eet_quantize_pack_device")
    return [q, packed, scales] if return_unprocessed_quantized_tensor else [packed, scales]


def quant_weights(origin_weight, quant_type, return_unprocessed_quantized_tensor=False, mode="ref128"):
    """symmetric_quantize_last_axis_of_tensor
    (3rdparty/cutlass_kernels/fpA_intB_gemm_wrapper.cu:26-105).  Returns
    [processed, scales] or [unprocessed, processed, scales]; `processed` is the
    gfx950 layout.  mode="sym127" selects the /127 generator (not a reference mode)."""
    w = origin_weight
    if w.device.type != "cpu":
        raise RuntimeError("weight must be a CPU tensor")
    if not w.is_contiguous():
        raise RuntimeError("weight must be contiguous")
    if w.numel() == 0:
        raise RuntimeError("weight should not be empty tensor")
    if w.dim() not in (2, 3):
        raise RuntimeError("Invalid dim. The dim of weight should be 2 or 3")
    if w.dtype not in (torch.float32, torch.float16):
        raise RuntimeError("Invalid datatype. Weight must be FP16 or FP32")
    if quant_type == torch.quint4x2:
        raise NotImplementedError("[EET][ERROR] quant_weights: int4 quantisation is not implemented")
    if quant_type != torch.int8:
        raise RuntimeError("Must be int4 or int8 quantization")
    m = {"ref128": 0, "sym127": 1}[mode]
    mats = [w] if w.dim() == 2 else list(w.unbind(0))
    qs, ps, ss = [], [], []
    for mat in mats:
        q, s = _quantize(mat.contiguous(), m)
        qs.append(q)
        ps.append(pack_weights(q))
        ss.append(s)
    if w.dim() == 2:
        unprocessed, processed, scales = qs[0], ps[0], ss[0]
    else:
        unprocessed, processed, scales = torch.stack(qs), torch.stack(ps), torch.stack(ss)
    if return_unprocessed_quantized_tensor:
        return [unprocessed, processed, scales]
    return [processed, scales]


def preprocess_weights(origin_weight, is_int4=False):
    """preprocess_weights_cuda (fpA_intB_gemm_wrapper.cu:107-126): row-major
    int8 [K, N] -> the layout the GEMM reads."""
    if is_int4:
        raise NotImplementedError("[EET][ERROR] preprocess_weights: int4 is not implemented")
    if origin_weight.device.type != "cpu":
        raise RuntimeError("origin_weight must be a CPU tensor")
    return pack_weights(origin_weight.contiguous())


def _not_on_this_path(name):
    class _Stub:
        def __init__(self, *a, **k):
            raise NotImplementedError(f"[EET][ERROR] {name} is not part of the int8 weight-only path "
                                      "implemented by this library")
    _Stub.__name__ = name
    return _Stub


# names the reference's Python imports from `EET` but that belong to other model families
GatedFeedForwardNetwork = _not_on_this_path("GatedFeedForwardNetwork")
FeedForwardNetwork = _not_on_this_path("FeedForwardNetwork")
MultiHeadAttention = _not_on_this_path("MultiHeadAttention")
CrossMultiHeadAttention = _not_on_this_path("CrossMultiHeadAttention")
MaskedMultiHeadAttention = _not_on_this_path("MaskedMultiHeadAttention")
Embedding = _not_on_this_path("Embedding")
