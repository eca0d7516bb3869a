"""The C-ABI library: loads without a GPU, exports exactly what include/eet_hip.h
declares, and validates arguments before touching the device."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from eet_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "eet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(eet_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    syms = declared_symbols()
    assert len(syms) >= 14
    assert sorted(_lib.SIGNATURES) == syms


def test_library_exports_every_declared_symbol():
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for s in declared_symbols():
        assert hasattr(handle, s), s


def test_layout_version_and_last_error():
    L = _lib.lib()
    assert L.eet_packed_layout_version() == 1
    rc = L.eet_pack_gfx950(None, 64, 16, None)
    assert rc == -1 and b"null pointer" in L.eet_last_error()


def test_quantize_argument_errors():
    L = _lib.lib()
    w = np.zeros((4, 4), np.float32)
    q = np.zeros((4, 4), np.int8)
    s = np.zeros(4, np.float32)
    assert L.eet_quantize_int8(w.ctypes.data, 7, 4, 4, 0, q.ctypes.data, s.ctypes.data) == -1
    assert L.eet_quantize_int8(w.ctypes.data, 0, 4, 4, 9, q.ctypes.data, s.ctypes.data) == -1
    assert L.eet_quantize_int8(None, 0, 4, 4, 0, q.ctypes.data, s.ctypes.data) == -1
    assert L.eet_quantize_int8(w.ctypes.data, 0, 4, 4, 0, q.ctypes.data, s.ctypes.data) == 0


def test_device_entry_points_validate_before_launch():
    """Bad arguments are refused on the host: no GPU is needed to see the error."""
    L = _lib.lib()
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data
    assert L.eet_gemm_w8a16(None, p, p, p, 1, 16, 64, None, 0, None) == -1
    assert L.eet_gemm_w8a16(p, p, p, p, 1, 16, 100, None, 0, None) == -2      # K % 64
    assert L.eet_gemm_w8a16(p, p, p, p, 1, 24, 64, None, 0, None) == -2       # N % 16
    assert b"K % 64" in L.eet_last_error()
    assert L.eet_gemm_w8a16(p, p, p, p, 0, 16, 64, None, 0, None) == 0        # empty batch: nothing to do
    # split-k workspace: none once the tiles fill the chip, ksplit x M x N fp32 for M in the tens to hundreds;
    # the small-M kernel's k split: counters + exchange slots for N = 4096 / 5120 at the rows that split
    assert L.eet_gemm_w8a16_workspace(8, 4096, 4096, 0) == 0 and L.eet_gemm_w8a16_workspace(8, 12288, 4096, 0) == 0
    assert L.eet_gemm_w8a16_workspace(32, 4096, 4096, 1) == 32768 + 128 * 2 * 2 * 2 * 1024     # counters + NT 2, 2 shares, 2 m-tiles
    assert L.eet_gemm_w8a16_workspace(16, 4096, 11008, 1) == 32768 + 64 * 4 * 4 * 1 * 1024      # NT 4, 4 shares
    assert L.eet_gemm_w8a16_workspace(8, 5120, 13696, 1) == 32768 + 64 * 4 * 5 * 1 * 1024       # NT 5, 4 shares
    assert L.eet_gemm_w8a16_workspace(32, 4096, 4096, 2) == 0                                     # not with SwiGLU
    assert L.eet_gemm_w8a16_workspace(2048, 4096, 4096, 0) == 0
    need = L.eet_gemm_w8a16_workspace(64, 4096, 11008, 0)
    assert need >= 2 * 64 * 4096 * 4 and need % (64 * 4096 * 4) == 0
    assert L.eet_gemm_w8a16_workspace(64, 4100, 11008, 0) == 0                # not a shape the GEMM accepts
    assert L.eet_mmha_decode(p, None, None, 0, p, p, p, None, None, 1, 1, 128, 9, 8, None, None, 0, None) == -1  # step > cap
    assert L.eet_mmha_decode(p, None, None, 0, p, p, p, None, None, 1, 1, 80, 1, 8, None, None, 0, None) == -2   # head size
    assert L.eet_mmha_decode(p, p, None, 0, p, p, p, None, None, 1, 1, 128, 1, 8, None, None, 0, None) == -1     # k without v
    assert L.eet_mmha_decode(p, None, None, 0, p, p, p, None, None, 1, 1, 128, 1, 8, p, None, 0, None) == -1  # rotary without k
    assert L.eet_mmha_decode_workspace(8, 32, 128, 1100) == 0     # one workgroup per (b, h): no partial results
    need = L.eet_mmha_decode_workspace(1, 8, 128, 1100)           # fewer heads than CUs: the time axis is split
    assert need > 0
    assert L.eet_mmha_decode(p, None, None, 0, p, p, p, None, None, 1, 8, 128, 1100, 1153, None, None, 0, None) == -4
    # operator-level decode calls: argument checks happen before any launch
    assert L.eet_mmha_int8_decode(None, p, 1e-6, p, p, p, p, p, p, None, None, None, p, p, p, 1, 1, 128, 128, 1, 8,
                                  None, 0, None, 0, None) == -1
    assert L.eet_mmha_int8_decode(p, p, 1e-6, p, p, p, p, p, p, None, None, None, p, p, p, 33, 1, 128, 128, 1, 8,
                                  None, 0, None, 0, None) == -2              # more than 32 rows
    assert L.eet_mmha_int8_decode(p, p, 1e-6, p, p, p, p, p, p, None, None, None, p, p, p, 1, 1, 128, 128, 1, 8,
                                  None, 0, None, 0, None) == -1              # out aliases x
    assert L.eet_gated_ffn_int8_decode(p, p, 1e-6, p, p, p, p, p, None, 1, 128, 256, 1, None, 0, None) == -1
    assert L.eet_gated_ffn_int8_decode(p, p, 1e-6, p, p, p, p, p, p, 40, 128, 256, 1, None, 0, None) == -2
    assert L.eet_mmha_int8_decode_workspace(8, 32, 128, 1100) == L.eet_mmha_decode_workspace(8, 32, 128, 1100)
    assert L.eet_rope_table(None, 4, 128, None) == -1
    assert L.eet_rmsnorm(p, p, p, 1, 20000, 1e-6, None) == -2
    assert L.eet_qkv_split(p, p, p, p, 1, 4, 1, 128, 1, -1, 6, 8, None) == -1  # rows past the cache end
    assert L.eet_swiglu(p, p, 1, 12, None) == -2
    assert L.eet_residual_add(p, None, 1, 16, None) == -1
    assert L.eet_prefill_attention(p, p, p, p, None, None, 1, 1, 4096, 80, 4096, None) == -2


def test_python_api_errors():
    import eet_amd
    with pytest.raises(RuntimeError, match="contiguous"):
        eet_amd.quant_weights(torch.zeros(64, 32).t(), torch.int8)
    with pytest.raises(RuntimeError, match="dim"):
        eet_amd.quant_weights(torch.zeros(64), torch.int8)
    with pytest.raises(RuntimeError, match="FP16 or FP32"):
        eet_amd.quant_weights(torch.zeros(64, 16, dtype=torch.float64), torch.int8)
    with pytest.raises(RuntimeError, match="empty"):
        eet_amd.quant_weights(torch.zeros(0, 16), torch.int8)
    with pytest.raises(RuntimeError, match="int4 or int8"):
        eet_amd.quant_weights(torch.zeros(64, 16), torch.int32)
    with pytest.raises(NotImplementedError):
        eet_amd.quant_weights(torch.zeros(64, 16), torch.quint4x2)
    p, s = eet_amd.quant_weights(torch.ones(64, 16), torch.int8)
    assert p.dtype == torch.int8 and p.shape == (64, 16) and s.dtype == torch.float32 and s.shape == (16,)
    u, p, s = eet_amd.quant_weights(torch.ones(2, 64, 16).half(), torch.int8, True)
    assert u.shape == (2, 64, 16) and s.shape == (2, 16) and s.dtype == torch.float16
    with pytest.raises(NotImplementedError):
        eet_amd.MultiHeadAttention()
    import EET
    for name in ("MetaDesc", "LlamaMmha", "BaichuanMmha", "GatedFeedForwardNetworkInt8", "GatedFeedForwardNetwork",
                 "Embedding", "preprocess_weights", "quant_weights", "FeedForwardNetwork", "MultiHeadAttention",
                 "CrossMultiHeadAttention", "MaskedMultiHeadAttention", "LayerNorm"):
        assert hasattr(EET, name)
    d = EET.MetaDesc(torch.float16, 8, 32, 4096, 32, 1024, 1153, "silu", 0, 11008, "cuda:0", False, 1e-6, True)
    assert d.max_full_seq_len == 1153 and d.d_ff == 11008 and d.is_int8
    with pytest.raises(NotImplementedError):
        EET.LlamaMmha(EET.MetaDesc(torch.float32, 1, 1, 64, 1, 8), *[torch.empty(0)] * 10)


def test_alibi_caller_matches_oracle():
    from eet_amd import decoder
    from oracle import ops as O
    assert np.allclose(decoder.alibi_slopes(40), O.alibi_slopes(40))
    m = decoder.alibi_mask(8, 6).numpy()
    assert np.array_equal(np.nan_to_num(m, neginf=-1), np.nan_to_num(O.alibi_mask(8, 6), neginf=-1))


def test_fused_argument_errors():
    from eet_amd._lib import lib
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data
    L = _lib.lib()
    assert L.eet_gemm_w8a16_fused(p, p, p, p, 1, 32, 64, 7, None, None, 0.0, None, 0, None) == -1          # unknown epilogue
    assert L.eet_gemm_w8a16_fused(p, p, p, p, 1, 32, 64, 1, None, None, 0.0, None, 0, None) == -1          # residual missing
    assert L.eet_gemm_w8a16_fused(p, p, p, p, 1, 32, 64, 0, p, None, 0.0, None, 0, None) == -1             # residual without the epilogue
    assert L.eet_gemm_w8a16_fused(p, p, p, p, 1, 48, 64, 2, None, None, 0.0, None, 0, None) == -2          # odd tile count
    assert L.eet_gemm_w8a16_fused(p, p, p, p, 64, 32, 64, 0, None, p, 1e-6, None, 0, None) == -2       # RMSnorm prologue, M > 32


def test_tuning_keys():
    """Every documented tuning key is accepted and cleared (host state only, no GPU); malformed values and
    unknown keys are refused with a message."""
    L = _lib.lib()
    for name, value in [("EET_GEMM_SMALL_M_CONFIG", "2,8,1"), ("EET_GEMM_SMALL_M_CONFIG", "2,8,1,2"),
                        ("EET_CHAIN_SPIN_LIMIT", "0"), ("EET_CHAIN_SLEEP", "4"), ("EET_GEMM_LARGE_M_TILE", "4,4"),
                        ("EET_GEMM_LARGE_M_TILE", "2,2,4"), ("EET_MMHA_NSPLIT", "2"), ("EET_MMHA_THREADS", "256"),
                        ("EET_MMHA_UNROLL", "4"), ("EET_PREFILL_LEGACY", "1"), ("EET_PREFILL_SHAPE", "2"),
                        ("EET_PREFILL_GROUP", "4"), ("EET_PREFILL_GROUP", "-1")]:
        assert L.eet_set_tuning(name.encode(), value.encode()) == 0, L.eet_last_error()
        assert L.eet_set_tuning(name.encode(), None) == 0
    assert L.eet_set_tuning(b"EET_GEMM_SMALL_M_CONFIG", b"2,8") != 0
    assert b"nt,waves,u" in L.eet_last_error()
    assert L.eet_set_tuning(b"EET_NO_SUCH_KEY", b"1") != 0
    assert b"unknown key" in L.eet_last_error()


def test_every_table_answer_has_a_kernel():
    """The small-M launch-shape table (formula, measured shapes, k split) only answers with shapes the library
    holds a kernel for -- plain, without the workspace and chained: the query decides this on the host, for
    every row count and a wide range of channel counts, with every prologue / epilogue."""
    L = _lib.lib()
    q = [ctypes.c_int() for _ in range(4)]
    widths = sorted(set(list(range(16, 2049, 16)) + [n * 16 for n in (160, 192, 200, 230, 240, 255, 256, 257, 300, 320, 344, 384,
                                                                         428, 480, 512, 640, 688, 768, 856, 960, 1024, 1376,
                                                                         1712, 2000, 2048, 2752, 4096)]))
    for K in (64, 4096, 5120, 11008, 13696):
        for N in widths:
            for M in (1, 2, 3, 4, 7, 8, 9, 16, 17, 24, 32):
                for epi, rms in ((0, 0), (1, 0), (0, 1), (1, 1), (2, 1), (2, 0)):
                    if epi == 2 and N % 32:
                        continue
                    rc = L.eet_gemm_w8a16_small_m_shape(M, N, K, epi, rms, *[ctypes.byref(x) for x in q])
                    assert rc == 0, L.eet_last_error().decode()
