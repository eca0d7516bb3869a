"""ctypes binding of libeet_hip.so (declared in include/eet_hip.h).

The library must have been built (python -m eet_amd.build); there is no
fallback: a missing library raises at import of the first symbol.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libeet_hip.so")

_c = ctypes
_vp, _i, _sz, _f, _l = _c.c_void_p, _c.c_int, _c.c_size_t, _c.c_float, _c.c_long

# name -> (restype, argtypes); mirrors include/eet_hip.h one to one
SIGNATURES = {
    "eet_last_error": (_c.c_char_p, []),
    "eet_packed_layout_version": (_i, []),
    "eet_set_tuning": (_i, [_c.c_char_p, _c.c_char_p]),
    "eet_quantize_int8": (_i, [_vp, _i, _sz, _sz, _i, _vp, _vp]),
    "eet_pack_gfx950": (_i, [_vp, _sz, _sz, _vp]),
    "eet_unpack_gfx950": (_i, [_vp, _sz, _sz, _vp]),
    "eet_preprocess_ref_sm80": (_i, [_vp, _sz, _sz, _vp]),
    "eet_unprocess_ref_sm80": (_i, [_vp, _sz, _sz, _vp]),
    "eet_quantize_pack_device_workspace": (_sz, [_sz]),
    "eet_quantize_pack_device": (_i, [_vp, _i, _sz, _sz, _i, _vp, _vp, _vp, _vp, _sz, _vp]),
    "eet_gemm_w8a16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp, _sz, _vp]),
    "eet_gemm_w8a16_workspace": (_sz, [_i, _i, _i, _i]),
    "eet_gemm_w8a16_fused": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _f, _vp, _sz, _vp]),
    "eet_gemm_w8a16_small_m_shape": (_i, [_i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "eet_gemm_w8a16_chained": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _f, _i, _vp]),
    "eet_chain_status": (_i, [_vp, _i, _vp]),
    "eet_mmha_decode_workspace": (_sz, [_i, _i, _i, _i]),
    "eet_mmha_decode": (_i, [_vp, _vp, _vp, _l, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "eet_mmha_decode_static_capacity": (_sz, []),
    "eet_mmha_decode_static": (_i, [_vp, _vp, _vp, _l, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp]),
    "eet_step_advance": (_i, [_vp, _i, _vp]),
    "eet_mmha_decode_replayable_workspace": (_sz, [_i, _i, _i, _i]),
    "eet_mmha_decode_replayable": (_i, [_vp, _vp, _vp, _l, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp, _i, _i, _vp, _vp,
                                        _sz, _vp]),
    "eet_mmha_int8_decode_replayable": (_i, [_vp, _vp, _f] + [_vp] * 7 + [_i] + [_vp] * 5 + [_i] * 4 + [_vp, _i, _i, _vp,
                                                                                                 _sz, _vp, _sz, _vp]),
    "eet_mmha_int8_decode_workspace": (_sz, [_i, _i, _i, _i]),
    "eet_mmha_int8_decode": (_i, [_vp, _vp, _f] + [_vp] * 12 + [_i] * 6 + [_vp, _sz, _vp, _sz, _vp]),
    "eet_gated_ffn_int8_decode": (_i, [_vp, _vp, _f] + [_vp] * 6 + [_i] * 4 + [_vp, _sz, _vp]),
    "eet_rope_table": (_i, [_vp, _i, _i, _vp]),
    "eet_rmsnorm": (_i, [_vp, _vp, _vp, _i, _i, _f, _vp]),
    "eet_layernorm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _f, _vp]),
    "eet_add_bias_residual_norm": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp]),
    "eet_add_bias": (_i, [_vp, _vp, _i, _i, _vp]),
    "eet_qkv_split": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "eet_swiglu": (_i, [_vp, _vp, _i, _i, _vp]),
    "eet_residual_add": (_i, [_vp, _vp, _i, _i, _vp]),
    "eet_kv_cache_reorder": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "eet_prefill_attention": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m eet_amd.build` (needs hipcc). "
                "There is no CPU fallback for the HIP kernels.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


# EET_HIP_DEBUG_SYNC=1: wait for the GPU after every library call and report a
# failure of its kernels under that call's name -- the reference's _DEBUG_MODE_
# build (cudaDeviceSynchronize + cudaGetLastError after each launch,
# csrc/op/common.hpp:12, csrc/op/llama_mmha.cpp:282-285).
DEBUG_SYNC = os.environ.get("EET_HIP_DEBUG_SYNC", "0") not in ("", "0")


def check(status, what=""):
    """Raise RuntimeError (what the reference's pybind layer turns its
    std::runtime_error into) when a C-ABI call returned non-zero."""
    if status != 0:
        msg = lib().eet_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"[EET][ERROR] {what or 'libeet_hip'}: {msg} (status {status})")
    if DEBUG_SYNC:
        import torch
        # no waiting while the stream records a HIP graph: a synchronisation there invalidates the capture
        if not torch.cuda.is_available() or torch.cuda.is_current_stream_capturing():
            return
        try:
            torch.cuda.synchronize()
        except RuntimeError as e:
            raise RuntimeError(f"[EET][ERROR] {what or 'libeet_hip'}: kernel failed: {e}") from e
