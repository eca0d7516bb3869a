// Operator-level entry points for the incremental (one token per sequence) call:
// everything LlamaMmha::forward_inc / BaichuanMmha::forward_inc
// (csrc/op/llama_mmha.cpp:202-266, csrc/op/baichuan_mmha.cpp:166-216) and
// GatedFeedForwardNetworkInt8::forward (csrc/op/gated_ffn_int8.cpp:98-132)
// launch, issued from one call each, as the reference's C++ operators do.  At
// decode sizes a token step is ~160 short kernels; driving each through its own
// foreign-function call costs more host time than the kernels take on the GPU
// once the batch is small.
//
// Host code only: the kernels are reached through the library's own C entry
// points, so every argument check and dispatch decision is theirs.
#include <cstddef>
#include <cstdint>

#include "common.h"

namespace {
// do the byte ranges [a, a + an) and [b, b + bn) share a byte?
bool overlaps(const void *a, size_t an, const void *b, size_t bn)
{
    const uintptr_t x = reinterpret_cast<uintptr_t>(a), y = reinterpret_cast<uintptr_t>(b);
    return x < y + bn && y < x + an;
}
}  // namespace

extern "C" size_t eet_mmha_int8_decode_workspace(int B, int H, int dh, int step)
{
    return eet_mmha_decode_workspace(B, H, dh, step);
}

extern "C" int eet_mmha_int8_decode(const void *x, const void *rms_gamma, float rms_eps, const void *qkv_w,
                                    const void *qkv_scale, const void *o_w, const void *o_scale, void *k_cache,
                                    void *v_cache, const void *alibi, const int64_t *pad, const float *rope_cos_sin,
                                    void *qkv_buf, void *ctx_buf, void *out, int B, int H, int dh, int hidden,
                                    int step, int T_cap, void *workspace, size_t workspace_bytes, void *gemm_workspace,
                                    size_t gemm_workspace_bytes, void *stream)
{
    EET_REQUIRE(x && rms_gamma && qkv_buf && ctx_buf && out, EET_ERR_INVALID_ARGUMENT,
                "eet_mmha_int8_decode: null pointer");
    EET_REQUIRE(B > 0 && B <= 32 && H > 0 && dh > 0 && hidden > 0, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_mmha_int8_decode: B=%d must be 1..32 (one token per sequence), H=%d dh=%d hidden=%d", B, H, dh,
                hidden);
    const int inner = H * dh;
    {
        // x is read by the first launch and again, as the residual, by the last; every
        // buffer written in between must stay clear of it and of what the launch that
        // writes it reads
        const size_t xb = (size_t)B * hidden * 2, qb = (size_t)B * 3 * inner * 2, cb = (size_t)B * inner * 2;
        EET_REQUIRE(!overlaps(out, xb, x, xb) && !overlaps(qkv_buf, qb, x, xb) && !overlaps(ctx_buf, cb, x, xb),
                    EET_ERR_INVALID_ARGUMENT,
                    "eet_mmha_int8_decode: out, qkv_buf and ctx_buf must not overlap x (x is the residual of the "
                    "last launch)");
        EET_REQUIRE(!overlaps(ctx_buf, cb, qkv_buf, qb) && !overlaps(out, xb, ctx_buf, cb), EET_ERR_INVALID_ARGUMENT,
                    "eet_mmha_int8_decode: ctx_buf must not overlap qkv_buf, nor out ctx_buf");
    }
    // RMSnorm + QKV projection (llama_mmha.cpp:222-227)
    if (int rc = eet_gemm_w8a16_fused(x, qkv_w, qkv_scale, qkv_buf, B, 3 * inner, hidden, EET_EPILOGUE_NONE, nullptr,
                                      rms_gamma, rms_eps, nullptr, 0, stream))
        return rc;
    // rotary (when a table row is given) + cache append + attention (:229-258): q, k, v are rows of qkv_buf
    const _Float16 *base = static_cast<const _Float16 *>(qkv_buf);
    if (int rc = eet_mmha_decode(base, base + inner, base + 2 * inner, 3L * inner, k_cache, v_cache, ctx_buf, alibi,
                                 pad, B, H, dh, step, T_cap, rope_cos_sin, workspace, workspace_bytes, stream))
        return rc;
    // output projection + residual (:260-262, 428-462)
    return eet_gemm_w8a16_fused(ctx_buf, o_w, o_scale, out, B, hidden, inner, EET_EPILOGUE_RESIDUAL, x, nullptr, 0.f,
                                gemm_workspace, gemm_workspace_bytes, stream);
}

extern "C" int eet_gated_ffn_int8_decode(const void *x, const void *rms_gamma, float rms_eps, const void *w01,
                                         const void *scale01, const void *w2, const void *scale2, void *act_buf,
                                         void *out, int B, int hidden, int d_ff, int add_residual,
                                         void *gemm_workspace, size_t gemm_workspace_bytes, void *stream)
{
    EET_REQUIRE(x && rms_gamma && act_buf && out, EET_ERR_INVALID_ARGUMENT, "eet_gated_ffn_int8_decode: null pointer");
    EET_REQUIRE(B > 0 && B <= 32 && hidden > 0 && d_ff > 0, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_gated_ffn_int8_decode: B=%d must be 1..32 (one token per sequence), hidden=%d d_ff=%d", B, hidden,
                d_ff);
    {
        const size_t xb = (size_t)B * hidden * 2, ab = (size_t)B * d_ff * 2;
        EET_REQUIRE(!overlaps(out, xb, x, xb) && !overlaps(act_buf, ab, x, xb) && !overlaps(out, xb, act_buf, ab),
                    EET_ERR_INVALID_ARGUMENT, "eet_gated_ffn_int8_decode: x, act_buf and out must not overlap");
    }
    // RMSnorm + gate and up projections + SwiGLU (gated_ffn_int8.cpp:112-120): w01 holds gate and up
    // interleaved by 16-channel tile
    if (int rc = eet_gemm_w8a16_fused(x, w01, scale01, act_buf, B, 2 * d_ff, hidden, EET_EPILOGUE_SWIGLU, nullptr,
                                      rms_gamma, rms_eps, nullptr, 0, stream))
        return rc;
    // down projection + residual (:122-128, 303-357)
    return eet_gemm_w8a16_fused(act_buf, w2, scale2, out, B, hidden, d_ff,
                                add_residual ? EET_EPILOGUE_RESIDUAL : EET_EPILOGUE_NONE, add_residual ? x : nullptr,
                                nullptr, 0.f, gemm_workspace, gemm_workspace_bytes, stream);
}

// The same incremental call in its replayable form (see eet_mmha_decode_replayable): recorded once
// into a HIP graph, it serves every later token.
extern "C" int eet_mmha_int8_decode_replayable(const void *x, const void *rms_gamma, float rms_eps, const void *qkv_w,
                                               const void *qkv_scale, const void *o_w, const void *o_scale,
                                               void *k_cache, void *v_cache, const void *alibi, int alibi_ld,
                                               const int64_t *pad, const float *rope_table, void *qkv_buf,
                                               void *ctx_buf, void *out, int B, int H, int dh, int hidden,
                                               const int *step_dev, int step_max, int T_cap, void *workspace,
                                               size_t workspace_bytes, void *gemm_workspace,
                                               size_t gemm_workspace_bytes, void *stream)
{
    EET_REQUIRE(x && rms_gamma && qkv_buf && ctx_buf && out, EET_ERR_INVALID_ARGUMENT,
                "eet_mmha_int8_decode_replayable: null pointer");
    EET_REQUIRE(B > 0 && B <= 32 && H > 0 && dh > 0 && hidden > 0, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_mmha_int8_decode_replayable: B=%d must be 1..32 (one token per sequence), H=%d dh=%d hidden=%d", B,
                H, dh, hidden);
    const int inner = H * dh;
    {
        const size_t xb = (size_t)B * hidden * 2, qb = (size_t)B * 3 * inner * 2, cb = (size_t)B * inner * 2;
        EET_REQUIRE(!overlaps(out, xb, x, xb) && !overlaps(qkv_buf, qb, x, xb) && !overlaps(ctx_buf, cb, x, xb) &&
                        !overlaps(ctx_buf, cb, qkv_buf, qb) && !overlaps(out, xb, ctx_buf, cb),
                    EET_ERR_INVALID_ARGUMENT, "eet_mmha_int8_decode_replayable: x, qkv_buf, ctx_buf and out must not overlap");
    }
    if (int rc = eet_gemm_w8a16_fused(x, qkv_w, qkv_scale, qkv_buf, B, 3 * inner, hidden, EET_EPILOGUE_NONE, nullptr,
                                      rms_gamma, rms_eps, nullptr, 0, stream))
        return rc;
    const _Float16 *base = static_cast<const _Float16 *>(qkv_buf);
    if (int rc = eet_mmha_decode_replayable(base, base + inner, base + 2 * inner, 3L * inner, k_cache, v_cache, ctx_buf,
                                            alibi, alibi_ld, pad, B, H, dh, step_dev, step_max, T_cap, rope_table,
                                            workspace, workspace_bytes, stream))
        return rc;
    return eet_gemm_w8a16_fused(ctx_buf, o_w, o_scale, out, B, hidden, inner, EET_EPILOGUE_RESIDUAL, x, nullptr, 0.f,
                                gemm_workspace, gemm_workspace_bytes, stream);
}
