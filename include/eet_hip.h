/*
 * eet_hip.h -- C ABI of libeet_hip.so: the MI355X (gfx950) implementation of
 * EET's int8 weight-only linear path and the decode attention beside it.
 *
 * This is the boundary a maintainer of the reference binds in place of the
 * pybind11 module `EET` (csrc/py11/eet2py.cpp) and the kernels under csrc/op,
 * csrc/core and 3rdparty/cutlass_kernels that it reaches.  Plain pointers and
 * sizes only; no torch types, no C++ exceptions cross it.
 *
 * Conventions
 *   - every function returns 0 on success and a negative eet_status on failure;
 *     eet_last_error() then returns a thread-local, human-readable message
 *     (the reference throws std::runtime_error: csrc/op/common.hpp:55-64,
 *     3rdparty/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm_template.h:156-176).
 *   - "half" buffers are IEEE binary16, passed as void*.
 *   - device functions enqueue on `stream` (a hipStream_t passed as void*;
 *     NULL = the legacy default stream) and return without synchronising.  The
 *     reference used one private stream (csrc/op/meta_desc.hpp:58-60); here the
 *     caller supplies its own.
 *   - weights are [K = in_features, N = out_features] (the reference's
 *     convention, python/eet/transformers/modeling_llama.py:764-766).
 */
#ifndef EET_HIP_H
#define EET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum eet_status {
    EET_OK = 0,
    EET_ERR_INVALID_ARGUMENT = -1, /* null pointer, negative size, bad enum */
    EET_ERR_UNSUPPORTED_SHAPE = -2, /* shape the kernels cannot take (e.g. K % 64 != 0) */
    EET_ERR_HIP = -3,               /* a HIP runtime call failed */
    EET_ERR_WORKSPACE = -4          /* workspace missing or too small */
} eet_status;

enum { EET_DTYPE_F32 = 0, EET_DTYPE_F16 = 1 };
enum { EET_QUANT_REF128 = 0, EET_QUANT_SYM127 = 1 };

/* Message of the last failure on the calling thread ("" if none). */
const char *eet_last_error(void);

/* Version tag of the packed weight layout produced by eet_pack_gfx950. */
int eet_packed_layout_version(void);

/* Overrides one of the library's launch-shape tables, for sweeps and for tests
 * that run every kernel variant; value NULL or "" restores the table.  Keys:
 *   EET_GEMM_SMALL_M_CONFIG "nt,waves,u[,ksplit]"   EET_GEMM_LARGE_M_TILE "tm,tn[,ksplit]"
 *   EET_MMHA_NSPLIT / EET_MMHA_THREADS / EET_MMHA_UNROLL "n"
 *   EET_PREFILL_LEGACY "1" (register-staged prefill attention at head size 128)
 *   EET_PREFILL_SHAPE "1" | "2" (launch shape of the head-size-128 prefill kernel)
 *   EET_PREFILL_GROUP "n" ((batch, head) pairs whose query blocks an XCD works on together in prefill
 *                         attention; "-1": every pair of a query block before the next block)
 *   EET_CHAIN_SPIN_LIMIT "n" / EET_CHAIN_SLEEP "n" (bounded wait of a chained launch)
 * An override naming a kernel variant that does not exist is ignored.  The same
 * keys are read from the environment once, at load, when EET_HIP_TUNING=1; no
 * launch reads the environment (the reference queries occupancy and runs its
 * heuristic on every call: fpA_intB_gemm_template.h:460-491).  Process-wide and
 * not synchronised: call it while no launch of this library is being issued. */
int eet_set_tuning(const char *name, const char *value);

/* ------------------------------------------------------------------------
 * Offline weight packer (host CPU, no GPU needed).
 * ---------------------------------------------------------------------- */

/* Per-output-channel symmetric int8 quantisation of w[K][N] (row-major,
 * w_dtype = EET_DTYPE_F32 or EET_DTYPE_F16).  Writes q[K][N] (row-major,
 * "unprocessed") and scale[N] in w's dtype.
 *   EET_QUANT_REF128: bit-exact with the reference quantiser: scale =
 *     absmax / 128, q = clamp(round(w / scale_fp32), -128, 127).
 *   EET_QUANT_SYM127: scale = absmax / 127, q in [-127, 127]; zero column -> 0.
 * Replaces ft::symmetric_quantize, int8 branch
 * (3rdparty/cutlass_kernels/cutlass_preprocessors.cc:581-678), reached from
 * symmetric_quantize_last_axis_of_tensor
 * (3rdparty/cutlass_kernels/fpA_intB_gemm_wrapper.cu:26-105). */
int eet_quantize_int8(const void *w, int w_dtype, size_t K, size_t N, int mode,
                      int8_t *q, void *scale);

/* Permute q[K][N] into the gfx950 tile-interleaved layout the GEMM kernels
 * read (K % 64 == 0, N % 16 == 0; same byte count).  Replaces
 * preprocess_weights_for_mixed_gemm (cutlass_preprocessors.cc:497-534), whose
 * sm75/sm80 layout has no meaning on gfx950.  eet_unpack_gfx950 is the inverse. */
int eet_pack_gfx950(const int8_t *q, size_t K, size_t N, int8_t *packed);
int eet_unpack_gfx950(const int8_t *packed, size_t K, size_t N, int8_t *q);

/* The reference's own processed layout for sm75..sm89 and its inverse, so that
 * int8 state dicts saved by the reference (cutlass_preprocessors.cc:497-534;
 * K % 64 == 0 and N % 64 == 0) can be re-packed for gfx950. */
int eet_preprocess_ref_sm80(const int8_t *q, size_t K, size_t N, int8_t *processed);
int eet_unprocess_ref_sm80(const int8_t *processed, size_t K, size_t N, int8_t *q);

/* ------------------------------------------------------------------------
 * Device kernels (gfx950).
 * ---------------------------------------------------------------------- */

/* The packer on the GPU, for weights that already live in HBM: w[K][N]
 * (row-major, w_dtype as above, K % 64 == 0, N % 16 == 0) -> packed[K][N] in the
 * gfx950 layout, scale[N] in w's dtype and, when q is not NULL, the
 * unprocessed q[K][N]; all device pointers.  Bit-identical to
 * eet_quantize_int8 followed by eet_pack_gfx950 in both modes.  workspace:
 * eet_quantize_pack_device_workspace(N) bytes of device memory.  The reference
 * quantises on one host core only (cutlass_preprocessors.cc:581-678, reached
 * from fpA_intB_gemm_wrapper.cu:26-105, which rejects CUDA tensors at :33);
 * this entry point has no counterpart there. */
size_t eet_quantize_pack_device_workspace(size_t N);
int eet_quantize_pack_device(const void *w, int w_dtype, size_t K, size_t N, int mode,
                             int8_t *q, int8_t *packed, void *scale, void *workspace,
                             size_t workspace_bytes, void *stream);

/* C[M][N] (half) = A[M][K] (half) . (int8 W[K][N] * scale[N] (half)), fp32
 * accumulation, one rounding to half.  Wpacked comes from eet_pack_gfx950.
 * M <= 32 takes the HBM-streaming small-M kernel, larger M the LDS-staged MFMA
 * kernel.  The workspace is optional (NULL / 0 accepted): with
 * eet_gemm_w8a16_workspace(M, N, K, epilogue) bytes of 16-byte aligned device
 * memory the library may split the k range of a launch -- the reference's
 * split-k workspace, which its callers never pass
 * (fpA_intB_gemm_template.h:443-495, cutlass_heuristic.cc:80-84):
 *   M > 32   a launch that has too few tiles to fill the chip (M in the tens to
 *            hundreds): raw fp32 sums, added in a second small kernel;
 *   M <= 32  a launch without the RMSnorm prologue whose N leaves about one 16-channel
 *            tile per CU (the O and down projections at N = 4096 / 5120): 2 or 4
 *            workgroups share a group of tiles, exchange their fp32 sums through the
 *            workspace and the last one to arrive finishes them -- one launch.
 *            For this use the first 32 KiB of the workspace (its arrival counters)
 *            must be ZERO before the first call that is handed the workspace; every
 *            call leaves them zero.  Keep such a workspace for
 *            M <= 32 calls only (an M > 32 call writes partial sums over the
 *            counters), and never hand one workspace to two calls that can overlap
 *            in time.
 * Replaces fastertransformer::gemm_fp16_int_bias_act<uint8_t>
 * (3rdparty/cutlass_kernels/fpA_intB_gemm.cu:35-62) as called with
 * bias = nullptr and no activation from csrc/op/llama_mmha.cpp:313-337,
 * 428-447 and csrc/op/gated_ffn_int8.cpp:253-326. */
int eet_gemm_w8a16(const void *A, const void *Wpacked, const void *scale, void *C,
                   int M, int N, int K, void *workspace, size_t workspace_bytes,
                   void *stream);
size_t eet_gemm_w8a16_workspace(int M, int N, int K, int epilogue);

/* The same GEMM with a fused epilogue.
 *   EET_EPILOGUE_NONE      C[M][N] as above.
 *   EET_EPILOGUE_RESIDUAL  C[M][N] = half(A.W) + residual[M][N] (fp16 add): the
 *       GEMM followed by add_bias_input_kernel with bias == nullptr, as at
 *       csrc/op/llama_mmha.cpp:428-462 and csrc/op/gated_ffn_int8.cpp:303-357.
 *   EET_EPILOGUE_SWIGLU    Wpacked / scale hold gate and up interleaved by
 *       16-channel tile (tile 2i = gate tile i, tile 2i+1 = up tile i; N =
 *       2 * d_ff); C[M][N/2] = up * gate / (1 + exp(-gate)): the two GEMMs and
 *       gated_act_kernel of csrc/op/gated_ffn_int8.cpp:253-301, 168-179 in one
 *       launch.  In the packed layout a 16-channel tile is one contiguous run of
 *       K*16 bytes, so interleaving is a row-wise merge of the two packed matrices.
 * residual must be NULL unless the epilogue is EET_EPILOGUE_RESIDUAL.
 * RMSnorm prologue (rms_gamma != NULL, M <= 32): A is the un-normalised input
 * and the result is that of eet_rmsnorm(A, rms_gamma, rms_eps) followed by the
 * GEMM -- the RMSnorm + GEMM pairs at csrc/op/llama_mmha.cpp:222-227 and
 * csrc/op/gated_ffn_int8.cpp:112-116 in one launch.  The kernel multiplies
 * x * gamma in fp16 on the way in, accumulates sum(x^2) per row, and applies
 * rsqrt(mean + eps) to the fp32 accumulator.
 * workspace / workspace_bytes as for eet_gemm_w8a16 (optional). */
enum { EET_EPILOGUE_NONE = 0, EET_EPILOGUE_RESIDUAL = 1, EET_EPILOGUE_SWIGLU = 2 };
int eet_gemm_w8a16_fused(const void *A, const void *Wpacked, const void *scale, void *C,
                         int M, int N, int K, int epilogue, const void *residual,
                         const void *rms_gamma, float rms_eps, void *workspace,
                         size_t workspace_bytes, void *stream);

/* The launch shape the small-M kernel (1 <= M <= 32) runs a call with: n-tiles per
 * workgroup, wavefronts per workgroup, k-tiles per register batch, and how many
 * workgroups share a tile's k range (1, 2 or 4; what a call runs with when it hands
 * over the workspace eet_gemm_w8a16_workspace asks for -- without it, 1) -- the tuning
 * override EET_GEMM_SMALL_M_CONFIG when a kernel of that shape exists for the
 * call, otherwise the table's choice.  For sweeps and for tests that must know
 * which variant ran.  It also checks, on the host, that the library holds a kernel
 * for what the table answers in every form of the call (with the workspace,
 * without it, chained) and fails with EET_ERR_INVALID_ARGUMENT if not.  The
 * reference's counterpart is the CutlassGemmConfig its
 * heuristic returns (cutlass_heuristic.cc:106-207). */
int eet_gemm_w8a16_small_m_shape(int M, int N, int K, int epilogue, int rms_prologue, int *nt,
                                 int *waves, int *k_tiles_per_batch, int *k_split);

/* Chained launches (1 <= M <= 32): eet_gemm_w8a16_fused for a sequence of launches
 * in which each reads what the previous one wrote -- the decode step of
 * csrc/op/llama_mmha.cpp:202-266 and csrc/op/gated_ffn_int8.cpp:98-132, which the
 * reference issues as serial launches on one stream.
 *   EET_CHAIN_FIRST  an ordinary launch (ordered behind all earlier work of the
 *                    stream) that also publishes a completion counter.
 *   EET_CHAIN_NEXT   enqueued without the queue's barrier: the kernel may start
 *                    while earlier launches of the stream still run, requests its
 *                    first weight batches, and then waits IN THE KERNEL for the
 *                    completion counter of the previous chained launch (which must
 *                    have been made on the same stream of the same device) before it
 *                    reads A or the residual rows.
 * Contract of a NEXT launch: everything it reads was written by the previous
 * chained launch or earlier, and no other work that it depends on, or that
 * depends on it, is enqueued on the stream between the two.  Ordinary launches
 * that follow a chain are ordered behind all of it as usual.  Outputs are written
 * with agent-scope stores and inputs read with agent-scope loads (coherent across
 * the XCDs' L2 caches); results are bit-identical to eet_gemm_w8a16_fused.
 * The wait is bounded: after EET_CHAIN_SPIN_LIMIT polls (eet_set_tuning; default
 * 65536, about 20 ms) a workgroup gives up, sets a device error word and goes on,
 * so that every kernel exits; the results of the chain are then undefined and
 * eet_chain_status reports it.  Not for streams that are being captured into a
 * HIP graph (refused).  A GPU that other processes or streams keep busy can delay
 * a producer for longer than the bound: chain only on a GPU the caller owns. */
enum { EET_CHAIN_OFF = 0, EET_CHAIN_FIRST = 1, EET_CHAIN_NEXT = 2 };
int eet_gemm_w8a16_chained(const void *A, const void *Wpacked, const void *scale, void *C,
                           int M, int N, int K, int epilogue, const void *residual,
                           const void *rms_gamma, float rms_eps, int chain, void *stream);

/* Waits for `stream`, then *gave_up = 1 if any chained wait on the current device
 * has given up since the word was last cleared (0 otherwise); clear != 0 resets it. */
int eet_chain_status(int *gave_up, int clear, void *stream);

/* Masked multi-head decode attention for one new token per sequence.
 *   dh        32, 64, 96 or 128, the head sizes the reference instantiates
 *   q, k, v   [B][H][dh] half; with qkv_stride != 0 they are rows of a fused
 *             buffer: element (b, h, d) at base[b * qkv_stride + h * dh + d]
 *   k_cache, v_cache  [B_cap][H][T_cap][dh] half; the new k, v are appended at
 *             row step-1, rows [0, step) are attended
 *   alibi     NULL or [H][step] half, added to the scaled logits
 *   pad       NULL or [B] int64: rows t < pad[b] get zero weight
 *   ctx       [B][H*dh] half
 *   rope_cos_sin  NULL, or the row of the eet_rope_table table for this token's
 *             position (dh floats: cos[dh/2] | sin[dh/2]); q and the appended k
 *             are then rotated NeoX-style in the kernel, which stands in for
 *             fused_QKV_neox_rotary_transpose (csrc/core/self_add_bias.cu:369-403)
 *             at decode time.  Needs k, v != NULL.
 *   workspace eet_mmha_decode_workspace(B, H, dh, step) bytes of device memory
 * softmax denominator carries the reference's + 1e-6.
 * Replaces masked_attention_dispatch (csrc/core/attention_dispatch.cu:888-928)
 * and fused_masked_attention_dispatch with q_bias == nullptr (:1338-1426). */
size_t eet_mmha_decode_workspace(int B, int H, int dh, int step);
int eet_mmha_decode(const void *q, const void *k, const void *v, long qkv_stride,
                    void *k_cache, void *v_cache, void *ctx, const void *alibi,
                    const int64_t *pad, int B, int H, int dh, int step, int T_cap,
                    const float *rope_cos_sin, void *workspace, size_t workspace_bytes,
                    void *stream);

/* eet_mmha_decode for callers that cannot allocate device memory or carry a
 * workspace around: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * arguments and results as eet_mmha_decode, without the workspace: the partial
 * results of a split launch (B*H < 256) live in a static device array of
 * eet_mmha_decode_static_capacity() bytes (260 KiB) that every GPU the library
 * runs on holds until the process ends.  Calls no hipMalloc / hipFree.  A call
 * whose B*H*nsplit*(dh+2)*4 bytes exceed the capacity (only reachable through a
 * tuning override) fails with EET_ERR_WORKSPACE.  All calls on one GPU share the
 * array: calls that overlap in time on different streams of one GPU race;
 * nothing needs clearing between calls.  The first call on each GPU looks the
 * array's device address up (hipGetSymbolAddress, a runtime query that may load
 * the code object): make that first call OUTSIDE a stream capture (one warm call
 * per device; eet_mmha_decode_static_capacity() does not count, it touches no
 * device).  `stream` must belong to the device that is current at the call. */
size_t eet_mmha_decode_static_capacity(void);
int eet_mmha_decode_static(const void *q, const void *k, const void *v, long qkv_stride,
                           void *k_cache, void *v_cache, void *ctx, const void *alibi,
                           const int64_t *pad, int B, int H, int dh, int step, int T_cap,
                           const float *rope_cos_sin, void *stream);

/* table[t][0 .. dh/2) = cos(t / 10000^(2i/dh)), table[t][dh/2 .. dh) = sin(...),
 * t in [0, T): the rotary coefficients of csrc/core/common.cuh:176-180 in fp32. */
int eet_rope_table(float *table, int T, int dh, void *stream);

/* out[M][N] = x * rsqrt(mean(x^2) + eps) * gamma.  Replaces RMSnorm
 * (csrc/core/layer_norm.cu:580-625). */
int eet_rmsnorm(const void *x, const void *gamma, void *out, int M, int N, float eps,
                void *stream);

/* out[M][N] = (x - mean(x)) * rsqrt(var(x) + eps) * gamma + beta: the LayerNorm the
 * ops use instead of RMSnorm when they are given biases.  fp32 statistics (mean,
 * then the variance of the centred values), one rounding.  Replaces layernorm
 * (csrc/core/layer_norm.cu:533-578, kernel :384-446). */
int eet_layernorm(const void *x, const void *gamma, const void *beta, void *out, int M, int N,
                  float eps, void *stream);

/* In place: out[M][N] = norm((out + input) [+ bias]) with the two adds in fp16 as the
 * reference makes them; norm is LayerNorm(gamma, beta) when beta is given and
 * RMSnorm(gamma) when beta is NULL; bias may be NULL.  The post-layernorm tail of
 * the feed-forward op.  Replaces add_bias_input_layernorm_kernel
 * (csrc/core/layer_norm.cu:627-668; kernels :39-80 and :103-131) without its
 * N <= 2048 limit. */
int eet_add_bias_residual_norm(void *out, const void *input, const void *bias, const void *gamma,
                               const void *beta, int M, int N, float eps, void *stream);

/* out[M][N] += bias[N] (fp16 add).  Replaces add_bias_kernel
 * (csrc/core/add_bias.cu:30-49) and the bias half of add_bias_input_kernel (:51-73). */
int eet_add_bias(void *out, const void *bias, int M, int N, void *stream);

/* Split a fused qkv[B][S][3][H][dh] row.  With rope != 0, q and k are rotated
 * NeoX-style (pairs i, i + dh/2) at position s (time_step < 0) or time_step.
 *   q_out  [B][H][S][dh]
 *   k and v go straight into the caches [B_cap][H][T_cap][dh] at rows
 *   t0 + s (t0 = 0 for prefill, step-1 for decode).
 * Replaces fused_QKV_bias_rotary_kernel / fused_QKV_transpose
 * (csrc/core/self_add_bias.cu:442-487, 303-360) plus copyKV_transpose
 * (csrc/core/transpose.cu:116-124). */
int eet_qkv_split(const void *qkv, void *q_out, void *k_cache, void *v_cache, int B, int S,
                  int H, int dh, int rope, int time_step, int t0, int T_cap, void *stream);

/* gate[M][N] = up * gate / (1 + exp(-gate)).  Replaces gated_act_kernel, silu
 * (csrc/core/activation_kernel.cu:275-338). */
int eet_swiglu(void *gate, const void *up, int M, int N, void *stream);

/* out[M][N] += residual[M][N].  Replaces add_bias_input_kernel with
 * bias == nullptr (csrc/core/add_bias.cu:51-73). */
int eet_residual_add(void *out, const void *residual, int M, int N, void *stream);

/* Beam-search cache reorder: dst[b][h][t][:] = src[reorder_index[b]][h][t][:]
 * for t < rows, K and V, caches [B][H][T_cap][dh] half, reorder_index int64[B]
 * in device memory (an entry outside [0, B) keeps the beam's own rows).  src
 * and dst must not overlap: the caller keeps two cache buffers and swaps them.
 * Replaces reorderKV_kernel (csrc/core/transpose.cu:135-162) as called from
 * LlamaMmha::reorder_cache (csrc/op/llama_mmha.cpp:248-252, 495-508), whose
 * in-place form does not order its reads before its writes. */
int eet_kv_cache_reorder(const void *k_src, const void *v_src, void *k_dst, void *v_dst,
                         const int64_t *reorder_index, int B, int H, int dh, int rows, int T_cap,
                         void *stream);

/* One incremental call (one new token per sequence, B <= 32) of the attention
 * sub-layer, all launches from one call: RMSnorm + QKV projection, rotary (when
 * rope_cos_sin is given) + cache append + masked attention, output projection +
 * residual.  x [B][hidden] is both the input and the residual; qkv_buf
 * [B][3*H*dh] and ctx_buf [B][H*dh] are scratch; out [B][hidden] must not
 * alias x.  Weights are packed int8 [hidden][3*H*dh] and [H*dh][hidden] with
 * their fp16 scales; the other arguments are those of eet_mmha_decode.
 * gemm_workspace: optional (NULL / 0), the eet_gemm_w8a16 workspace of the output
 * projection, eet_gemm_w8a16_workspace(B, hidden, H*dh, EET_EPILOGUE_RESIDUAL) bytes
 * under that function's rules (counters zero before first use).
 * Replaces LlamaMmha::forward_inc (csrc/op/llama_mmha.cpp:202-266) and
 * BaichuanMmha::forward_inc (csrc/op/baichuan_mmha.cpp:166-216) without the
 * beam reorder, which stays a separate call (eet_kv_cache_reorder). */
size_t eet_mmha_int8_decode_workspace(int B, int H, int dh, int step);
int eet_mmha_int8_decode(const void *x, const void *rms_gamma, float rms_eps, const void *qkv_w,
                         const void *qkv_scale, const void *o_w, const void *o_scale,
                         void *k_cache, void *v_cache, const void *alibi, const int64_t *pad,
                         const float *rope_cos_sin, void *qkv_buf, void *ctx_buf, void *out,
                         int B, int H, int dh, int hidden, int step, int T_cap, void *workspace,
                         size_t workspace_bytes, void *gemm_workspace, size_t gemm_workspace_bytes,
                         void *stream);

/* The gated FFN sub-layer for B <= 32 rows, both launches from one call:
 * RMSnorm + gate and up projections + SwiGLU (w01 / scale01: gate and up
 * interleaved by 16-channel tile, [hidden][2*d_ff]), then the down projection
 * (+ x when add_residual).  act_buf [B][d_ff] is scratch; out [B][hidden] must
 * not alias x.  gemm_workspace: optional (NULL / 0), the eet_gemm_w8a16 workspace of
 * the down projection, eet_gemm_w8a16_workspace(B, hidden, d_ff, epilogue) bytes under
 * that function's rules.  Replaces GatedFeedForwardNetworkInt8::forward
 * (csrc/op/gated_ffn_int8.cpp:98-132) at decode sizes. */
int eet_gated_ffn_int8_decode(const void *x, const void *rms_gamma, float rms_eps, const void *w01,
                              const void *scale01, const void *w2, const void *scale2,
                              void *act_buf, void *out, int B, int hidden, int d_ff,
                              int add_residual, void *gemm_workspace, size_t gemm_workspace_bytes,
                              void *stream);

/* Causal prefill attention over the prompt, reading K and V from the caches
 * filled by eet_qkv_split.  q [B][H][S][dh]; ctx [B][S][H*dh]; alibi NULL or
 * [H][S] half (slope * j, the diagonal row of the reference's mask); pad as in
 * eet_mmha_decode (padded query rows give zeros).  Replaces the unfused
 * QK^T / softmax / PV / transpose sequence of csrc/op/llama_mmha.cpp:160-186
 * and csrc/op/baichuan_mmha.cpp:120-150. */
int eet_prefill_attention(const void *q, const void *k_cache, const void *v_cache, void *ctx,
                          const void *alibi, const int64_t *pad, int B, int H, int S, int dh,
                          int T_cap, void *stream);

/* Replayable forms of the incremental attention call, for a decode step that is
 * recorded once into a HIP graph and replayed for every token (the reference
 * re-issues the launch sequence of csrc/op/llama_mmha.cpp:202-266 from the host
 * for every token).  What changes from step to step lives in device memory:
 *   step_dev    int32 in device memory: the step of this call (rows attended,
 *               the new token included); eet_step_advance(step_dev, 1, stream)
 *               recorded ahead of the layers moves it on at each replay.  The
 *               kernel clamps the value it reads into [1, step_max]: a replay past
 *               step_max repeats step_max instead of reading past the tables
 *   step_max    the largest step the recording will be replayed at (<= T_cap):
 *               launch shape and workspace are chosen for it
 *   rope_table  NULL or the BASE of the eet_rope_table table (>= step_max rows):
 *               the kernel picks row step-1 itself
 *   alibi       NULL or [H][alibi_ld] half with alibi_ld >= step_max
 * Everything else is as in eet_mmha_decode / eet_mmha_int8_decode; results are
 * bit-identical to those calls at the same step when the launch shapes agree. */
int eet_step_advance(int *step_dev, int by, void *stream);
size_t eet_mmha_decode_replayable_workspace(int B, int H, int dh, int step_max);
int eet_mmha_decode_replayable(const void *q, const void *k, const void *v, long qkv_stride,
                               void *k_cache, void *v_cache, void *ctx, const void *alibi,
                               int alibi_ld, const int64_t *pad, int B, int H, int dh,
                               const int *step_dev, int step_max, int T_cap,
                               const float *rope_table, void *workspace, size_t workspace_bytes,
                               void *stream);
int eet_mmha_int8_decode_replayable(const void *x, const void *rms_gamma, float rms_eps,
                                    const void *qkv_w, const void *qkv_scale, const void *o_w,
                                    const void *o_scale, void *k_cache, void *v_cache,
                                    const void *alibi, int alibi_ld, const int64_t *pad,
                                    const float *rope_table, void *qkv_buf, void *ctx_buf, void *out,
                                    int B, int H, int dh, int hidden, const int *step_dev,
                                    int step_max, int T_cap, void *workspace, size_t workspace_bytes,
                                    void *gemm_workspace, size_t gemm_workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* EET_HIP_H */
