// Offline weight packer (host only): per-output-channel symmetric int8
// quantisation and the gfx950 tile-interleaved layout.
//
// Quantiser semantics follow the reference's symmetric_quantize, int8 branch
// (3rdparty/cutlass_kernels/cutlass_preprocessors.cc:581-678); the work is
// split over host threads by column blocks, which cannot change any result
// because every column is independent.
//
// gfx950 layout, version 1.  The [K][N] int8 matrix is cut into tiles of
// 16 output channels x 64 input features (1 KiB).  Tiles are stored
// [n_tile][k_tile]; inside a tile, byte 16*lane + b (lane = 16*g + i, g in
// 0..3, i in 0..15) holds  q[64*k_tile + 16*g + b][16*n_tile + i] XOR 0x80.
// So one 64-lane wavefront fetches a whole tile with a single 128-bit load per
// lane, each lane receives 16 consecutive-k weights of one output channel --
// two ready-made 8-element operands of v_mfma_f32_16x16x32_f16 -- and the
// XOR 0x80 bias (q + 128 as an unsigned byte) lets the kernel widen a byte to
// fp16 with one byte-permute into 0x6400 | u8 (= 1024 + u8) and one packed
// subtract of 1152.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "common.h"

namespace eet {
std::string &last_error_slot()
{
    thread_local std::string s;
    return s;
}
}  // namespace eet

namespace {

constexpr int kLayoutVersion = 1;
constexpr size_t kTileN = 16, kTileK = 64;

template <typename F>
void parallel_for(size_t n, size_t grain, F f)
{
    size_t hw = std::max(1u, std::min(16u, std::thread::hardware_concurrency()));
    size_t chunks = std::min(hw, (n + grain - 1) / std::max<size_t>(grain, 1));
    if (chunks <= 1) {
        f(size_t(0), n);
        return;
    }
    std::vector<std::thread> th;
    size_t per = (n + chunks - 1) / chunks;
    for (size_t c = 0; c < chunks; ++c) {
        size_t lo = c * per, hi = std::min(n, lo + per);
        if (lo >= hi)
            break;
        th.emplace_back([=] { f(lo, hi); });
    }
    for (auto &t : th)
        t.join();
}

// The three row loops below are compiled twice, for the baseline x86-64 ISA and
// for AVX2 + F16C (chosen at load time): without F16C every fp16 -> fp32
// conversion is a library call.  Both versions do the same IEEE operations in the
// same order (no multiply-add pairs that could be contracted), so the results are
// identical bit for bit.
#define EET_ISA_CLONES __attribute__((target_clones("arch=x86-64-v3", "default")))

inline float widen(float x) { return x; }
inline float widen(_Float16 x) { return static_cast<float>(x); }

template <typename T>
inline void absmax_row(const T *row, size_t nc, float *s)
{
    for (size_t j = 0; j < nc; ++j) {
        const float a = std::fabs(widen(row[j]));
        s[j] = (s[j] < a) ? a : s[j];
    }
}

// round-half-away-from-zero of x / s, clamped to [lo, 127]; nan_to is what a NaN
// quotient (0 / 0 in an all-zero column) becomes.  Truncation through int32 is
// exact once the quotient is clamped to +-200 (which cannot change the clamped
// result), and v - trunc(v) is exact, so this equals clamp(std::round(x / s)).
template <typename T>
inline void quant_row(const T *row, const float *s, size_t nc, int8_t *q, float nan_to, int lo)
{
    for (size_t j = 0; j < nc; ++j) {
        float v = widen(row[j]) / s[j];
        v = (v == v) ? v : nan_to;
        v = (v < 200.f) ? v : 200.f;
        v = (v > -200.f) ? v : -200.f;
        int t = static_cast<int>(v);
        const float d = v - static_cast<float>(t);
        t += (d >= 0.5f) ? 1 : 0;
        t -= (d <= -0.5f) ? 1 : 0;
        t = (t < 127) ? t : 127;
        t = (t > lo) ? t : lo;
        q[j] = static_cast<int8_t>(t);
    }
}

EET_ISA_CLONES void absmax_rows_f16(const _Float16 *w, size_t K, size_t N, size_t nc, float *s)
{
    for (size_t k = 0; k < K; ++k)
        absmax_row(w + k * N, nc, s);
}
EET_ISA_CLONES void absmax_rows_f32(const float *w, size_t K, size_t N, size_t nc, float *s)
{
    for (size_t k = 0; k < K; ++k)
        absmax_row(w + k * N, nc, s);
}
EET_ISA_CLONES void quant_rows_f16(const _Float16 *w, size_t K, size_t N, size_t nc, const float *s, int8_t *q,
                                   float nan_to, int lo)
{
    for (size_t k = 0; k < K; ++k)
        quant_row(w + k * N, s, nc, q + k * N, nan_to, lo);
}
EET_ISA_CLONES void quant_rows_f32(const float *w, size_t K, size_t N, size_t nc, const float *s, int8_t *q,
                                   float nan_to, int lo)
{
    for (size_t k = 0; k < K; ++k)
        quant_row(w + k * N, s, nc, q + k * N, nan_to, lo);
}
inline void absmax_rows(const _Float16 *w, size_t K, size_t N, size_t nc, float *s) { absmax_rows_f16(w, K, N, nc, s); }
inline void absmax_rows(const float *w, size_t K, size_t N, size_t nc, float *s) { absmax_rows_f32(w, K, N, nc, s); }
inline void quant_rows(const _Float16 *w, size_t K, size_t N, size_t nc, const float *s, int8_t *q, float nan_to, int lo)
{
    quant_rows_f16(w, K, N, nc, s, q, nan_to, lo);
}
inline void quant_rows(const float *w, size_t K, size_t N, size_t nc, const float *s, int8_t *q, float nan_to, int lo)
{
    quant_rows_f32(w, K, N, nc, s, q, nan_to, lo);
}

// Columns [c0, c1): absmax per column, then the quotients.  EET_QUANT_REF128 is
// the reference's quantiser (cutlass_preprocessors.cc:581-678): scale = absmax /
// 128, clamp to [-128, 127], and an all-zero column (0 / 0) comes out as 127
// because the reference's std::min / std::max pass NaN through to the cast that
// way round; EET_QUANT_SYM127 divides by 127, clamps to +-127 and maps NaN to 0.
template <typename T>
void quantize_cols(const T *w, size_t K, size_t N, int mode, int8_t *q, T *scale, size_t c0, size_t c1)
{
    const size_t nc = c1 - c0;
    std::vector<float> s(nc, 0.f);
    absmax_rows(w + c0, K, N, nc, s.data());
    const bool ref = mode == EET_QUANT_REF128;
    for (size_t j = 0; j < nc; ++j) {
        s[j] = ref ? s[j] * (1.f / 128.f) : s[j] / 127.f;
        scale[c0 + j] = static_cast<T>(s[j]);
    }
    quant_rows(w + c0, K, N, nc, s.data(), q + c0, ref ? 1000.f : 0.f, ref ? -128 : -127);
}

// flat [K][N] index held by byte p of the reference's sm80 processed buffer:
// row permutation inside 16-row groups (cutlass_preprocessors.cc:182-183),
// transpose to [N][K], interleave of two columns in 64-row tiles (:474-493),
// swap of bytes 1 and 2 in every 4 (:355-357).
inline size_t ref_sm80_source(size_t p, size_t K, size_t N)
{
    size_t b = p & 3;
    b = (b == 1) ? 2 : (b == 2) ? 1 : b;
    const size_t word = p >> 2;
    const size_t nvr = K / 4;               // 32-bit words per column
    const size_t wcol = word / (nvr * 2);   // interleaved column pair
    const size_t wrow = word % (nvr * 2);
    const size_t base = (wrow / 32) * 16;   // first word row of the 64-row tile
    const size_t within = wrow % 32;
    const size_t col = wcol * 2 + within / 16;
    const size_t vrow = base + within % 16;
    const size_t prow = vrow * 4 + b;       // row after the 16-row permutation
    const size_t r = prow % 16;
    const size_t src_row = (prow - r) + 8 * ((r % 4) / 2) + r % 2 + 2 * (r / 4);
    return src_row * N + col;
}

}  // namespace

extern "C" {

const char *eet_last_error(void) { return eet::last_error_slot().c_str(); }

int eet_packed_layout_version(void) { return kLayoutVersion; }

int eet_quantize_int8(const void *w, int w_dtype, size_t K, size_t N, int mode, int8_t *q, void *scale)
{
    EET_REQUIRE(w && q && scale, EET_ERR_INVALID_ARGUMENT, "eet_quantize_int8: null pointer");
    EET_REQUIRE(w_dtype == EET_DTYPE_F32 || w_dtype == EET_DTYPE_F16, EET_ERR_INVALID_ARGUMENT,
                "eet_quantize_int8: w_dtype must be EET_DTYPE_F32 or EET_DTYPE_F16, got %d", w_dtype);
    EET_REQUIRE(mode == EET_QUANT_REF128 || mode == EET_QUANT_SYM127, EET_ERR_INVALID_ARGUMENT,
                "eet_quantize_int8: unknown mode %d", mode);
    if (N == 0)
        return EET_OK;
    if (w_dtype == EET_DTYPE_F32) {
        parallel_for(N, 64, [=](size_t lo, size_t hi) {
            quantize_cols(static_cast<const float *>(w), K, N, mode, q, static_cast<float *>(scale), lo, hi);
        });
    } else {
        parallel_for(N, 64, [=](size_t lo, size_t hi) {
            quantize_cols(static_cast<const _Float16 *>(w), K, N, mode, q, static_cast<_Float16 *>(scale), lo, hi);
        });
    }
    return EET_OK;
}

static int check_pack_shape(const char *fn, const void *a, const void *b, size_t K, size_t N)
{
    EET_REQUIRE(a && b, EET_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
    EET_REQUIRE(K > 0 && N > 0 && K % kTileK == 0 && N % kTileN == 0, EET_ERR_UNSUPPORTED_SHAPE,
                "%s: need K %% 64 == 0 and N %% 16 == 0, got K=%zu N=%zu", fn, K, N);
    return EET_OK;
}

int eet_pack_gfx950(const int8_t *q, size_t K, size_t N, int8_t *packed)
{
    if (int rc = check_pack_shape("eet_pack_gfx950", q, packed, K, N))
        return rc;
    const size_t kt_n = K / kTileK, nt_n = N / kTileN;
    parallel_for(nt_n, 4, [=](size_t lo, size_t hi) {
        for (size_t nt = lo; nt < hi; ++nt)
            for (size_t kt = 0; kt < kt_n; ++kt) {
                uint8_t *tile = reinterpret_cast<uint8_t *>(packed) + (nt * kt_n + kt) * 1024;
                for (size_t g = 0; g < 4; ++g)
                    for (size_t b = 0; b < 16; ++b) {
                        const int8_t *src = q + (kt * 64 + g * 16 + b) * N + nt * 16;
                        for (size_t i = 0; i < 16; ++i)
                            tile[(g * 16 + i) * 16 + b] = static_cast<uint8_t>(src[i]) ^ 0x80u;
                    }
            }
    });
    return EET_OK;
}

int eet_unpack_gfx950(const int8_t *packed, size_t K, size_t N, int8_t *q)
{
    if (int rc = check_pack_shape("eet_unpack_gfx950", q, packed, K, N))
        return rc;
    const size_t kt_n = K / kTileK, nt_n = N / kTileN;
    parallel_for(nt_n, 4, [=](size_t lo, size_t hi) {
        for (size_t nt = lo; nt < hi; ++nt)
            for (size_t kt = 0; kt < kt_n; ++kt) {
                const uint8_t *tile = reinterpret_cast<const uint8_t *>(packed) + (nt * kt_n + kt) * 1024;
                for (size_t g = 0; g < 4; ++g)
                    for (size_t b = 0; b < 16; ++b) {
                        int8_t *dst = q + (kt * 64 + g * 16 + b) * N + nt * 16;
                        for (size_t i = 0; i < 16; ++i)
                            dst[i] = static_cast<int8_t>(tile[(g * 16 + i) * 16 + b] ^ 0x80u);
                    }
            }
    });
    return EET_OK;
}

static int check_ref_shape(const char *fn, const void *a, const void *b, size_t K, size_t N)
{
    EET_REQUIRE(a && b, EET_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
    EET_REQUIRE(K > 0 && N > 0 && K % 64 == 0 && N % 64 == 0, EET_ERR_UNSUPPORTED_SHAPE,
                "%s: the reference layout needs K %% 64 == 0 and N %% 64 == 0, got K=%zu N=%zu", fn, K, N);
    return EET_OK;
}

int eet_preprocess_ref_sm80(const int8_t *q, size_t K, size_t N, int8_t *processed)
{
    if (int rc = check_ref_shape("eet_preprocess_ref_sm80", q, processed, K, N))
        return rc;
    parallel_for(K * N, 1 << 16, [=](size_t lo, size_t hi) {
        for (size_t p = lo; p < hi; ++p)
            processed[p] = static_cast<int8_t>(static_cast<uint8_t>(q[ref_sm80_source(p, K, N)]) + 128u);
    });
    return EET_OK;
}

int eet_unprocess_ref_sm80(const int8_t *processed, size_t K, size_t N, int8_t *q)
{
    if (int rc = check_ref_shape("eet_unprocess_ref_sm80", q, processed, K, N))
        return rc;
    parallel_for(K * N, 1 << 16, [=](size_t lo, size_t hi) {
        for (size_t p = lo; p < hi; ++p)
            q[ref_sm80_source(p, K, N)] = static_cast<int8_t>(static_cast<uint8_t>(processed[p]) - 128u);
    });
    return EET_OK;
}

}  // extern "C"
