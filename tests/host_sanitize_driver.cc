// Driver for tests/test_host_sanitizers.py: the host packer (eet_amd/csrc/packer.cc) linked with
// AddressSanitizer + UndefinedBehaviorSanitizer, over shapes with ragged tile counts, an all-zero column,
// both dtypes and both quantiser modes, plus the round trips of both layouts.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <cstdint>
#include "eet_hip.h"
int main() {
    unsigned seed = 1;
    auto rnd = [&]() { seed = seed * 1664525u + 1013904223u; return (seed >> 8) & 0xffff; };
    for (size_t K : {64, 128, 192, 1024}) for (size_t N : {16, 48, 64, 144, 1040}) {
        std::vector<float> w(K * N);
        for (auto &x : w) x = ((int)rnd() - 32768) / 65536.0f;
        for (size_t k = 0; k < K; ++k) w[k * N + 1] = 0.f;
        std::vector<_Float16> wh(K * N);
        for (size_t i = 0; i < K * N; ++i) wh[i] = (_Float16)w[i];
        std::vector<int8_t> q(K * N), p(K * N), u(K * N), q2(K * N);
        std::vector<float> s(N);
        std::vector<_Float16> sh(N);
        for (int mode = 0; mode < 2; ++mode) {
            if (eet_quantize_int8(w.data(), EET_DTYPE_F32, K, N, mode, q.data(), s.data())) return 1;
            if (eet_quantize_int8(wh.data(), EET_DTYPE_F16, K, N, mode, q2.data(), sh.data())) return 2;
        }
        if (eet_pack_gfx950(q.data(), K, N, p.data())) return 3;
        if (eet_unpack_gfx950(p.data(), K, N, u.data())) return 4;
        if (memcmp(q.data(), u.data(), K * N)) return 5;
        if (N % 64 == 0) {
            if (eet_preprocess_ref_sm80(q.data(), K, N, p.data())) return 6;
            if (eet_unprocess_ref_sm80(p.data(), K, N, u.data())) return 7;
            if (memcmp(q.data(), u.data(), K * N)) return 8;
        }
    }
    puts("host sanitizer run ok");
    return 0;
}
