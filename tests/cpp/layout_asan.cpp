// Host-only hardening check of the layout functions: exact-size heap buffers (so any access one
// element past an end trips the address sanitizer) through swizzle / unswizzle and the wave64
// repack / unrepack at several shapes and both storage geometries; also checks the round trips.
// Built by tests/test_layout.py around the layout source file with the host sanitizers.
#include "aeon_mi355.h"
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <random>

static int fail(const char* what, int N, int K) {
    std::printf("FAIL %s N=%d K=%d: %s\n", what, N, K, aeon_last_error());
    return 1;
}

int main() {
    std::mt19937 rng(7);
    const int shapes[][4] = {{16, 128, 8, 4}, {32, 256, 4, 8}, {64, 384, 8, 4}, {48, 512, 4, 8},
                             {16, 1024, 8, 4}, {128, 256, 4, 8}};
    for (const auto& sh : shapes) {
        const int N = sh[0], K = sh[1], rpw = sh[2], lpr = sh[3];
        const size_t words = size_t(N) * K / 8, scales = size_t(N) * K / 32;
        std::unique_ptr<uint32_t[]> src(new uint32_t[words]), swz(new uint32_t[words]), back(new uint32_t[words]);
        std::unique_ptr<uint16_t[]> ssrc(new uint16_t[scales]), sswz(new uint16_t[scales]), sback(new uint16_t[scales]);
        for (size_t i = 0; i < words; ++i) src[i] = rng();
        // one scale per (row, 128 columns), repeated over its four 32-column groups
        for (int r = 0; r < N; ++r)
            for (int g = 0; g < K / 32; ++g) ssrc[size_t(r) * (K / 32) + g] = uint16_t(0x2000 + ((r * 31 + g / 4) % 977));
        if (aeon_swizzle_w4a16(src.get(), ssrc.get(), swz.get(), sswz.get(), N, K, rpw, lpr)) return fail("swizzle", N, K);
        if (aeon_unswizzle_w4a16(swz.get(), sswz.get(), back.get(), sback.get(), N, K, rpw, lpr)) return fail("unswizzle", N, K);
        if (std::memcmp(src.get(), back.get(), words * 4) || std::memcmp(ssrc.get(), sback.get(), scales * 2)) return fail("round trip", N, K);
        // both scale groupings of the wave64 packing on exact-size buffers (the replicated
        // scales above are a valid input for either)
        for (const int scale_group : {128, 32}) {
            const size_t pb = aeon_a64_packed_bytes(N, K), sb = aeon_a64_scale_bytes(N, K, scale_group);
            std::unique_ptr<uint8_t[]> a64p(new uint8_t[pb]), a64s(new uint8_t[sb]);
            if (aeon_a64_repack_host(swz.get(), sswz.get(), N, K, rpw, lpr, scale_group,
                                     reinterpret_cast<uint32_t*>(a64p.get()),
                                     reinterpret_cast<uint16_t*>(a64s.get()))) return fail("repack", N, K);
            std::unique_ptr<uint32_t[]> swz2(new uint32_t[words]);
            std::unique_ptr<uint16_t[]> sswz2(new uint16_t[scales]);
            if (aeon_a64_unrepack_host(reinterpret_cast<const uint32_t*>(a64p.get()),
                                       reinterpret_cast<const uint16_t*>(a64s.get()), N, K, rpw, lpr,
                                       scale_group, swz2.get(), sswz2.get())) return fail("unrepack", N, K);
            if (std::memcmp(swz.get(), swz2.get(), words * 4) || std::memcmp(sswz.get(), sswz2.get(), scales * 2)) {
                return fail("repack round trip", N, K);
            }
        }
    }
    std::printf("ok\n");
    return 0;
}
