// Gate: the swizzled W4A16 GEMV and dual-GEMV entry points of the shim headers against a
// source-layout CPU loop -- the shapes and closed-form inputs of the reference's
// tests/test_w4a16_swizzled_gemv.cpp and test_w4a16_swizzled_dual_gemv.cpp (2048x4096 <8,4,8,16>,
// 4096x2048 <8,8,4,16>), plus the 7168-wide shapes of the benchmark configs.
#include "backend/swizzled_w4a16/kernels/aeon_w4a16_swizzle.hpp"
#include "backend/swizzled_w4a16/kernels/aeon_w4a16_swizzled_gemv.hpp"
#include "common.hpp"
#include "test_device.hpp"

namespace {

struct Fixture {
    std::vector<uint32_t> packed, swizzled;
    std::vector<half> scale, swizzled_scale, x;
    std::vector<float> want;
};

Fixture make_fixture(int N, int K, aeon::SwizzleCfg cfg, int seed) {
    Fixture f;
    const int groups = K / 32;
    f.packed.resize(static_cast<size_t>(N) * K / 8);
    f.scale.resize(static_cast<size_t>(N) * groups);
    f.x.resize(K);
    for (size_t i = 0; i < f.packed.size(); ++i) {
        uint32_t word = 0;
        for (int j = 0; j < 8; ++j) word |= static_cast<uint32_t>((i * 3 + j * 5 + seed) % 16) << (4 * j);
        f.packed[i] = word;
    }
    for (size_t i = 0; i < f.scale.size(); ++i) {
        f.scale[i] = __float2half(0.00390625f * static_cast<float>(1 + (i + seed) % 29));
    }
    for (int k = 0; k < K; ++k) f.x[k] = __float2half(static_cast<float>((k % 19) - 9) * 0.03125f);
    f.swizzled.resize(f.packed.size());
    f.swizzled_scale.resize(f.scale.size());
    aeon::swizzle_w4a16(f.packed.data(), f.scale.data(), f.swizzled.data(), f.swizzled_scale.data(),
                        N, K, cfg);
    f.want.assign(N, 0.0f);
    for (int row = 0; row < N; ++row) {
        float sum = 0.0f;
        for (int k = 0; k < K; ++k) {
            const uint32_t word = f.packed[static_cast<size_t>(row) * (K / 8) + k / 8];
            const int q = static_cast<int>((word >> (4 * (k % 8))) & 0xFu);
            sum += __half2float(f.x[k]) * static_cast<float>(q - 8) *
                   __half2float(f.scale[static_cast<size_t>(row) * groups + k / 32]);
        }
        f.want[row] = sum;
    }
    return f;
}

template <int RPW, int LPR, int ITERS>
void verify(const char* name, int N, int K, aeon::SwizzleCfg cfg) {
    const Fixture a = make_fixture(N, K, cfg, 1);
    const Fixture b = make_fixture(N, K, cfg, 7);
    half* d_x = to_device(a.x);
    uint32_t* d_pa = to_device(a.swizzled);
    half* d_sa = to_device(a.swizzled_scale);
    uint32_t* d_pb = to_device(b.swizzled);
    half* d_sb = to_device(b.swizzled_scale);
    half *d_oa, *d_ob, *d_da, *d_db;
    GATE_HIP(hipMalloc(&d_oa, N * sizeof(half)));
    GATE_HIP(hipMalloc(&d_ob, N * sizeof(half)));
    GATE_HIP(hipMalloc(&d_da, N * sizeof(half)));
    GATE_HIP(hipMalloc(&d_db, N * sizeof(half)));
    aeon::kernel::dispatch_aeon_w4a16_swizzled_gemv<8, RPW, LPR, ITERS>(d_x, d_pa, d_sa, d_oa, N, K);
    aeon::kernel::dispatch_aeon_w4a16_swizzled_gemv<8, RPW, LPR, ITERS>(d_x, d_pb, d_sb, d_ob, N, K);
    aeon::kernel::dispatch_aeon_w4a16_swizzled_dual_gemv<8, RPW, LPR, ITERS>(d_x, d_pa, d_sa, d_pb, d_sb,
                                                                             d_da, d_db, N, K);
    GATE_HIP(hipGetLastError());
    GATE_HIP(hipDeviceSynchronize());
    const std::vector<half> oa = to_host(d_oa, N), ob = to_host(d_ob, N);
    const std::vector<half> da = to_host(d_da, N), db = to_host(d_db, N);
    float max_a = 0.0f, max_b = 0.0f, peak = 0.0f;
    bool dual_equal = true;
    for (int i = 0; i < N; ++i) {
        max_a = std::fmax(max_a, std::fabs(__half2float(oa[i]) - a.want[i]));
        max_b = std::fmax(max_b, std::fabs(__half2float(ob[i]) - b.want[i]));
        peak = std::fmax(peak, std::fabs(a.want[i]));
        dual_equal = dual_equal && __half_as_ushort(oa[i]) == __half_as_ushort(da[i]) &&
                     __half_as_ushort(ob[i]) == __half_as_ushort(db[i]);
    }
    std::printf("%s: max error %.4g / %.4g (peak %.3g)\n", name, max_a, max_b, peak);
    expect(max_a < 0.05f && max_b < 0.05f && peak > 1.0f, "GEMV within 0.05 of the source-layout loop");
    expect(dual_equal, "dual-GEMV bit-equal to two single launches");
    GATE_HIP(hipFree(d_x)); GATE_HIP(hipFree(d_pa)); GATE_HIP(hipFree(d_sa)); GATE_HIP(hipFree(d_pb));
    GATE_HIP(hipFree(d_sb)); GATE_HIP(hipFree(d_oa)); GATE_HIP(hipFree(d_ob)); GATE_HIP(hipFree(d_da));
    GATE_HIP(hipFree(d_db));
}

}  // namespace

int main() {
    aeon::test::select_test_device(true);
    verify<4, 8, 16>("W1/W3 2048x4096", 2048, 4096, aeon::kCfgW13);
    verify<8, 4, 16>("W2 4096x2048", 4096, 2048, aeon::kCfgW2);
    verify<4, 8, 28>("W1/W3 2048x7168", 2048, 7168, aeon::kCfgW13);
    verify<8, 4, 16>("W2 7168x2048", 7168, 2048, aeon::kCfgW2);
    bool threw = false;
    try {
        aeon::kernel::dispatch_aeon_w4a16_swizzled_gemv<8, 4, 8, 16>(nullptr, nullptr, nullptr, nullptr,
                                                                     2048, 7168);
    } catch (const std::invalid_argument&) {
        threw = true;
    }
    expect(threw, "K != ITERS*LPR*32 throws std::invalid_argument");
    std::printf(g_failures == 0 ? "[PASS] swizzled GEMV shims\n" : "[FAIL] swizzled GEMV shims\n");
    return g_failures == 0 ? 0 : 1;
}
