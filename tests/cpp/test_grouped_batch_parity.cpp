// Gate: run_moe_grouped_expert_batch (permutation -> grouped gate/up and W2 per range of 8
// experts -> per-token fixed-order reduce) against the per-token GEMV trio on identical experts
// and routing. Fixture of the reference's tests/test_moe_grouped_batch_parity.cpp: 8 tokens,
// 6 slots, 32 local experts of which {0,1,8,9,16,17} receive draws (three launch ranges with
// empty experts between), each token's row in its own 16-row tile (pitch 16*H), payload bytes
// (i*37 + seed*11) & 0xFF with power-of-two scales, SplitMix seed 0xC0FFEE.
#include "architecture/deepseek_v4/kernels/moe_gemv_dispatch.hpp"
#include "architecture/deepseek_v4/moe/moe_grouped_batch.hpp"
#include "backend/swizzled_w4a16/core/swizzled_expert_format.hpp"
#include "common.hpp"
#include "platform/ops/moe_accumulate.hpp"
#include "test_device.hpp"

#include <cstring>

namespace kernel = aeon::kernel;
namespace core = aeon::core;

constexpr int kHidden = 4096, kIntermediate = 2048, kSlots = 6, kExperts = 32, kTokens = 8, kMPad = 16;
constexpr float kLimit = 10.0f;
constexpr int kDrawn[6] = {0, 1, 8, 9, 16, 17};

static std::vector<uint8_t> make_payload(int seed) {
    std::vector<uint8_t> p(core::AEON_SWIZZLED_EXPERT_BYTES);
    for (size_t i = 0; i < p.size(); ++i) p[i] = static_cast<uint8_t>((i * 37 + static_cast<size_t>(seed) * 11) & 0xFF);
    const size_t off[3] = {core::AEON_W1_SCALE_OFFSET, core::AEON_W2_SCALE_OFFSET, core::AEON_W3_SCALE_OFFSET};
    const size_t len[3] = {core::AEON_W1_SCALE_BYTES, core::AEON_W2_SCALE_BYTES, core::AEON_W3_SCALE_BYTES};
    for (int r = 0; r < 3; ++r) {
        for (size_t i = 0; i < len[r] / 2; ++i) {
            const uint16_t bits = static_cast<uint16_t>((-6 + static_cast<int>(i % 4) + 15) << 10);
            std::memcpy(p.data() + off[r] + 2 * i, &bits, 2);
        }
    }
    return p;
}

static void point_tables(const uint8_t* base, int j, kernel::SwizzledW13ExpertPtrs& w13,
                         kernel::SwizzledW2ExpertPtrs& w2) {
    w13.w1[j] = reinterpret_cast<const uint4*>(base + core::AEON_W1_PACKED_OFFSET);
    w13.s1[j] = reinterpret_cast<const half*>(base + core::AEON_W1_SCALE_OFFSET);
    w13.w3[j] = reinterpret_cast<const uint4*>(base + core::AEON_W3_PACKED_OFFSET);
    w13.s3[j] = reinterpret_cast<const half*>(base + core::AEON_W3_SCALE_OFFSET);
    w2.w2[j] = reinterpret_cast<const uint4*>(base + core::AEON_W2_PACKED_OFFSET);
    w2.s2[j] = reinterpret_cast<const half*>(base + core::AEON_W2_SCALE_OFFSET);
}

int main() {
    aeon::test::select_test_device(true);
    SplitMix rng{0xC0FFEEull};
    std::vector<int> ids(kTokens * kSlots);
    std::vector<float> weights(kTokens * kSlots);
    for (int t = 0; t < kTokens; ++t)
        for (int k = 0; k < kSlots; ++k) {
            ids[t * kSlots + k] = kDrawn[(k + t) % kSlots];
            weights[t * kSlots + k] = 0.6f / static_cast<float>(k + 1) + 0.02f;
        }
    std::vector<uint8_t*> d_payload(kExperts, nullptr);
    for (int e : kDrawn) d_payload[e] = to_device(make_payload(e));

    const int stride = kMPad * kHidden;
    std::vector<half> x(static_cast<size_t>(kTokens) * stride, __float2half(0.0f));
    for (int t = 0; t < kTokens; ++t)
        for (int k = 0; k < kHidden; ++k)
            x[static_cast<size_t>(t) * stride + k] = __float2half(static_cast<float>(rng.uniform() - 0.5));
    half* d_x = to_device(x);
    int* d_ids = to_device(ids);
    float* d_w = to_device(weights);

    constexpr int kHiddenTokens = 16;
    core::MoeGroupedBatchScratch scratch{};
    scratch.intermediate = kIntermediate;
    scratch.hidden = kHidden;
    scratch.hidden_tokens = kHiddenTokens;
    GATE_HIP(hipMalloc(&scratch.perm_offsets, (kExperts + 1) * sizeof(int)));
    GATE_HIP(hipMalloc(&scratch.perm_tokens, ids.size() * sizeof(int)));
    GATE_HIP(hipMalloc(&scratch.perm_draws, ids.size() * sizeof(int)));
    GATE_HIP(hipMalloc(&scratch.perm_weights, ids.size() * sizeof(float)));
    GATE_HIP(hipMalloc(&scratch.batch_offsets, (kernel::kAeonSwizzledMaxExperts + 1) * sizeof(int)));
    GATE_HIP(hipMalloc(&scratch.chunk_hidden, sizeof(half) * kernel::kAeonSwizzledMaxExperts * kHiddenTokens * kIntermediate));
    GATE_HIP(hipMalloc(&scratch.chunk_contrib, sizeof(float) * kTokens * kSlots * kHidden));
    half *d_grouped, *d_gemv;
    GATE_HIP(hipMalloc(&d_grouped, sizeof(half) * kTokens * stride));
    GATE_HIP(hipMalloc(&d_gemv, sizeof(half) * kTokens * stride));
    GATE_HIP(hipMemset(d_grouped, 0, sizeof(half) * kTokens * stride));
    GATE_HIP(hipMemset(d_gemv, 0, sizeof(half) * kTokens * stride));

    auto filler = [&](int expert, int j, int count, kernel::SwizzledW13ExpertPtrs& w13,
                      kernel::SwizzledW2ExpertPtrs& w2) {
        if (count == 0) return;
        point_tables(d_payload[expert], j, w13, w2);
    };
    core::run_moe_grouped_expert_batch(d_x, stride, d_ids, d_w, kTokens, kSlots, kExperts, kLimit,
                                       scratch, filler, d_grouped, stride);
    GATE_HIP(hipGetLastError());
    GATE_HIP(hipDeviceSynchronize());

    half* d_hidden;
    float* d_contrib;
    GATE_HIP(hipMalloc(&d_hidden, sizeof(half) * kernel::kAeonSwizzledMaxExperts * kIntermediate));
    GATE_HIP(hipMalloc(&d_contrib, sizeof(float) * kSlots * kHidden));
    for (int t = 0; t < kTokens; ++t) {
        kernel::SwizzledW13ExpertPtrs w13{};
        kernel::SwizzledW2ExpertPtrs w2{};
        for (int k = 0; k < kSlots; ++k) point_tables(d_payload[ids[t * kSlots + k]], k, w13, w2);
        kernel::dispatch_dsv4_moe_gemv_w13_swiglu<8, 4, 8, 16>(d_x + static_cast<size_t>(t) * stride, w13,
                                                               d_hidden, nullptr, kIntermediate, kSlots,
                                                               kIntermediate, kHidden, kLimit);
        kernel::dispatch_aeon_moe_fused_w2_contrib<8, 8, 4, 16>(d_hidden, w2, d_w + t * kSlots, d_contrib,
                                                                kSlots, kHidden, kIntermediate);
        kernel::moe_accumulate_fixed_order_kernel<<<(kHidden + 255) / 256, 256>>>(
            d_contrib, kSlots, nullptr, d_gemv + static_cast<size_t>(t) * stride, kHidden);
    }
    GATE_HIP(hipGetLastError());
    GATE_HIP(hipDeviceSynchronize());

    const std::vector<half> grouped = to_host(d_grouped, static_cast<size_t>(kTokens) * stride);
    const std::vector<half> gemv = to_host(d_gemv, static_cast<size_t>(kTokens) * stride);
    double max_abs = 0, max_rel = 0, peak_a = 0, peak_b = 0;
    for (int t = 0; t < kTokens; ++t)
        for (int i = 0; i < kHidden; ++i) {
            const double a = __half2float(gemv[static_cast<size_t>(t) * stride + i]);
            const double b = __half2float(grouped[static_cast<size_t>(t) * stride + i]);
            max_abs = std::fmax(max_abs, std::fabs(a - b));
            max_rel = std::fmax(max_rel, std::fabs(a - b) / std::fmax(1e-3, std::fabs(a)));
            peak_a = std::fmax(peak_a, std::fabs(a));
            peak_b = std::fmax(peak_b, std::fabs(b));
        }
    std::printf("  grouped vs per-token: max_abs=%.3e max_rel=%.3e peaks %.3e / %.3e\n", max_abs, max_rel,
                peak_a, peak_b);
    expect(peak_a > 1e-3 && peak_b > 1e-3, "signal present in both arms");
    expect(max_rel <= 1e-3, "grouped batch within a reorder band of the per-token path (1e-3)");

    // a chunk whose widest expert exceeds the scratch rows is refused, not truncated
    core::MoeGroupedBatchScratch narrow = scratch;
    narrow.hidden_tokens = 2;
    bool threw = false;
    try {
        core::run_moe_grouped_expert_batch(d_x, stride, d_ids, d_w, kTokens, kSlots, kExperts, kLimit,
                                           narrow, filler, d_grouped, stride);
    } catch (const std::invalid_argument&) {
        threw = true;
    }
    expect(threw, "widest expert > hidden_tokens throws std::invalid_argument");
    std::printf(g_failures == 0 ? "[PASS] grouped batch parity\n" : "[FAIL] grouped batch parity\n");
    return g_failures == 0 ? 0 : 1;
}
