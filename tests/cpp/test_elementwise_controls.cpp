// Gate: the element-wise kernels the reference's callers launch by name with <<<>>> --
// v4_swiglu_clamp_kernel (kernels/v4_swiglu_clamp.hpp:18-34, launched by the shared-expert pass,
// layer/v4_layer_body_moe.hpp:242) and the superseded fp16-chain control
// moe_accumulate_expert_kernel (platform/ops/moe_accumulate.hpp:32-44) -- plus the library's
// own aeon_swiglu_clamp, against their definitions evaluated on the host:
//   clamp:  out = fp16( silu(min(g, L)) * clamp(u, -L, +L) ), fp32 arithmetic, the gate bounded
//           from above only (probes of tests/test_v4_expert_oracle.cpp:302-406, gate < -L included);
//   chain:  accum = fp16( float(accum) + w * float(expert) ), one fp16 rounding per expert, so k
//           experts leave k roundings behind (the fixed-order reduce leaves one).
#include "architecture/deepseek_v4/kernels/v4_swiglu_clamp.hpp"
#include "platform/ops/moe_accumulate.hpp"
#include "aeon355/status.hpp"
#include "common.hpp"

#include <cstring>
#include "test_device.hpp"

namespace {

// the definition in double, rounded once to fp16; silu evaluated with the double exp
float clamp_definition(float gate, float up, float limit) {
    const double g = std::fmin(static_cast<double>(gate), static_cast<double>(limit));
    const double u = std::fmax(-static_cast<double>(limit), std::fmin(static_cast<double>(up), limit));
    return static_cast<float>(g / (1.0 + std::exp(-g)) * u);
}

uint16_t bits(half h) {
    uint16_t u;
    std::memcpy(&u, &h, 2);
    return u;
}

}  // namespace

int main() {
    aeon::test::select_test_device(true);
    const float limit = 7.0f;

    // ---- clamp: every pair of probes, then a seeded sweep ---------------------------------
    const float probes[] = {-40.0f, -12.0f, -5.0f, 0.0f, 5.0f, 12.0f, 40.0f, 3.0f};
    std::vector<half> gate, up;
    for (float g : probes)
        for (float u : probes) {
            gate.push_back(__float2half(g));
            up.push_back(__float2half(u));
        }
    SplitMix rng{0x5EEDC1A9ull};
    for (int i = 0; i < 4096 + 37; ++i) {   // not a multiple of the block size
        gate.push_back(__float2half(static_cast<float>(rng.uniform() * 30.0 - 15.0)));
        up.push_back(__float2half(static_cast<float>(rng.uniform() * 30.0 - 15.0)));
    }
    const int total = static_cast<int>(gate.size());
    half* d_gate = to_device(gate);
    half* d_up = to_device(up);
    half *d_kernel, *d_library;
    GATE_HIP(hipMalloc(&d_kernel, total * sizeof(half) + 64));
    GATE_HIP(hipMalloc(&d_library, total * sizeof(half) + 64));
    GATE_HIP(hipMemset(d_kernel, 0x7B, total * sizeof(half) + 64));
    GATE_HIP(hipMemset(d_library, 0x7B, total * sizeof(half) + 64));
    aeon::kernel::v4_swiglu_clamp_kernel<<<(total + 255) / 256, 256>>>(d_gate, d_up, d_kernel, total, limit);
    GATE_HIP(hipGetLastError());
    aeon355::throw_on_error(aeon_swiglu_clamp(d_gate, d_up, d_library, total, limit, nullptr));
    GATE_HIP(hipDeviceSynchronize());
    const std::vector<half> by_kernel = to_host(d_kernel, total + 32);
    const std::vector<half> by_library = to_host(d_library, total + 32);

    bool same = true, close = true, guard = true, asymmetric = true;
    double worst = 0.0;
    for (int i = 0; i < total; ++i) {
        same = same && bits(by_kernel[i]) == bits(by_library[i]);
        const float g = __half2float(gate[i]), u = __half2float(up[i]);
        const float want = clamp_definition(g, u, limit);
        const float got = __half2float(by_library[i]);
        // one fp16 rounding of a value computed with the device's expf: within 2^-10 relative
        // of the definition (plus the smallest subnormal)
        const double tol = std::fabs(want) * 0.0010 + 6e-8;
        worst = std::fmax(worst, std::fabs(got - want) - tol);
        close = close && std::fabs(got - want) <= tol;
        if (g <= -limit - 3.0f) {
            // the gate is NOT clamped from below: silu(g) of the raw gate, far from silu(-L)
            const float symmetric = clamp_definition(-limit, u, limit);
            if (std::fabs(u) >= 3.0f && std::fabs(symmetric) > 1e-3f) {
                asymmetric = asymmetric && std::fabs(got - symmetric) > 0.5f * std::fabs(symmetric);
            }
        }
    }
    for (int i = total; i < total + 32; ++i) {
        guard = guard && bits(by_kernel[i]) == 0x7B7B && bits(by_library[i]) == 0x7B7B;
    }
    expect(same, "v4_swiglu_clamp_kernel == aeon_swiglu_clamp, bit for bit");
    expect(close, "clamped SwiGLU within one fp16 rounding of its definition");
    expect(asymmetric, "a gate below -limit is not clamped (differs from the symmetric rule)");
    expect(guard, "nothing is written past total_elements");
    if (!close) std::printf("    worst excess over tolerance %.3e\n", worst);

    // ---- fp16 chain ---------------------------------------------------------------------------
    const int hidden = 7168 + 8, experts = 8;
    std::vector<half> accum(hidden);
    std::vector<std::vector<half>> outs(experts, std::vector<half>(hidden));
    std::vector<float> weights(experts);
    for (int i = 0; i < hidden; ++i) accum[i] = __float2half(static_cast<float>(rng.uniform() * 2.0 - 1.0));
    for (int e = 0; e < experts; ++e) {
        weights[e] = static_cast<float>(0.05 + 0.3 * rng.uniform());
        for (int i = 0; i < hidden; ++i) outs[e][i] = __float2half(static_cast<float>(rng.uniform() * 8.0 - 4.0));
    }
    half* d_accum = to_device(accum);
    for (int e = 0; e < experts; ++e) {
        half* d_out = to_device(outs[e]);
        aeon::kernel::moe_accumulate_expert_kernel<<<(hidden + 255) / 256, 256>>>(d_accum, d_out, weights[e], hidden);
        GATE_HIP(hipGetLastError());
        GATE_HIP(hipDeviceSynchronize());
        GATE_HIP(hipFree(d_out));
    }
    const std::vector<half> chained = to_host(d_accum, hidden);
    // The definition leaves the roundings inside a step open: a compiler may keep the product and
    // the sum apart (two fp32 roundings, then fp16), fuse them (one fp32 rounding, then fp16), or
    // use the mixed-precision fused multiply-add that rounds the exact sum to fp16 directly
    // (v_fma_mixlo_f16). Each reading is followed as a chain of its own; the kernel is compiled
    // one way, so it follows one of them through all the experts.
    bool chain_ok = true;
    int differs_from_single_rounding = 0;
    for (int i = 0; i < hidden; ++i) {
        float plain = __half2float(accum[i]), fused = plain, direct = plain;
        double exact = plain;
        for (int e = 0; e < experts; ++e) {
            const float x = __half2float(outs[e][i]);
            plain = __half2float(__float2half(plain + weights[e] * x));
            fused = __half2float(__float2half(std::fmaf(weights[e], x, fused)));
            direct = static_cast<float>(static_cast<_Float16>(static_cast<double>(direct) +
                                                              static_cast<double>(weights[e]) * x));
            exact += static_cast<double>(weights[e]) * x;
        }
        const float got = __half2float(chained[i]);
        if (!(got == plain || got == fused || got == direct) && chain_ok) {
            std::printf("    element %d: device %.9g, chains %.9g / %.9g / %.9g, exact %.9g\n", i, got,
                        plain, fused, direct, exact);
        }
        chain_ok = chain_ok && (got == plain || got == fused || got == direct);
        if (got != __half2float(__float2half(static_cast<float>(exact)))) ++differs_from_single_rounding;
    }
    expect(chain_ok, "moe_accumulate_expert_kernel == the fp16 chain, one rounding per expert");
    // non-vacuous: the chain is measurably not the single-rounding sum
    expect(differs_from_single_rounding > hidden / 20,
           "the chain's k roundings show (it is not the fixed-order reduce)");

    std::printf(g_failures == 0 ? "[PASS] element-wise controls\n" : "[FAIL] element-wise controls\n");
    return g_failures == 0 ? 0 : 1;
}
