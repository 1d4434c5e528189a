// Measurement aid: the rate at which this GPU sustains v_mfma_f32_16x16x32_f16 out of registers,
// with nothing else running. The sustained clock under dense MFMA work depends on the operand
// data (constant operands toggle few wires; random ones draw more power and clock lower), so the
// rate with random operands is the practical ceiling the grouped GEMM is read against, beside
// the published peak.
#include "common.hpp"

namespace aeon355 {

__device__ __forceinline__ uint32_t calibrate_hash(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

// Every wave runs `iterations` rounds of 16 independent MFMAs (16 accumulator tiles, 4 A and 4 B
// fragments held in registers).
template <bool RANDOM>
__global__ __launch_bounds__(256) void calibrate_mfma_kernel(float* sink, int iterations) {
    half8_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t r = calibrate_hash(threadIdx.x * 64 + i * 8 + j + blockIdx.x * 7919);
            a[i][j] = RANDOM ? static_cast<half_t>((static_cast<int>(r & 0xffff) - 32768) / 4096.0f)
                             : static_cast<half_t>(1.0f);
            b[i][j] = RANDOM ? static_cast<half_t>((static_cast<int>(r >> 16) - 32768) / 16384.0f)
                             : static_cast<half_t>(1.0f);
        }
    float4_t acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int m = 0; m < 16; ++m)
            acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m % 4], b[m / 4], acc[m], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_calibrate_mfma_f16(int random_operands, int iterations, int workgroups,
                                       float* d_sink, size_t sink_floats, double* flop,
                                       void* stream) {
    const char* who = "aeon_calibrate_mfma_f16";
    AEON_REQUIRE(d_sink != nullptr && iterations > 0 && workgroups > 0, AEON_ERR_INVALID_ARGUMENT,
                 "%s: bad arguments (iterations=%d workgroups=%d)", who, iterations, workgroups);
    AEON_REQUIRE(sink_floats >= static_cast<size_t>(workgroups) * 256, AEON_ERR_INVALID_ARGUMENT,
                 "%s: the sink holds %zu floats, %zu needed", who, sink_floats,
                 static_cast<size_t>(workgroups) * 256);
    if (random_operands) {
        calibrate_mfma_kernel<true><<<workgroups, 256, 0, as_stream(stream)>>>(d_sink, iterations);
    } else {
        calibrate_mfma_kernel<false><<<workgroups, 256, 0, as_stream(stream)>>>(d_sink, iterations);
    }
    AEON_LAUNCH_CHECK();
    // 4 waves a workgroup, 16 MFMAs a round, 2*16*16*32 FLOP an MFMA
    if (flop != nullptr) *flop = static_cast<double>(workgroups) * 4.0 * iterations * 16.0 * 16384.0;
    return AEON_OK;
}
