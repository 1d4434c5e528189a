// Measurement aids for reading the routed-expert kernels' figures against what this GPU sustains:
// none of them has a counterpart in the reference and none is part of the product library. Built
// into a library of their own (libaeon_calibrate.so, declared in aeon_calibrate.h), used only by
// the benchmark's --calibrate-* legs.
//
// First: the rate at which this GPU sustains v_mfma_f32_16x16x32_f16 out of registers,
// with nothing else running. The sustained clock under dense MFMA work depends on the operand
// data (constant operands toggle few wires; random ones draw more power and clock lower), so the
// rate with random operands is the practical ceiling the grouped GEMM is read against, beside
// the published peak.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "aeon_calibrate.h"

namespace {

thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, args);
    va_end(args);
}

}  // namespace

extern "C" const char* aeon_calibrate_last_error(void) { return g_error; }

#define AEON_REQUIRE(cond, code, ...) \
    do {                              \
        if (!(cond)) {                \
            set_error(__VA_ARGS__);   \
            return (code);            \
        }                             \
    } while (0)

#define AEON_LAUNCH_CHECK()                                                        \
    do {                                                                           \
        hipError_t launch_error_ = hipGetLastError();                              \
        if (launch_error_ != hipSuccess) {                                         \
            set_error("launch failed: %s", hipGetErrorString(launch_error_));      \
            return AEON_CALIBRATE_ERR_HIP;                                         \
        }                                                                          \
    } while (0)

typedef _Float16 half_t;
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

static inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

namespace {

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

// Third aid: the MFMA loop with the grouped GEMM's companions issued between the matrix
// instructions: VALU int4-unpack-style VALU instructions (v_and_or_b32, v_pk_add_f16, independent
// of the MFMAs) per 16-cycle matrix slot and LDS 16-byte LDS reads per 16 slots, at WAVES waves
// per SIMD, with the 16x16x32 shape (one MFMA a slot) or the 32x32x16 shape (one MFMA every two
// slots: the same FLOPs). MFMA and VALU leave a SIMD through one issue port, so the rate
// measured here is what an instruction mix can reach before any memory wait. A round is 32
// slots over 128 accumulator registers; the LDS reads of a round are waited for at its end,
// before their registers are folded (LDS reads issued from inline asm are not counted by the
// compiler).
template <int SHAPE, int VALU, int LDS, int WAVES>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES)))
void calibrate_mix_kernel(float* sink, int iterations) {
    __shared__ u32x4_t lds[256 * 4];
    half8_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t r = calibrate_hash(threadIdx.x * 64 + i * 8 + j + blockIdx.x * 7919);
            a[i][j] = static_cast<half_t>((static_cast<int>(r & 0xffff) - 32768) / 4096.0f);
            b[i][j] = static_cast<half_t>((static_cast<int>(r >> 16) - 32768) / 16384.0f);
        }
    for (int i = 0; i < 4; ++i) lds[threadIdx.x * 4 + i] = u32x4_t{calibrate_hash(threadIdx.x + i), 1u, 2u, 3u};
    __syncthreads();
    float4_t acc4[32];
    float16_t acc16[8];
#pragma unroll
    for (int i = 0; i < 32; ++i) acc4[i] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc16[i][j] = 0.0f;
    uint32_t x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = calibrate_hash(threadIdx.x * 8 + i);
    const uint32_t mask = 0x000f000f, magic = 0x64006400, minus = 0xe408e408;
    constexpr int kReadEvery = LDS > 0 ? 16 / LDS : 1;
    u32x4_t fold = {0u, 0u, 0u, 0u};
    u32x4_t landed[2 * (LDS > 0 ? LDS : 1)];
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int m = 0; m < 32; ++m) {
            // volatile: the order written here is the order issued
            if (SHAPE == 16) {
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                             : "+v"(acc4[m]) : "v"(a[m % 4]), "v"(b[(m / 4) % 4]));
            } else if ((m & 1) == 0) {
                asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0"
                             : "+v"(acc16[(m / 2) % 8]) : "v"(a[(m / 2) % 4]), "v"(b[(m / 8) % 4]));
            }
#pragma unroll
            for (int k = 0; k < VALU; ++k) {
                if (k & 1) asm volatile("v_pk_add_f16 %0, %0, %1" : "+v"(x[(m * VALU + k) % 8]) : "v"(minus));
                else asm volatile("v_and_or_b32 %0, %0, %1, %2" : "+v"(x[(m * VALU + k) % 8]) : "v"(mask), "v"(magic));
            }
            if (LDS > 0 && m % kReadEvery == 0) {
                asm volatile("ds_read_b128 %0, %1"
                             : "=v"(landed[m / kReadEvery])
                             : "v"(static_cast<uint32_t>(threadIdx.x * 16 + (m & 3) * 4096)));
            }
        }
        if (LDS > 0) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int i = 0; i < 2 * LDS; ++i) fold ^= landed[i];
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) s += acc4[i][0] + acc4[i][1] + acc4[i][2] + acc4[i][3];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) s += acc16[i][j];
    uint32_t bits = fold[0];
#pragma unroll
    for (int i = 0; i < 8; ++i) bits ^= x[i];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s + static_cast<float>(bits & 1u);
}

// Second aid: what a read-only stream sustains from HBM. Workgroup w reads its own contiguous
// share of the buffer, 16 bytes a lane and eight loads in flight per lane (each wave instruction
// one contiguous KiB, as a weight tile is), folds everything into one word per lane so the loads
// cannot be dropped, and writes nothing else.
__global__ __launch_bounds__(256) void calibrate_read_kernel(const u32x4_t* __restrict__ buf,
                                                             size_t units_per_workgroup,
                                                             uint32_t* sink) {
    const u32x4_t* mine = buf + blockIdx.x * units_per_workgroup + threadIdx.x;
    u32x4_t fold = {0u, 0u, 0u, 0u};
    for (size_t i = 0; i < units_per_workgroup; i += 8 * 256) {
        u32x4_t v[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) v[q] = __builtin_nontemporal_load(mine + i + q * 256);
#pragma unroll
        for (int q = 0; q < 8; ++q) fold ^= v[q];
    }
    sink[blockIdx.x * 256 + threadIdx.x] = fold[0] ^ fold[1] ^ fold[2] ^ fold[3];
}

// Fourth aid: what a 16-byte LDS read per lane costs when the lanes address a 1 KiB fragment in
// an order other than their own. PATTERN 0: unit = lane (linear); 1: unit = 4 n + chunk, the
// matrix instruction's lanes (n = lane % 16, chunk = lane / 16) reading a fragment stored
// position-major; 2: unit = 4 n + (chunk + n / 2) % 4, the same with each position's four pieces
// rotated by n / 2 (what the grouped kernel reads); 3: rotated by n / 4.
template <int PATTERN>
__global__ __launch_bounds__(256) void calibrate_lds_kernel(uint32_t* sink, int iterations) {
    __shared__ u32x4_t lds[8 * 64];
    for (int i = threadIdx.x; i < 8 * 64; i += 256) lds[i] = u32x4_t{static_cast<uint32_t>(i), 1u, 2u, 3u};
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int n = lane & 15, chunk = lane >> 4;
    const int unit = PATTERN == 0   ? lane
                     : PATTERN == 1 ? 4 * n + chunk
                     : PATTERN == 2 ? 4 * n + ((chunk + (n >> 1)) & 3)
                                    : 4 * n + ((chunk + (n >> 2)) & 3);
    u32x4_t fold = {0u, 0u, 0u, 0u};
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int f = 0; f < 8; ++f) {
            u32x4_t t;
            // volatile: every read is issued, and waited for before the next
            asm volatile("ds_read_b128 %0, %1 offset:%2\n\ts_waitcnt lgkmcnt(0)"
                         : "=v"(t)
                         : "v"(static_cast<uint32_t>(unit * 16)), "n"(f * 1024)
                         : "memory");
            fold ^= t;
        }
    }
    sink[blockIdx.x * 256 + threadIdx.x] = fold[0] ^ fold[1] ^ fold[2] ^ fold[3];
}

}  // namespace

extern "C" int aeon_calibrate_lds_read(int pattern, int iterations, int workgroups, uint32_t* d_sink,
                                       size_t sink_words, double* wave_reads, void* stream) {
    const char* who = "aeon_calibrate_lds_read";
    AEON_REQUIRE(d_sink != nullptr && iterations > 0 && workgroups > 0 && pattern >= 0 && pattern <= 3,
                 AEON_CALIBRATE_ERR_INVALID_ARGUMENT, "%s: bad arguments (pattern=%d iterations=%d workgroups=%d)",
                 who, pattern, iterations, workgroups);
    AEON_REQUIRE(sink_words >= static_cast<size_t>(workgroups) * 256, AEON_CALIBRATE_ERR_INVALID_ARGUMENT,
                 "%s: the sink holds %zu words, %zu needed", who, sink_words,
                 static_cast<size_t>(workgroups) * 256);
    hipStream_t s = as_stream(stream);
    switch (pattern) {
        case 0: calibrate_lds_kernel<0><<<workgroups, 256, 0, s>>>(d_sink, iterations); break;
        case 1: calibrate_lds_kernel<1><<<workgroups, 256, 0, s>>>(d_sink, iterations); break;
        case 2: calibrate_lds_kernel<2><<<workgroups, 256, 0, s>>>(d_sink, iterations); break;
        default: calibrate_lds_kernel<3><<<workgroups, 256, 0, s>>>(d_sink, iterations); break;
    }
    AEON_LAUNCH_CHECK();
    // four waves a workgroup, eight reads a round
    if (wave_reads != nullptr) *wave_reads = static_cast<double>(workgroups) * 4.0 * iterations * 8.0;
    return AEON_CALIBRATE_OK;
}

extern "C" int aeon_calibrate_read_stream(const void* d_buffer, size_t bytes, int workgroups,
                                          uint32_t* d_sink, size_t sink_words, void* stream) {
    const char* who = "aeon_calibrate_read_stream";
    AEON_REQUIRE(d_buffer != nullptr && d_sink != nullptr && workgroups > 0, AEON_CALIBRATE_ERR_INVALID_ARGUMENT,
                 "%s: bad arguments (workgroups=%d)", who, workgroups);
    const size_t per_workgroup = bytes / static_cast<size_t>(workgroups);
    AEON_REQUIRE(per_workgroup > 0 && per_workgroup % (8 * 256 * 16) == 0 &&
                     per_workgroup * workgroups == bytes,
                 AEON_CALIBRATE_ERR_INVALID_ARGUMENT, "%s: %zu bytes over %d workgroups is not a whole number "
                 "of 32 KiB rounds each", who, bytes, workgroups);
    AEON_REQUIRE(sink_words >= static_cast<size_t>(workgroups) * 256, AEON_CALIBRATE_ERR_INVALID_ARGUMENT,
                 "%s: the sink holds %zu words, %zu needed", who, sink_words,
                 static_cast<size_t>(workgroups) * 256);
    calibrate_read_kernel<<<workgroups, 256, 0, as_stream(stream)>>>(
        static_cast<const u32x4_t*>(d_buffer), per_workgroup / 16, d_sink);
    AEON_LAUNCH_CHECK();
    return AEON_CALIBRATE_OK;
}

extern "C" int aeon_calibrate_mfma_f16(int random_operands, int iterations, int workgroups,
                                       float* d_sink, size_t sink_floats, double* flop,
                                       void* stream) {
    const char* who = "aeon_calibrate_mfma_f16";
    AEON_REQUIRE(d_sink != nullptr && iterations > 0 && workgroups > 0, AEON_CALIBRATE_ERR_INVALID_ARGUMENT,
                 "%s: bad arguments (iterations=%d workgroups=%d)", who, iterations, workgroups);
    AEON_REQUIRE(sink_floats >= static_cast<size_t>(workgroups) * 256, AEON_CALIBRATE_ERR_INVALID_ARGUMENT,
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
    return AEON_CALIBRATE_OK;
}

extern "C" int aeon_calibrate_mfma_mix(int mfma_shape, int valu_per_slot, int lds_reads_per_16,
                                       int waves_per_simd, int iterations, int workgroups,
                                       float* d_sink, size_t sink_floats, double* flop, void* stream) {
    const char* who = "aeon_calibrate_mfma_mix";
    AEON_REQUIRE(d_sink != nullptr && iterations > 0 && workgroups > 0, AEON_CALIBRATE_ERR_INVALID_ARGUMENT,
                 "%s: bad arguments (iterations=%d workgroups=%d)", who, iterations, workgroups);
    AEON_REQUIRE(sink_floats >= static_cast<size_t>(workgroups) * 256, AEON_CALIBRATE_ERR_INVALID_ARGUMENT,
                 "%s: the sink holds %zu floats, %zu needed", who, sink_floats,
                 static_cast<size_t>(workgroups) * 256);
    hipStream_t s = as_stream(stream);
    const int key = ((mfma_shape * 10 + waves_per_simd) * 10 + valu_per_slot) * 10 + lds_reads_per_16;
#define AEON_MIX_CASE(shape_, waves_, v_, l_)                                                          \
    case (((shape_) * 10 + (waves_)) * 10 + (v_)) * 10 + (l_):                                         \
        calibrate_mix_kernel<shape_, v_, l_, waves_><<<workgroups, 256, 0, s>>>(d_sink, iterations);   \
        break;
#define AEON_MIX_SHAPES(waves_, v_, l_) AEON_MIX_CASE(16, waves_, v_, l_) AEON_MIX_CASE(32, waves_, v_, l_)
    switch (key) {
        AEON_MIX_SHAPES(2, 0, 0) AEON_MIX_SHAPES(2, 1, 0) AEON_MIX_SHAPES(2, 2, 0) AEON_MIX_SHAPES(2, 3, 0)
        AEON_MIX_SHAPES(2, 4, 0) AEON_MIX_SHAPES(2, 1, 4) AEON_MIX_SHAPES(2, 2, 4) AEON_MIX_SHAPES(2, 3, 4)
        AEON_MIX_SHAPES(2, 1, 8) AEON_MIX_SHAPES(2, 3, 8)
        AEON_MIX_SHAPES(1, 0, 0) AEON_MIX_SHAPES(1, 1, 4) AEON_MIX_SHAPES(1, 2, 4) AEON_MIX_SHAPES(1, 2, 2)
        default:
            AEON_REQUIRE(false, AEON_CALIBRATE_ERR_INVALID_ARGUMENT, "%s: no kernel for shape %d, %d waves per "
                         "SIMD, %d VALU per slot and %d LDS reads per 16", who, mfma_shape, waves_per_simd,
                         valu_per_slot, lds_reads_per_16);
    }
#undef AEON_MIX_SHAPES
#undef AEON_MIX_CASE
    AEON_LAUNCH_CHECK();
    // four waves a workgroup, 32 slots a round, 2*16*16*32 FLOP a slot
    if (flop != nullptr) *flop = static_cast<double>(workgroups) * 4.0 * iterations * 32.0 * 16384.0;
    return AEON_CALIBRATE_OK;
}
