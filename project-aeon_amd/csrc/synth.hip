// Device generator of synthetic int4 experts, for filling tens of gigabytes of HBM without a
// host copy. It evaluates the same counter-based function as the host generator
// (project-aeon_amd/synth.py): draw i of a stream is the SplitMix64 finaliser of
// key + (i+1)*golden; source word w of a matrix is the low or high half of draw w/2; the scale
// of (row, 128-group) is draw row*(K/128)+g mapped to [0.005, 0.02] in fp64 and rounded to
// fp16 (round to nearest even, done with integer arithmetic so host and device agree bit for
// bit). The output is the `.aeon` swizzled payload, either with one scale per 128 columns
// replicated over its four group-32 slots or (scale_group 32) with a scale of its own per
// (row, 32-column group): draw row*(K/32)+group of the same stream.
#include "common.hpp"

namespace aeon355 {

__host__ __device__ static inline uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__host__ __device__ static inline uint64_t stream_key(uint64_t seed, int stream, int unit) {
    uint64_t k = mix64(seed ^ (static_cast<uint64_t>(stream + 1) * 0xD6E8FEB86659FD93ull));
    k = mix64(k ^ (static_cast<uint64_t>(unit + 1) * 0x9E3779B97F4A7C15ull));
    return k != 0 ? k : 0x9E3779B97F4A7C15ull;
}

__host__ __device__ static inline uint64_t stream_draw(uint64_t key, uint64_t index) {
    return mix64(key + (index + 1) * 0x9E3779B97F4A7C15ull);
}

// fp64 -> fp16 bits, round to nearest even, for positive normal results (scales).
__host__ __device__ static inline uint16_t positive_double_to_half_bits(double value) {
    union { double d; uint64_t u; } v;
    v.d = value;
    const int e = static_cast<int>((v.u >> 52) & 0x7FF) - 1023;
    const uint64_t sig = (v.u & 0xFFFFFFFFFFFFFull) | (1ull << 52);
    uint64_t kept = sig >> 42;
    const uint64_t rest = sig & ((1ull << 42) - 1ull);
    const uint64_t half = 1ull << 41;
    if (rest > half || (rest == half && (kept & 1ull))) kept += 1;
    return static_cast<uint16_t>((static_cast<uint32_t>(e + 15 - 1) << 10) + static_cast<uint32_t>(kept));
}

__device__ static inline uint32_t permute_nibbles(uint32_t source) {
    // destination nibble p takes source nibble {0,2,4,6,1,3,5,7}[p]
    uint32_t out = 0;
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const int from = p < 4 ? 2 * p : 2 * (p - 4) + 1;
        out |= ((source >> (4 * from)) & 0xFu) << (4 * p);
    }
    return out;
}

__global__ __launch_bounds__(256) void synth_matrix_kernel(uint64_t packed_key, uint64_t scale_key,
                                                           int N, int K, int rpw, int lpr,
                                                           int scale_group,
                                                           uint4* __restrict__ packed,
                                                           uint16_t* __restrict__ scale) {
    // one thread per swizzled slot = (row, 32-column group)
    const int groups = K / 32;
    const int iterations = groups / lpr;
    const size_t slot = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (slot >= static_cast<size_t>(N) * groups) return;
    const int lane = static_cast<int>(slot % 32);
    const size_t bi = slot / 32;
    const int iteration = static_cast<int>(bi % iterations);
    const int block = static_cast<int>(bi / iterations);
    const int row = block * rpw + lane / lpr;
    const int group = iteration * lpr + lane % lpr;
    const uint64_t word0 = static_cast<uint64_t>(row) * (K / 8) + static_cast<uint64_t>(group) * 4;
    const uint64_t d0 = stream_draw(packed_key, word0 / 2);
    const uint64_t d1 = stream_draw(packed_key, word0 / 2 + 1);
    packed[slot] = make_uint4(permute_nibbles(static_cast<uint32_t>(d0)),
                              permute_nibbles(static_cast<uint32_t>(d0 >> 32)),
                              permute_nibbles(static_cast<uint32_t>(d1)),
                              permute_nibbles(static_cast<uint32_t>(d1 >> 32)));
    const uint64_t sd = scale_group == 32
                            ? stream_draw(scale_key, static_cast<uint64_t>(row) * (K / 32) + group)
                            : stream_draw(scale_key, static_cast<uint64_t>(row) * (K / 128) + group / 4);
    const double u = static_cast<double>(sd >> 11) * (1.0 / 9007199254740992.0);
    scale[slot] = positive_double_to_half_bits(0.005 + 0.015 * u);
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_synth_matrix_swizzled(uint64_t seed, int expert, int matrix, int N, int K,
                                          int rpw, int lpr, int scale_group, void* d_packed,
                                          void* d_scale, void* stream) {
    const char* who = "aeon_synth_matrix_swizzled";
    AEON_REQUIRE(d_packed && d_scale, AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(rpw > 0 && lpr > 0 && rpw * lpr == 32 && N > 0 && K > 0 && N % rpw == 0 &&
                     K % 128 == 0 && (K / 32) % lpr == 0 && matrix >= 0 && matrix <= 2,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad shape (N=%d K=%d rpw=%d lpr=%d matrix=%d)", who,
                 N, K, rpw, lpr, matrix);
    AEON_REQUIRE(scale_group == 128 || scale_group == 32, AEON_ERR_INVALID_ARGUMENT,
                 "%s: scale_group must be 128 or 32, not %d", who, scale_group);
    const size_t slots = static_cast<size_t>(N) * (K / 32);
    synth_matrix_kernel<<<static_cast<unsigned>((slots + 255) / 256), 256, 0, as_stream(stream)>>>(
        stream_key(seed, matrix, expert), stream_key(seed, 8 + matrix, expert), N, K, rpw, lpr,
        scale_group, static_cast<uint4*>(d_packed), static_cast<uint16_t*>(d_scale));
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}
