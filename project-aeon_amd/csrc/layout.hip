// Weight layouts: the reference's wave32 swizzle (host), and the gfx950 wave64 packing the
// decode and grouped kernels read ("A64"), with its host and device repack from the `.aeon`
// swizzled payload.
//
// A64 tile = 16 rows x 128 columns = 64 lanes x uint4 (1 KiB, one coalesced wave load).
// Lane l = (row l%16, chunk l/16); word s of the lane's uint4 holds columns
// 128g + 32s + 8*chunk + 0..7, which is exactly the A operand of one
// v_mfma_f32_16x16x32_f16 step (lane l supplies row l%16, k = 8*(l/16)..+7), so four
// MFMA steps consume one tile with no cross-lane movement; a VALU GEMV reads the same
// words against four 16-byte activation chunks. Scales come in two forms, chosen when the
// matrix is repacked: one fp16 per (row, 128-column group) at [tile][row%16] -- for payloads
// whose four group-32 scales inside every 128 columns are bit-equal -- or all four kept, at
// [tile][row%16][step], step s being the scale of columns 128g+32s..+31, i.e. of MFMA step s.
#include "common.hpp"

#include <cstring>

namespace aeon355 {

static const int kNibblePerm[8] = {0, 2, 4, 6, 1, 3, 5, 7};

static inline uint32_t permute_word(uint32_t source) {
    uint32_t out = 0;
    for (int p = 0; p < 8; ++p) out |= ((source >> (4 * kNibblePerm[p])) & 0xFu) << (4 * p);
    return out;
}

static inline uint32_t unpermute_word(uint32_t source) {
    uint32_t out = 0;
    for (int p = 0; p < 8; ++p) out |= ((source >> (4 * p)) & 0xFu) << (4 * kNibblePerm[p]);
    return out;
}

static bool swizzle_shape_ok(int N, int K, int rpw, int lpr) {
    return rpw > 0 && lpr > 0 && rpw * lpr == 32 && N > 0 && K > 0 && N % rpw == 0 &&
           K % 32 == 0 && (K / 32) % lpr == 0;
}

// Index of the uint4 slot that holds (row, 32-column group) in the swizzled payload.
__host__ __device__ static inline size_t swizzled_slot(int row, int group32, int rpw, int lpr,
                                                       int iterations) {
    const int block = row / rpw;
    const int lane = (row % rpw) * lpr + group32 % lpr;
    return (static_cast<size_t>(block) * iterations + group32 / lpr) * 32 + lane;
}

// Index of the uint4 slot of (row, 128-column group, chunk) in the A64 packing.
__host__ __device__ static inline size_t a64_slot(int row, int group128, int chunk, int groups) {
    const size_t tile = static_cast<size_t>(row / 16) * groups + group128;
    return tile * 64 + chunk * 16 + row % 16;
}

static bool a64_shape_ok(int N, int K, int rpw, int lpr) {
    return swizzle_shape_ok(N, K, rpw, lpr) && N % 16 == 0 && K % 128 == 0;
}

static bool scale_group_ok(int scale_group) { return scale_group == 128 || scale_group == 32; }

// Index of the fp16 scale of (row, 128-column group, MFMA step) in the A64 scale array.
__host__ __device__ static inline size_t a64_scale_index(int row, int group128, int step, int groups,
                                                         int per_group) {
    const size_t tile = static_cast<size_t>(row / 16) * groups + group128;
    return per_group == 4 ? (tile * 16 + row % 16) * 4 + step : tile * 16 + row % 16;
}

__global__ __launch_bounds__(256) void a64_repack_kernel(
    const uint32_t* __restrict__ swz_packed, const uint16_t* __restrict__ swz_scale,
    uint4* __restrict__ a64_packed, uint16_t* __restrict__ a64_scale, int N, int K, int rpw,
    int lpr, int per_group, int* __restrict__ mismatch) {
    // One thread per destination uint4: coalesced 16-byte stores; the four source words sit
    // in four different swizzled slots (one per 32-column step).
    const int groups = K / 128;
    const int iterations = (K / 32) / lpr;
    const size_t total = static_cast<size_t>(N) * groups * 4;
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int lane = static_cast<int>(idx % 64);
    const size_t tile = idx / 64;
    const int g = static_cast<int>(tile % groups);
    const int row = static_cast<int>(tile / groups) * 16 + lane % 16;
    const int chunk = lane / 16;
    uint32_t words[4];
    uint16_t scales[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        const size_t slot = swizzled_slot(row, g * 4 + s, rpw, lpr, iterations);
        words[s] = swz_packed[slot * 4 + chunk];
        scales[s] = swz_scale[slot];
    }
    a64_packed[idx] = make_uint4(words[0], words[1], words[2], words[3]);
    if (chunk == 0) {
        if (per_group == 4) {
            // 8 bytes per row: the row's four step scales side by side
            const uint2 four = make_uint2(scales[0] | (static_cast<uint32_t>(scales[1]) << 16),
                                          scales[2] | (static_cast<uint32_t>(scales[3]) << 16));
            reinterpret_cast<uint2*>(a64_scale)[tile * 16 + row % 16] = four;
        } else {
            a64_scale[tile * 16 + row % 16] = scales[0];
            if (mismatch != nullptr &&
                (scales[1] != scales[0] || scales[2] != scales[0] || scales[3] != scales[0])) {
                atomicAdd(mismatch, 1);
            }
        }
    }
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_swizzle_w4a16(const uint32_t* src_packed, const uint16_t* src_scale,
                                  uint32_t* dst_packed, uint16_t* dst_scale, int N, int K,
                                  int rpw, int lpr) {
    AEON_REQUIRE(src_packed && src_scale && dst_packed && dst_scale, AEON_ERR_INVALID_ARGUMENT,
                 "aeon_swizzle_w4a16: null buffer");
    AEON_REQUIRE(swizzle_shape_ok(N, K, rpw, lpr), AEON_ERR_INVALID_ARGUMENT,
                 "aeon_swizzle_w4a16: incompatible N/K/cfg (N=%d K=%d rpw=%d lpr=%d)", N, K, rpw, lpr);
    const int groups = K / 32;
    const int iterations = groups / lpr;
    const int words_per_row = K / 8;
    for (int row = 0; row < N; ++row) {
        for (int group = 0; group < groups; ++group) {
            const size_t slot = swizzled_slot(row, group, rpw, lpr, iterations);
            const uint32_t* src = src_packed + static_cast<size_t>(row) * words_per_row + group * 4;
            for (int w = 0; w < 4; ++w) dst_packed[slot * 4 + w] = permute_word(src[w]);
            dst_scale[slot] = src_scale[static_cast<size_t>(row) * groups + group];
        }
    }
    return AEON_OK;
}

extern "C" int aeon_unswizzle_w4a16(const uint32_t* src_packed, const uint16_t* src_scale,
                                    uint32_t* dst_packed, uint16_t* dst_scale, int N, int K,
                                    int rpw, int lpr) {
    AEON_REQUIRE(src_packed && src_scale && dst_packed && dst_scale, AEON_ERR_INVALID_ARGUMENT,
                 "aeon_unswizzle_w4a16: null buffer");
    AEON_REQUIRE(swizzle_shape_ok(N, K, rpw, lpr), AEON_ERR_INVALID_ARGUMENT,
                 "aeon_unswizzle_w4a16: incompatible N/K/cfg (N=%d K=%d rpw=%d lpr=%d)", N, K, rpw, lpr);
    const int groups = K / 32;
    const int iterations = groups / lpr;
    const int words_per_row = K / 8;
    for (int row = 0; row < N; ++row) {
        for (int group = 0; group < groups; ++group) {
            const size_t slot = swizzled_slot(row, group, rpw, lpr, iterations);
            uint32_t* dst = dst_packed + static_cast<size_t>(row) * words_per_row + group * 4;
            for (int w = 0; w < 4; ++w) dst[w] = unpermute_word(src_packed[slot * 4 + w]);
            dst_scale[static_cast<size_t>(row) * groups + group] = src_scale[slot];
        }
    }
    return AEON_OK;
}

extern "C" size_t aeon_a64_packed_bytes(int N, int K) {
    return static_cast<size_t>(N) * K / 2;
}

extern "C" size_t aeon_a64_scale_bytes(int N, int K, int scale_group) {
    if (!scale_group_ok(scale_group)) return 0;
    return static_cast<size_t>(N) * (K / 128) * 2 * (scale_group == 32 ? 4 : 1);
}

extern "C" int aeon_a64_repack_host(const uint32_t* swz_packed, const uint16_t* swz_scale, int N,
                                    int K, int rpw, int lpr, int scale_group,
                                    uint32_t* a64_packed, uint16_t* a64_scale) {
    AEON_REQUIRE(swz_packed && swz_scale && a64_packed && a64_scale, AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_repack_host: null buffer");
    AEON_REQUIRE(a64_shape_ok(N, K, rpw, lpr), AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_repack_host: needs N%%16==0, K%%128==0 and a valid swizzle cfg "
                 "(N=%d K=%d rpw=%d lpr=%d)", N, K, rpw, lpr);
    AEON_REQUIRE(scale_group_ok(scale_group), AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_repack_host: scale_group must be 128 or 32, not %d", scale_group);
    const int per_group = scale_group == 32 ? 4 : 1;
    const int groups = K / 128;
    const int iterations = (K / 32) / lpr;
    for (int row = 0; row < N; ++row) {
        for (int g = 0; g < groups; ++g) {
            uint16_t scales[4];
            for (int s = 0; s < 4; ++s) {
                const size_t slot = swizzled_slot(row, g * 4 + s, rpw, lpr, iterations);
                scales[s] = swz_scale[slot];
                for (int chunk = 0; chunk < 4; ++chunk) {
                    a64_packed[a64_slot(row, g, chunk, groups) * 4 + s] = swz_packed[slot * 4 + chunk];
                }
            }
            if (per_group == 4) {
                for (int s = 0; s < 4; ++s) a64_scale[a64_scale_index(row, g, s, groups, 4)] = scales[s];
                continue;
            }
            AEON_REQUIRE(scales[1] == scales[0] && scales[2] == scales[0] && scales[3] == scales[0],
                         AEON_ERR_INVALID_ARGUMENT,
                         "aeon_a64_repack_host: row %d, 128-group %d carries four different "
                         "group-32 scales; repack with scale_group 32 to keep them", row, g);
            a64_scale[a64_scale_index(row, g, 0, groups, 1)] = scales[0];
        }
    }
    return AEON_OK;
}

extern "C" int aeon_a64_unrepack_host(const uint32_t* a64_packed, const uint16_t* a64_scale, int N,
                                      int K, int rpw, int lpr, int scale_group,
                                      uint32_t* swz_packed, uint16_t* swz_scale) {
    AEON_REQUIRE(swz_packed && swz_scale && a64_packed && a64_scale, AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_unrepack_host: null buffer");
    AEON_REQUIRE(a64_shape_ok(N, K, rpw, lpr), AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_unrepack_host: needs N%%16==0, K%%128==0 and a valid swizzle cfg "
                 "(N=%d K=%d rpw=%d lpr=%d)", N, K, rpw, lpr);
    AEON_REQUIRE(scale_group_ok(scale_group), AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_unrepack_host: scale_group must be 128 or 32, not %d", scale_group);
    const int per_group = scale_group == 32 ? 4 : 1;
    const int groups = K / 128;
    const int iterations = (K / 32) / lpr;
    for (int row = 0; row < N; ++row) {
        for (int g = 0; g < groups; ++g) {
            for (int s = 0; s < 4; ++s) {
                const size_t slot = swizzled_slot(row, g * 4 + s, rpw, lpr, iterations);
                swz_scale[slot] = a64_scale[a64_scale_index(row, g, s, groups, per_group)];
                for (int chunk = 0; chunk < 4; ++chunk) {
                    swz_packed[slot * 4 + chunk] = a64_packed[a64_slot(row, g, chunk, groups) * 4 + s];
                }
            }
        }
    }
    return AEON_OK;
}

extern "C" int aeon_a64_repack_device(const void* d_swz_packed, const void* d_swz_scale, int N,
                                      int K, int rpw, int lpr, int scale_group,
                                      void* d_a64_packed, void* d_a64_scale, int* d_mismatch,
                                      void* stream) {
    AEON_REQUIRE(d_swz_packed && d_swz_scale && d_a64_packed && d_a64_scale,
                 AEON_ERR_INVALID_ARGUMENT, "aeon_a64_repack_device: null buffer");
    AEON_REQUIRE(a64_shape_ok(N, K, rpw, lpr), AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_repack_device: needs N%%16==0, K%%128==0 and a valid swizzle cfg "
                 "(N=%d K=%d rpw=%d lpr=%d)", N, K, rpw, lpr);
    AEON_REQUIRE(scale_group_ok(scale_group), AEON_ERR_INVALID_ARGUMENT,
                 "aeon_a64_repack_device: scale_group must be 128 or 32, not %d", scale_group);
    const size_t total = static_cast<size_t>(N) * (K / 128) * 4;
    const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
    a64_repack_kernel<<<blocks, 256, 0, as_stream(stream)>>>(
        static_cast<const uint32_t*>(d_swz_packed), static_cast<const uint16_t*>(d_swz_scale),
        static_cast<uint4*>(d_a64_packed), static_cast<uint16_t*>(d_a64_scale), N, K, rpw, lpr,
        scale_group == 32 ? 4 : 1, d_mismatch);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}
