// Prefill: grouped expert GEMM on fp16 MFMA with int4 dequantisation in registers.
//
// One workgroup = (a tile of up to 16*MT permuted positions of one expert) x (4 waves x R
// 16-row weight tiles). For every 128-column group:
//   * the activation tile (positions x 128 columns, fp16) is staged in LDS in MFMA-fragment
//     order, double-buffered, fetched one group ahead;
//   * each wave reads its NM*R weight tiles (1 KiB each, the wave64 packing) straight into
//     registers, one group ahead, unpacks a word into the A operand of
//     v_mfma_f32_16x16x32_f16 and multiplies by the row's fp16 scale (one rounding per weight,
//     as the reference's grouped feed does); the fragment is then reused for every token tile
//     of the window, which is what makes the dequantisation cheap next to the MFMAs;
//   * token tiles past the tile's live count are skipped, so an expert with a handful of
//     tokens costs its weight stream and little else.
// Weights are read once per (expert, position tile); tiles of one expert are adjacent in the
// grid so their re-reads meet in L2 / Infinity Cache.
#include "expert_a64.hpp"

namespace aeon355 {

constexpr int kGroupedMT = 8;                    // token tiles per workgroup window
static_assert(16 * kGroupedMT == kGroupedTokensPerTile, "window = the position-tile size");

__device__ __forceinline__ half8_t scaled_fragment(uint32_t word, half2_t scale2) {
    half2_t p[4];
    unpack8(word, p);
    p[0] *= scale2;
    p[1] *= scale2;
    p[2] *= scale2;
    p[3] *= scale2;
    half8_t v = {p[0][0], p[0][1], p[1][0], p[1][1], p[2][0], p[2][1], p[3][0], p[3][1]};
    return v;
}

template <bool GATE_UP, int R>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void a64_grouped_kernel(
    SegGateUpArgs gu, SegDownArgs dn) {
    constexpr int NM = GATE_UP ? 2 : 1;
    constexpr int MT = kGroupedMT;
    const SegmentList& seg = GATE_UP ? gu.seg : dn.seg;
    const int s = blockIdx.y;
    if (s >= *seg.total) return;
    const int first = seg.first[s];
    const int count = seg.count[s];
    const aeon_a64_expert e = (GATE_UP ? gu.experts : dn.experts)[seg.expert[s]];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;
    const int chunk = lane >> 4;
    const int tile0 = (blockIdx.x * 4 + wave) * R;
    const int live_tiles = (count + 15) >> 4;

    const int K = GATE_UP ? gu.H : dn.I;
    const int groups = K / 128;
    const AEON_GLOBAL u32x4_t* pm[NM];
    const AEON_GLOBAL uint16_t* sm[NM];
    pm[0] = as_global<u32x4_t>(GATE_UP ? e.w1_packed : e.w2_packed);
    sm[0] = as_global<uint16_t>(GATE_UP ? e.w1_scale : e.w2_scale);
    if (GATE_UP) {
        pm[NM - 1] = as_global<u32x4_t>(e.w3_packed);
        sm[NM - 1] = as_global<uint16_t>(e.w3_scale);
    }

    // Activation tile in LDS, fragment-major: [buffer][token tile][step][lane] x 16 bytes, so a
    // B operand is one conflict-free ds_read_b128 per lane.
    __shared__ half8_t xs[2][MT][4][64];

    // Staging assignment: the tile is MT*4 fragments of 1 KiB (token tile mt, MFMA step st); wave
    // w stages fragments w*kFrags .. +kFrags-1. Lane (n, chunk) of a fragment fetches 16 bytes of
    // row mt*16+n at column st*32 + chunk*8 and stores them at the lane's own 16-byte slot, so
    // the LDS write of a wave is one contiguous KiB (no bank conflicts) and is the exact image
    // the B-operand read wants.
    constexpr int kFrags = MT * 4 / 4;  // per wave
    const AEON_GLOBAL uint16_t* frag_src[kFrags];
#pragma unroll
    for (int j = 0; j < kFrags; ++j) {
        const int f = wave * kFrags + j;
        const int row = (f >> 2) * 16 + n;
        const int live_row = row < count ? row : count - 1;
        const int position = first + live_row;
        const int column = (f & 3) * 32 + chunk * 8;
        if (GATE_UP) {
            const long src_row = gu.row_index != nullptr ? gu.row_index[position] : position;
            frag_src[j] = as_global<uint16_t>(gu.x) + src_row * gu.x_stride + column;
        } else {
            frag_src[j] = as_global<uint16_t>(dn.hidden) + static_cast<size_t>(position) * dn.I + column;
        }
    }
    half8_t* xs_flat = &xs[0][0][0][0];
    constexpr int kBufferStride = MT * 4 * 64;

    float4_t acc[NM][R][MT];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[m][r][mt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    u32x4_t wq[NM][R];
    uint16_t sc[NM][R];
    auto load_weights = [&](int g) {
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const size_t t = static_cast<size_t>(tile0 + r) * groups + g;
                wq[m][r] = pm[m][t * 64 + lane];
                sc[m][r] = sm[m][t * 16 + n];  // the A operand's row is lane % 16
            }
    };

    // Activation fragments go from global memory straight into LDS (global_load_lds, 16 bytes
    // per lane landing at the lane's own slot of the fragment): no staging registers, no LDS
    // write instructions. The tile for group g+1 is requested at the top of step g into the
    // other buffer; every wave drains its own requests before the barrier that ends the step.
    auto fetch_tile = [&](int g, int buffer) {
#pragma unroll
        for (int j = 0; j < kFrags; ++j) {
            const int f = wave * kFrags + j;
            if ((f >> 2) < live_tiles) {
                __builtin_amdgcn_global_load_lds(
                    (const AEON_GLOBAL void*)(frag_src[j] + g * 128),
                    (__attribute__((address_space(3))) void*)(xs_flat + buffer * kBufferStride + f * 64),
                    16, 0, 0);
            }
        }
    };

    fetch_tile(0, 0);
    load_weights(0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    for (int g = 0; g < groups; ++g) {
        const int gn = g + 1 < groups ? g + 1 : g;  // the last step refetches its own group, unused
        u32x4_t wcur[NM][R];
        half2_t scur[NM][R];
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                wcur[m][r] = wq[m][r];
                union { uint16_t u; half_t h; } v;
                v.u = sc[m][r];
                scur[m][r] = half2_t{v.h, v.h};
            }
        fetch_tile(gn, (g + 1) & 1);
        load_weights(gn);
        const half8_t* xb = xs_flat + (g & 1) * kBufferStride;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            half8_t a[NM][R];
#pragma unroll
            for (int m = 0; m < NM; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r) a[m][r] = scaled_fragment(wcur[m][r][st], scur[m][r]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (mt < live_tiles) {
                    const half8_t b = xb[(mt * 4 + st) * 64 + lane];
#pragma unroll
                    for (int m = 0; m < NM; ++m)
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            acc[m][r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                a[m][r], b, acc[m][r][mt], 0, 0, 0);
                        }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    }

#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int row = mt * 16 + n;  // position within the tile
        if (row < count) {
            const int position = first + row;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int row0 = (tile0 + r) * 16 + chunk * 4;
                if (GATE_UP) {
                    const float4_t& ga = acc[0][r][mt];
                    const float4_t& up = acc[NM - 1][r][mt];
                    uint2 packed;
                    packed.x = float_to_half_bits(clamped_swiglu(ga[0], up[0], gu.limit)) |
                               (static_cast<uint32_t>(float_to_half_bits(
                                    clamped_swiglu(ga[1], up[1], gu.limit))) << 16);
                    packed.y = float_to_half_bits(clamped_swiglu(ga[2], up[2], gu.limit)) |
                               (static_cast<uint32_t>(float_to_half_bits(
                                    clamped_swiglu(ga[3], up[3], gu.limit))) << 16);
                    *reinterpret_cast<uint2*>(gu.hidden + static_cast<size_t>(position) * gu.I + row0) = packed;
                } else {
                    const float w = dn.weight[position];
                    const float4_t& a4 = acc[0][r][mt];
                    const float4_t v = {w * a4[0], w * a4[1], w * a4[2], w * a4[3]};
                    const size_t out_row = dn.out_row != nullptr ? dn.out_row[position] : position;
                    *reinterpret_cast<float4_t*>(dn.contrib + out_row * dn.H + row0) = v;
                }
            }
        }
    }
}

int launch_grouped_gate_up(const SegGateUpArgs& a, hipStream_t stream) {
    AEON_REQUIRE(a.H % 128 == 0 && a.I % 128 == 0 && a.x_stride % 8 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "grouped gate/up: need H%%128==0, I%%128==0 and an activation pitch that keeps "
                 "rows 16-byte aligned (H=%d I=%d pitch=%ld)", a.H, a.I, a.x_stride);
    AEON_REQUIRE(a.seg.total != nullptr, AEON_ERR_INVALID_ARGUMENT,
                 "grouped gate/up: needs a position-tile list");
    if (a.seg.capacity <= 0) return AEON_OK;
    a64_grouped_kernel<true, 2><<<dim3(a.I / 128, a.seg.capacity), 256, 0, stream>>>(a, SegDownArgs{});
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

int launch_grouped_down(const SegDownArgs& a, hipStream_t stream) {
    AEON_REQUIRE(a.I % 128 == 0 && a.H % 256 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "grouped down: need I%%128==0 and H%%256==0 (H=%d I=%d)", a.H, a.I);
    AEON_REQUIRE(a.seg.total != nullptr, AEON_ERR_INVALID_ARGUMENT,
                 "grouped down: needs a position-tile list");
    if (a.seg.capacity <= 0) return AEON_OK;
    a64_grouped_kernel<false, 4><<<dim3(a.H / 256, a.seg.capacity), 256, 0, stream>>>(SegGateUpArgs{}, a);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

}  // namespace aeon355
