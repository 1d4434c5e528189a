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
//   * the window's live count picks the body: 1, 2, 3 or 4 token tiles with three K groups in
//     flight (bound by the latency of the weight stream) or 6 or 8 with one (bound by
//     arithmetic), all hand-pipelined block by block (grouped_run), so an expert with a
//     handful of tokens costs its weight stream and little else and no window computes more
//     than two token tiles of padding.
// Weights are read once per (expert, position tile); tiles of one expert are adjacent in the
// grid so their re-reads meet in L2 / Infinity Cache.
#include <type_traits>

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

// s_waitcnt that only bounds the number of outstanding vector-memory loads (gfx9 encoding:
// vmcnt in bits 3:0 and 15:14, the export and LDS/scalar counters left at "no wait").
#define AEON_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | 0x0F70)

// The body for a window of LIVE token tiles (rows past the tile's live count are clamped reads
// whose results are never stored), with the weights and the activation window of DEPTH later K
// groups in flight while one is computed: small windows are bound by the latency of the weight
// stream and keep three groups in flight in the registers and LDS their few accumulators leave
// free, wide ones are bound by arithmetic and keep one.
//
// A K group is 4*LIVE blocks; block (st, mt) is the NM*R MFMAs of MFMA step st on token tile mt.
// VALU work hides behind the matrix pipe only when the same wave issues it right after an MFMA,
// so the group is software-pipelined by hand, block by block:
//   * the B fragments of a pair of blocks are read from LDS one pair early;
//   * the weight fragments of MFMA step st+1 (for st = 3: step 0 of the next K group) are
//     unpacked in shares spread over the blocks of step st, behind their MFMAs;
//   * the fragment registers alternate by step parity, so nothing is copied;
//   * a scheduling fence after every pair keeps the compiler from regrouping any of it.
// Loads complete in issue order and every group issues the same number, so "group g+1 has
// landed" is a bound on the count of outstanding loads; a group ends in a bare s_barrier (the
// fences of __syncthreads would wait for every LDS-DMA request and drain the ring).
template <bool GATE_UP, int R, int LIVE, int DEPTH, int SG, bool STREAM>
__device__ __forceinline__ void grouped_run(const SegGateUpArgs& gu, const SegDownArgs& dn,
                                                 const aeon_a64_expert& e, int first, int count,
                                                 half8_t* xs_flat, int nblock) {
    static_assert(LIVE >= 1 && LIVE <= kGroupedMT, "a window holds at most kGroupedMT token tiles");
    constexpr int NM = GATE_UP ? 2 : 1;
    constexpr int STAGES = DEPTH + 1;
    constexpr int kLoadsPerGroup = LIVE + NM * R * 2;
    static_assert(STAGES * LIVE <= 2 * kGroupedMT, "the ring must fit the window buffer");
    static_assert(STAGES >= 2 && STAGES <= 4, "the turn of the ring is written out for 2..4 slots");
    static_assert((DEPTH - 1) * kLoadsPerGroup < 64, "vmcnt is a 6-bit counter");
    constexpr int kFrags = NM * R;
    constexpr int kBufferStride = LIVE * 4 * 64;  // in 16-byte units
    constexpr int kBlocks = 4 * LIVE;
    static_assert(kFrags == 4, "one fragment is unpacked per two blocks");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: LDS-DMA targets stay scalar
    const int n = lane & 15;
    const int chunk = lane >> 4;
    const int tile0 = (nblock * 4 + wave) * R;

    const int K = GATE_UP ? gu.H : dn.I;
    const int groups = K / 128;
    const AEON_GLOBAL char* pm[NM];
    const AEON_GLOBAL char* sm[NM];
    pm[0] = as_global<char>(GATE_UP ? e.w1_packed : e.w2_packed);
    sm[0] = as_global<char>(GATE_UP ? e.w1_scale : e.w2_scale);
    if (GATE_UP) {
        pm[NM - 1] = as_global<char>(e.w3_packed);
        sm[NM - 1] = as_global<char>(e.w3_scale);
    }
    uint32_t woff[R], soff[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t t = static_cast<uint32_t>(tile0 + r) * groups;
        woff[r] = (t * 64 + lane) * 16;
        soff[r] = (t * 16 + n) * 2 * SG;   // the row's scale(s) of group 0: 2 or 8 bytes
    }
    const AEON_GLOBAL char* xbase = as_global<char>(GATE_UP ? static_cast<const void*>(gu.x)
                                                            : static_cast<const void*>(dn.hidden));
    // Activation fragments (16 positions x 32 columns = 16 x 64 bytes) go to LDS by DMA, lane l's
    // 16 bytes to byte 16 l of the fragment. In the matrix instruction's lane order (position
    // l%16, 16-byte piece l/16) every lane would be a cache access of its own, 64 per wave load.
    // Instead lanes 4q..4q+3 fetch the four pieces of position q, 64 contiguous bytes (16
    // accesses per load), rotated by q/2 so that the MFMA-order read-back -- lane (n, chunk)
    // takes unit 4n + (chunk + n/2) % 4 -- is as free of bank conflicts as a linear read
    // (measured with the benchmark's LDS read-order aid: 2.3 ns per wave read and CU, as the
    // linear read; 2.5-3.4 unrotated).
    const int load_row = lane >> 2;
    const int load_piece = ((lane & 3) - (load_row >> 1)) & 3;
    const int fragment_unit = 4 * n + ((chunk + (n >> 1)) & 3);
    uint32_t xoff[LIVE];
#pragma unroll
    for (int j = 0; j < LIVE; ++j) {
        const int row = j * 16 + load_row;
        const int live_row = row < count ? row : count - 1;
        const int position = first + live_row;
        const int column = wave * 32 + load_piece * 8;
        if (GATE_UP) {
            const long src_row = gu.row_index != nullptr ? gu.row_index[position] : position;
            xoff[j] = static_cast<uint32_t>((src_row * gu.x_stride + column) * 2);
        } else {
            xoff[j] = static_cast<uint32_t>((static_cast<size_t>(position) * dn.I + column) * 2);
        }
    }

    float4_t acc[NM][R][LIVE];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int mt = 0; mt < LIVE; ++mt) acc[m][r][mt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    u32x4_t wq[STAGES][NM][R];
    // the row's scale of the group, or its four (one per MFMA step): the step's weights are
    // multiplied by the step's scale in fp16, one rounding per weight either way
    using RowScales = std::conditional_t<SG == 4, u32x2_t, uint16_t>;
    RowScales sc[STAGES][NM][R];
#define AEON_FULL_ISSUE(g_, stage_)                                                                 \
    do {                                                                                            \
        const int gi_ = (g_) < groups ? (g_) : groups - 1;                                          \
        _Pragma("unroll") for (int j = 0; j < LIVE; ++j) {                                          \
            __builtin_amdgcn_global_load_lds(                                                       \
                (const AEON_GLOBAL void*)(xbase + (xoff[j] + static_cast<uint32_t>(gi_) * 256u)),   \
                (__attribute__((address_space(3))) void*)(xs_flat + (stage_) * kBufferStride +      \
                                                          (j * 4 + wave) * 64),                     \
                16, 0, 0);                                                                          \
        }                                                                                           \
        _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                            \
            _Pragma("unroll") for (int r = 0; r < R; ++r) {                                         \
                wq[stage_][m][r] = load_maybe_stream<STREAM>((const AEON_GLOBAL u32x4_t*)(          \
                    pm[m] + (woff[r] + static_cast<uint32_t>(gi_) * 1024u)));                       \
                sc[stage_][m][r] = *(const AEON_GLOBAL RowScales*)(                                 \
                    sm[m] + (soff[r] + static_cast<uint32_t>(gi_) * (32u * SG)));                   \
            }                                                                                       \
        }                                                                                           \
    } while (0)

    auto scale_pair = [](const RowScales& row, int st) {
        union { uint16_t u; half_t h; } v;
        if constexpr (SG == 4) {
            const uint32_t w = row[st >> 1];
            v.u = static_cast<uint16_t>((st & 1) ? (w >> 16) : (w & 0xFFFFu));
        } else {
            v.u = row;
        }
        return half2_t{v.h, v.h};
    };
    // B fragment of block i (token tile i % LIVE, MFMA step i / LIVE) of a ring slot.
    auto fragment = [&](int slot, int i) {
        return xs_flat[slot * kBufferStride + ((i % LIVE) * 4 + i / LIVE) * 64 + fragment_unit];
    };

    // Loads complete in issue order and every group issues the same number, so "group g+1 has
    // landed" is a bound on the number of younger requests still outstanding.
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) AEON_FULL_ISSUE(d, d);
    AEON_WAIT_VMCNT((DEPTH - 1) * kLoadsPerGroup);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);

    // weight fragments of the current MFMA step and of the next one: step st reads a[st % 2]
    // and fills a[(st + 1) % 2]; four steps a group keep the parity the same in every group
    half8_t a[2][NM][R];
    half8_t b[4];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) a[0][m][r] = scaled_fragment(wq[0][m][r][0], scale_pair(sc[0][m][r], 0));
    b[0] = fragment(0, 0);
    b[1] = fragment(0, 1);
    __builtin_amdgcn_sched_barrier(0);

    // One K group out of ring slot s; group g+DEPTH is requested first, into the slot the previous
    // group was computed from (free since the barrier that ended it).
    // Blocks go in pairs. While LDS-DMA requests are outstanding the compiler waits for every
    // LDS read at once, so the two reads of the next pair are placed behind the first MFMA of
    // this pair -- behind the wait for this pair's own fragments -- and have the pair's eight
    // MFMAs to land.
    auto step = [&](int g, auto slot) {
        constexpr int s = decltype(slot)::value;
        constexpr int sn = (s + 1) % STAGES;
        AEON_FULL_ISSUE(g + DEPTH, (s + DEPTH) % STAGES);
        __builtin_amdgcn_sched_barrier(0);
        // the MFMAs of block i and this block's share of the next MFMA step's weight fragments
        // (for the last step: of step 0 of the next K group, out of the next ring slot)
        auto block = [&](int i, bool skip_first) {
            const int st = i / LIVE, mt = i % LIVE;
#pragma unroll
            for (int m = 0; m < NM; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (!(skip_first && m + r == 0))
                        acc[m][r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[st % 2][m][r], b[i % 4],
                                                                                acc[m][r][mt], 0, 0, 0);
#pragma unroll
            for (int f = 0; f < kFrags; ++f) {
                if (f * LIVE / kFrags == mt) {
                    const int m = f / R, r = f % R;
                    a[(st + 1) % 2][m][r] =
                        st < 3 ? scaled_fragment(wq[s][m][r][st < 3 ? st + 1 : 0],
                                                 scale_pair(sc[s][m][r], st < 3 ? st + 1 : 0))
                               : scaled_fragment(wq[sn][m][r][0], scale_pair(sc[sn][m][r], 0));
                }
            }
        };
#pragma unroll
        for (int i = 0; i < kBlocks; i += 2) {
            if (i <= 3 * LIVE && 3 * LIVE < i + 2) {
                // the pair that starts the last MFMA step: from here on the weights of group
                // g+1 are unpacked, and this wave's requests for them are at least two thirds of
                // a group's arithmetic old
                AEON_WAIT_VMCNT((DEPTH - 1) * kLoadsPerGroup);
                __builtin_amdgcn_sched_barrier(0);
            }
            acc[0][0][i % LIVE] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                a[(i / LIVE) % 2][0][0], b[i % 4], acc[0][0][i % LIVE], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (i + 2 < kBlocks) {
                b[(i + 2) % 4] = fragment(s, i + 2);
                b[(i + 3) % 4] = fragment(s, i + 3);
            }
            block(i, true);
            block(i + 1, false);
            __builtin_amdgcn_sched_barrier(0);
        }
        // every wave's window of group g+1 has landed, and nobody reads slot s any more
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        b[0] = fragment(sn, 0);
        b[1] = fragment(sn, 1);
        __builtin_amdgcn_sched_barrier(0);
    };
    // whole turns of the ring as straight-line code, then the last partial turn
    int g = 0;
    for (; g + STAGES <= groups; g += STAGES) {
        step(g, std::integral_constant<int, 0>{});
        step(g + 1, std::integral_constant<int, 1>{});
        if constexpr (STAGES > 2) step(g + 2, std::integral_constant<int, 2>{});
        if constexpr (STAGES > 3) step(g + 3, std::integral_constant<int, 3>{});
    }
    if (g < groups) step(g, std::integral_constant<int, 0>{});
    if (g + 1 < groups) step(g + 1, std::integral_constant<int, 1>{});
    if constexpr (STAGES > 3) {
        if (g + 2 < groups) step(g + 2, std::integral_constant<int, 2>{});
    }
#undef AEON_FULL_ISSUE

#pragma unroll
    for (int mt = 0; mt < LIVE; ++mt) {
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

template <bool GATE_UP, int R, int SG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void a64_grouped_kernel(
    SegGateUpArgs gu, SegDownArgs dn) {
    const SegmentList& seg = GATE_UP ? gu.seg : dn.seg;
    // Workgroups go to the eight XCDs round robin by their linear index, and every XCD has an L2
    // of its own. Index i therefore serves window 8*(i/8/blocks) + i%8, row block (i/8)%blocks:
    // all row blocks of one window run on one XCD and fetch the window's activations into that
    // L2 once, not once per XCD.
    const int linear = blockIdx.y * gridDim.x + blockIdx.x;
    const int slot = linear >> 3;
    const int s = (slot / gridDim.x) * 8 + (linear & 7);
    const int nblock = slot % gridDim.x;
    if (s >= *seg.total) return;
    const int first = seg.first[s];
    const int count = seg.count[s];
    const aeon_a64_expert e = (GATE_UP ? gu.experts : dn.experts)[seg.expert[s]];

    // Activation windows in LDS, fragment-major: [ring slot][token tile][step][lane] x 16 bytes,
    // so a B operand is one conflict-free ds_read_b128 per lane. 64 KiB: two slots of a full
    // window, or a deeper ring of smaller ones.
    __shared__ half8_t xs[2 * kGroupedMT * 4 * 64];

    // A window that is its expert's only one reads weights nobody reads again: streamed past the
    // caches. The windows of a hot expert find each other's weights in L2 and load normally.
    const bool alone = seg.alone != nullptr && seg.alone[s] != 0;
    const int live_tiles = (count + 15) >> 4;
#define AEON_RUN(live_, depth_)                                                                  \
    do {                                                                                         \
        if (alone) grouped_run<GATE_UP, R, live_, depth_, SG, true>(gu, dn, e, first, count, xs, nblock);  \
        else grouped_run<GATE_UP, R, live_, depth_, SG, false>(gu, dn, e, first, count, xs, nblock);       \
    } while (0)
    if (live_tiles > 6) {
        AEON_RUN(8, 1);
    } else if (live_tiles > 4) {
        AEON_RUN(6, 1);
    } else if (live_tiles > 3) {
        AEON_RUN(4, 3);
    } else if (live_tiles > 2) {
        AEON_RUN(3, 3);
    } else if (live_tiles > 1) {
        AEON_RUN(2, 3);
    } else {
        AEON_RUN(1, 3);
    }
#undef AEON_RUN
}

int launch_grouped_gate_up(const SegGateUpArgs& a, hipStream_t stream) {
    AEON_REQUIRE(a.H % 128 == 0 && a.I % 128 == 0 && a.x_stride % 8 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "grouped gate/up: need H%%128==0, I%%128==0 and an activation pitch that keeps "
                 "rows 16-byte aligned (H=%d I=%d pitch=%ld)", a.H, a.I, a.x_stride);
    AEON_REQUIRE(a.seg.total != nullptr, AEON_ERR_INVALID_ARGUMENT,
                 "grouped gate/up: needs a position-tile list");
    if (a.seg.capacity <= 0) return AEON_OK;
    AEON_REQUIRE(a.scales_per_group == 1 || a.scales_per_group == 4, AEON_ERR_INVALID_ARGUMENT,
                 "grouped gate/up: %d scales per 128 columns (1 or 4)", a.scales_per_group);
    const int cap = (a.seg.capacity + 7) & ~7;   // whole rounds of the eight XCDs
    if (a.scales_per_group == 4) {
        a64_grouped_kernel<true, 2, 4><<<dim3(a.I / 128, cap), 256, 0, stream>>>(a, SegDownArgs{});
    } else {
        a64_grouped_kernel<true, 2, 1><<<dim3(a.I / 128, cap), 256, 0, stream>>>(a, SegDownArgs{});
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

int launch_grouped_down(const SegDownArgs& a, hipStream_t stream) {
    AEON_REQUIRE(a.I % 128 == 0 && a.H % 256 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "grouped down: need I%%128==0 and H%%256==0 (H=%d I=%d)", a.H, a.I);
    AEON_REQUIRE(a.seg.total != nullptr, AEON_ERR_INVALID_ARGUMENT,
                 "grouped down: needs a position-tile list");
    if (a.seg.capacity <= 0) return AEON_OK;
    AEON_REQUIRE(a.scales_per_group == 1 || a.scales_per_group == 4, AEON_ERR_INVALID_ARGUMENT,
                 "grouped down: %d scales per 128 columns (1 or 4)", a.scales_per_group);
    const int cap = (a.seg.capacity + 7) & ~7;
    if (a.scales_per_group == 4) {
        a64_grouped_kernel<false, 4, 4><<<dim3(a.H / 256, cap), 256, 0, stream>>>(SegGateUpArgs{}, a);
    } else {
        a64_grouped_kernel<false, 4, 1><<<dim3(a.H / 256, cap), 256, 0, stream>>>(SegGateUpArgs{}, a);
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

}  // namespace aeon355
