// Decode kernels over the wave64 ("A64") packing.
//
// Two families, both HBM-bound by construction (every weight byte is read once per segment in
// 1 KiB coalesced wave loads; scales at one fp16 per 128 columns, or -- template parameter
// SG = 4 -- the payload's own four per 128 columns, one per 32-column MFMA step):
//
//   * a64_gemv_kernel: VALU only. Lane (row l%16, chunk l/16) dequantises its 32 nibbles in
//     registers and feeds v_dot2_f32_f16 against four 16-byte activation chunks; the four
//     chunk lanes of a row meet through a wave xor-butterfly, K splits across the waves of the
//     workgroup meet through LDS. This is the GEMV / dual-GEMV of the decode path.
//   * a64_seg_kernel: for an expert that serves up to 16 tokens of a batch. The same 1 KiB
//     tile is, unchanged, the A operand of four v_mfma_f32_16x16x32_f16 steps whose B operand
//     is the 16 token rows, so the weight stream is read once however many of the 16 tokens are
//     live and the VALU work per byte does not grow with the token count. The scale is applied
//     in fp32 to the per-group MFMA result, so dequantisation stays exact.
#include "expert_a64.hpp"

#include <atomic>

namespace aeon355 {

// ---------------------------------------------------------------------------------------------
// VALU GEMV
// ---------------------------------------------------------------------------------------------

constexpr int kGemvPrefetch = 4;  // weight tiles a lane keeps in flight

struct GemvArgs {
    const uint16_t* x;
    long x_stride;
    const uint4* pa;
    const uint16_t* sa;
    const uint4* pb;
    const uint16_t* sb;
    uint16_t* out_a;
    uint16_t* out_b;
    long out_stride;
    int tokens;
    int N;
    int groups;  // K / 128
    // epilogue: 0 = fp16 rows of each matrix; 1 = out_a = half(clamped_swiglu(a, b));
    // 2 = out_f32[t][row] = tok_weight[t] * a (one writer per element)
    int epilogue;
    float limit;
    const float* tok_weight;
    float* out_f32;
    int scales_per_group;  // 1 (one fp16 per row and 128 columns) or 4 (one per 32 columns)
};

// HALF: a workgroup takes 8 of a tile's 16 rows (the lanes of the other 8 stay idle), so that a
// matrix with fewer than 256 row tiles still puts a workgroup on every CU: such a launch is a
// few microseconds long and bound by latency, not by the bytes a wave moves.
//
// XLDS: the batch's activation rows are copied to LDS once per workgroup and every lane reads
// its chunks from there. Without it a lane fetches 64 bytes per token and 128-column group from
// memory inside the token loop, and from four tokens on those dependent fetches are a sixth of
// the launch. (The copy comes first: with the first weights requested ahead of it the copy's
// LDS writes wait for the weights as well -- loads return in order -- and the launch is slower.)
template <int NMAT, int TOK, int WK, int SG, bool HALF, bool XLDS>
__global__ __launch_bounds__(WK * 64) void a64_gemv_kernel(GemvArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r = lane & 15;
    const int chunk = lane >> 4;
    const int tile = HALF ? blockIdx.x >> 1 : blockIdx.x;
    const size_t tile_base = static_cast<size_t>(tile) * a.groups;
    const bool mine = !HALF || (r >> 3) == static_cast<int>(blockIdx.x & 1);
    extern __shared__ uint4 x_lds[];  // XLDS: [tokens][groups * 16] 16-byte units
    const int row_units = a.groups * 16;
    if (XLDS) {
        for (int i = threadIdx.x; i < a.tokens * row_units; i += WK * 64) {
            const int t = i / row_units;
            x_lds[i] = *reinterpret_cast<const uint4*>(a.x + t * a.x_stride + (i - t * row_units) * 8);
        }
        __syncthreads();
    }

    float acc[NMAT][TOK];
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int t = 0; t < TOK; ++t) acc[m][t] = 0.0f;

    for (int g0 = wave; g0 < a.groups; g0 += WK * kGemvPrefetch) {
        uint4 wq[NMAT][kGemvPrefetch];
        // the row's scale(s) of the group: one fp16, or four (MFMA-step order) in 8 bytes
        uint2 sc[NMAT][kGemvPrefetch];
        auto load_scale = [&](const uint16_t* base, int g) {
            if (SG == 4) return *reinterpret_cast<const uint2*>(base + ((tile_base + g) * 16 + r) * 4);
            return make_uint2(base[(tile_base + g) * 16 + r], 0u);
        };
#pragma unroll
        for (int j = 0; j < kGemvPrefetch; ++j) {
            const int g = g0 + j * WK;
            if (g < a.groups && mine) {
                wq[0][j] = stream_load(&a.pa[(tile_base + g) * 64 + lane]);
                sc[0][j] = load_scale(a.sa, g);
                if (NMAT == 2) {
                    wq[1][j] = stream_load(&a.pb[(tile_base + g) * 64 + lane]);
                    sc[1][j] = load_scale(a.sb, g);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < kGemvPrefetch; ++j) {
            const int g = g0 + j * WK;
            if (g < a.groups && mine) {
                // the tile's nibbles become fp16 once, outside the token loop: every token of the
                // batch multiplies the same 32 weights of the lane
                half2_t q[NMAT][4][4];
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    unpack8(wq[m][j].x, q[m][0]);
                    unpack8(wq[m][j].y, q[m][1]);
                    unpack8(wq[m][j].z, q[m][2]);
                    unpack8(wq[m][j].w, q[m][3]);
                }
#pragma unroll
                for (int t = 0; t < TOK; ++t) {
                    if (t < a.tokens) {
                        uint4 x[4];
                        if (XLDS) {
                            const uint4* xp = x_lds + t * row_units + g * 16 + chunk;
                            x[0] = xp[0];
                            x[1] = xp[4];
                            x[2] = xp[8];
                            x[3] = xp[12];
                        } else {
                            const uint16_t* xp = a.x + t * a.x_stride + g * 128 + chunk * 8;
                            x[0] = *reinterpret_cast<const uint4*>(xp);
                            x[1] = *reinterpret_cast<const uint4*>(xp + 32);
                            x[2] = *reinterpret_cast<const uint4*>(xp + 64);
                            x[3] = *reinterpret_cast<const uint4*>(xp + 96);
                        }
#pragma unroll
                        for (int m = 0; m < NMAT; ++m) {
                            if (SG == 4) {
                                // word s of the lane holds columns of 32-column group s only
                                const uint2 s4 = sc[m][j];
                                const uint16_t step_scale[4] = {
                                    static_cast<uint16_t>(s4.x & 0xFFFFu), static_cast<uint16_t>(s4.x >> 16),
                                    static_cast<uint16_t>(s4.y & 0xFFFFu), static_cast<uint16_t>(s4.y >> 16)};
#pragma unroll
                                for (int st = 0; st < 4; ++st)
                                    acc[m][t] += half_bits_to_float(step_scale[st]) * dot8(q[m][st], x[st], 0.0f);
                            } else {
                                float d = 0.0f;
#pragma unroll
                                for (int st = 0; st < 4; ++st) d = dot8(q[m][st], x[st], d);
                                acc[m][t] += half_bits_to_float(static_cast<uint16_t>(sc[m][j].x)) * d;
                            }
                        }
                    }
                }
            }
        }
    }

    __shared__ float partial[WK][NMAT][TOK][16];
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int t = 0; t < TOK; ++t) {
            const float v = wave_xor_sum(acc[m][t], 16 | 32);
            if (chunk == 0) partial[wave][m][t][r] = v;
        }
    __syncthreads();

    for (int i = threadIdx.x; i < NMAT * TOK * 16; i += WK * 64) {
        const int row = i & 15;
        const int t = (i >> 4) % TOK;
        const int m = (i >> 4) / TOK;
        if (t < a.tokens && (!HALF || (row >> 3) == static_cast<int>(blockIdx.x & 1))) {
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < WK; ++w) sum += partial[w][m][t][row];
            const size_t at = t * a.out_stride + tile * 16 + row;
            if (a.epilogue == 0) {
                uint16_t* out = m == 0 ? a.out_a : a.out_b;
                out[at] = float_to_half_bits(sum);
            } else if (a.epilogue == 1) {
                if (m == 0) {
                    float up = 0.0f;
#pragma unroll
                    for (int w = 0; w < WK; ++w) up += partial[w][NMAT - 1][t][row];
                    a.out_a[at] = float_to_half_bits(clamped_swiglu(sum, up, a.limit));
                }
            } else {
                a.out_f32[at] = a.tok_weight[t] * sum;
            }
        }
    }
}

// From this many tokens on the activation rows are staged in LDS, where they fit beside the
// 16 KiB of partial sums (one or two tokens gain nothing from it: measured).
constexpr int kGemvXldsMinTokens = 4;
constexpr size_t kGemvXldsMaxBytes = 128 * 1024;

template <int NMAT, int TOK, int WK, int SG, bool HALF, bool XLDS>
static int launch_gemv_one(const GemvArgs& a, int blocks, size_t x_bytes, hipStream_t stream) {
    auto* kernel = a64_gemv_kernel<NMAT, TOK, WK, SG, HALF, XLDS>;
    if (XLDS) {
        // more dynamic LDS than the default limit has to be asked for, once per kernel and device
        static std::atomic<uint64_t> raised{0};
        int device = 0;
        AEON_HIP(hipGetDevice(&device));
        const uint64_t bit = 1ull << (device & 63);
        if (device >= 64 || (raised.load(std::memory_order_relaxed) & bit) == 0) {
            AEON_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize,
                                         static_cast<int>(kGemvXldsMaxBytes)));
            raised.fetch_or(bit, std::memory_order_relaxed);
        }
    }
    kernel<<<dim3(blocks), WK * 64, XLDS ? x_bytes : 0, stream>>>(a);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

template <int NMAT, int TOK, int SG, bool XLDS>
static int launch_gemv_wk_sg_x(const GemvArgs& a, int wk, size_t x_bytes, hipStream_t stream) {
    const int tiles = a.N / 16;
    if (wk >= 16 && tiles < 256 && TOK < 8) {
        return launch_gemv_one<NMAT, TOK, 16, SG, true, XLDS>(a, 2 * tiles, x_bytes, stream);
    } else if (wk >= 16) {
        return launch_gemv_one<NMAT, TOK, 16, SG, false, XLDS>(a, tiles, x_bytes, stream);
    } else if (wk >= 8) {
        return launch_gemv_one<NMAT, TOK, 8, SG, false, XLDS>(a, tiles, x_bytes, stream);
    }
    return launch_gemv_one<NMAT, TOK, 4, SG, false, XLDS>(a, tiles, x_bytes, stream);
}

template <int NMAT, int TOK, int SG>
static int launch_gemv_wk_sg(const GemvArgs& a, int wk, hipStream_t stream) {
    const size_t x_bytes = static_cast<size_t>(a.tokens) * a.groups * 256;
    if constexpr (TOK >= kGemvXldsMinTokens) {
        if (x_bytes <= kGemvXldsMaxBytes) return launch_gemv_wk_sg_x<NMAT, TOK, SG, true>(a, wk, x_bytes, stream);
    }
    return launch_gemv_wk_sg_x<NMAT, TOK, SG, false>(a, wk, x_bytes, stream);
}

template <int NMAT, int TOK>
static int launch_gemv_wk(const GemvArgs& a, int wk, hipStream_t stream) {
    return a.scales_per_group == 4 ? launch_gemv_wk_sg<NMAT, TOK, 4>(a, wk, stream)
                                   : launch_gemv_wk_sg<NMAT, TOK, 1>(a, wk, stream);
}

template <int NMAT>
static int launch_gemv(const GemvArgs& a, hipStream_t stream) {
    // Enough waves to cover 256 CUs a few times over: split K further when N is small.
    const int tiles = a.N / 16;
    int wk = 4;
    while (wk < 16 && tiles * wk < 2048 && a.groups >= 2 * wk) wk *= 2;
    if (a.tokens == 1) return launch_gemv_wk<NMAT, 1>(a, wk, stream);
    if (a.tokens == 2) return launch_gemv_wk<NMAT, 2>(a, wk, stream);
    if (a.tokens <= 4) return launch_gemv_wk<NMAT, 4>(a, wk, stream);
    return launch_gemv_wk<NMAT, 8>(a, wk, stream);
}

static int check_a64_shape(int N, int K, int scale_group, const char* who) {
    AEON_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && K % 128 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "%s: the wave64 packing needs N%%16==0 and K%%128==0 (N=%d K=%d)", who, N, K);
    AEON_REQUIRE(scale_group == 128 || scale_group == 32, AEON_ERR_INVALID_ARGUMENT,
                 "%s: scale_group must be 128 or 32, not %d", who, scale_group);
    return AEON_OK;
}

// ---------------------------------------------------------------------------------------------
// MFMA segment kernels
// ---------------------------------------------------------------------------------------------

// The matrix instruction is issued with the token rows as its first operand and the weight tile
// as its second: lane l supplies token l%16 / weight row l%16 and the 8-column chunk l/16 of a
// 32-column step (the two operands have the same lane pattern, so the packed tile needs no
// movement either way round) and ends up holding tokens 4*(l/16)..+3 of weight row l%16. A lane
// therefore needs the scales of one weight row only: one fp16 per 128 columns, or the row's four
// (one per 32-column step, 8 bytes side by side).
template <int SG>
struct RowScales;
template <>
struct RowScales<1> {
    uint16_t v;
    // `tile_scales` = the 16 rows' scales of one (tile, 128-column group), in memory or in LDS
    __device__ __forceinline__ void load(const AEON_GLOBAL uint16_t* tile_scales, int row) { v = tile_scales[row]; }
    __device__ __forceinline__ void load_lds(const uint16_t* tile_scales, int row) { v = tile_scales[row]; }
    __device__ __forceinline__ float get(int) const { return half_bits_to_float(v); }
};
template <>
struct RowScales<4> {
    u32x2_t v;
    __device__ __forceinline__ void load(const AEON_GLOBAL uint16_t* tile_scales, int row) {
        v = *reinterpret_cast<const AEON_GLOBAL u32x2_t*>(tile_scales + row * 4);
    }
    __device__ __forceinline__ void load_lds(const uint16_t* tile_scales, int row) {
        v = *reinterpret_cast<const u32x2_t*>(tile_scales + row * 4);
    }
    __device__ __forceinline__ float get(int st) const {
        const uint32_t w = v[st >> 1];
        return half_bits_to_float(static_cast<uint16_t>((st & 1) ? (w >> 16) : (w & 0xFFFFu)));
    }
};

// acc (tokens 4*(l/16)..+3 of weight row l%16) += the scaled product of one weight tile with the
// 16 token rows over one 128-column group. One scale per row: the four steps chain into one
// result, scaled once. Four per row: every step is a product of its own, scaled by the step's
// scale. In fp32 either way, so the dequantisation stays exact.
template <int SG>
__device__ __forceinline__ void mfma_scaled(float4_t& acc, const u32x4_t& wq, const half8_t xf[4],
                                            const RowScales<SG>& sc) {
    const float4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
    if constexpr (SG == 1) {
        float4_t t = zero;
#pragma unroll
        for (int st = 0; st < 4; ++st) t = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[st], unpack8_vec(wq[st]), t, 0, 0, 0);
        acc += sc.get(0) * t;
    } else {
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const float4_t t = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[st], unpack8_vec(wq[st]), zero, 0, 0, 0);
            acc += sc.get(st) * t;
        }
    }
}

// Stores of a lane's four results (tokens 4*chunk..+3 of one output row): the fp16 hidden value
// of the gate/up pair, or the weighted fp32 contribution (and, for a single slot, the reduce).
__device__ __forceinline__ void store_hidden(const SegGateUpArgs& gu, const float4_t& gate, const float4_t& up,
                                             int first, int token0, int count, int row) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        if (token0 + v < count) {
            gu.hidden[static_cast<size_t>(first + token0 + v) * gu.I + row] =
                float_to_half_bits(clamped_swiglu(gate[v], up[v], gu.limit));
        }
    }
}

__device__ __forceinline__ void store_contrib(const SegDownArgs& dn, const float4_t& acc, int first, int token0,
                                              int count, int row, bool unit_weight) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        if (token0 + v >= count) continue;
        const int position = first + token0 + v;
        const float w = unit_weight ? 1.0f : dn.weight[position];
        const float value = w * acc[v];
        const size_t out_row = dn.out_row != nullptr ? dn.out_row[position] : position;
        dn.contrib[out_row * dn.H + row] = value;
        if (dn.fused_out != nullptr) {
            // the reduce over a single slot, with its two roundings kept apart (no fused
            // multiply-add): the stored fp32 contribution, then one fp16 rounding of the sum
            const size_t at = static_cast<size_t>(position) * dn.H + row;
            const float start = dn.fused_initial != nullptr ? half_bits_to_float(dn.fused_initial[at]) : 0.0f;
            float product = value;
            asm volatile("" : "+v"(product));   // keeps the multiply out of an fma with the add
            dn.fused_out[at] = float_to_half_bits(start + product);
        }
    }
}

// One workgroup = (R consecutive 16-row tiles, one segment). The activation fragments of a
// 128-column group are loaded once and used by all R tiles (and both matrices of gate/up).
template <bool GATE_UP, int R, int WK, int D, int SG>
__global__ __launch_bounds__(WK * 64) void a64_seg_kernel(SegGateUpArgs gu, SegDownArgs dn) {
    constexpr int NM = GATE_UP ? 2 : 1;
    const SegmentList& seg = GATE_UP ? gu.seg : dn.seg;
    const int s = blockIdx.y;
    int first = 0;
    int count = GATE_UP ? gu.direct_count : dn.direct_count;
    aeon_a64_expert e = GATE_UP ? gu.direct_expert : dn.direct_expert;
    const bool slot_mode = seg.total == nullptr && seg.slot_experts > 0;
    if (seg.total != nullptr) {
        if (s >= *seg.total) return;
        first = seg.first[s];
        count = seg.count[s];
        e = (GATE_UP ? gu.experts : dn.experts)[seg.expert[s]];
    } else if (slot_mode) {
        const int id = s == seg.slot_shared ? seg.slot_experts : seg.expert[s];
        if (id < 0 || (id >= seg.slot_experts && s != seg.slot_shared)) return;
        first = s;
        count = s == seg.slot_shared ? seg.slot_tokens : 1;
        e = (GATE_UP ? gu.experts : dn.experts)[id];
    }

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;
    const int chunk = lane >> 4;
    const int tile0 = blockIdx.x * R;

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

    // A padded token row repeats the segment's last live position: always a valid row, and
    // its products land in results the stores below never write.
    const int position = first + (n < count ? n : count - 1);
    const AEON_GLOBAL uint16_t* xrow;
    if (GATE_UP) {
        const long row = slot_mode ? (s == seg.slot_shared ? position - first : s / seg.slot_top_k)
                         : gu.row_index != nullptr ? gu.row_index[position] : position;
        xrow = as_global<uint16_t>(gu.x) + row * gu.x_stride + chunk * 8;
    } else {
        xrow = as_global<uint16_t>(dn.hidden) + static_cast<size_t>(position) * dn.I + chunk * 8;
    }

    float4_t acc[NM][R];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // Software pipeline over the 128-column groups this wave owns (g = wave, wave+WK, ...):
    // D groups of weights, scales and activation fragments are in flight in registers; a
    // buffer is refilled for the group D steps ahead as soon as its MFMAs have been issued, so
    // every wave keeps D*NM*R KiB of HBM reads outstanding while it computes.
    u32x4_t wq[D][NM][R];
    RowScales<SG> sc[D][NM][R];
    half8_t xf[D][4];
    auto load_group = [&](int d, int g) {
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const size_t t = static_cast<size_t>(tile0 + r) * groups + g;
                wq[d][m][r] = stream_load(&pm[m][t * 64 + lane]);
                sc[d][m][r].load(sm[m] + t * (16 * SG), n);
            }
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            xf[d][st] = *reinterpret_cast<const AEON_GLOBAL half8_t*>(xrow + g * 128 + st * 32);
        }
    };
    // Group j of this wave is column group wave + j*WK; it owns `mine` of them. The loop is cut
    // in three so that the steady state has no conditional loads: a branch around a prefetch
    // makes the compiler wait for every outstanding load at the loop head (the two paths leave
    // different numbers in flight), which would serialise the pipeline.
    const int mine = (groups - wave + WK - 1) / WK;
    auto compute = [&](int d) {
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                mfma_scaled<SG>(acc[m][r], wq[d][m][r], xf[d], sc[d][m][r]);
            }
    };
#pragma unroll
    for (int d = 0; d < D; ++d) {
        // a short wave reloads its last group, unused; a wave with no group at all (fewer groups
        // than waves) reloads the matrix's last group so that every address stays inside it
        const int j = d < mine ? d : mine - 1;
        load_group(d, mine > 0 ? wave + j * WK : groups - 1);
    }
    int j0 = 0;
    for (; j0 + 2 * D <= mine; j0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            compute(d);
            load_group(d, wave + (j0 + d + D) * WK);
        }
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
        if (j0 + d < mine) {
            compute(d);
            if (j0 + d + D < mine) load_group(d, wave + (j0 + d + D) * WK);
        }
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
        if (j0 + D + d < mine) compute(d);
    }

    if (WK > 1) {
        __shared__ float4_t partial[WK][NM][R][64];
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) partial[wave][m][r][lane] = acc[m][r];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int w = 1; w < WK; ++w)
#pragma unroll
            for (int m = 0; m < NM; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r) acc[m][r] += partial[w][m][r][lane];
    }

    // the lane holds tokens 4*chunk..+3 of output row (tile, n)
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = (tile0 + r) * 16 + n;
        if (GATE_UP) {
            store_hidden(gu, acc[0][r], acc[NM - 1][r], first, chunk * 4, count, row);
        } else {
            store_contrib(dn, acc[0][r], first, chunk * 4, count, row, slot_mode && s == seg.slot_shared);
        }
    }
}

// The wide form for steps with many live segments: four waves per workgroup, each with its own
// R tiles and no K split. What limits the narrow form is the number of vector-memory
// instructions per weight byte (each wave issues 4 activation and NM*R scale loads beside its
// NM*R weight loads for every 128 columns), so this form takes both off that pipe:
//   * the scales of a wave's tiles (groups x 32 bytes each, contiguous) are copied into LDS
//     once, before the loop, and read back with one ds_read_b64 per tile and group;
//   * the four waves share one copy of the segment's activation fragments: per group every
//     wave fetches one fragment (16 tokens x 32 columns) and all four read them from LDS.
// Per wave and group that leaves NM*R weight loads + 1 activation load.
// A segment of the wide form holds up to kWideSegTokens positions of one expert: MT = 1 or 2
// token tiles of 16. Both tiles ride on one pass over the weights -- a word is unpacked once and
// multiplied into each tile -- so an expert that drew 17..32 tokens (or the always-on expert's
// long list) streams its weights once per 32 positions instead of once per 16.
static_assert(kWideSegTokens == kWideMaxTiles * kSegTokens, "segment length of the wide form");

// LDS of one wide-form workgroup: the activation ring (static) plus the scales of its four
// waves' tiles over the whole of K (dynamic).
constexpr size_t kWideActivationLdsBytes = 2 * kWideMaxTiles * 4 * 64 * 16;
size_t seg_wide_scale_lds_bytes(bool gate_up, int row_tiles, int k_dim, int scales_per_group) {
    return static_cast<size_t>(4) * (gate_up ? 2 : 1) * row_tiles * (k_dim / 128) * 32 * scales_per_group;
}
bool seg_wide_fits(bool gate_up, int row_tiles, int k_dim, int scales_per_group) {
    return kWideActivationLdsBytes + seg_wide_scale_lds_bytes(gate_up, row_tiles, k_dim, scales_per_group) <= 65536;
}

template <bool GATE_UP, int R, int D, int MT, int SG, bool SL>
__device__ __forceinline__ void seg_wide_item(const SegGateUpArgs& gu, const SegDownArgs& dn, int s,
                                              int row_block, half8_t* xs, u32x4_t* scale_lds) {
    constexpr int NM = GATE_UP ? 2 : 1;
    const SegmentList& seg = GATE_UP ? gu.seg : dn.seg;
    // slot mode (single token, no segment list): segment s is slot s of the caller's ids
    const bool slot_mode = seg.total == nullptr;
    const int first = slot_mode ? s : seg.first[s];
    const int count = slot_mode ? (s == seg.slot_shared ? seg.slot_tokens : 1) : seg.count[s];
    const int id = slot_mode && s == seg.slot_shared ? seg.slot_experts : seg.expert[s];
    const aeon_a64_expert e = (GATE_UP ? gu.experts : dn.experts)[id];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;
    const int chunk = lane >> 4;
    const int tile0 = (row_block * 4 + wave) * R;

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

    // this wave's share of a group's activations: MFMA step `wave` (columns 32*wave..+31) of
    // every token tile; a padded token column repeats the segment's last live position
    const AEON_GLOBAL uint16_t* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int token = mt * kSegTokens + n;
        const int position = first + (token < count ? token : count - 1);
        if (GATE_UP) {
            const long row = slot_mode ? (s == seg.slot_shared ? position - first : s / seg.slot_top_k)
                             : gu.row_index != nullptr ? gu.row_index[position] : position;
            xrow[mt] = as_global<uint16_t>(gu.x) + row * gu.x_stride + chunk * 8 + wave * 32;
        } else {
            xrow[mt] = as_global<uint16_t>(dn.hidden) + static_cast<size_t>(position) * dn.I + chunk * 8 +
                       wave * 32;
        }
    }

    // SL: the scales of this wave's tiles over all of K are copied to LDS once. Otherwise (four
    // scales per group over a K too long for that) they ride in the register ring with the
    // weights, fetched from memory a group at a time.
    const int tile_u4 = groups * 2 * SG;    // 32 (SG 1) or 128 (SG 4) bytes of scales per group
    u32x4_t* my_scales = scale_lds + static_cast<size_t>(wave) * NM * R * tile_u4;
    if constexpr (SL) {
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const AEON_GLOBAL u32x4_t* src = reinterpret_cast<const AEON_GLOBAL u32x4_t*>(
                    sm[m] + static_cast<size_t>(tile0 + r) * groups * (16 * SG));
                for (int i = lane; i < tile_u4; i += 64) my_scales[(m * R + r) * tile_u4 + i] = src[i];
            }
    }

    float4_t acc[NM][R][MT];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[m][r][mt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    u32x4_t wq[D][NM][R];
    RowScales<SG> ring_scales[SL ? 1 : D][NM][R];
    auto load_group = [&](int d, int g) {
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const size_t t = static_cast<size_t>(tile0 + r) * groups + g;
                wq[d][m][r] = stream_load(&pm[m][t * 64 + lane]);
                if constexpr (!SL) ring_scales[d][m][r].load(sm[m] + t * (16 * SG), n);
            }
    };
    // LDS image of a group's activations: [buffer][token tile][MFMA step][lane] x 16 bytes
    auto slot = [&](int buffer, int mt, int st) { return xs + ((buffer * kWideMaxTiles + mt) * 4 + st) * 64 + lane; };
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *slot(0, mt, wave) = *reinterpret_cast<const AEON_GLOBAL half8_t*>(xrow[mt]);
    // This wave's activation fragments of the next D groups wait in registers, fetched as far
    // ahead as the weights: loads complete in issue order, so a fragment fetched only one group
    // ahead would force every weight request older than it to have landed by the end of each
    // step and cut the weight pipeline to a single step whatever D is.
    half8_t xr[D][MT];
    auto load_x = [&](int g, int mt) {
        return *reinterpret_cast<const AEON_GLOBAL half8_t*>(xrow[mt] + (g < groups ? g : groups - 1) * 128);
    };
    // The requests of the first D groups go out in the order the loop keeps them in (weights
    // of group d, then the fragment of group d+1): the compiler's wait counts are static, so a
    // different order here would be the one every pass through the loop has to wait for.
#pragma unroll
    for (int d = 0; d < D; ++d) {
        load_group(d, d < groups ? d : groups - 1);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xr[(d + 1) % D][mt] = load_x(d + 1, mt);
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();

    // step g: read all four fragments of group g from LDS, multiply, publish this wave's
    // fragment of group g+1 (fetched D steps ago) into the other LDS buffer, then request group
    // g+D's weights and group g+1+D's fragment. One barrier per group: buffer (g+1)&1 was last
    // read in step g-1, before that step's barrier.
    const uint16_t* scale_halves = reinterpret_cast<const uint16_t*>(my_scales);
    auto step = [&](int d, int g, bool refill) {
        half8_t xf[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int st = 0; st < 4; ++st) xf[mt][st] = *slot(g & 1, mt, st);
        // this lane's weight row of each tile: its scale(s) of the group, 2 or 8 bytes from LDS
        RowScales<SG> sc[NM][R];
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if constexpr (SL) sc[m][r].load_lds(scale_halves + ((m * R + r) * tile_u4 + g * 2 * SG) * 8, n);
                else sc[m][r] = ring_scales[d][m][r];
            }
        // The K steps run outermost and the wave's tiles innermost, so that consecutive matrix
        // instructions belong to different accumulators: a chain of dependent ones would hold
        // the SIMD for the latency of each.
        const float4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
        float4_t t[NM][R][MT];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
#pragma unroll
            for (int m = 0; m < NM; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const half8_t a = unpack8_vec(wq[d][m][r][st]);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        t[m][r][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            xf[mt][st], a, (SG == 4 || st == 0) ? zero : t[m][r][mt], 0, 0, 0);
                }
            if (SG == 4 || st == 3) {
                // one scale per row: the four steps have chained into t; four per row: every
                // step's product takes the step's scale. fp32 either way.
#pragma unroll
                for (int m = 0; m < NM; ++m)
#pragma unroll
                    for (int r = 0; r < R; ++r)
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) acc[m][r][mt] += sc[m][r].get(SG == 4 ? st : 0) * t[m][r][mt];
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) *slot((g + 1) & 1, mt, wave) = xr[(d + 1) % D][mt];
        if (refill) {
            load_group(d, g + D);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) xr[(d + 1) % D][mt] = load_x(g + 1 + D, mt);
        }
        __syncthreads();
    };
    int g0 = 0;
    for (; g0 + 2 * D <= groups; g0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) step(d, g0 + d, true);
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
        if (g0 + d < groups) step(d, g0 + d, g0 + d + D < groups);
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
        if (g0 + D + d < groups) step(d, g0 + D + d, false);
    }

    // the lane holds tokens 16*mt + 4*chunk..+3 of output row (tile, n)
    if (GATE_UP) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                store_hidden(gu, acc[0][r][mt], acc[NM - 1][r][mt], first, mt * kSegTokens + chunk * 4, count,
                             (tile0 + r) * 16 + n);
            }
        return;
    }
    // Down: the fp32 contributions are the launch's largest output, and four tokens of one row
    // per lane would be four 4-byte stores each behind its own index and weight load. Every
    // 16 x 16 result tile is turned round through this wave's quarter of the (now idle)
    // activation buffer, so that a lane holds four consecutive rows of one token: one index,
    // one weight, one 16-byte store.
    float* turn = reinterpret_cast<float*>(xs) + wave * 1024;
    const bool unit_weight = slot_mode && s == seg.slot_shared;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int token = mt * kSegTokens + n;
        const bool live = token < count;
        const int position = first + (live ? token : 0);
        const float w = unit_weight ? 1.0f : dn.weight[position];
        const size_t out_row = dn.out_row != nullptr ? dn.out_row[position] : position;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float* tile = turn + ((mt * R + r) & 3) * 256;
#pragma unroll
            for (int v = 0; v < 4; ++v) tile[(chunk * 4 + v) * 16 + n] = acc[0][r][mt][v];
            __builtin_amdgcn_wave_barrier();
            const float4_t rows = *reinterpret_cast<const float4_t*>(tile + n * 16 + chunk * 4);
            if (live) {
                const float4_t value = {w * rows[0], w * rows[1], w * rows[2], w * rows[3]};
                *reinterpret_cast<float4_t*>(dn.contrib + out_row * dn.H + (tile0 + r) * 16 + chunk * 4) = value;
            }
        }
    }
}

// Four waves per SIMD (128 registers a wave) is what hides the weight stream's latency for the
// common one-tile segment; the rarer two-tile path is kept inside that budget by a shallower
// prefetch ring rather than allowed to halve everyone's occupancy.
template <bool GATE_UP, int R, int D, int SG, bool SL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void a64_seg_wide_kernel(
    SegGateUpArgs gu, SegDownArgs dn) {
    __shared__ half8_t xs[2 * kWideMaxTiles * 4 * 64];
    extern __shared__ u32x4_t scale_lds[];  // [wave][m][r][groups * 2] 16-byte units
    const SegmentList& seg = GATE_UP ? gu.seg : dn.seg;
    const int s = blockIdx.y;  // the list is ordered costliest first
    if (seg.total == nullptr) {
        // slot mode: segment s = draw s of a handful of tokens; a dropped id ends the workgroup
        if (s != seg.slot_shared) {
            const int id = seg.expert[s];
            if (id < 0 || id >= seg.slot_experts) return;
        }
        seg_wide_item<GATE_UP, R, D, 1, SG, SL>(gu, dn, s, blockIdx.x, xs, scale_lds);
        return;
    }
    if (s >= *seg.total) return;
    if (seg.count[s] > kSegTokens) {
        seg_wide_item<GATE_UP, R, (SG == 4 ? 1 : D > 2 ? 2 : D), 2, SG, SL>(gu, dn, s, blockIdx.x, xs, scale_lds);
    } else {
        seg_wide_item<GATE_UP, R, D, 1, SG, SL>(gu, dn, s, blockIdx.x, xs, scale_lds);
    }
}

template <bool GATE_UP, int R, int D, int SG>
static void launch_seg_rds(const SegGateUpArgs& gu, const SegDownArgs& dn, int tiles, int capacity,
                           int k_split, hipStream_t stream) {
    const dim3 grid(tiles / R, capacity);
    if (k_split == 0) {
        const size_t scale_bytes = seg_wide_scale_lds_bytes(GATE_UP, R, GATE_UP ? gu.H : dn.I, SG);
        const dim3 wide(tiles / (4 * R), capacity);
        if constexpr (SG == 4) {
            // Four scales per group: over a long K they do not fit the workgroup's LDS and come
            // with the weight ring instead (two registers per tile and group in flight). The
            // gate/up launch takes that form at every K: its LDS copy (32 KB at K 4096) would
            // cost a workgroup per CU, and the ring form measured 1-3 % faster there.
            if (GATE_UP || !seg_wide_fits(GATE_UP, R, GATE_UP ? gu.H : dn.I, SG)) {
                a64_seg_wide_kernel<GATE_UP, R, (D > 2 ? 2 : D), SG, false><<<wide, 256, 0, stream>>>(gu, dn);
                return;
            }
        }
        a64_seg_wide_kernel<GATE_UP, R, D, SG, true><<<wide, 256, scale_bytes, stream>>>(gu, dn);
    } else if (k_split >= 4 && (GATE_UP ? gu.H : dn.I) >= 4 * 128) {
        a64_seg_kernel<GATE_UP, R, 4, D, SG><<<grid, 256, 0, stream>>>(gu, dn);
    } else if (k_split >= 2 && (GATE_UP ? gu.H : dn.I) >= 2 * 128) {
        a64_seg_kernel<GATE_UP, R, 2, D, SG><<<grid, 128, 0, stream>>>(gu, dn);
    } else {
        a64_seg_kernel<GATE_UP, R, 1, D, SG><<<grid, 64, 0, stream>>>(gu, dn);
    }
}

template <bool GATE_UP, int R, int D>
static void launch_seg_rd(const SegGateUpArgs& gu, const SegDownArgs& dn, int tiles, int capacity,
                          int k_split, hipStream_t stream) {
    if ((GATE_UP ? gu.scales_per_group : dn.scales_per_group) == 4) {
        launch_seg_rds<GATE_UP, R, D, 4>(gu, dn, tiles, capacity, k_split, stream);
    } else {
        launch_seg_rds<GATE_UP, R, D, 1>(gu, dn, tiles, capacity, k_split, stream);
    }
}

template <bool GATE_UP, int R>
static void launch_seg_r(const SegGateUpArgs& gu, const SegDownArgs& dn, int tiles, int capacity,
                         int k_split, int depth, hipStream_t stream) {
    if (depth >= 4) {
        launch_seg_rd<GATE_UP, R, 4>(gu, dn, tiles, capacity, k_split, stream);
    } else if (depth == 3) {
        launch_seg_rd<GATE_UP, R, 3>(gu, dn, tiles, capacity, k_split, stream);
    } else if (depth == 2) {
        launch_seg_rd<GATE_UP, R, 2>(gu, dn, tiles, capacity, k_split, stream);
    } else {
        launch_seg_rd<GATE_UP, R, 1>(gu, dn, tiles, capacity, k_split, stream);
    }
}

template <bool GATE_UP>
static void launch_seg(const SegGateUpArgs& gu, const SegDownArgs& dn, int tiles, int capacity,
                       int k_split, int row_tiles, int depth, hipStream_t stream) {
    const SegmentList& list = GATE_UP ? gu.seg : dn.seg;
    const bool direct = list.total == nullptr && list.slot_experts == 0;
    if (k_split == 0 && (direct || tiles % (4 * (row_tiles >= 2 ? 2 : 1)) != 0)) {
        k_split = 1;  // the wide form needs a segment list and whole workgroups of tiles
    }
    if (k_split == 0 && row_tiles >= 2 && tiles % 2 == 0 &&
        !seg_wide_fits(GATE_UP, 2, GATE_UP ? gu.H : dn.I, GATE_UP ? gu.scales_per_group : dn.scales_per_group)) {
        row_tiles = 1;  // two row tiles per wave would not fit their scales into LDS
    }
    // Two row tiles per wave is the most the 128-register budget of the wide form carries.
    if (row_tiles >= 2 && tiles % 2 == 0) {
        launch_seg_r<GATE_UP, 2>(gu, dn, tiles, capacity, k_split, depth, stream);
    } else {
        launch_seg_r<GATE_UP, 1>(gu, dn, tiles, capacity, k_split, depth, stream);
    }
}

int launch_seg_gate_up(const SegGateUpArgs& a, int k_split, int row_tiles, int depth, hipStream_t stream) {
    AEON_REQUIRE(a.H % 128 == 0 && a.I % 16 == 0 && a.x_stride % 8 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "gate/up segments: need H%%128==0, I%%16==0 and an activation pitch that keeps "
                 "rows 16-byte aligned (H=%d I=%d pitch=%ld)", a.H, a.I, a.x_stride);
    AEON_REQUIRE(a.scales_per_group == 1 || a.scales_per_group == 4, AEON_ERR_INVALID_ARGUMENT,
                 "gate/up segments: %d scales per 128 columns (1 or 4)", a.scales_per_group);
    AEON_REQUIRE(k_split != 0 || a.scales_per_group == 4 || seg_wide_fits(true, 1, a.H, a.scales_per_group),
                 AEON_ERR_INVALID_ARGUMENT,
                 "gate/up segments: the scales of %d columns do not fit the wide form's LDS", a.H);
    if (a.seg.capacity <= 0) return AEON_OK;
    launch_seg<true>(a, SegDownArgs{}, a.I / 16, a.seg.capacity, k_split, row_tiles, depth, stream);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

int launch_seg_down(const SegDownArgs& a, int k_split, int row_tiles, int depth, hipStream_t stream) {
    AEON_REQUIRE(a.I % 128 == 0 && a.H % 16 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "down segments: need I%%128==0 and H%%16==0 (H=%d I=%d)", a.H, a.I);
    AEON_REQUIRE(a.scales_per_group == 1 || a.scales_per_group == 4, AEON_ERR_INVALID_ARGUMENT,
                 "down segments: %d scales per 128 columns (1 or 4)", a.scales_per_group);
    AEON_REQUIRE(k_split != 0 || a.scales_per_group == 4 || seg_wide_fits(false, 1, a.I, a.scales_per_group),
                 AEON_ERR_INVALID_ARGUMENT,
                 "down segments: the scales of %d columns do not fit the wide form's LDS", a.I);
    if (a.seg.capacity <= 0) return AEON_OK;
    launch_seg<false>(SegGateUpArgs{}, a, a.H / 16, a.seg.capacity, k_split, row_tiles, depth, stream);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

// ---------------------------------------------------------------------------------------------
// Fixed-order reduce over a token's slots
// ---------------------------------------------------------------------------------------------

// Four columns per thread (hidden is a multiple of 128): 16-byte loads of the fp32 contributions.
// `ids` (may be null) are the token's expert choices: a slot whose id is outside [0, experts) was
// dropped by the permutation, no kernel wrote its contribution row, and it is skipped here.
__global__ __launch_bounds__(256) void token_reduce_kernel(
    const float* __restrict__ contrib, int slots, int shared_base, const uint16_t* initial,
    long initial_stride, uint16_t* out, long out_stride, int hidden,
    const int32_t* __restrict__ ids, int experts) {
    const int t = blockIdx.y;
    const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= hidden) return;
    float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (shared_base >= 0) {
        // The shared expert enters as an fp16 value, as it does when a separate pass has
        // stored it into the token's accumulator first.
        const float4_t v = *reinterpret_cast<const float4_t*>(
            contrib + static_cast<size_t>(shared_base + t) * hidden + i);
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] = half_bits_to_float(float_to_half_bits(v[q]));
    } else if (initial != nullptr) {
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] = half_bits_to_float(initial[t * initial_stride + i + q]);
    }
    const float* c = contrib + static_cast<size_t>(t) * slots * hidden + i;
    // The contributions are read once (streaming loads). Eight slots at a time: their rows are requested first, whether they count or not (a
    // dropped slot's row is stale but addressable), so that no request waits for an id; the ids
    // only decide which of the loaded rows are added, in slot order.
    for (int s0 = 0; s0 < slots; s0 += 8) {
        float4_t v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int s = s0 + j < slots ? s0 + j : slots - 1;
            v[j] = stream_load(reinterpret_cast<const float4_t*>(c + static_cast<size_t>(s) * hidden));
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (s0 + j >= slots) break;
            if (ids != nullptr) {
                const int e = ids[t * slots + s0 + j];
                if (e < 0 || e >= experts) continue;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] += v[j][q];
        }
    }
    uint16_t* o = out + t * out_stride + i;
    if ((reinterpret_cast<uintptr_t>(o) & 7) == 0) {
        uint2 packed;
        packed.x = float_to_half_bits(acc[0]) | (static_cast<uint32_t>(float_to_half_bits(acc[1])) << 16);
        packed.y = float_to_half_bits(acc[2]) | (static_cast<uint32_t>(float_to_half_bits(acc[3])) << 16);
        *reinterpret_cast<uint2*>(o) = packed;
    } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = float_to_half_bits(acc[q]);
    }
}

int launch_token_reduce(const float* contrib, int tokens, int slots, int shared_base,
                        const uint16_t* initial, long initial_stride, uint16_t* out,
                        long out_stride, int hidden, hipStream_t stream, const int32_t* ids,
                        int experts) {
    if (tokens <= 0) return AEON_OK;
    AEON_REQUIRE(hidden % 4 == 0, AEON_ERR_INVALID_ARGUMENT, "token reduce: hidden %d is not a multiple of 4", hidden);
    token_reduce_kernel<<<dim3((hidden / 4 + 255) / 256, tokens), 256, 0, stream>>>(
        contrib, slots, shared_base, initial, initial_stride, out, out_stride, hidden, ids, experts);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

// token_reduce_kernel followed, in the same pass, by hc_post_kernel and (optionally) the next
// layer's hc_pre_combine_kernel: every value crosses a kernel boundary of the unfused sequence as
// fp16, so it is rounded to fp16 at the same three points here (the reduced row, the four
// expanded streams, the next layer's input) and the result is the unfused sequence's, bit for bit.
__global__ __launch_bounds__(256) void token_reduce_hc_post_kernel(
    const float* __restrict__ contrib, int slots, int shared_base, const uint16_t* initial,
    long initial_stride, uint16_t* out, long out_stride, int hidden,
    const int32_t* __restrict__ ids, int experts, aeon_hc_post_args hc) {
    const int t = blockIdx.y;
    const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i >= hidden) return;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (shared_base >= 0) {
        const float* sh = contrib + static_cast<size_t>(shared_base + t) * hidden + i;
        const float4_t a = *reinterpret_cast<const float4_t*>(sh);
        const float4_t b = *reinterpret_cast<const float4_t*>(sh + 4);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            acc[q] = half_bits_to_float(float_to_half_bits(a[q]));
            acc[4 + q] = half_bits_to_float(float_to_half_bits(b[q]));
        }
    } else if (initial != nullptr) {
        const half8_t v = *reinterpret_cast<const half8_t*>(initial + t * initial_stride + i);
#pragma unroll
        for (int q = 0; q < 8; ++q) acc[q] = static_cast<float>(v[q]);
    }
    const float* c = contrib + static_cast<size_t>(t) * slots * hidden + i;
    for (int s0 = 0; s0 < slots; s0 += 4) {
        float4_t v[4][2];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int s = s0 + j < slots ? s0 + j : slots - 1;
            const float4_t* row = reinterpret_cast<const float4_t*>(c + static_cast<size_t>(s) * hidden);
            v[j][0] = stream_load(row);
            v[j][1] = stream_load(row + 1);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (s0 + j >= slots) break;
            if (ids != nullptr) {
                const int e = ids[t * slots + s0 + j];
                if (e < 0 || e >= experts) continue;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                acc[q] += v[j][0][q];
                acc[4 + q] += v[j][1][q];
            }
        }
    }
    half8_t y;
#pragma unroll
    for (int q = 0; q < 8; ++q) y[q] = static_cast<half_t>(acc[q]);
    *reinterpret_cast<half8_t*>(out + t * out_stride + i) = y;

    const float* pm = hc.d_post_mix + static_cast<size_t>(t) * (hc.mix_per_token ? 4 : 0);
    const float* cm = hc.d_comb_mix + static_cast<size_t>(t) * (hc.mix_per_token ? 16 : 0);
    const uint16_t* res_in = static_cast<const uint16_t*>(hc.d_residual_in);
    uint16_t* res_out = static_cast<uint16_t*>(hc.d_residual_out);
    half8_t r[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        r[k] = *reinterpret_cast<const half8_t*>(res_in + t * hc.token_stride + k * hc.stream_stride + i);
    }
    float next[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const float* pre = hc.d_next_pre_mix != nullptr
                           ? hc.d_next_pre_mix + static_cast<size_t>(t) * hc.next_pre_token_stride
                           : nullptr;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        half8_t o;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            float v = pm[j] * static_cast<float>(y[q]);
#pragma unroll
            for (int k = 0; k < 4; ++k) v += cm[k * 4 + j] * static_cast<float>(r[k][q]);
            o[q] = static_cast<half_t>(v);
        }
        *reinterpret_cast<half8_t*>(res_out + t * hc.token_stride + j * hc.stream_stride + i) = o;
        if (pre != nullptr) {
            const float pj = pre[j];
#pragma unroll
            for (int q = 0; q < 8; ++q) next[q] += pj * static_cast<float>(o[q]);
        }
    }
    if (pre != nullptr) {
        half8_t x;
#pragma unroll
        for (int q = 0; q < 8; ++q) x[q] = static_cast<half_t>(next[q]);
        *reinterpret_cast<half8_t*>(static_cast<uint16_t*>(hc.d_next_layer_input) +
                                    t * hc.next_input_stride + i) = x;
    }
}

int launch_token_reduce_hc_post(const float* contrib, int tokens, int slots, int shared_base,
                                const uint16_t* initial, long initial_stride, uint16_t* out,
                                long out_stride, int hidden, const aeon_hc_post_args& hc,
                                hipStream_t stream, const int32_t* ids, int experts) {
    if (tokens <= 0) return AEON_OK;
    token_reduce_hc_post_kernel<<<dim3((hidden / 8 + 255) / 256, tokens), 256, 0, stream>>>(
        contrib, slots, shared_base, initial, initial_stride, out, out_stride, hidden, ids, experts, hc);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_moe_accumulate_fixed_order_tokens(const float* d_contrib, int tokens, int slots,
                                                      void* d_out, int out_stride, int hidden,
                                                      void* stream) {
    const char* who = "aeon_moe_accumulate_fixed_order_tokens";
    AEON_REQUIRE(d_contrib && d_out, AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && slots > 0 && hidden > 0 && hidden % 4 == 0 && out_stride >= hidden,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad shape (tokens=%d slots=%d hidden=%d pitch=%d)",
                 who, tokens, slots, hidden, out_stride);
    return launch_token_reduce(d_contrib, tokens, slots, -1, static_cast<const uint16_t*>(d_out),
                               out_stride, static_cast<uint16_t*>(d_out), out_stride, hidden,
                               as_stream(stream));
}

extern "C" int aeon_a64_gemv(const void* d_x, int x_stride, const void* d_packed,
                             const void* d_scale, int scale_group, void* d_out, int out_stride,
                             int tokens, int N, int K, void* stream) {
    const char* who = "aeon_a64_gemv";
    AEON_REQUIRE(d_x && d_packed && d_scale && d_out, AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    if (int rc = check_a64_shape(N, K, scale_group, who)) return rc;
    AEON_REQUIRE(tokens >= 1 && tokens <= 8, AEON_ERR_INVALID_ARGUMENT,
                 "%s: tokens=%d outside 1..8", who, tokens);
    AEON_REQUIRE(x_stride >= K && x_stride % 8 == 0 && out_stride >= N, AEON_ERR_INVALID_ARGUMENT,
                 "%s: bad row pitch (x_stride=%d out_stride=%d)", who, x_stride, out_stride);
    GemvArgs a{};
    a.scales_per_group = scale_group == 32 ? 4 : 1;
    a.x = static_cast<const uint16_t*>(d_x);
    a.x_stride = x_stride;
    a.pa = static_cast<const uint4*>(d_packed);
    a.sa = static_cast<const uint16_t*>(d_scale);
    a.out_a = static_cast<uint16_t*>(d_out);
    a.out_stride = out_stride;
    a.tokens = tokens;
    a.N = N;
    a.groups = K / 128;
    return launch_gemv<1>(a, as_stream(stream));
}

extern "C" int aeon_a64_dual_gemv(const void* d_x, int x_stride, const void* d_packed_a,
                                  const void* d_scale_a, const void* d_packed_b,
                                  const void* d_scale_b, int scale_group, void* d_out_a,
                                  void* d_out_b, int out_stride, int tokens, int N, int K,
                                  void* stream) {
    const char* who = "aeon_a64_dual_gemv";
    AEON_REQUIRE(d_x && d_packed_a && d_scale_a && d_packed_b && d_scale_b && d_out_a && d_out_b,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    if (int rc = check_a64_shape(N, K, scale_group, who)) return rc;
    AEON_REQUIRE(tokens >= 1 && tokens <= 8, AEON_ERR_INVALID_ARGUMENT,
                 "%s: tokens=%d outside 1..8", who, tokens);
    AEON_REQUIRE(x_stride >= K && x_stride % 8 == 0 && out_stride >= N, AEON_ERR_INVALID_ARGUMENT,
                 "%s: bad row pitch (x_stride=%d out_stride=%d)", who, x_stride, out_stride);
    GemvArgs a{};
    a.scales_per_group = scale_group == 32 ? 4 : 1;
    a.x = static_cast<const uint16_t*>(d_x);
    a.x_stride = x_stride;
    a.pa = static_cast<const uint4*>(d_packed_a);
    a.sa = static_cast<const uint16_t*>(d_scale_a);
    a.pb = static_cast<const uint4*>(d_packed_b);
    a.sb = static_cast<const uint16_t*>(d_scale_b);
    a.out_a = static_cast<uint16_t*>(d_out_a);
    a.out_b = static_cast<uint16_t*>(d_out_b);
    a.out_stride = out_stride;
    a.tokens = tokens;
    a.N = N;
    a.groups = K / 128;
    return launch_gemv<2>(a, as_stream(stream));
}

extern "C" int aeon_a64_expert_decode(const void* d_x, int tokens, const aeon_a64_expert* expert,
                                      int scale_group, const float* d_route_weights, void* d_hidden,
                                      float* d_contrib, const void* d_shared, void* d_out, int H,
                                      int I, float swiglu_limit, int use_mfma, void* stream) {
    const char* who = "aeon_a64_expert_decode";
    AEON_REQUIRE(d_x && expert && d_route_weights && d_hidden && d_contrib && d_out,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(expert->w1_packed && expert->w1_scale && expert->w3_packed && expert->w3_scale &&
                     expert->w2_packed && expert->w2_scale,
                 AEON_ERR_INVALID_ARGUMENT, "%s: the expert has a null sub-tensor", who);
    AEON_REQUIRE(H > 0 && I > 0 && H % 128 == 0 && I % 128 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "%s: need H%%128==0 and I%%128==0 (H=%d I=%d)", who, H, I);
    AEON_REQUIRE(scale_group == 128 || scale_group == 32, AEON_ERR_INVALID_ARGUMENT,
                 "%s: scale_group must be 128 or 32, not %d", who, scale_group);
    const int per_group = scale_group == 32 ? 4 : 1;
    AEON_REQUIRE(tokens >= 1 && tokens <= (use_mfma ? kSegTokens : 8), AEON_ERR_INVALID_ARGUMENT,
                 "%s: tokens=%d outside 1..%d for this kernel family", who, tokens,
                 use_mfma ? kSegTokens : 8);
    hipStream_t s = as_stream(stream);
    if (use_mfma) {
        SegGateUpArgs gu{};
        gu.x = static_cast<const uint16_t*>(d_x);
        gu.x_stride = H;
        gu.hidden = static_cast<uint16_t*>(d_hidden);
        gu.H = H;
        gu.I = I;
        gu.limit = swiglu_limit;
        gu.seg.capacity = 1;
        gu.direct_expert = *expert;
        gu.direct_count = tokens;
        gu.scales_per_group = per_group;
        if (int rc = launch_seg_gate_up(gu, 4, 1, 2, s)) return rc;
        SegDownArgs dn{};
        dn.hidden = static_cast<const uint16_t*>(d_hidden);
        dn.weight = d_route_weights;
        dn.contrib = d_contrib;
        dn.H = H;
        dn.I = I;
        dn.seg.capacity = 1;
        dn.direct_expert = *expert;
        dn.direct_count = tokens;
        dn.scales_per_group = per_group;
        dn.fused_out = static_cast<uint16_t*>(d_out);
        dn.fused_initial = static_cast<const uint16_t*>(d_shared);
        return launch_seg_down(dn, 4, 1, 2, s);   // the reduce over its one slot rides along
    } else {
        GemvArgs g{};
        g.x = static_cast<const uint16_t*>(d_x);
        g.x_stride = H;
        g.pa = static_cast<const uint4*>(expert->w1_packed);
        g.sa = static_cast<const uint16_t*>(expert->w1_scale);
        g.pb = static_cast<const uint4*>(expert->w3_packed);
        g.sb = static_cast<const uint16_t*>(expert->w3_scale);
        g.out_a = static_cast<uint16_t*>(d_hidden);
        g.out_stride = I;
        g.tokens = tokens;
        g.N = I;
        g.groups = H / 128;
        g.epilogue = 1;
        g.limit = swiglu_limit;
        g.scales_per_group = per_group;
        if (int rc = launch_gemv<2>(g, s)) return rc;
        GemvArgs d{};
        d.x = static_cast<const uint16_t*>(d_hidden);
        d.x_stride = I;
        d.pa = static_cast<const uint4*>(expert->w2_packed);
        d.sa = static_cast<const uint16_t*>(expert->w2_scale);
        d.out_f32 = d_contrib;
        d.out_stride = H;
        d.tokens = tokens;
        d.N = H;
        d.groups = I / 128;
        d.epilogue = 2;
        d.tok_weight = d_route_weights;
        d.scales_per_group = per_group;
        if (int rc = launch_gemv<1>(d, s)) return rc;
    }
    return launch_token_reduce(d_contrib, tokens, 1, -1, static_cast<const uint16_t*>(d_shared), H,
                               static_cast<uint16_t*>(d_out), H, H, s);
}
