// Dense fp16 projections of the real model beside the int4 experts: the router gate
// ([experts][hidden] fp16) and the shared expert (three row-major fp16 matrices).
//
//   y[t][o] = half( sum_i x[t][i] * w[o][i] ),  fp16 operands, fp32 accumulate, one rounding
//
// which is the contract of the reference's gemv_fp16_vec8_kernel (fp32 FMA chain per output,
// fp16 store); the order of the fp32 additions differs (matrix instruction over 32-column steps,
// then a fixed-order sum over the four waves that split K), the roundings do not.
//
// One workgroup = one 16-row tile of one matrix x up to 16*MT tokens; its four waves split K in
// 128-column groups (wave w takes groups w, w+4, ...). To the matrix instruction lane l supplies
// weight row l%16 / token l%16 and columns 32s + 8(l/16)..+7 of step s; the loads are issued in
// row order instead (lane l: row l/4, 16-byte piece l%4 of the step's 64 bytes) and the
// fragments change lanes through LDS. The lane ends up with rows 4(l/16)..+3 of token l%16, an
// 8-byte store. Bound by the weight stream for a decode batch. The shared expert
// is three launches: W1 and W3 (one grid, two matrices), the element-wise clamped SwiGLU, W2.
#include "common.hpp"

namespace aeon355 {

struct DenseArgs {
    const uint16_t* x;      // [tokens][x_stride] fp16
    long x_stride;
    const uint16_t* w[2];   // blockIdx.y picks the matrix: [out_dim][in_dim] row-major fp16
    uint16_t* y[2];         // [tokens][y_stride] fp16
    float* y32;             // optional (matrix 0): the fp16 result widened, [tokens][out_dim]
    long y_stride;
    int tokens, in_dim, out_dim;
};

// hidden[t][i] = half(clamped_swiglu(gate[t][i], up[t][i])): the reference's
// v4_swiglu_clamp_kernel between the shared expert's projections, eight elements a thread.
__global__ __launch_bounds__(256) void dense_swiglu_kernel(const u32x4_t* __restrict__ gate,
                                                           const u32x4_t* __restrict__ up,
                                                           u32x4_t* __restrict__ hidden, int units,
                                                           float limit) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= units) return;
    const u32x4_t g = gate[i], u = up[i];
    u32x4_t h;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float lo = clamped_swiglu(half_bits_to_float(static_cast<uint16_t>(g[q] & 0xFFFFu)),
                                        half_bits_to_float(static_cast<uint16_t>(u[q] & 0xFFFFu)), limit);
        const float hi = clamped_swiglu(half_bits_to_float(static_cast<uint16_t>(g[q] >> 16)),
                                        half_bits_to_float(static_cast<uint16_t>(u[q] >> 16)), limit);
        h[q] = float_to_half_bits(lo) | (static_cast<uint32_t>(float_to_half_bits(hi)) << 16);
    }
    hidden[i] = h;
}

template <int MT>
__global__ __launch_bounds__(256) void dense_f16_kernel(DenseArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;
    const int chunk = lane >> 4;
    const int tile = blockIdx.x;
    const int matrix = blockIdx.y;
    const int token0 = blockIdx.z * 16 * MT;
    const int groups = a.in_dim / 128;

    // Loads: lane l fetches 16 bytes of row l/4 at 16-byte piece l%4, so four neighbouring lanes
    // read 64 contiguous bytes (the matrix instruction's own lane order, row l%16 / piece l/16,
    // would make every lane a separate cache access: 64 per wave load instead of 16). The
    // fragments change lanes on their way into the MFMA,
    const int lrow = lane >> 2;
    const int lpiece = lane & 3;
    // through a wave-private LDS tile of 16 rows x 64 bytes (pitch 80 bytes: both the write in
    // load order and the read in MFMA order touch every bank evenly); LDS serves a wave's
    // accesses in order, so the wave needs no barrier between its write and its read
    __shared__ u32x4_t stage[4][2][(1 + MT) * 80];
    const int put = lrow * 5 + lpiece;
    const int take = n * 5 + chunk;
    const AEON_GLOBAL uint16_t* wrow =
        as_global<uint16_t>(a.w[matrix]) + static_cast<size_t>(tile * 16 + lrow) * a.in_dim + lpiece * 8;
    // a padded token column repeats the last live token: a valid row whose results are not stored
    const AEON_GLOBAL uint16_t* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int token = token0 + mt * 16 + lrow;
        token = token < a.tokens ? token : a.tokens - 1;
        xrow[mt] = as_global<uint16_t>(a.x) + token * a.x_stride + lpiece * 8;
    }
    float4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    // two groups in flight per wave: the next group's loads are issued before this one's MFMAs
    constexpr int D = 2;
    u32x4_t wq[D][4];
    u32x4_t xq[D][MT][4];
    auto load_group = [&](int d, int g) {
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            wq[d][st] = *reinterpret_cast<const AEON_GLOBAL u32x4_t*>(wrow + g * 128 + st * 32);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                xq[d][mt][st] = *reinterpret_cast<const AEON_GLOBAL u32x4_t*>(xrow[mt] + g * 128 + st * 32);
            }
        }
    };
    auto compute = [&](int d) {
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            u32x4_t* tile_slot = stage[wave][st & 1];
            tile_slot[put] = wq[d][st];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) tile_slot[(1 + mt) * 80 + put] = xq[d][mt][st];
            asm volatile("" ::: "memory");
            union { u32x4_t u; half8_t h; } wf, xf[MT];
            wf.u = tile_slot[take];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) xf[mt].u = tile_slot[(1 + mt) * 80 + take];
            asm volatile("" ::: "memory");
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf.h, xf[mt].h, acc[mt], 0, 0, 0);
            }
        }
    };
    const int mine = (groups - wave + 3) / 4;   // groups wave, wave+4, ...
#pragma unroll
    for (int d = 0; d < D; ++d) {
        const int j = d < mine ? d : mine - 1;
        load_group(d, mine > 0 ? wave + 4 * j : groups - 1);
    }
    int j0 = 0;
    for (; j0 + 2 * D <= mine; j0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            compute(d);
            load_group(d, wave + 4 * (j0 + d + D));
        }
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
        if (j0 + d < mine) {
            compute(d);
            if (j0 + d + D < mine) load_group(d, wave + 4 * (j0 + d + D));
        }
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
        if (j0 + D + d < mine) compute(d);
    }

    // the four waves' shares of K meet in LDS and are added in wave order
    __shared__ float4_t partial[3][MT][64];
    if (wave > 0) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) partial[wave - 1][mt][lane] = acc[mt];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int w = 0; w < 3; ++w) acc[mt] += partial[w][mt][lane];
        const int token = token0 + mt * 16 + n;
        if (token >= a.tokens) continue;
        const int row0 = tile * 16 + chunk * 4;
        uint16_t h[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) h[v] = float_to_half_bits(acc[mt][v]);
        uint2 packed;
        packed.x = h[0] | (static_cast<uint32_t>(h[1]) << 16);
        packed.y = h[2] | (static_cast<uint32_t>(h[3]) << 16);
        *reinterpret_cast<uint2*>(a.y[matrix] + token * a.y_stride + row0) = packed;
        if (a.y32 != nullptr && matrix == 0) {
            float4_t wide;
#pragma unroll
            for (int v = 0; v < 4; ++v) wide[v] = half_bits_to_float(h[v]);
            *reinterpret_cast<float4_t*>(a.y32 + static_cast<size_t>(token) * a.out_dim + row0) = wide;
        }
    }
}

static bool aligned_to(const void* p, uintptr_t bytes) {
    return (reinterpret_cast<uintptr_t>(p) & (bytes - 1)) == 0;
}

static int launch_dense(const DenseArgs& a, int matrices, hipStream_t stream) {
    if (a.tokens <= 0) return AEON_OK;
    // The kernel loads activations and weights 16 bytes a lane and stores four fp16 results
    // (8 bytes) or four fp32 (16 bytes) at a time: a base that is off those boundaries (a slice
    // of a larger tensor, say) would fault on the device instead of failing here.
    bool bases_ok = aligned_to(a.x, 16) && (a.y32 == nullptr || aligned_to(a.y32, 16));
    for (int m = 0; m < matrices; ++m) bases_ok = bases_ok && aligned_to(a.w[m], 16) && aligned_to(a.y[m], 8);
    AEON_REQUIRE(bases_ok, AEON_ERR_INVALID_ARGUMENT,
                 "dense fp16 GEMV: activations, weights and fp32 outputs must start on a 16-byte "
                 "boundary and fp16 outputs on an 8-byte one");
    const int tiles = a.out_dim / 16;
    if (a.tokens <= 16) {
        dense_f16_kernel<1><<<dim3(tiles, matrices, 1), 256, 0, stream>>>(a);
    } else if (a.tokens <= 32) {
        dense_f16_kernel<2><<<dim3(tiles, matrices, 1), 256, 0, stream>>>(a);
    } else {
        dense_f16_kernel<4><<<dim3(tiles, matrices, (a.tokens + 63) / 64), 256, 0, stream>>>(a);
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

static int check_dense_shape(int tokens, int in_dim, int out_dim, const char* who) {
    AEON_REQUIRE(tokens >= 0 && in_dim > 0 && out_dim > 0 && in_dim % 128 == 0 && out_dim % 16 == 0,
                 AEON_ERR_INVALID_ARGUMENT,
                 "%s: needs in_dim %% 128 == 0 and out_dim %% 16 == 0 (tokens=%d in_dim=%d out_dim=%d)", who,
                 tokens, in_dim, out_dim);
    return AEON_OK;
}

int launch_dense_gemv(const void* d_x, long x_stride, const void* d_w, void* d_y, long y_stride,
                      float* d_y32, int tokens, int in_dim, int out_dim, hipStream_t stream) {
    DenseArgs a{};
    a.x = static_cast<const uint16_t*>(d_x);
    a.x_stride = x_stride;
    a.w[0] = static_cast<const uint16_t*>(d_w);
    a.y[0] = static_cast<uint16_t*>(d_y);
    a.y32 = d_y32;
    a.y_stride = y_stride;
    a.tokens = tokens;
    a.in_dim = in_dim;
    a.out_dim = out_dim;
    return launch_dense(a, 1, stream);
}

int launch_dense_shared_expert(const void* d_x, long x_stride, int tokens, const void* d_w1,
                               const void* d_w3, const void* d_w2, void* d_gate, void* d_up,
                               void* d_hidden, void* d_out, long out_stride, int hidden,
                               int intermediate, float limit, hipStream_t stream) {
    if (tokens <= 0) return AEON_OK;
    DenseArgs gu{};
    gu.x = static_cast<const uint16_t*>(d_x);
    gu.x_stride = x_stride;
    gu.w[0] = static_cast<const uint16_t*>(d_w1);
    gu.w[1] = static_cast<const uint16_t*>(d_w3);
    gu.y[0] = static_cast<uint16_t*>(d_gate);
    gu.y[1] = static_cast<uint16_t*>(d_up);
    gu.y_stride = intermediate;
    gu.tokens = tokens;
    gu.in_dim = hidden;
    gu.out_dim = intermediate;
    if (int rc = launch_dense(gu, 2, stream)) return rc;
    // the activation is applied once, between the launches: inside the W2 launch every one of
    // its row-tile workgroups would redo it for all of the tokens' columns
    AEON_REQUIRE(aligned_to(d_hidden, 16), AEON_ERR_INVALID_ARGUMENT,
                 "dense shared expert: the gate, up and hidden scratch rows must start on a 16-byte boundary");
    const int units = tokens * (intermediate / 8);
    dense_swiglu_kernel<<<(units + 255) / 256, 256, 0, stream>>>(
        static_cast<const u32x4_t*>(d_gate), static_cast<const u32x4_t*>(d_up),
        static_cast<u32x4_t*>(d_hidden), units, limit);
    AEON_LAUNCH_CHECK();
    DenseArgs dn{};
    dn.x = static_cast<const uint16_t*>(d_hidden);
    dn.x_stride = intermediate;
    dn.w[0] = static_cast<const uint16_t*>(d_w2);
    dn.y[0] = static_cast<uint16_t*>(d_out);
    dn.y_stride = out_stride;
    dn.tokens = tokens;
    dn.in_dim = intermediate;
    dn.out_dim = hidden;
    return launch_dense(dn, 1, stream);
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_dense_gemv_f16(const void* d_x, int x_stride, const void* d_weight, void* d_y,
                                   int y_stride, int tokens, int in_dim, int out_dim, void* stream) {
    const char* who = "aeon_dense_gemv_f16";
    AEON_REQUIRE(d_x && d_weight && d_y, AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    if (int rc = check_dense_shape(tokens, in_dim, out_dim, who)) return rc;
    AEON_REQUIRE(x_stride >= in_dim && x_stride % 8 == 0 && y_stride >= out_dim && y_stride % 4 == 0,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad row pitch (x_stride=%d y_stride=%d)", who, x_stride,
                 y_stride);
    return launch_dense_gemv(d_x, x_stride, d_weight, d_y, y_stride, nullptr, tokens, in_dim, out_dim,
                             as_stream(stream));
}

extern "C" int aeon_dense_shared_expert_f16(const void* d_x, int x_stride, int tokens,
                                            const void* d_w1, const void* d_w3, const void* d_w2,
                                            void* d_gate, void* d_up, void* d_hidden, void* d_out,
                                            int out_stride, int hidden, int intermediate,
                                            float swiglu_limit, void* stream) {
    const char* who = "aeon_dense_shared_expert_f16";
    AEON_REQUIRE(d_x && d_w1 && d_w3 && d_w2 && d_gate && d_up && d_hidden && d_out, AEON_ERR_INVALID_ARGUMENT,
                 "%s: null buffer", who);
    if (int rc = check_dense_shape(tokens, hidden, intermediate, who)) return rc;
    if (int rc = check_dense_shape(tokens, intermediate, hidden, who)) return rc;
    AEON_REQUIRE(x_stride >= hidden && x_stride % 8 == 0 && out_stride >= hidden && out_stride % 4 == 0,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad row pitch (x_stride=%d out_stride=%d)", who, x_stride,
                 out_stride);
    return launch_dense_shared_expert(d_x, x_stride, tokens, d_w1, d_w3, d_w2, d_gate, d_up, d_hidden,
                                      d_out, out_stride, hidden, intermediate, swiglu_limit,
                                      as_stream(stream));
}

extern "C" int aeon_router_logits_f16(const void* d_x, int x_stride, const void* d_gate_weight,
                                      void* d_logits_half, float* d_logits, int tokens, int hidden,
                                      int experts, void* stream) {
    const char* who = "aeon_router_logits_f16";
    AEON_REQUIRE(d_x && d_gate_weight && d_logits_half && d_logits, AEON_ERR_INVALID_ARGUMENT,
                 "%s: null buffer", who);
    if (int rc = check_dense_shape(tokens, hidden, experts, who)) return rc;
    AEON_REQUIRE(x_stride >= hidden && x_stride % 8 == 0, AEON_ERR_INVALID_ARGUMENT,
                 "%s: bad row pitch (x_stride=%d)", who, x_stride);
    return launch_dense_gemv(d_x, x_stride, d_gate_weight, d_logits_half, experts, d_logits, tokens,
                             hidden, experts, as_stream(stream));
}
