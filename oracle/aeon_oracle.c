/*
 * CPU oracle for the routed-expert hot path (see aeon_oracle.h for scope, citations and the
 * pinning status of every function). Test infrastructure only: nothing shipped loads it.
 */
#include "aeon_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------ */
/* fp16 bit patterns                                                                     */
/* ------------------------------------------------------------------------------------ */

/* dsv4_oracle.hpp:1370-1391: normals assemble the double's bit pattern directly,
 * subnormals are mantissa * 2^-24, exponent 31 is NaN. */
double orc_half_bits_to_double(uint16_t bits) {
    const uint32_t sign = (uint32_t)(bits >> 15);
    const uint32_t exponent = (uint32_t)((bits >> 10) & 0x1Fu);
    const uint32_t mantissa = (uint32_t)(bits & 0x3FFu);
    if (exponent == 0) {
        const double value = ldexp((double)mantissa, -24);
        return sign ? -value : value;
    }
    if (exponent == 0x1F) {
        return sign ? -NAN : NAN;
    }
    const uint64_t pattern = ((uint64_t)sign << 63) |
                             ((uint64_t)(exponent - 15u + 1023u) << 52) |
                             ((uint64_t)mantissa << 42);
    double value;
    memcpy(&value, &pattern, sizeof value);
    return value;
}

uint16_t orc_double_to_half_bits(double value) {
    uint64_t u;
    memcpy(&u, &value, sizeof u);
    const uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
    const int exp64 = (int)((u >> 52) & 0x7FF);
    const uint64_t man = u & 0xFFFFFFFFFFFFFull;
    if (exp64 == 0x7FF) {
        return (uint16_t)(sign | (man ? 0x7E00u : 0x7C00u));
    }
    if (exp64 == 0) {
        return sign; /* fp64 subnormals are far below half the smallest fp16 subnormal */
    }
    const int e = exp64 - 1023; /* value = 1.man * 2^e */
    if (e > 15) {
        return (uint16_t)(sign | 0x7C00u);
    }
    /* significand with the implicit one: 53 bits */
    const uint64_t sig = man | (1ull << 52);
    int shift; /* number of low bits dropped to reach the fp16 grid */
    int base_exp;
    if (e >= -14) {
        shift = 42;          /* 53 -> 11 significant bits */
        base_exp = e + 15;   /* biased exponent of the result, before carry */
    } else {
        shift = 42 + (-14 - e); /* subnormal: grid spacing is fixed at 2^-24 */
        base_exp = 0;
        if (shift > 63) {
            return sign;
        }
    }
    uint64_t kept = sig >> shift;
    const uint64_t rest = sig & ((1ull << shift) - 1ull);
    const uint64_t half = 1ull << (shift - 1);
    if (rest > half || (rest == half && (kept & 1ull))) {
        kept += 1;
    }
    uint32_t out;
    if (base_exp > 0) {
        /* kept has the implicit bit at position 10; a carry to bit 11 bumps the exponent */
        out = (uint32_t)((uint32_t)(base_exp - 1) << 10) + (uint32_t)kept;
    } else {
        out = (uint32_t)kept; /* a carry into bit 10 lands on the smallest normal */
    }
    if (out >= 0x7C00u) {
        out = 0x7C00u;
    }
    return (uint16_t)(sign | out);
}

uint16_t orc_float_to_half_bits(float value) {
    /* fp32 -> fp64 is exact, so one RN-even step from the exact value is what is wanted. */
    return orc_double_to_half_bits((double)value);
}

/* ------------------------------------------------------------------------------------ */
/* SplitMix64, dsv4_oracle.hpp:42-74                                                     */
/* ------------------------------------------------------------------------------------ */

void orc_rng_seed(orc_rng* rng, uint64_t seed) {
    rng->state = seed != 0 ? seed : 0x9E3779B97F4A7C15ull;
}

uint64_t orc_rng_next_u64(orc_rng* rng) {
    rng->state += 0x9E3779B97F4A7C15ull;
    uint64_t z = rng->state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

double orc_rng_uniform01(orc_rng* rng) {
    return (double)(orc_rng_next_u64(rng) >> 11) * (1.0 / 9007199254740992.0);
}

double orc_rng_symmetric(orc_rng* rng, double scale) {
    return (orc_rng_uniform01(rng) * 2.0 - 1.0) * scale;
}

/* ------------------------------------------------------------------------------------ */
/* int4 storage permutation, aeon_w4a16_swizzle.hpp                                      */
/* ------------------------------------------------------------------------------------ */

static const int k_nibble_perm[8] = {0, 2, 4, 6, 1, 3, 5, 7}; /* :16 */

static uint32_t permute_word(uint32_t source) { /* :18-25 */
    uint32_t destination = 0;
    for (int position = 0; position < 8; ++position) {
        const uint32_t nibble = (source >> (4 * k_nibble_perm[position])) & 0xFu;
        destination |= nibble << (4 * position);
    }
    return destination;
}

static uint32_t unpermute_word(uint32_t source) { /* :27-34 */
    uint32_t destination = 0;
    for (int position = 0; position < 8; ++position) {
        const uint32_t nibble = (source >> (4 * position)) & 0xFu;
        destination |= nibble << (4 * k_nibble_perm[position]);
    }
    return destination;
}

static int swizzle_shape_ok(int N, int K, int rpw, int lpr) { /* :36-43 */
    return rpw > 0 && lpr > 0 && rpw * lpr == 32 && N > 0 && K > 0 && N % rpw == 0 &&
           K % 32 == 0 && (K / 32) % lpr == 0;
}

int orc_swizzle_w4a16(const uint32_t* src_packed, const uint16_t* src_scale,
                      uint32_t* dst_packed, uint16_t* dst_scale,
                      int N, int K, int rpw, int lpr) { /* :45-85 */
    if (!swizzle_shape_ok(N, K, rpw, lpr)) return -1;
    const int groups = K / 32;
    const int iterations = groups / lpr;
    const int row_blocks = N / rpw;
    const int words_per_row = K / 8;
    for (int block = 0; block < row_blocks; ++block)
        for (int iteration = 0; iteration < iterations; ++iteration)
            for (int row = 0; row < rpw; ++row)
                for (int slice = 0; slice < lpr; ++slice) {
                    const int source_row = block * rpw + row;
                    const int source_group = iteration * lpr + slice;
                    const int lane = row * lpr + slice;
                    const size_t dst_u4 = ((size_t)block * iterations + iteration) * 32 + lane;
                    const size_t src_word = (size_t)source_row * words_per_row +
                                            (size_t)source_group * 4;
                    for (int word = 0; word < 4; ++word)
                        dst_packed[dst_u4 * 4 + word] = permute_word(src_packed[src_word + word]);
                    dst_scale[dst_u4] = src_scale[(size_t)source_row * groups + source_group];
                }
    return 0;
}

int orc_unswizzle_w4a16(const uint32_t* src_packed, const uint16_t* src_scale,
                        uint32_t* dst_packed, uint16_t* dst_scale,
                        int N, int K, int rpw, int lpr) { /* :87-127 */
    if (!swizzle_shape_ok(N, K, rpw, lpr)) return -1;
    const int groups = K / 32;
    const int iterations = groups / lpr;
    const int row_blocks = N / rpw;
    const int words_per_row = K / 8;
    for (int block = 0; block < row_blocks; ++block)
        for (int iteration = 0; iteration < iterations; ++iteration)
            for (int row = 0; row < rpw; ++row)
                for (int slice = 0; slice < lpr; ++slice) {
                    const int dst_row = block * rpw + row;
                    const int dst_group = iteration * lpr + slice;
                    const int lane = row * lpr + slice;
                    const size_t src_u4 = ((size_t)block * iterations + iteration) * 32 + lane;
                    const size_t dst_word = (size_t)dst_row * words_per_row +
                                            (size_t)dst_group * 4;
                    for (int word = 0; word < 4; ++word)
                        dst_packed[dst_word + word] = unpermute_word(src_packed[src_u4 * 4 + word]);
                    dst_scale[(size_t)dst_row * groups + dst_group] = src_scale[src_u4];
                }
    return 0;
}

/* dsv4_oracle.hpp:1302-1305 */
static int nibble_slot(int s) {
    static const int slot[8] = {0, 4, 1, 5, 2, 6, 3, 7};
    return slot[s & 7];
}

/* dsv4_oracle.hpp:1313-1331 */
orc_swizzled_addr orc_swizzled_address(int columns, int rpw, int lpr, int row, int column) {
    const int iterations = (columns / 32) / lpr;
    const int group = column / 32;
    const int word_in_group = (column % 32) / 8;
    const int source_nibble = column % 8;
    const int iteration = group / lpr;
    const int slice = group % lpr;
    const int row_block = row / rpw;
    const int row_in_block = row % rpw;
    const int lane = row_in_block * lpr + slice;
    const size_t storage = ((size_t)row_block * (size_t)iterations + (size_t)iteration) * 32u +
                           (size_t)lane;
    orc_swizzled_addr a;
    a.storage_slot = storage;
    a.packed_word = storage * 4u + (size_t)word_in_group;
    a.nibble = nibble_slot(source_nibble);
    return a;
}

/* One swizzled row into doubles; the group-hoisted walk of dsv4_oracle.hpp:1442-1488. */
static void decode_row(const uint32_t* packed, const uint16_t* scale, int columns, int rpw,
                       int lpr, int row, int signed_zero_point, int permute_nibbles,
                       double* out_row) {
    const int groups = columns / 32;
    const int iterations = groups / lpr;
    const int row_block = row / rpw;
    const int row_in_block = row % rpw;
    for (int group = 0; group < groups; ++group) {
        const int iteration = group / lpr;
        const int slice = group % lpr;
        const int lane = row_in_block * lpr + slice;
        const size_t storage = ((size_t)row_block * (size_t)iterations + (size_t)iteration) * 32u +
                               (size_t)lane;
        const double s = orc_half_bits_to_double(scale[storage]);
        const uint32_t* words = packed + storage * 4u;
        double* out_group = out_row + (size_t)group * 32;
        for (int j = 0; j < 32; ++j) {
            const int nibble = permute_nibbles ? nibble_slot(j) : ((group * 32 + j) % 8);
            const uint32_t word = words[j / 8];
            const int value = (int)((word >> (4 * nibble)) & 0xFu);
            const double quantized = signed_zero_point ? (double)(value - 8) : (double)value;
            out_group[j] = quantized * s;
        }
    }
}

void orc_swizzled_decode(const uint32_t* packed, const uint16_t* scale,
                         int rows, int columns, int rpw, int lpr,
                         int signed_zero_point, int permute_nibbles, double* out) {
#pragma omp parallel for schedule(static) if (rows >= 8)
    for (int row = 0; row < rows; ++row) {
        decode_row(packed, scale, columns, rpw, lpr, row, signed_zero_point, permute_nibbles,
                   out + (size_t)row * columns);
    }
}

/* dsv4_oracle.hpp:1407-1411 */
static uint16_t half_bits_of_power_of_two(int exponent) {
    if (exponent < -14) exponent = -14;
    if (exponent > 15) exponent = 15;
    return (uint16_t)((exponent + 15) << 10);
}

/* dsv4_oracle.hpp:1525-1573 */
void orc_swizzled_encode(uint32_t* packed, uint16_t* scale,
                         int rows, int columns, int rpw, int lpr, const double* w) {
    memset(packed, 0, (size_t)rows * (size_t)columns / 2);
    memset(scale, 0, (size_t)rows * (size_t)columns / 32 * sizeof(uint16_t));
    for (int row = 0; row < rows; ++row) {
        for (int group = 0; group < columns / 32; ++group) {
            double peak = 0.0;
            for (int j = 0; j < 32; ++j)
                peak = fmax(peak, fabs(w[(size_t)row * columns + group * 32 + j]));
            const int exponent = peak > 0.0 ? (int)ceil(log2(peak / 7.0)) : -14;
            const uint16_t scale_bits = half_bits_of_power_of_two(exponent);
            const double s = orc_half_bits_to_double(scale_bits);
            for (int j = 0; j < 32; ++j) {
                const int column = group * 32 + j;
                const double value = w[(size_t)row * columns + column];
                int quantized = (int)lround(value / s);
                if (quantized < -8) quantized = -8;
                if (quantized > 7) quantized = 7;
                const orc_swizzled_addr a = orc_swizzled_address(columns, rpw, lpr, row, column);
                scale[a.storage_slot] = scale_bits;
                uint32_t word = packed[a.packed_word];
                word &= ~(0xFu << (4 * a.nibble));
                word |= (uint32_t)(quantized + 8) << (4 * a.nibble);
                packed[a.packed_word] = word;
            }
        }
    }
}

/* ------------------------------------------------------------------------------------ */
/* matvec / expert FFN                                                                   */
/* ------------------------------------------------------------------------------------ */

void orc_matvec(size_t out_dim, size_t in_dim, const double* w, const double* x, double* y) {
#pragma omp parallel for schedule(static) if (out_dim >= 8 && out_dim * in_dim >= 65536)
    for (size_t o = 0; o < out_dim; ++o) {
        double acc = 0.0;
        const double* row = w + o * in_dim;
        for (size_t i = 0; i < in_dim; ++i) acc += row[i] * x[i];
        y[o] = acc;
    }
}

void orc_swizzled_matvec(const uint32_t* packed, const uint16_t* scale,
                         int rows, int columns, int rpw, int lpr,
                         const double* x, int tokens, double* y) {
#pragma omp parallel
    {
        double* row_w = (double*)malloc((size_t)columns * sizeof(double));
#pragma omp for schedule(static)
        for (int row = 0; row < rows; ++row) {
            decode_row(packed, scale, columns, rpw, lpr, row, 1, 1, row_w);
            for (int t = 0; t < tokens; ++t) {
                const double* xt = x + (size_t)t * columns;
                double acc = 0.0;
                for (int i = 0; i < columns; ++i) acc += row_w[i] * xt[i];
                y[(size_t)t * rows + row] = acc;
            }
        }
        free(row_w);
    }
}

double orc_clamped_swiglu(double gate, double up, double limit, int mode) {
    switch (mode) {
        case 0:
            gate = fmin(gate, limit);
            up = fmin(fmax(up, -limit), limit);
            break;
        case 1:
            gate = fmin(fmax(gate, -limit), limit);
            up = fmin(fmax(up, -limit), limit);
            break;
        default:
            break;
    }
    return (gate / (1.0 + exp(-gate))) * up;
}

void orc_expert_ffn(const uint32_t* w1p, const uint16_t* w1s,
                    const uint32_t* w3p, const uint16_t* w3s,
                    const uint32_t* w2p, const uint16_t* w2s,
                    int H, int I, int rpw13, int lpr13, int rpw2, int lpr2,
                    const double* x, int tokens, double limit, int clamp_mode,
                    int round_hidden, double* hidden_out, double* out) {
    const size_t n = (size_t)tokens * (size_t)I;
    double* gate = (double*)malloc(n * sizeof(double));
    double* up = (double*)malloc(n * sizeof(double));
    double* hidden = hidden_out ? hidden_out : (double*)malloc(n * sizeof(double));
    orc_swizzled_matvec(w1p, w1s, I, H, rpw13, lpr13, x, tokens, gate);
    orc_swizzled_matvec(w3p, w3s, I, H, rpw13, lpr13, x, tokens, up);
    for (size_t i = 0; i < n; ++i) {
        double h = orc_clamped_swiglu(gate[i], up[i], limit, clamp_mode);
        if (round_hidden) h = orc_half_bits_to_double(orc_double_to_half_bits(h));
        hidden[i] = h;
    }
    orc_swizzled_matvec(w2p, w2s, H, I, rpw2, lpr2, hidden, tokens, out);
    free(gate);
    free(up);
    if (!hidden_out) free(hidden);
}

/* dsv4_oracle.hpp:1708-1753 (dense_ffn): the shared expert, an unquantised FFN with row-major
 * [out][in] weights, the same clamped SwiGLU, no rounding between the stages. w1, w3 are
 * [intermediate][hidden], w2 [hidden][intermediate], x [tokens][hidden]. `round_stages` != 0 is
 * the device's view of the same FFN (layer/v4_layer_body_moe.hpp:216-256: gate, up and the
 * activation are each stored as fp16 before the next stage reads them). */
void orc_dense_ffn(size_t intermediate, size_t hidden, const double* x, size_t tokens,
                   const double* w1, const double* w3, const double* w2, double limit,
                   int clamp_mode, int round_stages, double* hidden_out, double* out) {
    double* gate = (double*)malloc(intermediate * sizeof(double));
    double* up = (double*)malloc(intermediate * sizeof(double));
    double* act = (double*)malloc(intermediate * sizeof(double));
    for (size_t t = 0; t < tokens; ++t) {
        orc_matvec(intermediate, hidden, w1, x + t * hidden, gate);
        orc_matvec(intermediate, hidden, w3, x + t * hidden, up);
        for (size_t i = 0; i < intermediate; ++i) {
            double g = gate[i], u = up[i];
            if (round_stages) {
                g = orc_half_bits_to_double(orc_double_to_half_bits(g));
                u = orc_half_bits_to_double(orc_double_to_half_bits(u));
            }
            double h = orc_clamped_swiglu(g, u, limit, clamp_mode);
            if (round_stages) h = orc_half_bits_to_double(orc_double_to_half_bits(h));
            act[i] = h;
            if (hidden_out) hidden_out[t * intermediate + i] = h;
        }
        orc_matvec(hidden, intermediate, w2, act, out + t * hidden);
    }
    free(gate);
    free(up);
    free(act);
}

/* ------------------------------------------------------------------------------------ */
/* router                                                                                */
/* ------------------------------------------------------------------------------------ */

/* dsv4_oracle.hpp:1066-1081. A selection of the k best under the total order
 * (score descending, index ascending) is what the stable sort there returns. */
void orc_topk_indices(const double* scores, size_t n, size_t k, int32_t* ids) {
    const size_t take = k < n ? k : n;
    unsigned char* used = (unsigned char*)calloc(n ? n : 1, 1);
    for (size_t pick = 0; pick < take; ++pick) {
        long best = -1;
        for (size_t e = 0; e < n; ++e) {
            if (used[e]) continue;
            /* NaN never compares greater, as in the reference comparator (sa != sb, sa > sb) */
            if (best < 0 || scores[e] > scores[(size_t)best]) best = (long)e;
        }
        used[(size_t)best] = 1;
        ids[pick] = (int32_t)best;
    }
    free(used);
}

static double softplus(double x) { /* :1168-1172 */
    return x > 20.0 ? x : log1p(exp(x));
}

static double sigmoid(double x) { /* :485-487 */
    return 1.0 / (1.0 + exp(-x));
}

static double router_score(double logit, int score_kind) {
    return score_kind == 0 ? sqrt(softplus(logit)) : sigmoid(logit);
}

/* The fp64 scores the selection below compares, one per logit: for tests that need to know how
 * close two candidates are. */
void orc_router_scores(const double* logits, size_t n, int score_kind, double* scores) {
    for (size_t i = 0; i < n; ++i) scores[i] = router_score(logits[i], score_kind);
}

void orc_router_topk(const double* logits, const double* bias, size_t experts,
                     size_t top_k, double scaling, int score_kind,
                     int bias_before_activation, int32_t* ids, double* weights) {
    double* scores = (double*)malloc(experts * sizeof(double));
    double* selection = (double*)malloc(experts * sizeof(double));
    for (size_t e = 0; e < experts; ++e) {
        const double b = bias ? bias[e] : 0.0;
        scores[e] = bias_before_activation ? router_score(logits[e] + b, score_kind)
                                           : router_score(logits[e], score_kind);
        selection[e] = bias ? scores[e] + b : scores[e];
    }
    orc_topk_indices(selection, experts, top_k, ids);
    double sum = 0.0;
    for (size_t k = 0; k < top_k; ++k) {
        weights[k] = scores[(size_t)ids[k]];
        sum += weights[k];
    }
    for (size_t k = 0; k < top_k; ++k) {
        weights[k] /= sum;
        weights[k] *= scaling;
    }
    free(scores);
    free(selection);
}

/* ------------------------------------------------------------------------------------ */
/* permutation, expert_permutation.hpp:50-109                                            */
/* ------------------------------------------------------------------------------------ */

void orc_expert_permutation(const int32_t* ids, int tokens, int slots, int experts,
                            int32_t* offsets, int32_t* token_indices, int32_t* draw_indices) {
    const int draws = tokens * slots;
    int32_t* cursor = (int32_t*)calloc((size_t)experts + 1, sizeof(int32_t));
    for (int d = 0; d < draws; ++d)
        if (ids[d] >= 0 && ids[d] < experts) ++cursor[ids[d]];
    int32_t running = 0;
    for (int e = 0; e < experts; ++e) {
        offsets[e] = running;
        running += cursor[e];
        cursor[e] = offsets[e];
    }
    offsets[experts] = running;
    for (int d = 0; d < draws; ++d) {
        const int e = ids[d];
        if (e < 0 || e >= experts) continue;
        token_indices[cursor[e]] = d / slots;
        draw_indices[cursor[e]] = d;
        ++cursor[e];
    }
    free(cursor);
}

/* ------------------------------------------------------------------------------------ */
/* fixed-order combine                                                                   */
/* ------------------------------------------------------------------------------------ */

void orc_moe_combine(const double* contrib, int expert_count, const double* shared,
                     int hidden, double* out) {
    for (int i = 0; i < hidden; ++i) {
        double acc = shared ? shared[i] : 0.0;
        for (int e = 0; e < expert_count; ++e) acc += contrib[(size_t)e * hidden + i];
        out[i] = acc;
    }
}

/* ------------------------------------------------------------------------------------ */
/* hyper-connections                                                                     */
/* ------------------------------------------------------------------------------------ */

void orc_hc_default_params(orc_hc_params* p) { /* :489-495 */
    p->rms_eps = 1e-6;
    p->pre_eps = 1e-6;
    p->sinkhorn_eps = 1e-6;
    p->post_mult = 2.0;
    p->sinkhorn_iters = 20;
}

void orc_hc_sinkhorn(const double* mixes, const double* hc_scale, const double* hc_base,
                     int hc_mult, const orc_hc_params* p,
                     double* pre_mix, double* post_mix, double* C) { /* :529-592 */
    const int hc = hc_mult;
    for (int j = 0; j < hc; ++j)
        pre_mix[j] = sigmoid(mixes[j] * hc_scale[0] + hc_base[j]) + p->pre_eps;
    for (int j = 0; j < hc; ++j)
        post_mix[j] = sigmoid(mixes[j + hc] * hc_scale[1] + hc_base[j + hc]) * p->post_mult;
    for (int i = 0; i < hc; ++i)
        for (int j = 0; j < hc; ++j) {
            const int idx = 2 * hc + i * hc + j;
            C[i * hc + j] = mixes[idx] * hc_scale[2] + hc_base[idx];
        }
    for (int i = 0; i < hc; ++i) {
        double max_v = C[i * hc];
        for (int j = 1; j < hc; ++j) max_v = fmax(max_v, C[i * hc + j]);
        double sum_e = 0.0;
        for (int j = 0; j < hc; ++j) {
            const double e = exp(C[i * hc + j] - max_v);
            C[i * hc + j] = e;
            sum_e += e;
        }
        for (int j = 0; j < hc; ++j) C[i * hc + j] = C[i * hc + j] / sum_e + p->sinkhorn_eps;
    }
    for (int pass = 0; pass < 2 * p->sinkhorn_iters - 1; ++pass) {
        if (pass % 2 == 0) { /* normalize over i, the contraction axis */
            for (int j = 0; j < hc; ++j) {
                double col = 0.0;
                for (int i = 0; i < hc; ++i) col += C[i * hc + j];
                const double inv = 1.0 / (col + p->sinkhorn_eps);
                for (int i = 0; i < hc; ++i) C[i * hc + j] *= inv;
            }
        } else { /* normalize over j, the output axis */
            for (int i = 0; i < hc; ++i) {
                double row = 0.0;
                for (int j = 0; j < hc; ++j) row += C[i * hc + j];
                const double inv = 1.0 / (row + p->sinkhorn_eps);
                for (int j = 0; j < hc; ++j) C[i * hc + j] *= inv;
            }
        }
    }
}

void orc_hc_pre_combine(const double* residual, const double* pre_mix, int hc_mult,
                        size_t hidden, double* out) { /* :595-606 */
    for (size_t h = 0; h < hidden; ++h) {
        double acc = 0.0;
        for (int j = 0; j < hc_mult; ++j) acc += pre_mix[j] * residual[(size_t)j * hidden + h];
        out[h] = acc;
    }
}

void orc_hc_mixes(const double* residual, const double* fn, size_t mixes, size_t hc_hidden,
                  double rms_eps, double* out) { /* :509-524 */
    double sum_sq = 0.0;
    for (size_t k = 0; k < hc_hidden; ++k) sum_sq += residual[k] * residual[k];
    const double inv_rms = 1.0 / sqrt(sum_sq / (double)hc_hidden + rms_eps);
    for (size_t m = 0; m < mixes; ++m) {
        double dot = 0.0;
        for (size_t k = 0; k < hc_hidden; ++k) dot += residual[k] * fn[m * hc_hidden + k];
        out[m] = dot * inv_rms;
    }
}

void orc_rmsnorm(const double* x, const double* weight, size_t dim, double eps, double* out) {
    /* :146-169 */
    double sum_sq = 0.0;
    for (size_t i = 0; i < dim; ++i) sum_sq += x[i] * x[i];
    const double inv_rms = 1.0 / sqrt(sum_sq / (double)dim + eps);
    for (size_t i = 0; i < dim; ++i) out[i] = weight ? x[i] * inv_rms * weight[i] : x[i] * inv_rms;
}

void orc_hc_post(const double* layer_out, const double* residual, const double* post_mix,
                 const double* comb, int hc_mult, size_t hidden, int transpose_comb,
                 double* out) { /* :613-632 */
    for (int j = 0; j < hc_mult; ++j)
        for (size_t h = 0; h < hidden; ++h) {
            double acc = post_mix[j] * layer_out[h];
            for (int i = 0; i < hc_mult; ++i) {
                const double c = transpose_comb ? comb[j * hc_mult + i] : comb[i * hc_mult + j];
                acc += c * residual[(size_t)i * hidden + h];
            }
            out[(size_t)j * hidden + h] = acc;
        }
}

/* ------------------------------------------------------------------------------------ */
/* wave64 packing                                                                        */
/* ------------------------------------------------------------------------------------ */

orc_a64_addr orc_a64_address(int columns, int row, int column) {
    return orc_a64_address_g(columns, row, column, 128);
}

/* scale_group 128: one scale per (row, 128 columns) at [tile][row%16]; 32: the row's four
 * group-32 scales of the 128 columns side by side, [tile][row%16][step]. */
orc_a64_addr orc_a64_address_g(int columns, int row, int column, int scale_group) {
    const int groups = columns / 128;
    const int tile_row = row / 16;
    const int r = row % 16;
    const int g = column / 128;
    const int in_group = column % 128;
    const int s = in_group / 32;          /* which word of the lane's uint4 */
    const int chunk = (in_group % 32) / 8; /* which 8-column chunk of the 32-wide step */
    const int lane = chunk * 16 + r;
    const size_t tile = (size_t)tile_row * (size_t)groups + (size_t)g;
    orc_a64_addr a;
    a.packed_word = (tile * 64u + (size_t)lane) * 4u + (size_t)s;
    a.nibble = nibble_slot(column % 8);
    a.scale_index = scale_group == 32 ? (tile * 16u + (size_t)r) * 4u + (size_t)s
                                      : tile * 16u + (size_t)r;
    return a;
}

int orc_a64_pack(const uint32_t* src_packed, const uint16_t* src_scale32,
                 int rows, int columns, uint32_t* a64_packed, uint16_t* a64_scale) {
    return orc_a64_pack_g(src_packed, src_scale32, rows, columns, 128, a64_packed, a64_scale);
}

int orc_a64_pack_g(const uint32_t* src_packed, const uint16_t* src_scale32, int rows, int columns,
                   int scale_group, uint32_t* a64_packed, uint16_t* a64_scale) {
    if (rows <= 0 || columns <= 0 || rows % 16 != 0 || columns % 128 != 0) return -1;
    if (scale_group != 128 && scale_group != 32) return -3;
    const int groups32 = columns / 32;
    memset(a64_packed, 0, (size_t)rows * (size_t)columns / 2);
    for (int row = 0; row < rows; ++row) {
        for (int column = 0; column < columns; ++column) {
            const uint32_t word = src_packed[(size_t)row * (columns / 8) + column / 8];
            const uint32_t q = (word >> (4 * (column % 8))) & 0xFu;
            const orc_a64_addr a = orc_a64_address_g(columns, row, column, scale_group);
            a64_packed[a.packed_word] |= q << (4 * a.nibble);
            if (scale_group == 32) {
                if (column % 32 == 0) {
                    a64_scale[a.scale_index] = src_scale32[(size_t)row * groups32 + column / 32];
                }
            } else if (column % 128 == 0) {
                const uint16_t* s = src_scale32 + (size_t)row * groups32 + column / 32;
                if (s[0] != s[1] || s[0] != s[2] || s[0] != s[3]) return -2;
                a64_scale[a.scale_index] = s[0];
            }
        }
    }
    return 0;
}

void orc_a64_decode(const uint32_t* a64_packed, const uint16_t* a64_scale,
                    int rows, int columns, double* out) {
    orc_a64_decode_g(a64_packed, a64_scale, rows, columns, 128, out);
}

void orc_a64_decode_g(const uint32_t* a64_packed, const uint16_t* a64_scale, int rows, int columns,
                      int scale_group, double* out) {
    for (int row = 0; row < rows; ++row)
        for (int column = 0; column < columns; ++column) {
            const orc_a64_addr a = orc_a64_address_g(columns, row, column, scale_group);
            const int q = (int)((a64_packed[a.packed_word] >> (4 * a.nibble)) & 0xFu);
            out[(size_t)row * columns + column] =
                (double)(q - 8) * orc_half_bits_to_double(a64_scale[a.scale_index]);
        }
}
