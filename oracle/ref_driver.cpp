// C entry points over the reference's own host-only oracle and swizzle headers, compiled
// from the sources where they lie (-I/root/reference/src) into oracle/_ref/libaeon_ref.so
// by oracle/Makefile. It exists so the C restatement in aeon_oracle.c can be compared with
// the reference's code itself on the reference's fixed shapes (hidden 4096, intermediate
// 2048, group 32). Test infrastructure only; nothing here is a stand-in for a reference
// header, and no reference source is copied.
#include "architecture/deepseek_v4/reference/dsv4_oracle.hpp"
#include "backend/swizzled_w4a16/kernels/aeon_w4a16_swizzle.hpp"

#include <cstdint>
#include <cstring>
#include <vector>

namespace ref = aeon::reference;

namespace {
ref::SwizzledKind kind_of(int kind) {
    return kind == 0 ? ref::SwizzledKind::W1 : kind == 1 ? ref::SwizzledKind::W2 : ref::SwizzledKind::W3;
}
}

extern "C" {

uint64_t ref_rng_draws(uint64_t seed, int count, uint64_t* out_u64, double* out_uniform,
                       double* out_symmetric, double scale) {
    ref::Rng a(seed), b(seed), c(seed);
    uint64_t last = 0;
    for (int i = 0; i < count; ++i) {
        last = a.next_u64();
        if (out_u64) out_u64[i] = last;
        if (out_uniform) out_uniform[i] = b.uniform01();
        if (out_symmetric) out_symmetric[i] = c.symmetric(scale);
    }
    return last;
}

double ref_half_bits_to_double(uint16_t bits) { return ref::half_bits_to_double(bits); }

void ref_swizzle_u16(const uint32_t* sp, const uint16_t* ss, uint32_t* dp, uint16_t* ds,
                     int N, int K, int rpw, int lpr) {
    aeon::swizzle_w4a16(sp, ss, dp, ds, N, K, aeon::SwizzleCfg{rpw, lpr});
}

void ref_unswizzle_u16(const uint32_t* sp, const uint16_t* ss, uint32_t* dp, uint16_t* ds,
                       int N, int K, int rpw, int lpr) {
    aeon::unswizzle_w4a16(sp, ss, dp, ds, N, K, aeon::SwizzleCfg{rpw, lpr});
}

// kind: 0 = W1, 1 = W2, 2 = W3 of the reference's per-expert payload.
void ref_shape(int kind, size_t* packed_offset, size_t* scale_offset, int* rows, int* columns,
               int* rpw, int* lpr) {
    const ref::SwizzledShape s = ref::swizzled_shape(kind_of(kind));
    *packed_offset = s.packed_offset;
    *scale_offset = s.scale_offset;
    *rows = s.rows;
    *columns = s.columns;
    *rpw = s.rows_per_wave;
    *lpr = s.lanes_per_row;
}

void ref_swizzled_address(int kind, int row, int column, size_t* storage_slot,
                          size_t* packed_word, int* nibble) {
    const ref::SwizzledAddress a =
        ref::swizzled_address(ref::swizzled_shape(kind_of(kind)), row, column);
    *storage_slot = a.storage_slot;
    *packed_word = a.packed_word;
    *nibble = a.nibble;
}

void ref_swizzled_decode(const uint8_t* payload, int kind, int signed_zp, int permute,
                         double* out) {
    ref::SwizzledDecodeOptions o;
    o.signed_zero_point = signed_zp != 0;
    o.permute_nibbles = permute != 0;
    const std::vector<double> w = ref::swizzled_decode(payload, kind_of(kind), o);
    std::memcpy(out, w.data(), w.size() * sizeof(double));
}

void ref_swizzled_encode(uint8_t* payload, int kind, const double* w) {
    const ref::SwizzledShape s = ref::swizzled_shape(kind_of(kind));
    ref::swizzled_encode(payload, kind_of(kind), std::vector<double>(w, w + s.weight_count()));
}

void ref_matvec(size_t out_dim, size_t in_dim, const double* w, const double* x, double* y) {
    const std::vector<double> xv(x, x + in_dim);
    const std::vector<double> r = ref::matvec(
        out_dim, in_dim, xv, [&](size_t o, size_t i) { return w[o * in_dim + i]; });
    std::memcpy(y, r.data(), out_dim * sizeof(double));
}

double ref_clamped_swiglu(double gate, double up, double limit, int mode) {
    return ref::clamped_swiglu(gate, up, limit,
                               mode == 0 ? ref::ClampMode::Asymmetric
                               : mode == 1 ? ref::ClampMode::Symmetric
                                           : ref::ClampMode::None);
}

// One routed expert over the reference payload layout; activation [4096] -> out [4096].
void ref_expert_ffn(const uint8_t* payload, const double* activation, double limit, int mode,
                    double* out) {
    const std::vector<double> x(activation, activation + 4096);
    const std::vector<double> r = ref::expert_ffn(
        payload, x, limit,
        mode == 0 ? ref::ClampMode::Asymmetric
        : mode == 1 ? ref::ClampMode::Symmetric
                    : ref::ClampMode::None);
    std::memcpy(out, r.data(), r.size() * sizeof(double));
}

void ref_dense_ffn(size_t intermediate, size_t hidden, const double* x, const double* w1,
                   const double* w3, const double* w2, double limit, int mode, double* out) {
    const std::vector<double> r = ref::dense_ffn(
        intermediate, hidden, std::vector<double>(x, x + hidden),
        std::vector<double>(w1, w1 + intermediate * hidden),
        std::vector<double>(w3, w3 + intermediate * hidden),
        std::vector<double>(w2, w2 + hidden * intermediate), limit,
        mode == 0 ? ref::ClampMode::Asymmetric
        : mode == 1 ? ref::ClampMode::Symmetric
                    : ref::ClampMode::None);
    std::memcpy(out, r.data(), r.size() * sizeof(double));
}

void ref_topk_indices(const double* scores, size_t n, size_t k, int32_t* ids) {
    const std::vector<int32_t> r = ref::topk_indices(std::vector<double>(scores, scores + n), k);
    std::memcpy(ids, r.data(), r.size() * sizeof(int32_t));
}

void ref_router_topk(const double* logits, const double* bias, size_t experts, size_t top_k,
                     double scaling, int bias_before, int32_t* ids, double* weights) {
    const std::vector<double> l(logits, logits + experts);
    const std::vector<double> b = bias ? std::vector<double>(bias, bias + experts)
                                       : std::vector<double>();
    const ref::RouterSelection s = ref::router_topk(l, b, top_k, scaling, bias_before != 0);
    std::memcpy(ids, s.ids.data(), top_k * sizeof(int32_t));
    std::memcpy(weights, s.weights.data(), top_k * sizeof(double));
}

double ref_sigmoid(double x) { return ref::sigmoid(x); }

void ref_hc_sinkhorn(const double* mixes, const double* hc_scale, const double* hc_base,
                     int hc_mult, double pre_eps, double sinkhorn_eps, double post_mult,
                     int iters, double* pre, double* post, double* comb) {
    const size_t m3 = static_cast<size_t>(hc_mult) * (2 + hc_mult);
    ref::HcParams p;
    p.pre_eps = pre_eps;
    p.sinkhorn_eps = sinkhorn_eps;
    p.post_mult = post_mult;
    p.sinkhorn_iters = iters;
    ref::HcPreResult r;
    ref::hc_sinkhorn(std::vector<double>(mixes, mixes + m3),
                     std::vector<double>(hc_scale, hc_scale + 3),
                     std::vector<double>(hc_base, hc_base + m3), hc_mult, p, r);
    std::memcpy(pre, r.pre_mix.data(), hc_mult * sizeof(double));
    std::memcpy(post, r.post_mix.data(), hc_mult * sizeof(double));
    std::memcpy(comb, r.comb.data(), static_cast<size_t>(hc_mult) * hc_mult * sizeof(double));
}

void ref_hc_pre_combine(const double* residual, const double* pre, int hc_mult, size_t hidden,
                        double* out) {
    const std::vector<double> r = ref::hc_pre_combine(
        std::vector<double>(residual, residual + hc_mult * hidden),
        std::vector<double>(pre, pre + hc_mult), hidden);
    std::memcpy(out, r.data(), hidden * sizeof(double));
}

void ref_hc_mixes(const double* residual, const double* fn, size_t mixes, size_t hc_hidden,
                  double rms_eps, double* out) {
    const std::vector<double> r = ref::hc_mixes(
        std::vector<double>(residual, residual + hc_hidden), mixes,
        [&](size_t m, size_t k) { return fn[m * hc_hidden + k]; }, hc_hidden, rms_eps);
    std::memcpy(out, r.data(), mixes * sizeof(double));
}

void ref_rmsnorm(const double* x, const double* weight, size_t dim, double eps, double* out) {
    const std::vector<double> xv(x, x + dim);
    const std::vector<double> r = weight ? ref::rmsnorm(xv, std::vector<double>(weight, weight + dim), eps)
                                         : ref::rmsnorm_unit(xv, eps);
    std::memcpy(out, r.data(), dim * sizeof(double));
}

void ref_hc_post(const double* layer_out, const double* residual, const double* post,
                 const double* comb, int hc_mult, size_t hidden, int transpose, double* out) {
    const std::vector<double> r = ref::hc_post(
        std::vector<double>(layer_out, layer_out + hidden),
        std::vector<double>(residual, residual + hc_mult * hidden),
        std::vector<double>(post, post + hc_mult),
        std::vector<double>(comb, comb + hc_mult * hc_mult), hidden, transpose != 0);
    std::memcpy(out, r.data(), hc_mult * hidden * sizeof(double));
}

}  // extern "C"
