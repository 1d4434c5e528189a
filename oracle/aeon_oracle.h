/*
 * CPU oracle for the routed-expert hot path: a shape-parametrised restatement, in plain C
 * with fp64 accumulation, of the arithmetic the reference states in
 *   src/architecture/deepseek_v4/reference/dsv4_oracle.hpp   (host-only fp64 oracle)
 *   src/backend/swizzled_w4a16/kernels/aeon_w4a16_swizzle.hpp (int4 storage permutation)
 *   src/platform/ops/expert_permutation.hpp:3-34              (token -> expert permutation)
 *   src/platform/ops/moe_accumulate.hpp:46-92                 (fixed-order reduce)
 *   src/architecture/deepseek_v4/kernels/moe_router.hpp:154-188 (selection order)
 *
 * THIS IS TEST INFRASTRUCTURE. Only tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py may load it, and only as the checker. The HIP library never links,
 * loads or calls anything in this directory.
 *
 * Pinning status (what makes each function trustworthy without retyping it in a test):
 *   orc_swizzle/unswizzle, orc_swizzled_address, orc_swizzled_decode/encode,
 *   orc_half_bits_to_double, orc_matvec, orc_clamped_swiglu, orc_expert_ffn,
 *   orc_topk_indices, orc_router_topk (sqrt-softplus score), orc_hc_sinkhorn,
 *   orc_hc_pre_combine, orc_hc_post:
 *       compared against the reference's own code compiled from /root/reference into
 *       oracle/_ref (tests/test_oracle_vs_ref.py) on the reference's 4096/2048/group-32
 *       shapes, plus closed forms and brute force (tests/test_oracle_pins.py).
 *   orc_router_topk (sigmoid score), orc_expert_permutation, orc_moe_combine,
 *   orc_double_to_half_bits, orc_a64_*:
 *       no reference host code exists for them (the reference states them only as device
 *       kernels or not at all); pinned by definitional invariants, brute force on tiny
 *       inputs, exhaustive fp16 round trips and closed forms (tests/test_oracle_pins.py).
 *   No function here is "parity unpinned".
 */
#ifndef AEON_ORACLE_H
#define AEON_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fp16 bit patterns ------------------------------------------------------------ */
/* dsv4_oracle.hpp:1370-1391 */
double orc_half_bits_to_double(uint16_t bits);
/* Round-to-nearest-even double -> fp16 bits (what `__float2half` does to an fp32 that is
 * itself exact; used where the reference's device path stores fp16). */
uint16_t orc_double_to_half_bits(double value);
/* fp32 -> fp16 RN-even, the rounding `__float2half` applies to a device fp32 value. */
uint16_t orc_float_to_half_bits(float value);

/* ---- SplitMix64, dsv4_oracle.hpp:42-74 --------------------------------------------- */
typedef struct { uint64_t state; } orc_rng;
void orc_rng_seed(orc_rng* rng, uint64_t seed);
uint64_t orc_rng_next_u64(orc_rng* rng);
double orc_rng_uniform01(orc_rng* rng);
double orc_rng_symmetric(orc_rng* rng, double scale);

/* ---- int4 storage permutation, aeon_w4a16_swizzle.hpp:9-127 -------------------------- */
/* Source layout: packed [N][K/8] u32, nibble (k%8) at bits 4*(k%8); scales [N][K/32].
 * Returns 0, or -1 when (N,K,rpw,lpr) violates validate_w4a16_swizzle (:36-43). */
int orc_swizzle_w4a16(const uint32_t* src_packed, const uint16_t* src_scale,
                      uint32_t* dst_packed, uint16_t* dst_scale,
                      int N, int K, int rpw, int lpr);
int orc_unswizzle_w4a16(const uint32_t* src_packed, const uint16_t* src_scale,
                        uint32_t* dst_packed, uint16_t* dst_scale,
                        int N, int K, int rpw, int lpr);

/* dsv4_oracle.hpp:1302-1331, parametrised over (columns, rpw, lpr) */
typedef struct { size_t storage_slot; size_t packed_word; int nibble; } orc_swizzled_addr;
orc_swizzled_addr orc_swizzled_address(int columns, int rpw, int lpr, int row, int column);

/* dsv4_oracle.hpp:1442-1488. `packed`/`scale` point at one swizzled matrix; writes the
 * row-major [rows][columns] doubles. signed_zero_point / permute_nibbles are the two
 * deliberately-wrong readings of :1413-1416 (pass 1,1 for the format). */
void orc_swizzled_decode(const uint32_t* packed, const uint16_t* scale,
                         int rows, int columns, int rpw, int lpr,
                         int signed_zero_point, int permute_nibbles, double* out);
/* dsv4_oracle.hpp:1521-1573 (power-of-two scales). */
void orc_swizzled_encode(uint32_t* packed, uint16_t* scale,
                         int rows, int columns, int rpw, int lpr, const double* w);

/* ---- matvec / expert FFN ----------------------------------------------------------- */
/* dsv4_oracle.hpp:371-386: y[o] = sum_i w[o*in+i]*x[i], one fp64 accumulator per row,
 * i ascending; OpenMP over rows only (bit-neutral). */
void orc_matvec(size_t out_dim, size_t in_dim, const double* w, const double* x, double* y);
/* Same arithmetic, reading a swizzled matrix in place (decode of a row, then the row's
 * dot product): value-identical to orc_swizzled_decode + orc_matvec because (q-8)*scale is
 * exact in fp64. x is [tokens][columns], y is [tokens][rows]. */
void orc_swizzled_matvec(const uint32_t* packed, const uint16_t* scale,
                         int rows, int columns, int rpw, int lpr,
                         const double* x, int tokens, double* y);
/* dsv4_oracle.hpp:1591-1606. mode 0 = asymmetric (the format), 1 = symmetric, 2 = none. */
double orc_clamped_swiglu(double gate, double up, double limit, int mode);

/* dsv4_oracle.hpp:1633-1671 over swizzled matrices (W1,W3: [I][H] rpw13/lpr13; W2: [H][I]).
 * round_hidden: 0 keeps `hidden` in fp64 (the reference oracle); 1 rounds it to fp16 first,
 * as tests/test_v4_grouped_wmma_oracle.cpp:219-231 does to mirror the device store.
 * x is [tokens][H]; out is [tokens][H]; hidden_out (nullable) is [tokens][I]. */
void orc_expert_ffn(const uint32_t* w1p, const uint16_t* w1s,
                    const uint32_t* w3p, const uint16_t* w3s,
                    const uint32_t* w2p, const uint16_t* w2s,
                    int H, int I, int rpw13, int lpr13, int rpw2, int lpr2,
                    const double* x, int tokens, double limit, int clamp_mode,
                    int round_hidden, double* hidden_out, double* out);

/* ---- router ------------------------------------------------------------------------ */
/* dsv4_oracle.hpp:1066-1081: descending score, ties to the lower index. */
void orc_topk_indices(const double* scores, size_t n, size_t k, int32_t* ids);
/* dsv4_oracle.hpp:1186-1223. score_kind 0 = sqrt(softplus) (:1168-1176), 1 = sigmoid
 * (:485-487). bias may be NULL. weights[k] = unbiased score / sum * scaling. */
void orc_dense_ffn(size_t intermediate, size_t hidden, const double* x, size_t tokens,
                   const double* w1, const double* w3, const double* w2, double limit,
                   int clamp_mode, int round_stages, double* hidden_out, double* out);
void orc_router_scores(const double* logits, size_t n, int score_kind, double* scores);
void orc_router_topk(const double* logits, const double* bias, size_t experts,
                     size_t top_k, double scaling, int score_kind,
                     int bias_before_activation, int32_t* ids, double* weights);

/* ---- permutation, expert_permutation.hpp:3-34,50-128 -------------------------------- */
/* Stable counting sort of draws by expert id; ids outside [0,experts) are dropped. */
void orc_expert_permutation(const int32_t* ids, int tokens, int slots, int experts,
                            int32_t* offsets, int32_t* token_indices, int32_t* draw_indices);

/* ---- fixed-order combine, moe_accumulate.hpp:73-92 ---------------------------------- */
/* out[i] = half( float(shared[i]) + sum_{e ascending} contrib[e][i] ) evaluated in fp64
 * (the fp64 slot-order sum of tests/test_v4_moe_accum_oracle.cpp). shared may be NULL.
 * Returns the unrounded fp64 sums. */
void orc_moe_combine(const double* contrib, int expert_count, const double* shared,
                     int hidden, double* out);

/* ---- hyper-connections, dsv4_oracle.hpp:485-632 -------------------------------------- */
typedef struct {
    double rms_eps, pre_eps, sinkhorn_eps, post_mult;
    int sinkhorn_iters;
} orc_hc_params;
void orc_hc_default_params(orc_hc_params* p);
/* mixes [hc*(2+hc)], hc_scale [3], hc_base [hc*(2+hc)] -> pre [hc], post [hc], comb [hc*hc]
 * with comb[i*hc+j], i the contraction stream and j the output stream. */
void orc_hc_sinkhorn(const double* mixes, const double* hc_scale, const double* hc_base,
                     int hc_mult, const orc_hc_params* p,
                     double* pre_mix, double* post_mix, double* comb);
void orc_hc_pre_combine(const double* residual, const double* pre_mix, int hc_mult,
                        size_t hidden, double* out);
/* hc_mixes, dsv4_oracle.hpp:509-524: residual [hc_hidden] flattened, fn [mixes][hc_hidden]. */
void orc_hc_mixes(const double* residual, const double* fn, size_t mixes, size_t hc_hidden,
                  double rms_eps, double* out);
/* rmsnorm / rmsnorm_unit, dsv4_oracle.hpp:146-169: weight NULL = the weightless form. */
void orc_rmsnorm(const double* x, const double* weight, size_t dim, double eps, double* out);
void orc_hc_post(const double* layer_out, const double* residual, const double* post_mix,
                 const double* comb, int hc_mult, size_t hidden, int transpose_comb,
                 double* out);

/* ---- wave64 packing ("A64"), the build's own layout ---------------------------------- */
/* One tile = 16 rows x 128 columns = 64 lanes x uint4. Lane l = (row l%16, chunk l/16);
 * word s of the lane's uint4 holds columns 128g + 32s + 8*chunk + 0..7 in the swizzled
 * nibble order of dsv4_oracle.hpp:1302-1305. One fp16 scale per (row, 128-group).
 * Addresses are written out scalar by scalar, as orc_swizzled_address is. */
typedef struct { size_t packed_word; int nibble; size_t scale_index; } orc_a64_addr;
orc_a64_addr orc_a64_address(int columns, int row, int column);
/* The same with the scale grouping stated: 128 (as above) or 32 (four scales kept per 128
 * columns, [tile][row%16][32-column step]). */
orc_a64_addr orc_a64_address_g(int columns, int row, int column, int scale_group);
int orc_a64_pack_g(const uint32_t* src_packed, const uint16_t* src_scale32, int rows, int columns,
                   int scale_group, uint32_t* a64_packed, uint16_t* a64_scale);
void orc_a64_decode_g(const uint32_t* a64_packed, const uint16_t* a64_scale, int rows, int columns,
                      int scale_group, double* out);
/* From the source layout. Returns -1 on a bad shape (rows%16, columns%128) and -2 when the
 * four group-32 scales of a 128-group are not bit-equal. */
int orc_a64_pack(const uint32_t* src_packed, const uint16_t* src_scale32,
                 int rows, int columns, uint32_t* a64_packed, uint16_t* a64_scale);
void orc_a64_decode(const uint32_t* a64_packed, const uint16_t* a64_scale,
                    int rows, int columns, double* out);

#ifdef __cplusplus
}
#endif
#endif
