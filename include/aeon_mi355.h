/*
 * C ABI of the MI355X (gfx950, wave64) routed-expert hot path for project-aeon.
 *
 * Every entry point is what the reference's own C++ entry point for the same step would bind
 * (the file:line each one replaces is cited beside it; paths are relative to the reference
 * tree). Conventions, which are the reference's (src/infrastructure/hip_check.hpp:19-27,
 * aeon_w4a16_swizzled_gemv.hpp:176-181):
 *   - plain pointers and sizes only; every `const void*`/`void*` named `d_…` is a DEVICE
 *     pointer owned by the caller; `half` data is IEEE fp16 bits;
 *   - device work is enqueued asynchronously on `stream` (a hipStream_t passed as void*,
 *     NULL = the default stream) and nothing synchronizes unless stated;
 *   - the return value is AEON_OK or an AEON_ERR_* code, and aeon_last_error() returns the
 *     calling thread's message. The C++ shims re-throw the reference's exception types:
 *     AEON_ERR_INVALID_ARGUMENT -> std::invalid_argument, AEON_ERR_LOGIC -> std::logic_error,
 *     AEON_ERR_OUT_OF_RANGE -> std::out_of_range, AEON_ERR_HIP -> std::runtime_error;
 *   - nothing is thread-safe beyond the error string: one host thread drives one stream.
 */
#ifndef AEON_MI355_H
#define AEON_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AEON_OK 0
#define AEON_ERR_INVALID_ARGUMENT 1
#define AEON_ERR_LOGIC 2
#define AEON_ERR_OUT_OF_RANGE 3
#define AEON_ERR_HIP 4
#define AEON_ERR_IO 5 /* file missing, truncated or malformed: std::runtime_error in the shims */

const char* aeon_last_error(void);
/* ABI revision of this header. */
int aeon_abi_version(void);

/* ------------------------------------------------------------------------------------------
 * Weight layout (host side, load time)
 * ---------------------------------------------------------------------------------------- */

/* aeon::swizzle_w4a16 / aeon::unswizzle_w4a16,
 * src/backend/swizzled_w4a16/kernels/aeon_w4a16_swizzle.hpp:45-127, for 2-byte scales.
 * Source layout: packed [N][K/8] u32 with column k in nibble k%8; scales [N][K/32].
 * (rpw, lpr) is the reference SwizzleCfg: (4,8) for W1/W3, (8,4) for W2. Host pointers. */
int aeon_swizzle_w4a16(const uint32_t* src_packed, const uint16_t* src_scale,
                       uint32_t* dst_packed, uint16_t* dst_scale, int N, int K, int rpw, int lpr);
int aeon_unswizzle_w4a16(const uint32_t* src_packed, const uint16_t* src_scale,
                         uint32_t* dst_packed, uint16_t* dst_scale, int N, int K, int rpw, int lpr);

/* The gfx950 wave64 packing ("A64"), the load-time re-swizzle of the `.aeon` payload
 * (src/backend/swizzled_w4a16/core/swizzled_expert_format.hpp:9-30 is the layout it reads).
 * A tile is 16 rows x 128 columns = 64 lanes x 16 bytes, tiles ordered [row/16][column/128];
 * lane l holds row l%16 and, in word s of its uint4, columns 128g+32s+8(l/16)+0..7 in the
 * payload's own nibble order. Requires N%16==0, K%128==0.
 * `scale_group` (everywhere below) is the number of columns one fp16 scale covers:
 *   32  -- the payload's own scales, all kept (swizzled_expert_format.hpp:18-23: one per 32
 *          columns): [tile][row%16][s], s = 0..3 the scale of columns 128g+32s..+31;
 *   128 -- one scale per (row, 128 columns) at [tile][row%16], a quarter of the scale bytes;
 *          only for payloads whose four group-32 scales inside every 128 columns are bit-equal.
 * Sizes in bytes (aeon_a64_scale_bytes is 0 for any other scale_group): */
size_t aeon_a64_packed_bytes(int N, int K);
size_t aeon_a64_scale_bytes(int N, int K, int scale_group);
/* Host repack of one swizzled matrix. With scale_group 128 it fails with
 * AEON_ERR_INVALID_ARGUMENT when the four group-32 scales of any 128 columns are not bit-equal. */
int aeon_a64_repack_host(const uint32_t* swz_packed, const uint16_t* swz_scale, int N, int K,
                         int rpw, int lpr, int scale_group, uint32_t* a64_packed,
                         uint16_t* a64_scale);
int aeon_a64_unrepack_host(const uint32_t* a64_packed, const uint16_t* a64_scale, int N, int K,
                           int rpw, int lpr, int scale_group, uint32_t* swz_packed,
                           uint16_t* swz_scale);
/* Device repack (one launch). With scale_group 128, `d_mismatch` (int, nullable) is incremented
 * once per 128 columns of a row whose four group-32 scales differ; the caller zeroes and reads
 * it, and a non-zero count means the result must not be used. */
int aeon_a64_repack_device(const void* d_swz_packed, const void* d_swz_scale, int N, int K,
                           int rpw, int lpr, int scale_group, void* d_a64_packed,
                           void* d_a64_scale, int* d_mismatch, void* stream);

/* ------------------------------------------------------------------------------------------
 * Decode kernels over the `.aeon` swizzled layout (the drop-in entry points)
 * ---------------------------------------------------------------------------------------- */

/* dispatch_aeon_w4a16_swizzled_gemv<WAVES,RPW,LPR,ITERS>,
 * src/backend/swizzled_w4a16/kernels/aeon_w4a16_swizzled_gemv.hpp:166-190.
 * y[row] = sum_g scale[row,g] * dot(q[row,g,:]-8, x[32g..]); fp32 accumulate, fp16 out.
 * The template arguments become runtime ints; K must equal iters*lpr*32 and N%rpw==0. */
int aeon_w4a16_swizzled_gemv(const void* d_activation, const void* d_packed, const void* d_scale,
                             void* d_output, int N, int K, int rpw, int lpr, void* stream);
/* dispatch_aeon_w4a16_swizzled_dual_gemv, aeon_w4a16_swizzled_gemv.hpp:192-222. */
int aeon_w4a16_swizzled_dual_gemv(const void* d_activation, const void* d_packed_a,
                                  const void* d_scale_a, const void* d_packed_b,
                                  const void* d_scale_b, void* d_output_a, void* d_output_b,
                                  int N, int K, int rpw, int lpr, void* stream);

#define AEON_SWIZZLED_MAX_EXPERTS 8
/* SwizzledW13ExpertPtrs / SwizzledW2ExpertPtrs, aeon_moe_fused_w13.hpp:13-20 and
 * aeon_moe_fused_w2.hpp:12-15: by-value tables of device pointers, same member order. */
typedef struct {
    const void* w1[AEON_SWIZZLED_MAX_EXPERTS];
    const void* s1[AEON_SWIZZLED_MAX_EXPERTS];
    const void* w3[AEON_SWIZZLED_MAX_EXPERTS];
    const void* s3[AEON_SWIZZLED_MAX_EXPERTS];
} aeon_w13_table;
typedef struct {
    const void* w2[AEON_SWIZZLED_MAX_EXPERTS];
    const void* s2[AEON_SWIZZLED_MAX_EXPERTS];
} aeon_w2_table;

/* dispatch_dsv4_moe_gemv_w13_swiglu (src/architecture/deepseek_v4/kernels/
 * moe_gemv_dispatch.hpp:28-45) = dispatch_aeon_moe_fused_gate_up with
 * Dsv4ClampedSwiGLUEpilogue (aeon_moe_fused_w13.hpp:113-141, moe_grouped_epilogue.hpp:29-37):
 * expert_hidden[e*N+row] = half(silu(min(g,L)) * clamp(u,-L,L)). `d_output_f32` (nullable) is
 * zeroed for `output_dim` floats, as the reference kernel does (:55-61). */
int aeon_moe_gemv_w13_swiglu(const void* d_activation, const aeon_w13_table* weights,
                             void* d_expert_hidden, float* d_output_f32, int output_dim,
                             int expert_count, int N, int K, int rpw, int lpr, float swiglu_limit,
                             void* stream);
/* dispatch_aeon_moe_fused_w2_contrib, aeon_moe_fused_w2.hpp:231-256:
 * contrib[e*N+row] = topk_w[e] * (W2_e . hidden_e)[row], one writer per element. */
int aeon_moe_fused_w2_contrib(const void* d_expert_hidden, const aeon_w2_table* weights,
                              const float* d_topk_weights, float* d_contrib, int expert_count,
                              int N, int K, int rpw, int lpr, void* stream);

/* The one-launch accumulation control, aeon_moe_fused_w2_accum_kernel + dispatch
 * (aeon_moe_fused_w2.hpp:73-174): output_f32[row] += sum over e of topk_w[e] * (W2_e . hidden_e)[row]
 * (+ initial_output[row] with e = 0 when given), output_f16[row] = half(output_f32[row]). The
 * reference adds with atomicAdd in the scheduler's order and keeps per-block completion
 * counters; here one workgroup owns a row block and walks the experts in slot order, so the
 * result is reproducible and no counters are needed (the caller's stay untouched, i.e. at the
 * zero the reference leaves them at). */
int aeon_moe_fused_w2_accum(const void* d_expert_hidden, const aeon_w2_table* weights,
                            const float* d_topk_weights, const void* d_initial_output,
                            float* d_output_f32, void* d_output_f16, int expert_count, int N,
                            int K, int rpw, int lpr, void* stream);
/* moe_accumulate_fixed_order_kernel launch, src/platform/ops/moe_accumulate.hpp:73-92:
 * out[i] = half(float(shared[i]) + sum_{e ascending} contrib[e*hidden+i]); `d_shared` may be
 * NULL and may alias `d_out`. */
int aeon_moe_accumulate_fixed_order(const float* d_contrib, int expert_count,
                                    const void* d_shared, void* d_out, int hidden, void* stream);
/* The same reduce for every token of a chunk in one launch, in place of the per-token launches
 * of run_moe_grouped_expert_batch (src/architecture/deepseek_v4/moe/moe_grouped_batch.hpp:136-146):
 * out[t][i] = half(float(out[t][i]) + sum_{s ascending} contrib[(t*slots + s)*hidden + i]), i.e.
 * each token's row (pitch out_stride elements) is its own fp16 starting value. hidden % 4 == 0. */
int aeon_moe_accumulate_fixed_order_tokens(const float* d_contrib, int tokens, int slots,
                                           void* d_out, int out_stride, int hidden, void* stream);
/* v4_swiglu_clamp_kernel launch, src/architecture/deepseek_v4/kernels/v4_swiglu_clamp.hpp:18-34. */
int aeon_swiglu_clamp(const void* d_gate, const void* d_up, void* d_out, int total_elements,
                      float limit, void* stream);

/* dispatch_aeon_moe_grouped_w13_swiglu_wmma<WAVES,RPW,LPR,MTILES>, src/architecture/deepseek_v4/
 * kernels/moe_grouped_dispatch.hpp:45-64 (kernel: src/platform/rdna3/moe_grouped_ffn.hpp:75-188,
 * feed: swizzled_w4a16_feed.hpp:51-140): per expert e of the 8-slot table, over positions
 * expert_offsets[e]..[e+1): expert_hidden[(e*expert_hidden_tokens + m)*N + n] =
 * half(clamped_swiglu(W1_e x, W3_e x)) with x = activation row token_indices[position], row
 * pitch activation_stride (0 = K). Weights dequantised to fp16 with one rounding per weight. */
int aeon_moe_grouped_w13_swiglu(const void* d_activation, const int* d_expert_offsets,
                                const int* d_token_indices, const aeon_w13_table* weights,
                                void* d_expert_hidden, int expert_count, int expert_hidden_tokens,
                                int N, int K, int rpw, int lpr, float swiglu_limit,
                                int activation_stride, void* stream);
/* dispatch_aeon_moe_grouped_w2_wmma, moe_grouped_dispatch.hpp:66-88 (kernel
 * moe_grouped_ffn.hpp:197-288): contrib[draw_indices[p]*N + n] = draw_weights[p] *
 * (W2_e . expert_hidden[e][m])[n], one writer per element. */
int aeon_moe_grouped_w2(const void* d_expert_hidden, const int* d_expert_offsets,
                        const int* d_draw_indices, const float* d_draw_weights,
                        const aeon_w2_table* weights, float* d_contrib, int expert_count,
                        int expert_hidden_tokens, int N, int K, int rpw, int lpr, void* stream);

/* ------------------------------------------------------------------------------------------
 * Decode kernels over the wave64 packing (the MI355X-native path)
 * ---------------------------------------------------------------------------------------- */

/* W4A16 GEMV over an A64 matrix: same arithmetic contract as
 * dispatch_aeon_w4a16_swizzled_gemv (aeon_w4a16_swizzled_gemv.hpp:43-93,166-190): the scale is
 * applied in fp32 to the dot product of each scale group. VALU only (no MFMA): 1 KiB coalesced wave loads, in-register nibble
 * dequant, K split across the waves of a workgroup and reduced by wave shuffles.
 * `tokens` activations [tokens][K] (row pitch x_stride elements) give [tokens][N] outputs
 * (pitch out_stride); 1 <= tokens <= 8. */
int aeon_a64_gemv(const void* d_x, int x_stride, const void* d_packed, const void* d_scale,
                  int scale_group, void* d_out, int out_stride, int tokens, int N, int K,
                  void* stream);
/* dispatch_aeon_w4a16_swizzled_dual_gemv (aeon_w4a16_swizzled_gemv.hpp:95-164,192-222) on A64:
 * two matrices, one activation read. */
int aeon_a64_dual_gemv(const void* d_x, int x_stride, const void* d_packed_a,
                       const void* d_scale_a, const void* d_packed_b, const void* d_scale_b,
                       int scale_group, void* d_out_a, void* d_out_b, int out_stride, int tokens,
                       int N, int K, void* stream);

/* One expert's six A64 sub-tensors (device pointers): the wave64 counterpart of the slot
 * views UnifiedVRAMExpertPool::get_w{1,2,3}_{packed,scale} return
 * (src/backend/swizzled_w4a16/core/vram_expert_pool.hpp:22-82). W1/W3 are [I][H], W2 [H][I]. */
typedef struct {
    const void* w1_packed;
    const void* w1_scale;
    const void* w3_packed;
    const void* w3_scale;
    const void* w2_packed;
    const void* w2_scale;
} aeon_a64_expert;

/* One routed expert over `tokens` (1..16) activations [tokens][H]: the per-token trio of
 * V4TieredExpertExecutor::accumulate_routed (src/architecture/deepseek_v4/moe/
 * v4_expert_executor.hpp:298-370) for a single slot -- fused gate+up dual-GEMV with the
 * clamped SwiGLU (hidden fp16 [tokens][I] into d_hidden), W2 with the routing weight
 * (contrib fp32 [tokens][H] into d_contrib = w[t]*acc), then the fixed-order reduce with one
 * slot: out[t] = half(float(shared[t]) + contrib[t]); d_shared nullable, may alias d_out.
 * use_mfma 0 = VALU GEMV kernels (tokens <= 8), 1 = the MFMA segment kernels. */
int aeon_a64_expert_decode(const void* d_x, int tokens, const aeon_a64_expert* expert,
                           int scale_group, const float* d_route_weights, void* d_hidden, float* d_contrib,
                           const void* d_shared, void* d_out, int H, int I, float swiglu_limit,
                           int use_mfma, void* stream);

/* ------------------------------------------------------------------------------------------
 * Router, permutation, and one MoE layer on the device
 * ---------------------------------------------------------------------------------------- */

#define AEON_ROUTER_SCORE_SQRT_SOFTPLUS 0 /* sqrt(softplus(x)), moe_router.hpp:17-27 */
#define AEON_ROUTER_SCORE_SIGMOID 1       /* 1/(1+exp(-x)) */

/* Router logits: logits[t][e] = sum_h float(x[t][h]) * Wr[h][e], Wr fp32 [hidden][experts].
 * Replaces the gate GEMV + widening of dispatch_router (src/architecture/deepseek_v4/layer/
 * v4_layer_body_moe.hpp:124-159, gemv_fp16_vec8_kernel in src/platform/ops/gemv.hpp:72-110)
 * for an fp32 gate. Accumulation order is fixed (h ascending inside a chunk, chunks ascending),
 * so a run is bit-reproducible. The workspace holds the per-chunk partial sums. */
size_t aeon_router_logits_workspace_bytes(int tokens, int hidden, int experts);
int aeon_router_logits(const void* d_x, int x_stride, const float* d_router_weight,
                       float* d_logits, int tokens, int hidden, int experts, void* d_workspace,
                       size_t workspace_bytes, void* stream);

/* The same logits from the gate as the checkpoint stores it: gemv_fp16_vec8_kernel + the
 * widening of dispatch_router (src/platform/ops/gemv.hpp:72-110, layer/v4_layer_body_moe.hpp:
 * 135-142). d_gate_weight fp16 [experts][hidden]; logits_half[t][e] = half(sum_h x[t][h] *
 * w[e][h]) (fp32 accumulate, one rounding) and logits[t][e] = float(logits_half[t][e]).
 * hidden % 128 == 0, experts % 16 == 0. */
int aeon_router_logits_f16(const void* d_x, int x_stride, const void* d_gate_weight,
                           void* d_logits_half, float* d_logits, int tokens, int hidden,
                           int experts, void* stream);

/* gemv_fp16_vec8_kernel launch, src/platform/ops/gemv.hpp:72-110, for `tokens` rows at once:
 * y[t][o] = half(sum_i x[t][i] * w[o][i]), w fp16 [out_dim][in_dim] row-major, fp32 accumulate.
 * in_dim % 128 == 0, out_dim % 16 == 0, x_stride % 8 == 0, y_stride % 4 == 0. */
int aeon_dense_gemv_f16(const void* d_x, int x_stride, const void* d_weight, void* d_y,
                        int y_stride, int tokens, int in_dim, int out_dim, void* stream);
/* run_layer_body_moe_shared_expert, layer/v4_layer_body_moe.hpp:216-256 (oracle: dense_ffn,
 * reference/dsv4_oracle.hpp:1708-1753), for `tokens` tokens in three launches: gate = half(W1 x)
 * and up = half(W3 x) into d_gate / d_up, hidden = half(clamped_swiglu(gate, up)) into d_hidden
 * (the reference's d_shared_gate / d_shared_up / d_shared_swiglu; each [tokens][intermediate]
 * fp16, caller's scratch), then out[t] = half(W2 . hidden) -- the stage roundings of the
 * reference's four launches (three GEMVs and v4_swiglu_clamp_kernel). The reference's memset of
 * the accumulator is not needed: every element of the `hidden` columns of the output rows is
 * written. intermediate % 128 == 0 and hidden % 128 == 0. */
int aeon_dense_shared_expert_f16(const void* d_x, int x_stride, int tokens, const void* d_w1,
                                 const void* d_w3, const void* d_w2, void* d_gate, void* d_up,
                                 void* d_hidden, void* d_out, int out_stride, int hidden,
                                 int intermediate, float swiglu_limit, void* stream);

/* moe_router_kernel launch (src/architecture/deepseek_v4/kernels/moe_router.hpp:104-189; host
 * twin cpu_moe_router :29-100): score = f(logit); choice = score + bias (bias added after the
 * activation, nullable); ids = top_k by descending choice, ties to the lowest index; weights =
 * unbiased score / (sum + 1e-20) [if renormalize] * routed_scaling_factor. With a hash table
 * ([vocab][top_k] int64) and token ids the ids come from the table instead (:146-153).
 * experts <= 1024, top_k <= 64. Scores and selection are evaluated in fp64. */
int aeon_moe_router(const float* d_logits, const float* d_bias, const int64_t* d_hash_table,
                    const int32_t* d_token_ids, float* d_topk_weights, int32_t* d_topk_indices,
                    int tokens, int experts, int top_k, float routed_scaling_factor,
                    int renormalize, int score_kind, void* stream);

/* dispatch_expert_permutation, src/platform/ops/expert_permutation.hpp:130-175: ids
 * [token_count*slots] -> expert_offsets [expert_count+1], token_indices and draw_indices
 * [token_count*slots] (ascending draw inside an expert), and optionally the weights gathered
 * into position order. expert_count <= 1024; ids outside [0, expert_count) are dropped. */
int aeon_expert_permutation(const int32_t* d_topk_indices, int token_count, int slots,
                            int expert_count, int32_t* d_expert_offsets, int32_t* d_token_indices,
                            int32_t* d_draw_indices, const float* d_weights_by_draw,
                            float* d_weights_by_position, void* stream);

/* One MoE layer with every expert resident in HBM in the wave64 packing. `d_experts` is a
 * DEVICE array of `experts` entries (+1 when has_shared: the last entry is the always-on
 * expert) -- a table in memory instead of the 8-entry by-value tables of
 * aeon_moe_fused_w13.hpp:13-20, so one launch can address every expert of the layer. */
typedef struct {
    int hidden;
    int intermediate;
    int experts;  /* routed experts */
    int top_k;
    int has_shared;
    float swiglu_limit;
    int score_kind;
    float routed_scaling_factor;
    int renormalize;
    const float* d_router_weight; /* fp32 [hidden][experts]; only aeon_moe_layer_decode reads it */
    const float* d_router_bias;   /* fp32 [experts], nullable */
    const aeon_a64_expert* d_experts;
    /* Columns per scale of every expert in the table, 128 or 32: the value the table's experts
     * were packed with (aeon_a64_repack_*, aeon_resident_load_layer, V4ResidentExpertPool::
     * scale_group()). The table itself carries no record of it and the two groupings differ in
     * stride, so there is no default: any other value, 0 included, is refused with
     * AEON_ERR_INVALID_ARGUMENT. */
    int scale_group;
    /* The real model's dense fp16 pieces (all optional, NULL = absent):
     * the router gate as the checkpoint stores it, fp16 [experts][hidden], read by
     * aeon_moe_layer_decode when d_router_weight is NULL -- logits are then rounded to fp16 and
     * widened, as dispatch_router does (layer/v4_layer_body_moe.hpp:135-142); and the shared
     * expert's three row-major fp16 matrices (w1, w3 [intermediate][hidden], w2
     * [hidden][intermediate]; run_layer_body_moe_shared_expert, :216-256). With has_shared == 0
     * and the three given, the step writes the shared expert's fp16 output into the output rows
     * first and the routed sum is added to it -- the reference's order. */
    const void* d_router_weight_f16;
    const void* d_shared_w1_f16;
    const void* d_shared_w3_f16;
    const void* d_shared_w2_f16;
} aeon_moe_layer;

size_t aeon_moe_layer_workspace_bytes(const aeon_moe_layer* layer, int max_tokens);

/* V4RoutedExpertExecutor::accumulate_routed_batch for resident experts
 * (src/architecture/deepseek_v4/layer/v4_layer_body_moe.hpp:76-105, production override
 * src/architecture/deepseek_v4/moe/v4_expert_executor.hpp:379-461) at decode batch sizes:
 * given the routed ids/weights [tokens][top_k] on the device, out[t] = half(shared(x_t) as fp16
 * + sum_k w[t][k] * expert_{ids[t][k]}(x_t)) in slot order, fp32. Without a shared expert the
 * value already in d_out is the fp16 starting value, as moe_accum is in the reference. Each
 * distinct expert's weights are streamed once per 16 of its tokens. No host synchronisation.
 * An id outside [0, experts) contributes nothing (the reference's permutation drops it,
 * src/platform/ops/expert_permutation.hpp:64-70; here the reduce leaves its slot out as well). */
int aeon_moe_layer_routed(const aeon_moe_layer* layer, const void* d_x, int x_stride, int tokens,
                          const int32_t* d_topk_ids, const float* d_topk_weights, void* d_out,
                          int out_stride, void* d_workspace, size_t workspace_bytes, void* stream);

/* The same step cut into its launches, for measurement: runs only the stages named in
 * stage_mask, on the state earlier stages left in the workspace (so AEON_STAGE_GATE_UP alone
 * can be repeated between two events once a full step has run with the same arguments). With
 * one or two tokens the permutation stage launches nothing: the expert stages read the ids and
 * weights directly. */
#define AEON_STAGE_PERMUTATION 1
#define AEON_STAGE_GATE_UP 2
#define AEON_STAGE_DOWN 4
#define AEON_STAGE_REDUCE 8
#define AEON_STAGE_DENSE_SHARED 16 /* the dense fp16 shared expert, when the layer has one */
#define AEON_STAGE_ALL 31
int aeon_moe_layer_routed_stages(const aeon_moe_layer* layer, const void* d_x, int x_stride,
                                 int tokens, const int32_t* d_topk_ids,
                                 const float* d_topk_weights, void* d_out, int out_stride,
                                 void* d_workspace, size_t workspace_bytes, int stage_mask,
                                 void* stream);

/* Router + aeon_moe_layer_routed: the device half of run_layer_body_router
 * (v4_layer_body_moe.hpp:168-202) followed by run_layer_body_moe_and_post's expert part
 * (:285-312), with the per-layer D2H read-back and stream synchronisation of :188-192 removed.
 * d_topk_ids / d_topk_weights [tokens][top_k] are outputs. */
int aeon_moe_layer_decode(const aeon_moe_layer* layer, const void* d_x, int x_stride, int tokens,
                          void* d_out, int out_stride, int32_t* d_topk_ids, float* d_topk_weights,
                          void* d_workspace, size_t workspace_bytes, void* stream);
/* The hyper-connection expansion that follows the routed experts in a layer body
 * (run_layer_body_moe_and_post, layer/v4_layer_body_moe.hpp:259-312: experts, reduce, hc_post),
 * for aeon_moe_layer_decode_hc_post. Streams are fp16, element (t, j, h) of a residual at
 * t*token_stride + j*stream_stride + h; post [4] and comb [16] (comb[i*4+j]) per token
 * (mix_per_token 1) or shared by all tokens (0); input and output residual must not alias.
 * d_next_pre_mix (nullable): the NEXT layer's pre-mix ([4], next_pre_token_stride 4 = per token,
 * 0 = shared) -- then the next layer's input, sum_j pre[j] * residual_out[t][j][h]
 * (hc_pre_combine_kernel, kernels/hc_sinkhorn.hpp:94-147), is written to d_next_layer_input
 * (row pitch next_input_stride elements) in the same pass. */
typedef struct {
    const void* d_residual_in;
    long token_stride;
    long stream_stride;
    const float* d_post_mix;
    const float* d_comb_mix;
    int mix_per_token;
    void* d_residual_out;
    const float* d_next_pre_mix;
    int next_pre_token_stride;
    void* d_next_layer_input;
    long next_input_stride;
} aeon_hc_post_args;
/* aeon_moe_layer_decode with the fixed-order reduce, aeon_hc_post and (optionally) the next
 * layer's aeon_hc_pre_combine done by ONE launch instead of three: d_out still receives the
 * layer output rows, hc->d_residual_out the expanded streams. Every value is rounded to fp16
 * where it would cross a kernel boundary in the three-launch sequence, so the results are that
 * sequence's, bit for bit. hidden % 8 == 0, out_stride % 8 == 0 and 16-byte aligned rows. */
int aeon_moe_layer_decode_hc_post(const aeon_moe_layer* layer, const void* d_x, int x_stride,
                                  int tokens, void* d_out, int out_stride, int32_t* d_topk_ids,
                                  float* d_topk_weights, const aeon_hc_post_args* hc,
                                  void* d_workspace, size_t workspace_bytes, void* stream);
/* aeon_moe_layer_decode with no workspace argument and no allocation. It has no counterpart in
 * the reference: it is for callers that cannot allocate device memory or carry a workspace --
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. The
 * workspace is a fixed array of AEON_NOALLOC_WORKSPACE_BYTES inside the library's code object
 * (every GPU the library runs on holds one copy until the process ends); the call launches the
 * same kernels as aeon_moe_layer_decode on it and calls no hipMalloc, hipFree, hipMemset or
 * allocating library routine. The first call on a device looks the array's address up once
 * (hipGetSymbolAddress, with that device current) and is best made before any capture.
 * Limit: aeon_moe_layer_workspace_bytes(layer, tokens) <= AEON_NOALLOC_WORKSPACE_BYTES (batch 64
 * at hidden 7168 / intermediate 2048 / top-8 of 256 experts + always-on expert needs 19.1 MiB);
 * beyond it the call returns AEON_ERR_INVALID_ARGUMENT and launches nothing.
 * All calls on one GPU share that GPU's array: two calls that overlap in time on one GPU (two
 * streams, two threads) race and must be serialised by the caller. Nothing in the array has to
 * start at zero -- every word a kernel of the step reads was written earlier in the same step --
 * so a call is not affected by what the previous one left behind. */
#define AEON_NOALLOC_WORKSPACE_BYTES (24u << 20)
int aeon_moe_layer_decode_noalloc(const aeon_moe_layer* layer, const void* d_x, int x_stride,
                                  int tokens, void* d_out, int out_stride, int32_t* d_topk_ids,
                                  float* d_topk_weights, void* stream);
/* Device pointer to the fp32 logits [tokens][experts] the last aeon_moe_layer_decode call with
 * this workspace and token count left behind (what the ids were selected from). */
const float* aeon_moe_layer_logits(const aeon_moe_layer* layer, int tokens, void* d_workspace);

/* ------------------------------------------------------------------------------------------
 * Hyper-connection stream mix (hc_mult = 4)
 * ---------------------------------------------------------------------------------------- */

/* hc_project_kernel launch, src/architecture/deepseek_v4/kernels/hc_sinkhorn.hpp:22-90 (call sites
 * layer/v4_layer_body_attention.hpp:101-104,127-132): the per-token dynamic mixes,
 * mixes[t][m] = rsqrt(mean(r_t^2) + rms_eps) * sum_k r_t[k] * fn[m][k] for m < 24, r_t the token's
 * flattened 4 x hidden residual (element (t, j, h) at t*token_stride + j*stream_stride + h, fp32
 * as in the reference or fp16), fn fp32 [24][4*hidden] with k = j*hidden + h. */
int aeon_hc_project(const void* d_residual, int residual_is_f32, long token_stride,
                    long stream_stride, const float* d_fn, float* d_mixes, int tokens, int hidden,
                    float rms_eps, void* stream);
/* rmsnorm_wave32_kernel / rmsnorm_unit_wave32_kernel, src/platform/ops/rmsnorm.hpp:35-105 (the FFN
 * norm site, v4_layer_body_attention.hpp:113-115): out[t][i] = half(x[t][i] *
 * rsqrt(mean(x[t]^2) + eps) * weight[i]); fp16 in, out and weight, fp32 arithmetic;
 * d_weight NULL = the weightless form. Row pitches in elements. */
int aeon_rmsnorm(const void* d_x, long x_stride, const void* d_weight, void* d_out,
                 long out_stride, int tokens, int dim, float eps, void* stream);
/* hc_sinkhorn_normalize_kernel launch, src/architecture/deepseek_v4/kernels/
 * hc_sinkhorn.hpp:151-255: mixes [tokens][24] -> pre [tokens][4] = sigmoid(m*s0+b)+pre_eps,
 * post [tokens][4] = sigmoid(m*s1+b)*post_alpha, comb [tokens][16] (comb[i*4+j], i the
 * contraction stream, j the output stream): row softmax + eps, column normalisation, then
 * (iters-1) x (row, column), every denominator + sinkhorn_eps. */
int aeon_hc_sinkhorn_normalize(const float* d_mixes, const float* d_hc_scale,
                               const float* d_hc_base, float* d_pre_mix, float* d_post_mix,
                               float* d_comb_mix, int tokens, float hc_pre_eps,
                               float hc_sinkhorn_eps, float hc_post_alpha, int sinkhorn_iters,
                               void* stream);
/* hc_pre_combine_kernel launch, hc_sinkhorn.hpp:94-147: layer_input[t][h] =
 * sum_j pre[j]*residual[t][j][h] -> fp16. The residual is fp32 (the reference's) or fp16, element
 * (t, j, h) at t*token_stride + j*stream_stride + h; pre_token_stride 4 = per-token mixes,
 * 0 = one mix for every token. */
int aeon_hc_pre_combine(const void* d_residual, int residual_is_f32, long token_stride,
                        long stream_stride, const float* d_pre_mix, int pre_token_stride,
                        void* d_layer_input, long out_stride, int tokens, int hidden,
                        void* stream);
/* hc_post_kernel launch, hc_sinkhorn.hpp:259-290: out[t][j][h] = post[j]*layer_out[t][h] +
 * sum_i comb[i*4+j]*residual_in[t][i][h], fp16 streams, fp32 math. mix_per_token 1 = post/comb
 * per token, 0 = shared by all tokens. Input and output residuals must not alias. */
int aeon_hc_post(const void* d_layer_out, long layer_out_stride, const void* d_residual_in,
                 long token_stride, long stream_stride, const float* d_post_mix,
                 const float* d_comb_mix, int mix_per_token, void* d_residual_out, int tokens,
                 int hidden, void* stream);

/* ------------------------------------------------------------------------------------------
 * `.aeon` expert container -> HBM-resident experts in the wave64 packing (load time)
 * ---------------------------------------------------------------------------------------- */

/* The expert half of AeonModelLoader (src/infrastructure/artifact/aeon_loader.hpp:318-470,
 * get_expert_location :145-160, get_expert_data :163-166): the index file is a 32-byte header
 * {"AEON_EXPERTS" (12 bytes), u32 version, u32 layers, u32 experts_per_layer, u64 payload_bytes}
 * followed by one {u64 offset, u64 length} entry per (layer, expert), layer-major
 * (scripts/convert_safetensors_to_aeon.py:463-486); the experts file is mapped read-only.
 * Rejected with AEON_ERR_IO, as the reference rejects them with std::runtime_error: missing or
 * short files, a wrong magic, a version other than `expected_version`, an entry whose length is
 * not payload_bytes or whose offset is not a multiple of `sector_size` or runs past the file. */
typedef struct aeon_expert_catalog aeon_expert_catalog;
int aeon_expert_catalog_open(const char* index_path, const char* experts_path,
                             uint32_t expected_version, uint32_t sector_size,
                             aeon_expert_catalog** out);
void aeon_expert_catalog_close(aeon_expert_catalog* catalog);
int aeon_expert_catalog_info(const aeon_expert_catalog* catalog, uint32_t* layers,
                             uint32_t* experts_per_layer, uint64_t* payload_bytes,
                             uint32_t* version);
/* Host pointer to one expert's payload inside the mapping (AEON_ERR_OUT_OF_RANGE for an index
 * outside the catalog). */
int aeon_expert_catalog_payload(const aeon_expert_catalog* catalog, uint32_t layer,
                                uint32_t expert, const void** payload, uint64_t* bytes);

/* Byte offsets of the six sub-tensors inside one `.aeon` expert payload for an expert of shape
 * (hidden, intermediate): [W1 packed | W1 scale | W2 packed | W2 scale | W3 packed | W3 scale],
 * group-32 fp16 scales, no padding -- the order and sizes of
 * src/backend/swizzled_w4a16/core/swizzled_expert_format.hpp:11-30 (AEON_W1_PACKED_OFFSET ...
 * AEON_SWIZZLED_EXPERT_BYTES), which are this function at (4096, 2048). */
typedef struct {
    size_t w1_packed, w1_scale, w2_packed, w2_scale, w3_packed, w3_scale, total;
} aeon_payload_layout;
int aeon_payload_layout_for(int hidden, int intermediate, aeon_payload_layout* out);

/* One resident expert slot in the wave64 packing: bytes per slot (a multiple of 4096) and the
 * six device views of the slot at `d_slot` -- the counterpart of UnifiedVRAMExpertPool's slot
 * views (src/backend/swizzled_w4a16/core/vram_expert_pool.hpp:22-82) with every expert
 * resident. */
size_t aeon_a64_slot_bytes(int hidden, int intermediate, int scale_group);
int aeon_a64_slot_views(void* d_slot, int hidden, int intermediate, int scale_group,
                        aeon_a64_expert* out);

/* Loads experts [first, first+count) of `layer` into consecutive slots of `d_pool` (slot i at
 * d_pool + i*aeon_a64_slot_bytes): payload bytes are copied from the mapping to a device staging
 * buffer and re-swizzled there into the wave64 packing, copy and repack of neighbouring experts
 * overlapped on two streams of the library's own. `h_table[i]` receives
 * the views of slot i (host array; copy it to the device as the layer's expert table).
 * Blocks until the pool is complete. scale_group 32 keeps every scale of the container (the
 * choice for a real checkpoint); with 128 a payload whose four group-32 scales differ anywhere
 * inside 128 columns makes the call fail with AEON_ERR_INVALID_ARGUMENT (the pool is then not to
 * be used), never a pool that computes with the wrong weights. */
int aeon_resident_load_layer(const aeon_expert_catalog* catalog, uint32_t layer, uint32_t first,
                             uint32_t count, int hidden, int intermediate, int scale_group,
                             void* d_pool, size_t pool_bytes, aeon_a64_expert* h_table);

/* ------------------------------------------------------------------------------------------
 * Synthetic experts on the device (benchmarks and tests)
 * ---------------------------------------------------------------------------------------- */

/* Fills one matrix (matrix 0 = W1, 1 = W3, 2 = W2) of synthetic expert `expert` directly in
 * device memory in the `.aeon` swizzled layout (packed N*K/2 bytes, scales N*K/32 fp16): int4
 * uniform in [-8,7], scales uniform in [0.005,0.02] -- with scale_group 128 one per (row, 128
 * columns) replicated over its four group-32 slots, with 32 one of its own per slot -- a pure
 * function of (seed, expert, matrix, index). */
int aeon_synth_matrix_swizzled(uint64_t seed, int expert, int matrix, int N, int K, int rpw,
                               int lpr, int scale_group, void* d_packed, void* d_scale,
                               void* stream);

#ifdef __cplusplus
}
#endif
#endif
