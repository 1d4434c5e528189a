// Token -> expert permutation (a stable counting sort of the (token, slot) draws by expert id)
// and the segment list the decode kernels walk.
//
// Definition kept from the reference primitive: expert e owns positions
// offsets[e] .. offsets[e+1); inside an expert the draws appear in ascending draw index, so the
// placement is a pure function of the ids; an id outside [0, experts) is dropped.
// Histogram + scan run in one workgroup (LDS atomics on integers, so the totals do not depend
// on arrival order). The placement of a draw is its list's offset + the number of earlier draws
// of the same expert, found per chunk of 1024 draws (per-wave counts + a walk over the wave's
// own 64 draws) plus, for later chunks, a count of the chunks before: parallel over the draws,
// deterministic, and without the O(experts x draws) single-thread walk.
#include "permutation.hpp"

namespace aeon355 {

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const int other = __shfl_up(v, offset, 64);
        if (lane >= offset) v += other;
    }
    return v;
}

// Exclusive scan of one value per thread across a 1024-thread workgroup.
// Three scans in one: a list's position count (bits 0..23), its full segments (24..43) and its
// short one (44..63) ride in one 64-bit word, so the segment list costs no barriers of its own.
__device__ __forceinline__ unsigned long long block_exclusive_scan3(unsigned long long v,
                                                                    unsigned long long* wave_totals,
                                                                    unsigned long long* total) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    unsigned long long inclusive = v;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const unsigned long long other = __shfl_up(inclusive, offset, 64);
        if (lane >= offset) inclusive += other;
    }
    if (lane == 63) wave_totals[wave] = inclusive;
    __syncthreads();
    if (wave == 0) {
        const unsigned long long t = lane < 16 ? wave_totals[lane] : 0ull;
        unsigned long long scanned = t;
#pragma unroll
        for (int offset = 1; offset < 16; offset <<= 1) {
            const unsigned long long other = __shfl_up(scanned, offset, 64);
            if (lane >= offset) scanned += other;
        }
        if (lane < 16) wave_totals[lane] = scanned - t;
        if (lane == 15) *total = scanned;
    }
    __syncthreads();
    return inclusive - v + wave_totals[wave];
}

// A batch of at most this many draws is scattered by the workgroup that counts it (one launch
// instead of two: a decode step is short enough for a launch to show). Larger batches are
// scattered in chunks of this many draws, one workgroup each.
constexpr int kFusedScatterDraws = 1024;
constexpr int kWaveCountWords = (kFusedScatterDraws / 64) * (kMaxPermutationExperts + 1) / 2 + 1;

// Stable rank of each of a 1024-thread workgroup's draws among the workgroup's draws of the same
// expert: thread i holds draw i of the chunk (`mine` = its expert, -1 for none), wave w the draws
// 64w..64w+63. The earlier waves' share comes from per-wave counts in LDS (`wave_count`, zeroed
// here), the share of the lower lanes from the set of the wave's lanes with the same expert. Ends
// with the workgroup synchronised.
__device__ __forceinline__ int rank_in_chunk(int mine, int lists, uint32_t* wave_count_words) {
    unsigned short* wave_count = reinterpret_cast<unsigned short*>(wave_count_words);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < (16 * lists + 1) / 2; i += blockDim.x) wave_count_words[i] = 0;
    __syncthreads();
    // the lanes of the wave that hold the same list: one ballot per bit of the id (a list index
    // is at most kMaxPermutationExperts, 11 bits) and one for "no draw"
    static_assert(kMaxPermutationExperts < (1 << 11), "the ballots cover 11 bits of a list index");
    unsigned long long same = ~0ull;
#pragma unroll
    for (int b = 0; b <= 11; ++b) {
        const bool set = b < 11 ? ((mine >> b) & 1) != 0 : mine < 0;
        const unsigned long long ballot = __ballot(set);
        same &= set ? ballot : ~ballot;
    }
    int rank = __popcll(same & ((1ull << lane) - 1ull));
    const int later = __popcll(same & ~((2ull << lane) - 1ull));
    // the last lane of an expert in the wave knows the wave's count for it
    if (mine >= 0 && later == 0) wave_count[wave * lists + mine] = static_cast<unsigned short>(rank + 1);
    __syncthreads();
    if (mine >= 0) {
        for (int w = 0; w < wave; ++w) rank += wave_count[w * lists + mine];
    }
    return rank;
}

template <bool SCATTER>
__global__ __launch_bounds__(1024) void permutation_offsets_kernel(PermutationArgs a) {
    __shared__ int histogram[kMaxPermutationExperts + 1];
    __shared__ unsigned long long wave_totals[16];
    __shared__ unsigned long long total;
    __shared__ int draw_expert[SCATTER ? kFusedScatterDraws : 1];
    const int lists = a.experts + (a.shared_tokens > 0 ? 1 : 0);
    for (int e = threadIdx.x; e <= kMaxPermutationExperts; e += blockDim.x) histogram[e] = 0;
    __syncthreads();
    for (int d = threadIdx.x; d < a.draws; d += blockDim.x) {
        const int e = a.ids[d];
        const bool valid = e >= 0 && e < a.experts;
        if (valid) atomicAdd(&histogram[e], 1);
        if (SCATTER) draw_expert[d] = valid ? e : -1;
    }
    if (threadIdx.x == 0 && a.shared_tokens > 0) histogram[a.experts] = a.shared_tokens;
    __syncthreads();

    const int e = threadIdx.x;
    const int count = e < lists ? histogram[e] : 0;
    // Segments that are more than half full come first in the list, the short ones after
    // them: the launches walk the list in order, so the costliest workgroups are dispatched
    // first and the launch's tail is made of cheap ones.
    const bool with_segments = a.seg_expert != nullptr;
    const int segments = with_segments ? (count + a.seg_tokens - 1) / a.seg_tokens : 0;
    const int last_count = count - (segments - 1) * a.seg_tokens;
    const int light = segments > 0 && 2 * last_count <= a.seg_tokens ? 1 : 0;
    const int heavy = segments - light;
    // One 64-bit scan carries three sums: positions in bits 0..23, heavy segments in 24..43,
    // light ones from 44 up (launch_permutation refuses totals that would carry from one field
    // into the next). Without a segment list the position count has the whole word.
    const unsigned long long packed = static_cast<unsigned long long>(count) |
                                      (static_cast<unsigned long long>(heavy) << 24) |
                                      (static_cast<unsigned long long>(light) << 44);
    const unsigned long long before = block_exclusive_scan3(packed, wave_totals, &total);
    const unsigned long long sums = total;
    const unsigned long long count_field = with_segments ? 0xFFFFFFull : ~0ull;
    const int offset = static_cast<int>(before & count_field);
    if (e < lists) a.offsets[e] = offset;
    if (e == 0) a.offsets[lists] = static_cast<int>(sums & count_field);

    if (with_segments) {
        const int heavy_base = static_cast<int>((before >> 24) & 0xFFFFFull);
        const int light_base = static_cast<int>(before >> 44);
        const int heavy_total = static_cast<int>((sums >> 24) & 0xFFFFFull);
        const int all = heavy_total + static_cast<int>(sums >> 44);
        for (int s = 0; s < segments; ++s) {
            const int at = s < heavy ? heavy_base + s : heavy_total + light_base;
            if (at < a.seg_capacity) {
                a.seg_expert[at] = e;
                a.seg_first[at] = offset + s * a.seg_tokens;
                a.seg_count[at] = min(a.seg_tokens, count - s * a.seg_tokens);
                if (a.seg_alone != nullptr) a.seg_alone[at] = segments == 1 ? 1 : 0;
            }
        }
        if (e == 0) *a.seg_total = min(all, a.seg_capacity);
    }

    if (SCATTER) {
        // Draw d goes to its list's offset plus the number of earlier draws of the same expert
        // (ascending draw order inside a list).
        __shared__ uint32_t wave_count_words[kWaveCountWords];
        __syncthreads();
        if (e < lists) histogram[e] = offset;
        const int d = threadIdx.x;
        const int mine = d < a.draws ? draw_expert[d] : -1;
        const int rank = rank_in_chunk(mine, lists, wave_count_words);
        if (mine >= 0) {
            const int at = histogram[mine] + rank;
            a.token_indices[at] = d / a.slots;
            a.draw_indices[at] = d;
            if (a.weights_by_position != nullptr) a.weights_by_position[at] = a.weights_by_draw[d];
        }
        if (a.shared_tokens > 0) {
            const int base = histogram[a.experts];
            for (int t = threadIdx.x; t < a.shared_tokens; t += blockDim.x) {
                a.token_indices[base + t] = t;
                a.draw_indices[base + t] = a.draws + t;
                if (a.weights_by_position != nullptr) a.weights_by_position[base + t] = 1.0f;
            }
        }
    }
}

// Scatter of a large batch: workgroup c places draws 1024c..1024c+1023. A draw goes to its
// list's offset + the draws of the same expert in earlier chunks (counted here from the ids, an
// LDS histogram: counts do not depend on the order of the adds) + its stable rank inside the
// chunk. The workgroups past the last chunk write the always-on expert's list, which takes
// every token once, in token order, with weight 1 and its own output rows.
__global__ __launch_bounds__(1024) void permutation_scatter_kernel(PermutationArgs a) {
    __shared__ int before[kMaxPermutationExperts + 1];
    __shared__ uint32_t wave_count_words[kWaveCountWords];
    const int chunks = (a.draws + kFusedScatterDraws - 1) / kFusedScatterDraws;
    const int chunk = blockIdx.x;
    if (chunk >= chunks) {
        const int base = a.offsets[a.experts];
        for (int t = (chunk - chunks) * blockDim.x + threadIdx.x; t < a.shared_tokens;
             t += (gridDim.x - chunks) * blockDim.x) {
            a.token_indices[base + t] = t;
            a.draw_indices[base + t] = a.draws + t;
            if (a.weights_by_position != nullptr) a.weights_by_position[base + t] = 1.0f;
        }
        return;
    }
    const int lists = a.experts + (a.shared_tokens > 0 ? 1 : 0);
    for (int e = threadIdx.x; e < lists; e += blockDim.x) before[e] = 0;
    __syncthreads();
    const int first = chunk * kFusedScatterDraws;
    for (int d = threadIdx.x; d < first; d += blockDim.x) {
        const int e = a.ids[d];
        if (e >= 0 && e < a.experts) atomicAdd(&before[e], 1);
    }
    const int d = first + threadIdx.x;
    int mine = d < a.draws ? a.ids[d] : -1;
    if (mine < 0 || mine >= a.experts) mine = -1;  // out-of-range ids are dropped, not trusted
    const float weight = mine >= 0 && a.weights_by_draw != nullptr ? a.weights_by_draw[d] : 0.0f;
    const int rank = rank_in_chunk(mine, lists, wave_count_words);  // synchronises: `before` is complete
    if (mine >= 0) {
        const int at = a.offsets[mine] + before[mine] + rank;
        a.token_indices[at] = a.slots_reciprocal != 0
                                  ? static_cast<int>(__umulhi(static_cast<unsigned>(d), a.slots_reciprocal))
                                  : d / a.slots;
        a.draw_indices[at] = d;
        if (a.weights_by_position != nullptr) a.weights_by_position[at] = weight;
    }
}

int launch_permutation(const PermutationArgs& args, hipStream_t stream) {
    PermutationArgs a = args;
    if (a.seg_expert != nullptr) {
        // the packed scan of the offsets kernel: 24 bits of positions, 20 of segments per class
        const long long positions = static_cast<long long>(a.draws) + a.shared_tokens;
        const long long lists = a.experts + (a.shared_tokens > 0 ? 1 : 0);
        AEON_REQUIRE(a.seg_tokens > 0 && positions < (1ll << 24) &&
                         positions / a.seg_tokens + lists < (1ll << 20),
                     AEON_ERR_INVALID_ARGUMENT,
                     "permutation with a segment list: %lld positions in segments of %d exceed the "
                     "2^24 positions / 2^20 segments one launch orders; split the chunk",
                     positions, a.seg_tokens);
    }
    a.slots_reciprocal = 0;
    if (a.slots > 1 && static_cast<uint64_t>(a.draws) * a.slots < (1ull << 32)) {
        a.slots_reciprocal = static_cast<unsigned>(((1ull << 32) + a.slots - 1) / a.slots);
    }
    if (a.draws <= kFusedScatterDraws) {
        permutation_offsets_kernel<true><<<1, 1024, 0, stream>>>(a);
        AEON_LAUNCH_CHECK();
        return AEON_OK;
    }
    permutation_offsets_kernel<false><<<1, 1024, 0, stream>>>(a);
    AEON_LAUNCH_CHECK();
    const int chunks = (a.draws + kFusedScatterDraws - 1) / kFusedScatterDraws;
    const int shared_groups = a.shared_tokens > 0 ? (a.shared_tokens + 4095) / 4096 : 0;
    permutation_scatter_kernel<<<chunks + shared_groups, 1024, 0, stream>>>(a);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_expert_permutation(const int32_t* d_topk_indices, int token_count, int slots,
                                       int expert_count, int32_t* d_expert_offsets,
                                       int32_t* d_token_indices, int32_t* d_draw_indices,
                                       const float* d_weights_by_draw,
                                       float* d_weights_by_position, void* stream) {
    const char* who = "aeon_expert_permutation";
    AEON_REQUIRE(d_topk_indices && d_expert_offsets && d_token_indices && d_draw_indices,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(token_count >= 0 && slots > 0 &&
                     static_cast<long long>(token_count) * slots < (1ll << 31),
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad draw shape (tokens=%d slots=%d)", who,
                 token_count, slots);
    AEON_REQUIRE(expert_count > 0 && expert_count <= kMaxPermutationExperts,
                 AEON_ERR_INVALID_ARGUMENT, "%s: expert count out of range", who);
    AEON_REQUIRE((d_weights_by_draw == nullptr) == (d_weights_by_position == nullptr),
                 AEON_ERR_INVALID_ARGUMENT,
                 "%s: weights need both a source and a destination", who);
    PermutationArgs a{};
    a.ids = d_topk_indices;
    a.draws = token_count * slots;
    a.slots = slots;
    a.experts = expert_count;
    a.offsets = d_expert_offsets;
    a.token_indices = d_token_indices;
    a.draw_indices = d_draw_indices;
    a.weights_by_draw = d_weights_by_draw;
    a.weights_by_position = d_weights_by_position;
    return launch_permutation(a, as_stream(stream));
}
