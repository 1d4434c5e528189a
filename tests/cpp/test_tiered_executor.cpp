// Gate: the two-tier executor (HBM slots over pinned host copies) behind the
// V4RoutedExpertExecutor seam against the all-resident executor on the same synthetic experts:
// three layers of twelve experts served from eight HBM slots, so every layer evicts. The
// reference's gate of its tiered executor needs the real model (tests/test_v4_expert_executor.cpp:139);
// what it asserts there is asserted here on synthetic payloads: the same bits as the control
// (:275-353), the chunk form one deduplicated dispatch (:403-430), and the capacity fallback
// counted instead of thrown when the leases of a token exceed the pool (forced by a small pool,
// the way an 8-slot pool forces it there).
#include "architecture/deepseek_v4/moe/v4_resident_expert_executor.hpp"
#include "architecture/deepseek_v4/moe/v4_tiered_expert_executor.hpp"
#include "common.hpp"
#include "test_device.hpp"

#include <cstring>

namespace core = aeon::core;

constexpr int kHidden = 4096, kIntermediate = 2048, kSlots = 6, kExperts = 12, kLayers = 3, kTokens = 5;
constexpr int kHotSlots = 8, kScaleGroup = 128;
constexpr float kLimit = 10.0f;

// One expert as a slot image in device memory: synthetic `.aeon` payload -> wave64 packing.
static void* make_slot_image(int id, size_t slot_bytes, aeon_a64_expert* views) {
    void* slot = nullptr;
    GATE_HIP(hipMalloc(&slot, slot_bytes));
    aeon355::throw_on_error(aeon_a64_slot_views(slot, kHidden, kIntermediate, kScaleGroup, views));
    const void* dst[3][2] = {{views->w1_packed, views->w1_scale}, {views->w3_packed, views->w3_scale},
                             {views->w2_packed, views->w2_scale}};
    const int shape[3][4] = {{kIntermediate, kHidden, 4, 8}, {kIntermediate, kHidden, 4, 8}, {kHidden, kIntermediate, 8, 4}};
    for (int m = 0; m < 3; ++m) {
        void *packed = nullptr, *scale = nullptr;
        const size_t words = static_cast<size_t>(shape[m][0]) * shape[m][1] / 8;
        GATE_HIP(hipMalloc(&packed, words * 4));
        GATE_HIP(hipMalloc(&scale, static_cast<size_t>(shape[m][0]) * shape[m][1] / 32 * 2));
        aeon355::throw_on_error(aeon_synth_matrix_swizzled(91, id, m, shape[m][0], shape[m][1], shape[m][2],
                                                           shape[m][3], 128, packed, scale, nullptr));
        aeon355::throw_on_error(aeon_a64_repack_device(packed, scale, shape[m][0], shape[m][1], shape[m][2],
                                                       shape[m][3], kScaleGroup, const_cast<void*>(dst[m][0]),
                                                       const_cast<void*>(dst[m][1]), nullptr, nullptr));
        GATE_HIP(hipDeviceSynchronize());
        GATE_HIP(hipFree(packed));
        GATE_HIP(hipFree(scale));
    }
    return slot;
}

static bool same_bits(const half* a, const half* b, size_t n) {
    const std::vector<half> x = to_host(a, n), y = to_host(b, n);
    return std::memcmp(x.data(), y.data(), n * sizeof(half)) == 0;
}

int main() {
    aeon::test::select_test_device(true);
    const size_t slot_bytes = aeon_a64_slot_bytes(kHidden, kIntermediate, kScaleGroup);
    core::V4WarmExpertStore warm(kLayers, kExperts, kHidden, kIntermediate, kScaleGroup);
    std::vector<aeon_moe_layer> layers(kLayers);
    for (int l = 0; l < kLayers; ++l) {
        std::vector<aeon_a64_expert> table(kExperts);
        for (int e = 0; e < kExperts; ++e) {
            void* slot = make_slot_image(100 * l + e, slot_bytes, &table[e]);
            warm.store(l, e, slot);  // the control keeps reading the device copy
        }
        layers[l] = aeon_moe_layer{kHidden, kIntermediate, kExperts, kSlots, 0, kLimit, AEON_ROUTER_SCORE_SIGMOID,
                                   1.0f, 1, nullptr, nullptr, to_device(table), kScaleGroup};
    }
    core::V4TierStreams streams;
    GATE_HIP(hipStreamCreateWithFlags(&streams.compute, hipStreamNonBlocking));
    GATE_HIP(hipStreamCreateWithFlags(&streams.upload, hipStreamNonBlocking));
    core::V4HotExpertSlots hot(warm, kHotSlots);
    core::V4HbmTieredExpertExecutor tiered(warm, hot, layers, 16, streams);
    core::V4ResidentExpertExecutor resident(layers, 16, streams.compute);

    SplitMix rng{0x9A17ED0Bull};
    std::vector<half> x(static_cast<size_t>(kTokens) * kHidden), shared(static_cast<size_t>(kTokens) * kHidden);
    for (half& v : x) v = __float2half(static_cast<float>(rng.uniform() - 0.5));
    for (half& v : shared) v = __float2half(static_cast<float>(rng.uniform() - 0.5));
    half* d_x = to_device(x);
    const size_t row = kHidden;

    // --- per-token decode over all layers, leases handed back at each token boundary ---------
    // Run in both regimes: a pool that holds a token's 18 leases (20 slots: hits, evictions, no
    // drain) and one that does not (8 slots: the capacity fallback).
    auto decode = [&](core::V4HbmTieredExpertExecutor& executor, size_t capacity, bool* leases_ok) {
        bool bits = true;
        *leases_ok = true;
        for (int t = 0; t < kTokens; ++t) {
            for (int l = 0; l < kLayers; ++l) {
                std::vector<int32_t> ids;
                std::vector<float> w;
                for (int k = 0; k < kSlots; ++k) {
                    // six distinct ids: 7k mod 12 visits six different residues
                    ids.push_back((5 * t + 7 * k + 3 * l) % kExperts);
                    w.push_back(0.6f / static_cast<float>(k + 1) + 0.02f);
                }
                float* d_w = to_device(w);
                half* out_t = to_device(std::vector<half>(shared.begin() + t * row, shared.begin() + (t + 1) * row));
                half* out_r = to_device(std::vector<half>(shared.begin() + t * row, shared.begin() + (t + 1) * row));
                executor.on_routing_ready(l, t, ids, w);
                executor.accumulate_routed(l, t, d_x + t * row, d_w, out_t);
                executor.on_routed_consumed(l, t);
                resident.on_routing_ready(l, t, ids, w);
                resident.accumulate_routed(l, t, d_x + t * row, d_w, out_r);
                GATE_HIP(hipStreamSynchronize(streams.compute));
                bits = bits && same_bits(out_t, out_r, row);
                GATE_HIP(hipFree(d_w));
                GATE_HIP(hipFree(out_t));
                GATE_HIP(hipFree(out_r));
            }
            *leases_ok = *leases_ok && executor.outstanding_leases() <= capacity;
            GATE_HIP(hipStreamSynchronize(streams.compute));  // the token boundary
            executor.release_leases();
            *leases_ok = *leases_ok && executor.outstanding_leases() == 0;
        }
        const core::V4TierCounters c = executor.counters();
        std::printf("  decode, %zu slots: %llu hot hits, %llu uploads (%.1f MB), %llu evictions, %llu forced drains\n",
                    capacity, static_cast<unsigned long long>(c.hot_hits),
                    static_cast<unsigned long long>(c.warm_uploads), c.upload_bytes / 1e6,
                    static_cast<unsigned long long>(c.evictions), static_cast<unsigned long long>(c.forced_drains));
        return bits;
    };
    {
        core::V4HotExpertSlots roomy(warm, 20);
        core::V4HbmTieredExpertExecutor executor(warm, roomy, layers, 16, streams);
        bool leases_ok = false;
        const bool bits = decode(executor, 20, &leases_ok);
        const core::V4TierCounters c = executor.counters();
        expect(bits, "20 slots, per-token form: the same bits as the all-resident executor, every layer of every token");
        expect(c.hot_hits > 0 && c.evictions > 0 && c.warm_uploads > 20,
               "36 experts through 20 slots: some found resident, some evicted");
        expect(c.hot_hits + c.warm_uploads == static_cast<uint64_t>(kTokens) * kLayers * kSlots,
               "every routed expert was answered by exactly one tier");
        expect(c.forced_drains == 0 && leases_ok, "a pool that holds a token's leases never drains");

        // The same walk with no host synchronisation anywhere -- the leases go back at a token
        // "boundary" the compute stream has not reached -- so every eviction's copy is enqueued
        // while kernels that read the victim may still be queued: the upload stream's wait on
        // the compute stream's position is all that keeps them apart.
        std::vector<half*> outs_t, outs_r;
        std::vector<float*> ws;
        for (int t = 0; t < kTokens; ++t) {
            for (int l = 0; l < kLayers; ++l) {
                std::vector<int32_t> ids;
                std::vector<float> w;
                for (int k = 0; k < kSlots; ++k) {
                    ids.push_back((7 * t + 7 * k + 5 * l + 1) % kExperts);
                    w.push_back(0.4f / static_cast<float>(k + 1) + 0.05f);
                }
                ws.push_back(to_device(w));
                outs_t.push_back(to_device(std::vector<half>(shared.begin() + t * row, shared.begin() + (t + 1) * row)));
                outs_r.push_back(to_device(std::vector<half>(shared.begin() + t * row, shared.begin() + (t + 1) * row)));
                executor.on_routing_ready(l, 50 + t, ids, w);
                executor.accumulate_routed(l, 50 + t, d_x + t * row, ws.back(), outs_t.back());
                resident.on_routing_ready(l, 50 + t, ids, w);
                resident.accumulate_routed(l, 50 + t, d_x + t * row, ws.back(), outs_r.back());
            }
            executor.release_leases();
        }
        GATE_HIP(hipStreamSynchronize(streams.compute));
        bool unsynchronised_bits = true;
        for (size_t i = 0; i < outs_t.size(); ++i) unsynchronised_bits = unsynchronised_bits && same_bits(outs_t[i], outs_r[i], row);
        expect(unsynchronised_bits && executor.counters().evictions > c.evictions,
               "no host synchronisation between layers or tokens, evictions on the way: still the same bits");
    }
    bool leases_counted = false;
    const bool token_bits = decode(tiered, kHotSlots, &leases_counted);
    const core::V4TierCounters after_decode = tiered.counters();
    expect(token_bits, "8 slots, per-token form: the same bits as the all-resident executor");
    expect(after_decode.warm_uploads > kHotSlots && after_decode.evictions > 0,
           "the run evicted: more uploads than the pool has slots");
    expect(after_decode.hot_hits + after_decode.warm_uploads == static_cast<uint64_t>(kTokens) * kLayers * kSlots,
           "every routed expert was answered by exactly one tier");
    expect(after_decode.forced_drains > 0 && leases_counted,
           "a token's 18 leases over 8 slots: the capacity fallback ran and was counted, nothing threw");

    // --- the chunk form: one deduplicated dispatch per layer --------------------------------
    bool chunk_bits = true, dedup = true;
    for (int l = 0; l < kLayers; ++l) {
        std::vector<std::vector<int32_t>> ids(kTokens);
        std::vector<std::vector<float>> w(kTokens);
        std::vector<int32_t> flat_ids;
        std::vector<float> flat_w;
        for (int t = 0; t < kTokens; ++t)
            for (int k = 0; k < kSlots; ++k) {
                // the chunk's tokens share eight experts: the union fits the pool
                ids[t].push_back((t + k + 2 * l) % 8 + (l % 2) * 4);
                w[t].push_back(0.5f / static_cast<float>(k + 1) + 0.03f);
                flat_ids.push_back(ids[t].back());
                flat_w.push_back(w[t].back());
            }
        int* d_ids = to_device(flat_ids);
        float* d_w = to_device(flat_w);
        half* out_t = to_device(shared);
        half* out_r = to_device(shared);
        tiered.on_routing_ready_batch(l, 200, ids, w);
        dedup = dedup && tiered.last_dispatch_tokens() == kTokens && tiered.last_dispatch_experts() == 8;
        tiered.accumulate_routed_batch(l, 200, kTokens, d_x, kHidden, d_ids, kSlots, d_w, kSlots, out_t, kHidden);
        resident.on_routing_ready_batch(l, 200, ids, w);
        resident.accumulate_routed_batch(l, 200, kTokens, d_x, kHidden, d_ids, kSlots, d_w, kSlots, out_r, kHidden);
        GATE_HIP(hipStreamSynchronize(streams.compute));
        chunk_bits = chunk_bits && same_bits(out_t, out_r, static_cast<size_t>(kTokens) * row);
        tiered.release_leases();
    }
    expect(chunk_bits, "chunk form: the same bits as the all-resident executor");
    expect(dedup && tiered.batch_distinct() < tiered.batch_draws(),
           "a chunk is one dispatch over its distinct experts (30 draws, 8 leases)");

    // --- a stale slot must not survive: the expert evicted longest ago is uploaded again ----
    {
        const core::V4TierCounters before = tiered.counters();
        std::vector<int32_t> ids = {0, 1, 2, 3, 4, 5};
        std::vector<float> w(kSlots, 0.25f);
        float* d_w = to_device(w);
        half* out_t = to_device(std::vector<half>(shared.begin(), shared.begin() + row));
        half* out_r = to_device(std::vector<half>(shared.begin(), shared.begin() + row));
        // layer 0 has not been touched since the first chunk; layers 1 and 2 took the pool over
        tiered.on_routing_ready(0, 300, ids, w);
        tiered.accumulate_routed(0, 300, d_x, d_w, out_t);
        resident.on_routing_ready(0, 300, ids, w);
        resident.accumulate_routed(0, 300, d_x, d_w, out_r);
        GATE_HIP(hipStreamSynchronize(streams.compute));
        expect(same_bits(out_t, out_r, row) && tiered.counters().warm_uploads > before.warm_uploads,
               "experts that lost their slots are copied up again, not read from what replaced them");
        tiered.release_leases();
    }

    // --- protocol errors, the reference's types (v4_expert_executor.hpp:302-315,403-415) ----
    bool logic = false, range = false, shape = false, wide = false, layer_range = false;
    try { tiered.accumulate_routed(1, 7, d_x, nullptr, nullptr); } catch (const std::logic_error&) { logic = true; }
    try {
        tiered.on_routing_ready(1, 7, std::vector<int32_t>{0, 1, 2, 3, 4, 5}, std::vector<float>(kSlots, 1.0f));
        tiered.accumulate_routed(1, 9, d_x, nullptr, nullptr);
    } catch (const std::out_of_range&) { range = true; }
    tiered.release_leases();
    try {
        tiered.on_routing_ready(0, 0, std::vector<int32_t>(kSlots - 1, 0), std::vector<float>(kSlots - 1, 1.0f));
    } catch (const std::invalid_argument&) { shape = true; }
    try {
        // two tokens whose union is twelve experts: more than the pool holds at once
        tiered.on_routing_ready_batch(0, 0, {{0, 1, 2, 3, 4, 5}, {6, 7, 8, 9, 10, 11}},
                                      {std::vector<float>(kSlots, 1.0f), std::vector<float>(kSlots, 1.0f)});
    } catch (const std::invalid_argument&) { wide = true; }
    try {
        tiered.on_routing_ready(kLayers, 0, std::vector<int32_t>{0, 1, 2, 3, 4, 5}, std::vector<float>(kSlots, 1.0f));
    } catch (const std::out_of_range&) { layer_range = true; }
    expect(logic, "consume without a matching announcement throws std::logic_error");
    expect(range, "token index past the batch throws std::out_of_range");
    expect(shape, "ids not [token, top_k] throws std::invalid_argument");
    expect(wide, "a chunk over more distinct experts than the pool has slots is refused, not truncated");
    expect(layer_range, "a layer outside the store throws std::out_of_range");
    bool no_slots = false, few_slots = false;
    try { core::V4HotExpertSlots none(warm, 0); } catch (const std::invalid_argument&) { no_slots = true; }
    try {
        core::V4HotExpertSlots four(warm, 4);
        core::V4HbmTieredExpertExecutor small(warm, four, layers, 16, streams);
    } catch (const std::invalid_argument&) { few_slots = true; }
    expect(no_slots && few_slots, "a pool with no slots, or fewer than one token routes to, is refused at construction");

    // --- what the protocol costs when nothing misses: the same three layers again and again ----
    {
        core::V4HotExpertSlots roomy(warm, 20);
        core::V4HbmTieredExpertExecutor executor(warm, roomy, layers, 16, streams);
        std::vector<int32_t> ids = {0, 1, 2, 3, 4, 5};
        std::vector<float> w(kSlots, 0.2f);
        float* d_w = to_device(w);
        half* out = to_device(std::vector<half>(shared.begin(), shared.begin() + row));
        auto walk = [&](core::V4RoutedExpertExecutor& e, core::ExpertLeaseHolder* holder, int tokens) {
            for (int t = 0; t < tokens; ++t) {
                for (int l = 0; l < kLayers; ++l) {
                    e.on_routing_ready(l, 1000 + t, ids, w);
                    e.accumulate_routed(l, 1000 + t, d_x, d_w, out);
                    e.on_routed_consumed(l, 1000 + t);
                }
                if (holder != nullptr) holder->release_leases();
            }
            GATE_HIP(hipStreamSynchronize(streams.compute));
        };
        auto timed = [&](core::V4RoutedExpertExecutor& e, core::ExpertLeaseHolder* holder) {
            walk(e, holder, 20);
            hipEvent_t begin, end;
            GATE_HIP(hipEventCreate(&begin));
            GATE_HIP(hipEventCreate(&end));
            GATE_HIP(hipEventRecord(begin, streams.compute));
            walk(e, holder, 200);
            GATE_HIP(hipEventRecord(end, streams.compute));
            GATE_HIP(hipEventSynchronize(end));
            float ms = 0;
            GATE_HIP(hipEventElapsedTime(&ms, begin, end));
            return ms * 1000.0f / (200 * kLayers);
        };
        const float us_tiered = timed(executor, &executor);
        const float us_resident = timed(resident, nullptr);
        const core::V4TierCounters c = executor.counters();
        std::printf("  all resident in the pool: %.1f us per layer step through the two-tier executor, %.1f us through the "
                    "all-resident one (%llu uploads in %llu dispatches)\n", us_tiered, us_resident,
                    static_cast<unsigned long long>(c.warm_uploads),
                    static_cast<unsigned long long>((c.hot_hits + c.warm_uploads) / kSlots));
        expect(c.warm_uploads == static_cast<uint64_t>(kLayers) * kSlots && c.forced_drains == 0,
               "a working set that fits is uploaded once and then only found");
    }

    // --- what a miss costs: one slot image over the host link -------------------------------
    {
        hipEvent_t begin, end;
        GATE_HIP(hipEventCreate(&begin));
        GATE_HIP(hipEventCreate(&end));
        void* d_slot = nullptr;
        GATE_HIP(hipMalloc(&d_slot, slot_bytes * 4));
        GATE_HIP(hipStreamSynchronize(streams.upload));
        GATE_HIP(hipEventRecord(begin, streams.upload));
        for (int i = 0; i < 16; ++i) {
            GATE_HIP(hipMemcpyAsync(static_cast<char*>(d_slot) + (i % 4) * slot_bytes, warm.image(i % kLayers, i % kExperts),
                                    slot_bytes, hipMemcpyHostToDevice, streams.upload));
        }
        GATE_HIP(hipEventRecord(end, streams.upload));
        GATE_HIP(hipEventSynchronize(end));
        float ms = 0;
        GATE_HIP(hipEventElapsedTime(&ms, begin, end));
        std::printf("  one miss = %.1f MB from pinned memory: %.3f ms (%.1f GB/s)\n", slot_bytes / 1e6, ms / 16,
                    16 * slot_bytes / 1e6 / ms);
    }
    std::printf(g_failures == 0 ? "[PASS] tiered executor\n" : "[FAIL] tiered executor\n");
    return g_failures == 0 ? 0 : 1;
}
