// Gate: a model directory's expert container -> V4ResidentExpertPool -> V4ResidentExpertExecutor.
// The container is written here in the writer's format (32-byte "AEON_EXPERTS" header + one
// {offset, length} entry per expert, scripts/convert_safetensors_to_aeon.py:463-486) from
// synthetic payloads; the pool's slots must equal, byte for byte, a direct device repack of the
// same payloads, the executor over the pool's tables must give the bits of the executor over
// directly built tables, and the loader must reject what AeonModelLoader rejects.
#include "architecture/deepseek_v4/moe/v4_resident_expert_executor.hpp"
#include "architecture/deepseek_v4/moe/v4_resident_expert_pool.hpp"
#include "architecture/deepseek_v4/moe/v4_tiered_expert_executor.hpp"
#include "backend/swizzled_w4a16/core/swizzled_expert_format.hpp"
#include "common.hpp"
#include "test_device.hpp"

#include <cstring>
#include <filesystem>
#include <fstream>

#include <unistd.h>

namespace core = aeon::core;

constexpr int kHidden = 512, kIntermediate = 256, kExperts = 5, kLayers = 2, kSlots = 2, kTokens = 7;
constexpr core::SwizzledExpertLayout kL = core::swizzled_expert_layout(kHidden, kIntermediate);

static void write_container(const std::filesystem::path& dir, const std::vector<std::vector<uint8_t>>& payloads,
                            uint32_t version) {
    std::ofstream experts(dir / "model_experts_swizzled.aeon", std::ios::binary);
    std::ofstream index(dir / "model_experts_swizzled.index", std::ios::binary);
    const uint32_t layers = kLayers, per_layer = kExperts;
    const uint64_t bytes = kL.bytes;
    index.write("AEON_EXPERTS", 12);
    index.write(reinterpret_cast<const char*>(&version), 4);
    index.write(reinterpret_cast<const char*>(&layers), 4);
    index.write(reinterpret_cast<const char*>(&per_layer), 4);
    index.write(reinterpret_cast<const char*>(&bytes), 8);
    // payloads are stored last-to-first with a sector of filler between them: the index, not the
    // position in the file, says where an expert is
    std::vector<uint64_t> offset(payloads.size());
    uint64_t at = 0;
    const std::vector<char> filler(4096, '\x5A');
    for (size_t i = payloads.size(); i-- > 0;) {
        experts.write(filler.data(), filler.size());
        at += filler.size();
        offset[i] = at;
        experts.write(reinterpret_cast<const char*>(payloads[i].data()), payloads[i].size());
        at += payloads[i].size();
    }
    for (size_t i = 0; i < payloads.size(); ++i) {
        index.write(reinterpret_cast<const char*>(&offset[i]), 8);
        index.write(reinterpret_cast<const char*>(&bytes), 8);
    }
}

int main() {
    aeon::test::select_test_device(true);
    static_assert(kL.bytes % 4096 == 0, "payloads must keep the 4096-byte sector alignment");
    const size_t off[3][2] = {{kL.w1_packed, kL.w1_scale}, {kL.w3_packed, kL.w3_scale}, {kL.w2_packed, kL.w2_scale}};
    const int shape[3][4] = {{kIntermediate, kHidden, 4, 8}, {kIntermediate, kHidden, 4, 8}, {kHidden, kIntermediate, 8, 4}};

    // synthetic payloads on the device -> host -> container; the same payloads repacked directly.
    // Once with one scale per 128 columns (replicated over the payload's group-32 slots, one kept
    // in the pool) and once with a scale of its own per 32 columns, all kept: the real format.
    std::vector<std::vector<uint8_t>> payloads;
    uint8_t* d_payload = nullptr;
    GATE_HIP(hipMalloc(&d_payload, kL.bytes));
    const std::filesystem::path dir =
        std::filesystem::temp_directory_path() / ("aeon_pool_gate_" + std::to_string(::getpid()));
    std::filesystem::create_directories(dir);
    for (const int scale_group : {32, 128}) {
    payloads.clear();
    std::vector<std::vector<aeon_a64_expert>> direct(kLayers);
    for (int l = 0; l < kLayers; ++l)
        for (int e = 0; e < kExperts; ++e) {
            void* a64[6];
            for (int m = 0; m < 3; ++m) {
                aeon355::throw_on_error(aeon_synth_matrix_swizzled(31, 10 * l + e, m, shape[m][0], shape[m][1],
                                                                   shape[m][2], shape[m][3], scale_group,
                                                                   d_payload + off[m][0], d_payload + off[m][1],
                                                                   nullptr));
                GATE_HIP(hipMalloc(&a64[2 * m], aeon_a64_packed_bytes(shape[m][0], shape[m][1])));
                GATE_HIP(hipMalloc(&a64[2 * m + 1], aeon_a64_scale_bytes(shape[m][0], shape[m][1], scale_group)));
                aeon355::throw_on_error(aeon_a64_repack_device(d_payload + off[m][0], d_payload + off[m][1],
                                                               shape[m][0], shape[m][1], shape[m][2], shape[m][3],
                                                               scale_group, a64[2 * m], a64[2 * m + 1], nullptr,
                                                               nullptr));
            }
            GATE_HIP(hipDeviceSynchronize());
            payloads.push_back(to_host(d_payload, kL.bytes));
            direct[l].push_back(aeon_a64_expert{a64[0], a64[1], a64[2], a64[3], a64[4], a64[5]});
        }

    write_container(dir, payloads, 2);
    std::printf("  -- one scale per %d columns\n", scale_group);

    {
        core::V4ResidentExpertPool pool(dir.string(), kHidden, kIntermediate, 2, 4096, scale_group);
        expect(pool.layers() == kLayers && pool.experts_per_layer() == kExperts, "catalog shape read from the index");
        expect(pool.scale_group() == scale_group, "the pool reports its scale grouping");
        bool same = true;
        for (int l = 0; l < kLayers; ++l) {
            const std::vector<aeon_a64_expert> table = to_host(pool.table(l), kExperts);
            for (int e = 0; e < kExperts; ++e) {
                const void* got[6] = {table[e].w1_packed, table[e].w1_scale, table[e].w3_packed,
                                      table[e].w3_scale, table[e].w2_packed, table[e].w2_scale};
                const void* want[6] = {direct[l][e].w1_packed, direct[l][e].w1_scale, direct[l][e].w3_packed,
                                       direct[l][e].w3_scale, direct[l][e].w2_packed, direct[l][e].w2_scale};
                for (int j = 0; j < 6; ++j) {
                    const int m = j / 2;
                    const size_t n = j % 2 == 0 ? aeon_a64_packed_bytes(shape[m][0], shape[m][1])
                                                : aeon_a64_scale_bytes(shape[m][0], shape[m][1], scale_group);
                    same = same && to_host(static_cast<const uint8_t*>(got[j]), n) ==
                                       to_host(static_cast<const uint8_t*>(want[j]), n);
                }
            }
        }
        expect(same, "every slot equals the direct repack of its payload, byte for byte");

        // the executor over the pool's tables against the executor over the directly built ones
        std::vector<aeon_moe_layer> from_pool(kLayers), from_direct(kLayers);
        for (int l = 0; l < kLayers; ++l) {
            from_pool[l] = aeon_moe_layer{kHidden, kIntermediate, kExperts, kSlots, 0, 7.0f, AEON_ROUTER_SCORE_SIGMOID,
                                          1.0f, 1, nullptr, nullptr, pool.table(l), pool.scale_group()};
            from_direct[l] = from_pool[l];
            from_direct[l].d_experts = to_device(direct[l]);
        }
        core::V4ResidentExpertExecutor a(from_pool, 16, nullptr), b(from_direct, 16, nullptr);
        SplitMix rng{0xC0FFEEull};
        std::vector<half> x(static_cast<size_t>(kTokens) * kHidden), shared(x.size());
        for (half& v : x) v = __float2half(static_cast<float>(rng.uniform() - 0.5));
        for (half& v : shared) v = __float2half(static_cast<float>(rng.uniform() - 0.5));
        half* d_x = to_device(x);
        bool identical = true, moved = false;
        for (int l = 0; l < kLayers; ++l) {
            std::vector<std::vector<int32_t>> ids(kTokens);
            std::vector<std::vector<float>> weights(kTokens);
            std::vector<int32_t> flat_ids;
            std::vector<float> flat_w;
            for (int t = 0; t < kTokens; ++t)
                for (int k = 0; k < kSlots; ++k) {
                    ids[t].push_back((2 * t + 3 * k + l) % kExperts);
                    weights[t].push_back(0.5f + 0.1f * static_cast<float>(k));
                    flat_ids.push_back(ids[t].back());
                    flat_w.push_back(weights[t].back());
                }
            int* d_ids = to_device(flat_ids);
            float* d_w = to_device(flat_w);
            half* out_a = to_device(shared);
            half* out_b = to_device(shared);
            a.on_routing_ready_batch(l, 0, ids, weights);
            a.accumulate_routed_batch(l, 0, kTokens, d_x, kHidden, d_ids, kSlots, d_w, kSlots, out_a, kHidden);
            b.on_routing_ready_batch(l, 0, ids, weights);
            b.accumulate_routed_batch(l, 0, kTokens, d_x, kHidden, d_ids, kSlots, d_w, kSlots, out_b, kHidden);
            GATE_HIP(hipDeviceSynchronize());
            const std::vector<half> ra = to_host(out_a, x.size()), rb = to_host(out_b, x.size());
            identical = identical && std::memcmp(ra.data(), rb.data(), ra.size() * sizeof(half)) == 0;
            moved = moved || std::memcmp(ra.data(), shared.data(), ra.size() * sizeof(half)) != 0;
        }
        expect(identical, "executor over the loaded pool gives the bits of the directly built tables");
        expect(moved, "the routed experts changed the accumulator");
    }
    {
        // the same container into the pinned-memory store of the two-tier executor, two experts
        // at a time (five per layer: the last group is a short one)
        core::V4WarmExpertStore warm(dir.string(), kHidden, kIntermediate, 2, 4096, scale_group, /*staging_experts=*/2);
        expect(warm.layers() == kLayers && warm.experts_per_layer() == kExperts &&
                   warm.slot_bytes() == aeon_a64_slot_bytes(kHidden, kIntermediate, scale_group),
               "warm store: catalog shape and slot size");
        void* d_slot = nullptr;
        GATE_HIP(hipMalloc(&d_slot, warm.slot_bytes()));
        aeon_a64_expert views{};
        aeon355::throw_on_error(aeon_a64_slot_views(d_slot, kHidden, kIntermediate, scale_group, &views));
        bool same = true;
        for (int l = 0; l < kLayers; ++l)
            for (int e = 0; e < kExperts; ++e) {
                GATE_HIP(hipMemcpy(d_slot, warm.image(l, e), warm.slot_bytes(), hipMemcpyHostToDevice));
                const void* got[6] = {views.w1_packed, views.w1_scale, views.w3_packed,
                                      views.w3_scale, views.w2_packed, views.w2_scale};
                const void* want[6] = {direct[l][e].w1_packed, direct[l][e].w1_scale, direct[l][e].w3_packed,
                                       direct[l][e].w3_scale, direct[l][e].w2_packed, direct[l][e].w2_scale};
                for (int j = 0; j < 6; ++j) {
                    const int m = j / 2;
                    const size_t n = j % 2 == 0 ? aeon_a64_packed_bytes(shape[m][0], shape[m][1])
                                                : aeon_a64_scale_bytes(shape[m][0], shape[m][1], scale_group);
                    same = same && to_host(static_cast<const uint8_t*>(got[j]), n) ==
                                       to_host(static_cast<const uint8_t*>(want[j]), n);
                }
            }
        GATE_HIP(hipFree(d_slot));
        expect(same, "warm store: every pinned slot image equals the direct repack of its payload");

        // container -> warm store -> three HBM slots -> two-tier executor, against the executor
        // over the directly built tables: five experts a layer through three slots, so the walk
        // evicts, and every token of every layer has to come out with the same bits
        core::V4TierStreams streams;
        GATE_HIP(hipStreamCreateWithFlags(&streams.compute, hipStreamNonBlocking));
        GATE_HIP(hipStreamCreateWithFlags(&streams.upload, hipStreamNonBlocking));
        std::vector<aeon_moe_layer> routing(kLayers), from_direct(kLayers);
        for (int l = 0; l < kLayers; ++l) {
            routing[l] = aeon_moe_layer{kHidden, kIntermediate, kExperts, kSlots, 0, 7.0f, AEON_ROUTER_SCORE_SIGMOID,
                                        1.0f, 1, nullptr, nullptr, nullptr, scale_group};
            from_direct[l] = routing[l];
            from_direct[l].d_experts = to_device(direct[l]);
        }
        core::V4HotExpertSlots hot(warm, 3);
        core::V4HbmTieredExpertExecutor tiered(warm, hot, routing, 16, streams);
        core::V4ResidentExpertExecutor control(from_direct, 16, streams.compute);
        SplitMix rng{0x1207E8C0ull};
        std::vector<half> x(static_cast<size_t>(kTokens) * kHidden), shared(x.size());
        for (half& v : x) v = __float2half(static_cast<float>(rng.uniform() - 0.5));
        for (half& v : shared) v = __float2half(static_cast<float>(rng.uniform() - 0.5));
        half* d_x = to_device(x);
        half* out_t = to_device(shared);
        half* out_c = to_device(shared);
        for (int t = 0; t < kTokens; ++t) {
            for (int l = 0; l < kLayers; ++l) {
                const std::vector<int32_t> ids = {(2 * t + l) % kExperts, (2 * t + l + 3) % kExperts};
                const std::vector<float> w = {0.7f, 0.3f};
                float* d_w = to_device(w);
                tiered.on_routing_ready(l, t, ids, w);
                tiered.accumulate_routed(l, t, d_x + static_cast<size_t>(t) * kHidden, d_w,
                                         out_t + static_cast<size_t>(t) * kHidden);
                control.on_routing_ready(l, t, ids, w);
                control.accumulate_routed(l, t, d_x + static_cast<size_t>(t) * kHidden, d_w,
                                          out_c + static_cast<size_t>(t) * kHidden);
            }
            GATE_HIP(hipStreamSynchronize(streams.compute));
            tiered.release_leases();
        }
        const std::vector<half> rt = to_host(out_t, x.size()), rc = to_host(out_c, x.size());
        expect(std::memcmp(rt.data(), rc.data(), rt.size() * sizeof(half)) == 0 && tiered.counters().evictions > 0,
               "two-tier executor over the container, three slots for ten experts: the bits of the direct tables");
    }
    }   // scale_group

    bool version_rejected = false, shape_rejected = false, missing_rejected = false, scales_rejected = false;
    try {
        core::V4ResidentExpertPool pool(dir.string(), kHidden, kIntermediate, /*format_version=*/3);
    } catch (const std::runtime_error&) { version_rejected = true; }
    try {
        core::V4ResidentExpertPool pool(dir.string(), kHidden * 2, kIntermediate);
    } catch (const std::invalid_argument&) { shape_rejected = true; }
    try {
        core::V4ResidentExpertPool pool((dir / "nowhere").string(), kHidden, kIntermediate);
    } catch (const std::runtime_error&) { missing_rejected = true; }
    // the container on disk now holds the replicated payloads (the loop's last pass)
    payloads[3][kL.w3_scale + 2] ^= 0x04;  // one of four replicated group-32 scales no longer equal
    write_container(dir, payloads, 2);
    try {
        core::V4ResidentExpertPool pool(dir.string(), kHidden, kIntermediate, 2, 4096, /*scale_group=*/128);
    } catch (const std::invalid_argument&) { scales_rejected = true; }
    bool scales_kept = false;
    try {
        core::V4ResidentExpertPool pool(dir.string(), kHidden, kIntermediate);   // default: all scales kept
        scales_kept = pool.scale_group() == 32;
    } catch (const std::exception&) {}
    expect(version_rejected, "an index of another format version throws std::runtime_error");
    expect(shape_rejected, "a shape whose payload size differs from the catalog's throws std::invalid_argument");
    expect(missing_rejected, "a missing container throws std::runtime_error");
    expect(scales_rejected, "group-32 scales that differ inside 128 columns are refused by a one-scale pool");
    expect(scales_kept, "the same container loads into a pool that keeps every scale (the default)");
    std::filesystem::remove_all(dir);
    std::printf(g_failures == 0 ? "[PASS] resident pool\n" : "[FAIL] resident pool\n");
    return g_failures == 0 ? 0 : 1;
}
