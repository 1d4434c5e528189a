#pragma once
// V4HbmTieredExpertExecutor: the routed-expert executor for a model whose experts do not all fit
// in HBM. It fills the seam the reference's V4TieredExpertExecutor fills
// (src/architecture/deepseek_v4/moe/v4_expert_executor.hpp:192-634) and keeps that executor's
// protocol -- announce (on_routing_ready*), consume (accumulate_routed*), release at the token
// boundary (ExpertLeaseHolder, src/infrastructure/expert/expert_lease_holder.hpp:21-33), and the
// capacity fallback that drains and releases instead of failing (:525-572) -- over two tiers only:
//
//   hot   a pool of HBM slots in the wave64 packing (V4HotExpertSlots), fewer than the model has
//         experts, with an LRU choice of victim among the slots nobody holds a lease on;
//   warm  every expert of every layer in pinned host memory, already in the wave64 packing
//         (V4WarmExpertStore), so a miss is one DMA of a slot image and nothing is repacked twice.
//
// The reference's supply coordinator, registry, staging arena, NVMe tier and telemetry are not
// here; what a gate needs from them is in V4TierCounters.
//
// Ordering is by streams, not by the host. A dispatch that misses records the compute stream's
// position and makes the upload stream wait for it before the first slot is overwritten (the
// hazard the reference's lease policy exists for -- an incoming upload landing on a slot an
// earlier kernel still reads, v4_expert_executor.hpp:30-47 -- cannot occur whatever the caller
// does with its leases); after the last copy the upload stream records one event, and the
// compute stream waits for it once, when the dispatch is first consumed (one wait per dispatch,
// where the reference waits once per distinct expert, :553-567). The routed ids select rows of a
// per-layer device table whose entries are rewritten, on the upload stream, whenever an expert
// changes slot.
#include "aeon355/status.hpp"
#include "architecture/deepseek_v4/layer/v4_layer_body_moe.hpp"
#include "infrastructure/hip_check.hpp"

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#if __has_include("infrastructure/expert/expert_lease_holder.hpp")
#include "infrastructure/expert/expert_lease_holder.hpp"
#else
namespace aeon::core {
// The reference declares this contract in src/infrastructure/expert/expert_lease_holder.hpp:21-33;
// it is repeated here only when the reference tree is not on the include path.
class ExpertLeaseHolder {
public:
    virtual ~ExpertLeaseHolder() = default;
    virtual void release_leases() = 0;
    virtual size_t outstanding_leases() const = 0;
};
}  // namespace aeon::core
#endif

namespace aeon::core {

// What a gate reads to tell which regime a run was in (the reference's SupplyTelemetry keeps
// the answering-tier mix and record_forced_drain, v4_expert_executor.hpp:546-572,597-611).
struct V4TierCounters {
    uint64_t hot_hits{0};       // distinct experts of a dispatch found resident
    uint64_t warm_uploads{0};   // distinct experts of a dispatch copied from pinned memory
    uint64_t evictions{0};      // uploads that replaced another expert
    uint64_t forced_drains{0};  // capacity fallbacks: streams drained, leases released
    uint64_t upload_bytes{0};
};

// Every expert of every layer as a slot image (aeon_a64_slot_bytes, the six sub-tensors where
// aeon_a64_slot_views puts them) in pinned host memory.
class V4WarmExpertStore {
public:
    V4WarmExpertStore(uint32_t layers, uint32_t experts_per_layer, int hidden, int intermediate,
                      int scale_group)
        : layers_(layers), experts_(experts_per_layer), hidden_(hidden), intermediate_(intermediate),
          scale_group_(scale_group), slot_bytes_(aeon_a64_slot_bytes(hidden, intermediate, scale_group)) {
        if (layers == 0 || experts_per_layer == 0 || slot_bytes_ == 0) {
            throw std::invalid_argument("V4WarmExpertStore: no layers, no experts, or a shape the "
                                        "wave64 packing does not take");
        }
        // allocated pinned, never registered after the fact
        CHECK_HIP(hipHostMalloc(&images_, slot_bytes_ * experts_ * layers_, hipHostMallocDefault));
    }

    // From the `.aeon` expert container (the files and defaults of V4ResidentExpertPool): each
    // layer is repacked on the device, `staging_experts` experts at a time, and copied down.
    V4WarmExpertStore(const std::string& model_dir, int hidden, int intermediate,
                      uint32_t format_version = 2, uint32_t sector_size = 4096, int scale_group = 32,
                      uint32_t staging_experts = 16)
        : hidden_(hidden), intermediate_(intermediate), scale_group_(scale_group),
          slot_bytes_(aeon_a64_slot_bytes(hidden, intermediate, scale_group)) {
        if (slot_bytes_ == 0 || staging_experts == 0) {
            throw std::invalid_argument("V4WarmExpertStore: a shape the wave64 packing does not take");
        }
        aeon_expert_catalog* catalog = nullptr;
        aeon355::throw_on_error(aeon_expert_catalog_open(
            (model_dir + "/model_experts_swizzled.index").c_str(),
            (model_dir + "/model_experts_swizzled.aeon").c_str(), format_version, sector_size, &catalog));
        void* staging = nullptr;
        try {
            uint64_t payload = 0;
            uint32_t version = 0;
            aeon355::throw_on_error(aeon_expert_catalog_info(catalog, &layers_, &experts_, &payload, &version));
            CHECK_HIP(hipHostMalloc(&images_, slot_bytes_ * experts_ * layers_, hipHostMallocDefault));
            const uint32_t step = std::min(staging_experts, experts_);
            CHECK_HIP(hipMalloc(&staging, slot_bytes_ * step));
            std::vector<aeon_a64_expert> views(step);
            for (uint32_t l = 0; l < layers_; ++l) {
                for (uint32_t first = 0; first < experts_; first += step) {
                    const uint32_t count = std::min(step, experts_ - first);
                    aeon355::throw_on_error(aeon_resident_load_layer(catalog, l, first, count, hidden,
                                                                     intermediate, scale_group, staging,
                                                                     slot_bytes_ * count, views.data()));
                    CHECK_HIP(hipMemcpy(image(l, first), staging, slot_bytes_ * count, hipMemcpyDeviceToHost));
                }
            }
        } catch (...) {
            if (staging) (void)hipFree(staging);
            if (images_) (void)hipHostFree(images_);
            aeon_expert_catalog_close(catalog);
            throw;
        }
        (void)hipFree(staging);
        aeon_expert_catalog_close(catalog);
    }

    ~V4WarmExpertStore() { (void)hipHostFree(images_); }
    V4WarmExpertStore(const V4WarmExpertStore&) = delete;
    V4WarmExpertStore& operator=(const V4WarmExpertStore&) = delete;

    // Copies one slot image down from device memory (a store filled from experts that were
    // packed on the device). Blocks.
    void store(uint32_t layer, uint32_t expert, const void* d_slot_image) {
        CHECK_HIP(hipMemcpy(image(layer, expert), d_slot_image, slot_bytes_, hipMemcpyDeviceToHost));
    }

    void* image(uint32_t layer, uint32_t expert) const {
        if (layer >= layers_ || expert >= experts_) {
            throw std::out_of_range("V4WarmExpertStore: expert outside the store");
        }
        return static_cast<char*>(images_) + (static_cast<size_t>(layer) * experts_ + expert) * slot_bytes_;
    }
    uint32_t layers() const { return layers_; }
    uint32_t experts_per_layer() const { return experts_; }
    size_t slot_bytes() const { return slot_bytes_; }
    int hidden() const { return hidden_; }
    int intermediate() const { return intermediate_; }
    int scale_group() const { return scale_group_; }

private:
    uint32_t layers_{0}, experts_{0};
    int hidden_, intermediate_, scale_group_;
    size_t slot_bytes_;
    void* images_{nullptr};
};

// The hot tier: `slots` slot images in HBM and the registry of which expert sits where. Host
// bookkeeping only; nothing here is thread-safe (one host thread owns the engine, as in the
// reference).
class V4HotExpertSlots {
public:
    static constexpr int32_t kNone = -1;

    V4HotExpertSlots(const V4WarmExpertStore& warm, uint32_t slots)
        : warm_(warm), slot_of_(static_cast<size_t>(warm.layers()) * warm.experts_per_layer(), kNone),
          slots_(slots) {
        if (slots == 0) {
            throw std::invalid_argument("V4HotExpertSlots: the HBM expert pool has no slots");
        }
        CHECK_HIP(hipMalloc(&pool_, warm.slot_bytes() * slots));
        views_.resize(slots);
        for (uint32_t s = 0; s < slots; ++s) {
            aeon355::throw_on_error(aeon_a64_slot_views(static_cast<char*>(pool_) + s * warm.slot_bytes(),
                                                        warm.hidden(), warm.intermediate(),
                                                        warm.scale_group(), &views_[s]));
        }
    }
    ~V4HotExpertSlots() { (void)hipFree(pool_); }
    V4HotExpertSlots(const V4HotExpertSlots&) = delete;
    V4HotExpertSlots& operator=(const V4HotExpertSlots&) = delete;

    uint32_t capacity() const { return static_cast<uint32_t>(slots_.size()); }
    uint32_t global_id(uint32_t layer, uint32_t expert) const { return layer * warm_.experts_per_layer() + expert; }
    int32_t slot_of(uint32_t gid) const { return slot_of_[gid]; }
    const aeon_a64_expert& views(int32_t slot) const { return views_[static_cast<size_t>(slot)]; }
    void* slot_memory(int32_t slot) const { return static_cast<char*>(pool_) + static_cast<size_t>(slot) * warm_.slot_bytes(); }
    uint32_t leases(int32_t slot) const { return slots_[static_cast<size_t>(slot)].leases; }

    // A lease only keeps the slot from being chosen as a victim.
    void lease(int32_t slot) {
        ++slots_[static_cast<size_t>(slot)].leases;
        slots_[static_cast<size_t>(slot)].last_use = ++clock_;
    }
    void release_lease(uint32_t gid) {
        const int32_t slot = slot_of_[gid];
        if (slot == kNone || slots_[static_cast<size_t>(slot)].leases == 0) {
            throw std::logic_error("V4HotExpertSlots: release of a lease that is not held");
        }
        --slots_[static_cast<size_t>(slot)].leases;
    }

    // How many slots a dispatch could take right now: free ones and unleased ones.
    uint32_t reclaimable() const {
        uint32_t n = 0;
        for (const Slot& s : slots_) n += s.leases == 0 ? 1 : 0;
        return n;
    }

    // The slot `gid` moves into: a free one if any, else the least recently used among the
    // unleased. `evicted` receives the expert that loses it (kNone for a free slot).
    int32_t claim(uint32_t gid, int64_t* evicted) {
        int32_t best = kNone;
        for (size_t s = 0; s < slots_.size(); ++s) {
            if (slots_[s].leases != 0) continue;
            if (slots_[s].gid == kNone) { best = static_cast<int32_t>(s); break; }
            if (best == kNone || slots_[s].last_use < slots_[static_cast<size_t>(best)].last_use) {
                best = static_cast<int32_t>(s);
            }
        }
        if (best == kNone) {
            throw std::runtime_error("V4HotExpertSlots: no reclaimable HBM slot (every slot is leased)");
        }
        Slot& slot = slots_[static_cast<size_t>(best)];
        *evicted = slot.gid;
        if (slot.gid != kNone) slot_of_[static_cast<size_t>(slot.gid)] = kNone;
        slot.gid = static_cast<int64_t>(gid);
        slot_of_[gid] = best;
        return best;
    }

private:
    struct Slot {
        int64_t gid{kNone};
        uint32_t leases{0};
        uint64_t last_use{0};
    };
    const V4WarmExpertStore& warm_;
    std::vector<int32_t> slot_of_;
    std::vector<Slot> slots_;
    std::vector<aeon_a64_expert> views_;
    void* pool_{nullptr};
    uint64_t clock_{0};
};

// The two streams the executor enqueues on, borrowed from the host (the reference's
// DeviceStreams has four, src/infrastructure/device_streams.hpp:29-37; with no NVMe tier and no
// write-back of evicted experts -- the warm copy is never stale -- two carry everything).
struct V4TierStreams {
    hipStream_t compute{nullptr};
    hipStream_t upload{nullptr};
};

class V4HbmTieredExpertExecutor final : public V4RoutedExpertExecutor, public ExpertLeaseHolder {
public:
    // `routing[l]` carries layer l's top_k, clamp and the like; its geometry, expert count,
    // scale grouping and expert table are overwritten from the store, and the shared expert of
    // either kind is cleared (behind this seam the layer body has already run it into moe_accum).
    // `first_layer` is the offset between the graph's global layer ids and the store's local ones
    // (v4_expert_executor.hpp:262-264).
    V4HbmTieredExpertExecutor(const V4WarmExpertStore& warm, V4HotExpertSlots& hot,
                              std::vector<aeon_moe_layer> routing, int max_tokens,
                              const V4TierStreams& streams, uint32_t first_layer = 0)
        : warm_(warm), hot_(hot), layers_(std::move(routing)), max_tokens_(max_tokens),
          streams_(streams), first_layer_(first_layer) {
        if (streams_.compute == nullptr || streams_.upload == nullptr || streams_.compute == streams_.upload) {
            throw std::invalid_argument("V4HbmTieredExpertExecutor: a compute stream and a separate upload "
                                        "stream are required");
        }
        if (layers_.size() != warm.layers() || max_tokens <= 0) {
            throw std::invalid_argument("V4HbmTieredExpertExecutor: one layer description per stored layer "
                                        "and a positive token bound are required");
        }
        const size_t entries = static_cast<size_t>(warm.layers()) * warm.experts_per_layer();
        CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&d_tables_), sizeof(aeon_a64_expert) * entries));
        CHECK_HIP(hipMemset(d_tables_, 0, sizeof(aeon_a64_expert) * entries));
        CHECK_HIP(hipHostMalloc(reinterpret_cast<void**>(&h_tables_), sizeof(aeon_a64_expert) * entries,
                                hipHostMallocDefault));
        std::memset(h_tables_, 0, sizeof(aeon_a64_expert) * entries);
        int widest_top_k = 0;
        for (size_t l = 0; l < layers_.size(); ++l) {
            aeon_moe_layer& layer = layers_[l];
            layer.hidden = warm.hidden();
            layer.intermediate = warm.intermediate();
            layer.experts = static_cast<int>(warm.experts_per_layer());
            layer.scale_group = warm.scale_group();
            layer.d_experts = d_tables_ + l * warm.experts_per_layer();
            layer.has_shared = 0;
            layer.d_shared_w1_f16 = nullptr;
            layer.d_shared_w3_f16 = nullptr;
            layer.d_shared_w2_f16 = nullptr;
            if (layer.top_k <= 0 || static_cast<uint32_t>(layer.top_k) > hot.capacity()) {
                throw std::invalid_argument("V4HbmTieredExpertExecutor: the HBM pool holds fewer slots than "
                                            "one token routes to");
            }
            widest_top_k = std::max(widest_top_k, layer.top_k);
            workspace_bytes_ = std::max(workspace_bytes_, aeon_moe_layer_workspace_bytes(&layer, max_tokens));
        }
        CHECK_HIP(hipMalloc(&workspace_, workspace_bytes_));
        CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&d_ids_), sizeof(int32_t) * max_tokens * widest_top_k));
        ids_per_dispatch_ = static_cast<size_t>(max_tokens) * widest_top_k;
        CHECK_HIP(hipHostMalloc(reinterpret_cast<void**>(&h_ids_), sizeof(int32_t) * ids_per_dispatch_ * kIdRing,
                                hipHostMallocDefault));
        CHECK_HIP(hipEventCreateWithFlags(&compute_mark_, hipEventDisableTiming));
        CHECK_HIP(hipEventCreateWithFlags(&uploads_done_, hipEventDisableTiming));
        for (hipEvent_t& e : ids_consumed_) CHECK_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    }

    ~V4HbmTieredExpertExecutor() override {
        (void)hipStreamSynchronize(streams_.upload);
        (void)hipStreamSynchronize(streams_.compute);
        (void)hipEventDestroy(compute_mark_);
        (void)hipEventDestroy(uploads_done_);
        for (hipEvent_t e : ids_consumed_) (void)hipEventDestroy(e);
        (void)hipFree(workspace_);
        (void)hipFree(d_ids_);
        (void)hipFree(d_tables_);
        (void)hipHostFree(h_tables_);
        (void)hipHostFree(h_ids_);
    }
    V4HbmTieredExpertExecutor(const V4HbmTieredExpertExecutor&) = delete;
    V4HbmTieredExpertExecutor& operator=(const V4HbmTieredExpertExecutor&) = delete;

    void on_routing_ready(uint32_t layer_id, uint32_t position, const std::vector<int32_t>& ids,
                          const std::vector<float>& weights) override {
        on_routing_ready_batch(layer_id, position, {ids}, {weights});
    }

    // The layer-wide dispatch: the chunk's draws as one deduplicated set, each distinct expert
    // leased once and uploaded at most once (v4_expert_executor.hpp:266-291).
    void on_routing_ready_batch(uint32_t layer_id, uint32_t first_position,
                                const std::vector<std::vector<int32_t>>& ids,
                                const std::vector<std::vector<float>>& weights) override {
        const uint32_t local = local_layer(layer_id);
        if (ids.empty()) {
            throw std::invalid_argument("V4HbmTieredExpertExecutor: a layer-wide dispatch needs at least one token");
        }
        if (ids.size() != weights.size() || ids.size() > static_cast<size_t>(max_tokens_)) {
            throw std::invalid_argument("V4HbmTieredExpertExecutor: malformed routing batch");
        }
        const aeon_moe_layer& layer = layers_[local];
        std::vector<uint32_t> distinct;
        std::vector<int32_t> flat;
        for (const std::vector<int32_t>& row : ids) {
            if (row.size() != static_cast<size_t>(layer.top_k)) {
                throw std::invalid_argument("V4HbmTieredExpertExecutor: expected " + std::to_string(layer.top_k) +
                                            " routed experts, got " + std::to_string(row.size()));
            }
            for (int32_t id : row) {
                if (id < 0 || id >= layer.experts) {
                    throw std::out_of_range("V4HbmTieredExpertExecutor: routed id outside the layer");
                }
                flat.push_back(id);
                const uint32_t gid = hot_.global_id(local, static_cast<uint32_t>(id));
                if (std::find(distinct.begin(), distinct.end(), gid) == distinct.end()) distinct.push_back(gid);
            }
        }
        if (distinct.size() > hot_.capacity()) {
            throw std::invalid_argument("V4HbmTieredExpertExecutor: the chunk routes to " +
                                        std::to_string(distinct.size()) + " distinct experts, the HBM pool holds " +
                                        std::to_string(hot_.capacity()) + "; split the chunk");
        }
        ensure_pool_headroom(distinct);

        // the resident ones are leased before any victim is chosen, so a miss of the same
        // dispatch cannot take their slots
        for (const uint32_t gid : distinct) {
            const int32_t slot = hot_.slot_of(gid);
            if (slot == V4HotExpertSlots::kNone) continue;
            hot_.lease(slot);
            leases_.push_back(gid);
            ++counters_.hot_hits;
        }
        bool marked = false;
        for (const uint32_t gid : distinct) {
            if (hot_.slot_of(gid) != V4HotExpertSlots::kNone) continue;  // leased above
            if (!marked) {
                // nothing the compute stream was given so far may still read a slot once the
                // first copy of this dispatch lands
                CHECK_HIP(hipEventRecord(compute_mark_, streams_.compute));
                CHECK_HIP(hipStreamWaitEvent(streams_.upload, compute_mark_, 0));
                marked = true;
            }
            int64_t evicted = V4HotExpertSlots::kNone;
            const int32_t slot = hot_.claim(gid, &evicted);
            const uint32_t expert = gid % warm_.experts_per_layer();
            CHECK_HIP(hipMemcpyAsync(hot_.slot_memory(slot), warm_.image(local, expert), warm_.slot_bytes(),
                                     hipMemcpyHostToDevice, streams_.upload));
            // the pinned mirror of the entry is what the copy reads, so it is rewritten only
            // here, for the expert whose copy is enqueued right behind it
            h_tables_[gid] = hot_.views(slot);
            CHECK_HIP(hipMemcpyAsync(d_tables_ + gid, h_tables_ + gid, sizeof(aeon_a64_expert),
                                     hipMemcpyHostToDevice, streams_.upload));
            hot_.lease(slot);
            leases_.push_back(gid);
            ++counters_.warm_uploads;
            counters_.upload_bytes += warm_.slot_bytes();
            if (evicted != V4HotExpertSlots::kNone) ++counters_.evictions;
        }
        if (marked) CHECK_HIP(hipEventRecord(uploads_done_, streams_.upload));
        // a dispatch that was announced and never consumed leaves its wait to the next one
        awaiting_uploads_ = awaiting_uploads_ || marked;

        // the per-token path needs the ids on the device; a chunk passes its own device ids.
        // They are staged in a ring of pinned rows: the copy out of a row may still be queued
        // behind earlier layers' kernels, and the host only waits for it when the ring comes
        // round to that row again.
        const size_t turn = dispatches_++ % kIdRing;
        if (dispatches_ > kIdRing) CHECK_HIP(hipEventSynchronize(ids_consumed_[turn]));
        int32_t* staged = h_ids_ + turn * ids_per_dispatch_;
        std::memcpy(staged, flat.data(), flat.size() * sizeof(int32_t));
        CHECK_HIP(hipMemcpyAsync(d_ids_, staged, flat.size() * sizeof(int32_t), hipMemcpyHostToDevice,
                                 streams_.compute));
        CHECK_HIP(hipEventRecord(ids_consumed_[turn], streams_.compute));

        current_layer_ = static_cast<int64_t>(layer_id);
        first_position_ = first_position;
        token_count_ = static_cast<uint32_t>(ids.size());
        last_dispatch_experts_ = static_cast<uint32_t>(distinct.size());
        batch_draws_ += flat.size();
        batch_distinct_ += distinct.size();
    }

    void accumulate_routed(uint32_t layer_id, uint32_t position, const half* expert_input,
                           const float* expert_weights, half* moe_accum) override {
        if (current_layer_ != static_cast<int64_t>(layer_id)) {
            throw std::logic_error("V4HbmTieredExpertExecutor: accumulate_routed without a matching "
                                   "on_routing_ready");
        }
        if (position < first_position_) {
            throw std::logic_error("V4HbmTieredExpertExecutor: consume before the batch's first position");
        }
        const uint32_t token = position - first_position_;
        if (token >= token_count_) {
            throw std::out_of_range("V4HbmTieredExpertExecutor: token index past the batch's token count");
        }
        materialize_batch();
        const aeon_moe_layer& layer = layers_[local_layer(layer_id)];
        aeon355::throw_on_error(aeon_moe_layer_routed(
            &layer, expert_input, layer.hidden, 1, d_ids_ + static_cast<size_t>(token) * layer.top_k,
            expert_weights, moe_accum, layer.hidden, workspace_, workspace_bytes_, streams_.compute));
    }

    void accumulate_routed_batch(uint32_t layer_id, uint32_t first_position, uint32_t token_count,
                                 const half* batch_input, int input_stride, const int* batch_ids,
                                 int ids_stride, const float* batch_weights, int weights_stride,
                                 half* batch_output, int output_stride) override {
        if (token_count == 0) return;
        if (current_layer_ != static_cast<int64_t>(layer_id) || first_position != first_position_ ||
            token_count != token_count_) {
            throw std::logic_error("V4HbmTieredExpertExecutor: accumulate_routed_batch without a matching "
                                   "batch dispatch");
        }
        const aeon_moe_layer& layer = layers_[local_layer(layer_id)];
        if (batch_ids == nullptr || ids_stride != layer.top_k || weights_stride != layer.top_k) {
            throw std::invalid_argument("V4HbmTieredExpertExecutor: batch ids and weights must be [token, top_k]");
        }
        materialize_batch();
        aeon355::throw_on_error(aeon_moe_layer_routed(
            &layer, batch_input, input_stride, static_cast<int>(token_count), batch_ids, batch_weights,
            batch_output, output_stride, workspace_, workspace_bytes_, streams_.compute));
    }

    // The token boundary: the caller has a compute-stream boundary here, and every lease held
    // for the token goes back (v4_expert_executor.hpp:484-494).
    void release_leases() override {
        for (const uint32_t gid : leases_) hot_.release_lease(gid);
        leases_.clear();
    }
    size_t outstanding_leases() const noexcept override { return leases_.size(); }

    uint32_t last_dispatch_experts() const noexcept { return last_dispatch_experts_; }
    uint32_t last_dispatch_tokens() const noexcept { return token_count_; }
    uint64_t batch_draws() const noexcept { return batch_draws_; }
    uint64_t batch_distinct() const noexcept { return batch_distinct_; }
    const V4TierCounters& counters() const noexcept { return counters_; }

private:
    uint32_t local_layer(uint32_t layer_id) const {
        if (layer_id < first_layer_ || layer_id - first_layer_ >= layers_.size()) {
            throw std::out_of_range("V4HbmTieredExpertExecutor: layer id outside the stored layers");
        }
        return layer_id - first_layer_;
    }

    // Orders the compute stream behind the dispatch's copies, once.
    void materialize_batch() {
        if (!awaiting_uploads_) return;
        CHECK_HIP(hipStreamWaitEvent(streams_.compute, uploads_done_, 0));
        awaiting_uploads_ = false;
    }

    // A dispatch needs a victim for each of its misses, and only slots that nobody holds a lease
    // on -- and that do not hold another expert of the same dispatch -- qualify. When the leases
    // already held would leave too few, both streams are drained, so that the release means
    // what the lease contract says (no reader in flight), and the leases go back
    // (v4_expert_executor.hpp:569-590). A pool that holds a whole token's leases never gets here.
    void ensure_pool_headroom(const std::vector<uint32_t>& incoming) {
        uint32_t misses = 0, own_unleased = 0;
        for (const uint32_t gid : incoming) {
            const int32_t slot = hot_.slot_of(gid);
            if (slot == V4HotExpertSlots::kNone) ++misses;
            else if (hot_.leases(slot) == 0) ++own_unleased;
        }
        if (misses + own_unleased <= hot_.reclaimable()) return;
        CHECK_HIP(hipStreamSynchronize(streams_.compute));
        CHECK_HIP(hipStreamSynchronize(streams_.upload));
        release_leases();
        ++counters_.forced_drains;
    }

    const V4WarmExpertStore& warm_;
    V4HotExpertSlots& hot_;
    std::vector<aeon_moe_layer> layers_;
    int max_tokens_;
    V4TierStreams streams_;
    uint32_t first_layer_;

    aeon_a64_expert* d_tables_{nullptr};   // [layers][experts]: where each expert sits now
    aeon_a64_expert* h_tables_{nullptr};   // pinned mirror, the source of the entry copies
    void* workspace_{nullptr};
    size_t workspace_bytes_{0};
    int32_t* d_ids_{nullptr};
    int32_t* h_ids_{nullptr};
    static constexpr size_t kIdRing = 16;
    size_t ids_per_dispatch_{0};
    uint64_t dispatches_{0};
    hipEvent_t compute_mark_{nullptr}, uploads_done_{nullptr};
    hipEvent_t ids_consumed_[kIdRing] = {};
    bool awaiting_uploads_{false};

    int64_t current_layer_{-1};
    uint32_t first_position_{0};
    uint32_t token_count_{0};
    uint32_t last_dispatch_experts_{0};
    uint64_t batch_draws_{0}, batch_distinct_{0};
    std::vector<uint32_t> leases_;
    V4TierCounters counters_;
};

}  // namespace aeon::core
