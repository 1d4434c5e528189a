#pragma once
// V4ResidentExpertPool: every routed expert of a model, loaded once from the `.aeon` expert
// container into HBM in the wave64 packing. It takes the place of UnifiedVRAMExpertPool's slot
// views (src/backend/swizzled_w4a16/core/vram_expert_pool.hpp:22-82) plus the expert half of
// AeonModelLoader (src/infrastructure/artifact/aeon_loader.hpp:145-166,318-470) on a machine
// where nothing is ever evicted: layer l's experts sit in consecutive slots and `table(l)` is
// the device array V4ResidentExpertExecutor's aeon_moe_layer::d_experts points at.
#include "aeon355/status.hpp"
#include "infrastructure/hip_check.hpp"

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

namespace aeon::core {

class V4ResidentExpertPool {
public:
    // File names and format version are the reference's current artifact specification
    // (make_current_swizzled_artifact_spec: model_experts_swizzled.{aeon,index}, version 2,
    // 4096-byte sectors). `scale_group` = columns per scale in the pool: 32 keeps every scale of
    // the container (one per 32 columns, swizzled_expert_format.hpp:18-23 -- the default, right
    // for any checkpoint); 128 stores one per 128 columns and refuses, with
    // std::invalid_argument, a container whose four scales inside 128 columns are not all equal.
    V4ResidentExpertPool(const std::string& model_dir, int hidden, int intermediate,
                         uint32_t format_version = 2, uint32_t sector_size = 4096, int scale_group = 32)
        : hidden_(hidden), intermediate_(intermediate), scale_group_(scale_group) {
        aeon355::throw_on_error(aeon_expert_catalog_open(
            (model_dir + "/model_experts_swizzled.index").c_str(),
            (model_dir + "/model_experts_swizzled.aeon").c_str(), format_version, sector_size, &catalog_));
        uint64_t payload = 0;
        uint32_t version = 0;
        aeon355::throw_on_error(
            aeon_expert_catalog_info(catalog_, &layers_, &experts_per_layer_, &payload, &version));
        slot_bytes_ = aeon_a64_slot_bytes(hidden, intermediate, scale_group);
        if (slot_bytes_ == 0) {
            close();
            throw std::invalid_argument("V4ResidentExpertPool: hidden/intermediate must be multiples of 128 "
                                        "and scale_group 32 or 128");
        }
        try {
            const size_t layer_bytes = slot_bytes_ * experts_per_layer_;
            CHECK_HIP(hipMalloc(&pool_, layer_bytes * layers_));
            CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&tables_),
                                sizeof(aeon_a64_expert) * experts_per_layer_ * layers_));
            std::vector<aeon_a64_expert> host(experts_per_layer_);
            for (uint32_t l = 0; l < layers_; ++l) {
                aeon355::throw_on_error(aeon_resident_load_layer(
                    catalog_, l, 0, experts_per_layer_, hidden, intermediate, scale_group,
                    static_cast<char*>(pool_) + l * layer_bytes, layer_bytes, host.data()));
                CHECK_HIP(hipMemcpy(tables_ + static_cast<size_t>(l) * experts_per_layer_, host.data(),
                                    sizeof(aeon_a64_expert) * experts_per_layer_, hipMemcpyHostToDevice));
            }
        } catch (...) {
            close();
            throw;
        }
    }

    ~V4ResidentExpertPool() { close(); }
    V4ResidentExpertPool(const V4ResidentExpertPool&) = delete;
    V4ResidentExpertPool& operator=(const V4ResidentExpertPool&) = delete;

    uint32_t layers() const { return layers_; }
    uint32_t experts_per_layer() const { return experts_per_layer_; }
    size_t resident_bytes() const { return slot_bytes_ * experts_per_layer_ * layers_; }
    // What aeon_moe_layer::scale_group has to say for a layer over this pool's tables.
    int scale_group() const { return scale_group_; }
    // A layer description over this pool's table of layer l with the geometry and the scale
    // grouping the pool was built with filled in, so the two cannot disagree; the caller adds
    // the routing fields (top_k, score kind, gate, bias, ...).
    aeon_moe_layer describe_layer(uint32_t layer) const {
        aeon_moe_layer L{};
        L.hidden = hidden_;
        L.intermediate = intermediate_;
        L.experts = static_cast<int>(experts_per_layer_);
        L.d_experts = table(layer);
        L.scale_group = scale_group_;
        return L;
    }
    // Device table of layer l: experts_per_layer() entries.
    const aeon_a64_expert* table(uint32_t layer) const {
        if (layer >= layers_) throw std::out_of_range("V4ResidentExpertPool: layer past the catalog");
        return tables_ + static_cast<size_t>(layer) * experts_per_layer_;
    }

private:
    void close() {
        if (tables_) (void)hipFree(tables_);
        if (pool_) (void)hipFree(pool_);
        aeon_expert_catalog_close(catalog_);
        tables_ = nullptr;
        pool_ = nullptr;
        catalog_ = nullptr;
    }

    int hidden_, intermediate_, scale_group_;
    aeon_expert_catalog* catalog_ = nullptr;
    uint32_t layers_ = 0, experts_per_layer_ = 0;
    size_t slot_bytes_ = 0;
    void* pool_ = nullptr;
    aeon_a64_expert* tables_ = nullptr;
};

}  // namespace aeon::core
