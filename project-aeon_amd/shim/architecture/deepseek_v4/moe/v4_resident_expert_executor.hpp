#pragma once
// V4ResidentExpertExecutor: the routed-expert executor for a machine whose HBM holds every
// expert of every layer (288 GB on MI355X), in the wave64 packing. It fills the seam the
// reference's V4TieredExpertExecutor fills (src/architecture/deepseek_v4/moe/
// v4_expert_executor.hpp:192-461) with the supply system removed: no leases, no staging, no
// host round trip for the ids -- the routed ids stay on the device and select rows of a
// device-resident expert table.
//
// Protocol kept from the reference: accumulate_routed* without a matching on_routing_ready*
// for the same layer is a std::logic_error; a position outside the announced batch is a
// std::out_of_range / std::logic_error (v4_expert_executor.hpp:302-315); ids and weights of a
// chunk must be [token, top_k] (:411-415).
#include "aeon355/status.hpp"
#include "architecture/deepseek_v4/layer/v4_layer_body_moe.hpp"
#include "infrastructure/hip_check.hpp"

#include <stdexcept>
#include <vector>

namespace aeon::core {

class V4ResidentExpertExecutor final : public V4RoutedExpertExecutor {
public:
    // `layers[l]` describes layer l (experts resident). `max_tokens` sizes the workspace.
    // Behind this seam the reference's layer body has already run the shared expert into
    // moe_accum (run_layer_body_moe_shared_expert, layer/v4_layer_body_moe.hpp:216-256) before it
    // calls accumulate_routed*, and the routed sum is added to what it finds there. The executor's
    // copy of each layer therefore carries no shared expert of either kind: has_shared is cleared
    // and so are the dense fp16 shared-expert matrices, which only aeon_moe_layer_decode (the
    // whole step on the device) uses. A layer description filled for both uses can be passed as
    // it is.
    V4ResidentExpertExecutor(std::vector<aeon_moe_layer> layers, int max_tokens, hipStream_t stream)
        : layers_(std::move(layers)), max_tokens_(max_tokens), stream_(stream) {
        if (layers_.empty() || max_tokens <= 0) {
            throw std::invalid_argument("V4ResidentExpertExecutor: no layers or no tokens");
        }
        int widest_top_k = 0;
        for (aeon_moe_layer& layer : layers_) {
            layer.has_shared = 0;
            layer.d_shared_w1_f16 = nullptr;
            layer.d_shared_w3_f16 = nullptr;
            layer.d_shared_w2_f16 = nullptr;
            widest_top_k = std::max(widest_top_k, layer.top_k);
            workspace_bytes_ = std::max(workspace_bytes_, aeon_moe_layer_workspace_bytes(&layer, max_tokens));
        }
        CHECK_HIP(hipMalloc(&workspace_, workspace_bytes_));
        CHECK_HIP(hipMalloc(&d_ids_, sizeof(int32_t) * max_tokens * widest_top_k));
    }

    ~V4ResidentExpertExecutor() override {
        (void)hipFree(workspace_);
        (void)hipFree(d_ids_);
    }

    V4ResidentExpertExecutor(const V4ResidentExpertExecutor&) = delete;
    V4ResidentExpertExecutor& operator=(const V4ResidentExpertExecutor&) = delete;

    void on_routing_ready(uint32_t layer_id, uint32_t position, const std::vector<int32_t>& ids,
                          const std::vector<float>& weights) override {
        on_routing_ready_batch(layer_id, position, {ids}, {weights});
    }

    void on_routing_ready_batch(uint32_t layer_id, uint32_t first_position,
                                const std::vector<std::vector<int32_t>>& ids,
                                const std::vector<std::vector<float>>& weights) override {
        if (layer_id >= layers_.size()) {
            throw std::out_of_range("V4ResidentExpertExecutor: layer id past the resident layers");
        }
        if (ids.empty() || ids.size() != weights.size() ||
            ids.size() > static_cast<size_t>(max_tokens_)) {
            throw std::invalid_argument("V4ResidentExpertExecutor: malformed routing batch");
        }
        const int k = layers_[layer_id].top_k;
        host_ids_.clear();
        for (const std::vector<int32_t>& row : ids) {
            if (row.size() != static_cast<size_t>(k)) {
                throw std::invalid_argument("V4ResidentExpertExecutor: ids must be [token, top_k]");
            }
            for (int32_t id : row) {
                if (id < 0 || id >= layers_[layer_id].experts) {
                    throw std::out_of_range("V4ResidentExpertExecutor: routed id outside the layer");
                }
                host_ids_.push_back(id);
            }
        }
        // the per-token path needs the ids on the device; a chunk passes its own device ids
        CHECK_HIP(hipMemcpyAsync(d_ids_, host_ids_.data(), host_ids_.size() * sizeof(int32_t),
                                 hipMemcpyHostToDevice, stream_));
        current_layer_ = static_cast<int64_t>(layer_id);
        first_position_ = first_position;
        token_count_ = static_cast<uint32_t>(ids.size());
    }

    void accumulate_routed(uint32_t layer_id, uint32_t position, const half* expert_input,
                           const float* expert_weights, half* moe_accum) override {
        check_token(layer_id, position, "accumulate_routed");
        const aeon_moe_layer& layer = layers_[layer_id];
        const uint32_t token = position - first_position_;
        aeon355::throw_on_error(aeon_moe_layer_routed(
            &layer, expert_input, layer.hidden, 1, d_ids_ + static_cast<size_t>(token) * layer.top_k,
            expert_weights, moe_accum, layer.hidden, workspace_, workspace_bytes_, stream_));
    }

    void accumulate_routed_batch(uint32_t layer_id, uint32_t first_position, uint32_t token_count,
                                 const half* batch_input, int input_stride, const int* batch_ids,
                                 int ids_stride, const float* batch_weights, int weights_stride,
                                 half* batch_output, int output_stride) override {
        if (token_count == 0) return;
        if (current_layer_ != static_cast<int64_t>(layer_id) || first_position != first_position_ ||
            token_count != token_count_) {
            throw std::logic_error(
                "V4ResidentExpertExecutor: accumulate_routed_batch without a matching batch dispatch");
        }
        const aeon_moe_layer& layer = layers_[layer_id];
        if (batch_ids == nullptr || ids_stride != layer.top_k || weights_stride != layer.top_k) {
            throw std::invalid_argument(
                "V4ResidentExpertExecutor: batch ids and weights must be [token, top_k]");
        }
        aeon355::throw_on_error(aeon_moe_layer_routed(
            &layer, batch_input, input_stride, static_cast<int>(token_count), batch_ids,
            batch_weights, batch_output, output_stride, workspace_, workspace_bytes_, stream_));
    }

private:
    void check_token(uint32_t layer_id, uint32_t position, const char* who) const {
        if (current_layer_ != static_cast<int64_t>(layer_id)) {
            throw std::logic_error(std::string("V4ResidentExpertExecutor: ") + who +
                                   " without a matching on_routing_ready");
        }
        if (position < first_position_) {
            throw std::logic_error("V4ResidentExpertExecutor: consume before the batch's first position");
        }
        if (position - first_position_ >= token_count_) {
            throw std::out_of_range("V4ResidentExpertExecutor: token index past the batch's token count");
        }
    }

    std::vector<aeon_moe_layer> layers_;
    int max_tokens_;
    hipStream_t stream_;
    void* workspace_{nullptr};
    size_t workspace_bytes_{0};
    int32_t* d_ids_{nullptr};
    std::vector<int32_t> host_ids_;
    int64_t current_layer_{-1};
    uint32_t first_position_{0};
    uint32_t token_count_{0};
};

}  // namespace aeon::core
