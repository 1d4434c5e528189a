#pragma once
// The routed-expert seam of the layer body, src/architecture/deepseek_v4/layer/
// v4_layer_body_moe.hpp:32-112.
//
// When the reference tree follows this directory on the include path, this file steps aside:
// the reference's own header is taken whole (#include_next), so the layer body keeps
// dispatch_router, run_layer_body_router, run_layer_body_moe_shared_expert,
// run_layer_body_moe_post and run_layer_body_moe_and_post (:124-312) and its one definition of
// V4RoutedExpertExecutor, and nothing is added to it. Built without the reference tree (the
// gates of the resident executor), only the interface is declared here, with the reference's
// method names, argument meaning and defaults.
#if __has_include_next("architecture/deepseek_v4/layer/v4_layer_body_moe.hpp")
#include_next "architecture/deepseek_v4/layer/v4_layer_body_moe.hpp"
#else
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <vector>

namespace aeon::core {

class V4RoutedExpertExecutor {
public:
    virtual ~V4RoutedExpertExecutor() = default;

    // Once the routed ids are known and before any device work for the MoE.
    virtual void on_routing_ready(uint32_t layer_id, uint32_t position,
                                  const std::vector<int32_t>& ids,
                                  const std::vector<float>& weights) {
        (void)layer_id; (void)position; (void)ids; (void)weights;
    }

    // The layer-wide form; by default the per-token sequence.
    virtual void on_routing_ready_batch(uint32_t layer_id, uint32_t first_position,
                                        const std::vector<std::vector<int32_t>>& ids,
                                        const std::vector<std::vector<float>>& weights) {
        for (size_t i = 0; i < ids.size(); ++i) {
            on_routing_ready(layer_id, first_position + static_cast<uint32_t>(i), ids[i], weights[i]);
        }
    }

    // moe_accum (already holding the shared expert's output) += sum_k w_k * expert_k(expert_input)
    // in slot order, fp32, one rounding. expert_weights is a device fp32 vector.
    virtual void accumulate_routed(uint32_t layer_id, uint32_t position, const half* expert_input,
                                   const float* expert_weights, half* moe_accum) = 0;

    // The chunk-wide form over strided rows; by default the per-token sequence.
    virtual void accumulate_routed_batch(uint32_t layer_id, uint32_t first_position,
                                         uint32_t token_count, const half* batch_input,
                                         int input_stride, const int* batch_ids, int ids_stride,
                                         const float* batch_weights, int weights_stride,
                                         half* batch_output, int output_stride) {
        (void)batch_ids; (void)ids_stride;
        for (uint32_t t = 0; t < token_count; ++t) {
            accumulate_routed(layer_id, first_position + t,
                              batch_input + static_cast<size_t>(t) * input_stride,
                              batch_weights + static_cast<size_t>(t) * weights_stride,
                              batch_output + static_cast<size_t>(t) * output_stride);
        }
    }

    virtual void on_routed_consumed(uint32_t layer_id, uint32_t position) {
        (void)layer_id; (void)position;
    }
};

}  // namespace aeon::core
#endif
