// Nms operator: ops/Nms.hpp:15-118 over vkop_hip_nms.
#ifndef VKOP_HIP_OPS_NMS_HPP_
#define VKOP_HIP_OPS_NMS_HPP_

#include "ops/Operator.hpp"

namespace vkop {
namespace ops {
namespace nms {

// The reference's push-constant block (ops/Nms.hpp:16-24), kept as the
// operator's parameter record.
struct GpuNMSParam {
    int num_batch;
    int num_class;
    int num_spatial;
    int center_point_box;
    int max_output_boxes_per_class;
    float iou_threshold;
    float score_threshold;
};

}  // namespace nms

// inputs: boxes [B,N,4], scores [B,C,N] (float or half bits); output: Tensor<int>
// [M,3] of (batch, class, box index) records.  The records come in order of batch,
// class and selection and are followed by a (-1,-1,-1) record when the tensor has
// room (the reference appends in scheduling order through an atomic counter).
class Nms : public Operator {
  public:
    Nms() : Operator(OpType::NMS) { para_ = nms::GpuNMSParam{0, 0, 0, 0, 0, 0.0f, 0.0f}; }

    // "center_point_box", "iou_threshold", "score_threshold",
    // "max_output_boxes_per_class" (ops/Nms.hpp:45-64)
    void setAttribute(const std::unordered_map<std::string, std::string> &attributes) override {
        if (attributes.find("center_point_box") != attributes.end())
            para_.center_point_box = static_cast<int>(std::stol(attributes.at("center_point_box")));
        if (attributes.find("iou_threshold") != attributes.end()) para_.iou_threshold = std::stof(attributes.at("iou_threshold"));
        if (attributes.find("score_threshold") != attributes.end())
            para_.score_threshold = std::stof(attributes.at("score_threshold"));
        if (attributes.find("max_output_boxes_per_class") != attributes.end())
            para_.max_output_boxes_per_class = static_cast<int>(std::stol(attributes.at("max_output_boxes_per_class")));
    }

    // Records the last run produced (all of them, also when the output tensor
    // holds fewer), after the recorded work has been submitted and waited for.
    int selected_count(const std::shared_ptr<VulkanCommandPool> &pool) {
        int host[2] = {0, 0};
        if (count_ == nullptr) return 0;
        void *q = pool->getDevice()->getComputeQueue(0);
        if (vkop_hip_memcpy_d2h(host, count_, sizeof host, q) != VKOP_HIP_OK)
            throw std::runtime_error(std::string("Nms: ") + vkop_hip_last_error());
        return host[0];
    }

  private:
    void execute(const std::vector<std::shared_ptr<core::ITensor>> &inputs,
                 const std::vector<std::shared_ptr<core::ITensor>> &outputs) override {
        const auto box_shape = inputs[0]->getShape();
        const auto score_shape = inputs[1]->getShape();
        assert(box_shape.size() == 3 && score_shape.size() == 3 && box_shape[2] == 4);  // ops/Nms.hpp:80
        const int batch = box_shape[0], num_boxes = box_shape[1], num_class = score_shape[1];
        if (inputs[0]->dtype() != inputs[1]->dtype()) throw std::runtime_error("Nms: boxes and scores differ in type");

        auto output = core::as_tensor<int>(outputs[0]);
        if (!output) throw std::runtime_error("Nms: outputs[0] must be a Tensor<int>");
        if (output->size() == 0) {  // ops/Nms.hpp:84-91
            int output_num = 100;
            if (para_.max_output_boxes_per_class > 0) output_num = para_.max_output_boxes_per_class * num_class;
            output->resize(std::vector<int>{output_num, 3});
        }
        int32_t *out_ptr = static_cast<int32_t *>(output->as_storage_buffer(m_dev_)->data());
        const int capacity = output->num_elements() / 3;

        void *boxes = nullptr, *scores = nullptr;
        int dtype = VKOP_HIP_F32;
        dispatch_by_dtype(inputs[0]->dtype(), [&](auto dummy) {
            using T = decltype(dummy);
            if constexpr (std::is_same_v<T, float> || std::is_same_v<T, uint16_t>) {
                boxes = core::as_tensor<T>(inputs[0])->as_storage_buffer(m_dev_)->data();
                scores = core::as_tensor<T>(inputs[1])->as_storage_buffer(m_dev_)->data();
                dtype = std::is_same_v<T, uint16_t> ? VKOP_HIP_F16 : VKOP_HIP_F32;
            } else {
                throw std::runtime_error("Nms: unsupported element type");
            }
        });
        para_.num_batch = batch;
        para_.num_class = num_class;
        para_.num_spatial = num_boxes;

        // the two counters live behind the operator's workspace
        const size_t ws_bytes = vkop_hip_nms_workspace_bytes(batch, num_class, num_boxes, para_.max_output_boxes_per_class);
        char *ws = static_cast<char *>(workspace(ws_bytes + 256));
        const size_t ws_size = workspace_size() - 256;
        count_ = reinterpret_cast<int32_t *>(ws + ws_size);
        int32_t *count = count_;
        const nms::GpuNMSParam p = para_;
        m_cmd_->record([=](void *stream) {
            return vkop_hip_nms(boxes, scores, out_ptr, capacity, count, dtype, p.num_batch, p.num_class, p.num_spatial,
                                p.center_point_box, p.max_output_boxes_per_class, p.iou_threshold, p.score_threshold, ws,
                                ws_size, stream);
        });
    }

    nms::GpuNMSParam para_;
    int32_t *count_ = nullptr;
};

}  // namespace ops
}  // namespace vkop
#endif  // VKOP_HIP_OPS_NMS_HPP_
