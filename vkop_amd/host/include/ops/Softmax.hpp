// Softmax operator: ops/Softmax.hpp:14-145 over vkop_hip_softmax.
#ifndef VKOP_HIP_OPS_SOFTMAX_HPP_
#define VKOP_HIP_OPS_SOFTMAX_HPP_

#include "ops/Operator.hpp"

namespace vkop {
namespace ops {
namespace softmax {

// The reference's push-constant block (ops/Softmax.hpp:16-22), kept as the
// operator's parameter record.
struct GpuSoftMaxParam {
    ivec4 outShape;
    int axis;
    int fp16;
    int nanwhere;
    float nanvalue;
};

}  // namespace softmax

class Softmax : public Operator {
  public:
    // use_ssbo chose between the buffer and the image shader in the reference;
    // here every tensor is a buffer, so both values behave the same.
    explicit Softmax(bool use_ssbo = false) : Operator(OpType::SOFTMAX), use_ssbo_(use_ssbo) {
        para_ = softmax::GpuSoftMaxParam{{0, 0, 0, 0}, 0, 0, 0, 0.0f};
    }

    // "axis" or "dim", "nan_optimization" (presence switches it on),
    // "nan_replacement_value".  The reference reads only the first of these that
    // is present (an else-if chain, ops/Softmax.hpp:46-58); here each key that is
    // present takes effect, which gives the same result whenever one key is passed.
    void setAttribute(const std::unordered_map<std::string, std::string> &attributes) override {
        if (attributes.find("axis") != attributes.end()) para_.axis = static_cast<int>(std::stol(attributes.at("axis")));
        else if (attributes.find("dim") != attributes.end()) para_.axis = static_cast<int>(std::stol(attributes.at("dim")));
        if (attributes.find("nan_optimization") != attributes.end()) para_.nanwhere = 1;
        if (attributes.find("nan_replacement_value") != attributes.end())
            para_.nanvalue = std::stof(attributes.at("nan_replacement_value"));
    }

  private:
    void execute(const std::vector<std::shared_ptr<core::ITensor>> &inputs,
                 const std::vector<std::shared_ptr<core::ITensor>> &outputs) override {
        const auto shape = inputs[0]->getShape();
        const int rank = inputs[0]->num_dims();
        if (inputs[0]->dtype() != outputs[0]->dtype()) throw std::runtime_error("Softmax: input and output types differ");

        void *in_ptr = nullptr, *out_ptr = nullptr;
        dispatch_by_dtype(outputs[0]->dtype(), [&](auto dummy) {
            using T = decltype(dummy);
            if constexpr (std::is_same_v<T, float> || std::is_same_v<T, uint16_t>) {
                auto output = core::as_tensor<T>(outputs[0]);
                if (output->size() == 0) output->resize(shape);  // ops/Softmax.hpp:71-73
                out_ptr = output->as_storage_buffer(m_dev_)->data();
                auto input = core::as_tensor<T>(inputs[0]);
                in_ptr = input->as_storage_buffer(m_dev_)->data();
                para_.fp16 = std::is_same_v<T, uint16_t> ? 1 : 0;  // ops/Softmax.hpp:92-96
            } else {
                throw std::runtime_error("Softmax: unsupported element type");
            }
        });
        for (int i = 0; i < 4; i++) para_.outShape[i] = i < rank ? shape[static_cast<size_t>(i)] : 1;
        if (para_.axis < 0) para_.axis += rank;  // ops/Softmax.hpp:111-113
        // a vector is one row (ops/Softmax.hpp:116-120)
        std::vector<int> view = shape;
        int axis = para_.axis;
        if (rank == 1) {
            view = {1, shape[0]};
            axis = 1;
            para_.outShape[0] = 1;
            para_.outShape[1] = shape[0];
            para_.axis = 1;
        }
        assert(axis >= 0 && axis < static_cast<int>(view.size()));

        const int dtype = para_.fp16 ? VKOP_HIP_F16 : VKOP_HIP_F32;
        const int nan_where = para_.nanwhere;
        const float nan_value = para_.nanvalue;
        const size_t ws_bytes = vkop_hip_softmax_workspace_bytes(dtype, view.data(), static_cast<int>(view.size()), axis);
        void *ws = workspace(ws_bytes);
        const size_t ws_size = workspace_size();
        m_cmd_->record([=](void *stream) {
            return vkop_hip_softmax(in_ptr, out_ptr, dtype, view.data(), static_cast<int>(view.size()), axis, nan_where,
                                    nan_value, ws, ws_size, stream);
        });
    }

    softmax::GpuSoftMaxParam para_;
    bool use_ssbo_;
};

}  // namespace ops
}  // namespace vkop
#endif  // VKOP_HIP_OPS_SOFTMAX_HPP_
