// Reduce operator: ops/Reduce.hpp:12-154 over vkop_hip_reduce_max, and the
// Softmax + Reduce(max) pair over the same axis as one operator over
// vkop_hip_softmax_reduce_max.
//
// The reference's Reduce runs on 4-D images for ten kinds of reduction; the
// detection-style post-processing (class maximum of the class probabilities,
// example/yolo/main.cpp:60-127) needs one of them, "max" along one axis, on
// buffers of any rank up to four.  That is what is here: every attribute is
// read as the reference reads it, and executing any other kind, or a
// reduction over several axes at once, is an error that says so.
#ifndef VKOP_HIP_OPS_REDUCE_HPP_
#define VKOP_HIP_OPS_REDUCE_HPP_

#include "ops/Operator.hpp"

namespace vkop {
namespace ops {
namespace reduce {

enum class ReduceType { L1 = 0, L2, LOGSUM, LOGSUMEXP, MAX, MEAN, MIN, PROD, SUM, SUMSQUARE };  // ops/Reduce.hpp:13-24

struct GpuReduceParam {  // ops/Reduce.hpp:26-30
    ivec4 shape;
    int reduce_op;
    int axes_mask;
};

}  // namespace reduce

class Reduce : public Operator {
  public:
    Reduce() : Operator(OpType::REDUCE) {}

    // "reduce_op" (one of ten names), "axes" (a list), "keepdims" (ops/Reduce.hpp:40-76).
    void setAttribute(const std::unordered_map<std::string, std::string> &attributes) override {
        static const char *const names[] = {"l1_norm", "l2_norm", "log_sum", "log_sum_exp", "max",
                                            "mean",    "min",     "prod",    "sum",         "sum_square"};
        auto op = attributes.find("reduce_op");
        if (op != attributes.end())
            for (int i = 0; i < 10; i++)
                if (op->second == names[i]) reduce_op_ = i;
        if (attributes.find("axes") != attributes.end()) axes_ = parse_attr_list<int>(attributes.at("axes"));
        if (attributes.find("keepdims") != attributes.end()) keepdims_ = static_cast<int>(std::stol(attributes.at("keepdims")));
    }

    // Extents left after reducing `axes_input` (negative values count from the end, values outside the rank are
    // ignored); a reduced axis stays as 1 with keepdims (ops/Reduce.hpp:77-107).
    static std::vector<int> calculateOutputShape(const std::vector<int> &input_shape, const std::vector<int> &axes_input,
                                                 bool keepdims) {
        const int rank = static_cast<int>(input_shape.size());
        unsigned reduced = 0;
        for (int a : axes_input) {
            const int ax = a < 0 ? a + rank : a;
            if (ax >= 0 && ax < rank) reduced |= 1u << ax;
        }
        std::vector<int> out;
        for (int i = 0; i < rank; i++) {
            if (!((reduced >> i) & 1u)) out.push_back(input_shape[static_cast<size_t>(i)]);
            else if (keepdims) out.push_back(1);
        }
        return out;
    }

    int reduce_op() const { return reduce_op_; }
    const std::vector<int> &axes() const { return axes_; }
    int keepdims() const { return keepdims_; }

  protected:
    struct Bound {
        void *in = nullptr, *out = nullptr;
        int dtype = VKOP_HIP_F32, axis = 0;
        std::vector<int> shape;
    };

    // Checks the attributes against what the library has, sizes the output, and finds the device buffers.
    Bound bind(const std::vector<std::shared_ptr<core::ITensor>> &inputs, const std::vector<std::shared_ptr<core::ITensor>> &outputs,
               const char *who) {
        Bound b;
        b.shape = inputs[0]->getShape();
        const int rank = static_cast<int>(b.shape.size());
        if (reduce_op_ != static_cast<int>(reduce::ReduceType::MAX))
            throw std::runtime_error(std::string(who) + ": only reduce_op \"max\" is implemented");
        para_.axes_mask = 0;
        for (int a : axes_) {
            const int ax = a < 0 ? a + rank : a;
            if (ax >= 0 && ax < rank) para_.axes_mask |= 1 << ax;  // ops/Reduce.hpp:139-144
        }
        if (para_.axes_mask == 0 || (para_.axes_mask & (para_.axes_mask - 1)) != 0)
            throw std::runtime_error(std::string(who) + ": exactly one axis can be reduced at a time");
        while (!((para_.axes_mask >> b.axis) & 1)) b.axis++;
        for (int i = 0; i < 4; i++) para_.shape[i] = i < rank ? b.shape[static_cast<size_t>(i)] : 1;
        para_.reduce_op = reduce_op_;
        if (inputs[0]->dtype() != outputs[0]->dtype()) throw std::runtime_error(std::string(who) + ": input and output types differ");
        const auto out_shape = calculateOutputShape(b.shape, axes_, keepdims_ == 1);
        dispatch_by_dtype(outputs[0]->dtype(), [&](auto dummy) {
            using T = decltype(dummy);
            if constexpr (std::is_same_v<T, float> || std::is_same_v<T, uint16_t>) {
                auto output = core::as_tensor<T>(outputs[0]);
                if (output->size() == 0) output->resize(out_shape);  // ops/Reduce.hpp:119-121
                b.out = output->as_storage_buffer(m_dev_)->data();
                b.in = core::as_tensor<T>(inputs[0])->as_storage_buffer(m_dev_)->data();
                b.dtype = std::is_same_v<T, uint16_t> ? VKOP_HIP_F16 : VKOP_HIP_F32;
            } else {
                throw std::runtime_error(std::string(who) + ": unsupported element type");
            }
        });
        return b;
    }

  private:
    void execute(const std::vector<std::shared_ptr<core::ITensor>> &inputs,
                 const std::vector<std::shared_ptr<core::ITensor>> &outputs) override {
        const Bound b = bind(inputs, outputs, "Reduce");
        m_cmd_->record([=](void *stream) {
            return vkop_hip_reduce_max(b.in, b.out, b.dtype, b.shape.data(), static_cast<int>(b.shape.size()), b.axis, stream);
        });
    }

  protected:
    reduce::GpuReduceParam para_{{0, 0, 0, 0}, 0, 0};
    int reduce_op_ = 0;  // ops/Reduce.hpp:150
    std::vector<int> axes_;
    int keepdims_ = 1;
};

// max over an axis of the softmax along that axis, the softmax tensor never written.  Takes Reduce's attributes;
// reports OpType::REDUCE.
class SoftmaxReduceMax : public Reduce {
  private:
    void execute(const std::vector<std::shared_ptr<core::ITensor>> &inputs,
                 const std::vector<std::shared_ptr<core::ITensor>> &outputs) override {
        const Bound b = bind(inputs, outputs, "Softmax+Reduce");
        const size_t ws_bytes = vkop_hip_softmax_reduce_max_workspace_bytes(b.dtype, b.shape.data(), static_cast<int>(b.shape.size()), b.axis);
        void *ws = workspace(ws_bytes);
        const size_t ws_size = workspace_size();
        m_cmd_->record([=](void *stream) {
            return vkop_hip_softmax_reduce_max(b.in, b.out, b.dtype, b.shape.data(), static_cast<int>(b.shape.size()), b.axis, ws,
                                               ws_size, stream);
        });
    }
};

}  // namespace ops
}  // namespace vkop
#endif  // VKOP_HIP_OPS_REDUCE_HPP_
