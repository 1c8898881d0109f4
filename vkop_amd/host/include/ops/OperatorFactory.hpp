// create_from_type: the reference's factory (ops/OperatorFactory.hpp:56-143)
// for the operators this build implements; every other kind gives nullptr,
// which is the reference's answer for a kind it does not know.
#ifndef VKOP_HIP_OPS_OPERATOR_FACTORY_HPP_
#define VKOP_HIP_OPS_OPERATOR_FACTORY_HPP_

#include <memory>

#include "ops/Operator.hpp"
#include "ops/Nms.hpp"
#include "ops/Reduce.hpp"
#include "ops/Softmax.hpp"
#include "ops/Topk.hpp"

namespace vkop {
namespace ops {

static inline std::unique_ptr<Operator> create_from_type(OpType type, bool use_ssbo = false, int fp16 = 0,
                                                         bool use_tensorcore = false) {
    (void)use_tensorcore;
    switch (type) {
    case OpType::TOPK:
        return std::make_unique<Topk>(fp16);
    case OpType::SOFTMAX:
        return std::make_unique<Softmax>(use_ssbo);
    case OpType::NMS:
        return std::make_unique<Nms>();
    case OpType::REDUCE:
        return std::make_unique<Reduce>();
    default:
        return nullptr;
    }
}

}  // namespace ops
}  // namespace vkop
#endif  // VKOP_HIP_OPS_OPERATOR_FACTORY_HPP_
