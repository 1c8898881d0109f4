// Operator kinds and their names: the numbering and spelling of the reference
// (ops/Ops.hpp:11-189), because models, logs and callers refer to operators by
// these values.  Only SOFTMAX and TOPK have an implementation in this build;
// the other enumerators exist so that the numbering stays the reference's.
#ifndef VKOP_HIP_OPS_OPS_HPP_
#define VKOP_HIP_OPS_OPS_HPP_

#include <string>

namespace vkop {
namespace ops {

// X(enumerator, canonical name, alias accepted when parsing or nullptr)
#define VKOP_OP_TABLE(X)                                   \
    X(UNKNOWN, "Unknown", nullptr)                         \
    X(ADD, "Add", nullptr)                                 \
    X(ATAN, "Atan", nullptr)                               \
    X(AVERAGEPOOL, "AveragePool", nullptr)                 \
    X(BATCHNORM, "BatchNorm", "BatchNormalization")        \
    X(COL2IM, "Col2Im", nullptr)                           \
    X(CONCAT, "Concat", nullptr)                           \
    X(CONV2D, "Conv2d", "Conv")                            \
    X(DIV, "Div", nullptr)                                 \
    X(ERF, "Erf", nullptr)                                 \
    X(FLOOR, "Floor", nullptr)                             \
    X(GEMM, "Gemm", nullptr)                               \
    X(GLOBALAVERAGEPOOL, "GlobalAveragePool", nullptr)     \
    X(GRIDSAMPLE, "GridSample", nullptr)                   \
    X(LAYERNORM, "LayerNorm", "LayerNormalization")        \
    X(MATMUL, "MatMul", nullptr)                           \
    X(MAXPOOL2D, "MaxPool2d", "MaxPool")                   \
    X(MUL, "Mul", nullptr)                                 \
    X(POW, "Pow", nullptr)                                 \
    X(PRELU, "PRelu", nullptr)                             \
    X(REDUCE, "Reduce", nullptr)                           \
    X(RELU, "Relu", nullptr)                               \
    X(RESHAPE, "Reshape", nullptr)                         \
    X(RESIZE, "Resize", nullptr)                           \
    X(SIGMOID, "Sigmoid", nullptr)                         \
    X(SLICE, "Slice", nullptr)                             \
    X(SOFTMAX, "Softmax", nullptr)                         \
    X(SOFTPLUS, "Softplus", nullptr)                       \
    X(SPLIT, "Split", nullptr)                             \
    X(SUB, "Sub", nullptr)                                 \
    X(TOPK, "TopK", nullptr)                               \
    X(TRANSPOSE, "Transpose", nullptr)                     \
    X(NMS, "Nms", nullptr)                                 \
    X(GATHER, "Gather", nullptr)                           \
    X(RANGE, "Range", nullptr)                             \
    X(EXPAND, "Expand", nullptr)                           \
    X(SQRT, "Sqrt", nullptr)                               \
    X(SIN, "Sin", nullptr)                                 \
    X(COS, "Cos", nullptr)                                 \
    X(NEG, "Neg", nullptr)                                 \
    X(WHERE, "Where", nullptr)

enum class OpType {
#define VKOP_OP_ENUM(e, name, alias) e,
    VKOP_OP_TABLE(VKOP_OP_ENUM)
#undef VKOP_OP_ENUM
        TOTAL_NUM
};

static_assert(static_cast<int>(OpType::SOFTMAX) == 26 && static_cast<int>(OpType::TOPK) == 30,
              "operator numbering must stay the reference's (ops/Ops.hpp:11-54)");

// Out-of-range values name the unknown operator (ops/Ops.hpp:100-102).
inline std::string convert_optype_to_string(const OpType &type) {
    switch (type) {
#define VKOP_OP_NAME(e, name, alias) \
    case OpType::e:                  \
        return name;
        VKOP_OP_TABLE(VKOP_OP_NAME)
#undef VKOP_OP_NAME
    default:
        return "Unknown";
    }
}

// Unrecognised names give UNKNOWN (ops/Ops.hpp:105-189); "Unknown" itself is not a name.
inline OpType convert_opstring_to_enum(const std::string &name) {
#define VKOP_OP_PARSE(e, canonical, alias)                                                         \
    if (OpType::e != OpType::UNKNOWN && (name == canonical || (alias != nullptr && name == static_cast<const char *>(alias)))) \
        return OpType::e;
    VKOP_OP_TABLE(VKOP_OP_PARSE)
#undef VKOP_OP_PARSE
    return OpType::UNKNOWN;
}

}  // namespace ops
}  // namespace vkop
#endif  // VKOP_HIP_OPS_OPS_HPP_
