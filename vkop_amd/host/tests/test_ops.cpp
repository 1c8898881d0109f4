// Tests of the C++ operator interface, in the shape of the reference's own:
// tests/setup.hpp:107-294 (TestCase::run_test), tests/SoftmaxTest.cpp:100-230 and
// tests/TopkTest.cpp:40-127 -- same case lists, same seeds, expectations from
// libtorch's CPU softmax / topk computed at test time, same comparison rules
// (exact for integers, the three-band float tolerance), plus a stricter ulp bound
// and cases for the fused operator.  No test framework: each check prints a line
// and the process exits non-zero if any failed.
//
//   test_ops            all tests (needs an MI355X)
//   test_ops --no-gpu   host-side logic only
#include <torch/torch.h>

#include <cmath>
#include <cstdio>
#include <algorithm>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <functional>
#include <iterator>
#include <string>

#include "core/Runtime.hpp"
#include "ops/OperatorFactory.hpp"

using vkop::core::ITensor;
using vkop::core::Tensor;
namespace ops = vkop::ops;

static int g_failed = 0, g_checked = 0;
#define EXPECT(cond)                                                         \
    do {                                                                     \
        g_checked++;                                                         \
        if (!(cond)) {                                                       \
            g_failed++;                                                      \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);     \
        }                                                                    \
    } while (0)

static int64_t ulp_distance(float a, float b) {
    int32_t ia, ib;
    std::memcpy(&ia, &a, 4);
    std::memcpy(&ib, &b, 4);
    if (ia < 0) ia = static_cast<int32_t>(0x80000000u) - ia;
    if (ib < 0) ib = static_cast<int32_t>(0x80000000u) - ib;
    return std::llabs(static_cast<int64_t>(ia) - static_cast<int64_t>(ib));
}

struct TestEnv {
    static std::shared_ptr<vkop::VulkanDevice> dev;
    static std::shared_ptr<vkop::VulkanCommandPool> pool;
    static void initialize() {
        if (dev) return;
        dev = std::make_shared<vkop::VulkanDevice>(0);
        pool = std::make_shared<vkop::VulkanCommandPool>(dev);
        std::printf("device: %s, %d CUs\n", dev->getDeviceName().c_str(), dev->getComputeUnits());
    }
};
std::shared_ptr<vkop::VulkanDevice> TestEnv::dev;
std::shared_ptr<vkop::VulkanCommandPool> TestEnv::pool;

// float <-> kFloat32, uint16_t <-> kFloat16 bit copy, int <-> kInt (tests/setup.hpp:107-127)
template <typename TT> void fill_from_torch(std::shared_ptr<Tensor<TT>> &tensor, const torch::Tensor &t) {
    auto cpu = t.cpu().contiguous().flatten();
    std::vector<TT> data(static_cast<size_t>(cpu.numel()));
    if constexpr (std::is_same_v<TT, uint16_t>) std::memcpy(data.data(), cpu.data_ptr<at::Half>(), data.size() * 2);
    else std::memcpy(data.data(), cpu.data_ptr<TT>(), data.size() * sizeof(TT));
    tensor->fillToCPU(data);
}

template <typename T> struct TestCase {
    std::string name;
    int64_t max_ulp = 0;  // worst float distance seen (float outputs only)
    explicit TestCase(std::string n) : name(std::move(n)) { TestEnv::initialize(); }
    torch::TensorOptions conf() const {
        return torch::TensorOptions().dtype(std::is_same_v<T, float> ? torch::kFloat32 : torch::kFloat16);
    }

    // create -> set device -> attributes -> upload -> record -> submit -> wait ->
    // read back -> compare (tests/setup.hpp:129-294)
    bool run_test(const std::vector<std::shared_ptr<ITensor>> &inputs,
                  const std::vector<std::shared_ptr<ITensor>> &expect_outputs,
                  const std::function<void(std::unique_ptr<ops::Operator> &)> &attribute_func = nullptr,
                  std::unique_ptr<ops::Operator> op = nullptr) {
        auto dev = TestEnv::dev;
        auto pool = TestEnv::pool;
        if (!op)
            op = ops::create_from_type(ops::convert_opstring_to_enum(name), inputs[0]->num_dims() <= 2,
                                       typeid(T) == typeid(uint16_t) ? 1 : 0, dev->is_support_nv_tensor_core());
        if (!op) return false;
        op->set_runtime_device(dev, pool);
        if (attribute_func) attribute_func(op);
        std::vector<std::shared_ptr<ITensor>> outputs;
        for (const auto &e : expect_outputs) {
            if (e->dtype() == typeid(float)) {
                auto o = std::make_shared<Tensor<float>>(true);
                o->resize(e->getShape());
                outputs.push_back(o);
            } else if (e->dtype() == typeid(uint16_t)) {
                auto o = std::make_shared<Tensor<uint16_t>>(true);
                o->resize(e->getShape());
                outputs.push_back(o);
            } else if (e->dtype() == typeid(int)) {
                auto o = std::make_shared<Tensor<int>>(true);
                o->resize(e->getShape());
                outputs.push_back(o);
            } else {
                return false;
            }
        }
        for (const auto &in : inputs) {
            auto t = vkop::core::as_tensor<T>(in);
            t->as_storage_buffer(dev);
            t->copyToGPU(pool);
        }
        op->onExecute(inputs, outputs, 0);
        auto cmd = op->get_record();
        vkop::VulkanCommandBuffer::submit(dev->getComputeQueue(), {cmd->buildSubmitInfo()});
        cmd->wait();
        dev->wait_all_done();

        auto check = [&](size_t idx, auto tag) -> bool {
            using TT = decltype(tag);
            auto out = vkop::core::as_tensor<TT>(outputs[idx]);
            out->copyToCPU(pool);
            auto exp = vkop::core::as_tensor<TT>(expect_outputs[idx]);
            if (out->num_elements() != exp->num_elements()) return false;
            for (int i = 0; i < out->num_elements(); i++) {
                if constexpr (std::is_same_v<TT, int>) {
                    if ((*out)[i] != (*exp)[i]) {
                        std::printf("  index mismatch at %d: %d vs %d\n", i, (*out)[i], (*exp)[i]);
                        return false;
                    }
                } else {
                    const bool half = std::is_same_v<TT, uint16_t>;
                    float o, e;
                    if constexpr (std::is_same_v<TT, uint16_t>) {
                        o = ITensor::fp16_to_fp32((*out)[i]);
                        e = ITensor::fp16_to_fp32((*exp)[i]);
                    } else {
                        o = (*out)[i];
                        e = (*exp)[i];
                    }
                    if (std::isnan(e) || std::isnan(o)) return false;
                    const float a = std::fabs(e);
                    float thr;  // the reference's bands (tests/setup.hpp:219-262)
                    if (half) thr = a > 1.0f ? a * 0.02f : 0.02f;
                    else thr = a > 1.0f ? a * 0.01f : (a > 0.001f ? std::max(0.003f, a * 0.02f) : 0.002f);
                    if (std::fabs(o - e) > thr) {
                        std::printf("  value mismatch at %d: %g vs %g\n", i, o, e);
                        return false;
                    }
                    if (!half) max_ulp = std::max(max_ulp, ulp_distance(o, e));
                    else if ((*out)[i] != (*exp)[i]) max_ulp = std::max<int64_t>(max_ulp, std::abs(int((*out)[i]) - int((*exp)[i])));
                }
            }
            return true;
        };
        for (size_t idx = 0; idx < outputs.size(); idx++) {
            bool ok = false;
            if (outputs[idx]->dtype() == typeid(float)) ok = check(idx, float{});
            else if (outputs[idx]->dtype() == typeid(uint16_t)) ok = check(idx, uint16_t{});
            else if (outputs[idx]->dtype() == typeid(int)) ok = check(idx, int{});
            if (!ok) return false;
        }
        return true;
    }
};

static torch::Tensor randn_shape(const std::vector<int> &s, const torch::TensorOptions &o) {
    std::vector<int64_t> dims(s.begin(), s.end());
    return torch::randn(dims, o);
}
static std::vector<int> shape_of(const torch::Tensor &t) {
    std::vector<int> s;
    for (int64_t i = 0; i < t.dim(); i++) s.push_back(static_cast<int>(t.size(i)));
    return s;
}

// tests/SoftmaxTest.cpp:100-230: seed 42, randn, torch::softmax along `dim`
template <typename T> void softmax_case(const std::vector<int> &shape, int axis) {
    TestCase<T> tc("Softmax");
    torch::manual_seed(42);
    auto x = randn_shape(shape, tc.conf());
    auto y = torch::softmax(x, axis < 0 ? axis + x.dim() : axis);
    auto input = std::make_shared<Tensor<T>>(shape);
    fill_from_torch(input, x);
    auto expect = std::make_shared<Tensor<T>>(shape_of(y));
    fill_from_torch(expect, y);
    const std::unordered_map<std::string, std::string> dim = {{"dim", std::to_string(axis)}};
    const bool ok = tc.run_test({input}, {expect}, [&](std::unique_ptr<ops::Operator> &op) {
        auto *sm = dynamic_cast<ops::Softmax *>(op.get());
        EXPECT(sm != nullptr);
        if (sm) sm->setAttribute(dim);
    });
    std::printf("Softmax %s shape [", std::is_same_v<T, float> ? "fp32" : "fp16");
    for (int d : shape) std::printf("%d,", d);
    std::printf("] axis %d: %s, worst distance %lld %s\n", axis, ok ? "ok" : "FAILED", static_cast<long long>(tc.max_ulp),
                std::is_same_v<T, float> ? "ulp vs libtorch" : "half steps vs libtorch");
    EXPECT(ok);
    // libtorch itself is a few ulp from the correctly rounded value on these lines
    EXPECT(tc.max_ulp <= (std::is_same_v<T, float> ? 4 : 1));
}

// tests/TopkTest.cpp:40-127: seed 56, randn [r,c], torch::topk(k, axis, largest, sorted)
template <typename T> void topk_case(const std::vector<int> &shape, int k, int axis) {
    TestCase<T> tc("TopK");
    torch::manual_seed(56);
    auto x = randn_shape(shape, tc.conf());
    auto [v, i64] = torch::topk(x, k, axis, true, true);
    auto i32 = i64.to(torch::kInt);
    auto input = std::make_shared<Tensor<T>>(shape);
    fill_from_torch(input, x);
    auto out_shape = shape_of(v);
    auto ev = std::make_shared<Tensor<T>>(out_shape);
    fill_from_torch(ev, v);
    auto ei = std::make_shared<Tensor<int>>(out_shape);
    fill_from_torch(ei, i32);
    const std::unordered_map<std::string, std::string> attrs = {
        {"k", std::to_string(k)}, {"axis", std::to_string(axis)}, {"largest", "1"}, {"sorted", "1"}};
    // Half inputs can hold equal values, where libtorch's choice of index is its
    // own.  With a tie among the first k+1 the expected indices come from a
    // stable descending sort instead (equal values: lower index first); the
    // values are the same either way.
    auto sorted = torch::sort(x.to(torch::kFloat32), /*stable=*/true, /*dim=*/-1, /*descending=*/true);
    const auto &sv = std::get<0>(sorted);
    const bool ties = (sv.slice(-1, 0, k) == sv.slice(-1, 1, k + 1)).any().template item<bool>();
    if (ties) fill_from_torch(ei, std::get<1>(sorted).slice(-1, 0, k).to(torch::kInt));
    const bool ok = tc.run_test({input}, {ev, ei}, [&](std::unique_ptr<ops::Operator> &op) {
        auto *tk = dynamic_cast<ops::Topk *>(op.get());
        EXPECT(tk != nullptr);
        if (tk) tk->setAttribute(attrs);
    });
    std::printf("TopK %s shape [%d,%d] k %d axis %d: %s%s\n", std::is_same_v<T, float> ? "fp32" : "fp16", shape[0], shape[1],
                k, axis, ok ? "ok" : "FAILED", ties ? " (equal values among the first k+1: indices from a stable sort)" : "");
    EXPECT(ok);
    EXPECT(tc.max_ulp == 0);  // values are copies of input elements
}

// The fused operator against top-k of libtorch's softmax evaluated in float64 and
// rounded once to the tensor type (libtorch's float32 softmax accumulates in
// float32 and is itself tens of ulp off on 128K-long rows).  Equal probabilities:
// lower index first, which a stable descending sort gives.
template <typename T> void fused_case(const std::vector<int> &shape, int k) {
    TestCase<T> tc("TopK");
    torch::manual_seed(7);
    auto x = randn_shape(shape, tc.conf()) * 3;
    auto p = torch::softmax(x.to(torch::kFloat64), -1).to(tc.conf().dtype());
    auto sorted = torch::sort(p.to(torch::kFloat32), /*stable=*/true, /*dim=*/-1, /*descending=*/true);
    auto v = std::get<0>(sorted).slice(-1, 0, k).to(tc.conf().dtype());
    auto i64 = std::get<1>(sorted).slice(-1, 0, k);
    auto input = std::make_shared<Tensor<T>>(shape);
    fill_from_torch(input, x);
    auto ev = std::make_shared<Tensor<T>>(shape_of(v));
    fill_from_torch(ev, v);
    auto ei = std::make_shared<Tensor<int>>(shape_of(v));
    fill_from_torch(ei, i64.to(torch::kInt));
    const std::unordered_map<std::string, std::string> attrs = {{"k", std::to_string(k)}, {"axis", "-1"}};
    const bool ok = tc.run_test({input}, {ev, ei}, [&](std::unique_ptr<ops::Operator> &op) { op->setAttribute(attrs); },
                                std::make_unique<ops::SoftmaxTopk>(std::is_same_v<T, uint16_t> ? 1 : 0));
    std::printf("Softmax+TopK %s shape [%d,%d] k %d: %s, worst distance %lld\n", std::is_same_v<T, float> ? "fp32" : "fp16",
                shape[0], shape[1], k, ok ? "ok" : "FAILED", static_cast<long long>(tc.max_ulp));
    EXPECT(ok);
    EXPECT(tc.max_ulp <= 2);
}

// tests/NmsTest.cpp:62-160: per (batch, class) the boxes at or above the score
// threshold, best first, each kept box removing the later ones whose IoU with it
// exceeds the threshold.  Written here over an IoU matrix and a sort of the whole score row.
static std::vector<int> nms_expectation(const torch::Tensor &boxes, const torch::Tensor &scores, float iou_thr, float score_thr) {
    auto bf = boxes.to(torch::kFloat32), sf = scores.to(torch::kFloat32);
    const int64_t B = bf.size(0), N = bf.size(1), C = sf.size(1);
    std::vector<int> records;
    for (int64_t b = 0; b < B; b++) {
        auto x1 = bf[b].select(-1, 0), y1 = bf[b].select(-1, 1), x2 = bf[b].select(-1, 2), y2 = bf[b].select(-1, 3);
        auto area = (x2 - x1) * (y2 - y1);
        auto w = torch::clamp_min(torch::min(x2.unsqueeze(1), x2.unsqueeze(0)) - torch::max(x1.unsqueeze(1), x1.unsqueeze(0)), 0);
        auto h = torch::clamp_min(torch::min(y2.unsqueeze(1), y2.unsqueeze(0)) - torch::max(y1.unsqueeze(1), y1.unsqueeze(0)), 0);
        auto inter = w * h;
        auto uni = area.unsqueeze(1) + area.unsqueeze(0) - inter;
        auto iou = torch::where(uni > 1e-8F, inter / uni, torch::zeros_like(inter)).contiguous();
        const float *m = iou.template data_ptr<float>();
        for (int64_t c = 0; c < C; c++) {
            auto order = std::get<1>(torch::sort(sf[b][c], /*stable=*/true, /*dim=*/0, /*descending=*/true)).contiguous();
            const int64_t *o = order.template data_ptr<int64_t>();
            std::vector<char> dead(static_cast<size_t>(N), 0);
            for (int64_t p = 0; p < N; p++) {
                if (sf[b][c][o[p]].template item<float>() < score_thr) break;
                if (dead[static_cast<size_t>(p)]) continue;
                records.insert(records.end(), {static_cast<int>(b), static_cast<int>(c), static_cast<int>(o[p])});
                for (int64_t q = p + 1; q < N; q++)
                    if (m[o[p] * N + o[q]] > iou_thr) dead[static_cast<size_t>(q)] = 1;
            }
        }
    }
    return records;
}

// tests/NmsTest.cpp:29-160: boxes from uniform centres and sizes, uniform scores;
// expectation: per (batch, class) the boxes at or above the score threshold, best
// first, each kept box removing the later ones whose IoU with it exceeds the
// threshold.  Written here over an IoU matrix and a sort of the whole score row.
template <typename T>
void nms_case(const std::vector<int> &box_shape, const std::vector<int> &score_shape, int per_class, float iou_thr,
              float score_thr) {
    TestCase<T> tc("Nms");
    torch::manual_seed(11);
    const int64_t B = box_shape[0], N = box_shape[1], C = score_shape[1];
    auto scores = torch::rand({B, C, N}, tc.conf());
    auto centre = torch::rand({B, N, 2}, tc.conf()), size = torch::rand({B, N, 2}, tc.conf()) * 1.3F;
    auto boxes = torch::cat({torch::clamp(centre - size / 2, 0.0F, 1.0F), torch::clamp(centre + size / 2, 0.0F, 1.0F)}, -1);
    std::vector<int> records = nms_expectation(boxes, scores, iou_thr, score_thr);
    auto in_boxes = std::make_shared<Tensor<T>>(box_shape);
    fill_from_torch(in_boxes, boxes);
    auto in_scores = std::make_shared<Tensor<T>>(score_shape);
    fill_from_torch(in_scores, scores);
    const int M = static_cast<int>(records.size() / 3);
    auto expect = std::make_shared<Tensor<int>>(std::vector<int>{M, 3});
    expect->fillToCPU(records);
    const std::unordered_map<std::string, std::string> attrs = {{"max_output_boxes_per_class", std::to_string(per_class)},
                                                                {"iou_threshold", std::to_string(iou_thr)},
                                                                {"score_threshold", std::to_string(score_thr)}};
    bool ok = M > 0;
    if (M > 0)
        ok = tc.run_test({in_boxes, in_scores}, {expect}, [&](std::unique_ptr<ops::Operator> &op) {
            auto *nms = dynamic_cast<ops::Nms *>(op.get());
            EXPECT(nms != nullptr);
            if (nms) nms->setAttribute(attrs);
        });
    std::printf("Nms %s boxes [%d,%d,4] classes %d: %s, %d records\n", std::is_same_v<T, float> ? "fp32" : "fp16", box_shape[0],
                box_shape[1], score_shape[1], ok ? "ok" : "FAILED", M);
    EXPECT(ok);
}

// An operator written against the reference's base class as it stands
// (ops/Operator.hpp:21-23 constructor, 225-238 submit; the calling pattern of
// ops/Softmax.hpp:33-44,120-128): a SPIR-V blob, the kinds of its bindings and the size
// of its push constants go to the base constructor, execute() collects the bound
// resources in objs_ and ends in submit(&pc, gx, gy, gz).  It has to compile and run
// against this library's base unchanged.
namespace {
struct DummyPush {
    int n;
    float alpha;
};
uint8_t g_dummy_spv[8] = {0x03, 0x02, 0x23, 0x07, 0, 0, 1, 0};

class ReferenceStyleOp : public ops::Operator {
  public:
    explicit ReferenceStyleOp(bool own_submit)
        : Operator(ops::OpType::RELU, g_dummy_spv, sizeof(g_dummy_spv),
                   {VK_DESCRIPTOR_TYPE_STORAGE_IMAGE, VK_DESCRIPTOR_TYPE_COMBINED_IMAGE_SAMPLER, DESCRIPTOR_TYPE_STORAGE},
                   sizeof(DummyPush)),
          own_submit_(own_submit) {}

    // what execute() does between collecting its resources and returning, callable
    // without a device
    void record(int n) {
        DummyPush pc{n, 0.5F};
        objs_.emplace_back(std::shared_ptr<vkop::VulkanResource>());
        if (types_[2] == DESCRIPTOR_TYPE_STORAGE) submit(&pc, (n + 255) / 256, 1, 1);
        else submit(&pc, (n + 15) / 16, 16, 1);
    }
    size_t pc_size() const { return pc_size_; }
    size_t bindings() const { return types_.size(); }
    size_t collected() const { return objs_.size(); }
    DummyPush seen_pc{};
    int seen_grid[3] = {0, 0, 0};

  protected:
    void submit(void *ptr, int width, int height, int layers) override {
        if (!own_submit_) {
            Operator::submit(ptr, width, height, layers);
            return;
        }
        std::memcpy(&seen_pc, ptr, pc_size_);
        seen_grid[0] = width;
        seen_grid[1] = height;
        seen_grid[2] = layers;
    }

  private:
    void execute(const std::vector<std::shared_ptr<ITensor>> &inputs,
                 const std::vector<std::shared_ptr<ITensor>> &outputs) override {
        (void)outputs;
        record(inputs[0]->size() / 4);
    }
    bool own_submit_;
};
}  // namespace

static void reference_base_class_tests() {
    const int before = ops::Operator::instance_count_.load();
    {
        ReferenceStyleOp op(true);
        EXPECT(ops::Operator::instance_count_.load() == before + 1);
        EXPECT(op.get_type() == ops::OpType::RELU);
        EXPECT(op.pc_size() == sizeof(DummyPush) && op.bindings() == 3);
        op.record(1000);
        EXPECT(op.seen_pc.n == 1000 && op.seen_pc.alpha == 0.5F);
        EXPECT(op.seen_grid[0] == 4 && op.seen_grid[1] == 1 && op.seen_grid[2] == 1);
        EXPECT(op.collected() == 1);
    }
    {
        // the base submit has no pipeline to dispatch: it refuses, naming the operator
        ReferenceStyleOp op(false);
        std::string msg;
        try {
            op.record(64);
        } catch (const std::runtime_error &e) {
            msg = e.what();
        }
        EXPECT(msg.find("Relu") != std::string::npos);
        EXPECT(msg.find("1x1x1") != std::string::npos);
    }
    EXPECT(ops::Operator::instance_count_.load() == before);
}

static void host_logic_tests() {
    // names and numbering (ops/Ops.hpp)
    EXPECT(static_cast<int>(ops::OpType::SOFTMAX) == 26);
    EXPECT(static_cast<int>(ops::OpType::TOPK) == 30);
    EXPECT(static_cast<int>(ops::OpType::REDUCE) == 20 && static_cast<int>(ops::OpType::NMS) == 32);  // ops/Ops.hpp:78,90
    EXPECT(static_cast<int>(ops::OpType::WHERE) == 40);
    EXPECT(ops::convert_optype_to_string(ops::OpType::SOFTMAX) == "Softmax");
    EXPECT(ops::convert_optype_to_string(ops::OpType::TOPK) == "TopK");
    EXPECT(ops::convert_optype_to_string(ops::OpType::TOTAL_NUM) == "Unknown");
    EXPECT(ops::convert_opstring_to_enum("Softmax") == ops::OpType::SOFTMAX);
    EXPECT(ops::convert_opstring_to_enum("TopK") == ops::OpType::TOPK);
    EXPECT(ops::convert_opstring_to_enum("Conv") == ops::OpType::CONV2D);
    EXPECT(ops::convert_opstring_to_enum("BatchNormalization") == ops::OpType::BATCHNORM);
    EXPECT(ops::convert_opstring_to_enum("topk") == ops::OpType::UNKNOWN);
    EXPECT(ops::convert_opstring_to_enum("Unknown") == ops::OpType::UNKNOWN);
    for (int t = 1; t < static_cast<int>(ops::OpType::TOTAL_NUM); t++) {
        const auto ty = static_cast<ops::OpType>(t);
        EXPECT(ops::convert_opstring_to_enum(ops::convert_optype_to_string(ty)) == ty);
    }
    // factory (ops/OperatorFactory.hpp:56-143)
    const int before = ops::Operator::instance_count_.load();
    {
        auto sm = ops::create_from_type(ops::OpType::SOFTMAX, true);
        auto tk = ops::create_from_type(ops::OpType::TOPK, false, 1);
        EXPECT(sm && sm->get_type() == ops::OpType::SOFTMAX && dynamic_cast<ops::Softmax *>(sm.get()));
        EXPECT(tk && tk->get_type() == ops::OpType::TOPK && dynamic_cast<ops::Topk *>(tk.get()));
        EXPECT(ops::create_from_type(ops::OpType::CONV2D) == nullptr);
        {
            using ops::Reduce;
            EXPECT((Reduce::calculateOutputShape({16, 80, 8400}, {1}, false) == std::vector<int>{16, 8400}));
            EXPECT((Reduce::calculateOutputShape({16, 80, 8400}, {-2}, true) == std::vector<int>{16, 1, 8400}));
            EXPECT((Reduce::calculateOutputShape({2, 3, 4, 5}, {0, -1, 9}, false) == std::vector<int>{3, 4}));
            EXPECT((Reduce::calculateOutputShape({7}, {0}, false).empty()));
            auto rd = ops::create_from_type(ops::OpType::REDUCE);
            auto *r = dynamic_cast<Reduce *>(rd.get());
            EXPECT(r != nullptr && r->get_type() == ops::OpType::REDUCE);
            if (r) {
                EXPECT(r->reduce_op() == 0 && r->keepdims() == 1 && r->axes().empty());  // ops/Reduce.hpp:150-152
                r->setAttribute({{"reduce_op", "max"}, {"axes", "[1, -1]"}, {"keepdims", "0"}});
                EXPECT(r->reduce_op() == static_cast<int>(ops::reduce::ReduceType::MAX) && r->keepdims() == 0);
                EXPECT((r->axes() == std::vector<int>{1, -1}));
                r->setAttribute({{"reduce_op", "sum_square"}});
                EXPECT(r->reduce_op() == 9 && r->keepdims() == 0);
                r->setAttribute({{"reduce_op", "no such"}});
                EXPECT(r->reduce_op() == 9);  // unknown names leave it as it is (ops/Reduce.hpp:42-64)
            }
        }
        {
            auto nm = ops::create_from_type(ops::OpType::NMS);
            EXPECT(nm && nm->get_type() == ops::OpType::NMS && dynamic_cast<ops::Nms *>(nm.get()));
        }
        EXPECT(ops::create_from_type(ops::OpType::UNKNOWN) == nullptr);
        EXPECT(ops::Operator::instance_count_.load() == before + 2);
        sm->set_name("prob");
        EXPECT(sm->get_name() == "prob");
        EXPECT(sm->get_record() == nullptr);
        EXPECT((sm->parse_attr_list<int>("[1,2,3]") == std::vector<int>{1, 2, 3}));
        EXPECT(sm->parse_attr_list<float>("1,2").empty());
        bool threw = false;
        try {
            sm->parse_attr_list<int>("[1,x]");
        } catch (const std::runtime_error &) {
            threw = true;
        }
        EXPECT(threw);
        threw = false;
        try {
            sm->onExecute({}, {}, 0);  // no device yet
        } catch (const std::runtime_error &) {
            threw = true;
        }
        EXPECT(threw);
    }
    EXPECT(ops::Operator::instance_count_.load() == before);
    // tensors (core/Tensor.hpp)
    Tensor<float> t(std::vector<int>{3, 5});
    EXPECT(t.num_dims() == 2 && t.size() == 60 && t.num_elements() == 15 && t.dtype() == typeid(float));
    EXPECT((t.getShape() == std::vector<int>{3, 5}));
    EXPECT(!t.is_on_GPU());
    Tensor<uint16_t> h(true);
    EXPECT(h.size() == 0 && h.is_on_GPU() && h.dtype() == typeid(uint16_t));
    h.resize(std::vector<int>{2, 3, 4});
    EXPECT(h.size() == 48 && h.num_dims() == 3);
    std::shared_ptr<ITensor> it = std::make_shared<Tensor<int>>(std::vector<int>{7});
    EXPECT(vkop::core::as_tensor<int>(it) != nullptr && vkop::core::as_tensor<float>(it) == nullptr);
    // binary16 conversions against libtorch's, over every half and a float sweep
    int bad = 0;
    for (uint32_t b = 0; b < 65536; b++) {
        const at::Half hh(static_cast<uint16_t>(b), at::Half::from_bits());
        const float f = static_cast<float>(hh);
        const float g = ITensor::fp16_to_fp32(static_cast<uint16_t>(b));
        if (std::isnan(f) ? !std::isnan(g) : std::memcmp(&f, &g, 4) != 0) bad++;
        if (!std::isnan(f) && ITensor::fp32_to_fp16(f) != b) bad++;
    }
    EXPECT(bad == 0);
    bad = 0;
    uint32_t s = 12345;
    for (int i = 0; i < 2000000; i++) {
        s = s * 1664525u + 1013904223u;
        uint32_t bits = s;
        if (i & 1) bits = (bits & 0x807FFFFFu) | ((100u + (s >> 27)) << 23);  // exponents around the half range
        float f;
        std::memcpy(&f, &bits, 4);
        if (std::isnan(f)) continue;
        if (ITensor::fp32_to_fp16(f) != at::Half(f).x) bad++;
    }
    EXPECT(bad == 0);
}

// The benchmark's registration sequence (benchmark/main.cpp:85-137) on synthetic
// logits: SOFTMAX then TOPK, run repeatedly, results read back once.
static void runtime_postprocess_tests() {
    TestEnv::initialize();
    auto dev = TestEnv::dev;
    auto pool = TestEnv::pool;
    struct Case {
        std::vector<int> shape;
        int k;
    };
    for (const Case &c : {Case{{1, 1000}, 10}, Case{{64, 128256}, 50}}) {
        torch::manual_seed(11);
        auto x = torch::randn({c.shape[0], c.shape[1]}) * 2.5;
        auto p = torch::softmax(x.to(torch::kFloat64), -1).to(torch::kFloat32);
        auto sorted = torch::sort(p, /*stable=*/true, -1, /*descending=*/true);
        auto ev = std::get<0>(sorted).slice(-1, 0, c.k).contiguous();
        auto ei = std::get<1>(sorted).slice(-1, 0, c.k).to(torch::kInt).contiguous();
        std::vector<std::vector<float>> got_v(2);
        std::vector<std::vector<int>> got_i(2);
        for (int fuse = 0; fuse < 2; fuse++) {
            auto rt = std::make_shared<vkop::core::Runtime>(pool, "", 0);
            rt->set_postprocess_fusion(fuse == 1);
            auto cls = std::make_shared<Tensor<float>>(c.shape);
            fill_from_torch(cls, x);
            cls->as_storage_buffer(dev);
            cls->copyToGPU(pool);
            rt->SetOutput(cls);
            auto shape = vkop::core::as_tensor<float>(rt->GetOutput())->getShape();
            auto sf = std::make_shared<Tensor<float>>(shape, true);
            rt->RegisterPostProcess(ops::OpType::SOFTMAX, {{"axis", "-1"}}, {cls}, {sf});
            auto indexs = std::make_shared<Tensor<int>>(shape, true);      // full-size outputs, as the benchmark passes
            auto values = std::make_shared<Tensor<float>>(shape, true);
            rt->RegisterPostProcess(ops::OpType::TOPK, {{"k", std::to_string(c.k)}}, {sf}, {values, indexs});
            EXPECT(rt->num_nodes() == (fuse ? 1u : 2u));
            EXPECT(rt->GetRealOutputs().size() == 2 && rt->GetRealOutputs().count("post_TopK0") == 1);
            double ms = 0;
            for (int i = 0; i < 5; i++) ms = rt->Run();
            EXPECT(ms > 0.0);
            rt->ReadResult();
            const int rows = c.shape[0];
            bool ok = true;
            int64_t worst = 0;
            for (int r = 0; r < rows; r++) {
                for (int j = 0; j < c.k; j++) {
                    const size_t o = static_cast<size_t>(r) * c.k + j;
                    got_v[fuse].push_back((*values)[o]);
                    got_i[fuse].push_back((*indexs)[o]);
                    ok = ok && (*indexs)[o] == ei.data_ptr<int>()[o];
                    worst = std::max(worst, ulp_distance((*values)[o], ev.data_ptr<float>()[o]));
                }
            }
            std::printf("Runtime post-proc [%d,%d] k %d, %s: %s, worst distance %lld ulp, last Run() %.3f ms (%s)\n", c.shape[0],
                        c.shape[1], c.k, fuse ? "fused" : "two operators", ok ? "ok" : "FAILED", static_cast<long long>(worst), ms,
                        rt->node_name(rt->num_nodes() - 1).c_str());
            EXPECT(ok);
            EXPECT(worst <= 2);
        }
        EXPECT(got_i[0] == got_i[1]);
        int64_t between = 0;
        for (size_t i = 0; i < got_v[0].size(); i++) between = std::max(between, ulp_distance(got_v[0][i], got_v[1][i]));
        EXPECT(between <= 1);
    }
    // no fusion when the axes differ or the TOPK reads another tensor
    {
        auto rt = std::make_shared<vkop::core::Runtime>(pool, "", 0);
        auto a = std::make_shared<Tensor<float>>(std::vector<int>{8, 64});
        torch::manual_seed(21);
        fill_from_torch(a, torch::randn({8, 64}));
        a->as_storage_buffer(dev);
        a->copyToGPU(pool);
        auto sf = std::make_shared<Tensor<float>>(std::vector<int>{8, 64}, true);
        rt->RegisterPostProcess(ops::OpType::SOFTMAX, {{"axis", "0"}}, {a}, {sf});
        auto v = std::make_shared<Tensor<float>>(true);
        auto ix = std::make_shared<Tensor<int>>(true);
        rt->RegisterPostProcess(ops::OpType::TOPK, {{"k", "3"}, {"axis", "1"}}, {sf}, {v, ix});
        EXPECT(rt->num_nodes() == 2);
        rt->Run();
        rt->ReadResult();
        EXPECT((v->getShape() == std::vector<int>{8, 3}));
        auto want = torch::topk(torch::softmax(torch::from_blob(a->data(), {8, 64}).to(torch::kFloat64), 0).to(torch::kFloat32), 3, 1);
        bool ok = true;
        auto wi = std::get<1>(want).to(torch::kInt).contiguous();
        for (int i = 0; i < 24; i++) ok = ok && (*ix)[i] == wi.data_ptr<int>()[i];
        std::printf("Runtime post-proc softmax axis 0 then top-k axis 1 (not fusable): %s\n", ok ? "ok" : "FAILED");
        EXPECT(ok);
    }
}

static std::string g_golden;  // directory of the .vkopbin fixtures

static std::vector<uint8_t> file_bytes(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    return std::vector<uint8_t>(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
}

// The model file reader against the reference's own model file and the fixtures
// written by tests/golden/make_vkopbin.py; no device needed.
static void model_file_tests() {
    using vkop::load::VkModel;
    {
        // model/add_conv_model.vkopbin as the reference's converter wrote it (Add -> depthwise Conv, int8 weights)
        const VkModel m(g_golden + "/add_conv_model.vkopbin");
        EXPECT(m.inputs.size() == 2 && m.inputs[0].name == "input_x1" && m.inputs[1].name == "input_x2");
        EXPECT((m.inputs[1].dims == std::vector<uint32_t>{1, 16, 8, 8}));
        EXPECT(m.outputs.size() == 1 && m.outputs[0].name == "output");
        EXPECT(m.nodes.size() == 2 && m.nodes[0].op_type == "Add" && m.nodes[0].name == "node_add" && m.nodes[0].attributes.empty());
        EXPECT(m.nodes[0].dependencies.empty() && m.nodes[0].dependents.count("node_conv2d") == 1);
        const auto &conv = m.nodes[1];
        EXPECT(conv.op_type == "Conv" && conv.inputs.size() == 4 && conv.inputs[3].name == "conv.weight_scale");
        EXPECT(conv.attributes.at("group") == "16" && conv.attributes.at("pads") == "[1, 1, 1, 1]" &&
               conv.attributes.at("auto_pad") == "NOTSET" && conv.attributes.at("strides") == "[1, 1]");
        EXPECT(conv.dependencies.count("node_add") == 1 && conv.dependents.empty());
        EXPECT(m.initializers.size() == 3 && m.initializers.at("conv.weight").dtype == "int8");
        EXPECT((m.initializers.at("conv.weight").dims == std::vector<uint32_t>{16, 1, 3, 3}));
        const auto *w = reinterpret_cast<const int8_t *>(m.initializer_data("conv.weight"));
        EXPECT(w[0] == 39 && w[1] == 127 && w[2] == 61 && w[3] == 18);
        float bias0 = 0;
        std::memcpy(&bias0, m.initializer_data("conv.bias"), 4);
        EXPECT(std::fabs(bias0 - 0.03973345F) < 1e-8F);
        for (const auto &o : m.initializer_offsets) EXPECT(o.second % 64 == 0);
        EXPECT(m.initializer_bytes.at("conv.weight") == 144 && m.initializer_bytes.at("conv.bias") == 64);
        EXPECT(m.concurrent_execution_levels.size() == 2 && m.concurrent_execution_levels[1] == std::vector<std::string>{"node_conv2d"});
        EXPECT(!m.unified && !m.rgba);
        // a runtime refuses it by the first operator it lacks (the check comes before any device work)
        bool refused = false;
        try {
            vkop::core::Runtime rt(nullptr, g_golden + "/add_conv_model.vkopbin", 0);
            rt.LoadModel();
        } catch (const std::runtime_error &e) {
            refused = std::string(e.what()).find("Add") != std::string::npos;
        }
        EXPECT(refused);
    }
    {
        const VkModel m(g_golden + "/detection_tail.vkopbin");  // one attribute of each tagged kind
        const auto &a = m.nodes.at(0).attributes;
        EXPECT(m.nodes[0].op_type == "Nms" && a.size() == 7);
        EXPECT(a.at("center_point_box") == "0" && a.at("iou_threshold") == "0.500000" && a.at("score_threshold") == "0.250000");
        EXPECT(a.at("note") == "detection tail" && a.at("strides") == "[8, 16, 32]" && a.at("anchors") == "[1.500000, 2.250000]");
        EXPECT((m.outputs[0].dims == std::vector<uint32_t>{1800, 3}));
    }
    {
        const VkModel m(g_golden + "/classifier_head_k_input.vkopbin");
        EXPECT(m.initializers.at("k_value").dtype == "int64" && m.initializers.at("k_value").dims == std::vector<uint32_t>{1});
        int64_t k = 0;
        std::memcpy(&k, m.initializer_data("k_value"), 8);
        EXPECT(k == 7);
        EXPECT(m.nodes[1].attributes.count("K") == 0 && m.nodes[1].inputs.size() == 2);
    }
    {
        // every proper prefix of a file is refused with an exception, and so is a wrong tag, an
        // oversized count and an oversized string; nothing reads past the bytes given
        const auto bytes = file_bytes(g_golden + "/classifier_head.vkopbin");
        EXPECT(bytes.size() > 100);
        const VkModel whole(bytes.data(), bytes.size());
        EXPECT(whole.nodes.size() == 2 && whole.nodes[1].attributes.at("K") == "5");
        size_t refused = 0;
        for (size_t n = 0; n < bytes.size(); ++n) {
            std::vector<uint8_t> part(bytes.begin(), bytes.begin() + static_cast<std::ptrdiff_t>(n));  // exact-size heap block
            try {
                const VkModel m(part.data(), part.size());
            } catch (const std::runtime_error &) {
                refused++;
            }
        }
        EXPECT(refused == bytes.size());
        auto broken = [&](size_t at, uint8_t value) {
            auto copy = bytes;
            copy[at] = value;
            try {
                const VkModel m(copy.data(), copy.size());
            } catch (const std::runtime_error &) {
                return true;
            }
            return false;
        };
        EXPECT(broken(3, 0x7F));  // input count of 2 billion
        EXPECT(broken(7, 0x7F));  // name length of 2 billion
        const std::string key = "axis";
        auto it = std::search(bytes.begin(), bytes.end(), key.begin(), key.end());
        EXPECT(it != bytes.end());
        if (it != bytes.end()) EXPECT(broken(static_cast<size_t>(it - bytes.begin()) + 4, 9));  // attribute tag 9
    }
    {
        // Files nothing but their initializers: two of one name (the second, shorter one would
        // leave its offset to the first one's bytes) are refused by the reader; data shorter than
        // the dimensions promise is refused when a runtime loads the model (it copies
        // product-of-dims elements); both from exact-size heap blocks.
        struct Init {
            std::string name, dtype;
            std::vector<uint32_t> dims;
            std::vector<uint8_t> data;
        };
        auto file_of = [](const std::vector<Init> &inits) {
            std::vector<uint8_t> b;
            auto u32 = [&b](uint32_t v) { for (int i = 0; i < 4; i++) b.push_back(static_cast<uint8_t>(v >> (8 * i))); };
            auto str = [&](const std::string &t) { u32(static_cast<uint32_t>(t.size())); b.insert(b.end(), t.begin(), t.end()); };
            u32(0);  // inputs
            u32(0);  // outputs
            u32(0);  // nodes
            u32(static_cast<uint32_t>(inits.size()));
            for (const auto &i : inits) {
                str(i.name);
                str(i.dtype);
                u32(static_cast<uint32_t>(i.dims.size()));
                for (uint32_t d : i.dims) u32(d);
                const uint64_t n = i.data.size();
                for (int k = 0; k < 8; k++) b.push_back(static_cast<uint8_t>(n >> (8 * k)));
                b.insert(b.end(), i.data.begin(), i.data.end());
            }
            u32(0);  // levels
            return b;
        };
        const auto good = file_of({{"a", "float32", {1024}, std::vector<uint8_t>(4096, 1)}, {"b", "float32", {1}, std::vector<uint8_t>(4, 2)}});
        const VkModel m(good.data(), good.size());
        EXPECT(m.initializer_bytes.at("a") == 4096 && m.initializer_offsets.at("b") == 4096 && m.initializer_data("b")[0] == 2);
        EXPECT(m.initializer_data("a", 4)[4095] == 1);
        const auto twice = file_of({{"a", "float32", {1024}, std::vector<uint8_t>(4096, 1)}, {"a", "float32", {1}, std::vector<uint8_t>(4, 2)}});
        bool refused = false;
        try {
            const VkModel m2(twice.data(), twice.size());
        } catch (const std::runtime_error &e) {
            refused = std::string(e.what()).find("twice") != std::string::npos;
        }
        EXPECT(refused);
        const auto shorter = file_of({{"w", "float32", {1024}, std::vector<uint8_t>(16, 3)}});
        const VkModel m3(shorter.data(), shorter.size());  // the reader takes it: dims and data are separate fields
        refused = false;
        try {
            (void)m3.initializer_data("w", 4);
        } catch (const std::runtime_error &e) {
            refused = std::string(e.what()).find("16 bytes of data for 1024 elements") != std::string::npos;
        }
        EXPECT(refused);
        const std::string tmp = "build/short_initializer.vkopbin";
        {
            std::ofstream f(tmp, std::ios::binary);
            f.write(reinterpret_cast<const char *>(shorter.data()), static_cast<std::streamsize>(shorter.size()));
        }
        refused = false;
        try {
            vkop::core::Runtime rt(nullptr, tmp, 0);
            rt.LoadModel();
        } catch (const std::runtime_error &e) {
            refused = std::string(e.what()).find("bytes of data for") != std::string::npos;
        }
        EXPECT(refused);
    }
}

// Models from .vkopbin files through Runtime::LoadModel / Run / ReadResult.
template <typename T> static void model_head_case(const std::string &file, int rows, int k, bool fuse, size_t want_nodes) {
    auto pool = TestEnv::pool;
    const int precision = std::is_same_v<T, uint16_t> ? 1 : 0;
    vkop::core::Runtime rt(pool, g_golden + "/" + file, precision);
    rt.set_postprocess_fusion(fuse);
    rt.LoadModel();
    EXPECT(rt.num_nodes() == want_nodes);
    torch::manual_seed(5);
    auto x = (torch::randn({rows, 1000}) * 3).to(precision ? torch::kFloat16 : torch::kFloat32);
    auto in = vkop::core::as_tensor<T>(rt.GetInput("logits"));
    EXPECT(in != nullptr && rt.GetInput() == rt.GetInput("logits") && rt.GetInput("nothing") == nullptr);
    fill_from_torch(in, x);
    in->copyToGPU(pool);
    double ms = 0;
    for (int i = 0; i < 3; i++) ms = rt.Run();
    rt.ReadResult();
    auto p = torch::softmax(x.to(torch::kFloat64), -1).to(precision ? torch::kFloat16 : torch::kFloat32);
    auto sorted = torch::sort(p, /*stable=*/true, -1, /*descending=*/true);
    auto ev = std::get<0>(sorted).slice(-1, 0, k).to(torch::kFloat32).contiguous();
    auto ei = std::get<1>(sorted).slice(-1, 0, k).to(torch::kInt).contiguous();
    auto values = vkop::core::as_tensor<T>(rt.GetOutput("values"));
    auto indices = vkop::core::as_tensor<int>(rt.GetOutput("indices"));
    EXPECT(values != nullptr && indices != nullptr);
    bool ok = values && indices && values->getShape() == std::vector<int>{rows, k};
    double worst = 0;
    for (int i = 0; ok && i < rows * k; i++) {
        const float got = precision ? ITensor::fp16_to_fp32(static_cast<uint16_t>((*values)[static_cast<size_t>(i)]))
                                    : static_cast<float>((*values)[static_cast<size_t>(i)]);
        const float want = ev.data_ptr<float>()[i];
        worst = std::max(worst, static_cast<double>(std::fabs(got - want)) / std::max(1e-30, static_cast<double>(std::fabs(want))));
        // equal probabilities (frequent in half precision) may come in either order in the sorted expectation only
        // when they are equal: compare the index where the value is unique in its row
        const int r = i / k, j = i % k;
        const bool tied = (j > 0 && ev.data_ptr<float>()[i - 1] == want) || (j + 1 < k && ev.data_ptr<float>()[i + 1] == want) ||
                          (j + 1 == k && std::get<0>(sorted)[r][k].item<float>() == want);
        if (!tied) ok = ok && (*indices)[static_cast<size_t>(i)] == ei.data_ptr<int>()[i];
    }
    ok = ok && worst <= (precision ? 2e-3 : 3e-7);
    if (rt.GetOutput("probs")) {  // the variant that also returns the probabilities
        auto probs = vkop::core::as_tensor<T>(rt.GetOutput("probs"));
        double sum = 0;
        for (int i = 0; i < 1000; i++)
            sum += precision ? ITensor::fp16_to_fp32(static_cast<uint16_t>((*probs)[static_cast<size_t>(i)])) : static_cast<float>((*probs)[static_cast<size_t>(i)]);
        ok = ok && std::fabs(sum - 1.0) < (precision ? 2e-2 : 1e-5);
    }
    std::printf("Model %s %s [%d,1000] k %d, %zu operator(s) (%s): %s, worst relative difference %.2e, last Run() %.3f ms\n", file.c_str(),
                precision ? "fp16" : "fp32", rows, k, rt.num_nodes(), rt.node_name(rt.num_nodes() - 1).c_str(), ok ? "ok" : "FAILED", worst, ms);
    EXPECT(ok);
}

// Reduce "max" along one axis against torch::amax (exact: a maximum has no rounding), and the errors for what is not built.
template <typename T> static void reduce_case(const std::vector<int> &shape, int axis, int keepdims) {
    TestCase<T> tc("Reduce");
    torch::manual_seed(17);
    std::vector<int64_t> dims(shape.begin(), shape.end());
    auto x = torch::randn(dims, tc.conf());
    auto want = torch::amax(x, {axis}, keepdims == 1).contiguous();
    auto in = std::make_shared<Tensor<T>>(shape);
    fill_from_torch(in, x);
    std::vector<int> out_shape(want.sizes().begin(), want.sizes().end());
    auto expect = std::make_shared<Tensor<T>>(out_shape);
    fill_from_torch(expect, want);
    const std::unordered_map<std::string, std::string> attrs = {
        {"reduce_op", "max"}, {"axes", "[" + std::to_string(axis) + "]"}, {"keepdims", std::to_string(keepdims)}};
    const bool ok = tc.run_test({in}, {expect}, [&](std::unique_ptr<ops::Operator> &op) { op->setAttribute(attrs); });
    std::printf("Reduce max %s shape [", std::is_same_v<T, float> ? "fp32" : "fp16");
    for (size_t i = 0; i < shape.size(); i++) std::printf("%s%d", i ? "," : "", shape[i]);
    std::printf("] axis %d keepdims %d: %s\n", axis, keepdims, ok ? "ok" : "FAILED");
    EXPECT(ok);
}

// The detection-style chain from its model file: Softmax over classes, class maximum, top anchors.
static void model_chain_case(bool fuse, size_t want_nodes) {
    auto pool = TestEnv::pool;
    vkop::core::Runtime rt(pool, g_golden + "/detection_chain.vkopbin", 0);
    rt.set_postprocess_fusion(fuse);
    rt.LoadModel();
    EXPECT(rt.num_nodes() == want_nodes);
    torch::manual_seed(23);
    auto x = torch::randn({2, 80, 840}) * 2;
    auto in = vkop::core::as_tensor<float>(rt.GetInput());
    fill_from_torch(in, x);
    in->copyToGPU(pool);
    rt.Run();
    rt.ReadResult();
    auto best = torch::amax(torch::softmax(x.to(torch::kFloat64), 1).to(torch::kFloat32), {1});
    auto sorted = torch::sort(best, /*stable=*/true, -1, /*descending=*/true);
    auto ev = std::get<0>(sorted).slice(-1, 0, 30).contiguous();
    auto ei = std::get<1>(sorted).slice(-1, 0, 30).to(torch::kInt).contiguous();
    auto values = vkop::core::as_tensor<float>(rt.GetOutput("values"));
    auto anchors = vkop::core::as_tensor<int>(rt.GetOutput("anchors"));
    bool ok = values && anchors;
    int64_t worst = 0;
    for (int i = 0; ok && i < 60; i++) {
        const float want = ev.data_ptr<float>()[i];
        worst = std::max(worst, ulp_distance((*values)[static_cast<size_t>(i)], want));
        const int j = i % 30;
        const bool tied = (j > 0 && ev.data_ptr<float>()[i - 1] == want) || (j + 1 < 30 && ev.data_ptr<float>()[i + 1] == want);
        if (!tied) ok = (*anchors)[static_cast<size_t>(i)] == ei.data_ptr<int>()[i];
    }
    ok = ok && worst <= 2;
    std::printf("Model detection_chain.vkopbin, %zu operator(s): %s, worst distance %lld ulp\n", rt.num_nodes(), ok ? "ok" : "FAILED",
                static_cast<long long>(worst));
    EXPECT(ok);
}

// Two heads in one model: two nodes in the first level (one per queue), a dependency from the second level into it.
static void model_two_heads_case() {
    auto pool = TestEnv::pool;
    vkop::core::Runtime rt(pool, g_golden + "/two_heads.vkopbin", 0);
    rt.LoadModel();
    EXPECT(rt.num_nodes() == 3);
    torch::manual_seed(31);
    auto x = torch::randn({4, 1000}) * 3;
    auto scores = torch::rand({1, 4, 200});
    auto centre = torch::rand({1, 200, 2}), size = torch::rand({1, 200, 2}) * 0.4F;
    auto boxes = torch::cat({centre - size / 2, centre + size / 2}, -1);
    auto tl = vkop::core::as_tensor<float>(rt.GetInput("logits"));
    auto tb = vkop::core::as_tensor<float>(rt.GetInput("boxes"));
    auto ts = vkop::core::as_tensor<float>(rt.GetInput("scores"));
    fill_from_torch(tl, x);
    fill_from_torch(tb, boxes);
    fill_from_torch(ts, scores);
    tl->copyToGPU(pool);
    tb->copyToGPU(pool);
    ts->copyToGPU(pool);
    for (int i = 0; i < 3; i++) rt.Run();
    rt.ReadResult();
    auto p = torch::softmax(x.to(torch::kFloat64), -1).to(torch::kFloat32);
    auto want_top = torch::topk(p, 7, -1, true, true);
    auto wi = std::get<1>(want_top).to(torch::kInt).contiguous();
    auto indices = vkop::core::as_tensor<int>(rt.GetOutput("indices"));
    auto probs = vkop::core::as_tensor<float>(rt.GetOutput("probs"));
    auto selected = vkop::core::as_tensor<int>(rt.GetOutput("selected"));
    bool ok = indices && probs && selected;
    for (int i = 0; ok && i < 28; i++) ok = (*indices)[static_cast<size_t>(i)] == wi.data_ptr<int>()[i];
    // (all 4000 probabilities: the small ones carry the rounding of x - max in single precision, which the operator
    //  shares with libtorch's float kernel; against the double-precision expectation that is a relative 1e-6)
    double worst = 0;
    for (int i = 0; ok && i < 4000; i++) {
        const double w = p.contiguous().data_ptr<float>()[i];
        worst = std::max(worst, std::fabs((*probs)[static_cast<size_t>(i)] - w) / w);
    }
    const auto want = nms_expectation(boxes, scores, 0.4F, 0.5F);
    for (size_t i = 0; ok && i < want.size(); i++) ok = (*selected)[i] == want[i];
    ok = ok && worst <= 2e-6 && !want.empty() && (*selected)[want.size()] == -1;
    std::printf("Model two_heads.vkopbin, 3 operators in 2 levels: %s, %zu records, probabilities within %.1e relative\n", ok ? "ok" : "FAILED",
                want.size() / 3, worst);
    EXPECT(ok);
}

static void model_run_tests() {
    TestEnv::initialize();
    auto pool = TestEnv::pool;
    model_head_case<float>("classifier_head.vkopbin", 8, 5, true, 1);
    model_head_case<float>("classifier_head.vkopbin", 8, 5, false, 2);
    model_head_case<uint16_t>("classifier_head.vkopbin", 8, 5, true, 1);
    model_head_case<float>("classifier_head_k_input.vkopbin", 4, 7, true, 2);  // probabilities are an output: two operators
    model_head_case<uint16_t>("classifier_head_k_input.vkopbin", 4, 7, true, 2);
    model_chain_case(true, 2);   // Softmax + Reduce as one operator, then TopK
    model_chain_case(false, 3);
    model_two_heads_case();
    {
        vkop::core::Runtime rt(pool, g_golden + "/detection_tail.vkopbin", 0);
        rt.LoadModel();
        EXPECT(rt.num_nodes() == 1);
        bool threw = false;
        try {
            rt.GetInput();
        } catch (const std::runtime_error &) {
            threw = true;
        }
        EXPECT(threw);  // two inputs: a name is needed (core/runtime.cpp:366-369)
        torch::manual_seed(11);
        auto scores = torch::rand({2, 3, 300});
        auto centre = torch::rand({2, 300, 2}), size = torch::rand({2, 300, 2}) * 0.3F;
        auto boxes = torch::cat({centre - size / 2, centre + size / 2}, -1);
        auto tb = vkop::core::as_tensor<float>(rt.GetInput("boxes"));
        auto ts = vkop::core::as_tensor<float>(rt.GetInput("scores"));
        fill_from_torch(tb, boxes);
        fill_from_torch(ts, scores);
        tb->copyToGPU(pool);
        ts->copyToGPU(pool);
        rt.Run();
        rt.ReadResult();
        const auto want = nms_expectation(boxes, scores, 0.5F, 0.25F);
        auto out = vkop::core::as_tensor<int>(rt.GetOutput());
        bool ok = out && want.size() + 3 <= static_cast<size_t>(out->num_elements());
        for (size_t i = 0; ok && i < want.size(); i++) ok = (*out)[i] == want[i];
        for (size_t i = want.size(); ok && i < want.size() + 3; i++) ok = (*out)[i] == -1;  // the end of the list
        std::printf("Model detection_tail.vkopbin: %s, %zu records\n", ok ? "ok" : "FAILED", want.size() / 3);
        EXPECT(ok && !want.empty());
    }
}

// Every single-byte change of every fixture either parses or is refused with std::runtime_error; nothing else
// is thrown and nothing outside the (exact-size) buffer is touched.
static void model_file_mutation_tests() {
    size_t parsed = 0, refused = 0, other = 0;
    for (const char *name : {"classifier_head.vkopbin", "classifier_head_k_input.vkopbin", "detection_tail.vkopbin",
                             "detection_chain.vkopbin", "two_heads.vkopbin", "add_conv_model.vkopbin"}) {
        const auto bytes = file_bytes(g_golden + "/" + name);
        EXPECT(!bytes.empty());
        for (size_t at = 0; at < bytes.size(); ++at) {
            for (uint8_t value : {uint8_t{0x00}, uint8_t{0x7F}, uint8_t{0xFF}, static_cast<uint8_t>(bytes[at] ^ 0x01)}) {
                if (value == bytes[at]) continue;
                std::vector<uint8_t> copy(bytes);
                copy[at] = value;
                try {
                    const vkop::load::VkModel m(copy.data(), copy.size());
                    parsed++;
                } catch (const std::runtime_error &) {
                    refused++;
                } catch (...) {
                    other++;
                }
            }
        }
    }
    std::printf("Model file mutations: %zu parsed, %zu refused, %zu other\n", parsed, refused, other);
    EXPECT(other == 0 && refused > 1000 && parsed > 1000);
}

// `--bench-runtime [runs]`: the benchmark's loop (benchmark/main.cpp:112-137) on the headline
// tensor -- SOFTMAX and TOPK registered as post-processing of a [64,128256] float output,
// Runtime::Run() called `runs` times after 20 untimed calls -- and the mean of what Run() returns
// (host wall clock around record + submit + wait), once with the pair fused and once as two
// operators.  Prints one line of JSON per arrangement, nothing else.
static int bench_runtime(int runs) {
    TestEnv::initialize();
    auto dev = TestEnv::dev;
    auto pool = TestEnv::pool;
    const std::vector<int> shape{64, 128256};
    const int k = 50;
    torch::manual_seed(11);
    auto x = torch::randn({shape[0], shape[1]}) * 1.25;
    for (int fuse = 1; fuse >= 0; fuse--) {
        auto rt = std::make_shared<vkop::core::Runtime>(pool, "", 0);
        rt->set_postprocess_fusion(fuse == 1);
        auto cls = std::make_shared<Tensor<float>>(shape);
        fill_from_torch(cls, x);
        cls->as_storage_buffer(dev);
        cls->copyToGPU(pool);
        rt->SetOutput(cls);
        auto sf = std::make_shared<Tensor<float>>(shape, true);
        rt->RegisterPostProcess(ops::OpType::SOFTMAX, {{"axis", "-1"}}, {cls}, {sf});
        auto indexs = std::make_shared<Tensor<int>>(shape, true);
        auto values = std::make_shared<Tensor<float>>(shape, true);
        rt->RegisterPostProcess(ops::OpType::TOPK, {{"k", std::to_string(k)}}, {sf}, {values, indexs});
        for (int i = 0; i < 20; i++) rt->Run();
        double sum = 0, best = 1e30;
        for (int i = 0; i < runs; i++) {
            const double ms = rt->Run();
            sum += ms;
            best = std::min(best, ms);
        }
        std::printf("{\"what\": \"Runtime::Run() of the registered SOFTMAX + TOPK post-processing, host wall clock per run\", "
                    "\"shape\": [%d, %d], \"k\": %d, \"operators\": %zu, \"fused\": %s, \"runs\": %d, \"mean_ms\": %.6f, \"min_ms\": %.6f}\n",
                    shape[0], shape[1], k, rt->num_nodes(), fuse ? "true" : "false", runs, sum / runs, best);
    }
    return 0;
}

int main(int argc, char **argv) {
    if (argc > 1 && std::strcmp(argv[1], "--bench-runtime") == 0) return bench_runtime(argc > 2 ? std::max(1, std::atoi(argv[2])) : 200);
    const bool no_gpu = argc > 1 && std::strcmp(argv[1], "--no-gpu") == 0;
    g_golden = (std::filesystem::path(argv[0]).parent_path() / ".." / ".." / ".." / "tests" / "golden").string();
    host_logic_tests();
    reference_base_class_tests();
    model_file_tests();
    model_file_mutation_tests();
    if (!no_gpu) {
        const std::vector<std::pair<std::vector<int>, int>> softmax_cases = {
            {{1, 10, 7, 7}, 1}, {{1, 6, 8, 8}, 3}, {{2, 4, 10, 10}, 2}, {{1, 8, 6, 6}, 2}, {{1, 16, 5, 5}, 1}, {{4, 1000}, 1},
        };
        for (const auto &[shape, axis] : softmax_cases) {
            softmax_case<float>(shape, axis);
            softmax_case<uint16_t>(shape, axis);
        }
        softmax_case<float>({1000}, 0);   // a vector is one row
        softmax_case<float>({4, 1000}, -1);
        const std::vector<std::tuple<std::vector<int>, int, int>> topk_cases = {
            {{1, 200}, 7, -1}, {{1, 400}, 8, -1}, {{1, 600}, 7, -1}, {{3, 2000}, 7, -1}, {{1, 2000}, 6, -1},
        };
        for (const auto &[shape, k, axis] : topk_cases) {
            topk_case<float>(shape, k, axis);
            topk_case<uint16_t>(shape, k, axis);
        }
        fused_case<float>({1, 1000}, 5);
        fused_case<float>({256, 1000}, 5);
        fused_case<float>({4, 128256}, 50);
        fused_case<uint16_t>({64, 1000}, 5);
        // tests/NmsTest.cpp:165-169 (its expectation never applies the per-class limit: 0 here)
        nms_case<float>({1, 10, 4}, {1, 2, 10}, 0, 0.5F, 0.5F);
        nms_case<float>({1, 200, 4}, {1, 1, 200}, 0, 0.7F, 0.4F);
        nms_case<float>({1, 50, 4}, {1, 7, 50}, 0, 0.3F, 0.2F);
        nms_case<uint16_t>({2, 300, 4}, {2, 3, 300}, 0, 0.5F, 0.3F);
        reduce_case<float>({16, 80, 8400}, 1, 0);
        reduce_case<float>({16, 80, 8400}, 1, 1);
        reduce_case<uint16_t>({4, 80, 1000}, -2, 0);
        reduce_case<float>({4, 1000}, -1, 0);
        reduce_case<float>({3, 5, 7, 9}, 0, 1);
        model_run_tests();
        // the benchmark's arrangement: full-size outputs, the first k read back
        {
            TestEnv::initialize();
            auto dev = TestEnv::dev;
            auto pool = TestEnv::pool;
            torch::manual_seed(3);
            auto x = torch::randn({1, 1000}) * 3;
            auto [v, i64] = torch::topk(torch::softmax(x, -1), 5, -1, true, true);
            auto in = std::make_shared<Tensor<float>>(std::vector<int>{1, 1000});
            fill_from_torch(in, x);
            in->as_storage_buffer(dev);
            in->copyToGPU(pool);
            auto sf = std::make_shared<Tensor<float>>(true);
            auto values = std::make_shared<Tensor<float>>(std::vector<int>{1, 1000}, true);
            auto indexs = std::make_shared<Tensor<int>>(std::vector<int>{1, 1000}, true);
            auto sm = ops::create_from_type(ops::OpType::SOFTMAX, true);
            auto tk = ops::create_from_type(ops::OpType::TOPK, true, 0);
            sm->set_runtime_device(dev, pool);
            tk->set_runtime_device(dev, pool);
            sm->setAttribute({{"axis", "-1"}});
            tk->setAttribute({{"k", "5"}});
            sm->onExecute({in}, {sf}, 0);
            tk->onExecute({sf}, {values, indexs}, 0);
            vkop::VulkanCommandBuffer::submit(dev->getComputeQueue(0),
                                              {sm->get_record()->buildSubmitInfo(), tk->get_record()->buildSubmitInfo()});
            tk->get_record()->wait();
            values->copyToCPU(pool);
            indexs->copyToCPU(pool);
            bool ok = true;
            auto i32 = i64.to(torch::kInt).contiguous();
            for (int j = 0; j < 5; j++) {
                ok = ok && (*indexs)[j] == i32.data_ptr<int>()[j];
                ok = ok && ulp_distance((*values)[j], v.contiguous().data_ptr<float>()[j]) <= 4;
            }
            std::printf("Softmax then TopK into full-size outputs (benchmark arrangement): %s\n", ok ? "ok" : "FAILED");
            EXPECT(ok);
        }
    }
    if (!no_gpu) runtime_postprocess_tests();
    std::printf("%d checks, %d failed\n", g_checked, g_failed);
    return g_failed == 0 ? 0 : 1;
}
