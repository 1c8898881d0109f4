// Operator base class: the reference's lifecycle and call surface
// (ops/Operator.hpp:19-271) over HIP streams instead of Vulkan pipelines.
//
//   create -> set_runtime_device -> setAttribute -> onExecute (records) ->
//   caller submits get_record() and waits.
//
// The constructor and `submit` keep the reference's signatures
// (ops/Operator.hpp:21-23, 225-238), so an operator written against the reference's
// base class compiles against this one: the SPIR-V blob, the binding kinds and the
// push-constant size are taken and kept (types_, pc_size_) but nothing acts on them,
// and `submit` -- where the reference binds a pipeline, pushes constants and records
// a dispatch -- has nothing to dispatch here: the operators of this library call the
// C ABI from execute(), and the base `submit` refuses with an exception naming the
// operator, so that one ported without a HIP kernel fails loudly instead of doing
// nothing.  The short constructor (kind, fp16) is what the operators here use.
// Descriptor sets, pipelines and the dummy buffer statics have no counterpart.
// Errors are C++ exceptions and asserts, as in the reference; the factory returns
// nullptr for unknown kinds.
#ifndef VKOP_HIP_OPS_OPERATOR_HPP_
#define VKOP_HIP_OPS_OPERATOR_HPP_

#include <atomic>
#include <cassert>
#include <cstdio>
#include <iostream>
#include <memory>
#include <sstream>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "core/Tensor.hpp"
#include "ops/Ops.hpp"

namespace vkop {
namespace ops {

class Operator {
  public:
    explicit Operator(OpType type, int fp16 = 0) : type_(type), fp16_(fp16) { instance_count_.fetch_add(1); }
    // the reference's signature (ops/Operator.hpp:21-31)
    explicit Operator(OpType type, uint8_t *spv, uint32_t spv_len, const std::vector<VkDescriptorType> &types,
                      size_t pc_size = 0, int fp16 = 0)
        : type_(type), fp16_(fp16), pc_size_(pc_size), spv_(spv), spv_len_(spv_len), types_(types) {
        assert(pc_size_ <= 128);
        instance_count_.fetch_add(1);
        objs_.reserve(types_.size());
    }
    virtual ~Operator() { instance_count_.fetch_sub(1); }
    Operator(const Operator &) = delete;
    Operator &operator=(const Operator &) = delete;
    Operator(Operator &&) = delete;
    Operator &operator=(Operator &&) = delete;

    virtual void set_runtime_device(const std::shared_ptr<VulkanDevice> &dev,
                                    const std::shared_ptr<VulkanCommandPool> &cmdpool) {
        m_dev_ = dev;
        m_cmdpool_ = cmdpool;
    }

    // Base behaviour: unknown attributes are only reported (ops/Operator.hpp:83-92).
    virtual void setAttribute(const std::unordered_map<std::string, std::string> &attributes) {
        for (const auto &attr : attributes)
            std::cout << "attribute " << attr.first << ": " << attr.second << " in operator." << std::endl;
    }

    // "[1,2,3]" -> {1,2,3}; anything not in brackets gives an empty list
    // (ops/Operator.hpp:93-125).
    template <typename T> std::vector<T> parse_attr_list(const std::string &str) {
        std::vector<T> result;
        if (str.size() < 2 || str.front() != '[' || str.back() != ']') return result;
        std::stringstream ss(str.substr(1, str.size() - 2));
        std::string item;
        while (std::getline(ss, item, ',')) {
            try {
                if (std::is_same<T, float>::value) result.emplace_back(static_cast<T>(std::stof(item)));
                else result.emplace_back(static_cast<T>(std::stol(item)));
            } catch (const std::invalid_argument &) {
                throw std::runtime_error("Invalid number in attribute list: " + item);
            } catch (const std::out_of_range &) {
                throw std::runtime_error("Number out of range in attribute list: " + item);
            }
        }
        return result;
    }

    virtual OpType get_type() { return type_; }
    std::shared_ptr<VulkanCommandBuffer> get_record() { return m_cmd_; }

    // Records the operator's work for queue `id`; nothing runs until the caller
    // submits get_record() (ops/Operator.hpp:127-170).
    void onExecute(const std::vector<std::shared_ptr<core::ITensor>> &inputs,
                   const std::vector<std::shared_ptr<core::ITensor>> &outputs, int id) {
        if (!m_dev_ || !m_cmdpool_) throw std::runtime_error("onExecute before set_runtime_device");
        if (!m_cmd_ || m_cmd_->queue_id() != id) m_cmd_ = std::make_shared<VulkanCommandBuffer>(m_cmdpool_, id);
        m_id_ = id;
        objs_.clear();  // (ops/Operator.hpp:131)
        m_cmd_->begin();
        execute(inputs, outputs);
        m_cmd_->end();
        if (trace_) {
            VulkanCommandBuffer::submit(m_cmd_->stream(), {m_cmd_->buildSubmitInfo()});
            m_cmd_->wait();
            m_dev_->wait_all_done();
            std::printf("%s: %s\n", convert_optype_to_string(type_).c_str(), name_.c_str());
            dump("output 0", outputs[0]);
        }
    }
    void enable_trace() { trace_ = true; }
    void disable_trace() { trace_ = false; }
    void set_name(const std::string &name) { name_ = name; }
    std::string get_name() const { return name_; }

    static std::atomic<int> instance_count_;

  protected:
    std::shared_ptr<VulkanDevice> m_dev_;
    std::shared_ptr<VulkanCommandPool> m_cmdpool_;
    std::shared_ptr<VulkanCommandBuffer> m_cmd_ = nullptr;
    int m_id_ = 0;
    OpType type_;
    bool trace_ = false;
    std::string name_;
    int fp16_ = 0;  // 0: fp32, 1: fp16
    // what the reference's constructor is given (kept, not acted on) and what its
    // operators collect per call before they submit (ops/Operator.hpp:176-199)
    size_t pc_size_ = 0;
    uint8_t *spv_ = nullptr;
    uint32_t spv_len_ = 0;
    std::vector<VkDescriptorType> types_;
    std::vector<std::shared_ptr<VulkanResource>> objs_;

    // ops/Operator.hpp:225-238 binds the pipeline and its descriptor set, pushes pc_size_
    // bytes at `ptr` and records a dispatch of width x height x layers workgroups.  There
    // is no pipeline here: an operator either overrides this or, like the ones of this
    // library, calls the C ABI from execute() and never gets here.
    virtual void submit(void *ptr, int width, int height, int layers) {
        (void)ptr;
        throw std::runtime_error("Operator::submit: " + convert_optype_to_string(type_) + " (" + std::to_string(width) + "x" +
                                 std::to_string(height) + "x" + std::to_string(layers) +
                                 " workgroups) has no HIP kernel behind it in this library");
    }

    // Calls func(T{}) for the element type `dtype` names; throws for a type no
    // operator here handles (ops/Operator.hpp:198-222).
    using SupportedTypes = std::tuple<float, uint16_t, int, int64_t, int8_t>;
    template <typename Func> void dispatch_by_dtype(const std::type_info &dtype, Func &&func) {
        bool dispatched = false;
        std::apply(
            [&](auto... types) {
                (([&] {
                     using T = decltype(types);
                     if (dtype == typeid(T)) {
                         func(T{});
                         dispatched = true;
                     }
                 }()),
                 ...);
            },
            SupportedTypes{});
        if (!dispatched) throw std::runtime_error("Unsupported dtype: " + std::string(dtype.name()));
    }

    // Device workspace an operator keeps between calls (the reference's Topk
    // keeps ping-pong temporaries the same way, ops/Topk.hpp:46-55,221-224).
    // Grown on demand; cleared once whenever it is (re)allocated.
    void *workspace(size_t bytes) {
        if (bytes == 0) return nullptr;
        if (!workspace_ || workspace_->size() < bytes) {
            const size_t sz = (bytes + 255) / 256 * 256;
            workspace_ = std::make_shared<VulkanBuffer>(m_dev_, sz);
            void *q = m_dev_->getComputeQueue(m_id_);
            hip_check(vkop_hip_workspace_init(workspace_->data(), sz, q), "vkop_hip_workspace_init");
            hip_check(vkop_hip_stream_sync(q), "vkop_hip_stream_sync");
        }
        return workspace_->data();
    }
    size_t workspace_size() const { return workspace_ ? workspace_->size() : 0; }

  private:
    void dump(const char *what, const std::shared_ptr<core::ITensor> &t) {
        std::printf("%s:\n", what);
        dispatch_by_dtype(t->dtype(), [&](auto dummy) {
            using T = decltype(dummy);
            if constexpr (std::is_same_v<T, float> || std::is_same_v<T, uint16_t> || std::is_same_v<T, int>) {
                auto tt = core::as_tensor<T>(t);
                tt->copyToCPU(m_cmdpool_);
                tt->print_tensor(64);
                tt->toGPU();
            }
        });
    }
    virtual void execute(const std::vector<std::shared_ptr<core::ITensor>> &inputs,
                         const std::vector<std::shared_ptr<core::ITensor>> &outputs) = 0;

    std::shared_ptr<VulkanBuffer> workspace_;
};

// One definition program-wide (the reference defines its statics in
// core/runtime.cpp:14-16; an inline variable needs no such translation unit).
inline std::atomic<int> Operator::instance_count_{0};

}  // namespace ops
}  // namespace vkop
#endif  // VKOP_HIP_OPS_OPERATOR_HPP_
