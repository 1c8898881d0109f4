// The post-processing slice of the reference's Runtime (core/runtime.cpp):
// RegisterPostProcess (:480-520), Run (:404-458), ReadResult (:460-478).
//
// The model part of the reference's Runtime (loading a .vkopbin, building the
// operator graph) is not here; the tensor the model would produce is handed in
// with SetOutput().  Post-processing operators are appended one level at a
// time, each depending on the level before it, exactly as the reference does,
// with one addition: a TOPK registered on the output of the SOFTMAX registered
// just before it replaces the pair by one fused operator.  That is legal
// because every registration clears the set of tensors read back
// (core/runtime.cpp:515-519), so after the TOPK registration the softmax tensor
// is neither read back nor an input of anything else.
#ifndef VKOP_HIP_CORE_RUNTIME_HPP_
#define VKOP_HIP_CORE_RUNTIME_HPP_

#include <chrono>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "ops/OperatorFactory.hpp"

namespace vkop {
namespace core {

class Runtime {
  public:
    explicit Runtime(const std::shared_ptr<VulkanCommandPool> &cmdpool, const std::string &model_path = "",
                     int precision = 0)
        : m_cmdpool_(cmdpool), model_path_(model_path), precision_(precision) {}

    // Stands in for the model: the tensor post-processing starts from.
    void SetOutput(const std::shared_ptr<ITensor> &t) { output_ = t; }
    std::shared_ptr<ITensor> GetOutput() const { return output_; }

    // Switches the SOFTMAX + TOPK fusion off (for comparisons); on by default.
    void set_postprocess_fusion(bool on) { fuse_ = on; }

    void RegisterPostProcess(ops::OpType type, const std::unordered_map<std::string, std::string> &attributes,
                             const std::vector<std::shared_ptr<ITensor>> &inputs,
                             const std::vector<std::shared_ptr<ITensor>> &outputs) {
        auto dev = m_cmdpool_->getVulkanDevice();
        std::unique_ptr<ops::Operator> op;
        std::vector<std::shared_ptr<ITensor>> op_inputs = inputs;
        bool fused = false;
        if (fuse_ && type == ops::OpType::TOPK && !node_ops_.empty() && !level_node_indices_.empty() &&
            level_node_indices_.back().size() == 1) {
            const size_t prev = level_node_indices_.back()[0];
            if (node_ops_[prev]->get_type() == ops::OpType::SOFTMAX && node_is_post_[prev] &&
                node_output_tensors_[prev].size() == 1 && inputs.size() == 1 &&
                node_output_tensors_[prev][0] == inputs[0] && same_axis(prev, attributes, inputs[0])) {
                // the softmax node goes; the fused operator reads what it read
                op_inputs = node_input_tensors_[prev];
                remove_last_node();
                op = std::make_unique<ops::SoftmaxTopk>(precision_);
                fused = true;
            }
        }
        if (!op) op = ops::create_from_type(type, outputs[0]->num_dims() <= 2, precision_, dev->is_support_nv_tensor_core());
        if (!op) throw std::runtime_error("RegisterPostProcess: no operator for " + ops::convert_optype_to_string(type));
        op->set_name(std::string(fused ? "post_Softmax+" : "post_") + ops::convert_optype_to_string(type));
        op->set_runtime_device(dev, m_cmdpool_);
        op->setAttribute(attributes);

        const size_t idx = node_ops_.size();
        node_ops_.push_back(std::move(op));
        node_attrs_.push_back(attributes);
        node_input_tensors_.push_back(op_inputs);
        node_output_tensors_.push_back(outputs);
        node_is_post_.push_back(true);
        // depends on every node of the level before it (core/runtime.cpp:499-508)
        std::vector<int> deps;
        if (!level_node_indices_.empty())
            for (auto i : level_node_indices_.back()) deps.push_back(static_cast<int>(i));
        node_dependency_indices_.push_back(std::move(deps));
        level_node_indices_.push_back({idx});
        // only the newest operator's outputs are read back (core/runtime.cpp:515-519)
        real_outputs_.clear();
        for (size_t i = 0; i < outputs.size(); ++i)
            real_outputs_["post_" + ops::convert_optype_to_string(type) + std::to_string(i)] = outputs[i];
    }

    // Records every operator level by level, alternating over the kInflight
    // queues inside a level, submits, and waits for the last level.  Returns the
    // wall-clock time in milliseconds (core/runtime.cpp:404-458).
    double Run() {
        auto dev = m_cmdpool_->getVulkanDevice();
        const auto start = std::chrono::steady_clock::now();
        std::vector<std::shared_ptr<VulkanCommandBuffer>> last(kInflight);
        for (size_t level = 0; level < level_node_indices_.size(); level++) {
            int id = 0;
            for (auto node : level_node_indices_[level]) {
                node_ops_[node]->onExecute(node_input_tensors_[node], node_output_tensors_[node], id);
                auto cmd = node_ops_[node]->get_record();
                for (int dep : node_dependency_indices_[node]) cmd->addWait(node_ops_[static_cast<size_t>(dep)]->get_record());
                // Submitted at once, in level order: an event can only be waited for
                // after it has been recorded, so a dependency is always submitted first.
                VulkanCommandBuffer::submit(dev->getComputeQueue(id), {cmd->buildSubmitInfo()});
                if (level + 1 == level_node_indices_.size()) last[static_cast<size_t>(id)] = cmd;
                id = (id + 1) % kInflight;
            }
        }
        for (auto &cmd : last)
            if (cmd) cmd->wait();
        for (auto &op : node_ops_)
            if (op->get_record()) op->get_record()->clearWaits();
        const std::chrono::duration<double> elapsed = std::chrono::steady_clock::now() - start;
        return elapsed.count() * 1000.0;
    }

    // Brings the tensors of the newest post-processing operator to the host
    // (core/runtime.cpp:460-478).
    void ReadResult() {
        m_cmdpool_->getVulkanDevice()->wait_all_done();
        for (auto &p : real_outputs_) {
            if (p.second->dtype() == typeid(float)) as_tensor<float>(p.second)->copyToCPU(m_cmdpool_);
            else if (p.second->dtype() == typeid(int)) as_tensor<int>(p.second)->copyToCPU(m_cmdpool_);
            else if (p.second->dtype() == typeid(uint16_t)) as_tensor<uint16_t>(p.second)->copyToCPU(m_cmdpool_);
            else throw std::runtime_error("ReadResult: unsupported element type");
        }
    }

    const std::map<std::string, std::shared_ptr<ITensor>> &GetRealOutputs() const { return real_outputs_; }
    size_t num_nodes() const { return node_ops_.size(); }
    std::string node_name(size_t i) const { return node_ops_[i]->get_name(); }
    void TraceNode(const std::string &name) {
        for (auto &op : node_ops_)
            if (op->get_name() == name) op->enable_trace();
    }

  private:
    // The softmax must run along the axis the top-k selects on.
    bool same_axis(size_t softmax_node, const std::unordered_map<std::string, std::string> &topk_attrs,
                   const std::shared_ptr<ITensor> &t) const {
        const int rank = t->num_dims();
        auto norm = [rank](int a) { return a < 0 ? a + rank : a; };
        int sa = 0;  // Softmax's default (ops/Softmax.hpp: GpuSoftMaxParam starts at 0)
        const auto &s = node_attrs_[softmax_node];
        if (s.count("axis")) sa = std::stoi(s.at("axis"));
        else if (s.count("dim")) sa = std::stoi(s.at("dim"));
        int ta = -1;  // TopK's default (ops/Topk.hpp:41)
        if (topk_attrs.count("axis")) ta = std::stoi(topk_attrs.at("axis"));
        if (rank == 1) return true;
        return norm(sa) == norm(ta);
    }
    void remove_last_node() {
        node_ops_.pop_back();
        node_attrs_.pop_back();
        node_input_tensors_.pop_back();
        node_output_tensors_.pop_back();
        node_is_post_.pop_back();
        node_dependency_indices_.pop_back();
        level_node_indices_.pop_back();
    }

    std::shared_ptr<VulkanCommandPool> m_cmdpool_;
    std::string model_path_;
    int precision_ = 0;
    bool fuse_ = true;
    std::shared_ptr<ITensor> output_;
    std::vector<std::unique_ptr<ops::Operator>> node_ops_;
    std::vector<std::unordered_map<std::string, std::string>> node_attrs_;
    std::vector<std::vector<std::shared_ptr<ITensor>>> node_input_tensors_;
    std::vector<std::vector<std::shared_ptr<ITensor>>> node_output_tensors_;
    std::vector<bool> node_is_post_;
    std::vector<std::vector<int>> node_dependency_indices_;
    std::vector<std::vector<size_t>> level_node_indices_;
    std::map<std::string, std::shared_ptr<ITensor>> real_outputs_;
};

}  // namespace core
}  // namespace vkop
#endif  // VKOP_HIP_CORE_RUNTIME_HPP_
