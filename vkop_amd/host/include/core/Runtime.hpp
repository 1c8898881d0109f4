// The part of the reference's Runtime (core/runtime.cpp) around the operators
// of this library: LoadModel (:33-363) for models made of them, GetInput /
// GetOutput / GetInitializer (:365-402), RegisterPostProcess (:480-520), Run
// (:404-458), ReadResult (:460-478).
//
// LoadModel reads a .vkopbin (model/load.hpp), creates the tensors and builds
// the plan level by level from the file's concurrent levels and dependencies,
// as the reference does.  Differences, on purpose:
//   * a node whose operator this library does not have stops the load with an
//     error naming it (the reference skips the node and fails later);
//   * tensors of index outputs (TopK's second, Nms's) are int32 whatever the
//     precision; every intermediate tensor gets storage of its own;
//   * model inputs are plain buffers of the runtime's precision (the reference
//     makes them fp16 images for its convolution front end);
//   * a TopK node without a K attribute takes K from its second input when
//     that is an int64 initializer (ONNX keeps K there).
// Without a model, the tensor a model would produce is handed in with
// SetOutput().  Post-processing operators are appended one level at a time,
// each depending on the level before it, exactly as the reference does.
//
// One addition in both paths: a TopK that alone reads the output of a Softmax
// along the same axis replaces the pair by one fused operator (in a model also a
// Reduce "max" over that one axis: the class maximum of class probabilities).  For registered
// post-processing that is legal because every registration clears the set of
// tensors read back (core/runtime.cpp:515-519), so after the TOPK registration
// the softmax tensor is neither read back nor an input of anything else; for a
// model the softmax output must have that one consumer and not be a model output.
#ifndef VKOP_HIP_CORE_RUNTIME_HPP_
#define VKOP_HIP_CORE_RUNTIME_HPP_

#include <chrono>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "model/load.hpp"
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

    void setPrecision(int precision) { precision_ = precision; }
    int getPrecision() const { return precision_; }

    void LoadModel() {
        const load::VkModel model(model_path_);
        std::unordered_map<std::string, std::shared_ptr<ITensor>> tensor_map;
        std::unordered_map<std::string, int> consumers;
        std::unordered_map<std::string, const load::Node *> node_by_name, producer;
        std::unordered_map<std::string, size_t> output_slot;
        for (const auto &n : model.nodes) {
            node_by_name[n.name] = &n;
            for (const auto &in : n.inputs) consumers[in.name] += 1;
            for (size_t i = 0; i < n.outputs.size(); ++i) {
                producer[n.outputs[i].name] = &n;
                output_slot[n.outputs[i].name] = i;
            }
            if (ops::convert_opstring_to_enum(n.op_type) == ops::OpType::UNKNOWN || !ops::create_from_type(ops::convert_opstring_to_enum(n.op_type)))
                throw std::runtime_error("LoadModel: node " + n.name + " needs operator " + n.op_type + ", which this library does not have");
        }
        // every initializer's data is as long as its dimensions promise (checked before any device work)
        auto elem_size = [](const std::string &dtype) -> size_t {
            if (dtype == "int8" || dtype == "uint8" || dtype == "bool") return 1;
            if (dtype == "float16" || dtype == "bfloat16" || dtype == "int16" || dtype == "uint16") return 2;
            if (dtype == "int64" || dtype == "uint64" || dtype == "float64") return 8;
            return 4;
        };
        for (const auto &it : model.initializers) (void)model.initializer_data(it.first, elem_size(it.second.dtype));
        auto dev = m_cmdpool_->getVulkanDevice();
        auto make = [this](const std::vector<uint32_t> &dims, bool index, bool on_device = true) -> std::shared_ptr<ITensor> {
            if (index) return std::make_shared<Tensor<int>>(dims, on_device);
            if (precision_ == 1) return std::make_shared<Tensor<uint16_t>>(dims, on_device);
            return std::make_shared<Tensor<float>>(dims, on_device);
        };
        auto holds_indices = [&](const std::string &tensor) {
            auto it = producer.find(tensor);
            if (it == producer.end()) return false;
            const auto type = ops::convert_opstring_to_enum(it->second->op_type);
            return (type == ops::OpType::TOPK && output_slot[tensor] == 1) || type == ops::OpType::NMS;
        };
        for (const auto &i : model.inputs) {
            auto t = make(i.dims, false, /*on_device=*/false);  // filled on the host, then copyToGPU()
            t->set_ref_cnt_forever();
            inputs_[i.name] = t;
            tensor_map[i.name] = t;
        }
        for (const auto &o : model.outputs) {
            auto t = make(o.dims, holds_indices(o.name));
            t->set_ref_cnt_forever();
            outputs_[o.name] = t;
            tensor_map[o.name] = t;
            real_outputs_[o.name] = t;
        }
        for (const auto &it : model.initializers) {
            const auto &init = it.second;
            const uint8_t *src = model.initializer_data(init.name, elem_size(init.dtype));  // (length checked again)
            auto host_only = [&](auto t, const auto *data) {
                t->set_ref_cnt_forever();
                t->fillToCPU(data);
                tensor_map[init.name] = t;
                initializers_[init.name] = t;
            };
            auto on_device = [&](auto t, auto *data) {
                host_only(t, data);
                t->as_storage_buffer(dev);
                t->copyToGPU(m_cmdpool_);
            };
            if (init.dtype == "int64") host_only(std::make_shared<Tensor<int64_t>>(init.dims), reinterpret_cast<const int64_t *>(src));
            else if (init.dtype == "int32") host_only(std::make_shared<Tensor<int>>(init.dims), reinterpret_cast<const int *>(src));
            else if (init.dtype == "float32") on_device(std::make_shared<Tensor<float>>(init.dims), reinterpret_cast<const float *>(src));
            else if (init.dtype == "float16") on_device(std::make_shared<Tensor<uint16_t>>(init.dims), reinterpret_cast<const uint16_t *>(src));
            else throw std::runtime_error("Only float32/float16/int32/int64 initializer is supported for now " + init.dtype);
        }
        // a Softmax whose only reader is a TopK along the same axis is left out; the TopK becomes the fused operator
        std::unordered_map<std::string, const load::Node *> fused_softmax_of;  // TopK node name -> Softmax node
        if (fuse_) {
            for (const auto &n : model.nodes) {
                if (ops::convert_opstring_to_enum(n.op_type) != ops::OpType::TOPK || n.inputs.empty()) continue;
                auto p = producer.find(n.inputs[0].name);
                if (p == producer.end() || ops::convert_opstring_to_enum(p->second->op_type) != ops::OpType::SOFTMAX) continue;
                const auto &sm = *p->second;
                if (sm.outputs.size() != 1 || sm.inputs.size() != 1 || consumers[sm.outputs[0].name] != 1 || outputs_.count(sm.outputs[0].name)) continue;
                if (!same_axis(sm.attributes, n.attributes, static_cast<int>(sm.outputs[0].dims.size()))) continue;
                fused_softmax_of[n.name] = &sm;
            }
        }
        // the same for a Reduce "max" over the one axis the Softmax in front of it runs along
        if (fuse_) {
            for (const auto &n : model.nodes) {
                if (ops::convert_opstring_to_enum(n.op_type) != ops::OpType::REDUCE || n.inputs.empty()) continue;
                auto p = producer.find(n.inputs[0].name);
                if (p == producer.end() || ops::convert_opstring_to_enum(p->second->op_type) != ops::OpType::SOFTMAX) continue;
                const auto &sm = *p->second;
                if (sm.outputs.size() != 1 || sm.inputs.size() != 1 || consumers[sm.outputs[0].name] != 1 || outputs_.count(sm.outputs[0].name)) continue;
                ops::Reduce probe;
                probe.setAttribute(n.attributes);
                const int rank = static_cast<int>(sm.outputs[0].dims.size());
                if (probe.reduce_op() != static_cast<int>(ops::reduce::ReduceType::MAX) || probe.axes().size() != 1) continue;
                std::unordered_map<std::string, std::string> as_axis = {{"axis", std::to_string(probe.axes()[0])}};
                if (rank < 2 || !same_axis(sm.attributes, as_axis, rank)) continue;
                fused_softmax_of[n.name] = &sm;
            }
        }
        std::unordered_set<std::string> left_out;
        for (const auto &f : fused_softmax_of) left_out.insert(f.second->name);
        std::unordered_map<std::string, size_t> index_of_node;
        for (const auto &level : model.getConcurrentExecutionLevels()) {
            std::vector<size_t> level_indices;
            for (const auto &node_name : level) {
                auto found = node_by_name.find(node_name);
                if (found == node_by_name.end()) throw std::runtime_error("LoadModel: level names unknown node " + node_name);
                if (left_out.count(node_name)) continue;
                const load::Node &n = *found->second;
                const auto fused = fused_softmax_of.find(n.name);
                const load::Node &reads = fused == fused_softmax_of.end() ? n : *fused->second;  // whose inputs and dependencies count
                const auto type = ops::convert_opstring_to_enum(n.op_type);

                std::vector<int> deps;
                for (const auto &d : reads.dependencies) {
                    auto at = index_of_node.find(d);
                    if (at == index_of_node.end()) throw std::runtime_error("LoadModel: node " + n.name + " depends on " + d + ", which does not come before it");
                    deps.push_back(static_cast<int>(at->second));
                }
                std::vector<std::shared_ptr<ITensor>> node_inputs, node_outputs;
                for (const auto &in : reads.inputs) {
                    auto t = tensor_map.find(in.name);
                    if (t != tensor_map.end()) node_inputs.push_back(t->second);
                    else if (in.dims.empty()) node_inputs.push_back(nullptr);  // optional input left out
                    else throw std::runtime_error("LoadModel: node " + n.name + " reads " + in.name + ", which nothing produces");
                }
                for (size_t i = 0; i < n.outputs.size(); ++i) {
                    const auto &out = n.outputs[i];
                    auto t = tensor_map.find(out.name);
                    if (t == tensor_map.end()) {
                        auto made = make(out.dims, holds_indices(out.name));
                        made->set_ref_cnt(static_cast<uint16_t>(consumers[out.name]));
                        t = tensor_map.emplace(out.name, made).first;
                    }
                    node_outputs.push_back(t->second);
                }
                auto attributes = n.attributes;
                if (type == ops::OpType::TOPK && !attributes.count("K") && !attributes.count("k") && n.inputs.size() > 1) {
                    auto k = initializers_.find(n.inputs[1].name);
                    if (k != initializers_.end() && k->second->dtype() == typeid(int64_t) && as_tensor<int64_t>(k->second)->num_elements() >= 1)
                        attributes["K"] = std::to_string((*as_tensor<int64_t>(k->second))[0]);
                }
                if (type == ops::OpType::TOPK && node_inputs.size() > 1) node_inputs.resize(1);  // K is an attribute by now
                std::unique_ptr<ops::Operator> op;
                if (fused != fused_softmax_of.end() && type == ops::OpType::REDUCE) op = std::make_unique<ops::SoftmaxReduceMax>();
                else if (fused != fused_softmax_of.end()) op = std::make_unique<ops::SoftmaxTopk>(precision_);
                else op = ops::create_from_type(type, node_outputs[0]->num_dims() <= 2, precision_, dev->is_support_nv_tensor_core());
                op->set_name(n.name);
                op->set_runtime_device(dev, m_cmdpool_);
                op->setAttribute(attributes);

                const size_t idx = node_ops_.size();
                index_of_node[n.name] = idx;
                if (fused != fused_softmax_of.end()) index_of_node[fused->second->name] = idx;
                level_indices.push_back(idx);
                node_ops_.push_back(std::move(op));
                node_attrs_.push_back(std::move(attributes));
                node_input_tensors_.push_back(std::move(node_inputs));
                node_output_tensors_.push_back(std::move(node_outputs));
                node_is_post_.push_back(false);
                node_dependency_indices_.push_back(std::move(deps));
            }
            if (!level_indices.empty()) level_node_indices_.push_back(std::move(level_indices));
        }
        if (outputs_.size() == 1) output_ = outputs_.begin()->second;
    }

    // core/runtime.cpp:365-402
    std::shared_ptr<ITensor> GetInput(const std::string &name = "") const { return pick(inputs_, name, "Input"); }
    std::shared_ptr<ITensor> GetOutput(const std::string &name = "") const {
        if (name.empty() && outputs_.empty()) return output_;  // no model: what SetOutput() handed in
        return pick(outputs_, name, "Output");
    }
    std::shared_ptr<ITensor> GetInitializer(const std::string &name) const {
        auto it = initializers_.find(name);
        return it == initializers_.end() ? nullptr : it->second;
    }

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
    static bool same_axis(const std::unordered_map<std::string, std::string> &s, const std::unordered_map<std::string, std::string> &topk_attrs,
                          int rank) {
        auto norm = [rank](int a) { return a < 0 ? a + rank : a; };
        int sa = 0;  // Softmax's default (ops/Softmax.hpp: GpuSoftMaxParam starts at 0)
        if (s.count("axis")) sa = std::stoi(s.at("axis"));
        else if (s.count("dim")) sa = std::stoi(s.at("dim"));
        int ta = -1;  // TopK's default (ops/Topk.hpp:41)
        if (topk_attrs.count("axis")) ta = std::stoi(topk_attrs.at("axis"));
        if (rank == 1) return true;
        return norm(sa) == norm(ta);
    }
    bool same_axis(size_t softmax_node, const std::unordered_map<std::string, std::string> &topk_attrs,
                   const std::shared_ptr<ITensor> &t) const {
        return same_axis(node_attrs_[softmax_node], topk_attrs, t->num_dims());
    }
    static std::shared_ptr<ITensor> pick(const std::map<std::string, std::shared_ptr<ITensor>> &from, const std::string &name,
                                         const char *what) {
        if (name.empty() && from.size() > 1) throw std::runtime_error(std::string(what) + " name is empty but there are multiple");
        if (name.empty() && from.size() == 1) return from.begin()->second;
        auto it = from.find(name);
        return it == from.end() ? nullptr : it->second;
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
    std::map<std::string, std::shared_ptr<ITensor>> inputs_, outputs_, initializers_;
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
