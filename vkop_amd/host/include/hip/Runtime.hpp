// Device, queues and recorded work over the C ABI of libvkop_hip.so.
//
// These are the few pieces of the reference's Vulkan layer that the operator
// interface and its callers touch: a device (vulkan/VulkanDevice.hpp), a pool
// that hands out per-queue command buffers (vulkan/VulkanCommandPool.hpp), a
// command buffer that is recorded, submitted and waited for
// (vulkan/VulkanCommandBuffer.hpp) and a device buffer (vulkan/VulkanBuffer.hpp).
// Only the methods those callers use exist (core/runtime.cpp:418-446,
// tests/setup.hpp:134-201).  The reference's class names are kept as aliases so
// caller code compiles unchanged.
//
// "Recording" keeps a list of deferred launches; submit() enqueues them on the
// queue's HIP stream and wait() waits for an event recorded behind them.  A
// recording can be submitted any number of times.
#ifndef VKOP_HIP_RUNTIME_HPP_
#define VKOP_HIP_RUNTIME_HPP_

#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "vkop_hip.h"

// The two words of Vulkan vocabulary the reference's operator sources spell out when
// they call their base class (ops/Softmax.hpp:33-44, ops/Topk.hpp:33-37): the kind of
// each binding (values as in vulkan_core.h).  Nothing here acts on them; they are kept
// so that an operator written against the reference's base class compiles.  Global, as
// in vulkan_core.h, and skipped when that header is already in.
#ifndef VULKAN_CORE_H_
enum VkDescriptorType {
    VK_DESCRIPTOR_TYPE_SAMPLER = 0,
    VK_DESCRIPTOR_TYPE_COMBINED_IMAGE_SAMPLER = 1,
    VK_DESCRIPTOR_TYPE_SAMPLED_IMAGE = 2,
    VK_DESCRIPTOR_TYPE_STORAGE_IMAGE = 3,
    VK_DESCRIPTOR_TYPE_UNIFORM_TEXEL_BUFFER = 4,
    VK_DESCRIPTOR_TYPE_STORAGE_TEXEL_BUFFER = 5,
    VK_DESCRIPTOR_TYPE_UNIFORM_BUFFER = 6,
    VK_DESCRIPTOR_TYPE_STORAGE_BUFFER = 7
};
#endif
#ifndef DESCRIPTOR_TYPE_STORAGE
#define DESCRIPTOR_TYPE_STORAGE VK_DESCRIPTOR_TYPE_STORAGE_BUFFER        /* vulkan/VulkanResource.hpp:11 */
#define DESCRIPTOR_TYPE_UNIFORM VK_DESCRIPTOR_TYPE_UNIFORM_TEXEL_BUFFER  /* vulkan/VulkanResource.hpp:12 */
#endif

namespace vkop {

constexpr int kInflight = 2;  // queues in flight, as vulkan/VulkanDevice.hpp:13

// Device failures surface as std::runtime_error, like the reference's Vulkan
// wrappers; nothing above the C ABI returns status codes.
inline void hip_check(int status, const char *what) {
    if (status != VKOP_HIP_OK)
        throw std::runtime_error(std::string(what) + ": " + vkop_hip_last_error());
}

class HipDevice {
  public:
    explicit HipDevice(int index = 0) : index_(index) {
        hip_check(vkop_hip_init(index), "vkop_hip_init");
        char name[128] = "";
        hip_check(vkop_hip_device_info(name, sizeof name, &compute_units_, &memory_bytes_), "vkop_hip_device_info");
        name_ = name;
        for (auto &q : queues_) hip_check(vkop_hip_stream_create(&q), "vkop_hip_stream_create");
    }
    ~HipDevice() {
        for (auto &q : queues_) vkop_hip_stream_destroy(q);
    }
    HipDevice(const HipDevice &) = delete;
    HipDevice &operator=(const HipDevice &) = delete;

    const std::string &getDeviceName() const { return name_; }
    int getComputeUnits() const { return compute_units_; }
    size_t getMemoryBytes() const { return memory_bytes_; }
    // queue `id` of kInflight (a HIP stream); the reference hands out VkQueue
    void *getComputeQueue(int id = 0) const { return queues_[static_cast<size_t>(id) % kInflight]; }
    void wait_all_done() const {
        for (auto *q : queues_) hip_check(vkop_hip_stream_sync(q), "vkop_hip_stream_sync");
    }
    bool is_support_nv_tensor_core() const { return false; }
    bool is_support_host_image_copy() const { return false; }

  private:
    int index_;
    std::string name_;
    int compute_units_ = 0;
    size_t memory_bytes_ = 0;
    void *queues_[kInflight] = {nullptr, nullptr};
};

// Device memory owned by a tensor or an operator.
class HipBuffer {
  public:
    HipBuffer(std::shared_ptr<HipDevice> dev, size_t bytes) : dev_(std::move(dev)), bytes_(bytes) {
        hip_check(vkop_hip_malloc(&ptr_, bytes), "vkop_hip_malloc");
    }
    ~HipBuffer() { vkop_hip_free(ptr_); }
    HipBuffer(const HipBuffer &) = delete;
    HipBuffer &operator=(const HipBuffer &) = delete;
    void *data() const { return ptr_; }
    size_t size() const { return bytes_; }

  private:
    std::shared_ptr<HipDevice> dev_;
    void *ptr_ = nullptr;
    size_t bytes_ = 0;
};

class HipCommandPool {
  public:
    explicit HipCommandPool(std::shared_ptr<HipDevice> dev) : dev_(std::move(dev)) {}
    const std::shared_ptr<HipDevice> &getVulkanDevice() const { return dev_; }
    const std::shared_ptr<HipDevice> &getDevice() const { return dev_; }

  private:
    std::shared_ptr<HipDevice> dev_;
};

class HipCommandBuffer;
// What buildSubmitInfo() hands to submit(): the recording to run.
struct HipSubmitInfo {
    HipCommandBuffer *cmd = nullptr;
};

class HipCommandBuffer {
  public:
    using Launch = std::function<int(void *stream)>;

    HipCommandBuffer(std::shared_ptr<HipCommandPool> pool, int id) : pool_(std::move(pool)), id_(id) {
        hip_check(vkop_hip_event_create(&done_), "vkop_hip_event_create");
    }
    ~HipCommandBuffer() { vkop_hip_event_destroy(done_); }
    HipCommandBuffer(const HipCommandBuffer &) = delete;
    HipCommandBuffer &operator=(const HipCommandBuffer &) = delete;

    void begin() {
        launches_.clear();
        recording_ = true;
    }
    void end() { recording_ = false; }
    // called by operators while recording
    void record(Launch launch) {
        if (!recording_) throw std::runtime_error("record() outside begin()/end()");
        launches_.emplace_back(std::move(launch));
    }
    void *stream() const { return pool_->getDevice()->getComputeQueue(id_); }
    int queue_id() const { return id_; }

    // This recording starts only after `other`'s latest submission has finished
    // (the reference's addWait on a timeline semaphore, core/runtime.cpp:422-426).
    void addWait(const std::shared_ptr<HipCommandBuffer> &other) {
        if (other && other.get() != this) waits_.push_back(other);
    }
    void clearWaits() { waits_.clear(); }

    HipSubmitInfo buildSubmitInfo() { return HipSubmitInfo{this}; }
    // Enqueues every recording on `queue` in order (VulkanCommandBuffer::submit,
    // as used by core/runtime.cpp:435-441 and tests/setup.hpp:197-199).
    static void submit(void *queue, const std::vector<HipSubmitInfo> &infos) {
        for (const auto &info : infos) {
            for (const auto &w : info.cmd->waits_)
                if (w->submitted_) hip_check(vkop_hip_stream_wait_event(queue, w->done_), "vkop_hip_stream_wait_event");
            for (const auto &launch : info.cmd->launches_) hip_check(launch(queue), "recorded launch");
            hip_check(vkop_hip_event_record(info.cmd->done_, queue), "vkop_hip_event_record");
            info.cmd->submitted_ = true;
        }
    }
    void wait() {
        if (submitted_) hip_check(vkop_hip_event_sync(done_), "vkop_hip_event_sync");
    }
    size_t recorded() const { return launches_.size(); }

  private:
    std::shared_ptr<HipCommandPool> pool_;
    int id_;
    bool recording_ = false;
    bool submitted_ = false;
    void *done_ = nullptr;
    std::vector<Launch> launches_;
    std::vector<std::shared_ptr<HipCommandBuffer>> waits_;
};

// The reference's names, so that caller code written against it still compiles.
using VulkanDevice = HipDevice;
using VulkanResource = HipBuffer;  // what a tensor binds (vulkan/VulkanResource.hpp): here always a device buffer
using VulkanCommandPool = HipCommandPool;
using VulkanCommandBuffer = HipCommandBuffer;
using VulkanBuffer = HipBuffer;

}  // namespace vkop
#endif  // VKOP_HIP_RUNTIME_HPP_
