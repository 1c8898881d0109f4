// Host tensor with a lazily created device buffer: the part of the reference's
// core/Tensor.hpp (ITensor :35-209, Tensor<T> :211-1057) that the Softmax / TopK
// operators and their callers use.  Row-major, up to four extents, element
// types float, uint16_t (IEEE binary16 bits), int.  Images, uniform buffers and
// buffer views are Vulkan notions with no counterpart here: every tensor is a
// plain device buffer.
#ifndef VKOP_HIP_CORE_TENSOR_HPP_
#define VKOP_HIP_CORE_TENSOR_HPP_

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <memory>
#include <stdexcept>
#include <typeinfo>
#include <vector>

#include "hip/Runtime.hpp"

#define UP_DIV(x, y) (((x) + (y) - 1) / (y))

namespace vkop {
using ivec4 = int[4];

namespace core {

template <typename T> class Tensor;

class ITensor {
  public:
    virtual ~ITensor() = default;
    virtual const std::type_info &dtype() const = 0;

    uint8_t num_dims() const { return n_dims_; }
    int size() const { return size_; }  // bytes
    bool is_on_GPU() const { return converted_; }
    void toGPU() { converted_ = true; }
    void toCPU() { converted_ = false; }
    void ref_inc() { ref_cnt_++; }
    void ref_dec() { ref_cnt_--; }
    int ref_cnt() const { return ref_cnt_; }
    void set_ref_cnt(uint16_t cnt) { ref_cnt_ = cnt; }
    void set_ref_cnt_forever() { ref_cnt_ = std::numeric_limits<uint16_t>::max(); }

    // Trailing zero extents are not part of the shape (core/Tensor.hpp:56-67).
    std::vector<int> getShape() const {
        std::vector<int> s;
        int nd = dims_[3] ? 4 : dims_[2] ? 3 : dims_[1] ? 2 : 1;
        for (int i = 0; i < nd; i++) s.push_back(dims_[i]);
        return s;
    }

    // binary16 <-> binary32, round to nearest even, subnormals, inf and NaN kept
    // (the conversions core/Tensor.hpp:116-198 gets from _cvtsh_ss / _cvtss_sh).
    static float fp16_to_fp32(uint16_t h) {
        const uint32_t sign = (static_cast<uint32_t>(h) & 0x8000u) << 16;
        uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
        if (exp == 0) {
            if (man == 0) {
                bits = sign;
            } else {
                int e = -1;
                do {
                    man <<= 1;
                    e++;
                } while ((man & 0x400u) == 0);
                bits = sign | ((127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
            }
        } else if (exp == 31) {
            bits = sign | 0x7F800000u | (man << 13);
        } else {
            bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
        }
        float f;
        std::memcpy(&f, &bits, sizeof f);
        return f;
    }
    static uint16_t fp32_to_fp16(float f) {
        uint32_t x;
        std::memcpy(&x, &f, sizeof x);
        const uint16_t sign = static_cast<uint16_t>((x >> 16) & 0x8000u);
        const uint32_t abs = x & 0x7FFFFFFFu;
        if (abs >= 0x7F800000u)  // inf / NaN (a NaN keeps a non-zero payload)
            return static_cast<uint16_t>(sign | 0x7C00u | (abs > 0x7F800000u ? (0x200u | ((abs >> 13) & 0x3FFu)) : 0u));
        if (abs >= 0x477FF000u) return static_cast<uint16_t>(sign | 0x7C00u);  // rounds to inf
        if (abs < 0x33000001u) return sign;                                      // rounds to zero
        const int e = static_cast<int>(abs >> 23) - 127;
        uint32_t man = (abs & 0x7FFFFFu) | 0x800000u;
        int shift = e < -14 ? (13 + (-14 - e)) : 13;
        uint32_t half = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1u), mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1u))) half++;
        // for normals `half` still carries the hidden bit: adding the exponent field
        // with (e + 14) makes a mantissa carry spill into the exponent correctly
        const uint32_t out = e < -14 ? half : (static_cast<uint32_t>(e + 14) << 10) + half;
        return static_cast<uint16_t>(sign | out);
    }

  protected:
    ivec4 dims_ = {0, 0, 0, 0};
    int size_ = 0;
    uint16_t ref_cnt_ = 0;
    uint8_t n_dims_ = 0;
    bool converted_ = false;
};

template <typename T> class Tensor : public ITensor {
  public:
    explicit Tensor(bool is_on_GPU = false) {
        if (is_on_GPU) toGPU();
    }
    Tensor(int n, int c, int h, int w, bool is_on_GPU = false) {
        set_dims(std::vector<int>{n, c, h, w});
        n_dims_ = static_cast<uint8_t>((n != 0) + (c != 0) + (h != 0) + (w != 0));
        if (is_on_GPU) toGPU();
        else reserveOnCPU();
    }
    template <typename U> explicit Tensor(const std::vector<U> &dims, bool is_on_GPU = false) {
        set_dims(dims);
        if (is_on_GPU) toGPU();
        else reserveOnCPU();
    }

    const std::type_info &dtype() const override { return typeid(T); }

    // New extents; host storage follows unless the tensor lives on the device,
    // a device buffer that has become too small is dropped (core/Tensor.hpp:296-315).
    template <typename U> void resize(const std::vector<U> &dims) {
        set_dims(dims);
        if (!is_on_GPU()) reserveOnCPU();
        if (buffer_ && buffer_->size() < padded_bytes()) buffer_.reset();
    }
    void resize(int n, int c, int h, int w) { resize(std::vector<int>{n, c, h, w}); }

    int num_elements() const { return size_ / static_cast<int>(sizeof(T)); }
    T *data() { return data_.data(); }
    const std::vector<T> &vector() const { return data_; }
    T &operator[](std::size_t i) { return data_[i]; }
    const T &operator[](std::size_t i) const { return data_[i]; }
    T &at(std::size_t i) {
        if (i >= data_.size()) throw std::out_of_range("Tensor::at");
        return data_[i];
    }

    void fillToCPU(const std::vector<T> &data) {
        reserveOnCPU();
        std::memcpy(data_.data(), data.data(), std::min(data.size(), data_.size()) * sizeof(T));
    }
    void fillToCPU(const T *data) {
        reserveOnCPU();
        std::memcpy(data_.data(), data, data_.size() * sizeof(T));
    }
    void reserveOnCPU() { data_.resize(static_cast<size_t>(num_elements())); }

    // The device buffer, created on first use and padded to a multiple of four
    // elements (core/Tensor.hpp:722-729).
    std::shared_ptr<HipBuffer> as_storage_buffer(const std::shared_ptr<HipDevice> &dev,
                                                 const std::shared_ptr<HipCommandBuffer> & = nullptr) {
        if (!buffer_ || buffer_->size() < padded_bytes()) buffer_ = std::make_shared<HipBuffer>(dev, padded_bytes());
        return buffer_;
    }
    // Host -> device; blocking, like the reference's staging copy + submit
    // (core/Tensor.hpp:540-554, 765-801).  No-op if the data already lives there.
    void copyToGPU(const std::shared_ptr<HipCommandPool> &pool, T *data = nullptr) {
        if (is_on_GPU()) return;
        as_storage_buffer(pool->getDevice());
        const T *src = data ? data : data_.data();
        void *q = pool->getDevice()->getComputeQueue(0);
        hip_check(vkop_hip_memcpy_h2d(buffer_->data(), src, static_cast<size_t>(size_), q), "vkop_hip_memcpy_h2d");
        toGPU();
    }
    // Device -> host; blocking (core/Tensor.hpp:556-567, 803-832).
    void copyToCPU(const std::shared_ptr<HipCommandPool> &pool) {
        if (!is_on_GPU()) return;
        if (!buffer_) throw std::runtime_error("copyToCPU: tensor has no device buffer");
        reserveOnCPU();
        void *q = pool->getDevice()->getComputeQueue(0);
        hip_check(vkop_hip_memcpy_d2h(data_.data(), buffer_->data(), static_cast<size_t>(size_), q), "vkop_hip_memcpy_d2h");
        toCPU();
    }

    void print_tensor(int len = -1) const {
        int cnt = 0;
        for (const auto &v : data_) {
            if (len >= 0 && cnt++ >= len) break;
            if constexpr (std::is_same_v<T, uint16_t>) std::printf("%g ", fp16_to_fp32(v));
            else if constexpr (std::is_same_v<T, float>) std::printf("%g ", v);
            else std::printf("%lld ", static_cast<long long>(v));
        }
        std::printf("\n");
    }

  private:
    template <typename U> void set_dims(const std::vector<U> &dims) {
        if (dims.size() > 4) throw std::runtime_error("Tensor: at most four extents");
        std::memset(dims_, 0, sizeof dims_);
        n_dims_ = static_cast<uint8_t>(dims.size());
        long long bytes = dims.empty() ? 0 : static_cast<long long>(sizeof(T));
        int i = 0;
        for (auto d : dims) {
            bytes *= static_cast<long long>(d);
            dims_[i++] = static_cast<int>(d);
        }
        if (bytes > std::numeric_limits<int>::max()) throw std::runtime_error("Tensor: larger than 2 GiB");
        size_ = static_cast<int>(bytes);
    }
    size_t padded_bytes() const { return static_cast<size_t>(UP_DIV(num_elements(), 4)) * 4 * sizeof(T) + 16; }

    std::vector<T> data_;
    std::shared_ptr<HipBuffer> buffer_;
};

template <typename T> std::shared_ptr<Tensor<T>> as_tensor(const std::shared_ptr<ITensor> &t) {
    if (t == nullptr || t->dtype() != typeid(T)) return nullptr;
    return std::static_pointer_cast<Tensor<T>>(t);
}

}  // namespace core
}  // namespace vkop
#endif  // VKOP_HIP_CORE_TENSOR_HPP_
