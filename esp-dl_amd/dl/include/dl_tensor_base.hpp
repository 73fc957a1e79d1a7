// dl::TensorBase / dl::ExponentInfo: exponent-tagged NHWC tensors, host or device resident.
//
// Public surface follows esp-dl/dl/tensor/include/dl_tensor_base.hpp:22-211 (ExponentInfo) and
// :297-744 (TensorBase): real value = q * 2^exponent, exponent per tensor or per output channel,
// `assign()` requantizes between exponents / dtypes.  Differences made for the GPU executor:
//   - `caps` says where `data` lives (MALLOC_CAP_HOST / MALLOC_CAP_DEVICE);
//   - the leading dimension of an activation is the batch (the reference fixes it to 1);
//   - to_device() / to_host() / copy_from() move bytes across PCIe explicitly.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "dl_define.hpp"

namespace dl {

class ExponentInfo {
private:
    int m_exponent;
    std::vector<int> m_exponents; // non-empty only for per-channel

public:
    ExponentInfo(int exponent = 0) : m_exponent(exponent) {}
    ExponentInfo(const std::vector<int> &exponents) : m_exponent(0)
    {
        if (exponents.size() <= 1)
            m_exponent = exponents.empty() ? 0 : exponents[0];
        else
            m_exponents = exponents;
    }
    ExponentInfo &operator=(int value)
    {
        m_exponents.clear();
        m_exponent = value;
        return *this;
    }
    int get(int ch = -1) const { return (ch < 0 || m_exponents.empty()) ? m_exponent : m_exponents[ch]; }
    operator int() const { return m_exponent; }
    bool is_per_channel() const { return m_exponents.size() > 1; }
    int channel_size() const { return m_exponents.empty() ? 1 : (int)m_exponents.size(); }
    const int *data() const { return m_exponents.empty() ? &m_exponent : m_exponents.data(); }
    bool operator==(const ExponentInfo &o) const
    {
        if (is_per_channel() != o.is_per_channel())
            return false;
        return is_per_channel() ? m_exponents == o.m_exponents : m_exponent == o.m_exponent;
    }
    bool operator!=(const ExponentInfo &o) const { return !(*this == o); }
};

// Same numbering as the .espdl TensorDataType (esp-dl/fbs_loader/espdl.fbs:24-39).
typedef enum {
    DATA_TYPE_UNDEFINED = 0,
    DATA_TYPE_FLOAT = 1,
    DATA_TYPE_UINT8 = 2,
    DATA_TYPE_INT8 = 3,
    DATA_TYPE_UINT16 = 4,
    DATA_TYPE_INT16 = 5,
    DATA_TYPE_INT32 = 6,
    DATA_TYPE_INT64 = 7,
    DATA_TYPE_STRING = 8,
    DATA_TYPE_BOOL = 9,
    DATA_TYPE_FLOAT16 = 10,
    DATA_TYPE_DOUBLE = 11,
    DATA_TYPE_UINT32 = 12,
    DATA_TYPE_UINT64 = 13,
} dtype_t;

size_t dtype_sizeof(dtype_t dtype);
const char *dtype_to_string(dtype_t dtype);
std::string vector_to_string(const std::vector<int> &shape);

class TensorBase {
public:
    int64_t size;           ///< number of elements
    std::vector<int> shape; ///< NHWC for activations
    dtype_t dtype;
    ExponentInfo exponent;
    bool auto_free; ///< free `data` on destruction
    void *data;     ///< host or device pointer, see `caps`
    uint32_t caps;  ///< MALLOC_CAP_HOST / MALLOC_CAP_DEVICE
    /// Elements from one position of the last axis run to the next one in memory; 0 = shape.back() (dense).
    /// A model gives a device activation a larger pitch when it lives inside a wider tensor (an output of a
    /// channel Split that stays in its input, an input of a channel Concat that is written in place).  Only
    /// the copies to and from dense tensors below and the modules that say so (Module::reads_channel_slice /
    /// writes_channel_slice) understand such a tensor.
    int channel_pitch = 0;

    /// deep = true: allocate (host or device by `caps`) and copy `element` (a HOST pointer, may be
    /// null -> zero filled).  deep = false: wrap `element`, which must already live where `caps` says.
    TensorBase(std::vector<int> shape, const void *element, int exponent = 0, dtype_t dtype = DATA_TYPE_FLOAT,
               bool deep = true, uint32_t caps = MALLOC_CAP_DEFAULT);
    TensorBase(std::vector<int> shape, const void *element, const std::vector<int> &exponents,
               dtype_t dtype = DATA_TYPE_FLOAT, bool deep = true, uint32_t caps = MALLOC_CAP_DEFAULT);
    virtual ~TensorBase();
    TensorBase(const TensorBase &) = delete;
    TensorBase &operator=(const TensorBase &) = delete;

    bool on_device() const { return (caps & MALLOC_CAP_DEVICE) != 0; }
    bool is_dense() const { return channel_pitch == 0 || shape.empty() || channel_pitch == shape.back(); }
    /// elements between consecutive runs of the last axis
    int get_channel_pitch() const { return is_dense() ? (shape.empty() ? 1 : shape.back()) : channel_pitch; }
    int64_t get_size() const { return size; }
    size_t get_dtype_bytes() const { return dtype_sizeof(dtype); }
    size_t get_bytes() const { return (size_t)size * get_dtype_bytes(); }
    /// bytes rounded up to 256 so that every tensor carved from an arena starts 256-byte aligned
    size_t get_aligned_bytes() const { return (get_bytes() + 255) & ~(size_t)255; }
    void *get_element_ptr() { return data; }
    template <typename T>
    T *get_element_ptr()
    {
        return static_cast<T *>(data);
    }
    TensorBase &set_element_ptr(void *ptr)
    {
        data = ptr;
        return *this;
    }
    std::vector<int> get_shape() const { return shape; }
    TensorBase &set_shape(const std::vector<int> &new_shape);
    int get_exponent() const { return exponent; }
    dtype_t get_dtype() const { return dtype; }
    uint32_t get_caps() const { return caps; }
    bool is_same_shape(const TensorBase *tensor) const { return tensor && shape == tensor->shape; }

    /// Copy with requantization between exponents / int8 <-> int16 (reference: dl_tensor_base.cpp:223-401).
    /// Works for any mix of host and device tensors; device work is enqueued on `stream` and, when a
    /// host tensor is involved, completed before returning.
    bool assign(TensorBase *tensor, void *stream = nullptr);
    /// Raw byte copy from a same-sized tensor or host buffer (no requantization).
    bool copy_from(const TensorBase *tensor, void *stream = nullptr);
    bool copy_from_host(const void *host, size_t bytes, void *stream = nullptr);
    bool copy_to_host(void *host, size_t bytes, void *stream = nullptr) const;
    TensorBase *to_device(void *stream = nullptr) const;
    TensorBase *to_host(void *stream = nullptr) const;

    /// Element-wise comparison after bringing both sides to the host; `epsilon` as in the reference's
    /// Model::test (int8 exact, int16 within 1).
    bool equal(TensorBase *tensor, float epsilon = 1e-6, bool verbose = false);
    template <typename T>
    T get_element(int64_t index); // host tensors only
    void memset(int value, void *stream = nullptr);
    virtual void print(bool print_data = false);
};

} // namespace dl
