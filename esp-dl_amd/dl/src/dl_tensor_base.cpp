#include "dl_tensor_base.hpp"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>
#include <cstring>

#include "espdl_hip.h"

namespace dl {

const char *quant_type_to_string(quant_type_t type)
{
    switch (type) {
    case QUANT_TYPE_FLOAT32:
        return "QUANT_TYPE_FLOAT32";
    case QUANT_TYPE_SYMM_8BIT:
        return "QUANT_TYPE_SYMM_8BIT";
    case QUANT_TYPE_SYMM_16BIT:
        return "QUANT_TYPE_SYMM_16BIT";
    case QUANT_TYPE_SYMM_32BIT:
        return "QUANT_TYPE_SYMM_32BIT";
    default:
        return "QUANT_TYPE_NONE";
    }
}

const char *activation_type_to_string(activation_type_t type)
{
    switch (type) {
    case Linear:
        return "Linear";
    case ReLU:
        return "ReLU";
    case LeakyReLU:
        return "LeakyReLU";
    case PReLU:
        return "PReLU";
    }
    return "Undefined";
}

size_t dtype_sizeof(dtype_t dtype)
{
    switch (dtype) {
    case DATA_TYPE_FLOAT:
    case DATA_TYPE_INT32:
    case DATA_TYPE_UINT32:
        return 4;
    case DATA_TYPE_INT8:
    case DATA_TYPE_UINT8:
    case DATA_TYPE_BOOL:
        return 1;
    case DATA_TYPE_INT16:
    case DATA_TYPE_UINT16:
    case DATA_TYPE_FLOAT16:
        return 2;
    case DATA_TYPE_INT64:
    case DATA_TYPE_UINT64:
    case DATA_TYPE_DOUBLE:
        return 8;
    default:
        return 0;
    }
}

const char *dtype_to_string(dtype_t dtype)
{
    static const char *names[] = {"undefined", "float", "uint8", "int8",    "uint16", "int16",  "int32",
                                  "int64",     "string", "bool", "float16", "double", "uint32", "uint64"};
    return (dtype >= 0 && dtype <= DATA_TYPE_UINT64) ? names[dtype] : "undefined";
}

std::string vector_to_string(const std::vector<int> &shape)
{
    std::string s = "[";
    for (size_t i = 0; i < shape.size(); i++) {
        s += std::to_string(shape[i]);
        if (i + 1 != shape.size())
            s += ", ";
    }
    return s + "]";
}

namespace {

int64_t shape_size(const std::vector<int> &shape)
{
    int64_t n = 1;
    for (int d : shape)
        n *= d;
    return n;
}

bool hip_ok(hipError_t e, const char *what)
{
    if (e != hipSuccess) {
        DL_LOGE("TensorBase", "%s failed: %s", what, hipGetErrorString(e));
        return false;
    }
    return true;
}

void *alloc_bytes(size_t bytes, uint32_t caps)
{
    if (bytes == 0)
        bytes = 16;
    if (caps & MALLOC_CAP_DEVICE) {
        void *p = nullptr;
        return hip_ok(hipMalloc(&p, bytes), "hipMalloc") ? p : nullptr;
    }
    void *p = nullptr;
    if (posix_memalign(&p, 64, (bytes + 63) & ~(size_t)63) != 0)
        return nullptr;
    return p;
}

void free_bytes(void *p, uint32_t caps)
{
    if (!p)
        return;
    if (caps & MALLOC_CAP_DEVICE)
        (void)hipFree(p);
    else
        free(p);
}

// tool::round of the portable build (esp-dl/dl/tool/src/dl_tool.cpp:72-75)
inline int round_half_up(float v)
{
    return (int)floorf((float)((double)v + 0.5));
}

// quantize(dequantize(x)) of the reference (esp-dl/dl/tensor/src/dl_tensor_base.cpp:18-42, 362-392)
template <typename DT, typename ST>
void requantize_host(DT *dst, const ST *src, int64_t n, int dst_exp, int src_exp)
{
    const float src_scale = DL_SCALE(src_exp);
    const float inv_scale = (float)(1.0 / (double)(DL_SCALE(dst_exp)));
    const int lo = sizeof(DT) == 1 ? DL_QUANT8_MIN : DL_QUANT16_MIN;
    const int hi = sizeof(DT) == 1 ? DL_QUANT8_MAX : DL_QUANT16_MAX;
    for (int64_t i = 0; i < n; i++) {
        const float tmp = (float)src[i] * src_scale;
        const int q = round_half_up(tmp * inv_scale);
        dst[i] = (DT)DL_CLIP(q, lo, hi);
    }
}

} // namespace

TensorBase::TensorBase(std::vector<int> shape, const void *element, int exponent, dtype_t dtype, bool deep,
                       uint32_t caps) :
    size(shape_size(shape)), shape(shape), dtype(dtype), exponent(exponent), auto_free(deep), data(nullptr), caps(caps)
{
    if (deep) {
        data = alloc_bytes(get_bytes(), caps);
        if (data) {
            if (element)
                copy_from_host(element, get_bytes());
            else
                this->memset(0);
        }
    } else {
        data = const_cast<void *>(element);
    }
}

TensorBase::TensorBase(std::vector<int> shape, const void *element, const std::vector<int> &exponents, dtype_t dtype,
                       bool deep, uint32_t caps) :
    TensorBase(shape, element, 0, dtype, deep, caps)
{
    exponent = ExponentInfo(exponents);
}

TensorBase::~TensorBase()
{
    if (auto_free) {
        free_bytes(data, caps);
        data = nullptr;
    }
}

TensorBase &TensorBase::set_shape(const std::vector<int> &new_shape)
{
    if (shape_size(new_shape) != size) {
        DL_LOGE("TensorBase", "set_shape: %s does not hold %lld elements", vector_to_string(new_shape).c_str(),
                (long long)size);
        return *this;
    }
    shape = new_shape;
    return *this;
}

namespace {
// rows of a tensor (positions of all axes but the last) and the bytes of one row / between rows
struct RowView {
    size_t rows, row_bytes, pitch_bytes;
};
RowView row_view(const TensorBase *t)
{
    const size_t e = t->get_dtype_bytes();
    const size_t c = t->shape.empty() ? 1 : (size_t)t->shape.back();
    return {c ? (size_t)t->size / c : 0, c * e, (size_t)t->get_channel_pitch() * e};
}
} // namespace

bool TensorBase::copy_from_host(const void *host, size_t bytes, void *stream)
{
    if (!data || !host || bytes > get_bytes())
        return false;
    if (!is_dense()) {
        // a channel slice of a wider device tensor: whole tensors only, row by row
        const RowView v = row_view(this);
        if (!on_device() || bytes != get_bytes())
            return false;
        hipStream_t s2 = static_cast<hipStream_t>(stream);
        return hip_ok(hipMemcpy2DAsync(data, v.pitch_bytes, host, v.row_bytes, v.row_bytes, v.rows, hipMemcpyHostToDevice, s2),
                      "hipMemcpy2DAsync H2D") &&
            hip_ok(hipStreamSynchronize(s2), "hipStreamSynchronize");
    }
    if (!on_device()) {
        memcpy(data, host, bytes);
        return true;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    return hip_ok(hipMemcpyAsync(data, host, bytes, hipMemcpyHostToDevice, s), "hipMemcpyAsync H2D") &&
        hip_ok(hipStreamSynchronize(s), "hipStreamSynchronize");
}

bool TensorBase::copy_to_host(void *host, size_t bytes, void *stream) const
{
    if (!data || !host || bytes > get_bytes())
        return false;
    if (!is_dense()) {
        const RowView v = row_view(this);
        if (!on_device() || bytes != get_bytes())
            return false;
        hipStream_t s2 = static_cast<hipStream_t>(stream);
        return hip_ok(hipMemcpy2DAsync(host, v.row_bytes, data, v.pitch_bytes, v.row_bytes, v.rows, hipMemcpyDeviceToHost, s2),
                      "hipMemcpy2DAsync D2H") &&
            hip_ok(hipStreamSynchronize(s2), "hipStreamSynchronize");
    }
    if (!on_device()) {
        memcpy(host, data, bytes);
        return true;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    return hip_ok(hipMemcpyAsync(host, data, bytes, hipMemcpyDeviceToHost, s), "hipMemcpyAsync D2H") &&
        hip_ok(hipStreamSynchronize(s), "hipStreamSynchronize");
}

bool TensorBase::copy_from(const TensorBase *tensor, void *stream)
{
    if (!tensor || tensor->get_bytes() != get_bytes())
        return false;
    if (!tensor->on_device())
        return copy_from_host(tensor->data, get_bytes(), stream);
    if (!on_device())
        return tensor->copy_to_host(data, get_bytes(), stream);
    if (!is_dense() || !tensor->is_dense()) {
        const RowView d = row_view(this), v = row_view(tensor);
        if (d.row_bytes != v.row_bytes)
            return false;
        return espdl_hip_copy_rows(tensor->data, (int64_t)v.pitch_bytes, data, (int64_t)d.pitch_bytes, (int64_t)v.row_bytes,
                                   (int64_t)v.rows, stream) == ESPDL_HIP_OK;
    }
    return hip_ok(hipMemcpyAsync(data, tensor->data, get_bytes(), hipMemcpyDeviceToDevice,
                                 static_cast<hipStream_t>(stream)),
                  "hipMemcpyAsync D2D");
}

TensorBase *TensorBase::to_device(void *stream) const
{
    TensorBase *t = new TensorBase(shape, nullptr, 0, dtype, true, MALLOC_CAP_DEVICE);
    t->exponent = exponent;
    t->copy_from(this, stream);
    return t;
}

TensorBase *TensorBase::to_host(void *stream) const
{
    TensorBase *t = new TensorBase(shape, nullptr, 0, dtype, true, MALLOC_CAP_HOST);
    t->exponent = exponent;
    t->copy_from(this, stream);
    if (on_device())
        (void)hipStreamSynchronize(static_cast<hipStream_t>(stream));
    return t;
}

void TensorBase::memset(int value, void *stream)
{
    if (!data)
        return;
    if (on_device()) {
        hipStream_t s = static_cast<hipStream_t>(stream);
        if (!is_dense()) {
            const RowView v = row_view(this);
            (void)hip_ok(hipMemset2DAsync(data, v.pitch_bytes, value, v.row_bytes, v.rows, s), "hipMemset2DAsync");
            (void)hipStreamSynchronize(s);
            return;
        }
        (void)hip_ok(hipMemsetAsync(data, value, get_bytes(), s), "hipMemsetAsync");
        (void)hipStreamSynchronize(s);
    } else {
        ::memset(data, value, get_bytes());
    }
}

bool TensorBase::assign(TensorBase *tensor, void *stream)
{
    if (tensor == nullptr || get_size() != tensor->get_size())
        return false;
    const bool per_channel = exponent.is_per_channel() || tensor->exponent.is_per_channel();
    if (exponent == tensor->exponent && dtype == tensor->dtype)
        return copy_from(tensor, stream);
    if (!is_dense() || !tensor->is_dense()) {
        // channel slices of wider device tensors: int8 -> int8 row by row; anything else from a dense copy
        if (dtype == DATA_TYPE_INT8 && tensor->dtype == DATA_TYPE_INT8 && on_device() && tensor->on_device() && !per_channel) {
            const RowView d = row_view(this), v = row_view(tensor);
            return espdl_hip_requantize_s8_rows(static_cast<const int8_t *>(tensor->data), (int64_t)v.pitch_bytes,
                                                static_cast<int8_t *>(data), (int64_t)d.pitch_bytes, (int64_t)v.row_bytes,
                                                (int64_t)v.rows, tensor->exponent, exponent, stream) == ESPDL_HIP_OK;
        }
        if (!is_dense()) {
            DL_LOGE("TensorBase::assign", "only int8 device tensors can be requantized into a channel slice");
            return false;
        }
        TensorBase dense(tensor->shape, nullptr, 0, tensor->dtype, true, tensor->caps);
        dense.exponent = tensor->exponent;
        return dense.copy_from(tensor, stream) && assign(&dense, stream);
    }
    const bool ints = (dtype == DATA_TYPE_INT8 || dtype == DATA_TYPE_INT16) &&
        (tensor->dtype == DATA_TYPE_INT8 || tensor->dtype == DATA_TYPE_INT16);
    // float32 <-> quantized on the device (QuantizeLinear / DequantizeLinear,
    // esp-dl/dl/tensor/src/dl_tensor_base.cpp:251-268 and :286-299)
    if (on_device() && tensor->on_device()) {
        if (tensor->dtype == DATA_TYPE_FLOAT && (dtype == DATA_TYPE_INT8 || dtype == DATA_TYPE_INT16))
            return espdl_hip_quantize_f32(static_cast<const float *>(tensor->data), size, exponent,
                                          dtype == DATA_TYPE_INT8 ? 1 : 2, data, stream) == ESPDL_HIP_OK;
        if (dtype == DATA_TYPE_FLOAT && (tensor->dtype == DATA_TYPE_INT8 || tensor->dtype == DATA_TYPE_INT16))
            return espdl_hip_dequantize_f32(tensor->data, size, tensor->exponent, tensor->dtype == DATA_TYPE_INT8 ? 1 : 2,
                                            static_cast<float *>(data), stream) == ESPDL_HIP_OK;
    }
    if (!ints) {
        DL_LOGE("TensorBase::assign", "unsupported conversion %s -> %s", dtype_to_string(tensor->dtype),
                dtype_to_string(dtype));
        return false;
    }
    // device -> device: the requantize kernel
    if (on_device() && tensor->on_device()) {
        return espdl_hip_requantize(tensor->data, tensor->dtype == DATA_TYPE_INT16 ? ESPDL_HIP_S16 : ESPDL_HIP_S8, size,
                                    tensor->exponent, exponent, data,
                                    dtype == DATA_TYPE_INT16 ? ESPDL_HIP_S16 : ESPDL_HIP_S8, stream) == ESPDL_HIP_OK;
    }
    // everything else goes through host memory
    TensorBase *src_host = tensor->on_device() ? tensor->to_host(stream) : tensor;
    std::vector<uint8_t> staging;
    void *dst_ptr = data;
    if (on_device()) {
        staging.resize(get_bytes());
        dst_ptr = staging.data();
    }
    const int de = exponent, se = tensor->exponent;
    if (de == se) {
        // same exponent, different width: widen, or saturate (dl_tensor_base.cpp:321-336)
        if (dtype == DATA_TYPE_INT8) {
            const int16_t *s = static_cast<const int16_t *>(src_host->data);
            int8_t *d = static_cast<int8_t *>(dst_ptr);
            for (int64_t i = 0; i < size; i++)
                d[i] = (int8_t)DL_CLIP(s[i], DL_QUANT8_MIN, DL_QUANT8_MAX);
        } else {
            const int8_t *s = static_cast<const int8_t *>(src_host->data);
            int16_t *d = static_cast<int16_t *>(dst_ptr);
            for (int64_t i = 0; i < size; i++)
                d[i] = (int16_t)s[i];
        }
    } else if (dtype == DATA_TYPE_INT8 && tensor->dtype == DATA_TYPE_INT8) {
        requantize_host(static_cast<int8_t *>(dst_ptr), static_cast<const int8_t *>(src_host->data), size, de, se);
    } else if (dtype == DATA_TYPE_INT16 && tensor->dtype == DATA_TYPE_INT16) {
        requantize_host(static_cast<int16_t *>(dst_ptr), static_cast<const int16_t *>(src_host->data), size, de, se);
    } else if (dtype == DATA_TYPE_INT8) {
        requantize_host(static_cast<int8_t *>(dst_ptr), static_cast<const int16_t *>(src_host->data), size, de, se);
    } else {
        requantize_host(static_cast<int16_t *>(dst_ptr), static_cast<const int8_t *>(src_host->data), size, de, se);
    }
    if (src_host != tensor)
        delete src_host;
    if (on_device())
        return copy_from_host(staging.data(), get_bytes(), stream);
    return true;
}

template <typename T>
T TensorBase::get_element(int64_t index)
{
    return static_cast<T *>(data)[index];
}
template int8_t TensorBase::get_element<int8_t>(int64_t);
template int16_t TensorBase::get_element<int16_t>(int64_t);
template int32_t TensorBase::get_element<int32_t>(int64_t);
template int64_t TensorBase::get_element<int64_t>(int64_t);
template float TensorBase::get_element<float>(int64_t);

bool TensorBase::equal(TensorBase *tensor, float epsilon, bool verbose)
{
    if (!tensor || tensor->dtype != dtype || tensor->size != size) {
        if (verbose)
            DL_LOGE("TensorBase::equal", "dtype or size differ");
        return false;
    }
    TensorBase *a = on_device() ? to_host() : this;
    TensorBase *b = tensor->on_device() ? tensor->to_host() : tensor;
    bool same = true;
    auto cmp = [&](auto *pa, auto *pb) {
        for (int64_t i = 0; i < size && same; i++) {
            const double d = std::fabs((double)pa[i] - (double)pb[i]);
            if (d > epsilon) {
                same = false;
                if (verbose)
                    DL_LOGE("TensorBase::equal", "element %lld: %g vs %g", (long long)i, (double)pa[i], (double)pb[i]);
            }
        }
    };
    switch (dtype) {
    case DATA_TYPE_INT8:
        cmp(static_cast<int8_t *>(a->data), static_cast<int8_t *>(b->data));
        break;
    case DATA_TYPE_INT16:
        cmp(static_cast<int16_t *>(a->data), static_cast<int16_t *>(b->data));
        break;
    case DATA_TYPE_INT32:
        cmp(static_cast<int32_t *>(a->data), static_cast<int32_t *>(b->data));
        break;
    case DATA_TYPE_INT64:
        cmp(static_cast<int64_t *>(a->data), static_cast<int64_t *>(b->data));
        break;
    case DATA_TYPE_FLOAT:
        cmp(static_cast<float *>(a->data), static_cast<float *>(b->data));
        break;
    default:
        same = memcmp(a->data, b->data, get_bytes()) == 0;
    }
    if (a != this)
        delete a;
    if (b != tensor)
        delete b;
    return same;
}

void TensorBase::print(bool print_data)
{
    std::printf("TensorBase shape %s dtype %s exponent %d%s %s\n", vector_to_string(shape).c_str(),
                dtype_to_string(dtype), (int)exponent, exponent.is_per_channel() ? " (per-channel)" : "",
                on_device() ? "device" : "host");
    if (print_data && !on_device() && dtype == DATA_TYPE_INT8) {
        const int8_t *p = static_cast<const int8_t *>(data);
        for (int64_t i = 0; i < size && i < 64; i++)
            std::printf("%d ", p[i]);
        std::printf("\n");
    }
}

} // namespace dl
