// Data-movement and pooling operator objects: Concat, Split, Transpose, Resize, MaxPool, AveragePool,
// Slice, ReduceMean.  Each mirrors the
// reference module of the same name (same attributes, shape rules and error behaviour) and enqueues
// kernels of include/espdl_hip.h on the context's stream.
//   Concat     esp-dl/dl/module/include/dl_module_concat.hpp:14-127
//   Split      esp-dl/dl/module/include/dl_module_split.hpp:14-177
//   Transpose  esp-dl/dl/module/include/dl_module_transpose.hpp:12-88
//   Resize     esp-dl/dl/module/include/dl_module_resize.hpp:14-180 (nearest mode)
//   MaxPool    esp-dl/dl/module/include/dl_module_max_pool.hpp:13-131
//   AveragePool esp-dl/dl/module/include/dl_module_average_pool.hpp
//   Slice      esp-dl/dl/module/include/dl_module_slice.hpp
//   ReduceMean esp-dl/dl/module/include/dl_module_reduce_mean.hpp, dl_module_reduce_base.hpp
#pragma once

#include <algorithm>
#include <cassert>
#include <cstring>

#include "dl_module_base.hpp"
#include "dl_module_elementwise.hpp"
#include "espdl_hip.h"

namespace dl {
namespace module {

class Concat : public Module {
private:
    int m_axis;

public:
    Concat(const char *name = nullptr, int axis = 0, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_axis(axis)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        assert(!input_shapes.empty());
        const int dims = (int)input_shapes[0].size();
        if (m_axis < 0)
            m_axis += dims;
        assert(m_axis >= 0 && m_axis < dims);
        std::vector<int> out = input_shapes[0];
        out[m_axis] = 0;
        for (auto &s : input_shapes) {
            assert((int)s.size() == dims);
            out[m_axis] += s[m_axis];
        }
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!output || !output->on_device()) {
            DL_LOGE("Concat", "%s: needs device tensors", name.c_str());
            return;
        }
        const size_t esize = output->get_dtype_bytes();
        std::vector<const void *> ptrs;
        std::vector<int64_t> bytes;
        int64_t loop_times = 1;
        bool sliced = false; // an input is a channel slice (possibly of the output itself)
        for (size_t j = 0; j < m_inputs_index.size(); j++) {
            TensorBase *input = context->get_tensor(m_inputs_index[j]);
            if (!input || !input->on_device() || input->dtype != output->dtype) {
                DL_LOGE("Concat", "%s: input %d is missing, on the host or of another type", name.c_str(), (int)j);
                return;
            }
            int64_t n = 1;
            for (int i = m_axis; i < (int)input->shape.size(); i++)
                n *= input->shape[i];
            if (j == 0)
                for (int i = 0; i < m_axis; i++)
                    loop_times *= input->shape[i];
            ptrs.push_back(input->data);
            bytes.push_back(n * (int64_t)esize);
            sliced = sliced || !input->is_dense();
        }
        if (sliced) {
            // along the last axis only (the model makes no other slices): inputs that already lie in their
            // place inside the output were written there by their producers; the others are copied row by row
            if (m_axis != (int)output->shape.size() - 1 || !output->is_dense()) {
                DL_LOGE("Concat", "%s: channel slices along another axis than the last", name.c_str());
                return;
            }
            const int64_t out_row = (int64_t)output->shape.back() * (int64_t)esize;
            int64_t at = 0;
            for (size_t j = 0; j < ptrs.size(); j++) {
                TensorBase *input = context->get_tensor(m_inputs_index[j]);
                char *dst = static_cast<char *>(output->data) + at;
                at += bytes[j];
                if (ptrs[j] == dst && (int64_t)input->get_channel_pitch() * (int64_t)esize == out_row)
                    continue;
                const int rc = espdl_hip_copy_rows(ptrs[j], (int64_t)input->get_channel_pitch() * (int64_t)esize, dst, out_row,
                                                   bytes[j], loop_times, context->stream);
                if (rc != ESPDL_HIP_OK)
                    DL_LOGE("Concat", "%s: %s", name.c_str(), espdl_hip_last_error());
            }
            return;
        }
        const int rc =
            espdl_hip_concat((int32_t)ptrs.size(), ptrs.data(), bytes.data(), loop_times, output->data, context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Concat", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    int get_axis() const { return m_axis; }
    bool reads_channel_slice(int slot) const
    {
        (void)slot;
        return true; // along the last axis, which is the only one a model slices
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        int axis = 0;
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "axis", axis);
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        return new Concat(node_name.c_str(), axis, quant_type);
    }
    void print() { DL_LOGI("Concat", "axis: %d, quant_type: %s.", m_axis, quant_type_to_string(quant_type)); }
};

/// With a `split` parameter the outputs take those extents.  Without one the reference makes
/// ceil(extent / num_outputs) outputs of num_outputs elements each (the last one takes the rest):
/// the attribute acts as the piece size there, and this class does the same.
class Split : public Module {
private:
    std::vector<int64_t> m_split;
    int m_axis;
    int m_num_outputs;

public:
    Split(const std::vector<int64_t> &split = {}, int axis = 0, int num_outputs = -1, const char *name = nullptr,
          quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_split(split), m_axis(axis), m_num_outputs(num_outputs)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        assert(!input_shapes[0].empty());
        if (m_axis < 0)
            m_axis += (int)input_shapes[0].size();
        const int extent = input_shapes[0][m_axis];
        std::vector<std::vector<int>> out;
        if (!m_split.empty()) {
            int64_t total = 0;
            for (int64_t s : m_split) {
                out.push_back(input_shapes[0]);
                out.back()[m_axis] = (int)s;
                total += s;
            }
            assert(total == extent);
            (void)total;
        } else {
            assert(m_num_outputs > 0);
            const int n = (extent + m_num_outputs - 1) / m_num_outputs;
            for (int i = 0; i < n; i++) {
                out.push_back(input_shapes[0]);
                out.back()[m_axis] = i + 1 < n ? m_num_outputs : extent - (n - 1) * m_num_outputs;
            }
        }
        return out;
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        if (!input || !input->on_device() || input->shape.empty()) {
            DL_LOGE("Split", "%s: needs a device tensor of at least one dim", name.c_str());
            return;
        }
        int64_t num_slices = 1, slice_size = 1;
        for (int i = 0; i < m_axis; i++)
            num_slices *= input->shape[i];
        for (int i = m_axis + 1; i < (int)input->shape.size(); i++)
            slice_size *= input->shape[i];
        const int64_t esize = (int64_t)input->get_dtype_bytes();
        const int64_t in_axis = input->shape[m_axis];
        if (!input->is_dense() && m_axis != (int)input->shape.size() - 1) {
            DL_LOGE("Split", "%s: the input is a channel slice and the axis is not the last", name.c_str());
            return;
        }
        // bytes between consecutive runs of the input (a channel slice of a wider tensor has a larger pitch)
        const int64_t in_pitch = input->is_dense() ? slice_size * in_axis * esize : (int64_t)input->channel_pitch * esize;
        int64_t slice_index = 0;
        std::vector<void *> dsts;
        std::vector<int64_t> bytes;
        bool any = false;
        for (size_t i = 0; i < m_outputs_index.size(); i++) {
            TensorBase *output = context->get_tensor(m_outputs_index[i]);
            if (!output || !output->on_device() || output->dtype != input->dtype) {
                DL_LOGE("Split", "%s: output %d is missing, on the host or of another type", name.c_str(), (int)i);
                return;
            }
            const int64_t out_axis = output->shape[m_axis];
            const char *src = static_cast<const char *>(input->data) + slice_index * slice_size * esize;
            slice_index += out_axis;
            bytes.push_back(slice_size * out_axis * esize);
            // an output the model left inside the input is already there
            if (output->data == src && !output->is_dense() && (int64_t)output->channel_pitch * esize == in_pitch) {
                dsts.push_back(nullptr);
                continue;
            }
            if (!output->is_dense()) {
                DL_LOGE("Split", "%s: output %d is a channel slice of another tensor than the input", name.c_str(), (int)i);
                return;
            }
            dsts.push_back(output->data);
            any = true;
        }
        if (!any)
            return;
        const int rc = espdl_hip_split(input->data, in_pitch, (int32_t)dsts.size(), dsts.data(), bytes.data(), num_slices,
                                       context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Split", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    int get_axis() const { return m_axis; }
    bool reads_channel_slice(int slot) const { return slot == 0; }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        int axis = 0, num_outputs = -1;
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "axis", axis);
        fbs_model->get_operation_attribute(node_name, "num_outputs", num_outputs);
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        std::vector<int64_t> split;
        TensorBase *t = fbs_model->get_operation_parameter(node_name, 1);
        if (t) {
            if (t->dtype == DATA_TYPE_INT64) {
                const int64_t *p = t->get_element_ptr<int64_t>();
                split.assign(p, p + t->get_size());
            } else if (t->dtype == DATA_TYPE_INT32) {
                const int32_t *p = t->get_element_ptr<int32_t>();
                split.assign(p, p + t->get_size());
            }
            delete t;
        }
        return new Split(split, axis, num_outputs, node_name.c_str(), quant_type);
    }
    void print()
    {
        DL_LOGI("Split", "axis: %d, pieces: %d, quant_type: %s.", m_axis, (int)m_split.size(),
                quant_type_to_string(quant_type));
    }
};

class Transpose : public Module {
private:
    std::vector<int> m_perm;

public:
    Transpose(const char *name = nullptr, quant_type_t quant_type = QUANT_TYPE_NONE, std::vector<int> perm = {}) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_perm(perm)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const int dims = (int)input_shapes[0].size();
        assert((int)m_perm.size() == dims || m_perm.empty());
        if (m_perm.empty())
            for (int i = dims - 1; i >= 0; i--)
                m_perm.push_back(i);
        std::vector<int> out;
        for (int i = 0; i < dims; i++) {
            if (m_perm[i] < 0)
                m_perm[i] += dims;
            out.push_back(input_shapes[0][m_perm[i]]);
        }
        // a permutation that keeps the axes longer than 1 in their order moves no byte (the [N, 1, 1, C] -> [N, C, 1, 1]
        // in front of an exported classifier): the output is then a view of the input, as with Reshape
        int last = -1;
        bool view = true;
        for (int i = 0; i < dims; i++)
            if (input_shapes[0][m_perm[i]] > 1) {
                view = view && m_perm[i] > last;
                last = m_perm[i];
            }
        inplace = view ? MODULE_INPLACE_UNCHANGED_BUFFER : MODULE_NON_INPLACE;
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!on_device_all({input, output}) || input->dtype != output->dtype) {
            DL_LOGE("Transpose", "%s: needs device tensors of one type", name.c_str());
            return;
        }
        if (inplace == MODULE_INPLACE_UNCHANGED_BUFFER && input->data == output->data)
            return; // a view
        const int rc = espdl_hip_transpose(input->data, input->shape.data(), (int32_t)input->shape.size(), m_perm.data(),
                                           (int32_t)m_perm.size(), (int32_t)input->get_dtype_bytes(), output->data,
                                           context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Transpose", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        std::vector<int> perm;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "perm", perm);
        return new Transpose(node_name.c_str(), quant_type, perm);
    }
    void print() { DL_LOGI("Transpose", "dims: %d, quant_type: %s.", (int)m_perm.size(), quant_type_to_string(quant_type)); }
};

/// Nearest mode on int8 NHWC / NWC tensors.  Scales and sizes are in the exporter's NCHW order
/// (scales[2] = height, scales[3] = width), as in the reference.
class Resize : public Module {
private:
    std::string m_mode;
    std::vector<float> m_scales;
    std::vector<int64_t> m_sizes;

public:
    Resize(const char *name = nullptr, const std::string &mode = "nearest", const std::vector<float> &scales = {},
           const std::vector<int64_t> &sizes = {}, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_mode(mode), m_scales(scales), m_sizes(sizes)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        assert(in.size() == 3 || in.size() == 4);
        std::vector<int> out = in;
        if (!m_sizes.empty()) {
            std::vector<float> scales(in.size(), 1.0f);
            out[1] = (int)m_sizes[2];
            scales[2] = out[1] / (float)in[1];
            if (in.size() == 4) {
                out[2] = (int)m_sizes[3];
                scales[3] = out[2] / (float)in[2];
            }
            m_scales.swap(scales);
        } else {
            assert(m_scales.size() == in.size());
            out[1] = (int)(in[1] * m_scales[2]);
            if (in.size() == 4)
                out[2] = (int)(in[2] * m_scales[3]);
        }
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (quant_type != QUANT_TYPE_SYMM_8BIT || !on_device_all({input, output}) || m_mode != "nearest") {
            DL_LOGE("Resize", "%s: this build resizes int8 device tensors in nearest mode only", name.c_str());
            return;
        }
        const bool nwc = input->shape.size() == 3;
        // NWC runs as one row: height 1, height scale 1 (esp-dl/dl/base/dl_base_resize.hpp:39-51)
        const int h = nwc ? 1 : input->shape[1], w = nwc ? input->shape[1] : input->shape[2];
        const int c = nwc ? input->shape[2] : input->shape[3];
        const int oh = nwc ? 1 : output->shape[1], ow = nwc ? output->shape[1] : output->shape[2];
        const float sh = nwc ? 1.0f : m_scales[2], sw = nwc ? m_scales[2] : m_scales[3];
        const int rc = espdl_hip_resize_nearest_s8_pitched(
            static_cast<const int8_t *>(input->data), input->shape[0], h, w, c, oh, ow, sh, sw, input->exponent.get(),
            output->exponent.get(), input->is_dense() ? 0 : input->channel_pitch,
            output->is_dense() ? 0 : output->channel_pitch, static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Resize", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    /// The kernel takes a channel pitch on either side (an upsampled tensor is written into the Concat behind it).
    bool reads_channel_slice(int slot) const { return slot == 0 && quant_type == QUANT_TYPE_SYMM_8BIT; }
    bool writes_channel_slice(int slot) const { return slot == 0 && quant_type == QUANT_TYPE_SYMM_8BIT; }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        std::string mode = "nearest";
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "mode", mode);
        std::vector<float> scales;
        TensorBase *st = fbs_model->get_operation_parameter(node_name, 2);
        if (st && st->dtype == DATA_TYPE_FLOAT) {
            const float *p = st->get_element_ptr<float>();
            scales.assign(p, p + st->get_size());
        }
        delete st;
        std::vector<int64_t> sizes;
        TensorBase *zt = fbs_model->get_operation_parameter(node_name, 3);
        if (zt && zt->dtype == DATA_TYPE_INT64) {
            const int64_t *p = zt->get_element_ptr<int64_t>();
            sizes.assign(p, p + zt->get_size());
        }
        delete zt;
        if (quant_type != QUANT_TYPE_SYMM_8BIT && quant_type != QUANT_TYPE_SYMM_16BIT)
            return nullptr;
        return new Resize(node_name.c_str(), mode, scales, sizes, quant_type);
    }
    void print() { DL_LOGI("Resize", "mode: %s, quant_type: %s.", m_mode.c_str(), quant_type_to_string(quant_type)); }
};

class MaxPool : public Module {
private:
    std::vector<int> m_filter_shape;
    std::vector<int> m_padding; ///< [top, bottom, left, right] (NWC: [head, tail])
    std::vector<int> m_strides;

public:
    MaxPool(const char *name = nullptr, const std::vector<int> &filter_shape = {2, 2},
            const std::vector<int> &padding = {0, 0, 0, 0}, const std::vector<int> &strides = {1, 1},
            quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_filter_shape(filter_shape), m_padding(padding), m_strides(strides)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        assert(in.size() == 3 || in.size() == 4);
        std::vector<int> out = in;
        out[1] = (in[1] + m_padding[0] + m_padding[1] - m_filter_shape[0]) / m_strides[0] + 1;
        if (in.size() == 4)
            out[2] = (in[2] + m_padding[2] + m_padding[3] - m_filter_shape[1]) / m_strides[1] + 1;
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!on_device_all({input, output}) ||
            (quant_type != QUANT_TYPE_SYMM_8BIT && quant_type != QUANT_TYPE_SYMM_16BIT)) {
            DL_LOGE("MaxPool", "%s: needs int8 / int16 device tensors", name.c_str());
            return;
        }
        const bool nwc = input->shape.size() == 3;
        const int h = nwc ? 1 : input->shape[1], w = nwc ? input->shape[1] : input->shape[2];
        const int c = nwc ? input->shape[2] : input->shape[3];
        const int kh = nwc ? 1 : m_filter_shape[0], kw = nwc ? m_filter_shape[0] : m_filter_shape[1];
        const int sh = nwc ? 1 : m_strides[0], sw = nwc ? m_strides[0] : m_strides[1];
        const int pt = nwc ? 0 : m_padding[0], pb = nwc ? 0 : m_padding[1];
        const int pl = nwc ? m_padding[0] : m_padding[2], pr = nwc ? m_padding[1] : m_padding[3];
        const int rc =
            espdl_hip_max_pool_pitched(input->data, quant_type == QUANT_TYPE_SYMM_8BIT ? ESPDL_HIP_S8 : ESPDL_HIP_S16,
                                       input->shape[0], h, w, c, kh, kw, sh, sw, pt, pb, pl, pr,
                                       input->is_dense() ? 0 : input->channel_pitch,
                                       output->is_dense() ? 0 : output->channel_pitch, output->data, context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("MaxPool", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    /// The kernels take a channel pitch on either side (the pools of an SPPF block write into its Concat).
    bool reads_channel_slice(int slot) const { return slot == 0; }
    bool writes_channel_slice(int slot) const { return slot == 0; }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        std::vector<int> kernel_shape, pads, strides;
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "kernel_shape", kernel_shape);
        fbs_model->get_operation_attribute(node_name, "pads", pads);
        fbs_model->get_operation_attribute(node_name, "strides", strides);
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        if (quant_type != QUANT_TYPE_SYMM_8BIT && quant_type != QUANT_TYPE_SYMM_16BIT)
            return nullptr;
        if (kernel_shape.empty())
            return nullptr;
        if (pads.size() == 4) // ONNX [top, left, bottom, right] -> [top, bottom, left, right]
            pads = {pads[0], pads[2], pads[1], pads[3]};
        else if (pads.empty())
            pads = {0, 0, 0, 0};
        if (strides.empty())
            strides.assign(kernel_shape.size(), 1);
        return new MaxPool(node_name.c_str(), kernel_shape, pads, strides, quant_type);
    }
    void print()
    {
        DL_LOGI("MaxPool", "kernel: %dx%d, quant_type: %s.", m_filter_shape[0], m_filter_shape.size() > 1 ? m_filter_shape[1] : 1,
                quant_type_to_string(quant_type));
    }
};

/// AveragePool on int8 NHWC / NWC tensors, portable C path arithmetic
/// (esp-dl/dl/module/include/dl_module_average_pool.hpp; attributes as MaxPool; `ceil_mode` and
/// `count_include_pad` are read by neither the reference's shape rule nor its C kernel).
class AveragePool : public Module {
private:
    std::vector<int> m_kernel_shape, m_pads, m_strides;

public:
    AveragePool(const char *name = nullptr, const std::vector<int> &kernel_shape = {2, 2},
                const std::vector<int> &pads = {0, 0, 0, 0}, const std::vector<int> &strides = {1, 1},
                quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_kernel_shape(kernel_shape), m_pads(pads), m_strides(strides)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        assert(in.size() == 3 || in.size() == 4);
        std::vector<int> out = in;
        out[1] = (in[1] + m_pads[0] + m_pads[1] - m_kernel_shape[0]) / m_strides[0] + 1;
        if (in.size() == 4)
            out[2] = (in[2] + m_pads[2] + m_pads[3] - m_kernel_shape[1]) / m_strides[1] + 1;
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!on_device_all({input, output}) || (quant_type != QUANT_TYPE_SYMM_8BIT && quant_type != QUANT_TYPE_SYMM_16BIT)) {
            DL_LOGE("AveragePool", "%s: needs int8 or int16 device tensors", name.c_str());
            return;
        }
        const bool nwc = input->shape.size() == 3;
        const int h = nwc ? 1 : input->shape[1], w = nwc ? input->shape[1] : input->shape[2];
        const int c = nwc ? input->shape[2] : input->shape[3];
        const int kh = nwc ? 1 : m_kernel_shape[0], kw = nwc ? m_kernel_shape[0] : m_kernel_shape[1];
        const int sh = nwc ? 1 : m_strides[0], sw = nwc ? m_strides[0] : m_strides[1];
        const int pt = nwc ? 0 : m_pads[0], pb = nwc ? 0 : m_pads[1];
        const int pl = nwc ? m_pads[0] : m_pads[2], pr = nwc ? m_pads[1] : m_pads[3];
        const int rc = quant_type == QUANT_TYPE_SYMM_16BIT
            ? espdl_hip_avg_pool_s16(static_cast<const int16_t *>(input->data), input->shape[0], h, w, c, kh, kw, sh, sw, pt,
                                     pb, pl, pr, input->exponent.get(), output->exponent.get(),
                                     static_cast<int16_t *>(output->data), context->stream)
            : espdl_hip_avg_pool_s8(static_cast<const int8_t *>(input->data), input->shape[0], h, w, c, kh, kw, sh, sw, pt,
                                    pb, pl, pr, input->exponent.get(), output->exponent.get(),
                                    static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("AveragePool", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        std::vector<int> kernel_shape, pads, strides;
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "kernel_shape", kernel_shape);
        fbs_model->get_operation_attribute(node_name, "pads", pads);
        fbs_model->get_operation_attribute(node_name, "strides", strides);
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        if (kernel_shape.empty())
            return nullptr;
        if (pads.size() == 4) // ONNX [top, left, bottom, right] -> [top, bottom, left, right]
            pads = {pads[0], pads[2], pads[1], pads[3]};
        else if (pads.empty())
            pads.assign(kernel_shape.size() * 2, 0);
        if (strides.empty())
            strides.assign(kernel_shape.size(), 1);
        return new AveragePool(node_name.c_str(), kernel_shape, pads, strides, quant_type);
    }
    void print() { DL_LOGI("AveragePool", "kernel dims: %d, quant_type: %s.", (int)m_kernel_shape.size(), quant_type_to_string(quant_type)); }
};

/// Slice with positive steps (esp-dl/dl/module/include/dl_module_slice.hpp; ONNX index rules: negative
/// starts / ends count from the end, both are clamped to the extent).
class Slice : public Module {
private:
    std::vector<int64_t> m_start, m_end, m_axes, m_step;
    std::vector<int> m_norm_start, m_norm_step;

    bool normalize(const std::vector<int> &shape, std::vector<int> *out_shape)
    {
        const int nd = (int)shape.size();
        m_norm_start.assign(nd, 0);
        m_norm_step.assign(nd, 1);
        *out_shape = shape;
        for (size_t i = 0; i < m_start.size(); i++) {
            const int ax = m_axes.empty() ? (int)i : (int)((m_axes[i] + nd) % nd);
            const int64_t st = m_step.empty() ? 1 : m_step[i];
            if (ax < 0 || ax >= nd || st < 1)
                return false;
            const int64_t dim = shape[ax];
            int64_t s = m_start[i], e = m_end[i];
            s = s < 0 ? s + dim : s;
            e = e < 0 ? e + dim : e;
            s = std::min<int64_t>(std::max<int64_t>(s, 0), dim);
            e = std::min<int64_t>(std::max<int64_t>(e, 0), dim);
            m_norm_start[ax] = (int)s;
            m_norm_step[ax] = (int)st;
            (*out_shape)[ax] = e > s ? (int)((e - s + st - 1) / st) : 0;
        }
        return true;
    }

public:
    Slice(const char *name = nullptr, const std::vector<int64_t> &start = {}, const std::vector<int64_t> &end = {},
          const std::vector<int64_t> &axes = {}, const std::vector<int64_t> &step = {},
          quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_start(start), m_end(end), m_axes(axes), m_step(step)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        std::vector<int> out;
        if (!normalize(input_shapes[0], &out)) {
            DL_LOGE("Slice", "%s: bad axes or a step below 1 (negative steps are not part of this build)", name.c_str());
            return {input_shapes[0]};
        }
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!on_device_all({input, output}) || input->dtype != output->dtype) {
            DL_LOGE("Slice", "%s: needs device tensors of one type", name.c_str());
            return;
        }
        std::vector<int> out_shape;
        if (!normalize(input->shape, &out_shape) || out_shape != output->shape) {
            DL_LOGE("Slice", "%s: output shape does not match the slice", name.c_str());
            return;
        }
        const int rc = espdl_hip_slice(input->data, input->shape.data(), (int32_t)input->shape.size(), m_norm_start.data(),
                                       m_norm_step.data(), out_shape.data(), (int32_t)input->get_dtype_bytes(),
                                       output->data, context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Slice", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        std::vector<int64_t> v[4];
        for (int k = 0; k < 4; k++) {
            TensorBase *t = fbs_model->get_operation_parameter(node_name, k + 1);
            if (!t)
                continue;
            if (t->dtype == DATA_TYPE_INT64) {
                const int64_t *p = t->get_element_ptr<int64_t>();
                v[k].assign(p, p + t->get_size());
            } else if (t->dtype == DATA_TYPE_INT32) {
                const int32_t *p = t->get_element_ptr<int32_t>();
                v[k].assign(p, p + t->get_size());
            }
            delete t;
        }
        if (v[0].empty() || v[0].size() != v[1].size())
            return nullptr;
        return new Slice(node_name.c_str(), v[0], v[1], v[2], v[3], quant_type);
    }
    void print() { DL_LOGI("Slice", "axes: %d, quant_type: %s.", (int)m_start.size(), quant_type_to_string(quant_type)); }
};

/// ReduceMean on int8 tensors (esp-dl/dl/module/include/dl_module_reduce_mean.hpp, axes handling of
/// dl_module_reduce_base.hpp:262-298: `axes` is the second input; empty axes reduce everything unless
/// `noop_with_empty_axes` is set).
class ReduceMean : public Module {
private:
    int m_keepdims;
    std::vector<int64_t> m_axes;
    int m_noop_with_empty_axes;
    int m_int_op; ///< -1: mean; else ESPDL_HIP_REDUCE_MAX / _MIN / _SUM (the modules of dl_module_reduce_max.hpp,
                  ///< dl_module_reduce_min.hpp and dl_module_reduce_sum.hpp share the axes handling)

    std::vector<int32_t> flags_for(size_t rank) const
    {
        std::vector<int32_t> f(rank, 0);
        if (m_axes.empty()) {
            if (!m_noop_with_empty_axes)
                f.assign(rank, 1);
            return f;
        }
        for (int64_t a : m_axes) {
            const int64_t ax = a < 0 ? a + (int64_t)rank : a;
            if (ax >= 0 && ax < (int64_t)rank)
                f[(size_t)ax] = 1;
        }
        return f;
    }

public:
    ReduceMean(const char *name = nullptr, int keepdims = 1, const std::vector<int64_t> &axes = {},
               int noop_with_empty_axes = 0, quant_type_t quant_type = QUANT_TYPE_NONE, int int_op = -1) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_keepdims(keepdims), m_axes(axes),
        m_noop_with_empty_axes(noop_with_empty_axes), m_int_op(int_op)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        const std::vector<int32_t> f = flags_for(in.size());
        std::vector<int> out;
        for (size_t i = 0; i < in.size(); i++) {
            if (!f[i])
                out.push_back(in[i]);
            else if (m_keepdims)
                out.push_back(1);
        }
        if (out.empty())
            out.push_back(1);
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!on_device_all({input, output}) || (quant_type != QUANT_TYPE_SYMM_8BIT && quant_type != QUANT_TYPE_SYMM_16BIT) ||
            input->shape.size() > 8) {
            DL_LOGE("ReduceMean", "%s: needs int8 or int16 device tensors of at most 8 dims", name.c_str());
            return;
        }
        const std::vector<int32_t> f = flags_for(input->shape.size());
        if (m_int_op >= 0) {
            const int rc = espdl_hip_reduce_int(
                input->data, quant_type == QUANT_TYPE_SYMM_16BIT ? ESPDL_HIP_S16 : ESPDL_HIP_S8, input->shape.data(),
                (int32_t)input->shape.size(), f.data(), m_int_op,
                output->exponent.get() - input->exponent.get() * (m_int_op == ESPDL_HIP_REDUCE_SUM_SQUARE ? 2 : 1),
                context->round_mode == ROUND_MODE_HALF_EVEN ? ESPDL_HIP_ROUND_HALF_EVEN : ESPDL_HIP_ROUND_HALF_UP,
                output->data, context->stream);
            if (rc != ESPDL_HIP_OK)
                DL_LOGE("Reduce", "%s: %s", name.c_str(), espdl_hip_last_error());
            return;
        }
        const int rc = quant_type == QUANT_TYPE_SYMM_16BIT
            ? espdl_hip_reduce_mean_s16(static_cast<const int16_t *>(input->data), input->shape.data(),
                                        (int32_t)input->shape.size(), f.data(), input->exponent.get(),
                                        output->exponent.get(), static_cast<int16_t *>(output->data), context->stream)
            : espdl_hip_reduce_mean_s8(static_cast<const int8_t *>(input->data), input->shape.data(),
                                       (int32_t)input->shape.size(), f.data(), input->exponent.get(),
                                       output->exponent.get(), static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("ReduceMean", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name) { return make(fbs_model, node_name, -1); }
    static Module *deserialize_max(fbs::FbsModel *fbs_model, std::string node_name)
    {
        return make(fbs_model, node_name, ESPDL_HIP_REDUCE_MAX);
    }
    static Module *deserialize_min(fbs::FbsModel *fbs_model, std::string node_name)
    {
        return make(fbs_model, node_name, ESPDL_HIP_REDUCE_MIN);
    }
    static Module *deserialize_sum(fbs::FbsModel *fbs_model, std::string node_name)
    {
        return make(fbs_model, node_name, ESPDL_HIP_REDUCE_SUM);
    }
    static Module *deserialize_l1(fbs::FbsModel *fbs_model, std::string node_name)
    {
        return make(fbs_model, node_name, ESPDL_HIP_REDUCE_L1);
    }
    static Module *deserialize_sum_square(fbs::FbsModel *fbs_model, std::string node_name)
    {
        return make(fbs_model, node_name, ESPDL_HIP_REDUCE_SUM_SQUARE);
    }
    static Module *make(fbs::FbsModel *fbs_model, const std::string &node_name, int int_op)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        int keepdims = 1, noop = 0;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "keepdims", keepdims);
        fbs_model->get_operation_attribute(node_name, "noop_with_empty_axes", noop);
        std::vector<int64_t> axes;
        TensorBase *t = fbs_model->get_operation_parameter(node_name, 1);
        if (t) {
            if (t->dtype == DATA_TYPE_INT64) {
                const int64_t *p = t->get_element_ptr<int64_t>();
                axes.assign(p, p + t->get_size());
            } else if (t->dtype == DATA_TYPE_INT32) {
                const int32_t *p = t->get_element_ptr<int32_t>();
                axes.assign(p, p + t->get_size());
            }
            delete t;
        } else {
            std::vector<int> attr_axes; // older exports carry the axes as an attribute
            if (fbs_model->get_operation_attribute(node_name, "axes", attr_axes) == ESP_OK)
                axes.assign(attr_axes.begin(), attr_axes.end());
        }
        return new ReduceMean(node_name.c_str(), keepdims, axes, noop, quant_type, int_op);
    }
    void print() { DL_LOGI("ReduceMean", "keepdims: %d, quant_type: %s.", m_keepdims, quant_type_to_string(quant_type)); }
};

/// StreamingCache (esp-dl/dl/module/include/dl_module_streaming_cache.hpp): the output is the last
/// window_size - 1 frames of the previous call followed by this call's frames; the cache starts as zeros.
/// The reference copies whole byte blocks of its single image, which is a concatenation along axis 1;
/// here every image of the batch carries its own cache and the same block copies run once per image.
class StreamingCache : public Module {
private:
    int m_window_size, m_frame_axis;
    TensorBase *m_cache = nullptr; ///< [batch][cache bytes per image], device
    TensorBase *m_held = nullptr;  ///< copy of the cache while a discarded pass runs
    bool m_held_valid = false;

public:
    StreamingCache(const char *name = nullptr, int window_size = 1, int frame_axis = 1,
                   quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_window_size(window_size), m_frame_axis(frame_axis)
    {
    }
    ~StreamingCache()
    {
        delete m_cache;
        delete m_held;
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        std::vector<int> out = input_shapes[0];
        const int axis = m_frame_axis < 0 ? m_frame_axis + (int)out.size() : m_frame_axis;
        if (axis != 1 || out.size() < 2 || m_window_size < 1)
            return {{}}; // the block copies below are a concatenation only along axis 1
        out[1] += m_window_size - 1;
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!on_device_all({input, output}) || input->shape.size() < 2 || input->dtype != output->dtype) {
            DL_LOGE("StreamingCache", "%s: needs device tensors of one dtype", name.c_str());
            return;
        }
        const int64_t batch = input->shape[0];
        const int64_t in_bytes = (int64_t)input->get_bytes() / std::max<int64_t>(1, batch);
        const int64_t frame_bytes = in_bytes / std::max(1, input->shape[1]);
        const int64_t cache_bytes = frame_bytes * (m_window_size - 1);
        if (cache_bytes == 0) {
            output->copy_from(input, context->stream);
            return;
        }
        if (m_cache == nullptr || m_cache->get_bytes() != (size_t)(batch * cache_bytes)) {
            delete m_cache;
            m_cache = new TensorBase({(int)batch, (int)cache_bytes}, nullptr, 0, DATA_TYPE_INT8, true, MALLOC_CAP_DEVICE);
            if (!m_cache->data) { // a null element pointer asks for zero-filled storage
                DL_LOGE("StreamingCache", "%s: cannot allocate the cache", name.c_str());
                return;
            }
        }
        char *out = static_cast<char *>(output->data);
        const int64_t out_bytes = cache_bytes + in_bytes;
        int rc = espdl_hip_copy_rows(m_cache->data, cache_bytes, out, out_bytes, cache_bytes, batch, context->stream);
        if (rc == ESPDL_HIP_OK)
            rc = espdl_hip_copy_rows(input->data, in_bytes, out + cache_bytes, out_bytes, in_bytes, batch, context->stream);
        if (rc == ESPDL_HIP_OK)
            rc = espdl_hip_copy_rows(out + in_bytes, out_bytes, m_cache->data, cache_bytes, cache_bytes, batch, context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("StreamingCache", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    /// Forget the frames seen so far.
    void reset()
    {
        if (m_cache && m_cache->data)
            m_cache->memset(0, nullptr);
    }
    void hold_state(void *stream)
    {
        m_held_valid = false;
        if (!m_cache || !m_cache->data)
            return; // nothing seen yet: restore_state clears whatever the discarded pass leaves
        if (!m_held || m_held->get_bytes() != m_cache->get_bytes()) {
            delete m_held;
            m_held = new TensorBase(m_cache->shape, nullptr, 0, DATA_TYPE_INT8, true, MALLOC_CAP_DEVICE);
        }
        m_held_valid = m_held->copy_from(m_cache, stream);
    }
    void restore_state(void *stream)
    {
        if (!m_cache || !m_cache->data)
            return;
        if (m_held_valid && m_held && m_held->get_bytes() == m_cache->get_bytes())
            m_cache->copy_from(m_held, stream);
        else
            m_cache->memset(0, stream);
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        int window_size = 1, frame_axis = 1;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "window_size", window_size);
        fbs_model->get_operation_attribute(node_name, "frame_axis", frame_axis);
        return new StreamingCache(node_name.c_str(), window_size, frame_axis, quant_type);
    }
    void print()
    {
        DL_LOGI("StreamingCache", "window_size: %d, frame_axis: %d, quant_type: %s.", m_window_size, m_frame_axis,
                quant_type_to_string(quant_type));
    }
};

/// InsertZeros on [N, spatial..., C] tensors with one or two spatial dims
/// (esp-dl/dl/module/include/dl_module_insert_zeros.hpp): the exporter writes a transposed convolution as
/// InsertZeros followed by an ordinary Conv.
class InsertZeros : public Module {
private:
    std::vector<int> m_stride, m_output_padding;

    void normalize(size_t spatial)
    {
        if (m_stride.size() == 1 && spatial > 1)
            m_stride.assign(spatial, m_stride[0]);
        if (m_output_padding.size() == 1 && spatial > 1)
            m_output_padding.assign(spatial, m_output_padding[0]);
    }

public:
    InsertZeros(const char *name = nullptr, const std::vector<int> &stride = {1}, const std::vector<int> &output_padding = {0},
                quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_stride(stride), m_output_padding(output_padding)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        if (in.size() != 3 && in.size() != 4)
            return {{}};
        const size_t spatial = in.size() - 2;
        normalize(spatial);
        if (m_stride.size() != spatial || m_output_padding.size() != spatial)
            return {{}};
        std::vector<int> out = in;
        for (size_t i = 0; i < spatial; i++)
            out[1 + i] = in[1 + i] + (m_stride[i] - 1) * (in[1 + i] - 1) + m_output_padding[i];
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!on_device_all({input, output}) || (input->shape.size() != 3 && input->shape.size() != 4) ||
            input->dtype != output->dtype) {
            DL_LOGE("InsertZeros", "%s: needs device tensors of rank 3 or 4 and one dtype", name.c_str());
            return;
        }
        const bool one_d = input->shape.size() == 3;
        normalize(input->shape.size() - 2);
        const int rc = espdl_hip_insert_zeros(input->data, (int32_t)input->get_dtype_bytes(), input->shape[0], input->shape[1],
                                              one_d ? 1 : input->shape[2], input->shape.back(), m_stride[0],
                                              one_d ? 1 : m_stride[1], m_output_padding[0],
                                              one_d ? 0 : m_output_padding[1], output->data, context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("InsertZeros", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        std::vector<int> stride = {1}, output_padding = {0};
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "stride", stride);
        fbs_model->get_operation_attribute(node_name, "output_padding", output_padding);
        if (stride.empty())
            stride = {1};
        if (output_padding.empty())
            output_padding = {0};
        return new InsertZeros(node_name.c_str(), stride, output_padding, quant_type);
    }
    void print() { DL_LOGI("InsertZeros", "stride: %s, quant_type: %s.", vector_to_string(m_stride).c_str(), quant_type_to_string(quant_type)); }
};

/// SpaceToDepth and DepthToSpace on NHWC tensors (esp-dl/dl/module/include/dl_module_space_to_depth.hpp:17-44,
/// dl_module_depth_to_space.hpp:17-67).  Both are permutations of a six-axis view of the tensor, so they run
/// on the transpose kernel:
///   SpaceToDepth      [N, H/b, b, W/b, b, C] -> [N, H/b, W/b, C, b, b]      out_c = c * b^2 + (h % b) * b + w % b
///   DepthToSpace CRD  [N, H, W, C', b, b]    -> [N, H, b, W, b, C']         c = out_c * b^2 + hb * b + wb
///   DepthToSpace DCR  [N, H, W, b, b, C']    -> [N, H, b, W, b, C']         c = (hb * b + wb) * C' + out_c
/// The reference's DCR loop takes out_c = c % b, which is this permutation when C' == b and not a permutation
/// otherwise (output elements are written twice or never); the ONNX definition is used for every C'.
class SpaceDepth : public Module {
public:
    enum kind_t { SPACE_TO_DEPTH, DEPTH_TO_SPACE_CRD, DEPTH_TO_SPACE_DCR };

private:
    kind_t m_kind;
    int m_blocksize;

public:
    SpaceDepth(kind_t kind, int blocksize, const char *name = nullptr, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_kind(kind), m_blocksize(blocksize)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        const int b = m_blocksize;
        if (in.size() != 4 || b < 1)
            return {{}};
        if (m_kind == SPACE_TO_DEPTH) {
            if (in[1] % b || in[2] % b)
                return {{}};
            return {{in[0], in[1] / b, in[2] / b, in[3] * b * b}};
        }
        if (in[3] % (b * b))
            return {{}};
        return {{in[0], in[1] * b, in[2] * b, in[3] / (b * b)}};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        const char *tag = m_kind == SPACE_TO_DEPTH ? "SpaceToDepth" : "DepthToSpace";
        if (!on_device_all({input, output}) || input->shape.size() != 4 || input->dtype != output->dtype ||
            input->get_size() != output->get_size()) {
            DL_LOGE(tag, "%s: needs NHWC device tensors of one type", name.c_str());
            return;
        }
        const int b = m_blocksize, n = input->shape[0], h = input->shape[1], w = input->shape[2], c = input->shape[3];
        int32_t view[6], perm[6];
        if (m_kind == SPACE_TO_DEPTH) {
            const int32_t v[6] = {n, h / b, b, w / b, b, c}, p[6] = {0, 1, 3, 5, 2, 4};
            std::copy(v, v + 6, view);
            std::copy(p, p + 6, perm);
        } else if (m_kind == DEPTH_TO_SPACE_CRD) {
            const int32_t v[6] = {n, h, w, c / (b * b), b, b}, p[6] = {0, 1, 4, 2, 5, 3};
            std::copy(v, v + 6, view);
            std::copy(p, p + 6, perm);
        } else {
            const int32_t v[6] = {n, h, w, b, b, c / (b * b)}, p[6] = {0, 1, 3, 2, 4, 5};
            std::copy(v, v + 6, view);
            std::copy(p, p + 6, perm);
        }
        const int rc = espdl_hip_transpose(input->data, view, 6, perm, 6, (int32_t)input->get_dtype_bytes(), output->data,
                                           context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE(tag, "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize_space_to_depth(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        int blocksize = 2;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "blocksize", blocksize);
        return new SpaceDepth(SPACE_TO_DEPTH, blocksize, node_name.c_str(), quant_type);
    }
    static Module *deserialize_depth_to_space(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        int blocksize = 2;
        std::string mode_name = "DCR";
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "blocksize", blocksize);
        fbs_model->get_operation_attribute(node_name, "mode", mode_name);
        return new SpaceDepth(mode_name == "CRD" ? DEPTH_TO_SPACE_CRD : DEPTH_TO_SPACE_DCR, blocksize, node_name.c_str(),
                              quant_type);
    }
    void print()
    {
        DL_LOGI(m_kind == SPACE_TO_DEPTH ? "SpaceToDepth" : "DepthToSpace", "blocksize: %d, quant_type: %s.", m_blocksize,
                quant_type_to_string(quant_type));
    }
};

/// Gather with constant indices (esp-dl/dl/module/include/dl_module_gather.hpp:13-170): for every outer index, the
/// rows named by `indices` along `axis` are copied in order.  Runs of consecutive indices are one strided copy
/// (espdl_hip_copy_rows), so a single index or a range costs one launch.  Indices outside [0, extent) read
/// outside the tensor in the reference; they are rejected here.
class Gather : public Module {
private:
    std::vector<int64_t> m_indices;
    std::vector<int> m_indices_shape;
    int m_axis;

public:
    Gather(const std::vector<int64_t> &indices, const std::vector<int> &indices_shape, int axis, const char *name = nullptr,
           quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_indices(indices), m_indices_shape(indices_shape), m_axis(axis)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        const int axis = m_axis < 0 ? m_axis + (int)in.size() : m_axis;
        if (axis < 0 || axis >= (int)in.size())
            return {{}};
        for (int64_t i : m_indices)
            if (i < 0 || i >= in[axis])
                return {{}};
        std::vector<int> out(in.begin(), in.begin() + axis);
        out.insert(out.end(), m_indices_shape.begin(), m_indices_shape.end());
        out.insert(out.end(), in.begin() + axis + 1, in.end());
        if (out.empty())
            out.push_back(1);
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        const int rank = (int)input->shape.size(), axis = m_axis < 0 ? m_axis + rank : m_axis;
        if (!on_device_all({input, output}) || input->dtype != output->dtype || axis < 0 || axis >= rank) {
            DL_LOGE("Gather", "%s: needs device tensors of one type and an axis inside the tensor", name.c_str());
            return;
        }
        int64_t outer = 1, inner = input->get_dtype_bytes();
        for (int i = 0; i < axis; i++)
            outer *= input->shape[i];
        for (int i = axis + 1; i < rank; i++)
            inner *= input->shape[i];
        const int64_t extent = input->shape[axis], count = (int64_t)m_indices.size();
        if (output->get_size() * (int64_t)output->get_dtype_bytes() != outer * count * inner) {
            DL_LOGE("Gather", "%s: output size does not match", name.c_str());
            return;
        }
        const char *src = static_cast<const char *>(input->data);
        char *dst = static_cast<char *>(output->data);
        for (int64_t i = 0; i < count;) {
            int64_t run = 1;
            while (i + run < count && m_indices[i + run] == m_indices[i] + run)
                run++;
            if (m_indices[i] < 0 || m_indices[i] + run > extent) {
                DL_LOGE("Gather", "%s: index outside the axis", name.c_str());
                return;
            }
            const int rc = espdl_hip_copy_rows(src + m_indices[i] * inner, extent * inner, dst + i * inner, count * inner,
                                               run * inner, outer, context->stream);
            if (rc != ESPDL_HIP_OK) {
                DL_LOGE("Gather", "%s: %s", name.c_str(), espdl_hip_last_error());
                return;
            }
            i += run;
        }
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        int axis = 0;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "axis", axis);
        TensorBase *t = fbs_model->get_operation_parameter(node_name, 1);
        if (!t || (t->dtype != DATA_TYPE_INT64 && t->dtype != DATA_TYPE_INT32)) {
            DL_LOGE("Gather", "%s: indices must be an int64 or int32 initializer", node_name.c_str());
            delete t;
            return nullptr;
        }
        std::vector<int64_t> indices;
        for (int i = 0; i < t->get_size(); i++)
            indices.push_back(t->dtype == DATA_TYPE_INT64 ? t->get_element_ptr<int64_t>()[i]
                                                          : (int64_t)t->get_element_ptr<int32_t>()[i]);
        const std::vector<int> shape = t->shape;
        delete t;
        return new Gather(indices, shape, axis, node_name.c_str(), quant_type);
    }
    void print() { DL_LOGI("Gather", "axis: %d, indices: %d, quant_type: %s.", m_axis, (int)m_indices.size(), quant_type_to_string(quant_type)); }
};

/// Pad (esp-dl/dl/module/include/dl_module_pad.hpp:12-100): pads and the optional constant are initializer
/// operands; the constant is read as the tensor's element type, whatever its own exponent says
/// (TensorBase::pad, esp-dl/dl/tensor/src/dl_tensor_base.cpp:1231-1234).
class Pad : public Module {
private:
    std::vector<int> m_pads;
    int m_mode;
    int m_constant;

public:
    Pad(const std::vector<int> &pads, int mode, int constant, const char *name = nullptr,
        quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_pads(pads), m_mode(mode), m_constant(constant)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        if (m_pads.size() != 2 * in.size() || in.empty() || in.size() > 8)
            return {{}};
        std::vector<int> out = in;
        for (size_t i = 0; i < in.size(); i++) {
            if (m_pads[i] < 0 || m_pads[i + in.size()] < 0)
                return {{}};
            out[i] = in[i] + m_pads[i] + m_pads[i + in.size()];
        }
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (!on_device_all({input, output}) || input->dtype != output->dtype ||
            m_pads.size() != 2 * input->shape.size()) {
            DL_LOGE("Pad", "%s: needs device tensors of one dtype and two pads per axis", name.c_str());
            return;
        }
        const int rc = espdl_hip_pad(input->data, input->shape.data(), (int32_t)input->shape.size(), m_pads.data(), m_mode,
                                     m_constant, (int32_t)input->get_dtype_bytes(), output->data, context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Pad", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        std::string mode_name = "constant";
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "mode", mode_name);
        int mode;
        if (mode_name == "constant")
            mode = ESPDL_HIP_PAD_CONSTANT;
        else if (mode_name == "edge")
            mode = ESPDL_HIP_PAD_EDGE;
        else if (mode_name == "reflect")
            mode = ESPDL_HIP_PAD_REFLECT;
        else {
            DL_LOGE("Pad", "%s: mode %s is not supported", node_name.c_str(), mode_name.c_str());
            return nullptr;
        }
        std::vector<int> pads;
        TensorBase *t = fbs_model->get_operation_parameter(node_name, 1);
        if (!t || t->dtype != DATA_TYPE_INT64) {
            DL_LOGE("Pad", "%s: pads must be an int64 initializer", node_name.c_str());
            delete t;
            return nullptr;
        }
        for (int i = 0; i < t->get_size(); i++)
            pads.push_back((int)t->get_element_ptr<int64_t>()[i]);
        delete t;
        int constant = 0;
        if (TensorBase *c = fbs_model->get_operation_parameter(node_name, 2)) {
            if (c->get_size() > 0) {
                if (c->dtype == DATA_TYPE_INT8)
                    constant = c->get_element_ptr<int8_t>()[0];
                else if (c->dtype == DATA_TYPE_INT16)
                    constant = c->get_element_ptr<int16_t>()[0];
                else if (c->dtype == DATA_TYPE_INT32)
                    constant = c->get_element_ptr<int32_t>()[0];
            }
            delete c;
        }
        return new Pad(pads, mode, constant, node_name.c_str(), quant_type);
    }
    void print() { DL_LOGI("Pad", "pads: %s, quant_type: %s.", vector_to_string(m_pads).c_str(), quant_type_to_string(quant_type)); }
};

/// Softmax on an int8 tensor with a float32 result (esp-dl/dl/module/include/dl_module_softmax.hpp,
/// forward_lut): the exported graphs follow it with QuantizeLinear.
class Softmax : public Module {
private:
    int m_axis;

public:
    Softmax(const char *name = nullptr, int axis = -1, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_axis(axis)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        return {input_shapes[0]};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (quant_type != QUANT_TYPE_SYMM_8BIT || !input || !output || !input->on_device() || !output->on_device() ||
            input->dtype != DATA_TYPE_INT8 || output->dtype != DATA_TYPE_FLOAT || input->shape.empty()) {
            DL_LOGE("Softmax", "%s: needs an int8 device input and a float32 device output", name.c_str());
            return;
        }
        const int rank = (int)input->shape.size();
        const int axis = m_axis < 0 ? m_axis + rank : m_axis;
        if (axis < 0 || axis >= rank) {
            DL_LOGE("Softmax", "%s: axis %d outside rank %d", name.c_str(), m_axis, rank);
            return;
        }
        int64_t outer = 1, inner = 1;
        for (int i = 0; i < axis; i++)
            outer *= input->shape[i];
        for (int i = axis + 1; i < rank; i++)
            inner *= input->shape[i];
        const int rc = espdl_hip_softmax_s8(static_cast<const int8_t *>(input->data), outer, input->shape[axis], inner,
                                            input->exponent.get(), static_cast<float *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Softmax", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        int axis = -1;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "axis", axis);
        return new Softmax(node_name.c_str(), axis, quant_type);
    }
    void print() { DL_LOGI("Softmax", "axis: %d, quant_type: %s.", m_axis, quant_type_to_string(quant_type)); }
};

} // namespace module
} // namespace dl
