// dl::module::Conv — Conv2D / DepthwiseConv2D / Conv1D operator object.
//
// Mirrors esp-dl/dl/module/include/dl_module_conv.hpp:17-239: attributes (activation, pads
// {top,bottom,left,right}, dilations, strides, group), get_output_shape (:81-102), forward (:121-162),
// deserialize with the ONNX pad re-ordering [t,l,b,r] -> [t,b,l,r] (:167-195).  group == 1 is a dense
// convolution, anything else a depthwise one (:104-119).  forward() derives
// shift[c] = out_exp - filter_exp[c] - in_exp (esp-dl/dl/base/dl_base.hpp:243-261) and enqueues
// espdl_hip_conv2d; an optional 256-entry table fuses a following LUT module into the epilogue.
#pragma once

#include <cassert>

#include "dl_module_base.hpp"
#include "espdl_hip.h"

namespace dl {
namespace module {

/// Fill the requantization shifts of a Conv / Gemm / MatMul from the tensors' exponents.
inline std::vector<int32_t> conv_shifts(int out_exponent, TensorBase *input, TensorBase *filter, int out_c)
{
    std::vector<int32_t> shifts;
    if (filter->exponent.is_per_channel()) {
        shifts.resize(out_c);
        for (int c = 0; c < out_c; c++)
            shifts[c] = out_exponent - filter->exponent.get(c) - input->exponent.get();
    } else {
        shifts.push_back(out_exponent - filter->exponent.get() - input->exponent.get());
    }
    return shifts;
}
inline std::vector<int32_t> conv_shifts(TensorBase *output, TensorBase *input, TensorBase *filter, int out_c)
{
    return conv_shifts(output->exponent.get(), input, filter, out_c);
}

class Conv : public Module {
private:
    activation_type_t activation;
    std::vector<int> m_pads;      ///< {top, bottom, left, right} (2-D) or {left, right} (1-D)
    std::vector<int> m_dilations; ///< {h, w} or {w}
    std::vector<int> m_strides;   ///< {h, w} or {w}
    int m_group;
    TensorBase *m_fused_lut; ///< device int8[256] applied to the stored value, or nullptr (owned)
    DeviceInts m_shift;
    // A depthwise Conv may absorb the 1x1 Conv that follows it (and the Add after that): the three
    // run as one kernel and the depthwise result stays on chip.  The absorbed modules' parameter
    // indices are appended to m_inputs_index at the positions below.
    bool m_has_project = false;
    activation_type_t m_project_activation = Linear;
    int m_mid_exponent = 0;      ///< exponent of the (no longer materialized) depthwise output
    int m_lut_in_exponent = 0;   ///< exponent of the conv result that indexes a fused LUT
    int m_project_filter_pos = -1, m_project_bias_pos = -1, m_residual_pos = -1;
    int m_residual_shift = 0;
    bool m_has_gap = false;      // a GlobalAveragePool behind this (1x1) convolution runs in its launch
    int m_gap_in_exponent = 0;   // exponent of the tensor the convolution used to write
    int m_own_inputs = 0; ///< inputs of the Conv itself when a plain residual Add was absorbed
    bool m_has_pre_add_exponent = false;
    int m_pre_add_exponent = 0; ///< exponent of the tensor an absorbed Add used to read from this module
    DeviceInts m_shift_project;
    // A depthwise Conv that absorbed its project Conv may also absorb the 1x1 Conv in front of it: its first
    // input is then the block input and the expanded tensor is never materialized.
    bool m_has_expand = false;
    int m_fused_kernel = 0;
    activation_type_t m_expand_activation = Linear;
    int m_expand_exponent = 0; ///< exponent of the (no longer materialized) expanded tensor
    int m_expand_filter_pos = -1, m_expand_bias_pos = -1;
    DeviceInts m_shift_expand;
    // the absorbed Conv's own window: {1, 1} / {1, 1} / no padding for the usual 1x1 expand, anything else
    // for a stem convolution that took the expand stage's place
    std::vector<int> m_expand_kernel = {1, 1}, m_expand_strides = {1, 1}, m_expand_pads = {0, 0, 0, 0};
    // Clip modules with equal exponents that stood between the stages of the fused block: {on, min, max}
    int m_clip_expand[3] = {0, -128, 127}, m_clip_dw[3] = {0, -128, 127};

public:
    Conv(activation_type_t activation = Linear, std::vector<int> pads = {}, std::vector<int> dilations = {},
         std::vector<int> strides = {}, const char *name = nullptr, int group = 1,
         quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type),
        activation(activation),
        m_pads(pads),
        m_dilations(dilations),
        m_strides(strides),
        m_group(group),
        m_fused_lut(nullptr)
    {
    }
    ~Conv() { delete m_fused_lut; }

    int get_group() const { return m_group; }
    activation_type_t get_activation() const { return activation; }
    /// Take ownership of a LUT (host or device tensor of 256 int8) to apply in the epilogue.
    /// `table_in_exponent` is the exponent of the value the table is indexed with, i.e. of this
    /// convolution's own (no longer materialized) output: the requantization shift is derived from it,
    /// not from the exponent of the tensor the table's result is stored to.
    void fuse_lut(TensorBase *table, int table_in_exponent)
    {
        delete m_fused_lut;
        m_fused_lut = table;
        m_lut_in_exponent = table_in_exponent;
    }
    bool has_fused_lut() const { return m_fused_lut != nullptr; }
    bool has_fused_project() const { return m_has_project; }
    const std::vector<int> &get_pads() const { return m_pads; }
    const std::vector<int> &get_strides() const { return m_strides; }
    const std::vector<int> &get_dilations() const { return m_dilations; }
    /// Absorb a following 1x1 Conv (filter / bias indices, activation) and optionally the other
    /// operand of the Add after it.  The caller re-points m_outputs_index at the final tensor.
    /// `residual_shift`: the residual operand is requantized by that power of two inside the kernel (the pass
    /// absorbed the RequantizeLinear that did it: exponent of its input - exponent of its output).
    void fuse_project(int filter_index, int bias_index, activation_type_t act, int mid_exponent, int residual_index,
                      int project_out_exponent = 0, int residual_shift = 0)
    {
        m_residual_shift = residual_index >= 0 ? residual_shift : 0;
        if (residual_index >= 0) {
            m_has_pre_add_exponent = true;
            m_pre_add_exponent = project_out_exponent;
        }
        m_has_project = true;
        m_project_activation = act;
        m_mid_exponent = mid_exponent;
        m_project_filter_pos = (int)m_inputs_index.size();
        m_inputs_index.push_back(filter_index);
        if (bias_index >= 0) {
            m_project_bias_pos = (int)m_inputs_index.size();
            m_inputs_index.push_back(bias_index);
        }
        if (residual_index >= 0) {
            m_residual_pos = (int)m_inputs_index.size();
            m_inputs_index.push_back(residual_index);
        }
    }
    /// Absorb the Conv in front (after fuse_project): `input_index` is that Conv's input, which becomes
    /// this module's first input; `expand_exponent` the exponent of the tensor it used to write.  kernel /
    /// strides / pads ({top, bottom, left, right}) describe that Conv when it is not a plain 1x1.
    void fuse_expand(int input_index, int filter_index, int bias_index, activation_type_t act, int expand_exponent,
                     std::vector<int> kernel = {1, 1}, std::vector<int> strides = {1, 1},
                     std::vector<int> pads = {0, 0, 0, 0})
    {
        m_expand_kernel = kernel;
        m_expand_strides = strides;
        m_expand_pads = pads;
        m_has_expand = true;
        m_expand_activation = act;
        m_expand_exponent = expand_exponent;
        m_inputs_index[0] = input_index;
        m_expand_filter_pos = (int)m_inputs_index.size();
        m_inputs_index.push_back(filter_index);
        if (bias_index >= 0) {
            m_expand_bias_pos = (int)m_inputs_index.size();
            m_inputs_index.push_back(bias_index);
        }
    }
    /// A Clip (equal exponents: a clamp of the stored value) that stood behind the absorbed expand Conv
    /// (`stage` 0) or behind this depthwise Conv (`stage` 1) runs inside the fused launch.
    void fuse_clip(int stage, int min_q, int max_q)
    {
        int *c = stage == 0 ? m_clip_expand : m_clip_dw;
        c[0] = 1;
        c[1] = min_q;
        c[2] = max_q;
    }
    bool has_fused_expand() const { return m_has_expand; }
    bool expand_has_window() const
    {
        return m_has_expand &&
            (m_expand_kernel != std::vector<int>{1, 1} || m_expand_strides != std::vector<int>{1, 1} ||
             m_expand_pads != std::vector<int>{0, 0, 0, 0});
    }
    /// answer of espdl_hip_mbconv_s8_supported for the fused form at its last forward (0 before the first):
    /// which single-launch kernel runs it
    int fused_kernel() const { return m_fused_kernel; }
    /// Absorb the Add that follows a dense Conv: `residual_index` is the Add's other operand and
    /// `own_out_exponent` the exponent of the tensor the Conv used to write.  The Add sums stored integers
    /// whatever the exponents of its operands and result are (esp-dl/dl/base/dl_base_add.cpp:35-44), so the
    /// Conv keeps requantizing to its own exponent, not to the one of the tensor it now writes.
    void fuse_residual(int residual_index, int own_out_exponent)
    {
        m_has_pre_add_exponent = true;
        m_pre_add_exponent = own_out_exponent;
        m_own_inputs = (int)m_inputs_index.size();
        m_residual_pos = (int)m_inputs_index.size();
        m_inputs_index.push_back(residual_index);
    }
    bool has_fused_residual() const { return m_residual_pos >= 0; }
    /// A dense 8-bit convolution on its own (with or without a folded table or residual Add) passes channel
    /// pitches to the kernels for its data input, its residual and its output.
    bool handles_channel_slices() const
    {
        return quant_type == QUANT_TYPE_SYMM_8BIT && m_group == 1 && !m_has_project && !m_has_gap;
    }
    bool reads_channel_slice(int slot) const { return handles_channel_slices() && (slot == 0 || slot == m_residual_pos); }
    bool writes_channel_slice(int slot) const { return handles_channel_slices() && slot == 0; }
    /// Absorb the GlobalAveragePool that is the only reader of this convolution's output: the module then
    /// writes the pooled tensor [N, 1, 1, C] (espdl_hip_conv2d_gap_s8); `conv_out_exponent` is the exponent of
    /// the tensor the convolution used to write.
    void fuse_gap(int conv_out_exponent)
    {
        m_has_gap = true;
        m_gap_in_exponent = conv_out_exponent;
    }
    bool has_fused_gap() const { return m_has_gap; }
    /// Position of the depthwise bias in m_inputs_index, or -1.
    int own_bias_pos() const
    {
        const int own = m_has_project ? m_project_filter_pos : (m_own_inputs > 0 ? m_own_inputs : (int)m_inputs_index.size());
        return own == 3 ? 2 : -1;
    }

    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        assert(input_shapes.size() >= 2);
        assert(input_shapes[0].size() == 3 || input_shapes[0].size() == 4);
        std::vector<int> input_shape = input_shapes[0];
        std::vector<int> filter_shape = input_shapes[1];
        if (expand_has_window() && input_shape.size() == 4) {
            // the depthwise stage reads the absorbed convolution's output
            input_shape[1] = (input_shape[1] + m_expand_pads[0] + m_expand_pads[1] - m_expand_kernel[0]) / m_expand_strides[0] + 1;
            input_shape[2] = (input_shape[2] + m_expand_pads[2] + m_expand_pads[3] - m_expand_kernel[1]) / m_expand_strides[1] + 1;
        }
        std::vector<int> output_shape = input_shape;
        if (input_shape.size() == 3) {
            // [N, W, C], filter [kW, Cin, Cout] (dense) / [kW, 1, C] (depthwise)
            output_shape[1] = (input_shape[1] + m_pads[0] + m_pads[1] - m_dilations[0] * (filter_shape[0] - 1) - 1) /
                    m_strides[0] +
                1;
            output_shape[2] = m_group == 1 ? filter_shape[2] : input_shape[2];
        } else {
            output_shape[1] = (input_shape[1] + m_pads[0] + m_pads[1] - m_dilations[0] * (filter_shape[0] - 1) - 1) /
                    m_strides[0] +
                1;
            output_shape[2] = (input_shape[2] + m_pads[2] + m_pads[3] - m_dilations[1] * (filter_shape[1] - 1) - 1) /
                    m_strides[1] +
                1;
            output_shape[3] = m_group == 1 ? filter_shape[3] : input_shape[3];
            if (m_has_project)
                output_shape[3] = input_shapes[m_project_filter_pos][3];
            if (m_has_gap)
                output_shape[1] = output_shape[2] = 1;
        }
        return {output_shape};
    }

    int64_t get_macs(std::vector<std::vector<int>> &input_shapes)
    {
        std::vector<int> out = get_output_shape(input_shapes)[0];
        const std::vector<int> &f = input_shapes[1];
        if (m_has_gap) { // a 1x1 stride-1 convolution: as many output pixels as input pixels
            out[1] = input_shapes[0][1];
            out[2] = input_shapes[0][2];
        }
        int64_t pixels = 1;
        for (size_t i = 0; i + 1 < out.size(); i++)
            pixels *= out[i];
        const int64_t taps = out.size() == 3 ? f[0] : (int64_t)f[0] * f[1];
        const int64_t in_c = m_group == 1 ? input_shapes[0].back() : 1;
        if (m_has_project) { // [1x1 over the block input +] depthwise + 1x1 over the depthwise channels
            const int64_t dw_c = input_shapes[m_project_filter_pos][2];
            int64_t macs = pixels * dw_c * taps + pixels * out.back() * dw_c;
            if (m_has_expand) {
                // absorbed convolution: its output pixels x window x input channels x expanded channels
                const int64_t eh = (input_shapes[0][1] + m_expand_pads[0] + m_expand_pads[1] - m_expand_kernel[0]) / m_expand_strides[0] + 1;
                const int64_t ew = (input_shapes[0][2] + m_expand_pads[2] + m_expand_pads[3] - m_expand_kernel[1]) / m_expand_strides[1] + 1;
                macs += (int64_t)input_shapes[0][0] * eh * ew * m_expand_kernel[0] * m_expand_kernel[1] * input_shapes[0][3] * dw_c;
            }
            return macs;
        }
        return pixels * out.back() * taps * in_c;
    }

    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *filter = context->get_tensor(m_inputs_index[1]);
        TensorBase *bias = own_bias_pos() >= 0 ? context->get_tensor(m_inputs_index[own_bias_pos()]) : nullptr;
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (m_has_project) {
            forward_with_project(context, input, filter, bias, output);
            return;
        }
        if (!input || !filter || !output || !input->on_device() || !filter->on_device() || !output->on_device() ||
            (bias && !bias->on_device())) {
            DL_LOGE("Conv", "%s: tensors must be device tensors", name.c_str());
            return;
        }

        espdl_hip_conv_desc d = {};
        d.dtype = quant_type == QUANT_TYPE_SYMM_16BIT ? ESPDL_HIP_S16 : ESPDL_HIP_S8;
        d.batch = input->shape[0];
        if (input->shape.size() == 3) {
            d.in_h = 1;
            d.in_w = input->shape[1];
            d.in_c = input->shape[2];
            d.out_c = output->shape[2];
            d.k_h = 1;
            d.k_w = filter->shape[0];
            d.stride_h = 1;
            d.stride_w = m_strides[0];
            d.dil_h = 1;
            d.dil_w = m_dilations[0];
            d.pad_left = m_pads[0];
            d.pad_right = m_pads[1];
        } else if (input->shape.size() == 4) {
            d.in_h = input->shape[1];
            d.in_w = input->shape[2];
            d.in_c = input->shape[3];
            d.out_c = output->shape[3];
            d.k_h = filter->shape[0];
            d.k_w = filter->shape[1];
            d.stride_h = m_strides[0];
            d.stride_w = m_strides[1];
            d.dil_h = m_dilations[0];
            d.dil_w = m_dilations[1];
            d.pad_top = m_pads[0];
            d.pad_bottom = m_pads[1];
            d.pad_left = m_pads[2];
            d.pad_right = m_pads[3];
        } else {
            DL_LOGE("Conv", "Do not support input shape.");
            return;
        }
        d.group = m_group == 1 ? 1 : d.in_c;
        d.in_pitch = input->is_dense() ? 0 : input->channel_pitch;
        d.out_pitch = output->is_dense() ? 0 : output->channel_pitch;
        d.activation = activation == ReLU ? ESPDL_HIP_RELU : ESPDL_HIP_LINEAR;
        if (activation != Linear && activation != ReLU) {
            DL_LOGE("Conv", "%s: only Linear and ReLU can be fused into Conv", name.c_str());
            return;
        }
        d.round_mode = context->round_mode == ROUND_MODE_HALF_EVEN ? ESPDL_HIP_ROUND_HALF_EVEN : ESPDL_HIP_ROUND_HALF_UP;
        if (m_has_gap) {
            const std::vector<int32_t> gs = conv_shifts(m_gap_in_exponent, input, filter, d.out_c);
            d.n_shift = (int32_t)gs.size();
            const int rc = espdl_hip_conv2d_gap_s8(&d, static_cast<const int8_t *>(input->data),
                                                   static_cast<const int8_t *>(filter->data),
                                                   bias ? static_cast<const int32_t *>(bias->data) : nullptr, m_shift.sync(gs),
                                                   m_gap_in_exponent, output->exponent.get(),
                                                   static_cast<int8_t *>(output->data), context->stream);
            if (rc != ESPDL_HIP_OK)
                DL_LOGE("Conv", "%s: %s", name.c_str(), espdl_hip_last_error());
            return;
        }
        const std::vector<int32_t> shifts =
            conv_shifts(m_fused_lut ? m_lut_in_exponent
                                    : (m_has_pre_add_exponent ? m_pre_add_exponent : output->exponent.get()),
                        input, filter, d.out_c);
        d.n_shift = (int32_t)shifts.size();
        const int32_t *shift_dev = m_shift.sync(shifts);
        if (m_fused_lut && !m_fused_lut->on_device()) {
            TensorBase *dev = m_fused_lut->to_device(context->stream);
            delete m_fused_lut;
            m_fused_lut = dev;
        }
        TensorBase *residual = m_residual_pos >= 0 ? context->get_tensor(m_inputs_index[m_residual_pos]) : nullptr;
        if (residual && !residual->on_device()) {
            DL_LOGE("Conv", "%s: the residual must be a device tensor", name.c_str());
            return;
        }
        d.res_pitch = residual && !residual->is_dense() ? residual->channel_pitch : 0;
        const int rc = espdl_hip_conv2d_add(&d, input->data, filter->data, bias ? bias->data : nullptr, shift_dev,
                                            m_fused_lut ? static_cast<const int8_t *>(m_fused_lut->data) : nullptr,
                                            residual ? static_cast<const int8_t *>(residual->data) : nullptr, output->data,
                                            context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Conv", "%s: %s", name.c_str(), espdl_hip_last_error());
    }

    /// depthwise -> 1x1 project [-> Add] through espdl_hip_mbconv_s8 (has_expand = 0)
    void forward_with_project(ModelContext *context, TensorBase *input, TensorBase *filter, TensorBase *bias,
                              TensorBase *output)
    {
        TensorBase *pfilter = context->get_tensor(m_inputs_index[m_project_filter_pos]);
        TensorBase *pbias = m_project_bias_pos >= 0 ? context->get_tensor(m_inputs_index[m_project_bias_pos]) : nullptr;
        TensorBase *residual = m_residual_pos >= 0 ? context->get_tensor(m_inputs_index[m_residual_pos]) : nullptr;
        TensorBase *efilter = m_has_expand ? context->get_tensor(m_inputs_index[m_expand_filter_pos]) : nullptr;
        TensorBase *ebias = m_expand_bias_pos >= 0 ? context->get_tensor(m_inputs_index[m_expand_bias_pos]) : nullptr;
        if (!input || !filter || !output || !pfilter || !input->on_device() || !filter->on_device() ||
            !output->on_device() || !pfilter->on_device() || (bias && !bias->on_device()) ||
            (pbias && !pbias->on_device()) || (residual && !residual->on_device()) || input->shape.size() != 4 ||
            (m_has_expand && (!efilter || !efilter->on_device())) || (ebias && !ebias->on_device())) {
            DL_LOGE("Conv", "%s: fused depthwise+project needs 4-D device tensors", name.c_str());
            return;
        }
        espdl_hip_mbconv_desc d = {};
        d.batch = input->shape[0];
        d.in_h = input->shape[1];
        d.in_w = input->shape[2];
        d.in_c = input->shape[3];
        d.exp_c = m_has_expand ? pfilter->shape[2] : d.in_c;
        d.out_c = output->shape[3];
        d.has_expand = m_has_expand ? 1 : 0;
        if (expand_has_window()) {
            d.exp_k_h = m_expand_kernel[0];
            d.exp_k_w = m_expand_kernel[1];
            d.exp_stride_h = m_expand_strides[0];
            d.exp_stride_w = m_expand_strides[1];
            d.exp_pad_top = m_expand_pads[0];
            d.exp_pad_bottom = m_expand_pads[1];
            d.exp_pad_left = m_expand_pads[2];
            d.exp_pad_right = m_expand_pads[3];
        }
        d.act_expand = m_expand_activation == ReLU ? ESPDL_HIP_RELU : ESPDL_HIP_LINEAR;
        d.k_h = filter->shape[0];
        d.k_w = filter->shape[1];
        d.stride_h = m_strides[0];
        d.stride_w = m_strides[1];
        d.dil_h = m_dilations[0];
        d.dil_w = m_dilations[1];
        d.pad_top = m_pads[0];
        d.pad_bottom = m_pads[1];
        d.pad_left = m_pads[2];
        d.pad_right = m_pads[3];
        d.act_dw = activation == ReLU ? ESPDL_HIP_RELU : ESPDL_HIP_LINEAR;
        d.act_project = m_project_activation == ReLU ? ESPDL_HIP_RELU : ESPDL_HIP_LINEAR;
        d.round_mode = context->round_mode == ROUND_MODE_HALF_EVEN ? ESPDL_HIP_ROUND_HALF_EVEN : ESPDL_HIP_ROUND_HALF_UP;
        std::vector<int32_t> s_dw, s_pj, s_ex;
        const int dw_in_exponent = m_has_expand ? m_expand_exponent : input->exponent.get();
        if (filter->exponent.is_per_channel()) {
            for (int c = 0; c < d.exp_c; c++)
                s_dw.push_back(m_mid_exponent - filter->exponent.get(c) - dw_in_exponent);
        } else {
            s_dw.push_back(m_mid_exponent - filter->exponent.get() - dw_in_exponent);
        }
        if (m_has_expand) {
            if (efilter->exponent.is_per_channel()) {
                for (int c = 0; c < d.exp_c; c++)
                    s_ex.push_back(m_expand_exponent - efilter->exponent.get(c) - input->exponent.get());
            } else {
                s_ex.push_back(m_expand_exponent - efilter->exponent.get() - input->exponent.get());
            }
        }
        const int pj_out_exponent = m_has_pre_add_exponent ? m_pre_add_exponent : output->exponent.get();
        if (pfilter->exponent.is_per_channel()) {
            for (int c = 0; c < d.out_c; c++)
                s_pj.push_back(pj_out_exponent - pfilter->exponent.get(c) - m_mid_exponent);
        } else {
            s_pj.push_back(pj_out_exponent - pfilter->exponent.get() - m_mid_exponent);
        }
        d.n_shift_expand = m_has_expand ? (int32_t)s_ex.size() : 1;
        d.n_shift_dw = (int32_t)s_dw.size();
        d.n_shift_project = (int32_t)s_pj.size();
        // a residual operand whose RequantizeLinear the fusion pass absorbed is requantized inside the kernel
        d.residual_shift = residual ? m_residual_shift : 0;
        d.clip_expand = m_has_expand ? m_clip_expand[0] : 0;
        d.clip_expand_min = m_clip_expand[1];
        d.clip_expand_max = m_clip_expand[2];
        d.clip_dw = m_clip_dw[0];
        d.clip_dw_min = m_clip_dw[1];
        d.clip_dw_max = m_clip_dw[2];
        m_fused_kernel = espdl_hip_mbconv_s8_supported(&d);
        espdl_hip_mbconv_weights w = {};
        if (m_has_expand) {
            w.w_expand = static_cast<const int8_t *>(efilter->data);
            w.b_expand = ebias ? static_cast<const int32_t *>(ebias->data) : nullptr;
            w.s_expand = m_shift_expand.sync(s_ex);
        }
        w.w_dw = static_cast<const int8_t *>(filter->data);
        w.b_dw = bias ? static_cast<const int32_t *>(bias->data) : nullptr;
        w.s_dw = m_shift.sync(s_dw);
        w.w_project = static_cast<const int8_t *>(pfilter->data);
        w.b_project = pbias ? static_cast<const int32_t *>(pbias->data) : nullptr;
        w.s_project = m_shift_project.sync(s_pj);
        const int rc = espdl_hip_mbconv_s8(&d, static_cast<const int8_t *>(input->data), &w,
                                           residual ? static_cast<const int8_t *>(residual->data) : nullptr,
                                           static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Conv", "%s: %s", name.c_str(), espdl_hip_last_error());
    }

    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        Module *conv_op = nullptr;
        std::vector<int> pads, strides, dilations;
        int group = 1;
        activation_type_t activation_type = Linear;
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "pads", pads);
        fbs_model->get_operation_attribute(node_name, "strides", strides);
        fbs_model->get_operation_attribute(node_name, "dilations", dilations);
        fbs_model->get_operation_attribute(node_name, "group", group);
        fbs_model->get_operation_attribute(node_name, "activation", activation_type);
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        if (quant_type == QUANT_TYPE_SYMM_8BIT || quant_type == QUANT_TYPE_SYMM_16BIT) {
            if (pads.size() == 4)
                pads = {pads[0], pads[2], pads[1], pads[3]}; // ONNX [t,l,b,r] -> [t,b,l,r]
            else if (pads.size() == 0)
                pads = {0, 0, 0, 0};
            if (strides.empty())
                strides = {1, 1};
            if (dilations.empty())
                dilations = {1, 1};
            conv_op = new Conv(activation_type, pads, dilations, strides, node_name.c_str(), group, quant_type);
        }
        return conv_op;
    }

    void print()
    {
        DL_LOGI("Conv", "pads: %s, strides: %s, dilations: %s, group: %d, activation: %s, quant_type: %s%s.",
                vector_to_string(m_pads).c_str(), vector_to_string(m_strides).c_str(),
                vector_to_string(m_dilations).c_str(), m_group, activation_type_to_string(activation),
                quant_type_to_string(quant_type), m_fused_lut ? ", fused LUT" : "");
    }
};

} // namespace module
} // namespace dl
