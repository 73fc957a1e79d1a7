// dl::module::Gemm and dl::module::MatMul: y = x * W (+ bias) on the convolution path.
//
// As in the reference (esp-dl/dl/module/include/dl_module_gemm.hpp:17-168;
// dl_module_matmul.hpp:17-193) the input is viewed as {1, 1, M, K}, the filter tensor has shape
// [1, 1, K, N] over N-major memory, and the 1x1 convolution kernel does the work.  Gemm carries a
// bias and Linear/ReLU; MatMul has neither bias nor (in exported models) an activation other than
// Linear.  MatMul is implemented for a constant right-hand side of rank 2 (the weight case).
#pragma once

#include <cassert>

#include "dl_module_conv.hpp"

namespace dl {
namespace module {

inline void gemm_forward(const char *tag, const std::string &name, quant_type_t quant_type,
                         activation_type_t activation, ModelContext *context, TensorBase *input, TensorBase *filter,
                         TensorBase *bias, TensorBase *output, DeviceInts &shift_cache)
{
    if (!input || !filter || !output || !input->on_device() || !filter->on_device() || !output->on_device() ||
        (bias && !bias->on_device())) {
        DL_LOGE(tag, "%s: tensors must be device tensors", name.c_str());
        return;
    }
    const int k = input->shape.back();
    const int n = output->shape.back();
    const int64_t m = input->get_size() / k;
    espdl_hip_conv_desc d = {};
    d.dtype = quant_type == QUANT_TYPE_SYMM_16BIT ? ESPDL_HIP_S16 : ESPDL_HIP_S8;
    d.batch = 1;
    d.in_h = 1;
    d.in_w = (int32_t)m;
    d.in_c = k;
    d.out_c = n;
    d.k_h = d.k_w = d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1;
    d.group = 1;
    d.activation = activation == ReLU ? ESPDL_HIP_RELU : ESPDL_HIP_LINEAR;
    d.round_mode = context->round_mode == ROUND_MODE_HALF_EVEN ? ESPDL_HIP_ROUND_HALF_EVEN : ESPDL_HIP_ROUND_HALF_UP;
    const std::vector<int32_t> shifts = conv_shifts(output, input, filter, n);
    d.n_shift = (int32_t)shifts.size();
    const int32_t *shift_dev = shift_cache.sync(shifts);
    const int rc = espdl_hip_conv2d(&d, input->data, filter->data, bias ? bias->data : nullptr, shift_dev, nullptr,
                                    output->data, context->stream);
    if (rc != ESPDL_HIP_OK)
        DL_LOGE(tag, "%s: %s", name.c_str(), espdl_hip_last_error());
}

class Gemm : public Module {
private:
    activation_type_t activation;
    DeviceInts m_shift;

public:
    Gemm(activation_type_t activation = Linear, const char *name = nullptr, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), activation(activation)
    {
    }

    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        std::vector<int> filter_shape = input_shapes[1];
        if (input_shapes[0].empty() || filter_shape.size() != 4 || filter_shape[0] != 1 || filter_shape[1] != 1 ||
            input_shapes[0].back() != filter_shape[2])
            return {{}}; // an empty shape makes Model::build fail with the node's name
        std::vector<int> output_shape = input_shapes[0];
        output_shape.back() = filter_shape[3];
        return {output_shape};
    }

    int64_t get_macs(std::vector<std::vector<int>> &input_shapes)
    {
        int64_t m = 1;
        for (size_t i = 0; i + 1 < input_shapes[0].size(); i++)
            m *= input_shapes[0][i];
        return m * input_shapes[1][2] * input_shapes[1][3];
    }

    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *bias = m_inputs_index.size() == 3 ? context->get_tensor(m_inputs_index[2]) : nullptr;
        gemm_forward("Gemm", name, quant_type, activation, context, context->get_tensor(m_inputs_index[0]),
                     context->get_tensor(m_inputs_index[1]), bias, context->get_tensor(m_outputs_index[0]), m_shift);
    }

    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        activation_type_t activation_type = Linear;
        quant_type_t quant_type = QUANT_TYPE_NONE;
        int transA = -1, transB = -1;
        fbs_model->get_operation_attribute(node_name, "activation", activation_type);
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "transA", transA);
        fbs_model->get_operation_attribute(node_name, "transB", transB);
        if ((transA != -1 && transA != 0) || (transB != -1 && transB != 0)) {
            DL_LOGE("Gemm", "%s: transA/transB must be 0", node_name.c_str());
            return nullptr;
        }
        if (quant_type == QUANT_TYPE_SYMM_8BIT || quant_type == QUANT_TYPE_SYMM_16BIT)
            return new Gemm(activation_type, node_name.c_str(), quant_type);
        return nullptr;
    }

    void print()
    {
        DL_LOGI("Gemm", "activation: %s, quant_type: %s.", activation_type_to_string(activation),
                quant_type_to_string(quant_type));
    }
};

class MatMul : public Module {
private:
    activation_type_t m_activation;
    DeviceInts m_shift;

public:
    MatMul(activation_type_t activation = Linear, const char *name = nullptr,
           quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type), m_activation(activation)
    {
    }

    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &a = input_shapes[0], &b = input_shapes[1];
        if (batched_rhs(b)) {
            // both operands carry leading dims: numpy-style broadcast of up to two of them
            // (esp-dl/dl/module/include/dl_module_matmul.hpp: the rank-3 and rank-4 branches)
            if (a.size() < 2 || a.size() > 4 || a.back() != b[b.size() - 2])
                return {{}};
            int la[2], lb[2];
            leading(a, la);
            leading(b, lb);
            for (int i = 0; i < 2; i++)
                if (la[i] != lb[i] && la[i] != 1 && lb[i] != 1)
                    return {{}};
            std::vector<int> out;
            const size_t rank = std::max(a.size(), b.size());
            if (rank == 4)
                out.push_back(std::max(la[0], lb[0]));
            out.push_back(std::max(la[1], lb[1]));
            out.push_back(a[a.size() - 2]);
            out.push_back(b.back());
            return {out};
        }
        // right-hand side: [K, N] matrix, or the [1, 1, K, N] filter view of it
        const int k = b.size() == 4 ? b[2] : b[0];
        const int n = b.size() == 4 ? b[3] : (b.size() == 2 ? b[1] : 1);
        assert(a.back() == k);
        (void)k;
        std::vector<int> out = a;
        out.back() = n;
        return {out};
    }

    int64_t get_macs(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> out = get_output_shape(input_shapes)[0];
        if (out.empty() || input_shapes[0].empty())
            return 0;
        int64_t total = input_shapes[0].back(); // k multiply-accumulates per output element
        for (int d : out)
            total *= d;
        return total;
    }

    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *rhs = context->get_tensor(m_inputs_index[1]);
        if (rhs && m_inputs_index[1] < CONTEXT_PARAMETER_OFFSET) {
            forward_activations(context, context->get_tensor(m_inputs_index[0]), rhs,
                                context->get_tensor(m_outputs_index[0]));
            return;
        }
        if (!rhs || (rhs->shape.size() != 2 && rhs->shape.size() != 4)) {
            DL_LOGE("MatMul", "%s: a constant right-hand side must have rank 2 (or its rank-4 filter view)", name.c_str());
            return;
        }
        gemm_forward("MatMul", name, quant_type, m_activation, context, context->get_tensor(m_inputs_index[0]), rhs,
                     nullptr, context->get_tensor(m_outputs_index[0]), m_shift);
    }

    /// True when the right-hand side is a stack of matrices (an activation), not one [K, N] matrix.
    static bool batched_rhs(const std::vector<int> &b)
    {
        return b.size() == 3 || (b.size() == 4 && (b[0] != 1 || b[1] != 1));
    }
    /// The two leading extents of a rank 2..4 operand, padded with 1 in front.
    static void leading(const std::vector<int> &s, int lead[2])
    {
        lead[0] = s.size() == 4 ? s[0] : 1;
        lead[1] = s.size() >= 3 ? s[s.size() - 3] : 1;
    }

    /// Both operands are activations: every pair of matrices runs as the reference's 1x1 convolution
    /// with one shift (espdl_hip_matmul_s8).
    void forward_activations(ModelContext *context, TensorBase *a, TensorBase *b, TensorBase *output)
    {
        if (quant_type != QUANT_TYPE_SYMM_8BIT || !a || !output || !a->on_device() || !b->on_device() ||
            !output->on_device() || a->shape.size() < 2 || a->shape.size() > 4 || b->shape.size() < 2 ||
            b->shape.size() > 4 || a->shape.back() != b->shape[b->shape.size() - 2]) {
            DL_LOGE("MatMul", "%s: two activations need int8 device tensors of rank 2..4 with matching inner extent",
                    name.c_str());
            return;
        }
        int la[2], lb[2];
        leading(a->shape, la);
        leading(b->shape, lb);
        const int32_t m = a->shape[a->shape.size() - 2], k = a->shape.back(), n = b->shape.back();
        const int32_t lead[2] = {std::max(la[0], lb[0]), std::max(la[1], lb[1])};
        const int64_t mk = (int64_t)m * k, kn = (int64_t)k * n;
        const int64_t as[2] = {la[0] == 1 ? 0 : la[1] * mk, la[1] == 1 ? 0 : mk};
        const int64_t bs[2] = {lb[0] == 1 ? 0 : lb[1] * kn, lb[1] == 1 ? 0 : kn};
        const int shift = output->exponent.get() - a->exponent.get() - b->exponent.get();
        const int rc = espdl_hip_matmul_s8(static_cast<const int8_t *>(a->data), static_cast<const int8_t *>(b->data), m, k,
                                           n, lead, as, bs, shift,
                                           m_activation == ReLU ? ESPDL_HIP_RELU : ESPDL_HIP_LINEAR,
                                           context->round_mode == ROUND_MODE_HALF_EVEN ? ESPDL_HIP_ROUND_HALF_EVEN
                                                                                       : ESPDL_HIP_ROUND_HALF_UP,
                                           static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("MatMul", "%s: %s", name.c_str(), espdl_hip_last_error());
    }

    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        activation_type_t activation_type = Linear;
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "activation", activation_type);
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        if (quant_type == QUANT_TYPE_SYMM_8BIT || quant_type == QUANT_TYPE_SYMM_16BIT)
            return new MatMul(activation_type, node_name.c_str(), quant_type);
        return nullptr;
    }

    void print()
    {
        DL_LOGI("MatMul", "activation: %s, quant_type: %s.", activation_type_to_string(m_activation),
                quant_type_to_string(quant_type));
    }
};

} // namespace module
} // namespace dl
