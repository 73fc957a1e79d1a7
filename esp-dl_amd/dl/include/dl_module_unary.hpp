// The activation modules that the reference evaluates in float32 element by element, for int8 and int16
// tensors: Sigmoid, Tanh, HardSwish, Elu, Exp, Log, Sqrt, LeakyRelu, Swish, HardSigmoid, and the integer Neg.
// Each of them is a pure function of one stored integer, the two exponents and the attributes, so the module
// evaluates the reference's expression once per possible input on the host (256 or 65536 values, float / double
// promotions as the reference writes them), keeps the table in device memory and runs the table kernels
// (espdl_hip_lut_s8, espdl_hip_lut_s16 with a 65536-entry table).  The result is the reference's for every input;
// the tensor is read once and written once, whatever the function costs.
//   math::sigmoid, math::tanh   esp-dl/dl/math/include/dl_math.hpp:200-208
//   Sigmoid      esp-dl/dl/module/include/dl_module_sigmoid.hpp:27-103
//   Tanh         esp-dl/dl/module/include/dl_module_tanh.hpp:41-103
//   HardSwish    esp-dl/dl/module/include/dl_module_hard_swish.hpp:40-105
//   Elu          esp-dl/dl/module/include/dl_module_elu.hpp:35-111
//   Exp / Log / Sqrt   dl_module_exp.hpp:36-101, dl_module_log.hpp:36-101, dl_module_sqrt.hpp:36-100
//   LeakyRelu    esp-dl/dl/module/include/dl_module_leaky_relu.hpp:38-118
//   Swish        esp-dl/dl/module/include/dl_module_swish.hpp:40-105
//   HardSigmoid  esp-dl/dl/module/include/dl_module_hard_sigmoid.hpp:40-120
//   Neg          esp-dl/dl/module/include/dl_module_neg.hpp:42-114
//   tool::round  esp-dl/dl/tool/src/dl_tool.cpp:50-91
// A node that carries a `lut` attribute still becomes a LUT module, as in the reference's deserializers.
#pragma once

#include <cmath>
#include <vector>

#include "dl_module_elementwise.hpp"

namespace dl {
namespace module {

enum unary_kind_t {
    UNARY_SIGMOID,
    UNARY_TANH,
    UNARY_HARD_SWISH,
    UNARY_ELU,
    UNARY_EXP,
    UNARY_LOG,
    UNARY_SQRT,
    UNARY_LEAKY_RELU,
    UNARY_NEG,
    UNARY_SWISH,
    UNARY_HARD_SIGMOID,
};

class UnaryMath : public Module {
private:
    unary_kind_t m_kind;
    const char *m_tag;
    float m_alpha, m_beta;
    TensorBase *m_table;                                 ///< device table for the exponents below (owned)
    int m_table_in_exp, m_table_out_exp, m_table_round;  ///< what m_table was built for

    static float sigmoid(float x) { return 1.0 / (1.0 + expf(-x)); }

    /// tool::round of the ESP32-P4 build (round_half_even(double), dl_tool.cpp:50-68)
    static int round_half_even(double value)
    {
        const double rounded = value < 0 ? value - 0.5 : value + 0.5;
        int int_part = (int)rounded;
        if (std::fabs(rounded - int_part) < 1e-6 && (int_part & 1) != 0)
            int_part += value < 0 ? 1 : -1;
        return int_part;
    }

    int entry(int q, float in_scale, float out_scale, bool half_even, int lo, int hi) const
    {
        float temp = (float)q * in_scale, v = 0.f;
        switch (m_kind) {
        case UNARY_SIGMOID:
            v = sigmoid(temp) * out_scale;
            break;
        case UNARY_TANH:
            temp = 2 * sigmoid(2 * temp) - 1;
            v = temp * out_scale;
            break;
        case UNARY_HARD_SWISH:
            temp = DL_MAX(0, DL_MIN(1, 0.166667 * temp + 0.5)) * temp; // double until stored
            v = temp * out_scale;
            break;
        case UNARY_ELU:
            v = temp >= 0 ? temp * out_scale : m_alpha * (expf(temp) - 1) * out_scale;
            break;
        case UNARY_EXP:
            v = expf(temp) * out_scale;
            break;
        case UNARY_LOG:
            v = logf(temp) * out_scale;
            break;
        case UNARY_SQRT:
            v = sqrtf(temp) * out_scale;
            break;
        case UNARY_LEAKY_RELU:
            v = temp >= 0 ? temp * out_scale : temp * out_scale * m_alpha;
            break;
        case UNARY_SWISH:
            temp = sigmoid(temp) * temp;
            v = temp * out_scale;
            break;
        case UNARY_HARD_SIGMOID:
            temp = DL_MAX(0, DL_MIN(1, m_alpha * temp + m_beta));
            v = temp * out_scale;
            break;
        case UNARY_NEG:
            return q == lo ? hi : -q;
        }
        // the reference converts NaN and infinities to int, which is undefined: 0 and saturation here
        if (std::isnan(v))
            return 0;
        if (v >= 2147483520.f)
            return hi;
        if (v <= -2147483520.f)
            return lo;
        const int r = half_even ? round_half_even((double)v) : (int)floorf((float)((double)v + 0.5));
        return DL_CLIP(r, lo, hi);
    }

    template <typename T>
    void build_table(ModelContext *context, int in_exp, int out_exp, bool half_even)
    {
        const int lo = std::numeric_limits<T>::min(), hi = std::numeric_limits<T>::max(), n = hi - lo + 1;
        const float in_scale = DL_SCALE(in_exp), out_scale = DL_RESCALE(out_exp);
        std::vector<T> host(n);
        for (int q = lo; q <= hi; q++)
            host[q - lo] = (T)entry(q, in_scale, out_scale, half_even, lo, hi);
        TensorBase staged({n}, host.data(), out_exp, sizeof(T) == 1 ? DATA_TYPE_INT8 : DATA_TYPE_INT16);
        delete m_table;
        m_table = staged.to_device(context->stream);
        m_table_in_exp = in_exp;
        m_table_out_exp = out_exp;
        m_table_round = half_even;
    }

public:
    UnaryMath(unary_kind_t kind, const char *tag, const char *name, quant_type_t quant_type, float alpha = 0.f,
              float beta = 0.f) :
        Module(name, MODULE_INPLACE_CHANGED_BUFFER, quant_type),
        m_kind(kind),
        m_tag(tag),
        m_alpha(alpha),
        m_beta(beta),
        m_table(nullptr),
        m_table_in_exp(0),
        m_table_out_exp(0),
        m_table_round(-1)
    {
    }
    ~UnaryMath() { delete m_table; }

    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        return {input_shapes[0]};
    }

    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        const bool s8 = quant_type == QUANT_TYPE_SYMM_8BIT, s16 = quant_type == QUANT_TYPE_SYMM_16BIT;
        if ((!s8 && !s16) || !on_device_all({input, output}) || input->get_size() != output->get_size() ||
            input->dtype != (s8 ? DATA_TYPE_INT8 : DATA_TYPE_INT16) || output->dtype != input->dtype) {
            DL_LOGE(m_tag, "%s: needs int8 or int16 device tensors of one size", name.c_str());
            return;
        }
        const int in_exp = input->exponent.get(), out_exp = output->exponent.get();
        const bool half_even = context->round_mode == ROUND_MODE_HALF_EVEN;
        if (!m_table || m_table_in_exp != in_exp || m_table_out_exp != out_exp || m_table_round != (int)half_even) {
            if (s8)
                build_table<int8_t>(context, in_exp, out_exp, half_even);
            else
                build_table<int16_t>(context, in_exp, out_exp, half_even);
        }
        const int rc = s8
            ? espdl_hip_lut_s8(static_cast<const int8_t *>(input->data), input->get_size(),
                               static_cast<const int8_t *>(m_table->data), static_cast<int8_t *>(output->data),
                               context->stream)
            : espdl_hip_lut_s16(static_cast<const int16_t *>(input->data), input->get_size(),
                                static_cast<const int16_t *>(m_table->data), 65536, ESPDL_HIP_ROUND_HALF_UP,
                                static_cast<int16_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE(m_tag, "%s: %s", name.c_str(), espdl_hip_last_error());
    }

    void print() { DL_LOGI(m_tag, "quant_type: %s.", quant_type_to_string(quant_type)); }

    /// One deserializer per operator name; alpha / beta defaults are the reference's.
    template <int KIND>
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        static const struct {
            const char *tag;
            float alpha, beta;
        } info[] = {{"Sigmoid", 0.f, 0.f},   {"Tanh", 0.f, 0.f}, {"HardSwish", 0.f, 0.f},  {"Elu", 1.f, 0.f},
                    {"Exp", 0.f, 0.f},       {"Log", 0.f, 0.f},  {"Sqrt", 0.f, 0.f},       {"LeakyRelu", 0.01f, 0.f},
                    {"Neg", 0.f, 0.f},       {"Swish", 0.f, 0.f}, {"HardSigmoid", 0.2f, 0.5f}};
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        if (KIND != UNARY_NEG)
            if (Module *lut = lut_if_present(fbs_model, node_name, quant_type))
                return lut;
        float alpha = info[KIND].alpha, beta = info[KIND].beta;
        fbs_model->get_operation_attribute(node_name, "alpha", alpha);
        fbs_model->get_operation_attribute(node_name, "beta", beta);
        return new UnaryMath((unary_kind_t)KIND, info[KIND].tag, node_name.c_str(), quant_type, alpha, beta);
    }
};

} // namespace module
} // namespace dl
