// Bandwidth-bound operator objects: LUT, Relu, PRelu, Clip, Add, GlobalAveragePool,
// RequantizeLinear, Flatten.  Each mirrors the reference module of the same name and enqueues one
// kernel of include/espdl_hip.h on the context's stream.
//   LUT                 esp-dl/dl/module/include/dl_module_lut.hpp:15-104
//   Relu                esp-dl/dl/module/include/dl_module_relu.hpp:13-120
//   PRelu               esp-dl/dl/module/include/dl_module_prelu.hpp:15-160
//   Clip                esp-dl/dl/module/include/dl_module_clip.hpp:12-130
//   Add                 esp-dl/dl/module/include/dl_module_add.hpp:12-110
//   GlobalAveragePool   esp-dl/dl/module/include/dl_module_global_avg_pool.hpp
//   RequantizeLinear    esp-dl/dl/module/include/dl_module_requantize_linear.hpp (runs TensorBase::assign)
//   Flatten             esp-dl/dl/module/include/dl_module_flatten.hpp
// Activation-like ops whose node carries a `lut` attribute deserialize into a LUT module, as in the
// reference (esp-dl/dl/module/include/dl_module_clip.hpp:95-113).
#pragma once

#include <algorithm>
#include <cassert>
#include <limits>

#include "dl_module_base.hpp"
#include "espdl_hip.h"

namespace dl {
namespace module {

inline bool on_device_all(std::initializer_list<TensorBase *> ts)
{
    for (TensorBase *t : ts)
        if (!t || !t->on_device())
            return false;
    return true;
}

class LUT : public Module {
private:
    TensorBase *table; ///< 256 int8 entries, exponent == output exponent (owned)

public:
    LUT(const char *name = nullptr, TensorBase *table = nullptr,
        module_inplace_t inplace = MODULE_INPLACE_CHANGED_BUFFER, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, inplace, quant_type), table(table)
    {
    }
    ~LUT() { delete table; }

    /// Hand the table over (for fusing this LUT into the producing Conv); the module keeps nothing.
    TensorBase *release_table()
    {
        TensorBase *t = table;
        table = nullptr;
        return t;
    }
    TensorBase *get_table() { return table; }

    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        return {input_shapes[0]};
    }

    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (quant_type == QUANT_TYPE_SYMM_16BIT) {
            forward_s16(context, input, output);
            return;
        }
        if (quant_type != QUANT_TYPE_SYMM_8BIT) {
            DL_LOGE("LUT", "%s: only 8-bit and 16-bit tables are implemented", name.c_str());
            return;
        }
        if (!table || table->get_size() != 256 || !on_device_all({input, output})) {
            DL_LOGE("LUT", "%s: needs a 256-entry table and device tensors", name.c_str());
            return;
        }
        if (!table->on_device()) {
            TensorBase *dev = table->to_device(context->stream);
            delete table;
            table = dev;
        }
        const int rc = espdl_hip_lut_s8(static_cast<const int8_t *>(input->data), input->get_size(),
                                        static_cast<const int8_t *>(table->data), static_cast<int8_t *>(output->data),
                                        context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("LUT", "%s: %s", name.c_str(), espdl_hip_last_error());
    }

    /// int16: the table samples the function every 65536 / (entries - 1) input steps and the nearest entry is
    /// taken (esp-dl/dl/module/include/dl_module_lut.hpp:61-74); the ESP32-P4 tie rule goes with the
    /// context's half-even mode.
    void forward_s16(ModelContext *context, TensorBase *input, TensorBase *output)
    {
        if (!table || table->dtype != DATA_TYPE_INT16 || !on_device_all({input, output}) ||
            input->dtype != DATA_TYPE_INT16 || output->dtype != DATA_TYPE_INT16) {
            DL_LOGE("LUT", "%s: the 16-bit form needs an int16 table and int16 device tensors", name.c_str());
            return;
        }
        if (!table->on_device()) {
            TensorBase *dev = table->to_device(context->stream);
            delete table;
            table = dev;
        }
        const int rc = espdl_hip_lut_s16(static_cast<const int16_t *>(input->data), input->get_size(),
                                         static_cast<const int16_t *>(table->data), table->get_size(),
                                         context->round_mode == ROUND_MODE_HALF_EVEN ? ESPDL_HIP_ROUND_HALF_EVEN
                                                                                     : ESPDL_HIP_ROUND_HALF_UP,
                                         static_cast<int16_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("LUT", "%s: %s", name.c_str(), espdl_hip_last_error());
    }

    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        TensorBase *table = fbs_model->get_operation_lut(node_name);
        if (table == nullptr) {
            DL_LOGE("LUT", "Table is null!");
            return nullptr;
        }
        if (quant_type == QUANT_TYPE_SYMM_8BIT || (quant_type == QUANT_TYPE_SYMM_16BIT && table->dtype == DATA_TYPE_INT16))
            return new LUT(node_name.c_str(), table, MODULE_INPLACE_CHANGED_BUFFER, quant_type);
        DL_LOGE("LUT", "Only 8-bit tables and int16 tables of 16-bit nodes are implemented");
        delete table;
        return nullptr;
    }

    void print() { DL_LOGI("LUT", "quant_type: %s.", quant_type_to_string(quant_type)); }
};

/// Shared by every activation op: a node with a `lut` attribute becomes a LUT module.
inline Module *lut_if_present(fbs::FbsModel *fbs_model, const std::string &node_name, quant_type_t quant_type)
{
    if (quant_type != QUANT_TYPE_SYMM_8BIT && quant_type != QUANT_TYPE_SYMM_16BIT)
        return nullptr;
    TensorBase *table = fbs_model->get_operation_lut(node_name);
    if (table && quant_type == QUANT_TYPE_SYMM_16BIT && table->dtype != DATA_TYPE_INT16) {
        delete table;
        return nullptr;
    }
    return table ? new LUT(node_name.c_str(), table, MODULE_INPLACE_CHANGED_BUFFER, quant_type) : nullptr;
}

class Relu : public Module {
public:
    Relu(const char *name = nullptr, module_inplace_t inplace = MODULE_INPLACE_CHANGED_BUFFER,
         quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, inplace, quant_type)
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
        if (quant_type != QUANT_TYPE_SYMM_8BIT || !on_device_all({input, output})) {
            DL_LOGE("Relu", "%s: needs int8 device tensors", name.c_str());
            return;
        }
        const int rc = espdl_hip_relu_s8(static_cast<const int8_t *>(input->data), input->get_size(),
                                         input->exponent.get(), output->exponent.get(),
                                         static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Relu", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        Module *op = lut_if_present(fbs_model, node_name, quant_type);
        return op ? op : new Relu(node_name.c_str(), MODULE_INPLACE_CHANGED_BUFFER, quant_type);
    }
    void print() { DL_LOGI("Relu", "quant_type: %s.", quant_type_to_string(quant_type)); }
};

class PRelu : public Module {
private:
    TensorBase *m_alpha; ///< int8 slope per channel, shape [C,1,1] or [1] (owned)

public:
    PRelu(const char *name = nullptr, TensorBase *alpha = nullptr, module_inplace_t inplace = MODULE_NON_INPLACE,
          quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, inplace, quant_type), m_alpha(alpha)
    {
    }
    ~PRelu() { delete m_alpha; }

    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        return {input_shapes[0]};
    }

    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (quant_type != QUANT_TYPE_SYMM_8BIT || !m_alpha || !on_device_all({input, output})) {
            DL_LOGE("PRelu", "%s: needs int8 device tensors and an alpha", name.c_str());
            return;
        }
        const int channels = input->shape.back();
        if (m_alpha->get_size() != channels) {
            // a single slope is broadcast to every channel (dl_module_prelu.hpp:43-62)
            TensorBase *host = m_alpha->on_device() ? m_alpha->to_host(context->stream) : m_alpha;
            std::vector<int8_t> spread(channels, host->get_element<int8_t>(0));
            TensorBase *wide = new TensorBase({channels, 1, 1}, spread.data(), m_alpha->exponent.get(), DATA_TYPE_INT8,
                                              true, MALLOC_CAP_DEVICE);
            if (host != m_alpha)
                delete host;
            delete m_alpha;
            m_alpha = wide;
        }
        if (!m_alpha->on_device()) {
            TensorBase *dev = m_alpha->to_device(context->stream);
            delete m_alpha;
            m_alpha = dev;
        }
        const int shift = output->exponent.get() - input->exponent.get() - m_alpha->exponent.get();
        const int rc = espdl_hip_prelu_s8(static_cast<const int8_t *>(input->data), input->get_size() / channels,
                                          channels, static_cast<const int8_t *>(m_alpha->data), shift,
                                          static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("PRelu", "%s: %s", name.c_str(), espdl_hip_last_error());
    }

    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        Module *op = lut_if_present(fbs_model, node_name, quant_type);
        if (op)
            return op;
        TensorBase *alpha = fbs_model->get_operation_parameter(node_name, 1);
        if (!alpha) {
            DL_LOGE("PRelu", "%s: slope tensor missing", node_name.c_str());
            return nullptr;
        }
        return new PRelu(node_name.c_str(), alpha, MODULE_INPLACE_CHANGED_BUFFER, quant_type);
    }
    void print() { DL_LOGI("PRelu", "quant_type: %s.", quant_type_to_string(quant_type)); }
};

class Clip : public Module {
public:
    Clip(const char *name = nullptr, module_inplace_t inplace = MODULE_NON_INPLACE,
         quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, inplace, quant_type)
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
        if (quant_type != QUANT_TYPE_SYMM_8BIT || !on_device_all({input, output})) {
            DL_LOGE("Clip", "%s: needs int8 device tensors", name.c_str());
            return;
        }
        read_bounds(context);
        const int rc = espdl_hip_clip_s8(static_cast<const int8_t *>(input->data), input->get_size(), m_min, m_max,
                                         input->exponent.get(), output->exponent.get(),
                                         static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Clip", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        Module *op = lut_if_present(fbs_model, node_name, quant_type);
        return op ? op : new Clip(node_name.c_str(), MODULE_INPLACE_CHANGED_BUFFER, quant_type);
    }
    void print() { DL_LOGI("Clip", "quant_type: %s.", quant_type_to_string(quant_type)); }

    /// min / max are quantized scalars held as parameters (read once, on the host); also what a fusion pass
    /// asks for when it folds the clamp into the convolution in front
    void read_bounds(ModelContext *context)
    {
        if (m_bounds_read)
            return;
        m_min = std::numeric_limits<int8_t>::min();
        m_max = std::numeric_limits<int8_t>::max();
        for (size_t i = 1; i < m_inputs_index.size() && i < 3; i++) {
            TensorBase *b = context->get_tensor(m_inputs_index[i]);
            if (!b)
                continue;
            TensorBase *host = b->on_device() ? b->to_host(context->stream) : b;
            (i == 1 ? m_min : m_max) = host->get_element<int8_t>(0);
            if (host != b)
                delete host;
        }
        m_bounds_read = true;
    }
    int get_min() const { return m_min; }
    int get_max() const { return m_max; }

private:
    bool m_bounds_read = false;
    int m_min = -128, m_max = 127;
};

class Add : public Module {
public:
    Add(const char *name = nullptr, module_inplace_t inplace = MODULE_NON_INPLACE,
        quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, inplace, quant_type)
    {
    }

    /// numpy-style broadcast of the two shapes (get_elemwise_operation_args merges dims the same way,
    /// esp-dl/dl/base/dl_base_elemwise.cpp:38-178)
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &a = input_shapes[0], &b = input_shapes[1];
        const size_t rank = std::max(a.size(), b.size());
        std::vector<int> out(rank, 1);
        for (size_t i = 0; i < rank; i++) {
            const int da = i < rank - a.size() ? 1 : a[i - (rank - a.size())];
            const int db = i < rank - b.size() ? 1 : b[i - (rank - b.size())];
            assert(da == db || da == 1 || db == 1);
            out[i] = std::max(da, db);
        }
        return {out};
    }

    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input0 = context->get_tensor(m_inputs_index[0]);
        TensorBase *input1 = context->get_tensor(m_inputs_index[1]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if ((quant_type != QUANT_TYPE_SYMM_8BIT && quant_type != QUANT_TYPE_SYMM_16BIT) ||
            !on_device_all({input0, input1, output}) || output->shape.size() > 4) {
            DL_LOGE("Add", "%s: needs int8 or int16 device tensors of rank <= 4", name.c_str());
            return;
        }
        int32_t dims[4];
        int64_t s0[4], s1[4];
        broadcast_layout(input0, input1, output, dims, s0, s1);
        const int rc = quant_type == QUANT_TYPE_SYMM_16BIT
            ? espdl_hip_add_s16(dims, s0, s1, static_cast<const int16_t *>(input0->data),
                                static_cast<const int16_t *>(input1->data), static_cast<int16_t *>(output->data),
                                context->stream)
            : espdl_hip_add_s8(dims, s0, s1, static_cast<const int8_t *>(input0->data),
                               static_cast<const int8_t *>(input1->data), static_cast<int8_t *>(output->data),
                               context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Add", "%s: %s", name.c_str(), espdl_hip_last_error());
    }

    /// Output extents padded to 4 dims and element strides of both inputs per output dim (0 = broadcast).
    static void broadcast_layout(TensorBase *input0, TensorBase *input1, TensorBase *output, int32_t dims[4],
                                 int64_t s0[4], int64_t s1[4])
    {
        const size_t rank = output->shape.size();
        for (int i = 0; i < 4; i++) {
            dims[i] = 1;
            s0[i] = s1[i] = 0;
        }
        for (size_t i = 0; i < rank; i++)
            dims[4 - rank + i] = output->shape[i];
        auto strides = [&](TensorBase *t, int64_t *s) {
            const size_t r = t->shape.size();
            int64_t acc = 1;
            for (int i = (int)r - 1; i >= 0; i--) {
                s[4 - r + i] = t->shape[i] == 1 ? 0 : acc;
                acc *= t->shape[i];
            }
        };
        strides(input0, s0);
        strides(input1, s1);
    }

    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        return new Add(node_name.c_str(), MODULE_INPLACE_CHANGED_BUFFER, quant_type);
    }
    void print() { DL_LOGI("Add", "quant_type: %s.", quant_type_to_string(quant_type)); }
};

/// Mul with numpy-style broadcasting (esp-dl/dl/module/include/dl_module_mul.hpp, base::elemwise_mul).
/// Rounds like the rest of the model: half up for the portable C path, half even when the context
/// runs ESP32-P4 semantics (the P4 kernels of this operator set the hardware rounding that way).
class Mul : public Add {
public:
    Mul(const char *name = nullptr, module_inplace_t inplace = MODULE_NON_INPLACE,
        quant_type_t quant_type = QUANT_TYPE_NONE) :
        Add(name, inplace, quant_type)
    {
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input0 = context->get_tensor(m_inputs_index[0]);
        TensorBase *input1 = context->get_tensor(m_inputs_index[1]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if ((quant_type != QUANT_TYPE_SYMM_8BIT && quant_type != QUANT_TYPE_SYMM_16BIT) ||
            !on_device_all({input0, input1, output}) || output->shape.size() > 4) {
            DL_LOGE("Mul", "%s: needs int8 or int16 device tensors of rank <= 4", name.c_str());
            return;
        }
        int32_t dims[4];
        int64_t s0[4], s1[4];
        broadcast_layout(input0, input1, output, dims, s0, s1);
        const int shift = output->exponent.get() - input0->exponent.get() - input1->exponent.get();
        const int32_t rm = context->round_mode == ROUND_MODE_HALF_EVEN ? ESPDL_HIP_ROUND_HALF_EVEN : ESPDL_HIP_ROUND_HALF_UP;
        const int rc = quant_type == QUANT_TYPE_SYMM_16BIT
            ? espdl_hip_mul_s16(dims, s0, s1, static_cast<const int16_t *>(input0->data),
                                static_cast<const int16_t *>(input1->data), shift, rm,
                                static_cast<int16_t *>(output->data), context->stream)
            : espdl_hip_mul_s8(dims, s0, s1, static_cast<const int8_t *>(input0->data),
                               static_cast<const int8_t *>(input1->data), shift, rm, static_cast<int8_t *>(output->data),
                               context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("Mul", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        return new Mul(node_name.c_str(), MODULE_INPLACE_CHANGED_BUFFER, quant_type);
    }
    void print() { DL_LOGI("Mul", "quant_type: %s.", quant_type_to_string(quant_type)); }
};

/// Sub and Div on int16 tensors with numpy-style broadcasting (esp-dl/dl/module/include/dl_module_sub.hpp,
/// dl_module_div.hpp over base::elemwise_sub / base::elemwise_div).
class SubDiv : public Add {
private:
    bool m_div;

public:
    SubDiv(bool div, const char *name = nullptr, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Add(name, MODULE_NON_INPLACE, quant_type), m_div(div)
    {
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input0 = context->get_tensor(m_inputs_index[0]);
        TensorBase *input1 = context->get_tensor(m_inputs_index[1]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        const char *tag = m_div ? "Div" : "Sub";
        const bool s8 = quant_type == QUANT_TYPE_SYMM_8BIT;
        if ((!s8 && quant_type != QUANT_TYPE_SYMM_16BIT) || !on_device_all({input0, input1, output}) ||
            output->shape.size() > 4) {
            DL_LOGE(tag, "%s: needs int8 or int16 device tensors of rank <= 4", name.c_str());
            return;
        }
        int32_t dims[4];
        int64_t s0[4], s1[4];
        broadcast_layout(input0, input1, output, dims, s0, s1);
        const int div_shift = output->exponent.get() - input0->exponent.get() + input1->exponent.get();
        int rc;
        if (s8) {
            const int8_t *a = static_cast<const int8_t *>(input0->data), *b = static_cast<const int8_t *>(input1->data);
            int8_t *y = static_cast<int8_t *>(output->data);
            rc = m_div ? espdl_hip_div_s8(dims, s0, s1, a, b, div_shift, y, context->stream)
                       : espdl_hip_sub_s8(dims, s0, s1, a, b, y, context->stream);
        } else {
            const int16_t *a = static_cast<const int16_t *>(input0->data),
                          *b = static_cast<const int16_t *>(input1->data);
            int16_t *y = static_cast<int16_t *>(output->data);
            rc = m_div ? espdl_hip_div_s16(dims, s0, s1, a, b, div_shift, y, context->stream)
                       : espdl_hip_sub_s16(dims, s0, s1, a, b, y, context->stream);
        }
        if (rc != ESPDL_HIP_OK)
            DL_LOGE(tag, "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize_sub(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        return new SubDiv(false, node_name.c_str(), quant_type);
    }
    static Module *deserialize_div(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        return new SubDiv(true, node_name.c_str(), quant_type);
    }
    void print() { DL_LOGI(m_div ? "Div" : "Sub", "quant_type: %s.", quant_type_to_string(quant_type)); }
};

class GlobalAveragePool : public Module {
public:
    GlobalAveragePool(const char *name = nullptr, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_NON_INPLACE, quant_type)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        assert(input_shapes[0].size() == 4);
        return {{input_shapes[0][0], 1, 1, input_shapes[0][3]}};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (quant_type != QUANT_TYPE_SYMM_8BIT || !on_device_all({input, output}) || input->shape.size() != 4) {
            DL_LOGE("GlobalAveragePool", "%s: needs int8 NHWC device tensors", name.c_str());
            return;
        }
        const int rc = espdl_hip_global_avg_pool_s8(static_cast<const int8_t *>(input->data), input->shape[0],
                                                    input->shape[1], input->shape[2], input->shape[3],
                                                    input->exponent.get(), output->exponent.get(),
                                                    static_cast<int8_t *>(output->data), context->stream);
        if (rc != ESPDL_HIP_OK)
            DL_LOGE("GlobalAveragePool", "%s: %s", name.c_str(), espdl_hip_last_error());
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        return new GlobalAveragePool(node_name.c_str(), quant_type);
    }
    void print() { DL_LOGI("GlobalAveragePool", "quant_type: %s.", quant_type_to_string(quant_type)); }
};

class RequantizeLinear : public Module {
public:
    RequantizeLinear(const char *name = nullptr, module_inplace_t inplace = MODULE_NON_INPLACE,
                     quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, inplace, quant_type)
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
        if (!on_device_all({input, output}) || !output->assign(input, context->stream))
            DL_LOGE("RequantizeLinear", "%s: assign failed", name.c_str());
    }
    /// int8 -> int8 goes row by row when either side is a channel slice of a wider tensor; a model only makes such
    /// slices where both sides are int8 (TensorBase::assign handles nothing else with a pitch on the output).
    bool reads_channel_slice(int slot) const { return slot == 0 && quant_type == QUANT_TYPE_SYMM_8BIT; }
    bool writes_channel_slice(int slot) const { return slot == 0 && quant_type == QUANT_TYPE_SYMM_8BIT; }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        return new RequantizeLinear(node_name.c_str(), MODULE_INPLACE_CHANGED_BUFFER, quant_type);
    }
    void print() { DL_LOGI("RequantizeLinear", "quant_type: %s.", quant_type_to_string(quant_type)); }
};

/// Flatten to [N, rest]: a view, no bytes move (the planner aliases output onto input).
class Flatten : public Module {
private:
    int m_axis;

public:
    Flatten(const char *name = nullptr, int axis = 1, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_INPLACE_UNCHANGED_BUFFER, quant_type), m_axis(axis)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        int axis = m_axis < 0 ? m_axis + (int)in.size() : m_axis;
        int outer = 1, inner = 1;
        for (int i = 0; i < (int)in.size(); i++)
            (i < axis ? outer : inner) *= in[i];
        return {{outer, inner}};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (input && output && input->data != output->data)
            output->copy_from(input, context->stream);
    }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        int axis = 1;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, "axis", axis);
        return new Flatten(node_name.c_str(), axis, quant_type);
    }
    void print() { DL_LOGI("Flatten", "axis: %d, quant_type: %s.", m_axis, quant_type_to_string(quant_type)); }
};

/// Squeeze / Unsqueeze / Reshape: views that only change the shape (no bytes move).
///   esp-dl/dl/module/include/dl_module_squeeze.hpp, dl_module_unsqueeze.hpp, dl_module_reshape.hpp
class ShapeView : public Module {
public:
    enum Kind { SQUEEZE, UNSQUEEZE, RESHAPE };

private:
    Kind m_kind;
    std::vector<int> m_arg; ///< axes (Squeeze / Unsqueeze) or the per-image target shape with leading 1 (Reshape)
    bool m_allowzero = false;

public:
    ShapeView(const char *name, Kind kind, std::vector<int> arg, quant_type_t quant_type = QUANT_TYPE_NONE) :
        Module(name, MODULE_INPLACE_UNCHANGED_BUFFER, quant_type), m_kind(kind), m_arg(arg)
    {
    }
    std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes)
    {
        const std::vector<int> &in = input_shapes[0];
        std::vector<int> out;
        const int rank = (int)in.size();
        if (m_kind == SQUEEZE) {
            for (int i = 0; i < rank; i++) {
                bool drop = false;
                for (int a : m_arg)
                    if ((a < 0 ? a + rank : a) == i && in[i] == 1)
                        drop = true;
                // no axes: every extent-1 dimension goes, the leading one included when the batch is 1
                // (esp-dl/dl/module/include/dl_module_squeeze.hpp:37-41)
                if (m_arg.empty() && in[i] == 1)
                    drop = true;
                if (!drop)
                    out.push_back(in[i]);
            }
        } else if (m_kind == UNSQUEEZE) {
            const int out_rank = rank + (int)m_arg.size();
            int src = 0;
            for (int i = 0; i < out_rank; i++) {
                bool ins = false;
                for (int a : m_arg)
                    if ((a < 0 ? a + out_rank : a) == i)
                        ins = true;
                out.push_back(ins ? 1 : in[src++]);
            }
        } else {
            // The target shape is used as written, with the reference's two rules: a 0 copies the
            // input extent unless allowzero is set, one -1 is inferred from the element count
            // (esp-dl/dl/module/include/dl_module_reshape.hpp:36-75).  Exported targets describe one
            // image (leading 1); only that leading 1 is replaced by the batch.  A target that folds the
            // leading dimension into something else is valid for a batch of one only; anything whose
            // element count differs from the input's has no output shape, so that build() fails.
            int64_t total = 1, known = 1;
            for (int d : in)
                total *= d;
            out = m_arg;
            for (size_t i = 0; i < out.size(); i++)
                if (out[i] == 0 && !m_allowzero && i < in.size())
                    out[i] = in[i];
            if (!out.empty() && out[0] == 1 && !in.empty())
                out[0] = in[0];
            int infer = -1;
            for (size_t i = 0; i < out.size(); i++) {
                if (out[i] == -1) {
                    if (infer >= 0)
                        return {{}};
                    infer = (int)i;
                } else {
                    known *= out[i];
                }
            }
            if (infer >= 0) {
                if (known <= 0 || total % known != 0)
                    return {{}};
                out[infer] = (int)(total / known);
                known *= out[infer];
            }
            if (known != total)
                return {{}};
        }
        return {out};
    }
    void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO)
    {
        (void)mode;
        TensorBase *input = context->get_tensor(m_inputs_index[0]);
        TensorBase *output = context->get_tensor(m_outputs_index[0]);
        if (input && output && input->data != output->data)
            output->copy_from(input, context->stream);
    }
    static Module *deserialize_squeeze(fbs::FbsModel *fbs_model, std::string node_name)
    {
        return make(fbs_model, node_name, SQUEEZE, "axes");
    }
    static Module *deserialize_unsqueeze(fbs::FbsModel *fbs_model, std::string node_name)
    {
        return make(fbs_model, node_name, UNSQUEEZE, "axes");
    }
    static Module *deserialize_reshape(fbs::FbsModel *fbs_model, std::string node_name)
    {
        return make(fbs_model, node_name, RESHAPE, "shape");
    }
    void print() { DL_LOGI("ShapeView", "kind %d, arg %s.", (int)m_kind, vector_to_string(m_arg).c_str()); }

private:
    static Module *make(fbs::FbsModel *fbs_model, const std::string &node_name, Kind kind, const char *key)
    {
        quant_type_t quant_type = QUANT_TYPE_NONE;
        std::vector<int> arg;
        fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
        fbs_model->get_operation_attribute(node_name, key, arg);
        if (arg.empty()) {
            // exported graphs carry the axes / target shape as the second operand, an integer initializer
            // (esp-dl/dl/module/include/dl_module_reshape.hpp:107-118)
            TensorBase *t = fbs_model->get_operation_parameter(node_name, 1);
            if (t && t->dtype == DATA_TYPE_INT64) {
                const int64_t *p = t->get_element_ptr<int64_t>();
                for (int i = 0; i < t->get_size(); i++)
                    arg.push_back((int)p[i]);
            } else if (t && t->dtype == DATA_TYPE_INT32) {
                const int32_t *p = t->get_element_ptr<int32_t>();
                arg.assign(p, p + t->get_size());
            }
            delete t;
        }
        if (kind == RESHAPE) {
            int allowzero = 0;
            fbs_model->get_operation_attribute(node_name, "allowzero", allowzero);
            if (arg.empty()) {
                DL_LOGE("Reshape", "%s: no target shape (attribute or integer initializer)", node_name.c_str());
                return nullptr;
            }
            ShapeView *op = new ShapeView(node_name.c_str(), kind, arg, quant_type);
            op->m_allowzero = allowzero != 0;
            return op;
        }
        return new ShapeView(node_name.c_str(), kind, arg, quant_type);
    }
};

} // namespace module
} // namespace dl
