// dl::module::ModuleCreator: op-type string -> Module factory registry.
//
// Same contract as esp-dl/dl/module/include/dl_module_creator.hpp:35-205: a singleton,
// register_module(op_type, creator), create(fbs_model, op_type, node_name), and
// register_dl_modules() that installs the built-in operators on first use.  Only the operators on
// the quantized conv/gemm path exist here; the activation-like op types are accepted when their node
// carries a `lut` attribute, in which case they become LUT modules exactly as in the reference.
#pragma once

#include <functional>
#include <map>
#include <string>

#include "dl_module_base.hpp"
#include "dl_module_conv.hpp"
#include "dl_module_elementwise.hpp"
#include "dl_module_gemm.hpp"
#include "dl_module_layout.hpp"
#include "dl_module_unary.hpp"

namespace dl {
namespace module {

class ModuleCreator {
public:
    using Creator = std::function<Module *(fbs::FbsModel *, std::string)>;

    static ModuleCreator *get_instance()
    {
        static ModuleCreator instance;
        return &instance;
    }

    void register_module(const std::string &op_type, Creator creator) { m_creators[op_type] = creator; }

    Module *create(fbs::FbsModel *fbs_model, const std::string &op_type, const std::string &node_name)
    {
        register_dl_modules();
        auto it = m_creators.find(op_type);
        return it == m_creators.end() ? nullptr : it->second(fbs_model, node_name);
    }

    bool is_registered(const std::string &op_type)
    {
        register_dl_modules();
        return m_creators.count(op_type) != 0;
    }

    void register_dl_modules()
    {
        if (!m_creators.empty())
            return;
        register_module("Conv", Conv::deserialize);
        register_module("Gemm", Gemm::deserialize);
        register_module("MatMul", MatMul::deserialize);
        register_module("LUT", LUT::deserialize);
        register_module("Relu", Relu::deserialize);
        register_module("PRelu", PRelu::deserialize);
        register_module("Clip", Clip::deserialize);
        register_module("Add", Add::deserialize);
        register_module("Mul", Mul::deserialize);
        register_module("Sub", SubDiv::deserialize_sub);
        register_module("Div", SubDiv::deserialize_div);
        register_module("GlobalAveragePool", GlobalAveragePool::deserialize);
        register_module("RequantizeLinear", RequantizeLinear::deserialize);
        register_module("Flatten", Flatten::deserialize);
        register_module("Squeeze", ShapeView::deserialize_squeeze);
        register_module("Unsqueeze", ShapeView::deserialize_unsqueeze);
        register_module("Reshape", ShapeView::deserialize_reshape);
        register_module("Concat", Concat::deserialize);
        register_module("Split", Split::deserialize);
        register_module("Transpose", Transpose::deserialize);
        register_module("Resize", Resize::deserialize);
        register_module("MaxPool", MaxPool::deserialize);
        register_module("AveragePool", AveragePool::deserialize);
        register_module("Slice", Slice::deserialize);
        register_module("ReduceMean", ReduceMean::deserialize);
        register_module("ReduceMax", ReduceMean::deserialize_max);
        register_module("ReduceMin", ReduceMean::deserialize_min);
        register_module("ReduceSum", ReduceMean::deserialize_sum);
        register_module("ReduceL1", ReduceMean::deserialize_l1);
        register_module("ReduceSumSquare", ReduceMean::deserialize_sum_square);
        register_module("InsertZeros", InsertZeros::deserialize);
        register_module("Pad", Pad::deserialize);
        register_module("Gather", Gather::deserialize);
        register_module("SpaceToDepth", SpaceDepth::deserialize_space_to_depth);
        register_module("DepthToSpace", SpaceDepth::deserialize_depth_to_space);
        register_module("StreamingCache", StreamingCache::deserialize);
        register_module("Softmax", Softmax::deserialize);
        // both are TensorBase::assign between a float32 and a quantized tensor
        // (esp-dl/dl/module/include/dl_module_creator.hpp:154-155)
        register_module("QuantizeLinear", RequantizeLinear::deserialize);
        register_module("DequantizeLinear", RequantizeLinear::deserialize);
        // element-wise activations: a node with a precomputed table becomes a LUT, otherwise the reference's
        // float32 expression is evaluated per possible input (dl_module_unary.hpp)
        register_module("Sigmoid", UnaryMath::deserialize<UNARY_SIGMOID>);
        register_module("Tanh", UnaryMath::deserialize<UNARY_TANH>);
        register_module("HardSwish", UnaryMath::deserialize<UNARY_HARD_SWISH>);
        register_module("Elu", UnaryMath::deserialize<UNARY_ELU>);
        register_module("Exp", UnaryMath::deserialize<UNARY_EXP>);
        register_module("Log", UnaryMath::deserialize<UNARY_LOG>);
        register_module("Sqrt", UnaryMath::deserialize<UNARY_SQRT>);
        register_module("LeakyRelu", UnaryMath::deserialize<UNARY_LEAKY_RELU>);
        register_module("Neg", UnaryMath::deserialize<UNARY_NEG>);
        register_module("Swish", UnaryMath::deserialize<UNARY_SWISH>);
        register_module("HardSigmoid", UnaryMath::deserialize<UNARY_HARD_SIGMOID>);
        // Identity is output->assign(input) (esp-dl/dl/module/include/dl_module_identity.hpp:34-42)
        register_module("Identity", RequantizeLinear::deserialize);
        // exported only with a table (esp-dl/dl/module/include/dl_module_creator.hpp:151)
        for (const char *op : {"Gelu", "Softplus", "Mish"}) {
            const std::string op_type = op;
            register_module(op_type, [op_type](fbs::FbsModel *fbs_model, std::string node_name) -> Module * {
                quant_type_t quant_type = QUANT_TYPE_NONE;
                fbs_model->get_operation_attribute(node_name, "quant_type", quant_type);
                Module *m = lut_if_present(fbs_model, node_name, quant_type);
                if (!m)
                    DL_LOGE("ModuleCreator", "%s (%s) has no table; only the table form is implemented",
                            node_name.c_str(), op_type.c_str());
                return m;
            });
        }
    }

    void clear() { m_creators.clear(); }

private:
    ModuleCreator() {}
    std::map<std::string, Creator> m_creators;
};

} // namespace module
} // namespace dl
