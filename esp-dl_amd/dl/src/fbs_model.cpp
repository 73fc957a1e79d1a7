#include "fbs_model.hpp"

#include <algorithm>
#include <cstring>
#include <set>

namespace fbs {

namespace {
const char *TAG = "FbsModel";

Initializer make_init(const std::vector<int> &dims, dl::dtype_t dtype, const void *data,
                      const std::vector<int> &exponents)
{
    Initializer init;
    init.dims = dims;
    init.dtype = dtype;
    init.exponents = exponents;
    size_t n = dl::dtype_sizeof(dtype);
    for (int d : dims)
        n *= (size_t)d;
    init.bytes.resize(n);
    if (data && n)
        memcpy(init.bytes.data(), data, n);
    return init;
}
} // namespace

Node *FbsModel::add_node(const std::string &name, const std::string &op_type, const std::vector<std::string> &inputs,
                         const std::vector<std::string> &outputs)
{
    Node n;
    n.name = name;
    n.op_type = op_type;
    n.inputs = inputs;
    n.outputs = outputs;
    m_node_index[name] = m_nodes.size();
    m_nodes.push_back(n);
    return &m_nodes.back();
}

Node *FbsModel::get_node(const std::string &name)
{
    auto it = m_node_index.find(name);
    return it == m_node_index.end() ? nullptr : &m_nodes[it->second];
}

void FbsModel::add_initializer(const std::string &name, const std::vector<int> &dims, dl::dtype_t dtype,
                               const void *data, const std::vector<int> &exponents)
{
    m_initializers[name] = make_init(dims, dtype, data, exponents);
}

void FbsModel::add_value_info(const std::string &name, const std::vector<int> &dims, dl::dtype_t dtype, int exponent)
{
    ValueInfo v;
    v.dims = dims;
    v.dtype = dtype;
    v.exponent = exponent;
    m_value_info[name] = v;
}

void FbsModel::add_test_input(const std::string &name, const std::vector<int> &dims, dl::dtype_t dtype,
                              const void *data, int exponent)
{
    m_test_inputs[name] = make_init(dims, dtype, data, {exponent});
}

void FbsModel::add_test_output(const std::string &name, const std::vector<int> &dims, dl::dtype_t dtype,
                               const void *data, int exponent)
{
    if (!m_test_outputs.count(name))
        m_test_output_order.push_back(name);
    m_test_outputs[name] = make_init(dims, dtype, data, {exponent});
}

// Kahn's algorithm over tensor names; nodes whose inputs are all graph inputs / initializers come first,
// ties keep insertion order (the exporter already emits a valid order).
std::vector<std::string> FbsModel::topological_sort()
{
    std::set<std::string> ready(m_inputs.begin(), m_inputs.end());
    for (auto &kv : m_initializers)
        ready.insert(kv.first);
    ready.insert("");
    std::vector<bool> done(m_nodes.size(), false);
    std::vector<std::string> order;
    bool progress = true;
    while (order.size() < m_nodes.size() && progress) {
        progress = false;
        for (size_t i = 0; i < m_nodes.size(); i++) {
            if (done[i])
                continue;
            bool ok = true;
            for (auto &in : m_nodes[i].inputs)
                if (!ready.count(in)) {
                    ok = false;
                    break;
                }
            if (ok) {
                done[i] = true;
                progress = true;
                order.push_back(m_nodes[i].name);
                for (auto &out : m_nodes[i].outputs)
                    ready.insert(out);
            }
        }
    }
    if (order.size() != m_nodes.size())
        DL_LOGE(TAG, "graph has a cycle or a dangling input: %zu of %zu nodes could be ordered", order.size(),
                m_nodes.size());
    return order;
}

const Attribute *FbsModel::find_attribute(const std::string &node_name, const std::string &attribute_name)
{
    Node *n = get_node(node_name);
    if (!n)
        return nullptr;
    auto it = n->attributes.find(attribute_name);
    return it == n->attributes.end() ? nullptr : &it->second;
}

esp_err_t FbsModel::get_operation_attribute(std::string node_name, std::string attribute_name, int &ret_value)
{
    const Attribute *a = find_attribute(node_name, attribute_name);
    if (!a || a->kind != Attribute::INT)
        return ESP_FAIL;
    ret_value = (int)a->i;
    return ESP_OK;
}

esp_err_t FbsModel::get_operation_attribute(std::string node_name, std::string attribute_name, float &ret_value)
{
    const Attribute *a = find_attribute(node_name, attribute_name);
    if (!a || a->kind != Attribute::FLOAT)
        return ESP_FAIL;
    ret_value = a->f;
    return ESP_OK;
}

esp_err_t FbsModel::get_operation_attribute(std::string node_name, std::string attribute_name, std::string &ret_value)
{
    const Attribute *a = find_attribute(node_name, attribute_name);
    if (!a || a->kind != Attribute::STRING)
        return ESP_FAIL;
    ret_value = a->s;
    return ESP_OK;
}

esp_err_t FbsModel::get_operation_attribute(std::string node_name, std::string attribute_name,
                                            std::vector<int> &ret_value)
{
    const Attribute *a = find_attribute(node_name, attribute_name);
    if (!a || a->kind != Attribute::INTS)
        return ESP_FAIL;
    ret_value.assign(a->ints.begin(), a->ints.end());
    return ESP_OK;
}

esp_err_t FbsModel::get_operation_attribute(std::string node_name, std::string attribute_name,
                                            std::vector<float> &ret_value)
{
    const Attribute *a = find_attribute(node_name, attribute_name);
    if (!a || a->kind != Attribute::FLOATS)
        return ESP_FAIL;
    ret_value = a->floats;
    return ESP_OK;
}

// `quant_type` is exported as the string "S8" / "S16" / "F32" (seen in the reference's fixtures).
esp_err_t FbsModel::get_operation_attribute(std::string node_name, std::string attribute_name,
                                            dl::quant_type_t &ret_value)
{
    std::string s;
    ret_value = dl::QUANT_TYPE_NONE;
    if (get_operation_attribute(node_name, attribute_name, s) != ESP_OK)
        return ESP_FAIL;
    if (s == "S8")
        ret_value = dl::QUANT_TYPE_SYMM_8BIT;
    else if (s == "S16")
        ret_value = dl::QUANT_TYPE_SYMM_16BIT;
    else if (s == "F32")
        ret_value = dl::QUANT_TYPE_FLOAT32;
    else
        return ESP_FAIL;
    return ESP_OK;
}

// `activation` is exported as "Linear" / "Relu" / "LeakyRelu" / "PRelu".
esp_err_t FbsModel::get_operation_attribute(std::string node_name, std::string attribute_name,
                                            dl::activation_type_t &ret_value)
{
    std::string s;
    ret_value = dl::Linear;
    if (get_operation_attribute(node_name, attribute_name, s) != ESP_OK)
        return ESP_FAIL;
    if (s == "Linear" || s.empty())
        ret_value = dl::Linear;
    else if (s == "Relu" || s == "ReLU")
        ret_value = dl::ReLU;
    else if (s == "LeakyRelu" || s == "LeakyReLU")
        ret_value = dl::LeakyReLU;
    else if (s == "PRelu" || s == "PReLU")
        ret_value = dl::PReLU;
    else
        return ESP_FAIL;
    return ESP_OK;
}

esp_err_t FbsModel::get_operation_inputs_and_outputs(std::string node_name, std::vector<std::string> &inputs,
                                                     std::vector<std::string> &outputs)
{
    Node *n = get_node(node_name);
    if (!n)
        return ESP_FAIL;
    inputs = n->inputs;
    outputs = n->outputs;
    return ESP_OK;
}

std::string FbsModel::get_operation_type(std::string node_name)
{
    Node *n = get_node(node_name);
    return n ? n->op_type : std::string();
}

dl::TensorBase *FbsModel::tensor_from(const Initializer &init, uint32_t caps)
{
    dl::TensorBase *t = new dl::TensorBase(init.dims, init.bytes.data(), init.exponents, init.dtype, true, caps);
    return t;
}

dl::TensorBase *FbsModel::get_operation_parameter(std::string node_name, int index, uint32_t caps)
{
    Node *n = get_node(node_name);
    if (!n || index < 0 || index >= (int)n->inputs.size())
        return nullptr;
    auto it = m_initializers.find(n->inputs[index]);
    return it == m_initializers.end() ? nullptr : tensor_from(it->second, caps);
}

dl::TensorBase *FbsModel::get_operation_lut(std::string node_name, uint32_t caps, std::string attribute_name)
{
    std::string lut_name;
    if (get_operation_attribute(node_name, attribute_name, lut_name) != ESP_OK)
        return nullptr;
    auto it = m_initializers.find(lut_name);
    return it == m_initializers.end() ? nullptr : tensor_from(it->second, caps);
}

bool FbsModel::is_parameter(std::string name)
{
    return m_initializers.count(name) != 0;
}

const void *FbsModel::get_tensor_raw_data(std::string tensor_name)
{
    auto it = m_initializers.find(tensor_name);
    return it == m_initializers.end() ? nullptr : it->second.bytes.data();
}

dl::dtype_t FbsModel::get_tensor_dtype(std::string tensor_name)
{
    auto it = m_initializers.find(tensor_name);
    return it == m_initializers.end() ? dl::DATA_TYPE_UNDEFINED : it->second.dtype;
}

std::vector<int> FbsModel::get_tensor_shape(std::string tensor_name)
{
    auto it = m_initializers.find(tensor_name);
    return it == m_initializers.end() ? std::vector<int>() : it->second.dims;
}

std::vector<int> FbsModel::get_tensor_exponents(std::string tensor_name)
{
    auto it = m_initializers.find(tensor_name);
    return it == m_initializers.end() ? std::vector<int>() : it->second.exponents;
}

dl::dtype_t FbsModel::get_value_info_dtype(std::string var_name)
{
    auto it = m_value_info.find(var_name);
    return it == m_value_info.end() ? dl::DATA_TYPE_UNDEFINED : it->second.dtype;
}

std::vector<int> FbsModel::get_value_info_shape(std::string var_name)
{
    auto it = m_value_info.find(var_name);
    return it == m_value_info.end() ? std::vector<int>() : it->second.dims;
}

int FbsModel::get_value_info_exponent(std::string var_name)
{
    auto it = m_value_info.find(var_name);
    return it == m_value_info.end() ? 0 : it->second.exponent;
}

dl::TensorBase *FbsModel::get_test_input_tensor(std::string tensor_name)
{
    auto it = m_test_inputs.find(tensor_name);
    return it == m_test_inputs.end() ? nullptr : tensor_from(it->second, MALLOC_CAP_HOST);
}

dl::TensorBase *FbsModel::get_test_output_tensor(std::string tensor_name)
{
    auto it = m_test_outputs.find(tensor_name);
    return it == m_test_outputs.end() ? nullptr : tensor_from(it->second, MALLOC_CAP_HOST);
}

std::vector<std::string> FbsModel::get_test_outputs_name()
{
    return m_test_output_order;
}

std::string FbsModel::get_model_metadata_prop(const std::string &key)
{
    auto it = m_metadata.find(key);
    return it == m_metadata.end() ? std::string() : it->second;
}

void FbsModel::print()
{
    std::printf("model %s v%lld: %zu nodes, %zu initializers\n", m_name.c_str(), (long long)m_version, m_nodes.size(),
                m_initializers.size());
    for (auto &n : m_nodes)
        std::printf("  %-20s %s\n", n.op_type.c_str(), n.name.c_str());
}

} // namespace fbs
