#include "dl_model_context.hpp"

#include <hip/hip_runtime.h>

namespace dl {

int ModelContext::add_tensor(const std::string name, bool is_parameter, TensorBase *tensor)
{
    auto it = m_name2index.find(name);
    if (it != m_name2index.end()) {
        // the same initializer may feed several nodes: keep the first copy
        if (tensor && get_tensor(it->second) != tensor)
            delete tensor;
        return it->second;
    }
    int index;
    if (is_parameter) {
        m_parameters.push_back(tensor);
        index = (int)m_parameters.size() - 1 + CONTEXT_PARAMETER_OFFSET;
    } else {
        m_variables.push_back(tensor);
        index = (int)m_variables.size() - 1;
    }
    m_name2index[name] = index;
    return index;
}

int ModelContext::push_back_tensor(TensorBase *tensor, bool is_parameter)
{
    if (is_parameter) {
        m_parameters.push_back(tensor);
        return (int)m_parameters.size() - 1 + CONTEXT_PARAMETER_OFFSET;
    }
    m_variables.push_back(tensor);
    return (int)m_variables.size() - 1;
}

void ModelContext::update_tensor(int index, TensorBase *tensor)
{
    if (index >= CONTEXT_PARAMETER_OFFSET) {
        const int pi = index - CONTEXT_PARAMETER_OFFSET;
        if (pi > 0 && pi < (int)m_parameters.size())
            m_parameters[pi] = tensor;
    } else if (index > 0 && index < (int)m_variables.size()) {
        m_variables[index] = tensor;
    }
}

TensorBase *ModelContext::get_tensor(int index)
{
    if (index >= CONTEXT_PARAMETER_OFFSET) {
        const int pi = index - CONTEXT_PARAMETER_OFFSET;
        return (pi > 0 && pi < (int)m_parameters.size()) ? m_parameters[pi] : nullptr;
    }
    return (index > 0 && index < (int)m_variables.size()) ? m_variables[index] : nullptr;
}

TensorBase *ModelContext::get_tensor(const std::string &name)
{
    const int index = get_tensor_index(name);
    return index < 0 ? nullptr : get_tensor(index);
}

int ModelContext::get_tensor_index(const std::string &name)
{
    auto it = m_name2index.find(name);
    return it == m_name2index.end() ? -1 : it->second;
}

int ModelContext::get_variable_index(const std::string &name)
{
    const int index = get_tensor_index(name);
    return (index > 0 && index < CONTEXT_PARAMETER_OFFSET) ? index : -1;
}

std::string ModelContext::get_tensor_name(int index)
{
    for (auto &kv : m_name2index)
        if (kv.second == index)
            return kv.first;
    return std::string();
}

bool ModelContext::root_alloc(size_t device_bytes)
{
    root_free();
    if (device_bytes == 0)
        device_bytes = 256;
    if (hipMalloc(&m_device_root, device_bytes) != hipSuccess) {
        DL_LOGE("ModelContext", "hipMalloc of %zu bytes for the activation arena failed", device_bytes);
        m_device_root = nullptr;
        return false;
    }
    m_device_size = device_bytes;
    return true;
}

void ModelContext::root_free()
{
    if (m_device_root) {
        (void)hipFree(m_device_root);
        m_device_root = nullptr;
        m_device_size = 0;
    }
}

size_t ModelContext::get_parameter_memory_size()
{
    size_t total = 0;
    for (TensorBase *t : m_parameters)
        if (t)
            total += t->get_aligned_bytes();
    return total;
}

size_t ModelContext::get_variable_memory_size()
{
    return m_device_size;
}

void ModelContext::clear()
{
    if (owns_tensors) {
        for (TensorBase *t : m_variables)
            delete t;
        for (TensorBase *t : m_parameters)
            delete t;
    }
    root_free();
    m_variables.assign(1, nullptr);
    m_parameters.assign(1, nullptr);
    m_name2index.clear();
}

} // namespace dl
