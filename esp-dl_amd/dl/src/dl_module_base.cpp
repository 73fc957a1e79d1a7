#include "dl_module_base.hpp"

#include <hip/hip_runtime.h>

namespace dl {
namespace module {

void Module::run(TensorBase *input, TensorBase *output, runtime_mode_t mode, void *stream)
{
    ModelContext context;
    context.stream = stream;
    m_inputs_index.clear();
    m_outputs_index.clear();
    m_inputs_index.push_back(context.push_back_tensor(input));
    m_outputs_index.push_back(context.push_back_tensor(output));
    forward(&context, mode);
}

void Module::run(std::vector<dl::TensorBase *> inputs, std::vector<dl::TensorBase *> outputs, runtime_mode_t mode,
                 void *stream)
{
    ModelContext context;
    context.stream = stream;
    m_inputs_index.clear();
    m_outputs_index.clear();
    for (TensorBase *t : inputs)
        m_inputs_index.push_back(context.push_back_tensor(t));
    for (TensorBase *t : outputs)
        m_outputs_index.push_back(context.push_back_tensor(t));
    forward(&context, mode);
}

DeviceInts::~DeviceInts()
{
    if (m_dev)
        (void)hipFree(m_dev);
}

const int32_t *DeviceInts::sync(const std::vector<int32_t> &values)
{
    if (m_dev && values == m_host)
        return m_dev;
    if (m_dev && values.size() != m_host.size()) {
        (void)hipFree(m_dev);
        m_dev = nullptr;
    }
    if (!m_dev && hipMalloc(reinterpret_cast<void **>(&m_dev), values.size() * sizeof(int32_t) + 16) != hipSuccess) {
        DL_LOGE("Module", "hipMalloc for %zu shifts failed", values.size());
        m_dev = nullptr;
        return nullptr;
    }
    if (hipMemcpy(m_dev, values.data(), values.size() * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess) {
        DL_LOGE("Module", "upload of %zu shifts failed", values.size());
        return nullptr;
    }
    m_host = values;
    return m_dev;
}

} // namespace module
} // namespace dl
