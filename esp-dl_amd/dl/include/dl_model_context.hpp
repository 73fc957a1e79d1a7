// dl::ModelContext: owner and index of a model's tensors.
//
// Same role and accessor names as esp-dl/dl/model/include/dl_model_context.hpp:13-240: modules hold
// integer indices, variables (activations) and parameters live in two arrays, parameter indices are
// offset by CONTEXT_PARAMETER_OFFSET.  Instead of an internal-RAM/PSRAM pair of roots there is one
// device arena in HBM from which every variable is carved, plus the execution settings the batched
// GPU executor needs (stream, rounding flavour).
#pragma once

#include <map>
#include <string>
#include <vector>

#include "dl_tensor_base.hpp"

namespace dl {

#define CONTEXT_PARAMETER_OFFSET 10000000

class ModelContext {
public:
    std::vector<TensorBase *> m_variables;  ///< activations; entry 0 is nullptr
    std::vector<TensorBase *> m_parameters; ///< weights, biases, tables; entry 0 is nullptr
    void *stream = nullptr;                 ///< hipStream_t every module enqueues on
    round_mode_t round_mode = ROUND_MODE_HALF_UP;
    bool owns_tensors = false; ///< true for a Model's context, false for the temporary one of Module::run

    ModelContext()
    {
        m_variables.push_back(nullptr);
        m_parameters.push_back(nullptr);
    }
    ~ModelContext() { clear(); }

    /// Register a tensor name; returns its index (existing index when the name is known).
    int add_tensor(const std::string name, bool is_parameter = false, TensorBase *tensor = nullptr);
    /// Append an anonymous tensor (used by Module::run on bare tensors).
    int push_back_tensor(TensorBase *tensor, bool is_parameter = false);
    void update_tensor(int index, TensorBase *tensor);
    TensorBase *get_tensor(int index);
    TensorBase *get_tensor(const std::string &name);
    int get_tensor_index(const std::string &name);
    int get_variable_index(const std::string &name);
    std::string get_tensor_name(int index);
    int get_variable_count() { return (int)m_variables.size(); }
    int get_parameter_count() { return (int)m_parameters.size(); }

    /// One HBM allocation all variables are placed in.
    bool root_alloc(size_t device_bytes);
    void *get_device_root() { return m_device_root; }
    size_t get_device_size() { return m_device_size; }
    void root_free();
    size_t get_parameter_memory_size();
    size_t get_variable_memory_size();
    void clear();

private:
    void *m_device_root = nullptr;
    size_t m_device_size = 0;
    std::map<std::string, int> m_name2index;
};

} // namespace dl
