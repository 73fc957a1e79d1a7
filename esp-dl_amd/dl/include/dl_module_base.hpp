// dl::module::Module: the operator interface a dl::Model dispatches through.
//
// Signatures follow esp-dl/dl/module/include/dl_module_base.hpp:25-140: get_output_shape,
// forward(ModelContext*, runtime_mode_t), forward_args, deserialize(FbsModel*, node_name), run() on
// bare tensors, m_inputs_index / m_outputs_index.  forward() enqueues HIP kernels on the context's
// stream through the C ABI of include/espdl_hip.h; tensors handed to it must be device tensors.
#pragma once

#include <string>
#include <vector>

#include "dl_define.hpp"
#include "dl_model_context.hpp"
#include "dl_tensor_base.hpp"
#include "fbs_model.hpp"

namespace dl {

typedef enum {
    MODULE_NON_INPLACE = 0,              ///< output goes to separate memory
    MODULE_INPLACE_UNCHANGED_BUFFER = 1, ///< output aliases the input bytes unchanged (Reshape, Flatten)
    MODULE_INPLACE_CHANGED_BUFFER = 2    ///< output may overwrite the input buffer (Add, LUT, Relu ...)
} module_inplace_t;

namespace module {

class Module {
public:
    std::string name;
    module_inplace_t inplace;
    quant_type_t quant_type;
    std::vector<int> m_inputs_index;
    std::vector<int> m_outputs_index;

    Module(const char *name = nullptr, module_inplace_t inplace = MODULE_NON_INPLACE,
           quant_type_t quant_type = QUANT_TYPE_NONE) :
        name(name ? name : ""), inplace(inplace), quant_type(quant_type)
    {
    }
    virtual ~Module() {}

    virtual std::vector<int> get_outputs_index() { return m_outputs_index; }
    virtual std::vector<std::vector<int>> get_output_shape(std::vector<std::vector<int>> &input_shapes) = 0;
    virtual void forward(ModelContext *context, runtime_mode_t mode = RUNTIME_MODE_AUTO) = 0;
    virtual void forward_args(void *args) { (void)args; }
    static Module *deserialize(fbs::FbsModel *fbs_model, std::string node_name)
    {
        (void)fbs_model;
        (void)node_name;
        return nullptr;
    }
    virtual void print() {}
    virtual void reset() {}
    /// A module that carries data from one forward to the next saves it in hold_state and puts it back in
    /// restore_state: the model brackets passes whose results are discarded (the warm-up before a graph
    /// capture, profiling passes) with the two calls, on `stream`.
    virtual void hold_state(void *stream) { (void)stream; }
    virtual void restore_state(void *stream) { (void)stream; }
    /// Whether forward handles input `slot` (a position in m_inputs_index) / output `slot` being a channel
    /// slice of a wider tensor (TensorBase::channel_pitch).  A model only leaves the output of a channel Split
    /// inside the Split's input, or lets a producer write straight into the output of a channel Concat, when
    /// every module that touches the tensor says yes here.
    virtual bool reads_channel_slice(int slot) const
    {
        (void)slot;
        return false;
    }
    virtual bool writes_channel_slice(int slot) const
    {
        (void)slot;
        return false;
    }
    /// Multiply-accumulates one forward performs for the given input shapes (0 for data movement);
    /// used by Model::profile to report achieved int8 OP/s.
    virtual int64_t get_macs(std::vector<std::vector<int>> &input_shapes)
    {
        (void)input_shapes;
        return 0;
    }

    /// Stand-alone use on bare DEVICE tensors, as the reference's Module::run
    /// (esp-dl/dl/module/src/dl_module_base.cpp:120-144): wraps them in a temporary context.
    virtual void run(TensorBase *input, TensorBase *output, runtime_mode_t mode = RUNTIME_MODE_SINGLE_CORE,
                     void *stream = nullptr);
    virtual void run(std::vector<dl::TensorBase *> inputs, std::vector<dl::TensorBase *> outputs,
                     runtime_mode_t mode = RUNTIME_MODE_SINGLE_CORE, void *stream = nullptr);
};

/// Device-resident int32 array (requantization shifts) owned by a module.
class DeviceInts {
public:
    DeviceInts() {}
    ~DeviceInts();
    DeviceInts(const DeviceInts &) = delete;
    DeviceInts &operator=(const DeviceInts &) = delete;
    /// Upload `values` (synchronously) unless the same values are already resident.
    const int32_t *sync(const std::vector<int32_t> &values);
    int count() const { return (int)m_host.size(); }

private:
    int32_t *m_dev = nullptr;
    std::vector<int32_t> m_host;
};

} // namespace module
} // namespace dl
