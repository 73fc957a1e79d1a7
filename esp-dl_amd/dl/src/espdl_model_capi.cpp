// C handle API of include/espdl_model.h over fbs::FbsModel and dl::Model.
#include "espdl_model.h"

#include <cstring>
#include <string>
#include <vector>

#include "dl_model_base.hpp"
#include "dl_module_creator.hpp"
#include "fbs_loader.hpp"

struct espdl_graph {
    fbs::FbsModel fbs;
};

struct espdl_model {
    dl::Model *model = nullptr;
    std::vector<dl::module_info> last_profile;
};

namespace {
std::vector<int> to_dims(const int32_t *dims, int32_t n)
{
    return std::vector<int>(dims, dims + (n > 0 ? n : 0));
}
} // namespace

extern "C" {

espdl_graph *espdl_graph_create(const char *name)
{
    espdl_graph *g = new espdl_graph();
    g->fbs.set_model_info(name ? name : "");
    return g;
}

void espdl_graph_destroy(espdl_graph *g)
{
    delete g;
}

static thread_local std::string g_load_error;

static espdl_graph *graph_from_loader(fbs::FbsLoader &loader, int32_t model_index)
{
    fbs::FbsModel *m = loader.load(model_index);
    if (!m) {
        g_load_error = loader.last_error();
        return nullptr;
    }
    espdl_graph *g = new espdl_graph();
    g->fbs = std::move(*m);
    delete m;
    g_load_error.clear();
    return g;
}

espdl_graph *espdl_graph_load_file(const char *path, int32_t model_index)
{
    fbs::FbsLoader loader(path, fbs::MODEL_LOCATION_IN_SDCARD);
    return graph_from_loader(loader, model_index);
}

espdl_graph *espdl_graph_load_memory(const void *data, int64_t size, int32_t model_index)
{
    fbs::FbsLoader loader(data, size > 0 ? (size_t)size : 0);
    return graph_from_loader(loader, model_index);
}

const char *espdl_graph_load_error(void)
{
    return g_load_error.c_str();
}

int32_t espdl_graph_input_count(espdl_graph *g)
{
    return g ? (int32_t)g->fbs.get_graph_inputs().size() : -1;
}

int32_t espdl_graph_output_count(espdl_graph *g)
{
    return g ? (int32_t)g->fbs.get_graph_outputs().size() : -1;
}

static const char *io_name(espdl_graph *g, bool input, int32_t index)
{
    static thread_local std::string name;
    if (!g)
        return nullptr;
    const std::vector<std::string> names = input ? g->fbs.get_graph_inputs() : g->fbs.get_graph_outputs();
    if (index < 0 || index >= (int32_t)names.size())
        return nullptr;
    name = names[(size_t)index];
    return name.c_str();
}

int64_t espdl_graph_initializer_bytes(espdl_graph *g, const char *name, void *dst, int64_t capacity)
{
    if (!g || !name || !g->fbs.is_parameter(name))
        return -1;
    const void *raw = g->fbs.get_tensor_raw_data(name);
    size_t bytes = dl::dtype_sizeof(g->fbs.get_tensor_dtype(name));
    for (int d : g->fbs.get_tensor_shape(name))
        bytes *= (size_t)d;
    if (dst && capacity >= (int64_t)bytes && raw)
        std::memcpy(dst, raw, bytes);
    return (int64_t)bytes;
}

int32_t espdl_graph_node_count(espdl_graph *g)
{
    return g ? (int32_t)g->fbs.topological_sort().size() : -1;
}

const char *espdl_graph_node_op_type(espdl_graph *g, int32_t index)
{
    static thread_local std::string op;
    if (!g)
        return nullptr;
    const std::vector<std::string> order = g->fbs.topological_sort();
    if (index < 0 || index >= (int32_t)order.size())
        return nullptr;
    op = g->fbs.get_operation_type(order[(size_t)index]);
    return op.c_str();
}

int32_t espdl_module_is_registered(const char *op_type)
{
    return op_type && dl::module::ModuleCreator::get_instance()->is_registered(op_type) ? 1 : 0;
}

const char *espdl_graph_input_name(espdl_graph *g, int32_t index)
{
    return io_name(g, true, index);
}

const char *espdl_graph_output_name(espdl_graph *g, int32_t index)
{
    return io_name(g, false, index);
}

int espdl_graph_add_initializer(espdl_graph *g, const char *name, const int32_t *dims, int32_t n_dims, int32_t dtype,
                                const void *data, const int32_t *exponents, int32_t n_exponents)
{
    if (!g || !name || !data)
        return -1;
    std::vector<int> exps(exponents, exponents + (n_exponents > 0 ? n_exponents : 0));
    g->fbs.add_initializer(name, to_dims(dims, n_dims), (dl::dtype_t)dtype, data, exps);
    return 0;
}

int espdl_graph_add_value_info(espdl_graph *g, const char *name, const int32_t *dims, int32_t n_dims, int32_t dtype,
                               int32_t exponent)
{
    if (!g || !name)
        return -1;
    g->fbs.add_value_info(name, to_dims(dims, n_dims), (dl::dtype_t)dtype, exponent);
    return 0;
}

int espdl_graph_add_input(espdl_graph *g, const char *name)
{
    if (!g || !name)
        return -1;
    g->fbs.add_graph_input(name);
    return 0;
}

int espdl_graph_add_output(espdl_graph *g, const char *name)
{
    if (!g || !name)
        return -1;
    g->fbs.add_graph_output(name);
    return 0;
}

int espdl_graph_add_node(espdl_graph *g, const char *name, const char *op_type, const char *const *inputs,
                         int32_t n_inputs, const char *const *outputs, int32_t n_outputs)
{
    if (!g || !name || !op_type)
        return -1;
    std::vector<std::string> ins, outs;
    for (int i = 0; i < n_inputs; i++)
        ins.push_back(inputs[i] ? inputs[i] : "");
    for (int i = 0; i < n_outputs; i++)
        outs.push_back(outputs[i] ? outputs[i] : "");
    g->fbs.add_node(name, op_type, ins, outs);
    return 0;
}

int espdl_graph_node_set_int(espdl_graph *g, const char *node, const char *key, int64_t value)
{
    fbs::Node *n = g ? g->fbs.get_node(node) : nullptr;
    if (!n)
        return -1;
    fbs::Attribute a;
    a.kind = fbs::Attribute::INT;
    a.i = value;
    n->attributes[key] = a;
    return 0;
}

int espdl_graph_node_set_float(espdl_graph *g, const char *node, const char *key, float value)
{
    fbs::Node *n = g ? g->fbs.get_node(node) : nullptr;
    if (!n)
        return -1;
    fbs::Attribute a;
    a.kind = fbs::Attribute::FLOAT;
    a.f = value;
    n->attributes[key] = a;
    return 0;
}

int espdl_graph_node_set_ints(espdl_graph *g, const char *node, const char *key, const int64_t *values, int32_t count)
{
    fbs::Node *n = g ? g->fbs.get_node(node) : nullptr;
    if (!n)
        return -1;
    fbs::Attribute a;
    a.kind = fbs::Attribute::INTS;
    a.ints.assign(values, values + (count > 0 ? count : 0));
    n->attributes[key] = a;
    return 0;
}

int espdl_graph_node_set_string(espdl_graph *g, const char *node, const char *key, const char *value)
{
    fbs::Node *n = g ? g->fbs.get_node(node) : nullptr;
    if (!n)
        return -1;
    fbs::Attribute a;
    a.kind = fbs::Attribute::STRING;
    a.s = value ? value : "";
    n->attributes[key] = a;
    return 0;
}

int espdl_graph_add_test_input(espdl_graph *g, const char *name, const int32_t *dims, int32_t n_dims, int32_t dtype,
                               const void *data, int32_t exponent)
{
    if (!g || !name || !data)
        return -1;
    g->fbs.add_test_input(name, to_dims(dims, n_dims), (dl::dtype_t)dtype, data, exponent);
    return 0;
}

int espdl_graph_add_test_output(espdl_graph *g, const char *name, const int32_t *dims, int32_t n_dims, int32_t dtype,
                                const void *data, int32_t exponent)
{
    if (!g || !name || !data)
        return -1;
    g->fbs.add_test_output(name, to_dims(dims, n_dims), (dl::dtype_t)dtype, data, exponent);
    return 0;
}

espdl_model *espdl_model_create(espdl_graph *g, int32_t batch, int32_t round_mode, void *stream, int32_t fuse)
{
    if (!g || batch <= 0)
        return nullptr;
    espdl_model *m = new espdl_model();
    m->model = new dl::Model(&g->fbs, batch, round_mode == 1 ? dl::ROUND_MODE_HALF_EVEN : dl::ROUND_MODE_HALF_UP, stream,
                             (int)fuse);
    if (m->model->get_outputs().empty() || m->model->get_module_count() == 0) {
        delete m->model;
        delete m;
        return nullptr;
    }
    return m;
}

void espdl_model_destroy(espdl_model *m)
{
    if (m) {
        delete m->model;
        delete m;
    }
}

int espdl_model_run(espdl_model *m)
{
    if (!m)
        return -1;
    m->model->run();
    return m->model->last_run_failed() ? -2 : 0;
}

int espdl_model_run_async(espdl_model *m)
{
    if (!m)
        return -1;
    m->model->run_async();
    return m->model->last_run_failed() ? -2 : 0;
}

int espdl_model_synchronize(espdl_model *m)
{
    if (!m)
        return -1;
    m->model->synchronize();
    return m->model->last_run_failed() ? -2 : 0;
}

int espdl_model_enable_graph(espdl_model *m)
{
    return (m && m->model->enable_graph()) ? 0 : -1;
}

int espdl_model_disable_graph(espdl_model *m)
{
    if (!m)
        return -1;
    m->model->disable_graph();
    return 0;
}

int espdl_model_test(espdl_model *m)
{
    return (m && m->model->test() == ESP_OK) ? 0 : -1;
}

int espdl_model_module_count(espdl_model *m)
{
    return m ? (int)m->model->get_module_count() : -1;
}

int espdl_model_profile(espdl_model *m, int32_t repeats, int32_t capacity, const char **names, const char **types,
                        float *latency_us, int64_t *macs, int64_t *bytes)
{
    if (!m)
        return -1;
    m->last_profile = m->model->get_module_info(repeats);
    const int n = (int)m->last_profile.size();
    for (int i = 0; i < n && i < capacity; i++) {
        const dl::module_info &mi = m->last_profile[i];
        if (names)
            names[i] = mi.name.c_str();
        if (types)
            types[i] = mi.type.c_str();
        if (latency_us)
            latency_us[i] = mi.latency_us;
        if (macs)
            macs[i] = mi.macs;
        if (bytes)
            bytes[i] = mi.bytes;
    }
    return n;
}

void espdl_model_print_profile(espdl_model *m)
{
    if (m)
        m->model->profile(false);
}

void *espdl_model_tensor_device_ptr(espdl_model *m, const char *name)
{
    dl::TensorBase *t = (m && name) ? m->model->get_intermediate(name) : nullptr;
    return t ? t->data : nullptr;
}

int64_t espdl_model_tensor_bytes(espdl_model *m, const char *name)
{
    dl::TensorBase *t = (m && name) ? m->model->get_intermediate(name) : nullptr;
    return t ? (int64_t)t->get_bytes() : -1;
}

int espdl_model_tensor_shape(espdl_model *m, const char *name, int32_t *dims, int32_t capacity)
{
    dl::TensorBase *t = (m && name) ? m->model->get_intermediate(name) : nullptr;
    if (!t)
        return -1;
    for (int i = 0; i < (int)t->shape.size() && i < capacity; i++)
        dims[i] = t->shape[i];
    return (int)t->shape.size();
}

int espdl_model_tensor_exponent(espdl_model *m, const char *name, int32_t *exponent)
{
    dl::TensorBase *t = (m && name) ? m->model->get_intermediate(name) : nullptr;
    if (!t || !exponent)
        return -1;
    *exponent = t->exponent.get();
    return 0;
}

int espdl_model_tensor_channel_pitch(espdl_model *m, const char *name)
{
    dl::TensorBase *t = (m && name) ? m->model->get_intermediate(name) : nullptr;
    return t ? t->get_channel_pitch() : -1;
}

int espdl_model_set_input(espdl_model *m, const char *name, const void *host_data, int64_t bytes)
{
    dl::TensorBase *t = (m && name) ? m->model->get_input(name) : nullptr;
    if (!t || bytes != (int64_t)t->get_bytes())
        return -1;
    return t->copy_from_host(host_data, (size_t)bytes, m->model->get_stream()) ? 0 : -1;
}

int espdl_model_get_tensor(espdl_model *m, const char *name, void *host_data, int64_t bytes)
{
    dl::TensorBase *t = (m && name) ? m->model->get_intermediate(name) : nullptr;
    if (!t || bytes != (int64_t)t->get_bytes())
        return -1;
    return t->copy_to_host(host_data, (size_t)bytes, m->model->get_stream()) ? 0 : -1;
}

int64_t espdl_model_device_bytes(espdl_model *m)
{
    return m ? (int64_t)m->model->get_memory_info().device : -1;
}

void *espdl_model_stream(espdl_model *m)
{
    return m ? m->model->get_stream() : nullptr;
}

} // extern "C"
