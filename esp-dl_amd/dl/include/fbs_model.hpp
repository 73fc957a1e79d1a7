// fbs::FbsModel: the graph description a dl::Model is built from.
//
// In the reference this class wraps a FlatBuffers `.espdl` blob and ships only as a prebuilt
// library; its accessor surface is public (esp-dl/fbs_loader/include/fbs_model.hpp:23-424) and is
// what every Module::deserialize reads.  Here the same accessors sit on a plain in-memory graph that
// is filled programmatically (add_node / add_initializer / add_value_info ...), which is the
// loader-free construction path the reference lacks.
#pragma once

#include <map>
#include <string>
#include <vector>

#include "dl_tensor_base.hpp"

namespace fbs {

struct Attribute {
    enum Kind { NONE, INT, FLOAT, STRING, INTS, FLOATS } kind = NONE;
    int64_t i = 0;
    float f = 0.f;
    std::string s;
    std::vector<int64_t> ints;
    std::vector<float> floats;
};

struct Node {
    std::string name;
    std::string op_type;
    std::vector<std::string> inputs;
    std::vector<std::string> outputs;
    std::map<std::string, Attribute> attributes;
};

struct Initializer {
    std::vector<int> dims;
    dl::dtype_t dtype = dl::DATA_TYPE_UNDEFINED;
    std::vector<int> exponents;
    std::vector<uint8_t> bytes; // host copy, layout as the reference's `c` target stores it
};

struct ValueInfo {
    std::vector<int> dims; // per-image shape with a leading 1, as exported
    dl::dtype_t dtype = dl::DATA_TYPE_UNDEFINED;
    int exponent = 0;
};

class FbsModel {
public:
    FbsModel() {}
    ~FbsModel() {}

    // ---- construction ------------------------------------------------------------------------
    void set_model_info(const std::string &name, int64_t version = 0, const std::string &doc = "")
    {
        m_name = name;
        m_version = version;
        m_doc = doc;
    }
    void set_metadata_prop(const std::string &key, const std::string &value) { m_metadata[key] = value; }
    Node *add_node(const std::string &name, const std::string &op_type, const std::vector<std::string> &inputs,
                   const std::vector<std::string> &outputs);
    Node *get_node(const std::string &name);
    void add_initializer(const std::string &name, const std::vector<int> &dims, dl::dtype_t dtype, const void *data,
                         const std::vector<int> &exponents);
    void add_value_info(const std::string &name, const std::vector<int> &dims, dl::dtype_t dtype, int exponent);
    void add_graph_input(const std::string &name) { m_inputs.push_back(name); }
    void add_graph_output(const std::string &name) { m_outputs.push_back(name); }
    void add_test_input(const std::string &name, const std::vector<int> &dims, dl::dtype_t dtype, const void *data,
                        int exponent);
    void add_test_output(const std::string &name, const std::vector<int> &dims, dl::dtype_t dtype, const void *data,
                         int exponent);

    // ---- accessors with the reference's names ------------------------------------------------
    std::vector<std::string> topological_sort();
    esp_err_t get_operation_attribute(std::string node_name, std::string attribute_name, int &ret_value);
    esp_err_t get_operation_attribute(std::string node_name, std::string attribute_name, float &ret_value);
    esp_err_t get_operation_attribute(std::string node_name, std::string attribute_name, std::string &ret_value);
    esp_err_t get_operation_attribute(std::string node_name, std::string attribute_name, std::vector<int> &ret_value);
    esp_err_t get_operation_attribute(std::string node_name, std::string attribute_name, std::vector<float> &ret_value);
    esp_err_t get_operation_attribute(std::string node_name, std::string attribute_name, dl::quant_type_t &ret_value);
    esp_err_t get_operation_attribute(std::string node_name, std::string attribute_name,
                                      dl::activation_type_t &ret_value);
    esp_err_t get_operation_inputs_and_outputs(std::string node_name, std::vector<std::string> &inputs,
                                               std::vector<std::string> &outputs);
    std::string get_operation_type(std::string node_name);
    /// New host TensorBase holding a copy of the index-th input of the node when that input is an
    /// initializer, else nullptr.  The caller owns it.
    dl::TensorBase *get_operation_parameter(std::string node_name, int index = 1, uint32_t caps = MALLOC_CAP_DEFAULT);
    /// LUT initializer named by the node's string attribute `lut` (nullptr when absent).
    dl::TensorBase *get_operation_lut(std::string node_name, uint32_t caps = MALLOC_CAP_DEFAULT,
                                      std::string attribute_name = "lut");
    bool is_parameter(std::string name);
    const void *get_tensor_raw_data(std::string tensor_name);
    dl::dtype_t get_tensor_dtype(std::string tensor_name);
    std::vector<int> get_tensor_shape(std::string tensor_name);
    std::vector<int> get_tensor_exponents(std::string tensor_name);
    dl::dtype_t get_value_info_dtype(std::string var_name);
    std::vector<int> get_value_info_shape(std::string var_name);
    int get_value_info_exponent(std::string var_name);
    bool has_value_info(const std::string &var_name) { return m_value_info.count(var_name) != 0; }
    dl::TensorBase *get_test_input_tensor(std::string tensor_name);
    dl::TensorBase *get_test_output_tensor(std::string tensor_name);
    std::vector<std::string> get_test_outputs_name();
    std::vector<std::string> get_graph_inputs() { return m_inputs; }
    std::vector<std::string> get_graph_outputs() { return m_outputs; }
    std::string get_model_name() { return m_name; }
    int64_t get_model_version() { return m_version; }
    std::string get_model_doc_string() { return m_doc; }
    std::string get_model_metadata_prop(const std::string &key);
    void load_map() {}
    void clear_map() {}
    void print();

private:
    const Attribute *find_attribute(const std::string &node_name, const std::string &attribute_name);
    dl::TensorBase *tensor_from(const Initializer &init, uint32_t caps);

    std::string m_name, m_doc;
    int64_t m_version = 0;
    std::map<std::string, std::string> m_metadata;
    std::vector<Node> m_nodes;
    std::map<std::string, size_t> m_node_index;
    std::map<std::string, Initializer> m_initializers;
    std::map<std::string, ValueInfo> m_value_info;
    std::vector<std::string> m_inputs, m_outputs;
    std::map<std::string, Initializer> m_test_inputs, m_test_outputs;
    std::vector<std::string> m_test_output_order;
};

} // namespace fbs
