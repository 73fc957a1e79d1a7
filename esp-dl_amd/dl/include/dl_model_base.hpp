// dl::Model: single-GPU batched executor of a graph of dl::module::Module objects.
//
// Public surface follows esp-dl/dl/model/include/dl_model_base.hpp:84-441 for what the operator
// path needs: construct from an fbs::FbsModel, load() (topological plan + parameters), build()
// (shape inference + static activation plan), run() in its flavours, test(), profile / module info,
// get_inputs / get_outputs / get_intermediate, print, reset.  What replaces the reference's
// internals: the static planner carves all activations of a whole BATCH from one HBM arena
// (MemoryManagerGreedy's role, esp-dl/dl/model/src/dl_memory_manager_greedy.cpp), modules enqueue
// kernels on one HIP stream, and the launch-bound plan can be replayed from a HIP graph.
#pragma once

#include <map>
#include <string>
#include <vector>

#include "dl_model_context.hpp"
#include "dl_module_base.hpp"
#include "fbs_model.hpp"

namespace dl {

struct module_info {
    std::string name;
    std::string type;
    float latency_us; ///< GPU time of one forward, from HIP events
    int64_t macs;     ///< multiply-accumulates of one forward over the whole batch
    int64_t bytes;    ///< bytes of the tensors it reads and writes (each counted once)
};

enum { FUSE_CONV_LUT = 1, FUSE_DW_PROJECT = 2, FUSE_CONV_ADD = 4, FUSE_CONV_GAP = 8, FUSE_CHANNEL_SLICES = 16 };

class Model {
public:
    /// The model does not take ownership of `fbs_model`.  `stream` is a hipStream_t (nullptr: the
    /// model creates its own).  `fuse` is a bit mask of graph fusions: FUSE_CONV_LUT folds a LUT that directly follows a Conv
    /// into its epilogue, FUSE_DW_PROJECT runs depthwise Conv -> 1x1 Conv [-> Add] as one kernel,
    /// FUSE_CONV_ADD folds the Add behind a dense Conv into its epilogue, FUSE_CONV_GAP runs a 1x1 Conv and the
    /// GlobalAveragePool behind it as one kernel that writes the pooled tensor only, FUSE_CHANNEL_SLICES leaves the
    /// outputs of a Split along the last axis inside its input and lets dense 8-bit Convs write straight into the
    /// output of a Concat along the last axis (the modules stay in the plan and copy only what is not in place).
    /// All are exact and on by default.
    Model(fbs::FbsModel *fbs_model, int batch = 1, round_mode_t round_mode = ROUND_MODE_HALF_UP, void *stream = nullptr,
          int fuse = FUSE_CONV_LUT | FUSE_DW_PROJECT | FUSE_CONV_ADD | FUSE_CONV_GAP | FUSE_CHANNEL_SLICES);
    virtual ~Model();
    Model(const Model &) = delete;
    Model &operator=(const Model &) = delete;

    virtual esp_err_t load(fbs::FbsModel *fbs_model);
    /// Infer shapes for `batch` images and place every activation in the arena.
    virtual esp_err_t build(int batch);

    /// Enqueue the whole plan and wait for it (results are valid on return, as in the reference).
    virtual void run(runtime_mode_t mode = RUNTIME_MODE_SINGLE_CORE);
    /// Copy `input` (host or device, requantized if its exponent differs) into the single graph input, then run.
    virtual void run(TensorBase *input, runtime_mode_t mode = RUNTIME_MODE_SINGLE_CORE);
    virtual void run(std::map<std::string, TensorBase *> &user_inputs, runtime_mode_t mode = RUNTIME_MODE_SINGLE_CORE,
                     std::map<std::string, TensorBase *> user_outputs = {});
    /// Run segment `stage_index` of `stage_num` near-equal segments of the plan (dl_model_base.cpp:240-260).
    virtual void run(int stage_num, int stage_index, runtime_mode_t mode = RUNTIME_MODE_SINGLE_CORE);
    /// Enqueue only; pair with synchronize().  Uses the captured HIP graph when enable_graph() succeeded.
    void run_async(runtime_mode_t mode = RUNTIME_MODE_SINGLE_CORE);
    void synchronize();
    /// Capture the plan into a HIP graph (after one eager run has created every module's device state).
    bool enable_graph();
    void disable_graph();
    bool graph_enabled() const { return m_graph_exec != nullptr; }
    /// True when a module logged an error (a rejected kernel launch, a host tensor handed to a device
    /// module) or a HIP call failed since the last run / run_async / enable_graph / test began.  The
    /// tensors a failed pass leaves behind are not valid results.
    bool last_run_failed() const { return m_failed || error_log_count().load() != m_errors_at_start; }

    /// Compare every tensor that has a test vector in the FbsModel (int8 exact, int16 within 1).
    esp_err_t test();
    std::vector<module_info> get_module_info(int repeats = 3);
    void profile(bool sort_module_by_latency = false);
    mem_info_t get_memory_info();

    virtual std::map<std::string, TensorBase *> &get_inputs() { return m_inputs; }
    virtual TensorBase *get_input();
    virtual TensorBase *get_input(const std::string &name);
    virtual TensorBase *get_intermediate(const std::string &name);
    virtual std::map<std::string, TensorBase *> &get_outputs() { return m_outputs; }
    virtual TensorBase *get_output();
    virtual TensorBase *get_output(const std::string &name);
    std::string get_metadata_prop(const std::string &key);
    virtual void print();
    virtual void reset();
    virtual fbs::FbsModel *get_fbs_model() { return m_fbs_model; }
    ModelContext *get_context() { return m_model_context; }
    void *get_stream() { return m_stream; }
    int get_batch() const { return m_batch; }
    size_t get_module_count() const { return m_execution_plan.size(); }
    dl::module::Module *get_module(size_t i) { return i < m_execution_plan.size() ? m_execution_plan[i] : nullptr; }

private:
    void fuse_conv_lut();
    void fuse_dw_project();
    void fuse_conv_add();
    void fuse_conv_gap();

    fbs::FbsModel *m_fbs_model = nullptr;
    std::vector<dl::module::Module *> m_execution_plan;
    ModelContext *m_model_context = nullptr;
    std::map<std::string, TensorBase *> m_inputs, m_outputs;
    std::string m_name, m_doc_string;
    int64_t m_version = 0;
    int m_batch = 1;
    int m_fuse = FUSE_CONV_LUT | FUSE_DW_PROJECT | FUSE_CONV_ADD | FUSE_CONV_GAP | FUSE_CHANNEL_SLICES;
    void *m_stream = nullptr;
    bool m_own_stream = false;
    void *m_graph = nullptr;      // hipGraph_t
    void *m_graph_exec = nullptr; // hipGraphExec_t
    bool m_built = false;
    bool m_failed = false;
    long m_errors_at_start = 0;
    void begin_pass()
    {
        m_failed = false;
        m_errors_at_start = error_log_count().load();
    }
};

} // namespace dl
