#include "dl_model_base.hpp"
#include "espdl_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <set>
#include <typeinfo>

#include "dl_module_creator.hpp"

namespace dl {

namespace {
const char *TAG = "dl::Model";

bool hip_ok(hipError_t e, const char *what)
{
    if (e != hipSuccess) {
        DL_LOGE(TAG, "%s failed: %s", what, hipGetErrorString(e));
        return false;
    }
    return true;
}

dtype_t dtype_of(quant_type_t q)
{
    switch (q) {
    case QUANT_TYPE_SYMM_16BIT:
        return DATA_TYPE_INT16;
    case QUANT_TYPE_FLOAT32:
        return DATA_TYPE_FLOAT;
    default:
        return DATA_TYPE_INT8;
    }
}

// One block of the activation arena.
struct Block {
    size_t offset, bytes;
    int users; // tensors currently living in it
};

// First-fit free list over a linear arena: the role MemoryManagerGreedy plays in the reference.
class ArenaPlanner {
public:
    size_t alloc(size_t bytes)
    {
        bytes = (bytes + 255) & ~(size_t)255;
        if (bytes == 0)
            bytes = 256;
        size_t best = m_free.size();
        for (size_t i = 0; i < m_free.size(); i++)
            if (m_free[i].second >= bytes && (best == m_free.size() || m_free[i].second < m_free[best].second))
                best = i;
        if (best != m_free.size()) {
            const size_t off = m_free[best].first;
            if (m_free[best].second == bytes)
                m_free.erase(m_free.begin() + best);
            else {
                m_free[best].first += bytes;
                m_free[best].second -= bytes;
            }
            return off;
        }
        // grow; if the last free range touches the end of the arena, extend it instead
        if (!m_free.empty() && m_free.back().first + m_free.back().second == m_top) {
            const size_t off = m_free.back().first;
            m_top = off + bytes;
            m_free.pop_back();
            return off;
        }
        const size_t off = m_top;
        m_top += bytes;
        return off;
    }
    void release(size_t offset, size_t bytes)
    {
        bytes = (bytes + 255) & ~(size_t)255;
        if (bytes == 0)
            bytes = 256;
        m_free.push_back({offset, bytes});
        std::sort(m_free.begin(), m_free.end());
        for (size_t i = 0; i + 1 < m_free.size();) {
            if (m_free[i].first + m_free[i].second == m_free[i + 1].first) {
                m_free[i].second += m_free[i + 1].second;
                m_free.erase(m_free.begin() + i + 1);
            } else {
                i++;
            }
        }
    }
    size_t top() const { return m_top; }

private:
    std::vector<std::pair<size_t, size_t>> m_free;
    size_t m_top = 0;
};

} // namespace

Model::Model(fbs::FbsModel *fbs_model, int batch, round_mode_t round_mode, void *stream, int fuse) :
    m_batch(batch), m_fuse(fuse), m_stream(stream)
{
    m_model_context = new ModelContext();
    m_model_context->owns_tensors = true;
    m_model_context->round_mode = round_mode;
    if (!m_stream) {
        hipStream_t s = nullptr;
        if (hip_ok(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreateWithFlags")) {
            m_stream = s;
            m_own_stream = true;
        }
    }
    m_model_context->stream = m_stream;
    if (load(fbs_model) == ESP_OK)
        build(batch);
}

Model::~Model()
{
    disable_graph();
    if (m_stream)
        (void)hipStreamSynchronize(static_cast<hipStream_t>(m_stream));
    for (auto *m : m_execution_plan)
        delete m;
    m_execution_plan.clear();
    delete m_model_context;
    if (m_own_stream && m_stream)
        (void)hipStreamDestroy(static_cast<hipStream_t>(m_stream));
}

esp_err_t Model::load(fbs::FbsModel *fbs_model)
{
    if (!fbs_model) {
        DL_LOGE(TAG, "Fail to load model");
        return ESP_FAIL;
    }
    esp_err_t ret = ESP_OK;
    m_fbs_model = fbs_model;
    m_name = fbs_model->get_model_name();
    m_version = fbs_model->get_model_version();
    m_doc_string = fbs_model->get_model_doc_string();
    m_built = false;

    for (auto *m : m_execution_plan)
        delete m;
    m_execution_plan.clear();
    m_model_context->clear();
    auto *creator = dl::module::ModuleCreator::get_instance();
    std::vector<std::string> op_inputs, op_outputs;
    for (const std::string &node_name : fbs_model->topological_sort()) {
        const std::string op_type = fbs_model->get_operation_type(node_name);
        if (op_type.empty()) {
            DL_LOGE(TAG, "Can not find the operation %s", node_name.c_str());
            ret = ESP_FAIL;
            break;
        }
        dl::module::Module *module = creator->create(fbs_model, op_type, node_name);
        if (!module) {
            DL_LOGE(TAG, "Do not support %s, please implement and register it first.", op_type.c_str());
            ret = ESP_FAIL;
            break;
        }
        m_execution_plan.push_back(module);
        fbs_model->get_operation_inputs_and_outputs(node_name, op_inputs, op_outputs);
        for (size_t j = 0; j < op_inputs.size(); j++) {
            int index;
            if (fbs_model->is_parameter(op_inputs[j]) || op_inputs[j].empty()) {
                TensorBase *param = nullptr;
                if (m_model_context->get_tensor_index(op_inputs[j]) < 0)
                    param = fbs_model->get_operation_parameter(node_name, (int)j, MALLOC_CAP_DEVICE);
                index = m_model_context->add_tensor(op_inputs[j], true, param);
            } else {
                index = m_model_context->add_tensor(op_inputs[j], false, nullptr);
            }
            module->m_inputs_index.push_back(index);
        }
        for (size_t j = 0; j < op_outputs.size(); j++)
            module->m_outputs_index.push_back(m_model_context->add_tensor(op_outputs[j], false, nullptr));
    }
    if (ret == ESP_OK && (m_fuse & FUSE_CONV_LUT))
        fuse_conv_lut();
    if (ret == ESP_OK && (m_fuse & FUSE_DW_PROJECT))
        fuse_dw_project();
    if (ret == ESP_OK && (m_fuse & FUSE_CONV_ADD))
        fuse_conv_add();
    if (ret == ESP_OK && (m_fuse & FUSE_CONV_GAP))
        fuse_conv_gap();
    return ret;
}

// The module as an Add, or nullptr: classes derived from Add (Mul) share its operand handling but
// not its arithmetic, so they must never be absorbed as a residual addition.
static dl::module::Add *plain_add(dl::module::Module *m)
{
    return m && typeid(*m) == typeid(dl::module::Add) ? static_cast<dl::module::Add *>(m) : nullptr;
}

// Conv -> LUT with no other reader of the conv output: the table moves into the conv's epilogue and
// the conv writes the LUT's output tensor directly.
void Model::fuse_conv_lut()
{
    std::set<std::string> pinned; // tensors that must keep existing
    for (auto &n : m_fbs_model->get_graph_outputs())
        pinned.insert(n);
    for (auto &n : m_fbs_model->get_test_outputs_name())
        pinned.insert(n);
    for (size_t i = 0; i < m_execution_plan.size(); i++) {
        auto *conv = dynamic_cast<dl::module::Conv *>(m_execution_plan[i]);
        if (!conv || conv->quant_type != QUANT_TYPE_SYMM_8BIT || conv->has_fused_lut())
            continue;
        const int mid = conv->m_outputs_index[0];
        if (pinned.count(m_model_context->get_tensor_name(mid)))
            continue;
        int readers = 0;
        size_t lut_pos = 0;
        for (size_t j = 0; j < m_execution_plan.size(); j++)
            for (int in : m_execution_plan[j]->m_inputs_index)
                if (in == mid) {
                    readers++;
                    lut_pos = j;
                }
        if (readers != 1)
            continue;
        auto *lut = dynamic_cast<dl::module::LUT *>(m_execution_plan[lut_pos]);
        if (!lut || lut->quant_type != QUANT_TYPE_SYMM_8BIT || !lut->get_table() || lut->get_table()->get_size() != 256)
            continue;
        conv->fuse_lut(lut->release_table(),
                       m_fbs_model->get_value_info_exponent(m_model_context->get_tensor_name(mid)));
        conv->m_outputs_index[0] = lut->m_outputs_index[0];
        delete lut;
        m_execution_plan.erase(m_execution_plan.begin() + lut_pos);
        if (lut_pos < i)
            i--;
    }
}

// depthwise Conv -> 1x1 Conv [-> Add]: when the depthwise output has no other reader (and, for the
// Add, the project output has none either) the chain becomes one module that keeps the depthwise
// result on chip (espdl_hip_mbconv_s8 without expand stage).  Every value is formed exactly as the
// separate modules form it, so results do not change.  The fused module takes the place of the last
// module it absorbs, so everything it reads (the Add's other operand included) is produced before it.
void Model::fuse_dw_project()
{
    std::set<std::string> pinned;
    for (auto &n : m_fbs_model->get_graph_outputs())
        pinned.insert(n);
    for (auto &n : m_fbs_model->get_test_outputs_name())
        pinned.insert(n);
    auto single_reader = [&](int tensor, size_t *pos) {
        int readers = 0;
        for (size_t j = 0; j < m_execution_plan.size(); j++)
            for (int in : m_execution_plan[j]->m_inputs_index)
                if (in == tensor) {
                    readers++;
                    *pos = j;
                }
        return readers == 1 && !pinned.count(m_model_context->get_tensor_name(tensor));
    };
    // A Clip whose input and output exponents are equal is a clamp of the stored value
    // (esp-dl/dl/module/include/dl_module_clip.hpp:78-90 with a rescale factor of 1): between two stages of the
    // block it can run inside the launch.  Returns the module when `m` is such a Clip with one data input.
    auto clamp_only = [&](dl::module::Module *m) -> dl::module::Clip * {
        auto *clip = dynamic_cast<dl::module::Clip *>(m);
        if (!clip || clip->quant_type != QUANT_TYPE_SYMM_8BIT || clip->m_inputs_index.empty() || clip->m_outputs_index.size() != 1 ||
            clip->m_inputs_index[0] >= CONTEXT_PARAMETER_OFFSET)
            return nullptr;
        const std::string in_name = m_model_context->get_tensor_name(clip->m_inputs_index[0]);
        const std::string out_name = m_model_context->get_tensor_name(clip->m_outputs_index[0]);
        if (!m_fbs_model->has_value_info(in_name) || !m_fbs_model->has_value_info(out_name) ||
            m_fbs_model->get_value_info_exponent(in_name) != m_fbs_model->get_value_info_exponent(out_name))
            return nullptr;
        clip->read_bounds(m_model_context);
        return clip->get_min() <= clip->get_max() ? clip : nullptr;
    };
    auto plain_act = [](dl::module::Conv *c) { return c->get_activation() == Linear || c->get_activation() == ReLU; };
    for (size_t i = 0; i < m_execution_plan.size(); i++) {
        auto *dw = dynamic_cast<dl::module::Conv *>(m_execution_plan[i]);
        if (!dw || dw->quant_type != QUANT_TYPE_SYMM_8BIT || dw->get_group() == 1 || dw->has_fused_lut() ||
            dw->has_fused_project() || dw->get_pads().size() != 4 || !plain_act(dw))
            continue;
        int mid = dw->m_outputs_index[0]; // the tensor the project Conv reads
        size_t pj_pos = 0;
        if (!single_reader(mid, &pj_pos) || pj_pos <= i)
            continue;
        dl::module::Clip *clip_d = clamp_only(m_execution_plan[pj_pos]);
        if (clip_d) {
            mid = clip_d->m_outputs_index[0];
            if (!single_reader(mid, &pj_pos) || pj_pos <= i)
                continue;
        }
        auto *pj = dynamic_cast<dl::module::Conv *>(m_execution_plan[pj_pos]);
        if (!pj || pj->quant_type != QUANT_TYPE_SYMM_8BIT || pj->get_group() != 1 || pj->has_fused_lut() ||
            pj->has_fused_project() || pj->m_inputs_index[0] != mid || !plain_act(pj))
            continue;
        TensorBase *pf = m_model_context->get_tensor(pj->m_inputs_index[1]);
        TensorBase *df = m_model_context->get_tensor(dw->m_inputs_index[1]);
        const std::vector<int> in_shape = m_fbs_model->get_value_info_shape(m_model_context->get_tensor_name(dw->m_inputs_index[0]));
        if (!pf || !df || pf->shape.size() != 4 || df->shape.size() != 4 || pf->shape[0] != 1 || pf->shape[1] != 1 ||
            in_shape.size() != 4)
            continue;
        bool plain = true; // 1x1, stride 1, no padding, no dilation
        for (int v : pj->get_pads())
            plain = plain && v == 0;
        for (int v : pj->get_strides())
            plain = plain && v == 1;
        for (int v : pj->get_dilations())
            plain = plain && v == 1;
        if (!plain)
            continue;
        espdl_hip_mbconv_desc d = {};
        d.batch = 1;
        d.in_h = in_shape[1];
        d.in_w = in_shape[2];
        d.in_c = in_shape[3];
        d.exp_c = d.in_c;
        d.out_c = pf->shape[3];
        d.k_h = df->shape[0];
        d.k_w = df->shape[1];
        d.stride_h = dw->get_strides()[0];
        d.stride_w = dw->get_strides()[1];
        d.dil_h = dw->get_dilations()[0];
        d.dil_w = dw->get_dilations()[1];
        d.pad_top = dw->get_pads()[0];
        d.pad_bottom = dw->get_pads()[1];
        d.pad_left = dw->get_pads()[2];
        d.pad_right = dw->get_pads()[3];
        d.n_shift_expand = d.n_shift_dw = d.n_shift_project = 1;
        if (clip_d) {
            d.clip_dw = 1;
            d.clip_dw_min = clip_d->get_min();
            d.clip_dw_max = clip_d->get_max();
        }
        if (pf->shape[2] != d.in_c)
            continue;
        // The 1x1 Conv in front (the expand stage of an inverted-residual block) joins when the single
        // launch of the whole block is the preferred form for this batch; otherwise depthwise + project
        // fuse where the depthwise+project kernel applies.  A clamp-only Clip may stand between the two.
        dl::module::Conv *ex = nullptr;
        dl::module::Clip *clip_e = nullptr;
        int ex_kernel[2] = {1, 1};
        espdl_hip_mbconv_desc de = d; // the whole block, when a Conv in front joins
        {
            int dw_in = dw->m_inputs_index[0];
            size_t reader = 0;
            dl::module::Module *producer = nullptr;
            for (size_t j = 0; j < i; j++)
                if (m_execution_plan[j]->m_outputs_index.size() == 1 && m_execution_plan[j]->m_outputs_index[0] == dw_in)
                    producer = m_execution_plan[j];
            if (producer && (clip_e = clamp_only(producer)) != nullptr) {
                if (!single_reader(dw_in, &reader)) {
                    clip_e = nullptr;
                    producer = nullptr;
                } else {
                    dw_in = clip_e->m_inputs_index[0];
                    producer = nullptr;
                    for (size_t j = 0; j < i; j++)
                        if (m_execution_plan[j]->m_outputs_index.size() == 1 && m_execution_plan[j]->m_outputs_index[0] == dw_in)
                            producer = m_execution_plan[j];
                }
            }
            ex = dynamic_cast<dl::module::Conv *>(producer);
            if (ex && (ex->quant_type != QUANT_TYPE_SYMM_8BIT || ex->get_group() != 1 || ex->has_fused_lut() ||
                       ex->has_fused_project() || ex->has_fused_residual() || !single_reader(dw_in, &reader) ||
                       ex->get_pads().size() != 4 || !plain_act(ex)))
                ex = nullptr;
            TensorBase *ef = ex ? m_model_context->get_tensor(ex->m_inputs_index[1]) : nullptr;
            if (ex && (!ef || ef->shape.size() != 4 || ef->shape[3] != d.in_c))
                ex = nullptr;
            bool plain_ex = true; // 1x1, stride 1, no padding
            if (ex) {
                plain_ex = ef->shape[0] == 1 && ef->shape[1] == 1;
                for (int v : ex->get_pads())
                    plain_ex = plain_ex && v == 0;
                for (int v : ex->get_strides())
                    plain_ex = plain_ex && v == 1;
                for (int v : ex->get_dilations())
                    if (v != 1)
                        ex = nullptr; // no kernel takes a dilated expand stage
            }
            std::vector<int> ex_in_shape;
            if (ex) {
                ex_kernel[0] = ef->shape[0];
                ex_kernel[1] = ef->shape[1];
                ex_in_shape = m_fbs_model->get_value_info_shape(m_model_context->get_tensor_name(ex->m_inputs_index[0]));
                if (ex_in_shape.size() != 4 || ex->get_strides().size() != 2)
                    ex = nullptr;
            }
            if (ex) {
                de.batch = m_batch;
                de.has_expand = 1;
                de.exp_c = d.in_c;
                de.in_c = ef->shape[2];
                if (clip_e) {
                    de.clip_expand = 1;
                    de.clip_expand_min = clip_e->get_min();
                    de.clip_expand_max = clip_e->get_max();
                }
                if (!plain_ex) {
                    // a convolution with a window (a stem) as the expand stage: the block input is its input
                    de.in_h = ex_in_shape[1];
                    de.in_w = ex_in_shape[2];
                    de.exp_k_h = ef->shape[0];
                    de.exp_k_w = ef->shape[1];
                    de.exp_stride_h = ex->get_strides()[0];
                    de.exp_stride_w = ex->get_strides()[1];
                    de.exp_pad_top = ex->get_pads()[0];
                    de.exp_pad_bottom = ex->get_pads()[1];
                    de.exp_pad_left = ex->get_pads()[2];
                    de.exp_pad_right = ex->get_pads()[3];
                }
                if (espdl_hip_mbconv_s8_preferred(&de) != 1)
                    ex = nullptr;
            }
            if (!ex)
                clip_e = nullptr; // a Clip in front of a depthwise Conv that stays on its own stays too
        }
        if (!ex && espdl_hip_mbconv_s8_supported(&d) != 2)
            continue;

        // optional Add behind the project conv
        int out_index = pj->m_outputs_index[0];
        int residual = -1;
        size_t add_pos = 0;
        dl::module::Add *add = nullptr;
        if (single_reader(out_index, &add_pos) && add_pos > pj_pos) {
            add = plain_add(m_execution_plan[add_pos]);
            if (add && add->quant_type == QUANT_TYPE_SYMM_8BIT && add->m_inputs_index.size() == 2 &&
                add->m_inputs_index[0] != add->m_inputs_index[1]) {
                const int other = add->m_inputs_index[0] == out_index ? add->m_inputs_index[1] : add->m_inputs_index[0];
                const std::string other_name = m_model_context->get_tensor_name(other);
                const std::string out_name = m_model_context->get_tensor_name(out_index);
                if (other < CONTEXT_PARAMETER_OFFSET && m_fbs_model->has_value_info(other_name) &&
                    m_fbs_model->get_value_info_shape(other_name) == m_fbs_model->get_value_info_shape(out_name)) {
                    residual = other;
                    out_index = add->m_outputs_index[0];
                } else {
                    add = nullptr;
                }
            } else {
                add = nullptr;
            }
        }
        const int mid_exp = m_fbs_model->get_value_info_exponent(m_model_context->get_tensor_name(mid));
        const int pj_out_exp = m_fbs_model->get_value_info_exponent(m_model_context->get_tensor_name(pj->m_outputs_index[0]));
        // A RequantizeLinear whose only reader is the Add (the exporter's way of re-scaling the residual operand)
        // joins the launch of a whole block: the kernel requantizes the operand in registers (residual_shift
        // of the descriptor = exponent of the node's input - exponent of its output; the Add itself adds raw
        // values whatever the exponents say, as the reference's does).
        dl::module::Module *rq = nullptr;
        int rq_shift = 0;
        if (ex && residual >= 0) {
            size_t rq_reader = 0;
            for (size_t j = 0; j < add_pos; j++)
                if (m_execution_plan[j]->m_outputs_index.size() == 1 && m_execution_plan[j]->m_outputs_index[0] == residual)
                    rq = dynamic_cast<dl::module::RequantizeLinear *>(m_execution_plan[j]);
            // (exported files give the node its scale and zero point as further, constant inputs)
            if (rq && (rq->m_inputs_index.empty() || rq->m_inputs_index[0] >= CONTEXT_PARAMETER_OFFSET ||
                       !single_reader(residual, &rq_reader)))
                rq = nullptr;
            if (rq) {
                const std::string src_name = m_model_context->get_tensor_name(rq->m_inputs_index[0]);
                const std::string res_name = m_model_context->get_tensor_name(residual);
                const int shift = m_fbs_model->has_value_info(src_name)
                    ? m_fbs_model->get_value_info_exponent(src_name) - m_fbs_model->get_value_info_exponent(res_name)
                    : 0;
                de.residual_shift = shift;
                rq_shift = shift;
                if (!m_fbs_model->has_value_info(src_name) || m_fbs_model->get_value_info_dtype(src_name) != DATA_TYPE_INT8 ||
                    m_fbs_model->get_value_info_dtype(res_name) != DATA_TYPE_INT8 ||
                    m_fbs_model->get_value_info_shape(src_name) != m_fbs_model->get_value_info_shape(res_name) || shift == 0 ||
                    shift < -7 || shift > 7 || espdl_hip_mbconv_s8_preferred(&de) != 1)
                    rq = nullptr;
                else
                    residual = rq->m_inputs_index[0];
            }
        }
        dw->fuse_project(pj->m_inputs_index[1], pj->m_inputs_index.size() == 3 ? pj->m_inputs_index[2] : -1,
                         pj->get_activation(), mid_exp, residual, pj_out_exp, rq != nullptr ? rq_shift : 0);
        dw->m_outputs_index[0] = out_index;
        if (clip_d)
            dw->fuse_clip(1, clip_d->get_min(), clip_d->get_max());
        if (ex) {
            dw->fuse_expand(ex->m_inputs_index[0], ex->m_inputs_index[1],
                            ex->m_inputs_index.size() == 3 ? ex->m_inputs_index[2] : -1, ex->get_activation(),
                            m_fbs_model->get_value_info_exponent(m_model_context->get_tensor_name(ex->m_outputs_index[0])),
                            {ex_kernel[0], ex_kernel[1]}, ex->get_strides(), ex->get_pads());
            if (clip_e)
                dw->fuse_clip(0, clip_e->get_min(), clip_e->get_max());
        }
        // The fused module takes the slot of the last module it absorbs (everything it reads, the residual
        // operand included, is produced before that); the absorbed modules leave the plan.  The scan then starts
        // over: positions have moved, and modules already fused are skipped by their flag.
        dl::module::Module *last = add ? static_cast<dl::module::Module *>(add) : static_cast<dl::module::Module *>(pj);
        std::vector<dl::module::Module *> gone = {pj, add, ex, rq, clip_e, clip_d};
        std::vector<dl::module::Module *> plan;
        for (dl::module::Module *m : m_execution_plan) {
            if (m == dw)
                continue;
            if (m == last)
                plan.push_back(dw);
            if (std::find(gone.begin(), gone.end(), m) == gone.end())
                plan.push_back(m);
        }
        for (dl::module::Module *m : gone)
            delete m;
        m_execution_plan.swap(plan);
        i = (size_t)-1;
    }
}

// 1x1 Conv -> GlobalAveragePool with no other reader of the conv output (the head of a classification
// network): one kernel forms the convolution's int8 results, sums them per image and filter and writes the
// pooled tensor only (espdl_hip_conv2d_gap_s8); the convolution's output tensor disappears from the plan.
void Model::fuse_conv_gap()
{
    std::set<std::string> pinned;
    for (auto &n : m_fbs_model->get_graph_outputs())
        pinned.insert(n);
    for (auto &n : m_fbs_model->get_test_outputs_name())
        pinned.insert(n);
    for (size_t i = 0; i < m_execution_plan.size(); i++) {
        auto *conv = dynamic_cast<dl::module::Conv *>(m_execution_plan[i]);
        if (!conv || conv->quant_type != QUANT_TYPE_SYMM_8BIT || conv->get_group() != 1 || conv->has_fused_lut() ||
            conv->has_fused_project() || conv->has_fused_residual() || conv->has_fused_gap() || conv->get_pads().size() != 4 ||
            (conv->get_activation() != Linear && conv->get_activation() != ReLU))
            continue;
        const int mid = conv->m_outputs_index[0];
        const std::string mid_name = m_model_context->get_tensor_name(mid);
        if (pinned.count(mid_name))
            continue;
        int readers = 0;
        size_t gap_pos = 0;
        for (size_t j = 0; j < m_execution_plan.size(); j++)
            for (int in : m_execution_plan[j]->m_inputs_index)
                if (in == mid) {
                    readers++;
                    gap_pos = j;
                }
        if (readers != 1 || gap_pos <= i)
            continue;
        auto *gap = dynamic_cast<dl::module::GlobalAveragePool *>(m_execution_plan[gap_pos]);
        TensorBase *filter = m_model_context->get_tensor(conv->m_inputs_index[1]);
        const std::vector<int> in_shape = m_fbs_model->get_value_info_shape(m_model_context->get_tensor_name(conv->m_inputs_index[0]));
        if (!gap || gap->quant_type != QUANT_TYPE_SYMM_8BIT || !filter || filter->shape.size() != 4 || in_shape.size() != 4)
            continue;
        espdl_hip_conv_desc d = {};
        d.dtype = ESPDL_HIP_S8;
        d.batch = 1;
        d.in_h = in_shape[1];
        d.in_w = in_shape[2];
        d.in_c = in_shape[3];
        d.out_c = filter->shape[3];
        d.k_h = filter->shape[0];
        d.k_w = filter->shape[1];
        d.stride_h = conv->get_strides()[0];
        d.stride_w = conv->get_strides()[1];
        d.dil_h = conv->get_dilations()[0];
        d.dil_w = conv->get_dilations()[1];
        d.pad_top = conv->get_pads()[0];
        d.pad_bottom = conv->get_pads()[1];
        d.pad_left = conv->get_pads()[2];
        d.pad_right = conv->get_pads()[3];
        d.group = 1;
        d.n_shift = 1;
        if (espdl_hip_conv2d_gap_s8_supported(&d) != 1)
            continue;
        conv->fuse_gap(m_fbs_model->get_value_info_exponent(mid_name));
        conv->m_outputs_index[0] = gap->m_outputs_index[0];
        delete gap;
        m_execution_plan.erase(m_execution_plan.begin() + gap_pos);
    }
}

// dense Conv -> Add with no other reader of the conv output: the Add's other operand becomes the
// conv's residual input and the conv writes the Add's output (espdl_hip_conv2d_add).  The fused module
// takes the Add's place in the plan, so the other operand is produced before it.
void Model::fuse_conv_add()
{
    std::set<std::string> pinned;
    for (auto &n : m_fbs_model->get_graph_outputs())
        pinned.insert(n);
    for (auto &n : m_fbs_model->get_test_outputs_name())
        pinned.insert(n);
    for (size_t i = 0; i < m_execution_plan.size(); i++) {
        auto *conv = dynamic_cast<dl::module::Conv *>(m_execution_plan[i]);
        if (!conv || conv->quant_type != QUANT_TYPE_SYMM_8BIT || conv->get_group() != 1 || conv->has_fused_project() ||
            conv->has_fused_residual())
            continue;
        const int mid = conv->m_outputs_index[0];
        if (pinned.count(m_model_context->get_tensor_name(mid)))
            continue;
        int readers = 0;
        size_t add_pos = 0;
        for (size_t j = 0; j < m_execution_plan.size(); j++)
            for (int in : m_execution_plan[j]->m_inputs_index)
                if (in == mid) {
                    readers++;
                    add_pos = j;
                }
        if (readers != 1 || add_pos <= i)
            continue;
        auto *add = plain_add(m_execution_plan[add_pos]);
        if (!add || add->quant_type != QUANT_TYPE_SYMM_8BIT || add->m_inputs_index.size() != 2 ||
            add->m_inputs_index[0] == add->m_inputs_index[1])
            continue;
        const int other = add->m_inputs_index[0] == mid ? add->m_inputs_index[1] : add->m_inputs_index[0];
        const std::string other_name = m_model_context->get_tensor_name(other);
        const std::string mid_name = m_model_context->get_tensor_name(mid);
        if (other >= CONTEXT_PARAMETER_OFFSET || !m_fbs_model->has_value_info(other_name) ||
            m_fbs_model->get_value_info_shape(other_name) != m_fbs_model->get_value_info_shape(mid_name))
            continue;
        conv->fuse_residual(other, m_fbs_model->get_value_info_exponent(mid_name));
        conv->m_outputs_index[0] = add->m_outputs_index[0];
        delete add;
        m_execution_plan[add_pos] = conv;
        m_execution_plan.erase(m_execution_plan.begin() + i);
        i--;
    }
}

esp_err_t Model::build(int batch)
{
    if (!m_fbs_model || batch <= 0)
        return ESP_FAIL;
    disable_graph();
    m_batch = batch;
    ModelContext *ctx = m_model_context;
    const int n_var = ctx->get_variable_count();

    // drop activations of a previous build
    for (int i = 1; i < n_var; i++) {
        delete ctx->m_variables[i];
        ctx->m_variables[i] = nullptr;
    }
    ctx->root_free();

    // 1. shapes, dtypes and exponents of every variable
    struct VarInfo {
        std::vector<int> shape;
        dtype_t dtype = DATA_TYPE_INT8;
        int exponent = 0;
        int first = -1, last = -1; // producing module, last reading module
        bool known = false;
        int alias_of = -1; // view of another variable's bytes
        int slice_of = -1; // channel slice of this (wider) variable, starting at channel slice_at of it
        int slice_at = 0;
    };
    std::vector<VarInfo> vars(n_var);
    const int plan_size = (int)m_execution_plan.size();
    for (const std::string &name : m_fbs_model->get_graph_inputs()) {
        const int idx = ctx->get_variable_index(name);
        if (idx < 0) {
            DL_LOGE(TAG, "graph input %s feeds no node", name.c_str());
            return ESP_FAIL;
        }
        VarInfo &v = vars[idx];
        v.shape = m_fbs_model->get_value_info_shape(name);
        if (v.shape.empty()) {
            DL_LOGE(TAG, "graph input %s has no shape", name.c_str());
            return ESP_FAIL;
        }
        v.shape[0] *= batch; // exported shapes carry a leading 1
        v.dtype = m_fbs_model->get_value_info_dtype(name);
        v.exponent = m_fbs_model->get_value_info_exponent(name);
        v.known = true;
        v.first = -1;
    }
    for (int i = 0; i < plan_size; i++) {
        dl::module::Module *m = m_execution_plan[i];
        std::vector<std::vector<int>> in_shapes;
        for (int idx : m->m_inputs_index) {
            if (idx >= CONTEXT_PARAMETER_OFFSET) {
                TensorBase *p = ctx->get_tensor(idx);
                in_shapes.push_back(p ? p->shape : std::vector<int>());
            } else {
                if (!vars[idx].known) {
                    DL_LOGE(TAG, "%s reads %s before it is produced", m->name.c_str(), ctx->get_tensor_name(idx).c_str());
                    return ESP_FAIL;
                }
                in_shapes.push_back(vars[idx].shape);
                vars[idx].last = i;
            }
        }
        std::vector<std::vector<int>> out_shapes = m->get_output_shape(in_shapes);
        bool shapes_ok = out_shapes.size() >= m->m_outputs_index.size();
        for (size_t j = 0; shapes_ok && j < m->m_outputs_index.size(); j++) {
            shapes_ok = !out_shapes[j].empty();
            for (int d : out_shapes[j])
                shapes_ok = shapes_ok && d > 0;
        }
        if (!shapes_ok) {
            DL_LOGE(TAG, "module %s cannot derive its output shape from its inputs", m->name.c_str());
            return ESP_FAIL;
        }
        for (size_t j = 0; j < m->m_outputs_index.size(); j++) {
            const int idx = m->m_outputs_index[j];
            const std::string name = ctx->get_tensor_name(idx);
            VarInfo &v = vars[idx];
            v.shape = out_shapes[j];
            v.dtype = m_fbs_model->has_value_info(name) ? m_fbs_model->get_value_info_dtype(name) : dtype_of(m->quant_type);
            if (v.dtype == DATA_TYPE_UNDEFINED)
                v.dtype = dtype_of(m->quant_type);
            if (!m_fbs_model->has_value_info(name))
                DL_LOGW(TAG, "tensor %s has no value_info; exponent 0 assumed", name.c_str());
            v.exponent = m_fbs_model->get_value_info_exponent(name);
            v.known = true;
            v.first = i;
            if (m->inplace == MODULE_INPLACE_UNCHANGED_BUFFER && j == 0 && m->m_inputs_index[0] < CONTEXT_PARAMETER_OFFSET)
                v.alias_of = m->m_inputs_index[0];
        }
    }
    for (const std::string &name : m_fbs_model->get_graph_outputs()) {
        const int idx = ctx->get_variable_index(name);
        if (idx < 0 || !vars[idx].known) {
            DL_LOGE(TAG, "graph output %s is not produced", name.c_str());
            return ESP_FAIL;
        }
        vars[idx].last = plan_size; // alive to the end
    }
    for (const std::string &name : m_fbs_model->get_test_outputs_name()) {
        const int idx = ctx->get_variable_index(name);
        if (idx >= 0)
            vars[idx].last = plan_size;
    }
    // 1b. channel slices.  The outputs of a Split along the last axis stay inside its input when every module
    // that reads them takes a channel pitch; an input of a Concat along the last axis is written in its place
    // inside the Concat's output when its producer can write with a pitch and every reader can read with one.
    // The three outputs of [Split -> ... -> Concat of all pieces and more] (the C2f / C3k2 pattern) compose:
    // the Split's input itself then lives inside the Concat's output.  int8 only (pitches count elements).
    if (m_fuse & FUSE_CHANNEL_SLICES) {
        std::set<int> fixed; // tensors a caller may look at: stay dense
        for (const std::string &name : m_fbs_model->get_graph_inputs())
            fixed.insert(ctx->get_variable_index(name));
        for (const std::string &name : m_fbs_model->get_graph_outputs())
            fixed.insert(ctx->get_variable_index(name));
        for (const std::string &name : m_fbs_model->get_test_outputs_name())
            fixed.insert(ctx->get_variable_index(name));
        std::vector<std::vector<std::pair<int, int>>> readers(n_var); // (module, input slot)
        std::vector<bool> aliased(n_var, false);
        for (int i = 0; i < plan_size; i++) {
            dl::module::Module *m = m_execution_plan[i];
            for (size_t sidx = 0; sidx < m->m_inputs_index.size(); sidx++)
                if (m->m_inputs_index[sidx] > 0 && m->m_inputs_index[sidx] < CONTEXT_PARAMETER_OFFSET)
                    readers[m->m_inputs_index[sidx]].push_back({i, (int)sidx});
        }
        for (int v = 1; v < n_var; v++)
            if (vars[v].alias_of >= 0)
                aliased[vars[v].alias_of] = aliased[v] = true;
        auto sliceable = [&](int v) {
            return v > 0 && v < CONTEXT_PARAMETER_OFFSET && vars[v].known && vars[v].dtype == DATA_TYPE_INT8 &&
                vars[v].shape.size() >= 2 && !aliased[v];
        };
        // a RequantizeLinear handles pitches between int8 tensors only
        auto int8_only = [&](dl::module::Module *m) {
            if (typeid(*m) != typeid(dl::module::RequantizeLinear))
                return true;
            for (int idx : m->m_inputs_index)
                if (idx > 0 && idx < CONTEXT_PARAMETER_OFFSET && vars[idx].dtype != DATA_TYPE_INT8)
                    return false;
            for (int idx : m->m_outputs_index)
                if (vars[idx].dtype != DATA_TYPE_INT8)
                    return false;
            return true;
        };
        // every reader but module `except` takes the tensor with a pitch
        auto readers_take_pitch = [&](int v, int except) {
            for (auto &r : readers[v])
                if (r.first != except &&
                    (!m_execution_plan[r.first]->reads_channel_slice(r.second) || !int8_only(m_execution_plan[r.first])))
                    return false;
            return true;
        };
        auto last_axis = [&](int axis, const VarInfo &v) {
            return axis == (int)v.shape.size() - 1 || axis == -1;
        };
        for (int i = 0; i < plan_size; i++) {
            auto *split = dynamic_cast<dl::module::Split *>(m_execution_plan[i]);
            if (!split || split->m_inputs_index.empty())
                continue;
            const int x = split->m_inputs_index[0];
            if (!sliceable(x) || !last_axis(split->get_axis(), vars[x]))
                continue;
            int at = 0;
            for (size_t j = 0; j < split->m_outputs_index.size(); j++) {
                const int o = split->m_outputs_index[j];
                if (sliceable(o) && !fixed.count(o) && readers_take_pitch(o, -1)) {
                    vars[o].slice_of = x;
                    vars[o].slice_at = at;
                }
                at += vars[o].shape.back();
            }
        }
        for (int i = 0; i < plan_size; i++) {
            auto *cat = dynamic_cast<dl::module::Concat *>(m_execution_plan[i]);
            if (!cat || cat->m_outputs_index.empty())
                continue;
            const int c = cat->m_outputs_index[0];
            if (!sliceable(c) || !last_axis(cat->get_axis(), vars[c]))
                continue;
            // a tensor with storage of its own that may move into the Concat's output
            auto movable = [&](int v) {
                if (!sliceable(v) || fixed.count(v) || vars[v].slice_of >= 0 || vars[v].first < 0)
                    return false;
                dl::module::Module *producer = m_execution_plan[vars[v].first];
                int slot = -1;
                for (size_t k = 0; k < producer->m_outputs_index.size(); k++)
                    if (producer->m_outputs_index[k] == v)
                        slot = (int)k;
                if (slot < 0 || !producer->writes_channel_slice(slot) || !int8_only(producer) || !readers_take_pitch(v, i))
                    return false;
                // (a producer that may work in place simply does not when its output is a slice: the placement
                // below looks at slices first; one whose output IS its input's buffer never gets here, see aliased)
                return producer->inplace != MODULE_INPLACE_UNCHANGED_BUFFER;
            };
            const std::vector<int> &in = cat->m_inputs_index;
            int at = 0;
            for (size_t j = 0; j < in.size();) {
                const int v = in[j];
                if (v <= 0 || v >= CONTEXT_PARAMETER_OFFSET)
                    break; // a constant input: it and what follows are copied
                const int count_in_cat = (int)std::count(in.begin(), in.end(), v);
                if (count_in_cat == 1 && movable(v)) {
                    vars[v].slice_of = c;
                    vars[v].slice_at = at;
                    at += vars[v].shape.back();
                    j++;
                    continue;
                }
                // consecutive inputs that are, in order, all the slices of one tensor x: x moves
                const int x = vars[v].slice_of;
                if (x >= 0 && x != c && vars[v].slice_at == 0 && count_in_cat == 1) {
                    size_t k = j;
                    int covered = 0;
                    while (k < in.size() && in[k] > 0 && in[k] < CONTEXT_PARAMETER_OFFSET && vars[in[k]].slice_of == x &&
                           vars[in[k]].slice_at == covered && std::count(in.begin(), in.end(), in[k]) == 1) {
                        covered += vars[in[k]].shape.back();
                        k++;
                    }
                    if (covered == vars[x].shape.back() && movable(x)) {
                        vars[x].slice_of = c;
                        vars[x].slice_at = at;
                        at += covered;
                        j = k;
                        continue;
                    }
                }
                at += vars[v].shape.back();
                j++;
            }
        }
        // resolve chains (a Split output inside a tensor that moved into a Concat output)
        for (int v = 1; v < n_var; v++) {
            int hops = 0;
            while (vars[v].slice_of >= 0 && vars[vars[v].slice_of].slice_of >= 0 && hops++ < 8) {
                const int mid = vars[v].slice_of;
                vars[v].slice_at += vars[mid].slice_at;
                vars[v].slice_of = vars[mid].slice_of;
            }
        }
        // the wider tensor lives from its first writer to its last reader
        for (int v = 1; v < n_var; v++)
            if (vars[v].slice_of >= 0) {
                VarInfo &w = vars[vars[v].slice_of];
                w.last = std::max(w.last, vars[v].last);
                if (vars[v].first >= 0 && w.first >= 0 && vars[v].first < w.first)
                    w.first = vars[v].first; // a Concat output that a producer writes into before the Concat runs
            }
    }
    // a view keeps its source alive
    for (int i = n_var - 1; i >= 1; i--)
        if (vars[i].alias_of >= 0)
            vars[vars[i].alias_of].last = std::max(vars[vars[i].alias_of].last, vars[i].last);
    // 2. placement
    auto bytes_of = [&](const VarInfo &v) {
        size_t n = dtype_sizeof(v.dtype);
        for (int d : v.shape)
            n *= (size_t)d;
        return n;
    };
    std::vector<size_t> offset(n_var, 0);
    std::vector<bool> placed(n_var, false);
    ArenaPlanner arena;
    std::set<int> graph_io;
    for (const std::string &name : m_fbs_model->get_graph_inputs())
        graph_io.insert(ctx->get_variable_index(name));
    for (int idx : graph_io) {
        offset[idx] = arena.alloc(bytes_of(vars[idx]));
        placed[idx] = true;
    }
    auto release_dead = [&](int step) {
        for (int v = 1; v < n_var; v++)
            if (placed[v] && vars[v].alias_of < 0 && vars[v].last == step && !graph_io.count(v)) {
                // views that share the block die no later than their source (made sure above)
                arena.release(offset[v], bytes_of(vars[v]));
                placed[v] = false;
                vars[v].last = -2;
            }
    };
    for (int i = 0; i < plan_size; i++) {
        dl::module::Module *m = m_execution_plan[i];
        for (size_t j = 0; j < m->m_outputs_index.size(); j++) {
            const int idx = m->m_outputs_index[j];
            VarInfo &v = vars[idx];
            if (v.alias_of >= 0) {
                offset[idx] = offset[v.alias_of];
                continue;
            }
            if (placed[idx])
                continue; // the output of a Concat that an earlier producer already writes into
            if (v.slice_of >= 0) {
                // lives inside the wider tensor, which is placed when its first slice is written
                const int w = v.slice_of;
                if (!placed[w]) {
                    offset[w] = arena.alloc(bytes_of(vars[w]));
                    placed[w] = true;
                }
                continue;
            }
            // an in-place module may overwrite its first input when nobody reads that input later
            const int in0 = m->m_inputs_index.empty() ? -1 : m->m_inputs_index[0];
            if (m->inplace == MODULE_INPLACE_CHANGED_BUFFER && j == 0 && in0 > 0 && in0 < CONTEXT_PARAMETER_OFFSET &&
                placed[in0] && vars[in0].alias_of < 0 && vars[in0].last == i && !graph_io.count(in0) &&
                bytes_of(vars[in0]) == bytes_of(v)) {
                bool aliased_elsewhere = false;
                for (int k = 1; k < n_var; k++)
                    if (vars[k].alias_of == in0 || vars[k].slice_of == in0)
                        aliased_elsewhere = true;
                if (!aliased_elsewhere) {
                    offset[idx] = offset[in0];
                    placed[idx] = true;
                    placed[in0] = false;
                    vars[in0].last = -2;
                    continue;
                }
            }
            offset[idx] = arena.alloc(bytes_of(v));
            placed[idx] = true;
        }
        release_dead(i);
    }

    // 3. materialize
    if (!ctx->root_alloc(arena.top()))
        return ESP_FAIL;
    char *root = static_cast<char *>(ctx->get_device_root());
    for (int i = 1; i < n_var; i++) {
        if (!vars[i].known)
            continue;
        if (vars[i].slice_of >= 0) {
            const VarInfo &w = vars[vars[i].slice_of];
            ctx->m_variables[i] = new TensorBase(vars[i].shape, root + offset[vars[i].slice_of] + vars[i].slice_at, vars[i].exponent,
                                                 vars[i].dtype, false, MALLOC_CAP_DEVICE);
            ctx->m_variables[i]->channel_pitch = w.shape.back();
            continue;
        }
        ctx->m_variables[i] =
            new TensorBase(vars[i].shape, root + offset[i], vars[i].exponent, vars[i].dtype, false, MALLOC_CAP_DEVICE);
    }
    m_inputs.clear();
    m_outputs.clear();
    for (const std::string &name : m_fbs_model->get_graph_inputs())
        m_inputs.emplace(name, get_intermediate(name));
    for (const std::string &name : m_fbs_model->get_graph_outputs())
        m_outputs.emplace(name, get_intermediate(name));
    (void)hipMemsetAsync(root, 0, ctx->get_device_size(), static_cast<hipStream_t>(m_stream));
    (void)hipStreamSynchronize(static_cast<hipStream_t>(m_stream));
    m_built = true;
    return ESP_OK;
}

void Model::run_async(runtime_mode_t mode)
{
    begin_pass();
    if (!m_built) {
        m_failed = true;
        return;
    }
    if (m_graph_exec) {
        (void)hip_ok(hipGraphLaunch(static_cast<hipGraphExec_t>(m_graph_exec), static_cast<hipStream_t>(m_stream)),
                     "hipGraphLaunch");
        return;
    }
    for (auto *module : m_execution_plan)
        module->forward(m_model_context, mode);
}

void Model::synchronize()
{
    (void)hip_ok(hipStreamSynchronize(static_cast<hipStream_t>(m_stream)), "hipStreamSynchronize");
}

void Model::run(runtime_mode_t mode)
{
    run_async(mode);
    synchronize();
}

void Model::run(TensorBase *input, runtime_mode_t mode)
{
    if (m_inputs.size() != 1) {
        DL_LOGW(TAG, "The inputs of model is not just one! This API will assign data to first input");
    }
    TensorBase *model_input = m_inputs.begin()->second;
    if (!model_input->assign(input, m_stream)) {
        DL_LOGE(TAG, "Assign input failed");
        return;
    }
    run(mode);
}

void Model::run(std::map<std::string, TensorBase *> &user_inputs, runtime_mode_t mode,
                std::map<std::string, TensorBase *> user_outputs)
{
    if (user_inputs.size() != m_inputs.size()) {
        DL_LOGE(TAG, "The size of user_inputs(%zu) don't equal with the size of model inputs(%zu).", user_inputs.size(),
                m_inputs.size());
        return;
    }
    for (auto &kv : user_inputs) {
        auto it = m_inputs.find(kv.first);
        if (it == m_inputs.end() || !it->second->assign(kv.second, m_stream)) {
            DL_LOGE(TAG, "Assign input %s failed", kv.first.c_str());
            return;
        }
    }
    run(mode);
    for (auto &kv : user_outputs) {
        TensorBase *t = get_intermediate(kv.first);
        if (!t || !kv.second->assign(t, m_stream))
            DL_LOGE(TAG, "Assign output %s failed", kv.first.c_str());
    }
    synchronize();
}

void Model::run(int stage_num, int stage_index, runtime_mode_t mode)
{
    const int plan_size = (int)m_execution_plan.size();
    if (stage_num < 1)
        stage_num = 1;
    if (stage_index < 0 || stage_index >= stage_num) {
        DL_LOGE(TAG, "Invalid stage_index(%d), it should be in range [0, %d).", stage_index, stage_num);
        return;
    }
    begin_pass();
    const int start = stage_index * plan_size / stage_num;
    const int end = (stage_index + 1) * plan_size / stage_num;
    for (int i = start; i < end; i++)
        m_execution_plan[i]->forward(m_model_context, mode);
    synchronize();
}

bool Model::enable_graph()
{
    if (!m_built || m_graph_exec)
        return m_graph_exec != nullptr;
    begin_pass();
    hipStream_t s = static_cast<hipStream_t>(m_stream);
    // one eager pass so that every module has uploaded its shifts / tables before capture starts; modules that
    // carry data between passes (StreamingCache) get it back afterwards, the pass counts for nothing
    for (auto *module : m_execution_plan)
        module->hold_state(m_stream);
    for (auto *module : m_execution_plan)
        module->forward(m_model_context, RUNTIME_MODE_AUTO);
    for (auto *module : m_execution_plan)
        module->restore_state(m_stream);
    if (!hip_ok(hipStreamSynchronize(s), "hipStreamSynchronize") || last_run_failed())
        return false; // a plan with a rejected module must not be captured: the graph would miss its kernels
    if (!hip_ok(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture"))
        return false;
    for (auto *module : m_execution_plan)
        module->forward(m_model_context, RUNTIME_MODE_AUTO);
    hipGraph_t graph = nullptr;
    if (!hip_ok(hipStreamEndCapture(s, &graph), "hipStreamEndCapture") || !graph)
        return false;
    if (last_run_failed()) {
        (void)hipGraphDestroy(graph);
        return false;
    }
    hipGraphExec_t exec = nullptr;
    if (!hip_ok(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "hipGraphInstantiate")) {
        (void)hipGraphDestroy(graph);
        return false;
    }
    m_graph = graph;
    m_graph_exec = exec;
    return true;
}

void Model::disable_graph()
{
    if (m_graph_exec) {
        (void)hipStreamSynchronize(static_cast<hipStream_t>(m_stream));
        (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(m_graph_exec));
        m_graph_exec = nullptr;
    }
    if (m_graph) {
        (void)hipGraphDestroy(static_cast<hipGraph_t>(m_graph));
        m_graph = nullptr;
    }
}

esp_err_t Model::test()
{
    if (!m_built)
        return ESP_FAIL;
    begin_pass();
    for (auto &kv : m_inputs) {
        TensorBase *test_input = m_fbs_model->get_test_input_tensor(kv.first);
        if (!test_input) {
            DL_LOGE(TAG, "Model input %s doesn't have a corresponding test input.", kv.first.c_str());
            return ESP_FAIL;
        }
        const bool ok = kv.second->assign(test_input, m_stream);
        delete test_input;
        if (!ok) {
            DL_LOGE(TAG, "Assign input failed");
            return ESP_FAIL;
        }
    }
    std::vector<std::string> names = m_fbs_model->get_test_outputs_name();
    if (names.empty()) {
        DL_LOGE(TAG, "The model holds no test outputs");
        return ESP_FAIL;
    }
    for (const std::string &name : names)
        if (m_model_context->get_tensor_index(name) < 0) {
            DL_LOGE(TAG, "There's no intermediate result or output named %s in model.", name.c_str());
            return ESP_FAIL;
        }
    // run module by module so that every tested tensor is compared right after it is produced
    for (auto *module : m_execution_plan) {
        module->forward(m_model_context, RUNTIME_MODE_SINGLE_CORE);
        synchronize();
        if (last_run_failed()) {
            DL_LOGE(TAG, "Module %s failed", module->name.c_str());
            return ESP_FAIL;
        }
        for (int index : module->get_outputs_index()) {
            const std::string out_name = m_model_context->get_tensor_name(index);
            if (std::find(names.begin(), names.end(), out_name) == names.end())
                continue;
            TensorBase *output = m_model_context->get_tensor(index);
            TensorBase *output_gt = m_fbs_model->get_test_output_tensor(out_name);
            const float eps = (output->get_dtype() == DATA_TYPE_INT16) ? 1 + 1e-5f : 2e-5f;
            const bool same = output->equal(output_gt, eps, true);
            delete output_gt;
            if (!same) {
                DL_LOGE(TAG, "Test output %s does not match", out_name.c_str());
                return ESP_FAIL;
            }
        }
    }
    DL_LOGI(TAG, "Test Pass!");
    return ESP_OK;
}

std::vector<module_info> Model::get_module_info(int repeats)
{
    // Whole passes of the plan in execution order with one event between consecutive modules: every
    // module is timed with the cache state an ordinary run gives it (its input was just written by the
    // module before, not by an earlier repeat of itself), the per-module times add up to the time of a
    // pass, and the tensors hold an ordinary pass's results afterwards.
    std::vector<module_info> info;
    if (!m_built)
        return info;
    hipStream_t s = static_cast<hipStream_t>(m_stream);
    if (repeats < 1)
        repeats = 1;
    const size_t n = m_execution_plan.size();
    std::vector<hipEvent_t> ev(n + 1, nullptr);
    bool ok = true;
    for (auto &e : ev)
        ok = ok && hip_ok(hipEventCreate(&e), "hipEventCreate");
    std::vector<double> total_ms(n, 0.0);
    double gap_ms = 0.0; // what two events recorded back to back measure: the cost of the bracket itself
    if (ok) {
        for (int r = 0; r < 8; r++) {
            (void)hipEventRecord(ev[0], s);
            (void)hipEventRecord(ev[1], s);
            (void)hipEventSynchronize(ev[1]);
            float ms = 0.f;
            (void)hipEventElapsedTime(&ms, ev[0], ev[1]);
            gap_ms = (r == 0 || ms < gap_ms) ? ms : gap_ms;
        }
        for (auto *module : m_execution_plan)
            module->hold_state(m_stream); // timing passes leave no trace in modules that carry data between passes
        for (int r = -3; r < repeats; r++) { // three passes warm up (caches, clocks) and are not counted
            (void)hipEventRecord(ev[0], s);
            for (size_t i = 0; i < n; i++) {
                m_execution_plan[i]->forward(m_model_context, RUNTIME_MODE_AUTO);
                (void)hipEventRecord(ev[i + 1], s);
            }
            (void)hipEventSynchronize(ev[n]);
            for (size_t i = 0; i < n && r >= 0; i++) {
                float ms = 0.f;
                (void)hipEventElapsedTime(&ms, ev[i], ev[i + 1]);
                total_ms[i] += ms;
            }
        }
        for (auto *module : m_execution_plan)
            module->restore_state(m_stream);
        synchronize();
    }
    for (auto &e : ev)
        if (e)
            (void)hipEventDestroy(e);
    if (!ok)
        return info;
    for (size_t i = 0; i < n; i++) {
        dl::module::Module *module = m_execution_plan[i];
        module_info mi;
        mi.name = module->name;
        mi.type = m_fbs_model->get_operation_type(module->name);
        if (auto *conv = dynamic_cast<dl::module::Conv *>(module)) {
            // a Conv that absorbed its neighbours reports what it runs
            // and, after a colon, which single-launch kernel took it (the espdl_hip_mbconv_s8_supported answer)
            static const char *const kKernel[] = {"", ":fused", ":lds", ":lds", ":wave", ":group"};
            const int k = conv->fused_kernel();
            const char *suffix = k >= 0 && k <= 5 ? kKernel[k] : "";
            if (conv->has_fused_expand())
                mi.type = std::string("Conv>DepthwiseConv>Conv") + suffix;
            else if (conv->has_fused_project())
                mi.type = std::string("DepthwiseConv>Conv") + suffix;
        }
        mi.latency_us = (float)std::max(0.0, (total_ms[i] / repeats - gap_ms) * 1000.0);
        std::vector<std::vector<int>> in_shapes;
        mi.bytes = 0;
        for (int idx : module->m_inputs_index) {
            TensorBase *t = m_model_context->get_tensor(idx);
            in_shapes.push_back(t ? t->shape : std::vector<int>());
            if (t)
                mi.bytes += (int64_t)t->get_bytes();
        }
        for (int idx : module->m_outputs_index) {
            TensorBase *t = m_model_context->get_tensor(idx);
            if (t)
                mi.bytes += (int64_t)t->get_bytes();
        }
        if (mi.type == "Concat" || mi.type == "Split") {
            // pieces that already lie in their place inside the wide tensor (channel slices) are not moved:
            // only the copied pieces count, once read and once written
            const bool concat = mi.type == "Concat";
            const auto &wide_ids = concat ? module->m_outputs_index : module->m_inputs_index;
            const auto &piece_ids = concat ? module->m_inputs_index : module->m_outputs_index;
            TensorBase *wide = wide_ids.empty() ? nullptr : m_model_context->get_tensor(wide_ids[0]);
            if (wide && wide->data) {
                const char *lo = static_cast<const char *>(wide->data);
                const char *hi = lo + wide->get_bytes();
                mi.bytes = 0;
                for (int idx : piece_ids) {
                    TensorBase *t = m_model_context->get_tensor(idx);
                    if (!t || !t->data)
                        continue;
                    const char *p = static_cast<const char *>(t->data);
                    if (!(p >= lo && p < hi))
                        mi.bytes += 2 * (int64_t)t->get_bytes();
                }
            }
        }
        mi.macs = module->get_macs(in_shapes);
        info.push_back(mi);
    }
    return info;
}

void Model::profile(bool sort_module_by_latency)
{
    std::vector<module_info> info = get_module_info();
    if (sort_module_by_latency)
        std::sort(info.begin(), info.end(),
                  [](const module_info &a, const module_info &b) { return a.latency_us > b.latency_us; });
    double total = 0;
    for (auto &m : info)
        total += m.latency_us;
    std::printf("%-40s %-18s %12s %10s %10s\n", "name", "type", "latency(us)", "TOP/s", "GB/s");
    for (auto &m : info)
        std::printf("%-40s %-18s %12.2f %10.2f %10.1f\n", m.name.c_str(), m.type.c_str(), m.latency_us,
                    m.latency_us > 0 ? 2.0 * m.macs / m.latency_us * 1e-6 : 0.0,
                    m.latency_us > 0 ? m.bytes / m.latency_us * 1e-3 : 0.0);
    std::printf("total %.2f us for batch %d\n", total, m_batch);
    mem_info_t mem = get_memory_info();
    std::printf("device memory: %zu bytes (activation arena + parameters)\n", mem.device);
}

mem_info_t Model::get_memory_info()
{
    mem_info_t m;
    m.device = m_model_context->get_variable_memory_size() + m_model_context->get_parameter_memory_size();
    m.host = 0;
    return m;
}

TensorBase *Model::get_input()
{
    if (m_inputs.size() != 1)
        DL_LOGW(TAG, "The inputs of model is not just one! This API will return first input");
    return m_inputs.empty() ? nullptr : m_inputs.begin()->second;
}

TensorBase *Model::get_input(const std::string &name)
{
    auto it = m_inputs.find(name);
    return it == m_inputs.end() ? nullptr : it->second;
}

TensorBase *Model::get_intermediate(const std::string &name)
{
    return m_model_context->get_tensor(name);
}

TensorBase *Model::get_output()
{
    if (m_outputs.size() != 1)
        DL_LOGW(TAG, "The outputs of model is not just one! This API will return first output");
    return m_outputs.empty() ? nullptr : m_outputs.begin()->second;
}

TensorBase *Model::get_output(const std::string &name)
{
    auto it = m_outputs.find(name);
    return it == m_outputs.end() ? nullptr : it->second;
}

std::string Model::get_metadata_prop(const std::string &key)
{
    return m_fbs_model ? m_fbs_model->get_model_metadata_prop(key) : std::string();
}

void Model::print()
{
    std::printf("model %s (version %lld), batch %d, %zu modules\n", m_name.c_str(), (long long)m_version, m_batch,
                m_execution_plan.size());
    for (auto *module : m_execution_plan) {
        std::printf("------------------------------- %s\n", module->name.c_str());
        module->print();
        for (int idx : module->m_inputs_index) {
            TensorBase *t = m_model_context->get_tensor(idx);
            if (t)
                t->print();
        }
        for (int idx : module->m_outputs_index) {
            TensorBase *t = m_model_context->get_tensor(idx);
            if (t)
                t->print();
        }
    }
}

void Model::reset()
{
    for (auto *module : m_execution_plan)
        module->reset();
    if (m_model_context->get_device_root()) {
        synchronize();
        (void)hipMemset(m_model_context->get_device_root(), 0, m_model_context->get_device_size());
    }
}

} // namespace dl
