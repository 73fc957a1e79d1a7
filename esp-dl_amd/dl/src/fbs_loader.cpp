// `.espdl` container + FlatBuffers walker.  See fbs_loader.hpp.
#include "fbs_loader.hpp"

#include <cstdio>
#include <cstring>
#include <set>

namespace fbs {

namespace {

// Bounds-checked view of the FlatBuffers payload.  Any out-of-range access sets `bad` and yields zeros,
// so a truncated or hostile file ends in a failed load instead of a wild read.
struct Buf {
    const uint8_t *d;
    size_t n;
    bool bad = false;

    bool in(size_t p, size_t len)
    {
        if (p > n || len > n - p) {
            bad = true;
            return false;
        }
        return true;
    }
    template <typename T>
    T rd(size_t p)
    {
        T v = T();
        if (in(p, sizeof(T)))
            std::memcpy(&v, d + p, sizeof(T));
        return v;
    }
};

// One table: field number -> absolute position (0 = absent).
struct Table {
    Buf *b = nullptr;
    size_t pos = 0, vt = 0;
    uint16_t vt_size = 0;
    bool ok = false;

    Table() {}
    Table(Buf *buf, size_t p) : b(buf), pos(p)
    {
        const int32_t back = b->rd<int32_t>(p);
        const long long v = (long long)p - back;
        if (b->bad || v < 0 || (size_t)v + 4 > b->n) {
            b->bad = true;
            return;
        }
        vt = (size_t)v;
        vt_size = b->rd<uint16_t>(vt);
        ok = !b->bad;
    }
    size_t field(int idx)
    {
        if (!ok)
            return 0;
        const size_t off = 4 + 2 * (size_t)idx;
        if (off + 2 > vt_size)
            return 0;
        const uint16_t rel = b->rd<uint16_t>(vt + off);
        return rel ? pos + rel : 0;
    }
    size_t indirect(int idx)
    {
        const size_t p = field(idx);
        return p ? p + b->rd<uint32_t>(p) : 0;
    }
    Table table(int idx)
    {
        const size_t p = indirect(idx);
        return p ? Table(b, p) : Table();
    }
    std::string string(int idx)
    {
        const size_t p = indirect(idx);
        if (!p)
            return "";
        const uint32_t len = b->rd<uint32_t>(p);
        if (!b->in(p + 4, len))
            return "";
        return std::string(reinterpret_cast<const char *>(b->d + p + 4), len);
    }
    template <typename T>
    T scalar(int idx, T dflt)
    {
        const size_t p = field(idx);
        return p ? b->rd<T>(p) : dflt;
    }
    // vector: position of element 0 and element count
    size_t vector(int idx, uint32_t *count)
    {
        const size_t p = indirect(idx);
        *count = p ? b->rd<uint32_t>(p) : 0;
        return p ? p + 4 : 0;
    }
    template <typename T>
    std::vector<T> scalars(int idx)
    {
        uint32_t n = 0;
        const size_t p = vector(idx, &n);
        std::vector<T> out;
        if (p && b->in(p, (size_t)n * sizeof(T)))
            for (uint32_t i = 0; i < n; i++)
                out.push_back(b->rd<T>(p + (size_t)i * sizeof(T)));
        return out;
    }
    std::vector<Table> tables(int idx)
    {
        uint32_t n = 0;
        const size_t p = vector(idx, &n);
        std::vector<Table> out;
        if (p && b->in(p, (size_t)n * 4))
            for (uint32_t i = 0; i < n; i++) {
                const size_t e = p + 4 * (size_t)i;
                out.emplace_back(b, e + b->rd<uint32_t>(e));
            }
        return out;
    }
    std::vector<std::string> strings(int idx)
    {
        uint32_t n = 0;
        const size_t p = vector(idx, &n);
        std::vector<std::string> out;
        if (p && b->in(p, (size_t)n * 4))
            for (uint32_t i = 0; i < n; i++) {
                const size_t e = p + 4 * (size_t)i;
                const size_t s = e + b->rd<uint32_t>(e);
                const uint32_t len = b->rd<uint32_t>(s);
                out.push_back(b->in(s + 4, len) ? std::string(reinterpret_cast<const char *>(b->d + s + 4), len) : "");
            }
        return out;
    }
};

// TensorDataType of the schema -> dtype_t; anything outside the enumeration reads as UNDEFINED.
dl::dtype_t to_dtype(int32_t v)
{
    return v >= 0 && v <= (int32_t)dl::DATA_TYPE_UINT64 ? (dl::dtype_t)v : dl::DATA_TYPE_UNDEFINED;
}

struct RawTensor {
    std::string name, doc;
    std::vector<int> dims;
    dl::dtype_t dtype = dl::DATA_TYPE_UNDEFINED;
    std::vector<int> exponents;
    std::vector<uint8_t> bytes;
    bool ok = false;
};

// Tensor (espdl.fbs): 0 dims, 1 data_type, 2 float_data, 3 int32_data, 5 int64_data, 6 name, 7 doc_string,
// 8 raw_data ([AlignedBytes], 16 bytes each), 13 exponents.
RawTensor read_tensor(Table t)
{
    RawTensor r;
    for (int64_t d : t.scalars<int64_t>(0)) {
        if (d < 0 || d > 0x7fffffff)
            return r;
        r.dims.push_back((int)d);
    }
    r.dtype = to_dtype(t.scalar<int32_t>(1, 0));
    r.name = t.string(6);
    r.doc = t.string(7);
    for (int64_t e : t.scalars<int64_t>(13))
        r.exponents.push_back((int)e);
    const size_t esize = dl::dtype_sizeof(r.dtype);
    if (esize == 0)
        return r;
    size_t count = 1;
    for (int d : r.dims) {
        if (d != 0 && count > ((size_t)1 << 40) / (size_t)d)
            return r;
        count *= (size_t)d;
    }
    const size_t need = count * esize;
    uint32_t n = 0;
    size_t p = t.vector(8, &n);
    if (p) {
        if ((size_t)n * 16 < need || !t.b->in(p, need))
            return r;
        r.bytes.assign(t.b->d + p, t.b->d + p + need);
    } else {
        // typed arrays (small tensors written without raw_data)
        const int field = r.dtype == dl::DATA_TYPE_FLOAT ? 2 : r.dtype == dl::DATA_TYPE_INT32 ? 3
            : r.dtype == dl::DATA_TYPE_INT64                                              ? 5
                                                                                          : -1;
        if (field < 0 && need > 0)
            return r;
        if (field >= 0) {
            p = t.vector(field, &n);
            if ((size_t)n * esize < need || (need > 0 && !t.b->in(p, need)))
                return r;
            if (need > 0)
                r.bytes.assign(t.b->d + p, t.b->d + p + need);
        }
    }
    r.ok = !t.b->bad;
    return r;
}

// Output channels per block of the blocked filter layouts, 0 when the tensor is not blocked.
int layout_block(const std::string &doc)
{
    const size_t at = doc.find("==>");
    const std::string l = at == std::string::npos ? doc : doc.substr(at + 3);
    if (l.find("C16") != std::string::npos && (l.find("N/16") != std::string::npos || l.find("N16") != std::string::npos))
        return 16;
    if (l.find("C8") != std::string::npos && (l.find("N/8") != std::string::npos || l.find("N8") != std::string::npos))
        return 8;
    return 0;
}

// [N/B][spatial][C][B] followed by the N % B remaining filters in plain [rest][spatial][C] order
//   ->  [N][spatial][C].
// dims are [spatial..., C, N]; a depthwise filter ([spatial..., C, 1]) is blocked over its C filters of
// one input channel each and ends up as the `c` target's [spatial][C].
// The S3 / P4 files of the reference's Gemm fixtures hold the same weights as their `c` files, which
// fixes the body order; the order of the remainder and of depthwise filters is fixed by the shipped
// MobileNetV2 (N = 24 and depthwise layers): only this reading reproduces the top-5 classes that
// examples/mobilenetv2_cls/README.md lists for its cat.jpg.
bool unblock_filter(RawTensor &t, int block, bool depthwise)
{
    if (t.dims.size() < 2)
        return false;
    const size_t esize = dl::dtype_sizeof(t.dtype);
    const size_t last = (size_t)t.dims.back(), prev = (size_t)t.dims[t.dims.size() - 2];
    const size_t n = depthwise ? last * prev : last, c = depthwise ? 1 : prev;
    size_t sp = 1;
    for (size_t i = 0; i + 2 < t.dims.size(); i++)
        sp *= (size_t)t.dims[i];
    if (t.bytes.size() != n * sp * c * esize)
        return false;
    const size_t nb = n / (size_t)block;
    std::vector<uint8_t> nmajor(t.bytes.size());
    const uint8_t *src = t.bytes.data();
    for (size_t b = 0; b < nb; b++)
        for (size_t s = 0; s < sp; s++)
            for (size_t k = 0; k < c; k++)
                for (size_t j = 0; j < (size_t)block; j++) {
                    const size_t from = (((b * sp + s) * c + k) * block + j) * esize;
                    const size_t to = (((b * block + j) * sp + s) * c + k) * esize;
                    std::memcpy(&nmajor[to], src + from, esize);
                }
    const size_t done = nb * block * sp * c * esize;
    std::memcpy(nmajor.data() + done, src + done, t.bytes.size() - done); // remainder: already filter-major
    if (depthwise) {
        // [C][spatial] -> [spatial][C]
        std::vector<uint8_t> hwc(t.bytes.size());
        for (size_t ch = 0; ch < n; ch++)
            for (size_t s = 0; s < sp; s++)
                std::memcpy(&hwc[(s * n + ch) * esize], &nmajor[(ch * sp + s) * esize], esize);
        t.bytes.swap(hwc);
    } else {
        t.bytes.swap(nmajor);
    }
    return true;
}

// ValueInfo -> shape and element type through TypeInfo (union: field 0 type tag, field 1 value) ->
// TensorTypeAndShape (0 elem_type, 1 shape) -> TensorShape (0 dim) -> Dimension (0 value) ->
// DimensionValue (0 dim_type, 1 dim_value).
void read_value_info(Table v, std::string *name, std::vector<int> *dims, dl::dtype_t *dtype, int *exponent)
{
    *name = v.string(0);
    *dtype = dl::DATA_TYPE_UNDEFINED;
    *exponent = 0;
    std::vector<int64_t> exps = v.scalars<int64_t>(3);
    if (!exps.empty())
        *exponent = (int)exps[0];
    Table type = v.table(1);
    if (!type.ok || type.scalar<uint8_t>(0, 0) != 1) // 1 = tensor_type
        return;
    Table tts = type.table(1);
    if (!tts.ok)
        return;
    *dtype = to_dtype(tts.scalar<int32_t>(0, 0));
    Table shape = tts.table(1);
    if (!shape.ok)
        return;
    for (Table dim : shape.tables(0)) {
        Table dv = dim.table(0);
        const int64_t value = dv.ok ? dv.scalar<int64_t>(1, 0) : 0;
        dims->push_back(value > 0 && value <= 0x7fffffff ? (int)value : 1);
    }
}

} // namespace

FbsLoader::FbsLoader(const char *name, model_location_type_t location) : m_location(location)
{
    if (!name) {
        m_error = "null model name";
        return;
    }
    if (location != MODEL_LOCATION_IN_SDCARD) {
        m_error = "memory locations need the (data, size) constructor";
        return;
    }
    FILE *f = std::fopen(name, "rb");
    if (!f) {
        m_error = std::string("cannot open ") + name;
        return;
    }
    std::fseek(f, 0, SEEK_END);
    const long size = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    if (size > 0) {
        m_bytes.resize((size_t)size);
        if (std::fread(m_bytes.data(), 1, (size_t)size, f) != (size_t)size) {
            m_bytes.clear();
            m_error = std::string("short read of ") + name;
        }
    }
    std::fclose(f);
}

FbsLoader::FbsLoader(const void *data, size_t size) : m_location(MODEL_LOCATION_IN_FLASH_RODATA)
{
    if (data && size)
        m_bytes.assign(static_cast<const uint8_t *>(data), static_cast<const uint8_t *>(data) + size);
    else
        m_error = "empty buffer";
}

const char *FbsLoader::get_model_location_string()
{
    switch (m_location) {
    case MODEL_LOCATION_IN_FLASH_RODATA:
        return "memory";
    case MODEL_LOCATION_IN_FLASH_PARTITION:
        return "partition";
    default:
        return "file";
    }
}

bool FbsLoader::index()
{
    if (m_indexed)
        return !m_entries.empty();
    m_indexed = true;
    if (m_bytes.size() < 16) {
        if (m_error.empty())
            m_error = "container shorter than its header";
        return false;
    }
    const char *magic = reinterpret_cast<const char *>(m_bytes.data());
    auto u32 = [&](size_t p) {
        uint32_t v = 0;
        if (p + 4 <= m_bytes.size())
            std::memcpy(&v, m_bytes.data() + p, 4);
        return v;
    };
    if (!std::memcmp(magic, "EDL1", 4) || !std::memcmp(magic, "EDL2", 4)) {
        m_entries.push_back({"", 0, magic[3] == '1' ? 12 : 16});
        return true;
    }
    if (!std::memcmp(magic, "PDL1", 4) || !std::memcmp(magic, "PDL2", 4)) {
        const uint32_t num = u32(4);
        if (num > 4096 || 8 + (size_t)num * 12 > m_bytes.size()) {
            m_error = "bad package header";
            return false;
        }
        for (uint32_t i = 0; i < num; i++) {
            const size_t data_off = u32(8 + 12 * (size_t)i), name_off = u32(12 + 12 * (size_t)i),
                         name_len = u32(16 + 12 * (size_t)i);
            if (name_off > m_bytes.size() || name_len > m_bytes.size() - name_off || data_off + 16 > m_bytes.size()) {
                m_error = "package entry out of range";
                m_entries.clear();
                return false;
            }
            m_entries.push_back({std::string(magic + name_off, name_len), data_off, magic[3] == '1' ? 12 : 16});
        }
        return !m_entries.empty();
    }
    m_error = "unknown container magic (EDL1, EDL2, PDL1 and PDL2 are read)";
    return false;
}

int FbsLoader::get_model_num()
{
    return index() ? (int)m_entries.size() : 0;
}

void FbsLoader::list_models()
{
    if (!index())
        return;
    for (size_t i = 0; i < m_entries.size(); i++)
        std::printf("model %d: %s\n", (int)i, m_entries[i].name.c_str());
}

FbsModel *FbsLoader::load(const uint8_t *key, bool param_copy)
{
    return load(0, key, param_copy);
}

FbsModel *FbsLoader::load(int model_index, const uint8_t *key, bool param_copy)
{
    (void)param_copy; // parameters are always copied: they move to device memory anyway
    if (!index())
        return nullptr;
    if (model_index < 0 || model_index >= (int)m_entries.size()) {
        m_error = "model index out of range";
        return nullptr;
    }
    return parse(m_entries[(size_t)model_index], key);
}

FbsModel *FbsLoader::load(const char *model_name, const uint8_t *key, bool param_copy)
{
    (void)param_copy;
    if (!index())
        return nullptr;
    for (const Entry &e : m_entries)
        if (model_name && e.name == model_name)
            return parse(e, key);
    m_error = std::string("no model named ") + (model_name ? model_name : "(null)");
    return nullptr;
}

FbsModel *FbsLoader::parse(const Entry &e, const uint8_t *key)
{
    (void)key;
    uint32_t mode = 0, size = 0;
    std::memcpy(&mode, m_bytes.data() + e.offset + 4, 4);
    std::memcpy(&size, m_bytes.data() + e.offset + 8, 4);
    if (mode != 0) {
        m_error = "encrypted model (mode 1): decryption is not part of this build";
        return nullptr;
    }
    const size_t start = e.offset + (size_t)e.header;
    if (start > m_bytes.size() || size > m_bytes.size() - start || size < 8) {
        m_error = "payload size exceeds the container";
        return nullptr;
    }
    Buf buf{m_bytes.data() + start, size};
    Table model(&buf, buf.rd<uint32_t>(0));
    Table graph = model.table(7);
    if (!model.ok || !graph.ok) {
        m_error = "no graph in the model";
        return nullptr;
    }
    FbsModel *out = new FbsModel();
    out->set_model_info(graph.string(1).empty() ? e.name : graph.string(1), model.scalar<int64_t>(5, 0), model.string(6));
    for (Table kv : model.tables(8))
        out->set_metadata_prop(kv.string(0), kv.string(1));

    auto fail = [&](const std::string &why) -> FbsModel * {
        m_error = why;
        delete out;
        return nullptr;
    };

    // filters of grouped (depthwise) convolutions are blocked over their channels: find them first
    std::set<std::string> depthwise_filters;
    for (Table n : graph.tables(0)) {
        if (n.string(3) != "Conv")
            continue;
        int64_t group = 1;
        for (Table a : n.tables(5))
            if (a.string(0) == "group" && a.scalar<int32_t>(3, 0) == 2) {
                const size_t p = a.field(5);
                group = p ? buf.rd<int64_t>(p) : 1;
            }
        const std::vector<std::string> ins = n.strings(0);
        if (group != 1 && ins.size() > 1)
            depthwise_filters.insert(ins[1]);
    }
    for (Table t : graph.tables(2)) {
        RawTensor r = read_tensor(t);
        if (!r.ok)
            return fail("initializer " + r.name + ": unreadable tensor");
        const int block = layout_block(r.doc);
        if (block && !unblock_filter(r, block, depthwise_filters.count(r.name) != 0))
            return fail("initializer " + r.name + ": blocked layout does not fit its dims");
        out->add_initializer(r.name, r.dims, r.dtype, r.bytes.data(), r.exponents);
    }
    for (int field : {4, 5, 6}) { // graph inputs, outputs, value_info
        for (Table v : graph.tables(field)) {
            std::string name;
            std::vector<int> dims;
            dl::dtype_t dtype;
            int exponent;
            read_value_info(v, &name, &dims, &dtype, &exponent);
            out->add_value_info(name, dims, dtype, exponent);
            if (field == 4)
                out->add_graph_input(name);
            else if (field == 5)
                out->add_graph_output(name);
        }
    }
    for (Table n : graph.tables(0)) {
        Node *node = out->add_node(n.string(2), n.string(3), n.strings(0), n.strings(1));
        if (!node)
            return fail("duplicate or unnamed node " + n.string(2));
        // Attribute: 0 name, 3 attr_type, 4 f (struct), 5 i (struct), 6 s ([uint8]), 10 floats, 11 ints
        for (Table a : n.tables(5)) {
            Attribute attr;
            const std::string name = a.string(0);
            switch (a.scalar<int32_t>(3, 0)) {
            case 1: {
                const size_t p = a.field(4);
                attr.kind = Attribute::FLOAT;
                attr.f = p ? buf.rd<float>(p) : 0.f;
                break;
            }
            case 2: {
                const size_t p = a.field(5);
                attr.kind = Attribute::INT;
                attr.i = p ? buf.rd<int64_t>(p) : 0;
                break;
            }
            case 3: {
                std::vector<uint8_t> s = a.scalars<uint8_t>(6);
                attr.kind = Attribute::STRING;
                attr.s.assign(s.begin(), s.end());
                break;
            }
            case 6:
                attr.kind = Attribute::FLOATS;
                attr.floats = a.scalars<float>(10);
                break;
            case 7:
                attr.kind = Attribute::INTS;
                attr.ints = a.scalars<int64_t>(11);
                break;
            default:
                continue; // tensors, graphs: not used by the operators of this build
            }
            node->attributes[name] = attr;
        }
    }
    for (int field : {8, 9}) { // test_inputs_value, test_outputs_value
        for (Table t : graph.tables(field)) {
            RawTensor r = read_tensor(t);
            if (!r.ok)
                return fail("test tensor " + r.name + ": unreadable");
            const int exponent = r.exponents.empty() ? 0 : r.exponents[0];
            if (field == 8)
                out->add_test_input(r.name, r.dims, r.dtype, r.bytes.data(), exponent);
            else
                out->add_test_output(r.name, r.dims, r.dtype, r.bytes.data(), exponent);
        }
    }
    if (buf.bad)
        return fail("offset outside the payload: truncated or corrupt file");
    return out;
}

} // namespace fbs
