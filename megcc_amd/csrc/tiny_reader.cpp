// `.tiny` model reader: the FlatBuffers wire format read directly (no generated code, no flatcc
// runtime), field numbers as in runtime/schema/model.fbs (= the ids of the reference's generated
// runtime/src/cheader/model_reader.h:667-1113). What the reference reads with those accessors in
// runtime/src/parse.c:110-355 and runtime/src/vm/op.c:11-65, vm/memforward.c:24-41 is read here.
//
// Wire format in one paragraph: the file starts with a u32 offset to the root table. A table
// starts with an i32 that, subtracted from the table's position, gives its vtable: u16 vtable
// bytes, u16 table bytes, then one u16 per field number = the field's byte offset inside the table
// (0: absent, the schema default applies). Scalars sit in the table; strings, vectors and
// sub-tables are reached through a u32 that is added to its own position. A vector is a u32 count
// followed by the elements, a string a u32 length, the bytes and a NUL. A vector of unions is two
// vectors: the type bytes (field n-1) and the table offsets (field n).
#include "tiny_reader.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <stdexcept>

namespace mg {
namespace tiny {
namespace {

struct Bad : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct File {
    const uint8_t* p;
    size_t n;

    void need(size_t pos, size_t bytes, const char* what) const {
        if (pos > n || bytes > n - pos)
            throw Bad(std::string("truncated or corrupt file: ") + what);
    }
    template <typename T>
    T get(size_t pos, const char* what) const {
        need(pos, sizeof(T), what);
        T v;
        memcpy(&v, p + pos, sizeof(T));
        return v;
    }
};

struct Vec {
    const File* f = nullptr;
    size_t pos = 0;  // first element
    uint32_t count = 0;
    size_t elem = 0;

    template <typename T>
    T at(uint32_t i) const {
        return f->get<T>(pos + (size_t)i * elem, "vector element");
    }
};

struct Table {
    const File* f = nullptr;
    size_t pos = 0, vt = 0;
    uint16_t vt_bytes = 0, tab_bytes = 0;
    bool present = false;

    static Table at(const File* f, size_t pos) {
        Table t;
        t.f = f;
        t.pos = pos;
        const int32_t so = f->get<int32_t>(pos, "table header");
        const int64_t vt = (int64_t)pos - so;
        if (vt < 0 || (size_t)vt > f->n)
            throw Bad("corrupt file: vtable position");
        t.vt = (size_t)vt;
        t.vt_bytes = f->get<uint16_t>(t.vt, "vtable");
        t.tab_bytes = f->get<uint16_t>(t.vt + 2, "vtable");
        if (t.vt_bytes < 4 || (t.vt_bytes & 1))
            throw Bad("corrupt file: vtable size");
        f->need(t.vt, t.vt_bytes, "vtable");
        f->need(pos, t.tab_bytes, "table");
        t.present = true;
        return t;
    }
    // position of field `id` in the file, 0 when absent
    size_t field(int id, size_t bytes) const {
        const size_t slot = 4 + 2 * (size_t)id;
        if (!present || slot + 2 > vt_bytes)
            return 0;
        const uint16_t off = f->get<uint16_t>(vt + slot, "vtable entry");
        if (!off)
            return 0;
        if ((size_t)off + bytes > tab_bytes)
            throw Bad("corrupt file: field outside its table");
        return pos + off;
    }
    template <typename T>
    T scalar(int id, T dflt) const {
        const size_t at = field(id, sizeof(T));
        return at ? f->get<T>(at, "scalar field") : dflt;
    }
    size_t target(int id) const {
        const size_t at = field(id, 4);
        if (!at)
            return 0;
        const uint32_t off = f->get<uint32_t>(at, "offset field");
        if (off > f->n - at)
            throw Bad("corrupt file: offset beyond the file");
        return at + off;
    }
    Table table(int id) const {
        const size_t at = target(id);
        return at ? Table::at(f, at) : Table();
    }
    Vec vec(int id, size_t elem) const {
        Vec v;
        v.f = f;
        v.elem = elem;
        const size_t at = target(id);
        if (!at)
            return v;
        v.count = f->get<uint32_t>(at, "vector length");
        v.pos = at + 4;
        if (elem && v.count > (f->n - v.pos) / elem)
            throw Bad("corrupt file: vector longer than the file");
        return v;
    }
    std::string str(int id) const {
        const size_t at = target(id);
        if (!at)
            return std::string();
        return string_at(f, at);
    }
    static std::string string_at(const File* f, size_t at) {
        const uint32_t len = f->get<uint32_t>(at, "string length");
        f->need(at + 4, len, "string");
        return std::string((const char*)f->p + at + 4, len);
    }
};

Table elem_table(const Vec& v, uint32_t i) {
    const size_t at = v.pos + (size_t)i * 4;
    const uint32_t off = v.f->get<uint32_t>(at, "table vector element");
    if (off > v.f->n - at)
        throw Bad("corrupt file: offset beyond the file");
    return Table::at(v.f, at + off);
}

std::vector<int32_t> ints(const Vec& v) {
    std::vector<int32_t> r(v.count);
    for (uint32_t i = 0; i < v.count; ++i)
        r[i] = v.at<int32_t>(i);
    return r;
}

DType read_dtype(const Table& t) {  // table DType { type; param }
    DType d;
    if (!t.present)
        return d;
    d.type = t.scalar<int8_t>(0, 0);
    const Table p = t.table(1);
    d.has_param = p.present;
    if (p.present) {
        d.scale = p.scalar<float>(0, 1.0f);
        d.zero_point = p.scalar<uint8_t>(1, 0);
    }
    return d;
}

Layout read_layout(const Table& t) {  // table Layout { dims; stride; format }
    Layout l;
    if (!t.present)
        return l;
    l.dims = ints(t.vec(0, 4));
    l.stride = ints(t.vec(1, 4));
    l.format = t.scalar<int8_t>(2, 0);
    return l;
}

Instruction read_instruction(int kind, const Table& t) {
    Instruction in;
    in.kind = kind;
    if (kind == INST_Opr) {
        in.name = t.str(0);
        in.type = t.str(1);
        in.inputs = ints(t.vec(2, 4));
        const Vec ty = t.vec(3, 1);
        for (uint32_t i = 0; i < ty.count; ++i)
            in.input_types.push_back(ty.at<int8_t>(i));
        in.outputs = ints(t.vec(4, 4));
        const Table ws = t.table(5);
        if (ws.present) {
            in.ws_size = ws.scalar<int64_t>(0, 0);
            in.ws_offset = ws.scalar<int64_t>(1, 0);
        }
        in.init_id = t.scalar<int32_t>(6, -1);
        in.kernel_id = t.scalar<int32_t>(7, 0);
        in.workspace_id = t.scalar<int32_t>(8, -1);
        in.deduce_id = t.scalar<int32_t>(9, -1);
    } else if (kind == INST_MemForward) {
        in.fwd_input = t.scalar<int32_t>(0, 0);
        in.fwd_output = t.scalar<int32_t>(1, 0);
        in.fwd_offset = t.scalar<int32_t>(2, 0);
        in.fwd_type = t.scalar<int8_t>(3, 0);
    } else if (kind == INST_DevMemAlloc || kind == INST_DevMemFree) {
        in.mem_tensor = t.scalar<int32_t>(0, 0);
    }
    return in;
}

void read_all(const File& f, ModelInfo* m) {
    const uint32_t root = f.get<uint32_t>(0, "root offset");
    if (root > f.n)
        throw Bad("corrupt file: root offset");
    const Table model = Table::at(&f, root);

    const Vec weights = model.vec(0, 4);
    for (uint32_t i = 0; i < weights.count; ++i) {
        const Table t = elem_table(weights, i);
        WeightInfo w;
        w.dtype = read_dtype(t.table(0));
        w.layout = read_layout(t.table(1));
        w.use_count = t.scalar<int32_t>(2, 0);
        const Vec data = t.vec(3, 1);
        w.data = data.count ? (const int8_t*)f.p + data.pos : nullptr;
        w.data_bytes = data.count;
        w.name = t.str(4);
        w.checksum = t.scalar<uint32_t>(5, 0);
        w.compressed = t.scalar<uint8_t>(6, 0) != 0;
        m->weights.push_back(std::move(w));
    }

    const Vec dms = model.vec(1, 4);
    for (uint32_t i = 0; i < dms.count; ++i) {
        const Table t = elem_table(dms, i);
        DeviceModelInfo d;
        d.device = t.scalar<int8_t>(0, 0);
        const Vec tensors = t.vec(1, 4);
        for (uint32_t k = 0; k < tensors.count; ++k) {
            const Table tt = elem_table(tensors, k);
            TensorInfo ti;
            ti.dtype = read_dtype(tt.table(0));
            ti.layout = read_layout(tt.table(1));
            ti.offset = tt.scalar<int64_t>(2, 0);
            ti.dynamic = tt.scalar<uint8_t>(3, 0) != 0;
            ti.use_count = tt.scalar<int32_t>(4, 0);
            ti.name = tt.str(5);
            d.tensors.push_back(std::move(ti));
        }
        const Vec kinds = t.vec(2, 1), insts = t.vec(3, 4);
        if (kinds.count != insts.count)
            throw Bad("corrupt file: instruction type and value vectors differ in length");
        for (uint32_t k = 0; k < insts.count; ++k) {
            const int kind = kinds.at<uint8_t>(k);
            if (kind == 0) {  // NONE: no table behind it
                Instruction none;
                d.instructions.push_back(none);
                continue;
            }
            d.instructions.push_back(read_instruction(kind, elem_table(insts, k)));
        }
        d.tensor_memory = t.scalar<uint64_t>(4, 0);
        d.inputs = ints(t.vec(5, 4));
        d.outputs = ints(t.vec(6, 4));
        d.weight_outputs = ints(t.vec(7, 4));
        const Vec names = t.vec(8, 4);
        for (uint32_t k = 0; k < names.count; ++k) {
            const size_t at = names.pos + (size_t)k * 4;
            const uint32_t off = f.get<uint32_t>(at, "string vector element");
            if (off > f.n - at)
                throw Bad("corrupt file: offset beyond the file");
            d.weight_output_names.push_back(Table::string_at(&f, at + off));
        }
        m->device_models.push_back(std::move(d));
    }
    m->const_shape = model.scalar<uint8_t>(2, 0) != 0;
    m->name = model.str(3);
    m->model_id = model.scalar<uint64_t>(4, 0);
}

void put(std::string* s, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void put(std::string* s, const char* fmt, ...) {
    va_list ap, ap2;
    va_start(ap, fmt);
    va_copy(ap2, ap);
    const int len = vsnprintf(nullptr, 0, fmt, ap);
    va_end(ap);
    if (len > 0) {
        const size_t at = s->size();
        s->resize(at + (size_t)len + 1);
        vsnprintf(&(*s)[at], (size_t)len + 1, fmt, ap2);
        s->resize(at + (size_t)len);
    }
    va_end(ap2);
}

void put_ints(std::string* s, const char* key, const std::vector<int32_t>& v) {
    put(s, " %s=[", key);
    for (size_t i = 0; i < v.size(); ++i)
        put(s, i ? ",%d" : "%d", v[i]);
    *s += "]";
}

void put_typed(std::string* s, const DType& d, const Layout& l) {
    put(s, " dtype=%d scale=%.9g zero_point=%d", d.type, d.scale, d.zero_point);
    put_ints(s, "dims", l.dims);
    put_ints(s, "stride", l.stride);
    put(s, " format=%d", l.format);
}

}  // namespace

bool read_model(const void* buffer, size_t size, ModelInfo* out, std::string* error) {
    if (!buffer || size < 8) {
        *error = "empty model buffer";
        return false;
    }
    File f{(const uint8_t*)buffer, size};
    try {
        *out = ModelInfo();
        read_all(f, out);
    } catch (const Bad& e) {
        *error = e.what();
        return false;
    }
    return true;
}

std::string describe(const ModelInfo& m) {
    std::string s;
    put(&s, "model name=%s model_id=%llu const_shape=%d weights=%zu device_models=%zu\n",
        m.name.c_str(), (unsigned long long)m.model_id, m.const_shape ? 1 : 0, m.weights.size(),
        m.device_models.size());
    for (size_t i = 0; i < m.weights.size(); ++i) {
        const WeightInfo& w = m.weights[i];
        uint64_t h = 1469598103934665603ull;  // FNV-1a over the stored bytes
        for (size_t k = 0; k < w.data_bytes; ++k)
            h = (h ^ (uint8_t)w.data[k]) * 1099511628211ull;
        put(&s, "weight %zu name=%s", i, w.name.c_str());
        put_typed(&s, w.dtype, w.layout);
        put(&s, " use_count=%d checksum=%u compressed=%d bytes=%zu fnv=%016llx\n", w.use_count,
            w.checksum, w.compressed ? 1 : 0, w.data_bytes, (unsigned long long)h);
    }
    for (size_t i = 0; i < m.device_models.size(); ++i) {
        const DeviceModelInfo& d = m.device_models[i];
        put(&s, "device_model %zu device=%d tensors=%zu instructions=%zu tensor_memory=%llu", i,
            d.device, d.tensors.size(), d.instructions.size(), (unsigned long long)d.tensor_memory);
        put_ints(&s, "inputs", d.inputs);
        put_ints(&s, "outputs", d.outputs);
        put_ints(&s, "weight_outputs", d.weight_outputs);
        s += " weight_output_names=[";
        for (size_t k = 0; k < d.weight_output_names.size(); ++k)
            s += (k ? "," : "") + d.weight_output_names[k];
        s += "]\n";
        for (size_t k = 0; k < d.tensors.size(); ++k) {
            const TensorInfo& t = d.tensors[k];
            put(&s, "tensor %zu name=%s", k, t.name.c_str());
            put_typed(&s, t.dtype, t.layout);
            put(&s, " offset=%lld dynamic=%d use_count=%d\n", (long long)t.offset,
                t.dynamic ? 1 : 0, t.use_count);
        }
        for (size_t k = 0; k < d.instructions.size(); ++k) {
            const Instruction& in = d.instructions[k];
            if (in.kind == INST_Opr) {
                put(&s, "inst %zu Opr name=%s type=%s", k, in.name.c_str(), in.type.c_str());
                put_ints(&s, "inputs", in.inputs);
                put_ints(&s, "input_types",
                         std::vector<int32_t>(in.input_types.begin(), in.input_types.end()));
                put_ints(&s, "outputs", in.outputs);
                put(&s, " ws_size=%lld ws_offset=%lld init_id=%d kernel_id=%d workspace_id=%d deduce_id=%d\n",
                    (long long)in.ws_size, (long long)in.ws_offset, in.init_id, in.kernel_id,
                    in.workspace_id, in.deduce_id);
            } else if (in.kind == INST_MemForward) {
                put(&s, "inst %zu MemForward input=%d output=%d offset=%d type=%d\n", k,
                    in.fwd_input, in.fwd_output, in.fwd_offset, in.fwd_type);
            } else if (in.kind == INST_DevMemAlloc || in.kind == INST_DevMemFree) {
                put(&s, "inst %zu %s tensor=%d\n", k,
                    in.kind == INST_DevMemAlloc ? "DevMemAlloc" : "DevMemFree", in.mem_tensor);
            } else {
                put(&s, "inst %zu kind=%d\n", k, in.kind);
            }
        }
    }
    return s;
}

}  // namespace tiny
}  // namespace mg
