// Protobuf wire-format walker for ONNX models (see onnx_wire.hpp).
#include "onnx_wire.hpp"

#include <cstring>
#include <fstream>
#include <iterator>
#include <stdexcept>

namespace onnxwire {
namespace {

enum WireType { WT_VARINT = 0, WT_I64 = 1, WT_LEN = 2, WT_I32 = 5 };

struct Span {
    const uint8_t *p;
    const uint8_t *end;
    bool empty() const { return p >= end; }
};

[[noreturn]] void malformed(const char *what)
{
    throw std::runtime_error(std::string("malformed ONNX protobuf: ") + what);
}

uint64_t read_varint(Span &s)
{
    uint64_t v = 0;
    for (int shift = 0; shift < 64; shift += 7) {
        if (s.p >= s.end) malformed("truncated varint");
        const uint8_t b = *s.p++;
        v |= uint64_t(b & 0x7f) << shift;
        if (!(b & 0x80)) return v;
    }
    malformed("varint longer than 10 bytes");
}

Span read_len(Span &s)
{
    const uint64_t n = read_varint(s);
    if (n > uint64_t(s.end - s.p)) malformed("length-delimited field runs past its parent");
    Span sub{s.p, s.p + n};
    s.p += n;
    return sub;
}

uint32_t read_fixed32(Span &s)
{
    if (s.end - s.p < 4) malformed("truncated fixed32");
    uint32_t v;
    std::memcpy(&v, s.p, 4);
    s.p += 4;
    return v;
}

uint64_t read_fixed64(Span &s)
{
    if (s.end - s.p < 8) malformed("truncated fixed64");
    uint64_t v;
    std::memcpy(&v, s.p, 8);
    s.p += 8;
    return v;
}

void skip_field(Span &s, uint32_t wt)
{
    switch (wt) {
    case WT_VARINT: (void)read_varint(s); break;
    case WT_I64: (void)read_fixed64(s); break;
    case WT_LEN: (void)read_len(s); break;
    case WT_I32: (void)read_fixed32(s); break;
    default: malformed("unsupported wire type (groups are not used by ONNX)");
    }
}

std::string to_string(Span s) { return std::string(reinterpret_cast<const char *>(s.p), size_t(s.end - s.p)); }

float bits_to_float(uint32_t u)
{
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// Calls fn(field, wire_type, span) for every field of a message.
template <typename Fn>
void for_each_field(Span s, Fn &&fn)
{
    while (!s.empty()) {
        const uint64_t key = read_varint(s);
        const uint32_t field = uint32_t(key >> 3), wt = uint32_t(key & 7);
        if (field == 0) malformed("field number 0");
        if (!fn(field, wt, s)) skip_field(s, wt);
    }
}

// repeated int64, packed or not
bool read_int64s(uint32_t wt, Span &s, std::vector<int64_t> &out)
{
    if (wt == WT_VARINT) { out.push_back(int64_t(read_varint(s))); return true; }
    if (wt == WT_LEN) {
        Span sub = read_len(s);
        while (!sub.empty()) out.push_back(int64_t(read_varint(sub)));
        return true;
    }
    return false;
}

// repeated float, packed or not
bool read_floats(uint32_t wt, Span &s, std::vector<float> &out)
{
    if (wt == WT_I32) { out.push_back(bits_to_float(read_fixed32(s))); return true; }
    if (wt == WT_LEN) {
        Span sub = read_len(s);
        if ((sub.end - sub.p) % 4) malformed("packed float field is not a multiple of 4 bytes");
        out.reserve(out.size() + size_t(sub.end - sub.p) / 4);
        while (!sub.empty()) out.push_back(bits_to_float(read_fixed32(sub)));
        return true;
    }
    return false;
}

Tensor parse_tensor(Span s)
{
    Tensor t;
    for_each_field(s, [&](uint32_t f, uint32_t wt, Span &c) {
        switch (f) {
        case 1: return read_int64s(wt, c, t.dims);
        case 2: if (wt != WT_VARINT) return false; t.data_type = int32_t(read_varint(c)); return true;
        case 4: return read_floats(wt, c, t.float_data);
        case 7: return read_int64s(wt, c, t.int64_data);
        case 8: if (wt != WT_LEN) return false; t.name = to_string(read_len(c)); return true;
        case 9: if (wt != WT_LEN) return false; t.raw_data = to_string(read_len(c)); return true;
        default: return false;
        }
    });
    return t;
}

Attribute parse_attribute(Span s)
{
    Attribute a;
    for_each_field(s, [&](uint32_t f, uint32_t wt, Span &c) {
        switch (f) {
        case 1: if (wt != WT_LEN) return false; a.name = to_string(read_len(c)); return true;
        case 2: if (wt != WT_I32) return false; a.f = bits_to_float(read_fixed32(c)); return true;
        case 3: if (wt != WT_VARINT) return false; a.i = int64_t(read_varint(c)); return true;
        case 4: if (wt != WT_LEN) return false; a.s = to_string(read_len(c)); return true;
        case 7: return read_floats(wt, c, a.floats);
        case 8: return read_int64s(wt, c, a.ints);
        case 20: if (wt != WT_VARINT) return false; a.type = int32_t(read_varint(c)); return true;
        default: return false;
        }
    });
    return a;
}

Node parse_node(Span s)
{
    Node n;
    for_each_field(s, [&](uint32_t f, uint32_t wt, Span &c) {
        if (wt != WT_LEN) return false;
        switch (f) {
        case 1: n.input.push_back(to_string(read_len(c))); return true;
        case 2: n.output.push_back(to_string(read_len(c))); return true;
        case 3: n.name = to_string(read_len(c)); return true;
        case 4: n.op_type = to_string(read_len(c)); return true;
        case 5: n.attribute.push_back(parse_attribute(read_len(c))); return true;
        default: return false;
        }
    });
    return n;
}

Dimension parse_dimension(Span s)
{
    Dimension d;
    for_each_field(s, [&](uint32_t f, uint32_t wt, Span &c) {
        if (f == 1 && wt == WT_VARINT) { d.has_value = true; d.value = int64_t(read_varint(c)); return true; }
        if (f == 2 && wt == WT_LEN) { d.param = to_string(read_len(c)); return true; }
        return false;
    });
    return d;
}

void parse_tensor_type(Span s, ValueInfo &v)
{
    for_each_field(s, [&](uint32_t f, uint32_t wt, Span &c) {
        if (f == 1 && wt == WT_VARINT) { v.elem_type = int32_t(read_varint(c)); return true; }
        if (f == 2 && wt == WT_LEN) {
            v.has_shape = true;
            for_each_field(read_len(c), [&](uint32_t f2, uint32_t wt2, Span &c2) {
                if (f2 == 1 && wt2 == WT_LEN) { v.dims.push_back(parse_dimension(read_len(c2))); return true; }
                return false;
            });
            return true;
        }
        return false;
    });
}

ValueInfo parse_value_info(Span s)
{
    ValueInfo v;
    for_each_field(s, [&](uint32_t f, uint32_t wt, Span &c) {
        if (wt != WT_LEN) return false;
        if (f == 1) { v.name = to_string(read_len(c)); return true; }
        if (f == 2) {
            for_each_field(read_len(c), [&](uint32_t f2, uint32_t wt2, Span &c2) {
                if (f2 == 1 && wt2 == WT_LEN) { parse_tensor_type(read_len(c2), v); return true; }
                return false;
            });
            return true;
        }
        return false;
    });
    return v;
}

Graph parse_graph(Span s)
{
    Graph g;
    for_each_field(s, [&](uint32_t f, uint32_t wt, Span &c) {
        if (wt != WT_LEN) return false;
        switch (f) {
        case 1: g.node.push_back(parse_node(read_len(c))); return true;
        case 2: g.name = to_string(read_len(c)); return true;
        case 5: g.initializer.push_back(parse_tensor(read_len(c))); return true;
        case 11: g.input.push_back(parse_value_info(read_len(c))); return true;
        case 12: g.output.push_back(parse_value_info(read_len(c))); return true;
        default: return false;
        }
    });
    return g;
}

} // namespace

std::size_t Tensor::numel() const
{
    std::size_t n = 1;
    for (int64_t d : dims) {
        if (d < 0) throw std::runtime_error("ONNX tensor '" + name + "' has a negative dimension");
        n *= std::size_t(d);
    }
    return n;
}

std::vector<float> Tensor::floats() const
{
    const std::size_t n = numel();
    std::vector<float> out(n);
    if (!raw_data.empty()) {
        if (data_type != DT_FLOAT) throw std::runtime_error("ONNX tensor '" + name + "' is not float32");
        if (raw_data.size() != n * sizeof(float))
            throw std::runtime_error("ONNX tensor '" + name + "': raw_data size does not match dims");
        std::memcpy(out.data(), raw_data.data(), raw_data.size());
    } else if (!float_data.empty()) {
        if (float_data.size() != n)
            throw std::runtime_error("ONNX tensor '" + name + "': float_data size does not match dims");
        out = float_data;
    } else if (n != 0) {
        throw std::runtime_error("ONNX tensor has no weight data");
    }
    return out;
}

const Attribute *Node::find(const std::string &attr_name) const
{
    for (const Attribute &a : attribute)
        if (a.name == attr_name) return &a;
    return nullptr;
}

Model parse_model(const void *data, std::size_t size)
{
    Model m;
    Span s{static_cast<const uint8_t *>(data), static_cast<const uint8_t *>(data) + size};
    for_each_field(s, [&](uint32_t f, uint32_t wt, Span &c) {
        if (f == 1 && wt == WT_VARINT) { m.ir_version = int64_t(read_varint(c)); return true; }
        if (f == 2 && wt == WT_LEN) { m.producer_name = to_string(read_len(c)); return true; }
        if (f == 7 && wt == WT_LEN) { m.graph = parse_graph(read_len(c)); m.has_graph = true; return true; }
        if (f == 8 && wt == WT_LEN) {
            std::pair<std::string, int64_t> op{"", 0};
            for_each_field(read_len(c), [&](uint32_t f2, uint32_t wt2, Span &c2) {
                if (f2 == 1 && wt2 == WT_LEN) { op.first = to_string(read_len(c2)); return true; }
                if (f2 == 2 && wt2 == WT_VARINT) { op.second = int64_t(read_varint(c2)); return true; }
                return false;
            });
            m.opset_import.push_back(op);
            return true;
        }
        return false;
    });
    return m;
}

Model load_model(const std::string &path)
{
    std::ifstream in(path, std::ios::binary);
    if (!in) throw std::runtime_error("Failed to open/parse ONNX file: " + path);
    std::string bytes((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    try {
        Model m = parse_model(bytes.data(), bytes.size());
        if (!m.has_graph) throw std::runtime_error("no graph");
        return m;
    } catch (const std::runtime_error &e) {
        throw std::runtime_error("Failed to open/parse ONNX file: " + path + " (" + e.what() + ")");
    }
}

} // namespace onnxwire
