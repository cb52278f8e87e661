// ONNX protobuf wire format -> rmlk_graph, and a text summary of a graph.
//
// The reference reads `.onnx` files with generated quick-protobuf code and feeds its GraphBuilder
// (schema/src/onnx_import/transform.rs:76-260, traverse.rs:33-60). This is a hand-written reader of
// the same messages, by field number (schema/src/onnx/protos/onnx.proto): ModelProto.graph = 7;
// GraphProto node = 1, name = 2, initializer = 5, input = 11, output = 12; NodeProto input = 1,
// output = 2, name = 3, op_type = 4, attribute = 5, domain = 7; AttributeProto name = 1, f = 2,
// i = 3, s = 4, t = 5, g = 6, floats = 7, ints = 8, strings = 9, type = 20; TensorProto dims = 1,
// data_type = 2, float_data = 4, int32_data = 5, int64_data = 7, name = 8, raw_data = 9,
// double_data = 10, uint64_data = 11, external_data = 13, data_location = 14; ValueInfoProto
// name = 1, type = 2; TypeProto.tensor_type = 1 {elem_type = 1, shape = 2}; TensorShapeProto.dim = 1
// {dim_value = 1, dim_param = 2}. The visiting order and rules are the reference's: initializers
// first, then graph inputs (one that shares a name with an initializer is a defaulted input and
// keeps the constant only), outputs, then nodes in stored order; a symbolic or missing dim is
// dynamic (0); tensor payloads come from raw_data, from the typed repeated fields, or from an
// external file (location / offset / length, relative to the model's directory,
// schema/src/tensor.rs:149-233).
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iterator>
#include <sstream>

#include "core.hpp"

namespace rmlk {
namespace rt {
namespace {

[[noreturn]] void parse_fail(const std::string &m) {
    throw RtError(RMLK_ERR_GRAPH, "failed to parse ONNX model: " + m);
}

struct Span {
    const uint8_t *p = nullptr;
    size_t n = 0;
    std::string str() const { return std::string(reinterpret_cast<const char *>(p), n); }
};

// One protobuf message: iterate (field, wire type, value).
struct Reader {
    const uint8_t *p, *end;
    explicit Reader(Span s) : p(s.p), end(s.p + s.n) {}
    bool done() const { return p >= end; }
    uint64_t varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 70; shift += 7) {
            if (p >= end) parse_fail("truncated varint");
            const uint8_t c = *p++;
            v |= static_cast<uint64_t>(c & 0x7f) << shift;
            if (c < 0x80) return v;
        }
        parse_fail("varint longer than 10 bytes");
    }
    struct Field {
        uint32_t number;
        uint32_t wire;
        uint64_t value = 0;  // varint / fixed payload
        Span bytes;          // length-delimited payload
    };
    Field next() {
        Field f;
        const uint64_t key = varint();
        f.number = static_cast<uint32_t>(key >> 3);
        f.wire = static_cast<uint32_t>(key & 7);
        switch (f.wire) {
            case 0: f.value = varint(); break;
            case 1:
                if (end - p < 8) parse_fail("truncated fixed64");
                std::memcpy(&f.value, p, 8);
                p += 8;
                break;
            case 2: {
                const uint64_t len = varint();
                if (len > static_cast<uint64_t>(end - p)) parse_fail("length past the end of the message");
                f.bytes = Span{p, static_cast<size_t>(len)};
                p += len;
                break;
            }
            case 5: {
                if (end - p < 4) parse_fail("truncated fixed32");
                uint32_t v;
                std::memcpy(&v, p, 4);
                f.value = v;
                p += 4;
                break;
            }
            default: parse_fail("unsupported wire type " + std::to_string(f.wire));
        }
        return f;
    }
};

// repeated scalar fields arrive packed (one length-delimited blob) or one element per key
void add_varints(const Reader::Field &f, std::vector<int64_t> &out) {
    if (f.wire == 0) {
        out.push_back(static_cast<int64_t>(f.value));
    } else if (f.wire == 2) {
        Reader r(f.bytes);
        while (!r.done()) out.push_back(static_cast<int64_t>(r.varint()));
    } else {
        parse_fail("repeated integer field with wire type " + std::to_string(f.wire));
    }
}
template <typename T>
void add_fixed(const Reader::Field &f, std::vector<T> &out) {
    const uint32_t want = sizeof(T) == 4 ? 5 : 1;
    if (f.wire == want) {
        T v;
        std::memcpy(&v, &f.value, sizeof(T));
        out.push_back(v);
    } else if (f.wire == 2) {
        if (f.bytes.n % sizeof(T)) parse_fail("packed fixed field of odd length");
        const size_t n = f.bytes.n / sizeof(T);
        const size_t at = out.size();
        out.resize(at + n);
        std::memcpy(out.data() + at, f.bytes.p, f.bytes.n);
    } else {
        parse_fail("repeated fixed field with wire type " + std::to_string(f.wire));
    }
}

struct ParsedTensor {
    std::string name;
    HostTensor t;
};

std::vector<uint8_t> read_external(const std::string &base_dir, const std::string &location,
                                   bool has_offset, uint64_t offset, bool has_length,
                                   uint64_t length) {
    if (has_offset != has_length && !has_offset)
        parse_fail("external tensor with a length but no offset");
    std::string path = base_dir.empty() ? location : base_dir + "/" + location;
    std::ifstream f(path, std::ios::binary);
    if (!f) parse_fail("cannot open external data file `" + path + "`");
    f.seekg(0, std::ios::end);
    const uint64_t size = static_cast<uint64_t>(f.tellg());
    if (!has_offset) offset = 0;
    if (!has_length) length = size >= offset ? size - offset : 0;
    if (offset > size || length > size - offset)
        parse_fail("external data range outside `" + path + "`");
    std::vector<uint8_t> buf(length);
    f.seekg(static_cast<std::streamoff>(offset));
    if (length) f.read(reinterpret_cast<char *>(buf.data()), static_cast<std::streamsize>(length));
    if (!f) parse_fail("short read from `" + path + "`");
    return buf;
}

ParsedTensor parse_tensor(Span s, const std::string &base_dir) {
    ParsedTensor out;
    std::vector<int64_t> dims, i32, i64, u64;
    std::vector<float> f32;
    std::vector<double> f64;
    Span raw;
    bool has_raw = false, external = false;
    std::string location;
    bool has_offset = false, has_length = false;
    uint64_t offset = 0, length = 0;
    int32_t dtype = 0;
    Reader r(s);
    while (!r.done()) {
        Reader::Field f = r.next();
        switch (f.number) {
            case 1: add_varints(f, dims); break;
            case 2: dtype = static_cast<int32_t>(f.value); break;
            case 4: add_fixed<float>(f, f32); break;
            case 5: add_varints(f, i32); break;
            case 6: parse_fail("string tensors are not supported");
            case 7: add_varints(f, i64); break;
            case 8: out.name = f.bytes.str(); break;
            case 9:
                raw = f.bytes;
                has_raw = true;
                break;
            case 10: add_fixed<double>(f, f64); break;
            case 11: add_varints(f, u64); break;
            case 13: {  // StringStringEntryProto
                std::string key, value;
                Reader e(f.bytes);
                while (!e.done()) {
                    Reader::Field kv = e.next();
                    if (kv.number == 1) key = kv.bytes.str();
                    else if (kv.number == 2) value = kv.bytes.str();
                }
                if (key == "location") {
                    location = value;
                } else if (key == "offset") {
                    offset = std::stoull(value);
                    has_offset = true;
                } else if (key == "length") {
                    length = std::stoull(value);
                    has_length = true;
                }  // checksum: not verified (the reference ignores it too)
                break;
            }
            case 14: external = f.value == 1; break;
            default: break;  // segment, doc_string, metadata_props
        }
    }
    const size_t es = dtype_size(dtype);
    if (!es) fail_unsupported(dtype);
    if (dims.size() > RMLK_MAX_RANK) throw RtError(RMLK_ERR_BAD_RANK, "tensor `" + out.name + "`: rank above 8");
    int64_t numel = 1;
    for (int64_t d : dims) {
        if (d < 0) parse_fail("tensor `" + out.name + "` has a negative dim");
        numel *= d;
    }
    out.t.dtype = dtype;
    out.t.shape = dims;
    const size_t bytes = static_cast<size_t>(numel) * es;
    if (external) {
        if (location.empty()) parse_fail("external tensor `" + out.name + "` without a location");
        out.t.data = read_external(base_dir, location, has_offset, offset, has_length, length);
        if (out.t.data.size() != bytes)
            parse_fail("external tensor `" + out.name + "`: " + std::to_string(out.t.data.size()) +
                       " bytes for " + std::to_string(bytes));
        return out;
    }
    if (has_raw) {
        if (raw.n != bytes)
            parse_fail("tensor `" + out.name + "`: raw_data of " + std::to_string(raw.n) +
                       " bytes for " + std::to_string(bytes));
        out.t.data.assign(raw.p, raw.p + raw.n);
        return out;
    }
    // typed fields: narrow integers, bool and float16 bits travel in int32_data; uint32 / uint64
    // in uint64_data
    out.t.data.resize(bytes);
    auto need = [&](size_t have) {
        if (have != static_cast<size_t>(numel))
            parse_fail("tensor `" + out.name + "`: " + std::to_string(have) + " typed values for " +
                       std::to_string(numel) + " elements");
    };
    auto narrow = [&](const std::vector<int64_t> &src) {
        need(src.size());
        for (int64_t k = 0; k < numel; ++k) {
            const int64_t v = src[static_cast<size_t>(k)];
            std::memcpy(out.t.data.data() + static_cast<size_t>(k) * es, &v, es);  // little-endian
        }
    };
    switch (dtype) {
        case RMLK_FLOAT:
            need(f32.size());
            std::memcpy(out.t.data.data(), f32.data(), bytes);
            break;
        case RMLK_DOUBLE:
            need(f64.size());
            std::memcpy(out.t.data.data(), f64.data(), bytes);
            break;
        case RMLK_INT64: narrow(i64); break;
        case RMLK_UINT32:
        case RMLK_UINT64: narrow(u64); break;
        default: narrow(i32); break;  // int32, int16, int8, uint16, uint8, bool, float16
    }
    return out;
}

struct ParsedValueInfo {
    std::string name;
    int32_t dtype = 0;
    std::vector<int64_t> dims;
    bool has_type = false;
};

ParsedValueInfo parse_value_info(Span s) {
    ParsedValueInfo v;
    Reader r(s);
    while (!r.done()) {
        Reader::Field f = r.next();
        if (f.number == 1) {
            v.name = f.bytes.str();
        } else if (f.number == 2) {  // TypeProto
            Reader t(f.bytes);
            while (!t.done()) {
                Reader::Field tf = t.next();
                if (tf.number != 1) {
                    if (tf.number == 4 || tf.number == 5 || tf.number == 8 || tf.number == 9)
                        parse_fail("value `" + v.name + "`: only tensor types are supported");
                    continue;
                }
                v.has_type = true;
                Reader tt(tf.bytes);  // TypeProto.Tensor
                while (!tt.done()) {
                    Reader::Field ef = tt.next();
                    if (ef.number == 1) {
                        v.dtype = static_cast<int32_t>(ef.value);
                    } else if (ef.number == 2) {  // TensorShapeProto
                        Reader sh(ef.bytes);
                        while (!sh.done()) {
                            Reader::Field df = sh.next();
                            if (df.number != 1) continue;
                            int64_t dim = 0;  // dim_param or nothing: dynamic
                            Reader d(df.bytes);
                            while (!d.done()) {
                                Reader::Field x = d.next();
                                if (x.number == 1) dim = static_cast<int64_t>(x.value);
                            }
                            if (dim < 0) parse_fail("value `" + v.name + "` has a negative dim");
                            v.dims.push_back(dim);
                        }
                    }
                }
            }
        }
    }
    return v;
}

void check(int32_t st) {
    if (st != 0) throw RtError(st, rmlk_last_error());
}

void add_attribute(rmlk_graph *g, int32_t node, Span s, const std::string &base_dir) {
    std::string name;
    int64_t type = 0;
    bool has_f = false, has_i = false, has_s = false, has_t = false;
    float fv = 0.f;
    int64_t iv = 0;
    std::string sv;
    Span tv;
    std::vector<float> floats;
    std::vector<int64_t> ints;
    bool has_floats = false, has_ints = false;
    Reader r(s);
    while (!r.done()) {
        Reader::Field f = r.next();
        switch (f.number) {
            case 1: name = f.bytes.str(); break;
            case 2: {
                uint32_t bits = static_cast<uint32_t>(f.value);
                std::memcpy(&fv, &bits, 4);
                has_f = true;
                break;
            }
            case 3:
                iv = static_cast<int64_t>(f.value);
                has_i = true;
                break;
            case 4:
                sv = f.bytes.str();
                has_s = true;
                break;
            case 5:
                tv = f.bytes;
                has_t = true;
                break;
            case 6:
            case 11: parse_fail("attribute `" + name + "`: subgraphs are not supported");
            case 7:
                add_fixed<float>(f, floats);
                has_floats = true;
                break;
            case 8:
                add_varints(f, ints);
                has_ints = true;
                break;
            case 20: type = static_cast<int64_t>(f.value); break;
            default: break;  // strings, tensors, doc_string, ref_attr_name, type protos
        }
    }
    // `type` names the field in use (FLOAT 1, INT 2, STRING 3, TENSOR 4, FLOATS 6, INTS 7); older
    // files leave it out and the populated field decides
    if (type == 0)
        type = has_f ? 1 : has_i ? 2 : has_s ? 3 : has_t ? 4 : has_floats ? 6 : has_ints ? 7 : 0;
    switch (type) {
        case 1: check(rmlk_graph_attr_float(g, node, name.c_str(), fv)); break;
        case 2: check(rmlk_graph_attr_int(g, node, name.c_str(), iv)); break;
        case 3: check(rmlk_graph_attr_string(g, node, name.c_str(), sv.c_str())); break;
        case 4: {
            ParsedTensor t = parse_tensor(tv, base_dir);
            check(rmlk_graph_attr_tensor(g, node, name.c_str(), t.t.dtype, t.t.shape.data(),
                                         static_cast<int32_t>(t.t.shape.size()), t.t.data.data()));
            break;
        }
        case 6:
            check(rmlk_graph_attr_floats(g, node, name.c_str(), floats.data(),
                                         static_cast<int32_t>(floats.size())));
            break;
        case 7:
            check(rmlk_graph_attr_ints(g, node, name.c_str(), ints.data(),
                                       static_cast<int32_t>(ints.size())));
            break;
        default: break;  // attribute kinds no operator of the path reads
    }
}

void add_node(rmlk_graph *g, Span s, const std::string &base_dir) {
    std::vector<std::string> inputs, outputs;
    std::string op, domain;
    std::vector<Span> attrs;
    Reader r(s);
    while (!r.done()) {
        Reader::Field f = r.next();
        switch (f.number) {
            case 1: inputs.push_back(f.bytes.str()); break;
            case 2: outputs.push_back(f.bytes.str()); break;
            case 4: op = f.bytes.str(); break;
            case 5: attrs.push_back(f.bytes); break;
            case 7: domain = f.bytes.str(); break;
            default: break;
        }
    }
    if (!domain.empty() && domain != "ai.onnx")
        throw RtError(RMLK_ERR_OP, "unsupported operator `" + domain + "::" + op + "`");
    if (op.empty()) parse_fail("node without op_type");
    // trailing omitted inputs carry no information
    while (!inputs.empty() && inputs.back().empty()) inputs.pop_back();
    std::vector<const char *> in_c, out_c;
    for (const std::string &x : inputs) in_c.push_back(x.c_str());
    for (const std::string &x : outputs) out_c.push_back(x.c_str());
    const int32_t index = rmlk_graph_op(g, op.c_str(), in_c.data(), static_cast<int32_t>(in_c.size()),
                                        out_c.data(), static_cast<int32_t>(out_c.size()));
    if (index < 0) throw RtError(index, rmlk_last_error());
    for (Span a : attrs) add_attribute(g, index, a, base_dir);
}

void load_model(rmlk_graph *g, Span model, const std::string &base_dir) {
    Span graph;
    bool have_graph = false;
    {
        Reader r(model);
        while (!r.done()) {
            Reader::Field f = r.next();
            if (f.number == 7 && f.wire == 2) {
                graph = f.bytes;
                have_graph = true;
            }
        }
    }
    if (!have_graph) throw RtError(RMLK_ERR_GRAPH, "the model does not have a graph");
    std::vector<Span> nodes, initializers, inputs, outputs;
    Reader r(graph);
    while (!r.done()) {
        Reader::Field f = r.next();
        if (f.wire != 2) continue;
        switch (f.number) {
            case 1: nodes.push_back(f.bytes); break;
            case 5: initializers.push_back(f.bytes); break;
            case 11: inputs.push_back(f.bytes); break;
            case 12: outputs.push_back(f.bytes); break;
            case 15: parse_fail("sparse initializers are not supported");
            default: break;
        }
    }
    for (Span s : initializers) {
        ParsedTensor t = parse_tensor(s, base_dir);
        if (t.name.empty()) parse_fail("unnamed tensors are not supported");
        check(rmlk_graph_constant(g, t.name.c_str(), t.t.dtype, t.t.shape.data(),
                                  static_cast<int32_t>(t.t.shape.size()), t.t.data.data()));
    }
    for (Span s : inputs) {
        ParsedValueInfo v = parse_value_info(s);
        if (v.name.empty()) parse_fail("Unnamed inputs are not supported");
        if (g->by_name.count(v.name)) continue;  // defaulted input: the initializer stays
        if (!v.has_type) parse_fail("input `" + v.name + "` missing type");
        if (!dtype_size(v.dtype)) fail_unsupported(v.dtype);
        if (v.dims.size() > RMLK_MAX_RANK) throw RtError(RMLK_ERR_BAD_RANK, "input `" + v.name + "`: rank above 8");
        check(rmlk_graph_input(g, v.name.c_str(), v.dtype, v.dims.data(),
                               static_cast<int32_t>(v.dims.size())));
    }
    std::vector<std::string> output_names;
    for (Span s : outputs) {
        ParsedValueInfo v = parse_value_info(s);
        if (v.name.empty()) parse_fail("Unnamed outputs are not supported");
        output_names.push_back(v.name);
    }
    for (Span s : nodes) add_node(g, s, base_dir);
    for (const std::string &name : output_names) {
        const int32_t st = rmlk_graph_output(g, name.c_str());
        if (st != 0)
            throw RtError(st, "failed to register graph output `" + name + "`: " + rmlk_last_error());
    }
}

uint64_t fnv1a(const uint8_t *p, size_t n) {
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < n; ++i) {
        h ^= p[i];
        h *= 1099511628211ull;
    }
    return h;
}

void json_string(std::ostringstream &o, const std::string &s) {
    o << '"';
    for (char c : s) {
        if (c == '"' || c == '\\') o << '\\' << c;
        else if (static_cast<unsigned char>(c) < 0x20) o << ' ';
        else o << c;
    }
    o << '"';
}
void json_dims(std::ostringstream &o, const std::vector<int64_t> &d) {
    o << '[';
    for (size_t i = 0; i < d.size(); ++i) o << (i ? "," : "") << d[i];
    o << ']';
}

}  // namespace
}  // namespace rt
}  // namespace rmlk

using namespace rmlk::rt;

extern "C" {

int32_t rmlk_graph_load_onnx(const void *bytes, size_t size, const char *base_dir, rmlk_graph **out) {
    if (!out) return RMLK_ERR_NULL_POINTER;
    *out = nullptr;
    rmlk_graph *g = nullptr;
    int32_t st = rmlk_graph_create(&g);
    if (st != 0) return st;
    try {
        if (!bytes && size) throw RtError(RMLK_ERR_NULL_POINTER, "null model bytes");
        load_model(g, Span{static_cast<const uint8_t *>(bytes), size}, base_dir ? base_dir : "");
        *out = g;
        return 0;
    } catch (const RtError &e) {
        rmlk_graph_destroy(g);
        rmlk_set_last_error(e.what());
        return e.code ? e.code : RMLK_ERR_GRAPH;
    } catch (const std::exception &e) {
        rmlk_graph_destroy(g);
        rmlk_set_last_error((std::string("failed to parse ONNX model: ") + e.what()).c_str());
        return RMLK_ERR_GRAPH;
    }
}

int32_t rmlk_graph_load_onnx_file(const char *path, rmlk_graph **out) {
    if (!path || !out) return RMLK_ERR_NULL_POINTER;
    *out = nullptr;
    std::ifstream f(path, std::ios::binary);
    if (!f) {
        rmlk_set_last_error((std::string("cannot open `") + path + "`").c_str());
        return RMLK_ERR_GRAPH;
    }
    std::vector<char> buf((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    std::string dir(path);
    const size_t slash = dir.find_last_of('/');
    dir = slash == std::string::npos ? std::string() : dir.substr(0, slash);
    return rmlk_graph_load_onnx(buf.data(), buf.size(), dir.c_str(), out);
}

int64_t rmlk_graph_describe(const rmlk_graph *g, char *buf, int64_t size) {
    if (!g) return 0;
    std::ostringstream o;
    o << "{\"inputs\":[";
    for (size_t i = 0; i < g->inputs.size(); ++i) {
        const Value &v = g->values[g->inputs[i]];
        o << (i ? "," : "") << "{\"name\":";
        json_string(o, v.name);
        o << ",\"dtype\":" << v.dtype << ",\"dims\":";
        json_dims(o, v.shape);
        o << '}';
    }
    o << "],\"initializers\":[";
    bool first = true;
    for (const Value &v : g->values) {
        if (!v.is_initializer) continue;
        o << (first ? "" : ",") << "{\"name\":";
        first = false;
        json_string(o, v.name);
        o << ",\"dtype\":" << v.init.dtype << ",\"dims\":";
        json_dims(o, v.init.shape);
        o << ",\"bytes\":" << v.init.data.size() << ",\"fnv1a\":\"" << std::hex
          << fnv1a(v.init.data.data(), v.init.data.size()) << std::dec << "\"}";
    }
    o << "],\"nodes\":[";
    for (size_t n = 0; n < g->nodes.size(); ++n) {
        const Node &node = g->nodes[n];
        o << (n ? "," : "") << "{\"op\":";
        json_string(o, node.op);
        o << ",\"inputs\":[";
        for (size_t i = 0; i < node.inputs.size(); ++i) {
            o << (i ? "," : "");
            json_string(o, node.inputs[i] < 0 ? std::string() : g->values[node.inputs[i]].name);
        }
        o << "],\"outputs\":[";
        for (size_t i = 0; i < node.outputs.size(); ++i) {
            o << (i ? "," : "");
            json_string(o, g->values[node.outputs[i]].name);
        }
        o << "],\"attrs\":{";
        std::vector<std::string> names;
        for (const auto &kv : node.attrs) names.push_back(kv.first);
        std::sort(names.begin(), names.end());
        for (size_t i = 0; i < names.size(); ++i) {
            const Attr &a = node.attrs.at(names[i]);
            o << (i ? "," : "");
            json_string(o, names[i]);
            o << ':';
            switch (a.kind) {
                case Attr::Int: o << a.i; break;
                case Attr::Float: {
                    char tmp[40];
                    snprintf(tmp, sizeof(tmp), "%.9g", static_cast<double>(a.f));
                    o << tmp;
                    break;
                }
                case Attr::Ints: json_dims(o, a.ints); break;
                case Attr::Floats: {
                    o << '[';
                    for (size_t k = 0; k < a.floats.size(); ++k) {
                        char tmp[40];
                        snprintf(tmp, sizeof(tmp), "%.9g", static_cast<double>(a.floats[k]));
                        o << (k ? "," : "") << tmp;
                    }
                    o << ']';
                    break;
                }
                case Attr::String: json_string(o, a.s); break;
                case Attr::TensorK:
                    o << "{\"dtype\":" << a.t.dtype << ",\"dims\":";
                    json_dims(o, a.t.shape);
                    o << ",\"fnv1a\":\"" << std::hex << fnv1a(a.t.data.data(), a.t.data.size())
                      << std::dec << "\"}";
                    break;
            }
        }
        o << "}}";
    }
    o << "],\"outputs\":[";
    for (size_t i = 0; i < g->outputs.size(); ++i) {
        o << (i ? "," : "");
        json_string(o, g->values[g->outputs[i]].name);
    }
    o << "]}";
    const std::string s = o.str();
    if (buf && size > 0) {
        const size_t n = std::min(static_cast<size_t>(size - 1), s.size());
        std::memcpy(buf, s.data(), n);
        buf[n] = 0;
    }
    return static_cast<int64_t>(s.size()) + 1;
}

}  // extern "C"
