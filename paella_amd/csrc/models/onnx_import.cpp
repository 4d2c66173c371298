// ONNX model import: reads a .onnx file (protobuf wire format, decoded here -- no protobuf or onnx library) and
// turns its inference graph into the executor's static graph, batch 1, fp32.
//
// This stands where the reference compiles ONNX zoo files with TVM (reference
// sosp23_artifact/setup/onnx2tvm_all.sh:15-23): the same files can be served, with their trained weights, by the
// operators in paella_ops.h.  What the importer does with the graph, in ONNX node order:
//   * Conv / Gemm / MatMul become conv / dense stages; a following BatchNormalization is folded into the weights,
//     a following Add of a constant becomes the bias, a following Add of another activation becomes the conv's
//     residual input, a following Relu / Clip / PRelu its activation -- each only when the intermediate tensor has no
//     other reader, otherwise the operator is kept as a stage of its own;
//   * Concat along channels costs nothing: the buffers of its inputs are re-based into slices of one buffer;
//   * Flatten / Reshape / Squeeze / Unsqueeze / Dropout / Identity are views.
// Anything else (an operator or attribute combination the kernels do not cover) is refused with a message naming
// the node; nothing is approximated.

#include "graph.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <limits>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace paella {

namespace {

[[noreturn]] void fail(const std::string& what) { throw std::runtime_error("onnx import: " + what); }

// ------------------------------------------------------------------------------------------ wire format

struct Reader {
    const uint8_t* p;
    const uint8_t* end;

    bool done() const { return p >= end; }

    uint64_t varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 64; shift += 7) {
            if (p >= end) fail("truncated file");
            const uint8_t b = *p++;
            v |= (uint64_t)(b & 0x7f) << shift;
            if (!(b & 0x80)) return v;
        }
        fail("malformed varint");
    }

    // Returns the field number and stores the wire type.
    uint32_t tag(int* wire) {
        const uint64_t t = varint();
        *wire = (int)(t & 7);
        return (uint32_t)(t >> 3);
    }

    Reader sub() {
        const uint64_t n = varint();
        if (n > (uint64_t)(end - p)) fail("truncated file");
        Reader r{p, p + n};
        p += n;
        return r;
    }

    std::string str() {
        Reader r = sub();
        return std::string(reinterpret_cast<const char*>(r.p), (size_t)(r.end - r.p));
    }

    uint32_t fixed32() {
        if (end - p < 4) fail("truncated file");
        uint32_t v;
        std::memcpy(&v, p, 4);
        p += 4;
        return v;
    }

    uint64_t fixed64() {
        if (end - p < 8) fail("truncated file");
        uint64_t v;
        std::memcpy(&v, p, 8);
        p += 8;
        return v;
    }

    void skip(int wire) {
        switch (wire) {
            case 0: varint(); break;
            case 1: fixed64(); break;
            case 2: sub(); break;
            case 5: fixed32(); break;
            default: fail("unsupported protobuf wire type");
        }
    }

    // repeated int64, packed or not
    void ints(int wire, std::vector<int64_t>* out) {
        if (wire == 2) {
            Reader r = sub();
            while (!r.done()) out->push_back((int64_t)r.varint());
        } else {
            out->push_back((int64_t)varint());
        }
    }

    // repeated float, packed or not
    void floats(int wire, std::vector<float>* out) {
        auto one = [](uint32_t bits) {
            float f;
            std::memcpy(&f, &bits, 4);
            return f;
        };
        if (wire == 2) {
            Reader r = sub();
            while (!r.done()) out->push_back(one(r.fixed32()));
        } else {
            out->push_back(one(fixed32()));
        }
    }
};

// ------------------------------------------------------------------------------------------ ONNX messages (the subset read)

enum DataType { kFloat = 1, kInt32 = 6, kInt64 = 7, kFloat16 = 10, kDouble = 11 };

struct Tensor {
    std::string name;
    std::vector<int64_t> dims;
    int dtype = 0;
    std::vector<float> f;     // float, float16 and double tensors, widened/narrowed to float
    std::vector<int64_t> i;   // int32 and int64 tensors
    size_t numel() const {
        size_t n = 1;
        for (int64_t d : dims) n *= (size_t)d;
        return n;
    }
};

float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h >> 15) << 31, exp = (h >> 10) & 0x1f, man = h & 0x3ff;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: renormalise
            int e = -1;
            uint32_t m = man;
            do {
                ++e;
                m <<= 1;
            } while (!(m & 0x400));
            bits = sign | (uint32_t)(127 - 15 - e) << 23 | (m & 0x3ff) << 13;
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | man << 13;
    } else {
        bits = sign | (exp + 127 - 15) << 23 | man << 13;
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

Tensor parse_tensor(Reader r) {
    Tensor t;
    std::vector<float> float_data;
    std::vector<int64_t> int_data;
    std::vector<double> double_data;
    const uint8_t* raw = nullptr;
    size_t raw_len = 0;
    while (!r.done()) {
        int wire;
        switch (r.tag(&wire)) {
            case 1: r.ints(wire, &t.dims); break;
            case 2: t.dtype = (int)r.varint(); break;
            case 4: r.floats(wire, &float_data); break;
            case 5: r.ints(wire, &int_data); break;   // int32_data (also carries float16 bit patterns)
            case 7: r.ints(wire, &int_data); break;   // int64_data
            case 8: t.name = r.str(); break;
            case 9: {
                Reader b = r.sub();
                raw = b.p;
                raw_len = (size_t)(b.end - b.p);
                break;
            }
            case 10:
                if (wire == 2) {
                    Reader d = r.sub();
                    while (!d.done()) {
                        const uint64_t bits = d.fixed64();
                        double v;
                        std::memcpy(&v, &bits, 8);
                        double_data.push_back(v);
                    }
                } else {
                    const uint64_t bits = r.fixed64();
                    double v;
                    std::memcpy(&v, &bits, 8);
                    double_data.push_back(v);
                }
                break;
            case 14:
                if (r.varint() != 0) fail("tensor '" + t.name + "' keeps its data in an external file; only self-contained files are read");
                break;
            default: r.skip(wire);
        }
    }
    for (int64_t d : t.dims)
        if (d < 0 || d > (int64_t)1 << 32) fail("tensor '" + t.name + "' has an impossible dimension");
    const size_t n = t.numel();
    auto need = [&](size_t have, size_t elem) {
        if (have != n * elem) fail("tensor '" + t.name + "' holds " + std::to_string(have / elem) + " values for " + std::to_string(n) + " elements");
    };
    switch (t.dtype) {
        case kFloat:
            if (raw) {
                need(raw_len, 4);
                t.f.resize(n);
                std::memcpy(t.f.data(), raw, raw_len);
            } else {
                need(float_data.size(), 1);
                t.f = std::move(float_data);
            }
            break;
        case kDouble:
            if (raw) {
                need(raw_len, 8);
                t.f.resize(n);
                for (size_t k = 0; k < n; ++k) {
                    double v;
                    std::memcpy(&v, raw + 8 * k, 8);
                    t.f[k] = (float)v;
                }
            } else {
                need(double_data.size(), 1);
                t.f.resize(n);
                for (size_t k = 0; k < n; ++k) t.f[k] = (float)double_data[k];
            }
            break;
        case kFloat16:
            if (raw) {
                need(raw_len, 2);
                t.f.resize(n);
                for (size_t k = 0; k < n; ++k) {
                    uint16_t h;
                    std::memcpy(&h, raw + 2 * k, 2);
                    t.f[k] = half_to_float(h);
                }
            } else {
                need(int_data.size(), 1);
                t.f.resize(n);
                for (size_t k = 0; k < n; ++k) t.f[k] = half_to_float((uint16_t)int_data[k]);
            }
            break;
        case kInt64:
            if (raw) {
                need(raw_len, 8);
                t.i.resize(n);
                std::memcpy(t.i.data(), raw, raw_len);
            } else {
                need(int_data.size(), 1);
                t.i = std::move(int_data);
            }
            break;
        case kInt32:
            if (raw) {
                need(raw_len, 4);
                t.i.resize(n);
                for (size_t k = 0; k < n; ++k) {
                    int32_t v;
                    std::memcpy(&v, raw + 4 * k, 4);
                    t.i[k] = v;
                }
            } else {
                need(int_data.size(), 1);
                t.i = std::move(int_data);
            }
            break;
        default: break;  // other element types are only an error if a node needs the values
    }
    return t;
}

struct Attr {
    float f = 0;
    int64_t i = 0;
    std::string s;
    std::vector<int64_t> ints;
    std::vector<float> floats;
    std::shared_ptr<Tensor> t;
};

struct ONode {
    std::string op, name;
    std::vector<std::string> in, out;
    std::map<std::string, Attr> attr;

    std::string label() const { return op + " '" + (name.empty() ? (out.empty() ? std::string("?") : out[0]) : name) + "'"; }
    int64_t geti(const char* k, int64_t dflt) const {
        auto it = attr.find(k);
        return it == attr.end() ? dflt : it->second.i;
    }
    float getf(const char* k, float dflt) const {
        auto it = attr.find(k);
        return it == attr.end() ? dflt : it->second.f;
    }
    std::string gets(const char* k, const char* dflt) const {
        auto it = attr.find(k);
        return it == attr.end() ? std::string(dflt) : it->second.s;
    }
    std::vector<int64_t> getints(const char* k) const {
        auto it = attr.find(k);
        return it == attr.end() ? std::vector<int64_t>() : it->second.ints;
    }
};

ONode parse_node(Reader r) {
    ONode n;
    while (!r.done()) {
        int wire;
        switch (r.tag(&wire)) {
            case 1: n.in.push_back(r.str()); break;
            case 2: n.out.push_back(r.str()); break;
            case 3: n.name = r.str(); break;
            case 4: n.op = r.str(); break;
            case 5: {
                Reader a = r.sub();
                std::string key;
                Attr v;
                while (!a.done()) {
                    int w;
                    switch (a.tag(&w)) {
                        case 1: key = a.str(); break;
                        case 2: {
                            const uint32_t bits = a.fixed32();
                            std::memcpy(&v.f, &bits, 4);
                            break;
                        }
                        case 3: v.i = (int64_t)a.varint(); break;
                        case 4: v.s = a.str(); break;
                        case 5: v.t = std::make_shared<Tensor>(parse_tensor(a.sub())); break;
                        case 7: a.floats(w, &v.floats); break;
                        case 8: a.ints(w, &v.ints); break;
                        default: a.skip(w);
                    }
                }
                n.attr[key] = std::move(v);
                break;
            }
            default: r.skip(wire);
        }
    }
    return n;
}

struct ValueInfo {
    std::string name;
    std::vector<int64_t> dims;  // 0 where symbolic
};

ValueInfo parse_value_info(Reader r) {
    ValueInfo v;
    while (!r.done()) {
        int wire;
        const uint32_t f = r.tag(&wire);
        if (f == 1) {
            v.name = r.str();
        } else if (f == 2) {
            Reader type = r.sub();
            while (!type.done()) {
                int w;
                if (type.tag(&w) != 1) { type.skip(w); continue; }
                Reader tensor = type.sub();
                while (!tensor.done()) {
                    int w2;
                    if (tensor.tag(&w2) != 2) { tensor.skip(w2); continue; }
                    Reader shape = tensor.sub();
                    while (!shape.done()) {
                        int w3;
                        if (shape.tag(&w3) != 1) { shape.skip(w3); continue; }
                        Reader dim = shape.sub();
                        int64_t value = 0;
                        while (!dim.done()) {
                            int w4;
                            if (dim.tag(&w4) == 1) value = (int64_t)dim.varint();
                            else dim.skip(w4);
                        }
                        v.dims.push_back(value);
                    }
                }
            }
        } else {
            r.skip(wire);
        }
    }
    return v;
}

struct OModel {
    std::vector<ONode> nodes;
    std::map<std::string, Tensor> init;
    std::vector<ValueInfo> inputs;
    std::vector<std::string> outputs;
    int64_t opset = 0;
};

OModel parse_model(const std::vector<uint8_t>& bytes) {
    OModel m;
    Reader r{bytes.data(), bytes.data() + bytes.size()};
    bool have_graph = false;
    while (!r.done()) {
        int wire;
        const uint32_t f = r.tag(&wire);
        if (f == 7 && wire == 2) {
            have_graph = true;
            Reader g = r.sub();
            while (!g.done()) {
                int w;
                switch (g.tag(&w)) {
                    case 1: m.nodes.push_back(parse_node(g.sub())); break;
                    case 5: {
                        Tensor t = parse_tensor(g.sub());
                        std::string name = t.name;
                        m.init[name] = std::move(t);
                        break;
                    }
                    case 11: m.inputs.push_back(parse_value_info(g.sub())); break;
                    case 12: m.outputs.push_back(parse_value_info(g.sub()).name); break;
                    default: g.skip(w);
                }
            }
        } else if (f == 8 && wire == 2) {
            Reader o = r.sub();
            std::string domain;
            int64_t version = 0;
            while (!o.done()) {
                int w;
                switch (o.tag(&w)) {
                    case 1: domain = o.str(); break;
                    case 2: version = (int64_t)o.varint(); break;
                    default: o.skip(w);
                }
            }
            if (domain.empty() || domain == "ai.onnx") m.opset = version;
        } else {
            r.skip(wire);
        }
    }
    if (!have_graph) fail("no graph in the file (not an ONNX model?)");
    return m;
}

// ------------------------------------------------------------------------------------------ graph construction

struct Val {
    View v;
    std::vector<int64_t> shape;  // ONNX shape, batch dimension included
    int producer = -1;           // index of the stage whose output this is (same bytes, same extent), -1 otherwise
};

class Importer {
  public:
    explicit Importer(OModel m) : m_(std::move(m)) {}

    Graph run(const std::string& name) {
        g_.name = name;
        for (const ONode& n : m_.nodes)
            for (const std::string& s : n.in) ++uses_[s];
        for (const std::string& s : m_.outputs) ++uses_[s];
        for (ONode& n : m_.nodes)
            if (n.op == "Constant") {
                auto it = n.attr.find("value");
                if (it == n.attr.end() || !it->second.t || n.out.empty()) fail(n.label() + ": only tensor constants are read");
                Tensor t = *it->second.t;
                t.name = n.out[0];
                m_.init[n.out[0]] = std::move(t);
            }
        bind_input();
        for (const ONode& n : m_.nodes) node(n);
        if (m_.outputs.empty()) fail("the graph has no output");
        g_.output = val(m_.outputs[0], "graph output").v;
        compact();
        return std::move(g_);
    }

  private:
    // ---- values
    bool is_init(const std::string& s) const { return m_.init.count(s) != 0; }

    const Tensor& init_f(const ONode& n, const std::string& s) const {
        auto it = m_.init.find(s);
        if (it == m_.init.end()) fail(n.label() + ": input '" + s + "' must be a constant of the file");
        if (it->second.f.size() != it->second.numel() || it->second.f.empty()) fail(n.label() + ": constant '" + s + "' is not a float tensor");
        return it->second;
    }

    const Tensor& init_i(const ONode& n, const std::string& s) const {
        auto it = m_.init.find(s);
        if (it == m_.init.end() || it->second.i.size() != it->second.numel()) fail(n.label() + ": input '" + s + "' must be an integer constant of the file");
        return it->second;
    }

    const Val& val(const std::string& s, const std::string& who) const {
        auto it = vals_.find(s);
        if (it == vals_.end()) fail(who + ": tensor '" + s + "' is not produced by any supported node before its use");
        return it->second;
    }

    int uses(const std::string& s) const {
        auto it = uses_.find(s);
        return it == uses_.end() ? 0 : it->second;
    }

    static View view_of(View base, const std::vector<int64_t>& shape, const std::string& who) {
        // batch dimension dropped, the rest padded with ones to (C, H, W)
        if (shape.empty() || shape[0] != 1) fail(who + ": only batch 1 is served");
        if (shape.size() > 4) fail(who + ": tensors of more than 4 dimensions are not supported");
        View v = base;
        v.C = shape.size() > 1 ? (int)shape[1] : 1;
        v.H = shape.size() > 2 ? (int)shape[2] : 1;
        v.W = shape.size() > 3 ? (int)shape[3] : 1;
        if (v.numel() != base.numel()) fail(who + ": reshape changes the element count");
        return v;
    }

    View new_buffer(int C, int H, int W) {
        if (C <= 0 || H <= 0 || W <= 0) fail("empty tensor");
        Buffer b{C, H, W, 0};
        g_.buffers.push_back(b);
        View v;
        v.buf = (int)g_.buffers.size() - 1;
        v.C = C;
        v.H = H;
        v.W = W;
        return v;
    }

    int add_weight(std::vector<int> shape, std::vector<float> data) {
        WeightTensor t;
        t.shape = std::move(shape);
        t.fill = Fill::External;
        t.data = std::make_shared<std::vector<float>>(std::move(data));
        if (t.data->size() != t.numel()) fail("internal: weight size mismatch");
        g_.weights.push_back(std::move(t));
        return (int)g_.weights.size() - 1;
    }

    std::vector<float>& weight(int id) { return *g_.weights[id].data; }

    void set(const std::string& name, View v, std::vector<int64_t> shape, int producer) {
        Val x;
        x.v = v;
        x.shape = std::move(shape);
        x.producer = producer;
        vals_[name] = std::move(x);
    }

    int emit(const Node& n, const std::string& out, std::vector<int64_t> shape) {
        g_.nodes.push_back(n);
        const int idx = (int)g_.nodes.size() - 1;
        set(out, n.y, std::move(shape), idx);
        return idx;
    }

    // The stage that produced `s`, if this node is its only reader and may therefore change it.
    Node* sole_producer(const std::string& s) {
        const Val& v = val(s, "fusion");
        if (v.producer < 0 || uses(s) != 1) return nullptr;
        return &g_.nodes[v.producer];
    }

    void bind_input() {
        const ValueInfo* in = nullptr;
        for (const ValueInfo& v : m_.inputs)
            if (!is_init(v.name)) {
                if (in) fail("more than one graph input ('" + in->name + "', '" + v.name + "')");
                in = &v;
            }
        if (!in) fail("the graph has no input");
        std::vector<int64_t> shape = in->dims;
        if (shape.size() < 2 || shape.size() > 4) fail("input '" + in->name + "' must have 2 to 4 dimensions");
        if (shape[0] == 0) shape[0] = 1;  // symbolic batch
        for (int64_t d : shape)
            if (d <= 0) fail("input '" + in->name + "' has a symbolic dimension other than the batch");
        if (shape[0] != 1) fail("only batch 1 is served (input '" + in->name + "')");
        View v = new_buffer((int)shape[1], shape.size() > 2 ? (int)shape[2] : 1, shape.size() > 3 ? (int)shape[3] : 1);
        g_.input = v;
        set(in->name, v, shape, -1);
    }

    // ---- operators
    static void spatial_pads(const ONode& n, int in_h, int in_w, int kh, int kw, int sh, int sw, int dh, int dw, bool ceil_mode, int* ph, int* pw) {
        const std::string auto_pad = n.gets("auto_pad", "NOTSET");
        std::vector<int64_t> pads = n.getints("pads");
        if (auto_pad == "NOTSET" || auto_pad.empty()) {
            if (pads.empty()) pads = {0, 0, 0, 0};
            if (pads.size() != 4) fail(n.label() + ": only two spatial dimensions are supported");
            if (pads[0] != pads[2] || pads[1] != pads[3]) fail(n.label() + ": asymmetric padding is not supported");
            *ph = (int)pads[0];
            *pw = (int)pads[1];
        } else if (auto_pad == "VALID") {
            *ph = *pw = 0;
        } else if (auto_pad == "SAME_UPPER" || auto_pad == "SAME_LOWER") {
            auto total = [](int in, int k, int s, int d) {
                const int out = (in + s - 1) / s;
                const int t = (out - 1) * s + (k - 1) * d + 1 - in;
                return t > 0 ? t : 0;
            };
            const int th = total(in_h, kh, sh, dh), tw = total(in_w, kw, sw, dw);
            if ((th | tw) & 1) fail(n.label() + ": auto_pad needs asymmetric padding here, which is not supported");
            *ph = th / 2;
            *pw = tw / 2;
        } else {
            fail(n.label() + ": unknown auto_pad '" + auto_pad + "'");
        }
        (void)ceil_mode;
    }

    void op_conv(const ONode& n) {
        const Val& x = val(n.in.at(0), n.label());
        if (x.shape.size() != 4) fail(n.label() + ": input must be NCHW");
        const Tensor& w = init_f(n, n.in.at(1));
        if (w.dims.size() != 4) fail(n.label() + ": only 2-D convolutions are supported");
        const int K = (int)w.dims[0], cg = (int)w.dims[1], R = (int)w.dims[2], S = (int)w.dims[3];
        const int groups = (int)n.geti("group", 1);
        std::vector<int64_t> strides = n.getints("strides"), dil = n.getints("dilations"), ks = n.getints("kernel_shape");
        if (strides.empty()) strides = {1, 1};
        if (dil.empty()) dil = {1, 1};
        if (strides.size() != 2 || dil.size() != 2) fail(n.label() + ": only two spatial dimensions are supported");
        if (!ks.empty() && (ks.size() != 2 || ks[0] != R || ks[1] != S)) fail(n.label() + ": kernel_shape disagrees with the weight tensor");
        if (dil[0] != dil[1]) fail(n.label() + ": different dilations per axis are not supported");
        if (groups <= 0 || x.v.C != cg * groups || K % groups) fail(n.label() + ": channel counts do not match the weight tensor");
        Node node{};
        node.op = Op::Conv;
        node.x = x.v;
        paella_conv_desc& d = node.conv;
        d.C = x.v.C; d.H = x.v.H; d.W = x.v.W;
        d.K = K; d.R = R; d.S = S;
        d.stride_h = (int)strides[0]; d.stride_w = (int)strides[1];
        d.dil_h = d.dil_w = (int)dil[0];
        d.groups = groups;
        spatial_pads(n, d.H, d.W, R, S, d.stride_h, d.stride_w, d.dil_h, d.dil_w, false, &d.pad_h, &d.pad_w);
        d.act = PAELLA_ACT_NONE;
        const int P = (d.H + 2 * d.pad_h - d.dil_h * (R - 1) - 1) / d.stride_h + 1, Q = (d.W + 2 * d.pad_w - d.dil_w * (S - 1) - 1) / d.stride_w + 1;
        if (P <= 0 || Q <= 0) fail(n.label() + ": empty output");
        node.w = add_weight({K, cg, R, S}, w.f);
        std::vector<float> bias(K, 0.f);
        if (n.in.size() > 2 && !n.in[2].empty()) {
            const Tensor& b = init_f(n, n.in[2]);
            if ((int)b.numel() != K) fail(n.label() + ": bias length");
            bias = b.f;
        }
        node.bias = add_weight({K}, std::move(bias));
        node.y = new_buffer(K, P, Q);
        emit(node, n.out.at(0), {1, K, P, Q});
    }

    void op_batchnorm(const ONode& n) {
        const Val x = val(n.in.at(0), n.label());
        const Tensor &sc = init_f(n, n.in.at(1)), &b = init_f(n, n.in.at(2)), &mean = init_f(n, n.in.at(3)), &var = init_f(n, n.in.at(4));
        const int C = x.v.C;
        if ((int)sc.numel() != C || (int)b.numel() != C || (int)mean.numel() != C || (int)var.numel() != C) fail(n.label() + ": parameter length");
        const float eps = n.getf("epsilon", 1e-5f);
        std::vector<float> scale(C), shift(C);
        for (int c = 0; c < C; ++c) {
            const double s = (double)sc.f[c] / std::sqrt((double)var.f[c] + (double)eps);
            scale[c] = (float)s;
            shift[c] = (float)((double)b.f[c] - (double)mean.f[c] * s);
        }
        per_channel_affine(n, x, scale, shift);
    }

    // y = x * scale[c] + shift[c]: folded into the producing conv when nothing else reads x, a stage of its own otherwise.
    void per_channel_affine(const ONode& n, const Val& x, const std::vector<float>& scale, const std::vector<float>& shift) {
        const int C = x.v.C;
        Node* p = sole_producer(n.in.at(0));
        if (p && p->op == Op::Conv && p->act == PAELLA_ACT_NONE && p->x2.buf < 0 && p->conv.K == C) {
            std::vector<float>& w = weight(p->w);
            std::vector<float>& bias = weight(p->bias);
            const size_t per = w.size() / (size_t)C;
            for (int c = 0; c < C; ++c) {
                for (size_t k = 0; k < per; ++k) w[(size_t)c * per + k] = (float)((double)w[(size_t)c * per + k] * (double)scale[c]);
                bias[c] = (float)((double)bias[c] * (double)scale[c] + (double)shift[c]);
            }
            set(n.out.at(0), x.v, x.shape, x.producer);
            return;
        }
        Node node{};
        node.op = Op::Eltwise;
        node.x = x.v;
        node.act = PAELLA_ACT_NONE;
        node.scale = add_weight({C}, scale);
        node.shift = add_weight({C}, shift);
        node.y = new_buffer(x.v.C, x.v.H, x.v.W);
        emit(node, n.out.at(0), x.shape);
    }

    void activation(const ONode& n, int act, float lo, float hi, const std::vector<float>* slope) {
        const Val x = val(n.in.at(0), n.label());
        Node* p = sole_producer(n.in.at(0));
        const bool fusable = p && p->act == PAELLA_ACT_NONE && (p->op == Op::Conv || p->op == Op::Dense || p->op == Op::Eltwise) &&
                             (!slope || p->op != Op::Dense);
        Node fresh{};
        if (!fusable) {
            fresh.op = Op::Eltwise;
            fresh.x = x.v;
            fresh.y = new_buffer(x.v.C, x.v.H, x.v.W);
            p = &fresh;
        }
        p->act = act;
        p->lo = lo;
        p->hi = hi;
        if (p->op == Op::Conv) {
            p->conv.act = act;
            p->conv.act_lo = lo;
            p->conv.act_hi = hi;
        }
        if (slope) {
            std::vector<float> s = *slope;
            if (s.size() == 1) s.assign((size_t)x.v.C, s[0]);
            if ((int)s.size() != x.v.C) fail(n.label() + ": slope must be one value or one per channel");
            p->slope = add_weight({x.v.C}, std::move(s));
        }
        if (fusable) set(n.out.at(0), x.v, x.shape, x.producer);
        else emit(fresh, n.out.at(0), x.shape);
    }

    void op_clip(const ONode& n) {
        float lo = -std::numeric_limits<float>::infinity(), hi = std::numeric_limits<float>::infinity();
        if (n.attr.count("min")) lo = n.getf("min", lo);
        if (n.attr.count("max")) hi = n.getf("max", hi);
        if (n.in.size() > 1 && !n.in[1].empty()) lo = init_f(n, n.in[1]).f.at(0);
        if (n.in.size() > 2 && !n.in[2].empty()) hi = init_f(n, n.in[2]).f.at(0);
        if (lo == 0.f && hi == 6.f) activation(n, PAELLA_ACT_RELU6, 0.f, 0.f, nullptr);
        else if (lo == 0.f && std::isinf(hi)) activation(n, PAELLA_ACT_RELU, 0.f, 0.f, nullptr);
        else if (std::isinf(lo) || std::isinf(hi)) fail(n.label() + ": one-sided clip other than relu is not supported");
        else activation(n, PAELLA_ACT_CLIP, lo, hi, nullptr);
    }

    // Add / Sub / Mul / Div
    void op_arith(const ONode& n) {
        const bool a_const = is_init(n.in.at(0)), b_const = is_init(n.in.at(1));
        if (a_const && b_const) fail(n.label() + ": constant folding of two constants is not supported");
        if (!a_const && !b_const) {
            if (n.op != "Add") fail(n.label() + ": only Add takes two activations");
            add_activations(n);
            return;
        }
        if (a_const && (n.op == "Sub" || n.op == "Div")) fail(n.label() + ": constant on the left of " + n.op + " is not supported");
        const std::string& xs = a_const ? n.in[1] : n.in[0];
        const Tensor& c = init_f(n, a_const ? n.in[0] : n.in[1]);
        const Val x = val(xs, n.label());
        const int C = x.v.C;
        // the constant must be a scalar or, under ONNX's trailing-aligned broadcasting, one value per channel
        std::vector<float> per(C);
        if (c.numel() == 1) {
            per.assign(C, c.f[0]);
        } else {
            const size_t rank = x.shape.size(), cr = c.dims.size();
            bool ok = (int)c.numel() == C && cr <= rank;
            for (size_t k = 0; ok && k < cr; ++k) {
                const size_t axis = rank - cr + k;
                ok = c.dims[k] == 1 || (axis == 1 && c.dims[k] == C);
            }
            if (!ok) fail(n.label() + ": the constant must be a scalar or one value per channel");
            per = c.f;
        }
        std::vector<float> scale(C, 1.f), shift(C, 0.f);
        for (int k = 0; k < C; ++k) {
            if (n.op == "Add") shift[k] = per[k];
            else if (n.op == "Sub") shift[k] = -per[k];
            else if (n.op == "Mul") scale[k] = per[k];
            else scale[k] = 1.f / per[k];
        }
        // Into the bias of a dense stage if that is where it came from (MatMul + Add); convs take the general path.
        Node* p = sole_producer(xs);
        if (p && p->op == Op::Dense && p->act == PAELLA_ACT_NONE && n.op == "Add") {
            std::vector<float>& bias = weight(p->bias);
            for (int k = 0; k < C; ++k) bias[k] += per[k];
            set(n.out.at(0), x.v, x.shape, x.producer);
            return;
        }
        ONode alias = n;
        alias.in[0] = xs;
        per_channel_affine(alias, x, scale, shift);
    }

    void add_activations(const ONode& n) {
        const Val a = val(n.in[0], n.label()), b = val(n.in[1], n.label());
        if (a.v.C != b.v.C || a.v.H != b.v.H || a.v.W != b.v.W) fail(n.label() + ": broadcasting between activations is not supported");
        // The later of the two producers, if it is a conv nothing else reads, takes the other operand as its
        // residual input -- provided the other operand is complete by the time that conv runs.
        const int later = a.producer >= b.producer ? 0 : 1;
        for (int idx : {later, 1 - later}) {
            const Val& mine = idx == 0 ? a : b;
            const Val& other = idx == 0 ? b : a;
            Node* p = sole_producer(n.in[idx]);
            if (p && p->op == Op::Conv && p->act == PAELLA_ACT_NONE && p->x2.buf < 0 && n.in[0] != n.in[1] && other.producer < mine.producer &&
                available_before(other.v, mine.producer)) {
                p->x2 = other.v;
                set(n.out.at(0), mine.v, mine.shape, mine.producer);
                return;
            }
        }
        Node node{};
        node.op = Op::Eltwise;
        node.x = a.v;
        node.x2 = b.v;
        node.y = new_buffer(a.v.C, a.v.H, a.v.W);
        emit(node, n.out.at(0), a.shape);
    }

    // True if every stage writing into the bytes of `v` comes before stage `idx`.
    bool available_before(const View& v, int idx) const {
        for (int k = idx; k < (int)g_.nodes.size(); ++k) {
            const View& y = g_.nodes[k].y;
            if (y.buf == v.buf && y.off < v.off + v.numel() && v.off < y.off + y.numel()) return false;
        }
        return true;
    }

    void op_pool(const ONode& n, bool avg, bool global) {
        const Val& x = val(n.in.at(0), n.label());
        if (x.shape.size() != 4) fail(n.label() + ": input must be NCHW");
        if (global && avg) {
            Node node{};
            node.op = Op::GlobalAvgPool;
            node.x = x.v;
            node.y = new_buffer(x.v.C, 1, 1);
            emit(node, n.out.at(0), {1, x.v.C, 1, 1});
            return;
        }
        Node node{};
        node.op = Op::Pool;
        node.x = x.v;
        paella_pool_desc& d = node.pool;
        d.C = x.v.C; d.H = x.v.H; d.W = x.v.W;
        d.is_avg = avg;
        if (global) {
            d.R = d.H; d.S = d.W;
            d.stride_h = d.stride_w = 1;
        } else {
            std::vector<int64_t> ks = n.getints("kernel_shape"), strides = n.getints("strides"), dil = n.getints("dilations");
            if (ks.size() != 2) fail(n.label() + ": only two spatial dimensions are supported");
            if (strides.empty()) strides = {1, 1};
            for (int64_t v : dil)
                if (v != 1) fail(n.label() + ": dilated pooling is not supported");
            d.R = (int)ks[0]; d.S = (int)ks[1];
            d.stride_h = (int)strides[0]; d.stride_w = (int)strides[1];
            d.ceil_mode = (int)n.geti("ceil_mode", 0);
            d.count_include_pad = (int)n.geti("count_include_pad", 0);
            const std::vector<int64_t> pads = n.getints("pads");
            const std::string auto_pad = n.gets("auto_pad", "NOTSET");
            if ((auto_pad == "NOTSET" || auto_pad.empty()) && pads.size() == 4 && (pads[0] != pads[2] || pads[1] != pads[3])) {
                // More padding at the end than at the start (how converters of ceil-mode frameworks write their pools).
                // Padding is never selected by a max pool and never counted by an average pool that excludes it, so this
                // is the symmetric pool with the begin padding whenever one of the two rounding modes yields the same
                // number of windows on both axes.
                if (d.is_avg && d.count_include_pad) fail(n.label() + ": asymmetric padding that counts in the average is not supported");
                d.pad_h = (int)pads[0];
                d.pad_w = (int)pads[1];
                const int want_h = (d.H + (int)pads[0] + (int)pads[2] - d.R) / d.stride_h + 1, want_w = (d.W + (int)pads[1] + (int)pads[3] - d.S) / d.stride_w + 1;
                bool ok = false;
                if (!d.ceil_mode)
                    for (int ceil = 0; ceil < 2 && !ok; ++ceil)
                        if (paella_pool_out(d.H, d.R, d.stride_h, d.pad_h, ceil) == want_h && paella_pool_out(d.W, d.S, d.stride_w, d.pad_w, ceil) == want_w) {
                            d.ceil_mode = ceil;
                            ok = true;
                        }
                if (!ok) fail(n.label() + ": asymmetric padding is not supported");
            } else {
                spatial_pads(n, d.H, d.W, d.R, d.S, d.stride_h, d.stride_w, 1, 1, d.ceil_mode != 0, &d.pad_h, &d.pad_w);
            }
            if (n.geti("storage_order", 0) != 0) fail(n.label() + ": column-major storage order is not supported");
            if (n.out.size() > 1 && !n.out[1].empty() && uses(n.out[1])) fail(n.label() + ": the indices output is not supported");
        }
        const int P = paella_pool_out(d.H, d.R, d.stride_h, d.pad_h, d.ceil_mode), Q = paella_pool_out(d.W, d.S, d.stride_w, d.pad_w, d.ceil_mode);
        if (P <= 0 || Q <= 0) fail(n.label() + ": empty output");
        node.y = new_buffer(x.v.C, P, Q);
        emit(node, n.out.at(0), {1, x.v.C, P, Q});
    }

    void dense(const ONode& n, const Val& x, const Tensor& w, bool w_is_out_by_in, float alpha, const Tensor* c, float beta) {
        if (w.dims.size() != 2) fail(n.label() + ": the weight must be a matrix");
        const int I = (int)(w_is_out_by_in ? w.dims[1] : w.dims[0]), O = (int)(w_is_out_by_in ? w.dims[0] : w.dims[1]);
        if ((size_t)I != x.v.numel()) fail(n.label() + ": input has " + std::to_string(x.v.numel()) + " elements, the weight expects " + std::to_string(I));
        std::vector<float> wt((size_t)O * I);
        for (int o = 0; o < O; ++o)
            for (int i = 0; i < I; ++i) wt[(size_t)o * I + i] = alpha * (w_is_out_by_in ? w.f[(size_t)o * I + i] : w.f[(size_t)i * O + o]);
        std::vector<float> bias(O, 0.f);
        if (c) {
            if (c->numel() == 1) bias.assign(O, beta * c->f[0]);
            else if ((int)c->numel() == O) for (int o = 0; o < O; ++o) bias[o] = beta * c->f[o];
            else fail(n.label() + ": bias length");
        }
        Node node{};
        node.op = Op::Dense;
        node.x = x.v;
        node.dense_in = I;
        node.dense_out = O;
        node.w = add_weight({O, I}, std::move(wt));
        node.bias = add_weight({O}, std::move(bias));
        node.y = new_buffer(O, 1, 1);
        emit(node, n.out.at(0), {1, O});
    }

    void op_gemm(const ONode& n) {
        const Val& x = val(n.in.at(0), n.label());
        if (n.geti("transA", 0) != 0) fail(n.label() + ": transA is not supported");
        const Tensor* c = (n.in.size() > 2 && !n.in[2].empty()) ? &init_f(n, n.in[2]) : nullptr;
        dense(n, x, init_f(n, n.in.at(1)), n.geti("transB", 0) != 0, n.getf("alpha", 1.f), c, n.getf("beta", 1.f));
    }

    void op_matmul(const ONode& n) {
        if (is_init(n.in.at(0))) fail(n.label() + ": constant on the left of MatMul is not supported");
        dense(n, val(n.in.at(0), n.label()), init_f(n, n.in.at(1)), false, 1.f, nullptr, 0.f);
    }

    void op_view(const ONode& n) {
        // a view of a constant is a constant (exporters emit Identity on shared parameters)
        const bool on_const = is_init(n.in.at(0));
        Val cx;
        if (on_const) {
            cx.shape = m_.init.at(n.in[0]).dims;
            cx.v.C = (int)m_.init.at(n.in[0]).numel();  // only the element count is used below
            cx.v.H = cx.v.W = 1;
        }
        const Val x = on_const ? cx : val(n.in.at(0), n.label());
        std::vector<int64_t> shape;
        const int64_t rank = (int64_t)x.shape.size();
        if (n.op == "Flatten") {
            int64_t axis = n.geti("axis", 1);
            if (axis < 0) axis += rank;
            int64_t a = 1, b = 1;
            for (int64_t k = 0; k < rank; ++k) (k < axis ? a : b) *= x.shape[k];
            shape = {a, b};
        } else if (n.op == "Reshape") {
            const Tensor& t = init_i(n, n.in.at(1));
            int64_t known = 1, infer = -1;
            for (size_t k = 0; k < t.i.size(); ++k) {
                int64_t d = t.i[k];
                if (d == 0) d = k < x.shape.size() ? x.shape[k] : 1;
                if (d == -1) infer = (int64_t)k;
                else known *= d;
                shape.push_back(d);
            }
            if (infer >= 0) {
                if (known <= 0) fail(n.label() + ": cannot infer a dimension next to a zero-sized one");
                shape[(size_t)infer] = (int64_t)x.v.numel() / known;
            }
        } else if (n.op == "Squeeze" || n.op == "Unsqueeze") {
            std::vector<int64_t> axes = n.getints("axes");
            if (axes.empty() && n.in.size() > 1 && !n.in[1].empty()) axes = init_i(n, n.in[1]).i;
            if (n.op == "Squeeze") {
                for (int64_t k = 0; k < rank; ++k) {
                    bool drop = axes.empty() ? (x.shape[k] == 1 && k != 0) : false;
                    for (int64_t a : axes) drop = drop || (a < 0 ? a + rank : a) == k;
                    if (drop && x.shape[k] != 1) fail(n.label() + ": squeezed dimension is not 1");
                    if (!drop) shape.push_back(x.shape[k]);
                }
            } else {
                const int64_t out_rank = rank + (int64_t)axes.size();
                size_t src = 0;
                for (int64_t k = 0; k < out_rank; ++k) {
                    bool ins = false;
                    for (int64_t a : axes) ins = ins || (a < 0 ? a + out_rank : a) == k;
                    shape.push_back(ins ? 1 : x.shape.at(src++));
                }
            }
        } else {  // Dropout, Identity
            shape = x.shape;
        }
        if (on_const) {
            Tensor t = m_.init.at(n.in[0]);
            t.name = n.out.at(0);
            t.dims = shape;
            if (t.numel() != m_.init.at(n.in[0]).numel()) fail(n.label() + ": reshape of a constant changes the element count");
            m_.init[n.out[0]] = std::move(t);
            return;
        }
        const View v = view_of(x.v, shape, n.label());
        set(n.out.at(0), v, shape, v.C == x.v.C && v.H == x.v.H && v.W == x.v.W ? x.producer : -1);
    }

    void op_concat(const ONode& n) {
        std::vector<Val> in;
        for (const std::string& s : n.in) in.push_back(val(s, n.label()));
        if (in.empty()) fail(n.label() + ": no inputs");
        int64_t axis = n.geti("axis", 1);
        const int64_t rank = (int64_t)in[0].shape.size();
        if (axis < 0) axis += rank;
        // channels are the outermost dimension of a batch-1 tensor: concatenation along them is contiguous
        for (int64_t k = 1; k < axis; ++k)
            if (in[0].shape[k] != 1) fail(n.label() + ": only concatenation along the outermost non-batch dimension is supported");
        if (axis < 1) fail(n.label() + ": concatenation along the batch is not supported");
        // in terms of (C, H, W) views: every input is [c_i, inner]
        size_t inner = 1;
        for (int64_t k = axis + 1; k < rank; ++k) inner *= (size_t)in[0].shape[k];
        std::vector<int64_t> shape = in[0].shape;
        int64_t total = 0;
        for (const Val& v : in) {
            if ((int64_t)v.shape.size() != rank) fail(n.label() + ": inputs of different rank");
            for (int64_t k = 0; k < rank; ++k)
                if (k != axis && v.shape[k] != shape[k]) fail(n.label() + ": inputs of different shape");
            total += v.shape[axis];
        }
        shape[axis] = total;
        const View whole = view_of(raw_buffer(total * inner), shape, n.label());
        size_t off = 0;
        for (size_t k = 0; k < in.size(); ++k) {
            const View v = vals_.at(n.in[k]).v;  // current location: an earlier operand's re-basing may have moved it
            const Buffer& b = g_.buffers[v.buf];
            const bool whole_buffer = v.off == 0 && v.numel() == (size_t)b.C * b.H * b.W && v.buf != g_.input.buf && v.buf != whole.buf;
            if (whole_buffer) {
                rebase(v.buf, whole.buf, off);
            } else {
                // a slice of something else, the graph input, or the same tensor twice: copied by a stage of its own
                Node node{};
                node.op = Op::Eltwise;
                node.x = v;
                node.y = v;
                node.y.buf = whole.buf;
                node.y.off = off;
                g_.nodes.push_back(node);
            }
            off += v.numel();
        }
        set(n.out.at(0), whole, shape, -1);
    }

    View raw_buffer(size_t numel) { return new_buffer((int)numel, 1, 1); }

    // Every view into buffer `from` now points into buffer `to` at `offset` floats.
    void rebase(int from, int to, size_t offset) {
        auto fix = [&](View& v) {
            if (v.buf == from) {
                v.buf = to;
                v.off += offset;
            }
        };
        for (Node& node : g_.nodes) {
            fix(node.x);
            fix(node.x2);
            fix(node.y);
        }
        for (auto& kv : vals_) fix(kv.second.v);
    }

    // Shape / Gather / Concat / Cast over constants: the static shape arithmetic exporters leave in front of a Reshape.
    bool fold_constant(const ONode& n) {
        auto put = [&](std::vector<int64_t> dims, std::vector<int64_t> values) {
            Tensor t;
            t.name = n.out.at(0);
            t.dims = std::move(dims);
            t.dtype = kInt64;
            t.i = std::move(values);
            m_.init[t.name] = std::move(t);
        };
        if (n.op == "Shape") {
            if (is_init(n.in.at(0))) {
                const std::vector<int64_t> dims = m_.init.at(n.in[0]).dims;
                put({(int64_t)dims.size()}, dims);
            } else {
                const Val& x = val(n.in.at(0), n.label());
                put({(int64_t)x.shape.size()}, x.shape);
            }
            return true;
        }
        bool all_const = !n.in.empty();
        for (const std::string& s : n.in) all_const = all_const && (s.empty() || is_init(s));
        if (!all_const) return false;
        if (n.op == "Gather") {
            const Tensor &data = init_i(n, n.in.at(0)), &idx = init_i(n, n.in.at(1));
            if (data.dims.size() > 1 || n.geti("axis", 0) != 0) fail(n.label() + ": only gathers from a vector are folded");
            std::vector<int64_t> out;
            for (int64_t k : idx.i) out.push_back(data.i.at((size_t)(k < 0 ? k + (int64_t)data.i.size() : k)));
            put(idx.dims, out);
            return true;
        }
        if (n.op == "Concat") {
            std::vector<int64_t> out;
            for (const std::string& s : n.in) {
                const Tensor& t = init_i(n, s);
                if (t.dims.size() > 1) fail(n.label() + ": only vectors of integers are concatenated at import time");
                out.insert(out.end(), t.i.begin(), t.i.end());
            }
            put({(int64_t)out.size()}, out);
            return true;
        }
        if (n.op == "Cast") {
            Tensor t = m_.init.at(n.in.at(0));
            const int64_t to = n.geti("to", 0);
            if ((to == kInt64 || to == kInt32) && t.i.size() == t.numel()) {
                t.dtype = (int)to;
            } else if (to == kFloat && t.f.size() == t.numel()) {
                t.dtype = kFloat;
            } else if (to == kFloat && t.i.size() == t.numel()) {
                t.f.assign(t.i.begin(), t.i.end());
                t.i.clear();
                t.dtype = kFloat;
            } else {
                fail(n.label() + ": cast of a constant to this type is not supported");
            }
            t.name = n.out.at(0);
            m_.init[t.name] = std::move(t);
            return true;
        }
        return false;
    }

    void op_softmax(const ONode& n) {
        const Val& x = val(n.in.at(0), n.label());
        const int64_t rank = (int64_t)x.shape.size();
        int64_t axis = n.geti("axis", m_.opset >= 13 ? -1 : 1);
        if (axis < 0) axis += rank;
        size_t cols = 1;
        for (int64_t k = axis; k < rank; ++k) cols *= (size_t)x.shape[k];
        if (m_.opset >= 13) {
            // one axis only: it must be the last one that is not 1
            for (int64_t k = axis + 1; k < rank; ++k)
                if (x.shape[k] != 1) fail(n.label() + ": softmax over an inner axis is not supported");
        }
        Node node{};
        node.op = Op::Softmax;
        node.x = x.v;
        node.cols = (int)cols;
        node.rows = (int)(x.v.numel() / cols);
        node.y = new_buffer(x.v.C, x.v.H, x.v.W);
        emit(node, n.out.at(0), x.shape);
    }

    void op_lrn(const ONode& n) {
        const Val& x = val(n.in.at(0), n.label());
        Node node{};
        node.op = Op::Lrn;
        node.x = x.v;
        node.lrn_size = (int)n.geti("size", 0);
        if (node.lrn_size <= 0) fail(n.label() + ": size attribute missing");
        node.lrn_alpha = n.getf("alpha", 1e-4f);
        node.lrn_beta = n.getf("beta", 0.75f);
        node.lrn_k = n.getf("bias", 1.f);
        node.y = new_buffer(x.v.C, x.v.H, x.v.W);
        emit(node, n.out.at(0), x.shape);
    }

    void node(const ONode& n) {
        if (n.op == "Constant") return;
        if (n.out.empty()) fail(n.label() + ": no output");
        if ((n.op == "Shape" || n.op == "Gather" || n.op == "Concat" || n.op == "Cast") && fold_constant(n)) return;
        if (n.op == "Conv") op_conv(n);
        else if (n.op == "BatchNormalization") op_batchnorm(n);
        else if (n.op == "Relu") activation(n, PAELLA_ACT_RELU, 0.f, 0.f, nullptr);
        else if (n.op == "Clip") op_clip(n);
        else if (n.op == "PRelu") activation(n, PAELLA_ACT_PRELU, 0.f, 0.f, &init_f(n, n.in.at(1)).f);
        else if (n.op == "LeakyRelu") {
            const std::vector<float> slope{n.getf("alpha", 0.01f)};
            activation(n, PAELLA_ACT_PRELU, 0.f, 0.f, &slope);
        } else if (n.op == "Add" || n.op == "Sub" || n.op == "Mul" || n.op == "Div") op_arith(n);
        else if (n.op == "MaxPool") op_pool(n, false, false);
        else if (n.op == "AveragePool") op_pool(n, true, false);
        else if (n.op == "GlobalAveragePool") op_pool(n, true, true);
        else if (n.op == "GlobalMaxPool") op_pool(n, false, true);
        else if (n.op == "Gemm") op_gemm(n);
        else if (n.op == "MatMul") op_matmul(n);
        else if (n.op == "Flatten" || n.op == "Reshape" || n.op == "Squeeze" || n.op == "Unsqueeze" || n.op == "Dropout" || n.op == "Identity") op_view(n);
        else if (n.op == "Concat") op_concat(n);
        else if (n.op == "Softmax") op_softmax(n);
        else if (n.op == "LRN") op_lrn(n);
        else fail(n.label() + ": operator not supported");
    }

    // Drops buffers nothing refers to any more (re-based concat inputs) and lays the rest out in the arena.
    void compact() {
        std::vector<int> remap(g_.buffers.size(), -1);
        auto mark = [&](const View& v) {
            if (v.buf >= 0) remap[v.buf] = 0;
        };
        mark(g_.input);
        mark(g_.output);
        for (const Node& n : g_.nodes) {
            mark(n.x);
            mark(n.x2);
            mark(n.y);
        }
        std::vector<Buffer> kept;
        size_t arena = 0;
        for (size_t b = 0; b < g_.buffers.size(); ++b) {
            if (remap[b] < 0) continue;
            remap[b] = (int)kept.size();
            Buffer nb = g_.buffers[b];
            nb.offset = arena;
            arena += ((size_t)nb.C * nb.H * nb.W + 63) / 64 * 64;
            kept.push_back(nb);
        }
        auto fix = [&](View& v) {
            if (v.buf >= 0) v.buf = remap[v.buf];
        };
        fix(g_.input);
        fix(g_.output);
        for (Node& n : g_.nodes) {
            fix(n.x);
            fix(n.x2);
            fix(n.y);
        }
        g_.buffers = std::move(kept);
        g_.arena_floats = arena;
    }

    OModel m_;
    Graph g_;
    std::map<std::string, Val> vals_;
    std::map<std::string, int> uses_;
};

}  // namespace

Graph import_onnx(const std::string& path, const std::string& name) {
    std::ifstream f(path, std::ios::binary);
    if (!f) fail("cannot open " + path);
    std::vector<uint8_t> bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (bytes.empty()) fail(path + " is empty");
    return Importer(parse_model(bytes)).run(name);
}

}  // namespace paella
