#include "graph.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <stdexcept>

namespace paella {

namespace {

int conv_out(int in, int k, int stride, int pad, int dil) { return (in + 2 * pad - dil * (k - 1) - 1) / stride + 1; }

void require(bool ok, const char* what) {
    if (!ok) throw std::logic_error(std::string("graph construction: ") + what);
}

}  // namespace

View GraphBuilder::buffer(int C, int H, int W) {
    require(C > 0 && H > 0 && W > 0, "empty buffer");
    Buffer b{C, H, W, g_.arena_floats};
    // keep every buffer 256-byte aligned so 16-byte vector accesses are always legal
    g_.arena_floats += ((size_t)C * H * W + 63) / 64 * 64;
    g_.buffers.push_back(b);
    View v;
    v.buf = (int)g_.buffers.size() - 1;
    v.off = 0;
    v.C = C;
    v.H = H;
    v.W = W;
    return v;
}

View GraphBuilder::input(int C, int H, int W) {
    g_.input = buffer(C, H, W);
    return g_.input;
}

View GraphBuilder::slice(const View& v, int c_off, int C) {
    require(c_off >= 0 && C > 0 && c_off + C <= v.C, "slice out of range");
    View s = v;
    s.off = v.off + (size_t)c_off * v.H * v.W;
    s.C = C;
    return s;
}

View GraphBuilder::reshape(const View& x, int C, int H, int W) {
    require((size_t)C * H * W == x.numel(), "reshape changes the element count");
    View v = x;
    v.C = C;
    v.H = H;
    v.W = W;
    return v;
}

int GraphBuilder::add_weight(std::vector<int> shape, Fill fill, double a, double b) {
    WeightTensor t;
    t.shape = std::move(shape);
    t.fill = fill;
    t.a = a;
    t.b = b;
    g_.weights.push_back(t);
    return (int)g_.weights.size() - 1;
}

View GraphBuilder::out_view(int C, int H, int W, const View* dst) {
    if (!dst) return buffer(C, H, W);
    require(dst->C == C && dst->H == H && dst->W == W, "destination slice has the wrong shape");
    return *dst;
}

View GraphBuilder::conv(const View& x, int K, int R, int S, const ConvOpt& o, const View* residual, const View* dst) {
    Node n{};
    n.op = Op::Conv;
    n.x = x;
    paella_conv_desc& d = n.conv;
    d.C = x.C; d.H = x.H; d.W = x.W;
    d.K = K; d.R = R; d.S = S;
    d.stride_h = o.stride_h; d.stride_w = o.stride_w;
    d.pad_h = o.pad_h; d.pad_w = o.pad_w;
    d.dil_h = d.dil_w = o.dil;
    d.groups = o.groups;
    d.act = o.act; d.act_lo = o.lo; d.act_hi = o.hi;
    const int P = conv_out(x.H, R, o.stride_h, o.pad_h, o.dil), Q = conv_out(x.W, S, o.stride_w, o.pad_w, o.dil);
    require(P > 0 && Q > 0, "conv output is empty");
    require(x.C % o.groups == 0 && K % o.groups == 0, "channels not divisible by groups");
    const int cg = x.C / o.groups;
    const double fan_in = (double)cg * R * S;
    n.w = add_weight({K, cg, R, S}, Fill::Normal, o.gain * std::sqrt(2.0 / fan_in));
    if (o.bias) n.bias = bias_std_ > 0 ? add_weight({K}, Fill::Normal, bias_std_) : add_weight({K}, Fill::Constant, 0.0);
    if (o.act == PAELLA_ACT_PRELU) n.slope = add_weight({K}, Fill::Constant, 0.25);
    n.act = o.act; n.lo = o.lo; n.hi = o.hi;
    if (residual) {
        require(residual->C == K && residual->H == P && residual->W == Q, "residual shape mismatch");
        n.x2 = *residual;
    }
    n.y = out_view(K, P, Q, dst);
    g_.nodes.push_back(n);
    return n.y;
}

View GraphBuilder::conv(const View& x, int K, int k, int stride, int pad, int act, const View* residual, const View* dst, double gain) {
    ConvOpt o;
    o.stride_h = o.stride_w = stride;
    o.pad_h = o.pad_w = pad;
    o.act = act;
    o.gain = gain;
    return conv(x, K, k, k, o, residual, dst);
}

View GraphBuilder::dwconv(const View& x, int k, int stride, int pad, int act) {
    ConvOpt o;
    o.stride_h = o.stride_w = stride;
    o.pad_h = o.pad_w = pad;
    o.groups = x.C;
    o.act = act;
    return conv(x, x.C, k, k, o);
}

View GraphBuilder::dense(const View& x, int O, int act, double std_scale) {
    Node n{};
    n.op = Op::Dense;
    n.x = x;
    n.dense_in = (int)x.numel();
    n.dense_out = O;
    n.act = act;
    n.w = add_weight({O, n.dense_in}, Fill::Normal, std_scale * std::sqrt(2.0 / n.dense_in));
    n.bias = bias_std_ > 0 ? add_weight({O}, Fill::Normal, bias_std_) : add_weight({O}, Fill::Constant, 0.0);
    n.y = buffer(O, 1, 1);
    g_.nodes.push_back(n);
    return n.y;
}

View GraphBuilder::pool(const View& x, bool avg, int k, int stride, int pad, bool ceil_mode, bool count_include_pad, const View* dst) {
    Node n{};
    n.op = Op::Pool;
    n.x = x;
    paella_pool_desc& d = n.pool;
    d.C = x.C; d.H = x.H; d.W = x.W;
    d.R = d.S = k;
    d.stride_h = d.stride_w = stride;
    d.pad_h = d.pad_w = pad;
    d.ceil_mode = ceil_mode;
    d.is_avg = avg;
    d.count_include_pad = count_include_pad;
    auto out = [&](int in) {
        const int num = in + 2 * pad - k;
        int o = ceil_mode ? (num + stride - 1) / stride + 1 : num / stride + 1;
        if (ceil_mode && (o - 1) * stride >= in + pad) --o;
        return o;
    };
    n.y = out_view(x.C, out(x.H), out(x.W), dst);
    g_.nodes.push_back(n);
    return n.y;
}

View GraphBuilder::global_avgpool(const View& x) {
    Node n{};
    n.op = Op::GlobalAvgPool;
    n.x = x;
    n.y = buffer(x.C, 1, 1);
    g_.nodes.push_back(n);
    return n.y;
}

View GraphBuilder::add(const View& a, const View& b, int act) {
    require(a.C == b.C && a.H == b.H && a.W == b.W, "add shape mismatch");
    Node n{};
    n.op = Op::Eltwise;
    n.x = a;
    n.x2 = b;
    n.act = act;
    n.y = buffer(a.C, a.H, a.W);
    g_.nodes.push_back(n);
    return n.y;
}

View GraphBuilder::scale_shift(const View& x, int act, const View* dst) {
    Node n{};
    n.op = Op::Eltwise;
    n.x = x;
    n.act = act;
    n.scale = add_weight({x.C}, Fill::Uniform, 0.5, 1.5);
    n.shift = add_weight({x.C}, Fill::Normal, 0.1);
    n.y = out_view(x.C, x.H, x.W, dst);
    g_.nodes.push_back(n);
    return n.y;
}

View GraphBuilder::prelu(const View& x) {
    Node n{};
    n.op = Op::Eltwise;
    n.x = x;
    n.act = PAELLA_ACT_PRELU;
    n.slope = add_weight({x.C}, Fill::Constant, 0.25);
    n.y = buffer(x.C, x.H, x.W);
    g_.nodes.push_back(n);
    return n.y;
}

View GraphBuilder::softmax(const View& x, int rows, int cols) {
    require((size_t)rows * cols == x.numel(), "softmax shape mismatch");
    Node n{};
    n.op = Op::Softmax;
    n.x = x;
    n.rows = rows;
    n.cols = cols;
    n.y = buffer(x.C, x.H, x.W);
    g_.nodes.push_back(n);
    return n.y;
}

View GraphBuilder::lrn(const View& x, int size, float alpha, float beta, float k) {
    Node n{};
    n.op = Op::Lrn;
    n.x = x;
    n.lrn_size = size;
    n.lrn_alpha = alpha;
    n.lrn_beta = beta;
    n.lrn_k = k;
    n.y = buffer(x.C, x.H, x.W);
    g_.nodes.push_back(n);
    return n.y;
}

Graph GraphBuilder::finish(const View& output) {
    g_.output = output;
    return g_;
}

double Graph::macs() const {
    double total = 0;
    for (const Node& n : nodes) {
        if (n.op == Op::Conv) total += (double)n.conv.K * (n.conv.C / n.conv.groups) * n.conv.R * n.conv.S * n.y.H * n.y.W;
        if (n.op == Op::Dense) total += (double)n.dense_in * n.dense_out;
    }
    return total;
}

double Graph::params() const {
    double total = 0;
    for (const WeightTensor& w : weights) total += (double)w.numel();
    return total;
}

// ------------------------------------------------------------------------------------------ seeded fill

namespace {

inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline double u01(uint64_t seed, uint64_t stream, uint64_t idx) {
    const uint64_t key = seed * 0x9E3779B97F4A7C15ull + stream * 0xD1B54A32D192ED03ull + idx;
    return ((double)(splitmix64(key) >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}

}  // namespace

void fill_weight(const WeightTensor& t, uint64_t seed, uint64_t stream, float* out) {
    const size_t n = t.numel();
    if (t.fill == Fill::External) {
        if (!t.data || t.data->size() != n) throw std::logic_error("external weight tensor without values");
        std::copy(t.data->begin(), t.data->end(), out);
        return;
    }
    const double two_pi = 6.283185307179586476925286766559;
    for (size_t i = 0; i < n; ++i) {
        switch (t.fill) {
            case Fill::Normal: {
                const double u1 = u01(seed, stream, 2 * i), u2 = u01(seed, stream, 2 * i + 1);
                const double r = std::sqrt(-2.0 * std::log(u1));
                const double z = r * std::cos(two_pi * u2);
                out[i] = (float)(z * t.a);
                break;
            }
            case Fill::Uniform:
                out[i] = (float)(t.a + (t.b - t.a) * u01(seed, stream, 2 * i));
                break;
            case Fill::Constant:
                out[i] = (float)t.a;
                break;
            case Fill::External:
                break;
        }
    }
}

// ------------------------------------------------------------------------------------------ description

namespace {

void put_view(std::string& s, const char* key, const View& v) {
    char buf[160];
    std::snprintf(buf, sizeof(buf), "\"%s\": {\"buf\": %d, \"off\": %zu, \"C\": %d, \"H\": %d, \"W\": %d}", key, v.buf, v.off, v.C, v.H, v.W);
    s += buf;
}

}  // namespace

std::string describe_json(const Graph& g) {
    std::string s;
    char buf[512];
    s += "{\"name\": \"" + g.name + "\", ";
    std::snprintf(buf, sizeof(buf), "\"macs\": %.0f, \"params\": %.0f, \"arena_floats\": %zu, ", g.macs(), g.params(), g.arena_floats);
    s += buf;
    put_view(s, "input", g.input);
    s += ", ";
    put_view(s, "output", g.output);
    s += ", \"buffers\": [";
    for (size_t i = 0; i < g.buffers.size(); ++i) {
        std::snprintf(buf, sizeof(buf), "%s{\"C\": %d, \"H\": %d, \"W\": %d}", i ? ", " : "", g.buffers[i].C, g.buffers[i].H, g.buffers[i].W);
        s += buf;
    }
    s += "], \"weights\": [";
    for (size_t i = 0; i < g.weights.size(); ++i) {
        const WeightTensor& w = g.weights[i];
        s += i ? ", {\"shape\": [" : "{\"shape\": [";
        for (size_t d = 0; d < w.shape.size(); ++d) s += (d ? ", " : "") + std::to_string(w.shape[d]);
        const char* fill = w.fill == Fill::Normal ? "normal" : w.fill == Fill::Uniform ? "uniform" : w.fill == Fill::Constant ? "constant" : "external";
        std::snprintf(buf, sizeof(buf), "], \"fill\": \"%s\", \"a\": %.17g, \"b\": %.17g}", fill, w.a, w.b);
        s += buf;
    }
    s += "], \"nodes\": [";
    for (size_t i = 0; i < g.nodes.size(); ++i) {
        const Node& n = g.nodes[i];
        s += i ? ", {" : "{";
        const char* op = n.op == Op::Conv ? "conv" : n.op == Op::Dense ? "dense" : n.op == Op::Pool ? "pool" : n.op == Op::GlobalAvgPool ? "gap"
                       : n.op == Op::Eltwise ? "eltwise" : n.op == Op::Softmax ? "softmax" : "lrn";
        s += std::string("\"op\": \"") + op + "\", ";
        put_view(s, "x", n.x);
        s += ", ";
        put_view(s, "x2", n.x2);
        s += ", ";
        put_view(s, "y", n.y);
        std::snprintf(buf, sizeof(buf), ", \"act\": %d, \"lo\": %.9g, \"hi\": %.9g, \"w\": %d, \"bias\": %d, \"slope\": %d, \"scale\": %d, \"shift\": %d", n.act,
                      n.lo, n.hi, n.w, n.bias, n.slope, n.scale, n.shift);
        s += buf;
        if (n.op == Op::Conv) {
            const paella_conv_desc& d = n.conv;
            std::snprintf(buf, sizeof(buf), ", \"K\": %d, \"R\": %d, \"S\": %d, \"stride\": [%d, %d], \"pad\": [%d, %d], \"dil\": [%d, %d], \"groups\": %d", d.K,
                          d.R, d.S, d.stride_h, d.stride_w, d.pad_h, d.pad_w, d.dil_h, d.dil_w, d.groups);
            s += buf;
        } else if (n.op == Op::Pool) {
            const paella_pool_desc& d = n.pool;
            std::snprintf(buf, sizeof(buf), ", \"k\": [%d, %d], \"stride\": [%d, %d], \"pad\": [%d, %d], \"ceil\": %d, \"avg\": %d, \"count_include_pad\": %d",
                          d.R, d.S, d.stride_h, d.stride_w, d.pad_h, d.pad_w, d.ceil_mode, d.is_avg, d.count_include_pad);
            s += buf;
        } else if (n.op == Op::Dense) {
            std::snprintf(buf, sizeof(buf), ", \"I\": %d, \"O\": %d", n.dense_in, n.dense_out);
            s += buf;
        } else if (n.op == Op::Softmax) {
            std::snprintf(buf, sizeof(buf), ", \"rows\": %d, \"cols\": %d", n.rows, n.cols);
            s += buf;
        } else if (n.op == Op::Lrn) {
            std::snprintf(buf, sizeof(buf), ", \"size\": %d, \"alpha\": %.9g, \"beta\": %.9g, \"k\": %.9g", n.lrn_size, n.lrn_alpha, n.lrn_beta, n.lrn_k);
            s += buf;
        }
        s += "}";
    }
    s += "]}";
    return s;
}

}  // namespace paella
