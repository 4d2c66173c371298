// Topology tables of the served models (fp32, batch 1, batch-norm folded into the preceding conv's weight
// scale and bias wherever a conv precedes it).  They cover the model list of the reference's adapters
// (reference jobs/tvm_*/) and the configurations of the benchmark: the small CNN, ResNet-18/34/50,
// MobileNetV2, Inception-v3 at 299x299, SqueezeNet-1.1, GoogLeNet, DenseNet-121, a 320x240 face detector
// and the ResNet-100 face-embedding net.
//
// `kResGain` scales the He-normal std of the last conv of every residual branch (it plays the role of the
// folded batch-norm gamma) so activations stay O(1)..O(10) through up to 49 residual units.

#include "graph.h"

#include <cstring>
#include <functional>
#include <map>

namespace paella {

namespace {

constexpr double kResGain = 0.3;
constexpr int RELU = PAELLA_ACT_RELU, RELU6 = PAELLA_ACT_RELU6, NONE = PAELLA_ACT_NONE, PRELU = PAELLA_ACT_PRELU;

// ---------------------------------------------------------------- small CNN (mnist-8 topology)
Graph mnist() {
    GraphBuilder b("mnist", /*bias_std=*/0.0);
    View x = b.input(1, 28, 28);
    x = b.conv(x, 8, 5, 1, 2, RELU);
    x = b.pool(x, false, 2, 2, 0);
    x = b.conv(x, 16, 5, 1, 2, RELU);
    x = b.pool(x, false, 3, 3, 0);
    x = b.dense(GraphBuilder::reshape(x, 256, 1, 1), 10);
    return b.finish(x);
}

// ---------------------------------------------------------------- ResNet
View basic_block(GraphBuilder& b, View x, int planes, int stride) {
    View identity = x;
    if (stride != 1 || x.C != planes) identity = b.conv(x, planes, 1, stride, 0, NONE);
    View y = b.conv(x, planes, 3, stride, 1, RELU);
    return b.conv(y, planes, 3, 1, 1, RELU, &identity, nullptr, kResGain);
}

View bottleneck(GraphBuilder& b, View x, int planes, int stride) {
    View identity = x;
    if (stride != 1 || x.C != planes * 4) identity = b.conv(x, planes * 4, 1, stride, 0, NONE);
    View y = b.conv(x, planes, 1, 1, 0, RELU);
    y = b.conv(y, planes, 3, stride, 1, RELU);
    return b.conv(y, planes * 4, 1, 1, 0, RELU, &identity, nullptr, kResGain);
}

Graph resnet(const char* name, bool bottle, const int (&layers)[4]) {
    GraphBuilder b(name);
    View x = b.input(3, 224, 224);
    x = b.conv(x, 64, 7, 2, 3, RELU);
    x = b.pool(x, false, 3, 2, 1);
    const int planes[4] = {64, 128, 256, 512};
    for (int s = 0; s < 4; ++s)
        for (int i = 0; i < layers[s]; ++i) {
            const int stride = (i == 0 && s > 0) ? 2 : 1;
            x = bottle ? bottleneck(b, x, planes[s], stride) : basic_block(b, x, planes[s], stride);
        }
    x = b.global_avgpool(x);
    x = b.dense(x, 1000);
    return b.finish(x);
}

// ---------------------------------------------------------------- MobileNetV2 (width 1.0)
Graph mobilenetv2() {
    GraphBuilder b("mobilenetv2");
    View x = b.input(3, 224, 224);
    x = b.conv(x, 32, 3, 2, 1, RELU6);
    const int cfg[7][4] = {{1, 16, 1, 1}, {6, 24, 2, 2}, {6, 32, 3, 2}, {6, 64, 4, 2}, {6, 96, 3, 1}, {6, 160, 3, 2}, {6, 320, 1, 1}};
    for (const auto& c : cfg)
        for (int i = 0; i < c[2]; ++i) {
            const int stride = i == 0 ? c[3] : 1;
            const bool use_res = stride == 1 && x.C == c[1];
            View y = x;
            if (c[0] != 1) y = b.conv(y, x.C * c[0], 1, 1, 0, RELU6);
            y = b.dwconv(y, 3, stride, 1, RELU6);
            x = b.conv(y, c[1], 1, 1, 0, NONE, use_res ? &x : nullptr, nullptr, use_res ? kResGain : 1.0);
        }
    x = b.conv(x, 1280, 1, 1, 0, RELU6);
    x = b.global_avgpool(x);
    x = b.dense(x, 1000);
    return b.finish(x);
}

// ---------------------------------------------------------------- Inception-v3 (299 x 299)
View conv_rs(GraphBuilder& b, View x, int K, int R, int S, int ph, int pw, const View* dst = nullptr, int stride = 1) {
    GraphBuilder::ConvOpt o;
    o.pad_h = ph;
    o.pad_w = pw;
    o.stride_h = o.stride_w = stride;
    return b.conv(x, K, R, S, o, nullptr, dst);
}

View inception_a(GraphBuilder& b, View x, int pool_features) {
    View out = b.buffer(64 + 64 + 96 + pool_features, x.H, x.W);
    View d0 = GraphBuilder::slice(out, 0, 64), d1 = GraphBuilder::slice(out, 64, 64), d2 = GraphBuilder::slice(out, 128, 96),
         d3 = GraphBuilder::slice(out, 224, pool_features);
    b.conv(x, 64, 1, 1, 0, RELU, nullptr, &d0);
    View y = b.conv(x, 48, 1, 1, 0);
    b.conv(y, 64, 5, 1, 2, RELU, nullptr, &d1);
    y = b.conv(x, 64, 1, 1, 0);
    y = b.conv(y, 96, 3, 1, 1);
    b.conv(y, 96, 3, 1, 1, RELU, nullptr, &d2);
    y = b.pool(x, true, 3, 1, 1);
    b.conv(y, pool_features, 1, 1, 0, RELU, nullptr, &d3);
    return out;
}

View inception_b(GraphBuilder& b, View x) {
    const int H = (x.H - 3) / 2 + 1, W = (x.W - 3) / 2 + 1;
    View out = b.buffer(384 + 96 + x.C, H, W);
    View d0 = GraphBuilder::slice(out, 0, 384), d1 = GraphBuilder::slice(out, 384, 96), d2 = GraphBuilder::slice(out, 480, x.C);
    b.conv(x, 384, 3, 2, 0, RELU, nullptr, &d0);
    View y = b.conv(x, 64, 1, 1, 0);
    y = b.conv(y, 96, 3, 1, 1);
    b.conv(y, 96, 3, 2, 0, RELU, nullptr, &d1);
    b.pool(x, false, 3, 2, 0, false, true, &d2);
    return out;
}

View inception_c(GraphBuilder& b, View x, int c7) {
    View out = b.buffer(768, x.H, x.W);
    View d0 = GraphBuilder::slice(out, 0, 192), d1 = GraphBuilder::slice(out, 192, 192), d2 = GraphBuilder::slice(out, 384, 192),
         d3 = GraphBuilder::slice(out, 576, 192);
    b.conv(x, 192, 1, 1, 0, RELU, nullptr, &d0);
    View y = b.conv(x, c7, 1, 1, 0);
    y = conv_rs(b, y, c7, 1, 7, 0, 3);
    conv_rs(b, y, 192, 7, 1, 3, 0, &d1);
    y = b.conv(x, c7, 1, 1, 0);
    y = conv_rs(b, y, c7, 7, 1, 3, 0);
    y = conv_rs(b, y, c7, 1, 7, 0, 3);
    y = conv_rs(b, y, c7, 7, 1, 3, 0);
    conv_rs(b, y, 192, 1, 7, 0, 3, &d2);
    y = b.pool(x, true, 3, 1, 1);
    b.conv(y, 192, 1, 1, 0, RELU, nullptr, &d3);
    return out;
}

View inception_d(GraphBuilder& b, View x) {
    const int H = (x.H - 3) / 2 + 1, W = (x.W - 3) / 2 + 1;
    View out = b.buffer(320 + 192 + x.C, H, W);
    View d0 = GraphBuilder::slice(out, 0, 320), d1 = GraphBuilder::slice(out, 320, 192), d2 = GraphBuilder::slice(out, 512, x.C);
    View y = b.conv(x, 192, 1, 1, 0);
    b.conv(y, 320, 3, 2, 0, RELU, nullptr, &d0);
    y = b.conv(x, 192, 1, 1, 0);
    y = conv_rs(b, y, 192, 1, 7, 0, 3);
    y = conv_rs(b, y, 192, 7, 1, 3, 0);
    b.conv(y, 192, 3, 2, 0, RELU, nullptr, &d1);
    b.pool(x, false, 3, 2, 0, false, true, &d2);
    return out;
}

View inception_e(GraphBuilder& b, View x) {
    View out = b.buffer(2048, x.H, x.W);
    View d0 = GraphBuilder::slice(out, 0, 320), d1a = GraphBuilder::slice(out, 320, 384), d1b = GraphBuilder::slice(out, 704, 384),
         d2a = GraphBuilder::slice(out, 1088, 384), d2b = GraphBuilder::slice(out, 1472, 384), d3 = GraphBuilder::slice(out, 1856, 192);
    b.conv(x, 320, 1, 1, 0, RELU, nullptr, &d0);
    View y = b.conv(x, 384, 1, 1, 0);
    conv_rs(b, y, 384, 1, 3, 0, 1, &d1a);
    conv_rs(b, y, 384, 3, 1, 1, 0, &d1b);
    y = b.conv(x, 448, 1, 1, 0);
    y = b.conv(y, 384, 3, 1, 1);
    conv_rs(b, y, 384, 1, 3, 0, 1, &d2a);
    conv_rs(b, y, 384, 3, 1, 1, 0, &d2b);
    y = b.pool(x, true, 3, 1, 1);
    b.conv(y, 192, 1, 1, 0, RELU, nullptr, &d3);
    return out;
}

Graph inception_v3() {
    GraphBuilder b("inception_v3");
    View x = b.input(3, 299, 299);
    x = b.conv(x, 32, 3, 2, 0);
    x = b.conv(x, 32, 3, 1, 0);
    x = b.conv(x, 64, 3, 1, 1);
    x = b.pool(x, false, 3, 2, 0);
    x = b.conv(x, 80, 1, 1, 0);
    x = b.conv(x, 192, 3, 1, 0);
    x = b.pool(x, false, 3, 2, 0);
    x = inception_a(b, x, 32);
    x = inception_a(b, x, 64);
    x = inception_a(b, x, 64);
    x = inception_b(b, x);
    x = inception_c(b, x, 128);
    x = inception_c(b, x, 160);
    x = inception_c(b, x, 160);
    x = inception_c(b, x, 192);
    x = inception_d(b, x);
    x = inception_e(b, x);
    x = inception_e(b, x);
    x = b.global_avgpool(x);
    x = b.dense(x, 1000);
    return b.finish(x);
}

// ---------------------------------------------------------------- SqueezeNet 1.1
View fire(GraphBuilder& b, View x, int squeeze, int e1, int e3) {
    View s = b.conv(x, squeeze, 1, 1, 0);
    View out = b.buffer(e1 + e3, x.H, x.W);
    View d0 = GraphBuilder::slice(out, 0, e1), d1 = GraphBuilder::slice(out, e1, e3);
    b.conv(s, e1, 1, 1, 0, RELU, nullptr, &d0);
    b.conv(s, e3, 3, 1, 1, RELU, nullptr, &d1);
    return out;
}

Graph squeezenet1_1() {
    GraphBuilder b("squeezenet1_1");
    View x = b.input(3, 224, 224);
    x = b.conv(x, 64, 3, 2, 0);
    x = b.pool(x, false, 3, 2, 0, true);
    x = fire(b, x, 16, 64, 64);
    x = fire(b, x, 16, 64, 64);
    x = b.pool(x, false, 3, 2, 0, true);
    x = fire(b, x, 32, 128, 128);
    x = fire(b, x, 32, 128, 128);
    x = b.pool(x, false, 3, 2, 0, true);
    x = fire(b, x, 48, 192, 192);
    x = fire(b, x, 48, 192, 192);
    x = fire(b, x, 64, 256, 256);
    x = fire(b, x, 64, 256, 256);
    x = b.conv(x, 1000, 1, 1, 0);
    x = b.global_avgpool(x);
    return b.finish(x);
}

// ---------------------------------------------------------------- GoogLeNet (with LRN, softmax output)
View goog_inception(GraphBuilder& b, View x, int c1, int c3r, int c3, int c5r, int c5, int cp) {
    View out = b.buffer(c1 + c3 + c5 + cp, x.H, x.W);
    View d0 = GraphBuilder::slice(out, 0, c1), d1 = GraphBuilder::slice(out, c1, c3), d2 = GraphBuilder::slice(out, c1 + c3, c5),
         d3 = GraphBuilder::slice(out, c1 + c3 + c5, cp);
    b.conv(x, c1, 1, 1, 0, RELU, nullptr, &d0);
    View y = b.conv(x, c3r, 1, 1, 0);
    b.conv(y, c3, 3, 1, 1, RELU, nullptr, &d1);
    y = b.conv(x, c5r, 1, 1, 0);
    b.conv(y, c5, 5, 1, 2, RELU, nullptr, &d2);
    y = b.pool(x, false, 3, 1, 1);
    b.conv(y, cp, 1, 1, 0, RELU, nullptr, &d3);
    return out;
}

Graph googlenet() {
    GraphBuilder b("googlenet");
    View x = b.input(3, 224, 224);
    x = b.conv(x, 64, 7, 2, 3);
    x = b.pool(x, false, 3, 2, 0, true);
    x = b.lrn(x, 5, 1e-4f, 0.75f, 1.f);
    x = b.conv(x, 64, 1, 1, 0);
    x = b.conv(x, 192, 3, 1, 1);
    x = b.lrn(x, 5, 1e-4f, 0.75f, 1.f);
    x = b.pool(x, false, 3, 2, 0, true);
    x = goog_inception(b, x, 64, 96, 128, 16, 32, 32);
    x = goog_inception(b, x, 128, 128, 192, 32, 96, 64);
    x = b.pool(x, false, 3, 2, 0, true);
    x = goog_inception(b, x, 192, 96, 208, 16, 48, 64);
    x = goog_inception(b, x, 160, 112, 224, 24, 64, 64);
    x = goog_inception(b, x, 128, 128, 256, 24, 64, 64);
    x = goog_inception(b, x, 112, 144, 288, 32, 64, 64);
    x = goog_inception(b, x, 256, 160, 320, 32, 128, 128);
    x = b.pool(x, false, 3, 2, 0, true);
    x = goog_inception(b, x, 256, 160, 320, 32, 128, 128);
    x = goog_inception(b, x, 384, 192, 384, 48, 128, 128);
    x = b.global_avgpool(x);
    x = b.dense(x, 1000);
    x = b.softmax(x, 1, 1000);
    return b.finish(x);
}

// ---------------------------------------------------------------- DenseNet-121
Graph densenet121() {
    GraphBuilder b("densenet121");
    const int growth = 32, bn_size = 4;
    const int blocks[4] = {6, 12, 24, 16};
    View x = b.input(3, 224, 224);
    x = b.conv(x, 64, 7, 2, 3);
    int c = 64;
    View block = b.buffer(c + blocks[0] * growth, 56, 56);
    View head = GraphBuilder::slice(block, 0, c);
    b.pool(x, false, 3, 2, 1, false, true, &head);
    for (int s = 0; s < 4; ++s) {
        for (int i = 0; i < blocks[s]; ++i) {
            View in = GraphBuilder::slice(block, 0, c);                // everything produced so far in this block
            View y = b.scale_shift(in, RELU);                          // pre-activation norm over the concatenation
            y = b.conv(y, bn_size * growth, 1, 1, 0, RELU);
            View dst = GraphBuilder::slice(block, c, growth);
            b.conv(y, growth, 3, 1, 1, NONE, nullptr, &dst);
            c += growth;
        }
        if (s < 3) {
            View y = b.scale_shift(block, RELU);
            y = b.conv(y, c / 2, 1, 1, 0, NONE);
            c /= 2;
            View next = b.buffer(c + blocks[s + 1] * growth, block.H / 2, block.W / 2);
            View nhead = GraphBuilder::slice(next, 0, c);
            b.pool(y, true, 2, 2, 0, false, true, &nhead);
            block = next;
        }
    }
    x = b.scale_shift(block, RELU);
    x = b.global_avgpool(x);
    x = b.dense(x, 1000);
    return b.finish(x);
}

// ---------------------------------------------------------------- 320x240 face detector (depthwise-separable, scores head)
View conv_dw(GraphBuilder& b, View x, int out, int stride) {
    View y = b.dwconv(x, 3, stride, 1, RELU);
    return b.conv(y, out, 1, 1, 0, RELU);
}

Graph ultraface320() {
    GraphBuilder b("ultraface320");
    View x = b.input(3, 240, 320);
    x = b.conv(x, 16, 3, 2, 1);
    x = conv_dw(b, x, 32, 1);
    x = conv_dw(b, x, 32, 2);
    x = conv_dw(b, x, 32, 1);
    x = conv_dw(b, x, 64, 2);
    x = conv_dw(b, x, 64, 1);
    x = conv_dw(b, x, 64, 1);
    x = conv_dw(b, x, 64, 1);
    View f0 = x;  // 64 x 30 x 40
    x = conv_dw(b, x, 128, 2);
    x = conv_dw(b, x, 128, 1);
    x = conv_dw(b, x, 128, 1);
    View f1 = x;  // 128 x 15 x 20
    x = conv_dw(b, x, 256, 2);
    x = conv_dw(b, x, 256, 1);
    View f2 = x;  // 256 x 8 x 10
    x = b.conv(x, 64, 1, 1, 0);
    x = b.dwconv(x, 3, 2, 1, RELU);
    x = b.conv(x, 256, 1, 1, 0);
    View f3 = x;  // 256 x 4 x 5

    // Per feature map a separable conv produces anchors*2 logits per pixel, stored [anchors*2][H][W] one map
    // after the other in one flat buffer of 4420*2 floats.  The synthetic model DEFINES prior r as the pair of
    // consecutive floats (2r, 2r+1) of that buffer and applies the two-class softmax to each pair.
    const View feats[4] = {f0, f1, f2, f3};
    const int anchors[4] = {3, 2, 2, 3};
    int total = 0;
    for (int i = 0; i < 4; ++i) total += feats[i].H * feats[i].W * anchors[i];
    View logits = b.buffer(total * 2, 1, 1);
    int off = 0;
    for (int i = 0; i < 4; ++i) {
        View y = b.dwconv(feats[i], 3, 1, 1, RELU);
        const int n = feats[i].H * feats[i].W * anchors[i] * 2;
        View dst = GraphBuilder::slice(logits, off, n);
        View dst4 = dst;  // same bytes seen as [anchors*2][H][W]
        dst4.C = anchors[i] * 2;
        dst4.H = feats[i].H;
        dst4.W = feats[i].W;
        b.conv(y, anchors[i] * 2, 1, 1, 0, NONE, nullptr, &dst4);
        off += n;
    }
    View scores = b.softmax(logits, total, 2);
    return b.finish(scores);
}

// ---------------------------------------------------------------- ResNet-100 face embedding (IR units, PReLU)
Graph arcfaceresnet100() {
    GraphBuilder b("arcfaceresnet100");
    View x = b.input(3, 112, 112);
    x = b.conv(x, 64, 3, 1, 1, PRELU);
    const int units[4] = {3, 13, 30, 3};
    const int planes[4] = {64, 128, 256, 512};
    for (int s = 0; s < 4; ++s)
        for (int i = 0; i < units[s]; ++i) {
            const int stride = i == 0 ? 2 : 1;
            View shortcut = x;
            if (i == 0) shortcut = b.conv(x, planes[s], 1, stride, 0, NONE);
            View y = b.scale_shift(x, NONE);  // norm in front of a zero-padded conv cannot be folded
            y = b.conv(y, planes[s], 3, 1, 1, PRELU);
            x = b.conv(y, planes[s], 3, stride, 1, NONE, &shortcut, nullptr, kResGain);
        }
    x = b.scale_shift(x, NONE);
    // 49 residual units on seeded weights leave activations in the hundreds; the embedding layer brings the output back to
    // the order of one (the trained network ends in a normalisation that does the same)
    x = b.dense(GraphBuilder::reshape(x, 512 * 7 * 7, 1, 1), 512, NONE, 0.01);
    return b.finish(x);
}

const std::map<std::string, std::function<Graph()>>& zoo() {
    static const std::map<std::string, std::function<Graph()>> z = {
        {"mnist", mnist},
        {"resnet18", [] { return resnet("resnet18", false, {2, 2, 2, 2}); }},
        {"resnet34", [] { return resnet("resnet34", false, {3, 4, 6, 3}); }},
        {"resnet50", [] { return resnet("resnet50", true, {3, 4, 6, 3}); }},
        {"mobilenetv2", mobilenetv2},
        {"inception_v3", inception_v3},
        {"squeezenet1_1", squeezenet1_1},
        {"googlenet", googlenet},
        {"densenet121", densenet121},
        {"ultraface320", ultraface320},
        {"arcfaceresnet100", arcfaceresnet100},
    };
    return z;
}

}  // namespace

bool build_model(const std::string& name, Graph* out) {
    auto it = zoo().find(name);
    if (it == zoo().end()) return false;
    *out = it->second();
    return true;
}

const char* model_names() {
    static const std::string names = [] {
        std::string s;
        for (const auto& kv : zoo()) s += (s.empty() ? "" : ",") + kv.first;
        return s;
    }();
    return names.c_str();
}

}  // namespace paella
