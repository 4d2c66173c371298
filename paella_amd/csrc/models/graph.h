#pragma once
// Static inference graph: buffers, channel-slice views, seeded weight tensors and a list of operator nodes
// in execution (= scheduler stage) order.  Batch 1, fp32, NCHW.
//
// A view is a contiguous channel range of a buffer (for batch 1 a channel slice of an NCHW tensor is
// contiguous), which is how concatenation is expressed: producers write straight into their slice of the
// destination buffer and no copy kernel runs.

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "paella_ops.h"

namespace paella {

struct Buffer {
    int C, H, W;
    size_t offset = 0;  // float offset inside the activation arena
};

struct View {
    int buf = -1;
    size_t off = 0;  // float offset from the start of the buffer
    int C = 0, H = 0, W = 0;
    size_t numel() const { return (size_t)C * H * W; }
};

enum class Fill { Normal, Uniform, Constant, External };

struct WeightTensor {
    std::vector<int> shape;
    Fill fill = Fill::Normal;
    double a = 0, b = 0;  // Normal: std = a; Uniform: [a, b); Constant: a
    std::shared_ptr<std::vector<float>> data;  // External: the values themselves (imported models); the seed is ignored
    size_t numel() const {
        size_t n = 1;
        for (int d : shape) n *= (size_t)d;
        return n;
    }
};

enum class Op { Conv, Dense, Pool, GlobalAvgPool, Eltwise, Softmax, Lrn };

struct Node {
    Op op;
    View x, x2, y;             // x2: residual (Conv) or second addend (Eltwise); buf == -1 when absent
    paella_conv_desc conv{};   // Conv
    paella_pool_desc pool{};   // Pool
    int act = PAELLA_ACT_NONE;
    float lo = 0, hi = 0;
    int w = -1, bias = -1, slope = -1, scale = -1, shift = -1;  // weight tensor ids
    int dense_in = 0, dense_out = 0;
    int rows = 0, cols = 0;    // Softmax
    int lrn_size = 0;
    float lrn_alpha = 0, lrn_beta = 0, lrn_k = 0;
};

struct Graph {
    std::string name;
    std::vector<Buffer> buffers;
    std::vector<WeightTensor> weights;
    std::vector<Node> nodes;
    View input, output;
    size_t arena_floats = 0;

    double macs() const;
    double params() const;
};

// Fluent construction helper used by the zoo.
class GraphBuilder {
  public:
    explicit GraphBuilder(std::string name, double bias_std = 0.05) : bias_std_(bias_std) { g_.name = std::move(name); }

    View input(int C, int H, int W);
    View buffer(int C, int H, int W);
    static View slice(const View& v, int c_off, int C);

    struct ConvOpt {
        int stride_h = 1, stride_w = 1, pad_h = 0, pad_w = 0, dil = 1, groups = 1;
        int act = PAELLA_ACT_RELU;
        float lo = 0, hi = 0;
        double gain = 1.0;   // multiplies the He-normal std (stands for the folded batch-norm scale)
        bool bias = true;
    };
    // y = act(conv(x) + bias [+ residual]); dst (optional) is the slice to write into.
    View conv(const View& x, int K, int R, int S, const ConvOpt& o, const View* residual = nullptr, const View* dst = nullptr);
    // Shorthand: square kernel, symmetric stride/pad.
    View conv(const View& x, int K, int k, int stride, int pad, int act = PAELLA_ACT_RELU, const View* residual = nullptr,
              const View* dst = nullptr, double gain = 1.0);
    View dwconv(const View& x, int k, int stride, int pad, int act);
    View dense(const View& x, int O, int act = PAELLA_ACT_NONE, double std_scale = 1.0);
    View pool(const View& x, bool avg, int k, int stride, int pad, bool ceil_mode = false, bool count_include_pad = true, const View* dst = nullptr);
    View global_avgpool(const View& x);
    View add(const View& a, const View& b, int act);
    // Per-channel y = act(x * scale + shift): a batch-norm that cannot be folded into a neighbouring conv.
    View scale_shift(const View& x, int act, const View* dst = nullptr);
    View prelu(const View& x);
    View softmax(const View& x, int rows, int cols);
    View lrn(const View& x, int size, float alpha, float beta, float k);
    // Same bytes seen with another shape (flatten / reshape).
    static View reshape(const View& x, int C, int H, int W);

    Graph finish(const View& output);

  private:
    int add_weight(std::vector<int> shape, Fill fill, double a, double b = 0);
    View out_view(int C, int H, int W, const View* dst);

    Graph g_;
    double bias_std_;
};

// Reads an ONNX file into a graph with the file's own weights (throws std::runtime_error with the reason when the
// file uses something the operators do not cover).
Graph import_onnx(const std::string& path, const std::string& name);

// Zoo: returns false for an unknown name.
bool build_model(const std::string& name, Graph* out);
const char* model_names();

// Seeded generator (see include/paella_models.h).
void fill_weight(const WeightTensor& t, uint64_t seed, uint64_t stream, float* out);

std::string describe_json(const Graph& g);

}  // namespace paella
