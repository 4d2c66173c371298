// Graph executor behind include/paella_models.h: builds a model once per process (seeded weights, packed
// and uploaded), and issues it one operator per call so a scheduler can interleave requests.

#include "graph.h"

#include "paella_hip.h"
#include "paella_models.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <utility>
#include <vector>

using namespace paella;

struct StagePlan {
    const Node* node = nullptr;
    paella_conv_plan conv{};
    paella_launch_dims dims{};
    const char* op = "";
    double flops = 0, bytes = 0;
    // device pointers into the weight arena
    const void* w = nullptr;
    const float* bias = nullptr;
    const float* slope = nullptr;
    const float* scale = nullptr;
    const float* shift = nullptr;
};

// One launch: an operator, or up to PAELLA_CONV_GROUP_MAX convs that do not depend on each other sharing a grid.
struct Launch {
    int nodes[PAELLA_CONV_GROUP_MAX] = {-1, -1, -1, -1};  // node indices, in launch order
    int count = 0;
    int pre = -1;  // count == 1: the scale-shift node whose work the conv nodes[0] does on its input, if any
    int pool = -1;  // a pooling node that shares the launch with the convs (at most three then), or -1
    paella_launch_dims dims{};
};

struct paella_model {
    Graph g;
    // Split-reduction scratch of a request (stages of one request never overlap).  Every conv expects arrival
    // counters that read zero at the head of its workspace and partial tiles behind them, so the second to fourth
    // convs of a group get areas of their own: no conv's partial tiles land on another's counters.
    size_t workspace_bytes = 0;
    size_t ws_area[PAELLA_CONV_GROUP_MAX] = {0, 0, 0, 0};  // byte offset of the area of the k-th conv of a launch
    uint64_t seed = 0;
    bool pairing = true;
    char* weights_dev = nullptr;
    std::vector<StagePlan> plans;   // one per node
    std::vector<int> absorbed_by;   // per node: the conv that applies this scale-shift node to its own input, or -1
    std::vector<int> pre_of;        // per node: the scale-shift node this conv applies to its input, or -1
    std::vector<Launch> stages;     // in execution order
};

struct paella_exec {
    const paella_model* m = nullptr;
    float* arena = nullptr;
    void* workspace = nullptr;
    float* in_bound = nullptr;   // caller's memory standing for the input / output buffer (paella_exec_bind_*)
    float* out_bound = nullptr;
    float* ptr(const View& v) const {
        if (v.buf < 0) return nullptr;
        if (in_bound && v.buf == m->g.input.buf) return in_bound + v.off;
        if (out_bound && v.buf == m->g.output.buf) return out_bound + v.off;
        return arena + m->g.buffers[v.buf].offset + v.off;
    }
};

namespace {

std::mutex g_mtx;
std::map<std::pair<std::string, uint64_t>, std::unique_ptr<paella_model>> g_models;  // name + '|' + pairing -> model

// Whether models built now put two independent convs into one launch (the environment is read at every build, so
// a process can hold both forms of a model).
bool pairing_enabled() {
    const char* env = std::getenv("PAELLA_CONV_PAIRS");
    return !(env && env[0] == '0');
}
std::map<std::string, std::unique_ptr<Graph>> g_graphs;

const Graph* graph_of(const char* name) {
    if (!name) return nullptr;
    std::lock_guard<std::mutex> lk(g_mtx);
    auto it = g_graphs.find(name);
    if (it != g_graphs.end()) return it->second.get();
    auto g = std::make_unique<Graph>();
    try {
        if (std::strncmp(name, "onnx:", 5) == 0) *g = import_onnx(name + 5, name);
        else if (!build_model(name, g.get())) return nullptr;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "paella_models: %s: %s\n", name, e.what());
        return nullptr;
    }
    return (g_graphs[name] = std::move(g)).get();
}

size_t align256(size_t v) { return (v + 255) / 256 * 256; }

unsigned vgprs_or(const char* family, unsigned fallback) {
    unsigned v = 0;
    return paella_kernel_vgprs(family, &v) == 0 && v > 0 ? v : fallback;
}

int log2_ceil(int v) {
    int b = 0;
    while ((1 << b) < v) ++b;
    return b;
}

// Lays the nodes out as launches.  MFMA convs on the smallest tile go out together, up to four in one launch, when
// none reads or overwrites what another writes and the device is not full yet (PAELLA_CONV_PAIRS=0 switches this
// off, and the launches are the nodes in graph order).  Partners need not be neighbours in the graph's node list: the
// nodes are re-issued in an order that keeps every read-after-write, write-after-read and write-after-write pair of
// the list -- on the arena addresses, so that buffers sharing memory count -- and stays as close to the list as that
// allows.  Convs with fewer waves per workgroup are re-planned to the largest count of their group; their packed
// weights do not depend on that.
// A per-channel scale-shift stage (batch-norm, with or without ReLU) that feeds nothing but convs able to apply it
// to their own input is not launched: each of those convs reads the stage's input and transforms it while fetching
// operands (paella_conv2d_launch_transformed).  Conditions, on arena addresses so that buffers sharing memory count:
// every reader of the stage's output, up to the node that overwrites it, is such a conv and reads exactly that view;
// the output is not the model's; and nothing between the stage and its last reader overwrites the stage's input.
void absorb_scale_shifts(paella_model* m) {
    const Graph& g = m->g;
    const int n = (int)g.nodes.size();
    m->absorbed_by.assign(n, -1);
    m->pre_of.assign(n, -1);
    if (!m->pairing) return;
    auto overlap = [&](const View& a, const View& b) {
        if (a.buf < 0 || b.buf < 0) return false;
        const size_t a0 = g.buffers[a.buf].offset + a.off, b0 = g.buffers[b.buf].offset + b.off;
        return a0 < b0 + b.numel() && b0 < a0 + a.numel();
    };
    for (int e = 0; e < n; ++e) {
        const Node& el = g.nodes[e];
        if (el.op != Op::Eltwise || el.x2.buf >= 0 || el.scale < 0 || el.shift < 0 || el.slope >= 0) continue;
        if (el.act != PAELLA_ACT_NONE && el.act != PAELLA_ACT_RELU) continue;
        if (overlap(el.y, g.output) || overlap(el.y, el.x)) continue;
        std::vector<int> readers;
        bool ok = true;
        for (int j = e + 1; j < n && ok; ++j) {
            const Node& c = g.nodes[j];
            if (overlap(c.x, el.y) || overlap(c.x2, el.y)) {
                const bool same_view = c.x.buf == el.y.buf && c.x.off == el.y.off && c.x.C == el.y.C && c.x.H == el.y.H && c.x.W == el.y.W;
                ok = c.op == Op::Conv && same_view && !overlap(c.x2, el.y) && m->pre_of[j] < 0 &&
                     paella_conv2d_plan_takes_input_transform(&m->plans[j].conv) == 1;
                if (ok) readers.push_back(j);
            }
            if (overlap(c.y, el.y)) break;  // the output's memory starts a new life here
        }
        if (!ok || readers.empty()) continue;
        for (int k = e + 1; k < readers.back() && ok; ++k)
            if (overlap(g.nodes[k].y, el.x)) ok = false;
        if (!ok) continue;
        m->absorbed_by[e] = readers.front();
        for (int j : readers) m->pre_of[j] = e;
    }
}

void pair_up(paella_model* m) {
    const Graph& g = m->g;
    const int n = (int)g.nodes.size();
    auto overlap = [&](const View& a, const View& b) {
        if (a.buf < 0 || b.buf < 0) return false;
        const size_t a0 = g.buffers[a.buf].offset + a.off, b0 = g.buffers[b.buf].offset + b.off;
        return a0 < b0 + b.numel() && b0 < a0 + a.numel();
    };
    // What a node reads and writes once absorbed scale-shift stages are gone: the stage itself nothing, the conv
    // that does its work the stage's input.
    const View none;
    auto in1 = [&](int i) -> const View& { return m->absorbed_by[i] >= 0 ? none : m->pre_of[i] >= 0 ? g.nodes[m->pre_of[i]].x : g.nodes[i].x; };
    auto in2 = [&](int i) -> const View& { return m->absorbed_by[i] >= 0 ? none : g.nodes[i].x2; };
    auto out = [&](int i) -> const View& { return m->absorbed_by[i] >= 0 ? none : g.nodes[i].y; };
    auto ordered = [&](int a, int b) {  // b must stay behind a
        return overlap(out(a), in1(b)) || overlap(out(a), in2(b)) || overlap(out(a), out(b)) || overlap(out(b), in1(a)) || overlap(out(b), in2(a));
    };
    auto pairable = [&](int i) {
        const StagePlan& st = m->plans[i];
        return st.node->op == Op::Conv && st.conv.kind == 0 && st.conv.mi == 1 && st.conv.ni == 1 && m->pre_of[i] < 0;
    };
    // The plan of node i with kw waves per workgroup; false if that is not possible.
    auto with_waves = [&](int i, int kw, StagePlan* out) {
        *out = m->plans[i];
        if (out->conv.kw == kw) return true;
        const size_t blob = out->conv.blob_bytes;
        const int hint = log2_ceil(out->conv.splits) << 12 | 1 << 8 | 1 << 4 | log2_ceil(kw);
        if (paella_conv2d_plan(&out->node->conv, out->node->x2.buf >= 0, hint, &out->conv) != 0 || out->conv.blob_bytes != blob) return false;
        out->dims = out->conv.dims;
        return true;
    };

    std::vector<std::vector<int>> later(n);
    std::vector<int> waits_for(n, 0);
    for (int i = 0; i < n; ++i)
        for (int j = i + 1; j < n; ++j)
            if (m->pairing ? ordered(i, j) : j == i + 1) {
                later[i].push_back(j);
                ++waits_for[j];
            }
    std::set<int> ready;  // no two ready nodes are ordered with respect to each other
    for (int i = 0; i < n; ++i)
        if (waits_for[i] == 0 && m->absorbed_by[i] < 0) ready.insert(i);  // an absorbed stage goes out with its first reader

    m->stages.clear();
    size_t area[PAELLA_CONV_GROUP_MAX] = {0, 0, 0, 0};
    while (!ready.empty()) {
        Launch l;
        l.nodes[0] = *ready.begin();
        l.count = 1;
        if (m->pairing && pairable(l.nodes[0])) {
            // Candidates: ready convs of the same reduction order, taken while the launch leaves CUs idle or the newcomer is small.
            unsigned grid = m->plans[l.nodes[0]].dims.grid;
            int kw = m->plans[l.nodes[0]].conv.kw;
            for (int j : ready) {
                if (l.count == PAELLA_CONV_GROUP_MAX) break;
                if (j == l.nodes[0] || !pairable(j) || m->plans[j].conv.k_order != m->plans[l.nodes[0]].conv.k_order) continue;
                const unsigned gj = m->plans[j].dims.grid;
                if ((grid > 256 && gj > 256) || grid + gj > 1024) continue;
                l.nodes[l.count++] = j;
                grid += gj;
                if (m->plans[j].conv.kw > kw) kw = m->plans[j].conv.kw;
            }
            if (l.count > 1) {
                StagePlan re[PAELLA_CONV_GROUP_MAX];
                const paella_conv_plan* plans[PAELLA_CONV_GROUP_MAX];
                int kept = 0;
                for (int k = 0; k < l.count; ++k)
                    if (with_waves(l.nodes[k], kw, &re[kept])) {
                        l.nodes[kept] = l.nodes[k];
                        plans[kept] = &re[kept].conv;
                        ++kept;
                    } else if (k == 0) {
                        kept = 0;
                        break;
                    }
                if (kept > 1 && paella_conv2d_group_dims(plans, kept, &l.dims) == 0) {
                    for (int k = 0; k < kept; ++k) m->plans[l.nodes[k]] = re[k];
                    l.count = kept;
                } else {
                    l.nodes[0] = *ready.begin();
                    l.count = 1;
                }
                for (int k = l.count; k < PAELLA_CONV_GROUP_MAX; ++k) l.nodes[k] = -1;
            }
            // A ready pooling operator rides along with up to three tap-major convs (an inception module's 3x3 pool beside
            // its 1x1 convs): on its own it is a launch shorter than the cost of launching it.
            if (l.count <= 3 && m->plans[l.nodes[0]].conv.k_order == 1) {
                const paella_conv_plan* plans[PAELLA_CONV_GROUP_MAX];
                for (int k = 0; k < l.count; ++k) plans[k] = &m->plans[l.nodes[k]].conv;
                for (int j : ready) {
                    if (g.nodes[j].op != Op::Pool) continue;
                    paella_launch_dims with_pool;
                    if (paella_conv2d_group_pool_dims(plans, l.count, &g.nodes[j].pool, &with_pool) == 0 && with_pool.grid <= 2048) {
                        l.pool = j;
                        l.dims = with_pool;
                    }
                    break;
                }
            }
            if (l.count == 1 && l.pool < 0)  // an operator that is no such conv goes first if one is ready: it may release a partner
                for (int j : ready)
                    if (!pairable(j)) {
                        l.nodes[0] = j;
                        break;
                    }
        }
        if (l.count == 1) {
            if (l.pool < 0) l.dims = m->plans[l.nodes[0]].dims;
            const int pre = m->pre_of[l.nodes[0]];
            if (pre >= 0 && m->absorbed_by[pre] == l.nodes[0]) l.pre = pre;
            if (pre >= 0) (void)paella_conv2d_transformed_dims(&m->plans[l.nodes[0]].conv, &l.dims);  // the kernel that applies it uses more registers
        } else {
            // the convs whose workgroups run longer go first: the short ones fill in behind them
            std::stable_sort(l.nodes, l.nodes + l.count, [&](int a, int b) {
                return m->plans[a].flops / m->plans[a].dims.grid > m->plans[b].flops / m->plans[b].dims.grid;
            });
        }
        for (int k = 0; k < l.count; ++k) {
            const int done = l.nodes[k];
            ready.erase(done);
            for (int j : later[done])
                if (--waits_for[j] == 0) ready.insert(j);
            if (g.nodes[done].op == Op::Conv && m->plans[done].conv.workspace_bytes > area[k]) area[k] = m->plans[done].conv.workspace_bytes;
        }
        if (l.pool >= 0) {
            ready.erase(l.pool);
            for (int j : later[l.pool])
                if (--waits_for[j] == 0) ready.insert(j);
        }
        m->stages.push_back(l);
    }
    m->workspace_bytes = 0;
    for (int k = 0; k < PAELLA_CONV_GROUP_MAX; ++k) {
        m->ws_area[k] = m->workspace_bytes;
        m->workspace_bytes += align256(area[k]);
    }
}

// Plans every node and lays out the weight arena (host arithmetic only).
int plan_nodes(paella_model* m, std::vector<size_t>& tensor_off, std::vector<size_t>& blob_off, size_t& total) {
    const Graph& g = m->g;
    tensor_off.assign(g.weights.size(), (size_t)-1);
    blob_off.assign(g.nodes.size(), (size_t)-1);
    total = 0;
    m->plans.resize(g.nodes.size());
    for (size_t i = 0; i < g.nodes.size(); ++i) {
        const Node& n = g.nodes[i];
        StagePlan& st = m->plans[i];
        st.node = &n;
        int rc = 0;
        switch (n.op) {
            case Op::Conv:
                rc = paella_conv2d_plan(&n.conv, n.x2.buf >= 0, 0, &st.conv);
                if (rc) return rc;
                st.dims = st.conv.dims;
                st.op = st.conv.kind == 0 ? "conv" : "dwconv";
                st.flops = st.conv.flops;
                st.bytes = st.conv.bytes;
                paella_conv2d_dims(&st.conv, &st.dims);  // registers and static LDS of the kernel this plan launches
                blob_off[i] = total;
                total += align256(st.conv.blob_bytes);
                break;
            case Op::Dense:
                rc = paella_dense_dims(n.dense_in, n.dense_out, &st.dims);
                st.op = "dense";
                st.flops = 2.0 * n.dense_in * n.dense_out;
                st.bytes = 4.0 * ((double)n.dense_in * n.dense_out + n.dense_in + 2.0 * n.dense_out);
                st.dims.vgprs = vgprs_or("dense", st.dims.vgprs);
                break;
            case Op::Pool:
                rc = paella_pool2d_dims(&n.pool, &st.dims);
                st.op = "pool";
                st.bytes = 4.0 * (n.x.numel() + n.y.numel());
                st.dims.vgprs = vgprs_or("pool", st.dims.vgprs);
                break;
            case Op::GlobalAvgPool:
                rc = paella_global_avgpool_dims(n.x.C, n.x.H * n.x.W, &st.dims);
                st.op = "gap";
                st.bytes = 4.0 * (n.x.numel() + n.y.numel());
                st.dims.vgprs = vgprs_or("gap", st.dims.vgprs);
                break;
            case Op::Eltwise:
                rc = paella_eltwise_dims(n.x.C, n.x.H * n.x.W, &st.dims);
                st.op = "eltwise";
                st.bytes = 4.0 * (n.x.numel() * (n.x2.buf >= 0 ? 2 : 1) + n.y.numel());
                st.dims.vgprs = vgprs_or("eltwise", st.dims.vgprs);
                break;
            case Op::Softmax:
                rc = paella_softmax_dims(n.rows, n.cols, &st.dims);
                st.op = "softmax";
                st.bytes = 4.0 * (n.x.numel() + n.y.numel());
                st.dims.vgprs = vgprs_or("softmax", st.dims.vgprs);
                break;
            case Op::Lrn:
                rc = paella_lrn_dims(n.x.C, n.x.H * n.x.W, &st.dims);
                st.op = "lrn";
                st.bytes = 4.0 * (n.x.numel() + n.y.numel());
                st.dims.vgprs = vgprs_or("lrn", st.dims.vgprs);
                break;
        }
        if (rc) return rc;
        for (int id : {n.op == Op::Conv ? -1 : n.w, n.bias, n.slope, n.scale, n.shift}) {
            if (id >= 0 && tensor_off[id] == (size_t)-1) {
                tensor_off[id] = total;
                total += align256(g.weights[id].numel() * sizeof(float));
            }
        }
    }

    return 0;
}

int build(paella_model* m) {
    const Graph& g = m->g;
    std::vector<size_t> tensor_off, blob_off;
    size_t total = 0;
    if (int rc = plan_nodes(m, tensor_off, blob_off, total)) return rc;
    absorb_scale_shifts(m);
    pair_up(m);

    // Generate, pack, upload.
    std::vector<char> host(total, 0);
    std::vector<float> tmp;
    for (size_t t = 0; t < g.weights.size(); ++t) {
        if (tensor_off[t] == (size_t)-1) continue;
        fill_weight(g.weights[t], m->seed, t, reinterpret_cast<float*>(host.data() + tensor_off[t]));
    }
    for (size_t i = 0; i < g.nodes.size(); ++i) {
        const Node& n = g.nodes[i];
        if (n.op != Op::Conv) continue;
        tmp.resize(g.weights[n.w].numel());
        fill_weight(g.weights[n.w], m->seed, (uint64_t)n.w, tmp.data());
        int rc = paella_conv2d_pack(&m->plans[i].conv, tmp.data(), host.data() + blob_off[i]);
        if (rc) return rc;
    }
    void* dev = nullptr;
    int rc = llis_hip_device_malloc(&dev, total ? total : 256);
    if (rc) return rc;
    rc = llis_hip_memcpy(dev, host.data(), total, LLIS_HIP_H2D);
    if (rc) return rc;
    m->weights_dev = reinterpret_cast<char*>(dev);
    for (size_t i = 0; i < g.nodes.size(); ++i) {
        const Node& n = g.nodes[i];
        StagePlan& st = m->plans[i];
        auto at = [&](int id) -> const float* { return id >= 0 ? reinterpret_cast<const float*>(m->weights_dev + tensor_off[id]) : nullptr; };
        st.w = n.op == Op::Conv ? (const void*)(m->weights_dev + blob_off[i]) : (const void*)at(n.w);
        st.bias = at(n.bias);
        st.slope = at(n.slope);
        st.scale = at(n.scale);
        st.shift = at(n.shift);
    }
    return 0;
}

}  // namespace

extern "C" {

const char* paella_model_names(void) { return model_names(); }

int paella_model_io_bytes(const char* name, size_t* in_bytes, size_t* out_bytes) {
    const Graph* g = graph_of(name);
    if (!g) return PAELLA_EINVAL;
    if (in_bytes) *in_bytes = g->input.numel() * sizeof(float);
    if (out_bytes) *out_bytes = g->output.numel() * sizeof(float);
    return 0;
}

int paella_model_write_dim(const char* name, const char* path) {
    const Graph* g = graph_of(name);
    if (!g || !path) return PAELLA_EINVAL;
    FILE* fp = std::fopen(path, "w");
    if (!fp) return PAELLA_EINVAL;
    // input dims, -1, output dims, one number per line (the sidecar the reference keeps next to each compiled
    // model, reference sosp23_artifact/tvm_models_dim/*.dim); outputs without spatial extent are written as N x C
    std::fprintf(fp, "1\n%d\n%d\n%d\n-1\n1\n%d\n", g->input.C, g->input.H, g->input.W, g->output.C);
    if (g->output.H * g->output.W != 1) std::fprintf(fp, "%d\n%d\n", g->output.H, g->output.W);
    std::fclose(fp);
    return 0;
}

int paella_model_describe(const char* name, char* json, size_t cap, size_t* needed) {
    const Graph* g = graph_of(name);
    if (!g) return PAELLA_EINVAL;
    const std::string s = describe_json(*g);
    if (needed) *needed = s.size() + 1;
    if (json && cap) {
        const size_t n = s.size() < cap - 1 ? s.size() : cap - 1;
        std::memcpy(json, s.data(), n);
        json[n] = 0;
    }
    return 0;
}

int paella_model_totals(const char* name, double* macs, double* params, double* flops, double* bytes, int* stages) {
    const Graph* g = graph_of(name);
    if (!g) return PAELLA_EINVAL;
    if (macs) *macs = g->macs();
    if (params) *params = g->params();
    if (flops) *flops = 2.0 * g->macs();
    if (bytes) {
        double b = 4.0 * (g->input.numel() + g->output.numel()) + 4.0 * g->params();
        for (const Node& n : g->nodes) b += 4.0 * (n.x.numel() + n.y.numel() + (n.x2.buf >= 0 ? n.x2.numel() : 0));
        *bytes = b;
    }
    if (stages) *stages = (int)g->nodes.size();
    return 0;
}

int paella_model_launch_plan(const char* name, int* out, size_t capacity) {
    const Graph* g = graph_of(name);
    if (!g) return PAELLA_EINVAL;
    paella_model m;
    m.g = *g;
    m.pairing = pairing_enabled();
    std::vector<size_t> tensor_off, blob_off;
    size_t total = 0;
    if (int rc = plan_nodes(&m, tensor_off, blob_off, total)) return rc;
    absorb_scale_shifts(&m);
    pair_up(&m);
    size_t used = 0;
    for (const Launch& l : m.stages) {
        if (out && used < capacity) out[used] = l.count + (l.pre >= 0 ? 1 : 0) + (l.pool >= 0 ? 1 : 0);
        ++used;
        if (l.pre >= 0) {
            if (out && used < capacity) out[used] = l.pre;
            ++used;
        }
        for (int k = 0; k < l.count; ++k, ++used)
            if (out && used < capacity) out[used] = l.nodes[k];
        if (l.pool >= 0) {
            if (out && used < capacity) out[used] = l.pool;
            ++used;
        }
    }
    return (int)used;
}

int paella_model_weight_values(const char* name, uint64_t seed, int tensor, float* out, size_t count) {
    const Graph* g = graph_of(name);
    if (!g || tensor < 0 || (size_t)tensor >= g->weights.size() || !out || count != g->weights[tensor].numel()) return PAELLA_EINVAL;
    fill_weight(g->weights[tensor], seed, (uint64_t)tensor, out);
    return 0;
}

int paella_model_get(const char* name, uint64_t seed, paella_model** out) {
    const Graph* g = graph_of(name);
    if (!g || !out) return PAELLA_EINVAL;
    std::lock_guard<std::mutex> lk(g_mtx);
    const bool pairing = pairing_enabled();
    auto key = std::make_pair(std::string(name) + (pairing ? "|pairs" : "|single"), seed);
    auto it = g_models.find(key);
    if (it == g_models.end()) {
        auto m = std::make_unique<paella_model>();
        m->g = *g;
        m->seed = seed;
        m->pairing = pairing;
        if (int rc = build(m.get())) return rc;
        it = g_models.emplace(key, std::move(m)).first;
    }
    *out = it->second.get();
    return 0;
}

int paella_model_num_stages(const paella_model* m) { return m ? (int)m->stages.size() : PAELLA_EINVAL; }

int paella_model_stage_dims(const paella_model* m, int stage, paella_launch_dims* dims) {
    if (!m || !dims || stage < 0 || (size_t)stage >= m->stages.size()) return PAELLA_EINVAL;
    *dims = m->stages[stage].dims;
    return 0;
}

int paella_model_stage_work(const paella_model* m, int stage, const char** op, double* flops, double* bytes) {
    if (!m || stage < 0 || (size_t)stage >= m->stages.size()) return PAELLA_EINVAL;
    const Launch& l = m->stages[stage];
    if (op) *op = m->plans[l.nodes[0]].op;
    double f = 0, b = 0;
    for (int k = 0; k < l.count; ++k) {
        f += m->plans[l.nodes[k]].flops;
        b += m->plans[l.nodes[k]].bytes;
    }
    if (l.pool >= 0) b += m->plans[l.pool].bytes;
    if (flops) *flops = f;
    if (bytes) *bytes = b;
    return 0;
}

int paella_model_stage_nodes(const paella_model* m, int stage, int* nodes, int capacity) {
    if (!m || stage < 0 || (size_t)stage >= m->stages.size() || capacity < 0) return PAELLA_EINVAL;
    const Launch& l = m->stages[stage];
    int count = 0;
    if (l.pre >= 0) {
        if (nodes && count < capacity) nodes[count] = l.pre;
        ++count;
    }
    for (int k = 0; k < l.count; ++k, ++count)
        if (nodes && count < capacity) nodes[count] = l.nodes[k];
    if (l.pool >= 0) {
        if (nodes && count < capacity) nodes[count] = l.pool;
        ++count;
    }
    return count;
}

int paella_exec_create(const paella_model* m, paella_exec** out) {
    if (!m || !out) return PAELLA_EINVAL;
    void* dev = nullptr;
    if (int rc = llis_hip_device_malloc(&dev, m->g.arena_floats * sizeof(float))) return rc;
    paella_exec* e = new paella_exec();
    e->m = m;
    e->arena = reinterpret_cast<float*>(dev);
    if (m->workspace_bytes) {
        if (int rc = llis_hip_device_malloc(&e->workspace, m->workspace_bytes)) return rc;
        if (int rc = llis_hip_fill_u32_async(e->workspace, 0, m->workspace_bytes / 4, nullptr)) return rc;
        if (int rc = llis_hip_stream_synchronize(nullptr)) return rc;
    }
    *out = e;
    return 0;
}

int paella_exec_destroy(paella_exec* e) {
    if (!e) return PAELLA_EINVAL;
    llis_hip_device_free(e->arena);
    if (e->workspace) llis_hip_device_free(e->workspace);
    delete e;
    return 0;
}

int paella_exec_bind_input(paella_exec* e, void* p) {
    if (!e || ((uintptr_t)p & 15)) return PAELLA_EINVAL;
    const Graph& g = e->m->g;
    if (p) {
        if (g.input.off != 0) return PAELLA_ENOSUP;
        for (const Node& n : g.nodes)
            if (n.y.buf == g.input.buf) return PAELLA_ENOSUP;   // something writes into the input buffer (a concatenation re-based onto it)
    }
    e->in_bound = reinterpret_cast<float*>(p);
    return 0;
}

int paella_exec_bind_output(paella_exec* e, void* p) {
    if (!e || ((uintptr_t)p & 15)) return PAELLA_EINVAL;
    const Graph& g = e->m->g;
    if (p) {
        const Buffer& b = g.buffers[g.output.buf];
        if (g.output.off != 0 || g.output.numel() != (size_t)b.C * b.H * b.W || g.output.buf == g.input.buf) return PAELLA_ENOSUP;
        for (const Node& n : g.nodes)
            if (n.x.buf == g.output.buf || n.x2.buf == g.output.buf) return PAELLA_ENOSUP;   // a stage reads it back
    }
    e->out_bound = reinterpret_cast<float*>(p);
    return 0;
}

void* paella_exec_input(paella_exec* e) { return e ? e->ptr(e->m->g.input) : nullptr; }
void* paella_exec_output(paella_exec* e) { return e ? e->ptr(e->m->g.output) : nullptr; }

int paella_exec_launch_stage(paella_exec* e, int stage, void* stream, uint32_t job_id, void* notifier) {
    if (!e || stage < 0 || (size_t)stage >= e->m->stages.size()) return PAELLA_EINVAL;
    const Launch& l = e->m->stages[stage];
    if (l.count > 1 || l.pool >= 0) {
        paella_conv_operands members[PAELLA_CONV_GROUP_MAX];
        for (int k = 0; k < l.count; ++k) {
            const StagePlan& sk = e->m->plans[l.nodes[k]];
            const Node& nk = *sk.node;
            members[k] = paella_conv_operands{&sk.conv, e->ptr(nk.x), sk.w, sk.bias, e->ptr(nk.x2), sk.slope, e->ptr(nk.y),
                                              e->workspace ? static_cast<char*>(e->workspace) + e->m->ws_area[k] : nullptr};
        }
        if (l.pool >= 0) {
            const Node& pn = e->m->g.nodes[l.pool];
            return paella_conv2d_launch_group_pool(members, l.count, &pn.pool, e->ptr(pn.x), e->ptr(pn.y), stream, job_id, notifier);
        }
        return paella_conv2d_launch_group(members, l.count, stream, job_id, notifier);
    }
    const StagePlan& st = e->m->plans[l.nodes[0]];
    const Node& n = *st.node;
    const float* x = e->ptr(n.x);
    const float* x2 = e->ptr(n.x2);
    float* y = e->ptr(n.y);
    switch (n.op) {
        case Op::Conv:
            if (const int pre = e->m->pre_of[l.nodes[0]]; pre >= 0) {
                const StagePlan& sp = e->m->plans[pre];
                return paella_conv2d_launch_transformed(&st.conv, e->ptr(sp.node->x), sp.scale, sp.shift, sp.node->act, st.w, st.bias, x2,
                                                        st.slope, y, e->workspace, stream, job_id, notifier);
            }
            return paella_conv2d_launch(&st.conv, x, st.w, st.bias, x2, st.slope, y, e->workspace, stream, job_id, notifier);
        case Op::Dense:
            return paella_dense_launch(x, reinterpret_cast<const float*>(st.w), st.bias, y, n.dense_in, n.dense_out, n.act, stream, job_id, notifier);
        case Op::Pool:
            return paella_pool2d_launch(&n.pool, x, y, stream, job_id, notifier);
        case Op::GlobalAvgPool:
            return paella_global_avgpool_launch(x, y, n.x.C, n.x.H * n.x.W, stream, job_id, notifier);
        case Op::Eltwise:
            return paella_eltwise_launch(x, x2, st.scale, st.shift, st.slope, y, n.x.C, n.x.H * n.x.W, n.act, n.lo, n.hi, stream, job_id, notifier);
        case Op::Softmax:
            return paella_softmax_launch(x, y, n.rows, n.cols, stream, job_id, notifier);
        case Op::Lrn:
            return paella_lrn_launch(x, y, n.x.C, n.x.H * n.x.W, n.lrn_size, n.lrn_alpha, n.lrn_beta, n.lrn_k, stream, job_id, notifier);
    }
    return PAELLA_EINVAL;
}

int paella_exec_forward(paella_exec* e, void* stream) {
    if (!e) return PAELLA_EINVAL;
    for (size_t i = 0; i < e->m->stages.size(); ++i)
        if (int rc = paella_exec_launch_stage(e, (int)i, stream, 0, nullptr)) return rc;
    return 0;
}

}  // extern "C"
