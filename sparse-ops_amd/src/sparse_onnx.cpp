// SparseOnnxModel: graph loading.  Follows the semantics of the reference's loader
// (src/sparse_onnx.cpp:82-636) on top of the dependency-free protobuf reader, then
// places every weight and every activation buffer in HBM.
#include "sparse_onnx.hpp"

#include <algorithm>
#include <cstdlib>
#include <functional>
#include <stdexcept>
#include <unordered_set>

#include "model_impl.hpp"
#include "rbm_conv.hpp"
#include "onnx_wire.hpp"

using namespace sparseops;

namespace {

std::vector<float> transposed(const std::vector<float> &a, uint32_t rows, uint32_t cols)
{
    std::vector<float> t(a.size());
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t c = 0; c < cols; ++c) t[std::size_t(c) * rows + r] = a[std::size_t(r) * cols + c];
    return t;
}

std::size_t features_of(const std::vector<int> &shape)
{
    std::size_t f = 1;
    for (std::size_t d = 1; d < shape.size(); ++d) f *= std::size_t(shape[d]);
    return f;
}

int act_of(const std::string &op)
{
    if (op == "Relu") return SO_ACT_RELU;
    if (op == "Sigmoid") return SO_ACT_SIGMOID;
    if (op == "Tanh") return SO_ACT_TANH;
    return SO_ACT_NONE;
}

const char *act_name(int act)
{
    switch (act) {
    case SO_ACT_RELU: return "relu";
    case SO_ACT_SIGMOID: return "sigmoid";
    case SO_ACT_TANH: return "tanh";
    default: return "none";
    }
}

// A layer before slot assignment: tensor names instead of slot ids.
struct Pending {
    LayerPlan plan;
    std::vector<std::string> inputs;
    std::string output;
};

std::vector<int64_t> ints_attr(const onnxwire::Node &n, const char *name, std::size_t expect,
                               std::vector<int64_t> dflt)
{
    const onnxwire::Attribute *a = n.find(name);
    if (!a) return dflt;
    if (a->ints.size() != expect)
        throw std::runtime_error(n.op_type + ": attribute '" + name + "' must have " + std::to_string(expect) + " entries");
    return a->ints;
}

} // namespace

SparseOnnxModel::Impl::~Impl()
{
    so_ctx *ctx = nullptr;
    try { ctx = context(); } catch (...) { return; }
    if (graph) so_graph_free(ctx, graph);
    for (auto &L : layers) {
        if (L.conv) so_conv_plan_free(ctx, L.conv);
        if (L.rbm) so_rbm_free(ctx, L.rbm);
    }
}

SparseOnnxModel::~SparseOnnxModel() = default;
SparseOnnxModel::SparseOnnxModel(SparseOnnxModel &&) noexcept = default;
SparseOnnxModel &SparseOnnxModel::operator=(SparseOnnxModel &&) noexcept = default;

SparseOnnxModel::SparseOnnxModel(const std::string &onnx_path) : impl_(new Impl())
{
    Impl &M = *impl_;
    const onnxwire::Model model = onnxwire::load_model(onnx_path);
    const onnxwire::Graph &graph = model.graph;

    std::unordered_map<std::string, const onnxwire::Tensor *> init;
    for (const auto &t : graph.initializer) init[t.name] = &t;

    // Identity outputs are aliases of their input (src/sparse_onnx.cpp:522-534);
    // Flatten is an alias too because features are already in flatten order.
    std::unordered_map<std::string, std::string> alias;
    std::function<std::string(const std::string &)> resolve = [&](const std::string &nm) {
        auto it = alias.find(nm);
        return it == alias.end() ? nm : resolve(it->second);
    };

    // Graph input: first input that is not an initializer; exactly one output.
    const onnxwire::ValueInfo *in_vi = nullptr;
    for (const auto &vi : graph.input)
        if (!init.count(vi.name)) { in_vi = &vi; break; }
    if (!in_vi) throw std::runtime_error("No non-initializer input found in ONNX graph");
    if (graph.output.size() != 1) throw std::runtime_error("Expected exactly one graph output");
    M.input_name = in_vi->name;

    for (const auto &d : in_vi->dims) {
        if (!d.has_value || d.value <= 0) throw std::runtime_error("Dynamic dims not supported");
        M.input_dims.push_back(int(d.value));
    }
    if (M.input_dims.size() < 2) throw std::runtime_error("Input tensor must have rank >= 2");
    M.shape_map[M.input_name] = M.input_dims;
    M.in_features = features_of(M.input_dims);
    const int B0 = M.input_dims[0];

    std::vector<Pending> pend;
    auto shape_of = [&](const std::string &nm) -> const std::vector<int> & {
        auto it = M.shape_map.find(nm);
        if (it == M.shape_map.end()) throw std::runtime_error("Tensor '" + nm + "' is used before it is produced");
        return it->second;
    };

    for (const onnxwire::Node &node : graph.node) {
        const std::string &op = node.op_type;
        if (node.output.empty()) throw std::runtime_error(op + ": node without output");
        const std::string &out = node.output[0];
        auto need_inputs = [&](std::size_t k) {
            if (node.input.size() < k) throw std::runtime_error(op + ": expected at least " + std::to_string(k) + " inputs");
        };

        if (op == "MatMul" || op == "Gemm") {
            need_inputs(2);
            auto itW = init.find(resolve(node.input[1]));
            if (itW == init.end()) throw std::runtime_error("Weight '" + resolve(node.input[1]) + "' not found");
            const onnxwire::Tensor &Wt = *itW->second;
            if (Wt.dims.size() != 2) throw std::runtime_error("FC weight must be 2D");
            const uint32_t d0 = uint32_t(Wt.dims[0]), d1 = uint32_t(Wt.dims[1]);
            std::vector<float> W = Wt.floats();
            uint32_t Mo, N;
            if (op == "MatMul") {                       // X(B x N) * W(N x M)
                N = d0; Mo = d1;
                W = transposed(W, N, Mo);
            } else {
                // transB defaults to 1 here, as in the reference (src/sparse_onnx.cpp:204-216):
                // that is how PyTorch exports nn.Linear.
                int64_t transB = 1;
                if (const auto *a = node.find("transB")) transB = a->i;
                if (const auto *a = node.find("transA"))
                    if (a->i != 0) throw std::runtime_error("Gemm: transA is not supported");
                for (const char *nm : {"alpha", "beta"})
                    if (const auto *a = node.find(nm))
                        if (a->f != 1.0f) throw std::runtime_error(std::string("Gemm: ") + nm + " != 1 is not supported");
                if (transB == 1) { Mo = d0; N = d1; }
                else { N = d0; Mo = d1; W = transposed(W, N, Mo); }
            }
            const std::string x = resolve(node.input[0]);
            const auto &xs = shape_of(x);
            if (features_of(xs) != N)
                throw std::runtime_error(op + ": input has " + std::to_string(features_of(xs)) +
                                         " features, weight expects " + std::to_string(N));
            Pending p;
            p.plan.op = Op::MatMul;
            p.plan.name = op;
            M.weights.emplace_back(new Ellpack(convert_to_ellpack(W.data(), Mo, N)));
            p.plan.E = M.weights.back().get();
            p.plan.in_features = N;
            p.plan.out_features = Mo;
            if (op == "Gemm" && node.input.size() > 2 && !node.input[2].empty()) {
                auto itB = init.find(resolve(node.input[2]));
                if (itB != init.end()) {
                    p.plan.bias = itB->second->floats();
                    if (p.plan.bias.size() != Mo) throw std::runtime_error("Gemm: bias length must equal the output features");
                    p.plan.has_bias = true;
                }
            }
            p.inputs = {x};
            p.output = out;
            pend.push_back(std::move(p));
            M.shape_map[out] = {B0, int(Mo)};
            continue;
        }

        if (op == "Conv") {
            need_inputs(2);
            auto itW = init.find(resolve(node.input[1]));
            if (itW == init.end()) throw std::runtime_error("Conv weight initializer not found");
            const onnxwire::Tensor &Wt = *itW->second;
            if (Wt.dims.size() != 4) throw std::runtime_error("Conv weight must be 4D");
            const uint32_t Cout = uint32_t(Wt.dims[0]), Cin = uint32_t(Wt.dims[1]);
            const uint32_t kH = uint32_t(Wt.dims[2]), kW = uint32_t(Wt.dims[3]);
            const auto pads = ints_attr(node, "pads", 4, {0, 0, 0, 0});
            const auto strides = ints_attr(node, "strides", 2, {1, 1});
            const auto dil = ints_attr(node, "dilations", 2, {1, 1});
            int64_t group = 1;
            if (const auto *a = node.find("group")) group = a->i;
            if (group != 1) throw std::runtime_error("Grouped conv not supported (yet)");
            // The reference reads the begin pads only (src/sparse_onnx.cpp:411) and
            // sizes the output as if both sides were padded alike (:428-429);
            // asymmetric padding would silently compute something else, so refuse it.
            if (pads[0] != pads[2] || pads[1] != pads[3]) throw std::runtime_error("Conv: asymmetric pads are not supported");
            const std::string x = resolve(node.input[0]);
            const auto &xs = shape_of(x);
            if (xs.size() != 4) throw std::runtime_error("Conv input must be 4D");
            if (uint32_t(xs[1]) != Cin) throw std::runtime_error("Conv Cin mismatch");
            so_conv_geom g{};
            g.Cin = Cin; g.Cout = Cout; g.kH = kH; g.kW = kW;
            g.stride_h = uint32_t(strides[0]); g.stride_w = uint32_t(strides[1]);
            g.pad_h = uint32_t(pads[0]); g.pad_w = uint32_t(pads[1]);
            g.dil_h = uint32_t(dil[0]); g.dil_w = uint32_t(dil[1]);
            g.H_in = uint32_t(xs[2]); g.W_in = uint32_t(xs[3]);
            if (!g.stride_h || !g.stride_w || !g.dil_h || !g.dil_w || !kH || !kW)
                throw std::runtime_error("Conv: kernel, stride and dilation must be positive");
            if (g.H_in + 2 * g.pad_h < g.dil_h * (kH - 1) + 1 || g.W_in + 2 * g.pad_w < g.dil_w * (kW - 1) + 1)
                throw std::runtime_error("Conv: kernel window larger than the padded input");
            g.H_out = (g.H_in + 2 * g.pad_h - (g.dil_h * (kH - 1) + 1)) / g.stride_h + 1;
            g.W_out = (g.W_in + 2 * g.pad_w - (g.dil_w * (kW - 1) + 1)) / g.stride_w + 1;
            Pending p;
            p.plan.op = Op::Conv;
            p.plan.name = op;
            // [Cout][Cin][kH][kW] row-major is already the Cout x K matrix with
            // K ordered (cin, kh, kw) (src/sparse_onnx.cpp:394-405).
            const std::vector<float> W = Wt.floats();
            M.weights.emplace_back(new Ellpack(convert_to_ellpack(W.data(), Cout, Cin * kH * kW)));
            p.plan.E = M.weights.back().get();
            p.plan.cg = g;
            p.plan.in_features = std::size_t(Cin) * g.H_in * g.W_in;
            p.plan.out_features = std::size_t(Cout) * g.H_out * g.W_out;
            if (node.input.size() > 2 && !node.input[2].empty()) {
                auto itB = init.find(resolve(node.input[2]));
                if (itB != init.end()) {
                    p.plan.bias = itB->second->floats();
                    if (p.plan.bias.size() != Cout) throw std::runtime_error("Conv: bias length must equal Cout");
                    p.plan.has_bias = true;
                }
            }
            p.inputs = {x};
            p.output = out;
            pend.push_back(std::move(p));
            M.shape_map[out] = {B0, int(Cout), int(g.H_out), int(g.W_out)};
            continue;
        }

        if (op == "Relu" || op == "Sigmoid" || op == "Tanh") {
            need_inputs(1);
            const std::string x = resolve(node.input[0]);
            Pending p;
            p.plan.op = Op::Act;
            p.plan.name = op;
            p.plan.act = act_of(op);
            p.plan.out_features = features_of(shape_of(x));
            p.inputs = {x};
            p.output = out;
            pend.push_back(std::move(p));
            M.shape_map[out] = shape_of(x);
            continue;
        }

        if (op == "Add") {
            need_inputs(2);
            std::string a = resolve(node.input[0]), b = resolve(node.input[1]);
            // x + constant vector right after a bias-free FC layer is that layer's
            // bias (PyTorch exports nn.Linear on >2-D input this way).
            if (init.count(a)) std::swap(a, b);
            if (init.count(b)) {
                const onnxwire::Tensor &bt = *init[b];
                Pending *prod = nullptr;
                for (auto &q : pend)
                    if (q.output == a) prod = &q;
                if (init.count(a) || !prod || prod->plan.op != Op::MatMul || prod->plan.has_bias ||
                    bt.numel() != prod->plan.out_features)
                    throw std::runtime_error("Add with a constant operand is only supported as the bias of the preceding MatMul");
                prod->plan.bias = bt.floats();
                prod->plan.has_bias = true;
                prod->output = out;
                M.shape_map[out] = shape_of(a);
                continue;
            }
            if (shape_of(a) != shape_of(b)) throw std::runtime_error("Add: operand shapes differ (broadcasting is not supported)");
            Pending p;
            p.plan.op = Op::Add;
            p.plan.name = op;
            p.plan.out_features = features_of(shape_of(a));
            p.inputs = {a, b};
            p.output = out;
            pend.push_back(std::move(p));
            M.shape_map[out] = shape_of(a);
            continue;
        }

        if (op == "MaxPool" || op == "GlobalAveragePool") {
            need_inputs(1);
            const std::string x = resolve(node.input[0]);
            const auto xs = shape_of(x);
            if (xs.size() != 4) throw std::runtime_error("Pool input must be 4D");
            Pending p;
            p.plan.name = op;
            so_pool_geom g{};
            g.C = uint32_t(xs[1]); g.H = uint32_t(xs[2]); g.W = uint32_t(xs[3]);
            p.plan.in_features = features_of(xs);
            if (op == "GlobalAveragePool") {
                p.plan.op = Op::GlobalAveragePool;
                g.H_out = g.W_out = 1;
                // exposed as (B, C), as the reference does (src/sparse_onnx.cpp:334-336)
                M.shape_map[out] = {B0, int(g.C)};
                p.plan.out_features = g.C;
            } else {
                p.plan.op = Op::MaxPool;
                const auto k = ints_attr(node, "kernel_shape", 2, {1, 1});
                const auto s = ints_attr(node, "strides", 2, {1, 1});
                const auto pd = ints_attr(node, "pads", 4, {0, 0, 0, 0});
                if (const auto *a = node.find("ceil_mode"))
                    if (a->i != 0) throw std::runtime_error("MaxPool: ceil_mode is not supported");
                if (const auto *a = node.find("dilations"))
                    for (int64_t d : a->ints)
                        if (d != 1) throw std::runtime_error("MaxPool: dilations are not supported");
                if (k[0] <= 0 || k[1] <= 0 || s[0] <= 0 || s[1] <= 0) throw std::runtime_error("MaxPool: bad kernel/stride");
                g.kH = int32_t(k[0]); g.kW = int32_t(k[1]);
                g.sH = int32_t(s[0]); g.sW = int32_t(s[1]);
                g.padH0 = int32_t(pd[0]); g.padW0 = int32_t(pd[1]);
                const int hspan = int(g.H) + int(pd[0]) + int(pd[2]) - g.kH;
                const int wspan = int(g.W) + int(pd[1]) + int(pd[3]) - g.kW;
                if (hspan < 0 || wspan < 0) throw std::runtime_error("MaxPool: window larger than the padded input");
                g.H_out = uint32_t(hspan / g.sH + 1);   // src/sparse_onnx.cpp:338-339
                g.W_out = uint32_t(wspan / g.sW + 1);
                M.shape_map[out] = {B0, int(g.C), int(g.H_out), int(g.W_out)};
                p.plan.out_features = std::size_t(g.C) * g.H_out * g.W_out;
            }
            p.plan.pg = g;
            p.inputs = {x};
            p.output = out;
            pend.push_back(std::move(p));
            continue;
        }

        if (op == "Flatten") {
            need_inputs(1);
            int64_t axis = 1;
            if (const auto *a = node.find("axis")) axis = a->i;
            if (axis != 1) throw std::runtime_error("Flatten: only axis=1 is supported");
            const std::string x = resolve(node.input[0]);
            alias[out] = x;
            M.shape_map[out] = {B0, int(features_of(shape_of(x)))};
            continue;
        }

        if (op == "Identity") {
            need_inputs(1);
            const std::string x = resolve(node.input[0]);
            alias[out] = x;
            if (M.shape_map.count(x)) M.shape_map[out] = M.shape_map[x];
            continue;
        }

        throw std::runtime_error("Unsupported ONNX op: " + op);
    }

    const std::string graph_out = graph.output[0].name;
    M.output_name = resolve(graph_out);
    if (!M.shape_map.count(graph_out)) throw std::runtime_error("Graph output '" + graph_out + "' is never produced");
    const std::vector<int> out_shape = M.shape_map[graph_out];
    M.out_features = features_of(out_shape);
    M.output_dims = out_shape;

    // Fuse into the producing MatMul/Conv, when nothing else reads the intermediate:
    //  * a following activation (src/sparse_onnx.cpp:573-620, extended to Sigmoid/Tanh);
    //  * for Conv, a following residual Add whose other operand already exists when the
    //    convolution runs, and then the activation after that Add (the tail of a ResNet
    //    basic block: conv -> add(skip) -> relu becomes one launch, same arithmetic).
    {
        std::unordered_map<std::string, int> uses;
        for (const auto &p : pend)
            for (const auto &i : p.inputs) uses[i]++;
        uses[M.output_name]++;
        auto produced_before = [&](const std::string &t, std::size_t layer) {
            if (t == M.input_name) return true;
            for (std::size_t k = 0; k < layer; ++k)
                if (pend[k].output == t) return true;
            return false;
        };
        for (std::size_t i = 0; i + 1 < pend.size();) {
            Pending &A = pend[i], &Bn = pend[i + 1];
            const bool producer = A.plan.op == Op::MatMul || A.plan.op == Op::Conv;
            if (producer && A.plan.act == SO_ACT_NONE && Bn.plan.op == Op::Act && Bn.inputs[0] == A.output &&
                uses[A.output] == 1) {
                A.plan.act = Bn.plan.act;
                A.output = Bn.output;
                pend.erase(pend.begin() + long(i) + 1);
                continue;
            }
            if (A.plan.op == Op::Conv && A.plan.act == SO_ACT_NONE && !A.plan.residual && Bn.plan.op == Op::Add &&
                uses[A.output] == 1 && (Bn.inputs[0] == A.output) != (Bn.inputs[1] == A.output)) {
                const std::string skip = Bn.inputs[0] == A.output ? Bn.inputs[1] : Bn.inputs[0];
                if (produced_before(skip, i)) {
                    A.plan.residual = true;
                    A.inputs.push_back(skip);
                    A.output = Bn.output;
                    pend.erase(pend.begin() + long(i) + 1);
                    continue;                       // look at the same layer again: an activation may follow
                }
            }
            ++i;
        }
    }

    // Arena slots: a tensor keeps its slot until its last reader has been
    // enqueued; slots are then recycled, so the arena holds the live set only.
    {
        std::unordered_map<std::string, int> last_use, slot_of;
        for (std::size_t i = 0; i < pend.size(); ++i)
            for (const auto &nm : pend[i].inputs) last_use[nm] = int(i);
        last_use[M.output_name] = int(pend.size());  // never recycled
        std::vector<int> free_slots;
        // Smallest free slot that is large enough, else the largest one (it grows).
        auto acquire = [&](std::size_t feat) {
            int best = -1;
            for (int s : free_slots) {
                if (best < 0) { best = s; continue; }
                const bool fits = M.slots[s].features >= feat, best_fits = M.slots[best].features >= feat;
                if (fits && (!best_fits || M.slots[s].features < M.slots[best].features)) best = s;
                else if (!fits && !best_fits && M.slots[s].features > M.slots[best].features) best = s;
            }
            if (best < 0) {
                M.slots.push_back(Slot{feat, 0});
                return int(M.slots.size()) - 1;
            }
            free_slots.erase(std::find(free_slots.begin(), free_slots.end(), best));
            M.slots[best].features = std::max(M.slots[best].features, feat);
            return best;
        };
        M.input_slot = acquire(M.in_features);
        slot_of[M.input_name] = M.input_slot;
        for (std::size_t i = 0; i < pend.size(); ++i) {
            Pending &p = pend[i];
            for (const auto &nm : p.inputs)
                if (!slot_of.count(nm)) throw std::runtime_error("Tensor '" + nm + "' is used before it is produced");
            p.plan.in0 = slot_of[p.inputs[0]];
            if (p.inputs.size() > 1) p.plan.in1 = slot_of[p.inputs[1]];
            p.plan.out = acquire(p.plan.out_features);
            p.plan.out_tensor = p.output;
            slot_of[p.output] = p.plan.out;
            std::unordered_set<std::string> seen;
            for (const auto &nm : p.inputs)
                if (seen.insert(nm).second && last_use[nm] == int(i) && nm != M.output_name && nm != M.input_name)
                    free_slots.push_back(slot_of[nm]);
            if (!last_use.count(p.output)) free_slots.push_back(p.plan.out);  // dead result
        }
        if (!slot_of.count(M.output_name)) throw std::runtime_error("Graph output is never produced");
        M.output_slot = slot_of[M.output_name];
    }

    // Weights, conv plans and biases into HBM.
    so_ctx *ctx = context();
    std::size_t bias_total = 0;
    // Large fully connected layers run on the row-block-merged kernel (fp32 round-off accuracy, the fastest);
    // SPARSEOPS_MATMUL_RBM=0 at load time keeps every layer on the kernels that give the reference's bits.
    const char *rbm_env = std::getenv("SPARSEOPS_MATMUL_RBM");
    const bool fast_fc = !(rbm_env && rbm_env[0] == '0');
    for (auto &p : pend) {
        if (p.plan.op != Op::MatMul && p.plan.op != Op::Conv) continue;
        p.plan.dE = mirror(*p.plan.E, p.plan.op == Op::MatMul ? matmul_layouts(*p.plan.E, uint32_t(B0), fast_fc) : SO_LAYOUT_ROW);
        if (p.plan.op == Op::Conv) {
            check(so_conv_plan_create(ctx, p.plan.dE, &p.plan.cg, &p.plan.conv), "so_conv_plan_create");
            // The reference builds its row-block-merged plan for wide convolutions at load
            // (src/sparse_onnx.cpp:499-502: Cout >= 32 and K >= 64, blocks of 8 channels) and never
            // runs it; here the plan goes to the device library, whose so_conv2d walks it wherever
            // that is the faster kernel for the batch at hand.
            if (p.plan.cg.Cout >= 32 && p.plan.E->n >= 64) {
                p.plan.rbm = upload_rbm(build_rbm_from_ellpack(*p.plan.E, nullptr, 8));
                check(so_conv_plan_set_rbm(ctx, p.plan.conv, p.plan.rbm), "so_conv_plan_set_rbm");
            }
        }
        if (p.plan.has_bias) {
            p.plan.bias_offset = bias_total;
            bias_total += (p.plan.bias.size() + 63) / 64 * 64;
        }
    }
    if (bias_total) {
        std::vector<float> packed(bias_total, 0.0f);
        for (const auto &p : pend)
            if (p.plan.has_bias) std::copy(p.plan.bias.begin(), p.plan.bias.end(), packed.begin() + long(p.plan.bias_offset));
        M.bias_pool.reserve(bias_total * sizeof(float));
        check(so_h2d(ctx, M.bias_pool.get(), packed.data(), bias_total * sizeof(float)), "so_h2d(bias)");
    }
    for (auto &p : pend) M.layers.push_back(std::move(p.plan));

    // A recorded launch graph saves host time per launch but adds device time per kernel (measured on
    // a 4-layer MLP: 111 us per replay against 102 us for the same four launches in a row; on a
    // 23-launch CNN the two are within 1 %): record one only for chains of eight layers or more.
    // SPARSEOPS_NO_GRAPH=1 never records, =0 always does.
    M.use_graph = M.layers.size() >= 8;
    if (const char *e = std::getenv("SPARSEOPS_NO_GRAPH")) M.use_graph = !(e[0] && e[0] != '0');
    resize_buffers(uint32_t(B0));
}

std::vector<std::size_t> SparseOnnxModel::output_shape() const
{
    std::vector<std::size_t> dims(impl_->output_dims.begin(), impl_->output_dims.end());
    if (!dims.empty()) dims[0] = impl_->batch;
    return dims;
}

std::vector<std::size_t> SparseOnnxModel::input_shape() const
{
    std::vector<std::size_t> dims(impl_->input_dims.begin(), impl_->input_dims.end());
    if (!dims.empty()) dims[0] = impl_->batch;
    return dims;
}

uint32_t SparseOnnxModel::batch() const { return impl_->batch; }
std::size_t SparseOnnxModel::input_features() const { return impl_->in_features; }
std::size_t SparseOnnxModel::output_features() const { return impl_->out_features; }

std::vector<std::string> SparseOnnxModel::describe() const
{
    std::vector<std::string> out;
    for (const auto &L : impl_->layers) {
        std::string s = L.name;
        if (L.E) {
            uint64_t nnz = 0;
            for (uint32_t c : L.E->nnz) nnz += c;
            s += " " + std::to_string(L.E->m) + "x" + std::to_string(L.E->n) + " r=" + std::to_string(L.E->r) +
                 " nnz=" + std::to_string(nnz) + " act=" + act_name(L.act) + " bias=" + (L.has_bias ? "1" : "0");
            if (L.residual) s += " +residual";
        } else if (L.op == Op::Act) {
            s += std::string(" act=") + act_name(L.act);
        }
        s += " out_features=" + std::to_string(L.out_features);
        out.push_back(s);
    }
    return out;
}

double SparseOnnxModel::nnz_flops_per_sample() const
{
    double f = 0;
    for (const auto &L : impl_->layers) {
        if (!L.E) continue;
        uint64_t nnz = 0;
        for (uint32_t c : L.E->nnz) nnz += c;
        const double cols = L.op == Op::Conv ? double(L.cg.H_out) * L.cg.W_out : 1.0;
        f += 2.0 * double(nnz) * cols;
    }
    return f;
}
