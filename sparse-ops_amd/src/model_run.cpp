// SparseOnnxModel: buffer sizing and execution.  The reference walks the layers
// with a name->buffer map and allocates every output per call
// (src/model_run.cpp:3-140, src/layers/*.cpp); here every tensor has a fixed slot
// in one HBM arena, the chain is recorded once into a launch graph, and a call
// with an unchanged batch size allocates nothing.
#include "sparse_onnx.hpp"

#include <algorithm>
#include <stdexcept>

#include "model_impl.hpp"

using namespace sparseops;

void SparseOnnxModel::resize_buffers(uint32_t batch)
{
    Impl &M = *impl_;
    if (batch == 0) throw std::runtime_error("resize_buffers: batch must be positive");
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    if (M.graph) { so_graph_free(ctx, M.graph); M.graph = nullptr; }
    M.has_conv = false;
    for (const LayerPlan &L : M.layers) M.has_conv |= L.conv != nullptr;
    // The convolutions work on batch tiles of 16, 8 or 4 entries, and the larger the tile the less a
    // batch entry costs: a batch is carried in rows of 4 (up to 4 entries), 8 (up to 8) or the next
    // multiple of 16 (the extra columns are zeros on input and are never copied out; batch entries
    // do not interact).  Measured on a ResNet-18-shaped stack: 12 entries as 12 0.86 ms, as 16
    // 0.76 ms; 24 as 24 1.31 ms, as 32 1.24 ms.
    uint32_t pbatch = batch;
    if (M.has_conv) pbatch = batch <= 4 ? 4u : batch <= 8 ? 8u : (batch + 15u) / 16u * 16u;
    // Slot offsets for this batch, 256-byte aligned.
    std::size_t total = 0;
    std::size_t widest = std::max(M.in_features, M.out_features);
    for (Slot &s : M.slots) {
        s.offset = total;
        total += (s.features * pbatch + 63) / 64 * 64;
    }
    M.arena.reserve(total * sizeof(float));
    M.stage_in.reserve(M.in_features * batch * sizeof(float));
    M.stage_out.reserve(M.out_features * batch * sizeof(float));
    if (pbatch != batch) M.stage_mid.reserve(widest * batch * sizeof(float));
    M.batch = batch;
    M.pbatch = pbatch;
    for (const LayerPlan &L : M.layers) {
        if (L.conv) check(so_conv_plan_tune(ctx, L.conv, pbatch), "so_conv_plan_tune");
        // whatever so_matmul would allocate at this batch is allocated now (run() allocates nothing, and a
        // launch graph cannot be recorded across an allocation)
        else if (L.op == Op::MatMul && L.dE) check(so_matmul_reserve(ctx, L.dE, pbatch), "so_matmul_reserve");
    }
    if (M.use_graph && !M.layers.empty()) {
        check(so_graph_begin(ctx), "so_graph_begin");
        try {
            M.enqueue_layers();
        } catch (...) {
            so_graph *g = nullptr;
            so_graph_end(ctx, &g);
            so_graph_free(ctx, g);
            throw;
        }
        check(so_graph_end(ctx, &M.graph), "so_graph_end");
    }
}

void SparseOnnxModel::Impl::enqueue_layers() const
{
    so_ctx *ctx = context();
    const uint32_t B = pbatch;
    // Every layer reads and writes arena slots.  A slot id is shared by all tensors whose lifetimes
    // do not overlap, so it identifies neither the graph input nor the graph output: callers' buffers
    // are copied into the input slot before the chain and out of the output slot after it.
    auto src = [&](int s) -> const float * { return slot_ptr(s); };
    auto dst = [&](int s) -> float * { return slot_ptr(s); };
    for (const LayerPlan &L : layers) {
        const float *bias = L.has_bias ? bias_pool.f32() + L.bias_offset : nullptr;
        switch (L.op) {
        case Op::MatMul:
            check(so_matmul(ctx, L.dE, src(L.in0), B, bias, dst(L.out), L.act), "so_matmul");
            break;
        case Op::Conv:
            if (L.residual)
                check(so_conv2d_add(ctx, L.conv, src(L.in0), B, bias, src(L.in1), dst(L.out), L.act), "so_conv2d_add");
            else
                check(so_conv2d(ctx, L.conv, src(L.in0), B, bias, dst(L.out), L.act), "so_conv2d");
            break;
        case Op::Act:
            check(so_act(ctx, L.act, src(L.in0), L.out_features * B, dst(L.out)), "so_act");
            break;
        case Op::Add:
            check(so_add(ctx, src(L.in0), src(L.in1), L.out_features * B, dst(L.out)), "so_add");
            break;
        case Op::MaxPool:
            check(so_maxpool(ctx, &L.pg, src(L.in0), B, dst(L.out)), "so_maxpool");
            break;
        case Op::GlobalAveragePool:
            check(so_gap(ctx, L.pg.C, L.pg.H, L.pg.W, src(L.in0), B, dst(L.out)), "so_gap");
            break;
        }
    }
}

void SparseOnnxModel::Impl::launch_chain() const
{
    if (graph) check(so_graph_launch(context(), graph), "so_graph_launch");
    else enqueue_layers();
}

void SparseOnnxModel::Impl::rows_in(const float *d_rows) const
{
    check(so_copy_rows(context(), d_rows, batch, uint32_t(in_features), batch, slot_ptr(input_slot), pbatch, 1), "so_copy_rows(input)");
}

void SparseOnnxModel::Impl::rows_out(float *d_rows) const
{
    check(so_copy_rows(context(), slot_ptr(output_slot), pbatch, uint32_t(out_features), batch, d_rows, batch, 0), "so_copy_rows(output)");
}

void SparseOnnxModel::run(const float *input, uint32_t B, float *output) const
{
    Impl &M = *impl_;
    if (B != M.batch) const_cast<SparseOnnxModel *>(this)->resize_buffers(B);
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    if (!M.padded()) {
        check(so_h2d(ctx, M.slot_ptr(M.input_slot), input, M.in_features * B * sizeof(float)), "so_h2d(input)");
        M.launch_chain();
        check(so_d2h(ctx, output, M.slot_ptr(M.output_slot), M.out_features * B * sizeof(float)), "so_d2h(output)");
        return;
    }
    check(so_h2d(ctx, M.stage_in.get(), input, M.in_features * B * sizeof(float)), "so_h2d(input)");
    M.rows_in(M.stage_in.f32());
    M.launch_chain();
    M.rows_out(M.stage_out.f32());
    check(so_d2h(ctx, output, M.stage_out.get(), M.out_features * B * sizeof(float)), "so_d2h(output)");
}

void SparseOnnxModel::run_batch_major(const float *input, uint32_t B, float *output) const
{
    Impl &M = *impl_;
    if (B != M.batch) const_cast<SparseOnnxModel *>(this)->resize_buffers(B);
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    check(so_h2d(ctx, M.stage_in.get(), input, M.in_features * B * sizeof(float)), "so_h2d(input)");
    if (!M.padded()) {
        check(so_transpose(ctx, M.stage_in.f32(), B, uint32_t(M.in_features), M.slot_ptr(M.input_slot)), "so_transpose(input)");
        M.launch_chain();
        check(so_transpose(ctx, M.slot_ptr(M.output_slot), uint32_t(M.out_features), B, M.stage_out.f32()), "so_transpose(output)");
    } else {
        check(so_transpose(ctx, M.stage_in.f32(), B, uint32_t(M.in_features), M.stage_mid.f32()), "so_transpose(input)");
        M.rows_in(M.stage_mid.f32());
        M.launch_chain();
        M.rows_out(M.stage_mid.f32());
        check(so_transpose(ctx, M.stage_mid.f32(), uint32_t(M.out_features), B, M.stage_out.f32()), "so_transpose(output)");
    }
    check(so_d2h(ctx, output, M.stage_out.get(), M.out_features * B * sizeof(float)), "so_d2h(output)");
}

void SparseOnnxModel::run_device(const float *dInput, uint32_t B, float *dOutput) const
{
    Impl &M = *impl_;
    if (B != M.batch) const_cast<SparseOnnxModel *>(this)->resize_buffers(B);
    if (!dInput || !dOutput) throw std::runtime_error("run_device: null device pointer");
    std::lock_guard<std::mutex> lock(context_mutex());
    if (M.layers.empty()) {
        check(so_d2d(context(), dOutput, dInput, M.in_features * B * sizeof(float)), "so_d2d");
        return;
    }
    if (M.padded()) {
        M.rows_in(dInput);
        M.launch_chain();
        M.rows_out(dOutput);
        return;
    }
    so_ctx *ctx = context();
    check(so_d2d(ctx, M.slot_ptr(M.input_slot), dInput, M.in_features * B * sizeof(float)), "so_d2d(input)");
    M.launch_chain();
    check(so_d2d(ctx, dOutput, M.slot_ptr(M.output_slot), M.out_features * B * sizeof(float)), "so_d2d(output)");
}

double SparseOnnxModel::time_device(int steps, int warmup) const
{
    Impl &M = *impl_;
    if (steps <= 0) throw std::runtime_error("time_device: steps must be positive");
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    for (int i = 0; i < warmup; ++i) M.launch_chain();
    check(so_timer_begin(ctx), "so_timer_begin");
    for (int i = 0; i < steps; ++i) M.launch_chain();
    float ms = 0.0f;
    check(so_timer_end(ctx, &ms), "so_timer_end");
    return double(ms) / steps;
}
