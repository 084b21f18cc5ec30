// Context, memory, timing, launch graphs and the device-resident ELLPACK layouts.
#include "so_internal.h"

#include <algorithm>
#include <cstdarg>
#include <cstring>
#include <new>

static thread_local std::string g_last_error;

// Scratch memory of so_ellpack_encode_noalloc: the counting pass's header and per-workgroup partial
// results (layout further down, at the encoder).  Every GPU the library runs on holds its own copy
// at its own address; host code never uses this name as a pointer, only the address that so_init
// looks up for the context's device.
constexpr size_t kStaticScratchBytes = 256 + 65536 * 8;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

void so_set_error(const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

extern "C" const char *so_last_error(void) { return g_last_error.c_str(); }

extern "C" so_status so_device_count(int *n)
{
    SO_REQUIRE(n != nullptr, "so_device_count: n is null");
    *n = 0;
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e != hipSuccess || c <= 0) {
        (void)hipGetLastError();
        so_set_error("no HIP device available (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
        return SO_ERR_NO_DEVICE;
    }
    *n = c;
    return SO_OK;
}

hipError_t so_allow_big_lds(so_ctx *ctx, const void *kernel)
{
    for (const void *k : ctx->big_lds_kernels)
        if (k == kernel) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, ctx->max_lds_bytes);
    if (e == hipSuccess) ctx->big_lds_kernels.push_back(kernel);
    else (void)hipGetLastError();
    return e;
}

static int env_int(const char *name, int unset)
{
    const char *e = getenv(name);
    return (e && e[0]) ? atoi(e) : unset;
}

static void read_tuning(so_tuning &t)
{
    t = so_tuning();
    t.matmul_tiled = env_int("SPARSEOPS_MATMUL_TILED", -1);
    t.matmul_vec = env_int("SPARSEOPS_MATMUL_VEC", 0);
    t.matmul_share = env_int("SPARSEOPS_MATMUL_SHARE", -1);
    t.matmul_rbm = env_int("SPARSEOPS_MATMUL_RBM", -1);
    t.matmul_rbm_split = env_int("SPARSEOPS_MATMUL_RBM_SPLIT", 0);
    const int lanes = env_int("SPARSEOPS_MATVEC_LANES", 0);
    t.matvec_lanes = (lanes == 8 || lanes == 16 || lanes == 32 || lanes == 64) ? lanes : 0;
    t.matvec_idx16 = env_int("SPARSEOPS_MATVEC_IDX16", -1);
    t.conv_min_cg = env_int("SPARSEOPS_CONV_MIN_CG", 0);
    t.conv_window = env_int("SPARSEOPS_CONV_WINDOW", -1);
    t.conv_cpw = env_int("SPARSEOPS_CONV_CPW", 0);
    t.conv_tilepx = env_int("SPARSEOPS_CONV_TILEPX", 0);
    t.conv_vec = env_int("SPARSEOPS_CONV_VEC", 0);
    t.conv_rbm = env_int("SPARSEOPS_CONV_RBM", -1);
    t.wait_spins = env_int("SPARSEOPS_WAIT_SPINS", -1);
}

extern "C" so_status so_tuning_reload(so_ctx *ctx)
{
    SO_REQUIRE(ctx != nullptr, "so_tuning_reload: ctx is null");
    read_tuning(ctx->tune);
    return SO_OK;
}

extern "C" so_status so_init(int device, so_ctx **out)
{
    SO_REQUIRE(out != nullptr, "so_init: out is null");
    *out = nullptr;
    int c = 0;
    so_status s = so_device_count(&c);
    if (s != SO_OK) return s;
    SO_REQUIRE(device >= 0 && device < c, "so_init: device %d out of range (have %d)", device, c);
    SO_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    SO_HIP(hipGetDeviceProperties(&prop, device));
    so_ctx *ctx = new (std::nothrow) so_ctx();
    if (!ctx) { so_set_error("so_init: host allocation failed"); return SO_ERR_OOM; }
    ctx->device = device;
    ctx->compute_units = prop.multiProcessorCount;
    ctx->max_lds_bytes = (int)prop.sharedMemPerBlock;
    ctx->name = prop.gcnArchName;
    read_tuning(ctx->tune);
    hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev0);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev1);
    if (e != hipSuccess) {
        so_set_error("so_init: stream/event creation failed: %s", hipGetErrorString(e));
        so_destroy(ctx);
        return SO_ERR_HIP;
    }
    // this device's copy of the static scratch array (the device is current)
    e = hipGetSymbolAddress(&ctx->static_scratch, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ctx->static_scratch == nullptr) {
        so_set_error("so_init: hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
        so_destroy(ctx);
        return SO_ERR_HIP;
    }
    // the word in which waves that give up a bounded wait count themselves, and its pinned host copy
    e = hipMalloc((void **)&ctx->d_wait_gave_up, 64);
    if (e == hipSuccess) e = hipMemset(ctx->d_wait_gave_up, 0, 64);
    if (e == hipSuccess) e = hipHostMalloc((void **)&ctx->h_wait_gave_up, 64, hipHostMallocDefault);
    if (e != hipSuccess) {
        so_set_error("so_init: allocating the wait status word failed: %s", hipGetErrorString(e));
        so_destroy(ctx);
        return e == hipErrorOutOfMemory ? SO_ERR_OOM : SO_ERR_HIP;
    }
    *ctx->h_wait_gave_up = 0;
    *out = ctx;
    return SO_OK;
}

// Waits for the stream; when a kernel with bounded waits has run since the last look, its status word
// comes back with the same wait (one 4-byte copy queued behind the work) and is cleared if it was set.
so_status so_stream_wait(so_ctx *ctx, const char *who)
{
    const bool look = ctx->waits_pending;
    if (look) SO_HIP(hipMemcpyAsync(ctx->h_wait_gave_up, ctx->d_wait_gave_up, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    SO_HIP(hipStreamSynchronize(ctx->stream));
    if (!look) return SO_OK;
    ctx->waits_pending = false;
    const uint32_t gave_up = *ctx->h_wait_gave_up;
    if (gave_up == 0) return SO_OK;
    *ctx->h_wait_gave_up = 0;
    SO_HIP(hipMemsetAsync(ctx->d_wait_gave_up, 0, sizeof(uint32_t), ctx->stream));
    SO_HIP(hipStreamSynchronize(ctx->stream));
    so_set_error("%s: %u waits on LDS progress counters gave up in earlier launches; the results of those launches are invalid", who, gave_up);
    return SO_ERR_HIP;
}

extern "C" so_status so_destroy(so_ctx *ctx)
{
    if (!ctx) return SO_OK;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) { (void)hipStreamSynchronize(ctx->stream); (void)hipStreamDestroy(ctx->stream); }
    if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
    if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
    if (ctx->d_wait_gave_up) (void)hipFree(ctx->d_wait_gave_up);
    if (ctx->h_wait_gave_up) (void)hipHostFree(ctx->h_wait_gave_up);
    if (ctx->mm_part) (void)hipFree(ctx->mm_part);
    if (ctx->mm_counters) (void)hipFree(ctx->mm_counters);
    delete ctx;
    return SO_OK;
}

extern "C" so_status so_device_info(so_ctx *ctx, char *name, size_t name_len, int *compute_units)
{
    SO_REQUIRE(ctx != nullptr, "so_device_info: ctx is null");
    if (name && name_len) {
        std::strncpy(name, ctx->name.c_str(), name_len - 1);
        name[name_len - 1] = '\0';
    }
    if (compute_units) *compute_units = ctx->compute_units;
    return SO_OK;
}

extern "C" so_status so_malloc(so_ctx *ctx, size_t bytes, void **dptr)
{
    SO_REQUIRE(ctx && dptr, "so_malloc: null argument");
    SO_REQUIRE(!ctx->capturing, "so_malloc: not allowed while a graph is being recorded");
    *dptr = nullptr;
    if (bytes == 0) bytes = 4;  // a valid, distinct pointer even for empty tensors
    SO_HIP(hipSetDevice(ctx->device));
    SO_HIP(hipMalloc(dptr, bytes));
    return SO_OK;
}

extern "C" so_status so_free(so_ctx *ctx, void *dptr)
{
    SO_REQUIRE(ctx != nullptr, "so_free: ctx is null");
    if (!dptr) return SO_OK;
    SO_REQUIRE(!ctx->capturing, "so_free: not allowed while a graph is being recorded");
    SO_HIP(hipStreamSynchronize(ctx->stream));
    SO_HIP(hipFree(dptr));
    return SO_OK;
}

extern "C" so_status so_h2d(so_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    SO_REQUIRE(ctx != nullptr, "so_h2d: ctx is null");
    if (bytes == 0) return SO_OK;
    SO_REQUIRE(dst && src, "so_h2d: null pointer");
    SO_REQUIRE(!ctx->capturing, "so_h2d: not allowed while a graph is being recorded");
    SO_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    return so_stream_wait(ctx, "so_h2d");
}

extern "C" so_status so_d2h(so_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    SO_REQUIRE(ctx != nullptr, "so_d2h: ctx is null");
    if (bytes == 0) return SO_OK;
    SO_REQUIRE(dst && src, "so_d2h: null pointer");
    SO_REQUIRE(!ctx->capturing, "so_d2h: not allowed while a graph is being recorded");
    SO_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    return so_stream_wait(ctx, "so_d2h");
}

extern "C" so_status so_d2d(so_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    SO_REQUIRE(ctx != nullptr, "so_d2d: ctx is null");
    if (bytes == 0) return SO_OK;
    SO_REQUIRE(dst && src, "so_d2d: null pointer");
    SO_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return SO_OK;
}

__global__ void so_fill_zero_kernel(uint32_t *p, size_t words)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < words; i += stride) p[i] = 0u;
}

extern "C" so_status so_fill_zero(so_ctx *ctx, void *dptr, size_t bytes)
{
    SO_REQUIRE(ctx != nullptr, "so_fill_zero: ctx is null");
    if (bytes == 0) return SO_OK;
    SO_REQUIRE(dptr != nullptr && bytes % 4 == 0 && ((uintptr_t)dptr & 3) == 0,
               "so_fill_zero: pointer and size must be 4-byte multiples");
    const size_t words = bytes / 4;
    const uint32_t blocks = (uint32_t)std::min<size_t>((words + 255) / 256, 4096);
    so_fill_zero_kernel<<<blocks, 256, 0, ctx->stream>>>((uint32_t *)dptr, words);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

extern "C" so_status so_sync(so_ctx *ctx)
{
    SO_REQUIRE(ctx != nullptr, "so_sync: ctx is null");
    SO_REQUIRE(!ctx->capturing, "so_sync: not allowed while a graph is being recorded");
    // a kernel whose waves gave up waiting for one another has produced garbage: say so
    return so_stream_wait(ctx, "so_sync");
}

extern "C" so_status so_timer_begin(so_ctx *ctx)
{
    SO_REQUIRE(ctx != nullptr, "so_timer_begin: ctx is null");
    SO_REQUIRE(!ctx->capturing, "so_timer_begin: not allowed while a graph is being recorded");
    SO_HIP(hipEventRecord(ctx->ev0, ctx->stream));
    return SO_OK;
}

extern "C" so_status so_timer_end(so_ctx *ctx, float *ms)
{
    SO_REQUIRE(ctx && ms, "so_timer_end: null argument");
    SO_REQUIRE(!ctx->capturing, "so_timer_end: not allowed while a graph is being recorded");
    SO_HIP(hipEventRecord(ctx->ev1, ctx->stream));
    const so_status s = so_stream_wait(ctx, "so_timer_end");
    SO_HIP(hipEventElapsedTime(ms, ctx->ev0, ctx->ev1));
    return s;
}

// ---------------------------------------------------------------- launch graphs

extern "C" so_status so_graph_begin(so_ctx *ctx)
{
    SO_REQUIRE(ctx != nullptr, "so_graph_begin: ctx is null");
    SO_REQUIRE(!ctx->capturing, "so_graph_begin: already recording");
    SO_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return SO_OK;
}

extern "C" so_status so_graph_end(so_ctx *ctx, so_graph **out)
{
    SO_REQUIRE(ctx && out, "so_graph_end: null argument");
    SO_REQUIRE(ctx->capturing, "so_graph_end: not recording");
    *out = nullptr;
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    SO_HIP(hipStreamEndCapture(ctx->stream, &graph));
    so_graph *g = new (std::nothrow) so_graph();
    if (!g) { (void)hipGraphDestroy(graph); so_set_error("so_graph_end: host allocation failed"); return SO_ERR_OOM; }
    g->graph = graph;
    hipError_t e = hipGraphInstantiate(&g->exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        so_set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
        (void)hipGraphDestroy(graph);
        delete g;
        return SO_ERR_HIP;
    }
    *out = g;
    return SO_OK;
}

extern "C" so_status so_graph_launch(so_ctx *ctx, so_graph *g)
{
    SO_REQUIRE(ctx && g && g->exec, "so_graph_launch: null argument");
    SO_REQUIRE(!ctx->capturing, "so_graph_launch: not allowed while recording");
    SO_HIP(hipGraphLaunch(g->exec, ctx->stream));
    ctx->waits_pending = true;          // the graph may hold kernels with bounded waits
    return SO_OK;
}

extern "C" so_status so_graph_free(so_ctx *ctx, so_graph *g)
{
    if (!g) return SO_OK;
    if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
    return SO_OK;
}

// ------------------------------------------------------------ ELLPACK on device

static void free_ellpack_arrays(so_ellpack *E)
{
    if (E->d_Wd) (void)hipFree(E->d_Wd);
    if (E->d_idx) (void)hipFree(E->d_idx);
    if (E->d_nnz) (void)hipFree(E->d_nnz);
    if (E->d_WdT) (void)hipFree(E->d_WdT);
    if (E->d_idxT) (void)hipFree(E->d_idxT);
    if (E->d_idx16) (void)hipFree(E->d_idx16);
    if (E->d_idxT16) (void)hipFree(E->d_idxT16);
    for (auto &b : E->bins)
        if (b.d_rows) (void)hipFree(b.d_rows);
    if (E->tiled.d_entries) (void)hipFree(E->tiled.d_entries);
    if (E->tiled.d_info) (void)hipFree(E->tiled.d_info);
    if (E->tiled.d_rows) (void)hipFree(E->tiled.d_rows);
    so_rbmm_free(E);
}

// Device copy of a host array with 16 zeroed bytes after the last element, so a
// kernel may read whole aligned 16-byte groups that straddle the end.
template <typename T>
static so_status upload_array(so_ctx *ctx, const T *host, size_t count, T **dev)
{
    void *p = nullptr;
    so_status s = so_malloc(ctx, count * sizeof(T) + 16, &p);
    if (s != SO_OK) return s;
    *dev = (T *)p;
    SO_HIP(hipMemsetAsync((char *)p + count * sizeof(T), 0, 16, ctx->stream));
    return so_h2d(ctx, p, host, count * sizeof(T));
}

// K-tiled layout for the LDS-staged matmul (see so_tiled).  Rows are first ordered
// by stored-nonzero count (longest first, stable; over the whole matrix or inside
// each workgroup's block of 64 rows, see below) so that the four rows sharing a
// wavefront have similar lengths; the order only decides which rows share a wave,
// every row is still written to its own place in Y.
static so_status build_tiled(so_ctx *ctx, so_ellpack *E, const float *Wd, const uint32_t *idx, const uint32_t *nnz)
{
    const uint32_t m = E->m, n = E->n, r = E->r;
    constexpr uint32_t KT = so_tiled::kTileRows, ROWB = so_tiled::kSlabCols * 4;
    so_tiled &T = E->tiled;
    T.nquads = (m + 3) / 4;
    T.ntiles = std::max(1u, (n + KT - 1) / KT);
    // Two candidate orders: sorted by length over the whole matrix, or only inside blocks of 64
    // consecutive rows (the rows of one workgroup).  The second keeps a workgroup's rows of Y next
    // to each other, which is worth ~5 % of a launch; the first is needed when lengths vary so
    // much that rows of one block do not fit together.  Take the block-wise order unless the
    // global one saves more than 2 % of the steps.
    const auto longer_first = [&](uint32_t a, uint32_t b) { return nnz[a] > nnz[b]; };
    std::vector<uint32_t> order(m), blockwise(m);
    for (uint32_t i = 0; i < m; ++i) order[i] = blockwise[i] = i;
    std::stable_sort(order.begin(), order.end(), longer_first);
    for (uint32_t b0 = 0; b0 < m; b0 += 64)
        std::stable_sort(blockwise.begin() + b0, blockwise.begin() + std::min(m, b0 + 64), longer_first);
    if ((uint64_t)m * T.ntiles <= (1ull << 28)) {                     // the comparison needs 2 bytes per (row, tile)
        std::vector<uint16_t> per_tile((size_t)m * T.ntiles, 0);      // a tile has at most 256 columns
        for (uint32_t i = 0; i < m; ++i)
            for (uint32_t k = 0; k < nnz[i]; ++k) ++per_tile[(size_t)i * T.ntiles + idx[(size_t)i * r + k] / KT];
        const auto steps_of = [&](const std::vector<uint32_t> &ord) {
            uint64_t total = 0;
            for (uint32_t q0 = 0; q0 < m; q0 += 4)
                for (uint32_t t = 0; t < T.ntiles; ++t) {
                    uint32_t most = 0;
                    for (uint32_t g = q0; g < std::min(m, q0 + 4); ++g) most = std::max<uint32_t>(most, per_tile[(size_t)ord[g] * T.ntiles + t]);
                    total += (most + 3u) & ~3u;
                }
            return total;
        };
        if (steps_of(blockwise) * 100 <= steps_of(order) * 102) order.swap(blockwise);
    }
    std::vector<uint32_t> qrows((size_t)T.nquads * 4, 0xffffffffu);
    for (uint32_t i = 0; i < m; ++i) qrows[i] = order[i];

    std::vector<so_tile_info> info((size_t)T.nquads * T.ntiles);
    std::vector<so_tile_entry> entries;
    entries.reserve((size_t)E->total_nnz + (size_t)E->total_nnz / 3 + 256);
    uint64_t total_steps = 0;
    for (uint32_t q = 0; q < T.nquads; ++q) {
        uint32_t pos[4] = {0, 0, 0, 0};
        for (uint32_t t = 0; t < T.ntiles; ++t) {
            const uint64_t col_end = (uint64_t)(t + 1) * KT;
            uint32_t cnt[4] = {0, 0, 0, 0}, steps = 0;
            for (int g = 0; g < 4; ++g) {
                const uint32_t row = qrows[(size_t)q * 4 + g];
                if (row == 0xffffffffu) continue;
                const uint32_t *c = idx + (size_t)row * r;
                uint32_t p = pos[g];
                while (p < nnz[row] && c[p] < col_end) ++p;
                cnt[g] = p - pos[g];
                steps = std::max(steps, cnt[g]);
            }
            steps = (steps + 3u) & ~3u;
            if (entries.size() / 64 > 0xfffffff0ull) { so_set_error("so_ellpack_upload: matrix too large for the tiled layout"); return SO_ERR_INVALID; }
            info[(size_t)q * T.ntiles + t] = so_tile_info{(uint32_t)(entries.size() / 64), steps};
            total_steps += steps;
            // The zero row sits after both tile buffers; offsets are relative to the buffer the tile uses.
            // A padding step is fma(-0, +0, acc): adding -0 leaves every accumulator, -0 included, as it is.
            const uint32_t zero_off = so_tiled::kZeroRowOff - (t & 1u) * so_tiled::kTileBytes;
            const uint32_t nch = (steps + 15) / 16;
            for (uint32_t ch = 0; ch < nch; ++ch)
                for (int g = 0; g < 4; ++g) {
                    const uint32_t row = qrows[(size_t)q * 4 + g];
                    for (uint32_t k = 0; k < 16; ++k) {
                        const uint32_t sidx = ch * 16 + k;
                        so_tile_entry e{-0.0f, zero_off};
                        if (sidx < cnt[g]) {
                            const size_t slot = (size_t)row * r + pos[g] + sidx;
                            e.w = Wd[slot];
                            e.off = (idx[slot] - t * KT) * ROWB;
                        }
                        entries.push_back(e);
                    }
                }
            for (int g = 0; g < 4; ++g) pos[g] += cnt[g];
        }
    }
    // Three zero chunks of slack: the kernel always fetches three chunks per tile.
    entries.resize(entries.size() + 3 * 64, so_tile_entry{-0.0f, so_tiled::kZeroRowOff});
    T.total_steps = total_steps;
    so_status s = upload_array(ctx, entries.data(), entries.size(), &T.d_entries);
    if (s == SO_OK) s = upload_array(ctx, info.data(), info.size(), &T.d_info);
    if (s == SO_OK) s = upload_array(ctx, qrows.data(), qrows.size(), &T.d_rows);
    return s;
}

extern "C" so_status so_ellpack_upload(so_ctx *ctx, const float *Wd, const uint32_t *idx,
                                       const uint32_t *nnz, uint32_t m, uint32_t n, uint32_t r,
                                       int layouts, so_ellpack **out)
{
    SO_REQUIRE(ctx && out, "so_ellpack_upload: null argument");
    *out = nullptr;
    const size_t slots = (size_t)m * r;
    SO_REQUIRE(m == 0 || nnz != nullptr, "so_ellpack_upload: nnz is null");
    SO_REQUIRE(slots == 0 || (Wd && idx), "so_ellpack_upload: Wd/idx is null");
    SO_REQUIRE((layouts & ~(SO_LAYOUT_ROW | SO_LAYOUT_SLOT | SO_LAYOUT_BINS | SO_LAYOUT_TILED | SO_LAYOUT_RBM | SO_LAYOUT_IDX16)) == 0,
               "so_ellpack_upload: unknown layout bits 0x%x", layouts);
    SO_REQUIRE(!(layouts & SO_LAYOUT_IDX16) || n <= 65536u, "so_ellpack_upload: 16-bit columns need n <= 65536 (n = %u)", n);

    // Validate on the host before anything reaches a kernel: every stored slot must
    // name a column inside X, every count must fit the row.
    // The encoder stores a row's columns in strictly ascending order and the K-tiled matmul layout
    // and the convolution's windowed layout walk a row on that assumption; a matrix filled in by
    // hand in any other order (the reference's kernels take slots in whatever order they come) is
    // served by the kernels that do the same, and the ordered layouts are not built for it.
    uint64_t total = 0;
    uint32_t max_nnz = 0;
    bool ascending = true;
    for (uint32_t i = 0; i < m; ++i) {
        const uint32_t c = nnz[i];
        if (c > r) {
            so_set_error("so_ellpack_upload: nnz[%u] = %u exceeds r = %u", i, c, r);
            return SO_ERR_BOUNDS;
        }
        const uint32_t *row = idx + (size_t)i * r;
        for (uint32_t k = 0; k < c; ++k) {
            if (row[k] >= n) {
                so_set_error("so_ellpack_upload: idx[%u,%u] = %u is not below n = %u", i, k, row[k], n);
                return SO_ERR_BOUNDS;
            }
            if (k > 0 && row[k] <= row[k - 1]) ascending = false;
        }
        total += c;
        max_nnz = std::max(max_nnz, c);
    }

    so_ellpack *E = new (std::nothrow) so_ellpack();
    if (!E) { so_set_error("so_ellpack_upload: host allocation failed"); return SO_ERR_OOM; }
    E->m = m; E->n = n; E->r = r;
    E->total_nnz = total;
    E->max_nnz = max_nnz;
    E->ascending = ascending;
    if (!ascending) layouts &= ~SO_LAYOUT_TILED;
    E->layouts = layouts | SO_LAYOUT_ROW;

    so_status s = upload_array(ctx, Wd, slots, &E->d_Wd);
    if (s == SO_OK) s = upload_array(ctx, idx, slots, &E->d_idx);
    if (s == SO_OK) s = upload_array(ctx, nnz, (size_t)m, &E->d_nnz);

    if (s == SO_OK && (layouts & SO_LAYOUT_SLOT)) {
        std::vector<float> WdT(slots);
        std::vector<uint32_t> idxT(slots);
        for (uint32_t i = 0; i < m; ++i)
            for (uint32_t k = 0; k < r; ++k) {
                WdT[(size_t)k * m + i] = Wd[(size_t)i * r + k];
                idxT[(size_t)k * m + i] = idx[(size_t)i * r + k];
            }
        s = upload_array(ctx, WdT.data(), slots, &E->d_WdT);
        if (s == SO_OK) s = upload_array(ctx, idxT.data(), slots, &E->d_idxT);
        if (s == SO_OK && (layouts & SO_LAYOUT_IDX16)) {
            std::vector<uint16_t> idxT16(slots);
            for (size_t k = 0; k < slots; ++k) idxT16[k] = (uint16_t)idxT[k];
            s = upload_array(ctx, idxT16.data(), slots, &E->d_idxT16);
        }
    }

    if (s == SO_OK && (layouts & SO_LAYOUT_IDX16)) {
        // The same slots as d_idx, two bytes each: so_matvec streams 6 bytes per nonzero instead of 8.
        // Padding slots keep the low half of whatever they hold; no kernel uses them.
        std::vector<uint16_t> idx16(slots);
        for (size_t k = 0; k < slots; ++k) idx16[k] = (uint16_t)idx[k];
        s = upload_array(ctx, idx16.data(), slots, &E->d_idx16);
    }

    if (s == SO_OK && (layouts & SO_LAYOUT_BINS)) {
        // Length classes: <= 16 nonzeros -> 4 lanes per row, <= 128 -> 16 lanes, <= 4096 -> a whole
        // wave, longer -> a whole workgroup (a single wave would walk such a row long after every
        // other row is done).  Long rows first inside a class, so the last waves to start are the
        // short ones.
        static const uint32_t group[4] = {4, 16, 64, 1024};
        static const uint32_t limit[4] = {16, 128, 4096, 0xffffffffu};
        std::vector<uint32_t> rows[4];
        for (uint32_t i = 0; i < m; ++i) {
            int b = 0;
            while (nnz[i] > limit[b]) ++b;
            rows[b].push_back(i);
        }
        for (int b = 0; b < 4 && s == SO_OK; ++b) {
            std::stable_sort(rows[b].begin(), rows[b].end(),
                             [&](uint32_t a, uint32_t c) { return nnz[a] > nnz[c]; });
            E->bins[b].group = group[b];
            E->bins[b].count = (uint32_t)rows[b].size();
            // (row, its length) pairs: a wave learns where its row is and how long in one load
            std::vector<uint32_t> pairs(2 * rows[b].size());
            for (size_t k = 0; k < rows[b].size(); ++k) {
                pairs[2 * k] = rows[b][k];
                pairs[2 * k + 1] = nnz[rows[b][k]];
            }
            if (!pairs.empty()) s = upload_array(ctx, pairs.data(), pairs.size(), &E->bins[b].d_rows);
        }
    }

    if (s == SO_OK && (layouts & SO_LAYOUT_TILED) && m > 0) s = build_tiled(ctx, E, Wd, idx, nnz);
    if (s == SO_OK && (layouts & SO_LAYOUT_RBM) && m > 0) s = so_rbmm_build(ctx, E, Wd, idx, nnz);

    if (s != SO_OK) {
        free_ellpack_arrays(E);
        delete E;
        return s;
    }
    *out = E;
    return SO_OK;
}

extern "C" so_status so_ellpack_free(so_ctx *ctx, so_ellpack *E)
{
    if (!E) return SO_OK;
    if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    free_ellpack_arrays(E);
    delete E;
    return SO_OK;
}

extern "C" so_status so_ellpack_dims(const so_ellpack *E, uint32_t *m, uint32_t *n, uint32_t *r,
                                     uint64_t *total_nnz, int *layouts)
{
    SO_REQUIRE(E != nullptr, "so_ellpack_dims: E is null");
    if (m) *m = E->m;
    if (n) *n = E->n;
    if (r) *r = E->r;
    if (total_nnz) *total_nnz = E->total_nnz;
    if (layouts) *layouts = E->layouts;
    return SO_OK;
}

namespace {

// One wave per row: its stored nonzeros go to their columns (ascending, distinct, so no two
// lanes write the same element).
__global__ __launch_bounds__(256)
void ellpack_decode_kernel(const float *__restrict__ Wd, const uint32_t *__restrict__ idx,
                           const uint32_t *__restrict__ nnz, uint32_t m, uint32_t n, uint32_t r,
                           float *__restrict__ W)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t nwaves = gridDim.x * 4u;
    for (uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6); row < m; row += nwaves) {
        const uint32_t cnt = nnz[row];
        for (uint32_t k = lane; k < cnt; k += 64u)
            W[(size_t)row * n + idx[(size_t)row * r + k]] = Wd[(size_t)row * r + k];
    }
}

} // namespace

namespace {

// The encoder's counting pass leaves one partial result per workgroup -- the longest row and the
// number of nonzeros among the workgroup's kEncodeRowsPerBlock rows -- in a scratch buffer; a
// one-workgroup pass folds them into the buffer's header {r, total nnz (low, high), 0}, which the
// packing pass reads on the device, so the row pitch of the output never travels through the host.
// Layout of the scratch buffer: header (kEncodeHeaderBytes), then one uint2 {max, sum} per workgroup.
constexpr uint32_t kEncodeRowsPerBlock = 16;      // 4 waves x 4 rows
constexpr uint32_t kEncodeMaxBlocks = 65536;      // workgroups whose partials the static scratch array holds
constexpr uint32_t kEncodeHeaderBytes = 256;
constexpr uint32_t kEncodeMaxCols = (1u << 28) - 1;     // the 16 rows of a workgroup, all dense, still count in 32 bits
constexpr size_t kEncodeScratchBytes = kEncodeHeaderBytes + (size_t)kEncodeMaxBlocks * sizeof(uint2);
static_assert(kEncodeScratchBytes <= kStaticScratchBytes, "the static scratch array holds the encoder's partials");

static size_t encode_scratch_bytes(uint32_t m)
{
    return kEncodeHeaderBytes + (size_t)so_ceil_div(m, kEncodeRowsPerBlock) * sizeof(uint2);
}

// Pass 1: one wave per row counts the entries with v != 0.0f; the workgroup's maximum and sum go
// to partial[blockIdx.x].
__global__ __launch_bounds__(256)
void ellpack_count_kernel(const float *__restrict__ W, uint32_t m, uint32_t n, uint32_t *__restrict__ nnz,
                          uint2 *__restrict__ partial)
{
    __shared__ uint32_t wmax[4], wsum[4];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t vmax = 0, vsum = 0;
    for (uint32_t k = 0; k < kEncodeRowsPerBlock / 4u; ++k) {
        const uint32_t row = blockIdx.x * kEncodeRowsPerBlock + k * 4u + wave;
        if (row >= m) break;
        const float *wr = W + (size_t)row * n;
        uint32_t c = 0;
        for (uint32_t j = lane; j < n; j += 64u) c += wr[j] != 0.0f ? 1u : 0u;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, 64);
        if (lane == 0) nnz[row] = c;
        vmax = max(vmax, c);
        vsum += c;
    }
    if (lane == 0) { wmax[wave] = vmax; wsum[wave] = vsum; }
    __syncthreads();
    if (threadIdx.x == 0)
        partial[blockIdx.x] = make_uint2(max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3])),
                                         wsum[0] + wsum[1] + wsum[2] + wsum[3]);
}

// Folds the partials into header = {r, total nnz low word, high word, 0}.  One workgroup.
__global__ __launch_bounds__(1024)
void ellpack_count_fold_kernel(const uint2 *__restrict__ partial, uint32_t nblocks, uint32_t *__restrict__ header)
{
    __shared__ uint32_t smax[16];
    __shared__ unsigned long long ssum[16];
    uint32_t vmax = 0;
    unsigned long long vsum = 0;
    for (uint32_t i = threadIdx.x; i < nblocks; i += 1024u) {
        const uint2 p = partial[i];
        vmax = max(vmax, p.x);
        vsum += p.y;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        vmax = max(vmax, (uint32_t)__shfl_xor(vmax, off, 64));
        vsum += __shfl_xor(vsum, off, 64);
    }
    if ((threadIdx.x & 63u) == 0) { smax[threadIdx.x >> 6] = vmax; ssum[threadIdx.x >> 6] = vsum; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w) { vmax = max(vmax, smax[w]); vsum += ssum[w]; }
        header[0] = vmax;
        header[1] = (uint32_t)vsum;
        header[2] = (uint32_t)(vsum >> 32);
        header[3] = 0u;
    }
}

// Pass 2: one wave per row packs (value, column) in ascending column order with row pitch
// r = header[0], then zero-fills the row's remaining slots.  For each group of 64 columns the lanes
// that hold a nonzero get consecutive slots (a prefix count over the wave's ballot), so the order
// inside the row is the column order.  Writes nothing when r exceeds r_cap (the caller's arrays
// hold m * r_cap slots); the wave that owns the last row also clears `tail_words` words after the
// arrays' last slot.
__global__ __launch_bounds__(256)
void ellpack_pack_kernel(const float *__restrict__ W, uint32_t m, uint32_t n, const uint32_t *__restrict__ header,
                         uint32_t r_cap, const uint32_t *__restrict__ nnz, float *__restrict__ Wd,
                         uint32_t *__restrict__ idx, uint32_t tail_words)
{
    const uint32_t r = header[0];
    if (r > r_cap) return;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t nwaves = gridDim.x * 4u;
    for (uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6); row < m; row += nwaves) {
        const float *wr = W + (size_t)row * n;
        float *wd = Wd + (size_t)row * r;
        uint32_t *ix = idx + (size_t)row * r;
        uint32_t base = 0;
        for (uint32_t j0 = 0; j0 < n; j0 += 64u) {
            const uint32_t j = j0 + lane;
            const float v = j < n ? wr[j] : 0.0f;
            const bool keep = v != 0.0f;
            const uint64_t mask = __ballot(keep);
            if (keep) {
                const uint32_t pos = base + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
                wd[pos] = v;
                ix[pos] = j;
            }
            base += (uint32_t)__popcll(mask);
        }
        const uint32_t end = row + 1 == m ? r + tail_words : r;
        for (uint32_t k = nnz[row] + lane; k < end; k += 64u) { wd[k] = 0.0f; ix[k] = 0u; }
    }
}

// The three passes on the context's stream.  `scratch` holds encode_scratch_bytes(m) bytes; dWd and
// dIdx hold m * r_cap slots (+ tail_words).
so_status encode_launch(so_ctx *ctx, const float *dDense, uint32_t m, uint32_t n, void *scratch, uint32_t r_cap,
                        uint32_t *dNnz, float *dWd, uint32_t *dIdx, uint32_t tail_words, bool count, bool pack)
{
    uint32_t *header = (uint32_t *)scratch;
    uint2 *partial = (uint2 *)((char *)scratch + kEncodeHeaderBytes);
    const uint32_t nblocks = so_ceil_div(m, kEncodeRowsPerBlock);
    if (count) {
        if (nblocks) {
            ellpack_count_kernel<<<nblocks, 256, 0, ctx->stream>>>(dDense, m, n, dNnz, partial);
            SO_LAUNCH_CHECK();
        }
        ellpack_count_fold_kernel<<<1, 1024, 0, ctx->stream>>>(partial, nblocks, header);
        SO_LAUNCH_CHECK();
    }
    if (pack && m) {
        const uint32_t blocks = std::max(1u, std::min(so_ceil_div(m, 4u), 16u * (uint32_t)ctx->compute_units));
        ellpack_pack_kernel<<<blocks, 256, 0, ctx->stream>>>(dDense, m, n, header, r_cap, dNnz, dWd, dIdx, tail_words);
        SO_LAUNCH_CHECK();
    }
    return SO_OK;
}

} // namespace

extern "C" so_status so_ellpack_encode(so_ctx *ctx, const float *dDense, uint32_t m, uint32_t n, so_ellpack **out)
{
    SO_REQUIRE(ctx && out, "so_ellpack_encode: null argument");
    *out = nullptr;
    SO_REQUIRE(dDense != nullptr || (uint64_t)m * n == 0, "so_ellpack_encode: null matrix");
    SO_REQUIRE(n <= kEncodeMaxCols, "so_ellpack_encode: at most %u columns", kEncodeMaxCols);
    so_ellpack *E = new (std::nothrow) so_ellpack();
    if (!E) { so_set_error("so_ellpack_encode: host allocation failed"); return SO_ERR_OOM; }
    E->m = m; E->n = n;
    E->layouts = SO_LAYOUT_ROW;
    void *p = nullptr, *scratch = nullptr;
    uint32_t header[4] = {0, 0, 0, 0};
    so_status s = so_malloc(ctx, (size_t)m * sizeof(uint32_t) + 16, &p);
    if (s == SO_OK) { E->d_nnz = (uint32_t *)p; s = so_fill_zero(ctx, (char *)p + (size_t)m * sizeof(uint32_t), 16); }
    if (s == SO_OK) s = so_malloc(ctx, encode_scratch_bytes(m), &scratch);
    if (s == SO_OK) s = encode_launch(ctx, dDense, m, n, scratch, 0, E->d_nnz, nullptr, nullptr, 0, true, false);
    if (s == SO_OK) s = so_d2h(ctx, header, scratch, sizeof header);
    if (s == SO_OK) {
        E->r = E->max_nnz = header[0];                   // r = longest row (src/ellpack_encoder.cpp:10-17)
        E->total_nnz = (uint64_t)header[1] | ((uint64_t)header[2] << 32);
        const size_t bytes = (size_t)m * E->r * sizeof(float) + 16;
        s = so_malloc(ctx, bytes, &p);
        if (s == SO_OK) { E->d_Wd = (float *)p; s = so_malloc(ctx, bytes, &p); }
        if (s == SO_OK) E->d_idx = (uint32_t *)p;
        if (s == SO_OK && (size_t)m * E->r == 0) {
            s = so_fill_zero(ctx, E->d_Wd, 16);
            if (s == SO_OK) s = so_fill_zero(ctx, E->d_idx, 16);
        }
    }
    if (s == SO_OK && (size_t)m * E->r != 0)
        s = encode_launch(ctx, dDense, m, n, scratch, E->r, E->d_nnz, E->d_Wd, E->d_idx, 4, false, true);
    if (scratch) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(scratch);
    }
    if (s != SO_OK) {
        (void)so_ellpack_free(ctx, E);
        return s;
    }
    *out = E;
    return SO_OK;
}

extern "C" so_status so_ellpack_encode_noalloc(so_ctx *ctx, const float *dDense, uint32_t m, uint32_t n, uint32_t r_cap,
                                              float *dWd, uint32_t *dIdx, uint32_t *dNnz, uint32_t *r_out,
                                              uint64_t *total_nnz_out)
{
    SO_REQUIRE(ctx != nullptr, "so_ellpack_encode_noalloc: ctx is null");
    SO_REQUIRE(dDense != nullptr || (uint64_t)m * n == 0, "so_ellpack_encode_noalloc: null matrix");
    SO_REQUIRE(n <= kEncodeMaxCols, "so_ellpack_encode_noalloc: at most %u columns", kEncodeMaxCols);
    SO_REQUIRE(so_ceil_div(m, kEncodeRowsPerBlock) <= kEncodeMaxBlocks,
               "so_ellpack_encode_noalloc: %u rows need %u partial results, the static scratch array holds %u (at most %u rows)",
               m, so_ceil_div(m, kEncodeRowsPerBlock), kEncodeMaxBlocks, kEncodeMaxBlocks * kEncodeRowsPerBlock);
    SO_REQUIRE(m == 0 || dNnz != nullptr, "so_ellpack_encode_noalloc: dNnz is null");
    SO_REQUIRE((uint64_t)m * r_cap == 0 || (dWd != nullptr && dIdx != nullptr), "so_ellpack_encode_noalloc: dWd/dIdx is null");
    SO_REQUIRE(ctx->static_scratch != nullptr, "so_ellpack_encode_noalloc: the context has no scratch address");
    const so_status s = encode_launch(ctx, dDense, m, n, ctx->static_scratch, r_cap, dNnz, dWd, dIdx, 0, true,
                                      (uint64_t)m * r_cap != 0);
    if (s != SO_OK || (!r_out && !total_nnz_out)) return s;
    SO_REQUIRE(!ctx->capturing, "so_ellpack_encode_noalloc: r_out/total_nnz_out need a wait, which a graph recording forbids");
    uint32_t header[4] = {0, 0, 0, 0};
    SO_HIP(hipMemcpyAsync(header, ctx->static_scratch, sizeof header, hipMemcpyDeviceToHost, ctx->stream));
    const so_status waited = so_stream_wait(ctx, "so_ellpack_encode_noalloc");
    if (waited != SO_OK) return waited;
    if (r_out) *r_out = header[0];
    if (total_nnz_out) *total_nnz_out = (uint64_t)header[1] | ((uint64_t)header[2] << 32);
    SO_REQUIRE(header[0] <= r_cap, "so_ellpack_encode_noalloc: the longest row has %u nonzeros, dWd/dIdx hold %u per row (nothing was packed)",
               header[0], r_cap);
    return SO_OK;
}

extern "C" so_status so_ellpack_decode(so_ctx *ctx, const so_ellpack *E, float *dDense)
{
    SO_REQUIRE(ctx && E, "so_ellpack_decode: null argument");
    const size_t total = (size_t)E->m * E->n;
    if (total == 0) return SO_OK;
    SO_REQUIRE(dDense != nullptr, "so_ellpack_decode: null output");
    so_status s = so_fill_zero(ctx, dDense, total * sizeof(float));
    if (s != SO_OK) return s;
    if (E->r == 0) return SO_OK;
    const uint32_t blocks = std::max(1u, std::min(so_ceil_div(E->m, 4u), 16u * (uint32_t)ctx->compute_units));
    ellpack_decode_kernel<<<blocks, 256, 0, ctx->stream>>>(E->d_Wd, E->d_idx, E->d_nnz, E->m, E->n, E->r, dDense);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

extern "C" so_status so_ellpack_download(so_ctx *ctx, const so_ellpack *E, int layout,
                                         float *Wd, uint32_t *idx, uint32_t *nnz)
{
    SO_REQUIRE(ctx && E, "so_ellpack_download: null argument");
    SO_REQUIRE(layout == SO_LAYOUT_ROW || layout == SO_LAYOUT_SLOT,
               "so_ellpack_download: layout must be ROW or SLOT");
    SO_REQUIRE((E->layouts & layout) != 0, "so_ellpack_download: layout %d was not uploaded", layout);
    const size_t slots = (size_t)E->m * E->r;
    const float *w = layout == SO_LAYOUT_ROW ? E->d_Wd : E->d_WdT;
    const uint32_t *ix = layout == SO_LAYOUT_ROW ? E->d_idx : E->d_idxT;
    so_status s = SO_OK;
    if (Wd && slots) s = so_d2h(ctx, Wd, w, slots * sizeof(float));
    if (s == SO_OK && idx && slots) s = so_d2h(ctx, idx, ix, slots * sizeof(uint32_t));
    if (s == SO_OK && nnz && E->m) s = so_d2h(ctx, nnz, E->d_nnz, (size_t)E->m * sizeof(uint32_t));
    return s;
}
