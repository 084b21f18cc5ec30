// Internal definitions shared by the HIP translation units of libsparseops_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "sparseops_hip.h"

// Tuning overrides, read from the environment when the context is created (and again by
// so_tuning_reload), never per launch.  0 / -1 = the library's own choice.
struct so_tuning {
    int matmul_tiled = -1;   // SPARSEOPS_MATMUL_TILED: 1 forces the LDS-staged kernel, 0 forbids it
    int matmul_vec = 0;      // SPARSEOPS_MATMUL_VEC: 1 or 2 columns per lane at most
    int matmul_share = -1;   // SPARSEOPS_MATMUL_SHARE: 0 forbids the shared-gather kernel for few-row launches
    int matmul_rbm = -1;     // SPARSEOPS_MATMUL_RBM: 0 forbids the row-block-merged kernel on handles that carry its layout, 1 forces it
    int matmul_rbm_split = 0;   // SPARSEOPS_MATMUL_RBM_SPLIT: 1, 2 or 4 workgroups per tile for RBM layouts built from now on
    int matvec_lanes = 0;    // SPARSEOPS_MATVEC_LANES: 8, 16, 32 or 64 lanes per row
    int matvec_idx16 = -1;   // SPARSEOPS_MATVEC_IDX16: 0 keeps so_matvec on the 32-bit columns of a handle that has both
    int conv_min_cg = 0;     // SPARSEOPS_CONV_MIN_CG: fewest channel groups per workgroup a small grid may shrink to (16: never shrink)
    int conv_window = -1;    // SPARSEOPS_CONV_WINDOW: 1 forces the LDS-windowed kernel, 0 forbids it
    int conv_cpw = 0;        // SPARSEOPS_CONV_CPW: most output channels per wave
    int conv_tilepx = 0;     // SPARSEOPS_CONV_TILEPX: most output pixels per tile
    int conv_vec = 0;        // SPARSEOPS_CONV_VEC: most batch entries per lane in the gather kernel
    int wait_spins = -1;     // SPARSEOPS_WAIT_SPINS: most polls of a bounded wait on LDS progress counters (0: every wait gives up at once; tests)
    int conv_rbm = -1;       // SPARSEOPS_CONV_RBM: 0 forbids the row-block-merged kernel on plans that carry its streams
};

struct so_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    int compute_units = 0;
    int max_lds_bytes = 0;   // largest LDS allocation one workgroup may ask for
    bool capturing = false;
    void *static_scratch = nullptr;   // this device's address of the library's static scratch array (so_ellpack_encode_noalloc)
    // workspace of the row-block-merged matmul (csrc/matmul_rbm.hip): partial tiles of the workgroups that share a tile, a counter per tile
    // Bounded waits (csrc/lds_sync.h): a device word in which waves that gave up count themselves, its pinned
    // host copy, and whether a kernel that waits that way has been launched since the word was last looked at.
    uint32_t *d_wait_gave_up = nullptr;
    uint32_t *h_wait_gave_up = nullptr;
    bool waits_pending = false;
    float *mm_part = nullptr;
    size_t mm_part_bytes = 0;
    uint32_t *mm_counters = nullptr;
    size_t mm_counter_bytes = 0;
    std::string name;
    so_tuning tune;
    std::vector<const void *> big_lds_kernels;   // kernels already allowed max_lds_bytes of dynamic LDS on this device
};

// Rows of one length class for the binned matvec: `group` lanes cooperate on a row.
struct so_bin {
    uint32_t group = 0;      // 4, 16 or 64 lanes per row, 1024: a whole workgroup
    uint32_t count = 0;      // rows in this class
    uint32_t *d_rows = nullptr;   // count pairs (row, nonzeros of the row), longest rows first
};

// K-tiled copy of the matrix for the LDS-staged matmul.  Rows are grouped in
// quads (four rows share a wavefront, 16 lanes each); the dense operand is consumed
// in tiles of kTileRows rows.  For every (quad, tile) the nonzeros whose column
// falls in the tile are stored as "steps": step s holds one (weight, LDS byte
// offset of the X row inside the tile) pair per row of the quad, padded with
// (0, offset of a zero row) for rows that have fewer nonzeros in this tile.
// Steps are stored in chunks of 16: chunk[g][k] is the pair of row g for step k,
// so the 64 lanes of a wave fetch one chunk with a single coalesced 8-byte load.
struct so_tile_entry { float w; uint32_t off; };
struct so_tile_info { uint32_t chunk0; uint32_t steps; };   // steps is a multiple of 4
struct so_tiled {
    static constexpr uint32_t kTileRows = 256;   // X rows per LDS tile
    static constexpr uint32_t kWavesPerGroup = 16;   // quads (waves) per workgroup of the kernel
    static constexpr uint32_t kSlabCols = 64;    // dense columns per workgroup
    static constexpr uint32_t kTileBytes = kTileRows * kSlabCols * 4;
    static constexpr uint32_t kZeroRowOff = 2 * kTileBytes;      // after the two tile buffers
    static constexpr uint32_t kSyncOff = kZeroRowOff + kSlabCols * 4;    // the workgroup's progress counters (csrc/lds_sync.h)
    static constexpr uint32_t kLdsBytes = kSyncOff + 64;
    uint32_t nquads = 0, ntiles = 0;
    uint64_t total_steps = 0;
    so_tile_entry *d_entries = nullptr;   // [chunks + 3][64]
    so_tile_info *d_info = nullptr;       // [nquads][ntiles]
    uint32_t *d_rows = nullptr;           // [nquads*4] row id of each quad member (0xffffffff = none)
};

// Row-block-merged copy of the matrix for so_matmul (csrc/matmul_rbm.hip): per block of 128 rows and per
// stream (12 waves x ksplit workgroups) a run of 256-byte records, one per loop iteration, and at the same
// index of `w` the iteration's 64 weights.
struct so_rbmm {
    static constexpr uint32_t kBlockRows = 128;   // rows (accumulators) per tile
    static constexpr uint32_t kWaves = 12;        // waves per workgroup
    static constexpr uint32_t kMaxSplit = 4;      // most workgroups per tile
    uint32_t nb = 0, ksplit = 1;
    uint64_t nrec = 0;                            // records (= weight blocks), tails included
    uint64_t slots = 0, xloads = 0;               // multiply-adds a 64-column slab costs (padding included), X row segments it loads
    uint32_t *d_hdr = nullptr;                    // per block: iterations per class (6 dwords + 2 spare), then per stream {first record, first class}
    uint32_t *d_rec = nullptr;
    float *d_w = nullptr;
    uint32_t *d_xrows = nullptr;                  // [nrec][4]: the X rows of every record; the records hold row * pitch
    uint32_t pitch = 0;                           // row pitch of X (bytes) the records' offsets are written for; 0: none yet
};

struct so_ellpack {
    uint32_t m = 0, n = 0, r = 0;
    uint64_t total_nnz = 0;
    uint32_t max_nnz = 0;
    bool ascending = true;       // every row's stored columns are strictly ascending (what the encoder produces)
    int layouts = 0;
    float *d_Wd = nullptr;       // [m*r] row-major
    uint32_t *d_idx = nullptr;   // [m*r]
    uint32_t *d_nnz = nullptr;   // [m]
    float *d_WdT = nullptr;      // [r*m] slot-major (SO_LAYOUT_SLOT)
    uint32_t *d_idxT = nullptr;
    uint16_t *d_idx16 = nullptr; // [m*r] the columns of d_idx in 16 bits (SO_LAYOUT_IDX16, n <= 65536)
    uint16_t *d_idxT16 = nullptr;// [r*m] the same for d_idxT (SO_LAYOUT_SLOT with SO_LAYOUT_IDX16)
    so_bin bins[4];              // SO_LAYOUT_BINS
    so_tiled tiled;              // SO_LAYOUT_TILED
    so_rbmm rbmm;                // SO_LAYOUT_RBM
};

// Row-block-merged re-encoding of a matrix (include/rbm_conv.hpp:8-27 of the reference), flattened:
// block b holds rows [b*Ct_max, min(M, (b+1)*Ct_max)); its union columns are krel[block_union[b] ..
// block_union[b+1]) in ascending order; union column u owns the pairs colptr[u] .. colptr[u+1], each
// a (row inside the block, weight), rows ascending.  Kept on the host: convolution plans turn it
// into the record streams their kernel reads.
struct so_rbm {
    uint32_t M = 0, N = 0, Ct_max = 0, nblocks = 0;
    std::vector<uint32_t> block_union, krel, colptr;
    std::vector<uint16_t> pair_row;
    std::vector<float> pair_w;
};

struct so_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

void so_set_error(const char *fmt, ...);

// csrc/matmul_tiled.hip: launches the LDS-staged kernel on E's TILED copy (the caller has checked that it applies).
so_status so_matmul_tiled_launch(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C,
                                 const float *dBias, float *dY, int act);

// csrc/matmul_rbm.hip: the row-block-merged layout and its kernel.
so_status so_rbmm_build(so_ctx *ctx, so_ellpack *E, const float *Wd, const uint32_t *idx, const uint32_t *nnz);
void so_rbmm_free(so_ellpack *E);
bool so_matmul_rbm_applies(const so_ctx *ctx, const so_ellpack *E, uint32_t C);
so_status so_matmul_rbm_set_pitch(so_ctx *ctx, const so_ellpack *E, uint32_t C);
so_status so_matmul_rbm_reserve(so_ctx *ctx, const so_ellpack *E, uint32_t C);
so_status so_matmul_rbm_launch(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C,
                               const float *dBias, float *dY, int act);

// Waits for the context's stream and then reports, as SO_ERR_HIP, bounded waits that gave up in kernels launched
// since the last look (their results are invalid).  Every entry point that waits for the stream ends with this.
so_status so_stream_wait(so_ctx *ctx, const char *who);

// Kernels that ask for more than 48 KB of dynamic LDS must be told so once per device: this does
// it the first time `kernel` is seen on the context's device (hipSuccess when already done).
hipError_t so_allow_big_lds(so_ctx *ctx, const void *kernel);

#define SO_HIP(call)                                                              \
    do {                                                                          \
        hipError_t e_ = (call);                                                   \
        if (e_ != hipSuccess) {                                                   \
            so_set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_),   \
                         __FILE__, __LINE__);                                     \
            return e_ == hipErrorOutOfMemory ? SO_ERR_OOM : SO_ERR_HIP;           \
        }                                                                         \
    } while (0)

#define SO_REQUIRE(cond, ...)                                                     \
    do {                                                                          \
        if (!(cond)) {                                                            \
            so_set_error(__VA_ARGS__);                                            \
            return SO_ERR_INVALID;                                                \
        }                                                                         \
    } while (0)

// Launch check that is valid both eagerly and while a graph is being recorded.
#define SO_LAUNCH_CHECK()                                                         \
    do {                                                                          \
        hipError_t e_ = hipGetLastError();                                        \
        if (e_ != hipSuccess) {                                                   \
            so_set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(e_), \
                         __FILE__, __LINE__);                                     \
            return SO_ERR_HIP;                                                    \
        }                                                                         \
    } while (0)

static inline uint32_t so_ceil_div(uint64_t a, uint64_t b) { return (uint32_t)((a + b - 1) / b); }

// Epilogue shared by the matmul and conv kernels.  expf/tanhf are the accurate
// OCML routines (no fast-math), matching 1.0f/(1.0f+expf(-v)) and tanhf(v).
template <int ACT>
__device__ __forceinline__ float so_epilogue(float v)
{
    if (ACT == SO_ACT_RELU) return v > 0.0f ? v : 0.0f;
    if (ACT == SO_ACT_SIGMOID) return 1.0f / (1.0f + expf(-v));
    if (ACT == SO_ACT_TANH) return tanhf(v);
    return v;
}
