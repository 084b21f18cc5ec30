/*
 * sparseops_hip.h -- C ABI of libsparseops_hip.so, the MI355X (gfx950) device side
 * of the ELLPACK compute path.
 *
 * The reference is a CPU library whose consumers are C++ callers of its headers
 * and Python through pybind11; it has no FFI of its own.  This header is the
 * boundary a maintainer binds instead of the reference's CPU kernels: plain C,
 * opaque handles, caller-owned pointers and sizes, no C++ or torch types.  Each
 * entry point cites the reference interface it stands in for.
 *
 * Conventions
 *   - every function returns so_status (0 = ok) and never throws or aborts;
 *     so_last_error() gives the message of the calling thread's last failure.
 *   - "d" parameters are device pointers obtained from so_malloc (or any HIP
 *     allocation on the context's device); all others are host pointers.
 *   - every launch goes to the context's single stream; calls return without
 *     waiting for the device unless stated (so_d2h, so_sync, so_timer_end wait).
 *   - matrices are row-major; activations of the layer chain are
 *     [features x B] with the batch contiguous (include/sparse_onnx.hpp:148-154),
 *     4-D tensors are [C][H][W][B] (src/layers/conv_kernels.cpp:342-347).
 *   - all arithmetic is fp32; every output element is produced by the same
 *     rounding sequence as the reference (bias first, then one fused
 *     multiply-add per stored nonzero in ascending slot order), except so_matvec
 *     whose in-row summation order differs (wave reduction) and is accurate to
 *     fp32 round-off.
 */
#ifndef SPARSEOPS_HIP_H
#define SPARSEOPS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int so_status;
enum {
    SO_OK = 0,
    SO_ERR_NO_DEVICE = 1, /* no usable HIP device / HIP runtime failed to initialise */
    SO_ERR_INVALID = 2,   /* bad argument (null pointer, shape mismatch, bad enum) */
    SO_ERR_OOM = 3,       /* device or host allocation failed */
    SO_ERR_HIP = 4,       /* a HIP call failed; message holds hipGetErrorString */
    SO_ERR_BOUNDS = 5     /* ELLPACK content invalid: idx >= n or nnz > r */
};

/* Fused epilogue of so_matmul / so_conv2d.  NONE and RELU are the reference's
 * template flag FUSE_RELU (src/ellpack_matmul.cpp:68-70); SIGMOID and TANH equal
 * the reference's separate activation layers applied to the matmul result
 * (src/layers/activation.cpp:38-40, 58-60). */
enum { SO_ACT_NONE = 0, SO_ACT_RELU = 1, SO_ACT_SIGMOID = 2, SO_ACT_TANH = 3 };

/* Device layouts kept for an uploaded ELLPACK matrix (bit flags).
 * ROW  : Wd[i*r + k], idx[i*r + k]  -- the encoder's own layout
 *        (include/ellpack_encoder.hpp:6-23); used by so_matmul / so_conv2d and
 *        by so_matvec for long rows.
 * SLOT : WdT[k*m + i], idxT[k*m + i] -- slot-major transpose so that the k-th
 *        nonzeros of consecutive rows are contiguous; used by so_matvec when
 *        one lane owns one row.
 * BINS : rows grouped by nnz into length classes for so_matvec on skewed
 *        matrices, so padding is never streamed.
 * TILED: the nonzeros regrouped by tiles of 256 columns and quads of four rows
 *        (same values, same ascending order inside every row) for the variant
 *        of so_matmul that stages X through LDS; costs about 1.3x the ROW
 *        arrays in HBM.  so_matmul uses it whenever it is present and C is a
 *        multiple of 4; results are bit-identical to the ROW kernel.
 * RBM  : row-block-merged, the reference's blocked-CSC idea (include/rbm_conv.hpp:8-27,
 *        src/layers/rbm_conv.cpp:7-73) for so_matmul: rows in blocks of 128, a block's used
 *        columns walked once, each X row segment loaded once and multiplied into every row
 *        of the block that has a nonzero there.  The fastest so_matmul for large matrices;
 *        so_matmul uses it whenever it is present and the launch covers most of the chip.
 *        Sums are taken column by column, not in a row's slot order: results agree with
 *        the reference to fp32 round-off (max |y - ref| <= 1e-5 * max |ref|), are not
 *        bit-identical to it, and are the same bits on every launch.  Rows may be in any
 *        order.  Costs about 1.4x the ROW arrays in HBM; with it so_matmul keeps a
 *        workspace in the context that grows on first use of a larger output.
 * IDX16: a second copy of the columns in 16 bits (needs n <= 65536; costs 2 bytes per slot,
 *        and as much again for the SLOT copy when that is asked for too).  so_matvec then
 *        reads 6 bytes per nonzero instead of 8 -- the product is a stream from HBM, so
 *        about a fifth less time -- and gives the same bits.  Nothing else reads it;
 *        downloads come from the 32-bit arrays. */
enum { SO_LAYOUT_ROW = 1, SO_LAYOUT_SLOT = 2, SO_LAYOUT_BINS = 4, SO_LAYOUT_TILED = 8, SO_LAYOUT_RBM = 16, SO_LAYOUT_IDX16 = 32 };

typedef struct so_ctx so_ctx;         /* one device + one stream + staging arena */
typedef struct so_ellpack so_ellpack; /* device-resident ELLPACK matrix */

/* Geometry of one convolution as the reference's loader derives it
 * (ConvAttr, include/sparse_onnx.hpp:66-98; src/sparse_onnx.cpp:408-451).
 * Column k of the Cout x K weight matrix is (cin, kh, kw) with kw fastest. */
typedef struct {
    uint32_t Cin, Cout, kH, kW;
    uint32_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
    uint32_t H_in, W_in, H_out, W_out;
} so_conv_geom;

/* PoolAttr (include/sparse_onnx.hpp:101-112). */
typedef struct {
    uint32_t C, H, W, H_out, W_out;
    int32_t kH, kW, sH, sW, padH0, padW0;
} so_pool_geom;

/* ---- runtime ------------------------------------------------------------- */

/* Number of HIP devices; SO_ERR_NO_DEVICE (and *n = 0) when there is none. */
so_status so_device_count(int *n);
/* Create a context on `device` (its own non-blocking stream, default priority). */
so_status so_init(int device, so_ctx **out);
so_status so_destroy(so_ctx *ctx);
/* Message of the last failure on the calling thread ("" if none). */
const char *so_last_error(void);
/* Device name and compute-unit count of the context's device. */
so_status so_device_info(so_ctx *ctx, char *name, size_t name_len, int *compute_units);
/* The SPARSEOPS_* tuning overrides (kernel and layout choices: for tuning and tests, results never
 * depend on them) are read from the environment by so_init, not per launch as the reference reads
 * its thread count (src/ellpack_matmul.cpp:21); this reads them again for `ctx`. */
so_status so_tuning_reload(so_ctx *ctx);

so_status so_malloc(so_ctx *ctx, size_t bytes, void **dptr);
so_status so_free(so_ctx *ctx, void *dptr);
so_status so_h2d(so_ctx *ctx, void *dst, const void *src, size_t bytes); /* waits */
so_status so_d2h(so_ctx *ctx, void *dst, const void *src, size_t bytes); /* waits */
so_status so_d2d(so_ctx *ctx, void *dst, const void *src, size_t bytes);
so_status so_fill_zero(so_ctx *ctx, void *dptr, size_t bytes); /* fill kernel, graph-safe */
/* Waits for the context's stream.  The LDS-staged kernels synchronise their waves through counters
 * with a bounded wait instead of hanging; a wave that gives up counts itself in a status word of the
 * context.  Every call that waits for the stream -- so_sync, so_h2d, so_d2h, so_timer_end and the
 * encoder's read-backs -- reads that word with the wait (one 4-byte copy, only when such a kernel has
 * been launched since the last look) and returns SO_ERR_HIP when it is set: the results of the
 * launches since the last look are invalid.  The word is then cleared; the next wait reports SO_OK. */
so_status so_sync(so_ctx *ctx);

/* HIP-event stopwatch on the context's stream: begin records an event, end
 * records a second one, waits for it and returns the elapsed milliseconds. */
so_status so_timer_begin(so_ctx *ctx);
so_status so_timer_end(so_ctx *ctx, float *ms);

/* ---- ELLPACK on the device ---------------------------------------------- */

/* Upload the encoder's arrays once (struct Ellpack, include/ellpack_encoder.hpp:6-23:
 * Wd[m*r], idx[m*r], nnz[m]).  Validates nnz[i] <= r and idx < n for every stored
 * slot (the reference validates only in a benchmark,
 * benchmark-mkl/matvec/bench_matvec.cpp:83-98) and fails with SO_ERR_BOUNDS.
 * `layouts` is a mask of SO_LAYOUT_*; ROW is always kept.  m, n or r may be 0.
 * Column order inside a row: the encoder stores a row's columns strictly ascending
 * (src/ellpack_encoder.cpp:28-41) and the TILED layout and the convolution's LDS-windowed layout
 * rely on it.  Rows in any other order (or with a repeated column) are accepted, as the
 * reference's kernels accept them: TILED is then not built (so_ellpack_dims reports the layouts
 * kept), convolution plans on the handle use the gather kernel, and every kernel multiplies in
 * slot order.  so_ellpack_decode needs distinct columns per row. */
so_status so_ellpack_upload(so_ctx *ctx, const float *Wd, const uint32_t *idx,
                            const uint32_t *nnz, uint32_t m, uint32_t n, uint32_t r,
                            int layouts, so_ellpack **out);
so_status so_ellpack_free(so_ctx *ctx, so_ellpack *E);
so_status so_ellpack_dims(const so_ellpack *E, uint32_t *m, uint32_t *n, uint32_t *r,
                          uint64_t *total_nnz, int *layouts);
/* Read the device copy back, for the bit-exact layout check.  layout = ROW
 * returns Wd/idx as uploaded; layout = SLOT returns the slot-major arrays
 * (WdT[k*m+i]); nnz may be NULL. */
so_status so_ellpack_download(so_ctx *ctx, const so_ellpack *E, int layout,
                              float *Wd, uint32_t *idx, uint32_t *nnz);

/* convert_to_ellpack (src/ellpack_encoder.cpp:6-44) on the device: dDense is a row-major
 * [m x n] fp32 matrix in device memory; the handle holds the ROW layout with the same
 * contents the host encoder produces (per row the entries with v != 0.0f in ascending
 * column order, so -0.0f is dropped and NaN kept; r = longest row; zero padding).
 * Other layouts: download and upload again with the layouts wanted. */
so_status so_ellpack_encode(so_ctx *ctx, const float *dDense, uint32_t m, uint32_t n, so_ellpack **out);
/* so_ellpack_encode for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Calls no hipMalloc,
 * hipFree or allocating routine: the caller brings the outputs -- dNnz[m], dWd and dIdx of
 * m * r_cap slots each -- and the counting pass's partial results live in a static device array of
 * the library (524 544 bytes per GPU, held until the process ends), which limits a call to
 * 1 048 576 rows (more: SO_ERR_INVALID).  Output: dNnz[i] = nonzeros of row i, and dWd/dIdx packed
 * with row pitch r = the longest row, i.e. the first m * r slots hold exactly the arrays
 * so_ellpack_encode produces.  When r exceeds r_cap nothing is packed (dNnz is still valid).
 * r_out / total_nnz_out (host, may be NULL) receive r and the nonzero count; asking for either makes
 * the call wait for the device, and the call then fails with SO_ERR_INVALID when r > r_cap; with
 * both NULL it returns without waiting.  All calls on one GPU share the array: calls that overlap
 * on one GPU (two contexts, two threads) race. */
so_status so_ellpack_encode_noalloc(so_ctx *ctx, const float *dDense, uint32_t m, uint32_t n,
                                    uint32_t r_cap, float *dWd, uint32_t *dIdx, uint32_t *dNnz,
                                    uint32_t *r_out, uint64_t *total_nnz_out);
/* decode_from_ellpack (src/ellpack_encoder.cpp:46-60) on the device: dDense [m x n] row-major
 * is zeroed, then the first nnz[i] entries of every row are scattered into it. */
so_status so_ellpack_decode(so_ctx *ctx, const so_ellpack *E, float *dDense);

/* ---- kernels ------------------------------------------------------------ */

/* Y[m x C] = act(E * X[n x C] + bias): ellpack_matmul_fused<USE_MASK,FUSE_RELU>
 * (src/ellpack_matmul.cpp:11-92) and its dispatcher ellpack_matmul
 * (include/ellpack_matmul.hpp:23-43).  dBias may be NULL (zero start). */
so_status so_matmul(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C,
                    const float *dBias, float *dY, int act);
/* Makes sure a later so_matmul(ctx, E, ..., C, ...) allocates and prepares nothing: on a handle with the RBM
 * layout the context's workspace is grown to what C dense columns need and the handle's records are written
 * for that width (a no-op for every other layout).  so_matmul does both itself on first use of a larger output
 * or another width, but refuses to while a graph is being recorded: a caller that
 * records so_matmul into a graph calls this first (SparseOnnxModel::resize_buffers does, for every fully
 * connected layer -- the reference's documented way to get its allocation-free run(), README.md:146).
 * No counterpart in the reference. */
so_status so_matmul_reserve(so_ctx *ctx, const so_ellpack *E, uint32_t C);

/* y[m] = E * x[n] + bias: ellpack_matvec (src/ellpack_matvec.cpp:20-147).
 * `layout` picks the kernel: SO_LAYOUT_ROW (one wave per row), SO_LAYOUT_SLOT
 * (one lane per row on the slot-major copy), SO_LAYOUT_BINS (length classes),
 * or 0 to let the library choose from what was uploaded (length classes for skewed rows
 * and, on 16-bit columns, for matrices of 64 to 96 rows per compute unit; the lane-per-row
 * kernel for rows of at most 64 nonzeros; else one wave per row).  The kernels take the columns
 * from the SO_LAYOUT_IDX16 copy when the handle has one (same result). */
so_status so_matvec(so_ctx *ctx, const so_ellpack *E, const float *dx,
                    const float *dBias, float *dy, int layout);

/* Per-layer convolution plan, built once at load time: for every stored nonzero
 * of E (Cout x Cin*kH*kW) the input offset and (dh, dw) of its tap -- the role of
 * the reference's kmap (src/sparse_onnx.cpp:440-451); the (ho, wo, b)-dependent
 * part of the patch index is generated inside the kernel, so there is no
 * patch_indices table (src/sparse_onnx.cpp:476-497).  E must outlive the plan.
 * Checks H_out/W_out against the loader's formula (src/sparse_onnx.cpp:428-429). */
typedef struct so_conv_plan so_conv_plan;
so_status so_conv_plan_create(so_ctx *ctx, const so_ellpack *E, const so_conv_geom *g,
                              so_conv_plan **out);
so_status so_conv_plan_free(so_ctx *ctx, so_conv_plan *plan);
/* Re-sizes the plan's internal layouts for launches with batch B (how many output channels
 * a wave takes depends on how many workgroups the batch yields).  Optional: results never
 * depend on it; plans are created for batch 32.  Not to be called while a launch that uses
 * the plan may be in flight on another stream, nor during graph capture (it allocates).
 * No counterpart in the reference. */
so_status so_conv_plan_tune(so_ctx *ctx, so_conv_plan *plan, uint32_t B);
/* The LDS-windowed kernel's parameters for this plan (no counterpart in the reference:
 * a tuning/inspection aid): out = {tile_h, tile_w, window_h, window_w, channels per
 * chunk, chunks, output channels per wave, 0}; all zero when the geometry does not
 * suit that kernel and so_conv2d always takes the gather kernel. */
so_status so_conv_plan_window(const so_conv_plan *plan, uint32_t out[8]);

/* Sparse convolution by implicit im2col: conv2d_implicit_im2col_fmajor
 * (src/layers/conv.cpp:16-108), on the [C][H][W][B] layout of
 * conv2d_patchmajor_tiled (src/layers/conv_kernels.cpp:342-470), which is what
 * applyConv runs (src/layers/conv.cpp:118-135).  dX is [Cin][H_in][W_in][B],
 * dY is [Cout][H_out][W_out][B]; dBias may be NULL. */
so_status so_conv2d(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B,
                    const float *dBias, float *dY, int act);
/* The same convolution followed by the residual applyAdd (src/layers/add.cpp:9-76) and
 * then the activation, in one pass: dY = act((conv(dX) + bias) + dResidual).  The sum is
 * the fp32 addition applyAdd performs on the stored convolution output, so the result
 * has the same bits as the three separate layers.  dResidual is [Cout][H_out][W_out][B]
 * and must not alias dY. */
so_status so_conv2d_add(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B,
                        const float *dBias, const float *dResidual, float *dY, int act);

/* ---- row-block-merged (RBM) format ---------------------------------------
 * RBMPlan / RBMBlock / RBMColPair (include/rbm_conv.hpp:8-27) as build_rbm_from_ellpack
 * (src/layers/rbm_conv.cpp:7-73) produces them, flattened into five arrays: block b holds rows
 * [b*Ct_max, min(M, (b+1)*Ct_max)) of the M x N matrix; its union columns (RBMBlock::krel) are
 * krel[block_union[b] .. block_union[b+1]), ascending; union column u owns pairs colptr[u] ..
 * colptr[u+1] (RBMBlock::colptr made absolute over all blocks), and pair p is (pair_row[p], pair_w[p])
 * = RBMColPair{row inside the block, weight}, rows ascending.  The arrays are validated (SO_ERR_BOUNDS)
 * and copied; the handle is what convolution plans build their kernel streams from.  Biases are not
 * part of the handle: so_conv2d takes them per call, like the other kernels. */
typedef struct so_rbm so_rbm;
so_status so_rbm_upload(so_ctx *ctx, uint32_t M, uint32_t N, uint32_t Ct_max, uint32_t nblocks,
                        const uint32_t *block_union, const uint32_t *krel, const uint32_t *colptr,
                        const uint16_t *pair_row, const float *pair_w, so_rbm **out);
so_status so_rbm_free(so_ctx *ctx, so_rbm *R);
so_status so_rbm_dims(const so_rbm *R, uint32_t *M, uint32_t *N, uint32_t *Ct_max, uint32_t *nblocks,
                      uint64_t *total_union, uint64_t *total_pairs);
/* Attach the format to a convolution plan (ConvAttr::rbm / use_rbm, include/sparse_onnx.hpp:66-98;
 * the reference builds it at load for Cout >= 32 and K >= 64, src/sparse_onnx.cpp:499-502): so_conv2d
 * and so_conv2d_add then run conv2d_rbm_fmajor_implicit's algorithm (src/layers/conv_kernels.cpp:66-147)
 * -- every union column's input operand fetched once and applied to all rows of the block that use
 * it -- whenever the plan has its LDS-windowed layout and B is a multiple of 4, and the per-row
 * kernels otherwise; the results have the same bits either way.  Blocks of at most 8 rows.  R must
 * describe the plan's weights and outlive the plan; NULL detaches.  Not during graph capture. */
so_status so_conv_plan_set_rbm(so_ctx *ctx, so_conv_plan *plan, const so_rbm *R);
/* Inspection aid (no counterpart in the reference): out = {64-byte sets in the plan's streams,
 * real (row, weight) pairs, slots the kernel multiplies through, slots per record}; zeros when
 * the plan has no streams. */
so_status so_conv_plan_rbm_info(const so_conv_plan *plan, uint64_t out[4]);

/* applyMaxPool / applyGlobalAveragePool (src/layers/pool.cpp:28-101, 103-154)
 * on [C][H][W][B]; GAP writes [C][B]. */
so_status so_maxpool(so_ctx *ctx, const so_pool_geom *p, const float *dX, uint32_t B, float *dY);
so_status so_gap(so_ctx *ctx, uint32_t C, uint32_t H, uint32_t W, const float *dX,
                 uint32_t B, float *dY);
/* applyAdd (src/layers/add.cpp:9-76): D = A + B over len floats (D may alias A or B). */
so_status so_add(so_ctx *ctx, const float *dA, const float *dB, size_t len, float *dD);
/* applyRelu / applySigmoid / applyTanh (src/layers/activation.cpp:3-62). */
so_status so_act(so_ctx *ctx, int act, const float *dX, size_t len, float *dY);
/* dst[cols x rows] = transpose of src[rows x cols]; converts a C-order (B, F)
 * array to the kernels' [F x B] layout and back (the reference's Python tests
 * do this on the host with Fortran-order arrays, tests/full_test.py:77-88). */
so_status so_transpose(so_ctx *ctx, const float *dSrc, uint32_t rows, uint32_t cols, float *dDst);
/* dst[i2][i1][i0][:] = src[i0][i1][i2][:] for a [d0][d1][d2][inner] array: converts between the
 * kernels' [C][H][W][B] layout and a Fortran-order (B, C, H, W) array, which is [W][H][C][B] in memory
 * (what conv2d_rbm_fmajor_implicit and conv2d_tiled_im2col_fmajor take, include/conv_kernels.hpp:8-24;
 * the reference converts inside those kernels, src/layers/conv_kernels.cpp:96-123). */
so_status so_reverse_axes3(so_ctx *ctx, const float *dSrc, uint32_t d0, uint32_t d1, uint32_t d2,
                           uint32_t inner, float *dDst);
/* Copy a [rows x cols] matrix between buffers whose rows start src_stride / dst_stride floats
 * apart; with zero_fill the rest of every destination row (cols .. dst_stride) is set to zero.
 * No counterpart in the reference: the model runtime uses it to carry a batch inside buffers whose
 * rows hold 4, 8 or a multiple of 16 entries (what the convolution kernels' batch tiles need). */
so_status so_copy_rows(so_ctx *ctx, const float *dSrc, size_t src_stride, uint32_t rows, uint32_t cols,
                       float *dDst, size_t dst_stride, int zero_fill);

/* ---- launch graphs -------------------------------------------------------
 * Record every launch made on the context between begin and end into one
 * hipGraph, then replay it with a single submission (SparseOnnxModel::run uses
 * this for layer chains of eight layers or more, src/model_run.cpp:28-127).  No allocation, copy to
 * or from the host, or timer call may happen while recording. */
typedef struct so_graph so_graph;
so_status so_graph_begin(so_ctx *ctx);
so_status so_graph_end(so_ctx *ctx, so_graph **out);
so_status so_graph_launch(so_ctx *ctx, so_graph *g);
so_status so_graph_free(so_ctx *ctx, so_graph *g);

#ifdef __cplusplus
}
#endif
#endif /* SPARSEOPS_HIP_H */
