/*
 * lutgemm_c.h -- C ABI of the MI355X (gfx950) LUT-GEMM library (liblutgemm_hip.so).
 *
 * Plain pointers and sizes only; every function returns a lutgemm_status.  The C++ API of
 * the reference (namespace lutGEMM, headers "lutGEMM", "kernels.h", "nQWeight_fp16.h" in
 * this directory) is a header-only layer over these entry points.
 *
 * Citations name the interface of the reference tree that each entry point stands in for.
 *
 * Host-side input layout of a BCQ weight (identical to the reference's, so a caller's
 * existing packer keeps working):
 *   bW     uint32 [k/32][q][n]   bit t of bW[w][b][j] is the sign of weight (32 w + t, j) in
 *                                plane b, 1 = +1, 0 = -1
 *   alpha  float  [num_groups][q][n]   per-group scale, group length g = k / num_groups
 *   q_bias float  [num_groups][n] or NULL   per-group additive offset
 *   W[i][j] = sum_b alpha[i/g][b][j] * sign(b,i,j) + q_bias[i/g][j];   y[j] = sum_i x[i] W[i][j]
 * Inside the handle the planes are re-tiled for 64-lane wavefronts; the device layout is
 * private to the library.
 */
#ifndef LUTGEMM_C_H
#define LUTGEMM_C_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum lutgemm_status {
    LUTGEMM_OK = 0,
    LUTGEMM_ERR_NULL_POINTER = 1,  /* a required pointer argument is NULL */
    LUTGEMM_ERR_BAD_SHAPE = 2,     /* k, n, q, num_groups or m violate the preconditions */
    LUTGEMM_ERR_NO_DEVICE = 3,     /* no HIP device, or the current device is not the handle's */
    LUTGEMM_ERR_HIP = 4,           /* a HIP runtime call failed; see lutgemm_last_error() */
    LUTGEMM_ERR_OUT_OF_MEMORY = 5, /* host or device allocation failed */
    LUTGEMM_ERR_UNSUPPORTED = 6,   /* valid request outside what this build implements */
    LUTGEMM_ERR_IO = 7             /* a packed-weight file could not be read or written */
} lutgemm_status;

/* Opaque packed weight: device-resident sign tiles, scales and offsets plus the launch plan
 * and the workspace of the launching streams (split-k accumulators: 64-bit words, one per output and
 * activation row of a pass; staging rows of the column-batched form).  Stands in for class lutGEMM::nQWeight_fp16
 * (lutGEMM/include/nQWeight_fp16.h:27-52). */
typedef struct lutgemm_weight lutgemm_weight;

/* Shape record returned by lutgemm_weight_info(); field meanings follow the public data
 * members of nQWeight_fp16 (lutGEMM/include/nQWeight_fp16.h:29-37). */
typedef struct lutgemm_weight_info_t {
    int k;            /* kSize: reduction length */
    int n;            /* mSize: number of outputs */
    int q;            /* nb: bit-planes */
    int num_groups;   /* num_groups */
    int group_size;   /* k / num_groups */
    int has_offset;   /* q_bias != nullptr */
    size_t sign_bytes;   /* k*n*q/8: packed sign bytes streamed per matvec (unpadded) */
    size_t scale_bytes;  /* num_groups*q*n*2 (unpadded) */
    size_t offset_bytes; /* num_groups*n*2 or 0 (unpadded) */
    size_t device_bytes; /* bytes of device memory held by the handle: tiles, split-k accumulators and
                            staging rows of every stream set allocated so far */
} lutgemm_weight_info_t;

/* Build a packed weight from HOST arrays in the layout above (floats are rounded to fp16,
 * round-to-nearest-even).  Replaces nQWeight_fp16::parsing with is_row_wise_quantize=false
 * (lutGEMM/src/nQWeight_fp16.cu:60-91): same inputs, but the sign planes are re-tiled for
 * coalesced wave64 reads instead of being copied verbatim.
 * Preconditions (LUTGEMM_ERR_BAD_SHAPE otherwise): k > 0, k % 32 == 0, n > 0, 1 <= q <= 8,
 * num_groups >= 1, k % num_groups == 0 and (k / num_groups) % 32 == 0.
 * The handle lives on the current HIP device. */
int lutgemm_weight_create(const uint32_t *bW, const float *alpha, const float *q_bias, int k, int n,
                          int q, int num_groups, lutgemm_weight **out);

/* As above with alpha / q_bias already in fp16 (host arrays of binary16 bit patterns). */
int lutgemm_weight_create_f16(const uint32_t *bW, const uint16_t *alpha, const uint16_t *q_bias,
                              int k, int n, int q, int num_groups, lutgemm_weight **out);

/* Free everything the handle owns, each allocation exactly once; NULL is accepted.
 * Replaces nQWeight_fp16::~nQWeight_fp16 (lutGEMM/src/nQWeight_fp16.cu:101-105). */
int lutgemm_weight_destroy(lutgemm_weight *w);

int lutgemm_weight_info(const lutgemm_weight *w, lutgemm_weight_info_t *info);

/* y[r][0..n) = x[r][0..k) * W for r < m, fp16 in / fp16 out, fp32 accumulation, asynchronous
 * on `stream` (a hipStream_t passed as void*, NULL = the default stream).  x and y are
 * device pointers, row-major [m][k] and [m][n], x 16-byte aligned.  The offset term is applied
 * iff the weight was created with q_bias.  No memset of y is needed and none is issued; the
 * call allocates nothing.  The result is deterministic (bit-identical from launch to launch).
 * Replaces lutGEMM::matmul(void* output, void* input, nQWeight_fp16&, int m, int algo)
 * (lutGEMM/include/kernels.h:27, lutGEMM/src/kernels.cu:64-71), which for m == 1 runs
 * kernel::nqmv (mv_fp16.hpp:121) or kernel::nqmv_bias (mv_fp16_bias.hpp:143) and for m > 1
 * dequantises the whole weight and calls a library GEMM (kernels.cu:73-79); here every
 * 1 <= m <= LUTGEMM_MAX_BATCH streams the packed weight: m == 1 and m == 2 through the table-lookup
 * kernels (a two-row pass gives each row bit-identical to its own one-row call), m >= 3 through
 * the batch kernel, which takes up to 16 rows per pass over the weight and contracts them on the
 * matrix cores while a tile is in registers (any number of planes and any group size; weights of
 * more than four planes with workgroups of exactly eight wavefronts).  Batch results are deterministic and within
 * the same tolerance, but a row may differ in the last bit from its own one-row call (another order
 * of the fp32 additions).
 * Launches on one stream run one after the other and share one set of split-k accumulators of the
 * handle; every further stream that launches on the handle gets a set of its own, allocated at that
 * stream's first launch, so launches on different streams may overlap in time.  A first launch
 * under graph capture is refused with LUTGEMM_ERR_UNSUPPORTED before anything is allocated (launch
 * once on the stream before capturing), as are the calls that synchronise: the two autotune calls
 * and lutgemm_weight_reset_workspace.  A handle keeps four sets.  A fifth stream takes over the set of the stream that used
 * the handle least recently: at once if that stream's launches on the handle have completed,
 * otherwise the new stream is made to wait for them (hipStreamWaitEvent) first; to know, every
 * launch records an event once a handle serves more than one stream.  Launches issued under graph
 * capture are not tracked, and a set last used that way is never handed on
 * (LUTGEMM_ERR_UNSUPPORTED if no set can be taken over; lutgemm_weight_clone gives further streams
 * handles of their own).  Host threads may call on one handle at the same time as long as each uses a
 * stream of its own (a set that a call has claimed is not handed to another stream before the call has
 * issued its launches); launches from different host threads on the SAME stream must be serialised by
 * the caller, as for any stream.
 * Non-finite values follow IEEE arithmetic whatever the launch plan: a NaN activation gives NaN
 * outputs, infinite partial sums give an infinity of their sign, or NaN if both signs occur.  With
 * more than one k-split the partial sums are added as fixed-point integers (2^-24 resolution);
 * a finite partial sum beyond +-4.1e6 (64 times binary16's range) counts as an infinity. */
#define LUTGEMM_MAX_BATCH 4096
int lutgemm_matvec(const lutgemm_weight *w, const void *x, void *y, int m, void *stream);

/* lutgemm_matvec without any allocation, for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, same kernels and bit-identical results; the only difference is where
 * the split-k accumulators live: not in the handle's allocation but in a static device array of
 * the library (8 MiB on every device the library runs on, held until the process ends), whose
 * address is looked up once per device.  Limit: n <= 65,536 outputs (LUTGEMM_ERR_UNSUPPORTED
 * beyond).  The call performs no hipMalloc / hipFree and calls no allocating library routine.  All
 * calls on one device share that device's array, whatever the handle or stream: calls that overlap
 * in time on one device race on it (issue them on one stream, or use lutgemm_matvec, which keeps
 * accumulators per handle and stream).  Completed launches leave the array at zero; after a launch
 * that failed in the middle of a batched call the next call clears it with a fill kernel first. */
int lutgemm_matvec_static(const lutgemm_weight *w, const void *x, void *y, int m, void *stream);

/* Column-batched form: x is [k][m] and y is [n][m] (m vectors stored as columns).
 * Replaces lutGEMM::matmul(void* output, nQWeight_fp16&, void* input, int n, int algo)
 * (lutGEMM/include/kernels.h:26, lutGEMM/src/kernels.cu:56-63).  For m == 1 it is the same
 * operation as lutgemm_matvec.  For m > 1 the columns are first gathered into staging rows owned
 * by the handle (one buffer per launching stream).  Up to m = 16 nothing is allocated; a larger m
 * grows the stream's buffer the first time it occurs (synchronises that stream, frees, allocates). */
int lutgemm_matvec_cols(const lutgemm_weight *w, const void *x, void *y, int m, void *stream);

/* `count` matvecs with a single call (a decoder layer's projections, a benchmark loop): entry i
 * computes ys[i] = xs[i] * ws[i] with batch ms[i] exactly as lutgemm_matvec would, and the results
 * are those of the entries executed in order.  Consecutive entries that do not depend on each other
 * share ONE kernel launch (up to 32 per launch): entries that all have one activation row, that all
 * have two, or that all have 3 to 16 rows (the batch kernel), with the same q /
 * offset / group layout, distinct handles, and no output overlapping an input or output of another
 * entry of the launch.  The workgroups of such entries follow each other in one grid, so the memory
 * system stays busy while single workgroups start and finish, and the launch overhead is paid
 * once.  Such a launch has a shape of its own (wavefronts per workgroup, split along k) chosen for
 * the whole run, not the handles' plans, so a result may differ in the last bit from the same
 * entry's lutgemm_matvec call; it is deterministic (same entries, same bits) and within the same
 * tolerance.  Entries that do not qualify (a later entry reading an earlier output, more than 16
 * rows, another kernel instance) get launches of their own, in order, exactly as lutgemm_matvec issues them.  Has no counterpart in the reference, whose caller loops over lutGEMM::matmul
 * itself (tests/opt/fp16/int3_col_wise_matmul_fp16.cu:120-133).  Stops at the first failing entry. */
int lutgemm_matvec_many(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys,
                        const int *ms, int count, void *stream);

/* Replace the model's choice of the launch shape of fused launches by a measurement.  Walks the
 * list as lutgemm_matvec_many does; for every run of entries that share a launch it times the six
 * launch shapes (wavefronts per workgroup, k-blocks per workgroup) the cost model ranks best, the
 * model's own choice among them, with the entries themselves on `stream` (a few launches each; ys
 * receive valid results; the device is kept busy for 30 ms first so that the clocks are up) and
 * remembers the fastest (the model's choice unless another shape measured at least 2 % faster),
 * process-wide, under the shapes of the run: kernel instance, compute units,
 * and (k, n, rows) of its entries in order.  From then on every lutgemm_matvec_many run of those
 * shapes, whatever its handles and buffers, is launched that way.  The constants of the cost model
 * were fitted on one MI355X; this call is how a caller checks them on the box it runs on.
 * The buffers are measured as they are: a list whose weights fit the memory-side cache is timed
 * from that cache.  Entries that do not share a launch are launched once, as lutgemm_matvec does
 * (their plans belong to the handles: lutgemm_weight_autotune).  Synchronises `stream`.  No
 * counterpart in the reference, whose tile sizes are fixed
 * (lutGEMM/src/cuda/kernels/mv_fp16.hpp:122-124). */
int lutgemm_matvec_many_autotune(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys,
                                 const int *ms, int count, void *stream);

/* The launch shape lutgemm_matvec_many would use for the first launch of this list, for tests and
 * benchmarks: how many entries share it (1: the first entry is launched on its own and the other
 * outputs are 0), wavefronts and k-blocks per workgroup, and whether that shape was measured by
 * lutgemm_matvec_many_autotune (1) or comes from the cost model (0).  Any output may be NULL. */
int lutgemm_matvec_many_plan(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys,
                             const int *ms, int count, int *entries_in_first_launch, int *waves_per_group,
                             int *k_blocks_per_group, int *measured);

/* As lutgemm_matvec_many, but every entry gets a launch of its own (the call is a plain loop over
 * lutgemm_matvec): for per-launch timing and profiling. */
int lutgemm_matvec_each(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys,
                        const int *ms, int count, void *stream);

/* Put every split-k accumulator of the handle back to zero and forget which streams have
 * launched on it (synchronises the device, then runs fill kernels on `stream` and waits for them;
 * allocated sets stay allocated).
 * Only needed after a launch was aborted half way (a failed launch in the middle of a batched call,
 * a device fault): completed launches always leave their accumulators at zero.  No counterpart in
 * the reference, which clears its output with cudaMemset before every call
 * (lutGEMM/src/kernels.cu:66). */
int lutgemm_weight_reset_workspace(lutgemm_weight *w, void *stream);

/* Dense fp16 weight on the device, W[k][n] (transposed == 0) or W[n][k] (transposed != 0),
 * offset included.  d_fW is a device pointer to k*n halves.  Asynchronous on `stream`.
 * Replaces lutGEMM::dequantize_gpu (lutGEMM/src/nQWeight_fp16.cu:29-35); unlike it, the
 * group index is taken per weight and the offset is not dropped. */
int lutgemm_dequantize(const lutgemm_weight *w, void *d_fW, int transposed, void *stream);

/* Measurement aid without counterpart in the reference: for each of the `count` handles in turn,
 * streams its packed tiles once with a kernel that only reads: the grid of that handle's launch
 * plan, every wavefront fetching the bytes its matvec wavefront fetches in the same order with
 * the same number of 16-byte loads in flight, nothing computed or written.  The time per launch
 * is the device's pure-read time for a matvec's bytes, the floor the benchmark quotes next to it.
 * Asynchronous on `stream`. */
int lutgemm_read_probe(const lutgemm_weight *const *ws, int count, void *stream);

/* Comparator without counterpart in the reference's library (its test times cuBLAS next to the
 * LUT kernel, tests/opt/fp16/int3_col_wise_matmul_fp16.cu:302-313): a plain bandwidth-bound dense
 * fp16 matrix-vector product y[n] = sum_k W[n][k] x[k] for a dense weight stored as W^T [n][k]
 * (the layout lutgemm_dequantize writes with transposed = 1), fp32 accumulation, fp16 result.
 * k a multiple of 8; d_wt and d_x 16-byte aligned device pointers.  Asynchronous on `stream`. */
int lutgemm_dense_gemv_f16(const void *d_wt, const void *d_x, void *d_y, int k, int n, void *stream);

/* Copy the packed planes back into the host input layout (exact inverse of the re-tiling):
 * bW [k/32][q][n] uint32, alpha [num_groups][q][n] and q_bias [num_groups][n] as binary16
 * bit patterns; any output pointer may be NULL to skip it.  Synchronous. */
int lutgemm_weight_unpack(const lutgemm_weight *w, uint32_t *bW, uint16_t *alpha, uint16_t *q_bias);

/* Launch plan of the handle for launches with one activation row (for benchmarks and tests):
 * workgroup count, waves per workgroup, k-splits and 512-wide k-blocks per workgroup.  Passes
 * over two rows (m >= 2) have a plan of their own, equal to this one unless
 * lutgemm_weight_autotune has measured a better one. */
int lutgemm_weight_plan(const lutgemm_weight *w, int *workgroups, int *waves_per_group,
                        int *k_splits, int *k_blocks_per_group);

/* The same for the launches a call with m activation rows makes (m = 1: the plan above; m = 2:
 * the two-row plan; m >= 3: the batch kernel's plan for passes of min(m, 16) rows).  LUTGEMM_ERR_BAD_SHAPE for m outside
 * 1..LUTGEMM_MAX_BATCH.  No counterpart in the reference. */
int lutgemm_weight_plan_for(const lutgemm_weight *w, int m, int *workgroups, int *waves_per_group,
                            int *k_splits, int *k_blocks_per_group);

/* Override the launch plan of the table-lookup kernels, for one-row and two-row launches alike (0
 * keeps the automatic choice for that field; the batch kernel has lutgemm_weight_set_batch_plan);
 * synchronises the device first.  Returns LUTGEMM_ERR_BAD_SHAPE if the request cannot be launched
 * (1..12 wavefronts per workgroup, 1..min(k/512 rounded up, 128) k-splits). */
int lutgemm_weight_set_plan(lutgemm_weight *w, int waves_per_group, int k_splits);

/* Override the batch kernel's launch plan (calls with 3 or more rows): 8..16 wavefronts per
 * workgroup (exactly 8 for weights of more than four planes; fewer than 16 where four scale
 * groups per 128 k leave less LDS) and the k-splits; both 0: back to the automatic choice.
 * LUTGEMM_ERR_BAD_SHAPE if the request cannot be launched.  No launch on the handle may be in
 * flight. */
int lutgemm_weight_set_batch_plan(lutgemm_weight *w, int waves_per_group, int k_splits);

/* Measure the most promising launch plans on the device (a few launches each, on `stream`, with
 * scratch activations of its own) and keep the fastest, separately for launches with one
 * activation row and for two-row passes (which keep the k-split of the one-row plan, so that
 * rows stay bit-identical to their own one-row launches), and, where the batch kernel takes the
 * shape, for its passes of up to 8 and of 9 to 16 rows.  Optional: the automatic plan is chosen
 * from a model, this replaces it by a measurement.  The measurement streams the weight from
 * HBM as a decoder does: it rotates over temporary device copies of the packed weight (about
 * 1 GiB in total, at most 64 copies) so that no launch finds its weight in the memory-side
 * cache.  Synchronises `stream`; allocates and frees temporary device buffers.  No counterpart in the reference, whose tile sizes are fixed
 * (lutGEMM/src/cuda/kernels/mv_fp16.hpp:122-124). */
int lutgemm_weight_autotune(lutgemm_weight *w, void *stream);

/* Device pointers of the packed arrays, for the public data members of the C++ layer. */
int lutgemm_weight_device_ptrs(const lutgemm_weight *w, void **signs, void **scales, void **offsets);

/* ---- Host-only packer entry points: no HIP device is touched ------------------------------
 * The re-tiling that lutgemm_weight_create performs, exposed for offline packing and for tests.
 * They stand where the reference has a verbatim cudaMemcpy of the planes
 * (lutGEMM/src/nQWeight_fp16.cu:87-88). */

/* Bytes of the sign tiles and of the scale tiles (scales and offsets interleaved) for a shape. */
int lutgemm_packed_sizes(int k, int n, int q, int num_groups, int has_offset, size_t *sign_bytes,
                         size_t *scale_bytes);

/* Host input layout -> device tiles, into caller-provided host buffers of the sizes above.
 * alpha / q_bias are binary16 bit patterns; q_bias may be NULL. */
int lutgemm_pack_host(const uint32_t *bW, const uint16_t *alpha, const uint16_t *q_bias, int k, int n,
                      int q, int num_groups, void *signs_out, void *scales_out);

/* Exact inverse of lutgemm_pack_host; any of bW / alpha / q_bias may be NULL. */
int lutgemm_unpack_host(const void *signs, const void *scales, int k, int n, int q, int num_groups,
                        int has_offset, uint32_t *bW, uint16_t *alpha, uint16_t *q_bias);

/* ---- packed-weight files ------------------------------------------------------------------
 * The reference has no on-disk form of a packed weight: its Python examples only print the
 * converted tensors (examples/quant_model_rtn.py:86-99) and nQWeight_fp16::parsing re-reads host
 * arrays on every start (lutGEMM/src/nQWeight_fp16.cu:60-91).  A file written here holds the
 * device tiling itself (64-byte header: magic "LUTGEMMW", format version, tile layout id, k, n,
 * q, num_groups, has_offset, byte counts; then the sign tiles, then the scale tiles, all little
 * endian), so loading is one read and two copies to the device, with no packing work. */

/* Host only: pack host arrays (as for lutgemm_weight_create_f16) straight into a file. */
int lutgemm_pack_file(const uint32_t *bW, const uint16_t *alpha, const uint16_t *q_bias, int k, int n, int q,
                      int num_groups, const char *path);

/* Host only: read a file back into the host input layout; any of bW / alpha / q_bias may be
 * NULL, `info` (optional) receives the shape, so a first call with NULL arrays sizes a second. */
int lutgemm_unpack_file(const char *path, uint32_t *bW, uint16_t *alpha, uint16_t *q_bias,
                        lutgemm_weight_info_t *info);

/* Write the packed weight held by a handle / create a handle on the current device from a
 * file.  LUTGEMM_ERR_IO if the file cannot be opened, is not such a file, was written for
 * another tile layout or is truncated.  Synchronous. */
int lutgemm_weight_save(const lutgemm_weight *w, const char *path);
int lutgemm_weight_load(const char *path, lutgemm_weight **out);

/* A second, independent handle with its own device copy of the packed weight and its own
 * workspace (device-to-device copy, no packing), with the same launch plan. */
int lutgemm_weight_clone(const lutgemm_weight *w, lutgemm_weight **out);

/* float -> binary16 bit patterns, round to nearest even: the conversion applied to alpha and
 * q_bias at ingest (stands for the __float2half loops of lutGEMM/src/nQWeight_fp16.cu:81,85). */
int lutgemm_float_to_half(const float *src, uint16_t *dst, size_t count);

/* Thread-local text of the last failure in this library ("" if none). */
const char *lutgemm_last_error(void);
const char *lutgemm_status_string(int status);

/* Library / build identification, e.g. "lutgemm-hip gfx950". */
const char *lutgemm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* LUTGEMM_C_H */
