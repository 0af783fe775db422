// Launch interface between the C ABI host layer and the gfx950 kernels.
#ifndef LUTGEMM_KERNELS_H
#define LUTGEMM_KERNELS_H

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

namespace lutgemm_kernels {

struct MatvecArgs {
    const uint8_t *signs;   // sign tiles (layout.h)
    const uint16_t *scales; // scale tiles (layout.h)
    const void *x;          // fp16 activations, contiguous, 16-byte aligned
    void *y;                // fp16 outputs, element j at y[j * y_stride]
    unsigned long long *accum;  // [2][nb*32] split-k accumulators (count | flags | fixed-point sum), zero
                                // between launches; used when k_splits > 1
    int k, n;
    int ts, nb;             // k-blocks, output batches
    int ntiles;             // column tiles = ceil(nb / waves)
    int k_splits;           // workgroups along k
    int blocks_per_split;   // k-blocks per workgroup
    int y_stride;           // output j goes to y[j * y_stride]
    // rows == 2: a second activation row at x + x_row_stride goes to y + y_row_stride in the
    // same pass (strides in fp16 elements), with its accumulators at accum + accum_row_stride
    int rows;               // 1 or 2 activation rows (0 selects the read probe); 1..kBatchRows for launch_batch
    long long x_row_stride, y_row_stride, accum_row_stride;
};

// Activation rows the batch kernel takes in one pass over the weight (rows r at x + r * x_row_stride
// go to y + r * y_row_stride, with split-k accumulators at accum + r * accum_row_stride).
constexpr int kBatchRows = 16;

// Up to kMaxFused independent one-row matvecs for one launch: entry i owns the workgroups
// first_block[i] .. first_block[i+1]-1 of the grid (the last entry up to the end).
constexpr int kMaxFused = 32;
struct MultiMatvecArgs {
    int count;
    int first_block[kMaxFused];
    MatvecArgs entry[kMaxFused];
};

struct DequantArgs {
    const uint8_t *signs;
    const uint16_t *scales;
    void *out;              // fp16 [k][n] or [n][k]
    int k, n, q, has_offset, gsub, ts;
    int transposed;
};

// workgroups = ntiles * k_splits, `waves` wavefronts of 64 lanes per workgroup.
hipError_t launch_matvec(int q, int has_offset, int gsub, const MatvecArgs &a, int workgroups,
                         int waves, hipStream_t stream);

// entries that all have one row or all have two, sharing q, has_offset, gsub and the wavefronts per workgroup
hipError_t launch_matvec_multi(int q, int has_offset, int gsub, const MultiMatvecArgs &m, int workgroups, int waves,
                               hipStream_t stream);

// 1..kBatchRows activation rows in one pass (matrix cores), any number of planes up to kBatchMaxPlanes.
// A workgroup has kBatchWavesMin .. kBatchWaves wavefronts: wavefront w stages activation rows w and
// w + wavefronts, so eight cover the 16 rows of a pass.  A tile of more than kBatchWidePlanes planes
// needs more than 128 registers per lane, so such weights run with exactly kBatchWavesMin wavefronts
// (which may then use 256 registers each).
constexpr int kBatchMaxPlanes = 8;
constexpr int kBatchWidePlanes = 4;
constexpr int kBatchWaves = 16;
constexpr int kBatchWavesMin = 8;
// LDS of a workgroup of the batch kernel: two activation blocks of 17 rows of 2064 bytes (every
// activation as the pair -x, +x), and per wavefront a 1 KiB staging area plus the scales of its tile
// for the matrix lanes (64 bytes per (scale group of the k-block, plane or offset)).  A compute
// unit has 160 KiB, which bounds the wavefronts of a workgroup when there are four groups per 128 k.
constexpr int batch_scale_area_bytes(int gsub, int qo) { return 256 * gsub * qo; }
constexpr int batch_lds_bytes(int waves, int gsub, int qo)
{
    return 2 * 17 * 2064 + waves * (1024 + batch_scale_area_bytes(gsub, qo));
}
constexpr int batch_waves_max(int gsub, int q, int qo)
{
    int w = q > kBatchWidePlanes ? kBatchWavesMin : kBatchWaves;
    while (w > kBatchWavesMin && batch_lds_bytes(w, gsub, qo) > 160 * 1024) w--;
    return w;
}
static_assert(batch_lds_bytes(kBatchWavesMin, 4, kBatchMaxPlanes + 1) <= 160 * 1024, "LDS of a compute unit");
hipError_t launch_batch(int q, int has_offset, int gsub, const MatvecArgs &a, int workgroups, int waves, hipStream_t stream);
// A work list of independent batches in one launch: entries sharing q, has_offset, gsub and the
// wavefronts per workgroup, each with 1..kBatchRows rows and its own ntiles / k_splits / blocks_per_split;
// workgroups = sum of the entries' ntiles * k_splits, entry i starting at first_block[i].
hipError_t launch_batch_multi(int q, int has_offset, int gsub, const MultiMatvecArgs &m, int workgroups, int waves,
                              hipStream_t stream);

// words[0..count) = 0 (a fill kernel rather than a memset node, so that it can be captured)
hipError_t launch_fill_zero(unsigned long long *words, size_t count, hipStream_t stream);

// Split-k words of the allocation-free entry point: a static device array of kStaticSplitKWords
// 64-bit words (8 MiB on every device the library runs on, enough for 65,536 outputs per
// activation row of a pass of kBatchRows rows), zero at load and zero again after every completed
// launch.
// Returns its device address on `device`, which must be the current device (0 <= device <
// kMaxDevices); looked up once per device.
constexpr size_t kStaticSplitKWords = (size_t)1 << 20;
constexpr int kMaxDevices = 64;
hipError_t static_split_k_words(int device, unsigned long long **words);

// fp16 [k][m] -> [m][k]
hipError_t launch_gather_columns(const void *cols, void *rows, int k, int m, hipStream_t stream);

hipError_t launch_dequantize(const DequantArgs &a, hipStream_t stream);

// The matvec's loads without its arithmetic (same grid and arguments; x, y and accum unused):
// nothing is written.
hipError_t launch_read_probe(int q, int has_offset, int gsub, const MatvecArgs &a, int workgroups, int waves,
                             hipStream_t stream);

// Dense fp16 comparator: y[n] = sum_k W^T[n][k] x[k]; k a multiple of 8, pointers 16-byte aligned.
hipError_t launch_dense_gemv(const void *wt, const void *x, void *y, int k, int n, int compute_units,
                             hipStream_t stream);

}  // namespace lutgemm_kernels
#endif
