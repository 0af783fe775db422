// C ABI host layer (include/lutgemm_c.h): argument checks, packing, device memory, launch
// planning and kernel dispatch.  Calls the HIP runtime directly.
#include "../../include/lutgemm_c.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "kernels.h"
#include "layout.h"
#include "packer.h"

using namespace lutgemm_layout;

namespace {

thread_local char g_error[512] = "";

int fail(int status, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return status;
}

int hip_fail(hipError_t e, const char *what)
{
    return fail(e == hipErrorOutOfMemory ? LUTGEMM_ERR_OUT_OF_MEMORY : LUTGEMM_ERR_HIP, "%s: %s (%d)",
                what, hipGetErrorString(e), (int)e);
}

constexpr int kMaxWaves = 12;  // the kernel is compiled for at most 768 threads per workgroup
constexpr int kBuildRounds = 8;  // table parts per k-block (kernels.hip: kBuildParts)
constexpr int kMaxSplits = 128;  // the split-k arrival count has 8 bits, the sum room for 128 addends
constexpr int kStreamSlots = 4;  // sets of split-k words per handle: one per stream that launches on it
constexpr int kRowsPerPass = lutgemm_kernels::kBatchRows;  // activation rows a launch can take (rows of split-k words per set)
constexpr int kTableRows = 2;    // rows per pass of the table-lookup kernels
constexpr int kStagedColumns = 16;  // column-batched calls up to this m never allocate

struct Plan {
    int waves;             // wavefronts (= output batches) per workgroup
    int ntiles;            // column tiles
    int blocks_per_split;  // k-blocks per workgroup
    int k_splits;          // workgroups along k
};

}  // namespace

// What the launches of one stream on a handle share.  Launches on one stream run one after the other;
// every other stream that launches on the handle gets a set of its own, so launches that overlap on
// different streams never touch the same words.  Set 0 exists from creation (so a handle used from one
// stream never allocates in a launch call); further sets are allocated when a further stream first
// launches.  With all sets taken, a new stream takes over the least recently used set whose latest
// launch has completed (or, if none has, waits for the least recently used one's): for that, every
// launch records the set's event once the handle serves more than one stream.
struct StreamSet {
    void *stream;                // the stream the set serves
    unsigned long long *accum;   // kRowsPerPass x (padded outputs) split-k words, zero between launches
    void *xrows;                 // staging of column-batched activations: xrows_cols rows of k halves,
    int xrows_cols;              //   grown on demand
    hipEvent_t done;             // recorded behind the set's latest launch (only while done_valid)
    bool done_valid;
    unsigned long long last_use;
    int leases;                  // calls that have claimed the set and not yet issued all their launches
};

struct lutgemm_weight {
    Shape shape;
    int device;
    int compute_units;
    uint8_t *d_signs;
    uint16_t *d_scales;
    std::mutex slot_mutex;
    StreamSet set[kStreamSlots];
    int slots_used;               // sets that serve a stream
    unsigned long long use_clock;
    Plan plan;                    // launches with one activation row
    Plan plan2;                   // passes over two activation rows (m >= 2): same k-split as plan
    // Batch kernel (3 or more rows): measured plans for passes of up to 8 rows [0] and of 9..16 rows
    // [1], valid when batch_measured[i]; otherwise the model's choice is taken.
    Plan plan_batch[2];
    bool batch_measured[2];
};

namespace {

// Choose waves per workgroup and the k-split.  One workgroup owns `waves` batches of 32 outputs and
// `blocks_per_split` k-blocks and occupies a compute unit by itself.  The model below (times in
// microseconds) was fitted to measured times of all plans of twelve weight shapes on MI355X; over
// those shapes its choice is within 2 % of the best measured plan on average, 7 % at worst.
// A launch pays a fixed cost; every round of workgroups pays a start (first memory round trip,
// first table) and an end (reduction, split-k atomic); a k-block takes the longer of streaming
// `waves` tiles at the workgroup's share of HBM bandwidth (which grows less than proportionally
// when compute units stay idle) and of the lookups (wavefronts beyond four share a SIMD) plus the
// table build (eight parts spread over the wavefronts).
double plan_cost(const Shape &s, int cus, int waves, int splits, Plan *out)
{
    const double kLaunch = 2.72, kStartEnd = 0.48, kSplit = 0.8;
    const double kBytesPerCu = 6.83e6 / 256.0;  // HBM bytes per microsecond per compute unit, all busy
    const double kIdleExponent = 0.72;
    const double kLookup = 0.00622;  // per lookup of a wavefront
    const double kBuild = 0.289;     // per round of table parts
    const double kLatency = 1.05;    // a k-block cannot take less than one loaded memory round trip
    const double tile_bytes = (double)sign_tile_bytes(s) + (double)scale_tile_bytes(s);
    const int ntiles = div_up(s.nb, waves);
    const int bps = div_up(s.ts, splits);
    const int ks = div_up(s.ts, bps);
    if (ks != splits) return -1.0;  // same plan as a smaller `splits`
    const long wgs = (long)ntiles * ks;
    const double rounds = (double)((wgs + cus - 1) / cus);
    const double resident = (double)(wgs < cus ? wgs : cus);
    const double bandwidth = kBytesPerCu * cus * std::pow(resident / cus, kIdleExponent);
    double t_mem = waves * tile_bytes * resident / bandwidth;
    if (t_mem < kLatency) t_mem = kLatency;
    const double t_cmp = div_up(waves, 4) * 32.0 * s.q * kLookup + div_up(kBuildRounds, waves) * kBuild;
    *out = Plan{waves, ntiles, bps, ks};
    return kLaunch + rounds * (kStartEnd + bps * (t_mem > t_cmp ? t_mem : t_cmp) + (ks > 1 ? kSplit : 0.0));
}

Plan choose_plan(const Shape &s, int cus)
{
    Plan best{};
    double best_cost = 1e300;
    for (int waves = 1; waves <= kMaxWaves; waves++)
        for (int splits = 1; splits <= s.ts && splits <= kMaxSplits; splits++) {
            Plan p;
            const double cost = plan_cost(s, cus, waves, splits, &p);
            if (cost >= 0.0 && cost < best_cost - 1e-9) {
                best_cost = cost;
                best = p;
            }
        }
    return best;
}

// Launch shape of several independent one-row matvecs in one grid (lutgemm_matvec_many): one
// number of wavefronts per workgroup and one number of k-blocks per workgroup for all entries.
// A compute unit holds one workgroup at a time (its table sets take most of the LDS), so a unit
// works through its workgroups one after the other and pays for each its start (first memory
// round trip, first table) and its end (reduction, split-k atomic) in full; what the single grid
// removes is the idle time of the memory system: while one unit is between workgroups the others
// stream.  The grid runs in rounds of one workgroup per unit; a last round that does not fill
// the device streams faster per workgroup, but less than proportionally.  Long workgroups amortise
// start and end, short ones leave a smaller last round.  Constants (microseconds, bytes) fitted
// to measured times of 40 plans over five weight shapes and run lengths 3 to 32 on MI355X.
struct FusedPlan { int waves, blocks_per_group; };

struct FusedCandidate { double cost; FusedPlan plan; };

// `all` (optional) receives every launch shape the model considered with its cost
FusedPlan choose_fused_plan(const Shape *const *shapes, int count, int cus, int rows,
                            std::vector<FusedCandidate> *all = nullptr)
{
    // two-row passes: a k-block builds and looks up two table sets, bound by the lookups
    const double kBytesPerCu = (rows == 2 ? 4.8e6 : 7.0e6) / 256.0;  // streaming rate per compute unit with all units busy
    const double kBlockFloor = rows == 2 ? 2.6 : 1.7;  // a k-block takes at least one loaded memory round trip
    const double kStartEnd = rows == 2 ? 3.2 : 2.4, kStartEndPerWave = 0.17;  // per workgroup: 2.4 at 12 wavefronts, more with fewer
    const double kPartialExponent = 0.28;      // a round on a fraction f of the units streams f^0.28 as long
    int max_ts = 1;
    for (int e = 0; e < count; e++) max_ts = shapes[e]->ts > max_ts ? shapes[e]->ts : max_ts;
    FusedPlan best{kMaxWaves, max_ts};
    double best_cost = 1e300;
    for (int waves = 1; waves <= kMaxWaves; waves++)
        for (int bpg = div_up(max_ts, kMaxSplits); bpg <= max_ts; bpg++) {
            long groups = 0;
            double stream = 0.0;  // summed streaming time of all workgroups
            for (int e = 0; e < count; e++) {
                const Shape &s = *shapes[e];
                const int b = bpg < s.ts ? bpg : s.ts;
                const long g = (long)div_up(s.nb, waves) * div_up(s.ts, b);
                double t_block = waves * (double)(sign_tile_bytes(s) + scale_tile_bytes(s)) / kBytesPerCu;
                if (t_block < kBlockFloor) t_block = kBlockFloor;
                groups += g;
                stream += (double)g * b * t_block;
            }
            const double per_group = stream / (double)groups;
            const double start_end = kStartEnd + kStartEndPerWave * (kMaxWaves - waves);
            const long full = groups / cus, rest = groups % cus;
            double cost = (double)full * (per_group + start_end);
            if (rest) cost += per_group * std::pow((double)rest / cus, kPartialExponent) + start_end;
            if (all) all->push_back(FusedCandidate{cost, FusedPlan{waves, bpg}});
            if (cost < best_cost - 1e-9) {
                best_cost = cost;
                best = FusedPlan{waves, bpg};
            }
        }
    return best;
}

// Launch plan of the batch kernel (3..16 rows per pass on the matrix cores): wavefronts per
// workgroup and k-splits.  The kernel is bound on the compute units, not by the stream, so what
// matters is an even spread of the tiles over the compute units.
// Cost model in microseconds (-1 when `ks` names the same plan as a smaller number of k-splits).
// A compute unit holds one workgroup, so the grid runs in rounds of one workgroup per unit.  A
// workgroup costs a time per tile (wavefronts x k-blocks x planes) and a start and end of its own;
// the split-k atomics cost by their number in the whole launch (rows x outputs x k-splits: the
// memory side executes them at a fixed rate).  Constants fitted to 190 measured plans over eight
// shapes (k and n 4096 to 49152, two to four planes, eight rows; rms error 7 %); the fit names the
// fastest measured plan of every shape.
double batch_plan_cost(const Shape &s, int cus, int waves, int ks, int rows, Plan *out)
{
    const double tile_us = 0.1123 * s.q, group_us = 4.95, atomic_us = 7.08e-6;
    const int ntiles = div_up(s.nb, waves);
    const int bps = div_up(s.ts, ks);
    if (div_up(s.ts, bps) != ks) return -1.0;
    const long wgs = (long)ntiles * ks;
    const int rounds = (int)((wgs + cus - 1) / cus);
    *out = Plan{waves, ntiles, bps, ks};
    return rounds * (bps * waves * tile_us + group_us) + (ks > 1 ? atomic_us * (double)s.n * rows * ks : 0.0);
}

// `rows`: 8 for passes of up to 8 rows, 16 for larger ones (the two plans a handle keeps)
Plan choose_batch_plan(const Shape &s, int cus, int rows)
{
    const int wmax = lutgemm_kernels::batch_waves_max(s.gsub, s.q, s.qo), wmin = lutgemm_kernels::kBatchWavesMin;
    Plan best{wmax, div_up(s.nb, wmax), s.ts, 1};
    double best_cost = 1e30;
    for (int waves = wmin; waves <= wmax; waves++)
        for (int ks = 1; ks <= s.ts && ks <= kMaxSplits; ks++) {
            Plan p;
            const double cost = batch_plan_cost(s, cus, waves, ks, rows, &p);
            if (cost >= 0.0 && cost < best_cost) {
                best_cost = cost;
                best = p;
            }
        }
    return best;
}

static_assert(lutgemm_kernels::kBatchMaxPlanes == 8, "the batch kernel takes every plane count a weight can have");

// Launch shape of several independent batches in one grid (lutgemm_matvec_many): one number of
// wavefronts per workgroup and one number of k-blocks per workgroup for all entries.  The grid
// runs in rounds of one workgroup per compute unit.  A workgroup costs a time per tile (more when
// every wavefront stages two activation rows), a little per k-block, and a start and end of its own
// that grows with its wavefronts (first tiles, the wait for the slowest wavefront);
// the split-k atomics cost by their number in the whole launch (rows x outputs x k-splits), as
// the memory side executes them at a fixed rate.  Constants (microseconds) fitted to measured
// times of 330 plans over eight lists (3 to 12 entries, k and n 2048 to 12288, 1 to 4 planes,
// 4 to 16 rows) on MI355X; the fit names the fastest measured plan of each list.
FusedPlan choose_fused_batch_plan(const Shape *const *shapes, const int *rows, int count, int cus,
                                  std::vector<FusedCandidate> *all = nullptr)
{
    const double tile_us = 0.110, two_rows = 1.165, block_us = 0.35, group_us = 3.0, group_wave_us = 0.30;
    const double atomic_us = 2.5e-6;
    int max_ts = 1, wmax = lutgemm_kernels::kBatchWaves;
    for (int e = 0; e < count; e++) {
        max_ts = shapes[e]->ts > max_ts ? shapes[e]->ts : max_ts;
        const int w = lutgemm_kernels::batch_waves_max(shapes[e]->gsub, shapes[e]->q, shapes[e]->qo);
        wmax = w < wmax ? w : wmax;
    }
    FusedPlan best{wmax, max_ts};
    double best_cost = 1e300;
    for (int waves = lutgemm_kernels::kBatchWavesMin; waves <= wmax; waves++)
        for (int bpg = div_up(max_ts, kMaxSplits); bpg <= max_ts; bpg++) {
            long groups = 0;
            double work = 0.0;     // summed time of all workgroups
            double atomics = 0.0;  // 64-bit atomics of the launch
            for (int e = 0; e < count; e++) {
                const Shape &s = *shapes[e];
                const int b = bpg < s.ts ? bpg : s.ts;
                const int ks = div_up(s.ts, b);
                const long g = (long)div_up(s.nb, waves) * ks;
                const double tile = tile_us * s.q * (rows[e] > waves ? two_rows : 1.0);
                groups += g;
                work += (double)g * (b * (waves * tile + block_us) + group_us + group_wave_us * waves);
                if (ks > 1) atomics += (double)s.n * rows[e] * ks;
            }
            const double per_group = work / (double)groups;
            const long rounds = (groups + cus - 1) / cus;
            const double cost = (double)rounds * per_group + atomic_us * atomics;
            if (all) all->push_back(FusedCandidate{cost, FusedPlan{waves, bpg}});
            if (cost < best_cost - 1e-9) {
                best_cost = cost;
                best = FusedPlan{waves, bpg};
            }
        }
    return best;
}

// A handle's device memory belongs to the device that was current when it was created.
int check_device(const lutgemm_weight *w)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev != w->device)
        return fail(LUTGEMM_ERR_NO_DEVICE, "the weight lives on device %d but device %d is current", w->device, dev);
    return LUTGEMM_OK;
}

size_t set_words(const lutgemm_weight *w) { return (size_t)kRowsPerPass * w->shape.nb * kBatch; }

// Work of `stream` is being recorded into a graph: nothing may allocate, synchronise or time there.
bool stream_capturing(void *stream)
{
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capturing) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return capturing != hipStreamCaptureStatusNone;
}

int refuse_capture(void *stream, const char *what)
{
    if (!stream_capturing(stream)) return LUTGEMM_OK;
    return fail(LUTGEMM_ERR_UNSUPPORTED, "%s synchronises with the device and cannot run on a stream under graph capture", what);
}

// Device memory of set i (idempotent).  Allocates: not for a stream that is being captured.
int alloc_set(lutgemm_weight *w, int i)
{
    StreamSet &t = w->set[i];
    if (!t.accum) {
        const size_t bytes = set_words(w) * sizeof(unsigned long long);
        hipError_t e = hipMalloc((void **)&t.accum, bytes);
        if (e != hipSuccess) return hip_fail(e, "hipMalloc(split-k accumulators)");
        e = hipMemset(t.accum, 0, bytes);
        if (e != hipSuccess) return hip_fail(e, "hipMemset(split-k accumulators)");
    }
    if (!t.xrows) {
        hipError_t e = hipMalloc(&t.xrows, (size_t)kStagedColumns * w->shape.k * sizeof(uint16_t));
        if (e != hipSuccess) return hip_fail(e, "hipMalloc(column staging)");
        t.xrows_cols = kStagedColumns;
    }
    return LUTGEMM_OK;
}

int alloc_workspace(lutgemm_weight *w)
{
    return alloc_set(w, 0);
}

size_t workspace_bytes(const lutgemm_weight *w)
{
    size_t bytes = 0;
    for (int i = 0; i < kStreamSlots; i++) {
        if (w->set[i].accum) bytes += set_words(w) * sizeof(unsigned long long);
        if (w->set[i].xrows) bytes += (size_t)w->set[i].xrows_cols * w->shape.k * sizeof(uint16_t);
    }
    return bytes;
}

// The set launches on `stream` use.  The first launch of a stream on this handle claims one.  The
// caller holds the set (a lease) until release_set: launches are issued outside the lock, and a set
// that another host thread is about to launch on must not be handed to a further stream meanwhile.
constexpr int kSetsLeased = -1;   // internal: nothing to take over only because other calls hold their sets right now

int stream_set_once(lutgemm_weight *w, void *stream, int *slot, bool last_attempt)
{
    bool leased_elsewhere = false;
    std::lock_guard<std::mutex> lock(w->slot_mutex);
    for (int i = 0; i < w->slots_used; i++)
        if (w->set[i].stream == stream) {
            w->set[i].last_use = ++w->use_clock;
            w->set[i].leases++;
            *slot = i;
            return LUTGEMM_OK;
        }
    int take = -1;
    if (w->slots_used < kStreamSlots) {
        take = w->slots_used;
        if ((!w->set[take].accum || !w->set[take].xrows) && stream_capturing(stream))
            return fail(LUTGEMM_ERR_UNSUPPORTED,
                        "the first launch of a stream on this handle allocates the stream's split-k words, which "
                        "graph capture forbids: launch once on the stream before capturing, or capture "
                        "lutgemm_matvec_static");
        if (int st = alloc_set(w, take)) return st;
        if (!w->set[take].done) {
            hipError_t e = hipEventCreateWithFlags(&w->set[take].done, hipEventDisableTiming);
            if (e != hipSuccess) return hip_fail(e, "hipEventCreate");
        }
        w->slots_used++;
    } else {
        // all sets serve a stream: take over the least recently used one whose latest launch is known to
        // have completed; failing that, the least recently used one with a recorded event, after making
        // `stream` wait for it.  A set under lease is not a candidate.
        int idle = -1, busy = -1;
        for (int i = 0; i < kStreamSlots; i++) {
            const StreamSet &t = w->set[i];
            if (t.leases > 0) leased_elsewhere = true;
            if (!t.done_valid || t.leases > 0) continue;
            if (hipEventQuery(t.done) == hipSuccess) {
                if (idle < 0 || t.last_use < w->set[idle].last_use) idle = i;
            } else if (busy < 0 || t.last_use < w->set[busy].last_use) {
                busy = i;
            }
        }
        (void)hipGetLastError();  // hipErrorNotReady from the queries is not a failure
        take = idle >= 0 ? idle : busy;
        if (take < 0 && leased_elsewhere && !last_attempt) return kSetsLeased;
        if (take < 0)
            return fail(LUTGEMM_ERR_UNSUPPORTED,
                        "%d streams use this handle and none of their sets can be taken over (launches under "
                        "graph capture are not tracked); use lutgemm_weight_clone for further streams or "
                        "lutgemm_weight_reset_workspace to release the sets", kStreamSlots);
        if (idle < 0) {
            if (stream_capturing(stream))   // a captured stream cannot wait for work outside its graph
                return fail(LUTGEMM_ERR_UNSUPPORTED,
                            "%d other streams are still using this handle's sets and a stream under graph capture "
                            "cannot wait for them: launch once on the stream before capturing, or give it a handle "
                            "of its own (lutgemm_weight_clone)", kStreamSlots);
            hipError_t e = hipStreamWaitEvent(static_cast<hipStream_t>(stream), w->set[take].done, 0);
            if (e != hipSuccess) return hip_fail(e, "hipStreamWaitEvent");
        }
    }
    w->set[take].stream = stream;
    w->set[take].done_valid = false;
    w->set[take].last_use = ++w->use_clock;
    w->set[take].leases = 1;
    *slot = take;
    return LUTGEMM_OK;
}

int stream_set(lutgemm_weight *w, void *stream, int *slot)
{
    // A lease lasts as long as another host thread needs to issue its launches: when that is all that
    // stands in the way of a take-over, try again shortly instead of failing.
    constexpr int kAttempts = 200000;
    for (int attempt = 0;; attempt++) {
        const int st = stream_set_once(w, stream, slot, attempt + 1 >= kAttempts);
        if (st != kSetsLeased) return st;
        std::this_thread::yield();
    }
}

// End of a lease.  `launched`: the call has issued work on the set.  Once the handle serves more than
// one stream, remember where the stream stands, so that the set can be handed to another stream later.
// A stream under capture records nothing (the event would belong to the graph); its set is then not
// handed on.
void release_set(lutgemm_weight *w, int slot, void *stream, bool launched)
{
    std::lock_guard<std::mutex> lock(w->slot_mutex);
    StreamSet &t = w->set[slot];
    if (t.leases > 0) t.leases--;
    if (!launched || w->slots_used < 2) return;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capturing) != hipSuccess ||
        capturing != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        t.done_valid = false;
        return;
    }
    t.done_valid = hipEventRecord(t.done, static_cast<hipStream_t>(stream)) == hipSuccess;
}

struct SetLease {
    lutgemm_weight *w = nullptr;
    int slot = 0;
    void *stream = nullptr;
    bool launched = false;
    SetLease() = default;
    SetLease(const SetLease &) = delete;
    SetLease &operator=(const SetLease &) = delete;
    ~SetLease()
    {
        if (w) release_set(w, slot, stream, launched);
    }
};

// The allocation-free entry point marks a device whose static split-k words a failed call may
// have left non-zero; the next call on that device clears them first.
std::atomic<bool> g_static_dirty[lutgemm_kernels::kMaxDevices];

// New handle for shape s on the current device from tiles already in the device layout
// (host or device memory, `kind` says which).
int create_from_tiles(const Shape &s, const void *signs, const void *scales, hipMemcpyKind kind,
                      lutgemm_weight **out)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(LUTGEMM_ERR_NO_DEVICE, "no HIP device available (%s)",
                    e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    int dev = 0;
    e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDeviceProperties");

    lutgemm_weight *w = new (std::nothrow) lutgemm_weight();
    if (!w) return fail(LUTGEMM_ERR_OUT_OF_MEMORY, "host allocation failed");
    w->shape = s;
    w->device = dev;
    w->compute_units = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;

    const size_t sb = sign_bytes(s), cb = scale_bytes(s);
    int st = LUTGEMM_OK;
    e = hipMalloc((void **)&w->d_signs, sb);
    if (e != hipSuccess) st = hip_fail(e, "hipMalloc(signs)");
    if (st == LUTGEMM_OK) {
        e = hipMalloc((void **)&w->d_scales, cb);
        if (e != hipSuccess) st = hip_fail(e, "hipMalloc(scales)");
    }
    if (st == LUTGEMM_OK) {
        e = hipMemcpy(w->d_signs, signs, sb, kind);
        if (e != hipSuccess) st = hip_fail(e, "hipMemcpy(signs)");
    }
    if (st == LUTGEMM_OK) {
        e = hipMemcpy(w->d_scales, scales, cb, kind);
        if (e != hipSuccess) st = hip_fail(e, "hipMemcpy(scales)");
    }
    if (st == LUTGEMM_OK) {
        w->plan = w->plan2 = choose_plan(s, w->compute_units);
        w->batch_measured[0] = w->batch_measured[1] = false;
        st = alloc_workspace(w);
    }
    if (st != LUTGEMM_OK) {
        lutgemm_weight_destroy(w);
        return st;
    }
    *out = w;
    return LUTGEMM_OK;
}

void fill_info(const Shape &s, size_t workspace, lutgemm_weight_info_t *info)
{
    info->k = s.k;
    info->n = s.n;
    info->q = s.q;
    info->num_groups = s.num_groups;
    info->group_size = s.group_size;
    info->has_offset = s.has_offset;
    info->sign_bytes = (size_t)s.k / 8 * s.q * s.n;
    info->scale_bytes = (size_t)s.num_groups * s.q * s.n * 2;
    info->offset_bytes = s.has_offset ? (size_t)s.num_groups * s.n * 2 : 0;
    info->device_bytes = sign_bytes(s) + scale_bytes(s) + workspace;
}

int shape_or_fail(int k, int n, int q, int num_groups, bool has_offset, Shape *s)
{
    if (!make_shape(k, n, q, num_groups, has_offset, s))
        return fail(LUTGEMM_ERR_BAD_SHAPE,
                    "bad shape k=%d n=%d q=%d num_groups=%d (need k%%32==0, 1<=q<=8, "
                    "k%%num_groups==0, (k/num_groups)%%32==0)",
                    k, n, q, num_groups);
    return LUTGEMM_OK;
}

int pack_to_host(const Shape &s, const uint32_t *bW, const uint16_t *alpha_h, const uint16_t *q_bias_h,
                 std::vector<uint8_t> *signs, std::vector<uint16_t> *scales)
{
    try {
        signs->resize(sign_bytes(s));
        scales->resize(scale_bytes(s) / 2);
    } catch (const std::bad_alloc &) {
        return fail(LUTGEMM_ERR_OUT_OF_MEMORY, "host staging allocation failed (%zu bytes)",
                    sign_bytes(s) + scale_bytes(s));
    }
    lutgemm_packer::pack(s, bW, alpha_h, q_bias_h, signs->data(), scales->data());
    return LUTGEMM_OK;
}

int create_common(const uint32_t *bW, const uint16_t *alpha_h, const uint16_t *q_bias_h, int k, int n,
                  int q, int num_groups, lutgemm_weight **out)
{
    Shape s;
    int st = shape_or_fail(k, n, q, num_groups, q_bias_h != nullptr, &s);
    if (st != LUTGEMM_OK) return st;
    std::vector<uint8_t> signs;
    std::vector<uint16_t> scales;
    st = pack_to_host(s, bW, alpha_h, q_bias_h, &signs, &scales);
    if (st != LUTGEMM_OK) return st;
    return create_from_tiles(s, signs.data(), scales.data(), hipMemcpyHostToDevice, out);
}

// Packed-weight file: 64-byte little-endian header, the sign tiles, the scale tiles.
constexpr char kFileMagic[8] = {'L', 'U', 'T', 'G', 'E', 'M', 'M', 'W'};
constexpr uint32_t kFileVersion = 1;
// identifies the tile layout: lanes, chunk, batch (a file written for another tiling is refused)
constexpr uint32_t kFileLayout = (uint32_t)kLanes | ((uint32_t)kChunk << 8) | ((uint32_t)kBatch << 16);
struct FileHeader {
    char magic[8];
    uint32_t version, layout;
    uint32_t k, n, q, num_groups, has_offset, reserved;
    uint64_t sign_bytes, scale_bytes;
    uint64_t pad[1];
};
static_assert(sizeof(FileHeader) == 64, "file header is 64 bytes");

int write_file(const char *path, const Shape &s, const void *signs, const void *scales)
{
    FILE *f = std::fopen(path, "wb");
    if (!f) return fail(LUTGEMM_ERR_IO, "cannot open %s for writing", path);
    FileHeader h{};
    std::memcpy(h.magic, kFileMagic, 8);
    h.version = kFileVersion;
    h.layout = kFileLayout;
    h.k = (uint32_t)s.k;
    h.n = (uint32_t)s.n;
    h.q = (uint32_t)s.q;
    h.num_groups = (uint32_t)s.num_groups;
    h.has_offset = (uint32_t)s.has_offset;
    h.sign_bytes = sign_bytes(s);
    h.scale_bytes = scale_bytes(s);
    bool ok = std::fwrite(&h, sizeof(h), 1, f) == 1;
    ok = ok && std::fwrite(signs, 1, h.sign_bytes, f) == h.sign_bytes;
    ok = ok && std::fwrite(scales, 1, h.scale_bytes, f) == h.scale_bytes;
    ok = (std::fclose(f) == 0) && ok;
    if (!ok) return fail(LUTGEMM_ERR_IO, "short write to %s", path);
    return LUTGEMM_OK;
}

int read_file(const char *path, Shape *s, std::vector<uint8_t> *signs, std::vector<uint16_t> *scales)
{
    FILE *f = std::fopen(path, "rb");
    if (!f) return fail(LUTGEMM_ERR_IO, "cannot open %s", path);
    FileHeader h{};
    int st = LUTGEMM_OK;
    if (std::fread(&h, sizeof(h), 1, f) != 1 || std::memcmp(h.magic, kFileMagic, 8) != 0)
        st = fail(LUTGEMM_ERR_IO, "%s is not a packed-weight file", path);
    else if (h.version != kFileVersion || h.layout != kFileLayout)
        st = fail(LUTGEMM_ERR_IO, "%s: file version %u / layout 0x%x, this library reads %u / 0x%x", path,
                  h.version, h.layout, kFileVersion, kFileLayout);
    else if (h.k > 0x7fffffffu || h.n > 0x7fffffffu ||
             !make_shape((int)h.k, (int)h.n, (int)h.q, (int)h.num_groups, h.has_offset != 0, s) ||
             h.sign_bytes != sign_bytes(*s) || h.scale_bytes != scale_bytes(*s))
        st = fail(LUTGEMM_ERR_IO, "%s: inconsistent header", path);
    if (st == LUTGEMM_OK) {
        try {
            signs->resize(h.sign_bytes);
            scales->resize(h.scale_bytes / 2);
        } catch (const std::bad_alloc &) {
            st = fail(LUTGEMM_ERR_OUT_OF_MEMORY, "host staging allocation failed");
        }
    }
    if (st == LUTGEMM_OK && (std::fread(signs->data(), 1, h.sign_bytes, f) != h.sign_bytes ||
                             std::fread(scales->data(), 1, h.scale_bytes, f) != h.scale_bytes))
        st = fail(LUTGEMM_ERR_IO, "%s is truncated", path);
    std::fclose(f);
    return st;
}

// `static_ws`: take the split-k words from the static device array instead of the handle's
// per-stream sets (rows form only; nothing on this route allocates).
int run_matvec(const lutgemm_weight *w, const void *x, void *y, int m, void *stream, bool cols, bool static_ws)
{
    if (!w || !x || !y) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to matvec");
    if (m < 1 || m > LUTGEMM_MAX_BATCH)
        return fail(LUTGEMM_ERR_BAD_SHAPE, "m=%d outside 1..%d", m, LUTGEMM_MAX_BATCH);
    if (int st_dev = check_device(w)) return st_dev;
    const Shape &s = w->shape;
    lutgemm_weight *mw = const_cast<lutgemm_weight *>(w);
    lutgemm_kernels::MatvecArgs a{};
    a.signs = w->d_signs;
    a.scales = w->d_scales;
    a.k = s.k;
    a.n = s.n;
    a.ts = s.ts;
    a.nb = s.nb;
    const uint16_t *xh = static_cast<const uint16_t *>(x);
    uint16_t *yh = static_cast<uint16_t *>(y);
    if (((uintptr_t)x & 15u) != 0)  // rows of x are k fp16 apart and k is a multiple of 32
        return fail(LUTGEMM_ERR_BAD_SHAPE, "x must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    int slot = 0;
    SetLease lease;   // ends when this call returns
    if (static_ws) {
        const size_t words = lutgemm_kernels::kStaticSplitKWords;
        if ((size_t)kRowsPerPass * s.nb * kBatch > words)
            return fail(LUTGEMM_ERR_UNSUPPORTED,
                        "n=%d is beyond what the static workspace holds (%zu outputs per activation row)", s.n,
                        words / kRowsPerPass);
        hipError_t es = lutgemm_kernels::static_split_k_words(w->device, &a.accum);
        if (es != hipSuccess) return hip_fail(es, "hipGetSymbolAddress(static split-k words)");
        if (g_static_dirty[w->device].exchange(false)) {  // a launch failed half way through a call: start from zero again
            hipError_t e = lutgemm_kernels::launch_fill_zero(a.accum, words, st);
            if (e != hipSuccess) {
                g_static_dirty[w->device] = true;
                return hip_fail(e, "launch fill_zero_kernel");
            }
        }
    } else {
        if (int st_ws = stream_set(mw, stream, &slot)) return st_ws;
        lease.w = mw;
        lease.slot = slot;
        lease.stream = stream;
        a.accum = mw->set[slot].accum;
    }
    if (cols && m > 1) {
        // gather the m columns into contiguous rows first (the kernel reads 16 bytes per lane); the
        // staging rows belong to the stream's set, or, for the allocation-free entry point, to set 0
        StreamSet &t = mw->set[slot];
        if (m > t.xrows_cols) {
            if (stream_capturing(stream))
                return fail(LUTGEMM_ERR_UNSUPPORTED,
                            "m=%d columns need larger staging rows than the stream's set holds (%d), and graph capture "
                            "forbids the allocation: call once with this m before capturing", m, t.xrows_cols);
            // earlier launches of this stream may still read the old buffer
            hipError_t e = hipStreamSynchronize(st);
            if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
            std::lock_guard<std::mutex> lock(mw->slot_mutex);
            if (t.xrows) (void)hipFree(t.xrows);
            t.xrows = nullptr;
            t.xrows_cols = 0;
            e = hipMalloc(&t.xrows, (size_t)m * s.k * sizeof(uint16_t));
            if (e != hipSuccess) return hip_fail(e, "hipMalloc(column staging)");
            t.xrows_cols = m;
        }
        uint16_t *rows = static_cast<uint16_t *>(t.xrows);
        hipError_t e = lutgemm_kernels::launch_gather_columns(x, rows, s.k, m, st);
        if (e != hipSuccess) return hip_fail(e, "launch gather_columns_kernel");
        lease.launched = true;
        xh = rows;
    }
    a.x_row_stride = s.k;
    a.accum_row_stride = (long long)s.nb * kBatch;
    if (m >= 3) {
        // up to 16 rows per pass over the weight on the matrix cores
        const int pass_rows = m < kRowsPerPass ? m : kRowsPerPass;
        const Plan plan = w->batch_measured[pass_rows > 8] ? w->plan_batch[pass_rows > 8]
                                                            : choose_batch_plan(s, w->compute_units, pass_rows > 8 ? kRowsPerPass : 8);
        a.ntiles = plan.ntiles;
        a.k_splits = plan.k_splits;
        a.blocks_per_split = plan.blocks_per_split;
        for (int r = 0; r < m; r += kRowsPerPass) {
            a.rows = m - r < kRowsPerPass ? m - r : kRowsPerPass;
            a.x = xh + (size_t)r * s.k;
            if (cols) {  // y [n][m]
                a.y = yh + r;
                a.y_stride = m;
                a.y_row_stride = 1;
            } else {     // y [m][n]
                a.y = yh + (size_t)r * s.n;
                a.y_stride = 1;
                a.y_row_stride = s.n;
            }
            hipError_t e = lutgemm_kernels::launch_batch(s.q, s.has_offset, s.gsub, a, plan.ntiles * plan.k_splits, plan.waves, st);
            if (e != hipSuccess) {
                if (static_ws && r > 0) g_static_dirty[w->device] = true;
                return hip_fail(e, "launch lut_batch_kernel");
            }
            lease.launched = true;
        }
        return LUTGEMM_OK;
    }
    // two activation rows per pass over the weight, a last single row if m is odd
    for (int r = 0; r < m; r += 2) {
        a.rows = m - r >= 2 ? 2 : 1;
        const Plan &plan = a.rows == 2 ? w->plan2 : w->plan;
        a.ntiles = plan.ntiles;
        a.k_splits = plan.k_splits;
        a.blocks_per_split = plan.blocks_per_split;
        a.x = xh + (size_t)r * s.k;
        if (cols) {  // y [n][m]
            a.y = yh + r;
            a.y_stride = m;
            a.y_row_stride = 1;
        } else {     // y [m][n]
            a.y = yh + (size_t)r * s.n;
            a.y_stride = 1;
            a.y_row_stride = s.n;
        }
        hipError_t e = lutgemm_kernels::launch_matvec(s.q, s.has_offset, s.gsub, a, plan.ntiles * plan.k_splits,
                                                      plan.waves, st);
        if (e != hipSuccess) {
            if (static_ws && r > 0) g_static_dirty[w->device] = true;
            return hip_fail(e, "launch lut_matvec_kernel");
        }
        lease.launched = true;
    }
    return LUTGEMM_OK;
}

// ---- runs of independent entries that share one launch (lutgemm_matvec_many) ----------------
// kind: 1 one-row entries, 3 two-row entries (table-lookup kernels), 2 batches of 3 to 16 rows (the
// batch kernel); an entry of more than 16 rows is launched on its own.
struct FusedRun {
    int kind, count;
    lutgemm_kernels::MultiMatvecArgs multi;
    const lutgemm_weight *handle[lutgemm_kernels::kMaxFused];
    const Shape *shape[lutgemm_kernels::kMaxFused];
    int rows[lutgemm_kernels::kMaxFused];
};

int fused_kind(int m)
{
    if (m == 1) return 1;
    if (m == 2) return 3;
    if (m >= 3 && m <= kRowsPerPass) return 2;
    return 0;
}

// Longest run of entries starting at i that one launch can take: the same kind and kernel
// instance, no handle twice (its split-k words would be shared), and no output overlapping an
// input or output of another entry of the run, so that their order does not matter.  Returns the
// index behind the run (run->count is 0 when entry i cannot share a launch at all).
int form_run(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys, const int *ms, int count, int i,
             FusedRun *run)
{
    struct Range { uintptr_t lo, hi; };
    auto overlap = [](const Range &a, const Range &b) { return a.lo < b.hi && b.lo < a.hi; };
    Range xr[lutgemm_kernels::kMaxFused], yr[lutgemm_kernels::kMaxFused];
    run->multi = lutgemm_kernels::MultiMatvecArgs{};
    int j = i;
    const lutgemm_weight *w0 = ws[i];
    const int kind = w0 && xs[i] && ys[i] ? fused_kind(ms[i]) : 0;
    for (; kind != 0 && j < count && j - i < lutgemm_kernels::kMaxFused; j++) {
        const lutgemm_weight *w = ws[j];
        if (!w || !xs[j] || !ys[j] || ((uintptr_t)xs[j] & 15u) != 0 || fused_kind(ms[j]) != kind) break;
        const Shape &s = w->shape;
        if (s.q != w0->shape.q || s.has_offset != w0->shape.has_offset || s.gsub != w0->shape.gsub ||
            w->device != w0->device)
            break;
        const int e = j - i;
        xr[e] = Range{(uintptr_t)xs[j], (uintptr_t)xs[j] + (size_t)ms[j] * s.k * 2};
        yr[e] = Range{(uintptr_t)ys[j], (uintptr_t)ys[j] + (size_t)ms[j] * s.n * 2};
        bool independent = true;
        for (int p = 0; p < e && independent; p++)
            independent = ws[i + p] != w && !overlap(yr[e], yr[p]) && !overlap(yr[e], xr[p]) && !overlap(xr[e], yr[p]);
        if (!independent) break;
        run->handle[e] = w;
        run->shape[e] = &s;
        run->rows[e] = ms[j];
        lutgemm_kernels::MatvecArgs &a = run->multi.entry[e];
        a.signs = w->d_signs;
        a.scales = w->d_scales;
        a.k = s.k;
        a.n = s.n;
        a.ts = s.ts;
        a.nb = s.nb;
        a.x = xs[j];
        a.y = ys[j];
        a.y_stride = 1;
        a.rows = ms[j];
        a.x_row_stride = s.k;
        a.y_row_stride = s.n;
        a.accum_row_stride = (long long)s.nb * kBatch;
    }
    run->kind = kind;
    run->count = j - i;
    return j;
}

FusedPlan model_fused_plan(const FusedRun &run, std::vector<FusedCandidate> *all)
{
    const int cus = run.handle[0]->compute_units;
    return run.kind == 2 ? choose_fused_batch_plan(run.shape, run.rows, run.count, cus, all)
                         : choose_fused_plan(run.shape, run.count, cus, run.kind == 1 ? 1 : 2, all);
}

// two plans that give every entry of the run the same grid
bool same_launch(const FusedRun &run, const FusedPlan &a, const FusedPlan &b)
{
    if (a.waves != b.waves) return false;
    for (int e = 0; e < run.count; e++) {
        const int ts = run.shape[e]->ts;
        if ((a.blocks_per_group < ts ? a.blocks_per_group : ts) != (b.blocks_per_group < ts ? b.blocks_per_group : ts)) return false;
    }
    return true;
}

// Launch shapes measured by lutgemm_matvec_many_autotune, by what a run looks like: kind, kernel
// instance, compute units and the (k, n, rows) of its entries in order.  Any list with the same
// shapes finds the plan again, whatever its handles and buffers.
constexpr size_t kFusedCandidates = 6;
std::mutex g_fused_mutex;
std::map<std::vector<int>, FusedPlan> g_fused_plans;

std::vector<int> fused_key(const FusedRun &run)
{
    const Shape &s0 = *run.shape[0];
    std::vector<int> key = {run.kind, s0.q, s0.has_offset, s0.gsub, run.handle[0]->compute_units, run.count};
    for (int e = 0; e < run.count; e++) {
        key.push_back(run.shape[e]->k);
        key.push_back(run.shape[e]->n);
        key.push_back(run.rows[e]);
    }
    return key;
}

bool measured_fused_plan(const FusedRun &run, FusedPlan *out)
{
    std::lock_guard<std::mutex> lock(g_fused_mutex);
    if (g_fused_plans.empty()) return false;
    const auto it = g_fused_plans.find(fused_key(run));
    if (it == g_fused_plans.end()) return false;
    *out = it->second;
    return true;
}

void remember_fused_plan(const FusedRun &run, const FusedPlan &plan)
{
    std::lock_guard<std::mutex> lock(g_fused_mutex);
    g_fused_plans[fused_key(run)] = plan;
}

// One launch for the run with launch shape fp (asynchronous).
int launch_run(FusedRun &run, const FusedPlan &fp, void *stream)
{
    const Shape &s0 = *run.shape[0];
    int slots[lutgemm_kernels::kMaxFused];
    SetLease leases[lutgemm_kernels::kMaxFused];   // end when this call returns
    int blocks = 0;
    for (int e = 0; e < run.count; e++) {
        lutgemm_kernels::MatvecArgs &a = run.multi.entry[e];
        a.ntiles = div_up(a.nb, fp.waves);
        a.blocks_per_split = fp.blocks_per_group < a.ts ? fp.blocks_per_group : a.ts;
        a.k_splits = div_up(a.ts, a.blocks_per_split);
        run.multi.first_block[e] = blocks;
        blocks += a.ntiles * a.k_splits;
        lutgemm_weight *we = const_cast<lutgemm_weight *>(run.handle[e]);
        if (int st_ws = stream_set(we, stream, &slots[e])) return st_ws;
        leases[e].w = we;
        leases[e].slot = slots[e];
        leases[e].stream = stream;
        a.accum = we->set[slots[e]].accum;
    }
    run.multi.count = run.count;
    hipError_t e = run.kind != 2 ? lutgemm_kernels::launch_matvec_multi(s0.q, s0.has_offset, s0.gsub, run.multi, blocks, fp.waves,
                                                                       static_cast<hipStream_t>(stream))
                                 : lutgemm_kernels::launch_batch_multi(s0.q, s0.has_offset, s0.gsub, run.multi, blocks, fp.waves,
                                                                       static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, run.kind != 2 ? "launch lut_matvec_multi_kernel" : "launch lut_batch_multi_kernel");
    for (int en = 0; en < run.count; en++) leases[en].launched = true;
    return LUTGEMM_OK;
}

}  // namespace

extern "C" {

int lutgemm_weight_create_f16(const uint32_t *bW, const uint16_t *alpha, const uint16_t *q_bias, int k,
                              int n, int q, int num_groups, lutgemm_weight **out)
{
    if (!bW || !alpha || !out) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_create");
    *out = nullptr;
    return create_common(bW, alpha, q_bias, k, n, q, num_groups, out);
}

int lutgemm_weight_create(const uint32_t *bW, const float *alpha, const float *q_bias, int k, int n, int q,
                          int num_groups, lutgemm_weight **out)
{
    if (!bW || !alpha || !out) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_create");
    *out = nullptr;
    Shape s;
    if (!make_shape(k, n, q, num_groups, q_bias != nullptr, &s))
        return fail(LUTGEMM_ERR_BAD_SHAPE,
                    "bad shape k=%d n=%d q=%d num_groups=%d (need k%%32==0, 1<=q<=8, "
                    "k%%num_groups==0, (k/num_groups)%%32==0)",
                    k, n, q, num_groups);
    std::vector<uint16_t> ah, zh;
    try {
        ah.resize((size_t)num_groups * q * n);
        if (q_bias) zh.resize((size_t)num_groups * n);
    } catch (const std::bad_alloc &) {
        return fail(LUTGEMM_ERR_OUT_OF_MEMORY, "host allocation failed");
    }
    lutgemm_packer::floats_to_halves(alpha, ah.data(), ah.size());
    if (q_bias) lutgemm_packer::floats_to_halves(q_bias, zh.data(), zh.size());
    return create_common(bW, ah.data(), q_bias ? zh.data() : nullptr, k, n, q, num_groups, out);
}

int lutgemm_weight_clone(const lutgemm_weight *w, lutgemm_weight **out)
{
    if (!w || !out) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_clone");
    *out = nullptr;
    if (int st_dev = check_device(w)) return st_dev;
    int st = create_from_tiles(w->shape, w->d_signs, w->d_scales, hipMemcpyDeviceToDevice, out);
    if (st == LUTGEMM_OK) {
        (*out)->plan = w->plan;
        (*out)->plan2 = w->plan2;
        for (int i = 0; i < 2; i++) {
            (*out)->plan_batch[i] = w->plan_batch[i];
            (*out)->batch_measured[i] = w->batch_measured[i];
        }
    }
    return st;
}

int lutgemm_weight_save(const lutgemm_weight *w, const char *path)
{
    if (!w || !path) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_save");
    const Shape &s = w->shape;
    std::vector<uint8_t> signs;
    std::vector<uint16_t> scales;
    try {
        signs.resize(sign_bytes(s));
        scales.resize(scale_bytes(s) / 2);
    } catch (const std::bad_alloc &) {
        return fail(LUTGEMM_ERR_OUT_OF_MEMORY, "host staging allocation failed");
    }
    hipError_t e = hipMemcpy(signs.data(), w->d_signs, signs.size(), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "hipMemcpy(signs)");
    e = hipMemcpy(scales.data(), w->d_scales, scales.size() * 2, hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "hipMemcpy(scales)");
    return write_file(path, s, signs.data(), scales.data());
}

int lutgemm_weight_load(const char *path, lutgemm_weight **out)
{
    if (!path || !out) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_load");
    *out = nullptr;
    Shape s;
    std::vector<uint8_t> signs;
    std::vector<uint16_t> scales;
    int st = read_file(path, &s, &signs, &scales);
    if (st != LUTGEMM_OK) return st;
    return create_from_tiles(s, signs.data(), scales.data(), hipMemcpyHostToDevice, out);
}

int lutgemm_pack_file(const uint32_t *bW, const uint16_t *alpha, const uint16_t *q_bias, int k, int n, int q,
                      int num_groups, const char *path)
{
    if (!bW || !alpha || !path) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to pack_file");
    Shape s;
    int st = shape_or_fail(k, n, q, num_groups, q_bias != nullptr, &s);
    if (st != LUTGEMM_OK) return st;
    std::vector<uint8_t> signs;
    std::vector<uint16_t> scales;
    st = pack_to_host(s, bW, alpha, q_bias, &signs, &scales);
    if (st != LUTGEMM_OK) return st;
    return write_file(path, s, signs.data(), scales.data());
}

int lutgemm_unpack_file(const char *path, uint32_t *bW, uint16_t *alpha, uint16_t *q_bias,
                        lutgemm_weight_info_t *info)
{
    if (!path) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to unpack_file");
    Shape s;
    std::vector<uint8_t> signs;
    std::vector<uint16_t> scales;
    int st = read_file(path, &s, &signs, &scales);
    if (st != LUTGEMM_OK) return st;
    if (info) fill_info(s, 0, info);
    if (bW || alpha || q_bias)
        lutgemm_packer::unpack(s, signs.data(), scales.data(), bW, alpha, s.has_offset ? q_bias : nullptr);
    return LUTGEMM_OK;
}

int lutgemm_weight_destroy(lutgemm_weight *w)
{
    if (!w) return LUTGEMM_OK;
    int st = LUTGEMM_OK;
    std::vector<void *> ptrs = {w->d_signs, w->d_scales};
    for (StreamSet &t : w->set) {
        ptrs.push_back(t.accum);
        ptrs.push_back(t.xrows);
        if (t.done) (void)hipEventDestroy(t.done);
    }
    for (void *p : ptrs)
        if (p) {
            hipError_t e = hipFree(p);
            if (e != hipSuccess) st = hip_fail(e, "hipFree");
        }
    delete w;
    return st;
}

int lutgemm_weight_info(const lutgemm_weight *w, lutgemm_weight_info_t *info)
{
    if (!w || !info) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_info");
    fill_info(w->shape, workspace_bytes(w), info);
    return LUTGEMM_OK;
}

int lutgemm_matvec(const lutgemm_weight *w, const void *x, void *y, int m, void *stream)
{
    return run_matvec(w, x, y, m, stream, false, false);
}

int lutgemm_matvec_static(const lutgemm_weight *w, const void *x, void *y, int m, void *stream)
{
    return run_matvec(w, x, y, m, stream, false, true);
}

int lutgemm_weight_reset_workspace(lutgemm_weight *w, void *stream)
{
    if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_reset_workspace");
    if (int st_dev = check_device(w)) return st_dev;
    if (int st_cap = refuse_capture(stream, "lutgemm_weight_reset_workspace")) return st_cap;
    std::lock_guard<std::mutex> lock(w->slot_mutex);
    hipError_t e = hipDeviceSynchronize();  // no launch may still be using the words
    if (e != hipSuccess) return hip_fail(e, "hipDeviceSynchronize");
    for (StreamSet &t : w->set) {
        t.stream = nullptr;
        t.done_valid = false;
        if (!t.accum) continue;
        e = lutgemm_kernels::launch_fill_zero(t.accum, set_words(w), static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return hip_fail(e, "launch fill_zero_kernel");
    }
    e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    w->slots_used = 0;
    return LUTGEMM_OK;
}

int lutgemm_matvec_cols(const lutgemm_weight *w, const void *x, void *y, int m, void *stream)
{
    return run_matvec(w, x, y, m, stream, true, false);
}

int lutgemm_matvec_each(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys,
                        const int *ms, int count, void *stream)
{
    if (!ws || !xs || !ys || !ms) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to matvec_each");
    if (count < 0) return fail(LUTGEMM_ERR_BAD_SHAPE, "count=%d is negative", count);
    for (int i = 0; i < count; i++) {
        int st = run_matvec(ws[i], xs[i], ys[i], ms[i], stream, false, false);
        if (st != LUTGEMM_OK) return st;
    }
    return LUTGEMM_OK;
}

int lutgemm_matvec_many(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys,
                        const int *ms, int count, void *stream)
{
    if (!ws || !xs || !ys || !ms) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to matvec_many");
    if (count < 0) return fail(LUTGEMM_ERR_BAD_SHAPE, "count=%d is negative", count);
    int i = 0;
    while (i < count) {
        FusedRun run;
        const int j = form_run(ws, xs, ys, ms, count, i, &run);
        if (run.count < 2) {
            int st = run_matvec(ws[i], xs[i], ys[i], ms[i], stream, false, false);
            if (st != LUTGEMM_OK) return st;
            i++;
            continue;
        }
        if (int st_dev = check_device(ws[i])) return st_dev;
        FusedPlan fp;
        if (!measured_fused_plan(run, &fp)) fp = model_fused_plan(run, nullptr);
        if (int st = launch_run(run, fp, stream)) return st;
        i = j;
    }
    return LUTGEMM_OK;
}

int lutgemm_matvec_many_autotune(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys,
                                 const int *ms, int count, void *stream)
{
    if (!ws || !xs || !ys || !ms) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to matvec_many_autotune");
    if (count < 0) return fail(LUTGEMM_ERR_BAD_SHAPE, "count=%d is negative", count);
    if (int st_cap = refuse_capture(stream, "lutgemm_matvec_many_autotune")) return st_cap;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t he = hipEventCreate(&e0);
    if (he == hipSuccess) he = hipEventCreate(&e1);
    int status = he == hipSuccess ? LUTGEMM_OK : hip_fail(he, "hipEventCreate");
    int i = 0;
    while (status == LUTGEMM_OK && i < count) {
        FusedRun run;
        const int j = form_run(ws, xs, ys, ms, count, i, &run);
        if (run.count < 2) {   // launched on its own: the handle's plan applies (lutgemm_weight_autotune)
            status = run_matvec(ws[i], xs[i], ys[i], ms[i], stream, false, false);
            i++;
            continue;
        }
        status = check_device(ws[i]);
        if (status != LUTGEMM_OK) break;
        // the launch shapes the model ranks best, measured on the entries themselves
        std::vector<FusedCandidate> cands;
        const FusedPlan model = model_fused_plan(run, &cands);
        std::sort(cands.begin(), cands.end(), [](const FusedCandidate &a, const FusedCandidate &b) { return a.cost < b.cost; });
        // plans that differ only in k-blocks per workgroup beyond every entry's k-blocks are one launch shape
        std::vector<FusedPlan> plans;
        for (const FusedCandidate &c : cands) {
            bool seen = false;
            for (const FusedPlan &p : plans) seen = seen || same_launch(run, p, c.plan);
            if (!seen) plans.push_back(c.plan);
            if (plans.size() == kFusedCandidates) break;
        }
        auto time_plan = [&](const FusedPlan &p, int reps, float *us) -> int {
            int stt = launch_run(run, p, stream);   // untimed: first touch of this shape
            hipError_t e = hipEventRecord(e0, st);
            for (int r = 0; r < reps && stt == LUTGEMM_OK; r++) stt = launch_run(run, p, stream);
            if (stt != LUTGEMM_OK) return stt;
            if (e == hipSuccess) e = hipEventRecord(e1, st);
            if (e == hipSuccess) e = hipEventSynchronize(e1);
            float ms_ = 0.f;
            if (e == hipSuccess) e = hipEventElapsedTime(&ms_, e0, e1);
            if (e != hipSuccess) return hip_fail(e, "fused autotune timing");
            *us = ms_ * 1e3f / (float)reps;
            return LUTGEMM_OK;
        };
        // clocks up first (the candidates measured first would look slow), then two sweeps, the
        // minimum of which counts; the model's own choice is among the candidates (it ranks first)
        {
            const auto t0 = std::chrono::steady_clock::now();
            float us = 0.f;
            while (status == LUTGEMM_OK && std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < 0.03)
                status = time_plan(model, 8, &us);
        }
        std::vector<float> best(plans.size(), 1e30f);
        for (int sweep = 0; sweep < 3 && status == LUTGEMM_OK; sweep++)
            for (size_t c = 0; c < plans.size() && status == LUTGEMM_OK; c++) {
                float us = 0.f;
                status = time_plan(plans[c], 6, &us);
                if (status == LUTGEMM_OK && us < best[c]) best[c] = us;
            }
        if (status == LUTGEMM_OK) {
            // plans[0] is the model's own choice (lowest cost): another shape replaces it only if it
            // measured at least 2 % faster, so that timing noise does not trade it for an equal one
            size_t pick = 0;
            for (size_t c = 1; c < plans.size(); c++)
                if (best[c] < best[pick] && best[c] < 0.98f * best[0]) pick = c;
            remember_fused_plan(run, plans[pick]);
        }
        i = j;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    return status;
}

int lutgemm_matvec_many_plan(const lutgemm_weight *const *ws, const void *const *xs, void *const *ys,
                             const int *ms, int count, int *entries_in_first_launch, int *waves_per_group,
                             int *k_blocks_per_group, int *measured)
{
    if (!ws || !xs || !ys || !ms) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to matvec_many_plan");
    if (count < 1) return fail(LUTGEMM_ERR_BAD_SHAPE, "count=%d: no entry to plan", count);
    FusedRun run;
    form_run(ws, xs, ys, ms, count, 0, &run);
    if (entries_in_first_launch) *entries_in_first_launch = run.count < 2 ? 1 : run.count;
    FusedPlan fp{0, 0};
    bool have = false;
    if (run.count >= 2) {
        have = measured_fused_plan(run, &fp);
        if (!have) fp = model_fused_plan(run, nullptr);
    }
    if (waves_per_group) *waves_per_group = fp.waves;
    if (k_blocks_per_group) *k_blocks_per_group = fp.blocks_per_group;
    if (measured) *measured = have ? 1 : 0;
    return LUTGEMM_OK;
}

int lutgemm_dequantize(const lutgemm_weight *w, void *d_fW, int transposed, void *stream)
{
    if (!w || !d_fW) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to dequantize");
    if (int st_dev = check_device(w)) return st_dev;
    const Shape &s = w->shape;
    lutgemm_kernels::DequantArgs a{};
    a.signs = w->d_signs;
    a.scales = w->d_scales;
    a.out = d_fW;
    a.k = s.k;
    a.n = s.n;
    a.q = s.q;
    a.has_offset = s.has_offset;
    a.gsub = s.gsub;
    a.ts = s.ts;
    a.transposed = transposed ? 1 : 0;
    hipError_t e = lutgemm_kernels::launch_dequantize(a, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "launch dequantize_kernel");
    return LUTGEMM_OK;
}

int lutgemm_read_probe(const lutgemm_weight *const *ws, int count, void *stream)
{
    if (!ws) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to read_probe");
    if (count < 0) return fail(LUTGEMM_ERR_BAD_SHAPE, "count=%d is negative", count);
    for (int i = 0; i < count; i++) {
        const lutgemm_weight *w = ws[i];
        if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null handle in read_probe");
        if (int st_dev = check_device(w)) return st_dev;
        const Shape &s = w->shape;
        lutgemm_kernels::MatvecArgs a{};
        a.signs = w->d_signs;
        a.scales = w->d_scales;
        a.k = s.k;
        a.n = s.n;
        a.ts = s.ts;
        a.nb = s.nb;
        a.ntiles = w->plan.ntiles;
        a.k_splits = w->plan.k_splits;
        a.blocks_per_split = w->plan.blocks_per_split;
        hipError_t e = lutgemm_kernels::launch_read_probe(s.q, s.has_offset, s.gsub, a, w->plan.ntiles * w->plan.k_splits,
                                                          w->plan.waves, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return hip_fail(e, "launch read_probe_kernel");
    }
    return LUTGEMM_OK;
}

int lutgemm_dense_gemv_f16(const void *d_wt, const void *d_x, void *d_y, int k, int n, void *stream)
{
    if (!d_wt || !d_x || !d_y) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to dense_gemv_f16");
    if (k < 8 || k % 8 != 0 || n < 1)
        return fail(LUTGEMM_ERR_BAD_SHAPE, "dense_gemv_f16 needs k a positive multiple of 8 and n >= 1 (k=%d n=%d)", k, n);
    if ((((uintptr_t)d_wt | (uintptr_t)d_x) & 15u) != 0)
        return fail(LUTGEMM_ERR_BAD_SHAPE, "dense_gemv_f16 needs 16-byte aligned weight and activations");
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    int cus = 0;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return hip_fail(e, "hipDeviceGetAttribute");
    e = lutgemm_kernels::launch_dense_gemv(d_wt, d_x, d_y, k, n, cus > 0 ? cus : 256, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "launch dense_gemv_kernel");
    return LUTGEMM_OK;
}

int lutgemm_weight_unpack(const lutgemm_weight *w, uint32_t *bW, uint16_t *alpha, uint16_t *q_bias)
{
    if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_unpack");
    const Shape &s = w->shape;
    std::vector<uint8_t> signs;
    std::vector<uint16_t> scales;
    try {
        signs.resize(sign_bytes(s));
        scales.resize(scale_bytes(s) / 2);
    } catch (const std::bad_alloc &) {
        return fail(LUTGEMM_ERR_OUT_OF_MEMORY, "host staging allocation failed");
    }
    hipError_t e = hipMemcpy(signs.data(), w->d_signs, signs.size(), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "hipMemcpy(signs)");
    e = hipMemcpy(scales.data(), w->d_scales, scales.size() * 2, hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "hipMemcpy(scales)");
    lutgemm_packer::unpack(s, signs.data(), scales.data(), bW, alpha, s.has_offset ? q_bias : nullptr);
    return LUTGEMM_OK;
}

int lutgemm_weight_plan(const lutgemm_weight *w, int *workgroups, int *waves_per_group, int *k_splits,
                        int *k_blocks_per_group)
{
    if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_plan");
    if (workgroups) *workgroups = w->plan.ntiles * w->plan.k_splits;
    if (waves_per_group) *waves_per_group = w->plan.waves;
    if (k_splits) *k_splits = w->plan.k_splits;
    if (k_blocks_per_group) *k_blocks_per_group = w->plan.blocks_per_split;
    return LUTGEMM_OK;
}

int lutgemm_weight_plan_for(const lutgemm_weight *w, int m, int *workgroups, int *waves_per_group, int *k_splits,
                            int *k_blocks_per_group)
{
    if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_plan_for");
    if (m < 1 || m > LUTGEMM_MAX_BATCH)
        return fail(LUTGEMM_ERR_BAD_SHAPE, "m=%d outside 1..%d", m, LUTGEMM_MAX_BATCH);
    Plan p = m == 1 ? w->plan : w->plan2;
    if (m >= 3) {
        const int pass_rows = m < kRowsPerPass ? m : kRowsPerPass;
        p = w->batch_measured[pass_rows > 8] ? w->plan_batch[pass_rows > 8]
                                              : choose_batch_plan(w->shape, w->compute_units, pass_rows > 8 ? kRowsPerPass : 8);
    }
    if (workgroups) *workgroups = p.ntiles * p.k_splits;
    if (waves_per_group) *waves_per_group = p.waves;
    if (k_splits) *k_splits = p.k_splits;
    if (k_blocks_per_group) *k_blocks_per_group = p.blocks_per_split;
    return LUTGEMM_OK;
}

int lutgemm_weight_set_batch_plan(lutgemm_weight *w, int waves_per_group, int k_splits)
{
    if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_set_batch_plan");
    const Shape &s = w->shape;
    if (waves_per_group == 0 && k_splits == 0) {   // back to the model's choice
        w->batch_measured[0] = w->batch_measured[1] = false;
        return LUTGEMM_OK;
    }
    const int wmax = lutgemm_kernels::batch_waves_max(s.gsub, s.q, s.qo);
    if (waves_per_group < lutgemm_kernels::kBatchWavesMin || waves_per_group > wmax)
        return fail(LUTGEMM_ERR_BAD_SHAPE, "waves_per_group=%d outside %d..%d", waves_per_group,
                    lutgemm_kernels::kBatchWavesMin, wmax);
    if (k_splits < 1 || k_splits > s.ts || k_splits > kMaxSplits)
        return fail(LUTGEMM_ERR_BAD_SHAPE, "k_splits=%d outside 1..%d", k_splits, s.ts < kMaxSplits ? s.ts : kMaxSplits);
    Plan p;
    if (batch_plan_cost(s, w->compute_units, waves_per_group, k_splits, 8, &p) < 0.0)
        return fail(LUTGEMM_ERR_BAD_SHAPE, "k_splits=%d leaves a k-split without k-blocks (%d k-blocks)", k_splits, s.ts);
    w->plan_batch[0] = w->plan_batch[1] = p;
    w->batch_measured[0] = w->batch_measured[1] = true;
    return LUTGEMM_OK;
}

int lutgemm_weight_set_plan(lutgemm_weight *w, int waves_per_group, int k_splits)
{
    if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_set_plan");
    const Shape &s = w->shape;
    Plan p = choose_plan(s, w->compute_units);
    if (waves_per_group != 0) {
        if (waves_per_group < 1 || waves_per_group > kMaxWaves)
            return fail(LUTGEMM_ERR_BAD_SHAPE, "waves_per_group=%d outside 1..%d", waves_per_group, kMaxWaves);
        p.waves = waves_per_group;
        p.ntiles = div_up(s.nb, p.waves);
    }
    if (k_splits != 0) {
        if (k_splits < 1 || k_splits > s.ts || k_splits > kMaxSplits)
            return fail(LUTGEMM_ERR_BAD_SHAPE, "k_splits=%d outside 1..%d", k_splits,
                        s.ts < kMaxSplits ? s.ts : kMaxSplits);
        p.blocks_per_split = div_up(s.ts, k_splits);
        p.k_splits = div_up(s.ts, p.blocks_per_split);
    }
    hipError_t e = hipDeviceSynchronize();  // no launch may still be using the old workspace
    if (e != hipSuccess) return hip_fail(e, "hipDeviceSynchronize");
    w->plan = w->plan2 = p;
    return alloc_workspace(w);
}

int lutgemm_weight_autotune(lutgemm_weight *w, void *stream)
{
    if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_autotune");
    if (int st_dev = check_device(w)) return st_dev;
    if (int st_cap = refuse_capture(stream, "lutgemm_weight_autotune")) return st_cap;
    const Shape &s = w->shape;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // candidates: the best plans of the model, measured on the device
    struct Cand { double cost; Plan p; };
    std::vector<Cand> cands;
    for (int waves = 1; waves <= kMaxWaves; waves++)
        for (int splits = 1; splits <= s.ts && splits <= kMaxSplits; splits++) {
            Plan p;
            const double cost = plan_cost(s, w->compute_units, waves, splits, &p);
            if (cost >= 0.0) cands.push_back(Cand{cost, p});
        }
    std::sort(cands.begin(), cands.end(), [](const Cand &a, const Cand &b) { return a.cost < b.cost; });
    if (cands.size() > 24) cands.resize(24);
    // Workgroups with a single k-block need one table set only, so two of them share a compute
    // unit; the model does not describe that case, the measurement decides.
    if (s.ts <= kMaxSplits)
        for (int waves = 4; waves <= 8; waves++) {
            Plan p;
            const double cost = plan_cost(s, w->compute_units, waves, s.ts, &p);
            const long wgs = (long)p.ntiles * p.k_splits;
            if (cost >= 0.0 && wgs > w->compute_units && wgs <= 2L * w->compute_units) cands.push_back(Cand{cost, p});
        }

    // Measure as the weight will be used: streamed from HBM, not from the memory-side cache.
    // Temporary device copies are rotated so that more than four times the cache size passes
    // between two uses of the same copy (fewer if device memory is short: then the figures are
    // optimistic for all candidates alike).
    const size_t bytes = sign_bytes(s) + scale_bytes(s);
    const size_t rotation = (size_t)4 * 256 * 1024 * 1024;
    size_t want = (rotation + bytes - 1) / bytes + 1;
    if (want > 64) want = 64;
    std::vector<lutgemm_weight *> copies;
    copies.push_back(w);
    while (copies.size() < want) {
        lutgemm_weight *c = nullptr;
        if (create_from_tiles(s, w->d_signs, w->d_scales, hipMemcpyDeviceToDevice, &c) != LUTGEMM_OK) break;
        copies.push_back(c);
    }

    void *x = nullptr, *y = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int status = LUTGEMM_OK;
    const size_t max_rows = (size_t)kRowsPerPass;
    hipError_t e = hipMalloc(&x, max_rows * s.k * 2);
    if (e == hipSuccess) e = hipMalloc(&y, max_rows * s.n * 2);
    if (e == hipSuccess) e = hipMemsetAsync(x, 0, max_rows * s.k * 2, st);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e != hipSuccess) status = hip_fail(e, "autotune setup");
    const Plan before = w->plan, before2 = w->plan2;
    const Plan before_batch[2] = {w->plan_batch[0], w->plan_batch[1]};
    const bool before_measured[2] = {w->batch_measured[0], w->batch_measured[1]};
    size_t turn = 0;
    // time `reps` launches over `rows` activation rows with plan p, rotating over the copies
    auto measure = [&](const Plan &p, int rows, int reps, float *ms_out) -> int {
        for (lutgemm_weight *c : copies) {
            if (rows > kTableRows) {
                c->plan_batch[rows > 8] = p;
                c->batch_measured[rows > 8] = true;
            } else {
                (rows == 2 ? c->plan2 : c->plan) = p;
            }
        }
        int stt = LUTGEMM_OK;
        for (int r = 0; r < 2 && stt == LUTGEMM_OK; r++)
            stt = run_matvec(copies[turn++ % copies.size()], x, y, rows, stream, false, false);
        if (stt != LUTGEMM_OK) return stt;
        hipError_t he = hipEventRecord(e0, st);
        for (int r = 0; r < reps && stt == LUTGEMM_OK; r++)
            stt = run_matvec(copies[turn++ % copies.size()], x, y, rows, stream, false, false);
        if (stt != LUTGEMM_OK) return stt;
        if (he == hipSuccess) he = hipEventRecord(e1, st);
        if (he == hipSuccess) he = hipEventSynchronize(e1);
        if (he == hipSuccess) he = hipEventElapsedTime(ms_out, e0, e1);
        if (he != hipSuccess) return hip_fail(he, "autotune timing");
        *ms_out /= (float)reps;
        return LUTGEMM_OK;
    };
    // The device raises its clocks only under sustained load: launch for about 30 ms before
    // anything is timed, or the candidates measured first would look slow.
    {
        const auto t0 = std::chrono::steady_clock::now();
        float ms = 0.f;
        while (status == LUTGEMM_OK &&
               std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < 0.03)
            status = measure(before, 1, 50, &ms);
    }
    // Once for launches with one activation row, once for the two-row passes (a different
    // kernel with its own balance of table building and lookups).  Each time: two sweeps over all
    // candidates (the minimum of the two counts), then the four best again with more launches.
    Plan chosen[2] = {before, before2};
    for (int rows = 1; rows <= 2; rows++) {
        struct Timed { float ms; Plan p; };
        std::vector<Timed> timed;
        if (rows == 1) {
            for (size_t i = 0; status == LUTGEMM_OK && i < cands.size(); i++) timed.push_back(Timed{1e30f, cands[i].p});
        } else {
            // Rows of a two-row pass must come out bit for bit as their own one-row launch does:
            // same k-split (same partial sums); only the wavefronts per workgroup may differ.
            for (int waves = 1; waves <= kMaxWaves; waves++) {
                Plan p = chosen[0];
                p.waves = waves;
                p.ntiles = div_up(s.nb, waves);
                timed.push_back(Timed{1e30f, p});
            }
        }
        for (int sweep = 0; sweep < 2; sweep++)
            for (size_t i = 0; status == LUTGEMM_OK && i < timed.size(); i++) {
                float ms = 0.f;
                status = measure(timed[i].p, rows, 12, &ms);
                if (status == LUTGEMM_OK && ms < timed[i].ms) timed[i].ms = ms;
            }
        std::sort(timed.begin(), timed.end(), [](const Timed &a, const Timed &b) { return a.ms < b.ms; });
        float best_ms = 1e30f;
        for (int round = 0; round < 2; round++)
            for (size_t i = 0; status == LUTGEMM_OK && i < timed.size() && i < 4; i++) {
                float ms = 0.f;
                status = measure(timed[i].p, rows, 50, &ms);
                if (status == LUTGEMM_OK && ms < best_ms) {
                    best_ms = ms;
                    chosen[rows - 1] = timed[i].p;
                }
            }
    }
    // The batch kernel, for passes of up to 8 rows and of 9..16 rows: the model's ten best plans,
    // measured the same way.
    Plan chosen_batch[2] = {before_batch[0], before_batch[1]};
    bool have_batch[2] = {false, false};
    for (int bi = 0; bi < 2; bi++) {
        const int rows = bi ? kRowsPerPass : 8;
        struct Timed { float ms; double cost; Plan p; };
        std::vector<Timed> timed;
        for (int waves = lutgemm_kernels::kBatchWavesMin; waves <= lutgemm_kernels::batch_waves_max(s.gsub, s.q, s.qo); waves++)
            for (int ks = 1; ks <= s.ts && ks <= kMaxSplits; ks++) {
                Plan p;
                const double cost = batch_plan_cost(s, w->compute_units, waves, ks, rows, &p);
                if (cost >= 0.0) timed.push_back(Timed{1e30f, cost, p});
            }
        std::sort(timed.begin(), timed.end(), [](const Timed &a, const Timed &b) { return a.cost < b.cost; });
        if (timed.size() > 10) timed.resize(10);
        for (int sweep = 0; sweep < 2; sweep++)
            for (size_t i = 0; status == LUTGEMM_OK && i < timed.size(); i++) {
                float ms = 0.f;
                status = measure(timed[i].p, rows, 8, &ms);
                if (status == LUTGEMM_OK && ms < timed[i].ms) timed[i].ms = ms;
            }
        std::sort(timed.begin(), timed.end(), [](const Timed &a, const Timed &b) { return a.ms < b.ms; });
        float best_ms = 1e30f;
        for (int round = 0; round < 2; round++)
            for (size_t i = 0; status == LUTGEMM_OK && i < timed.size() && i < 3; i++) {
                float ms = 0.f;
                status = measure(timed[i].p, rows, 30, &ms);
                if (status == LUTGEMM_OK && ms < best_ms) {
                    best_ms = ms;
                    chosen_batch[bi] = timed[i].p;
                    have_batch[bi] = true;
                }
            }
    }
    w->plan = status == LUTGEMM_OK ? chosen[0] : before;
    w->plan2 = status == LUTGEMM_OK ? chosen[1] : before2;
    for (int bi = 0; bi < 2; bi++) {
        const bool ok = status == LUTGEMM_OK && have_batch[bi];
        w->plan_batch[bi] = ok ? chosen_batch[bi] : before_batch[bi];
        w->batch_measured[bi] = ok ? true : before_measured[bi];
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (x) (void)hipFree(x);
    if (y) (void)hipFree(y);
    for (size_t i = 1; i < copies.size(); i++) (void)lutgemm_weight_destroy(copies[i]);
    return status;
}

int lutgemm_weight_device_ptrs(const lutgemm_weight *w, void **signs, void **scales, void **offsets)
{
    if (!w) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to weight_device_ptrs");
    if (signs) *signs = w->d_signs;
    if (scales) *scales = w->d_scales;
    // offsets are interleaved with the scales in the scale tiles; non-null iff present
    if (offsets) *offsets = w->shape.has_offset ? (void *)w->d_scales : nullptr;
    return LUTGEMM_OK;
}

/* ---- host-only packer entry points (no device needed) ---- */

int lutgemm_packed_sizes(int k, int n, int q, int num_groups, int has_offset, size_t *sign_bytes_out,
                         size_t *scale_bytes_out)
{
    Shape s;
    if (!make_shape(k, n, q, num_groups, has_offset, &s))
        return fail(LUTGEMM_ERR_BAD_SHAPE, "bad shape k=%d n=%d q=%d num_groups=%d", k, n, q, num_groups);
    if (sign_bytes_out) *sign_bytes_out = sign_bytes(s);
    if (scale_bytes_out) *scale_bytes_out = scale_bytes(s);
    return LUTGEMM_OK;
}

int lutgemm_pack_host(const uint32_t *bW, const uint16_t *alpha, const uint16_t *q_bias, int k, int n, int q,
                      int num_groups, void *signs_out, void *scales_out)
{
    if (!bW || !alpha || !signs_out || !scales_out)
        return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to pack_host");
    Shape s;
    if (!make_shape(k, n, q, num_groups, q_bias != nullptr, &s))
        return fail(LUTGEMM_ERR_BAD_SHAPE, "bad shape k=%d n=%d q=%d num_groups=%d", k, n, q, num_groups);
    lutgemm_packer::pack(s, bW, alpha, q_bias, static_cast<uint8_t *>(signs_out),
                         static_cast<uint16_t *>(scales_out));
    return LUTGEMM_OK;
}

int lutgemm_unpack_host(const void *signs, const void *scales, int k, int n, int q, int num_groups,
                        int has_offset, uint32_t *bW, uint16_t *alpha, uint16_t *q_bias)
{
    if (!signs || !scales) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to unpack_host");
    Shape s;
    if (!make_shape(k, n, q, num_groups, has_offset, &s))
        return fail(LUTGEMM_ERR_BAD_SHAPE, "bad shape k=%d n=%d q=%d num_groups=%d", k, n, q, num_groups);
    lutgemm_packer::unpack(s, static_cast<const uint8_t *>(signs), static_cast<const uint16_t *>(scales), bW,
                           alpha, has_offset ? q_bias : nullptr);
    return LUTGEMM_OK;
}

int lutgemm_float_to_half(const float *src, uint16_t *dst, size_t count)
{
    if (!src || !dst) return fail(LUTGEMM_ERR_NULL_POINTER, "null argument to float_to_half");
    lutgemm_packer::floats_to_halves(src, dst, count);
    return LUTGEMM_OK;
}

const char *lutgemm_last_error(void) { return g_error; }

const char *lutgemm_status_string(int status)
{
    switch (status) {
        case LUTGEMM_OK: return "ok";
        case LUTGEMM_ERR_NULL_POINTER: return "null pointer";
        case LUTGEMM_ERR_BAD_SHAPE: return "bad shape";
        case LUTGEMM_ERR_NO_DEVICE: return "no device";
        case LUTGEMM_ERR_HIP: return "HIP runtime error";
        case LUTGEMM_ERR_OUT_OF_MEMORY: return "out of memory";
        case LUTGEMM_ERR_UNSUPPORTED: return "unsupported";
        case LUTGEMM_ERR_IO: return "file input/output failed";
        default: return "unknown status";
    }
}

const char *lutgemm_version(void) { return "lutgemm-hip 0.1 gfx950"; }

}  // extern "C"
