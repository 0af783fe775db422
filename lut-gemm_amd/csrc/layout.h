// Device layout of a packed BCQ weight ("wave64 tiles"), shared by the host packer and the
// kernels.  Everything here is plain integer arithmetic usable from host and device code.
//
// Vocabulary
//   chunk     8 consecutive k (one 256-entry partial-sum table, one sign byte per plane/output)
//   k-block   64 chunks = 512 consecutive k: one table set in LDS, one chunk per lane
//   row       16 consecutive lanes of a wavefront = 128 consecutive k (one DPP row)
//   batch     32 consecutive outputs, the unit of work of one wavefront
//
// Sign tiles (uint8), index order [batch][k-block][unit u = 2*plane + half][lane][byte p]:
//   byte p of lane L in unit (plane b, half h) of tile (batch nb, k-block ts) is the sign byte
//   of chunk ts*64 + L, plane b, output nb*32 + h*16 + p.  One unit is 64 lanes x 16 bytes =
//   1 KiB, read by a wavefront as a single fully coalesced 16-byte-per-lane load.
//
// Scale tiles (fp16), index order [batch][k-block][lane][slot t][plane-or-offset bo]:
//   The lanes of one row share 128 k, i.e. at most `gsub` = 1, 2 or 4 scale groups.  A row is
//   split into gsub sub-rows of subl = 16/gsub lanes; every sub-row stores the 32 outputs of
//   the batch once, nt = 32/subl = 2*gsub of them per lane: lane (row r, j) with
//   sub = j / subl, jj = j % subl holds, in slot t, the scale of output nb*32 + t*subl + jj
//   for the group that contains k = ts*512 + r*128 + sub*(128/gsub).  bo < q are the plane
//   scales, bo == q is the offset (only when the weight has one).  The kernel fetches a scale
//   from the lane that holds it with a DPP broadcast inside the row (gsub 1), half row
//   (gsub 2) or quad (gsub 4).
//
// k is padded up to a multiple of 512 and n up to a multiple of 32 with zero scales, so the
// padding never contributes.
#ifndef LUTGEMM_LAYOUT_H
#define LUTGEMM_LAYOUT_H

#include <stddef.h>
#include <stdint.h>

namespace lutgemm_layout {

constexpr int kLanes = 64;
constexpr int kChunk = 8;
constexpr int kBlockK = kLanes * kChunk;  // 512
constexpr int kBatch = 32;
constexpr int kUnitBytes = kLanes * 16;   // 1024

struct Shape {
    int k, n, q, num_groups, has_offset;
    int group_size;  // k / num_groups
    int gsub;        // scale groups per 128-k row: 1, 2 or 4
    int qo;          // q + has_offset
    int ts;          // k-blocks
    int nb;          // output batches
};

inline int div_up(int a, int b) { return (a + b - 1) / b; }

// Returns false if the shape violates the preconditions of the library.
inline bool make_shape(int k, int n, int q, int num_groups, int has_offset, Shape *s)
{
    if (k <= 0 || n <= 0 || q < 1 || q > 8 || num_groups < 1) return false;
    if (k % 32 != 0 || k % num_groups != 0) return false;
    int g = k / num_groups;
    if (g % 32 != 0) return false;
    s->k = k;
    s->n = n;
    s->q = q;
    s->num_groups = num_groups;
    s->has_offset = has_offset ? 1 : 0;
    s->group_size = g;
    s->gsub = (g % 128 == 0) ? 1 : (g % 64 == 0) ? 2 : 4;
    s->qo = q + s->has_offset;
    s->ts = div_up(k, kBlockK);
    s->nb = div_up(n, kBatch);
    return true;
}

inline size_t sign_tile_bytes(const Shape &s) { return (size_t)2 * s.q * kUnitBytes; }
inline size_t sign_bytes(const Shape &s) { return (size_t)s.nb * s.ts * sign_tile_bytes(s); }
// halves per lane in a scale tile
inline int scale_lane_halves(const Shape &s) { return 2 * s.gsub * s.qo; }
inline size_t scale_tile_bytes(const Shape &s) { return (size_t)kLanes * scale_lane_halves(s) * 2; }
inline size_t scale_bytes(const Shape &s) { return (size_t)s.nb * s.ts * scale_tile_bytes(s); }

}  // namespace lutgemm_layout
#endif
