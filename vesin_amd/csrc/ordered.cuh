// Search that produces a sorted list directly (options.sorted): rows grouped by first point in original index
// order and, within a point, ordered by second point and shift - the order the radix sort of sort.cuh produces,
// without sorting the rows as a whole.
//
// What makes that possible is giving up the half stencil: a tile's wave tests its points against the candidates of
// the whole (2s+1)^3 stencil, so every row (i, j, S) is found by the tile that holds i and by no other (a half
// list keeps i < j, or the self-image the reference's rule keeps, vesin/src/cpu_cell_list.cpp:101-133: the other
// orientation is found, and dropped, by the tile of j). Twice the distance tests of the other kernels, but then
//   COUNT  knows the number of rows of each of its points (one store per point, indexed by original index) and
//          leaves the hit column of every candidate in memory,
//   a scan over the points in original order gives every point its place in the output,
//   SORT   orders the candidates of every tile by (second point, shift without the wrap of the first point). All
//          points of a tile share that order: the wrap of the first point adds the same constant to the shift of
//          every one of its rows. One small sort per tile replaces a sort of the rows of every point,
//   WRITE  takes the candidates in that order, one per lane and unit, with their hit columns; point by point the
//          hits of the lanes, taken in lane order, are the rows in final order: they are compacted through LDS and
//          stored as runs of consecutive rows.
// Small systems (several waves per tile) skip SORT: their WRITE takes the candidates in table order and ranks the
// rows of every point by comparing all its keys (at most 256, read as LDS broadcasts).
// Rows per point beyond 256, candidates per tile beyond 1024, stencils beyond 64 cells or shifts and wraps beyond
// +-255 are reported in the status and the host falls back to the unsorted search followed by the radix sort.
//
// Arithmetic as everywhere (vesin/src/cpu_cell_list.cpp:135-138, vesin/src/types.hpp:232-243):
// S = cell shift - wrap_j + wrap_i, T = S . H left to right, v = (r_j - r_i) + T, d2 = vx*vx + vy*vy + vz*vz,
// keep iff d2 < cutoff^2.
#ifndef VESIN_HIP_ORDERED_CUH
#define VESIN_HIP_ORDERED_CUH

#include "fused.cuh"
#include "search.cuh"

namespace vesin_hip {

constexpr int ORDERED_WAVES = 4;
constexpr int ORDERED_BLOCK = ORDERED_WAVES * WAVE;
constexpr int ORDERED_R = 2;                            // units swept together
constexpr int ORDERED_UNITS = 16;                       // units of 64 candidates a tile may have
constexpr uint32_t ORDERED_CANDIDATES = ORDERED_UNITS * WAVE;
constexpr uint32_t ORDERED_MAX_ROWS = 256;              // rows of one point that are ranked in one go
constexpr int32_t ORDERED_SHIFT_LIMIT = 255;            // per operand: sums stay inside the key's 10-bit fields
constexpr uint32_t ORDERED_STAGED = ORDERED_MAX_ROWS + WAVE; // rows lined up before they are stored: what a run of
                                                             // consecutive rows left short of 64, and one point's

/// What the counting pass leaves to the writing pass per candidate of a work item: hit column against the item's
/// points, original index, biased shift less the wrap of the first point.
struct CandidateRecord {
    uint32_t column;
    uint32_t index;
    uint32_t biased;
};

/// What the counting pass found, for the host to decide between this path and the radix sort.
struct OrderedStatus {
    unsigned int max_rows;       // largest number of rows of one point
    unsigned int max_candidates; // largest number of candidates of one tile
    unsigned int unsuitable;     // tiles with a shift outside of the key's range
    unsigned int windowed;       // tiles whose candidates were ordered through the bit set
    unsigned int bucketed;       // tiles whose candidates were ordered through buckets
    unsigned int arrived;        // one-launch search, in the host's copy: workgroups of the launch
    unsigned int gave_up;        // one-launch search, in the host's copy: the workgroups did not wait for each other
    unsigned int padding;
};

/// What the host reads after the counting pass (pinned host memory, or a copy of it).
struct OrderedHostStatus {
    OrderedStatus found;
    unsigned long long total_rows;
    unsigned int first_bad_coordinate;
    unsigned int n_tiles; // of the cell list the passes worked on
};


struct OrderedArgs {
    SortedPoints sorted;
    const uint64_t* cell_scan;
    const Tile* tiles;
    uint32_t points_per_item;   // a tile's points are dealt to ceil(TILE_POINTS / points_per_item) waves
    uint32_t items_per_tile;
    uint32_t* rows_of_point;    // COUNT: [n_points], by original index
    CandidateRecord* records;   // COUNT -> WRITE: [work item][ORDERED_UNITS][64], candidates in table order: hit column,
                                // original index, biased shift (see CandidateRecord)
    uint32_t* candidates_of_item; // COUNT -> WRITE: [work item], how many of them there are
    const double* points;       // WRITE: the caller's points, by original index
    uint16_t* order;            // SORT -> WRITE: [tile][ORDERED_CANDIDATES], candidate number at each place of the order
    const uint64_t* first_row;  // WRITE: [n_points + 1], exclusive scan of rows_of_point
    OrderedStatus* status;
    uint32_t write_split;       // WRITE: waves that share the points of one work item of the counting pass (at least 1)
    uint32_t count_split;       // COUNT: waves that share the candidates of one work item (at least 1; more than 1:
                                // `rows_of_point` is zero on entry and the waves add to it)
    uint32_t report_order;      // SORT: count the tiles ordered either way (an atomic per tile on one word: for tests)
    uint32_t guarded;           // WRITE launched before the host has seen what COUNT found: write nothing unless the
                                // system suits this search and the rows fit the `capacity` of the arrays
    uint64_t capacity;
    SearchOutputs out;
    // WRITE launched before the host has seen what COUNT found: its first wave hands that to the host on the way
    // (everything is known when WRITE starts), which saves the launch that would do it afterwards.
    OrderedHostStatus* publish_to;
    const DeviceStatus* build_status;
    // COUNT: the single-precision pre-test (choose_prefilter, geometry.hpp); used when `sorted.l` is there
    Prefilter pre;
    // many systems in one launch (batched entry point; the kernels' BATCH variants): the grid of every system, its
    // first cell in the concatenated grids and its first point; rows_of_point and first_row go by first point of the
    // system + index in the system
    const GridParams* grids;
    const uint32_t* cell_base;
    const uint32_t* first_point;
    uint32_t total_cells;
    uint32_t total_points;
};

/// Systems of one cell and few points in a batch are searched over their images instead (images.cuh): the kernels
/// here leave their tiles alone.
constexpr uint32_t IMAGE_MAX_POINTS = 256;
constexpr uint32_t IMAGE_MAX_ENTRIES = 128; // a pair of points keeps a bit per image in two words

__host__ __device__ inline bool images_cover(const GridParams& g) {
    const uint64_t n_stencil = static_cast<uint64_t>(2 * g.s[0] + 1) * static_cast<uint64_t>(2 * g.s[1] + 1) *
                               static_cast<uint64_t>(2 * g.s[2] + 1);
    return g.n_cells == 1 && g.n_points <= IMAGE_MAX_POINTS && n_stencil <= IMAGE_MAX_ENTRIES;
}

/// LDS of one wave. What is known per candidate (hit column, position, original index, shift) stays in the
/// registers of the lane that loaded it: a lane only ever needs its own candidates until it hands a hit over as a key.
struct OrderedWaveShared {
    uint32_t tile_index[TILE_POINTS];
    double tile_x[TILE_POINTS], tile_y[TILE_POINTS], tile_z[TILE_POINTS];
    int32_t tile_wx[TILE_POINTS], tile_wy[TILE_POINTS], tile_wz[TILE_POINTS];
    uint64_t tile_row[TILE_POINTS];   // WRITE: first output row of each point
    uint32_t by_index[TILE_POINTS];   // WRITE: the tile's points in the order of their original indices
    // WRITE: the rows of one point: (second point << 32) | biased shift, and the position of the second point in
    // the cell-sorted arrays; read four at a time when they are ranked, hence the padding. With the candidates in
    // order: rows of points of consecutive original indices, which are consecutive rows of the list, and for each the
    // number of its first point in the tile
    __attribute__((aligned(16))) uint64_t keys[ORDERED_STAGED + 4];
    uint32_t key_at[ORDERED_STAGED];
};

/// LDS of one wave of the counting pass: the tables and the item's points. (A third of what the writing pass takes:
/// the ordering of the candidates runs beside the counting pass and needs 13 KB per wave itself; with the larger
/// struct the two kept each other's workgroups waiting for room.)
struct OrderedCountWaveShared: SearchTables {
    uint32_t tile_index[TILE_POINTS];
    double tile_x[TILE_POINTS], tile_y[TILE_POINTS], tile_z[TILE_POINTS];
    // for the single-precision pre-test (choose_prefilter, geometry.hpp): the places of the item's points inside
    // their cell, and the offsets of the stencil entries
    float tile_lx[TILE_POINTS], tile_ly[TILE_POINTS], tile_lz[TILE_POINTS];
    SearchOffsets offsets;
};

template <bool WRITE>
struct OrderedShared {
    std::conditional_t<WRITE, OrderedWaveShared, OrderedCountWaveShared> wave[ORDERED_WAVES];
};

/// The writing pass also keeps the records of one work item, for the launches in which the four waves of a workgroup
/// share a work item: they fetch the records together, once, instead of each for itself.
template <>
struct OrderedShared<true> {
    OrderedWaveShared wave[ORDERED_WAVES];
    CandidateRecord records[ORDERED_CANDIDATES];
};

__device__ __forceinline__ uint32_t biased_shift(int32_t sx, int32_t sy, int32_t sz) {
    return (static_cast<uint32_t>(sx + 512) << 20) | (static_cast<uint32_t>(sy + 512) << 10) |
           static_cast<uint32_t>(sz + 512);
}

__device__ __forceinline__ bool beyond(int32_t a, int32_t b, int32_t c, int32_t limit) {
    return a > limit || a < -limit || b > limit || b < -limit || c > limit || c < -limit;
}

/// sweep_columns for the counting pass of the in-order search, for a tile without wrapped points: what the
/// distance test does not decide is decided per test as well, and the rows of every point are counted on the way.
///   - candidate lanes whose `c.position` is the position of the point under test sit out: a point is no
///     neighbour of itself, and a half list keeps a point with its own image under the rule of the reference only;
///   - a half list keeps the orientation whose first index is the smaller one (!FULL);
///   - lane p of `rows` adds up the hits of the item's point p (a scalar population count per test).
template <int R, bool SHIFTED, bool FULL, typename Shared>
__device__ __forceinline__ void sweep_and_count(
    const Shared& sh, uint32_t first, uint32_t count, const SweepCandidates<R>& c, double cutoff2,
    const uint32_t (&original)[R], int lane, uint32_t (&column)[R], uint32_t& rows
) {
    // The item's points come from the wave's LDS (every lane reads the same words: broadcasts), four at a time:
    // the compiler keeps the reads of the next points in flight while the tests of these run, which the scalar
    // loads of the other sweeps, each waited for where it is issued, do not allow.
    for (uint32_t i0 = 0; i0 < count; i0 += POINTS_PER_LOAD) {
        double px[POINTS_PER_LOAD], py[POINTS_PER_LOAD], pz[POINTS_PER_LOAD];
        uint32_t pi[POINTS_PER_LOAD];
#pragma unroll
        for (int u = 0; u < POINTS_PER_LOAD; u++) {
            // (the arrays hold TILE_POINTS entries; what lies beyond `count` is read and not used)
            const uint32_t p = min(i0 + u, static_cast<uint32_t>(TILE_POINTS - 1));
            px[u] = sh.tile_x[p];
            py[u] = sh.tile_y[p];
            pz[u] = sh.tile_z[p];
            pi[u] = FULL ? 0u : sh.tile_index[p];
        }
#pragma unroll
        for (int u = 0; u < POINTS_PER_LOAD; u++) {
            if (u > 0 && i0 + u >= count) {
                break;
            }
            const double xi = px[u];
            const double yi = py[u];
            const double zi = pz[u];
            const uint32_t index_i = pi[u];
            const uint32_t at = first + i0 + u;
            uint32_t found = 0;
#pragma unroll
            for (int r = 0; r < R; r++) {
                double vx = c.x[r] - xi;
                double vy = c.y[r] - yi;
                double vz = c.z[r] - zi;
                if (SHIFTED) {
                    vx += c.tx[r];
                    vy += c.ty[r];
                    vz += c.tz[r];
                }
                const double d2 = vx * vx + vy * vy + vz * vz;
                uint64_t mask = __ballot(d2 < cutoff2) & __ballot(c.position[r] != at);
                if (!FULL) {
                    mask &= __ballot(index_i <= original[r]);
                }
                found += __popcll(mask);
                column[r] = shift_in(column[r], mask);
            }
            if (static_cast<uint32_t>(lane) == i0 + u) {
                rows += found;
            }
        }
    }
}

/// What a lane holds of a candidate for the single-precision pre-test (choose_prefilter, geometry.hpp): its place
/// as seen from the origin of the tile's cell. Lanes past the last candidate hold a place far away.
template <int R>
struct SweepPlaces {
    float x[R], y[R], z[R];
    uint32_t position[R]; // the candidate's position in the cell-sorted arrays when it must not pair with itself
};

constexpr float NOWHERE = 1.0e30f;

/// sweep_and_count in single precision: a pair whose squared distance falls below `lo32` is within the cutoff, one
/// above `hi32` is not, any pair in between sets its lane in `uncertain` and the caller repeats the candidates in
/// double precision. For any tile: the places account for points that were moved into the box.
template <int R, bool FULL, typename Shared>
__device__ __forceinline__ void sweep_and_count32(
    const Shared& sh, uint32_t first, uint32_t count, const SweepPlaces<R>& c, float lo32, float hi32,
    const uint32_t (&original)[R], int lane, uint32_t (&column)[R], uint32_t& rows, uint64_t& uncertain
) {
    for (uint32_t i0 = 0; i0 < count; i0 += POINTS_PER_LOAD) {
        float px[POINTS_PER_LOAD], py[POINTS_PER_LOAD], pz[POINTS_PER_LOAD];
        uint32_t pi[POINTS_PER_LOAD];
#pragma unroll
        for (int u = 0; u < POINTS_PER_LOAD; u++) {
            const uint32_t p = min(i0 + u, static_cast<uint32_t>(TILE_POINTS - 1));
            px[u] = sh.tile_lx[p];
            py[u] = sh.tile_ly[p];
            pz[u] = sh.tile_lz[p];
            pi[u] = FULL ? 0u : sh.tile_index[p];
        }
#pragma unroll
        for (int u = 0; u < POINTS_PER_LOAD; u++) {
            if (u > 0 && i0 + u >= count) {
                break;
            }
            const uint32_t at = first + i0 + u;
            uint32_t found = 0;
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float vx = c.x[r] - px[u];
                const float vy = c.y[r] - py[u];
                const float vz = c.z[r] - pz[u];
                const float d2 = __builtin_fmaf(vz, vz, __builtin_fmaf(vy, vy, vx * vx));
                const uint64_t within = __ballot(d2 < lo32);
                uncertain |= __ballot(d2 < hi32) & ~within;
                uint64_t mask = within & __ballot(c.position[r] != at);
                if (!FULL) {
                    mask &= __ballot(pi[u] <= original[r]);
                }
                found += __popcll(mask);
                column[r] = shift_in(column[r], mask);
            }
            if (static_cast<uint32_t>(lane) == i0 + u) {
                rows += found;
            }
        }
    }
}

/// Two units of candidates (numbers unit0 * 64 ... + 127 of the tables) against the item's points: hit columns
/// (the item's first point in the highest bit used); lane p of `rows` adds up the hits of the item's point p.
/// The same in single precision, for the counting pass of a work item whose points all have a place on record.
/// Returns false when some pair is too close to the cutoff to call, or some candidate has no place: nothing was
/// counted then, and the caller goes through ordered_sweep_pair.
template <bool FULL, typename Shared>
__device__ __forceinline__ bool ordered_sweep_pair32(
    const Shared& sh, const SortedPoints& sorted, float lo32, float hi32, uint32_t unit0, uint32_t n_stencil,
    uint32_t n_candidates, uint32_t first_i, uint32_t n_i, int lane, uint32_t (&column)[ORDERED_R], uint32_t& rows,
    bool& out_of_range, uint32_t (&at)[ORDERED_R], uint32_t (&original)[ORDERED_R], uint32_t (&biased)[ORDERED_R]
) {
    constexpr int R = ORDERED_R;
    SweepPlaces<R> c;
    uint64_t uncertain = 0;
    bool beyond_fields = false;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t k = (unit0 + r) * WAVE + lane;
        c.x[r] = c.y[r] = c.z[r] = NOWHERE;
        c.position[r] = 0xFFFFFFFFu;
        column[r] = 0;
        at[r] = 0xFFFFFFFFu;
        original[r] = 0;
        biased[r] = 0;
        bool unknown = false;
        if (k < n_candidates) {
            int32_t packed_q;
            uint32_t entry;
            locate_candidate(sh, n_stencil, k, at[r], packed_q, entry);
            int32_t qx, qy, qz;
            unpack_shift(packed_q, qx, qy, qz);
            const float4 place = sorted.l[at[r]];
            c.x[r] = place.x + sh.offsets.ent_dx[entry];
            c.y[r] = place.y + sh.offsets.ent_dy[entry];
            c.z[r] = place.z + sh.offsets.ent_dz[entry];
            unknown = !(place.x == place.x);
            original[r] = sorted.p[at[r]].index;
            const int32_t bx = qx - sorted.wx[at[r]];
            const int32_t by = qy - sorted.wy[at[r]];
            const int32_t bz = qz - sorted.wz[at[r]];
            biased[r] = biased_shift(bx, by, bz);
            beyond_fields = beyond_fields || beyond(bx, by, bz, ORDERED_SHIFT_LIMIT);
            // a point is no neighbour of itself (of its images it is: the unshifted entry of the tile's own cell is
            // meant); a half list keeps a point with its own image under the rule of the reference (the total
            // shift of such a pair is the cell shift, whatever box vectors the point itself was moved by)
            const bool never_with_itself = (qx | qy | qz) == 0 || (!FULL && !half_keeps_self_image(qx, qy, qz));
            c.position[r] = never_with_itself ? at[r] : 0xFFFFFFFFu;
        }
        uncertain |= __ballot(unknown);
    }
    if (uncertain != 0) {
        return false;
    }
    uint32_t counted = 0;
    sweep_and_count32<R, FULL>(sh, first_i, n_i, c, lo32, hi32, original, lane, column, counted, uncertain);
    if (uncertain != 0) {
        return false;
    }
    rows += counted;
    out_of_range = out_of_range || beyond_fields;
    return true;
}

template <bool FULL, bool WRAPPED, typename Shared>
__device__ __forceinline__ void ordered_sweep_pair(
    const Shared& sh, const SortedPoints& sorted, const GridParams& g, uint32_t unit0, uint32_t n_stencil,
    uint32_t n_candidates, uint32_t first_i, uint32_t n_i, int lane, uint32_t (&column)[ORDERED_R], uint32_t& rows,
    bool& out_of_range, uint32_t (&at)[ORDERED_R], uint32_t (&original)[ORDERED_R], uint32_t (&biased)[ORDERED_R]
) {
    constexpr int R = ORDERED_R;
    SweepCandidates<R> c;
    int32_t packed_q[R];
    bool any_shift = false;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint32_t k = (unit0 + r) * WAVE + lane;
        c.x[r] = c.y[r] = c.z[r] = __builtin_nan("");
        c.tx[r] = c.ty[r] = c.tz[r] = 0.0;
        c.shift[r] = 0;
        // sweep_columns_wrapped: no candidate is left to another tile, the whole stencil is this tile's;
        // sweep_and_count: the position of the candidate when it must not pair with itself
        c.position[r] = 0xFFFFFFFFu;
        column[r] = 0;
        at[r] = 0xFFFFFFFFu;
        original[r] = 0;
        biased[r] = 0;
        packed_q[r] = 0;
        int32_t bx = 0, by = 0, bz = 0;
        if (k < n_candidates) {
            locate_candidate(sh, n_stencil, k, at[r], packed_q[r]);
            int32_t qx, qy, qz;
            unpack_shift(packed_q[r], qx, qy, qz);
            c.x[r] = sorted.p[at[r]].x;
            c.y[r] = sorted.p[at[r]].y;
            c.z[r] = sorted.p[at[r]].z;
            original[r] = sorted.p[at[r]].index;
            bx = qx - sorted.wx[at[r]];
            by = qy - sorted.wy[at[r]];
            bz = qz - sorted.wz[at[r]];
            c.shift[r] = pack_shift(bx, by, bz);
            // what the writing pass keeps of the candidate (a shift outside of the fields makes the system unsuitable:
            // nothing is written then)
            biased[r] = biased_shift(bx, by, bz);
            out_of_range = out_of_range || beyond(bx, by, bz, ORDERED_SHIFT_LIMIT);
            if (!WRAPPED) {
                // a point is no neighbour of itself (of its images it is: the unshifted entry of the tile's own
                // cell is meant); a half list keeps a point with its own image under the rule of the reference
                // (the total shift of such a pair is the cell shift)
                const bool never_with_itself = (qx | qy | qz) == 0 || (!FULL && !half_keeps_self_image(qx, qy, qz));
                c.position[r] = never_with_itself ? at[r] : 0xFFFFFFFFu;
            }
        }
        any_shift = any_shift || (__ballot((bx | by | bz) != 0) != 0);
        if (any_shift) {
            // also read by the sweep of a tile with wrapped points, for its points that were not moved
            shift_vector(g, bx, by, bz, c.tx[r], c.ty[r], c.tz[r]);
        }
    }

    if (!WRAPPED) {
        if (any_shift) {
            sweep_and_count<R, true, FULL>(sh, first_i, n_i, c, g.cutoff2, original, lane, column, rows);
        } else {
            sweep_and_count<R, false, FULL>(sh, first_i, n_i, c, g.cutoff2, original, lane, column, rows);
        }
        return;
    }

    (void)sweep_columns_wrapped<R>(sorted, first_i, n_i, c, g, column);
    // what the distance test alone does not decide
#pragma unroll
    for (int r = 0; r < R; r++) {
        // a point is no neighbour of itself (of its images it is): the unshifted entry of the tile's own cell
        const uint32_t own = at[r] - first_i; // < n_i when the candidate is one of this item's points
        const bool is_own = own < n_i;
        const uint32_t own_bit = 1u << (n_i - 1 - (is_own ? own : 0));
        int32_t qx, qy, qz;
        unpack_shift(packed_q[r], qx, qy, qz);
        if (is_own && (qx | qy | qz) == 0) {
            column[r] &= ~own_bit;
        }
        if (!FULL) {
            // one orientation of every pair: the smaller index first; a point with its own image under the rule
            // of the reference (the total shift of such a pair is the cell shift)
            uint32_t smaller = 0;
            for (uint32_t p = 0; p < n_i; p++) {
                smaller = (smaller << 1) | (sh.tile_index[p] <= original[r] ? 1u : 0u);
            }
            column[r] &= smaller;
            if (is_own && !half_keeps_self_image(qx, qy, qz)) {
                column[r] &= ~own_bit;
            }
        }
    }
    for (uint32_t p = 0; p < n_i; p++) {
        const uint32_t bit = n_i - 1 - p;
        uint32_t found = 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            found += __popcll(__ballot(((column[r] >> bit) & 1u) != 0));
        }
        if (static_cast<uint32_t>(lane) == p) {
            rows += found;
        }
    }
}

/// Where write_rows_of_point reads the coordinates of a second point: the caller's array of points by original
/// index (x, y, z next to each other: one or two cache lines per point where the cell-sorted arrays take three), or
/// three arrays by a position of the caller's choice.
struct PointsByIndex {
    const double* points;
    __device__ __forceinline__ void load(uint32_t where, double& x, double& y, double& z) const {
        x = points[3 * static_cast<size_t>(where) + 0];
        y = points[3 * static_cast<size_t>(where) + 1];
        z = points[3 * static_cast<size_t>(where) + 2];
    }
};

struct PointsByPlace {
    const double* x;
    const double* y;
    const double* z;
    __device__ __forceinline__ void load(uint32_t where, double& px, double& py, double& pz) const {
        px = x[where];
        py = y[where];
        pz = z[where];
    }
};

/// The rows of one first point, from what the lanes hold per place of the order of the candidates (registers,
/// indexed by unit): hit columns (the point's bit is `bit`), where `coordinates` finds the candidate (`cand_where`;
/// the same array as `cand_index` when that is by original index), original indices and biased shifts without
/// the wrap of the first point (`wrap_i`: the three wraps in the fields of the key, added in one integer addition).
/// The hits are collected in lane order into `sh.keys` / `sh.key_at`, ranked where that is not their final order
/// (!PRESORTED), and stored from row `first_row` on.
template <bool PRESORTED, typename Shared, typename Coordinates>
__device__ __forceinline__ void write_rows_of_point(
    Shared& sh, const Coordinates& coordinates, const GridParams& g, const SearchOutputs& out,
    const uint32_t (&columns)[ORDERED_UNITS], const uint32_t (&cand_at)[ORDERED_UNITS],
    const uint32_t (&cand_index)[ORDERED_UNITS], const uint32_t (&cand_biased)[ORDERED_UNITS], uint32_t n_units,
    uint32_t bit, uint32_t wrap_i, double xi, double yi, double zi, uint32_t oi, uint64_t first_row, int lane
) {
    uint32_t n_rows = 0;
#pragma unroll
    for (int u = 0; u < ORDERED_UNITS; u++) {
        if (static_cast<uint32_t>(u) < n_units) {
            const bool hit = ((columns[u] >> bit) & 1u) != 0;
            const uint64_t mask = __ballot(hit);
            if (hit) {
                const uint32_t slot = n_rows + rank_in_mask(mask);
                sh.keys[slot] = (static_cast<uint64_t>(cand_index[u]) << 32) | (cand_biased[u] + wrap_i);
                sh.key_at[slot] = cand_at[u];
            }
            n_rows += __popcll(mask);
        }
    }
    if (n_rows == 0) {
        return;
    }
    if (!PRESORTED && lane < 4) {
        sh.keys[n_rows + lane] = ~0ull; // larger than any key: the ranking reads whole groups of four
    }
    wave_sync();

    for (uint32_t e0 = 0; e0 < n_rows; e0 += WAVE) {
        const uint32_t e = e0 + lane;
        const bool active = e < n_rows;
        const uint64_t key = active ? sh.keys[e] : ~0ull;
        // the position in the cell-sorted arrays is known before the rank is: the loads overlap the ranking
        const uint32_t at = active ? sh.key_at[e] : 0;
        double xj, yj, zj;
        coordinates.load(at, xj, yj, zj);
        uint32_t rank = e;
        if (!PRESORTED) {
            rank = 0;
            for (uint32_t other = 0; other < n_rows; other += 4) {
                // every lane reads the same 32 bytes: two LDS broadcasts for four comparisons
                const ulonglong2 first_two = *reinterpret_cast<const ulonglong2*>(&sh.keys[other]);
                const ulonglong2 next_two = *reinterpret_cast<const ulonglong2*>(&sh.keys[other + 2]);
                rank += (first_two.x < key ? 1u : 0u) + (first_two.y < key ? 1u : 0u);
                rank += (next_two.x < key ? 1u : 0u) + (next_two.y < key ? 1u : 0u);
            }
        }
        if (active) {
            const uint32_t oj = static_cast<uint32_t>(key >> 32);
            const uint32_t biased = static_cast<uint32_t>(key);
            const int32_t sx = static_cast<int32_t>((biased >> 20) & 0x3ffu) - 512;
            const int32_t sy = static_cast<int32_t>((biased >> 10) & 0x3ffu) - 512;
            const int32_t sz = static_cast<int32_t>(biased & 0x3ffu) - 512;
            double tx, ty, tz;
            shift_vector(g, sx, sy, sz, tx, ty, tz);
            const double vx = (xj - xi) + tx;
            const double vy = (yj - yi) + ty;
            const double vz = (zj - zi) + tz;
            // PRESORTED: consecutive lanes, consecutive rows
            const uint64_t row = first_row + rank;
            stream_store(out.pairs + 2 * row, PairRow{oi, oj});
            if (out.shifts != nullptr) {
                stream_store(out.shifts + 3 * row, ShiftRow{sx, sy, sz});
            }
            if (out.distances != nullptr) {
                stream_store(out.distances + row, sqrt(vx * vx + vy * vy + vz * vz));
            }
            if (out.vectors != nullptr) {
                stream_store(out.vectors + 3 * row, VectorHead{vx, vy});
                stream_store(out.vectors + 3 * row + 2, vz);
            }
        }
    }
    wave_sync(); // the keys are about to be overwritten by the next point's
}

/// The hits of one first point (number `point` of the tile), in lane order, behind the `staged` keys that wait in
/// `sh.keys`: returns how many there were. (Candidates in their final order: the hits are the point's rows in order.)
template <typename Shared>
__device__ __forceinline__ uint32_t stage_rows_of_point(
    Shared& sh, const uint32_t (&columns)[ORDERED_UNITS], const uint32_t (&cand_index)[ORDERED_UNITS],
    const uint32_t (&cand_biased)[ORDERED_UNITS], uint32_t n_units, uint32_t bit, uint32_t wrap_i, uint32_t point,
    uint32_t staged
) {
    uint32_t n_rows = 0;
#pragma unroll
    for (int u = 0; u < ORDERED_UNITS; u++) {
        if (static_cast<uint32_t>(u) < n_units) {
            const bool hit = ((columns[u] >> bit) & 1u) != 0;
            const uint64_t mask = __ballot(hit);
            if (hit) {
                const uint32_t slot = min(staged + n_rows + rank_in_mask(mask), ORDERED_STAGED - 1);
                sh.keys[slot] = (static_cast<uint64_t>(cand_index[u]) << 32) | (cand_biased[u] + wrap_i);
                sh.key_at[slot] = point;
            }
            n_rows += __popcll(mask);
        }
    }
    return n_rows;
}

/// Stores the first `count` staged keys as the rows `first_row` ... of the list: 64 consecutive rows per step, each
/// step ending on a multiple of 64 rows (whole cache lines in every output array; the first step stores fewer).
template <typename Shared>
__device__ __forceinline__ void store_staged_rows(
    const Shared& sh, const double* __restrict__ points, const GridParams& g, const SearchOutputs& out, uint32_t count,
    uint64_t first_row, int lane
) {
    const uint32_t skew = static_cast<uint32_t>(first_row % WAVE);
    for (uint32_t e0 = 0; e0 < count + skew; e0 += WAVE) {
        const uint32_t e = e0 + lane - skew;
        if (e >= count) {
            continue; // (before the first row as well: unsigned)
        }
        const uint64_t key = sh.keys[e];
        const uint32_t point = sh.key_at[e];
        const uint32_t oj = static_cast<uint32_t>(key >> 32);
        const double xj = points[3 * static_cast<size_t>(oj) + 0];
        const double yj = points[3 * static_cast<size_t>(oj) + 1];
        const double zj = points[3 * static_cast<size_t>(oj) + 2];
        const uint32_t biased = static_cast<uint32_t>(key);
        const int32_t sx = static_cast<int32_t>((biased >> 20) & 0x3ffu) - 512;
        const int32_t sy = static_cast<int32_t>((biased >> 10) & 0x3ffu) - 512;
        const int32_t sz = static_cast<int32_t>(biased & 0x3ffu) - 512;
        double tx, ty, tz;
        shift_vector(g, sx, sy, sz, tx, ty, tz);
        const double vx = (xj - sh.tile_x[point]) + tx;
        const double vy = (yj - sh.tile_y[point]) + ty;
        const double vz = (zj - sh.tile_z[point]) + tz;
        const uint64_t row = first_row + e;
        stream_store(out.pairs + 2 * row, PairRow{sh.tile_index[point], oj});
        if (out.shifts != nullptr) {
            stream_store(out.shifts + 3 * row, ShiftRow{sx, sy, sz});
        }
        if (out.distances != nullptr) {
            stream_store(out.distances + row, sqrt(vx * vx + vy * vy + vz * vz));
        }
        if (out.vectors != nullptr) {
            stream_store(out.vectors + 3 * row, VectorHead{vx, vy});
            stream_store(out.vectors + 3 * row + 2, vz);
        }
    }
}

/// PRESORTED (WRITE only): the candidates are taken in the order ordered_sort_kernel left for the tile, and the hits
/// of a point in lane order are its rows in final order. Otherwise (small systems, where one more launch costs more
/// than it saves) candidates come in table order and the rows of every point are ranked by comparing all its keys.
/// BATCH: the tiles of many systems (every tile knows its system, whose grid it takes); systems that the search over
/// images covers are skipped.
template <bool WRITE, bool FULL, bool PRESORTED = false, bool BATCH = false>
__global__ __launch_bounds__(ORDERED_BLOCK) __attribute__((amdgpu_waves_per_eu(4))) void ordered_search_kernel(OrderedArgs args, GridParams single_grid) {
    constexpr int R = ORDERED_R;
    __shared__ OrderedShared<WRITE> shared;
    const int lane = lane_id();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    auto& sh = shared.wave[wave];
    const uint32_t all_points = BATCH ? args.total_points : single_grid.n_points;
    const uint32_t all_cells = BATCH ? args.total_cells : single_grid.n_cells;
    if (WRITE && args.publish_to != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
        OrderedHostStatus report;
        report.found = *args.status;
        report.total_rows = args.first_row[all_points];
        report.first_bad_coordinate = args.build_status->first_bad_coordinate;
        report.n_tiles = static_cast<unsigned int>(args.cell_scan[all_cells] >> 32);
        *args.publish_to = report;
    }
    if (WRITE && args.guarded != 0) {
        const OrderedStatus found = *args.status;
        const bool suitable = found.max_rows <= ORDERED_MAX_ROWS && found.max_candidates <= ORDERED_CANDIDATES &&
                              found.unsuitable == 0 && args.first_row[all_points] <= args.capacity;
        if (!suitable) {
            return;
        }
    }
    const uint32_t n_tiles = static_cast<uint32_t>(args.cell_scan[all_cells] >> 32);
    // WRITE may deal the points of a work item of the counting pass to several waves (`write_split`): they read the
    // same records and each writes the rows of its share of the points
    // COUNT may deal the candidates of a work item to several waves (`count_split`), by pairs of units in turn
    const uint32_t split = WRITE ? args.write_split : args.count_split;
    const uint32_t part = (blockIdx.x * ORDERED_WAVES + wave) % split;
    const uint32_t work = (blockIdx.x * ORDERED_WAVES + wave) / split;
    const uint32_t slot = work / args.items_per_tile;
    const uint32_t item = work % args.items_per_tile;
    // workgroups are dealt to the 8 XCDs round-robin: each XCD walks one contiguous range of tiles, so that its L2
    // sees the same cells again and again (same mapping as the other search kernels)
    const uint32_t per_xcd = (n_tiles + N_XCD - 1) / N_XCD;
    const uint32_t xcd = (slot / ORDERED_WAVES) % N_XCD;
    const uint32_t within = (slot / (ORDERED_WAVES * N_XCD)) * ORDERED_WAVES + slot % ORDERED_WAVES;
    const uint32_t tile_id = xcd * per_xcd + within;
    if (within >= per_xcd || tile_id >= n_tiles) {
        return;
    }
    const SortedPoints& sorted = args.sorted;
    const Tile tile = args.tiles[tile_id];
    // this wave's share of the tile's points
    const uint32_t p_begin = item * args.points_per_item;
    if (p_begin >= tile.count) {
        return;
    }
    const uint32_t n_i = min(tile.count - p_begin, args.points_per_item);
    const uint32_t first_i = tile.first + p_begin;
    const bool tile_wrapped = (tile.wrapped & 1u) != 0;
    // the grid: the kernel's argument, or this tile's system's
    GridParams batch_grid;
    uint32_t first_cell = 0;
    uint32_t first_point = 0;
    if (BATCH) {
        const uint32_t system = tile_system(tile);
        batch_grid = args.grids[system];
        first_cell = args.cell_base[system];
        first_point = args.first_point[system];
        if (images_cover(batch_grid)) {
            return;
        }
    }
    const GridParams& g = BATCH ? batch_grid : single_grid;
    const uint64_t* __restrict__ cell_scan = args.cell_scan + first_cell;
    const uint32_t local_cell = tile.cell - first_cell;
    const int32_t cx = local_cell % g.n[0];
    const int32_t cy = (local_cell / g.n[0]) % g.n[1];
    const int32_t cz = local_cell / (g.n[0] * g.n[1]);

    bool out_of_range = false;
    // COUNT: the single-precision pre-test, when the grid allows it and every point of the item has a place on record
    bool pretest = !WRITE && args.pre.use32 != 0 && sorted.l != nullptr;
    bool place_unknown = false;
    if (static_cast<uint32_t>(lane) < n_i) {
        const uint32_t at = first_i + lane;
        const uint32_t original = sorted.p[at].index;
        sh.tile_index[lane] = original;
        const int32_t wx = sorted.wx[at];
        const int32_t wy = sorted.wy[at];
        const int32_t wz = sorted.wz[at];
        out_of_range = beyond(wx, wy, wz, ORDERED_SHIFT_LIMIT);
        sh.tile_x[lane] = sorted.p[at].x;
        sh.tile_y[lane] = sorted.p[at].y;
        sh.tile_z[lane] = sorted.p[at].z;
        if constexpr (!WRITE) {
            if (pretest) {
                const float4 place = sorted.l[at];
                sh.tile_lx[lane] = place.x;
                sh.tile_ly[lane] = place.y;
                sh.tile_lz[lane] = place.z;
                place_unknown = !(place.x == place.x);
            }
        }
        if constexpr (WRITE) {
            sh.tile_wx[lane] = wx;
            sh.tile_wy[lane] = wy;
            sh.tile_wz[lane] = wz;
            sh.tile_row[lane] = args.first_row[first_point + original];
        }
    }

    // the whole stencil, the tile's own cell included
    const int32_t span_y = 2 * g.s[1] + 1;
    const int32_t span_z = 2 * g.s[2] + 1;
    const uint32_t n_stencil = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z;
    if (n_stencil > MAX_ENTRIES) {
        // the host does not launch this kernel for such a stencil; in a batch some system may have one
        if (BATCH && !WRITE && lane == 0 && item == 0 && part == 0) {
            atomicAdd(&args.status->unsuitable, 1u);
        }
        return;
    }
    uint32_t n_candidates;
    if constexpr (WRITE) {
        // (the counting pass left the number: no tables here, everything about a candidate is in its record)
        n_candidates = uniform(args.candidates_of_item[work]);
    } else {
        pretest = pretest && __ballot(place_unknown) == 0;
        fill_stencil_tables(
            sh, lane, 0, n_stencil, cx, cy, cz, span_y, span_z, g, cell_scan, static_cast<const uint32_t*>(nullptr), 0u,
            pretest ? &sh.offsets : nullptr, &args.pre
        );
        n_candidates = __builtin_amdgcn_readfirstlane(sh.n_candidates);
        if (lane == 0 && part == 0) {
            args.candidates_of_item[work] = n_candidates;
        }
    }
    const uint32_t n_units = (n_candidates + WAVE - 1) / WAVE;

    if (!WRITE) {
        // thousands of waves report to the same words: an atomic only where it would change something
        if (lane == 0 && item == 0 && part == 0 &&
            n_candidates > __atomic_load_n(&args.status->max_candidates, __ATOMIC_RELAXED)) {
            atomicMax(&args.status->max_candidates, n_candidates);
        }
    }
    if (n_candidates > ORDERED_CANDIDATES) {
        return; // the host does not use this path for such a tile: nothing to count, nothing may be written
    }

    CandidateRecord* item_records = args.records + static_cast<size_t>(work) * (ORDERED_UNITS * WAVE);
    if constexpr (!WRITE) {
        // ---- COUNT: the number of rows of every point (lane p adds up the hits of point p) and, for the writing
        // pass, the hit column of every candidate: a plain loop over the pairs of units, small code
        uint32_t own_rows = 0;
        for (uint32_t unit0 = part * R; unit0 < n_units; unit0 += split * R) {
            uint32_t column[R], at[R], original[R], biased[R];
            if (pretest && ordered_sweep_pair32<FULL>(
                               sh, sorted, args.pre.lo32, args.pre.hi32, unit0, n_stencil, n_candidates, first_i, n_i, lane, column, own_rows,
                               out_of_range, at, original, biased
                           )) {
                // decided in single precision
            } else if (tile_wrapped) {
                ordered_sweep_pair<FULL, true>(
                    sh, sorted, g, unit0, n_stencil, n_candidates, first_i, n_i, lane, column, own_rows, out_of_range,
                    at, original, biased
                );
            } else {
                ordered_sweep_pair<FULL, false>(
                    sh, sorted, g, unit0, n_stencil, n_candidates, first_i, n_i, lane, column, own_rows, out_of_range,
                    at, original, biased
                );
            }
            // everything the writing pass needs of a candidate in one 12-byte record, so that it takes one load per
            // place of the tile's order instead of a table lookup and five scattered ones
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (unit0 + r < n_units) {
                    // (plain stores: the writing pass reads them soon, out of the caches where they still are)
                    item_records[(unit0 + r) * WAVE + lane] = CandidateRecord{column[r], original[r], biased[r]};
                }
            }
        }
        if (static_cast<uint32_t>(lane) < n_i) {
            if (split == 1) {
                args.rows_of_point[first_point + sh.tile_index[lane]] = own_rows;
            } else {
                // whichever wave of the item comes last sees the sum of the others: the largest number any of
                // them sees for a point is the point's number of rows
                own_rows += atomicAdd(&args.rows_of_point[first_point + sh.tile_index[lane]], own_rows);
            }
        }
        uint32_t most = own_rows;
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) {
            most = max(most, static_cast<uint32_t>(__shfl_xor(static_cast<int>(most), offset, WAVE)));
        }
        if (lane == 0 && most > __atomic_load_n(&args.status->max_rows, __ATOMIC_RELAXED)) {
            atomicMax(&args.status->max_rows, most);
        }
        if (__ballot(out_of_range) != 0 && lane == 0) {
            atomicAdd(&args.status->unsuitable, 1u);
        }
        return;
    }

    if constexpr (WRITE) {
        // ---- per place of the tile's order (registers of its lane, indexed by unit): the candidate there, the hit
        // column the counting pass found for it against this item's points, its original index and its shift
        // (biased, without the wrap of the first point: that one is added per point, field by field in one integer
        // addition)
        const uint16_t* tile_order = args.order + static_cast<size_t>(tile_id) * ORDERED_CANDIDATES;
        uint32_t columns[ORDERED_UNITS];
        uint32_t cand_index[ORDERED_UNITS];
        uint32_t cand_biased[ORDERED_UNITS];
        // The four waves of a workgroup that share a work item (every wave of the workgroup got this far then, or
        // none) bring its records to LDS together, already in the order of the tile: a place each per step, its
        // candidate number and then the record from memory, two round trips for the workgroup where every wave
        // made two per group of four units.
        const bool together = split == ORDERED_WAVES;
        if (together) {
            for (uint32_t place = threadIdx.x; place < n_candidates; place += ORDERED_BLOCK) {
                const uint32_t k = PRESORTED ? min(static_cast<uint32_t>(tile_order[place]), n_candidates - 1) : place;
                shared.records[place] = item_records[k];
            }
            __syncthreads();
        }
#pragma unroll
        for (int u = 0; u < ORDERED_UNITS; u++) {
            columns[u] = 0;
            cand_index[u] = 0;
            cand_biased[u] = 0;
            const uint32_t place = u * WAVE + lane;
            if (static_cast<uint32_t>(u) < n_units && place < n_candidates) {
                CandidateRecord record; // 12 bytes
                if (together) {
                    record = shared.records[place];
                } else {
                    const uint32_t k = PRESORTED ? min(static_cast<uint32_t>(tile_order[place]), n_candidates - 1) : place;
                    record = item_records[k];
                }
                columns[u] = record.column;
                cand_index[u] = record.index;
                cand_biased[u] = record.biased;
            }
            if (u % 4 == 3) {
                // four units' loads in flight at a time: with all sixteen, their addresses alone take 32 registers
                // (reading the places of all units first and then the records, eight at a time, took as long)
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // ---- WRITE: point by point, collect the hits in lane order, rank them where that is not their final order,
        // store the rows
        wave_sync();
        const uint32_t per_part = (n_i + split - 1) / split;
        const double* system_points = args.points + 3 * static_cast<size_t>(first_point);
        if constexpr (PRESORTED) {
            // The points in the order of their original indices: the rows of points with consecutive indices are
            // consecutive rows of the list (inputs in the order of a lattice have runs of them in every cell). Their
            // rows are lined up in LDS one point after the other and stored 64 at a time, from multiples of 64 rows.
            if (static_cast<uint32_t>(lane) < n_i) {
                const uint32_t own = sh.tile_index[lane];
                uint32_t smaller = 0;
                for (uint32_t other = 0; other < n_i; other++) {
                    smaller += sh.tile_index[other] < own ? 1u : 0u;
                }
                sh.by_index[smaller] = lane;
            }
            wave_sync();
            uint32_t staged = 0;
            uint64_t staged_row = 0; // row of the first staged key
            for (uint32_t turn = part * per_part; turn < min(n_i, (part + 1) * per_part); turn++) {
                const uint32_t p = uniform(sh.by_index[turn]);
                const uint64_t row_p = uniform(sh.tile_row[p]);
                if (staged != 0 && row_p != staged_row + staged) {
                    store_staged_rows(sh, system_points, g, args.out, staged, staged_row, lane);
                    staged = 0;
                    wave_sync();
                }
                if (staged == 0) {
                    staged_row = row_p;
                }
                const uint32_t wrap_i = (static_cast<uint32_t>(sh.tile_wx[p]) << 20) + (static_cast<uint32_t>(sh.tile_wy[p]) << 10) +
                                        static_cast<uint32_t>(sh.tile_wz[p]);
                staged += stage_rows_of_point(sh, columns, cand_index, cand_biased, n_units, n_i - 1 - p, wrap_i, p, staged);
                staged = min(staged, ORDERED_STAGED); // (a point has at most ORDERED_MAX_ROWS rows here)
                wave_sync();
                const uint64_t whole = ((staged_row + staged) & ~static_cast<uint64_t>(WAVE - 1));
                if (whole > staged_row) {
                    // everything up to the last multiple of 64 rows; what is left moves to the front
                    const uint32_t count = static_cast<uint32_t>(whole - staged_row);
                    store_staged_rows(sh, system_points, g, args.out, count, staged_row, lane);
                    const uint32_t left = staged - count; // < 64
                    const uint64_t key = sh.keys[min(count + lane, ORDERED_STAGED - 1)];
                    const uint32_t point = sh.key_at[min(count + lane, ORDERED_STAGED - 1)];
                    wave_sync();
                    if (static_cast<uint32_t>(lane) < left) {
                        sh.keys[lane] = key;
                        sh.key_at[lane] = point;
                    }
                    staged_row = whole;
                    staged = left;
                    wave_sync();
                }
            }
            if (staged != 0) {
                store_staged_rows(sh, system_points, g, args.out, staged, staged_row, lane);
            }
            return;
        }
        for (uint32_t p = part * per_part; p < min(n_i, (part + 1) * per_part); p++) {
            // every field of the sum stays inside its ten bits (operands within +-255), so the fields add independently
            const uint32_t wrap_i = (static_cast<uint32_t>(sh.tile_wx[p]) << 20) + (static_cast<uint32_t>(sh.tile_wy[p]) << 10) +
                                    static_cast<uint32_t>(sh.tile_wz[p]);
            // (the second points are looked up by their original index: no position to keep per candidate)
            write_rows_of_point<PRESORTED>(
                sh, PointsByIndex{system_points}, g, args.out, columns, cand_index, cand_index, cand_biased, n_units, n_i - 1 - p, wrap_i,
                sh.tile_x[p], sh.tile_y[p], sh.tile_z[p], sh.tile_index[p], sh.tile_row[p], lane
            );
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// SORT: the order of a tile's candidates

// one wave per workgroup: a wave's 13 KB of LDS are free again as soon as its tile is done (four waves held 52 KB
// until the slowest was, beside the counting pass's workgroups: measured a fifth slower)
constexpr int ORDER_WAVES = 1;
constexpr int ORDER_BLOCK = ORDER_WAVES * WAVE;
constexpr uint32_t ORDER_BUCKETS = 4 * WAVE;
constexpr uint32_t ORDER_BITS = 64 * 1024;        // original indices the bit set covers at a time
constexpr uint32_t ORDER_WORDS = ORDER_BITS / 32;
constexpr uint32_t ORDER_ROUNDS = 4;              // the window of indices ranked through the bit set: that many times ORDER_BITS

/// LDS of one wave, used in one of two ways.
union OrderScratch {
    struct {
        uint32_t index_of[ORDERED_CANDIDATES];      // original index by candidate number
        uint32_t grouped_index[ORDERED_CANDIDATES]; // original indices grouped by bucket
        uint16_t grouped[ORDERED_CANDIDATES];       // candidate numbers, same grouping
        uint32_t bucket_end[ORDER_BUCKETS];         // counts, then where the next key of the bucket goes, at last its end
    } buckets;
    struct {
        __attribute__((aligned(16))) uint32_t present[ORDER_WORDS]; // one bit per original index of the window
        uint16_t before[ORDER_WORDS / 4];                           // bits set before each group of four words
        uint16_t offset[ORDERED_CANDIDATES];                        // by candidate number: its bit ...
        uint8_t round_of[ORDERED_CANDIDATES];                       // ... in the round that covers its index
    } bits;
};

struct OrderWaveShared: SearchTables {
    OrderScratch scratch;
};

struct OrderShared {
    OrderWaveShared wave[ORDER_WAVES];
};

/// One wave per tile: writes, for every place of the order of the tile's candidates by (original index, shift less
/// the wrap of the first point), the number of the candidate in the stencil tables.
///
/// When the original indices the tile sees fit a window of ORDER_ROUNDS x ORDER_BITS and no point is seen twice (as
/// two images), the place of a candidate is the number of smaller indices present: one bit per index, counted with
/// prefix sums, ORDER_BITS indices at a time.
/// That is the case of inputs ordered like the lattice they were built from, where the candidates come as runs of
/// consecutive indices; the window may wrap around from the last index to the first, as the neighbourhood of a tile
/// at the edge of a periodic box does. Otherwise the range is cut into 256 buckets, monotonic in the index, and a
/// key is only compared with the keys of its own bucket: few when the indices are spread evenly, as they are in
/// inputs without any order. Loops over the units are kept rolled: this kernel is small work, it should be small
/// code.
template <bool BATCH = false>
__global__ __launch_bounds__(ORDER_BLOCK) void ordered_sort_kernel(OrderedArgs args, GridParams single_grid) {
    __shared__ OrderShared shared;
    const int lane = lane_id();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    OrderWaveShared& sh = shared.wave[wave];
    const uint32_t all_cells = BATCH ? args.total_cells : single_grid.n_cells;
    const uint32_t n_tiles = static_cast<uint32_t>(args.cell_scan[all_cells] >> 32);
    const uint32_t tile_id = blockIdx.x * ORDER_WAVES + wave;
    if (tile_id >= n_tiles) {
        return;
    }
    const SortedPoints& sorted = args.sorted;
    const Tile tile = args.tiles[tile_id];
    // the grid: the kernel's argument, or this tile's system's (indices count from the first point of the system)
    GridParams batch_grid;
    uint32_t first_cell = 0;
    if (BATCH) {
        const uint32_t system = tile_system(tile);
        batch_grid = args.grids[system];
        first_cell = args.cell_base[system];
        if (images_cover(batch_grid)) {
            return;
        }
    }
    const GridParams& g = BATCH ? batch_grid : single_grid;
    const uint64_t* __restrict__ cell_scan = args.cell_scan + first_cell;
    const uint32_t local_cell = tile.cell - first_cell;
    const int32_t cx = local_cell % g.n[0];
    const int32_t cy = (local_cell / g.n[0]) % g.n[1];
    const int32_t cz = local_cell / (g.n[0] * g.n[1]);
    const int32_t span_y = 2 * g.s[1] + 1;
    const int32_t span_z = 2 * g.s[2] + 1;
    const uint32_t n_stencil = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z;
    if (n_stencil > MAX_ENTRIES) {
        return;
    }
    fill_stencil_tables(sh, lane, 0, n_stencil, cx, cy, cz, span_y, span_z, g, cell_scan);
    const uint32_t n_candidates = __builtin_amdgcn_readfirstlane(sh.n_candidates);
    if (n_candidates > ORDERED_CANDIDATES || n_candidates == 0) {
        return; // the writing pass is not launched when a tile has too many
    }
    uint16_t* tile_order = args.order + static_cast<size_t>(tile_id) * ORDERED_CANDIDATES;

    // the range of original indices, and the same for each half of the index space
    const uint32_t half = g.n_points / 2;
    uint32_t lowest = 0xFFFFFFFFu;
    uint32_t highest = 0;
    uint32_t upper_lowest = 0xFFFFFFFFu;
    uint32_t lower_highest = 0;
#pragma unroll 4
    for (uint32_t k = lane; k < n_candidates; k += WAVE) {
        uint32_t at;
        int32_t packed_q;
        locate_candidate(sh, n_stencil, k, at, packed_q);
        const uint32_t index = sorted.p[at].index;
        lowest = min(lowest, index);
        highest = max(highest, index);
        if (index >= half) {
            upper_lowest = min(upper_lowest, index);
        } else {
            lower_highest = max(lower_highest, index);
        }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        lowest = min(lowest, static_cast<uint32_t>(__shfl_xor(static_cast<int>(lowest), offset, WAVE)));
        highest = max(highest, static_cast<uint32_t>(__shfl_xor(static_cast<int>(highest), offset, WAVE)));
        upper_lowest = min(upper_lowest, static_cast<uint32_t>(__shfl_xor(static_cast<int>(upper_lowest), offset, WAVE)));
        lower_highest = max(lower_highest, static_cast<uint32_t>(__shfl_xor(static_cast<int>(lower_highest), offset, WAVE)));
    }
    lowest = uniform(lowest);
    highest = uniform(highest);
    upper_lowest = uniform(upper_lowest);
    lower_highest = uniform(lower_highest);

    // The window: from `origin` on, ORDER_ROUNDS x ORDER_BITS indices, continuing at index 0 after the last one.
    // Either the whole range fits, or the indices of the upper half followed by those of the lower half do.
    constexpr uint32_t WINDOW = ORDER_ROUNDS * ORDER_BITS;
    uint32_t origin = lowest;
    uint32_t last = highest - lowest; // of the window
    if (last >= WINDOW && upper_lowest != 0xFFFFFFFFu && lowest < half &&
        static_cast<uint64_t>(g.n_points - upper_lowest) + lower_highest < WINDOW) {
        origin = upper_lowest;
        last = (g.n_points - upper_lowest) + lower_highest;
    }
    bool window = last < WINDOW;
    // a point can only be seen twice when the stencil wraps around the box along some direction
    for (int d = 0; d < 3; d++) {
        window = window && !(g.periodic[d] && g.n[d] < 2 * g.s[d] + 1);
    }
    if (args.report_order != 0 && lane == 0) {
        atomicAdd(window ? &args.status->windowed : &args.status->bucketed, 1u);
    }
    if (window) {
        auto& bits = sh.scratch.bits;
        uint32_t wrapped_around = 0; // candidates below the origin: first in the order, last in the window
#pragma unroll 4
        for (uint32_t k = lane; k < n_candidates; k += WAVE) {
            uint32_t at;
            int32_t packed_q;
            locate_candidate(sh, n_stencil, k, at, packed_q);
            const uint32_t index = sorted.p[at].index;
            const uint32_t offset = index >= origin ? index - origin : (g.n_points - origin) + index;
            wrapped_around += index < origin ? 1u : 0u;
            bits.offset[k] = static_cast<uint16_t>(offset % ORDER_BITS);
            bits.round_of[k] = static_cast<uint8_t>(offset / ORDER_BITS);
        }
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) {
            wrapped_around += static_cast<uint32_t>(__shfl_xor(static_cast<int>(wrapped_around), offset, WAVE));
        }
        const uint32_t in_window_first = n_candidates - wrapped_around; // candidates at or above the origin
        uint32_t carried = 0;                                           // candidates of the rounds before
        for (uint32_t round = 0; round <= last / ORDER_BITS; round++) {
            const uint32_t n_groups = (round < last / ORDER_BITS ? ORDER_BITS - 1 : last % ORDER_BITS) / 128 + 1;
            wave_sync();
            for (uint32_t group = lane; group < n_groups; group += WAVE) {
                *reinterpret_cast<uint4*>(&bits.present[4 * group]) = uint4{0u, 0u, 0u, 0u};
            }
            wave_sync();
#pragma unroll 4
            for (uint32_t k = lane; k < n_candidates; k += WAVE) {
                if (bits.round_of[k] == round) {
                    const uint32_t offset = bits.offset[k];
                    atomicOr(&bits.present[offset / 32], 1u << (offset % 32));
                }
            }
            wave_sync();
            const uint32_t carried_in = carried;
            for (uint32_t group0 = 0; group0 < n_groups; group0 += WAVE) {
                const uint32_t group = group0 + lane;
                uint32_t here = 0;
                if (group < n_groups) {
                    const uint4 words = *reinterpret_cast<const uint4*>(&bits.present[4 * group]);
                    here = __popc(words.x) + __popc(words.y) + __popc(words.z) + __popc(words.w);
                }
                const uint32_t through = wave_inclusive_scan(here);
                if (group < n_groups) {
                    bits.before[group] = static_cast<uint16_t>(carried + through - here);
                }
                carried += read_lane(through, WAVE - 1);
            }
            wave_sync();
            if (carried == carried_in) {
                continue; // no candidate in this stretch of the window
            }
#pragma unroll 4
            for (uint32_t k = lane; k < n_candidates; k += WAVE) {
                if (bits.round_of[k] == round) {
                    const uint32_t offset = bits.offset[k];
                    const uint32_t word = offset / 32;
                    const uint4 words = *reinterpret_cast<const uint4*>(&bits.present[word & ~3u]);
                    uint32_t place = bits.before[word / 4];
                    place += (word % 4 > 0) ? __popc(words.x) : 0;
                    place += (word % 4 > 1) ? __popc(words.y) : 0;
                    place += (word % 4 > 2) ? __popc(words.z) : 0;
                    const uint32_t own = word % 4 == 0 ? words.x : word % 4 == 1 ? words.y : word % 4 == 2 ? words.z : words.w;
                    place += __popc(own & ((1u << (offset % 32)) - 1u));
                    // the window's order starts at the origin, the order of the indices with those that wrapped around
                    place = place >= in_window_first ? place - in_window_first : place + wrapped_around;
                    tile_order[min(place, ORDERED_CANDIDATES - 1)] = static_cast<uint16_t>(k);
                }
            }
        }
        return;
    }

    auto& buckets = sh.scratch.buckets;
    const float per_index = static_cast<float>(ORDER_BUCKETS) / (static_cast<float>(highest - lowest) + 1.0f);
    auto bucket_of = [&](uint32_t index) {
        return min(ORDER_BUCKETS - 1, static_cast<uint32_t>(static_cast<float>(index - lowest) * per_index));
    };
    // the shift of a candidate, as it is ordered: only ever needed to tell two images of one point apart
    auto biased_of = [&](uint32_t k) {
        uint32_t at;
        int32_t packed_q;
        locate_candidate(sh, n_stencil, k, at, packed_q);
        int32_t qx, qy, qz;
        unpack_shift(packed_q, qx, qy, qz);
        // shifts beyond the key's fields make the counting pass call the whole search off: only memory safety
        // matters for them here
        return biased_shift(qx - sorted.wx[at], qy - sorted.wy[at], qz - sorted.wz[at]);
    };
#pragma unroll
    for (uint32_t b = 0; b < ORDER_BUCKETS / WAVE; b++) {
        buckets.bucket_end[b * WAVE + lane] = 0;
    }
    wave_sync();
#pragma unroll 4
    for (uint32_t k = lane; k < n_candidates; k += WAVE) {
        uint32_t at;
        int32_t packed_q;
        locate_candidate(sh, n_stencil, k, at, packed_q);
        const uint32_t index = sorted.p[at].index;
        buckets.index_of[k] = index;
        atomicAdd(&buckets.bucket_end[bucket_of(index)], 1u);
    }
    wave_sync();
    // lane l owns buckets 4l .. 4l+3
    uint32_t in_bucket[ORDER_BUCKETS / WAVE];
    uint32_t mine = 0;
#pragma unroll
    for (uint32_t b = 0; b < ORDER_BUCKETS / WAVE; b++) {
        in_bucket[b] = buckets.bucket_end[(ORDER_BUCKETS / WAVE) * lane + b];
        mine += in_bucket[b];
    }
    uint32_t before = wave_inclusive_scan(mine) - mine;
#pragma unroll
    for (uint32_t b = 0; b < ORDER_BUCKETS / WAVE; b++) {
        buckets.bucket_end[(ORDER_BUCKETS / WAVE) * lane + b] = before;
        before += in_bucket[b];
    }
    wave_sync();
#pragma unroll 4
    for (uint32_t k = lane; k < n_candidates; k += WAVE) {
        const uint32_t index = buckets.index_of[k];
        const uint32_t slot = min(atomicAdd(&buckets.bucket_end[bucket_of(index)], 1u), ORDERED_CANDIDATES - 1);
        buckets.grouped_index[slot] = index;
        buckets.grouped[slot] = static_cast<uint16_t>(k);
    }
    wave_sync();
    // every bucket now ends where the next one starts
#pragma unroll 2
    for (uint32_t slot = lane; slot < n_candidates; slot += WAVE) {
        const uint32_t index = buckets.grouped_index[slot];
        const uint32_t k = buckets.grouped[slot];
        const uint32_t bucket = bucket_of(index);
        const uint32_t first = bucket == 0 ? 0u : min(buckets.bucket_end[bucket - 1], ORDERED_CANDIDATES);
        const uint32_t end = min(buckets.bucket_end[bucket], ORDERED_CANDIDATES);
        uint32_t place = first;
        bool twice = false;
        for (uint32_t other = first; other < end; other++) {
            const uint32_t theirs = buckets.grouped_index[other];
            place += theirs < index ? 1u : 0u;
            twice = twice || (theirs == index && other != slot);
        }
        if (twice) {
            const uint32_t own = biased_of(k);
            for (uint32_t other = first; other < end; other++) {
                if (buckets.grouped_index[other] == index && other != slot) {
                    place += biased_of(buckets.grouped[other]) < own ? 1u : 0u;
                }
            }
        }
        tile_order[min(place, ORDERED_CANDIDATES - 1)] = static_cast<uint16_t>(k);
    }
}

} // namespace vesin_hip

#endif
