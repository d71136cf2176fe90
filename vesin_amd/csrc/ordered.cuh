// Search that produces a sorted list directly (options.sorted): rows grouped by first point in original index
// order and, within a point, ordered by second point and shift - the order the radix sort of sort.cuh produces,
// without sorting the rows as a whole.
//
// What makes that possible is giving up the half stencil: a tile's wave tests its points against the candidates of
// the whole (2s+1)^3 stencil, so every row (i, j, S) is found by the tile that holds i and by no other (a half
// list keeps i < j, or the self-image the reference's rule keeps, vesin/src/cpu_cell_list.cpp:101-133: the other
// orientation is found, and dropped, by the tile of j). Twice the distance tests of the other kernels, but then
//   COUNT  knows the number of rows of each of its points (one store per point, indexed by original index),
//   a scan over the points in original order gives every point its place in the output,
//   WRITE  keeps one hit column per candidate lane, then, point by point, collects the point's hits as 64-bit
//          keys (second point, biased shift) in LDS, ranks them (each lane counts the smaller keys: at most 256
//          keys, read as LDS broadcasts) and stores the row of rank r at the point's place + r.
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

/// What the counting pass found, for the host to decide between this path and the radix sort.
struct OrderedStatus {
    unsigned int max_rows;       // largest number of rows of one point
    unsigned int max_candidates; // largest number of candidates of one tile
    unsigned int unsuitable;     // tiles with a shift outside of the key's range
    unsigned int padding;
};

struct OrderedArgs {
    SortedPoints sorted;
    const uint64_t* cell_scan;
    const Tile* tiles;
    uint32_t points_per_item;   // a tile's points are dealt to ceil(TILE_POINTS / points_per_item) waves
    uint32_t items_per_tile;
    uint32_t* rows_of_point;    // COUNT: [n_points], by original index
    const uint64_t* first_row;  // WRITE: [n_points + 1], exclusive scan of rows_of_point
    OrderedStatus* status;
    SearchOutputs out;
};

/// LDS of one wave. What is known per candidate (hit column, position, original index, shift) stays in the
/// registers of the lane that loaded it: a lane only ever needs its own candidates until it hands a hit over as a key.
struct OrderedWaveShared: SearchTables {
    uint32_t tile_index[TILE_POINTS];
    double tile_x[TILE_POINTS], tile_y[TILE_POINTS], tile_z[TILE_POINTS];
    int32_t tile_wx[TILE_POINTS], tile_wy[TILE_POINTS], tile_wz[TILE_POINTS];
    uint64_t tile_row[TILE_POINTS];   // WRITE: first output row of each point
    // WRITE: (second point << 32) | biased shift, rows of one point; read four at a time, hence the padding
    __attribute__((aligned(16))) uint64_t keys[ORDERED_MAX_ROWS + 4];
    uint32_t key_at[ORDERED_MAX_ROWS];// WRITE: position of the second point in the cell-sorted arrays
};

struct OrderedShared {
    OrderedWaveShared wave[ORDERED_WAVES];
};

__device__ __forceinline__ uint32_t biased_shift(int32_t sx, int32_t sy, int32_t sz) {
    return (static_cast<uint32_t>(sx + 512) << 20) | (static_cast<uint32_t>(sy + 512) << 10) |
           static_cast<uint32_t>(sz + 512);
}

__device__ __forceinline__ bool beyond(int32_t a, int32_t b, int32_t c, int32_t limit) {
    return a > limit || a < -limit || b > limit || b < -limit || c > limit || c < -limit;
}

/// Two units of candidates (numbers unit0 * 64 ... + 127 of the tables) against the item's points: hit columns
/// (the item's first point in the highest bit used) and what the writing pass needs to know about each candidate.
template <bool FULL, bool WRAPPED>
__device__ __forceinline__ void ordered_sweep_pair(
    const OrderedWaveShared& sh, const SortedPoints& sorted, const GridParams& g, uint32_t unit0, uint32_t n_stencil,
    uint32_t n_candidates, uint32_t first_i, uint32_t n_i, int lane, uint32_t (&column)[ORDERED_R],
    uint32_t (&at)[ORDERED_R], uint32_t (&original)[ORDERED_R], int32_t (&packed_b)[ORDERED_R], bool& out_of_range
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
        c.position[r] = 0xFFFFFFFFu; // no candidate is left to another tile: the whole stencil is this tile's
        column[r] = 0;
        at[r] = 0xFFFFFFFFu;
        original[r] = 0;
        packed_q[r] = 0;
        int32_t bx = 0, by = 0, bz = 0;
        if (k < n_candidates) {
            locate_candidate(sh, n_stencil, k, at[r], packed_q[r]);
            int32_t qx, qy, qz;
            unpack_shift(packed_q[r], qx, qy, qz);
            c.x[r] = sorted.x[at[r]];
            c.y[r] = sorted.y[at[r]];
            c.z[r] = sorted.z[at[r]];
            original[r] = sorted.index[at[r]];
            bx = qx - sorted.wx[at[r]];
            by = qy - sorted.wy[at[r]];
            bz = qz - sorted.wz[at[r]];
            c.shift[r] = pack_shift(bx, by, bz);
            out_of_range = out_of_range || beyond(bx, by, bz, ORDERED_SHIFT_LIMIT);
        }
        packed_b[r] = c.shift[r];
        any_shift = any_shift || (__ballot((bx | by | bz) != 0) != 0);
        if (!WRAPPED && any_shift) {
            shift_vector(g, bx, by, bz, c.tx[r], c.ty[r], c.tz[r]);
        }
    }

    if (WRAPPED) {
        (void)sweep_columns_wrapped<R>(sorted, first_i, n_i, c, g, column);
    } else if (any_shift) {
        (void)sweep_columns<R, true, false>(sorted, first_i, n_i, c, g.cutoff2, column);
    } else {
        (void)sweep_columns<R, false, false>(sorted, first_i, n_i, c, g.cutoff2, column);
    }

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
}

template <bool WRITE, bool FULL>
__global__ __launch_bounds__(ORDERED_BLOCK) void ordered_search_kernel(OrderedArgs args, GridParams g) {
    constexpr int R = ORDERED_R;
    __shared__ OrderedShared shared;
    const int lane = lane_id();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    OrderedWaveShared& sh = shared.wave[wave];
    const uint32_t n_tiles = static_cast<uint32_t>(args.cell_scan[g.n_cells] >> 32);
    const uint32_t work = blockIdx.x * ORDERED_WAVES + wave;
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
    const int32_t cx = tile.cell % g.n[0];
    const int32_t cy = (tile.cell / g.n[0]) % g.n[1];
    const int32_t cz = tile.cell / (g.n[0] * g.n[1]);

    bool out_of_range = false;
    if (static_cast<uint32_t>(lane) < n_i) {
        const uint32_t at = first_i + lane;
        const uint32_t original = sorted.index[at];
        sh.tile_index[lane] = original;
        const int32_t wx = sorted.wx[at];
        const int32_t wy = sorted.wy[at];
        const int32_t wz = sorted.wz[at];
        out_of_range = beyond(wx, wy, wz, ORDERED_SHIFT_LIMIT);
        if (WRITE) {
            sh.tile_x[lane] = sorted.x[at];
            sh.tile_y[lane] = sorted.y[at];
            sh.tile_z[lane] = sorted.z[at];
            sh.tile_wx[lane] = wx;
            sh.tile_wy[lane] = wy;
            sh.tile_wz[lane] = wz;
            sh.tile_row[lane] = args.first_row[original];
        }
    }

    // the whole stencil, the tile's own cell included
    const int32_t span_y = 2 * g.s[1] + 1;
    const int32_t span_z = 2 * g.s[2] + 1;
    const uint32_t n_stencil = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z;
    if (n_stencil > MAX_ENTRIES) {
        return; // the host does not launch this kernel for such a stencil
    }
    fill_stencil_tables(sh, lane, 0, n_stencil, cx, cy, cz, span_y, span_z, g, args.cell_scan);
    const uint32_t n_candidates = __builtin_amdgcn_readfirstlane(sh.n_candidates);
    const uint32_t n_units = (n_candidates + WAVE - 1) / WAVE;

    if (!WRITE) {
        if (lane == 0 && item == 0) {
            atomicMax(&args.status->max_candidates, n_candidates);
        }
    }
    if (n_candidates > ORDERED_CANDIDATES) {
        return; // the host does not use this path for such a tile: nothing to count, nothing may be written
    }

    if constexpr (!WRITE) {
        // ---- COUNT: nothing is kept but the number of rows of every point (lane p adds up the hits of point p):
        // a plain loop over the pairs of units, small code
        uint32_t own_rows = 0;
        for (uint32_t unit0 = 0; unit0 < n_units; unit0 += R) {
            uint32_t column[R], at[R], original[R];
            int32_t packed_b[R];
            if (tile_wrapped) {
                ordered_sweep_pair<FULL, true>(
                    sh, sorted, g, unit0, n_stencil, n_candidates, first_i, n_i, lane, column, at, original, packed_b,
                    out_of_range
                );
            } else {
                ordered_sweep_pair<FULL, false>(
                    sh, sorted, g, unit0, n_stencil, n_candidates, first_i, n_i, lane, column, at, original, packed_b,
                    out_of_range
                );
            }
            for (uint32_t p = 0; p < n_i; p++) {
                const uint32_t bit = n_i - 1 - p;
                uint32_t rows = 0;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    rows += __popcll(__ballot(((column[r] >> bit) & 1u) != 0));
                }
                if (static_cast<uint32_t>(lane) == p) {
                    own_rows += rows;
                }
            }
        }
        if (static_cast<uint32_t>(lane) < n_i) {
            args.rows_of_point[sh.tile_index[lane]] = own_rows;
        }
        uint32_t most = own_rows;
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) {
            most = max(most, static_cast<uint32_t>(__shfl_xor(static_cast<int>(most), offset, WAVE)));
        }
        if (lane == 0) {
            atomicMax(&args.status->max_rows, most);
        }
        if (__ballot(out_of_range) != 0 && lane == 0) {
            atomicAdd(&args.status->unsuitable, 1u);
        }
        return;
    }

    // ---- sweep: per candidate (registers of its lane, indexed by unit) the hit column against this item's points
    uint32_t columns[ORDERED_UNITS];
    uint32_t cand_at[ORDERED_UNITS];
    uint32_t cand_index[ORDERED_UNITS];
    int32_t cand_shift[ORDERED_UNITS];
#pragma unroll
    for (int u = 0; u < ORDERED_UNITS; u++) {
        columns[u] = 0;
        cand_at[u] = 0;
        cand_index[u] = 0;
        cand_shift[u] = 0;
    }
#pragma unroll
    for (int pair = 0; pair < ORDERED_UNITS / R; pair++) {
        if (static_cast<uint32_t>(pair * R) < n_units) {
            uint32_t column[R], at[R], original[R];
            int32_t packed_b[R];
            if (tile_wrapped) {
                ordered_sweep_pair<FULL, true>(
                    sh, sorted, g, pair * R, n_stencil, n_candidates, first_i, n_i, lane, column, at, original, packed_b,
                    out_of_range
                );
            } else {
                ordered_sweep_pair<FULL, false>(
                    sh, sorted, g, pair * R, n_stencil, n_candidates, first_i, n_i, lane, column, at, original, packed_b,
                    out_of_range
                );
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                columns[pair * R + r] = column[r];
                if (WRITE) {
                    cand_at[pair * R + r] = at[r];
                    cand_index[pair * R + r] = original[r];
                    cand_shift[pair * R + r] = packed_b[r];
                }
            }
        }
    }

    // ---- WRITE: point by point, collect the hits, rank them, store the rows
    wave_sync();
    for (uint32_t p = 0; p < n_i; p++) {
        const uint32_t bit = n_i - 1 - p;
        const int32_t wix = sh.tile_wx[p];
        const int32_t wiy = sh.tile_wy[p];
        const int32_t wiz = sh.tile_wz[p];
        uint32_t n_rows = 0;
#pragma unroll
        for (int u = 0; u < ORDERED_UNITS; u++) {
            if (static_cast<uint32_t>(u) < n_units) {
                const bool hit = ((columns[u] >> bit) & 1u) != 0;
                const uint64_t mask = __ballot(hit);
                if (mask != 0) {
                    if (hit) {
                        int32_t bx, by, bz;
                        unpack_shift(cand_shift[u], bx, by, bz);
                        const uint32_t slot = n_rows + rank_in_mask(mask);
                        sh.keys[slot] = (static_cast<uint64_t>(cand_index[u]) << 32) |
                                        biased_shift(bx + wix, by + wiy, bz + wiz);
                        sh.key_at[slot] = cand_at[u];
                    }
                    n_rows += __popcll(mask);
                }
            }
        }
        if (n_rows == 0) {
            continue;
        }
        if (lane < 4) {
            sh.keys[n_rows + lane] = ~0ull; // larger than any key: the ranking reads whole groups of four
        }
        wave_sync();

        const double xi = sh.tile_x[p];
        const double yi = sh.tile_y[p];
        const double zi = sh.tile_z[p];
        const uint32_t oi = sh.tile_index[p];
        const uint64_t first_row = sh.tile_row[p];
        for (uint32_t e0 = 0; e0 < n_rows; e0 += WAVE) {
            const uint32_t e = e0 + lane;
            const bool active = e < n_rows;
            const uint64_t key = active ? sh.keys[e] : ~0ull;
            // the position in the cell-sorted arrays is known before the rank is: the loads overlap the ranking
            const uint32_t at = active ? sh.key_at[e] : 0;
            const double xj = sorted.x[at];
            const double yj = sorted.y[at];
            const double zj = sorted.z[at];
            uint32_t rank = 0;
            for (uint32_t other = 0; other < n_rows; other += 4) {
                // every lane reads the same 32 bytes: two LDS broadcasts for four comparisons
                const ulonglong2 first_two = *reinterpret_cast<const ulonglong2*>(&sh.keys[other]);
                const ulonglong2 next_two = *reinterpret_cast<const ulonglong2*>(&sh.keys[other + 2]);
                rank += (first_two.x < key ? 1u : 0u) + (first_two.y < key ? 1u : 0u);
                rank += (next_two.x < key ? 1u : 0u) + (next_two.y < key ? 1u : 0u);
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
                const uint64_t row = first_row + rank;
                args.out.pairs[2 * row + 0] = oi;
                args.out.pairs[2 * row + 1] = oj;
                if (args.out.shifts != nullptr) {
                    args.out.shifts[3 * row + 0] = sx;
                    args.out.shifts[3 * row + 1] = sy;
                    args.out.shifts[3 * row + 2] = sz;
                }
                if (args.out.distances != nullptr) {
                    args.out.distances[row] = sqrt(vx * vx + vy * vy + vz * vz);
                }
                if (args.out.vectors != nullptr) {
                    args.out.vectors[3 * row + 0] = vx;
                    args.out.vectors[3 * row + 1] = vy;
                    args.out.vectors[3 * row + 2] = vz;
                }
            }
        }
        wave_sync(); // the keys are about to be overwritten by the next point's
    }
}

} // namespace vesin_hip

#endif
