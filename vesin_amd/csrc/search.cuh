// Stencil search over the cell grid: the kernel that decides pair membership and produces the output arrays.
//
// One wave owns one tile = up to 32 points `i` of one cell. The candidates `j` are the points of the cells in
// the upper half of the (2s+1)^3 stencil around that cell (offsets that are lexicographically positive, plus the
// cell itself restricted to later points), periodic images included: every unordered pair {(i, j, S), (j, i, -S)}
// is tested exactly once, by the tile of one of its two points, and both rows are produced from that one test.
// A cell may appear several times in the stencil with different cell shifts when the box is narrower than the
// stencil: that is the multi-image path; with a single cell the stencil enumerates images only and the kernel is
// a tiled brute force, the candidates of a tile being sliced over several waves.
//
// Mapping: lanes hold candidates. A wave loads R groups of 64 consecutive candidates into registers (coalesced
// reads of the cell-sorted 32-byte records), then loops over the tile's points, whose coordinates come in
// through scalar loads (four points per round trip) and are used as scalar operands. One (i, group) test is 9 fp64
// VALU operations (12 when a shift vector has to be added) and yields a 64-bit hit mask in scalar registers. The
// loop is compiled in four variants (candidates shifted or not, tile's own cell among them or not), picked per
// group batch, plus a general variant for tiles holding points that were wrapped into the box.
//
// The same code runs twice:
//   COUNT  adds up popcounts: one 32-bit total per wave, no atomics;
//   WRITE  (after a device-wide scan of the totals gave every wave its output range) recomputes the masks and
//          compacts: hit lanes drop a 16-bit ticket (lane, group, i) into a per-wave LDS ring at the slot given by
//          mbcnt of the mask; whenever 64 tickets are pending, all 64 lanes redeem one each, pulling the
//          candidate's data out of the owning lane with ds_bpermute, recomputing shift / vector / distance and
//          storing the rows: (i, j, S) and its mirror (j, i, -S) for a full list, the one of the two that the
//          half-list rule keeps otherwise. A wave's rows are consecutive in the output.
//
// Arithmetic (bit-for-bit the CPU reference, vesin/src/cpu_cell_list.cpp:135-138 and vesin/src/types.hpp:232-243,
// vesin/src/math.hpp:14-16,111-117; compile with -ffp-contract=off):
//   T_k = S0*H0k + S1*H1k + S2*H2k (left to right), v_k = (r_jk - r_ik) + T_k, d2 = v0*v0 + v1*v1 + v2*v2,
//   keep iff d2 < cutoff*cutoff, d = sqrt(d2).
// Adding T may be skipped in the test when S = 0 (it is +-0 and cannot change d2); the stored vector always adds it.
// The mirror row is exact as well: r_i - r_j and T(-S) are the exact negations of r_j - r_i and T(S) (T(0) is not
// negated), so d2 is the same number and the vector is recomputed as (r_i - r_j) + T(-S).
//
// Workgroups are dealt to the 8 XCDs round-robin by the hardware; the work index is remapped so that each XCD
// walks one contiguous range of tiles (one slab of the grid) and its L2 sees the same cells again and again.
//
// Reference roles replaced: find_neighbors_cell_list (vesin/src/cuda/cell_list.cu:428-705), brute_force_*
// (vesin/src/cuda/bruteforce.cu:241-573); CPU twin CellList::foreach_pair + callback
// (vesin/src/cpu_cell_list.cpp:376-451, :100-163).
#ifndef VESIN_HIP_SEARCH_CUH
#define VESIN_HIP_SEARCH_CUH

#include <type_traits>

#include "cells.cuh"
#include "device_common.cuh"

namespace vesin_hip {

constexpr int SEARCH_WAVES = 4;    // waves per workgroup; every wave works on its own tile, they never synchronise
constexpr int SEARCH_BLOCK = SEARCH_WAVES * WAVE;
constexpr int MAX_ENTRIES = 64;    // stencil entries resident in LDS at a time (14 for the usual 3x3x3 stencil)
constexpr int RING = 128;          // tickets per wave ring (power of two, >= 2 * WAVE)
constexpr int N_XCD = 8;

struct SearchOutputs {
    unsigned long long* pairs; // [P][2]
    int32_t* shifts;           // [P][3] or null
    double* distances;         // [P] or null
    double* vectors;           // [P][3] or null
};

struct SearchArgs {
    SortedPoints sorted;
    const uint64_t* cell_scan; // [n_cells + 1]: points before the cell | (tiles before the cell << 32)
    const Tile* tiles;
    uint32_t* counts;          // COUNT: rows produced by every work item
    const uint64_t* offsets;   // WRITE: exclusive scan of counts
    SearchOutputs out;
    uint32_t n_slices;         // work items sharing one tile (each takes a slice of the candidates)
    uint32_t n_work;           // work items = tile slots * n_slices; tile slots are a multiple of
                               // N_XCD * SEARCH_WAVES and at least the number of tiles
    uint64_t capacity;         // WRITE: rows the output arrays hold; a launch that would overflow writes nothing
    const uint32_t* only;      // WRITE: when not null, only work items with a non-zero entry are processed
    // fixed-capacity layout of the cells (place_direct), understood by the single-pass search only; 0 otherwise
    uint32_t direct_capacity;  // slots per cell, a multiple of TILE_POINTS
    const uint32_t* direct_counts;  // points of every cell
    const uint32_t* direct_wrapped; // per tile: holds a point that was moved by a box vector
    // many systems in one launch (batched entry point); null / zero otherwise
    const GridParams* grids;   // one per system
    const uint32_t* cell_base; // first cell of every system in the concatenated grids, n_systems + 1 entries
    uint32_t total_cells;
};

/// In a batch the tile remembers its system next to the flag: bit 0 = holds wrapped points, bits 1.. = system.
__device__ __forceinline__ uint32_t tile_system(const Tile& tile) {
    return tile.wrapped >> 1;
}

__device__ __forceinline__ int32_t pack_shift(int32_t a, int32_t b, int32_t c) {
    // three signed 10-bit fields
    return (a & 0x3ff) | ((b & 0x3ff) << 10) | ((c & 0x3ff) << 20);
}

__device__ __forceinline__ void unpack_shift(int32_t packed, int32_t& a, int32_t& b, int32_t& c) {
    a = (packed << 22) >> 22;
    b = (packed << 12) >> 22;
    c = (packed << 2) >> 22;
}

/// Cartesian shift T = S . H with the reference's operation order.
__device__ __forceinline__ void shift_vector(
    const GridParams& g, int32_t sx, int32_t sy, int32_t sz, double& tx, double& ty, double& tz
) {
    double a = static_cast<double>(sx);
    double b = static_cast<double>(sy);
    double c = static_cast<double>(sz);
    tx = a * g.H[0] + b * g.H[3] + c * g.H[6];
    ty = a * g.H[1] + b * g.H[4] + c * g.H[7];
    tz = a * g.H[2] + b * g.H[5] + c * g.H[8];
}

/// Half-list rule of the reference (vesin/src/cpu_cell_list.cpp:101-133) for a pair of a point with its own image.
__device__ __forceinline__ bool half_keeps_self_image(int32_t sx, int32_t sy, int32_t sz) {
    int32_t sum = sx + sy + sz;
    if (sum < 0) {
        return false;
    }
    if (sum == 0 && (sz < 0 || (sz == 0 && sy < 0))) {
        return false;
    }
    return true;
}

/// R x 64 candidates held in registers by one wave.
template <int R>
struct Candidates {
    double x[R], y[R], z[R];    // position (NaN for lanes past the end: never a hit)
    double tx[R], ty[R], tz[R]; // shift vector against a tile point that was not wrapped
    int32_t bx[R], by[R], bz[R];// cell shift minus the candidate's own wrap shift
    uint32_t position[R];       // position in the cell-sorted arrays if the candidate comes from the tile's own
                                // cell with a zero cell shift (only later points are partners), else ~0
    bool any_shift;             // some lane has a non-zero base shift
    bool any_same;              // some lane comes from the tile's own, unshifted cell
};

/// LDS of one wave. The counting pass only needs the stencil tables.
struct SearchTables {
    uint32_t ent_prefix[MAX_ENTRIES + 1]; // candidates before each stencil entry
    uint32_t ent_start[MAX_ENTRIES];      // first sorted position of the entry's cell
    int32_t ent_shift[MAX_ENTRIES];       // packed cell shift, bit 30: the tile's own cell with a zero cell shift
    uint32_t n_candidates;
};

/// For the kernels with the single-precision pre-test (choose_prefilter in geometry.hpp): from the origin of the
/// tile's cell to the origin of each entry's cell, box shift included, in single precision.
struct SearchOffsets {
    float ent_dx[MAX_ENTRIES], ent_dy[MAX_ENTRIES], ent_dz[MAX_ENTRIES];
};

struct SearchSharedCount: SearchTables {
    uint16_t ring[1];
};

constexpr int MAX_R = 2;

struct SearchSharedWrite: SearchTables {
    // the tile's points, for the redeem phase
    double tile_x[TILE_POINTS], tile_y[TILE_POINTS], tile_z[TILE_POINTS];
    uint32_t tile_index[TILE_POINTS];
    int32_t tile_wx[TILE_POINTS], tile_wy[TILE_POINTS], tile_wz[TILE_POINTS];
    // the candidates currently held in registers, where any lane can fetch them when it redeems a ticket
    double cand_x[MAX_R * WAVE], cand_y[MAX_R * WAVE], cand_z[MAX_R * WAVE];
    uint32_t cand_index[MAX_R * WAVE];
    int32_t cand_bx[MAX_R * WAVE], cand_by[MAX_R * WAVE], cand_bz[MAX_R * WAVE];
    uint16_t ring[RING];
};

/// LDS written by some lanes is about to be read by others of the same wave: the hardware keeps one wave's LDS
/// operations in order, this only stops the compiler from reordering them.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
    __builtin_amdgcn_wave_barrier();
}

/// Stencil entries [first_linear, first_linear + n_batch) around cell (cx, cy, cz) go to the wave's LDS tables:
/// neighbour cell start, packed cell shift, and the running number of candidates (scanned in place). Linear stencil
/// offsets run dx major, dz minor. `cell_scan`: exclusive scan of the points per cell in the low 32 bits of its words.
template <typename ScanWord>
__device__ __forceinline__ void fill_stencil_tables(
    SearchTables& sh, int lane, uint32_t first_linear, uint32_t n_batch, int32_t cx, int32_t cy, int32_t cz,
    int32_t span_y, int32_t span_z, const GridParams& g, const ScanWord* __restrict__ cell_scan,
    const uint32_t* __restrict__ direct_counts = nullptr, uint32_t direct_capacity = 0, SearchOffsets* offsets = nullptr,
    const Prefilter* pre = nullptr
) {
    const uint32_t centre = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z / 2;
    for (uint32_t e = lane; e < n_batch; e += WAVE) {
        const uint32_t linear = first_linear + e;
        int32_t dx, dy, dz;
        if (span_y == 3 && span_z == 3) {
            // the usual stencil of radius one: divisions by constants
            dz = static_cast<int32_t>(linear % 3u) - 1;
            dy = static_cast<int32_t>((linear / 3u) % 3u) - 1;
            dx = static_cast<int32_t>(linear / 9u) - g.s[0];
        } else {
            dz = static_cast<int32_t>(linear % span_z) - g.s[2];
            dy = static_cast<int32_t>((linear / span_z) % span_y) - g.s[1];
            dx = static_cast<int32_t>(linear / (span_z * span_y)) - g.s[0];
        }
        int32_t cell[3] = {cx + dx, cy + dy, cz + dz};
        int32_t q[3] = {0, 0, 0};
        bool valid = true;
#pragma unroll
        for (int d = 0; d < 3; d++) {
            const int32_t n = g.n[d];
            if (g.periodic[d]) {
                if (g.s[d] <= n) {
                    // the neighbour is at most one box away: no division needed
                    if (cell[d] < 0) {
                        cell[d] += n;
                        q[d] = -1;
                    } else if (cell[d] >= n) {
                        cell[d] -= n;
                        q[d] = 1;
                    }
                } else {
                    int32_t quotient = cell[d] / n;
                    int32_t rest = cell[d] - quotient * n;
                    if (rest < 0) {
                        rest += n;
                        quotient -= 1;
                    }
                    q[d] = quotient;
                    cell[d] = rest;
                }
            } else if (cell[d] < 0 || cell[d] >= n) {
                valid = false;
            }
        }
        if (stencil_entry_too_far(g, dx, dy, dz)) {
            // points lie inside their cells: no pair between these two cells is within the cutoff
            valid = false;
        }
        uint32_t start = 0;
        uint32_t count = 0;
        int32_t packed = 0;
        if (valid) {
            uint32_t neighbour = (static_cast<uint32_t>(cell[2]) * g.n[1] + cell[1]) * g.n[0] + cell[0];
            if (direct_capacity != 0) {
                start = neighbour * direct_capacity;
                count = min(direct_counts[neighbour], direct_capacity);
            } else {
                start = static_cast<uint32_t>(cell_scan[neighbour]);
                count = static_cast<uint32_t>(cell_scan[neighbour + 1]) - start;
            }
            packed = pack_shift(q[0], q[1], q[2]);
            if (linear == centre) {
                packed |= 1 << 30;
            }
        }
        sh.ent_start[e] = start;
        sh.ent_shift[e] = packed;
        sh.ent_prefix[e + 1] = count; // scanned in place below
        if (offsets != nullptr) {
            const double ox = static_cast<double>(dx), oy = static_cast<double>(dy), oz = static_cast<double>(dz);
            offsets->ent_dx[e] = static_cast<float>(ox * pre->cell_edges[0] + oy * pre->cell_edges[3] + oz * pre->cell_edges[6]);
            offsets->ent_dy[e] = static_cast<float>(ox * pre->cell_edges[1] + oy * pre->cell_edges[4] + oz * pre->cell_edges[7]);
            offsets->ent_dz[e] = static_cast<float>(ox * pre->cell_edges[2] + oy * pre->cell_edges[5] + oz * pre->cell_edges[8]);
        }
    }
    wave_sync();

    uint32_t carry = 0;
    for (uint32_t base = 0; base < n_batch; base += WAVE) {
        uint32_t e = base + lane;
        uint32_t v = e < n_batch ? sh.ent_prefix[e + 1] : 0;
        uint32_t inclusive = wave_inclusive_scan(v) + carry;
        if (e < n_batch) {
            sh.ent_prefix[e + 1] = inclusive;
        }
        carry = read_lane(inclusive, WAVE - 1);
    }
    if (lane == 0) {
        sh.ent_prefix[0] = 0;
    }
    sh.n_candidates = carry;
    wave_sync();
}

/// Candidate number k of the tables: its position in the cell-sorted arrays and the packed shift of its cell.
__device__ __forceinline__ void locate_candidate(
    const SearchTables& sh, uint32_t n_batch, uint32_t k, uint32_t& at, int32_t& packed
) {
    // largest e < n_batch with ent_prefix[e] <= k: six steps without a branch, so that lookups that do not depend
    // on each other (the units a wave takes together) advance side by side instead of one loop after the other.
    // The table has MAX_ENTRIES + 1 words; what lies beyond n_batch is read and ignored.
    static_assert(MAX_ENTRIES <= 64, "six steps cover the table");
    uint32_t lo = 0;
#pragma unroll
    for (uint32_t step = 32; step > 0; step >>= 1) {
        const uint32_t probe = lo + step;
        const uint32_t before = sh.ent_prefix[min(probe, static_cast<uint32_t>(MAX_ENTRIES))];
        const uint32_t take = (probe < n_batch ? 1u : 0u) & (before <= k ? 1u : 0u);
        lo = take != 0 ? probe : lo;
    }
    at = sh.ent_start[lo] + (k - sh.ent_prefix[lo]);
    packed = sh.ent_shift[lo];
}

/// The same, also telling the entry the candidate belongs to.
__device__ __forceinline__ void locate_candidate(
    const SearchTables& sh, uint32_t n_batch, uint32_t k, uint32_t& at, int32_t& packed, uint32_t& entry
) {
    uint32_t lo = 0;
#pragma unroll
    for (uint32_t step = 32; step > 0; step >>= 1) {
        const uint32_t probe = lo + step;
        const uint32_t before = sh.ent_prefix[min(probe, static_cast<uint32_t>(MAX_ENTRIES))];
        const uint32_t take = (probe < n_batch ? 1u : 0u) & (before <= k ? 1u : 0u);
        lo = take != 0 ? probe : lo;
    }
    at = sh.ent_start[lo] + (k - sh.ent_prefix[lo]);
    packed = sh.ent_shift[lo];
    entry = lo;
}

/// Stores of 64 consecutive rows are fastest when they start on whole cache lines in all three arrays (16, 12 and
/// 8 bytes per row): at multiples of 32 rows. A wave's first row is wherever the rows before it ended, so its first
/// redeem takes just enough tickets to reach such a boundary.
constexpr uint32_t ROW_ALIGN = 32;

template <bool FULL>
__device__ __forceinline__ uint32_t aligning_batch(uint64_t cursor) {
    const uint32_t off = static_cast<uint32_t>(cursor) & (ROW_ALIGN - 1);
    if (off == 0) {
        return WAVE;
    }
    // a full list writes two rows per ticket (its cursor is always even)
    return FULL ? (ROW_ALIGN - off) / 2 : ROW_ALIGN - off;
}

/// Per-wave progress, kept in scalar registers.
struct WaveState {
    uint32_t total;      // COUNT: hits found so far
    uint64_t out_cursor; // WRITE: next output row of this wave
    uint32_t head;       // tickets appended to the ring
    uint32_t tail;       // tickets redeemed
    uint32_t batch;      // WRITE: tickets the next redeem takes, see aligning_batch
};

/// Constants of one work item.
struct SweepContext {
    double zero_tx, zero_ty, zero_tz; // shift vector of the zero shift: +0 or -0 per component
    bool tile_wrapped;
    int lane;
};

/// Redeem up to 64 tickets: every lane rebuilds one pair from its ticket and stores its row(s).
template <bool FULL, int R>
__device__ __forceinline__ void redeem(
    uint32_t n, WaveState& state, const Candidates<R>& c, SearchSharedWrite& sh, const SearchOutputs& out,
    const GridParams& g, const SweepContext& ctx
) {
    // tickets were written by other lanes of this wave: LDS operations of one wave complete in order, the fence only
    // keeps the compiler from moving the read above the writes
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int lane = ctx.lane;
    const bool active = static_cast<uint32_t>(lane) < n;
    const uint32_t ticket = sh.ring[(state.tail + lane) & (RING - 1)];
    const int slot = active ? ticket & (MAX_R * WAVE - 1) : 0; // group r, lane l -> r * 64 + l
    const int il = active ? (ticket >> 8) & 63 : 0;
    const bool need_shift = c.any_shift || ctx.tile_wrapped;

    const double xj = sh.cand_x[slot];
    const double yj = sh.cand_y[slot];
    const double zj = sh.cand_z[slot];
    const uint32_t oj = sh.cand_index[slot];
    int32_t sx = 0, sy = 0, sz = 0;
    if (need_shift) {
        sx = sh.cand_bx[slot];
        sy = sh.cand_by[slot];
        sz = sh.cand_bz[slot];
    }

    const double xi = sh.tile_x[il];
    const double yi = sh.tile_y[il];
    const double zi = sh.tile_z[il];
    const uint32_t oi = sh.tile_index[il];

    // the stored vector always adds T, even when S = 0 (T = +-0 then): bit-identical zeros.
    // (tx, ty, tz) = T(S); (mx, my, mz) = T(-S), which is -T(S) exactly unless S = 0
    double tx = ctx.zero_tx, ty = ctx.zero_ty, tz = ctx.zero_tz;
    double mx = ctx.zero_tx, my = ctx.zero_ty, mz = ctx.zero_tz;
    if (need_shift) {
        if (ctx.tile_wrapped) {
            sx += sh.tile_wx[il];
            sy += sh.tile_wy[il];
            sz += sh.tile_wz[il];
        }
        shift_vector(g, sx, sy, sz, tx, ty, tz);
        if ((sx | sy | sz) != 0) {
            mx = -tx;
            my = -ty;
            mz = -tz;
        }
    }
    const double vx = (xj - xi) + tx;
    const double vy = (yj - yi) + ty;
    const double vz = (zj - zi) + tz;
    const double wx = (xi - xj) + mx;
    const double wy = (yi - yj) + my;
    const double wz = (zi - zj) + mz;
    const double d2 = vx * vx + vy * vy + vz * vz;

    if (FULL) {
        // two rows per ticket: the n pairs first, then their n mirrors, so that every store instruction of the
        // wave covers one dense, contiguous range
        if (active) {
            const uint64_t forward_row = state.out_cursor + lane;
            const uint64_t mirror_row = forward_row + n;
            stream_store(reinterpret_cast<PairRow*>(out.pairs) + forward_row, PairRow{oi, oj});
            stream_store(reinterpret_cast<PairRow*>(out.pairs) + mirror_row, PairRow{oj, oi});
            if (out.shifts != nullptr) {
                stream_store(out.shifts + 3 * forward_row, ShiftRow{sx, sy, sz});
                stream_store(out.shifts + 3 * mirror_row, ShiftRow{-sx, -sy, -sz});
            }
            if (out.distances != nullptr) {
                const double d = sqrt(d2);
                stream_store(out.distances + forward_row, d);
                stream_store(out.distances + mirror_row, d);
            }
            if (out.vectors != nullptr) {
                stream_store(out.vectors + 3 * forward_row, VectorHead{vx, vy});
                stream_store(out.vectors + 3 * forward_row + 2, vz);
                stream_store(out.vectors + 3 * mirror_row, VectorHead{wx, wy});
                stream_store(out.vectors + 3 * mirror_row + 2, wz);
            }
        }
        state.out_cursor += 2 * n;
    } else {
        // one row per ticket, oriented like the reference's half list: smaller original index first; a point with
        // its own image keeps the shift the half-list rule accepts
        const bool flip = oi > oj || (oi == oj && !half_keeps_self_image(sx, sy, sz));
        if (active) {
            const uint64_t row = state.out_cursor + lane;
            stream_store(reinterpret_cast<PairRow*>(out.pairs) + row, PairRow{flip ? oj : oi, flip ? oi : oj});
            if (out.shifts != nullptr) {
                stream_store(out.shifts + 3 * row, ShiftRow{flip ? -sx : sx, flip ? -sy : sy, flip ? -sz : sz});
            }
            if (out.distances != nullptr) {
                stream_store(out.distances + row, sqrt(d2));
            }
            if (out.vectors != nullptr) {
                stream_store(out.vectors + 3 * row, VectorHead{flip ? wx : vx, flip ? wy : vy});
                stream_store(out.vectors + 3 * row + 2, flip ? wz : vz);
            }
        }
        state.out_cursor += n;
    }
    state.tail += n;
    state.batch = aligning_batch<FULL>(state.out_cursor);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

/// What happens to the hit mask of one (tile point, candidate group).
template <bool WRITE, bool FULL, int R, typename Shared>
__device__ __forceinline__ void consume(
    uint64_t mask, int r, uint32_t i, WaveState& state, const Candidates<R>& c, Shared& sh, const SearchOutputs& out,
    const GridParams& g, const SweepContext& ctx
) {
    if (mask != 0) {
        const uint32_t hits = __popcll(mask);
        if constexpr (WRITE) {
            if (__builtin_amdgcn_inverse_ballot_w64(mask)) {
                const uint32_t at = (state.head + rank_in_mask(mask)) & (RING - 1);
                sh.ring[at] = static_cast<uint16_t>(ctx.lane | (r << 6) | (i << 8));
            }
            state.head += hits;
            while (state.head - state.tail >= state.batch) {
                redeem<FULL, R>(state.batch, state, c, sh, out, g, ctx);
            }
        } else {
            state.total += hits;
        }
    }
}

typedef uint32_t ScalarWords8 __attribute__((ext_vector_type(8)));

constexpr int POINTS_PER_LOAD = 4;

/// Four consecutive cell-sorted points, in scalar registers: words 0-1 x, 2-3 y, 4-5 z, 6 index of each.
struct FourPoints {
    ScalarWords8 q[POINTS_PER_LOAD];
};

/// Four scalar loads (s_load_dwordx8, a point each) issued back to back and waited for inside one asm statement, so
/// the compiler never sees the registers before the data arrived. The address is wave-uniform. Reading up to three
/// points past the end of a tile is harmless: the array is padded.
__device__ __forceinline__ FourPoints load_four_points(const SortedPoint* first) {
    static_assert(sizeof(SortedPoint) == 32, "one s_load_dwordx8 per point");
    FourPoints p;
    asm volatile(
        "s_load_dwordx8 %0, %4, 0x0\n\t"
        "s_load_dwordx8 %1, %4, 0x20\n\t"
        "s_load_dwordx8 %2, %4, 0x40\n\t"
        "s_load_dwordx8 %3, %4, 0x60\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&s"(p.q[0]), "=&s"(p.q[1]), "=&s"(p.q[2]), "=&s"(p.q[3])
        : "s"(first)
    );
    return p;
}

typedef uint32_t ScalarWords4 __attribute__((ext_vector_type(4)));

/// The box vectors four consecutive cell-sorted points were moved by, in scalar registers (wave-uniform address;
/// the three arrays are padded like the coordinates).
struct FourWraps {
    ScalarWords4 x, y, z;
};

__device__ __forceinline__ FourWraps load_four_wraps(const int32_t* wx, const int32_t* wy, const int32_t* wz) {
    FourWraps w;
    asm volatile(
        "s_load_dwordx4 %0, %3, 0x0\n\t"
        "s_load_dwordx4 %1, %4, 0x0\n\t"
        "s_load_dwordx4 %2, %5, 0x0\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&s"(w.x), "=&s"(w.y), "=&s"(w.z)
        : "s"(wx), "s"(wy), "s"(wz)
    );
    return w;
}

__device__ __forceinline__ double words_to_double(uint32_t lo, uint32_t hi) {
    return __longlong_as_double(static_cast<long long>((static_cast<uint64_t>(hi) << 32) | lo));
}

/// Every tile point against the R x 64 candidates, for a tile none of whose points was wrapped: the shift of a
/// pair is the candidate's base shift. SHIFTED / SAME say what this batch of candidates can contain.
template <bool WRITE, bool FULL, int R, bool SHIFTED, bool SAME, typename Shared>
__device__ __forceinline__ void sweep_unwrapped(
    const SortedPoints& sorted, uint32_t first_i, uint32_t n_i,
    WaveState& state, const Candidates<R>& c, Shared& sh, const SearchOutputs& out,
    const GridParams& g, const SweepContext& ctx
) {
    for (uint32_t i0 = 0; i0 < n_i; i0 += POINTS_PER_LOAD) {
        const uint32_t at = first_i + i0;
        const FourPoints p = load_four_points(sorted.p + at);
#pragma unroll
        for (int u = 0; u < POINTS_PER_LOAD; u++) {
            if (u > 0 && i0 + u >= n_i) {
                break;
            }
            const uint32_t i = i0 + u;
            const double xi = words_to_double(p.q[u][0], p.q[u][1]);
            const double yi = words_to_double(p.q[u][2], p.q[u][3]);
            const double zi = words_to_double(p.q[u][4], p.q[u][5]);
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
                // each condition is one compare whose lane mask lands in scalar registers; they are combined there
                uint64_t mask = __ballot(d2 < g.cutoff2);
                if (SAME) {
                    // inside the tile's own cell only later points are partners (earlier ones find this point)
                    mask &= __ballot(c.position[r] > at + u);
                }
                consume<WRITE, FULL, R>(mask, r, i, state, c, sh, out, g, ctx);
            }
        }
    }
}

/// General variant: the tile holds wrapped points, so the shift depends on both points of a pair. Against a point
/// that was not moved itself the shift is the candidate's own, whose vector the candidates carry.
template <bool WRITE, bool FULL, int R, typename Shared>
__device__ __forceinline__ void sweep_wrapped(
    const SortedPoints& sorted, uint32_t first_i, uint32_t n_i,
    WaveState& state, const Candidates<R>& c, Shared& sh, const SearchOutputs& out,
    const GridParams& g, const SweepContext& ctx
) {
    for (uint32_t i = 0; i < n_i; i++) {
        const uint32_t at = first_i + i;
        const double xi = sorted.p[at].x;
        const double yi = sorted.p[at].y;
        const double zi = sorted.p[at].z;
        const int32_t wix = static_cast<int32_t>(uniform(static_cast<uint32_t>(sorted.wx[at])));
        const int32_t wiy = static_cast<int32_t>(uniform(static_cast<uint32_t>(sorted.wy[at])));
        const int32_t wiz = static_cast<int32_t>(uniform(static_cast<uint32_t>(sorted.wz[at])));
        const bool moved = (wix | wiy | wiz) != 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            double tx = c.tx[r];
            double ty = c.ty[r];
            double tz = c.tz[r];
            if (moved) {
                shift_vector(g, c.bx[r] + wix, c.by[r] + wiy, c.bz[r] + wiz, tx, ty, tz);
            }
            const double vx = (c.x[r] - xi) + tx;
            const double vy = (c.y[r] - yi) + ty;
            const double vz = (c.z[r] - zi) + tz;
            const double d2 = vx * vx + vy * vy + vz * vz;
            const uint64_t mask = __ballot(d2 < g.cutoff2) & __ballot(c.position[r] > at);
            consume<WRITE, FULL, R>(mask, r, i, state, c, sh, out, g, ctx);
        }
    }
}

/// One work item: one tile (or one slice of its candidates) searched by one wave.
template <bool WRITE, bool FULL, int R, bool BATCH, typename Shared>
__device__ __forceinline__ void search_work_item(
    uint32_t work, const SearchArgs& args, const GridParams& single_grid, Shared& sh, uint32_t n_tiles, int lane
) {
    const uint32_t slice = work % args.n_slices;

    // XCD-aware order: the hardware deals workgroups to the 8 XCDs round-robin, so slot u (wave u % 4 of workgroup
    // u / 4) runs on XCD (u / 4) % 8; each XCD walks its own contiguous range of tiles
    const uint32_t slot = work / args.n_slices;
    const uint32_t per_xcd = (n_tiles + N_XCD - 1) / N_XCD;
    const uint32_t xcd = (slot / SEARCH_WAVES) % N_XCD;
    const uint32_t within = (slot / (SEARCH_WAVES * N_XCD)) * SEARCH_WAVES + slot % SEARCH_WAVES;
    const uint32_t tile_id = xcd * per_xcd + within;

    if (within >= per_xcd || tile_id >= n_tiles) {
        if (!WRITE && !BATCH && lane == 0) {
            args.counts[work] = 0;
        }
        return;
    }
    // In a batch the rows of a work item are counted and placed under its tile's number, not under the number of
    // the wave that happens to run it: the rows of one system stay together (the host clears `counts` first).
    const uint32_t row_slot = BATCH ? tile_id * args.n_slices + slice : work;

    const Tile tile = args.tiles[tile_id];
    const uint32_t n_i = tile.count;
    const uint32_t first_i = tile.first;

    // the grid: the kernel's argument, or this tile's system's
    GridParams batch_grid;
    uint32_t first_cell = 0;
    if (BATCH) {
        const uint32_t system = tile_system(tile);
        batch_grid = args.grids[system];
        first_cell = args.cell_base[system];
    }
    const GridParams& g = BATCH ? batch_grid : single_grid;
    const uint64_t* __restrict__ cell_scan = args.cell_scan + first_cell;
    const uint32_t local_cell = tile.cell - first_cell;
    const int32_t cx = local_cell % g.n[0];
    const int32_t cy = (local_cell / g.n[0]) % g.n[1];
    const int32_t cz = local_cell / (g.n[0] * g.n[1]);

    const SortedPoint* __restrict__ pp = args.sorted.p;
    const int32_t* __restrict__ pwx = args.sorted.wx;
    const int32_t* __restrict__ pwy = args.sorted.wy;
    const int32_t* __restrict__ pwz = args.sorted.wz;

    if constexpr (WRITE) {
        if (static_cast<uint32_t>(lane) < n_i) {
            const uint32_t at = first_i + lane;
            sh.tile_x[lane] = pp[at].x;
            sh.tile_y[lane] = pp[at].y;
            sh.tile_z[lane] = pp[at].z;
            sh.tile_index[lane] = pp[at].index;
            sh.tile_wx[lane] = pwx[at];
            sh.tile_wy[lane] = pwy[at];
            sh.tile_wz[lane] = pwz[at];
        }
    }

    SweepContext ctx;
    ctx.tile_wrapped = (tile.wrapped & 1u) != 0;
    ctx.lane = lane;
    shift_vector(g, 0, 0, 0, ctx.zero_tx, ctx.zero_ty, ctx.zero_tz);

    // upper half of the stencil: linear offsets from the centre (the cell itself) to the last one, in the order
    // dx major, dz minor, are exactly the lexicographically non-negative offsets
    const int32_t span_y = 2 * g.s[1] + 1;
    const int32_t span_z = 2 * g.s[2] + 1;
    const uint32_t n_stencil = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z;
    const uint32_t centre = n_stencil / 2;
    const uint32_t n_entries = n_stencil - centre;

    WaveState state;
    state.total = 0;
    state.out_cursor = WRITE ? args.offsets[row_slot] : 0;
    state.head = 0;
    state.tail = 0;
    state.batch = aligning_batch<FULL>(state.out_cursor);

    for (uint32_t batch = 0; batch < n_entries; batch += MAX_ENTRIES) {
        const uint32_t n_batch = min(static_cast<uint32_t>(MAX_ENTRIES), n_entries - batch);
        wave_sync(); // done with the previous batch's tables

        fill_stencil_tables(sh, lane, centre + batch, n_batch, cx, cy, cz, span_y, span_z, g, cell_scan);

        const uint32_t n_candidates = __builtin_amdgcn_readfirstlane(sh.n_candidates);
        const uint32_t n_groups = (n_candidates + WAVE * R - 1) / (WAVE * R);
        const uint32_t per_slice = (n_groups + args.n_slices - 1) / args.n_slices;
        const uint32_t group_begin = slice * per_slice;
        const uint32_t group_end = min(n_groups, group_begin + per_slice);

        for (uint32_t group = group_begin; group < group_end; group++) {
            // ---- load R x 64 candidates into registers
            Candidates<R> c;
            c.any_shift = false;
            c.any_same = false;
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint32_t k = (group * R + r) * WAVE + lane;
                const bool valid = k < n_candidates;
                c.x[r] = c.y[r] = c.z[r] = __builtin_nan("");
                c.tx[r] = c.ty[r] = c.tz[r] = 0.0;
                c.bx[r] = c.by[r] = c.bz[r] = 0;
                c.position[r] = 0xFFFFFFFFu;
                bool same_cell = false;
                if (valid) {
                    uint32_t at;
                    int32_t packed;
                    locate_candidate(sh, n_batch, k, at, packed);
                    int32_t qx, qy, qz;
                    unpack_shift(packed, qx, qy, qz);
                    same_cell = (packed >> 30) & 1;
                    c.x[r] = pp[at].x;
                    c.y[r] = pp[at].y;
                    c.z[r] = pp[at].z;
                    c.bx[r] = qx - pwx[at];
                    c.by[r] = qy - pwy[at];
                    c.bz[r] = qz - pwz[at];
                    if (same_cell) {
                        c.position[r] = at;
                    }
                    if constexpr (WRITE) {
                        const int slot = r * WAVE + lane;
                        sh.cand_x[slot] = c.x[r];
                        sh.cand_y[slot] = c.y[r];
                        sh.cand_z[slot] = c.z[r];
                        sh.cand_index[slot] = pp[at].index;
                        sh.cand_bx[slot] = c.bx[r];
                        sh.cand_by[slot] = c.by[r];
                        sh.cand_bz[slot] = c.bz[r];
                    }
                }
                const bool shifted = (c.bx[r] | c.by[r] | c.bz[r]) != 0;
                c.any_shift = c.any_shift || (__ballot(shifted) != 0);
                c.any_same = c.any_same || (__ballot(same_cell) != 0);
            }
            if (c.any_shift) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    shift_vector(g, c.bx[r], c.by[r], c.bz[r], c.tx[r], c.ty[r], c.tz[r]);
                }
            }

            state.head = 0;
            state.tail = 0;
            if constexpr (WRITE) {
                wave_sync(); // candidate records are in LDS before any ticket is redeemed
            }

#define VESIN_SWEEP(SHIFTED, SAME)                                                                                    \
    sweep_unwrapped<WRITE, FULL, R, SHIFTED, SAME>(args.sorted, first_i, n_i, state, c, sh, args.out, g, ctx)
            if (ctx.tile_wrapped) {
                sweep_wrapped<WRITE, FULL, R>(args.sorted, first_i, n_i, state, c, sh, args.out, g, ctx);
            } else if (c.any_shift) {
                if (c.any_same) {
                    VESIN_SWEEP(true, true);
                } else {
                    VESIN_SWEEP(true, false);
                }
            } else {
                if (c.any_same) {
                    VESIN_SWEEP(false, true);
                } else {
                    VESIN_SWEEP(false, false);
                }
            }
#undef VESIN_SWEEP

            // the candidates leave the registers with this group: redeem what is left
            if constexpr (WRITE) {
                if (state.head != state.tail) {
                    redeem<FULL, R>(state.head - state.tail, state, c, sh, args.out, g, ctx);
                }
            }
        }
    }

    if (!WRITE && lane == 0) {
        // a full list gets two rows per hit: the pair and its mirror
        args.counts[row_slot] = FULL ? 2 * state.total : state.total;
    }
}

/// Four independent waves per workgroup, one work item each.
template <bool WRITE, bool FULL, int R>
__global__ __launch_bounds__(SEARCH_BLOCK) void search_kernel(SearchArgs args, GridParams g) {
    __shared__ std::conditional_t<WRITE, SearchSharedWrite, SearchSharedCount> shared[SEARCH_WAVES];
    const int lane = lane_id();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t n_tiles = static_cast<uint32_t>(args.cell_scan[g.n_cells] >> 32);
    const uint32_t work = blockIdx.x * SEARCH_WAVES + wave;
    if (WRITE && args.offsets[args.n_work] > args.capacity) {
        // launched before the host knew the number of rows, and they do not fit: the host grows the arrays and
        // launches again
        return;
    }
    if (work < args.n_work) {
        if (WRITE && args.only != nullptr && args.only[work] == 0) {
            return;
        }
        search_work_item<WRITE, FULL, R, false>(work, args, g, shared[wave], n_tiles, lane);
    }
}

/// The same search over the tiles of many systems: every tile brings its system's grid along.
template <bool WRITE, bool FULL, int R>
__global__ __launch_bounds__(SEARCH_BLOCK) void search_kernel_batch(SearchArgs args) {
    __shared__ std::conditional_t<WRITE, SearchSharedWrite, SearchSharedCount> shared[SEARCH_WAVES];
    const int lane = lane_id();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t n_tiles = static_cast<uint32_t>(args.cell_scan[args.total_cells] >> 32);
    const uint32_t work = blockIdx.x * SEARCH_WAVES + wave;
    if (work < args.n_work) {
        GridParams unused;
        search_work_item<WRITE, FULL, R, true>(work, args, unused, shared[wave], n_tiles, lane);
    }
}

} // namespace vesin_hip

#endif
