// Small systems (a few hundred to 2048 points): the whole calculation in ONE launch.
//
// At this size every pass of the other searches takes a few microseconds, most of them spent waiting for one memory
// access after the other, and the launches (cell build, counting pass, scan, report to the host, writing pass) with
// the gaps between dependent kernels cost several times what the passes do. Here one kernel does everything:
//
// * Every workgroup sorts ALL points into cells for itself, in LDS (the steps of build_cells_small: histogram with
//   the slot coming back from the atomic, scan, placement; the order inside a cell differs from workgroup to
//   workgroup, which no result depends on). From then on candidates are read from LDS.
// * One wave per work item. SORTED: an item is a point, in original order, with the candidates of its whole stencil
//   (the decisions of ordered_sweep_pair in ordered.cuh: every row (i, j, S) is found by the wave of i; a half list
//   keeps the smaller index first and a point's own image under the reference's rule). Otherwise an item is a point
//   and a slice of the candidates of the UPPER HALF of its stencil (the decisions of the single-pass search in
//   fused.cuh: every unordered pair is found once, a full list stores it with its mirror, a half list with the
//   smaller index first). The wave takes its candidates into registers, four units of 64 at a time with their
//   lookups interleaved, tests them with the arithmetic of the reference (vesin/src/cpu_cell_list.cpp:135-138,
//   vesin/src/types.hpp:232-243: S = cell shift - wrap_j + wrap_i, T = S . H left to right, v = (r_j - r_i) + T,
//   d2 = vx*vx + vy*vy + vz*vz, keep iff d2 < cutoff^2), keeps per candidate a hit bit, its place in LDS, original
//   index and shift, and stores the number of rows of its item.
// * All workgroups meet: they count themselves in one word and wait until all have. The grid (at most 240
//   workgroups, one or two per compute unit) is resident at once on a GPU that runs nothing else, and the wait is
//   bounded for the case that it is not: the first workgroup that stops waiting marks the word with a
//   compare-and-swap on a count that is not yet complete; a workgroup goes on iff it reads the complete count
//   without the mark, which cannot be set any more after that. So either all workgroups go on or none does; in the
//   second case workgroup 0 reports `gave_up` and the host goes on with the separate launches.
// * After the meeting every workgroup scans the rows of all items for itself (no second meeting), workgroup 0
//   reports to the host, and if the system suits the launch and the rows fit the arrays every wave writes the rows
//   of its item: ranked by (j, S) through write_rows_of_point (SORTED), or in the order of the candidates.
//
// What crosses from one workgroup to another is `rows_of_item` and the maxima of the meeting, all written and read
// with device-scope atomics (no cache-wide write-back or invalidation: those cost more than the passes).
// Limits, reported to the host, which then goes the general way: SORTED at most 256 rows and 1024 candidates per
// point; otherwise at most 1024 candidates per item; wraps and shifts within +-255; at most 64 stencil entries.
#ifndef VESIN_HIP_SMALL_CUH
#define VESIN_HIP_SMALL_CUH

#include "cells.cuh"
#include "ordered.cuh"

namespace vesin_hip {

constexpr uint32_t SMALL_POINTS = 2048;        // points (and cells, and work items) the largest shape takes
constexpr uint32_t SMALL_SPINS = 1u << 12;     // polls of a workgroup that waits for the others, at most
constexpr uint32_t SMALL_WAIT_TICKS = 50000;   // and the time it waits at most: 500 us of the 100 MHz clock, 25 times
                                               // what the whole launch takes when its workgroups run side by side
constexpr uint32_t SMALL_GAVE_UP = 1u << 31;   // in SmallMeeting::arrived: a workgroup stopped waiting
constexpr uint32_t SMALL_WORKGROUPS = 240;     // of a launch: fewer than there are compute units

/// Shapes of the launch: WAVES waves per workgroup, one work item each. Every workgroup holds all points, so the
/// grid must not have more workgroups than fit the GPU at once; few waves per workgroup spread the arithmetic over
/// more compute units, many allow more items.
template <int WAVES>
struct SmallShape {
    static constexpr int BLOCK_THREADS = WAVES * WAVE;
    static constexpr uint32_t PER_THREAD = WAVES == 16 ? 2 : 4;          // points (cells, items) a thread handles
    static constexpr uint32_t CAPACITY = PER_THREAD * BLOCK_THREADS;      // points, cells and items the LDS arrays hold
    static constexpr uint32_t MAX_ITEMS = WAVES == 16 ? CAPACITY : SMALL_WORKGROUPS * WAVES;
};
static_assert(SmallShape<16>::CAPACITY == SMALL_POINTS, "the largest shape takes every small system");
static_assert(SmallShape<16>::MAX_ITEMS <= SMALL_WORKGROUPS * 16, "a grid is at most SMALL_WORKGROUPS workgroups");

/// What the workgroups of one launch tell each other. A list keeps two of them and alternates: a launch works on
/// one and leaves the other cleared for the next launch.
struct SmallMeeting {
    unsigned int arrived;        // workgroups that are done counting (and SMALL_GAVE_UP)
    unsigned int max_rows;       // SORTED: most rows of a point
    unsigned int max_candidates; // most candidates of an item
    unsigned int unsuitable;     // items that met a wrap or shift outside of +-255
};

/// What the kernel takes besides the grid.
struct SmallArgs {
    const double* points;
    const double* box;           // null when the host has them already
    const bool* periodic;
    unsigned char* host_small;   // where the host reads box and periodic (see fetch_box)
    uint32_t* rows_of_item;      // [n_points * n_slices] work memory
    uint32_t n_slices;           // items per point (1 when SORTED)
    SmallMeeting* meeting;       // zero on entry
    SmallMeeting* next_meeting;  // cleared here
    OrderedHostStatus* host;
    BlockBounds* host_bounds;    // not null: workgroup 0 reports the extent of the points there (see bounding_kernel)
    uint32_t spin_limit;         // 0: no workgroup waits at all (tests)
    uint64_t capacity;
    SearchOutputs out;
};

/// LDS of one wave.
struct SmallWaveShared: SearchTables {
    __attribute__((aligned(16))) uint64_t keys[ORDERED_MAX_ROWS + 4];
    uint32_t key_at[ORDERED_MAX_ROWS];
};

/// LDS of a workgroup: its own cell-sorted copy of all points, and the waves' tables.
template <int WAVES>
struct SmallShared {
    static constexpr uint32_t CAPACITY = SmallShape<WAVES>::CAPACITY;
    double x[CAPACITY], y[CAPACITY], z[CAPACITY];
    uint32_t index[CAPACITY];
    uint32_t wraps[CAPACITY];          // biased_shift of the wrap, every component clamped to +-511
    uint32_t cell_start[CAPACITY + 1]; // points per cell, then their exclusive scan
    uint32_t first_row[CAPACITY + 1];  // after the meeting: exclusive scan of the rows of the items
    SmallWaveShared wave[WAVES];
    uint64_t wave_sums[WAVES];
    // the points of this workgroup's items, as the thread that placed them saw them
    double own_x[WAVES], own_y[WAVES], own_z[WAVES];
    uint32_t own_cell[WAVES];
    int32_t own_wx[WAVES], own_wy[WAVES], own_wz[WAVES];
    uint32_t first_bad;
    uint32_t all_arrived;
    BlockBounds extent[WAVES];   // workgroup 0: the waves' shares of the extent of the points
};

__device__ __forceinline__ double uniform(double v) {
    return __longlong_as_double(static_cast<long long>(uniform(static_cast<uint64_t>(__double_as_longlong(v)))));
}

/// Exclusive scan of one value per thread over the threads of a workgroup of WAVES waves; `total` for everybody.
template <int WAVES>
__device__ __forceinline__ uint64_t small_block_scan(uint64_t value, uint64_t& total, uint64_t* wave_sums) {
    const int lane = lane_id();
    const int wave = threadIdx.x / WAVE;
    const uint64_t inclusive = wave_inclusive_scan(value);
    if (lane == WAVE - 1) {
        wave_sums[wave] = inclusive;
    }
    __syncthreads();
    uint64_t before = 0;
    uint64_t all = 0;
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
        const uint64_t sum = wave_sums[w];
        before += w < wave ? sum : 0;
        all += sum;
    }
    __syncthreads();
    total = all;
    return before + inclusive - value;
}

/// locate_candidate for four candidates at once: the four searches advance together, one LDS round trip per step
/// for all of them instead of one per step and candidate.
__device__ __forceinline__ void locate_four_candidates(
    const SearchTables& sh, uint32_t n_batch, const uint32_t (&k)[4], uint32_t (&at)[4], int32_t (&packed)[4]
) {
    static_assert(MAX_ENTRIES <= 64, "six steps cover the table");
    uint32_t lo[4] = {0, 0, 0, 0};
#pragma unroll
    for (uint32_t step = 32; step > 0; step >>= 1) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            // largest e < n_batch with ent_prefix[e] <= k; the table has MAX_ENTRIES + 1 words, what lies beyond
            // n_batch is read and ignored
            const uint32_t probe = lo[r] + step;
            const uint32_t before = sh.ent_prefix[min(probe, static_cast<uint32_t>(MAX_ENTRIES))];
            const uint32_t take = (probe < n_batch ? 1u : 0u) & (before <= k[r] ? 1u : 0u); // no branch: the read is not skipped
            lo[r] = take != 0 ? probe : lo[r];
        }
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
        at[r] = sh.ent_start[lo[r]] + (k[r] - sh.ent_prefix[lo[r]]);
        packed[r] = sh.ent_shift[lo[r]];
    }
}

/// Rows of one point with the `n` candidates whose keys ((j << 32) | biased shift) and LDS places are in
/// `sh.keys` / `sh.key_at`, in that order, from row `cursor` on: the rows of redeem_fused (fused.cuh). A full list
/// stores the n pairs first, then their n mirrors; a half list stores every pair with the smaller index first (a
/// point's own image: the orientation the reference's rule keeps).
template <bool FULL>
__device__ __forceinline__ void write_unsorted_rows(
    const SmallWaveShared& sh, const double* xs, const double* ys, const double* zs, const GridParams& g,
    const SearchOutputs& out, uint32_t n, uint64_t cursor, double xi, double yi, double zi, uint32_t oi, int lane
) {
    double zero_tx, zero_ty, zero_tz;
    shift_vector(g, 0, 0, 0, zero_tx, zero_ty, zero_tz);
    for (uint32_t e0 = 0; e0 < n; e0 += WAVE) {
        const uint32_t e = e0 + lane;
        if (e < n) {
            const uint64_t key = sh.keys[e];
            const uint32_t at = sh.key_at[e];
            const double xj = xs[at];
            const double yj = ys[at];
            const double zj = zs[at];
            const uint32_t oj = static_cast<uint32_t>(key >> 32);
            const uint32_t biased = static_cast<uint32_t>(key);
            const int32_t sx = static_cast<int32_t>((biased >> 20) & 0x3ffu) - 512;
            const int32_t sy = static_cast<int32_t>((biased >> 10) & 0x3ffu) - 512;
            const int32_t sz = static_cast<int32_t>(biased & 0x3ffu) - 512;
            double tx, ty, tz;
            shift_vector(g, sx, sy, sz, tx, ty, tz);
            const bool shifted = (sx | sy | sz) != 0;
            const double mx = shifted ? -tx : zero_tx;
            const double my = shifted ? -ty : zero_ty;
            const double mz = shifted ? -tz : zero_tz;
            const double vx = (xj - xi) + tx;
            const double vy = (yj - yi) + ty;
            const double vz = (zj - zi) + tz;
            const double wx = (xi - xj) + mx;
            const double wy = (yi - yj) + my;
            const double wz = (zi - zj) + mz;
            const double d2 = vx * vx + vy * vy + vz * vz;
            if (FULL) {
                const uint64_t forward_row = cursor + e;
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
            } else {
                const bool flip = oi > oj || (oi == oj && !half_keeps_self_image(sx, sy, sz));
                const uint64_t row = cursor + e;
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
        }
    }
}

/// See the head of the file. Launch: ceil(n_points * n_slices / WAVES) workgroups of WAVES waves, at most
/// SmallShape<WAVES>::MAX_ITEMS items and ::CAPACITY points and cells.
template <bool FULL, int WAVES, bool SORTED>
__global__ __launch_bounds__(WAVES * WAVE) void small_system_kernel(SmallArgs args, GridParams g) {
    constexpr uint32_t BLOCK_THREADS = SmallShape<WAVES>::BLOCK_THREADS;
    constexpr uint32_t PER_THREAD = SmallShape<WAVES>::PER_THREAD;
    constexpr uint32_t CAPACITY = SmallShape<WAVES>::CAPACITY;
    __shared__ SmallShared<WAVES> shared;
    static_assert(sizeof(SmallShared<WAVES>) <= 160 * 1024, "a workgroup's LDS");
    static_assert(ORDERED_UNITS % 4 == 0, "units are taken four at a time");
    const uint32_t t = threadIdx.x;
    const int lane = lane_id();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(t / WAVE);
    SmallWaveShared& sh = shared.wave[wave];
    const uint32_t n = g.n_points;
    const uint32_t n_slices = SORTED ? 1u : args.n_slices;
    const uint32_t n_items = n * n_slices;
    const uint32_t first_item = blockIdx.x * WAVES;

    // ---- the cell list, in LDS
    if (blockIdx.x == 0 && args.box != nullptr) {
        if (t < 9) {
            reinterpret_cast<double*>(args.host_small)[t] = args.box[t];
        } else if (t < 12) {
            args.host_small[72 + (t - 9)] = args.periodic[t - 9] ? 1 : 0;
        }
    }
    if (t == 0) {
        shared.first_bad = 0xFFFFFFFFu;
    }
#pragma unroll
    for (uint32_t k = 0; k < PER_THREAD; k++) {
        shared.cell_start[k * BLOCK_THREADS + t] = 0;
    }
    __syncthreads();
    double px[PER_THREAD], py[PER_THREAD], pz[PER_THREAD];
    uint32_t cell_of[PER_THREAD], slot_of[PER_THREAD];
    int32_t pwx[PER_THREAD], pwy[PER_THREAD], pwz[PER_THREAD];
    const bool report_extent = args.host_bounds != nullptr && blockIdx.x == 0;
    double extent_lo[3] = {INFINITY, INFINITY, INFINITY};
    double extent_hi[3] = {-INFINITY, -INFINITY, -INFINITY};
#pragma unroll
    for (uint32_t k = 0; k < PER_THREAD; k++) {
        const uint32_t i = k * BLOCK_THREADS + t;
        cell_of[k] = 0;
        slot_of[k] = 0;
        pwx[k] = pwy[k] = pwz[k] = 0;
        px[k] = py[k] = pz[k] = 0.0;
        if (i < n) {
            px[k] = args.points[3 * static_cast<size_t>(i) + 0];
            py[k] = args.points[3 * static_cast<size_t>(i) + 1];
            pz[k] = args.points[3 * static_cast<size_t>(i) + 2];
            int32_t where[3] = {0, 0, 0};
            int32_t wrap[3] = {0, 0, 0};
            unsigned int axis;
            if (all_finite(px[k], py[k], pz[k], axis)) {
                locate(g, px[k], py[k], pz[k], where, wrap);
                if (report_extent) {
                    double f[3];
                    fractional(g, px[k], py[k], pz[k], f);
#pragma unroll
                    for (int d = 0; d < 3; d++) {
                        extent_lo[d] = fmin(extent_lo[d], f[d]);
                        extent_hi[d] = fmax(extent_hi[d], f[d]);
                    }
                }
            } else {
                atomicMin(&shared.first_bad, 3u * i + axis);
            }
            cell_of[k] = (static_cast<uint32_t>(where[2]) * g.n[1] + where[1]) * g.n[0] + where[0];
            pwx[k] = wrap[0];
            pwy[k] = wrap[1];
            pwz[k] = wrap[2];
            slot_of[k] = atomicAdd(&shared.cell_start[cell_of[k]], 1u);
            // the items of this workgroup that belong to point i
            const uint32_t begin = max(i * n_slices, first_item);
            const uint32_t end = min((i + 1) * n_slices, first_item + WAVES);
            for (uint32_t item = begin; item < end; item++) {
                const uint32_t w = item - first_item;
                shared.own_x[w] = px[k];
                shared.own_y[w] = py[k];
                shared.own_z[w] = pz[k];
                shared.own_cell[w] = cell_of[k];
                shared.own_wx[w] = pwx[k];
                shared.own_wy[w] = pwy[k];
                shared.own_wz[w] = pwz[k];
            }
        }
    }
    if (report_extent) {
        // the extent of the points, for the grid of the next call on this list (a list remembers it like its box)
#pragma unroll
        for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
#pragma unroll
            for (int d = 0; d < 3; d++) {
                extent_lo[d] = fmin(extent_lo[d], __shfl_xor(extent_lo[d], offset));
                extent_hi[d] = fmax(extent_hi[d], __shfl_xor(extent_hi[d], offset));
            }
        }
        if (lane == 0) {
#pragma unroll
            for (int d = 0; d < 3; d++) {
                shared.extent[wave].lo[d] = extent_lo[d];
                shared.extent[wave].hi[d] = extent_hi[d];
            }
        }
    }
    __syncthreads();
    if (report_extent && t == 0) {
        BlockBounds all = shared.extent[0];
        for (int w = 1; w < WAVES; w++) {
#pragma unroll
            for (int d = 0; d < 3; d++) {
                all.lo[d] = fmin(all.lo[d], shared.extent[w].lo[d]);
                all.hi[d] = fmax(all.hi[d], shared.extent[w].hi[d]);
            }
        }
        all.first_bad_coordinate = 0xFFFFFFFFu; // reported with the rest, below
        all.padding = 0;
        args.host_bounds[0] = all;
    }
    {
        uint32_t counts[PER_THREAD];
        uint64_t own_total = 0;
#pragma unroll
        for (uint32_t k = 0; k < PER_THREAD; k++) {
            const uint32_t c = t * PER_THREAD + k;
            counts[k] = c < g.n_cells ? shared.cell_start[c] : 0u;
            own_total += counts[k];
        }
        uint64_t total_points = 0;
        uint32_t running = static_cast<uint32_t>(small_block_scan<WAVES>(own_total, total_points, shared.wave_sums));
#pragma unroll
        for (uint32_t k = 0; k < PER_THREAD; k++) {
            shared.cell_start[t * PER_THREAD + k] = running;
            running += counts[k];
        }
        if (t == BLOCK_THREADS - 1) {
            shared.cell_start[CAPACITY] = running;
        }
    }
    __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < PER_THREAD; k++) {
        const uint32_t i = k * BLOCK_THREADS + t;
        if (i < n) {
            const uint32_t to = shared.cell_start[cell_of[k]] + slot_of[k];
            shared.x[to] = px[k];
            shared.y[to] = py[k];
            shared.z[to] = pz[k];
            shared.index[to] = i;
            shared.wraps[to] = biased_shift(max(-511, min(511, pwx[k])), max(-511, min(511, pwy[k])), max(-511, min(511, pwz[k])));
        }
    }
    __syncthreads();

    // ---- the candidates of this wave's item, its rows
    const uint32_t item = first_item + wave;
    const uint32_t oi = item / n_slices;
    const uint32_t slice = item - oi * n_slices;
    uint32_t columns[ORDERED_UNITS];
    uint32_t cand_at[ORDERED_UNITS];
    uint32_t cand_index[ORDERED_UNITS];
    uint32_t cand_biased[ORDERED_UNITS];
#pragma unroll
    for (int u = 0; u < ORDERED_UNITS; u++) {
        columns[u] = 0;
        cand_at[u] = 0;
        cand_index[u] = 0;
        cand_biased[u] = 0;
    }
    uint32_t n_units = 0;
    uint32_t hits = 0;
    double xi = 0.0, yi = 0.0, zi = 0.0;
    int32_t wix = 0, wiy = 0, wiz = 0;
    const int32_t span_y = 2 * g.s[1] + 1;
    const int32_t span_z = 2 * g.s[2] + 1;
    const uint32_t n_stencil = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z;
    // SORTED: the whole stencil; otherwise the centre cell and what follows it
    const uint32_t first_entry = SORTED ? 0u : n_stencil / 2;
    const uint32_t n_entries = n_stencil - first_entry;
    if (item < n_items && n_entries <= MAX_ENTRIES) {
        xi = uniform(shared.own_x[wave]);
        yi = uniform(shared.own_y[wave]);
        zi = uniform(shared.own_z[wave]);
        wix = static_cast<int32_t>(uniform(static_cast<uint32_t>(shared.own_wx[wave])));
        wiy = static_cast<int32_t>(uniform(static_cast<uint32_t>(shared.own_wy[wave])));
        wiz = static_cast<int32_t>(uniform(static_cast<uint32_t>(shared.own_wz[wave])));
        const uint32_t cell = uniform(shared.own_cell[wave]);
        const int32_t cx = cell % g.n[0];
        const int32_t cy = (cell / g.n[0]) % g.n[1];
        const int32_t cz = cell / (g.n[0] * g.n[1]);
        fill_stencil_tables(sh, lane, first_entry, n_entries, cx, cy, cz, span_y, span_z, g, shared.cell_start);
        const uint32_t n_candidates = __builtin_amdgcn_readfirstlane(sh.n_candidates);
        // This item's share of the candidates: whole stencil entries, cut where the running number of candidates
        // first reaches slice / n_slices of all of them. The slices of a point may be in different workgroups,
        // whose copies of the points differ in the order inside a cell: which points an entry holds is the same
        // for all of them, where in the entry a point sits is not.
        uint32_t k_begin = 0;
        uint32_t k_end = n_candidates;
        if (!SORTED) {
            const uint32_t lower = static_cast<uint32_t>(static_cast<uint64_t>(slice) * n_candidates / n_slices);
            const uint32_t upper = static_cast<uint32_t>(static_cast<uint64_t>(slice + 1) * n_candidates / n_slices);
            // first entry whose candidates start at or after the mark (lane e looks at entry e; none: the end)
            const uint32_t starts = static_cast<uint32_t>(lane) < n_entries ? sh.ent_prefix[lane] : n_candidates;
            const uint64_t from_lower = __ballot(starts >= lower);
            const uint64_t from_upper = __ballot(starts >= upper);
            k_begin = uniform(sh.ent_prefix[from_lower != 0 ? __ffsll(static_cast<unsigned long long>(from_lower)) - 1 : n_entries]);
            k_end = slice + 1 == n_slices
                        ? n_candidates
                        : uniform(sh.ent_prefix[from_upper != 0 ? __ffsll(static_cast<unsigned long long>(from_upper)) - 1 : n_entries]);
        }
        const uint32_t item_candidates = k_end - k_begin;
        if (lane == 0 && item_candidates > __hip_atomic_load(&args.meeting->max_candidates, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
            atomicMax(&args.meeting->max_candidates, item_candidates);
        }
        if (item_candidates <= ORDERED_CANDIDATES) {
            n_units = (item_candidates + WAVE - 1) / WAVE;
            bool out_of_range = beyond(wix, wiy, wiz, ORDERED_SHIFT_LIMIT);
#pragma unroll
            for (int chunk = 0; chunk < ORDERED_UNITS / 4; chunk++) {
                if (static_cast<uint32_t>(4 * chunk) < n_units) {
                    uint32_t k[4], at[4];
                    int32_t packed_q[4];
                    bool valid[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        k[r] = k_begin + static_cast<uint32_t>(4 * chunk + r) * WAVE + lane;
                        valid[r] = k[r] < k_end;
                        k[r] = valid[r] ? k[r] : 0u; // candidate 0 exists: every read below has an address
                    }
                    locate_four_candidates(sh, n_entries, k, at, packed_q);
                    double xj[4], yj[4], zj[4];
                    uint32_t oj[4], wj[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        xj[r] = shared.x[at[r]];
                        yj[r] = shared.y[at[r]];
                        zj[r] = shared.z[at[r]];
                        oj[r] = shared.index[at[r]];
                        wj[r] = shared.wraps[at[r]];
                    }
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int u = 4 * chunk + r;
                        int32_t qx, qy, qz;
                        unpack_shift(packed_q[r], qx, qy, qz);
                        const int32_t bx = qx - (static_cast<int32_t>((wj[r] >> 20) & 0x3ffu) - 512);
                        const int32_t by = qy - (static_cast<int32_t>((wj[r] >> 10) & 0x3ffu) - 512);
                        const int32_t bz = qz - (static_cast<int32_t>(wj[r] & 0x3ffu) - 512);
                        out_of_range = out_of_range || (valid[r] && beyond(bx, by, bz, ORDERED_SHIFT_LIMIT));
                        const int32_t sx = bx + wix;
                        const int32_t sy = by + wiy;
                        const int32_t sz = bz + wiz;
                        double tx, ty, tz;
                        shift_vector(g, sx, sy, sz, tx, ty, tz);
                        const double vx = (xj[r] - xi) + tx;
                        const double vy = (yj[r] - yi) + ty;
                        const double vz = (zj[r] - zi) + tz;
                        const double d2 = vx * vx + vy * vy + vz * vz;
                        bool keep;
                        if (SORTED) {
                            const bool shifted = (sx | sy | sz) != 0;
                            if (oj[r] == oi) {
                                // the point and one of its own images
                                keep = shifted && (FULL || half_keeps_self_image(sx, sy, sz));
                            } else {
                                keep = FULL || oi < oj[r];
                            }
                        } else {
                            // the point's own cell without a cell shift: every pair of its points once (and no
                            // point with itself); every other entry is somebody's upper half only once
                            const bool same_cell = ((packed_q[r] >> 30) & 1) != 0;
                            keep = !same_cell || oi < oj[r];
                        }
                        const bool hit = valid[r] && keep && d2 < g.cutoff2;
                        hits += __popcll(__ballot(hit));
                        columns[u] = hit ? 1u : 0u;
                        cand_at[u] = at[r];
                        cand_index[u] = oj[r];
                        // (a clamped wrap gives a wrong shift here: such a system is reported unsuitable)
                        cand_biased[u] = biased_shift(max(-511, min(511, bx)), max(-511, min(511, by)), max(-511, min(511, bz)));
                    }
                }
            }
            if (SORTED && lane == 0 && hits > __hip_atomic_load(&args.meeting->max_rows, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                atomicMax(&args.meeting->max_rows, hits);
            }
            if (__ballot(out_of_range) != 0 && lane == 0) {
                atomicAdd(&args.meeting->unsuitable, 1u);
            }
        }
    }
    const uint32_t rows = (!SORTED && FULL) ? 2 * hits : hits;
    if (item < n_items && lane == 0) {
        // read by other workgroups of this launch: straight to where the whole device sees it
        __hip_atomic_store(&args.rows_of_item[item], rows, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- all workgroups meet. Once a wave's device-scope stores have completed they are what any device-scope
    // load returns, so the workgroup's arrival only has to come after. This leans on two properties of this
    // architecture (gfx9 family, gfx950 included) instead of release / acquire orderings, whose cache-wide write-back
    // and invalidation doubled the launch's time when tried: vmcnt counts stores as well as loads, so vmcnt(0) means
    // that every store this wave issued has been acknowledged by the L2 cache, and device-scope atomic stores and loads
    // go to that cache, which all compute units of the device share.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (t == 0) {
        if (args.spin_limit == 0) {
            // no patience at all (how the tests reach the host's way back): marked before anybody can be the last
            __hip_atomic_fetch_or(&args.meeting->arrived, SMALL_GAVE_UP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __hip_atomic_fetch_add(&args.meeting->arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t spins = 0;
        bool all = false;
        const uint64_t since = wall_clock64();
        while (true) {
            uint32_t seen = __hip_atomic_load(&args.meeting->arrived, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((seen & SMALL_GAVE_UP) != 0) {
                break;
            }
            if (seen == gridDim.x) {
                all = true;
                break;
            }
            spins += 1;
            if (spins > args.spin_limit || wall_clock64() - since > SMALL_WAIT_TICKS) {
                if (__hip_atomic_compare_exchange_strong(
                        &args.meeting->arrived, &seen, seen | SMALL_GAVE_UP, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                        __HIP_MEMORY_SCOPE_AGENT
                    )) {
                    break;
                }
                continue; // somebody arrived or gave up in between: look again
            }
            __builtin_amdgcn_s_sleep(4);
        }
        shared.all_arrived = all ? 1u : 0u;
        if (blockIdx.x == 0) {
            // nobody looks at the other meeting during this launch: the next launch finds it cleared
            __hip_atomic_store(&args.next_meeting->arrived, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&args.next_meeting->max_rows, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&args.next_meeting->max_candidates, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&args.next_meeting->unsuitable, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __syncthreads();
    if (shared.all_arrived == 0) {
        if (blockIdx.x == 0 && t == 0) {
            args.host->found.gave_up = 1;
            args.host->first_bad_coordinate = shared.first_bad;
        }
        return;
    }

    // ---- the first row of every item: every workgroup scans the rows of all items
    {
        uint32_t rows_of[PER_THREAD];
        uint64_t local = 0;
#pragma unroll
        for (uint32_t k = 0; k < PER_THREAD; k++) {
            const uint32_t i = t * PER_THREAD + k;
            rows_of[k] = i < n_items ? __hip_atomic_load(&args.rows_of_item[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
            local += rows_of[k];
        }
        uint64_t total = 0;
        uint32_t running = static_cast<uint32_t>(small_block_scan<WAVES>(local, total, shared.wave_sums));
#pragma unroll
        for (uint32_t k = 0; k < PER_THREAD; k++) {
            shared.first_row[t * PER_THREAD + k] = running;
            running += rows_of[k];
        }
        if (t == BLOCK_THREADS - 1) {
            shared.first_row[CAPACITY] = running;
        }
    }
    __syncthreads();
    const uint64_t total = shared.first_row[CAPACITY];
    OrderedStatus found;
    found.max_rows = __hip_atomic_load(&args.meeting->max_rows, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    found.max_candidates = __hip_atomic_load(&args.meeting->max_candidates, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    found.unsuitable = __hip_atomic_load(&args.meeting->unsuitable, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    found.windowed = 0;
    found.bucketed = 0;
    found.arrived = gridDim.x;
    found.gave_up = 0;
    found.padding = 0;
    const bool suitable = found.max_rows <= ORDERED_MAX_ROWS && found.max_candidates <= ORDERED_CANDIDATES &&
                          found.unsuitable == 0 && shared.first_bad == 0xFFFFFFFFu;
    if (blockIdx.x == 0 && t == 0) {
        args.host->found = found;
        args.host->total_rows = total;
        args.host->first_bad_coordinate = shared.first_bad;
    }
    if (!suitable || total > args.capacity || hits == 0) {
        return;
    }

    // ---- the rows of the item
    const uint32_t wrap_i = (static_cast<uint32_t>(wix) << 20) + (static_cast<uint32_t>(wiy) << 10) + static_cast<uint32_t>(wiz);
    if (SORTED) {
        write_rows_of_point<false>(
            sh, PointsByPlace{shared.x, shared.y, shared.z}, g, args.out, columns, cand_at, cand_index, cand_biased, n_units, 0u, wrap_i, xi, yi, zi, oi,
            static_cast<uint64_t>(shared.first_row[item]), lane
        );
    } else {
        uint64_t cursor = shared.first_row[item];
#pragma unroll
        for (int chunk = 0; chunk < ORDERED_UNITS / 4; chunk++) {
            if (static_cast<uint32_t>(4 * chunk) < n_units) {
                // the hits of four units, in the order of the candidates: at most 256
                uint32_t n_rows = 0;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int u = 4 * chunk + r;
                    const bool hit = columns[u] != 0;
                    const uint64_t mask = __ballot(hit);
                    if (hit) {
                        const uint32_t slot = n_rows + rank_in_mask(mask);
                        sh.keys[slot] = (static_cast<uint64_t>(cand_index[u]) << 32) | (cand_biased[u] + wrap_i);
                        sh.key_at[slot] = cand_at[u];
                    }
                    n_rows += __popcll(mask);
                }
                if (n_rows != 0) {
                    wave_sync();
                    write_unsorted_rows<FULL>(sh, shared.x, shared.y, shared.z, g, args.out, n_rows, cursor, xi, yi, zi, oi, lane);
                    cursor += FULL ? 2 * n_rows : n_rows;
                    wave_sync(); // the keys are about to be overwritten by the next units'
                }
            }
        }
    }
}

} // namespace vesin_hip

#endif
