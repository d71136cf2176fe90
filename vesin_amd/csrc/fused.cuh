// Single-pass stencil search: count, place and write the rows of every tile in one kernel.
//
// The two-pass search (search.cuh) evaluates every candidate pair twice, once to count and once to write, with a
// device-wide scan between the two launches. Here a wave keeps the outcome of its tests instead: while it sweeps the
// tile's points over 64 candidates held in registers, every candidate lane shifts the hit bit of each tile point into
// a 32-bit column (one v_addc per test, fed by the compare's lane mask; a tile has at most 32 points). After the sweep the wave knows its number of
// rows; the four waves of a workgroup add theirs up and the workgroup takes its place in the output: with one atomic
// on the running total (rows in order of arrival), or, for an order that is the same on every run, by chaining with
// the earlier workgroups (64-bit words holding a flag and a value, written and polled with device-scope atomics;
// decoupled look-back over groups of workgroups).
// The wave finally replays its columns: each round every lane with hits left peels one bit off its column and drops
// a ticket (candidate slot, tile point) into the wave's LDS ring; whenever 64 tickets are pending all lanes redeem
// one each, exactly like the write pass of the two-pass search, and store dense rows.
//
// The leader of a group (its last workgroup) waits for workgroups with a smaller index; the other workgroups of a
// group wait for the word their leader publishes, i.e. for a workgroup with a larger index. The chain therefore
// advances only as long as the hardware starts workgroups in index order and a group's leader gets a wave slot while
// its members wait, which a grid of this shape has always done here but which nothing guarantees. Every wait is
// bounded for that reason, in time (CHAIN_WAIT_TICKS of the 100 MHz clock, 2 ms) and not in polls, whose duration
// depends on what else the GPU is doing: a wave that runs out of patience raises a flag and goes on with whatever it
// has (it writes nothing), every wave that polls afterwards sees the flag and gives up at once, so a launch whose
// chain is stuck ends a few milliseconds after the first wave lost patience, and the host starts the call over with
// the two-pass search and leaves the chain alone for a while (see Rest, policy.hpp).
//
// A work item with more than FUSED_UNITS x 64 candidates cannot keep its columns: it is swept and counted here, its
// rows are placed by the chain like all others, and its first row goes to `offsets` with a mark in `counts`; the
// host then launches the write pass of the two-pass search for the marked work items only.
//
// This kernel covers the common shape of the problem: at most MAX_ENTRIES stencil entries, shifts that fit the
// 10-bit packing. A work item outside of that shape raises the `general` count and produces nothing; the host then
// runs the two-pass search for the whole call.
//
// Arithmetic and row conventions are those of search.cuh.
#ifndef VESIN_HIP_FUSED_CUH
#define VESIN_HIP_FUSED_CUH

#include "search.cuh"

namespace vesin_hip {

constexpr int FUSED_UNITS = 32;         // 64-candidate units of one work item whose columns stay in registers
constexpr int FUSED_SLOTS = 2 * WAVE;   // candidate records in LDS: two units, so that tickets survive a unit change
constexpr int32_t PACKED_SHIFT_LIMIT = 500;
constexpr uint32_t CHAIN_SPIN_LIMIT = 1u << 18; // polls a wave makes at most before it gives up (FusedArgs::spin_limit)
constexpr uint32_t CHAIN_WAIT_TICKS = 200000;   // and how long it waits at most: 2 ms of the 100 MHz clock
constexpr uint32_t CHAIN_GROUP = 32;    // workgroups per group of the chain (at most 64)

constexpr uint64_t CHAIN_FLAG_SHIFT = 62;
constexpr uint64_t CHAIN_AGGREGATE = 1ull << CHAIN_FLAG_SHIFT; // value = rows of this workgroup
constexpr uint64_t CHAIN_PREFIX = 2ull << CHAIN_FLAG_SHIFT;    // value = rows of this and all earlier workgroups
constexpr uint64_t CHAIN_VALUE = (1ull << CHAIN_FLAG_SHIFT) - 1;
constexpr uint64_t CHAIN_GAVE_UP = ~0ull; // chain_position: the wave ran out of patience, its place is not known

/// The words through which the workgroups learn where their rows start; all zero on entry.
struct Chain {
    uint64_t* blocks; // [workgroups]: flag | rows of the workgroup
    uint64_t* groups; // [groups]: flag | rows of the group, later of all groups up to this one
    uint64_t* bases;  // [groups]: flag | rows of all earlier groups
};

struct FusedArgs {
    SearchArgs search;
    uint64_t* first_rows; // [work items]: first output row of the work items left to the write pass
    Chain chain;
    FusedStatus* status; // zero on entry
    uint32_t spin_limit; // polls of the chain before a wave gives up; 0 makes every wait fail at once (tests)
    uint32_t wait_ticks; // and the time it waits at most, in ticks of the 100 MHz clock
};

/// LDS of one wave. STAGED: with room to line up the vectors of 64 rows on their way to memory (the kernels of calls
/// that return vectors; the others keep the LDS, and the code, they had without it).
template <bool STAGED>
struct FusedWaveShared: SearchTables {
    double tile_x[TILE_POINTS], tile_y[TILE_POINTS], tile_z[TILE_POINTS];
    uint32_t tile_index[TILE_POINTS];
    int32_t tile_wx[TILE_POINTS], tile_wy[TILE_POINTS], tile_wz[TILE_POINTS];
    double cand_x[FUSED_SLOTS], cand_y[FUSED_SLOTS], cand_z[FUSED_SLOTS];
    uint32_t cand_index[FUSED_SLOTS];
    int32_t cand_shift[FUSED_SLOTS]; // packed: cell shift minus the candidate's own wrap shift
    uint16_t ring[RING];
    __attribute__((aligned(16))) double vector_stage[STAGED ? 3 * WAVE : 2];
};

template <bool STAGED>
struct FusedShared {
    FusedWaveShared<STAGED> wave[SEARCH_WAVES];
    uint32_t rows[SEARCH_WAVES];
    uint64_t base;     // first output row of the workgroup
    uint32_t writable; // the workgroup's rows fit the output arrays
};

/// col = 2 * col + (this lane's bit of mask): one VALU instruction, the mask is the carry-in.
__device__ __forceinline__ uint32_t shift_in(uint32_t col, uint64_t mask) {
    uint32_t result;
    uint64_t carry_out;
    asm("v_addc_co_u32_e64 %0, %1, %2, %2, %3" : "=v"(result), "=s"(carry_out) : "v"(col), "s"(mask));
    return result;
}

/// One candidate per lane: where it is, what it is shifted by.
struct UnitCandidates {
    uint32_t at;     // position in the cell-sorted arrays (valid lanes)
    int32_t bx, by, bz;
    bool valid;
    bool same_cell;  // from the tile's own cell with a zero cell shift
};

__device__ __forceinline__ UnitCandidates locate_unit(
    const SearchTables& sh, uint32_t n_batch, uint32_t n_candidates, uint32_t k, const SortedPoints& sorted
) {
    UnitCandidates u;
    u.valid = k < n_candidates;
    u.at = 0;
    u.bx = u.by = u.bz = 0;
    u.same_cell = false;
    if (u.valid) {
        int32_t packed;
        locate_candidate(sh, n_batch, k, u.at, packed);
        int32_t qx, qy, qz;
        unpack_shift(packed, qx, qy, qz);
        u.same_cell = (packed >> 30) & 1;
        u.bx = qx - sorted.wx[u.at];
        u.by = qy - sorted.wy[u.at];
        u.bz = qz - sorted.wz[u.at];
    }
    return u;
}

/// Registers of the sweep: R x 64 candidates.
template <int R>
struct SweepCandidates {
    double x[R], y[R], z[R];
    double tx[R], ty[R], tz[R];
    int32_t shift[R];      // packed
    uint32_t position[R];  // see Candidates::position
};

static_assert(TILE_POINTS <= 32, "the hit column of a candidate is one 32-bit register");

/// The tile's points (from cell-sorted position `first`) against the R x 64 candidates; every candidate lane
/// shifts its hit bits into `column` (the first point ends up in the highest bit used). Returns the number of hits.
template <int R, bool SHIFTED, bool SAME>
__device__ __forceinline__ uint32_t sweep_columns(
    const SortedPoints& sorted, uint32_t first, uint32_t count, const SweepCandidates<R>& c, double cutoff2,
    uint32_t (&column)[R]
) {
    uint32_t total = 0;
    for (uint32_t i0 = 0; i0 < count; i0 += POINTS_PER_LOAD) {
        const uint32_t at = first + i0;
        const FourPoints p = load_four_points(sorted.p + at);
#pragma unroll
        for (int u = 0; u < POINTS_PER_LOAD; u++) {
            if (u > 0 && i0 + u >= count) {
                break;
            }
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
                uint64_t mask = __ballot(d2 < cutoff2);
                if (SAME) {
                    mask &= __ballot(c.position[r] > at + u);
                }
                total += __popcll(mask);
                column[r] = shift_in(column[r], mask);
            }
        }
    }
    return total;
}

/// Variant for a tile holding points that were wrapped into the box: the shift of a pair depends on both points.
/// Only the wrapped points of the tile (usually a few) pay for it: against a point that was not moved the shift is
/// the candidate's own, whose vector `c.tx/ty/tz` holds (zero for a candidate without shift).
template <int R>
__device__ __forceinline__ uint32_t sweep_columns_wrapped(
    const SortedPoints& sorted, uint32_t first_i, uint32_t n_i, const SweepCandidates<R>& c, const GridParams& g,
    uint32_t (&column)[R]
) {
    uint32_t total = 0;
    for (uint32_t i0 = 0; i0 < n_i; i0 += POINTS_PER_LOAD) {
        // coordinates and wraps of four points come in through scalar loads, like in sweep_columns
        const uint32_t at0 = first_i + i0;
        const FourPoints p = load_four_points(sorted.p + at0);
        const FourWraps w = load_four_wraps(sorted.wx + at0, sorted.wy + at0, sorted.wz + at0);
#pragma unroll
        for (int u = 0; u < POINTS_PER_LOAD; u++) {
            if (u > 0 && i0 + u >= n_i) {
                break;
            }
            const uint32_t at = at0 + u;
            const double xi = words_to_double(p.q[u][0], p.q[u][1]);
            const double yi = words_to_double(p.q[u][2], p.q[u][3]);
            const double zi = words_to_double(p.q[u][4], p.q[u][5]);
            const int32_t wix = static_cast<int32_t>(w.x[u]);
            const int32_t wiy = static_cast<int32_t>(w.y[u]);
            const int32_t wiz = static_cast<int32_t>(w.z[u]);
            const bool moved = (wix | wiy | wiz) != 0;
#pragma unroll
            for (int r = 0; r < R; r++) {
                double tx = c.tx[r];
                double ty = c.ty[r];
                double tz = c.tz[r];
                if (moved) {
                    int32_t bx, by, bz;
                    unpack_shift(c.shift[r], bx, by, bz);
                    shift_vector(g, bx + wix, by + wiy, bz + wiz, tx, ty, tz);
                }
                const double vx = (c.x[r] - xi) + tx;
                const double vy = (c.y[r] - yi) + ty;
                const double vz = (c.z[r] - zi) + tz;
                const double d2 = vx * vx + vy * vy + vz * vz;
                const uint64_t mask = __ballot(d2 < g.cutoff2) & __ballot(c.position[r] > at);
                total += __popcll(mask);
                column[r] = shift_in(column[r], mask);
            }
        }
    }
    return total;
}

/// The vectors of n <= 64 consecutive rows (lane l holds row l) go to memory as 16-byte pieces of consecutive
/// addresses, one piece per lane and store instruction, after they were lined up in the wave's LDS. Stored row by row
/// instead (16 + 8 bytes per lane, 24 bytes apart), every store instruction leaves holes in the cache lines it
/// touches for the next one to fill, and rows with vectors reached 3.0 TB/s where rows without reach 4.5.
__device__ __forceinline__ void store_vector_rows(
    double* stage, char* rows, uint32_t n, bool active, uint32_t lane, double x, double y, double z
) {
    // (the lanes of a wave read what other lanes wrote: the LDS serves a wave's accesses in the order they were
    // issued, which a fence of wavefront scope tells the compiler to keep; nothing waits for the row stores in flight)
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (active) {
        stage[3 * lane + 0] = x;
        stage[3 * lane + 1] = y;
        stage[3 * lane + 2] = z;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const uint32_t bytes = n * 24u;
    if (lane * 16u + 16u <= bytes) {
        stream_store(rows + lane * 16u, VectorHead{stage[2 * lane], stage[2 * lane + 1]});
    }
    if (1024u + lane * 16u + 16u <= bytes) {
        stream_store(rows + 1024u + lane * 16u, VectorHead{stage[2 * WAVE + 2 * lane], stage[2 * WAVE + 2 * lane + 1]});
    }
    if ((n & 1u) != 0 && lane == 0) {
        // an odd number of rows ends with half a piece
        stream_store(rows + bytes - 8u, stage[3 * n - 1]);
    }
}

/// Constants of the replay phase of one work item.
struct ReplayContext {
    double zero_tx, zero_ty, zero_tz;
    bool need_shift;   // some candidate of the work item has a non-zero shift, or the tile holds wrapped points
    bool tile_wrapped;
    int lane;
    uint32_t last;     // tile point of bit 0 of a column: n_i - 1
};

struct ReplayState {
    uint64_t out_cursor;
    uint32_t head;
    uint32_t tail;
    uint32_t batch; // tickets the next redeem takes: 64, or fewer to bring the cursor to a multiple of ROW_ALIGN
};

/// Redeem n <= 64 tickets: same rows as `redeem` of the two-pass search, candidates and tile points read from LDS.
template <bool FULL, bool STAGED>
__device__ __forceinline__ void redeem_fused(
    uint32_t n, ReplayState& state, FusedWaveShared<STAGED>& sh, const SearchOutputs& out, const GridParams& g,
    const ReplayContext& ctx
) {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int lane = ctx.lane;
    const bool active = static_cast<uint32_t>(lane) < n;
    const uint32_t ticket = sh.ring[(state.tail + lane) & (RING - 1)];
    // ticket: candidate record (7 bits), bit of the column (5 bits, from bit 8); the tile's first point sits in the
    // highest bit used
    const int slot = active ? ticket & (FUSED_SLOTS - 1) : 0;
    const uint32_t bit = (ticket >> 8) & 31;
    const int il = active ? static_cast<int>(ctx.last - bit) : 0;

    const double xj = sh.cand_x[slot];
    const double yj = sh.cand_y[slot];
    const double zj = sh.cand_z[slot];
    const uint32_t oj = sh.cand_index[slot];
    const double xi = sh.tile_x[il];
    const double yi = sh.tile_y[il];
    const double zi = sh.tile_z[il];
    const uint32_t oi = sh.tile_index[il];

    int32_t sx = 0, sy = 0, sz = 0;
    double tx = ctx.zero_tx, ty = ctx.zero_ty, tz = ctx.zero_tz;
    double mx = ctx.zero_tx, my = ctx.zero_ty, mz = ctx.zero_tz;
    if (ctx.need_shift) {
        unpack_shift(sh.cand_shift[slot], sx, sy, sz);
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
    // A half list that returns vectors computes only the orientation it keeps, from its own operands (both
    // orientations alive until the vectors are stored cost registers the kernel does not have). The other one has
    // the same components up to their signs (r_i - r_j = -(r_j - r_i) exactly, the shift vector of -S is minus that
    // of S, and the vector of the zero shift only decides the sign of a zero), so the squared distance, a sum of
    // squares in the same order, is the same either way.
    const bool flip = !FULL && (oi > oj || (oi == oj && !half_keeps_self_image(sx, sy, sz)));
    const bool kept_only = !FULL && STAGED;
    const double vx = kept_only ? ((flip ? xi : xj) - (flip ? xj : xi)) + (flip ? mx : tx) : (xj - xi) + tx;
    const double vy = kept_only ? ((flip ? yi : yj) - (flip ? yj : yi)) + (flip ? my : ty) : (yj - yi) + ty;
    const double vz = kept_only ? ((flip ? zi : zj) - (flip ? zj : zi)) + (flip ? mz : tz) : (zj - zi) + tz;
    const double wx = (xi - xj) + mx;
    const double wy = (yi - yj) + my;
    const double wz = (zi - zj) + mz;
    const double d2 = vx * vx + vy * vy + vz * vz;

    // rows of this redeem start at the (wave-uniform) cursor: every address is a scalar base plus a 32-bit lane offset
    const uint64_t cursor = state.out_cursor;
    const uint32_t ulane = static_cast<uint32_t>(lane);
    if (FULL) {
        if (active) {
            char* pair_rows = reinterpret_cast<char*>(out.pairs) + cursor * 16;
            stream_store(pair_rows + ulane * 16u, PairRow{oi, oj});
            stream_store(pair_rows + n * 16u + ulane * 16u, PairRow{oj, oi});
            if (out.shifts != nullptr) {
                char* shift_rows = reinterpret_cast<char*>(out.shifts) + cursor * 12;
                stream_store(shift_rows + ulane * 12u, ShiftRow{sx, sy, sz});
                stream_store(shift_rows + n * 12u + ulane * 12u, ShiftRow{-sx, -sy, -sz});
            }
            if (out.distances != nullptr) {
                char* distance_rows = reinterpret_cast<char*>(out.distances) + cursor * 8;
                const double d = sqrt(d2);
                stream_store(distance_rows + ulane * 8u, d);
                stream_store(distance_rows + n * 8u + ulane * 8u, d);
            }
            if (!STAGED && out.vectors != nullptr) {
                char* vector_rows = reinterpret_cast<char*>(out.vectors) + cursor * 24;
                stream_store(vector_rows + ulane * 24u, VectorHead{vx, vy});
                stream_store(vector_rows + ulane * 24u + 16u, vz);
                stream_store(vector_rows + n * 24u + ulane * 24u, VectorHead{wx, wy});
                stream_store(vector_rows + n * 24u + ulane * 24u + 16u, wz);
            }
        }
        if (STAGED && out.vectors != nullptr) {
            char* vector_rows = reinterpret_cast<char*>(out.vectors) + cursor * 24;
            store_vector_rows(sh.vector_stage, vector_rows, n, active, ulane, vx, vy, vz);
            store_vector_rows(sh.vector_stage, vector_rows + n * 24u, n, active, ulane, wx, wy, wz);
        }
        state.out_cursor += 2 * n;
    } else {
        if (active) {
            stream_store(reinterpret_cast<char*>(out.pairs) + cursor * 16 + ulane * 16u, PairRow{flip ? oj : oi, flip ? oi : oj});
            if (out.shifts != nullptr) {
                stream_store(
                    reinterpret_cast<char*>(out.shifts) + cursor * 12 + ulane * 12u,
                    ShiftRow{flip ? -sx : sx, flip ? -sy : sy, flip ? -sz : sz}
                );
            }
            if (out.distances != nullptr) {
                stream_store(reinterpret_cast<char*>(out.distances) + cursor * 8 + ulane * 8u, sqrt(d2));
            }
            if (!STAGED && out.vectors != nullptr) {
                char* row = reinterpret_cast<char*>(out.vectors) + cursor * 24 + ulane * 24u;
                stream_store(row, VectorHead{flip ? wx : vx, flip ? wy : vy});
                stream_store(row + 16u, flip ? wz : vz);
            }
        }
        if (STAGED && out.vectors != nullptr) {
            store_vector_rows(sh.vector_stage, reinterpret_cast<char*>(out.vectors) + cursor * 24, n, active, ulane, vx, vy, vz);
        }
        state.out_cursor += n;
    }
    state.tail += n;
    state.batch = aligning_batch<FULL>(state.out_cursor);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

/// What one wave carries from the sweep to the replay.
struct WorkItem {
    bool valid;          // there is a tile for this work item and it fits the shape of this kernel
    bool deferred;       // too many candidates to keep the columns: counted here, written by the write pass
    bool any_shift;
    bool tile_wrapped;
    uint32_t first_i, n_i;
    uint32_t n_batch, n_candidates;
    uint32_t unit_begin, n_units;
    uint32_t hits;
};

__device__ __forceinline__ uint64_t chain_load(const uint64_t* word) {
    return __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void chain_store(uint64_t* word, uint64_t value) {
    __hip_atomic_store(word, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/// What a wave of the chain waits with: when it started waiting, how often it has polled.
struct ChainPatience {
    uint64_t since;
    uint32_t spins;
    uint32_t spin_limit;
    uint32_t wait_ticks;
};

__device__ __forceinline__ ChainPatience chain_patience(uint32_t spin_limit, uint32_t wait_ticks) {
    ChainPatience patience;
    patience.since = wall_clock64();
    patience.spins = 0;
    patience.spin_limit = spin_limit;
    patience.wait_ticks = wait_ticks;
    return patience;
}

/// Bounded wait between two polls of the chain; returns false when patience ran out: after `wait_ticks` of waiting
/// (the 100 MHz clock, the same on every compute unit whatever its own clock does), after `spin_limit` polls, or as
/// soon as another wave of the launch has given up (the rows of the launch are void then, there is nothing to wait for).
__device__ __forceinline__ bool chain_wait(ChainPatience& patience, int lane, FusedStatus* status) {
    patience.spins += 1;
    const bool someone_gave_up =
        (patience.spins & 7u) == 0 && __hip_atomic_load(&status->chain_timeout, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
    const bool out_of_patience =
        patience.spins > patience.spin_limit || someone_gave_up || wall_clock64() - patience.since > patience.wait_ticks;
    if (__ballot(out_of_patience) != 0) { // (the same answer for every lane of the wave)
        if (lane == 0) {
            atomicAdd(&status->chain_timeout, 1u);
        }
        return false;
    }
    __builtin_amdgcn_s_sleep(8);
    return true;
}

/// Sum of the rows of all earlier workgroups. Called by one full wave of every workgroup.
///
/// Two levels keep the polling light. Every workgroup publishes its rows in `chain.blocks`. Workgroups form groups
/// of CHAIN_GROUP consecutive ones; the last workgroup of a group waits for the rows of the others, publishes the
/// group's rows in `chain.groups`, finds the rows of all earlier groups by decoupled look-back over that (short)
/// array, and publishes them in `chain.bases`. The other workgroups of the group poll that one word, then add the
/// rows of the earlier workgroups of their group. Every word carries its own flag, so no fences are needed.
__device__ __forceinline__ uint64_t chain_position(
    const Chain& chain, uint32_t block, uint32_t n_blocks, uint64_t own_rows, int lane, FusedStatus* status,
    uint32_t spin_limit, uint32_t wait_ticks
) {
    if (lane == 0) {
        chain_store(&chain.blocks[block], CHAIN_AGGREGATE | own_rows);
    }
    const uint32_t group = block / CHAIN_GROUP;
    const uint32_t group_first = group * CHAIN_GROUP;
    const uint32_t member = block - group_first;
    const bool leader = member == CHAIN_GROUP - 1 || block == n_blocks - 1;
    ChainPatience patience = chain_patience(spin_limit, wait_ticks);
    bool gave_up = false;

    uint64_t group_before = 0;
    if (leader) {
        // ---- rows of the group: lanes 0..member-1 watch the other workgroups
        uint64_t rows_of_member = 0;
        while (true) {
            uint64_t word = CHAIN_AGGREGATE;
            if (static_cast<uint32_t>(lane) < member) {
                word = chain_load(&chain.blocks[group_first + lane]);
            }
            rows_of_member = word & CHAIN_VALUE;
            if (__ballot((word >> CHAIN_FLAG_SHIFT) == 0) == 0) {
                break;
            }
            if (!chain_wait(patience, lane, status)) {
                gave_up = true;
                break;
            }
        }
        const uint64_t group_rows = read_lane(wave_inclusive_scan(rows_of_member), WAVE - 1) + own_rows;
        if (group == 0) {
            if (lane == 0) {
                chain_store(&chain.groups[0], CHAIN_PREFIX | group_rows);
            }
        } else {
            if (lane == 0) {
                chain_store(&chain.groups[group], CHAIN_AGGREGATE | group_rows);
            }
            // ---- decoupled look-back over the groups: lane l looks at group nearest - l
            int64_t nearest = static_cast<int64_t>(group) - 1;
            bool done = false;
            while (!done) {
                const int64_t at = nearest - lane;
                uint64_t word = CHAIN_PREFIX; // before the first group: nothing
                if (at >= 0) {
                    word = chain_load(&chain.groups[at]);
                }
                const uint64_t flag = word >> CHAIN_FLAG_SHIFT;
                const uint64_t is_prefix = __ballot(flag == 2);
                const uint64_t is_missing = __ballot(flag == 0);
                // lanes [0, usable) hold aggregates, possibly ended by a prefix
                const uint32_t first_prefix =
                    is_prefix != 0 ? __ffsll(static_cast<unsigned long long>(is_prefix)) - 1 : WAVE;
                const uint32_t first_missing =
                    is_missing != 0 ? __ffsll(static_cast<unsigned long long>(is_missing)) - 1 : WAVE;
                const bool reaches_prefix = first_prefix < first_missing;
                const uint32_t usable = reaches_prefix ? first_prefix + 1 : first_missing;

                uint64_t value = static_cast<uint32_t>(lane) < usable ? (word & CHAIN_VALUE) : 0;
                value = wave_inclusive_scan(value);
                group_before += read_lane(value, WAVE - 1);
                nearest -= usable;
                if (reaches_prefix) {
                    done = true;
                } else if (usable == 0 && !chain_wait(patience, lane, status)) {
                    gave_up = true;
                    done = true;
                }
            }
            if (lane == 0) {
                chain_store(&chain.groups[group], CHAIN_PREFIX | ((group_before + group_rows) & CHAIN_VALUE));
            }
        }
        if (lane == 0) {
            chain_store(&chain.bases[group], CHAIN_PREFIX | (group_before & CHAIN_VALUE));
        }
        // (the words are published also by a leader that gave up: nobody should wait for them any longer)
        // rows of the earlier workgroups of this group: everything but the own rows
        return gave_up ? CHAIN_GAVE_UP : group_before + (group_rows - own_rows);
    }

    // ---- not the leader: wait for the group's base, then add the earlier members (all published by then)
    while (true) {
        const uint64_t word = chain_load(&chain.bases[group]);
        if ((word >> CHAIN_FLAG_SHIFT) != 0) {
            group_before = word & CHAIN_VALUE;
            break;
        }
        if (!chain_wait(patience, lane, status)) {
            return CHAIN_GAVE_UP;
        }
    }
    uint64_t rows_of_member = 0;
    if (static_cast<uint32_t>(lane) < member) {
        rows_of_member = chain_load(&chain.blocks[group_first + lane]) & CHAIN_VALUE;
    }
    return group_before + read_lane(wave_inclusive_scan(rows_of_member), WAVE - 1);
}

/// Four waves per workgroup, one work item each; the waves of a workgroup meet twice: to add up their rows, and to
/// learn their place. ORDERED: the rows come out in work-item order, the same on every run (the place comes from the
/// chain). Otherwise no workgroup waits for another and the rows come out in order of arrival, which varies from run
/// to run like the order of the reference's GPU kernels (vesin/src/cuda/cell_list.cu:664, an atomic per pair there).
/// BATCH: many systems in one launch (see search_kernel_batch): the grid is the one of the tile's system, tiles are
/// taken in their order (systems stay together) and every work item reports its first row, from which the host
/// learns where each system's rows start. Only used with ORDERED.
/// STAGED: for calls that return vectors: their rows are lined up in LDS before they are stored (store_vector_rows).
///
/// Five waves per SIMD: the kernel needs 96 vector registers for that (the 32 hit columns among them), one fewer
/// than the compiler takes when left alone, which would be four waves (measured: the clustered 500,000-atom system
/// 0.59 -> 0.54 ms, the batch of 4096 small cells 1.78 -> 1.75 ms, the 1,000,000-atom lattice unchanged, being bound
/// by its row stores; six waves with 8 columns instead of 32 made that one slower).
template <bool FULL, bool ORDERED, bool BATCH = false, bool STAGED = false>
__global__ __launch_bounds__(SEARCH_BLOCK) __attribute__((amdgpu_waves_per_eu(5, 5))) void fused_search_kernel(FusedArgs fargs, GridParams single_grid) {
    constexpr int R = 2;
    __shared__ FusedShared<STAGED> shared;
    const SearchArgs& args = fargs.search;
    const int lane = lane_id();
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    FusedWaveShared<STAGED>& sh = shared.wave[wave];
    GridParams batch_grid;
    const GridParams& g = BATCH ? batch_grid : single_grid;
    // fixed-capacity layout (never in a batch): every cell has the same number of tiles, some of them empty
    const uint32_t direct_capacity = BATCH ? 0 : args.direct_capacity;
    const uint32_t direct_tiles = direct_capacity / TILE_POINTS;
    const uint32_t n_tiles =
        direct_capacity != 0
            ? single_grid.n_cells * direct_tiles
            : static_cast<uint32_t>(args.cell_scan[BATCH ? args.total_cells : single_grid.n_cells] >> 32);
    const uint32_t work = blockIdx.x * SEARCH_WAVES + wave;
    const SortedPoints& sorted = args.sorted;

    WorkItem item;
    item.valid = false;
    item.deferred = false;
    item.any_shift = false;
    item.tile_wrapped = false;
    item.hits = 0;
    item.n_units = 0;
    item.unit_begin = 0;
    item.first_i = 0;
    item.n_i = 0;
    item.n_batch = 0;
    item.n_candidates = 0;
    // hit columns of the work item's units; indexed with wave-uniform values only
    uint32_t columns[FUSED_UNITS];
#pragma unroll
    for (int u = 0; u < FUSED_UNITS; u++) {
        columns[u] = 0;
    }

    // ---- phase 1: sweep, keep the columns
    bool general = false;
    if (work < args.n_work) {
        const uint32_t slice = work % args.n_slices;
        const uint32_t slot = work / args.n_slices;
        const uint32_t per_xcd = BATCH ? n_tiles : (n_tiles + N_XCD - 1) / N_XCD;
        const uint32_t xcd = BATCH ? 0 : (slot / SEARCH_WAVES) % N_XCD;
        const uint32_t within = BATCH ? slot : (slot / (SEARCH_WAVES * N_XCD)) * SEARCH_WAVES + slot % SEARCH_WAVES;
        const uint32_t tile_id = xcd * per_xcd + within;

        Tile tile = {};
        if (within < per_xcd && tile_id < n_tiles) {
            if (direct_capacity != 0) {
                const uint32_t cell = tile_id / direct_tiles;
                const uint32_t k = tile_id % direct_tiles;
                const uint32_t in_cell = min(args.direct_counts[cell], direct_capacity);
                tile.cell = cell;
                tile.first = cell * direct_capacity + k * TILE_POINTS;
                tile.count = in_cell > k * TILE_POINTS ? min(static_cast<uint32_t>(TILE_POINTS), in_cell - k * TILE_POINTS) : 0;
                tile.wrapped = args.direct_wrapped[tile_id];
            } else {
                tile = args.tiles[tile_id];
            }
        }
        if (tile.count != 0) {
            item.n_i = tile.count;
            item.first_i = tile.first;
            item.tile_wrapped = (tile.wrapped & 1u) != 0;
            uint32_t first_cell = 0;
            if (BATCH) {
                const uint32_t system = tile_system(tile);
                batch_grid = args.grids[system];
                first_cell = args.cell_base[system];
            }
            const uint64_t* __restrict__ cell_scan = args.cell_scan + first_cell;
            const uint32_t local_cell = tile.cell - first_cell;
            const int32_t cx = local_cell % g.n[0];
            const int32_t cy = (local_cell / g.n[0]) % g.n[1];
            const int32_t cz = local_cell / (g.n[0] * g.n[1]);

            const int32_t span_y = 2 * g.s[1] + 1;
            const int32_t span_z = 2 * g.s[2] + 1;
            const uint32_t n_stencil = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z;
            const uint32_t centre = n_stencil / 2;
            const uint32_t n_entries = n_stencil - centre;

            if (n_entries > MAX_ENTRIES) {
                general = true;
            } else {
                if (static_cast<uint32_t>(lane) < item.n_i) {
                    const uint32_t at = item.first_i + lane;
                    sh.tile_x[lane] = sorted.p[at].x;
                    sh.tile_y[lane] = sorted.p[at].y;
                    sh.tile_z[lane] = sorted.p[at].z;
                    sh.tile_index[lane] = sorted.p[at].index;
                    sh.tile_wx[lane] = sorted.wx[at];
                    sh.tile_wy[lane] = sorted.wy[at];
                    sh.tile_wz[lane] = sorted.wz[at];
                }
                item.n_batch = n_entries;
                fill_stencil_tables(
                    sh, lane, centre, n_entries, cx, cy, cz, span_y, span_z, g, cell_scan, args.direct_counts, direct_capacity
                );
                item.n_candidates = __builtin_amdgcn_readfirstlane(sh.n_candidates);

                const uint32_t n_groups = (item.n_candidates + WAVE * R - 1) / (WAVE * R);
                const uint32_t per_slice = (n_groups + args.n_slices - 1) / args.n_slices;
                const uint32_t group_begin = min(n_groups, slice * per_slice);
                const uint32_t group_end = min(n_groups, group_begin + per_slice);
                item.unit_begin = group_begin * R;
                item.n_units = (group_end - group_begin) * R;
                item.deferred = item.n_units > FUSED_UNITS;
            }

            if (!general) {
                item.valid = true;
                for (uint32_t pair = 0; pair < item.n_units / R; pair++) {
                    SweepCandidates<R> c;
                    bool any_shift = false;
                    bool any_same = false;
                    bool too_far = false;
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const uint32_t k = (item.unit_begin + pair * R + r) * WAVE + lane;
                        const UnitCandidates u = locate_unit(sh, item.n_batch, item.n_candidates, k, sorted);
                        c.x[r] = c.y[r] = c.z[r] = __builtin_nan("");
                        c.tx[r] = c.ty[r] = c.tz[r] = 0.0;
                        c.position[r] = 0xFFFFFFFFu;
                        if (u.valid) {
                            c.x[r] = sorted.p[u.at].x;
                            c.y[r] = sorted.p[u.at].y;
                            c.z[r] = sorted.p[u.at].z;
                            if (u.same_cell) {
                                c.position[r] = u.at;
                            }
                        }
                        c.shift[r] = pack_shift(u.bx, u.by, u.bz);
                        const bool shifted = (u.bx | u.by | u.bz) != 0;
                        const bool far = abs(u.bx) > PACKED_SHIFT_LIMIT || abs(u.by) > PACKED_SHIFT_LIMIT ||
                                         abs(u.bz) > PACKED_SHIFT_LIMIT;
                        any_shift = any_shift || (__ballot(shifted) != 0);
                        any_same = any_same || (__ballot(u.same_cell) != 0);
                        too_far = too_far || (__ballot(far) != 0);
                        if (shifted) {
                            shift_vector(g, u.bx, u.by, u.bz, c.tx[r], c.ty[r], c.tz[r]);
                        }
                    }
                    if (too_far) {
                        general = true;
                        break;
                    }
                    item.any_shift = item.any_shift || any_shift;

                    uint32_t column[R] = {0, 0};
                    uint32_t hits;
                    if (item.tile_wrapped) {
                        hits = sweep_columns_wrapped<R>(sorted, item.first_i, item.n_i, c, g, column);
                    } else if (any_shift) {
                        if (any_same) {
                            hits = sweep_columns<R, true, true>(sorted, item.first_i, item.n_i, c, g.cutoff2, column);
                        } else {
                            hits = sweep_columns<R, true, false>(sorted, item.first_i, item.n_i, c, g.cutoff2, column);
                        }
                    } else {
                        if (any_same) {
                            hits = sweep_columns<R, false, true>(sorted, item.first_i, item.n_i, c, g.cutoff2, column);
                        } else {
                            hits = sweep_columns<R, false, false>(sorted, item.first_i, item.n_i, c, g.cutoff2, column);
                        }
                    }
                    item.hits += hits;
                    if (pair * R < FUSED_UNITS) {
#pragma unroll
                        for (int r = 0; r < R; r++) {
                            columns[pair * R + r] = column[r];
                        }
                    }
                }
            }
            if (general) {
                item.valid = false;
                item.hits = 0;
                if (lane == 0) {
                    atomicAdd(&fargs.status->general, 1u);
                }
            }
        }
    }

    // ---- phase 2: the place of the wave's rows in the output. The workgroup adds up its waves and takes room for
    // all of them at once: thousands of waves asking the same counter one by one keep each other waiting (measured
    // on 1,000,000 atoms: 0.72 ms with an atomic per wave, 0.69 ms with one per workgroup of four).
    const uint32_t own_rows = FULL ? 2 * item.hits : item.hits;
    if (lane == 0) {
        shared.rows[wave] = own_rows;
    }
    __syncthreads();
    uint64_t rows_before_wave = 0;
    uint64_t block_rows = 0;
#pragma unroll
    for (int w = 0; w < SEARCH_WAVES; w++) {
        const uint32_t rows = uniform(shared.rows[w]);
        rows_before_wave += static_cast<uint32_t>(w) < wave ? rows : 0;
        block_rows += rows;
    }
    if (wave == 0) {
        uint64_t before = 0;
        if (ORDERED) {
            // rows in work-item order: the workgroup chains with the earlier workgroups
            before = chain_position(
                fargs.chain, blockIdx.x, gridDim.x, block_rows, lane, fargs.status, fargs.spin_limit, fargs.wait_ticks
            );
        } else if (lane == 0 && block_rows != 0) {
            // rows in order of arrival: no workgroup waits for another
            before = atomicAdd(&fargs.status->total_rows, static_cast<unsigned long long>(block_rows));
        }
        // (a workgroup that does not know its place writes nothing; the host reads `chain_timeout`)
        const bool placed = !ORDERED || before != CHAIN_GAVE_UP;
        const bool fits = placed && before + block_rows <= args.capacity;
        if (lane == 0) {
            shared.base = before;
            shared.writable = fits ? 1u : 0u;
            if (placed && !fits) {
                atomicAdd(&fargs.status->overflow, 1u);
            }
            if (ORDERED && blockIdx.x == gridDim.x - 1) {
                fargs.status->total_rows = before + block_rows;
            }
        }
    }
    __syncthreads();
    const uint64_t first_row = uniform(shared.base) + rows_before_wave;
    const bool writable = uniform(shared.writable) != 0;
    const bool leave_to_write_pass = item.valid && item.deferred && item.hits != 0 && writable;
    if (work < args.n_work && lane == 0) {
        if (BATCH) {
            fargs.first_rows[work] = first_row;
        }
        args.counts[work] = leave_to_write_pass ? 1u : 0u;
        if (leave_to_write_pass) {
            fargs.first_rows[work] = first_row;
            atomicAdd(&fargs.status->deferred, 1u);
            atomicAdd(&fargs.status->deferred_rows, static_cast<unsigned long long>(own_rows));
        }
    }
    if (!item.valid || item.deferred || item.hits == 0 || !writable) {
        return;
    }

    // ---- phase 3: replay the columns, write the rows
    ReplayContext ctx;
    ctx.lane = lane;
    ctx.tile_wrapped = item.tile_wrapped;
    ctx.need_shift = item.any_shift || item.tile_wrapped;
    shift_vector(g, 0, 0, 0, ctx.zero_tx, ctx.zero_ty, ctx.zero_tz);

    ReplayState state;
    state.out_cursor = first_row;
    state.head = 0;
    state.tail = 0;
    state.batch = aligning_batch<FULL>(state.out_cursor);
    ctx.last = item.n_i - 1;
    uint32_t filled[2] = {0, 0}; // value of head when the unit in each half of the candidate records was done

    for (uint32_t unit = 0; unit < item.n_units; unit++) {
        uint32_t column = columns[unit];
        if (__ballot(column != 0) == 0) {
            continue;
        }
        const uint32_t half = unit & 1;
        if (half == 0 ? state.tail < filled[0] : state.tail < filled[1]) {
            // pending tickets still point into the records about to be replaced
            redeem_fused<FULL, STAGED>(state.head - state.tail, state, sh, args.out, g, ctx);
        }
        const uint32_t k = (item.unit_begin + unit) * WAVE + lane;
        const UnitCandidates u = locate_unit(sh, item.n_batch, item.n_candidates, k, sorted);
        if (u.valid) {
            const int record = half * WAVE + lane;
            sh.cand_x[record] = sorted.p[u.at].x;
            sh.cand_y[record] = sorted.p[u.at].y;
            sh.cand_z[record] = sorted.p[u.at].z;
            sh.cand_index[record] = sorted.p[u.at].index;
            sh.cand_shift[record] = pack_shift(u.bx, u.by, u.bz);
        }
        wave_sync();

        // every round, each lane with hits left peels one bit off its column and drops a ticket
        const uint32_t record = half * WAVE + lane;
        while (true) {
            const uint64_t mask = __ballot(column != 0);
            if (mask == 0) {
                break;
            }
            if (column != 0) {
                const uint32_t bit = __builtin_ctz(column);
                column &= column - 1;
                const uint32_t at = (state.head + rank_in_mask(mask)) & (RING - 1);
                sh.ring[at] = static_cast<uint16_t>(record | (bit << 8));
            }
            state.head += __popcll(mask);
            while (state.head - state.tail >= state.batch) {
                redeem_fused<FULL, STAGED>(state.batch, state, sh, args.out, g, ctx);
            }
        }
        if (half == 0) {
            filled[0] = state.head;
        } else {
            filled[1] = state.head;
        }
    }
    if (state.head != state.tail) {
        redeem_fused<FULL, STAGED>(state.head - state.tail, state, sh, args.out, g, ctx);
    }
}

} // namespace vesin_hip

#endif
