// Stencil search over the cell grid: the kernel that decides pair membership and produces the output arrays.
//
// One workgroup (4 waves) owns one tile = up to 64 points `i` of one cell. The candidates `j` are the points of
// every cell in the (2s+1)^3 stencil around that cell, periodic images included (a cell may appear several
// times with different cell shifts when the box is narrower than the stencil: that is the multi-image path; with a
// single cell the stencil enumerates images only and the kernel is a tiled brute force, optionally split over
// several workgroups per tile).
//
// Mapping: lanes hold candidates. A wave loads R groups of 64 consecutive candidates into registers (coalesced
// reads from the cell-sorted structure-of-arrays), then loops over the tile's points `i`, whose coordinates come
// in through scalar loads. Each (i, group) test costs 9-12 fp64 VALU operations and yields a 64-bit hit mask in
// scalar registers.
//
// The same code runs twice:
//   COUNT  adds up popcounts: one 32-bit total per wave, no atomics;
//   WRITE  (after a device-wide scan of the totals gave every wave its output range) recomputes the masks and
//          compacts: hit lanes drop a 16-bit ticket (lane, group, i) into a per-wave LDS ring at the slot given by
//          mbcnt of the mask; whenever 64 tickets are pending, all 64 lanes redeem one each, pulling the
//          candidate's data out of the owning lane with ds_bpermute, recomputing shift / vector / distance and
//          storing 64 consecutive output rows.
//
// Arithmetic (bit-for-bit the CPU reference, vesin/src/cpu_cell_list.cpp:135-138 and vesin/src/types.hpp:232-243,
// vesin/src/math.hpp:14-16,111-117; compile with -ffp-contract=off):
//   T_k = S0*H0k + S1*H1k + S2*H2k (left to right), v_k = (r_jk - r_ik) + T_k, d2 = v0*v0 + v1*v1 + v2*v2,
//   keep iff d2 < cutoff*cutoff, d = sqrt(d2).
// Adding T may be skipped in the test when S = 0 (it is +-0 and cannot change d2); the stored vector always adds it.
//
// Reference roles replaced: find_neighbors_cell_list (vesin/src/cuda/cell_list.cu:428-705), brute_force_*
// (vesin/src/cuda/bruteforce.cu:241-573); CPU twin CellList::foreach_pair + callback
// (vesin/src/cpu_cell_list.cpp:376-451, :100-163).
#ifndef VESIN_HIP_SEARCH_CUH
#define VESIN_HIP_SEARCH_CUH

#include "cells.cuh"
#include "device_common.cuh"

namespace vesin_hip {

constexpr int MAX_ENTRIES = 512; // stencil entries resident in LDS at a time
constexpr int RING = 128;        // tickets per wave ring (power of two, >= 2 * WAVE)

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
    uint32_t* counts;          // COUNT: [gridDim.x * 4]
    const uint64_t* offsets;   // WRITE: [gridDim.x * 4 + 1] exclusive scan of counts
    SearchOutputs out;
    uint32_t n_slices;         // workgroups sharing one tile (each takes a slice of the candidates)
};

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

template <bool WRITE, bool FULL, int R>
__global__ __launch_bounds__(BLOCK) void search_kernel(SearchArgs args, GridParams g) {
    __shared__ uint32_t ent_prefix[MAX_ENTRIES + 1]; // candidates before each stencil entry
    __shared__ uint32_t ent_start[MAX_ENTRIES];      // first sorted position of the entry's cell
    __shared__ int32_t ent_shift[MAX_ENTRIES];       // packed cell shift, bit 30: same cell as the tile
    __shared__ uint32_t wave_carry;
    // tile points, for the redeem phase
    __shared__ double tile_x[WAVE], tile_y[WAVE], tile_z[WAVE];
    __shared__ uint32_t tile_index[WAVE];
    __shared__ int32_t tile_wx[WAVE], tile_wy[WAVE], tile_wz[WAVE];
    __shared__ uint16_t ring[WRITE ? WAVES_PER_BLOCK : 1][RING];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t tile_id = blockIdx.x / args.n_slices;
    const uint32_t slice = blockIdx.x % args.n_slices;
    const uint32_t n_tiles = static_cast<uint32_t>(args.cell_scan[g.n_cells] >> 32);
    const size_t wave_slot = static_cast<size_t>(blockIdx.x) * WAVES_PER_BLOCK + wave;

    if (tile_id >= n_tiles) {
        if (!WRITE && lane == 0) {
            args.counts[wave_slot] = 0;
        }
        return;
    }

    const Tile tile = args.tiles[tile_id];
    const uint32_t n_i = tile.count;
    const uint32_t first_i = tile.first;
    const int32_t cx = tile.cell % g.n[0];
    const int32_t cy = (tile.cell / g.n[0]) % g.n[1];
    const int32_t cz = tile.cell / (g.n[0] * g.n[1]);

    const double* __restrict__ px = args.sorted.x;
    const double* __restrict__ py = args.sorted.y;
    const double* __restrict__ pz = args.sorted.z;
    const uint32_t* __restrict__ pindex = args.sorted.index;
    const int32_t* __restrict__ pwx = args.sorted.wx;
    const int32_t* __restrict__ pwy = args.sorted.wy;
    const int32_t* __restrict__ pwz = args.sorted.wz;

    if (WRITE && threadIdx.x < n_i) {
        uint32_t at = first_i + threadIdx.x;
        tile_x[threadIdx.x] = px[at];
        tile_y[threadIdx.x] = py[at];
        tile_z[threadIdx.x] = pz[at];
        tile_index[threadIdx.x] = pindex[at];
        tile_wx[threadIdx.x] = pwx[at];
        tile_wy[threadIdx.x] = pwy[at];
        tile_wz[threadIdx.x] = pwz[at];
    }

    const int32_t span_y = 2 * g.s[1] + 1;
    const int32_t span_z = 2 * g.s[2] + 1;
    const uint32_t n_entries = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z;

    uint32_t wave_total = 0;                 // COUNT
    uint64_t out_cursor = 0;                 // WRITE: next output row of this wave
    if (WRITE) {
        out_cursor = args.offsets[wave_slot];
    }

    for (uint32_t batch = 0; batch < n_entries; batch += MAX_ENTRIES) {
        const uint32_t n_batch = min(static_cast<uint32_t>(MAX_ENTRIES), n_entries - batch);
        __syncthreads(); // everyone is done with the previous batch's tables (and the tile staging is visible)

        // ---- stencil entries of this batch: neighbour cell, its cell shift, how many points it holds
        for (uint32_t e = threadIdx.x; e < n_batch; e += BLOCK) {
            uint32_t linear = batch + e;
            int32_t dz = static_cast<int32_t>(linear % span_z) - g.s[2];
            int32_t dy = static_cast<int32_t>((linear / span_z) % span_y) - g.s[1];
            int32_t dx = static_cast<int32_t>(linear / (span_z * span_y)) - g.s[0];
            int32_t c[3] = {cx + dx, cy + dy, cz + dz};
            int32_t q[3] = {0, 0, 0};
            bool valid = true;
#pragma unroll
            for (int d = 0; d < 3; d++) {
                const int32_t n = g.n[d];
                if (g.periodic[d]) {
                    int32_t quotient = c[d] / n;
                    int32_t rest = c[d] - quotient * n;
                    if (rest < 0) {
                        rest += n;
                        quotient -= 1;
                    }
                    q[d] = quotient;
                    c[d] = rest;
                } else if (c[d] < 0 || c[d] >= n) {
                    valid = false;
                }
            }
            uint32_t start = 0;
            uint32_t count = 0;
            int32_t packed = 0;
            if (valid) {
                uint32_t neighbour = (static_cast<uint32_t>(c[2]) * g.n[1] + c[1]) * g.n[0] + c[0];
                start = static_cast<uint32_t>(args.cell_scan[neighbour]);
                count = static_cast<uint32_t>(args.cell_scan[neighbour + 1]) - start;
                packed = pack_shift(q[0], q[1], q[2]);
                if (neighbour == tile.cell) {
                    packed |= 1 << 30;
                }
            }
            ent_start[e] = start;
            ent_shift[e] = packed;
            ent_prefix[e + 1] = count; // scanned in place below
        }
        __syncthreads();

        if (wave == 0) {
            uint32_t carry = 0;
            for (uint32_t base = 0; base < n_batch; base += WAVE) {
                uint32_t e = base + lane;
                uint32_t v = e < n_batch ? ent_prefix[e + 1] : 0;
                uint32_t inclusive = wave_inclusive_scan(v) + carry;
                if (e < n_batch) {
                    ent_prefix[e + 1] = inclusive;
                }
                carry = read_lane(inclusive, WAVE - 1);
            }
            if (lane == 0) {
                ent_prefix[0] = 0;
                wave_carry = carry;
            }
        }
        __syncthreads();

        const uint32_t n_candidates = wave_carry;
        const uint32_t n_groups = (n_candidates + WAVE * R - 1) / (WAVE * R);
        const uint32_t per_slice = (n_groups + args.n_slices - 1) / args.n_slices;
        const uint32_t group_begin = slice * per_slice;
        const uint32_t group_end = min(n_groups, group_begin + per_slice);

        for (uint32_t group = group_begin + wave; group < group_end; group += WAVES_PER_BLOCK) {
            // ---- load R x 64 candidates into registers
            double xj[R], yj[R], zj[R];   // position
            double tx[R], ty[R], tz[R];   // shift vector for a tile point that was not wrapped
            int32_t bx[R], by[R], bz[R];  // cell shift minus the candidate's own wrap shift
            uint32_t oj[R];               // original index
            bool same_cell[R];
            bool any_shift[R];            // some lane of the group has a non-zero base shift
            bool any_same[R];             // some lane of the group is in the tile's own cell

#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint32_t k = (group * R + r) * WAVE + lane;
                const bool valid = k < n_candidates;
                xj[r] = yj[r] = zj[r] = __builtin_nan("");
                tx[r] = ty[r] = tz[r] = 0.0;
                bx[r] = by[r] = bz[r] = 0;
                oj[r] = 0xFFFFFFFFu;
                same_cell[r] = false;
                if (valid) {
                    // largest e with ent_prefix[e] <= k
                    uint32_t lo = 0;
                    uint32_t hi = n_batch;
                    while (hi - lo > 1) {
                        uint32_t mid = (lo + hi) >> 1;
                        if (ent_prefix[mid] <= k) {
                            lo = mid;
                        } else {
                            hi = mid;
                        }
                    }
                    const uint32_t at = ent_start[lo] + (k - ent_prefix[lo]);
                    const int32_t packed = ent_shift[lo];
                    int32_t qx, qy, qz;
                    unpack_shift(packed, qx, qy, qz);
                    same_cell[r] = (packed >> 30) & 1;
                    xj[r] = px[at];
                    yj[r] = py[at];
                    zj[r] = pz[at];
                    oj[r] = pindex[at];
                    bx[r] = qx - pwx[at];
                    by[r] = qy - pwy[at];
                    bz[r] = qz - pwz[at];
                    shift_vector(g, bx[r], by[r], bz[r], tx[r], ty[r], tz[r]);
                }
                any_shift[r] = __ballot((bx[r] | by[r] | bz[r]) != 0) != 0;
                any_same[r] = __ballot(same_cell[r]) != 0;
            }

            uint32_t pending_head = 0; // tickets appended / redeemed for this group (ring positions)
            uint32_t pending_tail = 0;

            // ---- redeem up to 64 tickets: all lanes write one output row each
            auto redeem = [&](uint32_t n) {
                __builtin_amdgcn_wave_barrier();
                const bool active = static_cast<uint32_t>(lane) < n;
                const uint32_t ticket = static_cast<const volatile uint16_t*>(ring[WRITE ? wave : 0])[(pending_tail + lane) & (RING - 1)];
                const int owner = ticket & 63;
                const int which = (ticket >> 6) & 3;
                const int il = active ? (ticket >> 8) & 63 : 0;

                double cxj = 0, cyj = 0, czj = 0;
                int32_t cbx = 0, cby = 0, cbz = 0;
                uint32_t coj = 0;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    double sx = __shfl(xj[r], owner);
                    double sy = __shfl(yj[r], owner);
                    double sz = __shfl(zj[r], owner);
                    int32_t sbx = __shfl(bx[r], owner);
                    int32_t sby = __shfl(by[r], owner);
                    int32_t sbz = __shfl(bz[r], owner);
                    uint32_t so = static_cast<uint32_t>(__shfl(static_cast<int>(oj[r]), owner));
                    if (which == r) {
                        cxj = sx;
                        cyj = sy;
                        czj = sz;
                        cbx = sbx;
                        cby = sby;
                        cbz = sbz;
                        coj = so;
                    }
                }

                const int32_t sx = cbx + tile_wx[il];
                const int32_t sy = cby + tile_wy[il];
                const int32_t sz = cbz + tile_wz[il];
                double ttx, tty, ttz;
                shift_vector(g, sx, sy, sz, ttx, tty, ttz);
                const double vx = (cxj - tile_x[il]) + ttx;
                const double vy = (cyj - tile_y[il]) + tty;
                const double vz = (czj - tile_z[il]) + ttz;
                const double d2 = vx * vx + vy * vy + vz * vz;

                if (active) {
                    const uint64_t row = out_cursor + lane;
                    ulonglong2 pair;
                    pair.x = tile_index[il];
                    pair.y = coj;
                    reinterpret_cast<ulonglong2*>(args.out.pairs)[row] = pair;
                    if (args.out.shifts != nullptr) {
                        int32_t* s = args.out.shifts + 3 * row;
                        s[0] = sx;
                        s[1] = sy;
                        s[2] = sz;
                    }
                    if (args.out.distances != nullptr) {
                        args.out.distances[row] = sqrt(d2);
                    }
                    if (args.out.vectors != nullptr) {
                        double* v = args.out.vectors + 3 * row;
                        v[0] = vx;
                        v[1] = vy;
                        v[2] = vz;
                    }
                }
                out_cursor += n;
                pending_tail += n;
                __builtin_amdgcn_wave_barrier();
            };

            // ---- every tile point against the R x 64 candidates
            for (uint32_t i = 0; i < n_i; i++) {
                const uint32_t at = first_i + i;
                const double xi = px[at];
                const double yi = py[at];
                const double zi = pz[at];
                const uint32_t oi = pindex[at];
                const int32_t wix = pwx[at];
                const int32_t wiy = pwy[at];
                const int32_t wiz = pwz[at];
                const bool i_wrapped = (wix | wiy | wiz) != 0;

#pragma unroll
                for (int r = 0; r < R; r++) {
                    double vx = xj[r] - xi;
                    double vy = yj[r] - yi;
                    double vz = zj[r] - zi;
                    if (i_wrapped) {
                        double ttx, tty, ttz;
                        shift_vector(g, bx[r] + wix, by[r] + wiy, bz[r] + wiz, ttx, tty, ttz);
                        vx += ttx;
                        vy += tty;
                        vz += ttz;
                    } else if (any_shift[r]) {
                        vx += tx[r];
                        vy += ty[r];
                        vz += tz[r];
                    }
                    const double d2 = vx * vx + vy * vy + vz * vz;
                    bool hit = d2 < g.cutoff2;

                    if (FULL) {
                        if (any_same[r]) {
                            // a point is not its own neighbour unless a non-zero shift separates the two
                            const bool zero = ((bx[r] + wix) | (by[r] + wiy) | (bz[r] + wiz)) == 0;
                            hit = hit && !(oj[r] == oi && zero);
                        }
                    } else {
                        bool keep = oi < oj[r];
                        if (any_same[r]) {
                            const int32_t sx = bx[r] + wix;
                            const int32_t sy = by[r] + wiy;
                            const int32_t sz = bz[r] + wiz;
                            const bool zero = (sx | sy | sz) == 0;
                            keep = keep || (oj[r] == oi && !zero && half_keeps_self_image(sx, sy, sz));
                        }
                        hit = hit && keep;
                    }

                    const uint64_t mask = __ballot(hit);
                    if (mask != 0) {
                        const uint32_t hits = __popcll(mask);
                        if (WRITE) {
                            if (hit) {
                                const uint32_t slot = (pending_head + rank_in_mask(mask)) & (RING - 1);
                                static_cast<volatile uint16_t*>(ring[wave])[slot] =
                                    static_cast<uint16_t>(lane | (r << 6) | (i << 8));
                            }
                            pending_head += hits;
                            if (pending_head - pending_tail >= WAVE) {
                                redeem(WAVE);
                            }
                        } else {
                            wave_total += hits;
                        }
                    }
                }
            }

            if (WRITE && pending_head != pending_tail) {
                redeem(pending_head - pending_tail);
            }
        }
    }

    if (!WRITE && lane == 0) {
        args.counts[wave_slot] = wave_total;
    }
}

} // namespace vesin_hip

#endif
