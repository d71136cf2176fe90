// Sorted lists of many small systems of one cell each (options.sorted on the batched entry point): rows in
// (first point, second point, shift) order straight from the search, without sorting anything.
//
// A system whose grid is a single cell is searched by brute force over the images of its points, and the order of
// the list is then the order of three nested loops: for a first point i, the second points j in index order and,
// for every j, the images in the lexicographic order of their cell shift q = (qx, qy, qz). The shift of the row is
// S = q - wrap_j + wrap_i (the wraps: box vectors the points were moved by to land inside the box), which for a
// given i and j differs from q by a constant: ascending q is ascending S.
//
// One workgroup per system. Its points go to LDS by their index in the system, the images that can hold a
// neighbour (the stencil of the single cell less the entries stencil_entry_too_far drops) to a table in LDS with
// their Cartesian shift.
//   COUNT  lanes hold second points j, a wave takes two first points i at a time and walks the images: (r_j - r_i)
//          is computed once per pair of points and the shift of an image is the same for every lane, so that one
//          test is 3 additions, the 5 operations of the squared norm and a comparison on all 64 lanes. Every pair
//          (i, j) keeps a bit per image, 64 images to a word, in memory; the bits set over all j are the rows of i.
//   A scan over the points of all systems gives every point its first row.
//   WRITE  reads the words of a first point, lane j those of (i, j): the bits set before a lane's own (a prefix sum
//          over the lanes) are the rows before those of j. Every lane walks its bits and leaves (j, image) in LDS
//          at the place of the row; the 64 lanes then take consecutive rows from there, compute shift, vector and
//          distance and store them: consecutive rows.
// Nothing here limits the rows of a point or the size of the shifts. Systems of more than one cell, of more than
// IMAGE_MAX_POINTS points or with more than IMAGE_MAX_ENTRIES stencil entries are left to the other searches.
//
// Arithmetic as everywhere (vesin/src/cpu_cell_list.cpp:135-138, vesin/src/types.hpp:232-243): T = S . H left to
// right, v = (r_j - r_i) + T, d2 = vx*vx + vy*vy + vz*vz, keep iff d2 < cutoff^2. A point is no neighbour of itself;
// a half list keeps i < j and, of a point with its own image, the shift the reference's rule keeps
// (vesin/src/cpu_cell_list.cpp:101-133). Order of the rows: vesin/include/vesin.h:55-57,
// vesin/src/cpu_cell_list.cpp:634-730.
#ifndef VESIN_HIP_IMAGES_CUH
#define VESIN_HIP_IMAGES_CUH

#include "ordered.cuh"
#include "search.cuh"

namespace vesin_hip {

// (IMAGE_MAX_POINTS, IMAGE_MAX_ENTRIES and images_cover, which say what systems this search covers: ordered.cuh)
constexpr uint32_t IMAGE_MAX_WORDS = IMAGE_MAX_ENTRIES / 64;
constexpr int IMAGE_WAVES = 4;
constexpr int IMAGE_BLOCK = IMAGE_WAVES * WAVE;
// Batches whose systems all have at most IMAGE_FEW_POINTS points give every system one wave instead of one workgroup
// (four systems per workgroup, each with its own part of the LDS; the kernels' FEW variants): three of the four waves
// of a workgroup would have nothing to do, and tens of thousands of small molecules are a common batch.
constexpr uint32_t IMAGE_FEW_POINTS = 32;
constexpr int IMAGE_GROUP = 2;             // units of 64 pairs of points a wave tests together
constexpr uint32_t IMAGE_ROWS = 8 * WAVE;  // rows that a wave lines up in LDS at a time (and up to 63 left over)
static_assert(IMAGE_MAX_POINTS <= 256 && IMAGE_MAX_ENTRIES <= 256, "a row is lined up as (first point << 16) | (second point << 8) | image");

/// Words of 64 images that a pair of points of this system keeps (an upper bound: before the stencil is pruned).
__host__ __device__ inline uint32_t image_words(const GridParams& g) {
    const uint32_t n_stencil = static_cast<uint32_t>(2 * g.s[0] + 1) * static_cast<uint32_t>(2 * g.s[1] + 1) *
                               static_cast<uint32_t>(2 * g.s[2] + 1);
    return (n_stencil + 63) / 64;
}

struct ImageArgs {
    SortedPoints sorted;
    const uint64_t* cell_scan;  // of the concatenated grids: points before every cell in the low 32 bits
    const GridParams* grids;    // one per system
    const uint32_t* cell_base;  // first cell of every system
    const uint32_t* first_point;// first point of every system, n_systems + 1 entries
    const uint64_t* pair_base;  // pairs of points (n^2 per system of at most IMAGE_MAX_POINTS points) before every system
    uint64_t* hits;             // COUNT -> WRITE: [pair_base + i * n + j][words]: the images of j that are neighbours of i
    uint32_t words;             // words of 64 images per pair (1 or 2), the same for every system of the batch
    double cutoff;              // COUNT: for the thresholds of the single-precision pre-test (choose_prefilter)
    uint32_t double_only;       // COUNT: not zero: every pair is tested in double precision (for tests)
    uint32_t n_systems;
    uint32_t total_points;
    uint32_t* rows_of_point;    // COUNT: [total_points], by first point of the system + index
    const uint64_t* first_row;  // WRITE: [total_points + 1], exclusive scan of rows_of_point
    uint32_t others_covered;    // systems this search does not cover are another kernel's: they are not reported
    OrderedStatus* status;      // `unsuitable` counts the systems this search does not cover
    uint32_t guarded;           // WRITE launched before the host has seen what COUNT found: write nothing unless every
                                // system suited its search and the rows fit the `capacity` of the arrays
    uint64_t capacity;
    SearchOutputs out;
    OrderedHostStatus* publish_to; // WRITE: when not null, the first workgroup hands the host what COUNT found
    const DeviceStatus* build_status;
};

template <uint32_t POINTS>
struct ImageShared {
    double x[POINTS], y[POINTS], z[POINTS]; // by index in the system
    int32_t wx[POINTS], wy[POINTS], wz[POINTS];
    double tx[IMAGE_MAX_ENTRIES], ty[IMAGE_MAX_ENTRIES], tz[IMAGE_MAX_ENTRIES]; // q . H of every image kept
    int32_t q[IMAGE_MAX_ENTRIES]; // packed cell shift of every image kept
    uint32_t n_entries;
    uint32_t moved_apart; // not zero: some points were moved into the box by other box vectors than the first one
};

template <uint32_t POINTS>
struct ImageCountShared: ImageShared<POINTS> {
    uint64_t with_itself[IMAGE_MAX_WORDS]; // the images of a point that may be its own neighbours
    uint32_t rows[POINTS];                 // rows of every point
    // The single-precision pre-test (choose_prefilter, geometry.hpp), in the form it takes for one cell: where the
    // points are after they were moved into the box, seen from one of them (r - w . H - the same of the first point:
    // within the extent of the box along every axis, or not a number), and the shifts of the images, rounded once.
    // v = (r_j - r_i) + (q - w_j + w_i) . H = (u_j - u_i) + q . H whatever the wraps are.
    float ux[POINTS], uy[POINTS], uz[POINTS];
    float sx[IMAGE_MAX_ENTRIES], sy[IMAGE_MAX_ENTRIES], sz[IMAGE_MAX_ENTRIES];
    uint32_t use32;
    float lo32, hi32;
};

/// STAGED: with room to line up the vectors of 64 rows per wave (the kernels of calls that return vectors).
template <uint32_t POINTS, int WAVES, bool STAGED>
struct ImageWriteShared: ImageShared<POINTS> {
    // (first point << 16) | (second point << 8) | image, at the place of the row: what a run of consecutive rows left
    // short of a multiple of 64, and the rows of the points behind it
    uint32_t rows[WAVES][IMAGE_ROWS + WAVE];
    // the vectors of 64 consecutive rows on their way to memory (store_vector_block), per wave
    __attribute__((aligned(16))) double vector_stage[WAVES][STAGED ? 3 * WAVE : 2];
};

/// The system's points by index, and the images that can hold a neighbour in the order of their cell shift.
/// FEW: the system is one wave's (`wave` is 0 then), not a workgroup's.
template <bool COUNT, bool FULL, bool FEW, uint32_t POINTS, typename Shared>
__device__ __forceinline__ void stage_system(
    Shared& sh, const ImageArgs& args, const GridParams& g, uint32_t system, uint32_t wave, int lane
) {
    const uint32_t n = g.n_points;
    const uint32_t at0 = static_cast<uint32_t>(args.cell_scan[args.cell_base[system]]);
    const uint32_t thread = FEW ? static_cast<uint32_t>(lane) : threadIdx.x;
    constexpr uint32_t THREADS = FEW ? WAVE : IMAGE_BLOCK;
    auto meet = [&]() {
        if constexpr (FEW) {
            wave_sync();
        } else {
            __syncthreads();
        }
    };
    if (thread == 0) {
        sh.moved_apart = 0;
    }
    meet();
    const int32_t wx0 = args.sorted.wx[at0];
    const int32_t wy0 = args.sorted.wy[at0];
    const int32_t wz0 = args.sorted.wz[at0];
    // COUNT: the first point after it was moved into the box, which the others are seen from, and how far from it a
    // point inside the box can be along every axis (twice that is the bound the thresholds were derived for)
    double seen_from[3] = {0.0, 0.0, 0.0};
    double reach[3] = {0.0, 0.0, 0.0};
    if constexpr (COUNT) {
        if (thread == 0) {
            Prefilter pre;
            choose_prefilter(g, args.cutoff, pre);
            sh.use32 = static_cast<uint32_t>(pre.use32);
            sh.lo32 = pre.lo32;
            sh.hi32 = pre.hi32;
        }
        const SortedPoint first_point = args.sorted.p[at0];
        double mx, my, mz;
        shift_vector(g, wx0, wy0, wz0, mx, my, mz);
        seen_from[0] = first_point.x - mx;
        seen_from[1] = first_point.y - my;
        seen_from[2] = first_point.z - mz;
        for (int d = 0; d < 3; d++) {
            const double scale = g.periodic[d] != 0 ? 1.0 : 1.0 / g.np_scale[d];
            for (int k = 0; k < 3; k++) {
                reach[k] += 2.0 * fabs(g.H[3 * d + k]) * scale;
            }
        }
    }
    for (uint32_t p = thread; p < n; p += THREADS) {
        const SortedPoint point = args.sorted.p[at0 + p];
        const uint32_t index = min(point.index, POINTS - 1);
        const int32_t wx = args.sorted.wx[at0 + p];
        const int32_t wy = args.sorted.wy[at0 + p];
        const int32_t wz = args.sorted.wz[at0 + p];
        sh.x[index] = point.x;
        sh.y[index] = point.y;
        sh.z[index] = point.z;
        sh.wx[index] = wx;
        sh.wy[index] = wy;
        sh.wz[index] = wz;
        if (wx != wx0 || wy != wy0 || wz != wz0) {
            sh.moved_apart = 1;
        }
        if constexpr (COUNT) {
            sh.rows[index] = 0;
            double mx, my, mz;
            shift_vector(g, wx, wy, wz, mx, my, mz);
            const double rx = (point.x - mx) - seen_from[0];
            const double ry = (point.y - my) - seen_from[1];
            const double rz = (point.z - mz) - seen_from[2];
            const bool usable = !beyond(wx, wy, wz, LOCAL_WRAP_LIMIT) && fabs(rx) <= reach[0] && fabs(ry) <= reach[1] &&
                                fabs(rz) <= reach[2];
            sh.ux[index] = usable ? static_cast<float>(rx) : __builtin_nanf("");
            sh.uy[index] = usable ? static_cast<float>(ry) : __builtin_nanf("");
            sh.uz[index] = usable ? static_cast<float>(rz) : __builtin_nanf("");
        }
    }
    if (wave == 0) {
        const int32_t span_y = 2 * g.s[1] + 1;
        const int32_t span_z = 2 * g.s[2] + 1;
        const uint32_t n_stencil = static_cast<uint32_t>(2 * g.s[0] + 1) * span_y * span_z;
        uint32_t kept = 0;
        for (uint32_t e0 = 0; e0 < n_stencil; e0 += WAVE) {
            const uint32_t linear = e0 + lane;
            const int32_t dz = static_cast<int32_t>(linear % span_z) - g.s[2];
            const int32_t dy = static_cast<int32_t>((linear / span_z) % span_y) - g.s[1];
            const int32_t dx = static_cast<int32_t>(linear / (span_z * span_y)) - g.s[0];
            bool valid = linear < n_stencil;
            // (the one cell of a direction that is not periodic has no images along it)
            valid = valid && (g.periodic[0] != 0 || dx == 0) && (g.periodic[1] != 0 || dy == 0) && (g.periodic[2] != 0 || dz == 0);
            valid = valid && !stencil_entry_too_far(g, dx, dy, dz);
            const uint64_t mask = __ballot(valid);
            if (valid) {
                const uint32_t slot = kept + rank_in_mask(mask);
                double tx, ty, tz;
                shift_vector(g, dx, dy, dz, tx, ty, tz);
                sh.q[slot] = pack_shift(dx, dy, dz);
                sh.tx[slot] = tx;
                sh.ty[slot] = ty;
                sh.tz[slot] = tz;
                if constexpr (COUNT) {
                    sh.sx[slot] = static_cast<float>(tx);
                    sh.sy[slot] = static_cast<float>(ty);
                    sh.sz[slot] = static_cast<float>(tz);
                }
            }
            kept += __popcll(mask);
        }
        if (lane == 0) {
            sh.n_entries = kept;
        }
        if constexpr (COUNT) {
            wave_sync();
            // a point is no neighbour of itself, only of its images; a half list keeps one of an image and its
            // opposite (the total shift of such a pair is the cell shift, whatever the point was moved by)
            for (uint32_t w = 0; w < IMAGE_MAX_WORDS; w++) {
                const uint32_t e = w * WAVE + lane;
                int32_t qx, qy, qz;
                unpack_shift(sh.q[min(e, IMAGE_MAX_ENTRIES - 1)], qx, qy, qz);
                const bool allowed = e < kept && (qx | qy | qz) != 0 && (FULL || half_keeps_self_image(qx, qy, qz));
                const uint64_t word = __ballot(allowed);
                if (lane == 0) {
                    sh.with_itself[w] = word;
                }
            }
        }
    }
    meet();
}

/// The images of i seen from j, from the images of j seen from i: image e of the `n_entries` becomes image
/// n_entries - 1 - e (the opposite cell shift: the table is in lexicographic order, and an entry is kept or dropped
/// together with its opposite).
__device__ __forceinline__ void opposite_images(uint64_t lo, uint64_t hi, uint32_t n_entries, uint64_t& back_lo, uint64_t& back_hi) {
    if (n_entries <= 64) {
        back_lo = __brevll(lo) >> (64 - n_entries);
        back_hi = 0;
    } else {
        const uint64_t upper = __brevll(lo);
        const uint64_t lower = __brevll(hi);
        const uint32_t down = 128 - n_entries; // 0 .. 63
        back_lo = down == 0 ? lower : (lower >> down) | (upper << (64 - down));
        back_hi = upper >> down;
    }
}

/// COUNT: one workgroup per system. A test decides two rows at once: image q of j is a neighbour of i exactly when
/// image -q of i is a neighbour of j (the same numbers with the opposite sign all the way, the same squared norm),
/// so only the pairs of points with i <= j are tested, 64 pairs to a wave's lanes.
template <bool FULL, bool FEW>
__global__ __launch_bounds__(IMAGE_BLOCK) void image_count_kernel(ImageArgs args) {
    constexpr uint32_t POINTS = FEW ? IMAGE_FEW_POINTS : IMAGE_MAX_POINTS;
    constexpr uint32_t WAVES = FEW ? 1 : IMAGE_WAVES;          // of a system
    constexpr uint32_t THREADS = FEW ? WAVE : IMAGE_BLOCK;
    __shared__ ImageCountShared<POINTS> shared[FEW ? IMAGE_WAVES : 1];
    const int lane = lane_id();
    const uint32_t wave_of_block = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t wave = FEW ? 0 : wave_of_block;              // within its system
    const uint32_t thread = FEW ? static_cast<uint32_t>(lane) : threadIdx.x;
    ImageCountShared<POINTS>& sh = shared[FEW ? wave_of_block : 0];
    const uint32_t system = FEW ? blockIdx.x * IMAGE_WAVES + wave_of_block : blockIdx.x;
    if (system >= args.n_systems) {
        return;
    }
    const GridParams g = args.grids[system];
    const uint32_t n = g.n_points;
    if (n == 0) {
        return;
    }
    if (!images_cover(g) || image_words(g) > args.words || n > POINTS) {
        if (thread == 0 && args.others_covered == 0) {
            atomicAdd(&args.status->unsuitable, 1u);
        }
        return;
    }
    stage_system<true, FULL, FEW, POINTS>(sh, args, g, system, wave, lane);
    const uint32_t n_entries = uniform(sh.n_entries);
    const bool use32 = uniform(sh.use32) != 0 && args.double_only == 0;
    const float lo32 = sh.lo32;
    const float hi32 = sh.hi32;
    const uint32_t first = args.first_point[system];
    const uint32_t words = args.words;
    uint64_t* system_hits = args.hits + args.pair_base[system] * words;

    // The pairs i <= j: row r of the triangle (n - r pairs) and row n - 1 - r (r + 1 pairs) make one line of n + 1
    // pairs; the lines one after the other are dealt to the lanes. (An odd n leaves the middle row a line of its own.)
    const uint32_t width = n + 1;
    const uint32_t n_lines = (n + 1) / 2;
    const uint32_t n_lanes = n_lines * width;
    for (uint32_t unit0 = wave * IMAGE_GROUP; unit0 * WAVE < n_lanes; unit0 += WAVES * IMAGE_GROUP) {
        uint32_t pi[IMAGE_GROUP], pj[IMAGE_GROUP];
        bool there[IMAGE_GROUP];
        double ax[IMAGE_GROUP], ay[IMAGE_GROUP], az[IMAGE_GROUP];
        int32_t bx[IMAGE_GROUP], by[IMAGE_GROUP], bz[IMAGE_GROUP]; // what the wraps add to the cell shift
        bool moved_alike = true;
#pragma unroll
        for (int u = 0; u < IMAGE_GROUP; u++) {
            const uint32_t at = (unit0 + u) * WAVE + lane;
            const uint32_t line = at / width;
            const uint32_t along = at - line * width;
            const bool upper = along < n - line;
            const uint32_t i = upper ? line : n - 1 - line;
            const uint32_t j = upper ? line + along : i + (along - (n - line));
            there[u] = at < n_lanes && (upper || 2 * line != n - 1);
            pi[u] = there[u] ? i : 0;
            pj[u] = there[u] ? j : 0;
            ax[u] = sh.x[pj[u]] - sh.x[pi[u]];
            ay[u] = sh.y[pj[u]] - sh.y[pi[u]];
            az[u] = sh.z[pj[u]] - sh.z[pi[u]];
            bx[u] = sh.wx[pi[u]] - sh.wx[pj[u]];
            by[u] = sh.wy[pi[u]] - sh.wy[pj[u]];
            bz[u] = sh.wz[pi[u]] - sh.wz[pj[u]];
            moved_alike = moved_alike && __ballot((bx[u] | by[u] | bz[u]) != 0) == 0;
        }
        // (a word of 64 images in two halves: the bits of a half are gathered in one register)
        uint32_t found[2 * IMAGE_MAX_WORDS][IMAGE_GROUP];
        if (use32) {
            // ---- single precision first: a squared distance below lo32 is within the cutoff, one above hi32 is not
            // (choose_prefilter); what lies in between, and every image of a pair with a point that has no place, is
            // decided below by the reference's own arithmetic
            float fx[IMAGE_GROUP], fy[IMAGE_GROUP], fz[IMAGE_GROUP];
            uint32_t maybe[2 * IMAGE_MAX_WORDS][IMAGE_GROUP];
#pragma unroll
            for (int u = 0; u < IMAGE_GROUP; u++) {
                fx[u] = sh.ux[pj[u]] - sh.ux[pi[u]];
                fy[u] = sh.uy[pj[u]] - sh.uy[pi[u]];
                fz[u] = sh.uz[pj[u]] - sh.uz[pi[u]];
            }
#pragma unroll
            for (int h = 0; h < 2 * static_cast<int>(IMAGE_MAX_WORDS); h++) {
#pragma unroll
                for (int u = 0; u < IMAGE_GROUP; u++) {
                    found[h][u] = 0;
                    maybe[h][u] = 0;
                }
                const uint32_t e_begin = h * 32;
                const uint32_t e_end = min(n_entries, e_begin + 32);
                for (uint32_t e = e_begin; e < e_end; e++) {
                    const float tx = sh.sx[e];
                    const float ty = sh.sy[e];
                    const float tz = sh.sz[e];
                    const uint32_t bit = 1u << (e % 32);
#pragma unroll
                    for (int u = 0; u < IMAGE_GROUP; u++) {
                        const float vx = fx[u] + tx;
                        const float vy = fy[u] + ty;
                        const float vz = fz[u] + tz;
                        const float d2 = __builtin_fmaf(vz, vz, __builtin_fmaf(vy, vy, vx * vx));
                        found[h][u] |= d2 < lo32 ? bit : 0u;
                        maybe[h][u] |= d2 < hi32 ? bit : 0u;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < IMAGE_GROUP; u++) {
                const bool unknown = !(fx[u] == fx[u]) || !(fy[u] == fy[u]) || !(fz[u] == fz[u]);
#pragma unroll
                for (int h = 0; h < 2 * static_cast<int>(IMAGE_MAX_WORDS); h++) {
                    const uint32_t in_table = n_entries >= (h + 1) * 32u ? ~0u : n_entries > h * 32u ? (1u << (n_entries - h * 32u)) - 1u : 0u;
                    uint32_t open = unknown ? in_table : (maybe[h][u] & ~found[h][u]);
                    uint32_t decided = unknown ? 0u : found[h][u];
                    while (__ballot(open != 0) != 0) {
                        if (open != 0) {
                            const uint32_t at_bit = static_cast<uint32_t>(__builtin_ctz(open));
                            open &= open - 1;
                            int32_t qx, qy, qz;
                            unpack_shift(sh.q[h * 32 + at_bit], qx, qy, qz);
                            double tx, ty, tz;
                            shift_vector(g, qx + bx[u], qy + by[u], qz + bz[u], tx, ty, tz);
                            const double vx = ax[u] + tx;
                            const double vy = ay[u] + ty;
                            const double vz = az[u] + tz;
                            const double d2 = vx * vx + vy * vy + vz * vz;
                            decided = d2 < g.cutoff2 ? decided | (1u << at_bit) : decided & ~(1u << at_bit);
                        }
                    }
                    found[h][u] = decided;
                }
            }
        } else {
        #pragma unroll
            for (int h = 0; h < 2 * static_cast<int>(IMAGE_MAX_WORDS); h++) {
    #pragma unroll
                for (int u = 0; u < IMAGE_GROUP; u++) {
                    found[h][u] = 0;
                }
                const uint32_t e_begin = h * 32;
                const uint32_t e_end = min(n_entries, e_begin + 32);
                if (moved_alike) {
                    // the shift of the row is the cell shift of the image: the same vector for every lane
                    for (uint32_t e = e_begin; e < e_end; e++) {
                        const double tx = sh.tx[e];
                        const double ty = sh.ty[e];
                        const double tz = sh.tz[e];
                        const uint32_t bit = 1u << (e % 32);
    #pragma unroll
                        for (int u = 0; u < IMAGE_GROUP; u++) {
                            const double vx = ax[u] + tx;
                            const double vy = ay[u] + ty;
                            const double vz = az[u] + tz;
                            const double d2 = vx * vx + vy * vy + vz * vz;
                            found[h][u] |= d2 < g.cutoff2 ? bit : 0u;
                        }
                    }
                } else {
                    for (uint32_t e = e_begin; e < e_end; e++) {
                        int32_t qx, qy, qz;
                        unpack_shift(sh.q[e], qx, qy, qz);
                        const uint32_t bit = 1u << (e % 32);
    #pragma unroll
                        for (int u = 0; u < IMAGE_GROUP; u++) {
                            double tx, ty, tz;
                            shift_vector(g, qx + bx[u], qy + by[u], qz + bz[u], tx, ty, tz);
                            const double vx = ax[u] + tx;
                            const double vy = ay[u] + ty;
                            const double vz = az[u] + tz;
                            const double d2 = vx * vx + vy * vy + vz * vz;
                            found[h][u] |= d2 < g.cutoff2 ? bit : 0u;
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < IMAGE_GROUP; u++) {
            uint64_t lo = found[0][u] | (static_cast<uint64_t>(found[1][u]) << 32);
            uint64_t hi = found[2][u] | (static_cast<uint64_t>(found[3][u]) << 32);
            const uint32_t i = pi[u];
            const uint32_t j = pj[u];
            if (i == j) {
                lo &= sh.with_itself[0];
                hi &= sh.with_itself[1];
            }
            if (there[u]) {
                const uint32_t n_rows = __popcll(lo) + __popcll(hi);
                uint64_t* forth = system_hits + (static_cast<size_t>(i) * n + j) * words;
                forth[0] = lo;
                if (words > 1) {
                    forth[1] = hi;
                }
                if (n_rows != 0) {
                    atomicAdd(&sh.rows[i], n_rows);
                }
                if (FULL && i != j) {
                    uint64_t back_lo, back_hi;
                    opposite_images(lo, hi, n_entries, back_lo, back_hi);
                    uint64_t* back = system_hits + (static_cast<size_t>(j) * n + i) * words;
                    back[0] = back_lo;
                    if (words > 1) {
                        back[1] = back_hi;
                    }
                    if (n_rows != 0) {
                        atomicAdd(&sh.rows[j], n_rows);
                    }
                }
            }
        }
    }
    if constexpr (FEW) {
        wave_sync();
    } else {
        __syncthreads();
    }
    for (uint32_t p = thread; p < n; p += THREADS) {
        args.rows_of_point[first + p] = sh.rows[p];
    }
}

/// Stores the first `count` rows lined up in `rows` as the rows `first_row` ... of the list: 64 consecutive rows per
/// step, each step ending on a multiple of 64 rows (whole cache lines in every output array; the first step stores
/// fewer).
template <bool STAGED, typename Shared>
__device__ __forceinline__ void store_image_rows(
    const Shared& sh, const uint32_t* rows, double* vector_stage, const GridParams& g, const SearchOutputs& out,
    bool moved_apart, uint32_t count, uint64_t first_row, int lane
) {
    const uint32_t skew = static_cast<uint32_t>(first_row % WAVE);
    for (uint32_t r0 = 0; r0 < count + skew; r0 += WAVE) {
        const uint32_t r = r0 + lane - skew;
        const bool active = r < count; // (false before the first row as well: unsigned)
        double vx = 0.0, vy = 0.0, vz = 0.0;
        if (active) {
            const uint32_t ticket = rows[r];
            const uint32_t i = ticket >> 16;
            const uint32_t j = (ticket >> 8) & 0xffu;
            const uint32_t e = ticket & 0xffu;
            int32_t sx, sy, sz;
            unpack_shift(sh.q[e], sx, sy, sz);
            double tx = sh.tx[e];
            double ty = sh.ty[e];
            double tz = sh.tz[e];
            if (moved_apart) {
                sx += sh.wx[i] - sh.wx[j];
                sy += sh.wy[i] - sh.wy[j];
                sz += sh.wz[i] - sh.wz[j];
                shift_vector(g, sx, sy, sz, tx, ty, tz);
            }
            vx = (sh.x[j] - sh.x[i]) + tx;
            vy = (sh.y[j] - sh.y[i]) + ty;
            vz = (sh.z[j] - sh.z[i]) + tz;
            const uint64_t row = first_row + r;
            stream_store(out.pairs + 2 * row, PairRow{i, j});
            if (out.shifts != nullptr) {
                stream_store(out.shifts + 3 * row, ShiftRow{sx, sy, sz});
            }
            if (out.distances != nullptr) {
                stream_store(out.distances + row, sqrt(vx * vx + vy * vy + vz * vz));
            }
            if (!STAGED && out.vectors != nullptr) {
                stream_store(out.vectors + 3 * row, VectorHead{vx, vy});
                stream_store(out.vectors + 3 * row + 2, vz);
            }
        }
        if (STAGED && out.vectors != nullptr) {
            // the block of 64 rows this step falls into, and its lanes that hold a row
            const uint64_t block_row = first_row + r0 - skew;
            const uint32_t lo = r0 == 0 ? skew : 0u;
            const uint32_t hi = min(static_cast<uint32_t>(WAVE), count + skew - r0);
            store_vector_block(
                vector_stage, reinterpret_cast<char*>(out.vectors + 3 * block_row), lo, hi, active,
                static_cast<uint32_t>(lane), vx, vy, vz
            );
        }
    }
}

/// WRITE: one workgroup per system, every wave a run of consecutive first points: their rows are consecutive rows of
/// the list, lined up in LDS one point after the other and stored whenever they reach a multiple of 64 rows.
/// STAGED: for calls that return vectors, which are lined up in LDS before they are stored (store_vector_block).
template <bool FULL, bool FEW, bool STAGED = false>
__global__ __launch_bounds__(IMAGE_BLOCK) void image_write_kernel(ImageArgs args) {
    constexpr uint32_t POINTS = FEW ? IMAGE_FEW_POINTS : IMAGE_MAX_POINTS;
    constexpr uint32_t WAVES = FEW ? 1 : IMAGE_WAVES; // of a system
    __shared__ ImageWriteShared<POINTS, WAVES, STAGED> shared[FEW ? IMAGE_WAVES : 1];
    const int lane = lane_id();
    const uint32_t wave_of_block = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t wave = FEW ? 0 : wave_of_block;    // within its system
    ImageWriteShared<POINTS, WAVES, STAGED>& sh = shared[FEW ? wave_of_block : 0];
    if (args.publish_to != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
        OrderedHostStatus report;
        report.found = *args.status;
        report.total_rows = args.first_row[args.total_points];
        report.first_bad_coordinate = args.build_status->first_bad_coordinate;
        report.n_tiles = 0;
        *args.publish_to = report;
    }
    if (args.guarded != 0) {
        // (the same decision as the writing pass over tiles, which may serve other systems of the batch)
        const OrderedStatus found = *args.status;
        const bool usable = found.unsuitable == 0 && found.max_rows <= ORDERED_MAX_ROWS &&
                            found.max_candidates <= ORDERED_CANDIDATES && args.first_row[args.total_points] <= args.capacity;
        if (!usable) {
            return;
        }
    }
    const uint32_t system = FEW ? blockIdx.x * IMAGE_WAVES + wave_of_block : blockIdx.x;
    if (system >= args.n_systems) {
        return;
    }
    const GridParams g = args.grids[system];
    const uint32_t n = g.n_points;
    if (n == 0 || !images_cover(g) || image_words(g) > args.words || n > POINTS) {
        return;
    }
    stage_system<false, FULL, FEW, POINTS>(sh, args, g, system, wave, lane);
    const bool moved_apart = uniform(sh.moved_apart) != 0;
    const uint32_t first = args.first_point[system];
    const uint32_t words = args.words;
    const uint64_t* system_hits = args.hits + args.pair_base[system] * words;
    uint32_t* rows = sh.rows[wave];
    double* vector_stage = sh.vector_stage[wave];
    const SearchOutputs& out = args.out;

    const uint32_t per_wave = (n + WAVES - 1) / WAVES;
    const uint32_t i_begin = wave * per_wave;
    const uint32_t i_end = min(n, i_begin + per_wave);
    if (i_begin >= i_end) {
        return;
    }
    uint64_t staged_row = uniform(args.first_row[first + i_begin]); // row of the list of the first row lined up
    uint32_t staged = 0;                                            // rows lined up
    uint64_t next_first = staged_row;
    for (uint32_t i = i_begin; i < i_end; i++) {
        const uint64_t first_row = next_first;
        next_first = uniform(args.first_row[first + i + 1]);
        const uint32_t n_rows = static_cast<uint32_t>(next_first - first_row);
        const uint64_t* hits_of_i = system_hits + static_cast<size_t>(i) * n * words;
        uint32_t done = 0; // rows of this point that are lined up or stored
        while (done < n_rows) {
            // as many rows of the point as there is room for (all of them, for all but the largest numbers of
            // neighbours): the rows [done, done + take) go behind the rows that wait
            const uint32_t take = min(IMAGE_ROWS + WAVE - staged, n_rows - done);
            uint32_t before = 0; // rows of the second points of earlier lanes
            for (uint32_t j0 = 0; j0 < n && before < done + take; j0 += WAVE) {
                const uint32_t j = j0 + lane;
                // (a half list: the second points before i have no rows, and the counting pass left no words for them)
                const bool there = j < n && (FULL || j >= i);
                uint64_t lo = 0, hi = 0;
                if (there) {
                    lo = hits_of_i[static_cast<size_t>(j) * words];
                    if (words > 1) {
                        hi = hits_of_i[static_cast<size_t>(j) * words + 1];
                    }
                }
                const uint32_t own = __popcll(lo) + __popcll(hi);
                const uint32_t through = wave_inclusive_scan(own);
                uint32_t place = before + through - own - done; // (rows before `done`: far beyond `take`, unsigned)
                before += read_lane(through, WAVE - 1);
                if (before <= done) {
                    continue; // the rows of these second points went out earlier
                }
                const uint32_t ticket = (i << 16) | (j << 8);
                while (__ballot(lo != 0) != 0) {
                    if (lo != 0) {
                        const uint32_t e = static_cast<uint32_t>(__builtin_ctzll(lo));
                        lo &= lo - 1;
                        if (place < take) {
                            rows[staged + place] = ticket | e;
                        }
                        place += 1;
                    }
                }
                while (__ballot(hi != 0) != 0) {
                    if (hi != 0) {
                        const uint32_t e = 64 + static_cast<uint32_t>(__builtin_ctzll(hi));
                        hi &= hi - 1;
                        if (place < take) {
                            rows[staged + place] = ticket | e;
                        }
                        place += 1;
                    }
                }
            }
            staged += take;
            done += take;
            wave_sync();
            const uint64_t whole = (staged_row + staged) & ~static_cast<uint64_t>(WAVE - 1);
            if (whole > staged_row) {
                // everything up to the last multiple of 64 rows; what is left moves to the front
                const uint32_t count = static_cast<uint32_t>(whole - staged_row);
                store_image_rows<STAGED>(sh, rows, vector_stage, g, out, moved_apart, count, staged_row, lane);
                const uint32_t left = staged - count; // < 64
                const uint32_t ticket = rows[min(count + lane, IMAGE_ROWS + WAVE - 1)];
                wave_sync();
                if (static_cast<uint32_t>(lane) < left) {
                    rows[lane] = ticket;
                }
                staged_row = whole;
                staged = left;
                wave_sync();
            }
        }
    }
    if (staged != 0) {
        store_image_rows<STAGED>(sh, rows, vector_stage, g, out, moved_apart, staged, staged_row, lane);
    }
}

/// first_pair[s] = first row of system s (the first row of its first point), first_pair[n_systems] = all rows.
__global__ void first_rows_of_systems_kernel(
    const uint64_t* __restrict__ first_row, const uint32_t* __restrict__ first_point, uint32_t n_systems,
    unsigned long long* __restrict__ first_pair
) {
    const uint32_t s = blockIdx.x * BLOCK + threadIdx.x;
    if (s <= n_systems) {
        first_pair[s] = first_row[first_point[s]];
    }
}

} // namespace vesin_hip

#endif
