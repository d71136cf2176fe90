// Host-side box normalisation and grid selection for the HIP neighbor-list path.
//
// The box handling reproduces the semantics of the reference's BoundingBox (vesin/src/types.hpp:20-97): rows
// of non-periodic directions are replaced by unit vectors orthogonal to the periodic ones, the box must be
// invertible (|det| >= 1e-30), and the distance between opposite faces bounds how many cells fit per direction.
// The operation order follows the reference so that the rows used for the shift vectors (T = S . H) carry the
// same bits; this file must be compiled with -ffp-contract=off.
//
// The grid itself is this library's own choice (the pair set does not depend on it): cells are at least
// cutoff * (1 + 1e-9) wide so that rounding in the cell assignment can never push a pair outside the stencil,
// non-periodic directions are binned along the replaced (orthogonal) box rows, and the total number of cells
// scales with the number of points.
#ifndef VESIN_HIP_GEOMETRY_HPP
#define VESIN_HIP_GEOMETRY_HPP

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <stdexcept>

namespace vesin_hip {

struct HostBox {
    double H[3][3];    // normalised box, one vector per row
    double Hinv[3][3]; // inverse of H: fractional = cartesian (row vector) * Hinv
    double face[3];    // distance between opposite faces (periodic directions only)
    bool periodic[3];
};

namespace detail {
    struct V3 {
        double x, y, z;
    };

    inline double dot(V3 a, V3 b) {
        return a.x * b.x + a.y * b.y + a.z * b.z;
    }

    inline V3 cross(V3 a, V3 b) {
        return V3{a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
    }

    inline V3 unit(V3 a) {
        double s = 1.0 / std::sqrt(dot(a, a));
        return V3{s * a.x, s * a.y, s * a.z};
    }

    inline V3 get_row(const double m[3][3], int i) {
        return V3{m[i][0], m[i][1], m[i][2]};
    }

    inline void put_row(double m[3][3], int i, V3 v) {
        m[i][0] = v.x;
        m[i][1] = v.y;
        m[i][2] = v.z;
    }
} // namespace detail

/// Build the normalised box. Throws std::runtime_error("the box matrix is not invertible") like the reference
/// (types.hpp:75-78).
inline HostBox normalise_box(const double box[9], const bool periodic[3]) {
    using namespace detail;
    HostBox out;
    int n_periodic = 0;
    int first = -1;
    int second = -1;
    for (int d = 0; d < 3; d++) {
        out.periodic[d] = periodic[d];
        for (int e = 0; e < 3; e++) {
            out.H[d][e] = box[3 * d + e];
        }
        if (periodic[d]) {
            n_periodic += 1;
            if (first < 0) {
                first = d;
            } else if (second < 0) {
                second = d;
            }
        }
    }

    if (n_periodic == 0) {
        for (int d = 0; d < 3; d++) {
            for (int e = 0; e < 3; e++) {
                out.H[d][e] = d == e ? 1.0 : 0.0;
            }
        }
    } else if (n_periodic == 1) {
        V3 a = get_row(out.H, first);
        V3 helper{0.0, 1.0, 0.0};
        if (std::abs(dot(unit(a), helper)) > 0.9) {
            helper = V3{0.0, 0.0, 1.0};
        }
        V3 c = unit(cross(a, helper));
        V3 b = unit(cross(c, a));
        put_row(out.H, (first + 1) % 3, b);
        put_row(out.H, (first + 2) % 3, c);
    } else if (n_periodic == 2) {
        V3 c = unit(cross(get_row(out.H, first), get_row(out.H, second)));
        put_row(out.H, 3 - first - second, c);
    }

    const auto& m = out.H;
    double det = m[0][0] * (m[1][1] * m[2][2] - m[2][1] * m[1][2])
               - m[0][1] * (m[1][0] * m[2][2] - m[1][2] * m[2][0])
               + m[0][2] * (m[1][0] * m[2][1] - m[1][1] * m[2][0]);
    if (!(std::abs(det) >= 1e-30)) {
        throw std::runtime_error("the box matrix is not invertible");
    }

    out.Hinv[0][0] = (m[1][1] * m[2][2] - m[2][1] * m[1][2]) / det;
    out.Hinv[0][1] = (m[0][2] * m[2][1] - m[0][1] * m[2][2]) / det;
    out.Hinv[0][2] = (m[0][1] * m[1][2] - m[0][2] * m[1][1]) / det;
    out.Hinv[1][0] = (m[1][2] * m[2][0] - m[1][0] * m[2][2]) / det;
    out.Hinv[1][1] = (m[0][0] * m[2][2] - m[0][2] * m[2][0]) / det;
    out.Hinv[1][2] = (m[1][0] * m[0][2] - m[0][0] * m[1][2]) / det;
    out.Hinv[2][0] = (m[1][0] * m[2][1] - m[2][0] * m[1][1]) / det;
    out.Hinv[2][1] = (m[2][0] * m[0][1] - m[0][0] * m[2][1]) / det;
    out.Hinv[2][2] = (m[0][0] * m[1][1] - m[1][0] * m[0][1]) / det;

    V3 a = get_row(out.H, 0);
    V3 b = get_row(out.H, 1);
    V3 c = get_row(out.H, 2);
    out.face[0] = std::abs(dot(unit(cross(b, c)), a));
    out.face[1] = std::abs(dot(unit(cross(c, a)), b));
    out.face[2] = std::abs(dot(unit(cross(a, b)), c));
    return out;
}

struct HostGrid {
    int32_t n[3];          // cells per direction
    int32_t s[3];          // stencil radius per direction (cells searched on each side)
    double np_min[3];      // non-periodic directions: smallest projected coordinate
    double np_scale[3];    // non-periodic directions: 1 / extent
    uint64_t n_cells;
};

constexpr double CELL_MARGIN = 1.0 + 1e-9;
constexpr int32_t MAX_STENCIL_RADIUS = 500;

// this header is read by the host compiler alone (tests) and by hipcc, where some of its functions also run in kernels
#ifdef __HIPCC__
#define VESIN_HOST_DEVICE __host__ __device__
#else
#define VESIN_HOST_DEVICE
#endif

/// Shrinks a grid of cells[0] x cells[1] x cells[2] cells (whole numbers, 1 at least) until it holds at most `most`
/// cells (1 at least), all directions that have more than one cell by the same factor. A direction that the factor
/// takes below one cell keeps one, and the others then shrink again: a long thin system (a stretched chain, a
/// dissociating pair) ends up with cells along its length only. The buffers of the callers are sized by `most`, so
/// the bound holds whatever the rounding of the roots does: the last loop takes single layers off the direction with
/// the most cells.
VESIN_HOST_DEVICE inline void limit_cells(double cells[3], double most) {
    for (int round = 0; round < 3; round++) {
        const double total = cells[0] * cells[1] * cells[2];
        if (total <= most) {
            return;
        }
        int wide = 0;
        for (int d = 0; d < 3; d++) {
            wide += cells[d] > 1.0 ? 1 : 0;
        }
        const double ratio = most / total;
        const double shrink = wide == 3 ? ::cbrt(ratio) : wide == 2 ? ::sqrt(ratio) : ratio;
        for (int d = 0; d < 3; d++) {
            if (cells[d] > 1.0) {
                cells[d] = ::fmax(::floor(cells[d] * shrink), 1.0);
            }
        }
    }
    while (cells[0] * cells[1] * cells[2] > most) {
        const int widest = cells[0] >= cells[1] ? (cells[0] >= cells[2] ? 0 : 2) : (cells[1] >= cells[2] ? 1 : 2);
        if (!(cells[widest] > 1.0)) {
            return;
        }
        cells[widest] -= 1.0;
    }
}

/// Choose the cell grid. `lo`/`hi` are the extrema of the fractional (projected) coordinates; they are only read
/// for non-periodic directions. With `single_cell` every point goes to one cell and the stencil enumerates the
/// periodic images directly (the brute-force and multi-image path).
inline HostGrid choose_grid(
    const HostBox& box, double cutoff, size_t n_points, const double lo[3], const double hi[3], bool single_cell
) {
    HostGrid grid;
    double extent[3];
    double cells[3];
    const double padded = cutoff * CELL_MARGIN;

    for (int d = 0; d < 3; d++) {
        if (box.periodic[d]) {
            extent[d] = box.face[d];
            grid.np_min[d] = 0.0;
            grid.np_scale[d] = 1.0;
        } else {
            // the replaced rows are unit vectors, so the projected coordinate is a length; add the same 1% margin
            // and 1.0 floor as the reference (types.hpp:180-198) so that every point is strictly inside
            double width = n_points > 0 ? hi[d] - lo[d] : 0.0;
            if (!(width >= 1e-6)) {
                width = 1.0;
            }
            extent[d] = width * 1.01;
            if (extent[d] < 1.0) {
                extent[d] = 1.0;
            }
            grid.np_min[d] = n_points > 0 ? lo[d] : 0.0;
            grid.np_scale[d] = 1.0 / extent[d];
        }

        cells[d] = std::floor(extent[d] / padded);
        if (!(cells[d] >= 1.0)) {
            cells[d] = 1.0;
        }
        if (cells[d] > 1048576.0) {
            cells[d] = 1048576.0;
        }
        if (single_cell) {
            cells[d] = 1.0;
        }
    }

    // keep the number of cells proportional to the number of points
    double max_cells = 2.0 * static_cast<double>(n_points);
    if (max_cells < 64.0) {
        max_cells = 64.0;
    }
    if (max_cells > 16777216.0) {
        max_cells = 16777216.0;
    }
    limit_cells(cells, max_cells);

    grid.n_cells = 1;
    for (int d = 0; d < 3; d++) {
        grid.n[d] = static_cast<int32_t>(cells[d]);
        grid.n_cells *= static_cast<uint64_t>(grid.n[d]);

        double radius = std::ceil(padded * cells[d] / extent[d]);
        if (!(radius >= 1.0)) {
            radius = 1.0;
        }
        if (!box.periodic[d]) {
            // nothing exists beyond the last cell of a non-periodic direction
            if (radius > cells[d] - 1.0) {
                radius = cells[d] - 1.0;
            }
        }
        if (radius > static_cast<double>(MAX_STENCIL_RADIUS)) {
            throw std::runtime_error(
                "cutoff is too large for this box: more than 500 periodic images would be needed in one direction"
            );
        }
        grid.s[d] = static_cast<int32_t>(radius);
    }
    return grid;
}

/// Whether the stencil entry (dx, dy, dz) is too far from the centre cell to hold a neighbour, from the fields
/// `choose_pruning` fills (GridParams::prune_edges).
template <typename Grid>
VESIN_HOST_DEVICE inline bool stencil_entry_too_far(const Grid& g, int32_t dx, int32_t dy, int32_t dz) {
    if (g.prune == 0) {
        return false;
    }
    const double fx = static_cast<double>(dx);
    const double fy = static_cast<double>(dy);
    const double fz = static_cast<double>(dz);
    const double ax =
        ::fmax(::fabs(fx * g.prune_edges[0] + fy * g.prune_edges[1] + fz * g.prune_edges[2]) - g.prune_slack[0], 0.0);
    const double ay = ::fmax(::fabs(fy * g.prune_edges[3] + fz * g.prune_edges[4]) - g.prune_slack[1], 0.0);
    const double az = ::fmax(::fabs(fz * g.prune_edges[5]) - g.prune_slack[2], 0.0);
    return ax * ax + ay * ay + az * az > g.prune_limit;
}

/// Which stencil entries can be dropped (see GridParams::prune_edges). Only when some direction has a stencil radius
/// of two or more: with radius one every cell of the stencil touches the centre cell. The slack carries a millionth
/// of a cell for the rounding of the fractional coordinates that put the points into their cells.
template <typename Grid>
inline void choose_pruning(const HostBox& box, const HostGrid& grid, double cutoff, Grid& g) {
    using namespace detail;
    g.prune = 0;
    g.prune_limit = cutoff * cutoff * CELL_MARGIN * CELL_MARGIN;
    for (int k = 0; k < 6; k++) {
        g.prune_edges[k] = 0.0;
    }
    for (int d = 0; d < 3; d++) {
        g.prune_slack[d] = 0.0;
    }
    if (grid.s[0] < 2 && grid.s[1] < 2 && grid.s[2] < 2) {
        return;
    }
    // edge vectors of one cell: a non-periodic row of the box is a unit vector, its cells divide the extent of the
    // points along it
    V3 edge[3];
    for (int d = 0; d < 3; d++) {
        const double scale = (box.periodic[d] ? 1.0 : 1.0 / grid.np_scale[d]) / static_cast<double>(grid.n[d]);
        const V3 row = get_row(box.H, d);
        edge[d] = V3{row.x * scale, row.y * scale, row.z * scale};
    }
    // orthonormal frame by Gram-Schmidt: q0 along edge 0, q1 in the plane of edges 0 and 1
    const double l00 = std::sqrt(dot(edge[0], edge[0]));
    if (!(l00 > 0.0) || !std::isfinite(l00)) {
        return;
    }
    const V3 q0 = V3{edge[0].x / l00, edge[0].y / l00, edge[0].z / l00};
    const double l10 = dot(edge[1], q0);
    const V3 rest1 = V3{edge[1].x - l10 * q0.x, edge[1].y - l10 * q0.y, edge[1].z - l10 * q0.z};
    const double l11 = std::sqrt(dot(rest1, rest1));
    if (!(l11 > 1e-9 * l00) || !std::isfinite(l11)) {
        return;
    }
    const V3 q1 = V3{rest1.x / l11, rest1.y / l11, rest1.z / l11};
    const double l20 = dot(edge[2], q0);
    const double l21 = dot(edge[2], q1);
    const V3 q2 = cross(q0, q1);
    const double l22 = dot(edge[2], q2);
    if (!(std::abs(l22) > 1e-9 * l00) || !std::isfinite(l22)) {
        return;
    }
    const double margin = 1.0 + 1e-6;
    g.prune_edges[0] = l00;
    g.prune_edges[1] = l10;
    g.prune_edges[2] = l20;
    g.prune_edges[3] = l11;
    g.prune_edges[4] = l21;
    g.prune_edges[5] = l22;
    g.prune_slack[0] = (std::abs(l00) + std::abs(l10) + std::abs(l20)) * margin;
    g.prune_slack[1] = (std::abs(l11) + std::abs(l21)) * margin;
    g.prune_slack[2] = std::abs(l22) * margin;
    g.prune = 1;
}

/// Largest number of box vectors a point may have been moved by (per direction) for its place inside its cell to be
/// kept in single precision (see choose_prefilter); points further out are tested in double precision only.
constexpr int32_t LOCAL_WRAP_LIMIT = 400;

/// The single-precision pre-test of the searches. Every cell-sorted point also carries its place inside its cell
/// as three floats: x_local = (x - w . H) - origin of the cell (w: the box vectors the point was moved by), computed
/// in double precision and rounded once. For a tile point i, a candidate j and the stencil offset (dx, dy, dz)
/// between their cells, the vector the reference tests, v = (r_j - r_i) + S . H, is
///     v = x_local_j + (dx E_0 + dy E_1 + dz E_2) - x_local_i          (E_d: the edge vectors of one cell)
/// whatever the wraps of the two points and the box shift of the entry are (they are what makes the cells
/// neighbours). The searches evaluate that in single precision, |v|^2 = d2_32, and decide
///     d2_32 < lo32: the pair is within the cutoff;   d2_32 > hi32: it is not;
///     otherwise (or when a place is not a number): the reference's own arithmetic in double precision decides,
/// so the result is the reference's bit for bit as long as |d2_32 - fl64(d2)| <= eps for every pair whose true
/// squared distance is at or near the cutoff, with lo32 = cutoff^2 - eps and hi32 = cutoff^2 + eps. The bound:
/// every place satisfies |x_local_k| <= R (R = twice the extent of a cell along the axis, twice because points of an
/// open direction may sit up to one cell outside theirs; places beyond that are stored as NaN), offsets satisfy
/// |offset_k| <= D (the stencil radius times the extent of a cell), each is rounded once (u = 2^-24 relative), the
/// sum x_local_j + offset is rounded, the difference is rounded: every component of v carries at most
/// A = u (3 R + 2 D) + u |v_k| of error, and the three squares and two sums add 3 u |v|^2. With |v| at the cutoff rc
/// that is |d2_32 - d2| <= 2 sqrt(3) rc A + 3 A^2 + 5 u rc^2 (first order in u), which the formula below doubles.
/// The double-precision quantities behind the places (fractional coordinates, cell origins) carry errors of the
/// order of 1e-16 x (box length) x (condition of the box) x (number of boxes the point was moved by): the pre-test is
/// switched off (use32 = 0) for boxes so skewed, or open systems so far from the origin, that this could come near
/// a thousandth of eps, and when eps is no longer small against the cutoff (cells much larger than the cutoff).
struct Prefilter {
    int32_t use32;        // the pre-test is used at all
    float lo32, hi32;     // squared distances below / above which a pair is certainly within / beyond the cutoff
    double cell_edges[9]; // row d: the Cartesian vector of one cell along direction d
};

template <typename Grid>
VESIN_HOST_DEVICE inline void choose_prefilter(const Grid& grid, double cutoff, Prefilter& g) {
    g.use32 = 0;
    g.lo32 = 0.0f;
    g.hi32 = 0.0f;
    double extent_of_cell[3] = {0.0, 0.0, 0.0}; // per Cartesian axis: sum over the directions of |E_dk|
    double reach[3] = {0.0, 0.0, 0.0};          // the same with every direction taken s_d times
    double box_size = 0.0;
    double inverse_size = 0.0;
    double far_from_origin = 0.0;
    for (int d = 0; d < 3; d++) {
        const double scale = (grid.periodic[d] ? 1.0 : 1.0 / grid.np_scale[d]) / static_cast<double>(grid.n[d]);
        double row = 0.0;
        double inverse_row = 0.0;
        for (int k = 0; k < 3; k++) {
            g.cell_edges[3 * d + k] = grid.H[3 * d + k] * scale;
            extent_of_cell[k] += ::fabs(g.cell_edges[3 * d + k]);
            reach[k] += static_cast<double>(grid.s[d]) * ::fabs(g.cell_edges[3 * d + k]);
            row += ::fabs(grid.H[3 * d + k]) * (grid.periodic[d] ? 1.0 : 1.0 / grid.np_scale[d]);
            inverse_row += ::fabs(grid.Hinv[3 * k + d]);
        }
        box_size = ::fmax(box_size, row);
        inverse_size = ::fmax(inverse_size, inverse_row * (grid.periodic[d] ? 1.0 : grid.np_scale[d]));
        if (!grid.periodic[d]) {
            far_from_origin = ::fmax(far_from_origin, ::fabs(grid.np_min[d]) + 1.0 / grid.np_scale[d]);
        }
    }
    const double R = 2.0 * ::fmax(extent_of_cell[0], ::fmax(extent_of_cell[1], extent_of_cell[2]));
    const double D = ::fmax(reach[0], ::fmax(reach[1], reach[2]));
    const double u = 5.9604644775390625e-08; // 2^-24
    const double A = u * (3.0 * R + 2.0 * D + cutoff);
    const double eps = 2.0 * (3.4641016151377544 * cutoff * A + 3.0 * A * A + 5.0 * u * cutoff * cutoff);
    // what double precision leaves in a place: fractional coordinates of a point up to LOCAL_WRAP_LIMIT boxes away,
    // turned back into a length; along open directions the projected coordinate of a point far from the origin
    const double u64 = 1.1102230246251565e-16;
    const double behind = 16.0 * u64 * ((LOCAL_WRAP_LIMIT + 2.0) * box_size * inverse_size * box_size + far_from_origin);
    const double cutoff2 = cutoff * cutoff;
    if (!(eps <= 0.01 * cutoff2) || !(4.0 * cutoff * behind <= 1e-3 * eps) || !(eps > 0.0)) {
        return;
    }
    // thresholds rounded away from the cutoff
    float lo = static_cast<float>(cutoff2 - eps);
    float hi = static_cast<float>(cutoff2 + eps);
    if (static_cast<double>(lo) > cutoff2 - eps) {
        lo = ::nextafterf(lo, 0.0f);
    }
    if (static_cast<double>(hi) < cutoff2 + eps) {
        hi = ::nextafterf(hi, 3.0e38f);
    }
    g.lo32 = lo;
    g.hi32 = hi;
    g.use32 = 1;
}

/// The place of a point inside its cell (see choose_prefilter), from the position of the point in units of cells
/// along every direction, counted from the origin of its cell (`inside[d]`: 0 to 1 for a point the cell holds).
/// Not a number when the point lies too far outside of its cell or was moved by too many box vectors.
VESIN_HOST_DEVICE inline void local_place(const Prefilter& g, const double inside[3], const int32_t wrap[3], float place[3]) {
    bool usable = true;
    for (int d = 0; d < 3; d++) {
        usable = usable && inside[d] >= -1.0 && inside[d] <= 2.0 && wrap[d] <= LOCAL_WRAP_LIMIT && wrap[d] >= -LOCAL_WRAP_LIMIT;
    }
    for (int k = 0; k < 3; k++) {
        const double value = inside[0] * g.cell_edges[k] + inside[1] * g.cell_edges[3 + k] + inside[2] * g.cell_edges[6 + k];
        place[k] = usable ? static_cast<float>(value) : __builtin_nanf("");
    }
}

} // namespace vesin_hip

#endif
