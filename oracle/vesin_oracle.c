/* CPU oracle for the neighbor-list path: TEST INFRASTRUCTURE ONLY (see vesin_oracle.h).
 *
 * A plain-C restatement of the algorithm of the reference's CPU engine, keeping the order of every
 * floating-point operation so that pair membership at the cutoff, distances and vectors come out bit-identical.
 * Build with -ffp-contract=off and without -march=native (FMA contraction changes d^2).
 *
 * Reference locations followed (relative to the reference checkout):
 *   vesin/src/math.hpp:14-31,82-117       dot / norm / normalize / cross / inverse / vector*matrix
 *   vesin/src/types.hpp:20-97             box normalisation, inverse, distances between faces
 *   vesin/src/types.hpp:111-126           cartesian -> fractional
 *   vesin/src/types.hpp:159-200           bounding box of the points, non-finite check, 1% margin
 *   vesin/src/types.hpp:232-243           shift -> cartesian
 *   vesin/src/cpu_cell_list.cpp:61-210    pair predicate, half-list rule, per-thread lists merged in thread order
 *   vesin/src/cpu_cell_list.cpp:253-263   divmod (Python convention)
 *   vesin/src/cpu_cell_list.cpp:277-351   grid: n_cells, cap at 1e5 cells, n_search, mixed-periodicity widening
 *   vesin/src/cpu_cell_list.cpp:353-374   assignment of a point to (cell, wrap shift)
 *   vesin/src/cpu_cell_list.cpp:376-451   enumeration of candidate pairs
 *   vesin/src/cpu_cell_list.cpp:634-730   sort by first index (the reference's is unstable; this one is stable)
 *   vesin/src/threadpool.hpp:156-159      static contiguous chunks of cells per thread
 *   vesin/src/vesin.cpp:70-78             cutoff validation
 *
 * Parity status: every function here is pinned by tests/test_oracle.py and tests/test_known_answers.py against the literal vectors of the
 * reference's own tests, against closed forms / brute force, and (where oracle/_ref builds) against the compiled
 * reference itself.
 */
#include "vesin_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct { double v[3]; } vec3;
typedef struct { double m[3][3]; } mat3;

/* math.hpp:14-16 */
static double dot(vec3 a, vec3 b) {
    return a.v[0] * b.v[0] + a.v[1] * b.v[1] + a.v[2] * b.v[2];
}

/* math.hpp:18-24 */
static vec3 normalize(vec3 a) {
    double s = 1.0 / sqrt(dot(a, a));
    vec3 r = {{s * a.v[0], s * a.v[1], s * a.v[2]}};
    return r;
}

/* math.hpp:26-32 */
static vec3 cross(vec3 a, vec3 b) {
    vec3 r = {{
        a.v[1] * b.v[2] - a.v[2] * b.v[1],
        a.v[2] * b.v[0] - a.v[0] * b.v[2],
        a.v[0] * b.v[1] - a.v[1] * b.v[0],
    }};
    return r;
}

static vec3 row(const mat3* m, int i) {
    vec3 r = {{m->m[i][0], m->m[i][1], m->m[i][2]}};
    return r;
}

static void set_row(mat3* m, int i, vec3 r) {
    m->m[i][0] = r.v[0];
    m->m[i][1] = r.v[1];
    m->m[i][2] = r.v[2];
}

/* math.hpp:74-80 */
static double determinant(const mat3* a) {
    return a->m[0][0] * (a->m[1][1] * a->m[2][2] - a->m[2][1] * a->m[1][2])
         - a->m[0][1] * (a->m[1][0] * a->m[2][2] - a->m[1][2] * a->m[2][0])
         + a->m[0][2] * (a->m[1][0] * a->m[2][1] - a->m[1][1] * a->m[2][0]);
}

/* math.hpp:82-100 */
static mat3 inverse(const mat3* a, double det) {
    mat3 r;
    r.m[0][0] = (a->m[1][1] * a->m[2][2] - a->m[2][1] * a->m[1][2]) / det;
    r.m[0][1] = (a->m[0][2] * a->m[2][1] - a->m[0][1] * a->m[2][2]) / det;
    r.m[0][2] = (a->m[0][1] * a->m[1][2] - a->m[0][2] * a->m[1][1]) / det;
    r.m[1][0] = (a->m[1][2] * a->m[2][0] - a->m[1][0] * a->m[2][2]) / det;
    r.m[1][1] = (a->m[0][0] * a->m[2][2] - a->m[0][2] * a->m[2][0]) / det;
    r.m[1][2] = (a->m[1][0] * a->m[0][2] - a->m[0][0] * a->m[1][2]) / det;
    r.m[2][0] = (a->m[1][0] * a->m[2][1] - a->m[2][0] * a->m[1][1]) / det;
    r.m[2][1] = (a->m[2][0] * a->m[0][1] - a->m[0][0] * a->m[2][1]) / det;
    r.m[2][2] = (a->m[0][0] * a->m[1][1] - a->m[1][0] * a->m[0][1]) / det;
    return r;
}

/* math.hpp:111-117: row vector times matrix */
static vec3 vec_mat(vec3 x, const mat3* a) {
    vec3 r = {{
        x.v[0] * a->m[0][0] + x.v[1] * a->m[1][0] + x.v[2] * a->m[2][0],
        x.v[0] * a->m[0][1] + x.v[1] * a->m[1][1] + x.v[2] * a->m[2][1],
        x.v[0] * a->m[0][2] + x.v[1] * a->m[1][2] + x.v[2] * a->m[2][2],
    }};
    return r;
}

typedef struct {
    mat3 matrix;
    mat3 inverse;
    int periodic[3];
    double min_pos[3];
    double max_pos[3];
    double face[3];
} bounding_box;

/* types.hpp:20-97 */
static int box_init(bounding_box* b, const double box[9], const uint8_t periodic[3], char* error, size_t error_len) {
    for (int i = 0; i < 3; i++) {
        for (int j = 0; j < 3; j++) {
            b->matrix.m[i][j] = box[3 * i + j];
        }
        b->periodic[i] = periodic[i] ? 1 : 0;
        b->max_pos[i] = -1e300;
        b->min_pos[i] = 1e300;
    }

    int n_periodic = 0, p1 = -1, p2 = -1;
    for (int i = 0; i < 3; i++) {
        if (b->periodic[i]) {
            n_periodic += 1;
            if (p1 == -1) {
                p1 = i;
            } else if (p2 == -1) {
                p2 = i;
            }
        }
    }

    if (n_periodic == 0) {
        memset(&b->matrix, 0, sizeof(mat3));
        b->matrix.m[0][0] = 1;
        b->matrix.m[1][1] = 1;
        b->matrix.m[2][2] = 1;
    } else if (n_periodic == 1) {
        vec3 a = row(&b->matrix, p1);
        vec3 bb = {{0, 1, 0}};
        if (fabs(dot(normalize(a), bb)) > 0.9) {
            vec3 z = {{0, 0, 1}};
            bb = z;
        }
        vec3 c = normalize(cross(a, bb));
        bb = normalize(cross(c, a));
        set_row(&b->matrix, (p1 + 1) % 3, bb);
        set_row(&b->matrix, (p1 + 2) % 3, c);
    } else if (n_periodic == 2) {
        vec3 a = row(&b->matrix, p1);
        vec3 bb = row(&b->matrix, p2);
        vec3 c = normalize(cross(a, bb));
        set_row(&b->matrix, 3 - p1 - p2, c);
    }

    double det = determinant(&b->matrix);
    /* The reference only tests `abs(det) < 1e-30`; a NaN determinant (a periodic direction with a zero box
       vector) passes that test there and leads to undefined behaviour (NaN cell counts cast to integers). The
       oracle refuses such a box instead of reproducing it. */
    if (fabs(det) < 1e-30 || det != det) {
        snprintf(error, error_len, "the box matrix is not invertible");
        return 1;
    }
    b->inverse = inverse(&b->matrix, det);

    vec3 a = row(&b->matrix, 0);
    vec3 bb = row(&b->matrix, 1);
    vec3 c = row(&b->matrix, 2);
    vec3 na = normalize(cross(bb, c));
    vec3 nb = normalize(cross(c, a));
    vec3 nc = normalize(cross(a, bb));

    b->face[0] = b->periodic[0] ? fabs(dot(na, a)) : b->max_pos[0] - b->min_pos[0];
    b->face[1] = b->periodic[1] ? fabs(dot(nb, bb)) : b->max_pos[1] - b->min_pos[1];
    b->face[2] = b->periodic[2] ? fabs(dot(nc, c)) : b->max_pos[2] - b->min_pos[2];
    return 0;
}

/* types.hpp:159-200 */
static int box_make_bounding_for(bounding_box* b, const double* points, size_t n, char* error, size_t error_len) {
    for (size_t i = 0; i < n; i++) {
        for (int d = 0; d < 3; d++) {
            double x = points[3 * i + d];
            if (!isfinite(x)) {
                snprintf(error, error_len, "point %zu has non-finite coordinate along axis %d: %f", i, d, x);
                return 1;
            }
            if (x < b->min_pos[d]) {
                b->min_pos[d] = x;
            }
            if (x > b->max_pos[d]) {
                b->max_pos[d] = x;
            }
        }
    }

    for (int d = 0; d < 3; d++) {
        if (b->max_pos[d] - b->min_pos[d] < 1e-6) {
            b->max_pos[d] = b->min_pos[d] + 1;
        }
        if (!b->periodic[d]) {
            b->face[d] = (b->max_pos[d] - b->min_pos[d]) * 1.01;
            if (b->face[d] < 1.0) {
                b->face[d] = 1.0;
            }
        }
    }
    return 0;
}

/* types.hpp:111-126 */
static vec3 cartesian_to_fractional(const bounding_box* b, vec3 x) {
    vec3 f = vec_mat(x, &b->inverse);
    for (int d = 0; d < 3; d++) {
        if (!b->periodic[d]) {
            f.v[d] = (x.v[d] - b->min_pos[d]) / b->face[d];
        }
    }
    return f;
}

/* cpu_cell_list.cpp:253-263 */
static void divmod(int32_t a, int32_t b, int32_t* quotient, int32_t* remainder) {
    int32_t q = a / b;
    int32_t r = a % b;
    if (r < 0) {
        r += b;
        q -= 1;
    }
    *quotient = q;
    *remainder = r;
}

static double clamp_low(double x, double low) {
    /* std::clamp(x, low, HUGE_VAL) */
    if (x < low) {
        return low;
    }
    if (HUGE_VAL < x) {
        return HUGE_VAL;
    }
    return x;
}

#define MAX_NUMBER_OF_CELLS 1e5

/* cpu_cell_list.cpp:277-351 */
static void grid_init(const bounding_box* b, double cutoff, int32_t shape[3], int32_t n_search[3]) {
    double n_cells[3];
    for (int d = 0; d < 3; d++) {
        n_cells[d] = clamp_low(trunc(b->face[d] / cutoff), 1.0);
    }

    double total = n_cells[0] * n_cells[1] * n_cells[2];
    if (total > MAX_NUMBER_OF_CELLS) {
        double ratio_x_y = n_cells[0] / n_cells[1];
        double ratio_y_z = n_cells[1] / n_cells[2];
        n_cells[2] = trunc(cbrt(MAX_NUMBER_OF_CELLS / (ratio_x_y * ratio_y_z * ratio_y_z)));
        n_cells[1] = trunc(ratio_y_z * n_cells[2]);
        n_cells[0] = trunc(ratio_x_y * n_cells[1]);
    }

    for (int d = 0; d < 3; d++) {
        n_search[d] = (int32_t)ceil(cutoff * n_cells[d] / b->face[d]);
        shape[d] = (int32_t)(size_t)n_cells[d];
        if (n_search[d] < 1) {
            n_search[d] = 1;
        }
    }

    int has_periodic = 0, has_non_periodic = 0;
    for (int d = 0; d < 3; d++) {
        if (b->periodic[d]) {
            has_periodic = 1;
        } else {
            has_non_periodic = 1;
        }
    }
    if (has_periodic && has_non_periodic) {
        for (int d = 0; d < 3; d++) {
            if (!b->periodic[d] && n_search[d] < shape[d] - 1) {
                n_search[d] = shape[d] - 1;
            }
        }
    }
}

/* cpu_cell_list.cpp:101-133 */
int vesin_oracle_half_list_keeps(size_t first, size_t second, const int32_t shift[3]) {
    if (first > second) {
        return 0;
    }
    if (first == second) {
        int32_t sum = shift[0] + shift[1] + shift[2];
        if (sum < 0) {
            return 0;
        }
        if (sum == 0 && (shift[2] < 0 || (shift[2] == 0 && shift[1] < 0))) {
            return 0;
        }
    }
    return 1;
}

typedef struct {
    size_t length;
    size_t capacity;
    size_t* pairs;
    int32_t* shifts;
    double* distances;
    double* vectors;
} growable;

static int growable_reserve(growable* g, size_t needed, const vesin_oracle_options* o) {
    if (needed <= g->capacity) {
        return 0;
    }
    size_t cap = g->capacity == 0 ? 1024 : g->capacity;
    while (cap < needed) {
        cap *= 2;
    }
    size_t* pairs = (size_t*)realloc(g->pairs, cap * 2 * sizeof(size_t));
    if (pairs == NULL) {
        return 1;
    }
    g->pairs = pairs;
    if (o->return_shifts) {
        int32_t* p = (int32_t*)realloc(g->shifts, cap * 3 * sizeof(int32_t));
        if (p == NULL) {
            return 1;
        }
        g->shifts = p;
    }
    if (o->return_distances) {
        double* p = (double*)realloc(g->distances, cap * sizeof(double));
        if (p == NULL) {
            return 1;
        }
        g->distances = p;
    }
    if (o->return_vectors) {
        double* p = (double*)realloc(g->vectors, cap * 3 * sizeof(double));
        if (p == NULL) {
            return 1;
        }
        g->vectors = p;
    }
    g->capacity = cap;
    return 0;
}

static void growable_free(growable* g) {
    free(g->pairs);
    free(g->shifts);
    free(g->distances);
    free(g->vectors);
    memset(g, 0, sizeof(*g));
}

typedef struct {
    const double* points;
    const bounding_box* box;
    const vesin_oracle_options* options;
    double cutoff2;
    int32_t shape[3];
    int32_t n_search[3];
    /* counting-sorted cells: atoms of cell c are cell_atoms[cell_start[c] .. cell_start[c+1]), in increasing
       point index (the order in which the reference's add_point pushes them) */
    const size_t* cell_start;
    const uint32_t* cell_atoms;
    const int32_t* wrap;      /* [n_points][3] shift of each point, cpu_cell_list.cpp:364-371 */
} search_context;

/* cpu_cell_list.cpp:376-451 (enumeration) with the callback of cpu_cell_list.cpp:100-163 inlined */
static int search_cell(const search_context* ctx, size_t linear_cell, growable* out) {
    const vesin_oracle_options* o = ctx->options;
    const bounding_box* b = ctx->box;
    const int32_t sx = ctx->shape[0], sy = ctx->shape[1], sz = ctx->shape[2];

    int32_t cx = (int32_t)(linear_cell % (size_t)sx);
    int32_t cy = (int32_t)((linear_cell / (size_t)sx) % (size_t)sy);
    int32_t cz = (int32_t)(linear_cell / ((size_t)sx * (size_t)sy));

    size_t i_begin = ctx->cell_start[linear_cell];
    size_t i_end = ctx->cell_start[linear_cell + 1];
    if (i_begin == i_end) {
        return 0;
    }

    for (int32_t dx = -ctx->n_search[0]; dx <= ctx->n_search[0]; dx++) {
        for (int32_t dy = -ctx->n_search[1]; dy <= ctx->n_search[1]; dy++) {
            for (int32_t dz = -ctx->n_search[2]; dz <= ctx->n_search[2]; dz++) {
                int32_t cell_shift[3] = {0, 0, 0};
                int32_t neighbor[3] = {cx + dx, cy + dy, cz + dz};
                const int32_t shape[3] = {sx, sy, sz};

                int valid = 1;
                for (int d = 0; d < 3; d++) {
                    if (b->periodic[d]) {
                        divmod(neighbor[d], shape[d], &cell_shift[d], &neighbor[d]);
                    } else if (neighbor[d] < 0 || neighbor[d] >= shape[d]) {
                        valid = 0;
                        break;
                    }
                }
                if (!valid) {
                    continue;
                }

                size_t neighbor_linear = ((size_t)sx * (size_t)sy * (size_t)neighbor[2]) +
                                         ((size_t)sx * (size_t)neighbor[1]) + (size_t)neighbor[0];
                size_t j_begin = ctx->cell_start[neighbor_linear];
                size_t j_end = ctx->cell_start[neighbor_linear + 1];

                for (size_t ii = i_begin; ii < i_end; ii++) {
                    size_t first = ctx->cell_atoms[ii];
                    const int32_t* wi = ctx->wrap + 3 * first;
                    for (size_t jj = j_begin; jj < j_end; jj++) {
                        size_t second = ctx->cell_atoms[jj];
                        const int32_t* wj = ctx->wrap + 3 * second;

                        int32_t shift[3] = {
                            cell_shift[0] + wi[0] - wj[0],
                            cell_shift[1] + wi[1] - wj[1],
                            cell_shift[2] + wi[2] - wj[2],
                        };
                        int shift_is_zero = shift[0] == 0 && shift[1] == 0 && shift[2] == 0;

                        if ((shift[0] != 0 && !b->periodic[0]) ||
                            (shift[1] != 0 && !b->periodic[1]) ||
                            (shift[2] != 0 && !b->periodic[2])) {
                            continue;
                        }
                        if (first == second && shift_is_zero) {
                            continue;
                        }
                        if (!o->full && !vesin_oracle_half_list_keeps(first, second, shift)) {
                            continue;
                        }

                        /* types.hpp:232-243 then cpu_cell_list.cpp:135-138 */
                        vec3 s = {{(double)shift[0], (double)shift[1], (double)shift[2]}};
                        vec3 t = vec_mat(s, &b->matrix);
                        const double* pi = ctx->points + 3 * first;
                        const double* pj = ctx->points + 3 * second;
                        vec3 v = {{
                            (pj[0] - pi[0]) + t.v[0],
                            (pj[1] - pi[1]) + t.v[1],
                            (pj[2] - pi[2]) + t.v[2],
                        }};
                        double d2 = dot(v, v);
                        if (d2 < ctx->cutoff2) {
                            if (growable_reserve(out, out->length + 1, o)) {
                                return 1;
                            }
                            size_t k = out->length;
                            out->pairs[2 * k + 0] = first;
                            out->pairs[2 * k + 1] = second;
                            if (o->return_shifts) {
                                out->shifts[3 * k + 0] = shift[0];
                                out->shifts[3 * k + 1] = shift[1];
                                out->shifts[3 * k + 2] = shift[2];
                            }
                            if (o->return_distances) {
                                out->distances[k] = sqrt(d2);
                            }
                            if (o->return_vectors) {
                                out->vectors[3 * k + 0] = v.v[0];
                                out->vectors[3 * k + 1] = v.v[1];
                                out->vectors[3 * k + 2] = v.v[2];
                            }
                            out->length += 1;
                        }
                    }
                }
            }
        }
    }
    return 0;
}

/* cpu_cell_list.cpp:634-730: sorted by first index only. The reference uses an unstable std::sort, leaving the
   order inside one `i` unspecified (vesin.h:55-57); a stable counting sort is used here. */
static int sort_by_first(growable* g, size_t n_points, const vesin_oracle_options* o) {
    size_t n = g->length;
    if (n == 0) {
        return 0;
    }
    size_t* start = (size_t*)calloc(n_points + 1, sizeof(size_t));
    size_t* order = (size_t*)malloc(n * sizeof(size_t));
    if (start == NULL || order == NULL) {
        free(start);
        free(order);
        return 1;
    }
    for (size_t k = 0; k < n; k++) {
        start[g->pairs[2 * k] + 1] += 1;
    }
    for (size_t i = 0; i < n_points; i++) {
        start[i + 1] += start[i];
    }
    for (size_t k = 0; k < n; k++) {
        order[start[g->pairs[2 * k]]++] = k;
    }
    free(start);

    growable s;
    memset(&s, 0, sizeof(s));
    if (growable_reserve(&s, n, o)) {
        growable_free(&s);
        free(order);
        return 1;
    }
    for (size_t k = 0; k < n; k++) {
        size_t from = order[k];
        s.pairs[2 * k + 0] = g->pairs[2 * from + 0];
        s.pairs[2 * k + 1] = g->pairs[2 * from + 1];
        if (o->return_shifts) {
            memcpy(s.shifts + 3 * k, g->shifts + 3 * from, 3 * sizeof(int32_t));
        }
        if (o->return_distances) {
            s.distances[k] = g->distances[from];
        }
        if (o->return_vectors) {
            memcpy(s.vectors + 3 * k, g->vectors + 3 * from, 3 * sizeof(double));
        }
    }
    s.length = n;
    free(order);
    growable_free(g);
    *g = s;
    return 0;
}

int vesin_oracle_neighbors(
    const double* points, size_t n_points,
    const double box[9], const uint8_t periodic[3],
    const vesin_oracle_options* options,
    vesin_oracle_list* out,
    vesin_oracle_grid* grid,
    char* error, size_t error_len
) {
    /* vesin.cpp:70-78 */
    if (!isfinite(options->cutoff) || options->cutoff <= 0) {
        snprintf(error, error_len, "cutoff must be a finite, positive number");
        return 1;
    }
    if (options->cutoff <= 1e-6) {
        snprintf(error, error_len, "cutoff is too small");
        return 1;
    }

    bounding_box b;
    if (box_init(&b, box, periodic, error, error_len)) {
        return 1;
    }
    if (box_make_bounding_for(&b, points, n_points, error, error_len)) {
        return 1;
    }

    search_context ctx;
    memset(&ctx, 0, sizeof(ctx));
    ctx.points = points;
    ctx.box = &b;
    ctx.options = options;
    ctx.cutoff2 = options->cutoff * options->cutoff; /* cpu_cell_list.cpp:77 */
    grid_init(&b, options->cutoff, ctx.shape, ctx.n_search);

    if (grid != NULL) {
        for (int d = 0; d < 3; d++) {
            grid->n_cells[d] = ctx.shape[d];
            grid->n_search[d] = ctx.n_search[d];
            grid->face_distances[d] = b.face[d];
            for (int e = 0; e < 3; e++) {
                grid->matrix[3 * d + e] = b.matrix.m[d][e];
                grid->inverse[3 * d + e] = b.inverse.m[d][e];
            }
        }
    }

    size_t total_cells = (size_t)ctx.shape[0] * (size_t)ctx.shape[1] * (size_t)ctx.shape[2];

    /* cpu_cell_list.cpp:353-374 for every point, stored as a counting sort instead of vector<vector<Point>> */
    size_t* cell_start = (size_t*)calloc(total_cells + 1, sizeof(size_t));
    size_t* cell_of = (size_t*)malloc((n_points ? n_points : 1) * sizeof(size_t));
    int32_t* wrap = (int32_t*)malloc((n_points ? n_points : 1) * 3 * sizeof(int32_t));
    uint32_t* cell_atoms = (uint32_t*)malloc((n_points ? n_points : 1) * sizeof(uint32_t));
    if (cell_start == NULL || cell_of == NULL || wrap == NULL || cell_atoms == NULL) {
        free(cell_start);
        free(cell_of);
        free(wrap);
        free(cell_atoms);
        snprintf(error, error_len, "failed to allocate memory");
        return 1;
    }

    for (size_t i = 0; i < n_points; i++) {
        vec3 x = {{points[3 * i], points[3 * i + 1], points[3 * i + 2]}};
        vec3 f = cartesian_to_fractional(&b, x);
        int32_t cell[3];
        for (int d = 0; d < 3; d++) {
            int32_t c = (int32_t)floor(f.v[d] * (double)(size_t)ctx.shape[d]);
            divmod(c, ctx.shape[d], &wrap[3 * i + d], &cell[d]);
        }
        size_t linear = ((size_t)ctx.shape[0] * (size_t)ctx.shape[1] * (size_t)cell[2]) +
                        ((size_t)ctx.shape[0] * (size_t)cell[1]) + (size_t)cell[0];
        cell_of[i] = linear;
        cell_start[linear + 1] += 1;
    }
    for (size_t c = 0; c < total_cells; c++) {
        cell_start[c + 1] += cell_start[c];
    }
    {
        size_t* cursor = (size_t*)malloc((total_cells + 1) * sizeof(size_t));
        if (cursor == NULL) {
            free(cell_start);
            free(cell_of);
            free(wrap);
            free(cell_atoms);
            snprintf(error, error_len, "failed to allocate memory");
            return 1;
        }
        memcpy(cursor, cell_start, (total_cells + 1) * sizeof(size_t));
        for (size_t i = 0; i < n_points; i++) {
            cell_atoms[cursor[cell_of[i]]++] = (uint32_t)i;
        }
        free(cursor);
    }
    ctx.cell_start = cell_start;
    ctx.cell_atoms = cell_atoms;
    ctx.wrap = wrap;

    /* cpu_cell_list.cpp:85-100 and threadpool.hpp:156-159: thread t owns cells [t*n/T, (t+1)*n/T) */
    int n_threads = options->n_threads;
#ifdef _OPENMP
    if (n_threads <= 0) {
        n_threads = omp_get_max_threads();
    }
#else
    n_threads = 1;
#endif
    if ((size_t)n_threads > total_cells) {
        n_threads = (int)total_cells;
    }
    if (n_threads < 1) {
        n_threads = 1;
    }

    growable* locals = (growable*)calloc((size_t)n_threads, sizeof(growable));
    int failed = locals == NULL;

    if (!failed) {
#ifdef _OPENMP
#pragma omp parallel num_threads(n_threads)
#endif
        {
#ifdef _OPENMP
            size_t t = (size_t)omp_get_thread_num();
            size_t active = (size_t)omp_get_num_threads();
#else
            size_t t = 0;
            size_t active = 1;
#endif
            size_t begin = (t * total_cells) / active;
            size_t end = ((t + 1) * total_cells) / active;
            for (size_t c = begin; c < end; c++) {
                if (search_cell(&ctx, c, &locals[t])) {
#ifdef _OPENMP
#pragma omp atomic write
#endif
                    failed = 1;
                    break;
                }
            }
        }
    }

    free(cell_start);
    free(cell_of);
    free(wrap);
    free(cell_atoms);

    if (failed) {
        if (locals != NULL) {
            for (int t = 0; t < n_threads; t++) {
                growable_free(&locals[t]);
            }
            free(locals);
        }
        snprintf(error, error_len, "failed to allocate memory");
        return 1;
    }

    /* cpu_cell_list.cpp:165-203: thread 0's list first, then threads 1..T-1 in order */
    growable merged;
    memset(&merged, 0, sizeof(merged));
    size_t total = 0;
    for (int t = 0; t < n_threads; t++) {
        total += locals[t].length;
    }
    if (growable_reserve(&merged, total > 0 ? total : 1, options)) {
        for (int t = 0; t < n_threads; t++) {
            growable_free(&locals[t]);
        }
        free(locals);
        growable_free(&merged);
        snprintf(error, error_len, "failed to allocate memory");
        return 1;
    }
    for (int t = 0; t < n_threads; t++) {
        growable* l = &locals[t];
        size_t at = merged.length;
        if (l->length > 0) {
            memcpy(merged.pairs + 2 * at, l->pairs, l->length * 2 * sizeof(size_t));
            if (options->return_shifts) {
                memcpy(merged.shifts + 3 * at, l->shifts, l->length * 3 * sizeof(int32_t));
            }
            if (options->return_distances) {
                memcpy(merged.distances + at, l->distances, l->length * sizeof(double));
            }
            if (options->return_vectors) {
                memcpy(merged.vectors + 3 * at, l->vectors, l->length * 3 * sizeof(double));
            }
        }
        merged.length += l->length;
        growable_free(l);
    }
    free(locals);

    if (options->sorted) {
        if (sort_by_first(&merged, n_points, options)) {
            growable_free(&merged);
            snprintf(error, error_len, "failed to allocate memory");
            return 1;
        }
    }

    vesin_oracle_free(out);
    out->length = merged.length;
    out->pairs = merged.pairs;
    out->shifts = merged.shifts;
    out->distances = merged.distances;
    out->vectors = merged.vectors;
    return 0;
}

void vesin_oracle_free(vesin_oracle_list* list) {
    if (list == NULL) {
        return;
    }
    free(list->pairs);
    free(list->shifts);
    free(list->distances);
    free(list->vectors);
    memset(list, 0, sizeof(*list));
}
