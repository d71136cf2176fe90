// Test-only shim: exposes the host-side box/grid logic of the HIP driver (vesin_amd/csrc/geometry.hpp) through a
// C interface so that pytest can compare it with the oracle. Compiled by tests/test_host_geometry.py with g++.
#include <cstring>

#include "geometry.hpp"
#include "policy.hpp"

extern "C" int probe_box(const double box[9], const unsigned char periodic[3], double H[9], double Hinv[9], double face[3]) {
    bool flags[3] = {periodic[0] != 0, periodic[1] != 0, periodic[2] != 0};
    try {
        auto out = vesin_hip::normalise_box(box, flags);
        std::memcpy(H, out.H, sizeof(out.H));
        std::memcpy(Hinv, out.Hinv, sizeof(out.Hinv));
        std::memcpy(face, out.face, sizeof(out.face));
    } catch (const std::exception&) {
        return 1;
    }
    return 0;
}

extern "C" int probe_grid(
    const double box[9], const unsigned char periodic[3], double cutoff, size_t n_points,
    const double lo[3], const double hi[3], int single_cell, int n[3], int s[3]
) {
    bool flags[3] = {periodic[0] != 0, periodic[1] != 0, periodic[2] != 0};
    try {
        auto hbox = vesin_hip::normalise_box(box, flags);
        auto grid = vesin_hip::choose_grid(hbox, cutoff, n_points, lo, hi, single_cell != 0);
        for (int d = 0; d < 3; d++) {
            n[d] = grid.n[d];
            s[d] = grid.s[d];
        }
    } catch (const std::exception&) {
        return 1;
    }
    return 0;
}

// The fields choose_pruning fills, without the rest of the kernels' grid description.
struct ProbePruning {
    double prune_edges[6];
    double prune_slack[3];
    double prune_limit;
    int prune;
};

/// Grid and pruning of a system; `dropped[((dx + s0) * (2 s1 + 1) + (dy + s1)) * (2 s2 + 1) + (dz + s2)]` tells
/// whether the stencil entry (dx, dy, dz) is dropped (room for `n_dropped` entries). Also returns the edge vectors of
/// one cell (rows of `cell`), which the caller needs to check the decision.
extern "C" int probe_pruning(
    const double box[9], const unsigned char periodic[3], double cutoff, size_t n_points,
    const double lo[3], const double hi[3], int single_cell, int n[3], int s[3], double cell[9],
    unsigned char* dropped, size_t n_dropped
) {
    bool flags[3] = {periodic[0] != 0, periodic[1] != 0, periodic[2] != 0};
    try {
        auto hbox = vesin_hip::normalise_box(box, flags);
        auto grid = vesin_hip::choose_grid(hbox, cutoff, n_points, lo, hi, single_cell != 0);
        ProbePruning g;
        vesin_hip::choose_pruning(hbox, grid, cutoff, g);
        size_t at = 0;
        for (int d = 0; d < 3; d++) {
            n[d] = grid.n[d];
            s[d] = grid.s[d];
            const double scale = (flags[d] ? 1.0 : 1.0 / grid.np_scale[d]) / grid.n[d];
            for (int e = 0; e < 3; e++) {
                cell[3 * d + e] = hbox.H[d][e] * scale;
            }
        }
        for (int dx = -grid.s[0]; dx <= grid.s[0]; dx++) {
            for (int dy = -grid.s[1]; dy <= grid.s[1]; dy++) {
                for (int dz = -grid.s[2]; dz <= grid.s[2]; dz++) {
                    if (at >= n_dropped) {
                        return 2;
                    }
                    dropped[at++] = vesin_hip::stencil_entry_too_far(g, dx, dy, dz) ? 1 : 0;
                }
            }
        }
    } catch (const std::exception&) {
        return 1;
    }
    return 0;
}

/// Runs the bookkeeping of the remembered box (vesin_hip::BoxGuess) over a sequence of calls. Call k asks for
/// `n_points[k]` points with cutoff `cutoff[k]` and finds that the box `changed[k]` (non-zero) since the call before.
/// `guessed[k]` receives whether the call started from the remembered box. The driver's use of the struct is
/// reproduced: a wrong guess is followed by a call that reads the box, which is then remembered.
extern "C" void probe_box_guess(
    const size_t* n_points, const double* cutoff, const unsigned char* changed, size_t n_calls, unsigned char* guessed
) {
    vesin_hip::BoxGuess guess;
    for (size_t k = 0; k < n_calls; k++) {
        const vesin_hip::BoxKey key = {n_points[k], cutoff[k], 0, true, false};
        const bool guessing = guess.begin(key);
        guessed[k] = guessing ? 1 : 0;
        if (guessing) {
            if (changed[k] == 0) {
                guess.was_right();
                continue;
            }
            guess.was_wrong();
        }
        guess.have_box = true; // the call read its box
        guess.stored(key);
    }
}

/// The cut of the in-order search's work into waves (policy.hpp), as the driver asks for it.
extern "C" unsigned int probe_ordered_share(size_t n_points, size_t n_cells, size_t tile_slots, int coarse) {
    return vesin_hip::ordered_share(n_points, n_cells, tile_slots, coarse != 0);
}

extern "C" unsigned int probe_ordered_write_split(size_t n_points, size_t tiles_before) {
    return vesin_hip::ordered_write_split(n_points, tiles_before);
}

extern "C" unsigned int probe_ordered_count_split(size_t n_points, size_t tiles_before) {
    return vesin_hip::ordered_count_split(n_points, tiles_before);
}

/// Runs the bookkeeping of a launch with waiting workgroups (vesin_hip::WaitRest) over a sequence of calls:
/// `gives_up[k]` says whether the launch would give up in call k if it were used; `used[k]` receives whether call k
/// used it.
extern "C" void probe_wait_rest(const unsigned char* gives_up, size_t n_calls, unsigned char* used) {
    vesin_hip::WaitRest rest;
    for (size_t k = 0; k < n_calls; k++) {
        if (rest.resting()) {
            used[k] = 0;
            continue;
        }
        used[k] = 1;
        if (gives_up[k] != 0) {
            rest.gave_up();
        } else {
            rest.went_through();
        }
    }
}

/// Runs the bookkeeping of kept candidates (vesin_hip::CandidateLifetime) over a sequence of calls with a skin:
/// `outdated[k]` says whether candidates that exist at call k are found outdated by it. `what[k]` receives what call
/// k does: 0 a direct search that keeps nothing, 1 a direct search followed by new candidates, 2 a filter of the kept
/// candidates, 3 a filter that fails followed by new candidates and their filter.
extern "C" void probe_candidate_lifetime(const unsigned char* outdated, size_t n_calls, unsigned char* what) {
    vesin_hip::CandidateLifetime lifetime;
    bool have = false;
    for (size_t k = 0; k < n_calls; k++) {
        if (!have) {
            if (lifetime.resting()) {
                what[k] = 0;
            } else {
                what[k] = 1;
                have = true;
            }
            continue;
        }
        if (outdated[k] != 0) {
            if (lifetime.outdated()) {
                what[k] = 0;
                have = false;
                continue;
            }
            what[k] = 3;
        } else {
            what[k] = 2;
        }
        lifetime.served();
    }
}

extern "C" int probe_ordered_records_fit(size_t n_points, size_t record_bytes) {
    return vesin_hip::ordered_records_fit(n_points, record_bytes) ? 1 : 0;
}

// The fields choose_prefilter reads of a grid.
struct ProbeGridForPrefilter {
    double H[9];
    double Hinv[9];
    double np_min[3];
    double np_scale[3];
    int n[3];
    int s[3];
    int periodic[3];
};

/// Grid of a system and the single-precision pre-test chosen for it: `out` receives use32, lo32, hi32 (as doubles)
/// and the nine components of the cell edges; `n` and `s` the grid.
extern "C" int probe_prefilter(
    const double box[9], const unsigned char periodic[3], double cutoff, size_t n_points,
    const double lo[3], const double hi[3], int single_cell, int n[3], int s[3], double out[12]
) {
    bool flags[3] = {periodic[0] != 0, periodic[1] != 0, periodic[2] != 0};
    try {
        auto hbox = vesin_hip::normalise_box(box, flags);
        auto grid = vesin_hip::choose_grid(hbox, cutoff, n_points, lo, hi, single_cell != 0);
        ProbeGridForPrefilter g;
        for (int d = 0; d < 3; d++) {
            for (int e = 0; e < 3; e++) {
                g.H[3 * d + e] = hbox.H[d][e];
                g.Hinv[3 * d + e] = hbox.Hinv[d][e];
            }
            g.np_min[d] = grid.np_min[d];
            g.np_scale[d] = grid.np_scale[d];
            g.n[d] = n[d] = grid.n[d];
            g.s[d] = s[d] = grid.s[d];
            g.periodic[d] = flags[d] ? 1 : 0;
        }
        vesin_hip::Prefilter pre;
        vesin_hip::choose_prefilter(g, cutoff, pre);
        out[0] = pre.use32;
        out[1] = pre.lo32;
        out[2] = pre.hi32;
        for (int k = 0; k < 9; k++) {
            out[3 + k] = pre.cell_edges[k];
        }
    } catch (const std::exception&) {
        return 1;
    }
    return 0;
}
