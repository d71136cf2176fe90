// Test-only shim: exposes the host-side box/grid logic of the HIP driver (vesin_amd/csrc/geometry.hpp) through a
// C interface so that pytest can compare it with the oracle. Compiled by tests/test_host_geometry.py with g++.
#include <cstring>

#include "geometry.hpp"

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
