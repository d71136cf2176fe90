// Host-side decisions of the driver that depend on a list's history, kept apart from the HIP code so that they can
// be compiled and tested on a machine without a GPU.
#ifndef VESIN_HIP_POLICY_HPP
#define VESIN_HIP_POLICY_HPP

#include <cstddef>

namespace vesin_hip {

/// What a call was asked for besides the box: a remembered box is only a good guess for the same question again.
struct BoxKey {
    size_t n_points;
    double cutoff;
    int algorithm;
    bool full;
    bool sorted;

    bool operator==(const BoxKey& other) const {
        return n_points == other.n_points && cutoff == other.cutoff && algorithm == other.algorithm &&
               full == other.full && sorted == other.sorted;
    }
};

constexpr int BOX_REST = 32;       // calls without a guess after the first wrong one
constexpr int BOX_REST_MAX = 4096; // and after many wrong ones in a row

/// The grid is picked on the host from the box, which lives on the device: reading it costs a round trip before
/// anything else can be launched. A call may instead start from the box of the call before and check the guess at
/// its last synchronisation; a wrong guess costs a whole search. This is the bookkeeping of when to guess:
///  * only a call that asks what the call that stored the box asked (same number of points, cutoff, algorithm and
///    kind of list): another system is likely to bring another box, and a box that is much too small for the points
///    puts them all into a few cells;
///  * after a wrong guess the list does not guess for `BOX_REST` calls, and every further wrong guess in a row
///    doubles that time (up to BOX_REST_MAX), so that a trajectory whose box changes with every step stops paying;
///    a right guess brings the time back to BOX_REST.
struct BoxGuess {
    bool have_box = false; // a box is remembered (set by the call that read one from the device)
    BoxKey key = {0, 0.0, 0, false, false};
    int rest = 0;
    int next_rest = BOX_REST;

    /// Once per call, before anything else: does this call start from the remembered box?
    bool begin(const BoxKey& now) {
        const bool guess = have_box && rest == 0 && now.n_points > 0 && key == now;
        if (rest > 0) {
            rest -= 1;
        }
        return guess;
    }

    void was_right() {
        next_rest = BOX_REST;
    }

    void was_wrong() {
        rest = next_rest;
        next_rest = next_rest >= BOX_REST_MAX / 2 ? BOX_REST_MAX : 2 * next_rest;
    }

    /// The call read its box from the device and remembered it.
    void stored(const BoxKey& now) {
        key = now;
    }
};

} // namespace vesin_hip

#endif
