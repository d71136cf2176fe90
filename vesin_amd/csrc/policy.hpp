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

constexpr int WAIT_REST = 64;        // calls that leave a launch with waiting workgroups alone after it gave up
constexpr int WAIT_REST_MAX = 4096;  // and after it gave up many times in a row

/// Some launches make workgroups wait for each other (the chain that places the rows of the single-pass search in
/// work-item order, the meeting of a small system's one launch). That only advances while the workgroups that are
/// waited for get to run, which holds on a GPU the launch has to itself and may not on one it shares with other
/// streams or processes. Every such wait is bounded, and a launch whose waves gave up is followed by the passes that
/// need no waiting; this is the bookkeeping that keeps a list from paying for the give-up on every call: after one,
/// the list leaves that launch alone for WAIT_REST calls, and every further give-up in a row doubles that, up to
/// WAIT_REST_MAX; a launch that went through brings the time back to WAIT_REST.
struct WaitRest {
    int rest = 0;
    int next_rest = WAIT_REST;

    /// Once per call that could use the launch: true while the list stays away from it.
    bool resting() {
        if (rest > 0) {
            rest -= 1;
            return true;
        }
        return false;
    }

    void gave_up() {
        rest = next_rest;
        next_rest = next_rest >= WAIT_REST_MAX / 2 ? WAIT_REST_MAX : 2 * next_rest;
    }

    void went_through() {
        next_rest = WAIT_REST;
    }
};

/// options.skin > 0: kept candidates pay when calls that only filter them outnumber the calls that compute them
/// again, which cost a failed filter and a search at cutoff + skin (two to three direct searches). A skin too thin
/// for how far the points move between calls turns that around, and in a batch, where one system past its limit
/// costs all systems their candidates, so does a large number of systems: candidates that serve fewer than
/// CANDIDATES_SHORT_LIVED filtering calls are short-lived, and after CANDIDATES_STRIKES such sets in a row the list
/// searches directly, keeping nothing, for CANDIDATES_REST calls before it tries candidates again. The rows are the
/// same either way.
constexpr int CANDIDATES_SHORT_LIVED = 4;
constexpr int CANDIDATES_STRIKES = 3;
constexpr int CANDIDATES_REST = 64;

struct CandidateLifetime {
    int filtered = 0; // calls that the current candidates served
    int strikes = 0;  // short-lived sets in a row
    int rest = 0;     // direct calls left before candidates are tried again

    void served() {
        filtered += 1;
    }

    /// The check found the candidates outdated. True: no new ones for a while.
    bool outdated() {
        strikes = filtered < CANDIDATES_SHORT_LIVED ? strikes + 1 : 0;
        filtered = 0;
        if (strikes >= CANDIDATES_STRIKES) {
            strikes = 0;
            rest = CANDIDATES_REST;
            return true;
        }
        return false;
    }

    /// Once per call without usable candidates: true while the list stays with the direct search.
    bool resting() {
        if (rest > 0) {
            rest -= 1;
            return true;
        }
        return false;
    }

    void reset() {
        filtered = 0;
        strikes = 0;
        rest = 0;
    }
};

// ---------------------------------------------------------------------------------------------------------------
// The search that writes a sorted list in order (ordered.cuh): how its work is cut into waves. Every choice gives
// the same list; the figures are what the passes were measured at on one MI355X (256 compute units, 1024 SIMDs).

constexpr unsigned int ORDERED_TILE_POINTS = 32; // the points a tile holds at most (TILE_POINTS of the kernels)

/// Points of a tile that one wave of the counting and the writing pass takes (a power of two, at most 32).
///
/// Large systems: a whole tile, and the candidates of every tile are put in order once by a launch of its own.
/// Systems of fewer than 2048 occupied cells (up to 3072 at 12 points per cell or fewer) are latency, not throughput:
/// either pass lasts as long as its slowest wave, which grows with the points the wave writes the rows of. Shares of
/// 8 points, of 4 where 8 would leave fewer than about 1300 waves with any points at all (per call, cutoff 5, full
/// lists, shares of 32 / 16 / 8 / 4 / 2 points: 10,000 atoms at 0.05 per cubic A 116 / 100 / 93 / 100 / 127 us, at
/// 0.1 137 / 125 / 101 / 108 / 115 us; 4,000 atoms 101 / 85 / 76 / 74 / 86 and 125 / 122 / 94 / 82 / 81 us). Shares
/// that most tiles have no points for cost next to nothing in time, their waves leave at once, but each has room for
/// its candidates' records: a caller with a fixed amount of work memory (`coarse`) keeps the rule for the smallest
/// systems only, which halves the share until every possible share of every tile slot makes 2048 waves.
inline unsigned int ordered_share(size_t n_points, size_t n_cells, size_t tile_slots, bool coarse) {
    unsigned int share = ORDERED_TILE_POINTS;
    const size_t occupied = n_cells < n_points ? n_cells : n_points;
    const double filled = occupied < 1 ? 1.0 : static_cast<double>(occupied);
    double mean = static_cast<double>(n_points) / filled;
    if (mean > ORDERED_TILE_POINTS) {
        mean = ORDERED_TILE_POINTS;
    }
    if (!coarse && (filled < 2048.0 || (filled < 3072.0 && mean <= 12.0))) {
        const double shares_of_eight = mean <= 8.0 ? 1.0 : (mean <= 16.0 ? 2.0 : (mean <= 24.0 ? 3.0 : 4.0));
        share = filled * shares_of_eight < 1300.0 ? 4 : 8;
    }
    while (share > 1 && tile_slots * (ORDERED_TILE_POINTS / share) < 2048) {
        share /= 2;
    }
    return share;
}

/// Whether the in-order search may take the work memory it asks for. Its counting pass leaves a record per
/// candidate for the writing pass, in a block of fixed size per tile *slot* (12 KB, room for 1024 candidates), and the
/// number of slots follows the cells as well as the points: a dense system takes about 1 KB per point (1,000,000
/// atoms of diamond: 0.9 GB), a sparse one with a cell per point would take 12 KB per point (17,000,000 points: 212
/// GB). Beyond 2 GiB + 1.5 KB per point the sorted list is made by the search that needs no such records, followed
/// by the radix sort.
inline bool ordered_records_fit(size_t n_points, size_t record_bytes) {
    const double allowed = 2147483648.0 + 1536.0 * static_cast<double>(n_points);
    return static_cast<double>(record_bytes) <= allowed;
}

/// Waves that share the points of a tile in the writing pass (1 or 4), from the number of tiles the call before had
/// on the same points (0: not known, one wave).
///
/// The pass keeps four waves per SIMD resident, 4096 on this GPU. A system of a few more tiles than that leaves the
/// stragglers running alone for as long as everything before them took (100,000 atoms, 4,260 tiles: 172 us where a
/// wave lives 110 us; four waves per tile 121 us). With four waves per tile a workgroup is a tile: its waves fetch
/// the tile's records together and each writes the rows of a quarter of the points, so the work comes in shorter
/// pieces at little extra cost. It pays for well-filled tiles up to about five times as many tiles as resident
/// waves (half lists at 24 points per tile, cutoff 6, per call with one wave -> four: 4,500 tiles 318 -> 283 us,
/// 9,000 tiles 551 -> 515 us, 19,000 tiles 833 -> 794 us, 39,000 tiles 1613 -> 1613 us; full lists at 23 points per
/// tile, 52,000 tiles: 2.04 -> 2.07 ms) and not for tiles of few points (12 per tile, full lists: 8,000 tiles 276 ->
/// 311 us, 27,000 tiles 483 -> 606 us).
inline unsigned int ordered_write_split(size_t n_points, size_t tiles_before) {
    if (tiles_before == 0) {
        return 1;
    }
    const double resident = 4096.0;
    const double tiles = static_cast<double>(tiles_before);
    if (static_cast<double>(n_points) < 16.0 * tiles) {
        return 1;
    }
    return tiles > 0.85 * resident && tiles <= 5.0 * resident ? 4 : 1;
}

/// Waves that share the candidates of a tile in the counting pass (1 or 2), decided like the other.
///
/// That pass runs seven waves per SIMD (7168 at a time) and lasts as long as its slowest wave, the one of the tile
/// with the most points and candidates. While the tiles of a system do not fill those slots much more than once, the
/// candidates of every well-filled tile are dealt to two waves, pairs of units of 64 in turn, that add up their rows
/// per point (half lists, cutoff 6, per call: 24 points per tile, 25,000 / 50,000 / 100,000 / 200,000 atoms 168 ->
/// 155, 217 -> 201, 312 -> 304, 529 -> 519 us; 400,000 atoms, 17,576 tiles: 833 -> 841 us; 12 points per tile,
/// 30,000 / 100,000 atoms: 137 -> 143, 275 -> 282 us).
inline unsigned int ordered_count_split(size_t n_points, size_t tiles_before) {
    if (tiles_before == 0 || tiles_before > 9216) {
        return 1;
    }
    return static_cast<double>(n_points) >= 16.0 * static_cast<double>(tiles_before) ? 2 : 1;
}

} // namespace vesin_hip

#endif
