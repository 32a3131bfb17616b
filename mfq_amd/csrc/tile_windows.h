// The LDS windows of the prefill tile kernel: how many steps a window serves, where it starts in a row's stream and
// which of its bytes a step reads, in plain integer code that compiles for the device (ops_prefill.hip uses it) and for
// the host (tests/cpp/tile_window_check.cpp sweeps it: every read of every step must fall inside what was staged).
// A step is 64 columns: two lane blocks of 32.
#pragma once

#include "fetch_at.h"

namespace mfq_amd {
namespace dev {

// ---- NINT group levels, MXFP4 block scales: `window` bytes per row and array, one byte per group ----
// Steps of one window.  A lane block of 32 columns lies in one group of 32 or in two of 16 and may straddle two of
// another size; it reads the level of its first group and of the next.  Where a step is a whole number of groups
// (16, 32) a window starts on a step's first group and serves window * group_size / 64 steps; elsewhere the window's
// first group may begin before the step does and the last block may reach one group further: two levels of slack.
MFQ_HD constexpr int level_window_run(int group_size, int window) {
    return 64 % group_size == 0 ? ((window * group_size / 64) & ~1) : (((window - 2) * group_size / 64) & ~1);
}
// First group of the window that serves steps [from, from + run).
MFQ_HD constexpr int level_window_first(int group_size, int from) { return 64 * from / group_size; }
// Bytes of a row the window holds: through the group behind the row's last one (never read as a level that counts).
MFQ_HD constexpr int level_window_bytes(int row_groups, int first, int window) {
    return row_groups - first + 1 < window ? row_groups - first + 1 : window;
}

// ---- NVQ sign masks (28 bits per lane block) and group states (4 bits per group of 24 columns) ----
// Per row and window of `run` steps: 7 bytes of sign masks per step and 4 more (a mask is read as a dword that may
// start in the last byte), at most 8/3 states per step and 4 more bytes, each part a whole number of dwords and the
// row an odd number of them, so that the rows of a wave meet no common bank.
MFQ_HD constexpr int side_window_sign_bytes(int run) { return (7 * run + 4 + 3) & ~3; }
MFQ_HD constexpr int side_window_pitch(int run) {
    const int bytes = side_window_sign_bytes(run) + (((4 * run + 3) / 3 + 4 + 3) & ~3);
    return (bytes & 4) ? bytes : bytes + 4;
}
// The longest run (even, at least 2, at most `longest` and the row's steps) whose windows of `rows` rows fit `room` bytes.
MFQ_HD constexpr int side_window_run(int room, int rows, int steps, int longest) {
    const int limit = steps < longest ? steps : longest;
    int run = 2;
    for (int w = 4; w <= limit; w += 2)
        if (rows * side_window_pitch(w) <= room) run = w;
    return run;
}
// First byte of the window of row `row` in the sign / state stream for a run that starts at step `from`.
MFQ_HD constexpr uint32_t side_window_sign_start(int row, int nsign4, int sign_bit0, int from) {
    return ((static_cast<uint32_t>(row) * static_cast<uint32_t>(nsign4) + 2u * static_cast<uint32_t>(from)) * 28u +
            static_cast<uint32_t>(sign_bit0)) >> 3;
}
MFQ_HD constexpr uint32_t side_window_state_start(int row, int groups, int state_bit0, int from) {
    return ((static_cast<uint32_t>(row) * static_cast<uint32_t>(groups) + 64u * static_cast<uint32_t>(from) / 24u) * 4u +
            static_cast<uint32_t>(state_bit0)) >> 3;
}
// First bit of the four sign masks of lane block `cb` of a row, and of the states of its groups from `group` on.
MFQ_HD constexpr uint32_t side_sign_bit(int row, int nsign4, int sign_bit0, int cb) {
    return (static_cast<uint32_t>(row) * static_cast<uint32_t>(nsign4) + static_cast<uint32_t>(cb)) * 28u + static_cast<uint32_t>(sign_bit0);
}
MFQ_HD constexpr uint32_t side_state_bit(int row, int groups, int state_bit0, int group) {
    return (static_cast<uint32_t>(row) * static_cast<uint32_t>(groups) + static_cast<uint32_t>(group)) * 4u + static_cast<uint32_t>(state_bit0);
}

}  // namespace dev
}  // namespace mfq_amd
