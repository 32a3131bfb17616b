// Host sweep of the LDS windows of the prefill tile kernel (mfq_amd/csrc/tile_windows.h, the code the device runs): the
// group levels of NINT rows, the block scales of MXFP4 rows and the sign masks and states of NVQ rows are staged per
// row for a run of steps, and every read of every step of a run must fall inside what its window holds.  Mirrors the
// loop of tiles_fast_block: windows of 64 levels (tiles of more than 64 pairs) and 88 (lower tiles), side windows of
// up to 8 and 16 steps, and the decode of a step's first chunk one step ahead, which at the end of a run reads the
// window of the run before (values nobody uses, but they must come from the row's own piece of LDS).
// Prints the number of reads checked; exits non-zero at the first violation.
#include "../../mfq_amd/csrc/tile_windows.h"

#include <cstdio>
#include <cstdlib>
#include <initializer_list>

using namespace mfq_amd::dev;

static long long checked = 0;

static void require(bool ok, const char* what, int a, int b, int c, int d, int e) {
    if (ok) return;
    std::fprintf(stderr, "window violation: %s (%d %d %d %d %d)\n", what, a, b, c, d, e);
    std::exit(1);
}

// NINT (one byte per group and array) and MXFP4 (mx: one scale byte per lane block)
template <int GS>
static void sweep_levels(bool mx, int window) {
    const int pitch = window + 4;
    const int run = level_window_run(GS, window);
    require(run >= 2 && run % 2 == 0, "run of a level window", GS, window, run, 0, 0);
    for (int width = 64; width <= 8192; width += 32) {
        const int blocks = width / kLaneColumns;
        const int steps = (blocks + 3) / 4 * 2;
        const int row_groups = mx ? width / 32 : (width + GS - 1) / GS;
        if (!mx && row_groups < 2) continue;                  // such pools take the exact kernels
        const int last = steps - 1;
        for (int from = 0; from < steps; from += run) {
            const int first = level_window_first(GS, from);
            const int bytes = level_window_bytes(row_groups, first, window);
            require(first >= 0 && first < row_groups && bytes >= 1 && bytes <= window, "window start", GS, window, width, from, first);
            const int to = from + run < steps ? from + run : steps;
            for (int step = from; step <= to; ++step) {       // `to`: the step decoded ahead at the end of the run
                const int s = step < last ? step : last;
                for (int h = 0; h < 2; ++h) {
                    const LaneBlock b = lane_block<GS>(2 * s + h, width, row_groups);
                    const int index = b.valid ? (mx ? b.cb : b.group) - first : 0;
                    const int reads = mx ? 1 : 2;             // the level of the block's first group and of the next
                    require(index >= 0 && index + reads <= pitch, "read leaves the row's piece of LDS", GS, window, width, step, h);
                    if (step < to) {
                        // the levels that count lie in what was staged
                        require(index < bytes, "first level not staged", GS, window, width, step, h);
                        if (!mx && b.valid && b.sel != 0u) require(index + 1 < bytes, "second level not staged", GS, window, width, step, h);
                        if (b.valid) require(first + index < row_groups, "level behind the row", GS, window, width, step, h);
                    }
                    ++checked;
                }
            }
        }
    }
}

// NVQ: 28 bits of sign masks per lane block, 4 bits of state per group of 24 columns
static void sweep_side(int longest) {
    for (int width = 64; width <= 8192; width += 32) {
        const int blocks = width / kLaneColumns;
        const int steps = (blocks + 3) / 4 * 2;
        const int groups = (width + 23) / 24, nsign4 = (width + 31) / 32;
        const int last = steps - 1;
        for (int room = 2 * 256 * 28; room <= 64 * 1024; room += 3 * 1024) {
            const int run = side_window_run(room, 256, steps, longest);
            const int sign_bytes = side_window_sign_bytes(run), pitch = side_window_pitch(run);
            require(run >= 2 && run % 2 == 0 && run <= longest && (run <= steps || run == 2), "side run", width, room, run, 0, 0);
            require(run == 2 || 256 * pitch <= room, "side windows exceed their room", width, room, run, pitch, 0);
            require(pitch % 8 == 4 && sign_bytes % 4 == 0, "pitch: an odd number of dwords", width, room, run, pitch, sign_bytes);
            for (int row : {0, 1, 2, 3, 5, 63, 64, 255})
                for (int sign_bit0 : {0, 4})
                    for (int state_bit0 : {0, 4})
                        for (int from = 0; from < steps; from += run) {
                            const int to = from + run < steps ? from + run : steps;
                            for (int step = from; step <= to; ++step) {
                                const int s = step < last ? step : last;
                                for (int h = 0; h < 2; ++h) {
                                    const LaneBlock b = lane_block<24>(2 * s + h, width, groups);
                                    const uint32_t sign_bit = side_sign_bit(row, nsign4, sign_bit0, b.cb);
                                    const uint32_t state_bit = side_state_bit(row, groups, state_bit0, b.group);
                                    const int64_t sign_at = b.valid ? static_cast<int64_t>(sign_bit >> 3) - side_window_sign_start(row, nsign4, sign_bit0, from) : 0;
                                    const int64_t state_at = b.valid ? static_cast<int64_t>(state_bit >> 3) - side_window_state_start(row, groups, state_bit0, from) : 0;
                                    if (step < to) {
                                        // a dword holds the block's 28 bits of masks, a halfword the states of its two groups
                                        require((sign_bit & 7u) + 28u <= 32u && (state_bit & 7u) + 8u <= 16u, "bits leave the word", width, run, row, step, h);
                                        require(sign_at >= 0 && sign_at + 4 <= sign_bytes, "sign masks not staged", width, run, row, step, h);
                                        require(state_at >= 0 && state_at + 2 <= pitch - sign_bytes, "states not staged", width, run, row, step, h);
                                    } else {
                                        // the decode ahead of the next window: anywhere in the row's own piece
                                        require(sign_at >= 0 && sign_at + 4 <= pitch && state_at >= 0 && sign_bytes + state_at + 2 <= pitch + 4,
                                                "read ahead leaves the row's piece of LDS", width, run, row, step, h);
                                    }
                                    ++checked;
                                }
                            }
                        }
        }
    }
}

int main() {
    for (int window : {64, 88}) {
        sweep_levels<16>(false, window);
        sweep_levels<24>(false, window);
        sweep_levels<32>(false, window);
        sweep_levels<48>(false, window);
        sweep_levels<32>(true, window);
    }
    sweep_side(8);
    sweep_side(16);
    std::printf("%lld window reads inside what was staged\n", checked);
    return 0;
}
