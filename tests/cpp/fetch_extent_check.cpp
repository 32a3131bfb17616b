// Host sweep of the streaming kernels' address arithmetic (mfq_amd/csrc/fetch_at.h, the code the device runs): for every
// kernel class, width, row count, expert and lane block, every byte a fetch reads must lie inside the packed field it
// reads from, with the field sizes the loader produces (NINT expert streams with their 8 guard bytes counted as
// outside; NVQ streams with no slack at all).  Counterpart of the guard-page tests of the reference
// (cpp_runtime/tests/packed_nint_cpu_test.cpp:128-162, nvq_group_cpu_test.cpp:32-67).  Prints the number of fetches
// checked; exits non-zero at the first violation.
#include "../../mfq_amd/csrc/fetch_at.h"

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>

using namespace mfq_amd::dev;

static long long checked = 0;

static void require(bool ok, const char* what, int cls, int width, int rows, int experts, int local, int row, int cb) {
    if (ok) return;
    std::fprintf(stderr, "read outside the field: %s (class %d width %d rows %d experts %d local %d row %d lane block %d)\n",
                 what, cls, width, rows, experts, local, row, cb);
    std::exit(1);
}

template <int GS>
static void sweep_nint(int bits, int dwords, int width, int rows, int experts) {
    const int groups = (width + GS - 1) / GS;
    if (groups < 2) return;                                   // such pools take the exact kernels
    const int row_bytes = groups * (GS * bits / 8);
    const int64_t stream = static_cast<int64_t>(rows) * row_bytes;        // + 8 guard bytes = q_expert_stride
    const int64_t levels = static_cast<int64_t>(rows) * groups;           // per expert; the arrays hold experts * levels
    for (int local = 0; local < experts; ++local)
        for (int row = 0; row < rows; ++row)
            for (int cb = 0; cb < 128; ++cb) {
                const LaneBlock b = lane_block<GS>(cb, width, groups);
                const NintFetchAt at = nint_fetch_at(row, row_bytes, groups, bits, GS, b);
                require(static_cast<int64_t>(at.code_byte) + 4 * dwords <= stream, "NINT codes", bits * 100 + GS, width, rows, experts, local, row, cb);
                const int level_bytes = GS == 32 ? 1 : 2;
                // the level arrays of the pool: [experts * rows, groups]
                const int64_t absolute = static_cast<int64_t>(local) * levels + at.level_byte;
                require(absolute + level_bytes <= static_cast<int64_t>(experts) * levels, "NINT levels", bits * 100 + GS, width, rows, experts, local, row, cb);
                require(static_cast<int64_t>(at.level_byte) + level_bytes <= static_cast<int64_t>(row + 1) * groups, "NINT levels leave their row", bits * 100 + GS, width, rows, experts, local, row, cb);
                ++checked;
            }
    // the level words of the decode row loop: each stays inside its row's levels, and every lane block finds both of
    // its levels in the word it takes them from, below bit 32 after the shift
    const int stride = nint_level_word_stride(GS);
    for (int words_per_row : {32, 8}) {
        const int lanes_per_row = words_per_row == 32 ? 64 : 16;
        if (width > lanes_per_row * kLaneColumns || !nint_level_words_cover(groups, stride, words_per_row)) continue;
        for (int row = 0; row < rows; ++row)
            for (int j = 0; j < words_per_row; ++j) {
                const int start = nint_level_word_start(groups, stride, j);
                require(start >= 0 && start + 4 <= groups, "NINT level word leaves its row", bits * 100 + GS, width, rows, experts, 0, row, j);
                ++checked;
            }
        for (int cb = 0; cb * kLaneColumns < width; ++cb) {
            const LaneBlock b = lane_block<GS>(cb, width, groups);
            const int first = GS == 32 ? b.group : b.level_at;
            const int word = nint_level_word_of(stride, first);
            const int start = nint_level_word_start(groups, stride, word);
            const int shift = 8 * (first - start) + (GS == 32 ? 0 : b.level_shift);
            require(word < words_per_row && first >= start && shift <= 24, "NINT level word does not hold the block's first level", bits * 100 + GS, width, rows, experts, 0, 0, cb);
            // the second level is wanted only when the block spans two groups
            if (b.sel != 0) require(shift <= 16, "NINT level word does not hold the block's second level", bits * 100 + GS, width, rows, experts, 0, 0, cb);
            ++checked;
        }
    }
}

static void sweep_mx(int width, int rows, int experts) {
    const int row_bytes = width / 2;
    for (int local = 0; local < experts; ++local)
        for (int row = 0; row < rows; ++row)
            for (int cb = 0; cb < 128; ++cb) {
                const LaneBlock b = lane_block<32>(cb, width, width / 32);
                const MxFetchAt at = mx_fetch_at(row, row_bytes, b);
                require(static_cast<int64_t>(at.code_byte) + 16 <= static_cast<int64_t>(rows) * row_bytes, "MXFP4 nibbles", 8, width, rows, experts, local, row, cb);
                require(static_cast<int64_t>(at.scale_byte) + 1 <= static_cast<int64_t>(rows) * (width / 32), "MXFP4 scales", 8, width, rows, experts, local, row, cb);
                ++checked;
            }
}

static void sweep_nvq(int index_bits, int width, int rows, int experts) {
    const int nvec = width / 4, nsign = width / 8, groups = (width + 23) / 24;
    const int nvec8 = nvec / 8, nsign4 = nsign / 4;
    const int64_t total = static_cast<int64_t>(rows) * experts;
    const int64_t size0 = (total * nvec * index_bits + 7) / 8, size1 = (total * nsign * 7 + 7) / 8, size2 = (total * groups * 4 + 7) / 8;
    if (size0 < 16 || size2 < 2) return;                      // such pools take the exact kernels
    for (int local = 0; local < experts; ++local) {
        const NvqExpertAt e = nvq_expert_at(static_cast<int64_t>(local) * rows, nvec8, index_bits, nsign4, groups, size0, size1, size2);
        for (int row = 0; row < rows; ++row)
            for (int cb = 0; cb < 128; ++cb) {
                const LaneBlock b = lane_block<24>(cb, width, groups);
                const NvqFetchAt at = nvq_fetch_at(row, nvec8, index_bits, nsign4, groups, e.limit0, e.limit2, e.sign_bit0, e.state_bit0, b);
                const int cls = 600 + index_bits;
                const int64_t index = e.index_byte + at.index_byte, third = e.index_byte + at.third_byte;
                const int64_t sign = e.sign_byte + at.sign_byte, state = e.state_byte + at.state_byte;
                require(index >= 0 && index + 8 <= size0, "NVQ indices", cls, width, rows, experts, local, row, cb);
                require(third >= 0 && third + 4 <= size0, "NVQ third index word", cls, width, rows, experts, local, row, cb);
                require(sign >= 0 && sign + 4 <= size1, "NVQ sign masks", cls, width, rows, experts, local, row, cb);
                require(state >= 0 && state + 2 <= size2, "NVQ states", cls, width, rows, experts, local, row, cb);
                // and the words hold what the kernel takes from them: 28 sign bits from the shifted word, the wanted
                // index bytes from the third word, both states of the block from the state word
                const uint32_t sign_shift = (at.shifts >> 8) & 0xffu, state_shift = at.shifts >> 16, index_shift = at.shifts & 0xffu;
                require(sign_shift + 28 <= 32, "NVQ sign masks leave their word", cls, width, rows, experts, local, row, cb);
                require(state_shift + 8 <= 16 || b.group + 1 >= groups, "NVQ states leave their word", cls, width, rows, experts, local, row, cb);
                require(index_shift % 8 == 0 && index_shift <= 24, "NVQ third index word shift", cls, width, rows, experts, local, row, cb);
                ++checked;
            }
    }
}

int main() {
    const int widths[] = {32, 64, 96, 128, 480, 512, 544, 1024, 2016, 2048, 2560, 4096};
    const int row_counts[] = {1, 2, 3, 4, 5, 16, 70};
    for (int width : widths)
        for (int rows : row_counts)
            for (int experts : {1, 2, 3}) {
                sweep_nint<16>(2, 2, width, rows, experts);
                sweep_nint<24>(3, 3, width, rows, experts);
                sweep_nint<24>(4, 4, width, rows, experts);
                sweep_nint<32>(4, 4, width, rows, experts);
                sweep_nint<48>(8, 8, width, rows, experts);
                sweep_mx(width, rows, experts);
                for (int index_bits : {8, 9, 10}) sweep_nvq(index_bits, width, rows, experts);
            }
    std::printf("%lld fetches inside their fields\n", checked);
    return 0;
}
