// Where the streaming kernels read: the address arithmetic of one (row, lane block) fetch, in plain integer code that
// compiles for the device (fast.cuh uses it) and for the host (tests/cpp/fetch_extent_check.cpp sweeps it against the
// extents of every packed field).  Offsets are bytes from the first byte of the expert's share of a field.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define MFQ_HD __host__ __device__ __forceinline__
#else
#define MFQ_HD inline
#endif

namespace mfq_amd {
namespace dev {

constexpr int kLaneColumns = 32;

// Per-lane constants of one lane block.
struct LaneBlock {
    int cb;            // index of the block in the row, clamped to a valid one
    bool valid;        // the block lies inside the row
    uint32_t sel;      // bit j: chunk j of the block belongs to the lane's second group
    int group;         // first group of the block
    int level_at;      // NINT: group index at which the 16-bit level window is loaded
    int level_shift;   //       and the shift that brings the block's first level to bit 0
};

template <int GS>
MFQ_HD LaneBlock lane_block(int cb, int width, int groups) {
    LaneBlock b;
    b.valid = cb * kLaneColumns < width;
    b.cb = b.valid ? cb : 0;
    b.group = (b.cb * kLaneColumns) / GS;
    // a lane block meets at most two groups (GS >= 16): chunk j lies in the second when it starts at or behind the
    // group's end.  One remainder and four compares; a division per chunk is what the compiler made of the direct form.
    static_assert(GS >= 16, "a lane block of 32 columns spans at most two groups");
    const int rest = GS - (b.cb * kLaneColumns - b.group * GS);     // columns of the first group inside the block
    b.sel = (8 >= rest ? 2u : 0u) | (16 >= rest ? 4u : 0u) | (24 >= rest ? 8u : 0u);
    // two consecutive levels come with one 16-bit load; the window slides back at the last group
    b.level_at = b.group < groups - 2 ? b.group : groups - 2;
    b.level_shift = 8 * (b.group - b.level_at);
    return b;
}

// NINT: `dwords` dwords of codes at code_byte; two bytes (one when a lane block is one group) of each level array at level_byte.
struct NintFetchAt { uint32_t code_byte, level_byte; };
MFQ_HD NintFetchAt nint_fetch_at(int row, int row_bytes, int groups, int bits, int group_size, const LaneBlock& b) {
    NintFetchAt at;
    at.code_byte = static_cast<uint32_t>(row) * static_cast<uint32_t>(row_bytes) + static_cast<uint32_t>(b.cb * (4 * bits));
    at.level_byte = static_cast<uint32_t>(row) * static_cast<uint32_t>(groups) + static_cast<uint32_t>(group_size == 32 ? b.group : b.level_at);
    return at;
}

// NINT level words (the row loop of the decode kernel): instead of every lane loading the two level bytes of its own
// lane block, 32 / rows_per_slot lanes per row and level array load one dword each and the wave hands the bytes out
// with lane permutes (one vector-memory instruction per row slot instead of two, each touching far fewer lanes).
// Word j of a row starts at level stride * j, slid back so that it stays inside the row's own levels; stride 3 where a
// lane block can begin at any level of a word (24- and 48-column groups), so that a block's two levels never straddle
// two words, stride 4 where they cannot (16- and 32-column groups).
MFQ_HD constexpr int nint_level_word_stride(int group_size) { return group_size == 16 || group_size == 32 ? 4 : 3; }
// First level (index inside the row) of word j; needs groups >= 4.
MFQ_HD int nint_level_word_start(int groups, int stride, int j) {
    const int start = stride * j;
    return start < groups - 4 ? start : groups - 4;
}
// The word that holds levels first and first + 1 (first <= groups - 2, or first <= groups - 1 when only one is wanted).
MFQ_HD int nint_level_word_of(int stride, int first) { return first / stride; }
// True when `words_per_row` words cover every lane block of a row.
MFQ_HD bool nint_level_words_cover(int groups, int stride, int words_per_row) {
    return groups >= 4 && nint_level_word_of(stride, groups - 1) < words_per_row;
}

// MXFP4: 16 bytes of nibbles at code_byte, one scale byte at scale_byte.
struct MxFetchAt { uint32_t code_byte, scale_byte; };
MFQ_HD MxFetchAt mx_fetch_at(int row, int row_bytes, const LaneBlock& b) {
    return MxFetchAt{static_cast<uint32_t>(row) * static_cast<uint32_t>(row_bytes) + static_cast<uint32_t>(b.cb * 16),
                     static_cast<uint32_t>(row) * static_cast<uint32_t>(row_bytes / 16) + static_cast<uint32_t>(b.cb)};
}

// NVQ (D4 formats, 4-bit states): what an expert's rows need to know about the flat streams of its pool.
struct NvqExpertAt {
    int64_t index_byte, sign_byte, state_byte;   // first byte of each stream that holds data of the expert
    int limit0, limit1, limit2;                  // bytes of the index / sign / state stream from that byte on (saturated)
    int sign_bit0, state_bit0;                   // bit of the expert's first sign mask / state inside its first byte
};
MFQ_HD NvqExpertAt nvq_expert_at(int64_t first_row, int nvec8, int index_bits, int nsign4, int groups, int64_t size0,
                                 int64_t size1, int64_t size2) {
    NvqExpertAt e;
    e.index_byte = first_row * nvec8 * index_bits;
    const int64_t sign_bit = first_row * nsign4 * 28;
    const int64_t state_bit = first_row * groups * 4;
    e.sign_byte = sign_bit >> 3;
    e.state_byte = state_bit >> 3;
    const int64_t left0 = size0 - e.index_byte, left1 = size1 - e.sign_byte, left2 = size2 - e.state_byte;
    e.limit0 = static_cast<int>(left0 < 0x7fffffff ? left0 : 0x7fffffff);
    e.limit1 = static_cast<int>(left1 < 0x7fffffff ? left1 : 0x7fffffff);
    e.limit2 = static_cast<int>(left2 < 0x7fffffff ? left2 : 0x7fffffff);
    e.sign_bit0 = static_cast<int>(sign_bit & 7);
    e.state_bit0 = static_cast<int>(state_bit & 7);
    return e;
}

// One lane block of one NVQ row: 8 bytes of indices at index_byte and 4 more at third_byte (the wanted position or,
// near the end of the stream, the last 4 bytes of it); 4 bytes of sign masks at sign_byte (28 bits that start on a
// nibble boundary never leave them); 2 bytes of states at state_byte (clamped likewise).  `shifts` carries the bit
// shifts that bring the three words into place: index word [0..7], sign word [8..15], state word [16..].
struct NvqFetchAt { uint32_t index_byte; int third_byte; uint32_t sign_byte; int state_byte; uint32_t shifts; };
MFQ_HD NvqFetchAt nvq_fetch_at(int row, int nvec8, int index_bits, int nsign4, int groups, int limit0, int limit2,
                               int sign_bit0, int state_bit0, const LaneBlock& b) {
    NvqFetchAt at;
    at.index_byte = static_cast<uint32_t>(row) * static_cast<uint32_t>(nvec8 * index_bits) + static_cast<uint32_t>(b.cb * index_bits);
    const int wanted = static_cast<int>(at.index_byte) + 8;
    at.third_byte = wanted < limit0 - 4 ? wanted : limit0 - 4;
    const uint32_t sign_bit = static_cast<uint32_t>(row) * static_cast<uint32_t>(nsign4 * 28) + static_cast<uint32_t>(b.cb * 28 + sign_bit0);
    at.sign_byte = sign_bit >> 3;
    const uint32_t state_bit = static_cast<uint32_t>(row) * static_cast<uint32_t>(groups * 4) + static_cast<uint32_t>(b.group * 4 + state_bit0);
    const int state_byte = static_cast<int>(state_bit >> 3);
    at.state_byte = state_byte < limit2 - 2 ? state_byte : limit2 - 2;
    at.shifts = ((8u * static_cast<uint32_t>(wanted - at.third_byte)) & 31u) | ((sign_bit & 7u) << 8) |
                (((state_bit & 7u) + 8u * static_cast<uint32_t>(state_byte - at.state_byte)) << 16);
    return at;
}

}  // namespace dev
}  // namespace mfq_amd
