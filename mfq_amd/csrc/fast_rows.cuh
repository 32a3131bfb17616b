// The row loop of the streaming kernels: keeps a ring of packed row data in flight and multiplies
// every row with the activations of up to NT tokens held in registers.
#pragma once

#include "fast.cuh"
#include "xpack.cuh"

#include <type_traits>

namespace mfq_amd {
namespace dev {

// Value of lane `index` (a constant) in every lane, through a scalar register.
__device__ __forceinline__ float uniform_lane(float v, int index) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), index));
}

// Value of lane `index` (0..15, a constant once the caller's loop is unrolled) of the lane's own row of 16 lanes:
// one data-parallel move where a shuffle is an LDS round trip.
__device__ __forceinline__ float row_lane(float v, int index) {
    switch (index) {
        case 0: return dpp<0x150>(v);   // row_newbcast:0
        case 1: return dpp<0x151>(v);
        case 2: return dpp<0x152>(v);
        case 3: return dpp<0x153>(v);
        case 4: return dpp<0x154>(v);
        case 5: return dpp<0x155>(v);
        case 6: return dpp<0x156>(v);
        case 7: return dpp<0x157>(v);
        case 8: return dpp<0x158>(v);
        case 9: return dpp<0x159>(v);
        case 10: return dpp<0x15A>(v);
        case 11: return dpp<0x15B>(v);
        case 12: return dpp<0x15C>(v);
        case 13: return dpp<0x15D>(v);
        case 14: return dpp<0x15E>(v);
        default: return dpp<0x15F>(v);
    }
}

// ------------------------------------------------------------ the row loop ----
// Where one token's activations come from.
struct XSource {
    const void* row;     // first element of the token's activation row, or of its packed form (xpack.cuh)
    int dtype;
    bool vector_ok;
    const float* scale;  // kXScaled: {2^-e, 2^e} of the row, readable once the prologue has run
};
constexpr int kXRaw = 0, kXPacked = 1, kXScaled = 2, kXStaged = 3;
// kXStaged: the block has packed the token's row into LDS once (stage_x_row): per lane block of 32 columns the 16
// fp16 pairs in the pair layout of the class and the four chunk sums, kXStagedDwords dwords; XSource::row points
// there and XSource::scale to the factor that scales results back.  Both are readable once the prologue has run.
constexpr int kXStagedDwords = 20;

// One token's activation row into LDS in the kXStaged form; every thread of the block calls it (two barriers inside).
// Thread t packs lane block t, with the arithmetic of pack_block(); `scratch` holds one float per wave.
template <int CLS>
__device__ __forceinline__ void stage_x_row(const void* src, int dtype, bool vector_ok, int width, uint32_t* dst, float* up_out,
                                            float* scratch) {
    const int lane_blocks = (width + kLaneColumns - 1) / kLaneColumns;
    const int t = threadIdx.x;
    const bool active = t < lane_blocks;
    float values[32];
    float largest = 0.0f;
    if (active) {
#pragma unroll
        for (int j = 0; j < 4; ++j) load_x8(src, dtype, 4 * t + j, width, vector_ok, &values[8 * j]);
#pragma unroll
        for (int i = 0; i < 32; ++i) largest = fmaxf(largest, fabsf(values[i]));
    }
    largest = wave_max(largest);
    if (t % kWave == 0) scratch[t / kWave] = largest;
    __syncthreads();
    const int waves = (static_cast<int>(blockDim.x) + kWave - 1) / kWave;
    for (int w = 0; w < waves; ++w) largest = fmaxf(largest, scratch[w]);
    float down, up;
    normaliser(largest, down, up);
    if (t == 0) *up_out = up;
    if (active) {
        _Float16 h[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) h[i] = static_cast<_Float16>(values[i] * down);
        uint32_t out[kXStagedDwords];
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const int first = pair_column<CLS>(k, 0), second = pair_column<CLS>(k, 1);
            half2_t pair;
            pair[0] = static_cast<_Float16>(static_cast<float>(h[first]) * pair_scale<CLS>(k));
            pair[1] = static_cast<_Float16>(static_cast<float>(h[second]) * pair_scale<CLS>(k));
            out[k] = __builtin_bit_cast(uint32_t, pair);
        }
        float plain[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 32; ++i) plain[i / 8] += static_cast<float>(h[i]);
#pragma unroll
        for (int j = 0; j < 4; ++j) out[16 + j] = __float_as_uint(plain[j]);
#pragma unroll
        for (int q = 0; q < kXStagedDwords / 4; ++q)
            *reinterpret_cast<u32x4*>(dst + t * kXStagedDwords + 4 * q) = u32x4{out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]};
    }
    __syncthreads();
}
struct NoPrologue { __device__ __forceinline__ void operator()() const {} };

// Rows [row_begin, row_end) of one expert times NT tokens.  LPR lanes share a row (64, or 16 when the
// row has at most 512 columns and a wave covers four rows at a time); SLABS lane blocks per lane.
// XMODE: where the activations come from.  kXRaw: rows of fp16 / bf16 values (global memory or LDS); the largest
// magnitude is found here.  kXPacked: rows in the packed form of xpack.cuh.  kXScaled: rows of fp16 values whose
// normaliser the caller already knows (XSource::scale_down / scale_up), e.g. values a block staged in LDS.
// `prologue()` runs once, after the first loads of packed rows have been issued and before the activations are
// read: block-wide work (it may contain barriers) that produces the activations overlaps those loads.
// The packed data of RING row slots is in flight at any time: a slot's registers are refilled with
// the slot RING places further on as soon as it has been consumed, so loads overlap the arithmetic
// of the RING - 1 slots in between.  SLOTS > 0: the call covers exactly SLOTS row slots starting at
// row_begin (rows at or beyond row_end are computed on clamped data and not stored) and the whole
// sequence is straight-line code, which lets the compiler wait for exactly the loads a slot needs;
// SLOTS == 0: any number of rows, looped.  store(n, row, value) is called by one lane per (token, row).
// IB: index bits of the NVQ format when known at compile time (0: looked up per row).
// LEVEL_WORDS (NINT classes, one lane block per lane): the group levels of a row slot come as level words (fetch_at.h)
// that the wave shares, instead of two small loads per lane; the caller has checked nint_level_words_cover().
template <int CLS, int LPR, int SLABS, int NT, int RING, int XMODE, int SLOTS, int IB = 0, bool LEVEL_WORDS = false, class Store,
          class Prologue = NoPrologue>
__device__ __forceinline__ void fast_rows(const FastCtx<CLS>& c, const XSource (&xs)[NT], int width, int row_begin,
                                          int row_end, int out_rows, Store&& store, Prologue&& prologue = Prologue()) {
    using C = FastClass<CLS>;
    constexpr int SUBS = kWave / LPR;          // rows per slot
    constexpr int R = RING < 4 ? RING : 4;     // slots whose totals are reduced together
    static_assert(RING % R == 0, "ring depth must be a multiple of the reduction width");
    static_assert(!LEVEL_WORDS || (C::kNint && SLABS == 1), "level words serve NINT rows with one lane block per lane");
    const int lane = threadIdx.x % kWave;
    const int sub = lane / LPR, li = lane % LPR;
    const int slots = (row_end - row_begin + SUBS - 1) / SUBS;

    LaneBlock blocks[SLABS];
#pragma unroll
    for (int s = 0; s < SLABS; ++s) blocks[s] = lane_block<C::kGs>(li + LPR * s, width, c.groups);

    // Level words.  As a loader, lanes 0..31 hold scale levels and lanes 32..63 minimum levels: word `word_j` of row
    // `word_sub` of the slot; as a consumer, the lane takes the word that holds the levels of its block from lane
    // `word_from` (+ 32 for the minima) and shifts them down by `word_shift`.
    constexpr int kWordStride = nint_level_word_stride(C::kGs);
    constexpr int kWordsPerRow = 32 / SUBS;
    const uint8_t* word_array = nullptr;
    int word_sub = 0, word_start = 0, word_from = 0, word_shift = 0;
    if constexpr (LEVEL_WORDS) {
        word_array = lane < 32 ? c.f1 : c.f2;
        word_sub = (lane & 31) / kWordsPerRow;
        word_start = nint_level_word_start(c.groups, kWordStride, (lane & 31) % kWordsPerRow);
        const int first = C::kGs == 32 ? blocks[0].group : blocks[0].level_at;
        const int word = nint_level_word_of(kWordStride, first);
        word_from = 4 * (sub * kWordsPerRow + word);
        word_shift = 8 * (first - nint_level_word_start(c.groups, kWordStride, word)) + (C::kGs == 32 ? 0 : blocks[0].level_shift);
        blocks[0].level_shift = 0;
    }

    auto fetch_slot = [&](int slot, FastRaw<CLS> (&raw)[SLABS]) {
        int row = row_begin + slot * SUBS + sub;
        row = row < out_rows ? row : out_rows - 1;
        if constexpr (LEVEL_WORDS) {
            raw[0] = fast_fetch<CLS, false>(c, blocks[0], row);
            int from = row_begin + slot * SUBS + word_sub;
            from = from < out_rows ? from : out_rows - 1;
            raw[0].a = load_u32_unaligned(word_array + static_cast<uint32_t>(from) * static_cast<uint32_t>(c.groups) +
                                          static_cast<uint32_t>(word_start));
        } else {
#pragma unroll
            for (int s = 0; s < SLABS; ++s) raw[s] = fast_fetch<CLS>(c, blocks[s], row);
        }
    };
    // The levels of the lane's block out of the slot's level words, in the form fast_accumulate() reads them.
    auto with_levels = [&](const FastRaw<CLS>& raw) {
        FastRaw<CLS> out = raw;
        if constexpr (LEVEL_WORDS) {
            out.a = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(word_from, static_cast<int>(raw.a))) >> word_shift;
            out.b = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(word_from + 128, static_cast<int>(raw.a))) >> word_shift;
        }
        return out;
    };

    // Row scalars (NINT scale and minimum, NVQ anchor) of one pass over the ring, one load per array and pass instead
    // of one per row.  64 lanes per row: lane l holds those of the l-th row of the pass.  16 lanes per row: lane i of
    // a row of 16 lanes holds those of that lane group's row in the i-th slot of the pass.
    constexpr int kScalars = C::kNint ? 2 : C::kNvq ? 1 : 0;
    static_assert(RING * SUBS <= kWave && SLOTS * SUBS <= kWave, "the rows of a pass must fit the lanes of a wave");
    static_assert(SUBS == 1 || (LPR == 16 && RING <= 16 && SLOTS <= 16), "a slot of the pass per lane of a row of 16");
    auto fetch_scalars = [&](int slot, float (&values)[2]) {
        int row = SUBS == 1 ? row_begin + slot + lane : row_begin + (slot + li) * SUBS + sub;
        row = row < out_rows ? row : out_rows - 1;
        values[0] = kScalars >= 1 ? gload<float>(c.f3 + row) : 0.0f;
        values[1] = kScalars >= 2 ? gload<float>(c.f4 + row) : 0.0f;
    };
    float scalars[2], next_scalars[2] = {0.0f, 0.0f};
    fetch_scalars(0, scalars);

    FastRaw<CLS> ring[RING][SLABS];
#pragma unroll
    for (int d = 0; d < RING; ++d) {
        if (SLOTS > 0 ? d < SLOTS : d < slots) {
            fetch_slot(d, ring[d]);
        } else {
#pragma unroll
            for (int s = 0; s < SLABS; ++s) ring[d][s] = FastRaw<CLS>{};
        }
    }

    prologue();

    // activations: already packed, or: load, find the largest magnitude of the token, normalise and pack
    XBlock x[SLABS][NT];
    float up[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        if constexpr (XMODE == kXPacked) {
            const uint32_t* row = static_cast<const uint32_t*>(xs[n].row);
            up[n] = gload<float>(row + xpack_scale_at(width));
#pragma unroll
            for (int s = 0; s < SLABS; ++s) xpack_load<CLS>(row, width, blocks[s], x[s][n]);
        } else if constexpr (XMODE == kXStaged) {
            typedef const __attribute__((address_space(3))) u32x4* lds4;
            up[n] = *xs[n].scale;
#pragma unroll
            for (int s = 0; s < SLABS; ++s) {
                const LaneBlock& b = blocks[s];
                const lds4 at = (lds4)(static_cast<const uint32_t*>(xs[n].row) + b.cb * kXStagedDwords);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const u32x4 v = at[i];
                    x[s][n].p[4 * i] = b.valid ? v[0] : 0u; x[s][n].p[4 * i + 1] = b.valid ? v[1] : 0u;
                    x[s][n].p[4 * i + 2] = b.valid ? v[2] : 0u; x[s][n].p[4 * i + 3] = b.valid ? v[3] : 0u;
                }
                const u32x4 plain = at[4];
                x[s][n].g0 = x[s][n].g1 = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool second = (b.sel >> j) & 1u;
                    const float value = b.valid ? __uint_as_float(plain[j]) : 0.0f;
                    x[s][n].g0 += second ? 0.0f : value;
                    x[s][n].g1 += second ? value : 0.0f;
                }
            }
        } else {
            float values[SLABS][32];
            float largest = 0.0f;
#pragma unroll
            for (int s = 0; s < SLABS; ++s) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    load_x8(xs[n].row, xs[n].dtype, 4 * blocks[s].cb + j, width, xs[n].vector_ok, &values[s][8 * j]);
#pragma unroll
                for (int i = 0; i < 32; ++i) largest = fmaxf(largest, blocks[s].valid ? fabsf(values[s][i]) : 0.0f);
            }
            float down;
            if constexpr (XMODE == kXScaled) {
                down = xs[n].scale[0]; up[n] = xs[n].scale[1];
            } else {
                largest = wave_max(largest);
                normaliser(largest, down, up[n]);
            }
#pragma unroll
            for (int s = 0; s < SLABS; ++s) pack_block<CLS>(values[s], down, blocks[s], x[s][n]);
        }
    }

    if constexpr (SLOTS > 0) {
        // lane l of `scalars` holds the scalars of row row_begin + l: all rows of the call
        static_assert(SLOTS % R == 0, "slot count must be a multiple of the reduction width");
#pragma unroll
        for (int g = 0; g < SLOTS / R; ++g) {
            float v[NT][R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int k = g * R + r, d = k % RING;
                float row_v[NT];
#pragma unroll
                for (int n = 0; n < NT; ++n) row_v[n] = 0.0f;
                float rs = 0.0f, rm = 0.0f;
                if (kScalars >= 1) rs = SUBS == 1 ? uniform_lane(scalars[0], k) : row_lane(scalars[0], k);
                if (kScalars >= 2) rm = SUBS == 1 ? uniform_lane(scalars[1], k) : row_lane(scalars[1], k);
#pragma unroll
                for (int s = 0; s < SLABS; ++s) {
                    if (s == 0 && !C::kNvq) fast_accumulate<CLS, NT, IB, false>(c, blocks[s], with_levels(ring[d][s]), rs, rm, x[s], row_v);
                    else fast_accumulate<CLS, NT, IB>(c, blocks[s], with_levels(ring[d][s]), rs, rm, x[s], row_v);
                }
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    asm volatile("" : "+v"(row_v[n]));
                    v[n][r] = row_v[n];
                }
                if (k + RING < SLOTS) fetch_slot(k + RING, ring[d]);
            }
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const float total = reduce_values<R, LPR>(v[n], lane);
                const int row = row_begin + (g * R + reduce_slot<R>(li)) * SUBS + sub;
                if (li < R && row < row_end && row < out_rows) store(n, row, total * up[n]);
            }
        }
        return;
    }

    // One pass over the ring: consume slots k0 .. k0+RING-1, R at a time.  REFILL: every slot is followed
    // by the load of the slot RING places on (the caller guarantees those exist), without branches,
    // so the compiler's wait counts stay exact; otherwise refills are conditional and slots behind
    // the end are skipped.
    auto pass = [&](int k0, auto refill) {
        constexpr bool REFILL = decltype(refill)::value;
        if (REFILL) fetch_scalars(k0 + RING, next_scalars);
#pragma unroll
        for (int g = 0; g < RING / R; ++g) {
            if (!REFILL && g > 0 && k0 + g * R >= slots) break;
            float v[NT][R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int d = g * R + r;
                float row_v[NT];
#pragma unroll
                for (int n = 0; n < NT; ++n) row_v[n] = 0.0f;
                // the scalars of the slot's row: lane d of the pass for 64 lanes per row, else lane d of the lane's
                // own row of 16
                float rs = 0.0f, rm = 0.0f;
                if (kScalars >= 1) rs = SUBS == 1 ? uniform_lane(scalars[0], d) : row_lane(scalars[0], d);
                if (kScalars >= 2) rm = SUBS == 1 ? uniform_lane(scalars[1], d) : row_lane(scalars[1], d);
#pragma unroll
                for (int s = 0; s < SLABS; ++s) {
                    if (s == 0 && !C::kNvq) fast_accumulate<CLS, NT, IB, false>(c, blocks[s], with_levels(ring[d][s]), rs, rm, x[s], row_v);
                    else fast_accumulate<CLS, NT, IB>(c, blocks[s], with_levels(ring[d][s]), rs, rm, x[s], row_v);
                }
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    // the slot's arithmetic stays ahead of its refill: the registers are reused in place
                    asm volatile("" : "+v"(row_v[n]));
                    v[n][r] = row_v[n];
                }
                if (REFILL || k0 + d + RING < slots) fetch_slot(k0 + d + RING, ring[d]);
            }
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const float total = reduce_values<R, LPR>(v[n], lane);
                const int row = row_begin + (k0 + g * R + reduce_slot<R>(li)) * SUBS + sub;
                if (li < R && row < row_end && row < out_rows) store(n, row, total * up[n]);
            }
        }
        if (REFILL) { scalars[0] = next_scalars[0]; scalars[1] = next_scalars[1]; }
    };
    int k0 = 0;
    for (; k0 + 2 * RING <= slots; k0 += RING) pass(k0, std::true_type{});
    for (; k0 < slots; k0 += RING) pass(k0, std::false_type{});
}

}  // namespace dev
}  // namespace mfq_amd
