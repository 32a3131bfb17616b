// Prefill: grouped GEMM over routed pairs with 32x32x16 fp16 MFMA into fp32 accumulators.  fp16
// (11-bit significand) is used for both operands: bf16 activations convert to fp16 exactly over the
// activation range, the dequantised weight is rounded once.
//
// Streaming kernel (moe_tiles_fast_kernel): one block = one expert x up to 128 of its routed pairs x
// 256 output rows.  Every lane dequantises the packed weights of its own two rows straight into the
// register layout of the MFMA B operand (fast.cuh: a lane block of 32 columns per load, a few integer
// and packed-fp16 operations per pair), so the weights never pass through LDS and are decoded once
// for all pairs of the tile; the activations of the tile go through LDS, already in the pair order
// of the weight format.  The contraction index of an MFMA may be permuted freely as long as both
// operands agree, which is what lets the weights stay in the order their bits give.
//
// Exact kernel (moe_tiles_kernel): 64 pairs x 64 rows per block on the exact decoders, for the pools
// and geometries the streaming kernel does not serve.
#include "common.h"
#include "decode.cuh"
#include "device_state.h"
#include "fast.cuh"
#include "fp8_split.h"
#include "launch.cuh"
#include "moe_args.h"
#include "tile_pack.cuh"
#include "tile_windows.h"
#include "xpack.cuh"

namespace mfq_amd {
namespace dev {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kExactTileM = 64;          // pairs per block of the exact kernel
constexpr int kTileK = 64;               // columns per slab
constexpr int kLdsStride = kTileK + 8;   // halves per LDS row: 16-byte padding skews the banks

template <int CLS>
__global__ void __launch_bounds__(256) moe_tiles_kernel(RowsArgs a) {
    extern __shared__ unsigned char lds[];
    _Float16* a_tile = reinterpret_cast<_Float16*>(lds);                 // [64 pairs][kLdsStride]
    _Float16* b_tile = a_tile + kExactTileM * kLdsStride;                // [64 rows][kLdsStride]
    unsigned char* tables = reinterpret_cast<unsigned char*>(b_tile + kPrefillTileN * kLdsStride);

    const int slot = a.slot_base + blockIdx.z;
    const int* offsets = a.tile_offsets + slot * kClassSlots;
    const int index = offsets[CLS] + blockIdx.y;
    if (index >= offsets[CLS + 1] || index >= a.tile_capacity) return;
    const int packed = a.tile_items[slot * a.tile_capacity + index];
    const int expert = packed & 0xffff, m_tile = packed >> 16;
    const int pool_index = a.expert_pool[slot * a.experts + expert];
    if (a.exact_only && !(a.pool_class[pool_index] & kPoolExactOnly)) return;
    const mfq_amd_projection& pool = a.pools[pool_index];
    const int local = pool.expert_local ? pool.expert_local[expert] : 0;
    Decoder<CLS> dec;
    dec.init(pool, tables);

    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    // a plan tile holds kPrefillTileM pairs: blockIdx.x walks its halves, then the row tiles
    const int halves = kPrefillTileM / kExactTileM;
    const int begin = a.expert_bounds[expert] + m_tile * kPrefillTileM + (blockIdx.x % halves) * kExactTileM;
    const int end = a.expert_bounds[expert + 1];
    if (begin >= end) return;
    const int n0 = (blockIdx.x / halves) * kPrefillTileN;

    // staging roles: thread -> (row of the tile, two chunks of the slab)
    const int stage_row = tid >> 2, stage_chunk = (tid & 3) * 2;
    const int my_pair = begin + stage_row < end ? a.ids_dst[begin + stage_row] : -1;
    const int element = a.in_dtype == MFQ_AMD_F32 ? 4 : 2;
    const int safe_pair = my_pair >= 0 ? my_pair : 0;
    const int64_t source = a.in_per_pair ? safe_pair : safe_pair / a.top_k;
    const char* x_row = static_cast<const char*>(a.in) + source * a.in_width * element;
    const bool w_valid = n0 + stage_row < a.out_rows;
    typename Decoder<CLS>::Row rr;
    dec.template row<false>(pool, local, w_valid ? n0 + stage_row : a.out_rows - 1, rr);
    __syncthreads();

    // MFMA roles: wave (wm, wn) owns the 32x32 block at (32 wm, 32 wn)
    const int wm = wave >> 1, wn = wave & 1;
    float16_t acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    const int chunks = (a.in_width + 7) / 8;
    for (int k0 = 0; k0 < a.in_width; k0 += kTileK) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int c = k0 / 8 + stage_chunk + j;
            float xv[8], wv[8];
            const int safe_c = c < chunks ? c : chunks - 1;
            load_x8(x_row, a.in_dtype, safe_c, a.in_width, a.in_vector_ok != 0, xv);
            dec.chunk(rr, safe_c, wv);
            half8_t xh, wh;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool inside = c * 8 + i < a.in_width;
                xh[i] = static_cast<_Float16>(inside && my_pair >= 0 ? xv[i] : 0.0f);
                wh[i] = static_cast<_Float16>(inside && w_valid ? wv[i] : 0.0f);
            }
            *reinterpret_cast<half8_t*>(a_tile + stage_row * kLdsStride + (stage_chunk + j) * 8) = xh;
            *reinterpret_cast<half8_t*>(b_tile + stage_row * kLdsStride + (stage_chunk + j) * 8) = wh;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kTileK; kk += 16) {
            const int col = kk + (lane >> 5) * 8;
            const half8_t av = *reinterpret_cast<const half8_t*>(a_tile + (wm * 32 + (lane & 31)) * kLdsStride + col);
            const half8_t bv = *reinterpret_cast<const half8_t*>(b_tile + (wn * 32 + (lane & 31)) * kLdsStride + col);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, acc, 0, 0, 0);
        }
        __syncthreads();
    }

    // D[m][n]: lane holds n = lane % 32 and m = 8*(i/4) + 4*(lane/32) + i%4 for i in 0..15
    const int n = n0 + wn * 32 + (lane & 31);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int m = wm * 32 + 8 * (i / 4) + 4 * (lane >> 5) + (i % 4);
        if (begin + m < end && n < a.out_rows) {
            const int pair = a.ids_dst[begin + m];
            a.out[pair * a.out_pair_stride + (slot - a.slot_base) * a.out_slot_stride + n] = float_to_half_bits(acc[i]);
        }
    }
}


// ------------------------------------------------------------ streaming ----
constexpr int kFastTileN = 256;          // output rows per block: 64 per wave
constexpr int kFastXRow = 144;           // bytes per LDS row: 64 columns of fp16 and 16 bytes that skew the banks
constexpr int kFastXBytes = kPrefillTileM * kFastXRow;
constexpr int kFastLdsBytes = 2 * kFastXBytes;      // activation buffers; the table region and the pair ids follow
// NINT group levels and MXFP4 block scales of the block's rows are staged in LDS for a run of steps at a
// time (in the place of the NVQ tables): a window of levels per row and array.  Reading them per step from
// memory would keep more cache lines per row alive for the whole block than the L2 can hold, and a load of
// one byte per lane touches as many cache lines as the wave has rows.
constexpr int kOutPitch = 2 * kFastTileN + 16;      // bytes per pair of the output tile staged in LDS
// NVQ sign masks and group states of the block's rows are staged the same way, behind the NVQ tables:
// what the tables of the pool leave of their region plus kSideExtraBytes, for runs of up to
// kSideMaxRun steps.
constexpr int kSideExtraBytes = 9600;
constexpr int kTilesFastLdsBytes = kFastLdsBytes + kNvqFastLdsBytes + kSideExtraBytes + kPrefillTileM * 4;   // dynamic LDS of the tile kernel
static_assert(kTilesFastLdsBytes == 80 * 1024, "two blocks share the 160 KB of a CU");
static_assert(kPrefillTileM * kOutPitch <= kFastLdsBytes + kNvqFastLdsBytes, "the output tile reuses the buffers and tables");
// Tiles of at most 64 pairs (two groups of 32) need 8 KB per activation buffer instead of 18: the table region
// starts that much earlier and holds longer windows, so that such a tile restages them less often or never.
constexpr int kLowTileGroups = 2;

__device__ __forceinline__ half8_t as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    return __builtin_bit_cast(half8_t, u32x4{a, b, c, d});
}

// Which of the four fp16 copies of the activations (the spare blocks of route_plan_kernel, swiglu_tiles_kernel) a class reads: the
// pair order of its weights, without the powers of two the row loop's packed form carries.
template <int CLS> __host__ __device__ constexpr int tile_layout() {
    return CLS == K_NINT_8_48 ? 1 : (CLS == K_NVQ_D4 || CLS == K_MXFP4) ? 2 : CLS == K_NINT_2_16 ? 3 : 0;
}

// Loads per call of fast_fetch without the NINT levels and the NVQ side streams (vector memory instructions), for
// exact wait counts.
template <int CLS>
constexpr int fetch_loads() {
    using C = FastClass<CLS>;
    return C::kNvq ? 2 : C::kQ == 8 ? 2 : 1;
}

// Swizzle of the packed activation tile in LDS: rows of 128 bytes, the 16-byte piece c of row r sits at
// position c ^ tile_swizzle(r), which spreads the pieces that the lanes of an MFMA operand read
// (same c, consecutive rows) over all banks.
__device__ __forceinline__ int tile_swizzle(int row) { return ((row & 7) + (row >> 3)) & 7; }

// PACKED: the activations come as fp16 in the pair order of the class (spare blocks of route_plan_kernel,
// swiglu_tiles_kernel) and go to LDS by direct loads; otherwise they are converted in the kernel.
template <int CLS, int MT, int IB, bool PACKED>
__device__ __forceinline__ void tiles_fast_block(const RowsArgs& a, int slot, int row_block, int pool_index, int local, int begin,
                                                 int count, unsigned char* lds) {
    using C = FastClass<CLS>;
    // LDS: two activation buffers | the waves' pieces for packed rows (kStaged) | tables and windows | pair ids
    constexpr bool kLow = PACKED && MT <= kLowTileGroups;
    constexpr bool kStaged = kLow && (CLS == K_NINT_4_24 || CLS == K_NINT_4_32 || CLS == K_MXFP4);
    constexpr int kXBytes = kLow ? kLowTileGroups * 32 * 128 : kFastXBytes;      // one activation buffer
    constexpr int kTablesAt = 2 * kXBytes + (kStaged ? 4 * 4096 : 0);
    constexpr int kTableRoom = kTilesFastLdsBytes - kPrefillTileM * 4 - kTablesAt;
    constexpr int kWindow = kLow ? 88 : 64;          // levels per row and array of a window
    constexpr int kPitch = kWindow + 4;              // an odd number of dwords: the rows of a wave meet no common bank
    constexpr int kSideMaxRun = kLow ? 16 : 8;       // steps per window of NVQ sign masks and states, at most
    static_assert(!(C::kNint || C::kMx) || (C::kMx ? 1 : 2) * kFastTileN * kPitch <= kTableRoom, "the level windows fit");
    unsigned char* x_lds = lds;
    unsigned char* tables = lds + kTablesAt;
    int* pair_ids = reinterpret_cast<int*>(lds + kTilesFastLdsBytes - kPrefillTileM * 4);
    const mfq_amd_projection& pool = a.pools[pool_index];
    if (C::kNvq) nvq_fast_tables(pool, tables);
    const FastCtx<CLS> ctx = fast_ctx<CLS>(pool, local, tables);

    const int tid = threadIdx.x, lane = tid % kWave, wave = uniform(static_cast<int>(tid / kWave));
    const int n = lane & 31, h = lane >> 5;
    const int width = a.in_width, blocks = width / kLaneColumns;
    const int steps = (blocks + 3) / 4 * 2;            // 64 columns per step, an even number of steps
    const bool ragged = !PACKED && blocks % 4 != 0;    // some step meets lane blocks beyond the row (never with packed activations)
    const bool half_in = a.in_dtype == MFQ_AMD_F16;

    // activation staging: thread -> (pair of the tile, one of the two lane blocks of a step)
    const int stage_row = tid >> 1, stage_half = tid & 1;
    const int stage_pair = stage_row < count ? a.ids_dst[begin + stage_row] : -1;
    if (tid < kPrefillTileM) pair_ids[tid] = tid < count ? a.ids_dst[begin + tid] : -1;
    const int64_t source = stage_pair < 0 ? 0 : a.in_per_pair ? stage_pair : stage_pair / a.top_k;
    const unsigned char* x_row = static_cast<const unsigned char*>(a.in) + source * width * 2;
    auto x_load = [&](int step, u32x4 (&raw)[4]) {
        int cb = 2 * step + stage_half;
        cb = cb < blocks ? cb : blocks - 1;
#pragma unroll
        for (int j = 0; j < 4; ++j) raw[j] = *(const MFQ_GLOBAL u32x4*)(x_row + cb * 64 + j * 16);
    };
    auto x_store = [&](int step, const u32x4 (&raw)[4]) {
        // Rows behind the tile's last pair hold finite values nobody uses (their outputs are not stored).
        // Lane blocks behind the end of the row are zero here; the weights they meet are those of a valid
        // block (the loads are clamped), so the products vanish.
        uint32_t p[16];
        if (half_in) x_pairs<CLS, true>(raw, p);
        else x_pairs<CLS, false>(raw, p);
        if (ragged && 2 * step + stage_half >= blocks) {
#pragma unroll
            for (int k = 0; k < 16; ++k) p[k] = 0u;
        }
        unsigned char* dst = x_lds + (step & 1) * kXBytes + stage_row * kFastXRow + stage_half * 64;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<u32x4*>(dst + 16 * j) = u32x4{p[4 * j], p[4 * j + 1], p[4 * j + 2], p[4 * j + 3]};
    };
    // packed activations: the block copies the 32 MT rows the MFMAs read per step, a wave 8 rows of every 32
    // with one direct load of 8 rows x 128 bytes; lane -> (row 32 i + 8 wave + lane / 8, position lane % 8
    // of the row in LDS).  The launch has checked that no step meets a lane block behind the end of the row and that
    // the copy of the activations is below 4 GB (tiles_packed_geometry), so a copy takes its address as a scalar base
    // (layout + step) plus a 32-bit lane offset that never changes: no vector arithmetic per step.
    const unsigned char* packed_base = nullptr;
    uint32_t packed_offset[MT];
    if constexpr (PACKED) {
        const uint16_t* base = a.in_tiles + tile_layout<CLS>() * a.in_tiles_layout_stride;
        packed_base = reinterpret_cast<const unsigned char*>(base);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int r = 32 * i + 8 * wave + lane / 8;
            const int pair = r < count ? a.ids_dst[begin + r] : -1;
            const int64_t from = pair < 0 ? 0 : a.in_per_pair ? pair : pair / a.top_k;
            const int piece = (lane % 8) ^ tile_swizzle(r);
            packed_offset[i] = static_cast<uint32_t>(from * width * 2 + piece * 16);
        }
    }
    auto x_direct = [&](int step) {
        // the same address in every lane; said so for the "s" operand below
        const uintptr_t address = reinterpret_cast<uintptr_t>(packed_base + step * 128);
        const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(address)));
        const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(address >> 32)));
        const unsigned char* from = reinterpret_cast<const unsigned char*>((static_cast<uintptr_t>(hi) << 32) | lo);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            unsigned char* to = x_lds + (step & 1) * kXBytes + (32 * i + 8 * wave) * 128;
            // written as assembly so that the compiler does not make every later LDS read wait for it; the
            // waits that cover these loads are the explicit ones before the barriers
            const uint32_t lds_at = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(
                reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char*)(to)))));
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :: "v"(packed_offset[i]), "s"(from), "s"(lds_at) : "memory", "m0");
        }
    };
    // byte offsets of the operand pieces a lane reads inside a group of 32 rows; the swizzle of row
    // 32 mt + m differs between even and odd mt
    int a_piece[2][4];
#pragma unroll
    for (int parity = 0; parity < 2; ++parity)
#pragma unroll
        for (int j = 0; j < 4; ++j) a_piece[parity][j] = n * 128 + (((4 * h + j) ^ tile_swizzle(n + 32 * parity)) << 4);

    // weights: lane -> rows n and n + 32 of the wave's 64, lane block 2 * step + h
    const int n0 = row_block * kFastTileN + wave * 64;
    int rows[2];
    WeightRow<CLS> scale[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        rows[t] = n0 + 32 * t + n;
        rows[t] = rows[t] < a.out_rows ? rows[t] : a.out_rows - 1;
        scale[t] = weight_row<CLS>(ctx, rows[t]);
    }
    auto fetch = [&](int step, FastRaw<CLS> (&raw)[2]) {
        int last = steps - 1;
        const LaneBlock b = lane_block<C::kGs>(2 * (step < last ? step : last) + h, width, ctx.groups);
#pragma unroll
        for (int t = 0; t < 2; ++t) raw[t] = fast_fetch<CLS, false>(ctx, b, rows[t]);   // levels, block scales, signs and states come from LDS
    };
    // NINT, MXFP4: steps [from, from + run) read their levels from a window of kWindow groups per row.  A lane block
    // of 32 columns lies in one group of 32 and may straddle two shorter or longer ones.
    constexpr bool kWindows = C::kNint || C::kMx;
    constexpr int kWindowArrays = C::kMx ? 1 : 2;
    const int row_groups = C::kMx ? ctx.row_bytes / 16 : ctx.groups;
    const int level_run = kWindows ? level_window_run(C::kGs, kWindow) : steps;
    int level_first = 0;           // first group of the staged window
    auto stage_levels = [&](int from) {
        level_first = level_window_first(C::kGs, from);
        // thread -> one row of the block: up to kWindow bytes of each array, every load issued before
        // the first store so that the copy costs one memory round trip
        const int64_t level_bytes = static_cast<int64_t>(pool.output_rows) * row_groups;   // per expert and array
        const int want = level_window_bytes(row_groups, level_first, kWindow);
        int row = row_block * kFastTileN + tid;
        row = row < a.out_rows ? row : a.out_rows - 1;
        const int64_t at = static_cast<int64_t>(row) * row_groups + level_first;
        constexpr int kPieces = (kWindow + 15) / 16;
        u32x4 piece[kWindowArrays][kPieces];
#pragma unroll
        for (int which = 0; which < kWindowArrays; ++which) {
            const uint8_t* base = which ? ctx.f2 : ctx.f1;
#pragma unroll
            for (int q = 0; q < kPieces; ++q) {
                piece[which][q] = u32x4{0u, 0u, 0u, 0u};
                if (16 * q >= want) continue;
                if (at + 16 * q + 16 <= level_bytes) {
                    piece[which][q] = *(const MFQ_GLOBAL u32x4_u*)(base + at + 16 * q);
                } else {
                    // the last bytes of the expert's array
                    for (int k = 0; k < 16; ++k)
                        if (at + 16 * q + k < level_bytes)
                            piece[which][q][k / 4] |= static_cast<uint32_t>(gload<uint8_t>(base + at + 16 * q + k)) << (8 * (k % 4));
                }
            }
        }
#pragma unroll
        for (int which = 0; which < kWindowArrays; ++which)
#pragma unroll
            for (int q = 0; q < kPieces; ++q)
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (16 * q + 4 * k < kPitch)
                        *reinterpret_cast<uint32_t*>(tables + (which * kFastTileN + tid) * kPitch + 16 * q + 4 * k) = piece[which][q][k];
    };
    auto level_pair = [&](int which, int t, const LaneBlock& b) {
        // (a lane block behind the end of the row, which only the converting path meets, multiplies zero activations; it
        // reads the window's first levels, which are there)
        const unsigned char* at = tables + (which * kFastTileN + wave * 64 + 32 * t + n) * kPitch + (PACKED || b.valid ? b.group - level_first : 0);
        return static_cast<uint32_t>(at[0]) | (static_cast<uint32_t>(at[1]) << 8);
    };
    // MXFP4: the scale byte of lane block b of row t (a lane block is one group)
    auto scale_byte = [&](int t, const LaneBlock& b) {
        // (behind the end of the row: the window's first scale, a finite factor for weights that meet zero activations)
        return static_cast<uint32_t>(tables[(wave * 64 + 32 * t + n) * kPitch + (PACKED || b.valid ? b.cb - level_first : 0)]);
    };

    // NVQ: steps [from, from + run) read sign masks and states from LDS windows of one row each
    unsigned char* side = tables;
    int side_run = steps, side_pitch = 0, side_sign_bytes = 0, side_from = 0;
    if constexpr (C::kNvq) {
        const int banks = nvq_format_jsc(pool.format) ? static_cast<uint8_t>(static_cast<const int8_t*>(pool.fields[4])[1]) : 1;
        const int used = (64 + 64 + 128 * 16 + banks * ctx.entries * 8 + 15) / 16 * 16;
        const int room = kTableRoom - used;
        side = tables + used;
        // per row and step: 7 bytes of sign masks (two lane blocks of 28 bits) and at most 8/3 states of 4 bits
        side_run = side_window_run(room, kFastTileN, steps, kSideMaxRun);
        side_sign_bytes = side_window_sign_bytes(side_run);
        side_pitch = side_window_pitch(side_run);
    }
    // first byte of the window of row `row` in the sign / state stream for a run that starts at step `from`
    auto sign_start = [&](int row, int from) { return side_window_sign_start(row, ctx.nsign4, ctx.sign_bit0, from); };
    auto state_start = [&](int row, int from) { return side_window_state_start(row, ctx.groups, ctx.state_bit0, from); };
    auto stage_side = [&](int from) {
        side_from = from;
        int row = row_block * kFastTileN + tid;
        row = row < a.out_rows ? row : a.out_rows - 1;
        constexpr int kSignPieces = (7 * kSideMaxRun + 4 + 15) / 16, kStatePieces = ((4 * kSideMaxRun + 3) / 3 + 4 + 15) / 16;
        u32x4 piece[kSignPieces + kStatePieces];
#pragma unroll
        for (int q = 0; q < kSignPieces + kStatePieces; ++q) {
            const bool sign = q < kSignPieces;
            const uint8_t* base = sign ? ctx.f1 : ctx.f2;
            const int64_t limit = sign ? ctx.limit1 : ctx.limit2;
            const int64_t at = (sign ? sign_start(row, from) : state_start(row, from)) + 16 * (sign ? q : q - kSignPieces);
            const int want = sign ? side_sign_bytes : side_pitch - side_sign_bytes;
            piece[q] = u32x4{0u, 0u, 0u, 0u};
            if (16 * (sign ? q : q - kSignPieces) >= want) continue;
            if (at + 16 <= limit) {
                piece[q] = *(const MFQ_GLOBAL u32x4_u*)(base + at);
            } else {
                for (int k = 0; k < 16; ++k)
                    if (at + k < limit) piece[q][k / 4] |= static_cast<uint32_t>(gload<uint8_t>(base + at + k)) << (8 * (k % 4));
            }
        }
        unsigned char* to = side + tid * side_pitch;
#pragma unroll
        for (int q = 0; q < kSignPieces + kStatePieces; ++q) {
            const bool sign = q < kSignPieces;
            const int offset = sign ? 16 * q : side_sign_bytes + 16 * (q - kSignPieces);
            const int end = sign ? side_sign_bytes : side_pitch;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (offset + 4 * k < end) *reinterpret_cast<uint32_t*>(to + offset + 4 * k) = piece[q][k];
        }
    };
    // sign masks (28 bits from bit 0) and states (8 bits from bit 0) of lane block b of row t
    auto side_pair = [&](int t, const LaneBlock& b, uint32_t& masks, uint32_t& states) {
        const unsigned char* window = side + (wave * 64 + 32 * t + n) * side_pitch;
        const uint32_t sign_bit = side_sign_bit(rows[t], ctx.nsign4, ctx.sign_bit0, b.cb);
        const uint32_t state_bit = side_state_bit(rows[t], ctx.groups, ctx.state_bit0, b.group);
        // (behind the end of the row: the window's first bytes)
        const uint32_t sign_at = PACKED || b.valid ? (sign_bit >> 3) - sign_start(rows[t], side_from) : 0u;
        const uint32_t state_at = PACKED || b.valid ? (state_bit >> 3) - state_start(rows[t], side_from) : 0u;
        const uint32_t sign_word = *reinterpret_cast<const unaligned_u32*>(window + sign_at);
        const uint32_t state_word = *reinterpret_cast<const unaligned_u16*>(window + side_sign_bytes + state_at);
        masks = sign_word >> (sign_bit & 7u);
        states = state_word >> (state_bit & 7u);
    };

    // Packed rows in coalesced runs (kStaged: tiles of at most 64 pairs, classes whose lane blocks hold 16 bytes).  A
    // weight load of the lane that will decode the data touches 32 rows x 32 bytes, and the address unit's time per load
    // instruction follows the cache lines it touches, not the bytes it brings.  Here a wave loads the 64-byte runs that
    // its 64 rows need for two steps with four lanes per row (16 rows per instruction: half the lines), parks them in a
    // 4 KB piece of LDS of its own and reads them back in the layout of the MFMA operand, one 16-byte piece per lane,
    // row and step.  Nothing is shared between waves, so no barrier is involved; the pieces of a row are swizzled so
    // that neither the writes nor the reads meet in a bank.  The runs of the pair of steps after next are requested when
    // those of the next pair have been read back, two steps before they are needed.
    u32x4 staged_rows[4] = {};
    unsigned char* wave_stage = lds + 2 * kXBytes + wave * 4096;
    auto stage_issue = [&](int pair_of_steps) {
        const int last = steps / 2 - 1;
        const int d = pair_of_steps < last ? pair_of_steps : last;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int row = row_block * kFastTileN + wave * 64 + 16 * i + (lane >> 2);
            row = row < a.out_rows ? row : a.out_rows - 1;
            const uint8_t* at = ctx.f0 + static_cast<uint32_t>(row) * static_cast<uint32_t>(ctx.row_bytes) +
                                static_cast<uint32_t>((4 * d + (lane & 3)) * 16);
            staged_rows[i] = *(const MFQ_GLOBAL u32x4_u*)at;
        }
    };
    auto stage_swizzle = [](int row) { return (row >> 1) & 3; };
    auto stage_commit = [&](FastRaw<CLS> (&even)[2], FastRaw<CLS> (&odd)[2]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 16 * i + (lane >> 2);
            *reinterpret_cast<u32x4*>(wave_stage + r * 64 + (((lane & 3) ^ stage_swizzle(r)) << 4)) = staged_rows[i];
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int r = 32 * t + n;
            const u32x4 first = *reinterpret_cast<const u32x4*>(wave_stage + r * 64 + ((h ^ stage_swizzle(r)) << 4));
            const u32x4 second = *reinterpret_cast<const u32x4*>(wave_stage + r * 64 + (((2 + h) ^ stage_swizzle(r)) << 4));
#pragma unroll
            for (int k = 0; k < 4; ++k) { even[t].q[k] = first[k]; odd[t].q[k] = second[k]; }
        }
    };

    float16_t acc[2][MT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[t][mt][i] = 0.0f;

    FastRaw<CLS> ring[2][2] = {};
    u32x4 x_raw[4];
    if constexpr (PACKED) {
        x_direct(0);
    } else {
        x_load(0, x_raw);
    }
    if constexpr (kStaged) {
        stage_issue(0);
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");   // the direct loads, not the weights
        stage_commit(ring[0], ring[1]);
        stage_issue(1);
    } else {
        fetch(0, ring[0]);
        fetch(1, ring[1]);
        if constexpr (PACKED) {
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * 2 * fetch_loads<CLS>()) : "memory");   // the direct loads, not the weights
        } else {
            x_store(0, x_raw);
        }
    }

    // One step: 64 columns.  The activations of the next step are requested first; the weights are
    // decoded chunk by chunk (8 columns per lane) between the MFMAs that consume them, and once the
    // last chunk is out of the packed registers those are refilled with the step after next.
    auto step_body = [&](int step, FastRaw<CLS> (&raw)[2]) {
        if constexpr (!PACKED) {
            x_load(step + 1 < steps ? step + 1 : steps - 1, x_raw);
            asm volatile("" ::: "memory");   // the requests go out now, a whole step ahead of their use
        }
        const LaneBlock b = lane_block<C::kGs>(2 * step + h, width, ctx.groups);
        WeightBlock<CLS> block[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            uint32_t scales = 0, minima = 0;
            if constexpr (C::kNint) { scales = level_pair(0, t, b); minima = level_pair(1, t, b); }
            if constexpr (C::kNvq) side_pair(t, b, scales, minima);
            if constexpr (C::kMx) raw[t].a = scale_byte(t, b);
            block[t] = weight_block<CLS>(ctx, b, raw[t], scale[t], scales, minima);
        }
        const unsigned char* x_tile = x_lds + (step & 1) * kXBytes + (PACKED ? 0 : n * kFastXRow + h * 64);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t w[2][4];
#pragma unroll
            for (int t = 0; t < 2; ++t) chunk_weights<CLS, IB>(block[t], raw[t], j, w[t]);
            if (PACKED && j == 0) {
                // The weights of this step have arrived (chunk 0 waited for them); the activations of the next
                // step are requested now, so that no wait for older loads also waits for these.
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int m = 0; m < 4; ++m) asm volatile("" : "+v"(w[t][m]));
                x_direct(step + 1 < steps ? step + 1 : steps - 1);
            }
            if (j == 3) {
                // every packed register has been read: pin that before the refill reuses them
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int m = 0; m < 4; ++m) asm volatile("" : "+v"(w[t][m]));
                fetch(step + 2, raw);
            }
            const half8_t b0 = as_half8(w[0][0], w[0][1], w[0][2], w[0][3]);
            const half8_t b1 = as_half8(w[1][0], w[1][1], w[1][2], w[1][3]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const half8_t av = PACKED ? *reinterpret_cast<const half8_t*>(x_tile + mt * 32 * 128 + a_piece[mt & 1][j])
                                          : *reinterpret_cast<const half8_t*>(x_tile + mt * 32 * kFastXRow + j * 16);
                acc[0][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, b0, acc[0][mt], 0, 0, 0);
                acc[1][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, b1, acc[1][mt], 0, 0, 0);
            }
        }
        if constexpr (PACKED) {
            // this wave's direct loads have landed; only the weight loads issued after them may be pending
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * fetch_loads<CLS>()) : "memory");
        } else {
            x_store(step + 1, x_raw);
        }
        __syncthreads();
    };
    // The same step as a software pipeline (packed activations): while the MFMAs of chunk j run, the weights of
    // chunk j + 1 are decoded and its activation operands read from LDS, so that the matrix pipe, the vector pipe
    // and the LDS work at the same time inside one wave.  The first chunk of a step is decoded during the last
    // chunk of the step before it (`block`, `wq` carry it across the barrier).  The order of the instructions of a
    // chunk is prescribed to the scheduler: one MFMA, an LDS read, a share of the vector instructions.
    WeightBlock<CLS> block[2];
    uint32_t wq[2][4];
    auto a_read = [&](int step, int j, half8_t (&av)[MT]) {
        const unsigned char* x_tile = x_lds + (step & 1) * kXBytes;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) av[mt] = *reinterpret_cast<const half8_t*>(x_tile + mt * 32 * 128 + a_piece[mt & 1][j]);
    };
    auto decode_first = [&](int step, FastRaw<CLS> (&raw)[2]) {
        const int last = steps - 1;
        const LaneBlock b = lane_block<C::kGs>(2 * (step < last ? step : last) + h, width, ctx.groups);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            uint32_t scales = 0, minima = 0;
            if constexpr (C::kNint) { scales = level_pair(0, t, b); minima = level_pair(1, t, b); }
            if constexpr (C::kNvq) side_pair(t, b, scales, minima);
            if constexpr (C::kMx) raw[t].a = scale_byte(t, b);
            block[t] = weight_block<CLS>(ctx, b, raw[t], scale[t], scales, minima);
            chunk_weights<CLS, IB>(block[t], raw[t], 0, wq[t]);
        }
    };
    // vector instructions of one chunk of two rows, roughly: what the scheduler spreads between the MFMAs
    constexpr int kChunkValu = C::kNvq ? 72 : C::kMx ? 12 : C::kBits == 3 ? 40 : 32;
    // ... and of the last chunk of a step, which also sets up the next step's lane blocks and requests packed rows
    constexpr int kLastValu = kChunkValu + (C::kNint ? 72 : C::kNvq ? 56 : 20);
    auto step_piped = [&](int step, FastRaw<CLS> (&raw)[2], FastRaw<CLS> (&raw_next)[2], auto odd_step) {
        constexpr bool kOdd = decltype(odd_step)::value;
        half8_t aq[MT];
        a_read(step, 0, aq);
        x_direct(step + 1 < steps ? step + 1 : steps - 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            __builtin_amdgcn_sched_barrier(0);
            uint32_t wn[2][4];
            half8_t an[MT];
            const half8_t b0 = as_half8(wq[0][0], wq[0][1], wq[0][2], wq[0][3]);
            const half8_t b1 = as_half8(wq[1][0], wq[1][1], wq[1][2], wq[1][3]);
            if (j < 3) {
#pragma unroll
                for (int t = 0; t < 2; ++t) chunk_weights<CLS, IB>(block[t], raw[t], j + 1, wn[t]);
                a_read(step, j + 1, an);
            } else {
                // every chunk of this step is decoded: the packed registers take the step after next, and the
                // first chunk of the next step is decoded from the other ring slot (into wq: b0 and b1 hold this chunk)
                if constexpr (kStaged) {
                    if constexpr (kOdd) {
                        // the runs of the next two steps into both ring slots, the runs of the two after them requested
                        stage_commit(raw_next, raw);
                        stage_issue((step + 3) / 2);
                    }
                } else {
                    fetch(step + 2, raw);
                }
                decode_first(step + 1, raw_next);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[0][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aq[mt], b0, acc[0][mt], 0, 0, 0);
                acc[1][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aq[mt], b1, acc[1][mt], 0, 0, 0);
            }
            constexpr int kShare = (kChunkValu + 2 * MT - 1) / (2 * MT), kLastShare = (kLastValu + 2 * MT - 1) / (2 * MT);
            if (j < 3) {
#pragma unroll
                for (int i = 0; i < 2 * MT; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);        // an LDS read
                    __builtin_amdgcn_sched_group_barrier(0x002, kShare, 0);   // vector instructions
                }
            } else {
#pragma unroll
                for (int i = 0; i < 2 * MT; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);        // a request for packed rows
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, kLastShare, 0);
                }
            }
            if (j < 3) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int m = 0; m < 4; ++m) wq[t][m] = wn[t][m];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) aq[mt] = an[mt];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // this wave's direct loads have landed; only the weight loads issued after them may be pending
        constexpr int kLoadsBehind = kStaged ? (kOdd ? 4 : 0) : 2 * fetch_loads<CLS>();
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kLoadsBehind) : "memory");
        __syncthreads();
    };
    const int run = C::kNvq ? side_run : level_run;
    for (int from = 0; from < steps; from += run) {
        // every wave is past the last step of the previous run (its closing barrier) when the window moves
        if constexpr (kWindows) stage_levels(from);
        if constexpr (C::kNvq) stage_side(from);
        __syncthreads();
        const int to = from + run < steps ? from + run : steps;
        if constexpr (PACKED) {
            decode_first(from, ring[0]);     // `from` is even: the run's first step reads ring slot 0
            for (int step = from; step < to; step += 2) {
                step_piped(step, ring[0], ring[1], std::false_type{});
                step_piped(step + 1, ring[1], ring[0], std::true_type{});
            }
        } else {
            for (int step = from; step < to; step += 2) {
                step_body(step, ring[0]);
                step_body(step + 1, ring[1]);
            }
        }
    }

    // D[m][n]: the lane holds row n of the weights and pairs m = 8 * (i / 4) + 4 * h + i % 4 of each 32.
    // The tile goes through LDS (every wave is past the last barrier, the buffers are free) so that a
    // pair's 256 outputs leave as 16-byte stores of one contiguous run.
    unsigned char* tile = lds;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int m = 32 * mt + 8 * (i / 4) + 4 * h + (i % 4);
                *reinterpret_cast<uint16_t*>(tile + m * kOutPitch + (wave * 64 + 32 * t + n) * 2) =
                    float_to_half_bits(acc[t][mt][i] * scale[t].factor);
            }
    __syncthreads();
    uint16_t* out = a.out + (slot - a.slot_base) * a.out_slot_stride + row_block * kFastTileN;
    const int columns = a.out_rows - row_block * kFastTileN;          // outputs of the block that exist
    const bool wide = (a.out_pair_stride % 8 == 0) && (a.out_slot_stride % 8 == 0) && (reinterpret_cast<uintptr_t>(a.out) % 16 == 0);
    const int piece = tid % 32, sub = tid / 32;
    for (int m = sub; m < count; m += 8) {
        const int pair = pair_ids[m];
        const u32x4 v = *reinterpret_cast<const u32x4*>(tile + m * kOutPitch + piece * 16);
        uint16_t* to = out + pair * a.out_pair_stride + piece * 8;
        if (wide && piece * 8 + 8 <= columns) {
            *reinterpret_cast<u32x4*>(to) = v;
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (piece * 8 + k < columns) to[k] = static_cast<uint16_t>(v[k / 2] >> (16 * (k % 2)));
        }
    }
}

template <int CLS, int IB, bool PACKED>
__device__ __forceinline__ void tiles_fast_sized(const RowsArgs& a, int slot, int row_block, int pool, int local, int begin,
                                                 int count, unsigned char* lds) {
    if (count <= 32) tiles_fast_block<CLS, 1, IB, PACKED>(a, slot, row_block, pool, local, begin, count, lds);
    else if (count <= 64) tiles_fast_block<CLS, 2, IB, PACKED>(a, slot, row_block, pool, local, begin, count, lds);
    else if (count <= 96) tiles_fast_block<CLS, 3, IB, PACKED>(a, slot, row_block, pool, local, begin, count, lds);
    else tiles_fast_block<CLS, 4, IB, PACKED>(a, slot, row_block, pool, local, begin, count, lds);
}

template <int CLS, bool PACKED>
__device__ __forceinline__ void tiles_fast_class(const RowsArgs& a, int slot, int row_block, int pool, int local, int begin,
                                                 int count, unsigned char* lds) {
    if constexpr (CLS == K_NVQ_D4) {
        const int index_bits = nvq_format_index_bits(a.pools[pool].format);
        if (index_bits == 10) tiles_fast_sized<CLS, 10, PACKED>(a, slot, row_block, pool, local, begin, count, lds);
        else if (index_bits == 9) tiles_fast_sized<CLS, 9, PACKED>(a, slot, row_block, pool, local, begin, count, lds);
        else tiles_fast_sized<CLS, 8, PACKED>(a, slot, row_block, pool, local, begin, count, lds);
    } else {
        tiles_fast_sized<CLS, 0, PACKED>(a, slot, row_block, pool, local, begin, count, lds);
    }
}

// One launch for every format the streaming path serves: blockIdx.y walks the plan's tiles of all
// classes and each block branches once into the class of its expert's pool.
template <bool PACKED>
__global__ void __launch_bounds__(256, 2) moe_tiles_fast_kernel(RowsArgs a) {
    extern __shared__ unsigned char lds[];
    // Workgroups go to the eight XCDs round-robin by their linear index.  The blocks that read the same
    // activation tile (every row block and slot of one plan tile) take indices 8 apart, so they run on
    // one XCD at about the same time and its L2 serves all but the first read of the tile.
    const int row_blocks = (a.out_rows + kFastTileN - 1) / kFastTileN;
    const int sharers = row_blocks * a.tile_slots;
    const int id = blockIdx.x;
    const int index = id / (8 * sharers) * 8 + id % 8;
    const int sub = id % (8 * sharers) / 8;
    const int row_block = sub / a.tile_slots;
    const int slot = a.slot_base + sub % a.tile_slots;
    const int* offsets = a.tile_offsets + slot * kClassSlots;
    if (index >= offsets[K_CLASS_COUNT] || index >= a.tile_capacity) return;
    const int packed = a.tile_items[slot * a.tile_capacity + index];
    const int expert = packed & 0xffff, m_tile = packed >> 16;
    int pool, local, cls;
    if (a.expert_info != nullptr) {
        const ExpertInfo info = a.expert_info[slot * a.experts + expert];
        pool = info.pool; local = info.local; cls = info.cls;
    } else {
        pool = a.expert_pool[slot * a.experts + expert];
        if (pool < 0) return;
        local = a.pools[pool].expert_local ? a.pools[pool].expert_local[expert] : 0;
        cls = a.pool_class[pool];
    }
    if (pool < 0) return;
    const int begin = a.expert_bounds[expert] + m_tile * kPrefillTileM;
    const int left = a.expert_bounds[expert + 1] - begin;
    const int count = left < kPrefillTileM ? left : kPrefillTileM;
    if (count <= 0) return;
    switch (cls) {
        case K_NINT_2_16: tiles_fast_class<K_NINT_2_16, PACKED>(a, slot, row_block, pool, local, begin, count, lds); break;
        case K_NINT_3_24: tiles_fast_class<K_NINT_3_24, PACKED>(a, slot, row_block, pool, local, begin, count, lds); break;
        case K_NINT_4_24: tiles_fast_class<K_NINT_4_24, PACKED>(a, slot, row_block, pool, local, begin, count, lds); break;
        case K_NINT_4_32: tiles_fast_class<K_NINT_4_32, PACKED>(a, slot, row_block, pool, local, begin, count, lds); break;
        case K_NINT_8_48: tiles_fast_class<K_NINT_8_48, PACKED>(a, slot, row_block, pool, local, begin, count, lds); break;
        case K_NVQ_D4: tiles_fast_class<K_NVQ_D4, PACKED>(a, slot, row_block, pool, local, begin, count, lds); break;
        case K_MXFP4: if (!a.skip_mxfp4) tiles_fast_class<K_MXFP4, PACKED>(a, slot, row_block, pool, local, begin, count, lds); break;
        default: break;   // pools marked kPoolExactOnly and classes without a streaming path
    }
}

// ------------------------------------------------- MXFP4 on the block-scaled MFMA ----
// v_mfma_scale_f32_32x32x64_f8f6f4: D[32 x 32] += (A * 2^(sa-127)) (B * 2^(sb-127)) over 64 columns in two blocks of 32,
// one E8M0 scale per row and block: lanes 0..31 bring the scales of block 0, lanes 32..63 those of block 1.  Where the
// columns lie depends on the operand's format.  A 4-bit operand has its lane hold the 32 columns of its block (16 bytes,
// low nibble first), which is the MXFP4 storage itself: 16 bytes of nibbles and one scale byte per 32 columns of a
// weight row go into B as they lie in memory, no arithmetic.  An 8-bit operand has lane half h hold columns
// 16 h .. 16 h + 15 of block 0 in its first four registers and the same columns of block 1 in the other four.  The
// activations come as E4M3 terms (fp8_split.h) that add up to the source exactly, one MFMA per term; fp32 accumulation.
// A block = one plan tile (up to 128 pairs of one expert) x 256 output rows, a wave 64 of the rows, as in the
// streaming tile kernel.  Every lane of a wave must be active at the MFMA: lanes switched off read as zero operands.
typedef int i32x8 __attribute__((ext_vector_type(8)));

template <int MT, int TERMS>
__device__ __forceinline__ void tiles_mx_scaled_block(const RowsArgs& a, int slot, int row_block, const mfq_amd_projection& pool, int local,
                                                      int begin, int count) {
    const int tid = threadIdx.x, lane = tid % kWave, wave = uniform(static_cast<int>(tid / kWave));
    const int n = lane & 31, h = lane >> 5;
    const int width = a.in_width, blocks = width / kLaneColumns;
    const int steps = (blocks + 1) / 2;
    const int64_t first_row = static_cast<int64_t>(local) * pool.output_rows;
    const uint8_t* codes = static_cast<const uint8_t*>(pool.fields[0]) + first_row * (width / 2);
    const uint8_t* scales = static_cast<const uint8_t*>(pool.fields[1]) + first_row * blocks;
    // weights: lane -> rows n and n + 32 of the wave's 64
    const int n0 = row_block * kFastTileN + wave * 64;
    int rows[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        rows[t] = n0 + 32 * t + n;
        rows[t] = rows[t] < a.out_rows ? rows[t] : a.out_rows - 1;
    }
    // activations: lane -> pair 32 mt + n of the tile (clamped: rows behind the last pair are computed and not stored)
    const uint8_t* x_rows[MT];
    const uint8_t* x_scales[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = 32 * mt + n;
        const int pair = a.ids_dst[begin + (m < count ? m : 0)];
        const int64_t source = a.in_per_pair ? pair : pair / a.top_k;
        x_rows[mt] = a.in_fp8 + source * TERMS * width;
        x_scales[mt] = a.in_fp8_scales + source * TERMS * blocks;
    }
    float16_t acc[2][MT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[t][mt][i] = 0.0f;

    for (int step = 0; step < steps; ++step) {
        int cb = 2 * step + h;
        const bool inside = cb < blocks;
        cb = inside ? cb : blocks - 1;
        i32x8 b[2];
        int sb[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const u32x4 q = *(const MFQ_GLOBAL u32x4*)(codes + static_cast<int64_t>(rows[t]) * (width / 2) + cb * 16);
            // a lane block behind the end of the row (odd block counts) contributes nothing: zero codes
            b[t] = i32x8{inside ? static_cast<int>(q[0]) : 0, inside ? static_cast<int>(q[1]) : 0, inside ? static_cast<int>(q[2]) : 0,
                         inside ? static_cast<int>(q[3]) : 0, 0, 0, 0, 0};
            sb[t] = gload<uint8_t>(scales + static_cast<int64_t>(rows[t]) * blocks + cb);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int term = 0; term < TERMS; ++term) {
                const uint8_t* at = x_rows[mt] + term * width + step * 64 + 16 * h;
                const u32x4 lo = *(const MFQ_GLOBAL u32x4*)at;
                u32x4 hi = {0u, 0u, 0u, 0u};                                    // no second block behind an odd count
                if (2 * step + 1 < blocks) hi = *(const MFQ_GLOBAL u32x4*)(at + 32);
                const i32x8 av = {static_cast<int>(lo[0]), static_cast<int>(lo[1]), static_cast<int>(lo[2]), static_cast<int>(lo[3]),
                                  static_cast<int>(hi[0]), static_cast<int>(hi[1]), static_cast<int>(hi[2]), static_cast<int>(hi[3])};
                const int sa = gload<uint8_t>(x_scales[mt] + term * blocks + cb);
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    acc[t][mt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, b[t], acc[t][mt], 0 /* A: E4M3 */, 4 /* B: E2M1 */,
                                                                                   0, sa, 0, sb[t]);
            }
        }
    }
    // D[m][n]: the lane holds row n of the weights and pairs m = 8 * (i / 4) + 4 * h + i % 4 of each 32
    uint16_t* out = a.out + (slot - a.slot_base) * a.out_slot_stride;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int row = n0 + 32 * t + n;
        if (row >= a.out_rows) continue;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int m = 32 * mt + 8 * (i / 4) + 4 * h + (i % 4);
                if (m < count) out[static_cast<int64_t>(a.ids_dst[begin + m]) * a.out_pair_stride + row] = float_to_half_bits(acc[t][mt][i]);
            }
    }
}

template <int TERMS>
__global__ void __launch_bounds__(256) moe_tiles_mx_scaled_kernel(RowsArgs a) {
    // same block -> (tile, row block, slot) order as the streaming tile kernel
    const int row_blocks = (a.out_rows + kFastTileN - 1) / kFastTileN;
    const int sharers = row_blocks * a.tile_slots;
    const int id = blockIdx.x;
    const int index = id / (8 * sharers) * 8 + id % 8;
    const int sub = id % (8 * sharers) / 8;
    const int row_block = sub / a.tile_slots;
    const int slot = a.slot_base + sub % a.tile_slots;
    const int* offsets = a.tile_offsets + slot * kClassSlots;
    // tile_items is sorted by class: only the MXFP4 range concerns this kernel
    if (index < offsets[K_MXFP4] || index >= offsets[K_MXFP4 + 1] || index >= a.tile_capacity) return;
    const int packed = a.tile_items[slot * a.tile_capacity + index];
    const int expert = packed & 0xffff, m_tile = packed >> 16;
    const ExpertInfo info = a.expert_info[slot * a.experts + expert];
    if (info.pool < 0 || info.cls != K_MXFP4) return;
    const int begin = a.expert_bounds[expert] + m_tile * kPrefillTileM;
    const int left = a.expert_bounds[expert + 1] - begin;
    const int count = left < kPrefillTileM ? left : kPrefillTileM;
    if (count <= 0) return;
    const mfq_amd_projection& pool = a.pools[info.pool];
    if (count <= 32) tiles_mx_scaled_block<1, TERMS>(a, slot, row_block, pool, info.local, begin, count);
    else if (count <= 64) tiles_mx_scaled_block<2, TERMS>(a, slot, row_block, pool, info.local, begin, count);
    else if (count <= 96) tiles_mx_scaled_block<3, TERMS>(a, slot, row_block, pool, info.local, begin, count);
    else tiles_mx_scaled_block<4, TERMS>(a, slot, row_block, pool, info.local, begin, count);
}

// One thread per (row, block of 32 columns): the E4M3 terms and their scales.
__global__ void __launch_bounds__(256) fp8_split_kernel(const uint16_t* src, int half_in, int64_t items, int width, int terms,
                                                        uint8_t* dst, uint8_t* scales) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (item >= items) return;
    const int blocks = width / kLaneColumns;
    const int64_t row = item / blocks;
    const int cb = static_cast<int>(item % blocks);
    float x[32];
    const uint16_t* from = src + row * width + cb * kLaneColumns;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const u32x4 raw = *(const MFQ_GLOBAL u32x4*)(from + 8 * j);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint16_t lo = static_cast<uint16_t>(raw[k] & 0xffffu), hi = static_cast<uint16_t>(raw[k] >> 16);
            x[8 * j + 2 * k] = half_in ? half_bits_to_float(lo) : bf16_bits_to_float(lo);
            x[8 * j + 2 * k + 1] = half_in ? half_bits_to_float(hi) : bf16_bits_to_float(hi);
        }
    }
    for (int term = 0; term < terms; ++term) {
        float largest = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) largest = fmaxf(largest, fabsf(x[i]));
        const uint8_t s = block_scale_byte(largest);
        const float down = scale_inverse(s), up = scale_value(s);
        uint32_t words[8];
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            uint32_t word = 0u;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint8_t byte = e4m3_from_float(x[4 * w + k] * down);
                x[4 * w + k] = x[4 * w + k] - e4m3_to_float(byte) * up;        // the residual: the next term's source
                word |= static_cast<uint32_t>(byte) << (8 * k);
            }
            words[w] = word;
        }
        uint8_t* to = dst + (row * terms + term) * width + cb * kLaneColumns;
        *reinterpret_cast<u32x4*>(to) = u32x4{words[0], words[1], words[2], words[3]};
        *reinterpret_cast<u32x4*>(to + 16) = u32x4{words[4], words[5], words[6], words[7]};
        scales[(row * terms + term) * blocks + cb] = s;
    }
}


// ------------------------------------------------ activations for the tiles ----
// hidden[pair] = swiglu(gate[pair], up[pair]) as fp16, every 32 columns in the pair order that the
// pair's down projection reads: the layout of its pool's class when the streaming tile kernel serves
// the pool, plain column order otherwise (which is also layout 2).  One thread per lane block.
__device__ __forceinline__ void swiglu_tiles_item(int64_t item, const uint16_t* gate, const uint16_t* up, int64_t gate_stride,
                                                  int inner, float limit, const uint16_t* table, const int32_t* ids,
                                                  const ExpertInfo* down_info, int experts, uint16_t* hidden) {
    const int blocks = inner / kLaneColumns;
    const int64_t pair = item / blocks;
    const int cb = static_cast<int>(item % blocks);
    const uint16_t* g = gate + pair * gate_stride + cb * kLaneColumns;
    const uint16_t* u = up + pair * gate_stride + cb * kLaneColumns;
    u32x4 graw[4], uraw[4], out[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        graw[j] = *(const MFQ_GLOBAL u32x4*)(g + 8 * j);
        uraw[j] = *(const MFQ_GLOBAL u32x4*)(u + 8 * j);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t lo = swiglu_bits(static_cast<uint16_t>(graw[j][k] & 0xffffu), static_cast<uint16_t>(uraw[j][k] & 0xffffu), limit, table);
            const uint32_t hi = swiglu_bits(static_cast<uint16_t>(graw[j][k] >> 16), static_cast<uint16_t>(uraw[j][k] >> 16), limit, table);
            out[j][k] = lo | (hi << 16);
        }
    int layout = 2;
    const int expert = ids[pair];
    if (static_cast<unsigned>(expert) < static_cast<unsigned>(experts)) {
        const int cls = down_info[expert].cls;
        if (!(cls & kPoolExactOnly)) {
            switch (cls) {
                case K_NINT_3_24: case K_NINT_4_24: case K_NINT_4_32: layout = 0; break;
                case K_NINT_8_48: layout = 1; break;
                case K_NINT_2_16: layout = 3; break;
                default: layout = 2; break;
            }
        }
    }
    uint16_t* to = hidden + item * kLaneColumns;
    if (layout == 0) store_layout<0>(out, true, to);
    else if (layout == 1) store_layout<1>(out, true, to);
    else if (layout == 3) store_layout<3>(out, true, to);
    else store_layout<2>(out, true, to);
}

__global__ void __launch_bounds__(256) swiglu_tiles_kernel(const uint16_t* gate, const uint16_t* up, int64_t gate_stride, int inner,
                                                           int pairs, float limit, const uint16_t* table, const int32_t* ids,
                                                           const ExpertInfo* down_info, int experts, uint16_t* hidden) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (item >= static_cast<int64_t>(pairs) * (inner / kLaneColumns)) return;
    swiglu_tiles_item(item, gate, up, gate_stride, inner, limit, table, ids, down_info, experts, hidden);
}

// The same for large batches: a resident grid (one block of 1024 threads per CU) that first copies the sigmoid
// table (65536 halves) into LDS.  Out of global memory the 32 lookups of a thread are 32 gathers of scattered
// 2-byte addresses, and the address unit, not the memory, sets the pace of the kernel.
constexpr int kSigmoidTableBytes = 65536 * 2;
__global__ void __launch_bounds__(1024) swiglu_tiles_lds_kernel(const uint16_t* gate, const uint16_t* up, int64_t gate_stride,
                                                                int inner, int pairs, const uint16_t* table, const int32_t* ids,
                                                                const ExpertInfo* down_info, int experts, uint16_t* hidden) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    for (int i = threadIdx.x; i < kSigmoidTableBytes / 16; i += blockDim.x)
        reinterpret_cast<u32x4*>(lds)[i] = *((const MFQ_GLOBAL u32x4*)table + i);
    __syncthreads();
    const int64_t items = static_cast<int64_t>(pairs) * (inner / kLaneColumns);
    for (int64_t item = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; item < items;
         item += static_cast<int64_t>(gridDim.x) * blockDim.x)
        swiglu_tiles_item(item, gate, up, gate_stride, inner, 0.0f, reinterpret_cast<const uint16_t*>(lds), ids, down_info,
                          experts, hidden);
}

struct TilesLaunch {
    RowsArgs a; int slots; int tiles; hipStream_t stream;
    template <int CLS> void run() const {
        const dim3 grid((a.out_rows + kPrefillTileN - 1) / kPrefillTileN * (kPrefillTileM / kExactTileM), tiles, slots);
        const int table_bytes = (CLS == K_NVQ_D4 || CLS == K_NVQ_E8) ? 4 * 1024 * 8 + 128 : class_lds_bytes(CLS, 0);
        const int bytes = 2 * (kExactTileM + kPrefillTileN) * kLdsStride + table_bytes;
        hipLaunchKernelGGL(moe_tiles_kernel<CLS>, grid, dim3(256), bytes, stream, a);
    }
};

}  // namespace dev

void raise_prefill_limits() {
    MFQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dev::moe_tiles_fast_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, dev::kTilesFastLdsBytes));
    MFQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dev::moe_tiles_fast_kernel<false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, dev::kTilesFastLdsBytes));
    MFQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dev::swiglu_tiles_lds_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, dev::kSigmoidTableBytes));
}

bool tiles_packed_geometry(int in_width, int64_t in_rows) {
    return in_width % (4 * dev::kLaneColumns) == 0 && in_rows * in_width * 2 < (int64_t(1) << 32);
}

bool tiles_fast_geometry(int in_width, int in_dtype, int in_vector_ok) {
    return in_width % dev::kLaneColumns == 0 && in_width >= 2 * dev::kLaneColumns && in_dtype != MFQ_AMD_F32 && in_vector_ok != 0;
}

void launch_tiles_fast(const RowsArgs& args, int slots, int max_tiles, bool nvq, hipStream_t stream) {
    if (max_tiles <= 0) return;
    MFQ_REQUIRE(tiles_fast_geometry(args.in_width, args.in_dtype, args.in_vector_ok), "geometry is not served by the streaming tile kernel");
    RowsArgs a = args;
    a.tile_slots = slots;
    const int row_blocks = (args.out_rows + dev::kFastTileN - 1) / dev::kFastTileN;
    const dim3 grid((max_tiles + 7) / 8 * 8 * row_blocks * slots);
    (void)nvq;   // the table region also holds the NINT level windows
    const int bytes = dev::kTilesFastLdsBytes;   // more than the default 64 KB of dynamic LDS: raised by device_state()
    (void)device_state();
    MFQ_REQUIRE(a.in_tiles == nullptr || tiles_packed_geometry(a.in_width, a.in_per_pair ? a.pairs : (a.pairs + a.top_k - 1) / a.top_k),
                "packed activation tiles need rows of whole steps and a copy below 4 GB");
    if (a.in_tiles != nullptr) hipLaunchKernelGGL(dev::moe_tiles_fast_kernel<true>, grid, dim3(256), bytes, stream, a);
    else hipLaunchKernelGGL(dev::moe_tiles_fast_kernel<false>, grid, dim3(256), bytes, stream, a);
    check_launch("moe_tiles_fast_kernel");
}

void launch_tiles_mx_scaled(const RowsArgs& args, int slots, int max_tiles, hipStream_t stream) {
    if (max_tiles <= 0) return;
    MFQ_REQUIRE(args.in_fp8 != nullptr && args.in_fp8_scales != nullptr && args.expert_info != nullptr &&
                    (args.in_fp8_terms == 2 || args.in_fp8_terms == 3) && args.in_width % dev::kLaneColumns == 0,
                "the block-scaled MFMA kernel needs the activations as two or three E4M3 terms");
    RowsArgs a = args;
    a.tile_slots = slots;
    const int row_blocks = (args.out_rows + dev::kFastTileN - 1) / dev::kFastTileN;
    const dim3 grid((max_tiles + 7) / 8 * 8 * row_blocks * slots);
    if (a.in_fp8_terms == 2) hipLaunchKernelGGL(dev::moe_tiles_mx_scaled_kernel<2>, grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(dev::moe_tiles_mx_scaled_kernel<3>, grid, dim3(256), 0, stream, a);
    check_launch("moe_tiles_mx_scaled_kernel");
}

void launch_fp8_split(const void* src, int dtype, int rows, int width, int terms, uint8_t* dst, uint8_t* scales, hipStream_t stream) {
    if (rows <= 0) return;
    MFQ_REQUIRE(width % dev::kLaneColumns == 0 && dtype != MFQ_AMD_F32 && reinterpret_cast<uintptr_t>(src) % 16 == 0 &&
                    (terms == 2 || terms == 3), "geometry is not served by the E4M3 split");
    const int64_t items = static_cast<int64_t>(rows) * (width / dev::kLaneColumns);
    hipLaunchKernelGGL(dev::fp8_split_kernel, dim3(static_cast<unsigned>((items + 255) / 256)), dim3(256), 0, stream,
                       static_cast<const uint16_t*>(src), dtype == MFQ_AMD_F16 ? 1 : 0, items, width, terms, dst, scales);
    check_launch("fp8_split_kernel");
}

void launch_swiglu_tiles(const uint16_t* gate, const uint16_t* up, int64_t gate_stride, int inner, int pairs, float limit,
                         const uint16_t* table, const int32_t* ids, const ExpertInfo* down_info, int experts, uint16_t* hidden,
                         hipStream_t stream) {
    if (pairs <= 0) return;
    MFQ_REQUIRE(inner % dev::kLaneColumns == 0 && gate_stride % 8 == 0, "geometry is not served by the tile SwiGLU kernel");
    const int64_t items = static_cast<int64_t>(pairs) * (inner / dev::kLaneColumns);
    constexpr int kResidentBlocks = 256;    // one per CU: the table takes 128 KB of a CU's 160 KB of LDS
    if (limit <= 0.0f && items >= static_cast<int64_t>(kResidentBlocks) * 1024 * 2 && reinterpret_cast<uintptr_t>(table) % 16 == 0) {
        (void)device_state();   // the kernel's dynamic-LDS limit is raised there
        hipLaunchKernelGGL(dev::swiglu_tiles_lds_kernel, dim3(kResidentBlocks), dim3(1024), dev::kSigmoidTableBytes, stream, gate, up,
                           gate_stride, inner, pairs, table, ids, down_info, experts, hidden);
        check_launch("swiglu_tiles_lds_kernel");
        return;
    }
    hipLaunchKernelGGL(dev::swiglu_tiles_kernel, dim3(static_cast<unsigned>((items + 255) / 256)), dim3(256), 0, stream, gate, up,
                       gate_stride, inner, pairs, limit, table, ids, down_info, experts, hidden);
    check_launch("swiglu_tiles_kernel");
}

int tile_layout_of_class(int cls) {
    switch (cls) {
        case dev::K_NINT_3_24: case dev::K_NINT_4_24: case dev::K_NINT_4_32: return 0;
        case dev::K_NINT_8_48: return 1;
        case dev::K_NINT_2_16: return 3;
        default: return 2;
    }
}

void launch_rows_prefill(const RowsArgs& args, int slots, const int* present, const int* max_tiles, hipStream_t stream) {
    for (int c = 0; c < dev::K_CLASS_COUNT; ++c) {
        if (!present[c] || max_tiles[c] <= 0) continue;
        dev::TilesLaunch launch{args, slots, max_tiles[c], stream};
        dev::dispatch_class(c, launch);
        check_launch("moe_tiles_kernel");
    }
}

}  // namespace mfq_amd
