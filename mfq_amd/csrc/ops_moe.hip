// Mixed-format MoE: the streaming rows kernel that serves decode (fused dequantise-and-multiply
// GEMV over every active expert of one kernel class), SwiGLU, the route-weighted reduce, the
// grouped projection entry point and the fused FFN object.
#include "common.h"
#include "decode.cuh"
#include "device_state.h"
#include "fast_rows.cuh"
#include "launch.cuh"
#include "moe_args.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

namespace mfq_amd {
namespace dev {

constexpr int kPassTokens = 4;   // tokens an exact pass multiplies with one decode of the weights

// Where the activations of routed pair `pair` start.
__device__ __forceinline__ const void* pair_source(const RowsArgs& a, int pair) {
    const int element = a.in_dtype == MFQ_AMD_F32 ? 4 : 2;
    const int64_t source = a.in_per_pair ? pair : pair / a.top_k;
    return static_cast<const char*>(a.in) + source * a.in_width * element;
}

// ---------------------------------------------------------------- exact ----
// One block = one active expert x 64 output rows x every pair routed to it, on the exact decoders:
// a wave takes one row at a time, lanes stride over its chunks, and every decoded chunk multiplies
// up to four tokens.  Serves whatever the streaming kernel below does not.
template <int CLS>
__global__ void __launch_bounds__(256) moe_rows_exact_kernel(RowsArgs a) {
    extern __shared__ unsigned char lds[];
    const int slot = a.slot_base + blockIdx.z;
    const int* offsets = a.class_offsets + slot * kClassSlots;
    const int index = offsets[CLS] + blockIdx.y;
    if (index >= offsets[CLS + 1]) return;
    const PlanItem item = a.item_info[slot * a.experts + index];
    if (a.exact_only && !(item.cls & kPoolExactOnly)) return;
    const mfq_amd_projection& pool = a.pools[item.pool];
    Decoder<CLS> dec;
    dec.init(pool, lds);
    __syncthreads();
    const int wave = uniform(static_cast<int>(threadIdx.x / kWave)), lane = threadIdx.x % kWave;
    const int chunks = (a.in_width + 7) / 8;
    for (int first = item.begin; first < item.begin + item.count; first += kPassTokens) {
        const int here = item.begin + item.count - first < kPassTokens ? item.begin + item.count - first : kPassTokens;
        int pair[kPassTokens];
        const void* source[kPassTokens];
#pragma unroll
        for (int t = 0; t < kPassTokens; ++t) {
            pair[t] = a.ids_dst[first + (t < here ? t : 0)];
            source[t] = pair_source(a, pair[t]);
        }
        for (int r = wave; r < kRowsBlockRows; r += 4) {
            const int row = blockIdx.x * kRowsBlockRows + r;
            if (row >= a.out_rows) break;
            typename Decoder<CLS>::Row rr;
            dec.row(pool, item.local, row, rr);
            float acc[kPassTokens] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int c = lane; c < chunks; c += kWave) {
                float w[8];
                dec.chunk(rr, c, w);
#pragma unroll
                for (int t = 0; t < kPassTokens; ++t) {
                    if (t >= here) continue;
                    float x[8];
                    load_x8(source[t], a.in_dtype, c, a.in_width, a.in_vector_ok != 0, x);
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[t] = fmaf(c * 8 + i < a.in_width ? w[i] : 0.0f, x[i], acc[t]);
                }
            }
#pragma unroll
            for (int t = 0; t < kPassTokens; ++t) {
                const float total = wave_sum(acc[t]);
                if (lane == 0 && t < here)
                    a.out[pair[t] * a.out_pair_stride + (slot - a.slot_base) * a.out_slot_stride + row] =
                        float_to_half_bits(total);
            }
        }
    }
}

// ------------------------------------------------------------ streaming ----
// One block = one routed pair x rows_per_block output rows of its expert; a quarter of the rows per
// wave.  Pairs of one expert sit next to each other in the grid, and the same row tile of
// neighbouring pairs lands on the same XCD, so an expert's weights come from HBM once.
// LDS a block of the down projection keeps for the hidden row of its pair: the fp16 values, the largest magnitude
// (as fp16 bits) and the normaliser {2^-e, 2^e} derived from it.
struct HiddenLds {
    uint16_t values[16 * kLaneColumns];
    uint32_t wave_largest[4];
    float scale[2];
};

// Every lane returns the largest value of the wave.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    auto step = [](uint32_t x, uint32_t other) { return other > x ? other : x; };
    v = step(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, false)));
    v = step(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, false)));
    v = step(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x141, 0xF, 0xF, false)));
    v = step(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x140, 0xF, 0xF, false)));
    // across the rows of 16 lanes and the halves of the wave: register swaps leave the lane's value and its partner's
    // in the two results
    const auto rows = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    v = step(static_cast<uint32_t>(rows[0]), static_cast<uint32_t>(rows[1]));
    const auto halves = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return step(static_cast<uint32_t>(halves[0]), static_cast<uint32_t>(halves[1]));
}

// hidden = swiglu(gate, up) of one routed pair, computed by the block that multiplies it: two columns per thread, the
// row's largest magnitude per wave.  Contains one barrier; every thread of the block calls it once.
__device__ __forceinline__ void hidden_to_lds(const RowsArgs& a, int pair, HiddenLds* hidden) {
    const uint16_t* gate = a.gu + static_cast<int64_t>(pair) * 2 * a.in_width;
    const uint16_t* up = gate + a.in_width;
    uint32_t largest = 0u;
    auto count = [&](uint16_t h) {
        const uint32_t magnitude = h & 0x7fffu;
        largest = magnitude > largest && magnitude <= 0x7c00u ? magnitude : largest;     // NaN does not count, as with fmaxf
    };
    // two columns per thread (rows are multiples of 32 columns and start at multiples of four bytes): a row of 512 columns
    // is one round of loads and one round of table lookups for the block
    for (int col = 2 * threadIdx.x; col < a.in_width; col += 2 * blockDim.x) {
        const uint32_t g = *reinterpret_cast<const uint32_t*>(gate + col), u = *reinterpret_cast<const uint32_t*>(up + col);
        const uint16_t lo = swiglu_bits(static_cast<uint16_t>(g & 0xffffu), static_cast<uint16_t>(u & 0xffffu), a.swiglu_limit, a.sigmoid);
        const uint16_t hi = swiglu_bits(static_cast<uint16_t>(g >> 16), static_cast<uint16_t>(u >> 16), a.swiglu_limit, a.sigmoid);
        *reinterpret_cast<uint32_t*>(&hidden->values[col]) = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
        count(lo); count(hi);
    }
    largest = wave_max_u32(largest);       // the bits of non-negative halves order like their values
    if (threadIdx.x % kWave == 0) hidden->wave_largest[threadIdx.x / kWave] = largest;
    __syncthreads();
}

// One block = one routed pair x rows_per_block output rows of its expert; a quarter of the rows per
// wave.  Pairs of one expert sit next to each other in the grid, and the same row tile of
// neighbouring pairs lands on the same XCD, so an expert's weights come from HBM once.
// NT > 1: the block multiplies the rows with the activations of up to NT pairs that the plan grouped because they are
// routed to the same expert (PairItem::cls carries their number above bit 16): the packed rows are fetched and decoded
// once for the group.  `pairs[n]` for n >= count repeat the first pair and store nothing.
template <int CLS, int LPR, int XMODE, int SLOTS, int IB, int NT>
__device__ __forceinline__ void rows_fast_pair(const RowsArgs& a, const mfq_amd_projection& pool, const PairItem& item, int slot,
                                               unsigned char* lds, HiddenLds* hidden, const int (&pairs)[NT], int count) {
    const FastCtx<CLS> ctx = fast_ctx<CLS>(pool, item.local, lds);
    const int wave = uniform(static_cast<int>(threadIdx.x / kWave));
    const int rows_per_wave = a.rows_per_block / 4;
    const int row_begin = blockIdx.x * a.rows_per_block + wave * rows_per_wave;
    // the hidden rows of the pairs: computed while the first packed rows are on their way
    auto prologue = [&] {
        if constexpr (XMODE == kXScaled) {
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                if (n > 0 && n >= count) break;           // uniform over the block: every thread takes the same turns
                hidden_to_lds(a, pairs[n], &hidden[n]);
            }
            if (threadIdx.x < NT && static_cast<int>(threadIdx.x) < (count > 1 ? count : 1)) {
                HiddenLds* h = &hidden[threadIdx.x];
                float down, up;
                uint32_t largest = h->wave_largest[0];
                for (int w = 1; w < 4; ++w) largest = h->wave_largest[w] > largest ? h->wave_largest[w] : largest;
                normaliser(half_bits_to_float(static_cast<uint16_t>(largest)), down, up);
                h->scale[0] = down; h->scale[1] = up;
            }
            __syncthreads();
        }
    };
    if (row_begin >= a.out_rows) { prologue(); return; }
    const int row_end = row_begin + rows_per_wave < a.out_rows ? row_begin + rows_per_wave : a.out_rows;
    uint16_t* outs[NT];
    XSource xs[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        const int pair = pairs[n];
        const int staged = n < count ? n : 0;
        outs[n] = a.out + (slot - a.slot_base) * a.out_slot_stride + pair * a.out_pair_stride;
        const int64_t source = a.in_per_pair ? pair : pair / a.top_k;
        xs[n] = XSource{XMODE == kXPacked ? static_cast<const void*>(a.in_packed + source * a.in_packed_stride)
                        : XMODE == kXScaled ? static_cast<const void*>(hidden[staged].values) : pair_source(a, pair),
                        XMODE == kXScaled ? MFQ_AMD_F16 : a.in_dtype, XMODE == kXScaled ? true : a.in_vector_ok != 0,
                        hidden[staged].scale};
    }
    constexpr int kRing = FastClass<CLS>::kRing < SLOTS || SLOTS == 0 ? FastClass<CLS>::kRing : SLOTS;
    auto store = [&](int n, int row, float value) { if (NT == 1 || n < count) outs[n][row] = float_to_half_bits(value); };
    if constexpr (FastClass<CLS>::kNint && SLOTS > 0) {
        // straight-line variants: the levels of a row slot as shared level words where the row's geometry allows
        if (nint_level_words_cover(ctx.groups, nint_level_word_stride(FastClass<CLS>::kGs), 32 / (kWave / LPR))) {
            fast_rows<CLS, LPR, 1, NT, kRing, XMODE, SLOTS, IB, true>(ctx, xs, a.in_width, row_begin, row_end, a.out_rows, store, prologue);
            return;
        }
    }
    fast_rows<CLS, LPR, 1, NT, kRing, XMODE, SLOTS, IB>(ctx, xs, a.in_width, row_begin, row_end, a.out_rows, store, prologue);
}

template <int CLS, int LPR, int XMODE, int SLOTS, int NT>
__device__ __forceinline__ void rows_fast_block(const RowsArgs& a, const PairItem& item, int slot, unsigned char* lds, HiddenLds* hidden,
                                                const int (&pairs)[NT], int count) {
    const mfq_amd_projection& pool = a.pools[item.pool];
    if constexpr (FastClass<CLS>::kNvq) {
        nvq_fast_tables(pool, lds);
        __syncthreads();
        // the index width of the format fixes the bit positions of every index: one copy of the row loop each
        const int index_bits = nvq_format_index_bits(pool.format);
        if (index_bits == 10) rows_fast_pair<CLS, LPR, XMODE, SLOTS, 10, NT>(a, pool, item, slot, lds, hidden, pairs, count);
        else if (index_bits == 9) rows_fast_pair<CLS, LPR, XMODE, SLOTS, 9, NT>(a, pool, item, slot, lds, hidden, pairs, count);
        else rows_fast_pair<CLS, LPR, XMODE, SLOTS, 8, NT>(a, pool, item, slot, lds, hidden, pairs, count);
    } else {
        rows_fast_pair<CLS, LPR, XMODE, SLOTS, 0, NT>(a, pool, item, slot, lds, hidden, pairs, count);
    }
}

// One launch for every format: blockIdx.y walks the routed pairs and each block branches once
// (uniformly) into the kernel class of its expert's pool.
// SLOTS: row slots per wave (a slot is one row for LPR 64 and four rows for LPR 16), so a block
// covers 4 * SLOTS * (64 / LPR) rows; 0 = taken from rows_per_block at run time.
// XMODE: kXRaw / kXPacked: activations from RowsArgs::in / in_packed; kXScaled: the block computes the hidden row of
// its pair from RowsArgs::gu first (down projection of the FFN; rows of at most 512 columns).
// NT: 1: a block per pair.  kGroupPairs: the plan has grouped up to that many neighbouring pairs of one expert; the
// block of a group's first pair multiplies for all of them and the blocks of the others return at once.
template <int LPR, int XMODE, int SLOTS, int NT>
__global__ void __launch_bounds__(256) moe_rows_fast_kernel(RowsArgs a) {
    // The NVQ tables sit in statically sized LDS: their addresses are then constants of the instruction
    // stream.  Four blocks of a CU hold 4 x 35 KB of the 160 KB, which the register budget allows anyway.
    __shared__ __attribute__((aligned(16))) unsigned char lds[kNvqFastLdsBytes];
    __shared__ __attribute__((aligned(16))) HiddenLds hidden[NT];
    const int slot = a.slot_base + blockIdx.z;
    const PairItem* list = a.pair_items + static_cast<int64_t>(slot) * a.pairs;
    PairItem item = list[blockIdx.y];
    int pairs[NT];
    int count = 1;
    pairs[0] = item.pair;
    if constexpr (NT > 1) {
        if (item.cls < 0) return;
        count = item.cls >> kGroupCountShift;
        item.cls &= (1 << kGroupCountShift) - 1;
        if (count == 0) return;                           // a pair that the block of its group's first pair serves
#pragma unroll
        for (int n = 1; n < NT; ++n) pairs[n] = n < count ? list[blockIdx.y + n].pair : item.pair;
    }
    switch (item.cls) {
        case K_NINT_2_16: rows_fast_block<K_NINT_2_16, LPR, XMODE, SLOTS, NT>(a, item, slot, lds, hidden, pairs, count); break;
        case K_NINT_3_24: rows_fast_block<K_NINT_3_24, LPR, XMODE, SLOTS, NT>(a, item, slot, lds, hidden, pairs, count); break;
        case K_NINT_4_24: rows_fast_block<K_NINT_4_24, LPR, XMODE, SLOTS, NT>(a, item, slot, lds, hidden, pairs, count); break;
        case K_NINT_4_32: rows_fast_block<K_NINT_4_32, LPR, XMODE, SLOTS, NT>(a, item, slot, lds, hidden, pairs, count); break;
        case K_NINT_8_48: rows_fast_block<K_NINT_8_48, LPR, XMODE, SLOTS, NT>(a, item, slot, lds, hidden, pairs, count); break;
        case K_NVQ_D4: rows_fast_block<K_NVQ_D4, LPR, XMODE, SLOTS, NT>(a, item, slot, lds, hidden, pairs, count); break;
        case K_MXFP4: rows_fast_block<K_MXFP4, LPR, XMODE, SLOTS, NT>(a, item, slot, lds, hidden, pairs, count); break;
        default: break;   // unrouted, exact-only pools and classes without a fast path
    }
}

struct RowsExactLaunch {
    RowsArgs a; int slots; int items; hipStream_t stream;
    template <int CLS> void run() const {
        const dim3 grid((a.out_rows + kRowsBlockRows - 1) / kRowsBlockRows, items, slots);
        const int bytes = (CLS == K_NVQ_D4 || CLS == K_NVQ_E8) ? 4 * 1024 * 8 + 128 : class_lds_bytes(CLS, 0);
        hipLaunchKernelGGL(moe_rows_exact_kernel<CLS>, grid, dim3(256), bytes, stream, a);
    }
};

// hidden = swiglu(gate, up) elementwise on fp16; `table` maps the bits of a half g to half(sigmoid(g))
// computed in double (mfq/kernels/cuda/moe.cu:1536-1542 builds the same table for the fused path).
__global__ void swiglu_kernel(const uint16_t* gate, const uint16_t* up, int64_t count, int64_t gate_stride,
                              int64_t inner, float limit, const uint16_t* table, uint16_t* hidden) {
    const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= count) return;
    const int64_t row = index / inner, col = index % inner;
    const uint16_t gb = gate[row * gate_stride + col], ub = up[row * gate_stride + col];
    hidden[index] = swiglu_bits(gb, ub, limit, table);
}

// One block per routed pair: the same hidden values, written as fp16 and in the packed form the
// streaming kernels read.  Dynamic LDS: inner halves, then one float per wave.
__global__ void __launch_bounds__(256) swiglu_pack_kernel(const uint16_t* gate, const uint16_t* up, int64_t gate_stride,
                                                          int inner, float limit, const uint16_t* table,
                                                          uint16_t* hidden, uint32_t* packed, int64_t packed_stride) {
    extern __shared__ unsigned char lds[];
    uint16_t* staged = reinterpret_cast<uint16_t*>(lds);
    float* scratch = reinterpret_cast<float*>(lds + ((static_cast<size_t>(inner) * 2 + 15) / 16) * 16);
    const int64_t row = blockIdx.x;
    const bool pairs_ok = inner % 2 == 0 && gate_stride % 2 == 0 && (reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) |
                                                                     reinterpret_cast<uintptr_t>(hidden)) % 4 == 0;
    if (pairs_ok) {
        // two columns per thread: a row of 512 columns is one round of loads and one round of table lookups for the block
        // (one column per thread made it two of each, one after the other)
        for (int col = 2 * threadIdx.x; col < inner; col += 2 * blockDim.x) {
            const uint32_t g = *reinterpret_cast<const uint32_t*>(gate + row * gate_stride + col);
            const uint32_t u = *reinterpret_cast<const uint32_t*>(up + row * gate_stride + col);
            const uint32_t lo = swiglu_bits(static_cast<uint16_t>(g & 0xffffu), static_cast<uint16_t>(u & 0xffffu), limit, table);
            const uint32_t hi = swiglu_bits(static_cast<uint16_t>(g >> 16), static_cast<uint16_t>(u >> 16), limit, table);
            *reinterpret_cast<uint32_t*>(hidden + row * inner + col) = lo | (hi << 16);
            *reinterpret_cast<uint32_t*>(staged + col) = lo | (hi << 16);
        }
    } else {
        for (int col = threadIdx.x; col < inner; col += blockDim.x) {
            const uint16_t gb = gate[row * gate_stride + col], ub = up[row * gate_stride + col];
            const uint16_t result = swiglu_bits(gb, ub, limit, table);
            hidden[row * inner + col] = result;
            staged[col] = result;
        }
    }
    __syncthreads();
    xpack_row(staged, MFQ_AMD_F16, true, inner, packed + row * packed_stride, scratch);
}

// out[t, c] = sum_r w[t, r] * pair[t, r, c], fp32, routes ascending (mfq/kernels/cuda/moe.cu:1495-1515).
// Routes whose expert id is outside [0, experts) contribute nothing.
// K > 0: top_k known at compile time; the ids, weights and pair values of a thread are all requested before the
// first add (a loop that tests the id first makes ten dependent round trips of what is one), the adds keep their order.
template <int K>
__global__ void weighted_reduce_kernel(const uint16_t* pairs, const float* weights, const int32_t* ids, int experts,
                                       int tokens, int top_k, int width, void* out, int out_dtype) {
    const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= static_cast<int64_t>(tokens) * width) return;
    const int64_t t = index / width, c = index % width;
    float sum = 0.0f;
    if constexpr (K > 0) {
        int32_t id[K];
        float w[K];
        uint16_t v[K];
#pragma unroll
        for (int r = 0; r < K; ++r) {
            id[r] = ids != nullptr ? ids[t * K + r] : 0;
            w[r] = weights[t * K + r];
            v[r] = pairs[(t * K + r) * width + c];
        }
#pragma unroll
        for (int r = 0; r < K; ++r) {
            const float term = w[r] * half_bits_to_float(v[r]);
            if (static_cast<unsigned>(id[r]) < static_cast<unsigned>(ids != nullptr ? experts : 1)) sum = sum + term;
        }
    } else {
        for (int r = 0; r < top_k; ++r) {
            if (ids != nullptr && static_cast<unsigned>(ids[t * top_k + r]) >= static_cast<unsigned>(experts)) continue;
            const float term = weights[t * top_k + r] * half_bits_to_float(pairs[(t * top_k + r) * width + c]);
            sum = sum + term;
        }
    }
    if (out_dtype == MFQ_AMD_F32) static_cast<float*>(out)[index] = sum;
    else static_cast<uint16_t*>(out)[index] = float_to_half_bits(sum);
}

// The same sums, eight columns per thread (width a multiple of 8): 16-byte loads, the same order of operations.
__global__ void __launch_bounds__(256) weighted_reduce8_kernel(const uint16_t* pairs, const float* weights, const int32_t* ids,
                                                               int experts, int tokens, int top_k, int width, void* out,
                                                               int out_dtype) {
    const int per_row = width / 8;
    const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= static_cast<int64_t>(tokens) * per_row) return;
    const int64_t t = index / per_row, c = (index % per_row) * 8;
    float sum[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int r = 0; r < top_k; ++r) {
        if (ids != nullptr && static_cast<unsigned>(ids[t * top_k + r]) >= static_cast<unsigned>(experts)) continue;
        const float w = weights[t * top_k + r];
        const u32x4 v = *(const MFQ_GLOBAL u32x4*)(pairs + (t * top_k + r) * width + c);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float term = w * half_bits_to_float(static_cast<uint16_t>(v[i / 2] >> (16 * (i % 2))));
            sum[i] = sum[i] + term;
        }
    }
    if (out_dtype == MFQ_AMD_F32) {
        float4* to = reinterpret_cast<float4*>(static_cast<float*>(out) + t * width + c);
        to[0] = float4{sum[0], sum[1], sum[2], sum[3]};
        to[1] = float4{sum[4], sum[5], sum[6], sum[7]};
    } else {
        u32x4 packed;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            packed[i] = static_cast<uint32_t>(float_to_half_bits(sum[2 * i])) | (static_cast<uint32_t>(float_to_half_bits(sum[2 * i + 1])) << 16);
        *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(out) + t * width + c) = packed;
    }
}

// Shared-expert epilogue.  out = half(routed + sigmoid(gate_logits[row]) * shared) with routed either given
// (pairs == nullptr) or half(sum_r w * pair), routes ascending
// (moe_add_shared_gate_kernel and moe_weighted_reduce_shared_gate_kernel, mfq/kernels/cuda/moe.cu:1557-1596).
__global__ void shared_gate_kernel(const uint16_t* routed, const uint16_t* pairs, const float* weights, const uint16_t* shared,
                                   const float* gate_logits, int tokens, int top_k, int width, uint16_t* out) {
    const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= static_cast<int64_t>(tokens) * width) return;
    const int64_t t = index / width, c = index % width;
    float value;
    if (pairs != nullptr) {
        float sum = 0.0f;
        for (int r = 0; r < top_k; ++r) {
            const float term = weights[t * top_k + r] * half_bits_to_float(pairs[(t * top_k + r) * width + c]);
            sum = sum + term;
        }
        value = half_bits_to_float(float_to_half_bits(sum));
    } else {
        value = half_bits_to_float(routed[index]);
    }
    const float gate = 1.0f / (1.0f + routing_expf(-gate_logits[t]));
    const float term = gate * half_bits_to_float(shared[index]);
    out[index] = float_to_half_bits(value + term);
}

// Epilogue of a layer with a shared expert (the last lines of mfe_ffn_down_reduce_kernel,
// mfq/kernels/cuda/mfe_ffn_device.cuh:1249-1263): routed = half(sum_r w * pair), routes ascending; contribution =
// shared * gate in fp32 (rounded to fp16 when the gate values are fp16: shared_product_half); out = routed + contribution.
// The gate values arrive evaluated (MfeFfnBatch::shared_gate), as float32, float16 or bfloat16.
__global__ void shared_expert_reduce_kernel(const uint16_t* pairs, const float* weights, const int32_t* ids, int experts,
                                            const uint16_t* shared, const void* gate, int gate_dtype, int tokens, int top_k, int width,
                                            void* out, int out_dtype) {
    const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= static_cast<int64_t>(tokens) * width) return;
    const int64_t t = index / width, c = index % width;
    float sum = 0.0f;
    for (int r = 0; r < top_k; ++r) {
        if (ids != nullptr && static_cast<unsigned>(ids[t * top_k + r]) >= static_cast<unsigned>(experts)) continue;
        const float term = weights[t * top_k + r] * half_bits_to_float(pairs[(t * top_k + r) * width + c]);
        sum = sum + term;
    }
    const float routed = half_bits_to_float(float_to_half_bits(sum));
    const float g = gate_dtype == MFQ_AMD_F32 ? static_cast<const float*>(gate)[t]
                  : gate_dtype == MFQ_AMD_F16 ? half_bits_to_float(static_cast<const uint16_t*>(gate)[t])
                                              : bf16_bits_to_float(static_cast<const uint16_t*>(gate)[t]);
    float contribution = half_bits_to_float(shared[index]) * g;
    if (gate_dtype == MFQ_AMD_F16) contribution = half_bits_to_float(float_to_half_bits(contribution));
    const float value = routed + contribution;
    if (out_dtype == MFQ_AMD_F32) static_cast<float*>(out)[index] = value;
    else static_cast<uint16_t*>(out)[index] = float_to_half_bits(value);
}

}  // namespace dev

namespace {
// The down blocks compute the hidden row of their pair themselves up to this many routed pairs, or, beyond that, up to
// this many down blocks per pair (every block of a pair repeats the SwiGLU of its row).
constexpr int kFusedSwigluPairs = 100, kFusedSwigluBlocks = 8;

void launch_weighted_reduce(const uint16_t* pairs, const float* weights, const int32_t* ids, int experts, int tokens, int top_k,
                            int width, void* out, int out_dtype, hipStream_t stream) {
    // small outputs want many threads rather than wide ones
    const bool wide = width % 8 == 0 && reinterpret_cast<uintptr_t>(pairs) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                      static_cast<int64_t>(tokens) * width >= (1 << 18);
    if (wide) {
        const int64_t count = static_cast<int64_t>(tokens) * (width / 8);
        hipLaunchKernelGGL(dev::weighted_reduce8_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, stream,
                           pairs, weights, ids, experts, tokens, top_k, width, out, out_dtype);
    } else {
        const int64_t count = static_cast<int64_t>(tokens) * width;
        const dim3 grid(static_cast<unsigned>((count + 255) / 256));
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, pairs, weights, ids, experts, tokens, top_k, width, out, out_dtype);
        };
        switch (top_k) {
            case 1: launch(dev::weighted_reduce_kernel<1>); break;
            case 2: launch(dev::weighted_reduce_kernel<2>); break;
            case 4: launch(dev::weighted_reduce_kernel<4>); break;
            case 6: launch(dev::weighted_reduce_kernel<6>); break;
            case 8: launch(dev::weighted_reduce_kernel<8>); break;
            case 10: launch(dev::weighted_reduce_kernel<10>); break;
            default: launch(dev::weighted_reduce_kernel<0>); break;
        }
    }
    check_launch("weighted_reduce_kernel");
}
}  // namespace

bool rows_fast_geometry(int in_width, int in_dtype) {
    return in_width % dev::kLaneColumns == 0 && in_width <= dev::kWave * dev::kLaneColumns && in_dtype != MFQ_AMD_F32;
}

// A wave step covers 4 rows when 64 lanes share a row and 16 rows when 16 lanes do; a block has four waves.
int rows_fast_min_block(int in_width) { return in_width <= 16 * dev::kLaneColumns ? 64 : 16; }

bool pool_fast_layout(const mfq_amd_projection& p) {
    const int cls = projection_class(p);
    if (!dev::fast_class(cls) || p.input_width % dev::kLaneColumns != 0) return false;
    if (p.family == MFQ_AMD_FAMILY_NINT) return p.groups >= 2;
    if (p.family == MFQ_AMD_FAMILY_NVQ)
        return p.sub_bits == 4 && p.sign_mode == 0 && p.sizes[0] >= 16 && p.sizes[2] >= 2;
    return true;
}

void launch_rows_fast(const RowsArgs& args, int slots, bool nvq, hipStream_t stream) {
    if (args.pairs <= 0) return;
    MFQ_REQUIRE(rows_fast_geometry(args.in_width, args.in_dtype), "geometry is not served by the streaming kernel");
    const int least = rows_fast_min_block(args.in_width);
    MFQ_REQUIRE(args.rows_per_block >= least && args.rows_per_block % least == 0, "invalid rows per block");
    (void)nvq;
    const int bytes = 0;
    const dim3 grid((args.out_rows + args.rows_per_block - 1) / args.rows_per_block, args.pairs, slots);
    const bool narrow = args.in_width <= 16 * dev::kLaneColumns;
    const int wave_slots = args.rows_per_block / (narrow ? 16 : 4);
    auto launch = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(256), bytes, stream, args); };
    // by the number of row slots per wave: straight-line variants for the block heights the FFN uses, the looped kernel
    // (0) for the rest; by the activations: hidden rows computed by the block, rows in the packed form, plain rows
    auto by_slots = [&](auto lpr, auto xmode, auto nt) {
        constexpr int L = decltype(lpr)::value, X = decltype(xmode)::value, N = decltype(nt)::value;
        if (wave_slots == 4) launch(dev::moe_rows_fast_kernel<L, X, 4, N>);
        else if (wave_slots == 8) launch(dev::moe_rows_fast_kernel<L, X, 8, N>);
        else if (wave_slots == 16) launch(dev::moe_rows_fast_kernel<L, X, 16, N>);
        else launch(dev::moe_rows_fast_kernel<L, X, 0, N>);
    };
    auto by_group = [&](auto lpr, auto xmode) {
        if (args.grouped) by_slots(lpr, xmode, std::integral_constant<int, kGroupPairs>{});
        else by_slots(lpr, xmode, std::integral_constant<int, 1>{});
    };
    using lanes16 = std::integral_constant<int, 16>;
    using lanes64 = std::integral_constant<int, 64>;
    if (args.gu != nullptr) {
        MFQ_REQUIRE(narrow && args.in_per_pair && args.sigmoid != nullptr, "the fused SwiGLU serves rows of at most 512 columns");
        by_group(lanes16{}, std::integral_constant<int, dev::kXScaled>{});
    } else if (args.in_packed != nullptr) {
        if (narrow) by_group(lanes16{}, std::integral_constant<int, dev::kXPacked>{});
        else by_group(lanes64{}, std::integral_constant<int, dev::kXPacked>{});
    } else {
        MFQ_REQUIRE(!args.grouped, "grouped pairs are served from packed activations");
        if (narrow) launch(dev::moe_rows_fast_kernel<16, dev::kXRaw, 0, 1>);
        else launch(dev::moe_rows_fast_kernel<64, dev::kXRaw, 0, 1>);
    }
    check_launch("moe_rows_fast_kernel");
}

void launch_rows_exact(const RowsArgs& args, int slots, const int* present, const int* max_items, hipStream_t stream) {
    for (int c = 0; c < dev::K_CLASS_COUNT; ++c) {
        if (!present[c] || max_items[c] <= 0) continue;
        dev::RowsExactLaunch launch{args, slots, max_items[c], stream};
        dev::dispatch_class(c, launch);
        check_launch("moe_rows_exact_kernel");
    }
}

// IEEE binary64 -> binary16 with one rounding (the reference's half type converts a double directly).
uint16_t double_to_half(double value) {
    uint64_t u;
    std::memcpy(&u, &value, 8);
    const uint16_t sign = static_cast<uint16_t>((u >> 48) & 0x8000u);
    const int64_t exp = static_cast<int64_t>((u >> 52) & 0x7ff);
    const uint64_t man = u & 0xfffffffffffffull;
    if (exp == 0x7ff) return static_cast<uint16_t>(sign | 0x7c00u | (man ? 0x200u : 0u));
    if (exp == 0) return sign;
    const int64_t e = exp - 1023;
    const uint64_t sig = man | (1ull << 52);
    int shift;
    int64_t half_exp;
    if (e >= -14) { shift = 42; half_exp = e + 15; }
    else {
        const int64_t extra = -14 - e;
        if (extra > 12) return sign;
        shift = 42 + static_cast<int>(extra); half_exp = 0;
    }
    uint64_t kept = sig >> shift;
    const uint64_t rem = sig & ((1ull << shift) - 1ull), halfway = 1ull << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1ull))) ++kept;
    uint32_t out = half_exp > 0 ? static_cast<uint32_t>((half_exp - 1) << 10) + static_cast<uint32_t>(kept)
                                : static_cast<uint32_t>(kept);
    if (out >= 0x7c00u) out = 0x7c00u;
    return static_cast<uint16_t>(sign | out);
}

float half_to_float_host(uint16_t h) {
    const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    float v;
    if (exp == 0) v = std::ldexp(static_cast<float>(man), -24);
    else if (exp == 31) v = man ? NAN : INFINITY;
    else v = std::ldexp(static_cast<float>(man | 0x400u), static_cast<int>(exp) - 25);
    return sign ? -v : v;
}

namespace {

template <class T>
T* device_alloc(size_t count) {
    void* p = nullptr;
    MFQ_HIP(hipMalloc(&p, sizeof(T) * (count ? count : 1)));
    return static_cast<T*>(p);
}

// Scratch memory of mfq_amd_grouped_matmul_static: one copy per device that loads the library, held until the
// process ends.  In host code the name stands for the symbol, not for device memory: its per-device address comes
// from hipGetSymbolAddress (device_state()) and only that address is handed to kernels.
constexpr int64_t kStaticScratchBytes = 128 * 1024;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_state_mutex;
DeviceState g_states[kMaxDevices];
bool g_state_ready[kMaxDevices];

// Device-side tables of a set of pools: descriptors, kernel classes, per-expert bytes.
struct PoolTables {
    std::vector<mfq_amd_projection> pools;
    std::vector<int32_t> classes;
    std::vector<int64_t> bytes;
    int slot_begin[kSlots + 1] = {0, 0, 0, 0};
    int present[kSlots][dev::K_CLASS_COUNT] = {};         // classes with at least one pool
    int exact_present[kSlots][dev::K_CLASS_COUNT] = {};   // classes with a pool the streaming kernel cannot serve
    int class_experts[kSlots][dev::K_CLASS_COUNT] = {};
    int fast_nvq[kSlots] = {};                            // the slot has an NVQ pool on the streaming path

    void add_slot(int slot, const mfq_amd_moe_tensor& t) {
        MFQ_REQUIRE(t.pools && t.pool_count > 0 && t.pool_count <= kMaxPoolsPerTensor, "1..12 pools per tensor");
        MFQ_REQUIRE(t.experts > 0 && t.out_per_expert > 0 && t.neuron_len > 0, "invalid MoE tensor geometry");
        slot_begin[slot] = static_cast<int>(pools.size());
        for (int i = 0; i < t.pool_count; ++i) {
            const mfq_amd_projection p = canonical_projection(t.pools[i]);
            validate_projection(p, 0);
            MFQ_REQUIRE(p.output_rows == t.out_per_expert && p.input_width == t.neuron_len,
                        "pool geometry does not match its tensor");
            MFQ_REQUIRE(p.expert_local != nullptr || t.pool_count == 1, "pools of a mixed tensor need expert_local maps");
            const int cls = projection_class(p);
            const bool fast = pool_fast_layout(p);
            pools.push_back(p);
            classes.push_back(fast ? cls : (cls | kPoolExactOnly));
            bytes.push_back(projection_expert_bytes(p));
            present[slot][cls] = 1;
            if (!fast) exact_present[slot][cls] = 1;
            if (fast && p.family == MFQ_AMD_FAMILY_NVQ) fast_nvq[slot] = 1;
            class_experts[slot][cls] += p.local_experts;
        }
        slot_begin[slot + 1] = static_cast<int>(pools.size());
    }
};

}  // namespace

const DeviceState& device_state() {
    int device = 0;
    MFQ_HIP(hipGetDevice(&device));
    MFQ_REQUIRE(device >= 0 && device < kMaxDevices, "device index out of range");
    std::lock_guard<std::mutex> lock(g_state_mutex);
    if (!g_state_ready[device]) {
        std::vector<uint16_t> table(65536);
        for (uint32_t h = 0; h < 65536; ++h) {
            const double g = static_cast<double>(half_to_float_host(static_cast<uint16_t>(h)));
            table[h] = double_to_half(1.0 / (1.0 + std::exp(-g)));
        }
        uint16_t* sigmoid = device_alloc<uint16_t>(65536);   // lives until the process ends
        MFQ_HIP(hipMemcpy(sigmoid, table.data(), sizeof(uint16_t) * 65536, hipMemcpyHostToDevice));
        raise_routing_limits();
        raise_prefill_limits();
        void* scratch_at = nullptr;
        MFQ_HIP(hipGetSymbolAddress(&scratch_at, HIP_SYMBOL(scratch)));
        MFQ_REQUIRE(scratch_at != nullptr && reinterpret_cast<uintptr_t>(scratch_at) % 256 == 0, "static scratch array has no usable device address");
        g_states[device].static_scratch = scratch_at;
        g_states[device].sigmoid_table = sigmoid;
        g_state_ready[device] = true;
    }
    return g_states[device];
}

const DeviceState* device_state_if_ready() {
    int device = 0;
    MFQ_HIP(hipGetDevice(&device));
    MFQ_REQUIRE(device >= 0 && device < kMaxDevices, "device index out of range");
    std::lock_guard<std::mutex> lock(g_state_mutex);
    return g_state_ready[device] ? &g_states[device] : nullptr;
}

}  // namespace mfq_amd

using namespace mfq_amd;

extern "C" int mfq_amd_init(void) {
    return guarded([&] { (void)device_state(); });
}

extern "C" int32_t mfq_amd_moe_ffn_decode_limit(int32_t requested, int32_t top_k) {
    if (top_k < 1) return 0;
    const int32_t limit = requested > 0 ? requested : 32;
    const int32_t most = kPlanThreads / top_k;    // a decode plan is one thread per routed pair
    return limit < most ? limit : most;
}

struct mfq_amd_moe_ffn {
    mfq_amd_moe_ffn_config config{};
    PoolTables tables;
    int experts = 0, hidden = 0, intermediate = 0, top_k = 0, max_tokens = 0, decode_limit = 32;
    mfq_amd_projection* d_pools = nullptr;
    int32_t* d_pool_class = nullptr;
    int64_t* d_pool_bytes = nullptr;
    PlanItem* d_item_info = nullptr;
    PairItem* d_pair_items = nullptr;
    ExpertInfo* d_expert_info = nullptr;
    uint32_t* d_expert_words = nullptr;
    int32_t *d_expert_pool = nullptr, *d_items = nullptr, *d_class_offsets = nullptr, *d_tile_items = nullptr,
            *d_tile_offsets = nullptr, *d_counts = nullptr, *d_bounds = nullptr,
            *d_ids_dst = nullptr, *d_distinct = nullptr;
    int64_t* d_touched = nullptr;
    uint16_t *d_gu = nullptr, *d_hidden = nullptr, *d_pairs = nullptr;
    const uint16_t* d_sigmoid = nullptr;   // the device's table: not owned
    int32_t* d_wave_base = nullptr;      // scratch of the two-kernel route plan
    float activation_limit = 0.0f;       // what swiglu_bits() takes: the clamp of the gated activation, or kActivationRelu2
    float* d_logits = nullptr;           // router logits of run_router
    int32_t* d_route_ids = nullptr;      // routes selected by run_logits
    float* d_route_weights = nullptr;
    uint32_t *d_x_packed = nullptr, *d_hidden_packed = nullptr;
    uint8_t *d_fp8 = nullptr, *d_fp8_scales = nullptr;   // prefill, block-scaled MFMA: activations as E4M3 terms and their block scales
    bool mx_scaled[kSlots] = {false, false, false};      // the slot has MXFP4 pools that run on the block-scaled MFMA
    uint16_t* d_x_tiles = nullptr;       // prefill: fp16 copies of the token rows in the pair layouts of the gate/up pools
    uint32_t x_tile_layouts = 0;         // mask of those layouts   // decode only: activations as the streaming kernels read them
    int tile_capacity = 0;
    hipStream_t last_stream = nullptr;
    const int32_t* last_ids = nullptr;   // routing of the last run (for touched_bytes)
    int last_pairs = 0;
    // the layer's shared expert: a dense FFN of one expert that every token runs (set_shared), its route (expert 0, weight 1)
    // and its output rows
    mfq_amd_moe_ffn* shared = nullptr;
    int32_t* d_shared_ids = nullptr;
    float* d_shared_weights = nullptr;
    uint16_t* d_shared_out = nullptr;
    bool decode_needs_items = true;   // some decode work runs on the exact kernels, which read the item lists
    bool timing = false;
    hipEvent_t events[7] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};   // the last closes an empty bracket

    ~mfq_amd_moe_ffn() {
        void* all[] = {d_pools, d_pool_class, d_pool_bytes, d_expert_pool, d_expert_info, d_expert_words, d_item_info, d_pair_items, d_items, d_class_offsets, d_tile_items,
                       d_tile_offsets, d_counts, d_bounds, d_ids_dst, d_distinct,
                       d_touched, d_gu, d_hidden, d_pairs, d_logits, d_x_packed, d_hidden_packed, d_route_ids, d_route_weights, d_x_tiles, d_wave_base, d_fp8, d_fp8_scales,
                       d_shared_ids, d_shared_weights, d_shared_out};
        for (void* p : all) if (p) (void)hipFree(p);
        delete shared;
        for (hipEvent_t e : events) if (e) (void)hipEventDestroy(e);
    }
    void mark(int index, hipStream_t stream) {
        if (timing) MFQ_HIP(hipEventRecord(events[index], stream));
    }
};

extern "C" int mfq_amd_moe_ffn_create(const mfq_amd_moe_ffn_config* config, mfq_amd_moe_ffn** out) {
    return guarded([&] {
        MFQ_REQUIRE(config && out, "null argument");
        auto f = std::make_unique<mfq_amd_moe_ffn>();
        f->config = *config;
        const auto& c = *config;
        MFQ_REQUIRE(c.top_k >= 1 && c.top_k <= 32 && c.max_tokens >= 1, "invalid FFN batch geometry");
        MFQ_REQUIRE(c.x_dtype >= MFQ_AMD_F32 && c.x_dtype <= MFQ_AMD_BF16, "unknown activation dtype");
        MFQ_REQUIRE(c.out_dtype == MFQ_AMD_F32 || c.out_dtype == MFQ_AMD_F16, "output must be float32 or float16");
        MFQ_REQUIRE(c.launch_mode == 0 || c.launch_mode == 1, "unknown launch mode");
        MFQ_REQUIRE(c.mx_scaled_mfma == 0 || c.mx_scaled_mfma == 1, "mx_scaled_mfma must be 0 or 1");
        MFQ_REQUIRE(c.expert_activation == 0 || c.expert_activation == 1, "expert_activation must be 0 or 1");
        MFQ_REQUIRE(c.group_pairs == 0 || c.group_pairs == 1, "group_pairs must be 0 or 1");
        MFQ_REQUIRE(c.swiglu_limit >= 0.0f, "swiglu_limit must not be negative");
        const bool gated = c.expert_activation == 0;
        if (gated) {
            MFQ_REQUIRE(c.gate.experts == c.up.experts && c.gate.neuron_len == c.up.neuron_len &&
                        c.gate.out_per_expert == c.up.out_per_expert, "gate and up shapes differ");
        } else {
            MFQ_REQUIRE(c.gate.pool_count == 0 && c.gate.pools == nullptr, "the relu-squared activation has no gate projection");
            MFQ_REQUIRE(c.swiglu_limit == 0.0f, "swiglu_limit applies to the gated activation only");
        }
        MFQ_REQUIRE(c.up.experts == c.down.experts, "expert counts differ");
        MFQ_REQUIRE(c.down.neuron_len == c.up.out_per_expert && c.down.out_per_expert == c.up.neuron_len,
                    "gate/up/down shapes do not form an FFN");
        MFQ_REQUIRE(c.up.experts <= kPlanMaxExperts, "at most 1024 experts");
        f->experts = c.up.experts; f->hidden = c.up.neuron_len; f->intermediate = c.up.out_per_expert;
        f->top_k = c.top_k; f->max_tokens = c.max_tokens;
        f->decode_limit = mfq_amd_moe_ffn_decode_limit(c.decode_token_limit, c.top_k);
        f->activation_limit = gated ? c.swiglu_limit : dev::kActivationRelu2;
        if (gated) f->tables.add_slot(0, c.gate);      // no gate: the slot has no pools and every expert is absent from it
        f->tables.add_slot(1, c.up);
        f->tables.add_slot(2, c.down);
        // every expert must live in exactly one pool of every slot
        const int E = f->experts;
        std::vector<int32_t> expert_pool(static_cast<size_t>(kSlots) * E, -1), expert_local(static_cast<size_t>(kSlots) * E, 0);
        for (int s = 0; s < kSlots; ++s) {
            std::vector<int> owners(E, 0);
            for (int j = f->tables.slot_begin[s]; j < f->tables.slot_begin[s + 1]; ++j) {
                const auto& p = f->tables.pools[j];
                if (!p.expert_local) {
                    MFQ_REQUIRE(E == 1, "a dense pool can only serve a single expert");
                    owners[0]++; expert_pool[static_cast<size_t>(s) * E] = j;
                    continue;
                }
                std::vector<int32_t> local(E);
                MFQ_HIP(hipMemcpy(local.data(), p.expert_local, sizeof(int32_t) * E, hipMemcpyDeviceToHost));
                for (int e = 0; e < E; ++e) {
                    MFQ_REQUIRE(local[e] < p.local_experts, "expert_local index exceeds the pool");
                    if (local[e] >= 0) {
                        owners[e]++;
                        expert_pool[static_cast<size_t>(s) * E + e] = j;
                        expert_local[static_cast<size_t>(s) * E + e] = local[e];
                    }
                }
            }
            for (int e = 0; e < E; ++e)
                if (owners[e] != (s == 0 && !gated ? 0 : 1)) fail_unsupported("every expert must belong to exactly one pool of each projection");
        }
        const size_t pools = f->tables.pools.size();
        f->d_pools = device_alloc<mfq_amd_projection>(pools);
        f->d_pool_class = device_alloc<int32_t>(pools);
        f->d_pool_bytes = device_alloc<int64_t>(pools);
        MFQ_HIP(hipMemcpy(f->d_pools, f->tables.pools.data(), sizeof(mfq_amd_projection) * pools, hipMemcpyHostToDevice));
        MFQ_HIP(hipMemcpy(f->d_pool_class, f->tables.classes.data(), sizeof(int32_t) * pools, hipMemcpyHostToDevice));
        MFQ_HIP(hipMemcpy(f->d_pool_bytes, f->tables.bytes.data(), sizeof(int64_t) * pools, hipMemcpyHostToDevice));
        const int64_t pairs = static_cast<int64_t>(c.max_tokens) * c.top_k;
        f->tile_capacity = static_cast<int>(pairs / kPrefillTileM + E + 1);
        f->d_expert_pool = device_alloc<int32_t>(kSlots * E);
        MFQ_HIP(hipMemcpy(f->d_expert_pool, expert_pool.data(), sizeof(int32_t) * kSlots * E, hipMemcpyHostToDevice));
        {
            std::vector<ExpertInfo> info(static_cast<size_t>(kSlots) * E);
            for (size_t i = 0; i < info.size(); ++i) {
                const int pool = expert_pool[i];
                info[i] = ExpertInfo{pool, expert_local[i], pool >= 0 ? f->tables.classes[pool] : -1, 0,
                                     pool >= 0 ? f->tables.bytes[pool] : 0};
            }
            f->d_expert_info = device_alloc<ExpertInfo>(info.size());
            MFQ_HIP(hipMemcpy(f->d_expert_info, info.data(), sizeof(ExpertInfo) * info.size(), hipMemcpyHostToDevice));
            MFQ_REQUIRE(pools <= 64, "at most 64 pools per FFN");
            std::vector<uint32_t> words(info.size());
            for (size_t i = 0; i < info.size(); ++i) words[i] = expert_word(info[i].pool, info[i].local, info[i].cls);
            f->d_expert_words = device_alloc<uint32_t>(words.size());
            MFQ_HIP(hipMemcpy(f->d_expert_words, words.data(), sizeof(uint32_t) * words.size(), hipMemcpyHostToDevice));
        }
        f->d_items = device_alloc<int32_t>(kSlots * E);
        f->d_item_info = device_alloc<PlanItem>(kSlots * E);
        f->d_pair_items = device_alloc<PairItem>(kSlots * pairs);
        f->d_class_offsets = device_alloc<int32_t>(kSlots * kClassSlots);
        f->d_tile_items = device_alloc<int32_t>(static_cast<size_t>(kSlots) * f->tile_capacity);
        f->d_tile_offsets = device_alloc<int32_t>(kSlots * kClassSlots);
        f->d_counts = device_alloc<int32_t>(E);
        f->d_bounds = device_alloc<int32_t>(E + 1);
        f->d_ids_dst = device_alloc<int32_t>(pairs);
        f->d_distinct = device_alloc<int32_t>(1);
        f->d_touched = device_alloc<int64_t>(1);
        f->d_gu = device_alloc<uint16_t>(pairs * 2 * f->intermediate);
        f->d_hidden = device_alloc<uint16_t>(pairs * f->intermediate);
        f->d_pairs = device_alloc<uint16_t>(pairs * f->hidden);
        f->d_sigmoid = device_state().sigmoid_table;
        f->d_logits = device_alloc<float>(static_cast<size_t>(c.max_tokens) * E);
        f->d_route_ids = device_alloc<int32_t>(pairs);
        f->d_route_weights = device_alloc<float>(pairs);
        f->d_wave_base = device_alloc<int32_t>(static_cast<size_t>(kPlanThreads / 64) * E);
        if (c.launch_mode == 0 && c.max_tokens > f->decode_limit && tiles_fast_geometry(f->hidden, c.x_dtype, 1)) {
            for (int s = 0; s < 2; ++s)
                for (int i = f->tables.slot_begin[s]; i < f->tables.slot_begin[s + 1]; ++i)
                    if (!(f->tables.classes[i] & kPoolExactOnly)) f->x_tile_layouts |= 1u << tile_layout_of_class(f->tables.classes[i]);
            if (f->x_tile_layouts) f->d_x_tiles = device_alloc<uint16_t>(static_cast<size_t>(4) * c.max_tokens * f->hidden);
            if (c.mx_scaled_mfma && c.x_dtype != MFQ_AMD_F32 && tiles_fast_geometry(f->intermediate, MFQ_AMD_F16, 1)) {
                bool any = false;
                for (int s = 0; s < kSlots; ++s) {
                    f->mx_scaled[s] = f->tables.present[s][dev::K_MXFP4] && !f->tables.exact_present[s][dev::K_MXFP4];
                    any = any || f->mx_scaled[s];
                }
                if (any) {
                    const size_t most = std::max(static_cast<size_t>(c.max_tokens) * f->hidden, static_cast<size_t>(pairs) * f->intermediate) * 3;
                    f->d_fp8 = device_alloc<uint8_t>(most);
                    f->d_fp8_scales = device_alloc<uint8_t>(most / dev::kLaneColumns);
                }
            }
        }
        {
            bool exact_work = c.launch_mode != 0 || !rows_fast_geometry(f->hidden, c.x_dtype) ||
                              !rows_fast_geometry(f->intermediate, MFQ_AMD_F16);
            for (int s = 0; s < kSlots; ++s)
                for (int k = 0; k < dev::K_CLASS_COUNT; ++k) exact_work = exact_work || f->tables.exact_present[s][k];
            f->decode_needs_items = exact_work;
        }
        {
            const int64_t decode_tokens = f->decode_limit < c.max_tokens ? f->decode_limit : c.max_tokens;
            if (rows_fast_geometry(f->hidden, c.x_dtype))
                f->d_x_packed = device_alloc<uint32_t>(decode_tokens * dev::xpack_row_dwords(f->hidden));
            if (rows_fast_geometry(f->intermediate, MFQ_AMD_F16))
                f->d_hidden_packed = device_alloc<uint32_t>(decode_tokens * c.top_k * dev::xpack_row_dwords(f->intermediate));
        }
        MFQ_HIP(hipMemset(f->d_gu, 0, sizeof(uint16_t) * pairs * 2 * f->intermediate));
        MFQ_HIP(hipMemset(f->d_pairs, 0, sizeof(uint16_t) * pairs * f->hidden));
        MFQ_HIP(hipDeviceSynchronize());
        *out = f.release();
    });
}

namespace {
// One layer.  `route`: select the routes from logits inside the plan kernel (decode sizes only) into
// the object's own id and weight buffers; otherwise ids_dev / route_weights_dev are the caller's.
void ffn_run(mfq_amd_moe_ffn* f, const void* x_dev, const int32_t* ids_dev, const float* route_weights_dev, int tokens,
             void* out_dev, hipStream_t stream, const PlanRoute* route, bool reduce = true) {
    {
        f->last_stream = stream;
        f->last_ids = ids_dev;
        f->last_pairs = tokens * f->top_k;
        const int E = f->experts, k = f->top_k, H = f->hidden, I = f->intermediate;
        const int pairs = tokens * k;
        const bool decode = tokens <= f->decode_limit;

        PlanArgs plan{};
        plan.ids = ids_dev; plan.pairs = pairs; plan.experts = E; plan.tile_m = 8; plan.top_k = k;
        plan.counts = f->d_counts; plan.expert_bounds = f->d_bounds; plan.ids_dst = f->d_ids_dst;
        // the per-8-route tile lists of the reference plan are not consumed by the decode kernels
        // (the route tile tables of mfq_amd_route_plan are not asked for: the kernels here walk tile_items)
        plan.wave_base = !decode && pairs > 4 * kPlanThreads ? f->d_wave_base : nullptr;
        auto& x = plan.extras;
        x.pools = f->d_pools; x.pool_class = f->d_pool_class; x.pool_bytes = f->d_pool_bytes;
        for (int s = 0; s <= kSlots; ++s) x.slot_pool_begin[s] = f->tables.slot_begin[s];
        x.slots = kSlots;
        x.expert_pool = nullptr; x.expert_info = f->d_expert_info; x.expert_words = f->d_expert_words;
        x.items = f->d_items; x.item_info = f->d_item_info; x.pair_items = decode ? f->d_pair_items : nullptr; x.class_offsets = f->d_class_offsets;
        x.tile_items = f->d_tile_items; x.tile_offsets = f->d_tile_offsets;
        x.touched_bytes = f->d_touched; x.distinct = f->d_distinct;
        x.tile_capacity = f->tile_capacity; x.prefill_tile_m = kPrefillTileM; x.want_tiles = decode ? 0 : 1;
        x.want_items = !decode || f->decode_needs_items;
        // a streaming decode step needs nothing but the pair lists
        x.pairs_only = decode && !x.want_items && f->config.launch_mode == 0 && pairs <= kPlanSortPairs;
        const bool fast_mode = decode && f->config.launch_mode == 0;
        const bool pack_x = fast_mode && f->d_x_packed != nullptr;
        // the down blocks compute the hidden row of their pair themselves when nothing else reads it
        // (every block of a pair repeats the SwiGLU and the packing of its row: a kernel less against that.  Measured at
        // 512 experts x (2048 <-> 512), top-10, per step: batch 1 -4 us, batch 4 -5 us; batch 16 +0.5 us with sixteen
        // down blocks per pair and -2.7 us with eight, batch 32 -3.1 us with eight)
        int down_height = 256;     // as rows_per_block() below will choose it for the down launch
        while (down_height > 64 && static_cast<int64_t>(pairs) * ((H + down_height - 1) / down_height) < 1024) down_height /= 2;
        const bool fuse_swiglu = fast_mode && !f->decode_needs_items && I <= 16 * dev::kLaneColumns && rows_fast_geometry(I, MFQ_AMD_F16) &&
                                 (pairs <= kFusedSwigluPairs || (H + down_height - 1) / down_height <= kFusedSwigluBlocks);
        const bool pack_hidden = fast_mode && !fuse_swiglu && f->d_hidden_packed != nullptr;
        // On request the plan groups up to kGroupPairs neighbouring pairs of one expert and a block of the rows kernels
        // fetches and decodes the expert's rows once for the group (the reference's per-token-group form,
        // mfq/kernels/cuda/mfe_mxfp4_dot.cuh:36-68).  Not the default: with the pairs of an expert next to each other its
        // rows come out of the L2 for all but the first pair anyway, and the group's blocks hold twice the registers, so
        // half the waves (2048 <-> 512 layer of 16..64 experts, top-8, batches 4..32: 38..130 us per step in groups
        // against 28..90 us with a block per pair).
        x.group_pairs = x.pairs_only && pack_x && (fuse_swiglu || pack_hidden) && f->config.group_pairs == 1;
        if (pack_x) {
            plan.pack.src = x_dev; plan.pack.dst = f->d_x_packed; plan.pack.stride = dev::xpack_row_dwords(H);
            plan.pack.rows = tokens; plan.pack.width = H; plan.pack.dtype = f->config.x_dtype;
            plan.pack.vector_ok = reinterpret_cast<uintptr_t>(x_dev) % 16 == 0 &&
                                  (static_cast<int64_t>(H) * (f->config.x_dtype == MFQ_AMD_F32 ? 4 : 2)) % 16 == 0;
        }
        // prefill: the fp16 copies of the activations in the pair layouts of the tile kernel are made by the spare
        // blocks of the plan kernel (the plan itself keeps one CU busy)
        const int x_element = f->config.x_dtype == MFQ_AMD_F32 ? 4 : 2;
        const bool x_vector_ok = reinterpret_cast<uintptr_t>(x_dev) % 16 == 0 && (static_cast<int64_t>(H) * x_element) % 16 == 0;
        const bool x_tiles = !decode && f->d_x_tiles != nullptr && tiles_fast_geometry(H, f->config.x_dtype, x_vector_ok) &&
                             tiles_packed_geometry(H, tokens);
        if (x_tiles) {
            plan.tiles.src = x_dev; plan.tiles.dst = f->d_x_tiles; plan.tiles.layout_stride = static_cast<int64_t>(tokens) * H;
            plan.tiles.rows = tokens; plan.tiles.width = H; plan.tiles.dtype = f->config.x_dtype; plan.tiles.layouts = f->x_tile_layouts;
        }
        f->mark(0, stream);
        if (route != nullptr) plan.route = *route;
        launch_route_plan(plan, stream);
        f->mark(1, stream);

        RowsArgs rows{};
        rows.pools = f->d_pools; rows.expert_pool = f->d_expert_pool; rows.expert_info = f->d_expert_info;
        rows.pool_class = f->d_pool_class; rows.items = f->d_items;
        rows.item_info = f->d_item_info; rows.pair_items = f->d_pair_items; rows.pairs = pairs;
        rows.class_offsets = f->d_class_offsets; rows.tile_items = f->d_tile_items; rows.tile_offsets = f->d_tile_offsets;
        rows.expert_bounds = f->d_bounds; rows.ids_dst = f->d_ids_dst;
        rows.experts = E; rows.top_k = k; rows.tile_capacity = f->tile_capacity;
        rows.grouped = x.group_pairs;

        int present[dev::K_CLASS_COUNT], bound[dev::K_CLASS_COUNT];
        // classes to launch over slots [slot_lo, slot_hi): every present class, or only those with
        // pools the streaming kernel cannot serve
        auto class_bounds = [&](int slot_lo, int slot_hi, bool tiles, bool exact_only) {
            bool any = false;
            for (int c = 0; c < dev::K_CLASS_COUNT; ++c) {
                present[c] = 0; bound[c] = 0;
                for (int s = slot_lo; s < slot_hi; ++s) {
                    present[c] |= exact_only ? f->tables.exact_present[s][c] : f->tables.present[s][c];
                    const int experts_c = f->tables.class_experts[s][c];
                    const int limit = tiles ? pairs / kPrefillTileM + experts_c : (pairs < experts_c ? pairs : experts_c);
                    bound[c] = bound[c] > limit ? bound[c] : limit;
                }
                any = any || present[c];
            }
            return any;
        };
        const int active_bound = pairs < E ? pairs : E;
        int rows_in_width = 0;
        // Enough blocks to fill the chip at small batches, long row runs per wave at large ones: the tallest block with
        // straight-line code (16 row slots per wave: 64 rows of more than 512 columns, 256 rows of at most 512, about
        // 64 KB of packed rows either way), halved while the
        // launch has fewer blocks than the chip holds at once (measured at 512 experts x (2048 <-> 512), top-10: a floor
        // of 1024 blocks against 2048 gives 41.9 vs 43.1 us per step at batch 4 and 57.2 vs 60.1 us at batch 8, and
        // leaves batches 1, 2 and 16 where they were; 512 is slower everywhere.  At batch 16 the down launch takes
        // 22.7 us with 256 rows per block against 23.7 with 128; gate+up with 128 rows per block 39.8 against 38.7)
        auto rows_per_block = [&](int out_rows, int slots) {
            const int least = rows_fast_min_block(rows_in_width);
            int height = rows_in_width > 16 * dev::kLaneColumns ? 64 : 256;
            // blocks of the launch along the pair axis: the pairs, or about the groups where blocks serve groups of pairs
            int64_t units = pairs;
            if (rows.grouped) units = std::max<int64_t>(std::min<int64_t>(pairs, E), (pairs + kGroupPairs - 1) / kGroupPairs);
            while (height > least && units * slots * ((out_rows + height - 1) / height) < 1024) height /= 2;
            return height;
        };
        auto run_rows = [&](int slot_lo, int slot_hi) {
            const int slots = slot_hi - slot_lo;
            if (!decode) {
                const bool tiles = f->config.launch_mode == 0 && tiles_fast_geometry(rows.in_width, rows.in_dtype, rows.in_vector_ok);
                if (!tiles) rows.in_tiles = nullptr;
                if (tiles) {
                    bool nvq = false, mx = false;
                    for (int s = slot_lo; s < slot_hi; ++s) { nvq = nvq || f->tables.fast_nvq[s]; mx = mx || f->mx_scaled[s]; }
                    mx = mx && f->d_fp8 != nullptr;
                    if (mx) {
                        // MXFP4 tiles on the block-scaled MFMA: the activations of the stage as E4M3 terms first.  The
                        // split reads its rows in plain column order; hidden rows written for the tile kernel are in the
                        // layout of their down pool's class, which for MXFP4 must therefore be the plain one.
                        MFQ_REQUIRE(tile_layout_of_class(dev::K_MXFP4) == 2, "the E4M3 split reads MXFP4 rows in column order");
                        const int terms = rows.in_dtype == MFQ_AMD_BF16 ? 2 : 3;
                        launch_fp8_split(rows.in, rows.in_dtype, rows.in_per_pair ? pairs : tokens, rows.in_width, terms, f->d_fp8,
                                         f->d_fp8_scales, stream);
                        rows.in_fp8 = f->d_fp8; rows.in_fp8_scales = f->d_fp8_scales; rows.in_fp8_terms = terms;
                    }
                    rows.skip_mxfp4 = mx ? 1 : 0;
                    launch_tiles_fast(rows, slots, pairs / kPrefillTileM + active_bound, nvq, stream);
                    if (mx) launch_tiles_mx_scaled(rows, slots, pairs / kPrefillTileM + active_bound, stream);
                }
                rows.exact_only = tiles ? 1 : 0;
                if (class_bounds(slot_lo, slot_hi, true, tiles)) launch_rows_prefill(rows, slots, present, bound, stream);
                return;
            }
            const bool fast = f->config.launch_mode == 0 && rows_fast_geometry(rows.in_width, rows.in_dtype);
            if (fast) {
                bool nvq = false;
                for (int s = slot_lo; s < slot_hi; ++s) nvq = nvq || f->tables.fast_nvq[s];
                rows_in_width = rows.in_width;
                rows.rows_per_block = rows_per_block(rows.out_rows, slots);
                launch_rows_fast(rows, slots, nvq, stream);
            }
            rows.exact_only = fast ? 1 : 0;
            if (class_bounds(slot_lo, slot_hi, false, fast)) launch_rows_exact(rows, slots, present, bound, stream);
        };

        // gate and up: x[token] -> gu[pair][slot][I]
        const int element = f->config.x_dtype == MFQ_AMD_F32 ? 4 : 2;
        rows.in = x_dev; rows.in_dtype = f->config.x_dtype; rows.in_per_pair = 0; rows.in_width = H;
        rows.in_vector_ok = reinterpret_cast<uintptr_t>(x_dev) % 16 == 0 && (static_cast<int64_t>(H) * element) % 16 == 0;
        rows.out = f->d_gu; rows.out_pair_stride = 2 * static_cast<int64_t>(I); rows.out_slot_stride = I;
        rows.slot_base = 0; rows.out_rows = I;
        rows.in_packed = pack_x ? f->d_x_packed : nullptr; rows.in_packed_stride = dev::xpack_row_dwords(H);
        if (x_tiles) { rows.in_tiles = f->d_x_tiles; rows.in_tiles_layout_stride = static_cast<int64_t>(tokens) * H; }
        run_rows(0, 2);
        f->mark(2, stream);

        const bool hidden_tiles = !decode && f->config.launch_mode == 0 && f->d_expert_info != nullptr &&
                                  tiles_fast_geometry(I, MFQ_AMD_F16, 1) && tiles_packed_geometry(I, pairs);
        if (fuse_swiglu) {
            // no kernel of its own
        } else if (hidden_tiles) {
            launch_swiglu_tiles(f->d_gu, f->d_gu + I, 2 * static_cast<int64_t>(I), I, pairs, f->activation_limit, f->d_sigmoid,
                                ids_dev, f->d_expert_info + 2 * static_cast<int64_t>(E), E, f->d_hidden, stream);
        } else if (pack_hidden) {
            const size_t bytes = (static_cast<size_t>(I) * 2 + 15) / 16 * 16 + 64;
            hipLaunchKernelGGL(dev::swiglu_pack_kernel, dim3(pairs), dim3(256), bytes, stream, f->d_gu, f->d_gu + I,
                               2 * static_cast<int64_t>(I), I, f->activation_limit, f->d_sigmoid, f->d_hidden,
                               f->d_hidden_packed, dev::xpack_row_dwords(I));
            check_launch("swiglu_pack_kernel");
        } else {
            const int64_t count = static_cast<int64_t>(pairs) * I;
            hipLaunchKernelGGL(dev::swiglu_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, stream,
                               f->d_gu, f->d_gu + I, count, 2 * static_cast<int64_t>(I), static_cast<int64_t>(I), f->activation_limit,
                               f->d_sigmoid, f->d_hidden);
            check_launch("swiglu_kernel");
        }
        f->mark(3, stream);

        // down: hidden[pair] -> pairs[pair][H]
        rows.in = f->d_hidden; rows.in_dtype = MFQ_AMD_F16; rows.in_per_pair = 1; rows.in_width = I;
        rows.in_vector_ok = (static_cast<int64_t>(I) * 2) % 16 == 0;
        rows.out = f->d_pairs; rows.out_pair_stride = H; rows.out_slot_stride = 0;
        rows.slot_base = 2; rows.out_rows = H;
        rows.in_packed = pack_hidden ? f->d_hidden_packed : nullptr; rows.in_packed_stride = dev::xpack_row_dwords(I);
        if (fuse_swiglu) { rows.gu = f->d_gu; rows.sigmoid = f->d_sigmoid; rows.swiglu_limit = f->activation_limit; }
        rows.in_tiles = hidden_tiles ? f->d_hidden : nullptr; rows.in_tiles_layout_stride = 0;
        run_rows(2, 3);
        f->mark(4, stream);

        // (a layer with a shared expert sums the pair rows in its own epilogue)
        if (reduce) launch_weighted_reduce(f->d_pairs, route_weights_dev, ids_dev, E, tokens, k, H, out_dev, f->config.out_dtype, stream);
        f->mark(5, stream); f->mark(6, stream);
    }
}
}  // namespace

extern "C" int mfq_amd_moe_ffn_run(mfq_amd_moe_ffn* f, const void* x_dev, const int32_t* ids_dev,
                                   const float* route_weights_dev, int32_t tokens, void* out_dev, void* stream_ptr) {
    return guarded([&] {
        MFQ_REQUIRE(f, "null argument");
        MFQ_REQUIRE(tokens >= 0 && tokens <= f->max_tokens, "token count exceeds the workspace capacity");
        if (tokens == 0) return;                   // an empty batch: nothing is read, the buffers may be null
        MFQ_REQUIRE(x_dev && ids_dev && route_weights_dev && out_dev, "null argument");
        ffn_run(f, x_dev, ids_dev, route_weights_dev, tokens, out_dev, as_stream(stream_ptr), nullptr);
    });
}

extern "C" int mfq_amd_moe_ffn_run_logits(mfq_amd_moe_ffn* f, const void* x_dev, const void* logits_dev,
                                          int32_t logits_dtype, int32_t normalize, float norm_floor, float scale,
                                          int32_t tokens, void* out_dev, void* stream_ptr) {
    return guarded([&] {
        MFQ_REQUIRE(f, "null argument");
        MFQ_REQUIRE(tokens >= 0 && tokens <= f->max_tokens, "token count exceeds the workspace capacity");
        MFQ_REQUIRE(logits_dtype >= MFQ_AMD_F32 && logits_dtype <= MFQ_AMD_BF16, "logits must be float32, float16 or bfloat16");
        MFQ_REQUIRE(f->top_k <= f->experts, "top_k exceeds the number of experts");
        if (tokens == 0) return;
        MFQ_REQUIRE(x_dev && logits_dev && out_dev, "null argument");
        hipStream_t stream = as_stream(stream_ptr);
        PlanRoute route{};
        route.logits = logits_dev; route.dtype = logits_dtype; route.tokens = tokens; route.normalize = normalize;
        route.norm_floor = norm_floor; route.scale = scale; route.ids_out = f->d_route_ids; route.weights_out = f->d_route_weights;
        const bool fused = tokens <= f->decode_limit && tokens <= kPlanThreads / 32 && tokens * f->top_k <= kPlanThreads;
        if (!fused) {
            // larger batches: the stand-alone top-k kernel, then the layer
            const int status = mfq_amd_topk(logits_dev, logits_dtype, tokens, f->experts, f->top_k, normalize, norm_floor, scale,
                                            f->d_route_ids, f->d_route_weights, stream_ptr);
            if (status != MFQ_AMD_OK) throw std::runtime_error(mfq_amd_last_error());
        }
        ffn_run(f, x_dev, f->d_route_ids, f->d_route_weights, tokens, out_dev, stream, fused ? &route : nullptr);
    });
}

extern "C" int mfq_amd_moe_ffn_run_router(mfq_amd_moe_ffn* f, const void* x_dev, const void* router_dev, int32_t router_dtype,
                                          int32_t normalize, float norm_floor, float scale, int32_t tokens, void* out_dev,
                                          void* stream_ptr) {
    const int status = guarded([&] {
        MFQ_REQUIRE(f, "null argument");
        MFQ_REQUIRE(tokens >= 0 && tokens <= f->max_tokens, "token count exceeds the workspace capacity");
        MFQ_REQUIRE(router_dtype >= MFQ_AMD_F32 && router_dtype <= MFQ_AMD_BF16, "router weights must be float32, float16 or bfloat16");
        if (tokens == 0) return;
        MFQ_REQUIRE(x_dev && router_dev && out_dev, "null argument");
        launch_router_logits(x_dev, f->config.x_dtype, router_dev, router_dtype, tokens, f->experts, f->hidden, f->d_logits,
                             as_stream(stream_ptr));
    });
    if (status != MFQ_AMD_OK || tokens == 0) return status;
    return mfq_amd_moe_ffn_run_logits(f, x_dev, f->d_logits, MFQ_AMD_F32, normalize, norm_floor, scale, tokens, out_dev, stream_ptr);
}

extern "C" int mfq_amd_moe_ffn_set_shared(mfq_amd_moe_ffn* f, const mfq_amd_projection* gate, const mfq_amd_projection* up,
                                          const mfq_amd_projection* down, int32_t shared_activation) {
    return guarded([&] {
        MFQ_REQUIRE(f && up && down, "null argument");
        MFQ_REQUIRE(shared_activation == 0 || shared_activation == 1, "shared_activation must be 0 or 1");
        MFQ_REQUIRE((gate != nullptr) == (shared_activation == 0), "the gate projection is absent exactly for the relu-squared activation");
        MFQ_REQUIRE(up->local_experts == 1 && down->local_experts == 1 && (!gate || gate->local_experts == 1),
                    "the shared expert is a dense FFN: one expert per projection");
        MFQ_REQUIRE(up->input_width == f->hidden && down->output_rows == f->hidden, "the shared expert does not fit the layer's width");
        mfq_amd_moe_ffn_config c{};
        auto dense = [](const mfq_amd_projection* p) {
            mfq_amd_moe_tensor t{};
            if (p != nullptr) { t.pools = p; t.pool_count = 1; t.experts = 1; t.out_per_expert = p->output_rows; t.neuron_len = p->input_width; }
            return t;
        };
        c.gate = dense(gate); c.up = dense(up); c.down = dense(down);
        c.top_k = 1; c.max_tokens = f->max_tokens; c.x_dtype = f->config.x_dtype; c.out_dtype = MFQ_AMD_F16;
        c.swiglu_limit = shared_activation == 0 ? f->config.swiglu_limit : 0.0f;
        c.decode_token_limit = f->config.decode_token_limit; c.launch_mode = f->config.launch_mode;
        c.expert_activation = shared_activation;
        mfq_amd_moe_ffn* made = nullptr;
        if (mfq_amd_moe_ffn_create(&c, &made) != MFQ_AMD_OK) throw std::runtime_error(mfq_amd_last_error());
        delete f->shared;
        f->shared = made;
        if (f->d_shared_ids == nullptr) {
            f->d_shared_ids = device_alloc<int32_t>(f->max_tokens);
            f->d_shared_weights = device_alloc<float>(f->max_tokens);
            f->d_shared_out = device_alloc<uint16_t>(static_cast<size_t>(f->max_tokens) * f->hidden);
            std::vector<float> ones(f->max_tokens, 1.0f);
            MFQ_HIP(hipMemset(f->d_shared_ids, 0, sizeof(int32_t) * f->max_tokens));
            MFQ_HIP(hipMemcpy(f->d_shared_weights, ones.data(), sizeof(float) * ones.size(), hipMemcpyHostToDevice));
        }
    });
}

extern "C" int mfq_amd_moe_ffn_run_shared(mfq_amd_moe_ffn* f, const void* x_dev, const int32_t* ids_dev, const float* route_weights_dev,
                                          const void* shared_gate_dev, int32_t shared_gate_dtype, int32_t tokens, void* out_dev,
                                          void* stream_ptr) {
    return guarded([&] {
        MFQ_REQUIRE(f, "null argument");
        MFQ_REQUIRE(f->shared != nullptr, "the layer has no shared expert: call mfq_amd_moe_ffn_set_shared first");
        MFQ_REQUIRE(shared_gate_dtype >= MFQ_AMD_F32 && shared_gate_dtype <= MFQ_AMD_BF16, "shared gate values must be float32, float16 or bfloat16");
        MFQ_REQUIRE(tokens >= 0 && tokens <= f->max_tokens, "token count exceeds the workspace capacity");
        if (tokens == 0) return;
        MFQ_REQUIRE(x_dev && ids_dev && route_weights_dev && shared_gate_dev && out_dev, "null argument");
        hipStream_t stream = as_stream(stream_ptr);
        ffn_run(f, x_dev, ids_dev, route_weights_dev, tokens, nullptr, stream, nullptr, false);
        ffn_run(f->shared, x_dev, f->d_shared_ids, f->d_shared_weights, tokens, f->d_shared_out, stream, nullptr);
        const int64_t count = static_cast<int64_t>(tokens) * f->hidden;
        hipLaunchKernelGGL(dev::shared_expert_reduce_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, stream,
                           f->d_pairs, route_weights_dev, ids_dev, f->experts, f->d_shared_out, shared_gate_dev, shared_gate_dtype, tokens,
                           f->top_k, f->hidden, out_dev, f->config.out_dtype);
        check_launch("shared_expert_reduce_kernel");
    });
}

extern "C" int mfq_amd_moe_ffn_routes(mfq_amd_moe_ffn* f, const int32_t** ids_dev, const float** weights_dev) {
    return guarded([&] {
        MFQ_REQUIRE(f, "null argument");
        if (ids_dev) *ids_dev = f->d_route_ids;
        if (weights_dev) *weights_dev = f->d_route_weights;
    });
}

extern "C" int mfq_amd_moe_ffn_mx_scaled_slots(mfq_amd_moe_ffn* f, int32_t* mask) {
    return guarded([&] {
        MFQ_REQUIRE(f && mask, "null argument");
        *mask = 0;
        for (int s = 0; s < kSlots; ++s)
            if (f->mx_scaled[s] && f->d_fp8) *mask |= 1 << s;
    });
}

extern "C" int mfq_amd_moe_ffn_enable_timing(mfq_amd_moe_ffn* f, int32_t enable) {
    return guarded([&] {
        MFQ_REQUIRE(f, "null argument");
        if (enable && !f->events[0])
            for (auto& e : f->events) MFQ_HIP(hipEventCreate(&e));
        f->timing = enable != 0;
    });
}

extern "C" int mfq_amd_moe_ffn_stage_times(mfq_amd_moe_ffn* f, float* ms5) {
    return guarded([&] {
        MFQ_REQUIRE(f && ms5, "null argument");
        MFQ_REQUIRE(f->timing && f->events[0], "stage timing is not enabled");
        MFQ_HIP(hipEventSynchronize(f->events[5]));
        for (int i = 0; i < 5; ++i) MFQ_HIP(hipEventElapsedTime(&ms5[i], f->events[i], f->events[i + 1]));
    });
}

extern "C" int mfq_amd_moe_ffn_empty_bracket_ms(mfq_amd_moe_ffn* f, float* ms) {
    return guarded([&] {
        MFQ_REQUIRE(f && ms, "null argument");
        MFQ_REQUIRE(f->timing && f->events[0], "stage timing is not enabled");
        MFQ_HIP(hipEventSynchronize(f->events[6]));
        MFQ_HIP(hipEventElapsedTime(ms, f->events[5], f->events[6]));
    });
}

extern "C" int mfq_amd_moe_ffn_buffers(mfq_amd_moe_ffn* f, const void** gate_up_f16, const void** pairs_f16) {
    return guarded([&] {
        MFQ_REQUIRE(f, "null argument");
        if (gate_up_f16) *gate_up_f16 = f->d_gu;
        if (pairs_f16) *pairs_f16 = f->d_pairs;
    });
}

extern "C" int mfq_amd_moe_ffn_touched_bytes(mfq_amd_moe_ffn* f, int64_t* bytes, int32_t* distinct_experts) {
    return guarded([&] {
        MFQ_REQUIRE(f, "null argument");
        MFQ_REQUIRE(f->last_ids != nullptr, "no run yet");
        launch_touched_bytes(f->last_ids, f->last_pairs, f->experts, kSlots, f->d_expert_info, f->d_touched, f->d_distinct,
                             f->last_stream);
        MFQ_HIP(hipStreamSynchronize(f->last_stream));
        if (bytes) MFQ_HIP(hipMemcpy(bytes, f->d_touched, sizeof(int64_t), hipMemcpyDeviceToHost));
        if (distinct_experts) MFQ_HIP(hipMemcpy(distinct_experts, f->d_distinct, sizeof(int32_t), hipMemcpyDeviceToHost));
    });
}

extern "C" void mfq_amd_moe_ffn_destroy(mfq_amd_moe_ffn* f) { delete f; }

// ------------------------------------------------------------------------------------------------
// grouped projection over one mixed tensor
// ------------------------------------------------------------------------------------------------
namespace {
struct GroupedLayout {
    int64_t pools, pool_class, pool_bytes, expert_pool, items, item_info, pair_items, class_offsets, tile_items, tile_offsets, counts, bounds,
            ids_dst, touched, distinct, total;
    int tile_capacity;
};
GroupedLayout grouped_layout(int tokens, int top_k, int experts) {
    GroupedLayout g{};
    const int64_t pairs = static_cast<int64_t>(tokens) * top_k;
    g.tile_capacity = static_cast<int>(pairs / kPrefillTileM + experts + 1);
    int64_t off = 0;
    auto take = [&](int64_t bytes) { const int64_t at = off; off += (bytes + 255) / 256 * 256; return at; };
    g.pools = take(sizeof(mfq_amd_projection) * kMaxPoolsPerTensor);
    g.pool_class = take(4 * kMaxPoolsPerTensor);
    g.pool_bytes = take(8 * kMaxPoolsPerTensor);
    g.expert_pool = take(4 * experts);
    g.items = take(4 * experts);
    g.item_info = take(static_cast<int64_t>(sizeof(PlanItem)) * experts);
    g.pair_items = take(static_cast<int64_t>(sizeof(PairItem)) * (pairs + 1));
    g.class_offsets = take(4 * kClassSlots);
    g.tile_items = take(4 * static_cast<int64_t>(g.tile_capacity));
    g.tile_offsets = take(4 * kClassSlots);
    g.counts = take(4 * experts);
    g.bounds = take(4 * (experts + 1));
    g.ids_dst = take(4 * (pairs + 1));
    g.touched = take(8);
    g.distinct = take(4);
    g.total = off;
    return g;
}

struct PoolBlock {
    mfq_amd_projection pools[kMaxPoolsPerTensor];
    int32_t classes[kMaxPoolsPerTensor];
    int64_t bytes[kMaxPoolsPerTensor];
    int32_t count;
};
}  // namespace

namespace mfq_amd { namespace dev {
// Copies the descriptor block (a kernel argument) into device memory so that later kernels can
// index it; keeps the whole call free of host-to-device copies.
__global__ void stage_pools_kernel(PoolBlock block, mfq_amd_projection* pools, int32_t* classes, int64_t* bytes) {
    const int i = threadIdx.x;
    if (i < block.count) { pools[i] = block.pools[i]; classes[i] = block.classes[i]; bytes[i] = block.bytes[i]; }
}
}}

extern "C" int64_t mfq_amd_grouped_matmul_workspace(int32_t tokens, int32_t top_k, int32_t experts) {
    if (tokens < 0 || top_k <= 0 || experts <= 0) return 0;
    return grouped_layout(tokens, top_k, experts).total;
}

namespace {
void grouped_matmul(const mfq_amd_moe_tensor* tensor, const void* x_dev, int32_t x_dtype, int32_t x_rows_per_token,
                    const int32_t* ids_dev, int32_t tokens, int32_t top_k, void* out_f16_dev, void* workspace_dev,
                    int64_t workspace_bytes, void* stream_ptr) {
    {
        MFQ_REQUIRE(tensor && x_dev && ids_dev && out_f16_dev && workspace_dev, "null argument");
        MFQ_REQUIRE(tokens >= 0 && top_k >= 1, "invalid route geometry");
        MFQ_REQUIRE(x_rows_per_token == 1 || x_rows_per_token == top_k, "x must be [tokens, K] or [tokens, routes, K]");
        MFQ_REQUIRE(x_dtype >= MFQ_AMD_F32 && x_dtype <= MFQ_AMD_BF16, "unknown activation dtype");
        MFQ_REQUIRE(tensor->experts <= kPlanMaxExperts, "at most 1024 experts");
        if (tokens == 0) return;
        PoolTables tables;
        tables.add_slot(0, *tensor);
        const GroupedLayout g = grouped_layout(tokens, top_k, tensor->experts);
        MFQ_REQUIRE(workspace_bytes >= g.total, "workspace is too small");
        MFQ_REQUIRE(reinterpret_cast<uintptr_t>(workspace_dev) % 256 == 0, "workspace must be 256-byte aligned");
        hipStream_t stream = as_stream(stream_ptr);
        char* ws = static_cast<char*>(workspace_dev);
        auto at = [&](int64_t off) { return ws + off; };
        PoolBlock block{};
        block.count = static_cast<int32_t>(tables.pools.size());
        for (int i = 0; i < block.count; ++i) {
            block.pools[i] = tables.pools[i]; block.classes[i] = tables.classes[i]; block.bytes[i] = tables.bytes[i];
        }
        hipLaunchKernelGGL(dev::stage_pools_kernel, dim3(1), dim3(64), 0, stream, block,
                           reinterpret_cast<mfq_amd_projection*>(at(g.pools)), reinterpret_cast<int32_t*>(at(g.pool_class)),
                           reinterpret_cast<int64_t*>(at(g.pool_bytes)));
        check_launch("stage_pools_kernel");

        const int E = tensor->experts, pairs = tokens * top_k;
        PlanArgs plan{};
        plan.ids = ids_dev; plan.pairs = pairs; plan.experts = E; plan.tile_m = 8; plan.top_k = top_k;
        plan.counts = reinterpret_cast<int32_t*>(at(g.counts));
        plan.expert_bounds = reinterpret_cast<int32_t*>(at(g.bounds));
        plan.ids_dst = reinterpret_cast<int32_t*>(at(g.ids_dst));
        auto& x = plan.extras;
        x.pools = reinterpret_cast<const mfq_amd_projection*>(at(g.pools));
        x.pool_class = reinterpret_cast<const int32_t*>(at(g.pool_class));
        x.pool_bytes = reinterpret_cast<const int64_t*>(at(g.pool_bytes));
        x.slot_pool_begin[0] = 0; x.slot_pool_begin[1] = block.count; x.slots = 1;
        x.expert_pool = reinterpret_cast<int32_t*>(at(g.expert_pool)); x.expert_info = nullptr;
        x.items = reinterpret_cast<int32_t*>(at(g.items));
        x.item_info = reinterpret_cast<PlanItem*>(at(g.item_info));
        x.pair_items = reinterpret_cast<PairItem*>(at(g.pair_items));
        x.class_offsets = reinterpret_cast<int32_t*>(at(g.class_offsets));
        x.tile_items = reinterpret_cast<int32_t*>(at(g.tile_items));
        x.tile_offsets = reinterpret_cast<int32_t*>(at(g.tile_offsets));
        x.touched_bytes = reinterpret_cast<int64_t*>(at(g.touched));
        x.distinct = reinterpret_cast<int32_t*>(at(g.distinct));
        x.tile_capacity = g.tile_capacity; x.prefill_tile_m = kPrefillTileM; x.want_tiles = tokens <= 8 ? 0 : 1; x.want_items = 1;
        launch_route_plan(plan, stream);

        RowsArgs rows{};
        rows.pools = x.pools; rows.expert_pool = x.expert_pool; rows.expert_info = nullptr; rows.pool_class = x.pool_class; rows.items = x.items; rows.item_info = x.item_info; rows.pair_items = x.pair_items; rows.pairs = pairs;
        rows.class_offsets = x.class_offsets;
        rows.tile_items = x.tile_items; rows.tile_offsets = x.tile_offsets; rows.expert_bounds = plan.expert_bounds;
        rows.ids_dst = plan.ids_dst; rows.experts = E; rows.top_k = top_k; rows.tile_capacity = g.tile_capacity;
        const int element = x_dtype == MFQ_AMD_F32 ? 4 : 2;
        rows.in = x_dev; rows.in_dtype = x_dtype; rows.in_per_pair = x_rows_per_token == 1 ? 0 : 1;
        rows.in_width = tensor->neuron_len;
        rows.in_vector_ok = reinterpret_cast<uintptr_t>(x_dev) % 16 == 0 &&
                            (static_cast<int64_t>(tensor->neuron_len) * element) % 16 == 0;
        rows.out = static_cast<uint16_t*>(out_f16_dev); rows.out_pair_stride = tensor->out_per_expert;
        rows.out_slot_stride = 0; rows.slot_base = 0; rows.out_rows = tensor->out_per_expert;
        // same split as the reference: up to 8 tokens stream, more use the tile kernels
        // (cpp_runtime/backends/cuda/ops/moe.cpp:275, :1639)
        const bool decode = tokens <= 8;
        int bound[dev::K_CLASS_COUNT];
        for (int c = 0; c < dev::K_CLASS_COUNT; ++c) {
            const int experts_c = tables.class_experts[0][c];
            bound[c] = decode ? (pairs < experts_c ? pairs : experts_c) : pairs / kPrefillTileM + experts_c;
        }
        if (!decode) {
            const bool tiles = tiles_fast_geometry(rows.in_width, rows.in_dtype, rows.in_vector_ok);
            if (tiles) launch_tiles_fast(rows, 1, pairs / kPrefillTileM + (pairs < E ? pairs : E), tables.fast_nvq[0] != 0, stream);
            rows.exact_only = tiles ? 1 : 0;
            bool any = false;
            for (int c = 0; c < dev::K_CLASS_COUNT; ++c) any = any || (tiles ? tables.exact_present[0][c] : tables.present[0][c]);
            if (any) launch_rows_prefill(rows, 1, tiles ? tables.exact_present[0] : tables.present[0], bound, stream);
            return;
        }
        const bool fast = rows_fast_geometry(rows.in_width, rows.in_dtype);
        if (fast) {
            rows.rows_per_block = 64;   // a multiple of both minimum block heights
            launch_rows_fast(rows, 1, tables.fast_nvq[0] != 0, stream);
        }
        rows.exact_only = fast ? 1 : 0;
        bool any = false;
        for (int c = 0; c < dev::K_CLASS_COUNT; ++c) any = any || (fast ? tables.exact_present[0][c] : tables.present[0][c]);
        if (any) launch_rows_exact(rows, 1, fast ? tables.exact_present[0] : tables.present[0], bound, stream);
    }
}
}  // namespace

extern "C" int mfq_amd_grouped_matmul(const mfq_amd_moe_tensor* tensor, const void* x_dev, int32_t x_dtype,
                                      int32_t x_rows_per_token, const int32_t* ids_dev, int32_t tokens, int32_t top_k,
                                      void* out_f16_dev, void* workspace_dev, int64_t workspace_bytes, void* stream_ptr) {
    return guarded([&] {
        grouped_matmul(tensor, x_dev, x_dtype, x_rows_per_token, ids_dev, tokens, top_k, out_f16_dev, workspace_dev,
                       workspace_bytes, stream_ptr);
    });
}

extern "C" int64_t mfq_amd_grouped_matmul_static_capacity(void) { return kStaticScratchBytes; }

extern "C" int mfq_amd_grouped_matmul_static(const mfq_amd_moe_tensor* tensor, const void* x_dev, int32_t x_dtype,
                                             int32_t x_rows_per_token, const int32_t* ids_dev, int32_t tokens,
                                             int32_t top_k, void* out_f16_dev, void* stream_ptr) {
    return guarded([&] {
        MFQ_REQUIRE(tensor, "null argument");
        MFQ_REQUIRE(tokens >= 0 && top_k >= 1 && tensor->experts > 0, "invalid route geometry");
        MFQ_REQUIRE(tensor && tokens >= 0 && top_k >= 1 && tensor->experts > 0 && tensor->experts <= kPlanMaxExperts,
                    "invalid route geometry");
        const int64_t needed = mfq_amd_grouped_matmul_workspace(tokens, top_k, tensor->experts);
        if (needed > kStaticScratchBytes)
            fail_invalid("route plan of " + std::to_string(needed) + " bytes exceeds the static scratch of " +
                         std::to_string(kStaticScratchBytes) + " bytes: use mfq_amd_grouped_matmul with a workspace");
        const DeviceState* state = device_state_if_ready();
        MFQ_REQUIRE(state != nullptr, "mfq_amd_init() must have run on this device before the allocation-free entry point");
        // every plan list is written before it is read, so nothing of the previous call's contents needs clearing
        grouped_matmul(tensor, x_dev, x_dtype, x_rows_per_token, ids_dev, tokens, top_k, out_f16_dev, state->static_scratch,
                       kStaticScratchBytes, stream_ptr);
    });
}

extern "C" int mfq_amd_swiglu(const void* gate_f16_dev, const void* up_f16_dev, int64_t count, float swiglu_limit,
                              void* hidden_f16_dev, void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(gate_f16_dev && up_f16_dev && hidden_f16_dev && count >= 0, "invalid argument");
        if (!count) return;
        const uint16_t* table = device_state().sigmoid_table;
        hipLaunchKernelGGL(dev::swiglu_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0,
                           as_stream(stream), static_cast<const uint16_t*>(gate_f16_dev),
                           static_cast<const uint16_t*>(up_f16_dev), count, count, count,
                           swiglu_limit, table, static_cast<uint16_t*>(hidden_f16_dev));
        check_launch("swiglu_kernel");
    });
}

extern "C" int mfq_amd_weighted_reduce(const void* pairs_f16_dev, const float* weights_dev, int32_t tokens, int32_t top_k,
                                       int32_t width, void* out_dev, int32_t out_dtype, void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(pairs_f16_dev && weights_dev && out_dev, "null argument");
        MFQ_REQUIRE(tokens >= 0 && top_k > 0 && width > 0, "invalid reduce geometry");
        MFQ_REQUIRE(out_dtype == MFQ_AMD_F32 || out_dtype == MFQ_AMD_F16, "output must be float32 or float16");
        if (!tokens) return;
        launch_weighted_reduce(static_cast<const uint16_t*>(pairs_f16_dev), weights_dev, nullptr, 0, tokens, top_k, width, out_dev,
                               out_dtype, as_stream(stream));
    });
}

extern "C" int mfq_amd_weighted_reduce_shared_gate(const void* pairs_f16_dev, const float* weights_dev,
                                                   const void* shared_f16_dev, const float* gate_logits_dev, int32_t tokens,
                                                   int32_t top_k, int32_t width, void* out_f16_dev, void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(tokens >= 0 && top_k > 0 && width > 0, "invalid reduce geometry");
        if (!tokens) return;
        MFQ_REQUIRE(pairs_f16_dev && weights_dev && shared_f16_dev && gate_logits_dev && out_f16_dev, "null argument");
        const int64_t count = static_cast<int64_t>(tokens) * width;
        hipLaunchKernelGGL(dev::shared_gate_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0,
                           as_stream(stream), static_cast<const uint16_t*>(nullptr), static_cast<const uint16_t*>(pairs_f16_dev),
                           weights_dev, static_cast<const uint16_t*>(shared_f16_dev), gate_logits_dev, tokens, top_k, width,
                           static_cast<uint16_t*>(out_f16_dev));
        check_launch("shared_gate_kernel");
    });
}

extern "C" int mfq_amd_add_shared_gate(const void* routed_f16_dev, const void* shared_f16_dev, const float* gate_logits_dev,
                                       int32_t rows, int32_t width, void* out_f16_dev, void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(rows >= 0 && width > 0, "invalid geometry");
        if (!rows) return;
        MFQ_REQUIRE(routed_f16_dev && shared_f16_dev && gate_logits_dev && out_f16_dev, "null argument");
        const int64_t count = static_cast<int64_t>(rows) * width;
        hipLaunchKernelGGL(dev::shared_gate_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0,
                           as_stream(stream), static_cast<const uint16_t*>(routed_f16_dev), static_cast<const uint16_t*>(nullptr),
                           static_cast<const float*>(nullptr), static_cast<const uint16_t*>(shared_f16_dev), gate_logits_dev, rows,
                           1, width, static_cast<uint16_t*>(out_f16_dev));
        check_launch("shared_gate_kernel");
    });
}
