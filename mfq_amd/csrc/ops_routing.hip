// Routing: reproducible router logits, softmax top-k, and the pair-by-expert route plan.
#include "common.h"
#include "decode.cuh"
#include "device_state.h"
#include "plan.h"
#include "tile_pack.cuh"
#include "xpack.cuh"

namespace mfq_amd {
namespace dev {

// ------------------------------------------------------------ logits ----
// One block = one token x 64 experts.  Router rows are staged through LDS so global reads are
// coalesced; each thread then adds its expert's products in ascending column order with a
// separate multiply and add, which fixes the fp32 result independently of the launch shape.
__global__ void __launch_bounds__(64) router_logits_kernel(const void* x, int x_dtype, const void* router,
                                                           int router_dtype, int experts, int width, float* logits) {
    __shared__ float tile[64][65];
    __shared__ float xs[64];
    const int token = blockIdx.y, e0 = blockIdx.x * 64, lane = threadIdx.x;
    const int xe = x_dtype == MFQ_AMD_F32 ? 4 : 2, re = router_dtype == MFQ_AMD_F32 ? 4 : 2;
    float sum = 0.0f;
    for (int c0 = 0; c0 < width; c0 += 64) {
        const int c = c0 + lane;
        float xv = 0.0f;
        if (c < width) {
            const char* p = static_cast<const char*>(x) + (static_cast<int64_t>(token) * width + c) * xe;
            xv = x_dtype == MFQ_AMD_F32 ? *reinterpret_cast<const float*>(p)
               : x_dtype == MFQ_AMD_F16 ? half_bits_to_float(*reinterpret_cast<const uint16_t*>(p))
                                        : bf16_bits_to_float(*reinterpret_cast<const uint16_t*>(p));
        }
        xs[lane] = xv;
        for (int r = 0; r < 64; ++r) {
            float wv = 0.0f;
            if (e0 + r < experts && c < width) {
                const char* p = static_cast<const char*>(router) + (static_cast<int64_t>(e0 + r) * width + c) * re;
                wv = router_dtype == MFQ_AMD_F32 ? *reinterpret_cast<const float*>(p)
                   : router_dtype == MFQ_AMD_F16 ? half_bits_to_float(*reinterpret_cast<const uint16_t*>(p))
                                                 : bf16_bits_to_float(*reinterpret_cast<const uint16_t*>(p));
            }
            tile[r][lane] = wv;
        }
        __syncthreads();
        const int n = width - c0 < 64 ? width - c0 : 64;
        for (int i = 0; i < n; ++i) {
            const float term = xs[i] * tile[lane][i];
            sum = sum + term;
        }
        __syncthreads();
    }
    if (e0 + lane < experts) logits[static_cast<int64_t>(token) * experts + e0 + lane] = sum;
}

// The same logits for fp16 / bf16 operands, one thread per (token, expert).  The product of two such values is exact
// in fp32, so a fused multiply-add gives the very sum of the separate multiply and add above (products below 2^-126
// excepted, which cannot move a sum of ordinary magnitude); what remains is the chain of `width` dependent additions
// the fixed order asks for, and every chain has a thread of its own.  A block = 64 experts x 4 tokens (one wave per
// token): the router rows pass through LDS in tiles of 128 columns, loaded with coalesced 16-byte requests one tile
// ahead of their use; a wave's activations are wave-uniform.
constexpr int kRouterTile = 64;                        // columns per LDS tile
constexpr int kRouterPitch = kRouterTile * 4 + 16;     // bytes per expert row in LDS (fp32): the pad keeps 16-byte reads conflict-free
__global__ void __launch_bounds__(256) router_logits_chain_kernel(const uint16_t* x, int x_half, const uint16_t* router, int router_half,
                                                                  int tokens, int experts, int width, float* logits) {
    // Both operands are widened to fp32 once, by the thread that stages them: a single wave per SIMD issues an
    // instruction every five cycles or so, so the inner loop is kept to the fused multiply-add and its LDS reads.
    __shared__ __attribute__((aligned(16))) unsigned char tile[2][64 * kRouterPitch];
    __shared__ __attribute__((aligned(16))) float x_tile[2][4 * kRouterTile];      // the four tokens' columns of the tile
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int e0 = blockIdx.x * 64;
    const int token = blockIdx.y * 4 + wave;
    auto widen = [](uint32_t bits, int half) { return half ? half_bits_to_float(static_cast<uint16_t>(bits)) : bits_to_float(bits << 16); };
    // staging role: thread -> rows tid / 8 and tid / 8 + 32 of the tile, its 16-byte piece tid % 8 (eight columns)
    const int piece = tid & 7, first_row = tid >> 3;
    uint4 staged[2], staged_x = {0u, 0u, 0u, 0u};
    const int x_token = blockIdx.y * 4 + (tid >> 3) < tokens ? blockIdx.y * 4 + (tid >> 3) : tokens - 1;   // threads 0..31: token tid / 8
    auto load_tile = [&](int c0) {
        if (tid < 32) staged_x = *reinterpret_cast<const uint4*>(x + static_cast<int64_t>(x_token) * width + c0 + piece * 8);
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int row = first_row + 32 * k;
            const int expert = e0 + row < experts ? e0 + row : experts - 1;
            staged[k] = *reinterpret_cast<const uint4*>(router + static_cast<int64_t>(expert) * width + c0 + piece * 8);
        }
    };
    auto store_wide = [&](const uint4& v, int half, float* to) {
        const uint32_t words[4] = {v.x, v.y, v.z, v.w};
        float4 lo, hi;
        lo.x = widen(words[0] & 0xffffu, half); lo.y = widen(words[0] >> 16, half);
        lo.z = widen(words[1] & 0xffffu, half); lo.w = widen(words[1] >> 16, half);
        hi.x = widen(words[2] & 0xffffu, half); hi.y = widen(words[2] >> 16, half);
        hi.z = widen(words[3] & 0xffffu, half); hi.w = widen(words[3] >> 16, half);
        reinterpret_cast<float4*>(to)[0] = lo;
        reinterpret_cast<float4*>(to)[1] = hi;
    };
    auto store_tile = [&](int buffer) {
        if (tid < 32) store_wide(staged_x, x_half, &x_tile[buffer][(tid >> 3) * kRouterTile + piece * 8]);
#pragma unroll
        for (int k = 0; k < 2; ++k)
            store_wide(staged[k], router_half, reinterpret_cast<float*>(tile[buffer] + (first_row + 32 * k) * kRouterPitch) + piece * 8);
    };
    const int full = width / kRouterTile * kRouterTile;          // columns covered by whole tiles
    float sum = 0.0f;
    if (full > 0) load_tile(0);
    for (int c0 = 0; c0 < full; c0 += kRouterTile) {
        const int buffer = (c0 / kRouterTile) & 1;
        store_tile(buffer);
        __syncthreads();
        if (c0 + kRouterTile < full) load_tile(c0 + kRouterTile);
        const float* mine = reinterpret_cast<const float*>(tile[buffer] + lane * kRouterPitch);
        const float* xs = &x_tile[buffer][wave * kRouterTile];
#pragma unroll
        for (int c = 0; c < kRouterTile; c += 4) {
            const float4 wv = *reinterpret_cast<const float4*>(mine + c);
            const float4 xv = *reinterpret_cast<const float4*>(xs + c);
            sum = fmaf(xv.x, wv.x, sum);
            sum = fmaf(xv.y, wv.y, sum);
            sum = fmaf(xv.z, wv.z, sum);
            sum = fmaf(xv.w, wv.w, sum);
        }
        // the buffer written two tiles from now is the one just read: every wave must be done with it first
        __syncthreads();
    }
    const int expert = e0 + lane;
    const uint16_t* w = router + static_cast<int64_t>(expert < experts ? expert : experts - 1) * width;
    const uint16_t* xr = x + static_cast<int64_t>(token < tokens ? token : tokens - 1) * width;
    for (int c = full; c < width; ++c) sum = fmaf(widen(xr[c], x_half), widen(w[c], router_half), sum);
    if (expert < experts && token < tokens) logits[static_cast<int64_t>(token) * experts + expert] = sum;
}

// ------------------------------------------------------------- top-k ----
__device__ __forceinline__ float load_logit(const void* logits, int dtype, int64_t index) {
    float raw;
    if (dtype == MFQ_AMD_F32) raw = static_cast<const float*>(logits)[index];
    else if (dtype == MFQ_AMD_F16) raw = half_bits_to_float(static_cast<const uint16_t*>(logits)[index]);
    else raw = bf16_bits_to_float(static_cast<const uint16_t*>(logits)[index]);
    return raw != raw ? -3.402823466e+38f : raw;
}

// Exchanges between lanes without the LDS round trip of a shuffle.  swap_rows<16>: the value of the lane 16 places away
// inside its group of 32 (both lanes end up with the same two values, `low` the one of the lower lane); swap_rows<32>:
// the same between the halves of the wave.
template <int DISTANCE>
__device__ __forceinline__ void swap_rows(float v, float& low, float& high) {
    const unsigned bits = __float_as_uint(v);
    const auto swapped = DISTANCE == 16 ? __builtin_amdgcn_permlane16_swap(bits, bits, false, false)
                                        : __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    low = __uint_as_float(static_cast<unsigned>(swapped[0]));
    high = __uint_as_float(static_cast<unsigned>(swapped[1]));
}
template <int CTRL>
__device__ __forceinline__ float dpp32(float v) {
    return __uint_as_float(static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(__float_as_uint(v)), CTRL, 0xF, 0xF, false)));
}

// Lane 0 of a 32-lane shuffle-down tree, offsets 16, 8, 4, 2, 1 (v[i] + v[i + offset] at every step, the order of
// additions the reference's reduction has), in every lane of the group of 32.  Only the lanes that feed lane 0 hold
// the tree's values on the way, which is all the result needs.
__device__ __forceinline__ float tree32_sum(float v) {
    float low, high;
    swap_rows<16>(v, low, high);
    v = low + high;                  // lanes 0..15 of the group: v[i] + v[i + 16]
    v = v + dpp32<0x108>(v);         // row_shl:8
    v = v + dpp32<0x104>(v);         // row_shl:4
    v = v + dpp32<0x102>(v);         // row_shl:2
    v = v + dpp32<0x101>(v);         // row_shl:1
    v = dpp32<0x150>(v);             // row_newbcast:0: lane 0 of each row of 16
    swap_rows<16>(v, low, high);     // the lower row's value in both rows of the group
    return low;
}
// Largest value of each group of LANES (32 or 64) lanes, in every lane of the group.
template <int LANES>
__device__ __forceinline__ float group_max(float v) {
    v = fmaxf(v, dpp32<0xB1>(v));    // lane ^ 1
    v = fmaxf(v, dpp32<0x4E>(v));    // lane ^ 2
    v = fmaxf(v, dpp32<0x141>(v));   // mirror inside 8 lanes
    v = fmaxf(v, dpp32<0x140>(v));   // mirror inside 16 lanes
    float low, high;
    swap_rows<16>(v, low, high);
    v = fmaxf(low, high);
    if constexpr (LANES == 64) {
        swap_rows<32>(v, low, high);
        v = fmaxf(low, high);
    }
    return v;
}

constexpr int kTopkSlots = 32;   // experts <= 32 * kTopkSlots

template <int CTRL>
__device__ __forceinline__ long long dpp64(long long v) {
    const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, false);
    const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(v >> 32), CTRL, 0xF, 0xF, false);
    return (static_cast<long long>(hi) << 32) | static_cast<uint32_t>(lo);
}
__device__ __forceinline__ long long max64(long long a, long long b) { return a > b ? a : b; }

// LDS scratch of one lane group of topk_token.
constexpr int kTopkCandidates = 64;
struct TopkScratch {
    unsigned long long candidates[kTopkCandidates];   // (probability bits << 32) | ~expert: larger wins
    int lane_best[64];                                // the best key of every lane
    int selected[32];                                 // probability bits of rank r
    int threshold;                                    // top_k-th largest of lane_best
    int count;                                        // candidates found
};

// One group of LANES lanes per token; lane l owns experts l, l + LANES, ... (SLOTS of them).  The softmax
// denominator is summed in the order of the reference kernels, whose 32 lanes each add experts lane, lane + 32, ...
// and then meet in a shuffle-down tree (mfq/kernels/cuda/moe.cu:1383-1446).  With LANES = 32 that is this layout;
// with LANES = 64 (a whole wave per token: half the instructions per wave, and a wave issues one dependent
// instruction every five cycles or so, which is what a small batch waits for) lane l < 32 fetches the numerators of
// lane l + 32 and adds both sets alternately, which is the same sequence of additions.  Selection works on integer
// keys: the bits of a non-negative probability order like the value, an absent entry is -1, and ties go to the lower
// expert id; that order is total, so how the lanes share the entries does not change the result.
//
// The top_k-th largest of the per-lane maxima is a lower bound of the top_k-th largest entry (at least top_k
// entries reach it), so only entries at or above it can be selected: usually one or two dozen.  They are
// collected in LDS and every one counts the candidates that beat it; its rank is that count.  When more than
// kTopkCandidates entries reach the bound (many equal probabilities, or the large ones crowded into few lanes) the
// group falls back to one selection round per rank: the best of the lane candidates by lane exchanges, and the
// winning lane rescans its entries.  Both give the same ids.
//
// Every lane of a token's wave calls it (the lanes of a wave synchronise among themselves, no block barrier); groups with
// active == false select nothing.  A caller that reads `local_ids` from other waves puts its own barrier in between.
// `local_ids`, when given, also receives the ids (any address space, e.g. LDS).
// The lanes of a token (half a wave or a whole one) exchange data through LDS: the LDS operations of a wave complete
// in program order, so it is enough that the wave waits for its own and the compiler keeps the order.  A block barrier
// here would make every wave of the block wait for every other token's, and for the acknowledgement of its own global
// stores each time.
__device__ __forceinline__ void wave_lds_sync() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
}

template <int SLOTS, int LANES = 32>
__device__ __forceinline__ void topk_token(const void* logits, int dtype, int token, bool active, int experts, int top_k,
                                           int normalize, float norm_floor, float scale, int32_t* ids,
                                           float* weights, int* local_ids, TopkScratch* scratch) {
    static_assert(LANES == 32 || LANES == 64, "a token takes half a wave or a whole one");
    const int lane = threadIdx.x & (LANES - 1);
    const bool busy = __ballot(active) != 0ull;          // waves without a token have nothing to do
    float cached[SLOTS];
    float total = 1.0f;
    int lane_best = -1;
    if (busy) {
        const int64_t base = static_cast<int64_t>(active ? token : 0) * experts;
        // all loads of the lane are issued before the first value is looked at: the type switch sits
        // outside the loops and absent entries read a valid address
        if (dtype == MFQ_AMD_F32) {
            const float* p = static_cast<const float*>(logits) + base;
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot) cached[slot] = p[lane + slot * LANES < experts ? lane + slot * LANES : 0];
        } else {
            const uint16_t* p = static_cast<const uint16_t*>(logits) + base;
            uint16_t raw[SLOTS];
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot) raw[slot] = p[lane + slot * LANES < experts ? lane + slot * LANES : 0];
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot)
                cached[slot] = dtype == MFQ_AMD_F16 ? half_bits_to_float(raw[slot]) : bf16_bits_to_float(raw[slot]);
        }
        float maximum = -__builtin_inff();
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot) {
            const float v = cached[slot];
            cached[slot] = lane + slot * LANES >= experts ? -__builtin_inff() : v != v ? -3.402823466e+38f : v;
            maximum = fmaxf(maximum, cached[slot]);
        }
        maximum = group_max<LANES>(maximum);
        float sum = 0.0f;
        if constexpr (LANES == 32) {
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot) {
                if (lane + slot * 32 < experts) {
                    cached[slot] = routing_expf(cached[slot] - maximum);
                    sum = sum + cached[slot];
                } else {
                    cached[slot] = -1.0f;                     // absent: the bits of a negative number are a negative key
                }
            }
        } else {
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot)
                cached[slot] = lane + slot * 64 < experts ? routing_expf(cached[slot] - maximum) : -1.0f;
            // lane l < 32 adds experts l, l + 32, l + 64, ... in that order: its own entries and those of lane l + 32 in turn
            // (the upper lanes run the same code on values nobody reads)
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot) {
                float own, other;                          // of lane l < 32: its value and that of lane l + 32
                swap_rows<32>(cached[slot], own, other);
                const int first = (lane & 31) + slot * 64;
                if (first < experts) sum = sum + cached[slot];
                if (first + 32 < experts) sum = sum + other;
            }
        }
        total = tree32_sum(sum);
        if constexpr (LANES == 64) total = __uint_as_float(static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(__float_as_uint(total)), 0)));
        // The numerators order like the probabilities (division by the common total is monotone), except that
        // numerators a few units in the last place apart may give the same probability: the bound below is taken
        // on the numerators and lowered by that much, the probabilities themselves are computed for candidates only.
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot) {
            const int bits = active ? static_cast<int>(__float_as_uint(cached[slot])) : -1;
            lane_best = bits > lane_best ? bits : lane_best;
        }
        scratch->lane_best[lane] = lane_best;
        if (lane == 0) { scratch->threshold = 0x7fffffff; scratch->count = 0; }
    }
    wave_lds_sync();
    if (busy) {
        // the top_k-th largest lane maximum: the smallest one that fewer than top_k others exceed
        int greater = 0;
#pragma unroll
        for (int i = 0; i < LANES; i += 4) {
            const int4 v = *reinterpret_cast<const int4*>(&scratch->lane_best[i]);
            greater += (v.x > lane_best) + (v.y > lane_best) + (v.z > lane_best) + (v.w > lane_best);
        }
        if (greater < top_k) atomicMin(&scratch->threshold, lane_best);
    }
    wave_lds_sync();
    if (busy) {
        const int bound = scratch->threshold - 8 > 0 ? scratch->threshold - 8 : 0;
        int mine = 0;
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot) mine += active && static_cast<int>(__float_as_uint(cached[slot])) >= bound;
        int at = mine > 0 ? atomicAdd(&scratch->count, mine) : 0;
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot) {
            const uint32_t bits = __float_as_uint(cached[slot]);
            if (active && static_cast<int>(bits) >= bound) {
                if (at < kTopkCandidates)
                    scratch->candidates[at] = (static_cast<unsigned long long>(bits) << 32) | static_cast<uint32_t>(~(lane + LANES * slot));
                ++at;
            }
        }
    }
    wave_lds_sync();
    const int found = busy ? scratch->count : 0;
    // (numerators below 2^-100 can give subnormal probabilities, where many more numerators share one quotient)
    const bool by_rounds = active && (found > kTopkCandidates || found < top_k || scratch->threshold < 0x0D800000);
    unsigned long long mine2[kTopkCandidates / LANES];
    if (busy && active && !by_rounds) {
        // numerator -> probability, for the candidates only
#pragma unroll
        for (int j = 0; j < kTopkCandidates / LANES; ++j) {
            const int at = lane + LANES * j;
            mine2[j] = 0ull;
            if (at < found) {
                const unsigned long long c = scratch->candidates[at];
                const float probability = __uint_as_float(static_cast<uint32_t>(c >> 32)) / total;
                mine2[j] = (static_cast<unsigned long long>(__float_as_uint(probability)) << 32) | (c & 0xffffffffull);
            }
        }
    }
    wave_lds_sync();
    if (busy && active && !by_rounds) {
#pragma unroll
        for (int j = 0; j < kTopkCandidates / LANES; ++j)
            if (lane + LANES * j < found) scratch->candidates[lane + LANES * j] = mine2[j];
    }
    wave_lds_sync();
    if (busy && active && !by_rounds) {
#pragma unroll
        for (int j = 0; j < kTopkCandidates / LANES; ++j) {
            if (lane + LANES * j >= found) continue;
            const unsigned long long me = mine2[j];
            int rank = 0;
            for (int i = 0; i < found; ++i) rank += scratch->candidates[i] > me;
            if (rank < top_k) {
                const int expert = static_cast<int>(~static_cast<uint32_t>(me));
                ids[static_cast<int64_t>(token) * top_k + rank] = expert;
                if (local_ids != nullptr) local_ids[token * top_k + rank] = expert;
                scratch->selected[rank] = static_cast<int>(me >> 32);
            }
        }
    }
    if (by_rounds) {
        // one selection round per rank on the probabilities of every entry
        int key[SLOTS];
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot)
            key[slot] = lane + slot * LANES < experts ? static_cast<int>(__float_as_uint(cached[slot] / total)) : -1;
        auto local_best = [&](int& best, int& best_slot) {
            best = -1; best_slot = 0;
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot)
                if (key[slot] > best) { best = key[slot]; best_slot = slot; }
        };
        int best, best_slot;
        local_best(best, best_slot);
        for (int rank = 0; rank < top_k; ++rank) {
            // candidate of this lane: (probability bits, ~expert); larger wins
            long long candidate = (static_cast<long long>(best) << 32) | static_cast<uint32_t>(~(lane + LANES * best_slot));
            candidate = max64(candidate, dpp64<0xB1>(candidate));    // lane ^ 1
            candidate = max64(candidate, dpp64<0x4E>(candidate));    // lane ^ 2
            candidate = max64(candidate, dpp64<0x141>(candidate));   // mirror inside 8 lanes
            candidate = max64(candidate, dpp64<0x140>(candidate));   // mirror inside 16 lanes
            candidate = max64(candidate, __shfl_xor(candidate, 16, LANES));
            if constexpr (LANES == 64) candidate = max64(candidate, __shfl_xor(candidate, 32, 64));
            const int expert = static_cast<int>(~static_cast<uint32_t>(candidate));
            const int bits = static_cast<int>(candidate >> 32);
            if (lane == rank) {
                scratch->selected[rank] = bits;
                ids[static_cast<int64_t>(token) * top_k + rank] = expert;
                if (local_ids != nullptr) local_ids[token * top_k + rank] = expert;
            }
            if (lane == (expert & (LANES - 1))) {
                const int taken = expert / LANES;
#pragma unroll
                for (int slot = 0; slot < SLOTS; ++slot)
                    if (slot == taken) key[slot] = -1;
                local_best(best, best_slot);
            }
        }
    }
    wave_lds_sync();
    if (busy) {
        const float selected = active && lane < top_k ? __uint_as_float(static_cast<uint32_t>(scratch->selected[lane])) : 0.0f;
        float denominator = 1.0f;
        if (normalize) denominator = fmaxf(tree32_sum(selected), norm_floor);
        if (active && lane < top_k) {
            const float value = normalize ? selected / denominator : selected;
            weights[static_cast<int64_t>(token) * top_k + lane] = value * scale;
        }
    }
}

template <int SLOTS>
__global__ void __launch_bounds__(64) topk_kernel(const void* logits, int dtype, int tokens, int experts,
                                                  int top_k, int normalize, float norm_floor, float scale,
                                                  int32_t* ids, float* weights) {
    __shared__ TopkScratch scratch[2];
    const int token = blockIdx.x * 2 + (threadIdx.x >> 5);
    topk_token<SLOTS>(logits, dtype, token, token < tokens, experts, top_k, normalize, norm_floor, scale, ids, weights, nullptr,
                      &scratch[threadIdx.x >> 5]);
}

// -------------------------------------------------------- route plan ----
// Inclusive prefix sum over the 64 lanes of a wave with data-parallel-primitive moves (shifts inside rows of 16 lanes,
// then the last lane of a row broadcast to the rows behind it): six adds, no LDS traffic as the lane shuffles have.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);    // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);    // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);    // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);    // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);    // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);    // row_bcast:31 into rows 2 and 3
    return v;
}

// Barrier for data the block exchanges through LDS only: a wave waits for its own LDS operations, not for its global
// stores.  (__syncthreads() is also a fence for global memory: every wave first waits until each of its stores has
// been acknowledged, about a microsecond wherever stores precede it.)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ int block_inclusive_scan(int value, int* wave_totals) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    value = wave_inclusive_scan(value);
    lds_barrier();
    if (lane == 63) wave_totals[wave] = value;
    lds_barrier();
    int prefix = 0;
    for (int w = 0; w < wave; ++w) prefix += wave_totals[w];
    return value + prefix;
}

// Where the blocks of a pair go in a decode launch: pairs whose rows take longest first, so that the last round of
// blocks of a launch is made of the short ones (measured at batch 16, cfg4 formats: 104.6 -> 95.0 us per step).
// Groups by the time one row block takes (all experts in one format, gate+up at batch 16: NINT8 61 us, NVQ 54,
// NINT3 45, NINT4 41, MXFP4 34, NINT2 31); pools the streaming kernel cannot serve come first of all, routed
// pairs whose expert has no pool in the slot (their blocks return at once) sit with the cheapest.
constexpr int kCostGroups = 5;
constexpr int kCostBits = 11;      // at most 1024 pairs per plan of this kernel
__device__ __forceinline__ int cost_group(int word) {
    if (word < 0) return 4;
    if (word & kPoolExactOnly) return 0;
    switch (word & 0xff) {
        case K_NINT_8_48: case K_NVQ_D4: return 1;
        case K_NINT_3_24: return 2;
        case K_NINT_4_24: case K_NINT_4_32: return 3;
        case K_MXFP4: case K_NINT_2_16: return 4;
        default: return 0;
    }
}

// Places the pairs [lo, hi) of one wave: 64 at a time, lanes holding the same expert rank themselves by
// ballot, so the destination runs keep ascending pair order.  next[e] (LDS, private to the wave) is
// the number of pairs of expert e the wave has placed so far, base[e] where the wave's run starts.
__device__ __forceinline__ void place_pairs(const int32_t* ids, int32_t* ids_dst, int E, int lo, int hi, int lane, int* next,
                                            const int* base) {
    // the ids of eight steps are requested together: a step is a dependent chain of ballots, and one round trip
    // per step was most of the time this took
    constexpr int kBatch = 8;
    for (int first0 = lo; first0 < hi; first0 += 64 * kBatch) {
        int loaded[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int p = first0 + 64 * j + lane;
            loaded[j] = p < hi ? ids[p] : -1;
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int first = first0 + 64 * j;
            if (first >= hi) break;
            const int p = first + lane;
            int e = loaded[j];
            if (static_cast<unsigned>(e) >= static_cast<unsigned>(E)) e = -1;
            unsigned long long remaining = __ballot(e >= 0);
            int rank = 0, group = 0;
            while (remaining) {
                const int leader = __ffsll(static_cast<long long>(remaining)) - 1;
                const int le = __shfl(e, leader, 64);
                const unsigned long long same = __ballot(e == le);
                if (e == le) {
                    rank = __popcll(same & ((1ull << lane) - 1ull));
                    group = __popcll(same);
                }
                remaining &= ~same;
            }
            if (e >= 0) ids_dst[base[e] + next[e] + rank] = p;
            __threadfence_block();
            if (e >= 0 && rank == group - 1) next[e] += group;
            __threadfence_block();
        }
    }
}

// Adds the ids of pairs [lo, hi) to the wave's histogram counts[E] (LDS).  The ids of a pass (16 per lane) are all
// requested before the first is counted: one memory round trip per pass instead of one per 64 pairs.
__device__ __forceinline__ void count_ids(const int32_t* ids, int E, int lo, int hi, int lane, int* counts) {
    constexpr int kBatch = 16;
    for (int first = lo; first < hi; first += 64 * kBatch) {
        int loaded[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int p = first + 64 * j + lane;
            loaded[j] = p < hi ? ids[p] : -1;
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
            if (static_cast<unsigned>(loaded[j]) < static_cast<unsigned>(E)) atomicAdd(&counts[loaded[j]], 1);
    }
}

// The contiguous range of pairs wave `wave` of kWaves handles: a multiple of 64 pairs per wave.
__device__ __forceinline__ void wave_range(int pairs, int waves, int wave, int begin, int& lo, int& hi) {
    const int per_wave = ((pairs + waves - 1) / waves + 63) / 64 * 64;
    lo = begin + (wave * per_wave < pairs ? wave * per_wave : pairs);
    hi = lo + per_wave < begin + pairs ? lo + per_wave : begin + pairs;
}

// Work lists of a plan per slot: active experts ordered by (kernel class, expert id), their prefill tiles in the same
// order, the per-pair records where asked for, and the byte and expert totals.  One block of kPlanThreads threads;
// cnt[e], start[e] (LDS) hold the pairs of expert e and where they begin in ids_dst.  scratch [kWaves], wave_items and
// wave_tiles [K_CLASS_COUNT][kWaves], totals [8] are LDS work arrays; lds is the base of the block's dynamic LDS.
// The block builds the lists of slots [slot_lo, slot_hi).  `whole`: these are all the slots of the plan and the block
// stores the totals itself; otherwise the blocks of the other slots run beside it, each adds its bytes to the total
// (zeroed by the kernel in front) and the block of slot 0 stores the expert count.
__device__ __forceinline__ void plan_work_lists(const PlanArgs& a, int* lds, int* cnt, int* start, int* scratch, int* wave_items,
                                                int* wave_tiles, int* totals, int slot_lo, int slot_hi, bool whole) {
    const int E = a.experts;
    constexpr int kWaves = kPlanThreads / 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const PlanExtras& x = a.extras;
    // Work lists per slot: active experts ordered by (kernel class, expert id), and their prefill
    // tiles in the same order.  Ranks come from per-class ballots inside a wave plus a small table
    // of per-(class, wave) totals.
    lds_barrier();
    int* total_distinct = totals;
    unsigned long long* total_bytes = reinterpret_cast<unsigned long long*>(
        lds + ((totals + 2 - lds + 1) & ~1));                 // 8-byte aligned slot behind the counters
    const bool active = tid < E && cnt[tid] > 0;
    const int my_tiles = active ? (cnt[tid] + x.prefill_tile_m - 1) / x.prefill_tile_m : 0;
    if (tid == 0) { *total_bytes = 0ull; *total_distinct = 0; }
    unsigned long long my_bytes = 0ull;
    for (int s = slot_lo; s < slot_hi; ++s) {
        lds_barrier();
        int my_pool = -1;
        ExpertInfo info{-1, 0, -1, 0, 0};
        if (tid < E) {
            if (x.expert_info != nullptr) {
                info = x.expert_info[s * E + tid];
                my_pool = info.pool;
            } else {
                for (int j = x.slot_pool_begin[s]; j < x.slot_pool_begin[s + 1]; ++j) {
                    const int32_t* local = x.pools[j].expert_local;
                    if (local == nullptr || local[tid] >= 0) { my_pool = j; break; }
                }
                x.expert_pool[s * E + tid] = my_pool;
            }
        }
        const int my_class_word = !(active && my_pool >= 0) ? -1 : x.expert_info != nullptr ? info.cls : x.pool_class[my_pool];
        const int my_class = my_class_word >= 0 ? (my_class_word & 0xff) : -1;
        if (my_class >= 0)
            my_bytes += static_cast<unsigned long long>(x.expert_info != nullptr ? info.bytes : x.pool_bytes[my_pool]);
        int my_rank = 0, my_tile_rank = 0;
        for (int c = 0; c < K_CLASS_COUNT; ++c) {
            const bool flag = my_class == c;
            const unsigned long long mask = __ballot(flag);
            const int scan = wave_inclusive_scan(flag ? my_tiles : 0);
            if (flag) {
                my_rank = __popcll(mask & ((1ull << lane) - 1ull));
                my_tile_rank = scan - my_tiles;
            }
            const int wave_total = __builtin_amdgcn_readlane(scan, 63);
            if (lane == 0) { wave_items[c * kWaves + wave] = __popcll(mask); wave_tiles[c * kWaves + wave] = wave_total; }
        }
        lds_barrier();
        {
            // exclusive prefix over the (class, wave) cells in class-major order, as two block scans
            constexpr int kCells = K_CLASS_COUNT * kWaves;
            static_assert(kCells <= kPlanThreads, "one thread per (class, wave) cell");
            const int n = tid < kCells ? wave_items[tid] : 0, t = tid < kCells ? wave_tiles[tid] : 0;
            const int items_through = block_inclusive_scan(n, scratch);
            const int tiles_through = block_inclusive_scan(t, scratch);
            if (tid < kCells) {
                wave_items[tid] = items_through - n;
                wave_tiles[tid] = tiles_through - t;
                if (tid % kWaves == 0) {
                    x.class_offsets[s * kClassSlots + tid / kWaves] = items_through - n;
                    x.tile_offsets[s * kClassSlots + tid / kWaves] = tiles_through - t;
                }
                if (tid == kCells - 1) {
                    x.class_offsets[s * kClassSlots + K_CLASS_COUNT] = items_through;
                    x.tile_offsets[s * kClassSlots + K_CLASS_COUNT] = tiles_through;
                }
            }
        }
        lds_barrier();
        if (my_class >= 0) {
            const int at = s * E + wave_items[my_class * kWaves + wave] + my_rank;
            x.items[at] = tid;
            int local = 0;
            if (x.expert_info != nullptr) local = info.local;
            else if (x.pools[my_pool].expert_local != nullptr) local = x.pools[my_pool].expert_local[tid];
            PlanItem item{};
            item.expert = tid; item.pool = my_pool; item.local = local;
            item.begin = start[tid]; item.count = cnt[tid]; item.cls = my_class_word;
            x.item_info[at] = item;
            const int first = wave_tiles[my_class * kWaves + wave] + my_tile_rank;
            for (int m = 0; m < my_tiles; ++m)
                if (first + m < x.tile_capacity) x.tile_items[s * x.tile_capacity + first + m] = tid | (m << 16);
        }
    }
    if (active) {
        atomicAdd(total_bytes, my_bytes);
        atomicAdd(total_distinct, 1);
    }
    // per-pair records in ids_dst order; this block wrote ids_dst and expert_pool itself
    __threadfence_block();
    __syncthreads();
    if (x.pair_items != nullptr) {
        const int routed = start[E - 1] + cnt[E - 1];
        for (int j = tid; j < a.pairs; j += kPlanThreads) {
            const int p = j < routed ? a.ids_dst[j] : -1;
            const int e = p >= 0 ? a.ids[p] : 0;
            for (int s = 0; s < x.slots; ++s) {
                PairItem item{-1, 0, 0, -1};
                if (p >= 0 && x.expert_info != nullptr) {
                    const ExpertInfo info = x.expert_info[s * E + e];
                    if (info.pool >= 0) item = PairItem{p, info.pool, info.local, info.cls};
                } else if (p >= 0) {
                    const int pool = x.expert_pool[s * E + e];
                    if (pool >= 0) {
                        const int local = x.pools[pool].expert_local != nullptr ? x.pools[pool].expert_local[e] : 0;
                        item = PairItem{p, pool, local, x.pool_class[pool]};
                    }
                }
                x.pair_items[static_cast<int64_t>(s) * a.pairs + j] = item;
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        if (whole) {
            *x.touched_bytes = static_cast<int64_t>(*total_bytes);
            *x.distinct = *total_distinct;
        } else {
            atomicAdd(reinterpret_cast<unsigned long long*>(x.touched_bytes), *total_bytes);
            if (slot_lo == 0) *x.distinct = *total_distinct;
        }
    }
}

// Second kernel of a large plan: block b places the pairs of wave range b of route_plan_kernel, split
// again over its own waves; wave_base[b][e] (written by route_plan_kernel) is where the block's run of
// expert e starts.
__global__ void __launch_bounds__(kPlanThreads) route_scatter_kernel(PlanArgs a) {
    extern __shared__ int lds[];
    const int E = a.experts;
    constexpr int kWaves = kPlanThreads / 64;
    int* hist = lds;                    // [kWaves][E]: counts, then pairs placed so far
    int* base = hist + kWaves * E;      // [kWaves][E]: start of the run of (wave, expert)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (blockIdx.x >= kWaves) {
        // the blocks behind the placing ones: the work lists of one slot each, from the counts and bounds route_plan_kernel left
        const int slot = blockIdx.x - kWaves;
        int* cnt = lds;
        int* start = cnt + E;
        int* scratch = start + E;
        int* wave_items = scratch + kWaves;
        int* wave_tiles = wave_items + K_CLASS_COUNT * kWaves;
        int* totals = wave_tiles + K_CLASS_COUNT * kWaves;
        if (tid < E) { cnt[tid] = a.counts[tid]; start[tid] = a.expert_bounds[tid]; }
        if (slot >= a.lists_in_scatter) {
            // spare blocks: the part of the activation copies that route_plan_kernel's spare blocks left
            const int64_t item = a.tiles.first_item + static_cast<int64_t>(slot - a.lists_in_scatter) * kPlanThreads + threadIdx.x;
            tile_pack_item(item, a.tiles.src, a.tiles.dtype, a.tiles.rows, a.tiles.width, a.tiles.layouts, a.tiles.dst, a.tiles.layout_stride);
            return;
        }
        plan_work_lists(a, lds, cnt, start, scratch, wave_items, wave_tiles, totals, slot, slot + 1, a.extras.slots == 1);
        return;
    }
    int block_lo, block_hi, lo, hi;
    wave_range(a.pairs, kWaves, blockIdx.x, 0, block_lo, block_hi);
    wave_range(block_hi - block_lo, kWaves, wave, block_lo, lo, hi);
    for (int i = tid; i < kWaves * E; i += kPlanThreads) hist[i] = 0;
    __syncthreads();
    count_ids(a.ids, E, lo, hi, lane, hist + wave * E);
    __syncthreads();
    if (tid < E) {
        int before = a.wave_base[blockIdx.x * E + tid];
        for (int w = 0; w < kWaves; ++w) {
            base[w * E + tid] = before;
            before += hist[w * E + tid];
            hist[w * E + tid] = 0;
        }
    }
    __syncthreads();
    place_pairs(a.ids, a.ids_dst, E, lo, hi, lane, hist + wave * E, base + wave * E);
}

// One block.  Stable counting sort of pairs by expert: per-wave histograms over contiguous pair
// ranges give every (expert, wave) its own destination run, and inside a wave lanes holding the
// same expert rank themselves by ballot, so compact slots keep ascending pair order.
__global__ void __launch_bounds__(kPlanThreads) route_plan_kernel(PlanArgs a) {
    extern __shared__ int lds[];
    if (blockIdx.x > 0 && a.tiles.src != nullptr) {
        // blocks behind the first copy the activations into the pair layouts of the tile kernel while the first builds the plan
        const int64_t item = a.tiles.first_item + static_cast<int64_t>(blockIdx.x - 1) * kPlanThreads + threadIdx.x;
        tile_pack_item(item, a.tiles.src, a.tiles.dtype, a.tiles.rows, a.tiles.width, a.tiles.layouts, a.tiles.dst, a.tiles.layout_stride);
        return;
    }
    if (blockIdx.x > 0) {
        // blocks behind the first pack one activation row each while the first builds the plan
        const int row = blockIdx.x - 1;
        const int element = a.pack.dtype == MFQ_AMD_F32 ? 4 : 2;
        xpack_row(static_cast<const char*>(a.pack.src) + static_cast<int64_t>(row) * a.pack.width * element, a.pack.dtype,
                  a.pack.vector_ok != 0, a.pack.width, a.pack.dst + row * a.pack.stride, reinterpret_cast<float*>(lds));
        return;
    }
    const int E = a.experts;
    constexpr int kWaves = kPlanThreads / 64;
    int* hist = lds;                    // [kWaves][E]
    int* cnt = hist + kWaves * E;       // [E]
    int* start = cnt + E;               // [E]
    int* scratch = start + E;           // [kWaves]
    int* wave_items = scratch + kWaves; // [K_CLASS_COUNT][kWaves]
    int* wave_tiles = wave_items + K_CLASS_COUNT * kWaves;
    int* totals = wave_tiles + K_CLASS_COUNT * kWaves;   // distinct, pad, 64-bit byte total
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    for (int i = tid; i < kWaves * E; i += kPlanThreads) hist[i] = 0;
    lds_barrier();
    int lo, hi;
    wave_range(a.pairs, kWaves, wave, 0, lo, hi);
    count_ids(a.ids, E, lo, hi, lane, hist + wave * E);
    lds_barrier();
    int count = 0;
    if (tid < E) {
        for (int w = 0; w < kWaves; ++w) { const int c = hist[w * E + tid]; hist[w * E + tid] = count; count += c; }
        cnt[tid] = count;
        a.counts[tid] = count;
    }
    const int pair_scan = block_inclusive_scan(tid < E ? count : 0, scratch);
    const int route_tiles = tid < E ? (count + a.tile_m - 1) / a.tile_m : 0;
    const int tile_scan = block_inclusive_scan(route_tiles, scratch);
    const bool want_route_tiles = a.tile_bounds != nullptr && a.tile_experts != nullptr;
    if (tid < E) {
        start[tid] = pair_scan - count;
        a.expert_bounds[tid + 1] = pair_scan;
        if (want_route_tiles) {
            a.tile_bounds[tid + 1] = tile_scan;
            for (int t = tile_scan - route_tiles; t < tile_scan; ++t) a.tile_experts[t] = tid;
        }
    }
    if (tid == 0) { a.expert_bounds[0] = 0; if (want_route_tiles) a.tile_bounds[0] = 0; }
    lds_barrier();

    if (a.wave_base != nullptr) {
        // the pairs are placed by route_scatter_kernel, one block per wave range of this kernel
        if (tid < E)
            for (int w = 0; w < kWaves; ++w) a.wave_base[w * E + tid] = start[tid] + hist[w * E + tid];
    } else {
        place_pairs(a.ids, a.ids_dst, E, lo, hi, lane, hist + wave * E, start);
    }

    const PlanExtras& x = a.extras;
    if (x.items == nullptr) return;
    if (a.wave_base != nullptr && a.lists_in_scatter) {
        // the blocks behind route_scatter_kernel's build them meanwhile, one per slot, and add up the byte total
        if (tid == 0 && x.slots > 1) *x.touched_bytes = 0;
        return;
    }
    plan_work_lists(a, lds, cnt, start, scratch, wave_items, wave_tiles, totals, 0, x.slots, true);
}

// The same plan for at most kPlanThreads pairs (decode): one thread per pair and per expert, no
// per-wave histograms.  A pair's rank inside its expert is the number of earlier pairs of the same
// expert.  With at most 64 tokens whose routes name distinct experts (what top-k produces) that is
// a population count over a per-expert token bitmap; otherwise every pair counts against a copy of
// the ids in LDS.  Work lists per (slot, class) are built only when `want_items` asks for them;
// prefill tile lists are never produced here.
// TOPK_SLOTS > 0: the ids are not given but selected here first, from router logits of at most
// kPlanThreads / 32 tokens and 32 * TOPK_SLOTS experts (one 32-lane group per token), and written out
// together with the route weights.
template <int TOPK_SLOTS>
__global__ void __launch_bounds__(kPlanThreads) route_plan_small_kernel(PlanArgs a) {
    __shared__ __align__(16) int expert_of[kPlanThreads];
    __shared__ unsigned long long token_mask[kPlanMaxExperts];
    __shared__ int cnt[kPlanMaxExperts], start[kPlanMaxExperts];
    __shared__ int class_of[kSlots][kPlanMaxExperts], rank_of[kSlots][kPlanMaxExperts], pool_of[kSlots][kPlanMaxExperts];
    __shared__ int local_of[kSlots][kPlanMaxExperts], word_of[kSlots][kPlanMaxExperts];
    __shared__ int class_total[kSlots][K_CLASS_COUNT + 1];
    __shared__ int scratch[kPlanThreads / 64];
    __shared__ int pair_at[kPlanThreads];                                   // pair at a position of ids_dst
    __shared__ unsigned long long group_counts[kSlots][kPlanThreads / 64];  // per wave of positions: pairs per cost group
    __shared__ unsigned long long total_bytes;
    __shared__ int total_distinct, repeated;
    __shared__ TopkScratch topk_scratch[TOPK_SLOTS > 0 ? kPlanThreads / 32 : 1];
    if (blockIdx.x > 0) {
        const int row = blockIdx.x - 1;
        const int element = a.pack.dtype == MFQ_AMD_F32 ? 4 : 2;
        xpack_row(static_cast<const char*>(a.pack.src) + static_cast<int64_t>(row) * a.pack.width * element, a.pack.dtype,
                  a.pack.vector_ok != 0, a.pack.width, a.pack.dst + row * a.pack.stride, reinterpret_cast<float*>(scratch));
        return;
    }
    const int E = a.experts, P = a.pairs;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int kWaves = kPlanThreads / 64;
    const PlanExtras& x = a.extras;

    // issued first, consumed last: the per-expert records of every slot
    ExpertInfo info[kSlots];
#pragma unroll
    for (int s = 0; s < kSlots; ++s)
        info[s] = x.items != nullptr && x.expert_info != nullptr && s < x.slots && tid < E ? x.expert_info[s * E + tid]
                                                                                                       : ExpertInfo{-1, 0, -1, 0, 0};
    int expert = -1;
    if (TOPK_SLOTS > 0) {
        expert_of[tid] = -1;
        __syncthreads();
        // a whole wave per token while the block has a wave for each (sixteen), half a wave beyond that
        if (a.route.tokens <= kPlanThreads / 64) {
            const int token = tid >> 6;
            topk_token<(TOPK_SLOTS >= 2 ? TOPK_SLOTS / 2 : 1), 64>(a.route.logits, a.route.dtype, token, token < a.route.tokens, E, a.top_k,
                                                                   a.route.normalize, a.route.norm_floor, a.route.scale, a.route.ids_out,
                                                                   a.route.weights_out, expert_of, &topk_scratch[token]);
        } else {
            const int token = tid >> 5;
            topk_token<(TOPK_SLOTS > 0 ? TOPK_SLOTS : 1)>(a.route.logits, a.route.dtype, token, token < a.route.tokens, E, a.top_k,
                                                          a.route.normalize, a.route.norm_floor, a.route.scale, a.route.ids_out,
                                                          a.route.weights_out, expert_of, &topk_scratch[token]);
        }
        __syncthreads();
        expert = expert_of[tid];
    } else {
        if (tid < P) { expert = a.ids[tid]; if (static_cast<unsigned>(expert) >= static_cast<unsigned>(E)) expert = -1; }
        expert_of[tid] = expert;
    }
    if (tid < E) { cnt[tid] = 0; token_mask[tid] = 0ull; }
    if (tid == 0) { total_bytes = 0ull; total_distinct = 0; repeated = 0; }
    __syncthreads();
    const int k = a.top_k;
    const bool bitmap = k > 0 && P <= 64 * k;
    const int token = bitmap ? tid / k : 0;
    if (expert >= 0) {
        atomicAdd(&cnt[expert], 1);
        if (bitmap) {
            atomicOr(&token_mask[expert], 1ull << token);
            for (int q = token * k; q < tid; ++q)
                if (expert_of[q] == expert) repeated = 1;      // a token naming an expert twice
        }
    }
    __syncthreads();
    int rank = 0;
    if (bitmap && !repeated) {
        if (expert >= 0) rank = __popcll(token_mask[expert] & ((1ull << token) - 1ull));
    } else if (wave * 64 < P) {
        // the wave scans the ids up to its own last pair, four per read
        const int limit = wave * 64 + 64 < P ? wave * 64 + 64 : P;
        for (int q = 0; q < limit; q += 4) {
            const int4 v = *reinterpret_cast<const int4*>(&expert_of[q]);
            rank += (v.x == expert && q < tid) + (v.y == expert && q + 1 < tid) + (v.z == expert && q + 2 < tid) +
                    (v.w == expert && q + 3 < tid);
        }
    }
    const int count = tid < E ? cnt[tid] : 0;
    if (tid < E) a.counts[tid] = count;
    const int pair_scan = block_inclusive_scan(count, scratch);
    if (tid < E) {
        start[tid] = pair_scan - count;
        a.expert_bounds[tid + 1] = pair_scan;
    }
    if (tid == 0) a.expert_bounds[0] = 0;
    if (a.tile_bounds != nullptr && a.tile_experts != nullptr) {
        const int route_tiles = tid < E ? (count + a.tile_m - 1) / a.tile_m : 0;
        const int tile_scan = block_inclusive_scan(route_tiles, scratch);
        if (tid < E) {
            a.tile_bounds[tid + 1] = tile_scan;
            for (int t = tile_scan - route_tiles; t < tile_scan; ++t) a.tile_experts[t] = tid;
        }
        if (tid == 0) a.tile_bounds[0] = 0;
    }
    __syncthreads();
    const int destination = expert >= 0 ? start[expert] + rank : -1;
    if (expert >= 0) { a.ids_dst[destination] = tid; pair_at[destination] = tid; }

    if (x.items == nullptr) return;
    const bool active = tid < E && count > 0;
    unsigned long long my_bytes = 0ull;
    int my_pool[kSlots], my_word[kSlots], my_local[kSlots];
    if (x.expert_info != nullptr) {
#pragma unroll
        for (int s = 0; s < kSlots; ++s) {
            my_pool[s] = info[s].pool;
            my_local[s] = info[s].local;
            my_word[s] = active && info[s].pool >= 0 ? info[s].cls : -1;
            if (my_word[s] >= 0) my_bytes += static_cast<unsigned long long>(info[s].bytes);
        }
    } else {
        for (int s = 0; s < kSlots; ++s) {
            int pool = -1, local = 0;
            if (tid < E && s < x.slots) {
                for (int j = x.slot_pool_begin[s]; j < x.slot_pool_begin[s + 1]; ++j) {
                    const int32_t* map = x.pools[j].expert_local;
                    if (map == nullptr || map[tid] >= 0) { pool = j; local = map != nullptr ? map[tid] : 0; break; }
                }
                x.expert_pool[s * E + tid] = pool;
            }
            my_pool[s] = pool;
            my_local[s] = local;
            my_word[s] = active && pool >= 0 ? x.pool_class[pool] : -1;
            if (my_word[s] >= 0) my_bytes += static_cast<unsigned long long>(x.pool_bytes[pool]);
        }
    }
    for (int s = 0; s < x.slots; ++s) {
        if (tid < E) {
            class_of[s][tid] = my_word[s] >= 0 ? (my_word[s] & 0xff) : -1;
            pool_of[s][tid] = my_pool[s];
            local_of[s][tid] = my_local[s];
            word_of[s][tid] = my_word[s];
        }
    }
    if (active) {
        atomicAdd(&total_bytes, my_bytes);
        atomicAdd(&total_distinct, 1);
    }
    __syncthreads();
    if (x.want_items) {
        // one wave per (slot, class): ranks of the class's active experts in ascending id order
        for (int combo = wave; combo < x.slots * K_CLASS_COUNT; combo += kWaves) {
            const int s = combo / K_CLASS_COUNT, c = combo % K_CLASS_COUNT;
            int before = 0;
            for (int e0 = 0; e0 < E; e0 += 64) {
                const int e = e0 + lane;
                const bool flag = e < E && class_of[s][e] == c;
                const unsigned long long mask = __ballot(flag);
                if (flag) rank_of[s][e] = before + __popcll(mask & ((1ull << lane) - 1ull));
                before += __popcll(mask);
            }
            if (lane == 0) class_total[s][c] = before;
        }
        __syncthreads();
            if (tid < x.slots * kClassSlots) {
            const int s = tid / kClassSlots, c = tid % kClassSlots;
            int before = 0;
            for (int q = 0; q < c; ++q) before += class_total[s][q];
            x.class_offsets[s * kClassSlots + c] = before;
            x.tile_offsets[s * kClassSlots + c] = 0;
        }
        for (int s = 0; s < x.slots; ++s) {
            if (my_word[s] < 0) continue;
            const int cls = my_word[s] & 0xff;
            int at = rank_of[s][tid];
            for (int q = 0; q < cls; ++q) at += class_total[s][q];
            at += s * E;
            x.items[at] = tid;
            PlanItem item{};
            item.expert = tid; item.pool = my_pool[s]; item.local = my_local[s];
            item.begin = start[tid]; item.count = count; item.cls = my_word[s];
            x.item_info[at] = item;
        }
    }
    if (x.pair_items != nullptr) {
        // Per slot the pairs are listed by cost group, inside a group in ids_dst order (pairs of one expert stay
        // adjacent, so its weights leave HBM once).  Thread i takes position i of ids_dst: ballots rank it among the
        // positions of its wave, a small table of per-wave counts (one bit field per group) gives the rest.
        const int routed = start[E - 1] + cnt[E - 1];
        const bool placed = tid < routed;
        const int pair = placed ? pair_at[tid] : 0;
        const int owner = placed ? expert_of[pair] : 0;
        int group[kSlots], below[kSlots];   // indexed by unrolled loops only, so that they stay in registers
#pragma unroll
        for (int s = 0; s < kSlots; ++s) {
            group[s] = below[s] = 0;
            if (s >= x.slots) continue;
            group[s] = placed ? cost_group(word_of[s][owner]) : kCostGroups;
            if (wave * 64 >= routed) continue;          // no position of this wave is taken (uniform per wave)
            unsigned long long counts = 0ull;
#pragma unroll
            for (int g = 0; g < kCostGroups; ++g) {
                const unsigned long long mask = __ballot(group[s] == g);
                counts |= static_cast<unsigned long long>(__popcll(mask)) << (kCostBits * g);
                if (group[s] == g) below[s] = __popcll(mask & ((1ull << lane) - 1ull));
            }
            if (lane == 0) group_counts[s][wave] = counts;
        }
        __syncthreads();
        if (placed) {
            const int used = (routed + 63) / 64;
#pragma unroll
            for (int s = 0; s < kSlots; ++s) {
                if (s >= x.slots) continue;
                unsigned long long before = 0ull, all = 0ull;
                for (int w = 0; w < used; ++w) {
                    const unsigned long long c = group_counts[s][w];
                    if (w < wave) before += c;
                    all += c;
                }
                int j = below[s] + static_cast<int>((before >> (kCostBits * group[s])) & ((1u << kCostBits) - 1u));
#pragma unroll
                for (int g = 0; g < kCostGroups - 1; ++g)
                    j += g < group[s] ? static_cast<int>((all >> (kCostBits * g)) & ((1u << kCostBits) - 1u)) : 0;
                PairItem item{-1, 0, 0, -1};
                if (word_of[s][owner] >= 0) item = PairItem{pair, pool_of[s][owner], local_of[s][owner], word_of[s][owner]};
                x.pair_items[static_cast<int64_t>(s) * P + j] = item;
            }
        }
        if (tid < P && expert < 0) {
            // unrouted pairs fill the tail, in pair order
            int unrouted_before = 0;
            for (int q = 0; q < tid; ++q) unrouted_before += expert_of[q] < 0;
            for (int s = 0; s < x.slots; ++s)
                x.pair_items[static_cast<int64_t>(s) * P + routed + unrouted_before] = PairItem{-1, 0, 0, -1};
        }
    }
    if (tid == 0) { *x.touched_bytes = static_cast<int64_t>(total_bytes); *x.distinct = total_distinct; }
}

// The plan of a streaming decode step: nothing but the per-slot pair lists, costliest group first and inside a
// group by expert (pairs of one expert adjacent, so its weights leave HBM once), then by pair.  That order is a
// total order on a 23-bit key per (slot, pair), so a pair's position is the number of smaller keys: every
// (slot, pair) counts them against the keys in LDS, split over `parts` neighbouring lanes when threads are to spare.
// No histograms, scans or per-expert lists; one barrier after the keys are written.
// TOPK_SLOTS > 0: the ids are selected here first from router logits, as in route_plan_small_kernel.
template <int TOPK_SLOTS>
__global__ void __launch_bounds__(kPlanThreads) route_plan_pairs_kernel(PlanArgs a) {
    __shared__ __align__(16) uint32_t keys[kSlots][kPlanSortPairs];
    __shared__ __align__(16) int4 records[kSlots][kPlanSortPairs];      // PairItem of (slot, pair)
    __shared__ int expert_of[kPlanThreads];
    __shared__ uint32_t expert_words[kSlots][kPlanMaxExperts];
    __shared__ float pack_scratch[kPlanThreads / 64];
    __shared__ TopkScratch topk_scratch[TOPK_SLOTS > 0 ? kPlanThreads / 32 : 1];
    if (blockIdx.x > 0) {
        const int row = blockIdx.x - 1;
        const int element = a.pack.dtype == MFQ_AMD_F32 ? 4 : 2;
        xpack_row(static_cast<const char*>(a.pack.src) + static_cast<int64_t>(row) * a.pack.width * element, a.pack.dtype,
                  a.pack.vector_ok != 0, a.pack.width, a.pack.dst + row * a.pack.stride, pack_scratch);
        return;
    }
    const int E = a.experts, P = a.pairs;
    const int tid = threadIdx.x;
    const PlanExtras& x = a.extras;
    // the per-expert records of every slot, requested first and parked in LDS once the routes are known
    uint32_t words[kSlots];
#pragma unroll
    for (int s = 0; s < kSlots; ++s) words[s] = s < x.slots && tid < E ? x.expert_words[s * E + tid] : kExpertAbsent;
    if (TOPK_SLOTS > 0) {
        // a whole wave per token while the block has a wave for each (sixteen), half a wave beyond that
        if (a.route.tokens <= kPlanThreads / 64) {
            const int token = tid >> 6;
            topk_token<(TOPK_SLOTS >= 2 ? TOPK_SLOTS / 2 : 1), 64>(a.route.logits, a.route.dtype, token, token < a.route.tokens, E, a.top_k,
                                                                   a.route.normalize, a.route.norm_floor, a.route.scale, a.route.ids_out,
                                                                   a.route.weights_out, expert_of, &topk_scratch[token]);
        } else {
            const int token = tid >> 5;
            topk_token<(TOPK_SLOTS > 0 ? TOPK_SLOTS : 1)>(a.route.logits, a.route.dtype, token, token < a.route.tokens, E, a.top_k,
                                                          a.route.normalize, a.route.norm_floor, a.route.scale, a.route.ids_out,
                                                          a.route.weights_out, expert_of, &topk_scratch[token]);
        }
    } else if (tid < P) {
        expert_of[tid] = a.ids[tid];
    }
#pragma unroll
    for (int s = 0; s < kSlots; ++s) expert_words[s][tid] = words[s];
    __syncthreads();
    // keys and records of every (slot, pair)
    const int items = x.slots * P;
    for (int item = tid; item < items; item += kPlanThreads) {
        const int s = item / P, p = item - s * P;
        const int expert = expert_of[p];
        int4 record = {-1, 0, 0, -1};
        int group = 7;                                    // unrouted pairs and experts without a pool: behind everything
        if (static_cast<unsigned>(expert) < static_cast<unsigned>(E)) {
            const uint32_t word = expert_words[s][expert];
            if (word != kExpertAbsent) {
                const int cls = static_cast<int>(word & 0x1ffu);
                record = int4{p, static_cast<int>((word >> 9) & 0x3fu), static_cast<int>((word >> 15) & 0x3ffu), cls};
                group = cost_group(cls);
            }
        }
        records[s][p] = record;
        keys[s][p] = (static_cast<uint32_t>(group) << 20) | (static_cast<uint32_t>(record.x >= 0 ? expert : 0) << 10) |
                     static_cast<uint32_t>(p);
    }
    // keys behind the last pair compare larger than any real one, so that whole vectors can be scanned
    for (int i = tid; i < kSlots * 4; i += kPlanThreads)
        if (P + (i & 3) < kPlanSortPairs) keys[i >> 2][P + (i & 3)] = 0xffffffffu;
    __syncthreads();
    int parts = 1;
    while (parts < 8 && items * parts * 2 <= kPlanThreads) parts *= 2;
    const int chunk = ((P + parts - 1) / parts + 3) & ~3;     // keys per part, a multiple of four
    const int rounds = (items * parts + kPlanThreads - 1) / kPlanThreads;
    for (int round = 0; round < rounds; ++round) {
        const int index = round * kPlanThreads + tid;
        const int item = index / parts, part = index - item * parts;
        const bool live = item < items;
        const int s = live ? item / P : 0, p = live ? item - s * P : 0;
        const uint32_t mine = keys[s][p];
        int smaller = 0;
        const int begin = part * chunk, end = begin + chunk < P ? begin + chunk : P;
        auto below = [mine](const uint4& v) { return (v.x < mine) + (v.y < mine) + (v.z < mine) + (v.w < mine); };
        int q = begin;
        // sixteen keys at a time while they last, their four LDS reads requested together: one read per turn of the loop
        // is one round trip per four keys, and a thread scans up to 128 of them
        for (; q + 16 <= end; q += 16) {
            const uint4* from = reinterpret_cast<const uint4*>(&keys[s][q]);
            const uint4 v0 = from[0], v1 = from[1], v2 = from[2], v3 = from[3];
            smaller += below(v0) + below(v1) + below(v2) + below(v3);
        }
        for (; q < end; q += 4) smaller += below(*reinterpret_cast<const uint4*>(&keys[s][q]));
        // Groups: the pairs of one expert share the key's upper bits and sit next to each other in the order; a pair's
        // place among them and their number are two more counts over the same keys (those below the expert's first
        // possible key and those below the next expert's).  Every kGroupPairs-th pair of an expert opens a group.
        int before_expert = 0, through_expert = 0;
        if (x.group_pairs) {
            const uint32_t first = mine & ~0x3ffu, next = first + 0x400u;
            auto under = [](const uint4& v, uint32_t bound) { return (v.x < bound) + (v.y < bound) + (v.z < bound) + (v.w < bound); };
            for (int g = begin; g < end; g += 4) {
                const uint4 v = *reinterpret_cast<const uint4*>(&keys[s][g]);
                before_expert += under(v, first);
                through_expert += under(v, next);
            }
        }
        // the parts of an item sit in neighbouring lanes (2, 4 or 8 of them): data-parallel moves, no LDS round trip
        auto over_parts = [parts](int v) {
            if (parts > 1) v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);    // lane ^ 1
            if (parts > 2) v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);    // lane ^ 2
            if (parts > 4) v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, false);   // the other quad of eight lanes
            return v;
        };
        smaller = over_parts(smaller);
        if (x.group_pairs) { before_expert = over_parts(before_expert); through_expert = over_parts(through_expert); }
        if (live && part == 0) {
            const int4 record = records[s][p];
            int cls = record.w;
            if (x.group_pairs && cls >= 0) {
                const int place = smaller - before_expert, left = through_expert - smaller;      // left counts this pair
                const int count = place % kGroupPairs == 0 ? (left < kGroupPairs ? left : kGroupPairs) : 0;
                cls |= count << kGroupCountShift;
            }
            x.pair_items[static_cast<int64_t>(s) * P + smaller] = PairItem{record.x, record.y, record.z, cls};
        }
    }
}

// Packed bytes and distinct experts of a routing: a measurement aid, off the step's path.
__global__ void __launch_bounds__(kPlanThreads) touched_bytes_kernel(const int32_t* ids, int pairs, int experts, int slots,
                                                                     const ExpertInfo* expert_info, int64_t* touched_bytes,
                                                                     int32_t* distinct) {
    __shared__ int seen[kPlanMaxExperts];
    __shared__ unsigned long long total_bytes;
    __shared__ int total_distinct;
    const int tid = threadIdx.x;
    if (tid < experts) seen[tid] = 0;
    if (tid == 0) { total_bytes = 0ull; total_distinct = 0; }
    __syncthreads();
    for (int p = tid; p < pairs; p += kPlanThreads) {
        const int e = ids[p];
        if (static_cast<unsigned>(e) < static_cast<unsigned>(experts)) seen[e] = 1;
    }
    __syncthreads();
    if (tid < experts && seen[tid]) {
        unsigned long long bytes = 0ull;
        bool any = false;
        for (int s = 0; s < slots; ++s) {
            const ExpertInfo info = expert_info[s * experts + tid];
            if (info.pool >= 0) { bytes += static_cast<unsigned long long>(info.bytes); any = true; }
        }
        atomicAdd(&total_bytes, bytes);
        (void)any;
        atomicAdd(&total_distinct, 1);
    }
    __syncthreads();
    if (tid == 0) { *touched_bytes = static_cast<int64_t>(total_bytes); *distinct = total_distinct; }
}

}  // namespace dev

void launch_router_logits(const void* x, int x_dtype, const void* router, int router_dtype, int tokens, int experts, int width,
                          float* logits, hipStream_t stream) {
    if (x_dtype != MFQ_AMD_F32 && router_dtype != MFQ_AMD_F32) {
        // products of 16-bit operands are exact: one chain per thread
        const bool aligned = width % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(router) % 16 == 0;
        if (aligned) {
            hipLaunchKernelGGL(dev::router_logits_chain_kernel, dim3((experts + 63) / 64, (tokens + 3) / 4), dim3(256), 0, stream,
                               static_cast<const uint16_t*>(x), x_dtype == MFQ_AMD_F16 ? 1 : 0, static_cast<const uint16_t*>(router),
                               router_dtype == MFQ_AMD_F16 ? 1 : 0, tokens, experts, width, logits);
            check_launch("router_logits_chain_kernel");
            return;
        }
    }
    hipLaunchKernelGGL(dev::router_logits_kernel, dim3((experts + 63) / 64, tokens), dim3(64), 0, stream, x, x_dtype, router,
                       router_dtype, experts, width, logits);
    check_launch("router_logits_kernel");
}

void launch_touched_bytes(const int32_t* ids, int pairs, int experts, int slots, const ExpertInfo* expert_info,
                          int64_t* touched_bytes, int32_t* distinct, hipStream_t stream) {
    MFQ_REQUIRE(experts > 0 && experts <= kPlanMaxExperts && pairs >= 0, "invalid routing geometry");
    hipLaunchKernelGGL(dev::touched_bytes_kernel, dim3(1), dim3(kPlanThreads), 0, stream, ids, pairs, experts, slots, expert_info,
                       touched_bytes, distinct);
    check_launch("touched_bytes_kernel");
}

void raise_routing_limits() {
    MFQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dev::route_plan_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    MFQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dev::route_scatter_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 136 * 1024));
}

void launch_route_plan(const PlanArgs& args, hipStream_t stream) {
    MFQ_REQUIRE(args.experts > 0 && args.experts <= kPlanMaxExperts, "route plan supports 1..1024 experts");
    MFQ_REQUIRE(args.pairs >= 0 && args.tile_m > 0, "invalid route plan geometry");
    const size_t lds = sizeof(int) * (static_cast<size_t>(kPlanThreads / 64) * args.experts + 2 * args.experts +
                                      kPlanThreads / 64 + 2 * dev::K_CLASS_COUNT * (kPlanThreads / 64) + 8);
    if (lds > 64 * 1024) (void)device_state();   // the kernel's dynamic-LDS limit is raised there
    const int pack_rows = args.pack.src != nullptr ? args.pack.rows : 0;
    MFQ_REQUIRE(pack_rows == 0 || (args.pack.width % dev::kLaneColumns == 0 && args.pack.width <= dev::kLaneColumns * kPlanThreads),
                "activation width cannot be packed");
    // decode-sized plans that need no prefill tiles take the one-thread-per-pair kernel
    const bool large = !args.extras.pairs_only && !(args.pairs <= kPlanThreads && (args.extras.items == nullptr || !args.extras.want_tiles));
    MFQ_REQUIRE(args.tiles.src == nullptr || large, "only the large plan kernel copies activations into the tile layouts");
    if (args.extras.pairs_only) {
        MFQ_REQUIRE(args.pairs <= kPlanSortPairs && args.extras.expert_words != nullptr && args.extras.pair_items != nullptr &&
                        !args.extras.want_tiles && !args.extras.want_items && args.extras.slots >= 1 && args.extras.slots <= kSlots,
                    "the pairs-only plan needs resolved expert records and at most 512 pairs");
        const dim3 grid(1 + pack_rows);
        auto launch = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(kPlanThreads), 0, stream, args); };
        if (args.route.logits == nullptr) {
            launch(dev::route_plan_pairs_kernel<0>);
        } else {
            MFQ_REQUIRE(args.route.tokens <= kPlanThreads / 32 && args.route.tokens * args.top_k == args.pairs &&
                        args.top_k >= 1 && args.top_k <= 32 && args.top_k <= args.experts,
                        "fused routing serves at most 32 tokens");
            if (args.experts <= 128) launch(dev::route_plan_pairs_kernel<4>);
            else if (args.experts <= 256) launch(dev::route_plan_pairs_kernel<8>);
            else if (args.experts <= 512) launch(dev::route_plan_pairs_kernel<16>);
            else launch(dev::route_plan_pairs_kernel<32>);
        }
        check_launch("route_plan_pairs_kernel");
        return;
    }
    if (args.pairs <= kPlanThreads && (args.extras.items == nullptr || !args.extras.want_tiles)) {
        const dim3 grid(1 + pack_rows);
        auto launch = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(kPlanThreads), 0, stream, args); };
        if (args.route.logits == nullptr) {
            launch(dev::route_plan_small_kernel<0>);
        } else {
            MFQ_REQUIRE(args.route.tokens <= kPlanThreads / 32 && args.route.tokens * args.top_k == args.pairs &&
                        args.top_k >= 1 && args.top_k <= 32 && args.top_k <= args.experts,
                        "fused routing serves at most 32 tokens");
            if (args.experts <= 128) launch(dev::route_plan_small_kernel<4>);
            else if (args.experts <= 256) launch(dev::route_plan_small_kernel<8>);
            else if (args.experts <= 512) launch(dev::route_plan_small_kernel<16>);
            else launch(dev::route_plan_small_kernel<32>);
        }
        check_launch("route_plan_small_kernel");
        return;
    }
    MFQ_REQUIRE(args.route.logits == nullptr, "fused routing needs a decode-sized plan");
    MFQ_REQUIRE(args.wave_base == nullptr || args.extras.pair_items == nullptr, "per-pair records need the one-kernel plan");
    int spare_blocks = pack_rows;
    int later_blocks = 0;      // of the activation copies, left to the spare blocks of the scatter launch
    if (args.tiles.src != nullptr) {
        MFQ_REQUIRE(pack_rows == 0 && args.tiles.dst != nullptr && args.tiles.width % dev::kLaneColumns == 0 && args.tiles.dtype != MFQ_AMD_F32 &&
                        reinterpret_cast<uintptr_t>(args.tiles.src) % 16 == 0,
                    "activations cannot be copied into the tile layouts by the plan kernel");
        const int64_t items = static_cast<int64_t>(args.tiles.rows) * (args.tiles.width / dev::kLaneColumns);
        spare_blocks = static_cast<int>((items + kPlanThreads - 1) / kPlanThreads);
        // The copies move more bytes than the plan block takes time for (four layouts of 4096 x 2048: 80 MB, 34 us
        // against 21), and the scatter launch leaves most of the chip idle too: it takes half of them.
        if (args.wave_base != nullptr && args.extras.items != nullptr) { later_blocks = spare_blocks / 2; spare_blocks -= later_blocks; }
    }
    // with a scatter launch behind it, the plan kernel stops after the bounds; the work lists are built by more blocks
    // of the scatter launch, one per slot, beside the blocks that place the pairs
    PlanArgs large_args = args;
    large_args.lists_in_scatter = args.wave_base != nullptr && args.extras.items != nullptr ? args.extras.slots : 0;
    large_args.tiles.first_item = 0;
    hipLaunchKernelGGL(dev::route_plan_kernel, dim3(1 + spare_blocks), dim3(kPlanThreads), lds, stream, large_args);
    check_launch("route_plan_kernel");
    if (args.wave_base != nullptr) {
        const size_t place_lds = sizeof(int) * 2 * (kPlanThreads / 64) * args.experts;
        const size_t scatter_lds = place_lds > lds ? place_lds : lds;       // the lists block lays its LDS out as the plan kernel does
        if (scatter_lds > 64 * 1024) (void)device_state();
        large_args.tiles.first_item = static_cast<int64_t>(spare_blocks) * kPlanThreads;
        hipLaunchKernelGGL(dev::route_scatter_kernel, dim3(kPlanThreads / 64 + large_args.lists_in_scatter + later_blocks), dim3(kPlanThreads), scatter_lds,
                           stream, large_args);
        check_launch("route_scatter_kernel");
    }
}

}  // namespace mfq_amd

using namespace mfq_amd;

extern "C" int mfq_amd_router_logits(const void* x_dev, int32_t x_dtype, const void* router_dev, int32_t router_dtype,
                                     int32_t tokens, int32_t experts, int32_t width, float* logits_dev, void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(x_dev && router_dev && logits_dev, "null argument");
        MFQ_REQUIRE(tokens >= 0 && experts > 0 && width > 0, "invalid router geometry");
        MFQ_REQUIRE(x_dtype >= 0 && x_dtype <= 2 && router_dtype >= 0 && router_dtype <= 2, "unknown dtype");
        if (!tokens) return;
        launch_router_logits(x_dev, x_dtype, router_dev, router_dtype, tokens, experts, width, logits_dev, as_stream(stream));
    });
}

extern "C" int mfq_amd_topk(const void* logits_dev, int32_t logits_dtype, int32_t tokens, int32_t experts, int32_t top_k,
                            int32_t normalize, float norm_floor, float scale, int32_t* ids_dev, float* weights_dev,
                            void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(logits_dev && ids_dev && weights_dev, "null argument");
        // same argument rules as moe_topk_cuda (mfq/kernels/cuda/moe.cu:1969-1973)
        MFQ_REQUIRE(tokens > 0 && experts > 0, "logits dimensions must be nonzero");
        MFQ_REQUIRE(top_k >= 1 && top_k <= 32 && top_k <= experts, "top_k must be in [1, min(32, experts)]");
        MFQ_REQUIRE(logits_dtype >= 0 && logits_dtype <= 2, "logits must be float32, float16 or bfloat16");
        if (experts > 32 * dev::kTopkSlots) fail_unsupported("top-k supports at most 1024 experts");
        const dim3 grid((tokens + 1) / 2);
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, grid, dim3(64), 0, as_stream(stream), logits_dev, logits_dtype, tokens, experts,
                               top_k, normalize, norm_floor, scale, ids_dev, weights_dev);
        };
        if (experts <= 128) launch(dev::topk_kernel<4>);
        else if (experts <= 256) launch(dev::topk_kernel<8>);
        else if (experts <= 512) launch(dev::topk_kernel<16>);
        else launch(dev::topk_kernel<32>);
        check_launch("topk_kernel");
    });
}

extern "C" int mfq_amd_route_plan(const int32_t* ids_dev, int32_t tokens, int32_t top_k, int32_t experts, int32_t tile_m,
                                  int32_t* counts_dev, int32_t* expert_bounds_dev, int32_t* tile_bounds_dev,
                                  int32_t* tile_experts_dev, int32_t* ids_dst_dev, void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(ids_dev && counts_dev && expert_bounds_dev && tile_bounds_dev && tile_experts_dev && ids_dst_dev,
                    "null argument");
        MFQ_REQUIRE(tokens >= 0 && top_k > 0, "invalid route geometry");
        PlanArgs args{};
        args.ids = ids_dev; args.pairs = tokens * top_k; args.experts = experts; args.tile_m = tile_m; args.top_k = top_k;
        args.counts = counts_dev; args.expert_bounds = expert_bounds_dev; args.tile_bounds = tile_bounds_dev;
        args.tile_experts = tile_experts_dev; args.ids_dst = ids_dst_dev;
        launch_route_plan(args, as_stream(stream));
    });
}
