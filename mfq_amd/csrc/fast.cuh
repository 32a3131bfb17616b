// Streaming dot products over packed rows: the decode hot path.
//
// A row is cut into lane blocks of 32 consecutive columns.  A lane owns one block (per slab),
// keeps its 32 activations in registers as 16 packed fp16 pairs and, for every row, loads its 32
// packed weights with one wide load, turns them into fp16 pairs with a few integer operations and
// multiplies with v_dot2_f32_f16 (fp16 products, fp32 accumulation).  Nothing is dequantised to
// fp32; the affine terms of a format are applied to per-block sums instead of per weight:
//   NINT   sum_i (S q_i - M) x_i = S (sum_i q_i x_i) - M (sum_i x_i),  S = row_scale*level, M = row_min*level
//          (cpp_runtime/backends/cpu/ops/packed_nint.cpp:77-83 gives the per-weight form)
//   NVQ    (anchor*multiplier[state]) * sum_i (+-codeword_i) x_i        (cuda/ops/vq.cpp:228-246)
//   MXFP4  2^(s-127) * sum_i e2m1_i x_i                                 (cuda/ops/mx.cpp:420-447)
// Integer codes become fp16 without arithmetic: the masked bits of a half are the fp16 denormal q * 2^(p-24)
// for a code at bit p (v_dot2_f32_f16 keeps denormals exactly); the packed activations carry 2^-p and the coded
// sums 2^24.  (The tile kernel instead ORs the code into the mantissa of 1024.0, 0x6400, so that the pair holds
// 1024+q in the normal range its fp16 arithmetic needs.)  Activations are scaled by a
// power of two per token so that the largest magnitude sits in [2^14, 2^15): bf16 and fp16 inputs
// then convert to fp16 without rounding (values 2^-38 below the largest flush to zero) and the
// result is scaled back at the end.  Results differ from the per-weight fp32 form only by
// summation order and fp32 rounding of partial sums.
//
// Geometry served here: width a multiple of 32, NINT pools with one code width whose rows are
// byte-contiguous (uniform_bits), NVQ D4 formats with 4-bit states, MXFP4.  Everything else runs on
// the exact decoders of decode.cuh.
#pragma once

#include "decode.cuh"
#include "fetch_at.h"

#include <type_traits>

namespace mfq_amd {
namespace dev {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x2 __attribute__((aligned(1))) u32x2_u;
typedef u32x3 __attribute__((aligned(1))) u32x3_u;
typedef u32x4 __attribute__((aligned(1))) u32x4_u;
typedef uint16_t __attribute__((aligned(1))) unaligned_u16;

constexpr uint32_t kMagicPair = 0x64006400u;   // two halves of 1024.0

__device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, w), __builtin_bit_cast(half2_t, x), acc, false);
}

// The same product written to a register of its own.  The compiler prefers the two-operand form
// (accumulate in place) and pays a copy wherever the old sum is still needed or the sum starts at
// zero; the three-operand encoding takes the addend from anywhere.
__device__ __forceinline__ float dot2_from(uint32_t w, uint32_t x, float acc) {
    float d;
    asm("v_dot2_f32_f16 %0, %1, %2, %3" : "=v"(d) : "v"(w), "v"(x), "v"(acc));
    return d;
}
__device__ __forceinline__ float dot2_first(uint32_t w, uint32_t x) {
    float d;
    asm("v_dot2_f32_f16 %0, %1, %2, 0" : "=v"(d) : "v"(w), "v"(x));
    return d;
}

__host__ __device__ constexpr bool fast_class(int cls) {
    return (cls >= K_NINT_2_16 && cls <= K_NINT_8_48) || cls == K_NVQ_D4 || cls == K_MXFP4;
}

template <int CLS>
struct FastClass {
    static constexpr bool kNint = CLS >= K_NINT_2_16 && CLS <= K_NINT_8_48;
    static constexpr bool kNvq = CLS == K_NVQ_D4;
    static constexpr bool kMx = CLS == K_MXFP4;
    static constexpr int kBits = CLS == K_NINT_2_16 ? 2 : CLS == K_NINT_3_24 ? 3 : CLS == K_NINT_8_48 ? 8 : 4;
    static constexpr int kGs = CLS == K_NINT_2_16 ? 16 : CLS == K_NINT_4_32 ? 32 : CLS == K_NINT_8_48 ? 48
                               : kMx ? 32 : 24;
    // dwords of codes a lane loads per row: 32 weights of kBits, or 8 NVQ indices of up to 10 bits
    static constexpr int kQ = kNint ? kBits : kNvq ? 3 : 4;
    // row slots a wave keeps in flight (one wide load of codes per lane and slot)
    static constexpr int kRing = ((kNint && kBits == 8) || kNvq) ? 4 : 8;
};

// ------------------------------------------------------------ reductions ----
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
// The lane's value and that of the lane DISTANCE (16 or 32) positions away, in an order that depends on the lane: for
// operations that commute.  One register swap between the rows of the wave, where a shuffle is an LDS round trip.
template <int DISTANCE>
__device__ __forceinline__ void lane_and_partner(float v, float& one, float& other) {
    static_assert(DISTANCE == 16 || DISTANCE == 32, "rows of 16 lanes or halves of 32");
    const unsigned bits = __builtin_bit_cast(unsigned, v);
    const auto swapped = DISTANCE == 16 ? __builtin_amdgcn_permlane16_swap(bits, bits, false, false)
                                        : __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    one = __builtin_bit_cast(float, static_cast<unsigned>(swapped[0]));
    other = __builtin_bit_cast(float, static_cast<unsigned>(swapped[1]));
}
template <int DISTANCE>
__device__ __forceinline__ float add_partner(float v) {
    float one, other;
    lane_and_partner<DISTANCE>(v, one, other);
    return one + other;
}

// Every lane returns the maximum over the wave.
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp<0xB1>(v));
    v = fmaxf(v, dpp<0x4E>(v));
    v = fmaxf(v, dpp<0x141>(v));
    v = fmaxf(v, dpp<0x140>(v));
    float one, other;
    lane_and_partner<16>(v, one, other);
    v = fmaxf(one, other);
    lane_and_partner<32>(v, one, other);
    return fmaxf(one, other);
}

// Sums N per-lane values over the LANES lanes of a row group in a fixed order.  On return the lane
// whose index within the group is l < N holds the total of value reduce_slot<N>(l); other lanes hold
// copies.  The first log2(N) steps halve the number of live values while exchanging with the lane
// one and two (and four) positions away, so N totals cost little more than one.
template <int N>
__device__ __forceinline__ int reduce_slot(int l) {
    if (N == 1) return 0;
    if (N == 2) return l & 1;
    if (N == 4) return 2 * (l & 1) + ((l >> 1) & 1);
    return 4 * (l & 1) + 2 * ((l >> 1) & 1) + ((l >> 2) & 1);
}

template <int N, int LANES>
__device__ __forceinline__ float reduce_values(const float (&v)[N], int lane) {
    static_assert(N == 1 || N == 2 || N == 4, "1, 2 or 4 values");
    float a;
    if (N == 4) {
        const bool odd = lane & 1;
        const float k0 = odd ? v[2] : v[0], k1 = odd ? v[3] : v[1];
        const float s0 = odd ? v[0] : v[2], s1 = odd ? v[1] : v[3];
        const float a0 = k0 + dpp<0xB1>(s0), a1 = k1 + dpp<0xB1>(s1);
        const bool second = lane & 2;
        const float keep = second ? a1 : a0, send = second ? a0 : a1;
        a = keep + dpp<0x4E>(send);
    } else if (N == 2) {
        const bool odd = lane & 1;
        const float keep = odd ? v[1] : v[0], send = odd ? v[0] : v[1];
        a = keep + dpp<0xB1>(send);
        a = a + dpp<0x4E>(a);
    } else {
        a = v[0] + dpp<0xB1>(v[0]);
        a = a + dpp<0x4E>(a);
    }
    a = a + dpp<0x124>(a);   // row_ror:4
    a = a + dpp<0x128>(a);   // row_ror:8
    if (LANES == 64) {
        a = add_partner<16>(a);
        a = add_partner<32>(a);
    }
    return a;
}

// --------------------------------------------------- activations of a lane ----
// 16 fp16 pairs of the lane block, normalised by 2^-e (and by the pair_scale of the weight class), plus the
// plain sum of the activations per quantisation group the block touches (g0: first group, g1: second group).
struct XBlock {
    uint32_t p[16];
    float g0, g1;
};

// Pair k (0..15) of a lane block multiplies columns pair_column(k, 0) and pair_column(k, 1) of the block
// in one dot2.  The layout follows where the codes of the two columns sit in the packed words, so
// that one AND/OR produces both halves of the weight pair:
//   NINT4, NINT3          chunk j = k/4: columns (8j+m, 8j+m+4)         codes m and m+4 of a word
//   NINT8                 chunk j: (0,2) (1,3) (4,6) (5,7)              bytes 0/2 and 1/3 of a dword
//   NINT2                 dword d = k/8: columns (16d+i, 16d+i+8)       codes i and i+8 of a dword
//   NVQ, MXFP4            chunk j: (8j+2m, 8j+2m+1)                     halves of a codebook dword, nibbles of a byte
template <int CLS>
__device__ constexpr int pair_column(int k, int half) {
    if (CLS == K_NINT_2_16) return 16 * (k / 8) + (k % 8) + 8 * half;
    if (CLS == K_NINT_8_48) return 8 * (k / 4) + ((k % 4) < 2 ? (k % 4) : (k % 4) + 2) + 2 * half;
    if (CLS == K_NVQ_D4 || CLS == K_MXFP4) return 8 * (k / 4) + 2 * (k % 4) + half;
    return 8 * (k / 4) + (k % 4) + 4 * half;
}

// A code q OR-ed into the mantissa of a power of two chosen so that the fp16 value is offset+q; codes that
// sit higher in their word use a smaller power.  Zero for formats without offset.
template <int CLS>
__device__ constexpr float magic_offset(int k) {
    if (CLS == K_NINT_2_16) return (k % 4) == 0 ? 1024.0f : (k % 4) == 1 ? 256.0f : (k % 4) == 2 ? 64.0f : 16.0f;
    if (CLS == K_NINT_3_24) return (k % 4) == 0 ? 1024.0f : (k % 4) == 1 ? 128.0f : 16.0f;
    if (CLS == K_NINT_4_24 || CLS == K_NINT_4_32) return (k % 2) == 0 ? 1024.0f : 64.0f;
    if (CLS == K_NINT_8_48) return 1024.0f;
    return 0.0f;
}

// Classes whose codes enter the row loop's dot products as fp16 denormals instead: the masked bits of a
// half are the value q * 2^(p - 24) for a code at bit p, v_dot2_f32_f16 keeps denormal inputs exactly, one AND
// makes a pair and there is no offset to take out again.  The packed activations of such a class carry 2^-p
// per pair (pair_scale) and the coded sums are multiplied by 2^24 at the end of the row.
template <int CLS>
__device__ constexpr bool denormal_codes() {
    return CLS == K_NINT_2_16 || CLS == K_NINT_3_24 || CLS == K_NINT_4_24 || CLS == K_NINT_4_32 || CLS == K_NINT_8_48;
}
template <int CLS>
__device__ constexpr float pair_scale(int k) {
    if (CLS == K_NINT_2_16) return (k % 4) == 0 ? 1.0f : (k % 4) == 1 ? 0.25f : (k % 4) == 2 ? 0.0625f : 0.015625f;
    if (CLS == K_NINT_3_24) return (k % 4) == 0 ? 1.0f : (k % 4) == 1 ? 0.125f : 0.015625f;
    if (CLS == K_NINT_4_24 || CLS == K_NINT_4_32) return (k % 2) == 0 ? 1.0f : 0.0625f;
    return 1.0f;
}

// Scale 2^-e that brings `largest` (>= 0) into [2^14, 2^15), and its inverse.
__device__ __forceinline__ void normaliser(float largest, float& down, float& up) {
    int e = static_cast<int>((__float_as_uint(largest) >> 23) & 0xffu) - 127 - 14;
    e = e < -100 ? -100 : e > 100 ? 100 : e;
    down = __uint_as_float(static_cast<uint32_t>(127 - e) << 23);
    up = __uint_as_float(static_cast<uint32_t>(127 + e) << 23);
}

template <int CLS>
__device__ __forceinline__ void pack_block(const float (&x)[32], float down, const LaneBlock& b, XBlock& out) {
    _Float16 h[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) h[i] = static_cast<_Float16>(b.valid ? x[i] * down : 0.0f);
    float plain[4] = {0.0f, 0.0f, 0.0f, 0.0f};   // per chunk, columns added in ascending order (as xpack_row does)
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        const int first = pair_column<CLS>(k, 0), second = pair_column<CLS>(k, 1);
        half2_t pair;
        pair[0] = static_cast<_Float16>(static_cast<float>(h[first]) * pair_scale<CLS>(k));
        pair[1] = static_cast<_Float16>(static_cast<float>(h[second]) * pair_scale<CLS>(k));
        out.p[k] = __builtin_bit_cast(uint32_t, pair);
    }
#pragma unroll
    for (int i = 0; i < 32; ++i) plain[i / 8] += static_cast<float>(h[i]);
    out.g0 = out.g1 = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const bool second = (b.sel >> j) & 1u;
        out.g0 += second ? 0.0f : plain[j];
        out.g1 += second ? plain[j] : 0.0f;
    }
}

// ------------------------------------------------------- per-class state ----
// Uniform (per block) view of one expert of a pool.
template <int CLS>
struct FastCtx {
    const uint8_t* f0;        // NINT: expert code stream   NVQ: expert index stream   MX: expert nibbles
    const uint8_t* f1;        // NINT: expert scale levels  NVQ: expert sign stream    MX: expert scales
    const uint8_t* f2;        // NINT: expert min levels    NVQ: expert state stream
    const float* f3;          // NINT: expert row scales    NVQ: expert anchors
    const float* f4;          // NINT: expert row minima
    int groups, row_bytes;
    // NVQ: streams are addressed relative to the first byte that holds data of the expert
    int limit0, limit1, limit2;   // bytes of the index / sign / state stream from that byte on (saturated)
    int sign_bit0, state_bit0;   // bit of the expert's first sign mask / state inside its first byte
    int nvec8, nsign4;        // vectors / 8 and sign masks / 4 per row
    int index_bits, entries;
    // LDS tables (NVQ)
    const float* multiplier;  // [16]
    const int* bank_byte;     // [16] byte offset of the state's bank inside `codebook`
    const unsigned char* signs;     // [128] x 16 bytes
    const unsigned char* codebook;  // fp16x4 per entry
};

constexpr int kNvqFastLdsBytes = 64 + 64 + 128 * 16 + 4 * 1024 * 8;

// Builds the per-block LDS tables of an NVQ D4 pool; every thread calls it, then __syncthreads().
__device__ __forceinline__ void nvq_fast_tables(const mfq_amd_projection& p, unsigned char* lds) {
    float* mult = reinterpret_cast<float*>(lds);
    int* bank_byte = reinterpret_cast<int*>(lds + 64);
    uint32_t* signs = reinterpret_cast<uint32_t*>(lds + 128);
    uint32_t* book = reinterpret_cast<uint32_t*>(lds + 128 + 128 * 16);
    const int8_t* meta = static_cast<const int8_t*>(p.fields[4]);
    const bool jsc = nvq_format_jsc(p.format);
    const int entries = nvq_format_entries(p.format);
    const int banks = jsc ? static_cast<uint8_t>(meta[1]) : 1;
    const uint8_t* tables = reinterpret_cast<const uint8_t*>(meta) + (jsc ? 64 : 0);
    // Four entries (16 bytes of the pool's table) per thread and pass, and the loads of up to four passes requested
    // before the first entry is converted: with one entry per pass a block of 256 threads made sixteen dependent
    // round trips for a table of 4096 entries, more than the rows of a down block take to multiply.
    constexpr int kPasses = 4;
    const int total = banks * entries;                 // a multiple of four (256, 512 or 1024 entries per bank)
    for (int first = 0; first < total; first += kPasses * 4 * static_cast<int>(blockDim.x)) {
        u32x4 words[kPasses];
#pragma unroll
        for (int pass = 0; pass < kPasses; ++pass) {
            const int i = first + 4 * (pass * static_cast<int>(blockDim.x) + static_cast<int>(threadIdx.x));
            words[pass] = i < total ? *(const MFQ_GLOBAL u32x4_u*)(tables + 4 * i) : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int pass = 0; pass < kPasses; ++pass) {
            const int i = first + 4 * (pass * static_cast<int>(blockDim.x) + static_cast<int>(threadIdx.x));
            if (i >= total) continue;
            u32x4 out[2];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t word = words[pass][e];
                half2_t lo, hi;
                lo[0] = static_cast<_Float16>(static_cast<float>(word & 0xffu));
                lo[1] = static_cast<_Float16>(static_cast<float>((word >> 8) & 0xffu));
                hi[0] = static_cast<_Float16>(static_cast<float>((word >> 16) & 0xffu));
                hi[1] = static_cast<_Float16>(static_cast<float>(word >> 24));
                out[e / 2][2 * (e % 2)] = __builtin_bit_cast(uint32_t, lo);
                out[e / 2][2 * (e % 2) + 1] = __builtin_bit_cast(uint32_t, hi);
            }
            *reinterpret_cast<u32x4*>(book + 2 * i) = out[0];
            *reinterpret_cast<u32x4*>(book + 2 * i + 4) = out[1];
        }
    }
    if (threadIdx.x < 128) {
        const uint32_t mask7 = threadIdx.x;
        const uint32_t mask8 = mask7 | (parity7(mask7) << 7);
#pragma unroll
        for (int m = 0; m < 4; ++m)
            signs[4 * mask7 + m] = (((mask8 >> (2 * m)) & 1u) << 15) | (((mask8 >> (2 * m + 1)) & 1u) << 31);
    }
    if (threadIdx.x < 16) {
        const int state = threadIdx.x;
        float multiplier;
        int bank = 0;
        if (jsc) {
            uint16_t h;
            __builtin_memcpy(&h, meta + 4 + 2 * state, 2);
            multiplier = half_bits_to_float(h);
            bank = static_cast<uint8_t>(meta[36 + state]);
        } else {
            multiplier = static_cast<float>(state);
        }
        mult[state] = multiplier;
        bank_byte[state] = bank * entries * 8;
    }
}

template <int CLS>
__device__ __forceinline__ FastCtx<CLS> fast_ctx(const mfq_amd_projection& p, int local, unsigned char* lds) {
    using C = FastClass<CLS>;
    FastCtx<CLS> c{};
    const int64_t first_row = static_cast<int64_t>(local) * p.output_rows;
    c.groups = p.groups;
    if constexpr (C::kNint) {
        c.row_bytes = p.groups * (C::kGs * C::kBits / 8);
        c.f0 = static_cast<const uint8_t*>(p.fields[0]) + static_cast<int64_t>(local) * p.q_expert_stride;
        c.f1 = static_cast<const uint8_t*>(p.fields[3]) + first_row * p.groups;
        c.f2 = static_cast<const uint8_t*>(p.fields[4]) + first_row * p.groups;
        c.f3 = static_cast<const float*>(p.fields[5]) + first_row;
        c.f4 = static_cast<const float*>(p.fields[6]) + first_row;
    } else if constexpr (C::kMx) {
        c.row_bytes = p.input_width / 2;
        c.f0 = static_cast<const uint8_t*>(p.fields[0]) + first_row * (p.input_width / 2);
        c.f1 = static_cast<const uint8_t*>(p.fields[1]) + first_row * (p.input_width / 32);
    } else {
        c.index_bits = nvq_format_index_bits(p.format);
        c.entries = nvq_format_entries(p.format);
        c.nvec8 = p.nvec / 8;
        c.nsign4 = p.nsign / 4;
        const NvqExpertAt at = nvq_expert_at(first_row, c.nvec8, c.index_bits, c.nsign4, p.groups, p.sizes[0], p.sizes[1], p.sizes[2]);
        c.f0 = static_cast<const uint8_t*>(p.fields[0]) + at.index_byte;
        c.f1 = static_cast<const uint8_t*>(p.fields[1]) + at.sign_byte;
        c.f2 = static_cast<const uint8_t*>(p.fields[2]) + at.state_byte;
        c.f3 = static_cast<const float*>(p.fields[3]) + first_row;
        c.limit0 = at.limit0; c.limit1 = at.limit1; c.limit2 = at.limit2;
        c.sign_bit0 = at.sign_bit0; c.state_bit0 = at.state_bit0;
        c.multiplier = reinterpret_cast<const float*>(lds);
        c.bank_byte = reinterpret_cast<const int*>(lds + 64);
        c.signs = lds + 128;
        c.codebook = lds + 128 + 128 * 16;
    }
    return c;
}

// Packed data of one lane block of one row.
template <int CLS>
struct FastRaw {
    uint32_t q[FastClass<CLS>::kQ];
    uint32_t a, b, c;     // NINT: scale levels, min levels   NVQ: sign window, -, states   MX: scale byte
};

template <int N>
__device__ __forceinline__ void load_dwords(const uint8_t* p, uint32_t (&out)[N]) {
    if constexpr (N == 2) { const u32x2 v = *(const MFQ_GLOBAL u32x2_u*)p; out[0] = v[0]; out[1] = v[1]; }
    else if constexpr (N == 3) { const u32x3 v = *(const MFQ_GLOBAL u32x3_u*)p; out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; }
    else if constexpr (N == 4) { const u32x4 v = *(const MFQ_GLOBAL u32x4_u*)p; out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; out[3] = v[3]; }
    else if constexpr (N == 8) {
        const u32x4 v = *(const MFQ_GLOBAL u32x4_u*)p;
        const u32x4 w = *(const MFQ_GLOBAL u32x4_u*)(p + 16);
        out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; out[3] = v[3];
        out[4] = w[0]; out[5] = w[1]; out[6] = w[2]; out[7] = w[3];
    }
}

// Issues the loads of (row, lane block); `row` is the row inside the expert.  LEVELS = false leaves
// out the group levels of NINT rows, the block scales of MXFP4 rows and the sign and state streams of NVQ rows
// (for callers that hold them elsewhere).
template <int CLS, bool LEVELS = true>
__device__ __forceinline__ FastRaw<CLS> fast_fetch(const FastCtx<CLS>& c, const LaneBlock& b, int row) {
    using C = FastClass<CLS>;
    FastRaw<CLS> raw{};
    if constexpr (C::kNint) {
        // (the row part of every address is the same in all lanes when a wave works on one row, and then stays in
        // scalar registers)
        const NintFetchAt at = nint_fetch_at(row, c.row_bytes, c.groups, C::kBits, C::kGs, b);
        load_dwords<C::kQ>(c.f0 + at.code_byte, raw.q);
        if constexpr (LEVELS) {
            if constexpr (C::kGs == 32) {
                raw.a = gload<uint8_t>(c.f1 + at.level_byte);
                raw.b = gload<uint8_t>(c.f2 + at.level_byte);
            } else {
                raw.a = *(const MFQ_GLOBAL unaligned_u16*)(c.f1 + at.level_byte);
                raw.b = *(const MFQ_GLOBAL unaligned_u16*)(c.f2 + at.level_byte);
            }
        }
    } else if constexpr (C::kMx) {
        const MxFetchAt at = mx_fetch_at(row, c.row_bytes, b);
        load_dwords<4>(c.f0 + at.code_byte, raw.q);
        if constexpr (LEVELS) raw.a = gload<uint8_t>(c.f1 + at.scale_byte);
    } else {
        const NvqFetchAt at = nvq_fetch_at(row, c.nvec8, c.index_bits, c.nsign4, c.groups, c.limit0, c.limit2, c.sign_bit0,
                                           c.state_bit0, b);
        // eight indices: index_bits bytes, byte aligned because a row holds a multiple of 8 vectors
        const u32x2 lo = *(const MFQ_GLOBAL u32x2_u*)(c.f0 + at.index_byte);
        raw.q[0] = lo[0]; raw.q[1] = lo[1];
        raw.q[2] = load_u32_unaligned(c.f0 + at.third_byte);
        if constexpr (LEVELS) {
            raw.a = load_u32_unaligned(c.f1 + at.sign_byte);     // four 7-bit sign masks
            raw.c = *(const MFQ_GLOBAL unaligned_u16*)(c.f2 + at.state_byte);   // the states of the block's two groups
            // shifts that bring the three loaded words into place; applied when the data is consumed so that
            // nothing here waits for a load
            raw.b = at.shifts;
        } else {
            raw.b = at.shifts & 0xffu;
        }
    }
    return raw;
}

// (a & mask) | bits in one instruction; the constants live in registers.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t bits) {
    uint32_t d;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(mask), "v"(bits));
    return d;
}

// (a & mask) | (b & ~mask) in one instruction.
__device__ __forceinline__ uint32_t bit_select(uint32_t mask, uint32_t a, uint32_t b) {
    uint32_t d;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(d) : "s"(mask), "v"(a), "v"(b));
    return d;
}

// fp16 bit pattern of 2^LOG2, in both halves.  A template constant, not a function of a float: a loop over
// floats is not folded by the compiler, and as a call it ran (ten iterations per use) inside the tile kernel's steps.
template <int LOG2>
constexpr uint32_t kMagicOf = (static_cast<uint32_t>(15 + LOG2) << 10) * 0x00010001u;
static_assert(kMagicOf<10> == 0x64006400u, "1024.0 in both halves");

// The fp16 pairs 4j .. 4j+3 of a lane block (NINT3, NINT4, NINT8, MXFP4): chunk j of the row.
// MAGIC: integer codes as offset + q whatever the class (the tile kernel's form); otherwise as the row loop takes them.
template <int CLS, bool MAGIC = false>
__device__ __forceinline__ void chunk_pairs(const FastRaw<CLS>& raw, int j, uint32_t (&t)[4]) {
    using C = FastClass<CLS>;
    constexpr bool kDenormal = !MAGIC && denormal_codes<CLS>();
    if constexpr (C::kMx) {
        // byte m of the word holds columns 2m and 2m+1; the hardware converts a byte of two E2M1 codes
        // to an fp16 pair (low nibble first)
        const uint32_t w = raw.q[j];
        t[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 0));
        t[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 1));
        t[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 2));
        t[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 3));
    } else if constexpr (C::kBits == 4) {
        // codes m and m+4 sit at bits 4m of the two halves; bits 8..15 come down by one shift
        const uint32_t w = raw.q[j], high = w >> 8;
        if constexpr (kDenormal) {
            t[0] = w & 0x000f000fu; t[1] = w & 0x00f000f0u; t[2] = high & 0x000f000fu; t[3] = high & 0x00f000f0u;
        } else {
            t[0] = and_or(w, 0x000f000fu, kMagicOf<10>);
            t[1] = and_or(w, 0x00f000f0u, kMagicOf<6>);
            t[2] = and_or(high, 0x000f000fu, kMagicOf<10>);
            t[3] = and_or(high, 0x00f000f0u, kMagicOf<6>);
        }
    } else if constexpr (C::kBits == 8) {
        const uint32_t lo = raw.q[2 * j], hi = raw.q[2 * j + 1];
        if constexpr (kDenormal) {
            t[0] = lo & 0x00ff00ffu; t[1] = (lo >> 8) & 0x00ff00ffu; t[2] = hi & 0x00ff00ffu; t[3] = (hi >> 8) & 0x00ff00ffu;
        } else {
            t[0] = and_or(lo, 0x00ff00ffu, kMagicPair);
            t[1] = and_or(lo >> 8, 0x00ff00ffu, kMagicPair);
            t[2] = and_or(hi, 0x00ff00ffu, kMagicPair);
            t[3] = and_or(hi >> 8, 0x00ff00ffu, kMagicPair);
        }
    } else {
        static_assert(C::kBits == 3, "2-bit rows are handled per dword");
        // 24 bits of the chunk, then codes 4..7 (bits 12..23) move to the upper half
        const uint32_t w = j == 0 ? raw.q[0]
                         : j == 1 ? __builtin_amdgcn_alignbit(raw.q[1], raw.q[0], 24)
                         : j == 2 ? __builtin_amdgcn_alignbit(raw.q[2], raw.q[1], 16)
                                  : raw.q[2] >> 8;
        // (one bit-select; left to the compiler the two halves are masked separately and every field below is then
        // formed from both parts: two more instructions per chunk)
        const uint32_t u = bit_select(0xffff0000u, w << 4, w);
        if constexpr (kDenormal) {
            t[0] = u & 0x00070007u; t[1] = u & 0x00380038u; t[2] = u & 0x01c001c0u; t[3] = (u >> 3) & 0x01c001c0u;
        } else {
            t[0] = and_or(u, 0x00070007u, kMagicOf<10>);
            t[1] = and_or(u, 0x00380038u, kMagicOf<7>);
            t[2] = and_or(u, 0x01c001c0u, kMagicOf<4>);
            t[3] = and_or(u >> 3, 0x01c001c0u, kMagicOf<4>);
        }
    }
}

// The eight fp16 pairs of dword d of a 2-bit lane block: codes i and i+8 at bits 2i of the two halves.
__device__ __forceinline__ void dword_pairs_2bit(uint32_t w, uint32_t (&t)[8]) {
    const uint32_t high = w >> 8;
    static_assert(denormal_codes<K_NINT_2_16>(), "the masked bits are the pair");
    t[0] = w & 0x00030003u; t[1] = w & 0x000c000cu; t[2] = w & 0x00300030u; t[3] = w & 0x00c000c0u;
    t[4] = high & 0x00030003u; t[5] = high & 0x000c000cu; t[6] = high & 0x00300030u; t[7] = high & 0x00c000c0u;
}

// Bit field [OFFSET, OFFSET + WIDTH) of v, and (a << SHIFT) + b, each as the one instruction the
// hardware has for it (the compiler rewrites the C forms into shift, mask and add).
template <int OFFSET, int WIDTH>
__device__ __forceinline__ uint32_t bit_field(uint32_t v) {
    uint32_t d;
    asm("v_bfe_u32 %0, %1, %2, %3" : "=v"(d) : "v"(v), "n"(OFFSET), "n"(WIDTH));
    return d;
}
template <int SHIFT>
__device__ __forceinline__ uint32_t shift_add(uint32_t a, uint32_t b) {
    uint32_t d;
    asm("v_lshl_add_u32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "n"(SHIFT), "v"(b));
    return d;
}

// Index K of the eight IB-bit indices in q.
template <int IB, int K>
__device__ __forceinline__ uint32_t nvq_index(const uint32_t (&q)[3]) {
    constexpr int bit = K * IB, word = bit >> 5, shift = bit & 31;
    if constexpr (shift + IB > 32)   // the index straddles two words: funnel shift, then the low IB bits
        return bit_field<0, IB>(__builtin_amdgcn_alignbit(q[word + 1], q[word], shift));
    else
        return bit_field<shift, IB>(q[word]);
}

template <int IB, int NT>
__device__ __forceinline__ void nvq_accumulate(const FastCtx<K_NVQ_D4>& c, const LaneBlock& b, const FastRaw<K_NVQ_D4>& raw,
                                               float anchor, const XBlock (&x)[NT], float (&v)[NT]) {
    const uint32_t states = raw.c >> (raw.b >> 16);
    const uint32_t masks = raw.a >> ((raw.b >> 8) & 0xffu);
    const uint32_t q[3] = {raw.q[0], raw.q[1], raw.q[2] >> (raw.b & 0xffu)};
    const uint32_t state0 = states & 15u, state1 = __builtin_amdgcn_ubfe(states, 4, 4);
    const float scale0 = anchor * c.multiplier[state0], scale1 = anchor * c.multiplier[state1];
    const unsigned char* bank0 = c.codebook + c.bank_byte[state0];
    const unsigned char* bank1 = c.codebook + c.bank_byte[state1];
    // Groups hold 24 columns, so of the block's four chunks the first always belongs to the block's
    // first group and the last to its second (sel is 1000, 1100 or 1110).  One running sum over the
    // chunks; the first group's share is the running sum after its last chunk.
    float run[NT], after[3][NT];
    // LDS byte addresses: codebook entries hold 8 bytes, sign patterns 16
    const uint32_t bank_at[2] = {static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) unsigned char*)bank0)),
                                 static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) unsigned char*)bank1))};
    const uint32_t signs_at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) unsigned char*)c.signs));
    auto chunk = [&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const bool second = j == 0 ? false : j == 3 ? true : ((b.sel >> j) & 1u) != 0;
        const uint32_t bank = second ? bank_at[1] : bank_at[0];
        typedef const __attribute__((address_space(3))) u32x2* lds2;
        typedef const __attribute__((address_space(3))) u32x4* lds4;
        const u32x2 lo = *(lds2)(uintptr_t)shift_add<3>(nvq_index<IB, 2 * j>(q), bank);
        const u32x2 hi = *(lds2)(uintptr_t)shift_add<3>(nvq_index<IB, 2 * j + 1>(q), bank);
        const u32x4 sign = *(lds4)(uintptr_t)shift_add<4>(bit_field<7 * j, 7>(masks), signs_at);
        const uint32_t t[4] = {lo[0] ^ sign[0], lo[1] ^ sign[1], hi[0] ^ sign[2], hi[1] ^ sign[3]};
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            if constexpr (j == 0) run[n] = dot2_first(t[0], x[n].p[0]);
            else run[n] = dot2_from(t[0], x[n].p[4 * j], after[j - 1][n]);
#pragma unroll
            for (int m = 1; m < 4; ++m) run[n] = dot2(t[m], x[n].p[4 * j + m], run[n]);
            if constexpr (j < 3) after[j][n] = run[n];
        }
    };
    chunk(std::integral_constant<int, 0>{});
    chunk(std::integral_constant<int, 1>{});
    chunk(std::integral_constant<int, 2>{});
    chunk(std::integral_constant<int, 3>{});
    const bool from1 = (b.sel & 2u) != 0, from2 = (b.sel & 4u) != 0;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        const float first = from1 ? after[0][n] : from2 ? after[1][n] : after[2][n];
        v[n] = fmaf(scale1, run[n] - first, fmaf(scale0, first, v[n]));
    }
}

// Adds the lane's share of (row . x[n]) to v[n] for every token n.  rs, rm: the row's scale and
// minimum (NINT) or its anchor (NVQ, in rs).
// IB: index bits of an NVQ format when the caller knows them at compile time, 0 = decided here per call.
// ADD = false: v receives the share instead of growing by it (a float add of zero is not free).
template <int CLS, int NT, int IB = 0, bool ADD = true>
__device__ __forceinline__ void fast_accumulate(const FastCtx<CLS>& c, const LaneBlock& b, const FastRaw<CLS>& raw,
                                                float rs, float rm, const XBlock (&x)[NT], float (&v)[NT]) {
    using C = FastClass<CLS>;
    if constexpr (C::kNvq) {
        if constexpr (IB != 0) nvq_accumulate<IB, NT>(c, b, raw, rs, x, v);
        else if (c.index_bits == 10) nvq_accumulate<10, NT>(c, b, raw, rs, x, v);
        else if (c.index_bits == 9) nvq_accumulate<9, NT>(c, b, raw, rs, x, v);
        else nvq_accumulate<8, NT>(c, b, raw, rs, x, v);
    } else if constexpr (C::kMx) {
        float partial[NT];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t t[4];
            chunk_pairs<CLS>(raw, j, t);
#pragma unroll
            for (int n = 0; n < NT; ++n)
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    partial[n] = (j == 0 && m == 0) ? dot2_first(t[0], x[n].p[0]) : dot2(t[m], x[n].p[4 * j + m], partial[n]);
        }
        const float scale = bits_to_float(raw.a ? (raw.a << 23) : 0x00400000u);   // 2^(s-127)
#pragma unroll
        for (int n = 0; n < NT; ++n) v[n] = ADD ? fmaf(scale, partial[n], v[n]) : scale * partial[n];
    } else {
        // the 16-bit level window starts level_shift bits before the block's first level
        const uint32_t scales = C::kGs == 32 ? raw.a : raw.a >> b.level_shift;
        const uint32_t minima = C::kGs == 32 ? raw.b : raw.b >> b.level_shift;
        const float s0 = static_cast<float>(scales & 0xffu), s1 = static_cast<float>((scales >> 8) & 0xffu);
        const float m0 = static_cast<float>(minima & 0xffu), m1 = static_cast<float>((minima >> 8) & 0xffu);
        static_assert(denormal_codes<CLS>(), "the row loop takes every NINT code as an fp16 denormal");
        const float rs_codes = rs * 16777216.0f;    // denormal codes are q * 2^-24
        float coded[NT];   // sum over groups of level * sum q x, times 2^-24
#pragma unroll
        for (int n = 0; n < NT; ++n) coded[n] = 0.0f;
        if constexpr (C::kGs == 32) {
            // one group per lane block
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t t[4];
                chunk_pairs<CLS>(raw, j, t);
#pragma unroll
                for (int n = 0; n < NT; ++n)
#pragma unroll
                    for (int m = 0; m < 4; ++m)
                        coded[n] = (j == 0 && m == 0) ? dot2_first(t[0], x[n].p[0]) : dot2(t[m], x[n].p[4 * j + m], coded[n]);
            }
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const float share = rs_codes * (s0 * coded[n]) - rm * (m0 * x[n].g0);
                v[n] = ADD ? v[n] + share : share;
            }
        } else {
            if constexpr (C::kBits == 2) {
                // a dword holds one 16-column group
#pragma unroll
                for (int d = 0; d < 2; ++d) {
                    uint32_t t[8];
                    dword_pairs_2bit(raw.q[d], t);
#pragma unroll
                    for (int n = 0; n < NT; ++n) {
                        float partial = dot2_first(t[0], x[n].p[8 * d]);
#pragma unroll
                        for (int i = 1; i < 8; ++i) partial = dot2(t[i], x[n].p[8 * d + i], partial);
                        coded[n] = fmaf(d ? s1 : s0, partial, coded[n]);
                    }
                }
            } else {
                // One running sum over the four chunks.  The chunks of the second group are the last ones
                // (sel is 0000, 1000, 1100 or 1110), so the first group's share is the running sum after
                // its last chunk and the second group's share is the rest.
                float run[NT], after[3][NT];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t t[4];
                    chunk_pairs<CLS>(raw, j, t);
#pragma unroll
                    for (int n = 0; n < NT; ++n) {
                        // the first product of a chunk leaves the sum after the previous chunk in place
                        run[n] = j == 0 ? dot2_first(t[0], x[n].p[0]) : dot2_from(t[0], x[n].p[4 * j], after[j - 1][n]);
#pragma unroll
                        for (int m = 1; m < 4; ++m) run[n] = dot2(t[m], x[n].p[4 * j + m], run[n]);
                        if (j < 3) after[j][n] = run[n];
                    }
                }
                const bool from1 = (b.sel & 2u) != 0, from2 = (b.sel & 4u) != 0, from3 = (b.sel & 8u) != 0;
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    const float first = from1 ? after[0][n] : from2 ? after[1][n] : from3 ? after[2][n] : run[n];
                    coded[n] = fmaf(s1, run[n] - first, s0 * first);
                }
            }
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const float minimum = fmaf(m1, x[n].g1, m0 * x[n].g0);
                const float share = rs_codes * coded[n] - rm * minimum;
                v[n] = ADD ? v[n] + share : share;
            }
        }
    }
}

// ------------------------------------------------- weights as fp16 pairs ----
// The same packed data turned into the weights themselves, for the MFMA tile kernel: 16 fp16 pairs
// per lane block in the pair order of pair_column<CLS>, in units of a per-row factor that the caller
// applies to its accumulators (so the fp16 range does not depend on the magnitude of the weights):
//   NINT   w / rs = s q - (rm / rs) m = s (q - c) + (s c - (rm / rs) m),  c = half the code range:
//          q - c is exact in fp16, s is an integer level, one rounding in the fused multiply-add
//   NVQ    w / anchor = multiplier[state] * (+-codeword)
//   MXFP4  w itself: the hardware conversion applies the block scale
template <int CLS>
struct WeightRow {
    float factor;   // multiplies the accumulators of the row
    float coef;     // NINT: 1, or 0 when the row scale is zero (the weights are then -rm m)
    float ratio;    // NINT: rm / factor
};

template <int CLS>
__device__ __forceinline__ WeightRow<CLS> weight_row(const FastCtx<CLS>& c, int row) {
    using C = FastClass<CLS>;
    WeightRow<CLS> r{1.0f, 1.0f, 0.0f};
    if constexpr (C::kNint) {
        const float rs = gload<float>(c.f3 + row), rm = gload<float>(c.f4 + row);
        r.factor = rs != 0.0f ? rs : 1.0f;
        r.coef = rs != 0.0f ? 1.0f : 0.0f;
        r.ratio = rm / r.factor;
    } else if constexpr (C::kNvq) {
        r.factor = gload<float>(c.f3 + row);
    }
    return r;
}

__device__ __forceinline__ half2_t splat_half(float v) {
    const _Float16 h = static_cast<_Float16>(v);
    return half2_t{h, h};
}

// What the chunks of one (row, lane block) share, set up once per block.
template <int CLS>
struct WeightBlock {
    uint32_t sel;                        // bit j: chunk j belongs to the block's second group
    half2_t level[2], shift[2];          // NINT: per group, both halves equal
    half2_t scale[2];                    // NVQ: multiplier of the state of each group
    uint32_t bank_at[2];                 // NVQ: LDS byte address of the codebook bank of each group
    uint32_t signs_at;                   // NVQ: LDS byte address of the sign table
    uint32_t masks;                      // NVQ: the four 7-bit sign masks
    uint32_t q2;                         // NVQ: third index word, aligned
    float block_scale;                   // MXFP4: 2^(s-127)
};

// `scales`, `minima`: NINT: the levels of the block's first group in bits 0..7 and of the next group in bits 8..15;
// NVQ: the block's four sign masks from bit 0, and the states of its two groups from bit 0.
template <int CLS>
__device__ __forceinline__ WeightBlock<CLS> weight_block(const FastCtx<CLS>& c, const LaneBlock& b, const FastRaw<CLS>& raw,
                                                         const WeightRow<CLS>& r, uint32_t scales, uint32_t minima) {
    using C = FastClass<CLS>;
    WeightBlock<CLS> k{};
    k.sel = b.sel;
    if constexpr (C::kNvq) {
        const uint32_t states = minima;
        k.masks = scales;
        k.q2 = raw.q[2] >> (raw.b & 0xffu);
        const uint32_t state0 = states & 15u, state1 = (states >> 4) & 15u;
        k.scale[0] = splat_half(c.multiplier[state0]);
        k.scale[1] = splat_half(c.multiplier[state1]);
        typedef const __attribute__((address_space(3))) unsigned char* lds_bytes;
        k.bank_at[0] = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_bytes)(c.codebook + c.bank_byte[state0])));
        k.bank_at[1] = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_bytes)(c.codebook + c.bank_byte[state1])));
        k.signs_at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_bytes)c.signs));
    } else if constexpr (C::kMx) {
        k.block_scale = bits_to_float(raw.a ? (raw.a << 23) : 0x00400000u);
    } else {
        constexpr float center = static_cast<float>(1 << (C::kBits - 1));
        const float s0 = r.coef * static_cast<float>(scales & 0xffu), s1 = r.coef * static_cast<float>((scales >> 8) & 0xffu);
        const float m0 = static_cast<float>(minima & 0xffu), m1 = static_cast<float>((minima >> 8) & 0xffu);
        k.level[0] = splat_half(s0);
        k.level[1] = splat_half(s1);
        k.shift[0] = splat_half(fmaf(s0, center, -(r.ratio * m0)));
        k.shift[1] = splat_half(fmaf(s1, center, -(r.ratio * m1)));
    }
    return k;
}

// The fp16 weight pairs 4j .. 4j+3 of the block.  IB: index bits of an NVQ format (ignored otherwise).
template <int CLS, int IB>
__device__ __forceinline__ void chunk_weights(const WeightBlock<CLS>& k, const FastRaw<CLS>& raw, int j, uint32_t (&w)[4]) {
    using C = FastClass<CLS>;
    if constexpr (C::kNvq) {
        static_assert(C::kGs == 24, "the first chunk of a lane block lies in its first group, the last in its second");
        const uint32_t q[3] = {raw.q[0], raw.q[1], k.q2};
        // the chunk as a compile-time constant: index fields and LDS addresses each as the one instruction the hardware has
        auto chunk = [&](auto jc) {
            constexpr int J = decltype(jc)::value;
            const bool second = J == 0 ? false : J == 3 ? true : ((k.sel >> J) & 1u) != 0;
            const uint32_t bank = second ? k.bank_at[1] : k.bank_at[0];
            typedef const __attribute__((address_space(3))) u32x2* lds2;
            typedef const __attribute__((address_space(3))) u32x4* lds4;
            const u32x2 lo = *(lds2)(uintptr_t)shift_add<3>(nvq_index<IB, 2 * J>(q), bank);
            const u32x2 hi = *(lds2)(uintptr_t)shift_add<3>(nvq_index<IB, 2 * J + 1>(q), bank);
            const u32x4 sign = *(lds4)(uintptr_t)shift_add<4>(bit_field<7 * J, 7>(k.masks), k.signs_at);
            const uint32_t t[4] = {lo[0] ^ sign[0], lo[1] ^ sign[1], hi[0] ^ sign[2], hi[1] ^ sign[3]};
            const half2_t scale = second ? k.scale[1] : k.scale[0];
#pragma unroll
            for (int m = 0; m < 4; ++m) w[m] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, t[m]) * scale);
        };
        if (j == 0) chunk(std::integral_constant<int, 0>{});
        else if (j == 1) chunk(std::integral_constant<int, 1>{});
        else if (j == 2) chunk(std::integral_constant<int, 2>{});
        else chunk(std::integral_constant<int, 3>{});
    } else if constexpr (C::kMx) {
        w[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(raw.q[j], k.block_scale, 0));
        w[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(raw.q[j], k.block_scale, 1));
        w[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(raw.q[j], k.block_scale, 2));
        w[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(raw.q[j], k.block_scale, 3));
    } else {
        constexpr float center = static_cast<float>(1 << (C::kBits - 1));
        uint32_t t[4];
        if constexpr (C::kBits == 2) {
            // pairs 8d .. 8d+7 come from dword d: chunk j takes the (j % 2)-th four of dword j / 2
            const uint32_t word = raw.q[j / 2], high = word >> 8;
            const uint32_t from = (j % 2) ? high : word;
            t[0] = and_or(from, 0x00030003u, kMagicOf<10>);
            t[1] = and_or(from, 0x000c000cu, kMagicOf<8>);
            t[2] = and_or(from, 0x00300030u, kMagicOf<6>);
            t[3] = and_or(from, 0x00c000c0u, kMagicOf<4>);
        } else {
            chunk_pairs<CLS, true>(raw, j, t);
        }
        // dword j / 2 of a 2-bit block is one group; elsewhere sel flags the chunks of the second group (groups of 24
        // columns: the first chunk of a block always lies in its first group and the last in its second)
        const bool second = C::kGs == 32 ? false : C::kBits == 2 ? j >= 2
                          : (C::kGs == 24 && j == 0) ? false : (C::kGs == 24 && j == 3) ? true : ((k.sel >> j) & 1u) != 0;
        const half2_t level = second ? k.level[1] : k.level[0], shift = second ? k.shift[1] : k.shift[0];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const _Float16 remove = static_cast<_Float16>(-(magic_offset<CLS>(4 * j + m) + center));
            const half2_t code = __builtin_bit_cast(half2_t, t[m]) + half2_t{remove, remove};
            w[m] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(code, level, shift));
        }
    }
}

}  // namespace dev
}  // namespace mfq_amd
