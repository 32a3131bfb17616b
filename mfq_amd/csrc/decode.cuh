// Device-side decoders of the three packed weight families.  A "chunk" is eight
// consecutive columns [8c, 8c+8) of one weight row; every decoder turns one chunk
// into eight fp32 weights that are bit-identical to the reference dequantiser:
//   NINT   w = (row_scale*group_scale)*q - (row_min*group_min)      two roundings, then one more
//          (cpp_runtime/backends/cpu/ops/packed_nint.cpp:77-83)
//   NVQ    w = (anchor*multiplier[state]) * (+-codeword)            (cuda/ops/vq.cpp:228-246, :279-342)
//   MXFP4  w = +-(E2M1 * 2^(s-127))                                 (cuda/ops/mx.cpp:420-447)
// This file is compiled with -ffp-contract=off: a*b-c here is a multiply and a
// subtract; fused operations are written as fmaf().
#pragma once

#include "../../include/mfq_amd.h"
#include "decode_classes.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mfq_amd {
namespace dev {

constexpr int kWave = 64;

// Loads through the global address space (pointers taken from descriptors in memory are generic
// to the compiler, which would otherwise emit slower flat loads).
#define MFQ_GLOBAL __attribute__((address_space(1)))
typedef uint32_t __attribute__((aligned(1))) unaligned_u32;

template <class T>
__device__ __forceinline__ T gload(const void* p) {
    return *(const MFQ_GLOBAL T*)(p);
}
__device__ __forceinline__ uint32_t load_u32_unaligned(const uint8_t* p) {
    return *(const MFQ_GLOBAL unaligned_u32*)(p);
}

// Values that are the same in every lane of the wave, moved to scalar registers.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float uniform(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}
__device__ __forceinline__ int64_t uniform(int64_t v) {
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v & 0xffffffff)));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v >> 32)));
    return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

// n (<= 25) bits starting at absolute bit position `bit`; bits at or beyond byte `size` read as
// zero.  Branch-free: near the end of the stream the 4-byte window slides back inside it and the
// value is shifted down further.  The buffer must be readable for max(size, 4) bytes.
__device__ __forceinline__ uint32_t stream_bits(const uint8_t* base, int64_t size, int64_t bit, int n) {
    const int64_t byte = bit >> 3;
    const int64_t last = size > 4 ? size - 4 : 0;
    const int64_t addr = byte < last ? byte : last;
    const int64_t total = 8 * (byte - addr) + (bit & 7);
    const uint64_t word = load_u32_unaligned(base + addr);
    return static_cast<uint32_t>(word >> (total < 63 ? total : 63)) & ((1u << n) - 1u);
}

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __uint_as_float(u); }

__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return static_cast<float>(__builtin_bit_cast(_Float16, h));
}
__device__ __forceinline__ uint16_t float_to_half_bits(float v) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));   // round to nearest even
}
__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return bits_to_float(static_cast<uint32_t>(b) << 16); }
// half(a * b) with the product rounded to fp32 first, as the reference's __float2half(a * b).  float_to_half_bits(a * b)
// is not that for every input: the compiler fuses the multiply into the conversion as v_fma_mixlo_f16 a, b, +0, and the
// +0 addend turns a product of -0 (a gate of -0.0) into +0.  The empty statement keeps the two apart.
__device__ __forceinline__ uint16_t product_to_half_bits(float a, float b) {
    float product = a * b;
    asm("" : "+v"(product));
    return float_to_half_bits(product);
}

// exp() of the routing softmax and of the shared-expert gate, defined operation by operation so that any IEEE machine
// produces the same bits: n = rint(x*log2e); r = x - n*ln2 in two fma steps; degree-5 Horner
// in fma (Cephes coefficients); r*r folded with one more fma; +1; scaled by 2^n through the
// exponent field.  Inputs below -87 return 0.
__device__ __forceinline__ float routing_expf(float x) {
    // straight-line: the polynomial runs on the argument clamped into its range and the three special results are
    // selected at the end (inside the range the arithmetic, and so every bit, is what the branching form gives)
    const float input = x;
    x = fminf(fmaxf(x, -87.0f), 88.0f);
    const float n = __builtin_rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    const float r2 = r * r;
    p = fmaf(p, r2, r);
    p = p + 1.0f;
    const int ni = static_cast<int>(n);
    float result = p * bits_to_float(static_cast<uint32_t>(ni + 127) << 23);
    result = input < -87.0f ? 0.0f : result;
    result = input > 88.0f ? __builtin_inff() : result;
    return input != input ? input : result;
}

// `limit` value that selects the gate-less expert activation relu(up)^2 in swiglu_bits().
constexpr float kActivationRelu2 = -1.0f;

// One SwiGLU output on fp16 bits.  limit > 0: clipped form in fp32.  limit == 0: `table` maps the bits of a
// half g to half(sigmoid(g)) and every product rounds to fp16, as the reference's fused path does
// (mfq/kernels/cuda/moe.cu:1536-1542).  limit < 0 (kActivationRelu2): half(relu(up)^2), the gate is not read
// (mfq/kernels/cuda/mfe_ffn.h:107-110, expert_activation == 1).
__device__ __forceinline__ uint16_t swiglu_bits(uint16_t gb, uint16_t ub, float limit, const uint16_t* table) {
    const float g = half_bits_to_float(gb), u = half_bits_to_float(ub);
    if (limit < 0.0f) {
        const float positive = fmaxf(u, 0.0f);
        return float_to_half_bits(positive * positive);
    }
    if (limit > 0.0f) {
        const float clipped = fminf(g, limit);
        const float value = fminf(fmaxf(u, -limit), limit);
        return product_to_half_bits(clipped / (1.0f + expf(-clipped)), value);
    }
    const float sigmoid = half_bits_to_float(table[gb]);
    const float first = half_bits_to_float(product_to_half_bits(g, sigmoid));
    return product_to_half_bits(first, u);
}

// ---------------------------------------------------------------- NINT ----
struct NintRow {
    const uint8_t* stream;     // start of the expert's q stream
    int64_t bit_off;           // first code of the row, relative to stream
    const uint8_t* gscale;     // the row's group levels [groups]
    const uint8_t* gmin;
    float rs, rm;
    int bits;
};

// UNIFORM: all lanes of the wave work on the same row, so the row state moves to scalar registers.
template <bool UNIFORM>
__device__ __forceinline__ NintRow nint_row(const mfq_amd_projection& p, int local_expert, int row_in_expert) {
    const int64_t row = static_cast<int64_t>(local_expert) * p.output_rows + row_in_expert;
    NintRow r;
    r.stream = static_cast<const uint8_t*>(p.fields[0]) + static_cast<int64_t>(local_expert) * p.q_expert_stride;
    r.bits = gload<uint8_t>(static_cast<const uint8_t*>(p.fields[1]) + row);
    r.bit_off = gload<int64_t>(static_cast<const int64_t*>(p.fields[2]) + row);
    r.gscale = static_cast<const uint8_t*>(p.fields[3]) + row * p.groups;
    r.gmin = static_cast<const uint8_t*>(p.fields[4]) + row * p.groups;
    r.rs = gload<float>(static_cast<const float*>(p.fields[5]) + row);
    r.rm = gload<float>(static_cast<const float*>(p.fields[6]) + row);
    if (UNIFORM) { r.bits = uniform(r.bits); r.bit_off = uniform(r.bit_off); r.rs = uniform(r.rs); r.rm = uniform(r.rm); }
    return r;
}

// Raw bytes of one chunk, fetched first so that the loads of many chunks are in flight together.
struct Raw { uint32_t a, b, c, d; };

// Byte-aligned row, group size a multiple of 8, every row BITS wide.  Reads at most 7 bytes
// past the last code of the row; the runtime layout keeps 8 guard bytes behind every stream.
template <int BITS, int GS>
__device__ __forceinline__ Raw nint_fetch(const NintRow& r, int chunk) {
    const uint8_t* p = r.stream + (r.bit_off >> 3) + chunk * BITS;
    const int group = (chunk * 8) / GS;
    Raw raw;
    raw.a = load_u32_unaligned(p);
    raw.b = BITS > 4 ? load_u32_unaligned(p + 4) : 0u;
    raw.c = gload<uint8_t>(r.gscale + group);
    raw.d = gload<uint8_t>(r.gmin + group);
    return raw;
}

template <int BITS, int GS>
__device__ __forceinline__ void nint_decode(const NintRow& r, const Raw& raw, float w[8]) {
    const float scale = r.rs * static_cast<float>(raw.c);
    const float minimum = r.rm * static_cast<float>(raw.d);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int bit = i * BITS;
        uint32_t q;
        if (bit + BITS <= 32) q = raw.a >> bit;
        else if (bit >= 32) q = raw.b >> (bit - 32);
        else q = (raw.a >> bit) | (raw.b << (32 - bit));
        q &= (1u << BITS) - 1u;
        w[i] = scale * static_cast<float>(q) - minimum;
    }
}

// Any width, group size and bit offset; columns at or beyond `width` decode to zero.  Loads use
// a clamped column so the code stays free of branches.
__device__ __forceinline__ void nint_chunk_generic(const NintRow& r, int chunk, int width, int gs, float w[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int col = chunk * 8 + i;
        const int safe = col < width ? col : width - 1;
        const int64_t bit = r.bit_off + static_cast<int64_t>(safe) * r.bits;
        const uint8_t* p = r.stream + (bit >> 3);
        const uint32_t word = static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 8);
        const uint32_t q = (word >> (bit & 7)) & ((1u << r.bits) - 1u);
        const int group = safe / gs;
        const float scale = r.rs * static_cast<float>(r.gscale[group]);
        const float minimum = r.rm * static_cast<float>(r.gmin[group]);
        const float value = scale * static_cast<float>(q) - minimum;
        w[i] = col < width ? value : 0.0f;
    }
}

// ----------------------------------------------------------------- NVQ ----
// Per-block LDS tables built from fields[4].
struct NvqTables {
    const uint32_t* codebook;  // D4: one dword per entry; E8: two dwords per entry; banks back to back
    const float* multiplier;   // [16]
    const int* bank_offset;    // [16] offset of the state's bank in dwords
};

__device__ __forceinline__ bool nvq_format_d4(int format) {
    return format == 3 || format == 10 || format == 12 || format == 15;
}
__device__ __forceinline__ bool nvq_format_jsc(int format) {
    return format == 5 || format == 10 || format == 12 || format == 13 || format == 14 || format == 15;
}
__host__ __device__ __forceinline__ int nvq_format_index_bits(int format) {
    return format == 12 ? 9 : (format == 13 || format == 15) ? 10 : format == 14 ? 12 : 8;
}
__host__ __device__ __forceinline__ int nvq_format_entries(int format) {
    return format == 12 ? 512 : (format == 13 || format == 15) ? 1024 : format == 14 ? 4096 : 256;
}
// The 4096-entry lattice (up to 4 banks x 32 KB) stays in global memory; every other codebook is copied to LDS.
__host__ __device__ __forceinline__ bool nvq_format_tables_in_lds(int format) { return format != 14; }
__host__ __device__ __forceinline__ int nvq_format_banks_max() { return 4; }

// Fills the LDS tables; call by every thread of the block, then __syncthreads().
// lds_words: banks*entries*(D4 ? 1 : 2) dwords (unused when the format keeps its codebook in global memory);
// lds_mult[16]; lds_bank[16].  Returns where the codebook words are read from.
__device__ __forceinline__ const uint32_t* nvq_build_tables(const mfq_amd_projection& p, uint32_t* lds_words,
                                                            float* lds_mult, int* lds_bank) {
    const int8_t* meta = static_cast<const int8_t*>(p.fields[4]);
    const bool jsc = nvq_format_jsc(p.format);
    const bool d4 = nvq_format_d4(p.format);
    const int entries = nvq_format_entries(p.format);
    const int words_per_entry = d4 ? 1 : 2;
    const int banks = jsc ? static_cast<uint8_t>(meta[1]) : 1;
    const uint8_t* tables = reinterpret_cast<const uint8_t*>(meta) + (jsc ? 64 : 0);
    const int total = banks * entries * words_per_entry;
    const bool in_lds = nvq_format_tables_in_lds(p.format);
    if (in_lds)
        for (int i = threadIdx.x; i < total; i += blockDim.x) lds_words[i] = load_u32_unaligned(tables + 4 * i);
    if (threadIdx.x < 16) {
        const int state = threadIdx.x;
        float multiplier;
        int bank = 0;
        if (jsc) {
            uint16_t h;
            __builtin_memcpy(&h, meta + 4 + 2 * state, 2);
            multiplier = 1.0f * half_bits_to_float(h);
            bank = static_cast<uint8_t>(meta[36 + state]);
        } else {
            multiplier = 1.0f * static_cast<float>(state);
        }
        lds_mult[state] = multiplier;
        lds_bank[state] = bank * entries * words_per_entry;
    }
    // the metadata block is a device allocation of its own and the header is 64 bytes: the words are aligned
    return in_lds ? lds_words : reinterpret_cast<const uint32_t*>(tables);
}

struct NvqRow {
    const uint8_t* indices; int64_t index_bytes;
    const uint8_t* aux;     int64_t aux_bytes;
    const uint8_t* states;  int64_t state_bytes;
    int64_t row;               // row inside the pool
    float anchor;
    int nvec, nsign, groups, index_bits, state_bits;
    bool d4, index_parity;
};

template <bool UNIFORM>
__device__ __forceinline__ NvqRow nvq_row(const mfq_amd_projection& p, int local_expert, int row_in_expert) {
    NvqRow r;
    r.indices = static_cast<const uint8_t*>(p.fields[0]); r.index_bytes = p.sizes[0];
    r.aux = static_cast<const uint8_t*>(p.fields[1]);     r.aux_bytes = p.sizes[1];
    r.states = static_cast<const uint8_t*>(p.fields[2]);  r.state_bytes = p.sizes[2];
    r.row = static_cast<int64_t>(local_expert) * p.output_rows + row_in_expert;
    r.anchor = gload<float>(static_cast<const float*>(p.fields[3]) + r.row);
    if (UNIFORM) r.anchor = uniform(r.anchor);
    r.nvec = p.nvec; r.nsign = p.nsign; r.groups = p.groups;
    r.index_bits = nvq_format_index_bits(p.format);
    r.state_bits = p.sub_bits;
    r.d4 = nvq_format_d4(p.format);
    r.index_parity = p.format == 2 && p.sign_mode != 0;
    return r;
}

__device__ __forceinline__ uint32_t parity7(uint32_t v) {
    return static_cast<uint32_t>(__builtin_popcount(v & 0x7fu)) & 1u;
}

// Segment `seg` (eight weights) of the row: state, two D4 indices (or one E8 index) and the sign mask.
template <bool D4>
__device__ __forceinline__ Raw nvq_fetch(const NvqRow& r, int seg) {
    Raw raw;
    raw.a = stream_bits(r.states, r.state_bytes, (r.row * r.groups + seg / 3) * r.state_bits, r.state_bits);
    raw.b = stream_bits(r.aux, r.aux_bytes, (r.row * r.nsign + seg) * 7, 7);
    raw.c = D4 ? stream_bits(r.indices, r.index_bytes, (r.row * r.nvec + 2 * seg) * r.index_bits, 2 * r.index_bits)
               : stream_bits(r.indices, r.index_bytes, (r.row * r.nvec + seg) * r.index_bits, r.index_bits);
    raw.d = 0;
    return raw;
}

template <bool D4>
__device__ __forceinline__ void nvq_decode(const NvqRow& r, const NvqTables& t, const Raw& raw, int seg, float w[8]) {
    const uint32_t state = raw.a, mask7 = raw.b;
    const uint32_t* bank = t.codebook + t.bank_offset[state];
    uint32_t lo, hi, first;
    if (D4) {
        first = raw.c & ((1u << r.index_bits) - 1u);
        lo = bank[first];
        const uint32_t second = bank[raw.c >> r.index_bits];
        hi = (2 * seg + 1 < r.nvec) ? second : 0u;
    } else {
        first = raw.c;
        lo = bank[2 * first];
        hi = bank[2 * first + 1];
    }
    const float scale = r.anchor * t.multiplier[state];
    const uint32_t last = parity7(mask7) ^ (r.index_parity ? ((first >> 7) & 1u) : 0u);
    const uint32_t mask8 = mask7 | (last << 7);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t word = i < 4 ? lo : hi;
        const int magnitude = static_cast<int8_t>((word >> (8 * (i & 3))) & 0xffu);
        const int value = ((mask8 >> i) & 1u) ? -magnitude : magnitude;
        w[i] = scale * static_cast<float>(value);
    }
}

// --------------------------------------------------------------- MXFP4 ----
struct MxRow {
    const uint8_t* values;   // the row's nibbles
    const uint8_t* scales;   // the row's E8M0 scales
};

__device__ __forceinline__ MxRow mx_row(const mfq_amd_projection& p, int local_expert, int row_in_expert) {
    const int64_t row = static_cast<int64_t>(local_expert) * p.output_rows + row_in_expert;
    MxRow r;
    r.values = static_cast<const uint8_t*>(p.fields[0]) + row * (p.input_width / 2);
    r.scales = static_cast<const uint8_t*>(p.fields[1]) + row * (p.input_width / 32);
    return r;
}

__device__ __forceinline__ void mx_build_table(float* lds_e2m1) {
    if (threadIdx.x < 16) {
        // E2M1 magnitude: codes 0,1 are 0 and 0.5; code c >= 2 has fp32 bits (c << 22) + 0x3F000000.
        const uint32_t c = threadIdx.x & 7;
        const float m = c >= 2 ? bits_to_float((c << 22) + 0x3F000000u) : 0.5f * static_cast<float>(c);
        lds_e2m1[threadIdx.x] = (threadIdx.x & 8) ? -m : m;
    }
}

__device__ __forceinline__ Raw mx_fetch(const MxRow& r, int chunk) {
    Raw raw;
    raw.a = load_u32_unaligned(r.values + 4 * chunk);
    raw.b = gload<uint8_t>(r.scales + (chunk >> 2));
    raw.c = raw.d = 0;
    return raw;
}

__device__ __forceinline__ void mx_decode(const Raw& raw, const float* lds_e2m1, float w[8]) {
    const float scale = bits_to_float(raw.b ? (raw.b << 23) : 0x00400000u);   // 2^(s-127); s = 0 is subnormal
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = lds_e2m1[(raw.a >> (4 * i)) & 15u] * scale;
}

// ------------------------------------------------- class-generic wrapper ----
// LDS needed by a class (bytes) for its decode tables.
__host__ __device__ inline int class_lds_bytes(int cls, int format) {
    if (cls == K_NVQ_D4) return 4 * nvq_format_entries(format) * 4 + 16 * 8;
    if (cls == K_NVQ_E8) return (nvq_format_tables_in_lds(format) ? 4 * nvq_format_entries(format) * 8 : 0) + 16 * 8;
    if (cls == K_MXFP4) return 64;
    return 0;
}

template <int CLS>
struct Decoder {
    NvqTables nvq;
    const float* e2m1;
    int width, gs;

    // `lds` must hold class_lds_bytes(CLS, p.format) bytes; call from every thread, then sync.
    __device__ __forceinline__ void init(const mfq_amd_projection& p, unsigned char* lds) {
        width = p.input_width;
        gs = p.group_size;
        if (CLS == K_NVQ_D4 || CLS == K_NVQ_E8) {
            float* mult = reinterpret_cast<float*>(lds);
            int* bank = reinterpret_cast<int*>(lds + 64);
            uint32_t* words = reinterpret_cast<uint32_t*>(lds + 128);
            nvq.codebook = nvq_build_tables(p, words, mult, bank);
            nvq.multiplier = mult; nvq.bank_offset = bank;
        } else if (CLS == K_MXFP4) {
            float* table = reinterpret_cast<float*>(lds);
            mx_build_table(table);
            e2m1 = table;
        }
    }

    struct Row {
        NintRow nint;
        NvqRow nvq;
        MxRow mx;
        bool fast;
    };

    template <bool UNIFORM = true>
    __device__ __forceinline__ void row(const mfq_amd_projection& p, int local_expert, int r, Row& out) const {
        if (CLS <= K_NINT_8_48) {
            constexpr int kBits = CLS == K_NINT_2_16 ? 2 : CLS == K_NINT_3_24 ? 3 : CLS == K_NINT_8_48 ? 8 : 4;
            out.nint = nint_row<UNIFORM>(p, local_expert, r);
            out.fast = CLS == K_NINT_GENERIC || ((out.nint.bit_off & 7) == 0 && out.nint.bits == kBits);
        } else if (CLS == K_NVQ_D4 || CLS == K_NVQ_E8) {
            out.nvq = nvq_row<UNIFORM>(p, local_expert, r);
            out.fast = true;
        } else {
            out.mx = mx_row(p, local_expert, r);
            out.fast = true;
        }
    }

    // Eight weights of columns [8*chunk, 8*chunk+8) in two phases: fetch() only issues loads, decode()
    // only computes, so a caller can put many chunks in flight before consuming the first.  Both need
    // row.fast for the fixed-width NINT classes; chunk() works for every row.  Columns >= width are
    // unspecified for the non-generic paths (callers mask them) and zero for the generic one.
    __device__ __forceinline__ Raw fetch(const Row& r, int c) const {
        if (CLS == K_NINT_2_16) return nint_fetch<2, 16>(r.nint, c);
        if (CLS == K_NINT_3_24) return nint_fetch<3, 24>(r.nint, c);
        if (CLS == K_NINT_4_24) return nint_fetch<4, 24>(r.nint, c);
        if (CLS == K_NINT_4_32) return nint_fetch<4, 32>(r.nint, c);
        if (CLS == K_NINT_8_48) return nint_fetch<8, 48>(r.nint, c);
        if (CLS == K_NVQ_D4) return nvq_fetch<true>(r.nvq, c);
        if (CLS == K_NVQ_E8) return nvq_fetch<false>(r.nvq, c);
        if (CLS == K_MXFP4) return mx_fetch(r.mx, c);
        return Raw{0u, 0u, 0u, 0u};
    }
    __device__ __forceinline__ void decode(const Row& r, const Raw& raw, int c, float w[8]) const {
        if (CLS == K_NINT_2_16) nint_decode<2, 16>(r.nint, raw, w);
        else if (CLS == K_NINT_3_24) nint_decode<3, 24>(r.nint, raw, w);
        else if (CLS == K_NINT_4_24) nint_decode<4, 24>(r.nint, raw, w);
        else if (CLS == K_NINT_4_32) nint_decode<4, 32>(r.nint, raw, w);
        else if (CLS == K_NINT_8_48) nint_decode<8, 48>(r.nint, raw, w);
        else if (CLS == K_NINT_GENERIC) nint_chunk_generic(r.nint, c, width, gs, w);
        else if (CLS == K_NVQ_D4) nvq_decode<true>(r.nvq, nvq, raw, c, w);
        else if (CLS == K_NVQ_E8) nvq_decode<false>(r.nvq, nvq, raw, c, w);
        else mx_decode(raw, e2m1, w);
    }
    __device__ __forceinline__ void chunk(const Row& r, int c, float w[8]) const {
        if (CLS >= K_NINT_2_16 && CLS <= K_NINT_8_48 && !r.fast) nint_chunk_generic(r.nint, c, width, gs, w);
        else decode(r, fetch(r, c), c, w);
    }
};

// ------------------------------------------------------ wave reduction ----
// Sum over the 64 lanes in a fixed order; every lane returns the total.
__device__ __forceinline__ float wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));  // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false));  // row_mirror
    // every lane of a 16-lane row now holds its row sum
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (r0 + r1) + (r2 + r3);
}

// ------------------------------------------------- activation loading ----
// Eight consecutive activations [8*chunk, 8*chunk+8) of a row as fp32, zero beyond `width`.
// `vector_ok`: the row base and stride are 16-byte aligned for the element type.
__device__ __forceinline__ void load_x8(const void* row, int dtype, int chunk, int width, bool vector_ok, float x[8]) {
    const int first = chunk * 8;
    if (first + 8 <= width && vector_ok) {
        if (dtype == MFQ_AMD_F32) {
            const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(row) + first);
            const float4 a = p[0], b = p[1];
            x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
        } else {
            const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(row) + first);
            const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint16_t lo = static_cast<uint16_t>(words[i] & 0xffffu), hi = static_cast<uint16_t>(words[i] >> 16);
                x[2 * i] = dtype == MFQ_AMD_F16 ? half_bits_to_float(lo) : bf16_bits_to_float(lo);
                x[2 * i + 1] = dtype == MFQ_AMD_F16 ? half_bits_to_float(hi) : bf16_bits_to_float(hi);
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int col = first + i;
        float v = 0.0f;
        if (col < width) {
            if (dtype == MFQ_AMD_F32) v = static_cast<const float*>(row)[col];
            else {
                const uint16_t raw = static_cast<const uint16_t*>(row)[col];
                v = dtype == MFQ_AMD_F16 ? half_bits_to_float(raw) : bf16_bits_to_float(raw);
            }
        }
        x[i] = v;
    }
}

}  // namespace dev
}  // namespace mfq_amd
