// Activations as the streaming MFMA tile kernel reads them: fp16, every 32 columns in the pair order of a weight
// class (pair_column<CLS>).  Shared by the tile pack kernel and the route plan kernel, whose spare blocks do the
// same work while its first block builds the plan.
#pragma once

#include "common.h"
#include "decode.cuh"
#include "fast.cuh"

namespace mfq_amd {
namespace dev {

// Converts 32 consecutive activations (64 bytes as loaded) to the 16 fp16 pairs of the class.
template <int CLS, bool HALF>
__device__ __forceinline__ void x_pairs(const u32x4 (&raw)[4], uint32_t (&p)[16]) {
    const uint32_t words[16] = {raw[0][0], raw[0][1], raw[0][2], raw[0][3], raw[1][0], raw[1][1], raw[1][2], raw[1][3],
                                raw[2][0], raw[2][1], raw[2][2], raw[2][3], raw[3][0], raw[3][1], raw[3][2], raw[3][3]};
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        const int first = pair_column<CLS>(k, 0), second = pair_column<CLS>(k, 1);
        if (HALF) {
            // select two of the four halves of two words: one byte permute
            const uint32_t selector = ((first & 1) ? 0x0302u : 0x0100u) | ((second & 1) ? 0x07060000u : 0x05040000u);
            p[k] = __builtin_amdgcn_perm(words[second / 2], words[first / 2], selector);
        } else {
            // bf16 -> fp32 is a shift; values inside the fp16 range convert without rounding
            const uint32_t a = (first & 1) ? words[first / 2] & 0xffff0000u : words[first / 2] << 16;
            const uint32_t b = (second & 1) ? words[second / 2] & 0xffff0000u : words[second / 2] << 16;
            p[k] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bits_to_float(a), bits_to_float(b)));
        }
    }
}

// The four pair layouts of tile_layout<CLS>() as classes that have them.
template <int LAYOUT> struct LayoutClass;
template <> struct LayoutClass<0> { static constexpr int value = K_NINT_4_24; };
template <> struct LayoutClass<1> { static constexpr int value = K_NINT_8_48; };
template <> struct LayoutClass<2> { static constexpr int value = K_NVQ_D4; };
template <> struct LayoutClass<3> { static constexpr int value = K_NINT_2_16; };

template <int LAYOUT>
__device__ __forceinline__ void store_layout(const u32x4 (&raw)[4], bool half_in, uint16_t* dst) {
    uint32_t p[16];
    if (half_in) x_pairs<LayoutClass<LAYOUT>::value, true>(raw, p);
    else x_pairs<LayoutClass<LAYOUT>::value, false>(raw, p);
#pragma unroll
    for (int j = 0; j < 4; ++j)
        *reinterpret_cast<u32x4*>(dst + 8 * j) = u32x4{p[4 * j], p[4 * j + 1], p[4 * j + 2], p[4 * j + 3]};
}

// One lane block (32 columns) of the copies: item = row * (width / 32) + lane block.
__device__ __forceinline__ void tile_pack_item(int64_t item, const void* src, int dtype, int rows, int width, uint32_t layouts,
                                               uint16_t* dst, int64_t layout_stride) {
    const int blocks = width / kLaneColumns;
    if (item >= static_cast<int64_t>(rows) * blocks) return;
    const unsigned char* from = static_cast<const unsigned char*>(src) + item * 64;
    u32x4 raw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) raw[j] = *(const MFQ_GLOBAL u32x4*)(from + 16 * j);
    const bool half_in = dtype == MFQ_AMD_F16;
    uint16_t* to = dst + item * kLaneColumns;
    if (layouts & 1u) store_layout<0>(raw, half_in, to);
    if (layouts & 2u) store_layout<1>(raw, half_in, to + layout_stride);
    if (layouts & 4u) store_layout<2>(raw, half_in, to + 2 * layout_stride);
    if (layouts & 8u) store_layout<3>(raw, half_in, to + 3 * layout_stride);
}

}  // namespace dev
}  // namespace mfq_amd
