// ref_shim.cpp -- C-ABI doorway into the reference's own CPU compressed-math
// library, compiled from the reference's sources where they lie (never copied
// into this repository).  TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile
// into oracle/_ref/libmfq_ref.so; used to pin the C restatement bit-for-bit and
// as the "reference" CPU baseline.
//
// Wrapped entry points (reference checkout paths):
//   mfq::cpu::packed_nint_matmul            cpp_runtime/backends/cpu/ops/packed_nint.h:34-37
//   mfq::cpu::packed_nint_rows_kernel       cpp_runtime/backends/cpu/ops/packed_nint.h:26-29
//   mfq::cpu::detail::packed_nint_scalar_rows  packed_nint.h:40-42
//   mfq::cpu::nvq_rows_dot_kernel           cpp_runtime/backends/cpu/ops/nvq_group.h:33-34
//   mfq::cpu::scaled_i8_dot_kernel          cpp_runtime/backends/cpu/ops/quant_dot.h
//   mfq::cpu::expert_pool().rows            cpp_runtime/core/include/mfq/cpu_expert_pool.h:39-55
#include "mfq_oracle.h"      // descriptor structs of the C restatement (this directory), shared by the layer driver below
#include "packed_nint.h"
#include "nvq_group.h"
#include "quant_dot.h"
#include "mfq/cpu_expert_pool.h"
#include "mfq/host_parallel.h"

#include <cstdint>
#include <cstring>
#include <exception>
#include <vector>

namespace {
mfq::cpu::PackedNintView nint_view(const std::uint8_t* packed, std::int64_t packed_bytes,
        const std::uint8_t* row_bits, const std::int64_t* row_bit_offsets,
        const std::uint8_t* group_scale, const std::uint8_t* group_min,
        const float* row_scale, const float* row_min,
        std::int64_t outputs, std::int64_t width, std::int64_t group_size) {
    mfq::cpu::PackedNintView v;
    v.packed = packed; v.packed_bytes = static_cast<std::size_t>(packed_bytes);
    v.row_bits = row_bits; v.row_bit_offsets = row_bit_offsets;
    v.group_scale = group_scale; v.group_min = group_min;
    v.row_scale = row_scale; v.row_min = row_min;
    v.outputs = outputs; v.width = width; v.group_size = group_size;
    return v;
}
}

extern "C" {

int ref_has_avx2() { return mfq::cpu::packed_nint_has_avx2() ? 1 : 0; }

// kernel: 0 automatic (AVX2 when the host has it), 1 scalar.  Returns 0, or -1
// when the reference rejects the descriptor (std::invalid_argument).
int ref_packed_nint_matmul(const std::uint8_t* packed, std::int64_t packed_bytes,
        const std::uint8_t* row_bits, const std::int64_t* row_bit_offsets,
        const std::uint8_t* group_scale, const std::uint8_t* group_min,
        const float* row_scale, const float* row_min,
        std::int64_t outputs, std::int64_t width, std::int64_t group_size,
        const float* input, std::int64_t batch, std::int64_t input_stride,
        float* output, std::int64_t output_stride, int threads, int kernel) {
    try {
        const auto v = nint_view(packed, packed_bytes, row_bits, row_bit_offsets, group_scale,
            group_min, row_scale, row_min, outputs, width, group_size);
        mfq::cpu::packed_nint_matmul(v, input, batch, input_stride, output, output_stride, threads,
            kernel ? mfq::cpu::PackedNintKernel::scalar : mfq::cpu::PackedNintKernel::automatic);
        return 0;
    } catch (const std::exception&) { return -1; }
}

// Rows [begin,end) through the kernel the reference selects per expert job.
void ref_packed_nint_rows(const std::uint8_t* packed, std::int64_t packed_bytes,
        const std::uint8_t* row_bits, const std::int64_t* row_bit_offsets,
        const std::uint8_t* group_scale, const std::uint8_t* group_min,
        const float* row_scale, const float* row_min,
        std::int64_t outputs, std::int64_t width, std::int64_t group_size,
        const float* input, std::int64_t batch, std::int64_t input_stride,
        float* output, std::int64_t output_stride, std::int64_t begin, std::int64_t end, int pooled) {
    const auto v = nint_view(packed, packed_bytes, row_bits, row_bit_offsets, group_scale,
        group_min, row_scale, row_min, outputs, width, group_size);
    const auto rows = mfq::cpu::packed_nint_rows_kernel();
    if (pooled) {
        mfq::cpu::expert_pool().rows(end - begin, [&](std::int64_t b, std::int64_t e) {
            rows(v, input, batch, input_stride, output, output_stride, begin + b, begin + e);
        });
    } else rows(v, input, batch, input_stride, output, output_stride, begin, end);
}

// NVQ rows through nvq_rows_dot_kernel(format).  banks[s]/multipliers[s] are
// the per-state tables the reference loader prepares (cuda/ops/vq.cpp:364-368).
// Returns -1 when the reference has no fused kernel for the format on this host.
int ref_nvq_rows(int format, const std::uint8_t* indices, std::int64_t index_bytes,
        const std::uint8_t* aux, std::int64_t aux_bytes,
        const std::uint8_t* states, std::int64_t state_bytes, int state_bits,
        const float* anchors, const std::int8_t* const* banks, const float* multipliers,
        int nvec, int nsign, int groups, int sign_mode, std::int64_t width,
        const float* input, std::int64_t batch, std::int64_t input_stride,
        float* output, std::int64_t output_stride, std::int64_t begin, std::int64_t end, int pooled) {
    mfq::cpu::NvqDecodeView v{};
    v.indices = indices; v.aux = aux; v.index_bytes = index_bytes; v.aux_bytes = aux_bytes;
    v.nvec = nvec; v.nsign = nsign; v.groups = groups; v.sign_mode = sign_mode;
    for (int s = 0; s < (1 << state_bits) && s < 16; ++s) { v.banks[s] = banks[s]; v.multipliers[s] = multipliers[s]; }
    v.states = states; v.state_bytes = state_bytes; v.anchors = anchors; v.width = width;
    v.state_bits = state_bits;
    const auto rows = mfq::cpu::nvq_rows_dot_kernel(format);
    if (!rows) return -1;
    if (pooled) {
        mfq::cpu::expert_pool().rows(end - begin, [&](std::int64_t b, std::int64_t e) {
            rows(v, input, batch, input_stride, output, output_stride, begin + b, begin + e);
        });
    } else rows(v, input, batch, input_stride, output, output_stride, begin, end);
    return 0;
}

float ref_scaled_i8_dot(const std::int8_t* weights, const float* input, int count, float scale, int scalar) {
    return scalar ? mfq::cpu::scaled_i8_dot_scalar(weights, input, count, scale)
                  : mfq::cpu::scaled_i8_dot_kernel()(weights, input, count, scale);
}

int ref_pool_participants() { return mfq::cpu::expert_pool().participants(); }

// What the reference's CPU library does not contain (MXFP4 rows live behind its CUDA tensor class, the SwiGLU chain in
// its storage pipeline) comes from the C restatement through these pointers, so that one call covers a whole layer.
struct ref_layer_fns {
    void (*mx_rows)(const orc_mxfp4_view*, const float*, std::int64_t, std::int64_t, float*, std::int64_t, std::int64_t, std::int64_t);
    void (*swiglu)(const std::uint16_t*, const std::uint16_t*, std::int64_t, float, std::uint16_t*);
    std::uint16_t (*f32_to_f16)(float);
    float (*f16_to_f32)(std::uint16_t);
    float (*nvq_multiplier)(const orc_nvq_view*, std::uint32_t);
    const std::int8_t* (*nvq_bank)(const orc_nvq_view*, std::uint32_t);
};

namespace {
void layer_rows(const orc_projection& p, const ref_layer_fns& fns, const float* input, std::int64_t batch, std::int64_t width,
                float* output, std::int64_t outputs, bool pooled) {
    auto split = [&](auto&& rows) {
        if (pooled) mfq::cpu::expert_pool().rows(outputs, [&](std::int64_t b, std::int64_t e) { rows(b, e); });
        else rows(0, outputs);
    };
    if (p.family == ORC_FAMILY_NINT) {
        const auto& n = p.nint;
        const auto v = nint_view(n.packed, n.packed_bytes, n.row_bits, n.row_bit_offsets, n.group_scale, n.group_min,
                                 n.row_scale, n.row_min, n.outputs, n.width, n.group_size);
        const auto kernel = mfq::cpu::packed_nint_rows_kernel();
        split([&](std::int64_t b, std::int64_t e) { kernel(v, input, batch, width, output, outputs, b, e); });
    } else if (p.family == ORC_FAMILY_NVQ) {
        const auto& q = p.nvq;
        const bool d4 = q.format == 3 || q.format == 10 || q.format == 11 || q.format == 12 || q.format == 15;
        mfq::cpu::NvqDecodeView v{};
        v.indices = q.indices; v.aux = q.aux; v.index_bytes = q.index_bytes; v.aux_bytes = q.aux_bytes;
        v.nvec = static_cast<int>((q.width + (d4 ? 3 : 7)) / (d4 ? 4 : 8)); v.nsign = static_cast<int>((q.width + 7) / 8);
        v.groups = static_cast<int>((q.width + 23) / 24); v.sign_mode = q.sign_mode;
        for (int s = 0; s < (1 << q.state_bits) && s < 16; ++s) {
            v.banks[s] = fns.nvq_bank(&q, static_cast<std::uint32_t>(s));
            v.multipliers[s] = fns.nvq_multiplier(&q, static_cast<std::uint32_t>(s));
        }
        v.states = q.states; v.state_bytes = q.state_bytes; v.anchors = q.anchors; v.width = q.width; v.state_bits = q.state_bits;
        const auto kernel = mfq::cpu::nvq_rows_dot_kernel(q.format);
        // the pool's streams are flat over all its rows: this expert's rows start at row_offset; results go to columns
        // [0, outputs) of `output`
        float* shifted = output - q.row_offset;
        split([&](std::int64_t b, std::int64_t e) {
            kernel(v, input, batch, width, shifted, outputs, q.row_offset + b, q.row_offset + e);
        });
    } else {
        split([&](std::int64_t b, std::int64_t e) { fns.mx_rows(&p.mxfp4, input, batch, width, output, outputs, b, e); });
    }
}
}  // namespace

// One MoE layer for the routed tokens of `experts` experts: per expert, gate and up rows of its tokens, the fp16 SwiGLU
// chain, down rows (cuda/storage/moe_ffn_pipeline.cpp:142-180).  projections: [experts][3] (gate, up, down);
// token_offsets [experts + 1] into token_ids; x [tokens, hidden].  pooled: rows split over the reference's pinned expert
// pool (all cores), else on the calling thread.  out [pairs routed, hidden] in expert order.  Returns 0, or -1 when the
// reference has no fused kernel for a format on this host.
int ref_layer(const orc_projection* projections, const std::int32_t* token_offsets, const std::int32_t* token_ids, int experts,
              const float* x, std::int64_t hidden, std::int64_t inter, int pooled, const ref_layer_fns* fns, float* out) {
    std::vector<float> input, gate, up, mid;
    std::vector<std::uint16_t> g16, u16, h16;
    for (int e = 0; e < experts; ++e) {
        const std::int64_t first = token_offsets[e], count = token_offsets[e + 1] - first;
        if (count <= 0) continue;
        input.resize(count * hidden); gate.resize(count * inter); up.resize(count * inter); mid.resize(count * inter);
        g16.resize(count * inter); u16.resize(count * inter); h16.resize(count * inter);
        for (std::int64_t i = 0; i < count; ++i)
            std::memcpy(&input[i * hidden], x + static_cast<std::int64_t>(token_ids[first + i]) * hidden, sizeof(float) * hidden);
        const orc_projection* p = projections + 3 * e;
        if (p[1].family == ORC_FAMILY_NVQ && !mfq::cpu::nvq_rows_dot_kernel(p[1].nvq.format)) return -1;
        layer_rows(p[0], *fns, input.data(), count, hidden, gate.data(), inter, pooled != 0);
        layer_rows(p[1], *fns, input.data(), count, hidden, up.data(), inter, pooled != 0);
        for (std::int64_t i = 0; i < count * inter; ++i) { g16[i] = fns->f32_to_f16(gate[i]); u16[i] = fns->f32_to_f16(up[i]); }
        fns->swiglu(g16.data(), u16.data(), count * inter, 0.0f, h16.data());
        for (std::int64_t i = 0; i < count * inter; ++i) mid[i] = fns->f16_to_f32(h16[i]);
        layer_rows(p[2], *fns, mid.data(), count, inter, out + first * hidden, hidden, pooled != 0);
    }
    return 0;
}

}  // extern "C"
