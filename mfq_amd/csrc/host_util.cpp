// Error state, descriptor validation and kernel-class selection (host only).
#include "common.h"
#include "decode_classes.h"

#include <cstring>

namespace mfq_amd {

namespace {
thread_local char g_error[512] = "";
}

void set_error(const char* format, ...) {
    va_list args;
    va_start(args, format);
    std::vsnprintf(g_error, sizeof(g_error), format, args);
    va_end(args);
}

static bool nvq_format_supported(int format) {
    return format == 2 || format == 3 || format == 5 || format == 10 || format == 12 || format == 13 || format == 14 ||
           format == 15;
}

// The reference's loader marks an NVQ3J pool whose two banks and state scales follow the analytic rule with
// kernel format 11 (cpp_runtime/backends/cuda/ops/vq.cpp:1695-1700): bank = state & 1 and scale = (state >> 1) + 1,
// which is what the tables of such a pool hold (vq.cpp:214-216, :242-244), so it decodes as format 10.
mfq_amd_projection canonical_projection(const mfq_amd_projection& p) {
    mfq_amd_projection q = p;
    if (q.family == MFQ_AMD_FAMILY_NVQ && q.format == 11) q.format = 10;
    return q;
}

// Mirrors the reference's descriptor checks (cpp_runtime/backends/cpu/ops/packed_nint.cpp:15-34 for
// NINT geometry and storage; cuda/ops/mfe_ffn.cpp:75-79 for group geometry) as far as a host can
// see them: device buffers are not dereferenced here.
void validate_projection(const mfq_amd_projection& p, int local_expert) {
    MFQ_REQUIRE(p.family >= MFQ_AMD_FAMILY_NINT && p.family <= MFQ_AMD_FAMILY_MXFP4, "unknown projection family");
    MFQ_REQUIRE(p.local_experts > 0 && p.output_rows > 0 && p.input_width > 0, "invalid projection geometry");
    MFQ_REQUIRE(local_expert >= 0 && local_expert < p.local_experts, "local expert out of range");
    if (p.family == MFQ_AMD_FAMILY_NINT) {
        MFQ_REQUIRE(p.group_size > 0, "invalid packed NINT geometry");
        MFQ_REQUIRE(p.groups == 1 + (p.input_width - 1) / p.group_size, "NINT group count does not match width");
        for (int i = 0; i < 7; ++i) MFQ_REQUIRE(p.fields[i] != nullptr, "missing packed NINT storage");
        MFQ_REQUIRE(p.local_experts == 1 || p.q_expert_stride > 0, "MFE NINT pools need q_expert_stride");
        MFQ_REQUIRE(p.uniform_bits >= 0 && p.uniform_bits <= 8, "NINT code width must be 1..8 (0 = per-row widths)");
        // the code stream of one expert: rows * groups * group_size codes of uniform_bits each (per-row widths: at
        // least one bit each); every expert's stream must fit its stride and the last one the storage
        const int64_t codes = static_cast<int64_t>(p.output_rows) * p.groups * p.group_size;
        const int64_t stream = (codes * (p.uniform_bits ? p.uniform_bits : 1) + 7) / 8;
        MFQ_REQUIRE(p.q_expert_stride >= 0 && (p.local_experts == 1 || p.q_expert_stride >= stream),
                    "packed NINT expert stream exceeds its stride");
        MFQ_REQUIRE(p.sizes[0] >= (p.local_experts - 1) * p.q_expert_stride + stream, "packed NINT row exceeds storage");
    } else if (p.family == MFQ_AMD_FAMILY_NVQ) {
        if (!nvq_format_supported(p.format)) fail_unsupported("NVQ runtime format is not implemented");
        MFQ_REQUIRE(p.group_size == 24, "NVQ requires 24-value groups");
        MFQ_REQUIRE(p.sub_bits >= 1 && p.sub_bits <= 4, "NVQ state width must be 1..4");
        const bool d4 = p.format == 3 || p.format == 10 || p.format == 12 || p.format == 15;
        MFQ_REQUIRE(p.groups == (p.input_width + 23) / 24, "NVQ group count does not match width");
        MFQ_REQUIRE(p.nvec == (p.input_width + (d4 ? 3 : 7)) / (d4 ? 4 : 8), "NVQ vector count does not match width");
        MFQ_REQUIRE(p.nsign == (p.input_width + 7) / 8, "NVQ sign count does not match width");
        for (int i = 0; i < 5; ++i) MFQ_REQUIRE(p.fields[i] != nullptr, "missing packed NVQ storage");
        const int64_t rows = static_cast<int64_t>(p.local_experts) * p.output_rows;
        const int index_bits = p.format == 12 ? 9 : (p.format == 13 || p.format == 15) ? 10 : p.format == 14 ? 12 : 8;
        MFQ_REQUIRE(p.sizes[0] >= (rows * p.nvec * index_bits + 7) / 8, "NVQ index stream is too short");
        MFQ_REQUIRE(p.format != 14 || reinterpret_cast<uintptr_t>(p.fields[4]) % 4 == 0,
                    "NVQ2J-XL codebooks must be 4-byte aligned");
        MFQ_REQUIRE(p.sizes[1] >= (rows * p.nsign * 7 + 7) / 8, "NVQ sign stream is too short");
        MFQ_REQUIRE(p.sizes[2] >= (rows * p.groups * p.sub_bits + 7) / 8, "NVQ state stream is too short");
    } else {
        MFQ_REQUIRE(p.input_width % 32 == 0, "MXFP4 columns must be divisible by 32");
        MFQ_REQUIRE(p.fields[0] != nullptr && p.fields[1] != nullptr, "missing packed MXFP4 storage");
        MFQ_REQUIRE(reinterpret_cast<uintptr_t>(p.fields[0]) % 4 == 0, "MXFP4 values must be 4-byte aligned");
    }
}

int projection_class(const mfq_amd_projection& p) {
    using namespace dev;
    if (p.family == MFQ_AMD_FAMILY_NINT) {
        if (p.group_size % 8 == 0) {
            if (p.uniform_bits == 2 && p.group_size == 16) return K_NINT_2_16;
            if (p.uniform_bits == 3 && p.group_size == 24) return K_NINT_3_24;
            if (p.uniform_bits == 4 && p.group_size == 24) return K_NINT_4_24;
            if (p.uniform_bits == 4 && p.group_size == 32) return K_NINT_4_32;
            if (p.uniform_bits == 8 && p.group_size == 48) return K_NINT_8_48;
        }
        return K_NINT_GENERIC;
    }
    if (p.family == MFQ_AMD_FAMILY_NVQ)
        return (p.format == 3 || p.format == 10 || p.format == 12 || p.format == 15) ? K_NVQ_D4 : K_NVQ_E8;
    return K_MXFP4;
}

// Runtime-layout bytes one expert contributes when every packed field is read once.  NINT: q codes
// (uniform width assumed from uniform_bits, else 8) + two level bytes per group + 17 bytes of row
// metadata (two f32 anchors, width byte, i64 offset); NVQ: index/sign/state bits + f32 anchor;
// MXFP4: nibbles + scales.  Codebooks and lookup tables are excluded.
int64_t projection_expert_bytes(const mfq_amd_projection& p) {
    const int64_t rows = p.output_rows;
    if (p.family == MFQ_AMD_FAMILY_NINT) {
        const int bits = p.uniform_bits ? p.uniform_bits : 8;
        const int64_t row_bits = static_cast<int64_t>(p.groups) * p.group_size * bits;
        return rows * ((row_bits + 7) / 8 + 2 * p.groups + 17);
    }
    if (p.family == MFQ_AMD_FAMILY_NVQ) {
        const int index_bits = p.format == 12 ? 9 : (p.format == 13 || p.format == 15) ? 10 : p.format == 14 ? 12 : 8;
        const int64_t bits = static_cast<int64_t>(p.nvec) * index_bits + static_cast<int64_t>(p.nsign) * 7 +
                             static_cast<int64_t>(p.groups) * p.sub_bits;
        return (rows * bits + 7) / 8 + rows * 4;
    }
    return rows * (p.input_width / 2 + p.input_width / 32);
}

}  // namespace mfq_amd

extern "C" const char* mfq_amd_last_error(void) { return mfq_amd::g_error; }
extern "C" int mfq_amd_abi_version(void) { return 1; }
