// Canonical blobs -> runtime packed layout, and upload to the device.
//
// NINT  (blob: mfq/formats/io.py:181, :381-407; runtime: cpp_runtime/backends/cuda/ops/nint.cpp:750-964,
//        MFE re-streaming :1384-1459)
// NVQ   (blob: mfq/formats/nvq.py:791-929; runtime: ops/vq.cpp:1030-1330)
// MXFP4 (blob: mfq/formats/mx.py:20-25, :145-181; runtime: ops/mx.cpp:380-420)
// MFE   (container: mfq/formats/io.py:486-493, :723-760; runtime: ops/moe.cpp:25-182)
#include "common.h"

#include <algorithm>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

namespace mfq_amd {
namespace tables {
extern const uint16_t kE8_256[256];
extern const uint16_t kD4_256[256];
extern const uint16_t kD4_512[512];
}

namespace {

struct Reader {
    const uint8_t* data;
    int64_t size;
    int64_t off = 0;
    int64_t left() const { return size - off; }
    // compares against the bytes that remain, so that a length near the top of the range cannot wrap the sum
    // (cpp_runtime/backends/cuda/ops/moe.cpp:70-87 does the same)
    void need(int64_t n, const char* what) const {
        if (n < 0 || n > size - off) fail_invalid(std::string("truncated ") + what);
    }
    void need_u64(uint64_t n, const char* what) const {
        if (n > static_cast<uint64_t>(size - off)) fail_invalid(std::string("truncated ") + what);
    }
    template <class T> T get(const char* what) {
        need(sizeof(T), what);
        T v;
        std::memcpy(&v, data + off, sizeof(T));
        off += sizeof(T);
        return v;
    }
    const uint8_t* take(int64_t n, const char* what) {
        need(n, what);
        const uint8_t* p = data + off;
        off += n;
        return p;
    }
};

// a * b for non-negative operands; fails instead of wrapping (every product here counts bytes or bits of a blob)
inline int64_t checked_mul(int64_t a, int64_t b, const char* what) {
    if (a < 0 || b < 0 || (b != 0 && a > (int64_t(1) << 59) / b)) fail_invalid(std::string("oversized ") + what);
    return a * b;
}

inline int64_t stream_bytes(int64_t count, int bits) { return (checked_mul(count, bits, "bit stream") + 7) / 8; }

// LSB-first bit stream reader for metadata streams (values <= 8 bits).
std::vector<uint8_t> unpack_bits(Reader& in, int64_t count, int bits, const char* what) {
    MFQ_REQUIRE(count >= 0 && bits >= 1 && bits <= 8, "invalid bit stream geometry");
    const uint8_t* p = in.take(stream_bytes(count, bits), what);   // fails before anything is allocated
    std::vector<uint8_t> out(static_cast<size_t>(count));
    for (int64_t i = 0; i < count; ++i) {
        const int64_t bit = i * bits;
        uint32_t word = p[bit >> 3];
        if ((bit & 7) + bits > 8) word |= static_cast<uint32_t>(p[(bit >> 3) + 1]) << 8;
        out[static_cast<size_t>(i)] = static_cast<uint8_t>((word >> (bit & 7)) & ((1u << bits) - 1u));
    }
    return out;
}

// Copies `count` bits from bit `src_bit` of src to bit `dst_bit` of dst (dst pre-zeroed).
void copy_bits(const uint8_t* src, int64_t src_bit, uint8_t* dst, int64_t dst_bit, int64_t count) {
    if (((src_bit | dst_bit) & 7) == 0) {
        std::memcpy(dst + (dst_bit >> 3), src + (src_bit >> 3), static_cast<size_t>(count >> 3));
        src_bit += count & ~int64_t(7); dst_bit += count & ~int64_t(7); count &= 7;
    }
    for (int64_t i = 0; i < count; ++i) {
        const int64_t s = src_bit + i, d = dst_bit + i;
        if ((src[s >> 3] >> (s & 7)) & 1u) dst[d >> 3] |= static_cast<uint8_t>(1u << (d & 7));
    }
}

float half_to_float(uint16_t h) {
    const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {
            int shift = 0;
            uint32_t m = man;
            while (!(m & 0x400u)) { m <<= 1; ++shift; }
            bits = sign | ((113u - shift) << 23) | ((m & 0x3ffu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112u) << 23) | (man << 13);
    float v;
    std::memcpy(&v, &bits, 4);
    return v;
}

template <class T> std::vector<uint8_t> as_bytes(const std::vector<T>& v) {
    std::vector<uint8_t> out(v.size() * sizeof(T));
    if (!v.empty()) std::memcpy(out.data(), v.data(), out.size());
    return out;
}

constexpr int kGuardBytes = 8;

}  // namespace
}  // namespace mfq_amd

using namespace mfq_amd;

struct mfq_amd_tensor {
    mfq_amd_projection geom{};            // geometry; pointers filled per view
    std::vector<uint8_t> host[7];         // field payloads (exact sizes in payload_bytes)
    int64_t payload_bytes[7] = {0, 0, 0, 0, 0, 0, 0};
    void* dev[7] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    int32_t* dev_expert_local = nullptr;
    bool uploaded = false;
    int field_count = 0;

    ~mfq_amd_tensor() {
        for (void* p : dev) if (p) (void)hipFree(p);
        if (dev_expert_local) (void)hipFree(dev_expert_local);
    }
    void set_field(int i, std::vector<uint8_t> bytes) {
        payload_bytes[i] = static_cast<int64_t>(bytes.size());
        bytes.resize(bytes.size() + kGuardBytes, 0);     // readable slack behind every field
        host[i] = std::move(bytes);
        field_count = std::max(field_count, i + 1);
    }
    void fill_view(mfq_amd_projection& view, bool device) const {
        view = geom;
        for (int i = 0; i < 9; ++i) view.fields[i] = nullptr;
        for (int i = 0; i < field_count; ++i)
            view.fields[i] = device ? dev[i] : static_cast<const void*>(host[i].data());
        for (int i = 0; i < 3; ++i) view.sizes[i] = payload_bytes[i];
        view.expert_local = device ? dev_expert_local : nullptr;
    }
};

namespace {

// ---------------------------------------------------------------- NINT ----
std::unique_ptr<mfq_amd_tensor> load_nint(const uint8_t* blob, int64_t nbytes, int out_per_expert) {
    Reader in{blob, nbytes};
    const int raw_bits = in.get<uint8_t>("NINT header");
    const int sub_bits = in.get<uint8_t>("NINT header");
    const int gs = in.get<int32_t>("NINT header");
    const int axis = in.get<int32_t>("NINT header");
    const int neuron_len = in.get<int32_t>("NINT header");
    const uint32_t ndim = in.get<uint32_t>("NINT header");
    // bit 7 set: per-row widths with selector streams; clear: the uniform bit-packed storage older files hold
    // (cpp_runtime/backends/cuda/ops/nint.cpp:758, :873-875, :927-958)
    const bool per_row_widths = (raw_bits & 0x80) != 0;
    const int bits = raw_bits & 0x7f;
    MFQ_REQUIRE(bits >= 1 && bits <= 8 && sub_bits >= 1 && sub_bits <= 8 && gs > 0 && axis >= 0 &&
                neuron_len > 0 && ndim > 0 && ndim <= 8 && axis < static_cast<int>(ndim), "invalid NINT header");
    std::vector<int64_t> shape(ndim);
    for (auto& d : shape) d = in.get<int64_t>("NINT dimensions");
    const int64_t out = in.get<uint32_t>("NINT dimensions");
    const int64_t ng = in.get<uint32_t>("NINT dimensions");
    MFQ_REQUIRE(out > 0 && ng > 0 && ng == (static_cast<int64_t>(neuron_len) + gs - 1) / gs,
                "inconsistent NINT tensor dimensions");
    // nothing is allocated from header counts the remaining bytes cannot back: two fp16 anchors per row, and at
    // least one bit per group level, group minimum and code
    in.need(checked_mul(out, 4, "NINT neuron metadata"), "NINT neuron metadata");
    const int64_t level_count = checked_mul(out, ng, "NINT group metadata");
    const int64_t values_per_row = checked_mul(ng, gs, "NINT row");
    MFQ_REQUIRE(level_count / 4 <= in.left() && checked_mul(out, values_per_row, "NINT packed values") / 8 <= in.left(),
                "truncated NINT payload");
    std::vector<float> scale(out), minimum(out);
    {
        const uint8_t* p = in.take(out * 2, "NINT neuron metadata");
        const uint8_t* q = in.take(out * 2, "NINT neuron metadata");
        for (int64_t r = 0; r < out; ++r) {
            uint16_t a, b;
            std::memcpy(&a, p + 2 * r, 2);
            std::memcpy(&b, q + 2 * r, 2);
            MFQ_REQUIRE((a & 0x7c00u) != 0x7c00u && (b & 0x7c00u) != 0x7c00u, "NINT neuron metadata must be finite");
            scale[r] = half_to_float(a);
            minimum[r] = half_to_float(b);
        }
    }
    // group levels: 2-bit width selector per row, then per selector the levels and minima of its rows
    std::vector<uint8_t> sub_scale(out * ng), sub_min(out * ng);
    if (!per_row_widths) {
        sub_scale = unpack_bits(in, out * ng, sub_bits, "NINT group levels");
        sub_min = unpack_bits(in, out * ng, sub_bits, "NINT group minima");
    }
    const auto k_sel = per_row_widths ? unpack_bits(in, out, 2, "NINT k selectors") : std::vector<uint8_t>();
    for (int sel = 0; per_row_widths && sel < 4; ++sel) {
        const int64_t rows = std::count(k_sel.begin(), k_sel.end(), static_cast<uint8_t>(sel));
        if (!rows) continue;
        const int width = sub_bits - 1 + sel;
        MFQ_REQUIRE(width >= 1 && width <= 8, "invalid NINT v2 subgroup width");
        const auto levels = unpack_bits(in, rows * ng, width, "NINT group levels");
        const auto minima = unpack_bits(in, rows * ng, width, "NINT group minima");
        int64_t local = 0;
        for (int64_t r = 0; r < out; ++r) {
            if (k_sel[r] != sel) continue;
            std::copy_n(levels.begin() + local * ng, ng, sub_scale.begin() + r * ng);
            std::copy_n(minima.begin() + local * ng, ng, sub_min.begin() + r * ng);
            ++local;
        }
    }
    // codes: 3-bit width selector per row, then one bit-packed cohort per width in ascending order
    const auto q_sel = per_row_widths ? unpack_bits(in, out, 3, "NINT q selectors") : std::vector<uint8_t>();
    std::vector<uint8_t> row_bits(out);
    std::vector<int64_t> offsets(out);
    std::vector<uint8_t> packed;
    if (!per_row_widths) {
        const int64_t bytes = stream_bytes(out * values_per_row, bits);
        const uint8_t* p = in.take(bytes, "NINT packed values");
        packed.assign(p, p + bytes);
        for (int64_t r = 0; r < out; ++r) {
            row_bits[r] = static_cast<uint8_t>(bits);
            offsets[r] = r * values_per_row * bits;
        }
    }
    for (int sel = 0; per_row_widths && sel < 8; ++sel) {
        const int64_t rows = std::count(q_sel.begin(), q_sel.end(), static_cast<uint8_t>(sel));
        if (!rows) continue;
        const int width = sel + 1;
        const int64_t cohort_bytes = stream_bytes(rows * values_per_row, width);
        const uint8_t* p = in.take(cohort_bytes, "NINT mixed-q value stream");
        const int64_t start_bits = static_cast<int64_t>(packed.size()) * 8;
        packed.insert(packed.end(), p, p + cohort_bytes);
        int64_t local = 0;
        for (int64_t r = 0; r < out; ++r) {
            if (q_sel[r] != sel) continue;
            row_bits[r] = static_cast<uint8_t>(width);
            offsets[r] = start_bits + local * values_per_row * width;
            ++local;
        }
    }
    MFQ_REQUIRE(in.off == nbytes, "invalid NINT trailing bytes");

    auto t = std::make_unique<mfq_amd_tensor>();
    auto& g = t->geom;
    g.family = MFQ_AMD_FAMILY_NINT;
    g.input_width = neuron_len; g.groups = static_cast<int32_t>(ng); g.group_size = gs; g.sub_bits = sub_bits;
    int uniform = row_bits[0];
    for (auto b : row_bits) if (b != uniform) uniform = 0;
    g.uniform_bits = uniform;
    if (out_per_expert > 0) {
        MFQ_REQUIRE(out % out_per_expert == 0, "invalid MFE NINT expert geometry");
        const int64_t experts = out / out_per_expert;
        int64_t max_bits = 0;
        for (int64_t e = 0; e < experts; ++e) {
            int64_t bits_e = 0;
            for (int64_t r = e * out_per_expert; r < (e + 1) * out_per_expert; ++r) bits_e += values_per_row * row_bits[r];
            max_bits = std::max(max_bits, bits_e);
        }
        const int64_t stride = (max_bits + 7) / 8 + 8;
        std::vector<uint8_t> streams(static_cast<size_t>(experts * stride), 0);
        std::vector<int64_t> relative(out);
        for (int64_t e = 0; e < experts; ++e) {
            int64_t cursor = 0;
            for (int64_t r = e * out_per_expert; r < (e + 1) * out_per_expert; ++r) {
                const int64_t n = values_per_row * row_bits[r];
                relative[r] = cursor;
                copy_bits(packed.data(), offsets[r], streams.data(), e * stride * 8 + cursor, n);
                cursor += n;
            }
        }
        g.local_experts = static_cast<int32_t>(experts); g.output_rows = out_per_expert; g.q_expert_stride = stride;
        t->set_field(0, std::move(streams));
        t->set_field(2, as_bytes(relative));
    } else {
        packed.insert(packed.end(), 8, 0);
        g.local_experts = 1; g.output_rows = static_cast<int32_t>(out); g.q_expert_stride = 0;
        t->set_field(0, std::move(packed));
        t->set_field(2, as_bytes(offsets));
    }
    t->set_field(1, std::move(row_bits));
    t->set_field(3, std::move(sub_scale));
    t->set_field(4, std::move(sub_min));
    t->set_field(5, as_bytes(scale));
    t->set_field(6, as_bytes(minimum));
    return t;
}

// ----------------------------------------------------------------- NVQ ----
std::vector<int8_t> expand_grid(const uint16_t* words, int count, int dims, int digit_bits) {
    std::vector<int8_t> out(static_cast<size_t>(count) * dims);
    for (int e = 0; e < count; ++e)
        for (int i = 0; i < dims; ++i)
            out[static_cast<size_t>(e) * dims + i] =
                static_cast<int8_t>(2 * ((words[e] >> (digit_bits * i)) & ((1 << digit_bits) - 1)) + 1);
    return out;
}

// Nested extension of a base lattice by unused points in bit-reversed id order (mfq/formats/nvq.py:223-264).
std::vector<uint16_t> extend_grid(const uint16_t* base, int base_count, int total_bits, int entries) {
    std::vector<uint8_t> used(size_t(1) << total_bits, 0);
    std::vector<uint16_t> out(base, base + base_count);
    for (int i = 0; i < base_count; ++i) used[base[i]] = 1;
    for (uint32_t i = 0; i < (1u << total_bits) && static_cast<int>(out.size()) < entries; ++i) {
        uint32_t rev = 0;
        for (int b = 0; b < total_bits; ++b) rev |= ((i >> b) & 1u) << (total_bits - 1 - b);
        if (!used[rev]) out.push_back(static_cast<uint16_t>(rev));
    }
    return out;
}

std::vector<int8_t> builtin_grid(const std::string& name, int& entries, int& dim) {
    if (name == "e8_256") { entries = 256; dim = 8; return expand_grid(tables::kE8_256, 256, 8, 2); }
    if (name == "d4_256") { entries = 256; dim = 4; return expand_grid(tables::kD4_256, 256, 4, 3); }
    if (name == "d4_512") { entries = 512; dim = 4; return expand_grid(tables::kD4_512, 512, 4, 3); }
    if (name == "d4_1024") {
        entries = 1024; dim = 4;
        const auto words = extend_grid(tables::kD4_512, 512, 12, 1024);
        return expand_grid(words.data(), 1024, 4, 3);
    }
    if (name == "e8_1024") {
        entries = 1024; dim = 8;
        const auto words = extend_grid(tables::kE8_256, 256, 16, 1024);
        return expand_grid(words.data(), 1024, 8, 2);
    }
    fail_invalid("unknown NVQ lattice: " + name);
}

std::unique_ptr<mfq_amd_tensor> load_nvq(const uint8_t* blob, int64_t nbytes, int out_per_expert) {
    Reader in{blob, nbytes};
    const uint8_t* magic = in.take(4, "NVQ header");
    MFQ_REQUIRE(std::memcmp(magic, "NVQ1", 4) == 0 || std::memcmp(magic, "NIQ1", 4) == 0, "invalid NVQ magic");
    const int profile = in.get<uint8_t>("NVQ header");
    const int sub_bits = in.get<uint8_t>("NVQ header");
    const int gs = in.get<uint16_t>("NVQ header");
    const int axis = in.get<int32_t>("NVQ header");
    const int neuron_len = in.get<int32_t>("NVQ header");
    const uint32_t ndim = in.get<uint32_t>("NVQ header");
    MFQ_REQUIRE(ndim > 0 && ndim <= 8, "invalid NVQ ndim");
    std::vector<int64_t> shape(ndim);
    for (auto& d : shape) d = in.get<int64_t>("NVQ dimensions");
    const int64_t out = in.get<uint32_t>("NVQ dimensions");
    const bool jsc = profile & 0x20, custom = profile & 0x40, index_parity = profile & 0x80;
    const int codebook_id = profile & ~(0x80 | 0x40 | 0x20);
    int format = 0;
    if (jsc) format = codebook_id == 1 ? 5 : codebook_id == 2 ? 10 : codebook_id == 3 ? 12 : codebook_id == 4 ? 13
                    : codebook_id == 5 ? 14 : codebook_id == 6 ? 15 : 0;
    else format = codebook_id == 1 ? 2 : codebook_id == 2 ? 3 : 0;
    MFQ_REQUIRE(format != 0, "unsupported NVQ payload profile");
    MFQ_REQUIRE(gs == 24 && sub_bits >= 1 && sub_bits <= 4, "NVQ runtime requires gs24 and sub_bits in [1,4]");
    MFQ_REQUIRE(axis == 0 && ndim == 2 && shape[0] == out && shape[1] == neuron_len && neuron_len > 0,
                "NVQ runtime requires row-major rank-2 axis=0 weights");
    MFQ_REQUIRE(!(jsc && (custom || index_parity || sub_bits != 4)), "invalid NVQ-JSC profile flags");
    MFQ_REQUIRE(!index_parity || format == 2, "NVQ index parity requires NVQ2");
    const bool d4 = format == 3 || format == 10 || format == 12 || format == 15;
    const int dim = d4 ? 4 : 8;
    const int entries = format == 12 ? 512 : (format == 13 || format == 15) ? 1024 : format == 14 ? 4096 : 256;
    const int index_bits = format == 12 ? 9 : (format == 13 || format == 15) ? 10 : format == 14 ? 12 : 8;

    std::vector<uint8_t> metadata;
    bool group64 = false;   // one 64-bit record per 24-group instead of three streams (NVQ2J-XL only)
    if (jsc) {
        in.need(64, "NVQ-JSC metadata header");
        const uint8_t* header = blob + in.off;
        const int banks = header[1];
        MFQ_REQUIRE((header[0] == 1 || header[0] == 2) && (banks == 1 || banks == 2 || banks == 4) && header[2] == 16,
                    "unsupported NVQ-JSC metadata dimensions");
        // metadata version 2 marks the record storage (cpp_runtime/backends/cuda/ops/vq.cpp:1217-1227)
        if (header[0] == 1) {
            MFQ_REQUIRE(header[52] == 0, "invalid NVQ-JSC v1 storage layout");
        } else {
            MFQ_REQUIRE(format == 14 && header[52] == 1, "NVQ-JSC group64 storage requires NVQ2J-XL");
            group64 = true;
        }
        MFQ_REQUIRE(header[3] <= 1, "invalid NVQ-JSC state mode");
        for (int s = 0; s < 16; ++s) {
            uint16_t alpha;
            std::memcpy(&alpha, header + 4 + 2 * s, 2);
            MFQ_REQUIRE(!(alpha & 0x8000u) && (alpha & 0x7c00u) != 0x7c00u, "NVQ-JSC scale LUT must be finite and non-negative");
            MFQ_REQUIRE(header[36 + s] < banks, "NVQ-JSC state references a missing bank");
            if (header[3] == 1) {
                // analytic tables: the file must hold exactly the values the mode promises
                // (cpp_runtime/backends/cuda/ops/vq.cpp:1240-1256); all of them are exact in fp16
                const int rank = s / banks;
                const float expected = banks == 1 ? static_cast<float>(s)
                                     : dim == 4   ? static_cast<float>(rank + 1)
                                                  : 15.0f * static_cast<float>(rank + 1) / static_cast<float>(16 / banks);
                MFQ_REQUIRE(header[36 + s] == s % banks && half_to_float(alpha) == expected,
                            "invalid analytic NVQ-JSC state tables");
            }
        }
        for (int i = group64 ? 53 : 52; i < 64; ++i) MFQ_REQUIRE(header[i] == 0, "invalid NVQ-JSC reserved metadata bytes");
        const int64_t total = 64 + static_cast<int64_t>(banks) * entries * dim;
        const uint8_t* p = in.take(total, "NVQ-JSC metadata");
        for (int64_t i = 64; i < total; ++i) MFQ_REQUIRE(p[i] <= 127, "NVQ-JSC codebook value exceeds int8");
        for (int64_t word = 64; word < total; word += dim)
            MFQ_REQUIRE(std::any_of(p + word, p + word + dim, [](uint8_t v) { return v != 0; }),
                        "NVQ-JSC codeword must not be all zero");
        metadata.assign(p, p + total);
    } else if (custom) {
        const uint8_t* p = in.take(entries * 2, "NVQ custom codebook");
        std::vector<uint16_t> words(entries);
        std::memcpy(words.data(), p, entries * 2);
        metadata = as_bytes(expand_grid(words.data(), entries, dim, d4 ? 3 : 2));
    } else {
        int e, d;
        metadata = as_bytes(builtin_grid(d4 ? "d4_256" : "e8_256", e, d));
    }
    const int64_t ng = (neuron_len + 23) / 24, nvec = (neuron_len + dim - 1) / dim, nsign = (neuron_len + 7) / 8;
    MFQ_REQUIRE(out > 0, "NVQ tensor has no rows");
    in.need(checked_mul(out, 2, "NVQ neuron anchors"), "NVQ neuron anchors");
    std::vector<float> anchors(out);
    {
        const uint8_t* p = in.take(out * 2, "NVQ neuron anchors");
        for (int64_t r = 0; r < out; ++r) {
            uint16_t a;
            std::memcpy(&a, p + 2 * r, 2);
            MFQ_REQUIRE((a & 0x7c00u) != 0x7c00u && !(a & 0x8000u), "NVQ neuron anchors must be finite and non-negative");
            anchors[r] = half_to_float(a);
        }
    }
    const int64_t state_bytes = stream_bytes(checked_mul(out, ng, "NVQ state stream"), sub_bits);
    const int64_t index_bytes = stream_bytes(checked_mul(out, nvec, "NVQ index stream"), index_bits);
    const int64_t sign_bytes = stream_bytes(checked_mul(out, nsign, "NVQ sign stream"), 7);
    // the streams (or the records they are rebuilt from) must be present before anything of their size is allocated
    if (group64) in.need(checked_mul(checked_mul(out, ng, "NVQ group64 stream"), 8, "NVQ group64 stream"), "NVQ group64 stream");
    else in.need(state_bytes + index_bytes + sign_bytes, "NVQ streams");
    std::vector<uint8_t> unpacked[3];   // states, indices, signs rebuilt from records
    const uint8_t *states, *indices, *signs;
    if (group64) {
        // record = state << 60 | three segments of 20 bits: 12-bit index, 7 sign bits and their parity
        // (cpp_runtime/backends/cuda/ops/vq.cpp:1319-1361); the runtime layout is the three streams
        const int64_t records = out * ng;
        const uint8_t* p = in.take(checked_mul(records, 8, "NVQ group64 stream"), "NVQ group64 stream");
        unpacked[0].assign(static_cast<size_t>(state_bytes), 0);
        unpacked[1].assign(static_cast<size_t>(index_bytes), 0);
        unpacked[2].assign(static_cast<size_t>(sign_bytes), 0);
        const auto store = [](std::vector<uint8_t>& stream, int64_t bit, int bits, uint32_t value) {
            for (int i = 0; i < bits; ++i, ++bit)
                if ((value >> i) & 1u) stream[static_cast<size_t>(bit >> 3)] |= static_cast<uint8_t>(1u << (bit & 7));
        };
        for (int64_t linear = 0; linear < records; ++linear) {
            uint64_t record;
            std::memcpy(&record, p + 8 * linear, 8);
            store(unpacked[0], linear * sub_bits, sub_bits, static_cast<uint32_t>(record >> 60));
            const int64_t row = linear / ng, group = linear % ng;
            for (int local = 0; local < 3; ++local) {
                const uint32_t segment = static_cast<uint32_t>(record >> (20 * local)) & 0xfffffu;
                const uint32_t mask8 = segment >> 12;
                MFQ_REQUIRE((mask8 >> 7) == (static_cast<uint32_t>(__builtin_popcount(mask8 & 0x7fu)) & 1u),
                            "invalid NVQ-JSC group64 parity bit");
                const int64_t vector = group * 3 + local;
                if (vector >= nvec) {
                    MFQ_REQUIRE(segment == 0, "NVQ-JSC group64 padding must be zero");
                    continue;
                }
                store(unpacked[1], (row * nvec + vector) * index_bits, index_bits, segment & 0xfffu);
                store(unpacked[2], (row * nsign + vector) * 7, 7, mask8 & 0x7fu);
            }
        }
        states = unpacked[0].data(); indices = unpacked[1].data(); signs = unpacked[2].data();
    } else {
        states = in.take(state_bytes, "NVQ state stream");
        indices = in.take(index_bytes, "NVQ index stream");
        signs = in.take(sign_bytes, "NVQ sign stream");
    }
    MFQ_REQUIRE(in.off == nbytes, "invalid NVQ blob tail");

    auto t = std::make_unique<mfq_amd_tensor>();
    auto& g = t->geom;
    g.family = MFQ_AMD_FAMILY_NVQ;
    g.input_width = neuron_len; g.groups = static_cast<int32_t>(ng); g.group_size = 24;
    g.format = format; g.sub_bits = sub_bits; g.sign_mode = index_parity ? 1 : 0;
    g.nvec = static_cast<int32_t>(nvec); g.nsign = static_cast<int32_t>(nsign);
    if (out_per_expert > 0) {
        MFQ_REQUIRE(out % out_per_expert == 0, "invalid MFE NVQ expert geometry");
        g.local_experts = static_cast<int32_t>(out / out_per_expert); g.output_rows = out_per_expert;
    } else { g.local_experts = 1; g.output_rows = static_cast<int32_t>(out); }
    t->set_field(0, std::vector<uint8_t>(indices, indices + index_bytes));
    t->set_field(1, std::vector<uint8_t>(signs, signs + sign_bytes));
    t->set_field(2, std::vector<uint8_t>(states, states + state_bytes));
    t->set_field(3, as_bytes(anchors));
    t->set_field(4, std::move(metadata));
    return t;
}

// --------------------------------------------------------------- MXFP4 ----
std::unique_ptr<mfq_amd_tensor> load_mxfp4(const uint8_t* blob, int64_t nbytes, int out_per_expert) {
    Reader in{blob, nbytes};
    const uint8_t* magic = in.take(4, "MXFP4 header");
    MFQ_REQUIRE(std::memcmp(magic, "MXT1", 4) == 0, "invalid MX magic");
    const int version = in.get<uint8_t>("MXFP4 header");
    const int kind = in.get<uint8_t>("MXFP4 header");
    const int reserved = in.get<uint16_t>("MXFP4 header");
    uint64_t dims[6];
    for (auto& d : dims) d = in.get<uint64_t>("MXFP4 header");
    MFQ_REQUIRE(version == 1 && kind == 4 && reserved == 0, "not an MXFP4 payload");
    MFQ_REQUIRE(dims[0] <= (uint64_t(1) << 31) && dims[1] <= (uint64_t(1) << 31), "oversized MXFP4 geometry");
    const int64_t rows = static_cast<int64_t>(dims[0]), cols = static_cast<int64_t>(dims[1]);
    MFQ_REQUIRE(rows > 0 && cols > 0 && cols % 32 == 0 && dims[2] == dims[0] && dims[3] == dims[1] / 2 &&
                dims[4] == dims[0] && dims[5] == dims[1] / 32, "inconsistent MXFP4 geometry");
    const uint8_t* values = in.take(rows * cols / 2, "MXFP4 values");
    const uint8_t* scales = in.take(rows * cols / 32, "MXFP4 scales");
    MFQ_REQUIRE(in.off == nbytes, "invalid MXFP4 payload size");
    MFQ_REQUIRE(std::find(scales, scales + rows * cols / 32, uint8_t(255)) == scales + rows * cols / 32,
                "MXFP4 payload contains an E8M0 NaN scale");
    auto t = std::make_unique<mfq_amd_tensor>();
    auto& g = t->geom;
    g.family = MFQ_AMD_FAMILY_MXFP4;
    g.input_width = static_cast<int32_t>(cols); g.group_size = 32; g.groups = static_cast<int32_t>(cols / 32);
    if (out_per_expert > 0) {
        MFQ_REQUIRE(rows % out_per_expert == 0, "invalid MFE MXFP4 expert geometry");
        g.local_experts = static_cast<int32_t>(rows / out_per_expert); g.output_rows = out_per_expert;
    } else { g.local_experts = 1; g.output_rows = static_cast<int32_t>(rows); }
    t->set_field(0, std::vector<uint8_t>(values, values + rows * cols / 2));
    t->set_field(1, std::vector<uint8_t>(scales, scales + rows * cols / 32));
    return t;
}

// Family a stored dtype label belongs to: files carry the family name or one of the profile and
// older names the reference maps onto it (cpp_runtime/core/compat/mfq_format_compat.h:17-57).
std::string canonical_dtype(const std::string& dtype) {
    if (dtype == "NINTv2" || (dtype.size() == 5 && dtype.compare(0, 4, "NINT") == 0 && dtype[4] >= '1' && dtype[4] <= '8'))
        return "NINT";
    for (const char* name : {"NIQ2", "NIQ2J", "NIQ3", "NVQ2", "NVQ2J", "NVQ2J-L", "NVQ2J-XL", "NVQ3", "NVQ3J",
                             "NVQ3J-512", "NVQ3J-L"})
        if (dtype == name) return "NVQ";
    return dtype;
}

std::unique_ptr<mfq_amd_tensor> load_any(const std::string& stored_dtype, const uint8_t* blob, int64_t nbytes,
                                         int out_per_expert) {
    MFQ_REQUIRE(blob && nbytes > 0, "empty tensor payload");
    MFQ_REQUIRE(out_per_expert >= 0, "negative expert geometry");
    const std::string dtype = canonical_dtype(stored_dtype);
    if (dtype == "NINT") return load_nint(blob, nbytes, out_per_expert);
    if (dtype == "NVQ") return load_nvq(blob, nbytes, out_per_expert);
    if (dtype == "MXFP4") return load_mxfp4(blob, nbytes, out_per_expert);
    fail_unsupported("unsupported tensor dtype: " + dtype);
}

void upload(mfq_amd_tensor& t, const int32_t* expert_local, int experts) {
    if (!t.uploaded) {
        for (int i = 0; i < t.field_count; ++i) {
            if (t.host[i].empty()) continue;
            MFQ_HIP(hipMalloc(&t.dev[i], t.host[i].size()));
            MFQ_HIP(hipMemcpy(t.dev[i], t.host[i].data(), t.host[i].size(), hipMemcpyHostToDevice));
        }
        t.uploaded = true;
    }
    if (expert_local) {
        MFQ_REQUIRE(experts > 0, "expert map needs a positive expert count");
        if (t.dev_expert_local) { MFQ_HIP(hipFree(t.dev_expert_local)); t.dev_expert_local = nullptr; }
        MFQ_HIP(hipMalloc(reinterpret_cast<void**>(&t.dev_expert_local), sizeof(int32_t) * experts));
        MFQ_HIP(hipMemcpy(t.dev_expert_local, expert_local, sizeof(int32_t) * experts, hipMemcpyHostToDevice));
    }
}

}  // namespace

struct mfq_amd_mfe {
    int32_t experts = 0, out_per_expert = 0, neuron_len = 0;
    std::vector<std::unique_ptr<mfq_amd_tensor>> tensors;
    std::vector<std::vector<int32_t>> expert_ids;
};

extern "C" {

int mfq_amd_tensor_load(const char* dtype, const uint8_t* blob, int64_t nbytes, int32_t out_per_expert,
                        mfq_amd_tensor** out) {
    return guarded([&] {
        MFQ_REQUIRE(dtype && out, "null argument");
        *out = load_any(dtype, blob, nbytes, out_per_expert).release();
    });
}

int mfq_amd_tensor_host_view(const mfq_amd_tensor* tensor, mfq_amd_projection* view) {
    return guarded([&] {
        MFQ_REQUIRE(tensor && view, "null argument");
        tensor->fill_view(*view, false);
    });
}

int mfq_amd_tensor_upload(mfq_amd_tensor* tensor, const int32_t* expert_local_host, int32_t experts,
                          mfq_amd_projection* view) {
    return guarded([&] {
        MFQ_REQUIRE(tensor && view, "null argument");
        upload(*tensor, expert_local_host, experts);
        tensor->fill_view(*view, true);
    });
}

void mfq_amd_tensor_free(mfq_amd_tensor* tensor) { delete tensor; }

int mfq_amd_mfe_load(const uint8_t* blob, int64_t nbytes, mfq_amd_mfe** out) {
    return guarded([&] {
        MFQ_REQUIRE(blob && out, "null argument");
        Reader in{blob, nbytes};
        // "MFE1" and the older "NIM2" share one layout; "NIM1" pools have a short header and hold NINT only;
        // delta containers cover some experts only and are not full tensors
        // (cpp_runtime/backends/cuda/ops/moe.cpp:31-41, :55-61)
        const uint8_t* magic = in.take(4, "MFE header");
        MFQ_REQUIRE(std::memcmp(magic, "MFD1", 4) != 0 && std::memcmp(magic, "NID2", 4) != 0,
                    "MFE delta cannot be loaded as a full tensor");
        const bool short_pools = std::memcmp(magic, "NIM1", 4) == 0;
        MFQ_REQUIRE(short_pools || std::memcmp(magic, "MFE1", 4) == 0 || std::memcmp(magic, "NIM2", 4) == 0,
                    "invalid MFE magic");
        auto mfe = std::make_unique<mfq_amd_mfe>();
        mfe->experts = static_cast<int32_t>(in.get<uint32_t>("MFE header"));
        mfe->out_per_expert = static_cast<int32_t>(in.get<uint32_t>("MFE header"));
        mfe->neuron_len = static_cast<int32_t>(in.get<uint32_t>("MFE header"));
        const uint32_t pools = in.get<uint32_t>("MFE header");
        MFQ_REQUIRE(mfe->experts > 0 && mfe->out_per_expert > 0 && mfe->neuron_len > 0 && pools > 0 &&
                    pools <= static_cast<uint32_t>(mfe->experts), "invalid MFE header");
        std::vector<uint8_t> seen(mfe->experts, 0);
        for (uint32_t i = 0; i < pools; ++i) {
            const uint32_t count = in.get<uint32_t>("MFE pool header");
            const uint32_t dtype_len = short_pools ? 0 : in.get<uint32_t>("MFE pool header");
            const uint64_t payload_len = in.get<uint64_t>("MFE pool header");
            const uint64_t runtime_len = short_pools ? 0 : in.get<uint64_t>("MFE pool header");
            MFQ_REQUIRE(count > 0 && (short_pools || dtype_len > 0) && dtype_len <= 32, "invalid MFE pool header");
            MFQ_REQUIRE(count <= static_cast<uint32_t>(mfe->experts), "MFE pool lists more experts than the tensor has");
            in.need(int64_t(count) * 4, "MFE expert ids");
            std::vector<int32_t> ids(count);
            std::memcpy(ids.data(), in.take(int64_t(count) * 4, "MFE expert ids"), size_t(count) * 4);
            for (int32_t e : ids) {
                MFQ_REQUIRE(e >= 0 && e < mfe->experts && !seen[e], "MFE expert ids must be unique and in range");
                seen[e] = 1;
            }
            const std::string dtype = short_pools ? std::string("NINT")
                : std::string(reinterpret_cast<const char*>(in.take(dtype_len, "MFE dtype")), dtype_len);
            in.need_u64(runtime_len, "MFE runtime payload");
            (void)in.take(static_cast<int64_t>(runtime_len), "MFE runtime payload");
            in.need_u64(payload_len, "MFE tensor payload");
            const uint8_t* payload = in.take(static_cast<int64_t>(payload_len), "MFE tensor payload");
            auto tensor = load_any(dtype, payload, static_cast<int64_t>(payload_len), mfe->out_per_expert);
            MFQ_REQUIRE(tensor->geom.local_experts == static_cast<int32_t>(count) &&
                        tensor->geom.input_width == mfe->neuron_len, "MFE pool tensor does not match its header");
            mfe->tensors.push_back(std::move(tensor));
            mfe->expert_ids.push_back(std::move(ids));
        }
        MFQ_REQUIRE(in.off == nbytes, "invalid MFE trailing bytes");
        MFQ_REQUIRE(std::find(seen.begin(), seen.end(), 0) == seen.end(), "MFE pools do not cover every expert");
        *out = mfe.release();
    });
}

int mfq_amd_mfe_info(const mfq_amd_mfe* mfe, int32_t* experts, int32_t* out_per_expert, int32_t* neuron_len,
                     int32_t* pools) {
    return guarded([&] {
        MFQ_REQUIRE(mfe, "null argument");
        if (experts) *experts = mfe->experts;
        if (out_per_expert) *out_per_expert = mfe->out_per_expert;
        if (neuron_len) *neuron_len = mfe->neuron_len;
        if (pools) *pools = static_cast<int32_t>(mfe->tensors.size());
    });
}

int mfq_amd_mfe_pool(mfq_amd_mfe* mfe, int32_t index, mfq_amd_tensor** tensor, const int32_t** expert_ids,
                     int32_t* expert_count) {
    return guarded([&] {
        MFQ_REQUIRE(mfe && index >= 0 && index < static_cast<int32_t>(mfe->tensors.size()), "MFE pool index out of range");
        if (tensor) *tensor = mfe->tensors[index].get();
        if (expert_ids) *expert_ids = mfe->expert_ids[index].data();
        if (expert_count) *expert_count = static_cast<int32_t>(mfe->expert_ids[index].size());
    });
}

int mfq_amd_mfe_upload(mfq_amd_mfe* mfe, mfq_amd_projection* views, int32_t capacity) {
    return guarded([&] {
        MFQ_REQUIRE(mfe && views && capacity >= static_cast<int32_t>(mfe->tensors.size()), "view array is too small");
        for (size_t i = 0; i < mfe->tensors.size(); ++i) {
            std::vector<int32_t> local(mfe->experts, -1);
            for (size_t j = 0; j < mfe->expert_ids[i].size(); ++j) local[mfe->expert_ids[i][j]] = static_cast<int32_t>(j);
            upload(*mfe->tensors[i], local.data(), mfe->experts);
            mfe->tensors[i]->fill_view(views[i], true);
        }
    });
}

void mfq_amd_mfe_free(mfq_amd_mfe* mfe) { delete mfe; }

int mfq_amd_nvq_grid(const char* name, int8_t* out, int64_t capacity, int32_t* entries, int32_t* dim) {
    return guarded([&] {
        MFQ_REQUIRE(name && out, "null argument");
        int e = 0, d = 0;
        const auto grid = builtin_grid(name, e, d);
        MFQ_REQUIRE(capacity >= static_cast<int64_t>(grid.size()), "grid buffer is too small");
        std::memcpy(out, grid.data(), grid.size());
        if (entries) *entries = e;
        if (dim) *dim = d;
    });
}

}  // extern "C"
