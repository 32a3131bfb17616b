// Single-projection operators: whole-matrix dequantisation (the bit-exact gate for the
// decoders) and the dense streaming GEMV.
#include "common.h"
#include "decode.cuh"
#include "fast_rows.cuh"
#include "launch.cuh"
#include "moe_args.h"

namespace mfq_amd {
namespace dev {

// One thread per (row, chunk): eight fp32 weights to out[row, 8c .. 8c+8).
template <int CLS>
__global__ void __launch_bounds__(256) dequant_kernel(mfq_amd_projection p, int local_expert, float* out) {
    extern __shared__ unsigned char lds[];
    Decoder<CLS> dec;
    dec.init(p, lds);
    __syncthreads();
    const int chunks = (p.input_width + 7) / 8;
    const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= static_cast<int64_t>(p.output_rows) * chunks) return;
    const int row = static_cast<int>(index / chunks);
    const int c = static_cast<int>(index % chunks);
    typename Decoder<CLS>::Row r;
    dec.template row<false>(p, local_expert, row, r);
    float w[8];
    dec.chunk(r, c, w);
    float* dst = out + static_cast<int64_t>(row) * p.input_width + c * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        if (c * 8 + i < p.input_width) dst[i] = w[i];
}

struct DequantLaunch {
    mfq_amd_projection p; int local_expert; float* out; hipStream_t stream;
    template <int CLS> void run() const {
        const int chunks = (p.input_width + 7) / 8;
        const int64_t items = static_cast<int64_t>(p.output_rows) * chunks;
        const unsigned blocks = static_cast<unsigned>((items + 255) / 256);
        hipLaunchKernelGGL(dequant_kernel<CLS>, dim3(blocks), dim3(256), class_lds_bytes(CLS, p.format), stream,
                           p, local_expert, out);
    }
};

// Streaming GEMV.  A block is four waves; wave w owns RW consecutive rows.  Each lane keeps the
// activations of its CPL chunks (columns 8*(lane + 64 j) ...) in registers for NT tokens and walks
// the rows, so a weight byte is read once per pass and an activation once per block.
constexpr int kGemvRowsPerWave = 4;

template <int CLS, int NT, int CPL>
__global__ void __launch_bounds__(256) gemv_kernel(mfq_amd_projection p, int local_expert, const void* x,
                                                   int x_dtype, int batch, int64_t x_stride, float* y,
                                                   int64_t y_stride, int vector_ok) {
    extern __shared__ unsigned char lds[];
    Decoder<CLS> dec;
    dec.init(p, lds);
    __syncthreads();
    const int wave = uniform(static_cast<int>(threadIdx.x / kWave)), lane = threadIdx.x % kWave;
    const int row0 = (blockIdx.x * 4 + wave) * kGemvRowsPerWave;
    if (row0 >= p.output_rows) return;
    const int token0 = blockIdx.y * NT;
    const int chunks = (p.input_width + 7) / 8;
    const int element = x_dtype == MFQ_AMD_F32 ? 4 : 2;
    const int slabs = (chunks + kWave * CPL - 1) / (kWave * CPL);

    // Row descriptors first, then per slab the activations and the weights; indices are clamped
    // rather than branched on so the loads of a slab are issued together.
    typename Decoder<CLS>::Row rr[kGemvRowsPerWave];
    bool fast = true;
#pragma unroll
    for (int r = 0; r < kGemvRowsPerWave; ++r) {
        const int row = row0 + r < p.output_rows ? row0 + r : p.output_rows - 1;
        dec.row(p, local_expert, row, rr[r]);
        fast = fast && rr[r].fast;
    }
    float acc[kGemvRowsPerWave][NT];
#pragma unroll
    for (int r = 0; r < kGemvRowsPerWave; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = 0.0f;

    for (int slab = 0; slab < slabs; ++slab) {
        float xr[NT][CPL][8];
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                const int c = (slab * CPL + j) * kWave + lane;
                const int token = token0 + t < batch ? token0 + t : batch - 1;
                const char* row = static_cast<const char*>(x) + static_cast<int64_t>(token) * x_stride * element;
                load_x8(row, x_dtype, c < chunks ? c : chunks - 1, p.input_width, vector_ok != 0, xr[t][j]);
                const bool keep = c < chunks && token0 + t < batch;
#pragma unroll
                for (int i = 0; i < 8; ++i) xr[t][j][i] = keep ? xr[t][j][i] : 0.0f;
            }
        if (fast) {
            Raw raw[kGemvRowsPerWave][CPL];
#pragma unroll
            for (int r = 0; r < kGemvRowsPerWave; ++r)
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    const int c = (slab * CPL + j) * kWave + lane;
                    raw[r][j] = dec.fetch(rr[r], c < chunks ? c : chunks - 1);
                }
#pragma unroll
            for (int r = 0; r < kGemvRowsPerWave; ++r)
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    const int c = (slab * CPL + j) * kWave + lane;
                    float w[8];
                    dec.decode(rr[r], raw[r][j], c < chunks ? c : chunks - 1, w);
#pragma unroll
                    for (int t = 0; t < NT; ++t)
#pragma unroll
                        for (int i = 0; i < 8; ++i) acc[r][t] = fmaf(w[i], xr[t][j][i], acc[r][t]);
                }
        } else {
#pragma unroll
            for (int r = 0; r < kGemvRowsPerWave; ++r)
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    const int c = (slab * CPL + j) * kWave + lane;
                    float w[8];
                    dec.chunk(rr[r], c < chunks ? c : chunks - 1, w);
#pragma unroll
                    for (int t = 0; t < NT; ++t)
#pragma unroll
                        for (int i = 0; i < 8; ++i) acc[r][t] = fmaf(w[i], xr[t][j][i], acc[r][t]);
                }
        }
    }
#pragma unroll
    for (int r = 0; r < kGemvRowsPerWave; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float total = wave_sum(acc[r][t]);
            if (lane == 0 && row0 + r < p.output_rows && token0 + t < batch)
                y[static_cast<int64_t>(token0 + t) * y_stride + row0 + r] = total;
        }
}

struct GemvLaunch {
    mfq_amd_projection p; int local_expert; const void* x; int x_dtype; int batch; int64_t x_stride;
    float* y; int64_t y_stride; int vector_ok; hipStream_t stream;
    template <int CLS, int NT, int CPL> void go() const {
        const unsigned row_blocks = (p.output_rows + 4 * kGemvRowsPerWave - 1) / (4 * kGemvRowsPerWave);
        hipLaunchKernelGGL((gemv_kernel<CLS, NT, CPL>), dim3(row_blocks, (batch + NT - 1) / NT), dim3(256),
                           class_lds_bytes(CLS, p.format), stream, p, local_expert, x, x_dtype, batch, x_stride,
                           y, y_stride, vector_ok);
    }
    template <int CLS> void run() const {
        const bool narrow = (p.input_width + 7) / 8 <= kWave;
        if (batch == 1) { if (narrow) go<CLS, 1, 1>(); else go<CLS, 1, 4>(); }
        else { if (narrow) go<CLS, 4, 1>(); else go<CLS, 4, 4>(); }
    }
};

// Streaming GEMV on the decode row loop (fast_rows.cuh): a block covers 4 * SLOTS * (64 / LPR) rows of
// NT tokens (blockIdx.y walks the token groups), so a row is decoded once per NT tokens; the same row tile
// of neighbouring groups lands on the same XCD when the number of row tiles is a multiple of eight, so the
// weights are read from HBM once.  A group that reaches beyond the batch repeats the last token and
// stores nothing for the repeats.
template <int CLS, int LPR, int SLABS, int SLOTS, int NT>
__global__ void __launch_bounds__(256) gemv_fast_kernel(mfq_amd_projection p, int local_expert, const void* x,
                                                        int x_dtype, int batch, int64_t x_stride, float* y,
                                                        int64_t y_stride, int vector_ok) {
    extern __shared__ unsigned char lds[];
    // LDS: the tables of an NVQ pool | scale per token, a float per wave | the packed rows of the block's tokens
    unsigned char* x_area = lds + (FastClass<CLS>::kNvq ? kNvqFastLdsBytes : 0);
    float* x_up = reinterpret_cast<float*>(x_area);
    float* x_scratch = x_up + 8;
    uint32_t* x_rows = reinterpret_cast<uint32_t*>(x_area + 64);
    const int lane_blocks = (p.input_width + kLaneColumns - 1) / kLaneColumns;
    const int element = x_dtype == MFQ_AMD_F32 ? 4 : 2;
    const int first = blockIdx.y * NT;
    // Behind the first requests for packed rows (every wave of the block takes part: there are barriers inside) the
    // block builds the LDS tables of an NVQ pool and packs the activation rows of its tokens, once for its four
    // waves: a wave that packs its own copy spends more instructions on that than on the rows it multiplies.
    auto prologue = [&] {
        if (FastClass<CLS>::kNvq) {
            nvq_fast_tables(p, lds);
            __syncthreads();
        }
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            const int token = first + n < batch ? first + n : batch - 1;
            stage_x_row<CLS>(static_cast<const char*>(x) + static_cast<int64_t>(token) * x_stride * element, x_dtype,
                             vector_ok != 0, p.input_width, x_rows + n * lane_blocks * kXStagedDwords, x_up + n, x_scratch);
        }
    };
    const FastCtx<CLS> ctx = fast_ctx<CLS>(p, local_expert, lds);
    constexpr int kRowsPerWave = SLOTS * (kWave / LPR);
    const int wave = uniform(static_cast<int>(threadIdx.x / kWave));
    const int row_begin = (blockIdx.x * 4 + wave) * kRowsPerWave;
    if (row_begin >= p.output_rows) { prologue(); return; }
    const int row_end = row_begin + kRowsPerWave < p.output_rows ? row_begin + kRowsPerWave : p.output_rows;
    constexpr int kRing = SLABS > 1 ? (SLOTS < 4 ? SLOTS : 4) : (FastClass<CLS>::kRing < SLOTS ? FastClass<CLS>::kRing : SLOTS);
    XSource xs[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) xs[n] = XSource{x_rows + n * lane_blocks * kXStagedDwords, x_dtype, false, x_up + n};
    fast_rows<CLS, LPR, SLABS, NT, kRing, kXStaged, SLOTS>(ctx, xs, p.input_width, row_begin, row_end, p.output_rows,
        [&](int n, int row, float value) { if (first + n < batch) y[static_cast<int64_t>(first + n) * y_stride + row] = value; }, prologue);
}

struct GemvFastLaunch {
    mfq_amd_projection p; int local_expert; const void* x; int x_dtype; int batch; int64_t x_stride;
    float* y; int64_t y_stride; int vector_ok; hipStream_t stream;
    template <int CLS, int LPR, int SLABS, int SLOTS> void go() const {
        constexpr int kRowsPerBlock = 4 * SLOTS * (kWave / LPR);
        const unsigned blocks = (p.output_rows + kRowsPerBlock - 1) / kRowsPerBlock;
        const int lane_blocks = (p.input_width + kLaneColumns - 1) / kLaneColumns;
        auto lds_bytes = [&](int tokens) { return (FastClass<CLS>::kNvq ? kNvqFastLdsBytes : 0) + 64 + tokens * lane_blocks * kXStagedDwords * 4; };
        // Two tokens per block where decoding a row costs more than reading it again: NVQ rows of two slabs
        // (measured at 4096 x 4096: batch 16 in 38 us instead of 57 us; the other classes lose parallelism
        // and run slower in groups).
        if constexpr (FastClass<CLS>::kNvq && SLABS > 1) {
            if (batch >= 2) {
                hipLaunchKernelGGL((gemv_fast_kernel<CLS, LPR, SLABS, SLOTS, 2>), dim3(blocks, (batch + 1) / 2), dim3(256), lds_bytes(2),
                                   stream, p, local_expert, x, x_dtype, batch, x_stride, y, y_stride, vector_ok);
                return;
            }
        }
        hipLaunchKernelGGL((gemv_fast_kernel<CLS, LPR, SLABS, SLOTS, 1>), dim3(blocks, batch), dim3(256), lds_bytes(1), stream, p,
                           local_expert, x, x_dtype, batch, x_stride, y, y_stride, vector_ok);
    }
    template <int CLS> void run() const {
        if constexpr (fast_class(CLS)) {
            // 16 rows per wave where that still gives a few blocks per CU, else 4
            const int group = FastClass<CLS>::kNvq && p.input_width > kWave * kLaneColumns ? 2 : 1;   // tokens per block, as in go()
            // (NVQ, 4096 x 4096, batch 8 in two-token groups: 20.7 us with 8 rows per wave, 27.0 us with 4; batch 4: 16.4 / 15.6)
            const int64_t enough = FastClass<CLS>::kNvq ? 64 * 256 : 64 * 512;
            const bool tall = static_cast<int64_t>(p.output_rows) * ((batch + group - 1) / group) >= enough;
            if (p.input_width <= 16 * kLaneColumns) { if (tall) go<CLS, 16, 1, 8>(); else go<CLS, 16, 1, 4>(); }
            else if (p.input_width <= kWave * kLaneColumns) { if (tall) go<CLS, 64, 1, 16>(); else go<CLS, 64, 1, 4>(); }
            else {
                // (NVQ, 4096 x 4096, one token group: 8.5 us with 2 rows per wave, 9.2 us with 4; two groups: 19.2 / 14.2;
                // NINT4: 6.7 / 6.2 us.  Four tokens per block instead of two: batch 8 in 20.9 us against 20.3.)
                const bool one_group = (batch + group - 1) / group == 1;
                if (tall) go<CLS, 64, 2, 8>();
                else if (FastClass<CLS>::kNvq && one_group) go<CLS, 64, 2, 2>();
                else go<CLS, 64, 2, 4>();
            }
        }
    }
};

}  // namespace dev
}  // namespace mfq_amd

using namespace mfq_amd;

extern "C" int mfq_amd_dequant(const mfq_amd_projection* proj, int32_t local_expert, float* out_dev, void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(proj, "null argument");
        const mfq_amd_projection p = canonical_projection(*proj);
        validate_projection(p, local_expert);
        MFQ_REQUIRE(out_dev, "null argument");
        dev::DequantLaunch launch{p, local_expert, out_dev, as_stream(stream)};
        dev::dispatch_class(projection_class(p), launch);
        check_launch("dequant_kernel");
    });
}

extern "C" int mfq_amd_gemv(const mfq_amd_projection* proj, int32_t local_expert, const void* x_dev, int32_t x_dtype,
                            int32_t batch, int64_t x_stride, float* y_dev, int64_t y_stride, void* stream) {
    return guarded([&] {
        MFQ_REQUIRE(proj && x_dev && y_dev, "null argument");
        const mfq_amd_projection canonical = canonical_projection(*proj);
        proj = &canonical;
        validate_projection(*proj, local_expert);
        MFQ_REQUIRE(x_dtype >= MFQ_AMD_F32 && x_dtype <= MFQ_AMD_BF16, "unknown activation dtype");
        // same geometry rule as packed_nint_matmul (cpp_runtime/backends/cpu/ops/packed_nint.cpp:98-100)
        MFQ_REQUIRE(batch >= 0 && x_stride >= proj->input_width && y_stride >= proj->output_rows,
                    "invalid activation geometry");
        if (batch == 0) return;
        const int element = x_dtype == MFQ_AMD_F32 ? 4 : 2;
        const int vector_ok = reinterpret_cast<uintptr_t>(x_dev) % 16 == 0 && (x_stride * element) % 16 == 0;
        // the streaming row loop where the geometry allows it, the exact decoders otherwise
        if (x_dtype != MFQ_AMD_F32 && proj->input_width <= 2 * dev::kWave * dev::kLaneColumns && pool_fast_layout(*proj)) {
            dev::GemvFastLaunch launch{*proj, local_expert, x_dev, x_dtype, batch, x_stride, y_dev, y_stride, vector_ok,
                                       as_stream(stream)};
            dev::dispatch_class(projection_class(*proj), launch);
            check_launch("gemv_fast_kernel");
            return;
        }
        dev::GemvLaunch launch{*proj, local_expert, x_dev, x_dtype, batch, x_stride, y_dev, y_stride, vector_ok,
                               as_stream(stream)};
        dev::dispatch_class(projection_class(*proj), launch);
        check_launch("gemv_kernel");
    });
}
