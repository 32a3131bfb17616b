/* C++ host side above the C ABI of mfq_amd.h: the classes a C++ runtime holds for the mixed-format MoE
 * expert FFN, named and shaped after the ones they stand in for in the reference runtime.
 *
 *   mfq_amd::MixedMoeRuntime   one logical [experts, out, in] tensor stored as per-format pools, loaded from an
 *                              MFE container and resident on the device; forward() is one projection of routed
 *                              pairs (cpp_runtime/backends/cuda/ops/include/moe.h:133-189, MixedMoeRuntime).
 *   mfq_amd::MfeFfnRuntime     the fused routed FFN over three such tensors; built once per layer, run() per step
 *                              (cpp_runtime/backends/cuda/ops/include/mfe_ffn_runtime.h:9-97, MfeFfnRuntime, whose
 *                              constructor also takes the array of its three MixedMoeRuntime projections).
 *   mfq_amd::moe_topk          softmax top-k (moe_topk_cuda, mfq/kernels/cuda/moe.cu:1953-2079).
 *
 * Header-only, C++17, no dependency beyond the C ABI; device memory and streams stay the caller's (plain
 * pointers and a void* stream, as in the C ABI).  A failed call throws mfq_amd::Error with the library's
 * message, the way the reference's MFQ_RUNTIME_CHECK throws std::runtime_error. */
#ifndef MFQ_AMD_HPP
#define MFQ_AMD_HPP

#include <array>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "mfq_amd.h"

namespace mfq_amd {

class Error : public std::runtime_error {
public:
    Error(int status, const std::string& message) : std::runtime_error(message), status_(status) {}
    int status() const noexcept { return status_; }   /* one of the MFQ_AMD_ERR_* codes */
private:
    int status_;
};

inline void check(int status) {
    if (status != MFQ_AMD_OK) {
        const char* message = mfq_amd_last_error();
        throw Error(status, message && *message ? message : "mfq_amd call failed");
    }
}

/* One mixed-format expert tensor on the device. */
class MixedMoeRuntime {
public:
    /* blob: an MFE container (magics and dtype labels as the reference's unpack_mfe accepts them).  Parses on
     * the host, then uploads every pool to the current device. */
    MixedMoeRuntime(const std::uint8_t* blob, std::int64_t nbytes) {
        check(mfq_amd_mfe_load(blob, nbytes, &mfe_));
        try {
            std::int32_t pools = 0;
            check(mfq_amd_mfe_info(mfe_, &experts_, &out_per_expert_, &neuron_len_, &pools));
            views_.resize(static_cast<std::size_t>(pools));
            check(mfq_amd_mfe_upload(mfe_, views_.data(), pools));
        } catch (...) {
            mfq_amd_mfe_free(mfe_);
            throw;
        }
    }
    explicit MixedMoeRuntime(const std::vector<std::uint8_t>& blob)
        : MixedMoeRuntime(blob.data(), static_cast<std::int64_t>(blob.size())) {}
    MixedMoeRuntime(const MixedMoeRuntime&) = delete;
    MixedMoeRuntime& operator=(const MixedMoeRuntime&) = delete;
    MixedMoeRuntime(MixedMoeRuntime&& other) noexcept { swap(other); }
    MixedMoeRuntime& operator=(MixedMoeRuntime&& other) noexcept { swap(other); return *this; }
    ~MixedMoeRuntime() { if (mfe_) mfq_amd_mfe_free(mfe_); }

    int experts() const noexcept { return experts_; }
    int out_per_expert() const noexcept { return out_per_expert_; }
    int neuron_len() const noexcept { return neuron_len_; }
    int pool_count() const noexcept { return static_cast<int>(views_.size()); }
    /* Global expert ids owned by pool `index`. */
    std::vector<std::int32_t> pool_experts(int index) const {
        const std::int32_t* ids = nullptr;
        std::int32_t count = 0;
        check(mfq_amd_mfe_pool(mfe_, index, nullptr, &ids, &count));
        return std::vector<std::int32_t>(ids, ids + count);
    }
    /* The descriptor the C ABI takes; valid while this object lives. */
    mfq_amd_moe_tensor tensor() const noexcept {
        return mfq_amd_moe_tensor{views_.data(), static_cast<std::int32_t>(views_.size()), experts_, out_per_expert_,
                                  neuron_len_};
    }
    static std::int64_t workspace_bytes(int tokens, int top_k, int experts) {
        return mfq_amd_grouped_matmul_workspace(tokens, top_k, experts);
    }
    /* out_f16[tokens, k, out_per_expert] = W[ids[t, r]] . x; x is [tokens, K] (x_rows_per_token 1) or
     * [tokens, k, K] (x_rows_per_token k).  All pointers are device memory. */
    void forward(const void* x, int x_dtype, int x_rows_per_token, const std::int32_t* ids, int tokens, int top_k,
                 void* out_f16, void* workspace, std::int64_t workspace_nbytes, void* stream) const {
        const mfq_amd_moe_tensor t = tensor();
        check(mfq_amd_grouped_matmul(&t, x, x_dtype, x_rows_per_token, ids, tokens, top_k, out_f16, workspace,
                                     workspace_nbytes, stream));
    }

private:
    void swap(MixedMoeRuntime& other) noexcept {
        std::swap(mfe_, other.mfe_);
        std::swap(views_, other.views_);
        std::swap(experts_, other.experts_);
        std::swap(out_per_expert_, other.out_per_expert_);
        std::swap(neuron_len_, other.neuron_len_);
    }
    mfq_amd_mfe* mfe_ = nullptr;
    std::vector<mfq_amd_projection> views_;
    std::int32_t experts_ = 0, out_per_expert_ = 0, neuron_len_ = 0;
};

struct MfeFfnOptions {
    int top_k = 1;
    int max_tokens = 1;
    int x_dtype = MFQ_AMD_BF16;
    int out_dtype = MFQ_AMD_F32;
    float swiglu_limit = 0.0f;
    int decode_token_limit = 0;   /* 0 = the library's default */
    int launch_mode = 0;
    int expert_activation = 0;    /* 1: relu(up)^2, the gate projection is then a null pointer */
    bool mx_scaled_mfma = false;  /* prefill tiles of MXFP4 pools on the block-scaled MFMA (an experiment) */
};

/* The routed FFN of one layer: gate and up per routed pair, SwiGLU, down per pair, route-weighted reduce. */
class MfeFfnRuntime {
public:
    /* projections = {gate, up, down}; they must outlive this object (their device buffers are borrowed). */
    MfeFfnRuntime(const std::array<const MixedMoeRuntime*, 3>& projections, const MfeFfnOptions& options)
        : top_k_(options.top_k), max_tokens_(options.max_tokens) {
        const bool gated = options.expert_activation == 0;
        if (!projections[1] || !projections[2] || (projections[0] != nullptr) != gated)
            throw Error(MFQ_AMD_ERR_INVALID, "MfeFfnRuntime needs up and down projections, and gate exactly for the gated activation");
        mfq_amd_moe_ffn_config config{};
        if (gated) config.gate = projections[0]->tensor();
        config.up = projections[1]->tensor();
        config.down = projections[2]->tensor();
        config.top_k = options.top_k;
        config.max_tokens = options.max_tokens;
        config.x_dtype = options.x_dtype;
        config.out_dtype = options.out_dtype;
        config.swiglu_limit = options.swiglu_limit;
        config.decode_token_limit = options.decode_token_limit;
        config.launch_mode = options.launch_mode;
        config.expert_activation = options.expert_activation;
        config.mx_scaled_mfma = options.mx_scaled_mfma ? 1 : 0;
        check(mfq_amd_moe_ffn_create(&config, &ffn_));
    }
    MfeFfnRuntime(const MfeFfnRuntime&) = delete;
    MfeFfnRuntime& operator=(const MfeFfnRuntime&) = delete;
    ~MfeFfnRuntime() { if (ffn_) mfq_amd_moe_ffn_destroy(ffn_); }

    int top_k() const noexcept { return top_k_; }
    int max_tokens() const noexcept { return max_tokens_; }

    /* out[tokens, hidden] from x[tokens, hidden], ids i32 [tokens, k], route weights f32 [tokens, k]; device
     * pointers; allocates nothing and does not synchronise. */
    void run(const void* x, const std::int32_t* ids, const float* route_weights, int tokens, void* out, void* stream) {
        check(mfq_amd_moe_ffn_run(ffn_, x, ids, route_weights, tokens, out, stream));
    }
    /* The same with the softmax top-k of logits[tokens, experts] selected inside (moe_topk_cuda followed by
     * MfeFfnRuntime::run in the reference). */
    void run_logits(const void* x, const void* logits, int logits_dtype, int tokens, void* out, void* stream,
                    bool normalize = true, float norm_floor = 1e-20f, float scale = 1.0f) {
        check(mfq_amd_moe_ffn_run_logits(ffn_, x, logits, logits_dtype, normalize ? 1 : 0, norm_floor, scale, tokens, out,
                                         stream));
    }
    /* The same from x and the router weights[experts, hidden]: the router matmul runs in front. */
    void run_router(const void* x, const void* router, int router_dtype, int tokens, void* out, void* stream,
                    bool normalize = true, float norm_floor = 1e-20f, float scale = 1.0f) {
        check(mfq_amd_moe_ffn_run_router(ffn_, x, router, router_dtype, normalize ? 1 : 0, norm_floor, scale, tokens, out, stream));
    }
    /* The layer's shared expert (MfeFfnBatch::shared): dense projections with one expert each; gate is null for
     * shared_activation 1.  The descriptors are copied, their device buffers stay borrowed. */
    void set_shared(const mfq_amd_projection* gate, const mfq_amd_projection* up, const mfq_amd_projection* down,
                    int shared_activation = 0) {
        check(mfq_amd_moe_ffn_set_shared(ffn_, gate, up, down, shared_activation));
    }
    /* run() plus the shared expert: out = half(routed) + shared_ffn(x) * shared_gate[token] (one evaluated gate value per
     * token, of shared_gate_dtype). */
    void run_shared(const void* x, const std::int32_t* ids, const float* route_weights, const void* shared_gate,
                    int shared_gate_dtype, int tokens, void* out, void* stream) {
        check(mfq_amd_moe_ffn_run_shared(ffn_, x, ids, route_weights, shared_gate, shared_gate_dtype, tokens, out, stream));
    }
    /* Device pointers to the routes run_logits selected: ids i32 [tokens, k], weights f32 [tokens, k]. */
    std::pair<const std::int32_t*, const float*> routes() {
        const std::int32_t* ids = nullptr;
        const float* weights = nullptr;
        check(mfq_amd_moe_ffn_routes(ffn_, &ids, &weights));
        return {ids, weights};
    }
    mfq_amd_moe_ffn* handle() noexcept { return ffn_; }

private:
    mfq_amd_moe_ffn* ffn_ = nullptr;
    int top_k_, max_tokens_;
};

/* Softmax top-k with selected-weight normalisation: ids descending by weight, ties to the lower id. */
inline void moe_topk(const void* logits, int logits_dtype, int tokens, int experts, int top_k, std::int32_t* ids,
                     float* weights, void* stream, bool normalize = true, float norm_floor = 1e-20f, float scale = 1.0f) {
    check(mfq_amd_topk(logits, logits_dtype, tokens, experts, top_k, normalize ? 1 : 0, norm_floor, scale, ids, weights,
                       stream));
}

}  // namespace mfq_amd

#endif /* MFQ_AMD_HPP */
