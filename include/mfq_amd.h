/*
 * mfq_amd.h -- C ABI of the MI355X (gfx950) implementation of MFQ's mixed-format
 * quantised MoE expert FFN.
 *
 * Every entry point returns an int status (MFQ_AMD_OK or a negative code), never
 * throws, and keeps a thread-local message readable with mfq_amd_last_error().
 * Pointers named *_dev are device pointers; all storage is borrowed for the
 * duration of the call (host side) or until the stream reaches the end of the
 * enqueued work (device side).  `stream` is a hipStream_t passed as void*
 * (NULL = the default stream); no entry point synchronises the stream unless its
 * comment says so.
 *
 * Descriptors mirror the reference runtime's packed-weight layout so that the
 * reference loader's device buffers can be passed through unchanged.  Reference
 * citations are paths inside the MFQ checkout.
 */
#ifndef MFQ_AMD_H
#define MFQ_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MFQ_AMD_OK 0
#define MFQ_AMD_ERR_INVALID (-1)      /* bad argument / malformed descriptor or blob (reference: std::invalid_argument) */
#define MFQ_AMD_ERR_RUNTIME (-2)      /* HIP call or launch failed (reference: std::runtime_error) */
#define MFQ_AMD_ERR_UNSUPPORTED (-3)  /* valid, but not implemented by this build */

enum { MFQ_AMD_FAMILY_NINT = 1, MFQ_AMD_FAMILY_NVQ = 2, MFQ_AMD_FAMILY_MXFP4 = 3 };
enum { MFQ_AMD_F32 = 0, MFQ_AMD_F16 = 1, MFQ_AMD_BF16 = 2 };

/*
 * One pool (homogeneous cohort) of one projection.
 * Replaces mfq::cuda::MfePackedProjection (mfq/kernels/cuda/mfe_ffn.h:9-35); field
 * meaning per family as filled by pool_view (cpp_runtime/backends/cuda/ops/mfe_ffn.cpp:32-82):
 *
 *  NINT   fields[0] q stream u8 [local_experts, q_expert_stride] (rows bit-contiguous, 8 guard bytes)
 *         fields[1] row_q_bits u8 [rows]        fields[2] row_q_bit_offsets i64 [rows] (expert-relative)
 *         fields[3] sub_scale u8 [rows, groups] fields[4] sub_min u8 [rows, groups]
 *         fields[5] neuron_scale f32 [rows]     fields[6] neuron_min f32 [rows]
 *         sizes[0] = bytes of fields[0]
 *  NVQ    fields[0] index bit stream  fields[1] 7-bit sign-mask stream  fields[2] state stream
 *         fields[3] anchors f32 [rows]
 *         fields[4] metadata i8: format 2/3 = [256][dim] table; JSC formats = 64-byte header + banks
 *         sizes[0..2] = bytes of fields[0..2]; streams are flat over all rows of the pool
 *         format = the loader's runtime format id (cuda/ops/vq.cpp:1047-1071): 2 NVQ2, 3 NVQ3, 5 NVQ2J, 10 NVQ3J,
 *         12 NVQ3J-512, 13 NVQ2J-L, 14 NVQ2J-XL (banks read from fields[4] in place: 4-byte aligned), 15 NVQ3J-L;
 *         11, which the reference's loader writes for an NVQ3J pool with analytic two-bank tables
 *         (vq.cpp:1695-1700), is taken as 10.  Other ids return MFQ_AMD_ERR_UNSUPPORTED.
 *  MXFP4  fields[0] nibbles u8 [rows, width/2]  fields[1] E8M0 u8 [rows, width/32]
 *
 * rows = local_experts * output_rows; row of (local expert l, neuron r) = l*output_rows + r.
 * expert_local: i32 [experts] global expert -> local index in this pool, -1 = absent; may be
 * NULL for a dense (single expert) tensor.
 */
typedef struct mfq_amd_projection {
    const void* fields[9];
    int64_t sizes[3];
    const int32_t* expert_local;
    int32_t family;
    int32_t local_experts, output_rows, input_width, groups, group_size;
    int32_t format, sub_bits, sign_mode, nvec, nsign;
    int32_t uniform_bits;      /* NINT: q width shared by every row, 0 = mixed (NintWeight::uniform_qbits, ops/include/nint.h:63).
                                * Non-zero also promises that row r of an expert starts at bit
                                * r*groups*group_size*uniform_bits of the expert's stream (what the reference
                                * loader produces for a single-width tensor); the streaming decode kernels rely
                                * on it.  Set it to 0 for any other arrangement: the exact kernels then read
                                * fields[1] and fields[2] per row. */
    int64_t q_expert_stride;   /* NINT: bytes between expert streams; 0 for a dense tensor */
    int64_t reserved[2];
} mfq_amd_projection;

const char* mfq_amd_last_error(void);
int mfq_amd_abi_version(void);
/* One-time set-up of the current device: the SwiGLU sigmoid table (the reference builds the same table once per
 * process with moe_swiglu_sigmoid_table_cuda, mfq/kernels/cuda/moe.cu:2657-2665) and the dynamic-LDS limits of the
 * kernels that need more than 64 KB.  Allocates and synchronises.  Optional: mfq_amd_moe_ffn_create, and the first
 * call on a device of mfq_amd_swiglu, of a route plan over more than 1024 pairs or of a prefill-sized projection do
 * it themselves (thread-safe), so call it beforehand when that first call would sit inside a stream capture. */
int mfq_amd_init(void);

/* ---------------------------------------------------------------------------
 * Loading: canonical blob -> runtime packed layout.
 * Replaces unpack_nint / to_device_mfe_nint (cpp_runtime/backends/cuda/ops/nint.cpp:750-964, :1384-1459),
 * unpack_nvq / to_device_nvq (ops/vq.cpp:1030-1330, :1660-1760), unpack_mxfp4 (ops/mx.cpp) and
 * unpack_mfe_impl (ops/moe.cpp:25-182).
 * ------------------------------------------------------------------------- */
typedef struct mfq_amd_tensor mfq_amd_tensor;   /* owns the host (and, once uploaded, device) buffers of one pool */

/* dtype: "NINT", "NVQ" or "MXFP4".  out_per_expert = 0 loads a dense tensor; otherwise the
 * tensor's rows are local_experts * out_per_expert and NINT q codes are re-streamed per expert.
 * NINT blobs are read in both storages of the reference's loader: per-row widths (first byte has bit 7 set)
 * and the uniform bit-packed streams of older files (nint.cpp:758, :873-875, :927-958). */
int mfq_amd_tensor_load(const char* dtype, const uint8_t* blob, int64_t nbytes, int32_t out_per_expert,
                        mfq_amd_tensor** out);
/* Host-pointer view (for CPU-side checks); expert_local is NULL. */
int mfq_amd_tensor_host_view(const mfq_amd_tensor* tensor, mfq_amd_projection* view);
/* Copies every field to the current device (hipMalloc + synchronous hipMemcpy) once and fills a
 * device-pointer view.  expert_local_host (i32 [experts]) may be NULL. */
int mfq_amd_tensor_upload(mfq_amd_tensor* tensor, const int32_t* expert_local_host, int32_t experts,
                          mfq_amd_projection* view);
void mfq_amd_tensor_free(mfq_amd_tensor* tensor);

/* MFE container: header + per-pool records (mfq/formats/io.py:486-493, :723-760).  As unpack_mfe
 * (cpp_runtime/backends/cuda/ops/moe.cpp:25-185) it reads the magics "MFE1", "NIM2" (same layout) and "NIM1"
 * (short pool headers, NINT only), maps the older and per-profile dtype labels onto their family
 * (core/compat/mfq_format_compat.h:17-57), rejects delta containers ("MFD1", "NID2") and requires every
 * expert to be owned by exactly one pool. */
typedef struct mfq_amd_mfe mfq_amd_mfe;
int mfq_amd_mfe_load(const uint8_t* blob, int64_t nbytes, mfq_amd_mfe** out);
int mfq_amd_mfe_info(const mfq_amd_mfe* mfe, int32_t* experts, int32_t* out_per_expert, int32_t* neuron_len,
                     int32_t* pools);
/* Pool `index`: its tensor (owned by the container) and its global expert ids. */
int mfq_amd_mfe_pool(mfq_amd_mfe* mfe, int32_t index, mfq_amd_tensor** tensor, const int32_t** expert_ids,
                     int32_t* expert_count);
/* Uploads every pool; views[pools] receive device descriptors with expert_local maps. */
int mfq_amd_mfe_upload(mfq_amd_mfe* mfe, mfq_amd_projection* views, int32_t capacity);
void mfq_amd_mfe_free(mfq_amd_mfe* mfe);

/* The built-in lattice tables (mfq/formats/nvq.py:56-264): name in {"e8_256","d4_256","d4_512","d4_1024",
 * "e8_1024"}; writes entries*dim int8 values. */
int mfq_amd_nvq_grid(const char* name, int8_t* out, int64_t capacity, int32_t* entries, int32_t* dim);

/* ---------------------------------------------------------------------------
 * Single-projection operators.
 * ------------------------------------------------------------------------- */

/* Dense fp32 weights of one local expert, out_dev[output_rows, input_width], bit-exact with the
 * reference dequantiser.  Replaces nint_decode_f32_cuda (backends/cuda/include/mfq_cuda_quant_ops.h:97-102;
 * kernel mfq/kernels/cuda/nint_matmul.cu:120-156), nvq_dequant_kernel (nvq_matmul.cu:36-92) and
 * mxfp4_dequant_kernel (mx_matmul.cu:715). */
int mfq_amd_dequant(const mfq_amd_projection* proj, int32_t local_expert, float* out_dev, void* stream);

/* y[b, r] = sum_c W[r, c] * x[b, c] for one local expert; fp32 accumulate, original (unquantised)
 * activations.  x_dev[batch, x_stride] of x_dtype, y_dev[batch, y_stride] fp32.
 * Replaces nint_matmul / nvq_matmul / mxfp4_matmul (ops/include/nint.h:74-77, vq.h:71-74, mx.h:41-42)
 * with the numerics of the CPU path (backends/cpu/ops/packed_nint.h:31-37). */
int mfq_amd_gemv(const mfq_amd_projection* proj, int32_t local_expert, const void* x_dev, int32_t x_dtype,
                 int32_t batch, int64_t x_stride, float* y_dev, int64_t y_stride, void* stream);

/* ---------------------------------------------------------------------------
 * Routing.
 * ------------------------------------------------------------------------- */

/* logits_dev[tokens, experts] = x_dev[tokens, width] . router_dev[experts, width]^T, fp32, columns
 * accumulated in ascending order per output (stands in for the cuBLAS call at
 * cpp_runtime/backends/cuda/core/ffn.cpp:443-447 with a reproducible summation order). */
int mfq_amd_router_logits(const void* x_dev, int32_t x_dtype, const void* router_dev, int32_t router_dtype,
                          int32_t tokens, int32_t experts, int32_t width, float* logits_dev, void* stream);

/* Softmax top-k with selected-weight normalisation.  Replaces moe_topk_cuda
 * (mfq/kernels/cuda/moe.cu:1953-2079; kernels moe_topk512.cuh:5-114, moe.cu:326-476) for
 * use_sigmoid = use_sqrt_softplus = delayed_softmax = false, bias = none.
 * ids_dev i32 [tokens, k] descending weight, ties to the lower id; weights_dev f32 [tokens, k]. */
int mfq_amd_topk(const void* logits_dev, int32_t logits_dtype, int32_t tokens, int32_t experts, int32_t top_k,
                 int32_t normalize, float norm_floor, float scale, int32_t* ids_dev, float* weights_dev,
                 void* stream);

/* Pair compaction by expert.  Replaces moe_build_expert_map_cuda (moe.cu:2118-2193; kernels :679-917)
 * and build_moe_route_plan (cpp_runtime/backends/cuda/ops/moe.cpp:257-320).
 * counts_dev[experts], expert_bounds_dev[experts+1], tile_bounds_dev[experts+1],
 * tile_experts_dev[pairs/tile_m + experts], ids_dst_dev[pairs] (compact slot -> pair, ascending pair
 * order inside an expert).  Pairs whose id is outside [0, experts) are skipped. */
int mfq_amd_route_plan(const int32_t* ids_dev, int32_t tokens, int32_t top_k, int32_t experts, int32_t tile_m,
                       int32_t* counts_dev, int32_t* expert_bounds_dev, int32_t* tile_bounds_dev,
                       int32_t* tile_experts_dev, int32_t* ids_dst_dev, void* stream);

/* ---------------------------------------------------------------------------
 * Mixed-format MoE projection and fused FFN.
 * ------------------------------------------------------------------------- */

/* One logical [experts, out, in] tensor stored as pools.  Replaces MixedMoeRuntime
 * (cpp_runtime/backends/cuda/ops/include/moe.h:133-189). */
typedef struct mfq_amd_moe_tensor {
    const mfq_amd_projection* pools;   /* host array of device-pointer descriptors */
    int32_t pool_count;
    int32_t experts, out_per_expert, neuron_len;
} mfq_amd_moe_tensor;

/* Whole routed FFN: gate/up per pair -> SwiGLU -> down per pair -> route-weighted reduce.
 * Replaces MfeFfnRuntime (ops/include/mfe_ffn_runtime.h:9-97) / MfeFfnBatch + mfe_ffn_prepare /
 * mfe_ffn_gate_up / mfe_ffn_down_reduce (mfq/kernels/cuda/mfe_ffn.h:41-132) and, for more than
 * decode_token_limit tokens, the unfused prefill path of FFN::forward_impl
 * (cpp_runtime/backends/cuda/core/ffn.cpp:676-835) over MixedMoeRuntime::forward. */
typedef struct mfq_amd_moe_ffn mfq_amd_moe_ffn;
typedef struct mfq_amd_moe_ffn_config {
    mfq_amd_moe_tensor gate, up, down;
    int32_t top_k;
    int32_t max_tokens;        /* workspace capacity; run() rejects more */
    int32_t x_dtype;           /* MFQ_AMD_F32 / F16 / BF16 */
    int32_t out_dtype;         /* MFQ_AMD_F32 or MFQ_AMD_F16 */
    float swiglu_limit;        /* > 0: clamped variant (mfe_ffn.h:111-114) */
    int32_t decode_token_limit;/* tokens <= limit use the streaming GEMV kernels, more use the grouped GEMM; 0 = default (32).
                                * Clamped to 1024 / top_k: a decode plan is one thread per routed pair
                                * (mfq_amd_moe_ffn_decode_limit gives the value create will use). */
    int32_t launch_mode;       /* decode: 0 = one launch per stage covering every format (blocks sorted by
                                  format), 1 = one launch per format and stage */
    int32_t mx_scaled_mfma;    /* 1: prefill tiles of MXFP4 pools run on the block-scaled MFMA (v_mfma_scale_f32_32x32x64_f8f6f4:
                                  fp4 weights with their E8M0 scales as stored, activations as E4M3 terms that add up to the
                                  source exactly); 0: on the fp16 tiles like every other format.  Counterpart of
                                  mxfp4_moe_grouped_tensor_kernel (mfq/kernels/cuda/mx_matmul.cu:954). */
    int32_t expert_activation; /* 0: hidden = silu(gate) * up; 1: hidden = relu(up)^2 and no gate projection: gate.pool_count
                                  must be 0 and swiglu_limit 0 (MfeFfnBatch::expert_activation, mfq/kernels/cuda/mfe_ffn.h:79-82,
                                  :107-110) */
    int32_t group_pairs;       /* decode: 1 = a block of the rows kernels serves up to four pairs that are routed to the same
                                  expert (the expert's rows are fetched and decoded once for the group: the per-token-group
                                  form of mfq/kernels/cuda/mfe_mxfp4_dot.cuh:36-68, mfe_ffn_device.cuh:916-1006); 0 = one pair
                                  per block, pairs of one expert next to each other so that its rows leave HBM once (the
                                  default: it measured faster at every batch and expert count tried, the groups' blocks hold
                                  twice the registers and half the waves) */
} mfq_amd_moe_ffn_config;

/* create may allocate and synchronise; run allocates nothing, does not synchronise and can be
 * captured into a HIP graph (workspaces are fixed at create, as the reference fixes them per capacity
 * bucket, ops/include/mfe_weight.h:49-72). */
int mfq_amd_moe_ffn_create(const mfq_amd_moe_ffn_config* config, mfq_amd_moe_ffn** out);
/* The decode token limit create uses for a requested limit (0 = default) and top_k; pure, needs no device.
 * Counterpart of the capacity buckets the reference fixes per runtime (ops/include/mfe_weight.h:49-72). */
int32_t mfq_amd_moe_ffn_decode_limit(int32_t requested, int32_t top_k);
int mfq_amd_moe_ffn_run(mfq_amd_moe_ffn* ffn, const void* x_dev, const int32_t* ids_dev,
                        const float* route_weights_dev, int32_t tokens, void* out_dev, void* stream);
/* The layer's shared expert inside the FFN object (MfeFfnBatch::shared, shared_gate, shared_activation;
 * mfq/kernels/cuda/mfe_ffn.h:45,60,79-82): a dense FFN (one expert per projection, gate NULL for shared_activation 1)
 * that every token runs beside its routed experts.  set_shared may allocate and synchronise; the descriptors are
 * copied, their device buffers stay borrowed.  run_shared is run() with the epilogue of mfe_ffn_down_reduce_kernel
 * (mfq/kernels/cuda/mfe_ffn_device.cuh:1249-1263): out = half(sum_r w * pair) + shared_ffn(x)[half] * shared_gate[token]
 * in fp32, written as config.out_dtype; shared_gate_dev holds one evaluated gate value per token (float32, float16 or
 * bfloat16; with float16 the product is rounded to fp16 first, the reference's shared_product_half).  The routed sum
 * adds w * pair per route in route order with a separate multiply and add, which is what the oracle fixes; the
 * reference's kernels write value += w * x (mfq/kernels/cuda/moe.cu:1511, mfe_ffn_device.cuh:1249-1263), which their
 * compiler may contract to an FMA, so bit parity with them before the fp16 rounding is not pinned (no fixture of the
 * reference covers it).  Allocates nothing, does not synchronise. */
int mfq_amd_moe_ffn_set_shared(mfq_amd_moe_ffn* ffn, const mfq_amd_projection* gate, const mfq_amd_projection* up,
                               const mfq_amd_projection* down, int32_t shared_activation);
int mfq_amd_moe_ffn_run_shared(mfq_amd_moe_ffn* ffn, const void* x_dev, const int32_t* ids_dev, const float* route_weights_dev,
                               const void* shared_gate_dev, int32_t shared_gate_dtype, int32_t tokens, void* out_dev,
                               void* stream);
/* The same layer with routing fused in: softmax top-k of logits_dev[tokens, experts] (arguments as
 * mfq_amd_topk) is selected inside the route-plan kernel when tokens <= min(decode_token_limit, 32),
 * by the top-k kernel otherwise.  Replaces the moe_topk_cuda + MfeFfnRuntime::run pair of calls
 * (mfq/kernels/cuda/moe.cu:1953-2079, mfe_ffn_runtime.h:52-97) with one. */
int mfq_amd_moe_ffn_run_logits(mfq_amd_moe_ffn* ffn, const void* x_dev, const void* logits_dev, int32_t logits_dtype,
                               int32_t normalize, float norm_floor, float scale, int32_t tokens, void* out_dev,
                               void* stream);
/* The same with the router matmul in front: logits = x . router^T (as mfq_amd_router_logits, into a buffer of the
 * object), then mfq_amd_moe_ffn_run_logits.  router_dev[experts, hidden].  Replaces the router GEMM + moe_topk_cuda +
 * MfeFfnRuntime::run sequence of FFN::forward_impl (cpp_runtime/backends/cuda/core/ffn.cpp:443-447, :676-835). */
int mfq_amd_moe_ffn_run_router(mfq_amd_moe_ffn* ffn, const void* x_dev, const void* router_dev, int32_t router_dtype,
                               int32_t normalize, float norm_floor, float scale, int32_t tokens, void* out_dev, void* stream);
/* Routes of the last mfq_amd_moe_ffn_run_logits: ids i32 [tokens, k], weights f32 [tokens, k]. */
int mfq_amd_moe_ffn_routes(mfq_amd_moe_ffn* ffn, const int32_t** ids_dev, const float** weights_dev);
/* Which projections (bit 0 gate, bit 1 up, bit 2 down) have their MXFP4 prefill tiles on the block-scaled MFMA.  create
 * honours mx_scaled_mfma = 1 only for 16-bit activations, launch_mode 0, max_tokens above the decode limit and widths the
 * streaming tile kernel serves; this says what it decided.  No counterpart in the reference. */
int mfq_amd_moe_ffn_mx_scaled_slots(mfq_amd_moe_ffn* ffn, int32_t* mask);
/* Stage buffers of the last run (device pointers, valid until destroy): gate_up f16 [tokens, k, 2, I]
 * (gate then up), pairs f16 [tokens, k, H]. */
int mfq_amd_moe_ffn_buffers(mfq_amd_moe_ffn* ffn, const void** gate_up_f16, const void** pairs_f16);
/* Packed-weight bytes (all packed fields of every distinct routed expert, codebooks excluded) that
 * the last run's routing touched.  A measurement aid: runs a small kernel over the ids of the last run (which
 * must still be valid) on the stream it ran on, and synchronises that stream. */
int mfq_amd_moe_ffn_touched_bytes(mfq_amd_moe_ffn* ffn, int64_t* bytes, int32_t* distinct_experts);
/* Measurement aid: when enabled, run() records HIP events on its stream around the five stages
 * (route plan, gate+up, SwiGLU, down, reduce) without synchronising; stage_times() synchronises the
 * last run's stream and returns the elapsed milliseconds of each stage of that run.  With
 * launch_mode 0 the gate+up and down stages are one kernel each.  No counterpart in the reference,
 * which times stages with CudaProfiler::measure (ops/include/cuda_execution.h:109-150). */
int mfq_amd_moe_ffn_enable_timing(mfq_amd_moe_ffn* ffn, int32_t enable);
int mfq_amd_moe_ffn_stage_times(mfq_amd_moe_ffn* ffn, float* ms5);
/* What a stage bracket reads when nothing is launched inside it: the elapsed time between two events recorded back to
 * back behind the last stage of the same run (a few microseconds on this part).  Stage times of short kernels are read
 * net of it. */
int mfq_amd_moe_ffn_empty_bracket_ms(mfq_amd_moe_ffn* ffn, float* ms);
void mfq_amd_moe_ffn_destroy(mfq_amd_moe_ffn* ffn);

/* One mixed-format projection for routed pairs: out_dev f16 [tokens, k, out_per_expert].
 * x_rows_per_token = 1 (x_dev[tokens, K], gate/up) or k (x_dev[tokens, k, K], down).
 * Replaces MixedMoeRuntime::forward (cpp_runtime/backends/cuda/ops/moe.cpp:1489-1990).
 * workspace_dev: mfq_amd_grouped_matmul_workspace(tokens, k, experts) bytes. */
int64_t mfq_amd_grouped_matmul_workspace(int32_t tokens, int32_t top_k, int32_t experts);
int mfq_amd_grouped_matmul(const mfq_amd_moe_tensor* tensor, const void* x_dev, int32_t x_dtype,
                           int32_t x_rows_per_token, const int32_t* ids_dev, int32_t tokens, int32_t top_k,
                           void* out_f16_dev, void* workspace_dev, int64_t workspace_bytes, void* stream);

/* The same projection without a workspace argument and without any allocation, for callers that cannot allocate
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  The route plan lives in a static device array of mfq_amd_grouped_matmul_static_capacity() bytes
 * (128 KiB per GPU, held until the process ends): calls whose mfq_amd_grouped_matmul_workspace(tokens, top_k,
 * experts) exceeds it return MFQ_AMD_ERR_INVALID.  mfq_amd_init() must have run on the device (it allocates; this
 * entry point does not).  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams,
 * or two graphs replayed at the same time) race; calls on one stream are ordered and safe. */
int64_t mfq_amd_grouped_matmul_static_capacity(void);
int mfq_amd_grouped_matmul_static(const mfq_amd_moe_tensor* tensor, const void* x_dev, int32_t x_dtype,
                                  int32_t x_rows_per_token, const int32_t* ids_dev, int32_t tokens, int32_t top_k,
                                  void* out_f16_dev, void* stream);

/* hidden = swiglu(gate, up) with the reference's fp16 rounding chain
 * (mfq/kernels/cuda/mfe_ffn.h:105-118; cuda/storage/moe_ffn_pipeline.cpp:154-169).  Uses the device's sigmoid
 * table (see mfq_amd_init). */
int mfq_amd_swiglu(const void* gate_f16_dev, const void* up_f16_dev, int64_t count, float swiglu_limit,
                   void* hidden_f16_dev, void* stream);
/* out[t, c] = sum_r w[t, r] * pair[t, r, c], fp32, routes ascending.  Replaces
 * moe_weighted_reduce_cuda (mfq/kernels/cuda/moe.cu:1495-1515, :2620-2655). */
int mfq_amd_weighted_reduce(const void* pairs_f16_dev, const float* weights_dev, int32_t tokens, int32_t top_k,
                            int32_t width, void* out_dev, int32_t out_dtype, void* stream);
/* The reduce followed by the shared expert's gated contribution, fp16 out:
 * out[t, c] = half(half(sum_r w[t, r] * pair[t, r, c]) + sigmoid(gate_logits[t]) * shared[t, c]).  Replaces
 * moe_weighted_reduce_shared_gate_kernel (mfq/kernels/cuda/moe.cu:1573-1596).  The shared expert itself is an
 * mfq_amd_moe_ffn with one expert and top_k = 1. */
int mfq_amd_weighted_reduce_shared_gate(const void* pairs_f16_dev, const float* weights_dev, const void* shared_f16_dev,
                                        const float* gate_logits_dev, int32_t tokens, int32_t top_k, int32_t width,
                                        void* out_f16_dev, void* stream);
/* out[r, c] = half(routed[r, c] + sigmoid(gate_logits[r]) * shared[r, c]), all fp16.  Replaces
 * moe_add_shared_gate_kernel (mfq/kernels/cuda/moe.cu:1557-1571). */
int mfq_amd_add_shared_gate(const void* routed_f16_dev, const void* shared_f16_dev, const float* gate_logits_dev,
                            int32_t rows, int32_t width, void* out_f16_dev, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MFQ_AMD_H */
