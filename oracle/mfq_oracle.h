/*
 * mfq_oracle.h -- CPU restatement of the reference's mixed-format MoE expert-FFN
 * arithmetic.  TEST INFRASTRUCTURE ONLY: nothing under mfq_amd/ (the product) may
 * include, link or call this file.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py use it, and only as the checker.
 *
 * Every function names the reference file:line it restates (paths relative to
 * the reference checkout).  Plain C99, scalar code, built with
 * -ffp-contract=off so that no multiply-add is fused: the reference dequantiser
 * is defined with a separate multiply and subtract
 * (cpp_runtime/backends/cpu/ops/packed_nint.cpp:77-83).
 *
 * Pinning status (what independent evidence fixes each function):
 *   orc_bits_at, orc_pack_bits      closed form + np.packbits(little) (tests/test_oracle_bits.py)
 *   orc_nint_*                      reference CPU library built from its own sources
 *                                   (oracle/_ref, bit-for-bit) + FP64 decoded-weight oracle
 *   orc_nvq_*                       same (formats 3 and 15), + brute-force sign rule
 *   orc_mxfp4_*                     exhaustive 16 codes x 255 scales vs OCP closed form
 *   orc_f32_to_f16 / orc_f16_to_f32 exhaustive vs numpy float16
 *   orc_expert_ffn                  composition of the above; rounding chain vs numpy float16
 *   orc_topk                        brute-force double softmax + sort on tie-free inputs;
 *                                   tie rule by construction of equal logits
 *   orc_route_plan                  bincount / cumsum
 *   orc_*_shared_gate               closed form in numpy (float64 sigmoid, fp16 roundings): equal
 *                                   up to one fp16 step where orc_expf and libm differ
 *   orc_expf                        <= 1 ulp vs libm on the routing range (selection only
 *                                   needs monotonicity; the reference's device expf is not
 *                                   reproducible off its GPU)
 */
#ifndef MFQ_ORACLE_H
#define MFQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- bit streams (mfq/formats/io.py:321-352, packed_nint.cpp:36-42) ---- */
uint32_t orc_bits_at(const uint8_t* data, int64_t nbytes, int64_t bit, int bits);
void orc_pack_bits(const uint32_t* values, int64_t count, int bits, uint8_t* out, int64_t out_bytes);

/* ---- half / bfloat conversions (IEEE round-to-nearest-even) ---- */
uint16_t orc_f32_to_f16(float value);
float orc_f16_to_f32(uint16_t bits);
uint16_t orc_f64_to_f16(double value);
uint16_t orc_f32_to_bf16(float value);
float orc_bf16_to_f32(uint16_t bits);

/* ---- NINT (cpp_runtime/backends/cpu/ops/packed_nint.h:10-22) ---- */
typedef struct orc_nint_view {
    const uint8_t* packed;
    int64_t packed_bytes;
    const uint8_t* row_bits;          /* [outputs] 1..8 */
    const int64_t* row_bit_offsets;   /* [outputs] */
    const uint8_t* group_scale;       /* [outputs*groups] */
    const uint8_t* group_min;         /* [outputs*groups] */
    const float* row_scale;           /* [outputs] */
    const float* row_min;             /* [outputs] */
    int64_t outputs, width, group_size;
} orc_nint_view;

/* returns 0 when valid, else a negative code (packed_nint.cpp:15-34) */
int orc_nint_validate(const orc_nint_view* w);
/* dense fp32 weights [outputs, width]: w = (rs*gs)*q - (rm*gm) */
void orc_nint_dequant(const orc_nint_view* w, float* out);
/* packed_nint.cpp:66-92 -- sequential fp32 accumulation */
void orc_nint_rows_scalar(const orc_nint_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end);
/* packed_nint_avx2.cpp:78-158 -- eight strided partial sums + fixed horizontal reduce */
void orc_nint_rows_avx2(const orc_nint_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end);

/* ---- NVQ (cpp_runtime/backends/cpu/ops/nvq_group.h:8-24) ---- */
typedef struct orc_nvq_view {
    const uint8_t* indices; int64_t index_bytes;
    const uint8_t* aux;     int64_t aux_bytes;     /* 7-bit sign masks */
    const uint8_t* states;  int64_t state_bytes;
    const float* anchors;                          /* [outputs] */
    const int8_t* metadata;                        /* format 3: [256][4]; JSC: 64 B header + banks */
    int format;                                    /* 3 = NVQ3 (D4_256), 15 = NVQ3J-L (D4_1024 JSC),
                                                      2 = NVQ2 (E8_256), 5/10/12/13 JSC variants */
    int state_bits, sign_mode;
    int64_t outputs, width;
    int64_t row_offset;                            /* rows of the pool that precede this view (streams are flat
                                                      over the whole pool; anchors are indexed absolutely too) */
} orc_nvq_view;

int orc_nvq_index_bits(int format);
int orc_nvq_is_d4(int format);
/* cuda/ops/vq.cpp:228-246, :204-226 */
float orc_nvq_multiplier(const orc_nvq_view* w, uint32_t state);
const int8_t* orc_nvq_bank(const orc_nvq_view* w, uint32_t state);
/* cuda/ops/vq.cpp:279-342 -- signed int8 values of one 24-weight group */
void orc_nvq_decode_group(const orc_nvq_view* w, int64_t row, int group, uint32_t state, int8_t values[24]);
void orc_nvq_dequant(const orc_nvq_view* w, float* out);
/* nvq_group_avx2.cpp:144-219 (rows_dot / rows_dot_single share one summation order) */
void orc_nvq_rows_avx2(const orc_nvq_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end);
/* cuda/ops/vq.cpp:377-394 + quant_dot.cpp:5-12 -- portable per-group scaled int8 dot */
void orc_nvq_rows_scalar(const orc_nvq_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end);

/* ---- MXFP4 (cuda/ops/mx.cpp:8-33, :420-447) ---- */
typedef struct orc_mxfp4_view {
    const uint8_t* values;   /* [outputs, width/2], low nibble = even column */
    const uint8_t* scales;   /* [outputs, width/32] E8M0 */
    int64_t outputs, width;
} orc_mxfp4_view;
void orc_mxfp4_dequant(const orc_mxfp4_view* w, float* out);
void orc_mxfp4_rows(const orc_mxfp4_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end);

/* ---- one projection of any family ---- */
enum { ORC_FAMILY_NINT = 1, ORC_FAMILY_NVQ = 2, ORC_FAMILY_MXFP4 = 3 };
typedef struct orc_projection {
    int family;
    orc_nint_view nint;
    orc_nvq_view nvq;
    orc_mxfp4_view mxfp4;
} orc_projection;
int64_t orc_projection_outputs(const orc_projection* p);
int64_t orc_projection_width(const orc_projection* p);
/* order: 0 = the AVX2 summation order the reference selects on this class of host,
          1 = portable scalar order */
void orc_projection_rows(const orc_projection* p, int order, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end);
void orc_projection_dequant(const orc_projection* p, float* out);

/* ---- SwiGLU rounding chain (cuda/storage/moe_ffn_pipeline.cpp:154-169) ---- */
uint16_t orc_swiglu_f16(uint16_t gate, uint16_t up, float swiglu_limit);
void orc_swiglu_array(const uint16_t* gate, const uint16_t* up, int64_t count, float swiglu_limit, uint16_t* out);
uint16_t orc_relu2_f16(uint16_t up);
void orc_relu2_array(const uint16_t* up, int64_t count, uint16_t* out);
/* x [count, width] f32 -> out [count, width] f32 through gate/up/down of one expert;
   gate/up/hidden scratch are [count, intermediate] */
void orc_expert_ffn(const orc_projection* gate, const orc_projection* up, const orc_projection* down,
    int order, const float* x, int64_t count, float swiglu_limit,
    float* gate_buf, float* up_buf, float* hidden_buf, float* out);

/* ---- routing (mfq/kernels/cuda/moe_topk512.cuh:5-114, moe.cu:326-476) ---- */
float orc_expf(float x);
void orc_topk(const float* logits, int64_t tokens, int experts, int top_k, int normalize,
    float norm_floor, float scale, int32_t* ids, float* weights);
/* fixed-order fp32 router dot: logits[t,e] = sum_c x[t,c]*router[e,c], c ascending */
void orc_router_logits(const float* x, const float* router, int64_t tokens, int experts,
    int64_t width, float* logits);
/* moe.cu:679-917; slots inside one expert are in ascending pair order here
   (the reference's order inside an expert comes from atomics and is unspecified) */
void orc_route_plan(const int32_t* ids, int64_t pairs, int experts, int tile_m,
    int32_t* counts, int32_t* expert_bounds, int32_t* tile_bounds, int32_t* tile_experts,
    int32_t* ids_dst);
/* moe.cu:1495-1515 with pairs rounded to fp16 first (mfe_ffn_device.cuh:1247-1262) */
void orc_weighted_reduce(const uint16_t* pairs_f16, const float* weights, int64_t tokens,
    int routes, int64_t width, float* out);
/* shared-expert epilogue: moe_add_shared_gate_kernel (moe.cu:1557-1571) and
   moe_weighted_reduce_shared_gate_kernel (moe.cu:1573-1596) */
void orc_add_shared_gate(const uint16_t* routed_f16, const uint16_t* shared_f16, const float* gate_logits,
    int64_t rows, int64_t width, uint16_t* out_f16);
void orc_weighted_reduce_shared_gate(const uint16_t* pairs_f16, const float* weights, const uint16_t* shared_f16,
    const float* gate_logits, int64_t tokens, int routes, int64_t width, uint16_t* out_f16);

#ifdef __cplusplus
}
#endif
#endif
