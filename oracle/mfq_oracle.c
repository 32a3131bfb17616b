/*
 * mfq_oracle.c -- see mfq_oracle.h.  TEST INFRASTRUCTURE ONLY.
 * Build: gcc -std=c99 -O2 -ffp-contract=off -fPIC -shared (oracle/Makefile).
 */
#include "mfq_oracle.h"

#include <math.h>
#include <string.h>
#include <float.h>
#include <limits.h>
#include <stdlib.h>

/* ------------------------------------------------------------------ */
/* bit streams                                                          */
/* ------------------------------------------------------------------ */

/* Value i of width b occupies bits [i*b, (i+1)*b) of a little-endian byte
 * stream, least significant bit first (mfq/formats/io.py:321-352;
 * cpp_runtime/backends/cpu/ops/packed_nint.cpp:36-42).  Never reads past nbytes. */
uint32_t orc_bits_at(const uint8_t* data, int64_t nbytes, int64_t bit, int bits) {
    uint64_t word = 0;
    int64_t byte = bit >> 3;
    int shift = (int)(bit & 7);
    int need = (shift + bits + 7) >> 3;
    for (int i = 0; i < need && byte + i < nbytes; ++i) word |= (uint64_t)data[byte + i] << (8 * i);
    return (uint32_t)((word >> shift) & ((bits >= 32) ? 0xffffffffull : ((1ull << bits) - 1ull)));
}

void orc_pack_bits(const uint32_t* values, int64_t count, int bits, uint8_t* out, int64_t out_bytes) {
    memset(out, 0, (size_t)out_bytes);
    for (int64_t i = 0; i < count; ++i) {
        uint64_t v = values[i] & ((bits >= 32) ? 0xffffffffull : ((1ull << bits) - 1ull));
        int64_t bit = i * bits;
        for (int b = 0; b < bits; ++b, ++bit)
            if ((v >> b) & 1u) out[bit >> 3] |= (uint8_t)(1u << (bit & 7));
    }
}

/* ------------------------------------------------------------------ */
/* half / bfloat16                                                      */
/* ------------------------------------------------------------------ */

static uint32_t f32_bits(float v) { uint32_t u; memcpy(&u, &v, 4); return u; }
static float bits_f32(uint32_t u) { float v; memcpy(&v, &u, 4); return v; }

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* IEEE binary64 -> binary16, one rounding (round to nearest, ties to even). */
uint16_t orc_f64_to_f16(double value) {
    uint64_t u; memcpy(&u, &value, 8);
    uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
    int64_t exp = (int64_t)((u >> 52) & 0x7ff);
    uint64_t man = u & 0xfffffffffffffull;
    if (exp == 0x7ff) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0u));
    if (exp == 0) return sign;                         /* double subnormal: far below half range */
    int64_t e = exp - 1023;                            /* unbiased */
    uint64_t sig = man | (1ull << 52);                 /* 53-bit significand */
    int shift;                                         /* bits to drop from sig */
    int64_t half_exp;
    if (e >= -14) { shift = 42; half_exp = e + 15; }   /* normal half: keep 11 bits */
    else {
        int64_t extra = -14 - e;                       /* subnormal half */
        if (extra > 12) return sign;                   /* below half of the least subnormal */
        shift = 42 + (int)extra; half_exp = 0;
    }
    uint64_t kept = sig >> shift;
    uint64_t rem = sig & ((1ull << shift) - 1ull);
    uint64_t halfway = 1ull << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1ull))) ++kept;
    uint32_t out;
    if (half_exp > 0) out = (uint32_t)((half_exp - 1) << 10) + (uint32_t)kept;   /* carry rolls the exponent */
    else out = (uint32_t)kept;                                                    /* 0x400 == least normal */
    if (out >= 0x7c00u) out = 0x7c00u;
    return (uint16_t)(sign | out);
}

uint16_t orc_f32_to_f16(float value) {
    /* binary32 -> binary64 is exact, so one rounding happens in orc_f64_to_f16. */
    if (value != value) return (uint16_t)(((f32_bits(value) >> 16) & 0x8000u) | 0x7e00u);
    return orc_f64_to_f16((double)value);
}

uint16_t orc_f32_to_bf16(float value) {
    uint32_t u = f32_bits(value);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float orc_bf16_to_f32(uint16_t bits) { return bits_f32((uint32_t)bits << 16); }

/* ------------------------------------------------------------------ */
/* NINT                                                                 */
/* ------------------------------------------------------------------ */

/* cpp_runtime/backends/cpu/ops/packed_nint.cpp:15-34 */
int orc_nint_validate(const orc_nint_view* w) {
    if (w->outputs < 0 || w->width <= 0 || w->group_size <= 0) return -1;
    if (!w->outputs) return 0;
    if (!w->packed || !w->row_bits || !w->row_bit_offsets || !w->group_scale ||
        !w->group_min || !w->row_scale || !w->row_min) return -2;
    uint64_t capacity = (uint64_t)w->packed_bytes * 8u;
    uint64_t width = (uint64_t)w->width;
    for (int64_t row = 0; row < w->outputs; ++row) {
        int bits = w->row_bits[row];
        int64_t offset = w->row_bit_offsets[row];
        if (bits < 1 || bits > 8 || offset < 0 || (uint64_t)offset > capacity ||
            width > (capacity - (uint64_t)offset) / (uint64_t)bits) return -3;
    }
    return 0;
}

static int64_t nint_groups(const orc_nint_view* w) { return 1 + (w->width - 1) / w->group_size; }

static uint32_t nint_code(const orc_nint_view* w, uint64_t bit, int bits) {
    /* packed_nint.cpp:36-42 */
    size_t byte = (size_t)(bit >> 3);
    unsigned shift = (unsigned)(bit & 7);
    uint32_t word = w->packed[byte];
    if (shift + (unsigned)bits > 8) word |= (uint32_t)w->packed[byte + 1] << 8;
    return (word >> shift) & ((1u << bits) - 1u);
}

void orc_nint_dequant(const orc_nint_view* w, float* out) {
    int64_t groups = nint_groups(w);
    for (int64_t row = 0; row < w->outputs; ++row) {
        int bits = w->row_bits[row];
        uint64_t bit = (uint64_t)w->row_bit_offsets[row];
        for (int64_t group = 0; group < groups; ++group) {
            int64_t meta = row * groups + group;
            float scale = w->row_scale[row] * (float)w->group_scale[meta];
            float minimum = w->row_min[row] * (float)w->group_min[meta];
            int64_t start = group * w->group_size;
            int64_t stop = start + (w->group_size < w->width - start ? w->group_size : w->width - start);
            for (int64_t column = start; column < stop; ++column, bit += (uint64_t)bits) {
                float product = scale * (float)nint_code(w, bit, bits);
                out[row * w->width + column] = product - minimum;
            }
        }
    }
}

/* packed_nint.cpp:66-92 */
void orc_nint_rows_scalar(const orc_nint_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end) {
    int64_t groups = nint_groups(w);
    for (int64_t row = begin; row < end; ++row) {
        for (int64_t sample = 0; sample < batch; ++sample) {
            float sum = 0.0f;
            int bits = w->row_bits[row];
            uint64_t bit = (uint64_t)w->row_bit_offsets[row];
            for (int64_t group = 0; group < groups; ++group) {
                int64_t meta = row * groups + group;
                float scale = w->row_scale[row] * (float)w->group_scale[meta];
                float minimum = w->row_min[row] * (float)w->group_min[meta];
                int64_t start = group * w->group_size;
                int64_t stop = start + (w->group_size < w->width - start ? w->group_size : w->width - start);
                for (int64_t column = start; column < stop; ++column, bit += (uint64_t)bits) {
                    float product = scale * (float)nint_code(w, bit, bits);
                    float decoded = product - minimum;
                    float term = decoded * input[sample * input_stride + column];
                    sum = sum + term;
                }
            }
            output[sample * output_stride + row] = sum;
        }
    }
}

/* Horizontal reduce of eight lanes in the order of packed_nint_avx2.cpp:70-75
 * (= nvq_group_avx2.cpp:24-29): (l + l+4), then (l + l+2), then lane0 + lane1. */
static float reduce8(const float acc[8]) {
    float s4[4], s2[2];
    for (int j = 0; j < 4; ++j) s4[j] = acc[j] + acc[j + 4];
    s2[0] = s4[0] + s4[2];
    s2[1] = s4[1] + s4[3];
    return s2[0] + s2[1];
}

/* packed_nint_avx2.cpp:78-158.  Lane j of the 8-wide accumulator takes columns
 * start+j, start+8+j, ... of every group; a short tail adds +0*+0 to the idle lanes. */
void orc_nint_rows_avx2(const orc_nint_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end) {
    int64_t groups = nint_groups(w);
    for (int64_t row = begin; row < end; ++row) {
        int bits = w->row_bits[row];
        for (int64_t sample = 0; sample < batch; ++sample) {
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            uint64_t bit = (uint64_t)w->row_bit_offsets[row];
            const float* x = input + sample * input_stride;
            for (int64_t group = 0; group < groups; ++group) {
                int64_t meta = row * groups + group;
                float scale = w->row_scale[row] * (float)w->group_scale[meta];
                float minimum = w->row_min[row] * (float)w->group_min[meta];
                int64_t column = group * w->group_size;
                int64_t stop = column + (w->group_size < w->width - column ? w->group_size : w->width - column);
                for (; column < stop; column += 8) {
                    int valid = (int)(stop - column < 8 ? stop - column : 8);
                    for (int j = 0; j < 8; ++j) {
                        float term;
                        if (j < valid) {
                            float product = scale * (float)nint_code(w, bit + (uint64_t)(j * bits), bits);
                            float decoded = product - minimum;
                            term = decoded * x[column + j];
                        } else {
                            term = 0.0f * 0.0f;
                        }
                        acc[j] = acc[j] + term;
                    }
                    bit += (uint64_t)valid * (uint64_t)bits;
                }
            }
            output[sample * output_stride + row] = reduce8(acc);
        }
    }
}

/* ------------------------------------------------------------------ */
/* NVQ                                                                  */
/* ------------------------------------------------------------------ */

int orc_nvq_is_d4(int format) {
    /* cuda/ops/vq.cpp:200-203 */
    return format == 3 || format == 10 || format == 11 || format == 12 || format == 15;
}

int orc_nvq_index_bits(int format) {
    /* cuda/ops/vq.cpp:283-285 */
    switch (format) {
        case 1: return 11; case 7: return 7; case 8: case 12: return 9; case 9: return 6;
        case 13: case 15: return 10; case 14: return 12; default: return 8;
    }
}

static int nvq_entries(int format) {
    switch (format) { case 12: return 512; case 13: case 15: return 1024; case 14: return 4096; default: return 256; }
}

static int nvq_is_jsc(int format) {
    return format == 5 || format == 10 || format == 12 || format == 13 || format == 14 || format == 15;
}

/* cuda/ops/vq.cpp:204-226 */
const int8_t* orc_nvq_bank(const orc_nvq_view* w, uint32_t state) {
    if (w->format == 11) return w->metadata + 64 + (int64_t)(state & 1u) * 256 * 4;   /* vq.cpp:214-220 */
    if (!nvq_is_jsc(w->format)) return w->metadata;
    uint32_t bank = (uint8_t)w->metadata[36 + state];
    int dim = orc_nvq_is_d4(w->format) ? 4 : 8;
    return w->metadata + 64 + (int64_t)bank * nvq_entries(w->format) * dim;
}

/* cuda/ops/vq.cpp:228-246 with anchor = 1 (the multipliers[] table of vq.cpp:364-367) */
float orc_nvq_multiplier(const orc_nvq_view* w, uint32_t state) {
    if (w->format == 11) return 1.0f * (float)((state >> 1) + 1u);                      /* vq.cpp:242-244 */
    if (!nvq_is_jsc(w->format)) return 1.0f * (float)state;
    uint16_t h;
    memcpy(&h, w->metadata + 4 + 2 * (int64_t)state, 2);
    return 1.0f * orc_f16_to_f32(h);
}

static uint32_t parity7(uint32_t v) { v &= 0x7fu; v ^= v >> 4; v ^= v >> 2; v ^= v >> 1; return v & 1u; }

/* cuda/ops/vq.cpp:279-342 */
void orc_nvq_decode_group(const orc_nvq_view* w, int64_t view_row, int group, uint32_t state, int8_t values[24]) {
    int64_t row = view_row + w->row_offset;
    int d4 = orc_nvq_is_d4(w->format);
    int bits = orc_nvq_index_bits(w->format);
    int64_t nvec = (w->width + (d4 ? 3 : 7)) / (d4 ? 4 : 8);
    int64_t nsign = (w->width + 7) / 8;
    const int8_t* bank = orc_nvq_bank(w, state);
    for (int chunk = 0; chunk < 3; ++chunk) {
        int64_t vector8 = (int64_t)group * 3 + chunk;
        int64_t vector = d4 ? vector8 * 2 : vector8;
        if (vector >= nvec) { memset(values + chunk * 8, 0, 8); continue; }
        int64_t linear = row * nvec + vector;
        uint32_t code = orc_bits_at(w->indices, w->index_bytes, linear * bits, bits);
        int8_t decoded[8];
        if (d4) {
            memcpy(decoded, bank + (int64_t)code * 4, 4);
            if (vector + 1 < nvec) {
                uint32_t second = orc_bits_at(w->indices, w->index_bytes, (linear + 1) * bits, bits);
                memcpy(decoded + 4, bank + (int64_t)second * 4, 4);
            } else memset(decoded + 4, 0, 4);
        } else memcpy(decoded, bank + (int64_t)code * 8, 8);
        uint32_t mask7 = orc_bits_at(w->aux, w->aux_bytes, (row * nsign + vector8) * 7, 7);
        uint32_t last = parity7(mask7) ^ ((w->format == 2 && w->sign_mode != 0) ? ((code >> 7) & 1u) : 0u);
        uint32_t mask8 = mask7 | (last << 7);
        for (int i = 0; i < 8; ++i) {
            int value = decoded[i];
            value *= 1 - 2 * (int)((mask8 >> i) & 1u);
            values[chunk * 8 + i] = (int8_t)value;
        }
    }
}

static int64_t nvq_groups(const orc_nvq_view* w) { return (w->width + 23) / 24; }

static uint32_t nvq_state(const orc_nvq_view* w, int64_t row, int64_t group) {
    return orc_bits_at(w->states, w->state_bytes, ((row + w->row_offset) * nvq_groups(w) + group) * w->state_bits, w->state_bits);
}

void orc_nvq_dequant(const orc_nvq_view* w, float* out) {
    int64_t groups = nvq_groups(w);
    for (int64_t row = 0; row < w->outputs; ++row)
        for (int64_t group = 0; group < groups; ++group) {
            uint32_t state = nvq_state(w, row, group);
            float scale = w->anchors[row + w->row_offset] * orc_nvq_multiplier(w, state);
            int8_t values[24];
            orc_nvq_decode_group(w, row, (int)group, state, values);
            for (int i = 0; i < 24 && group * 24 + i < w->width; ++i)
                out[row * w->width + group * 24 + i] = scale * (float)values[i];
        }
}

/* nvq_group_avx2.cpp:144-176 and :178-219 (same order for batch 1 and batch n) */
void orc_nvq_rows_avx2(const orc_nvq_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end) {
    int64_t groups = nvq_groups(w);
    for (int64_t row = begin; row < end; ++row)
        for (int64_t sample = 0; sample < batch; ++sample) {
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            const float* x = input + sample * input_stride;
            for (int64_t group = 0; group < groups; ++group) {
                uint32_t state = nvq_state(w, row, group);
                float scale = w->anchors[row + w->row_offset] * orc_nvq_multiplier(w, state);
                int64_t start = group * 24;
                int valid = (int)(w->width - start < 24 ? w->width - start : 24);
                int8_t values[24];
                orc_nvq_decode_group(w, row, (int)group, state, values);
                for (int chunk = 0; chunk < (valid + 7) / 8; ++chunk)
                    for (int j = 0; j < 8; ++j) {
                        float decoded = scale * (float)values[chunk * 8 + j];
                        float xv = (chunk * 8 + j < valid) ? x[start + chunk * 8 + j] : 0.0f;
                        float term = decoded * xv;
                        acc[j] = acc[j] + term;
                    }
            }
            output[sample * output_stride + row] = reduce8(acc);
        }
}

/* make_cpu_projection_rows(const NvqWeight&) scalar_rows closure, cuda/ops/vq.cpp:377-392,
 * with quant_dot.cpp:5-12 as the dot */
void orc_nvq_rows_scalar(const orc_nvq_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end) {
    int64_t groups = nvq_groups(w);
    for (int64_t row = begin; row < end; ++row) {
        for (int64_t t = 0; t < batch; ++t) output[t * output_stride + row] = 0.0f;
        for (int64_t group = 0; group < groups; ++group) {
            uint32_t state = nvq_state(w, row, group);
            float scale = w->anchors[row + w->row_offset] * orc_nvq_multiplier(w, state);
            int8_t codes[24];
            orc_nvq_decode_group(w, row, (int)group, state, codes);
            int valid = (int)(w->width - group * 24 < 24 ? w->width - group * 24 : 24);
            for (int64_t t = 0; t < batch; ++t) {
                const float* x = input + t * input_stride + group * 24;
                float result = 0.0f;
                for (int i = 0; i < valid; ++i) {
                    float decoded = scale * (float)codes[i];
                    float term = decoded * x[i];
                    result = result + term;
                }
                output[t * output_stride + row] = output[t * output_stride + row] + result;
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* MXFP4                                                                */
/* ------------------------------------------------------------------ */

static const float kE2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

/* cuda/ops/mx.cpp:420-447: magnitude * 2^(s-127), then the sign */
void orc_mxfp4_dequant(const orc_mxfp4_view* w, float* out) {
    int64_t packed_columns = w->width / 2, scale_columns = w->width / 32;
    for (int64_t row = 0; row < w->outputs; ++row)
        for (int64_t column = 0; column < w->width; ++column) {
            uint8_t packed = w->values[row * packed_columns + column / 2];
            uint8_t code = (uint8_t)((packed >> ((column & 1) * 4)) & 15u);
            uint8_t raw = w->scales[row * scale_columns + column / 32];
            float scale = raw == 255u ? NAN : ldexpf(1.0f, (int)raw - 127);
            float value = kE2M1[code & 7u] * scale;
            out[row * w->width + column] = (code & 8u) ? -value : value;
        }
}

/* cuda/ops/mx.cpp:8-33: weights rounded to fp16, x*w accumulated sequentially in fp32 */
void orc_mxfp4_rows(const orc_mxfp4_view* w, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end) {
    int64_t width = w->width;
    for (int64_t row = begin; row < end; ++row)
        for (int64_t token = 0; token < batch; ++token) {
            float sum = 0.0f;
            for (int64_t group = 0; group < width / 32; ++group) {
                float scale = ldexpf(1.0f, (int)w->scales[row * (width / 32) + group] - 127);
                const uint8_t* packed = w->values + row * (width / 2) + group * 16;
                const float* x = input + token * input_stride + group * 32;
                for (int i = 0; i < 16; ++i) {
                    float lo = orc_f16_to_f32(orc_f32_to_f16(kE2M1[packed[i] & 15] * scale));
                    float hi = orc_f16_to_f32(orc_f32_to_f16(kE2M1[packed[i] >> 4] * scale));
                    float t0 = x[2 * i] * lo;
                    sum = sum + t0;
                    float t1 = x[2 * i + 1] * hi;
                    sum = sum + t1;
                }
            }
            output[token * output_stride + row] = sum;
        }
}

/* ------------------------------------------------------------------ */
/* family dispatch                                                      */
/* ------------------------------------------------------------------ */

int64_t orc_projection_outputs(const orc_projection* p) {
    return p->family == ORC_FAMILY_NINT ? p->nint.outputs : p->family == ORC_FAMILY_NVQ ? p->nvq.outputs : p->mxfp4.outputs;
}
int64_t orc_projection_width(const orc_projection* p) {
    return p->family == ORC_FAMILY_NINT ? p->nint.width : p->family == ORC_FAMILY_NVQ ? p->nvq.width : p->mxfp4.width;
}

void orc_projection_rows(const orc_projection* p, int order, const float* input, int64_t batch,
    int64_t input_stride, float* output, int64_t output_stride, int64_t begin, int64_t end) {
    if (p->family == ORC_FAMILY_NINT) {
        if (order == 0) orc_nint_rows_avx2(&p->nint, input, batch, input_stride, output, output_stride, begin, end);
        else orc_nint_rows_scalar(&p->nint, input, batch, input_stride, output, output_stride, begin, end);
    } else if (p->family == ORC_FAMILY_NVQ) {
        if (order == 0) orc_nvq_rows_avx2(&p->nvq, input, batch, input_stride, output, output_stride, begin, end);
        else orc_nvq_rows_scalar(&p->nvq, input, batch, input_stride, output, output_stride, begin, end);
    } else {
        orc_mxfp4_rows(&p->mxfp4, input, batch, input_stride, output, output_stride, begin, end);
    }
}

void orc_projection_dequant(const orc_projection* p, float* out) {
    if (p->family == ORC_FAMILY_NINT) orc_nint_dequant(&p->nint, out);
    else if (p->family == ORC_FAMILY_NVQ) orc_nvq_dequant(&p->nvq, out);
    else orc_mxfp4_dequant(&p->mxfp4, out);
}

/* ------------------------------------------------------------------ */
/* expert FFN                                                           */
/* ------------------------------------------------------------------ */

/* cuda/storage/moe_ffn_pipeline.cpp:154-169.  The half type there converts a
 * double with one rounding; gate and up arrive already rounded to fp16. */
uint16_t orc_swiglu_f16(uint16_t gate, uint16_t up, float swiglu_limit) {
    float g = orc_f16_to_f32(gate), u = orc_f16_to_f32(up);
    if (swiglu_limit > 0) {
        float clipped = g < swiglu_limit ? g : swiglu_limit;
        float value = u < -swiglu_limit ? -swiglu_limit : (u > swiglu_limit ? swiglu_limit : u);
        float activated = clipped / (1.0f + expf(-clipped));
        return orc_f32_to_f16(activated * value);
    }
    uint16_t sigmoid = orc_f64_to_f16(1.0 / (1.0 + exp(-(double)g)));
    uint16_t first = orc_f32_to_f16(g * orc_f16_to_f32(sigmoid));
    return orc_f32_to_f16(orc_f16_to_f32(first) * u);
}

/* Gate-less expert activation relu(up)^2 (mfq/kernels/cuda/mfe_ffn.h:107-110, expert_activation == 1): the square is
 * taken in float and rounded to fp16 once. */
uint16_t orc_relu2_f16(uint16_t up) {
    float u = orc_f16_to_f32(up);
    float positive = u > 0.0f ? u : 0.0f;
    return orc_f32_to_f16(positive * positive);
}

void orc_relu2_array(const uint16_t* up, int64_t count, uint16_t* out) {
    for (int64_t i = 0; i < count; ++i) out[i] = orc_relu2_f16(up[i]);
}

void orc_swiglu_array(const uint16_t* gate, const uint16_t* up, int64_t count, float swiglu_limit, uint16_t* out) {
    for (int64_t i = 0; i < count; ++i) out[i] = orc_swiglu_f16(gate[i], up[i], swiglu_limit);
}

/* cuda/storage/moe_ffn_pipeline.cpp:142-180 */
void orc_expert_ffn(const orc_projection* gate, const orc_projection* up, const orc_projection* down,
    int order, const float* x, int64_t count, float swiglu_limit,
    float* gate_buf, float* up_buf, float* hidden_buf, float* out) {
    int64_t width = orc_projection_width(gate);
    int64_t intermediate = orc_projection_outputs(gate);
    int64_t outputs = orc_projection_outputs(down);
    orc_projection_rows(gate, order, x, count, width, gate_buf, intermediate, 0, intermediate);
    orc_projection_rows(up, order, x, count, width, up_buf, intermediate, 0, intermediate);
    for (int64_t i = 0; i < count * intermediate; ++i)
        hidden_buf[i] = orc_f16_to_f32(orc_swiglu_f16(orc_f32_to_f16(gate_buf[i]), orc_f32_to_f16(up_buf[i]), swiglu_limit));
    orc_projection_rows(down, order, hidden_buf, count, intermediate, out, outputs, 0, outputs);
}

/* ------------------------------------------------------------------ */
/* routing                                                              */
/* ------------------------------------------------------------------ */

/* exp for the softmax.  The reference calls its device's expf, which cannot be
 * reproduced bit-for-bit elsewhere; selection only needs one fixed, monotone,
 * accurate routine evaluated identically wherever ids are compared.  Definition:
 * n = rint(x*log2e); r = x - n*ln2 (two-step fma); degree-5 minimax on r in
 * [-ln2/2, ln2/2] (Cephes coefficients), Horner with fma; times 2^n by exponent
 * arithmetic.  Inputs below -87 (results under FLT_MIN) return 0. */
float orc_expf(float x) {
    if (x != x) return x;
    if (x < -87.0f) return 0.0f;
    if (x > 88.0f) return INFINITY;
    float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float r2 = r * r;
    p = fmaf(p, r2, r);
    p = p + 1.0f;
    int ni = (int)n;
    return p * bits_f32((uint32_t)(ni + 127) << 23);
}

/* Lane 0 of a 32-lane shuffle-down tree, offsets 16,8,4,2,1 (moe.cu:127-133). */
static float tree32(float lanes[32]) {
    for (int offset = 16; offset > 0; offset >>= 1)
        for (int l = 0; l < offset; ++l) lanes[l] = lanes[l] + lanes[l + offset];
    return lanes[0];
}

/* moe_topk512.cuh:5-114 and moe.cu:326-476 (softmax + selected-weight normalisation) */
void orc_topk(const float* logits, int64_t tokens, int experts, int top_k, int normalize,
    float norm_floor, float scale, int32_t* ids, float* weights) {
    float* cached = (float*)malloc(sizeof(float) * (size_t)experts);
    for (int64_t t = 0; t < tokens; ++t) {
        const float* row = logits + t * experts;
        float maximum = -INFINITY;
        for (int e = 0; e < experts; ++e) {
            float v = row[e] != row[e] ? -FLT_MAX : row[e];
            maximum = v > maximum ? v : maximum;
        }
        float lanes[32];
        for (int lane = 0; lane < 32; ++lane) {
            float sum = 0.0f;
            for (int e = lane; e < experts; e += 32) {
                float v = row[e] != row[e] ? -FLT_MAX : row[e];
                sum = sum + orc_expf(v - maximum);
            }
            lanes[lane] = sum;
        }
        float total = tree32(lanes);
        /* selection over weight = expf(v-max)/total, ties to the lower id */
        float selected[32];
        int32_t chosen[32];
        for (int e = 0; e < experts; ++e) {
            float v = row[e] != row[e] ? -FLT_MAX : row[e];
            cached[e] = orc_expf(v - maximum) / total;
        }
        for (int rank = 0; rank < top_k; ++rank) {
            float best = -INFINITY; int32_t best_id = INT_MAX;
            for (int e = 0; e < experts; ++e) {
                float weight = cached[e];
                if (weight > best || (weight == best && e < best_id)) { best = weight; best_id = e; }
            }
            chosen[rank] = best_id; selected[rank] = best;
            if (best_id != INT_MAX) cached[best_id] = -INFINITY;
        }
        for (int lane = 0; lane < 32; ++lane) lanes[lane] = lane < top_k ? selected[lane] : 0.0f;
        float denominator = 1.0f;
        if (normalize) { denominator = tree32(lanes); denominator = denominator > norm_floor ? denominator : norm_floor; }
        for (int rank = 0; rank < top_k; ++rank) {
            ids[t * top_k + rank] = chosen[rank];
            float value = normalize ? selected[rank] / denominator : selected[rank];
            weights[t * top_k + rank] = value * scale;
        }
    }
    free(cached);
}

void orc_router_logits(const float* x, const float* router, int64_t tokens, int experts,
    int64_t width, float* logits) {
    for (int64_t t = 0; t < tokens; ++t)
        for (int e = 0; e < experts; ++e) {
            float sum = 0.0f;
            for (int64_t c = 0; c < width; ++c) {
                float term = x[t * width + c] * router[(int64_t)e * width + c];
                sum = sum + term;
            }
            logits[t * experts + e] = sum;
        }
}

/* moe.cu:679-917 (count_experts, scan_expert_counts, fill_tile_experts, scatter_routes) */
void orc_route_plan(const int32_t* ids, int64_t pairs, int experts, int tile_m,
    int32_t* counts, int32_t* expert_bounds, int32_t* tile_bounds, int32_t* tile_experts,
    int32_t* ids_dst) {
    for (int e = 0; e < experts; ++e) counts[e] = 0;
    for (int64_t p = 0; p < pairs; ++p)
        if ((uint32_t)ids[p] < (uint32_t)experts) counts[ids[p]]++;
    expert_bounds[0] = 0; tile_bounds[0] = 0;
    for (int e = 0; e < experts; ++e) {
        expert_bounds[e + 1] = expert_bounds[e] + counts[e];
        tile_bounds[e + 1] = tile_bounds[e] + (counts[e] + tile_m - 1) / tile_m;
        for (int tile = tile_bounds[e]; tile < tile_bounds[e + 1]; ++tile) tile_experts[tile] = e;
    }
    /* cursor per expert, ascending pair order */
    for (int e = 0; e < experts; ++e) counts[e] = 0;
    for (int64_t p = 0; p < pairs; ++p) {
        int32_t e = ids[p];
        if ((uint32_t)e >= (uint32_t)experts) continue;
        ids_dst[expert_bounds[e] + counts[e]++] = (int32_t)p;
    }
}

void orc_weighted_reduce(const uint16_t* pairs_f16, const float* weights, int64_t tokens,
    int routes, int64_t width, float* out) {
    for (int64_t t = 0; t < tokens; ++t)
        for (int64_t c = 0; c < width; ++c) {
            float sum = 0.0f;
            for (int r = 0; r < routes; ++r) {
                float term = weights[t * routes + r] * orc_f16_to_f32(pairs_f16[(t * routes + r) * width + c]);
                sum = sum + term;
            }
            out[t * width + c] = sum;
        }
}

/* moe.cu:1557-1571 (add) and :1573-1596 (reduce + add): the routed sum is rounded to fp16 before the
   shared expert's contribution, gated by sigmoid(gate_logits[token]) = 1 / (1 + exp(-g)) in fp32,
   is added; the result is rounded to fp16 again.  exp is orc_expf. */
static float orc_sigmoidf(float g) { return 1.0f / (1.0f + orc_expf(-g)); }

void orc_add_shared_gate(const uint16_t* routed_f16, const uint16_t* shared_f16, const float* gate_logits,
    int64_t rows, int64_t width, uint16_t* out_f16) {
    for (int64_t t = 0; t < rows; ++t) {
        const float gate = orc_sigmoidf(gate_logits[t]);
        for (int64_t c = 0; c < width; ++c) {
            float term = gate * orc_f16_to_f32(shared_f16[t * width + c]);
            float value = orc_f16_to_f32(routed_f16[t * width + c]) + term;
            out_f16[t * width + c] = orc_f32_to_f16(value);
        }
    }
}

void orc_weighted_reduce_shared_gate(const uint16_t* pairs_f16, const float* weights, const uint16_t* shared_f16,
    const float* gate_logits, int64_t tokens, int routes, int64_t width, uint16_t* out_f16) {
    for (int64_t t = 0; t < tokens; ++t) {
        const float gate = orc_sigmoidf(gate_logits[t]);
        for (int64_t c = 0; c < width; ++c) {
            float sum = 0.0f;
            for (int r = 0; r < routes; ++r) {
                float term = weights[t * routes + r] * orc_f16_to_f32(pairs_f16[(t * routes + r) * width + c]);
                sum = sum + term;
            }
            float routed = orc_f16_to_f32(orc_f32_to_f16(sum));
            float term = gate * orc_f16_to_f32(shared_f16[t * width + c]);
            float value = routed + term;
            out_f16[t * width + c] = orc_f32_to_f16(value);
        }
    }
}
