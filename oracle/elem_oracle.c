/*
 * elem_oracle.c -- CPU restatement of the reference's element arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the library ships may call into this file: it exists so that tests,
 * the smoke check and the benchmark's cpu_baseline leg have an independent statement of what the HIP
 * kernels must compute.  Plain C, no GPU.
 *
 * Reference followed (paths relative to the reference tree):
 *   orc_fp16_to_fp32      Fp16ToFp32          src/ops/op_common/template/wrapper/alg_data_trans_wrapper.cc:1003-1058
 *   orc_fp32_to_fp16      Fp32ToFp16          ...wrapper.cc:1087-1138, Fp32DenormToFp16 :1064-1085
 *   orc_reduce            AicpuReduce         ...wrapper.cc:1165-1210  (dispatch by data type)
 *                         AicpuReduceTemplate ...wrapper.cc:1212-1252  (dst[i] = src[i] (+) dst[i])
 *                         AicpuReduceFp16     ...wrapper.cc:1140-1163  (widen, fp32 op, narrow)
 *
 * Types the reference reduces on the CPU: int8, int32, fp16, fp32, int64, uint64, fp64 (:1176-1203).
 * int16 and bf16 (and every SUM/MAX/MIN on the types above when the op is not PROD and the type is not
 * 64-bit) are reduced by HCOMM hardware whose source is not in the reference tree; for those this file
 * applies the same C expressions (int16) or fp32 arithmetic with one round-to-nearest-even narrowing
 * (bf16).  PARITY UNPINNED for the bit pattern of a NaN result: the reference computes NaNs with the
 * host FPU, whose payload rules are not part of its source; callers compare NaNs as a class.
 *
 * What pins this file (tests/test_oracle_elem.py): decode of all 65,536 half values and a dense sweep of
 * encodes against numpy's IEEE conversions; every int8 pair for SUM/PROD/MAX/MIN against two's-complement
 * arithmetic written independently in numpy; fp16 SUM/PROD against numpy float16 arithmetic (correctly
 * rounded); bf16 narrowing against an integer-only reimplementation.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "elem_oracle.h"

/* ---- fp16 <-> fp32, bit for bit as the reference writes them ---------------------------------- */

float orc_fp16_to_fp32(uint16_t h)
{
    uint32_t sign = (h >> 15) & 0x1u;
    uint32_t exponent = (h >> 10) & 0x1Fu;
    uint32_t mantissa = h & 0x3FFu;
    uint32_t result;
    if (exponent == 0) {
        if (mantissa == 0) {
            result = sign << 31;
        } else {
            int shift = 0;
            while ((mantissa & 0x400u) == 0) { /* normalise the subnormal */
                mantissa <<= 1;
                shift++;
            }
            mantissa &= 0x3FFu;
            int32_t e32 = 127 - 15 + 1 - shift;
            if (e32 <= 0) {
                result = sign << 31;
            } else {
                result = (sign << 31) | ((uint32_t)e32 << 23) | (mantissa << 13);
            }
        }
    } else if (exponent == 0x1Fu) {
        result = (sign << 31) | (0xFFu << 23) | (mantissa << 13); /* Inf, or NaN with its payload */
    } else {
        result = (sign << 31) | ((exponent + 112u) << 23) | (mantissa << 13);
    }
    float f;
    memcpy(&f, &result, sizeof(f));
    return f;
}

static uint16_t fp32_denorm_to_fp16(uint32_t sign, uint32_t mantissa, int32_t e16)
{
    if (e16 < -10) {
        return (uint16_t)(sign << 15);
    }
    mantissa |= 0x800000u;
    int32_t total_shift = 14 - e16;
    uint32_t round_bit = (mantissa >> (total_shift - 1)) & 0x1u;
    uint32_t truncated = mantissa & ((1u << (total_shift - 1)) - 1u);
    uint32_t sticky = (truncated != 0) ? 1u : 0u;
    uint16_t m16 = (uint16_t)(mantissa >> total_shift);
    m16 = (uint16_t)(m16 + (round_bit && (sticky || (m16 & 0x1u))));
    if (m16 & 0x400u) {
        return (uint16_t)((sign << 15) | (1u << 10));
    }
    return (uint16_t)((sign << 15) | m16);
}

uint16_t orc_fp32_to_fp16(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, sizeof(bits));
    uint32_t sign = (bits >> 31) & 0x1u;
    uint32_t exponent = (bits >> 23) & 0xFFu;
    uint32_t mantissa = bits & 0x7FFFFFu;
    if (exponent == 0) {
        return (uint16_t)(sign << 15); /* fp32 zero or subnormal */
    }
    if (exponent == 0xFFu) {
        if (mantissa == 0) {
            return (uint16_t)((sign << 15) | 0x7C00u);
        }
        uint16_t m16 = (uint16_t)(mantissa >> 13);
        if (m16 == 0) {
            m16 = 1;
        }
        return (uint16_t)((sign << 15) | 0x7C00u | m16);
    }
    int32_t e16 = (int32_t)exponent - 127 + 15;
    if (e16 >= 31) {
        return (uint16_t)((sign << 15) | 0x7C00u);
    }
    if (e16 <= 0) {
        return fp32_denorm_to_fp16(sign, mantissa, e16);
    }
    uint32_t discarded = mantissa & 0x1FFFu;
    uint16_t m16 = (uint16_t)(mantissa >> 13);
    uint32_t round_bit = (discarded >> 12) & 0x1u;
    uint32_t sticky = (discarded & 0xFFFu) ? 1u : 0u;
    m16 = (uint16_t)(m16 + (round_bit && (sticky || (m16 & 0x1u))));
    if (m16 == 0x400u) {
        m16 = 0;
        e16++;
    }
    if (e16 >= 31) {
        return (uint16_t)((sign << 15) | 0x7C00u);
    }
    return (uint16_t)((sign << 15) | ((uint32_t)e16 << 10) | m16);
}

/* ---- bf16: the upper half of an fp32; narrowing rounds to nearest even --------------------------- */

float orc_bf16_to_fp32(uint16_t b)
{
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, sizeof(f));
    return f;
}

uint16_t orc_fp32_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, sizeof(u));
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

/* ---- the scalar loop, op switch inside, as AicpuReduceTemplate writes it --------------------- */

#define ORC_LOOP(T, SUM_EXPR, PROD_EXPR)                                     \
    do {                                                                     \
        T *d = (T *)dst;                                                     \
        const T *s = (const T *)src;                                         \
        for (uint64_t i = 0; i < count; ++i) {                               \
            T dstData = d[i];                                                \
            T srcData = s[i];                                                \
            switch (op) {                                                    \
                case ORC_SUM: d[i] = (T)(SUM_EXPR); break;                   \
                case ORC_PROD: d[i] = (T)(PROD_EXPR); break;                 \
                case ORC_MAX: d[i] = (srcData < dstData) ? dstData : srcData; break; /* std::max(src, dst) */ \
                case ORC_MIN: d[i] = (dstData < srcData) ? dstData : srcData; break; /* std::min(src, dst) */ \
                default: return ORC_E_INTERNAL;                              \
            }                                                                \
        }                                                                    \
    } while (0)

static float f32_apply(float srcData, float dstData, int op)
{
    switch (op) {
        case ORC_SUM: return srcData + dstData;
        case ORC_PROD: return srcData * dstData;
        case ORC_MAX: return (srcData < dstData) ? dstData : srcData;
        default: return (dstData < srcData) ? dstData : srcData;
    }
}

int orc_reduce(void *dst, const void *src, uint64_t count, int dtype, int op)
{
    if (op < ORC_SUM || op > ORC_MIN) {
        return ORC_E_INTERNAL;
    }
    switch (dtype) {
        case ORC_INT8:
            ORC_LOOP(int8_t, (uint8_t)((uint8_t)srcData + (uint8_t)dstData),
                     (uint8_t)((uint8_t)srcData * (uint8_t)dstData));
            return 0;
        case ORC_INT16:
            ORC_LOOP(int16_t, (uint16_t)((uint16_t)srcData + (uint16_t)dstData),
                     (uint16_t)((uint16_t)srcData * (uint16_t)dstData));
            return 0;
        case ORC_INT32:
            ORC_LOOP(int32_t, (uint32_t)srcData + (uint32_t)dstData, (uint32_t)srcData * (uint32_t)dstData);
            return 0;
        case ORC_INT64:
            ORC_LOOP(int64_t, (uint64_t)srcData + (uint64_t)dstData, (uint64_t)srcData * (uint64_t)dstData);
            return 0;
        case ORC_UINT64:
            ORC_LOOP(uint64_t, srcData + dstData, srcData * dstData);
            return 0;
        case ORC_FP32:
            ORC_LOOP(float, srcData + dstData, srcData * dstData);
            return 0;
        case ORC_FP64:
            ORC_LOOP(double, srcData + dstData, srcData * dstData);
            return 0;
        case ORC_FP16: {
            /* AicpuReduceFp16: widen everything, reduce in fp32, narrow everything */
            uint16_t *d = (uint16_t *)dst;
            const uint16_t *s = (const uint16_t *)src;
            for (uint64_t i = 0; i < count; ++i) {
                d[i] = orc_fp32_to_fp16(f32_apply(orc_fp16_to_fp32(s[i]), orc_fp16_to_fp32(d[i]), op));
            }
            return 0;
        }
        case ORC_BFP16: {
            uint16_t *d = (uint16_t *)dst;
            const uint16_t *s = (const uint16_t *)src;
            for (uint64_t i = 0; i < count; ++i) {
                d[i] = orc_fp32_to_bf16(f32_apply(orc_bf16_to_fp32(s[i]), orc_bf16_to_fp32(d[i]), op));
            }
            return 0;
        }
        default:
            return ORC_E_INTERNAL; /* "DataType not support", wrapper.cc:1204-1207 */
    }
}

/* ---- the same arithmetic with the op switch hoisted and the loop spread over host cores ------- */

#define ORC_FAST(T, EXPR)                                        \
    do {                                                         \
        T *d = (T *)dst;                                         \
        const T *s = (const T *)src;                             \
        _Pragma("omp parallel for schedule(static)")             \
        for (int64_t i = 0; i < (int64_t)count; ++i) {           \
            T dstData = d[i];                                    \
            T srcData = s[i];                                    \
            d[i] = (T)(EXPR);                                    \
        }                                                        \
    } while (0)

#define ORC_FAST_OPS(T, U)                                                        \
    switch (op) {                                                                 \
        case ORC_SUM: ORC_FAST(T, (U)((U)srcData + (U)dstData)); break;           \
        case ORC_PROD: ORC_FAST(T, (U)((U)srcData * (U)dstData)); break;          \
        case ORC_MAX: ORC_FAST(T, (srcData < dstData) ? dstData : srcData); break; \
        default: ORC_FAST(T, (dstData < srcData) ? dstData : srcData); break;     \
    }

int orc_reduce_parallel(void *dst, const void *src, uint64_t count, int dtype, int op)
{
    if (op < ORC_SUM || op > ORC_MIN) {
        return ORC_E_INTERNAL;
    }
    switch (dtype) {
        case ORC_INT8: ORC_FAST_OPS(int8_t, uint8_t) return 0;
        case ORC_INT16: ORC_FAST_OPS(int16_t, uint16_t) return 0;
        case ORC_INT32: ORC_FAST_OPS(int32_t, uint32_t) return 0;
        case ORC_INT64: ORC_FAST_OPS(int64_t, uint64_t) return 0;
        case ORC_UINT64: ORC_FAST_OPS(uint64_t, uint64_t) return 0;
        case ORC_FP32: ORC_FAST_OPS(float, float) return 0;
        case ORC_FP64: ORC_FAST_OPS(double, double) return 0;
        case ORC_FP16:
        case ORC_BFP16: {
            uint16_t *d = (uint16_t *)dst;
            const uint16_t *s = (const uint16_t *)src;
            const int half = (dtype == ORC_FP16);
#pragma omp parallel for schedule(static)
            for (int64_t i = 0; i < (int64_t)count; ++i) {
                float a = half ? orc_fp16_to_fp32(s[i]) : orc_bf16_to_fp32(s[i]);
                float b = half ? orc_fp16_to_fp32(d[i]) : orc_bf16_to_fp32(d[i]);
                float r = f32_apply(a, b, op);
                d[i] = half ? orc_fp32_to_fp16(r) : orc_fp32_to_bf16(r);
            }
            return 0;
        }
        default:
            return ORC_E_INTERNAL;
    }
}

/* ---- conversions of whole arrays (used to run a schedule with an fp32 accumulator) ------------ */

void orc_widen16(float *dst, const uint16_t *src, uint64_t count, int dtype)
{
    for (uint64_t i = 0; i < count; ++i) {
        dst[i] = (dtype == ORC_FP16) ? orc_fp16_to_fp32(src[i]) : orc_bf16_to_fp32(src[i]);
    }
}

void orc_narrow16(uint16_t *dst, const float *src, uint64_t count, int dtype)
{
    for (uint64_t i = 0; i < count; ++i) {
        dst[i] = (dtype == ORC_FP16) ? orc_fp32_to_fp16(src[i]) : orc_fp32_to_bf16(src[i]);
    }
}

uint32_t orc_dtype_size(int dtype)
{
    /* DATATYPE_SIZE_TABLE, src/ops/op_common/inc/alg_param.h:43-45 */
    static const uint32_t table[18] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1};
    return (dtype >= 0 && dtype < 18) ? table[dtype] : 0;
}
