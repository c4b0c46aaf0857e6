/* elem_oracle.h -- interface of the CPU restatement of the reference's element arithmetic.
 * TEST INFRASTRUCTURE ONLY: see elem_oracle.c. */
#ifndef HCCL_AMD_ORACLE_ELEM_H_
#define HCCL_AMD_ORACLE_ELEM_H_
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* HcclDataType / HcclReduceOp values (order of DATATYPE_SIZE_TABLE, alg_param.h:43-45). */
enum { ORC_INT8 = 0, ORC_INT16 = 1, ORC_INT32 = 2, ORC_FP16 = 3, ORC_FP32 = 4, ORC_INT64 = 5, ORC_UINT64 = 6,
       ORC_FP64 = 10, ORC_BFP16 = 11 };
enum { ORC_SUM = 0, ORC_PROD = 1, ORC_MAX = 2, ORC_MIN = 3 };
enum { ORC_E_INTERNAL = 4 };

float orc_fp16_to_fp32(uint16_t h);
uint16_t orc_fp32_to_fp16(float value);
float orc_bf16_to_fp32(uint16_t b);
uint16_t orc_fp32_to_bf16(float f);

/* dst[i] = src[i] (+) dst[i], one thread, op switch inside the loop (the reference's form). */
int orc_reduce(void *dst, const void *src, uint64_t count, int dtype, int op);
/* Same results; op switch hoisted, OpenMP over all host cores. */
int orc_reduce_parallel(void *dst, const void *src, uint64_t count, int dtype, int op);

void orc_widen16(float *dst, const uint16_t *src, uint64_t count, int dtype);
void orc_narrow16(uint16_t *dst, const float *src, uint64_t count, int dtype);
uint32_t orc_dtype_size(int dtype);

#ifdef __cplusplus
}
#endif
#endif
