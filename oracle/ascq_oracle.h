/*
 * ascq_oracle.h - CPU restatement of the asc-devkit quantized-inference operators.
 * TEST INFRASTRUCTURE ONLY: see ascq_oracle.c.  Host pointers everywhere; descriptors are the ones of ascq.h.
 */
#ifndef ASCQ_ORACLE_H
#define ASCQ_ORACLE_H

#include "../include/ascq.h"

#ifdef __cplusplus
extern "C" {
#endif

void orc_set_threads(int n);
int orc_get_threads(void);

uint16_t orc_f64_to_f16(double d);
uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t b);
uint16_t orc_f16_mul(uint16_t a, uint16_t b);
uint16_t orc_f16_add(uint16_t a, uint16_t b);
uint16_t orc_bf16_mul(uint16_t a, uint16_t b);
uint16_t orc_bf16_add(uint16_t a, uint16_t b);
int8_t orc_round_sat8(double v, int round_mode);
float orc_faster_gelu(float x);
float orc_swiglu(float src0, float src1, float beta);
float orc_quant_word_scale(uint64_t w, int scale_format);
float orc_prescaled_accumulator(int32_t acc, uint64_t qword, int scale_format, int out_dtype);

uint8_t orc_f32_to_fp8(float f, int e5m2);
float orc_fp8_to_f32(uint8_t code, int e5m2);
uint8_t orc_f32_to_hif8(float f);
float orc_hif8_to_f32(uint8_t code);
uint8_t orc_f32_to_fp4(float f, int e1m2, int round_mode);
float orc_fp4_to_f32(uint8_t code, int e1m2);
int orc_quant(const ascq_quant_desc* d, int8_t* dst, const void* src, const void* scale, const void* offset);
int orc_dynamic_quant_per_token(int src_dtype, uint32_t m, uint32_t n, int8_t* q, float* tok_scale, const void* x);
uint32_t orc_dequant_dst_stride(int dst_dtype, uint32_t n);
int orc_dequant(const ascq_dequant_desc* d, void* dst, const void* src, const void* scale);
int orc_antiquant(const ascq_antiquant_desc* d, void* dst, const void* src, const void* offset, const void* scale);
int orc_matmul_w8a8(const ascq_matmul_desc* d, void* c, const int8_t* a, const int8_t* b, const void* bias,
                    const void* quant_vector, const float* tok_scale);
int orc_matmul_w8a8_rows(const ascq_matmul_desc* d, void* c, const int8_t* a, const int8_t* b, const void* bias,
                         const void* quant_vector, const float* tok_scale, uint32_t r0, uint32_t r1);
int orc_group_matmul_w8a8(const ascq_group_matmul_desc* g, void* y, const int8_t* x, const int8_t* w,
                          const void* bias, const float* scale, const float* tok_scale, const int64_t* group_list);
int orc_matmul_w4a16(const ascq_w4a16_desc* d, uint16_t* y, const uint16_t* x, const uint8_t* w,
                     const uint16_t* scale, const uint16_t* offset);
int orc_matmul_w4a16_cols(const ascq_w4a16_desc* d, uint16_t* y, const uint16_t* x, const uint8_t* w,
                          const uint16_t* scale, const uint16_t* offset, uint32_t j0, uint32_t j1);
int orc_antiquant_policy(const ascq_antiquant_policy_desc* d, void* dst, const uint8_t* src, const void* scale,
                         const void* offset);
int orc_matmul_w8a16(const ascq_w8a16_desc* d, void* y, const uint16_t* x, const int8_t* w, const uint16_t* offset,
                     const uint16_t* scale);

int orc_matmul_mx(const ascq_mx_desc* d, void* c, const uint8_t* a, const uint8_t* b, const uint8_t* sa,
                  const uint8_t* sb, const float* bias, uint32_t r0, uint32_t r1, uint32_t c0, uint32_t c1);
void orc_f32_to_f16_array(uint16_t* dst, const float* src, size_t n);
void orc_f16_to_f32_array(float* dst, const uint16_t* src, size_t n);
void orc_f32_to_bf16_array(uint16_t* dst, const float* src, size_t n);
void orc_f16_mul_array(uint16_t* dst, const uint16_t* a, const uint16_t* b, size_t n);
void orc_f16_add_array(uint16_t* dst, const uint16_t* a, const uint16_t* b, size_t n);
void orc_round_sat8_array(int8_t* dst, const float* src, size_t n, int round_mode);

#ifdef __cplusplus
}
#endif
#endif
