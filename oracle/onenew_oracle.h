/*
 * onenew_oracle.h -- CPU restatement of the oneNew x86 Conv / MatMul / Gemm arithmetic.
 * TEST INFRASTRUCTURE ONLY: parity checker and timed CPU baseline, never part of the shipped
 * library.  All pointers are host memory.  Functions return 0, -1 (bad argument), -2 (no memory).
 */
#ifndef ONENEW_ORACLE_H
#define ONENEW_ORACLE_H

#include <stdint.h>
#include "../include/onenew_hip.h" /* onhip_conv_desc_t, ACT_TYPE_E values */

#define ORACLE_LUT_LEN 8192

void oracle_set_threads(int t);
int oracle_get_threads(void);
int oracle_conv_out_shape(const onhip_conv_desc_t *d, int32_t *oh, int32_t *ow);

void oracle_build_silu_lut(float *lut);
void oracle_build_gelu_lut(float *lut);
void oracle_lut_act_f32(const float *x, const float *lut, float *y, int64_t count);

int oracle_conv2d_f32(const onhip_conv_desc_t *d, const float *x, const float *w, const float *bias,
                      const float *silu_lut, float *y);

void oracle_quantize_s8(const float *x, float scale, int8_t *q, int64_t count);
void oracle_requantize_s8(const float *y, float output_scale, int8_t *q, int64_t count);
int oracle_conv2d_w8a32(const onhip_conv_desc_t *d, const float *x, const int8_t *w8, const int32_t *bias32,
                        const float *weight_aux, const float *silu_lut, void *y, int32_t *acc32);
void oracle_quant_weight_bias(const float *w, const float *bias, int cout, int per_channel, int8_t *w8,
                              int32_t *bias32, float *weight_aux);

int oracle_add_f32(int ndim, const int32_t *large_shape, const int32_t *small_shape, const float *large,
                   const float *small, float *out);
void oracle_relu_f32(const float *x, float *y, int64_t n);
int oracle_maxpool_f32(int n, int c, int h, int w, int kh, int kw, int stride_w, int stride_h, int pad, int oh, int ow,
                       const float *x, float *y);
void oracle_global_avgpool_f32(int n, int c, int h, int w, const float *x, float *y);

void oracle_layernorm_f32(int rows, int reduce, int strided, const float *x, const float *w, const float *b, float *y);
void oracle_softmax_f32(int rows, int reduce, int strided, const float *x, float *y);
int oracle_transpose_f32(int ndim, const int32_t *in_shape, const int32_t *perm, const float *x, float *y);

#define ORACLE_CALIB_BINS 2048
float oracle_calib_abs_max(const float *x, int64_t n, float running_max);
void oracle_calib_histogram(const float *x, int64_t n, float max_abs, float *hist);
void oracle_calib_kl_curve(const float *hist, int64_t elem_count, float *kl_out);
void oracle_calib_mse_curve(const float *hist, int64_t elem_count, float *loss_out);
float oracle_calib_threshold_kl(const float *hist, int64_t elem_count, float max_abs);
float oracle_calib_threshold_mse(const float *hist, int64_t elem_count, float max_abs);
float oracle_calib_threshold_percent(const float *x, int images, int32_t elems);

int oracle_matmul_f32(int batch, int M, int K, int N, int b_shared, const float *A, const float *B, float *C);
int oracle_gemm_f32(int M, int K, int N, const float *A, const float *W, const float *bias, float *C);
int oracle_matmul_bias_gelu_f32(int batch, int M, int K, int N, int b_shared, const float *A, const float *B,
                                const float *bias, const float *gelu_lut, float *C);
void oracle_round_bf16(const float *x, float *y, int64_t count);
void oracle_round_f16(const float *x, float *y, int64_t count);

#endif
