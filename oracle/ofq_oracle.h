/*
 * CPU oracle for OneFlow's quantized-inference op family -- declarations.
 * TEST INFRASTRUCTURE ONLY: loaded by tests/, the smoke check and the benchmark's CPU-baseline
 * leg; the shipped HIP library never calls it.
 */
#ifndef OFQ_ORACLE_H_
#define OFQ_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { OFQ_REF_F32 = 0, OFQ_REF_F16 = 1, OFQ_REF_BF16 = 2 };
enum { OFQ_REF_SCHEME_SYMMETRIC = 0, OFQ_REF_SCHEME_AFFINE = 1 };
enum { OFQ_REF_FORMULA_GOOGLE = 0, OFQ_REF_FORMULA_CAMBRICON = 1 };

float ofq_ref_half_to_float(uint16_t h);
uint16_t ofq_ref_float_to_half(float f);
uint16_t ofq_ref_float_to_bf16(float f);
float ofq_ref_bf16_to_float(uint16_t b);

/* outer = 1 (per-layer) or in.shape[0] (per-channel) */
int ofq_ref_min_max_observer_f32(const float* in, int64_t elem_cnt, int64_t outer, int bits,
                                 int scheme, int formula, float* scale, float* zero_point);
int ofq_ref_min_max_observer_f64(const double* in, int64_t elem_cnt, int64_t outer, int bits,
                                 int scheme, int formula, double* scale, double* zero_point);

/* zp_mode 0 = CPU rule (uint8-rounded zero point), 1 = CUDA rule (float zero point);
 * fake 0 = quantization, 1 = fake_quantization */
int ofq_ref_quantization_f32(const float* in, const float* scale, const float* zero_point,
                             float* out, int64_t elem_cnt, int64_t scale_size, int64_t shape0,
                             int bits, int scheme, int formula, int zp_mode, int fake);
int ofq_ref_quantization_f64(const double* in, const double* scale, const double* zero_point,
                             double* out, int64_t elem_cnt, int64_t scale_size, int64_t shape0,
                             int bits, int scheme, int formula, int zp_mode, int fake);

int ofq_ref_groupwise_dequantize(const void* in, const void* scale, const void* zero, void* out,
                                 int in_is_signed, int t, int bits, int symmetric, int64_t outer,
                                 int64_t group_size, int64_t inner);

/* moving_max / moving_min are updated in place */
int ofq_ref_moving_average_min_max_observer_f32(
    const float* in, int64_t elem_cnt, int64_t current_train_step,
    int64_t stop_update_after_iters, int training, int bits, int scheme, int formula,
    float momentum, float* moving_max, float* moving_min, float* scale, float* zero_point);
int ofq_ref_moving_average_min_max_observer_f64(
    const double* in, int64_t elem_cnt, int64_t current_train_step,
    int64_t stop_update_after_iters, int training, int bits, int scheme, int formula,
    float momentum, double* moving_max, double* moving_min, double* scale, double* zero_point);

/* weight quantiser + int4 packer of the reference's own test (x is [n,k]) */
int ofq_ref_groupwise_quantize(const void* x, void* q, void* scale, void* zero, int t,
                               int q_is_signed, int bits, int symmetric, int group_dim,
                               int64_t group_size, int64_t n, int64_t k);

int ofq_ref_fused_linear(const void* x, const void* w, const void* scale, const void* zero,
                         const void* bias, void* out, int w_is_signed, int t, int bits,
                         int symmetric, int group_dim, int64_t group_size, int64_t m, int64_t n,
                         int64_t k, int acc_mode);

int ofq_ref_layer_norm_min_max_observer(const void* x, const void* gamma, const void* beta,
                                        void* y, float* scale, float* zero_point, int64_t rows,
                                        int64_t cols, double eps, int t, int bits);
int ofq_ref_skip_layer_norm_min_max_observer(const void* x, const void* bias, const void* skip,
                                             double alpha, const void* gamma, const void* beta,
                                             void* y, float* scale, float* zero_point,
                                             int64_t rows, int64_t cols, double eps, int t,
                                             int bits);
int ofq_ref_glu_gate(const void* matmul_wx, const void* matmul_vx, void* y, int64_t m, int64_t n,
                     int64_t stride, int t, int act);

int ofq_ref_quantize_to_int8(const void* in, const float* scale, int8_t* out, int64_t elem_cnt,
                             int64_t scale_size, int64_t shape0, int t, int bits);

int ofq_ref_matmul_quant(const int8_t* a, const int8_t* b, const float* a_scale,
                         const float* b_scale, const void* bias, void* out, int t, int64_t m,
                         int64_t n, int64_t k);

#ifdef __cplusplus
}
#endif
#endif /* OFQ_ORACLE_H_ */
