/*
 * fp_qref.h -- C interface of the CPU parity oracle for the floating-point
 * quantization modes (test infrastructure only; see fp_qref.c for the reference
 * lines each function follows).  dtype as in affine_qref.h.
 */
#ifndef FP_QREF_H
#define FP_QREF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { FPQ_MXFP4 = 0, FPQ_MXFP8 = 1, FPQ_NVFP4 = 2 };

int fpq_group_size(int mode);
int fpq_bits(int mode);
uint8_t fpq_to_fp8(float f);
float fpq_from_fp8(uint8_t x);
uint8_t fpq_e8m0(float x);
uint8_t fpq_e2m1(float x);

/* w: n elements; wq: n * bits / 8 bytes; scales: n / group_size bytes */
int fpq_quantize(const void* w, uint32_t* wq, uint8_t* scales, size_t n, int mode, int dtype);
int fpq_dequantize(
    const uint32_t* wq, const uint8_t* scales, void* out, size_t n, int mode, int dtype);
int fpq_quantize_dequantize(const void* w, void* out, size_t n, int mode, int dtype);
/* transposed_w != 0: w [N, K*bits/32], scales [N, K/gs]; otherwise w [K, N*bits/32],
 * scales [K, N/gs] */
int fpq_qmm(
    void* result, const void* x, const uint32_t* w, const uint8_t* scales, int M, int N, int K,
    int mode, int transposed_w, int dtype);

#ifdef __cplusplus
}
#endif
#endif
