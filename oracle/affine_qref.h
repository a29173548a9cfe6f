/*
 * affine_qref.h -- C interface of the CPU parity oracle (test infrastructure
 * only; the product library never links it).  See affine_qref.c for the
 * reference lines each function follows.
 *
 * dtype: 0 = float32, 1 = float16, 2 = bfloat16 (16-bit types are passed as
 * raw uint16_t storage).  Functions return 0, or -1 for an unsupported
 * bits / group_size / dtype.
 */
#ifndef AFFINE_QREF_H
#define AFFINE_QREF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { QREF_F32 = 0, QREF_F16 = 1, QREF_BF16 = 2 };

uint16_t qref_bf16_from_f32(float x);
float qref_bf16_to_f32(uint16_t b);
uint16_t qref_f16_from_f32(float x);
float qref_f16_to_f32(uint16_t h);

int qref_pack_factor(int bits, int wsize);
int qref_bytes_per_pack(int bits, int wsize);

/* w: w_size elements; out: w_size*bits/8 bytes; scales/biases: w_size/group_size */
int qref_quantize(
    const void* w,
    void* out,
    void* scales,
    void* biases,
    int bits,
    int group_size,
    size_t w_size,
    int dtype);

int qref_dequantize(
    const uint32_t* wq,
    const void* scales,
    const void* biases,
    void* out,
    size_t n_elems,
    int group_size,
    int bits,
    int dtype);

/* transposed_w != 0: w [N, K*bits/32], scales/biases [N, K/group_size]
 * transposed_w == 0: w [K, N*bits/32], scales/biases [K, N/group_size] */
int qref_qmm(
    void* result,
    const void* x,
    const uint32_t* w,
    const void* scales,
    const void* biases,
    int M,
    int N,
    int K,
    int group_size,
    int bits,
    int transposed_w,
    int dtype);

/* strides in elements (uint32 words for w); w/sb stride 0 broadcasts w */
int qref_qmm_batched(
    void* result,
    const void* x,
    const uint32_t* w,
    const void* scales,
    const void* biases,
    int M,
    int N,
    int K,
    int batch,
    size_t x_batch_stride,
    size_t w_batch_stride,
    size_t sb_batch_stride,
    int group_size,
    int bits,
    int transposed_w,
    int dtype);

int qref_gather_qmm(
    void* result,
    const void* x,
    const uint32_t* w,
    const void* scales,
    const void* biases,
    const uint32_t* lhs_indices,
    const uint32_t* rhs_indices,
    int n_indices,
    int M,
    int N,
    int K,
    size_t x_batch_stride,
    size_t w_batch_stride,
    size_t sb_batch_stride,
    int group_size,
    int bits,
    int transposed_w,
    int dtype);

#ifdef __cplusplus
}
#endif
#endif
