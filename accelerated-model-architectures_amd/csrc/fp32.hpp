// fp32 variants of the ops (fp32.hip); the C entry points forward to these for dtype XMA_ROCM_F32 after their argument
// checks.  FwdArgs / DwArgs are shared with the 16-bit kernels: their uint16_t pointers are float pointers here and the
// leading dimensions count floats.
#pragma once

#include "gemm_common.hpp"

int f32_scatter2scatter(const FwdArgs &a, int w_is_kn, int epilogue, hipStream_t st);
int f32_group_bwd_W(const DwArgs &a, hipStream_t st);
int f32_combine(const void *in, int64_t ld_in, const void *w, void *y, int64_t ldy, int64_t T, int k, int H, hipStream_t st);
int f32_combine_bwd(const void *in, int64_t ld_in, const void *dy, int64_t lddy, void *d_w, int64_t T, int k, int H,
                    hipStream_t st);
int f32_group(const void *A, int64_t lda, const int64_t *idx, void *out, int64_t ldo, const void *coeff, int64_t M, int K,
              int fan_out, hipStream_t st);
int f32_swiglu_packed_forward(const void *x, int64_t ldx, void *y, int64_t ldy, int64_t rows, int cols_out, hipStream_t st);
int f32_swiglu_packed_backward(const void *x, int64_t ldx, const void *dy, int64_t lddy, void *dx, int64_t lddx, int64_t rows,
                               int cols_out, hipStream_t st);
