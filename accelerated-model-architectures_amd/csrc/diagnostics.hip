// Measurement aid, not part of the MoE path: a stream of independent v_mfma_f32_32x32x16_bf16 on every compute unit with
// operands held in registers and no memory traffic in the loop.  Its rate is what the matrix pipes sustain at the
// clock the power limit allows for the given operand bits (all-zero operands toggle nothing and run at the full clock;
// random operands do not), i.e. the ceiling for any kernel that multiplies real data.
#include "common.hpp"

namespace {

__global__ __launch_bounds__(256, 1) void mfma_stream_kernel(const u32x4 *__restrict__ operands, float *__restrict__ out,
                                                             int iters) {
    u32x4 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = operands[i * 256 + threadIdx.x];
        b[i] = operands[(8 + i) * 256 + threadIdx.x];
    }
    f32x16 acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < 64; ++m) acc[m & 15] = Elem<__bf16>::mfma(a[(m >> 2) & 7], b[m & 7], acc[m & 15]);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[i][0];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

} // namespace

extern "C" int xma_rocm_diag_mfma_stream(const void *operands, int32_t iters, float *out, int32_t workgroups, void *stream) {
    XMA_REQUIRE(operands && out && iters >= 1 && workgroups >= 1 && ((uintptr_t)operands & 15) == 0, XMA_ROCM_EINVAL,
                "diag_mfma_stream: operands (16 x 256 x 16 bytes), out (workgroups x 256 floats), iters >= 1");
    mfma_stream_kernel<<<workgroups, 256, 0, (hipStream_t)stream>>>((const u32x4 *)operands, out, iters);
    return xma_check_launch("mfma_stream_kernel");
}
