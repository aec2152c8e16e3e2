// Gradient of the experts' bias: per-expert column sums of a row-major matrix whose rows are taken in grouped order
// (optionally through the scattered index, optionally times a per-row scale).  HBM-bound: every row is read once.
#include "common.hpp"

namespace {

constexpr int CS_THREADS = 256;
constexpr int CS_COLS = 128;                   // columns per workgroup: a wave reads 256 (fp32: 512) contiguous bytes of a row
constexpr int CS_PHASES = CS_THREADS / WAVE;   // rows a workgroup has in flight per step (times the unroll)

template <typename T> struct Pair; // two neighbouring elements of a row as floats
template <> struct Pair<float> {
    static __device__ __forceinline__ float2 load(const void *row, int c) { return *(const float2 *)((const float *)row + c); }
    static __device__ __forceinline__ float scalar(const void *v, int64_t i) { return ((const float *)v)[i]; }
    static __device__ __forceinline__ void store(void *row, int c, float a, float b) { *(float2 *)((float *)row + c) = make_float2(a, b); }
};
template <> struct Pair<__bf16> {
    static __device__ __forceinline__ float2 load(const void *row, int c) {
        const uint32_t w = *(const uint32_t *)((const uint16_t *)row + c);
        return make_float2(Elem<__bf16>::lo(w), Elem<__bf16>::hi(w));
    }
    static __device__ __forceinline__ float scalar(const void *v, int64_t i) { return Elem<__bf16>::lo(((const uint16_t *)v)[i]); }
    static __device__ __forceinline__ void store(void *row, int c, float a, float b) {
        *(uint32_t *)((uint16_t *)row + c) = Elem<__bf16>::pack(a, b);
    }
};
template <> struct Pair<_Float16> {
    static __device__ __forceinline__ float2 load(const void *row, int c) {
        const uint32_t w = *(const uint32_t *)((const uint16_t *)row + c);
        return make_float2(Elem<_Float16>::lo(w), Elem<_Float16>::hi(w));
    }
    static __device__ __forceinline__ float scalar(const void *v, int64_t i) { return Elem<_Float16>::lo(((const uint16_t *)v)[i]); }
    static __device__ __forceinline__ void store(void *row, int c, float a, float b) {
        *(uint32_t *)((uint16_t *)row + c) = Elem<_Float16>::pack(a, b);
    }
};

// out[e, c] = sum over the grouped rows n of expert e of A[src(n), c] * scale[idx[n]], src(n) = n (idx == NULL) or
// idx[n] / fan_out.  Workgroup (column block, expert); the rows are dealt to the four waves round-robin and added in a
// fixed order (per wave in row order, then the waves in order), so the result does not depend on timing.  Experts
// without rows get zeros.
template <typename T>
__global__ __launch_bounds__(CS_THREADS) void expert_column_sums_kernel(const void *__restrict__ A, int64_t lda,
                                                                        const int64_t *__restrict__ idx, FastDiv fan_div,
                                                                        const void *__restrict__ scale,
                                                                        const int64_t *__restrict__ offs, void *__restrict__ out,
                                                                        int64_t ldo, int N) {
    __shared__ float2 s_part[CS_PHASES][WAVE];
    constexpr int ES = sizeof(T);
    const int e = blockIdx.y, lane = threadIdx.x & 63, phase = threadIdx.x >> 6;
    int c = blockIdx.x * CS_COLS + 2 * lane;
    const bool col_ok = c < N;
    if (!col_ok) c = N - 2; // clamped, never stored
    const int64_t lo = e ? offs[e - 1] : 0, hi = offs[e];
    float s0 = 0.f, s1 = 0.f;
    for (int64_t r0 = lo + phase; r0 < hi; r0 += 4 * CS_PHASES) {
        float2 v[4];
        float w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t r = r0 + u * CS_PHASES;
            v[u] = make_float2(0.f, 0.f);
            w[u] = 1.f;
            if (r < hi) {
                int64_t src = r;
                if (idx) {
                    const int64_t s = idx[r];
                    src = fastdiv((uint32_t)s, fan_div);
                    if (scale) w[u] = Pair<T>::scalar(scale, s);
                }
                v[u] = Pair<T>::load((const char *)A + src * lda * ES, c);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) s0 += v[u].x * w[u], s1 += v[u].y * w[u];
    }
    s_part[phase][lane] = make_float2(s0, s1);
    __syncthreads();
    if (phase == 0 && col_ok) {
        float a = 0.f, b = 0.f;
#pragma unroll
        for (int p = 0; p < CS_PHASES; ++p) a += s_part[p][lane].x, b += s_part[p][lane].y;
        Pair<T>::store((char *)out + (int64_t)e * ldo * ES, c, a, b);
    }
}

} // namespace

extern "C" int xma_rocm_expert_column_sums(const void *A, int64_t lda, const int64_t *sorted_scattered_idxs, int32_t fan_out,
                                           const void *row_scale, const int64_t *expert_offsets, void *out, int64_t ldo,
                                           int32_t N, int32_t E, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED,
                "expert_column_sums: dtype %d", dtype);
    XMA_REQUIRE(N >= 2 && N % 2 == 0 && E >= 1 && E <= 65535 && fan_out >= 1 && lda % 2 == 0 && ldo % 2 == 0 && lda >= N && ldo >= N,
                XMA_ROCM_EINVAL, "expert_column_sums: N=%d E=%d fan_out=%d lda=%lld ldo=%lld (N and the leading dimensions even)", N,
                E, fan_out, (long long)lda, (long long)ldo);
    XMA_REQUIRE(A && expert_offsets && out && ((uintptr_t)A & 7) == 0 && ((uintptr_t)out & 7) == 0, XMA_ROCM_EINVAL,
                "expert_column_sums: null or misaligned pointer");
    XMA_REQUIRE(!row_scale || sorted_scattered_idxs, XMA_ROCM_EINVAL,
                "expert_column_sums: the row scale is indexed through sorted_scattered_idxs");
    const dim3 grid((N + CS_COLS - 1) / CS_COLS, E);
    hipStream_t st = (hipStream_t)stream;
    const FastDiv fd = make_fastdiv((uint32_t)fan_out);
    if (dtype == XMA_ROCM_BF16)
        expert_column_sums_kernel<__bf16><<<grid, CS_THREADS, 0, st>>>(A, lda, sorted_scattered_idxs, fd, row_scale, expert_offsets, out, ldo, N);
    else if (dtype == XMA_ROCM_F16)
        expert_column_sums_kernel<_Float16><<<grid, CS_THREADS, 0, st>>>(A, lda, sorted_scattered_idxs, fd, row_scale, expert_offsets, out, ldo, N);
    else
        expert_column_sums_kernel<float><<<grid, CS_THREADS, 0, st>>>(A, lda, sorted_scattered_idxs, fd, row_scale, expert_offsets, out, ldo, N);
    return xma_check_launch("expert_column_sums_kernel");
}
