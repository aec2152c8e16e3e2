// HBM-bound row kernels of the MoE path: top-k combine (forward and the router
// weight gradient), the gather copy `group`, and stand-alone packed SwiGLU.
// All move 16 bytes per lane per access and accumulate in fp32.
#include "common.hpp"
#include "fp32.hpp"

namespace {

constexpr int EW_THREADS = 256;

// streaming accesses: data that is read or written exactly once by the kernel
__device__ __forceinline__ u32x4 load_once(const uint16_t *p) { return __builtin_nontemporal_load((const u32x4 *)p); }
__device__ __forceinline__ void store_once(uint16_t *p, u32x4 v) { __builtin_nontemporal_store(v, (u32x4 *)p); }

// y[t, c..c+7] = sum_j w[t, j] * in[t*k + j, c..c+7].  The k rows are fetched four at a time (independent loads in
// flight) and added in slot order, so the result does not depend on the grouping.
template <typename ET>
__global__ __launch_bounds__(EW_THREADS) void combine_kernel(const uint16_t *__restrict__ in, int64_t ld_in,
                                                             const uint16_t *__restrict__ w, uint16_t *__restrict__ y,
                                                             int64_t ldy, int64_t T, int k, int chunks_per_row,
                                                             FastDiv cpr_div) {
    const int64_t g = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x;
    if (g >= T * chunks_per_row) return;
    int64_t t;
    int c;
    split_row(g, chunks_per_row, cpr_div, t, c);
    c *= 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const uint16_t *row = in + t * k * ld_in + c;
    const uint16_t *wt = w ? w + t * k : nullptr;
    auto add = [&](const u32x4 v, float s) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            acc[2 * q] += s * Elem<ET>::lo(v[q]);
            acc[2 * q + 1] += s * Elem<ET>::hi(v[q]);
        }
    };
    int j = 0;
    for (; j + 4 <= k; j += 4) {
        u32x4 v[4];
        float s[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            v[q] = load_once(row + (int64_t)(j + q) * ld_in);
            s[q] = wt ? Elem<ET>::lo((uint32_t)wt[j + q]) : 1.0f;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) add(v[q], s[q]);
    }
    if (j + 2 <= k) {
        const u32x4 v0 = load_once(row + (int64_t)j * ld_in), v1 = load_once(row + (int64_t)(j + 1) * ld_in);
        const float s0 = wt ? Elem<ET>::lo((uint32_t)wt[j]) : 1.0f, s1 = wt ? Elem<ET>::lo((uint32_t)wt[j + 1]) : 1.0f;
        add(v0, s0);
        add(v1, s1);
        j += 2;
    }
    if (j < k) add(load_once(row + (int64_t)j * ld_in), wt ? Elem<ET>::lo((uint32_t)wt[j]) : 1.0f);
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = Elem<ET>::pack(acc[2 * q], acc[2 * q + 1]);
    *(u32x4 *)(y + t * ldy + c) = o;
}

// one wave per (t, j): d_w[t, j] = <in[t*k + j, :], dy[t, :]>; two 16-byte chunks of each row in flight per lane
template <typename ET>
__global__ __launch_bounds__(EW_THREADS) void combine_bwd_kernel(const uint16_t *__restrict__ in, int64_t ld_in,
                                                                 const uint16_t *__restrict__ dy, int64_t lddy,
                                                                 uint16_t *__restrict__ d_w, int64_t Tk, int k, int H,
                                                                 FastDiv k_div) {
    const int lane = threadIdx.x % WAVE;
    const int64_t row = (int64_t)blockIdx.x * (EW_THREADS / WAVE) + threadIdx.x / WAVE;
    if (row >= Tk) return;
    const int64_t t = (row < ((int64_t)1 << 31)) ? (int64_t)fastdiv((uint32_t)row, k_div) : row / k;
    const uint16_t *a_row = in + row * ld_in, *b_row = dy + t * lddy;
    float acc = 0.f;
    auto dot = [&](const u32x4 a, const u32x4 b) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            acc += Elem<ET>::lo(a[q]) * Elem<ET>::lo(b[q]);
            acc += Elem<ET>::hi(a[q]) * Elem<ET>::hi(b[q]);
        }
    };
    int c = lane * 8;
    for (; c + WAVE * 8 < H; c += 2 * WAVE * 8) {
        const u32x4 a0 = load_once(a_row + c), a1 = load_once(a_row + c + WAVE * 8);
        const u32x4 b0 = *(const u32x4 *)(b_row + c), b1 = *(const u32x4 *)(b_row + c + WAVE * 8);
        dot(a0, b0);
        dot(a1, b1);
    }
    if (c < H) dot(load_once(a_row + c), *(const u32x4 *)(b_row + c));
#pragma unroll
    for (int d = WAVE / 2; d > 0; d >>= 1) acc += __shfl_xor(acc, d);
    if (lane == 0) d_w[row] = (uint16_t)(Elem<ET>::pack(acc, 0.f) & 0xffffu);
}

// out[n, :] = A[idx[n] / fan_out, :] * coeff[idx[n]].  A thread moves one 16-byte chunk of GROUP_ROWS consecutive
// output rows: the index, coefficient and data loads of the rows are independent, so each of the three dependent
// round trips is paid once per thread, not once per chunk.
constexpr int GROUP_ROWS = 4;
template <typename ET>
__global__ __launch_bounds__(EW_THREADS) void group_kernel(const uint16_t *__restrict__ A, int64_t lda,
                                                           const int64_t *__restrict__ idx, uint16_t *__restrict__ out,
                                                           int64_t ldo, const uint16_t *__restrict__ coeff, int64_t M,
                                                           int chunks_per_row, int fan_out, FastDiv cpr_div,
                                                           FastDiv fan_div) {
    const int64_t g = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x;
    int64_t n0;
    int c;
    split_row(g, chunks_per_row, cpr_div, n0, c);
    n0 *= GROUP_ROWS;
    if (n0 >= M) return;
    c *= 8;
    int64_t s[GROUP_ROWS];
#pragma unroll
    for (int r = 0; r < GROUP_ROWS; ++r) s[r] = idx[n0 + r < M ? n0 + r : M - 1];
    float f[GROUP_ROWS];
    u32x4 v[GROUP_ROWS];
#pragma unroll
    for (int r = 0; r < GROUP_ROWS; ++r) {
        f[r] = coeff ? Elem<ET>::lo((uint32_t)coeff[s[r]]) : 1.0f;
        const int64_t src = (s[r] < ((int64_t)1 << 31)) ? (int64_t)fastdiv((uint32_t)s[r], fan_div) : s[r] / fan_out;
        v[r] = *(const u32x4 *)(A + src * lda + c);
    }
#pragma unroll
    for (int r = 0; r < GROUP_ROWS; ++r) {
        if (n0 + r >= M) break;
        if (coeff) {
#pragma unroll
            for (int q = 0; q < 4; ++q) v[r][q] = Elem<ET>::pack(f[r] * Elem<ET>::lo(v[r][q]), f[r] * Elem<ET>::hi(v[r][q]));
        }
        store_once(out + (n0 + r) * ldo + c, v[r]);
    }
}

// y[r, c..c+7] from x[r, 2c..2c+15]
template <typename ET>
__global__ __launch_bounds__(EW_THREADS) void swiglu_packed_fwd_kernel(const uint16_t *__restrict__ x, int64_t ldx,
                                                                       uint16_t *__restrict__ y, int64_t ldy,
                                                                       int64_t rows, int chunks_per_row, FastDiv cpr_div) {
    const int64_t g = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x;
    if (g >= rows * chunks_per_row) return;
    int64_t r;
    int c;
    split_row(g, chunks_per_row, cpr_div, r, c);
    c *= 8;
    const u32x4 a = *(const u32x4 *)(x + r * ldx + 2 * c);
    const u32x4 b = *(const u32x4 *)(x + r * ldx + 2 * c + 8);
    float h[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        float g0 = Elem<ET>::lo(a[q]), u0 = Elem<ET>::hi(a[q]);
        float g1 = Elem<ET>::lo(b[q]), u1 = Elem<ET>::hi(b[q]);
        h[q] = u0 * g0 * sigmoidf_fast(g0);
        h[4 + q] = u1 * g1 * sigmoidf_fast(g1);
    }
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = Elem<ET>::pack(h[2 * q], h[2 * q + 1]);
    *(u32x4 *)(y + r * ldy + c) = o;
}

template <typename ET>
__global__ __launch_bounds__(EW_THREADS) void swiglu_packed_bwd_kernel(const uint16_t *__restrict__ x, int64_t ldx,
                                                                       const uint16_t *__restrict__ dy, int64_t lddy,
                                                                       uint16_t *__restrict__ dx, int64_t lddx,
                                                                       int64_t rows, int chunks_per_row, FastDiv cpr_div) {
    const int64_t g = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x;
    if (g >= rows * chunks_per_row) return;
    int64_t r;
    int c;
    split_row(g, chunks_per_row, cpr_div, r, c);
    c *= 8;
    const u32x4 d = *(const u32x4 *)(dy + r * lddy + c);
    float dv[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        dv[2 * q] = Elem<ET>::lo(d[q]);
        dv[2 * q + 1] = Elem<ET>::hi(d[q]);
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const u32x4 a = *(const u32x4 *)(x + r * ldx + 2 * c + 8 * half);
        u32x4 o;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float gg = Elem<ET>::lo(a[q]), uu = Elem<ET>::hi(a[q]), dd = dv[4 * half + q];
            const float s = sigmoidf_fast(gg), silu = gg * s;
            o[q] = Elem<ET>::pack(dd * uu * (s + silu * (1.f - s)), dd * silu);
        }
        *(u32x4 *)(dx + r * lddx + 2 * c + 8 * half) = o;
    }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }
inline int grid_for(int64_t work) { return (int)((work + EW_THREADS - 1) / EW_THREADS); }

} // namespace

#define DISPATCH_T(dtype, ...)                                      \
    do {                                                            \
        if ((dtype) == XMA_ROCM_BF16) {                             \
            typedef __bf16 ET;                                       \
            __VA_ARGS__;                                            \
        } else {                                                    \
            typedef _Float16 ET;                                     \
            __VA_ARGS__;                                            \
        }                                                           \
    } while (0)

extern "C" int xma_rocm_combine(const void *expert_out, int64_t ld_in, const void *w, void *y, int64_t ldy, int64_t T,
                                int32_t k, int32_t H, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED, "combine: dtype %d", dtype);
    XMA_REQUIRE(T >= 0 && k >= 1 && H >= 8 && H % 8 == 0 && ld_in % 8 == 0 && ldy % 8 == 0, XMA_ROCM_EINVAL,
                "combine: T=%lld k=%d H=%d ld_in=%lld ldy=%lld (H, ld %% 8 == 0)", (long long)T, k, H, (long long)ld_in,
                (long long)ldy);
    XMA_REQUIRE(T == 0 || (expert_out && y && aligned16(expert_out) && aligned16(y)), XMA_ROCM_EINVAL,
                "combine: null or misaligned pointer");
    if (T == 0) return XMA_ROCM_OK;
    if (dtype == XMA_ROCM_F32) return f32_combine(expert_out, ld_in, w, y, ldy, T, k, H, (hipStream_t)stream);
    const int cpr = H / 8;
    XMA_REQUIRE(T * cpr < ((int64_t)1 << 31) * EW_THREADS, XMA_ROCM_EUNSUPPORTED, "combine: too large");
    hipStream_t st = (hipStream_t)stream;
    DISPATCH_T(dtype, (combine_kernel<ET><<<grid_for(T * cpr), EW_THREADS, 0, st>>>(
                          (const uint16_t *)expert_out, ld_in, (const uint16_t *)w, (uint16_t *)y, ldy, T, k, cpr,
                          make_fastdiv((uint32_t)cpr))));
    return xma_check_launch("combine_kernel");
}

extern "C" int xma_rocm_combine_bwd(const void *expert_out, int64_t ld_in, const void *dy, int64_t lddy, void *d_w,
                                    int64_t T, int32_t k, int32_t H, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED, "combine_bwd: dtype %d", dtype);
    XMA_REQUIRE(T >= 0 && k >= 1 && H >= 8 && H % 8 == 0 && ld_in % 8 == 0 && lddy % 8 == 0, XMA_ROCM_EINVAL,
                "combine_bwd: T=%lld k=%d H=%d", (long long)T, k, H);
    XMA_REQUIRE(T == 0 || (expert_out && dy && d_w && aligned16(expert_out) && aligned16(dy)), XMA_ROCM_EINVAL,
                "combine_bwd: null or misaligned pointer");
    if (T == 0) return XMA_ROCM_OK;
    if (dtype == XMA_ROCM_F32) return f32_combine_bwd(expert_out, ld_in, dy, lddy, d_w, T, k, H, (hipStream_t)stream);
    const int64_t rows = T * k;
    const int64_t blocks = (rows + (EW_THREADS / WAVE) - 1) / (EW_THREADS / WAVE);
    XMA_REQUIRE(blocks < ((int64_t)1 << 31), XMA_ROCM_EUNSUPPORTED, "combine_bwd: too large");
    hipStream_t st = (hipStream_t)stream;
    DISPATCH_T(dtype, (combine_bwd_kernel<ET><<<(int)blocks, EW_THREADS, 0, st>>>(
                          (const uint16_t *)expert_out, ld_in, (const uint16_t *)dy, lddy, (uint16_t *)d_w, rows, k, H,
                          make_fastdiv((uint32_t)k))));
    return xma_check_launch("combine_bwd_kernel");
}

extern "C" int xma_rocm_group(const void *A, int64_t lda, const int64_t *idx, void *out, int64_t ldo, const void *coeff,
                              int64_t M, int32_t K, int32_t fan_out, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED, "group: dtype %d", dtype);
    XMA_REQUIRE(M >= 0 && K >= 8 && K % 8 == 0 && lda % 8 == 0 && ldo % 8 == 0 && fan_out >= 1, XMA_ROCM_EINVAL,
                "group: M=%lld K=%d fan_out=%d", (long long)M, K, fan_out);
    XMA_REQUIRE(M == 0 || (A && idx && out && aligned16(A) && aligned16(out)), XMA_ROCM_EINVAL,
                "group: null or misaligned pointer");
    if (M == 0) return XMA_ROCM_OK;
    if (dtype == XMA_ROCM_F32) return f32_group(A, lda, idx, out, ldo, coeff, M, K, fan_out, (hipStream_t)stream);
    const int cpr = K / 8;
    hipStream_t st = (hipStream_t)stream;
    DISPATCH_T(dtype, (group_kernel<ET><<<grid_for((M + GROUP_ROWS - 1) / GROUP_ROWS * cpr), EW_THREADS, 0, st>>>(
                          (const uint16_t *)A, lda, idx, (uint16_t *)out, ldo, (const uint16_t *)coeff, M, cpr, fan_out,
                          make_fastdiv((uint32_t)cpr), make_fastdiv((uint32_t)fan_out))));
    return xma_check_launch("group_kernel");
}

// the columns the 16-byte kernels leave over, or everything when rows are not 16-byte aligned (swiglu.hip)
int xma_swiglu_packed_forward_elems(const void *x, int64_t ldx, void *y, int64_t ldy, int64_t rows, int c0, int cols_out,
                                    int dtype, hipStream_t st);
int xma_swiglu_packed_backward_elems(const void *x, int64_t ldx, const void *dy, int64_t lddy, void *dx, int64_t lddx,
                                     int64_t rows, int c0, int cols_out, int dtype, hipStream_t st);

// output columns that the 16-byte kernels take: the largest multiple of 8 (fp32: 4) if every row start is 16-byte aligned
static int packed_vector_cols(int dtype, int cols_out, bool rows_aligned) {
    if (!rows_aligned) return 0;
    return dtype == XMA_ROCM_F32 ? cols_out / 4 * 4 : cols_out / 8 * 8;
}
static bool rows_aligned16(const void *p, int64_t ld, int dtype) {
    return aligned16(p) && (ld * (dtype == XMA_ROCM_F32 ? 4 : 2)) % 16 == 0;
}

extern "C" int xma_rocm_swiglu_packed_forward(const void *x, int64_t ldx, void *y, int64_t ldy, int64_t rows,
                                              int32_t cols_out, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED, "swiglu_packed: dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && cols_out >= 1 && ldx >= 2 * (int64_t)cols_out && ldy >= cols_out, XMA_ROCM_EINVAL,
                "swiglu_packed: rows=%lld cols_out=%d ldx=%lld ldy=%lld", (long long)rows, cols_out, (long long)ldx,
                (long long)ldy);
    const int esz = dtype == XMA_ROCM_F32 ? 4 : 2;
    XMA_REQUIRE(rows == 0 || (x && y && (uintptr_t)x % esz == 0 && (uintptr_t)y % esz == 0), XMA_ROCM_EINVAL,
                "swiglu_packed: null or misaligned pointer");
    if (rows == 0) return XMA_ROCM_OK;
    hipStream_t st = (hipStream_t)stream;
    const int vcols = packed_vector_cols(dtype, cols_out, rows_aligned16(x, ldx, dtype) && rows_aligned16(y, ldy, dtype));
    if (vcols) {
        if (dtype == XMA_ROCM_F32) {
            int rc = f32_swiglu_packed_forward(x, ldx, y, ldy, rows, vcols, st);
            if (rc) return rc;
        } else {
            const int cpr = vcols / 8;
            DISPATCH_T(dtype, (swiglu_packed_fwd_kernel<ET><<<grid_for(rows * cpr), EW_THREADS, 0, st>>>(
                                  (const uint16_t *)x, ldx, (uint16_t *)y, ldy, rows, cpr, make_fastdiv((uint32_t)cpr))));
            int rc = xma_check_launch("swiglu_packed_fwd_kernel");
            if (rc) return rc;
        }
    }
    return xma_swiglu_packed_forward_elems(x, ldx, y, ldy, rows, vcols, cols_out, dtype, st);
}

extern "C" int xma_rocm_swiglu_packed_backward(const void *x, int64_t ldx, const void *dy, int64_t lddy, void *dx,
                                               int64_t lddx, int64_t rows, int32_t cols_out, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED, "swiglu_packed_bwd: dtype %d",
                dtype);
    XMA_REQUIRE(rows >= 0 && cols_out >= 1 && ldx >= 2 * (int64_t)cols_out && lddy >= cols_out && lddx >= 2 * (int64_t)cols_out,
                XMA_ROCM_EINVAL, "swiglu_packed_bwd: rows=%lld cols_out=%d", (long long)rows, cols_out);
    const int esz = dtype == XMA_ROCM_F32 ? 4 : 2;
    XMA_REQUIRE(rows == 0 || (x && dy && dx && (uintptr_t)x % esz == 0 && (uintptr_t)dy % esz == 0 && (uintptr_t)dx % esz == 0),
                XMA_ROCM_EINVAL, "swiglu_packed_bwd: null or misaligned pointer");
    if (rows == 0) return XMA_ROCM_OK;
    hipStream_t st = (hipStream_t)stream;
    const int vcols = packed_vector_cols(
        dtype, cols_out, rows_aligned16(x, ldx, dtype) && rows_aligned16(dy, lddy, dtype) && rows_aligned16(dx, lddx, dtype));
    if (vcols) {
        if (dtype == XMA_ROCM_F32) {
            int rc = f32_swiglu_packed_backward(x, ldx, dy, lddy, dx, lddx, rows, vcols, st);
            if (rc) return rc;
        } else {
            const int cpr = vcols / 8;
            DISPATCH_T(dtype, (swiglu_packed_bwd_kernel<ET><<<grid_for(rows * cpr), EW_THREADS, 0, st>>>(
                                  (const uint16_t *)x, ldx, (const uint16_t *)dy, lddy, (uint16_t *)dx, lddx, rows, cpr,
                                  make_fastdiv((uint32_t)cpr))));
            int rc = xma_check_launch("swiglu_packed_bwd_kernel");
            if (rc) return rc;
        }
    }
    return xma_swiglu_packed_backward_elems(x, ldx, dy, lddy, dx, lddx, rows, vcols, cols_out, dtype, st);
}
