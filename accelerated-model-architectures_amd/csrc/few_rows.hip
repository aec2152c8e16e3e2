// Kernels for the few-token regime: every expert has a handful of rows, so a grouped GEMM is a stream over the weights
// (or, for the weight gradient, a stream of stores) with next to no arithmetic.  The 256 x 256 MFMA tiles of
// grouped_gemm.hip are built for arithmetic: with one K step per tile, or one stage of weights in flight per compute unit,
// they move 3.3-3.8 TB/s.  Here the work is laid out for bandwidth: 16 bytes per lane, many short workgroups per compute
// unit, vector FMAs on fp32 accumulators.  Correct for any number of rows, but the cost grows with rows x weights: the
// caller picks these entry points by the total number of rows.
#include "gemm_common.hpp"

namespace {

constexpr int FR_THREADS = 256;
constexpr int FR_NB = 8; // output rows (n) per workgroup of the weight gradient
constexpr int FR_RC = 4; // rows of the expert per step

template <typename T> __device__ __forceinline__ float fr_scalar(const uint16_t *p, int64_t i) { return Elem<T>::lo(p[i]); }

template <typename T> __device__ __forceinline__ void fr_unpack(const u32x4 v, float (&f)[8]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) f[2 * q] = Elem<T>::lo(v[q]), f[2 * q + 1] = Elem<T>::hi(v[q]);
}

// DW[e][n][k] = sum over the rows r of expert e of DY[dsrc(r)][n] * scale[idx[r]] * X[xsrc(r)][k]: an outer product per
// row.  Workgroup = (2048 columns k, FR_NB rows n, expert); a thread owns 8 consecutive k of every n: it loads its 16 bytes
// of each X row once, takes the FR_NB values of DY from LDS, and leaves FR_NB stores of 16 bytes.  fp32 sums in row order.
// Every element of DW is written exactly once, zeros for an expert without rows.
template <typename T> __global__ __launch_bounds__(FR_THREADS) void dw_few_rows_kernel(const DwArgs a) {
    __shared__ float s_dy[2][FR_RC][FR_NB];
    const int e = blockIdx.z, tid = threadIdx.x;
    const int n0 = blockIdx.y * FR_NB;
    const int k0 = (blockIdx.x * FR_THREADS + tid) * 8;
    const bool k_ok = k0 < a.K_in;
    const int64_t lo = e ? a.offs[e - 1] : 0, hi = a.offs[e];
    float acc[FR_NB][8];
#pragma unroll
    for (int j = 0; j < FR_NB; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[j][i] = 0.f;
    int buf = 0;
    for (int64_t r0 = lo; r0 < hi; r0 += FR_RC, buf ^= 1) {
        if (tid < FR_RC * FR_NB) { // the step's FR_RC x FR_NB values of dY, scaled
            const int u = tid / FR_NB, j = tid % FR_NB;
            const int64_t r = r0 + u;
            float v = 0.f;
            if (r < hi && n0 + j < a.N_out) {
                const int64_t s = a.idx ? a.idx[r] : r;
                const int64_t src = a.dy_grouped ? r : (int64_t)fastdiv((uint32_t)s, a.dy_div);
                v = fr_scalar<T>(a.DY, src * a.lddy + n0 + j);
                if (a.scale) v *= fr_scalar<T>(a.scale, s);
            }
            s_dy[buf][u][j] = v;
        }
        u32x4 x[FR_RC];
#pragma unroll
        for (int u = 0; u < FR_RC; ++u) {
            const int64_t r = r0 + u;
            x[u] = u32x4{0u, 0u, 0u, 0u};
            if (r < hi && k_ok) {
                const int64_t src = a.x_grouped ? r : (int64_t)fastdiv((uint32_t)a.idx[r], a.x_div);
                x[u] = *(const u32x4 *)(a.X + src * a.ldx + k0);
            }
        }
        __syncthreads(); // two buffers: the next step's values are written while a slow wave still reads this step's
#pragma unroll
        for (int u = 0; u < FR_RC; ++u) {
            float xf[8];
            fr_unpack<T>(x[u], xf);
#pragma unroll
            for (int j = 0; j < FR_NB; ++j) {
                const float d = s_dy[buf][u][j];
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[j][i] = __builtin_fmaf(d, xf[i], acc[j][i]);
            }
        }
    }
    if (!k_ok) return;
    uint16_t *out = a.DW + (int64_t)e * a.dw_es + k0;
#pragma unroll
    for (int j = 0; j < FR_NB; ++j) {
        if (n0 + j < a.N_out) {
            const u32x4 v = {Elem<T>::pack(acc[j][0], acc[j][1]), Elem<T>::pack(acc[j][2], acc[j][3]),
                             Elem<T>::pack(acc[j][4], acc[j][5]), Elem<T>::pack(acc[j][6], acc[j][7])};
            __builtin_nontemporal_store(v, (u32x4 *)(out + (int64_t)(n0 + j) * a.lddw));
        }
    }
}

} // namespace

extern "C" int xma_rocm_group_bwd_W_few_rows(const void *DY, int64_t lddy, int dy_grouped, int32_t dy_fan_out,
                                             const void *dy_scale, const void *X, int64_t ldx, int x_grouped,
                                             int32_t x_fan_out, const int64_t *sorted_scattered_idxs,
                                             const int64_t *expert_offsets, void *DW, int64_t dw_expert_stride, int64_t lddw,
                                             int32_t N_out, int32_t K_in, int32_t E, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16, XMA_ROCM_EUNSUPPORTED, "group_bwd_W_few_rows: dtype %d", dtype);
    XMA_REQUIRE(N_out >= 1 && K_in >= 8 && E >= 1 && E <= 65535 && dy_fan_out >= 1 && x_fan_out >= 1, XMA_ROCM_EINVAL,
                "group_bwd_W_few_rows: N_out=%d K_in=%d E=%d", N_out, K_in, E);
    XMA_REQUIRE(K_in % 8 == 0 && ldx % 8 == 0 && lddw % 8 == 0 && dw_expert_stride % 8 == 0, XMA_ROCM_EUNSUPPORTED,
                "group_bwd_W_few_rows: K_in=%d, ldx, lddw and the expert stride must be multiples of 8", K_in);
    XMA_REQUIRE(DY && X && DW && expert_offsets && ((uintptr_t)X & 15) == 0 && ((uintptr_t)DW & 15) == 0 &&
                    ((uintptr_t)DY & 1) == 0,
                XMA_ROCM_EINVAL, "group_bwd_W_few_rows: null or misaligned operand");
    XMA_REQUIRE(sorted_scattered_idxs || (dy_grouped && x_grouped && !dy_scale), XMA_ROCM_EINVAL,
                "group_bwd_W_few_rows: sorted_scattered_idxs is required unless everything is grouped");
    const int64_t rows_n = ((int64_t)N_out + FR_NB - 1) / FR_NB;
    XMA_REQUIRE(rows_n <= 65535, XMA_ROCM_EUNSUPPORTED, "group_bwd_W_few_rows: N_out=%d exceeds %d", N_out, 65535 * FR_NB);
    DwArgs a;
    a.DY = (const uint16_t *)DY;
    a.lddy = lddy;
    a.X = (const uint16_t *)X;
    a.ldx = ldx;
    a.scale = (const uint16_t *)dy_scale;
    a.idx = sorted_scattered_idxs;
    a.offs = expert_offsets;
    a.DW = (uint16_t *)DW;
    a.dw_es = dw_expert_stride;
    a.lddw = lddw;
    a.N_out = N_out;
    a.K_in = K_in;
    a.E = E;
    a.dy_grouped = dy_grouped;
    a.dy_fan_out = dy_fan_out;
    a.x_grouped = x_grouped;
    a.x_fan_out = x_fan_out;
    a.dy_div = make_fastdiv((uint32_t)dy_fan_out);
    a.x_div = make_fastdiv((uint32_t)x_fan_out);
    const dim3 grid((K_in / 8 + FR_THREADS - 1) / FR_THREADS, (unsigned)rows_n, E);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == XMA_ROCM_BF16)
        dw_few_rows_kernel<__bf16><<<grid, FR_THREADS, 0, st>>>(a);
    else
        dw_few_rows_kernel<_Float16><<<grid, FR_THREADS, 0, st>>>(a);
    return xma_check_launch("dw_few_rows_kernel");
}
