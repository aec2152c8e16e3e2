// Stand-alone SwiGLU with separate gate and up operands, y = up * gate * sigmoid(gate), and its closed-form
// backward, for bf16 / fp16 / fp32 and any 2-D size; plus the any-width form of the packed variant (gate = even columns,
// up = odd columns), which the 16-byte kernels of elementwise.hip and fp32.hip do not cover.
//
// HBM-bound (forward 3, backward 5 elements of traffic per element).  Rows whose starts are 16-byte aligned (all
// leading dimensions multiples of 16 bytes) go through 16-byte accesses, one per lane and operand, over the largest
// multiple of 16 bytes of the width; what is left of each row, or everything if rows are not aligned, is done one element
// per lane.  All arithmetic in fp32, one rounding at the end.
#include "common.hpp"

namespace {

constexpr int SW_THREADS = 256;

template <typename ST> struct Scalar;
template <> struct Scalar<__bf16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float get(const void *p, int64_t i) { return (float)((const __bf16 *)p)[i]; }
    static __device__ __forceinline__ void put(void *p, int64_t i, float v) { ((__bf16 *)p)[i] = (__bf16)v; }
    static __device__ __forceinline__ float sigmoid(float x) { return sigmoidf_fast(x); }
};
template <> struct Scalar<_Float16> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float get(const void *p, int64_t i) { return (float)((const _Float16 *)p)[i]; }
    static __device__ __forceinline__ void put(void *p, int64_t i, float v) { ((_Float16 *)p)[i] = (_Float16)v; }
    static __device__ __forceinline__ float sigmoid(float x) { return sigmoidf_fast(x); }
};
template <> struct Scalar<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ float get(const void *p, int64_t i) { return ((const float *)p)[i]; }
    static __device__ __forceinline__ void put(void *p, int64_t i, float v) { ((float *)p)[i] = v; }
    static __device__ __forceinline__ float sigmoid(float x) { return 1.0f / (1.0f + __expf(-x)); } // IEEE division
};

template <typename ST> struct Vec {
    static constexpr int N = Scalar<ST>::VEC;
    float v[N];
    static __device__ __forceinline__ Vec load(const void *p, int64_t i) {
        Vec r;
        const u32x4 w = __builtin_nontemporal_load((const u32x4 *)((const ST *)p + i));
        if constexpr (N == 4) {
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            const f32x4 f = __builtin_bit_cast(f32x4, w); // (a bit cast of a single vector element reads element 0)
#pragma unroll
            for (int q = 0; q < 4; ++q) r.v[q] = f[q];
        } else {
            typedef ST st8 __attribute__((ext_vector_type(8)));
            const st8 h = __builtin_bit_cast(st8, w);
#pragma unroll
            for (int q = 0; q < 8; ++q) r.v[q] = (float)h[q];
        }
        return r;
    }
    __device__ __forceinline__ void store(void *p, int64_t i) const {
        u32x4 w;
        if constexpr (N == 4) {
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            f32x4 f;
#pragma unroll
            for (int q = 0; q < 4; ++q) f[q] = v[q];
            w = __builtin_bit_cast(u32x4, f);
        } else {
            typedef ST st8 __attribute__((ext_vector_type(8)));
            st8 h;
#pragma unroll
            for (int q = 0; q < 8; ++q) h[q] = (ST)v[q];
            w = __builtin_bit_cast(u32x4, h);
        }
        __builtin_nontemporal_store(w, (u32x4 *)((ST *)p + i));
    }
};

template <typename ST> __device__ __forceinline__ float fwd_one(float g, float u) { return u * g * Scalar<ST>::sigmoid(g); }
template <typename ST> __device__ __forceinline__ void bwd_one(float g, float u, float d, float &dg, float &du) {
    const float s = Scalar<ST>::sigmoid(g), silu = g * s;
    dg = d * u * (s + silu * (1.f - s));
    du = d * silu;
}

// columns [0, vcols) of every row, vcols a multiple of VEC: one 16-byte access per lane and operand
template <typename ST>
__global__ __launch_bounds__(SW_THREADS) void swiglu_fwd_vec_kernel(const void *g, int64_t ldg, const void *u, int64_t ldu,
                                                                    void *y, int64_t ldy, int64_t rows, int vchunks,
                                                                    FastDiv vdiv) {
    constexpr int N = Scalar<ST>::VEC;
    const int64_t t = (int64_t)blockIdx.x * SW_THREADS + threadIdx.x;
    if (t >= rows * vchunks) return;
    int64_t r;
    int c;
    split_row(t, vchunks, vdiv, r, c);
    c *= N;
    const Vec<ST> a = Vec<ST>::load(g, r * ldg + c), b = Vec<ST>::load(u, r * ldu + c);
    Vec<ST> o;
#pragma unroll
    for (int q = 0; q < N; ++q) o.v[q] = fwd_one<ST>(a.v[q], b.v[q]);
    o.store(y, r * ldy + c);
}

template <typename ST>
__global__ __launch_bounds__(SW_THREADS) void swiglu_bwd_vec_kernel(const void *g, int64_t ldg, const void *u, int64_t ldu,
                                                                    const void *dy, int64_t lddy, void *dg, int64_t lddg,
                                                                    void *du, int64_t lddu, int64_t rows, int vchunks,
                                                                    FastDiv vdiv) {
    constexpr int N = Scalar<ST>::VEC;
    const int64_t t = (int64_t)blockIdx.x * SW_THREADS + threadIdx.x;
    if (t >= rows * vchunks) return;
    int64_t r;
    int c;
    split_row(t, vchunks, vdiv, r, c);
    c *= N;
    const Vec<ST> a = Vec<ST>::load(g, r * ldg + c), b = Vec<ST>::load(u, r * ldu + c), d = Vec<ST>::load(dy, r * lddy + c);
    Vec<ST> og, ou;
#pragma unroll
    for (int q = 0; q < N; ++q) bwd_one<ST>(a.v[q], b.v[q], d.v[q], og.v[q], ou.v[q]);
    og.store(dg, r * lddg + c);
    ou.store(du, r * lddu + c);
}

// columns [c0, cols) of every row, one element per lane.  STEP = 1: separate operands; STEP = 2: g and u are the same
// packed tensor (gate at 2 c, up at 2 c + 1), and so are dg and du.
template <typename ST, int STEP>
__global__ __launch_bounds__(SW_THREADS) void swiglu_fwd_elem_kernel(const void *g, int64_t ldg, const void *u, int64_t ldu,
                                                                     void *y, int64_t ldy, int64_t rows, int c0, int cols,
                                                                     FastDiv wdiv) {
    const int w = cols - c0;
    const int64_t t = (int64_t)blockIdx.x * SW_THREADS + threadIdx.x;
    if (t >= rows * w) return;
    int64_t r;
    int c;
    split_row(t, w, wdiv, r, c);
    c += c0;
    const float a = Scalar<ST>::get(g, r * ldg + STEP * c), b = Scalar<ST>::get(u, r * ldu + STEP * c + (STEP - 1));
    Scalar<ST>::put(y, r * ldy + c, fwd_one<ST>(a, b));
}

template <typename ST, int STEP>
__global__ __launch_bounds__(SW_THREADS) void swiglu_bwd_elem_kernel(const void *g, int64_t ldg, const void *u, int64_t ldu,
                                                                     const void *dy, int64_t lddy, void *dg, int64_t lddg,
                                                                     void *du, int64_t lddu, int64_t rows, int c0, int cols,
                                                                     FastDiv wdiv) {
    const int w = cols - c0;
    const int64_t t = (int64_t)blockIdx.x * SW_THREADS + threadIdx.x;
    if (t >= rows * w) return;
    int64_t r;
    int c;
    split_row(t, w, wdiv, r, c);
    c += c0;
    const float a = Scalar<ST>::get(g, r * ldg + STEP * c), b = Scalar<ST>::get(u, r * ldu + STEP * c + (STEP - 1));
    float og, ou;
    bwd_one<ST>(a, b, Scalar<ST>::get(dy, r * lddy + c), og, ou);
    Scalar<ST>::put(dg, r * lddg + STEP * c, og);
    Scalar<ST>::put(du, r * lddu + STEP * c + (STEP - 1), ou);
}

inline int64_t blocks_of(int64_t work) { return (work + SW_THREADS - 1) / SW_THREADS; }
inline bool fits_grid(int64_t work) { return blocks_of(work) < ((int64_t)1 << 31); }

template <typename ST>
int fwd_launch(const void *g, int64_t ldg, const void *u, int64_t ldu, void *y, int64_t ldy, int64_t rows, int cols,
               bool rows_aligned, hipStream_t st) {
    constexpr int N = Scalar<ST>::VEC;
    const int vcols = rows_aligned ? cols / N * N : 0;
    if (vcols) {
        swiglu_fwd_vec_kernel<ST><<<(unsigned)blocks_of(rows * (vcols / N)), SW_THREADS, 0, st>>>(g, ldg, u, ldu, y, ldy, rows,
                                                                                                 vcols / N, make_fastdiv(vcols / N));
        int rc = xma_check_launch("swiglu_fwd_vec_kernel");
        if (rc) return rc;
    }
    if (vcols < cols) {
        swiglu_fwd_elem_kernel<ST, 1><<<(unsigned)blocks_of(rows * (cols - vcols)), SW_THREADS, 0, st>>>(g, ldg, u, ldu, y, ldy,
                                                                                                        rows, vcols, cols, make_fastdiv(cols - vcols));
        return xma_check_launch("swiglu_fwd_elem_kernel");
    }
    return XMA_ROCM_OK;
}

template <typename ST>
int bwd_launch(const void *g, int64_t ldg, const void *u, int64_t ldu, const void *dy, int64_t lddy, void *dg, int64_t lddg,
               void *du, int64_t lddu, int64_t rows, int cols, bool rows_aligned, hipStream_t st) {
    constexpr int N = Scalar<ST>::VEC;
    const int vcols = rows_aligned ? cols / N * N : 0;
    if (vcols) {
        swiglu_bwd_vec_kernel<ST><<<(unsigned)blocks_of(rows * (vcols / N)), SW_THREADS, 0, st>>>(
            g, ldg, u, ldu, dy, lddy, dg, lddg, du, lddu, rows, vcols / N, make_fastdiv(vcols / N));
        int rc = xma_check_launch("swiglu_bwd_vec_kernel");
        if (rc) return rc;
    }
    if (vcols < cols) {
        swiglu_bwd_elem_kernel<ST, 1><<<(unsigned)blocks_of(rows * (cols - vcols)), SW_THREADS, 0, st>>>(
            g, ldg, u, ldu, dy, lddy, dg, lddg, du, lddu, rows, vcols, cols, make_fastdiv(cols - vcols));
        return xma_check_launch("swiglu_bwd_elem_kernel");
    }
    return XMA_ROCM_OK;
}

inline int elem_bytes(int dtype) { return dtype == XMA_ROCM_F32 ? 4 : 2; }
inline bool aligned_rows(const void *p, int64_t ld, int dtype) {
    return ((uintptr_t)p & 15) == 0 && (ld * elem_bytes(dtype)) % 16 == 0;
}
inline bool aligned_elem(const void *p, int dtype) { return ((uintptr_t)p % elem_bytes(dtype)) == 0; }

} // namespace

extern "C" int xma_rocm_swiglu_forward(const void *gate, int64_t ld_gate, const void *up, int64_t ld_up, void *y, int64_t ldy,
                                       int64_t rows, int32_t cols, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED,
                "swiglu: dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && cols >= 1 && ld_gate >= cols && ld_up >= cols && ldy >= cols, XMA_ROCM_EINVAL,
                "swiglu: rows=%lld cols=%d ld=(%lld, %lld, %lld)", (long long)rows, cols, (long long)ld_gate, (long long)ld_up,
                (long long)ldy);
    if (rows == 0) return XMA_ROCM_OK;
    XMA_REQUIRE(gate && up && y && aligned_elem(gate, dtype) && aligned_elem(up, dtype) && aligned_elem(y, dtype),
                XMA_ROCM_EINVAL, "swiglu: null or misaligned pointer");
    XMA_REQUIRE(fits_grid(rows * cols), XMA_ROCM_EUNSUPPORTED, "swiglu: too large");
    const bool al = aligned_rows(gate, ld_gate, dtype) && aligned_rows(up, ld_up, dtype) && aligned_rows(y, ldy, dtype);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == XMA_ROCM_BF16) return fwd_launch<__bf16>(gate, ld_gate, up, ld_up, y, ldy, rows, cols, al, st);
    if (dtype == XMA_ROCM_F16) return fwd_launch<_Float16>(gate, ld_gate, up, ld_up, y, ldy, rows, cols, al, st);
    return fwd_launch<float>(gate, ld_gate, up, ld_up, y, ldy, rows, cols, al, st);
}

extern "C" int xma_rocm_swiglu_backward(const void *gate, int64_t ld_gate, const void *up, int64_t ld_up, const void *dy,
                                        int64_t lddy, void *d_gate, int64_t ld_dgate, void *d_up, int64_t ld_dup, int64_t rows,
                                        int32_t cols, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED,
                "swiglu_bwd: dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && cols >= 1 && ld_gate >= cols && ld_up >= cols && lddy >= cols && ld_dgate >= cols &&
                    ld_dup >= cols,
                XMA_ROCM_EINVAL, "swiglu_bwd: rows=%lld cols=%d", (long long)rows, cols);
    if (rows == 0) return XMA_ROCM_OK;
    XMA_REQUIRE(gate && up && dy && d_gate && d_up && aligned_elem(gate, dtype) && aligned_elem(up, dtype) &&
                    aligned_elem(dy, dtype) && aligned_elem(d_gate, dtype) && aligned_elem(d_up, dtype),
                XMA_ROCM_EINVAL, "swiglu_bwd: null or misaligned pointer");
    XMA_REQUIRE(fits_grid(rows * cols), XMA_ROCM_EUNSUPPORTED, "swiglu_bwd: too large");
    const bool al = aligned_rows(gate, ld_gate, dtype) && aligned_rows(up, ld_up, dtype) && aligned_rows(dy, lddy, dtype) &&
                    aligned_rows(d_gate, ld_dgate, dtype) && aligned_rows(d_up, ld_dup, dtype);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == XMA_ROCM_BF16)
        return bwd_launch<__bf16>(gate, ld_gate, up, ld_up, dy, lddy, d_gate, ld_dgate, d_up, ld_dup, rows, cols, al, st);
    if (dtype == XMA_ROCM_F16)
        return bwd_launch<_Float16>(gate, ld_gate, up, ld_up, dy, lddy, d_gate, ld_dgate, d_up, ld_dup, rows, cols, al, st);
    return bwd_launch<float>(gate, ld_gate, up, ld_up, dy, lddy, d_gate, ld_dgate, d_up, ld_dup, rows, cols, al, st);
}

// packed form, output columns [c0, cols_out) one element per lane (elementwise.hip forwards here for the columns its
// 16-byte kernels leave over, or for everything when rows are not 16-byte aligned)
int xma_swiglu_packed_forward_elems(const void *x, int64_t ldx, void *y, int64_t ldy, int64_t rows, int c0, int cols_out,
                                    int dtype, hipStream_t st) {
    if (c0 >= cols_out || rows == 0) return XMA_ROCM_OK;
    const unsigned grid = (unsigned)blocks_of(rows * (cols_out - c0));
    if (dtype == XMA_ROCM_BF16)
        swiglu_fwd_elem_kernel<__bf16, 2><<<grid, SW_THREADS, 0, st>>>(x, ldx, x, ldx, y, ldy, rows, c0, cols_out, make_fastdiv(cols_out - c0));
    else if (dtype == XMA_ROCM_F16)
        swiglu_fwd_elem_kernel<_Float16, 2><<<grid, SW_THREADS, 0, st>>>(x, ldx, x, ldx, y, ldy, rows, c0, cols_out, make_fastdiv(cols_out - c0));
    else
        swiglu_fwd_elem_kernel<float, 2><<<grid, SW_THREADS, 0, st>>>(x, ldx, x, ldx, y, ldy, rows, c0, cols_out, make_fastdiv(cols_out - c0));
    return xma_check_launch("swiglu_fwd_elem_kernel (packed)");
}

int xma_swiglu_packed_backward_elems(const void *x, int64_t ldx, const void *dy, int64_t lddy, void *dx, int64_t lddx,
                                     int64_t rows, int c0, int cols_out, int dtype, hipStream_t st) {
    if (c0 >= cols_out || rows == 0) return XMA_ROCM_OK;
    const unsigned grid = (unsigned)blocks_of(rows * (cols_out - c0));
    if (dtype == XMA_ROCM_BF16)
        swiglu_bwd_elem_kernel<__bf16, 2><<<grid, SW_THREADS, 0, st>>>(x, ldx, x, ldx, dy, lddy, dx, lddx, dx, lddx, rows, c0, cols_out, make_fastdiv(cols_out - c0));
    else if (dtype == XMA_ROCM_F16)
        swiglu_bwd_elem_kernel<_Float16, 2><<<grid, SW_THREADS, 0, st>>>(x, ldx, x, ldx, dy, lddy, dx, lddx, dx, lddx, rows, c0, cols_out, make_fastdiv(cols_out - c0));
    else
        swiglu_bwd_elem_kernel<float, 2><<<grid, SW_THREADS, 0, st>>>(x, ldx, x, ldx, dy, lddy, dx, lddx, dx, lddx, rows, c0, cols_out, make_fastdiv(cols_out - c0));
    return xma_check_launch("swiglu_bwd_elem_kernel (packed)");
}
