// fp32 variants of every op of the library (dtype XMA_ROCM_F32).
//
// The MoE layer is meant to run in bf16/fp16; fp32 is the dtype of parity runs against the CPU path and of the
// reference's own test grid.  These kernels are therefore written for exactness and simplicity, not for the roofline:
// v_mfma_f32_32x32x2_f32 with fp32 operands and accumulators (no reduced-precision pass anywhere), 128 x 128 output
// tiles, K steps of 16, operands staged through registers into k-major LDS tiles.  Schedule, operand roles, gather /
// scatter semantics and epilogues are those of the 16-bit kernels in grouped_gemm.hip:
//   forward / dX :  Q = activation rows (tokens),  P = weight rows (output features)
//   dW           :  Q = dY columns (out features), P = X columns (in features), K = tokens of the expert
// The MFMA "A" operand is the P fragment, so a lane owns output row (lane & 31) of a 32 x 32 block and four
// consecutive columns per accumulator quad.
#include "fp32.hpp"

namespace {

constexpr int FBM = 128, FBN = 128, FBK = 16;
constexpr int FLD = 132; // floats per k-row of an LDS tile [16 k][128 + 4]: 16-byte aligned rows, conflict-free columns
constexpr int FTHREADS = 256;

typedef float f32x4 __attribute__((ext_vector_type(4)));

struct TileRegs {
    f32x4 v[2];
};

// ---- operand tile loaders: 128 "rows" x 16 k per tile, two float4 per thread
// K-contiguous source ([row][k]): thread t -> row t / 2, k = 8 (t & 1) + {0..7}
__device__ __forceinline__ void load_kcontig(TileRegs &r, const float *row_ptr, int k0, int K, int tid) {
    const int kb = k0 + (tid & 1) * 8;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int k = kb + 4 * h;
        r.v[h] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (k < K) r.v[h] = *(const f32x4 *)(row_ptr + k); // K % 4 == 0: a float4 is inside or outside as a whole
    }
}
__device__ __forceinline__ void store_kcontig(float *tile, const TileRegs &r, int tid) {
    const int row = tid >> 1, kb = (tid & 1) * 8;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int q = 0; q < 4; ++q) tile[(kb + 4 * h + q) * FLD + row] = r.v[h][q];
}
// K-strided source ([k][row], rows contiguous): thread t -> k = t / 32 + 8 pass, rows 4 (t & 31) + {0..3}
__device__ __forceinline__ void store_kstrided(float *tile, const TileRegs &r, int tid) {
#pragma unroll
    for (int h = 0; h < 2; ++h) *(f32x4 *)(tile + ((tid >> 5) + 8 * h) * FLD + (tid & 31) * 4) = r.v[h];
}

__device__ __forceinline__ void zero_acc(f32x16 (&acc)[2][2]) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;
}

// the 16 k of the LDS tiles: 8 MFMA steps of k = 2
__device__ __forceinline__ void mma_tiles(const float *sP, const float *sQ, f32x16 (&acc)[2][2], int wp, int wq, int lane) {
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
        const int k = 2 * kk + (lane >> 5);
        float p[2], q[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            p[b] = sP[k * FLD + wp + b * 32 + (lane & 31)];
            q[b] = sQ[k * FLD + wq + b * 32 + (lane & 31)];
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 2; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(p[j], q[i], acc[j][i], 0, 0, 0);
    }
}

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }

// ------------------------------------------------------------------------------------------------ forward / dX
template <int WT, int EPI>
__global__ __launch_bounds__(FTHREADS) void gemm_f32_kernel(const FwdArgs a) {
    extern __shared__ int s_pre[]; // [E + 1]
    __shared__ __attribute__((aligned(16))) float sQ[FBK * FLD];
    __shared__ __attribute__((aligned(16))) float sP[FBK * FLD];
    __shared__ int s_sched[2];
    const float *X = (const float *)a.X, *W = (const float *)a.W, *scale = (const float *)a.scale;
    float *out = (float *)a.out, *aux = (float *)a.aux;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int NT = (a.N + FBN - 1) / FBN;

    // expert-major schedule from the inclusive offsets (one prefix entry per expert, serial scan by thread 0: E is small
    // next to the work of a tile)
    if (tid == 0) {
        int run = 0;
        for (int e = 0; e < a.E; ++e) {
            s_pre[e] = run;
            const int64_t cnt = a.offs[e] - (e ? a.offs[e - 1] : 0);
            run += (int)((cnt + FBM - 1) / FBM) * NT;
        }
        s_pre[a.E] = run;
        s_sched[0] = -1;
    }
    __syncthreads();
    const int L = blockIdx.x;
    for (int e = tid; e < a.E; e += FTHREADS)
        if (s_pre[e] <= L && L < s_pre[e + 1]) {
            s_sched[0] = e;
            s_sched[1] = L - s_pre[e];
        }
    __syncthreads();
    const int e = s_sched[0];
    if (e < 0) return; // the grid is an upper bound
    const int64_t row_lo = e ? a.offs[e - 1] : 0, row_hi = a.offs[e];
    const int tiles_m = (int)((row_hi - row_lo + FBM - 1) / FBM);
    const int64_t row0 = row_lo + (int64_t)(s_sched[1] % tiles_m) * FBM;
    const int n0 = (s_sched[1] / tiles_m) * FBN;
    const int rows_valid = (int)((row_hi - row0 < FBM) ? row_hi - row0 : FBM);

    // loader set-up
    const float *q_row; // this thread's activation row (K-contiguous source)
    {
        int r = tid >> 1;
        if (r >= rows_valid) r = rows_valid - 1; // duplicates, masked at the store
        const int64_t n = row0 + r;
        const int64_t src = a.x_grouped ? n : a.idx[n] / a.fan_out;
        q_row = X + src * a.ldx;
    }
    const float *We = W + (int64_t)e * a.w_es;
    const float *p_row = nullptr; // WT == 0: weight row n0 + tid / 2
    int p_col = 0;                // WT == 1: first of this thread's 4 columns
    if (WT == 0) {
        int r = n0 + (tid >> 1);
        if (r >= a.N) r = a.N - 1;
        p_row = We + (int64_t)r * a.ldw;
    } else {
        p_col = n0 + (tid & 31) * 4;
        if (p_col >= a.N) p_col = a.N - 4; // masked at the store
    }
    auto load_p = [&](TileRegs &r, int k0) {
        if (WT == 0) {
            load_kcontig(r, p_row, k0, a.K, tid);
        } else {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int k = k0 + (tid >> 5) + 8 * h;
                r.v[h] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (k < a.K) r.v[h] = *(const f32x4 *)(We + (int64_t)k * a.ldw + p_col);
            }
        }
    };

    f32x16 acc[2][2];
    zero_acc(acc);
    const int wq = (wave & 1) * 64, wp = (wave >> 1) * 64;
    if (a.bias) { // the expert's bias is the first term of every sum (see the epilogue for a lane's columns)
        const float *b = (const float *)a.bias + (int64_t)e * a.bias_es;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                int col = n0 + wp + j * 32 + g * 8 + (lane >> 5) * 4;
                if (col > a.N - 4) col = a.N - 4;
                const f32x4 v = *(const f32x4 *)(b + col);
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q) acc[j][i][4 * g + q] = v[q];
            }
    }
    const int KT = (a.K + FBK - 1) / FBK;
    TileRegs rq, rp;
    load_kcontig(rq, q_row, 0, a.K, tid);
    load_p(rp, 0);
    for (int kt = 0; kt < KT; ++kt) {
        __syncthreads(); // the previous step's fragments have been read
        store_kcontig(sQ, rq, tid);
        if (WT == 0)
            store_kcontig(sP, rp, tid);
        else
            store_kstrided(sP, rp, tid);
        __syncthreads();
        if (kt + 1 < KT) { // next step's loads fly while this one multiplies
            load_kcontig(rq, q_row, (kt + 1) * FBK, a.K, tid);
            load_p(rp, (kt + 1) * FBK);
        }
        mma_tiles(sP, sQ, acc, wp, wq, lane);
    }

    // epilogue: lane owns row (lane & 31) of each 32-row block, 4 consecutive columns per quad
    const int lrow = lane & 31, lhalf = lane >> 5;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = wq + i * 32 + lrow;
        if (r >= rows_valid) continue;
        const int64_t n = row0 + r;
        int64_t sidx = 0;
        if (!a.y_grouped || scale) sidx = a.idx[n];
        const int64_t dst = a.y_grouped ? n : sidx;
        const float sc = scale ? scale[sidx] : 1.f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = n0 + wp + j * 32 + g * 8 + lhalf * 4;
                if (col >= a.N) continue;
                const f32x4 v = {acc[j][i][4 * g] * sc, acc[j][i][4 * g + 1] * sc, acc[j][i][4 * g + 2] * sc,
                                 acc[j][i][4 * g + 3] * sc};
                if (EPI == XMA_ROCM_EPI_STORE) {
                    *(f32x4 *)(out + dst * a.ldo + col) = v;
                } else if (EPI == XMA_ROCM_EPI_SWIGLU) {
                    if (out) *(f32x4 *)(out + dst * a.ldo + col) = v;
                    // columns are (gate, up, gate, up)
                    float2 h = {v[1] * v[0] * sigmoid_f32(v[0]), v[3] * v[2] * sigmoid_f32(v[2])};
                    *(float2 *)(aux + dst * a.ldaux + (col >> 1)) = h;
                } else { // SWIGLU_BWD: v = d h of 4 columns; z and dz have 8 columns (g, u) x 4, grouped rows
                    const f32x4 z0 = *(const f32x4 *)(aux + n * a.ldaux + 2 * col);
                    const f32x4 z1 = *(const f32x4 *)(aux + n * a.ldaux + 2 * col + 4);
                    const float zz[8] = {z0[0], z0[1], z0[2], z0[3], z1[0], z1[1], z1[2], z1[3]};
                    float o[8];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float gg = zz[2 * q], uu = zz[2 * q + 1];
                        const float sg = sigmoid_f32(gg), silu = gg * sg;
                        o[2 * q] = v[q] * uu * (sg + silu * (1.f - sg));
                        o[2 * q + 1] = v[q] * silu;
                    }
                    *(f32x4 *)(out + n * a.ldo + 2 * col) = f32x4{o[0], o[1], o[2], o[3]};
                    *(f32x4 *)(out + n * a.ldo + 2 * col + 4) = f32x4{o[4], o[5], o[6], o[7]};
                }
            }
    }
}

// ------------------------------------------------------------------------------------------------ dW
__global__ __launch_bounds__(FTHREADS) void dw_f32_kernel(const DwArgs a) {
    __shared__ __attribute__((aligned(16))) float sQ[FBK * FLD];
    __shared__ __attribute__((aligned(16))) float sP[FBK * FLD];
    const float *DY = (const float *)a.DY, *X = (const float *)a.X, *scale = (const float *)a.scale;
    float *DW = (float *)a.DW;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int OT = (a.N_out + FBM - 1) / FBM, IT = (a.K_in + FBN - 1) / FBN;
    const int e = blockIdx.x / (OT * IT), rem = blockIdx.x % (OT * IT);
    const int o0 = (rem / IT) * FBM, i0 = (rem % IT) * FBN;
    const int64_t row_lo = e ? a.offs[e - 1] : 0, row_hi = a.offs[e];
    const int rows = (int)(row_hi - row_lo);
    const int KT = (rows + FBK - 1) / FBK;
    int q_col = o0 + (tid & 31) * 4, p_col = i0 + (tid & 31) * 4;
    if (q_col >= a.N_out) q_col = a.N_out - 4; // masked at the store
    if (p_col >= a.K_in) p_col = a.K_in - 4;

    // k-rows are tokens of the expert: thread t takes rows t / 32 and t / 32 + 8 of a step, through the index if the
    // operand is in scattered order; dY may carry a per-token scale
    auto load_tiles = [&](TileRegs &rq, TileRegs &rp, int k0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = k0 + (tid >> 5) + 8 * h;
            rq.v[h] = f32x4{0.f, 0.f, 0.f, 0.f};
            rp.v[h] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (k < rows) {
                const int64_t n = row_lo + k;
                int64_t sidx = 0;
                if (!a.dy_grouped || !a.x_grouped || scale) sidx = a.idx[n];
                const int64_t dsrc = a.dy_grouped ? n : sidx / a.dy_fan_out;
                const int64_t xsrc = a.x_grouped ? n : sidx / a.x_fan_out;
                rq.v[h] = *(const f32x4 *)(DY + dsrc * a.lddy + q_col);
                if (scale) rq.v[h] *= scale[sidx];
                rp.v[h] = *(const f32x4 *)(X + xsrc * a.ldx + p_col);
            }
        }
    };

    f32x16 acc[2][2];
    zero_acc(acc);
    const int wq = (wave & 1) * 64, wp = (wave >> 1) * 64;
    TileRegs rq, rp;
    if (KT > 0) load_tiles(rq, rp, 0);
    for (int kt = 0; kt < KT; ++kt) {
        __syncthreads();
        store_kstrided(sQ, rq, tid);
        store_kstrided(sP, rp, tid);
        __syncthreads();
        if (kt + 1 < KT) load_tiles(rq, rp, (kt + 1) * FBK);
        mma_tiles(sP, sQ, acc, wp, wq, lane);
    }
    // every element of DW[e] is written, zeros for an expert without tokens
    const int lrow = lane & 31, lhalf = lane >> 5;
    float *DWe = DW + (int64_t)e * a.dw_es;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int o = o0 + wq + i * 32 + lrow;
        if (o >= a.N_out) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = i0 + wp + j * 32 + g * 8 + lhalf * 4;
                if (col >= a.K_in) continue;
                *(f32x4 *)(DWe + (int64_t)o * a.lddw + col) =
                    f32x4{acc[j][i][4 * g], acc[j][i][4 * g + 1], acc[j][i][4 * g + 2], acc[j][i][4 * g + 3]};
            }
    }
}

// ------------------------------------------------------------------------------------------------ elementwise
// one thread per float4 of the output
__global__ __launch_bounds__(FTHREADS) void combine_f32_kernel(const float *in, int64_t ld_in, const float *w, float *y,
                                                                int64_t ldy, int64_t T, int k, int cpr) {
    const int64_t id = (int64_t)blockIdx.x * FTHREADS + threadIdx.x;
    if (id >= T * cpr) return;
    const int64_t t = id / cpr;
    const int c = (int)(id % cpr) * 4;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
        const float s = w ? w[t * k + j] : 1.f;
        acc += s * *(const f32x4 *)(in + (t * k + j) * ld_in + c);
    }
    *(f32x4 *)(y + t * ldy + c) = acc;
}

// one wave per (token, slot): d_w[t, j] = <in[t k + j, :], dy[t, :]>
__global__ __launch_bounds__(FTHREADS) void combine_bwd_f32_kernel(const float *in, int64_t ld_in, const float *dy,
                                                                    int64_t lddy, float *d_w, int64_t rows, int k, int H) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (FTHREADS / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t t = row / k;
    float acc = 0.f;
    for (int c = lane * 4; c < H; c += 256) {
        const f32x4 x = *(const f32x4 *)(in + row * ld_in + c), g = *(const f32x4 *)(dy + t * lddy + c);
        acc += x[0] * g[0] + x[1] * g[1] + x[2] * g[2] + x[3] * g[3];
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) acc += __shfl_down(acc, d);
    if (lane == 0) d_w[row] = acc;
}

__global__ __launch_bounds__(FTHREADS) void group_f32_kernel(const float *A, int64_t lda, const int64_t *idx, float *out,
                                                              int64_t ldo, const float *coeff, int64_t M, int cpr,
                                                              int fan_out) {
    const int64_t id = (int64_t)blockIdx.x * FTHREADS + threadIdx.x;
    if (id >= M * cpr) return;
    const int64_t n = id / cpr;
    const int c = (int)(id % cpr) * 4;
    const int64_t s = idx[n];
    f32x4 v = *(const f32x4 *)(A + (s / fan_out) * lda + c);
    if (coeff) v *= coeff[s];
    *(f32x4 *)(out + n * ldo + c) = v;
}

// y[r, c] = up * gate * sigmoid(gate), x = (gate, up) interleaved; one thread per 4 outputs
__global__ __launch_bounds__(FTHREADS) void swiglu_fwd_f32_kernel(const float *x, int64_t ldx, float *y, int64_t ldy,
                                                                   int64_t rows, int cpr) {
    const int64_t id = (int64_t)blockIdx.x * FTHREADS + threadIdx.x;
    if (id >= rows * cpr) return;
    const int64_t r = id / cpr;
    const int c = (int)(id % cpr) * 4;
    const f32x4 a = *(const f32x4 *)(x + r * ldx + 2 * c), b = *(const f32x4 *)(x + r * ldx + 2 * c + 4);
    *(f32x4 *)(y + r * ldy + c) = f32x4{a[1] * a[0] * sigmoid_f32(a[0]), a[3] * a[2] * sigmoid_f32(a[2]),
                                        b[1] * b[0] * sigmoid_f32(b[0]), b[3] * b[2] * sigmoid_f32(b[2])};
}

__global__ __launch_bounds__(FTHREADS) void swiglu_bwd_f32_kernel(const float *x, int64_t ldx, const float *dy, int64_t lddy,
                                                                   float *dx, int64_t lddx, int64_t rows, int cpr) {
    const int64_t id = (int64_t)blockIdx.x * FTHREADS + threadIdx.x;
    if (id >= rows * cpr) return;
    const int64_t r = id / cpr;
    const int c = (int)(id % cpr) * 4;
    const f32x4 d = *(const f32x4 *)(dy + r * lddy + c);
    const f32x4 a = *(const f32x4 *)(x + r * ldx + 2 * c), b = *(const f32x4 *)(x + r * ldx + 2 * c + 4);
    const float zz[8] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    float o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float gg = zz[2 * q], uu = zz[2 * q + 1];
        const float sg = sigmoid_f32(gg), silu = gg * sg;
        o[2 * q] = d[q] * uu * (sg + silu * (1.f - sg));
        o[2 * q + 1] = d[q] * silu;
    }
    *(f32x4 *)(dx + r * lddx + 2 * c) = f32x4{o[0], o[1], o[2], o[3]};
    *(f32x4 *)(dx + r * lddx + 2 * c + 4) = f32x4{o[4], o[5], o[6], o[7]};
}

inline int blocks_for(int64_t work) { return (int)((work + FTHREADS - 1) / FTHREADS); }

template <int WT> int launch_gemm(const FwdArgs &a, int epi, int grid, size_t lds, hipStream_t st) {
    if (epi == XMA_ROCM_EPI_STORE)
        gemm_f32_kernel<WT, XMA_ROCM_EPI_STORE><<<grid, FTHREADS, lds, st>>>(a);
    else if (epi == XMA_ROCM_EPI_SWIGLU)
        gemm_f32_kernel<WT, XMA_ROCM_EPI_SWIGLU><<<grid, FTHREADS, lds, st>>>(a);
    else
        gemm_f32_kernel<WT, XMA_ROCM_EPI_SWIGLU_BWD><<<grid, FTHREADS, lds, st>>>(a);
    return xma_check_launch("gemm_f32_kernel");
}

} // namespace

int f32_scatter2scatter(const FwdArgs &a, int w_is_kn, int epilogue, hipStream_t st) {
    const int64_t grid = (a.M / FBM + a.E) * ((a.N + FBN - 1) / FBN); // sum_e ceil(c_e / 128) <= floor(M / 128) + E
    XMA_REQUIRE(grid < ((int64_t)1 << 31), XMA_ROCM_EUNSUPPORTED, "scatter2scatter (fp32): grid too large");
    XMA_REQUIRE(a.E <= 8192, XMA_ROCM_EUNSUPPORTED, "scatter2scatter (fp32): E=%d > 8192", a.E);
    const size_t lds = (size_t)(a.E + 1) * sizeof(int);
    return w_is_kn ? launch_gemm<1>(a, epilogue, (int)grid, lds, st) : launch_gemm<0>(a, epilogue, (int)grid, lds, st);
}

int f32_group_bwd_W(const DwArgs &a, hipStream_t st) {
    const int64_t grid = (int64_t)a.E * ((a.N_out + FBM - 1) / FBM) * ((a.K_in + FBN - 1) / FBN);
    XMA_REQUIRE(grid < ((int64_t)1 << 31), XMA_ROCM_EUNSUPPORTED, "group_bwd_W (fp32): grid too large");
    dw_f32_kernel<<<(int)grid, FTHREADS, 0, st>>>(a);
    return xma_check_launch("dw_f32_kernel");
}

int f32_combine(const void *in, int64_t ld_in, const void *w, void *y, int64_t ldy, int64_t T, int k, int H, hipStream_t st) {
    const int cpr = H / 4;
    combine_f32_kernel<<<blocks_for(T * cpr), FTHREADS, 0, st>>>((const float *)in, ld_in, (const float *)w, (float *)y, ldy,
                                                                 T, k, cpr);
    return xma_check_launch("combine_f32_kernel");
}

int f32_combine_bwd(const void *in, int64_t ld_in, const void *dy, int64_t lddy, void *d_w, int64_t T, int k, int H,
                    hipStream_t st) {
    const int64_t rows = T * k;
    const int64_t blocks = (rows + (FTHREADS / 64) - 1) / (FTHREADS / 64);
    combine_bwd_f32_kernel<<<(int)blocks, FTHREADS, 0, st>>>((const float *)in, ld_in, (const float *)dy, lddy, (float *)d_w,
                                                             rows, k, H);
    return xma_check_launch("combine_bwd_f32_kernel");
}

int f32_group(const void *A, int64_t lda, const int64_t *idx, void *out, int64_t ldo, const void *coeff, int64_t M, int K,
              int fan_out, hipStream_t st) {
    const int cpr = K / 4;
    group_f32_kernel<<<blocks_for(M * cpr), FTHREADS, 0, st>>>((const float *)A, lda, idx, (float *)out, ldo,
                                                               (const float *)coeff, M, cpr, fan_out);
    return xma_check_launch("group_f32_kernel");
}

int f32_swiglu_packed_forward(const void *x, int64_t ldx, void *y, int64_t ldy, int64_t rows, int cols_out, hipStream_t st) {
    const int cpr = cols_out / 4;
    swiglu_fwd_f32_kernel<<<blocks_for(rows * cpr), FTHREADS, 0, st>>>((const float *)x, ldx, (float *)y, ldy, rows, cpr);
    return xma_check_launch("swiglu_fwd_f32_kernel");
}

int f32_swiglu_packed_backward(const void *x, int64_t ldx, const void *dy, int64_t lddy, void *dx, int64_t lddx, int64_t rows,
                               int cols_out, hipStream_t st) {
    const int cpr = cols_out / 4;
    swiglu_bwd_f32_kernel<<<blocks_for(rows * cpr), FTHREADS, 0, st>>>((const float *)x, ldx, (const float *)dy, lddy,
                                                                       (float *)dx, lddx, rows, cpr);
    return xma_check_launch("swiglu_bwd_f32_kernel");
}
