// Grouped (per-expert, ragged) GEMMs of the MoE layer on CDNA4 MFMA.
//
// One workgroup = 256 threads = 4 waves (2 x 2), output tile 256 x 256, K step 64.
// Each wave owns 128 x 128 = 4 x 4 v_mfma_f32_32x32x16 tiles (256 fp32 accumulators per lane).
// Operand tiles live in LDS as [256 rows][64 k] 16-bit elements, 16-byte chunks XOR-swizzled,
// double buffered (2 x 64 KB); global loads for step s+1 are issued before the MFMAs of step
// s and written to the other buffer behind them, one barrier per K step.
//
// MFMA operand roles: the "P" tile supplies the rows of the 32x32 result (register dimension:
// a lane holds 4 consecutive P indices per accumulator quad) and the "Q" tile supplies its
// columns (lane % 32).  P is always the dimension that is contiguous in the OUTPUT, so a lane
// stores 8 contiguous bytes per quad and owns one output row: gather/scatter indices, row
// scales and the SwiGLU pairs (adjacent columns) are all lane-local.
//
//   forward / dX :  Q = activation rows (tokens),     P = weight rows (output features)
//   dW           :  Q = dY columns (out features),    P = X columns (in features), K = tokens
//
// Tiles never straddle experts: the schedule is expert-major, derived on the device from the
// inclusive expert offsets in each workgroup's prologue (no host read of the counts).
#include "common.hpp"

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int THREADS = 256;
constexpr int TILE_CHUNKS = 256 * 8;                              // 16-byte chunks per operand tile
constexpr int SMEM_BYTES = 2 /*stages*/ * 2 /*operands*/ * TILE_CHUNKS * 16; // 128 KB

struct FwdArgs {
    const uint16_t *X;
    int64_t ldx;
    const uint16_t *W;
    int64_t w_es, ldw;
    const int64_t *idx;
    const int64_t *offs;
    uint16_t *out;
    int64_t ldo;
    uint16_t *aux;
    int64_t ldaux;
    const uint16_t *scale;
    int64_t M;
    int N, K, E, fan_out, x_grouped, y_grouped;
};

struct DwArgs {
    const uint16_t *DY;
    int64_t lddy;
    const uint16_t *X;
    int64_t ldx;
    const uint16_t *scale;
    const int64_t *idx;
    const int64_t *offs;
    uint16_t *DW;
    int64_t dw_es, lddw;
    int N_out, K_in, E, dy_grouped, dy_fan_out, x_grouped, x_fan_out;
};

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Inside every aligned run of
// 256 ids give each XCD 32 consecutive logical tiles, so tiles that share operand panels
// meet in one XCD's L2.
__device__ __forceinline__ int xcd_remap(int bid, int grid) {
    const int full = grid & ~255;
    if (bid >= full) return bid;
    const int w = bid & 255;
    return (bid & ~255) + (w & 7) * 32 + (w >> 3);
}

// One K step of MFMA work for a wave: 4 k16 sub-steps x (4 P fragments, 4 Q fragments, 16 MFMAs).
template <typename T>
__device__ __forceinline__ void mma_tile(const u32x4 *__restrict__ sP, const u32x4 *__restrict__ sQ, int p_row0,
                                         int q_row0, int lane, f32x16 (&acc)[4][4]) {
    const int r = lane & 31, kc = lane >> 5;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
        u32x4 pf[4], qf[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            pf[i] = sP[lds_chunk(p_row0 + i * 32 + r, kk * 2 + kc)];
            qf[i] = sQ[lds_chunk(q_row0 + i * 32 + r, kk * 2 + kc)];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[j][i] = Elem<T>::mfma(pf[j], qf[i], acc[j][i]);
    }
}

// ------------------------------------------------------------------------------------------------
// forward / dX kernel
//   WT = 0: W[e] is (N, K) with K contiguous (x @ W^T)      -> P tile loaded row-major
//   WT = 1: W[e] is (K, N) with N contiguous (dy @ W)       -> P tile transposed in registers
// ------------------------------------------------------------------------------------------------
template <typename T, int WT, int EPI>
__global__ __launch_bounds__(THREADS, 1) void grouped_gemm_kernel(const FwdArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int s_sched[4];
    u32x4 *tiles = (u32x4 *)smem;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int NT = (a.N + BN - 1) / BN;

    // ---- expert-major schedule: work[e] = ceil(rows_e / BM) * NT, prefix, locate this tile
    int *s_pre = (int *)smem; // [E + 1], dead before the first tile store
    if (tid == 0) s_sched[0] = -1;
    if (wave == 0) {
        int carry = 0;
        for (int b = 0; b < a.E; b += WAVE) {
            const int e = b + lane;
            int v = 0;
            if (e < a.E) {
                const int64_t cnt = a.offs[e] - (e ? a.offs[e - 1] : 0);
                v = (int)((cnt + BM - 1) / BM) * NT;
            }
            int s = v;
#pragma unroll
            for (int d = 1; d < WAVE; d <<= 1) {
                const int t = __shfl_up(s, d);
                if (lane >= d) s += t;
            }
            if (e < a.E) s_pre[e] = carry + s - v;
            carry += __shfl(s, WAVE - 1);
        }
        if (lane == 0) s_pre[a.E] = carry;
    }
    __syncthreads();
    const int L = xcd_remap(blockIdx.x, gridDim.x);
    for (int e = tid; e < a.E; e += THREADS)
        if (s_pre[e] <= L && L < s_pre[e + 1]) {
            s_sched[0] = e;
            s_sched[1] = L - s_pre[e];
        }
    __syncthreads();
    const int e = s_sched[0];
    if (e < 0) return; // beyond the last tile (the grid is an upper bound)
    const int64_t row_lo = e ? a.offs[e - 1] : 0, row_hi = a.offs[e];
    const int tiles_m = (int)((row_hi - row_lo + BM - 1) / BM);
    const int m_tile = s_sched[1] % tiles_m, n_tile = s_sched[1] / tiles_m;
    const int64_t row0 = row_lo + (int64_t)m_tile * BM;
    const int rows_valid = (int)((row_hi - row0 < BM) ? row_hi - row0 : BM);
    const int n0 = n_tile * BN;
    __syncthreads(); // s_pre is dead from here on

    // ---- loader set-up
    // row-major loader: thread -> chunk (tid & 7) of rows (tid >> 3) + 32 i
    const int lc = tid & 7, lr = tid >> 3;
    const uint16_t *q_ptr[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int r = lr + 32 * i;
        if (r >= rows_valid) r = rows_valid - 1; // duplicates, masked at the store
        const int64_t n = row0 + r;
        const int64_t src = a.x_grouped ? n : a.idx[n] / a.fan_out;
        q_ptr[i] = a.X + src * a.ldx + lc * 8;
    }
    const uint16_t *We = a.W + (int64_t)e * a.w_es;
    const uint16_t *p_ptr[8];
    // transposing loader: thread -> 8 k-rows (8 * (tid >> 5) + j) x 8 columns (8 * (tid & 31))
    const int tc = tid & 31, tk = tid >> 5;
    if (WT == 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int r = n0 + lr + 32 * i;
            if (r >= a.N) r = a.N - 1;
            p_ptr[i] = We + (int64_t)r * a.ldw + lc * 8;
        }
    } else {
        int c = n0 + tc * 8;
        if (c >= a.N) c = a.N - 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) p_ptr[j] = We + (int64_t)(tk * 8 + j) * a.ldw + c;
    }

    u32x4 q_reg[8], p_reg[8];
    const u32x4 zero4 = {0u, 0u, 0u, 0u};

    auto load_tiles = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const bool ok = k0 + lc * 8 < a.K;
            q_reg[i] = ok ? *(const u32x4 *)(q_ptr[i] + k0) : zero4;
        }
        if (WT == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool ok = k0 + lc * 8 < a.K;
                p_reg[i] = ok ? *(const u32x4 *)(p_ptr[i] + k0) : zero4;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const bool ok = k0 + tk * 8 + j < a.K;
                p_reg[j] = ok ? *(const u32x4 *)(p_ptr[j] + (int64_t)k0 * a.ldw) : zero4;
            }
        }
    };
    auto store_tiles = [&](int stage) {
        u32x4 *sQ = tiles + stage * 2 * TILE_CHUNKS, *sP = sQ + TILE_CHUNKS;
#pragma unroll
        for (int i = 0; i < 8; ++i) sQ[lds_chunk(lr + 32 * i, lc)] = q_reg[i];
        if (WT == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) sP[lds_chunk(lr + 32 * i, lc)] = p_reg[i];
        } else {
            u32x4 t[8];
            transpose8x8_b16(p_reg, t);
#pragma unroll
            for (int c = 0; c < 8; ++c) sP[lds_chunk(tc * 8 + c, tk)] = t[c];
        }
    };

    f32x16 acc[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;

    const int wq = (wave & 1) * 128, wp = (wave >> 1) * 128; // wave's 128 x 128 corner inside the tile
    const int KT = (a.K + BK - 1) / BK;

    load_tiles(0);
    store_tiles(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int stage = kt & 1;
        if (kt + 1 < KT) load_tiles((kt + 1) * BK);
        const u32x4 *sQ = tiles + stage * 2 * TILE_CHUNKS, *sP = sQ + TILE_CHUNKS;
        mma_tile<T>(sP, sQ, wp, wq, lane, acc);
        if (kt + 1 < KT) store_tiles(stage ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane owns row (lane & 31) of each 32-row block; quad g of tile (j, i) holds
    //      columns n0 + wp + 32 j + 8 g + 4 (lane >> 5) + {0..3}
    const int lrow = lane & 31, lhalf = lane >> 5;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = wq + i * 32 + lrow;
        if (r >= rows_valid) continue;
        const int64_t n = row0 + r;
        int64_t sidx = 0;
        if (!a.y_grouped || a.scale) sidx = a.idx[n];
        const int64_t dst = a.y_grouped ? n : sidx;
        float sc = 1.f;
        if (a.scale) sc = Elem<T>::lo((uint32_t)a.scale[sidx]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = n0 + wp + j * 32 + g * 8 + lhalf * 4;
                if (col >= a.N) continue;
                const float v0 = acc[j][i][4 * g] * sc, v1 = acc[j][i][4 * g + 1] * sc;
                const float v2 = acc[j][i][4 * g + 2] * sc, v3 = acc[j][i][4 * g + 3] * sc;
                if (EPI == XMA_ROCM_EPI_STORE) {
                    u32x2 o = {Elem<T>::pack(v0, v1), Elem<T>::pack(v2, v3)};
                    *(u32x2 *)(a.out + dst * a.ldo + col) = o;
                } else if (EPI == XMA_ROCM_EPI_SWIGLU) {
                    // columns are (gate, up, gate, up); the activation is taken from the rounded
                    // pre-activations, exactly what a separate pass over the stored z would see
                    const uint32_t z0 = Elem<T>::pack(v0, v1), z1 = Elem<T>::pack(v2, v3);
                    if (a.out) {
                        u32x2 o = {z0, z1};
                        *(u32x2 *)(a.out + dst * a.ldo + col) = o;
                    }
                    const float g0 = Elem<T>::lo(z0), u0 = Elem<T>::hi(z0);
                    const float g1 = Elem<T>::lo(z1), u1 = Elem<T>::hi(z1);
                    const float h0 = u0 * g0 * sigmoidf_fast(g0), h1 = u1 * g1 * sigmoidf_fast(g1);
                    *(uint32_t *)(a.aux + dst * a.ldaux + (col >> 1)) = Elem<T>::pack(h0, h1);
                } else { // EPI_SWIGLU_BWD: v* = d h for 4 columns; z has 8 columns (g, u) x 4
                    const u32x4 z = *(const u32x4 *)(a.aux + n * a.ldaux + 2 * col);
                    const float dh[4] = {v0, v1, v2, v3};
                    u32x4 o;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float gg = Elem<T>::lo(z[q]), uu = Elem<T>::hi(z[q]);
                        const float s = sigmoidf_fast(gg), silu = gg * s;
                        o[q] = Elem<T>::pack(dh[q] * uu * (s + silu * (1.f - s)), dh[q] * silu);
                    }
                    *(u32x4 *)(a.out + dst * a.ldo + 2 * col) = o;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// dW kernel: DW[e][o][i] = sum_n DY[n][o] X[n][i]; both operands are token-major, so both tiles go
// through the transposing loader; the K loop runs over the expert's row range (zero-filled tail).
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(THREADS, 1) void grouped_gemm_dw_kernel(const DwArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    u32x4 *tiles = (u32x4 *)smem;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int OT = (a.N_out + 255) / 256, IT = (a.K_in + 255) / 256;
    const int L = xcd_remap(blockIdx.x, gridDim.x);
    const int e = L / (OT * IT);
    const int rem = L % (OT * IT);
    const int o0 = (rem / IT) * 256, i0 = (rem % IT) * 256;
    const int64_t row_lo = e ? a.offs[e - 1] : 0, row_hi = a.offs[e];
    const int rows = (int)(row_hi - row_lo);
    const int KT = (rows + BK - 1) / BK;

    const int tc = tid & 31, tk = tid >> 5;
    int oc = o0 + tc * 8, ic = i0 + tc * 8;
    if (oc >= a.N_out) oc = a.N_out - 8;
    if (ic >= a.K_in) ic = a.K_in - 8;

    int64_t nxt_idx[8]; // scattered index of the 8 tokens this thread loads in the NEXT step
    float q_scale[8];
    u32x4 q_reg[8], p_reg[8];
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    const bool need_idx = !a.dy_grouped || !a.x_grouped || a.scale;

    auto load_idx = [&](int kt) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int r = kt * BK + tk * 8 + j;
            nxt_idx[j] = (need_idx && r < rows) ? a.idx[row_lo + r] : 0;
        }
    };
    auto load_tiles = [&](int kt) { // uses nxt_idx of step kt
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int r = kt * BK + tk * 8 + j;
            const bool ok = r < rows;
            const int64_t n = row_lo + r;
            const int64_t dsrc = a.dy_grouped ? n : nxt_idx[j] / a.dy_fan_out;
            const int64_t xsrc = a.x_grouped ? n : nxt_idx[j] / a.x_fan_out;
            q_reg[j] = ok ? *(const u32x4 *)(a.DY + dsrc * a.lddy + oc) : zero4;
            p_reg[j] = ok ? *(const u32x4 *)(a.X + xsrc * a.ldx + ic) : zero4;
            q_scale[j] = (ok && a.scale) ? Elem<T>::lo((uint32_t)a.scale[nxt_idx[j]]) : 1.f;
        }
    };
    auto store_tiles = [&](int stage) {
        u32x4 *sQ = tiles + stage * 2 * TILE_CHUNKS, *sP = sQ + TILE_CHUNKS;
        if (a.scale) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    q_reg[j][q] = Elem<T>::pack(q_scale[j] * Elem<T>::lo(q_reg[j][q]), q_scale[j] * Elem<T>::hi(q_reg[j][q]));
        }
        u32x4 t[8];
        transpose8x8_b16(q_reg, t);
#pragma unroll
        for (int c = 0; c < 8; ++c) sQ[lds_chunk(tc * 8 + c, tk)] = t[c];
        transpose8x8_b16(p_reg, t);
#pragma unroll
        for (int c = 0; c < 8; ++c) sP[lds_chunk(tc * 8 + c, tk)] = t[c];
    };

    f32x16 acc[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;

    const int wq = (wave & 1) * 128, wp = (wave >> 1) * 128;
    if (KT > 0) {
        load_idx(0);
        load_tiles(0);
        if (KT > 1) load_idx(1);
        store_tiles(0);
        __syncthreads();
        for (int kt = 0; kt < KT; ++kt) {
            const int stage = kt & 1;
            if (kt + 1 < KT) load_tiles(kt + 1);
            if (kt + 2 < KT) load_idx(kt + 2);
            const u32x4 *sQ = tiles + stage * 2 * TILE_CHUNKS, *sP = sQ + TILE_CHUNKS;
            mma_tile<T>(sP, sQ, wp, wq, lane, acc);
            if (kt + 1 < KT) store_tiles(stage ^ 1);
            __syncthreads();
        }
    }

    // lane owns DW row o (from the Q tile), 4 consecutive in-features per quad
    const int lrow = lane & 31, lhalf = lane >> 5;
    uint16_t *DWe = a.DW + (int64_t)e * a.dw_es;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int o = o0 + wq + i * 32 + lrow;
        if (o >= a.N_out) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = i0 + wp + j * 32 + g * 8 + lhalf * 4;
                if (col >= a.K_in) continue;
                u32x2 v = {Elem<T>::pack(acc[j][i][4 * g], acc[j][i][4 * g + 1]),
                           Elem<T>::pack(acc[j][i][4 * g + 2], acc[j][i][4 * g + 3])};
                *(u32x2 *)(DWe + (int64_t)o * a.lddw + col) = v;
            }
    }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

template <typename K> int set_smem(K kernel) {
    hipError_t err = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
    if (err != hipSuccess) {
        xma_set_error("hipFuncSetAttribute(max dynamic LDS = %d): %s", SMEM_BYTES, hipGetErrorString(err));
        return XMA_ROCM_ELAUNCH;
    }
    return XMA_ROCM_OK;
}

template <typename T, int WT, int EPI> int launch_fwd(const FwdArgs &a, int grid, hipStream_t st) {
    int rc = set_smem(grouped_gemm_kernel<T, WT, EPI>);
    if (rc) return rc;
    grouped_gemm_kernel<T, WT, EPI><<<grid, THREADS, SMEM_BYTES, st>>>(a);
    return xma_check_launch("grouped_gemm_kernel");
}

template <typename T> int dispatch_fwd(const FwdArgs &a, int wt, int epi, int grid, hipStream_t st) {
    if (wt == 0) {
        if (epi == XMA_ROCM_EPI_STORE) return launch_fwd<T, 0, XMA_ROCM_EPI_STORE>(a, grid, st);
        if (epi == XMA_ROCM_EPI_SWIGLU) return launch_fwd<T, 0, XMA_ROCM_EPI_SWIGLU>(a, grid, st);
        return launch_fwd<T, 0, XMA_ROCM_EPI_SWIGLU_BWD>(a, grid, st);
    }
    if (epi == XMA_ROCM_EPI_STORE) return launch_fwd<T, 1, XMA_ROCM_EPI_STORE>(a, grid, st);
    if (epi == XMA_ROCM_EPI_SWIGLU) return launch_fwd<T, 1, XMA_ROCM_EPI_SWIGLU>(a, grid, st);
    return launch_fwd<T, 1, XMA_ROCM_EPI_SWIGLU_BWD>(a, grid, st);
}

} // namespace

extern "C" int xma_rocm_scatter2scatter(const void *X, int64_t ldx, const void *W, int64_t w_expert_stride, int64_t ldw,
                                        int w_is_kn, const int64_t *sorted_scattered_idxs,
                                        const int64_t *expert_offsets, void *out, int64_t ldo, void *aux, int64_t ldaux,
                                        const void *row_scale, int64_t M, int32_t N, int32_t K, int32_t E,
                                        int32_t fan_out, int x_grouped, int y_grouped, int epilogue, int dtype,
                                        void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16, XMA_ROCM_EUNSUPPORTED, "scatter2scatter: dtype %d", dtype);
    XMA_REQUIRE(epilogue >= XMA_ROCM_EPI_STORE && epilogue <= XMA_ROCM_EPI_SWIGLU_BWD, XMA_ROCM_EINVAL,
                "scatter2scatter: epilogue %d", epilogue);
    XMA_REQUIRE(M >= 0 && M < ((int64_t)1 << 31) && N >= 8 && K >= 8 && E >= 1 && fan_out >= 1, XMA_ROCM_EINVAL,
                "scatter2scatter: M=%lld N=%d K=%d E=%d fan_out=%d", (long long)M, N, K, E, fan_out);
    XMA_REQUIRE(N % 8 == 0 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldo % 8 == 0 && w_expert_stride % 8 == 0,
                XMA_ROCM_EUNSUPPORTED, "scatter2scatter: N=%d K=%d ldx=%lld ldw=%lld ldo=%lld must be multiples of 8", N,
                K, (long long)ldx, (long long)ldw, (long long)ldo);
    XMA_REQUIRE(E <= 16384, XMA_ROCM_EUNSUPPORTED, "scatter2scatter: E=%d > 16384", E);
    if (M == 0) return XMA_ROCM_OK;
    XMA_REQUIRE(X && W && expert_offsets && aligned16(X) && aligned16(W), XMA_ROCM_EINVAL,
                "scatter2scatter: null or misaligned operand");
    XMA_REQUIRE(sorted_scattered_idxs || (x_grouped && y_grouped && !row_scale), XMA_ROCM_EINVAL,
                "scatter2scatter: sorted_scattered_idxs is required unless everything is grouped");
    if (epilogue == XMA_ROCM_EPI_STORE) {
        XMA_REQUIRE(out && aligned16(out), XMA_ROCM_EINVAL, "scatter2scatter: out is null or misaligned");
    } else if (epilogue == XMA_ROCM_EPI_SWIGLU) {
        XMA_REQUIRE(aux && aligned16(aux) && ldaux % 8 == 0 && N % 16 == 0, XMA_ROCM_EINVAL,
                    "scatter2scatter: SWIGLU needs aux (M, N/2), ldaux %% 8 == 0, N %% 16 == 0");
        XMA_REQUIRE(!out || aligned16(out), XMA_ROCM_EINVAL, "scatter2scatter: misaligned out");
    } else {
        XMA_REQUIRE(out && aux && aligned16(out) && aligned16(aux) && ldaux % 8 == 0 && y_grouped, XMA_ROCM_EINVAL,
                    "scatter2scatter: SWIGLU_BWD needs out, aux (z) and y_grouped");
    }
    FwdArgs a;
    a.X = (const uint16_t *)X;
    a.ldx = ldx;
    a.W = (const uint16_t *)W;
    a.w_es = w_expert_stride;
    a.ldw = ldw;
    a.idx = sorted_scattered_idxs;
    a.offs = expert_offsets;
    a.out = (uint16_t *)out;
    a.ldo = ldo;
    a.aux = (uint16_t *)aux;
    a.ldaux = ldaux;
    a.scale = (const uint16_t *)row_scale;
    a.M = M;
    a.N = N;
    a.K = K;
    a.E = E;
    a.fan_out = fan_out;
    a.x_grouped = x_grouped;
    a.y_grouped = y_grouped;
    const int64_t NT = (N + BN - 1) / BN;
    const int64_t max_m_tiles = M / BM + E; // sum_e ceil(c_e / BM) <= floor(M / BM) + E
    const int64_t grid = max_m_tiles * NT;
    XMA_REQUIRE(grid < ((int64_t)1 << 31), XMA_ROCM_EUNSUPPORTED, "scatter2scatter: grid too large");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == XMA_ROCM_BF16) return dispatch_fwd<__bf16>(a, w_is_kn ? 1 : 0, epilogue, (int)grid, st);
    return dispatch_fwd<_Float16>(a, w_is_kn ? 1 : 0, epilogue, (int)grid, st);
}

extern "C" int xma_rocm_group_bwd_W(const void *DY, int64_t lddy, int dy_grouped, int32_t dy_fan_out,
                                    const void *dy_scale, const void *X, int64_t ldx, int x_grouped, int32_t x_fan_out,
                                    const int64_t *sorted_scattered_idxs, const int64_t *expert_offsets, void *DW,
                                    int64_t dw_expert_stride, int64_t lddw, int32_t N_out, int32_t K_in, int32_t E,
                                    int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16, XMA_ROCM_EUNSUPPORTED, "group_bwd_W: dtype %d", dtype);
    XMA_REQUIRE(N_out >= 8 && K_in >= 8 && E >= 1 && dy_fan_out >= 1 && x_fan_out >= 1, XMA_ROCM_EINVAL,
                "group_bwd_W: N_out=%d K_in=%d E=%d", N_out, K_in, E);
    XMA_REQUIRE(N_out % 8 == 0 && K_in % 8 == 0 && lddy % 8 == 0 && ldx % 8 == 0 && lddw % 8 == 0 &&
                    dw_expert_stride % 8 == 0,
                XMA_ROCM_EUNSUPPORTED, "group_bwd_W: N_out=%d K_in=%d and leading dimensions must be multiples of 8",
                N_out, K_in);
    XMA_REQUIRE(DY && X && DW && expert_offsets && aligned16(DY) && aligned16(X) && aligned16(DW), XMA_ROCM_EINVAL,
                "group_bwd_W: null or misaligned operand");
    XMA_REQUIRE(sorted_scattered_idxs || (dy_grouped && x_grouped && !dy_scale), XMA_ROCM_EINVAL,
                "group_bwd_W: sorted_scattered_idxs is required unless everything is grouped");
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
    const int64_t grid = (int64_t)E * ((N_out + 255) / 256) * ((K_in + 255) / 256);
    XMA_REQUIRE(grid < ((int64_t)1 << 31), XMA_ROCM_EUNSUPPORTED, "group_bwd_W: grid too large");
    hipStream_t st = (hipStream_t)stream;
    int rc;
    if (dtype == XMA_ROCM_BF16) {
        if ((rc = set_smem(grouped_gemm_dw_kernel<__bf16>))) return rc;
        grouped_gemm_dw_kernel<__bf16><<<(int)grid, THREADS, SMEM_BYTES, st>>>(a);
    } else {
        if ((rc = set_smem(grouped_gemm_dw_kernel<_Float16>))) return rc;
        grouped_gemm_dw_kernel<_Float16><<<(int)grid, THREADS, SMEM_BYTES, st>>>(a);
    }
    return xma_check_launch("grouped_gemm_dw_kernel");
}
