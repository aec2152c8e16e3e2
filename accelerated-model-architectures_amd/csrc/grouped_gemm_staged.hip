// dW grouped GEMM with a per-token scale on dY: register-staged variant.
//
// Both operands are token-major, so each thread loads an 8 (tokens) x 8 (columns) block, applies the scale to the dY
// rows, transposes the block in registers and stores K-contiguous 16-byte chunks to LDS.  Used only when the caller
// passes dy_scale; the unscaled dW, forward and dX GEMMs (grouped_gemm.hip) load straight into LDS instead.
#include "gemm_common.hpp"

namespace xma_rocm {

constexpr int BK = 64;
constexpr int TILE_CHUNKS = 256 * 8;                                          // 16-byte chunks per operand tile
constexpr int GEMM_SMEM_BYTES = 2 /*stages*/ * 2 /*operands*/ * TILE_CHUNKS * 16; // 128 KB of the 160 KB LDS

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

// DW[e][o][i] = sum_n s_n DY[n][o] X[n][i]; the K loop runs over the expert's row range (zero-filled tail).
template <typename T>
__global__ __launch_bounds__(GEMM_THREADS, 1) void grouped_gemm_dw_scaled_kernel(const DwArgs a) {
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
            const int64_t dsrc = a.dy_grouped ? n : (int64_t)fastdiv((uint32_t)nxt_idx[j], a.dy_div);
            const int64_t xsrc = a.x_grouped ? n : (int64_t)fastdiv((uint32_t)nxt_idx[j], a.x_div);
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

} // namespace xma_rocm

int launch_dw_scaled(const DwArgs &a, int dtype, int grid, hipStream_t st) {
    using namespace xma_rocm;
    int rc;
    if (dtype == XMA_ROCM_BF16) {
        if ((rc = gemm_set_smem(grouped_gemm_dw_scaled_kernel<__bf16>, GEMM_SMEM_BYTES))) return rc;
        grouped_gemm_dw_scaled_kernel<__bf16><<<grid, GEMM_THREADS, GEMM_SMEM_BYTES, st>>>(a);
    } else {
        if ((rc = gemm_set_smem(grouped_gemm_dw_scaled_kernel<_Float16>, GEMM_SMEM_BYTES))) return rc;
        grouped_gemm_dw_scaled_kernel<_Float16><<<grid, GEMM_THREADS, GEMM_SMEM_BYTES, st>>>(a);
    }
    return xma_check_launch("grouped_gemm_dw_scaled_kernel");
}
