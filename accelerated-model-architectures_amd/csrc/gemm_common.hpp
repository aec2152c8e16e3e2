// Argument blocks, tile constants and the workgroup -> tile mapping shared by the grouped GEMM kernels.
#pragma once

#include "common.hpp"

constexpr int BM = 256, BN = 256; // output tile of every grouped GEMM kernel
constexpr int GEMM_THREADS = 256;

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
    uint16_t *aux2; // SWIGLU_BWD only, may be NULL: (M, N) = swiglu_packed(z) * row_scale in grouped order
    int64_t ldaux2;
    const uint16_t *scale;
    const uint16_t *bias; // (E, N) added to the product before the epilogue, or NULL
    int64_t bias_es;      // elements between the bias rows of two experts
    int64_t M;
    int N, K, E, fan_out, x_grouped, y_grouped;
    FastDiv fan_div; // division of a scattered index by fan_out (indices are below 2^31)
    float *partial;  // workspace for the K slices of the tiles of the last round, or NULL (no tile is split)
    int split_cus;   // compute units of the device = tiles per round
    int grid_main;   // workgroups that take whole tiles (an upper bound of the tile count); split_cus more follow
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
    FastDiv dy_div, x_div;
};

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Inside every aligned run of 256 ids give each XCD
// 32 consecutive logical tiles, so tiles that share operand panels meet in one XCD's L2.
__device__ __forceinline__ int xcd_remap(int bid, int grid) {
    const int full = grid & ~255;
    if (bid >= full) return bid;
    const int w = bid & 255;
    return (bid & ~255) + (w & 7) * 32 + (w >> 3);
}

// Raises a kernel's dynamic-LDS limit; the attribute belongs to (kernel, device) and is set on the first launch only.
template <typename K> inline int gemm_set_smem(K kernel, int bytes) { return xma_set_max_lds_once((const void *)kernel, bytes); }

// dW with a per-token scale on dY (register-staged loader, grouped_gemm_staged.hip)
int launch_dw_scaled(const DwArgs &a, int dtype, int grid, hipStream_t st);
