// Kernels for the few-token regime: every expert has a handful of rows, so a grouped GEMM is a stream over the weights
// (or, for the weight gradient, a stream of stores) with next to no arithmetic.  The 256 x 256 MFMA tiles of
// grouped_gemm.hip are built for arithmetic: with one K step per tile, or one stage of weights in flight per compute unit,
// they move 3.3-3.8 TB/s.  Here the work is laid out for bandwidth: 16 bytes per lane, 256 contiguous bytes per row and
// load instruction, many short workgroups per compute unit; vector FMAs for one or two rows per expert, small MFMA tiles
// beyond.  Correct for any number of rows, but the forward-type kernels stream the weights once per 32 rows of an expert:
// the caller picks these entry points by the number of rows per expert.
#include "gemm_common.hpp"

namespace {

constexpr int FR_THREADS = 256;

template <typename T> __device__ __forceinline__ float fr_scalar(const uint16_t *p, int64_t i) { return Elem<T>::lo(p[i]); }

template <typename T> __device__ __forceinline__ void fr_unpack(const u32x4 v, float (&f)[8]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) f[2 * q] = Elem<T>::lo(v[q]), f[2 * q + 1] = Elem<T>::hi(v[q]);
}

// DW[e][n][k] = sum over the rows r of expert e of DY[dsrc(r)][n] * scale[idx[r]] * X[xsrc(r)][k]: MFMAs whose K dimension is
// the expert's rows, 32 at a time, zeros beyond the last.  With few rows the launch is its stores (a vector-FMA version, a
// thread owning 8 k of 8 rows n, was as fast up to 8 rows per expert and three times slower at 32).  Workgroup = a TN x TK
// tile of DW[e] (32 KB of stores) for (k block, n block, expert); the operand tiles are [32 rows][columns] as they lie in
// memory, and ds_read_b64_tr_b16 hands a lane 4 consecutive rows of one column (st_slot_kn and the fragment offsets of
// fr_tile_kernel below).  A wave owns one block of 32 rows n and four blocks of 32 columns k: 4 accumulator blocks, where
// lane l holds row n = l % 32 and quads of 4 consecutive k.  The tile leaves through LDS as whole rows, 16 bytes per lane.
// Any number of rows (more passes), every element written exactly once, zeros for an expert without rows.
constexpr int DT_ROWS = 32, DT_OPERAND = DT_ROWS * 128 * 2; // rows of a pass; bytes of the dY tile [32][128]
constexpr int DW_WIDE_ROWS_PER_EXPERT = 24;              // on average: up to here the 64 x 256 tile
// 16-byte slot of (k-row, chunk) in a tile of 256-byte rows that is read down its columns: chunk c of k-row kr sits at
// c ^ ((kr & 3) << 2)
__device__ __forceinline__ int st_slot_kn(int kr, int chunk) { return kr * 256 + ((chunk ^ ((kr & 3) << 2)) << 4); }

template <typename T, int TN, int TK> __global__ __launch_bounds__(FR_THREADS, 4) void dw_tile_kernel(const DwArgs a) {
    // TN x TK = 16384: TN rows n of DW[e] x TK columns k per workgroup; dY tile [32 rows][128 columns, TN used], X tile
    // [32 rows][TK columns], then the output tile [TN][TK] in their place
    static_assert(TN * TK == 16384 && TN >= 32 && TK >= 128, "a wave owns 4 blocks of 32 x 32");
    // 64 x 256 (512-byte rows out: 87 / 45 instead of 98 / 50 us for dW1 / dW2 of 8 experts of H = 2048, I = 8192) while a
    // pass or two cover an expert; 128 x 128 beyond, whose pass reads 16 KB of operands instead of 20 (32 x 512: the eight
    // gathered rows per thread spill, twice the time)
    constexpr int XROW = 2 * TK, XCH = TK / 8, DYCH = TN / 8, NBN = TN / 32; // bytes and 16-byte chunks per tile row, n blocks
    constexpr int OPERANDS = DT_OPERAND + DT_ROWS * XROW, OUT = TN * TK * 2;
    __shared__ __attribute__((aligned(16))) unsigned char s_t[OPERANDS > OUT ? OPERANDS : OUT];
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4s *lds_v4s;
    const int e = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int k0 = blockIdx.x * TK, n0 = blockIdx.y * TN;
    const int64_t lo = e ? a.offs[e - 1] : 0, hi = a.offs[e];
    const int nb = wave % NBN, kb0 = (wave / NBN) * 4; // this wave's n block and its four k blocks
    // this lane's fragment of column block `blk` of an operand tile, rows 0-3 of its 8 (the other 4: 4 rows on, rows + 16: 16 rows on)
    const int p = lane & 15, G = lane >> 4, kr = ((G >> 1) << 3) + (p >> 2), m_in = ((G & 1) << 4) + ((p & 3) << 2);
    auto frag_off = [&](int blk, int row_bytes) {
        const int m = blk * 32 + m_in;
        return kr * row_bytes + (((m >> 3) ^ ((kr & 3) << 2)) << 4) + ((m & 7) << 1);
    };
    auto frag = [&](const unsigned char *at, int row_bytes) {
        const v4s r03 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)at);
        const v4s r47 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(at + 4 * row_bytes));
        const u32x2 a01 = __builtin_bit_cast(u32x2, r03), a23 = __builtin_bit_cast(u32x2, r47);
        return u32x4{a01[0], a01[1], a23[0], a23[1]};
    };
    f32x16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
    constexpr int DY_IT = (DT_ROWS * DYCH + FR_THREADS - 1) / FR_THREADS, X_IT = DT_ROWS * XCH / FR_THREADS;
    for (int64_t r0 = lo; r0 < hi; r0 += DT_ROWS) {
        u32x4 dyv[DY_IT], xv[X_IT];
#pragma unroll
        for (int i = 0; i < DY_IT; ++i) { // chunk c of the dY tile: row c / DYCH, 16-byte chunk c % DYCH
            const int c = tid + FR_THREADS * i, row = c / DYCH, ch = c % DYCH;
            const int64_t r = r0 + row;
            dyv[i] = u32x4{0u, 0u, 0u, 0u}; // rows past the expert's last add nothing
            if (row < DT_ROWS && r < hi && n0 + 8 * ch < a.N_out) {
                const int64_t s = a.idx ? a.idx[r] : r;
                const int64_t src = a.dy_grouped ? r : (int64_t)fastdiv((uint32_t)s, a.dy_div);
                dyv[i] = *(const u32x4 *)(a.DY + src * a.lddy + n0 + 8 * ch);
                if (a.scale) { // the scaled row rounded to the operand type, as a scaled grouped copy of dY would hold it
                    const float sc = fr_scalar<T>(a.scale, s);
                    float f[8];
                    fr_unpack<T>(dyv[i], f);
#pragma unroll
                    for (int q = 0; q < 4; ++q) dyv[i][q] = Elem<T>::pack(f[2 * q] * sc, f[2 * q + 1] * sc);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < X_IT; ++i) {
            const int c = tid + FR_THREADS * i, row = c / XCH, ch = c % XCH;
            const int64_t r = r0 + row;
            xv[i] = u32x4{0u, 0u, 0u, 0u};
            if (r < hi && k0 + 8 * ch < a.K_in) {
                const int64_t src = a.x_grouped ? r : (int64_t)fastdiv((uint32_t)a.idx[r], a.x_div);
                xv[i] = *(const u32x4 *)(a.X + src * a.ldx + k0 + 8 * ch);
            }
        }
        __syncthreads(); // the pass before no longer reads the tiles
#pragma unroll
        for (int i = 0; i < DY_IT; ++i) {
            const int c = tid + FR_THREADS * i, row = c / DYCH, ch = c % DYCH;
            if (row < DT_ROWS) *(u32x4 *)(s_t + st_slot_kn(row, ch)) = dyv[i];
        }
#pragma unroll
        for (int i = 0; i < X_IT; ++i) {
            const int c = tid + FR_THREADS * i, row = c / XCH, ch = c % XCH;
            *(u32x4 *)(s_t + DT_OPERAND + row * XROW + ((ch ^ ((row & 3) << 2)) << 4)) = xv[i];
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const u32x4 dy_f = frag(s_t + frag_off(nb, 256) + kk * 16 * 256, 256);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[j] = Elem<T>::mfma(frag(s_t + DT_OPERAND + frag_off(kb0 + j, XROW) + kk * 16 * XROW, XROW), dy_f, acc[j]);
        }
    }
    __syncthreads(); // the operand tiles are done with: the output tile takes their place
    // acc[j][4 g + q] = DW[n0 + 32 nb + l32][k0 + 32 (kb0 + j) + 8 g + 4 half + q]; the 16-byte chunk c of row n sits at c ^ (n % 16)
    const int n_l = nb * 32 + l32;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g)
            *(u32x2 *)(s_t + n_l * XROW + (((4 * (kb0 + j) + g) ^ (n_l & 15)) << 4) + 8 * half) =
                u32x2{Elem<T>::pack(acc[j][4 * g], acc[j][4 * g + 1]), Elem<T>::pack(acc[j][4 * g + 2], acc[j][4 * g + 3])};
    __syncthreads();
    uint16_t *out = a.DW + (int64_t)e * a.dw_es + k0;
#pragma unroll
    for (int i = 0; i < 8; ++i) { // whole rows of the tile out: XCH lanes side by side per row
        const int c = tid + FR_THREADS * i, row = c / XCH, ch = c % XCH;
        if (n0 + row < a.N_out && k0 + 8 * ch < a.K_in)
            __builtin_nontemporal_store(*(const u32x4 *)(s_t + row * XROW + ((ch ^ (row & 15)) << 4)),
                                        (u32x4 *)(out + (int64_t)(n0 + row) * a.lddw + 8 * ch));
    }
}

} // namespace

extern "C" int xma_rocm_group_bwd_W_few_rows(const void *DY, int64_t lddy, int dy_grouped, int32_t dy_fan_out,
                                             const void *dy_scale, const void *X, int64_t ldx, int x_grouped,
                                             int32_t x_fan_out, const int64_t *sorted_scattered_idxs,
                                             const int64_t *expert_offsets, void *DW, int64_t dw_expert_stride, int64_t lddw,
                                             int32_t N_out, int32_t K_in, int32_t E, int64_t M, int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16, XMA_ROCM_EUNSUPPORTED, "group_bwd_W_few_rows: dtype %d", dtype);
    XMA_REQUIRE(N_out >= 8 && K_in >= 8 && E >= 1 && E <= 65535 && dy_fan_out >= 1 && x_fan_out >= 1, XMA_ROCM_EINVAL,
                "group_bwd_W_few_rows: N_out=%d K_in=%d E=%d", N_out, K_in, E);
    XMA_REQUIRE(N_out % 8 == 0 && K_in % 8 == 0 && lddy % 8 == 0 && ldx % 8 == 0 && lddw % 8 == 0 && dw_expert_stride % 8 == 0,
                XMA_ROCM_EUNSUPPORTED, "group_bwd_W_few_rows: N_out=%d K_in=%d and the leading dimensions must be multiples of 8",
                N_out, K_in);
    auto al16 = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
    XMA_REQUIRE(DY && X && DW && expert_offsets && al16(DY) && al16(X) && al16(DW), XMA_ROCM_EINVAL,
                "group_bwd_W_few_rows: null or misaligned operand");
    XMA_REQUIRE(sorted_scattered_idxs || (dy_grouped && x_grouped && !dy_scale), XMA_ROCM_EINVAL,
                "group_bwd_W_few_rows: sorted_scattered_idxs is required unless everything is grouped");
    XMA_REQUIRE((N_out + 31) / 32 <= 65535, XMA_ROCM_EUNSUPPORTED, "group_bwd_W_few_rows: N_out=%d exceeds %d", N_out, 65535 * 32);
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
    hipStream_t st = (hipStream_t)stream;
    const bool wide = M > 0 && M <= (int64_t)DW_WIDE_ROWS_PER_EXPERT * E;
    const int TN = wide ? 64 : 128, TK = 16384 / TN;
    const dim3 grid((K_in + TK - 1) / TK, (N_out + TN - 1) / TN, E);
    if (dtype == XMA_ROCM_BF16) {
        if (wide)
            dw_tile_kernel<__bf16, 64, 256><<<grid, FR_THREADS, 0, st>>>(a);
        else
            dw_tile_kernel<__bf16, 128, 128><<<grid, FR_THREADS, 0, st>>>(a);
    } else {
        if (wide)
            dw_tile_kernel<_Float16, 64, 256><<<grid, FR_THREADS, 0, st>>>(a);
        else
            dw_tile_kernel<_Float16, 128, 128><<<grid, FR_THREADS, 0, st>>>(a);
    }
    return xma_check_launch("dw_tile_kernel");
}

namespace {

// ------------------------------------------------------------------------------------------------
// Forward-type product for one or two rows per expert, W[e] as (N, K), K contiguous (x @ W^T): acc[r][n] = sum_k
// X[src(r)][k] * W_e[n][k] in fp32 with vector FMAs.  A wave takes two rows of W at a time, its lanes split K in 16-byte
// pieces, the expert's rows of X wait in LDS (2048 columns at a time), and the lanes' partial dot products meet in a
// butterfly.  For the STORE and SWIGLU epilogues the wave finishes the job itself: no workspace, no second kernel;
// SWIGLU_BWD writes its sums to the workspace part[1][M][N] for fr_epilogue_kernel.  (W[e] as (K, N) had a vector kernel
// of its own, a thread owning 8 columns and walking the rows k of a K range; the small MFMA tile below beat it at every
// number of rows once its K ranges were few enough, 82 against 90 us for dX1 with one row per expert.)
// ------------------------------------------------------------------------------------------------
constexpr int FR_NT_ROWS = 32;  // rows of W per workgroup (8 per wave, two at a time); 8 when the rows are short
constexpr int FR_NT_VALU_ROWS_PER_EXPERT = 2; // on average; beyond that x @ W^T takes the small MFMA tile,
constexpr int FR_NT_VALU_ROWS = 64;             // and beyond this many rows in all (the vector kernel's work per row)
constexpr int FR_NT_PIECE = 2048; // elements of K whose X values are staged in LDS at a time (4 rows: 16 KB)
constexpr int FR_NT_PAIRS = FR_NT_ROWS / 8; // pairs of rows of W per wave

__device__ __forceinline__ int64_t fr_src_row(const FwdArgs &a, int64_t r) {
    return a.x_grouped ? r : (int64_t)fastdiv((uint32_t)a.idx[r], a.fan_div);
}

template <typename T, int RC, int EPI>
__device__ __forceinline__ void fr_nt_rows(const FwdArgs &a, float *__restrict__ part, uint16_t *s_x, int e, int64_t lo,
                                           int64_t hi, int n_first, int n_count) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int64_t r0 = lo; r0 < hi; r0 += RC) {
        // pair j of this wave = rows wave * 2 + 8 j (+ 1) of the workgroup's block; n_count is even
        float s[FR_NT_PAIRS][RC][2];
#pragma unroll
        for (int j = 0; j < FR_NT_PAIRS; ++j)
#pragma unroll
            for (int u = 0; u < RC; ++u) s[j][u][0] = s[j][u][1] = 0.f;
        for (int kp = 0; kp < a.K; kp += FR_NT_PIECE) { // K in pieces of 2048: RC x 4 KB of X in LDS at a time
            const int pc = ((a.K - kp < FR_NT_PIECE) ? a.K - kp : FR_NT_PIECE) >> 3; // 16-byte pieces of this step, <= 256
            __syncthreads(); // the piece before is no longer read
            for (int i = tid; i < RC * pc; i += FR_THREADS) {
                const int u = i / pc, c = i - u * pc;
                u32x4 v = {0u, 0u, 0u, 0u};
                if (r0 + u < hi) v = *(const u32x4 *)(a.X + fr_src_row(a, r0 + u) * a.ldx + kp + 8 * c);
                *(u32x4 *)(s_x + (u * (FR_NT_PIECE / 8) + c) * 8) = v;
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < FR_NT_PAIRS; ++j) {
                const int p = wave * 2 + 8 * j;
                if (p < n_count) { // wave-uniform
                    const uint16_t *w_a = a.W + (int64_t)e * a.w_es + (int64_t)(n_first + p) * a.ldw + kp;
                    const uint16_t *w_b = w_a + a.ldw;
                    u32x4 wa[4], wb[4]; // this lane's pieces lane, lane + 64, ... of either row, all in flight
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int c = lane + 64 * q;
                        wa[q] = wb[q] = u32x4{0u, 0u, 0u, 0u};
                        if (c < pc) {
                            wa[q] = __builtin_nontemporal_load((const u32x4 *)(w_a + 8 * c));
                            wb[q] = __builtin_nontemporal_load((const u32x4 *)(w_b + 8 * c));
                        }
                    }
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int c = lane + 64 * q;
                        if (c < pc) {
                            float fa[8], fb[8];
                            fr_unpack<T>(wa[q], fa);
                            fr_unpack<T>(wb[q], fb);
#pragma unroll
                            for (int u = 0; u < RC; ++u) {
                                float fx[8];
                                fr_unpack<T>(*(const u32x4 *)(s_x + (u * (FR_NT_PIECE / 8) + c) * 8), fx);
#pragma unroll
                                for (int i = 0; i < 8; ++i) {
                                    s[j][u][0] = __builtin_fmaf(fx[i], fa[i], s[j][u][0]);
                                    s[j][u][1] = __builtin_fmaf(fx[i], fb[i], s[j][u][1]);
                                }
                            }
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < FR_NT_PAIRS; ++j) {
            const int p = wave * 2 + 8 * j;
            if (p >= n_count) break; // wave-uniform
            const int n_a = n_first + p, n_b = n_a + 1;
#pragma unroll
            for (int u = 0; u < RC; ++u)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int d = 32; d > 0; d >>= 1) s[j][u][h] += __shfl_xor(s[j][u][h], d);
            if (lane == 0) {
#pragma unroll
                for (int u = 0; u < RC; ++u) {
                    const int64_t r = r0 + u;
                    if (r >= hi) continue;
                    if constexpr (EPI < 0) { // the sums go to the workspace, the epilogue kernel follows
                        part[r * a.N + n_a] = s[j][u][0];
                        part[r * a.N + n_b] = s[j][u][1];
                    } else { // the only part there is: bias, scale and the epilogue right here (n_a is even)
                        const int64_t s_idx = a.idx ? a.idx[r] : r;
                        const float sc = a.scale ? fr_scalar<T>(a.scale, s_idx) : 1.f;
                        const int64_t dst = a.y_grouped ? r : s_idx;
                        float v0 = s[j][u][0], v1 = s[j][u][1];
                        if (a.bias) v0 += fr_scalar<T>(a.bias, (int64_t)e * a.bias_es + n_a), v1 += fr_scalar<T>(a.bias, (int64_t)e * a.bias_es + n_b);
                        const uint32_t z = Elem<T>::pack(v0 * sc, v1 * sc);
                        if (a.out) *(uint32_t *)(a.out + dst * a.ldo + n_a) = z;
                        if constexpr (EPI == XMA_ROCM_EPI_SWIGLU) {
                            const float g = Elem<T>::lo(z), up = Elem<T>::hi(z);
                            a.aux[dst * a.ldaux + (n_a >> 1)] = (uint16_t)(Elem<T>::pack(up * g * sigmoidf_fast(g), 0.f) & 0xffffu);
                        }
                    }
                }
            }
        }
    }
}

// EPI = XMA_ROCM_EPI_STORE or _SWIGLU: the wave that holds a pair of sums applies bias, scale and epilogue itself (the
// columns of a pair are (gate, up)); EPI = -1: the sums go to the workspace for fr_epilogue_kernel.
template <typename T, int EPI>
__global__ __launch_bounds__(FR_THREADS, 4) void fr_nt_kernel(const FwdArgs a, float *__restrict__ part, int rows_per_wg) {
    __shared__ __attribute__((aligned(16))) uint16_t s_x_nt[4 * FR_NT_PIECE];
    const int e = blockIdx.y;
    const int64_t lo = e ? a.offs[e - 1] : 0, hi = a.offs[e];
    if (lo >= hi) return; // uniform
    const int n_first = blockIdx.x * rows_per_wg;
    const int n_count = (a.N - n_first < rows_per_wg) ? a.N - n_first : rows_per_wg;
    if (hi - lo <= 2)
        fr_nt_rows<T, 2, EPI>(a, part, s_x_nt, e, lo, hi, n_first, n_count);
    else
        fr_nt_rows<T, 4, EPI>(a, part, s_x_nt, e, lo, hi, n_first, n_count);
}

// One workgroup per row and 512 columns: the S parts are added in order, the bias joins, and the epilogue of the MFMA kernels is applied
// with the same arithmetic (tile_epilogue in grouped_gemm.hip): STORE rounds acc * scale; SWIGLU rounds the
// pre-activations and takes the activation from the rounded pair; SWIGLU_BWD turns d h = acc * scale and the stored
// pre-activations into (d gate, d up) and, on request, the scaled activation.
template <typename T, int EPI>
__global__ __launch_bounds__(FR_THREADS) void fr_epilogue_kernel(const FwdArgs a, const float *__restrict__ part, int S) {
    __shared__ int s_e;
    const int64_t r = blockIdx.y;
    if (threadIdx.x == 0) { // the expert of row r: first e with offs[e] > r
        int lo = 0, hi = a.E - 1;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (a.offs[mid] > r) hi = mid; else lo = mid + 1;
        }
        s_e = lo;
    }
    __syncthreads();
    const int e = s_e;
    const int64_t s_idx = a.idx ? a.idx[r] : r;
    const float sc = a.scale ? fr_scalar<T>(a.scale, s_idx) : 1.f;
    const int64_t dst = a.y_grouped ? r : s_idx;
    const uint16_t *bias = a.bias ? a.bias + (int64_t)e * a.bias_es : nullptr;
    const int n = 2 * (blockIdx.x * FR_THREADS + threadIdx.x); // N is even: a thread takes a pair of columns
    if (n < a.N) {
        float v0 = bias ? fr_scalar<T>(bias, n) : 0.f, v1 = bias ? fr_scalar<T>(bias, n + 1) : 0.f;
        const float *p0 = part + r * a.N + n;
        const int64_t step = a.M * a.N;
        for (int s0 = 0; s0 < S; s0 += 8) { // eight parts in flight, added in order
            float2 p[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) p[q] = (s0 + q < S) ? *(const float2 *)(p0 + (s0 + q) * step) : make_float2(0.f, 0.f);
#pragma unroll
            for (int q = 0; q < 8; ++q) v0 += p[q].x, v1 += p[q].y;
        }
        if constexpr (EPI == XMA_ROCM_EPI_SWIGLU_BWD) {
            // columns n, n + 1 of d h belong to the pairs (2n, 2n + 1) and (2n + 2, 2n + 3) of z and dz
            const uint32_t z0 = *(const uint32_t *)(a.aux + r * a.ldaux + 2 * n), z1 = *(const uint32_t *)(a.aux + r * a.ldaux + 2 * n + 2);
            uint32_t o[2];
            float hv[2];
            const uint32_t zz[2] = {z0, z1};
            const float dh[2] = {v0 * sc, v1 * sc};
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const float gg = Elem<T>::lo(zz[q]), uu = Elem<T>::hi(zz[q]);
                const float sg = sigmoidf_fast(gg), silu = gg * sg;
                o[q] = Elem<T>::pack(dh[q] * uu * (sg + silu * (1.f - sg)), dh[q] * silu);
                hv[q] = uu * silu * sc;
            }
            *(u32x2 *)(a.out + r * a.ldo + 2 * n) = u32x2{o[0], o[1]};
            if (a.aux2) *(uint32_t *)(a.aux2 + r * a.ldaux2 + n) = Elem<T>::pack(hv[0], hv[1]);
        } else {
            const uint32_t z = Elem<T>::pack(v0 * sc, v1 * sc);
            if (a.out) *(uint32_t *)(a.out + dst * a.ldo + n) = z;
            if constexpr (EPI == XMA_ROCM_EPI_SWIGLU) {
                const float g = Elem<T>::lo(z), u = Elem<T>::hi(z);
                a.aux[dst * a.ldaux + (n >> 1)] = (uint16_t)(Elem<T>::pack(u * g * sigmoidf_fast(g), 0.f) & 0xffffu);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// 3 to 128 rows per expert: too many for vector FMAs (one pass over the weights per 4 or 8 rows), too few for the
// 256 x 256 tiles (one 32 KB stage of weights in flight per compute unit).  A small MFMA tile instead: 32 (or 128) rows of
// the expert x 128 output columns, operands through registers into 40 (64) KB of LDS, so that four (two) workgroups
// share a compute unit and keep 80 (128) KB of loads in flight.  One v_mfma_f32_32x32x16 block per wave; lane l holds 16 sums of row l % 32 in
// quads of 4 consecutive columns, so bias, row scale and the epilogues are lane-local, with the arithmetic of
// tile_epilogue in grouped_gemm.hip.  An expert's rows are taken 32 or 128 at a time.  Every load instruction of a workgroup
// asks for 256 contiguous bytes per row of memory (128-byte pieces of 128 rows of W measured 4.4 TB/s, 256-byte pieces
// the 5.6 TB/s of a copy):
//   WT = 0, W[e] as (N, K): K in steps of 128; the W tile is [128 n][128 k] in one LDS stage, read back with ds_read_b128
//       like the X tile; the next step waits in registers while this one is multiplied.
//   WT = 1, W[e] as (K, N): K in steps of 64, two LDS stages of 20 KB; the W tile is [64 k][128 n] as it lies in memory;
//       ds_read_b64_tr_b16 hands a lane 4 consecutive k of one column (groups of 16 lanes: lane p addresses 4 columns of
//       k-row p / 4 and receives column p).
// ------------------------------------------------------------------------------------------------
constexpr int ST_M = 32, ST_N = 128, ST_K = 64, ST_K_NT = 128;
constexpr int ST_W_BYTES = ST_N * ST_K * 2, ST_X_BYTES = ST_M * ST_K * 2, ST_STAGE = ST_W_BYTES + ST_X_BYTES;
constexpr int ST_W_BYTES_NT = ST_N * ST_K_NT * 2;
__host__ __device__ constexpr int st_k(int wt) { return wt ? ST_K : ST_K_NT; } // K of a step

// 16-byte slot of (row, chunk) in a tile of 128-byte rows: chunk ^ (row & 7) keeps 8 consecutive rows off each other's banks
__device__ __forceinline__ int st_slot(int row, int chunk) { return row * 128 + ((chunk ^ (row & 7)) << 4); }
// (the [64 k][128 n] tile of 256-byte rows uses st_slot_kn above)
// and for tiles of 256-byte rows read along the row (WT = 0): chunk 0..15, the same rotation inside each half
__device__ __forceinline__ int st_slot_nt(int row, int chunk) { return row * 256 + ((chunk ^ (row & 7)) << 4); }

// EPI = -1: the launch is cut along K (blockIdx.z takes `steps_per` steps) because N alone gives too few workgroups; the
// fp32 sums go to part[blockIdx.z][M][N] and fr_epilogue_kernel finishes.
// MB = 32-row blocks of the expert per pass (1 or 4): the weights are streamed once per pass.
template <typename T, int WT, int EPI, int MB>
__global__ __launch_bounds__(FR_THREADS, MB == 1 ? 4 : 2) void fr_tile_kernel(const FwdArgs a, float *__restrict__ part, int steps_per) {
    constexpr int X_BYTES = MB * ST_X_BYTES, STAGE = ST_W_BYTES + X_BYTES; // WT = 1, per stage
    __shared__ __attribute__((aligned(16))) unsigned char s_t[WT == 0 ? ST_W_BYTES_NT + 2 * X_BYTES : 2 * STAGE];
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4s *lds_v4s;
    const int e = blockIdx.y;
    const int64_t lo = e ? a.offs[e - 1] : 0, hi = a.offs[e];
    if (lo >= hi) return; // uniform
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int n0 = blockIdx.x * ST_N;
    const int steps_all = (a.K + st_k(WT) - 1) / st_k(WT);
    const int s_begin = (EPI < 0) ? blockIdx.z * steps_per : 0;
    const int s_end = (EPI < 0 && s_begin + steps_per < steps_all) ? s_begin + steps_per : steps_all;
    if (s_begin >= s_end) return; // uniform; the host launches no empty range
    // loaders.  WT = 0: thread = (row tid / 16 + 16 i, 16-byte chunk tid % 16 of the step's 128 k) for both tiles, rows of W
    // past N clamped (computed, never stored).  WT = 1: W thread = (k-row tid / 16 + 16 i, 16-byte chunk tid % 16 of the 128
    // columns), X thread = (row tid / 8, chunk tid % 8 of the step's 64 k)
    const int ld_row = tid >> 3, ld_chunk = tid & 7;
    const int kn_row = tid >> 4, kn_chunk = tid & 15;
    const bool kn_ok = n0 + 8 * kn_chunk < a.N; // N % 8 == 0: a chunk is inside or outside
    // WT = 0 addresses its 8 rows as a uniform base + 32-bit byte offsets (the host checks that N * ldw * 2 fits)
    const unsigned char *w_base = (const unsigned char *)(a.W + (int64_t)e * a.w_es);
    uint32_t w_off[8];
    const uint16_t *w_src[4];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int n = n0 + kn_row + 16 * i;
        if (n >= a.N) n = a.N - 1;
        w_off[i] = ((uint32_t)n * (uint32_t)a.ldw + 8u * kn_chunk) * 2u;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) w_src[i] = a.W + (int64_t)e * a.w_es + (int64_t)(kn_row + 16 * i) * a.ldw + n0 + 8 * kn_chunk;
    // this lane's fragment of the W tile (byte offset inside a stage, k slice 0)
    int w_frag = 0;
    if constexpr (WT == 1) {
        const int p = lane & 15, G = lane >> 4;
        const int m = wave * 32 + ((G & 1) << 4) + ((p & 3) << 2), kr = ((G >> 1) << 3) + (p >> 2);
        w_frag = kr * 256 + ((((m >> 3) ^ ((kr & 3) << 2))) << 4) + ((m & 7) << 1);
    }
    for (int64_t r0 = lo; r0 < hi; r0 += MB * ST_M) {
        f32x16 acc[MB];
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[b][i] = 0.f;
        const u32x4 zero = {0u, 0u, 0u, 0u};
        if constexpr (WT == 0) {
            const uint16_t *x_src[2 * MB];
#pragma unroll
            for (int i = 0; i < 2 * MB; ++i) {
                int64_t xr = r0 + kn_row + 16 * i;
                if (xr >= hi) xr = hi - 1;
                x_src[i] = a.X + fr_src_row(a, xr) * a.ldx + 8 * kn_chunk;
            }
            u32x4 wv[8], xv[2 * MB];
            auto fetch = [&](int s) {
                const bool ok = s * ST_K_NT + 8 * kn_chunk < a.K; // chunks past K are zeros
#pragma unroll
                for (int i = 0; i < 2 * MB; ++i) xv[i] = ok ? *(const u32x4 *)(x_src[i] + s * ST_K_NT) : zero;
#pragma unroll
                for (int i = 0; i < 8; ++i) wv[i] = ok ? __builtin_nontemporal_load((const u32x4 *)(w_base + (size_t)s * (ST_K_NT * 2) + w_off[i])) : zero;
            };
            // Workgroups that run at the same time are at about the same step, and with every one walking K from the front
            // all their requests of a moment would fall on the same 256 bytes of every 4 KB of a row, a fraction of the
            // memory channels: each workgroup starts at a step of its own and wraps around (the fp32 sums of different
            // column blocks are added in different orders).
            const int n_steps = s_end - s_begin;
            int s_at = s_begin + (int)((blockIdx.x + 3u * blockIdx.y) % (unsigned)n_steps);
            auto next_step = [&](int s) { return s + 1 < s_end ? s + 1 : s_begin; };
            fetch(s_at);
            // the 26 LDS addresses of a step are recomputed in every step from two values the compiler cannot see through
            // (the vector ALU is idle here, and kept in registers they would cost the fourth workgroup per compute unit)
            int slot_st = st_slot_nt(kn_row, kn_chunk), row_rd = l32;
            for (int done = 0; done < n_steps; ++done) {
                asm volatile("" : "+v"(slot_st), "+v"(row_rd));
                __syncthreads(); // the step (or the pass) before no longer reads the stage
#pragma unroll
                for (int i = 0; i < 8; ++i) *(u32x4 *)(s_t + slot_st + 16 * 256 * i) = wv[i]; // rows + 16 i: the same rotation
#pragma unroll
                for (int i = 0; i < 2 * MB; ++i) *(u32x4 *)(s_t + ST_W_BYTES_NT + slot_st + 16 * 256 * i) = xv[i];
                __syncthreads();
                s_at = next_step(s_at);
                if (done + 1 < n_steps) fetch(s_at); // in flight while this step is multiplied
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) {
                    const int slot = st_slot_nt(row_rd, 2 * kk + half);
                    const u32x4 wa = *(const u32x4 *)(s_t + wave * (32 * 256) + slot);
#pragma unroll
                    for (int b = 0; b < MB; ++b) acc[b] = Elem<T>::mfma(wa, *(const u32x4 *)(s_t + ST_W_BYTES_NT + b * (32 * 256) + slot), acc[b]);
                }
            }
        } else {
            const uint16_t *x_src[MB];
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                int64_t xr = r0 + ld_row + 32 * b;
                if (xr >= hi) xr = hi - 1;
                x_src[b] = a.X + fr_src_row(a, xr) * a.ldx + 8 * ld_chunk;
            }
            u32x4 wv[4], xv[MB];
            auto fetch = [&](int s) {
#pragma unroll
                for (int b = 0; b < MB; ++b) xv[b] = (s * ST_K + 8 * ld_chunk < a.K) ? *(const u32x4 *)(x_src[b] + s * ST_K) : zero; // chunks past K are zeros
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool ok = kn_ok && s * ST_K + kn_row + 16 * i < a.K;
                    wv[i] = ok ? __builtin_nontemporal_load((const u32x4 *)(w_src[i] + (int64_t)s * ST_K * a.ldw)) : zero;
                }
            };
            auto stash = [&](int stage) {
                unsigned char *base = s_t + stage * STAGE;
#pragma unroll
                for (int i = 0; i < 4; ++i) *(u32x4 *)(base + st_slot_kn(kn_row + 16 * i, kn_chunk)) = wv[i];
#pragma unroll
                for (int b = 0; b < MB; ++b) *(u32x4 *)(base + ST_W_BYTES + st_slot(ld_row + 32 * b, ld_chunk)) = xv[b];
            };
            __syncthreads(); // the pass before no longer reads the stages
            fetch(s_begin);
            stash(s_begin & 1);
            __syncthreads();
            for (int s = s_begin; s < s_end; ++s) {
                if (s + 1 < s_end) fetch(s + 1); // in flight while this step computes
                unsigned char *base = s_t + (s & 1) * STAGE;
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) { // k-rows 16 kk + ..: the swizzle depends on kr & 3 only, so kk adds 16 rows = 4096 bytes
                    const v4s k03 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(base + w_frag + kk * 4096));
                    const v4s k47 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(base + w_frag + kk * 4096 + 1024));
                    const u32x2 a01 = __builtin_bit_cast(u32x2, k03), a23 = __builtin_bit_cast(u32x2, k47);
                    const u32x4 wa = u32x4{a01[0], a01[1], a23[0], a23[1]};
#pragma unroll
                    for (int b = 0; b < MB; ++b)
                        acc[b] = Elem<T>::mfma(wa, *(const u32x4 *)(base + ST_W_BYTES + st_slot(l32 + 32 * b, 2 * kk + half)), acc[b]);
                }
                if (s + 1 < s_end) stash((s + 1) & 1); // that stage was last read in step s - 1, behind a barrier
                __syncthreads();
            }
        }
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const int64_t r = r0 + 32 * b + l32;
            if (r >= hi) continue;
            if constexpr (EPI < 0) {
                float *mine = part + ((int64_t)blockIdx.z * a.M + r) * a.N;
    #pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = n0 + wave * 32 + 8 * g + 4 * half;
                    if (n < a.N) *(float4 *)(mine + n) = make_float4(acc[b][4 * g], acc[b][4 * g + 1], acc[b][4 * g + 2], acc[b][4 * g + 3]);
                }
                continue;
            }
            const int64_t s_idx = a.idx ? a.idx[r] : r;
            const float sc = a.scale ? fr_scalar<T>(a.scale, s_idx) : 1.f;
            const int64_t dst = a.y_grouped ? r : s_idx;
    #pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wave * 32 + 8 * g + 4 * half; // acc[b][4 g + q] is column n + q of row r
                if (n >= a.N) continue;
                if constexpr (EPI == XMA_ROCM_EPI_SWIGLU_BWD) {
                    // d h of 4 columns -> (d gate, d up) of their 4 pairs; rows are grouped on both sides
                    const u32x4 z = *(const u32x4 *)(a.aux + r * a.ldaux + 2 * n);
                    u32x4 o;
                    float hv[4];
    #pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float dh = acc[b][4 * g + q] * sc;
                        const float gg = Elem<T>::lo(z[q]), uu = Elem<T>::hi(z[q]);
                        const float sg = sigmoidf_fast(gg), silu = gg * sg;
                        o[q] = Elem<T>::pack(dh * uu * (sg + silu * (1.f - sg)), dh * silu);
                        hv[q] = uu * silu * sc;
                    }
                    *(u32x4 *)(a.out + r * a.ldo + 2 * n) = o;
                    if (a.aux2) *(u32x2 *)(a.aux2 + r * a.ldaux2 + n) = u32x2{Elem<T>::pack(hv[0], hv[1]), Elem<T>::pack(hv[2], hv[3])};
                } else {
                    float v[4];
    #pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        v[q] = acc[b][4 * g + q];
                        if (a.bias) v[q] += fr_scalar<T>(a.bias, (int64_t)e * a.bias_es + n + q);
                        v[q] *= sc;
                    }
                    const uint32_t z0 = Elem<T>::pack(v[0], v[1]), z1 = Elem<T>::pack(v[2], v[3]);
                    if (a.out) *(u32x2 *)(a.out + dst * a.ldo + n) = u32x2{z0, z1};
                    if constexpr (EPI == XMA_ROCM_EPI_SWIGLU) {
                        const float g0 = Elem<T>::lo(z0), u0 = Elem<T>::hi(z0), g1 = Elem<T>::lo(z1), u1 = Elem<T>::hi(z1);
                        *(uint32_t *)(a.aux + dst * a.ldaux + (n >> 1)) = Elem<T>::pack(u0 * g0 * sigmoidf_fast(g0), u1 * g1 * sigmoidf_fast(g1));
                    }
                }
            }
        }
    }
}

// W[e] as (K, N), more than a pass or two of the vector kernel per expert, or rows of W shorter than the 4 KB a wave of
// the vector kernel takes at a time -> the small MFMA tile (128 experts of H = 576, I = 256, 7 tokens: forward 0.036
// instead of 0.045 ms with it; 8 experts of H = 2048, I = 8192: 0.161 instead of 0.155)
inline bool fr_takes_tile(int64_t M, int K, int E, int w_is_kn) {
    return w_is_kn || M > (int64_t)FR_NT_VALU_ROWS_PER_EXPERT * E || M > FR_NT_VALU_ROWS || K < FR_NT_PIECE;
}

// passes of 128 rows once many experts have more than 32: two workgroups per compute unit instead of four (registers
// and 64 KB of LDS), 3-10 % slower than passes of 32 rows where those suffice; passes of 64 rows and three workgroups were
// no faster than these anywhere
inline int fr_tile_row_blocks(int64_t M, int E) { return M > (int64_t)24 * E ? 4 : 1; }

// K ranges of the small MFMA tile: enough workgroups for two per compute unit of a 256-CU device, ranges of at least 512
// columns of K.  Measured (8 experts, 16 rows each, down-projection / dX1 / dX2): 1024 workgroups 61 / 99 / 57 us, 512
// 52 / 91 / 46, 256 55 / 137 / 46: beyond two per compute unit the partial sums and their kernel cost more than the
// parallelism brings.
inline int fr_tile_splits(int N, int K, int E, int w_is_kn) {
    const int64_t wgs = (int64_t)((N + ST_N - 1) / ST_N) * E;
    const int ks = st_k(w_is_kn), steps = (K + ks - 1) / ks, min_steps = 512 / ks;
    int S = (int)((512 + wgs - 1) / wgs);
    if (S > steps / min_steps) S = steps / min_steps;
    return S < 1 ? 1 : S;
}

template <typename T, int EPI> int fr_launch_epilogue(const FwdArgs &a, const float *part, int S, hipStream_t st) {
    const dim3 egrid((a.N / 2 + FR_THREADS - 1) / FR_THREADS, (unsigned)a.M);
    fr_epilogue_kernel<T, EPI><<<egrid, FR_THREADS, 0, st>>>(a, part, S);
    return xma_check_launch("fr_epilogue_kernel");
}

template <typename T, int WT, int EPI, int MB> int fr_launch_tile_mb(const FwdArgs &a, float *part, hipStream_t st) {
    const int S_max = fr_tile_splits(a.N, a.K, a.E, WT);
    const int steps_all = (a.K + st_k(WT) - 1) / st_k(WT), steps_per = (steps_all + S_max - 1) / S_max;
    const int S = (steps_all + steps_per - 1) / steps_per; // ranges that hold a step (25 steps in 6 ranges of 5: only 5 do)
    const dim3 grid((a.N + ST_N - 1) / ST_N, a.E, S);
    if (S == 1) {
        fr_tile_kernel<T, WT, EPI, MB><<<grid, FR_THREADS, 0, st>>>(a, nullptr, steps_all);
        return xma_check_launch("fr_tile_kernel");
    }
    fr_tile_kernel<T, WT, -1, MB><<<grid, FR_THREADS, 0, st>>>(a, part, steps_per);
    int rc = xma_check_launch("fr_tile_kernel");
    if (rc) return rc;
    return fr_launch_epilogue<T, EPI>(a, part, S, st);
}

template <typename T, int WT, int EPI> int fr_launch_tile(const FwdArgs &a, float *part, hipStream_t st) {
    return fr_tile_row_blocks(a.M, a.E) == 4 ? fr_launch_tile_mb<T, WT, EPI, 4>(a, part, st) : fr_launch_tile_mb<T, WT, EPI, 1>(a, part, st);
}

template <typename T, int EPI> int fr_launch_epi(const FwdArgs &a, int w_is_kn, float *part, hipStream_t st) {
    int rc;
    if (fr_takes_tile(a.M, a.K, a.E, w_is_kn)) return w_is_kn ? fr_launch_tile<T, 1, EPI>(a, part, st) : fr_launch_tile<T, 0, EPI>(a, part, st);
    // one pair of rows per wave instead of four where the rows are short or the launch would have few workgroups
    const int rows_per_wg = (a.K >= 2048 && (int64_t)(a.N / FR_NT_ROWS) * a.E >= 2048) ? FR_NT_ROWS : 8;
    const dim3 grid((a.N + rows_per_wg - 1) / rows_per_wg, a.E);
    if constexpr (EPI == XMA_ROCM_EPI_SWIGLU_BWD) {
        fr_nt_kernel<T, -1><<<grid, FR_THREADS, 0, st>>>(a, part, rows_per_wg);
        if ((rc = xma_check_launch("fr_nt_kernel"))) return rc;
        return fr_launch_epilogue<T, EPI>(a, part, 1, st);
    } else {
        fr_nt_kernel<T, EPI><<<grid, FR_THREADS, 0, st>>>(a, part, rows_per_wg);
        return xma_check_launch("fr_nt_kernel");
    }
}

template <typename T> int fr_launch(const FwdArgs &a, int w_is_kn, int epilogue, float *part, hipStream_t st) {
    if (epilogue == XMA_ROCM_EPI_STORE) return fr_launch_epi<T, XMA_ROCM_EPI_STORE>(a, w_is_kn, part, st);
    if (epilogue == XMA_ROCM_EPI_SWIGLU) return fr_launch_epi<T, XMA_ROCM_EPI_SWIGLU>(a, w_is_kn, part, st);
    return fr_launch_epi<T, XMA_ROCM_EPI_SWIGLU_BWD>(a, w_is_kn, part, st);
}

} // namespace

extern "C" size_t xma_rocm_scatter2scatter_few_rows_workspace_bytes(int64_t M, int32_t N, int32_t K, int32_t E, int w_is_kn,
                                                                    int epilogue) {
    if (M <= 0 || N <= 0 || K <= 0 || E <= 0) return 0;
    int S;
    if (fr_takes_tile(M, K, E, w_is_kn)) { // the small MFMA tile, cut along K or not
        S = fr_tile_splits(N, K, E, w_is_kn);
        if (S == 1) return 0;
    } else if (epilogue == XMA_ROCM_EPI_SWIGLU_BWD) {
        S = 1; // the vector kernel's sums go to the epilogue kernel
    } else {
        return 0; // the vector kernel finishes the job itself
    }
    return (size_t)S * (size_t)M * (size_t)N * sizeof(float);
}

extern "C" int xma_rocm_scatter2scatter_few_rows(const void *X, int64_t ldx, const void *W, int64_t w_expert_stride,
                                                 int64_t ldw, int w_is_kn, const int64_t *sorted_scattered_idxs,
                                                 const int64_t *expert_offsets, void *out, int64_t ldo, void *aux,
                                                 int64_t ldaux, void *aux2, int64_t ldaux2, const void *row_scale,
                                                 const void *bias, int64_t bias_expert_stride, int64_t M, int32_t N,
                                                 int32_t K, int32_t E, int32_t fan_out, int x_grouped, int y_grouped,
                                                 int epilogue, int dtype, void *workspace, size_t workspace_bytes,
                                                 void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16, XMA_ROCM_EUNSUPPORTED, "scatter2scatter_few_rows: dtype %d", dtype);
    XMA_REQUIRE(epilogue >= XMA_ROCM_EPI_STORE && epilogue <= XMA_ROCM_EPI_SWIGLU_BWD, XMA_ROCM_EINVAL,
                "scatter2scatter_few_rows: epilogue %d", epilogue);
    XMA_REQUIRE(M >= 0 && M <= 65535 && N >= 8 && K >= 8 && E >= 1 && E <= 65535 && fan_out >= 1, XMA_ROCM_EINVAL,
                "scatter2scatter_few_rows: M=%lld N=%d K=%d E=%d fan_out=%d (M and E at most 65535)", (long long)M, N, K, E, fan_out);
    XMA_REQUIRE(N % 8 == 0 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldo % 8 == 0 && w_expert_stride % 8 == 0,
                XMA_ROCM_EUNSUPPORTED, "scatter2scatter_few_rows: N=%d K=%d and the leading dimensions must be multiples of 8", N, K);
    XMA_REQUIRE(w_is_kn || (int64_t)N * ldw < ((int64_t)1 << 31) - 128, XMA_ROCM_EUNSUPPORTED,
                "scatter2scatter_few_rows: N * ldw = %lld exceeds 2^31 - 128 elements for W as (N, K)", (long long)N * (long long)ldw);
    if (M == 0) return XMA_ROCM_OK;
    auto al16 = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
    XMA_REQUIRE(X && W && expert_offsets && al16(X) && al16(W), XMA_ROCM_EINVAL, "scatter2scatter_few_rows: null or misaligned operand");
    XMA_REQUIRE(sorted_scattered_idxs || (x_grouped && y_grouped && !row_scale), XMA_ROCM_EINVAL,
                "scatter2scatter_few_rows: sorted_scattered_idxs is required unless everything is grouped");
    if (epilogue == XMA_ROCM_EPI_STORE) {
        XMA_REQUIRE(out && al16(out), XMA_ROCM_EINVAL, "scatter2scatter_few_rows: out is null or misaligned");
    } else if (epilogue == XMA_ROCM_EPI_SWIGLU) {
        XMA_REQUIRE(aux && al16(aux) && ldaux % 8 == 0 && N % 16 == 0 && (!out || al16(out)), XMA_ROCM_EINVAL,
                    "scatter2scatter_few_rows: SWIGLU needs aux (M, N/2), ldaux %% 8 == 0, N %% 16 == 0");
    } else {
        XMA_REQUIRE(out && aux && al16(out) && al16(aux) && ldaux % 8 == 0 && y_grouped && !bias, XMA_ROCM_EINVAL,
                    "scatter2scatter_few_rows: SWIGLU_BWD needs out, aux (z), y_grouped and no bias");
    }
    XMA_REQUIRE(!aux2 || (epilogue == XMA_ROCM_EPI_SWIGLU_BWD && al16(aux2) && ldaux2 % 8 == 0 && ldaux2 >= N), XMA_ROCM_EINVAL,
                "scatter2scatter_few_rows: scaled activations go with SWIGLU_BWD, 16-byte aligned rows");
    XMA_REQUIRE(!bias || (al16(bias) && bias_expert_stride % 8 == 0 && bias_expert_stride >= 0), XMA_ROCM_EINVAL,
                "scatter2scatter_few_rows: bias (E, N) must be 16-byte aligned with an expert stride that is a multiple of 8");
    const size_t need = xma_rocm_scatter2scatter_few_rows_workspace_bytes(M, N, K, E, w_is_kn, epilogue);
    XMA_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && al16(workspace)), XMA_ROCM_EWORKSPACE,
                "scatter2scatter_few_rows: workspace of %zu bytes, %zu needed (16-byte aligned)", workspace ? workspace_bytes : (size_t)0, need);
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
    a.aux2 = (uint16_t *)aux2;
    a.ldaux2 = ldaux2;
    a.scale = (const uint16_t *)row_scale;
    a.bias = (const uint16_t *)bias;
    a.bias_es = bias_expert_stride;
    a.M = M;
    a.N = N;
    a.K = K;
    a.E = E;
    a.fan_out = fan_out;
    a.fan_div = make_fastdiv((uint32_t)fan_out);
    a.x_grouped = x_grouped;
    a.y_grouped = y_grouped;
    a.partial = nullptr;
    a.split_cus = 0;
    a.grid_main = 0;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == XMA_ROCM_BF16) return fr_launch<__bf16>(a, w_is_kn ? 1 : 0, epilogue, (float *)workspace, st);
    return fr_launch<_Float16>(a, w_is_kn ? 1 : 0, epilogue, (float *)workspace, st);
}
