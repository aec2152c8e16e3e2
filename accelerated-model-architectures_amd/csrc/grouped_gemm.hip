// Grouped (per-expert, ragged) GEMMs of the MoE layer on CDNA4 MFMA.
//
// One workgroup = 256 threads = 4 wave64 (2 x 2), output tile 256 x 256, K step 64.  Each wave owns 128 x 128 =
// 4 x 4 v_mfma_f32_32x32x16 tiles (256 fp32 accumulators per lane, one wave per SIMD).
//
// Operand tiles go from HBM straight into LDS with global_load_lds_dwordx4 (no VGPR staging, no ds_write): a wave
// instruction moves 64 x 16 bytes to 1 KB of consecutive LDS, and the swizzle is applied on the GLOBAL side (which
// lane fetches which 16-byte chunk).  Every such instruction covers whole 128-byte lines (8 per instruction): the
// texture addresser works line by line, and half-line requests (a 32-wide K step) were measured at a third of the
// throughput.  Two LDS layouts, both 32 KB per 256 x 64 operand tile:
//   row-major source (K contiguous in memory):  LDS [256 rows][8 chunks], chunk c of row r at slot c ^ swz(r);
//       MFMA fragments are one ds_read_b128 per lane.
//   transposed source (K is the row index in memory: weights for dX, both operands for dW):
//       LDS [64 k][32 chunks] exactly as in memory, chunk c of k-row kr at slot c ^ ((kr & 3) << 1);
//       MFMA fragments are two ds_read_b64_tr_b16 per lane, which hand each lane 4 consecutive k of one column.
//
// Pipeline: two stages (128 KB of the 160 KB LDS), one barrier per K step.  A K step is four k16 sub-steps of 16 MFMAs;
// the fragments of sub-step kk + 1 are read while sub-step kk multiplies.  The barrier sits between sub-steps 2 and 3:
// by then a wave holds the last fragments of the step in registers, so behind the barrier the other stage (step s + 1,
// waited for with vmcnt(0) just before) is readable and this stage is free.  The loads of step s + 2 are issued one per
// MFMA slot during sub-steps 0 and 1 of step s + 1, which leaves them a step and a half to land.  A wave issues in
// order, so everything that is not an MFMA is pinned between MFMAs (sched_barrier) instead of in front of them.
//
// MFMA operand roles: the "P" tile supplies the rows of the 32x32 result (register dimension: a lane holds 4
// consecutive P indices per accumulator quad) and the "Q" tile supplies its columns (lane % 32).  P is always the
// dimension that is contiguous in the OUTPUT, so a lane stores 8 contiguous bytes per quad and owns one output row:
// gather/scatter indices, row scales and the SwiGLU (gate, up) pairs are all lane-local.
//
//   forward / dX :  Q = activation rows (tokens),     P = weight rows (output features)
//   dW           :  Q = dY columns (out features),    P = X columns (in features), K = tokens
//
// Tiles never straddle experts: the schedule is expert-major, derived on the device from the inclusive expert
// offsets in each workgroup's prologue (no host read of the counts).  With a workspace, the tiles of a last, partial
// round of a launch are computed as K slices by a second launch and summed by grouped_gemm_fixup_kernel.
//
// Epilogues (plain store with optional row scale and scatter, SwiGLU forward, SwiGLU backward) stage every 32-row block
// of a wave's corner in wave-private LDS and write whole rows: in the accumulator layout a store instruction would
// touch 32 rows with 16 bytes each.
#include <atomic>

#include "fp32.hpp"
#include "gemm_common.hpp"

namespace xma_rocm {

constexpr int BK = 64, NSTAGE = 2;
// The 16 LDS-DMA pieces of a K step are issued one per MFMA slot: DMA_N0 in the sub-step right behind the barrier that
// frees their stage, DMA_N1 and DMA_N2 in the two sub-steps after it.
// (8, 8, 0) measured best; (6, 6, 4), (12, 4, 0) the same within noise, all 16 in the first sub-step slower.
constexpr int DMA_N0 = 8, DMA_N1 = 8, DMA_N2 = 0;
static_assert(DMA_N0 + DMA_N1 + DMA_N2 == 16 && DMA_N0 <= 16 && DMA_N1 <= 8 && DMA_N2 <= 8, "piece schedule");
constexpr int OP_CHUNKS = 256 * 8;                          // 16-byte chunks per operand tile (32 KB)
constexpr int STAGE_CHUNKS = 2 * OP_CHUNKS;                 // Q tile then P tile
constexpr int GEMM_SMEM_BYTES = NSTAGE * STAGE_CHUNKS * 16; // 128 KB

// 1 KB of zeros: the source of every chunk that lies beyond the K extent of an operand
__device__ __attribute__((aligned(16))) uint32_t g_zero_page[256];

typedef short s16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void lds_dma16(const uint16_t *src, u32x4 *lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                     (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
}

template <int N> struct IC {
    static constexpr int value = N;
};
// compile-time loop: f(IC<0>{}), ..., f(IC<N-1>{}) - the index is a constant expression inside f (asm immediates)
template <int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(IC<N - 1>{});
    }
}

// ---- LDS layouts (byte offsets inside one 32 KB operand tile)
//
// The LDS serves 16 lanes of a ds_read_b128 (32 lanes of a 64-bit read) at a time from 64 banks of 4 bytes, so the 16-byte
// pieces those lanes ask for must fall on 16 different positions modulo 256 bytes.  Both layouts below are arranged for
// that (measured with the fragment patterns alone, 4 waves per CU: 344 bytes/ns/CU against 281 for swizzles that only
// spread 8 consecutive lanes over 128 bytes).
//
// Row-major tile [256 rows][8 chunks of 16 B]: chunk c of row r sits at slot c ^ ((r >> 1) & 7); rows 2 m and 2 m + 1
// share the permutation and are 128 bytes apart.  An LDS-DMA instruction covers 8 rows (1 KB); wave w loads rows
// 64 w + 8 i + (lane >> 3), i = 0..7, and lane fills slot lane & 7, i.e. it fetches logical chunk
// (lane & 7) ^ (4 (i & 1) + (lane >> 4)): one of two per-lane constants, so a lane's global address of piece i is a fixed
// per-lane pointer plus the K offset of the step.
__device__ __forceinline__ int rowmajor_lane_chunk(int i, int lane) { return (lane & 7) ^ (((i & 1) << 2) + (lane >> 4)); }
// MFMA fragment of rows R0 + 32 i + (lane & 31), k16 sub-step kk: R0 and 32 i are multiples of 16, so the slot is
// ((2 kk + (lane >> 5)) ^ ((lane >> 1) & 7)): one per-lane byte offset per kk, and i is an immediate (4096 i).
__device__ __forceinline__ uint32_t rowmajor_frag_offset(int R0, int kk, int lane) {
    return (uint32_t)((R0 + (lane & 31)) * 128 + (((2 * kk + (lane >> 5)) ^ ((lane >> 1) & 7)) << 4));
}
//
// Transposed tile [64 k-rows][32 chunks of 16 B], exactly as in memory: chunk c of k-row kr sits at slot
// c ^ ((kr & 3) << 2).  An LDS-DMA instruction covers 2 k-rows; wave w loads k-rows 16 w + 2 j + (lane >> 5), j = 0..7,
// and lane fills slot lane & 31, i.e. it fetches logical chunk (lane & 31) ^ (((2 j + (lane >> 5)) & 3) << 2).
__device__ __forceinline__ int transposed_lane_chunk(int j, int lane) {
    return (lane & 31) ^ (((2 * j + (lane >> 5)) & 3) << 2);
}
// MFMA fragment through ds_read_b64_tr_b16, which works on groups of 16 lanes: lane p of a group supplies the
// address of 4 columns at one k-row and receives 4 consecutive k of one column.  With
// p -> (k-row kb + p / 4, columns mb + 4 (p % 4)) lane p ends up with column mb + p, k = kb .. kb + 3; two reads
// (kb and kb + 4) give the 8 k of an MFMA operand.  A pass of 32 lanes (groups 0 and 1: 32 columns at 4 k-rows) reads
// eight 32-byte pieces; the column pair picks bit 1 of the chunk index, the k-row bits 2 and 3, so they are 8
// different positions modulo 256 bytes.  The 32-row block i of the wave's 128 rows adds 4 i to the chunk index, which
// the XOR does not commute with: one per-lane offset per block; kk adds 8192 bytes, the second read 2048.
__device__ __forceinline__ uint32_t transposed_frag_offset(int R0, int blk, int lane) {
    const int p = lane & 15, G = lane >> 4;
    const int m = R0 + blk * 32 + ((G & 1) << 4) + ((p & 3) << 2);
    const int kr = ((G >> 1) << 3) + (p >> 2);
    return (uint32_t)(kr * 512 + ((((m >> 3) ^ ((kr & 3) << 2))) << 4) + ((m & 7) << 1));
}

// per-lane LDS byte addresses of one operand's fragments in the CURRENT stage
template <int TR> struct FragBase {
    uint32_t b[4]; // row-major: one per kk; transposed: one per 32-row block
};

template <int TR> __device__ __forceinline__ void make_frag_base(FragBase<TR> &f, uint32_t tile_lds_addr, int R0, int lane) {
    if constexpr (TR == 0) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) f.b[kk] = tile_lds_addr + rowmajor_frag_offset(R0, kk, lane);
    } else {
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) f.b[blk] = tile_lds_addr + transposed_frag_offset(R0, blk, lane);
    }
}
template <int TR> __device__ __forceinline__ void flip_stage(FragBase<TR> &f) {
#pragma unroll
    for (int q = 0; q < 4; ++q) f.b[q] ^= (uint32_t)(STAGE_CHUNKS * 16);
}

// All fragment reads are inline assembly with an immediate offset: (1) after an LDS-DMA load the compiler guards every
// LDS read it cannot prove disjoint with s_waitcnt vmcnt(0), which would drain the load pipeline at each fragment;
// (2) it keeps address arithmetic out of the MFMA stream.  The compiler therefore does not know these reads are in
// flight: wait_frags() must precede their use.
template <int TR, int I, int KK> __device__ __forceinline__ u32x4 read_frag(const FragBase<TR> &f) {
    if constexpr (TR == 0) {
        u32x4 r;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(f.b[KK]), "n"(I * 4096));
        return r;
    } else {
        u32x2 lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(f.b[I]), "n"(KK * 8192));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(f.b[I]), "n"(KK * 8192 + 2048));
        u32x4 r = {lo[0], lo[1], hi[0], hi[1]};
        return r;
    }
}

struct Frags {
    u32x4 p[4], q[4];
};

// All LDS reads of this wave have returned; the fragments are tied to the statement so that no MFMA using them can be
// moved above it.
__device__ __forceinline__ void wait_frags(Frags &f) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.p[0]), "+v"(f.p[1]), "+v"(f.p[2]), "+v"(f.p[3]), "+v"(f.q[0]), "+v"(f.q[1]), "+v"(f.q[2]),
                   "+v"(f.q[3]));
}

template <int PTR, int QTR, int KK>
__device__ __forceinline__ void load_frags(Frags &f, const FragBase<PTR> &pb, const FragBase<QTR> &qb) {
    static_for<4>([&](auto I) {
        f.p[I.value] = read_frag<PTR, I.value, KK>(pb);
        f.q[I.value] = read_frag<QTR, I.value, KK>(qb);
    });
}

// The 16 MFMAs of one k16 sub-step on `cur` in pinned slots of MMA_GROUP MFMAs, each followed by its share of the other
// instructions: the 8 fragment reads of sub-step KK (of the stage pb/qb point at) into `nxt` during the first half of
// the sub-step, so that the second half covers their latency, and the 8 calls `hook(IC<0..7>)`, which the callers use
// to issue one LDS-DMA or index load each.  A wave issues in order, so anything not placed between MFMAs would leave the
// matrix pipe idle for as long as it takes to issue.  Pairs of MFMAs measured best in the kernels (single MFMAs 2-3 %
// slower, although an isolated instruction-mix benchmark prefers them).  NI < 4: only the first NI of the wave's four
// 32-wide Q blocks hold valid rows; the MFMAs and fragment reads of the others are left out.
constexpr int MMA_GROUP = 2;
// READ_NEXT = 0: no fragment reads (the last sub-step of a tile whose hooks hold compiler-generated code: fragments read
// ahead there would never be used, so the compiler would treat their registers as free while the reads are in flight).
template <typename T, int PTR, int QTR, int KK, int NI = 4, int READ_NEXT = 1, typename Hook>
__device__ __forceinline__ void mma_step(Frags &cur, Frags &nxt, const FragBase<PTR> &pb, const FragBase<QTR> &qb,
                                         f32x16 (&acc)[4][4], Hook hook) {
    wait_frags(cur); // issued at least 8 MFMAs ago
    constexpr int SLOTS = 16 / MMA_GROUP;
    static_for<SLOTS>([&](auto S) {
        constexpr int t = S.value;
        __builtin_amdgcn_sched_barrier(0);
        static_for<MMA_GROUP>([&](auto M) {
            // the 4 x 4 blocks in boustrophedon order: consecutive MFMAs differ in one operand only (measured 0 - 1 % faster
            // than row by row on the six GEMMs of the Mixtral-shaped layer; the sums are the same)
            constexpr int m = t * MMA_GROUP + M.value, j = m >> 2, i = (j & 1) ? 3 - (m & 3) : (m & 3);
            if constexpr (i < NI) acc[j][i] = Elem<T>::mfma(cur.p[j], cur.q[i], acc[j][i]);
        });
        __builtin_amdgcn_sched_barrier(0);
        // fragment reads: 8 (4 P, 4 Q) over the first SLOTS / 2 slots
        constexpr int RPS = 16 / SLOTS; // reads per slot of the first half
        if constexpr (t < SLOTS / 2 && READ_NEXT != 0) {
            static_for<RPS>([&](auto R) {
                constexpr int r = t * RPS + R.value, f = r >> 1;
                if constexpr ((r & 1) == 0) {
                    if constexpr (NI > 0) nxt.p[f] = read_frag<PTR, f, KK>(pb);
                } else {
                    if constexpr (f < NI) nxt.q[f] = read_frag<QTR, f, KK>(qb);
                }
            });
        }
        // hooks: 8 over all slots (two per slot for groups of 4, every other slot for single MFMAs)
        if constexpr (SLOTS == 4) {
            hook(IC<2 * t>{});
            hook(IC<2 * t + 1>{});
        } else if constexpr (SLOTS == 8) {
            hook(S);
        } else if constexpr ((t & 1) == 1) {
            hook(IC<t / 2>{});
        }
    });
    __builtin_amdgcn_sched_barrier(0);
}

struct NoHook {
    template <typename G> __device__ __forceinline__ void operator()(G) const {}
};

__device__ __forceinline__ uint32_t lds_addr_of(const void *p) {
    return (uint32_t)(size_t)((__attribute__((address_space(3))) const char *)p);
}

// Every LDS-DMA load of this wave has landed and its LDS reads have returned; then meet the other waves.  "memory"
// keeps the compiler from moving LDS accesses across it.
#define XMA_WAIT_LOADS_AND_BARRIER() asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory")
#define XMA_WAIT_ALL_LOADS() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")

// Epilogue staging in LDS, private to a wave: one 32-row block of its 128 x 128 corner as 16-bit values (rows padded
// by 16 bytes against bank conflicts), followed by the 32 x 64 block of SwiGLU activations.
constexpr int EPI_Z_STRIDE = 128 * 2 + 16, EPI_H_STRIDE = 64 * 2 + 16;
// Internal epilogue code beside the public XMA_ROCM_EPI_*: SWIGLU_BWD with the second output FwdArgs::aux2.  A variant of
// its own, so that the launches without that output keep their code and register allocation unchanged.
constexpr int EPI_SWIGLU_BWD_SCALED_ACT = 3;
constexpr int EPI_WAVE_BYTES = 32 * EPI_Z_STRIDE + 32 * EPI_H_STRIDE;
// SwiGLU backward stages 32 rows of 256 pre-activation columns per wave
constexpr int EPI_BWD_STRIDE = 256 * 2 + 16, EPI_BWD_WAVE_BYTES = 32 * EPI_BWD_STRIDE;
static_assert(4 * EPI_WAVE_BYTES <= GEMM_SMEM_BYTES && 4 * EPI_BWD_WAVE_BYTES <= GEMM_SMEM_BYTES,
              "epilogue staging must fit into the operand stages");

// LDS written by some lanes of a wave is read by others of the same wave: instructions of one wave reach the LDS in
// order, so only the compiler has to be kept from reordering.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int N> __device__ __forceinline__ void zero_acc(f32x16 (&acc)[N][N]) {
#pragma unroll
    for (int j = 0; j < N; ++j)
#pragma unroll
        for (int i = 0; i < N; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;
}

// The experts' bias enters a tile as a rank-one update of the cleared accumulators, ones (rows) x bias (columns), through
// the matrix pipe: one k16 step whose only non-zero k holds 1 in the Q fragments and the bias of the lane's column in the P
// fragments.  The product 1 x b is exact and it is the first term of the fp32 sum, so the result is rounded once, as a
// linear layer with a bias rounds it, and no epilogue has to know about the bias.  (Writing the bias into the
// accumulators directly, 256 register writes from loaded values, made the register allocation spill around the main loop.)
template <typename T> __device__ __forceinline__ uint32_t one_bits();
template <> __device__ __forceinline__ uint32_t one_bits<__bf16>() { return 0x3f80u; }
template <> __device__ __forceinline__ uint32_t one_bits<_Float16>() { return 0x3c00u; }
template <typename T>
__device__ __forceinline__ void add_bias(const FwdArgs &a, f32x16 (&acc)[4][4], int e, int n0, int wp, int lane) {
    const uint16_t *b = a.bias + (int64_t)e * a.bias_es;
    const bool k0 = lane < 32; // lanes 0..31 hold k = 0..7 of their row, lanes 32..63 k = 8..15
    u32x4 q = {k0 ? one_bits<T>() : 0u, 0u, 0u, 0u};
    u32x4 p[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int col = n0 + wp + 32 * j + (lane & 31);
        if (col >= a.N) col = a.N - 1; // columns past N are computed and never stored
        const uint32_t v = b[col];
        p[j] = u32x4{k0 ? v : 0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[j][i] = Elem<T>::mfma(p[j], q, acc[j][i]);
}

// The accumulators of a tile set to its expert's bias, or to zero without one, by sixteen MFMAs of that rank-one product
// onto a constant zero: the matrix pipe clears the 256 registers in half the cycles that 256 register writes take.
template <typename T>
__device__ __forceinline__ void init_acc(const FwdArgs &a, f32x16 (&acc)[4][4], int e, int n0, int wp, int lane) {
    const bool k0 = lane < 32;
    const u32x4 q = {k0 ? one_bits<T>() : 0u, 0u, 0u, 0u};
    uint32_t v[4] = {0u, 0u, 0u, 0u};
    if (a.bias != nullptr) { // uniform
        const uint16_t *b = a.bias + (int64_t)e * a.bias_es;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int col = n0 + wp + 32 * j + (lane & 31);
            if (col >= a.N) col = a.N - 1;
            v[j] = b[col];
        }
    }
    f32x16 zero;
#pragma unroll
    for (int c = 0; c < 16; ++c) zero[c] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const u32x4 p = {k0 ? v[j] : 0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[j][i] = Elem<T>::mfma(p, q, zero);
    }
}

// Which tile a workgroup works on.
struct TileSched {
    int e, rows_valid, n0; // expert, valid rows of the row tile, first output column
    int64_t row0;          // first grouped row
    int part, parts;       // K slice of a split tile (parts == 1: the whole K range)
    int tail_index;        // index of a split tile among the tiles of the last round
};

// Order of an expert's tiles.  The 32 consecutive tiles that xcd_remap hands to an XCD share operand panels in that XCD's
// L2: r row tiles x c column tiles need r activation panels and c weight panels for r c tiles, and the K loop runs as
// fast as those panels arrive.  Walking all row tiles of a column before the next column suits an expert of up to a
// dozen row tiles (measured best for 9: 9 + 3.6 panels, and the same activation panels in every round of the launch);
// an expert of 48 row tiles would have 32 tiles share one weight panel and fetch 32 activation panels (measured: the
// K loop of an expert of 64 row tiles takes 142 us instead of 100).  So the row tiles of a larger expert are cut into
// bands of equal height, at most FWD_BAND, and the walk goes down a band's column, then along the band, then to the next
// band.  Low bands measured better than square ones (4 x 8 before 6 x 5 before 8 x 4): a weight panel is one
// contiguous block, an activation panel 256 gathered rows.  local: index of the tile among the expert's tiles_m x NT.
constexpr int FWD_SINGLE_BAND_TILES = 12;
#ifdef XMA_PST_TIMING
__device__ int g_pst_band = 6; // A/B switch of the timing build
#define FWD_BAND g_pst_band
#else
constexpr int FWD_BAND = 6;
#endif
__device__ __forceinline__ void tile_of_expert(int local, int tiles_m, int NT, int &m_tile, int &n_tile) {
    if (tiles_m <= FWD_SINGLE_BAND_TILES) {
        m_tile = local % tiles_m, n_tile = local / tiles_m;
        return;
    }
    const int bands = (tiles_m + FWD_BAND - 1) / FWD_BAND;
    const int h = (tiles_m + bands - 1) / bands; // height of every band but the last, which has what is left
    int band = local / (h * NT);
    if (band > bands - 1) band = bands - 1;
    const int in_band = local - band * h * NT;
    const int rows = (band == bands - 1) ? tiles_m - h * (bands - 1) : h;
    m_tile = band * h + in_band % rows;
    n_tile = in_band / rows;
}

constexpr int SPLIT_MIN_STEPS = 8; // a K slice is at least this many K steps

// Expert-major schedule: work[e] = ceil(rows_e / BM) * n_tiles, prefix sum over the experts in LDS, then the tile of
// this workgroup.  With a workspace (a.partial) the tiles of the last, partial round of the launch - total mod
// split_cus of them, the workgroups that would otherwise run while most CUs idle - are cut into `parts` K slices, each
// taken by a workgroup of its own in a second launch of the kernel (ROLE_SLICES, at most split_cus workgroups); a
// third launch (ROLE_FIXUP, workgroup b = split tile b) adds the slices.  ROLE_TILES takes all other tiles.  Returns
// false if the workgroup has nothing to do.
constexpr int ROLE_TILES = 0, ROLE_SLICES = 1, ROLE_FIXUP = 2;
// grouped_gemm_kernel is the fallback of launch_fwd for launches that grouped_gemm_persistent_kernel does not take, and
// the kernel of the K slices.  Its SwiGLU-backward instantiations also walk several tiles per workgroup (one workgroup
// per compute unit), the others run one workgroup per tile.
__host__ __device__ constexpr bool fwd_persistent(int epi, int role) {
    return role == ROLE_TILES && (epi == XMA_ROCM_EPI_SWIGLU_BWD || epi == EPI_SWIGLU_BWD_SCALED_ACT);
}
template <int ROLE>
__device__ __forceinline__ bool locate_tile(const FwdArgs &a, unsigned char *smem, int *s_sched, TileSched &ts,
                                            int b, int tid) {
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int NT = (a.N + BN - 1) / BN;
    int full = 0, rest = 0, parts = 1, part = 0, L = 0;
    // from the number of tiles: which one is this workgroup's (false: none)
    auto pick = [&](int total) -> bool {
        full = total;
        if (a.partial) {
            const int KT = (a.K + BK - 1) / BK;
            full = total / a.split_cus * a.split_cus;
            rest = total - full;
            parts = rest ? a.split_cus / rest : 1;
            if (parts > KT / SPLIT_MIN_STEPS) parts = KT / SPLIT_MIN_STEPS;
            if (parts < 2) parts = 1, full = total, rest = 0;
        }
        if (ROLE == ROLE_FIXUP) {
            if ((b >> 2) >= rest) return false; // four workgroups per split tile
            L = full + (b >> 2);
        } else if (ROLE == ROLE_SLICES) {
            if (rest == 0) return false;
            const int q = xcd_remap(b, a.split_cus); // neighbouring tiles of one slice index meet in one XCD's L2
            part = q / rest;
            if (part >= parts) return false;
            L = full + q % rest;
        } else {
            L = xcd_remap(b, a.grid_main);
            if (L >= full) return false; // beyond the last tile (the grid is an upper bound), or a tile that is split
        }
        return true;
    };
    int e, local;
    int64_t row_lo, row_hi;
    if (a.E <= WAVE) {
        // every wave scans the experts in registers: lane = expert; no LDS, no barrier, one load per lane
        const int64_t hi = a.offs[lane < a.E ? lane : a.E - 1];
        int64_t lo = __shfl_up(hi, 1);
        if (lane == 0) lo = 0;
        const int v = (int)((hi - lo + BM - 1) / BM) * NT; // 0 for the lanes past E
        int s = v;
#pragma unroll
        for (int d = 1; d < WAVE; d <<= 1) {
            const int t = __shfl_up(s, d);
            if (lane >= d) s += t;
        }
        if (!pick(__builtin_amdgcn_readlane(s, WAVE - 1))) return false;
        const uint64_t hit = __ballot(s - v <= L && L < s); // exactly one lane
        e = __builtin_ctzll(hit);
        local = L - __builtin_amdgcn_readlane(s - v, e);
        row_lo = ((int64_t)__builtin_amdgcn_readlane((int)(lo >> 32), e) << 32) |
                 (uint32_t)__builtin_amdgcn_readlane((int)lo, e);
        row_hi = ((int64_t)__builtin_amdgcn_readlane((int)(hi >> 32), e) << 32) |
                 (uint32_t)__builtin_amdgcn_readlane((int)hi, e);
    } else {
        int *s_pre = (int *)smem; // [E + 1], dead before the first tile load
        if (wave == 0) {
            int carry = 0;
            for (int b = 0; b < a.E; b += WAVE) {
                const int x = b + lane;
                int v = 0;
                if (x < a.E) {
                    const int64_t cnt = a.offs[x] - (x ? a.offs[x - 1] : 0);
                    v = (int)((cnt + BM - 1) / BM) * NT;
                }
                int s = v;
#pragma unroll
                for (int d = 1; d < WAVE; d <<= 1) {
                    const int t = __shfl_up(s, d);
                    if (lane >= d) s += t;
                }
                if (x < a.E) s_pre[x] = carry + s - v;
                carry += __shfl(s, WAVE - 1);
            }
            if (lane == 0) s_pre[a.E] = carry;
        }
        __syncthreads();
        if (!pick(__builtin_amdgcn_readfirstlane(s_pre[a.E]))) return false;
        for (int x = tid; x < a.E; x += GEMM_THREADS)
            if (s_pre[x] <= L && L < s_pre[x + 1]) {
                s_sched[0] = x;
                s_sched[1] = L - s_pre[x];
            }
        __syncthreads();
        e = __builtin_amdgcn_readfirstlane(s_sched[0]);
        local = __builtin_amdgcn_readfirstlane(s_sched[1]);
        row_lo = e ? a.offs[e - 1] : 0;
        row_hi = a.offs[e];
        __syncthreads(); // s_pre is dead from here on
    }
    const int tiles_m = (int)((row_hi - row_lo + BM - 1) / BM);
    int m_tile, n_tile;
    tile_of_expert(local, tiles_m, NT, m_tile, n_tile);
    ts.e = e;
    ts.row0 = row_lo + (int64_t)m_tile * BM;
    ts.rows_valid = (int)((row_hi - ts.row0 < BM) ? row_hi - ts.row0 : BM);
    ts.n0 = n_tile * BN;
    ts.part = part;
    ts.parts = (L >= full) ? parts : 1;
    ts.tail_index = L - full;
    return true;
}

// Scattered index and row scale of a lane's row in each of the four 32-row blocks of its wave (row wq + 32 i + lane % 32
// of the tile, clamped to the last valid row), when the caller has fetched them ahead of the epilogue.
struct EpiRows {
    int idx[4];
    float sc[4];
};

// ---- epilogue of one 256 x 256 tile; smem: staging area that no wave reads operand tiles from any more
template <typename T, int EPI>
__device__ __forceinline__ void tile_epilogue(const FwdArgs &a, f32x16 (&acc)[4][4], unsigned char *smem, int64_t row0,
                                              int rows_valid, int n0, int tid, int only_i = -1,
                                              const EpiRows *pre = nullptr) {
    // only_i >= 0: just the 32-row block only_i of every wave (the fix-up kernel spreads a tile over four workgroups)
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wq = (wave & 1) * 128, wp = (wave >> 1) * 128; // wave's 128 x 128 corner inside the tile
    // lane owns row (lane & 31) of each 32-row block; quad g of tile (j, i) holds
    //      columns n0 + wp + 32 j + 8 g + 4 (lane >> 5) + {0..3}
    const int lrow = lane & 31, lhalf = lane >> 5;
    if constexpr (EPI != XMA_ROCM_EPI_SWIGLU_BWD && EPI != EPI_SWIGLU_BWD_SCALED_ACT) {
        // A store instruction of the accumulator layout would touch 32 rows with 16 bytes each.  Instead every
        // 32-row block goes through a wave-private LDS area and leaves as whole rows: 16 lanes x 16 bytes per row of
        // 128 columns (8 lanes per row of the 64 activation columns), i.e. full 128-byte lines.
        unsigned char *stage = smem + wave * EPI_WAVE_BYTES;
        unsigned char *z_w = stage + lrow * EPI_Z_STRIDE + lhalf * 8;
        unsigned char *h_w = stage + 32 * EPI_Z_STRIDE + lrow * EPI_H_STRIDE + lhalf * 4;
        const unsigned char *z_r = stage + (lane >> 4) * EPI_Z_STRIDE + (lane & 15) * 16;
        const unsigned char *h_r = stage + 32 * EPI_Z_STRIDE + (lane >> 3) * EPI_H_STRIDE + (lane & 7) * 16;
        const int cz = n0 + wp + (lane & 15) * 8;        // this lane's 8 output columns on the way out
        const int ch = ((n0 + wp) >> 1) + (lane & 7) * 8; // and its 8 activation columns
        const bool write_z = (EPI == XMA_ROCM_EPI_STORE) || a.out != nullptr;
        // destination row and scale of this lane's row in each of the four blocks, fetched before the first store:
        // loads and stores retire in order, so a load between the blocks would wait for the stores before it
        int dst_i[4];
        float sc_i[4];
        const bool need_idx = !a.y_grouped || a.scale != nullptr;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int r = wq + i * 32 + lrow;
            if (r >= rows_valid) r = rows_valid - 1; // duplicates are computed and never stored
            const int64_t n = row0 + r;
            dst_i[i] = need_idx ? (pre ? pre->idx[i] : (int)a.idx[n]) : (int)n;
        }
        if (a.scale && pre) {
#pragma unroll
            for (int i = 0; i < 4; ++i) sc_i[i] = pre->sc[i];
        } else if (a.scale) {
            uint16_t raw[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) raw[i] = a.scale[dst_i[i]];
#pragma unroll
            for (int i = 0; i < 4; ++i) sc_i[i] = Elem<T>::lo((uint32_t)raw[i]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) sc_i[i] = 1.f;
        }
        if (a.y_grouped) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int r = wq + i * 32 + lrow;
                if (r >= rows_valid) r = rows_valid - 1;
                dst_i[i] = (int)(row0 + r);
            }
        }
        // two copies of the loop: without a row scale the 256 multiplications by one are left out
        auto blocks = [&](auto SCALED) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (wq + i * 32 >= rows_valid) break; // wave-uniform
            if (only_i >= 0 && i != only_i) continue;
            const int dst = dst_i[i];
            const float sc = sc_i[i];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float v0 = acc[j][i][4 * g], v1 = acc[j][i][4 * g + 1];
                    float v2 = acc[j][i][4 * g + 2], v3 = acc[j][i][4 * g + 3];
                    if constexpr (SCALED.value) v0 *= sc, v1 *= sc, v2 *= sc, v3 *= sc;
                    const uint32_t z0 = Elem<T>::pack(v0, v1), z1 = Elem<T>::pack(v2, v3);
                    u32x2 o = {z0, z1};
                    *(u32x2 *)(z_w + (j * 32 + g * 8) * 2) = o;
                    if constexpr (EPI == XMA_ROCM_EPI_SWIGLU) {
                        // columns are (gate, up, gate, up); the activation is taken from the rounded
                        // pre-activations, exactly what a separate pass over the stored z would see
                        const float g0 = Elem<T>::lo(z0), u0 = Elem<T>::hi(z0);
                        const float g1 = Elem<T>::lo(z1), u1 = Elem<T>::hi(z1);
                        const float h0 = u0 * g0 * sigmoidf_fast(g0), h1 = u1 * g1 * sigmoidf_fast(g1);
                        *(uint32_t *)(h_w + (j * 16 + g * 4) * 2) = Elem<T>::pack(h0, h1);
                    }
                }
            }
            wave_lds_sync();
            const int rbase = wq + i * 32;
            if (write_z) {
#pragma unroll
                for (int it = 0; it < 8; ++it) {
                    const int rr = 4 * it + (lane >> 4);
                    const u32x4 v = *(const u32x4 *)(z_r + it * 4 * EPI_Z_STRIDE);
                    const int d = __shfl(dst, rr);
                    if (rbase + rr < rows_valid && cz < a.N) *(u32x4 *)(a.out + (int64_t)d * a.ldo + cz) = v;
                }
            }
            if constexpr (EPI == XMA_ROCM_EPI_SWIGLU) {
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int rr = 8 * it + (lane >> 3);
                    const u32x4 v = *(const u32x4 *)(h_r + it * 8 * EPI_H_STRIDE);
                    const int d = __shfl(dst, rr);
                    if (rbase + rr < rows_valid && 2 * ch < a.N) *(u32x4 *)(a.aux + (int64_t)d * a.ldaux + ch) = v;
                }
            }
            wave_lds_sync(); // the next block overwrites the area
        }
        };
        if (a.scale)
            blocks(IC<1>{});
        else
            blocks(IC<0>{});
    } else {
        // SwiGLU backward: the accumulators are d h for the wave's 128 columns; z and dz have twice as many (gate, up
        // interleaved).  Each 32-row block of z comes in as whole rows (2 rows of 512 bytes per instruction) through
        // the wave-private LDS area, every lane turns its own 16-byte pieces into dz in place, and the block leaves
        // the same way.  The z rows of block i + 1 are requested before the stores of block i go out: loads and
        // stores retire in order, so a load issued behind the stores would wait for them.
        unsigned char *stage = smem + wave * EPI_BWD_WAVE_BYTES;
        unsigned char *row_io = stage + (lane >> 5) * EPI_BWD_STRIDE + (lane & 31) * 16; // + 2 it rows (way in)
        unsigned char *mine = stage + lrow * EPI_BWD_STRIDE + lhalf * 16;                // + (32 j + 8 g) * 4 bytes
        // Loads and stores of this epilogue are unconditional: a lane whose row or column lies outside the tile's valid
        // part repeats the access of a lane inside it (same address, and for stores the same data, read from the same place
        // of the staging area).  Memory operations under a per-lane condition sit in branches, and the compiler then waits
        // for all of them (vmcnt(0)) where it would otherwise count: every block would wait for the stores of the one
        // before it to complete before it could bring its own rows of z into LDS.
        // this wave's 128 columns lie past N: nothing to do, and nothing in here joins other waves (the value is uniform;
        // readfirstlane tells the compiler so, which keeps the branch scalar)
        if (__builtin_amdgcn_readfirstlane(n0 + wp) >= a.N) return;
        const int piece = (2 * (n0 + wp) + (lane & 31) * 8 < 2 * a.N) ? (lane & 31) : 0; // piece 0 is inside N
        const int cz = 2 * (n0 + wp) + piece * 8; // this lane's 8 columns of z / dz on the way in and out
        float sc_i[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int r = wq + i * 32 + lrow;
            if (r >= rows_valid) r = rows_valid - 1;
            sc_i[i] = 1.f;
            if (a.scale) sc_i[i] = pre ? pre->sc[i] : Elem<T>::lo((uint32_t)a.scale[a.idx[row0 + r]]);
        }
        u32x4 zin[16];
        auto load_block = [&](int i) {
#pragma unroll
            for (int it = 0; it < 16; ++it) {
                int r = wq + i * 32 + 2 * it + (lane >> 5);
                if (r >= rows_valid) r = rows_valid - 1;
                zin[it] = *(const u32x4 *)(a.aux + (row0 + r) * a.ldaux + cz);
            }
        };
        const int i_first = only_i >= 0 ? only_i : 0, i_last = only_i >= 0 ? only_i : 3;
        if (wq + i_first * 32 < rows_valid) load_block(i_first);
        // HS: a second output, the activations scaled by the row scale, (M, N) in grouped order.  A lane keeps its 128
        // values of a block, packed in 32 registers, until the dz rows have left; then the block takes the same way out
        // through the staging area (32 rows of 128 columns, the layout of the plain store epilogue).  The 32 registers
        // are accumulation registers - the 64 of the block's own accumulators are free by then - written and read with
        // v_accvgpr moves: as ordinary variables they push the kernel's register allocation into spilling.  (Storing
        // each quad straight from registers, 8 bytes per lane = 16 bytes of 32 rows per instruction, measured slower.)
        auto park = [](uint32_t v) {
            uint32_t r;
            asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(r) : "v"(v));
            return r;
        };
        auto unpark = [](uint32_t r) {
            uint32_t v;
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(r));
            return v;
        };
        auto blocks = [&](auto HS) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (wq + i * 32 >= rows_valid) break; // wave-uniform
            if (i < i_first || i > i_last) continue;
#pragma unroll
            for (int it = 0; it < 16; ++it) *(u32x4 *)(row_io + 2 * it * EPI_BWD_STRIDE) = zin[it];
            if (i < i_last && wq + (i + 1) * 32 < rows_valid) load_block(i + 1);
            wave_lds_sync();
            const float sc = sc_i[i];
            uint32_t hs[HS.value ? 32 : 1];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x4 *zp = (u32x4 *)(mine + (j * 32 + g * 8) * 4);
                    const u32x4 z = *zp;
                    u32x4 o;
                    float hv[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float dh = acc[j][i][4 * g + q] * sc;
                        const float gg = Elem<T>::lo(z[q]), uu = Elem<T>::hi(z[q]);
                        const float sg = sigmoidf_fast(gg), silu = gg * sg;
                        o[q] = Elem<T>::pack(dh * uu * (sg + silu * (1.f - sg)), dh * silu);
                        hv[q] = uu * silu * sc;
                    }
                    *zp = o;
                    if constexpr (HS.value != 0) {
                        hs[2 * (j * 4 + g)] = park(Elem<T>::pack(hv[0], hv[1]));
                        hs[2 * (j * 4 + g) + 1] = park(Elem<T>::pack(hv[2], hv[3]));
                    }
                }
            }
            wave_lds_sync();
#pragma unroll
            for (int it = 0; it < 16; ++it) {
                int br = 2 * it + (lane >> 5); // row of the block; the block's first row is valid
                if (wq + i * 32 + br >= rows_valid) br = rows_valid - 1 - (wq + i * 32);
                const u32x4 v = *(const u32x4 *)(stage + br * EPI_BWD_STRIDE + piece * 16);
                *(u32x4 *)(a.out + (row0 + wq + i * 32 + br) * a.ldo + cz) = v;
            }
            wave_lds_sync(); // the next block overwrites the area
            if constexpr (HS.value != 0) {
                unsigned char *h_w = stage + lrow * EPI_Z_STRIDE + lhalf * 8;
                const int hpiece = (n0 + wp + (lane & 15) * 8 < a.N) ? (lane & 15) : 0; // as above: no store is conditional
                const int ch = n0 + wp + hpiece * 8; // this lane's 8 activation columns on the way out
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        *(u32x2 *)(h_w + (j * 32 + g * 8) * 2) = u32x2{unpark(hs[2 * (j * 4 + g)]), unpark(hs[2 * (j * 4 + g) + 1])};
                wave_lds_sync();
#pragma unroll
                for (int it = 0; it < 8; ++it) {
                    int br = 4 * it + (lane >> 4);
                    if (wq + i * 32 + br >= rows_valid) br = rows_valid - 1 - (wq + i * 32);
                    const u32x4 v = *(const u32x4 *)(stage + br * EPI_Z_STRIDE + hpiece * 16);
                    *(u32x4 *)(a.aux2 + (row0 + wq + i * 32 + br) * a.ldaux2 + ch) = v;
                }
                wave_lds_sync();
            }
        }
        };
        blocks(IC<(EPI == EPI_SWIGLU_BWD_SCALED_ACT) ? 1 : 0>{});
    }
}

// ------------------------------------------------------------------------------------------------
// forward / dX kernel
//   WT = 0: W[e] is (N, K) with K contiguous (x @ W^T)      -> P tile row-major
//   WT = 1: W[e] is (K, N) with N contiguous (dy @ W)       -> P tile transposed source
// ------------------------------------------------------------------------------------------------
template <typename T, int WT, int EPI, int ROLE>
__global__ __launch_bounds__(GEMM_THREADS, 1) void grouped_gemm_kernel(const FwdArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int s_sched[4];
    u32x4 *tiles = (u32x4 *)smem;
    // A persistent launch has one workgroup per compute unit, which walks the tiles b, b + gridDim.x, ... of the launch.
    const int b_end = fwd_persistent(EPI, ROLE) ? a.grid_main : (int)blockIdx.x + 1;
    for (int b = blockIdx.x; b < b_end; b += gridDim.x) {
    if (b != (int)blockIdx.x) __syncthreads(); // the staging areas of the last epilogue are dead in every wave
    // Everything derived from the thread index is derived again for every tile (the compiler cannot see through the
    // empty statement): hoisted out of the tile loop, those values would live across the main loop, which has no
    // register to spare, and be spilled.
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    TileSched ts;
    if (!locate_tile<ROLE>(a, smem, s_sched, ts, b, tid)) continue;
    const int e = ts.e, rows_valid = ts.rows_valid, n0 = ts.n0;
    const int64_t row0 = ts.row0;

    // ---- loader set-up: one fixed per-lane global pointer per LDS-DMA piece (k = 0); a step adds a uniform offset
    const uint16_t *zero = (const uint16_t *)g_zero_page;
    const int KT = (a.K + BK - 1) / BK;
    const bool k_tail = (a.K & (BK - 1)) != 0; // the last step has chunks past K: they are fetched from the zero page
    // K steps [kt0, kt1) of this workgroup: all of them, or one of ts.parts slices of a tile of the last round.  kt0 is
    // even, so step kt lives in stage kt & 1 in either case.
    const int kt0 = (ROLE == ROLE_SLICES) ? ((ts.part * KT / ts.parts) & ~1) : 0;
    const int kt1 = (ROLE == ROLE_SLICES && ts.part + 1 < ts.parts) ? (((ts.part + 1) * KT / ts.parts) & ~1) : KT;
    const uint16_t *q_ptr[8], *p_ptr[8];
    {
        const uint16_t *We = a.W + (int64_t)e * a.w_es;
        if (WT == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                int r = n0 + wave * 64 + i * 8 + (lane >> 3);
                if (r >= a.N) r = a.N - 1;
                p_ptr[i] = We + (int64_t)r * a.ldw + rowmajor_lane_chunk(i, lane) * 8;
            }
        } else {
            const int max_chunk = ((a.N - n0) >> 3) - 1; // last valid 16-byte chunk of the tile's column range
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                int cj = transposed_lane_chunk(j, lane);
                if (cj > max_chunk) cj = max_chunk; // columns past the edge are masked at the store
                p_ptr[j] = We + (int64_t)(wave * 16 + 2 * j + (lane >> 5)) * a.ldw + n0 + cj * 8;
            }
        }
    }
    const int64_t p_step = (WT == 0) ? BK : (int64_t)BK * a.ldw; // elements per K step along the P pointers
    const uint32_t lds0 = lds_addr_of(smem);

    // piece 0..15 of K step kt -> stage kt & 1 (pieces 0..7 = Q tile, 8..15 = P tile).  FULL: the caller guarantees
    // that step kt exists and has no chunk past K, so the piece is one M0 update, one 64-bit add and the load; a wave
    // with a single instruction stream cannot afford more than a few instructions per MFMA.
    auto issue_piece = [&](int kt, auto PIECE, auto FULL) {
        constexpr int piece = PIECE.value;
        constexpr int slot =
            (piece >> 3) * OP_CHUNKS + ((piece < 8 || WT == 0) ? (piece & 7) * 64 : (piece & 7) * 64); // 1 KB per piece
        if constexpr (!FULL.value) {
            if (kt >= kt1) return; // uniform
        }
        u32x4 *dst = tiles + (kt & 1) * STAGE_CHUNKS + slot + wave * 512; // a wave's 8 pieces are 8 KB apart per wave
        const uint16_t *src;
        if constexpr (piece < 8)
            src = q_ptr[piece] + (int64_t)kt * BK;
        else
            src = p_ptr[piece - 8] + (int64_t)kt * p_step;
        if constexpr (!FULL.value) {
            if (k_tail && kt == KT - 1) { // uniform branch, taken by at most one step of a tile
                asm volatile("" ::: "memory"); // keeps this rare path a branch instead of selects in every piece
                if (piece < 8 || WT == 0) {
                    if (kt * BK + rowmajor_lane_chunk(piece & 7, lane) * 8 >= a.K) src = zero;
                } else {
                    if (kt * BK + wave * 16 + 2 * (piece - 8) + (lane >> 5) >= a.K) src = zero;
                }
            }
        }
        lds_dma16(src, dst);
    };

    f32x16 acc[4][4];
    zero_acc(acc);
    const int wq = (wave & 1) * 128, wp = (wave >> 1) * 128; // wave's 128 x 128 corner inside the tile
    if (a.bias != nullptr && kt0 == 0) add_bias<T>(a, acc, e, n0, wp, lane); // the first K slice of a split tile only
    FragBase<0> qb;
    FragBase<WT> pb;
    make_frag_base<0>(qb, lds0, wq, lane);
    make_frag_base<WT>(pb, lds0 + OP_CHUNKS * 16, wp, lane);

    // The weight pieces of the first step go out before the activation rows are known: their addresses need only
    // the schedule, while the rows of a gathered tile take another dependent load (the scattered index).
    static_for<8>([&](auto P) { issue_piece(kt0, IC<8 + P.value>{}, IC<0>{}); });
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int r = wave * 64 + i * 8 + (lane >> 3);
        if (r >= rows_valid) r = rows_valid - 1; // duplicates, masked at the store
        const int64_t n = row0 + r;
        const int64_t src = a.x_grouped ? n : (int64_t)fastdiv((uint32_t)a.idx[n], a.fan_div);
        q_ptr[i] = a.X + src * a.ldx + rowmajor_lane_chunk(i, lane) * 8;
    }
    static_for<8>([&](auto P) { issue_piece(kt0, P, IC<0>{}); });
    static_for<DMA_N0>([&](auto P) { issue_piece(kt0 + 1, P, IC<0>{}); });
    // the first step has landed in every wave (the first loads of the second may be in flight)
    if (kt1 - kt0 > 1)
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(DMA_N0) : "memory");
    else
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    // Q blocks (32 rows) of this wave that hold valid rows: 4 except in an expert's last row tile.  A wave with fewer
    // skips the MFMAs and fragment reads of the empty blocks (rounded up to 0, 1, 2 or 4 blocks); it still issues its
    // share of the loads and meets every barrier.
    const int q_blocks = (rows_valid > wq) ? (rows_valid - wq + 31) >> 5 : 0;
    const int KT_full = (a.K / BK < kt1) ? a.K / BK : kt1; // end of the steps without a chunk past K
    auto main_loop = [&](auto NI_) {
        constexpr int NI = NI_.value;
        Frags f0, f1;
        if constexpr (NI > 0) {
            static_for<4>([&](auto I) { f0.p[I.value] = read_frag<WT, I.value, 0>(pb); });
            static_for<NI>([&](auto I) { f0.q[I.value] = read_frag<0, I.value, 0>(qb); });
        }
        // one K step; FULL: steps kt + 1 and kt + 2 exist and are complete
        auto k_step = [&](int kt, auto FULL) {
            // The step numbers of the loads are made opaque: otherwise the compiler turns "pointer + kt * step" into 16
            // running pointers and advances all of them with 64-bit vector adds in one lump at the end of the loop body,
            // where nothing hides them.
            int kt_a = kt + 1, kt_b = kt + 2;
            asm volatile("" : "+s"(kt_a), "+s"(kt_b));
            // rest of the loads of step kt + 1 (the first DMA_N0 went out behind the previous barrier)
            mma_step<T, WT, 0, 1, NI>(f0, f1, pb, qb, acc, [&](auto G) {
                if constexpr (G.value < DMA_N1) issue_piece(kt_a, IC<DMA_N0 + G.value>{}, FULL);
            });
            mma_step<T, WT, 0, 2, NI>(f1, f0, pb, qb, acc, [&](auto G) {
                if constexpr (G.value < DMA_N2) issue_piece(kt_a, IC<DMA_N0 + DMA_N1 + G.value>{}, FULL);
            });
            mma_step<T, WT, 0, 3, NI>(f0, f1, pb, qb, acc, NoHook());
            XMA_WAIT_LOADS_AND_BARRIER(); // step kt + 1 has landed; nobody reads this stage any more
            flip_stage(pb);
            flip_stage(qb);
            // the stage just left is free: first loads of step kt + 2; fragments of sub-step 0 of step kt + 1
            mma_step<T, WT, 0, 0, NI>(f1, f0, pb, qb, acc, [&](auto G) {
                if constexpr (G.value < DMA_N0) issue_piece(kt_b, G, FULL);
                if constexpr (G.value + 8 < DMA_N0) issue_piece(kt_b, IC<G.value + 8>{}, FULL);
            });
        };
        int kt = kt0;
        if constexpr (NI == 4)
            for (; kt + 2 < KT_full; ++kt) k_step(kt, IC<1>{});
        for (; kt < kt1; ++kt) k_step(kt, IC<0>{});
    };
    if (q_blocks > 2)
        main_loop(IC<4>{});
    else if (q_blocks == 2)
        main_loop(IC<2>{});
    else if (q_blocks == 1)
        main_loop(IC<1>{});
    else
        main_loop(IC<0>{});
    // every load has landed, every fragment read has returned (the last sub-step reads ahead into registers nobody
    // uses), and no wave touches the operand tiles any more: LDS becomes the staging area of the epilogue
    XMA_WAIT_LOADS_AND_BARRIER();

    if constexpr (ROLE == ROLE_SLICES) {
        // one K slice of a tile of the last round: the fp32 accumulators go to the workspace, 16 bytes per lane and
        // consecutive lanes side by side; grouped_gemm_fixup_kernel adds the slices and runs the epilogue
        float4 *dst = (float4 *)a.partial + (size_t)(ts.tail_index * ts.parts + ts.part) * (BM * BN / 4) + tid;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    dst[((j * 4 + i) * 4 + g) * GEMM_THREADS] =
                        make_float4(acc[j][i][4 * g], acc[j][i][4 * g + 1], acc[j][i][4 * g + 2], acc[j][i][4 * g + 3]);
    } else {
        int tid_e = threadIdx.x;
        asm volatile("" : "+v"(tid_e));
        tile_epilogue<T, EPI>(a, acc, smem, row0, rows_valid, n0, tid_e);
    }
    }
}

// Sum of the K slices of the split tiles of the last round, then the epilogue of the GEMM kernel.  Four workgroups
// per split tile, one per 32-row block of the waves' corners (a quarter of the loads each: the kernel is a chain of
// dependent round trips, so it is as fast as it is parallel); the slices are added in a fixed order, so the result does
// not depend on timing.
template <typename T, int EPI>
__global__ __launch_bounds__(GEMM_THREADS, 1) void grouped_gemm_fixup_kernel(const FwdArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int s_sched[4];
    TileSched ts;
    if (!locate_tile<ROLE_FIXUP>(a, smem, s_sched, ts, (int)blockIdx.x, (int)threadIdx.x)) return;
    const int tid = threadIdx.x;
    const int iblk = blockIdx.x & 3;
    f32x16 acc[4][4];
    zero_acc(acc);
    for (int p = 0; p < ts.parts; ++p) {
        const float4 *src = (const float4 *)a.partial + (size_t)(ts.tail_index * ts.parts + p) * (BM * BN / 4) + tid;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (i != iblk) continue;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float4 v = src[((j * 4 + i) * 4 + g) * GEMM_THREADS];
                    acc[j][i][4 * g] += v.x, acc[j][i][4 * g + 1] += v.y, acc[j][i][4 * g + 2] += v.z, acc[j][i][4 * g + 3] += v.w;
                }
            }
    }
    tile_epilogue<T, EPI>(a, acc, smem, ts.row0, ts.rows_valid, ts.n0, (int)threadIdx.x, iblk);
}

// ------------------------------------------------------------------------------------------------
// Persistent forward / dX kernel: one workgroup per compute unit walks the tiles b, b + gridDim.x, ... of the launch and
// overlaps the set-up of a tile with the epilogue of the tile before it.
//
// Between two main loops a workgroup has to find its next tile, fetch the scattered row indices, and wait for the first
// K step to arrive from HBM: three dependent round trips with idle matrix pipes, as long as the epilogue itself.  Here
// everything a tile needs is fetched one tile ahead: while tile i is in its main loop the schedule entry, the gathered
// row indices and the epilogue's indices of tile i + 1 are loaded into registers, and the 16 LDS-DMA pieces of the first
// K step of tile i + 1 go out right behind the last barrier of tile i's main loop, before its epilogue starts.  They land
// in stage 0 while the epilogue stages its rows in the LDS above it (stage 1 and the 32 KB that the two stages leave
// free), so the next main loop starts as soon as the epilogue's stores have been handed over.
//
// The LDS-DMA loads are issued from inline assembly here (M0 is written next to the load): the compiler guards every
// LDS access it cannot prove disjoint from an LDS-DMA load it knows of with s_waitcnt vmcnt(0), which would make the
// epilogue wait for the loads it is supposed to hide.  What the compiler does not know it cannot wait for too little
// either: vmcnt retires in order, so a wait sized for the compiler's own loads only ever covers more than it has to; the
// waits that protect the operand tiles are all explicit.
//
// The expert-major schedule (tiles before each expert, row offsets) is computed once per workgroup into LDS instead of
// once per tile.  E <= PST_MAX_E; launches with more experts use grouped_gemm_kernel.
// ------------------------------------------------------------------------------------------------
constexpr int PST_MAX_E = 1023;
constexpr int PST_SMEM_BYTES = 160 * 1024 - 64;
constexpr int PST_STAGING_OFF = STAGE_CHUNKS * 16; // the epilogue's staging area starts above stage 0
// Rows fetched one tile ahead wait in LDS, one dword per lane and item (1 KB per item), so that no register is held
// across the main loop: 8 gathered rows of the next tile, 2 x 4 rows of the epilogue (next tile's arrive while this
// tile's are still needed), 4 row scales of this tile.
constexpr int PST_ROWS_OFF = PST_STAGING_OFF + 4 * EPI_BWD_WAVE_BYTES;
constexpr int PST_QR = 0, PST_ER = 8, PST_SC = 16, PST_ROW_ITEMS = 20;
constexpr int PST_TABLE_OFF = PST_SMEM_BYTES - 2 * (PST_MAX_E + 1) * (int)sizeof(int);
constexpr int PST_STEP_LDS_OFF = PST_ROWS_OFF + PST_ROW_ITEMS * 1024; // timing build: 8 bytes per K step, up to the tables
static_assert(EPI_BWD_WAVE_BYTES >= EPI_WAVE_BYTES && PST_ROWS_OFF + PST_ROW_ITEMS * 1024 <= PST_TABLE_OFF,
              "epilogue staging and the prefetched rows must fit between stage 0 and the schedule tables");

__device__ __forceinline__ void lds_dma16_raw(const void *src, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_wave_base), "v"(src)
                 : "memory", "m0");
}
// one dword per lane: lane l's value lands at lds_wave_base + 4 l
__device__ __forceinline__ void lds_dma4_raw(const void *src, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_wave_base), "v"(src)
                 : "memory", "m0");
}

// Optional phase stamps of the persistent kernel (builds with -DXMA_PST_TIMING only): workgroup b writes the 100 MHz
// real-time counter at six points of each of its first PST_TIMING_TILES tiles; xma_rocm_debug_pst_times copies them out.
#ifdef XMA_PST_TIMING
constexpr int PST_TIMING_TILES = 48;
__device__ uint64_t g_pst_times[256][PST_TIMING_TILES][8];
__device__ uint64_t g_pst_cycles[256][PST_TIMING_TILES][8]; // the shader clock counter at the same points
__device__ int g_pst_no_ovl; // A/B switch of the timing build: 1 = no tile overlaps its neighbours' set-up
// the shader clock counter behind every K step of one tile per workgroup (the PST_STEP_TILE-th): written to a spare
// corner of LDS inside the loop (a vector store to memory would enter the loop's vmcnt waits), copied out behind the tile
constexpr int PST_STEP_TILE = 3, PST_MAX_STEPS = 240;
__device__ uint64_t g_pst_steps[256][PST_MAX_STEPS];
#define PST_STEP_STAMP(kt)                                                                             \
    do {                                                                                               \
        if (tile_no == PST_STEP_TILE && threadIdx.x == 0 && (kt) < PST_MAX_STEPS)                      \
            ((uint64_t *)(smem + PST_STEP_LDS_OFF))[(kt)] = __builtin_amdgcn_s_memtime();             \
    } while (0)
#define PST_STAMP(k)                                                                                   \
    do {                                                                                               \
        if (threadIdx.x == 0 && blockIdx.x < 256 && tile_no < PST_TIMING_TILES) {                      \
            g_pst_times[blockIdx.x][tile_no][k] = __builtin_amdgcn_s_memrealtime();                    \
            g_pst_cycles[blockIdx.x][tile_no][k] = __builtin_amdgcn_s_memtime();                       \
        }                                                                                              \
    } while (0)
#else
#define PST_STAMP(k) \
    do {             \
    } while (0)
#define PST_STEP_STAMP(kt) \
    do {                   \
    } while (0)
#endif

struct PstTile {
    int valid, t, e, n0, rows_valid, row0; // t: position in the workgroup's walk (linear tile id before the XCD remap)
};

template <typename T, int WT, int EPI>
__global__ __launch_bounds__(GEMM_THREADS, 1) void grouped_gemm_persistent_kernel(const FwdArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    int *s_pre = (int *)(smem + PST_TABLE_OFF); // [E + 1] tiles of the experts before e
    int *s_hi = s_pre + (PST_MAX_E + 1);        // [E] inclusive row offsets
    const int NT = (a.N + BN - 1) / BN;
    const int KT = (a.K + BK - 1) / BK;
    const int KT_full = a.K / BK;                // end of the steps without a chunk past K
    const bool k_tail = (a.K & (BK - 1)) != 0;
    const uint16_t *zero = (const uint16_t *)g_zero_page;
    const uint32_t lds0 = lds_addr_of(smem);

    // ---- schedule tables, once per workgroup
    {
        const int tid0 = threadIdx.x, lane0 = tid0 & 63;
        if (tid0 < WAVE) {
            int carry = 0;
            for (int b = 0; b < a.E; b += WAVE) {
                const int x = b + lane0;
                int v = 0;
                if (x < a.E) {
                    const int64_t hi = a.offs[x];
                    const int64_t cnt = hi - (x ? a.offs[x - 1] : 0);
                    v = (int)((cnt + BM - 1) / BM) * NT;
                    s_hi[x] = (int)hi;
                }
                int s = v;
#pragma unroll
                for (int d = 1; d < WAVE; d <<= 1) {
                    const int t = __shfl_up(s, d);
                    if (lane0 >= d) s += t;
                }
                if (x < a.E) s_pre[x] = carry + s - v;
                carry += __shfl(s, WAVE - 1);
            }
            if (lane0 == 0) s_pre[a.E] = carry;
        }
        __syncthreads();
    }
    int full = __builtin_amdgcn_readfirstlane(s_pre[a.E]); // tiles this launch computes whole
    if (a.partial) { // the tiles of a last, partial round are left to the K-slice and fix-up launches (see locate_tile)
        const int total = full;
        full = total / a.split_cus * a.split_cus;
        const int rest = total - full;
        int parts = rest ? a.split_cus / rest : 1;
        if (parts > KT / SPLIT_MIN_STEPS) parts = KT / SPLIT_MIN_STEPS;
        if (parts < 2) full = total;
    }

    // first tile at or behind position t of this workgroup's walk (every wave computes the same, from LDS only)
    auto lookup = [&](int t, int lane) -> PstTile {
        PstTile r = {0, 0, 0, 0, 0, 0};
        for (; t < a.grid_main; t += gridDim.x) {
            const int L = xcd_remap(t, a.grid_main);
            if (L >= full) continue;
            int e;
            if (a.E <= WAVE) {
                const int x = lane < a.E ? lane : a.E;
                const int lo = s_pre[x], hi = s_pre[x < a.E ? x + 1 : a.E];
                e = __builtin_ctzll(__ballot(lo <= L && L < hi));
            } else { // two levels of 64-way search
                const int seg = (a.E + WAVE - 1) / WAVE;
                const int x1 = lane * seg < a.E ? lane * seg : a.E;
                const int b0 = (63 - __builtin_clzll(__ballot(s_pre[x1] <= L))) * seg;
                const int x = b0 + lane < a.E ? b0 + lane : a.E;
                const int lo = s_pre[x], hi = s_pre[x < a.E ? x + 1 : a.E];
                e = b0 + __builtin_ctzll(__ballot(lane < seg && lo <= L && L < hi));
            }
            e = __builtin_amdgcn_readfirstlane(e);
            const int local = L - __builtin_amdgcn_readfirstlane(s_pre[e]);
            const int row_hi = __builtin_amdgcn_readfirstlane(s_hi[e]);
            const int row_lo = e ? __builtin_amdgcn_readfirstlane(s_hi[e - 1]) : 0;
            const int tiles_m = (row_hi - row_lo + BM - 1) / BM;
            int m_tile, n_tile;
            tile_of_expert(local, tiles_m, NT, m_tile, n_tile);
            r.valid = 1;
            r.t = t;
            r.e = e;
            r.row0 = row_lo + m_tile * BM;
            r.rows_valid = (row_hi - r.row0 < BM) ? row_hi - r.row0 : BM;
            r.n0 = n_tile * BN;
            break;
        }
        return r;
    };
    // Rows of a lane: the 8 rows of its LDS-DMA pieces (q) and the 4 rows of its epilogue (e), clamped to the tile's last
    // valid row (duplicates are computed and never stored).  Where a row's scattered index is needed, its low dword is
    // fetched by a 4-byte LDS-DMA load into the lane's slot of an item of the row area and read back behind the main loop.
    const uint32_t *idx32 = (const uint32_t *)a.idx;
    const bool need_q_idx = !a.x_grouped, need_e_idx = !a.y_grouped || a.scale != nullptr;
    auto q_row = [&](const PstTile &t, int i, int lane, int wave) {
        const int r = wave * 64 + i * 8 + (lane >> 3);
        return t.row0 + (r < t.rows_valid ? r : t.rows_valid - 1);
    };
    auto e_row = [&](const PstTile &t, int i, int lane, int wave) {
        const int r = (wave & 1) * 128 + i * 32 + (lane & 31);
        return t.row0 + (r < t.rows_valid ? r : t.rows_valid - 1);
    };
    auto row_item_lds = [&](int item, int wave) { return lds0 + (uint32_t)(PST_ROWS_OFF + item * 1024 + wave * 256); };
    auto row_item = [&](int item, int tid) { return ((const uint32_t *)(smem + PST_ROWS_OFF + item * 1024))[tid]; };
    auto prefetch_rows = [&](const PstTile &t, int lane, int wave, bool q, int e_buf) {
        if (q && need_q_idx) {
#pragma unroll
            for (int i = 0; i < 8; ++i) lds_dma4_raw(idx32 + 2 * (int64_t)q_row(t, i, lane, wave), row_item_lds(PST_QR + i, wave));
        }
        if (need_e_idx) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                lds_dma4_raw(idx32 + 2 * (int64_t)e_row(t, i, lane, wave), row_item_lds(PST_ER + 4 * e_buf + i, wave));
        }
    };

    // The same fetches as 16 items of one LDS-DMA load each, for the first K step of a tile to issue one by one between
    // its MFMAs: 0..7 the gathered rows of the next tile, 8..11 the rows of its epilogue, 12..15 the row scales of this
    // tile.  An item that is not needed loads from the zero page instead, so that their number is always 16 and the wait
    // in front of that step's barrier can leave exactly these loads in flight.
    auto prefetch_item = [&](auto ITEM, const PstTile &t, int lane, int wave, int tid, int e_buf) {
        constexpr int it = ITEM.value;
        const void *src = zero;
        uint32_t dst;
        if constexpr (it < 8) {
            dst = row_item_lds(PST_QR + it, wave);
            if (t.valid && need_q_idx) src = idx32 + 2 * (int64_t)q_row(t, it, lane, wave);
        } else if constexpr (it < 12) {
            dst = row_item_lds(PST_ER + 4 * (e_buf ^ 1) + (it - 8), wave);
            if (t.valid && need_e_idx) src = idx32 + 2 * (int64_t)e_row(t, it - 8, lane, wave);
        } else {
            dst = row_item_lds(PST_SC + (it - 12), wave);
            if (a.scale) src = (const uint32_t *)a.scale + (row_item(PST_ER + 4 * e_buf + (it - 12), tid) >> 1);
        }
        lds_dma4_raw(src, dst);
    };

    // Addresses of the 16 LDS-DMA pieces of a tile: a uniform base per operand (SGPRs: the tile's corner of the weight
    // matrix; the activations' first row for a gathered operand, the tile's first row for a grouped one) and one 32-bit
    // byte offset per piece and lane.  A K step adds a uniform amount to the bases, so a piece in the loop is the M0
    // update and the load, without any vector address arithmetic.  The host has checked that the offsets fit 32 bits.
    uint32_t q_off[8], p_off[8];
    const char *q_base = nullptr, *p_base = nullptr;
    const int64_t p_step_b = (WT == 0) ? 2 * BK : (int64_t)2 * BK * a.ldw; // bytes per K step along the weights
    // offsets of pieces i (activations) and 8 + i (weights); i == 0 also sets the two bases; raw: the row of piece i (its
    // scattered index for a gathered operand)
    auto make_pointer = [&](const PstTile &t, auto I_, int lane, int wave, uint32_t raw) {
        constexpr int i = I_.value;
        if constexpr (i == 0) {
            const uint16_t *We = a.W + (int64_t)t.e * a.w_es;
            p_base = (WT == 0) ? (const char *)(We + (int64_t)t.n0 * a.ldw) : (const char *)(We + t.n0);
            q_base = (const char *)(need_q_idx ? a.X : a.X + (int64_t)t.row0 * a.ldx);
        }
        if (WT == 0) {
            int r = wave * 64 + i * 8 + (lane >> 3);
            if (t.n0 + r >= a.N) r = a.N - 1 - t.n0;
            p_off[i] = (uint32_t)r * (uint32_t)(2 * a.ldw) + rowmajor_lane_chunk(i, lane) * 16;
        } else {
            const int max_chunk = ((a.N - t.n0) >> 3) - 1;
            int cj = transposed_lane_chunk(i, lane);
            if (cj > max_chunk) cj = max_chunk;
            p_off[i] = (uint32_t)(wave * 16 + 2 * i + (lane >> 5)) * (uint32_t)(2 * a.ldw) + cj * 16;
        }
        const uint32_t src = need_q_idx ? fastdiv(raw, a.fan_div) : raw - (uint32_t)t.row0;
        q_off[i] = src * (uint32_t)(2 * a.ldx) + rowmajor_lane_chunk(i, lane) * 16;
    };
    auto make_pointers = [&](const PstTile &t, int lane, int wave, const uint32_t (&raw)[8]) {
        static_for<8>([&](auto I) { make_pointer(t, I, lane, wave, raw[I.value]); });
    };
    // piece 0..15 of K step kt of the tile the bases and offsets describe -> stage kt & 1; FULL: the step exists and has
    // no chunk past K
    int wave_u = 0; // this wave's index, set per tile (uniform)
    int lane_v = 0;
    auto issue_piece = [&](int kt, auto PIECE, auto FULL) {
        constexpr int piece = PIECE.value;
        if constexpr (!FULL.value) {
            if (kt >= KT) return; // uniform
        }
        // LDS destination = the piece's place in stage 0 (loop invariant) + the stage; both uniform
        const uint32_t dst0 = lds0 + (uint32_t)(((piece >> 3) * OP_CHUNKS + (piece & 7) * 64 + wave_u * 512) * 16);
        const uint32_t stage = (uint32_t)((kt & 1) * STAGE_CHUNKS * 16);
        const uint32_t dst = dst0 + stage;
        const char *base = (piece < 8) ? q_base + (int64_t)kt * (2 * BK) : p_base + (int64_t)kt * p_step_b; // uniform
        const uint32_t off = (piece < 8) ? q_off[piece] : p_off[piece - 8];
        if constexpr (FULL.value) {
            // the base is uniform by construction; where the register allocation keeps it in vector registers all the
            // same, the two readfirstlane bring it back (they fold away where it already is scalar)
            const uint64_t b64 = (uint64_t)base;
            const char *ubase = (const char *)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b64 >> 32)) << 32) |
                                               (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b64));
            asm volatile("s_add_i32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3" ::"s"(dst0), "s"(stage), "v"(off),
                         "s"(ubase)
                         : "memory", "m0", "scc");
        } else {
            const char *src = base + off;
            if (k_tail && kt == KT - 1) {
                asm volatile("" ::: "memory");
                if (piece < 8 || WT == 0) {
                    if (kt * BK + rowmajor_lane_chunk(piece & 7, lane_v) * 8 >= a.K) src = (const char *)zero;
                } else {
                    if (kt * BK + wave_u * 16 + 2 * (piece - 8) + (lane_v >> 5) >= a.K) src = (const char *)zero;
                }
            }
            lds_dma16_raw(src, dst);
        }
    };

    // ---- first tile: its gathered rows are fetched on the spot, the rows of its epilogue go the way of all later ones
    PstTile cur;
    int e_buf = 0; // which of the two epilogue-row buffers holds the current tile's
    {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        cur = lookup((int)blockIdx.x, lane);
        if (!cur.valid) return;
        uint32_t q_raw[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int n = q_row(cur, i, lane, wave);
            q_raw[i] = need_q_idx ? idx32[2 * (int64_t)n] : (uint32_t)n;
        }
        make_pointers(cur, lane, wave, q_raw);
        wave_u = wave, lane_v = lane;
        static_for<16>([&](auto P) { issue_piece(0, P, IC<0>{}); });
        prefetch_rows(cur, lane, wave, false, e_buf);
    }

#ifdef XMA_PST_TIMING
    const bool ovl_allowed = !g_pst_no_ovl;
#else
    constexpr bool ovl_allowed = true;
#endif
    [[maybe_unused]] int tile_no = 0;
    for (;; ++tile_no) {
        PST_STAMP(0);
        // Everything derived from the thread index is derived again for every tile behind an opaque copy of it: hoisted
        // out of the tile loop those values would live across the main loop and be spilled.
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        wave_u = wave, lane_v = lane;
        // the first K step and the rows of this tile's epilogue have landed in every wave, the stores of the last
        // epilogue have been handed over and its staging area is dead
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        PST_STAMP(1);
        if (KT_full >= 2) // the second K step exists and is complete: the short form of the loads
            static_for<DMA_N0>([&](auto P) { issue_piece(1, P, IC<1>{}); });
        else
            static_for<DMA_N0>([&](auto P) { issue_piece(1, P, IC<0>{}); });

        // One tile ahead: the next tile's schedule entry and rows, and this tile's row scales (their addresses are the
        // epilogue's row indices, fetched a tile ago); all of it lands in LDS during the main loop.  A full tile with an
        // even number of at least four K steps does this between the MFMAs of its first K step, and sets up and issues
        // the first K step of the next tile between the MFMAs of its last one (`ovl`); any other tile does it here and
        // behind the loop, with idle matrix pipes.
        const int wq = (wave & 1) * 128, wp = (wave >> 1) * 128;
        const int q_blocks = (cur.rows_valid > wq) ? (cur.rows_valid - wq + 31) >> 5 : 0;
        // uniform over the workgroup: the waves of a tile's lower half (wq == 0) and upper half disagree on q_blocks, so
        // the decision is taken on the tile's row count
        const bool ovl = cur.rows_valid > 128 + 64 && (KT & 1) == 0 && KT >= 4 && ovl_allowed;
        PstTile nxt = {0, 0, 0, 0, 0, 0};
        if (!ovl) {
            nxt = lookup(cur.t + (int)gridDim.x, lane);
            if (nxt.valid) prefetch_rows(nxt, lane, wave, true, e_buf ^ 1);
            if (a.scale) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // the aligned dword that holds the 16-bit scale (the host checks that the vector starts on 4 bytes)
                    const uint32_t s_idx = row_item(PST_ER + 4 * e_buf + i, tid);
                    lds_dma4_raw((const uint32_t *)a.scale + (s_idx >> 1), row_item_lds(PST_SC + i, wave));
                }
            }
        }

        PST_STAMP(2);
        f32x16 acc[4][4];
        init_acc<T>(a, acc, cur.e, cur.n0, wp, lane);
        FragBase<0> qb;
        FragBase<WT> pb;
        make_frag_base<0>(qb, lds0, wq, lane);
        make_frag_base<WT>(pb, lds0 + OP_CHUNKS * 16, wp, lane);
        auto main_loop = [&](auto NI_) {
            constexpr int NI = NI_.value;
            Frags f0, f1;
            if constexpr (NI > 0) {
                static_for<4>([&](auto I) { f0.p[I.value] = read_frag<WT, I.value, 0>(pb); });
                static_for<NI>([&](auto I) { f0.q[I.value] = read_frag<0, I.value, 0>(qb); });
            }
            // One K step.  FULL = 1: steps kt + 1 and kt + 2 exist and are complete; FULL = 2: step kt + 1 exists and is
            // complete and is the tile's last (nothing is loaded for kt + 2); FULL = 0: every piece checks.  MODE 1, the first step of a tile that
            // overlaps (`ovl`): the free slots of its second half take the next tile's schedule entry and the 16 row
            // items; they are the youngest loads at the step's barrier, which leaves exactly them in flight.  MODE 2, the
            // last step of such a tile (it lives in stage 1, stage 0 has been free since the barrier before): its slots
            // take the operand addresses of the next tile and the 16 pieces of that tile's first K step, which stay in
            // flight through the epilogue.  The loads of this tile have all been issued by then.
            auto k_step = [&](int kt, auto FULL, auto MODE) {
                constexpr int mode = MODE.value;
                int kt_a = kt + 1, kt_b = kt + 2;
                asm volatile("" : "+s"(kt_a), "+s"(kt_b));
                // MODE 2: the next tile's eight gathered rows, read from the row area in one go in front of the step's MFMAs
                // (one wait for all of them; read inside the slots, each would stall the MFMA stream for an LDS round trip)
                [[maybe_unused]] uint32_t nxt_rows[8];
                if constexpr (mode == 2) {
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        nxt_rows[i] = need_q_idx ? row_item(PST_QR + i, tid) : (uint32_t)q_row(nxt, i, lane, wave);
                }
                mma_step<T, WT, 0, 1, NI>(f0, f1, pb, qb, acc, [&](auto G) {
                    if constexpr (mode == 2) {
                        // also when there is no next tile (all fields zero then: addresses that nothing is loaded from):
                        // a branch here would only add a join of sixteen registers to the loop
                        make_pointer(nxt, G, lane, wave, nxt_rows[G.value]);
                    } else if constexpr (G.value < DMA_N1) {
                        issue_piece(kt_a, IC<DMA_N0 + G.value>{}, IC<(FULL.value != 0) ? 1 : 0>{});
                    }
                });
                mma_step<T, WT, 0, 2, NI>(f1, f0, pb, qb, acc, [&](auto G) {
                    if constexpr (mode == 1) {
                        if constexpr (G.value == 0) nxt = lookup(cur.t + (int)gridDim.x, lane);
                    } else if constexpr (mode == 2) {
                        if (nxt.valid) issue_piece(0, G, IC<1>{});
                    } else if constexpr (G.value < DMA_N2) {
                        issue_piece(kt_a, IC<DMA_N0 + DMA_N1 + G.value>{}, IC<(FULL.value != 0) ? 1 : 0>{});
                    }
                });
                mma_step<T, WT, 0, 3, NI>(f0, f1, pb, qb, acc, [&](auto G) {
                    if constexpr (mode == 1) {
                        prefetch_item(IC<2 * G.value>{}, nxt, lane, wave, tid, e_buf);
                        prefetch_item(IC<2 * G.value + 1>{}, nxt, lane, wave, tid, e_buf);
                    } else if constexpr (mode == 2) {
                        if (nxt.valid) issue_piece(0, IC<8 + G.value>{}, IC<1>{});
                    }
                });
                if constexpr (mode == 0)
                    XMA_WAIT_LOADS_AND_BARRIER(); // step kt + 1 has landed; nobody reads this stage any more
                else
                    asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory"); // all but the 16 youngest
                flip_stage(pb);
                flip_stage(qb);
                mma_step<T, WT, 0, 0, NI, (mode == 2 ? 0 : 1)>(f1, f0, pb, qb, acc, [&](auto G) {
                    if constexpr (mode != 2 && FULL.value != 2) {
                        if constexpr (G.value < DMA_N0) issue_piece(kt_b, G, FULL);
                        if constexpr (G.value + 8 < DMA_N0) issue_piece(kt_b, IC<G.value + 8>{}, FULL);
                    }
                });
                PST_STEP_STAMP(kt);
            };
            int kt = 0, kt_end = KT;
            if constexpr (NI == 4) {
                if (ovl) { // KT >= 4, so the first step is followed by two complete ones
                    k_step(0, IC<1>{}, IC<1>{});
                    kt = 1, kt_end = KT - 1;
                }
                for (; kt + 2 < KT_full && kt < kt_end; ++kt) k_step(kt, IC<1>{}, IC<0>{});
                if (kt + 2 == KT && kt + 1 < KT_full && kt < kt_end) { // the step in front of a complete last step
                    k_step(kt, IC<2>{}, IC<0>{});
                    ++kt;
                }
            }
            for (; kt < kt_end; ++kt) k_step(kt, IC<0>{}, IC<0>{});
            if constexpr (NI == 4) {
                if (ovl) k_step(KT - 1, IC<0>{}, IC<2>{});
            }
        };
        if (q_blocks > 2)
            main_loop(IC<4>{});
        else if (q_blocks == 2)
            main_loop(IC<2>{});
        else if (q_blocks == 1)
            main_loop(IC<1>{});
        else
            main_loop(IC<0>{});
        if (ovl) {
            // The waves met at the last step's barrier with their reads of stage 1 done (the last sub-step reads no
            // fragments ahead); only the next tile's first K step is in flight, into stage 0.
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        } else {
            // every load has landed (the index loads above as well), no wave touches the operand tiles any more
            XMA_WAIT_LOADS_AND_BARRIER();
        }
        PST_STAMP(3);

        int tid_e = threadIdx.x;
        asm volatile("" : "+v"(tid_e));
        const int lane_e = tid_e & 63, wave_e = __builtin_amdgcn_readfirstlane(tid_e >> 6);
        if (!ovl && nxt.valid) { // first K step of the next tile: in flight during the epilogue
            uint32_t q_raw[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                q_raw[i] = need_q_idx ? row_item(PST_QR + i, tid_e) : (uint32_t)q_row(nxt, i, lane_e, wave_e);
            make_pointers(nxt, lane_e, wave_e, q_raw);
            wave_u = wave_e, lane_v = lane_e;
            static_for<16>([&](auto P) { issue_piece(0, P, IC<0>{}); });
        }
        PST_STAMP(4);
        EpiRows er;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t s_idx = need_e_idx ? row_item(PST_ER + 4 * e_buf + i, tid_e) : 0u;
            er.idx[i] = (int)s_idx;
            er.sc[i] = 1.f;
            if (a.scale) {
                const uint32_t w = row_item(PST_SC + i, tid_e);
                er.sc[i] = (s_idx & 1) ? Elem<T>::hi(w) : Elem<T>::lo(w);
            }
        }
        tile_epilogue<T, EPI>(a, acc, smem + PST_STAGING_OFF, cur.row0, cur.rows_valid, cur.n0, tid_e, -1, &er);
        PST_STAMP(5);
#ifdef XMA_PST_TIMING
        if (tile_no == PST_STEP_TILE && threadIdx.x == 0 && blockIdx.x < 256)
            for (int q = 0; q < KT && q < PST_MAX_STEPS; ++q) g_pst_steps[blockIdx.x][q] = ((uint64_t *)(smem + PST_STEP_LDS_OFF))[q];
#endif
        if (!nxt.valid) break;
        cur = nxt;
        e_buf ^= 1;
    }
}

// ------------------------------------------------------------------------------------------------
// dW kernel: DW[e][o][i] = sum_n DY[n][o] X[n][i]; both operands are token-major = transposed sources; the K loop
// runs over the expert's row range, k-rows past its end come from the zero page.
//   GQ / GP = 1: the rows of dY / X are taken through sorted_scattered_idxs (index / fan_out); 0: grouped order
// ------------------------------------------------------------------------------------------------
constexpr int DW_BAND = 4;
#ifdef XMA_PST_TIMING
// timing build: shader clock counter of the first DW_TIMING_TILES workgroups at the start of the kernel, in front of and
// behind the K loop and at the end, and the tile's K step count
constexpr int DW_TIMING_TILES = 8192;
__device__ uint64_t g_dw_cycles[DW_TIMING_TILES][6];
#define DW_STAMP(k)                                                                   \
    do {                                                                              \
        if (threadIdx.x == 0 && blockIdx.x < DW_TIMING_TILES)                          \
            g_dw_cycles[blockIdx.x][k] = (k) == 4 ? (uint64_t)KT : __builtin_amdgcn_s_memtime(); \
    } while (0)
#else
#define DW_STAMP(k) \
    do {            \
    } while (0)
#endif
template <typename T, int GQ, int GP>
__global__ __launch_bounds__(GEMM_THREADS, 1) void grouped_gemm_dw_kernel(const DwArgs a) {
    constexpr int GATHER = GQ | GP;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    u32x4 *tiles = (u32x4 *)smem;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int OT = (a.N_out + 255) / 256, IT = (a.K_in + 255) / 256;
    // Tile walk: inside an expert the tiles are taken in bands of DW_BAND tile rows, down the band first, so that the 32
    // consecutive tiles an XCD gets from xcd_remap form a DW_BAND x (32 / DW_BAND) block that shares DW_BAND dY panels and
    // 32 / DW_BAND X panels in that XCD's L2 (a row-by-row walk shares 1 + 32).
    const int L = xcd_remap(blockIdx.x, gridDim.x);
    const int rem = L % (OT * IT);
    // Experts are taken in the order of decreasing row count (equal counts: lower index first), the longest K loops
    // first: a tile's duration is proportional to its expert's rows, and with skewed routing a large expert that came up
    // last would keep a few compute units busy long after all others have finished.  Every wave ranks the experts in
    // registers (lane = expert); with more experts than lanes the order stays the index order.
    int e = L / (OT * IT);
    if (a.E <= WAVE) {
        const int64_t hi = a.offs[lane < a.E ? lane : a.E - 1];
        int64_t lo = __shfl_up(hi, 1);
        if (lane == 0) lo = 0;
        const int cnt = (lane < a.E) ? (int)(hi - lo) : -1;
        int rank = 0;
        for (int i = 0; i < a.E; ++i) {
            const int ci = __builtin_amdgcn_readlane(cnt, i);
            rank += (ci > cnt || (ci == cnt && i < lane)) ? 1 : 0;
        }
        e = __builtin_ctzll(__ballot(rank == e && lane < a.E)); // exactly one lane
    }
    const int band = rem / (DW_BAND * IT), in_band = rem % (DW_BAND * IT);
    const int band_rows = (OT - band * DW_BAND < DW_BAND) ? OT - band * DW_BAND : DW_BAND;
    const int o0 = (band * DW_BAND + in_band % band_rows) * 256, i0 = (in_band / band_rows) * 256;
    const int64_t row_lo = e ? a.offs[e - 1] : 0, row_hi = a.offs[e];
    const int rows = (int)(row_hi - row_lo);
    const int KT = (rows + BK - 1) / BK;
    DW_STAMP(0);
    DW_STAMP(4);
    const uint16_t *zero = (const uint16_t *)g_zero_page;
    const int q_max_chunk = ((a.N_out - o0) >> 3) - 1, p_max_chunk = ((a.K_in - i0) >> 3) - 1;
    const int kr_lane = wave * 16 + (lane >> 5); // this lane's k-rows of a step: kr_lane + 2 j, j = 0..7

    // Per-lane column offsets (elements) of the 8 pieces of each operand; rows change every step.  For an operand in
    // grouped order the row is row_lo + 64 kt + kr, so the piece pointer advances by a uniform 64 ld per step.
    int q_col[8], p_col[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        int cq = transposed_lane_chunk(j, lane), cp = cq;
        if (cq > q_max_chunk) cq = q_max_chunk; // columns past the edge are masked at the store
        if (cp > p_max_chunk) cp = p_max_chunk;
        q_col[j] = o0 + cq * 8;
        p_col[j] = i0 + cp * 8;
    }
    // Per-lane byte pointers of the 8 pieces of each operand: for an operand in grouped order the address of step 0
    // (the row is row_lo + 64 kt + kr, so a step adds a uniform 64 rows); for a gathered operand the column position in
    // row 0, to which token * row pitch is added (one 32 x 32 -> 64-bit multiply-add per piece).
    const uint32_t lddy_b = (uint32_t)a.lddy * 2, ldx_b = (uint32_t)a.ldx * 2;
    const char *q_base[8], *p_base[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        q_base[j] = (const char *)(a.DY + q_col[j]) + (GQ ? 0 : (row_lo + kr_lane + 2 * j) * (int64_t)lddy_b);
        p_base[j] = (const char *)(a.X + p_col[j]) + (GP ? 0 : (row_lo + kr_lane + 2 * j) * (int64_t)ldx_b);
    }

    // Scattered indices of this lane's 8 tokens of the step that is loaded next.  They are fetched one step ahead with
    // inline assembly (low dword of the int64 index): the compiler would guard the later use of a loop-carried loaded
    // register with a wait of its own choosing; here the wait is the vmcnt(0) in front of each step's barrier, and
    // use_idx() ties the registers to a point behind it.  FULL: all rows of the step lie inside the expert, the address
    // is one per-lane pointer plus an immediate.
    uint32_t idx_next[8];
    const int64_t *idx_lane = a.idx + row_lo + kr_lane;
    auto load_idx_one = [&](int kt, auto J, auto FULL) {
        constexpr int j = J.value;
        if constexpr (FULL.value) {
            const int64_t *src = idx_lane + (int64_t)kt * BK;
            asm volatile("global_load_dword %0, %1, off offset:%2" : "=v"(idx_next[j]) : "v"(src), "n"(16 * j) : "memory");
        } else {
            int r = kt * BK + kr_lane + 2 * j;
            if (r >= rows) r = rows - 1; // clamped, never predicated
            const int64_t *src = a.idx + row_lo + r;
            asm volatile("global_load_dword %0, %1, off" : "=v"(idx_next[j]) : "v"(src) : "memory");
        }
    };
    auto load_idx = [&](int kt) { static_for<8>([&](auto J) { load_idx_one(kt, J, IC<0>{}); }); };
    auto use_idx = [&]() {
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(idx_next[0]), "+v"(idx_next[1]), "+v"(idx_next[2]), "+v"(idx_next[3]), "+v"(idx_next[4]),
                       "+v"(idx_next[5]), "+v"(idx_next[6]), "+v"(idx_next[7]));
    };
    // piece 0..15 of K step kt (0..7 = dY tile, 8..15 = X tile); FULL: step kt exists and lies inside the expert's rows
    auto issue_piece = [&](int kt, auto PIECE, auto FULL) {
        constexpr int piece = PIECE.value, j = piece & 7;
        if constexpr (!FULL.value) {
            if (kt >= KT) return; // uniform
        }
        u32x4 *dst = tiles + (kt & 1) * STAGE_CHUNKS + (piece >> 3) * OP_CHUNKS + j * 64 + wave * 512;
        const char *src;
        if constexpr (piece < 8) {
            if (GQ)
                src = q_base[j] + (uint64_t)fastdiv(idx_next[j], a.dy_div) * lddy_b;
            else
                src = q_base[j] + (uint64_t)(uint32_t)(kt * BK) * lddy_b;
        } else {
            if (GP)
                src = p_base[j] + (uint64_t)fastdiv(idx_next[j], a.x_div) * ldx_b;
            else
                src = p_base[j] + (uint64_t)(uint32_t)(kt * BK) * ldx_b;
        }
        if constexpr (!FULL.value) {
            if (kt == KT - 1) { // uniform branch: k-rows past the expert's range come from the zero page
                asm volatile("" ::: "memory"); // keeps this rare path a branch
                if (kt * BK + kr_lane + 2 * j >= rows) src = (const char *)zero;
            }
        }
        lds_dma16((const uint16_t *)src, dst);
    };

    f32x16 acc[4][4];
    zero_acc(acc);
    const int wq = (wave & 1) * 128, wp = (wave >> 1) * 128;
    if (KT > 0) {
        // VMEM order per wave: idx(0) | dma(0) idx(1) | dma(1)[0..7] idx(2)? - see below; in the loop the indices of a
        // step are always loaded before a vmcnt(0) that precedes their use.
        const uint32_t lds0 = lds_addr_of(smem);
        FragBase<1> qb, pb;
        make_frag_base<1>(qb, lds0, wq, lane);
        make_frag_base<1>(pb, lds0 + OP_CHUNKS * 16, wp, lane);
        // the operand that is not gathered needs no index: its first step goes out while the indices are on their way
        if (GATHER) load_idx(0);
        if (!GQ) static_for<8>([&](auto P) { issue_piece(0, P, IC<0>{}); });
        if (!GP) static_for<8>([&](auto P) { issue_piece(0, IC<8 + P.value>{}, IC<0>{}); });
        if (GATHER) use_idx();
        if (GQ) static_for<8>([&](auto P) { issue_piece(0, P, IC<0>{}); });
        if (GP) static_for<8>([&](auto P) { issue_piece(0, IC<8 + P.value>{}, IC<0>{}); });
        __builtin_amdgcn_sched_barrier(0);
        if (GATHER) {
            load_idx(1);
            use_idx(); // vmcnt(0): step 0 has landed as well
        }
        static_for<8>([&](auto P) { issue_piece(1, P, IC<0>{}); });
        __builtin_amdgcn_sched_barrier(0);
        // step 0 has landed in every wave; behind it at most the first half of step 1 (none if this is the only step)
        if (KT > 1)
            asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        Frags f0, f1;
        load_frags<1, 1, 0>(f0, pb, qb);
        DW_STAMP(1);
        // one K step; FULL: steps kt + 1 and kt + 2 lie completely inside the expert's rows
        auto k_step = [&](int kt, auto FULL) {
            // idx_next holds the indices of step kt + 1 here; the second half of that step's loads goes out now, then
            // the indices of step kt + 2 are requested (they land before the barrier's vmcnt(0))
            mma_step<T, 1, 1, 1>(f0, f1, pb, qb, acc, [&](auto G) { issue_piece(kt + 1, IC<8 + G.value>{}, FULL); });
            mma_step<T, 1, 1, 2>(f1, f0, pb, qb, acc, [&](auto G) {
                if constexpr (GATHER != 0) load_idx_one(kt + 2, G, FULL);
            });
            mma_step<T, 1, 1, 3>(f0, f1, pb, qb, acc, NoHook());
            XMA_WAIT_LOADS_AND_BARRIER();
            if (GATHER) use_idx();
            flip_stage(pb);
            flip_stage(qb);
            mma_step<T, 1, 1, 0>(f1, f0, pb, qb, acc, [&](auto G) { issue_piece(kt + 2, G, FULL); });
        };
        const int KT_full = rows / BK;
        int kt = 0;
        for (; kt + 2 < KT_full; ++kt) k_step(kt, IC<1>{});
        for (; kt < KT; ++kt) k_step(kt, IC<0>{});
        XMA_WAIT_ALL_LOADS();
        DW_STAMP(2);
    }

    // lane owns DW row o (from the Q tile), 4 consecutive in-features per quad; each 32-row block is staged in a
    // wave-private LDS area and leaves as whole rows (see the forward kernel's epilogue)
    XMA_WAIT_LOADS_AND_BARRIER(); // no wave reads the operand tiles any more
    const int lrow = lane & 31, lhalf = lane >> 5;
    uint16_t *DWe = a.DW + (int64_t)e * a.dw_es;
    unsigned char *stage = smem + wave * EPI_WAVE_BYTES;
    unsigned char *z_w = stage + lrow * EPI_Z_STRIDE + lhalf * 8;
    const unsigned char *z_r = stage + (lane >> 4) * EPI_Z_STRIDE + (lane & 15) * 16;
    const int cz = i0 + wp + (lane & 15) * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int obase = o0 + wq + i * 32;
        if (obase >= a.N_out) break; // wave-uniform
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 v = {Elem<T>::pack(acc[j][i][4 * g], acc[j][i][4 * g + 1]),
                           Elem<T>::pack(acc[j][i][4 * g + 2], acc[j][i][4 * g + 3])};
                *(u32x2 *)(z_w + (j * 32 + g * 8) * 2) = v;
            }
        wave_lds_sync();
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int o = obase + 4 * it + (lane >> 4);
            const u32x4 v = *(const u32x4 *)(z_r + it * 4 * EPI_Z_STRIDE);
            if (o < a.N_out && cz < a.K_in) *(u32x4 *)(DWe + (int64_t)o * a.lddw + cz) = v;
        }
        wave_lds_sync(); // the next block overwrites the area
    }
    DW_STAMP(3);
}

inline int device_cus();
template <typename T, int WT, int EPI> int launch_fwd(const FwdArgs &a, hipStream_t st) {
    int rc;
    const int cus = device_cus();
    // The persistent kernel fetches a row scale as the aligned dword around it and addresses the operands of a tile with
    // 32-bit byte offsets from a uniform base: 256 rows of W or of a grouped X, any row of a gathered X.
    const int64_t x_rows = a.x_grouped ? 256 : (a.M + a.fan_out - 1) / a.fan_out;
    const bool offsets_fit = x_rows * a.ldx * 2 < ((int64_t)1 << 32) && (int64_t)256 * a.ldw * 2 < ((int64_t)1 << 32);
    // The persistent kernel exists for the operand layouts the layer launches: x @ W^T with any epilogue, dy @ W with a
    // plain store or the SwiGLU backward.  (dy @ W with the SwiGLU forward epilogue, reachable through the C ABI only,
    // would be the one instantiation whose register allocation spills inside the K loop.)
    constexpr bool persistent_variant = !(WT == 1 && EPI == XMA_ROCM_EPI_SWIGLU);
    bool persistent = false;
    if constexpr (persistent_variant) {
        if (a.E <= PST_MAX_E && cus > 0 && ((uintptr_t)a.scale & 3) == 0 && offsets_fit) {
            // whole tiles: one persistent workgroup per compute unit
            if ((rc = gemm_set_smem(grouped_gemm_persistent_kernel<T, WT, EPI>, PST_SMEM_BYTES))) return rc;
            const int launch_grid = cus < a.grid_main ? cus : a.grid_main;
            grouped_gemm_persistent_kernel<T, WT, EPI><<<launch_grid, GEMM_THREADS, PST_SMEM_BYTES, st>>>(a);
            if ((rc = xma_check_launch("grouped_gemm_persistent_kernel"))) return rc;
            persistent = true;
        }
    }
    if (!persistent) {
        if ((rc = gemm_set_smem(grouped_gemm_kernel<T, WT, EPI, ROLE_TILES>, GEMM_SMEM_BYTES))) return rc;
        int launch_grid = a.grid_main;
        if (fwd_persistent(EPI, ROLE_TILES) && cus > 0 && cus < launch_grid) launch_grid = cus;
        grouped_gemm_kernel<T, WT, EPI, ROLE_TILES><<<launch_grid, GEMM_THREADS, GEMM_SMEM_BYTES, st>>>(a);
        if ((rc = xma_check_launch("grouped_gemm_kernel"))) return rc;
    }
    if (!a.partial) return XMA_ROCM_OK;
    // the tiles of the last round as K slices (no epilogue: one instantiation serves all), then their sum + epilogue
    if ((rc = gemm_set_smem(grouped_gemm_kernel<T, WT, XMA_ROCM_EPI_STORE, ROLE_SLICES>, GEMM_SMEM_BYTES))) return rc;
    grouped_gemm_kernel<T, WT, XMA_ROCM_EPI_STORE, ROLE_SLICES><<<a.split_cus, GEMM_THREADS, GEMM_SMEM_BYTES, st>>>(a);
    if ((rc = xma_check_launch("grouped_gemm_kernel (K slices)"))) return rc;
    if ((rc = gemm_set_smem(grouped_gemm_fixup_kernel<T, EPI>, GEMM_SMEM_BYTES))) return rc;
    grouped_gemm_fixup_kernel<T, EPI><<<4 * a.split_cus, GEMM_THREADS, GEMM_SMEM_BYTES, st>>>(a);
    return xma_check_launch("grouped_gemm_fixup_kernel");
}

template <typename T, int GQ, int GP> int launch_dw(const DwArgs &a, int grid, hipStream_t st) {
    int rc = gemm_set_smem(grouped_gemm_dw_kernel<T, GQ, GP>, GEMM_SMEM_BYTES);
    if (rc) return rc;
    grouped_gemm_dw_kernel<T, GQ, GP><<<grid, GEMM_THREADS, GEMM_SMEM_BYTES, st>>>(a);
    return xma_check_launch("grouped_gemm_dw_kernel");
}

template <typename T> int dispatch_dw(const DwArgs &a, int grid, hipStream_t st) {
    if (a.dy_grouped) return a.x_grouped ? launch_dw<T, 0, 0>(a, grid, st) : launch_dw<T, 0, 1>(a, grid, st);
    return a.x_grouped ? launch_dw<T, 1, 0>(a, grid, st) : launch_dw<T, 1, 1>(a, grid, st);
}

template <typename T> int dispatch_fwd(const FwdArgs &a, int wt, int epi, hipStream_t st) {
    if (wt == 0) {
        if (epi == XMA_ROCM_EPI_STORE) return launch_fwd<T, 0, XMA_ROCM_EPI_STORE>(a, st);
        if (epi == XMA_ROCM_EPI_SWIGLU) return launch_fwd<T, 0, XMA_ROCM_EPI_SWIGLU>(a, st);
        return launch_fwd<T, 0, XMA_ROCM_EPI_SWIGLU_BWD>(a, st);
    }
    if (epi == XMA_ROCM_EPI_STORE) return launch_fwd<T, 1, XMA_ROCM_EPI_STORE>(a, st);
    if (epi == XMA_ROCM_EPI_SWIGLU) return launch_fwd<T, 1, XMA_ROCM_EPI_SWIGLU>(a, st);
    if (a.aux2) return launch_fwd<T, 1, EPI_SWIGLU_BWD_SCALED_ACT>(a, st);
    return launch_fwd<T, 1, XMA_ROCM_EPI_SWIGLU_BWD>(a, st);
}

// Compute units of the current device (tiles that run at the same time), looked up once per device.
inline int device_cus() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached[dev].store(n, std::memory_order_relaxed); // every thread that races here stores the same value
    }
    return n;
}

// Launches of fewer rounds than this may split the tiles of their last round over the idle CUs.
constexpr int64_t SPLIT_MAX_ROUNDS = 12;

inline size_t fwd_workspace_bytes(int64_t M, int32_t N, int32_t K, int32_t E) {
    const int cus = device_cus();
    if (cus <= 0) return 0;
    // a tile is cut into at least two slices of SPLIT_MIN_STEPS K steps or not at all: short K never splits, and the two
    // launches that would find nothing to do are not made
    if ((K + BK - 1) / BK < 2 * SPLIT_MIN_STEPS) return 0;
    const int64_t tiles = (M / BM + E) * ((N + BN - 1) / BN);
    if (tiles > SPLIT_MAX_ROUNDS * cus) return 0;
    return (size_t)cus * BM * BN * sizeof(float);
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

} // namespace xma_rocm

using namespace xma_rocm;

static int scatter2scatter_impl(const void *X, int64_t ldx, const void *W, int64_t w_expert_stride, int64_t ldw,
                                int w_is_kn, const int64_t *sorted_scattered_idxs, const int64_t *expert_offsets,
                                void *out, int64_t ldo, void *aux, int64_t ldaux, void *aux2, int64_t ldaux2,
                                const void *row_scale, const void *bias, int64_t bias_expert_stride, int64_t M, int32_t N,
                                int32_t K, int32_t E, int32_t fan_out, int x_grouped, int y_grouped, int epilogue, int dtype,
                                void *workspace, size_t workspace_bytes, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED,
                "scatter2scatter: dtype %d", dtype);
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
    XMA_REQUIRE(!aux2 || (epilogue == XMA_ROCM_EPI_SWIGLU_BWD && aligned16(aux2) && ldaux2 % 8 == 0 && ldaux2 >= N),
                XMA_ROCM_EINVAL, "scatter2scatter: scaled activations go with SWIGLU_BWD, 16-byte aligned rows");
    XMA_REQUIRE(!aux2 || (dtype != XMA_ROCM_F32 && w_is_kn), XMA_ROCM_EUNSUPPORTED,
                "scatter2scatter: scaled activations need bf16 / fp16 and W[e] as (K, N) with N contiguous (dy @ W)");
    XMA_REQUIRE(!bias || (aligned16(bias) && bias_expert_stride % 8 == 0 && bias_expert_stride >= 0 &&
                          epilogue != XMA_ROCM_EPI_SWIGLU_BWD),
                XMA_ROCM_EINVAL, "scatter2scatter: bias (E, N) must be 16-byte aligned with an expert stride that is a "
                                 "multiple of 8 elements, and goes with the STORE and SWIGLU epilogues");
    FwdArgs a;
    a.bias = (const uint16_t *)bias;
    a.bias_es = bias_expert_stride;
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
    if (dtype == XMA_ROCM_F32) return f32_scatter2scatter(a, w_is_kn ? 1 : 0, epilogue, (hipStream_t)stream);
    const int64_t NT = (N + BN - 1) / BN;
    const int64_t max_m_tiles = M / BM + E; // sum_e ceil(c_e / BM) <= floor(M / BM) + E
    const int64_t grid = max_m_tiles * NT;
    XMA_REQUIRE(grid < ((int64_t)1 << 30), XMA_ROCM_EUNSUPPORTED, "scatter2scatter: grid too large");
    a.grid_main = (int)grid;
    a.partial = nullptr;
    a.split_cus = 0;
    const size_t ws_need = fwd_workspace_bytes(M, N, K, E);
    if (workspace && ws_need) {
        XMA_REQUIRE(workspace_bytes >= ws_need && aligned16(workspace), XMA_ROCM_EWORKSPACE,
                    "scatter2scatter: workspace of %zu bytes, %zu needed (16-byte aligned)", workspace_bytes, ws_need);
        a.partial = (float *)workspace;
        a.split_cus = device_cus();
    }
    hipStream_t st = (hipStream_t)stream;
    if (dtype == XMA_ROCM_BF16) return dispatch_fwd<__bf16>(a, w_is_kn ? 1 : 0, epilogue, st);
    return dispatch_fwd<_Float16>(a, w_is_kn ? 1 : 0, epilogue, st);
}

extern "C" int xma_rocm_scatter2scatter(const void *X, int64_t ldx, const void *W, int64_t w_expert_stride, int64_t ldw,
                                        int w_is_kn, const int64_t *sorted_scattered_idxs,
                                        const int64_t *expert_offsets, void *out, int64_t ldo, void *aux, int64_t ldaux,
                                        const void *row_scale, int64_t M, int32_t N, int32_t K, int32_t E,
                                        int32_t fan_out, int x_grouped, int y_grouped, int epilogue, int dtype,
                                        void *workspace, size_t workspace_bytes, void *stream) {
    return scatter2scatter_impl(X, ldx, W, w_expert_stride, ldw, w_is_kn, sorted_scattered_idxs, expert_offsets, out, ldo,
                                aux, ldaux, nullptr, 0, row_scale, nullptr, 0, M, N, K, E, fan_out, x_grouped, y_grouped,
                                epilogue, dtype, workspace, workspace_bytes, stream);
}

extern "C" int xma_rocm_scatter2scatter_bias(const void *X, int64_t ldx, const void *W, int64_t w_expert_stride,
                                             int64_t ldw, int w_is_kn, const int64_t *sorted_scattered_idxs,
                                             const int64_t *expert_offsets, void *out, int64_t ldo, void *aux,
                                             int64_t ldaux, const void *row_scale, const void *bias,
                                             int64_t bias_expert_stride, int64_t M, int32_t N, int32_t K, int32_t E,
                                             int32_t fan_out, int x_grouped, int y_grouped, int epilogue, int dtype,
                                             void *workspace, size_t workspace_bytes, void *stream) {
    return scatter2scatter_impl(X, ldx, W, w_expert_stride, ldw, w_is_kn, sorted_scattered_idxs, expert_offsets, out, ldo,
                                aux, ldaux, nullptr, 0, row_scale, bias, bias_expert_stride, M, N, K, E, fan_out, x_grouped,
                                y_grouped, epilogue, dtype, workspace, workspace_bytes, stream);
}

extern "C" int xma_rocm_down_projection_dx_swiglu(const void *dY, int64_t lddy, const void *W, int64_t w_expert_stride,
                                                  int64_t ldw, const int64_t *sorted_scattered_idxs,
                                                  const int64_t *expert_offsets, const void *z, int64_t ldz, void *dz,
                                                  int64_t lddz, void *scaled_act, int64_t ld_scaled_act,
                                                  const void *row_scale, int64_t M, int32_t N, int32_t K, int32_t E,
                                                  int32_t fan_out, int dtype, void *workspace, size_t workspace_bytes,
                                                  void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16, XMA_ROCM_EUNSUPPORTED,
                "down_projection_dx_swiglu: dtype %d (bf16 and fp16 only)", dtype);
    XMA_REQUIRE(row_scale && scaled_act, XMA_ROCM_EINVAL, "down_projection_dx_swiglu: row_scale and scaled_act are required");
    return scatter2scatter_impl(dY, lddy, W, w_expert_stride, ldw, 1, sorted_scattered_idxs, expert_offsets, dz, lddz,
                                const_cast<void *>(z), ldz, scaled_act, ld_scaled_act, row_scale, nullptr, 0, M, N, K, E,
                                fan_out, 0, 1, XMA_ROCM_EPI_SWIGLU_BWD, dtype, workspace, workspace_bytes, stream);
}

#ifdef XMA_PST_TIMING
extern "C" __attribute__((visibility("default"))) int xma_rocm_debug_pst_times(void *host_out) {
    return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(g_pst_times), sizeof(g_pst_times));
}
extern "C" __attribute__((visibility("default"))) int xma_rocm_debug_pst_cycles(void *host_out) {
    return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(g_pst_cycles), sizeof(g_pst_cycles));
}
extern "C" __attribute__((visibility("default"))) int xma_rocm_debug_pst_steps(void *host_out) {
    return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(g_pst_steps), sizeof(g_pst_steps));
}
extern "C" __attribute__((visibility("default"))) int xma_rocm_debug_dw_cycles(void *host_out) {
    return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(g_dw_cycles), sizeof(g_dw_cycles));
}
extern "C" __attribute__((visibility("default"))) int xma_rocm_debug_pst_band(int v) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_pst_band), &v, sizeof(v));
}
extern "C" __attribute__((visibility("default"))) int xma_rocm_debug_pst_no_ovl(int v) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_pst_no_ovl), &v, sizeof(v));
}
extern "C" __attribute__((visibility("default"))) int xma_rocm_debug_pst_reset(void) {
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_pst_times)) != hipSuccess) return -1;
    return (int)hipMemset(p, 0, sizeof(g_pst_times));
}
#endif

extern "C" size_t xma_rocm_scatter2scatter_workspace_bytes(int64_t M, int32_t N, int32_t K, int32_t E) {
    if (M <= 0 || N <= 0 || K <= 0 || E <= 0) return 0;
    return fwd_workspace_bytes(M, N, K, E);
}

extern "C" int xma_rocm_group_bwd_W(const void *DY, int64_t lddy, int dy_grouped, int32_t dy_fan_out,
                                    const void *dy_scale, const void *X, int64_t ldx, int x_grouped, int32_t x_fan_out,
                                    const int64_t *sorted_scattered_idxs, const int64_t *expert_offsets, void *DW,
                                    int64_t dw_expert_stride, int64_t lddw, int32_t N_out, int32_t K_in, int32_t E,
                                    int dtype, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED,
                "group_bwd_W: dtype %d", dtype);
    XMA_REQUIRE(N_out >= 8 && K_in >= 8 && E >= 1 && dy_fan_out >= 1 && x_fan_out >= 1, XMA_ROCM_EINVAL,
                "group_bwd_W: N_out=%d K_in=%d E=%d", N_out, K_in, E);
    XMA_REQUIRE(N_out % 8 == 0 && K_in % 8 == 0 && lddy % 8 == 0 && ldx % 8 == 0 && lddw % 8 == 0 &&
                    dw_expert_stride % 8 == 0,
                XMA_ROCM_EUNSUPPORTED, "group_bwd_W: N_out=%d K_in=%d and leading dimensions must be multiples of 8",
                N_out, K_in);
    XMA_REQUIRE(lddy < ((int64_t)1 << 30) && ldx < ((int64_t)1 << 30) && lddy > 0 && ldx > 0, XMA_ROCM_EUNSUPPORTED,
                "group_bwd_W: leading dimensions must be below 2^30 elements");
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
    a.dy_div = make_fastdiv((uint32_t)dy_fan_out);
    a.x_div = make_fastdiv((uint32_t)x_fan_out);
    if (dtype == XMA_ROCM_F32) return f32_group_bwd_W(a, st);
    if (dy_scale) return launch_dw_scaled(a, dtype, (int)grid, st);
    if (dtype == XMA_ROCM_BF16) return dispatch_dw<__bf16>(a, (int)grid, st);
    return dispatch_dw<_Float16>(a, (int)grid, st);
}
