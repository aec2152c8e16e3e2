// Expert histogram (continuous_count) and the one-op routing (counts, offsets,
// stable expert-major permutation) for gfx950.  HBM-bound integer work: wide
// coalesced loads, LDS-privatised counters, wave64 ballots for stable ranks.
#include "common.hpp"

namespace {

constexpr int HIST_THREADS = 256;
constexpr int HIST_LDS_WORDS = 8192; // 32 KB of counters per workgroup

// ------------------------------------------------------------------------------------------
// continuous_count: LDS histogram replicated `copies` times (copy = thread % copies, odd stride
// so that one bin of all copies spreads over the banks); a hot bin under skewed routing then
// costs at most wave/copies serialised LDS atomics instead of 64.  One global atomic per
// non-empty bin and workgroup at the end.
// ------------------------------------------------------------------------------------------
template <typename IdT>
__device__ __forceinline__ void hist_add(uint32_t *h, IdT id, int bins) {
    if ((uint64_t)id < (uint64_t)bins) atomicAdd(&h[(int)id], 1u);
}

template <typename IdT>
__global__ __launch_bounds__(HIST_THREADS) void histogram_kernel(const IdT *__restrict__ ids, int64_t n,
                                                                 uint32_t *__restrict__ counts, int bins, int copies,
                                                                 int stride) {
    extern __shared__ uint32_t s_hist[];
    const int tid = threadIdx.x;
    for (int i = tid; i < copies * stride; i += HIST_THREADS) s_hist[i] = 0;
    __syncthreads();

    uint32_t *mine = s_hist + (tid % copies) * stride;
    constexpr int VEC = 16 / sizeof(IdT);
    typedef IdT vec_t __attribute__((ext_vector_type(VEC)));

    // elements before the first 16-byte boundary and after the last full vector
    const uintptr_t addr = (uintptr_t)ids;
    int64_t head = ((16 - (addr & 15)) & 15) / sizeof(IdT);
    if (head > n) head = n;
    const int64_t nvec = (n - head) / VEC;
    const int64_t tail_start = head + nvec * VEC;
    const vec_t *vp = (const vec_t *)(ids + head);

    const int64_t gtid = (int64_t)blockIdx.x * HIST_THREADS + tid;
    const int64_t gstride = (int64_t)gridDim.x * HIST_THREADS;
    int64_t i = gtid;
    // two vectors in flight per thread
    for (; i + gstride < nvec; i += 2 * gstride) {
        vec_t a = __builtin_nontemporal_load(vp + i);
        vec_t b = __builtin_nontemporal_load(vp + i + gstride);
#pragma unroll
        for (int j = 0; j < VEC; ++j) hist_add<IdT>(mine, a[j], bins);
#pragma unroll
        for (int j = 0; j < VEC; ++j) hist_add<IdT>(mine, b[j], bins);
    }
    for (; i < nvec; i += gstride) {
        vec_t a = __builtin_nontemporal_load(vp + i);
#pragma unroll
        for (int j = 0; j < VEC; ++j) hist_add<IdT>(mine, a[j], bins);
    }
    if (blockIdx.x == 0) {
        if (tid < head) hist_add<IdT>(mine, ids[tid], bins);
        if (tail_start + tid < n) hist_add<IdT>(mine, ids[tail_start + tid], bins); // tail < VEC <= 4 elements
    }
    __syncthreads();

    for (int b = tid; b < bins; b += HIST_THREADS) {
        uint32_t s = 0;
        for (int c = 0; c < copies; ++c) s += s_hist[c * stride + b];
        if (s) atomicAdd(&counts[b], s);
    }
}

// bins too many for LDS: straight global atomics (not a MoE-sized case)
template <typename IdT>
__global__ __launch_bounds__(HIST_THREADS) void histogram_global_kernel(const IdT *__restrict__ ids, int64_t n,
                                                                        uint32_t *__restrict__ counts, int bins) {
    int64_t i = (int64_t)blockIdx.x * HIST_THREADS + threadIdx.x;
    const int64_t gstride = (int64_t)gridDim.x * HIST_THREADS;
    for (; i < n; i += gstride) {
        IdT id = ids[i];
        if ((uint64_t)id < (uint64_t)bins) atomicAdd(&counts[(int)id], 1u);
    }
}

// ------------------------------------------------------------------------------------------
// route, pass 1: one wave per UNIT consecutive ids -> unit_hist[u][e]
// ------------------------------------------------------------------------------------------
constexpr int ROUTE_THREADS = 256;
constexpr int ROUTE_WAVES = ROUTE_THREADS / WAVE;
constexpr int ROUTE_UNIT = 2048; // ids per wave
constexpr int ROUTE_MAX_E = 2048; // (ROUTE_WAVES + 1) * E counters must fit 64 KB of LDS

template <typename IdT>
__global__ __launch_bounds__(ROUTE_THREADS) void route_unit_hist_kernel(const IdT *__restrict__ ids, int64_t n, int E,
                                                                        uint32_t *__restrict__ unit_hist,
                                                                        int64_t num_units) {
    extern __shared__ uint32_t s_cnt[]; // [ROUTE_WAVES][E]
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    uint32_t *mine = s_cnt + wave * E;
    for (int e = lane; e < E; e += WAVE) mine[e] = 0;
    // a wave's counters are private to it, and a wave's LDS operations execute in order: no barrier needed
    const int64_t unit = (int64_t)blockIdx.x * ROUTE_WAVES + wave;
    if (unit >= num_units) return;
    const int64_t base = unit * ROUTE_UNIT;
#pragma unroll 8
    for (int s = 0; s < ROUTE_UNIT / WAVE; ++s) {
        int64_t i = base + s * WAVE + lane;
        if (i < n) {
            IdT id = ids[i];
            if ((uint64_t)id < (uint64_t)E) atomicAdd(&mine[(int)id], 1u);
        }
    }
    for (int e = lane; e < E; e += WAVE) unit_hist[unit * E + e] = mine[e];
}

// ------------------------------------------------------------------------------------------
// route, pass 2: block e turns column e of unit_hist into exclusive prefixes over units and
// writes counts[e]
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(ROUTE_THREADS) void route_scan_kernel(uint32_t *__restrict__ unit_hist, int64_t num_units,
                                                                   int E, uint32_t *__restrict__ counts) {
    __shared__ uint32_t s_part[ROUTE_THREADS];
    const int e = blockIdx.x, tid = threadIdx.x;
    const int64_t per = (num_units + ROUTE_THREADS - 1) / ROUTE_THREADS;
    const int64_t u0 = tid * per, u1 = (u0 + per < num_units) ? u0 + per : num_units;
    uint32_t sum = 0;
    for (int64_t u = u0; u < u1; ++u) sum += unit_hist[u * E + e];
    s_part[tid] = sum;
    __syncthreads();
    // Hillis-Steele inclusive scan over the 256 partial sums
    for (int d = 1; d < ROUTE_THREADS; d <<= 1) {
        uint32_t v = (tid >= d) ? s_part[tid - d] : 0;
        __syncthreads();
        s_part[tid] += v;
        __syncthreads();
    }
    uint32_t run = s_part[tid] - sum; // exclusive prefix of this thread's range
    for (int64_t u = u0; u < u1; ++u) {
        uint32_t c = unit_hist[u * E + e];
        unit_hist[u * E + e] = run;
        run += c;
    }
    if (tid == ROUTE_THREADS - 1) counts[e] = s_part[tid];
}

// ------------------------------------------------------------------------------------------
// route, pass 3: stable scatter.  Each wave walks its unit in order, 64 ids per step.  For a
// step, `peers` = lanes holding the same id (nbits ballots), rank = peers below me, and the
// running counter of the id (wave-private LDS, seeded with the global start of this unit's
// run for that expert) gives the destination.
// ------------------------------------------------------------------------------------------
template <typename IdT>
__global__ __launch_bounds__(ROUTE_THREADS) void route_scatter_kernel(
    const IdT *__restrict__ ids, int64_t n, int E, int nbits, const uint32_t *__restrict__ unit_base,
    const uint32_t *__restrict__ counts, int64_t num_units, int64_t *__restrict__ offs_incl,
    int64_t *__restrict__ offs_excl, IdT *__restrict__ sorted_ids, int64_t *__restrict__ sorted_pos) {
    extern __shared__ uint32_t s_mem[]; // [E] exclusive offsets, then [ROUTE_WAVES][E] running counters
    uint32_t *s_excl = s_mem;
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;

    // exclusive scan of counts over experts (E <= 2048), wave 0, 64 experts per step
    if (wave == 0) {
        uint32_t carry = 0;
        for (int b = 0; b < E; b += WAVE) {
            int e = b + lane;
            uint32_t v = (e < E) ? counts[e] : 0, s = v;
#pragma unroll
            for (int d = 1; d < WAVE; d <<= 1) {
                uint32_t t = __shfl_up(s, d);
                if (lane >= d) s += t;
            }
            if (e < E) {
                s_excl[e] = carry + s - v;
                if (blockIdx.x == 0) {
                    offs_incl[e] = (int64_t)(carry + s);
                    if (offs_excl) offs_excl[e] = (int64_t)(carry + s - v);
                }
            }
            carry += __shfl(s, WAVE - 1);
        }
    }
    __syncthreads();

    const int64_t unit = (int64_t)blockIdx.x * ROUTE_WAVES + wave;
    if (unit >= num_units) return;
    uint32_t *ctr = s_mem + E + wave * E;
    for (int e = lane; e < E; e += WAVE) ctr[e] = s_excl[e] + unit_base[unit * E + e];

    const int64_t base = unit * ROUTE_UNIT;
    const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int s = 0; s < ROUTE_UNIT / WAVE; ++s) {
        const int64_t i = base + s * WAVE + lane;
        if (base + s * WAVE >= n) break; // wave-uniform
        const bool live = i < n;
        const IdT id = live ? ids[i] : (IdT)0;
        const bool ok = live && (uint64_t)id < (uint64_t)E;
        const uint32_t key = ok ? (uint32_t)id : 0u;
        uint64_t peers = __ballot(ok);
        for (int b = 0; b < nbits; ++b) {
            const uint64_t set = __ballot((key >> b) & 1u);
            peers &= ((key >> b) & 1u) ? set : ~set;
        }
        if (ok) {
            const uint32_t rank = __popcll(peers & below);
            const uint32_t start = ctr[key];
            const uint32_t pos = start + rank;
            // the highest peer advances the counter after every peer has read it
            if ((peers >> lane) == 1ull) ctr[key] = start + (uint32_t)__popcll(peers);
            sorted_pos[pos] = i;
            if (sorted_ids) sorted_ids[pos] = id;
        }
    }
}

int hist_launch(const void *ids, int is64, int64_t n, uint32_t *counts, int bins, hipStream_t st) {
    if (n == 0) return XMA_ROCM_OK;
    const int elems_per_block = HIST_THREADS * 16;
    int64_t blocks = (n + elems_per_block - 1) / elems_per_block;
    if (blocks > 1024) blocks = 1024;
    if (bins > HIST_LDS_WORDS) {
        if (is64)
            histogram_global_kernel<int64_t><<<(int)blocks, HIST_THREADS, 0, st>>>((const int64_t *)ids, n, counts, bins);
        else
            histogram_global_kernel<int32_t><<<(int)blocks, HIST_THREADS, 0, st>>>((const int32_t *)ids, n, counts, bins);
        return xma_check_launch("histogram_global_kernel");
    }
    const int stride = bins | 1;
    int copies = 1;
    while (copies < 32 && (copies * 2) * stride <= HIST_LDS_WORDS) copies *= 2;
    const size_t lds = (size_t)copies * stride * sizeof(uint32_t);
    if (is64)
        histogram_kernel<int64_t>
            <<<(int)blocks, HIST_THREADS, lds, st>>>((const int64_t *)ids, n, counts, bins, copies, stride);
    else
        histogram_kernel<int32_t>
            <<<(int)blocks, HIST_THREADS, lds, st>>>((const int32_t *)ids, n, counts, bins, copies, stride);
    return xma_check_launch("histogram_kernel");
}

} // namespace

extern "C" int xma_rocm_continuous_count(const void *ids, int ids_are_int64, int64_t n, uint32_t *counts, int32_t bins,
                                         void *stream) {
    XMA_REQUIRE(n >= 0 && bins >= 1, XMA_ROCM_EINVAL, "continuous_count: n=%lld bins=%d", (long long)n, bins);
    XMA_REQUIRE(counts != nullptr && (ids != nullptr || n == 0), XMA_ROCM_EINVAL, "continuous_count: null pointer");
    XMA_REQUIRE(((uintptr_t)ids % (ids_are_int64 ? 8 : 4)) == 0, XMA_ROCM_EINVAL, "continuous_count: misaligned ids");
    return hist_launch(ids, ids_are_int64, n, counts, bins, (hipStream_t)stream);
}

extern "C" size_t xma_rocm_route_workspace_bytes(int64_t n, int32_t num_experts) {
    if (n < 0 || num_experts < 1) return 0;
    int64_t units = (n + ROUTE_UNIT - 1) / ROUTE_UNIT;
    if (units < 1) units = 1;
    return (size_t)units * (size_t)num_experts * sizeof(uint32_t);
}

extern "C" int xma_rocm_route(const void *ids, int ids_are_int64, int64_t n, int32_t E, uint32_t *counts,
                              int64_t *offsets_inclusive, int64_t *offsets_exclusive, void *sorted_expert_idxs,
                              int64_t *sorted_scattered_idxs, void *workspace, size_t workspace_bytes, void *stream) {
    XMA_REQUIRE(n >= 0 && E >= 1 && E <= ROUTE_MAX_E, XMA_ROCM_EINVAL, "route: n=%lld E=%d (E <= %d)", (long long)n, E,
                ROUTE_MAX_E);
    XMA_REQUIRE(n < (int64_t)1 << 31, XMA_ROCM_EUNSUPPORTED, "route: n=%lld does not fit 31 bits", (long long)n);
    XMA_REQUIRE(counts && offsets_inclusive && workspace && (n == 0 || (ids && sorted_scattered_idxs)),
                XMA_ROCM_EINVAL, "route: null pointer");
    XMA_REQUIRE(workspace_bytes >= xma_rocm_route_workspace_bytes(n, E), XMA_ROCM_EWORKSPACE,
                "route: workspace %zu < %zu bytes", workspace_bytes, xma_rocm_route_workspace_bytes(n, E));
    hipStream_t st = (hipStream_t)stream;
    int64_t units = (n + ROUTE_UNIT - 1) / ROUTE_UNIT;
    if (units < 1) units = 1;
    const int blocks = (int)((units + ROUTE_WAVES - 1) / ROUTE_WAVES);
    uint32_t *unit_hist = (uint32_t *)workspace;
    int nbits = 0;
    while ((1 << nbits) < E) ++nbits;
    const size_t lds1 = (size_t)ROUTE_WAVES * E * sizeof(uint32_t);
    const size_t lds3 = (size_t)(ROUTE_WAVES + 1) * E * sizeof(uint32_t);
    int rc;
    if (ids_are_int64) {
        route_unit_hist_kernel<int64_t><<<blocks, ROUTE_THREADS, lds1, st>>>((const int64_t *)ids, n, E, unit_hist, units);
        if ((rc = xma_check_launch("route_unit_hist_kernel"))) return rc;
        route_scan_kernel<<<E, ROUTE_THREADS, 0, st>>>(unit_hist, units, E, counts);
        if ((rc = xma_check_launch("route_scan_kernel"))) return rc;
        route_scatter_kernel<int64_t><<<blocks, ROUTE_THREADS, lds3, st>>>(
            (const int64_t *)ids, n, E, nbits, unit_hist, counts, units, offsets_inclusive, offsets_exclusive,
            (int64_t *)sorted_expert_idxs, sorted_scattered_idxs);
        return xma_check_launch("route_scatter_kernel");
    }
    route_unit_hist_kernel<int32_t><<<blocks, ROUTE_THREADS, lds1, st>>>((const int32_t *)ids, n, E, unit_hist, units);
    if ((rc = xma_check_launch("route_unit_hist_kernel"))) return rc;
    route_scan_kernel<<<E, ROUTE_THREADS, 0, st>>>(unit_hist, units, E, counts);
    if ((rc = xma_check_launch("route_scan_kernel"))) return rc;
    route_scatter_kernel<int32_t><<<blocks, ROUTE_THREADS, lds3, st>>>(
        (const int32_t *)ids, n, E, nbits, unit_hist, counts, units, offsets_inclusive, offsets_exclusive,
        (int32_t *)sorted_expert_idxs, sorted_scattered_idxs);
    return xma_check_launch("route_scatter_kernel");
}
