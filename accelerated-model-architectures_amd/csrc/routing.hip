// Expert histogram (continuous_count) and the one-op routing (counts, offsets, stable expert-major permutation) for
// gfx950.  HBM-bound integer work: wide coalesced loads, LDS-privatised counters, wave64 ballots for stable ranks,
// LDS-staged output so that the scatter leaves the workgroup as contiguous runs.
#include <atomic>
#include <mutex>

#include "common.hpp"

namespace xma_rocm {

// Scratch of xma_rocm_route_static: the per-unit histograms live in this file-scope device array instead of a caller's
// workspace, so that entry point allocates nothing.  Every GPU the library runs on holds its own copy at its own address
// until the process ends; in host code the name is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t ROUTE_STATIC_WORDS = (size_t)1 << 18; // 1 MiB: units x experts <= 262144
static __device__ __align__(256) uint32_t scratch[ROUTE_STATIC_WORDS];

constexpr int HIST_THREADS = 512;
constexpr int HIST_LDS_WORDS = 8192;  // 32 KB of counters per workgroup
constexpr int HIST_MAX_UNITS = 2048;  // partial histograms of the two-pass path
constexpr int64_t HIST_TWO_PASS_MIN = 1 << 16;
constexpr int UNIT_IDS = 4096;        // ids per workgroup of the unit histogram and of the routing scatter

// ------------------------------------------------------------------------------------------------
// Histograms.  LDS histogram replicated `copies` times (copy = thread % copies, odd stride so that one bin of all
// copies spreads over the banks): a hot bin under skewed routing costs at most wave / copies serialised LDS atomics
// instead of 64.  Thousands of device-scope atomics on the same 64 addresses serialise (measured: 23 us for 4 Mi ids
// against 3 us of HBM time), so large inputs go through per-unit histograms that a second kernel adds up.
// ------------------------------------------------------------------------------------------------
template <typename IdT> __device__ __forceinline__ void hist_add(uint32_t *h, IdT id, int bins) {
    if ((uint64_t)id < (uint64_t)bins) atomicAdd(&h[(int)id], 1u);
}

// LDS histogram of ids[begin, end) by one workgroup of NT threads: 16-byte loads, UNROLL of them in flight per thread
// (for a unit of 4096 ids that is the whole unit at once: the kernels that call this are a single dependent chain of
// load -> count -> store, so their duration is the latency of that chain, not bandwidth), scalar loads for the few
// elements in front of and behind the aligned middle.  `zero_and_sync` runs between the issue of the first batch of
// loads and its use: the caller clears its counters there, behind the loads instead of in front of them.
template <typename IdT, int NT, int UNROLL, typename ZeroAndSync>
__device__ __forceinline__ void block_histogram(const IdT *__restrict__ ids, int64_t begin, int64_t end, uint32_t *mine,
                                                int bins, int tid, ZeroAndSync zero_and_sync) {
    constexpr int VEC = 16 / sizeof(IdT);
    typedef IdT vec_t __attribute__((ext_vector_type(VEC)));
    if (begin >= end) { // uniform
        zero_and_sync();
        return;
    }
    const uintptr_t addr = (uintptr_t)(ids + begin);
    int64_t head = ((16 - (addr & 15)) & 15) / sizeof(IdT);
    if (head > end - begin) head = end - begin;
    const int64_t nvec = (end - begin - head) / VEC;
    const int64_t tail_start = begin + head + nvec * VEC;
    const vec_t *vp = (const vec_t *)(ids + begin + head);
    vec_t v[UNROLL];
    auto fetch = [&](int64_t i0) {
#pragma unroll
        for (int q = 0; q < UNROLL; ++q) {
            const int64_t i = i0 + q * NT;
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[q][j] = (IdT)-1; // out of range: not counted
            if (i < nvec) v[q] = __builtin_nontemporal_load(vp + i);
        }
    };
    auto count = [&]() {
#pragma unroll
        for (int q = 0; q < UNROLL; ++q)
#pragma unroll
            for (int j = 0; j < VEC; ++j) hist_add<IdT>(mine, v[q][j], bins);
    };
    fetch(tid);
    IdT edge0 = (IdT)-1, edge1 = (IdT)-1;
    if (tid < head) edge0 = ids[begin + tid];
    if (tail_start + tid < end) edge1 = ids[tail_start + tid]; // fewer than VEC <= 4 elements
    zero_and_sync();
    count();
    hist_add<IdT>(mine, edge0, bins);
    hist_add<IdT>(mine, edge1, bins);
    for (int64_t i0 = tid + (int64_t)UNROLL * NT; i0 < nvec; i0 += (int64_t)UNROLL * NT) {
        fetch(i0);
        count();
    }
}

// One workgroup per contiguous chunk of `chunk` ids (a multiple of 16, so every chunk keeps the alignment of the first).
//   TABLE = 0: the histogram is added to out[bins] with one global atomic per non-empty bin (small inputs);
//   TABLE = 1: it is stored to column blockIdx.x of out[bins][gridDim.x] - bin-major, so that the kernel that follows
//              (histogram_reduce_kernel, route_scan_kernel) reads every bin's row of per-unit counts coalesced.
template <typename IdT, int TABLE>
__global__ __launch_bounds__(HIST_THREADS) void histogram_kernel(const IdT *__restrict__ ids, int64_t n, int64_t chunk,
                                                                 uint32_t *__restrict__ out, int bins, int copies,
                                                                 int stride) {
    extern __shared__ uint32_t s_hist[];
    const int tid = threadIdx.x;
    const int64_t begin = (int64_t)blockIdx.x * chunk;
    const int64_t end = (begin + chunk < n) ? begin + chunk : n;
    block_histogram<IdT, HIST_THREADS, 4>(ids, begin, end, s_hist + (tid % copies) * stride, bins, tid, [&]() {
        for (int i = tid; i < copies * stride; i += HIST_THREADS) s_hist[i] = 0;
        __syncthreads();
    });
    __syncthreads();
    for (int b = tid; b < bins; b += HIST_THREADS) {
        uint32_t s = 0;
        for (int c = 0; c < copies; ++c) s += s_hist[c * stride + b];
        if (TABLE)
            out[(int64_t)b * gridDim.x + blockIdx.x] = s;
        else if (s)
            atomicAdd(&out[b], s);
    }
}

// counts[b] (+)= sum of row b of table[bins][units]; one workgroup per bin, four independent loads in flight per thread.
// ACCUMULATE = 0 overwrites counts, so the caller need not clear them.
template <int ACCUMULATE>
__global__ __launch_bounds__(256) void histogram_reduce_kernel(const uint32_t *__restrict__ table, int units, int bins,
                                                               uint32_t *__restrict__ counts) {
    __shared__ uint32_t s_part[256 / WAVE];
    const int tid = threadIdx.x, b = blockIdx.x;
    const uint32_t *row = table + (int64_t)b * units;
    uint32_t s = 0;
    int u = tid;
    for (; u + 3 * 256 < units; u += 4 * 256) s += (row[u] + row[u + 256]) + (row[u + 512] + row[u + 768]);
    for (; u < units; u += 256) s += row[u];
#pragma unroll
    for (int d = WAVE / 2; d > 0; d >>= 1) s += __shfl_xor(s, d);
    if (tid % WAVE == 0) s_part[tid / WAVE] = s;
    __syncthreads();
    if (tid == 0) counts[b] = (ACCUMULATE ? counts[b] : 0u) + s_part[0] + s_part[1] + s_part[2] + s_part[3];
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

// ------------------------------------------------------------------------------------------------
// route: a unit is the ROUTE_CHUNK consecutive ids of one workgroup (8 waves x 512).
//   pass 1  histogram_kernel<., 1>: unit_hist[e][u]  (LDS atomics; bin-major table)
//   pass 2  block e: exclusive prefix over the units of row e (in place) and counts[e]
//   pass 3  per unit: per-wave counts -> local offsets; stable rank of every id inside its wave (64 ids per step, from
//           returning LDS atomic adds on wave-private counters or from ballots, see route_scatter_kernel); the unit is
//           sorted into LDS and leaves as one contiguous run per expert.
// ------------------------------------------------------------------------------------------------
constexpr int ROUTE_THREADS = 512;
constexpr int ROUTE_WAVES = ROUTE_THREADS / WAVE;
constexpr int ROUTE_WAVE_IDS = 512;
constexpr int ROUTE_STEPS = ROUTE_WAVE_IDS / WAVE;          // 8 ids per lane
constexpr int ROUTE_CHUNK = ROUTE_WAVES * ROUTE_WAVE_IDS;   // 4096 ids per workgroup
constexpr int ROUTE_MAX_E = 2048;
static_assert(ROUTE_CHUNK == UNIT_IDS && ROUTE_THREADS == HIST_THREADS, "pass 1 of route is histogram_kernel<., 1>");

// inclusive scan of one value per thread over the workgroup: wave scans by shuffles, then the wave totals
__device__ __forceinline__ uint32_t block_inclusive_scan(uint32_t v, uint32_t *s_wave /* [ROUTE_WAVES] */, int tid) {
    const int lane = tid % WAVE, wave = tid / WAVE;
    uint32_t s = v;
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
        const uint32_t t = __shfl_up(s, d);
        if (lane >= d) s += t;
    }
    if (lane == WAVE - 1) s_wave[wave] = s;
    __syncthreads();
    uint32_t before = 0;
#pragma unroll
    for (int w = 0; w < ROUTE_WAVES; ++w)
        if (w < wave) before += s_wave[w];
    return s + before;
}

// block e: exclusive prefix over the units of row e of unit_hist[E][units] (in place) and counts[e]; a thread takes
// `per` consecutive units, so a wave reads and writes a contiguous stretch of the row
__global__ __launch_bounds__(ROUTE_THREADS) void route_scan_kernel(uint32_t *__restrict__ unit_hist, int units,
                                                                   uint32_t *__restrict__ counts) {
    __shared__ uint32_t s_wave[ROUTE_WAVES];
    const int e = blockIdx.x, tid = threadIdx.x;
    uint32_t *row = unit_hist + (int64_t)e * units;
    if (units <= 4 * ROUTE_THREADS) { // up to 4 units per thread, held in registers between the two passes
        const int per = (units + ROUTE_THREADS - 1) / ROUTE_THREADS;
        uint32_t c[4], sum = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int u = tid * per + q;
            c[q] = (q < per && u < units) ? row[u] : 0u;
            sum += c[q];
        }
        const uint32_t incl = block_inclusive_scan(sum, s_wave, tid);
        uint32_t run = incl - sum;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int u = tid * per + q;
            if (q < per && u < units) row[u] = run;
            run += c[q];
        }
        if (tid == ROUTE_THREADS - 1) counts[e] = incl;
        return;
    }
    const int per = (units + ROUTE_THREADS - 1) / ROUTE_THREADS;
    const int u0 = tid * per, u1 = (u0 + per < units) ? u0 + per : units;
    uint32_t sum = 0;
    for (int u = u0; u < u1; ++u) sum += row[u];
    const uint32_t incl = block_inclusive_scan(sum, s_wave, tid);
    uint32_t run = incl - sum; // exclusive prefix of this thread's range
    for (int u = u0; u < u1; ++u) {
        const uint32_t c = row[u];
        row[u] = run;
        run += c;
    }
    if (tid == ROUTE_THREADS - 1) counts[e] = incl;
}

// SINGLE = 1: the whole problem is one unit (n <= ROUTE_CHUNK, the few-token regime) and this kernel is the whole call:
// the local sorted order is the global one, and the counts and offsets come out of the per-wave counters (no unit
// histogram, no scan kernel; unit_base is not read and counts is written instead).
template <typename IdT, int BALLOT, int SINGLE>
__global__ __launch_bounds__(ROUTE_THREADS) void route_scatter_kernel(
    const IdT *__restrict__ ids, int64_t n, int E, int nbits, const uint32_t *__restrict__ unit_base,
    uint32_t *__restrict__ counts, int64_t *__restrict__ offs_incl, int64_t *__restrict__ offs_excl,
    IdT *__restrict__ sorted_ids, int64_t *__restrict__ sorted_pos) {
    // LDS: [E] global start of each expert's local run minus its local start, [WAVES][E] per-wave counters,
    //      [256] scan scratch, then the staged unit: local index and expert id of every sorted position
    extern __shared__ uint32_t s_mem[];
    uint32_t *s_gbase = s_mem;
    uint32_t *s_ctr = s_mem + E;
    uint32_t *s_scan = s_ctr + ROUTE_WAVES * E;
    uint16_t *s_idx = (uint16_t *)(s_scan + ROUTE_THREADS);
    uint16_t *s_exp = s_idx + ROUTE_CHUNK;
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int64_t base = (int64_t)blockIdx.x * ROUTE_CHUNK;
    const int units = gridDim.x;

    // this wave's ids into registers; the loads go out first, the set-up below runs while they are on their way
    IdT raw[ROUTE_STEPS];
    const int64_t wbase = base + wave * ROUTE_WAVE_IDS;
#pragma unroll
    for (int s = 0; s < ROUTE_STEPS; ++s) {
        const int64_t i = wbase + s * WAVE + lane;
        raw[s] = (IdT)-1;
        if (i < n) raw[s] = __builtin_nontemporal_load(ids + i);
    }

    // global exclusive scan of counts over experts (wave 0, 64 experts per step) -> s_gbase; block 0 writes the offsets
    if (SINGLE == 0 && wave == 0) {
        uint32_t carry = 0;
        for (int b = 0; b < E; b += WAVE) {
            const int e = b + lane;
            const uint32_t v = (e < E) ? counts[e] : 0;
            const uint32_t ub = (e < E) ? unit_base[(int64_t)e * units + blockIdx.x] : 0;
            uint32_t s = v;
#pragma unroll
            for (int d = 1; d < WAVE; d <<= 1) {
                const uint32_t t = __shfl_up(s, d);
                if (lane >= d) s += t;
            }
            if (e < E) {
                s_gbase[e] = carry + s - v + ub;
                if (blockIdx.x == 0) {
                    offs_incl[e] = (int64_t)(carry + s);
                    if (offs_excl) offs_excl[e] = (int64_t)(carry + s - v);
                }
            }
            carry += __shfl(s, WAVE - 1);
        }
    }
    for (int i = tid; i < ROUTE_WAVES * E; i += ROUTE_THREADS) s_ctr[i] = 0;
    __syncthreads();

    // phase 1: per-wave counts
    uint32_t key[ROUTE_STEPS];
#pragma unroll
    for (int s = 0; s < ROUTE_STEPS; ++s) key[s] = ((uint64_t)raw[s] < (uint64_t)E) ? (uint32_t)raw[s] : 0xffffffffu;
    uint32_t *my_ctr = s_ctr + wave * E;
    // BALLOT = 0, counting and ranking in one pass: ds_add_rtn_u32 applies the lanes of one wave instruction that hit the
    // same address in lane order, and a wave's LDS instructions execute in program order, so the value returned from the
    // wave-private counter is the stable rank of the id among the wave's ids of the same expert, and the counter ends up
    // as their number.  The lane order is what gfx950 does, not something its ISA manual promises; BALLOT = 1 derives the
    // ranks from log2(E) ballots per step instead and relies on nothing of the kind.  Both are compiled, the host picks
    // one (xma_rocm_route_set_rank_method), and the routing tests require bit-equal results from both.
    uint32_t rank[ROUTE_STEPS];
#pragma unroll
    for (int s = 0; s < ROUTE_STEPS; ++s) {
        rank[s] = 0;
        if (key[s] != 0xffffffffu) rank[s] = atomicAdd(&my_ctr[key[s]], 1u);
    }
    __syncthreads();

    // phase 2: local start of every (wave, expert) run: experts major, waves minor.  Thread t owns experts
    // [t * per, (t + 1) * per).
    const int per = (E + ROUTE_THREADS - 1) / ROUTE_THREADS;
    const int e0 = tid * per, e1 = (e0 + per < E) ? e0 + per : E;
    uint32_t mine = 0;
    for (int e = e0; e < e1; ++e)
        for (int w = 0; w < ROUTE_WAVES; ++w) mine += s_ctr[w * E + e];
    const uint32_t incl = block_inclusive_scan(mine, s_scan, tid);
    if (tid == ROUTE_THREADS - 1) s_scan[ROUTE_WAVES] = incl;
    uint32_t run = incl - mine;
    for (int e = e0; e < e1; ++e) {
        const uint32_t start = run;
        for (int w = 0; w < ROUTE_WAVES; ++w) {
            const uint32_t c = s_ctr[w * E + e];
            s_ctr[w * E + e] = run;
            run += c;
        }
        if constexpr (SINGLE != 0) {
            s_gbase[e] = 0; // local sorted position = global sorted position
            counts[e] = run - start;
            offs_incl[e] = (int64_t)run;
            if (offs_excl) offs_excl[e] = (int64_t)start;
        } else {
            s_gbase[e] -= start; // destination of local sorted position j of expert e = s_gbase[e] + j
        }
    }
    __syncthreads();
    const uint32_t total = s_scan[ROUTE_WAVES]; // ids of this unit that are in range

    // phase 3: the unit sorted into LDS: local position = start of the (wave, expert) run + rank
    if constexpr (BALLOT == 0) {
#pragma unroll
        for (int s = 0; s < ROUTE_STEPS; ++s) {
            if (key[s] != 0xffffffffu) {
                const uint32_t pos = my_ctr[key[s]] + rank[s];
                s_idx[pos] = (uint16_t)(wave * ROUTE_WAVE_IDS + s * WAVE + lane);
                s_exp[pos] = (uint16_t)key[s];
            }
        }
    } else {
        const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
        for (int s = 0; s < ROUTE_STEPS; ++s) {
            const bool ok = key[s] != 0xffffffffu;
            const uint32_t k = ok ? key[s] : 0u;
            uint64_t peers = __ballot(ok);
            for (int b = 0; b < nbits; ++b) {
                const uint64_t set = __ballot((k >> b) & 1u);
                peers &= ((k >> b) & 1u) ? set : ~set;
            }
            if (ok) {
                const uint32_t start = my_ctr[k];
                const uint32_t pos = start + (uint32_t)__popcll(peers & below);
                // the highest peer advances the counter after every peer has read it (a wave's LDS operations are in order)
                if ((peers >> lane) == 1ull) my_ctr[k] = start + (uint32_t)__popcll(peers);
                s_idx[pos] = (uint16_t)(wave * ROUTE_WAVE_IDS + s * WAVE + lane);
                s_exp[pos] = (uint16_t)k;
            }
        }
    }
    __syncthreads();

    // phase 4: contiguous runs out
    for (uint32_t j = tid; j < total; j += ROUTE_THREADS) {
        const uint32_t e = s_exp[j];
        const uint32_t g = s_gbase[e] + j;
        sorted_pos[g] = base + s_idx[j];
        if (sorted_ids) sorted_ids[g] = (IdT)e;
    }
}

// 0: ranks from the lane order of same-address LDS atomics, 1: ranks from ballots (xma_rocm_route_set_rank_method)
static std::atomic<int> g_route_rank_method{0};

inline size_t route_scatter_lds(int E) {
    return (size_t)(E + ROUTE_WAVES * E + ROUTE_THREADS) * sizeof(uint32_t) + (size_t)2 * ROUTE_CHUNK * sizeof(uint16_t);
}

inline void hist_lds_layout(int bins, int &copies, int &stride) {
    stride = bins | 1;
    copies = 1;
    while (copies < 32 && (copies * 2) * stride <= HIST_LDS_WORDS) copies *= 2;
}

template <typename IdT>
int route_launch(const IdT *ids, int64_t n, int E, uint32_t *counts, int64_t *incl, int64_t *excl, IdT *sorted_ids,
                 int64_t *sorted_pos, uint32_t *unit_hist, hipStream_t st) {
    int64_t units = (n + ROUTE_CHUNK - 1) / ROUTE_CHUNK;
    if (units < 1) units = 1;
    int nbits = 0;
    while ((1 << nbits) < E) ++nbits;
    const size_t lds3 = route_scatter_lds(E);
    const bool ballot = g_route_rank_method.load(std::memory_order_relaxed) == 1;
    // both size classes get their LDS limit on the first call, whatever its size: a caller that warms up with one size
    // and captures another into a graph makes no attribute call under capture
    const void *single = ballot ? (const void *)route_scatter_kernel<IdT, 1, 1> : (const void *)route_scatter_kernel<IdT, 0, 1>;
    const void *scatter = ballot ? (const void *)route_scatter_kernel<IdT, 1, 0> : (const void *)route_scatter_kernel<IdT, 0, 0>;
    if (xma_set_max_lds_once(single, (int)route_scatter_lds(ROUTE_MAX_E))) return XMA_ROCM_ELAUNCH;
    if (xma_set_max_lds_once(scatter, (int)route_scatter_lds(ROUTE_MAX_E))) return XMA_ROCM_ELAUNCH;
    if (units == 1) { // a single unit: one kernel counts, scans and sorts
        if (ballot)
            route_scatter_kernel<IdT, 1, 1><<<1, ROUTE_THREADS, lds3, st>>>(ids, n, E, nbits, nullptr, counts, incl, excl, sorted_ids, sorted_pos);
        else
            route_scatter_kernel<IdT, 0, 1><<<1, ROUTE_THREADS, lds3, st>>>(ids, n, E, nbits, nullptr, counts, incl, excl, sorted_ids, sorted_pos);
        return xma_check_launch("route_scatter_kernel (single unit)");
    }
    int rc, copies, stride;
    hist_lds_layout(E, copies, stride);
    histogram_kernel<IdT, 1><<<(int)units, HIST_THREADS, (size_t)copies * stride * sizeof(uint32_t), st>>>(
        ids, n, ROUTE_CHUNK, unit_hist, E, copies, stride);
    if ((rc = xma_check_launch("histogram_kernel (route)"))) return rc;
    route_scan_kernel<<<E, ROUTE_THREADS, 0, st>>>(unit_hist, (int)units, counts);
    if ((rc = xma_check_launch("route_scan_kernel"))) return rc;
    if (ballot)
        route_scatter_kernel<IdT, 1, 0><<<(int)units, ROUTE_THREADS, lds3, st>>>(ids, n, E, nbits, unit_hist, counts, incl,
                                                                                 excl, sorted_ids, sorted_pos);
    else
        route_scatter_kernel<IdT, 0, 0><<<(int)units, ROUTE_THREADS, lds3, st>>>(ids, n, E, nbits, unit_hist, counts, incl,
                                                                                 excl, sorted_ids, sorted_pos);
    return xma_check_launch("route_scatter_kernel");
}

// chunk of ids per workgroup and number of workgroups of the two-pass histogram
inline void hist_units(int64_t n, int64_t &chunk, int64_t &units) {
    chunk = UNIT_IDS;
    if ((n + chunk - 1) / chunk > HIST_MAX_UNITS) {
        chunk = (n + HIST_MAX_UNITS - 1) / HIST_MAX_UNITS;
        chunk = (chunk + UNIT_IDS - 1) / UNIT_IDS * UNIT_IDS;
    }
    units = (n + chunk - 1) / chunk;
}

template <typename IdT>
int hist_launch_t(const IdT *ids, int64_t n, uint32_t *counts, int bins, uint32_t *table, size_t table_bytes,
                  hipStream_t st, bool overwrite = false) {
    if (overwrite) {
        // counts are written, not added to: per-unit histograms and a reduction that stores its sums.  A single unit's
        // histogram is the result itself (a table of one column is the counts vector).
        int copies, stride;
        hist_lds_layout(bins, copies, stride);
        int64_t chunk, units;
        hist_units(n, chunk, units);
        if (units < 1) units = 1;
        const size_t lds = (size_t)copies * stride * sizeof(uint32_t);
        if (units == 1) {
            histogram_kernel<IdT, 1><<<1, HIST_THREADS, lds, st>>>(ids, n, chunk, counts, bins, copies, stride);
            return xma_check_launch("histogram_kernel");
        }
        histogram_kernel<IdT, 1><<<(int)units, HIST_THREADS, lds, st>>>(ids, n, chunk, table, bins, copies, stride);
        int rc = xma_check_launch("histogram_kernel");
        if (rc) return rc;
        histogram_reduce_kernel<0><<<bins, 256, 0, st>>>(table, (int)units, bins, counts);
        return xma_check_launch("histogram_reduce_kernel");
    }
    if (bins > HIST_LDS_WORDS) {
        int64_t blocks = (n + HIST_THREADS * 16 - 1) / (HIST_THREADS * 16);
        if (blocks > 2048) blocks = 2048;
        histogram_global_kernel<IdT><<<(int)blocks, HIST_THREADS, 0, st>>>(ids, n, counts, bins);
        return xma_check_launch("histogram_global_kernel");
    }
    int copies, stride;
    hist_lds_layout(bins, copies, stride);
    const size_t lds = (size_t)copies * stride * sizeof(uint32_t);
    int64_t chunk, units;
    hist_units(n, chunk, units);
    const bool two_pass = table && n >= HIST_TWO_PASS_MIN && table_bytes >= (size_t)units * bins * sizeof(uint32_t);
    if (!two_pass) {
        // one pass, one global atomic per non-empty bin and workgroup: few workgroups, so few atomics per address
        int64_t blocks = (n + HIST_THREADS * 16 - 1) / (HIST_THREADS * 16);
        if (blocks > 256) blocks = 256;
        chunk = (n + blocks - 1) / blocks;
        chunk = (chunk + 15) & ~(int64_t)15;
        blocks = (n + chunk - 1) / chunk;
        histogram_kernel<IdT, 0><<<(int)blocks, HIST_THREADS, lds, st>>>(ids, n, chunk, counts, bins, copies, stride);
        return xma_check_launch("histogram_kernel");
    }
    histogram_kernel<IdT, 1><<<(int)units, HIST_THREADS, lds, st>>>(ids, n, chunk, table, bins, copies, stride);
    int rc = xma_check_launch("histogram_kernel");
    if (rc) return rc;
    histogram_reduce_kernel<1><<<bins, 256, 0, st>>>(table, (int)units, bins, counts);
    return xma_check_launch("histogram_reduce_kernel");
}

} // namespace xma_rocm

using namespace xma_rocm;

extern "C" size_t xma_rocm_continuous_count_workspace_bytes(int64_t n, int32_t bins) {
    if (n < HIST_TWO_PASS_MIN || bins < 1 || bins > HIST_LDS_WORDS) return 0;
    int64_t chunk, units;
    hist_units(n, chunk, units);
    return (size_t)units * (size_t)bins * sizeof(uint32_t);
}

extern "C" int xma_rocm_continuous_count(const void *ids, int ids_are_int64, int64_t n, uint32_t *counts, int32_t bins,
                                         void *workspace, size_t workspace_bytes, void *stream) {
    XMA_REQUIRE(n >= 0 && bins >= 1, XMA_ROCM_EINVAL, "continuous_count: n=%lld bins=%d", (long long)n, bins);
    XMA_REQUIRE(counts != nullptr && (ids != nullptr || n == 0), XMA_ROCM_EINVAL, "continuous_count: null pointer");
    XMA_REQUIRE(((uintptr_t)ids % (ids_are_int64 ? 8 : 4)) == 0, XMA_ROCM_EINVAL, "continuous_count: misaligned ids");
    if (n == 0) return XMA_ROCM_OK;
    hipStream_t st = (hipStream_t)stream;
    if (ids_are_int64)
        return hist_launch_t<int64_t>((const int64_t *)ids, n, counts, bins, (uint32_t *)workspace, workspace_bytes, st);
    return hist_launch_t<int32_t>((const int32_t *)ids, n, counts, bins, (uint32_t *)workspace, workspace_bytes, st);
}

extern "C" size_t xma_rocm_continuous_count_set_workspace_bytes(int64_t n, int32_t bins) {
    if (n <= UNIT_IDS || bins < 1 || bins > HIST_LDS_WORDS) return 0; // one workgroup writes the counts itself
    int64_t chunk, units;
    hist_units(n, chunk, units);
    return (size_t)units * (size_t)bins * sizeof(uint32_t);
}

extern "C" int xma_rocm_continuous_count_set(const void *ids, int ids_are_int64, int64_t n, uint32_t *counts, int32_t bins,
                                             void *workspace, size_t workspace_bytes, void *stream) {
    XMA_REQUIRE(n >= 0 && bins >= 1 && bins <= HIST_LDS_WORDS, XMA_ROCM_EINVAL, "continuous_count_set: n=%lld bins=%d (bins <= %d)",
                (long long)n, bins, HIST_LDS_WORDS);
    XMA_REQUIRE(counts != nullptr && (ids != nullptr || n == 0), XMA_ROCM_EINVAL, "continuous_count_set: null pointer");
    XMA_REQUIRE(((uintptr_t)ids % (ids_are_int64 ? 8 : 4)) == 0, XMA_ROCM_EINVAL, "continuous_count_set: misaligned ids");
    const size_t need = xma_rocm_continuous_count_set_workspace_bytes(n, bins);
    XMA_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), XMA_ROCM_EWORKSPACE,
                "continuous_count_set: workspace %zu < %zu bytes", workspace ? workspace_bytes : (size_t)0, need);
    hipStream_t st = (hipStream_t)stream;
    if (ids_are_int64)
        return hist_launch_t<int64_t>((const int64_t *)ids, n, counts, bins, (uint32_t *)workspace, workspace_bytes, st, true);
    return hist_launch_t<int32_t>((const int32_t *)ids, n, counts, bins, (uint32_t *)workspace, workspace_bytes, st, true);
}

extern "C" int xma_rocm_route_set_rank_method(int method) {
    XMA_REQUIRE(method == 0 || method == 1, XMA_ROCM_EINVAL, "route_set_rank_method: %d (0 = LDS atomic order, 1 = ballots)",
                method);
    g_route_rank_method.store(method, std::memory_order_relaxed);
    return XMA_ROCM_OK;
}

extern "C" size_t xma_rocm_route_workspace_bytes(int64_t n, int32_t num_experts) {
    if (n < 0 || num_experts < 1) return 0;
    int64_t units = (n + ROUTE_CHUNK - 1) / ROUTE_CHUNK;
    if (units < 1) units = 1;
    return (size_t)units * (size_t)num_experts * sizeof(uint32_t);
}

// Device address of `scratch` on the current device, looked up once per device (with that device current).
static int route_static_scratch(uint32_t **out) {
    constexpr int MAX_DEVICES = 64;
    static std::mutex lock;
    static uint32_t *ptr[MAX_DEVICES] = {nullptr};
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        xma_set_error("route_static: hipGetDevice: %s (device %d)", hipGetErrorString(err), dev);
        return XMA_ROCM_ELAUNCH;
    }
    std::lock_guard<std::mutex> guard(lock);
    if (!ptr[dev]) {
        uint32_t *p = nullptr;
        err = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !p) {
            xma_set_error("route_static: hipGetSymbolAddress(scratch): %s", hipGetErrorString(err));
            return XMA_ROCM_ELAUNCH;
        }
        ptr[dev] = p;
    }
    *out = ptr[dev];
    return XMA_ROCM_OK;
}

extern "C" size_t xma_rocm_route_static_max_units_times_experts(void) { return ROUTE_STATIC_WORDS; }

extern "C" int xma_rocm_route_static(const void *ids, int ids_are_int64, int64_t n, int32_t E, uint32_t *counts,
                                     int64_t *offsets_inclusive, int64_t *offsets_exclusive, void *sorted_expert_idxs,
                                     int64_t *sorted_scattered_idxs, void *stream) {
    XMA_REQUIRE(n >= 0 && E >= 1 && E <= ROUTE_MAX_E, XMA_ROCM_EINVAL, "route_static: n=%lld E=%d (E <= %d)",
                (long long)n, E, ROUTE_MAX_E);
    XMA_REQUIRE(n < (int64_t)1 << 31, XMA_ROCM_EUNSUPPORTED, "route_static: n=%lld does not fit 31 bits", (long long)n);
    XMA_REQUIRE(counts && offsets_inclusive && (n == 0 || (ids && sorted_scattered_idxs)), XMA_ROCM_EINVAL,
                "route_static: null pointer");
    const size_t need = xma_rocm_route_workspace_bytes(n, E);
    XMA_REQUIRE(need <= ROUTE_STATIC_WORDS * sizeof(uint32_t), XMA_ROCM_EWORKSPACE,
                "route_static: ceil(n / %d) * E = %zu exceeds the static scratch of %zu words; use xma_rocm_route with a "
                "workspace",
                ROUTE_CHUNK, need / sizeof(uint32_t), ROUTE_STATIC_WORDS);
    uint32_t *ws = nullptr;
    int rc = route_static_scratch(&ws);
    if (rc) return rc;
    // every word of the scratch that the scatter reads is written by the unit histogram pass of the same call: nothing
    // of an earlier call is carried over, nothing has to be cleared
    hipStream_t st = (hipStream_t)stream;
    if (ids_are_int64)
        return route_launch<int64_t>((const int64_t *)ids, n, E, counts, offsets_inclusive, offsets_exclusive,
                                     (int64_t *)sorted_expert_idxs, sorted_scattered_idxs, ws, st);
    return route_launch<int32_t>((const int32_t *)ids, n, E, counts, offsets_inclusive, offsets_exclusive,
                                 (int32_t *)sorted_expert_idxs, sorted_scattered_idxs, ws, st);
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
    if (ids_are_int64)
        return route_launch<int64_t>((const int64_t *)ids, n, E, counts, offsets_inclusive, offsets_exclusive,
                                     (int64_t *)sorted_expert_idxs, sorted_scattered_idxs, (uint32_t *)workspace, st);
    return route_launch<int32_t>((const int32_t *)ids, n, E, counts, offsets_inclusive, offsets_exclusive,
                                 (int32_t *)sorted_expert_idxs, sorted_scattered_idxs, (uint32_t *)workspace, st);
}
