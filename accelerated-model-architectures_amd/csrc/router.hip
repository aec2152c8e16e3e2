// Router of the MoE layer behind the gate GEMM: top-k selection over each row of expert logits, fp32 softmax over the
// k selected values and the selected expert ids in one pass (xma/layers/moe/__init__.py:186-193 and :256-262), and the
// backward of that chain (gradient of the logits from the gradient of the router weights).
//
// A row is held in registers by a group of G = min(64, next power of two >= E) lanes of a wave, VPL = ceil(E / G)
// values per lane (element e lives in lane e % G), so a wave takes 64 / G rows.  Selection is k rounds of "largest
// remaining value, lowest index among equals" by a butterfly over the group; round r leaves its winner in lane r, so
// the k results of a row come out of k neighbouring lanes.  HBM traffic is the logits once in, (weights, ids) once out.
#include "common.hpp"

namespace {

constexpr int RT_THREADS = 256;
constexpr int RT_MAX_E = 2048, RT_MAX_K = 64;

// monotone map float -> uint32 (a larger value has a larger key).  NaN is the largest value, as in torch.topk;
// -0 and +0 are equal; every key is > 0, so 0 marks "not a candidate".
__device__ __forceinline__ uint32_t order_key(float v) {
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    if (v != v) return 0xffffffffu;
    if (u == 0x80000000u) u = 0;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t key) {
    if (key == 0xffffffffu) return __builtin_nanf("");
    const uint32_t u = (key & 0x80000000u) ? (key ^ 0x80000000u) : ~key;
    return __builtin_bit_cast(float, u);
}

template <int DT> struct Scalar;
template <> struct Scalar<XMA_ROCM_BF16> {
    typedef uint16_t type;
    static __device__ __forceinline__ float load(const void *p, int64_t i) {
        return Elem<__bf16>::lo((uint32_t)((const uint16_t *)p)[i]);
    }
    static __device__ __forceinline__ void store(void *p, int64_t i, float v) {
        ((uint16_t *)p)[i] = (uint16_t)(Elem<__bf16>::pack(v, 0.f) & 0xffffu);
    }
};
template <> struct Scalar<XMA_ROCM_F16> {
    typedef uint16_t type;
    static __device__ __forceinline__ float load(const void *p, int64_t i) {
        return Elem<_Float16>::lo((uint32_t)((const uint16_t *)p)[i]);
    }
    static __device__ __forceinline__ void store(void *p, int64_t i, float v) {
        ((uint16_t *)p)[i] = (uint16_t)(Elem<_Float16>::pack(v, 0.f) & 0xffffu);
    }
};
template <> struct Scalar<XMA_ROCM_F32> {
    typedef float type;
    static __device__ __forceinline__ float load(const void *p, int64_t i) { return ((const float *)p)[i]; }
    static __device__ __forceinline__ void store(void *p, int64_t i, float v) { ((float *)p)[i] = v; }
};

// A lane's own value and that of the lane whose index differs in bit log2(M) (for 4 and 8: of the mirrored lane of the
// 8- or 16-lane block, which lies in the other half just the same), as an unordered pair - which of the two members is
// the lane's own differs from lane to lane, so only commutative use is meant.  Inside a row of 16 lanes the partner is a
// DPP operand of the consuming VALU instruction; rows are exchanged by v_permlane16_swap / v_permlane32_swap, which swap
// the odd rows (the upper half) of one register with the even rows (the lower half) of another.  No LDS round trip.
struct LanePair {
    uint32_t a, b;
};
template <int M> __device__ __forceinline__ LanePair pair_exchange(uint32_t v) {
    const int x = (int)v;
    if constexpr (M == 1) return {v, (uint32_t)__builtin_amdgcn_mov_dpp(x, 0xB1, 0xf, 0xf, true)};  // quad_perm 1,0,3,2
    if constexpr (M == 2) return {v, (uint32_t)__builtin_amdgcn_mov_dpp(x, 0x4E, 0xf, 0xf, true)};  // quad_perm 2,3,0,1
    if constexpr (M == 4) return {v, (uint32_t)__builtin_amdgcn_mov_dpp(x, 0x141, 0xf, 0xf, true)}; // row_half_mirror
    if constexpr (M == 8) return {v, (uint32_t)__builtin_amdgcn_mov_dpp(x, 0x140, 0xf, 0xf, true)}; // row_mirror
    if constexpr (M == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
        return {r[0], r[1]};
    }
    if constexpr (M == 32) {
        const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
        return {r[0], r[1]};
    }
}

// all-reduce over the G lanes of a group; op(a, b) must be commutative and associative
template <int G, int M = 1, typename Op> __device__ __forceinline__ uint32_t group_reduce(uint32_t v, Op op) {
    if constexpr (M < G) {
        const LanePair p = pair_exchange<M>(v);
        return group_reduce<G, M * 2>(op(p.a, p.b), op);
    } else
        return v;
}
template <int G> __device__ __forceinline__ float group_sum(float v) {
    const uint32_t r = group_reduce<G>(__builtin_bit_cast(uint32_t, v), [](uint32_t a, uint32_t b) {
        return __builtin_bit_cast(uint32_t, __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b));
    });
    return __builtin_bit_cast(float, r);
}

// softmax over the values held by lanes 0..k-1 of a group; lane 0 holds the largest (NaN propagates like in torch)
template <int G> __device__ __forceinline__ float group_softmax(float my_val, int g, int k, int group_lane0) {
    const float vmax = __shfl(my_val, group_lane0);
    const float ex = (g < k) ? expf(my_val - vmax) : 0.f;
    return ex / group_sum<G>(ex);
}

// A candidate of the selection: larger value first, lower expert index among equal values.  16-bit logits have
// 16-bit keys, so key and inverted index share one word and the butterfly is a plain integer maximum; fp32 logits
// carry the index in a second word.  The all-zero candidate loses against every real one.
template <int DT> struct Cand {
    uint32_t packed; // key16 << 16 | (0xffff - index)
    static __device__ __forceinline__ Cand none() { return {0u}; }
    static __device__ __forceinline__ Cand make(const void *row, int e) { return from_bits(((const uint16_t *)row)[e], e); }
    static __device__ __forceinline__ Cand from_bits(uint32_t b, int e) {
        const uint32_t inf = (DT == XMA_ROCM_BF16) ? 0x7f80u : 0x7c00u;
        uint32_t key;
        if ((b & 0x7fffu) > inf)
            key = 0xffffu;
        else if (b == 0x8000u)
            key = 0x8000u;
        else
            key = (b & 0x8000u) ? (~b & 0xffffu) : (b | 0x8000u);
        return {(key << 16) | (0xffffu - (uint32_t)e)};
    }
    __device__ __forceinline__ bool beats(const Cand &o) const { return packed > o.packed; }
    __device__ __forceinline__ bool same(const Cand &o) const { return packed == o.packed; } // value and index
    __device__ __forceinline__ bool is_none() const { return packed == 0u; }
    __device__ __forceinline__ int index() const { return (int)(0xffffu - (packed & 0xffffu)); }
    __device__ __forceinline__ float value() const {
        const uint32_t key = packed >> 16;
        const uint32_t b = (key == 0xffffu) ? 0x7fffu : ((key & 0x8000u) ? (key ^ 0x8000u) : (~key & 0xffffu));
        return (DT == XMA_ROCM_BF16) ? Elem<__bf16>::lo(b) : Elem<_Float16>::lo(b);
    }
    template <int G> __device__ __forceinline__ Cand group_best() const {
        return {group_reduce<G>(packed, [](uint32_t a, uint32_t b) { return a > b ? a : b; })};
    }
};
template <> struct Cand<XMA_ROCM_F32> {
    uint32_t key;
    int idx;
    static __device__ __forceinline__ Cand none() { return {0u, 0x7fffffff}; }
    static __device__ __forceinline__ Cand make(const void *row, int e) { return {order_key(((const float *)row)[e]), e}; }
    __device__ __forceinline__ bool beats(const Cand &o) const { return key > o.key || (key == o.key && idx < o.idx); }
    __device__ __forceinline__ bool same(const Cand &o) const { return key == o.key && idx == o.idx; }
    __device__ __forceinline__ bool is_none() const { return key == 0u; }
    __device__ __forceinline__ int index() const { return idx; }
    __device__ __forceinline__ float value() const { return key_value(key); }
    template <int G, int M = 1> __device__ __forceinline__ Cand group_best() const {
        if constexpr (M < G) {
            const LanePair pk = pair_exchange<M>(key), pi = pair_exchange<M>((uint32_t)idx);
            const Cand a = {pk.a, (int)pi.a}, b = {pk.b, (int)pi.b};
            const Cand w = b.beats(a) ? b : a;
            return w.template group_best<G, M * 2>();
        } else
            return *this;
    }
};

template <int DT, int G, int VPL>
__global__ __launch_bounds__(RT_THREADS) void router_topk_kernel(const void *__restrict__ logits, int64_t ld, int64_t T,
                                                                int E, int k, void *__restrict__ weights,
                                                                void *__restrict__ ids, int ids_i64) {
    const int lane = threadIdx.x & 63;
    const int g = lane & (G - 1);
    const int64_t wave = (int64_t)blockIdx.x * (RT_THREADS / 64) + (threadIdx.x >> 6);
    const int64_t t = wave * (64 / G) + lane / G;
    const bool live = t < T; // the same for all lanes of a group; dead groups still take part in the exchanges
    const void *row = (const char *)logits + (live ? t : 0) * ld * (int64_t)sizeof(typename Scalar<DT>::type);
    Cand<DT> c[VPL];
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const int e = g + v * G;
        c[v] = (live && e < E) ? Cand<DT>::make(row, e) : Cand<DT>::none();
    }
    Cand<DT> mine = Cand<DT>::none();
    for (int r = 0; r < k; ++r) {
        Cand<DT> best = c[0];
#pragma unroll
        for (int v = 1; v < VPL; ++v)
            if (c[v].beats(best)) best = c[v];
        best = best.template group_best<G>();
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            if (c[v].same(best)) c[v] = Cand<DT>::none(); // taken (an index occurs once: at most one lane and slot matches)
        if (g == r) mine = best;
    }
    const float w = group_softmax<G>(mine.value(), g, k, lane - g);
    if (live && g < k) {
        Scalar<DT>::store(weights, t * k + g, w);
        if (ids_i64)
            ((int64_t *)ids)[t * k + g] = mine.index();
        else
            ((int32_t *)ids)[t * k + g] = mine.index();
    }
}

// d_logits[t, :] = 0 except d_logits[t, ids[t, j]] = w_j * (d_w[t, j] - sum_i w_i d_w[t, i]), w = the fp32 softmax of
// the selected logits, recomputed exactly as in the forward kernel.  Writes every element of d_logits.
template <int DT, int G, int VPL>
__global__ __launch_bounds__(RT_THREADS) void router_topk_bwd_kernel(const void *__restrict__ logits, int64_t ld,
                                                                    int64_t T, int E, int k,
                                                                    const void *__restrict__ ids, int ids_i64,
                                                                    const void *__restrict__ d_w,
                                                                    void *__restrict__ d_logits, int64_t ldd) {
    const int lane = threadIdx.x & 63;
    const int g = lane & (G - 1);
    const int64_t wave = (int64_t)blockIdx.x * (RT_THREADS / 64) + (threadIdx.x >> 6);
    const int64_t t = wave * (64 / G) + lane / G;
    const bool live = t < T;
    int my_idx = -1;
    float my_val = 0.f, my_dw = 0.f;
    if (live && g < k) {
        my_idx = ids_i64 ? (int)((const int64_t *)ids)[t * k + g] : ((const int32_t *)ids)[t * k + g];
        my_idx = my_idx < 0 ? 0 : (my_idx >= E ? E - 1 : my_idx); // ids come from the forward; never read outside the row
        my_val = key_value(order_key(Scalar<DT>::load(logits, t * ld + my_idx)));
        my_dw = Scalar<DT>::load(d_w, t * k + g);
    }
    const float w = group_softmax<G>(my_val, g, k, lane - g);
    const float dot = group_sum<G>((g < k) ? w * my_dw : 0.f);
    const float dv = w * (my_dw - dot);
    float out[VPL];
#pragma unroll
    for (int v = 0; v < VPL; ++v) out[v] = 0.f;
    for (int j = 0; j < k; ++j) {
        const int ej = __shfl(my_idx, lane - g + j);
        const float dj = __shfl(dv, lane - g + j);
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            if (g + v * G == ej) out[v] = dj;
    }
    if (live) {
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            const int e = g + v * G;
            if (e < E) Scalar<DT>::store(d_logits, t * ldd + e, out[v]);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Gate projection fused with the router: logits = x @ Wg^T (fp32 accumulation, rounded to the activation dtype as the
// stock linear layer does), then top-k, fp32 softmax and expert ids from the rounded logits, in one kernel
// (xma/layers/moe/__init__.py:182-195, 256-262).  x (T, H) is streamed from HBM exactly once; Wg (E, H) stays in cache.
//
// A workgroup of 4 waves takes 32 tokens and splits H into four K ranges, one per wave, so that even a layer of a few
// thousand tokens puts four waves on every SIMD and keeps enough loads in flight.  A wave multiplies its 32 x (H / 4)
// slice of x with Wg by v_mfma_f32_32x32x16 (tokens = register dimension, experts = lanes, NB blocks of 32 experts); both
// operands come straight from global memory, 64 contiguous bytes per lane and K step - a step's 64 k are dealt to the two
// half-waves as 32 + 32, which is the same permutation of k for both operands and therefore leaves the product unchanged.
// The four partial results meet in LDS; wave w then owns 8 of the 32 tokens: their logits sit across the 32 lanes of a
// half-wave, NB per lane, exactly the layout the selection network of router_topk_kernel works on (G = 32).
// ------------------------------------------------------------------------------------------------
// S accumulator slots of the gate product at once: in a slot the lanes of a half-wave hold one token's logits, lane r
// the experts 32 b + r (sum_of(s, b) = fp32 sum of block b of slot s; token_of(s) = the token of this lane's half).
// Rounds them to the activation dtype, stores them, selects the k largest (lowest index among equals), and stores
// fp32-softmax weights and expert ids.  A round of the selection is a chain of dependent cross-lane exchanges; the S
// slots are S independent chains for the scheduler to interleave.
template <typename T, int DT, int NB, int S, typename TokenOf, typename SumOf>
__device__ __forceinline__ void gate_finish_slots(int64_t n_tokens, int r, int lane, int E, int k, TokenOf token_of,
                                                  SumOf sum_of, uint16_t *__restrict__ logits, int64_t ldl,
                                                  void *__restrict__ weights, void *__restrict__ ids, int ids_i64) {
    const int g = r;
    int64_t t[S];
    bool live[S];
    Cand<DT> c[S][NB], mine[S];
    // all sums are read before anything is decided on them: the empty asm statements keep the compiler from sinking
    // each read into the predicated region of its store, where every one of them would be waited for on its own
    float sum[S][NB];
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
        for (int b = 0; b < NB; ++b) sum[s][b] = sum_of(s, b);
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
        for (int b = 0; b < NB; ++b) asm volatile("" : "+v"(sum[s][b]));
#pragma unroll
    for (int s = 0; s < S; ++s) {
        t[s] = token_of(s);
        live[s] = t[s] < n_tokens;
        mine[s] = Cand<DT>::none();
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint32_t bits = Elem<T>::pack(sum[s][b], 0.f) & 0xffffu;
            const int e = b * 32 + r;
            if (live[s] && e < E) logits[t[s] * ldl + e] = (uint16_t)bits;
            c[s][b] = (live[s] && e < E) ? Cand<DT>::from_bits(bits, e) : Cand<DT>::none();
        }
    }
    for (int round = 0; round < k; ++round) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
            Cand<DT> best = c[s][0];
#pragma unroll
            for (int b = 1; b < NB; ++b)
                if (c[s][b].beats(best)) best = c[s][b];
            best = best.template group_best<32>();
#pragma unroll
            for (int b = 0; b < NB; ++b)
                if (c[s][b].same(best)) c[s][b] = Cand<DT>::none(); // taken (an index occurs once: at most one match)
            if (g == round) mine[s] = best;
        }
    }
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const float w = group_softmax<32>(mine[s].value(), g, k, lane - g);
        if (live[s] && g < k) {
            Scalar<DT>::store(weights, t[s] * k + g, w);
            if (ids_i64)
                ((int64_t *)ids)[t[s] * k + g] = mine[s].index();
            else
                ((int32_t *)ids)[t[s] * k + g] = mine[s].index();
        }
    }
}

constexpr int RG_THREADS = 256, RG_TOKENS = 32, RG_MAX_E = 128, RG_MAX_K = 32;

template <typename T, int DT, int NB>
__global__ __launch_bounds__(RG_THREADS) void router_gate_topk_kernel(const uint16_t *__restrict__ x, int64_t ldx,
                                                                      const uint16_t *__restrict__ wg, int64_t ldw,
                                                                      int64_t n_tokens, int H, int E, int k,
                                                                      uint16_t *__restrict__ logits, int64_t ldl,
                                                                      void *__restrict__ weights, void *__restrict__ ids,
                                                                      int ids_i64) {
    __shared__ float s_part[4][16 * NB][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // a scalar: K ranges and their branches are uniform
    const int r = lane & 31, half = lane >> 5;
    const int64_t t0 = (int64_t)blockIdx.x * RG_TOKENS;
    const int64_t my_t = (t0 + r < n_tokens) ? t0 + r : n_tokens - 1; // clamped: rows past the end are never stored
    const int steps = (H + 63) / 64;
    const int s_begin = wave * steps / 4, s_end = (wave + 1) * steps / 4;
    const uint16_t *xrow = x + my_t * ldx + half * 32;
    const uint16_t *wrow[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int e = b * 32 + r; // lanes past E read row E - 1: their accumulator columns are never looked at
        wrow[b] = wg + (int64_t)(e < E ? e : E - 1) * ldw + half * 32;
    }
    struct Stage {
        u32x4 xa[4];
        u32x4 wb[NB][4];
    };
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    // Steps inside H are plain loads, nothing selected and no branch per lane, so the compiler can count the loads in
    // flight and wait only for the stage it multiplies.  The last step of an H that is no multiple of 64 runs apart
    // from the loop: it reads each 16-byte chunk only where it lies inside the row (H is a multiple of 8) and takes
    // zeros elsewhere.
    const int steps_full = H / 64;
    auto fetch = [&](Stage &st, int step) {
        const int k0 = step * 64;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            st.xa[q] = *(const u32x4 *)(xrow + k0 + 8 * q);
#pragma unroll
            for (int b = 0; b < NB; ++b) st.wb[b][q] = *(const u32x4 *)(wrow[b] + k0 + 8 * q);
        }
    };
    auto fetch_partial = [&](Stage &st, int step) {
        const int k0 = step * 64;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const bool in = k0 + half * 32 + 8 * q < H;
            st.xa[q] = in ? *(const u32x4 *)(xrow + k0 + 8 * q) : zero4;
#pragma unroll
            for (int b = 0; b < NB; ++b) st.wb[b][q] = in ? *(const u32x4 *)(wrow[b] + k0 + 8 * q) : zero4;
        }
    };
    f32x16 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;
    auto multiply = [&](const Stage &st) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[b] = Elem<T>::mfma(st.xa[q], st.wb[b][q], acc[b]);
    };
    // two stages of operands in registers: the loads of step s + 1 are in flight while step s multiplies
    // (every workgroup starts its wave's K range at a step of its own and wraps around: workgroups that run together are
    // at about the same step, and walking from the front they would all ask for the same 128 bytes of every row of x)
    Stage s0, s1;
    const int f_end = s_end < steps_full ? s_end : steps_full;
    const int cnt = f_end - s_begin, rot = cnt > 0 ? (int)((blockIdx.x * 3u) % (unsigned)cnt) : 0;
    auto step_of = [&](int i) {
        const int j = i + rot;
        return s_begin + (j < cnt ? j : j - cnt);
    };
    if (cnt > 0) fetch(s0, step_of(0));
    for (int i = 0; i < cnt; i += 2) {
        if (i + 1 < cnt) fetch(s1, step_of(i + 1));
        multiply(s0);
        if (i + 1 < cnt) {
            if (i + 2 < cnt) fetch(s0, step_of(i + 2));
            multiply(s1);
        }
    }
    if (s_end > steps_full) { // the last wave, when H is no multiple of 64
        fetch_partial(s0, steps_full);
        multiply(s0);
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) s_part[wave][b * 16 + v][lane] = acc[b][v];
    __syncthreads();

    // wave w finishes accumulator slots v = 4 w .. 4 w + 3: in slot v the lanes of half h hold token
    // 8 (v / 4) + 4 h + v % 4 of the tile, lane r of the half the experts 32 b + r
    gate_finish_slots<T, DT, NB, 4>(
        n_tokens, r, lane, E, k, [&](int s) { return t0 + 8 * wave + 4 * half + s; },
        [&](int s, int b) {
            const int v = 4 * wave + s;
            return (s_part[0][b * 16 + v][lane] + s_part[1][b * 16 + v][lane]) +
                   (s_part[2][b * 16 + v][lane] + s_part[3][b * 16 + v][lane]);
        },
        logits, ldl, weights, ids, ids_i64);
}

// The same product for layers of more than 32 experts, where Wg no longer is a small operand: every lane fetching its
// own expert row per K step (32 rows of 64 bytes per load instruction, NB times per step) makes the texture path, not
// HBM, the limit.  Here a workgroup takes 64 tokens, two waves of 32, and each K step's slice of Wg (32 NB rows x 64 k)
// is loaded once for both with coalesced 16-byte loads (8 lanes per row), kept in LDS in two stages and read from there
// as MFMA operands; a row of the slice takes 144 bytes of LDS, so the 16 lanes of a ds_read_b128 phase fall into 16
// different 4-bank groups.  x still comes straight from global memory, 64 contiguous bytes per lane and step, DEPTH
// steps ahead in registers.  With KS = 2 the workgroup has a second pair of waves that takes the other half of the K
// range (with its own slices), which puts a wave on every SIMD when the layer has too few tokens for that otherwise.
// The accumulators pass through LDS; the pairs share out the 16 accumulator slots for the selection, which adds the
// KS partial sums as it reads them.
constexpr int RL_TOKENS = 64, RL_ROW = 72;
constexpr int64_t RL_SPLIT_K_BELOW = 98304; // tokens: fewer leave a 256-CU device less than three waves per SIMD at one wave per 32 tokens
                                            // (with two, one wave's selection tail runs beside the other's K loop)

template <int NB, int KS> constexpr int rl_lds_bytes() { return 2 * KS * NB * 32 * RL_ROW * 2; }

template <typename T, int DT, int NB, int KS>
__global__ __launch_bounds__(128 * KS) void router_gate_topk_lds_kernel(const uint16_t *__restrict__ x, int64_t ldx,
                                                                        const uint16_t *__restrict__ wg, int64_t ldw,
                                                                        int64_t n_tokens, int H, int E, int k,
                                                                        uint16_t *__restrict__ logits, int64_t ldl,
                                                                        void *__restrict__ weights, void *__restrict__ ids,
                                                                        int ids_i64) {
    constexpr int SLICE = NB * 32 * RL_ROW;      // halfwords of one slice
    constexpr int DEPTH = NB <= 2 ? 8 : 4;       // steps of x in flight: what fits beside the accumulators at 2 waves per SIMD
    constexpr int W_CHUNKS = NB * 32 * 8 / 128;  // 16-byte chunks of a slice per thread of the pair that loads it
    static_assert(rl_lds_bytes<NB, KS>() >= 2 * KS * NB * 16 * 64 * 4, "the accumulators pass through the operand stages");
    extern __shared__ __attribute__((aligned(16))) uint16_t s_w[]; // [2 stages][KS][SLICE]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tb = wave & 1, kh = wave >> 1, ptid = tid & 127; // token block, K range, thread of the pair
    const int r = lane & 31, half = lane >> 5;
    const int64_t t0 = (int64_t)blockIdx.x * RL_TOKENS + tb * 32;
    const int64_t my_t = (t0 + r < n_tokens) ? t0 + r : n_tokens - 1; // clamped: rows past the end are never stored
    const uint16_t *xrow = x + my_t * ldx + half * 32;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};

    f32x16 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;

    // Steps inside H are plain loads (nothing selected, no branch per lane: the compiler counts the loads in flight
    // and waits only for what a step uses); loads for steps past the pair's last one re-read step 0 and are never
    // used.  Rows of the slice past E re-read row E - 1: their accumulator columns are never looked at.
    const int steps_full = H / 64, per = (steps_full + KS - 1) / KS; // every pair runs `per` rounds of barriers
    const int s_lo = kh * per, my_steps = steps_full - s_lo < per ? (steps_full - s_lo > 0 ? steps_full - s_lo : 0) : per;
    // Workgroups that run together are at about the same step; with all of them walking K from the front, the requests of
    // a moment fall on the same 128 bytes of every row of x, a fraction of the memory channels.  Every workgroup starts
    // at a step of its own and wraps around inside its pair's K range.
    const int rot = my_steps > 0 ? (int)((blockIdx.x * 3u) % (unsigned)my_steps) : 0;
    auto step_of = [&](int i) {
        const int j = i + rot;
        return s_lo + (j < my_steps ? j : j - my_steps);
    };
    auto fetch_x = [&](u32x4(&d)[4], int i) {
        const int k0 = (i < my_steps ? step_of(i) : 0) * 64;
#pragma unroll
        for (int q = 0; q < 4; ++q) d[q] = *(const u32x4 *)(xrow + k0 + 8 * q);
    };
    // chunk c of a slice: expert row c / 8, k offset 8 (c % 8)
    auto fetch_w = [&](u32x4(&d)[W_CHUNKS], int i) {
        const int k0 = step_of(i) * 64;
#pragma unroll
        for (int j = 0; j < W_CHUNKS; ++j) {
            const int c = ptid + 128 * j, e = c >> 3;
            d[j] = *(const u32x4 *)(wg + (int64_t)(e < E ? e : E - 1) * ldw + k0 + 8 * (c & 7));
        }
    };
    auto store_w = [&](const u32x4(&d)[W_CHUNKS], int buf) {
#pragma unroll
        for (int j = 0; j < W_CHUNKS; ++j) {
            const int c = ptid + 128 * j;
            *(u32x4 *)(s_w + (buf * KS + kh) * SLICE + (c >> 3) * RL_ROW + 8 * (c & 7)) = d[j];
        }
    };
    auto multiply = [&](const u32x4(&xa)[4], int buf) {
        const uint16_t *ws = s_w + (buf * KS + kh) * SLICE + r * RL_ROW + half * 32;
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const u32x4 wb = *(const u32x4 *)(ws + b * 32 * RL_ROW + 8 * q);
                acc[b] = Elem<T>::mfma(xa[q], wb, acc[b]);
            }
    };

    u32x4 xs[DEPTH][4];
    u32x4 wr[W_CHUNKS];
    if (steps_full > 0) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) fetch_x(xs[d], d);
        if (my_steps > 0) {
            fetch_w(wr, 0);
            store_w(wr, 0);
        }
    }
    __syncthreads();
    for (int base = 0; base < per; base += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const int i = base + u;
            if (i < per) { // uniform over the workgroup; what follows is uniform over the pair
                const bool more = i + 1 < my_steps;
                if (more) fetch_w(wr, i + 1);
                if (i < my_steps) multiply(xs[u], u & 1);
                fetch_x(xs[u], i + DEPTH);
                if (more) store_w(wr, (u + 1) & 1);
                __syncthreads();
            }
        }
    }
    if (steps_full * 64 < H) {
        // the last, partial step of an H that is no multiple of 64, taken by the first pair: a 16-byte chunk lies
        // inside the row or outside (H is a multiple of 8); the chunks outside are zeros in both operands
        const int k0 = steps_full * 64, buf = per & 1; // this stage was last read before the previous barrier
        u32x4 xa[4];
        if (kh == 0) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                xa[q] = (k0 + half * 32 + 8 * q < H) ? *(const u32x4 *)(xrow + k0 + 8 * q) : zero4;
#pragma unroll
            for (int j = 0; j < W_CHUNKS; ++j) {
                const int c = ptid + 128 * j, e = c >> 3, kk = k0 + 8 * (c & 7);
                wr[j] = (kk < H) ? *(const u32x4 *)(wg + (int64_t)(e < E ? e : E - 1) * ldw + kk) : zero4;
            }
            store_w(wr, buf);
        }
        __syncthreads();
        if (kh == 0) multiply(xa, buf);
        __syncthreads();
    }
    // after the last barrier nobody reads the operand stages any more
    float *s_acc = (float *)s_w;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) s_acc[(wave * NB * 16 + b * 16 + v) * 64 + lane] = acc[b][v];
    if constexpr (KS > 1) __syncthreads(); // with one pair every lane reads back only what it wrote itself
    for (int v0 = kh * (16 / KS); v0 < (kh + 1) * (16 / KS); v0 += 4)
        gate_finish_slots<T, DT, NB, 4>(
            n_tokens, r, lane, E, k, [&](int s) { return t0 + 2 * v0 + 4 * half + s; },
            [&](int s, int b) {
                float sum = s_acc[(tb * NB * 16 + b * 16 + v0 + s) * 64 + lane];
#pragma unroll
                for (int h = 1; h < KS; ++h) sum += s_acc[((2 * h + tb) * NB * 16 + b * 16 + v0 + s) * 64 + lane];
                return sum;
            },
            logits, ldl, weights, ids, ids_i64);
}

template <typename T, int DT>
int router_gate_launch(const void *x, int64_t ldx, const void *wg, int64_t ldw, int64_t n_tokens, int H, int E, int k,
                       void *logits, int64_t ldl, void *weights, void *ids, int ids_i64, hipStream_t st) {
#define RG_ARGS                                                                                                    \
    (const uint16_t *)x, ldx, (const uint16_t *)wg, ldw, n_tokens, H, E, k, (uint16_t *)logits, ldl, weights, ids, ids_i64
#define RL_LAUNCH(NB, KS)                                                                                          \
    {                                                                                                              \
        auto kernel = router_gate_topk_lds_kernel<T, DT, NB, KS>;                                                  \
        if (int rc = xma_set_max_lds_once((const void *)kernel, rl_lds_bytes<NB, KS>())) return rc;                \
        kernel<<<(unsigned)((n_tokens + RL_TOKENS - 1) / RL_TOKENS), 128 * KS, rl_lds_bytes<NB, KS>(), st>>>(RG_ARGS); \
    }
#define RL_LAUNCH_NB(NB)          \
    if (split_k)                  \
        RL_LAUNCH(NB, 2)          \
    else                          \
        RL_LAUNCH(NB, 1)
    const bool split_k = n_tokens < RL_SPLIT_K_BELOW;
    if (E <= 32)
        router_gate_topk_kernel<T, DT, 1><<<(unsigned)((n_tokens + RG_TOKENS - 1) / RG_TOKENS), RG_THREADS, 0, st>>>(RG_ARGS);
    else if (E <= 64)
        RL_LAUNCH_NB(2)
    else if (E <= 96)
        RL_LAUNCH_NB(3)
    else
        RL_LAUNCH_NB(4)
#undef RL_LAUNCH_NB
#undef RL_LAUNCH
#undef RG_ARGS
    return xma_check_launch("router_gate_topk_kernel");
}

struct RouterShape {
    int G, vpl;
    int64_t blocks;
};

int router_shape(const char *what, int64_t T, int E, int k, int dtype, RouterShape &s) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16 || dtype == XMA_ROCM_F32, XMA_ROCM_EUNSUPPORTED,
                "%s: dtype %d", what, dtype);
    XMA_REQUIRE(T >= 0 && E >= 1 && k >= 1 && k <= E, XMA_ROCM_EINVAL, "%s: T=%lld E=%d k=%d (1 <= k <= E)", what,
                (long long)T, E, k);
    XMA_REQUIRE(E <= RT_MAX_E && k <= RT_MAX_K, XMA_ROCM_EUNSUPPORTED, "%s: E=%d k=%d (E <= %d, k <= %d)", what, E, k,
                RT_MAX_E, RT_MAX_K);
    int G = 1;
    while (G < E && G < 64) G <<= 1;
    int vpl = 1;
    while (G * vpl < E) vpl <<= 1;
    s.G = G;
    s.vpl = vpl;
    const int64_t rows_per_block = (int64_t)(RT_THREADS / 64) * (64 / G);
    s.blocks = (T + rows_per_block - 1) / rows_per_block;
    XMA_REQUIRE(s.blocks < ((int64_t)1 << 31), XMA_ROCM_EUNSUPPORTED, "%s: too many rows", what);
    return XMA_ROCM_OK;
}

#define ROUTER_CASE(g_, v_, CALL)   \
    {                               \
        constexpr int G = g_;       \
        constexpr int VPL = v_;     \
        CALL;                       \
    }                               \
    break;
#define ROUTER_DISPATCH_SHAPE(s, CALL)        \
    switch ((s).G * (s).vpl) {                \
    case 1: ROUTER_CASE(1, 1, CALL)           \
    case 2: ROUTER_CASE(2, 1, CALL)           \
    case 4: ROUTER_CASE(4, 1, CALL)           \
    case 8: ROUTER_CASE(8, 1, CALL)           \
    case 16: ROUTER_CASE(16, 1, CALL)         \
    case 32: ROUTER_CASE(32, 1, CALL)         \
    case 64: ROUTER_CASE(64, 1, CALL)         \
    case 128: ROUTER_CASE(64, 2, CALL)        \
    case 256: ROUTER_CASE(64, 4, CALL)        \
    case 512: ROUTER_CASE(64, 8, CALL)        \
    case 1024: ROUTER_CASE(64, 16, CALL)      \
    default: ROUTER_CASE(64, 32, CALL)        \
    }
#define ROUTER_DISPATCH(dtype, s, CALL)           \
    if (dtype == XMA_ROCM_BF16) {                 \
        constexpr int DT = XMA_ROCM_BF16;         \
        ROUTER_DISPATCH_SHAPE(s, CALL)            \
    } else if (dtype == XMA_ROCM_F16) {           \
        constexpr int DT = XMA_ROCM_F16;          \
        ROUTER_DISPATCH_SHAPE(s, CALL)            \
    } else {                                      \
        constexpr int DT = XMA_ROCM_F32;          \
        ROUTER_DISPATCH_SHAPE(s, CALL)            \
    }

} // namespace

extern "C" int xma_rocm_router_topk(const void *logits, int64_t ld, int64_t T, int32_t E, int32_t k, int dtype,
                                    void *weights, void *ids, int ids_is_i64, void *stream) {
    RouterShape s;
    if (int rc = router_shape("router_topk", T, E, k, dtype, s)) return rc;
    XMA_REQUIRE(ld >= E, XMA_ROCM_EINVAL, "router_topk: ld=%lld < E=%d", (long long)ld, E);
    XMA_REQUIRE(T == 0 || (logits && weights && ids), XMA_ROCM_EINVAL, "router_topk: null pointer");
    if (T == 0) return XMA_ROCM_OK;
    hipStream_t st = (hipStream_t)stream;
    ROUTER_DISPATCH(dtype, s, (router_topk_kernel<DT, G, VPL><<<(int)s.blocks, RT_THREADS, 0, st>>>(
                                  logits, ld, T, E, k, weights, ids, ids_is_i64)));
    return xma_check_launch("router_topk_kernel");
}

extern "C" int xma_rocm_router_gate_topk_supported(int32_t H, int32_t E, int32_t k, int dtype) {
    return (dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16) && H >= 8 && H % 8 == 0 && E >= 1 && E <= RG_MAX_E && k >= 1 &&
           k <= E && k <= RG_MAX_K;
}

extern "C" int xma_rocm_router_gate_topk(const void *x, int64_t ldx, const void *gate_weight, int64_t ldw, int64_t T,
                                         int32_t H, int32_t E, int32_t k, int dtype, void *logits, int64_t ldl,
                                         void *weights, void *ids, int ids_is_i64, void *stream) {
    XMA_REQUIRE(dtype == XMA_ROCM_BF16 || dtype == XMA_ROCM_F16, XMA_ROCM_EUNSUPPORTED,
                "router_gate_topk: dtype %d (bf16 and fp16 only; fp32 goes through a linear layer and xma_rocm_router_topk)",
                dtype);
    XMA_REQUIRE(T >= 0 && H >= 8 && E >= 1 && k >= 1 && k <= E, XMA_ROCM_EINVAL,
                "router_gate_topk: T=%lld H=%d E=%d k=%d (1 <= k <= E)", (long long)T, H, E, k);
    XMA_REQUIRE(E <= RG_MAX_E && k <= RG_MAX_K && H % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0, XMA_ROCM_EUNSUPPORTED,
                "router_gate_topk: E=%d k=%d H=%d ldx=%lld ldw=%lld (E <= %d, k <= %d, H and ld %% 8 == 0)", E, k, H,
                (long long)ldx, (long long)ldw, RG_MAX_E, RG_MAX_K);
    XMA_REQUIRE(ldx >= H && ldw >= H && ldl >= E, XMA_ROCM_EINVAL, "router_gate_topk: leading dimension shorter than a row");
    if (T == 0) return XMA_ROCM_OK;
    XMA_REQUIRE(x && gate_weight && logits && weights && ids && ((uintptr_t)x & 15) == 0 && ((uintptr_t)gate_weight & 15) == 0,
                XMA_ROCM_EINVAL, "router_gate_topk: null or misaligned pointer");
    XMA_REQUIRE((T + RG_TOKENS - 1) / RG_TOKENS < ((int64_t)1 << 31), XMA_ROCM_EUNSUPPORTED, "router_gate_topk: too many rows");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == XMA_ROCM_BF16)
        return router_gate_launch<__bf16, XMA_ROCM_BF16>(x, ldx, gate_weight, ldw, T, H, E, k, logits, ldl, weights, ids,
                                                         ids_is_i64, st);
    return router_gate_launch<_Float16, XMA_ROCM_F16>(x, ldx, gate_weight, ldw, T, H, E, k, logits, ldl, weights, ids,
                                                      ids_is_i64, st);
}

extern "C" int xma_rocm_router_topk_bwd(const void *logits, int64_t ld, int64_t T, int32_t E, int32_t k, int dtype,
                                        const void *ids, int ids_is_i64, const void *d_weights, void *d_logits,
                                        int64_t ldd, void *stream) {
    RouterShape s;
    if (int rc = router_shape("router_topk_bwd", T, E, k, dtype, s)) return rc;
    XMA_REQUIRE(ld >= E && ldd >= E, XMA_ROCM_EINVAL, "router_topk_bwd: ld=%lld ldd=%lld < E=%d", (long long)ld,
                (long long)ldd, E);
    XMA_REQUIRE(T == 0 || (logits && ids && d_weights && d_logits), XMA_ROCM_EINVAL, "router_topk_bwd: null pointer");
    if (T == 0) return XMA_ROCM_OK;
    hipStream_t st = (hipStream_t)stream;
    ROUTER_DISPATCH(dtype, s, (router_topk_bwd_kernel<DT, G, VPL><<<(int)s.blocks, RT_THREADS, 0, st>>>(
                                  logits, ld, T, E, k, ids, ids_is_i64, d_weights, d_logits, ldd)));
    return xma_check_launch("router_topk_bwd_kernel");
}
