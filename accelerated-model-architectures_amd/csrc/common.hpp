// Shared device helpers for the gfx950 (CDNA4) MoE kernels: element traits for
// bf16/fp16, MFMA wrappers, the LDS tile swizzle and the thread-local error slot.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "xma_rocm.h"

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define WAVE 64

// ---------------------------------------------------------------- error slot
void xma_set_error(const char *fmt, ...);
int xma_check_launch(const char *what);
// hipFuncSetAttribute(MaxDynamicSharedMemorySize) on the first call per (kernel, device); later calls only look it up
int xma_set_max_lds_once(const void *kernel, int bytes);

#define XMA_REQUIRE(cond, code, ...)   \
    do {                               \
        if (!(cond)) {                 \
            xma_set_error(__VA_ARGS__); \
            return (code);             \
        }                              \
    } while (0)

// ---------------------------------------------------------------- division by a launch constant
// exact n / d for 0 <= n < 2^31 in three 32-bit instructions: with s = ceil(log2 d) and magic = ceil(2^(31+s) / d)
// (which fits 32 bits), n / d = mulhi(2 n, magic) >> s
struct FastDiv {
    uint32_t magic;
    int shift;
};
inline FastDiv make_fastdiv(uint32_t d) {
    int s = 0;
    while ((1u << s) < d) ++s;
    FastDiv f;
    f.shift = s;
    f.magic = (uint32_t)((((uint64_t)1 << (31 + s)) + d - 1) / d);
    return f;
}
__device__ __forceinline__ uint32_t fastdiv(uint32_t n, FastDiv f) { return __umulhi(n << 1, f.magic) >> f.shift; }

// Index of a lane's piece of work -> (row, piece inside the row) for rows of `per_row` pieces: the multiply-high form
// while the index fits 31 bits, the 64-bit division (a hundred instructions) only beyond that.
__device__ __forceinline__ void split_row(int64_t g, int per_row, FastDiv d, int64_t &row, int &piece) {
    if (g < ((int64_t)1 << 31)) {
        const uint32_t r = fastdiv((uint32_t)g, d);
        row = r;
        piece = (int)((uint32_t)g - r * (uint32_t)per_row);
    } else {
        row = g / per_row;
        piece = (int)(g % per_row);
    }
}

// ---------------------------------------------------------------- element traits
template <typename T> struct Elem;

template <> struct Elem<__bf16> {
    static __device__ __forceinline__ float to_f(uint32_t bits16) { return __builtin_bit_cast(float, bits16 << 16); }
    static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
    // two floats -> packed pair, round to nearest even
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        bf16x2 v;
        v[0] = (__bf16)a;
        v[1] = (__bf16)b;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    }
};

template <> struct Elem<_Float16> {
    static __device__ __forceinline__ float lo(uint32_t w) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
    }
    static __device__ __forceinline__ float hi(uint32_t w) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
    }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        f16x2 v;
        v[0] = (_Float16)a;
        v[1] = (_Float16)b;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
    }
};

// ---------------------------------------------------------------- LDS tile layout
// An operand tile is [rows][64 k] of 16-bit elements = 8 chunks of 16 bytes per
// row.  Chunk c of row r lives at chunk slot c ^ swz(r).  Mixing in row>>3 keeps
// the transposing loader (which writes rows 8 apart from neighbouring lanes)
// conflict free as well as the MFMA fragment reads (32 consecutive rows).
__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }
__device__ __forceinline__ int lds_chunk(int row, int chunk) { return row * 8 + (chunk ^ swz(row)); }

// 8x8 transpose of 16-bit elements held as 8 row vectors of 4 dwords:
// out[c] (c = column 0..7) = the 8 values of column c, one per input row.
__device__ __forceinline__ void transpose8x8_b16(const u32x4 in[8], u32x4 out[8]) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t a = in[2 * q][w], b = in[2 * q + 1][w];
            // plain bit operations; the compiler folds each line into one v_perm_b32
            out[2 * w][q] = (a & 0xffffu) | (b << 16);
            out[2 * w + 1][q] = (a >> 16) | (b & 0xffff0000u);
        }
    }
}

// v_exp_f32 and v_rcp_f32 (1 ulp each) instead of an IEEE division: the result is rounded to 16 bits anyway
__device__ __forceinline__ float sigmoidf_fast(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
