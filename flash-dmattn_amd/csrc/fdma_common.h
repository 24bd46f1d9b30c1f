// Shared device-side helpers for the gfx950 dynamic-mask attention kernels.
//
// Register-tile conventions used by every kernel in this directory
// (v_mfma_f32_32x32x16_{bf16,f16}, wave64, lane l, r = l % 32, g = l / 32):
//   A operand  : lane supplies A[m = r][k = 8g .. 8g+7]            (8 x 16-bit = 16 bytes)
//   B operand  : lane supplies B[k = 8g .. 8g+7][n = r]
//   C/D        : lane holds D[m = 8*(i/4) + 4g + i%4][n = r], i = 0..15
// Rows of the A tile are fetched through the permutation pi() below, so that register i of the
// accumulator corresponds to the tile row 16*(i/8) + 8g + i%8: eight consecutive rows per lane.
// That makes an accumulator directly usable as the B operand of a following MFMA whose
// contraction index is that row index (registers 8*blk..8*blk+7 <-> k = 8g..8g+7 of the
// 16-wide contraction block blk), with no cross-lane traffic.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fdma {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

struct bf16_tag {};
struct fp16_tag {};

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// tile row held by MFMA row m  (see header comment)
__device__ __forceinline__ int pi_row(int m) {
    int a = m >> 3, gp = (m >> 2) & 1, c = m & 3;
    return 16 * (a >> 1) + 8 * gp + 4 * (a & 1) + c;
}

template <typename T> struct Elem;

template <> struct Elem<bf16_tag> {
    static __device__ __forceinline__ f32x16_t mfma(u32x4_t a, u32x4_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f32x2_t f = {lo, hi};
        bf16x2_t h = __builtin_convertvector(f, bf16x2_t);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ float lo(uint32_t u) { return __uint_as_float(u << 16); }
    static __device__ __forceinline__ float hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
};

template <> struct Elem<fp16_tag> {
    static __device__ __forceinline__ f32x16_t mfma(u32x4_t a, u32x4_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f32x2_t f = {lo, hi};
        f16x2_t h = __builtin_convertvector(f, f16x2_t);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ float lo(uint32_t u) {
        f16x2_t h = __builtin_bit_cast(f16x2_t, u);
        return (float)h[0];
    }
    static __device__ __forceinline__ float hi(uint32_t u) {
        f16x2_t h = __builtin_bit_cast(f16x2_t, u);
        return (float)h[1];
    }
};

typedef __attribute__((address_space(3))) char lds_char_t;
typedef __attribute__((address_space(3))) s16x4_t lds_s16x4_t;

// Transposing LDS read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane j = 4e + c
// supplies the address of four consecutive 16-bit elements: row e, columns 4c..4c+3 of a
// 4 x 16 block; lane i of the group receives column i of that block (rows 0..3).
__device__ __forceinline__ u32x2_t lds_read_tr16(const char *smem_base, uint32_t byte_off) {
    const lds_char_t *p = (const lds_char_t *)smem_base + byte_off;
    s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t *)p);
    return __builtin_bit_cast(u32x2_t, v);
}

// max / sum across the two 32-lane halves of a wave (lanes l and l ^ 32)
__device__ __forceinline__ float xhalf_max(float x) {
    uint32_t u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
    uint32_t u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

}  // namespace fdma
