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
    // acc + lo(pk) + hi(pk) in one instruction (v_dot2c_f32_bf16 with the constant (1, 1))
    static __device__ __forceinline__ float add_pair(uint32_t pk, float acc) {
        const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pk), ones, acc, false);
    }
    // Side-row arithmetic (see fdma_fwd_colmask.hip): an fp32 number x is handed to the MFMA as 16-bit pieces.
    // kPieceScale: the pieces of a bias value hold x * kPieceScale and meet the constant 1 / kPieceScale (keeps the
    // pieces inside the type's range).  kRefWeight: weight of the coarse piece of a reference point.  bf16 has the
    // range of fp32, so both are 1.
    static constexpr float kPieceScale = 1.f, kRefWeight = 1.f, kMaxFinite = 3.3895314e38f;
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
    static __device__ __forceinline__ float add_pair(uint32_t pk, float acc) {
        const f16x2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, pk), ones, acc, false);
    }
    // fp16 ends at 65504: bias pieces hold x / 2 (|bias * log2e| < 94507), the coarse reference piece x / 64
    static constexpr float kPieceScale = 0.5f, kRefWeight = 64.f, kMaxFinite = 65504.f;
};

// Three 16-bit pieces whose sum (in fp32) is x * kPieceScale to the last bit of x (8 or 11 significant bits each);
// a non-finite x goes into the first piece alone.  Returned as {piece0 | piece1 << 16, piece2}.
template <typename T> __device__ __forceinline__ u32x2_t split3(float x) {
    using E = Elem<T>;
    const float u = x * E::kPieceScale;
    const uint32_t w0 = E::pack2(u, 0.f);
    const float r1 = (__builtin_fabsf(u) <= 3.0e38f) ? u - E::lo(w0) : 0.f;
    const uint32_t w1 = E::pack2(r1, 0.f);
    const float r2 = r1 - E::lo(w1);
    u32x2_t out;
    out[0] = (w0 & 0xffffu) | (w1 << 16);
    out[1] = E::pack2(r2, 0.f) & 0xffffu;
    return out;
}

// Reference point of a softmax row as the MFMA sees it: minus the reference in two 16-bit pieces (a, b), worth
// kRefWeight * a + b.  Returns the packed pair (a low, b high) and, in `enc`, the number the pair really stands for.
template <typename T> __device__ __forceinline__ uint32_t encode_ref(float ref, float &enc) {
    using E = Elem<T>;
    const float lim = E::kMaxFinite;
    float a = -ref * (1.f / E::kRefWeight);
    a = fminf(fmaxf(a, -lim), lim);
    const float ra = E::lo(E::pack2(a, 0.f)) * E::kRefWeight;
    float b = -ref - ra;
    b = fminf(fmaxf(b, -lim), lim);
    const uint32_t w = E::pack2(a, b);
    enc = -(E::lo(w) * E::kRefWeight + E::hi(w));
    return w;
}

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

// LDS accesses by absolute byte address.  A lane keeps its part of an address (row, chunk, swizzle) in one register
// that already includes the start of the workgroup's dynamic LDS; what is added to it at compile time then lands
// in the offset field of the instruction.  (XOR-ing compile-time bits below 256 into such an address equals XOR-ing
// them into the offset alone as long as the dynamic LDS starts at a multiple of 256 bytes: declare it aligned(256).)
__device__ __forceinline__ uint32_t lds_addr(const void *p) { return (uint32_t)(uintptr_t)(const lds_char_t *)p; }
__device__ __forceinline__ u32x4_t lds_ld128(uint32_t addr) {
    return *(const __attribute__((address_space(3))) u32x4_t *)(uintptr_t)addr;
}
__device__ __forceinline__ u32x2_t lds_ld_tr16(uint32_t addr) {
    s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t *)(uintptr_t)addr);
    return __builtin_bit_cast(u32x2_t, v);
}
__device__ __forceinline__ uint32_t lds_ld32(uint32_t addr) { return *(const __attribute__((address_space(3))) uint32_t *)(uintptr_t)addr; }
__device__ __forceinline__ void lds_st32(uint32_t addr, uint32_t v) { *(__attribute__((address_space(3))) uint32_t *)(uintptr_t)addr = v; }

// Eight mask bits (key j in bit j, lowest first) to the eight 0 / 1 bytes of the bool mask's form.  (Bits i of a
// nibble times 0x00204081 land on positions 8 i, among others that the mask removes; no two products share a bit.)
__device__ __forceinline__ u32x2_t mask_bits_to_bytes(uint32_t b) {
    u32x2_t r;
    r[0] = ((b & 0xfu) * 0x00204081u) & 0x01010101u;
    r[1] = (((b >> 4) & 0xfu) * 0x00204081u) & 0x01010101u;
    return r;
}

// The byte with the bits of keys kk .. kk+7 (kk a multiple of 8) out of the aligned 8-byte piece of a bit row that
// holds it -- the kernels fetch bits in the same 8-byte loads as mask bytes, so that one instruction serves both forms.
__device__ __forceinline__ uint32_t mask_bits_byte(u32x2_t piece, int kk) {
    const int sh = ((kk >> 3) & 7) * 8;
    return ((sh & 32) ? piece[1] >> (sh & 31) : piece[0] >> sh) & 0xffu;
}

// Row-major LDS tile of 16-bit elements ([row][head dim]) that is read two ways: as MFMA fragments (ds_read_b128:
// lane (r, g) takes the 16 bytes of chunk 2*ks + g of row pi_row(r)) and through transposing reads (lds_read_tr16:
// 16 lanes take four 8-byte pieces of each of four consecutive rows), and written row by row (16 lanes per row).
// At head dim 128 a row is exactly 256 bytes, the width of the LDS banks, and the 16-byte chunks of a row are
// permuted by a XOR with a function of the row: chunk c of row `row` lives at chunk c ^ swz(row) with
// swz(row) = 4*(row & 3) + ((row >> 2) & 3).  Four consecutive rows then sit in four different 64-byte quarters of
// the banks (what the transposing reads need: measured 145 bytes/clk per CU against 60 with rows padded to 272
// bytes) and sixteen consecutive rows in sixteen different chunks (what the fragment reads need: 230 bytes/clk, the
// same as with padding).  Other head dims keep rows padded by 8 elements.
// Offsets are bytes; a "base" is a lane constant, the *_at functions add the compile-time part.
template <int D> struct LdsTile {
    static constexpr bool SWZ = D == 128;
    static constexpr int S = SWZ ? D : D + 8;  // row stride, elements
    static constexpr int ROW_BYTES = S * 2;
    static __device__ __forceinline__ uint32_t swz(int row) { return (uint32_t)(((row & 3) << 2) | ((row >> 2) & 3)); }
    // 16-byte chunk c of a row (tile writes)
    static __device__ __forceinline__ uint32_t chunk(int row, int c) {
        return SWZ ? (uint32_t)row * 256u + ((((uint32_t)c) ^ swz(row)) << 4) : (uint32_t)((row * S + c * 8) * 2);
    }
    // fragment reads: chunk 2*ks + g of `row`; rows 32 apart share the base (add 32 * ROW_BYTES)
    static __device__ __forceinline__ uint32_t frag_base(int row, int g) {
        return SWZ ? (uint32_t)row * 256u + ((((uint32_t)g) ^ swz(row)) << 4) : (uint32_t)((row * S + g * 8) * 2);
    }
    static __device__ __forceinline__ uint32_t frag_at(uint32_t base, int ks) {
        return SWZ ? (base ^ ((uint32_t)ks << 5)) : base + (uint32_t)ks * 32u;
    }
    // transposing reads: lane (g, te, tdh, tcp) supplies row 8*g + te, elements 16*tdh + 4*tcp .. +3 of a 32-element
    // block db, in 16-row block rb; hi = 1: the same four rows further down
    static __device__ __forceinline__ uint32_t tr_base(int g, int te, int tdh, int tcp) {
        return SWZ ? (uint32_t)(8 * g + te) * 256u + (((uint32_t)te << 6) | ((((uint32_t)(2 * tdh + (tcp >> 1))) ^ (uint32_t)(2 * g)) << 4) |
                                                     ((uint32_t)(tcp & 1) << 3))
                   : (uint32_t)(((8 * g + te) * S + 16 * tdh + 4 * tcp) * 2);
    }
    static __device__ __forceinline__ uint32_t tr_at(uint32_t base, int rb, int db, int hi) {
        return SWZ ? (base ^ (((uint32_t)db << 6) | ((uint32_t)hi << 4))) + (uint32_t)(hi * 4 * 256 + rb * 16 * 256)
                   : base + (uint32_t)(((16 * rb + 4 * hi) * S + 32 * db) * 2);
    }
};

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
