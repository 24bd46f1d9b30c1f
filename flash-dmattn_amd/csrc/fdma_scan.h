// Ordered list of the kept columns of one keep-mask row, with inclusive prefix counts: the form in which the
// attention kernels consume a query-broadcast mask (Compact in fdma_params.h).  Used by the compaction pre-pass
// (fdma_compact.hip) and, as an optional second output, by the keep-mask builder (fdma_mask.hip), whose selection
// then reaches the attention kernels without a second pass over the mask.
#pragma once

#include "fdma_common.h"

namespace fdma {

constexpr int SCAN_KEYS = 16;  // mask bytes per thread per pass

// One workgroup of NT threads (a multiple of 64) walks the row in passes of NT * 16 columns.
//   irow[c]  = original column of the c-th kept key (ascending), c < *count_out
//   crow[j]  = kept keys among the columns 0 .. j (inclusive), written for j < round_up(Lk, 16): the row has room
//   s_wave   : NT / 64 ints of LDS
// `padded`: the mask row is readable in 16-byte pieces up to round_up(Lk, 16) and 16-byte aligned (the attention
// entry points require that of their masks); otherwise the last, partial piece is read byte by byte.
template <int NT>
__device__ __forceinline__ void scan_mask_row(const uint8_t *mrow, int Lk, int32_t *irow, int32_t *crow,
                                              int32_t *count_out, int *s_wave, bool padded) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool vec = padded || (((uintptr_t)mrow & 15) == 0);
    int base = 0;
    for (int c0 = 0; c0 < Lk; c0 += NT * SCAN_KEYS) {
        const int col = c0 + tid * SCAN_KEYS;
        uint32_t bits = 0;
        if (col < Lk) {
            if (vec && (padded || col + SCAN_KEYS <= Lk)) {
                const u32x4_t mv = *(const u32x4_t *)(mrow + col);
#pragma unroll
                for (int e = 0; e < SCAN_KEYS; e++) {
                    const uint32_t byte = (mv[e >> 2] >> (8 * (e & 3))) & 0xffu;
                    if (byte && col + e < Lk) bits |= 1u << e;
                }
            } else {
                for (int e = 0; e < SCAN_KEYS && col + e < Lk; e++)
                    if (mrow[col + e]) bits |= 1u << e;
            }
        }
        const int n = __builtin_popcount(bits);
        int incl = n;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        int woff = 0, total = 0;
#pragma unroll
        for (int w = 0; w < NT / 64; w++) {
            const int v = s_wave[w];
            if (w < wave) woff += v;
            total += v;
        }
        if (col < Lk) {
            int run = base + woff + incl - n;
            int32_t cv[SCAN_KEYS];
#pragma unroll
            for (int e = 0; e < SCAN_KEYS; e++) {
                if (bits & (1u << e)) irow[run++] = col + e;
                cv[e] = run;
            }
#pragma unroll
            for (int q = 0; q < SCAN_KEYS / 4; q++) {
                u32x4_t w = {(uint32_t)cv[4 * q], (uint32_t)cv[4 * q + 1], (uint32_t)cv[4 * q + 2], (uint32_t)cv[4 * q + 3]};
                *(u32x4_t *)(crow + col + 4 * q) = w;  // (the row stride is a multiple of 16)
            }
        }
        base += total;
        __syncthreads();
    }
    if (tid == 0) *count_out = base;
}

}  // namespace fdma
