// D = rowsum(dO * O), the first step of the backward (softmax_d; padded rows are zero): the work of one 256-thread
// block, shared by the stand-alone kernel and by the compacted backward's pre-pass launch.
#pragma once

#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

// rows one block covers (8 or 16 lanes cooperate on a row of d elements)
__host__ __device__ inline int bwd_dot_rows_per_block(int d) { return (d + 7) / 8 <= 8 ? 32 : 16; }

template <typename T>
__device__ __forceinline__ void bwd_dot_block(const BwdParams &p, int block_x, int h, int b) {
    using E = Elem<T>;
    const int CH = (p.f.d + 7) / 8;               // 16-byte chunks per row
    const int lanes = CH <= 8 ? 8 : 16;           // lanes cooperating on one row (power of two)
    const int rows_per_block = 256 / lanes;
    const int sub = threadIdx.x % lanes;
    const int row = block_x * rows_per_block + threadIdx.x / lanes;
    // a ragged batch is one run of total_q rows (its batch strides are 0 and the grid has one batch entry)
    const int n_rows = p.f.cu_q ? p.f.total_q : p.f.Lq, n_out = p.f.cu_q ? p.f.total_q : p.Lq_rounded;
    float acc = 0.f;
    if (row < n_rows) {
        const uint16_t *op = (const uint16_t *)p.f.o + b * p.f.o_b + (int64_t)row * p.f.o_r + h * p.f.o_h;
        const uint16_t *dp = (const uint16_t *)p.dout + b * p.do_b + (int64_t)row * p.do_r + h * p.do_h;
        for (int c = sub; c < CH; c += lanes) {
            u32x4_t ov = *(const u32x4_t *)(op + c * 8);
            u32x4_t dv = *(const u32x4_t *)(dp + c * 8);
#pragma unroll
            for (int e = 0; e < 4; e++) acc += E::lo(ov[e]) * E::lo(dv[e]) + E::hi(ov[e]) * E::hi(dv[e]);
        }
    }
    for (int off = lanes / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (sub == 0 && row < n_out) p.softmax_d[b * p.sd_b + h * p.sd_h + row] = acc;
}

}  // namespace fdma
