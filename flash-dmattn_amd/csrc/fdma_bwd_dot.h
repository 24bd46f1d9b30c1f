// D = rowsum(dO * O), the first step of the backward (softmax_d; padded rows are zero): the work of one 256-thread
// block, shared by the stand-alone kernel and by the compacted backward's pre-pass launch.
#pragma once

#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

// rows one block covers: 8 or 16 lanes cooperate on a row of d elements, and a thread takes DOT_ROWS rows (all its
// loads requested before the first is used: with a single pair of 16-byte loads per thread the launch was a stream of
// 8 KB workgroups, and reached four fifths of what a copy does)
constexpr int DOT_ROWS = 4;
__host__ __device__ inline int bwd_dot_rows_per_block(int d) { return ((d + 7) / 8 <= 8 ? 32 : 16) * DOT_ROWS; }

template <typename T>
__device__ __forceinline__ void bwd_dot_block(const BwdParams &p, int block_x, int h, int b) {
    using E = Elem<T>;
    const int CH = (p.f.d + 7) / 8;               // 16-byte chunks per row
    const int lanes = CH <= 8 ? 8 : 16;           // lanes cooperating on one row (power of two)
    const int rows_per_pass = 256 / lanes;
    const int sub = threadIdx.x % lanes;
    const int row0 = block_x * rows_per_pass * DOT_ROWS + threadIdx.x / lanes;
    // a ragged batch is one run of total_q rows (its batch strides are 0 and the grid has one batch entry)
    const int n_rows = p.f.cu_q ? p.f.total_q : p.f.Lq, n_out = p.f.cu_q ? p.f.total_q : p.Lq_rounded;
    const uint16_t *ob = (const uint16_t *)p.f.o + b * p.f.o_b + h * p.f.o_h;
    const uint16_t *db = (const uint16_t *)p.dout + b * p.do_b + h * p.do_h;
    float acc[DOT_ROWS];
    if (CH <= 2 * lanes) {  // (head dims up to 256: at most two chunks per lane and row)
        u32x4_t ov[DOT_ROWS][2], dv[DOT_ROWS][2];
#pragma unroll
        for (int i = 0; i < DOT_ROWS; i++) {
            const int row = row0 + i * rows_per_pass;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int c = sub + j * lanes;
                const bool on = row < n_rows && c < CH;
                ov[i][j] = on ? *(const u32x4_t *)(ob + (int64_t)row * p.f.o_r + c * 8) : u32x4_t{0, 0, 0, 0};
                dv[i][j] = on ? *(const u32x4_t *)(db + (int64_t)row * p.do_r + c * 8) : u32x4_t{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int i = 0; i < DOT_ROWS; i++) {
            acc[i] = 0.f;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[i] += E::lo(ov[i][j][e]) * E::lo(dv[i][j][e]) + E::hi(ov[i][j][e]) * E::hi(dv[i][j][e]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < DOT_ROWS; i++) {
            const int row = row0 + i * rows_per_pass;
            acc[i] = 0.f;
            if (row < n_rows)
                for (int c = sub; c < CH; c += lanes) {
                    const u32x4_t ov = *(const u32x4_t *)(ob + (int64_t)row * p.f.o_r + c * 8);
                    const u32x4_t dv = *(const u32x4_t *)(db + (int64_t)row * p.do_r + c * 8);
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[i] += E::lo(ov[e]) * E::lo(dv[e]) + E::hi(ov[e]) * E::hi(dv[e]);
                }
        }
    }
#pragma unroll
    for (int i = 0; i < DOT_ROWS; i++) {
        float a = acc[i];
        for (int off = lanes / 2; off > 0; off >>= 1) a += __shfl_xor(a, off);
        const int row = row0 + i * rows_per_pass;
        if (sub == 0 && row < n_out) p.softmax_d[b * p.sd_b + h * p.sd_h + row] = a;
    }
}

}  // namespace fdma
