// Forward dynamic-mask attention for gfx950.
//
// Replaces compute_attn_1rowblock (csrc/flash_sparse_attn/src/flash_fwd_kernel.h:53-804) with its
// online softmax (src/softmax.h:127-221), masking (src/mask.h:94-161) and mask-tile OR skip
// (src/utils.h:339-352) of the reference.  Same math:
//     S = Q K^T * scale + bias ; S[~mask or non-causal] = -inf ; P = softmax(S) ; O = P V
// with the causal mask aligned bottom-right, O = 0 and LSE = +inf for rows with no visible key.
//
// One workgroup = 4 waves = BM (128) query rows of one (batch, head); each wave owns 32 rows.
// The wave computes the TRANSPOSED score tile S^T = K Q^T with K rows as the MFMA A operand read
// from LDS and its Q rows held in registers as the B operand, so a lane owns one query row and
// the row max / row sum are in-lane reductions plus one cross-half swap.  P^T then feeds
// O^T = V^T P^T straight from the accumulator registers; V^T comes from the row-major V tile in
// LDS through transposing LDS reads.
#include "fdma_common.h"
#include "fdma_params.h"

#include <cstdlib>

namespace fdma {

namespace {

constexpr int BM = 128;
constexpr int BN = 64;
constexpr int NTHREADS = 256;

template <int D> struct FwdSmem {
    static constexpr int SK = D + 8;    // K tile row stride (elements): conflict-free 16-byte row reads
    static constexpr int SV = D + 32;   // V tile row stride: conflict-free transposing reads
    static constexpr int K_BYTES = BN * SK * 2;
    static constexpr int V_BYTES = BN * SV * 2;
    static constexpr int TOTAL = K_BYTES + V_BYTES;
};

// nonzero bytes of x -> bit k of the result is set iff byte k of x != 0
__device__ __forceinline__ uint32_t nz_bytes_to_bits(uint32_t x) {
    uint32_t y = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;  // 0x80 per nonzero byte
    return ((y >> 7) * 0x10204080u) >> 28;
}

template <typename T, int D, bool CAUSAL>
__global__ void __launch_bounds__(NTHREADS, 2) fwd_kernel(const FwdParams p) {
    using E = Elem<T>;
    using SM = FwdSmem<D>;
    constexpr int KS = D / 16;  // contraction steps of Q K^T
    constexpr int DB = D / 32;  // 32-wide blocks of the head dimension

    __shared__ __attribute__((aligned(16))) char smem[SM::TOTAL];
    char *sK = smem;
    char *sV = smem + SM::K_BYTES;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int r = lane & 31;
    const int g = lane >> 5;

    const int m_block = gridDim.x - 1 - blockIdx.x;  // heaviest (most KV tiles) first under causal
    const int h = blockIdx.y;
    const int b = blockIdx.z;
    const int hk = h / (p.H / p.Hk);
    const int m0 = m_block * BM;
    const int qrow = m0 + wave * 32 + r;
    const int qrow_c = qrow < p.Lq ? qrow : p.Lq - 1;
    const int shift = p.Lk - p.Lq;  // bottom-right causal alignment

    // ---- Q fragments (B operand of S^T = K Q^T), kept in registers for the whole KV loop
    u32x4_t qf[KS];
    {
        const uint16_t *qp = (const uint16_t *)p.q + b * p.q_b + (int64_t)qrow_c * p.q_r + h * p.q_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            int c = ks * 16 + g * 8;
            u32x4_t v = {0, 0, 0, 0};
            if (qrow < p.Lq && c < p.d) v = *(const u32x4_t *)(qp + c);
            qf[ks] = v;
        }
    }

    int n_end = (p.Lk + BN - 1) / BN;
    if (CAUSAL) {
        int lim = m0 + BM + shift;  // first invisible column for the last row of the block
        if (lim < 0) lim = 0;
        int ne = (lim + BN - 1) / BN;
        if (ne < n_end) n_end = ne;
    }

    f32x16_t o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    float row_max = -INFINITY;  // log2 domain
    float row_sum = 0.f;        // per-lane partial (this lane's half of the keys)

    const int hm = p.mask ? (p.Hm == p.H ? h : (p.Hm == 1 ? 0 : h / (p.H / p.Hm))) : 0;
    const int hb = p.bias ? (p.Hb == p.H ? h : (p.Hb == 1 ? 0 : h / (p.H / p.Hb))) : 0;
    const uint8_t *mrow = p.mask ? p.mask + b * p.m_b + hm * p.m_h + (int64_t)qrow_c * p.m_r : nullptr;
    const uint16_t *brow = p.bias ? (const uint16_t *)p.bias + b * p.bi_b + hb * p.bi_h + (int64_t)qrow_c * p.bi_r : nullptr;

    const uint16_t *kbase = (const uint16_t *)p.k + b * p.k_b + hk * p.k_h;
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.v_b + hk * p.v_h;

    // A-operand row of this lane inside a 32-row block of K
    const int a_row = pi_row(r);
    // transposing-read supplier coordinates (see lds_read_tr16)
    const int tj = lane & 15, te = tj >> 2, tc = tj & 3;
    const int tcp = (tc == 1) ? 2 : (tc == 2 ? 1 : tc);
    const int tdh = (lane >> 4) & 1;
    const uint32_t v_tr_off = (uint32_t)(((8 * g + te) * SM::SV + 16 * tdh + 4 * tcp) * 2);

    for (int j = 0; j < n_end; j++) {
        const int n0 = j * BN;
        // ---- keep bits of this lane's 32 score elements: bit 16*mb + i  <->  key n0 + 32mb + 16(i/8) + 8g + i%8
        uint32_t keep = 0;
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                int c0 = n0 + 32 * mb + 16 * blk + 8 * g;
                uint32_t bits = 0xffu;
                if (mrow) {
                    bits = 0;
                    if (c0 < p.Lk) {
                        u32x2_t mv = *(const u32x2_t *)(mrow + c0);
                        bits = nz_bytes_to_bits(mv[0]) | (nz_bytes_to_bits(mv[1]) << 4);
                    }
                }
                int lim = p.Lk;
                if (CAUSAL) { int cl = qrow + 1 + shift; lim = cl < lim ? cl : lim; }
                int nvis = lim - c0;  // columns c0 .. c0+nvis-1 visible
                uint32_t vis = nvis >= 8 ? 0xffu : (nvis <= 0 ? 0u : ((1u << nvis) - 1u));
                bits &= vis;
                if (qrow >= p.Lq) bits = 0;
                keep |= bits << (16 * mb + 8 * blk);
            }
        // workgroup-uniform activity; the barrier also fences LDS reuse from the previous tile
        const int active = __syncthreads_or(keep != 0);
        if (!active) continue;

        // ---- stage K and V tiles into LDS (rows beyond Lk are zero-filled)
        {
            constexpr int CH = D / 8;           // 16-byte chunks per row
            constexpr int RPP = NTHREADS / CH;  // rows per pass
            const int c = tid % CH;
            const int r0 = tid / CH;
#pragma unroll
            for (int it = 0; it < BN / RPP; it++) {
                int row = r0 + it * RPP;
                int key = n0 + row;
                u32x4_t kv = {0, 0, 0, 0}, vv = {0, 0, 0, 0};
                if (key < p.Lk && c * 8 < p.d) {
                    kv = *(const u32x4_t *)(kbase + (int64_t)key * p.k_r + c * 8);
                    vv = *(const u32x4_t *)(vbase + (int64_t)key * p.v_r + c * 8);
                }
                *(u32x4_t *)(sK + (row * SM::SK + c * 8) * 2) = kv;
                *(u32x4_t *)(sV + (row * SM::SV + c * 8) * 2) = vv;
            }
        }
        // bias fragment for this lane (log2 domain), fetched while the tile lands
        float bl2[32];
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                int c0 = n0 + 32 * mb + 16 * blk + 8 * g;
                u32x4_t bv = {0, 0, 0, 0};
                if (brow && c0 < p.Lk) bv = *(const u32x4_t *)(brow + c0);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    bl2[16 * mb + 8 * blk + 2 * e] = E::lo(bv[e]) * kLog2e;
                    bl2[16 * mb + 8 * blk + 2 * e + 1] = E::hi(bv[e]) * kLog2e;
                }
            }
        __syncthreads();

        // ---- S^T = K Q^T
        f32x16_t s[2];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
#pragma unroll
            for (int i = 0; i < 16; i++) s[mb][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                u32x4_t a = *(const u32x4_t *)(sK + ((32 * mb + a_row) * SM::SK + ks * 16 + g * 8) * 2);
                s[mb] = E::mfma(a, qf[ks], s[mb]);
            }
        }

        // ---- scale, bias, mask, online softmax (log2 domain)
        float tmax = -INFINITY;
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float x = fmaf(s[mb][i], p.scale_log2, bl2[16 * mb + i]);
                x = ((keep >> (16 * mb + i)) & 1u) ? x : -INFINITY;
                s[mb][i] = x;
                tmax = fmaxf(tmax, x);
            }
        tmax = xhalf_max(tmax);
        const float new_max = fmaxf(row_max, tmax);
        const float safe_max = new_max == -INFINITY ? 0.f : new_max;
        const float alpha = fast_exp2(row_max - safe_max);  // row_max = -inf -> 0
        row_max = new_max;
        float psum = 0.f;
        uint32_t pk[16];
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                float p0 = fast_exp2(s[mb][i] - safe_max);
                float p1 = fast_exp2(s[mb][i + 1] - safe_max);
                psum += p0 + p1;
                pk[8 * mb + i / 2] = E::pack2(p0, p1);
            }
        row_sum = row_sum * alpha + psum;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) o[db][i] *= alpha;

        // ---- O^T += V^T P^T
#pragma unroll
        for (int kb = 0; kb < 4; kb++) {
            u32x4_t bop = {pk[4 * kb], pk[4 * kb + 1], pk[4 * kb + 2], pk[4 * kb + 3]};
#pragma unroll
            for (int db = 0; db < DB; db++) {
                uint32_t off = v_tr_off + (uint32_t)((16 * kb * SM::SV + 32 * db) * 2);
                u32x2_t lo = lds_read_tr16(sV, off);
                u32x2_t hi = lds_read_tr16(sV, off + 4 * SM::SV * 2);
                u32x4_t a = {lo[0], lo[1], hi[0], hi[1]};
                o[db] = E::mfma(a, bop, o[db]);
            }
        }
    }

    // ---- epilogue: normalise, store O and LSE
    const float total = xhalf_sum(row_sum);
    const float inv = total > 0.f ? 1.f / total : 0.f;
    if (qrow < p.Lq) {
        uint16_t *op = (uint16_t *)p.o + b * p.o_b + (int64_t)qrow * p.o_r + h * p.o_h;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                int c = 32 * db + 16 * blk + 8 * g;
                if (c < p.d) {
                    u32x4_t w;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        w[e] = E::pack2(o[db][8 * blk + 2 * e] * inv, o[db][8 * blk + 2 * e + 1] * inv);
                    *(u32x4_t *)(op + c) = w;
                }
            }
        if (g == 0) {
            float lse = total > 0.f ? (row_max + __builtin_amdgcn_logf(total)) * kLn2 : INFINITY;
            p.lse[((int64_t)b * p.H + h) * p.Lq + qrow] = lse;
        }
    }
}

template <typename T, int D>
hipError_t launch_fwd_t(const FwdParams &p, hipStream_t stream) {
    dim3 grid((p.Lq + BM - 1) / BM, p.H, p.B);
    dim3 block(NTHREADS);
    if (p.causal)
        hipLaunchKernelGGL((fwd_kernel<T, D, true>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((fwd_kernel<T, D, false>), grid, block, 0, stream, p);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_fwd(const FwdParams &p, int dtype, hipStream_t stream) {
    if (p.Lq <= 0 || p.B <= 0) return hipSuccess;
    if (fwd_colmask_applicable(p)) {
        return launch_fwd_colmask(p, dtype, 1, stream);
    }
    const bool d64 = p.d <= 64;
    if (dtype == 0) return d64 ? launch_fwd_t<bf16_tag, 64>(p, stream) : launch_fwd_t<bf16_tag, 128>(p, stream);
    return d64 ? launch_fwd_t<fp16_tag, 64>(p, stream) : launch_fwd_t<fp16_tag, 128>(p, stream);
}

}  // namespace fdma
