// Backward dynamic-mask attention for gfx950, general form (mask and / or bias vary per query row): the dQ kernel.
//
// Third kernel of the backward pass (see fdma_bwd.hip): one workgroup per (128-query block, batch, head) loops over
// the key tiles like the forward kernel and computes, per 64-key tile,
//     S^T = K Q^T (+ bias, mask),  P^T = exp2(S^T - LSE),  dP^T = V dO^T,  dS^T = P^T o (dP^T - D),  dQ^T += K^T dS^T
// -- the dQ part of compute_dq_dk_dv_1colblock (csrc/flash_sparse_attn/src/flash_bwd_kernel.h:79-1142 of the
// reference), with Q-stationary accumulation instead of fp32 atomics into a dQ workspace plus a convert pass
// (flash_bwd_kernel.h:940, flash_bwd_preprocess_kernel.h:212-304).
//
// Like the general forward kernel (fdma_fwd.hip) it is built around the mask / bias stream, which bounds this path:
// coalesced loads of every 128 x 64 mask and bias tile, fused in registers into one 16-bit tile in LDS that the score
// accumulators start from; K, V and the fused tile double-buffered and fetched a tile ahead, the mask two tiles
// ahead so that a tile without any kept element costs its mask bytes only; one barrier per tile (the OR reduction).
#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

namespace {

// Workgroups have 4 waves (128 query rows; two per CU at d <= 64) or, at d = 128 on grids that stay large enough,
// 8 waves (256 rows): one workgroup fits on a CU there, and a second wave per SIMD hides what a single wave's
// in-order issue cannot.  Key tiles have 64 keys with 4 waves and 32 with 8 (the 64-key tile's score and dP accumulators
// do not fit next to dQ and the Q / dO fragments in the 256 registers a wave has when two share a SIMD).
template <int D, int BM, int BN> struct DqSmem {
    static constexpr int S = D + 8;      // K / V tile row stride (elements)
    static constexpr int SF = BN + 8;    // fused mask+bias tile row stride
    static constexpr int K_BYTES = BN * S * 2;
    static constexpr int F_BYTES = BM * SF * 2;
    static constexpr int STAGE = 2 * K_BYTES + F_BYTES;
    static constexpr int TOTAL = 2 * STAGE;
};

template <typename T> struct NegInf2;
template <> struct NegInf2<bf16_tag> { static constexpr uint32_t value = 0xFF80FF80u; };
template <> struct NegInf2<fp16_tag> { static constexpr uint32_t value = 0xFC00FC00u; };

template <typename T, int D, bool CAUSAL, int NW>
__global__ void __launch_bounds__(64 * NW, (D <= 64 && NW == 4) ? 2 : 1) bwd_dq_kernel(const BwdParams p) {
    constexpr int NTHREADS = 64 * NW, BM = 32 * NW, BN = (NW == 8 || D > 128) ? 32 : 64;
    constexpr int FCH = BN / 8;             // 8-key chunks per mask / bias row of a tile
    constexpr int F_RPP = NTHREADS / FCH;   // mask / bias rows staged per pass
    using E = Elem<T>;
    using SM = DqSmem<D, BM, BN>;
    constexpr int KS = D / 16, DB = D / 32, MB = BN / 32, KB = BN / 16;
    constexpr int CH = D / 8;               // 16-byte chunks per K / V row
    constexpr int K_RPP = NTHREADS / CH;    // rows staged per pass
    constexpr int K_IT = BN / K_RPP;
    constexpr int F_IT = BM * FCH / NTHREADS;  // 8-key chunks of the mask / bias tile per thread

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const FwdParams &f = p.f;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, g = lane >> 5;
    // linear workgroup id -> (query block, head, batch) with the query block OUTERMOST and descending: under causal
    // masking the blocks with the most KV tiles of every head start first, the light ones fill the tail
    const int hb_count = f.H * f.B;
    const int m_block = (int)gridDim.x / hb_count - 1 - (int)blockIdx.x / hb_count;
    const int h = ((int)blockIdx.x % hb_count) % f.H, b = ((int)blockIdx.x % hb_count) / f.H;
    const int hk = h / (f.H / f.Hk);
    const int m0 = m_block * BM;
    const int wrow0 = m0 + wave * 32;
    const int qrow = wrow0 + r;
    const int qrow_c = qrow < f.Lq ? qrow : f.Lq - 1;
    const int shift = f.Lk - f.Lq;

    // ---- Q (scaled by softmax_scale * log2(e): it only feeds the scores here) and dO fragments, row statistics
    u32x4_t qf[KS], dof[KS];
    {
        const uint16_t *qp = (const uint16_t *)f.q + b * f.q_b + (int64_t)qrow_c * f.q_r + h * f.q_h;
        const uint16_t *dp = (const uint16_t *)p.dout + b * p.do_b + (int64_t)qrow_c * p.do_r + h * p.do_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + g * 8;
            u32x4_t qv = {0, 0, 0, 0}, dv = {0, 0, 0, 0};
            if (qrow < f.Lq && c < f.d) { qv = *(const u32x4_t *)(qp + c); dv = *(const u32x4_t *)(dp + c); }
#pragma unroll
            for (int e = 0; e < 4; e++) qv[e] = E::pack2(E::lo(qv[e]) * f.scale_log2, E::hi(qv[e]) * f.scale_log2);
            qf[ks] = qv;
            dof[ks] = dv;
        }
    }
    float lse2 = INFINITY, dd = 0.f;
    if (qrow < f.Lq) {
        lse2 = f.lse[((int64_t)b * f.H + h) * f.Lq + qrow] * kLog2e;
        dd = p.softmax_d[((int64_t)b * f.H + h) * p.Lq_rounded + qrow];
    }

    int n_end = (f.Lk + BN - 1) / BN;
    if (CAUSAL) {
        int lim = m0 + BM + shift;
        if (lim > f.Lq + shift) lim = f.Lq + shift;
        if (lim < 0) lim = 0;
        const int ne = (lim + BN - 1) / BN;
        if (ne < n_end) n_end = ne;
    }

    f32x16_t dq[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) dq[db][i] = 0.f;

    const int hm = f.mask ? (f.Hm == f.H ? h : (f.Hm == 1 ? 0 : h / (f.H / f.Hm))) : 0;
    const int hb = f.bias ? (f.Hb == f.H ? h : (f.Hb == 1 ? 0 : h / (f.H / f.Hb))) : 0;
    const uint8_t *mbase = f.mask ? f.mask + b * f.m_b + hm * f.m_h : nullptr;
    const uint16_t *bbase = f.bias ? (const uint16_t *)f.bias + b * f.bi_b + hb * f.bi_h : nullptr;
    const uint16_t *kbase = (const uint16_t *)f.k + b * f.k_b + hk * f.k_h;
    const uint16_t *vbase = (const uint16_t *)f.v + b * f.v_b + hk * f.v_h;

    // ---- staging maps; all tile loads are unconditional, from clamped (always valid) addresses: rows of K / V beyond
    // Lk and head-dim chunks beyond d are finite duplicates that meet a -inf score or a zero fragment, and the mask
    // words are ANDed with a validity pattern when they are consumed
    const int kc = tid % CH, kr0 = tid / CH;
    const int kcol = kc * 8 < f.d ? kc * 8 : 0;
    const int fc = tid % FCH, fr0 = tid / FCH;  // mask / bias: 8-key chunk, first row (rows fr0 + F_RPP it)
    u32x4_t kreg[K_IT], vreg[K_IT], breg[F_IT];
    u32x2_t mreg[F_IT], mnext[F_IT];

    // (a mask that comes packed to bits: one byte per 8-key chunk instead of eight, expanded where it is looked at)
    const uint8_t *mbits = (mbase && f.mbits) ? f.mbits + b * f.mb_b + hm * f.mb_h : nullptr;
    auto load_mask = [&](int j, u32x2_t (&dst)[F_IT]) {
        if (!mbase) return;
        int kk = j * BN + 8 * fc;
        kk = kk < f.Lk ? kk : 0;
#pragma unroll
        for (int it = 0; it < F_IT; it++) {
            int row = m0 + fr0 + F_RPP * it;
            row = row < f.Lq ? row : f.Lq - 1;
            // (one 8-byte load either way, from an address chosen without a branch: mask bytes of the chunk, or the
            // aligned piece of the bit row that holds the chunk's byte)
            const uint8_t *src = mbits ? mbits + (int64_t)row * f.mb_r + ((kk >> 3) & ~7) : mbase + (int64_t)row * f.m_r + kk;
            dst[it] = *(const u32x2_t *)src;
        }
    };
    auto finish_mask = [&](int j, u32x2_t (&dst)[F_IT]) -> bool {
        const int kk = j * BN + 8 * fc;
        uint32_t any = 0;
#pragma unroll
        for (int it = 0; it < F_IT; it++) {
            const int row = m0 + fr0 + F_RPP * it;
            u32x2_t mv = mbase ? (mbits ? mask_bits_to_bytes(mask_bits_byte(dst[it], kk)) : dst[it]) : u32x2_t{0x01010101u, 0x01010101u};
            const bool ok = row < f.Lq && kk < f.Lk && !(CAUSAL && kk > row + shift);
            uint64_t keepm = ok ? ~0ull : 0ull;
            if (kk + 8 > f.Lk && kk < f.Lk) keepm = (1ull << (8 * (f.Lk - kk))) - 1ull;
            mv[0] &= (uint32_t)keepm;
            mv[1] &= (uint32_t)(keepm >> 32);
            dst[it] = mv;
            any |= mv[0] | mv[1];
        }
        return any != 0;
    };
    auto load_rest = [&](int j) {
        const int n0 = j * BN;
        if (bbase) {
            int kk = n0 + 8 * fc;
            kk = kk < f.Lk ? kk : 0;
#pragma unroll
            for (int it = 0; it < F_IT; it++) {
                int row = m0 + fr0 + F_RPP * it;
                row = row < f.Lq ? row : f.Lq - 1;
                breg[it] = *(const u32x4_t *)(bbase + (int64_t)row * f.bi_r + kk);
            }
        } else {
#pragma unroll
            for (int it = 0; it < F_IT; it++) breg[it] = u32x4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int it = 0; it < K_IT; it++) {
            int key = n0 + kr0 + it * K_RPP;
            key = key < f.Lk ? key : f.Lk - 1;
            kreg[it] = *(const u32x4_t *)(kbase + (int64_t)key * f.k_r + kcol);
            vreg[it] = *(const u32x4_t *)(vbase + (int64_t)key * f.v_r + kcol);
        }
    };
    auto store_stage = [&](int buf, const u32x2_t (&mv)[F_IT]) {
        char *sK = smem + buf * SM::STAGE;
        char *sV = sK + SM::K_BYTES;
        char *sF = sV + SM::K_BYTES;
#pragma unroll
        for (int it = 0; it < K_IT; it++) {
            const int off = ((kr0 + it * K_RPP) * SM::S + kc * 8) * 2;
            *(u32x4_t *)(sK + off) = kreg[it];
            *(u32x4_t *)(sV + off) = vreg[it];
        }
#pragma unroll
        for (int it = 0; it < F_IT; it++) {
            u32x4_t bv = breg[it];
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                uint32_t x = mv[it][hlf];
                x = ((((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) >> 7) & 0x01010101u;  // nonzero byte -> 0x01
                const uint32_t z = (x << 8) - x;                                      // 0x01 -> 0xFF per byte
                const uint32_t m0w = __builtin_amdgcn_perm(0, z, 0x01010000u);        // [b0 b0 b1 b1]
                const uint32_t m1w = __builtin_amdgcn_perm(0, z, 0x03030202u);        // [b2 b2 b3 b3]
                bv[2 * hlf] = (bv[2 * hlf] & m0w) | (NegInf2<T>::value & ~m0w);
                bv[2 * hlf + 1] = (bv[2 * hlf + 1] & m1w) | (NegInf2<T>::value & ~m1w);
            }
            *(u32x4_t *)(sF + ((fr0 + F_RPP * it) * SM::SF + 8 * fc) * 2) = bv;
        }
    };

    const int a_row = pi_row(r);
    const uint32_t a_off = (uint32_t)((a_row * SM::S + g * 8) * 2);
    const int tj = lane & 15, te = tj >> 2, tc = tj & 3;
    const int tcp = (tc == 1) ? 2 : (tc == 2 ? 1 : tc);
    const int tdh = (lane >> 4) & 1;
    const uint32_t tr_off = (uint32_t)(((8 * g + te) * SM::S + 16 * tdh + 4 * tcp) * 2);

    auto compute = [&](int j, int buf) {
        const int n0 = j * BN;
        const char *sK = smem + buf * SM::STAGE;
        const char *sV = sK + SM::K_BYTES;
        const char *sF = sV + SM::K_BYTES + ((wave * 32 + r) * SM::SF + 8 * g) * 2;
        // ---- S^T = K Q^T on top of the fused mask+bias tile, dP^T = V dO^T
        f32x16_t s[MB], dp[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                const u32x4_t fv = *(const u32x4_t *)(sF + (32 * mb + 16 * blk) * 2);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    s[mb][8 * blk + 2 * e] = E::lo(fv[e]) * kLog2e;
                    s[mb][8 * blk + 2 * e + 1] = E::hi(fv[e]) * kLog2e;
                    dp[mb][8 * blk + 2 * e] = 0.f;
                    dp[mb][8 * blk + 2 * e + 1] = 0.f;
                }
            }
        {
            constexpr int NF = 2 * MB * KS, FR = 8;  // fragment fi: (ks, mb, which) with which = 0: K, 1: V
            u32x4_t a[NF];
            auto frag = [&](int fi) {
                const int which = fi & 1, mb = (fi >> 1) % MB, ks = (fi >> 1) / MB;
                return *(const u32x4_t *)((which ? sV : sK) + a_off + (32 * mb * SM::S + ks * 16) * 2);
            };
#pragma unroll
            for (int fi = 0; fi < FR; fi++) a[fi] = frag(fi);
#pragma unroll
            for (int fi = 0; fi < NF; fi++) {
                if (fi + FR < NF) a[fi + FR] = frag(fi + FR);
                const int which = fi & 1, mb = (fi >> 1) % MB, ks = (fi >> 1) / MB;
                if (which) dp[mb] = E::mfma(a[fi], dof[ks], dp[mb]);
                else s[mb] = E::mfma(a[fi], qf[ks], s[mb]);
            }
        }
        // ---- dS^T = P^T o (dP^T - D); causal selects on diagonal tiles only (wave-uniform branch)
        const bool diag = CAUSAL && (n0 + BN - 1 > wrow0 + shift);
        uint32_t dpk[8 * MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                float pv[8];
#pragma unroll
                for (int e = 0; e < 8; e++) pv[e] = fast_exp2(s[mb][8 * blk + e] - lse2);
                if (diag) {
                    asm volatile("" ::: "memory");
                    const int lim = qrow + shift - n0 - 32 * mb - 16 * blk - 8 * g;  // local columns e <= lim are visible
#pragma unroll
                    for (int e = 0; e < 8; e++) pv[e] = e <= lim ? pv[e] : 0.f;
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float d0 = pv[2 * e] * (dp[mb][8 * blk + 2 * e] - dd);
                    const float d1 = pv[2 * e + 1] * (dp[mb][8 * blk + 2 * e + 1] - dd);
                    dpk[8 * mb + 4 * blk + e] = E::pack2(d0, d1);
                }
            }
        // ---- dQ^T += K^T dS^T  (K^T through transposing LDS reads of the row-major K tile, one pair ahead)
        {
            constexpr int NP = KB * DB;
            u32x4_t a[2];
            auto frag = [&](int idx, int slot) {
                const int kb = idx / DB, db = idx % DB;
                const uint32_t off = tr_off + (uint32_t)((16 * kb * SM::S + 32 * db) * 2);
                const u32x2_t lo = lds_read_tr16(sK, off), hi = lds_read_tr16(sK, off + 4 * SM::S * 2);
                a[slot] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
            };
            frag(0, 0);
#pragma unroll
            for (int idx = 0; idx < NP; idx++) {
                if (idx + 1 < NP) frag(idx + 1, (idx + 1) & 1);
                const int kb = idx / DB, db = idx % DB;
                const u32x4_t bop = {dpk[4 * kb], dpk[4 * kb + 1], dpk[4 * kb + 2], dpk[4 * kb + 3]};
                dq[db] = E::mfma(a[idx & 1], bop, dq[db]);
            }
        }
    };

    // ---- main loop.  At the top of iteration j: tile j sits in LDS stage j&1 if it is active, the mask of tile j+1 is
    // in registers (finished) and `act_next` says whether that tile has any kept element.
    if (n_end > 0) {
        load_mask(0, mreg);
        if (n_end > 1) load_mask(1, mnext);
        bool act_cur = __syncthreads_or(finish_mask(0, mreg));
        if (act_cur) {
            load_rest(0);
            store_stage(0, mreg);
        }
        bool act_next = __syncthreads_or(n_end > 1 && finish_mask(1, mnext));
        auto step = [&](int j, u32x2_t (&m_next)[F_IT], u32x2_t (&m_new)[F_IT]) {
            const bool have_next = j + 1 < n_end && act_next;
            if (have_next) load_rest(j + 1);
            if (j + 2 < n_end) load_mask(j + 2, m_new);
            __builtin_amdgcn_sched_barrier(0);  // loads above, their first use below the compute
            if (act_cur) compute(j, j & 1);
            __builtin_amdgcn_sched_barrier(0);
            if (have_next) store_stage((j + 1) & 1, m_next);
            const bool act_nn = __syncthreads_or(j + 2 < n_end && finish_mask(j + 2, m_new));
            act_cur = have_next;
            act_next = act_nn;
        };
        for (int j = 0; j < n_end; j += 2) {
            step(j, mnext, mreg);
            if (j + 1 < n_end) step(j + 1, mreg, mnext);
        }
    }

    if (qrow < f.Lq) {
        uint16_t *dqp = (uint16_t *)p.dq + b * p.dq_b + (int64_t)qrow * p.dq_r + h * p.dq_h;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                const int c = 32 * db + 16 * blk + 8 * g;
                if (c < f.d) {
                    u32x4_t w;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        w[e] = E::pack2(dq[db][8 * blk + 2 * e] * f.scale, dq[db][8 * blk + 2 * e + 1] * f.scale);
                    *(u32x4_t *)(dqp + c) = w;
                }
            }
    }
}

template <typename T, int D, bool CAUSAL, int NW>
hipError_t launch_dq_n(const BwdParams &p, hipStream_t stream) {
    constexpr int BM = 32 * NW, NTHREADS = 64 * NW, BN = (NW == 8 || D > 128) ? 32 : 64;
    auto kern = bwd_dq_kernel<T, D, CAUSAL, NW>;
    const int smem = DqSmem<D, BM, BN>::TOTAL;
    static DynSmemLimit smem_limit;
    hipError_t e = smem_limit.ensure((const void *)kern, (int)smem);
    if (e != hipSuccess) return e;
    dim3 grid(((p.f.Lq + BM - 1) / BM) * p.f.H * p.f.B);
    hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), smem, stream, p);
    return hipGetLastError();
}

template <typename T, int D, bool CAUSAL>
hipError_t launch_dq_c(const BwdParams &p, hipStream_t stream) {
    if constexpr (D > 64 && D <= 128) {
        // 256-row workgroups while the grid still covers the chip about twice
        if ((int64_t)p.f.B * p.f.H * ((p.f.Lq + 255) / 256) >= 512) return launch_dq_n<T, D, CAUSAL, 8>(p, stream);
    }
    return launch_dq_n<T, D, CAUSAL, 4>(p, stream);
}

}  // namespace

hipError_t launch_bwd_dq(const BwdParams &p, int dtype, hipStream_t stream) {
    // head dims up to 64 / 128 / 256 (a head dim in between runs in the next larger instantiation)
    const int dc = p.f.d <= 64 ? 0 : (p.f.d <= 128 ? 1 : 2);
    const bool c = p.f.causal != 0;
    if (dtype == 0) {
        if (dc == 0) return c ? launch_dq_c<bf16_tag, 64, true>(p, stream) : launch_dq_c<bf16_tag, 64, false>(p, stream);
        if (dc == 1) return c ? launch_dq_c<bf16_tag, 128, true>(p, stream) : launch_dq_c<bf16_tag, 128, false>(p, stream);
        return c ? launch_dq_c<bf16_tag, 256, true>(p, stream) : launch_dq_c<bf16_tag, 256, false>(p, stream);
    }
    if (dc == 0) return c ? launch_dq_c<fp16_tag, 64, true>(p, stream) : launch_dq_c<fp16_tag, 64, false>(p, stream);
    if (dc == 1) return c ? launch_dq_c<fp16_tag, 128, true>(p, stream) : launch_dq_c<fp16_tag, 128, false>(p, stream);
    return c ? launch_dq_c<fp16_tag, 256, true>(p, stream) : launch_dq_c<fp16_tag, 256, false>(p, stream);
}

}  // namespace fdma
