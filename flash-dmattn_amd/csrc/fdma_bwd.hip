// Backward dynamic-mask attention for gfx950.
//
// Replaces the reference's backward pipeline (csrc/flash_sparse_attn/src/flash_bwd_launch_template.h:71-117):
//   flash_bwd_dot_do_o_kernel                       src/flash_bwd_preprocess_kernel.h:24-162
//   flash_bwd_dq_dk_dv_loop_seqk_parallel_kernel    src/flash_bwd_kernel.h:79-1142
//   flash_bwd_convert_dq_kernel                     src/flash_bwd_preprocess_kernel.h:212-304
// and the host-side GQA / broadcast reductions of mha_bwd (csrc/flash_sparse_attn/flash_api.cpp:970-983, 1027-1047).
//
// Same math, recomputing P from the saved LSE:
//     P = exp(S - LSE) ; dP = dO V^T ; D = rowsum(dO * O) ; dS = P * (dP - D)
//     dQ = scale * dS K ; dK = scale * dS^T Q ; dV = P^T dO ; dBias = dS (summed over broadcast dims)
//
// Different structure: no fp32 dQ accumulator, no atomics on dQ/dK/dV, no expanded GQA buffers.
//   1. bwd_dot_kernel   : D = rowsum(dO * O)
//   2. bwd_dkdv_kernel  : one workgroup per (key block, batch, KV head); K/V stationary, loops over the
//                         query heads of the group and over query blocks; dK, dV and dBias complete in
//                         registers (S is computed un-transposed so a lane owns one key column);
//   3. bwd_dq_kernel    : (fdma_bwd_dq.hip) one workgroup per (query block, batch, head); loops over key blocks like
//                         the forward kernel (transposed scores, a lane owns one query row).
// Work is therefore 7 tile GEMMs instead of 5, in exchange for a deterministic result and no
// read-modify-write traffic.
#include "fdma_common.h"
#include "fdma_params.h"
#include "fdma_bwd_dot.h"

#include <type_traits>

namespace fdma {

namespace {

constexpr int NTHREADS = 256;

// nonzero bytes of x -> bit k of the result is set iff byte k of x != 0
__device__ __forceinline__ uint32_t nz_bytes_to_bits(uint32_t x) {
    uint32_t y = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
    return ((y >> 7) * 0x10204080u) >> 28;
}

// ------------------------------------------------------------------------------------------------
// 1. D = rowsum(dO * O)   (softmax_d, padded rows are zero)
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) bwd_dot_kernel(const BwdParams p) {
    bwd_dot_block<T>(p, blockIdx.x, blockIdx.y, blockIdx.z);
}

// ------------------------------------------------------------------------------------------------
// 2. dK / dV / dBias with a per-query mask and / or bias
// ------------------------------------------------------------------------------------------------
// One workgroup = 128 keys (32 per wave) of one (batch, kv head); K and V stay in registers as MFMA B
// operands.  Per step (64 query rows of one query head) the workgroup stages Q, dO, LSE, D and a FUSED
// bias tile through LDS: fused[q][k] = bias[q][k] where (mask[q][k] and k < Lk), else -inf, built from
// coalesced 16-byte bias / 8-byte mask loads (broadcast dims simply have stride 0).  exp2(-inf) = 0 does
// the masking.  dS goes back through an LDS tile so that dBias is written with coalesced 16-byte stores
// at the bias's own shape.  GSUM: a per-query bias with fewer heads than queries -- dS is summed over the
// query heads of the group in registers first and leaves through a tile of its own.  Otherwise every lane
// writes its dS over the fused-bias elements it has just read (same rows, its own column), which saves the
// extra tile and 64 registers: at d <= 64 two workgroups then fit on a CU and cover each other's phases.
constexpr int KV_BN = 128;  // key columns per workgroup (32 per wave)

// query rows per step: 64, or 32 at head dims above 128 (LDS and registers)
template <int D> struct KvRows { static constexpr int value = D > 128 ? 32 : 64; };

template <int D, bool GSUM> struct KvSmem {
    static constexpr int KV_BM = KvRows<D>::value;
    static constexpr int S = D + 8;          // Q / dO row stride (elements)
    static constexpr int SB = KV_BN + 8;     // fused-bias / dS tile row stride (elements)
    static constexpr int Q_BYTES = KV_BM * S * 2;
    static constexpr int FB_BYTES = KV_BM * SB * 2;
    static constexpr int STAGE = 2 * Q_BYTES + 2 * KV_BM * 4 + FB_BYTES;  // Q, dO, LSE, D, fused bias
    static constexpr int OFF_DS = 2 * STAGE;
    static constexpr int TOTAL = OFF_DS + (GSUM ? FB_BYTES : 0);
};

template <typename T> struct NegInfPair;
template <> struct NegInfPair<bf16_tag> { static constexpr uint32_t value = 0xFF80FF80u; };
template <> struct NegInfPair<fp16_tag> { static constexpr uint32_t value = 0xFC00FC00u; };

template <typename T, int D, bool CAUSAL, bool GSUM>
__global__ void __launch_bounds__(NTHREADS, (D <= 64 && !GSUM) ? 2 : 1) bwd_dkdv_kernel(const BwdParams p) {
    using E = Elem<T>;
    using SM = KvSmem<D, GSUM>;
    constexpr int KV_BM = KvRows<D>::value;  // (query rows per step)
    constexpr int FB_IT = KV_BM / 16;        // passes of 16 rows over the fused-bias tile
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int MB = KV_BM / 32;
    constexpr int CH = D / 8, RPP = NTHREADS / CH, Q_IT = KV_BM / RPP;

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const FwdParams &f = p.f;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, g = lane >> 5;
    // linear workgroup id -> (key block, kv head, batch), key block OUTERMOST and ascending: under causal masking the low
    // key blocks are seen by the most queries, so the heaviest workgroups of every head start first
    const int hb_count = f.Hk * f.B;
    const int n_block = (int)blockIdx.x / hb_count, hk = ((int)blockIdx.x % hb_count) % f.Hk, b = ((int)blockIdx.x % hb_count) / f.Hk;
    const int G = f.H / f.Hk;
    const int n0 = n_block * KV_BN;
    const int key = n0 + wave * 32 + r;  // the key column this lane owns
    const int key_c = key < f.Lk ? key : f.Lk - 1;
    const int shift = f.Lk - f.Lq;

    // ---- stationary K / V fragments (B operands)
    u32x4_t kf[KS], vf[KS];
    {
        const uint16_t *kp = (const uint16_t *)f.k + b * f.k_b + (int64_t)key_c * f.k_r + hk * f.k_h;
        const uint16_t *vp = (const uint16_t *)f.v + b * f.v_b + (int64_t)key_c * f.v_r + hk * f.v_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + g * 8;
            u32x4_t kv = {0, 0, 0, 0}, vv = {0, 0, 0, 0};
            if (c < f.d) { kv = *(const u32x4_t *)(kp + c); vv = *(const u32x4_t *)(vp + c); }
            kf[ks] = kv;
            vf[ks] = vv;
        }
    }

    f32x16_t dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) { dk[db][i] = 0.f; dv[db][i] = 0.f; }

    const int M_blocks = (f.Lq + KV_BM - 1) / KV_BM;
    int m_start = 0;
    if (CAUSAL) {
        const int first_q = n0 - shift;  // first query row that sees key n0
        if (first_q > 0) m_start = first_q / KV_BM;
        if (m_start > M_blocks) m_start = M_blocks;
    }

    const bool has_bias = f.bias != nullptr;
    const bool bias_rows = has_bias && f.bi_r != 0;   // per-query bias (and dbias) rows
    const bool use_accum = p.dbias_accum != nullptr;   // several workgroups share a dbias element
    // loop order: per-query dbias wants (m outer, g inner) to sum dS over the group in registers;
    // row-broadcast dbias wants (g outer, m inner) to keep one column sum per bias head.  Query blocks
    // are walked from the last one down so that neighbouring workgroups stream the same tiles together.
    const bool m_outer = bias_rows;
    const int n_m = M_blocks - m_start;
    const int n_steps = n_m * G;

    // zero the part of a per-query dbias this workgroup owns but never visits (above the causal diagonal)
    if (bias_rows && !use_accum && m_start > 0) {
        const int ngh = (f.Hb == f.H) ? G : 1;
        for (int gh = 0; gh < ngh; gh++) {
            const int hb = f.Hb == f.H ? hk * G + gh : (f.Hb == 1 ? 0 : hk);
            uint16_t *dbp = (uint16_t *)p.dbias + b * p.db_b + hb * p.db_h;
            const int rows = m_start * KV_BM < f.Lq ? m_start * KV_BM : f.Lq;
            for (int idx = tid; idx < rows * 16; idx += NTHREADS) {
                const int row = idx >> 4, c = idx & 15;
                const int kk = n0 + c * 8;
                if (kk < f.Lk) *(u32x4_t *)(dbp + (int64_t)row * p.db_r + kk) = u32x4_t{0, 0, 0, 0};
            }
        }
    }

    // ---- staging for one step (global -> registers -> LDS)
    const int qc = tid % CH, qr0 = tid / CH;
    const int qcol = (qc * 8 < f.d) ? qc * 8 : 0;
    const int bc = tid & 15, br0 = tid >> 4;  // fused-bias tile: 8-key chunk and first row of this thread
    u32x4_t qreg[Q_IT], doreg[Q_IT], braw[FB_IT];
    u32x2_t mraw[FB_IT];
    float lreg = INFINITY, dreg = 0.f;
    bool stat_ok = false;
    // Every load of a step is unconditional and raw (clamped rows / keys; an absent mask or bias is read from K, any
    // valid address, and ignored later): a conditional load or a value that is looked at right away would make the
    // wait for it -- and for every load issued before it -- land in front of the matrix work instead of behind it.
    const uint8_t *mask_ld = f.mask ? f.mask : (const uint8_t *)f.k;
    const uint16_t *bias_ld = has_bias ? (const uint16_t *)f.bias : (const uint16_t *)f.k;
    auto step_head = [&](int step, int &gi, int &mi) {
        gi = m_outer ? step % G : step / n_m;
        mi = M_blocks - 1 - (m_outer ? step / G : step % n_m);
    };
    auto load_step = [&](int step) {
        int gi, mi;
        step_head(step, gi, mi);
        const int h = hk * G + gi, m0 = mi * KV_BM;
        const uint16_t *qbase = (const uint16_t *)f.q + b * f.q_b + h * f.q_h + qcol;
        const uint16_t *dobase = (const uint16_t *)p.dout + b * p.do_b + h * p.do_h + qcol;
#pragma unroll
        for (int it = 0; it < Q_IT; it++) {
            int qq = m0 + qr0 + it * RPP;
            qq = qq < f.Lq ? qq : f.Lq - 1;
            qreg[it] = *(const u32x4_t *)(qbase + (int64_t)qq * f.q_r);
            doreg[it] = *(const u32x4_t *)(dobase + (int64_t)qq * p.do_r);
        }
        {
            const int qq = m0 + (tid & (KV_BM - 1));
            stat_ok = qq < f.Lq;
            const int qc = stat_ok ? qq : f.Lq - 1;
            lreg = f.lse[((int64_t)b * f.H + h) * f.Lq + qc];
            dreg = p.softmax_d[((int64_t)b * f.H + h) * p.Lq_rounded + qc];
        }
        // mask / bias chunks: rows br0 + 16*it, keys n0 + 8*bc .. +8
        const int hm = f.mask ? (f.Hm == f.H ? h : (f.Hm == 1 ? 0 : hk)) : 0;
        const int hb = has_bias ? (f.Hb == f.H ? h : (f.Hb == 1 ? 0 : hk)) : 0;
        const int kk = n0 + 8 * bc;
        const int kk_c = kk < f.Lk ? kk : 0;
        const int64_t moff = f.mask ? b * f.m_b + hm * f.m_h + kk_c : 0;
        const int64_t boff = has_bias ? b * f.bi_b + hb * f.bi_h + kk_c : 0;
#pragma unroll
        for (int it = 0; it < FB_IT; it++) {
            int qq = m0 + br0 + 16 * it;
            qq = qq < f.Lq ? qq : f.Lq - 1;
            braw[it] = *(const u32x4_t *)(bias_ld + boff + (has_bias ? (int64_t)qq * f.bi_r : 0));
            // (one 8-byte load either way, from an address chosen without a branch: mask bytes of the chunk, or --
            // a mask packed to bits -- the aligned piece of the bit row that holds the chunk's byte)
            const uint8_t *src = (f.mask && f.mbits) ? f.mbits + b * f.mb_b + hm * f.mb_h + (int64_t)qq * f.mb_r + ((kk_c >> 3) & ~7)
                                                     : mask_ld + moff + (f.mask ? (int64_t)qq * f.m_r : 0);
            mraw[it] = *(const u32x2_t *)src;
        }
    };
    auto store_step = [&](int buf) {
        char *base = smem + buf * SM::STAGE;
#pragma unroll
        for (int it = 0; it < Q_IT; it++) {
            const int off = ((qr0 + it * RPP) * SM::S + qc * 8) * 2;
            *(u32x4_t *)(base + off) = qreg[it];
            *(u32x4_t *)(base + SM::Q_BYTES + off) = doreg[it];
        }
        if (tid < KV_BM) {
            ((float *)(base + 2 * SM::Q_BYTES))[tid] = stat_ok ? lreg * kLog2e : INFINITY;
            ((float *)(base + 2 * SM::Q_BYTES + KV_BM * 4))[tid] = stat_ok ? dreg : 0.f;
        }
        // fuse mask and bias: bias where kept, -inf where dropped or beyond Lk
        char *fb = base + 2 * SM::Q_BYTES + 2 * KV_BM * 4;
        const int kk = n0 + 8 * bc;
#pragma unroll
        for (int it = 0; it < FB_IT; it++) {
            u32x4_t bv = has_bias ? braw[it] : u32x4_t{0, 0, 0, 0};
            u32x2_t mv = f.mask ? (f.mbits ? mask_bits_to_bytes(mask_bits_byte(mraw[it], kk < f.Lk ? kk : 0)) : mraw[it])
                                : u32x2_t{0x01010101u, 0x01010101u};
            uint64_t keepm = kk < f.Lk ? ~0ull : 0ull;
            if (kk + 8 > f.Lk && kk < f.Lk) keepm = (1ull << (8 * (f.Lk - kk))) - 1ull;  // chunk straddles the end of the keys
            mv[0] &= (uint32_t)keepm;
            mv[1] &= (uint32_t)(keepm >> 32);
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++) {
                uint32_t x = mv[hlf];
                x = ((((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) >> 7) & 0x01010101u;  // nonzero byte -> 0x01
                const uint32_t z = (x << 8) - x;                                      // 0x01 -> 0xFF per byte
                const uint32_t m0w = __builtin_amdgcn_perm(0, z, 0x01010000u);        // [b0 b0 b1 b1]
                const uint32_t m1w = __builtin_amdgcn_perm(0, z, 0x03030202u);        // [b2 b2 b3 b3]
                bv[2 * hlf] = (bv[2 * hlf] & m0w) | (NegInfPair<T>::value & ~m0w);
                bv[2 * hlf + 1] = (bv[2 * hlf + 1] & m1w) | (NegInfPair<T>::value & ~m1w);
            }
            *(u32x4_t *)(fb + ((br0 + 16 * it) * SM::SB + 8 * bc) * 2) = bv;
        }
    };

    const int a_row = pi_row(r);
    const int tj = lane & 15, te = tj >> 2, tc = tj & 3;
    const int tcp = (tc == 1) ? 2 : (tc == 2 ? 1 : tc);
    const int tdh = (lane >> 4) & 1;
    const uint32_t tr_off = (uint32_t)(((8 * g + te) * SM::S + 16 * tdh + 4 * tcp) * 2);
    const uint32_t a_off = (uint32_t)((a_row * SM::S + g * 8) * 2);

    float colsum = 0.f;       // row-broadcast dbias: sum over queries of dS for this lane's key
    f32x16_t dsum[GSUM ? MB : 1];  // per-query dbias with bias heads < H: sum over the group
    if (GSUM) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int i = 0; i < 16; i++) dsum[mb][i] = 0.f;
    }

    if (n_steps > 0) {
        load_step(0);
        store_step(0);
        __syncthreads();
    }

    for (int step = 0; step < n_steps; step++) {
        int gi, mi;
        step_head(step, gi, mi);
        const int h = hk * G + gi;
        const int m0 = mi * KV_BM;
        const int buf = step & 1;
        const int hb = has_bias ? (f.Hb == f.H ? h : (f.Hb == 1 ? 0 : hk)) : 0;

        const char *sQ = smem + buf * SM::STAGE;
        const char *sDO = sQ + SM::Q_BYTES;
        const float *sLSE = (const float *)(sQ + 2 * SM::Q_BYTES);
        const float *sDD = sLSE + KV_BM;
        uint16_t *sFB = (uint16_t *)(smem + buf * SM::STAGE + 2 * SM::Q_BYTES + 2 * KV_BM * 4) + wave * 32 + r;  // this lane's column
        uint16_t *sDS = GSUM ? (uint16_t *)(smem + SM::OFF_DS) : (uint16_t *)(smem + buf * SM::STAGE + 2 * SM::Q_BYTES + 2 * KV_BM * 4);

        // ---- S = Q K^T and dP = dO V^T
        f32x16_t s[MB], dp[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int i = 0; i < 16; i++) { s[mb][i] = 0.f; dp[mb][i] = 0.f; }
        {
            constexpr int NF = 2 * MB * KS, FR = (D <= 64 && !GSUM) ? 4 : 8;  // (two workgroups per CU cover the rest of the LDS latency)
            u32x4_t a[NF];
            auto frag = [&](int fi) {
                const int which = fi & 1, mb = (fi >> 1) % MB, ks = (fi >> 1) / MB;
                return *(const u32x4_t *)((which ? sDO : sQ) + a_off + (32 * mb * SM::S + ks * 16) * 2);
            };
#pragma unroll
            for (int fi = 0; fi < FR; fi++) a[fi] = frag(fi);
#pragma unroll
            for (int fi = 0; fi < NF; fi++) {
                if (fi + FR < NF) a[fi + FR] = frag(fi + FR);
                const int which = fi & 1, mb = (fi >> 1) % MB, ks = (fi >> 1) / MB;
                if (which) dp[mb] = E::mfma(a[fi], vf[ks], dp[mb]);
                else s[mb] = E::mfma(a[fi], kf[ks], s[mb]);
            }
        }
        // Global loads of the next step: issued here, behind the first GEMM pair, not at the top of the step -- the
        // compiler puts a wait for all outstanding loads in front of the first MFMA (it cannot prove that the
        // registers involved have no load pending from the previous trip), which is free only while nothing is in
        // flight.  The softmax and the dK / dV GEMMs below cover the latency.
        __builtin_amdgcn_sched_barrier(0);
        if (GSUM || D > 64) {
            if (step + 1 < n_steps) load_step(step + 1);
            __builtin_amdgcn_sched_barrier(0);
        }

        // ---- P = exp2((S*scale + fused)*log2e - LSE*log2e) ; dS = P * (dP - D)
        const bool diag = CAUSAL && (n0 + wave * 32 + 31 > m0 + shift);
        uint32_t ppk[MB * 8], dpk[MB * 8];
        f32x16_t ds[GSUM ? MB : 1];
        float part = 0.f;
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                const int q0l = 32 * mb + 16 * blk + 8 * g;  // first local query row of these 8 registers
                const f32x4_t l0 = *(const f32x4_t *)(sLSE + q0l), l1 = *(const f32x4_t *)(sLSE + q0l + 4);
                const f32x4_t d0 = *(const f32x4_t *)(sDD + q0l), d1 = *(const f32x4_t *)(sDD + q0l + 4);
                float pv[8], dsv[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int ii = 8 * blk + e;
                    const float lse2 = e < 4 ? l0[e] : l1[e - 4];
                    const float dd = e < 4 ? d0[e] : d1[e - 4];
                    const float fb = E::lo((uint32_t)sFB[(q0l + e) * SM::SB]);
                    const float x = fmaf(fmaf(s[mb][ii], f.scale, fb), kLog2e, -lse2);
                    pv[e] = fast_exp2(x);
                    dsv[e] = dp[mb][ii] - dd;
                }
                if (diag) {
                    asm volatile("" ::: "memory");
                    const int lim = key - shift - m0 - q0l;  // rows e >= lim see this key
#pragma unroll
                    for (int e = 0; e < 8; e++) pv[e] = e >= lim ? pv[e] : 0.f;
                }
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    dsv[e] *= pv[e];
                    if (GSUM) ds[mb][8 * blk + e] = dsv[e];
                    else part += dsv[e];
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    ppk[mb * 8 + blk * 4 + e] = E::pack2(pv[2 * e], pv[2 * e + 1]);
                    dpk[mb * 8 + blk * 4 + e] = E::pack2(dsv[2 * e], dsv[2 * e + 1]);
                }
                if (!GSUM && bias_rows && !use_accum) {
                    // dS replaces the fused-bias elements this lane has just read: same rows, its own column
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t w = dpk[mb * 8 + blk * 4 + e];
                        sFB[(q0l + 2 * e) * SM::SB] = (uint16_t)(w & 0xffffu);
                        sFB[(q0l + 2 * e + 1) * SM::SB] = (uint16_t)(w >> 16);
                    }
                }
            }

        // (two workgroups per CU: the staging registers of the next step would not fit next to the softmax's, so its
        // loads are issued here, behind the softmax; the other workgroup covers what the GEMMs below do not)
        if (!GSUM && D <= 64) {
            __builtin_amdgcn_sched_barrier(0);
            if (step + 1 < n_steps) load_step(step + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- dV^T += dO^T P ; dK^T += Q^T dS
#pragma unroll
        for (int qb = 0; qb < KV_BM / 16; qb++) {
            const u32x4_t pb = {ppk[4 * qb], ppk[4 * qb + 1], ppk[4 * qb + 2], ppk[4 * qb + 3]};
            const u32x4_t sb = {dpk[4 * qb], dpk[4 * qb + 1], dpk[4 * qb + 2], dpk[4 * qb + 3]};
#pragma unroll
            for (int db = 0; db < DB; db++) {
                const uint32_t off = tr_off + (uint32_t)((16 * qb * SM::S + 32 * db) * 2);
                const u32x2_t lo = lds_read_tr16(sDO, off), hi = lds_read_tr16(sDO, off + 4 * SM::S * 2);
                const u32x2_t lo2 = lds_read_tr16(sQ, off), hi2 = lds_read_tr16(sQ, off + 4 * SM::S * 2);
                const u32x4_t a1 = {lo[0], lo[1], hi[0], hi[1]};
                const u32x4_t a2 = {lo2[0], lo2[1], hi2[0], hi2[1]};
                dv[db] = E::mfma(a1, pb, dv[db]);
                dk[db] = E::mfma(a2, sb, dk[db]);
            }
        }

        // ---- dBias
        bool tile_out = false;  // this step leaves a dS tile in LDS to be stored (uniform)
        if (has_bias) {
            if (!bias_rows) {
                if (GSUM) {
#pragma unroll
                    for (int mb = 0; mb < MB; mb++)
#pragma unroll
                        for (int i = 0; i < 16; i++) part += ds[mb][i];
                }
                colsum += part;
                const bool last_m = (step % n_m) == n_m - 1;
                if (last_m && (f.Hb == f.H || gi == G - 1)) {
                    const float tot = xhalf_sum(colsum);
                    if (g == 0 && key < f.Lk) {
                        if (use_accum) atomicAdd(p.dbias_accum + b * p.dba_b + hb * p.dba_h + key, tot);
                        else ((uint16_t *)p.dbias)[b * p.db_b + hb * p.db_h + key] = (uint16_t)(E::pack2(tot, 0.f) & 0xffffu);
                    }
                    colsum = 0.f;
                }
            } else if (!GSUM) {
                // every step owns its dbias tile (bias per query head, or one query head per bias head); dbias
                // elements shared between workgroups take the GSUM variant and its fp32 atomics
                tile_out = true;
            } else {
                const bool per_head = f.Hb == f.H;
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) dsum[mb][i] = (per_head || gi == 0) ? ds[mb][i] : dsum[mb][i] + ds[mb][i];
                if (per_head || gi == G - 1) {
                    if (use_accum) {
#pragma unroll
                        for (int mb = 0; mb < MB; mb++)
#pragma unroll
                            for (int i = 0; i < 16; i++) {
                                const int qq = m0 + 32 * mb + 16 * (i >> 3) + 8 * g + (i & 7);
                                if (qq < f.Lq && key < f.Lk)
                                    atomicAdd(p.dbias_accum + b * p.dba_b + hb * p.dba_h + (int64_t)qq * p.dba_r + key, dsum[mb][i]);
                            }
                    } else {
                        tile_out = true;
#pragma unroll
                        for (int mb = 0; mb < MB; mb++)
#pragma unroll
                            for (int i = 0; i < 16; i++) {
                                const int ql = 32 * mb + 16 * (i >> 3) + 8 * g + (i & 7);
                                sDS[ql * SM::SB + wave * 32 + r] = (uint16_t)(E::pack2(dsum[mb][i], 0.f) & 0xffffu);
                            }
                    }
                }
            }
        }
        if (tile_out) __syncthreads();  // the dS tile is complete
        if (step + 1 < n_steps) store_step(buf ^ 1);
        if (tile_out) {
            uint16_t *dbp = (uint16_t *)p.dbias + b * p.db_b + hb * p.db_h;
            const int kk = n0 + 8 * bc;
#pragma unroll
            for (int it = 0; it < FB_IT; it++) {
                const int ql = br0 + 16 * it, qq = m0 + ql;
                if (qq < f.Lq && kk < f.Lk)
                    *(u32x4_t *)(dbp + (int64_t)qq * p.db_r + kk) = *(const u32x4_t *)(sDS + ql * SM::SB + 8 * bc);
            }
        }
        __syncthreads();
    }

    // a key block that no query can see still owns its dbias column (row-broadcast case)
    if (has_bias && !bias_rows && n_steps == 0 && !use_accum && g == 0 && key < f.Lk) {
        const int ngh = (f.Hb == f.H) ? G : 1;
        for (int gh = 0; gh < ngh; gh++) {
            const int hb = f.Hb == f.H ? hk * G + gh : (f.Hb == 1 ? 0 : hk);
            ((uint16_t *)p.dbias)[b * p.db_b + hb * p.db_h + key] = 0;
        }
    }

    // ---- store dK (scaled) and dV
    if (key < f.Lk) {
        uint16_t *dkp = (uint16_t *)p.dk + b * p.dk_b + (int64_t)key * p.dk_r + hk * p.dk_h;
        uint16_t *dvp = (uint16_t *)p.dv + b * p.dv_b + (int64_t)key * p.dv_r + hk * p.dv_h;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                const int c = 32 * db + 16 * blk + 8 * g;
                if (c < f.d) {
                    u32x4_t wk, wv;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        wk[e] = E::pack2(dk[db][8 * blk + 2 * e] * f.scale, dk[db][8 * blk + 2 * e + 1] * f.scale);
                        wv[e] = E::pack2(dv[db][8 * blk + 2 * e], dv[db][8 * blk + 2 * e + 1]);
                    }
                    *(u32x4_t *)(dkp + c) = wk;
                    *(u32x4_t *)(dvp + c) = wv;
                }
            }
    }
}

// ------------------------------------------------------------------------------------------------
// fp32 dbias accumulator helpers (only when several workgroups share a dbias element)
// ------------------------------------------------------------------------------------------------
__global__ void fill_zero_kernel(float *ptr, size_t n) {
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) ptr[i] = 0.f;
}

template <typename T>
__global__ void dbias_convert_kernel(const BwdParams p, int nb, int nh, int nr, int lk) {
    using E = Elem<T>;
    size_t total = (size_t)nb * nh * nr * lk;
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    for (; i < total; i += stride) {
        int k = (int)(i % lk);
        size_t t = i / lk;
        int rr = (int)(t % nr); t /= nr;
        int hh = (int)(t % nh);
        int bb = (int)(t / nh);
        float v = p.dbias_accum[bb * p.dba_b + hh * p.dba_h + (int64_t)rr * p.dba_r + k];
        ((uint16_t *)p.dbias)[bb * p.db_b + hh * p.db_h + (int64_t)rr * p.db_r + k] = (uint16_t)(E::pack2(v, 0.f) & 0xffffu);
    }
}

template <typename T, int D>
hipError_t launch_bwd_t(const BwdParams &p, hipStream_t stream) {
    const FwdParams &f = p.f;
    hipError_t e;
    // 1. D = rowsum(dO * O)  (the compacted backward has done it in its pre-pass launch)
    if (!p.dot_done) {
        const int rpb = bwd_dot_rows_per_block(f.d);
        dim3 grid(((f.cu_q ? f.total_q : p.Lq_rounded) + rpb - 1) / rpb, f.H, f.cu_q ? 1 : f.B);
        hipLaunchKernelGGL((bwd_dot_kernel<T>), grid, dim3(256), 0, stream, p);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    const int nb = f.bi_b == 0 ? 1 : f.B, nr = f.bi_r == 0 ? 1 : f.Lq;
    if (p.dbias_accum) {
        size_t n = (size_t)nb * f.Hb * nr * ((f.Lk + 7) / 8 * 8);
        hipLaunchKernelGGL(fill_zero_kernel, dim3(1024), dim3(256), 0, stream, p.dbias_accum, n);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    // 2. dK, dV, dBias
    const int dtype_code = std::is_same<T, bf16_tag>::value ? 0 : 1;
    const bool colmask = bwd_colmask_applicable(p);
    if (f.Lk > 0 && colmask) {
        if ((e = launch_bwd_dkdv_colmask(p, dtype_code, stream)) != hipSuccess) return e;
    } else if (f.Lk > 0) {
        dim3 grid(((f.Lk + KV_BN - 1) / KV_BN) * f.Hk * f.B);
        // a per-query bias shared by several query heads: dS is summed over the group before it is written; one
        // shared by several workgroups (broadcast over the batch or over kv heads) is accumulated with fp32 atomics
        const bool gsum = f.bias != nullptr && f.bi_r != 0 && ((f.Hb != f.H && f.H / f.Hk > 1) || p.dbias_accum != nullptr);
        auto launch = [&](auto kern, size_t smem) -> hipError_t {
            static DynSmemLimit smem_limit;  // one per kernel: the lambda is instantiated per kernel type
            hipError_t e2 = smem_limit.ensure((const void *)kern, (int)smem);
            if (e2 != hipSuccess) return e2;
            hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), smem, stream, p);
            return hipGetLastError();
        };
        if (gsum) e = f.causal ? launch(bwd_dkdv_kernel<T, D, true, true>, KvSmem<D, true>::TOTAL) : launch(bwd_dkdv_kernel<T, D, false, true>, KvSmem<D, true>::TOTAL);
        else e = f.causal ? launch(bwd_dkdv_kernel<T, D, true, false>, KvSmem<D, false>::TOTAL) : launch(bwd_dkdv_kernel<T, D, false, false>, KvSmem<D, false>::TOTAL);
        if (e != hipSuccess) return e;
    }
    // 3. dQ (the launch of a compacted backward also sums the dK / dV / dBias partial results of step 2)
    if (colmask) {
        if ((e = launch_bwd_dq_colmask(p, dtype_code, stream)) != hipSuccess) return e;
    } else if (f.Lk > 0 && bwd_dq_from_ds_applicable(p)) {
        // (step 2 has written dS itself as dBias: dQ = scale * dS K without a second pass over mask and bias)
        if ((e = launch_bwd_dq_from_ds(p, dtype_code, stream)) != hipSuccess) return e;
    } else {
        if ((e = launch_bwd_dq(p, dtype_code, stream)) != hipSuccess) return e;
    }
    // 4. shared dBias elements: fp32 sums to the output type
    if (p.dbias_accum) {
        hipLaunchKernelGGL((dbias_convert_kernel<T>), dim3(1024), dim3(256), 0, stream, p, nb, f.Hb, nr, f.Lk);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace

hipError_t launch_bwd(const BwdParams &p, int dtype, hipStream_t stream) {
    if (p.f.B <= 0 || p.f.Lq <= 0) return hipSuccess;
    // head dims up to 64 / 128 / 256 (a head dim in between runs in the next larger instantiation)
    const int d = p.f.d;
    if (dtype == 0) return d <= 64 ? launch_bwd_t<bf16_tag, 64>(p, stream) : d <= 128 ? launch_bwd_t<bf16_tag, 128>(p, stream) : launch_bwd_t<bf16_tag, 256>(p, stream);
    return d <= 64 ? launch_bwd_t<fp16_tag, 64>(p, stream) : d <= 128 ? launch_bwd_t<fp16_tag, 128>(p, stream) : launch_bwd_t<fp16_tag, 256>(p, stream);
}

}  // namespace fdma
