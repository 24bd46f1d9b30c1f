// Forward dynamic-mask attention for gfx950, column-mask specialisation.
//
// Same math and same reference counterparts as fdma_fwd.hip (compute_attn_1rowblock,
// csrc/flash_sparse_attn/src/flash_fwd_kernel.h:53-804 of the reference), for the case that dominates
// dynamic-mask attention in practice: mask and bias are absent or broadcast over the query
// dimension (shape [B, {1,Hk,H}, 1, Lk]), so "keep" is a property of the key column and the
// per-query part of the mask is only the causal triangle.
//
// What that buys:
//   * the set of KV tiles with at least one kept key is known before the main loop: the workgroup
//     scans its mask row once into an LDS bitmap and then visits active tiles only -- no per-tile
//     workgroup-wide OR, no loads and no MFMA work for skipped tiles;
//   * bias and mask fuse into one fp32 vector per tile (bias*log2e, or -inf where masked or beyond
//     Lk) staged in LDS, so the score epilogue is a single FMA per element;
//   * causal masking costs instructions on diagonal tiles only.
//
// Pipeline: K, V^T (V is transposed in registers while being staged) and the fused bias vector are
// double-buffered in LDS.  Tile i is computed from buffers i&1 while the global loads of tile i+1 are in
// flight; their LDS stores go to the other buffers after the compute, so one barrier per tile suffices.
// Q is scaled by softmax_scale*log2(e) once and the score accumulators start from the fused bias vector,
// so the MFMA result is the exp2-domain score with bias and mask applied and the softmax spends five
// vector instructions per element (max, sub, exp2, add, half a convert).  LDS fragment reads run a batch
// ahead of the MFMAs that consume them.  Workgroup ids are remapped so that the workgroups sharing one
// XCD's L2 also share K / V.
#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

namespace {

constexpr int MAX_TILES = 16384;  // bitmap capacity: Lk <= 1 Mi keys

template <int D, int BN> struct CmSmem {
    static constexpr int SK = D + 8;        // K tile row stride (elements)
    static constexpr int SVT = BN + 8;      // V^T tile row stride (elements)
    static constexpr int K_BYTES = BN * SK * 2;
    static constexpr int VT_BYTES = D * SVT * 2;
    static constexpr int OFF_K = 0;
    static constexpr int OFF_VT = OFF_K + 2 * K_BYTES;
    static constexpr int OFF_BIAS = OFF_VT + 2 * VT_BYTES;
    static constexpr int OFF_BITS = OFF_BIAS + 2 * BN * 4;
    static constexpr int TOTAL = OFF_BITS + MAX_TILES / 8;
};

// CMP: K / V are the compacted copies of the kept columns (see fdma_compact.hip).  The key axis then has
// `count` columns, all kept; the fused bias vector comes pre-gathered, and the causal limit of a query row
// is the number of kept columns at or below its diagonal instead of the column index itself.
template <typename T, int D, int NQ, int BN, bool CAUSAL, int NW, bool CMP>
__global__ void __launch_bounds__(64 * NW, (NQ == 1 && NW == 4) ? 2 : 1) fwd_colmask_kernel(const FwdParams p) {
    constexpr int NTHREADS = 64 * NW;
    constexpr int STHREADS = NTHREADS;        // threads staging one operand
    using E = Elem<T>;
    using SM = CmSmem<D, BN>;
    constexpr int MB = BN / 32;               // 32-key blocks per tile
    constexpr int KB = BN / 16;               // 16-key contraction blocks per tile
    constexpr int KQ = BN / 4;                // key quads per tile
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int BM = 32 * NQ * NW;
    constexpr int CH = D / 8;                 // 16-byte chunks per K row
    constexpr int K_RPP = STHREADS / CH;      // K rows staged per pass
    constexpr int K_IT = BN / K_RPP;          // passes (registers) per K tile
    constexpr int V_ITEMS = KQ * CH;          // (key quad, d chunk) items of a V tile

    extern __shared__ __attribute__((aligned(16))) char smem[];
    float *sBias = (float *)(smem + SM::OFF_BIAS);
    uint32_t *sBits = (uint32_t *)(smem + SM::OFF_BITS);

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int r = lane & 31;
    const int g = lane >> 5;

    // Workgroup -> (batch, kv head, query head, query block), XCD-aware.  Workgroups are dealt to the 8
    // XCDs round-robin by linear id and every XCD has its own L2.  The id is remapped so that the
    // workgroups running at the same time on one XCD share K / V: the (batch, kv head) pairs are
    // split into k = 8 / gcd(pairs, 8) interleaved lists of query blocks each, the resulting
    // multiple-of-8 lists are dealt to the XCDs, and an XCD walks its lists one after the other,
    // heaviest query block first, the G query heads of a block side by side.  Re-reads of K / V
    // tiles then hit in that XCD's L2, and every XCD gets the same amount of work.
    const int n_mb = (p.Lq + BM - 1) / BM;
    const int G = p.H / p.Hk;
    const int pairs = p.B * p.Hk;
    const int gcd8 = (pairs % 8 == 0) ? 8 : ((pairs % 4 == 0) ? 4 : ((pairs % 2 == 0) ? 2 : 1));
    const int k_split = 8 / gcd8;
    const int list_len = ((n_mb + k_split - 1) / k_split) * G;  // workgroups per list
    const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
    const int vlist = xcd + 8 * (slot / list_len);
    const int pos = slot % list_len;
    const int pair = vlist / k_split;
    const int mslot = (pos / G) * k_split + vlist % k_split;
    if (mslot >= n_mb) return;
    const int m_block = n_mb - 1 - mslot;
    const int b = pair / p.Hk;
    const int h = (pair % p.Hk) * G + pos % G;
    const int hk = h / (p.H / p.Hk);
    const int m0 = m_block * BM;
    const int shift = p.Lk - p.Lq;
    const int wrow0 = m0 + wave * 32 * NQ;  // first query row of this wave

    const int hm = p.mask ? (p.Hm == p.H ? h : (p.Hm == 1 ? 0 : h / (p.H / p.Hm))) : 0;
    const int hb = p.bias ? (p.Hb == p.H ? h : (p.Hb == 1 ? 0 : h / (p.H / p.Hb))) : 0;
    const uint8_t *mrow = p.mask ? p.mask + b * p.m_b + hm * p.m_h : nullptr;
    const uint16_t *brow = p.bias ? (const uint16_t *)p.bias + b * p.bi_b + hb * p.bi_h : nullptr;
    const uint16_t *kbase = (const uint16_t *)p.k + b * p.k_b + hk * p.k_h;
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.v_b + hk * p.v_h;

    // key columns this workgroup iterates over, and the number of them a query row may see
    const int Lk = CMP ? p.cmp.count[b * p.Hk + hk] : p.Lk;
    const int32_t *ccnt = CMP ? p.cmp.cnt + (int64_t)(b * p.Hk + hk) * p.cmp.ld : nullptr;
    const float *fbrow = CMP ? p.cmp.fb + (int64_t)(b * p.cmp.Hfb + (p.cmp.Hfb == p.H ? h : hk)) * p.cmp.ld : nullptr;
    auto visible = [&](int row) -> int {  // columns [0, visible(row)) pass the causal test for `row`
        if (row >= p.Lq) row = p.Lq - 1;
        int c = row + shift;
        if (!CMP) return c + 1;
        if (c < 0) return 0;
        return ccnt[c < p.Lk ? c : p.Lk - 1];
    };

    int n_end = (Lk + BN - 1) / BN;
    if (CAUSAL) {
        int lim = visible(m0 + BM - 1);
        if (lim < 0) lim = 0;
        int ne = (lim + BN - 1) / BN;
        if (ne < n_end) n_end = ne;
    }

    // ---- active-tile bitmap
    for (int base = 0; !CMP && base < n_end; base += NTHREADS) {
        const int j = base + tid;
        bool act = false;
        if (j < n_end) {
            if (mrow) {
                uint32_t any = 0;
#pragma unroll
                for (int c = 0; c < BN / 16; c++) {
                    const int col = j * BN + c * 16;
                    if (col < p.Lk) {
                        u32x4_t mv = *(const u32x4_t *)(mrow + col);
                        any |= mv[0] | mv[1] | mv[2] | mv[3];
                    }
                }
                act = any != 0;
            } else {
                act = true;
            }
        }
        const uint64_t ball = __ballot(act);
        if (lane == 0) {
            const int w0 = (base + wave * 64) >> 5;
            sBits[w0] = (uint32_t)ball;
            sBits[w0 + 1] = (uint32_t)(ball >> 32);
        }
    }
    __syncthreads();

    // smallest active tile >= j, or n_end.  The bitmap word comes from LDS; readfirstlane tells the compiler that
    // the result is wave-uniform, so tile bases, loop conditions and load addresses stay in scalar registers.
    auto next_active = [&](int j) -> int {
        if (CMP) return j < n_end ? j : n_end;
        while (j < n_end) {
            const uint32_t w = __builtin_amdgcn_readfirstlane(sBits[j >> 5]) >> (j & 31);
            if (w) {
                j += __builtin_ctz(w);
                return j < n_end ? j : n_end;
            }
            j = (j | 31) + 1;
        }
        return n_end;
    };

    // ---- Q fragments
    u32x4_t qf[NQ][KS];
#pragma unroll
    for (int nb = 0; nb < NQ; nb++) {
        const int qrow = wrow0 + nb * 32 + r;
        const int qc = qrow < p.Lq ? qrow : p.Lq - 1;
        const uint16_t *qp = (const uint16_t *)p.q + b * p.q_b + (int64_t)qc * p.q_r + h * p.q_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + g * 8;
            u32x4_t v = {0, 0, 0, 0};
            if (qrow < p.Lq && c < p.d) v = *(const u32x4_t *)(qp + c);
            // Q is scaled by softmax_scale * log2(e) once, here (the reference also rounds the scaled Q to the
            // input type, flash_fwd_kernel.h:428-439): the MFMA then accumulates exp2-domain scores directly on
            // top of the fused bias, with no per-element multiply afterwards
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = E::pack2(E::lo(v[e]) * p.scale_log2, E::hi(v[e]) * p.scale_log2);
            qf[nb][ks] = v;
        }
    }

    f32x16_t o[NQ][DB];
    float row_max[NQ], row_sum[NQ];
#pragma unroll
    for (int nb = 0; nb < NQ; nb++) {
        row_max[nb] = -INFINITY;
        row_sum[nb] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) o[nb][db][i] = 0.f;
    }

    // ---- staging helpers (global -> registers -> LDS)
    // Every load is unconditional, from an always valid address: rows beyond the end of the keys are clamped to
    // the last row (their fused bias is -inf, so the duplicate never counts) and head-dim chunks beyond d to chunk
    // 0 (they meet zero Q fragments / columns of O that are not stored).  That keeps the loads free of branches,
    // so that they can be issued one by one between the MFMAs of the tile being computed.
    const int ktid = tid;
    const int kc = ktid % CH, kr0 = ktid / CH;
    const int vkg = tid % KQ, vc = (tid / KQ) % CH;  // V: key quad and d chunk of this thread
    const uint32_t k_r2 = (uint32_t)(p.k_r * 2), v_r2 = (uint32_t)(p.v_r * 2);  // bytes per row
    const uint32_t kcolb = (kc * 8 < p.d ? kc * 16 : 0), vcolb = (vc * 8 < p.d ? vc * 16 : 0);
    u32x4_t kreg[K_IT], vreg[4];  // staging registers
    uint32_t braw = 0, mraw = 0;  // raw bias / mask of this thread's column of the tile in flight
    // an absent mask / bias is read from K instead (any valid address) and ignored when the value is used
    const uint8_t *mrow_ld = mrow ? mrow : (const uint8_t *)kbase;
    const uint16_t *brow_ld = brow ? brow : kbase;
    bool bcol_ok = false;
    int bias_col = 0;
    const char *ktb = nullptr, *vtb = nullptr;  // base of the tile in flight
    int last_row = 0;                           // its last valid row

    auto begin_tile = [&](int j) {
        const int n0 = j * BN;
        ktb = (const char *)kbase + (int64_t)n0 * p.k_r * 2;
        vtb = (const char *)vbase + (int64_t)n0 * p.v_r * 2;
        last_row = (Lk - n0 < BN ? Lk - n0 : BN) - 1;
        bias_col = n0 + ktid;
    };
    // fused bias of the tile's columns: only the raw loads here -- the values are looked at in store_k, after the
    // compute.  Issued after the scores, not at the top of the iteration: with loads in flight there, the waits the
    // compiler places in front of the first LDS fragment reads (it cannot prove that the registers they overwrite
    // have no load pending from the previous iteration) would stall on them.
    auto load_bias_raw = [&]() {
        if (ktid < BN) {
            const int col = bias_col;
            const int cc = col < Lk ? col : 0;
            bcol_ok = col < Lk;
            // (unconditional loads: a load in one arm of a select would have to be waited for right here)
            if (CMP) {
                braw = __float_as_uint(fbrow[cc]);
            } else {
                mraw = mrow_ld[cc];
                braw = brow_ld[cc];
            }
        }
    };
    auto load_k_item = [&](int it) {
        int row = kr0 + it * K_RPP;
        row = row < last_row ? row : last_row;
        kreg[it] = *(const u32x4_t *)(ktb + (uint32_t)row * k_r2 + kcolb);
    };
    auto load_v_item = [&](int i) {
        int row = 4 * vkg + i;
        row = row < last_row ? row : last_row;
        vreg[i] = *(const u32x4_t *)(vtb + (uint32_t)row * v_r2 + vcolb);
    };
    auto load_k = [&](int j) {
        begin_tile(j);
        load_bias_raw();
#pragma unroll
        for (int it = 0; it < K_IT; it++) load_k_item(it);
    };
    auto load_v = [&](int j) {
        (void)j;
#pragma unroll
        for (int i = 0; i < 4; i++) load_v_item(i);
    };
    auto store_k = [&](int buf, int slot) {
        char *sK = smem + SM::OFF_K + buf * SM::K_BYTES;
#pragma unroll
        for (int it = 0; it < K_IT; it++)
            *(u32x4_t *)(sK + ((kr0 + it * K_RPP) * SM::SK + kc * 8) * 2) = kreg[it];
        if (ktid < BN) {
            float v = -INFINITY;
            if (CMP) {
                if (bcol_ok) v = __uint_as_float(braw);
            } else if (bcol_ok && (!mrow || mraw)) {
                v = brow ? E::lo(braw) * kLog2e : 0.f;
            }
            sBias[slot * BN + ktid] = v;
        }
    };
    auto store_v = [&](int buf) {  // transpose 4 keys x 8 d in registers, write V^T[d][key quad]
        char *sVt = smem + SM::OFF_VT + buf * SM::VT_BYTES;
        if (tid < V_ITEMS) {
#pragma unroll
            for (int dd = 0; dd < 8; dd++) {
                const int w = dd >> 1;
                const uint32_t sel = (dd & 1) ? 0x07060302u : 0x05040100u;
                u32x2_t out;
                out[0] = __builtin_amdgcn_perm(vreg[1][w], vreg[0][w], sel);
                out[1] = __builtin_amdgcn_perm(vreg[3][w], vreg[2][w], sel);
                *(u32x2_t *)(sVt + ((vc * 8 + dd) * SM::SVT + 4 * vkg) * 2) = out;
            }
        }
    };

    const int a_row = pi_row(r);

    // causal limits: columns below vis_lane[nb] are visible to this lane's query row, and a tile that ends at
    // or below vis_wave[nb] (the limit of the block's first row) needs no masking at all
    int vis_lane[NQ], vis_wave[NQ];
#pragma unroll
    for (int nb = 0; nb < NQ; nb++) {
        vis_lane[nb] = CAUSAL ? visible(wrow0 + nb * 32 + r) : 0;
        vis_wave[nb] = CAUSAL ? visible(wrow0 + nb * 32) : 0;
    }

    // `prefetch`: the K loads of the tile in flight are issued between the MFMAs
    auto qk = [&](f32x16_t (&s)[NQ][MB], int buf, int slot) {
        const char *sK = smem + SM::OFF_K + buf * SM::K_BYTES;
        // the accumulators start from the fused bias vector (bias * log2e, -inf for dropped keys) of the tile
        const float *bs = sBias + slot * BN + 8 * g;
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                const f32x4_t b0 = *(const f32x4_t *)(bs + 32 * mb + 16 * blk);
                const f32x4_t b1 = *(const f32x4_t *)(bs + 32 * mb + 16 * blk + 4);
#pragma unroll
                for (int nb = 0; nb < NQ; nb++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        s[nb][mb][8 * blk + e] = b0[e];
                        s[nb][mb][8 * blk + 4 + e] = b1[e];
                    }
            }
        // fragment reads run FR ahead of the MFMAs that consume them, so the LDS latency is paid once
        // per batch instead of once per MFMA; (ks, mb) order alternates accumulators
        constexpr int NF = MB * KS, FR = NF < 8 ? NF : 8;
        u32x4_t a[NF];
        auto frag = [&](int f) {
            const int ks = f / MB, mb = f % MB;
            return *(const u32x4_t *)(sK + ((32 * mb + a_row) * SM::SK + ks * 16 + g * 8) * 2);
        };
#pragma unroll
        for (int f = 0; f < FR; f++) a[f] = frag(f);
#pragma unroll
        for (int f = 0; f < NF; f++) {
            if (f + FR < NF) a[f + FR] = frag(f + FR);
            const int ks = f / MB, mb = f % MB;
#pragma unroll
            for (int nb = 0; nb < NQ; nb++) s[nb][mb] = E::mfma(a[f], qf[nb][ks], s[nb][mb]);
            if (f % (NF / K_IT) == 0) load_k_item(f / (NF / K_IT));
        }
        __builtin_amdgcn_sched_group_barrier(0x100, FR + 4 * MB, 0);
#pragma unroll
        for (int f = 0; f < NF - FR; f++) {
            __builtin_amdgcn_sched_group_barrier(0x008, NQ, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, FR * NQ, 0);
    };

    // softmax of one tile: scores in `s` (exp2 domain, bias and mask already in) -> packed probabilities `pk`
    auto softmax = [&](f32x16_t (&s)[NQ][MB], int j, uint32_t (&pk)[NQ][8 * MB]) {
        const int n0 = j * BN;
#pragma unroll
        for (int nb = 0; nb < NQ; nb++) {
            // diagonal tile for this 32-row block? (wave-uniform)
            const bool diag = CAUSAL && (n0 + BN > vis_wave[nb]);
            float tmax = -INFINITY;
            if (diag) {
                asm volatile("" ::: "memory");  // keep this a real (wave-uniform) branch: only diagonal tiles pay
                const int lim = vis_lane[nb] - 1 - n0 - 8 * g;  // local column limit for this lane
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int lc = 32 * mb + 16 * (i >> 3) + (i & 7);
                        s[nb][mb][i] = lc <= lim ? s[nb][mb][i] : -INFINITY;
                    }
            }
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[nb][mb][i]);
            tmax = xhalf_max(tmax);
            if (__any(tmax > row_max[nb])) {
                const float new_max = fmaxf(row_max[nb], tmax);
                const float safe = new_max == -INFINITY ? 0.f : new_max;
                const float alpha = fast_exp2(row_max[nb] - safe);
                row_max[nb] = new_max;
                row_sum[nb] *= alpha;
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) o[nb][db][i] *= alpha;
            }
            const float m_use = row_max[nb] == -INFINITY ? 0.f : row_max[nb];
            float psum = 0.f;
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int i = 0; i < 16; i += 2) {
                    const float p0 = fast_exp2(s[nb][mb][i] - m_use);
                    const float p1 = fast_exp2(s[nb][mb][i + 1] - m_use);
                    psum += p0 + p1;
                    pk[nb][8 * mb + i / 2] = E::pack2(p0, p1);
                }
            row_sum[nb] += psum;
        }
    };
    // O^T += V^T P^T for one tile
    auto pv = [&](const uint32_t (&pk)[NQ][8 * MB], int vbuf) {
        const char *sVt = smem + SM::OFF_VT + vbuf * SM::VT_BYTES;
        {
            constexpr int NF = KB * DB, FR = NF < 8 ? NF : 8;
            u32x4_t a[NF];
            auto frag = [&](int f) {
                const int kb = f / DB, db = f % DB;
                return *(const u32x4_t *)(sVt + ((32 * db + a_row) * SM::SVT + 16 * kb + 8 * g) * 2);
            };
#pragma unroll
            for (int f = 0; f < FR; f++) a[f] = frag(f);
#pragma unroll
            for (int f = 0; f < NF; f++) {
                if (f + FR < NF) a[f + FR] = frag(f + FR);
                const int kb = f / DB, db = f % DB;
#pragma unroll
                for (int nb = 0; nb < NQ; nb++) {
                    u32x4_t bop = {pk[nb][4 * kb], pk[nb][4 * kb + 1], pk[nb][4 * kb + 2], pk[nb][4 * kb + 3]};
                    o[nb][db] = E::mfma(a[f], bop, o[nb][db]);
                }
            }
        }
    };

    // ---- main loop: tile i is computed from LDS buffers i&1 while tile i+1 travels global -> registers; its LDS
    // stores go to the other buffers (last read in iteration i-1) after the compute, one barrier per tile
    int jc = next_active(0);
    if (jc < n_end) {
        load_k(jc);
        load_v(jc);
        store_k(0, 0);
        store_v(0);
        __syncthreads();

        f32x16_t sa[NQ][MB];
        int i = 0;
        while (jc < n_end) {
            const int jn = next_active(jc + 1);
            // the loads of the next tile are spread over the MFMAs of this one (after the last tile the current
            // one is simply fetched again and dropped): eight waves issuing all their loads at once right after
            // the barrier would queue up at the CU's address unit while the matrix pipe idles
            begin_tile(jn < n_end ? jn : jc);
            __builtin_amdgcn_sched_barrier(0);
            qk(sa, i & 1, i & 1);
            load_bias_raw();
            load_v(jc);  // V of the tile in flight: issued before the softmax so that softmax and PV cover the latency
            __builtin_amdgcn_sched_barrier(0);
            uint32_t pk[NQ][8 * MB];
            softmax(sa, jc, pk);
            pv(pk, i & 1);
            __builtin_amdgcn_sched_barrier(0);
            if (jn < n_end) {
                store_k((i + 1) & 1, (i + 1) & 1);
                store_v((i + 1) & 1);
            }
            __syncthreads();
            i++; jc = jn;
        }
    }

    // ---- epilogue
#pragma unroll
    for (int nb = 0; nb < NQ; nb++) {
        const int qrow = wrow0 + nb * 32 + r;
        const float total = xhalf_sum(row_sum[nb]);
        const float inv = total > 0.f ? 1.f / total : 0.f;
        if (qrow < p.Lq) {
            uint16_t *op = (uint16_t *)p.o + b * p.o_b + (int64_t)qrow * p.o_r + h * p.o_h;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int blk = 0; blk < 2; blk++) {
                    const int c = 32 * db + 16 * blk + 8 * g;
                    if (c < p.d) {
                        u32x4_t w;
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            w[e] = E::pack2(o[nb][db][8 * blk + 2 * e] * inv, o[nb][db][8 * blk + 2 * e + 1] * inv);
                        *(u32x4_t *)(op + c) = w;
                    }
                }
            if (g == 0) {
                const float lse = total > 0.f ? (row_max[nb] + __builtin_amdgcn_logf(total)) * kLn2 : INFINITY;
                p.lse[((int64_t)b * p.H + h) * p.Lq + qrow] = lse;
            }
        }
    }
}

template <typename T, int D, int NQ, int BN, bool CAUSAL, bool CMP, int NW = 4>
hipError_t launch_one(const FwdParams &p, hipStream_t stream) {
    constexpr int BM = 32 * NQ * NW;
    auto kern = fwd_colmask_kernel<T, D, NQ, BN, CAUSAL, NW, CMP>;
    const int smem = CmSmem<D, BN>::TOTAL;
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    const int n_mb = (p.Lq + BM - 1) / BM, G = p.H / p.Hk, pairs = p.B * p.Hk;
    const int gcd8 = (pairs % 8 == 0) ? 8 : ((pairs % 4 == 0) ? 4 : ((pairs % 2 == 0) ? 2 : 1));
    const int k_split = 8 / gcd8;
    dim3 grid(pairs * k_split * ((n_mb + k_split - 1) / k_split) * G);
    hipLaunchKernelGGL(kern, grid, dim3(64 * NW), smem, stream, p);
    return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_d(const FwdParams &p, int variant, hipStream_t stream) {
    (void)variant;
    if (p.cmp.on) return p.causal ? launch_one<T, D, 1, 64, true, true>(p, stream) : launch_one<T, D, 1, 64, false, true>(p, stream);
    return p.causal ? launch_one<T, D, 1, 64, true, false>(p, stream) : launch_one<T, D, 1, 64, false, false>(p, stream);
}

}  // namespace

bool fwd_colmask_applicable(const FwdParams &p) {
    const bool mask_ok = !p.mask || p.m_r == 0;
    const bool bias_ok = !p.bias || p.bi_r == 0;
    return mask_ok && bias_ok && (p.Lk + 31) / 32 <= MAX_TILES;
}

hipError_t launch_fwd_colmask(const FwdParams &p, int dtype, int nq, hipStream_t stream) {
    const bool d64 = p.d <= 64;
    if (dtype == 0) return d64 ? launch_d<bf16_tag, 64>(p, nq, stream) : launch_d<bf16_tag, 128>(p, nq, stream);
    return d64 ? launch_d<fp16_tag, 64>(p, nq, stream) : launch_d<fp16_tag, 128>(p, nq, stream);
}

}  // namespace fdma
