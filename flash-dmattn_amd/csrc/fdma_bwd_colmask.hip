// Backward dynamic-mask attention for gfx950, column-mask specialisation of the two main kernels.
//
// Same math and same reference counterparts as fdma_bwd.hip
// (compute_dq_dk_dv_1colblock, csrc/flash_sparse_attn/src/flash_bwd_kernel.h:79-1142 of the reference), for
// mask and bias that are absent or broadcast over the query dimension ([B, {1,Hk,H}, 1, Lk]).
// "Keep" and the bias are then properties of the key column:
//   * in the dK/dV kernel a lane owns one key column for the whole kernel, so mask and bias
//     collapse to one fused per-lane constant (bias*log2e, or -inf when masked / beyond Lk): no
//     mask or bias loads in the loop, no selects -- exp2(-inf) = 0 does the masking;
//   * dBias is the column sum of dS, accumulated in a register and written once;
//   * in the dQ kernel the fused vector is staged per tile exactly as in the forward kernel and
//     fully masked 64-key tiles are skipped through the same LDS bitmap.
// K and V are stationary in the dK/dV kernel (B operands: in registers, except V at d = 128, which every
// lane parks in LDS as a private spill so that two workgroups fit on a CU); Q / dO tiles and the row
// statistics stream through double-buffered LDS, fetched two steps ahead of their use.  Workgroup ids
// are remapped so that workgroups sharing an XCD's L2 share the streamed operands.
#include <type_traits>

#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

namespace {

constexpr int NTHREADS = 256;

// XCD-aware work distribution shared by both kernels: `pairs` independent (batch, kv head) pairs with
// `n_units` units of work each (heaviest first); see the forward column-mask kernel for the rationale.
struct XcdMap {
    int pair, unit;
    bool valid;
};
__device__ __forceinline__ XcdMap xcd_map(int lid, int pairs, int n_units, int per_unit) {
    const int gcd8 = (pairs % 8 == 0) ? 8 : ((pairs % 4 == 0) ? 4 : ((pairs % 2 == 0) ? 2 : 1));
    const int k_split = 8 / gcd8;
    const int list_len = ((n_units + k_split - 1) / k_split) * per_unit;
    const int xcd = lid % 8, slot = lid / 8;
    const int vlist = xcd + 8 * (slot / list_len);
    const int pos = slot % list_len;
    XcdMap m;
    m.pair = vlist / k_split;
    m.unit = (pos / per_unit) * k_split + vlist % k_split;
    m.valid = m.unit < n_units;
    return m;
}
inline int xcd_grid(int pairs, int n_units, int per_unit) {
    const int gcd8 = (pairs % 8 == 0) ? 8 : ((pairs % 4 == 0) ? 4 : ((pairs % 2 == 0) ? 2 : 1));
    const int k_split = 8 / gcd8;
    return pairs * k_split * ((n_units + k_split - 1) / k_split) * per_unit;
}

// ------------------------------------------------------------------------------------------------
// dK / dV / dBias
// ------------------------------------------------------------------------------------------------
constexpr int KV_BM = 64;   // query rows per planning block (the work split counts these)
constexpr int KV_BN = 128;  // key columns per workgroup (32 per wave)

// Query rows per step.  At d = 128 the stationary K / V fragments and the dK / dV accumulators alone take 192 registers
// per lane; with 32-row steps and V parked in LDS (every lane re-reads its own row: a private spill, no sharing) the
// kernel fits in 256 registers and 70 KB of LDS, so that two workgroups share a CU and fill each other's stalls.
template <int D> struct KvcSmem {
    static constexpr int BM = D > 64 ? 32 : 64;
    static constexpr bool V_LDS = D > 64;
    static constexpr int S = LdsTile<D>::S;
    static constexpr int Q_BYTES = BM * S * 2;
    static constexpr int STAGE = 2 * Q_BYTES + 2 * BM * 4;  // Q, dO, LSE, D
    static constexpr int OFF_V = 2 * STAGE;
    static constexpr int TOTAL = OFF_V + (V_LDS ? KV_BN * S * 2 : 0);
};

// CMP: the key axis is the compacted list of kept columns (fdma_compact.hip); a lane still owns one key,
// reads it from the dense copies, and writes its gradients to the key's original row / column.
template <typename T, int D, bool CAUSAL, bool CMP>
__global__ void __launch_bounds__(NTHREADS, D <= 128 ? 2 : 1) bwd_dkdv_colmask_kernel(const BwdParams p) {
    using E = Elem<T>;
    using SM = KvcSmem<D>;
    using TL = LdsTile<D>;
    constexpr int BM = SM::BM;       // query rows per step
    constexpr int SUB = KV_BM / BM;  // steps per planning block
    constexpr bool V_LDS = SM::V_LDS;
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int MB = BM / 32;
    constexpr int CH = D / 8, RPP = NTHREADS / CH, Q_IT = BM / RPP;
    // DMA: the Q / dO tiles and the row statistics of a step go from global memory straight into LDS
    // (global_load_lds: a wave writes 64 consecutive 16-byte or 4-byte pieces, so the swizzle of the tile is applied
    // to the GLOBAL address of each lane's piece); no staging registers, no LDS stores, and the loads are issued
    // between the MFMAs a whole step ahead of the barrier that publishes them.  Needs rows of exactly 256 bytes.
    constexpr bool DMA = TL::SWZ;
    static_assert(!DMA || (BM == 32 && NTHREADS == 256), "the direct loads are laid out for 32-row steps and four waves");

    extern __shared__ __attribute__((aligned(256))) char smem[];
    const uint32_t lds0 = lds_addr(smem);  // (a multiple of 256)

    const FwdParams &f = p.f;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = tid & 63, r = lane & 31, g = lane >> 5;
    const int G = f.H / f.Hk;
    // work item: a 128-key block of one (batch, kv head) pair, over query heads [g_lo, g_hi) and segment
    // `seg` of `Sm` of the query range; `slot` >= 0 when the block is shared by several workgroups
    int pair, n_block, g_lo = 0, g_hi = G, seg = 0, Sm = 1, Q = 1 << 30, slot = -1;
    if (CMP) {
        const int32_t *plan = f.cmp.plan;
        const int Gs = plan[1];
        Sm = plan[2];
        Q = plan[4];
        const int per = Gs * Sm;
        int sub;
        const int x = blockIdx.x % 8, l = blockIdx.x / 8;
        if (per > 1) {
            // Split units: the plan holds, per XCD, the list of the parts that exist -- (pair, unit, part of the
            // unit), longest parts first.  Workgroup l of an XCD takes entry l; consecutive workgroups of an XCD go
            // to its shader engines in turn, and with the existing parts side by side every engine gets its share.
            const int cap = gridDim.x / 8;
            const int32_t *lists = plan + plan[5];
            if (l >= lists[x]) return;
            const int32_t *e = lists + 8 + 2 * ((int64_t)x * cap + l);
            pair = e[0];
            n_block = e[1] & 0xffff;
            sub = e[1] >> 16;
        } else {
            // unit lists per XCD: the units of a pair are dealt to its k lists, the lists to the XCDs
            const int P = f.B * f.Hk, k = dkdv_lists_per_pair(P);
            const int list_len = plan[3];
            if (list_len == 0) return;
            const int ls = l / list_len, pos = l % list_len;
            if (ls >= P * k / 8) return;
            const int vlist = x + 8 * ls, fold = vlist % k;
            pair = vlist / k;
            n_block = dkdv_unit_at(pos, fold, k);
            if (n_block >= plan[DKDV_PLAN_HDR + pair + 1] - plan[DKDV_PLAN_HDR + pair]) return;
            sub = 0;
        }
        const int unit = plan[DKDV_PLAN_HDR + pair] + n_block;
        const int gper = G / Gs;
        g_lo = (sub / Sm) * gper;
        g_hi = g_lo + gper;
        seg = sub % Sm;
        if (per > 1) slot = unit * per + sub;
    } else {
        const int n_nb = (f.Lk + KV_BN - 1) / KV_BN;
        const XcdMap wm = xcd_map(blockIdx.x, f.B * f.Hk, n_nb, 1);
        if (!wm.valid) return;
        n_block = wm.unit;  // low key blocks are seen by the most queries under causal: heaviest first
        pair = wm.pair;
    }
    const int b = pair / f.Hk, hk = pair % f.Hk;
    const int n0 = n_block * KV_BN;
    const SeqInfo sq = seq_info(f, b);  // this batch entry's lengths and first rows (ragged batch: from cu_seqlens)
    const int LqS = sq.Lq, LkS = sq.Lk;
    const int Lk = CMP ? f.cmp.count[pair] : LkS;  // key columns on this pair's (possibly compacted) key axis
    if (n0 >= Lk) return;  // the compacted list, or a shorter sequence of a ragged batch, ends before this block
    const int key = n0 + wave * 32 + r;  // the key column this lane owns
    const int key_c = key < Lk ? key : Lk - 1;
    const int shift = LkS - LqS;
    // original column indices: of this lane's key, of the workgroup's first key and of the wave's last key
    const int32_t *cidx = CMP ? f.cmp.idx + (int64_t)pair * f.cmp.ld : nullptr;
    const int okey = CMP ? cidx[key_c] : key;
    const int okey_first = CMP ? cidx[n0] : n0;
    const int okey_wlast = CMP ? cidx[n0 + wave * 32 + 31 < Lk ? n0 + wave * 32 + 31 : Lk - 1] : n0 + wave * 32 + 31;

    // ---- stationary K / V fragments (B operands): lane holds K[key][16ks + 8g .. +8]
    u32x4_t kf[KS], vf[V_LDS ? 1 : KS];
    char *sVt = smem + SM::OFF_V;
    uint32_t v_base = TL::frag_base(wave * 32 + r, g);  // V_LDS: this lane's V row, its chunks
    {
        const uint16_t *kp = (const uint16_t *)f.k + b * f.k_b + (sq.k0 + key_c) * f.k_r + hk * f.k_h;
        const uint16_t *vp = (const uint16_t *)f.v + b * f.v_b + (sq.k0 + key_c) * f.v_r + hk * f.v_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + g * 8;
            u32x4_t kv = {0, 0, 0, 0}, vv = {0, 0, 0, 0};
            if (c < f.d) { kv = *(const u32x4_t *)(kp + c); vv = *(const u32x4_t *)(vp + c); }
            // K is only used for the scores here: scale it by softmax_scale * log2(e) once, so that the MFMA
            // accumulates exp2-domain scores on top of the column constant (no multiply per element later)
#pragma unroll
            for (int e = 0; e < 4; e++) kv[e] = E::pack2(E::lo(kv[e]) * f.scale_log2, E::hi(kv[e]) * f.scale_log2);
            kf[ks] = kv;
            if (V_LDS) *(u32x4_t *)(sVt + TL::frag_at(v_base, ks)) = vv;
            else vf[ks] = vv;
        }
    }

    v_base += lds0 + SM::OFF_V;  // from here on an absolute LDS address (see lds_ld128)

    f32x16_t dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) { dk[db][i] = 0.f; dv[db][i] = 0.f; }

    const int M_blocks = (LqS + KV_BM - 1) / KV_BM;
    // query blocks that see the workgroup's first key: [m_start, M_blocks)
    const int m_start = M_blocks - dkdv_query_blocks(LqS, LkS, CAUSAL, okey_first);
    // this workgroup's query blocks [m_lo, m_hi): all of them, or one of the unit's equal segments
    int m_lo = m_start, m_hi = M_blocks;
    if (slot >= 0) {
        const int n_seg = dkdv_segments(M_blocks - m_start, Q, Sm);
        if (seg >= n_seg) return;  // the reduce kernel knows that this slot stays unwritten
        const int len = (M_blocks - m_start + n_seg - 1) / n_seg;
        m_lo = m_start + seg * len;
        m_hi = m_lo + len < M_blocks ? m_lo + len : M_blocks;
    }
    // the planning blocks [m_lo, m_hi) in steps of BM rows: [s_lo, s_hi), without steps entirely beyond Lq
    const int S_blocks = (LqS + BM - 1) / BM;
    const int s_lo = m_lo * SUB, s_hi = m_hi * SUB < S_blocks ? m_hi * SUB : S_blocks;
    const int n_m = s_hi > s_lo ? s_hi - s_lo : 0;
    // (g outer, m inner); the query blocks are walked from the LAST one down, so that the
    // workgroups of one (batch, kv head) pair, which run side by side on an XCD, all begin at the same
    // Q / dO tile and stream the same tiles at the same time (L2 hits instead of re-fetches)
    const int n_steps = n_m * (g_hi - g_lo);

    const bool has_bias = f.bias != nullptr;
    const bool use_accum = p.dbias_accum != nullptr;

    // Fused per-lane column constant for query head h: bias*log2e, or -inf when the column is dropped.  It travels
    // with the prefetch of the step that needs it: raw, unconditional loads (an absent mask / bias is read from K,
    // any valid address, and ignored) issued first in load_step, turned into the constant after the compute.
    uint32_t cm_raw = 1, cb_raw = 0;
    const uint8_t *mask_ld = f.mask ? f.mask : (const uint8_t *)f.k;
    const uint16_t *bias_ld = has_bias ? (const uint16_t *)f.bias : (const uint16_t *)f.k;
    auto column_const_load = [&](int h) {
        if (CMP) {
            cb_raw = __float_as_uint(f.cmp.fb[(int64_t)(b * f.cmp.Hfb + (f.cmp.Hfb == f.H ? h : hk)) * f.cmp.ld + key_c]);
        } else {
            const int hm = f.mask ? (f.Hm == f.H ? h : (f.Hm == 1 ? 0 : hk)) : 0;
            const int hb = has_bias ? (f.Hb == f.H ? h : (f.Hb == 1 ? 0 : hk)) : 0;
            cm_raw = mask_ld[f.mask ? b * f.m_b + hm * f.m_h + key_c : 0];
            cb_raw = bias_ld[has_bias ? b * f.bi_b + hb * f.bi_h + key_c : 0];
        }
    };
    auto column_const_value = [&]() -> float {
        if (key >= Lk) return -INFINITY;
        if (CMP) return __uint_as_float(cb_raw);
        if (f.mask && !cm_raw) return -INFINITY;
        return has_bias ? E::lo(cb_raw) * kLog2e : 0.f;
    };

    // ---- staging of Q / dO / LSE / D for one step (global -> registers -> LDS)
    const int qc = tid % CH, qr0 = tid / CH;
    const int qcol = (qc * 8 < f.d) ? qc * 8 : 0;  // head-dim chunks beyond d: re-read chunk 0 (K/V fragments there are zero)
    u32x4_t qreg[Q_IT], doreg[Q_IT];
    float lreg = INFINITY, dreg = 0.f;
    bool stat_ok = false;
    // Byte offsets of this thread's loads inside a 64-row block are loop invariants -- one set for full blocks, one
    // for the (only) partial block at the end of the queries, whose rows beyond Lq are clamped to the last row
    // (finite duplicates, cancelled by LSE = +inf) -- so a load is one instruction with a scalar block base.
    typedef const __attribute__((address_space(1))) char *gptr_t;
    auto uniform_ptr = [](const void *ptr) -> gptr_t {
        const uint64_t v = (uint64_t)ptr;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (gptr_t)(((uint64_t)hi << 32) | lo);
    };
    const int m_last = (LqS - 1) / BM, row_last = (LqS - 1) % BM;
    uint32_t qoff[Q_IT], qoff_l[Q_IT], dooff[Q_IT], dooff_l[Q_IT];
#pragma unroll
    for (int it = 0; it < Q_IT; it++) {
        // DMA: load n = 2 * wave + it of a tile fills LDS bytes [1024 n, 1024 n + 1024): rows 4n .. 4n+3, lane l the
        // chunk POSITION l % 16 of row 4n + l / 16, which holds chunk position ^ swz(row) of the global row
        const int n = 2 * wave + it;
        const int row = DMA ? 4 * n + (lane >> 4) : qr0 + it * RPP, row_c = row < row_last ? row : row_last;
        const int chunk = (lane & 15) ^ (int)TL::swz(row);
        const int col = DMA ? ((chunk * 8 < f.d) ? chunk * 8 : 0) : qcol;
        qoff[it] = (uint32_t)(row * f.q_r + col) * 2;
        qoff_l[it] = (uint32_t)(row_c * f.q_r + col) * 2;
        dooff[it] = (uint32_t)(row * p.do_r + col) * 2;
        dooff_l[it] = (uint32_t)(row_c * p.do_r + col) * 2;
    }
    gptr_t ld_qbase = nullptr, ld_dobase = nullptr;  // block bases of the step being fetched (scalar registers)
    bool ld_partial = false;
    // tile load `n` of the step being fetched: 0 .. Q_IT-1 are Q rows, Q_IT .. 2*Q_IT-1 dO rows
    auto load_item = [&](int n) {
        if (n < Q_IT) qreg[n] = *(const __attribute__((address_space(1))) u32x4_t *)(ld_qbase + (ld_partial ? qoff_l[n] : qoff[n]));
        else doreg[n - Q_IT] = *(const __attribute__((address_space(1))) u32x4_t *)(ld_dobase + (ld_partial ? dooff_l[n - Q_IT] : dooff[n - Q_IT]));
    };
    // everything of a step's fetch except the tile loads: block bases, column constant, row statistics
    auto load_step = [&](int step, bool with_tiles) {
        const int gi = g_lo + step / n_m, mi = s_hi - 1 - step % n_m;  // last query block first: see below
        const int h = hk * G + gi, m0 = mi * BM;
        column_const_load(h);
        ld_qbase = uniform_ptr((const uint16_t *)f.q + b * f.q_b + h * f.q_h + (sq.q0 + m0) * f.q_r);
        ld_dobase = uniform_ptr((const uint16_t *)p.dout + b * p.do_b + h * p.do_h + (sq.q0 + m0) * p.do_r);
        ld_partial = mi == m_last;
        if (with_tiles) {
#pragma unroll
            for (int n = 0; n < 2 * Q_IT; n++) load_item(n);
        }
        // row statistics: raw, unconditional loads from a clamped row (nothing may look at a loaded value here, or the
        // wait for it would also cover the tile loads above); range check and scaling happen in store_step
        {
            const int qq = m0 + (tid & (BM - 1));
            stat_ok = qq < LqS;
            const int qc = stat_ok ? qq : LqS - 1;
            lreg = f.lse[b * f.lse_b + h * f.lse_h + sq.q0 + qc];
            dreg = p.softmax_d[b * p.sd_b + h * p.sd_h + sq.q0 + qc];
        }
    };
    auto store_step = [&](int buf) {
        char *base = smem + buf * SM::STAGE;
#pragma unroll
        for (int it = 0; it < Q_IT; it++) {
            const uint32_t off = TL::chunk(qr0 + it * RPP, qc);
            *(u32x4_t *)(base + off) = qreg[it];
            *(u32x4_t *)(base + SM::Q_BYTES + off) = doreg[it];
        }
        if (tid < BM) {
            ((float *)(base + 2 * SM::Q_BYTES))[tid] = stat_ok ? lreg * kLog2e : INFINITY;
            ((float *)(base + 2 * SM::Q_BYTES + BM * 4))[tid] = stat_ok ? dreg : 0.f;
        }
    };

    // ---- DMA staging: block bases of the step being fetched, and its pieces one by one.  Piece 0 .. 2*Q_IT-1: this
    // wave's Q / dO loads (1 KB each); piece 2*Q_IT (wave 3 only): the row statistics, 32 LSE values and 32 D values
    // as ONE 4-byte load (lanes 0-31 / 32-63), raw -- log2(e) is applied where the LSE is used, and rows beyond the
    // end of the queries are clamped here and masked there.
    typedef __attribute__((address_space(3))) void lds_void_t;
    typedef const __attribute__((address_space(1))) void gvoid_t;
    // The steps are walked with counters and running pointers (no division, no 64-bit products per step): inside a
    // query head the query block index falls by one per step, at a head change everything jumps by loop constants.
    typedef const __attribute__((address_space(1))) char *gbytes_t;
    int dma_gi = g_lo, dma_mi = s_hi - 1;  // head and query block of the step being fetched
    gbytes_t dma_q = nullptr, dma_do = nullptr, dma_stat = nullptr;  // its Q / dO block bases, this lane's statistic
    char *dma_dst = nullptr;
    const int64_t q_step = -(int64_t)BM * f.q_r * 2, do_step = -(int64_t)BM * p.do_r * 2;
    const int64_t q_head = (int64_t)f.q_h * 2 - (int64_t)(n_m - 1) * q_step, do_head = (int64_t)p.do_h * 2 - (int64_t)(n_m - 1) * do_step;
    const int64_t stat_head = (int64_t)(lane < 32 ? f.lse_h : p.sd_h) * 4 + (int64_t)(n_m - 1) * BM * 4;
    if (DMA && n_steps > 0) {
        const int h0 = hk * G + g_lo, m00 = dma_mi * BM;
        dma_q = (gbytes_t)((const uint16_t *)f.q + b * f.q_b + h0 * f.q_h + (sq.q0 + m00) * f.q_r);
        dma_do = (gbytes_t)((const uint16_t *)p.dout + b * p.do_b + h0 * p.do_h + (sq.q0 + m00) * p.do_r);
        dma_stat = (gbytes_t)(lane < 32 ? f.lse + b * f.lse_b + h0 * f.lse_h + sq.q0 + m00 + (lane & 31)
                                        : p.softmax_d + b * p.sd_b + h0 * p.sd_h + sq.q0 + m00 + (lane & 31));
    }
    // sets up the fetch of the step the counters stand at (into stage `buf`)
    auto dma_begin = [&](int buf) {
        ld_qbase = dma_q;
        ld_dobase = dma_do;
        ld_partial = dma_mi == m_last;
        dma_dst = smem + buf * SM::STAGE;
    };
    // moves the counters to the following step; past the last step they stay (its tiles are fetched again and dropped)
    auto dma_advance = [&](bool more) {
        if (!more) return;
        if (dma_mi == s_lo) {
            dma_mi = s_hi - 1;
            dma_gi++;
            dma_q += q_head; dma_do += do_head; dma_stat += stat_head;
        } else {
            dma_mi--;
            dma_q += q_step; dma_do += do_step; dma_stat -= BM * 4;
        }
    };
    // The direct loads are written in assembly and waited for by hand (publish() below): issued through the
    // compiler's builtin, every LDS read behind one of them waited for all LDS operations in flight -- the compiler
    // cannot tell which stage a direct load fills -- and the fragment reads could not run ahead of their MFMAs.
    // (m0 carries the LDS address of a direct load; it is a reserved register that nothing else in this kernel uses.)
    auto dma_piece = [&](int n) {
        const uint32_t dst = lds_addr(dma_dst);
        if (n < Q_IT) {
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         : : "v"(ld_partial ? qoff_l[n] : qoff[n]), "s"(ld_qbase), "s"(__builtin_amdgcn_readfirstlane(dst + (2 * wave + n) * 1024)));
        } else if (n < 2 * Q_IT) {
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         : : "v"(ld_partial ? dooff_l[n - Q_IT] : dooff[n - Q_IT]), "s"(ld_dobase),
                             "s"(__builtin_amdgcn_readfirstlane(dst + SM::Q_BYTES + (2 * wave + n - Q_IT) * 1024)));
        } else {
            // (every wave fetches the same 256 bytes: cheaper than a branch in the middle of the MFMAs.)  In the last,
            // partial block the rows beyond the end of the queries read the last row's numbers (masked where used).
            const int over = ld_partial ? (lane & 31) - row_last : 0;
            gbytes_t sp = dma_stat - (over > 0 ? over * 4 : 0);
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
                         : : "v"(sp), "s"(__builtin_amdgcn_readfirstlane(dst + 2 * SM::Q_BYTES)));
        }
    };
    // end of a step: a wave waits for its own direct loads (and LDS stores), then the barrier publishes everybody's
    auto publish = [&]() {
        if constexpr (DMA) {
            __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0); expcnt not waited for
            __builtin_amdgcn_s_barrier();
        } else {
            __syncthreads();
        }
    };

    const int a_row = pi_row(r);
    const int tj = lane & 15, te = tj >> 2, tc = tj & 3;
    const int tcp = (tc == 1) ? 2 : (tc == 2 ? 1 : tc);
    const int tdh = (lane >> 4) & 1;
    uint32_t tr_off = lds0 + TL::tr_base(g, te, tdh, tcp);  // (absolute LDS addresses of stage 0's Q tile)
    uint32_t a_off = lds0 + TL::frag_base(a_row, g);
    const uint32_t stat_off = lds0 + 32 * g;  // this lane's eight rows of a block of sixteen row statistics

    float colsum = 0.f;
    float cconst = 0.f;

    // Pipeline: step i is computed from LDS stage i & 1.  The registers hold step i+1 (fetched during the dK / dV
    // MFMAs of step i-1, a whole step earlier -- these tiles come from HBM, not from a cache); they go to the other
    // stage between the first GEMM pair and the softmax of step i, and the loads of step i+2 then reuse them, issued
    // one by one between the dK / dV MFMAs (all at once, from every wave at the same moment, they would queue up at the
    // CU's address unit while the matrix pipe idles).
    if (n_steps > 0) {
        if constexpr (DMA) {
            column_const_load(hk * G + g_lo);
            dma_begin(0);
#pragma unroll
            for (int n = 0; n <= 2 * Q_IT; n++) dma_piece(n);
            dma_advance(n_steps > 1);
            cconst = column_const_value();
        } else {
            load_step(0, true);
            store_step(0);
            cconst = column_const_value();
            load_step(n_steps > 1 ? 1 : 0, true);
        }
        publish();
    }

    int cur_gi = g_lo, cur_mi = s_hi - 1;  // (DMA: head and query block of the current step, walked like the fetch)
    // (one step; the LDS stage is a compile-time constant -- the loop below runs the steps in pairs -- so that every
    // stage base folds into the offset field of the LDS instructions instead of costing an addition per access)
    auto one_step = [&](auto buf_c, const int step) {
        constexpr int buf = decltype(buf_c)::value;
        const int gi = DMA ? cur_gi : g_lo + step / n_m, mi = DMA ? cur_mi : s_hi - 1 - step % n_m;  // last query block first: see below
        const int h = hk * G + gi;
        const int m0 = mi * BM;
        // The swizzled addresses are these lane constants XOR a compile-time value: recomputed where they are used
        // (one VALU operation each); hoisted out of the loop they would cost 30 registers that the kernel does not have.
        if (TL::SWZ) asm volatile("" : "+v"(a_off), "+v"(tr_off), "+v"(v_base));
        // DMA: the next step's tiles go to the other stage (its readers finished before the last barrier), a piece
        // every few MFMAs; the column constant is fetched again only when the next step belongs to another query head
        const bool head_next = DMA && step + 1 < n_steps && mi == s_lo;
        if constexpr (DMA) {
            dma_begin(buf ^ 1);
            if (head_next) column_const_load(h + 1);
        }

        // ---- S = Q K^T and dP = dO V^T (M = query, N = key); fragment reads run a batch ahead
        f32x16_t s[MB], dp[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                // (one move per accumulator register, written out: as a plain splat the compiler builds the vector in
                // other registers first and copies it over, 31 instructions for 16)
                asm volatile("v_mov_b32 %0, %1" : "=v"(s[mb][i]) : "v"(cconst));
                dp[mb][i] = 0.f;
            }
        {
            constexpr int NF = 2 * MB * KS, FR = D > 64 ? 3 : 8;  // fragment f: (ks, mb, which) with which = 0: Q, 1: dO
            u32x4_t a[NF];
            auto frag = [&](int fi) {
                const int which = fi & 1, mb = (fi >> 1) % MB, ks = (fi >> 1) / MB;
                return lds_ld128(TL::frag_at(a_off, ks) + (uint32_t)(buf * SM::STAGE + which * SM::Q_BYTES + 32 * mb * TL::ROW_BYTES));
            };
            // (V parked in LDS: its fragment of a k-step is read one k-step ahead as well -- read where it is used, every
            // dP MFMA waited for its own read; a scheduling barrier per MFMA keeps the reads ahead)
            constexpr int FRV = 1;
            u32x4_t vl[V_LDS ? KS : 1];
            if constexpr (V_LDS) {
#pragma unroll
                for (int ks = 0; ks < FRV; ks++) vl[ks] = lds_ld128(TL::frag_at(v_base, ks));
            }
#pragma unroll
            for (int fi = 0; fi < FR; fi++) a[fi] = frag(fi);
#pragma unroll
            for (int fi = 0; fi < NF; fi++) {
                if (fi + FR < NF) a[fi + FR] = frag(fi + FR);
                const int which = fi & 1, mb = (fi >> 1) % MB, ks = (fi >> 1) / MB;
                if constexpr (V_LDS) {
                    if (which && mb == 0 && ks + FRV < KS) vl[ks + FRV] = lds_ld128(TL::frag_at(v_base, ks + FRV));
                }
                if (which) dp[mb] = E::mfma(a[fi], V_LDS ? vl[V_LDS ? ks : 0] : vf[V_LDS ? 0 : ks], dp[mb]);
                else s[mb] = E::mfma(a[fi], kf[ks], s[mb]);
                if constexpr (DMA) {
                    if (fi % 3 == 1 && fi / 3 <= 2 * Q_IT) dma_piece(fi / 3);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the registers (step i+1) go to the other LDS stage, whose readers finished before the last barrier
        __builtin_amdgcn_sched_barrier(0);
        float cconst_next = cconst;
        if constexpr (!DMA) {
            if (step + 1 < n_steps) {
                store_step(buf ^ 1);
                cconst_next = column_const_value();
            }
        }
        __builtin_amdgcn_sched_barrier(0);

        // ---- P = exp2(S - LSE*log2e), S already scaled and offset by the column constant ; dS = P * (dP - D)
        // diagonal step: some (query, key) pairs of this wave are above the causal diagonal
        // (DMA: the statistics are raw, so rows beyond the end of the queries -- clamped duplicates in the last, partial
        // block -- are masked here as well)
        const bool diag = (CAUSAL && (okey_wlast > m0 + shift)) || (DMA && m0 + BM > LqS);
        uint32_t ppk[MB * 8], dpk[MB * 8];
        float part = 0.f;
        // softmax and dS of one block of 16 query rows (8 per lane) in three pieces, so that the MFMAs of the rows whose
        // probabilities are finished can be issued between the pieces of the next block: A = statistics, exp2, dP - D;
        // M = masking (diagonal steps only: rows above the causal diagonal or beyond the end of the queries give
        // P = 0); B = dS, column sum, conversion to 16 bits
        float pv[8], dsv[8];
        auto soft_a = [&](auto mb_c, auto blk_c) {
            constexpr int mb = decltype(mb_c)::value, blk = decltype(blk_c)::value;
            const uint32_t so = buf * SM::STAGE + 2 * SM::Q_BYTES + (32 * mb + 16 * blk) * 4;  // LSE; D is BM floats on
            const f32x4_t l0 = __builtin_bit_cast(f32x4_t, lds_ld128(stat_off + so)), l1 = __builtin_bit_cast(f32x4_t, lds_ld128(stat_off + so + 16));
            const f32x4_t d0 = __builtin_bit_cast(f32x4_t, lds_ld128(stat_off + so + BM * 4)), d1 = __builtin_bit_cast(f32x4_t, lds_ld128(stat_off + so + BM * 4 + 16));
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int ii = 8 * blk + e;
                const float lse2 = e < 4 ? l0[e] : l1[e - 4];
                const float dd = e < 4 ? d0[e] : d1[e - 4];
                pv[e] = fast_exp2(DMA ? __builtin_fmaf(lse2, -kLog2e, s[mb][ii]) : s[mb][ii] - lse2);
                dsv[e] = dp[mb][ii] - dd;
            }
        };
        auto soft_m = [&](auto mb_c, auto blk_c) {
            constexpr int mb = decltype(mb_c)::value, blk = decltype(blk_c)::value;
            if (diag) {
                asm volatile("" ::: "memory");  // keep a real branch: only diagonal steps pay
                int lim = CAUSAL ? okey - shift - m0 - 32 * mb - 16 * blk - 8 * g : 0;  // rows e >= lim see this key
                int lim_hi = DMA ? LqS - m0 - 32 * mb - 16 * blk - 8 * g : 8;            // rows e < lim_hi exist
                asm volatile("" : "+v"(lim), "+v"(lim_hi));  // (the comparisons stay inside the branch)
#pragma unroll
                for (int e = 0; e < 8; e++) pv[e] = (e >= lim && e < lim_hi) ? pv[e] : 0.f;
            }
        };
        auto soft_b = [&](auto mb_c, auto blk_c) {
            constexpr int mb = decltype(mb_c)::value, blk = decltype(blk_c)::value;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                dsv[e] *= pv[e];
                part += dsv[e];
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                ppk[mb * 8 + blk * 4 + e] = E::pack2(pv[2 * e], pv[2 * e + 1]);
                dpk[mb * 8 + blk * 4 + e] = E::pack2(dsv[2 * e], dsv[2 * e + 1]);
            }
        };
        // ---- dV^T += dO^T P ; dK^T += Q^T dS   (M = d, N = key, contraction = query), pairs [idx0, idx1) of (16-row
        // block, d block); the transposing fragment reads run one pair ahead of the MFMAs that use them
        constexpr int NP = (BM / 16) * DB;
        u32x4_t a1[2], a2[2];
        auto tr_frag = [&](int idx, int slot) {
            const int qb = idx / DB, db = idx % DB;
            const uint32_t off = TL::tr_at(tr_off, qb, db, 0), off_hi = TL::tr_at(tr_off, qb, db, 1);
            constexpr uint32_t st = buf * SM::STAGE;
            const u32x2_t lo = lds_ld_tr16(off + st + SM::Q_BYTES), hi = lds_ld_tr16(off_hi + st + SM::Q_BYTES);
            const u32x2_t lo2 = lds_ld_tr16(off + st), hi2 = lds_ld_tr16(off_hi + st);
            a1[slot] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
            a2[slot] = u32x4_t{lo2[0], lo2[1], hi2[0], hi2[1]};
        };
        auto gemm2 = [&](auto idx0_c, auto idx1_c) {
            constexpr int idx0 = decltype(idx0_c)::value, idx1 = decltype(idx1_c)::value;
#pragma unroll
            for (int idx = idx0; idx < idx1; idx++) {
                if (idx + 1 < NP) tr_frag(idx + 1, (idx + 1) & 1);
                const int qb = idx / DB, db = idx % DB;
                const u32x4_t pb = {ppk[4 * qb], ppk[4 * qb + 1], ppk[4 * qb + 2], ppk[4 * qb + 3]};
                const u32x4_t sb = {dpk[4 * qb], dpk[4 * qb + 1], dpk[4 * qb + 2], dpk[4 * qb + 3]};
                dv[db] = E::mfma(a1[idx & 1], pb, dv[db]);
                dk[db] = E::mfma(a2[idx & 1], sb, dk[db]);
                if constexpr (!DMA) {
#pragma unroll
                    for (int n = idx * 2 * Q_IT / NP; n < (idx + 1) * 2 * Q_IT / NP; n++) load_item(n);
                }
            }
        };
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        // (after the last steps an existing tile is fetched again and dropped)
        if constexpr (!DMA) load_step(step + 2 < n_steps ? step + 2 : step, false);
        if constexpr (MB == 1) {
            // the MFMAs of the first 16 rows need the probabilities of those rows only: the softmax of the other 16
            // rows is issued between them
            soft_a(I0(), I0()); soft_m(I0(), I0()); soft_b(I0(), I0());
            tr_frag(0, 0);
            gemm2(I0(), std::integral_constant<int, DB / 2>());
            soft_a(I0(), I1());
            soft_m(I0(), I1());
            gemm2(std::integral_constant<int, DB / 2>(), std::integral_constant<int, DB>());
            soft_b(I0(), I1());
            gemm2(std::integral_constant<int, DB>(), std::integral_constant<int, NP>());
        } else {
            static_assert(MB <= 2, "steps of 32 or 64 query rows");
            soft_a(I0(), I0()); soft_m(I0(), I0()); soft_b(I0(), I0());
            soft_a(I0(), I1()); soft_m(I0(), I1()); soft_b(I0(), I1());
            soft_a(I1(), I0()); soft_m(I1(), I0()); soft_b(I1(), I0());
            soft_a(I1(), I1()); soft_m(I1(), I1()); soft_b(I1(), I1());
            tr_frag(0, 0);
            gemm2(I0(), std::integral_constant<int, NP>());
            // pin the order: reads of pair idx+1, then the two MFMAs of pair idx
            __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
            for (int idx = 0; idx < NP; idx++) {
                if (idx + 1 < NP) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
        }
        colsum += part;

        // ---- dBias column sum: flush when the bias head changes
        if (has_bias) {
            const bool last_m = mi == s_lo;
            if (last_m && (slot >= 0 || f.Hb == f.H || gi == G - 1)) {
                const float tot = xhalf_sum(colsum);
                const int hb = f.Hb == f.H ? h : (f.Hb == 1 ? 0 : hk);
                if (slot >= 0) {  // per-head partial column sums; the reduce kernel folds them
                    if (g == 0) p.db_part[((int64_t)slot * G + (gi - g_lo)) * KV_BN + (key - n0)] = tot;
                } else if (g == 0 && key < Lk) {
                    if (use_accum) atomicAdd(p.dbias_accum + b * p.dba_b + hb * p.dba_h + okey, tot);
                    else ((uint16_t *)p.dbias)[b * p.db_b + hb * p.db_h + okey] = (uint16_t)(E::pack2(tot, 0.f) & 0xffffu);
                }
                colsum = 0.f;
            }
        }

        if constexpr (DMA) {
            if (head_next) cconst = column_const_value();
            dma_advance(step + 2 < n_steps);
            if (cur_mi == s_lo) { cur_mi = s_hi - 1; cur_gi++; } else cur_mi--;
        } else {
            cconst = cconst_next;
        }
        publish();
    };
    for (int step = 0; step < n_steps; step += 2) {
        one_step(std::integral_constant<int, 0>(), step);
        if (step + 1 < n_steps) one_step(std::integral_constant<int, 1>(), step + 1);
    }

    // a key block that no query can see still owns its dbias column
    if (has_bias && n_steps == 0 && slot >= 0 && g == 0) {
        for (int gl = 0; gl < g_hi - g_lo; gl++) p.db_part[((int64_t)slot * G + gl) * KV_BN + (key - n0)] = 0.f;
    }
    if (has_bias && n_steps == 0 && slot < 0 && !use_accum && g == 0 && key < Lk) {
        const int ngh = (f.Hb == f.H) ? G : 1;
        for (int gh = 0; gh < ngh; gh++) {
            const int hb = f.Hb == f.H ? hk * G + gh : (f.Hb == 1 ? 0 : hk);
            ((uint16_t *)p.dbias)[b * p.db_b + hb * p.db_h + okey] = 0;
        }
    }

    // ---- shared block: fp32 partial dK^T / dV^T, [which][d][key] so that a wave writes 128-byte runs
    if (slot >= 0) {
        float *pk = p.dkv_part + (int64_t)slot * 2 * D * KV_BN + (key - n0);
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int dcol = 32 * db + 16 * (i >> 3) + 8 * g + (i & 7);
                pk[dcol * KV_BN] = dk[db][i];
                pk[(D + dcol) * KV_BN] = dv[db][i];
            }
        return;
    }

    // ---- store dK (scaled) and dV
    if (key < Lk) {
        uint16_t *dkp = (uint16_t *)p.dk + b * p.dk_b + (sq.k0 + okey) * p.dk_r + hk * p.dk_h;
        uint16_t *dvp = (uint16_t *)p.dv + b * p.dv_b + (sq.k0 + okey) * p.dv_r + hk * p.dv_h;
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

// Sums the partial results of one unit that the compacted dK/dV kernel split over several workgroups, in a fixed
// order, and writes dK (scaled), dV and dBias to the original rows / columns of the kept keys.  `y` picks a pair of
// 8-wide head-dim chunks (0 .. D/16 - 1), so that few units still give many work items; item y == 0 also folds the
// unit's dBias columns.  Called by the workgroups that the dQ launch sets aside for it (see bwd_dq_colmask_kernel).
template <typename T, int D>
__device__ __forceinline__ void dkdv_reduce_item(const BwdParams &p, const int unit, const int y) {
    using E = Elem<T>;
    const FwdParams &f = p.f;
    const int32_t *plan = f.cmp.plan;
    const int Gs = plan[1], Sm = plan[2], Q = plan[4], per = Gs * Sm;
    // a plan whose lists overflowed left parts uncomputed: every sum starts from NaN then
    const float start = plan[6] != 0 ? __builtin_nanf("") : 0.f;
    int lo = 0, hi = f.B * f.Hk;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (plan[DKDV_PLAN_HDR + mid] <= unit) lo = mid;
        else hi = mid;
    }
    const int pair = lo, b = pair / f.Hk, hk = pair % f.Hk;
    const int n0 = (unit - plan[DKDV_PLAN_HDR + pair]) * KV_BN;
    const int Lk = f.cmp.count[pair];
    const int G = f.H / f.Hk;
    const int tid = threadIdx.x, kk = tid % KV_BN, half = tid / KV_BN;
    const bool live = n0 + kk < Lk;
    const int okey = live ? f.cmp.idx[(int64_t)pair * f.cmp.ld + n0 + kk] : 0;
    // segments of this unit that were written (same rule as in the main kernel)
    const int n_seg = dkdv_segments(dkdv_query_blocks(f.Lq, f.Lk, f.causal, f.cmp.idx[(int64_t)pair * f.cmp.ld + n0]), Q, Sm);
    const float *base = p.dkv_part + (int64_t)unit * per * 2 * D * KV_BN + kk;
    for (int c = 2 * y + half; c == 2 * y + half && c * 8 < f.d; c += NTHREADS / KV_BN) {
        float ak[8], av[8];
#pragma unroll
        for (int e = 0; e < 8; e++) { ak[e] = start; av[e] = start; }
        // written slots in a fixed order, four at a time: a workgroup here sits beside the dQ workgroups and should
        // give its place back soon, so the loads of four slots are in flight together (slots past the end repeat
        // the last one and are not added)
        const int n_w = Gs * n_seg;
        for (int j = 0; j < n_w; j += 4) {
            float kq[4][8], vq[4][8];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int jt = j + t < n_w ? j + t : n_w - 1;
                const float *pt = base + (int64_t)((jt / n_seg) * Sm + jt % n_seg) * 2 * D * KV_BN;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    kq[t][e] = pt[(c * 8 + e) * KV_BN];
                    vq[t][e] = pt[(D + c * 8 + e) * KV_BN];
                }
            }
#pragma unroll
            for (int t = 0; t < 4; t++)
                if (j + t < n_w) {
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        ak[e] += kq[t][e];
                        av[e] += vq[t][e];
                    }
                }
        }
        if (live) {
            u32x4_t wk, wv;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                wk[e] = E::pack2(ak[2 * e] * f.scale, ak[2 * e + 1] * f.scale);
                wv[e] = E::pack2(av[2 * e], av[2 * e + 1]);
            }
            *(u32x4_t *)((uint16_t *)p.dk + b * p.dk_b + (int64_t)okey * p.dk_r + hk * p.dk_h + c * 8) = wk;
            *(u32x4_t *)((uint16_t *)p.dv + b * p.dv_b + (int64_t)okey * p.dv_r + hk * p.dv_h + c * 8) = wv;
        }
    }
    if (f.bias && live && y == 0) {
        const int gper = G / Gs;
        const float *dbp = p.db_part + (int64_t)unit * per * G * KV_BN + kk;  // [part][local head][key]
        auto emit = [&](int hb, float tot) {
            if (p.dbias_accum) atomicAdd(p.dbias_accum + b * p.dba_b + hb * p.dba_h + okey, tot);
            else ((uint16_t *)p.dbias)[b * p.db_b + hb * p.db_h + okey] = (uint16_t)(E::pack2(tot, 0.f) & 0xffffu);
        };
        if (f.Hb == f.H) {
            for (int gi = half; gi < G; gi += NTHREADS / KV_BN) {
                float tot = start;
                for (int sg = 0; sg < n_seg; sg++) tot += dbp[((int64_t)((gi / gper) * Sm + sg) * G + gi % gper) * KV_BN];
                emit(hk * G + gi, tot);
            }
        } else if (half == 0) {
            float tot = start;
            for (int gs = 0; gs < Gs; gs++)
                for (int sg = 0; sg < n_seg; sg++)
                    for (int gl = 0; gl < gper; gl++) tot += dbp[((int64_t)(gs * Sm + sg) * G + gl) * KV_BN];
            emit(f.Hb == 1 ? 0 : hk, tot);
        }
    }
}

// Workgroup `rb` of `nrb` reducing workgroups takes every nrb-th of the U units x D/16 chunk pairs.  The first item
// goes to the workgroup in the middle: when there are fewer items than workgroups (few units, each cut into many
// parts: long sums) they run in the middle of the launch's interleaved stretch, neither beside the heaviest dQ
// workgroups at its start nor in its tail.
template <typename T, int D>
__device__ __forceinline__ void dkdv_reduce_blocks(const BwdParams &p, const int rb, const int nrb) {
    const int32_t *plan = p.f.cmp.plan;
    const int U = plan[0];
    if (plan[1] * plan[2] == 1) return;  // no unit was split: the dK/dV kernel wrote the results itself
    const int first = rb >= nrb / 2 ? rb - nrb / 2 : rb + nrb - nrb / 2;
    for (int item = first; item < U * (D / 16); item += nrb) dkdv_reduce_item<T, D>(p, item / (D / 16), item % (D / 16));
}

// The dQ launch of a compacted backward carries the reduction of the dK/dV partials along: `red_octets` groups of 8
// consecutive workgroups (one per XCD) do that instead of dQ work, one such group after every `period - 1` groups
// of dQ workgroups.  The reduction only moves memory while the dQ workgroups keep the matrix units busy, so side by
// side it costs next to nothing; as a launch of its own it took as long as its memory traffic.
struct RedInterleave {
    int red_octets, period, start;
};
inline RedInterleave red_interleave(int dq_octets, int items) {
    RedInterleave r;
    r.red_octets = (items < 1024 ? items : 1024) / 8;
    if (r.red_octets < 1) r.red_octets = 1;
    r.period = (dq_octets + r.red_octets) / r.red_octets;
    r.period = r.period < 2 ? 2 : (r.period > 4 ? 4 : r.period);
    if (r.red_octets > dq_octets / (r.period - 1)) r.red_octets = dq_octets / (r.period - 1);
    if (r.red_octets < 1) r.red_octets = 1;  // (dq_octets >= 1 and period == 2 then)
    // the interleaved stretch ends with the launch; the dQ groups in front of it are the heaviest ones
    r.start = dq_octets - r.red_octets * (r.period - 1);
    return r;
}

template <typename T, int D, bool CAUSAL, bool CMP>
hipError_t launch_dkdv_c(const BwdParams &p, hipStream_t stream) {
    const FwdParams &f = p.f;
    auto kern = bwd_dkdv_colmask_kernel<T, D, CAUSAL, CMP>;
    const int smem = KvcSmem<D>::TOTAL;
    static DynSmemLimit smem_limit;
    hipError_t e = smem_limit.ensure((const void *)kern, (int)smem);
    if (e != hipSuccess) return e;
    if (CMP) {
        int grid, slots;
        dkdv_split_bounds(f.B * f.Hk, (f.Lk + KV_BN - 1) / KV_BN, f.H / f.Hk, grid, slots);
        hipLaunchKernelGGL(kern, dim3(grid), dim3(NTHREADS), smem, stream, p);
        return hipGetLastError();  // (the partial results are summed by workgroups of the dQ launch)
    }
    dim3 grid(xcd_grid(f.B * f.Hk, (f.Lk + KV_BN - 1) / KV_BN, 1));
    hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), smem, stream, p);
    return hipGetLastError();
}
template <typename T, int D, bool CAUSAL>
hipError_t launch_dkdv(const BwdParams &p, hipStream_t stream) {
    return p.f.cmp.on ? launch_dkdv_c<T, D, CAUSAL, true>(p, stream) : launch_dkdv_c<T, D, CAUSAL, false>(p, stream);
}


// ------------------------------------------------------------------------------------------------
// dQ
// ------------------------------------------------------------------------------------------------
constexpr int Q_BM = 128;
constexpr int MAX_TILES = 16384;


template <int D, int BN> struct DqcSmem {
    static constexpr int S = LdsTile<D>::S;
    static constexpr int K_BYTES = BN * S * 2;
    static constexpr int NST = LdsTile<D>::SWZ ? 3 : 2;  // K / V stages: three where the tiles are fetched two ahead
    static constexpr int OFF_K = 0;
    static constexpr int OFF_V = OFF_K + NST * K_BYTES;
    static constexpr int OFF_BIAS = OFF_V + NST * K_BYTES;
    static constexpr int OFF_BITS = OFF_BIAS + 3 * 256;  // three bias columns (a direct load fills 256 bytes)
    static constexpr int TOTAL = OFF_BITS + MAX_TILES / 8;
};

template <typename T, int D, int BN, bool CAUSAL, bool CMP>
__global__ void __launch_bounds__(NTHREADS, D <= 128 ? 2 : 1) bwd_dq_colmask_kernel(const BwdParams p) {
    using E = Elem<T>;
    using SM = DqcSmem<D, BN>;
    using TL = LdsTile<D>;
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int MB = BN / 32;
    constexpr int KB = BN / 16;
    constexpr int CH = D / 8, RPP = NTHREADS / CH, K_IT = BN / RPP;
    // DMA (compacted keys, rows of exactly 256 bytes): the K / V tiles and the fused bias column go from global memory
    // straight into LDS (global_load_lds: a wave writes 64 consecutive 16-byte or 4-byte pieces, so the swizzle of the
    // tile is applied to the GLOBAL address of each lane's piece), TWO tiles ahead, into a third stage: no staging
    // registers, no LDS stores, and a tile has a whole tile time more to arrive.  (Through registers, loaded between the
    // MFMAs of the tile whose end stores them, the stores waited for the loads: without the loads the kernel was 12 %
    // shorter.)  The instruction is written in assembly: issued through the compiler's builtin, every later LDS read
    // waited for ALL direct loads in flight -- the compiler cannot tell which stage they fill -- and the loads of
    // the tile after the next one would be waited for at once.  The waits are placed by hand (publish()).
    constexpr bool DMA = TL::SWZ && CMP;
    constexpr int NST = SM::NST;
    static_assert(!DMA || (RPP == 16 && NTHREADS == 256), "the direct loads are laid out for 16 chunks per row and four waves");

    // (LDS is read and written by absolute address in the tile loop: an access through a pointer into `smem` makes the
    // compiler wait for every direct load in flight first)
    extern __shared__ __attribute__((aligned(256))) char smem[];
    const uint32_t lds0 = lds_addr(smem);  // (a multiple of 256)
    uint32_t *sBits = (uint32_t *)(smem + SM::OFF_BITS);

    const FwdParams &f = p.f;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = tid & 63, r = lane & 31, g = lane >> 5;
    const int G = f.H / f.Hk;
    const int n_mb = (f.Lq + Q_BM - 1) / Q_BM;
    int lid = blockIdx.x;  // index among the dQ workgroups
    if (CMP) {
        // groups of 8 workgroups (one per XCD): every `period`-th of the first red_octets * period groups sums
        // partial results of the dK/dV kernel instead
        const int R = p.red_octets, period = p.red_period;
        int o = lid >> 3;
        const int o2 = o - p.red_start;  // the groups before red_start are all dQ groups
        if (o2 >= 0) {
            if (o2 < R * period) {
                if (o2 % period == period - 1) {
                    dkdv_reduce_blocks<T, D>(p, (o2 / period) * 8 + (lid & 7), R * 8);
                    return;
                }
                o -= o2 / period;
            } else {
                o -= R;
            }
        }
        lid = o * 8 + (lid & 7);
    }
    const XcdMap wm = xcd_map(lid, f.B * f.Hk, n_mb, G);
    if (!wm.valid) return;
    const int m_block = n_mb - 1 - wm.unit;  // heaviest first under causal
    const int b = wm.pair / f.Hk, hk = wm.pair % f.Hk;
    const int h = hk * G + (lid / 8) % G;
    const int m0 = m_block * Q_BM;
    const SeqInfo sq = seq_info(f, b);  // this batch entry's lengths and first rows (ragged batch: from cu_seqlens)
    const int LqS = sq.Lq, LkS = sq.Lk;
    if (m0 >= LqS) return;
    const int qrow = m0 + wave * 32 + r;
    const int qrow_c = qrow < LqS ? qrow : LqS - 1;
    const int shift = LkS - LqS;

    const int hm = f.mask ? (f.Hm == f.H ? h : (f.Hm == 1 ? 0 : hk)) : 0;
    const int hb = f.bias ? (f.Hb == f.H ? h : (f.Hb == 1 ? 0 : hk)) : 0;
    const uint8_t *mrow = f.mask ? f.mask + b * f.m_b + hm * f.m_h : nullptr;
    const uint16_t *brow = f.bias ? (const uint16_t *)f.bias + b * f.bi_b + hb * f.bi_h : nullptr;
    const uint16_t *kbase = (const uint16_t *)f.k + b * f.k_b + sq.k0 * f.k_r + hk * f.k_h;
    const uint16_t *vbase = (const uint16_t *)f.v + b * f.v_b + sq.k0 * f.v_r + hk * f.v_h;

    // key columns this workgroup iterates over (the compacted list with CMP), and how many a row may see
    const int Lk = CMP ? f.cmp.count[wm.pair] : LkS;
    const int32_t *ccnt = CMP ? f.cmp.cnt + (int64_t)wm.pair * f.cmp.ld : nullptr;
    const float *fbrow = CMP ? f.cmp.fb + (int64_t)(b * f.cmp.Hfb + (f.cmp.Hfb == f.H ? h : hk)) * f.cmp.ld : nullptr;
    auto visible = [&](int row) -> int {  // columns [0, visible(row)) pass the causal test for `row`
        if (row >= LqS) row = LqS - 1;
        const int c = row + shift;
        if (!CMP) return c + 1;
        if (c < 0) return 0;
        return ccnt[c < LkS ? c : LkS - 1];
    };
    const int vis_lane = CAUSAL ? visible(qrow) : 0;
    const int vis_wave = CAUSAL ? visible(m0 + wave * 32) : 0;

    int n_end = (Lk + BN - 1) / BN;
    if (CAUSAL) {
        int lim = visible(m0 + Q_BM - 1);
        if (lim < 0) lim = 0;
        const int ne = (lim + BN - 1) / BN;
        if (ne < n_end) n_end = ne;
    }

    // ---- active-tile bitmap (tiles with at least one kept key)
    for (int base = 0; !CMP && base < n_end; base += NTHREADS) {
        const int j = base + tid;
        bool act = false;
        if (j < n_end) {
            if (mrow) {
                uint32_t any = 0;
#pragma unroll
                for (int c = 0; c < BN / 16; c++) {
                    const int col = j * BN + c * 16;
                    if (col < LkS) {
                        const u32x4_t mv = *(const u32x4_t *)(mrow + col);
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
    auto next_active = [&](int j) -> int {  // wave-uniform: keeps tile bases and loop conditions scalar
        if (CMP) return j < n_end ? j : n_end;
        while (j < n_end) {
            const uint32_t w = __builtin_amdgcn_readfirstlane(lds_ld32(lds0 + SM::OFF_BITS + 4 * (j >> 5))) >> (j & 31);
            if (w) {
                j += __builtin_ctz(w);
                return j < n_end ? j : n_end;
            }
            j = (j | 31) + 1;
        }
        return n_end;
    };

    // ---- Q and dO fragments (B operands), row statistics
    u32x4_t qf[KS], dof[KS];
    {
        const uint16_t *qp = (const uint16_t *)f.q + b * f.q_b + (sq.q0 + qrow_c) * f.q_r + h * f.q_h;
        const uint16_t *dp = (const uint16_t *)p.dout + b * p.do_b + (sq.q0 + qrow_c) * p.do_r + h * p.do_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + g * 8;
            u32x4_t qv = {0, 0, 0, 0}, dv = {0, 0, 0, 0};
            if (qrow < LqS && c < f.d) { qv = *(const u32x4_t *)(qp + c); dv = *(const u32x4_t *)(dp + c); }
            // Q only feeds the scores in this kernel: scale it by softmax_scale * log2(e) once
#pragma unroll
            for (int e = 0; e < 4; e++) qv[e] = E::pack2(E::lo(qv[e]) * f.scale_log2, E::hi(qv[e]) * f.scale_log2);
            qf[ks] = qv;
            dof[ks] = dv;
        }
    }
    float lse2 = INFINITY, dd = 0.f;
    if (qrow < LqS) {
        lse2 = f.lse[b * f.lse_b + h * f.lse_h + sq.q0 + qrow] * kLog2e;
        dd = p.softmax_d[b * p.sd_b + h * p.sd_h + sq.q0 + qrow];
    }

    f32x16_t dq[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) dq[db][i] = 0.f;

    // ---- staging: rows beyond Lk are clamped (their fused bias is -inf), head-dim chunks beyond d re-read chunk 0
    const int kc = tid % CH, kr0 = tid / CH;
    // (DMA: the lane fills chunk POSITION kc of its row, which holds chunk kc ^ swz(row) of the global row; rows 16
    // apart have the same swizzle)
    const int kc_g = DMA ? (kc ^ (int)TL::swz(kr0)) : kc;
    const int kcol = (kc_g * 8 < f.d) ? kc_g * 8 : 0;
    u32x4_t kreg[DMA ? 1 : K_IT], vreg[DMA ? 1 : K_IT];
    // Byte offsets of this thread's loads inside a tile are loop invariants -- one set for full tiles, one for the
    // (only) partial tile at the end of the keys -- so a load is one instruction with a scalar tile base, and the
    // loads of the next tile can be issued one by one between the MFMAs of the current one.  The bias / mask of the
    // thread's column travel as raw, unconditional loads (an absent one is read from K and ignored) and are looked
    // at when they are stored.
    typedef const __attribute__((address_space(1))) char *gptr_t;
    auto uniform_ptr = [](const void *ptr) -> gptr_t {
        const uint64_t v = (uint64_t)ptr;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (gptr_t)(((uint64_t)hi << 32) | lo);
    };
    const int j_last = Lk > 0 ? (Lk - 1) / BN : 0, last_row = Lk > 0 ? (Lk - 1) % BN : 0;
    uint32_t koff[K_IT], koff_l[K_IT], voff[K_IT], voff_l[K_IT];
#pragma unroll
    for (int it = 0; it < K_IT; it++) {
        const int row = kr0 + it * RPP, row_c = row < last_row ? row : last_row;
        koff[it] = (uint32_t)(row * f.k_r + kcol) * 2;
        koff_l[it] = (uint32_t)(row_c * f.k_r + kcol) * 2;
        voff[it] = (uint32_t)(row * f.v_r + kcol) * 2;
        voff_l[it] = (uint32_t)(row_c * f.v_r + kcol) * 2;
    }
    gptr_t tb_k = nullptr, tb_v = nullptr;
    bool t_last = false, bcol_ok = false;
    uint32_t braw = 0, mraw = 0;
    const uint8_t *mrow_ld = mrow ? mrow : (const uint8_t *)kbase;
    const uint16_t *brow_ld = brow ? brow : kbase;
    gptr_t tb_b = nullptr;  // DMA: the fused bias row, and this lane's offset in it for the tile being fetched
    uint32_t boff = 0;
    // bases of the tile whose K / V are fetched next; the bias / mask column of tile jb
    auto set_tile = [&](int j, int jb) {
        tb_k = uniform_ptr(kbase + (int64_t)j * BN * f.k_r);
        tb_v = uniform_ptr(vbase + (int64_t)j * BN * f.v_r);
        t_last = j == j_last;
        if constexpr (DMA) {
            // columns beyond the end of the kept keys read the last one (masked where the column is used)
            tb_b = uniform_ptr(fbrow);
            const int col = j * BN + (lane & 31);
            boff = (uint32_t)(col < Lk ? col : Lk - 1) * 4u;
        }
        if (!DMA && tid < BN) {
            j = jb;
            const int col = j * BN + tid;
            bcol_ok = col < Lk;
            const int cc = bcol_ok ? col : 0;
            if (CMP) {
                braw = __float_as_uint(fbrow[cc]);
            } else {
                mraw = mrow_ld[cc];
                braw = brow_ld[cc];
            }
        }
    };
    // one direct load: 64 lanes x 16 (or 4) bytes from `base` (wave-uniform) + this lane's offset to LDS address `dst`
    // (wave-uniform) onwards, lane after lane.  (m0 carries the LDS address; it is a reserved register that nothing
    // else in this kernel uses, and it is written immediately in front of every use.)
    auto dma16 = [](gptr_t base, uint32_t off, uint32_t dst) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(base), "s"(dst));
    };
    auto dma4 = [](gptr_t base, uint32_t off, uint32_t dst) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" : : "v"(off), "s"(base), "s"(dst));
    };
    constexpr int N_DMA = 2 * K_IT + 1;  // direct loads of a wave per tile
    int dma_stage = 0;                   // stage the tile being fetched goes to (DMA)
    auto load_item = [&](int n) {  // 0 .. K_IT-1: K rows, K_IT .. 2*K_IT-1: V rows, 2*K_IT: the bias column (DMA)
        if constexpr (DMA) {
            // this wave's piece `it` of a tile: LDS bytes [1024 (wave + 4 it), + 1024), rows 4 wave + 16 it .. + 3
            const uint32_t st0 = lds0 + (uint32_t)(dma_stage * SM::K_BYTES);
            if (n < K_IT) dma16(tb_k, t_last ? koff_l[n] : koff[n], __builtin_amdgcn_readfirstlane(st0 + SM::OFF_K + (wave + 4 * n) * 1024));
            else if (n < 2 * K_IT)
                dma16(tb_v, t_last ? voff_l[n - K_IT] : voff[n - K_IT], __builtin_amdgcn_readfirstlane(st0 + SM::OFF_V + (wave + 4 * (n - K_IT)) * 1024));
            else  // (every wave fetches the same 256 bytes -- lanes 32-63 repeat lanes 0-31 -- : no branch between the MFMAs)
                dma4(tb_b, boff, __builtin_amdgcn_readfirstlane(lds0 + SM::OFF_BIAS + dma_stage * 256));
        } else {
            if (n < K_IT) kreg[n] = *(const __attribute__((address_space(1))) u32x4_t *)(tb_k + (t_last ? koff_l[n] : koff[n]));
            else if (n < 2 * K_IT) vreg[n - K_IT] = *(const __attribute__((address_space(1))) u32x4_t *)(tb_v + (t_last ? voff_l[n - K_IT] : voff[n - K_IT]));
        }
    };
    auto load_tile = [&](int j, int jb) {
        set_tile(j, jb);
#pragma unroll
        for (int n = 0; n < (DMA ? N_DMA : 2 * K_IT); n++) load_item(n);
    };
    // registers -> LDS stage `buf` (not with DMA), and the fused bias column of that tile into slot `slot`
    auto store_tile = [&](int buf, int slot) {
        if constexpr (!DMA) {
            char *sK = smem + SM::OFF_K + buf * SM::K_BYTES;
            char *sV = smem + SM::OFF_V + buf * SM::K_BYTES;
#pragma unroll
            for (int it = 0; it < K_IT; it++) {
                const uint32_t off = TL::chunk(kr0 + it * RPP, kc);
                *(u32x4_t *)(sK + off) = kreg[it];
                *(u32x4_t *)(sV + off) = vreg[it];
            }
        }
        if (!DMA && tid < BN) {
            float v = -INFINITY;
            if (CMP) {
                if (bcol_ok) v = __uint_as_float(braw);
            } else if (bcol_ok && (!mrow || mraw)) {
                v = brow ? E::lo(braw) * kLog2e : 0.f;
            }
            lds_st32(lds0 + SM::OFF_BIAS + 4 * (slot * BN + tid), __float_as_uint(v));
        }
    };

    const int a_row = pi_row(r);
    const uint32_t a_off = lds0 + SM::OFF_K + TL::frag_base(a_row, g);  // (absolute, stage 0 of K)
    const int tj = lane & 15, te = tj >> 2, tc = tj & 3;
    const int tcp = (tc == 1) ? 2 : (tc == 2 ? 1 : tc);
    const int tdh = (lane >> 4) & 1;
    const uint32_t tr_off = lds0 + SM::OFF_K + TL::tr_base(g, te, tdh, tcp);

    // A wave waits for its own pieces of the next tile, then the barrier publishes everybody's (DMA: by hand -- the
    // N_DMA loads of the tile after that, issued later, stay in flight; vmcnt in bits 3:0, lgkmcnt 0, expcnt not
    // waited for)
    auto publish = [&]() {
        if constexpr (DMA) {
            __builtin_amdgcn_s_waitcnt(0x0070 | N_DMA);
            __builtin_amdgcn_s_barrier();
        } else {
            __syncthreads();
        }
    };
    int jc = next_active(0), jn = n_end, jnn = n_end;
    if (jc < n_end) {
        jn = next_active(jc + 1);
        load_tile(jc, jc);
        store_tile(0, 0);
        if constexpr (DMA) {  // the second tile is on its way before the first is looked at
            jnn = next_active(jn + 1);
            dma_stage = 1;
            load_tile(jn < n_end ? jn : jc, jc);
        }
        publish();
    }
    int i = 0;
    constexpr bool S_EARLY = DMA && MB == 1;
    f32x16_t s[MB];
    while (jc < n_end) {
        if constexpr (!DMA) jn = next_active(jc + 1);
        const int n0 = jc * BN;
        const int st = DMA ? i % 3 : (i & 1);
        const uint32_t st_off = (uint32_t)(st * SM::K_BYTES);  // (a multiple of 256: the swizzles stay XORs)
        const uint32_t a_cur = a_off + st_off, tr_cur = tr_off + st_off;
        const uint32_t bs = lds0 + SM::OFF_BIAS + (DMA ? (i % 3) * 256 + 32 * g : 4 * ((i % 3) * BN + 8 * g));

        // ---- S^T = K Q^T, dP^T = V dO^T, dS^T = P^T * (dP^T - D), dQ^T += K^T dS^T.  A wave issues in program
        // order, so the vector work has to sit BETWEEN the MFMAs to run under them; the tile is written slot by slot --
        // one MFMA, the fragment read of the MFMA FR slots later, a share of the vector work, a piece of the next tile's
        // loads -- with a scheduling barrier after every slot:
        //   slots of S (all k-steps), then slots of dP with the exp2 of the finished scores between them, then the dQ
        //   slots of one 16-key block with the dS arithmetic of the next block between them.
        // The score accumulators start from the fused bias vector minus the row's log-sum-exp and the dP accumulators
        // from minus D, so that the MFMAs deliver the exp2 argument and dP - D themselves.
        // (direct loads: every wave fetches the whole bias column of a tile itself, two tiles ahead, so a wave can read
        // the next tile's column as soon as its own load has landed; the score accumulators of the NEXT tile are set up
        // between the last dQ MFMAs of this one -- `s` is free from the last exp2 on -- instead of in front of the first
        // MFMA, where nothing covers the LDS reads and the 16 subtractions)
        f32x16_t dp[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                if (!S_EARLY || i == 0) {
                    const f32x4_t b0 = __builtin_bit_cast(f32x4_t, lds_ld128(bs + 4 * (32 * mb + 16 * blk)));
                    const f32x4_t b1 = __builtin_bit_cast(f32x4_t, lds_ld128(bs + 4 * (32 * mb + 16 * blk + 4)));
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        s[mb][8 * blk + e] = b0[e] - lse2;
                        s[mb][8 * blk + 4 + e] = b1[e] - lse2;
                    }
                }
#pragma unroll
                for (int e = 0; e < 8; e++) dp[mb][8 * blk + e] = -dd;
                if (DMA && jc == j_last) {  // (the bias column came as it is in memory: columns beyond the kept keys)
                    const int lim = Lk - n0 - 32 * mb - 16 * blk - 8 * g;  // local columns e < lim exist
#pragma unroll
                    for (int e = 0; e < 8; e++) s[mb][8 * blk + e] = e < lim ? s[mb][8 * blk + e] : -INFINITY;
                }
            }
        // the next tile's bases and side inputs (after the last tile the current one is fetched again and dropped); behind
        // the accumulator set-up: the load of the bias / mask column must not be waited for with the LDS reads above
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (DMA) {  // K / V of the tile after the next one into the stage the last tile has left
            dma_stage = (i + 2) % 3;
            set_tile(jnn < n_end ? jnn : jc, jn < n_end ? jn : jc);
        } else {
            set_tile(jn < n_end ? jn : jc, jn < n_end ? jn : jc);
        }
        float pv[16 * MB];
        {
            constexpr int NH = MB * KS, NF = 2 * NH, FR = 3;
            u32x4_t a[NF];
            auto frag = [&](int fi) {  // S slots first (K tile), then dP slots (V tile); k-step major, row block minor
                const int which = fi / NH, mb = (fi % NH) % MB, ks = (fi % NH) / MB;
                return lds_ld128(TL::frag_at(a_cur, ks) + (uint32_t)(which * (SM::OFF_V - SM::OFF_K) + 32 * mb * TL::ROW_BYTES));
            };
#pragma unroll
            for (int fi = 0; fi < FR; fi++) a[fi] = frag(fi);
#pragma unroll
            for (int fi = 0; fi < NF; fi++) {
                if (fi + FR < NF) a[fi + FR] = frag(fi + FR);
                const int which = fi / NH, mb = (fi % NH) % MB, ks = (fi % NH) / MB;
                if (which) dp[mb] = E::mfma(a[fi], dof[ks], dp[mb]);
                else s[mb] = E::mfma(a[fi], qf[ks], s[mb]);
                constexpr int NLD = DMA ? N_DMA : 2 * K_IT;
#pragma unroll
                for (int n = fi * NLD / NF; n < (fi + 1) * NLD / NF; n++) load_item(n);
                if (which) {
#pragma unroll
                    for (int e = 0; e < 16 * MB; e++)
                        if (e * NH / (16 * MB) == fi - NH) pv[e] = fast_exp2(s[e / 16][e % 16]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        const bool diag = CAUSAL && (n0 + BN > vis_wave);
        if (diag) {
            asm volatile("" ::: "memory");  // (keeps this a branch: as selects, every tile would pay for the diagonal ones)
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int blk = 0; blk < 2; blk++) {
                    const int lim = vis_lane - 1 - n0 - 32 * mb - 16 * blk - 8 * g;  // local columns e <= lim are visible
#pragma unroll
                    for (int e = 0; e < 8; e++) pv[16 * mb + 8 * blk + e] = e <= lim ? pv[16 * mb + 8 * blk + e] : 0.f;
                }
        }
        __builtin_amdgcn_sched_barrier(0);
        uint32_t dpk[8 * MB];
        auto ds_piece = [&](int kb, int e) {  // two elements of 16-key block kb: dS = P * (dP - D), rounded to 16 bits
            const int mb = kb >> 1, blk = kb & 1;
            const float d0 = pv[16 * mb + 8 * blk + 2 * e] * dp[mb][8 * blk + 2 * e];
            const float d1 = pv[16 * mb + 8 * blk + 2 * e + 1] * dp[mb][8 * blk + 2 * e + 1];
            dpk[4 * kb + e] = E::pack2(d0, d1);
        };
        {
            // K^T through transposing LDS reads of the row-major K tile, two reads per MFMA, FR2 MFMAs ahead (the first
            // ones in front of the first block's dS arithmetic)
            constexpr int NG = KB * DB, FR2 = 2;
            u32x2_t tl[NG], th[NG];
            f32x4_t nb[4];  // (S_EARLY: the next tile's bias column, 16 keys of this lane's half)
            auto tr_read = [&](int gi) {
                const int kb = gi / DB, db = gi % DB;
                tl[gi] = lds_ld_tr16(TL::tr_at(tr_cur, kb, db, 0));
                th[gi] = lds_ld_tr16(TL::tr_at(tr_cur, kb, db, 1));
            };
#pragma unroll
            for (int gi = 0; gi < FR2; gi++) tr_read(gi);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int e = 0; e < 4; e++) ds_piece(0, e);
#pragma unroll
            for (int gi = 0; gi < NG; gi++) {
                if (gi + FR2 < NG) tr_read(gi + FR2);
                const int kb = gi / DB, db = gi % DB;
                const u32x4_t bop = {dpk[4 * kb], dpk[4 * kb + 1], dpk[4 * kb + 2], dpk[4 * kb + 3]};
                const u32x4_t av = {tl[gi][0], tl[gi][1], th[gi][0], th[gi][1]};
                dq[db] = E::mfma(av, bop, dq[db]);
                if (kb + 1 < KB) {  // the next block's dS, spread over this block's slots
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (e * DB / 4 == db) ds_piece(kb + 1, e);
                }
                if constexpr (S_EARLY) {
                    // the next tile's bias column (slot (i + 1) % 3, complete since the last barrier): read in the slots
                    // of the first key block, used in those of the last
                    const uint32_t bs_n = lds0 + SM::OFF_BIAS + (uint32_t)(((i + 1) % 3) * 256 + 32 * g);
                    // (this wave's own copy of that column was fetched a tile ago, in front of the N_DMA loads of the
                    // tile after it: wait for it alone -- vmcnt N_DMA, no wait for LDS reads or exports)
                    if (kb == 0 && db == 0) __builtin_amdgcn_s_waitcnt(0x0F70 | N_DMA);
                    if (kb == 0 && db < 4) nb[db] = __builtin_bit_cast(f32x4_t, lds_ld128(bs_n + 16 * (db & 1) + 64 * (db >> 1)));
                    if (kb == KB - 1 && db < 4) {
#pragma unroll
                        for (int e = 0; e < 4; e++) s[0][4 * db + e] = nb[db][e] - lse2;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (jn < n_end) store_tile((i + 1) & 1, (i + 1) % 3);
        publish();
        i++;
        jc = jn;
        if constexpr (DMA) {
            jn = jnn;
            jnn = next_active(jn + 1);
        }
    }

    // (direct loads still in flight -- tiles fetched past the last one -- must not land in LDS that belongs to the next
    // workgroup by then)
    if constexpr (DMA) __builtin_amdgcn_s_waitcnt(0x0070);
    if (qrow < LqS) {
        uint16_t *dqp = (uint16_t *)p.dq + b * p.dq_b + (sq.q0 + qrow) * p.dq_r + h * p.dq_h;
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

template <typename T, int D, bool CAUSAL>
hipError_t launch_dq(const BwdParams &p, hipStream_t stream) {
    const FwdParams &f = p.f;
    constexpr int BN = D > 64 ? 32 : 64;  // at d = 128 a 64-key tile would spill registers
    auto kern = p.f.cmp.on ? bwd_dq_colmask_kernel<T, D, BN, CAUSAL, true> : bwd_dq_colmask_kernel<T, D, BN, CAUSAL, false>;
    const int smem = DqcSmem<D, BN>::TOTAL;
    static DynSmemLimit smem_limit[2];  // one per instantiation: the limit is a property of the kernel
    hipError_t e = smem_limit[p.f.cmp.on ? 1 : 0].ensure((const void *)kern, (int)smem);
    if (e != hipSuccess) return e;
    const int n_dq = xcd_grid(f.B * f.Hk, (f.Lq + Q_BM - 1) / Q_BM, f.H / f.Hk);  // a multiple of 8
    if (p.f.cmp.on) {
        const int units_max = f.B * f.Hk * ((f.Lk + KV_BN - 1) / KV_BN);
        const RedInterleave ri = red_interleave(n_dq / 8, units_max * (D / 16));
        BwdParams pr = p;
        pr.red_octets = ri.red_octets;
        pr.red_period = ri.period;
        pr.red_start = ri.start;
        hipLaunchKernelGGL(kern, dim3(n_dq + 8 * ri.red_octets), dim3(NTHREADS), smem, stream, pr);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(kern, dim3(n_dq), dim3(NTHREADS), smem, stream, p);
    return hipGetLastError();
}

}  // namespace

bool bwd_colmask_applicable(const BwdParams &p) {
    const bool mask_ok = !p.f.mask || p.f.m_r == 0;
    const bool bias_ok = !p.f.bias || p.f.bi_r == 0;
    return mask_ok && bias_ok && (p.f.Lk + 63) / 64 <= MAX_TILES;
}

hipError_t launch_bwd_dkdv_colmask(const BwdParams &p, int dtype, hipStream_t stream) {
    // head dims up to 64 / 128 / 256 (a head dim in between runs in the next larger instantiation)
    const int dc = p.f.d <= 64 ? 0 : (p.f.d <= 128 ? 1 : 2);
    const bool c = p.f.causal != 0;
    if (dtype == 0) {
        if (dc == 0) return c ? launch_dkdv<bf16_tag, 64, true>(p, stream) : launch_dkdv<bf16_tag, 64, false>(p, stream);
        if (dc == 1) return c ? launch_dkdv<bf16_tag, 128, true>(p, stream) : launch_dkdv<bf16_tag, 128, false>(p, stream);
        return c ? launch_dkdv<bf16_tag, 256, true>(p, stream) : launch_dkdv<bf16_tag, 256, false>(p, stream);
    }
    if (dc == 0) return c ? launch_dkdv<fp16_tag, 64, true>(p, stream) : launch_dkdv<fp16_tag, 64, false>(p, stream);
    if (dc == 1) return c ? launch_dkdv<fp16_tag, 128, true>(p, stream) : launch_dkdv<fp16_tag, 128, false>(p, stream);
    return c ? launch_dkdv<fp16_tag, 256, true>(p, stream) : launch_dkdv<fp16_tag, 256, false>(p, stream);
}

}  // namespace fdma

namespace fdma {
hipError_t launch_bwd_dq_colmask(const BwdParams &p, int dtype, hipStream_t stream) {
    const int dc = p.f.d <= 64 ? 0 : (p.f.d <= 128 ? 1 : 2);
    const bool c = p.f.causal != 0;
    if (dtype == 0) {
        if (dc == 0) return c ? launch_dq<bf16_tag, 64, true>(p, stream) : launch_dq<bf16_tag, 64, false>(p, stream);
        if (dc == 1) return c ? launch_dq<bf16_tag, 128, true>(p, stream) : launch_dq<bf16_tag, 128, false>(p, stream);
        return c ? launch_dq<bf16_tag, 256, true>(p, stream) : launch_dq<bf16_tag, 256, false>(p, stream);
    }
    if (dc == 0) return c ? launch_dq<fp16_tag, 64, true>(p, stream) : launch_dq<fp16_tag, 64, false>(p, stream);
    if (dc == 1) return c ? launch_dq<fp16_tag, 128, true>(p, stream) : launch_dq<fp16_tag, 128, false>(p, stream);
    return c ? launch_dq<fp16_tag, 256, true>(p, stream) : launch_dq<fp16_tag, 256, false>(p, stream);
}
}  // namespace fdma
