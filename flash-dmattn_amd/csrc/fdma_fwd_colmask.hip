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
// double-buffered in LDS.  Tile i is computed from buffers i&1; the registers hold tile i+1, whose LDS stores go
// to the other buffers between the scores and the softmax of tile i (the LDS port is idle there), and the global
// loads of tile i+2 are then issued between the PV MFMAs, each a single instruction (scalar tile base + a
// loop-invariant per-thread offset).  One barrier per tile.  Workgroups have 256 rows (8 waves: four stage V,
// four stage K and the bias) when the grid stays large enough, else 128 rows (4 waves doing both).
// Q is scaled by softmax_scale*log2(e) once and the score accumulators start from the fused bias vector,
// so the MFMA result is the exp2-domain score with bias and mask applied and the softmax spends five
// vector instructions per element (max, sub, exp2, add, half a convert); the running maximum moves only when a
// score exceeds it by 2^8, so the rescale of O is rare.  LDS fragment reads run a batch ahead of the MFMAs that
// consume them.  Workgroup ids are remapped so that the workgroups sharing one XCD's L2 also share K / V.
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
    constexpr int STHREADS = 256;             // threads staging one operand
    constexpr bool SPLIT = NW == 8;           // 8 waves: the first four stage V, the last four K and the bias
    static_assert(NW == 4 || NW == 8, "staging maps are written for 256 or 512 threads");
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
    constexpr int NL = SPLIT ? 4 : K_IT + 4;  // 16-byte loads per thread and tile
    constexpr int VB = SPLIT ? 0 : K_IT;      // first V staging register
    static_assert(!SPLIT || K_IT == 4, "the role split assumes four loads per thread for either operand");

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
    const int n_mb = (p.Lq + BM - 1) / BM;  // p.Lq, p.Lk: the longest sequence of a ragged batch
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
    const SeqInfo sq = seq_info(p, b);  // this batch entry's lengths and first rows (ragged batch: from cu_seqlens)
    const int LqS = sq.Lq, LkS = sq.Lk;
    if (m0 >= LqS) return;
    const int shift = LkS - LqS;
    const int wrow0 = m0 + wave * 32 * NQ;  // first query row of this wave

    const int hm = p.mask ? (p.Hm == p.H ? h : (p.Hm == 1 ? 0 : h / (p.H / p.Hm))) : 0;
    const int hb = p.bias ? (p.Hb == p.H ? h : (p.Hb == 1 ? 0 : h / (p.H / p.Hb))) : 0;
    const uint8_t *mrow = p.mask ? p.mask + b * p.m_b + hm * p.m_h : nullptr;
    const uint16_t *brow = p.bias ? (const uint16_t *)p.bias + b * p.bi_b + hb * p.bi_h : nullptr;
    const uint16_t *kbase = (const uint16_t *)p.k + b * p.k_b + sq.k0 * p.k_r + hk * p.k_h;
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.v_b + sq.k0 * p.v_r + hk * p.v_h;

    // key columns this workgroup iterates over, and the number of them a query row may see
    const int Lk = CMP ? p.cmp.count[b * p.Hk + hk] : LkS;
    const int32_t *ccnt = CMP ? p.cmp.cnt + (int64_t)(b * p.Hk + hk) * p.cmp.ld : nullptr;
    const float *fbrow = CMP ? p.cmp.fb + (int64_t)(b * p.cmp.Hfb + (p.cmp.Hfb == p.H ? h : hk)) * p.cmp.ld : nullptr;
    auto visible = [&](int row) -> int {  // columns [0, visible(row)) pass the causal test for `row`
        if (row >= LqS) row = LqS - 1;
        int c = row + shift;
        if (!CMP) return c + 1;
        if (c < 0) return 0;
        return ccnt[c < LkS ? c : LkS - 1];
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
                    if (col < LkS) {
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
    if (!CMP) __syncthreads();  // (compacted keys have no bitmap: every tile up to n_end is active)

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
        const int qc = qrow < LqS ? qrow : LqS - 1;
        const uint16_t *qp = (const uint16_t *)p.q + b * p.q_b + (sq.q0 + qc) * p.q_r + h * p.q_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + g * 8;
            u32x4_t v = {0, 0, 0, 0};
            if (qrow < LqS && c < p.d) v = *(const u32x4_t *)(qp + c);
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

    // ---- staging (global -> registers -> LDS).  A tile is BN * CH 16-byte chunks of K plus V_ITEMS (key quad, d chunk)
    // items of V with four loads each (V is transposed in registers on its way to LDS).  Every load is unconditional,
    // from an always valid address: rows beyond the end of the keys are clamped to the last row (their fused bias is
    // -inf, so the duplicate never counts) and head-dim chunks beyond d to chunk 0 (they meet zero Q fragments /
    // columns of O that are not stored).  The per-thread byte offsets are loop invariants -- one set for full tiles,
    // one for the (only) partial tile at the end of the keys -- so a load is one instruction with a scalar tile base,
    // and the loads of a tile can be issued one by one between the MFMAs of the tile being computed.
    const bool role_v = !SPLIT || wave < 4, role_k = !SPLIT || wave >= 4;  // wave-uniform
    const int kt = tid & (STHREADS - 1);
    const int kc = kt % CH, kr0 = kt / CH;
    const int vkg = kt % KQ, vc = (kt / KQ) % CH;  // V: key quad and d chunk of this thread
    const uint32_t k_r2 = (uint32_t)(p.k_r * 2), v_r2 = (uint32_t)(p.v_r * 2);  // bytes per row
    const uint32_t kcolb = (kc * 8 < p.d ? kc * 16 : 0), vcolb = (vc * 8 < p.d ? vc * 16 : 0);
    const int j_last = Lk > 0 ? (Lk - 1) / BN : 0, last_row = Lk > 0 ? (Lk - 1) % BN : 0;
    uint32_t soff[NL], soff_l[NL];  // byte offsets of this thread's loads inside a full / the last tile
#pragma unroll
    for (int n = 0; n < NL; n++) {
        const bool is_v = SPLIT ? role_v : n >= K_IT;
        const int item = SPLIT ? n : (n >= K_IT ? n - K_IT : n);
        const int row = is_v ? 4 * vkg + item : kr0 + item * K_RPP;
        const uint32_t r2 = is_v ? v_r2 : k_r2, colb = is_v ? vcolb : kcolb;
        soff[n] = (uint32_t)row * r2 + colb;
        soff_l[n] = (uint32_t)(row < last_row ? row : last_row) * r2 + colb;
    }
    u32x4_t sreg[NL];             // staging registers
    uint32_t braw = 0, mraw = 0;  // raw bias / mask of this thread's column of the tile in flight
    // an absent mask / bias is read from K instead (any valid address) and ignored when the value is used
    const uint8_t *mrow_ld = mrow ? mrow : (const uint8_t *)kbase;
    const uint16_t *brow_ld = brow ? brow : kbase;
    bool bcol_ok = false;
    int bias_col = 0;
    typedef const __attribute__((address_space(1))) char *gptr_t;  // global address space survives the integer round trip
    gptr_t tb_k = nullptr, tb_v = nullptr;        // tile bases (wave-uniform, in scalar registers)
    bool t_last = false;                          // the tile in flight is the partial one

    auto uniform_ptr = [](const char *ptr) -> gptr_t {
        const uint64_t v = (uint64_t)ptr;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (gptr_t)(((uint64_t)hi << 32) | lo);
    };
    auto set_tile = [&](int j) {
        const int n0 = j * BN;
        const char *tk = (const char *)kbase + (int64_t)n0 * p.k_r * 2;
        const char *tv = (const char *)vbase + (int64_t)n0 * p.v_r * 2;
        if (SPLIT) {
            tb_k = tb_v = uniform_ptr(role_v ? tv : tk);
        } else {
            tb_k = uniform_ptr(tk);
            tb_v = uniform_ptr(tv);
        }
        t_last = j == j_last;
        bias_col = n0 + kt;
    };
    auto issue_load = [&](int n) {
        const gptr_t base = (SPLIT || n < K_IT) ? tb_k : tb_v;
        sreg[n] = *(const __attribute__((address_space(1))) u32x4_t *)(base + (t_last ? soff_l[n] : soff[n]));
    };
    // fused bias of the tile's columns: only the raw loads here -- the values are looked at when they are stored
    auto load_bias_raw = [&]() {
        if (role_k && kt < BN) {
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
    auto load_tile = [&](int j) {
        set_tile(j);
        load_bias_raw();
#pragma unroll
        for (int n = 0; n < NL; n++) issue_load(n);
    };
    auto store_stage = [&](int buf, int slot) {
        if (role_k) {
            char *sK = smem + SM::OFF_K + buf * SM::K_BYTES;
#pragma unroll
            for (int it = 0; it < K_IT; it++)
                *(u32x4_t *)(sK + ((kr0 + it * K_RPP) * SM::SK + kc * 8) * 2) = sreg[it];
            if (kt < BN) {
                float v = -INFINITY;
                if (CMP) {
                    if (bcol_ok) v = __uint_as_float(braw);
                } else if (bcol_ok && (!mrow || mraw)) {
                    v = brow ? E::lo(braw) * kLog2e : 0.f;
                }
                sBias[slot * BN + kt] = v;
            }
        }
        if (role_v && kt < V_ITEMS) {  // transpose 4 keys x 8 d in registers, write V^T[d][key quad]
            char *sVt = smem + SM::OFF_VT + buf * SM::VT_BYTES;
#pragma unroll
            for (int dd = 0; dd < 8; dd++) {
                const int w = dd >> 1;
                const uint32_t sel = (dd & 1) ? 0x07060302u : 0x05040100u;
                u32x2_t out;
                out[0] = __builtin_amdgcn_perm(sreg[VB + 1][w], sreg[VB + 0][w], sel);
                out[1] = __builtin_amdgcn_perm(sreg[VB + 3][w], sreg[VB + 2][w], sel);
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
            // Lazy rescale: the running maximum is only a reference point of the exp2 (any value gives the same
            // softmax), so it is moved -- and O and the row sums rescaled -- only when a score exceeds it by more
            // than 2^8; below that the probabilities stay far inside the range of the 16-bit operand and of the fp32
            // sums, and almost every tile skips the rescale.
            if (__any(tmax > row_max[nb] + 8.f)) {
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
            // pin the sum here: left alone, the compiler sinks the whole chain of additions below the PV MFMAs (its
            // result is not needed before the next tile), where nothing hides it, and keeps all 32 probabilities
            // alive in fp32 until then
            asm volatile("" : "+v"(row_sum[nb]));
        }
    };
    // O^T += V^T P^T for one tile; the global loads of the tile two ahead are issued between the MFMAs (a burst of
    // loads from every wave right after a barrier would queue up at the CU's address unit with the matrix pipe idle)
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
#pragma unroll
                for (int n = f * NL / NF; n < (f + 1) * NL / NF; n++) issue_load(n);  // spread evenly over the MFMAs
            }
        }
    };

    // ---- main loop.  Tile i is computed from LDS buffers i&1.  The registers hold tile i+1 (loaded during the PV
    // MFMAs of the previous iteration); its LDS stores go to the other buffers -- last read before the previous
    // barrier -- between the scores and the softmax, when the LDS port is idle; the loads of tile i+2 then reuse the
    // registers during the PV MFMAs.  One barrier per tile.
    const int j0 = next_active(0);
    if (j0 < n_end) {
        const int j1 = next_active(j0 + 1);
        load_tile(j0);
        store_stage(0, 0);
        load_tile(j1 < n_end ? j1 : j0);
        __syncthreads();

        f32x16_t sa[NQ][MB];
        int i = 0, jc = j0, jn1 = j1;
        while (jc < n_end) {
            const int jn2 = jn1 < n_end ? next_active(jn1 + 1) : n_end;
            qk(sa, i & 1, i & 1);
            __builtin_amdgcn_sched_barrier(0);
            if (jn1 < n_end) store_stage((i + 1) & 1, (i + 1) & 1);
            uint32_t pk[NQ][8 * MB];
            softmax(sa, jc, pk);
            __builtin_amdgcn_sched_barrier(0);
            set_tile(jn2 < n_end ? jn2 : jc);  // (after the last tile an existing one is fetched again and dropped)
            pv(pk, i & 1);
            load_bias_raw();
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            i++; jc = jn1; jn1 = jn2;
        }
    }

    // ---- epilogue
#pragma unroll
    for (int nb = 0; nb < NQ; nb++) {
        const int qrow = wrow0 + nb * 32 + r;
        const float total = xhalf_sum(row_sum[nb]);
        const float inv = total > 0.f ? 1.f / total : 0.f;
        if (qrow < LqS) {
            uint16_t *op = (uint16_t *)p.o + b * p.o_b + (sq.q0 + qrow) * p.o_r + h * p.o_h;
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
                p.lse[b * p.lse_b + h * p.lse_h + sq.q0 + qrow] = lse;
            }
        }
    }
}

template <typename T, int D, int NQ, int BN, bool CAUSAL, bool CMP, int NW = 4>
hipError_t launch_one(const FwdParams &p, hipStream_t stream) {
    constexpr int BM = 32 * NQ * NW;
    auto kern = fwd_colmask_kernel<T, D, NQ, BN, CAUSAL, NW, CMP>;
    const int smem = CmSmem<D, BN>::TOTAL;
    static DynSmemLimit smem_limit;
    hipError_t e = smem_limit.ensure((const void *)kern, (int)smem);
    if (e != hipSuccess) return e;
    const int n_mb = (p.Lq + BM - 1) / BM, G = p.H / p.Hk, pairs = p.B * p.Hk;
    const int gcd8 = (pairs % 8 == 0) ? 8 : ((pairs % 4 == 0) ? 4 : ((pairs % 2 == 0) ? 2 : 1));
    const int k_split = 8 / gcd8;
    dim3 grid(pairs * k_split * ((n_mb + k_split - 1) / k_split) * G);
    hipLaunchKernelGGL(kern, grid, dim3(64 * NW), smem, stream, p);
    return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_d(const FwdParams &p, hipStream_t stream) {
    // 256-row workgroups (8 waves, one workgroup per CU) stage every K / V tile once for twice the rows and win
    // whenever the grid still has a few workgroups per CU; smaller problems keep 128-row workgroups, two per CU
    const int64_t groups256 = (int64_t)p.B * p.H * ((p.Lq + 255) / 256);
    if constexpr (D == 128) if (groups256 >= 512) {
        if (p.cmp.on) return p.causal ? launch_one<T, D, 1, 64, true, true, 8>(p, stream) : launch_one<T, D, 1, 64, false, true, 8>(p, stream);
        return p.causal ? launch_one<T, D, 1, 64, true, false, 8>(p, stream) : launch_one<T, D, 1, 64, false, false, 8>(p, stream);
    }
    if (p.cmp.on) return p.causal ? launch_one<T, D, 1, 64, true, true>(p, stream) : launch_one<T, D, 1, 64, false, true>(p, stream);
    return p.causal ? launch_one<T, D, 1, 64, true, false>(p, stream) : launch_one<T, D, 1, 64, false, false>(p, stream);
}

}  // namespace

bool fwd_colmask_applicable(const FwdParams &p) {
    const bool mask_ok = !p.mask || p.m_r == 0;
    const bool bias_ok = !p.bias || p.bi_r == 0;
    return mask_ok && bias_ok && (p.Lk + 31) / 32 <= MAX_TILES;
}

hipError_t launch_fwd_colmask(const FwdParams &p, int dtype, hipStream_t stream) {
    const bool d64 = p.d <= 64;
    if (dtype == 0) return d64 ? launch_d<bf16_tag, 64>(p, stream) : launch_d<bf16_tag, 128>(p, stream);
    return d64 ? launch_d<fp16_tag, 64>(p, stream) : launch_d<fp16_tag, 128>(p, stream);
}

}  // namespace fdma
