// Forward dynamic-mask attention for gfx950, general form: mask and / or bias vary per query row.
//
// Replaces compute_attn_1rowblock (csrc/flash_sparse_attn/src/flash_fwd_kernel.h:53-804) with its
// online softmax (src/softmax.h:127-221), masking (src/mask.h:94-161) and mask-tile OR skip
// (src/utils.h:339-352) of the reference.  Same math:
//     S = Q K^T * scale + bias ; S[~mask or non-causal] = -inf ; P = softmax(S) ; O = P V
// with the causal mask aligned bottom-right, O = 0 and LSE = +inf for rows with no visible key.
// (Mask and bias that are absent or broadcast over queries take the kernels of fdma_fwd_colmask.hip.)
//
// One workgroup = 4 waves = 128 query rows of one (batch, head); each wave owns 32 rows and computes the
// TRANSPOSED score tile S^T = K Q^T (K rows from LDS as the MFMA A operand, its pre-scaled Q rows in
// registers as the B operand), so a lane owns one query row and row max / row sum are in-lane reductions
// plus one cross-half swap.  P^T feeds O^T = V^T P^T straight from the accumulator registers; V^T comes out of the
// row-major V tile through transposing LDS reads.
//
// With a [Lq, Lk] bias (2 B) and mask (1 B) per score this path is bound by HBM, not by the matrix pipe, so the
// kernel is built around the mask / bias stream:
//   * every 128 x 64 mask and bias tile is fetched with coalesced 8- / 16-byte loads (a row's 64 keys are
//     contiguous), fused in registers into one 16-bit tile (bias where kept, -inf where dropped or beyond Lk) and
//     parked in LDS; the score accumulators then START from that tile, so bias and mask cost nothing later;
//   * everything is double-buffered and fetched a tile ahead, the mask two tiles ahead: the workgroup-wide OR
//     of the next tile's mask is known before that tile's bias / K / V loads are issued, and a tile without
//     any kept element costs its mask bytes only (no bias, K, V traffic, no MFMA work);
//   * one barrier per tile: the OR reduction is that barrier.
#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

namespace {

// Workgroups have 4 waves (128 query rows; two per CU at d <= 64) or, at d = 128 on grids that stay large enough,
// 8 waves (256 rows): at d = 128 only one workgroup fits on a CU, and with a single wave per SIMD nothing hides the
// in-order issue of that wave -- a second wave per SIMD does.
constexpr int BN_DEFAULT = 64;  // keys per tile (32 at head dims above 128: LDS)

template <int D, int BM, int BN> struct FwdSmem {
    static constexpr int SK = D + 8;     // K tile row stride (elements): conflict-free 16-byte row reads
    static constexpr int SV = LdsTile<D>::S;  // V tile row stride (row-major like K, read through transposing LDS reads)
    static constexpr int SF = BN + 8;    // fused mask+bias tile row stride
    static constexpr int K_BYTES = BN * SK * 2;
    static constexpr int VT_BYTES = BN * SV * 2;
    static constexpr int F_BYTES = BM * SF * 2;
    static constexpr int STAGE = K_BYTES + VT_BYTES + F_BYTES;
    static constexpr int TOTAL = 2 * STAGE;
};

template <typename T> struct NegInf2;
template <> struct NegInf2<bf16_tag> { static constexpr uint32_t value = 0xFF80FF80u; };
template <> struct NegInf2<fp16_tag> { static constexpr uint32_t value = 0xFC00FC00u; };

template <typename T, int D, bool CAUSAL, int NW, int BN>
__global__ void __launch_bounds__(64 * NW, (D <= 64 && NW == 4) ? 2 : 1) fwd_kernel(const FwdParams p) {
    constexpr int NTHREADS = 64 * NW, BM = 32 * NW;
    constexpr int FCH = BN / 8;             // 8-key chunks per mask / bias row of a tile
    constexpr int F_RPP = NTHREADS / FCH;   // mask / bias rows staged per pass (FCH threads cover the keys of a row)
    using E = Elem<T>;
    using SM = FwdSmem<D, BM, BN>;
    constexpr int KS = D / 16;  // contraction steps of Q K^T
    constexpr int DB = D / 32;  // 32-wide blocks of the head dimension
    constexpr int MB = BN / 32, KB = BN / 16;
    constexpr int CH = D / 8;               // 16-byte chunks per K row
    constexpr int K_RPP = NTHREADS / CH;    // K rows staged per pass
    constexpr int K_IT = BN / K_RPP;
    constexpr int F_IT = BM * (BN / 8) / NTHREADS;  // 8-key chunks of the mask / bias tile per thread (4)

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, g = lane >> 5;
    // linear workgroup id -> (query block, head, batch) with the query block OUTERMOST and descending: under causal
    // masking the blocks with the most KV tiles of every head start first, the light ones fill the tail
    const int hb_count = p.H * p.B;
    const int m_block = (int)gridDim.x / hb_count - 1 - (int)blockIdx.x / hb_count;
    const int h = ((int)blockIdx.x % hb_count) % p.H, b = ((int)blockIdx.x % hb_count) / p.H;
    const int hk = h / (p.H / p.Hk);
    const int m0 = m_block * BM;
    const int wrow0 = m0 + wave * 32;
    const int qrow = wrow0 + r;
    const int shift = p.Lk - p.Lq;  // bottom-right causal alignment

    // ---- Q fragments (B operand of S^T = K Q^T), scaled by softmax_scale * log2(e) once (the reference also rounds
    // the scaled Q to the input type, flash_fwd_kernel.h:428-439) and kept in registers for the whole KV loop
    u32x4_t qf[KS];
    {
        const int qc = qrow < p.Lq ? qrow : p.Lq - 1;
        const uint16_t *qp = (const uint16_t *)p.q + b * p.q_b + (int64_t)qc * p.q_r + h * p.q_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + g * 8;
            u32x4_t v = {0, 0, 0, 0};
            if (qrow < p.Lq && c < p.d) v = *(const u32x4_t *)(qp + c);
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = E::pack2(E::lo(v[e]) * p.scale_log2, E::hi(v[e]) * p.scale_log2);
            qf[ks] = v;
        }
    }

    int n_end = (p.Lk + BN - 1) / BN;
    if (CAUSAL) {
        int lim = m0 + BM + shift;  // first invisible column for the last row of the block
        if (lim > p.Lq + shift) lim = p.Lq + shift;
        if (lim < 0) lim = 0;
        const int ne = (lim + BN - 1) / BN;
        if (ne < n_end) n_end = ne;
    }

    f32x16_t o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    float row_max = -INFINITY;  // exp2 domain
    float row_sum = 0.f;        // per-lane partial (this lane's half of the keys)

    const int hm = p.mask ? (p.Hm == p.H ? h : (p.Hm == 1 ? 0 : h / (p.H / p.Hm))) : 0;
    const int hb = p.bias ? (p.Hb == p.H ? h : (p.Hb == 1 ? 0 : h / (p.H / p.Hb))) : 0;
    const uint8_t *mbase = p.mask ? p.mask + b * p.m_b + hm * p.m_h : nullptr;
    const uint16_t *bbase = p.bias ? (const uint16_t *)p.bias + b * p.bi_b + hb * p.bi_h : nullptr;
    const uint16_t *kbase = (const uint16_t *)p.k + b * p.k_b + hk * p.k_h;
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.v_b + hk * p.v_h;

    // ---- staging maps
    const int kc = tid % CH, kr0 = tid / CH;             // K: d chunk, first row
    const bool k_dvalid = kc * 8 < p.d;
    const int fc = tid % FCH, fr0 = tid / FCH;           // mask / bias: 8-key chunk, first row (rows fr0 + F_RPP it)
    u32x4_t kreg[K_IT], vreg[K_IT], breg[F_IT];
    u32x2_t mreg[F_IT], mnext[F_IT];

    // All tile loads are unconditional, from clamped (always valid) addresses, so that they can be issued early and
    // stay in flight; what a clamped load fetched in place of a missing element is neutralised later: the mask
    // words are ANDed with a validity pattern when they are consumed, rows of K / V beyond Lk and head-dim chunks
    // beyond d are finite duplicates that meet a -inf score or a zero Q fragment.
    const int kcol = k_dvalid ? kc * 8 : 0;
    // (a mask that comes packed to bits: one byte per 8-key chunk instead of eight, expanded where it is looked at)
    const uint8_t *mbits = (mbase && p.mbits) ? p.mbits + b * p.mb_b + hm * p.mb_h : nullptr;
    auto load_mask = [&](int j, u32x2_t (&dst)[F_IT]) {
        if (!mbase) return;
        int kk = j * BN + 8 * fc;
        kk = kk < p.Lk ? kk : 0;
#pragma unroll
        for (int it = 0; it < F_IT; it++) {
            int row = m0 + fr0 + F_RPP * it;
            row = row < p.Lq ? row : p.Lq - 1;
            // (one 8-byte load either way, from an address chosen without a branch: mask bytes of the chunk, or the
            // aligned piece of the bit row that holds the chunk's byte)
            const uint8_t *src = mbits ? mbits + (int64_t)row * p.mb_r + ((kk >> 3) & ~7) : mbase + (int64_t)row * p.m_r + kk;
            dst[it] = *(const u32x2_t *)src;
        }
    };
    // validity of the chunks (rows < Lq, keys < Lk, not entirely above the causal diagonal) applied to the loaded
    // mask words; returns "any element kept"
    auto finish_mask = [&](int j, u32x2_t (&dst)[F_IT]) -> bool {
        const int kk = j * BN + 8 * fc;
        uint32_t any = 0;
#pragma unroll
        for (int it = 0; it < F_IT; it++) {
            const int row = m0 + fr0 + F_RPP * it;
            u32x2_t mv = mbase ? (mbits ? mask_bits_to_bytes(mask_bits_byte(dst[it], kk)) : dst[it]) : u32x2_t{0x01010101u, 0x01010101u};
            const bool ok = row < p.Lq && kk < p.Lk && !(CAUSAL && kk > row + shift);
            uint64_t keepm = ok ? ~0ull : 0ull;
            if (kk + 8 > p.Lk && kk < p.Lk) keepm = (1ull << (8 * (p.Lk - kk))) - 1ull;  // chunk straddles the end of the keys
            mv[0] &= (uint32_t)keepm;
            mv[1] &= (uint32_t)(keepm >> 32);
            dst[it] = mv;
            any |= mv[0] | mv[1];
        }
        return any != 0;
    };
    // bias of tile j into registers
    auto load_bias = [&](int j, u32x4_t (&dst)[F_IT]) {
        const int n0 = j * BN;
        if (bbase) {
            int kk = n0 + 8 * fc;
            kk = kk < p.Lk ? kk : 0;
#pragma unroll
            for (int it = 0; it < F_IT; it++) {
                int row = m0 + fr0 + F_RPP * it;
                row = row < p.Lq ? row : p.Lq - 1;
                dst[it] = *(const u32x4_t *)(bbase + (int64_t)row * p.bi_r + kk);
            }
        } else {
#pragma unroll
            for (int it = 0; it < F_IT; it++) dst[it] = u32x4_t{0, 0, 0, 0};
        }
    };
    // K and V of tile j into registers
    auto load_kv = [&](int j) {
        const int n0 = j * BN;
#pragma unroll
        for (int it = 0; it < K_IT; it++) {
            int key = n0 + kr0 + it * K_RPP;
            key = key < p.Lk ? key : p.Lk - 1;
            kreg[it] = *(const u32x4_t *)(kbase + (int64_t)key * p.k_r + kcol);
            // (V rows the same way: a wave's load covers whole rows -- one cache line per row at head dim 64 -- where a
            // (key quad, d chunk) item per thread, as a transposition in registers wants it, touched every line twice)
            vreg[it] = *(const u32x4_t *)(vbase + (int64_t)key * p.v_r + kcol);
        }
    };
    auto load_rest = [&](int j) {
        load_bias(j, breg);
        load_kv(j);
    };
    // registers -> LDS stage `buf`: K and V rows, mask and bias fused (bias where kept, -inf elsewhere)
    auto store_stage = [&](int buf, const u32x2_t (&mv)[F_IT], const u32x4_t (&bsrc)[F_IT]) {
        char *sK = smem + buf * SM::STAGE;
        char *sVt = sK + SM::K_BYTES;
        char *sF = sVt + SM::VT_BYTES;
#pragma unroll
        for (int it = 0; it < K_IT; it++) {
            *(u32x4_t *)(sK + ((kr0 + it * K_RPP) * SM::SK + kc * 8) * 2) = kreg[it];
            *(u32x4_t *)(sVt + LdsTile<D>::chunk(kr0 + it * K_RPP, kc)) = vreg[it];
        }
#pragma unroll
        for (int it = 0; it < F_IT; it++) {
            u32x4_t bv = bsrc[it];
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
    // (this lane's part of the address of a transposing read of the V tile)
    const uint32_t tr_lane = LdsTile<D>::tr_base(g, (lane & 15) >> 2, (lane >> 4) & 1, (lane & 3) == 1 ? 2 : ((lane & 3) == 2 ? 1 : (lane & 3)));

    // ---- one tile from LDS stage `buf`
    auto compute = [&](int j, int buf) {
        const int n0 = j * BN;
        const char *sK = smem + buf * SM::STAGE;
        const char *sVt = sK + SM::K_BYTES;
        const char *sF = sVt + SM::VT_BYTES + ((wave * 32 + r) * SM::SF + 8 * g) * 2;
        // scores start from the fused mask+bias tile (exp2 domain)
        f32x16_t s[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                const u32x4_t fv = *(const u32x4_t *)(sF + (32 * mb + 16 * blk) * 2);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    s[mb][8 * blk + 2 * e] = E::lo(fv[e]) * kLog2e;
                    s[mb][8 * blk + 2 * e + 1] = E::hi(fv[e]) * kLog2e;
                }
            }
        {
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
                s[f % MB] = E::mfma(a[f], qf[f / MB], s[f % MB]);
            }
        }
        // causal selects on diagonal tiles only (wave-uniform branch)
        if (CAUSAL && n0 + BN - 1 > wrow0 + shift) {
            asm volatile("" ::: "memory");
            const int lim = qrow + shift - n0 - 8 * g;  // local column limit for this lane
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int lc = 32 * mb + 16 * (i >> 3) + (i & 7);
                    s[mb][i] = lc <= lim ? s[mb][i] : -INFINITY;
                }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[mb][i]);
        tmax = xhalf_max(tmax);
        // lazy rescale: the running maximum is only the reference point of the exp2, so it moves (and O and the row
        // sums are rescaled) only when a score exceeds it by more than 2^8 -- rare after the first tiles
        if (__any(tmax > row_max + 8.f)) {
            const float new_max = fmaxf(row_max, tmax);
            const float safe = new_max == -INFINITY ? 0.f : new_max;
            const float alpha = fast_exp2(row_max - safe);
            row_max = new_max;
            row_sum *= alpha;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[db][i] *= alpha;
        }
        const float m_use = row_max == -INFINITY ? 0.f : row_max;
        float psum = 0.f;
        uint32_t pk[8 * MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                const float p0 = fast_exp2(s[mb][i] - m_use);
                const float p1 = fast_exp2(s[mb][i + 1] - m_use);
                psum += p0 + p1;
                pk[8 * mb + i / 2] = E::pack2(p0, p1);
            }
        row_sum += psum;
        {
            // V^T (rows of the A operand = head dim) through transposing reads of the row-major V tile
            constexpr int NF = KB * DB, FR = NF < 8 ? NF : 8;
            u32x4_t a[NF];
            const uint32_t tr_v = lds_addr(sVt) + tr_lane;
            auto frag = [&](int f) {
                const int kb = f / DB, db = f % DB;
                const u32x2_t lo = lds_ld_tr16(LdsTile<D>::tr_at(tr_v, kb, db, 0)), hi = lds_ld_tr16(LdsTile<D>::tr_at(tr_v, kb, db, 1));
                return u32x4_t{lo[0], lo[1], hi[0], hi[1]};
            };
#pragma unroll
            for (int f = 0; f < FR; f++) a[f] = frag(f);
#pragma unroll
            for (int f = 0; f < NF; f++) {
                if (f + FR < NF) a[f + FR] = frag(f + FR);
                const int kb = f / DB, db = f % DB;
                const u32x4_t bop = {pk[4 * kb], pk[4 * kb + 1], pk[4 * kb + 2], pk[4 * kb + 3]};
                o[db] = E::mfma(a[f], bop, o[db]);
            }
        }
    };

    // ---- main loop.  At the top of iteration j: tile j sits in LDS stage j&1 if it is active, `mreg` holds
    // the mask of tile j+1 and `act_next` says whether that tile has any kept element.
    // DEEP (head dims up to 64, where the registers are there): mask and bias -- the bytes that come from HBM -- stay in
    // flight for TWO iterations instead of one.  With one, every iteration contained a whole trip to memory (the mask
    // requested at its top decided, at its end, whether the tile after the next is fetched at all), and the launch moved
    // what it had in flight once per trip: 64 KB per CU every 3.5 us.  Now the mask of tile j+4 and the bias of tile
    // j+2 are requested at the top of iteration j, behind K / V of tile j+1 (cache hits; waiting for those must not
    // mean waiting for the younger requests: loads come back in the order they were issued).
    constexpr bool DEEP = D <= 64;
    if (n_end > 0 && DEEP) {
        u32x2_t m1[F_IT], m2[F_IT], m3[F_IT];            // with mreg: the masks of tiles j .. j+3 at the top of iteration j
        u32x4_t b1[F_IT], b2[F_IT];                      // bias of tiles j+1 (requested an iteration ago), j+2
        load_mask(0, mreg);
        load_mask(1, m1);
        load_mask(2, m2);
        load_mask(3, m3);
        bool act_cur = __syncthreads_or(finish_mask(0, mreg));
        if (act_cur) {
            load_rest(0);
            store_stage(0, mreg, breg);
        }
        bool act_1 = __syncthreads_or(n_end > 1 && finish_mask(1, m1));
        if (act_1) load_bias(1, b1);
        bool act_2 = __syncthreads_or(n_end > 2 && finish_mask(2, m2));
        // one iteration; the register sets change roles from one iteration to the next (written out four iterations
        // at a time: a move between sets would have to wait for a load that is still in flight)
        auto step = [&](int j, u32x2_t (&ma)[F_IT], u32x2_t (&mc)[F_IT], u32x2_t (&md)[F_IT], u32x4_t (&ba)[F_IT], u32x4_t (&bb)[F_IT]) {
            // ma: mask of tile j+1 (finished); mc: of tile j+3 (in flight since the iteration before); md: receives tile j+4
            // ba: bias of tile j+1 (requested an iteration ago); bb: receives tile j+2
            const bool have_next = j + 1 < n_end && act_1;
            if (have_next) load_kv(j + 1);
            __builtin_amdgcn_sched_barrier(0);
            if (j + 4 < n_end) load_mask(j + 4, md);
            __builtin_amdgcn_sched_barrier(0);
            if (j + 2 < n_end && act_2) load_bias(j + 2, bb);
            __builtin_amdgcn_sched_barrier(0);
            if (act_cur) compute(j, j & 1);
            __builtin_amdgcn_sched_barrier(0);
            if (have_next) store_stage((j + 1) & 1, ma, ba);
            const bool act_3 = __syncthreads_or(j + 3 < n_end && finish_mask(j + 3, mc));
            act_cur = have_next;
            act_1 = act_2;
            act_2 = act_3;
        };
#pragma unroll 1
        for (int j = 0; j < n_end; j += 4) {
            step(j, m1, m3, mreg, b1, b2);  // (mreg, the set of tile j, is free: it receives tile j+4)
            if (j + 1 < n_end) step(j + 1, m2, mreg, m1, b2, b1);
            if (j + 2 < n_end) step(j + 2, m3, m1, m2, b1, b2);
            if (j + 3 < n_end) step(j + 3, mreg, m2, m3, b2, b1);
        }
    } else if (n_end > 0) {
        load_mask(0, mreg);
        if (n_end > 1) load_mask(1, mnext);
        bool act_cur = __syncthreads_or(finish_mask(0, mreg));
        if (act_cur) {
            load_rest(0);
            store_stage(0, mreg, breg);
        }
        bool act_next = __syncthreads_or(n_end > 1 && finish_mask(1, mnext));
        // one iteration; `m_next` holds the (finished) mask of tile j+1, `m_new` receives the mask of tile j+2.
        // The scheduling barriers keep the loads at the top and their first use below the compute: their
        // latency is then covered by the MFMA work instead of being waited for right away.
        auto step = [&](int j, u32x2_t (&m_next)[F_IT], u32x2_t (&m_new)[F_IT]) {
            const bool have_next = j + 1 < n_end && act_next;
            if (have_next) load_rest(j + 1);
            if (j + 2 < n_end) load_mask(j + 2, m_new);
            __builtin_amdgcn_sched_barrier(0);
            if (act_cur) compute(j, j & 1);
            __builtin_amdgcn_sched_barrier(0);
            if (have_next) store_stage((j + 1) & 1, m_next, breg);
            const bool act_nn = __syncthreads_or(j + 2 < n_end && finish_mask(j + 2, m_new));
            act_cur = have_next;
            act_next = act_nn;
        };
        for (int j = 0; j < n_end; j += 2) {
            step(j, mnext, mreg);
            if (j + 1 < n_end) step(j + 1, mreg, mnext);
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
                const int c = 32 * db + 16 * blk + 8 * g;
                if (c < p.d) {
                    u32x4_t w;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        w[e] = E::pack2(o[db][8 * blk + 2 * e] * inv, o[db][8 * blk + 2 * e + 1] * inv);
                    *(u32x4_t *)(op + c) = w;
                }
            }
        if (g == 0) {
            const float lse = total > 0.f ? (row_max + __builtin_amdgcn_logf(total)) * kLn2 : INFINITY;
            p.lse[((int64_t)b * p.H + h) * p.Lq + qrow] = lse;
        }
    }
}

template <typename T, int D, bool CAUSAL, int NW>
hipError_t launch_fwd_c(const FwdParams &p, hipStream_t stream) {
    constexpr int BM = 32 * NW, NTHREADS = 64 * NW, BN = D > 128 ? 32 : BN_DEFAULT;
    auto kern = fwd_kernel<T, D, CAUSAL, NW, BN>;
    const int smem = FwdSmem<D, BM, BN>::TOTAL;
    static DynSmemLimit smem_limit;
    hipError_t e = smem_limit.ensure((const void *)kern, (int)smem);
    if (e != hipSuccess) return e;
    dim3 grid(((p.Lq + BM - 1) / BM) * p.H * p.B);
    hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), smem, stream, p);
    return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_fwd_t(const FwdParams &p, hipStream_t stream) {
    if constexpr (D > 64 && D <= 128) {
        // 256-row workgroups while the grid still covers the chip about twice
        if ((int64_t)p.B * p.H * ((p.Lq + 255) / 256) >= 512)
            return p.causal ? launch_fwd_c<T, D, true, 8>(p, stream) : launch_fwd_c<T, D, false, 8>(p, stream);
    }
    return p.causal ? launch_fwd_c<T, D, true, 4>(p, stream) : launch_fwd_c<T, D, false, 4>(p, stream);
}

}  // namespace

hipError_t launch_fwd(const FwdParams &p, int dtype, hipStream_t stream) {
    if (p.Lq <= 0 || p.B <= 0) return hipSuccess;
    if (fwd_colmask_applicable(p)) return launch_fwd_colmask(p, dtype, stream);
    // head dims up to 64 / 128 / 256 (a head dim in between runs in the next larger instantiation)
    if (dtype == 0) return p.d <= 64 ? launch_fwd_t<bf16_tag, 64>(p, stream) : p.d <= 128 ? launch_fwd_t<bf16_tag, 128>(p, stream) : launch_fwd_t<bf16_tag, 256>(p, stream);
    return p.d <= 64 ? launch_fwd_t<fp16_tag, 64>(p, stream) : p.d <= 128 ? launch_fwd_t<fp16_tag, 128>(p, stream) : launch_fwd_t<fp16_tag, 256>(p, stream);
}

}  // namespace fdma
