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
//   * bias and mask fuse into one 16-element side row per key (pieces of bias*log2e, 0 / -inf for the mask and
//     for keys beyond Lk) staged in LDS, which the score MFMAs contract as one more k-step;
//   * causal masking costs instructions on diagonal tiles only.
//
// The matrix pipe is what the kernel is priced against, so the vector ALU gets as little as possible and what is
// left runs UNDER the MFMAs.
//   Softmax on the matrix pipe.  Q is scaled by softmax_scale*log2(e) once, and every key carries a 16-element
// side row in LDS that is contracted as one more 16-wide k-step of the score MFMAs against constants held per
// query row: three 16-bit pieces of bias*log2(e) (together the exact fp32 value) times 1, the mask (0 / -inf) times
// 1, and two ones that meet the two 16-bit pieces of MINUS the row's softmax reference point.  The accumulators
// start from the constant 0, and what leaves the MFMAs is the finished exp2 argument.  The reference point of a
// row is any number near its running maximum (the softmax does not depend on it); it is set by the first tile and
// then left alone as long as no probability exceeds 2^14 -- which the sum of the probabilities shows, so the
// common path has no maximum at all: exp2, convert to 16 bits (two per instruction), one addition to the row sum
// (plain fp32 additions: a 16-bit dot product with (1, 1) would halve their number, but it runs on the matrix pipe's
// side of the SIMD and cost 2-3 % of the kernel): 2.5 vector instructions per score.  A half tile that fails the check (or a wave whose rows have no
// reference yet) takes the classic path: maximum, new reference, rescale of O and of the sums.
//   Software pipeline over HALF tiles (32 keys).  One step issues the score MFMAs of half tile h+1, the P V MFMAs
// of half tile h-1 and, between them, the softmax instructions of half tile h: the three have no dependence on one
// another, so the vector instructions issue while the matrix pipe works, and the two waves of a SIMD no longer
// have to be in different phases for anything to overlap (phase by phase -- scores, softmax, P V -- the same loop
// ran at 49 % of the MFMA rate, the pipelined one is bound by LDS fragment reads and exp2 at 75-80 %).  A half tile
// in flight costs 16 score and 8 probability registers, two of them 48 -- what one whole tile cost before.
//   Staging.  K, V^T (V is transposed in registers while being staged) and the side rows are double-buffered in LDS;
// K runs one tile ahead of V (the P V product of a tile is issued a tile after its scores).  With 8 waves (256 query
// rows per workgroup) four waves stage V and four K and the side rows; one barrier per tile.  Global loads are one
// instruction each (scalar tile base + a loop-invariant per-thread offset) and sit a whole tile in front of their
// LDS stores.  Workgroup ids are remapped so that the workgroups sharing one XCD's L2 also share K / V.
#include <type_traits>

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
    static constexpr int X_BYTES = BN * 32;  // side rows: 16 elements of 16 bits per key
    static constexpr int OFF_X = OFF_VT + 2 * VT_BYTES;
    static constexpr int OFF_BITS = OFF_X + 2 * X_BYTES;
    static constexpr int OFF_FLAG = OFF_BITS + MAX_TILES / 8;  // one word: a wave left the range of the common path
    static constexpr int TOTAL = OFF_FLAG + 16;
};

// CMP: K / V are the compacted copies of the kept columns (see fdma_compact.hip).  The key axis then has
// `count` columns, all kept; the fused bias vector comes pre-gathered, and the causal limit of a query row
// is the number of kept columns at or below its diagonal instead of the column index itself.
template <typename T, int D, int BN, bool CAUSAL, int NW, bool CMP>
__global__ void __launch_bounds__(64 * NW, (NW == 4 && D <= 128) ? 2 : 1) fwd_colmask_kernel(const FwdParams p) {
    constexpr int NTHREADS = 64 * NW;
    constexpr int STHREADS = 256;             // threads staging one operand
    constexpr bool SPLIT = NW == 8;           // 8 waves: the first four stage V, the last four K and the side rows
    static_assert(NW == 4 || NW == 8, "staging maps are written for 256 or 512 threads");
    static_assert(BN == 64, "the pipeline works on the two 32-key halves of a 64-key tile");
    using E = Elem<T>;
    using SM = CmSmem<D, BN>;
    constexpr int KQ = BN / 4;                // key quads per tile
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int BM = 32 * NW;
    constexpr int CH = D / 8;                 // 16-byte chunks per K row
    constexpr int K_RPP = STHREADS / CH;      // K rows staged per pass
    constexpr int K_IT = BN / K_RPP;          // passes (registers) per K tile
    constexpr int V_ITEMS = KQ * CH;          // (key quad, d chunk) items of a V tile
    constexpr int V_IT = (V_ITEMS + STHREADS - 1) / STHREADS;  // items per staging thread (two at head dims above 128)
    constexpr int NL = SPLIT ? 4 : K_IT + 4 * V_IT;  // 16-byte loads per thread and tile
    constexpr int VB = SPLIT ? 0 : K_IT;      // first V staging register
    static_assert(!SPLIT || V_IT == 1, "the role split assumes one V item per thread");
    static_assert(!SPLIT || K_IT == 4, "the role split assumes four loads per thread for either operand");

    extern __shared__ __attribute__((aligned(16))) char smem[];
    uint32_t *sBits = (uint32_t *)(smem + SM::OFF_BITS);
    uint32_t *sFlag = (uint32_t *)(smem + SM::OFF_FLAG);

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (tells the compiler that it is wave-uniform)
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
    const int wrow0 = m0 + wave * 32;  // first query row of this wave

    // ---- Q fragments: the loads are issued first of all (they depend on the workgroup's coordinates only), the
    // values are looked at -- scaled -- after the set-up below, whose own memory traffic they overlap with
    u32x4_t qf[KS];
    {
        const int qrow = wrow0 + r;
        const int qc = qrow < LqS ? qrow : LqS - 1;
        const uint16_t *qp = (const uint16_t *)p.q + b * p.q_b + (sq.q0 + qc) * p.q_r + h * p.q_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + g * 8;
            qf[ks] = *(const u32x4_t *)(qp + (c < p.d ? c : 0));  // (chunks beyond d are cleared when scaled)
        }
    }

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
    // The upper halves of the side rows (both stages) are zero for good; the staging writes the lower halves.  V^T
    // stage 1 is cleared as well: the first pipeline step multiplies it with zero probabilities (there is no half tile
    // in front of the first one), and what an earlier workgroup left there need not be a number.  (All of it is made
    // visible by the barrier in front of the main loop.)
    if (tid < 2 * BN) *(u32x4_t *)(smem + SM::OFF_X + tid * 32 + 16) = u32x4_t{0, 0, 0, 0};
    for (int i = tid; i < SM::VT_BYTES / 16; i += NTHREADS)
        *(u32x4_t *)(smem + SM::OFF_VT + SM::VT_BYTES + i * 16) = u32x4_t{0, 0, 0, 0};
    if (!CMP) __syncthreads();  // (compacted keys have no bitmap: every tile up to n_end is active)

    // Iterator over the active tiles in ascending order (n_end once they are exhausted).  The current bitmap word
    // lives in a scalar register and loses a bit per call; LDS is read again only when a word runs out (readfirstlane
    // tells the compiler that the value is wave-uniform, so tile numbers, loop conditions and load addresses stay in
    // scalar registers).  Compacted keys have no bitmap: every tile up to n_end is active.
    uint32_t it_word = 0;
    int it_base = -32, it_next = 0;
    auto next_tile = [&]() -> int {
        if (CMP) {
            const int j = it_next < n_end ? it_next : n_end;
            it_next = j + 1;
            return j;
        }
        while (it_word == 0) {
            it_base += 32;
            if (it_base >= n_end) {
                it_base = n_end;  // (stays exhausted)
                return n_end;
            }
            it_word = __builtin_amdgcn_readfirstlane(sBits[it_base >> 5]);
        }
        const int j = it_base + __builtin_ctz(it_word);
        it_word &= it_word - 1;
        return j < n_end ? j : n_end;
    };

    f32x16_t o[DB];
    float row_sum = 0.f;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;

    // ---- staging (global -> registers -> LDS).  A tile is BN * CH 16-byte chunks of K plus V_ITEMS (key quad, d chunk)
    // items of V with four loads each (V is transposed in registers on its way to LDS).  Every load is unconditional,
    // from an always valid address: rows beyond the end of the keys are clamped to the last row (their side row says
    // -inf, so the duplicate never counts) and head-dim chunks beyond d to chunk 0 (they meet zero Q fragments /
    // columns of O that are not stored).  The per-thread byte offsets are loop invariants -- one set for full tiles,
    // one for the (only) partial tile at the end of the keys -- so a load is one instruction with a scalar tile base.
    const bool role_v = !SPLIT || wave < 4, role_k = !SPLIT || wave >= 4;  // wave-uniform
    const bool role_x = wave == 0;  // the side rows of a tile: lane l of wave 0 makes the row of key l
    const int kt = tid & (STHREADS - 1);
    const int kc = kt % CH, kr0 = kt / CH;
    const int vkg = kt % KQ, vc = (kt / KQ) % CH;  // V: key quad and d chunk of this thread
    const uint32_t k_r2 = (uint32_t)(p.k_r * 2), v_r2 = (uint32_t)(p.v_r * 2);  // bytes per row
    const uint32_t kcolb = (kc * 8 < p.d ? kc * 16 : 0);
    auto vchunk = [&](int j) -> int { return vc + j * (STHREADS / KQ); };  // d chunk of this thread's j-th V item
    const int j_last = Lk > 0 ? (Lk - 1) / BN : 0, last_row = Lk > 0 ? (Lk - 1) % BN : 0;
    uint32_t soff[NL], soff_l[NL];  // byte offsets of this thread's loads inside a full / the last tile
#pragma unroll
    for (int n = 0; n < NL; n++) {
        const bool is_v = SPLIT ? role_v : n >= K_IT;
        const int item = SPLIT ? n : (n >= K_IT ? n - K_IT : n);  // V: four loads (keys of the quad) per item
        const int row = is_v ? 4 * vkg + (item & 3) : kr0 + item * K_RPP;
        const uint32_t vcolb = (vchunk(item >> 2) * 8 < p.d ? vchunk(item >> 2) * 16 : 0);
        const uint32_t r2 = is_v ? v_r2 : k_r2, colb = is_v ? vcolb : kcolb;
        soff[n] = (uint32_t)row * r2 + colb;
        soff_l[n] = (uint32_t)(row < last_row ? row : last_row) * r2 + colb;
    }
    u32x4_t sreg[NL];             // staging registers
    uint32_t braw = 0, mraw = 0;  // raw bias / mask of this thread's column of the tile whose side rows are in flight
    // an absent mask / bias is read from K instead (any valid address) and ignored when the value is used
    const uint8_t *mrow_ld = mrow ? mrow : (const uint8_t *)kbase;
    const uint16_t *brow_ld = brow ? brow : kbase;
    bool bcol_ok = false;
    typedef const __attribute__((address_space(1))) char *gptr_t;  // global address space survives the integer round trip
    gptr_t tb_k = nullptr, tb_v = nullptr;        // tile bases (wave-uniform, in scalar registers)
    bool last_k = false, last_v = false;          // the K / V tile in flight is the partial one

    auto uniform_ptr = [](const char *ptr) -> gptr_t {
        const uint64_t v = (uint64_t)ptr;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (gptr_t)(((uint64_t)hi << 32) | lo);
    };
    // next fetches: K and the side-row inputs of tile jk / V of tile jv (with split roles a wave has one of the two)
    auto set_tile_k = [&](int jk) {
        if (!role_k) return;
        tb_k = uniform_ptr((const char *)kbase + (int64_t)jk * BN * p.k_r * 2);
        last_k = jk == j_last;
    };
    // side-row inputs of this thread's column of tile jx: only the raw loads here -- the values are looked at when
    // the row is stored
    auto set_tile_x = [&](int jx) {
        if (!role_x) return;
        const int col = jx * BN + lane;
        const int cc = col < Lk ? col : 0;
        bcol_ok = col < Lk;
        // (unconditional loads: a load in one arm of a select would have to be waited for right here)
        if (CMP) {
            braw = __float_as_uint(fbrow[cc]);
        } else {
            mraw = mrow_ld[cc];
            braw = brow_ld[cc];
        }
    };
    auto set_tile_v = [&](int jv) {
        if (!role_v) return;
        tb_v = uniform_ptr((const char *)vbase + (int64_t)jv * BN * p.v_r * 2);
        last_v = jv == j_last;
    };
    // the loads of this thread's K registers / V registers (with split roles: all NL registers, in the waves of that role)
    auto load_regs = [&](bool v) {
        if (SPLIT ? (v ? !role_v : !role_k) : false) return;
        const gptr_t base = v ? tb_v : tb_k;
        const bool last = v ? last_v : last_k;
        const int n0 = SPLIT ? 0 : (v ? K_IT : 0), n1 = SPLIT ? NL : (v ? NL : K_IT);
#pragma unroll
        for (int n = n0; n < n1; n++)
            sreg[n] = *(const __attribute__((address_space(1))) u32x4_t *)(base + (last ? soff_l[n] : soff[n]));
    };
    // registers -> LDS: K into stage kbuf, the side rows into stage xbuf, V^T into stage vbuf
    auto store_k = [&](int kbuf) {
        if (role_k) {
            char *sK = smem + SM::OFF_K + kbuf * SM::K_BYTES;
#pragma unroll
            for (int it = 0; it < K_IT; it++)
                *(u32x4_t *)(sK + ((kr0 + it * K_RPP) * SM::SK + kc * 8) * 2) = sreg[it];
        }
    };
    auto store_x = [&](int xbuf) {
        if (role_x) {  // side row of this lane's key: pieces of bias * log2e, the mask term, the two ones
            float v = 0.f;
            bool keep = bcol_ok;
            if (CMP) {
                v = __uint_as_float(braw);
            } else {
                keep = keep && (!mrow || mraw);
                if (brow) v = E::lo(braw) * kLog2e;
            }
            const u32x2_t pc = split3<T>(keep ? v : 0.f);
            u32x4_t row;
            row[0] = pc[0];
            row[1] = pc[1] | (E::pack2(0.f, keep ? 0.f : -INFINITY) & 0xffff0000u);
            row[2] = E::pack2(E::kRefWeight, 1.f);
            row[3] = 0;
            *(u32x4_t *)(smem + SM::OFF_X + xbuf * SM::X_BYTES + lane * 32) = row;
        }
    };
    auto store_v = [&](int vbuf) {
        if (role_v && kt < V_ITEMS) {  // transpose 4 keys x 8 d in registers, write V^T[d][key quad]
            char *sVt = smem + SM::OFF_VT + vbuf * SM::VT_BYTES;
#pragma unroll
            for (int dj = 0; dj < 8 * V_IT; dj++) {
                const int j = dj >> 3, dd = dj & 7, w = dd >> 1;
                const uint32_t sel = (dd & 1) ? 0x07060302u : 0x05040100u;
                u32x2_t out;
                out[0] = __builtin_amdgcn_perm(sreg[VB + 4 * j + 1][w], sreg[VB + 4 * j + 0][w], sel);
                out[1] = __builtin_amdgcn_perm(sreg[VB + 4 * j + 3][w], sreg[VB + 4 * j + 2][w], sel);
                *(u32x2_t *)(sVt + ((vchunk(j) * 8 + dd) * SM::SVT + 4 * vkg) * 2) = out;
            }
        }
    };

    const int a_row = pi_row(r);

    // causal limits: columns below vis_lane are visible to this lane's query row, and a half tile that ends at
    // or below vis_wave (the limit of the wave's first row) needs no masking at all
    const int vis_lane = CAUSAL ? visible(wrow0 + r) : 0;
    const int vis_wave = CAUSAL ? visible(wrow0) : 0;

    // Constants of a query row that meet the side rows of the keys (B operand of the extra k-step; the lanes of
    // the upper half supply zeros against the zero half of the side rows): 1 / kPieceScale for the three bias
    // pieces, 1 for the mask term, and the two pieces of minus the row's reference point.
    const float side_mult = 1.f / E::kPieceScale;
    u32x4_t qx;
    qx[0] = g == 0 ? E::pack2(side_mult, side_mult) : 0u;
    qx[1] = g == 0 ? E::pack2(side_mult, 1.f) : 0u;
    qx[2] = 0u;
    qx[3] = 0u;
    // Softmax state of a row: O and row_sum are relative to exp2(row_ref); enc_ref is what the pieces in qx stand
    // for, i.e. what the score MFMAs subtract.  row_ref = -inf: no visible key met yet (enc_ref is 0 then).  On the
    // common path row_ref == enc_ref for every row of the wave (`fast`, wave-uniform).
    float row_ref = -INFINITY, enc_ref = 0.f;
    bool fast = false;

    // Fragment addresses of a half tile.  Scores: side rows + KS k-steps of K for the 32 keys of half `kh` of stage
    // `kbuf`; P V: the two 16-key k-steps of half `vh` of V^T stage `vbuf`, DB row blocks each.
    constexpr int NQK = KS + 1, NPV = 2 * DB, NF = NQK + NPV;
    constexpr int FR = 4;  // fragment reads run FR MFMAs ahead of their MFMAs (8 ahead: 19 spilled registers)
    auto frag_ptr = [&](int f, int kbuf, int kh, int vbuf, int vh) -> const u32x4_t * {
        if (f == 0) return (const u32x4_t *)(smem + SM::OFF_X + kbuf * SM::X_BYTES + (32 * kh + a_row) * 32 + g * 16);
        if (f < NQK)
            return (const u32x4_t *)(smem + SM::OFF_K + kbuf * SM::K_BYTES + ((32 * kh + a_row) * SM::SK + (f - 1) * 16 + g * 8) * 2);
        const int kb = (f - NQK) / DB, db = (f - NQK) % DB;
        return (const u32x4_t *)(smem + SM::OFF_VT + vbuf * SM::VT_BYTES + ((32 * db + a_row) * SM::SVT + 32 * vh + 16 * kb + 8 * g) * 2);
    };
    const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // causal masking of a half tile whose first column is col0 (register i <-> column 16 (i / 8) + 8 g + i % 8)
    auto causal_mask = [&](f32x16_t &s, int col0) {
        const int lim = vis_lane - 1 - col0 - 8 * g;  // local column limit for this lane
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int lc = 16 * (i >> 3) + (i & 7);
            s[i] = lc <= lim ? s[i] : -INFINITY;
        }
    };

    // Classic softmax of one half tile (the safe path, and the first tile of the common path's set-up): maximum, a new
    // reference point where the row has none yet or a score exceeds the old one by more than 2^8 (then O and the sums are
    // rescaled, and the pieces in qx replaced), probabilities.  The scores in `s` are relative to enc_ref as it is on entry.
    auto classic = [&](f32x16_t &s, uint32_t (&pk)[8], int col0) {
        if (CAUSAL && col0 + 32 > vis_wave) causal_mask(s, col0);
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[i]);
        tmax = xhalf_max(tmax);
        const bool unset = row_ref == -INFINITY;
        const float cand = enc_ref + tmax;  // the half tile's maximum as an absolute score
        const bool move = unset ? tmax > -INFINITY : cand > row_ref + 8.f;
        float shift_s = unset ? 0.f : enc_ref - row_ref;  // probabilities are exp2(s + shift_s)
        if (__any(move)) {
            float enc;
            const uint32_t w = encode_ref<T>(cand, enc);
            // the reference becomes exactly what the pieces stand for, unless they cannot express it (fp16,
            // scores beyond 4e6): then the remainder stays in shift_s
            const float new_ref = move ? (fabsf(enc - cand) <= 0.5f ? enc : cand) : row_ref;
            const float alpha = (move && !unset) ? fast_exp2(row_ref - new_ref) : 1.f;
            row_sum *= alpha;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[db][i] *= alpha;
            if (move) {
                shift_s = enc_ref - new_ref;
                enc_ref = enc;
                if (g == 0) qx[2] = w;
            }
            row_ref = new_ref;
        }
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const uint32_t w = E::pack2(fast_exp2(s[i] + shift_s), fast_exp2(s[i + 1] + shift_s));
            psum = E::add_pair(w, psum);
            pk[i / 2] = w;
        }
        row_sum += psum;
    };
    // scores of half kh of K stage kbuf / P V of half vh of V^T stage vbuf, on their own (set-up, tail, safe path)
    auto scores_half = [&](f32x16_t &s, int kbuf, int kh) {
        u32x4_t a[NQK];
#pragma unroll
        for (int f = 0; f < NQK; f++) a[f] = *frag_ptr(f, kbuf, kh, 0, 0);
        s = E::mfma(a[0], qx, zero16);
#pragma unroll
        for (int f = 1; f < NQK; f++) s = E::mfma(a[f], qf[f - 1], s);
    };
    auto pv_half = [&](const uint32_t (&pk)[8], int vbuf, int vh) {
        u32x4_t a[NPV];
#pragma unroll
        for (int f = 0; f < NPV; f++) a[f] = *frag_ptr(NQK + f, 0, 0, vbuf, vh);
#pragma unroll
        for (int f = 0; f < NPV; f++) {
            const int kb = f / DB, db = f % DB;
            const u32x4_t bop = {pk[4 * kb], pk[4 * kb + 1], pk[4 * kb + 2], pk[4 * kb + 3]};
            o[db] = E::mfma(a[f], bop, o[db]);
        }
    };

    // One step of the pipeline.  MFMAs: scores of the NEXT half tile (half kh of K stage kbuf) into `snext`, and
    // O^T += V^T P^T of the PREVIOUS half tile (probabilities pprev, half vh of V^T stage vbuf).  Vector ALU, between
    // them: softmax of the CURRENT half tile `scur` (first column col0) into `pcur` -- the common path, no maximum.
    // A step also moves one staged operand from the registers to LDS, piece by piece between its MFMAs, and issues that
    // operand's next loads behind them: V (and, in wave 0, the side rows) in the first step of a tile (STAGE), K in the
    // second.  With split roles the two waves of a SIMD have different roles.  (Staging as a phase of its own, after or
    // in front of the MFMAs, left the matrix pipe to the SIMD's other wave alone for a fifth of every tile.  Half tiles
    // on the causal diagonal are masked before the step, in code of their own: only they pay for it.)
    auto step = [&](auto stage_c, auto do_v_c, auto do_k_c, f32x16_t &scur, f32x16_t &snext, uint32_t (&pcur)[8],
                    const uint32_t (&pprev)[8], int kbuf, int kh, int vbuf, int vh, int j_next, int jx_next) {
        constexpr bool STAGE = decltype(stage_c)::value;
        constexpr bool DO_V = STAGE && decltype(do_v_c)::value, DO_K = !STAGE && decltype(do_k_c)::value;
        char *const sVt_w = smem + SM::OFF_VT + (vbuf ^ 1) * SM::VT_BYTES;  // V(t) goes to the stage the P V product has left
        char *const sK_w = smem + SM::OFF_K + (kbuf ^ 1) * SM::K_BYTES;     // K(t+2) to the stage whose scores are finished
        // Order of issue: a wave issues in program order, so the vector instructions have to sit BETWEEN the MFMAs to run
        // under them.  The step is written slot by slot -- one MFMA, the fragment read of the MFMA FR slots later, an even
        // share of the softmax (the two exp2 of a pair of scores in one slot, their conversion to 16 bits and their
        // addition to the row sum in the next, a piece of the staging) -- with a scheduling barrier after every slot.
        // The probabilities are relative to the reference the MFMAs have already subtracted; the row sum adds the
        // fp32 values, as the reference does (src/softmax.h: the sum is taken before the conversion to 16 bits).
        if (DO_K) set_tile_k(j_next);  // base of the tile whose pieces are requested between the MFMAs below
        u32x4_t a[NF];
#pragma unroll
        for (int f = 0; f < FR; f++) a[f] = *frag_ptr(f, kbuf, kh, vbuf, vh);
        float psum0 = 0.f, psum1 = 0.f, x0[8], x1[8];
#pragma unroll
        for (int f = 0; f < NF; f++) {
            if (f + FR < NF) a[f + FR] = *frag_ptr(f + FR, kbuf, kh, vbuf, vh);
            if (f == 0) {
                snext = E::mfma(a[f], qx, zero16);
            } else if (f < NQK) {
                snext = E::mfma(a[f], qf[f - 1], snext);
            } else {
                const int kb = (f - NQK) / DB, db = (f - NQK) % DB;
                const u32x4_t bop = {pprev[4 * kb], pprev[4 * kb + 1], pprev[4 * kb + 2], pprev[4 * kb + 3]};
                o[db] = E::mfma(a[f], bop, o[db]);
            }
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int slot = k * (NF - 1) / 8;  // the pair's exp2 slot; its conversion follows one slot later
                if (slot == f) {
                    x0[k] = fast_exp2(scur[2 * k]);
                    x1[k] = fast_exp2(scur[2 * k + 1]);
                }
                if (slot + 1 == f) {
                    pcur[k] = E::pack2(x0[k], x1[k]);
                    psum0 += x0[k];
                    psum1 += x1[k];
                }
            }
            // staging, a piece per slot: one transposed row pair of V (two permutes, one 8-byte store) / one 16-byte
            // chunk of K
            if (DO_V) {
#pragma unroll
                for (int dj = 0; dj < 8 * V_IT; dj++)
                    if (f == 1 + dj * ((NF - 1) / (8 * V_IT))) {
                        const int j = dj >> 3, dd = dj & 7, w = dd >> 1;
                        const uint32_t sel = (dd & 1) ? 0x07060302u : 0x05040100u;
                        u32x2_t out;
                        out[0] = __builtin_amdgcn_perm(sreg[VB + 4 * j + 1][w], sreg[VB + 4 * j + 0][w], sel);
                        out[1] = __builtin_amdgcn_perm(sreg[VB + 4 * j + 3][w], sreg[VB + 4 * j + 2][w], sel);
                        *(u32x2_t *)(sVt_w + ((vchunk(j) * 8 + dd) * SM::SVT + 4 * vkg) * 2) = out;
                    }
            }
            if (DO_K) {
                // (a register goes back to fetching -- the same piece of K(j_next) -- as soon as it is stored: a whole
                // tile then lies between every load and its store; all four loads behind the last MFMA had half a tile)
#pragma unroll
                for (int it = 0; it < K_IT; it++)
                    if (f == 1 + it * ((NF - 1) / K_IT)) {
                        *(u32x4_t *)(sK_w + ((kr0 + it * K_RPP) * SM::SK + kc * 8) * 2) = sreg[it];
                        sreg[it] = *(const __attribute__((address_space(1))) u32x4_t *)(tb_k + (last_k ? soff_l[it] : soff[it]));
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        const float psum = psum0 + psum1;
        row_sum += psum;
        // (the results are pinned here: left alone, the compiler sinks the softmax below the staging code that follows,
        // away from the MFMAs it is meant to run under)
#pragma unroll
        for (int i = 0; i < 8; i++) asm volatile("" : "+v"(pcur[i]));
        asm volatile("" : "+v"(row_sum));
        __builtin_amdgcn_sched_barrier(0);
        if (STAGE) {  // the loads of V(j_next); side rows of the next tile, inputs of those of the tile after it
            store_x(kbuf ^ 1);  // (in front of the new loads: its inputs must not be waited for together with them)
            if (DO_V) {
                set_tile_v(j_next);
                load_regs(true);
            }
            set_tile_x(jx_next);
        }
        if (__any(!(psum <= 16384.f))) *sFlag = 1u;
    };

    const int j0 = next_tile();
    bool redo = false;
    if (j0 < n_end) {
        // ---- common path.  Set-up: the first tile is staged, its scores are computed once just for their row maxima,
        // and the reference point of every row is put kRefMargin above its maximum: probabilities start around
        // 2^-margin, and the rest of the row may exceed the first tile by margin + 14 before the check fails.
        int jc = j0, jn1 = next_tile(), jn2 = next_tile(), jn3 = next_tile();
        if (tid == 0) *sFlag = 0u;
        // K(0), K(1) and the side rows of tile 0 go to LDS; the registers then fetch K(2), V(0) (kept until step A)
        // and the side-row inputs of tile 1
        set_tile_k(j0);
        set_tile_v(j0);
        set_tile_x(j0);
        load_regs(false);
        load_regs(true);
        u32x4_t k1[K_IT];  // K(1) travels in registers of its own, together with K(0)
        set_tile_k(jn1 < n_end ? jn1 : j0);
        if (role_k) {
#pragma unroll
            for (int it = 0; it < K_IT; it++)
                k1[it] = *(const __attribute__((address_space(1))) u32x4_t *)(tb_k + (last_k ? soff_l[it] : soff[it]));
        }
        store_k(0);
        store_x(0);
        set_tile_x(jn1 < n_end ? jn1 : j0);
        if (role_k) {
#pragma unroll
            for (int it = 0; it < K_IT; it++) sreg[it] = k1[it];
        }
        store_k(1);
        set_tile_k(jn2 < n_end ? jn2 : j0);
        load_regs(false);
        // Q is scaled by softmax_scale * log2(e) once, here (the reference also rounds the scaled Q to the input type,
        // flash_fwd_kernel.h:428-439): the MFMAs then produce exp2-domain scores directly
        {
            const bool row_ok = wrow0 + r < LqS;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                const bool ok = row_ok && ks * 16 + g * 8 < p.d;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    qf[ks][e] = ok ? E::pack2(E::lo(qf[ks][e]) * p.scale_log2, E::hi(qf[ks][e]) * p.scale_log2) : 0u;
            }
        }
        __syncthreads();

        f32x16_t sA, sB;
        uint32_t pA[8], pB[8];
        {
            scores_half(sA, 0, 0);
            scores_half(sB, 0, 1);
            const int col0 = j0 * BN;
            if (CAUSAL && col0 + 32 > vis_wave) causal_mask(sA, col0);
            if (CAUSAL && col0 + 64 > vis_wave) causal_mask(sB, col0 + 32);
            float tmax = -INFINITY;
#pragma unroll
            for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, fmaxf(sA[i], sB[i]));
            tmax = xhalf_max(tmax);
            bool bad = false;
            if (tmax > -INFINITY) {  // (a row that sees nothing in the first tile sees nothing at all)
                const float want = tmax + (std::is_same<T, bf16_tag>::value ? 8.f : 4.f);
                float enc;
                const uint32_t w = encode_ref<T>(want, enc);
                bad = !(fabsf(enc - want) <= 0.5f);  // the pieces cannot express it: safe path
                enc_ref = row_ref = enc;
                if (g == 0) qx[2] = w;
            }
            if (__any(bad)) *sFlag = 1u;
            scores_half(sA, 0, 0);  // again, against the reference
        }
#pragma unroll
        for (int i = 0; i < 8; i++) pB[i] = 0u;

        // ---- main loop.  Iteration t works on active tile t (halves 2t and 2t+1 go through the softmax).  On entry K(t)
        // and K(t+1) are in the two K stages (K(t) in stage t & 1), the side rows of tile t in stage t & 1 and V(t-1) in
        // V^T stage (t-1) & 1; the registers hold K(t+2), V(t) and the side-row inputs of tile t+1; sA holds the scores of
        // half 2t, pB the probabilities of half 2t-1.
        //   step A: scores of half 2t+1 (K(t), second half), softmax of half 2t, P V of half 2t-1 (V(t-1), second half);
        //           then V(t) -> V^T stage t & 1 and the loads of V(t+1); side rows of tile t+1 -> stage (t+1) & 1,
        //           inputs of those of tile t+2
        //   barrier
        //   step B: K(t+2) -> K stage t & 1 and the loads of K(t+3); then scores of half 2t+2 (K(t+1), first half),
        //           softmax of half 2t+1, P V of half 2t (V(t), first half)
        // A stage is written after the barrier that follows its last read, and read after the barrier that follows its
        // write.  Past the last tile an existing tile is fetched and stored again and what is computed from it is dropped.
        const std::true_type yes;
        const std::false_type no;
        int t = 0;
        // (the loop exists once per staging role, so that the staging pieces inside the steps are unconditional code)
        auto tile_loop = [&](auto do_v_c, auto do_k_c) {
            while (true) {
                const int kb = t & 1;
                const int col0 = jc * BN;
                if (CAUSAL && col0 + 32 > vis_wave) causal_mask(sA, col0);
                __builtin_amdgcn_sched_barrier(0);
                step(yes, do_v_c, do_k_c, sA, sB, pA, pB, kb, 1, kb ^ 1, 1, jn1 < n_end ? jn1 : jc, jn2 < n_end ? jn2 : jc);
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
                if (CAUSAL && col0 + 64 > vis_wave) causal_mask(sB, col0 + 32);
                step(no, do_v_c, do_k_c, sB, sA, pB, pA, kb ^ 1, 0, kb, 0, jn3 < n_end ? jn3 : jc, 0);
                __builtin_amdgcn_sched_barrier(0);
                t++;
                jc = jn1; jn1 = jn2; jn2 = jn3;
                if (jc >= n_end) break;
                jn3 = next_tile();
            }
        };
        const bool do_v = __builtin_amdgcn_readfirstlane((int)(role_v && kt < V_ITEMS)) != 0;
        if (do_v) {
            tile_loop(yes, std::integral_constant<bool, !SPLIT>());
        } else {
            tile_loop(no, yes);
        }
        pv_half(pB, (t - 1) & 1, 1);  // P V of the last half: V of the last tile, second half
        __syncthreads();
        redo = *sFlag != 0u;  // (the same for every wave)
    }
    if (redo) {
        // ---- safe path: the whole workgroup again, tile by tile, with the classic softmax (maximum per half tile,
        // reference moved and O rescaled as needed).  One stage, no prefetch: this path is for inputs whose scores
        // climb by more than the common path's range after the first tile, not for speed.
        row_sum = 0.f;
        row_ref = -INFINITY;
        enc_ref = 0.f;
        qx[2] = 0u;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) o[db][i] = 0.f;
        it_word = 0;
        it_base = -32;
        it_next = 0;
        for (int j = next_tile(); j < n_end; j = next_tile()) {
            set_tile_k(j);
            set_tile_v(j);
            set_tile_x(j);
            load_regs(false);
            load_regs(true);
            __syncthreads();  // every wave is done with the stage
            store_k(0);
            store_v(0);
            store_x(0);
            __syncthreads();
            f32x16_t s0, s1;
            uint32_t p0[8], p1[8];
            scores_half(s0, 0, 0);
            scores_half(s1, 0, 1);  // (both against the same pieces: classic() below may replace them)
            const float enc_before = enc_ref;
            classic(s0, p0, j * BN);
            pv_half(p0, 0, 0);  // (before the second half may move the reference and rescale O again)
            const float fix = enc_before - enc_ref;
#pragma unroll
            for (int i = 0; i < 16; i++) s1[i] += fix;
            classic(s1, p1, j * BN + 32);
            pv_half(p1, 0, 1);
        }
    }

    // ---- epilogue
    {
        const int qrow = wrow0 + r;
        const float total = xhalf_sum(row_sum);
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
                            w[e] = E::pack2(o[db][8 * blk + 2 * e] * inv, o[db][8 * blk + 2 * e + 1] * inv);
                        *(u32x4_t *)(op + c) = w;
                    }
                }
            if (g == 0) {
                const float lse = total > 0.f ? (row_ref + __builtin_amdgcn_logf(total)) * kLn2 : INFINITY;
                p.lse[b * p.lse_b + h * p.lse_h + sq.q0 + qrow] = lse;
            }
        }
    }
}

template <typename T, int D, int BN, bool CAUSAL, bool CMP, int NW = 4>
hipError_t launch_one(const FwdParams &p, hipStream_t stream) {
    constexpr int BM = 32 * NW;
    auto kern = fwd_colmask_kernel<T, D, BN, CAUSAL, NW, CMP>;
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
        if (p.cmp.on) return p.causal ? launch_one<T, D, 64, true, true, 8>(p, stream) : launch_one<T, D, 64, false, true, 8>(p, stream);
        return p.causal ? launch_one<T, D, 64, true, false, 8>(p, stream) : launch_one<T, D, 64, false, false, 8>(p, stream);
    }
    if (p.cmp.on) return p.causal ? launch_one<T, D, 64, true, true>(p, stream) : launch_one<T, D, 64, false, true>(p, stream);
    return p.causal ? launch_one<T, D, 64, true, false>(p, stream) : launch_one<T, D, 64, false, false>(p, stream);
}

}  // namespace

bool fwd_colmask_applicable(const FwdParams &p) {
    const bool mask_ok = !p.mask || p.m_r == 0;
    const bool bias_ok = !p.bias || p.bi_r == 0;
    return mask_ok && bias_ok && (p.Lk + 31) / 32 <= MAX_TILES;
}

hipError_t launch_fwd_colmask(const FwdParams &p, int dtype, hipStream_t stream) {
    if (p.cmp.on && p.cmp.img_kv) return launch_fwd_stream(p, dtype, stream);  // (the pre-pass has written tile images)
    // head dims up to 64 / 128 / 256 (a head dim in between runs in the next larger instantiation)
    if (dtype == 0) return p.d <= 64 ? launch_d<bf16_tag, 64>(p, stream) : p.d <= 128 ? launch_d<bf16_tag, 128>(p, stream) : launch_d<bf16_tag, 256>(p, stream);
    return p.d <= 64 ? launch_d<fp16_tag, 64>(p, stream) : p.d <= 128 ? launch_d<fp16_tag, 128>(p, stream) : launch_d<fp16_tag, 256>(p, stream);
}

}  // namespace fdma
