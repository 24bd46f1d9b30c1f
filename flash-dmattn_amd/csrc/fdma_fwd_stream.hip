// Forward dynamic-mask attention for gfx950 on compacted keys, streaming form: head dim 128, 256 query rows per
// workgroup, one resident workgroup per CU.
//
// Same math and same reference counterpart as fdma_fwd_colmask.hip (compute_attn_1rowblock,
// csrc/flash_sparse_attn/src/flash_fwd_kernel.h:53-804 of the reference; its hot loop :454-731), and the same tile
// program: scores through the matrix pipe with the softmax's bias / mask / reference point folded into one more
// k-step (the 16-element side rows), a software pipeline over 32-key half tiles, no row maximum on the common path.
// What differs is everything around the tile program:
//   * Tile images.  The compaction pre-pass (compact_scan_image_kernel / compact_image_kernel, fdma_compact.hip) has
//     written, per 64-key tile of the compacted key axis, exactly the bytes this kernel keeps in LDS: the K tile with
//     padded rows -- already multiplied by softmax_scale * log2(e), so Q is used as it lies in memory -- followed
//     by V already transposed, and the side rows of the keys.  A tile is fetched with contiguous direct
//     global->LDS loads (global_load_lds_dwordx4: a wave moves 1 KB per instruction, lane after lane): no staging
//     registers, no permutes, no LDS stores, no staging roles -- V is transposed once per (batch, kv head) pair
//     instead of once per workgroup that reads it.
//   * One stream of tiles per workgroup.  A workgroup is resident and walks its share of the (query block, head)
//     items; the tiles of all its items form one sequence that is fetched THREE tiles ahead of the tile being
//     worked on, through a ring of four LDS slots, regardless of where one item ends and the next begins: when an
//     item starts, its first tiles are in LDS already.  (With a workgroup per item every item paid for its own
//     first fetch with nothing else running on the CU: a quarter of the launch at 17 tiles per item.)
//   * The rare items whose scores leave the common path's range (or whose reference point cannot be expressed)
//     are noted in an LDS bit set and redone at the end of the workgroup's life by a plain tile-by-tile path that
//     reads its fragments straight from the images in global memory.
//   * Output rows leave under the next item's matrix work: an item ends by packing its rows into registers, and the
//     next item's first step behind a barrier issues the stores one per slot (see pack_rows / store_piece).
// Items are dealt to the workgroups of an XCD in rounds, odd rounds reversed: heaviest query blocks first, every
// workgroup the same causal work, K / V of a (batch, kv head) pair in one XCD's L2.
#include <type_traits>

#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

#ifdef FDMA_DBG
__device__ uint64_t g_stream_dbg[1024 * 64];
#define FDMA_STAMP(slot) do { if (tid == 0 && (slot) < 64) g_stream_dbg[blockIdx.x * 64 + (slot)] = wall_clock64(); } while (0)
#else
#define FDMA_STAMP(slot) do { } while (0)
#endif

namespace {

constexpr int ST_NW = 8, ST_THREADS = 64 * ST_NW, ST_BM = 32 * ST_NW;
constexpr int ST_D = 128, ST_BN = IMG_BN;
constexpr int ST_SLOTS = 4;        // ring of tile slots: one being worked on, one whose V is still needed, two on their way
constexpr int ST_MAX_ROUNDS = 4096;  // items a workgroup may walk (LDS: tile counts and the redo bit set)
constexpr int ST_NDMA = 5;         // direct loads per wave and tile: 35 pieces of K | V^T, 2 of side rows, 3 repeats = 40

struct StSmem {
    static constexpr int OFF_KV = 0;                                  // [slot][K tile | V^T tile]
    static constexpr int OFF_X = OFF_KV + ST_SLOTS * IMG_KV_BYTES;    // [slot][side rows]
    static constexpr int OFF_NT = OFF_X + ST_SLOTS * IMG_X_BYTES;     // tiles of this workgroup's item of every round (u16)
    static constexpr int OFF_REDO = OFF_NT + ST_MAX_ROUNDS * 2;       // bit per round: redo with the classic softmax
    static constexpr int TOTAL = OFF_REDO + ST_MAX_ROUNDS / 8;
};
static_assert(StSmem::TOTAL <= 160 * 1024, "LDS of one CU");
static_assert(IMG_KV_BYTES == 35 * 1024 && IMG_X_BYTES == 2 * 1024, "the piece map below");

template <typename T, bool CAUSAL>
__global__ void __launch_bounds__(ST_THREADS, 1) fwd_stream_kernel(const FwdParams p, int items_per_xcd, int wgs_per_xcd, int rounds) {
    using E = Elem<T>;
    using SM = StSmem;
    constexpr int D = ST_D, BN = ST_BN, BM = ST_BM;
    constexpr int DB = D / 32;
    constexpr int SK = IMG_SK, SVT = IMG_SVT;

    // (LDS is addressed by absolute byte address throughout: the direct loads are written in assembly, see dma16)
    extern __shared__ __attribute__((aligned(256))) char smem[];
    const uint32_t lds0 = lds_addr(smem);
    uint16_t *sNt = (uint16_t *)(smem + SM::OFF_NT);
    uint32_t *sRedo = (uint32_t *)(smem + SM::OFF_REDO);

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int r = lane & 31;
    const int g = lane >> 5;
    FDMA_STAMP(0);
#ifdef FDMA_DBG
    if (tid == 0) g_stream_dbg[blockIdx.x * 64 + 38] = __builtin_amdgcn_s_memtime();
#endif

    // ---- items.  The (batch, kv head) pairs are split into k = 8 / gcd(pairs, 8) interleaved lists of query blocks
    // each, the lists are dealt to the 8 XCDs (workgroup id % 8), an XCD walks its lists one after the other, heaviest
    // query block first, the G query heads of a block side by side: item `slot` of the XCD.  Round `rd` gives this
    // workgroup slot rd * W + (its place among the W workgroups of the XCD, reversed in odd rounds).
    const int n_mb = (p.Lq + BM - 1) / BM;
    const int G = p.H / p.Hk;
    const int pairs = p.B * p.Hk;
    const int gcd8 = (pairs % 8 == 0) ? 8 : ((pairs % 4 == 0) ? 4 : ((pairs % 2 == 0) ? 2 : 1));
    const int k_split = 8 / gcd8;
    const int list_len = ((n_mb + k_split - 1) / k_split) * G;
    const int xcd = blockIdx.x & 7, place = blockIdx.x >> 3;
    const int Lq = p.Lq, LkO = p.Lk, shift = LkO - Lq;
    struct Item { int pair, h, m0; };
    auto item_of = [&](int rd, Item &it) -> bool {
        const int slot = rd * wgs_per_xcd + ((rd & 1) ? wgs_per_xcd - 1 - place : place);
        if (slot >= items_per_xcd) return false;
        const int vlist = xcd + 8 * (slot / list_len);
        const int pos = slot % list_len;
        const int mslot = (pos / G) * k_split + vlist % k_split;
        if (mslot >= n_mb) return false;
        it.pair = vlist / k_split;
        it.h = (it.pair % p.Hk) * G + pos % G;
        it.m0 = (n_mb - 1 - mslot) * BM;
        return it.m0 < Lq;
    };
    // compacted columns that pass the causal test for query row `row` of pair `pair`
    auto visible = [&](int pair, int row) -> int {
        if (row >= Lq) row = Lq - 1;
        const int c = row + shift;
        if (c < 0) return 0;
        return p.cmp.cnt[(int64_t)pair * p.cmp.ld + (c < LkO ? c : LkO - 1)];
    };

    constexpr int KS = ST_D / 16;
    u32x4_t qf[KS];
    int vis_lane = 0;
    // (What the item-boundary code below computes per lane -- row numbers, addresses -- is made to depend on a value the
    // compiler cannot see through: left alone it computes all of it at the top of the item, in front of the tile loop,
    // and the results then sit in registers that the tile loop needs.)
    auto opaque = [](int x) -> int {
        asm volatile("" : "+v"(x));
        return x;
    };
    // Q fragments of an item's rows, as they lie in memory: the K rows of the images carry softmax_scale * log2(e).  (Rows
    // beyond the end repeat the last row; they are never stored.)
    auto load_q = [&](const Item &it) {
        const int b = it.pair / p.Hk;
        const int qrow = it.m0 + wave * 32 + opaque(r);
        const int qc = qrow < Lq ? qrow : Lq - 1;
        const uint16_t *qp = (const uint16_t *)p.q + b * p.q_b + (int64_t)qc * p.q_r + it.h * p.q_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) qf[ks] = *(const u32x4_t *)(qp + ks * 16 + g * 8);
        if (CAUSAL) vis_lane = visible(it.pair, qrow);
    };
    // ---- the first item with rows: its Q is requested first of all (the tables and the first tiles travel meanwhile);
    // later items request theirs a step before they start
    int rd = 0;
    Item cur;
    while (rd < rounds && !item_of(rd, cur)) rd++;
    if (rd < rounds) load_q(cur);
    // ---- tiles of every round's item (0 for rounds without an item); the redo bit set; the slot the first step
    // multiplies with zero probabilities holds numbers
#pragma unroll 1
    for (int rd = tid; rd < rounds; rd += ST_THREADS) {
        Item it;
        int nt = 0;
        if (item_of(rd, it)) {
            int lim = p.cmp.count[it.pair];
            if (CAUSAL) {
                const int v = visible(it.pair, it.m0 + BM - 1);
                lim = v < lim ? v : lim;
            }
            nt = (lim + BN - 1) / BN;
        }
        sNt[rd] = (uint16_t)nt;
    }
    for (int i = tid; i < ST_MAX_ROUNDS / 32; i += ST_THREADS) sRedo[i] = 0u;
    for (int i = tid; i < IMG_VT_BYTES / 16; i += ST_THREADS)
        *(u32x4_t *)(smem + SM::OFF_KV + (ST_SLOTS - 1) * IMG_KV_BYTES + IMG_K_BYTES + i * 16) = u32x4_t{0, 0, 0, 0};
    __syncthreads();

    // ---- the fetch side.  One direct load: 64 lanes x 16 bytes from `base` (wave-uniform) + lane * 16 to the LDS
    // address `dst` (wave-uniform) onwards, lane after lane.  Written in assembly: issued through the compiler's
    // builtin, every later LDS read would wait for all direct loads in flight (the compiler cannot tell which slot they
    // fill); the waits are placed by hand (publish()).  m0 carries the LDS address; nothing else here uses it.
    typedef const __attribute__((address_space(1))) char *gptr_t;
    const uint32_t lane16 = (uint32_t)lane * 16u;
    auto dma16 = [&](gptr_t base, uint32_t dst) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     : : "v"(lane16), "s"(base), "s"(__builtin_amdgcn_readfirstlane(dst)) : "memory");
    };
    auto uniform_ptr = [](const char *ptr) -> gptr_t {
        const uint64_t v = (uint64_t)ptr;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (gptr_t)(((uint64_t)hi << 32) | lo);
    };
    // Fetch cursor: the tile fetched next is tile f_tile of the item of round f_round (f_nt tiles), at f_kv / f_x; it goes
    // to ring slot f_pos & 3.  Past the last tile of the last item the last tile is fetched again (the slot is free by
    // then and nobody reads it): every wave issues ST_NDMA loads per tile, always, which is what the waits count on.
    int f_round = -1, f_tile = 0, f_nt = 0;
    uint32_t f_pos = 0;
    gptr_t f_kv = nullptr, f_x = nullptr;
    auto fetch_enter_next_item = [&]() -> bool {  // moves the cursor to the next round that has tiles
        int rd = f_round + 1;
        while (rd < rounds && __builtin_amdgcn_readfirstlane((int)sNt[rd]) == 0) rd++;
        if (rd >= rounds) return false;
        Item it;
        item_of(rd, it);
        const int hfb = p.cmp.Hfb == p.H ? it.h : it.pair % p.Hk;
        const int b = it.pair / p.Hk;
        f_round = rd;
        f_tile = 0;
        f_nt = __builtin_amdgcn_readfirstlane((int)sNt[rd]);
        f_kv = uniform_ptr(p.cmp.img_kv + (int64_t)it.pair * p.cmp.img_tiles * IMG_KV_BYTES);
        f_x = uniform_ptr(p.cmp.img_x + ((int64_t)b * p.cmp.Hfb + hfb) * p.cmp.img_tiles * IMG_X_BYTES);
        return true;
    };
    // this wave's piece i (0 .. 4) of the tile at the cursor: pieces wave + 8 i of the 40.  The fifth piece is K | V^T
    // for waves 0 .. 2, a piece of the side rows for the others (waves 5 .. 7 repeat the second one) -- chosen by
    // selects, not by a branch: a branch between the MFMAs of a step splits the step into blocks, and the compiler then
    // moves the softmax instructions out of the MFMA slots into the last block.
    const bool fifth_kv = wave < 3;
    const uint32_t fifth_src = fifth_kv ? (uint32_t)(wave + 32) * 1024u : (wave == 3 ? 0u : 1024u);
    const uint32_t fifth_dst = fifth_kv ? SM::OFF_KV + (uint32_t)(wave + 32) * 1024u : SM::OFF_X + (wave == 3 ? 0u : 1024u);
    const uint32_t fifth_slot_bytes = fifth_kv ? IMG_KV_BYTES : IMG_X_BYTES;
    auto fetch_piece = [&](int i) {
        const uint32_t slot = f_pos & (ST_SLOTS - 1);
        if (i < 4) {
            const int n = wave + 8 * i;
            dma16(f_kv + n * 1024, lds0 + SM::OFF_KV + slot * IMG_KV_BYTES + n * 1024);
        } else {
            const gptr_t src = fifth_kv ? f_kv : f_x;
            dma16(src + fifth_src, lds0 + fifth_dst + slot * fifth_slot_bytes);
        }
    };
    auto fetch_advance = [&]() {
        f_pos++;
        if (f_tile + 1 < f_nt) {
            f_tile++;
            f_kv += IMG_KV_BYTES;
            f_x += IMG_X_BYTES;
        } else {
            fetch_enter_next_item();  // (no further item: the cursor stays on the last tile)
        }
    };
    // A wave waits for its own pieces of the tile TWO ahead -- all it has requested so far -- then the barrier publishes
    // everybody's.  (One tile more than the step behind the barrier needs: that step's first fragments are read in front
    // of the barrier, from a tile that the barrier before has published.)
    auto publish = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };

    FDMA_STAMP(1);
    const bool any_tiles = fetch_enter_next_item();  // (the same for every wave)
    if (any_tiles) {
#pragma unroll 1
        for (int t = 0; t < 3; t++) {
#pragma unroll
            for (int i = 0; i < ST_NDMA; i++) fetch_piece(i);
            fetch_advance();
        }
        // tiles 0 and 1 have landed for this wave; the barrier shows them to the others
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(ST_NDMA) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }

    FDMA_STAMP(2);
    // ---- the tile program (see fdma_fwd_colmask.hip for the reasoning behind its shape)
    const int a_row = pi_row(r);
    const uint32_t aK = lds0 + SM::OFF_KV + (uint32_t)((a_row * SK + g * 8) * 2);
    const uint32_t aV = lds0 + SM::OFF_KV + IMG_K_BYTES + (uint32_t)((a_row * SVT + 8 * g) * 2);
    const uint32_t aX = lds0 + SM::OFF_X + (uint32_t)(a_row * 32 + g * 16);
    constexpr int NQK = KS + 1, NPV = 2 * DB;
    constexpr int FR = 4;  // fragment reads run FR MFMAs ahead of their MFMAs (6 and 8: the same time, more registers)
    const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const float side_mult = 1.f / E::kPieceScale;

    f32x16_t o[DB];
    float row_sum, row_ref, enc_ref;
    u32x4_t qx;
    int vis_wave = 0;

    // rows of the previous item on their way out (see pack_rows)
    u32x4_t po[2 * DB];
    uint16_t *st_ptr = nullptr;
    uint64_t st_mask = 0;
    auto store_piece = [&](int k) {  // piece k: columns 32 (k / 2) + 16 (k % 2) + 8 g .. + 7 of this lane's row
        uint64_t keep;
        asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %1\n\ts_cbranch_execz 1f\n\t"
                     "global_store_dwordx4 %2, %3, off offset:%4\n1:\n\ts_mov_b64 exec, %0"
                     : "=&s"(keep) : "s"(st_mask), "v"(st_ptr), "v"(po[k]), "n"(64 * (k / 2) + 32 * (k % 2)) : "memory");
    };

    auto causal_mask = [&](f32x16_t &s, int col0) {
        const int lim = vis_lane - 1 - col0 - 8 * g;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int lc = 16 * (i >> 3) + (i & 7);
            s[i] = lc <= lim ? s[i] : -INFINITY;
        }
    };
    // fragment address f of a step: side rows and K of half kh of ring slot ks, V^T of half vh of ring slot vs
    auto frag_addr = [&](int f, uint32_t kslot_kv, uint32_t kslot_x, uint32_t vslot_kv, int kh, int vh) -> uint32_t {
        if (f == 0) return aX + kslot_x + (uint32_t)(32 * kh * 32);
        if (f < NQK) return aK + kslot_kv + (uint32_t)((32 * kh * SK + (f - 1) * 16) * 2);
        const int kb = (f - NQK) / DB, db = (f - NQK) % DB;
        return aV + vslot_kv + (uint32_t)((32 * db * SVT + 32 * vh + 16 * kb) * 2);
    };
    auto scores_half = [&](f32x16_t &s, uint32_t pos, int kh) {
        const uint32_t kv = (pos & (ST_SLOTS - 1)) * IMG_KV_BYTES, x = (pos & (ST_SLOTS - 1)) * IMG_X_BYTES;
        u32x4_t a[NQK];
#pragma unroll
        for (int f = 0; f < NQK; f++) a[f] = lds_ld128(frag_addr(f, kv, x, 0, kh, 0));
        s = E::mfma(a[0], qx, zero16);
#pragma unroll
        for (int f = 1; f < NQK; f++) s = E::mfma(a[f], qf[f - 1], s);
    };
    auto pv_half = [&](const uint32_t (&pk)[8], uint32_t pos, int vh) {
        const uint32_t kv = (pos & (ST_SLOTS - 1)) * IMG_KV_BYTES;
        u32x4_t a[NPV];
#pragma unroll
        for (int f = 0; f < NPV; f++) a[f] = lds_ld128(frag_addr(NQK + f, 0, 0, kv, 0, vh));
#pragma unroll
        for (int f = 0; f < NPV; f++) {
            const int kb = f / DB, db = f % DB;
            const u32x4_t bop = {pk[4 * kb], pk[4 * kb + 1], pk[4 * kb + 2], pk[4 * kb + 3]};
            o[db] = E::mfma(a[f], bop, o[db]);
        }
    };

    // One step of the pipeline.  MFMAs: (SCORES) the scores of the NEXT half tile -- half kh of the tile at stream
    // position kpos -- into `snext`, and O^T += V^T P^T of the PREVIOUS half tile (probabilities pprev, half vh of the
    // tile at vpos).  Vector ALU, between them: softmax of the CURRENT half tile `scur` into `pcur`, the common path.
    // (FETCH) this wave's five pieces of the tile at the fetch cursor are requested between the first MFMAs.  Written slot
    // by slot -- one MFMA, the fragment read of the MFMA FR slots later, an even share of the vector work -- with a
    // scheduling barrier after every slot.  Returns the sum of the half tile's probabilities.
    // The step in front of the barrier (PRE_OUT) reads, in its last slots, the first FR fragments of the step behind the
    // barrier into `pre` (PRE_IN takes them from there): the tile they come from was published a barrier earlier, so the
    // first MFMAs behind a barrier do not wait for LDS with every wave of the workgroup at the same point.
    auto step = [&](auto scores_c, auto fetch_c, auto next_scores_c, f32x16_t &scur, f32x16_t &snext, uint32_t (&pcur)[8],
                    const uint32_t (&pprev)[8], uint32_t kpos, auto kh_c, uint32_t vpos, auto vh_c, int rd, u32x4_t (&pre)[FR]) {
        constexpr bool SCORES = decltype(scores_c)::value, FETCH = decltype(fetch_c)::value;
        constexpr bool PRE_IN = FETCH, PRE_OUT = !FETCH, NEXT_SCORES = decltype(next_scores_c)::value;
        constexpr int kh = decltype(kh_c)::value, vh = decltype(vh_c)::value;
        constexpr int F0 = SCORES ? 0 : NQK, NF = NQK + NPV - F0;  // fragments F0 .. NQK + NPV - 1
        const uint32_t kv = (kpos & (ST_SLOTS - 1)) * IMG_KV_BYTES, kx = (kpos & (ST_SLOTS - 1)) * IMG_X_BYTES;
        const uint32_t vv = (vpos & (ST_SLOTS - 1)) * IMG_KV_BYTES;
        // the step behind the barrier (PRE_OUT): scores of half 0 of tile kpos + 1 (NEXT_SCORES), P V of half 0 of tile kpos
        const uint32_t nkv = ((kpos + 1) & (ST_SLOTS - 1)) * IMG_KV_BYTES, nkx = ((kpos + 1) & (ST_SLOTS - 1)) * IMG_X_BYTES;
        constexpr int NF0 = NEXT_SCORES ? 0 : NQK;
        u32x4_t a[NF];
#pragma unroll
        for (int f = 0; f < FR; f++) a[f] = PRE_IN ? pre[f] : lds_ld128(frag_addr(F0 + f, kv, kx, vv, kh, vh));
        float psum0 = 0.f, psum1 = 0.f, x0[8], x1[8];
#pragma unroll
        for (int f = 0; f < NF; f++) {
            if (f + FR < NF) a[f + FR] = lds_ld128(frag_addr(F0 + f + FR, kv, kx, vv, kh, vh));
            else if (PRE_OUT) pre[f + FR - NF] = lds_ld128(frag_addr(NF0 + f + FR - NF, nkv, nkx, kv, 0, 0));
            const int ff = F0 + f;
            if (ff == 0) {
                snext = E::mfma(a[f], qx, zero16);
            } else if (ff < NQK) {
                snext = E::mfma(a[f], qf[ff - 1], snext);
            } else {
                const int kb = (ff - NQK) / DB, db = (ff - NQK) % DB;
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
            if (FETCH) {
#pragma unroll
                for (int i = 0; i < ST_NDMA; i++)
                    if (f == (SCORES ? 1 + 3 * i : 1 + i)) fetch_piece(i);
            }
            if (FETCH) {  // the previous item's output rows, one piece per slot (a step behind the barrier: see store_piece)
#pragma unroll
                for (int k = 0; k < 8; k++)
                    if (f == (SCORES ? 2 + 3 * (k / 2) + (k & 1) : k)) store_piece(k);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (FETCH) st_mask = 0;
        const float psum = psum0 + psum1;
        row_sum += psum;
#pragma unroll
        for (int i = 0; i < 8; i++) asm volatile("" : "+v"(pcur[i]));
        asm volatile("" : "+v"(row_sum));
        __builtin_amdgcn_sched_barrier(0);
        if (FETCH) fetch_advance();
        // a probability beyond 2^14 (the sum shows it): the item leaves the common path and is redone at the end
        if (__any(!(psum <= 16384.f)) && lane == 0) atomicOr(&sRedo[rd >> 5], 1u << (rd & 31));
    };

    // Output rows of an item.  pack_rows() turns the accumulators into 16-bit rows (O / sum) held in `po`, writes the
    // LSE and notes which lanes have a row to store (st_mask); the stores themselves -- eight of 16 bytes per lane -- are
    // issued one per slot by the NEXT item's first step behind a barrier (store_piece), where they travel under matrix
    // work: issued in one go they fill the CU's store path for more than a microsecond per item with every wave waiting,
    // and issued in front of a barrier they would be waited for there (publish() waits for everything in flight).
    // A store is written in assembly: lanes without a row are switched off through exec (restored at once), and when no
    // store is pending (st_mask == 0: every step but the first of an item) the instruction is jumped over.
    auto write_rows = [&](const Item &it) {  // at once (items without tiles, the redo pass)
        const int b = it.pair / p.Hk;
        const int qrow = it.m0 + wave * 32 + opaque(r);
        const float total = xhalf_sum(row_sum);
        const float inv = total > 0.f ? 1.f / total : 0.f;
        if (qrow < Lq) {
            uint16_t *op = (uint16_t *)p.o + b * p.o_b + (int64_t)qrow * p.o_r + it.h * p.o_h;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int blk = 0; blk < 2; blk++) {
                    const int c = 32 * db + 16 * blk + 8 * g;
                    u32x4_t w;
#pragma unroll
                    for (int e = 0; e < 4; e++) w[e] = E::pack2(o[db][8 * blk + 2 * e] * inv, o[db][8 * blk + 2 * e + 1] * inv);
                    *(u32x4_t *)(op + c) = w;
                }
            if (g == 0) {
                const float lse = total > 0.f ? (row_ref + __builtin_amdgcn_logf(total)) * kLn2 : INFINITY;
                p.lse[b * p.lse_b + it.h * p.lse_h + qrow] = lse;
            }
        }
    };
    auto pack_rows = [&](const Item &it) {
        const int b = it.pair / p.Hk;
        const int qrow = it.m0 + wave * 32 + opaque(r);
        const float total = xhalf_sum(row_sum);
        const float inv = total > 0.f ? 1.f / total : 0.f;
        const bool valid = qrow < Lq;
        st_ptr = (uint16_t *)p.o + b * p.o_b + (int64_t)(valid ? qrow : 0) * p.o_r + it.h * p.o_h + 8 * g;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    po[2 * db + blk][e] = E::pack2(o[db][8 * blk + 2 * e] * inv, o[db][8 * blk + 2 * e + 1] * inv);
        st_mask = __ballot(valid);
        if (valid && g == 0) {
            const float lse = total > 0.f ? (row_ref + __builtin_amdgcn_logf(total)) * kLn2 : INFINITY;
            p.lse[b * p.lse_b + it.h * p.lse_h + qrow] = lse;
        }
    };
    auto flush_rows = [&]() {  // whatever is pending, at once
#pragma unroll
        for (int k = 0; k < 8; k++) store_piece(k);
        st_mask = 0;
    };
    auto reset_rows = [&]() {
        row_sum = 0.f;
        row_ref = -INFINITY;
        enc_ref = 0.f;
        qx[0] = g == 0 ? E::pack2(side_mult, side_mult) : 0u;
        qx[1] = g == 0 ? E::pack2(side_mult, 1.f) : 0u;
        qx[2] = 0u;
        qx[3] = 0u;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    };

    const std::true_type yes;
    const std::false_type no;
    const std::integral_constant<int, 0> c0;
    const std::integral_constant<int, 1> c1;

    uint32_t pos = 0;  // stream position of the tile being worked on
    while (rd < rounds) {
        const int nt = __builtin_amdgcn_readfirstlane((int)sNt[rd]);
        // the next round with an item (past the last one: this item again, whose Q is then fetched once more and dropped --
        // an unconditional fetch keeps the Q registers one live range across the item boundary)
        int rd_next = rd + 1;
        Item nxt;
        while (rd_next < rounds && !item_of(rd_next, nxt)) rd_next++;
        if (rd_next >= rounds) nxt = cur;
        reset_rows();
        FDMA_STAMP(4 + 4 * rd);
        if (nt > 0) {
            if (CAUSAL) vis_wave = __builtin_amdgcn_readfirstlane(vis_lane);  // (lane 0 holds the wave's first row)
            FDMA_STAMP(5 + 4 * rd);
#ifdef FDMA_DBG
            if (tid == 0 && rd < 4) g_stream_dbg[blockIdx.x * 64 + 56 + rd] = __builtin_amdgcn_s_memtime();
#endif
            // ---- set-up: the scores of the first half tile against the reference point 0; the reference of every row is
            // put a margin above their maximum (any number near the row's maximum will do: probabilities then start around
            // 2^-margin, and the rest of the row may exceed this half tile by margin + 14 before the item is redone) and
            // taken off the scores just made.  (Key 0 of the compacted axis is in this half tile: a row that sees nothing
            // here sees nothing at all.)
            f32x16_t sA, sB;
            uint32_t pA[8], pB[8];
            {
                scores_half(sA, pos, 0);
                if (CAUSAL && 32 > vis_wave) causal_mask(sA, 0);
                float tmax = -INFINITY;
#pragma unroll
                for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, sA[i]);
                tmax = xhalf_max(tmax);
                bool bad = false;
                if (tmax > -INFINITY) {
                    const float want = tmax + (std::is_same<T, bf16_tag>::value ? 8.f : 4.f);
                    float enc;
                    const uint32_t w = encode_ref<T>(want, enc);
                    bad = !(fabsf(enc - want) <= 0.5f);  // the pieces cannot express it: redo
                    enc_ref = row_ref = enc;
                    if (g == 0) qx[2] = w;
                }
                if (__any(bad) && lane == 0) atomicOr(&sRedo[rd >> 5], 1u << (rd & 31));
#pragma unroll
                for (int i = 0; i < 16; i++) sA[i] -= enc_ref;
            }
#pragma unroll
            for (int i = 0; i < 8; i++) pB[i] = 0u;
            // ---- tiles.  Iteration t: step A (scores of half 2t+1, softmax of half 2t, P V of half 2t-1), the barrier that
            // publishes the tile after this one, step B (scores of half 2t+2 from that tile, softmax of half 2t+1, P V of
            // half 2t, and the requests for the tile three ahead).  The last tile's step B has no scores to compute:
            // it requests the next item's Q instead.
            int col0 = 0;
            u32x4_t pre[FR];
#pragma unroll 1
            for (int t = 0; t + 1 < nt; t++, col0 += BN) {
                if (CAUSAL && col0 + 32 > vis_wave) causal_mask(sA, col0);
                __builtin_amdgcn_sched_barrier(0);
                step(yes, no, yes, sA, sB, pA, pB, pos, c1, pos - 1, c1, rd, pre);
                publish();
                if (CAUSAL && col0 + 64 > vis_wave) causal_mask(sB, col0 + 32);
                step(yes, yes, no, sB, sA, pB, pA, pos + 1, c0, pos, c0, rd, pre);
                __builtin_amdgcn_sched_barrier(0);
                pos++;
            }
            {   // the last tile
                if (CAUSAL && col0 + 32 > vis_wave) causal_mask(sA, col0);
                __builtin_amdgcn_sched_barrier(0);
                step(yes, no, no, sA, sB, pA, pB, pos, c1, pos - 1, c1, rd, pre);
                publish();
                if (CAUSAL && col0 + 64 > vis_wave) causal_mask(sB, col0 + 32);
                __builtin_amdgcn_sched_barrier(0);
                // (qf is free from here on; with the loads in front of the step they travel under it)
                load_q(nxt);
                __builtin_amdgcn_sched_barrier(0);
                step(no, yes, no, sB, sA, pB, pA, pos + 1, c0, pos, c0, rd, pre);
                __builtin_amdgcn_sched_barrier(0);
                pv_half(pB, pos, 1);  // P V of the last half: V of the last tile, second half
                pos++;
            }
            FDMA_STAMP(6 + 4 * rd);
#ifdef FDMA_DBG
            if (tid == 0 && rd < 4) g_stream_dbg[blockIdx.x * 64 + 60 + rd] = __builtin_amdgcn_s_memtime();
#endif
            pack_rows(cur);
            FDMA_STAMP(7 + 4 * rd);
        } else {
            flush_rows();
            write_rows(cur);  // no visible key: zeros and LSE = +inf
            load_q(nxt);
        }
        cur = nxt;
        rd = rd_next;
    }

    flush_rows();  // the last item's rows
    // ---- drain: nothing of this workgroup's may land in the LDS of the next one
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    FDMA_STAMP(3);
#ifdef FDMA_DBG
    if (tid == 0) g_stream_dbg[blockIdx.x * 64 + 39] = __builtin_amdgcn_s_memtime();
#endif

    // ---- redo: items that left the common path, tile by tile with the classic softmax (maximum per half tile, reference
    // moved and O rescaled as needed), fragments straight from the images in global memory.  Not for speed.
    for (int w = 0; w < (rounds + 31) / 32; w++) {
        uint32_t bits = __builtin_amdgcn_readfirstlane(sRedo[w]);
        while (bits) {
            const int rdo = w * 32 + __builtin_ctz(bits);
            bits &= bits - 1;
            Item it;
            if (!item_of(rdo, it)) continue;
            const int nt = sNt[rdo];
            const int b = it.pair / p.Hk;
            const int hfb = p.cmp.Hfb == p.H ? it.h : it.pair % p.Hk;
            const char *kvimg = p.cmp.img_kv + (int64_t)it.pair * p.cmp.img_tiles * IMG_KV_BYTES;
            const char *ximg = p.cmp.img_x + ((int64_t)b * p.cmp.Hfb + hfb) * p.cmp.img_tiles * IMG_X_BYTES;
            load_q(it);
            reset_rows();
            if (CAUSAL) vis_wave = __builtin_amdgcn_readfirstlane(vis_lane);
            const uint32_t oK = (uint32_t)((a_row * SK + g * 8) * 2), oV = IMG_K_BYTES + (uint32_t)((a_row * SVT + 8 * g) * 2);
            const uint32_t oX = (uint32_t)(a_row * 32 + g * 16);
            for (int t = 0; t < nt; t++) {
                const char *kvt = kvimg + (int64_t)t * IMG_KV_BYTES, *xt = ximg + (int64_t)t * IMG_X_BYTES;
#pragma unroll 1
                for (int half = 0; half < 2; half++) {
                    f32x16_t s = E::mfma(*(const u32x4_t *)(xt + oX + 32 * half * 32), qx, zero16);
#pragma unroll
                    for (int ks = 0; ks < KS; ks++)
                        s = E::mfma(*(const u32x4_t *)(kvt + oK + (32 * half * SK + ks * 16) * 2), qf[ks], s);
                    const int col0 = t * BN + 32 * half;
                    if (CAUSAL && col0 + 32 > vis_wave) causal_mask(s, col0);
                    // classic softmax of the half tile; the scores are relative to enc_ref as it was when they were made
                    float tmax = -INFINITY;
#pragma unroll
                    for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[i]);
                    tmax = xhalf_max(tmax);
                    const bool unset = row_ref == -INFINITY;
                    const float cand = enc_ref + tmax;
                    const bool move = unset ? tmax > -INFINITY : cand > row_ref + 8.f;
                    float shift_s = unset ? 0.f : enc_ref - row_ref;
                    if (__any(move)) {
                        float enc;
                        const uint32_t wq = encode_ref<T>(cand, enc);
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
                            if (g == 0) qx[2] = wq;
                        }
                        row_ref = new_ref;
                    }
                    uint32_t pk[8];
                    float psum = 0.f;
#pragma unroll
                    for (int i = 0; i < 16; i += 2) {
                        const float e0 = fast_exp2(s[i] + shift_s), e1 = fast_exp2(s[i + 1] + shift_s);
                        psum += e0 + e1;
                        pk[i / 2] = E::pack2(e0, e1);
                    }
                    row_sum += psum;
#pragma unroll
                    for (int f = 0; f < NPV; f++) {
                        const int kb = f / DB, db = f % DB;
                        const u32x4_t av = *(const u32x4_t *)(kvt + oV + (32 * db * SVT + 32 * half + 16 * kb) * 2);
                        const u32x4_t bop = {pk[4 * kb], pk[4 * kb + 1], pk[4 * kb + 2], pk[4 * kb + 3]};
                        o[db] = E::mfma(av, bop, o[db]);
                    }
                }
            }
            write_rows(it);
        }
    }
}

template <typename T, bool CAUSAL>
hipError_t launch_stream(const FwdParams &p, hipStream_t stream) {
    auto kern = fwd_stream_kernel<T, CAUSAL>;
    static DynSmemLimit smem_limit;
    hipError_t e = smem_limit.ensure((const void *)kern, StSmem::TOTAL);
    if (e != hipSuccess) return e;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
        static std::atomic<int> cached[16];
        int n = dev >= 0 && dev < 16 ? cached[dev].load(std::memory_order_relaxed) : 0;
        if (n == 0) {
            if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
            if (dev >= 0 && dev < 16) cached[dev].store(n, std::memory_order_relaxed);
        }
        cus = n;
    }
    const int n_mb = (p.Lq + ST_BM - 1) / ST_BM, G = p.H / p.Hk, pairs = p.B * p.Hk;
    const int gcd8 = (pairs % 8 == 0) ? 8 : ((pairs % 4 == 0) ? 4 : ((pairs % 2 == 0) ? 2 : 1));
    const int k_split = 8 / gcd8;
    const int64_t items = (int64_t)pairs * k_split * ((n_mb + k_split - 1) / k_split) * G;
    const int items_per_xcd = (int)(items / 8);
    int wgs_per_xcd = cus / 8 > 0 ? cus / 8 : 1;
    if (wgs_per_xcd > items_per_xcd) wgs_per_xcd = items_per_xcd;
    const int rounds = (items_per_xcd + wgs_per_xcd - 1) / wgs_per_xcd;
    if (rounds > ST_MAX_ROUNDS || items > 0x7fffffff) return hipErrorInvalidValue;  // (fwd_stream_applicable keeps such problems away)
    hipLaunchKernelGGL(kern, dim3(8 * wgs_per_xcd), dim3(ST_THREADS), StSmem::TOTAL, stream, p, items_per_xcd, wgs_per_xcd, rounds);
    return hipGetLastError();
}

}  // namespace

// The streaming forward takes compacted problems at head dim 128 whose grid fills the device several times over
// (what the 256-row workgroups of the column-mask forward ask for as well), with a key axis the one-launch image
// pre-pass can count (65536 keys) and few enough items per workgroup for its LDS tables.  Decided from the problem
// alone: the pre-pass, the forward and the backward of a problem have to agree on the workspace layout.
static std::atomic<int> g_stream_min_items{512};

void set_stream_min_items(int n) { g_stream_min_items.store(n < 1 ? 1 : n, std::memory_order_relaxed); }
int get_stream_min_items() { return g_stream_min_items.load(std::memory_order_relaxed); }

bool fwd_stream_applicable(const FwdParams &p) {
    if (p.d != ST_D || p.cu_q != nullptr || p.Lk < 1 || p.Lk > (1 << 16) || p.Lq < 2) return false;
    const int64_t items = (int64_t)p.B * p.H * ((p.Lq + ST_BM - 1) / ST_BM);
    if (items < get_stream_min_items()) return false;
    // (rounds = items of an XCD over its workgroups; 16 workgroups per XCD is the fewest a device here has)
    return 2 * items / (8 * 16) <= ST_MAX_ROUNDS;
}

#ifdef FDMA_DBG
extern "C" int fdma_dbg_read_stream(uint64_t *host) {
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_stream_dbg), sizeof(uint64_t) * 1024 * 64);
}
#endif

hipError_t launch_fwd_stream(const FwdParams &p, int dtype, hipStream_t stream) {
    if (dtype == 0) return p.causal ? launch_stream<bf16_tag, true>(p, stream) : launch_stream<bf16_tag, false>(p, stream);
    return p.causal ? launch_stream<fp16_tag, true>(p, stream) : launch_stream<fp16_tag, false>(p, stream);
}

}  // namespace fdma
