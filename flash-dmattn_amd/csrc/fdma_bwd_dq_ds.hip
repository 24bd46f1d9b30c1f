// dQ from the dS that the dK/dV kernel has just written out as dBias, for gfx950.
//
// Same place in the reference's backward as bwd_dq_kernel (fdma_bwd_dq.hip): the dQ part of
// flash_bwd_dq_dk_dv_loop_seqk_parallel_kernel (csrc/flash_sparse_attn/src/flash_bwd_kernel.h:79-1142), whose dQ is
// dS K with dS rounded to the input type (its tdSrdS fragments feed both the dQ and the dK MMAs).
//
// When the bias differs per query AND per query head (or there is one query head per bias head), the gradient of the
// bias IS dS: the dK/dV kernel computes it anyway and writes it, rounded to 16 bits, at the bias's own shape -- zeros
// where the mask drops a key, above the causal diagonal and for keys beyond Lk.  dQ = scale * dS K then needs neither
// Q, V, dO, the row statistics, the mask nor the bias a second time: this kernel streams the dS tiles of its 128 query
// rows (eight lanes per 128-byte row piece, whole lines per load instruction; then through LDS into the B operand of
// the MFMA, where a lane owns a query row and eight consecutive keys of it -- fetched in that layout directly, every
// line is asked for in four pieces of 32 bytes by four instructions, and the launch moved 2.7 TB/s) against K tiles in
// LDS (K^T through transposing reads of the row-major rows, as the decode kernel reads V^T).  One tile GEMM instead of
// three, two thirds of the bytes (no mask), no softmax, and the loads of three tiles in flight: a stream, where
// bwd_dq_kernel holds a trip to memory in every iteration.
#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

namespace {

constexpr int DS_THREADS = 256, DS_BM = 128, DS_BN = 64;
constexpr int DS_PF = 4;  // dS tiles in flight

template <int D> struct DqdsSmem {
    static constexpr int S = D + 8;      // K tile row stride (elements): 16 bytes of padding
    static constexpr int SD = DS_BN + 8; // dS tile row stride
    static constexpr int TILE_BYTES = DS_BN * S * 2;
    static constexpr int DS_BYTES = DS_BM * SD * 2;
    static constexpr int STAGE = TILE_BYTES + DS_BYTES;
    static constexpr int TOTAL = 2 * STAGE;
};

template <typename T, int D, bool CAUSAL>
__global__ void __launch_bounds__(DS_THREADS) bwd_dq_ds_kernel(const BwdParams p) {
    using E = Elem<T>;
    using SM = DqdsSmem<D>;
    constexpr int BN = DS_BN, BM = DS_BM;
    constexpr int DB = D / 32, KB = BN / 16;
    constexpr int CH = D / 8, K_RPP = DS_THREADS / CH, K_IT = BN / K_RPP;
    static_assert(K_IT >= 1 && K_IT * K_RPP == BN, "a K tile is a whole number of passes of the workgroup");
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const FwdParams &f = p.f;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 31, g = lane >> 5;
    // query block outermost and descending: under causal masking the blocks with the most tiles start first
    const int hb_count = f.H * f.B;
    const int m_block = (int)gridDim.x / hb_count - 1 - (int)blockIdx.x / hb_count;
    const int h = ((int)blockIdx.x % hb_count) % f.H, b = ((int)blockIdx.x % hb_count) / f.H;
    const int hk = h / (f.H / f.Hk);
    const int m0 = m_block * BM;
    const int qrow = m0 + wave * 32 + r;
    const int shift = f.Lk - f.Lq;

    int n_end = (f.Lk + BN - 1) / BN;
    if (CAUSAL) {
        int lim = m0 + BM + shift;  // first invisible column for the last row of the block
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

    const int hb = f.Hb == f.H ? h : (f.Hb == 1 ? 0 : hk);
    const uint16_t *dsbase = (const uint16_t *)p.dbias + b * p.db_b + hb * p.db_h;
    const uint16_t *kbase = (const uint16_t *)f.k + b * f.k_b + hk * f.k_h;

    // K staging: d chunk and first row of this thread; chunks beyond d re-read chunk 0 (the dQ columns they feed are
    // not stored)
    const int kc = tid % CH, kr0 = tid / CH;
    const int kcol = kc * 8 < f.d ? kc * 8 : 0;
    auto load_k = [&](int j, u32x4_t (&dst)[K_IT]) {
#pragma unroll
        for (int it = 0; it < K_IT; it++) {
            int key = j * BN + kr0 + it * K_RPP;
            key = key < f.Lk ? key : f.Lk - 1;  // (rows beyond Lk meet dS = 0)
            dst[it] = *(const u32x4_t *)(kbase + (int64_t)key * f.k_r + kcol);
        }
    };
    // dS staging: 8-key chunk and first row of this thread (rows fr0 + 32 it); eight lanes fetch the 128 bytes of a row
    constexpr int F_IT = BM * (BN / 8) / DS_THREADS;  // 4
    const int fc = tid & 7, fr0 = tid >> 3;
    // A chunk that starts beyond Lk is fetched from the row's start and cleared, one that straddles Lk keeps its keys
    // below Lk (what lies behind them in the row is not the kernel's to read as numbers); rows beyond Lq repeat the last
    // row (their dQ is not stored).
    auto load_ds = [&](int j, u32x4_t (&dst)[F_IT]) {
        const int kk = j * BN + 8 * fc;
#pragma unroll
        for (int it = 0; it < F_IT; it++) {
            int row = m0 + fr0 + 32 * it;
            row = row < f.Lq ? row : f.Lq - 1;
            dst[it] = *(const u32x4_t *)(dsbase + (int64_t)row * p.db_r + (kk < f.Lk ? kk : 0));
        }
    };
    auto store_stage = [&](int pos, int j, const u32x4_t (&src)[F_IT], const u32x4_t (&ksrc)[K_IT]) {  // tile j to stage pos & 1
        char *sK = smem + (pos & 1) * SM::STAGE;
        char *sD = sK + SM::TILE_BYTES;
#pragma unroll
        for (int it = 0; it < K_IT; it++) *(u32x4_t *)(sK + ((kr0 + it * K_RPP) * SM::S + kc * 8) * 2) = ksrc[it];
        const int left = f.Lk - (j * BN + 8 * fc);  // keys of this thread's chunk below Lk
#pragma unroll
        for (int it = 0; it < F_IT; it++) {
            u32x4_t v = src[it];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] &= left >= 2 * e + 2 ? 0xffffffffu : (left == 2 * e + 1 ? 0x0000ffffu : 0u);
            *(u32x4_t *)(sD + ((fr0 + 32 * it) * SM::SD + 8 * fc) * 2) = v;
        }
    };

    // transposing reads of the row-major K rows (see fdma_common.h): A operand = K^T, 32 head-dim rows x 16 keys
    const int tj = lane & 15, te = tj >> 2, tc = tj & 3;
    const int tcp = (tc == 1) ? 2 : (tc == 2 ? 1 : tc);
    const int tdh = (lane >> 4) & 1;
    const uint32_t tr_off = (uint32_t)(((8 * g + te) * SM::S + 16 * tdh + 4 * tcp) * 2);
    // B operand = dS^T: keys 16 kb + 8 g .. + 7 of this lane's query row
    const uint32_t b_off = (uint32_t)(SM::TILE_BYTES + ((wave * 32 + r) * SM::SD + 8 * g) * 2);

    // Tile j is computed from LDS stage j & 1; the dS of tiles j + 1 .. j + 4 sit in four register sets and K of
    // tiles j + 1, j + 2 in two, and the sets change roles from one iteration to the next (the loop is written out four
    // iterations at a time: a move between sets would have to wait for a load still in flight).  With K a single
    // iteration ahead every iteration held a trip to the L2.  Every load is unconditional, from a clamped tile number:
    // behind a condition the compiler has to assume that the younger loads may not have been issued, and waits for ALL
    // of them where it only needs the oldest -- the stream would be one tile deep again.  For the same reason the loop
    // always runs whole groups of iterations; one past the last tile is skipped by the matrix work alone.
    // The tiles are walked from a starting tile that differs from workgroup to workgroup, round to the front again: dQ
    // is a plain sum over the tiles, and workgroups that all begin at key 0 and move along rows of the same power-of-two
    // pitch ask the same few memory channels for their data at the same time.
    static_assert(DS_PF == 4, "the loop below is written out for four sets");
    if (n_end > 0) {
        const int last = n_end - 1;
        const int start = (int)(((uint32_t)blockIdx.x * 2654435761u) >> 8) % n_end;
        auto tile = [&](int i) -> int {  // tile of loop position i (positions beyond the last repeat the last)
            i = i < last ? i : last;
            return i + start < n_end ? i + start : i + start - n_end;
        };
        u32x4_t dsA[F_IT], dsB[F_IT], dsC[F_IT], dsD[F_IT], kA[K_IT], kB[K_IT];
        load_k(tile(0), kA);
        load_ds(tile(0), dsA);
        load_ds(tile(1), dsB);
        load_ds(tile(2), dsC);
        load_ds(tile(3), dsD);
        store_stage(0, tile(0), dsA, kA);
        load_k(tile(1), kA);
        load_k(tile(2), kB);
        load_ds(tile(4), dsA);
        __syncthreads();
        // iteration j: `nxt` / `knxt` hold tile j + 1 (the oldest requests in flight) and receive tiles j + 5 / j + 3
        auto iteration = [&](int j, u32x4_t (&nxt)[F_IT], u32x4_t (&knxt)[K_IT]) {
            const char *st = smem + (j & 1) * SM::STAGE;
            if (j < n_end) {
#pragma unroll
                for (int kb = 0; kb < KB; kb++) {
                    const u32x4_t bop = *(const u32x4_t *)(st + b_off + 16 * kb * 2);
#pragma unroll
                    for (int db = 0; db < DB; db++) {
                        const uint32_t off = tr_off + (uint32_t)((16 * kb * SM::S + 32 * db) * 2);
                        const u32x2_t lo_ = lds_read_tr16(st, off), hi_ = lds_read_tr16(st, off + 4 * SM::S * 2);
                        const u32x4_t a = {lo_[0], lo_[1], hi_[0], hi_[1]};
                        dq[db] = E::mfma(a, bop, dq[db]);
                    }
                }
            }
            // tile j + 1 to the other stage (requested two iterations ago and more: what is younger stays in flight,
            // loads come back in the order they were issued), then the next requests
            store_stage(j + 1, tile(j + 1), nxt, knxt);
            load_k(tile(j + 3), knxt);
            __builtin_amdgcn_sched_barrier(0);
            load_ds(tile(j + DS_PF + 1), nxt);
            __syncthreads();
        };
#pragma unroll 1
        for (int j = 0; j < n_end; j += 4) {
            iteration(j, dsB, kA);
            iteration(j + 1, dsC, kB);
            iteration(j + 2, dsD, kA);
            iteration(j + 3, dsA, kB);
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
                    for (int e = 0; e < 4; e++) w[e] = E::pack2(dq[db][8 * blk + 2 * e] * f.scale, dq[db][8 * blk + 2 * e + 1] * f.scale);
                    *(u32x4_t *)(dqp + c) = w;
                }
            }
    }
}

template <typename T, int D>
hipError_t launch_dq_ds(const BwdParams &p, hipStream_t stream) {
    const FwdParams &f = p.f;
    const dim3 grid(((f.Lq + DS_BM - 1) / DS_BM) * f.H * f.B);
    auto kern = f.causal ? bwd_dq_ds_kernel<T, D, true> : bwd_dq_ds_kernel<T, D, false>;
    static DynSmemLimit smem_limit[2];  // one per instantiation: the limit is a property of the kernel
    const hipError_t e = smem_limit[f.causal ? 1 : 0].ensure((const void *)kern, DqdsSmem<D>::TOTAL);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, dim3(DS_THREADS), DqdsSmem<D>::TOTAL, stream, p);
    return hipGetLastError();
}

}  // namespace

bool bwd_dq_from_ds_applicable(const BwdParams &p) {
    const FwdParams &f = p.f;
    if (!f.bias || f.bi_r == 0 || !p.dbias || p.db_r == 0 || p.dbias_accum) return false;  // a per-query dBias, written directly
    if (f.cu_q || f.Lk < 1 || f.Lq < 1) return false;
    // ... that is dS itself: a bias row per query head and per batch entry (nothing summed into it)
    return f.Hb == f.H && (f.B == 1 || (f.bi_b != 0 && p.db_b != 0));
}

hipError_t launch_bwd_dq_from_ds(const BwdParams &p, int dtype, hipStream_t stream) {
    const int d = p.f.d;
    if (dtype == 0) return d <= 64 ? launch_dq_ds<bf16_tag, 64>(p, stream) : d <= 128 ? launch_dq_ds<bf16_tag, 128>(p, stream) : launch_dq_ds<bf16_tag, 256>(p, stream);
    return d <= 64 ? launch_dq_ds<fp16_tag, 64>(p, stream) : d <= 128 ? launch_dq_ds<fp16_tag, 128>(p, stream) : launch_dq_ds<fp16_tag, 256>(p, stream);
}

}  // namespace fdma
