// Single-token decode (seqlen_q == 1) for gfx950: split-KV partial attention + LSE-weighted combine -- in ONE launch
// when the caller provides arrival counters (the last workgroup of a (batch entry, head chunk) to finish merges the
// splits), otherwise as a second launch.
//
// Replaces the reference's decode route: the `seqlenq_ngroups_swapped` reshaping of mha_fwd
// (csrc/flash_sparse_attn/flash_api.cpp:443-475, 541-551), num_splits_heuristic (:275-349),
// compute_attn_1rowblock_splitkv (csrc/flash_sparse_attn/src/flash_fwd_kernel.h:808-1587) and
// combine_attn_seqk_parallel (:1618-1813).
//
// The path is bound by HBM reads of K and V.  A key/value row of one KV head is d*2 contiguous bytes,
// so skipping can be done per KEY instead of per 64-key tile: each workgroup first compacts the
// keys of its range that any query head of the group keeps (ordered, by prefix sums), then gathers
// only those rows.  With a top-W mask that reads W rows instead of every 64-key tile that holds one.
// The query heads of a KV group are the 32 columns of an MFMA tile (unused columns carry zeros), so
// every gathered row is used by all of them: a wave stages 32 gathered K and V rows in its own
// piece of LDS (no barrier: nobody else reads it), S^T = K Q^T and O^T += V^T P^T run on the matrix
// pipe, and the vector ALU is left with one exp2 per (key, column).
#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

namespace {

constexpr int DEC_THREADS = 256;
constexpr int DEC_RANGE = 16 * DEC_THREADS;  // keys compacted per pass (16 per thread)
constexpr int DEC_NJ = 4;                    // sub-ranges per pass: the mask of 4 x 4096 keys is fetched in one go
constexpr int DEC_SUPER = DEC_NJ * DEC_RANGE;
static_assert(DEC_NJ == 4, "the list builder selects among four mask words");
constexpr int DEC_TILE = 32;                 // gathered keys per wave and step
constexpr int DEC_COLS = 32;                 // query heads per workgroup (columns of the MFMA tile)

template <int D> struct DecSmem {
    static constexpr int S = D + 8;  // row stride of a staged tile in elements (16 bytes of padding)
    static constexpr int TILE_BYTES = DEC_TILE * S * 2;
    static constexpr int WAVE_BYTES = 2 * TILE_BYTES + DEC_TILE * 4;  // K rows, V rows, fused bias
    static constexpr int OFF_IDX = 4 * WAVE_BYTES;
    static constexpr int TOTAL = OFF_IDX + DEC_RANGE * 2;
    static constexpr int SO = D + 4;  // row stride of a wave's partial output in floats (rows fall into different banks)
    static_assert(DEC_COLS * SO * 4 <= WAVE_BYTES, "a wave's partial output must fit its own piece");
};

// Inclusive prefix sum of x over the lanes of a wave, and the wave's total (uniform).  Four shifted adds inside
// each row of 16 lanes (data-parallel primitives: no LDS traffic), then the row totals through scalar registers.
__device__ __forceinline__ int wave_scan(int x, int lane, int &total) {
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);  // row_shr:1 (lanes without a source add 0)
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);  // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);  // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);  // row_shr:8
    const int t0 = __builtin_amdgcn_readlane(x, 15), t1 = __builtin_amdgcn_readlane(x, 31);
    const int t2 = __builtin_amdgcn_readlane(x, 47), t3 = __builtin_amdgcn_readlane(x, 63);
    const int row = lane >> 4;
    x += (row >= 1 ? t0 : 0) + (row >= 2 ? t1 : 0) + (row >= 3 ? t2 : 0);
    total = t0 + t1 + t2 + t3;
    return x;
}

// nonzero bytes of x -> bit k of the result is set iff byte k of x != 0
__device__ __forceinline__ uint32_t nz_bytes_to_bits(uint32_t x) {
    uint32_t y = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
    return ((y >> 7) * 0x10204080u) >> 28;
}

// PERHEAD: mask or bias differ between the query heads of a group, so a lane fetches the mask byte and the
// bias of its own (key, head) pairs; otherwise one fused value per key serves all columns.
// out[b,h,:] = sum_s exp(lse_s - lse) * o_s ;  lse = logsumexp_s lse_s  (empty everywhere: 0 / +inf) for one (b, h) row,
// by ONE wave: lane s (and s + 64) fetches lse_s, the weights are made once and left in the wave's own piece of LDS
// (`s_w`, room for 128 floats), then lane e sums its head-dim elements over the splits with the loads of eight splits
// in flight: two dependent trips to memory per row, whatever the number of splits.  COHERENT: the partials were written
// by other workgroups of the SAME launch (possibly on another XCD, behind another L2): they are fetched with
// device-scope loads.  Both users of this function sum in the same order, so their results agree bit for bit.
template <bool COHERENT> __device__ __forceinline__ float part_load(const float *ptr) {
    if (COHERENT) return __uint_as_float(__hip_atomic_load((const uint32_t *)ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    return *ptr;
}

__device__ __forceinline__ void part_store(float *ptr, float v) {
    __hip_atomic_store((uint32_t *)ptr, __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T, bool COHERENT>
__device__ __forceinline__ void combine_row(const FwdParams &p, int64_t row, int lane, float *s_w) {
    using E = Elem<T>;
    const int64_t rows = (int64_t)p.B * p.H;
    const float lv0 = lane < p.splits ? part_load<COHERENT>(p.lse_part + (int64_t)lane * rows + row) : -INFINITY;
    const float lv1 = lane + 64 < p.splits ? part_load<COHERENT>(p.lse_part + (int64_t)(lane + 64) * rows + row) : -INFINITY;
    // the partial outputs of the first eight splits for this lane's first two elements are requested right behind
    // the LSEs (they do not depend on them): one trip to memory instead of two for up to eight splits
    const int64_t step = rows * p.d;
    const float *op_row = p.o_part + row * p.d;
    const int n0 = p.splits < 8 ? p.splits : 8;
    float v0[8], v1[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
        v0[u] = (u < n0 && lane < p.d) ? part_load<COHERENT>(op_row + lane + (int64_t)u * step) : 0.f;
        v1[u] = (u < n0 && lane + 64 < p.d) ? part_load<COHERENT>(op_row + lane + 64 + (int64_t)u * step) : 0.f;
    }
    float mx = fmaxf(lv0, lv1);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    const float w0 = mx == -INFINITY ? 0.f : __expf(lv0 - mx), w1 = mx == -INFINITY ? 0.f : __expf(lv1 - mx);  // exp(-inf) = 0 for empty splits
    float sum = w0 + w1;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off);
    s_w[lane] = w0;
    s_w[lane + 64] = w1;
    __builtin_amdgcn_wave_barrier();  // (the LDS operations of one wave execute in order: the weights are readable below)
    const float inv = sum > 0.f ? 1.f / sum : 0.f;
    const int b = (int)(row / p.H), h = (int)(row % p.H);
    for (int e = lane, n = 0; e < p.d; e += 64, n++) {
        const float *op = op_row + e;
        float acc = 0.f;
        int s = 0;
        if (n < 2) {  // (the splits in ascending order, as everywhere: sums do not depend on how they were fetched)
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (u < n0) acc = fmaf(s_w[u], n == 0 ? v0[u] : v1[u], acc);
            s = n0;
        }
        for (; s + 8 <= p.splits; s += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = part_load<COHERENT>(op + (int64_t)(s + u) * step);
#pragma unroll
            for (int u = 0; u < 8; u++) acc = fmaf(s_w[s + u], v[u], acc);
        }
        for (; s < p.splits; s++) acc = fmaf(s_w[s], part_load<COHERENT>(op + (int64_t)s * step), acc);
        ((uint16_t *)p.o)[b * p.o_b + h * p.o_h + e] = (uint16_t)(E::pack2(acc * inv, 0.f) & 0xffffu);
    }
    if (lane == 0) p.lse[row] = mx == -INFINITY ? INFINITY : mx + __logf(sum);
    __builtin_amdgcn_wave_barrier();  // (s_w is rewritten for the wave's next row)
}

template <typename T, int D, bool PERHEAD, bool WIDE>
__global__ void __launch_bounds__(DEC_THREADS, D <= 128 ? 2 : 1) decode_kernel(const FwdParams p, int keys_per_split) {
    using E = Elem<T>;
    using SM = DecSmem<D>;
    constexpr int CH = D / 8;         // 16-byte chunks per row
    constexpr int RPI = 64 / CH;      // rows covered by one load instruction of a wave
    constexpr int NI = DEC_TILE / RPI;
    constexpr int KS = D / 16, DB = D / 32;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int s_wcount[DEC_NJ][4];
    __shared__ float s_m[4][DEC_COLS], s_l[4][DEC_COLS];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, g = lane >> 5;
    const int split = blockIdx.x, b = blockIdx.z;
    const int G = p.H / p.Hk;
    const int chunks = (G + DEC_COLS - 1) / DEC_COLS;
    const int hk = blockIdx.y / chunks;
    const int g0 = (blockIdx.y % chunks) * DEC_COLS;  // first query head (within the group) of this workgroup
    const int ncol = G - g0 < DEC_COLS ? G - g0 : DEC_COLS;
    const bool col_ok = r < ncol;
    const int h = hk * G + g0 + (col_ok ? r : 0);     // this lane's query head
    const int nchunk = p.d / 8;

    uint16_t *s_idx = (uint16_t *)(smem + SM::OFF_IDX);  // kept keys of the current pass, relative to its first key
    char *sK = smem + wave * SM::WAVE_BYTES;
    char *sV = sK + SM::TILE_BYTES;
    float *sB = (float *)(sV + SM::TILE_BYTES);

    const int lo = split * keys_per_split;
    int hi = lo + keys_per_split;
    if (hi > p.Lk) hi = p.Lk;

    // B operands of S^T = K Q^T: lane supplies Q[head r][16 ks + 8 g .. + 7]; columns without a head are zero
    u32x4_t qf[KS];
    {
        const uint16_t *qp = (const uint16_t *)p.q + b * p.q_b + (int64_t)h * p.q_h;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            qf[ks] = u32x4_t{0, 0, 0, 0};
            if (col_ok && 2 * ks + g < nchunk) qf[ks] = *(const u32x4_t *)(qp + 16 * ks + 8 * g);
        }
    }
    const int hm = p.Hm == p.H ? h : (p.Hm == 1 ? 0 : hk);
    const int hb = p.Hb == p.H ? h : (p.Hb == 1 ? 0 : hk);
    const uint8_t *mrow = p.mask ? p.mask + b * p.m_b + hm * p.m_h : nullptr;
    const uint16_t *brow = p.bias ? (const uint16_t *)p.bias + b * p.bi_b + hb * p.bi_h : nullptr;

    float m = -INFINITY, l = 0.f;  // running maximum of the column (log2 domain), sum over this lane's keys
    f32x16_t o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;

    const uint16_t *kbase = (const uint16_t *)p.k + b * p.k_b + hk * p.k_h;
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.v_b + hk * p.v_h;

    // fragment addresses inside a staged tile (see fdma_common.h)
    const uint32_t a_off = (uint32_t)((pi_row(r) * SM::S + g * 8) * 2);
    const int tj = lane & 15, te = tj >> 2, tc = tj & 3;
    const int tcp = (tc == 1) ? 2 : (tc == 2 ? 1 : tc);
    const int tdh = (lane >> 4) & 1;
    const uint32_t tr_off = (uint32_t)(((8 * g + te) * SM::S + 16 * tdh + 4 * tcp) * 2);
    // staging: this lane's row within a load instruction and its chunk
    const int srow = lane / CH, sc = lane % CH;
    const uint32_t st_off = (uint32_t)((srow * SM::S + sc * 8) * 2);
    const bool pad_lane = sc >= nchunk;             // head dimension below D: these lanes stage zeros
    const int scl = pad_lane ? nchunk - 1 : sc;

    typedef const __attribute__((address_space(1))) char *gptr_t;  // global address space survives the integer round trip
    auto uniform_ptr = [](const void *ptr) -> gptr_t {
        const uint64_t v = (uint64_t)ptr;
        const uint32_t lo32 = __builtin_amdgcn_readfirstlane((uint32_t)v), hi32 = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return (gptr_t)(((uint64_t)hi32 << 32) | lo32);
    };

    for (int r0 = lo; r0 < hi; r0 += DEC_SUPER) {
        // ---- phase 1: ordered list of the kept keys of [r0, r0 + DEC_SUPER).  A thread tests 16 keys of each of
        // the DEC_NJ sub-ranges (one 16-byte mask load per mask row, all of them in flight together); wave scans
        // and one barrier order the output.  Entries are relative to r0.
        uint32_t bits[DEC_NJ];
        {
            u32x4_t mv[DEC_NJ];
#pragma unroll
            for (int j = 0; j < DEC_NJ; j++) {
                const int key0 = r0 + j * DEC_RANGE + 16 * tid;
                mv[j] = u32x4_t{0, 0, 0, 0};
                if (key0 < hi) {
                    if (!p.mask) {
                        mv[j] = u32x4_t{~0u, ~0u, ~0u, ~0u};
                    } else if (!PERHEAD || p.Hm != p.H) {
                        mv[j] = *(const u32x4_t *)(p.mask + b * p.m_b + (int64_t)(p.Hm == 1 ? 0 : hk) * p.m_h + key0);
                    } else {  // union of the mask rows of this workgroup's columns
                        for (int q = 0; q < ncol; q++) {
                            const u32x4_t x = *(const u32x4_t *)(p.mask + b * p.m_b + (int64_t)(hk * G + g0 + q) * p.m_h + key0);
#pragma unroll
                            for (int e = 0; e < 4; e++) mv[j][e] |= x[e];
                        }
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < DEC_NJ; j++) {
                const int nval = hi - (r0 + j * DEC_RANGE + 16 * tid);  // keys of this thread inside the range
                const uint32_t inrange = nval >= 16 ? 0xffffu : (nval <= 0 ? 0u : ((1u << nval) - 1u));
                bits[j] = (nz_bytes_to_bits(mv[j][0]) | (nz_bytes_to_bits(mv[j][1]) << 4) | (nz_bytes_to_bits(mv[j][2]) << 8) |
                           (nz_bytes_to_bits(mv[j][3]) << 12)) & inrange;
            }
        }
        // bits[j] also carries, in its upper half, the kept keys of the lower lanes of this wave in sub-range j
        const int nj = (hi - r0 + DEC_RANGE - 1) / DEC_RANGE < DEC_NJ ? (hi - r0 + DEC_RANGE - 1) / DEC_RANGE : DEC_NJ;
#pragma unroll
        for (int j = 0; j < DEC_NJ; j++) {
            if (j < nj) {
                const int cnt = __popc(bits[j]);
                int wave_total;
                const int incl = wave_scan(cnt, lane, wave_total);
                if (lane == 0) s_wcount[j][wave] = wave_total;
                bits[j] |= (uint32_t)(incl - cnt) << 16;
            }
        }
        __syncthreads();

        // ---- phase 2 (called once the list is complete): a wave takes every fourth batch of 32 kept keys.  The
        // rows of the next batch are in flight (in registers) while the current one is worked on from LDS.
        const gptr_t kb0 = uniform_ptr(kbase + (int64_t)r0 * p.k_r), vb0 = uniform_ptr(vbase + (int64_t)r0 * p.v_r);
        const gptr_t bb0 = uniform_ptr(brow ? brow + r0 : kbase);
        auto process = [&](int total) {
            u32x4_t kreg[NI], vreg[NI];
            uint32_t braw = 0;
            bool bvalid = false;
            auto load_batch = [&](int t0) {
                // rows beyond the list repeat its last row (their scores are dropped below); lanes beyond the head
                // dimension fetch its last chunk and are cleared when the batch is staged
#pragma unroll
                for (int j = 0; j < NI; j++) {
                    const int t = t0 + j * RPI + srow;
                    const uint32_t rel = s_idx[t < total ? t : total - 1];
                    if (WIDE) {
                        kreg[j] = *(const __attribute__((address_space(1))) u32x4_t *)(kb0 + ((int64_t)rel * p.k_r + scl * 8) * 2);
                        vreg[j] = *(const __attribute__((address_space(1))) u32x4_t *)(vb0 + ((int64_t)rel * p.v_r + scl * 8) * 2);
                    } else {
                        kreg[j] = *(const __attribute__((address_space(1))) u32x4_t *)(kb0 + (rel * (uint32_t)p.k_r + scl * 8) * 2u);
                        vreg[j] = *(const __attribute__((address_space(1))) u32x4_t *)(vb0 + (rel * (uint32_t)p.v_r + scl * 8) * 2u);
                    }
                }
                if (!PERHEAD) {  // one fused value per key: lane i < 32 fetches the bias of the batch's key i
                    bvalid = lane < DEC_TILE && t0 + lane < total;
                    braw = 0;
                    if (bvalid && brow) braw = *(const __attribute__((address_space(1))) uint16_t *)(bb0 + 2u * s_idx[t0 + lane]);
                }
            };
            int t0 = wave * DEC_TILE;
            if (t0 < total) load_batch(t0);
            while (t0 < total) {
                // stage the batch (LDS operations of one wave execute in order: the reads of the previous batch are done)
#pragma unroll
                for (int j = 0; j < NI; j++) {
                    *(u32x4_t *)(sK + st_off + j * RPI * SM::S * 2) = pad_lane ? u32x4_t{0, 0, 0, 0} : kreg[j];
                    *(u32x4_t *)(sV + st_off + j * RPI * SM::S * 2) = pad_lane ? u32x4_t{0, 0, 0, 0} : vreg[j];
                }
                if (!PERHEAD && lane < DEC_TILE) sB[lane] = bvalid ? E::lo(braw) * kLog2e : -INFINITY;
                // additive term of this lane's 16 (key, column) pairs: register 8 blk + e <-> key 16 blk + 8 g + e of the batch
                float badd[16];
                if (PERHEAD) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int t = t0 + 16 * (i >> 3) + 8 * g + (i & 7);
                        badd[i] = -INFINITY;
                        if (t < total) {
                            const int key = r0 + (int)s_idx[t];
                            const bool keep = !mrow || mrow[key];
                            const float bv = brow ? E::lo((uint32_t)brow[key]) * kLog2e : 0.f;
                            badd[i] = keep ? bv : -INFINITY;
                        }
                    }
                }
                const int tn = t0 + 4 * DEC_TILE;
                if (tn < total) load_batch(tn);

                // S^T = K Q^T
                f32x16_t s;
#pragma unroll
                for (int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    const u32x4_t a = *(const u32x4_t *)(sK + a_off + ks * 32);
                    s = E::mfma(a, qf[ks], s);
                }
                if (!PERHEAD) {
#pragma unroll
                    for (int blk = 0; blk < 2; blk++) {
                        const f32x4_t b0 = *(const f32x4_t *)(sB + 16 * blk + 8 * g);
                        const f32x4_t b1 = *(const f32x4_t *)(sB + 16 * blk + 8 * g + 4);
#pragma unroll
                        for (int e = 0; e < 4; e++) { badd[8 * blk + e] = b0[e]; badd[8 * blk + 4 + e] = b1[e]; }
                    }
                }
                float mt = -INFINITY;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    s[i] = fmaf(s[i], p.scale_log2, badd[i]);
                    mt = fmaxf(mt, s[i]);
                }
                mt = xhalf_max(mt);
                const float mn = fmaxf(m, mt);
                const float ms = mn == -INFINITY ? 0.f : mn;
                if (__any(mn > m)) {
                    const float alpha = fast_exp2(m - ms);
                    l *= alpha;
#pragma unroll
                    for (int db = 0; db < DB; db++)
#pragma unroll
                        for (int i = 0; i < 16; i++) o[db][i] *= alpha;
                }
                m = mn;
                uint32_t pk[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float p0 = fast_exp2(s[2 * e] - ms), p1 = fast_exp2(s[2 * e + 1] - ms);
                    l += p0 + p1;
                    pk[e] = E::pack2(p0, p1);
                }
                // O^T += V^T P^T (V^T through transposing LDS reads of the row-major rows)
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
                    const u32x4_t bop = {pk[4 * kb], pk[4 * kb + 1], pk[4 * kb + 2], pk[4 * kb + 3]};
#pragma unroll
                    for (int db = 0; db < DB; db++) {
                        const uint32_t off = tr_off + (uint32_t)((16 * kb * SM::S + 32 * db) * 2);
                        const u32x2_t lo_ = lds_read_tr16(sV, off), hi_ = lds_read_tr16(sV, off + 4 * SM::S * 2);
                        const u32x4_t a = {lo_[0], lo_[1], hi_[0], hi_[1]};
                        o[db] = E::mfma(a, bop, o[db]);
                    }
                }
                t0 = tn;
            }
        };

        // append sub-ranges to the list while they fit, work the list off, go on with the rest (dense masks only)
        for (int j = 0; j < nj;) {
            int total = 0;
            for (; j < nj; j++) {
                const int wg_cnt = s_wcount[j][0] + s_wcount[j][1] + s_wcount[j][2] + s_wcount[j][3];
                if (total + wg_cnt > DEC_RANGE) break;
                const uint32_t bj = j == 0 ? bits[0] : (j == 1 ? bits[1] : (j == 2 ? bits[2] : bits[3]));
                int pos = total + (int)(bj >> 16);
                for (int w = 0; w < wave; w++) pos += s_wcount[j][w];
                uint32_t u = bj & 0xffffu;
                while (u) {
                    const int k = __builtin_ctz(u);
                    u &= u - 1;
                    s_idx[pos++] = (uint16_t)(j * DEC_RANGE + 16 * tid + k);
                }
                total += wg_cnt;
            }
            __syncthreads();
            process(total);
            __syncthreads();  // the list (and, after the last round, the counts) are rebuilt next
        }
    }

    // ---- phase 3: every wave leaves its partial result in its own piece of LDS, then the four are merged
    l = xhalf_sum(l);
    if (g == 0 && col_ok) { s_m[wave][r] = m; s_l[wave][r] = l; }
    if (col_ok) {
        float *so = (float *)sK + r * SM::SO;  // [column][d]
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int blk = 0; blk < 2; blk++) {
                const int c = 32 * db + 16 * blk + 8 * g;
                *(f32x4_t *)(so + c) = f32x4_t{o[db][8 * blk], o[db][8 * blk + 1], o[db][8 * blk + 2], o[db][8 * blk + 3]};
                *(f32x4_t *)(so + c + 4) = f32x4_t{o[db][8 * blk + 4], o[db][8 * blk + 5], o[db][8 * blk + 6], o[db][8 * blk + 7]};
            }
    }
    __syncthreads();
    for (int idx = tid; idx < ncol * D; idx += DEC_THREADS) {
        const int col = idx / D, e = idx % D;
        if (e >= p.d) continue;
        float mx = -INFINITY;
#pragma unroll
        for (int q = 0; q < 4; q++) mx = fmaxf(mx, s_m[q][col]);
        float lt = 0.f, ot = 0.f;
        if (mx != -INFINITY) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float w = fast_exp2(s_m[q][col] - mx);
                lt += w * s_l[q][col];
                ot += w * ((const float *)(smem + q * SM::WAVE_BYTES))[col * SM::SO + e];
            }
        }
        const int hh = hk * G + g0 + col;
        const float inv = lt > 0.f ? 1.f / lt : 0.f;
        if (p.splits > 1) {
            // (device-scope stores: written through to where every XCD sees them, so that the merging workgroup of
            // this launch -- or the merge launch -- reads them whichever L2 it sits behind)
            const int64_t row = ((int64_t)split * p.B + b) * p.H + hh;
            part_store(p.o_part + row * p.d + e, ot * inv);
            if (e == 0) part_store(p.lse_part + row, lt > 0.f ? (mx + __builtin_amdgcn_logf(lt)) * kLn2 : -INFINITY);
        } else {
            uint16_t *op = (uint16_t *)p.o + b * p.o_b + hh * p.o_h;
            op[e] = (uint16_t)(E::pack2(ot * inv, 0.f) & 0xffffu);
            if (e == 0) p.lse[(int64_t)b * p.H + hh] = lt > 0.f ? (mx + __builtin_amdgcn_logf(lt)) * kLn2 : INFINITY;
        }
    }
    // ---- phase 4 (arrival counters given): the workgroup that finishes last among the splits of its (batch entry,
    // head chunk) merges their partial results, so the call is one launch.  The partials above are device-scope
    // stores; every wave waits until its own have been acknowledged, the barrier collects the waves, and one thread
    // then counts the workgroup in with a device-scope atomic (no cache write-back or invalidate is involved: a fence
    // would walk the whole L2 in every workgroup, which made this launch four times longer than the two it replaces).
    // The counter starts at zero, and the last arrival puts it back to zero for the next call.  Nothing waits for
    // another workgroup: one that is not last just ends.
    if (p.splits > 1 && p.dec_counter) {
        __shared__ int s_last;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            int32_t *cnt = p.dec_counter + ((int64_t)b * gridDim.y + blockIdx.y);
            const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int last = old == p.splits - 1;
            if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = last;
        }
        __syncthreads();
        if (s_last) {
            for (int col = wave; col < ncol; col += 4)
                combine_row<T, true>(p, (int64_t)b * p.H + hk * G + g0 + col, lane, (float *)(smem + wave * 512));
        }
    }
}

// The merge as a launch of its own (no arrival counters given): one wave per (b, h) row, four rows per workgroup.
constexpr int CMB_THREADS = 256;
constexpr int CMB_MAX_SPLITS = 128;  // >= the largest number of splits (decode_num_splits): a lane holds two of them

template <typename T>
__global__ void __launch_bounds__(CMB_THREADS) decode_combine_kernel(const FwdParams p) {
    __shared__ float s_w[CMB_THREADS / 64][CMB_MAX_SPLITS];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (CMB_THREADS / 64) + wave;
    if (row < (int64_t)p.B * p.H) combine_row<T, false>(p, row, lane, s_w[wave]);
}

template <typename T, int D, bool PERHEAD, bool WIDE>
hipError_t launch_decode_w(const FwdParams &p, int keys_per_split, hipStream_t stream) {
    const int G = p.H / p.Hk;
    const int chunks = (G + DEC_COLS - 1) / DEC_COLS;
    dim3 grid(p.splits, p.Hk * chunks, p.B);
    auto kern = decode_kernel<T, D, PERHEAD, WIDE>;
    static DynSmemLimit smem_limit;
    hipError_t e = smem_limit.ensure((const void *)kern, DecSmem<D>::TOTAL);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, dim3(DEC_THREADS), DecSmem<D>::TOTAL, stream, p, keys_per_split);
    return hipGetLastError();
}

template <typename T, int D, bool PERHEAD>
hipError_t launch_decode_d(const FwdParams &p, int keys_per_split, hipStream_t stream) {
    // byte offsets of a gathered row relative to the first row of a pass fit 32 bits unless the row stride is huge
    const int64_t rmax = p.k_r > p.v_r ? p.k_r : p.v_r;
    const bool wide = ((int64_t)DEC_SUPER * rmax + D) * 2 >= ((int64_t)1 << 32);
    return wide ? launch_decode_w<T, D, PERHEAD, true>(p, keys_per_split, stream) : launch_decode_w<T, D, PERHEAD, false>(p, keys_per_split, stream);
}

template <typename T>
hipError_t launch_decode_t(const FwdParams &p, hipStream_t stream) {
    const int G = p.H / p.Hk;
    const int keys_per_split = ((p.Lk + p.splits - 1) / p.splits + DEC_THREADS - 1) / DEC_THREADS * DEC_THREADS;
    const bool perhead = G > 1 && ((p.mask && p.Hm == p.H) || (p.bias && p.Hb == p.H));
    hipError_t e;
    if (p.d <= 64) e = perhead ? launch_decode_d<T, 64, true>(p, keys_per_split, stream) : launch_decode_d<T, 64, false>(p, keys_per_split, stream);
    else if (p.d <= 128) e = perhead ? launch_decode_d<T, 128, true>(p, keys_per_split, stream) : launch_decode_d<T, 128, false>(p, keys_per_split, stream);
    else e = perhead ? launch_decode_d<T, 256, true>(p, keys_per_split, stream) : launch_decode_d<T, 256, false>(p, keys_per_split, stream);
    if (e != hipSuccess) return e;
    if (p.splits > 1 && !p.dec_counter) {  // (with arrival counters the decode launch has merged its splits itself)
        const int64_t rows = (int64_t)p.B * p.H;
        hipLaunchKernelGGL((decode_combine_kernel<T>), dim3((unsigned)((rows + CMB_THREADS / 64 - 1) / (CMB_THREADS / 64))), dim3(CMB_THREADS), 0, stream, p);
        e = hipGetLastError();
    }
    return e;
}

}  // namespace

// Decode route: one query token and a head dimension one lane-group can hold (16 lanes x 8).
bool use_decode_path(int Lq, int H, int Hk) {
    (void)H; (void)Hk;
    return Lq == 1;
}

// Workgroups have a fixed cost of several microseconds (mask fetch, list, merge), so few fat ones win: two per CU
// (all resident at once) when a split then still spans 8192 keys, otherwise one per CU; at least 256 keys per
// split.  With keys_per_split rounded up to 256 every split is non-empty.
int decode_num_splits(int B, int Hk, int Lk) {
    const int pairs = B * Hk > 0 ? B * Hk : 1;
    int splits = (512 + pairs - 1) / pairs;
    if ((int64_t)splits * 8192 > Lk) splits = (256 + pairs - 1) / pairs;
    const int max_by_len = (Lk + 255) / 256;
    if (splits > max_by_len) splits = max_by_len;
    if (splits > CMB_MAX_SPLITS) splits = CMB_MAX_SPLITS;
    if (splits < 1) splits = 1;
    // shrink so that no split is empty after rounding keys_per_split up to a multiple of 256
    while (splits > 1) {
        const int kps = ((Lk + splits - 1) / splits + 255) / 256 * 256;
        if ((int64_t)(splits - 1) * kps < Lk) break;
        splits--;
    }
    return splits;
}

int64_t decode_num_counters(int B, int H, int Hk, int Lk) {
    if (B <= 0 || Hk <= 0 || decode_num_splits(B, Hk, Lk) <= 1) return 0;
    const int G = H / Hk;
    return (int64_t)B * Hk * ((G + DEC_COLS - 1) / DEC_COLS);
}

hipError_t launch_fwd_decode(const FwdParams &p, int dtype, hipStream_t stream) {
    if (p.B <= 0) return hipSuccess;
    return dtype == 0 ? launch_decode_t<bf16_tag>(p, stream) : launch_decode_t<fp16_tag>(p, stream);
}

}  // namespace fdma
