// Column compaction pre-pass for keep-masks that are broadcast over the query dimension.
//
// With a mask of shape [B, {1,Hk}, 1, Lk] a key column is kept or dropped for every query of a
// (batch, kv head) pair at once, so attention over the kept columns only is the same function as
// masked attention over all of them (the reference shows the equivalence on the CPU in
// benchmarks/grad_equivalence.py:55-140, and its Triton variant gathers K / V the same way,
// flash_sparse_attn/flash_dmattn_triton.py:50-211).  Tile skipping cannot exploit such a mask when the
// kept columns are scattered -- nearly every 64-key tile holds a kept key -- but gathering them makes
// the work proportional to the number of kept keys:
//   scan    one workgroup per (batch, kv head): ordered list `idx` of kept columns, inclusive prefix
//           counts `cnt` (what a causal query row needs: how many kept columns are <= its limit), total;
//   gather  wide grid: K / V rows of the kept columns copied into dense [B, Hk, count, d] buffers, bias
//           gathered and pre-scaled into an fp32 vector;
//   (forward, up to 65536 keys) scan and gather in ONE launch: a workgroup per 256 original columns counts the kept
//           columns in front of its segment itself;
//   (backward) zero   rows of dK / dV and columns of dBias that belong to dropped keys.
// All of this is O(Lk * d) traffic in front of O(Lq * count * d) MFMA work.
#include <atomic>

#include "fdma_common.h"
#include "fdma_params.h"
#include "fdma_bwd_dot.h"
#include "fdma_scan.h"

namespace fdma {

namespace {

constexpr int SCAN_THREADS = 1024;
constexpr int GATHER_KEYS = 64;                        // compacted keys per gather workgroup

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct Layout {
    size_t off_idx, off_cnt, off_count, off_fb, off_k, off_v, off_plan, off_part_kv, off_part_db, total;
    size_t off_bk, off_bv;  // backward on a forward workspace that holds tile images: its own row-major copies
    int ld, Hfb;
    bool img;       // the forward part holds tile images (off_k: K | V^T per tile, off_v: side rows) instead of copies
    int img_tiles;  // tiles per (batch, kv head) pair
};

Layout layout_of(const FwdParams &p, bool backward) {
    Layout l;
    l.ld = (p.Lk + 15) / 16 * 16;
    l.Hfb = (p.bias && p.Hb == p.H) ? p.H : p.Hk;
    l.img = fwd_stream_applicable(p);
    l.img_tiles = (p.Lk + IMG_BN - 1) / IMG_BN;
    const size_t pairs = (size_t)p.B * p.Hk;
    size_t o = 0;
    l.off_idx = o;   o += align256(pairs * l.ld * 4);
    l.off_cnt = o;   o += align256(pairs * l.ld * 4);
    l.off_count = o; o += align256(pairs * 4);
    l.off_fb = o;    o += align256((size_t)p.B * l.Hfb * l.ld * 4);
    if (l.img) {
        l.off_k = o; o += align256(pairs * l.img_tiles * IMG_KV_BYTES);
        l.off_v = o; o += align256((size_t)p.B * l.Hfb * l.img_tiles * IMG_X_BYTES);
    } else {
        l.off_k = o; o += align256(pairs * p.Lk * p.d * 2);
        l.off_v = o; o += align256(pairs * p.Lk * p.d * 2);
    }
    l.off_plan = l.off_part_kv = l.off_part_db = l.off_bk = l.off_bv = o;
    if (backward) {
        if (l.img) {  // (the backward kernels read row-major copies: made by the backward's own pre-pass)
            l.off_bk = o; o += align256(pairs * p.Lk * p.d * 2);
            l.off_bv = o; o += align256(pairs * p.Lk * p.d * 2);
        }
        int grid, slots;
        dkdv_split_bounds((int)pairs, (p.Lk + 127) / 128, p.H / p.Hk, grid, slots);
        const int dpad = p.d <= 64 ? 64 : (p.d <= 128 ? 128 : 256);
        // header, prefix of the units over the pairs and, per XCD, the list of the parts that exist (two ints each;
        // the kernel's grid bounds their number)
        l.off_plan = o;    o += align256((DKDV_PLAN_HDR + pairs + 1 + 8 + 2 * (size_t)grid) * 4);
        l.off_part_kv = o; o += align256((size_t)slots * 2 * dpad * 128 * 4);
        l.off_part_db = o; o += align256((size_t)slots * (p.H / p.Hk) * 128 * 4);
    }
    l.total = o;
    return l;
}

__global__ void __launch_bounds__(SCAN_THREADS) compact_scan_kernel(const FwdParams p, int32_t *idx, int32_t *cnt,
                                                                     int32_t *count, int ld) {
    __shared__ int s_wave[SCAN_THREADS / 64];
    const int pair = blockIdx.x, b = pair / p.Hk, hk = pair % p.Hk;
    const int hm = p.Hm == 1 ? 0 : hk;
    scan_mask_row<SCAN_THREADS>(p.mask + b * p.m_b + hm * p.m_h, p.Lk, idx + (size_t)pair * ld, cnt + (size_t)pair * ld,
                                count + pair, s_wave, true);
}

// orig: the caller's tensors.  kc / vc: dense [B*Hk, Lk, d] destinations.
// copies_only: the per-pair lists and the fused bias exist already (made by the forward call whose workspace this is);
// only the K / V rows are copied.
template <typename T>
__device__ __forceinline__ void gather_block(const FwdParams &p, const int32_t *idx, int32_t *cnt, const int32_t *count, float *fb,
                                             uint16_t *kc, uint16_t *vc, int ld, int Hfb, int block_x, int pair, bool copies_only = false) {
    using E = Elem<T>;
    const int b = pair / p.Hk, hk = pair % p.Hk;
    const int tid = threadIdx.x;
    const int c0 = block_x * GATHER_KEYS;
    // Lists handed over by the caller (one row per mask row): this block copies its 64 entries of the row into the
    // per-pair arrays the kernels index (in place of the scan), and reads its own inputs from the source
    const int32_t *src_idx = idx + (size_t)pair * ld;
    int n;
    if (p.kept_idx && !copies_only) {
        const int srow = (p.m_b == 0 ? 0 : b) * p.Hm + (p.Hm == 1 ? 0 : hk);
        src_idx = p.kept_idx + (size_t)srow * p.kept_ld;
        // (lists are device data the host cannot check: a list made for a longer key axis than this call's must not
        // take reads or gradient writes past the tensors, so counts and columns are held inside [0, Lk))
        n = p.kept_count[srow];
        n = n < p.Lk ? n : p.Lk;
        if (tid < GATHER_KEYS && c0 + tid < ld) {
            const int32_t col = src_idx[c0 + tid], have = p.kept_cnt[(size_t)srow * p.kept_ld + c0 + tid];
            ((int32_t *)idx)[(size_t)pair * ld + c0 + tid] = col < p.Lk ? col : p.Lk - 1;
            cnt[(size_t)pair * ld + c0 + tid] = have < n ? have : n;
        }
        if (block_x == 0 && tid == 0) ((int32_t *)count)[pair] = n;
    } else {
        n = count[pair];
    }
    if (c0 >= n) return;
    __shared__ int s_src[GATHER_KEYS];
    if (tid < GATHER_KEYS) {
        const int32_t col = (c0 + tid < n) ? src_idx[c0 + tid] : -1;
        s_src[tid] = col < p.Lk ? col : p.Lk - 1;
    }
    __syncthreads();
    const int CH = p.d / 8;
    const uint16_t *kb = (const uint16_t *)p.k + b * p.k_b + kv_head(p, hk) * p.k_h;
    const uint16_t *vb = (const uint16_t *)p.v + b * p.v_b + kv_head(p, hk) * p.v_h;
    uint16_t *kd = kc + ((size_t)pair * p.Lk + c0) * p.d;
    uint16_t *vd = vc + ((size_t)pair * p.Lk + c0) * p.d;
    for (int it = tid; it < GATHER_KEYS * CH; it += 256) {
        const int rr = it / CH, ch = it - rr * CH;
        const int src = s_src[rr];
        if (src >= 0) {
            const u32x4_t kv = *(const u32x4_t *)(kb + (int64_t)src * p.k_r + ch * 8);
            const u32x4_t vv = *(const u32x4_t *)(vb + (int64_t)src * p.v_r + ch * 8);
            *(u32x4_t *)(kd + (size_t)rr * p.d + ch * 8) = kv;
            *(u32x4_t *)(vd + (size_t)rr * p.d + ch * 8) = vv;
        }
    }
    if (copies_only) return;
    // fused bias of the compacted keys, one vector per bias class of this kv head
    const int G = p.H / p.Hk;
    const int nfb = Hfb == p.H ? G : 1;
    for (int it = tid; it < GATHER_KEYS * nfb; it += 256) {
        const int gi = it / GATHER_KEYS, rr = it - gi * GATHER_KEYS;
        const int src = s_src[rr];
        if (src < 0) continue;
        const int hfb = Hfb == p.H ? hk * G + gi : hk;
        float v = 0.f;
        if (p.bias) {
            const int hb = p.Hb == p.H ? hfb : (p.Hb == 1 ? 0 : kv_head(p, hk));
            v = E::lo((uint32_t)((const uint16_t *)p.bias)[b * p.bi_b + hb * p.bi_h + src]) * kLog2e;
        }
        fb[((size_t)b * Hfb + hfb) * ld + c0 + rr] = v;
    }
}

template <typename T>
__global__ void __launch_bounds__(256) compact_gather_kernel(const FwdParams p, const int32_t *idx, int32_t *cnt, const int32_t *count,
                                                              float *fb, uint16_t *kc, uint16_t *vc, int ld, int Hfb) {
    gather_block<T>(p, idx, cnt, count, fb, kc, vc, ld, Hfb, blockIdx.x, blockIdx.y);
}

// Scan and gather of the forward in one launch: a workgroup owns SEG_KEYS consecutive ORIGINAL columns of a pair.  It
// counts the kept columns in front of its segment itself (at most Lk mask bytes, which all workgroups of the pair read
// and the L2 serves), numbers its own, writes its part of `idx` and `cnt` and copies its kept K / V rows and bias values
// to their compacted places.  One launch less in front of the attention kernel than scan + gather.
constexpr int SEG_KEYS = 256;

template <typename T>
__global__ void __launch_bounds__(256) compact_scan_gather_kernel(const FwdParams p, int32_t *idx, int32_t *cnt, int32_t *count,
                                                                   float *fb, uint16_t *kc, uint16_t *vc, int ld, int Hfb) {
    using E = Elem<T>;
    __shared__ int s_wave[4], s_src[SEG_KEYS];
    const int pair = blockIdx.y, b = pair / p.Hk, hk = pair % p.Hk;
    const int hm = p.Hm == 1 ? 0 : hk;
    const uint8_t *mrow = p.mask + b * p.m_b + hm * p.m_h;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int s0 = blockIdx.x * SEG_KEYS;
    // kept columns in front of the segment (s0 is a multiple of 16; mask rows are readable in 16-byte pieces)
    int before = 0;
    for (int c = tid * 16; c < s0; c += 256 * 16) {
        const u32x4_t mv = *(const u32x4_t *)(mrow + c);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            // a byte is non-zero <=> bit 7 of ((x & 0x7f) + 0x7f) | x is set
            const uint32_t x = mv[e];
            before += __builtin_popcount((((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off);
    if (lane == 0) s_wave[wave] = before;
    __syncthreads();
    const int base = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
    __syncthreads();
    // this segment: one column per thread
    const int col = s0 + tid;
    const bool kept = col < p.Lk && mrow[col] != 0;
    const uint64_t vote = __ballot(kept);
    const int excl_w = __builtin_popcountll(vote & ((1ull << lane) - 1ull));
    if (lane == 0) s_wave[wave] = __builtin_popcountll(vote);
    __syncthreads();
    int woff = 0, n_seg = 0;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const int v = s_wave[w];
        if (w < wave) woff += v;
        n_seg += v;
    }
    const int excl = woff + excl_w;  // kept columns of the segment in front of this one
    int32_t *irow = idx + (size_t)pair * ld, *crow = cnt + (size_t)pair * ld;
    if (kept) {
        irow[base + excl] = col;
        s_src[excl] = col;
    }
    if (col < ld) crow[col] = base + excl + (kept ? 1 : 0);  // (columns from Lk to ld repeat the total)
    if (s0 + SEG_KEYS >= ld && tid == 0) count[pair] = base + n_seg;
    __syncthreads();
    if (n_seg == 0) return;
    const int CH = p.d / 8;
    const uint16_t *kb = (const uint16_t *)p.k + b * p.k_b + kv_head(p, hk) * p.k_h;
    const uint16_t *vb = (const uint16_t *)p.v + b * p.v_b + kv_head(p, hk) * p.v_h;
    uint16_t *kd = kc + ((size_t)pair * p.Lk + base) * p.d;
    uint16_t *vd = vc + ((size_t)pair * p.Lk + base) * p.d;
    for (int it = tid; it < n_seg * CH; it += 256) {
        const int rr = it / CH, ch = it - rr * CH;
        const int src = s_src[rr];
        const u32x4_t kv = *(const u32x4_t *)(kb + (int64_t)src * p.k_r + ch * 8);
        const u32x4_t vv = *(const u32x4_t *)(vb + (int64_t)src * p.v_r + ch * 8);
        *(u32x4_t *)(kd + (size_t)rr * p.d + ch * 8) = kv;
        *(u32x4_t *)(vd + (size_t)rr * p.d + ch * 8) = vv;
    }
    // fused bias of the compacted keys, one vector per bias class of this kv head
    const int G = p.H / p.Hk;
    const int nfb = Hfb == p.H ? G : 1;
    for (int it = tid; it < n_seg * nfb; it += 256) {
        const int gi = it / n_seg, rr = it - gi * n_seg;
        const int src = s_src[rr];
        const int hfb = Hfb == p.H ? hk * G + gi : hk;
        float v = 0.f;
        if (p.bias) {
            const int hb = p.Hb == p.H ? hfb : (p.Hb == 1 ? 0 : kv_head(p, hk));
            v = E::lo((uint32_t)((const uint16_t *)p.bias)[b * p.bi_b + hb * p.bi_h + src]) * kLog2e;
        }
        fb[((size_t)b * Hfb + hfb) * ld + base + rr] = v;
    }
}

// Tile images for the streaming forward (fdma_fwd_stream.hip), scan included, in ONE launch: workgroup j of a (batch,
// kv head) pair owns tile j of the compacted key axis -- the kept columns of rank 64 j .. 64 j + 63.  It finds them by
// counting the whole mask row itself (every thread a contiguous piece of it; at most 64 KB per pair, read by all
// workgroups of the pair and served by the L2), writes its part of the lists (idx for its ranks; cnt for the original
// columns in front of which 64 j .. 64 j + 63 kept columns lie -- every column belongs to exactly one tile that way, the
// columns behind the last kept one included) and then the tile as the forward keeps it in LDS: K rows padded to
// IMG_SK elements, V transposed (rows of IMG_SVT elements), and per bias class the 16-element side rows (three 16-bit
// pieces of bias * log2(e), the mask term, two ones, zeros).  Rows beyond the last kept key are zeros with a side row
// that says "masked": the forward needs no row limit.  With lists handed over by the caller nothing is counted.
// Eight 16-bit elements times a factor (the K rows of a tile image carry softmax_scale * log2(e): the streaming forward
// then uses Q as it lies in memory, and what would be a scaling pass over Q per work item is paid once per key here)
template <typename T> __device__ __forceinline__ u32x4_t scale8(u32x4_t v, float f) {
    using E = Elem<T>;
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = E::pack2(E::lo(v[e]) * f, E::hi(v[e]) * f);
    return v;
}

template <typename T>
__global__ void __launch_bounds__(256) compact_image_kernel(const FwdParams p, int32_t *idx, int32_t *cnt, int32_t *count, float *fb,
                                                            char *img_kv, char *img_x, int ld, int Hfb, int tiles) {
    using E = Elem<T>;
    __shared__ int s_wave[4], s_src[IMG_BN];
    const int pair = blockIdx.y, b = pair / p.Hk, hk = pair % p.Hk;
    const int j = blockIdx.x, lo = j * IMG_BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int32_t *irow = idx + (size_t)pair * ld, *crow = cnt + (size_t)pair * ld;
    if (tid < IMG_BN) s_src[tid] = -1;
    __syncthreads();
    int total;
    if (p.kept_idx) {
        const int srow = (p.m_b == 0 ? 0 : b) * p.Hm + (p.Hm == 1 ? 0 : hk);
        const int32_t *src_idx = p.kept_idx + (size_t)srow * p.kept_ld;
        total = p.kept_count[srow];
        total = total < p.Lk ? total : p.Lk;  // (lists are device data: held inside [0, Lk), see gather_block)
        if (tid < IMG_BN && lo + tid < ld) {
            int32_t col = src_idx[lo + tid];
            const int32_t have = p.kept_cnt[(size_t)srow * p.kept_ld + lo + tid];
            col = col < p.Lk ? col : p.Lk - 1;
            irow[lo + tid] = col;
            crow[lo + tid] = have < total ? have : total;
            if (lo + tid < total) s_src[tid] = col < 0 ? 0 : col;
        }
    } else {
        const int hm = p.Hm == 1 ? 0 : hk;
        const uint8_t *mrow = p.mask + b * p.m_b + hm * p.m_h;
        const int cpt = (((ld + 255) >> 8) + 15) & ~15;  // columns per thread: a multiple of 16
        const int c0 = tid * cpt, c1 = c0 + cpt < p.Lk ? c0 + cpt : p.Lk;
        // nonzero bytes of a 4-byte word whose first byte is column c, bytes at or beyond Lk dropped: bit 8 k + 7 for byte k
        auto kept_bits = [&](uint32_t x, int c) -> uint32_t {
            uint32_t y = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
            const int valid = p.Lk - c;
            if (valid < 4) y &= valid <= 0 ? 0u : (0xffffffffu >> (8 * (4 - valid)));
            return y;
        };
        // (a piece of up to 64 columns stays in registers for the second look; longer ones are fetched again)
        constexpr int KEEP = 4;
        const bool keep = cpt <= 16 * KEEP;
        u32x4_t held[KEEP];
#pragma unroll
        for (int w = 0; w < KEEP; w++) held[w] = u32x4_t{0, 0, 0, 0};
        int mine = 0;
        if (keep) {
#pragma unroll
            for (int w = 0; w < KEEP; w++) {
                const int c = c0 + 16 * w;
                if (w * 16 < cpt && c < c1) held[w] = *(const u32x4_t *)(mrow + c);
            }
#pragma unroll
            for (int w = 0; w < KEEP; w++)
#pragma unroll
                for (int e = 0; e < 4; e++) mine += __builtin_popcount(kept_bits(held[w][e], c0 + 16 * w + 4 * e));
        } else {
            for (int c = c0; c < c1; c += 16) {
                const u32x4_t mv = *(const u32x4_t *)(mrow + c);
#pragma unroll
                for (int e = 0; e < 4; e++) mine += __builtin_popcount(kept_bits(mv[e], c + 4 * e));
            }
        }
        int incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        int woff = 0;
        total = 0;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const int v = s_wave[w];
            if (w < wave) woff += v;
            total += v;
        }
        const int r0 = woff + incl - mine;  // kept columns in front of this thread's piece
        // this thread's columns see r0 .. r0 + mine kept columns in front of them: walk the piece again when some of
        // them belong to this tile
        if (c0 < c1 && r0 <= lo + IMG_BN - 1 && r0 + mine >= lo) {
            int run = r0;
            auto walk = [&](const u32x4_t mv, int c) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t y = kept_bits(mv[e], c + 4 * e);
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const int col = c + 4 * e + k;
                        const bool kept = (y >> (8 * k + 7)) & 1u;
                        if (col < p.Lk && run >= lo && run < lo + IMG_BN) {  // `run` kept columns in front of col
                            crow[col] = run + (kept ? 1 : 0);
                            if (kept) {
                                irow[run] = col;
                                s_src[run - lo] = col;
                            }
                        }
                        run += kept ? 1 : 0;
                    }
                }
            };
            if (keep) {
#pragma unroll
                for (int w = 0; w < KEEP; w++)
                    if (c0 + 16 * w < c1) walk(held[w], c0 + 16 * w);
            } else {
                for (int c = c0; c < c1; c += 16) walk(*(const u32x4_t *)(mrow + c), c);
            }
        }
        // (columns from Lk to the end of the row repeat the total)
        if (total >= lo && total < lo + IMG_BN)
            for (int c = p.Lk + tid; c < ld; c += 256) crow[c] = total;
    }
    if (j == 0 && tid == 0) count[pair] = total;
    __syncthreads();
    const int n = total - lo < IMG_BN ? total - lo : IMG_BN;  // kept keys of this tile
    if (n <= 0 || j >= tiles) return;
    // ---- K rows: thread (row, 16-byte chunk), four passes; V^T: thread (key quad, d chunk) transposes 4 keys x 8 d in
    // registers (as the forward used to while staging).  All sixteen row pieces of a thread are requested before the
    // first is stored: one trip to memory for the tile.
    const uint16_t *kb = (const uint16_t *)p.k + b * p.k_b + kv_head(p, hk) * p.k_h;
    const uint16_t *vb = (const uint16_t *)p.v + b * p.v_b + kv_head(p, hk) * p.v_h;
    char *tile = img_kv + ((size_t)pair * tiles + j) * IMG_KV_BYTES;
    const u32x4_t zero4 = {0, 0, 0, 0};
    const int G = p.H / p.Hk;
    const int nfb = Hfb == p.H ? G : 1;
    {
        const int ch = tid & 15, rr0 = tid >> 4;
        const int vkg = tid & 15, vc = tid >> 4;
        u32x4_t kv[4], vv[4];
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int src = s_src[rr0 + 16 * it];
            kv[it] = src >= 0 ? *(const u32x4_t *)(kb + (int64_t)src * p.k_r + ch * 8) : zero4;
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int src = s_src[4 * vkg + q];
            vv[q] = src >= 0 ? *(const u32x4_t *)(vb + (int64_t)src * p.v_r + vc * 8) : zero4;
        }
        // (the bias value of this thread's first side row travels with the rows)
        uint32_t braw0 = 0;
        if (p.bias && tid < IMG_BN * nfb) {
            const int gi = tid / IMG_BN, src = s_src[tid - gi * IMG_BN];
            const int hfb = Hfb == p.H ? hk * G + gi : hk;
            const int hb = p.Hb == p.H ? hfb : (p.Hb == 1 ? 0 : kv_head(p, hk));
            if (src >= 0) braw0 = ((const uint16_t *)p.bias)[b * p.bi_b + hb * p.bi_h + src];
        }
#pragma unroll
        for (int it = 0; it < 4; it++) *(u32x4_t *)(tile + (rr0 + 16 * it) * (IMG_SK * 2) + ch * 16) = scale8<T>(kv[it], p.scale_log2);
        char *vt = tile + IMG_K_BYTES;
#pragma unroll
        for (int dd = 0; dd < 8; dd++) {
            const int w = dd >> 1;
            const uint32_t sel = (dd & 1) ? 0x07060302u : 0x05040100u;
            u32x2_t out;
            out[0] = __builtin_amdgcn_perm(vv[1][w], vv[0][w], sel);
            out[1] = __builtin_amdgcn_perm(vv[3][w], vv[2][w], sel);
            *(u32x2_t *)(vt + ((vc * 8 + dd) * IMG_SVT + 4 * vkg) * 2) = out;
        }
        // ---- side rows and the fused bias vector (which the backward reads), one set per bias class of this kv head
        for (int it = tid; it < IMG_BN * nfb; it += 256) {
            const int gi = it / IMG_BN, rr = it - gi * IMG_BN;
            const int src = s_src[rr];
            const int hfb = Hfb == p.H ? hk * G + gi : hk;
            float v = 0.f;
            if (src >= 0 && p.bias) {
                uint32_t braw = braw0;
                if (it != tid) {
                    const int hb = p.Hb == p.H ? hfb : (p.Hb == 1 ? 0 : kv_head(p, hk));
                    braw = ((const uint16_t *)p.bias)[b * p.bi_b + hb * p.bi_h + src];
                }
                v = E::lo(braw) * kLog2e;
            }
            if (src >= 0) fb[((size_t)b * Hfb + hfb) * ld + lo + rr] = v;
            const u32x2_t pc = split3<T>(v);
            u32x4_t row;
            row[0] = pc[0];
            row[1] = pc[1] | (E::pack2(0.f, src >= 0 ? 0.f : -INFINITY) & 0xffff0000u);
            row[2] = E::pack2(E::kRefWeight, 1.f);
            row[3] = 0;
            char *xr = img_x + (((size_t)b * Hfb + hfb) * tiles + j) * IMG_X_BYTES + rr * 32;
            *(u32x4_t *)xr = row;
            *(u32x4_t *)(xr + 16) = zero4;
        }
    }
}

// The same images from a plain bool mask, in one launch, with the work split over ORIGINAL columns (as in
// compact_scan_gather_kernel): a workgroup owns SEG_KEYS consecutive columns of a pair, counts the kept columns in
// front of them (at most Lk mask bytes, served by the L2), numbers its own, writes its part of the lists and puts its
// kept keys where their ranks say: K rows and side rows are whole pieces of a tile image, V goes in transposed through
// LDS -- neighbouring ranks of one head-dim element are neighbours in the image, whichever workgroup owns them.  The workgroup that owns the end of the row also clears what is left of the pair's last tile.  (A
// workgroup per tile, each counting the whole row for itself, took 34 us on 4 x 32768 keys; this takes a quarter.)
template <typename T>
__global__ void __launch_bounds__(256) compact_scan_image_kernel(const FwdParams p, int32_t *idx, int32_t *cnt, int32_t *count, float *fb,
                                                                 char *img_kv, char *img_x, int ld, int Hfb, int tiles) {
    using E = Elem<T>;
    constexpr int VT_CHUNK = 128, VT_PITCH = 130;  // V rows parked in LDS at a time; their pitch in elements (odd in 32-bit words)
    __shared__ int s_wave[4], s_src[SEG_KEYS];
    __shared__ __attribute__((aligned(16))) uint16_t s_v[VT_CHUNK * VT_PITCH];
    const int pair = blockIdx.y, b = pair / p.Hk, hk = pair % p.Hk;
    const int hm = p.Hm == 1 ? 0 : hk;
    const uint8_t *mrow = p.mask + b * p.m_b + hm * p.m_h;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int s0 = blockIdx.x * SEG_KEYS;
    // (this thread's own column and up to four pieces of the row in front of the segment are requested together: the
    // launch is a chain of trips to memory, not a stream of bytes)
    const int col = s0 + tid;
    const uint8_t own = col < p.Lk ? mrow[col] : (uint8_t)0;
    int before = 0;
    for (int c = tid * 16; c < s0; c += 4 * 256 * 16) {
        u32x4_t mv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int cc = c + u * 256 * 16;
            mv[u] = cc < s0 ? *(const u32x4_t *)(mrow + cc) : u32x4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t x = mv[u][e];
                before += __builtin_popcount((((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u);
            }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off);
    if (lane == 0) s_wave[wave] = before;
    __syncthreads();
    const int base = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
    __syncthreads();
    const bool kept = own != 0;
    const uint64_t vote = __ballot(kept);
    const int excl_w = __builtin_popcountll(vote & ((1ull << lane) - 1ull));
    if (lane == 0) s_wave[wave] = __builtin_popcountll(vote);
    __syncthreads();
    int woff = 0, n_seg = 0;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const int v = s_wave[w];
        if (w < wave) woff += v;
        n_seg += v;
    }
    const int excl = woff + excl_w;
    int32_t *irow = idx + (size_t)pair * ld, *crow = cnt + (size_t)pair * ld;
    if (kept) {
        irow[base + excl] = col;
        s_src[excl] = col;
    }
    if (col < ld) crow[col] = base + excl + (kept ? 1 : 0);  // (columns from Lk to ld repeat the total)
    const bool owns_end = s0 + SEG_KEYS >= ld;
    const int total = base + n_seg;  // (the pair's total only where owns_end)
    if (owns_end && tid == 0) count[pair] = total;
    __syncthreads();
    const uint16_t *kb = (const uint16_t *)p.k + b * p.k_b + kv_head(p, hk) * p.k_h;
    const uint16_t *vb = (const uint16_t *)p.v + b * p.v_b + kv_head(p, hk) * p.v_h;
    char *pair_img = img_kv + (size_t)pair * tiles * IMG_KV_BYTES;
    const u32x4_t zero4 = {0, 0, 0, 0};
    const int G = p.H / p.Hk;
    const int nfb = Hfb == p.H ? G : 1;
    // rows of rank base .. base + n_seg - 1; and (owns_end) cleared rows up to the end of the last tile.  At most
    // VT_CHUNK rows at a time: their K rows go straight to the image as 16-byte pieces (all loads of up to four pieces
    // per thread requested before the first store), their V rows are parked in LDS and leave transposed, eight
    // neighbouring ranks of one head-dim element per 16-byte store; only where eight ranks are shared with the
    // neighbouring workgroup (or chunk) do they leave one by one.  (One 16-bit store per (key, d) kept the L2 busy with
    // two million two-byte requests per launch on 8 x 2048 kept keys.)
    const int n_pad = owns_end ? ((total + IMG_BN - 1) / IMG_BN) * IMG_BN - total : 0;
    const int n_rows = n_seg + n_pad;
    // (the bias value of this thread's first side row travels with the rows)
    uint32_t braw0 = 0;
    if (p.bias && tid < n_rows * nfb) {
        const int gi = tid / n_rows, rr = tid - gi * n_rows;
        const int hfb = Hfb == p.H ? hk * G + gi : hk;
        const int hb = p.Hb == p.H ? hfb : (p.Hb == 1 ? 0 : kv_head(p, hk));
        if (rr < n_seg) braw0 = ((const uint16_t *)p.bias)[b * p.bi_b + hb * p.bi_h + s_src[rr]];
    }
    for (int c0 = 0; c0 < n_rows; c0 += VT_CHUNK) {
        const int nc = n_rows - c0 < VT_CHUNK ? n_rows - c0 : VT_CHUNK;
        for (int it0 = tid; it0 < nc * 16; it0 += 256 * 4) {
            u32x4_t kv[4], vv[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int it = it0 + 256 * u, rr = c0 + (it >> 4), ch = it & 15;
                kv[u] = zero4;
                vv[u] = zero4;
                if (it < nc * 16 && rr < n_seg) {
                    const int src = s_src[rr];
                    kv[u] = *(const u32x4_t *)(kb + (int64_t)src * p.k_r + ch * 8);
                    vv[u] = *(const u32x4_t *)(vb + (int64_t)src * p.v_r + ch * 8);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int it = it0 + 256 * u, lr = it >> 4, ch = it & 15;
                if (it < nc * 16) {
                    const int rank = base + c0 + lr, tl = rank / IMG_BN, row = rank % IMG_BN;
                    *(u32x4_t *)(pair_img + (size_t)tl * IMG_KV_BYTES + row * (IMG_SK * 2) + ch * 16) = scale8<T>(kv[u], p.scale_log2);
                    uint32_t *sv = (uint32_t *)(s_v + lr * VT_PITCH + ch * 8);
#pragma unroll
                    for (int e = 0; e < 4; e++) sv[e] = vv[u][e];
                }
            }
        }
        __syncthreads();
        const int r_lo = base + c0, r_hi = r_lo + nc;  // ranks of this chunk
        const int o_lo = r_lo >> 3, n_oct = ((r_hi + 7) >> 3) - o_lo;
        for (int i = tid; i < n_oct * 128; i += 256) {
            const int d = i / n_oct, rank0 = (o_lo + (i - d * n_oct)) * 8;
            uint16_t *dst = (uint16_t *)(pair_img + (size_t)(rank0 / IMG_BN) * IMG_KV_BYTES + IMG_K_BYTES) + d * IMG_SVT + rank0 % IMG_BN;
            if (rank0 >= r_lo && rank0 + 8 <= r_hi) {
                const uint16_t *src = s_v + (rank0 - r_lo) * VT_PITCH + d;
                u32x4_t w;
#pragma unroll
                for (int e = 0; e < 4; e++) w[e] = (uint32_t)src[(2 * e) * VT_PITCH] | ((uint32_t)src[(2 * e + 1) * VT_PITCH] << 16);
                *(u32x4_t *)dst = w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++)
                    if (rank0 + e >= r_lo && rank0 + e < r_hi) dst[e] = s_v[(rank0 + e - r_lo) * VT_PITCH + d];
            }
        }
        __syncthreads();
    }
    for (int it = tid; it < (n_seg + n_pad) * nfb; it += 256) {
        const int gi = it / (n_seg + n_pad), rr = it - gi * (n_seg + n_pad);
        const int rank = base + rr, tl = rank / IMG_BN, row = rank % IMG_BN;
        const bool real = rr < n_seg;
        const int hfb = Hfb == p.H ? hk * G + gi : hk;
        float v = 0.f;
        if (real && p.bias) {
            const int hb = p.Hb == p.H ? hfb : (p.Hb == 1 ? 0 : kv_head(p, hk));
            const uint32_t braw = it == tid ? braw0 : (uint32_t)((const uint16_t *)p.bias)[b * p.bi_b + hb * p.bi_h + s_src[rr]];
            v = E::lo(braw) * kLog2e;
        }
        if (real) fb[((size_t)b * Hfb + hfb) * ld + rank] = v;
        const u32x2_t pc = split3<T>(v);
        u32x4_t xrow;
        xrow[0] = pc[0];
        xrow[1] = pc[1] | (E::pack2(0.f, real ? 0.f : -INFINITY) & 0xffff0000u);
        xrow[2] = E::pack2(E::kRefWeight, 1.f);
        xrow[3] = 0;
        char *xr = img_x + (((size_t)b * Hfb + hfb) * tiles + tl) * IMG_X_BYTES + row * 32;
        *(u32x4_t *)xr = xrow;
        *(u32x4_t *)(xr + 16) = zero4;
    }
}

// Gradient rows (dK, dV) and columns (dBias) of dropped keys: no workgroup of the compacted backward
// owns them, and the operator's contract is that they come back as zeros.
__device__ __forceinline__ void zero_block(const BwdParams &p, bool dbias_direct, int block_x, int pair) {
    const FwdParams &f = p.f;  // (the caller's tensors: the mask is the original one)
    const int b = pair / f.Hk, hk = pair % f.Hk;
    const int hm = f.Hm == 1 ? 0 : hk;
    const uint8_t *mrow = f.mask + b * f.m_b + hm * f.m_h;
    const int c0 = block_x * GATHER_KEYS;
    const int tid = threadIdx.x;
    const int CH = f.d / 8;
    uint16_t *dkb = (uint16_t *)p.dk + b * p.dk_b + hk * p.dk_h;
    uint16_t *dvb = (uint16_t *)p.dv + b * p.dv_b + hk * p.dv_h;
    const u32x4_t z = {0, 0, 0, 0};
    for (int it = tid; it < GATHER_KEYS * CH; it += 256) {
        const int rr = it / CH, ch = it - rr * CH;
        const int key = c0 + rr;
        if (key < f.Lk && !mrow[key]) {
            *(u32x4_t *)(dkb + (int64_t)key * p.dk_r + ch * 8) = z;
            *(u32x4_t *)(dvb + (int64_t)key * p.dv_r + ch * 8) = z;
        }
    }
    if (dbias_direct) {
        const int G = f.H / f.Hk;
        const int nh = f.Hb == f.H ? G : 1;
        for (int it = tid; it < GATHER_KEYS * nh; it += 256) {
            const int gi = it / GATHER_KEYS, key = c0 + (it - gi * GATHER_KEYS);
            if (key < f.Lk && !mrow[key]) {
                const int hb = f.Hb == f.H ? hk * G + gi : (f.Hb == 1 ? 0 : hk);
                ((uint16_t *)p.dbias)[b * p.db_b + hb * p.db_h + key] = 0;
            }
        }
    }
}

// One workgroup: prefix of 128-key units over the pairs, the split the dK/dV kernel will use and, when units are
// split, the per-XCD lists of the parts that exist.  `slots`: workgroups of the dK/dV kernel the device holds at a
// time; `cap`: entries a per-XCD list has room for (that kernel's workgroups per XCD).
__device__ __forceinline__ void plan_block(const int32_t *count, const int32_t *idx, int ld, int32_t *plan, int pairs, int G,
                                           int Lq, int Lk, int causal, int slots, int cap) {
    constexpr int MAXU = DKDV_ENOUGH_UNITS;  // units are split only below this many (and there are no more pairs than units)
    constexpr int MAXL = 1024;               // ... and with at most this many unit lists (LDS: every block of the launch pays for it)
    __shared__ int s_sum, s_max, s_n[256], s_units;
    __shared__ int s_Gs, s_Sm, s_Q, s_fit, s_q1, s_parts2, s_over2;
    __shared__ int s_first[MAXU + 1], s_nt[MAXU], s_len[MAXU], s_nseg[MAXU], s_uoff[MAXU], s_lcount[MAXL], s_cand[64][8];
    const int tid = threadIdx.x;
    // units per pair and their prefix: the counts are fetched 256 at a time by all threads (one memory latency per
    // chunk instead of one per pair), the prefix over a chunk is then taken from LDS by one thread
    int u = 0, n_max = 0;  // (meaningful in thread 0)
    for (int base = 0; base < pairs; base += 256) {
        if (base + tid < pairs) s_n[tid] = (count[base + tid] + 127) / 128;
        __syncthreads();
        if (tid == 0) {
            const int m = pairs - base < 256 ? pairs - base : 256;
            for (int i = 0; i < m; i++) {
                plan[DKDV_PLAN_HDR + base + i] = u;
                if (base + i < MAXU) s_first[base + i] = u;
                u += s_n[i];
                n_max = s_n[i] > n_max ? s_n[i] : n_max;
            }
        }
        __syncthreads();
    }
    if (tid == 0) {
        plan[DKDV_PLAN_HDR + pairs] = u;
        plan[0] = u;
        plan[6] = 0;  // set below when a per-XCD list does not hold all of its parts
        plan[3] = dkdv_list_len(n_max, dkdv_lists_per_pair(pairs));
        if (pairs <= MAXU) s_first[pairs] = u;
        s_units = u;
        s_sum = 0;
        s_max = 0;
    }
    __syncthreads();
    const int U = s_units;
    int Gs0, Sm0;
    dkdv_split(U, G, Gs0, Sm0);
    if (Gs0 * Sm0 <= 1 || pairs >= MAXU || pairs * dkdv_lists_per_pair(pairs) > MAXL) {  // no split (or hardly any pair with keys): nothing else to plan
        if (tid == 0) { plan[1] = 1; plan[2] = 1; plan[4] = 1 << 30; }
        return;
    }
    // From here on U < MAXU, hence pairs < MAXU and (pairs being at most 256 then or not) every count is in reach:
    // thread g works on unit g.  Its pair: the last one that starts at or before g.
    auto pair_of = [&](int g) -> int {
        int lo = 0, hi = pairs;  // s_first[lo] <= g < s_first[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (s_first[mid] <= g) lo = mid; else hi = mid;
        }
        return lo;
    };
    // query blocks per unit: their sum sizes the parts, their maximum the number of segment slots
    int sum = 0, mx = 0;
    for (int g = tid; g < U; g += 256) {
        const int i = pair_of(g);
        const int nt = dkdv_query_blocks(Lq, Lk, causal, idx[(size_t)i * ld + (g - s_first[i]) * 128]);
        s_nt[g] = nt;
        sum += nt;
        mx = nt > mx ? nt : mx;
    }
    atomicAdd(&s_sum, sum);
    atomicMax(&s_max, mx);
    __syncthreads();
    if (tid == 0) {
        int Q = 1 << 30, fit = 1;
        if (Sm0 > 1) {
            const int64_t even = ((int64_t)G * s_sum + DKDV_TARGET_PARTS - 1) / DKDV_TARGET_PARTS;
            fit = (s_max + Sm0 - 1) / Sm0;  // Sm slots must cover the longest unit
            if (fit < 1) fit = 1;
            Q = (int)(even > fit ? even : fit);
        }
        s_Gs = Gs0; s_Sm = Sm0; s_Q = Q; s_fit = fit;
        s_q1 = 1 << 30;
        s_parts2 = 0;
        s_over2 = 0;
    }
    if (tid < 64) {
#pragma unroll
        for (int e = 0; e < 8; e++) s_cand[tid][e] = 0;
    }
    __syncthreads();
    const int k = dkdv_lists_per_pair(pairs);
    // Segment length.  Q above gives about DKDV_TARGET_PARTS parts, i.e. more than one round of workgroups: with
    // parts of unequal length (many units, few segments each) the short ones fill the gaps behind the long ones, but
    // nearly equal parts queue up in whole rounds and the last one is mostly empty.  So the smallest Q whose parts all
    // fit the device at once is looked for as well (the number of parts falls with Q), and the two are compared by an
    // estimate of the time of the last workgroup, in query blocks: one round ends with its longest part; several
    // rounds take the even share plus about half a longest part (measured), and every round pays the start-up and the
    // partial-result write of a workgroup (about 2.5 blocks).  64 candidates (the last one is Q itself), four
    // threads each: a thread takes every fourth unit and adds the parts it finds to the candidate's eight XCD counters
    // (the dK/dV kernel deals the units of a pair to k lists, dkdv_list_of, and the lists to the XCDs).
    if (Sm0 > 1) {
        const int Sm = Sm0, fit = s_fit;
        const int cand = tid & 63, quarter = tid >> 6;
        const int step = (s_max - fit + 61) / 62 > 0 ? (s_max - fit + 61) / 62 : 1;
        const int Qc = cand == 63 ? s_Q : fit + cand * step;
        const float rq = 1.0f / (float)Qc;
        int c[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int i = 0;
        for (int g = quarter; g < U; g += 4) {
            while (s_first[i + 1] <= g) i++;
            const int x = (i * k + dkdv_list_of(g - s_first[i], k)) & 7;
            // ceil(nt / Qc), exactly: the half keeps the float quotient off the integers
            int ns = (int)(((float)(s_nt[g] + Qc - 1) + 0.5f) * rq);
            ns = ns < Sm ? ns : Sm;
#pragma unroll
            for (int e = 0; e < 8; e++) c[e] += x == e ? ns : 0;
        }
#pragma unroll
        for (int e = 0; e < 8; e++) if (c[e]) atomicAdd(&s_cand[cand][e], c[e]);
        __syncthreads();
        if (tid < 64) {
            int worst = 0, parts = 0;
#pragma unroll
            for (int e = 0; e < 8; e++) { worst = s_cand[tid][e] > worst ? s_cand[tid][e] : worst; parts += s_cand[tid][e]; }
            if (tid == 63) { s_parts2 = parts * Gs0; s_over2 = worst * Gs0 * 8 > slots; }  // (more than one round on some XCD)
            else if (worst * Gs0 * 8 <= slots) atomicMin(&s_q1, Qc);
        }
    }
    __syncthreads();
    if (tid == 0) {
        int Sm = Sm0, Q = s_Q;
        if (Sm > 1) {
            if (s_over2 && s_q1 < (1 << 30)) {
                const int r = (s_parts2 + slots - 1) / slots;
                const float rounds = (float)(r < 2 ? 2 : r);
                const float several = (float)Gs0 * (float)s_sum / (float)slots + 0.45f * (float)Q + 2.5f * rounds;
                const float one = (float)s_q1 + 2.5f;
                if (one < several) Q = s_q1;
            }
            if (Q < 1) Q = 1;
            Sm = dkdv_segments(s_max, Q, Sm);
            if (Sm < 1) Sm = 1;
        }
        plan[1] = Gs0;
        plan[2] = Sm;
        plan[4] = Q;
        plan[5] = DKDV_PLAN_HDR + pairs + 1;  // where the lists begin
        s_Q = Q; s_Sm = Sm;
    }
    const int n_lists = pairs * k;  // a multiple of 8, at most MAXL
    for (int vl = tid; vl < n_lists; vl += 256) s_lcount[vl] = 0;
    __syncthreads();
    // The parts that exist, per XCD: list after list (an XCD holds every eighth list); inside a list the units with
    // the longest parts first (all parts of a unit are equally long: its query blocks cut into equal segments), the
    // parts of a unit side by side.  The kernel's workgroups start in this order: the short ones fill the gaps at the
    // end.  Which units a list holds stays as dealt -- that balances the lists; only their order inside it is by length.
    const int Q = s_Q, Sm = s_Sm;
    for (int g = tid; g < U; g += 256) {
        const int n_seg = dkdv_segments(s_nt[g], Q, Sm);
        s_nseg[g] = n_seg;
        s_len[g] = n_seg > 0 ? (s_nt[g] + n_seg - 1) / n_seg : 0;
    }
    __syncthreads();
    for (int g = tid; g < U; g += 256) {
        const int i = pair_of(g), first = s_first[i], n = s_first[i + 1] - first, un = g - first;
        const int mine = s_len[g], fold = dkdv_list_of(un, k);
        int before = 0;  // parts of the units of the same list that come first
        for (int v = 0; v < n; v++) {
            const bool first_v = dkdv_list_of(v, k) == fold && (s_len[first + v] > mine || (s_len[first + v] == mine && v < un));
            before += first_v ? s_nseg[first + v] : 0;
        }
        s_uoff[g] = Gs0 * before;
        atomicAdd(&s_lcount[i * k + fold], Gs0 * s_nseg[g]);
    }
    __syncthreads();
    int32_t *lists = plan + DKDV_PLAN_HDR + pairs + 1;
    if (tid < 8) {
        int off = 0;
        for (int vl = tid; vl < n_lists; vl += 8) {
            const int t = s_lcount[vl];
            s_lcount[vl] = off;  // from here on: where the list begins in its XCD's entries
            off += t;
        }
        lists[tid] = off < cap ? off : cap;  // (the grid is sized for every part: off <= cap)
        // Should that ever not hold, parts would be missing from the sums: say so, and the reduce kernel turns the
        // gradients of the whole call into NaN instead of handing out sums with parts left out.
        if (off > cap) plan[6] = 1;
    }
    __syncthreads();
    for (int g = tid; g < U; g += 256) {
        const int i = pair_of(g), un = g - s_first[i], vl = i * k + dkdv_list_of(un, k), ns = s_nseg[g];
        int o = s_lcount[vl] + s_uoff[g];
        int32_t *e = lists + 8 + 2 * ((size_t)(vl & 7) * cap);
        for (int gi = 0; gi < Gs0; gi++)
            for (int sg = 0; sg < ns; sg++) {
                if (o < cap) {
                    e[2 * o] = i;
                    e[2 * o + 1] = un | ((gi * Sm + sg) << 16);
                }
                o++;
            }
    }
}

// Everything the compacted backward needs after the scan, in one launch: layer 0 of the grid gathers K / V rows,
// layer 1 clears the gradients of dropped keys, one workgroup of layer 2 makes the dK/dV plan, and the layers from 3
// on compute D = rowsum(dO * O), which depends on none of the others.
// The plan is a chain of dependent steps of a single workgroup (18 us); side by side with the other two it costs nothing.
template <typename T>
__global__ void __launch_bounds__(256) compact_bwd_prepass_kernel(const BwdParams bp, const int32_t *idx, int32_t *cnt,
                                                                   const int32_t *count, float *fb, uint16_t *kc, uint16_t *vc,
                                                                   int ld, int Hfb, int32_t *plan, int slots, int cap, int do_gather) {
    const FwdParams &f = bp.f;
    if (blockIdx.z == 0) {
        // (not when the lists and copies exist already: made by an earlier launch, or by the forward call)
        if (do_gather) gather_block<T>(f, idx, cnt, count, fb, kc, vc, ld, Hfb, blockIdx.x, blockIdx.y, do_gather == 2);
    } else if (blockIdx.z == 1) {
        zero_block(bp, bp.dbias != nullptr && bp.dbias_accum == nullptr, blockIdx.x, blockIdx.y);
    } else if (blockIdx.z == 2) {
        if (blockIdx.x == 0 && blockIdx.y == 0)
            plan_block(count, idx, ld, plan, f.B * f.Hk, f.H / f.Hk, f.Lq, f.Lk, f.causal, slots, cap);
    } else {  // the blocks of D = rowsum(dO * O), laid out over the remaining layers
        const int nbx = (bp.Lq_rounded + bwd_dot_rows_per_block(f.d) - 1) / bwd_dot_rows_per_block(f.d);
        const int64_t lin = ((int64_t)(blockIdx.z - 3) * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        if (lin >= (int64_t)nbx * f.H * f.B) return;
        bwd_dot_block<T>(bp, (int)(lin % nbx), (int)((lin / nbx) % f.H), (int)(lin / ((int64_t)nbx * f.H)));
    }
}

}  // namespace

bool compact_per_query_head(const FwdParams &p, FwdParams &pv) {
    if (!p.mask || p.m_r != 0 || p.Hm != p.H || p.Hk <= 0 || p.H == p.Hk) return false;
    pv = p;
    pv.kv_share = p.H / p.Hk;
    pv.Hk = p.H;
    return use_compact(pv);
}

bool use_compact(const FwdParams &p) {
    const int mode = p.compact_mode;  // 0 = when it pays, 1 = never, 2 = whenever the mask form allows it
    if (mode == 1 || !p.mask || p.m_r != 0) return false;
    if (p.bias && p.bi_r != 0) return false;
    if (!(p.Hm == 1 || p.Hm == p.Hk)) return false;
    if (p.Lq < 2 || p.Lk < 1 || (int64_t)p.Lk * p.d >= (int64_t)1 << 31) return false;
    if ((int64_t)p.B * p.Hk > 65535) return false;  // (the pre-pass launches carry the pair in the grid's y dimension)
    if (mode == 2) return true;
    // the pre-pass costs about one copy of K and V plus a small launch or two; it pays once the attention
    // itself is a few million (query, key) pairs per kv head
    return p.Lq >= 128 && p.Lk >= 128 && (int64_t)p.Lq * (p.H / p.Hk) * p.Lk >= (int64_t)1 << 21;
}

size_t compact_bytes(const FwdParams &p, bool backward, bool reuse_fwd) {
    const Layout l = layout_of(p, backward);
    // (with the forward's workspace: plan and partial sums only -- and the row-major copies when the forward's are images)
    return backward && reuse_fwd ? l.total - (l.img ? l.off_bk : l.off_plan) : l.total;
}

// compute units of the current device (cached per device)
static int device_cus() {
    static std::atomic<int> cus[16];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 256;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

hipError_t compact_setup(FwdParams &p, void *ws, int dtype, hipStream_t stream, BwdParams *bp, const void *fwd_ws) {
    const Layout l = layout_of(p, bp != nullptr);
    // the lists and the K / V copies: in this call's workspace, or (backward) where the forward call left them
    char *w = fwd_ws ? const_cast<char *>(static_cast<const char *>(fwd_ws)) : static_cast<char *>(ws);
    // what only the backward has (its row-major copies when the forward's are tile images, the plan, the partial
    // sums): behind the forward part, or alone in `ws` when that part is the forward call's
    char *wb = fwd_ws ? static_cast<char *>(ws) - (l.img ? l.off_bk : l.off_plan) : static_cast<char *>(ws);
    int32_t *idx = (int32_t *)(w + l.off_idx), *cnt = (int32_t *)(w + l.off_cnt), *count = (int32_t *)(w + l.off_count);
    float *fb = (float *)(w + l.off_fb);
    // row-major copies: the backward's own when the forward part holds images
    uint16_t *kc = (uint16_t *)(l.img ? wb + l.off_bk : w + l.off_k), *vc = (uint16_t *)(l.img ? wb + l.off_bv : w + l.off_v);
    const int pairs = p.B * p.Hk;
    hipError_t e;
    if (l.img && !bp) {
        // forward on tile images: lists, fused bias and images in one launch
        char *img_kv = w + l.off_k, *img_x = w + l.off_v;
        if (p.kept_idx) {  // lists handed over: a workgroup per tile copies its part of them and builds the tile
            const dim3 igrid(p.Lk / IMG_BN + 1, pairs);
            if (dtype == 0)
                hipLaunchKernelGGL((compact_image_kernel<bf16_tag>), igrid, dim3(256), 0, stream, p, idx, cnt, count, fb, img_kv, img_x, l.ld, l.Hfb, l.img_tiles);
            else
                hipLaunchKernelGGL((compact_image_kernel<fp16_tag>), igrid, dim3(256), 0, stream, p, idx, cnt, count, fb, img_kv, img_x, l.ld, l.Hfb, l.img_tiles);
        } else {           // a plain mask: a workgroup per SEG_KEYS original columns
            const dim3 sgrid((l.ld + SEG_KEYS - 1) / SEG_KEYS, pairs);
            if (dtype == 0)
                hipLaunchKernelGGL((compact_scan_image_kernel<bf16_tag>), sgrid, dim3(256), 0, stream, p, idx, cnt, count, fb, img_kv, img_x, l.ld, l.Hfb, l.img_tiles);
            else
                hipLaunchKernelGGL((compact_scan_image_kernel<fp16_tag>), sgrid, dim3(256), 0, stream, p, idx, cnt, count, fb, img_kv, img_x, l.ld, l.Hfb, l.img_tiles);
        }
        if ((e = hipGetLastError()) != hipSuccess) return e;
        p.cmp.idx = idx;
        p.cmp.cnt = cnt;
        p.cmp.count = count;
        p.cmp.fb = fb;
        p.cmp.ld = l.ld;
        p.cmp.Hfb = l.Hfb;
        p.cmp.on = 1;
        p.cmp.img_kv = img_kv;
        p.cmp.img_x = img_x;
        p.cmp.img_tiles = l.img_tiles;
        return hipSuccess;
    }
    const bool have_lists = fwd_ws != nullptr || p.kept_idx != nullptr;
    // forward without lists: scan and gather in one launch -- up to 65536 keys: every workgroup of that launch counts the
    // mask bytes in front of its segment, Lk / 2 of them on average, which grows with the square of Lk per pair
    const bool fused_scan = !have_lists && !bp && p.Lk <= (1 << 16);
    if (fused_scan) {
        const dim3 sgrid((l.ld + SEG_KEYS - 1) / SEG_KEYS, pairs);
        if (dtype == 0)
            hipLaunchKernelGGL((compact_scan_gather_kernel<bf16_tag>), sgrid, dim3(256), 0, stream, p, idx, cnt, count, fb, kc, vc, l.ld, l.Hfb);
        else
            hipLaunchKernelGGL((compact_scan_gather_kernel<fp16_tag>), sgrid, dim3(256), 0, stream, p, idx, cnt, count, fb, kc, vc, l.ld, l.Hfb);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    } else if (!have_lists) {
        hipLaunchKernelGGL(compact_scan_kernel, dim3(pairs), dim3(SCAN_THREADS), 0, stream, p, idx, cnt, count, l.ld);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    const dim3 grid((p.Lk + GATHER_KEYS - 1) / GATHER_KEYS, pairs);
    // (handed-over lists: the gather launch also copies them into the per-pair arrays, which the backward's other
    // pre-pass layers read -- so it runs on its own in front of them)
    const bool gather_alone = !bp || (p.kept_idx != nullptr && !fwd_ws);
    if (gather_alone && !fwd_ws && !fused_scan) {
        if (dtype == 0)
            hipLaunchKernelGGL((compact_gather_kernel<bf16_tag>), grid, dim3(256), 0, stream, p, idx, cnt, count, fb, kc, vc, l.ld, l.Hfb);
        else
            hipLaunchKernelGGL((compact_gather_kernel<fp16_tag>), grid, dim3(256), 0, stream, p, idx, cnt, count, fb, kc, vc, l.ld, l.Hfb);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    if (bp) {
        // (p is bp->f, still describing the caller's tensors here)
        int32_t *plan = (int32_t *)(wb + l.off_plan);
        int dkdv_grid, slots;
        dkdv_split_bounds(pairs, (p.Lk + 127) / 128, p.H / p.Hk, dkdv_grid, slots);
        const int plan_cap = dkdv_grid / 8;  // entries per XCD list: the dK/dV kernel's workgroups per XCD
        const int dot_rows = bwd_dot_rows_per_block(p.d);
        const int64_t dot_blocks = (int64_t)((bp->Lq_rounded + dot_rows - 1) / dot_rows) * p.H * p.B;
        const int64_t layer = (int64_t)grid.x * pairs;
        const int64_t dot_layers = (dot_blocks + layer - 1) / layer;
        const bool with_dot = p.cu_q == nullptr && 3 + dot_layers <= 65535;
        const dim3 grid3(grid.x, pairs, with_dot ? (unsigned)(3 + dot_layers) : 3);
        // 0: lists and copies exist; 1: gather here; 2: the lists are the forward call's, whose copies are tile images --
        // only the row-major K / V copies are made here
        const int do_gather = fwd_ws ? (l.img ? 2 : 0) : (gather_alone ? 0 : 1);
        if (dtype == 0)
            hipLaunchKernelGGL((compact_bwd_prepass_kernel<bf16_tag>), grid3, dim3(256), 0, stream, *bp, idx, cnt, count, fb, kc, vc,
                               l.ld, l.Hfb, plan, 2 * device_cus(), plan_cap, do_gather);
        else
            hipLaunchKernelGGL((compact_bwd_prepass_kernel<fp16_tag>), grid3, dim3(256), 0, stream, *bp, idx, cnt, count, fb, kc, vc,
                               l.ld, l.Hfb, plan, 2 * device_cus(), plan_cap, do_gather);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        bp->dot_done = with_dot ? 1 : 0;
        p.cmp.plan = plan;
        bp->dkv_part = (float *)(wb + l.off_part_kv);
        bp->db_part = (float *)(wb + l.off_part_db);
    }
    p.k = kc;
    p.v = vc;
    p.k_r = p.v_r = p.d;
    p.k_h = p.v_h = (int64_t)p.Lk * p.d;
    p.k_b = p.v_b = (int64_t)p.Hk * p.Lk * p.d;
    p.cmp.idx = idx;
    p.cmp.cnt = cnt;
    p.cmp.count = count;
    p.cmp.fb = fb;
    p.cmp.ld = l.ld;
    p.cmp.Hfb = l.Hfb;
    p.cmp.on = 1;
    return hipSuccess;
}


}  // namespace fdma
