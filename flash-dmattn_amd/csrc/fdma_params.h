// Kernel argument blocks (device side) and the launch functions each .hip file exports to the
// C-ABI layer in fdma_api.cpp.  Plays the role of the reference's Flash_fwd_params /
// Flash_bwd_params (csrc/flash_sparse_attn/src/flash.h:20-198) without any torch types.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace fdma {

// Column compaction for keep-masks that are broadcast over queries: the kept keys of every
// (batch, kv head) pair are gathered, in ascending column order, into dense copies of K and V, and the
// main kernels then run over `count` keys instead of Lk.  Causal masking compares against the number of
// kept columns a query can see (`cnt`), and gradients are written back through `idx`.
struct Compact {
    const int32_t *idx;    // (B*Hk, ld): original column of compacted key c, c < count
    const int32_t *cnt;    // (B*Hk, ld): kept keys among the original columns 0..j (inclusive)
    const int32_t *count;  // (B*Hk): kept keys
    const float *fb;       // (B*Hfb, ld): bias * log2(e) of compacted key c (0 without a bias)
    const int32_t *plan;   // backward only: work split of the dK/dV kernel, see DkdvPlan
    int32_t ld;            // row stride of the arrays above (Lk rounded up to 16)
    int32_t Hfb;           // heads of fb: Hk, or H when the bias differs per query head
    int32_t on;            // 0 = no compaction: k / v are the caller's tensors
    // Tile images (forward at head dim 128 on large grids, see fwd_stream_applicable): instead of row-major copies the
    // pre-pass writes, per 64-key tile of the compacted key axis, exactly the bytes the forward kernel keeps in LDS --
    // the K tile with padded rows (times softmax_scale * log2(e)) followed by V already transposed (img_kv, IMG_KV_BYTES per tile, img_tiles tiles per
    // (batch, kv head) pair) and the 16-element side rows of the keys (img_x, IMG_X_BYTES per tile, per (batch, fb
    // head)) -- so that the forward fetches a tile with contiguous global->LDS loads.  nullptr = row-major copies.
    const char *img_kv;
    const char *img_x;
    int32_t img_tiles;
};
constexpr int IMG_BN = 64;                                // keys per tile image
constexpr int IMG_SK = 128 + 8, IMG_SVT = IMG_BN + 8;     // row strides (elements) of the K tile and of V^T
constexpr int IMG_K_BYTES = IMG_BN * IMG_SK * 2;          // 17408
constexpr int IMG_VT_BYTES = 128 * IMG_SVT * 2;           // 18432
constexpr int IMG_KV_BYTES = IMG_K_BYTES + IMG_VT_BYTES;  // 35840 = 35 pieces of 1 KB
constexpr int IMG_X_BYTES = IMG_BN * 32;                  // 2048

// Work split of the compacted dK/dV kernel, made on the device once the kept-key counts are known.
// A unit is one 128-key block of one (batch, kv head) pair; U = number of units.  With few units the
// chip would idle (the kernel keeps K / V stationary and loops over query heads and query blocks), so
// every unit is split over `Gs` groups of query heads and, once every head has its own group, over
// segments of at most `Q` query blocks (a unit that fewer queries see gets fewer segments, so that parts
// are of similar size); each part writes fp32 partial results that a reduce kernel sums in a fixed order.
// Units go to the 8 XCDs (workgroup id % 8) pair by pair so that workgroups sharing an L2 stream the same
// Q / dO tiles; with fewer than 8 pairs (or a pair count that 8 does not divide) a pair is folded into
// k = 8 / gcd(pairs, 8) lists, unit u going to list snake(u mod 2k) -- low key blocks see the most queries
// under a causal mask, and the fold gives every list the same mix of heavy and light units.
//   plan[0] = U, plan[1] = Gs, plan[2] = Sm (segment slots per unit and head group), plan[3] = list length
//   bound (units), plan[4] = Q, plan[5] = where the lists begin, plan[6] = 1 when a per-XCD list overflowed (the
//   reduce kernel then writes NaN gradients), plan[8 + i] = first unit of pair i (i = 0..pairs)
constexpr int DKDV_PLAN_HDR = 8;
#ifndef FDMA_DKDV_TARGET
#define FDMA_DKDV_TARGET 768
#endif
constexpr int DKDV_TARGET_PARTS = FDMA_DKDV_TARGET;   // parts wanted (3 per CU, two of them resident at a time: measured best)
constexpr int DKDV_ENOUGH_UNITS = 384;    // from here on the units alone fill the chip
__host__ __device__ inline void dkdv_split(int U, int G, int &Gs, int &Sm) {
    Gs = 1;
    Sm = 1;
    if (U <= 0 || U >= DKDV_ENOUGH_UNITS) return;
    const int want = (DKDV_TARGET_PARTS + U - 1) / U;
    for (int c = 2; c <= G && c <= want; c++)
        if (G % c == 0) Gs = c;  // query heads first: largest divisor of G not above `want`
    if (Gs == G) {  // upper bound of the segments per unit: twice the even split, units differ in length
        Sm = 2 * want / G;
        Sm = Sm < 1 ? 1 : (Sm > 16 ? 16 : Sm);
    }
}
// query blocks (of 64 rows) that see a key block whose first key sits at original column `okey_first`
__host__ __device__ inline int dkdv_query_blocks(int Lq, int Lk, int causal, int okey_first) {
    const int M_blocks = (Lq + 63) / 64;
    int m_start = 0;
    if (causal) {
        const int first_q = okey_first - (Lk - Lq);
        if (first_q > 0) m_start = first_q / 64;
        if (m_start > M_blocks) m_start = M_blocks;
    }
    return M_blocks - m_start;
}
// segments a unit with n_tot query blocks is cut into
__host__ __device__ inline int dkdv_segments(int n_tot, int Q, int Sm) {
    const int s = (n_tot + Q - 1) / Q;
    return s < Sm ? s : Sm;
}

__host__ __device__ inline int dkdv_lists_per_pair(int pairs) {
    return pairs % 8 == 0 ? 1 : (pairs % 4 == 0 ? 2 : (pairs % 2 == 0 ? 4 : 8));
}
// The units of a pair are dealt to its k lists in a snake (0 .. k-1, k-1 .. 0, ...): position `pos` of list `fold`
// holds unit dkdv_unit_at(pos, fold, k); unit u sits in list dkdv_list_of(u, k).
__host__ __device__ inline int dkdv_unit_at(int pos, int fold, int k) {
    return 2 * k * (pos >> 1) + ((pos & 1) ? 2 * k - 1 - fold : fold);
}
__host__ __device__ inline int dkdv_list_of(int u, int k) {
    const int rem = u % (2 * k);
    return rem < k ? rem : 2 * k - 1 - rem;
}
__host__ __device__ inline int dkdv_list_len(int units_in_largest_pair, int k) {
    return 2 * ((units_in_largest_pair + 2 * k - 1) / (2 * k));
}

struct FwdParams {
    const void *q, *k, *v;
    const uint8_t *mask;  // nullptr = absent
    const void *bias;     // nullptr = absent
    void *o;
    float *lse;           // element (b, h, row) at b * lse_b + h * lse_h + first row of b + row
    int64_t lse_b, lse_h; // (B, H, Lq): H * Lq, Lq; ragged batch (H, total_q): 0, total_q
    // Ragged batch (the reference's "varlen" layout, csrc/flash_sparse_attn/flash_api.cpp:556-790): q / k / v hold the
    // sequences back to back, (total rows, heads, d), batch entry b owns rows cu[b] .. cu[b + 1] - 1 and the batch
    // strides are 0.  Lq / Lk below are then the longest sequences (they size the grids).  nullptr = fixed lengths.
    const int32_t *cu_q, *cu_k;
    int32_t total_q, total_k;  // rows of the ragged q / k tensors
    int64_t q_b, q_r, q_h;
    int64_t k_b, k_r, k_h;
    int64_t v_b, v_r, v_h;
    int64_t o_b, o_r, o_h;
    int64_t m_b, m_h, m_r;  // mask strides (batch, head, row); 0 = broadcast
    int64_t bi_b, bi_h, bi_r;
    int32_t B, Lq, Lk, H, Hk, Hm, Hb, d;
    int32_t causal;
    float scale;        // softmax scale
    float scale_log2;   // scale * log2(e)
    // split-KV decode
    float *o_part;      // (splits, B, H, Lq, d) fp32
    float *lse_part;    // (splits, B, H, Lq) fp32, natural log, -inf for an empty split
    int32_t splits;
    // split-KV decode in one launch: one arrival counter per (batch entry, workgroup row of the grid), zero on entry and
    // left zero (fdma_fwd_args.counters of the C ABI); nullptr = the merge is a launch of its own
    int32_t *dec_counter;
    int32_t compact_mode;  // FDMA_COMPACT_* of the C ABI: 0 = decide from the problem, 1 = never, 2 = whenever the mask form allows
    Compact cmp;        // when cmp.on, k / v (and their strides) describe the compacted copies
    // kept-column lists handed over by the caller (fdma_kept_keys of the C ABI; nullptr = scan the mask): one row per
    // (mask batch entry, mask head)
    const int32_t *kept_idx, *kept_cnt, *kept_count;
    int32_t kept_ld;
    // Forward compaction for a query-broadcast mask with one row per QUERY head (Hm == H > kv heads): every query head
    // keeps its own keys, so the heads of a kv group share no compacted K / V.  The compaction layer then sees H "kv
    // heads" (Hk == H above, one compacted copy per query head) and finds the caller's K / V / bias head of such a head
    // by dividing by kv_share (= query heads per real kv head).  0 or 1: heads are what they say.
    int32_t kv_share;
    // the mask packed to one bit per key (fdma_mask_bits of the C ABI; nullptr = read the bool mask): strides in bytes,
    // broadcast like the mask
    const uint8_t *mbits;
    int64_t mb_b, mb_h, mb_r;
};

// the caller's kv head behind head `hk` of the compaction layer (see FwdParams::kv_share)
__host__ __device__ inline int kv_head(const FwdParams &p, int hk) { return p.kv_share > 1 ? hk / p.kv_share : hk; }

// lengths and first rows of batch entry b
struct SeqInfo {
    int32_t Lq, Lk;
    int64_t q0, k0;
};
__device__ inline SeqInfo seq_info(const FwdParams &p, int b) {
    SeqInfo s;
    if (p.cu_q) {
        const int32_t q0 = p.cu_q[b], k0 = p.cu_k[b];
        s.q0 = q0;
        s.k0 = k0;
        s.Lq = p.cu_q[b + 1] - q0;
        s.Lk = p.cu_k[b + 1] - k0;
    } else {
        s.q0 = 0;
        s.k0 = 0;
        s.Lq = p.Lq;
        s.Lk = p.Lk;
    }
    return s;
}

struct BwdParams {
    FwdParams f;  // f.o = forward output (read), f.lse = forward LSE (read)
    const void *dout;
    void *dq, *dk, *dv, *dbias;
    int64_t do_b, do_r, do_h;
    int64_t dq_b, dq_r, dq_h;
    int64_t dk_b, dk_r, dk_h;
    int64_t dv_b, dv_r, dv_h;
    int64_t db_b, db_h, db_r;  // dbias strides (batch, head, row); 0 = broadcast
    float *softmax_d;          // laid out like lse: b * sd_b + h * sd_h + first row of b + row
    int64_t sd_b, sd_h;        // (B, H, Lq_rounded): H * Lq_rounded, Lq_rounded; ragged batch: 0, total_q
    int32_t Lq_rounded;
    float *dbias_accum;        // fp32 scratch at the dbias shape when several workgroups share an element
    int64_t dba_b, dba_h, dba_r;
    // compacted dK/dV kernel, split mode: per part [2][Dpad][128] fp32 (dK^T, dV^T) and [G][128] fp32 (dBias)
    float *dkv_part;
    float *db_part;
    int32_t dot_done;          // softmax_d has been computed by an earlier launch of this call
    int32_t red_octets, red_period, red_start;  // compacted backward: workgroups of the dQ launch that sum the dK/dV partials (set by that launch)
};

// Keep-mask builder (fdma_mask.hip): one row of `Lk` 16-bit bias values per (batch, head, row).
struct MaskParams {
    const void *bias;
    const uint8_t *mask_in;  // nullptr = absent; 0 strides broadcast
    uint8_t *mask_out;
    int64_t bi_b, bi_h, bi_r;
    int64_t mi_b, mi_h, mi_r;
    int64_t mo_b, mo_h, mo_r;
    int32_t batch, heads, rows, Lk;
    int32_t window;      // top-k: entries kept per row
    int32_t block_size;  // > 1: majority vote inside aligned key blocks afterwards
    int32_t type;        // 0 = top-k, 1 = relu
    int32_t dtype;       // 0 = bf16, 1 = fp16
    uint32_t min_bits;   // the fill value for entries the incoming mask excludes, as bits of the bias type
    int32_t *kept_idx, *kept_cnt, *kept_count;  // optional second output (nullptr = not wanted): see scan_mask_row
    int32_t kept_ld;
    uint8_t *bits;           // optional third output (nullptr = not wanted): the mask packed to one bit per key
    int64_t bits_row_bytes;
};
hipError_t launch_make_mask(const MaskParams &p, hipStream_t stream);

// Bias producer (fdma_bias.hip): bias[b, j, 0, l] = A[j] * softplus(V_flat[b, l, :] . W[j, :] + pb[j]).
struct DynBiasParams {
    const void *v;        // (B, L, Hk, d): strides batch / row / head in elements, d contiguous
    const void *w;        // (Hk, Hk * d) row-major
    const void *pb;       // (Hk) or nullptr
    const void *a;        // (Hk)
    void *bias;           // out (forward): element (b, j, l) at b * bias_b + j * bias_h + l
    float *dt;            // (B * L, Hk) fp32: written by forward, read by backward
    int64_t v_b, v_r, v_h;
    int64_t bias_b, bias_h;
    int32_t B, L, Hk, d;
    // backward
    const void *dbias;    // (b, j, l) at b * dbias_b + j * dbias_h + l
    int64_t dbias_b, dbias_h;
    void *dv;             // (B, L, Hk, d), strides below
    int64_t dv_b, dv_r, dv_h;
    void *dw, *da, *dpb;  // (Hk, Hk * d), (Hk), (Hk) or nullptr
    float *part;          // n_wg partials of part_stride floats: dW (Hk * Hk * d), dA (Hk), dpb (Hk)
    int64_t part_stride;
    int32_t n_wg, rows_per_wg;
};
hipError_t launch_dyn_bias_fwd(const DynBiasParams &p, int dtype, hipStream_t stream);
hipError_t launch_dyn_bias_bwd(const DynBiasParams &p, int dtype, hipStream_t stream);
int dyn_bias_bwd_workgroups(int64_t n_rows, int *rows_per_wg);

// Dynamic-LDS limit of a kernel, raised once per device (and again only for a larger request) instead of on every
// launch: one `static DynSmemLimit` per launch site.  Later launches make no runtime call besides the launch itself.
struct DynSmemLimit {
    static constexpr int kDevices = 16;
    std::atomic<int> set_bytes[kDevices] = {};
    hipError_t ensure(const void *kernel, int bytes) {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        const bool tracked = dev >= 0 && dev < kDevices;
        if (tracked && set_bytes[dev].load(std::memory_order_acquire) >= bytes) return hipSuccess;
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e == hipSuccess && tracked) {
            int seen = set_bytes[dev].load(std::memory_order_relaxed);
            while (seen < bytes && !set_bytes[dev].compare_exchange_weak(seen, bytes, std::memory_order_release)) {}
        }
        return e;
    }
};

// dtype: 0 = bf16, 1 = fp16.  All launches are asynchronous on `stream`; return hipError_t.
hipError_t launch_fwd(const FwdParams &p, int dtype, hipStream_t stream);
// column-mask specialisation (mask / bias absent or broadcast over queries); nq = 32-row blocks per wave
bool fwd_colmask_applicable(const FwdParams &p);
hipError_t launch_fwd_colmask(const FwdParams &p, int dtype, hipStream_t stream);
// compacted forward on tile images (fdma_fwd_stream.hip): resident workgroups that walk their share of the
// (query block, head) items with the tiles of the next item already on their way.  `fwd_stream_applicable` decides from
// the problem alone (the pre-pass, the forward and the backward of a problem must agree on the workspace layout).
bool fwd_stream_applicable(const FwdParams &p);
// smallest number of (256-row query block, head) items for which it is taken (process-wide; default 512)
void set_stream_min_items(int n);
int get_stream_min_items();
hipError_t launch_fwd_stream(const FwdParams &p, int dtype, hipStream_t stream);
hipError_t launch_fwd_decode(const FwdParams &p, int dtype, hipStream_t stream);
hipError_t launch_bwd(const BwdParams &p, int dtype, hipStream_t stream);
// column-mask specialisations of the two main backward kernels
bool bwd_colmask_applicable(const BwdParams &p);
hipError_t launch_bwd_dkdv_colmask(const BwdParams &p, int dtype, hipStream_t stream);
hipError_t launch_bwd_dq_colmask(const BwdParams &p, int dtype, hipStream_t stream);
// dQ from the dS tiles that the general dK/dV kernel has written as dBias (a per-query bias with a row per query head
// and batch entry, dBias written directly): one tile GEMM and no second pass over mask, bias, Q, V, dO
bool bwd_dq_from_ds_applicable(const BwdParams &p);
hipError_t launch_bwd_dq_from_ds(const BwdParams &p, int dtype, hipStream_t stream);
// general dQ kernel (mask / bias per query row), fdma_bwd_dq.hip
hipError_t launch_bwd_dq(const BwdParams &p, int dtype, hipStream_t stream);

// Column compaction: use_compact() decides from the problem alone (no device data), compact_bytes() is
// the scratch it needs, compact_setup() launches the gather pre-pass into `ws` and rewrites p.k / p.v /
// p.cmp; for a backward call (bp given) the same launch zero-fills the gradient rows / columns of dropped keys
// and makes the dK/dV plan.
bool use_compact(const FwdParams &p);
// forward only: `p` has a query-broadcast mask with a row per query head and grouped kv heads, and `pv` -- the same
// problem as the compaction layer takes it (see FwdParams::kv_share) -- is one that use_compact() accepts
bool compact_per_query_head(const FwdParams &p, FwdParams &pv);
size_t compact_bytes(const FwdParams &p, bool backward, bool reuse_fwd = false);
// bp != nullptr: backward -- also plans the dK/dV split and sets bp->dkv_part / bp->db_part
// `fwd_ws` (backward only): the workspace a forward call of the same problem filled; its lists and copies are used
// instead of being made again, and `ws` then holds the backward's plan and partial sums alone.
hipError_t compact_setup(FwdParams &p, void *ws, int dtype, hipStream_t stream, BwdParams *bp = nullptr,
                         const void *fwd_ws = nullptr);
// host-side bounds over every possible unit count 1..U_max: workgroups to launch, partial slots to hold
// (n_max = units of one pair at most)
inline void dkdv_split_bounds(int pairs, int n_max, int G, int &grid, int &slots) {
    const int k = dkdv_lists_per_pair(pairs);
    const int lists_per_xcd = pairs * k / 8;
    // n = units of the largest pair; the total U is then between n and pairs * n, and the split factor does
    // not grow with U: the split of U = n bounds the workgroups, U * split(U) bounds the partial slots
    int64_t items = 1, sl = 1;
    for (int n = 1; n <= n_max; n++) {
        int Gs, Sm;
        dkdv_split(n, G, Gs, Sm);
        const int64_t it = (int64_t)dkdv_list_len(n, k) * Gs * Sm;
        if (it > items) items = it;
        if (n >= DKDV_ENOUGH_UNITS) {  // no split from here on: the bound grows with n alone
            const int64_t last = dkdv_list_len(n_max, k);
            if (last > items) items = last;
            break;
        }
    }
    const int U_max = pairs * n_max < DKDV_ENOUGH_UNITS ? pairs * n_max : DKDV_ENOUGH_UNITS - 1;
    for (int U = 1; U <= U_max; U++) {
        int Gs, Sm;
        dkdv_split(U, G, Gs, Sm);
        if (Gs * Sm > 1 && (int64_t)U * Gs * Sm > sl) sl = (int64_t)U * Gs * Sm;
    }
    grid = (int)(8 * lists_per_xcd * items);
    slots = (int)sl;
}

// number of KV splits the decode path uses for this shape (1 = no workspace needed)
int decode_num_splits(int B, int Hk, int Lk);
// arrival counters the one-launch decode needs for this shape (0 without splits)
int64_t decode_num_counters(int B, int H, int Hk, int Lk);
bool use_decode_path(int Lq, int H, int Hk);

}  // namespace fdma
