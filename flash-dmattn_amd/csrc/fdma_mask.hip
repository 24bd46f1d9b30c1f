// Keep-mask builders on the device: the reference's topk_mask / relu_mask / block_smooth
// (flash_sparse_attn/utils/mask.py:47-160) as ONE kernel per call instead of masked_fill + topk + zeros + scatter
// (+ view / sum / copy for the smoothing) through a tensor library.
//
// One workgroup (4 or 16 waves) owns one row of `seqlen_k` bias values (16-bit floats).  The `window` largest are
// found by a two-level radix select on an order-preserving 16-bit key: a 256-bin histogram of the high byte in LDS (one copy per
// LDS bank: the high byte is sign and exponent, so most of a row falls into a handful of bins),
// a wave-parallel suffix scan that finds the bin holding the window-th largest value, the same again for the low
// byte inside that bin.  That yields the exact threshold value T, the number of entries above it and how many
// entries EQUAL to T are still needed; those are taken in ascending column order (the reference's torch.topk leaves
// the choice among equal values unspecified).  HBM traffic is one read of the row (the second and third pass hit in
// L2 / L1) and one write of the mask row.
//
// As in the reference, entries excluded by an incoming mask are pushed to `min_value` before the selection, and a
// selected entry whose value equals `min_value` is not kept; the optional block smoothing then replaces every
// aligned block of `block_size` keys by the majority vote of its entries (a shorter tail block votes over its own
// length; exactly half is dropped).
#include "fdma_common.h"
#include "fdma_params.h"
#include "fdma_scan.h"

namespace fdma {
namespace {


// 16-bit float bits (bf16 or fp16: sign, exponent, mantissa) -> key whose unsigned order is the numeric order
__device__ __forceinline__ uint32_t order_key(uint32_t bits) { return (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u); }

// hist[256] (LDS), k >= 1, sum(hist) >= k.  Wave 0 finds the bin b with count(bins > b) < k <= count(bins >= b) and
// writes {b, count(bins > b)} to res[0..1].  Lane l owns bins 255-4l .. 252-4l.
__device__ __forceinline__ void find_bin(const uint32_t *hist, uint32_t k, uint32_t *res) {
    const int lane = threadIdx.x & 63;
    uint32_t c[4], s = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        c[j] = hist[255 - 4 * lane - j];
        s += c[j];
    }
    uint32_t incl = s;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t t = __shfl_up(incl, off);
        if (lane >= off) incl += t;
    }
    uint32_t a = incl - s;
    if (a < k && k <= incl) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (a < k && k <= a + c[j]) {
                res[0] = 255 - 4 * lane - j;
                res[1] = a;
            }
            a += c[j];
        }
    }
}

// NT threads own one row.  A thread handles 8 consecutive columns at a time (one 16-byte load of bias, one 8-byte
// load of the incoming mask, one 8-byte store of the result when the row addresses allow it).
// REP copies of the histogram, copy = lane % REP, laid out [bin][copy] so that the copies of a bin sit in different
// LDS banks: lanes that hit the same bin do not serialise (32 copies for long rows; 8 for short ones, where clearing
// and folding the copies would cost more than the conflicts).
template <int NT, int REP>
__global__ void __launch_bounds__(NT) make_mask_kernel(const MaskParams p) {
    __shared__ uint32_t hist[256 * REP];  // [bin][copy]
    __shared__ uint32_t hsum[256];
    __shared__ uint32_t res[4];
    __shared__ uint32_t wave_cnt[NT / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.x;
    const int r = row % p.rows, h = (row / p.rows) % p.heads, b = row / (p.rows * p.heads);
    const uint16_t *brow = (const uint16_t *)p.bias + b * p.bi_b + h * p.bi_h + (int64_t)r * p.bi_r;
    const uint8_t *mrow = p.mask_in ? p.mask_in + b * p.mi_b + h * p.mi_h + (int64_t)r * p.mi_r : nullptr;
    uint8_t *orow = p.mask_out + b * p.mo_b + h * p.mo_h + (int64_t)r * p.mo_r;
    const int Lk = p.Lk;
    const uint32_t min_bits = p.min_bits;
    const bool vec_b = ((uintptr_t)brow & 15) == 0, vec_m = ((uintptr_t)mrow & 7) == 0, vec_o = ((uintptr_t)orow & 7) == 0;

    // values of columns idx .. idx+7 after the masked fill, as bits of the bias type; returns how many are in range
    auto load8 = [&](int idx, uint32_t (&v)[8]) -> int {
        const int n = Lk - idx < 8 ? Lk - idx : 8;
        if (vec_b && n == 8) {
            const u32x4_t t = *(const u32x4_t *)(brow + idx);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[2 * j] = t[j] & 0xffffu;
                v[2 * j + 1] = t[j] >> 16;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = j < n ? brow[idx + j] : 0;
        }
        if (mrow) {
            if (vec_m && n == 8) {
                const uint64_t mm = *(const uint64_t *)(mrow + idx);
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (!((mm >> (8 * j)) & 0xffu)) v[j] = min_bits;
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (j < n && !mrow[idx + j]) v[j] = min_bits;
            }
        }
        return n;
    };
    auto store8 = [&](int idx, int n, uint64_t bytes) {
        if (vec_o && n == 8) {
            *(uint64_t *)(orow + idx) = bytes;
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (j < n) orow[idx + j] = (uint8_t)((bytes >> (8 * j)) & 0xffu);
        }
    };
    // "is the fill value" compares numerically (+0 == -0)
    auto is_min = [&](uint32_t v) -> bool { return v == min_bits || (((v | min_bits) & 0x7fffu) == 0); };
    auto clear_hist = [&]() {
        for (int i = tid; i < 256 * REP; i += NT) hist[i] = 0;
    };
    // sum of the copies of every bin -> hsum; copy (t + i) % REP in step i keeps the lanes on different banks
    auto fold_hist = [&]() {
        for (int t = tid; t < 256; t += NT) {
            uint32_t s = 0;
#pragma unroll
            for (int i = 0; i < REP; i++) s += hist[t * REP + ((t + i) & (REP - 1))];
            hsum[t] = s;
        }
    };

    if (p.type == 1) {  // relu: keep strictly positive values (NaN is not > 0)
        const uint32_t inf = p.dtype == 0 ? 0x7f80u : 0x7c00u;
        for (int idx = tid * 8; idx < Lk; idx += NT * 8) {
            uint32_t v[8];
            const int n = load8(idx, v);
            uint64_t bytes = 0;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t mag = v[j] & 0x7fffu;
                if (!(v[j] & 0x8000u) && mag != 0 && mag <= inf) bytes |= 1ull << (8 * j);
            }
            store8(idx, n, bytes);
        }
    } else {
        const uint32_t k = (uint32_t)(p.window < Lk ? p.window : Lk);
        if (k == 0) {
            for (int idx = tid * 8; idx < Lk; idx += NT * 8) store8(idx, Lk - idx < 8 ? Lk - idx : 8, 0);
        } else {
            const int rep = lane & (REP - 1);
            // ---- level 1: high byte
            clear_hist();
            __syncthreads();
            for (int idx = tid * 8; idx < Lk; idx += NT * 8) {
                uint32_t v[8];
                const int n = load8(idx, v);
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (j < n) atomicAdd(&hist[(order_key(v[j]) >> 8) * REP + rep], 1u);
            }
            __syncthreads();
            fold_hist();
            __syncthreads();
            if (wave == 0) find_bin(hsum, k, res);
            clear_hist();
            __syncthreads();
            const uint32_t bin1 = res[0], above1 = res[1];
            // ---- level 2: low byte inside bin1
            for (int idx = tid * 8; idx < Lk; idx += NT * 8) {
                uint32_t v[8];
                const int n = load8(idx, v);
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const uint32_t key = order_key(v[j]);
                    if (j < n && (key >> 8) == bin1) atomicAdd(&hist[(key & 0xffu) * REP + rep], 1u);
                }
            }
            __syncthreads();
            fold_hist();
            __syncthreads();
            if (wave == 0) find_bin(hsum, k - above1, res + 2);
            __syncthreads();
            const uint32_t T = (bin1 << 8) | res[2];
            const uint32_t need_eq = k - above1 - res[3];  // >= 1 entries equal to T still to take
            const uint32_t total_eq = hsum[res[2]];
            if (need_eq >= total_eq) {  // every entry equal to the threshold is taken: no ordering needed
                for (int idx = tid * 8; idx < Lk; idx += NT * 8) {
                    uint32_t v[8];
                    const int n = load8(idx, v);
                    uint64_t bytes = 0;
#pragma unroll
                    for (int j = 0; j < 8; j++)
                        if (order_key(v[j]) >= T && !is_min(v[j])) bytes |= 1ull << (8 * j);
                    store8(idx, n, bytes);
                }
            } else {
                // Ties across the threshold: the first need_eq of them in column order.  Columns are walked in
                // chunks of NT * 8 in order: a prefix over the lanes' counts inside the wave, per-wave counts through LDS.
                uint32_t taken = 0;  // entries equal to T seen in earlier chunks (uniform)
                for (int base = 0; base < Lk; base += NT * 8) {
                    const int idx = base + tid * 8;
                    uint32_t v[8];
                    const int n = idx < Lk ? load8(idx, v) : 0;
                    uint32_t mine = 0;
#pragma unroll
                    for (int j = 0; j < 8; j++)
                        if (j < n && order_key(v[j]) == T) mine++;
                    uint32_t incl = mine;
#pragma unroll
                    for (int off = 1; off < 64; off <<= 1) {
                        const uint32_t t = __shfl_up(incl, off);
                        if (lane >= off) incl += t;
                    }
                    if (lane == 63) wave_cnt[wave] = incl;
                    __syncthreads();
                    uint32_t rank = taken + incl - mine, chunk_total = 0;
                    for (int w = 0; w < NT / 64; w++) {
                        if (w < wave) rank += wave_cnt[w];
                        chunk_total += wave_cnt[w];
                    }
                    uint64_t bytes = 0;
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const uint32_t key = order_key(v[j]);
                        const bool eq = j < n && key == T;
                        if (j < n && (key > T || (eq && rank < need_eq)) && !is_min(v[j])) bytes |= 1ull << (8 * j);
                        if (eq) rank++;
                    }
                    if (n > 0) store8(idx, n, bytes);
                    taken += chunk_total;
                    __syncthreads();
                }
            }
        }
    }

    // ---- block smoothing (majority vote), on the row this workgroup has just written
    const int bs = p.block_size;
    if (bs > 1) {
        __syncthreads();  // the row's stores are visible to the whole workgroup
        const int n_full = Lk / bs, tail = Lk - n_full * bs;
        const int n_blocks = n_full + (tail ? 1 : 0);
        for (int blk = tid; blk < n_blocks; blk += NT) {
            const int c0 = blk * bs, len = blk < n_full ? bs : tail;
            int votes = 0;
            for (int c = 0; c < len; c++) votes += orow[c0 + c];
            const uint8_t keep = (2 * votes > len) ? 1 : 0;
            for (int c = 0; c < len; c++) orow[c0 + c] = keep;
        }
    }

    // ---- optional second output: the row as an ordered list of kept columns with prefix counts, the form the
    // compaction path of the attention kernels works on (they then need no pass of their own over the mask)
    if (p.kept_idx) {
        __syncthreads();  // the row's stores are visible to the whole workgroup
        scan_mask_row<NT>(orow, Lk, p.kept_idx + (size_t)row * p.kept_ld, p.kept_cnt + (size_t)row * p.kept_ld,
                          p.kept_count + row, (int *)wave_cnt, false);
    }

    // ---- optional third output: the row packed to one bit per key (key j in bit j % 8 of byte j / 8), the form in
    // which the per-query attention kernels take a mask at an eighth of its traffic.  A thread packs 32 keys into
    // one word; the row it reads was written by this workgroup a moment ago.
    if (p.bits) {
        __syncthreads();  // the row's stores are visible to the whole workgroup
        uint8_t *bits_row = p.bits + (size_t)row * p.bits_row_bytes;
        const int n_bytes = (Lk + 7) / 8;
        for (int w = tid; w * 4 < n_bytes; w += NT) {
            uint32_t word = 0;
            const int c0 = w * 32;
            if (vec_o && c0 + 32 <= Lk) {
#pragma unroll
                for (int q8 = 0; q8 < 4; q8++) {
                    const uint64_t m8 = *(const uint64_t *)(orow + c0 + 8 * q8);  // eight 0 / 1 bytes
                    // (bit 8 i of m8 to bit i: the product gathers them in its top byte)
                    word |= (uint32_t)(((m8 & 0x0101010101010101ull) * 0x0102040810204080ull) >> 56) << (8 * q8);
                }
            } else {
                for (int c = 0; c < 32 && c0 + c < Lk; c++) word |= (orow[c0 + c] ? 1u : 0u) << c;
            }
            if (w * 4 + 4 <= n_bytes) {
                *(uint32_t *)(bits_row + w * 4) = word;  // (rows are 4-byte aligned: bits_row_bytes is a multiple of 4)
            } else {
                for (int k = 0; w * 4 + k < n_bytes; k++) bits_row[w * 4 + k] = (uint8_t)(word >> (8 * k));
            }
        }
    }
}

}  // namespace

hipError_t launch_make_mask(const MaskParams &p, hipStream_t stream) {
    const int64_t n_rows = (int64_t)p.batch * p.heads * p.rows;
    if (n_rows <= 0 || p.Lk <= 0) return hipSuccess;
    // few long rows: 16 waves per row; many rows: 4 waves per row and several rows per CU
    if (p.Lk >= 8192 && n_rows < 2048) hipLaunchKernelGGL((make_mask_kernel<1024, 32>), dim3((unsigned)n_rows), dim3(1024), 0, stream, p);
    else if (p.Lk >= 16384) hipLaunchKernelGGL((make_mask_kernel<256, 32>), dim3((unsigned)n_rows), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((make_mask_kernel<256, 8>), dim3((unsigned)n_rows), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace fdma
