// Single-token decode (seqlen_q == 1) for gfx950: split-KV partial attention + LSE-weighted combine.
//
// Replaces the reference's decode route: the `seqlenq_ngroups_swapped` reshaping of mha_fwd
// (csrc/flash_sparse_attn/flash_api.cpp:443-475, 541-551), num_splits_heuristic (:275-349),
// compute_attn_1rowblock_splitkv (csrc/flash_sparse_attn/src/flash_fwd_kernel.h:808-1587) and
// combine_attn_seqk_parallel (:1618-1813).
//
// The path is bound by HBM reads of K and V.  A key/value row of one KV head is d*2 contiguous bytes,
// so skipping can be done per KEY instead of per 64-key tile: each workgroup first compacts the
// keys of its range that any query head of the group keeps (ordered, ballot based), then gathers
// only those rows.  With a top-W mask that reads W rows instead of every 64-key tile that holds one.
// The G query heads of a KV group share every gathered row.  Dot products run on the vector ALU:
// 16 lanes cover one row (8 elements each), so a wave works on 4 keys at a time.
#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {

namespace {

constexpr int DEC_THREADS = 256;
constexpr int DEC_RANGE = 2048;  // keys compacted per pass
constexpr int DEC_GROUPS = DEC_THREADS / 16;

template <typename T, int GC>
__global__ void __launch_bounds__(DEC_THREADS) decode_kernel(const FwdParams p, int keys_per_split, int g_base_stride) {
    using E = Elem<T>;
    __shared__ int s_idx[DEC_RANGE];
    __shared__ uint32_t s_bits[DEC_RANGE];
    __shared__ int s_wcount[4];
    __shared__ float s_m[DEC_GROUPS][GC], s_l[DEC_GROUPS][GC];
    extern __shared__ __attribute__((aligned(16))) float s_o[];  // [DEC_GROUPS][GC][Dpad]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int grp = tid >> 4, c = tid & 15;  // 16-lane group and 16-byte chunk of the row
    const int split = blockIdx.x, b = blockIdx.z;
    const int G = p.H / p.Hk;
    const int chunks = (G + GC - 1) / GC;
    const int hk = blockIdx.y / chunks;
    const int g0 = (blockIdx.y % chunks) * GC;  // first query head (within the group) of this workgroup
    (void)g_base_stride;
    const int Dpad = (p.d + 127) / 128 * 128;
    const int nchunk = p.d / 8;                 // 16-byte chunks per row
    const int per_lane = Dpad / 128;            // chunks handled by one lane (1 for d <= 128)

    const int lo = split * keys_per_split;
    int hi = lo + keys_per_split;
    if (hi > p.Lk) hi = p.Lk;

    // query fragments (fp32, pre-scaled into the log2 domain)
    float qf[GC][8];
#pragma unroll
    for (int gg = 0; gg < GC; gg++) {
        const int g = g0 + gg;
        u32x4_t v = {0, 0, 0, 0};
        if (g < G && c < nchunk) {
            const uint16_t *qp = (const uint16_t *)p.q + b * p.q_b + (int64_t)(hk * G + g) * p.q_h;
            v = *(const u32x4_t *)(qp + c * 8);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {
            qf[gg][2 * e] = E::lo(v[e]) * p.scale_log2;
            qf[gg][2 * e + 1] = E::hi(v[e]) * p.scale_log2;
        }
    }
    (void)per_lane;

    float m[GC], l[GC], o[GC][8];
#pragma unroll
    for (int gg = 0; gg < GC; gg++) {
        m[gg] = -INFINITY;
        l[gg] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) o[gg][e] = 0.f;
    }

    const uint16_t *kbase = (const uint16_t *)p.k + b * p.k_b + hk * p.k_h;
    const uint16_t *vbase = (const uint16_t *)p.v + b * p.v_b + hk * p.v_h;

    for (int r0 = lo; r0 < hi; r0 += DEC_RANGE) {
        // ---- phase 1: ordered compaction of the kept keys of [r0, r0 + DEC_RANGE)
        int total = 0;
        for (int base = r0; base < r0 + DEC_RANGE && base < hi; base += DEC_THREADS) {
            const int key = base + tid;
            uint32_t bits = 0;
            if (key < hi) {
                if (p.mask) {
#pragma unroll
                    for (int gg = 0; gg < GC; gg++) {
                        const int g = g0 + gg;
                        if (g < G) {
                            const int h = hk * G + g;
                            const int hm = p.Hm == p.H ? h : (p.Hm == 1 ? 0 : hk);
                            if (p.mask[b * p.m_b + hm * p.m_h + key]) bits |= 1u << gg;
                        }
                    }
                } else {
                    bits = (GC >= 32) ? 0xffffffffu : ((1u << GC) - 1u);
                }
            }
            const uint64_t ball = __ballot(bits != 0);
            const int wcount = __popcll(ball);
            const int woff = __popcll(ball & ((1ull << lane) - 1ull));
            if (lane == 0) s_wcount[wave] = wcount;
            __syncthreads();
            int wbase = total;
            for (int w = 0; w < wave; w++) wbase += s_wcount[w];
            if (bits != 0) {
                s_idx[wbase + woff] = key;
                s_bits[wbase + woff] = bits;
            }
            total += s_wcount[0] + s_wcount[1] + s_wcount[2] + s_wcount[3];
            __syncthreads();
        }

        // ---- phase 2: gather the kept rows; each 16-lane group takes keys grp, grp+16, ... four at a time
        for (int t0 = grp * 4; t0 < total; t0 += DEC_GROUPS * 4) {
            u32x4_t kv[4], vv[4];
            int key[4];
            uint32_t kbits[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int t = t0 + u;
                key[u] = t < total ? s_idx[t] : -1;
                kbits[u] = t < total ? s_bits[t] : 0u;
                kv[u] = u32x4_t{0, 0, 0, 0};
                vv[u] = u32x4_t{0, 0, 0, 0};
                if (key[u] >= 0 && c < nchunk) {
                    kv[u] = *(const u32x4_t *)(kbase + (int64_t)key[u] * p.k_r + c * 8);
                    vv[u] = *(const u32x4_t *)(vbase + (int64_t)key[u] * p.v_r + c * 8);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (key[u] < 0) continue;  // uniform within the 16-lane group
                float kf[8], vf[8];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    kf[2 * e] = E::lo(kv[u][e]); kf[2 * e + 1] = E::hi(kv[u][e]);
                    vf[2 * e] = E::lo(vv[u][e]); vf[2 * e + 1] = E::hi(vv[u][e]);
                }
#pragma unroll
                for (int gg = 0; gg < GC; gg++) {
                    float part = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; e++) part = fmaf(qf[gg][e], kf[e], part);
                    part += __shfl_xor(part, 1);
                    part += __shfl_xor(part, 2);
                    part += __shfl_xor(part, 4);
                    part += __shfl_xor(part, 8);
                    const int g = g0 + gg;
                    float s = -INFINITY;
                    if ((kbits[u] >> gg) & 1u) {
                        float bl2 = 0.f;
                        if (p.bias) {
                            const int h = hk * G + (g < G ? g : 0);
                            const int hb = p.Hb == p.H ? h : (p.Hb == 1 ? 0 : hk);
                            uint32_t raw = ((const uint16_t *)p.bias)[b * p.bi_b + hb * p.bi_h + key[u]];
                            bl2 = E::lo(raw) * kLog2e;
                        }
                        s = part + bl2;
                    }
                    const float mn = fmaxf(m[gg], s);
                    const float ms = mn == -INFINITY ? 0.f : mn;
                    const float alpha = fast_exp2(m[gg] - ms);
                    const float pe = fast_exp2(s - ms);
                    m[gg] = mn;
                    l[gg] = l[gg] * alpha + pe;
#pragma unroll
                    for (int e = 0; e < 8; e++) o[gg][e] = fmaf(o[gg][e], alpha, pe * vf[e]);
                }
            }
        }
        __syncthreads();  // the list is rebuilt by the next pass
    }

    // ---- phase 3: merge the 16 groups of the workgroup
#pragma unroll
    for (int gg = 0; gg < GC; gg++) {
        if (c == 0) { s_m[grp][gg] = m[gg]; s_l[grp][gg] = l[gg]; }
#pragma unroll
        for (int e = 0; e < 8; e++) s_o[(grp * GC + gg) * Dpad + c * 8 + e] = o[gg][e];
    }
    __syncthreads();
    for (int idx = tid; idx < GC * Dpad; idx += DEC_THREADS) {
        const int gg = idx / Dpad, e = idx % Dpad;
        const int g = g0 + gg;
        if (g >= G || e >= p.d) continue;
        float mx = -INFINITY;
#pragma unroll
        for (int q = 0; q < DEC_GROUPS; q++) mx = fmaxf(mx, s_m[q][gg]);
        float lt = 0.f, ot = 0.f;
        if (mx != -INFINITY) {
#pragma unroll
            for (int q = 0; q < DEC_GROUPS; q++) {
                const float w = fast_exp2(s_m[q][gg] - mx);
                lt += w * s_l[q][gg];
                ot += w * s_o[(q * GC + gg) * Dpad + e];
            }
        }
        const int h = hk * G + g;
        const float inv = lt > 0.f ? 1.f / lt : 0.f;
        if (p.splits > 1) {
            const int64_t row = ((int64_t)split * p.B + b) * p.H + h;
            p.o_part[row * p.d + e] = ot * inv;
            if (e == 0) p.lse_part[row] = lt > 0.f ? (mx + __builtin_amdgcn_logf(lt)) * kLn2 : -INFINITY;
        } else {
            uint16_t *op = (uint16_t *)p.o + b * p.o_b + h * p.o_h;
            op[e] = (uint16_t)(E::pack2(ot * inv, 0.f) & 0xffffu);
            if (e == 0) p.lse[(int64_t)b * p.H + h] = lt > 0.f ? (mx + __builtin_amdgcn_logf(lt)) * kLn2 : INFINITY;
        }
    }
}

// out[b,h,:] = sum_s exp(lse_s - lse) * o_s ;  lse = logsumexp_s lse_s  (empty everywhere: 0 / +inf)
template <typename T>
__global__ void __launch_bounds__(256) decode_combine_kernel(const FwdParams p) {
    using E = Elem<T>;
    const int64_t rows = (int64_t)p.B * p.H;
    const int row = blockIdx.x * (256 / 64) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= rows) return;
    float mx = -INFINITY;
    for (int s = lane; s < p.splits; s += 64) mx = fmaxf(mx, p.lse_part[(int64_t)s * rows + row]);
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    float sum = 0.f;
    if (mx != -INFINITY)
        for (int s = lane; s < p.splits; s += 64) sum += __expf(p.lse_part[(int64_t)s * rows + row] - mx);
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    const int b = row / p.H, h = row % p.H;
    const float lse = mx == -INFINITY ? INFINITY : mx + __logf(sum);
    if (lane == 0) p.lse[row] = lse;
    uint16_t *op = (uint16_t *)p.o + b * p.o_b + h * p.o_h;
    for (int e = lane; e < p.d; e += 64) {
        float acc = 0.f;
        if (mx != -INFINITY)
            for (int s = 0; s < p.splits; s++) {
                const float ls = p.lse_part[(int64_t)s * rows + row];
                if (ls != -INFINITY) acc += __expf(ls - lse) * p.o_part[((int64_t)s * rows + row) * p.d + e];
            }
        op[e] = (uint16_t)(E::pack2(acc, 0.f) & 0xffffu);
    }
}

template <typename T, int GC>
hipError_t launch_decode_gc(const FwdParams &p, int keys_per_split, hipStream_t stream) {
    const int G = p.H / p.Hk;
    const int chunks = (G + GC - 1) / GC;
    const int Dpad = (p.d + 127) / 128 * 128;
    dim3 grid(p.splits, p.Hk * chunks, p.B);
    const size_t smem = (size_t)DEC_GROUPS * GC * Dpad * sizeof(float);
    auto kern = decode_kernel<T, GC>;
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, dim3(DEC_THREADS), smem, stream, p, keys_per_split, 0);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_decode_t(const FwdParams &p, hipStream_t stream) {
    const int G = p.H / p.Hk;
    const int keys_per_split = ((p.Lk + p.splits - 1) / p.splits + DEC_THREADS - 1) / DEC_THREADS * DEC_THREADS;
    hipError_t e;
    if (G == 1) e = launch_decode_gc<T, 1>(p, keys_per_split, stream);
    else if (G == 2) e = launch_decode_gc<T, 2>(p, keys_per_split, stream);
    else if (G <= 4) e = launch_decode_gc<T, 4>(p, keys_per_split, stream);
    else e = launch_decode_gc<T, 8>(p, keys_per_split, stream);
    if (e != hipSuccess) return e;
    if (p.splits > 1) {
        const int64_t rows = (int64_t)p.B * p.H;
        hipLaunchKernelGGL((decode_combine_kernel<T>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, p);
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

// Enough workgroups to cover the 256 CUs about four times, at least 256 keys per split.
// With keys_per_split rounded up to 256 every split is non-empty.
int decode_num_splits(int B, int Hk, int Lk) {
    const int pairs = B * Hk > 0 ? B * Hk : 1;
    int splits = (1024 + pairs - 1) / pairs;
    const int max_by_len = (Lk + 255) / 256;
    if (splits > max_by_len) splits = max_by_len;
    if (splits > 128) splits = 128;
    if (splits < 1) splits = 1;
    // shrink so that no split is empty after rounding keys_per_split up to a multiple of 256
    while (splits > 1) {
        const int kps = ((Lk + splits - 1) / splits + 255) / 256 * 256;
        if ((int64_t)(splits - 1) * kps < Lk) break;
        splits--;
    }
    return splits;
}

hipError_t launch_fwd_decode(const FwdParams &p, int dtype, hipStream_t stream) {
    if (p.B <= 0) return hipSuccess;
    return dtype == 0 ? launch_decode_t<bf16_tag>(p, stream) : launch_decode_t<fp16_tag>(p, stream);
}

}  // namespace fdma
