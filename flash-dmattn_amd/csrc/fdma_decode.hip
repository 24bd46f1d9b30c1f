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
constexpr int DEC_RANGE = 16 * DEC_THREADS;  // keys compacted per pass (16 per thread)
constexpr int DEC_GROUPS = DEC_THREADS / 16;
constexpr int DEC_KPI = 8;  // keys per 16-lane group and iteration

// nonzero bytes of x -> bit k of the result is set iff byte k of x != 0
__device__ __forceinline__ uint32_t nz_bytes_to_bits(uint32_t x) {
    uint32_t y = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
    return ((y >> 7) * 0x10204080u) >> 28;
}

template <typename T, int GC>
__global__ void __launch_bounds__(DEC_THREADS) decode_kernel(const FwdParams p, int keys_per_split, int g_base_stride) {
    using E = Elem<T>;
    __shared__ uint16_t s_idx[DEC_RANGE];  // kept keys of the current pass, relative to its first key
    __shared__ uint8_t s_bits[DEC_RANGE];   // which query heads of the chunk keep the key
    __shared__ int s_wcount[4];
    __shared__ float s_m[4][GC], s_l[4][GC];
    extern __shared__ __attribute__((aligned(16))) float s_o[];  // [4 waves][GC][Dpad]

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
        // ---- phase 1: ordered compaction of the kept keys of [r0, r0 + DEC_RANGE): every thread tests 16
        // keys with one 16-byte mask load per query head, a wave scan + one barrier orders the output
        int total;
        {
            const int key0 = r0 + 16 * tid;
            uint32_t hbits[GC];  // bit k of hbits[gg]: key0 + k is kept by query head g0 + gg
            uint32_t uni = 0;
            const int nval = hi - key0;  // keys of this thread inside the range
            const uint32_t inrange = nval >= 16 ? 0xffffu : (nval <= 0 ? 0u : ((1u << nval) - 1u));
#pragma unroll
            for (int gg = 0; gg < GC; gg++) {
                uint32_t bits = 0;
                const int g = g0 + gg;
                if (g < G && nval > 0) {
                    if (p.mask) {
                        const int h = hk * G + g;
                        const int hm = p.Hm == p.H ? h : (p.Hm == 1 ? 0 : hk);
                        if (gg == 0 || p.Hm == p.H) {
                            const u32x4_t mv = *(const u32x4_t *)(p.mask + b * p.m_b + hm * p.m_h + key0);
                            bits = nz_bytes_to_bits(mv[0]) | (nz_bytes_to_bits(mv[1]) << 4) | (nz_bytes_to_bits(mv[2]) << 8) |
                                   (nz_bytes_to_bits(mv[3]) << 12);
                        } else {
                            bits = hbits[0];  // heads of the group share the mask row
                        }
                    } else {
                        bits = 0xffffu;
                    }
                }
                bits &= inrange;
                hbits[gg] = bits;
                uni |= bits;
            }
            const int cnt = __popc(uni);
            int incl = cnt;  // inclusive wave scan
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int v = __shfl_up(incl, off);
                if (lane >= off) incl += v;
            }
            if (lane == 63) s_wcount[wave] = incl;
            __syncthreads();
            int base = 0;
            for (int w = 0; w < wave; w++) base += s_wcount[w];
            total = s_wcount[0] + s_wcount[1] + s_wcount[2] + s_wcount[3];
            int pos = base + incl - cnt;
            uint32_t u = uni;
            while (u) {
                const int k = __builtin_ctz(u);
                u &= u - 1;
                uint32_t kb = 0;
#pragma unroll
                for (int gg = 0; gg < GC; gg++) kb |= ((hbits[gg] >> k) & 1u) << gg;
                s_idx[pos] = (uint16_t)(16 * tid + k);
                s_bits[pos] = (uint8_t)kb;
                pos++;
            }
            __syncthreads();
        }

        // ---- phase 2: gather the kept rows; each 16-lane group takes DEC_KPI keys per iteration, with all
        // of their K / V / bias loads in flight together, and does one online-softmax update per batch
        for (int t0 = grp * DEC_KPI; t0 < total; t0 += DEC_GROUPS * DEC_KPI) {
            u32x4_t kv[DEC_KPI], vv[DEC_KPI];
            int key[DEC_KPI];
            uint32_t kbits[DEC_KPI];
            uint32_t braw[DEC_KPI][GC];
#pragma unroll
            for (int u = 0; u < DEC_KPI; u++) {
                const int t = t0 + u;
                key[u] = t < total ? r0 + (int)s_idx[t] : -1;
                kbits[u] = t < total ? (uint32_t)s_bits[t] : 0u;
                kv[u] = u32x4_t{0, 0, 0, 0};
                vv[u] = u32x4_t{0, 0, 0, 0};
                if (key[u] >= 0 && c < nchunk) {
                    kv[u] = *(const u32x4_t *)(kbase + (int64_t)key[u] * p.k_r + c * 8);
                    vv[u] = *(const u32x4_t *)(vbase + (int64_t)key[u] * p.v_r + c * 8);
                }
#pragma unroll
                for (int gg = 0; gg < GC; gg++) {
                    braw[u][gg] = 0;
                    if (p.bias && key[u] >= 0) {
                        if (gg == 0 || p.Hb == p.H) {
                            const int g = g0 + gg < G ? g0 + gg : 0;
                            const int h = hk * G + g;
                            const int hb = p.Hb == p.H ? h : (p.Hb == 1 ? 0 : hk);
                            braw[u][gg] = ((const uint16_t *)p.bias)[b * p.bi_b + hb * p.bi_h + key[u]];
                        } else {
                            braw[u][gg] = braw[u][0];
                        }
                    }
                }
            }
            // scores of the batch (log2 domain); dropped (key, head) pairs are -inf
            float sc[DEC_KPI][GC];
#pragma unroll
            for (int u = 0; u < DEC_KPI; u++) {
                float kf[8];
#pragma unroll
                for (int e = 0; e < 4; e++) { kf[2 * e] = E::lo(kv[u][e]); kf[2 * e + 1] = E::hi(kv[u][e]); }
#pragma unroll
                for (int gg = 0; gg < GC; gg++) {
                    float part = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; e++) part = fmaf(qf[gg][e], kf[e], part);
                    part += __shfl_xor(part, 1);
                    part += __shfl_xor(part, 2);
                    part += __shfl_xor(part, 4);
                    part += __shfl_xor(part, 8);
                    sc[u][gg] = ((kbits[u] >> gg) & 1u) ? part + E::lo(braw[u][gg]) * kLog2e : -INFINITY;
                }
            }
#pragma unroll
            for (int gg = 0; gg < GC; gg++) {
                float mn = m[gg];
#pragma unroll
                for (int u = 0; u < DEC_KPI; u++) mn = fmaxf(mn, sc[u][gg]);
                const float ms = mn == -INFINITY ? 0.f : mn;
                const float alpha = fast_exp2(m[gg] - ms);
                m[gg] = mn;
                l[gg] *= alpha;
#pragma unroll
                for (int e = 0; e < 8; e++) o[gg][e] *= alpha;
#pragma unroll
                for (int u = 0; u < DEC_KPI; u++) {
                    const float pe = fast_exp2(sc[u][gg] - ms);
                    l[gg] += pe;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        o[gg][2 * e] = fmaf(pe, E::lo(vv[u][e]), o[gg][2 * e]);
                        o[gg][2 * e + 1] = fmaf(pe, E::hi(vv[u][e]), o[gg][2 * e + 1]);
                    }
                }
            }
        }
        __syncthreads();  // the list is rebuilt by the next pass
    }

    // ---- phase 3: merge the four 16-lane groups of each wave in registers, then the four waves through LDS
#pragma unroll
    for (int off = 16; off <= 32; off <<= 1) {
#pragma unroll
        for (int gg = 0; gg < GC; gg++) {
            const float mo = __shfl_xor(m[gg], off), lo_ = __shfl_xor(l[gg], off);
            const float mn = fmaxf(m[gg], mo);
            const float ms = mn == -INFINITY ? 0.f : mn;
            const float wa = fast_exp2(m[gg] - ms), wb = fast_exp2(mo - ms);
            l[gg] = l[gg] * wa + lo_ * wb;
#pragma unroll
            for (int e = 0; e < 8; e++) o[gg][e] = o[gg][e] * wa + __shfl_xor(o[gg][e], off) * wb;
            m[gg] = mn;
        }
    }
    if (lane < 16) {
#pragma unroll
        for (int gg = 0; gg < GC; gg++) {
            if (c == 0) { s_m[wave][gg] = m[gg]; s_l[wave][gg] = l[gg]; }
#pragma unroll
            for (int e = 0; e < 8; e++) s_o[(wave * GC + gg) * Dpad + c * 8 + e] = o[gg][e];
        }
    }
    __syncthreads();
    for (int idx = tid; idx < GC * Dpad; idx += DEC_THREADS) {
        const int gg = idx / Dpad, e = idx % Dpad;
        const int g = g0 + gg;
        if (g >= G || e >= p.d) continue;
        float mx = -INFINITY;
#pragma unroll
        for (int q = 0; q < 4; q++) mx = fmaxf(mx, s_m[q][gg]);
        float lt = 0.f, ot = 0.f;
        if (mx != -INFINITY) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
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

// out[b,h,:] = sum_s exp(lse_s - lse) * o_s ;  lse = logsumexp_s lse_s  (empty everywhere: 0 / +inf).
// One thread per (row, head-dim element); the split loop is short and its loads are independent.
template <typename T>
__global__ void __launch_bounds__(256) decode_combine_kernel(const FwdParams p) {
    using E = Elem<T>;
    const int64_t rows = (int64_t)p.B * p.H;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t row = idx / p.d;
    const int e = (int)(idx % p.d);
    if (row >= rows) return;
    float mx = -INFINITY;
    for (int s = 0; s < p.splits; s++) mx = fmaxf(mx, p.lse_part[(int64_t)s * rows + row]);
    float sum = 0.f, acc = 0.f;
    if (mx != -INFINITY) {
        for (int s = 0; s < p.splits; s++) {
            const float w = __expf(p.lse_part[(int64_t)s * rows + row] - mx);  // exp(-inf) = 0 for empty splits
            sum += w;
            acc += w * p.o_part[((int64_t)s * rows + row) * p.d + e];
        }
        acc /= sum;
    }
    const int b = (int)(row / p.H), h = (int)(row % p.H);
    if (e == 0) p.lse[row] = mx == -INFINITY ? INFINITY : mx + __logf(sum);
    ((uint16_t *)p.o)[b * p.o_b + h * p.o_h + e] = (uint16_t)(E::pack2(acc, 0.f) & 0xffffu);
}

template <typename T, int GC>
hipError_t launch_decode_gc(const FwdParams &p, int keys_per_split, hipStream_t stream) {
    const int G = p.H / p.Hk;
    const int chunks = (G + GC - 1) / GC;
    const int Dpad = (p.d + 127) / 128 * 128;
    dim3 grid(p.splits, p.Hk * chunks, p.B);
    const size_t smem = (size_t)4 * GC * Dpad * sizeof(float);
    auto kern = decode_kernel<T, GC>;
    static DynSmemLimit smem_limit;
    hipError_t e = smem_limit.ensure((const void *)kern, (int)smem);
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
        hipLaunchKernelGGL((decode_combine_kernel<T>), dim3((unsigned)((rows * p.d + 255) / 256)), dim3(256), 0, stream, p);
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

// Enough workgroups to cover the 256 CUs about twice (measured best on cfg5-like shapes), at least 256 keys per split.
// With keys_per_split rounded up to 256 every split is non-empty.
int decode_num_splits(int B, int Hk, int Lk) {
    const int pairs = B * Hk > 0 ? B * Hk : 1;
    int splits = (512 + pairs - 1) / pairs;
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
