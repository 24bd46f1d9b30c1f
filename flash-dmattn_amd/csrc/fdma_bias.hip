// Producer of the dynamic-mask attention bias, fused: bias[b, j, 0, l] = A[j] * softplus(dt[b, l, j]) with
// dt = V_flat[b, l, :] . W[j, :] (+ pb[j]), V_flat the value states of all kv heads of a token side by side -- the
// `A * softplus(dt_proj(V))` of the reference's Doge caller (examples/modeling/modeling_doge.py:217-222), which there is a
// linear layer, a softplus, a multiply, a transpose and a cast through the tensor library in front of every attention
// call, and the same again backwards.  The column-summed dBias that the attention backward returns in the bias's own
// [B, Hkv, 1, Lk] shape is consumed here directly.
//
// Forward: a workgroup owns 32 tokens, each of its four waves a quarter of the columns.  V rows are the A operand and W rows the B operand of MFMA 32x32x16, both straight
// from global memory (every lane reads 16 contiguous bytes of its own row per step: no LDS, no transposes); the
// accumulator column of lane j < Hkv holds dt of 16 of the tokens, finished in place.  HBM traffic is one read of V.
// Backward: a workgroup owns a run of tokens; d_dt = dBias * A * sigmoid(dt) goes to LDS, then a thread owns four
// columns of V_flat and walks the tokens: dV = d_dt W and the workgroup's share of dW = d_dt^T V_flat, dA and dpb, which
// go to fp32 partials that a second kernel folds in a fixed order (bit-reproducible).
#include "fdma_common.h"
#include "fdma_params.h"

namespace fdma {
namespace {

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(__expf(x)); }  // torch: beta 1, threshold 20
__device__ __forceinline__ float sigmoid_f(float x) { return x > 20.f ? 1.f : 1.f / (1.f + __expf(-x)); }  // d softplus / dx, same threshold

// SPLITK: the four waves of a workgroup share 32 tokens, a quarter of the columns each (few tokens: more waves in
// flight); otherwise every wave owns 32 tokens of its own and reads whole rows.
template <typename T, bool SPLITK>
__global__ void __launch_bounds__(256) dyn_bias_fwd_kernel(const DynBiasParams p) {
    using E = Elem<T>;
    __shared__ float s_acc[SPLITK ? 3 : 1][16][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, g = lane >> 5;
    const int64_t n_rows = (int64_t)p.B * p.L;
    const int64_t row0 = SPLITK ? (int64_t)blockIdx.x * 32 : ((int64_t)blockIdx.x * 4 + wave) * 32;
    if (!SPLITK && row0 >= n_rows) return;  // (no barrier on this path)
    const int K = p.Hk * p.d;
    int64_t row = row0 + r;
    if (row >= n_rows) row = n_rows - 1;  // clamped duplicate, never stored
    const int b = (int)(row / p.L), l = (int)(row % p.L);
    const uint16_t *vrow = (const uint16_t *)p.v + b * p.v_b + (int64_t)l * p.v_r;
    const uint16_t *wrow = (const uint16_t *)p.w + (int64_t)(r < p.Hk ? r : 0) * K;
    const uint32_t wmask = r < p.Hk ? 0xffffffffu : 0u;  // output columns beyond Hkv: zero operand (no branch around the load)
    f32x16_t acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    // eight k-steps per trip: a lane pair then reads one whole 128-byte line of its V row per trip (with fewer, the
    // second half of a line is asked for a trip later, when the line may have left the caches again), and all loads
    // of a trip are issued before its first MFMA
    constexpr int KU = 8;
    const int n_ks = K / 16, per_wave = SPLITK ? ((n_ks + 3) / 4 + KU - 1) / KU * KU : n_ks;
    const int ks_begin = SPLITK ? wave * per_wave : 0;
    const int ks_end = ks_begin + per_wave < n_ks ? ks_begin + per_wave : n_ks;
    for (int ks0 = ks_begin; ks0 < ks_end; ks0 += KU) {
        u32x4_t a[KU], bw[KU];
#pragma unroll
        for (int u = 0; u < KU; u++) {
            const int ks = ks0 + u < ks_end ? ks0 + u : ks_end - 1;  // (a short last trip re-reads the last step and drops it)
            const int kk = ks * 16 + 8 * g, head = kk / p.d, dd = kk - head * p.d;
            a[u] = *(const u32x4_t *)(vrow + (int64_t)head * p.v_h + dd);
            bw[u] = *(const u32x4_t *)(wrow + kk);
        }
#pragma unroll
        for (int u = 0; u < KU; u++) {
            const uint32_t m = (ks0 + u < ks_end) ? wmask : 0u;
#pragma unroll
            for (int e = 0; e < 4; e++) bw[u][e] &= m;
            acc = E::mfma(a[u], bw[u], acc);
        }
    }
    if (SPLITK) {
        if (wave > 0) {
#pragma unroll
            for (int i = 0; i < 16; i++) s_acc[wave - 1][i][lane] = acc[i];
        }
        __syncthreads();
    }
    if ((!SPLITK || wave == 0) && r < p.Hk) {
        const float a_j = E::lo((uint32_t)((const uint16_t *)p.a)[r]);
        const float pb_j = p.pb ? E::lo((uint32_t)((const uint16_t *)p.pb)[r]) : 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int64_t rr = row0 + 8 * (i / 4) + 4 * g + (i % 4);  // accumulator register i: this tile row, column r
            if (rr < n_rows) {
                const int bb = (int)(rr / p.L), ll = (int)(rr % p.L);
                float dt = acc[i];
                if (SPLITK) dt = ((dt + s_acc[0][i][lane]) + s_acc[1][i][lane]) + s_acc[2][i][lane];
                dt += pb_j;
                p.dt[rr * p.Hk + r] = dt;
                ((uint16_t *)p.bias)[bb * p.bias_b + (int64_t)r * p.bias_h + ll] = (uint16_t)(E::pack2(a_j * softplus_f(dt), 0.f) & 0xffffu);
            }
        }
    }
}

// Backward, first stage.  Workgroup `c` owns token rows [c * rows_per_wg, ...).  HM = Hkv rounded up to 8, 16 or 32:
// thread t works on output head t % HM for the per-head sums, so each sum is built in a fixed order; in the main part
// a thread owns CPT adjacent columns of V_flat (4; 2 when 32 heads' worth of accumulators must fit the registers or
// when V_flat has too few columns to give every thread four).
template <typename T, int HM, int CPT>
__global__ void __launch_bounds__(256) dyn_bias_bwd_kernel(const DynBiasParams p) {
    using E = Elem<T>;
    constexpr int RB = 64;                   // tokens per pass through LDS
    __shared__ float s_ddt[RB * HM];
    __shared__ float s_red[2 * 256];
    const int tid = threadIdx.x;
    const int Hk = p.Hk, K = Hk * p.d;
    const int64_t wg_row0 = (int64_t)blockIdx.x * p.rows_per_wg;
    const int64_t n_rows = (int64_t)p.B * p.L;
    const int64_t wg_row1 = wg_row0 + p.rows_per_wg < n_rows ? wg_row0 + p.rows_per_wg : n_rows;
    const int j_mine = tid % HM, rgroup = tid / HM;
    constexpr int RSTEP = 256 / HM;
    const float a_mine = j_mine < Hk ? E::lo((uint32_t)((const uint16_t *)p.a)[j_mine]) : 0.f;
    float sum_a = 0.f, sum_pb = 0.f;  // this thread's share of dA[j_mine], dpb[j_mine]
    float *part_w = p.part + (int64_t)blockIdx.x * p.part_stride;
    const int n_groups = (K + 256 * CPT - 1) / (256 * CPT);  // column groups: the same trip count for every thread

    for (int grp = 0; grp < n_groups; grp++) {
        const int k0 = grp * 256 * CPT + tid * CPT;
        const bool has_cols = k0 < K;
        const int head = has_cols ? k0 / p.d : 0, dd = has_cols ? k0 - head * p.d : 0;
        float wj[HM][CPT], dw[HM][CPT];
#pragma unroll
        for (int j = 0; j < HM; j++) {
#pragma unroll
            for (int e = 0; e < CPT; e += 2) {
                const uint32_t wv = (has_cols && j < Hk) ? *(const uint32_t *)((const uint16_t *)p.w + (int64_t)j * K + k0 + e) : 0u;
                wj[j][e] = E::lo(wv);
                wj[j][e + 1] = E::hi(wv);
                dw[j][e] = dw[j][e + 1] = 0.f;
            }
        }
        for (int64_t base = wg_row0; base < wg_row1; base += RB) {
            __syncthreads();
            // d_dt of the RB tokens of this pass -> LDS; the per-head sums are taken on the first column group
            for (int rr = rgroup; rr < RB; rr += RSTEP) {
                const int64_t row = base + rr;
                float ddt = 0.f;
                if (j_mine < Hk && row < wg_row1) {
                    const int b = (int)(row / p.L), l = (int)(row % p.L);
                    const float gb = E::lo((uint32_t)((const uint16_t *)p.dbias)[b * p.dbias_b + (int64_t)j_mine * p.dbias_h + l]);
                    const float dt = p.dt[row * Hk + j_mine];
                    ddt = gb * a_mine * sigmoid_f(dt);
                    if (grp == 0) {
                        sum_a += gb * softplus_f(dt);
                        sum_pb += ddt;
                    }
                }
                s_ddt[rr * HM + j_mine] = ddt;
            }
            __syncthreads();
            if (has_cols) {
                const int n = (int)(wg_row1 - base < RB ? wg_row1 - base : RB);
                for (int rr0 = 0; rr0 < n; rr0 += 4) {  // four tokens at a time: their loads are issued together
                    uint32_t vraw[4][CPT / 2];
                    uint16_t *op[4];
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const int64_t row = base + (rr0 + u < n ? rr0 + u : n - 1);
                        const int b = (int)(row / p.L), l = (int)(row % p.L);
                        const uint16_t *vp = (const uint16_t *)p.v + b * p.v_b + (int64_t)l * p.v_r + (int64_t)head * p.v_h + dd;
                        op[u] = (uint16_t *)p.dv + b * p.dv_b + (int64_t)l * p.dv_r + (int64_t)head * p.dv_h + dd;
#pragma unroll
                        for (int e = 0; e < CPT / 2; e++) vraw[u][e] = *(const uint32_t *)(vp + 2 * e);
                    }
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        if (rr0 + u < n) {
                            float v4[CPT], dv[CPT];
#pragma unroll
                            for (int e = 0; e < CPT; e += 2) {
                                v4[e] = E::lo(vraw[u][e / 2]);
                                v4[e + 1] = E::hi(vraw[u][e / 2]);
                                dv[e] = dv[e + 1] = 0.f;
                            }
#pragma unroll
                            for (int j = 0; j < HM; j++) {
                                const float ddt = s_ddt[(rr0 + u) * HM + j];  // same address for the whole wave: a broadcast read; 0 beyond Hkv
#pragma unroll
                                for (int e = 0; e < CPT; e++) {
                                    dw[j][e] += ddt * v4[e];
                                    dv[e] += ddt * wj[j][e];
                                }
                            }
#pragma unroll
                            for (int e = 0; e < CPT; e += 2) *(uint32_t *)(op[u] + e) = E::pack2(dv[e], dv[e + 1]);
                        }
                    }
                }
            }
        }
        if (has_cols) {
#pragma unroll
            for (int j = 0; j < HM; j++)
                if (j < Hk) {
#pragma unroll
                    for (int e = 0; e < CPT; e++) part_w[(int64_t)j * K + k0 + e] = dw[j][e];
                }
        }
    }
    // per-head sums: the 256 / HM threads of a head, folded in thread order
    __syncthreads();
    s_red[tid] = sum_a;
    s_red[256 + tid] = sum_pb;
    __syncthreads();
    if (tid < Hk) {
        float sa = 0.f, sb = 0.f;
        for (int t = tid; t < 256; t += HM) {
            sa += s_red[t];
            sb += s_red[256 + t];
        }
        part_w[(int64_t)Hk * K + tid] = sa;
        part_w[(int64_t)Hk * K + Hk + tid] = sb;
    }
}

// Backward, second stage: dW, dA, dpb = sum of the workgroups' partials, in workgroup order.
template <typename T>
__global__ void __launch_bounds__(256) dyn_bias_reduce_kernel(const DynBiasParams p) {
    using E = Elem<T>;
    const int Hk = p.Hk, K = Hk * p.d;
    const int64_t per = (int64_t)Hk * K + 2 * Hk;
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= per) return;
    float s = 0.f;
#pragma unroll 8
    for (int c = 0; c < p.n_wg; c++) s += p.part[c * p.part_stride + e];  // (independent loads, one chain of additions)
    const uint16_t out = (uint16_t)(E::pack2(s, 0.f) & 0xffffu);
    if (e < (int64_t)Hk * K) ((uint16_t *)p.dw)[e] = out;
    else if (e < (int64_t)Hk * K + Hk) ((uint16_t *)p.da)[e - (int64_t)Hk * K] = out;
    else if (p.dpb) ((uint16_t *)p.dpb)[e - (int64_t)Hk * K - Hk] = out;
}

}  // namespace

hipError_t launch_dyn_bias_fwd(const DynBiasParams &p, int dtype, hipStream_t stream) {
    const int64_t n_rows = (int64_t)p.B * p.L;
    if (n_rows <= 0) return hipSuccess;
    if (n_rows < 131072) {  // fewer than 4096 token tiles: split the columns over the waves as well
        const dim3 grid((unsigned)((n_rows + 31) / 32));
        if (dtype == 0) hipLaunchKernelGGL((dyn_bias_fwd_kernel<bf16_tag, true>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((dyn_bias_fwd_kernel<fp16_tag, true>), grid, dim3(256), 0, stream, p);
    } else {
        const dim3 grid((unsigned)((n_rows + 127) / 128));
        if (dtype == 0) hipLaunchKernelGGL((dyn_bias_fwd_kernel<bf16_tag, false>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((dyn_bias_fwd_kernel<fp16_tag, false>), grid, dim3(256), 0, stream, p);
    }
    return hipGetLastError();
}

int dyn_bias_bwd_workgroups(int64_t n_rows, int *rows_per_wg) {
    // runs of 32 tokens while that gives at most 512 workgroups (the partials are Hkv * Hkv * d floats each), else
    // longer runs of whole 64-token passes
    int64_t rows = 32;
    if ((n_rows + 31) / 32 > 512) {
        rows = (n_rows + 511) / 512;
        rows = (rows + 63) / 64 * 64;
    }
    *rows_per_wg = (int)rows;
    return (int)((n_rows + rows - 1) / rows);
}

hipError_t launch_dyn_bias_bwd(const DynBiasParams &p, int dtype, hipStream_t stream) {
    const int64_t n_rows = (int64_t)p.B * p.L;
    if (n_rows <= 0) return hipSuccess;
    auto go = [&](auto kern) { hipLaunchKernelGGL(kern, dim3(p.n_wg), dim3(256), 0, stream, p); };
    const bool wide = p.Hk * p.d >= 1024;  // enough columns for four per thread
    if (dtype == 0) {
        if (p.Hk <= 8) wide ? go(dyn_bias_bwd_kernel<bf16_tag, 8, 4>) : go(dyn_bias_bwd_kernel<bf16_tag, 8, 2>);
        else if (p.Hk <= 16) wide ? go(dyn_bias_bwd_kernel<bf16_tag, 16, 4>) : go(dyn_bias_bwd_kernel<bf16_tag, 16, 2>);
        else go(dyn_bias_bwd_kernel<bf16_tag, 32, 2>);
    } else {
        if (p.Hk <= 8) wide ? go(dyn_bias_bwd_kernel<fp16_tag, 8, 4>) : go(dyn_bias_bwd_kernel<fp16_tag, 8, 2>);
        else if (p.Hk <= 16) wide ? go(dyn_bias_bwd_kernel<fp16_tag, 16, 4>) : go(dyn_bias_bwd_kernel<fp16_tag, 16, 2>);
        else go(dyn_bias_bwd_kernel<fp16_tag, 32, 2>);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t per = (int64_t)p.Hk * p.Hk * p.d + 2 * p.Hk;
    const dim3 grid((unsigned)((per + 255) / 256));
    if (dtype == 0) hipLaunchKernelGGL(dyn_bias_reduce_kernel<bf16_tag>, grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(dyn_bias_reduce_kernel<fp16_tag>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace fdma
