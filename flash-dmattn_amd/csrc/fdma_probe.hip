// Matrix-pipe probe for bench.py (measurement infrastructure, not part of the attention path): what rate of
// v_mfma_f32_32x32x16_bf16 does this device sustain -- register-fed, with one LDS fragment read per MFMA, and with the
// forward kernel's vector work per MFMA on top -- on constant and on random operands?  The published 2.5 PFLOP/s assume
// 2.4 GHz; under the switching activity of real operands the device runs slower, and the attention kernels' roofline
// fraction has to be read against that.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ inline f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ inline uint32_t hash(uint32_t x) {
    x *= 2654435761u; x ^= x >> 13; x *= 0x5bd1e995u; x ^= x >> 15;
    return x;
}
// bf16 pairs: random sign and mantissa, exponent of 0.5 .. 1 (random) or the constant 0.0078 (not random)
__device__ inline uint32_t operand(uint32_t seed, bool random) { return random ? ((hash(seed) & 0x807f807fu) | 0x3f003f00u) : 0x3c003c00u; }

// MODE 0: operands in registers.  1: the A operand of every MFMA comes from LDS (ds_read_b128, four MFMAs ahead).
// 2: mode 1 plus, per MFMA, two exp2, one conversion of two floats to 16 bits and two additions.
// 8 waves per workgroup, one workgroup per CU: two waves per SIMD, as in the attention kernels.
template <int MODE>
__global__ void __launch_bounds__(512, 1) probe_kernel(uint32_t *out, int iters, int random) {
    __shared__ __attribute__((aligned(16))) char lds[36864];
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, g = lane >> 5;
    for (int i = tid; i < 36864 / 4; i += 512) ((uint32_t *)lds)[i] = operand(i + blockIdx.x * 7919u, random != 0);
    __syncthreads();
    const uint32_t base = r * 272 + g * 16;
    f32x16 acc[4];
    for (int j = 0; j < 4; j++)
        for (int i = 0; i < 16; i++) acc[j][i] = 0.f;
    u32x4 b[8];
    for (int j = 0; j < 8; j++)
        for (int e = 0; e < 4; e++) b[j][e] = operand((tid * 8 + j) * 4 + e + 1, random != 0);
    float x[16], s0 = 0.f, s1 = 0.f;
    uint32_t pk[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = 0; i < 16; i++) x[i] = -1.f - 0.01f * i - 0.001f * lane;
    for (int it = 0; it < iters; it++) {
        u32x4 a[16];
        if (MODE >= 1) {
#pragma unroll
            for (int f = 0; f < 4; f++) a[f] = *(const u32x4 *)(lds + base + (f & 7) * 32 + ((it + f) & 1) * 8704);
        }
#pragma unroll
        for (int f = 0; f < 16; f++) {
            if (MODE >= 1) {
                if (f + 4 < 16) a[f + 4] = *(const u32x4 *)(lds + base + ((f + 4) & 7) * 32 + ((it + f) & 1) * 8704 + ((f + 4) >> 3) * 17408);
                acc[f & 3] = mfma(a[f], b[f & 7], acc[f & 3]);
            } else {
                acc[f & 3] = mfma(b[(f + 1) & 7], b[f & 7], acc[f & 3]);
            }
            if (MODE == 2) {
                const int k = f & 7;
                x[2 * k] = __builtin_amdgcn_exp2f(x[2 * k]);
                x[2 * k + 1] = __builtin_amdgcn_exp2f(x[2 * k + 1]);
                const f32x2 ff = {x[2 * k], x[2 * k + 1]};
                pk[k] = __builtin_bit_cast(uint32_t, __builtin_convertvector(ff, bf16x2));
                s0 += x[2 * k];
                s1 += x[2 * k + 1];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = s0 + s1;
    for (int j = 0; j < 4; j++) s += acc[j][0];
    for (int i = 0; i < 8; i++) s += __uint_as_float(pk[i]);
    if (s == 12345.678f) out[0] = 1;  // (keeps the results alive)
}

template <int MODE>
int run(int random, int iters, int wgs, float *ms_out) {
    uint32_t *d_out = nullptr;
    if (hipMalloc(&d_out, 64) != hipSuccess) return -1;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    for (int w = 0; w < 20; w++) hipLaunchKernelGGL(probe_kernel<MODE>, dim3(wgs), dim3(512), 0, 0, d_out, iters, random);  // clock ramp
    (void)hipDeviceSynchronize();
    float best = 1e30f;
    for (int rep = 0; rep < 3; rep++) {
        (void)hipEventRecord(e0, 0);
        hipLaunchKernelGGL(probe_kernel<MODE>, dim3(wgs), dim3(512), 0, 0, d_out, iters, random);
        (void)hipEventRecord(e1, 0);
        (void)hipEventSynchronize(e1);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, e0, e1);
        if (ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(d_out);
    *ms_out = best;
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace

// mode 0 / 1 / 2 as above; random 0 / 1; returns the sustained TFLOP/s of the MFMAs alone (< 0 on error)
extern "C" double fdma_probe_mfma_tflops(int mode, int random) {
    const int iters = 4000, wgs = 256;
    float ms = 0.f;
    int rc = mode == 0 ? run<0>(random, iters, wgs, &ms) : mode == 1 ? run<1>(random, iters, wgs, &ms) : run<2>(random, iters, wgs, &ms);
    if (rc != 0 || ms <= 0.f) return -1.0;
    const double mfmas = (double)wgs * 8 * iters * 16;
    return mfmas * 32768.0 / (ms * 1e-3) / 1e12;
}

// ---- HBM probes: what rate of bytes the device delivers to kernels that do nothing but read, as context for the
// HBM-bound shapes (per-query bias, decode).  `rows` rows of 256 bytes (a K or V row at head dim 128) are read from a
// buffer of `total_rows` rows, 16 lanes x 16 bytes per row, eight rows of a wave in flight per lane -- one after the
// other (a streaming read) or at hashed positions (what decode's gather of the kept keys looks like to the memory).
namespace {

__global__ void __launch_bounds__(256) read_rows_kernel(const u32x4 *base, uint32_t total_rows, uint32_t rows_per_wave, int scattered,
                                                        uint32_t seed, uint32_t *out, int lanes_log2) {
    const uint32_t wave = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    const uint32_t first = wave * rows_per_wave;
    const uint32_t rows_per_load = 64u >> lanes_log2, lanes_mask = (1u << lanes_log2) - 1u;  // (lanes_log2 = 4: rows of 256 bytes)
    u32x4 acc = {0, 0, 0, 0};
    for (uint32_t i = 0; i < rows_per_wave; i += 8 * rows_per_load) {
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t n = first + i + rows_per_load * j + (lane >> lanes_log2);
            uint32_t row = (scattered == 1 ? hash(n ^ seed) : n) & (total_rows - 1);  // (a power of two)
            if (scattered == 2) {
                // the walk of a kernel over tiles of a row-major matrix with rows of 8 KB: a wave's 32 matrix rows, one
                // piece of each, then the next piece of the same rows
                const uint32_t pieces_per_row = 8192u >> (lanes_log2 + 4);
                const uint32_t i = n - first, mrow = (wave * 32 + (i & 31)) & (total_rows / pieces_per_row - 1);
                row = mrow * pieces_per_row + ((i >> 5) & (pieces_per_row - 1));
            }
            v[j] = base[((size_t)row << lanes_log2) + (lane & lanes_mask)];
        }
#pragma unroll
        for (int j = 0; j < 8; j++) acc ^= v[j];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[wave] = acc[0];  // (keeps the loads alive)
}

}  // namespace

// GB/s of one launch that reads `rows` rows of 256 bytes from a buffer of `buffer_mib` MiB (a power of two), scattered or
// not: 32 / 64 / 128 / 256 rows per wave are tried (more, smaller workgroups ramp up faster; fewer, fatter ones issue
// fewer instructions per byte), five timed launches each, and the best launch counts -- launch ramp included (< 0 on error)
extern "C" double fdma_probe_read_rows_gbs(int64_t rows, int row_bytes, int scattered, int buffer_mib);
extern "C" double fdma_probe_read_gbs(int64_t rows, int scattered, int buffer_mib) {
    return fdma_probe_read_rows_gbs(rows, 256, scattered, buffer_mib);
}
// ... the same with rows of 64, 128, 256 or 512 bytes (a mask / bias row of a 64-key tile is 64 / 128 bytes)
extern "C" double fdma_probe_read_rows_gbs(int64_t rows, int row_bytes, int scattered, int buffer_mib) {
    const int lanes_log2 = row_bytes == 64 ? 2 : row_bytes == 128 ? 3 : row_bytes == 256 ? 4 : row_bytes == 512 ? 5 : -1;
    if (lanes_log2 < 0) return -1.0;
    const size_t bytes = (size_t)buffer_mib << 20;
    void *buf = nullptr;
    uint32_t *d_out = nullptr;
    if (rows <= 0 || buffer_mib <= 0 || (buffer_mib & (buffer_mib - 1)) || hipMalloc(&buf, bytes) != hipSuccess) return -1.0;
    const size_t max_waves = (size_t)(rows / (8u * (64u >> lanes_log2)) + 8);
    if (hipMalloc((void **)&d_out, max_waves * sizeof(uint32_t)) != hipSuccess) { (void)hipFree(buf); return -1.0; }
    (void)hipMemset(buf, 0x5a, bytes);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    double best_gbs = -1.0;
    const uint32_t rows_per_pass = 8u * (64u >> lanes_log2);  // rows a wave has in flight
    for (uint32_t rows_per_wave = rows_per_pass; rows_per_wave <= 8 * rows_per_pass; rows_per_wave *= 2) {
        const uint32_t wgs = (uint32_t)((rows + 4 * rows_per_wave - 1) / (4 * rows_per_wave));
        float best = 1e30f;
        for (int rep = 0; rep < 7; rep++) {
            (void)hipEventRecord(e0, 0);
            hipLaunchKernelGGL(read_rows_kernel, dim3(wgs), dim3(256), 0, 0, (const u32x4 *)buf, (uint32_t)(bytes / row_bytes), rows_per_wave,
                               scattered, 0x9e3779b9u * (uint32_t)(rep + 1), d_out, lanes_log2);
            (void)hipEventRecord(e1, 0);
            (void)hipEventSynchronize(e1);
            float ms = 0.f;
            (void)hipEventElapsedTime(&ms, e0, e1);
            if (rep >= 2 && ms < best) best = ms;
        }
        const double gbs = (double)wgs * 4 * rows_per_wave * row_bytes / (best * 1e-3) / 1e9;
        if (best > 0.f && best < 1e29f && gbs > best_gbs) best_gbs = gbs;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(d_out);
    (void)hipFree(buf);
    return hipGetLastError() == hipSuccess ? best_gbs : -1.0;
}

// ---- the walk of the general forward kernel over a per-query bias (2 bytes) and mask (1 byte), without the kernel: 32
// matrices of 4096 x 4096 (cfg3's shapes); a workgroup of four waves owns 128 rows of one matrix and reads 64 columns
// per step -- 128 pieces of 128 bytes at a pitch of 8 KB and 128 pieces of 64 bytes at a pitch of 4 KB, eight rows per
// load instruction --, the next step's loads in flight while it waits for this step's, one barrier per step; with two
// workgroups per CU that is the kernel's own occupancy and depth.  What this reaches is what the access pattern leaves of the
// HBM rate at that occupancy; the kernel's own rate is to be read against it.
namespace {

template <bool MASK, bool BIAS>
__global__ void __launch_bounds__(256, 2) tile_walk_kernel(const char *bias, const char *mask, uint32_t steps, uint32_t *out) {
    const uint32_t tid = threadIdx.x, fc = tid % 8, fr0 = tid / 8;
    const uint32_t mat = blockIdx.x % 32, mblk = (blockIdx.x / 32) % 32;
    const char *bb = bias + (size_t)mat * (4096u * 8192u) + (size_t)(mblk * 128 + fr0) * 8192 + fc * 16;
    const char *mb = mask + (size_t)mat * (4096u * 4096u) + (size_t)(mblk * 128 + fr0) * 4096 + fc * 8;
    u32x4 acc = {0, 0, 0, 0};
    u32x4 b0[4], b1[4];
    uint2 m0[4], m1[4];
    auto ld = [&](uint32_t st, u32x4 (&b)[4], uint2 (&m)[4]) {
#pragma unroll
        for (int it = 0; it < 4; it++) {
            if (MASK) m[it] = *(const uint2 *)(mb + (size_t)it * 32 * 4096 + st * 64);
            if (BIAS) b[it] = *(const u32x4 *)(bb + (size_t)it * 32 * 8192 + st * 128);
        }
    };
    auto use = [&](u32x4 (&b)[4], uint2 (&m)[4]) {
#pragma unroll
        for (int it = 0; it < 4; it++) {
            if (BIAS) acc ^= b[it];
            if (MASK) { acc[0] ^= m[it].x; acc[1] ^= m[it].y; }
        }
    };
    ld(0, b0, m0);
    for (uint32_t st = 0; st < steps; st += 2) {  // (steps is even and at most 62: step `steps` still lies inside the row)
        ld(st + 1, b1, m1);
        use(b0, m0);
        __builtin_amdgcn_s_barrier();
        ld(st + 2, b0, m0);
        use(b1, m1);
        __builtin_amdgcn_s_barrier();
    }
    use(b0, m0);
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[blockIdx.x] = acc[0];  // (keeps the loads alive)
}

}  // namespace

// GB/s of that walk: 1024 workgroups x 32 steps (0.8 GB with mask and bias), best of four timed launches (< 0 on error).
// `lds_kb`: LDS per workgroup, which sets how many a CU holds (64: two, as the forward kernel; 0: as many as the launch has, four)
extern "C" double fdma_probe_tile_walk_gbs(int with_mask, int with_bias, int lds_kb) {
    if ((!with_mask && !with_bias) || lds_kb > 64) return -1.0;
    void *bias = nullptr, *mask = nullptr;
    uint32_t *d_out = nullptr;
    if (hipMalloc(&bias, (size_t)32 * 4096 * 8192) != hipSuccess) return -1.0;
    if (hipMalloc(&mask, (size_t)32 * 4096 * 4096) != hipSuccess) { (void)hipFree(bias); return -1.0; }
    if (hipMalloc((void **)&d_out, 1024 * sizeof(uint32_t)) != hipSuccess) { (void)hipFree(bias); (void)hipFree(mask); return -1.0; }
    (void)hipMemset(bias, 0x5a, (size_t)32 * 4096 * 8192);
    (void)hipMemset(mask, 0x01, (size_t)32 * 4096 * 4096);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    const uint32_t steps = 32;
    const size_t lds = lds_kb > 0 ? (size_t)lds_kb << 10 : 0;  // (dynamic LDS nobody touches: it only limits the workgroups a CU holds)
    float best = 1e30f;
    for (int rep = 0; rep < 6; rep++) {
        (void)hipEventRecord(e0, 0);
        if (with_mask && with_bias) hipLaunchKernelGGL((tile_walk_kernel<true, true>), dim3(1024), dim3(256), lds, 0, (const char *)bias, (const char *)mask, steps, d_out);
        else if (with_bias) hipLaunchKernelGGL((tile_walk_kernel<false, true>), dim3(1024), dim3(256), lds, 0, (const char *)bias, (const char *)mask, steps, d_out);
        else hipLaunchKernelGGL((tile_walk_kernel<true, false>), dim3(1024), dim3(256), lds, 0, (const char *)bias, (const char *)mask, steps, d_out);
        (void)hipEventRecord(e1, 0);
        (void)hipEventSynchronize(e1);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, e0, e1);
        if (rep >= 2 && ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(d_out);
    (void)hipFree(mask);
    (void)hipFree(bias);
    const double bytes = 1024.0 * steps * 128 * ((with_bias ? 128 : 0) + (with_mask ? 64 : 0));
    return hipGetLastError() == hipSuccess && best < 1e29f ? bytes / (best * 1e-3) / 1e9 : -1.0;
}
