// Kernel argument blocks (device side) and the launch functions each .hip file exports to the
// C-ABI layer in fdma_api.cpp.  Plays the role of the reference's Flash_fwd_params /
// Flash_bwd_params (csrc/flash_sparse_attn/src/flash.h:20-198) without any torch types.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

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
    int32_t ld;            // row stride of the arrays above (Lk rounded up to 16)
    int32_t Hfb;           // heads of fb: Hk, or H when the bias differs per query head
    int32_t on;            // 0 = no compaction: k / v are the caller's tensors
};

struct FwdParams {
    const void *q, *k, *v;
    const uint8_t *mask;  // nullptr = absent
    const void *bias;     // nullptr = absent
    void *o;
    float *lse;           // (B, H, Lq)
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
    Compact cmp;        // when cmp.on, k / v (and their strides) describe the compacted copies
};

struct BwdParams {
    FwdParams f;  // f.o = forward output (read), f.lse = forward LSE (read)
    const void *dout;
    void *dq, *dk, *dv, *dbias;
    int64_t do_b, do_r, do_h;
    int64_t dq_b, dq_r, dq_h;
    int64_t dk_b, dk_r, dk_h;
    int64_t dv_b, dv_r, dv_h;
    int64_t db_b, db_h, db_r;  // dbias strides (batch, head, row); 0 = broadcast
    float *softmax_d;          // (B, H, Lq_rounded)
    int32_t Lq_rounded;
    float *dbias_accum;        // fp32 scratch at the dbias shape when several workgroups share an element
    int64_t dba_b, dba_h, dba_r;
};

// dtype: 0 = bf16, 1 = fp16.  All launches are asynchronous on `stream`; return hipError_t.
hipError_t launch_fwd(const FwdParams &p, int dtype, hipStream_t stream);
// column-mask specialisation (mask / bias absent or broadcast over queries); nq = 32-row blocks per wave
bool fwd_colmask_applicable(const FwdParams &p);
hipError_t launch_fwd_colmask(const FwdParams &p, int dtype, int nq, hipStream_t stream);
hipError_t launch_fwd_decode(const FwdParams &p, int dtype, hipStream_t stream);
hipError_t launch_bwd(const BwdParams &p, int dtype, hipStream_t stream);
// column-mask specialisations of the two main backward kernels
bool bwd_colmask_applicable(const BwdParams &p);
hipError_t launch_bwd_dkdv_colmask(const BwdParams &p, int dtype, hipStream_t stream);
hipError_t launch_bwd_dq_colmask(const BwdParams &p, int dtype, hipStream_t stream);

// Column compaction: use_compact() decides from the problem alone (no device data), compact_bytes() is
// the scratch it needs, compact_setup() launches the gather pre-pass into `ws` and rewrites p.k / p.v /
// p.cmp; compact_zero_dropped() zero-fills the gradient rows / columns of dropped keys.
bool use_compact(const FwdParams &p);
size_t compact_bytes(const FwdParams &p);
hipError_t compact_setup(FwdParams &p, void *ws, int dtype, hipStream_t stream);
hipError_t compact_zero_dropped(const BwdParams &p, const FwdParams &orig, hipStream_t stream);

// number of KV splits the decode path uses for this shape (1 = no workspace needed)
int decode_num_splits(int B, int Hk, int Lk);
bool use_decode_path(int Lq, int H, int Hk);

}  // namespace fdma
