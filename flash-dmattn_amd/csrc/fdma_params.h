// Kernel argument blocks (device side) and the launch functions each .hip file exports to the
// C-ABI layer in fdma_api.cpp.  Plays the role of the reference's Flash_fwd_params /
// Flash_bwd_params (csrc/flash_sparse_attn/src/flash.h:20-198) without any torch types.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fdma {

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

// number of KV splits the decode path uses for this shape (1 = no workspace needed)
int decode_num_splits(int B, int Hk, int Lk);
bool use_decode_path(int Lq, int H, int Hk);

}  // namespace fdma
