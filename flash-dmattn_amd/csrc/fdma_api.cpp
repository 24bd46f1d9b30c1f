// C-ABI layer of libfdma_hip.so: argument validation, kernel-parameter set-up and dispatch.
//
// Host-side counterpart of mha_fwd / mha_bwd with set_params_fprop / set_params_dgrad
// (csrc/flash_sparse_attn/flash_api.cpp:24-249, 351-554, 792-1050 of the reference).  The checks and
// their messages follow the reference's TORCH_CHECKs so callers see the same errors; everything
// torch-specific (allocation, device guard, current stream) stays with the caller.
#include "../../include/fdma.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "fdma_params.h"

namespace {

thread_local char g_err[512] = "";

constexpr int64_t kMaxRowStride = (int64_t)1 << 24;  // elements

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

bool strides_ok(const int64_t s[3], int mult) {
    for (int i = 0; i < 3; i++)
        if (s[i] % mult != 0) return false;
    return true;
}

// Shape / dtype / stride rules of flash_api.cpp:371-438 (forward) -- shared by backward (:824-898).
int validate_common(const fdma_fwd_args *a, bool backward) {
    if (!a) return fail(FDMA_ERR_INVALID, "args must not be NULL");
    if (a->dtype != FDMA_DTYPE_BF16 && a->dtype != FDMA_DTYPE_FP16)
        return fail(FDMA_ERR_INVALID, "FlashSparseAttention only support fp16 and bf16 data type");
    if (a->batch <= 0) return fail(FDMA_ERR_INVALID, "batch size must be positive");
    if (a->seqlen_q < 0 || a->seqlen_k < 0) return fail(FDMA_ERR_INVALID, "sequence lengths must be non-negative");
    if (a->num_heads <= 0 || a->num_heads_k <= 0) return fail(FDMA_ERR_INVALID, "number of heads must be positive");
    if (a->head_dim > 256)
        return fail(FDMA_ERR_INVALID, "FlashSparseAttention %s only supports head dimension at most 256", backward ? "backward" : "forward");
    if (a->head_dim <= 0 || a->head_dim % 8 != 0)
        return fail(FDMA_ERR_INVALID, backward ? "head_size should be a multiple of 8"
                                               : "query, key, value, and out_ must have a head_size that is a multiple of 8");
    if (a->mask_bits.bits) {
        if (!a->mask) return fail(FDMA_ERR_INVALID, "mask_bits without a mask");
        // (broadcast exactly where the mask is: a zero stride of one and not of the other would describe two masks)
        for (int i = 0; i < 3; i++)
            if ((a->mask_bits.strides[i] == 0) != (a->mask_strides[i] == 0))
                return fail(FDMA_ERR_INVALID, "mask_bits must be broadcast over the same dimensions as the mask");
        if (a->seqlen_q > 1 && a->mask_bits.strides[2] != 0 && a->mask_bits.strides[2] < ((a->seqlen_k + 7) / 8 + 7) / 8 * 8)
            return fail(FDMA_ERR_INVALID, "mask_bits rows must hold ceil(seqlen_k / 8) bytes rounded up to 8");
        if ((reinterpret_cast<uintptr_t>(a->mask_bits.bits) | (uintptr_t)a->mask_bits.strides[0] | (uintptr_t)a->mask_bits.strides[1] |
             (uintptr_t)a->mask_bits.strides[2]) & 7)
            return fail(FDMA_ERR_INVALID, "mask_bits and its strides must be multiples of 8 bytes");
    }
    if (a->kept.idx || a->kept.cnt || a->kept.count) {
        if (!(a->kept.idx && a->kept.cnt && a->kept.count))
            return fail(FDMA_ERR_INVALID, "kept: idx, cnt and count must be given together");
        if (a->kept.ld < a->seqlen_k || a->kept.ld % 16 != 0)
            return fail(FDMA_ERR_INVALID, "kept.ld must be a multiple of 16 and at least seqlen_k");
        if ((reinterpret_cast<uintptr_t>(a->kept.cnt) | reinterpret_cast<uintptr_t>(a->kept.idx)) & 15)
            return fail(FDMA_ERR_INVALID, "kept.idx and kept.cnt must be 16-byte aligned");
    }
    if (a->num_heads % a->num_heads_k != 0)
        return fail(FDMA_ERR_INVALID, "Number of heads in key/value must divide number of heads in query");
    if (!a->q || ((!a->k || !a->v) && a->seqlen_k > 0)) return fail(FDMA_ERR_INVALID, "q, k, v must be device pointers");
    if (!a->out) return fail(FDMA_ERR_INVALID, "out must be a device pointer");
    if (!a->lse) return fail(FDMA_ERR_INVALID, "softmax_lse must be a device pointer");
    if (a->mask) {
        const int hm = a->num_heads_mask;
        if (!(hm == 1 || hm == a->num_heads_k || hm == a->num_heads))
            return fail(FDMA_ERR_INVALID, "Number of heads in mask must be 1, h_k or h");
        if (!aligned16(a->mask) || !strides_ok(a->mask_strides, 16))
            return fail(FDMA_ERR_INVALID, "mask must be 16-byte aligned with strides that are multiples of 16 (pad the key dimension)");
    }
    if (a->bias) {
        const int hb = a->num_heads_bias;
        if (!(hb == 1 || hb == a->num_heads_k || hb == a->num_heads))
            return fail(FDMA_ERR_INVALID, "Number of heads in bias must be 1, h_k or h");
        if (!aligned16(a->bias) || !strides_ok(a->bias_strides, 8))
            return fail(FDMA_ERR_INVALID, "bias must be 16-byte aligned with strides that are multiples of 8 (pad the key dimension)");
    }
    if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->out) || !strides_ok(a->q_strides, 8) ||
        !strides_ok(a->k_strides, 8) || !strides_ok(a->v_strides, 8) || !strides_ok(a->o_strides, 8))
        return fail(FDMA_ERR_INVALID, "q, k, v, out must be 16-byte aligned with strides that are multiples of 8 elements");
    // the kernels address the rows of a tile with 32-bit byte offsets from a 64-bit tile base
    if (a->q_strides[1] >= kMaxRowStride || a->k_strides[1] >= kMaxRowStride || a->v_strides[1] >= kMaxRowStride)
        return fail(FDMA_ERR_UNSUPPORTED, "q, k, v row strides of 2^24 elements or more are not supported");
    if (a->softcap != 0.f) return fail(FDMA_ERR_UNSUPPORTED, "softcap is not supported by this build");
    if (!std::isfinite(a->softmax_scale)) return fail(FDMA_ERR_INVALID, "softmax_scale must be finite");
    if (a->compact_mode < FDMA_COMPACT_AUTO || a->compact_mode > FDMA_COMPACT_ALWAYS)
        return fail(FDMA_ERR_INVALID, "compact_mode must be FDMA_COMPACT_AUTO, _NEVER or _ALWAYS (got %d)", a->compact_mode);
    return FDMA_OK;
}

void fill_fwd_params(const fdma_fwd_args *a, fdma::FwdParams &p) {
    std::memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.v = a->v;
    p.mask = static_cast<const uint8_t *>(a->mask);
    p.bias = a->bias;
    p.o = a->out;
    p.lse = a->lse;
    p.q_b = a->q_strides[0]; p.q_r = a->q_strides[1]; p.q_h = a->q_strides[2];
    p.k_b = a->k_strides[0]; p.k_r = a->k_strides[1]; p.k_h = a->k_strides[2];
    p.v_b = a->v_strides[0]; p.v_r = a->v_strides[1]; p.v_h = a->v_strides[2];
    p.o_b = a->o_strides[0]; p.o_r = a->o_strides[1]; p.o_h = a->o_strides[2];
    if (a->mask) { p.m_b = a->mask_strides[0]; p.m_h = a->mask_strides[1]; p.m_r = a->seqlen_q == 1 ? 0 : a->mask_strides[2]; }
    if (a->bias) { p.bi_b = a->bias_strides[0]; p.bi_h = a->bias_strides[1]; p.bi_r = a->seqlen_q == 1 ? 0 : a->bias_strides[2]; }
    p.B = a->batch; p.Lq = a->seqlen_q; p.Lk = a->seqlen_k;
    p.H = a->num_heads; p.Hk = a->num_heads_k;
    p.Hm = a->mask ? a->num_heads_mask : 1;
    p.Hb = a->bias ? a->num_heads_bias : 1;
    p.d = a->head_dim;
    // seqlen_q == 1 makes causal a no-op (flash_api.cpp:441)
    p.causal = (a->is_causal && a->seqlen_q != 1) ? 1 : 0;
    p.scale = a->softmax_scale;
    p.scale_log2 = a->softmax_scale * 1.4426950408889634f;
    p.splits = 1;
    p.compact_mode = a->compact_mode;
    if (a->mask && a->kept.idx && a->kept.cnt && a->kept.count) {  // (validate_common has checked the row stride)
        p.kept_idx = a->kept.idx; p.kept_cnt = a->kept.cnt; p.kept_count = a->kept.count;
        p.kept_ld = a->kept.ld;
    }
    if (a->mask && a->mask_bits.bits) {
        p.mbits = a->mask_bits.bits;
        p.mb_b = a->mask_bits.strides[0]; p.mb_h = a->mask_bits.strides[1];
        p.mb_r = a->seqlen_q == 1 ? 0 : a->mask_bits.strides[2];
    }
    p.lse_b = (int64_t)a->num_heads * a->seqlen_q;
    p.lse_h = a->seqlen_q;
}

// Ragged batch: rules of flash_api.cpp:583-660 (forward), shared by backward (:1090-1150).
int validate_varlen(const fdma_varlen_fwd_args *a, bool backward) {
    if (!a) return fail(FDMA_ERR_INVALID, "args must not be NULL");
    if (a->dtype != FDMA_DTYPE_BF16 && a->dtype != FDMA_DTYPE_FP16)
        return fail(FDMA_ERR_INVALID, "FlashSparseAttention only support fp16 and bf16 data type");
    if (a->batch <= 0) return fail(FDMA_ERR_INVALID, "batch size must be positive");
    if (a->total_q < 0 || a->total_k < 0 || a->max_seqlen_q < 0 || a->max_seqlen_k < 0)
        return fail(FDMA_ERR_INVALID, "sequence lengths must be non-negative");
    if (a->num_heads <= 0 || a->num_heads_k <= 0) return fail(FDMA_ERR_INVALID, "number of heads must be positive");
    if (a->head_dim > 256)
        return fail(FDMA_ERR_INVALID, "FlashSparseAttention %s only supports head dimension at most 256", backward ? "backward" : "forward");
    if (a->head_dim <= 0 || a->head_dim % 8 != 0)
        return fail(FDMA_ERR_INVALID, backward ? "head_size should be a multiple of 8"
                                               : "query, key, value, and out_ must have a head_size that is a multiple of 8");
    if (a->num_heads % a->num_heads_k != 0)
        return fail(FDMA_ERR_INVALID, "Number of heads in key/value must divide number of heads in query");
    if (!a->cu_seqlens_q || !a->cu_seqlens_k) return fail(FDMA_ERR_INVALID, "cu_seqlens_q and cu_seqlens_k must be device pointers");
    if ((reinterpret_cast<uintptr_t>(a->cu_seqlens_q) | reinterpret_cast<uintptr_t>(a->cu_seqlens_k)) & 3)
        return fail(FDMA_ERR_INVALID, "cu_seqlens_q and cu_seqlens_k must be 4-byte aligned int32 arrays");
    if ((!a->q && a->total_q > 0) || ((!a->k || !a->v) && a->total_k > 0)) return fail(FDMA_ERR_INVALID, "q, k, v must be device pointers");
    if (a->total_q > 0 && !a->out) return fail(FDMA_ERR_INVALID, "out must be a device pointer");
    if (a->total_q > 0 && !a->lse) return fail(FDMA_ERR_INVALID, "softmax_lse must be a device pointer");
    const int64_t *st[4] = {a->q_strides, a->k_strides, a->v_strides, a->o_strides};
    for (int i = 0; i < 4; i++)
        if (st[i][0] % 8 != 0 || st[i][1] % 8 != 0)
            return fail(FDMA_ERR_INVALID, "q, k, v, out must be 16-byte aligned with strides that are multiples of 8 elements");
    if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->out))
        return fail(FDMA_ERR_INVALID, "q, k, v, out must be 16-byte aligned with strides that are multiples of 8 elements");
    if (a->q_strides[0] >= kMaxRowStride || a->k_strides[0] >= kMaxRowStride || a->v_strides[0] >= kMaxRowStride)
        return fail(FDMA_ERR_UNSUPPORTED, "q, k, v row strides of 2^24 elements or more are not supported");
    if (a->softcap != 0.f) return fail(FDMA_ERR_UNSUPPORTED, "softcap is not supported by this build");
    if (!std::isfinite(a->softmax_scale)) return fail(FDMA_ERR_INVALID, "softmax_scale must be finite");
    return FDMA_OK;
}

// The ragged batch runs through the column-mask kernels (no mask, no bias): batch strides 0, per-entry first rows
// and lengths from cu_seqlens on the device, grids sized by the longest sequences.
int fill_varlen_params(const fdma_varlen_fwd_args *a, fdma::FwdParams &p) {
    std::memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.v = a->v;
    p.o = a->out;
    p.lse = a->lse;
    p.q_r = a->q_strides[0]; p.q_h = a->q_strides[1];
    p.k_r = a->k_strides[0]; p.k_h = a->k_strides[1];
    p.v_r = a->v_strides[0]; p.v_h = a->v_strides[1];
    p.o_r = a->o_strides[0]; p.o_h = a->o_strides[1];
    p.B = a->batch;
    p.Lq = a->max_seqlen_q < a->total_q ? a->max_seqlen_q : a->total_q;
    p.Lk = a->max_seqlen_k < a->total_k ? a->max_seqlen_k : a->total_k;
    p.H = a->num_heads; p.Hk = a->num_heads_k;
    p.Hm = 1; p.Hb = 1;
    p.d = a->head_dim;
    p.causal = (a->is_causal && a->max_seqlen_q != 1) ? 1 : 0;  // flash_api.cpp:628
    p.scale = a->softmax_scale;
    p.scale_log2 = a->softmax_scale * 1.4426950408889634f;
    p.splits = 1;
    p.lse_b = 0;
    p.lse_h = a->total_q;
    p.cu_q = a->cu_seqlens_q; p.cu_k = a->cu_seqlens_k;
    p.total_q = a->total_q; p.total_k = a->total_k;
    if (!fdma::fwd_colmask_applicable(p))
        return fail(FDMA_ERR_UNSUPPORTED, "ragged batches with sequences of more than 2^19 keys are not supported (max_seqlen_k = %d)", a->max_seqlen_k);
    return FDMA_OK;
}

}  // namespace

// Scratch of fdma_fwd_noalloc: one array per GPU, part of the library's code object, alive until the process ends.
// In host code the name below is only a handle for hipGetSymbolAddress -- it is not a device address; the address
// that kernels and copies may use is looked up once per device (each GPU has its own copy at its own address).
static __device__ __align__(256) unsigned char scratch[FDMA_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int kScratchDevices = 64;
std::atomic<void *> g_scratch_ptr[kScratchDevices];

// device address of `scratch` on the current device
int scratch_of_current_device(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "hipGetDevice failed: %s", hipGetErrorString(e));
    const bool cached = dev >= 0 && dev < kScratchDevices;
    void *ptr = cached ? g_scratch_ptr[dev].load(std::memory_order_acquire) : nullptr;
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(FDMA_ERR_LAUNCH, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
        if (cached) g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return FDMA_OK;
}

// A stream that is being captured into a HIP graph is refused: the one capture of forward + backward through the
// tensor library ended in a host-side crash when the capture was closed, the cause is not known, and until it is
// the library does not record its launches into graphs.  A clear error here replaces that crash.
int refuse_capture(void *hip_stream, const char *who) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    const hipError_t e = hipStreamIsCapturing(static_cast<hipStream_t>(hip_stream), &st);
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "%s: hipStreamIsCapturing failed: %s", who, hipGetErrorString(e));
    if (st != hipStreamCaptureStatusNone)
        return fail(FDMA_ERR_UNSUPPORTED, "%s: the stream is being captured into a HIP graph; capture of this library's launches is not supported", who);
    return FDMA_OK;
}

}  // namespace

extern "C" {

const char *fdma_last_error(void) { return g_err; }
int fdma_abi_version(void) { return FDMA_ABI_VERSION; }
size_t fdma_sizeof_fwd_args(void) { return sizeof(fdma_fwd_args); }
size_t fdma_sizeof_bwd_args(void) { return sizeof(fdma_bwd_args); }

int fdma_fwd_validate(const fdma_fwd_args *a) {
    g_err[0] = 0;
    return validate_common(a, false);
}

int fdma_set_stream_min_items(int n) {
    const int before = fdma::get_stream_min_items();
    if (n > 0) fdma::set_stream_min_items(n);
    return before;
}

size_t fdma_fwd_counter_bytes(const fdma_fwd_args *a) {
    if (!a || a->seqlen_k <= 0 || a->num_heads_k <= 0 || !fdma::use_decode_path(a->seqlen_q, a->num_heads, a->num_heads_k)) return 0;
    return (size_t)round_up(fdma::decode_num_counters(a->batch, a->num_heads, a->num_heads_k, a->seqlen_k) * 4, 256);
}

size_t fdma_fwd_workspace_bytes(const fdma_fwd_args *a) {
    if (!a) return 0;
    if (!fdma::use_decode_path(a->seqlen_q, a->num_heads, a->num_heads_k)) {
        fdma::FwdParams p, pv;
        fill_fwd_params(a, p);
        if (fdma::compact_per_query_head(p, pv)) return fdma::compact_bytes(pv, false);
        return fdma::use_compact(p) ? fdma::compact_bytes(p, false) : 0;
    }
    const int splits = fdma::decode_num_splits(a->batch, a->num_heads_k, a->seqlen_k);
    if (splits <= 1) return 0;
    const size_t rows = (size_t)splits * a->batch * a->num_heads * a->seqlen_q;
    return rows * (size_t)(a->head_dim + 1) * sizeof(float);
}

int fdma_fwd(const fdma_fwd_args *a, void *hip_stream) {
    if (int cap = refuse_capture(hip_stream, "fdma_fwd")) return cap;
    g_err[0] = 0;
    int rc = validate_common(a, false);
    if (rc != FDMA_OK) return rc;
    fdma::FwdParams p;
    fill_fwd_params(a, p);
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    hipError_t e;
    if (a->seqlen_q == 0) return FDMA_OK;
    if (fdma::use_decode_path(a->seqlen_q, a->num_heads, a->num_heads_k) && a->seqlen_k > 0) {
        p.splits = fdma::decode_num_splits(a->batch, a->num_heads_k, a->seqlen_k);
        if (p.splits > 1) {
            const size_t need = fdma_fwd_workspace_bytes(a);
            if (!a->workspace || a->workspace_bytes < need)
                return fail(FDMA_ERR_WORKSPACE, "forward workspace too small: need %zu bytes, got %zu", need, a->workspace_bytes);
            const size_t rows = (size_t)p.splits * a->batch * a->num_heads * a->seqlen_q;
            p.o_part = static_cast<float *>(a->workspace);
            p.lse_part = p.o_part + rows * a->head_dim;
            if (a->counters) {
                const size_t cneed = fdma_fwd_counter_bytes(a);
                if (a->counters_bytes < cneed)
                    return fail(FDMA_ERR_WORKSPACE, "decode arrival counters too small: need %zu bytes, got %zu", cneed, a->counters_bytes);
                if (reinterpret_cast<uintptr_t>(a->counters) & 3) return fail(FDMA_ERR_INVALID, "counters must be 4-byte aligned");
                p.dec_counter = a->counters;
            }
        }
        e = fdma::launch_fwd_decode(p, a->dtype, stream);
    } else {
        // seqlen_k == 0 falls out of the kernel as O = 0, LSE = +inf (flash_api.cpp:535-539)
        // (a query-broadcast mask with a row per query head: compacted per query head -- forward only; the backward of
        // that form skips tiles instead)
        fdma::FwdParams pv;
        if (fdma::compact_per_query_head(p, pv)) p = pv;
        if (fdma::use_compact(p)) {
            const size_t need = fdma::compact_bytes(p, false);
            if (!a->workspace || a->workspace_bytes < need)
                return fail(FDMA_ERR_WORKSPACE, "forward workspace too small: need %zu bytes, got %zu", need, a->workspace_bytes);
            if ((e = fdma::compact_setup(p, a->workspace, a->dtype, stream)) != hipSuccess)
                return fail(FDMA_ERR_LAUNCH, "forward launch failed: %s", hipGetErrorString(e));
        }
        e = fdma::launch_fwd(p, a->dtype, stream);
    }
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "forward launch failed: %s", hipGetErrorString(e));
    return FDMA_OK;
}

int fdma_fwd_noalloc(const fdma_fwd_args *a, void *hip_stream) {
    g_err[0] = 0;
    int rc = validate_common(a, false);
    if (rc != FDMA_OK) return rc;
    const size_t need = fdma_fwd_workspace_bytes(a);
    constexpr size_t kUsable = (size_t)FDMA_NOALLOC_SCRATCH_BYTES - FDMA_NOALLOC_COUNTER_BYTES;
    if (need > kUsable)
        return fail(FDMA_ERR_WORKSPACE, "fdma_fwd_noalloc: this problem needs %zu bytes of scratch, the library's static scratch holds %zu",
                    need, kUsable);
    fdma_fwd_args with_scratch = *a;
    with_scratch.workspace = nullptr;
    with_scratch.workspace_bytes = 0;
    with_scratch.counters = nullptr;
    with_scratch.counters_bytes = 0;
    if (need) {
        void *ptr = nullptr;
        if ((rc = scratch_of_current_device(&ptr)) != FDMA_OK) return rc;
        with_scratch.workspace = ptr;
        with_scratch.workspace_bytes = kUsable;
        // the array's tail: zero since the library was loaded, put back to zero by every decode call that used it
        // (more counters than fit there: the merge stays a launch of its own)
        if (fdma_fwd_counter_bytes(a) <= (size_t)FDMA_NOALLOC_COUNTER_BYTES) {
            with_scratch.counters = reinterpret_cast<int32_t *>(static_cast<unsigned char *>(ptr) + kUsable);
            with_scratch.counters_bytes = FDMA_NOALLOC_COUNTER_BYTES;
        }
    }
    return fdma_fwd(&with_scratch, hip_stream);
}

int fdma_bwd_validate(const fdma_bwd_args *a) {
    g_err[0] = 0;
    if (!a) return fail(FDMA_ERR_INVALID, "args must not be NULL");
    int rc = validate_common(&a->f, true);
    if (rc != FDMA_OK) return rc;
    if (!a->dout || !a->dq || !a->dk || !a->dv) return fail(FDMA_ERR_INVALID, "dout, dq, dk, dv must be device pointers");
    if (!a->softmax_d) return fail(FDMA_ERR_INVALID, "softmax_d must be a device pointer");
    if ((a->f.bias != nullptr) != (a->dbias != nullptr))
        return fail(FDMA_ERR_INVALID, "dbias must be given exactly when bias is given");
    if (!aligned16(a->dout) || !aligned16(a->dq) || !aligned16(a->dk) || !aligned16(a->dv) || !strides_ok(a->do_strides, 8) ||
        !strides_ok(a->dq_strides, 8) || !strides_ok(a->dk_strides, 8) || !strides_ok(a->dv_strides, 8))
        return fail(FDMA_ERR_INVALID, "dout, dq, dk, dv must be 16-byte aligned with strides that are multiples of 8 elements");
    if (a->do_strides[1] >= kMaxRowStride)
        return fail(FDMA_ERR_UNSUPPORTED, "dout row strides of 2^24 elements or more are not supported");
    if (a->dbias) {
        if (!aligned16(a->dbias) || !strides_ok(a->dbias_strides, 8))
            return fail(FDMA_ERR_INVALID, "dbias must be 16-byte aligned with strides that are multiples of 8");
        for (int i = 0; i < 3; i++)
            if ((a->dbias_strides[i] == 0) != (a->f.bias_strides[i] == 0))
                return fail(FDMA_ERR_INVALID, "dbias must have the broadcast pattern of bias");
    }
    return FDMA_OK;
}

// fp32 accumulation scratch for dbias when several workgroups add into one dbias element:
// bias broadcast over batch (with batch > 1) or over kv-head groups (bias heads == 1 < Hk).
static bool dbias_shared(const fdma_bwd_args *a) {
    if (!a->dbias) return false;
    const bool batch_bcast = a->f.batch > 1 && a->f.bias_strides[0] == 0;
    const bool head_bcast = a->f.num_heads_bias == 1 && a->f.num_heads_k > 1;
    return batch_bcast || head_bcast;
}

static size_t dbias_accum_elems(const fdma_bwd_args *a) {
    const size_t nb = a->f.bias_strides[0] == 0 ? 1 : a->f.batch;
    const size_t nr = a->f.bias_strides[2] == 0 ? 1 : a->f.seqlen_q;
    return nb * a->f.num_heads_bias * nr * (size_t)round_up(a->f.seqlen_k, 8);
}

static size_t dbias_accum_bytes(const fdma_bwd_args *a) {
    return dbias_shared(a) ? (size_t)round_up(dbias_accum_elems(a) * sizeof(float), 256) : 0;
}

size_t fdma_bwd_workspace_bytes(const fdma_bwd_args *a) {
    if (!a) return 0;
    fdma::FwdParams p;
    fill_fwd_params(&a->f, p);
    return dbias_accum_bytes(a) + (fdma::use_compact(p) ? fdma::compact_bytes(p, true, a->fwd_workspace != nullptr) : 0);
}

int fdma_bwd(const fdma_bwd_args *a, void *hip_stream) {
    if (int cap = refuse_capture(hip_stream, "fdma_bwd")) return cap;
    int rc = fdma_bwd_validate(a);
    if (rc != FDMA_OK) return rc;
    fdma::BwdParams p;
    std::memset(&p, 0, sizeof(p));
    fill_fwd_params(&a->f, p.f);
    p.dout = a->dout; p.dq = a->dq; p.dk = a->dk; p.dv = a->dv; p.dbias = a->dbias;
    p.do_b = a->do_strides[0]; p.do_r = a->do_strides[1]; p.do_h = a->do_strides[2];
    p.dq_b = a->dq_strides[0]; p.dq_r = a->dq_strides[1]; p.dq_h = a->dq_strides[2];
    p.dk_b = a->dk_strides[0]; p.dk_r = a->dk_strides[1]; p.dk_h = a->dk_strides[2];
    p.dv_b = a->dv_strides[0]; p.dv_r = a->dv_strides[1]; p.dv_h = a->dv_strides[2];
    if (a->dbias) { p.db_b = a->dbias_strides[0]; p.db_h = a->dbias_strides[1]; p.db_r = a->dbias_strides[2]; }
    p.softmax_d = a->softmax_d;
    p.Lq_rounded = (int32_t)round_up(a->f.seqlen_q, 128);
    p.sd_b = (int64_t)a->f.num_heads * p.Lq_rounded;
    p.sd_h = p.Lq_rounded;
    const size_t need = fdma_bwd_workspace_bytes(a);
    if (need && (!a->workspace || a->workspace_bytes < need))
        return fail(FDMA_ERR_WORKSPACE, "backward workspace too small: need %zu bytes, got %zu", need, a->workspace_bytes);
    if (dbias_shared(a)) {
        p.dbias_accum = static_cast<float *>(a->workspace);
        const int64_t lkr = round_up(a->f.seqlen_k, 8);
        const int64_t nr = a->f.bias_strides[2] == 0 ? 1 : a->f.seqlen_q;
        p.dba_r = a->f.bias_strides[2] == 0 ? 0 : lkr;
        p.dba_h = nr * lkr;
        p.dba_b = a->f.bias_strides[0] == 0 ? 0 : p.dba_h * a->f.num_heads_bias;
    }
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    hipError_t e;
    if (a->f.seqlen_q > 0 && fdma::use_compact(p.f)) {
        if (a->fwd_workspace && a->fwd_workspace_bytes < fdma::compact_bytes(p.f, false))
            return fail(FDMA_ERR_WORKSPACE, "fwd_workspace too small: the forward call of this problem needs %zu bytes, got %zu",
                        fdma::compact_bytes(p.f, false), a->fwd_workspace_bytes);
        e = fdma::compact_setup(p.f, static_cast<char *>(a->workspace) + dbias_accum_bytes(a), a->f.dtype, stream, &p,
                                a->fwd_workspace);
        if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "backward launch failed: %s", hipGetErrorString(e));
    }
    e = fdma::launch_bwd(p, a->f.dtype, stream);
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "backward launch failed: %s", hipGetErrorString(e));
    return FDMA_OK;
}

size_t fdma_sizeof_varlen_fwd_args(void) { return sizeof(fdma_varlen_fwd_args); }
size_t fdma_sizeof_varlen_bwd_args(void) { return sizeof(fdma_varlen_bwd_args); }

int fdma_varlen_fwd_validate(const fdma_varlen_fwd_args *a) {
    g_err[0] = 0;
    return validate_varlen(a, false);
}

int fdma_varlen_fwd(const fdma_varlen_fwd_args *a, void *hip_stream) {
    if (int cap = refuse_capture(hip_stream, "fdma_varlen_fwd")) return cap;
    g_err[0] = 0;
    int rc = validate_varlen(a, false);
    if (rc != FDMA_OK) return rc;
    fdma::FwdParams p;
    if ((rc = fill_varlen_params(a, p)) != FDMA_OK) return rc;
    if (a->total_q == 0 || p.Lq == 0) return FDMA_OK;
    const hipError_t e = fdma::launch_fwd_colmask(p, a->dtype, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "forward launch failed: %s", hipGetErrorString(e));
    return FDMA_OK;
}

int fdma_varlen_bwd_validate(const fdma_varlen_bwd_args *a) {
    g_err[0] = 0;
    if (!a) return fail(FDMA_ERR_INVALID, "args must not be NULL");
    int rc = validate_varlen(&a->f, true);
    if (rc != FDMA_OK) return rc;
    if ((a->f.total_q > 0 && (!a->dout || !a->dq)) || (a->f.total_k > 0 && (!a->dk || !a->dv)))
        return fail(FDMA_ERR_INVALID, "dout, dq, dk, dv must be device pointers");
    if (a->f.total_q > 0 && !a->softmax_d) return fail(FDMA_ERR_INVALID, "softmax_d must be a device pointer");
    const int64_t *st[4] = {a->do_strides, a->dq_strides, a->dk_strides, a->dv_strides};
    for (int i = 0; i < 4; i++)
        if (st[i][0] % 8 != 0 || st[i][1] % 8 != 0)
            return fail(FDMA_ERR_INVALID, "dout, dq, dk, dv must be 16-byte aligned with strides that are multiples of 8 elements");
    if (!aligned16(a->dout) || !aligned16(a->dq) || !aligned16(a->dk) || !aligned16(a->dv))
        return fail(FDMA_ERR_INVALID, "dout, dq, dk, dv must be 16-byte aligned with strides that are multiples of 8 elements");
    if (a->do_strides[0] >= kMaxRowStride)
        return fail(FDMA_ERR_UNSUPPORTED, "dout row strides of 2^24 elements or more are not supported");
    return FDMA_OK;
}

int fdma_varlen_bwd(const fdma_varlen_bwd_args *a, void *hip_stream) {
    if (int cap = refuse_capture(hip_stream, "fdma_varlen_bwd")) return cap;
    int rc = fdma_varlen_bwd_validate(a);
    if (rc != FDMA_OK) return rc;
    fdma::BwdParams p;
    std::memset(&p, 0, sizeof(p));
    if ((rc = fill_varlen_params(&a->f, p.f)) != FDMA_OK) return rc;
    p.dout = a->dout; p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
    p.do_r = a->do_strides[0]; p.do_h = a->do_strides[1];
    p.dq_r = a->dq_strides[0]; p.dq_h = a->dq_strides[1];
    p.dk_r = a->dk_strides[0]; p.dk_h = a->dk_strides[1];
    p.dv_r = a->dv_strides[0]; p.dv_h = a->dv_strides[1];
    p.softmax_d = a->softmax_d;
    p.Lq_rounded = p.f.Lq;
    p.sd_b = 0;
    p.sd_h = a->f.total_q;
    // Key rows no query can see get zero dK / dV from the dK/dV kernel itself; with no query rows at all, or no
    // key rows at all, one of the two grids is empty and the other kernel still writes its (zero) outputs.
    if (p.f.Lq == 0 && p.f.Lk == 0) return FDMA_OK;
    if (!fdma::bwd_colmask_applicable(p))
        return fail(FDMA_ERR_UNSUPPORTED, "ragged batches with sequences of more than 2^19 keys are not supported (max_seqlen_k = %d)", a->f.max_seqlen_k);
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const hipError_t e = p.f.Lq == 0 ? fdma::launch_bwd_dkdv_colmask(p, a->f.dtype, stream) : fdma::launch_bwd(p, a->f.dtype, stream);
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "backward launch failed: %s", hipGetErrorString(e));
    return FDMA_OK;
}

size_t fdma_sizeof_mask_args(void) { return sizeof(fdma_mask_args); }

int fdma_create_mask_validate(const fdma_mask_args *a) {
    g_err[0] = 0;
    if (!a) return fail(FDMA_ERR_INVALID, "args must not be NULL");
    if (a->dtype != FDMA_DTYPE_BF16 && a->dtype != FDMA_DTYPE_FP16)
        return fail(FDMA_ERR_INVALID, "attention_bias must be fp16 or bf16");
    if (a->type != FDMA_MASK_TOPK && a->type != FDMA_MASK_RELU)
        return fail(FDMA_ERR_INVALID, "Unsupported mask type: %d. Supported types are 'topk' and 'relu'.", a->type);
    if (a->batch < 0 || a->heads < 0 || a->rows < 0 || a->seqlen_k < 0) return fail(FDMA_ERR_INVALID, "mask dimensions must be non-negative");
    if ((int64_t)a->batch * a->heads * a->rows > 0x7fffffff) return fail(FDMA_ERR_UNSUPPORTED, "more than 2^31 - 1 mask rows");
    if (a->type == FDMA_MASK_TOPK && a->window < 0) return fail(FDMA_ERR_INVALID, "window_size must be non-negative");
    if (a->block_size < 0) return fail(FDMA_ERR_INVALID, "block_size must be a positive integer, got %d.", a->block_size);
    const bool empty = (int64_t)a->batch * a->heads * a->rows * a->seqlen_k == 0;
    if (!empty && (!a->bias || !a->mask_out)) return fail(FDMA_ERR_INVALID, "bias and mask_out must be device pointers");
    if (reinterpret_cast<uintptr_t>(a->bias) & 1) return fail(FDMA_ERR_INVALID, "bias must be 2-byte aligned");
    if (std::isnan(a->min_value)) return fail(FDMA_ERR_INVALID, "min_dtype must not be NaN");
    if (a->bits && (a->bits_row_bytes % 8 != 0 || a->bits_row_bytes < ((a->seqlen_k + 7) / 8 + 7) / 8 * 8))
        return fail(FDMA_ERR_INVALID, "bits_row_bytes must be a multiple of 8 and at least ceil(seqlen_k / 8) rounded up to 8");
    if (a->bits && (reinterpret_cast<uintptr_t>(a->bits) & 7))
        return fail(FDMA_ERR_INVALID, "bits must be 8-byte aligned");
    if (a->kept_idx || a->kept_cnt || a->kept_count) {
        if (!(a->kept_idx && a->kept_cnt && a->kept_count))
            return fail(FDMA_ERR_INVALID, "kept_idx, kept_cnt and kept_count must be given together");
        if (a->kept_ld < a->seqlen_k || a->kept_ld % 16 != 0)
            return fail(FDMA_ERR_INVALID, "kept_ld must be a multiple of 16 and at least seqlen_k");
        if ((reinterpret_cast<uintptr_t>(a->kept_cnt) | reinterpret_cast<uintptr_t>(a->kept_idx)) & 15)
            return fail(FDMA_ERR_INVALID, "kept_idx and kept_cnt must be 16-byte aligned");
    }
    return FDMA_OK;
}

// float -> bits of the bias type, round to nearest even, overflow to infinity
static uint32_t to_bits16(float x, int dtype) {
    uint32_t u;
    std::memcpy(&u, &x, 4);
    if (dtype == FDMA_DTYPE_BF16) {
        u += 0x7fffu + ((u >> 16) & 1u);
        return u >> 16;
    }
    const uint32_t sign = (u >> 16) & 0x8000u;
    const float ax = std::fabs(x);
    if (!(ax < 65520.f)) return sign | 0x7c00u;
    if (ax < 6.103515625e-05f) {  // subnormal half: units of 2^-24
        const float scaled = ax * 16777216.f;
        const uint32_t m = (uint32_t)std::nearbyintf(scaled);
        return sign | m;
    }
    uint32_t a;
    std::memcpy(&a, &ax, 4);
    a += 0xfffu + ((a >> 13) & 1u);  // round the 13 dropped mantissa bits to nearest even
    const uint32_t e = (a >> 23) - 127 + 15, m = (a >> 13) & 0x3ffu;
    return sign | (e << 10) | m;
}

int fdma_create_mask(const fdma_mask_args *a, void *hip_stream) {
    if (int cap = refuse_capture(hip_stream, "fdma_create_mask")) return cap;
    int rc = fdma_create_mask_validate(a);
    if (rc != FDMA_OK) return rc;
    fdma::MaskParams p;
    std::memset(&p, 0, sizeof(p));
    p.bias = a->bias;
    p.mask_in = static_cast<const uint8_t *>(a->mask_in);
    p.mask_out = static_cast<uint8_t *>(a->mask_out);
    p.bi_b = a->bias_strides[0]; p.bi_h = a->bias_strides[1]; p.bi_r = a->bias_strides[2];
    p.mi_b = a->mask_in_strides[0]; p.mi_h = a->mask_in_strides[1]; p.mi_r = a->mask_in_strides[2];
    p.mo_b = a->mask_out_strides[0]; p.mo_h = a->mask_out_strides[1]; p.mo_r = a->mask_out_strides[2];
    p.batch = a->batch; p.heads = a->heads; p.rows = a->rows; p.Lk = a->seqlen_k;
    p.window = a->window;
    p.block_size = a->block_size;
    p.type = a->type;
    p.dtype = a->dtype;
    p.min_bits = to_bits16(a->min_value, a->dtype);
    p.kept_idx = a->kept_idx; p.kept_cnt = a->kept_cnt; p.kept_count = a->kept_count;
    p.kept_ld = a->kept_ld;
    p.bits = a->bits; p.bits_row_bytes = a->bits_row_bytes;
    const hipError_t e = fdma::launch_make_mask(p, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "mask launch failed: %s", hipGetErrorString(e));
    return FDMA_OK;
}

size_t fdma_sizeof_dyn_bias_args(void) { return sizeof(fdma_dyn_bias_args); }

int fdma_dyn_bias_validate(const fdma_dyn_bias_args *a, int backward) {
    g_err[0] = 0;
    if (!a) return fail(FDMA_ERR_INVALID, "args must not be NULL");
    if (a->dtype != FDMA_DTYPE_BF16 && a->dtype != FDMA_DTYPE_FP16) return fail(FDMA_ERR_INVALID, "value states must be fp16 or bf16");
    if (a->batch < 0 || a->seqlen_k < 0) return fail(FDMA_ERR_INVALID, "batch and seqlen_k must be non-negative");
    if (a->num_heads_k <= 0 || a->num_heads_k > 32) return fail(FDMA_ERR_UNSUPPORTED, "the bias producer is built for 1 to 32 kv heads (got %d)", a->num_heads_k);
    if (a->head_dim <= 0 || a->head_dim % 8 != 0 || (a->num_heads_k * a->head_dim) % 16 != 0)
        return fail(FDMA_ERR_UNSUPPORTED, "head_dim must be a multiple of 8 and num_heads_k * head_dim a multiple of 16");
    const bool empty = (int64_t)a->batch * a->seqlen_k == 0;
    if (!a->weight || !a->a || (!empty && (!a->value || !a->bias || !a->dt))) return fail(FDMA_ERR_INVALID, "value, weight, a, bias, dt must be device pointers");
    if (!aligned16(a->value) || !aligned16(a->weight) || !strides_ok(a->value_strides, 8))
        return fail(FDMA_ERR_INVALID, "value and weight must be 16-byte aligned, value strides multiples of 8 elements");
    if (backward) {
        if (!a->dweight || !a->da || (!empty && (!a->dbias || !a->dvalue))) return fail(FDMA_ERR_INVALID, "dbias, dvalue, dweight, da must be device pointers");
        if ((a->proj_bias != nullptr) != (a->dproj_bias != nullptr)) return fail(FDMA_ERR_INVALID, "dproj_bias must be given exactly when proj_bias is given");
        if ((reinterpret_cast<uintptr_t>(a->dvalue) & 7) || a->dvalue_strides[0] % 4 || a->dvalue_strides[1] % 4 || a->dvalue_strides[2] % 4)
            return fail(FDMA_ERR_INVALID, "dvalue must be 8-byte aligned with strides that are multiples of 4 elements");
    }
    return FDMA_OK;
}

static void fill_dyn_bias(const fdma_dyn_bias_args *a, fdma::DynBiasParams &p) {
    std::memset(&p, 0, sizeof(p));
    p.v = a->value; p.w = a->weight; p.pb = a->proj_bias; p.a = a->a;
    p.bias = a->bias; p.dt = a->dt;
    p.v_b = a->value_strides[0]; p.v_r = a->value_strides[1]; p.v_h = a->value_strides[2];
    p.bias_b = a->bias_strides[0]; p.bias_h = a->bias_strides[1];
    p.B = a->batch; p.L = a->seqlen_k; p.Hk = a->num_heads_k; p.d = a->head_dim;
    p.dbias = a->dbias; p.dbias_b = a->dbias_strides[0]; p.dbias_h = a->dbias_strides[1];
    p.dv = a->dvalue; p.dv_b = a->dvalue_strides[0]; p.dv_r = a->dvalue_strides[1]; p.dv_h = a->dvalue_strides[2];
    p.dw = a->dweight; p.da = a->da; p.dpb = a->dproj_bias;
    p.n_wg = fdma::dyn_bias_bwd_workgroups((int64_t)a->batch * a->seqlen_k, &p.rows_per_wg);
    p.part_stride = round_up((int64_t)a->num_heads_k * a->num_heads_k * a->head_dim + 2 * a->num_heads_k, 4);
}

size_t fdma_dyn_bias_bwd_workspace_bytes(const fdma_dyn_bias_args *a) {
    if (!a || (int64_t)a->batch * a->seqlen_k <= 0) return 0;
    fdma::DynBiasParams p;
    fill_dyn_bias(a, p);
    return (size_t)p.n_wg * p.part_stride * sizeof(float);
}

int fdma_dyn_bias_fwd(const fdma_dyn_bias_args *a, void *hip_stream) {
    if (int cap = refuse_capture(hip_stream, "fdma_dyn_bias_fwd")) return cap;
    int rc = fdma_dyn_bias_validate(a, 0);
    if (rc != FDMA_OK) return rc;
    fdma::DynBiasParams p;
    fill_dyn_bias(a, p);
    const hipError_t e = fdma::launch_dyn_bias_fwd(p, a->dtype, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "bias producer launch failed: %s", hipGetErrorString(e));
    return FDMA_OK;
}

int fdma_dyn_bias_bwd(const fdma_dyn_bias_args *a, void *hip_stream) {
    if (int cap = refuse_capture(hip_stream, "fdma_dyn_bias_bwd")) return cap;
    int rc = fdma_dyn_bias_validate(a, 1);
    if (rc != FDMA_OK) return rc;
    fdma::DynBiasParams p;
    fill_dyn_bias(a, p);
    const size_t need = fdma_dyn_bias_bwd_workspace_bytes(a);
    if (need && (!a->workspace || a->workspace_bytes < need))
        return fail(FDMA_ERR_WORKSPACE, "bias producer backward workspace too small: need %zu bytes, got %zu", need, a->workspace_bytes);
    p.part = static_cast<float *>(a->workspace);
    const hipError_t e = fdma::launch_dyn_bias_bwd(p, a->dtype, static_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(FDMA_ERR_LAUNCH, "bias producer launch failed: %s", hipGetErrorString(e));
    return FDMA_OK;
}

}  // extern "C"
