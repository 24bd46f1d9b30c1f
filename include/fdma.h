/*
 * fdma.h -- C ABI of libfdma_hip.so, the gfx950 (MI355X) implementation of Flash Dynamic Mask
 * Attention (dense path: Q,K,V + boolean keep-mask + additive bias, causal, MQA/GQA,
 * dQ/dK/dV/dBias).
 *
 * The library is a drop-in for the compiled extension of SmallDoges/flash-dmattn: each entry point
 * below replaces one function the reference's Python operator binds from `flash_sparse_attn_cuda`
 * (reference paths are relative to its checkout):
 *
 *   fdma_fwd   <-  mha_fwd            csrc/flash_sparse_attn/flash_api.cpp:351-554  (pybind "fwd",  :1272)
 *   fdma_bwd   <-  mha_bwd            csrc/flash_sparse_attn/flash_api.cpp:792-1050 (pybind "bwd",  :1274)
 *   fdma_varlen_fwd <- mha_varlen_fwd csrc/flash_sparse_attn/flash_api.cpp:556-790  (pybind "varlen_fwd", :1273)
 *   fdma_varlen_bwd <- mha_varlen_bwd csrc/flash_sparse_attn/flash_api.cpp:1052-1268 (pybind "varlen_bwd", :1275)
 *   fdma_fwd_args / fdma_bwd_args
 *              <-  Flash_fwd_params / Flash_bwd_params   csrc/flash_sparse_attn/src/flash.h:20-198
 *
 * Differences from the reference boundary, all on purpose:
 *   - plain C: device pointers, sizes and element strides; no torch / pybind types;
 *   - the caller owns every buffer (outputs, LSE, softmax_d, workspace); the library never
 *     allocates, frees or synchronises and launches on the HIP stream it is handed;
 *   - dK/dV are written at their true (Hkv) shape and dBias at the bias's own broadcast shape,
 *     so there are no "expanded" temporaries and no host-side reductions
 *     (flash_api.cpp:970-983, 1027-1047 are fused into the kernels);
 *   - errors are returned as negative codes with a thread-local message (fdma_last_error)
 *     carrying the same text the reference's TORCH_CHECKs raise.
 *
 * Layouts (all strides in ELEMENTS, innermost dimension contiguous):
 *   q, out, dout, dq : (batch, seqlen_q, num_heads,   head_dim)   strides {batch, row, head}
 *   k, v, dk, dv     : (batch, seqlen_k, num_heads_k, head_dim)   strides {batch, row, head}
 *   mask  (uint8 / bool, 1 = keep) : ({batch|1}, {1|Hk|H}, {seqlen_q|1}, >= round_up(seqlen_k, 16) READABLE)
 *   bias, dbias (same dtype as q)  : ({batch|1}, {1|Hk|H}, {seqlen_q|1}, >= round_up(seqlen_k, 8)  READABLE)
 *                                     strides {batch, head, row}; 0 marks a broadcast dim
 *                                     (rows are read in 16-byte vectors, see "Readable lengths" below)
 *   lse       : (batch, num_heads, seqlen_q) fp32, contiguous; +inf for rows with no visible key
 *   softmax_d : (batch, num_heads, round_up(seqlen_q,128)) fp32, contiguous
 */
#ifndef FDMA_H_
#define FDMA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FDMA_ABI_VERSION 6 /* 6: fdma_fwd_args.counters (split-KV decode in one launch), fdma_fwd_counter_bytes; 5: fdma_mask_bits (fdma_fwd_args.mask_bits, fdma_mask_args.bits); 4: fdma_kept_keys (fdma_fwd_args.kept, fdma_mask_args.kept_*), fdma_bwd_args.fwd_workspace (the structs grew);
                              3: fdma_fwd_args.compact_mode, fdma_fwd_noalloc; 2: fdma_varlen_*, fdma_create_mask, fdma_dyn_bias_* */

enum { FDMA_DTYPE_BF16 = 0, FDMA_DTYPE_FP16 = 1 };

enum {
    FDMA_OK = 0,
    FDMA_ERR_INVALID = -1,     /* argument validation failed (the reference raises RuntimeError) */
    FDMA_ERR_UNSUPPORTED = -2, /* valid for the reference, not built here (softcap, row strides of 2^24
                                  elements or more, a stream under HIP graph capture)            */
    FDMA_ERR_WORKSPACE = -3,   /* workspace missing or too small                                  */
    FDMA_ERR_LAUNCH = -4       /* the HIP runtime refused a launch                                */
};

/* HIP graph capture: NOT supported.  Every entry point that launches work first asks hipStreamIsCapturing about
 * `hip_stream` and returns FDMA_ERR_UNSUPPORTED, launching nothing, when the stream is being captured.  (The one
 * capture of forward + backward through the tensor library ended in a host crash when the capture was closed; its
 * cause is not known, so the library refuses instead.)
 *
 * Readable lengths of mask and bias rows.  The kernels read mask rows in 16-byte and bias rows in 16-byte
 * (8-element) vectors: each row of `mask` must be readable up to seqlen_k rounded up to 16 bytes, each row of `bias`
 * up to seqlen_k rounded up to 8 elements, whatever lies there; this also holds for the last row of the buffer, and for a fully
 * broadcast mask or bias of a single row.  The library cannot check it (it never sees the row length).  The reference
 * asks for more: rows of exactly round_up(seqlen_k, 128) elements (flash_api.cpp:420, 431, 437).  Values beyond
 * seqlen_k are never used, and dbias is only written up to seqlen_k. */

/* Column compaction (fdma_fwd_args.compact_mode).  A keep-mask that is broadcast over the queries, with 1 or
 * num_heads_k heads, drops whole key columns; the library can then gather the kept K / V rows into dense copies
 * (in the workspace) and run attention over those alone, so that the work follows the number of kept keys.
 * The result is the same function of the inputs either way.  The mode decides the workspace size, so the
 * *_workspace_bytes call and the launch must see the same value (a mismatch is caught: FDMA_ERR_WORKSPACE).
 * A query-broadcast mask with a row per QUERY head over grouped kv heads (num_heads_mask == num_heads > num_heads_k)
 * is compacted per query head by fdma_fwd (a copy of the kept rows per query head); fdma_bwd does not compact that
 * form as a whole -- a caller that wants it compacted calls fdma_bwd once per member g of the kv groups, on the
 * query heads g, g + G, ... (pointers offset by g heads, head strides times G, num_heads = num_heads_mask =
 * num_heads_k), and sums dk / dv (and a dbias shared by the group) over the members, as the Python operator does. */
enum {
    FDMA_COMPACT_AUTO = 0,  /* compact when the mask form allows it and the problem is large enough to pay for the pre-pass */
    FDMA_COMPACT_NEVER = 1, /* tile skipping only */
    FDMA_COMPACT_ALWAYS = 2 /* compact whenever the mask form allows it */
};

/* The kept key columns of a query-broadcast keep-mask as lists, the form the compaction path works on.  Optional
 * second output of fdma_create_mask and optional input of fdma_fwd / fdma_bwd: when a caller hands the lists over,
 * the attention call does not scan the bool mask again (the mask itself must still be passed: it decides the path and
 * is what the non-compacting kernels read).  One row per mask row, in (batch entry, mask head) order -- batch entry 0
 * only when the mask is broadcast over the batch:
 *   idx   : (rows, ld) int32, the original columns of the kept keys of a row in ascending order, count[row] of them
 *   cnt   : (rows, ld) int32, cnt[row][j] = kept keys among the columns 0 .. j (inclusive), for j < seqlen_k
 *   count : (rows) int32
 *   ld    : row stride in elements, a multiple of 16 and >= seqlen_k
 * The lists must describe exactly the mask that is passed; nothing checks it.  The reference has no counterpart (its
 * kernels take the bool mask only); the precedent for index lists is its Triton backend,
 * flash_sparse_attn/flash_dmattn_triton.py:50-211. */
typedef struct fdma_kept_keys {
    const int32_t *idx, *cnt, *count; /* all NULL = not given */
    int32_t ld;
} fdma_kept_keys;

/* A keep-mask that varies per query row, packed to one bit per key: the form in which the per-query kernels can
 * take it at an eighth of the bool mask's memory traffic (these kernels are bound by the mask and bias streams).
 * Optional second output of fdma_create_mask and optional input of fdma_fwd / fdma_bwd; the bool mask itself must
 * still be passed (it decides the path, and kernels that do not read bits read it).  Byte j / 8 of a row holds key j
 * in bit j % 8 (least significant bit first); bits beyond seqlen_k are not looked at.  The kernels read a row in
 * aligned 8-byte pieces: `bits` and every stride are multiples of 8, and a row is readable up to ceil(seqlen_k / 8)
 * rounded up to 8 bytes, whatever lies there.  Strides in BYTES, in the order of mask_strides (batch, head, row),
 * 0 = broadcast exactly where the mask is.  The bits must describe exactly the mask that is passed; nothing checks it.  The reference has no
 * counterpart (its kernels take the bool mask only). */
typedef struct fdma_mask_bits {
    const uint8_t *bits; /* NULL = not given */
    int64_t strides[3];
} fdma_mask_bits;

typedef struct fdma_fwd_args {
    const void *q, *k, *v;
    const void *mask; /* NULL = no mask */
    const void *bias; /* NULL = no bias */
    void *out;
    float *lse;
    int64_t q_strides[3], k_strides[3], v_strides[3], o_strides[3];
    int64_t mask_strides[3], bias_strides[3];
    int32_t batch, seqlen_q, seqlen_k;
    int32_t num_heads, num_heads_k, num_heads_mask, num_heads_bias;
    int32_t head_dim;
    int32_t dtype;
    int32_t is_causal;
    float softmax_scale;
    float softcap; /* must be 0: softcapping is not built */
    int32_t compact_mode;   /* FDMA_COMPACT_*; 0 = let the library decide */
    void *workspace;        /* split-KV partials (decode) or the compacted K / V copies; may be NULL if bytes == 0 */
    size_t workspace_bytes; /* >= fdma_fwd_workspace_bytes(args) */
    fdma_kept_keys kept;    /* optional: the mask's kept columns as lists (see fdma_kept_keys) */
    fdma_mask_bits mask_bits; /* optional: a per-query mask packed to bits (see fdma_mask_bits) */
    /* Optional: arrival counters of the split-KV decode path (seqlen_q == 1), fdma_fwd_counter_bytes(args) bytes of
     * device memory, 4-byte aligned, that hold ZEROS when the call starts.  With them the decode is ONE launch: the
     * workgroup that finishes last among the splits of a (batch entry, kv head) merges their partial results (the
     * reference always runs its combine as a second kernel, flash_fwd_launch_template.h:91-143) and puts its counter
     * back to zero, so the same buffer serves the next call as it is -- clear it once, when it is allocated.  Calls
     * that may overlap on the device (different streams) need a buffer each.  NULL = the merge is a second launch.
     * Results are the same bit for bit either way.  Other paths ignore the field. */
    int32_t *counters;
    size_t counters_bytes; /* >= fdma_fwd_counter_bytes(args) */
} fdma_fwd_args;

typedef struct fdma_bwd_args {
    fdma_fwd_args f; /* q,k,v,mask,bias as in forward; f.out and f.lse are the forward RESULTS (read) */
    const void *dout;
    void *dq, *dk, *dv;
    void *dbias; /* NULL iff f.bias == NULL; shape and broadcast pattern of the bias */
    int64_t do_strides[3], dq_strides[3], dk_strides[3], dv_strides[3];
    int64_t dbias_strides[3];
    float *softmax_d; /* out: rowsum(dO * O) */
    /* Accepted for parity with mha_bwd (flash_api.cpp:809).  dq, dk, dv never depend on it: they are written without
     * atomics.  dbias elements that several (batch, kv head) pairs share -- bias strides[0] == 0 with batch > 1, or
     * num_heads_bias == 1 < num_heads_k -- are accumulated with fp32 atomics whatever this says; a caller that needs
     * them bit-reproducible passes a bias / dbias expanded over those dimensions and sums the slices itself, as the
     * Python operator does for deterministic=True. */
    int32_t deterministic;
    void *workspace;
    size_t workspace_bytes; /* >= fdma_bwd_workspace_bytes(args) */
    /* Optional: the workspace the forward call of the SAME problem (same f.* arguments, compact_mode included) left
     * behind, untouched since.  When the compaction path runs, the backward then reuses the forward's index lists and
     * compacted K / V copies instead of scanning and gathering again, and fdma_bwd_workspace_bytes() shrinks by their
     * size.  NULL = the backward makes its own. */
    const void *fwd_workspace;
    size_t fwd_workspace_bytes; /* >= fdma_fwd_workspace_bytes(&args->f) */
} fdma_bwd_args;

/* Forward attention.  Asynchronous on `hip_stream` (a hipStream_t).  Returns FDMA_OK or < 0. */
int fdma_fwd(const fdma_fwd_args *args, void *hip_stream);

/* Backward attention: dq, dk, dv, dbias, softmax_d.  Every output element is written exactly once
 * (no zero-fill needed by the caller), including masked / skipped regions of dbias. */
int fdma_bwd(const fdma_bwd_args *args, void *hip_stream);

/*
 * fdma_fwd for callers that cannot allocate device memory: tight serving loops, harnesses that forbid hipMalloc
 * (and code under HIP graph capture, once capture is supported: today this call refuses a capturing stream like
 * every other).  It has no counterpart in the reference (whose mha_fwd allocates its split-KV
 * partials with torch, flash_api.cpp:340-345).  args->workspace / workspace_bytes are ignored; the scratch of the
 * decode path (split-KV partials) or of the compaction path lives in a static device array of
 * FDMA_NOALLOC_SCRATCH_BYTES inside the library, which every GPU the library runs on holds until the process ends.
 * A problem whose fdma_fwd_workspace_bytes() exceeds that returns FDMA_ERR_WORKSPACE and launches nothing.  The
 * call makes no hipMalloc / hipFree (nor any other allocating call); results are bit-identical to fdma_fwd's.
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (different streams or host
 * threads) race on it -- serialise them.  The last FDMA_NOALLOC_COUNTER_BYTES of the array are the decode path's
 * arrival counters (args->counters is ignored as well): they are zero when the library is loaded and every call
 * leaves them zero; the rest of the array need not start at anything, every call overwrites what it reads.  The
 * scratch a problem may need is therefore FDMA_NOALLOC_SCRATCH_BYTES - FDMA_NOALLOC_COUNTER_BYTES at most.
 */
#define FDMA_NOALLOC_SCRATCH_BYTES (8u << 20)
#define FDMA_NOALLOC_COUNTER_BYTES (64u << 10)
int fdma_fwd_noalloc(const fdma_fwd_args *args, void *hip_stream);

/* Tuning knob of the column-compaction path, process-wide.  At head dim 128 the compacted forward has two forms: one
 * workgroup per 128 or 256 query rows of a head over row-major copies of the kept K / V rows, and -- for problems of
 * at least `n` (256-row query block, head) items, default 512: a grid that fills the device several times -- resident
 * workgroups that stream "tile images" written by the pre-pass (fdma_fwd_stream.hip).  The threshold decides the
 * workspace LAYOUT: a forward call and the backward call that is handed its workspace (fwd_workspace) must run under
 * the same value.  n <= 0 only queries.  Returns the value before the call.  No counterpart in the reference. */
int fdma_set_stream_min_items(int n);

/* Scratch the caller must provide.  0 when none is needed.  Validate nothing but shapes. */
size_t fdma_fwd_workspace_bytes(const fdma_fwd_args *args);
/* Size of the optional arrival counters (fdma_fwd_args.counters); 0 when the call would not use them. */
size_t fdma_fwd_counter_bytes(const fdma_fwd_args *args);
size_t fdma_bwd_workspace_bytes(const fdma_bwd_args *args);

/* Argument validation only (no GPU work, callable on a host without a device). */
int fdma_fwd_validate(const fdma_fwd_args *args);
int fdma_bwd_validate(const fdma_bwd_args *args);

/*
 * Ragged batches ("varlen"): the sequences of a batch lie back to back in q (total_q, num_heads, head_dim)
 * and k / v (total_k, num_heads_k, head_dim); batch entry i owns query rows cu_seqlens_q[i] .. cu_seqlens_q[i+1]-1
 * and key rows cu_seqlens_k[i] .. cu_seqlens_k[i+1]-1.  cu_seqlens_* are DEVICE arrays of batch+1 int32, starting
 * at 0 and non-decreasing (the library never reads them on the host and never synchronises).  As in the
 * reference this path takes no mask and no bias; the causal mask is aligned bottom-right per sequence.
 *   lse       : (num_heads, total_q) fp32, contiguous; +inf for rows with no visible key
 *   softmax_d : (num_heads, total_q) fp32, contiguous
 * Strides are {row, head} in elements, innermost dimension contiguous.  max_seqlen_* must be upper bounds
 * of the sequence lengths (they size the launch); rows of sequences longer than that are not computed.
 * Not built: paged KV (block_table), seqused_k, leftpad_k (flash_api.cpp:564-566).
 */
typedef struct fdma_varlen_fwd_args {
    const void *q, *k, *v;
    void *out;
    float *lse;
    const int32_t *cu_seqlens_q, *cu_seqlens_k;
    int64_t q_strides[2], k_strides[2], v_strides[2], o_strides[2];
    int32_t batch, total_q, total_k, max_seqlen_q, max_seqlen_k;
    int32_t num_heads, num_heads_k, head_dim;
    int32_t dtype;
    int32_t is_causal;
    float softmax_scale;
    float softcap; /* must be 0 */
} fdma_varlen_fwd_args;

typedef struct fdma_varlen_bwd_args {
    fdma_varlen_fwd_args f; /* f.out and f.lse are the forward RESULTS (read) */
    const void *dout;
    void *dq, *dk, *dv;
    int64_t do_strides[2], dq_strides[2], dk_strides[2], dv_strides[2];
    float *softmax_d; /* out: rowsum(dO * O) */
    int32_t deterministic;
} fdma_varlen_bwd_args;

/* Forward / backward over a ragged batch.  No workspace is needed.  Every row of out / lse / dq / dk / dv that
 * belongs to a sequence is written exactly once. */
int fdma_varlen_fwd(const fdma_varlen_fwd_args *args, void *hip_stream);
int fdma_varlen_bwd(const fdma_varlen_bwd_args *args, void *hip_stream);
int fdma_varlen_fwd_validate(const fdma_varlen_fwd_args *args);
int fdma_varlen_bwd_validate(const fdma_varlen_bwd_args *args);
size_t fdma_sizeof_varlen_fwd_args(void);
size_t fdma_sizeof_varlen_bwd_args(void);

/*
 * Keep-mask builder: topk_mask / relu_mask with the optional block_smooth of the reference's
 * flash_sparse_attn/utils/mask.py:47-160, one kernel per call.
 *   bias     : ({batch|1}, {heads}, {rows}, seqlen_k) bf16 / fp16, strides {batch, head, row} in elements
 *   mask_in  : NULL, or bool (uint8) broadcastable to the bias: strides {batch, head, row} in bytes, 0 = broadcast
 *   mask_out : bool (uint8), one row of seqlen_k bytes per bias row, strides {batch, head, row} in bytes
 * type 0 (top-k): per row, entries excluded by mask_in are replaced by min_value, the `window` largest values are
 * selected (all of them when window >= seqlen_k) and a selected entry is kept unless its value equals min_value.
 * Among entries equal to the smallest selected value the lowest columns win (the reference leaves this choice to
 * torch.topk, which does not define it).  type 1 (relu): an entry is kept when its value, after the same
 * replacement, is > 0.  block_size > 1 then replaces every aligned block of block_size keys by the majority vote
 * of its entries (strictly more than half; a shorter tail block votes over its own length).
 */
enum { FDMA_MASK_TOPK = 0, FDMA_MASK_RELU = 1 };
typedef struct fdma_mask_args {
    const void *bias;
    const void *mask_in;
    void *mask_out;
    int64_t bias_strides[3], mask_in_strides[3], mask_out_strides[3];
    int32_t batch, heads, rows, seqlen_k;
    int32_t window;
    int32_t block_size; /* 0 or 1 = no smoothing */
    int32_t type;
    int32_t dtype;
    float min_value;
    /* optional second output: the kept columns of every mask row as lists (fdma_kept_keys), one row per bias row in
     * (batch, head, row) order; all NULL = not wanted */
    int32_t *kept_idx, *kept_cnt, *kept_count;
    int32_t kept_ld; /* multiple of 16, >= seqlen_k */
    /* optional third output: the mask packed to bits (fdma_mask_bits), one row of bits_row_bytes bytes per bias row in
     * (batch, head, row) order; NULL = not wanted.  bits and bits_row_bytes: multiples of 8, bits_row_bytes >=
     * ceil(seqlen_k / 8) rounded up to 8; the bytes of a row up to ceil(seqlen_k / 8) are written, bits beyond
     * seqlen_k as zeros */
    uint8_t *bits;
    int64_t bits_row_bytes;
} fdma_mask_args;
int fdma_create_mask(const fdma_mask_args *args, void *hip_stream);
int fdma_create_mask_validate(const fdma_mask_args *args);
size_t fdma_sizeof_mask_args(void);

/*
 * Producer of the dynamic-mask bias, fused:  bias[b, j, 0, l] = a[j] * softplus(value[b, l, :, :] . weight[j, :] + proj_bias[j])
 * -- the `A * softplus(dt_proj(V))` in front of the attention call of the reference's Doge caller
 * (examples/modeling/modeling_doge.py:217-222; there a chain of tensor-library calls, so this entry point has no
 * counterpart in the reference's extension) -- and its backward, which takes the attention's dbias in the bias's own
 * (batch, num_heads_k, 1, seqlen_k) shape and returns the gradients of value, weight, a and proj_bias.
 *   value, dvalue : (batch, seqlen_k, num_heads_k, head_dim), strides {batch, row, head} in elements
 *   weight, dweight : (num_heads_k, num_heads_k * head_dim), contiguous;  a, da, proj_bias, dproj_bias : (num_heads_k)
 *   bias, dbias   : (batch, num_heads_k, 1, >= seqlen_k), strides {batch, head} in elements, key dimension contiguous
 *   dt            : (batch * seqlen_k, num_heads_k) fp32, written by forward and read by backward
 * All tensors have the dtype given; num_heads_k <= 32, head_dim % 8 == 0, (num_heads_k * head_dim) % 16 == 0.
 * Backward needs fdma_dyn_bias_bwd_workspace_bytes() of scratch; its sums are folded in a fixed order (bit-reproducible).
 */
typedef struct fdma_dyn_bias_args {
    const void *value, *weight, *proj_bias /* may be NULL */, *a;
    void *bias;
    float *dt;
    int64_t value_strides[3], bias_strides[2];
    int32_t batch, seqlen_k, num_heads_k, head_dim, dtype;
    /* backward only */
    const void *dbias;
    int64_t dbias_strides[2];
    void *dvalue;
    int64_t dvalue_strides[3];
    void *dweight, *da, *dproj_bias /* NULL iff proj_bias is NULL */;
    void *workspace;
    size_t workspace_bytes;
} fdma_dyn_bias_args;
int fdma_dyn_bias_fwd(const fdma_dyn_bias_args *args, void *hip_stream);
int fdma_dyn_bias_bwd(const fdma_dyn_bias_args *args, void *hip_stream);
size_t fdma_dyn_bias_bwd_workspace_bytes(const fdma_dyn_bias_args *args);
int fdma_dyn_bias_validate(const fdma_dyn_bias_args *args, int backward);
size_t fdma_sizeof_dyn_bias_args(void);

/* Message of the last error raised on the calling thread ("" if none). */
const char *fdma_last_error(void);

int fdma_abi_version(void);

/* sizeof() of the two argument blocks as compiled, so a foreign-language binding can check its
 * struct packing before the first call. */
size_t fdma_sizeof_fwd_args(void);
size_t fdma_sizeof_bwd_args(void);

#ifdef __cplusplus
}
#endif
#endif /* FDMA_H_ */
