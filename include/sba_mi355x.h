/*
 * C ABI of libsba_mi355x.so: stick-breaking attention for AMD MI355X (gfx950).
 *
 * Plain pointers and sizes only; no torch types.  All tensor pointers are device
 * pointers (HIP), all launches are asynchronous on `stream`, nothing is allocated and
 * nothing synchronises, so every entry point may be called from any thread.  Process-wide
 * state: the compute-unit count of each device and the address of sba_bwd_static()'s array are
 * looked up once and kept; the SBA_* environment switches (experiments and tests only) are read
 * when a call dispatches, so they must not change between an sba_fwd and the sba_bwd that
 * consumes its workspace.  Return value: 0 on success, a negative SBA_ERR_* code otherwise
 * (sba_error_string() gives the text).
 *
 * The reference has no native code; what each entry point replaces is the Python host
 * launcher plus the Triton kernel it starts (paths relative to the reference tree,
 * custom_models/sba/stickbreaking_attention/):
 *
 *   sba_fwd  <-  sb_attn/sb_fwd.py:139-253   (_fwd / _compileable_fwd -> dense _forward)
 *                sb_varlen/sb_varlen_fwd.py:408-516 (varlen_fwd -> varlen _forward)
 *   sba_bwd  <-  sb_attn/sb_bwd.py:163-297   (_bwd / _compileable_backward -> dense _backward)
 *                sb_varlen/sb_varlen_bwd.py:459-615 (varlen_bwd -> varlen _backward)
 *
 * Tensor layout.  One descriptor covers both reference layouts:
 *   dense  [B, H, T, D]  : n_seq = B, seq_len = T, cu_seqlens = NULL,
 *                          element (b,h,t,d) at  base + b*stride_b + h*stride_h + t*stride_t + d
 *   packed [H, sumT, D]  : n_seq = number of documents, cu_seqlens = device int32[n_seq+1]
 *                          with cu_seqlens[0] == 0, stride_b = 0,
 *                          element (h,t,d) at    base + h*stride_h + t*stride_t + d
 * Strides are in elements; the innermost (D) stride is 1.  head_dim is at most 256 (the reference
 * pads it to the next power of two, sb_attn/sb_fwd.py:199).  Problems at head_dim 64 / 128, and
 * bf16 / float16 ones at 256 (the matrix-core kernels) need 16-byte aligned tensor pointers, outer strides that are
 * multiples of 16 bytes - 8 bf16 / float16 or 4 fp32 elements - and a token stride below 2^23 elements
 * (the tile copies address a 64-row tile with 32-bit byte offsets); SBA_ERR_SHAPE otherwise.
 * rem / d_rem are contiguous along tokens.
 * Wherever the comments below say bf16, float16 (SBA_DTYPE_F16) is sized and handled the same way.
 */
#ifndef SBA_MI355X_H
#define SBA_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SBA_ABI_VERSION 6
#define SBA_SCHEDULE_INTS 8   /* int32 per scheduled job, see sba_build_schedule() */
#define SBA_DOC_MAJOR_GRID 8192 /* workgroups from which the schedule is document-major */

enum { SBA_DTYPE_F32 = 0, SBA_DTYPE_BF16 = 1, SBA_DTYPE_F16 = 2 };   /* (the reference's kernels take whatever dtype the tensors have, sb_attn/sb_fwd.py:144-146) */

enum {
    SBA_OK = 0,
    SBA_ERR_NULL = -1,        /* a required pointer is NULL */
    SBA_ERR_SHAPE = -2,       /* non-positive size, head_dim unsupported, bad strides */
    SBA_ERR_DTYPE = -3,       /* unknown dtype */
    SBA_ERR_WORKSPACE = -4,   /* workspace or bwd_scratch missing or too small */
    SBA_ERR_SCHEDULE = -5,    /* packed layout without a row-block schedule */
    SBA_ERR_LAUNCH = -6,      /* hipGetLastError() after a launch was not hipSuccess */
    SBA_ERR_ABI = -7,         /* struct_size does not match this library */
    SBA_ERR_STATIC_LIMIT = -8 /* sba_bwd_static(): the problem needs more scratch than the library holds */
};

/* One tensor of q/k/v/o/do/dq/dk/dv shape. */
typedef struct SbaTensor {
    void*   ptr;
    int64_t stride_b;   /* 0 for the packed layout */
    int64_t stride_h;
    int64_t stride_t;
} SbaTensor;

/* One per-token vector (rem, drem): element (b,h,t) at ptr + b*stride_b + h*stride_h + t. */
typedef struct SbaVector {
    void*   ptr;
    int64_t stride_b;
    int64_t stride_h;
} SbaVector;

typedef struct SbaParams {
    uint32_t struct_size;      /* = sizeof(SbaParams); checked */
    int32_t  dtype;            /* SBA_DTYPE_*: element type of q,k,v,o,rem,do,drem,dq,dk,dv */
    int32_t  n_seq;            /* B (dense) or number of documents (packed) */
    int32_t  n_heads;
    int32_t  seq_len;          /* T (dense) or max document length (packed: an upper bound is accepted; the kernels
                                  are chosen from it, so the exact longest document chooses best) */
    int32_t  total_tokens;     /* T (dense) or sumT (packed) */
    int32_t  head_dim;         /* D <= 256 */
    int32_t  attend_current;   /* 0: keys j < i;  1: keys j <= i */
    float    scale;            /* logit scale ("inv_temp") in natural-log units */
    int32_t  save_for_backward;/* forward only: also fill the carry table in workspace */
    int32_t  bwd_phases;       /* backward only: 0 = whole backward; 1 = first kernel only (dq and the
                                  prefix table), 2 = second kernel only (dk, dv; needs phase 1 done on
                                  the same workspace).  Lets a profiler time the kernels one by one */

    const int32_t* cu_seqlens; /* device, n_seq+1 entries, or NULL for dense */
    const int32_t* schedule;   /* device, from sba_build_schedule(); packed layout only */
    int32_t  n_schedule;       /* number of row-block jobs in `schedule` */
    int64_t  table_cols;       /* packed layout only: sba_table_columns() of the same cu_seqlens */

    SbaTensor q, k, v;         /* inputs */
    SbaTensor o;               /* forward output            / backward: unused */
    SbaVector rem;             /* forward output            / backward: unused */
    SbaTensor d_o;             /* backward input  (grad of o) */
    SbaVector d_rem;           /* backward input  (grad of rem); ptr may be NULL = zeros */
    SbaTensor dq, dk, dv;      /* backward outputs */

    void*    workspace;        /* device memory that lives from sba_fwd to sba_bwd, see sba_workspace_bytes() */
    size_t   workspace_bytes;
    void*    bwd_scratch;      /* backward only: device memory for the call, see sba_bwd_scratch_bytes() */
    size_t   bwd_scratch_bytes;
    void*    stream;           /* hipStream_t */
} SbaParams;

/* Library identity: SBA_ABI_VERSION it was built with. */
int sba_abi_version(void);

/* Text for an SBA_ERR_* code (static storage). */
const char* sba_error_string(int code);

/*
 * Bytes of device workspace the pair (sba_fwd with save_for_backward, sba_bwd) shares for
 * this problem.  The forward writes its per-key-block carry tables there (bf16: two, the carry
 * entering the right and the left half of every 64-key block; fp32: one) and the backward
 * reads them back, so the SAME buffer, untouched in between, must be given to both calls
 * (the Python layer keeps it in the autograd context the way the reference keeps
 * neg_log_acc, sb_attn/__init__.py:30).  Only the size fields of `p` are read.
 */
size_t sba_workspace_bytes(const SbaParams* p);

/*
 * Bytes of device memory sba_bwd needs for the duration of the call only (the prefix tables that
 * its first kernel hands to its second - two in bf16, one in fp32 -, for bf16 at head_dim 64 also a
 * bf16 copy of q times the logit scale, total_tokens x n_heads x 128 bytes, which the first kernel
 * writes and the second reads in place of q; or the generic path's fp32 accumulators): allocate
 * before the call, free after it has run.  With bwd_phases 1 and 2 issued
 * as two calls, the same buffer goes to both.  For bf16 at head_dim 64 / 128 / 256 the last 256 bytes
 * hold an error word (int32): the first kernel of a backward (bwd_phases 0 or 1) clears it, and a
 * kernel that abandoned one of its bounded internal waits sets it to 1 (the gradients are then
 * invalid); a bwd_phases = 2 call leaves what phase 1 left.  sba_bwd_gave_up() reads it.
 *
 * Memory-lean mode: a forward run WITHOUT save_for_backward keeps nothing, and sba_bwd called
 * with workspace = NULL first repeats the forward's sweep for the carries alone (about 0.7 of
 * a forward) into further tables of the scratch; this function then asks for twice as many
 * tables (it looks at whether p->workspace is NULL).
 */
size_t sba_bwd_scratch_bytes(const SbaParams* p);

/*
 * Row-block schedule for the packed layout, built on the host from host cu_seqlens
 * (n_seq+1 entries, leading 0).  Writes up to `capacity` rows of SBA_SCHEDULE_INTS (8)
 * int32 each into `out` (host memory) and returns the number of jobs: ints 0-3 of row i are
 * {first_token, doc_len, row_block, first carry-table column of the document} of the i-th job,
 * longest row-blocks first;
 * ints 4-7 are the same four of the job that comes i-th for the dK/dV kernel, whose sweeps
 * run from a row-block to the END of its document (or the number needed when
 * `out` is NULL or capacity is too small).  `n_heads` is the head count the schedule will be
 * launched with (0 if unknown): from SBA_DOC_MAJOR_GRID workgroups (jobs x heads) on, the
 * jobs of a document stay together, longest document first, so that its K and V stay in
 * the L2 of one XCD (a third of the HBM reads); smaller launches need the strict
 * longest-first order for their balance.  The caller copies the schedule to the device and
 * passes it as SbaParams.schedule.  Replaces the reference's 3-D launch grid
 * (n_docs, ceil(H/2), ceil(max_len/64)+1) and its long/short head pairing
 * (sb_varlen_fwd.py:288-289, 472-475).
 */
int sba_build_schedule(const int32_t* cu_seqlens_host, int n_seq, int n_heads, int32_t* out, int capacity);

/* Rows of queries one scheduled job covers (the kernels' row-block height). */
int sba_row_block(void);

/*
 * Size of the carry tables of a packed batch, in columns of sba_row_block() floats per head:
 * the sum over the documents of n*(n+1), n = ceil(len / sba_row_block()) (a row block keeps one
 * entry per query for every 64-key block it can see, nothing for the blocks right of the
 * diagonal).  From host cu_seqlens (n_seq+1 entries); the value goes into SbaParams.table_cols
 * and sizes sba_workspace_bytes() / sba_bwd_scratch_bytes().  The dense layout needs no call:
 * the library derives n_seq * n*(n+1) from seq_len.  (The reference keeps one float per query,
 * sb_fwd.py:146; the tables are what makes the backward atomic-free.)
 */
int64_t sba_table_columns(const int32_t* cu_seqlens_host, int n_seq);

/* Forward: o, rem (and the carry table when save_for_backward). */
int sba_fwd(const SbaParams* p);

/* Backward: dq, dk, dv from d_o, d_rem, q, k, v and the forward's carry table. */
int sba_bwd(const SbaParams* p);

/*
 * The attention weights A_ij themselves, in fp32: the reference forward's `return_attention` debug output
 * (sb_attn/sb_fwd.py:141-172 `W`, sb_varlen/sb_varlen_fwd.py:195-201 and :409-446).  Reads q, k, scale,
 * attend_current and the layout fields of *p (any dtype and head_dim; o, rem and the workspace are not
 * touched) and writes weights[b][h][i][j] (dense, [n_seq, n_heads, seq_len, seq_len] contiguous) or
 * weights[h][i][j] (packed, [n_heads, total_tokens, total_tokens] contiguous, i and j token positions in the
 * pack) for every allowed pair; all other entries are left as they are (zero-fill first, as the reference does).
 * A vector-ALU kernel: for inspection and tests, not for speed; its logits are the fp32 products of the inputs,
 * where the 16-bit matrix-core kernels round q times the logit scale to 16 bits first.
 */
int sba_attention_weights(const SbaParams* p, float* weights);

/*
 * Error word of the last backward that ran on this problem's scratch: *gave_up = 1 if one of its
 * kernels abandoned a bounded internal wait (its gradients are invalid), else 0.  `p` is the
 * SbaParams of that backward (sizes, workspace, bwd_scratch, stream); pass static_scratch_used = 1
 * after sba_bwd_static(), whose scratch the caller does not see.  Copies four bytes to the host on
 * p->stream and WAITS for that stream: a debugging and testing aid, not for a training loop or a
 * graph capture.  Problems without such waits (fp32, generic kernels) report 0 without a copy.
 * The reference's counterpart is the spin lock of locked_add (sb_varlen/sb_varlen_bwd.py:13-52),
 * which waits without bound and reports nothing.
 */
int sba_bwd_gave_up(const SbaParams* p, int static_scratch_used, int* gave_up);

/*
 * Backward without any allocation.  No counterpart in the reference: it is for callers that
 * cannot allocate device memory around the call (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  Same contract as sba_bwd(), except that
 * p->bwd_scratch / p->bwd_scratch_bytes are ignored: the scratch is an array of
 * SBA_STATIC_SCRATCH_BYTES that the library itself holds on every GPU it runs on, until the
 * process ends.  Problems with sba_bwd_scratch_bytes(p) above that limit are refused with
 * SBA_ERR_STATIC_LIMIT and nothing is launched.  The call allocates nothing and frees nothing;
 * the very first call on a device looks up the array's address there (make one call before a
 * graph capture starts).  All calls on one GPU share the one array, which keeps the previous
 * call's contents: calls that overlap on the same GPU (different streams or threads) race and
 * must be serialised by the caller; calls on different GPUs are independent.
 */
#define SBA_STATIC_SCRATCH_BYTES (64u << 20)
int sba_bwd_static(const SbaParams* p);

#ifdef __cplusplus
}
#endif
#endif /* SBA_MI355X_H */
