// C ABI of libsba_mi355x.so: argument checking, schedule building, kernel dispatch.
// Declarations and the reference interfaces they replace: include/sba_mi355x.h.
#include "sba_common.h"

#include <algorithm>
#include <climits>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

// Backward scratch of sba_bwd_static(): one array per GPU that loads this library, held until
// the process ends.  In host code this name is only a handle of the symbol, never a device
// address: the address on a given GPU comes from hipGetSymbolAddress (static_scratch() below).
static __device__ __align__(256) unsigned char scratch[SBA_STATIC_SCRATCH_BYTES];

namespace {

using sba::KParams;

bool force_generic() {
    const char* e = getenv("SBA_FORCE_GENERIC");
    return e && e[0] == '1';
}

bool is_16bit(const SbaParams* p) { return p->dtype == SBA_DTYPE_BF16 || p->dtype == SBA_DTYPE_F16; }

// The matrix-core kernels cover bf16, float16 and fp32 with head_dim 64 or 128 and the 16-bit types with head_dim
// 256; everything else takes the generic vector-ALU kernels.
bool use_mfma(const SbaParams* p) {
    if (force_generic()) return false;
    if (is_16bit(p) && p->head_dim == 256) return true;
    return (p->dtype == SBA_DTYPE_F32 || is_16bit(p)) && (p->head_dim == 64 || p->head_dim == 128);
}

// The MFMA backward is a separate switch so that the two directions can be brought up
// (and, with SBA_FORCE_GENERIC_BWD=1, cross-checked) independently.
bool use_mfma_bwd(const SbaParams* p) {
    const char* e = getenv("SBA_FORCE_GENERIC_BWD");
    if (e && e[0] == '1') return false;
    return use_mfma(p) && sba_mfma_bwd_available();
}

int64_t tab_tokens(const SbaParams* p) {
    return p->cu_seqlens ? (int64_t)p->total_tokens : (int64_t)p->n_seq * p->seq_len;
}

// Columns (128 floats) per head of one carry table: a sequence of n row blocks takes n*(n+1)
// (row block qb holds the 2*qb + 2 key blocks it can see); the packed layout's total comes from
// the caller (sba_table_columns() of the same cu_seqlens).
int64_t columns_of(int64_t len) {
    const int64_t n = (len + sba::kRowBlock - 1) / sba::kRowBlock;
    return n * (n + 1);
}
int64_t table_columns(const SbaParams* p) {
    return p->cu_seqlens ? p->table_cols : (int64_t)p->n_seq * columns_of(p->seq_len);
}
size_t table_bytes(const SbaParams* p) {
    size_t b = (size_t)p->n_heads * (size_t)table_columns(p) * sba::kRowBlock * sizeof(float);
    return (b + 255) & ~(size_t)255;
}

size_t generic_acc_bytes(const SbaParams* p) {
    size_t b = (size_t)2 * tab_tokens(p) * p->n_heads * sba_generic_padded_dim(p->head_dim) * sizeof(float);
    return (b + 255) & ~(size_t)255;
}

constexpr size_t kErrorWordBytes = 256;     // tail of the bf16 matrix-core backward's scratch: the error word

// Carry tables of the matrix-core path.  bf16, four in all: the forward writes two - the product of (1 - beta)
// entering the right 32 keys of every 64-key step (`rtab`) and the one entering its left 32 keys (`rmid`), so
// that every lane of the backward starts its chain from its own carry - and the dQ pass the two prefix tables
// (`gtab`, `gmid`).  fp32, two in all: the forward writes `rtab`, the dQ pass `gtab`.
int forward_tables(const SbaParams* p) { return is_16bit(p) ? 2 : 1; }
// tables in the backward's scratch: the dQ pass's own, plus the forward's when no workspace brings them
int scratch_tables(const SbaParams* p) { return forward_tables(p) * (p->workspace ? 1 : 2); }
// the bounded waits (and with them the error word) exist in the bf16 matrix-core backward only
bool has_error_word(const SbaParams* p) { return use_mfma_bwd(p) && is_16bit(p); }
// bf16 at head_dim 64: the dQ pass leaves a copy of q times the logit scale (bf16, [sequence][head][token][64], dense)
// behind the tables, for the key-owner stream kernel, whose score MFMAs then deliver base-2 logits
size_t scaled_q_bytes(const SbaParams* p) {
    if (!use_mfma_bwd(p) || !is_16bit(p) || p->head_dim != 64) return 0;
    size_t b = (size_t)tab_tokens(p) * p->n_heads * 64 * 2;
    return (b + 255) & ~(size_t)255;
}

sba::TensorArg cvt(const SbaTensor& t) { return sba::TensorArg{(char*)t.ptr, t.stride_b, t.stride_h, t.stride_t}; }
sba::VectorArg cvt(const SbaVector& t) { return sba::VectorArg{(char*)t.ptr, t.stride_b, t.stride_h}; }

// Largest token stride (elements) the matrix-core kernels take: 64 rows of it, in bytes of the wider
// element type, stay below 2^31.
constexpr int64_t kMaxTokenStride = (INT64_C(1) << 31) / (64 * 4) - 1;

int check_common(const SbaParams* p) {
    if (!p) return SBA_ERR_NULL;
    if (p->struct_size != sizeof(SbaParams)) return SBA_ERR_ABI;
    if (p->dtype != SBA_DTYPE_F32 && !is_16bit(p)) return SBA_ERR_DTYPE;
    if (p->n_seq <= 0 || p->n_heads <= 0 || p->seq_len <= 0 || p->total_tokens <= 0) return SBA_ERR_SHAPE;
    if (p->head_dim <= 0 || p->head_dim > sba::kMaxHeadDim) return SBA_ERR_SHAPE;
    if (!p->q.ptr || !p->k.ptr || !p->v.ptr) return SBA_ERR_NULL;
    if (p->cu_seqlens) {
        if (!p->schedule || p->n_schedule <= 0 || p->table_cols <= 0) return SBA_ERR_SCHEDULE;
    } else if (p->total_tokens != p->seq_len) {
        return SBA_ERR_SHAPE;
    }
    if (use_mfma(p)) {
        // the matrix-core kernels move 16-byte chunks: aligned rows, outer strides in whole chunks
        const int64_t per16 = p->dtype == SBA_DTYPE_F32 ? 3 : 7;
        for (const SbaTensor* t : {&p->q, &p->k, &p->v, &p->o, &p->d_o, &p->dq, &p->dk, &p->dv}) {
            if (!t->ptr) continue;          // presence is checked per direction
            if (((uintptr_t)t->ptr & 15) || (t->stride_b & per16) || (t->stride_h & per16) || (t->stride_t & per16)) return SBA_ERR_SHAPE;
            // the tile copies address a 64-row tile with 32-bit byte offsets from its first row
            if (t->stride_t < 0 || t->stride_t > kMaxTokenStride) return SBA_ERR_SHAPE;
        }
    }
    return SBA_OK;
}

KParams make_kparams(const SbaParams* p) {
    KParams kp;
    memset(&kp, 0, sizeof(kp));
    kp.n_seq = p->n_seq; kp.n_heads = p->n_heads; kp.seq_len = p->seq_len;
    kp.total_tokens = p->total_tokens; kp.head_dim = p->head_dim;
    kp.attend_current = p->attend_current ? 1 : 0;
    kp.save = p->save_for_backward ? 1 : 0;
    kp.scale = p->scale; kp.scale2 = p->scale * sba::kLog2e;
    kp.cu_seqlens = p->cu_seqlens; kp.schedule = p->schedule;
    if (p->cu_seqlens) {
        kp.n_jobs = p->n_schedule;
    } else {
        kp.n_jobs = p->n_seq * ((p->seq_len + sba::kRowBlock - 1) / sba::kRowBlock);
    }
    kp.q = cvt(p->q); kp.k = cvt(p->k); kp.v = cvt(p->v); kp.o = cvt(p->o);
    kp.d_o = cvt(p->d_o); kp.dq = cvt(p->dq); kp.dk = cvt(p->dk); kp.dv = cvt(p->dv);
    kp.rem = cvt(p->rem); kp.d_rem = cvt(p->d_rem);
    kp.tab_head_stride = table_columns(p) * sba::kRowBlock;
    kp.tab_tokens = tab_tokens(p);
    const size_t tb = table_bytes(p);
    const bool two = forward_tables(p) == 2;
    // Layout rule that the dQ kernels rely on: gmid - rtab == gtab - rmid (one table size both times), so that a
    // lane finds its prefix entry at one uniform distance from its carry entry whichever half-wave it is in.
    if (p->workspace && use_mfma(p)) {
        if (two) { kp.rmid = (float*)p->workspace; kp.rtab = (float*)((char*)p->workspace + tb); }
        else kp.rtab = (float*)p->workspace;
    }
    char* bs = (char*)p->bwd_scratch;
    if (bs && use_mfma_bwd(p)) {
        int slot = 0;
        kp.gtab = (float*)(bs + tb * slot++);
        if (two) kp.gmid = (float*)(bs + tb * slot++);
        if (!p->workspace) {                       // the forward's tables, recomputed by sba_bwd
            if (two) kp.rmid = (float*)(bs + tb * slot++);
            kp.rtab = (float*)(bs + tb * slot++);
        }
        char* tail = bs + tb * slot;
        if (scaled_q_bytes(p)) {
            const int64_t per_head = (p->cu_seqlens ? (int64_t)p->total_tokens : (int64_t)p->seq_len) * 64;
            kp.q_scaled = sba::TensorArg{tail, p->cu_seqlens ? 0 : per_head * p->n_heads, per_head, 64};
            tail += scaled_q_bytes(p);
        }
        if (has_error_word(p)) kp.gave_up = (int*)tail;
    } else if (bs) {
        kp.dkv32 = (float*)bs;
    }
    return kp;
}

// Device address of the static scratch array on the CURRENT device: asked once per device
// (every GPU holds its own copy of the array at its own address) and kept.
int static_scratch(void** out) {
    constexpr int kMaxDevices = 64;
    static void* ptrs[kMaxDevices] = {nullptr};
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SBA_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return SBA_ERR_LAUNCH;
        ptrs[dev] = ptr;
    }
    *out = ptrs[dev];
    return SBA_OK;
}

}  // namespace

extern "C" {

int sba_abi_version(void) { return SBA_ABI_VERSION; }

const char* sba_error_string(int code) {
    switch (code) {
        case SBA_OK: return "ok";
        case SBA_ERR_NULL: return "a required pointer is NULL";
        case SBA_ERR_SHAPE: return "bad shape: sizes must be positive, head_dim <= 256, dense total_tokens == seq_len; at head_dim 64 / 128 (the matrix-core kernels, bf16 and fp32) and 256 (bf16) tensors need 16-byte aligned pointers, outer strides that are multiples of 16 bytes and a token stride below 2^23 elements";
        case SBA_ERR_DTYPE: return "unsupported dtype (SBA_DTYPE_F32, SBA_DTYPE_BF16 or SBA_DTYPE_F16)";
        case SBA_ERR_WORKSPACE: return "workspace / bwd_scratch missing or smaller than sba_workspace_bytes() / sba_bwd_scratch_bytes()";
        case SBA_ERR_SCHEDULE: return "packed layout needs a row-block schedule from sba_build_schedule()";
        case SBA_ERR_LAUNCH: return "kernel launch failed";
        case SBA_ERR_ABI: return "SbaParams.struct_size does not match this library";
        case SBA_ERR_STATIC_LIMIT: return "problem needs more backward scratch than sba_bwd_static() holds (SBA_STATIC_SCRATCH_BYTES); use sba_bwd() with a caller-allocated bwd_scratch";
        default: return "unknown error";
    }
}

size_t sba_workspace_bytes(const SbaParams* p) {
    if (!p || p->n_heads <= 0 || p->seq_len <= 0 || p->head_dim <= 0 || p->head_dim > sba::kMaxHeadDim) return 0;
    if (p->cu_seqlens && p->table_cols <= 0) return 0;
    return use_mfma(p) ? forward_tables(p) * table_bytes(p) : 0;
}

size_t sba_bwd_scratch_bytes(const SbaParams* p) {
    if (!p || p->n_heads <= 0 || p->seq_len <= 0 || p->head_dim <= 0 || p->head_dim > sba::kMaxHeadDim) return 0;
    if (p->cu_seqlens && p->table_cols <= 0 && use_mfma_bwd(p)) return 0;
    // without a workspace the backward recomputes the forward's tables first, into slots of its own
    if (!use_mfma_bwd(p)) return generic_acc_bytes(p);
    return scratch_tables(p) * table_bytes(p) + scaled_q_bytes(p) + (has_error_word(p) ? kErrorWordBytes : 0);
}

int sba_row_block(void) { return sba::kRowBlock; }

int64_t sba_table_columns(const int32_t* cu, int n_seq) {
    if (!cu || n_seq <= 0) return 0;
    int64_t cols = 0;
    for (int s = 0; s < n_seq; ++s) cols += columns_of(std::max(cu[s + 1] - cu[s], 0));
    return cols;
}

int sba_build_schedule(const int32_t* cu, int n_seq, int n_heads, int32_t* out, int capacity) {
    if (!cu || n_seq <= 0) return 0;
    struct J { int32_t tok0, len, rb, doc, tab0; };
    std::vector<J> jobs;
    int64_t cols = 0;                  // carry-table columns of the documents so far
    for (int s = 0; s < n_seq; ++s) {
        int32_t len = cu[s + 1] - cu[s];
        if (len <= 0) continue;
        int n_rb = (len + sba::kRowBlock - 1) / sba::kRowBlock;
        if (cols + columns_of(len) > INT32_MAX) return 0;       // tables of this size are out of reach anyway
        for (int rb = 0; rb < n_rb; ++rb) jobs.push_back(J{cu[s], len, rb, s, (int32_t)cols});
        cols += columns_of(len);
    }
    int n = (int)jobs.size();
    // Longest sweeps first; a stable order keeps the schedule deterministic.  Very large launches
    // keep the jobs of a document together instead (longest document first, its longest sweeps
    // first): with thousands of workgroups the balance takes care of itself, and the K/V of the
    // documents in flight then fit the L2 of the XCD that runs them.
    const bool doc_major = (int64_t)n * n_heads >= SBA_DOC_MAJOR_GRID;
    if (doc_major)
        std::stable_sort(jobs.begin(), jobs.end(), [](const J& a, const J& b) {
            return a.len != b.len ? a.len > b.len : a.doc != b.doc ? a.doc < b.doc : a.rb > b.rb; });
    else
        std::stable_sort(jobs.begin(), jobs.end(), [](const J& a, const J& b) { return a.rb > b.rb; });
    if (out && capacity >= n) {
        // second half of row i: the job that comes i-th for the key-owner kernels, whose sweep
        // from a job's row-block to the end of its sequence is (blocks of the sequence - rb) long
        std::vector<int> key_order(n);
        for (int i = 0; i < n; ++i) key_order[i] = i;
        auto key_len = [&](int i) { return (jobs[i].len + sba::kRowBlock - 1) / sba::kRowBlock - jobs[i].rb; };
        if (doc_major)      // `jobs` is document-major already; the key owners want rb ascending inside a document
            std::stable_sort(key_order.begin(), key_order.end(), [&](int a, int b) {
                const J& x = jobs[a]; const J& y = jobs[b];
                return x.len != y.len ? x.len > y.len : x.doc != y.doc ? x.doc < y.doc : x.rb < y.rb; });
        else
            std::stable_sort(key_order.begin(), key_order.end(), [&](int a, int b) { return key_len(a) > key_len(b); });
        for (int i = 0; i < n; ++i) {
            int32_t* o = out + (size_t)sba::kScheduleInts * i;
            const J& k = jobs[key_order[i]];
            o[0] = jobs[i].tok0; o[1] = jobs[i].len; o[2] = jobs[i].rb; o[3] = jobs[i].tab0;
            o[4] = k.tok0; o[5] = k.len; o[6] = k.rb; o[7] = k.tab0;
        }
    }
    return n;
}

int sba_fwd(const SbaParams* p) {
    int rc = check_common(p);
    if (rc) return rc;
    if (!p->o.ptr || !p->rem.ptr) return SBA_ERR_NULL;
    const bool mfma = use_mfma(p);
    if (mfma && p->save_for_backward) {
        if (!p->workspace || p->workspace_bytes < sba_workspace_bytes(p)) return SBA_ERR_WORKSPACE;
    }
    KParams kp = make_kparams(p);
    hipStream_t s = (hipStream_t)p->stream;
    if (mfma && p->dtype == SBA_DTYPE_F32) return sba_launch_mfma_f32_fwd(kp, s);
    if (mfma && p->dtype == SBA_DTYPE_F16) return sba_launch_mfma_f16_fwd(kp, s);
    return mfma ? sba_launch_mfma_fwd(kp, s) : sba_launch_generic_fwd(kp, p->dtype, s);
}

int sba_attention_weights(const SbaParams* p, float* weights) {
    int rc = check_common(p);
    if (rc) return rc;
    if (!weights) return SBA_ERR_NULL;
    KParams kp = make_kparams(p);
    kp.weights = weights;
    return sba_launch_generic_weights(kp, p->dtype, (hipStream_t)p->stream);
}

int sba_bwd(const SbaParams* p) {
    int rc = check_common(p);
    if (rc) return rc;
    if (!p->d_o.ptr || !p->dq.ptr || !p->dk.ptr || !p->dv.ptr) return SBA_ERR_NULL;
    if (p->bwd_phases < 0 || p->bwd_phases > 2) return SBA_ERR_SHAPE;
    if (use_mfma_bwd(p) && p->workspace && p->workspace_bytes < sba_workspace_bytes(p)) return SBA_ERR_WORKSPACE;
    if (!p->bwd_scratch || p->bwd_scratch_bytes < sba_bwd_scratch_bytes(p)) return SBA_ERR_WORKSPACE;
    KParams kp = make_kparams(p);
    hipStream_t s = (hipStream_t)p->stream;
    if (use_mfma_bwd(p) && !p->workspace && p->bwd_phases != 2) {
        // no table from the forward: run its sweep again for the carries alone (no P*V, no outputs)
        KParams carry = kp;
        carry.save = 1;
        carry.carry_only = 1;
        rc = p->dtype == SBA_DTYPE_F32 ? sba_launch_mfma_f32_fwd(carry, s)
           : p->dtype == SBA_DTYPE_F16 ? sba_launch_mfma_f16_fwd(carry, s) : sba_launch_mfma_fwd(carry, s);
        if (rc) return rc;
    }
    // the generic backward is one piece: it all runs in phase 1
    if (!use_mfma_bwd(p) && p->bwd_phases == 2) return SBA_OK;
    if (use_mfma_bwd(p) && p->dtype == SBA_DTYPE_F32) return sba_launch_mfma_f32_bwd(kp, p->bwd_phases, s);
    if (use_mfma_bwd(p) && p->dtype == SBA_DTYPE_F16) return sba_launch_mfma_f16_bwd(kp, p->bwd_phases, s);
    return use_mfma_bwd(p) ? sba_launch_mfma_bwd(kp, p->bwd_phases, s) : sba_launch_generic_bwd(kp, p->dtype, s);
}

int sba_bwd_gave_up(const SbaParams* p, int static_scratch_used, int* gave_up) {
    if (!gave_up) return SBA_ERR_NULL;
    *gave_up = 0;
    int rc = check_common(p);
    if (rc) return rc;
    if (!has_error_word(p)) return SBA_OK;
    void* bs = p->bwd_scratch;
    if (static_scratch_used) {
        rc = static_scratch(&bs);
        if (rc) return rc;
    }
    if (!bs) return SBA_ERR_WORKSPACE;
    const char* word = (const char*)bs + scratch_tables(p) * table_bytes(p) + scaled_q_bytes(p);
    hipStream_t s = (hipStream_t)p->stream;
    int host = 0;
    if (hipMemcpyAsync(&host, word, sizeof(int), hipMemcpyDeviceToHost, s) != hipSuccess) return SBA_ERR_LAUNCH;
    if (hipStreamSynchronize(s) != hipSuccess) return SBA_ERR_LAUNCH;
    *gave_up = host;
    return SBA_OK;
}

int sba_bwd_static(const SbaParams* p) {
    int rc = check_common(p);
    if (rc) return rc;
    if (sba_bwd_scratch_bytes(p) > (size_t)SBA_STATIC_SCRATCH_BYTES) return SBA_ERR_STATIC_LIMIT;
    void* ptr = nullptr;
    rc = static_scratch(&ptr);
    if (rc) return rc;
    // Nothing in the array has to start at zero: the matrix-core kernels write every table entry
    // before they read it, and the generic path clears its accumulators with a fill kernel.
    SbaParams q = *p;
    q.bwd_scratch = ptr;
    q.bwd_scratch_bytes = SBA_STATIC_SCRATCH_BYTES;
    return sba_bwd(&q);
}

}  // extern "C"
