// Shared device/host helpers for the stick-breaking attention kernels (gfx950).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <atomic>
#include "../../include/sba_mi355x.h"

namespace sba {

constexpr int kRowBlock = 128;   // query rows per scheduled job (one workgroup)
constexpr int kMaxHeadDim = 256; // bf16: matrix-core kernels at 64, 128 and 256; every other size and type up to here: generic kernels
constexpr int kKeyBlock = 64;    // keys per sweep step of the MFMA kernels / carry-table column

// Generic (fp32 / any head dim) kernels only: logits above this (in base-2 units) are clamped;
// sigmoid(z) differs from 1 by < 2^-30 there, so outputs move by < 1e-9, and exp2 of the clamped
// value cannot overflow.  The matrix-core kernels do not clamp: their product chains let
// 1 + e^z overflow to +inf (see sba_mfma.h).
constexpr float kMaxLogit2 = 30.0f;
constexpr float kLog2e = 1.4426950408889634f;

struct TensorArg { char* ptr; int64_t sb, sh, st; };
struct VectorArg { char* ptr; int64_t sb, sh; };

// Kernel-side copy of SbaParams (by value in the launch).
struct KParams {
    int n_seq, n_heads, seq_len, total_tokens, head_dim, attend_current, save, n_jobs;
    int carry_only;                // forward kernels: write the carry table and nothing else (no P*V, no o / rem)
    float scale2;                  // scale * log2(e): logits in base-2 units
    float scale;                   // natural-unit scale (for dq/dk)
    const int32_t* cu_seqlens;
    const int32_t* schedule;
    TensorArg q, k, v, o, d_o, dq, dk, dv;
    VectorArg rem, d_rem;
    float* rtab;                   // forward carry table (layout: tab_index() below): the product of (1 - beta) over all keys
                                   //   right of a 64-key block, i.e. the carry entering its RIGHT 32 keys
    float* gtab;                   // backward prefix table, same shape: sum of g over all keys left of the block
    float* rmid;                   // the carry entering the block's LEFT 32 keys (bf16: written by the forward)
    float* gmid;                   // the prefix entering the block's RIGHT 32 keys (written by the dQ pass, like gtab);
                                   //   the bf16 dQ kernels rely on gmid - rtab == gtab - rmid
    TensorArg q_scaled;            // bf16 head_dim 64 backward: q times scale2, rounded to bf16, written by the dQ pass for
                                   //   the key-owner stream kernel (ptr NULL: not wanted)
    float* dkv32;                  // generic path: fp32 dk|dv accumulators
    float* weights;                // sba_attention_weights(): the attention weights, fp32 (debug output)
    int* gave_up;                  // backward error word (set if a kernel abandoned a bounded internal wait)
    int64_t tab_head_stride;       // floats per head in each carry table
    int64_t tab_tokens;            // generic path: tokens per head in the fp32 accumulators (n_seq*T dense, sumT packed)
};

// tab0: first carry-table column of the job's sequence
struct Job { int tok0, len, rb, seq, tab0; };

// Workgroup -> (job, head).  blockIdx.x = slot * n_heads + head, so that consecutive
// workgroups (which the dispatcher deals round-robin to the 8 XCDs) are different heads of
// the same job and a head stays on one XCD's L2.  Jobs are sorted by decreasing sweep
// length (longest first); `longest_last` walks the list from its other end (the key-owner
// pass, whose work grows as the row-block index falls).
__device__ inline int order_job(int slot, int n_jobs, bool longest_last) {
    return longest_last ? n_jobs - 1 - slot : slot;
}

// Dense jobs are generated arithmetically (row-blocks in decreasing order); packed jobs
// come from the host-built schedule, which has the same order.  Row i of the schedule:
// {first_token, doc_len, row_block, first table column of the document} of the i-th job, then
// the same four of the job that comes i-th for the key-owner kernels.
constexpr int kScheduleInts = 8;

// The schedule is read-only for the kernels and indexed with wave-uniform values: read it
// through the constant address space, so that the loads are scalar (one per wave, and no wait
// for the vector-memory traffic in flight).
typedef const __attribute__((address_space(4))) int32_t* ScheduleRow;
__device__ inline ScheduleRow schedule_row(const KParams& p, int i, int offset) {
    return (ScheduleRow)(uintptr_t)(p.schedule + kScheduleInts * (int64_t)i + offset);
}

__device__ inline Job dense_job(const KParams& p, int job) {
    Job j;
    int n_rb = (p.seq_len + kRowBlock - 1) / kRowBlock;
    j.rb = n_rb - 1 - job / p.n_seq;
    j.seq = job % p.n_seq;
    j.tok0 = 0;
    j.len = p.seq_len;
    j.tab0 = j.seq * n_rb * (n_rb + 1);
    return j;
}

__device__ inline Job decode_job(const KParams& p, int job) {
    if (p.cu_seqlens == nullptr) return dense_job(p, job);
    const ScheduleRow s = schedule_row(p, job, 0);
    Job j;
    j.tok0 = s[0]; j.len = s[1]; j.rb = s[2]; j.seq = 0; j.tab0 = s[3];
    return j;
}

// The key-owner (dK/dV) kernels sweep from a job's row-block to the END of its sequence:
// their longest sweeps are the FIRST row-blocks of the longest sequences.  i-th job in that
// order: arithmetic for the dense layout, the second half of row i of the host-built schedule
// for the packed.
__device__ inline Job decode_key_job(const KParams& p, int i) {
    if (p.cu_seqlens == nullptr) return dense_job(p, p.n_jobs - 1 - i);
    const ScheduleRow s = schedule_row(p, i, 4);
    Job j;
    j.tok0 = s[0]; j.len = s[1]; j.rb = s[2]; j.seq = 0; j.tab0 = s[3];
    return j;
}

// Token index inside the generic path's fp32 accumulators.
__device__ inline int64_t tab_token(const KParams& p, const Job& j, int local) {
    return (p.cu_seqlens == nullptr) ? (int64_t)j.seq * p.seq_len + local : (int64_t)j.tok0 + local;
}

// Carry tables, compact layout: every sequence has one slab per 128-query row block qb that
// holds exactly the 2*qb + 2 key blocks (64 keys each) that row block can see, as
// [key block][128 queries] fp32.  The slabs of a sequence follow each other (row block qb
// starts qb*(qb+1) columns into the sequence's part, a column being 128 floats), the sequences
// follow each other (Job::tab0), heads are outermost.  A sequence of n row blocks takes
// n*(n+1) columns: half of a full [key blocks][tokens] rectangle.
// Returns the index of (row block qb, key block kb, query 0 of the row block).
__device__ inline int64_t tab_index(const KParams& p, int head, const Job& j, int qb, int kb) {
    return (int64_t)head * p.tab_head_stride + ((int64_t)j.tab0 + qb * (qb + 1) + kb) * kRowBlock;
}

__device__ inline float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ inline uint16_t f32_to_bf16(float f) {   // round to nearest even
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    __device__ static float load(const char* p, int64_t i) { return ((const float*)p)[i]; }
    __device__ static void store(char* p, int64_t i, float v) { ((float*)p)[i] = v; }
};
template <> struct Elem<_Float16> {
    __device__ static float load(const char* p, int64_t i) { return (float)((const _Float16*)p)[i]; }
    __device__ static void store(char* p, int64_t i, float v) { ((_Float16*)p)[i] = (_Float16)v; }
};
template <> struct Elem<uint16_t> {   // bf16 bits
    __device__ static float load(const char* p, int64_t i) { return bf16_to_f32(((const uint16_t*)p)[i]); }
    __device__ static void store(char* p, int64_t i, float v) { ((uint16_t*)p)[i] = f32_to_bf16(v); }
};

}  // namespace sba

// SBA_TWO_STEP_MAX_GRID (experiments and tests; read once per process): grids of at most this many workgroups take
// the kernels that split a sweep inside the workgroup (head_dim 64), larger ones do not.  -1: not set.
inline int sba_two_step_env() {
    static const int v = [] {
        const char* e = getenv("SBA_TWO_STEP_MAX_GRID");
        return e ? atoi(e) : -1;
    }();
    return v;
}
inline unsigned sba_two_step_max_grid(unsigned by_default) {
    return sba_two_step_env() >= 0 ? (unsigned)sba_two_step_env() : by_default;
}
// The two-steps-per-iteration dQ kernel up to 544 workgroups (measured at H = 16: 103.9 us against the one-step
// kernel's 106.4 at 528 workgroups, 122.0 against 120.6 at 576).  The forward's rule is in sba_launch_mfma_fwd().
constexpr unsigned kTwoStepDqMaxGrid = 544;

// compute units of the current device (asked once per device)
inline int sba_cu_count() {
    static std::atomic<int> cached[64];       // zero-initialised; threads that race here store the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// How long a launch's longest sweep is against the work of an average workgroup slot when every workgroup runs
// one sweep and a CU holds four of them:  r = longest sweep x (4 x CUs) / all sweep steps of the launch  (steps of
// 64 keys; a sequence of n row blocks has n (n + 1) of them per head, which is also its number of carry-table
// columns).  A launch cannot end before its longest sweep has; for r well above 1 most of the chip idles behind
// it, and the kernels that cut a sweep into pieces pay.  seq_len is the longest sequence of the launch.
inline double sba_tail_ratio(const sba::KParams& kp, unsigned grid) {
    const double longest = 2.0 * ((kp.seq_len + sba::kRowBlock - 1) / sba::kRowBlock);
    double steps = (double)(kp.tab_head_stride / sba::kRowBlock) * kp.n_heads;
    if (steps <= 0) steps = (double)grid * (longest / 2 + 1);          // (no table size given: every sweep half the longest)
    return longest * 4.0 * sba_cu_count() / steps;
}

// Launchers implemented in the kernel translation units.
int sba_generic_padded_dim(int D);
int sba_launch_generic_fwd(const sba::KParams& kp, int dtype, hipStream_t s);
int sba_launch_generic_bwd(const sba::KParams& kp, int dtype, hipStream_t s);
int sba_launch_generic_weights(const sba::KParams& kp, int dtype, hipStream_t s);
int sba_launch_mfma_fwd(const sba::KParams& kp, hipStream_t s);
int sba_launch_mfma_bwd(const sba::KParams& kp, int phases, hipStream_t s);
int sba_launch_mfma_f16_fwd(const sba::KParams& kp, hipStream_t s);       // the same kernels compiled for float16 elements
int sba_launch_mfma_f16_bwd(const sba::KParams& kp, int phases, hipStream_t s);
int sba_launch_mfma_f32_fwd(const sba::KParams& kp, hipStream_t s);
int sba_launch_mfma_f32_bwd(const sba::KParams& kp, int phases, hipStream_t s);
bool sba_mfma_bwd_available();
