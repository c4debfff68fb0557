// bf16 MFMA forward kernel (head_dim 64 / 128).
// Replaces the reference's `_forward_one_row` sweep (sb_varlen/sb_varlen_fwd.py:81-215):
// one workgroup per (sequence, head, 128-query row-block), keys swept right-to-left from
// the diagonal in steps of 64, K/V tiles double-buffered in LDS, running product of
// (1 - beta) per query in a register.  Layout and arithmetic: sba_mfma.h.
#include "sba_mfma.h"

namespace sba {

// kCarryOnly: write the carry table and nothing else (no P*V, no o / rem): the backward's way of
// getting the table when the forward kept none.
template <int D, bool kCarryOnly>
__global__ __launch_bounds__(kThreads) void mfma_fwd_kernel(KParams p) {
    constexpr int kTile = 64 * D * 2;            // bytes per K or V tile
    __shared__ __attribute__((aligned(16))) char lds[4 * kTile];   // K0 V0 K1 V1

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform, keep it scalar
    const int n = lane & 31, h = lane >> 5;
    LaneOffsets<D> lo;
    lo.init(lane);
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_job(p, order_job(blockIdx.x / p.n_heads, p.n_jobs, false));
    const int strict = p.attend_current ? 0 : 1;
    const int m0 = job.rb * kRowBlock;
    const int q0w = m0 + 32 * wave;              // first query of this wave
    const int qi = q0w + n;                      // this lane's query
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;

    bf16x8 qf[D / 16];
    load_row_frags<D>(qf, p.q, qbase, qi, job.len, lane);

    f32x16 oacc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) oacc[db] = f32x16{0};
    float R = 1.0f;

    const int imax = min(m0 + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;                       // last key any row of the block sees
    const int n_steps = kmax >= 0 ? kmax / kKeyBlock + 1 : 0;
    const int64_t tabq = tab_index(p, head, job, job.rb, 0) + 32 * wave + n;   // + step * kRowBlock

    TileDma<D> kc, vc;
    kc.init(lane, wave, p.k, kbase);
    vc.init(lane, wave, p.v, vbase);
    if (n_steps > 0) {
        kc.issue((n_steps - 1) * kKeyBlock, job.len, lds);
        if (!kCarryOnly) vc.issue((n_steps - 1) * kKeyBlock, job.len, lds + kTile);
    }
    wait_global_memory();
    __syncthreads();

    for (int step = n_steps - 1, buf = 0; step >= 0; --step, buf ^= 1) {
        const char* ktile = lds + buf * 2 * kTile;
        const char* vtile = ktile + kTile;
        const bool more = step > 0;
        const int key0 = step * kKeyBlock;
        // whole step right of this wave's last query: nothing visible
        const bool skip = key0 + strict > q0w + 31;
        // The carry-table store goes FIRST: vector-memory operations retire in order, so the
        // wait for the tile loads at the end of the step then also covers this store, long
        // after it has completed, instead of stalling the next iteration's loads on it.
        if (!skip && p.save && h == 0 && qi < job.len)
            p.rtab[tabq + step * kRowBlock] = R;
        if (more) {       // next tiles, straight into the other buffer (free since the last barrier)
            kc.issue((step - 1) * kKeyBlock, job.len, lds + (buf ^ 1) * 2 * kTile);
            if (!kCarryOnly) vc.issue((step - 1) * kKeyBlock, job.len, lds + (buf ^ 1) * 2 * kTile + kTile);
        }
        if (!skip) {
            float x[32];
            score_tiles_o<D>(x, ktile, lo, qf, p.scale2);
            if (key0 + 63 + strict > q0w) {     // diagonal region: mask invisible pairs
mask_step(x, key0 + 32 * h, qi, strict);
            }
            float dummy[1];
            stick_weights<false>(x, dummy, R, lane);
            if (!kCarryOnly) {
                bf16x8 pf[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) pf[c] = pack8(&x[8 * c]);
                if (D == 128) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {      // (operands of a key group requested together, see score_raw_o)
                        bf16x8 vt[D / 32];
#pragma unroll
                        for (int db = 0; db < D / 32; ++db) vt[db] = fetch_cols_o<D>(vtile, lo, db, c);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int db = 0; db < D / 32; ++db) oacc[db] = mfma(vt[db], pf[c], oacc[db]);
                    }
                } else {
#pragma unroll
                    for (int db = 0; db < D / 32; ++db)
#pragma unroll
                        for (int c = 0; c < 4; ++c)
                            oacc[db] = mfma(fetch_cols_o<D>(vtile, lo, db, c), pf[c], oacc[db]);
                }
            }
        }
        wait_global_memory();                  // the next tiles have landed
        __syncthreads();
    }

    if (qi < job.len && !kCarryOnly) {
        const int64_t obase = (int64_t)job.seq * p.o.sb + (int64_t)head * p.o.sh + (int64_t)(job.tok0 + qi) * p.o.st;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                // rows d = 32*db + 8*g + 4*h + 0..3 of O^T, column = this query
                f32x2 a = {oacc[db][4 * g], oacc[db][4 * g + 1]};
                f32x2 b = {oacc[db][4 * g + 2], oacc[db][4 * g + 3]};
                bf16x2 pa = __builtin_convertvector(a, bf16x2), pb = __builtin_convertvector(b, bf16x2);
                uint2 w;
                w.x = __builtin_bit_cast(uint32_t, pa);
                w.y = __builtin_bit_cast(uint32_t, pb);
                *(uint2*)(p.o.ptr + 2 * (obase + 32 * db + 8 * g + 4 * h)) = w;
            }
        if (h == 0)
            Elem<uint16_t>::store(p.rem.ptr, (int64_t)job.seq * p.rem.sb + (int64_t)head * p.rem.sh + job.tok0 + qi, R);
    }
}

// ---------------------------------------------------------------- two steps per iteration
// Same sweep with 8 waves: wave-group 0 (waves 0-3) and wave-group 1 (waves 4-7) take two
// CONSECUTIVE 64-key steps of the same 128 queries in every iteration.  All the heavy work of
// a step (scores, exp/rcp, the in-step product chain, P*V) only needs the step's own keys; what
// couples neighbouring steps is one number per query, the product of (1 - beta) over the
// step.  The groups swap those totals through LDS at a barrier, the left group multiplies the
// right group's total into its carry, and each group accumulates its own partial O, summed once
// at the end.  The longest dependent chain of a kernel launch (the sweep of the last row-block)
// is halved, which is what bounds the time when the whole problem is only two waves per SIMD.
template <int D, bool kCarryOnly>
__global__ __launch_bounds__(2 * kThreads) void mfma_fwd2_kernel(KParams p) {
    constexpr int kTile = 64 * D * 2;
    // tile(buf, grp, kv) = lds + ((buf * 2 + grp) * 2 + kv) * kTile
    __shared__ __attribute__((aligned(16))) char lds[8 * kTile];
    __shared__ float xch[2][kRowBlock];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int grp = wave >> 2, qs = wave & 3;
    const int n = lane & 31, h = lane >> 5;
    LaneOffsets<D> lo;
    lo.init(lane);
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_job(p, order_job(blockIdx.x / p.n_heads, p.n_jobs, false));
    const int strict = p.attend_current ? 0 : 1;
    const int m0 = job.rb * kRowBlock;
    const int q0w = m0 + 32 * qs;
    const int qi = q0w + n;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;

    bf16x8 qf[D / 16];
    load_row_frags<D>(qf, p.q, qbase, qi, job.len, lane);
    f32x16 oacc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) oacc[db] = f32x16{0};
    float R = 1.0f;

    const int imax = min(m0 + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    const int n_steps = kmax >= 0 ? kmax / kKeyBlock + 1 : 0;
    const int n_it = (n_steps + 1) / 2;
    const int64_t tabq = tab_index(p, head, job, job.rb, 0) + 32 * qs + n;   // + step * kRowBlock
    char* my_tiles = lds + grp * 2 * kTile;          // + buf * 4 * kTile

    // each group copies its own tiles (256 threads per tile pair)
    TileDma<D> kc, vc;
    kc.init(lane, qs, p.k, kbase);
    vc.init(lane, qs, p.v, vbase);
    {
        const int s0 = n_steps - 1 - grp;
        if (s0 >= 0) {
            kc.issue(s0 * kKeyBlock, job.len, my_tiles);
            if (!kCarryOnly) vc.issue(s0 * kKeyBlock, job.len, my_tiles + kTile);
        }
    }
    wait_global_memory();
    __syncthreads();

    for (int it = 0, buf = 0; it < n_it; ++it, buf ^= 1) {
        const int step = n_steps - 1 - 2 * it - grp;          // -1: this group idles in the last iteration
        const char* ktile = my_tiles + buf * 4 * kTile;
        const char* vtile = ktile + kTile;
        const bool more = step - 2 >= 0;
        if (more) {       // next tiles, straight into the other buffer (free since the last barrier)
            kc.issue((step - 2) * kKeyBlock, job.len, my_tiles + (buf ^ 1) * 4 * kTile);
            if (!kCarryOnly) vc.issue((step - 2) * kKeyBlock, job.len, my_tiles + (buf ^ 1) * 4 * kTile + kTile);
        }
        const int key0 = step * kKeyBlock;
        const bool active = step >= 0 && !(key0 + strict > q0w + 31);
        float x[32];
        float total = 1.0f, fac = 1.0f;
        if (active) {
            score_tiles_o<D, true>(x, ktile, lo, qf, p.scale2);
            if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
            float dummy[1];
            fac = stick_weights_local<false>(x, dummy, total, lane);
        }
        if (h == 0) xch[grp][32 * qs + n] = total;
        __syncthreads();
        const float other = xch[grp ^ 1][32 * qs + n];
        // group 0 holds the right step of the pair: its carry is R; group 1's also contains
        // group 0's total
        const float Rmy = grp == 0 ? R : R * other;
        R = R * total * other;
        if (active) {
            if (p.save && h == 0 && qi < job.len)
                p.rtab[tabq + step * kRowBlock] = Rmy;
            if (!kCarryOnly) {
                scale_clamped<32>(x, fac * Rmy);
                bf16x8 pf[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) pf[c] = pack8(&x[8 * c]);
#pragma unroll
                for (int c2 = 0; c2 < 2; ++c2) {   // operands of two key groups requested together, ahead of their MFMAs
                    bf16x8 vt[2][D / 32];
#pragma unroll
                    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                        for (int db = 0; db < D / 32; ++db) vt[cc][db] = fetch_cols_o<D>(vtile, lo, db, 2 * c2 + cc);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                        for (int db = 0; db < D / 32; ++db) oacc[db] = mfma(vt[cc][db], pf[2 * c2 + cc], oacc[db]);
                }
            }
        }
        wait_global_memory();                  // the next tiles have landed
        __syncthreads();
    }
    if (kCarryOnly) return;

    // ---- O = O(group 0) + O(group 1): group 1 parks its accumulators in LDS
    float* park = (float*)lds;                              // [qs][db][r][lane]
    if (grp == 1) {
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) park[((qs * (D / 32) + db) * 16 + r) * 64 + lane] = oacc[db][r];
    }
    __syncthreads();
    if (grp == 0 && qi < job.len) {
        const int64_t obase = (int64_t)job.seq * p.o.sb + (int64_t)head * p.o.sh + (int64_t)(job.tok0 + qi) * p.o.st;
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[db][r] += park[((qs * (D / 32) + db) * 16 + r) * 64 + lane];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x2 a = {oacc[db][4 * g], oacc[db][4 * g + 1]};
                f32x2 b = {oacc[db][4 * g + 2], oacc[db][4 * g + 3]};
                bf16x2 pa = __builtin_convertvector(a, bf16x2), pb = __builtin_convertvector(b, bf16x2);
                uint2 w;
                w.x = __builtin_bit_cast(uint32_t, pa);
                w.y = __builtin_bit_cast(uint32_t, pb);
                *(uint2*)(p.o.ptr + 2 * (obase + 32 * db + 8 * g + 4 * h)) = w;
            }
        }
        if (h == 0)
            Elem<uint16_t>::store(p.rem.ptr, (int64_t)job.seq * p.rem.sb + (int64_t)head * p.rem.sh + job.tok0 + qi, R);
    }
}

}  // namespace sba

int sba_launch_mfma_fwd(const sba::KParams& kp, hipStream_t s) {
    using namespace sba;
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    // A grid this small cannot give every SIMD more than two waves, and the launch lasts as long
    // as its longest sweep: take the variant that halves that chain.  Larger grids are bound
    // by throughput, where the 4-wave kernel (3 waves per SIMD) is ahead (measured: already at
    // 640 workgroups).
    const bool small_grid = grid.x <= sba_two_step_max_grid();
    if (kp.carry_only) {
        if (kp.head_dim == 64 && small_grid)
            hipLaunchKernelGGL((mfma_fwd2_kernel<64, true>), grid, dim3(2 * kThreads), 0, s, kp);
        else if (kp.head_dim == 64)
            hipLaunchKernelGGL((mfma_fwd_kernel<64, true>), grid, dim3(kThreads), 0, s, kp);
        else
            hipLaunchKernelGGL((mfma_fwd_kernel<128, true>), grid, dim3(kThreads), 0, s, kp);
    } else if (kp.head_dim == 64 && small_grid)
        hipLaunchKernelGGL((mfma_fwd2_kernel<64, false>), grid, dim3(2 * kThreads), 0, s, kp);
    else if (kp.head_dim == 64)
        hipLaunchKernelGGL((mfma_fwd_kernel<64, false>), grid, dim3(kThreads), 0, s, kp);
    else
        hipLaunchKernelGGL((mfma_fwd_kernel<128, false>), grid, dim3(kThreads), 0, s, kp);
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}
