// bf16 MFMA forward kernels (head_dim 64 / 128 / 256; at 256 the one-sweep kernel only: two K / V tile pairs are 128 KB of LDS).
// Replace the reference's `_forward_one_row` sweep (sb_varlen/sb_varlen_fwd.py:81-215):
// one workgroup per (sequence, head, 128-query row-block), keys swept right-to-left from
// the diagonal in steps of 64, K/V tiles double-buffered in LDS, running product of
// (1 - beta) per query in a register.  Layout and arithmetic: sba_mfma.h.
#include "sba_mfma.h"

namespace sba {
inline namespace SBA_ELEM_NS {

// One sweep step of one wave: 32 queries x 64 keys.  Scores (from the pre-scaled Q fragments),
// mask on the diagonal, weights, O^T += V^T P^T.  kFast: the one-reciprocal chain; it may refuse
// the step (returns false, nothing changed), see forward_weights_fast().  lane_carry: the product of
// (1 - beta) over all keys right of this LANE's 32 keys (the right half-wave's is the carry that entered
// the step), which is what the carry tables keep.
template <int D, bool kCarryOnly, bool kFast, bool kPinBase>
__device__ inline bool fwd_step(const char* ktile, const char* vtile, const LaneOffsets<D>& lo,
                                const h16x8 (&qf)[D / 16], f32x16 (&oacc)[D / 32], float& R, int lane,
                                int key0, int q0w, int qi, int strict, float& lane_carry) {
    const int h = lane >> 5;
    float x[32];
    score_tiles_ps<D>(x, ktile, lo, qf);
    if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);     // diagonal region
    h16x8 pf[4];
    if (kFast) {
        if (!forward_weights_fast<!kCarryOnly>(x, pf, R, lane, lane_carry)) return false;
    } else {
        float dummy[1];
        stick_weights<false>(x, dummy, R, lane, &lane_carry);
        if (!kCarryOnly) {
#pragma unroll
            for (int c = 0; c < 4; ++c) pf[c] = pack8(&x[8 * c]);
        }
    }
    if (!kCarryOnly) {
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {   // operands of two key groups requested together, ahead of their MFMAs
            h16x8 vt[2][D / 32];
#pragma unroll
            for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                for (int db = 0; db < D / 32; ++db) vt[cc][db] = fetch_cols_o<D, kPinBase>(vtile, lo, db, 2 * c2 + cc);
            if (D == 128) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                for (int db = 0; db < D / 32; ++db) oacc[db] = mfma(vt[cc][db], pf[2 * c2 + cc], oacc[db]);
        }
    }
    return true;
}

// rows d = 32*db + 8*g + 4*h + 0..3 of O^T, column = this lane's query
template <int D>
__device__ inline void store_o_row(const KParams& p, const Job& job, int head, int qi, int lane,
                                   const f32x16 (&oacc)[D / 32]) {
    const int h = lane >> 5;
    const int64_t obase = (int64_t)job.seq * p.o.sb + (int64_t)head * p.o.sh + (int64_t)(job.tok0 + qi) * p.o.st;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            f32x2 a = {oacc[db][4 * g], oacc[db][4 * g + 1]};
            f32x2 b = {oacc[db][4 * g + 2], oacc[db][4 * g + 3]};
            h16x2 pa = __builtin_convertvector(a, h16x2), pb = __builtin_convertvector(b, h16x2);
            uint2 w;
            w.x = __builtin_bit_cast(uint32_t, pa);
            w.y = __builtin_bit_cast(uint32_t, pb);
            *(uint2*)(p.o.ptr + 2 * (obase + 32 * db + 8 * g + 4 * h)) = w;
        }
}

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
    const bool rows_full = q0w + 31 < job.len;   // wave-uniform
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;

    h16x8 qf[D / 16];
    load_row_frags<D>(qf, p.q, qbase, qi, job.len, lane);
    prescale_frags(qf, p.scale2);

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

    // Carry tables: the right half-wave's carries go to `rtab`, the left one's to `rmid` (one store of the whole
    // wave).  A step's carries are only known after its chain (the left half's contain the right half's
    // product) and are stored at the top of the NEXT step, in front of its tile loads: vector-memory
    // operations retire in order, so the wait for those loads at the end of that step also covers the store,
    // long after it has completed, and no wait ever falls on a fresh store.
    float* const my_tab = h ? p.rtab : p.rmid;
    float carry_out = 1.0f;
    int carry_step = -1;                       // wave-uniform: the step whose carries wait to be stored
    auto store_carries = [&]() {
        if (carry_step >= 0 && p.save) {
            if (rows_full) my_tab[tabq + carry_step * kRowBlock] = carry_out;      // no lane mask
            else if (qi < job.len) my_tab[tabq + carry_step * kRowBlock] = carry_out;
        }
        carry_step = -1;
    };
    // what a step does before its arithmetic
    auto open_step = [&](int step, int buf, bool skip) {
        store_carries();
        if (step > 0) {   // next tiles, straight into the other buffer (free since the last barrier);
                          // every tile left of the sweep's first lies inside the sequence
            kc.issue_full((step - 1) * kKeyBlock, lds + (buf ^ 1) * 2 * kTile);
            if (!kCarryOnly) vc.issue_full((step - 1) * kKeyBlock, lds + (buf ^ 1) * 2 * kTile + kTile);
        }
    };
    // The sweep runs with the one-reciprocal chain until a step refuses it (logits too large for
    // it); from that step on this wave continues with the reciprocal-per-key chain.  Every wave
    // executes one barrier per step whichever loop it is in.
    int step = n_steps - 1, buf = 0;
    bool redo = false;
    for (; step >= 0; --step, buf ^= 1) {
        const char* ktile = lds + buf * 2 * kTile;
        const int key0 = step * kKeyBlock;
        // whole step right of this wave's last query, or all of this wave's queries past the end of the sequence
        const bool skip = key0 + strict > q0w + 31 || q0w >= job.len;
        open_step(step, buf, skip);
        if (!skip) {
            if (!fwd_step<D, kCarryOnly, true, D == 128>(ktile, ktile + kTile, lo, qf, oacc, R, lane, key0, q0w, qi, strict, carry_out)) {
                redo = true;
                break;
            }
            carry_step = step;
        }
        wait_global_memory();                  // the next tiles have landed
        __syncthreads();
    }
    for (; step >= 0; --step, buf ^= 1) {
        const char* ktile = lds + buf * 2 * kTile;
        const int key0 = step * kKeyBlock;
        const bool skip = key0 + strict > q0w + 31 || q0w >= job.len;
        if (!redo) open_step(step, buf, skip);
        redo = false;
        if (!skip) {
            fwd_step<D, kCarryOnly, false, D == 128>(ktile, ktile + kTile, lo, qf, oacc, R, lane, key0, q0w, qi, strict, carry_out);
            carry_step = step;
        }
        wait_global_memory();
        __syncthreads();
    }
    store_carries();

    if (qi < job.len && !kCarryOnly) {
        store_o_row<D>(p, job, head, qi, lane, oacc);
        if (h == 0)
            Elem16::store(p.rem.ptr, (int64_t)job.seq * p.rem.sb + (int64_t)head * p.rem.sh + job.tok0 + qi, R);
    }
}

// ---------------------------------------------------------------- small grids: G segments per sweep
// A launch of a few hundred workgroups cannot fill the SIMDs with one-sweep-per-workgroup work,
// and lasts as long as its longest sweep.  Here a workgroup has G groups of four waves, and the
// sweep of its 128 queries is cut into G CONTIGUOUS segments of keys, one per group (group 0 the
// rightmost, with the diagonal).  Every group runs the ordinary sweep over its segment from a
// carry of 1 - nothing couples the segments but one number per query, the product of (1 - beta)
// over a whole segment - and at the end
//     O = sum_g F_g O_g,   F_g = product of the totals of the segments right of g,
// is formed through LDS, the carry-table entries that a group wrote relative to its own right
// edge are multiplied by F_g, and rem is the product of all totals.  No exchange inside the
// sweep; the groups only share the workgroup barrier that hands over the tiles.
template <int D, int G, bool kCarryOnly>
__global__ __launch_bounds__(G * kThreads) void mfma_fwd_seg_kernel(KParams p) {
    constexpr int kTile = 64 * D * 2;
    // tile(grp, buf, kv) = lds + ((grp * 2 + buf) * 2 + kv) * kTile
    __shared__ __attribute__((aligned(16))) char lds[G * 4 * kTile];
    __shared__ float totals[G][kRowBlock];

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
    const bool rows_full = q0w + 31 < job.len;      // wave-uniform
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;

    h16x8 qf[D / 16];
    load_row_frags<D>(qf, p.q, qbase, qi, job.len, lane);
    prescale_frags(qf, p.scale2);
    f32x16 oacc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) oacc[db] = f32x16{0};
    float R = 1.0f;

    const int imax = min(m0 + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    const int n_steps = kmax >= 0 ? kmax / kKeyBlock + 1 : 0;
    const int chunk = (n_steps + G - 1) / G;              // iterations of every group
    const int hi = n_steps - grp * chunk;                  // this group sweeps steps hi-1 .. low
    const int low = max(hi - chunk, 0);
    const int64_t tabq = tab_index(p, head, job, job.rb, 0) + 32 * qs + n;   // + step * kRowBlock
    char* my_tiles = lds + grp * 4 * kTile;                // + buf * 2 * kTile

    TileDma<D> kc, vc;
    kc.init(lane, qs, p.k, kbase);
    vc.init(lane, qs, p.v, vbase);
    if (hi - 1 >= low) {
        kc.issue((hi - 1) * kKeyBlock, job.len, my_tiles);
        if (!kCarryOnly) vc.issue((hi - 1) * kKeyBlock, job.len, my_tiles + kTile);
    }
    wait_global_memory();
    __syncthreads();

    // carry tables as in mfma_fwd_kernel (right half-wave -> rtab, left -> rmid, stored a step late), here
    // relative to the segment's right edge
    float* const my_tab = h ? p.rtab : p.rmid;
    float carry_out = 1.0f;
    int carry_step = -1;
    auto store_carries = [&]() {
        if (carry_step >= 0 && p.save) {
            if (rows_full) my_tab[tabq + carry_step * kRowBlock] = carry_out;
            else if (qi < job.len) my_tab[tabq + carry_step * kRowBlock] = carry_out;
        }
        carry_step = -1;
    };
    auto open_step = [&](int step, int buf, bool skip) {
        store_carries();
        if (step - 1 >= low) {
            kc.issue_full((step - 1) * kKeyBlock, my_tiles + (buf ^ 1) * 2 * kTile);
            if (!kCarryOnly) vc.issue_full((step - 1) * kKeyBlock, my_tiles + (buf ^ 1) * 2 * kTile + kTile);
        }
    };
    int it = 0, buf = 0;
    bool redo = false;
    for (; it < chunk; ++it, buf ^= 1) {
        const int step = hi - 1 - it;
        const char* ktile = my_tiles + buf * 2 * kTile;
        const int key0 = step * kKeyBlock;
        const bool skip = step < low || key0 + strict > q0w + 31;
        open_step(step, buf, skip);
        if (!skip) {
            if (!fwd_step<D, kCarryOnly, true, true>(ktile, ktile + kTile, lo, qf, oacc, R, lane, key0, q0w, qi, strict, carry_out)) {
                redo = true;
                break;
            }
            carry_step = step;
        }
        wait_global_memory();
        __syncthreads();
    }
    for (; it < chunk; ++it, buf ^= 1) {       // reciprocal-per-key chain from the refused step on
        const int step = hi - 1 - it;
        const char* ktile = my_tiles + buf * 2 * kTile;
        const int key0 = step * kKeyBlock;
        const bool skip = step < low || key0 + strict > q0w + 31;
        if (!redo) open_step(step, buf, skip);
        redo = false;
        if (!skip) {
            fwd_step<D, kCarryOnly, false, true>(ktile, ktile + kTile, lo, qf, oacc, R, lane, key0, q0w, qi, strict, carry_out);
            carry_step = step;
        }
        wait_global_memory();
        __syncthreads();
    }
    store_carries();
    wait_global_memory();                      // the group's last entries are in memory before they are rescaled below

    // ---- segment totals -> F (what this group's results are relative to) and rem
    if (h == 0) totals[grp][32 * qs + n] = R;
    __syncthreads();
    float F = 1.0f, all = 1.0f;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const float t = totals[g][32 * qs + n];
        if (g < grp) F *= t;
        all *= t;
    }
    // carry-table entries of this group, written relative to its own right edge: times F.  Every lane
    // rescales the entries it wrote (the half-waves have a table each); the loads go out in batches so that
    // their latencies overlap.  Its stores have completed (wait above).
    if (p.save && grp > 0 && qi < job.len) {
        for (int s0 = low; s0 < hi; s0 += 8) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (s0 + j < hi) v[j] = my_tab[tabq + (s0 + j) * kRowBlock];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (s0 + j < hi) my_tab[tabq + (s0 + j) * kRowBlock] = v[j] * F;
        }
    }
    if (kCarryOnly) return;

    // ---- O = sum_g F_g O_g: groups 1.. park their scaled accumulators in LDS (the tiles are free
    // since the last barrier of the sweep), group 0 adds them up
    float* park = (float*)lds;                              // [grp - 1][qs][db][r][lane]
    if (grp > 0) {
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                park[((((grp - 1) * 4 + qs) * (D / 32) + db) * 16 + r) * 64 + lane] = oacc[db][r] * F;
    }
    __syncthreads();
    if (grp == 0 && qi < job.len) {
#pragma unroll
        for (int g = 1; g < G; ++g)
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    oacc[db][r] += park[((((g - 1) * 4 + qs) * (D / 32) + db) * 16 + r) * 64 + lane];
        store_o_row<D>(p, job, head, qi, lane, oacc);
        if (h == 0)
            Elem16::store(p.rem.ptr, (int64_t)job.seq * p.rem.sb + (int64_t)head * p.rem.sh + job.tok0 + qi, all);
    }
}

}  // inline namespace SBA_ELEM_NS
}  // namespace sba

// Key segments per sweep for the forward: 4 or 2 (head_dim 128: 2), or 0 = one sweep per workgroup.
//
// What decides is how long the launch's longest sweep is against the work of an average workgroup slot, the tail
// ratio r of sba_tail_ratio().  Two segments halve the longest sweep at 8 waves per workgroup (two workgroups per CU),
// four quarter it at 16 waves (one workgroup per CU: worth it only while the grid is at most two rounds of them).
// Measured on MI355X, forward time in us, one sweep / two segments / four segments:
//     B=1 H=16 T=3584 (r 4.4)   64.8 / 55.8 / 51.1      B=2 H=16 T=2304 (r 3.4)   47.7 / 42.6 / 52.4
//     B=1 H=16 T=4096 (r 3.9)   74.5 / 63.9 / 60.4      B=4 H=16 T=1024 (r 3.6, 512 workgroups)  26.2 / 26.1 / 29.7
//     B=1 H=16 T=4224 (r 3.8)   76.5 / 66.9 / 69.6      B=8 H=16 T=512  (r 3.2, 512 workgroups)  18.5 / 18.8 / 24.9
//     B=1 H=16 T=5120 (r 3.1)   95.7 / 82.8 / 93.3      B=1 H=32 T=4096 (r 1.9)   96.8 / 96.6 / 112.8
//     B=1 H=16 T=6144 (r 2.6)  115.8 / 110.0 / 120.0    B=2 H=16 T=4096 (r 1.9)   98.4 / 97.3 / 112.7
//     B=1 H=16 T=8192 (r 2.0)  179.8 / 170.9 / 181.9    B=5 H=16 T=2048 (r 1.5)   65.4 / 70.8 / -
//     B=1 H=16 T=10240 (r 1.6) 253.7 / 248.6 / -        B=3 H=16 T=4096 (r 1.3)  127.6 / 132.5 / -
//     packs of log-normal documents, H=16 (tokens, longest document, r): one sweep / two segments
//         8192, 2802, r 3.2   57.7 / 51.2 (four: 69.8)     8192, 4096, r 2.8   81.5 / 72.3     4096, 1393, r 4.7   31.0 / 28.0
//         6000, 1162, r 3.3   30.5 / 31.5                  10000, 2243, r 2.4  51.1 / 56.0     12288, 2069, r 1.9  56.4 / 64.7
// Two segments pay from r = 1.7 on for dense batches but lose 10-16 % on packs (one long document among many short
// ones) up to r = 2.4: the rule takes them from 2.7 on.
// SBA_FWD_GROUPS=2|3|4 forces the number of segments where the rule picks any; SBA_TWO_STEP_MAX_GRID=n replaces
// the rule by "segments (4, or as forced) up to n workgroups".
static int forward_segments(const sba::KParams& kp, unsigned grid) {
    if (kp.head_dim == 256) return 0;      // two K / V tile pairs are 128 KB of LDS: one group of waves per workgroup
    if (kp.head_dim == 128) {
        // head_dim 128: the one-sweep kernel holds two workgroups per CU, the two-segment one (8 waves, 129 KB of
        // LDS) one; it pays while the grid is at most two rounds of those and the longest sweep dominates.  B=1,
        // H=16, one sweep / two segments in us: T=1024 29.8 / 26.2, T=2048 50.4 / 41.6, T=3072 77.2 / 60.0, T=4096
        // 105.5 / 91.8, T=5120 131.1 / 138.7, T=8192 276.2 / 291.7; B=2 T=2048 60.0 / 57.0; H=8 T=4096 89.7 / 70.8.
        if (sba_two_step_env() >= 0) return grid <= (unsigned)sba_two_step_env() ? 2 : 0;
        return grid <= 2u * (unsigned)sba_cu_count() && sba_tail_ratio(kp, grid) >= 3.7 ? 2 : 0;
    }
    const char* e = getenv("SBA_FWD_GROUPS");
    const int forced = e ? atoi(e) : 0;
    const bool force = forced == 2 || forced == 3 || forced == 4;
    if (sba_two_step_env() >= 0) return grid <= (unsigned)sba_two_step_env() ? (force ? forced : 4) : 0;
    const double r = sba_tail_ratio(kp, grid);
    const int segments = (r >= 3.8 && grid <= 2u * (unsigned)sba_cu_count()) ? 4 : (r >= 2.7 ? 2 : 0);
    return segments && force ? forced : segments;
}

template <bool kCarryOnly>
static void launch_seg(int groups, dim3 grid, hipStream_t s, const sba::KParams& kp) {
    using namespace sba;
    if (kp.head_dim == 128) hipLaunchKernelGGL((mfma_fwd_seg_kernel<128, 2, kCarryOnly>), grid, dim3(2 * kThreads), 0, s, kp);
    else if (groups == 2) hipLaunchKernelGGL((mfma_fwd_seg_kernel<64, 2, kCarryOnly>), grid, dim3(2 * kThreads), 0, s, kp);
    else if (groups == 3) hipLaunchKernelGGL((mfma_fwd_seg_kernel<64, 3, kCarryOnly>), grid, dim3(3 * kThreads), 0, s, kp);
    else hipLaunchKernelGGL((mfma_fwd_seg_kernel<64, 4, kCarryOnly>), grid, dim3(4 * kThreads), 0, s, kp);
}

#ifdef SBA_ELEM_F16
int sba_launch_mfma_f16_fwd(const sba::KParams& kp, hipStream_t s) {
#else
int sba_launch_mfma_fwd(const sba::KParams& kp, hipStream_t s) {
#endif
    using namespace sba;
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    const int segments = forward_segments(kp, grid.x);
    if (segments) {
        if (kp.carry_only) launch_seg<true>(segments, grid, s, kp);
        else launch_seg<false>(segments, grid, s, kp);
    } else if (kp.head_dim == 64) {
        if (kp.carry_only) hipLaunchKernelGGL((mfma_fwd_kernel<64, true>), grid, dim3(kThreads), 0, s, kp);
        else hipLaunchKernelGGL((mfma_fwd_kernel<64, false>), grid, dim3(kThreads), 0, s, kp);
    } else if (kp.head_dim == 128) {
        if (kp.carry_only) hipLaunchKernelGGL((mfma_fwd_kernel<128, true>), grid, dim3(kThreads), 0, s, kp);
        else hipLaunchKernelGGL((mfma_fwd_kernel<128, false>), grid, dim3(kThreads), 0, s, kp);
    } else {
        if (kp.carry_only) hipLaunchKernelGGL((mfma_fwd_kernel<256, true>), grid, dim3(kThreads), 0, s, kp);
        else hipLaunchKernelGGL((mfma_fwd_kernel<256, false>), grid, dim3(kThreads), 0, s, kp);
    }
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}
