// bf16 MFMA backward kernels (head_dim 64 / 128 / 256): two passes, no atomics, deterministic.
//
// The reference (`_backward_one_row`, sb_varlen/sb_varlen_bwd.py:274-456) owns a query
// row-block, keeps dq in registers and adds every dk/dv tile into global memory under a
// spin lock (`locked_add`, :13-52).  Here the two reductions are separated instead:
//
//   pass 1  (row owner, like the forward): recomputes the weights of each 64-key step from
//           the forward's carry table, forms dz, accumulates dQ in registers, and records
//           for every (query, key block) the prefix  sum_{j left of the block} g_ij  in a
//           second table.  g_ij = a_ij * (dO_i . v_j) here: the gradient of rem enters as the
//           constant d_rem_i * rem_i that every prefix of row i starts from, which is all it
//           contributes to dz (sum_j a_ij + rem_i = 1), so pass 2 never reads d_rem.
//   pass 2  (key owner): the owner of a block of keys sweeps the query blocks at or below the
//           diagonal, recomputes weights and dz of its tiles from the tables, transposes them
//           through LDS and accumulates dK = dZ^T Q and dV = P^T dO in registers.  Four
//           kernels, chosen by grid size and head_dim: every wave owning 32 keys outright
//           (d = 64, large grids), two waves sharing 32 keys (d = 128, large grids), a resident
//           producer/consumer stream over 64-key items (d = 64, small grids), one workgroup
//           per 64-key block (d = 128, small grids).  d = 256: every wave on its own 32 keys, two
//           workgroups per key block that each take half of the columns of dK and dV.
//
// Every element of the score matrix is therefore evaluated twice in the backward (once per
// pass); in exchange nothing is reduced through memory.
#include <string.h>
#include <atomic>
#include <type_traits>
#include "sba_mfma.h"

namespace sba {
inline namespace SBA_ELEM_NS {

// The dQ pass leaves its pre-scaled Q fragments (q times scale * log2 e, rounded to bf16: the operand every
// row-owner kernel multiplies with) behind for the key-owner stream kernel, which then needs no scaling of its
// own and sees bit for bit the logits that the forward's carries were made from.  Row qi of q_scaled gets this
// lane's four 16-byte chunks (columns 16 ks + 8 h ..).  head_dim 64 only, and only where the launcher asks for it.
template <int D>
__device__ inline void store_scaled_q(const KParams& p, const Job& job, int head, int qi, int lane,
                                      const h16x8 (&qf)[D / 16]) {
    if (D != 64 || !p.q_scaled.ptr || qi >= job.len) return;
    char* row = p.q_scaled.ptr + 2 * ((int64_t)job.seq * p.q_scaled.sb + (int64_t)head * p.q_scaled.sh +
                                      (int64_t)(job.tok0 + qi) * p.q_scaled.st + 8 * (lane >> 5));
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) *(u32x4*)(row + 32 * ks) = __builtin_bit_cast(u32x4, qf[ks]);
}

// ---------------------------------------------------------------- pass 1: dQ + prefix table
// kLean (head_dim 64): the register-lean arrangement of the step that head_dim 128 always uses, held to three waves
// per SIMD.  Ahead on large launches, whose SIMDs it fills better (the packed benchmark's dQ -5.6 %, short documents
// -6 %); on launches that last as long as their longest sweep the plain arrangement's shorter step is ahead.
template <int D, bool kLean = false>
__global__ __launch_bounds__(kThreads, (D == 64 && kLean) ? 3 : (D <= 128 ? 2 : 1)) void mfma_bwd_dq_kernel(KParams p) {
    constexpr int kTile = 64 * D * 2;
    __shared__ __attribute__((aligned(16))) char lds[4 * kTile];   // K0 V0 K1 V1

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform, keep it scalar
    const int n = lane & 31, h = lane >> 5;
    LaneOffsets<D> lo;
    lo.init(lane);
    lo.rebase(lds);                        // absolute addresses: the loop below runs in one copy per tile buffer
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_job(p, order_job(blockIdx.x / p.n_heads, p.n_jobs, false));
    const int strict = p.attend_current ? 0 : 1;
    const int m0 = job.rb * kRowBlock;
    const int q0w = m0 + 32 * wave;
    const int qi = q0w + n;
    const bool row_ok = qi < job.len;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;

    if (blockIdx.x == 0 && threadIdx.x == 0 && p.gave_up) *p.gave_up = 0;     // error word of the launch pair, see wait_for_count()
    h16x8 qf[D / 16], dof[D / 16];
    load_row_frags<D>(qf, p.q, qbase, qi, job.len, lane);
    prescale_frags(qf, p.scale2);          // the score MFMAs then deliver base-2 logits
    load_row_frags<D>(dof, p.d_o, dobase, qi, job.len, lane);

    f32x16 dqacc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) dqacc[db] = f32x16{0};
    float Gc = 0.f;

    const int imax = min(m0 + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    const int n_steps = kmax >= 0 ? kmax / kKeyBlock + 1 : 0;

    TileDma<D, false, D == 64 && kLean> kc, vc;
    kc.init(lane, wave, p.k, kbase);
    vc.init(lane, wave, p.v, vbase);
    if (n_steps > 0) {
        kc.issue(0, job.len, lds);
        vc.issue(0, job.len, lds + kTile);
    }

    // carry-table traffic is kept off the critical path: the value of the NEXT step is loaded
    // while this one is computed, and this step's prefix is stored before the tile loads are
    // issued (vector memory operations retire in order)
    // Per lane ONE cursor into the tables: the entry of (this query, the step at hand) in the table of the forward
    // that holds the carry entering this LANE's 32 keys (right half-wave: rtab, left: rmid).  The prefix entering
    // the same 32 keys goes to the same entry of gmid / gtab, which lies the same distance from the cursor for
    // both half-waves (gmid - rtab == gtab - rmid: the library lays the tables out that way).
    constexpr int64_t tstride = kRowBlock;
    const float* rcur = (h ? p.rtab : p.rmid) + tab_index(p, head, job, job.rb, 0) + 32 * wave + n;
    const int64_t g_from_r = (const char*)p.gtab - (const char*)p.rmid;
    float Rnext = (row_ok && n_steps > 0) ? *rcur : 1.0f;
    float Gstore = 0.f;
    bool g_pending = false;
    // (last of the prologue's loads: its conversion waits for it, and with it for everything requested before)
    float dr = 0.f;
    if (row_ok && p.d_rem.ptr)
        dr = Elem16::load(p.d_rem.ptr, (int64_t)job.seq * p.d_rem.sb + (int64_t)head * p.d_rem.sh + job.tok0 + qi);
    wait_global_memory();
    __syncthreads();
    // (behind the prologue's loads: a store in front of them would keep the compiler from issuing them together,
    // and the wait above would fall on it; here it retires under the first step)
    store_scaled_q<D>(p, job, head, qi, lane, qf);
    auto do_step = [&](int step, auto buf_c) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        constexpr TileAt ktile = {buf * 2 * kTile};
        constexpr TileAt vtile = {buf * 2 * kTile + kTile};
        const bool more = step + 1 < n_steps;
        const int key0 = step * kKeyBlock;
        const bool skip = key0 + strict > q0w + 31 || q0w >= job.len;     // nothing visible, or no query of this wave inside the sequence
        // the prefixes that entered the previous step (the first block's are only known once that
        // block's weights are: they start at d_rem * rem, see below)
        if (g_pending && row_ok) *(float*)((char*)(rcur - tstride) + g_from_r) = Gstore;
        g_pending = false;
        const float F = Rnext;
        if (more) {
            if (row_ok) Rnext = rcur[tstride];
            // next tiles, straight into the other buffer (free since the last barrier)
            kc.issue((step + 1) * kKeyBlock, job.len, lds + (buf ^ 1) * 2 * kTile);
            vc.issue((step + 1) * kKeyBlock, job.len, lds + (buf ^ 1) * 2 * kTile + kTile);
        }
        if (!skip) {
            h16x8 zf[4];
            if constexpr (D == 128 || kLean) {
                // Register-lean arrangement (two arrays of 32 live instead of four: two waves per SIMD
                // instead of one): scores and dP first, then the chain over both in place.
                float x[32], dp[32];
                score_tiles_ps<D>(x, ktile, lo, qf);
                dp_tiles_o<D>(dp, vtile, lo, dof);
                if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
                float gsum;
                const float Lend = carried_beta_g(x, dp, F, gsum);
                if (step == 0) {                         // the gradient of rem rides in the prefix, see below
                    float Llo, Lup;
                    half_values(Lend, Llo, Lup);
                    Gc = dr * Llo;                       // what leaves the left half of the leftmost block is rem
                }
                float clo, cup;
                half_values(gsum, clo, cup);
                const float Glane = h ? Gc + clo : Gc;   // the prefix entering this lane's 32 keys: block edge (left half-wave) or middle
                Gc = Gc + clo + cup;
                Gstore = Glane;
                g_pending = true;
                walk_logit_grads_g(x, dp, Glane, zf);
            } else {
                float x[32], beta[32], dp[32];
                float Glane;
                score_tiles_ps<D>(x, ktile, lo, qf);
                if (key0 + 63 + strict > q0w) {
    mask_step(x, key0 + 32 * h, qi, strict);
                }
                // dP does not depend on the weights: its MFMAs go between the segments of the chain,
                // where the chain's exp/rcp overlap them
                const float Lend = carried_weights_and_dp<D>(x, beta, dp, F, vtile, lo, dof);
                // The gradient of rem rides in the prefix: g is formed from the plain dP, and the term
                // -beta_ik * d_rem_i * rem_i that d_rem adds to dz_ik is a constant d_rem_i * rem_i in
                // the running prefix.  What leaves the left half of the leftmost block is the product over
                // all keys, rem_i.
                if (step == 0) {
                    float Llo, Lup;
                    half_values(Lend, Llo, Lup);
                    Gc = dr * Llo;
                }
                logit_grads<false>(x, beta, dp, Gc, lane, &Glane);
                // the prefix entering this lane's 32 keys - the block's edge for the left half-wave, its middle
                // (for the key-owner pass whose waves own 32 keys) for the right one -, stored at the top of the
                // next iteration
                Gstore = Glane;
                g_pending = true;
#pragma unroll
                for (int c = 0; c < 4; ++c) zf[c] = pack8(&dp[8 * c]);
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {      // (operands of a key group requested together, see score_raw_o)
                h16x8 kt[D / 32];
#pragma unroll
                for (int db = 0; db < D / 32; ++db) kt[db] = fetch_cols_o<D>(ktile, lo, db, c);
                if (D == 128) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int db = 0; db < D / 32; ++db) dqacc[db] = mfma(kt[db], zf[c], dqacc[db]);
            }
        }
        rcur += tstride;
        wait_global_memory();                  // the next tiles have landed
        __syncthreads();
    };
    for (int step = 0; step < n_steps; step += 2) {
        do_step(step, std::integral_constant<int, 0>{});
        if (step + 1 < n_steps) do_step(step + 1, std::integral_constant<int, 1>{});
    }
    if (g_pending && row_ok) *(float*)((char*)(rcur - tstride) + g_from_r) = Gstore;

    if (row_ok) {
        const int64_t ob = (int64_t)job.seq * p.dq.sb + (int64_t)head * p.dq.sh + (int64_t)(job.tok0 + qi) * p.dq.st;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x2 a = {dqacc[db][4 * g] * p.scale, dqacc[db][4 * g + 1] * p.scale};
                f32x2 b = {dqacc[db][4 * g + 2] * p.scale, dqacc[db][4 * g + 3] * p.scale};
                h16x2 pa = __builtin_convertvector(a, h16x2), pb = __builtin_convertvector(b, h16x2);
                uint2 w;
                w.x = __builtin_bit_cast(uint32_t, pa);
                w.y = __builtin_bit_cast(uint32_t, pb);
                *(uint2*)(p.dq.ptr + 2 * (ob + 32 * db + 8 * g + 4 * h)) = w;
            }
    }
}

// ---------------------------------------------------------------- pass 1, two steps per iteration
// Same sweep with 8 waves: wave-group 0 (waves 0-3) and wave-group 1 (waves 4-7) take two
// CONSECUTIVE 64-key steps of the same 128 queries in every iteration (group 1 the right one).
// All the heavy work of a step (scores, weights, dP, g = a*dP and its prefix sums inside the
// step) only needs the step's own keys and the forward's carry table; what couples neighbouring
// steps is one number per query, the sum of g over the step.  The groups swap those totals
// through LDS at a barrier, the right group adds the left group's total to its prefix, and each
// group accumulates its own partial dQ, summed once at the end.  The longest dependent chain
// of a launch (the sweep of the last row-block) is halved, which is what bounds the time when
// the whole problem is only two waves per SIMD.
template <int D>
__global__ __launch_bounds__(2 * kThreads, 2) void mfma_bwd_dq2_kernel(KParams p) {
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
    const bool row_ok = qi < job.len;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;

    if (blockIdx.x == 0 && threadIdx.x == 0 && p.gave_up) *p.gave_up = 0;     // error word of the launch pair, see wait_for_count()
    h16x8 qf[D / 16], dof[D / 16];
    load_row_frags<D>(qf, p.q, qbase, qi, job.len, lane);
    prescale_frags(qf, p.scale2);          // the score MFMAs then deliver base-2 logits
    load_row_frags<D>(dof, p.d_o, dobase, qi, job.len, lane);

    f32x16 dqacc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) dqacc[db] = f32x16{0};
    float Gc = 0.f;

    const int imax = min(m0 + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    const int n_steps = kmax >= 0 ? kmax / kKeyBlock + 1 : 0;
    const int n_it = (n_steps + 1) / 2;
    char* my_tiles = lds + grp * 2 * kTile;          // + buf * 4 * kTile

    // each group copies its own tiles (256 threads per tile pair)
    TileDma<D> kc, vc;
    kc.init(lane, qs, p.k, kbase);
    vc.init(lane, qs, p.v, vbase);
    if (grp < n_steps) {
        kc.issue(grp * kKeyBlock, job.len, my_tiles);
        vc.issue(grp * kKeyBlock, job.len, my_tiles + kTile);
    }

    // the forward's carry for this group's NEXT step is loaded while this one is computed
    constexpr int64_t tstride = kRowBlock;
    // this lane's cursor into the carry tables and the distance to its prefix entry, see the one-step kernel
    const float* rcur = (h ? p.rtab : p.rmid) + tab_index(p, head, job, job.rb, 0) + 32 * qs + n + grp * tstride;
    const int64_t g_from_r = (const char*)p.gtab - (const char*)p.rmid;
    float Rnext = (row_ok && grp < n_steps) ? *rcur : 1.0f;
    float Gstore = 0.f;
    bool g_pending = false;
    // (last of the prologue's loads: its conversion waits for it, and with it for everything requested before)
    float dr = 0.f;
    if (row_ok && p.d_rem.ptr)
        dr = Elem16::load(p.d_rem.ptr, (int64_t)job.seq * p.d_rem.sb + (int64_t)head * p.d_rem.sh + job.tok0 + qi);
    wait_global_memory();
    __syncthreads();
    if (grp == 0) store_scaled_q<D>(p, job, head, qi, lane, qf);      // (placed as in the one-step kernel)
    // Every LDS address of the loop is a sweep-constant register plus an immediate: the lane offsets are made absolute
    // for this group's tiles once, and the loop runs in one copy per tile buffer (see the one-step kernel).
    lo.rebase(my_tiles);
    auto do_iteration = [&](int it, auto buf_c) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        constexpr TileAt ktile = {buf * 4 * kTile};
        constexpr TileAt vtile = {buf * 4 * kTile + kTile};
        const int step = 2 * it + grp;                   // == n_steps: this group idles in the last iteration
        const bool more = step + 2 < n_steps;
        const int key0 = step * kKeyBlock;
        const bool active = step < n_steps && !(key0 + strict > q0w + 31) && q0w < job.len;
        if (g_pending && row_ok) *(float*)((char*)(rcur - 2 * tstride) + g_from_r) = Gstore;
        g_pending = false;
        const float F = Rnext;
        if (more) {
            if (row_ok) Rnext = rcur[2 * tstride];
            // next tiles, straight into the other buffer (free since the last barrier)
            kc.issue((step + 2) * kKeyBlock, job.len, my_tiles + (buf ^ 1) * 4 * kTile);
            vc.issue((step + 2) * kKeyBlock, job.len, my_tiles + (buf ^ 1) * 4 * kTile + kTile);
        }
        // (an active wave's whole step sits in one branch, exchange barrier included: were the step split around the
        // barrier, its 64 weights and gradients would have to hold a value on the idle path too, and the compiler
        // clears half of them at the top of every step)
        if (active) {
            float x[32], beta[32], dp[32];
            float total = 0.f;
            score_tiles_ps<D, true>(x, ktile, lo, qf);
            if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
            const float Lend = carried_weights_and_dp<D, true>(x, beta, dp, F, vtile, lo, dof);
            float start = logit_grads_local(x, dp, total, lane);
            // the gradient of rem rides in the prefix as the constant d_rem * rem (see the one-step
            // kernel).  The leftmost block is group 0's first step: the constant joins its total
            // (which carries it to the other group and into Gc) and its own prefix
            if (step == 0) {
                float Llo, Lup;
                half_values(Lend, Llo, Lup);
                const float c0 = dr * Llo;
                total += c0;
                start += c0;
            }
            if (h == 0) xch[grp][32 * qs + n] = total;
            __syncthreads();
            const float other = xch[grp ^ 1][32 * qs + n];
            // group 1 holds the right step of the pair: its prefix also contains group 0's total
            const float Gmy = grp == 0 ? Gc : Gc + other;
            Gc = Gc + total + other;
            const float Glane = Gmy + start;       // the prefix entering this lane's 32 keys: block edge or middle (see the one-step kernel)
            Gstore = Glane;
            g_pending = true;
            logit_grads_apply(beta, dp, Glane);
            h16x8 zf[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) zf[c] = pack8(&dp[8 * c]);
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    dqacc[db] = mfma(fetch_cols_o<D>(ktile, lo, db, c), zf[c], dqacc[db]);
        } else {
            if (h == 0) xch[grp][32 * qs + n] = 0.f;
            __syncthreads();
            Gc = Gc + xch[grp ^ 1][32 * qs + n];
        }
        rcur += 2 * tstride;
        wait_global_memory();                  // the next tiles have landed
        __syncthreads();
    };
    for (int it = 0; it < n_it; it += 2) {
        do_iteration(it, std::integral_constant<int, 0>{});
        if (it + 1 < n_it) do_iteration(it + 1, std::integral_constant<int, 1>{});
    }

    if (g_pending && row_ok) *(float*)((char*)(rcur - 2 * tstride) + g_from_r) = Gstore;

    // ---- dQ = dQ(group 0) + dQ(group 1): group 1 parks its accumulators in LDS
    float* park = (float*)lds;                              // [qs][db][r][lane]
    if (grp == 1) {
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) park[((qs * (D / 32) + db) * 16 + r) * 64 + lane] = dqacc[db][r];
    }
    __syncthreads();
    if (grp == 0 && row_ok) {
        const int64_t ob = (int64_t)job.seq * p.dq.sb + (int64_t)head * p.dq.sh + (int64_t)(job.tok0 + qi) * p.dq.st;
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
#pragma unroll
            for (int r = 0; r < 16; ++r) dqacc[db][r] += park[((qs * (D / 32) + db) * 16 + r) * 64 + lane];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x2 a = {dqacc[db][4 * g] * p.scale, dqacc[db][4 * g + 1] * p.scale};
                f32x2 b = {dqacc[db][4 * g + 2] * p.scale, dqacc[db][4 * g + 3] * p.scale};
                h16x2 pa = __builtin_convertvector(a, h16x2), pb = __builtin_convertvector(b, h16x2);
                uint2 w;
                w.x = __builtin_bit_cast(uint32_t, pa);
                w.y = __builtin_bit_cast(uint32_t, pb);
                *(uint2*)(p.dq.ptr + 2 * (ob + 32 * db + 8 * g + 4 * h)) = w;
            }
        }
    }
}

// ---------------------------------------------------------------- pass 2: dK, dV
// One workgroup per 64-key block; a step covers 128 queries (32 per wave).  Each wave
// turns its 32 queries into weights (a, dz), writes them as bf16 [query][key] rows into a
// tile shared by the workgroup, and after a barrier reduces ONE [32 keys x 32 d] tile of
// dK and of dV over all 128 queries, so its accumulators are 2 x 16 x D/64 registers and
// two workgroups fit on a CU.  Every Q / dO row is fetched from global memory once, as the
// per-lane row fragments that the score / dP MFMAs need (Q a step ahead, dO at the top of
// the step, hidden behind the weights); the same registers are then stored into the shared
// Q and dO tiles that the reduction reads transposed.  Per-query scalars (carry tables,
// drem) are prefetched one step ahead.
template <int D>
__global__ __launch_bounds__(kThreads, 2) void mfma_bwd_dkv_kernel(KParams p) {
    constexpr int kTile = 64 * D * 2;          // K or V tile (64 keys)
    constexpr int kQTile = 128 * D * 2;        // Q or dO tile (128 queries)
    constexpr int kZTile = 128 * 64 * 2;       // weights of one step, [query][key] bf16
    // the tiles read with the transposing fetch come first so that their offsets fit the
    // 16-bit immediate of the LDS instructions
    __shared__ __attribute__((aligned(1024))) char lds[2 * kTile + 2 * kQTile + 2 * kZTile];
    char* zp = lds;
    char* zd = zp + kZTile;
    char* qtile = zd + kZTile;
    char* dotile = qtile + kQTile;
    char* ktile = dotile + kQTile;
    char* vtile = ktile + kTile;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 31, h = lane >> 5;
    LaneOffsets<D> lo;
    lo.init(lane);
    LaneOffsets<64> lz;                        // the weight tiles have 64-key rows whatever D is
    lz.init(lane);
    const int head = blockIdx.x % p.n_heads;
    const int slot = blockIdx.x / p.n_heads;   // two 64-key blocks per scheduled 128-row job
    const Job job = decode_key_job(p, slot >> 1);
    const int kb = 2 * job.rb + (slot & 1);
    const int key0 = kb * kKeyBlock;
    if (key0 >= job.len) return;               // uniform over the workgroup
    const int strict = p.attend_current ? 0 : 1;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;
    const int n_qb = (job.len + kRowBlock - 1) / kRowBlock;
    const int kh = wave & 1;                   // which 32 keys this wave reduces
    const int dbw = wave >> 1;                 // and which d-blocks: dbw + 2*i
    // lane offsets of this wave's operand columns, picked once (no run-time table indexing)
    const int za0 = pick_nat<64>(lz, 0, kh), za1 = pick_nat<64>(lz, 1, kh);
    int qb0o[D / 64], qb1o[D / 64];
#pragma unroll
    for (int i = 0; i < D / 64; ++i) { qb0o[i] = pick_nat<D>(lo, 0, dbw + 2 * i); qb1o[i] = pick_nat<D>(lo, 1, dbw + 2 * i); }

    {
        TileCopy<D> kc, vc;
        kc.load(p.k, kbase, key0, job.len);
        vc.load(p.v, vbase, key0, job.len);
        kc.scale(p.scale2);                    // K times the logit scale: the score MFMAs deliver base-2 logits
        kc.store(ktile);
        vc.store(vtile);
    }
    f32x16 dkacc[D / 64], dvacc[D / 64];
#pragma unroll
    for (int i = 0; i < D / 64; ++i) { dkacc[i] = f32x16{0}; dvacc[i] = f32x16{0}; }

    const int qb0 = job.rb;
    // prefetched state of the first step
    float Rn = 1.0f, Gn = 0.0f;
    h16x8 qfn[D / 16];
    {
        const int qi0 = qb0 * kRowBlock + 32 * wave + n;
        load_row_frags<D>(qfn, p.q, qbase, qi0, job.len, lane);
        if (qi0 < job.len) {
            const int64_t t = tab_index(p, head, job, qb0, kb) + 32 * wave + n;
            Rn = p.rtab[t]; Gn = p.gtab[t];
        }
    }
    __syncthreads();                           // K, V tiles visible

    wait_global_memory();
    for (int qb = qb0; qb < n_qb; ++qb) {
        const int m0 = qb * kRowBlock;
        const int q0w = m0 + 32 * wave;
        const int qi = q0w + n;
        // (1) this lane's Q row fragments were prefetched during the previous step; its dO
        //     fragments are requested now and not needed before the weights are done.  Each
        //     row is fetched from global memory exactly once: the fragments are also what the
        //     shared Q / dO tiles of the reduction are assembled from.
        h16x8 qf[D / 16], dof[D / 16];
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) qf[ks] = qfn[ks];
        load_row_frags<D>(dof, p.d_o, dobase, qi, job.len, lane);
        float R = Rn, Gc = Gn;
        if (qb + 1 < n_qb) {
            const int qin = qi + kRowBlock;
            load_row_frags<D>(qfn, p.q, qbase, qin, job.len, lane);
            Rn = 1.0f; Gn = 0.0f;
            if (qin < job.len) {
                const int64_t t = tab_index(p, head, job, qb + 1, kb) + 32 * wave + n;
                Rn = p.rtab[t]; Gn = p.gtab[t];
            }
        }
        // (2) row 32*wave + n of the shared Q tile (every wave passed the barrier that ends the
        //     previous step's reduction, so the tiles are free)
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks)
            *(h16x8*)(qtile + tile_offset<D>(32 * wave + n, 2 * ks + h)) = qf[ks];
        // (3) weights of this wave's 32 queries
        float x[32], dp[32];
        const bool skip = key0 + strict > q0w + 31 || q0w >= job.len;
        if (!skip) {
            float beta[32];
            score_tiles_ps<D>(x, ktile, lo, qf);
            if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
            stick_weights<true>(x, beta, R, lane);
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks)
                *(h16x8*)(dotile + tile_offset<D>(32 * wave + n, 2 * ks + h)) = dof[ks];
            dp_tiles_o<D>(dp, vtile, lo, dof);
            logit_grads<true>(x, beta, dp, Gc, lane);
        } else {
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks)
                *(h16x8*)(dotile + tile_offset<D>(32 * wave + n, 2 * ks + h)) = dof[ks];
#pragma unroll
            for (int idx = 0; idx < 32; ++idx) { x[idx] = 0.f; dp[idx] = 0.f; }
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            *(h16x8*)(zp + tile_offset<64>(32 * wave + n, 4 * h + c)) = pack8(&x[8 * c]);
            *(h16x8*)(zd + tile_offset<64>(32 * wave + n, 4 * h + c)) = pack8(&dp[8 * c]);
        }
        __syncthreads();                       // weights and tiles of all waves visible
        // (4) dK[key][d] += sum_q dz[q][key] Q[q][d];  dV[key][d] += sum_q a[q][key] dO[q][d]
#pragma unroll
        for (int c2 = 0; c2 < 8; ++c2) {
            h16x8 az = fetch_nat_2<64>(zd, za0, za1, 16 * c2);
            h16x8 ap = fetch_nat_2<64>(zp, za0, za1, 16 * c2);
#pragma unroll
            for (int i = 0; i < D / 64; ++i) {
                dkacc[i] = mfma(az, fetch_nat_2<D>(qtile, qb0o[i], qb1o[i], 16 * c2), dkacc[i]);
                dvacc[i] = mfma(ap, fetch_nat_2<D>(dotile, qb0o[i], qb1o[i], 16 * c2), dvacc[i]);
            }
        }
        wait_global_memory();                  // nothing in flight across the back edge
        __syncthreads();                       // reduction done: tiles may be overwritten
    }
    // accumulator rows are keys 32*kh + ..., columns d = 32*(dbw + 2*i) + n (the weight tiles
    // are in natural key order); the last barrier of the loop has freed the weight tiles
    char* stage_k = zp;                        // [64 keys][D] bf16 each: kZTile >= kTile
    char* stage_v = zd;
#pragma unroll
    for (int i = 0; i < D / 64; ++i) {
        stage_acc_tile<D>(stage_k, 32 * kh, 32 * (dbw + 2 * i), dkacc[i], p.scale, lane);
        stage_acc_tile<D>(stage_v, 32 * kh, 32 * (dbw + 2 * i), dvacc[i], 1.0f, lane);
    }
    __syncthreads();
    const int64_t dkbase = (int64_t)job.seq * p.dk.sb + (int64_t)head * p.dk.sh + (int64_t)job.tok0 * p.dk.st;
    const int64_t dvbase = (int64_t)job.seq * p.dv.sb + (int64_t)head * p.dv.sh + (int64_t)job.tok0 * p.dv.st;
    store_staged_rows<D>(stage_k, p.dk, dkbase, key0, job.len, threadIdx.x, kThreads);
    store_staged_rows<D>(stage_v, p.dv, dvbase, key0, job.len, threadIdx.x, kThreads);
}

// ---------------------------------------------------------------- pass 2, head_dim 64
// dK/dV as ONE resident workgroup per CU that runs its share of the (key block, head) items
// back to back as a single stream of 128-query steps, with the two halves of a step given to
// different waves:
//   waves 0..3 ("producers") turn 32 queries x 64 keys each into weights and logit gradients
//     and leave them, as bf16 [query][key] rows, in one of two LDS buffers;
//   waves 4..7 ("consumers") reduce the buffer of the previous step into dK and dV with
//     MFMAs, and stage what the next step needs (Q / dO tiles, per-query carries, and at an
//     item boundary the next K / V tiles) from global memory into LDS with coalesced loads.
// A SIMD holds one wave of each kind, so matrix and memory work run under the producers'
// vector work, and because the stream never stops at an item boundary nothing of an item's
// set-up (launch, K/V fetch, first tiles) or tear-down (dK/dV store) is exposed.
//
// One iteration s of the stream (workgroup barrier A at its end):
//   producers:  fragments of tile[s&1] -> scores, weights, dP, dz -> Z[s&1]                    | A
//   consumers:  store a staged dK/dV; request step s+1;
//               reduce Z/tile[(s-1)&1]; [B] stage a finished dK/dV into Z[(s-1)&1];
//               deposit step s+1 -> tile[(s+1)&1]                                              | A
// A consumer wave deposits exactly the part of the tiles that its own reduction reads, so the
// refill of buffer (s+1)&1 = (s-1)&1 only has to follow that wave's own reads.  B, needed only
// where a finished dK/dV is staged into the Z buffer that all four consumers have just read, is
// a barrier of the consumer waves alone (a running count in LDS): the producers - the critical
// path - never wait in the middle of a step.  Two rarer hand-overs: a staged dK/dV occupies the Z buffer that the producers write in the next
// iteration, so that iteration has one more workgroup barrier (X) after the consumers' store;
// and the K tile is refilled only after a second LDS count says that every producer holds
// the current item's K fragments.
// An item's accumulators are complete after the reduction that follows its last step; they are
// staged after that iteration's B and written to global memory before the next iteration's B.
// The stream kernel's two internal waits are on counters in LDS that waves of the same
// (resident) workgroup bump, so they end within microseconds.  They are bounded all the same: a
// wave that has slept through kSpinLimit polls stops waiting, raises the launch's error word
// (KParams::gave_up, the last 256 bytes of the backward scratch) and runs on, so that the kernel
// always drains; its results are then meaningless.
constexpr int kSpinLimit = 1 << 22;            // polls of 64+ clocks each: more than 0.1 s
__device__ inline void wait_for_count(int* counter, int target, int* gave_up) {
    for (int i = 0; i < kSpinLimit; ++i) {
        if (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= target) return;
        __builtin_amdgcn_s_sleep(1);
    }
    if (gave_up && (threadIdx.x & 63) == 0) *gave_up = 1;
}

// Weights and logit gradients of ONE [32 keys x 32 queries] tile whose lanes hold 16 consecutive keys
// (the own-keys kernel and the eight-producer stream): the carries enter per 32 keys.
template <class Between>
__device__ inline void own_tile_weights(float (&x)[16], float (&beta)[16], float Rin, int lane, Between&& between) {
    const float L = product_chain_with<true, 16>(x, beta, between);
    float Llo, Lup;
    half_values(L, Llo, Lup);
    scale_clamped<16>(x, (lane >= 32) ? Rin : Rin * Lup);         // upper half-wave: the right 16 keys
}
__device__ inline void own_tile_grads(const float (&a)[16], const float (&beta)[16], float (&dp)[16], float Gin,
                                      int lane) {
    float c = 0.f, pre[16];
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) {
        dp[idx] = a[idx] * dp[idx];     // g
        c += dp[idx];
        pre[idx] = c;
    }
    float clo, cup;
    half_values(c, clo, cup);
    const float F = (lane >= 32) ? Gin + clo : Gin;
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) dp[idx] = __builtin_fmaf(-beta[idx], pre[idx] + F, dp[idx]);
}

struct KeyItem {
    Job job;
    int head, kb, key0, n_steps;
    bool valid;
};

__device__ inline KeyItem decode_item(const KParams& p, int idx) {
    KeyItem r;
    r.valid = idx >= 0;
    if (idx < 0) idx = 0;
    r.head = idx % p.n_heads;
    const int slot = idx / p.n_heads;          // two 64-key blocks per scheduled 128-row job
    r.job = decode_key_job(p, slot >> 1);
    r.kb = 2 * r.job.rb + (slot & 1);
    r.key0 = r.kb * kKeyBlock;
    r.n_steps = (r.job.len + kRowBlock - 1) / kRowBlock - r.job.rb;
    return r;
}

// NP = number of producer waves.  4: producer w does queries 32w.. of the step against all 64 keys
// (one wave per SIMD computes weights).  8: producer w does queries 32(w%4).. against the 32 keys
// 32(w/4).. of the block - two producers per SIMD, which is what lets a SIMD issue their vector
// instructions back to back (one wave alone issues one every 2.2-2.7 ns, two together one every
// 1.1-1.2 ns); the half blocks take the mid-block carries of the dQ pass, like the own-keys kernel.
template <int D, int NP>
__global__ __launch_bounds__((NP + 4) * 64, NP == 4 ? 2 : 3) void mfma_bwd_dkv_stream_kernel(KParams p) {
    constexpr int kTile = 64 * D * 2;          // K or V tile (64 keys)
    constexpr int kQTile = 128 * D * 2;        // Q or dO tile (128 queries)
    constexpr int kZTile = 128 * 64 * 2;       // weights of one step, [query][key] bf16
    constexpr int kBuf = 2 * kZTile + 2 * kQTile;
    constexpr int kCarry = kRowBlock * 16;      // {R, G, R mid-block, G mid-block} per query
    __shared__ __attribute__((aligned(1024))) char lds[3 * kTile + 2 * kCarry + 2 * kBuf];
    __shared__ int consumers_done;             // consumer waves that have finished a reduction, running total
    __shared__ int producers_took_k;           // producer waves that hold an item's K fragments, running total
    char* vtiles = lds;                        // V of item j in vtiles + (j&1)*kTile
    char* ktile = vtiles + 2 * kTile;          // read once per item, into the producers' registers
    char* carry = ktile + kTile;
    char* bufs = carry + 2 * kCarry;           // per buffer: zp, zd, qtile, dotile

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool producer = wave < NP;
    const int w4 = wave & 3;
    const int n = lane & 31, h = lane >> 5;
    const int strict = p.attend_current ? 0 : 1;
    const int n_items = 2 * p.n_jobs * p.n_heads;

    // Items are taken in list order (longest sweeps first).  A job's second key block can lie
    // beyond the end of its sequence: such an item runs like any other, its one step finds
    // nothing to do and nothing is stored, which is cheaper than teaching the pipeline to skip.
    const int G = gridDim.x, g = blockIdx.x;
    // items of class c = index % 8 go to the workgroups of XCD c (workgroups are dealt to the
    // XCDs round-robin): with the head count a multiple of 8 a head's K, V, Q, dO and carries
    // then stay in one XCD's L2.  Inside a class the workgroups walk the list boustrophedon,
    // which evens out the sweep lengths (the list is sorted by them).
    const int W = G >> 3, w = g >> 3, c8 = g & 7;
    auto static_item = [&](int r) { const int i = 8 * (r * W + ((r & 1) ? W - 1 - w : w)) + c8; return i < n_items ? i : -1; };
    int cur_idx = static_item(0);
    int nxt_idx = static_item(1);
    KeyItem cur = decode_item(p, cur_idx);
    if (!cur.valid) return;                    // uniform over the workgroup
    KeyItem nxt = decode_item(p, nxt_idx);
    int ring = 2;                              // round of the item after `nxt`
    if (threadIdx.x == 0) { consumers_done = 0; producers_took_k = 0; }

    if (producer) {
        LaneOffsets<D> lo;
        lo.init(lane);
        __syncthreads();                       // first item's tiles and carries visible
        int s = 0;
        bool staged_prev = false;              // the consumers staged a dK/dV in the previous iteration
        // (no logit scale here: the Q tiles hold q times scale * log2 e, see store_scaled_q)
        if constexpr (NP == 8) {
        const int kh = wave >> 2;              // this wave's half of the 64-key block
        for (int item = 0;; ++item) {
            const char* vtile = vtiles + (item & 1) * kTile;
            // rows 32kh.. of the K and V tiles are this wave's keys, in the order that puts 16
            // consecutive keys into a lane's accumulator registers (see request_keys)
            h16x8 kfr[D / 16], vfr[D / 16];
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks) {
                kfr[ks] = fetch_rows_o<D>(ktile, lo, kh, ks);
                vfr[ks] = fetch_rows_o<D>(vtile, lo, kh, ks);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            if (lane == 0) __hip_atomic_fetch_add(&producers_took_k, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            const int key0 = cur.key0 + 32 * kh;
            const int len = cur.job.len;
            for (int it = 0; it < cur.n_steps; ++it, ++s) {
                const bool x_now = staged_prev;
                staged_prev = it == 0 && item > 0;
                char* zp = bufs + (s & 1) * kBuf;
                char* zd = zp + kZTile;
                const char* qtile = zd + kZTile;
                const char* dotile = qtile + kQTile;
                const int q0w = (cur.job.rb + it) * kRowBlock + 32 * w4;
                const int qi = q0w + n;
                const bool skip = key0 + strict > q0w + 31 || q0w >= len || key0 >= len;
                // (one branch holds the whole step of a wave that has work: split in two around barrier X, the
                // weights would be values that "flow" through the idle path as well, and the compiler then keeps
                // a copy of all of them across the loop)
                if (!skip) {
                    float x[16], beta[16], dp[16];
                    const float4 cv = *(const float4*)(carry + (s & 1) * kCarry + (32 * w4 + n) * 16);
                    // table entries of pairs that no query of the row sees are not written
                    const bool sees = qi < len && qi - strict - key0 + 1 > 0;
                    const float Rt = sees ? (kh ? cv.x : cv.z) : 1.0f;
                    const float Gt = sees ? (kh ? cv.w : cv.y) : 0.0f;
                    h16x8 qf[D / 16], dof[D / 16];
#pragma unroll
                    for (int ks = 0; ks < D / 16; ++ks) {
                        qf[ks] = fetch_rows_o<D>(qtile, lo, w4, ks);
                        dof[ks] = fetch_rows_o<D>(dotile, lo, w4, ks);
                    }
                    f32x16 acc = {0};
#pragma unroll
                    for (int ks = 0; ks < D / 16; ++ks) acc = mfma(kfr[ks], qf[ks], acc);
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[r] = acc[r];
                    if (key0 + 31 + strict > q0w || q0w + 31 >= len) {        // diagonal or ragged tile
                        const int nvis = qi < len ? qi - strict - (key0 + 16 * h) + 1 : 0;
#pragma unroll
                        for (int idx = 0; idx < 16; ++idx)
                            if (idx >= nvis) x[idx] = -INFINITY;
                    }
                    // dP = dO V^T: one MFMA behind each of the chain's four segments
                    static_assert(D == 64, "one dP MFMA per chain segment");
                    f32x16 dacc;
                    own_tile_weights(x, beta, Rt, lane, [&](int seg) {
                        dacc = mfma(vfr[seg], dof[seg], seg == 0 ? f32x16{0} : dacc);
                    });
#pragma unroll
                    for (int r = 0; r < 16; ++r) dp[r] = dacc[r];
                    if (x_now) __syncthreads();    // X
                    own_tile_grads(x, beta, dp, Gt, lane);
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        *(h16x8*)(zp + tile_offset<64>(32 * w4 + n, 4 * kh + 2 * h + c)) = pack8(&x[8 * c]);
                        *(h16x8*)(zd + tile_offset<64>(32 * w4 + n, 4 * kh + 2 * h + c)) = pack8(&dp[8 * c]);
                    }
                } else {
                    if (x_now) __syncthreads();    // X
                    const h16x8 none = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        *(h16x8*)(zp + tile_offset<64>(32 * w4 + n, 4 * kh + 2 * h + c)) = none;
                        *(h16x8*)(zd + tile_offset<64>(32 * w4 + n, 4 * kh + 2 * h + c)) = none;
                    }
                }
                __syncthreads();               // A
            }
            if (!nxt.valid) break;
            cur = nxt;
            nxt = decode_item(p, static_item(ring));
            ++ring;
        }
        } else {
        for (int item = 0;; ++item) {
            const char* vtile = vtiles + (item & 1) * kTile;
            // the key block of an item never changes: its score and dP operands stay in registers
            h16x8 kfr[2][D / 16], vfr[2][D / 16];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int ks = 0; ks < D / 16; ++ks) {
                    kfr[t][ks] = fetch_rows_o<D>(ktile, lo, t, ks);
                    vfr[t][ks] = fetch_rows_o<D>(vtile, lo, t, ks);
                }

            // tell the consumers that the K tile may be refilled
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            if (lane == 0) __hip_atomic_fetch_add(&producers_took_k, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            const int key0 = cur.key0;
            const int len = cur.job.len;
            for (int it = 0; it < cur.n_steps; ++it, ++s) {
                // A dK/dV staged in the previous iteration sits in the Z buffer this iteration
                // writes: wait (barrier X) until the consumers have stored it.
                const bool x_now = staged_prev;
                staged_prev = it == 0 && item > 0;
                char* zp = bufs + (s & 1) * kBuf;
                char* zd = zp + kZTile;
                const char* qtile = zd + kZTile;
                const char* dotile = qtile + kQTile;
                const int q0w = (cur.job.rb + it) * kRowBlock + 32 * w4;
                const int qi = q0w + n;
                const bool skip = key0 + strict > q0w + 31 || q0w >= len;
                // (one branch for the whole step, see above)
                if (!skip) {
                    float x[32], beta[32], dp[32];
                    // Both carries that enter this LANE's 32 keys come from the tables: the right half-wave
                    // takes the forward's block-edge product and the mid-block prefix, the left one the
                    // mid-block product and the block-edge prefix - no exchange between the halves, and the
                    // prefix sums run in one pass.  Entries of (query, half block) pairs that the query does not
                    // see are not written: their weights are zero whatever the carry.  Rows past the end of
                    // the sequence hold copies of its last row: a zero carry makes their weights and
                    // gradients exactly zero.
                    const float4 cv = *(const float4*)(carry + (s & 1) * kCarry + (32 * w4 + n) * 16);
                    const bool sees = qi < len && qi - strict - (key0 + 32 * h) + 1 > 0;
                    const float R = sees ? (h ? cv.x : cv.z) : (qi < len ? 1.0f : 0.0f);
                    const float Gc = sees ? (h ? cv.w : cv.y) : 0.0f;
                    h16x8 qf[D / 16], dof[D / 16];
#pragma unroll
                    for (int ks = 0; ks < D / 16; ++ks) {
                        qf[ks] = fetch_rows_o<D>(qtile, lo, w4, ks);
                        dof[ks] = fetch_rows_o<D>(dotile, lo, w4, ks);
                    }
                    f32x16 raw[2];
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        f32x16 acc = {0};
#pragma unroll
                        for (int ks = 0; ks < D / 16; ++ks) acc = mfma(kfr[t][ks], qf[ks], acc);
                        raw[t] = acc;
                    }
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int r = 0; r < 16; ++r) x[16 * t + r] = raw[t][r];
                    if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
                    // dP = dO V^T does not depend on the weights: its eight MFMAs go between the
                    // segments of the chain, where the chain's exp/rcp overlap them
                    static_assert(D == 64, "one dP MFMA per chain segment");
                    f32x16 dacc[2];
                    carried_chain_with<true, 32>(x, beta, R, [&](int seg) {      // finished weights: no scaling pass
                        const int t = seg & 1, ks = seg >> 1;
                        dacc[t] = mfma(vfr[t][ks], dof[ks], ks == 0 ? f32x16{0} : dacc[t]);
                    });
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int r = 0; r < 16; ++r) dp[16 * t + r] = dacc[t][r];
                    if (x_now) __syncthreads();    // X
                    logit_grads_from<32>(x, beta, dp, Gc);
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        *(h16x8*)(zp + tile_offset<64>(32 * w4 + n, 4 * h + c)) = pack8(&x[8 * c]);
                        *(h16x8*)(zd + tile_offset<64>(32 * w4 + n, 4 * h + c)) = pack8(&dp[8 * c]);
                    }
                } else {
                    if (x_now) __syncthreads();    // X
                    const h16x8 none = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        *(h16x8*)(zp + tile_offset<64>(32 * w4 + n, 4 * h + c)) = none;
                        *(h16x8*)(zd + tile_offset<64>(32 * w4 + n, 4 * h + c)) = none;
                    }
                }
                __syncthreads();               // A
            }
            if (!nxt.valid) break;
            cur = nxt;
            nxt = decode_item(p, static_item(ring));
            ++ring;
        }
        }
        __syncthreads();                       // A of the draining iteration
    } else {
        LaneOffsets<D> lo;
        lo.init(lane);
        LaneOffsets<64> lz;                    // the weight tiles have 64-key rows whatever D is
        lz.init(lane);
        const int ct = threadIdx.x & (kThreads - 1);
        // Wave w4 reduces ONE of the two outputs (even: dK from dz and Q, odd: dV from a and dO),
        // all 64 keys of it and one 32-wide d-block: the two key halves share the Q / dO operand,
        // three operand fetches per two MFMAs instead of four.
        static_assert(D == 64, "the consumers' tiling assumes two 32-wide d-blocks");
        const bool is_dv = w4 & 1;
        const int dbw = w4 >> 1;
        int za[2][2];
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) { za[kh][0] = pick_nat<64>(lz, 0, kh); za[kh][1] = pick_nat<64>(lz, 1, kh); }
        const int qb0o = pick_nat<D>(lo, 0, dbw), qb1o = pick_nat<D>(lo, 1, dbw);
        f32x16 acc[2];                         // key halves
        acc[0] = f32x16{0}; acc[1] = f32x16{0};

        // Staging registers of one step.  A consumer wave stages exactly the part of the step's
        // tiles that its own reduction reads - the 32-wide d-block `dbw` of Q (dK waves) or of dO
        // (dV waves), all 128 rows: lane l holds the 16-byte chunk l%4 of rows l/4 + 16*part - so
        // refilling a tile buffer needs no barrier among the consumers (the producers, who read
        // whole rows, are kept apart from it by A).  Threads ct < 128 also stage the carries of
        // query ct.  Every request is unconditional, with rows clamped to the sequence, and every
        // iteration consumes what it requested: no register is "perhaps still being loaded" on
        // some path, so the compiler's wait-count bookkeeping stays exact.
        u32x4 tx[8];
        float cR, cG, cRm = 1.f, cGm = 0.f;
        // Four lanes fill the 64 bytes of a row that this wave reduces; an LDS write cycle takes eight
        // lanes, i.e. two rows, whose swizzles must differ in the bit that selects the other half of the
        // row's banks: rows r and r + 2 do (r and r + 1 would collide), hence the order 0 2 1 3 ...
        const int crow4 = lane >> 2;
        const int crow = (crow4 & ~3) | ((crow4 & 1) << 1) | ((crow4 >> 1) & 1), cch = 4 * dbw + (lane & 3);
        // Per-item base pointers, worked out once per item and held in VECTOR registers (which
        // the consumers have to spare): a step's requests then cost a few vector instructions.
        // Left to itself the compiler keeps such uniform values in scalar registers, runs out
        // of them, and re-derives the pointers from the kernel arguments in every iteration
        // (a wave issues one instruction every four or five cycles, scalar ones included, and
        // the consumers' share of a step is short).
        struct ItemPtrs {
            const char* x;                     // Q or dO: row 0 of the sequence, this head, this thread's chunk
            const float *rt, *gt;              // carries of this (head, key block): row block 0, query 0
            const float *rm, *gm;              // the mid-block carries
            int row0, len;                     // first query of the item's sweep; sequence length
        };
        auto item_ptrs = [&](const KeyItem& t) {
            ItemPtrs r;
            const TensorArg& xt = is_dv ? p.d_o : p.q_scaled;      // Q as the dQ pass left it: times scale * log2 e
            r.x = xt.ptr + 2 * ((int64_t)t.job.seq * xt.sb + (int64_t)t.head * xt.sh + (int64_t)t.job.tok0 * xt.st) + cch * 16;
            const int64_t tk = tab_index(p, t.head, t.job, 0, t.kb);
            r.rt = p.rtab + tk;
            r.gt = p.gtab + tk;
            r.rm = p.rmid + tk;
            r.gm = p.gmid + tk;
            r.row0 = t.job.rb * kRowBlock;
            r.len = t.job.len;
            asm volatile("" : "+v"(r.x), "+v"(r.rt), "+v"(r.gt));
            asm volatile("" : "+v"(r.rm), "+v"(r.gm));
            return r;
        };
        const uint32_t x_st2 = 2u * (uint32_t)(is_dv ? p.d_o.st : p.q_scaled.st);
        auto request_step = [&](const ItemPtrs& t, int row0) {
            const int qi = min(row0 + (ct & (kRowBlock - 1)), t.len - 1);
            const int qb = qi >> 7;            // row block of the query: its slab starts qb*(qb+1) columns in
            const int64_t ix = (int64_t)qb * (qb + 1) * kRowBlock + (qi & (kRowBlock - 1));
            // (The pointers went through registers that the compiler cannot see into, see item_ptrs: it no longer knows
            // that they point to global memory, and plain loads would become FLAT instructions, which also count as LDS
            // traffic - every wait for an LDS read in the reduction would wait for these loads too.)
            auto gl = [](const float* q) { return *(const __attribute__((address_space(1))) float*)q; };
            cR = gl(t.rt + ix); cG = gl(t.gt + ix);
            cRm = gl(t.rm + ix); cGm = gl(t.gm + ix);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t row = (uint32_t)min(row0 + crow + 16 * i, t.len - 1);
                tx[i] = *(const __attribute__((address_space(1))) u32x4*)(t.x + (size_t)row * x_st2);
            }
        };
        constexpr int kLoadsPerStep = 8 + 4;        // per lane: what request_step issues
        // K and V tiles of an item go straight from global memory into LDS (no registers, and
        // nothing for the wait-count bookkeeping to track): every instruction moves 64 x 16 bytes
        // into 1 KB of consecutive LDS, the lane picks the global chunk that belongs at its LDS
        // position (rows in MFMA order, chunks swizzled).  Rows past the end are clamped: those
        // keys are masked for every valid query and their dK/dV rows are not stored.
        auto request_keys = [&](const KeyItem& t, char* vdst) {
            const int64_t kbase = (int64_t)t.job.seq * p.k.sb + (int64_t)t.head * p.k.sh + (int64_t)t.job.tok0 * p.k.st;
            const int64_t vbase = (int64_t)t.job.seq * p.v.sb + (int64_t)t.head * p.v.sh + (int64_t)t.job.tok0 * p.v.st;
#pragma unroll
            for (int i2 = 0; i2 < 2; ++i2) {
                const int inst = w4 + 4 * i2;              // 8 instructions per tile over 4 waves
                const int pos = inst * 64 + lane;          // LDS chunk position
                const int r = pos / (D / 8), pc = pos % (D / 8);
                const int c = pc ^ swz<D>(r);
                // NP = 4: the accumulator registers of a producer lane are 32 consecutive keys over its two
                // tiles; NP = 8: 16 consecutive keys of the one tile (rows 32kh..) of producer half kh
                const int kl = NP == 4 ? (((r >> 2) & 1) << 5) | (((r >> 5) & 1) << 4) | (((r >> 3) & 3) << 2) | (r & 3)
                                       : (((r >> 5) & 1) << 5) | (((r >> 2) & 1) << 4) | (((r >> 3) & 3) << 2) | (r & 3);
                const int row = min(t.key0 + kl, t.job.len - 1);
                // (the copy as inline assembly, see TileDma: through the builtin, the first LDS fetch of EVERY iteration's
                // reduction waited for all vector-memory traffic, the tiles just requested for step s + 2 included)
                dma16(p.k.ptr + 2 * kbase, 2u * (uint32_t)(row * (int)p.k.st + c * 8), lds_address(ktile + inst * 1024));
                dma16(p.v.ptr + 2 * vbase, 2u * (uint32_t)(row * (int)p.v.st + c * 8), lds_address(vdst + inst * 1024));
            }
        };
        auto deposit = [&](int s) {
            char* xtile = bufs + (s & 1) * kBuf + 2 * kZTile + (is_dv ? kQTile : 0);
#pragma unroll
            for (int i = 0; i < 8; ++i) *(u32x4*)(xtile + tile_offset<D>(crow + 16 * i, cch)) = tx[i];
            if (ct < kRowBlock) {
                *(float4*)(carry + (s & 1) * kCarry + ct * 16) = float4{cR, cG, cRm, cGm};
            }
        };
        auto store_staged = [&](int idx, const char* staging) {
            const KeyItem t = decode_item(p, idx);
            const int64_t dkbase = (int64_t)t.job.seq * p.dk.sb + (int64_t)t.head * p.dk.sh + (int64_t)t.job.tok0 * p.dk.st;
            const int64_t dvbase = (int64_t)t.job.seq * p.dv.sb + (int64_t)t.head * p.dv.sh + (int64_t)t.job.tok0 * p.dv.st;
            store_staged_rows<D>(staging, p.dk, dkbase, t.key0, t.job.len, ct, kThreads);
            store_staged_rows<D>(staging + kTile, p.dv, dvbase, t.key0, t.job.len, ct, kThreads);
        };
        auto stage = [&](char* staging) {
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
                // the Q rows carried scale * log2 e: dK = scale * dZ^T Q = (scale / scale2) * the sum
                stage_acc_tile<D>(staging + (is_dv ? kTile : 0), 32 * kh, 32 * dbw, acc[kh], is_dv ? 1.0f : p.scale / p.scale2, lane);
                acc[kh] = f32x16{0};
            }
        };
        // dK[key][d] += sum_q dz[q][key] Q[q][d]  or  dV[key][d] += sum_q a[q][key] dO[q][d].
        // The operands of four 16-query groups are fetched as one batch, so that the MFMAs wait
        // for LDS once per batch rather than once each; `between(b)` (the tile requests) goes
        // behind the fetches of batch b.
        auto reduce = [&](int s_done) {
            const char* zt = bufs + (s_done & 1) * kBuf + (is_dv ? 0 : kZTile);            // a or dz
            const char* xt = bufs + (s_done & 1) * kBuf + 2 * kZTile + (is_dv ? kQTile : 0); // dO or Q
            constexpr int kBatch = NP == 8 ? 2 : 4;        // NP = 8: three waves per SIMD, fewer registers
#pragma unroll
            for (int b = 0; b < 8 / kBatch; ++b) {
                h16x8 aw[kBatch][2], bx[kBatch];
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const int c2 = kBatch * b + j;
                    aw[j][0] = fetch_nat_2<64>(zt, za[0][0], za[0][1], 16 * c2);
                    aw[j][1] = fetch_nat_2<64>(zt, za[1][0], za[1][1], 16 * c2);
                    bx[j] = fetch_nat_2<D>(xt, qb0o, qb1o, 16 * c2);
                }
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    acc[0] = mfma(aw[j][0], bx[j], acc[0]);
                    acc[1] = mfma(aw[j][1], bx[j], acc[1]);
                }
                if (NP == 8) __builtin_amdgcn_sched_barrier(0);
            }
        };

        // A step's tiles and carries are requested right after the previous step's have been
        // deposited, almost a whole iteration before their own deposit (an iteration is shorter than
        // a round trip to memory plus the reduction: requested at the start of the iteration that
        // deposits them, as an earlier version did, they were waited for).  `front` is the position of
        // the next request in the stream of (item, step) pairs; past the end of the stream it stays on
        // the last step (a harmless repeat).
        struct Front {
            ItemPtrs ptrs;
            int it, n_steps, ring;
            bool done;
        } front;
        front.ptrs = item_ptrs(cur);
        front.it = 0; front.n_steps = cur.n_steps; front.ring = 1; front.done = false;
        auto request_front = [&]() {
            request_step(front.ptrs, front.ptrs.row0 + front.it * kRowBlock);
            if (front.done) return;
            if (front.it + 1 < front.n_steps) { ++front.it; return; }
            const int idx = static_item(front.ring);
            if (idx < 0) { front.done = true; return; }
            const KeyItem t = decode_item(p, idx);
            front.ptrs = item_ptrs(t);
            front.it = 0; front.n_steps = t.n_steps; ++front.ring;
        };
        // Memory operations complete in order: with one step's requests in flight, everything issued
        // before them (a deposited step, K / V tiles, stores) has landed.
        static_assert(kLoadsPerStep < 16, "wait-count immediate");
        auto wait_all_but_requests = [&]() { __builtin_amdgcn_s_waitcnt(0x0F70 | kLoadsPerStep); };
        request_keys(cur, vtiles);
        request_front();
        deposit(0);
        request_front();
        wait_all_but_requests();
        __syncthreads();                       // first item's tiles and carries visible

        int s = 0;
        bool finish_after_reduce = false;      // the step about to be reduced is its item's last
        bool store_pending = false;            // a staged dK/dV waits in Z[s&1] to be stored
        int fin_stage = cur_idx, fin_store = cur_idx;
        // B, a barrier of the four consumer waves only (the producers have no part in what it
        // protects and must not be held up by it): a running count in LDS, bumped by each wave,
        // and a short, bounded spin (all four waves are resident).
        int sync_target = 0;
        auto consumer_sync = [&]() {
            sync_target += 4;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            if (lane == 0) __hip_atomic_fetch_add(&consumers_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            wait_for_count(&consumers_done, sync_target, p.gave_up);
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        };
        // One iteration of the stream: the producers work on step s meanwhile.
        auto iteration = [&](bool last, bool keys_now, int item) {
            if (store_pending) {               // staged in the previous iteration
                store_staged(fin_store, bufs + (s & 1) * kBuf);
                store_pending = false;
                __syncthreads();               // X: the producers may overwrite the staging
            }
            if (keys_now) {
                // the K tile is free once every producer holds this item's fragments; V goes to the
                // tile of the other parity
                wait_for_count(&producers_took_k, NP * (item + 1), p.gave_up);
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                request_keys(decode_item(p, nxt_idx), vtiles + ((item + 1) & 1) * kTile);
            }
            if (s > 0) reduce(s - 1);
            // B, only where a finished dK/dV is staged into the Z buffer just reduced: every
            // consumer must be through with it
            if (finish_after_reduce) {
                consumer_sync();
                stage(bufs + ((s - 1) & 1) * kBuf);
                fin_store = fin_stage;
                store_pending = true;
            }
            deposit(s + 1);                    // requested at the end of the previous iteration
            finish_after_reduce = last;
            if (last) fin_stage = cur_idx;
            __builtin_amdgcn_sched_barrier(0);
            request_front();                   // step s + 2
            wait_all_but_requests();
            __syncthreads();                   // A
            ++s;
        };
        for (int item = 0;; ++item) {
            // The next item's K and V are requested in the second-to-last step
            const int n_steps = cur.n_steps;
            const bool has_next = nxt.valid;
            const int keys_at = n_steps >= 2 ? n_steps - 2 : 0;
            for (int it = 0; it < n_steps; ++it) iteration(it + 1 == n_steps, has_next && it == keys_at, item);
            if (!has_next) break;
            cur_idx = nxt_idx;
            cur = nxt;
            nxt_idx = static_item(ring);
            nxt = decode_item(p, nxt_idx);
            ++ring;
        }
        // draining iteration: the last step of the last item
        if (store_pending) store_staged(fin_store, bufs + (s & 1) * kBuf);
        reduce(s - 1);
        consumer_sync();                       // B
        stage(bufs + ((s - 1) & 1) * kBuf);
        __syncthreads();                       // A (consumers only need each other's staging)
        store_staged(fin_stage, bufs + ((s - 1) & 1) * kBuf);
    }
}

// ---------------------------------------------------------------- pass 2, every wave on its own keys
// One workgroup per (128-key block, head); wave w owns the 32 keys 32w..32w+31 of the block for
// the whole sweep, K and V fragments in registers, and accumulates its [32 keys x D] slices of
// dK and dV itself: nothing is exchanged between waves, and the only workgroup barrier is the
// one that publishes the next 64-query Q / dO tiles (global -> LDS DMA, double-buffered).
// A step covers 64 queries as two [32 keys x 32 queries] score tiles; lane (n, h) holds the 16
// consecutive keys 16h..16h+15 of one query per tile.  The carries that enter the wave's 32 keys
// come from the tables of the forward and of the dQ pass: the block-edge ones for the half of
// a 64-key block that touches the edge, the mid-block ones for the other half.  Weights and
// logit gradients go as bf16 [query][32 a | 32 dz] rows into a tile private to the wave and
// come back transposed as the A operands of  dV += A^T dO  and  dK += dZ^T Q.
// kSplit: at head_dim 256 the [32 keys x 256] accumulators of dK and dV alone are 256 registers a lane, on top of 128
// for the K and V fragments.  There the grid has kSplit = 2 workgroups per (key block, head), blockIdx.y = 0, 1, and
// workgroup `part` accumulates and stores columns 128 * part .. 128 * part + 127 of dK and dV only; scores, weights and
// logit gradients are formed in both.
template <int D, int kSplit = 1>
__global__ __launch_bounds__(kThreads, D == 64 ? 2 : 1) void mfma_bwd_dkv_own_kernel(KParams p) {
    constexpr int kNB = D / 32 / kSplit;         // 32-wide column blocks of dK / dV accumulated here
    const int part = kSplit > 1 ? (int)blockIdx.y : 0;
    static_assert(32 * (D / kSplit) * 2 <= 64 * 64 * 2, "a wave stages its [32 keys x columns] outputs in its weight tile");
    constexpr int kQTile = 64 * D * 2;           // Q or dO tile of one step (64 queries)
    constexpr int kZTile = 64 * 64 * 2;          // per wave: [64 queries][32 a | 32 dz] bf16
    constexpr int kStep = 64;
    // At head_dim 128 a SIMD holds one wave, so nothing but the wave itself can keep the matrix cores
    // busy during its exp/rcp: there the reduction over a step's second tile waits for the NEXT step
    // and goes between the segments of that step's first chain.  The Q / dO tiles of a step then
    // have to outlive it by one step: three tile buffers instead of two.
    constexpr bool kDefer = D == 128;
    // LDS fetches with the pinned base (see fetch_cols_o): -1.6 % at head_dim 64, +2.5 % at 128 (registers)
    constexpr bool kOwnPin = D == 64;
    constexpr int kNBuf = kDefer ? 3 : 2;
    __shared__ __attribute__((aligned(16))) char lds[2 * kNBuf * kQTile + 4 * kZTile];   // Q, dO per buffer | one Z tile per wave

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 31, h = lane >> 5;
    LaneOffsets<D> lo;
    lo.init(lane);
    LaneOffsets<64> lz;
    lz.init(lane);
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_key_job(p, blockIdx.x / p.n_heads);
    const int strict = p.attend_current ? 0 : 1;
    const int q_begin = job.rb * kRowBlock;            // first key of the block = first query that may see it
    const int kb0 = q_begin + 32 * wave;               // first key of this wave
    char* ztile = lds + 2 * kNBuf * kQTile + wave * kZTile;

    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;

    // A operands of the score tiles: MFMA row m holds key 16*((m>>2)&1) + 4*(m>>3) + (m&3) of
    // the wave, so that the accumulator registers of a lane are 16 consecutive keys
    h16x8 kfr[D / 16], vfr[D / 16];
    {
        const int m = lane & 31;
        const int key = kb0 + 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3);
        load_row_frags<D>(kfr, p.k, kbase, key, job.len, lane);
        load_row_frags<D>(vfr, p.v, vbase, key, job.len, lane);
        prescale_frags(kfr, p.scale2);         // K times the logit scale: the score MFMAs deliver base-2 logits
    }

    f32x16 dkacc[kNB], dvacc[kNB];
#pragma unroll
    for (int db = 0; db < kNB; ++db) { dkacc[db] = f32x16{0}; dvacc[db] = f32x16{0}; }

    const int n_steps = q_begin < job.len ? (job.len - q_begin + kStep - 1) / kStep : 0;

    TileDma<D, true> qc, dc;
    qc.init(lane, wave, p.q, qbase);
    dc.init(lane, wave, p.d_o, dobase);
    if (n_steps > 0) {
        qc.issue(q_begin, job.len, lds);
        dc.issue(q_begin, job.len, lds + kQTile);
    }

    // carries of a (query, this wave's 32 keys) pair: the right half of a 64-key block takes the
    // forward's block-edge carry and the mid-block prefix, the left half the other two
    const int kb64 = (q_begin + 32 * wave) / kKeyBlock;      // 2*rb or 2*rb + 1: a column of every row block's slab from rb on
    const float* rsrc = ((wave & 1) ? p.rtab : p.rmid) + tab_index(p, head, job, 0, kb64) + n;
    const float* gsrc = ((wave & 1) ? p.gmid : p.gtab) + tab_index(p, head, job, 0, kb64) + n;
    float Rn[2] = {1.f, 1.f}, Gn[2] = {0.f, 0.f};
    // A step's 64 queries lie inside one 128-row block: the table index is a uniform base plus the lane's row.
    // Rows past the end of the sequence are read too (the tables are allocated in whole row blocks) and not used.
    auto request_carries = [&](int q0) {
        const int qb = q0 >> 7;
        const int64_t ix = (int64_t)qb * (qb + 1) * kRowBlock + (q0 & (kRowBlock - 1));      // uniform
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            Rn[t] = rsrc[ix + 32 * t];
            Gn[t] = gsrc[ix + 32 * t];
        }
    };
    if (n_steps > 0) request_carries(q_begin);
    wait_global_memory();
    __syncthreads();

    // Every LDS address of the loop is "a register that is fixed for the whole sweep + a constant": the lane offsets are
    // made absolute once (Q / dO tiles from the start of the array, the weight tile from this wave's tile), and the loop
    // runs in one copy per tile buffer, so that buffer and row offsets are compile-time numbers in the offset fields of
    // the fetches (with the tile address in a scalar register each fetch or pinned sum costs a vector add with a scalar
    // operand: 25 of them per step here).
    if (kSplit > 1) {
        // this workgroup's column blocks: kNB blocks are 4 * kNB sixteen-byte chunks, a multiple of 16, and the swizzle
        // only touches chunk bits 0..3, so block b + part * kNB lies part * kNB * 64 bytes further along the same row
        static_assert(kSplit == 1 || kNB % 4 == 0, "the shift must not meet the swizzled chunk bits");
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < kNB; ++b) lo.nat[a][b] += part * (kNB * 64);
    }
    lo.rebase(lds);
    lz.rebase(ztile);
    constexpr TileAt zt{0};
    uint32_t zst[4];              // this lane's row of the weight tile: chunks 2h, 2h + 1 (a) and 4 + 2h, 4 + 2h + 1 (dz)
#pragma unroll
    for (int c = 0; c < 4; ++c) zst[c] = lds_lane_base(ztile, tile_offset<64>(n, (c >> 1) * 4 + 2 * h + (c & 1)));
    auto put_z = [&](int c, int t, h16x8 v) __attribute__((always_inline)) {
        *(__attribute__((address_space(3))) h16x8*)((__attribute__((address_space(3))) char*)(uintptr_t)zst[c] + t * 32 * 64 * 2) = v;
    };

    auto second_tile_reduction = [&](auto qt, auto dot) __attribute__((always_inline)) {
#pragma unroll
        for (int kk = 2; kk < 4; ++kk) {
            const h16x8 af = fetch_nat_o<64>(zt, lz, 16 * kk, 0);
            const h16x8 zf = fetch_nat_o<64>(zt, lz, 16 * kk, 1);
#pragma unroll
            for (int db = 0; db < kNB; ++db) {
                dvacc[db] = mfma(af, fetch_nat_o<D>(dot, lo, 16 * kk, db), dvacc[db]);
                dkacc[db] = mfma(zf, fetch_nat_o<D>(qt, lo, 16 * kk, db), dkacc[db]);
            }
        }
    };
    bool pending = false;                      // the previous step left its second tile's reduction to this one
    auto do_step = [&](int step, auto buf_c) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        constexpr int nbuf = buf + 1 == kNBuf ? 0 : buf + 1;
        constexpr int pbuf = buf == 0 ? kNBuf - 1 : buf - 1;
        constexpr TileAt qtile{buf * 2 * kQTile}, dotile{buf * 2 * kQTile + kQTile};
        constexpr TileAt pqtile{pbuf * 2 * kQTile}, pdotile{pbuf * 2 * kQTile + kQTile};      // the previous step's tiles (kDefer)
        const int q0 = q_begin + step * kStep;
        const bool more = step + 1 < n_steps;
        float Rin[2], Gin[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) { Rin[t] = Rn[t]; Gin[t] = Gn[t]; }
        if (more) {       // next tiles, straight into the next buffer (nobody reads it since the last barrier)
            qc.issue(q0 + kStep, job.len, lds + nbuf * 2 * kQTile);
            dc.issue(q0 + kStep, job.len, lds + nbuf * 2 * kQTile + kQTile);
            request_carries(q0 + kStep);
        }
        // whole step left of this wave's first key: nothing visible
        const bool skip = kb0 + strict > q0 + kStep - 1 || kb0 >= job.len;
        if (!skip) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int qt0 = q0 + 32 * t;
                const int qi = qt0 + n;
                // visible keys among this lane's 16 (queries past the end see none)
                const int nvis = qi < job.len ? qi - strict - (kb0 + 16 * h) + 1 : 0;
                const bool sees_wave = qi < job.len && qi - strict - kb0 + 1 > 0;
                const float Rt = sees_wave ? Rin[t] : 1.0f;      // table entries of invisible pairs are not written
                const float Gt = sees_wave ? Gin[t] : 0.0f;
                float x[16], beta[16], dp[16];
                {
                    // with one wave on the SIMD (d = 128) nothing hides an LDS round trip in front of
                    // each MFMA: all operands of the tile are requested first
                    h16x8 bq[D / 16];
#pragma unroll
                    for (int ks = 0; ks < D / 16; ++ks) bq[ks] = fetch_rows_o<D>(qtile, lo, t, ks);
                    if (D == 128) __builtin_amdgcn_sched_barrier(0);
                    f32x16 acc = {0};
#pragma unroll
                    for (int ks = 0; ks < D / 16; ++ks) acc = mfma(kfr[ks], bq[ks], acc);
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[r] = acc[r];
                }
                if (kb0 + 31 + strict > qt0 || qt0 + 31 >= job.len) {     // diagonal or ragged tile
#pragma unroll
                    for (int idx = 0; idx < 16; ++idx)
                        if (idx >= nvis) x[idx] = -INFINITY;
                }
                if (t == 0 && kDefer && pending) {
                    // the previous step's second tile: rows 32.. of the wave's weight tile (not yet
                    // overwritten: this step's second tile comes later) and of the previous Q / dO tiles
                    auto red_a = [&](int seg) { return fetch_nat_o<64>(zt, lz, 32 + 16 * (seg >> 1), seg & 1); };
                    auto red_b = [&](int seg, int db) {
                        return (seg & 1) ? fetch_nat_o<D>(pqtile, lo, 32 + 16 * (seg >> 1), db) : fetch_nat_o<D>(pdotile, lo, 32 + 16 * (seg >> 1), db);
                    };
                    h16x8 na = red_a(0), nb[kNB];
#pragma unroll
                    for (int db = 0; db < kNB; ++db) nb[db] = red_b(0, db);
                    own_tile_weights(x, beta, Rt, lane, [&](int seg) {
                        const h16x8 ca = na;
                        h16x8 cb[kNB];
#pragma unroll
                        for (int db = 0; db < kNB; ++db) cb[db] = nb[db];
                        if (seg < 3) {
                            na = red_a(seg + 1);
#pragma unroll
                            for (int db = 0; db < kNB; ++db) nb[db] = red_b(seg + 1, db);
                        }
#pragma unroll
                        for (int db = 0; db < kNB; ++db) {
                            if (seg & 1) dkacc[db] = mfma(ca, cb[db], dkacc[db]);
                            else dvacc[db] = mfma(ca, cb[db], dvacc[db]);
                        }
                    });
                } else if (t == 0) {
                    own_tile_weights(x, beta, Rt, lane, [](int) {});
                } else {
                    // The reduction over the first tile's 32 queries only needs that tile's weights, which
                    // this wave wrote above: its MFMAs go between the segments of the second tile's chain,
                    // whose exp/rcp overlap them.  Segment 2kk: dV += A^T dO, segment 2kk + 1: dK += dZ^T Q.
                    auto red_a = [&](int seg) { return fetch_nat_o<64>(zt, lz, 16 * (seg >> 1), seg & 1); };
                    auto red_b = [&](int seg, int db) {
                        return (seg & 1) ? fetch_nat_o<D>(qtile, lo, 16 * (seg >> 1), db) : fetch_nat_o<D>(dotile, lo, 16 * (seg >> 1), db);
                    };
                    h16x8 na = red_a(0), nb[kNB];
#pragma unroll
                    for (int db = 0; db < kNB; ++db) nb[db] = red_b(0, db);
                    own_tile_weights(x, beta, Rt, lane, [&](int seg) {
                        const h16x8 ca = na;
                        h16x8 cb[kNB];
#pragma unroll
                        for (int db = 0; db < kNB; ++db) cb[db] = nb[db];
                        if (seg < 3) {
                            na = red_a(seg + 1);
#pragma unroll
                            for (int db = 0; db < kNB; ++db) nb[db] = red_b(seg + 1, db);
                        }
#pragma unroll
                        for (int db = 0; db < kNB; ++db) {
                            if (seg & 1) dkacc[db] = mfma(ca, cb[db], dkacc[db]);
                            else dvacc[db] = mfma(ca, cb[db], dvacc[db]);
                        }
                    });
                }
                {
                    h16x8 bd[D / 16];
#pragma unroll
                    for (int ks = 0; ks < D / 16; ++ks) bd[ks] = fetch_rows_o<D>(dotile, lo, t, ks);
                    if (D == 128) __builtin_amdgcn_sched_barrier(0);
                    f32x16 acc = {0};
#pragma unroll
                    for (int ks = 0; ks < D / 16; ++ks) acc = mfma(vfr[ks], bd[ks], acc);
#pragma unroll
                    for (int r = 0; r < 16; ++r) dp[r] = acc[r];
                }
                // a -> columns 16h.. of row (32t + n), dz -> columns 32 + 16h..
                put_z(0, t, pack8(&x[0]));
                put_z(1, t, pack8(&x[8]));
                own_tile_grads(x, beta, dp, Gt, lane);
                put_z(2, t, pack8(&dp[0]));
                put_z(3, t, pack8(&dp[8]));
            }
            // dV += A^T dO, dK += dZ^T Q over the second tile's queries (the first tile's went with the
            // second chain): now, or with the next step's first chain
            if (!kDefer) second_tile_reduction(qtile, dotile);
            pending = kDefer;
        }
        wait_global_memory();                  // the next tiles and carries have landed
        __syncthreads();
    };
    // one copy of the step per tile buffer
    int last_buf = 0;
    for (int step = 0; step < n_steps; step += kNBuf) {
        do_step(step, std::integral_constant<int, 0>{});
        last_buf = 0;
        if (step + 1 < n_steps) { do_step(step + 1, std::integral_constant<int, 1>{}); last_buf = 1; }
        if (kNBuf == 3 && step + 2 < n_steps) { do_step(step + 2, std::integral_constant<int, kNBuf - 1>{}); last_buf = 2; }
    }
    if (kDefer && pending) {
        if (last_buf == 0) second_tile_reduction(TileAt{0}, TileAt{kQTile});
        else if (last_buf == 1) second_tile_reduction(TileAt{2 * kQTile}, TileAt{3 * kQTile});
        else second_tile_reduction(TileAt{(kNBuf - 1) * 2 * kQTile}, TileAt{(kNBuf - 1) * 2 * kQTile + kQTile});
    }

    // ---- rows kb0.. of dK (scaled) and dV, through the wave's own tile as coalesced 16-byte stores
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const TensorArg& out = which == 0 ? p.dk : p.dv;
        const int64_t ob = (int64_t)job.seq * out.sb + (int64_t)head * out.sh + (int64_t)job.tok0 * out.st;
        constexpr int kCols = D / kSplit;          // columns part * kCols .. of the rows
#pragma unroll
        for (int db = 0; db < kNB; ++db)
            stage_acc_tile<kCols>(ztile, 0, 32 * db, which == 0 ? dkacc[db] : dvacc[db], which == 0 ? p.scale : 1.0f, lane);
        for (int c = lane; c < 32 * kCols / 8; c += 64) {
            const int row = c / (kCols / 8), cc = c % (kCols / 8);
            if (kb0 + row < job.len)
                *(u32x4*)(out.ptr + 2 * (ob + (int64_t)(kb0 + row) * out.st + part * kCols + cc * 8)) = *(const u32x4*)(ztile + row * (kCols * 2) + cc * 16);
        }
    }
}


// ---------------------------------------------------------------- pass 2, two waves per 32 keys
// What a wave of the own-keys kernel holds for its 32 keys at head_dim 128 - K and V fragments and the
// [32 keys x 128] accumulators of dK and dV - is 190 registers: one wave per SIMD.  Here TWO waves share
// 32 keys.  Both hold the K and V fragments; wave r of the pair turns query tile r of the step (32 of
// its 64 queries) into weights and logit gradients and writes them to the pair's tile in LDS; after a
// barrier each wave reduces ALL 64 queries of the step for ITS half of the head dim (column blocks
// 2r, 2r + 1 at head_dim 128), so it accumulates [32 keys x D/2] of dK and of dV only.  The vector work
// of a step is split between the two, the reductions too: eight waves per workgroup (128 keys), two per
// SIMD.  Two workgroup barriers per step (weights complete; tiles handed over).
template <int D>
__global__ __launch_bounds__(2 * kThreads, 2) void mfma_bwd_dkv_pair_kernel(KParams p) {
    constexpr int kQTile = 64 * D * 2;           // Q or dO tile of one step (64 queries)
    constexpr int kZTile = 64 * 64 * 2;          // per pair: [64 queries][32 a | 32 dz] bf16
    constexpr int kStep = 64;
    constexpr bool kPairPin = true;              // LDS fetch bases pinned in registers: 3 % faster here
    constexpr int kBlocks = D / 64;              // 32-wide column blocks of dK / dV per wave
    static_assert(32 * D * 2 <= kZTile, "the pair's tile doubles as the staging of its [32 keys x D] outputs");
    __shared__ __attribute__((aligned(16))) char lds[4 * kQTile + 4 * kZTile];   // (Q, dO) x 2 buffers | one Z tile per pair

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int grp = wave >> 1, r = wave & 1;
    const int n = lane & 31, h = lane >> 5;
    LaneOffsets<D> lo;
    lo.init(lane);
    LaneOffsets<64> lz;
    lz.init(lane);
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_key_job(p, blockIdx.x / p.n_heads);
    const int strict = p.attend_current ? 0 : 1;
    const int q_begin = job.rb * kRowBlock;            // first key of the block = first query that may see it
    const int kb0 = q_begin + 32 * grp;                // first key of this pair
    char* ztile = lds + 4 * kQTile + grp * kZTile;

    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;

    // A operands of the score tile: MFMA row m holds key 16*((m>>2)&1) + 4*(m>>3) + (m&3) of the pair,
    // so that the accumulator registers of a lane are 16 consecutive keys (as in the own-keys kernel)
    h16x8 kfr[D / 16], vfr[D / 16];
    {
        const int m = lane & 31;
        const int key = kb0 + 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3);
        load_row_frags<D>(kfr, p.k, kbase, key, job.len, lane);
        load_row_frags<D>(vfr, p.v, vbase, key, job.len, lane);
        prescale_frags(kfr, p.scale2);
    }
    f32x16 dkacc[kBlocks], dvacc[kBlocks];
#pragma unroll
    for (int j = 0; j < kBlocks; ++j) { dkacc[j] = f32x16{0}; dvacc[j] = f32x16{0}; }

    const int n_steps = q_begin < job.len ? (job.len - q_begin + kStep - 1) / kStep : 0;

    // waves 0-3 copy the Q tiles, waves 4-7 the dO tiles
    TileDma<D, true> tc;
    tc.init(lane, wave & 3, wave < 4 ? p.q : p.d_o, wave < 4 ? qbase : dobase);
    const int my_tile = wave < 4 ? 0 : kQTile;
    if (n_steps > 0) tc.issue(q_begin, job.len, lds + my_tile);

    // carries of a (query, this pair's 32 keys) pair, see the own-keys kernel
    const int kb64 = kb0 / kKeyBlock;
    const float* rsrc = ((grp & 1) ? p.rtab : p.rmid) + tab_index(p, head, job, 0, kb64);
    const float* gsrc = ((grp & 1) ? p.gmid : p.gtab) + tab_index(p, head, job, 0, kb64);
    float Rn = 1.f, Gn = 0.f;
    // A step's 64 queries lie inside one 128-row block: the table index is a uniform base plus the lane's
    // row.  Rows past the end of the sequence are read too (the tables are allocated in whole row blocks)
    // and not used.
    const int my_row = 32 * r + n;
    auto request_carries = [&](int q0) __attribute__((always_inline)) {
        const int qb = q0 >> 7;
        const int64_t ix = (int64_t)qb * (qb + 1) * kRowBlock + (q0 & (kRowBlock - 1));      // uniform
        Rn = rsrc[ix + my_row];
        Gn = gsrc[ix + my_row];
    };
    if (n_steps > 0) request_carries(q_begin);
    wait_global_memory();
    __syncthreads();

    // Every LDS address of the loop is "a register that is fixed for the whole sweep + a constant": the sums of
    // LDS base, lane offset and this wave's share (query tile r, column blocks 2r.., the pair's weight tile) are
    // made once, and the loop runs in two copies, one per tile buffer, so that buffer and row offsets are compile-time
    // numbers that go into the offset fields of the fetches.  (With the tile address in a scalar register each
    // fetch costs one or two vector adds with a scalar operand, 1.8 ns each: 40 of them per step.)
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
    uint32_t row_at[D / 16], nat_at[2][kBlocks], z_at[2][2];
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) row_at[ks] = lds_lane_base(lds + r * 32 * D * 2, lo.rows[ks]);
    {
        const int hh = lane >> 5, G1 = (lane >> 4) & 1, sl = lane & 15;
#pragma unroll
        for (int a2 = 0; a2 < 2; ++a2) {
#pragma unroll
            for (int j = 0; j < kBlocks; ++j) {
                const int chunk = 4 * (kBlocks * r + j) + 2 * G1 + ((sl & 3) >> 1);
                nat_at[a2][j] = lds_lane_base(lds, tile_offset<D>(8 * hh + 4 * a2 + (sl >> 2), chunk) + ((sl & 1) << 3));
            }
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) z_at[a2][cb] = lds_lane_base(ztile, lz.nat[a2][cb]);
        }
    }
    (void)lds0;
    auto rows_at = [&](uint32_t base, int imm) __attribute__((always_inline)) {
        return *(const __attribute__((address_space(3))) h16x8*)((__attribute__((address_space(3))) char*)(uintptr_t)base + imm);
    };
    auto nat_pair = [&](const uint32_t (&at)[2][2], int col, int imm) __attribute__((always_inline)) {
        union { s16x4 v[2]; h16x8 b; } u;
        u.v[0] = lds_read_tr_at(at[0][col], imm);
        u.v[1] = lds_read_tr_at(at[1][col], imm);
        return u.b;
    };

    auto do_step = [&](int step, auto buf_c) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        constexpr int kQ = buf * 2 * kQTile;             // byte offsets of this step's Q and dO tiles
        constexpr int kDO = kQ + kQTile;
        const int q0 = q_begin + step * kStep;
        const float Rin = Rn, Gin = Gn;
        // the score operands are requested first: their LDS round trip passes under the scalar work of the tile requests
        h16x8 bq[D / 16];
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) bq[ks] = rows_at(row_at[ks], kQ);
        __builtin_amdgcn_sched_barrier(0);
        if (step + 1 < n_steps) {     // next tiles, straight into the other buffer (nobody reads it since the last barrier)
            tc.issue(q0 + kStep, job.len, lds + (buf ^ 1) * 2 * kQTile + my_tile);
            request_carries(q0 + kStep);
        }
        __builtin_amdgcn_sched_barrier(0);
        // whole step left of this pair's first key: nothing visible (the same for both waves of the pair)
        const bool skip = kb0 + strict > q0 + kStep - 1 || kb0 >= job.len;
        if (!skip) {
            const int qt0 = q0 + 32 * r;
            const int qi = qt0 + n;
            if (kb0 + strict > qt0 + 31) {             // this wave's query tile sees none of the keys (the other one does)
                const h16x8 none = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int c = 0; c < 4; ++c) *(h16x8*)(ztile + tile_offset<64>(32 * r + n, 2 * c + h)) = none;
            } else {
                float x[16], dp[16];
                const int nvis = qi < job.len ? qi - strict - (kb0 + 16 * h) + 1 : 0;
                const bool sees = qi < job.len && qi - strict - kb0 + 1 > 0;
                const float Rt = sees ? Rin : 1.0f;      // table entries of invisible pairs are not written
                const float Gt = sees ? Gin : 0.0f;
                float beta[16];
                __builtin_amdgcn_s_setprio(3);     // paced like the two-step dQ kernel's chain: the wave behind goes first
                {
                    f32x16 acc = {0};
#pragma unroll
                    for (int ks = 0; ks < D / 16; ++ks) acc = mfma(kfr[ks], bq[ks], acc);
#pragma unroll
                    for (int i = 0; i < 16; ++i) x[i] = acc[i];
                }
                if (kb0 + 31 + strict > qt0 || qt0 + 31 >= job.len) {     // diagonal or ragged tile
#pragma unroll
                    for (int idx = 0; idx < 16; ++idx)
                        if (idx >= nvis) x[idx] = -INFINITY;
                }
                // dP = dO V^T between the segments of the chain, its operands fetched one segment ahead
                constexpr int kPer = D / 64;
                h16x8 nx[kPer];
#pragma unroll
                for (int i = 0; i < kPer; ++i) nx[i] = rows_at(row_at[i], kDO);
                f32x16 dacc;
                own_tile_weights(x, beta, Rt, lane, [&](int seg) {
                    h16x8 cur[kPer];
#pragma unroll
                    for (int i = 0; i < kPer; ++i) cur[i] = nx[i];
                    if (seg < 3) {
#pragma unroll
                        for (int i = 0; i < kPer; ++i) nx[i] = rows_at(row_at[kPer * (seg + 1) + i], kDO);
                    }
#pragma unroll
                    for (int i = 0; i < kPer; ++i) {
                        const int ks = kPer * seg + i;
                        dacc = mfma(vfr[ks], cur[i], ks == 0 ? f32x16{0} : dacc);
                    }
                    if (seg == 1) __builtin_amdgcn_s_setprio(2);
                });
                __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int i = 0; i < 16; ++i) dp[i] = dacc[i];
                // a -> columns 16h.. of row (32r + n) now, dz -> columns 32 + 16h.. below
                *(h16x8*)(ztile + tile_offset<64>(32 * r + n, 2 * h)) = pack8(&x[0]);
                *(h16x8*)(ztile + tile_offset<64>(32 * r + n, 2 * h + 1)) = pack8(&x[8]);
                own_tile_grads(x, beta, dp, Gt, lane);
                *(h16x8*)(ztile + tile_offset<64>(32 * r + n, 4 + 2 * h)) = pack8(&dp[0]);
                *(h16x8*)(ztile + tile_offset<64>(32 * r + n, 4 + 2 * h + 1)) = pack8(&dp[8]);
                __builtin_amdgcn_s_setprio(0);
            }
        }
        __syncthreads();                       // the pair's weights are complete
        if (!skip) {
            // dV += A^T dO, dK += dZ^T Q over the step's 64 queries, this wave's column blocks.  The operands of
            // 16 queries are requested while the MFMAs of the 16 before them run (left to itself the compiler
            // requests them right before their MFMA, which then waits for the LDS round trip: 16 per step).
            h16x8 w[2][2], o[2][2 * kBlocks];
            auto fetch_kk = [&](int kk, h16x8 (&ww)[2], h16x8 (&oo)[2 * kBlocks]) __attribute__((always_inline)) {
                ww[0] = nat_pair(z_at, 0, 16 * kk * 64 * 2);
                ww[1] = nat_pair(z_at, 1, 16 * kk * 64 * 2);
#pragma unroll
                for (int j = 0; j < kBlocks; ++j) {
                    oo[2 * j] = nat_pair(nat_at, j, kDO + 16 * kk * D * 2);
                    oo[2 * j + 1] = nat_pair(nat_at, j, kQ + 16 * kk * D * 2);
                }
            };
            fetch_kk(0, w[0], o[0]);
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                if (kk < 3) fetch_kk(kk + 1, w[(kk + 1) & 1], o[(kk + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < kBlocks; ++j) {
                    dvacc[j] = mfma(w[kk & 1][0], o[kk & 1][2 * j], dvacc[j]);
                    dkacc[j] = mfma(w[kk & 1][1], o[kk & 1][2 * j + 1], dkacc[j]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        wait_global_memory();                  // the next tiles and carries have landed
        __syncthreads();                       // ... and everybody is through with this step's tiles
    };
    for (int step = 0; step < n_steps; step += 2) {
        do_step(step, std::integral_constant<int, 0>{});
        if (step + 1 < n_steps) do_step(step + 1, std::integral_constant<int, 1>{});
    }

    // ---- rows kb0.. of dK (scaled) and dV: each wave stages its column blocks in the pair's tile, the pair
    // stores whole rows as coalesced 16-byte chunks
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const TensorArg& out = which == 0 ? p.dk : p.dv;
        const int64_t ob = (int64_t)job.seq * out.sb + (int64_t)head * out.sh + (int64_t)job.tok0 * out.st;
#pragma unroll
        for (int j = 0; j < kBlocks; ++j)
            stage_acc_tile<D>(ztile, 0, 32 * (kBlocks * r + j), which == 0 ? dkacc[j] : dvacc[j], which == 0 ? p.scale : 1.0f, lane);
        __syncthreads();
        for (int c = lane + 64 * r; c < 32 * D / 8; c += 128) {
            const int row = c / (D / 8), cc = c % (D / 8);
            if (kb0 + row < job.len)
                *(u32x4*)(out.ptr + 2 * (ob + (int64_t)(kb0 + row) * out.st + cc * 8)) = *(const u32x4*)(ztile + row * (D * 2) + cc * 16);
        }
        __syncthreads();
    }
}

}  // inline namespace SBA_ELEM_NS
}  // namespace sba

#ifndef SBA_ELEM_F16
bool sba_mfma_bwd_available() { return true; }
#endif

// SBA_DKV_KERNEL=own / =other overrides the choice between the key-owner kernels (tests run
// both on the same inputs).
static bool own_keys_kernel(bool by_size) {
    const char* e = getenv("SBA_DKV_KERNEL");
    if (e && (!strcmp(e, "own") || !strcmp(e, "pair"))) return true;
    if (e && !strcmp(e, "other")) return false;
    return by_size;
}

// SBA_DQ_KERNEL=lean / =plain overrides the choice between the two arrangements of the one-step dQ kernel at
// head_dim 64 (tests run both on the same inputs).
static bool lean_dq_kernel(bool by_size) {
    const char* e = getenv("SBA_DQ_KERNEL");
    if (e && !strcmp(e, "lean")) return true;
    if (e && !strcmp(e, "plain")) return false;
    return by_size;
}

#ifdef SBA_ELEM_F16
int sba_launch_mfma_f16_bwd(const sba::KParams& kp_in, int phases, hipStream_t s) {
#else
int sba_launch_mfma_bwd(const sba::KParams& kp_in, int phases, hipStream_t s) {
#endif
    using namespace sba;
    KParams kp = kp_in;
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    const bool p1 = phases != 2, p2 = phases != 1;
    // the dQ kernels reach a lane's prefix entry from its carry entry by one uniform distance (see there)
    if (!kp.rtab || !kp.rmid || !kp.gtab || !kp.gmid ||
        (const char*)kp.gmid - (const char*)kp.rtab != (const char*)kp.gtab - (const char*)kp.rmid) return SBA_ERR_WORKSPACE;
    // Key-owner pass.  head_dim 64: from about three workgroups per CU on, the kernel whose waves
    // own their keys outright is ahead; below, the resident producer/consumer stream, which splits
    // the work into twice as many items and balances them itself.  head_dim 128: the paired kernel at
    // every size (on 64 ... 256 workgroups of B=1, H=16 it takes 27 / 44 / 62 / 81 us where the kernel
    // with one workgroup per 64-key block takes 33 / 55 / 73 / 103); SBA_DKV_KERNEL=other still selects that one.
    // Batches of short sequences (sweeps of at most 16 steps) also take the own-keys kernel at any size: on
    // 512 workgroups B=8, T=512 takes 27.3 us against the stream's 33.0, B=4, T=1024 44.0 against 45.3.
    const unsigned cus = (unsigned)sba_cu_count();
    const bool short_sweeps = kp.seq_len <= 8 * kRowBlock;
    // One dense sequence per head from 4096 tokens on keeps the stream up to four and a half workgroups per CU (B=1, H=16:
    // T=7168 297 against 309 us, T=8192 363 against 391, T=9216 445 against 460; from T=10240 on, and for batches of
    // shorter sequences and packs on the same grids, the own-keys kernel is ahead by 2-5 %).
    const bool long_dense = !kp.cu_seqlens && kp.seq_len >= 4096 && 2u * grid.x <= 9u * cus;
    const bool own = own_keys_kernel(kp.head_dim == 64 ? (grid.x >= 3u * cus && !long_dense) || (short_sweeps && grid.x >= 2u * cus) : true);
    const char* which = getenv("SBA_DKV_KERNEL");
    const bool plain = which && !strcmp(which, "plain");
    // the stream with eight half-block producers (12 waves): behind the one with four full-block producers
    // (107 against 99.5 us at B=1 H=16 T=4096), which stays the default
    const bool stream8 = which && !strcmp(which, "stream8");
    // the scaled copy of q is for the stream kernel: no other key-owner kernel reads it, so the dQ pass skips it
    const bool stream = kp.head_dim == 64 && !plain && !own;
    if (stream && !kp.q_scaled.ptr) return SBA_ERR_WORKSPACE;
    if (!stream) kp.q_scaled.ptr = nullptr;
    if (kp.head_dim == 64) {
        // Small grids that last as long as their longest sweep (tail ratio from 3.7: B=1, H=16 up to T=4096) take the
        // variant that halves it; batches of short sequences on the same number of workgroups do not (B=8, T=512:
        // 23.8 us with one step per iteration against 27.4, B=4, T=1024 36.0 against 37.7).
        const bool two_steps = sba_two_step_env() >= 0 ? grid.x <= (unsigned)sba_two_step_env()
                                                       : grid.x <= kTwoStepDqMaxGrid && sba_tail_ratio(kp, grid.x) >= 3.7;
        if (p1 && two_steps) hipLaunchKernelGGL((mfma_bwd_dq2_kernel<64>), grid, dim3(2 * kThreads), 0, s, kp);
        // The register-lean arrangement (three waves per SIMD) from five workgroups per CU on, unless the launch hangs on
        // one long sweep (tail ratio above 2.5: there the plain arrangement's shorter step is ahead, e.g. 111 against 118 us
        // on an 8192-token pack with a 4096-token document); from eight workgroups per CU on always.  On 1280-3232
        // workgroups of 15 dense and packed shapes it is 0-5 % ahead of the plain one; at four workgroups per CU (six
        // shapes of 1024 workgroups) the plain one is, by 1-3 %.
        else if (p1 && lean_dq_kernel(grid.x >= 8u * cus || (grid.x >= 5u * cus && sba_tail_ratio(kp, grid.x) <= 2.5)))
            hipLaunchKernelGGL((mfma_bwd_dq_kernel<64, true>), grid, dim3(kThreads), 0, s, kp);
        else if (p1) hipLaunchKernelGGL((mfma_bwd_dq_kernel<64>), grid, dim3(kThreads), 0, s, kp);
        if (p2 && plain) {
            hipLaunchKernelGGL((mfma_bwd_dkv_kernel<64>), dim3(2 * grid.x), dim3(kThreads), 0, s, kp);
        } else if (p2 && own) {
            hipLaunchKernelGGL((mfma_bwd_dkv_own_kernel<64>), grid, dim3(kThreads), 0, s, kp);
        } else if (p2) {
            // one resident workgroup per CU, in whole rounds of the 8 XCDs (surplus workgroups
            // find no item)
            const unsigned n_items = 2 * grid.x;
            unsigned n_wg = n_items < cus ? n_items : cus;
            n_wg = (n_wg + 7) & ~7u;
            if (stream8) hipLaunchKernelGGL((mfma_bwd_dkv_stream_kernel<64, 8>), dim3(n_wg), dim3(12 * 64), 0, s, kp);
            else hipLaunchKernelGGL((mfma_bwd_dkv_stream_kernel<64, 4>), dim3(n_wg), dim3(8 * 64), 0, s, kp);
        }
    } else if (kp.head_dim == 256) {
        // one wave per SIMD in both passes; every wave of the key-owner pass on its own 32 keys, two workgroups per
        // key block that each accumulate one half of the columns of dK and dV - the other key-owner kernels do not
        // fit the CU here
        if (p1) hipLaunchKernelGGL((mfma_bwd_dq_kernel<256>), grid, dim3(kThreads), 0, s, kp);
        if (p2) {
            hipLaunchKernelGGL((mfma_bwd_dkv_own_kernel<256, 2>), dim3(grid.x, 2), dim3(kThreads), 0, s, kp);
        }
    } else {
        if (p1) hipLaunchKernelGGL((mfma_bwd_dq_kernel<128>), grid, dim3(kThreads), 0, s, kp);
        // key owners at head_dim 128: two waves per 32 keys (6-9 % faster than one wave per 32 keys,
        // which SBA_DKV_KERNEL=own still selects)
        const bool pair = !(which && !strcmp(which, "own"));
        if (p2 && own && pair) hipLaunchKernelGGL((mfma_bwd_dkv_pair_kernel<128>), grid, dim3(2 * kThreads), 0, s, kp);
        else if (p2 && own) hipLaunchKernelGGL((mfma_bwd_dkv_own_kernel<128>), grid, dim3(kThreads), 0, s, kp);
        else if (p2) hipLaunchKernelGGL((mfma_bwd_dkv_kernel<128>), dim3(2 * grid.x), dim3(kThreads), 0, s, kp);
    }
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}
