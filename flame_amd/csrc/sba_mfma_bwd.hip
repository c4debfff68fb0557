// bf16 MFMA backward kernels (head_dim 64 / 128): two passes, no atomics, deterministic.
//
// The reference (`_backward_one_row`, sb_varlen/sb_varlen_bwd.py:274-456) owns a query
// row-block, keeps dq in registers and adds every dk/dv tile into global memory under a
// spin lock (`locked_add`, :13-52).  Here the two reductions are separated instead:
//
//   pass 1  (row owner, like the forward): recomputes the weights of each 64-key step from
//           the forward's carry table, forms dz, accumulates dQ in registers, and records
//           for every (query, key block) the prefix  sum_{j left of the block} g_ij  in a
//           second table.
//   pass 2  (key owner): a workgroup owns one 64-key block, sweeps the query blocks at or
//           below the diagonal, recomputes weights and dz of its tile from the two tables,
//           transposes them through LDS and accumulates dK = dZ^T Q and dV = P^T dO in
//           registers.
//
// Every element of the score matrix is therefore evaluated twice in the backward (once per
// pass); in exchange nothing is reduced through memory.
#include "sba_mfma.h"

namespace sba {

// ---------------------------------------------------------------- pass 1: dQ + prefix table
template <int D>
__global__ __launch_bounds__(kThreads) void mfma_bwd_dq_kernel(KParams p) {
    constexpr int kTile = 64 * D * 2;
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
    const int q0w = m0 + 32 * wave;
    const int qi = q0w + n;
    const bool row_ok = qi < job.len;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;

    bf16x8 qf[D / 16], dof[D / 16];
    load_row_frags<D>(qf, p.q, qbase, qi, job.len, lane);
    load_row_frags<D>(dof, p.d_o, dobase, qi, job.len, lane);
    float dr = 0.f;
    if (row_ok && p.d_rem.ptr)
        dr = Elem<uint16_t>::load(p.d_rem.ptr, (int64_t)job.seq * p.d_rem.sb + (int64_t)head * p.d_rem.sh + job.tok0 + qi);

    f32x16 dqacc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) dqacc[db] = f32x16{0};
    float Gc = 0.f;

    const int imax = min(m0 + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    const int n_steps = kmax >= 0 ? kmax / kKeyBlock + 1 : 0;
    const int64_t tabtok = tab_token(p, job, qi);

    TileCopy<D> kc, vc;
    if (n_steps > 0) {
        kc.load(p.k, kbase, 0, job.len);
        vc.load(p.v, vbase, 0, job.len);
        kc.store(lds);
        vc.store(lds + kTile);
    }
    __syncthreads();

    // carry-table traffic is kept off the critical path: the value of the NEXT step is loaded
    // while this one is computed, and this step's prefix is stored before the tile loads are
    // issued (vector memory operations retire in order)
    const int64_t tstride = p.tab_tokens;
    const int64_t tix0 = (int64_t)head * p.n_kb * p.tab_tokens + tabtok;
    float Rnext = (row_ok && n_steps > 0) ? p.rtab[tix0] : 1.0f;
    for (int step = 0, buf = 0; step < n_steps; ++step, buf ^= 1) {
        const char* ktile = lds + buf * 2 * kTile;
        const char* vtile = ktile + kTile;
        const bool more = step + 1 < n_steps;
        const int key0 = step * kKeyBlock;
        const bool skip = key0 + strict > q0w + 31;
        const int64_t tix = tix0 + step * tstride;
        if (!skip && row_ok && h == 0) p.gtab[tix] = Gc;
        float R = Rnext;
        if (more) {
            if (row_ok) Rnext = p.rtab[tix + tstride];
            kc.load(p.k, kbase, (step + 1) * kKeyBlock, job.len);
            vc.load(p.v, vbase, (step + 1) * kKeyBlock, job.len);
        }
        if (!skip) {
            float x[32], beta[32], dp[32];
            score_tiles_o<D>(x, ktile, lo, qf, p.scale2);
            if (key0 + 63 + strict > q0w) {
mask_step(x, key0 + 32 * h, qi, strict);
            }
            stick_weights<true>(x, beta, R, lane);
            dp_tiles_o<D>(dp, vtile, lo, dof, dr);
            logit_grads<false>(x, beta, dp, Gc, lane);
            bf16x8 zf[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) zf[c] = pack8(&dp[8 * c]);
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    dqacc[db] = mfma(fetch_cols_o<D>(ktile, lo, db, c), zf[c], dqacc[db]);
        }
        if (more) {
            kc.store(lds + (buf ^ 1) * 2 * kTile);
            vc.store(lds + (buf ^ 1) * 2 * kTile + kTile);
        }
        __syncthreads();
    }

    if (row_ok) {
        const int64_t ob = (int64_t)job.seq * p.dq.sb + (int64_t)head * p.dq.sh + (int64_t)(job.tok0 + qi) * p.dq.st;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x2 a = {dqacc[db][4 * g] * p.scale, dqacc[db][4 * g + 1] * p.scale};
                f32x2 b = {dqacc[db][4 * g + 2] * p.scale, dqacc[db][4 * g + 3] * p.scale};
                bf16x2 pa = __builtin_convertvector(a, bf16x2), pb = __builtin_convertvector(b, bf16x2);
                uint2 w;
                w.x = __builtin_bit_cast(uint32_t, pa);
                w.y = __builtin_bit_cast(uint32_t, pb);
                *(uint2*)(p.dq.ptr + 2 * (ob + 32 * db + 8 * g + 4 * h)) = w;
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
    const Job job = decode_job(p, order_job(slot >> 1, p.n_jobs, true));
    const int kb = 2 * job.rb + (slot & 1);
    const int key0 = kb * kKeyBlock;
    if (key0 >= job.len) return;               // uniform over the workgroup
    const int strict = p.attend_current ? 0 : 1;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;
    const int64_t dr_base = (int64_t)job.seq * p.d_rem.sb + (int64_t)head * p.d_rem.sh + job.tok0;
    const int64_t trow = ((int64_t)head * p.n_kb + kb) * p.tab_tokens;
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
        kc.store(ktile);
        vc.store(vtile);
    }
    f32x16 dkacc[D / 64], dvacc[D / 64];
#pragma unroll
    for (int i = 0; i < D / 64; ++i) { dkacc[i] = f32x16{0}; dvacc[i] = f32x16{0}; }

    const int qb0 = job.rb;
    // prefetched state of the first step
    float Rn = 1.0f, Gn = 0.0f, drn = 0.0f;
    bf16x8 qfn[D / 16];
    {
        const int qi0 = qb0 * kRowBlock + 32 * wave + n;
        load_row_frags<D>(qfn, p.q, qbase, qi0, job.len, lane);
        if (qi0 < job.len) {
            const int64_t t = trow + tab_token(p, job, qi0);
            Rn = p.rtab[t]; Gn = p.gtab[t];
            if (p.d_rem.ptr) drn = Elem<uint16_t>::load(p.d_rem.ptr, dr_base + qi0);
        }
    }
    __syncthreads();                           // K, V tiles visible

    for (int qb = qb0; qb < n_qb; ++qb) {
        const int m0 = qb * kRowBlock;
        const int q0w = m0 + 32 * wave;
        const int qi = q0w + n;
        // (1) this lane's Q row fragments were prefetched during the previous step; its dO
        //     fragments are requested now and not needed before the weights are done.  Each
        //     row is fetched from global memory exactly once: the fragments are also what the
        //     shared Q / dO tiles of the reduction are assembled from.
        bf16x8 qf[D / 16], dof[D / 16];
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) qf[ks] = qfn[ks];
        load_row_frags<D>(dof, p.d_o, dobase, qi, job.len, lane);
        float R = Rn, Gc = Gn, dr = drn;
        if (qb + 1 < n_qb) {
            const int qin = qi + kRowBlock;
            load_row_frags<D>(qfn, p.q, qbase, qin, job.len, lane);
            Rn = 1.0f; Gn = 0.0f; drn = 0.0f;
            if (qin < job.len) {
                const int64_t t = trow + tab_token(p, job, qin);
                Rn = p.rtab[t]; Gn = p.gtab[t];
                if (p.d_rem.ptr) drn = Elem<uint16_t>::load(p.d_rem.ptr, dr_base + qin);
            }
        }
        // (2) row 32*wave + n of the shared Q tile (every wave passed the barrier that ends the
        //     previous step's reduction, so the tiles are free)
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks)
            *(bf16x8*)(qtile + tile_offset<D>(32 * wave + n, 2 * ks + h)) = qf[ks];
        // (3) weights of this wave's 32 queries
        float x[32], dp[32];
        const bool skip = key0 + strict > q0w + 31 || q0w >= job.len;
        if (!skip) {
            float beta[32];
            score_tiles_o<D>(x, ktile, lo, qf, p.scale2);
            if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
            stick_weights<true>(x, beta, R, lane);
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks)
                *(bf16x8*)(dotile + tile_offset<D>(32 * wave + n, 2 * ks + h)) = dof[ks];
            dp_tiles_o<D>(dp, vtile, lo, dof, dr);
            logit_grads<true>(x, beta, dp, Gc, lane);
        } else {
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks)
                *(bf16x8*)(dotile + tile_offset<D>(32 * wave + n, 2 * ks + h)) = dof[ks];
#pragma unroll
            for (int idx = 0; idx < 32; ++idx) { x[idx] = 0.f; dp[idx] = 0.f; }
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            *(bf16x8*)(zp + tile_offset<64>(32 * wave + n, 4 * h + c)) = pack8(&x[8 * c]);
            *(bf16x8*)(zd + tile_offset<64>(32 * wave + n, 4 * h + c)) = pack8(&dp[8 * c]);
        }
        __syncthreads();                       // weights and tiles of all waves visible
        // (4) dK[key][d] += sum_q dz[q][key] Q[q][d];  dV[key][d] += sum_q a[q][key] dO[q][d]
#pragma unroll
        for (int c2 = 0; c2 < 8; ++c2) {
            bf16x8 az = fetch_nat_2<64>(zd, za0, za1, 16 * c2);
            bf16x8 ap = fetch_nat_2<64>(zp, za0, za1, 16 * c2);
#pragma unroll
            for (int i = 0; i < D / 64; ++i) {
                dkacc[i] = mfma(az, fetch_nat_2<D>(qtile, qb0o[i], qb1o[i], 16 * c2), dkacc[i]);
                dvacc[i] = mfma(ap, fetch_nat_2<D>(dotile, qb0o[i], qb1o[i], 16 * c2), dvacc[i]);
            }
        }
        __syncthreads();                       // reduction done: tiles may be overwritten
    }
    // accumulator layout: lane (n = d within the block, h), register r -> key 8*(r/4) + 4*h + r%4
    // of this wave's 32 keys (the weight tiles are in natural key order)
#pragma unroll
    for (int i = 0; i < D / 64; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            int key = key0 + 32 * kh + 8 * (r >> 2) + 4 * h + (r & 3);
            if (key < job.len) {
                int d = 32 * (dbw + 2 * i) + n;
                int64_t kof = (int64_t)job.seq * p.dk.sb + (int64_t)head * p.dk.sh + (int64_t)(job.tok0 + key) * p.dk.st + d;
                int64_t vof = (int64_t)job.seq * p.dv.sb + (int64_t)head * p.dv.sh + (int64_t)(job.tok0 + key) * p.dv.st + d;
                Elem<uint16_t>::store(p.dk.ptr, kof, dkacc[i][r] * p.scale);
                Elem<uint16_t>::store(p.dv.ptr, vof, dvacc[i][r]);
            }
        }
}

}  // namespace sba

bool sba_mfma_bwd_available() { return true; }

int sba_launch_mfma_bwd(const sba::KParams& kp, int phases, hipStream_t s) {
    using namespace sba;
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    const bool p1 = phases != 2, p2 = phases != 1;
    if (kp.head_dim == 64) {
        if (p1) hipLaunchKernelGGL((mfma_bwd_dq_kernel<64>), grid, dim3(kThreads), 0, s, kp);
        if (p2) hipLaunchKernelGGL((mfma_bwd_dkv_kernel<64>), dim3(2 * grid.x), dim3(kThreads), 0, s, kp);
    } else {
        if (p1) hipLaunchKernelGGL((mfma_bwd_dq_kernel<128>), grid, dim3(kThreads), 0, s, kp);
        if (p2) hipLaunchKernelGGL((mfma_bwd_dkv_kernel<128>), dim3(2 * grid.x), dim3(kThreads), 0, s, kp);
    }
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}
