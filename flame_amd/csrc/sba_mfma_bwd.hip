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
//   pass 2  (key owner): a workgroup owns one 64-key block (head_dim 64; two blocks, one
//           after the other, in the head_dim 128 variant),
//           sweeps the query blocks at or below the diagonal, recomputes weights and dz of
//           its tile from the two tables, transposes them through LDS and accumulates
//           dK = dZ^T Q and dV = P^T dO in registers.
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

    for (int step = 0, buf = 0; step < n_steps; ++step, buf ^= 1) {
        const char* ktile = lds + buf * 2 * kTile;
        const char* vtile = ktile + kTile;
        const bool more = step + 1 < n_steps;
        if (more) {
            kc.load(p.k, kbase, (step + 1) * kKeyBlock, job.len);
            vc.load(p.v, vbase, (step + 1) * kKeyBlock, job.len);
        }
        const int key0 = step * kKeyBlock;
        const bool skip = key0 + strict > q0w + 31;
        if (!skip) {
            const int64_t tix = ((int64_t)head * p.n_kb + step) * p.tab_tokens + tabtok;
            float x[32], beta[32], dp[32];
            score_tiles<D>(x, ktile, qf, p.scale2, lane);
            if (key0 + 63 + strict > q0w) {
mask_step(x, key0 + 32 * h, qi, strict);
            }
            float R = row_ok ? p.rtab[tix] : 1.0f;
            stick_weights<true>(x, beta, R, lane);
            dp_tiles<D>(dp, vtile, dof, dr, lane);
            if (row_ok && h == 0) p.gtab[tix] = Gc;
            logit_grads<false>(x, beta, dp, Gc, lane);
            bf16x8 zf[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) zf[c] = pack8(&dp[8 * c]);
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    dqacc[db] = mfma(fetch_cols<D>(ktile, db, c, lane), zf[c], dqacc[db]);
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
// Natural-order copy of `rows` rows x D bf16 (global -> LDS), rows >= len zero-filled.
template <int D>
__device__ inline void copy_rows_nat(char* tile, const TensorArg& t, int64_t base, int row0, int len, int rows) {
    for (int cid = threadIdx.x; cid < rows * (D / 8); cid += kThreads) {
        int r = cid / (D / 8), c = cid % (D / 8);
        int row = row0 + r;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (row < len) v = *(const u32x4*)(t.ptr + 2 * (base + (int64_t)row * t.st + c * 8));
        *(u32x4*)(tile + tile_offset<D>(r, c)) = v;
    }
}

template <int D>
__global__ __launch_bounds__(kThreads) void mfma_bwd_dkv_shared_kernel(KParams p) {
    constexpr int kTile = 64 * D * 2;          // K or V tile (64 keys)
    constexpr int kQTile = 128 * D * 2;        // Q or dO tile (128 queries)
    constexpr int kZTile = 128 * 64 * 2;       // weights of one step, [query][key] bf16
    __shared__ __attribute__((aligned(16))) char lds[2 * kTile + 2 * kQTile + 2 * kZTile];
    char* ktile = lds;
    char* vtile = lds + kTile;
    char* qtile = lds + 2 * kTile;
    char* dotile = qtile + kQTile;
    char* zp = dotile + kQTile;                // bf16 attention weights
    char* zd = zp + kZTile;                    // bf16 dz

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform, keep it scalar
    const int n = lane & 31, h = lane >> 5;
    const int head = blockIdx.x % p.n_heads;
    // longest key blocks (leftmost) first: walk the row-block schedule backwards
    const Job job = decode_job(p, order_job(blockIdx.x / p.n_heads, p.n_jobs, true));
    const int strict = p.attend_current ? 0 : 1;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;
    const int n_qb = (job.len + kRowBlock - 1) / kRowBlock;
    const int kh = wave & 1;                   // which 32 keys of the block this wave reduces
    const int dbw = wave >> 1;                 // and which d-blocks: dbw + 2*i

    for (int half = 0; half < 2; ++half) {
        const int kb = 2 * job.rb + half;
        const int key0 = kb * kKeyBlock;
        if (key0 >= job.len) break;            // uniform over the workgroup

        __syncthreads();
        {   // K, V of the owned block in MFMA row order
            TileCopy<D> kc, vc;
            kc.load(p.k, kbase, key0, job.len);
            vc.load(p.v, vbase, key0, job.len);
            kc.store(ktile);
            vc.store(vtile);
        }
        f32x16 dkacc[D / 64], dvacc[D / 64];
#pragma unroll
        for (int i = 0; i < D / 64; ++i) { dkacc[i] = f32x16{0}; dvacc[i] = f32x16{0}; }

        for (int qb = job.rb; qb < n_qb; ++qb) {
            const int m0 = qb * kRowBlock;
            __syncthreads();                   // previous step's readers of q/do/z tiles are done
            copy_rows_nat<D>(qtile, p.q, qbase, m0, job.len, kRowBlock);
            copy_rows_nat<D>(dotile, p.d_o, dobase, m0, job.len, kRowBlock);
            __syncthreads();

            const int q0w = m0 + 32 * wave;
            const int qi = q0w + n;
            const bool row_ok = qi < job.len;
            const bool skip = key0 + strict > q0w + 31;
            float x[32], dp[32];
            if (!skip) {
                bf16x8 qf[D / 16], dof[D / 16];
#pragma unroll
                for (int ks = 0; ks < D / 16; ++ks) {
                    qf[ks] = fetch_row_nat<D>(qtile, 32 * wave + n, ks, lane);
                    dof[ks] = fetch_row_nat<D>(dotile, 32 * wave + n, ks, lane);
                }
                float beta[32];
                score_tiles<D>(x, ktile, qf, p.scale2, lane);
                if (key0 + 63 + strict > q0w) {
mask_step(x, key0 + 32 * h, qi, strict);
                }
                const int64_t tix = ((int64_t)head * p.n_kb + kb) * p.tab_tokens + tab_token(p, job, qi);
                float R = row_ok ? p.rtab[tix] : 1.0f;
                float Gc = row_ok ? p.gtab[tix] : 0.0f;
                float dr = 0.f;
                if (row_ok && p.d_rem.ptr)
                    dr = Elem<uint16_t>::load(p.d_rem.ptr, (int64_t)job.seq * p.d_rem.sb + (int64_t)head * p.d_rem.sh + job.tok0 + qi);
                stick_weights<true>(x, beta, R, lane);
                dp_tiles<D>(dp, vtile, dof, dr, lane);
                logit_grads<false>(x, beta, dp, Gc, lane);
            } else {
#pragma unroll
                for (int idx = 0; idx < 32; ++idx) { x[idx] = 0.f; dp[idx] = 0.f; }
            }
            // weights of query 32*wave+n, keys 32*h .. 32*h+31 -> row of the [query][key] tiles
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                *(bf16x8*)(zp + tile_offset<64>(32 * wave + n, 4 * h + c)) = pack8(&x[8 * c]);
                *(bf16x8*)(zd + tile_offset<64>(32 * wave + n, 4 * h + c)) = pack8(&dp[8 * c]);
            }
            __syncthreads();
            // dK[key][d] += sum_q dz[q][key] Q[q][d];  dV[key][d] += sum_q a[q][key] dO[q][d]
#pragma unroll
            for (int c2 = 0; c2 < 8; ++c2) {
                bf16x8 az = fetch_cols_nat<64>(zd, 16 * c2, kh, lane);
                bf16x8 ap = fetch_cols_nat<64>(zp, 16 * c2, kh, lane);
#pragma unroll
                for (int i = 0; i < D / 64; ++i) {
                    dkacc[i] = mfma(az, fetch_cols_nat<D>(qtile, 16 * c2, dbw + 2 * i, lane), dkacc[i]);
                    dvacc[i] = mfma(ap, fetch_cols_nat<D>(dotile, 16 * c2, dbw + 2 * i, lane), dvacc[i]);
                }
            }
        }
        // accumulator layout: lane (n = d within the block, h), register r -> key 8*(r/4) + 4*h + r%4
        // of this wave's 32 keys.  The weight tiles were written in natural key order, so row m of
        // the A operand IS key 32*kh + m.
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
}

// ---------------------------------------------------------------- pass 2, head_dim 64
// Wave-private variant: every wave reduces over its OWN 32 queries of each step, so the
// sweep has no workgroup barrier at all.  Per step a wave
//   * copies its 32 rows of Q and dO (prefetched one step ahead) into its LDS slice,
//   * computes S^T and dP^T for the 64 owned keys, the weights a and dz,
//   * writes a, dz as bf16 [query][key] rows into its LDS slice and reads them back
//     transposed (ds_read_b64_tr_b16) as the A operands of
//         dK[key][d] += dz^T Q,   dV[key][d] += a^T dO        (K dimension = its 32 queries)
//     with Q, dO read transposed from the same slice as B operands.
// The four partial dK/dV accumulators of the workgroup are summed through LDS once per
// 64-key block.
__device__ inline void wave_rows_load(u32x4 (&r)[4], const TensorArg& t, int64_t base, int row0, int len, int lane) {
    // 32 rows x 64 bf16 = 256 chunks of 16 bytes; lane takes chunks lane + 64*i
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int cid = lane + 64 * i;
        int row = row0 + (cid >> 3), c = cid & 7;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (row < len) v = *(const u32x4*)(t.ptr + 2 * (base + (int64_t)row * t.st + c * 8));
        r[i] = v;
    }
}
__device__ inline void wave_rows_store(char* buf, const u32x4 (&r)[4], int lane) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int cid = lane + 64 * i;
        *(u32x4*)(buf + tile_offset<64>(cid >> 3, cid & 7)) = r[i];
    }
}

__global__ __launch_bounds__(kThreads) void mfma_bwd_dkv64_kernel(KParams p) {
    constexpr int D = 64;
    constexpr int kTile = 64 * D * 2;          // 8 KB: K or V tile (64 keys)
    constexpr int kSlice = 32 * 64 * 2;        // 4 KB: 32 rows x 64 bf16
    // K V | per wave: Q dO Zp Zd  (4 x 16 KB)
    __shared__ __attribute__((aligned(16))) char lds[2 * kTile + 4 * 4 * kSlice];
    char* ktile = lds;
    char* vtile = lds + kTile;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 31, h = lane >> 5;
    char* qbuf = lds + 2 * kTile + wave * 4 * kSlice;
    char* dobuf = qbuf + kSlice;
    char* zp = dobuf + kSlice;
    char* zd = zp + kSlice;
    const int head = blockIdx.x % p.n_heads;
    // one workgroup per 64-key block: two per scheduled 128-row job, leftmost keys (longest
    // sweeps) first
    const int slot = blockIdx.x / p.n_heads;
    const Job job = decode_job(p, order_job(slot >> 1, p.n_jobs, true));
    const int half = slot & 1;
    const int strict = p.attend_current ? 0 : 1;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;
    const int n_qb = (job.len + kRowBlock - 1) / kRowBlock;

    {
        const int kb = 2 * job.rb + half;
        const int key0 = kb * kKeyBlock;
        if (key0 >= job.len) return;           // uniform over the workgroup

        {
            TileCopy<D> kc, vc;
            kc.load(p.k, kbase, key0, job.len);
            vc.load(p.v, vbase, key0, job.len);
            kc.store(ktile);
            vc.store(vtile);
        }
        __syncthreads();

        f32x16 dkacc[2][2], dvacc[2][2];       // [key half][d block]
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b) { dkacc[a][b] = f32x16{0}; dvacc[a][b] = f32x16{0}; }

        // first query this wave ever needs: rows of the diagonal block at or right of the keys
        const int qb0 = job.rb;
        u32x4 qr[4], dor[4];
        wave_rows_load(qr, p.q, qbase, qb0 * kRowBlock + 32 * wave, job.len, lane);
        wave_rows_load(dor, p.d_o, dobase, qb0 * kRowBlock + 32 * wave, job.len, lane);

        for (int qb = qb0; qb < n_qb; ++qb) {
            const int q0w = qb * kRowBlock + 32 * wave;
            const int qi = q0w + n;
            const bool row_ok = qi < job.len;
            // this wave's rows of the step: registers -> LDS slice; prefetch the next step's
            wave_rows_store(qbuf, qr, lane);
            wave_rows_store(dobuf, dor, lane);
            if (qb + 1 < n_qb) {
                wave_rows_load(qr, p.q, qbase, q0w + kRowBlock, job.len, lane);
                wave_rows_load(dor, p.d_o, dobase, q0w + kRowBlock, job.len, lane);
            }
            if (key0 + strict > q0w + 31 || q0w >= job.len) continue;   // nothing visible / no rows

            bf16x8 qf[D / 16], dof[D / 16];
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks) {
                qf[ks] = fetch_row_nat<D>(qbuf, n, ks, lane);
                dof[ks] = fetch_row_nat<D>(dobuf, n, ks, lane);
            }
            float x[32], beta[32], dp[32];
            score_tiles<D>(x, ktile, qf, p.scale2, lane);
            if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
            const int64_t tix = ((int64_t)head * p.n_kb + kb) * p.tab_tokens + tab_token(p, job, qi);
            float R = row_ok ? p.rtab[tix] : 1.0f;
            float Gc = row_ok ? p.gtab[tix] : 0.0f;
            float dr = 0.f;
            if (row_ok && p.d_rem.ptr)
                dr = Elem<uint16_t>::load(p.d_rem.ptr, (int64_t)job.seq * p.d_rem.sb + (int64_t)head * p.d_rem.sh + job.tok0 + qi);
            stick_weights<true>(x, beta, R, lane);
            dp_tiles<D>(dp, vtile, dof, dr, lane);
            logit_grads<true>(x, beta, dp, Gc, lane);
            // row n of the [query][key] slices: keys 32*h .. 32*h+31
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                *(bf16x8*)(zp + tile_offset<64>(n, 4 * h + c)) = pack8(&x[8 * c]);
                *(bf16x8*)(zd + tile_offset<64>(n, 4 * h + c)) = pack8(&dp[8 * c]);
            }
            // same wave wrote and reads: the compiler's lgkmcnt wait orders it
#pragma unroll
            for (int c2 = 0; c2 < 2; ++c2) {
                bf16x8 bq[2], bdo[2];
#pragma unroll
                for (int db = 0; db < 2; ++db) {
                    bq[db] = fetch_cols_nat<64>(qbuf, 16 * c2, db, lane);
                    bdo[db] = fetch_cols_nat<64>(dobuf, 16 * c2, db, lane);
                }
#pragma unroll
                for (int kh = 0; kh < 2; ++kh) {
                    bf16x8 az = fetch_cols_nat<64>(zd, 16 * c2, kh, lane);
                    bf16x8 ap = fetch_cols_nat<64>(zp, 16 * c2, kh, lane);
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
                        dkacc[kh][db] = mfma(az, bq[db], dkacc[kh][db]);
                        dvacc[kh][db] = mfma(ap, bdo[db], dvacc[kh][db]);
                    }
                }
            }
        }

        // ---- sum the four waves' partial tiles through LDS and store.
        // accumulator layout: lane (n = d within its block, h), register r ->
        // key 32*kh + 8*(r/4) + 4*h + r%4.  Reduction buffer: [wave][key 64][d 64] fp32 = 16 KB
        // per wave, reusing the per-wave slices (dK first, then dV).
        float* red = (float*)(lds + 2 * kTile);
#pragma unroll
        for (int which = 0; which < 2; ++which) {
            __syncthreads();
#pragma unroll
            for (int kh = 0; kh < 2; ++kh)
#pragma unroll
                for (int db = 0; db < 2; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        int key = 32 * kh + 8 * (r >> 2) + 4 * h + (r & 3);
                        float v = which == 0 ? dkacc[kh][db][r] : dvacc[kh][db][r];
                        red[(wave * 64 + key) * 64 + 32 * db + n] = v;
                    }
            __syncthreads();
            const TensorArg& out = which == 0 ? p.dk : p.dv;
            const float mul = which == 0 ? p.scale : 1.0f;
            // 64 x 64 outputs, 256 threads: thread -> (key = tid/4, 16 consecutive d)
            const int key = threadIdx.x >> 2, d0 = (threadIdx.x & 3) * 16;
            if (key0 + key < job.len) {
                const int64_t ob = (int64_t)job.seq * out.sb + (int64_t)head * out.sh + (int64_t)(job.tok0 + key0 + key) * out.st + d0;
                uint32_t w[8];
#pragma unroll
                for (int j = 0; j < 16; j += 2) {
                    float s0 = 0.f, s1 = 0.f;
#pragma unroll
                    for (int wv = 0; wv < 4; ++wv) {
                        s0 += red[(wv * 64 + key) * 64 + d0 + j];
                        s1 += red[(wv * 64 + key) * 64 + d0 + j + 1];
                    }
                    f32x2 pr = {s0 * mul, s1 * mul};
                    w[j >> 1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf16x2));
                }
                u32x4* dst = (u32x4*)(out.ptr + 2 * ob);
                dst[0] = u32x4{w[0], w[1], w[2], w[3]};
                dst[1] = u32x4{w[4], w[5], w[6], w[7]};
            }
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
        if (p2) hipLaunchKernelGGL(mfma_bwd_dkv64_kernel, dim3(2 * grid.x), dim3(kThreads), 0, s, kp);
    } else {
        if (p1) hipLaunchKernelGGL((mfma_bwd_dq_kernel<128>), grid, dim3(kThreads), 0, s, kp);
        if (p2) hipLaunchKernelGGL((mfma_bwd_dkv_shared_kernel<128>), grid, dim3(kThreads), 0, s, kp);
    }
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}
